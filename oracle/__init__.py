"""Checkers for the attention + RG-LRU step.  Test infrastructure only."""
