"""MI355X (gfx950) implementation of the Yemong trunk's per-timestep hot path.

Masked multi-head attention over each environment's entity tokens followed by the
per-entity RG-LRU recurrence step, as hand-written HIP kernels behind a C ABI
(``include/bnb_amd.h`` -> ``_lib/libbnb_amd.so``), plus torch modules that keep the
reference policy's layer interfaces and ``state_dict`` names.

    ops       sdpa_masked, sdpa_cross, rglru_step, conv_step, temporal_step, rglru_scan, conv_seq, add_rmsnorm,
              gelu_mul, norm_linear, ffn_fused, team_pool
    trunk     TransformerBlock, RGLRU, GriffinTemporalBlock, YemongBlock, YemongTrunk, GraphedTrunk, TeamPMA
    harness   benchmark workloads, traffic model, AttnRglruStep
    build     compiles the HIP sources
"""

from . import _native, harness, ops, trunk
from .ops import conv_seq, conv_step, rglru_scan, rglru_step, sdpa_cross, sdpa_masked
from .trunk import (
    CONV_KERNEL,
    GatedMLP,
    EagerTrunkStepper,
    GraphedTrunk,
    GriffinTemporalBlock,
    LibraryDispatchWarning,
    ModelConfig,
    RGLRU,
    TeamPMA,
    TransformerBlock,
    YemongBlock,
    YemongTrunk,
    forbid_library_dispatch,
    separate_heads,
    trunk_stepper,
    invalidate_weight_caches,
    library_dispatches,
)

__all__ = [
    "CONV_KERNEL", "GatedMLP", "GraphedTrunk", "EagerTrunkStepper", "trunk_stepper", "GriffinTemporalBlock", "ModelConfig", "RGLRU", "TeamPMA", "TransformerBlock",
    "YemongBlock", "YemongTrunk", "conv_seq", "conv_step", "rglru_scan", "rglru_step", "sdpa_cross", "sdpa_masked", "ops",
    "trunk", "harness", "LibraryDispatchWarning", "forbid_library_dispatch", "separate_heads", "invalidate_weight_caches", "library_dispatches",
]
