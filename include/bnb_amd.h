/*
 * C ABI of libbnb_amd.so: the masked-attention and RG-LRU step kernels for gfx950.
 *
 * The reference has no FFI or operator registry; the seam it offers is two Python
 * call sites inside its policy trunk.  Each entry point below names the reference
 * lines it stands in for (paths relative to the reference checkout,
 * src/boost_and_broadside/).
 *
 * Conventions shared by every entry point
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is allocated,
 *     freed or copied to the host, and no call synchronises the stream;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); work is
 *     enqueued on it and the call returns immediately;
 *   - the return value is 0 on success, a BNB_ERR_* code for a rejected argument, or
 *     a hipError_t value if the launch itself failed; bnb_error_string() names it;
 *   - calls are re-entrant and keep no state between calls.
 */
#ifndef BNB_AMD_H
#define BNB_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BNB_ABI_VERSION 28

/* element types of activation buffers */
#define BNB_F32 0
#define BNB_BF16 1

/* argument errors (kept clear of the hipError_t range) */
#define BNB_ERR_NULL_POINTER 10001  /* a required pointer is NULL */
#define BNB_ERR_BAD_DTYPE 10002     /* dtype is neither BNB_F32 nor BNB_BF16 */
#define BNB_ERR_BAD_SHAPE 10003     /* negative size, H*dh mismatch, stride smaller than a row */
#define BNB_ERR_UNSUPPORTED 10004   /* shape outside what the kernels cover (see each entry point) */
#define BNB_ERR_MISALIGNED 10005    /* pointer or stride breaks the stated alignment */
#define BNB_ERR_SCRATCH_LIMIT 10006 /* the call needs more workspace than the library's built-in buffer holds */

/* Bumped on any change of a signature or of the meaning of an argument. */
int bnb_abi_version(void);

/* Architecture the device code was compiled for ("gfx950"). */
const char *bnb_build_arch(void);

/* Static, human-readable name of a code returned by the entry points below. */
const char *bnb_error_string(int code);

/*
 * Masked multi-head attention over each environment's entity tokens.
 *
 * Replaces, in models/yemong/attention.py: the key-bias construction (:101-112,
 * :142-145), F.scaled_dot_product_attention(q, k, v, attn_mask=bias) (:147) and the
 * head-merge copy permute(0,2,1,3).reshape(B,N,D) (:168).  The packed projection
 * `qkv = self.qkv(x)` (:135) goes in as it is, the tensor handed to `out_proj` (:169)
 * comes out.
 *
 *   qkv    (B, NM, 3*H*dh) rows of `qkv_row_stride` elements, columns [Q | K | V],
 *          each third split into H runs of dh columns; environments follow each other
 *          every NM rows
 *   alive  (B, NM) bytes, non-zero = the entity exists; NULL = no masking.  A dead key
 *          receives weight exactly 0 whenever its environment has a live key; an
 *          environment with no live key averages V uniformly over all NM keys (what the
 *          reference's additive finfo.min/2 bias produces); dead queries are computed
 *   out    (B, NM, H*dh) contiguous, heads merged head-major, same dtype as qkv
 *   dtype  BNB_F32 or BNB_BF16 (bf16 in/out, fp32 scores, softmax and accumulation)
 *
 * Requirements: dh in {8,16,32,64}; NM <= 512 and NM*(dh+4)*8 bytes of K/V for one head
 * within 160 KB of LDS (else BNB_ERR_UNSUPPORTED); qkv, out and the row stride aligned to
 * 16 bytes.  B == 0 or NM == 0 is a no-op.
 */
int bnb_sdpa_masked_fwd(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, void *out,
                        int B, int NM, int H, int dh, int dtype, void *stream);

/*
 * Same as bnb_sdpa_masked_fwd with the kernel chosen by the caller instead of by shape;
 * used by tests and the benchmark to run both kernels on one input.  No reference
 * counterpart beyond the one above.
 *   BNB_SDPA_PATH_AUTO  what bnb_sdpa_masked_fwd does: the bf16 matrix-core kernel for bf16,
 *                       dh == 32 and NM <= 160; the fp32 matrix-core kernel for fp32, dh == 32
 *                       and NM <= 512; the vector-ALU kernel otherwise
 *   BNB_SDPA_PATH_VALU  vector-ALU kernel (any supported shape and dtype)
 *   BNB_SDPA_PATH_MFMA  bf16 matrix-core kernel, one work-group per (environment, head) (bf16, dh == 32,
 *                       NM <= 160; else BNB_ERR_UNSUPPORTED)
 *   BNB_SDPA_PATH_ENV   bf16 matrix-core kernel, one work-group per environment with the heads streamed
 *                       through LDS (bf16, H == 4, dh == 32, NM <= 160; else BNB_ERR_UNSUPPORTED)
 */
#define BNB_SDPA_PATH_AUTO 0
#define BNB_SDPA_PATH_VALU 1
#define BNB_SDPA_PATH_MFMA 2
#define BNB_SDPA_PATH_ENV 3
#define BNB_SDPA_PATH_HEAD 4 /* one work-group per (environment, head) with the rows loaded straight into LDS (bf16, dh == 32, NM <= 160) */
int bnb_sdpa_masked_fwd_path(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, void *out,
                             int B, int NM, int H, int dh, int dtype, int path, void *stream);

/*
 * Cross-attention of the entity queries to a second set of key/value rows (the bullet read),
 * on the matrix-core kernel.
 *
 * Replaces, in models/yemong/attention.py:149-166: the head split of kb/vb (:152-153), the key
 * bias (:154), F.scaled_dot_product_attention(q, kb, vb, attn_mask=bias) (:155-157), the
 * `any_active` gate (:158-165: an environment without an active key contributes exactly 0
 * instead of the uniform average) and `out = out + bullet_out` (:166).
 *
 *   q        (B, NQ, >= H*dh) rows of q_row_stride elements: the Q third of the packed
 *            projection, heads head-major
 *   k, v     (B, NK, >= H*dh) rows of kv_row_stride elements each (the two halves of
 *            kv_bullet's output work: v = k + H*dh)
 *   key_mask (B, NK) bytes, non-zero = active; NULL = all active
 *   accum    optional (B, NQ, H*dh) contiguous: the self-attention output to add to (bf16
 *            addition as torch performs it); may equal out
 *   out      (B, NQ, H*dh) contiguous
 * Requirements: dh == 32, 16-byte aligned rows; BNB_BF16 with 1 <= NK <= 2048, NQ <= 160, or
 * BNB_F32 (evaluation without autocast, evaluation/agents.py:214-219; true fp32 products on the
 * matrix cores, fp32 addition into accum) with 1 <= NK <= 4096, NQ <= 512; anything else returns
 * BNB_ERR_UNSUPPORTED and the caller keeps its library path.  Up to 160 keys are staged in LDS at
 * once; longer key axes (the shipped scenarios have 10 bullet slots per ship, 80 .. 1520 keys)
 * are streamed in tiles of the active keys only, so the cost follows the number of bullets in
 * flight, not the number of slots.
 */
int bnb_sdpa_cross_fwd(const void *q, int64_t q_row_stride, int NQ, const void *k, const void *v,
                       int64_t kv_row_stride, int NK, const uint8_t *key_mask, const void *accum,
                       void *out, int B, int H, int dh, int dtype, void *stream);

/*
 * bnb_sdpa_cross_fwd over key/value rows that were compacted beforehand: kv_rows holds the
 * [K | V] rows (2*H*dh wide, kv_row_stride elements apart) of the active keys of all
 * environments back to back, and environment b owns rows ranges[b] .. ranges[b+1]-1 (int32,
 * B+1 entries, e.g. the offsets of bnb_mask_fill with kv_rows = bnb_norm_linear_fwd over the
 * same list).  No mask is scanned; an environment with an empty range contributes exactly 0.
 * Any number of keys per environment; kv_capacity = rows allocated in kv_rows (addressed with
 * 32-bit element offsets: kv_capacity * kv_row_stride < 2^32).  Other arguments and
 * requirements as bnb_sdpa_cross_fwd.
 */
int bnb_sdpa_cross_ranges_fwd(const void *q, int64_t q_row_stride, int NQ, const void *kv_rows,
                              int64_t kv_row_stride, const int32_t *ranges, int64_t kv_capacity,
                              const void *accum, void *out, int B, int H, int dh, int dtype, void *stream);

/*
 * bnb_sdpa_cross_ranges_fwd that also hands over what the update needs from this pass: lse, (B, H, NQ)
 * float32, the base-2 logarithm of the sum over an environment's keys of exp2(score * log2(e) / sqrt(dh))
 * per head and query, for bnb_sdpa_cross_stream_bwd_lse (the backward of the same read,
 * models/yemong/attention.py:149-166 under train/rl/ppo.py:1417-1425), which otherwise recomputes it
 * from every key.  Entries of environments with an empty range carry no meaning and are not read there.
 */
int bnb_sdpa_cross_ranges_fwd_lse(const void *q, int64_t q_row_stride, int NQ, const void *kv_rows,
                                  int64_t kv_row_stride, const int32_t *ranges, int64_t kv_capacity,
                                  const void *accum, void *out, float *lse, int B, int H, int dh, int dtype,
                                  void *stream);

/*
 * One RG-LRU recurrence step over R = B*n_rec entity rows of D channels.
 *
 * Replaces the element-wise chain of models/yemong/griffin.py:179-185 (RGLRU._step),
 * equally :208-212 plus the T=1 scan of :45-64 (out = a*h0 + b): the two sigmoids,
 * a = sigmoid(log_lambda)^(c*r), gate = sqrt(clamp((1-a)(1+a), 1e-6)),
 * h' = a*h + gate*(i*x).  The two gate projections linear_a / linear_x (:166-167)
 * stay GEMMs on the caller's side and arrive as one (R, 2*D) buffer.
 *
 *   x          (R, D) contiguous, x_dtype
 *   gates_pre  (R, 2*D) contiguous, g_dtype: [linear_a(x) | linear_x(x)], biases included
 *   log_lambda (D) fp32
 *   c          the exponent constant (8 in the reference)
 *   h_in       previous state, fp32, row r at h_in + r*h_in_row_stride (floats); a stride
 *              of 4*D addresses the packed hidden tensor of models/yemong/policy.py:323
 *   h_out      new state, fp32, same addressing; may equal h_in (in-place update)
 *   y          optional (R, D) copy of the new state in y_dtype (the layer output under
 *              bf16 autocast); NULL to skip it
 *
 * With bf16 gate pre-activations the roundings of the reference's autocast path are
 * reproduced (r, i and c*r are rounded to bf16; i*x is rounded to bf16 when x is bf16
 * too); state, decay and gate are always fp32.
 *
 * Requirements: D >= 1; R >= 0.  Rows whose pointers and strides are 16-byte aligned
 * with D % 8 == 0 take the vector path; anything else takes a scalar path.
 */
int bnb_rglru_step_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                       const float *log_lambda, float c,
                       const float *h_in, int64_t h_in_row_stride,
                       float *h_out, int64_t h_out_row_stride,
                       void *y, int y_dtype, int64_t R, int D, void *stream);

/*
 * bnb_rglru_step_fwd with an optional per-environment reset folded into the read of the
 * previous state: rows r with reset[r / rows_per_env] != 0 use h = 0.  This is the effect of
 * the reference's reset_hidden_for_envs (models/yemong/policy.py:268-285, a full read+write of
 * the packed state after every step) applied to the RG-LRU columns, without that pass.
 * reset == NULL behaves exactly like bnb_rglru_step_fwd; reset holds one byte per environment
 * and rows are environment-major (models/yemong/griffin.py:408).
 */
int bnb_rglru_step_reset_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                             const float *log_lambda, float c,
                             const float *h_in, int64_t h_in_row_stride,
                             float *h_out, int64_t h_out_row_stride,
                             void *y, int y_dtype, const uint8_t *reset, int rows_per_env,
                             int64_t R, int D, void *stream);

/*
 * bnb_rglru_step_reset_fwd with the output y laid out per environment: with
 * y_group_stride != 0, row r of y is at y + (r / rows_per_env) * y_group_stride +
 * (r % rows_per_env) * D elements (y_group_stride >= rows_per_env * D, a multiple of 8), which
 * addresses the ship tokens inside a (B, N+M, D) token tensor (models/yemong/griffin.py:390-417
 * slices and concatenates ship and field tokens around the temporal operator; writing in
 * place removes both copies).  y_group_stride == 0: contiguous (R, D).  rows_per_env is used
 * for the grouping also when reset is NULL.
 */
int bnb_rglru_step_rows_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                            const float *log_lambda, float c,
                            const float *h_in, int64_t h_in_row_stride,
                            float *h_out, int64_t h_out_row_stride,
                            void *y, int y_dtype, int64_t y_group_stride,
                            const uint8_t *reset, int rows_per_env,
                            int64_t R, int D, void *stream);

/*
 * Causal depthwise conv (kernel 4) for one timestep plus the shift of the stored inputs.
 *
 * Replaces, in models/yemong/griffin.py at T = 1: `padded = cat([conv_buf, b1])` (:275), the
 * tap loop of _causal_depthwise_conv (:127-139: out = sum_k padded[:, k] * weight[:, k] + bias)
 * and `new_conv_buf = padded[:, -3:]` (:277); and, in models/yemong/policy.py, the re-packing
 * cat of the conv columns (:346-354) because the new inputs are written where they live.
 *
 *   b1        (R, D) contiguous, b1_dtype: this step's linear1 output (bf16 under autocast)
 *   conv_in   previous three inputs of row r at conv_in + r*conv_in_row_stride, laid out
 *             [p0 | p1 | p2] (oldest first), D floats each; a stride of 4*D with conv_in =
 *             state + D addresses the packed hidden tensor (policy.py:324)
 *   weight    (D, 4) fp32 = conv.weight.squeeze(1); tap k multiplies padded[:, k], so the
 *             current input meets weight[:, 3]
 *   bias      (D) fp32 or NULL
 *   reset     optional, one byte per environment of rows_per_env rows: a non-zero byte makes
 *             the stored inputs read as zero (reset_hidden_for_envs folded in)
 *   v_out     (R, D) fp32 contiguous: the conv output (input of the RG-LRU)
 *   v_bf16_out optional (R, D) bf16 contiguous copy of v_out (what autocast would feed the
 *             gate projections), or NULL
 *   conv_out  new stored inputs [p1 | p2 | b1], same addressing as conv_in; may equal conv_in
 *
 * Requirements: D >= 1, strides >= 3*D.  16-byte aligned rows with D % 8 == 0 take the vector
 * path; anything else takes a scalar path.
 */
int bnb_conv_step_fwd(const void *b1, int b1_dtype,
                      const float *conv_in, int64_t conv_in_row_stride,
                      const float *weight, const float *bias,
                      const uint8_t *reset, int rows_per_env,
                      float *v_out, void *v_bf16_out, float *conv_out, int64_t conv_out_row_stride,
                      int64_t R, int D, void *stream);

/*
 * bnb_conv_step_fwd with the input b1 laid out per environment: with b1_group_stride != 0,
 * row r of b1 is at b1 + (r / rows_per_env) * b1_group_stride + (r % rows_per_env) * D elements
 * (the ship tokens inside a (B, N+M, D) tensor of linear1 outputs).  0: contiguous (R, D).
 * b1_row_stride (elements, 0 = D) is the distance between consecutive rows, for a b1 that is a
 * column block of a wider projection output (e.g. [linear1 | linear2] computed together).
 */
int bnb_conv_step_rows_fwd(const void *b1, int b1_dtype, int64_t b1_group_stride, int64_t b1_row_stride,
                           const float *conv_in, int64_t conv_in_row_stride,
                           const float *weight, const float *bias,
                           const uint8_t *reset, int rows_per_env,
                           float *v_out, void *v_bf16_out, float *conv_out, int64_t conv_out_row_stride,
                           int64_t R, int D, void *stream);

/*
 * Weight gradient of a bias-free or biased Linear layer:  dw[n][k] (+)= sum_r dy[r][n] * x[r][k],
 * bf16 operands, fp32 accumulation on the matrix cores, fp32 result.
 *
 * Replaces what autograd computes for `weight.grad` of the trunk's nn.Linear layers
 * (models/yemong/attention.py:60-74, models/yemong/griffin.py:165-167,238-247) when the PPO update
 * back-propagates through them (train/rl/ppo.py:1417-1425): there the contraction runs over
 * several hundred thousand token rows while N and K are 128..512, a shape the library GEMM
 * runs far from the HBM bound.
 *
 *   dy       (R, N) bf16, rows dy_row_stride elements apart: gradient of the layer's output
 *   x        (R, K) bf16, rows x_row_stride elements apart: the layer's input (as autocast cast it)
 *   partials (slices, N, K) fp32 workspace owned by the caller; slices >= 1, a good value comes
 *            from bnb_linear_wgrad_slices(R, N, K)
 *   dw       (N, K) fp32 contiguous: overwritten, or added to when accumulate != 0
 *
 * The rows are split into `slices` ranges, one work-group per (128 x 128 output tile, slice);
 * a second kernel adds the slices in a fixed order, so the result does not depend on timing.
 * Requirements: N % 128 == 0, K % 128 == 0, 16-byte aligned pointers, strides multiples of 8.
 */
int bnb_linear_wgrad_slices(int64_t R, int N, int K);
/* Which kernel computes the product, for tests and benchmarks: AUTO = DMA (operand rows global -> LDS directly,
 * transposed by the LDS read); STAGED = through registers with a transpose in registers.  Changes what
 * bnb_linear_wgrad_slices returns: set it before sizing the workspace. */
#define BNB_WGRAD_PATH_AUTO 0
#define BNB_WGRAD_PATH_STAGED 1
#define BNB_WGRAD_PATH_DMA 2
int bnb_linear_wgrad_path(int path);
int bnb_linear_wgrad_fwd(const void *dy, int64_t dy_row_stride, const void *x, int64_t x_row_stride,
                         float *partials, int slices, float *dw, int accumulate,
                         int64_t R, int N, int K, void *stream);
/*
 * The same with operands that may be stored tile by tile: the 128 columns 128j .. 128j+127 of dy
 * start dy_tile_stride elements after those of tile j-1 (128 = plain row-major rows; R * 128 with
 * dy_row_stride 128 = a (N/128, R, 128) array), likewise x.  bnb_ffn_bwd writes such operands.
 */
int bnb_linear_wgrad_tiled_fwd(const void *dy, int64_t dy_row_stride, int64_t dy_tile_stride, const void *x,
                               int64_t x_row_stride, int64_t x_tile_stride, float *partials, int slices, float *dw,
                               int accumulate, int64_t R, int N, int K, void *stream);

/*
 * Bias gradient of a Linear layer:  out[n] (+)= sum_r x[r][n], fp32 sums of bf16 or fp32 rows.
 *
 * Replaces what autograd computes for `bias.grad` of the RG-LRU's two gate projections
 * (models/yemong/griffin.py:165-167) in the PPO update (train/rl/ppo.py:1417-1425): a column sum over
 * several hundred thousand rows of the (R, 256) gate gradient.
 *
 *   x        (R, N) bf16 or fp32 (x_dtype), rows x_row_stride elements apart
 *   partials (slices, N) fp32 workspace owned by the caller; slices from bnb_column_sums_slices(R, N)
 *   out      (N) fp32: overwritten, or added to when accumulate != 0
 *
 * Each work-group adds a run of consecutive rows, a second kernel the work-groups' rows, both in a fixed order.
 * Requirements: N % 64 == 0, N <= 2048, 16-byte aligned pointers, x_row_stride a multiple of 8.
 */
int bnb_column_sums_slices(int64_t R, int N);
int bnb_column_sums(const void *x, int x_dtype, int64_t x_row_stride, float *partials, int slices, float *out,
                    int accumulate, int64_t R, int N, void *stream);

/*
 * Backward of bnb_sdpa_masked_fwd for small token counts: what autograd computes through
 * models/yemong/attention.py:136-147 (head split, key bias on dead entities, SDPA, head merge)
 * in the PPO update (train/rl/ppo.py:1417-1425).
 *
 *   qkv    (B, NM, 3*H*dh) as passed to the forward, rows qkv_row_stride elements apart
 *          (environments NM rows apart)
 *   alive  (B, NM) bytes or NULL, as in the forward
 *   out    (B, NM, H*dh) contiguous: the forward's result
 *   dout   (B, NM, H*dh) contiguous: its gradient
 *   dqkv   (B, NM, 3*H*dh) contiguous: gradient of qkv
 * all in `dtype` (BNB_F32 or BNB_BF16), arithmetic in fp32, every sum in a fixed order.
 * Requirements: dh == 32 and either NM <= 32 with H <= 8 (vector-ALU kernel, fp32 or bf16) or bf16
 * with NM <= 160 (matrix-core kernel); 16-byte aligned rows.  Other shapes return
 * BNB_ERR_UNSUPPORTED (the caller keeps the library's differentiable attention for them).
 * bnb_sdpa_masked_bwd_path selects the kernel (BNB_SDPA_PATH_*; AUTO = vector-ALU kernel up to 32
 * tokens, matrix cores above), for tests and benchmarks.
 */
int bnb_sdpa_masked_bwd(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, const void *out,
                        const void *dout, void *dqkv, int64_t B, int NM, int H, int dh, int dtype, void *stream);
int bnb_sdpa_masked_bwd_path(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, const void *out,
                             const void *dout, void *dqkv, int64_t B, int NM, int H, int dh, int dtype, int path,
                             void *stream);

/*
 * Backward of bnb_sdpa_cross_fwd called without accumulator (autograd through the bullet read,
 * models/yemong/attention.py:149-166, in the PPO update): bf16, dh == 32, NQ <= 160, NK <= 160.
 *
 *   q, kv, key_mask  as passed to the forward (q = the packed entity projection, only its first
 *                    H*dh columns are read; kv = [K | V] rows)
 *   out, dout        (B, NQ, H*dh) contiguous: the read's own result and its gradient
 *   dq               (B, NQ, H*dh) contiguous;  dkv (B, NK, 2*H*dh) contiguous
 * An environment without an active key was gated off in the forward: its gradients are zero.
 */
int bnb_sdpa_cross_bwd(const void *q, int64_t q_row_stride, int NQ, const void *kv, int64_t kv_row_stride, int NK,
                       const uint8_t *key_mask, const void *out, const void *dout, void *dq, void *dkv,
                       int64_t B, int H, int dh, int dtype, void *stream);

/*
 * The same backward over key/value rows compacted beforehand (the counterpart of
 * bnb_sdpa_cross_ranges_fwd): environment b reads rows ranges[b] .. ranges[b+1]-1 of kv_rows
 * (capacity rows of [K | V], all of them live), at most max_keys <= 160 per environment;
 * dkv_rows has kv_rows' layout.  An environment with an empty range gets a zero dq.
 */
int bnb_sdpa_cross_ranges_bwd(const void *q, int64_t q_row_stride, int NQ, const void *kv_rows, int64_t kv_row_stride,
                              const int32_t *ranges, int64_t capacity, int max_keys, const void *out, const void *dout,
                              void *dq, void *dkv_rows, int64_t B, int H, int dh, int dtype, void *stream);

/*
 * The bullet read's backward for ANY number of live keys per environment (bf16, dh = 32, NQ <= 160):
 * what autograd computes through models/yemong/attention.py:149-166 when the bullet axis is longer
 * than 160 slots (10 slots per ship, config/defaults.py:29; caller train/rl/ppo.py:1417-1425).
 * Environment b's keys are list entries ranges[b] .. ranges[b+1]-1 (clamped to `capacity` entries in
 * all).  row_index == NULL: entry e is row e of kv (rows compacted beforehand, as for
 * bnb_sdpa_cross_ranges_bwd).  row_index != NULL: entry e is row row_index[e] of kv, i.e. the (B, NK, 2D)
 * buffer is read in place through the list of its live slots (bnb_mask_count / bnb_mask_fill); dkv then
 * has that layout too and the rows of slots that are not listed are NOT written (zero them beforehand).
 * out is the read's own result (nothing accumulated), dq (B, NQ, D) contiguous, dkv has kv's row
 * stride 2D.  stats: workspace of 2 * B * H * NQ floats (per query and head: log2-sum-exp and
 * rowsum(dout * out), written by the first kernel, read by the second).  An environment with an
 * empty range gets a zero dq.
 */
int bnb_sdpa_cross_stream_bwd(const void *q, int64_t q_row_stride, int NQ, const void *kv, int64_t kv_row_stride,
                              const int32_t *ranges, const int32_t *row_index, int64_t capacity, const void *out,
                              const void *dout, void *dq, void *dkv, float *stats, int64_t B, int H, int dh, int dtype,
                              void *stream);

/*
 * bnb_sdpa_cross_stream_bwd with the log2-sum-exp of every query taken from the forward pass
 * (lse as written by bnb_sdpa_cross_ranges_fwd_lse over the same q, keys and ranges) instead of being
 * recomputed: the first kernel then passes over the keys once instead of twice.  Everything else,
 * stats included, as bnb_sdpa_cross_stream_bwd.
 */
int bnb_sdpa_cross_stream_bwd_lse(const void *q, int64_t q_row_stride, int NQ, const void *kv, int64_t kv_row_stride,
                                  const int32_t *ranges, const int32_t *row_index, int64_t capacity, const void *out,
                                  const void *dout, const float *lse, void *dq, void *dkv, float *stats, int64_t B,
                                  int H, int dh, int dtype, void *stream);

/*
 * RMSNorm backward:  y = x * rsqrt(mean(x^2) + eps) * weight
 *   dx[r] = rstd * (dy[r] * weight) - x[r] * rstd^3 * mean(dy[r] * weight * x[r])  (+ grad_sum[r])
 *   dw    = sum_r dy[r] * x[r] * rstd
 *
 * Replaces what autograd runs for the trunk's nn.RMSNorm modules (models/yemong/attention.py:60,73,
 * 94-98; models/yemong/griffin.py:238,246,269,284-285) in the PPO update (train/rl/ppo.py:1417-1425):
 * the cast of a bf16 gradient to fp32, the library's two norm-backward kernels and, with
 * grad_sum, the add of the gradient that reaches x past the norm (the residual branch).
 *
 *   x        (R, D) fp32, rows x_row_stride elements apart: the norm's input
 *   dy       (R, D) bf16 or fp32 (dy_dtype), rows dy_row_stride apart: gradient of the norm's output
 *   grad_sum (R, D) fp32 contiguous or NULL
 *   dx       (R, D) fp32 contiguous (may alias grad_sum)
 *   dx_bf16  optional (R, D) bf16 contiguous copy of dx (the gradient of a bf16 residual delta), or NULL
 *   partials (blocks, D) fp32 workspace of the caller; blocks from bnb_rmsnorm_bwd_blocks(R, D)
 *   dw       (D) fp32, overwritten; rows are added in a fixed order (no atomics)
 * Requirements: D in {64, 128, 256, 512}; 16-byte aligned pointers; x_row_stride % 4 == 0,
 * dy_row_stride % 8 == 0.
 */
int bnb_rmsnorm_bwd_blocks(int64_t R, int D);
int bnb_rmsnorm_bwd(const float *x, int64_t x_row_stride, const void *dy, int dy_dtype, int64_t dy_row_stride,
                    const float *weight, float eps, const float *grad_sum, float *dx, void *dx_bf16,
                    float *partials, int blocks, float *dw, int64_t R, int D, void *stream);

/*
 * bnb_rmsnorm_bwd without the caller's workspace and without any allocation.
 *
 * No counterpart in the reference.  It is for callers that cannot allocate device memory around the
 * call: code under HIP graph capture, tight loops that must not touch the allocator, harnesses that
 * forbid hipMalloc.  The per-work-group partial weight gradients (the `partials` argument of
 * bnb_rmsnorm_bwd) live in a buffer built into the library, bnb_rmsnorm_bwd_static_limit() bytes
 * (2.5 MiB) per GPU, held until the process ends; its device address is looked up once per device on
 * the first call made with that device current.  The call itself calls no hipMalloc / hipFree.
 *
 * Arguments and results as bnb_rmsnorm_bwd (the number of work-groups is chosen as
 * bnb_rmsnorm_bwd_blocks(R, D) would).  D above 512 returns BNB_ERR_SCRATCH_LIMIT: the partials of one
 * launch would not fit the buffer.  All calls on one GPU share that GPU's buffer: two calls that
 * may run at the same time on one GPU (different streams, different threads) race on it and must be
 * ordered by the caller; calls on one stream are ordered already.
 */
int64_t bnb_rmsnorm_bwd_static_limit(void);
int bnb_rmsnorm_bwd_static(const float *x, int64_t x_row_stride, const void *dy, int dy_dtype, int64_t dy_row_stride,
                           const float *weight, float eps, const float *grad_sum, float *dx, void *dx_bf16,
                           float *dw, int64_t R, int D, void *stream);

/*
 * Pooling by multi-head attention over each team's alive ships, broadcast back to the ships:
 * two kernels with one plain fp32 GEMM of the caller's between them.
 *
 * Together they replace TeamPMA.forward, models/yemong/policy.py:94-120: the two
 * nn.MultiheadAttention calls with a learned seed as the only query (keys = alive ships of
 * team t), nan_to_num, the has_ship gate, RMSNorm, and the gather that hands every ship the
 * vector of team clamp(team_id, 0, 1).  The seed being a constant of the model, the caller folds
 * the weights once per weight update (attn.in_proj_weight = [W_q; W_k; W_v], heads = slices hs):
 *
 *   score_vectors (2H, D) fp32: row t*H + h = W_k[hs, :]^T (W_q seeds[t])[hs] * log2(e) / sqrt(dh)
 *   M             (H*D, D) fp32: rows h*D .. (h+1)*D = (attn.out_proj.weight[:, hs] W_v[hs, :])^T
 *
 * bnb_team_attend_fwd: z[b, t, h, :] = sum_j softmax_j(x[b, j] . score_vectors[t*H + h]) x[b, j]
 * over the alive ships j of team t (all zero when there is none).
 *   x        (B, N, D) fp32 ship rows: x[b, n] at b*x_env_stride + n*x_row_stride (a [:, :N]
 *            view of the (B, N+M, D) trunk output works)
 *   team_id  (B, N) int32, row b at b*team_env_stride; alive (B, N) bytes, likewise
 *   z        (B, 2, H, D) fp32 contiguous
 * The caller then forms pre = z.view(B*2, H*D) @ M (library GEMM, fp32).
 *
 * bnb_team_norm_broadcast_fwd: pool = RMSNorm(pre) (a zero row stays zero), out[b, n] =
 * pool[b, clamp(team_id[b, n], 0, 1)].
 *   pre      (B, 2, D) fp32 contiguous; norm_weight (D) fp32, eps
 *   pool     (B, 2, D) fp32 or NULL; out (B, N, D) fp32 at b*out_env_stride + n*out_row_stride,
 *            or NULL (then team_id may be NULL too)
 *
 * Requirements: D == 128, H in {2, 4}, 16-byte aligned x / out, strides multiples of 4 elements.
 */
int bnb_team_attend_fwd(const float *x, int64_t x_env_stride, int64_t x_row_stride,
                        const int32_t *team_id, int64_t team_env_stride,
                        const uint8_t *alive, int64_t alive_env_stride,
                        const float *score_vectors, float *z,
                        int B, int N, int H, int D, void *stream);
int bnb_team_norm_broadcast_fwd(const float *pre, const float *norm_weight, float eps,
                                const int32_t *team_id, int64_t team_env_stride,
                                float *pool, float *out, int64_t out_env_stride, int64_t out_row_stride,
                                int B, int N, int D, void *stream);

/*
 * Backward of bnb_team_attend_fwd for the update path (autograd through the attention weights of
 * TeamPMA.forward, models/yemong/policy.py:94-120, in train/rl/ppo.py:1417-1425).
 *
 *   x, team_id, alive, score_vectors  as passed to the forward
 *   z, dz     (B, 2, H, 128) fp32: the forward's result and its gradient
 *   dx        (B, N, 128) fp32 contiguous: gradient of the ship rows
 *   ds        (B*N, 2H) fp32 workspace/result: gradient of the base-2 scores (zero under the other team's heads)
 *   partials  (bnb_team_attend_bwd_partial_rows(), 2H, 128) fp32 workspace
 *   du        (2H, 128) fp32: gradient of score_vectors, rows added in a fixed order
 */
int bnb_team_attend_bwd(const float *x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *team_id,
                        int64_t team_env_stride, const uint8_t *alive, int64_t alive_env_stride,
                        const float *score_vectors, const float *z, const float *dz, float *dx, float *ds,
                        float *partials, float *du, int B, int N, int H, int D, void *stream);
int bnb_team_attend_bwd_partial_rows(void);

/*
 * Backward of the hand-out of bnb_team_norm_broadcast_fwd: dpool (B, 2, 128) = per team the sum of
 * dout (B, N, 128, contiguous) over the ships that hold that team's vector, zero for a team without
 * an alive ship of its own.
 */
int bnb_team_gather_bwd(const float *dout, const int32_t *team_id, int64_t team_env_stride, const uint8_t *alive,
                        int64_t alive_env_stride, float *dpool, int B, int N, int D, void *stream);

/*
 * One timestep of the temporal sublayer's state path in one launch: conv taps + buffer shift
 * (bnb_conv_step_rows_fwd), the two RG-LRU gate projections, and the recurrence
 * (bnb_rglru_step_rows_fwd), under the dtype flow of bfloat16 autocast.
 *
 * Replaces, in models/yemong/griffin.py at T = 1: :275-277 (cat, _causal_depthwise_conv :127-139,
 * buffer slice) and RGLRU.forward_sequence :206-219 with its linear_a / linear_x (:166-167), i.e.
 * everything between `linear1` and the `rglru_out * gate` product of :279-281.  The conv output
 * and the gate pre-activations stay on chip (4608 instead of 7168 bytes of traffic per row).
 *
 *   b1, b1_group_stride, b1_row_stride   bf16 linear1 outputs, addressed as in bnb_conv_step_rows_fwd
 *   conv_in / conv_out  [p0|p1|p2] per row, fp32, as in bnb_conv_step_fwd (may be the same buffer)
 *   h_in / h_out        fp32 state rows, as in bnb_rglru_step_fwd (may be the same buffer)
 *   conv_weight (D,4), conv_bias (D) or NULL, fp32
 *   gate_weight_packed  bf16 [linear_a.weight ; linear_x.weight] (2D, D) in matrix-core operand
 *                       order [hf][q][ks][l][e], 32768 entries: entry = W[row, col] with
 *                       row = (q/2)*D + 64*hf + 32*(q%2) + 16*((l%32/4)%2) + 4*(l%32/8) + l%4,
 *                       col = 16*ks + 8*(l/32) + e     (hf<2, q<4, ks<8, l<64, e<8)
 *   gate_bias           fp32 (2D) = [linear_a.bias | linear_x.bias]; rounded to bf16 inside, as
 *                       autocast hands it to the GEMM
 *   log_lambda (D) fp32, c
 *   y, y_group_stride, y_row_stride   bf16 layer output = bf16(h'): row r at r*y_row_stride, or with
 *                       y_group_stride != 0 at (r / rows_per_env)*y_group_stride + (r % rows_per_env)*y_row_stride
 *                       (y_row_stride 0 = D; a column block of a wider tensor works)
 *   reset, rows_per_env as in the two kernels it replaces
 *
 * Requirements: D == 128, R < 2^31, 16-byte aligned pointers, row strides multiples of 4 (fp32)
 * or 8 (bf16) elements.  Gate pre-activations are accumulated in fp32 on the matrix cores and
 * rounded to bf16 once (the library GEMM's rounding point); summation order differs from the
 * library's, so single pre-activations may differ by one bf16 ulp.
 */
int bnb_temporal_step_fwd(const void *b1, int64_t b1_group_stride, int64_t b1_row_stride,
                          const float *conv_in, int64_t conv_in_row_stride,
                          float *conv_out, int64_t conv_out_row_stride,
                          const float *h_in, int64_t h_in_row_stride,
                          float *h_out, int64_t h_out_row_stride,
                          const float *conv_weight, const float *conv_bias,
                          const void *gate_weight_packed, const float *gate_bias,
                          const float *log_lambda, float c,
                          void *y, int64_t y_group_stride, int64_t y_row_stride,
                          const uint8_t *reset, int rows_per_env,
                          int64_t R, int D, void *stream);

/*
 * The same causal depthwise conv over a whole sequence of T steps per row, with episode
 * boundaries.
 *
 * Replaces, in models/yemong/griffin.py: `padded = cat([conv_buf, b1], dim=1)` (:275),
 * _causal_conv_tap_validity (:67-93), the tap loop of _causal_depthwise_conv (:127-139) and
 * `new_conv_buf = padded[:, -3:]` (:277) of GriffinTemporalBlock.forward_sequence.
 *
 *   b1        (R, T, D) contiguous, b1_dtype; with time_major != 0 the sequence tensors
 *             b1, v_out and v_bf16_out are (T, R, D) instead (every step's rows together,
 *             the layout the policy keeps rollouts in); done stays (R, T)
 *   conv_in   the three inputs stored before the sequence, [p0 | p1 | p2] per row as in
 *             bnb_conv_step_fwd; they count as part of the episode running at t = 0
 *   done      optional (R, T) bytes: non-zero at t ends an episode at t, so outputs after t
 *             take no tap from inputs at or before t; NULL = no boundaries
 *   v_out     (R, T, D) fp32 contiguous; v_bf16_out optional bf16 copy
 *   conv_out  the last three entries of [conv_in, b1] per row (not cut at boundaries, as in
 *             the reference); may equal conv_in
 * Requirements: T >= 1, strides >= 3*D; vector path as for bnb_conv_step_fwd (weight 16-byte
 * aligned), scalar path otherwise.
 *
 * rows_per_env, env_row_pitch (both 0: b1 holds exactly the R rows): with time_major, b1 may be a wider token
 * tensor (T, R / rows_per_env * env_row_pitch, D) of which this call's rows are the first rows_per_env of every
 * env_row_pitch rows; the reference runs its temporal block on the ship tokens of a (ships | fields) tensor
 * (models/yemong/policy.py: the split before the temporal sublayer), this reads them where they lie.  The
 * outputs stay dense (R rows).  bnb_conv_seq_bwd: b1 and db1 are placed that way (db1's other rows are not written);
 * bnb_rglru_scan_fwd: y; bnb_rglru_scan_bwd: y and dy.
 */
int bnb_conv_seq_fwd(const void *b1, int b1_dtype,
                     const float *conv_in, int64_t conv_in_row_stride,
                     const float *weight, const float *bias, const uint8_t *done,
                     float *v_out, void *v_bf16_out, float *conv_out, int64_t conv_out_row_stride,
                     int64_t R, int T, int D, int time_major, int rows_per_env, int env_row_pitch, void *stream);

/*
 * Backward of bnb_conv_seq_fwd: what autograd computes through griffin.py:67-140,275-277 in the
 * PPO update (train/rl/ppo.py:1417-1425), where the reference's tap loop becomes a dozen
 * element-wise kernels per tap and direction.
 *
 *   b1, conv_in, weight, done, time_major  as passed to the forward
 *   dv         gradient of v_out, fp32, b1's layout
 *   dv_bf16    gradient of v_bf16_out (bf16, b1's layout), added to dv element by element, or NULL
 *   dconv_out  gradient of conv_out, (R, 3, D) fp32 contiguous, or NULL
 *   db1        gradient of b1, b1's dtype and layout
 *   dconv_in   gradient of conv_in, (R, 3, D) fp32 contiguous
 *   partials   (blocks, 5*D) fp32 workspace; blocks from bnb_conv_seq_bwd_blocks(R, T, D)
 *   dwb        5*D floats, overwritten: the tap gradients as (D, 4), then the bias gradient (D);
 *              rows and steps are added in a fixed order (no atomics)
 * Requirements: D in {64, 128, 256, 512}, 16-byte aligned pointers, conv_in_row_stride % 4 == 0.
 */
int bnb_conv_seq_bwd_blocks(int64_t R, int T, int D);
int bnb_conv_seq_bwd(const void *b1, int b1_dtype, const float *conv_in, int64_t conv_in_row_stride,
                     const float *weight, const uint8_t *done, const float *dv, const void *dv_bf16,
                     const float *dconv_out, void *db1, float *dconv_in, float *partials, int blocks, float *dwb,
                     int64_t R, int T, int D, int time_major, int rows_per_env, int env_row_pitch, void *stream);

/*
 * RG-LRU over a whole sequence: T recurrence steps per row in one pass.
 *
 * Replaces RGLRU.forward_sequence, models/yemong/griffin.py:188-219: the gate sigmoids, the
 * decay a = sigmoid(log_lambda)^(c r), b = sqrt(clamp((1-a)(1+a), 1e-6)) (i x), the reset of
 * a after an episode end (:213-218) and the Hillis-Steele scan (:25-64) that evaluates
 * h_t = a_t h_{t-1} + b_t in log2(T) rounds over padded copies of a and b.  Here the
 * recurrence is evaluated in time order with the state in registers, so a and b are never
 * stored; results agree with the scan to fp32 rounding (the order of the multiply-adds
 * differs).  Element arithmetic and roundings as in bnb_rglru_step_fwd.
 *
 *   x          (R, T, D) contiguous, x_dtype; with time_major != 0, x, gates_pre and y are
 *              (T, R, .) instead; done stays (R, T)
 *   gates_pre  (R, T, 2*D) contiguous, g_dtype: [linear_a(x) | linear_x(x)] per step
 *   h0         (R, D) fp32 state before the sequence, row stride h0_row_stride floats
 *   done       optional (R, T) bytes: non-zero at t makes step t+1 start from a zero state
 *   y          (R, T, D) contiguous in y_dtype: every state h_0 .. h_{T-1}
 *   h_last     (R, D) fp32 state after the sequence (= h_{T-1}); may equal h0
 * T == 0 copies h0 to h_last.
 */
int bnb_rglru_scan_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                       const float *log_lambda, float c,
                       const float *h0, int64_t h0_row_stride, const uint8_t *done,
                       void *y, int y_dtype, float *h_last, int64_t h_last_row_stride,
                       int64_t R, int T, int D, int time_major, int rows_per_env, int env_row_pitch, void *stream);

/*
 * Backward of bnb_rglru_scan_fwd: what autograd computes through the reference's coefficient
 * chain and log-depth scan (models/yemong/griffin.py:206-219, :25-64), as one reverse-time
 * pass.  The forward's inputs and its states y are passed back in; r, i, a and the gate are
 * recomputed from them.
 *
 *   x, gates_pre, log_lambda, c, h0, done, time_major   as given to the forward
 *   y          the forward's states, y_dtype (float32 keeps h_{t-1} exact)
 *   dy         gradient of y, same dtype and layout as y, or NULL (zero)
 *   dh_last    optional (R, D) fp32 gradient of the final state
 *   dx         out, x's dtype and layout
 *   dgates     out, gates_pre's dtype and layout: [d linear_a | d linear_x]
 *   dh0        out (R, D) fp32 contiguous
 *   dlam_rows  out (R, D) fp32 contiguous: each row's contribution to d log_lambda; the
 *              caller sums over rows (kept separate so that the sum has a fixed order)
 * Requirements: T >= 1.
 */
int bnb_rglru_scan_bwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                       const float *log_lambda, float c,
                       const float *h0, int64_t h0_row_stride, const uint8_t *done,
                       const void *y, int y_dtype, const void *dy,
                       const float *dh_last, int64_t dh_last_row_stride,
                       void *dx, void *dgates, float *dh0, float *dlam_rows,
                       int64_t R, int T, int D, int time_major, int rows_per_env, int env_row_pitch, void *stream);

/*
 * Residual add + RMSNorm (+ the cast in front of the next projection) in one pass:
 *     s = x + delta            (delta optional)
 *     n = s * rsqrt(mean(s^2) + eps) * weight
 * Replaces `x = x + <sublayer output>` followed by `self.norm*(x)` in
 * models/yemong/attention.py:97-98 and models/yemong/griffin.py:269,284-285 (nn.RMSNorm(D),
 * eps = finfo(float32).eps), and the fp32 -> bf16 copy autocast puts before the next Linear.
 *
 *   x         (R, D) fp32 residual stream, row r at x + r*x_row_stride
 *   delta     optional (R, D) contiguous, delta_dtype (a bf16 Linear output under autocast)
 *   weight    (D) fp32
 *   sum_out   optional (R, D) fp32 contiguous: s (only with delta)
 *   norm_out  (R, D) contiguous in out_dtype
 * Requirements: D in {8,16,32,64,128,256,512}; 16-byte aligned pointers.
 */
int bnb_add_rmsnorm_fwd(const float *x, int64_t x_row_stride, const void *delta, int delta_dtype,
                        const float *weight, float eps, float *sum_out, void *norm_out, int out_dtype,
                        int64_t R, int D, void *stream);

/*
 * RMSNorm + Linear in one matrix-core kernel (bf16 projection), optionally over gathered rows:
 *     out[r] = bf16( rmsnorm(x[src(r)]) * norm_weight @ W^T + bias ),   src(r) = row_index ? row_index[r] : r
 * Replaces `self.kv_bullet(self.norm_bullet(bullets))` (models/yemong/attention.py:150-151),
 * `self.qkv(self.norm1(x))` (:94-96,132) and `self.linear1(self.norm1(x))`
 * (models/yemong/griffin.py:269-272) as they run under bf16 autocast.
 *
 *   x              fp32 rows of 128 channels, x_row_stride floats apart
 *   row_index      optional int32 list: output row r reads x row row_index[r] (a compact list of
 *                  the bullets in flight, see bnb_mask_fill); NULL = identity
 *   n_rows         optional device-side int32 count: only the first *n_rows rows are produced
 *                  (work-groups past it exit), so a data-dependent row count never reaches the
 *                  host; NULL = R rows.  R is then the capacity the grid is sized for.
 *   weight_packed  W (N, 128) in bf16, arranged as [fb][ks][l][e] =
 *                  W[32fb + 16((r/8)/2) + 8((r/4)%2) + 4((r/8)%2) + r%4][16ks + 8(e/4) + 4(l/32) + e%4],
 *                  r = l%32, fb = 0..N/32-1, ks = 0..7, l = 0..63, e = 0..7
 *   bias           optional fp32 (N)
 *   out            (R, N) bf16 contiguous
 * Requirements: D == 128, N % 64 == 0, 16-byte aligned pointers.  The normalisation factor
 * is applied to the products (a per-row scalar), the operand is bf16(x * norm_weight).
 */
int bnb_norm_linear_fwd(const float *x, int64_t x_row_stride, const int32_t *row_index,
                        const int32_t *n_rows, const float *norm_weight, float eps,
                        const void *weight_packed, const float *bias, void *out,
                        int64_t R, int D, int N, void *stream);

/*
 * bnb_norm_linear_fwd for the PPO update (train/rl/ppo.py:1417-1425 re-evaluates the rollout in grad mode): the same
 * launch also writes the normalised rows the projection multiplied, n = bf16(rmsnorm(x) * norm_weight), which are what
 * autograd would keep of `self.qkv(self.norm1(x))` (models/yemong/attention.py:94-96,132) and
 * `self.linear1(self.norm1(x))` (models/yemong/griffin.py:269-272) for the weight gradient; the norm's own forward
 * launch and the re-read of n by the projection disappear.
 *   n_out   (R, 128) bf16 contiguous
 *   other arguments as bnb_norm_linear_fwd (all rows, no bias)
 */
int bnb_norm_linear_train_fwd(const float *x, int64_t x_row_stride, const float *norm_weight, float eps,
                              const void *weight_packed, void *out, void *n_out, int64_t R, int D, int N, void *stream);

/*
 * A float32 Linear layer with its neighbours folded in, on the fp32 matrix cores (true fp32 products):
 *     out[r] = A[r] W^T + bias (+ resid[r]),   A[r] = x[r]                          (norm_weight, x2 NULL)
 *                                                   | rmsnorm(x[r]) * norm_weight     (norm_weight given; K == 128)
 *                                                   | gelu(x[r]) * x2[r]              (x2 given)
 *     gate != 0: W holds gate_proj and up_proj interleaved in blocks of 32 rows, out[r][u] = gelu(g[r][u]) * up[r][u]
 * Replaces, for a policy that runs without autocast (evaluation/agents.py:214-219), every Linear of the trunk
 * together with the element-wise passes around it: `self.qkv(self.norm1(x))` (models/yemong/attention.py:94-96,
 * 132-135), `x + self.out_proj(..)` (:97,168-169), `F.gelu(gate_proj(n)) * up_proj(n)` on `norm2(x)` (:36-37,98),
 * `x + down_proj(..)` (:37,98); `linear1` / `linear2` on `norm1(x)` (models/yemong/griffin.py:269-272,279),
 * `linear_a` / `linear_x` (:166-167,208-209), `x + linear_out(b1_out * gelu(linear2(..)))` (:281-284) and the same
 * gated MLP (:285-286).
 *
 *   x, x2          (R, K) fp32 rows, x_row_stride / x2_row_stride floats apart (multiples of 4, 16-byte aligned)
 *   norm_weight    (128) fp32 or NULL; eps as in nn.RMSNorm
 *   weight_packed  W (N, K) as [fb][s4][l][e] = W[32 fb + l%32][(l/32) K/2 + 4 s4 + e], fb < N/32, s4 < K/8,
 *                  l < 64, e < 4 (with gate: blocks 2u, 2u+1 = rows 32u.. of gate_proj, of up_proj)
 *   bias           (N) fp32 or NULL (not with gate)
 *   resid          optional (R, N_out) fp32 rows added to the result; may equal out
 *   out            (R, N_out) fp32 rows, N_out = N, or N/2 with gate
 * Requirements: K % 128 == 0, N % 32 == 0 (N % 64 with gate); anything else returns BNB_ERR_UNSUPPORTED.
 */
int bnb_linear_f32_fwd(const float *x, int64_t x_row_stride, const float *x2, int64_t x2_row_stride,
                       const float *norm_weight, float eps, const float *weight_packed, const float *bias,
                       const float *resid, int64_t resid_row_stride, float *out, int64_t out_row_stride, int64_t R,
                       int K, int N, int gate, void *stream);

/*
 * Compact list of the set entries of a byte mask (B, n), e.g. the bullets in flight of
 * models/yemong/policy.py:222-228: bnb_mask_count writes the number of set bytes per row;
 * the caller turns the counts into exclusive offsets (B+1, last = total); bnb_mask_fill writes
 * index[offsets[b] + k] = b*n + j for the k-th set byte j of row b, ascending.  Nothing is
 * copied to the host.
 */
int bnb_mask_count(const uint8_t *mask, int32_t *counts, int B, int n, void *stream);
int bnb_mask_fill(const uint8_t *mask, const int32_t *offsets, int32_t *index, int B, int n, void *stream);

/*
 * Residual add + RMSNorm + gated MLP + residual add in one matrix-core kernel (bf16 compute):
 *     s = x + delta;  n = rmsnorm(s) * norm_weight;  out = s + Wd (gelu(Wg n) * (Wu n))
 * Replaces `x = x + <attention output>` and `x + self.ffn(self.norm2(x))` of
 * models/yemong/attention.py:97-99 with GatedMLP (:21-37), and the same tail of the temporal
 * block (models/yemong/griffin.py:284-286), as they run under bf16 autocast: the residual add,
 * nn.RMSNorm, the casts, three Linear layers, F.gelu, the product and the last residual add.
 *
 *   x               (R, 128) fp32 residual stream, row stride x_row_stride floats
 *   delta           optional (R, 128) bf16 contiguous (the sublayer output to add first); NULL = none
 *   norm_weight     (128) fp32; eps as in nn.RMSNorm
 *   weights_packed  gate_proj, up_proj (512 x 128) and down_proj (128 x 512) in bf16, arranged
 *                   as the kernel's operand order (16 chunks of 32 hidden units, 24 KB each):
 *                   [c][0][ks][l][e] = Wg[32c + l%32][16ks + 8(e/4) + 4(l/32) + e%4]
 *                   [c][1][ks][l][e] = Wu[...same...]                          ks = 0..7
 *                   [c][2][cb][t][l][e] = Wd[32cb + l%32][32c + 16t + 8(e/4) + 4(l/32) + e%4]
 *                   with l = 0..63, e = 0..7, cb = 0..3, t = 0..1
 *   out             (R, 128) fp32 contiguous; may equal x when x is contiguous
 * Requirements: D == 128, hidden == 512 (else BNB_ERR_UNSUPPORTED), 16-byte aligned pointers.
 * Operands of the three projections are bf16 as under autocast; between them the kernel rounds
 * less often than the library composition (gate/up results stay fp32 until gelu(g) * u is
 * rounded once; the down projection is added to s in fp32).
 */
int bnb_ffn_fused_fwd(const float *x, int64_t x_row_stride, const void *delta, int delta_dtype,
                      const float *norm_weight, float eps, const void *weights_packed, float *out,
                      int64_t R, int D, int hidden, void *stream);

/*
 * bnb_ffn_fused_proj_fwd that goes on to the head of the NEXT sublayer: a norm and a projection of the rows it
 * has just produced (`self.qkv(self.norm1(x))`, models/yemong/attention.py:94-96,132; `linear1` / `linear2` of
 * `self.norm1(x)`, models/yemong/griffin.py:269-283), so that those rows do not come back from memory for it and
 * the separate norm + projection launch (bnb_norm_linear_fwd) disappears:
 *     next_out = bf16( bf16(rmsnorm(out) * next_norm_weight) Wh^T )
 *
 *   next_packed    Wh (next_features, 128) in bf16, 64 features per chunk:
 *                  [c][b][ks][l][e] = Wh[64c + 32b + pi(l%32)][16ks + 8(e/4) + 4(l/32) + e%4],
 *                  b = 0..1, ks = 0..7, l = 0..63, e = 0..7, pi(m) = 16(m/16) + 8((m/4)%2) + 4((m/8)%2) + m%4
 *   next_out       (next_out_rows, next_features) bf16 contiguous; next_out_rows >= R rounded up to a multiple of
 *                  128: the kernel stores whole work-groups of 128 rows (rows past R receive don't-care values)
 *   next_features  a multiple of 64, at least 128
 *   other arguments as bnb_ffn_fused_proj_fwd (rows_b == NULL: plain projection; else the gelu-gate form)
 */
int bnb_ffn_fused_proj_next_fwd(const float *x, int64_t x_row_stride, const void *rows_a, int64_t rows_a_stride,
                                const void *rows_b, int64_t rows_b_stride, const void *proj_packed,
                                const float *norm_weight, float eps, const void *weights_packed, float *out,
                                const float *next_norm_weight, float next_eps, const void *next_packed,
                                void *next_out, int next_features, int64_t next_out_rows, int64_t R, int D,
                                int hidden, void *stream);

/*
 * bnb_ffn_fused_fwd for the PPO update (train/rl/ppo.py:1417-1425 evaluating the trunk in grad mode):
 * the same kernel also writes what the backward needs and the forward would otherwise not keep,
 *   s_out  (R, 128) fp32 contiguous: s = x + delta (required with a delta; ignored without, where s is x)
 *   n_out  (R, 128) bf16 contiguous: the normalised rows that entered gate_proj / up_proj
 * so that none of the 512/1024-wide activations has to be saved (bnb_ffn_bwd recomputes them).
 */
int bnb_ffn_fused_train_fwd(const float *x, int64_t x_row_stride, const void *delta, int delta_dtype,
                            const float *norm_weight, float eps, const void *weights_packed, float *out,
                            float *s_out, void *n_out, int64_t R, int D, int hidden, void *stream);

/*
 * bnb_ffn_fused_train_fwd with the sublayer's output projection inside, as bnb_ffn_fused_proj_fwd has it
 * (rows_b == NULL form): s = x + rows_a Wp^T is formed on the matrix cores and written to s_out; the
 * projection's output never exists in memory.  For `x + out_proj(merged heads)` followed by the gated-MLP
 * tail (models/yemong/attention.py:97-99,168-169) in the PPO update.
 */
int bnb_ffn_fused_proj_train_fwd(const float *x, int64_t x_row_stride, const void *rows_a, int64_t rows_a_stride,
                                 const void *proj_packed, const float *norm_weight, float eps,
                                 const void *weights_packed, float *out, float *s_out, void *n_out, int64_t R,
                                 int D, int hidden, void *stream);

/*
 * Backward of the gated MLP  y = Wd (gelu(Wg n) * (Wu n))  of models/yemong/attention.py:21-37 (what autograd
 * runs through GatedMLP.forward under bf16 autocast) as one matrix-core kernel that recomputes the
 * gate/up activations from n:
 *     g, u = Wg n, Wu n;   dh = Wd^T dy;   h = bf16(gelu(g) u);
 *     dg = bf16(dh u gelu'(g));  du = bf16(dh gelu(g));   dn = bf16(Wg^T dg + Wu^T du)
 *
 *   n    (R, 128) bf16 contiguous (bnb_ffn_fused_train_fwd's n_out)
 *   dy   (R, 128) fp32 or bf16 (dy_dtype), rows dy_row_stride elements apart; used rounded to bf16
 *   weights_packed  the three matrices in bf16 in the kernel's operand order, 16 chunks of 32 hidden
 *        units, 40 KB each; with l = 0..63, m = l%32, b = l/32, e = 0..7,
 *        pi(m) = 16(m/16) + 8((m/4)%2) + 4((m/8)%2) + m%4:
 *          [c][0][ks][l][e] = Wg[32c + pi(m)][16ks + 8b + e]      ks = 0..7
 *          [c][1][ks][l][e] = Wu[32c + pi(m)][16ks + 8b + e]
 *          [c][2][ks][l][e] = Wd[16ks + 8b + e][32c + pi(m)]
 *          [c][3][cb][t][l][e] = Wg[32c + 16t + 8b + e][32cb + pi(m)]   cb = 0..3, t = 0..1
 *          [c][4][cb][t][l][e] = Wu[32c + 16t + 8b + e][32cb + pi(m)]
 *   out_rows  rows that every result has room for: a multiple of 256, >= R.  The kernel stores whole
 *        work-groups of 256 rows without a bounds test (rows R .. out_rows-1 receive don't-care values)
 *   dn   (out_rows, 128) bf16 contiguous: gradient of n in rows 0 .. R-1
 *   dgu  (8, out_rows, 128) bf16: tile p holds, for hidden chunks 2p and 2p+1 (32 units each),
 *        [dg chunk 2p | du chunk 2p | dg chunk 2p+1 | du chunk 2p+1]
 *   h    (4, out_rows, 128) bf16: tile q holds hidden units 128q .. 128q+127
 *        (both are operands for bnb_linear_wgrad_tiled_fwd with tile stride out_rows * 128: dW(gate,up) =
 *        dgu^T n in dgu's column order, dWd = dy^T h)
 *   dy_bf16  optional (out_rows, 128) bf16 contiguous: dy rounded to bf16, when dy is fp32 (the other operand of dWd)
 * Requirements: D == 128, hidden == 512 (else BNB_ERR_UNSUPPORTED), 16-byte aligned pointers.
 */
int bnb_ffn_bwd(const void *n, const void *dy, int dy_dtype, int64_t dy_row_stride, const void *weights_packed,
                void *dn, void *dgu, void *h, void *dy_bf16, int64_t R, int64_t out_rows, int D, int hidden,
                void *stream);

/*
 * bnb_ffn_fused_fwd with the sublayer's output projection folded in: the tensor added to x
 * before the norm is  rows_a Wp^T  (rows_b == NULL: `out_proj` of models/yemong/attention.py:168-169
 * applied to the merged attention heads) or  (bf16(gelu(rows_a)) * rows_b) Wp^T  (the temporal
 * block's `linear_out(b1_out * gelu(linear2(normed)))`, models/yemong/griffin.py:281-284),
 * computed on the matrix cores and accumulated straight onto x; the projection's output never
 * exists in memory.
 *
 *   rows_a, rows_b  (R, 128) bf16, rows rows_a_stride / rows_b_stride elements apart
 *                   (0 = 128; a column block of a wider projection output works)
 *   proj_packed     Wp (128, 128) in bf16 as [cb][ks][l][e] = Wp[32cb + l%32][16ks + 8(e/4) + 4(l/32) + e%4]
 *   other arguments as bnb_ffn_fused_fwd
 */
int bnb_ffn_fused_proj_fwd(const float *x, int64_t x_row_stride, const void *rows_a, int64_t rows_a_stride,
                           const void *rows_b, int64_t rows_b_stride,
                           const void *proj_packed, const float *norm_weight, float eps,
                           const void *weights_packed, float *out, int64_t R, int D, int hidden, void *stream);

/*
 * out = gelu(a) * b with the exact (erf) GELU, the gelu rounded to a's dtype as F.gelu does and
 * the product rounded once to out_dtype.  Replaces `F.gelu(gate_proj(x)) * up_proj(x)`
 * (models/yemong/attention.py:36-37) and `b1_out * F.gelu(linear2(normed))`
 * (models/yemong/griffin.py:281-282).  a and b are (R, H) with row strides in elements (the
 * two halves of one (R, 2H) projection output work), out is (R, H) contiguous.
 * Requirements: H % 8 == 0; 16-byte aligned rows.
 */
int bnb_gelu_mul_fwd(const void *a, int a_dtype, int64_t a_row_stride, const void *b, int b_dtype,
                     int64_t b_row_stride, void *out, int out_dtype, int64_t R, int H, void *stream);

/*
 * Backward of bnb_gelu_mul_fwd: da = dout * b * gelu'(a), db = dout * gelu(a), each rounded once
 * to its tensor's dtype; what autograd runs as two multiplications and a gelu-backward kernel
 * through attention.py:36-37 / griffin.py:281-282 in the PPO update (train/rl/ppo.py:1417-1425).
 * dout is (R, H) contiguous in out_dtype; da and db are (R, H) with row strides in elements.
 * Requirements as for the forward.
 */
int bnb_gelu_mul_bwd(const void *a, int a_dtype, int64_t a_row_stride, const void *b, int b_dtype,
                     int64_t b_row_stride, const void *dout, int out_dtype, void *da, int64_t da_row_stride,
                     void *db, int64_t db_row_stride, int64_t R, int H, void *stream);

/*
 * Plain device-to-device copy of `bytes` bytes (multiple of 16, 16-byte aligned) by a
 * grid of 16-byte loads and stores.  It has no counterpart in the reference: it is the
 * yardstick the benchmark uses for achievable HBM bandwidth and for scaling hardware
 * byte counters.
 */
int bnb_copy_bytes(const void *src, void *dst, int64_t bytes, void *stream);

/*
 * Issue-rate yardstick.  It has no counterpart in the reference: like bnb_copy_bytes for the bandwidth-bound
 * kernels, it gives the benchmark the hardware figure that bounds the matrix-core kernels of this library (the
 * gated MLP of models/yemong/attention.py:21-37 and the attention of :147 spend their time issuing matrix
 * products and vector arithmetic on the same SIMDs).  One launch runs, on `waves_per_simd` (1 or 2) waves per SIMD
 * of every compute unit, `iters` rounds of four slots; a slot is one 32x32x16 bf16 matrix product (if
 * `with_mfma`) followed by `valu_per_mfma` (0, 2, 4, 8, 10, 12 or 16) independent vector instructions:
 * multiply-adds, every fifth one an exp2 if `with_transcendentals`.  The caller times the launch; time /
 * (4 iters waves_per_simd) is the issue time of one slot on one SIMD.  `sink` (>= 1 KiB) is never written.
 */
int bnb_issue_probe(int valu_per_mfma, int with_mfma, int with_transcendentals, int waves_per_simd, int iters,
                    float *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BNB_AMD_H */
