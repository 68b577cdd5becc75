/*
 * Plain-C restatement of the attention + RG-LRU step.  TEST INFRASTRUCTURE ONLY:
 * the shipped library never links or loads this file; tests, the smoke check and
 * the benchmark's CPU-baseline leg use it as a checker that shares no code with
 * the HIP kernels or with torch.
 *
 * Inputs are float32 arrays (bf16 data is widened by the caller), arithmetic is
 * double, results are rounded to float32 once at the end.  Paths cited below are
 * relative to the reference checkout, src/boost_and_broadside/.
 *
 * Build: make -C oracle   (gcc -O2 -shared -fPIC, output oracle/libbnb_oracle.so)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

/* fp32 and bf16 flavours of finfo(dtype).min / 2, models/yemong/attention.py:110-112 */
static const double NEG_F32 = -1.7014117331926443e38;
static const double NEG_BF16 = -1.6947656946257677e38;

/*
 * Masked multi-head attention for B environments of NM tokens.
 *   qkv    (B, NM, 3*H*dh) rows of `row_stride` floats, columns [Q | K | V], each
 *          third split into H runs of dh columns (models/yemong/attention.py:135-140)
 *   alive  (B, NM) bytes, non-zero = exists; NULL = no mask (attention.py:142-145)
 *   out    (B, NM, H*dh) contiguous, heads merged head-major (attention.py:168)
 * A dead key gets the additive constant above; the sum score+constant is rounded
 * to float32, which is what turns an all-dead environment into an exactly uniform
 * average over every key (attention.py:147 with the bias of :101-112).
 */
int oracle_sdpa_masked(const float *qkv, int64_t row_stride, const uint8_t *alive, float *out,
                       int B, int NM, int H, int dh, int bf16_bias)
{
    const int D = H * dh;
    const double neg = bf16_bias ? NEG_BF16 : NEG_F32;
    const double scale = 1.0 / sqrt((double)dh);
    double *w = (double *)malloc(sizeof(double) * (size_t)NM);
    if (!w) return 1;
    for (int b = 0; b < B; ++b) {
        const float *env = qkv + (int64_t)b * NM * row_stride;
        for (int hd = 0; hd < H; ++hd) {
            for (int i = 0; i < NM; ++i) {
                const float *q = env + (int64_t)i * row_stride + hd * dh;
                double m = -INFINITY;
                for (int j = 0; j < NM; ++j) {
                    const float *k = env + (int64_t)j * row_stride + D + hd * dh;
                    double s = 0.0;
                    for (int d = 0; d < dh; ++d) s += (double)q[d] * (double)k[d];
                    s *= scale;
                    if (alive && !alive[(int64_t)b * NM + j]) s = (double)((float)s + (float)neg);
                    w[j] = s;
                    if (s > m) m = s;
                }
                double z = 0.0;
                for (int j = 0; j < NM; ++j) { w[j] = exp(w[j] - m); z += w[j]; }
                float *o = out + ((int64_t)b * NM + i) * D + hd * dh;
                for (int d = 0; d < dh; ++d) {
                    double acc = 0.0;
                    for (int j = 0; j < NM; ++j)
                        acc += w[j] * (double)env[(int64_t)j * row_stride + 2 * D + hd * dh + d];
                    o[d] = (float)(acc / z);
                }
            }
        }
    }
    free(w);
    return 0;
}

/*
 * One RG-LRU update for R rows of D channels (models/yemong/griffin.py:179-186):
 *   r = sigmoid(gates[:, :D]); i = sigmoid(gates[:, D:]); a = sigmoid(lambda)^(c r)
 *   h' = a h + sqrt(max((1-a)(1+a), 1e-6)) (i x)
 * gates (R, 2D) holds linear_a(x) then linear_x(x) (griffin.py:166-167); h_in and
 * h_out are addressed through row strides in floats so that they may point into a
 * packed (.., 4D) state tensor (models/yemong/policy.py:323).
 */
int oracle_rglru_step(const float *x, const float *gates, const float *log_lambda, float c,
                      const float *h_in, int64_t h_in_stride, float *h_out, int64_t h_out_stride,
                      int64_t R, int D)
{
    for (int64_t row = 0; row < R; ++row) {
        for (int d = 0; d < D; ++d) {
            double r = 1.0 / (1.0 + exp(-(double)gates[row * 2 * D + d]));
            double i = 1.0 / (1.0 + exp(-(double)gates[row * 2 * D + D + d]));
            double sig = 1.0 / (1.0 + exp(-(double)log_lambda[d]));
            double a = pow(sig, (double)c * r);
            double g = (1.0 - a) * (1.0 + a);
            if (g < 1e-6) g = 1e-6;
            h_out[row * h_out_stride + d] =
                (float)(a * (double)h_in[row * h_in_stride + d] + sqrt(g) * (i * (double)x[row * D + d]));
        }
    }
    return 0;
}
