// Masked self-attention, one work-group per environment, heads streamed through LDS (gfx950).
//
// Same function as sdpa_mfma_kernel (models/yemong/attention.py:101-112,136-147,168): bf16, four
// heads of 32 channels, up to 160 tokens, dead keys compacted away, an environment without a live
// key averages V over all keys.  What differs is how the data gets to the matrix cores:
//
//   * The work-group owns ALL heads of its environment.  The alive row is read once and the list
//     of live keys (position -> token index) is built once, instead of once per head.
//   * K and V rows travel global -> LDS directly (global_load_lds_dwordx4: a wave moves 1 KB per
//     instruction, lane l filling LDS bytes 16 l .. 16 l + 15 of the wave's kilobyte), never
//     through registers, so the next head's rows are in flight while the current head is being
//     computed and no lane spends instructions on staging.  Two LDS buffers alternate.
//   * A staged key is 128 bytes: [K 64 B | V 64 B] of one head, i.e. eight 16-byte chunks.  A
//     lane may fetch ANY global chunk into its fixed LDS slot, so chunk c of position p is kept in
//     slot c ^ f(p), f(p) = 2 (p%4) + (p/4)%2: eight consecutive keys put one chunk into eight
//     different slots (K operand reads: 16 B of each of 32 keys), and four consecutive keys put a
//     32-byte chunk pair into four different pairs (V operand reads: 32 B of each of 4 keys per
//     16 lanes), so both spread over all banks although the key pitch is a power of two.
//   * V stays row-major.  The A operand of O^T = V^T P^T needs, per lane, eight keys of ONE
//     channel; ds_read_b64_tr_b16 delivers exactly that from row-major data: inside a group of 16
//     lanes, lane i receives element i%4 of the 8-byte pieces addressed by lanes i/4, i/4 + 4,
//     i/4 + 8, i/4 + 12.  Source lane r therefore points at key (r/4) of the four keys wanted and
//     at the 4-channel block r%4 of the group's 16 output rows.  The eight 2-byte LDS writes per
//     item that a transposed copy of V costs are gone.
//
// Thread roles: wave w owns queries 32w .. 32w+31 (S^T = K Q^T with keys on the M axis, so a lane
// holds 16 scores of one query per key block; softmax reductions are in-lane plus one exchange
// between the wave's halves), for every head in turn.  Padding (positions [0, pad) of key block 0)
// is filled with a copy of the first live key and enters as -inf through the initial accumulator.

#include "common.h"

#include <stdlib.h>

#include <type_traits>

namespace bnb {

constexpr int kEnvDh = 32;
constexpr int kEnvHeads = 4;
constexpr int kEnvD = kEnvDh * kEnvHeads;
constexpr int kEnvKeyBytes = 128;  // one staged key of one head: [K | V]

// 16 bytes per lane from `sbase + voff` to LDS byte address lds_base + 16 * lane.  No immediate
// offset: the instruction would add it to the LDS address as well as to the global one.
__device__ __forceinline__ void dma_row16(const void *sbase, uint32_t voff, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                 :
                 : "s"(sbase), "v"(voff), "s"(lds_base)
                 : "memory", "m0");
}

// slot permutation of the eight 16-byte chunks of staged key p (p % 8 passed in)
__device__ __forceinline__ int swizzle(int p8) { return ((p8 & 3) << 1) | ((p8 >> 2) & 1); }

__device__ __forceinline__ bf16x8 lds_tr_pair(const uint16_t *p)
{
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    typedef bf16x4_t __attribute__((address_space(3))) * lds_ptr;
    const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)p);
    const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)(p + 8 * kEnvKeyBytes / 2));  // eight keys further on
    return bf16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

template <int NQB>
__global__ __launch_bounds__(kWave * NQB, 4) void sdpa_env_kernel(const uint16_t *__restrict__ qkv, int64_t stride,
                                                              const uint8_t *__restrict__ alive, uint16_t *__restrict__ out,
                                                              int B, int NM, int envs_per_group, float scale_log2e)
{
    constexpr int KCAP = NQB * 32;
    constexpr int H = kEnvHeads, D = kEnvD;
    // exactly 2 x 20 KB at 160 tokens: three work-groups share a CU only up to 40 KB each (measured), so the
    // list of live keys is kept out of LDS memory (every wave derives its part from the alive row by itself)
    __shared__ __align__(1024) uint16_t s_buf[2][KCAP * kEnvKeyBytes / 2];

    // A work-group walks environments first, first + step, ...; while it computes one, the next one's
    // alive row, key list, queries and first head are already on their way.
    const int first = blockIdx.x;
    const int step = envs_per_group;  // = gridDim.x
    const int last = B;               // exclusive
    if (first >= B) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;
    const int64_t env_pitch = (int64_t)NM * stride * step;

    // this lane's query: column m of every S^T block this wave forms
    const int qrow = wave * 32 + m;
    const int qsafe = qrow < NM ? qrow : NM - 1;
    const uint32_t q_off = (uint32_t)qsafe * (uint32_t)stride + half * 8;
    u32x4 qw[H][2];
    auto load_q = [&](const uint16_t *base, auto head_tag) {
        constexpr int h = decltype(head_tag)::value;
        qw[h][0] = *reinterpret_cast<const u32x4 *>(base + q_off + h * kEnvDh);
        qw[h][1] = *reinterpret_cast<const u32x4 *>(base + q_off + h * kEnvDh + 16);
    };

    // ---- list of live keys (position -> token), once per environment, per wave, without LDS memory ----
    // Every wave reads the whole alive row (lane l: tokens l, l + 64, l + 128) and keeps it as three
    // 64-bit masks; the token at live position n is the index of the n-th set bit.
    struct AliveRow { uint32_t a[3]; };
    auto load_alive = [&](int env) -> AliveRow {
        AliveRow r;
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            const int tok = lane + 64 * w;
            r.a[w] = 0u;
            if (w * 64 < KCAP) {
                const uint32_t in = tok < NM ? 1u : 0u;
                r.a[w] = alive == nullptr ? in : (in ? (uint32_t)alive[(int64_t)env * NM + tok] : 0u);
            }
        }
        return r;
    };
    struct KeyList { uint64_t m[3]; int c0, c1, cnt; bool uniform; };
    auto make_list = [&](const AliveRow &r) -> KeyList {
        KeyList k;
#pragma unroll
        for (int w = 0; w < 3; ++w) k.m[w] = __ballot(r.a[w] != 0);
        k.c0 = (int)__popcll(k.m[0]);
        k.c1 = (int)__popcll(k.m[1]);
        k.cnt = k.c0 + k.c1 + (int)__popcll(k.m[2]);
        // no live key at all: every key takes part with the same weight (all scores equal)
        k.uniform = k.cnt == 0;
        if (k.uniform) {
#pragma unroll
            for (int w = 0; w < 3; ++w) k.m[w] = __ballot(lane + 64 * w < NM);
            k.c0 = (int)__popcll(k.m[0]);
            k.c1 = (int)__popcll(k.m[1]);
            k.cnt = NM;
        }
        return k;
    };
    // index of the n-th set bit (n counted from 0, n < cnt) of the 160-bit row
    auto nth_live = [&](const KeyList &k, int n) -> int {
        uint64_t w = k.m[0];
        int base = 0;
        if (n >= k.c0) {
            n -= k.c0, w = k.m[1], base = 64;
            if (n >= k.c1) n -= k.c1, w = k.m[2], base = 128;
        }
        uint32_t x = (uint32_t)w;
        int c = __popc(x);
        if (n >= c) n -= c, x = (uint32_t)(w >> 32), base += 32;
#pragma unroll
        for (int width = 16; width >= 1; width >>= 1) {
            c = __popc(x & ((1u << width) - 1u));
            if (n >= c) n -= c, x >>= width, base += width;
        }
        return base;
    };

    // ---- the load instructions this wave issues per head: j = wave, wave + NQB, ... < 4 nkb ----
    // instruction j fills LDS kilobyte j of the buffer: lane l -> position 8j + l/8, slot l%8, which
    // holds global chunk (l%8) ^ f(position % 8) = (l%8) ^ f((l/8)%8)
    const int chunk = (lane & 7) ^ swizzle((lane >> 3) & 7);
    const uint32_t chan_bytes = (uint32_t)(((1 + (chunk >> 2)) * D + (chunk & 3) * 8) * 2);
    uint32_t voff[4];
    auto make_offsets = [&](const KeyList &k, int pad) {
        // lane t (and t + 32) works out the token of the wave's t-th position: instruction t/8, position t%8 in it;
        // padding positions hold a copy of the first live key; instructions past 4 nkb are never issued
        const int t = lane & 31;
        int n = (wave + (t >> 3) * NQB) * 8 + (t & 7) - pad;
        n = n > 0 ? n : 0;
        n = n < k.cnt ? n : k.cnt - 1;
        const int token = nth_live(k, n);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int tok = __builtin_amdgcn_ds_bpermute((jj * 8 + (lane >> 3)) * 4, token);
            voff[jj] = (uint32_t)tok * (uint32_t)stride * 2u + chan_bytes;
        }
    };
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)&s_buf[0][0];
    constexpr uint32_t kBufBytes = KCAP * kEnvKeyBytes;
    auto issue = [&](const uint16_t *base, auto head_tag, int ninstr) {
        constexpr int h = decltype(head_tag)::value;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int j = wave + jj * NQB;
            if (j < ninstr) dma_row16(base + h * kEnvDh, voff[jj], lds0 + (uint32_t)(h & 1) * kBufBytes + (uint32_t)j * 1024u);
        }
    };

    // ---- per-lane LDS offsets (halfs) of the operands inside a buffer, key block 0 ----
    // K (A operand of S^T): key m, channels 8 half .. (first product) and 16 + 8 half .. (second)
    const int ksw = swizzle(m & 7);
    const int k_off0 = m * (kEnvKeyBytes / 2) + ((half ^ ksw) * 8);
    const int k_off1 = m * (kEnvKeyBytes / 2) + (((2 + half) ^ ksw) * 8);
    // V (A operand of O^T through the transposing read): as SOURCE lane r = lane % 16 of group g = lane / 16
    // this lane points at key 4 (g/2) + r/4 of the 16 keys of one product and at output-row block
    // rb = 4 (g%2) + r%4, which is channel block cb(rb) (see the output stage: MFMA row 8i + 4 half + j
    // is channel 16 (i/2) + 8 half + 4 (i%2) + j, i.e. row block 2i + half -> channel block 4 (i/2) + 2 half + i%2)
    const int grp = lane >> 4, r = lane & 15;
    const int rb = 4 * (grp & 1) + (r & 3);
    const int cb = 4 * (rb >> 2) + 2 * (rb & 1) + ((rb >> 1) & 1);
    const int vkey = 4 * (grp >> 1) + (r >> 2);  // + 16 t + 32 kb (+ 8 for the second half of the operand)
    const int v_off = vkey * (kEnvKeyBytes / 2) + (((4 + (cb >> 1)) ^ swizzle(vkey & 7)) * 8) + (cb & 1) * 4;

    // ---- state of the environment being computed ----
    int nkb, pad;
    bool uniform;
    auto set_padding = [&](int cnt) {
        nkb = (cnt + 31) >> 5;
        pad = nkb * 32 - cnt;
    };
    // -inf for the padding positions of key block 0, as the initial accumulator there (made where it is used)
    auto pad_bias = [&](int pad_rows) -> f32x16 {
        f32x16 b;
#pragma unroll
        for (int v = 0; v < 16; ++v) b[v] = (8 * (v >> 2) + 4 * half + (v & 3) < pad_rows) ? -INFINITY : 0.0f;
        return b;
    };
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    u32x4 held[2];  // the last computed head's output, stored after the next barrier
    auto compute = [&](auto head_tag) {
        constexpr int h = decltype(head_tag)::value;
        const uint16_t *buf = &s_buf[h & 1][0];
        // with no live key every score is the same constant: zero queries give exactly that
        const bf16x8 qb0 = __builtin_bit_cast(bf16x8, uniform ? zero4 : qw[h][0]);
        const bf16x8 qb1 = __builtin_bit_cast(bf16x8, uniform ? zero4 : qw[h][1]);
        auto scores = [&](int kb, int pad_rows) -> f32x16 {
            const uint16_t *kp = buf + kb * 32 * (kEnvKeyBytes / 2);
            const bf16x8 ka0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp + k_off0));
            const bf16x8 ka1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp + k_off1));
            f32x16 z = {0.0f};
            if (kb == 0) z = pad_bias(pad_rows);
            z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0, qb0, z, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka1, qb1, z, 0, 0, 0);
        };
        // weights without a shift first (one sweep), with the maximum as shift when a query's sum leaves the safe
        // exponent range: the same arithmetic as sdpa_mfma_kernel, whose results this kernel repeats bit for bit
        const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        float sum = 0.0f;
        f32x16 o = {0.0f};
        auto sweep = [&](auto shifted, float mc, int pad_rows) {
            sum = 0.0f;
#pragma unroll
            for (int v = 0; v < 16; ++v) o[v] = 0.0f;
            for (int kb = 0; kb < nkb; ++kb) {
                const f32x16 z = scores(kb, pad_rows);
                float p[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    if constexpr (decltype(shifted)::value) p[v] = __builtin_amdgcn_exp2f(fmaf(z[v], scale_log2e, -mc));
                    else p[v] = __builtin_amdgcn_exp2f(z[v] * scale_log2e);
                }
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    bf16x8 pb;
#pragma unroll
                    for (int e = 0; e < 8; ++e) pb[e] = (__bf16)p[8 * t + e];
#pragma unroll
                    for (int e = 0; e < 8; e += 2) sum = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{pb[e], pb[e + 1]}, ones, sum, false);
                    const bf16x8 va = lds_tr_pair(buf + (kb * 32 + 16 * t) * (kEnvKeyBytes / 2) + v_off);
                    o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb, o, 0, 0, 0);
                }
            }
            sum += __shfl_xor(sum, 32);
        };
        sweep(std::false_type{}, 0.0f, pad);
        if (!__all(sum >= 0x1p-60f && sum <= 0x1p60f)) {
            int pad_again = pad;
            asm volatile("" : "+v"(pad_again));  // a value of its own: nothing of the first try is kept for this one
            float mx = -INFINITY;
            for (int kb = 0; kb < nkb; ++kb) {
                const f32x16 z = scores(kb, pad_again);
#pragma unroll
                for (int v = 0; v < 16; ++v) mx = fmaxf(mx, z[v]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            sweep(std::true_type{}, mx * scale_log2e, pad_again);
        }
        const float inv = __builtin_amdgcn_rcpf(sum);
#pragma unroll
        for (int g = 0; g < 2; ++g)
            held[g] = u32x4{pack_bf16x2(o[8 * g + 0] * inv, o[8 * g + 1] * inv), pack_bf16x2(o[8 * g + 2] * inv, o[8 * g + 3] * inv),
                            pack_bf16x2(o[8 * g + 4] * inv, o[8 * g + 5] * inv), pack_bf16x2(o[8 * g + 6] * inv, o[8 * g + 7] * inv)};
    };
    auto store = [&](int env, int h) {
        if (qrow < NM) {
            uint16_t *op = out + ((int64_t)env * NM + qrow) * D + h * kEnvDh + 8 * half;
            *reinterpret_cast<u32x4 *>(op) = held[0];
            *reinterpret_cast<u32x4 *>(op + 16) = held[1];
        }
    };
    // Everything a wave has in flight (its share of a head's rows, queries of the next environment,
    // the previous head's output) was issued a whole head earlier, so the wait is a plain vmcnt(0);
    // the barrier then says both "everybody's rows of this head have landed" and "everybody is done
    // with the previous head", whose buffer the head after this one may now overwrite.
    auto next_head = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
        __syncthreads();
    };
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    using H2 = std::integral_constant<int, 2>;
    using H3 = std::integral_constant<int, 3>;

    // ---- first environment of the run: nothing to hide the set-up behind ----
    int env = first;
    const uint16_t *env_base = qkv + (int64_t)env * NM * stride;
    load_q(env_base, H0{});
    load_q(env_base, H1{});
    load_q(env_base, H2{});
    load_q(env_base, H3{});
    {
        const KeyList k = make_list(load_alive(env));
        uniform = k.uniform;
        set_padding(k.cnt);
        make_offsets(k, pad);
        issue(env_base, H0{}, nkb * 4);
    }

    AliveRow row_next = {{0u, 0u, 0u}};
    for (;;) {
        const bool more = env + step < last;
        const uint16_t *next_base = env_base + env_pitch;
        // ---- head 0 (buffer 0); head 1 starts to land in buffer 1 ----
        next_head();
        if (env != first) store(env - step, 3);
        issue(env_base, H1{}, nkb * 4);
        if (more) row_next = load_alive(env + step);
        compute(H0{});
        // ---- head 1; head 2 into buffer 0 ----
        next_head();
        store(env, 0);
        issue(env_base, H2{}, nkb * 4);
        if (more) load_q(next_base, H0{});
        compute(H1{});
        // ---- head 2; head 3 into buffer 1 ----
        next_head();
        store(env, 1);
        issue(env_base, H3{}, nkb * 4);
        if (more) load_q(next_base, H1{});
        compute(H2{});
        // ---- head 3; the next environment's key list, and its head 0 into buffer 0 ----
        next_head();
        store(env, 2);
        bool uniform_next = false;
        int cnt_next = 0;
        if (more) {
            load_q(next_base, H2{});
            const KeyList k = make_list(row_next);
            uniform_next = k.uniform;
            cnt_next = k.cnt;
            const int nkb_next = (cnt_next + 31) >> 5;
            make_offsets(k, nkb_next * 32 - cnt_next);
            issue(next_base, H0{}, nkb_next * 4);
        }
        compute(H3{});
        if (!more) break;
        load_q(next_base, H3{});
        uniform = uniform_next;
        set_padding(cnt_next);
        env_base = next_base;
        env += step;
    }
    store(env, 3);
}

// ------------------------------------------------------------------------------------
// One work-group per (environment, head): the same data path (rows straight into LDS, key list per wave from
// the alive row, V through the transposing read) with the occupancy of the small work-group: 20 KB of LDS and
// 64 registers, so six work-groups of five waves share a CU and one's loads hide behind the others' arithmetic.
// One barrier per work-group; nothing is staged by the lanes.
// ------------------------------------------------------------------------------------
template <int NQB>
__global__ __launch_bounds__(kWave * NQB, 8) void sdpa_head_kernel(const uint16_t *__restrict__ qkv, int64_t stride,
                                                                  const uint8_t *__restrict__ alive, uint16_t *__restrict__ out,
                                                                  int B, int NM, int H, float scale_log2e)
{
    constexpr int KCAP = NQB * 32;
    __shared__ __align__(1024) uint16_t s_buf[KCAP * kEnvKeyBytes / 2];

    // work-groups are dealt round-robin to the 8 XCDs; hand each XCD a contiguous run of (environment, head)
    // pairs so the heads of an environment (adjacent 64-byte segments of the same rows) share one L2
    const int chunk_wg = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk_wg + (blockIdx.x >> 3);
    if (logical >= B * H) return;
    const int env = logical / H;
    const int head = logical - env * H;
    const int D = H * kEnvDh;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;
    const uint16_t *env_base = qkv + (int64_t)env * NM * stride + head * kEnvDh;

    // this lane's query
    const int qrow = wave * 32 + m;
    const int qsafe = qrow < NM ? qrow : NM - 1;
    const uint16_t *qp = env_base + (uint32_t)qsafe * (uint32_t)stride + half * 8;
    u32x4 qw0 = *reinterpret_cast<const u32x4 *>(qp);
    u32x4 qw1 = *reinterpret_cast<const u32x4 *>(qp + 16);

    // the alive row as three 64-bit masks (lane l: tokens l, l + 64, l + 128)
    uint64_t mk[3];
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        const int tok = lane + 64 * w;
        uint32_t a = 0u;
        if (w * 64 < KCAP) {
            const uint32_t in = tok < NM ? 1u : 0u;
            a = alive == nullptr ? in : (in ? (uint32_t)alive[(int64_t)env * NM + tok] : 0u);
        }
        mk[w] = __ballot(a != 0);
    }
    int c0 = (int)__popcll(mk[0]), c1 = (int)__popcll(mk[1]);
    int cnt = c0 + c1 + (int)__popcll(mk[2]);
    // no live key at all: every key takes part with the same weight (all scores equal)
    const bool uniform = cnt == 0;
    if (uniform) {
#pragma unroll
        for (int w = 0; w < 3; ++w) mk[w] = __ballot(lane + 64 * w < NM);
        c0 = (int)__popcll(mk[0]), c1 = (int)__popcll(mk[1]);
        cnt = NM;
    }
    const int nkb = (cnt + 31) >> 5;
    const int pad = nkb * 32 - cnt;  // positions [0, pad) of key block 0 hold a copy of the first live key

    // the token of this wave's t-th staged position (t = lane % 32: instruction t/8, position t%8 in it)
    int token;
    {
        const int t = lane & 31;
        int n = (wave + (t >> 3) * NQB) * 8 + (t & 7) - pad;
        n = n > 0 ? n : 0;
        n = n < cnt ? n : cnt - 1;
        uint64_t w = mk[0];
        int base = 0;
        if (n >= c0) {
            n -= c0, w = mk[1], base = 64;
            if (n >= c1) n -= c1, w = mk[2], base = 128;
        }
        uint32_t x = (uint32_t)w;
        int c = __popc(x);
        if (n >= c) n -= c, x = (uint32_t)(w >> 32), base += 32;
#pragma unroll
        for (int width = 16; width >= 1; width >>= 1) {
            c = __popc(x & ((1u << width) - 1u));
            if (n >= c) n -= c, x >>= width, base += width;
        }
        token = base;
    }
    // instruction j = wave + jj * NQB fills LDS kilobyte j: lane l -> position 8j + l/8, slot l%8 = chunk ^ f(position)
    const int chunk = (lane & 7) ^ swizzle((lane >> 3) & 7);
    const uint32_t chan_bytes = (uint32_t)(((1 + (chunk >> 2)) * D + (chunk & 3) * 8) * 2);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)&s_buf[0];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        const int j = wave + jj * NQB;
        const int tok = __builtin_amdgcn_ds_bpermute((jj * 8 + (lane >> 3)) * 4, token);
        if (j < nkb * 4) dma_row16(env_base, (uint32_t)tok * (uint32_t)stride * 2u + chan_bytes, lds0 + (uint32_t)j * 1024u);
    }

    const int ksw = swizzle(m & 7);
    const int k_off0 = m * (kEnvKeyBytes / 2) + ((half ^ ksw) * 8);
    const int k_off1 = m * (kEnvKeyBytes / 2) + (((2 + half) ^ ksw) * 8);
    const int grp = lane >> 4, r = lane & 15;
    const int rb = 4 * (grp & 1) + (r & 3);
    const int cb = 4 * (rb >> 2) + 2 * (rb & 1) + ((rb >> 1) & 1);
    const int vkey = 4 * (grp >> 1) + (r >> 2);
    const int v_off = vkey * (kEnvKeyBytes / 2) + (((4 + (cb >> 1)) ^ swizzle(vkey & 7)) * 8) + (cb & 1) * 4;

    if (uniform) qw0 = qw1 = u32x4{0u, 0u, 0u, 0u};
    const bf16x8 qb0 = __builtin_bit_cast(bf16x8, qw0);
    const bf16x8 qb1 = __builtin_bit_cast(bf16x8, qw1);
    auto pad_bias = [&](int pad_rows) -> f32x16 {
        f32x16 b;
#pragma unroll
        for (int v = 0; v < 16; ++v) b[v] = (8 * (v >> 2) + 4 * half + (v & 3) < pad_rows) ? -INFINITY : 0.0f;
        return b;
    };

    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's rows and its queries
    __syncthreads();                      // everybody's rows

    auto scores = [&](int kb, int pad_rows) -> f32x16 {
        const uint16_t *kp = s_buf + kb * 32 * (kEnvKeyBytes / 2);
        const bf16x8 ka0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp + k_off0));
        const bf16x8 ka1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp + k_off1));
        f32x16 z = {0.0f};
        if (kb == 0) z = pad_bias(pad_rows);
        z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0, qb0, z, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka1, qb1, z, 0, 0, 0);
    };
    // weights without a shift first (one sweep), with the maximum as shift when a query's sum leaves the safe
    // exponent range: the same arithmetic as sdpa_mfma_kernel, whose results this kernel repeats bit for bit
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    float sum = 0.0f;
    f32x16 o = {0.0f};
    auto sweep = [&](auto shifted, float mc, int pad_rows) {
        sum = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) o[v] = 0.0f;
        for (int kb = 0; kb < nkb; ++kb) {
            const f32x16 z = scores(kb, pad_rows);
            float p[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                if constexpr (decltype(shifted)::value) p[v] = __builtin_amdgcn_exp2f(fmaf(z[v], scale_log2e, -mc));
                else p[v] = __builtin_amdgcn_exp2f(z[v] * scale_log2e);
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                bf16x8 pb;
#pragma unroll
                for (int e = 0; e < 8; ++e) pb[e] = (__bf16)p[8 * t + e];
#pragma unroll
                for (int e = 0; e < 8; e += 2) sum = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{pb[e], pb[e + 1]}, ones, sum, false);
                const bf16x8 va = lds_tr_pair(s_buf + (kb * 32 + 16 * t) * (kEnvKeyBytes / 2) + v_off);
                o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb, o, 0, 0, 0);
            }
        }
        sum += __shfl_xor(sum, 32);
    };
    sweep(std::false_type{}, 0.0f, pad);
    if (!__all(sum >= 0x1p-60f && sum <= 0x1p60f)) {
        int pad_again = pad;
        asm volatile("" : "+v"(pad_again));  // a value of its own: nothing of the first try is kept for this one
        float mx = -INFINITY;
        for (int kb = 0; kb < nkb; ++kb) {
            const f32x16 z = scores(kb, pad_again);
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, z[v]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        sweep(std::true_type{}, mx * scale_log2e, pad_again);
    }
    const float inv = __builtin_amdgcn_rcpf(sum);
    if (qrow < NM) {
        uint16_t *op = out + ((int64_t)env * NM + qrow) * D + head * kEnvDh + 8 * half;
#pragma unroll
        for (int g = 0; g < 2; ++g)
            *reinterpret_cast<u32x4 *>(op + 16 * g) =
                u32x4{pack_bf16x2(o[8 * g + 0] * inv, o[8 * g + 1] * inv), pack_bf16x2(o[8 * g + 2] * inv, o[8 * g + 3] * inv),
                      pack_bf16x2(o[8 * g + 4] * inv, o[8 * g + 5] * inv), pack_bf16x2(o[8 * g + 6] * inv, o[8 * g + 7] * inv)};
    }
}

template <int NQB>
static int launch_head(const void *qkv, int64_t stride, const uint8_t *alive, void *out, int B, int NM, int H, hipStream_t stream)
{
    const int64_t pairs = (int64_t)B * H;
    const int64_t blocks = (pairs + 7) / 8 * 8;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((sdpa_head_kernel<NQB>), dim3((unsigned)blocks), dim3(kWave * NQB), 0, stream, (const uint16_t *)qkv, stride,
                       alive, (uint16_t *)out, B, NM, H, 1.4426950408889634f / sqrtf((float)kEnvDh));
    return (int)hipGetLastError();
}

// bf16, heads of 32 channels, 1 <= NM <= 160, rows of one environment within 2^31 bytes.
int dispatch_head(const void *qkv, int64_t stride, const uint8_t *alive, void *out, int B, int NM, int H, hipStream_t stream)
{
    switch ((NM + 31) / 32) {
        case 1: return launch_head<1>(qkv, stride, alive, out, B, NM, H, stream);
        case 2: return launch_head<2>(qkv, stride, alive, out, B, NM, H, stream);
        case 3: return launch_head<3>(qkv, stride, alive, out, B, NM, H, stream);
        case 4: return launch_head<4>(qkv, stride, alive, out, B, NM, H, stream);
        case 5: return launch_head<5>(qkv, stride, alive, out, B, NM, H, stream);
        default: return BNB_ERR_UNSUPPORTED;
    }
}

template <int NQB>
static int launch_env(const void *qkv, int64_t stride, const uint8_t *alive, void *out, int B, int NM, hipStream_t stream)
{
    // environments per work-group: long enough runs to hide each environment's set-up behind the one before,
    // short enough that the hardware still has several times more work-groups than slots to balance with
    // (BNB_ENV_GROUP overrides the choice: a tuning and testing knob)
    int groups = B;
    if (const char *e = getenv("BNB_ENV_GROUP")) groups = atoi(e) > 0 ? atoi(e) : groups;
    if (groups > B) groups = B;
    const int per = groups;
    hipLaunchKernelGGL((sdpa_env_kernel<NQB>), dim3((unsigned)groups), dim3(kWave * NQB), 0, stream, (const uint16_t *)qkv, stride,
                       alive, (uint16_t *)out, B, NM, per, 1.4426950408889634f / sqrtf((float)kEnvDh));
    return (int)hipGetLastError();
}

// bf16, 4 heads of 32 channels, 1 <= NM <= 160, rows of one environment within 2^31 bytes.
int dispatch_env(const void *qkv, int64_t stride, const uint8_t *alive, void *out, int B, int NM, hipStream_t stream)
{
    switch ((NM + 31) / 32) {
        case 1: return launch_env<1>(qkv, stride, alive, out, B, NM, stream);
        case 2: return launch_env<2>(qkv, stride, alive, out, B, NM, stream);
        case 3: return launch_env<3>(qkv, stride, alive, out, B, NM, stream);
        case 4: return launch_env<4>(qkv, stride, alive, out, B, NM, stream);
        case 5: return launch_env<5>(qkv, stride, alive, out, B, NM, stream);
        default: return BNB_ERR_UNSUPPORTED;
    }
}

}  // namespace bnb
