// libbonsai_decode.so: the ops between the packed GEMVs of one decode step on gfx950.
//
//   qk_norm_rope_kernel   split + per-head q/k RMSNorm + RoPE + KV write
//                         (src/bonsai_sft/gpu/model.py:388-436)
//   attn_mfma_kernel      softmax(q k^T) v over a run of 64-slot chunks of the shared KV for a
//                         tile of (row, query head) pairs, on the matrix cores
//   attn_combine_parts_kernel   merges the runs, rounds to bf16 and quantises per token
//                         (src/bonsai_sft/gpu/model.py:996-1005)
//   attn_partial_kernel / attn_combine_kernel   the VALU form of the same two steps
//                         (one wave per query head, row group and chunk), selectable
//   kv_commit_kernel      workspace rows -> history rows (fast_runtime.py:467-508)
//   draft_rows_kernel / draft_accept_kernel   argmax + confidence chain
//                         (src/bonsai_sft/gpu/fast_generate.py:111-130)
//   bf16_linear_kernel    bf16 lm_head of a sign-weight backbone (model.py:1296)
//   fp8_quant_rows_kernel / fp8_linear_kernel   E4M3 draft projection (model.py:1168-1194,
//                         1268-1275)
//
// Attention is HBM/L2-bound integer-free fp work: per layer it reads
// 2 * n_kv * (cache_len + M) * 256 bytes of KV once per tile of 16 (row, query head) pairs.  The mask
// is not a tensor: history visibility is `slot < cache_len && slot != hide`, workspace
// visibility one 32-bit word per row, both read from a small device descriptor, so a
// replayed graph only touches the live part of the buffer.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>

#include "../../include/bonsai_decode.h"
#include "wave_reduce.h"

namespace {

constexpr int kHd = BONSAI_HEAD_DIM;
constexpr int kChunk = BONSAI_ATTN_CHUNK;
constexpr int kPartStride = kHd + 4;  // 128 accumulators + running max + running sum, 16-byte pitch

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ float bf16_round(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    bf16x2_t x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    return __builtin_amdgcn_fdot2_f32_bf16(x, y, c, false);
}

__device__ __forceinline__ float wave_max(float v) { return bonsai_wave::max64(v); }
__device__ __forceinline__ float wave_sum(float v) { return bonsai_wave::sum64(v); }

// ---------------------------------------------------------------------------
// q/k RMSNorm + RoPE + KV write.  One wave per (token, head); lane i holds the
// element pair (i, i + 64), which is the pair rotate_half exchanges.
// The sum of squares is accumulated in fp64 (lane pair, then an xor butterfly), so
// its fp32 value does not depend on the summation order to within one rounding.
// ---------------------------------------------------------------------------
struct RopeArgs {
    const uint16_t *xqkv;
    const uint16_t *qw;
    const uint16_t *kw;
    const uint16_t *cos_t;
    const uint16_t *sin_t;
    const int32_t *positions;
    uint16_t *q_out;
    uint16_t *k_layer;
    uint16_t *v_layer;
    float eps;
    int M, n_heads, n_kv, slots, write_slot, max_pos;
};

// RMSNorm + RoPE of one 128-wide head row by one wave: lane i holds the pair (i, i + 64) in
// (r0, r1) and receives the finished pair in (o0b, o1b) as bf16 bits.
// What a lane holds of one such row (bf16 bits): the pair, its norm weights, the cos / sin entries
// of the row's position.  Loading and arithmetic are apart so that a wave can have several rows'
// loads in flight.
struct RopeRowIn {
    uint32_t r0, r1, w0, w1, c0, c1, s0, s1;
};

__device__ __forceinline__ RopeRowIn rope_row_load(const uint16_t *x, const uint16_t *w,
                                                   const uint16_t *cos_t, const uint16_t *sin_t, int pos,
                                                   int max_pos, int lane) {
    pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
    const uint16_t *cr = cos_t + (size_t)pos * kHd;
    const uint16_t *sr = sin_t + (size_t)pos * kHd;
    return RopeRowIn{x[lane], x[lane + 64], w[lane], w[lane + 64], cr[lane], cr[lane + 64], sr[lane],
                     sr[lane + 64]};
}

__device__ __forceinline__ void rope_row_math(const RopeRowIn &in, float eps, uint32_t &o0b, uint32_t &o1b) {
    const float f0 = bf16_bits_to_f32(in.r0), f1 = bf16_bits_to_f32(in.r1);
    const double ss = bonsai_wave::sum64((double)(f0 * f0) + (double)(f1 * f1));
    const float var = (float)ss / (float)kHd;
    const float rs = 1.0f / sqrtf(var + eps);
    const float n0 = bf16_round(bf16_bits_to_f32(in.w0) * bf16_round(f0 * rs));
    const float n1 = bf16_round(bf16_bits_to_f32(in.w1) * bf16_round(f1 * rs));
    const float c0 = bf16_bits_to_f32(in.c0), c1 = bf16_bits_to_f32(in.c1);
    const float s0 = bf16_bits_to_f32(in.s0), s1 = bf16_bits_to_f32(in.s1);
    // rotate_half(n) = [-n_hi, n_lo]
    const float o0 = bf16_round(bf16_round(n0 * c0) + bf16_round(-n1 * s0));
    const float o1 = bf16_round(bf16_round(n1 * c1) + bf16_round(n0 * s1));
    o0b = f32_to_bf16_bits(o0);
    o1b = f32_to_bf16_bits(o1);
}

__global__ void __launch_bounds__(256)
qk_norm_rope_kernel(const uint16_t *pxqkv, const uint16_t *pqw, const uint16_t *pkw,
                    const uint16_t *pcos, const uint16_t *psin, const int32_t *ppos,
                    uint16_t *pq, uint16_t *pk, uint16_t *pv, float peps, int pM, int pheads,
                    int pkv, int pslots, int pwrite, int pmaxpos) {
    // scalar parameters (instead of one struct) so that they can be preloaded into SGPRs
    const RopeArgs a{pxqkv, pqw, pkw, pcos, psin, ppos, pq, pk, pv, peps,
                     pM, pheads, pkv, pslots, pwrite, pmaxpos};
    const int lane = threadIdx.x & 63;
    const int head = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int m = blockIdx.y;
    const int total_heads = a.n_heads + 2 * a.n_kv;
    if (head >= total_heads) return;
    const uint16_t *x = a.xqkv + ((size_t)m * total_heads + head) * kHd;
    const uint32_t r0 = x[lane], r1 = x[lane + 64];

    if (head >= a.n_heads + a.n_kv) {  // V: plain copy into the workspace row
        const int vh = head - a.n_heads - a.n_kv;
        uint16_t *dst = a.v_layer + ((size_t)vh * a.slots + a.write_slot + m) * kHd;
        dst[lane] = (uint16_t)r0;
        dst[lane + 64] = (uint16_t)r1;
        return;
    }
    const bool is_q = head < a.n_heads;
    uint32_t o0, o1;
    rope_row_math(rope_row_load(x, is_q ? a.qw : a.kw, a.cos_t, a.sin_t, a.positions[m], a.max_pos, lane),
                  a.eps, o0, o1);
    uint16_t *dst = is_q ? a.q_out + ((size_t)m * a.n_heads + head) * kHd
                         : a.k_layer + ((size_t)(head - a.n_heads) * a.slots + a.write_slot + m) * kHd;
    dst[lane] = (uint16_t)o0;
    dst[lane + 64] = (uint16_t)o1;
}

// ---------------------------------------------------------------------------
// Attention, split over KV chunks.  One wave per (kv head, query head of the group,
// chunk, row group of RW rows).  Logical sequence index t in [0, cache_len + M):
// t < cache_len is history slot t, otherwise workspace slot sigma + (t - cache_len).
//   phase 1 (lane = slot):  the lane keeps its K row (64 dwords) in registers; the q
//                           row is wave-uniform; s = scale * <q, k> with v_dot2_f32_bf16
//   softmax statistics of the chunk per row (wave reductions), p parked in LDS
//   phase 2 (lane = 2 dims): acc[r] += p[r][slot] * V[slot][dims], V rows read
//                           coalesced (256 B per slot)
// Partials: [M][n_heads][n_chunks][132] fp32 = 128 unnormalised sums, max, sum, 2 unused.
// The workgroup id puts the kv head in the low three bits, so with 8 kv heads all
// waves that share a kv head run on one XCD and share its L2.
// ---------------------------------------------------------------------------
struct AttnArgs {
    const uint32_t *q;        // [M][n_heads][64] bf16 pairs
    const uint32_t *k_layer;  // [n_kv][slots][64]
    const uint32_t *v_layer;
    const int32_t *meta;
    float *part;
    float scale_log2e;        // scale * log2(e): softmax runs in base 2
    int M, n_heads, n_kv, hpg, slots, sigma, n_chunks, row_groups;
};

template <int RW>
__global__ void __launch_bounds__(64)
attn_partial_kernel(const uint32_t *pq, const uint32_t *pk, const uint32_t *pv, const int32_t *pmeta,
                    float *ppart, float pscale, int pM, int pheads, int pkv, int phpg, int pslots,
                    int psigma, int pchunks, int prow_groups) {
    // scalar parameters (instead of one struct) so that they can be preloaded into SGPRs
    const AttnArgs a{pq, pk, pv, pmeta, ppart, pscale, pM, pheads, pkv, phpg, pslots,
                     psigma, pchunks, prow_groups};
    __shared__ __attribute__((aligned(16))) float p_lds[RW][kChunk];
    const int lane = threadIdx.x;
    int id = blockIdx.x;
    const int kvh = id % a.n_kv;
    id /= a.n_kv;
    const int chunk = id % a.n_chunks;
    id /= a.n_chunks;
    const int g = id % a.hpg;
    const int rg = id / a.hpg;
    const int head = kvh * a.hpg + g;

    // a descriptor that does not fit the segment is clamped, never followed out of bounds
    const int cache_len = min(max(a.meta[0], 0), a.sigma);
    const int hide = a.meta[1];
    const int total = cache_len + a.M;
    const int t0 = chunk * kChunk;
    if (t0 >= total) return;  // nothing live in this chunk; the combine step skips it too
    const int n_live = min(kChunk, total - t0);

    // ---- phase 1: scores of this lane's slot against RW rows
    const int t = t0 + lane;
    const bool live = lane < n_live;
    const int tc = live ? t : t0;  // clamped: dead lanes read a valid row and are masked
    const int slot = tc < cache_len ? tc : a.sigma + (tc - cache_len);
    const uint4 *krow = reinterpret_cast<const uint4 *>(a.k_layer + ((size_t)kvh * a.slots + slot) * 64);
    uint4 kreg[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) kreg[i] = krow[i];
    // the V rows of the chunk (lane = 2 dims) are requested now as well, so that the
    // kernel is one memory round trip long; rows past the live part repeat the last one
    const uint32_t *vbase = a.v_layer + (size_t)kvh * a.slots * 64 + lane;
    uint32_t vreg[kChunk];
#pragma unroll
    for (int j = 0; j < kChunk; ++j) {
        const int tj = min(t0 + j, total - 1);
        const int sj = tj < cache_len ? tj : a.sigma + (tj - cache_len);
        vreg[j] = vbase[(size_t)sj * 64];
    }

    const int row0 = rg * RW;
    float mrow[RW], lrow[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const int m = min(row0 + r, a.M - 1);
        const uint4 *qrow = reinterpret_cast<const uint4 *>(a.q + ((size_t)m * a.n_heads + head) * 64);
        float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint4 qv = qrow[i];  // wave-uniform address
            acc0 = dot2_bf16(kreg[i].x, qv.x, acc0);
            acc1 = dot2_bf16(kreg[i].y, qv.y, acc1);
            acc0 = dot2_bf16(kreg[i].z, qv.z, acc0);
            acc1 = dot2_bf16(kreg[i].w, qv.w, acc1);
        }
        bool vis = live;
        if (t < cache_len) {
            vis = vis && (t != hide);
        } else {
            const uint32_t wmask = (uint32_t)a.meta[2 + m];
            vis = vis && ((wmask >> ((t - cache_len) & 31)) & 1u);
        }
        const float sc = vis ? (acc0 + acc1) * a.scale_log2e : -INFINITY;
        const float mx = wave_max(sc);
        const float p = (mx == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(sc - mx);
        mrow[r] = mx;
        lrow[r] = wave_sum(p);
        p_lds[r][lane] = p;   // dead lanes hold 0
    }
    __syncthreads();

    // ---- phase 2: acc[r][2 dims] over the slots of the chunk (p is 0 for dead slots)
    float acc[RW][2];
#pragma unroll
    for (int r = 0; r < RW; ++r) acc[r][0] = acc[r][1] = 0.0f;
#pragma unroll
    for (int j = 0; j < kChunk; j += 4) {
        float4 pj[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) pj[r] = *reinterpret_cast<const float4 *>(&p_lds[r][j]);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float v0 = bf16_bits_to_f32(vreg[j + u] & 0xffffu);
            const float v1 = __uint_as_float(vreg[j + u] & 0xffff0000u);
#pragma unroll
            for (int r = 0; r < RW; ++r) {
                const float p = u == 0 ? pj[r].x : (u == 1 ? pj[r].y : (u == 2 ? pj[r].z : pj[r].w));
                acc[r][0] = fmaf(p, v0, acc[r][0]);
                acc[r][1] = fmaf(p, v1, acc[r][1]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const int m = row0 + r;
        if (m < a.M) {
            float *dst = a.part + (((size_t)m * a.n_heads + head) * a.n_chunks + chunk) * kPartStride;
            reinterpret_cast<float2 *>(dst)[lane] = make_float2(acc[r][0], acc[r][1]);
            if (lane == 0) {
                dst[kHd] = mrow[r];
                dst[kHd + 1] = lrow[r];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Matrix-core form of the chunk pass.  The VALU form above gives every (query head, row
// group) its own wave, so a chunk of K/V is fetched from L2 by heads-per-group x row-groups
// waves, each lane loading its own 256-byte row; from a few hundred slots on that L2
// traffic is what the launch waits for.  Here a workgroup of four waves takes a tile of up
// to 16 (row, query head) pairs of one kv head -- all query heads of the group and as many
// block rows as fit -- and a run of consecutive 64-slot chunks.  Wave w owns slots
// 16 w .. 16 w + 15 of the chunk for the scores and dims 32 w .. 32 w + 31 of the output:
//   S = Q K^T      4 x v_mfma_f32_16x16x32_bf16 per wave: A = the pair tile's q rows, B = K
//                  rows loaded straight in operand layout (lane = (slot, 8 dims of a 32-dim
//                  block): four lanes cover 64 contiguous bytes of a K row);
//   softmax        running max / sum per pair in base 2: the D layout keeps a pair's 16
//                  scores of the wave in one 16-lane row (DPP row reductions), the four
//                  waves exchange their maxima and sums through LDS; p is rounded to bf16
//                  as the reference's probabilities are (model.py:1001) and the sum is
//                  taken over the rounded values;
//   O += P V       4 more MFMAs per wave: V rows are fetched coalesced, staged in LDS (row
//                  pitch 288 bytes: conflict-free) and read back as 8 slots x 1 dim per
//                  lane; P goes through LDS into A-operand order.  The slot <-> (K-block,
//                  element) assignment of this MFMA is 32 js + 4 e + kb for both operands.
// The live chunks (from the descriptor) are divided evenly among the `parts` workgroups of
// a (kv head, pair tile); each writes one partial per pair: [M][n_heads][parts][132].
// ---------------------------------------------------------------------------
constexpr int kPairTile = 16;
constexpr int kVPitch = 2 * kHd + 32;      // bytes per staged V row
constexpr int kPPitch = 2 * kChunk + 16;   // bytes per staged P row
constexpr int kMaxParts = 16;
constexpr int kAttnWaves = 4;

typedef __bf16 attn_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float attn_f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ attn_bf16x8_t attn_as_bf16x8(const uint4 v) {
    attn_bf16x8_t r;
    __builtin_memcpy(&r, &v, 16);
    return r;
}

template <int CTRL>
__device__ __forceinline__ float row_share(float v) {
    const int x = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_update_dpp(x, x, CTRL, 0xF, 0xF, false));
}

// The merge of the partials of one (row, head): the 16 lanes of a DPP row hold the head, lane j
// dims 8 j .. + 8 of every live partial and the statistics of part j.  num = sum over the parts,
// in ascending order, of weight x accumulator, the weights normalised over the parts.
//
// DEVICE_SCOPE: the partials were stored by other workgroups of the SAME launch (device-scope
// stores, part_store below): the loads carry the device scope too, so that no L2 of another XCD's
// making is trusted for them.
constexpr int kBufferWord3 = 0x00020000;   // raw buffer, 32-bit format, range check on
constexpr int kDeviceScope = 16;           // cache-policy bit sc1 of buffer loads and stores

// `hbase` = part + head_off floats; with DEVICE_SCOPE `part` and `part_bytes` must be uniform.
template <bool DEVICE_SCOPE>
__device__ __forceinline__ void combine_head_slice(const float *part, int part_bytes, int head_off, int live,
                                                   int j, float (&num)[8]) {
    const float *hbase = part + head_off;
    // this thread's 8 dims of every live partial, and part j's statistics
    float4 x0[kMaxParts], x1[kMaxParts];
    float2 ml = make_float2(-INFINITY, 0.0f);
    if constexpr (DEVICE_SCOPE) {
        typedef unsigned int v4u __attribute__((ext_vector_type(4)));
        typedef unsigned int v2u __attribute__((ext_vector_type(2)));
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(part), 0, part_bytes, kBufferWord3);
#pragma unroll
        for (int c = 0; c < kMaxParts; ++c) {
            if (c < live) {  // uniform
                const int off = (head_off + c * kPartStride + 8 * j) * 4;
                const v4u a = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, kDeviceScope);
                const v4u b = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off + 16, 0, kDeviceScope);
                x0[c] = make_float4(__uint_as_float(a.x), __uint_as_float(a.y), __uint_as_float(a.z),
                                    __uint_as_float(a.w));
                x1[c] = make_float4(__uint_as_float(b.x), __uint_as_float(b.y), __uint_as_float(b.z),
                                    __uint_as_float(b.w));
            }
        }
        if (j < live) {
            const v2u t = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (head_off + j * kPartStride + kHd) * 4, 0, kDeviceScope);
            ml = make_float2(__uint_as_float(t.x), __uint_as_float(t.y));
        }
    } else {
#pragma unroll
        for (int c = 0; c < kMaxParts; ++c) {
            if (c < live) {  // uniform
                const float4 *src = reinterpret_cast<const float4 *>(hbase + (size_t)c * kPartStride + 8 * j);
                x0[c] = src[0];
                x1[c] = src[1];
            }
        }
        if (j < live) ml = *reinterpret_cast<const float2 *>(hbase + (size_t)j * kPartStride + kHd);
    }

    const float mx = bonsai_wave::max16(ml.x);
    const float e = (ml.x == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ml.x - mx);
    const float den = bonsai_wave::sum16(e * ml.y);
    const float wj = e * (den > 0.0f ? 1.0f / den : 0.0f);  // weight of part j

#pragma unroll
    for (int i = 0; i < 8; ++i) num[i] = 0.0f;
#define BONSAI_COMBINE_PART(C)                                                      \
    {                                                                               \
        const float wc = row_share<0x150 + (C)>(wj);                                \
        if ((C) < live) {                                                           \
            num[0] = fmaf(wc, x0[C].x, num[0]); num[1] = fmaf(wc, x0[C].y, num[1]); \
            num[2] = fmaf(wc, x0[C].z, num[2]); num[3] = fmaf(wc, x0[C].w, num[3]); \
            num[4] = fmaf(wc, x1[C].x, num[4]); num[5] = fmaf(wc, x1[C].y, num[5]); \
            num[6] = fmaf(wc, x1[C].z, num[6]); num[7] = fmaf(wc, x1[C].w, num[7]); \
        }                                                                           \
    }
    BONSAI_COMBINE_PART(0) BONSAI_COMBINE_PART(1) BONSAI_COMBINE_PART(2) BONSAI_COMBINE_PART(3)
    BONSAI_COMBINE_PART(4) BONSAI_COMBINE_PART(5) BONSAI_COMBINE_PART(6) BONSAI_COMBINE_PART(7)
    BONSAI_COMBINE_PART(8) BONSAI_COMBINE_PART(9) BONSAI_COMBINE_PART(10) BONSAI_COMBINE_PART(11)
    BONSAI_COMBINE_PART(12) BONSAI_COMBINE_PART(13) BONSAI_COMBINE_PART(14) BONSAI_COMBINE_PART(15)
#undef BONSAI_COMBINE_PART
}

// live parts of a step: the live chunks split into runs of ceil(live / parts)
__host__ __device__ inline int attn_chunks_per_part(int live_chunks, int parts) {
    return (live_chunks + parts - 1) / parts;
}

// ROPE: the launch takes the merged q|k|v projection instead of finished q rows and does the work
// of qk_norm_rope_kernel itself (a decode step of one token spends as long on that launch as on
// this one).  Every workgroup derives the q rows of its pair tile -- one wave per (token, head)
// row, the very arithmetic of qk_norm_rope_kernel -- and hands them to its waves through LDS; a workgroup whose chunks reach the block's own rows
// (logical index >= cache_len) derives those K rows the same way and takes the V rows from the
// projection, never from the cache, so no workgroup uses what another one writes; the workgroup
// of pair tile 0 that owns a row's chunk also writes it to the cache for the steps to come.
struct RopeIn {
    const uint16_t *qw, *kw, *cos_t, *sin_t;
    const int32_t *positions;
    float eps;
    int max_pos;
};

// FIN: no second launch.  A workgroup makes its partials visible to the device and counts itself
// in on its kv head's arrival counter; the one that finds all the others there merges the
// partials of its pair tile (combine_head_slice, what attn_combine_parts_kernel does), stores the
// rows as bf16 with one maximum of |value| per (row, kv head) -- the parts a projection with the
// maxima prologue quantises from -- and puts the counter back to zero.  Nobody waits.  Single
// pair tile only (M x heads per kv head <= 16).
struct FinOut {
    unsigned *arrivals;   // [n_kv], zero between launches
    uint16_t *out;        // bf16 [M, n_heads x 128]
    uint16_t *amax;       // bf16 [M, amax_ld]: entries n_kv .. amax_ld - 1 are set to zero
    int amax_ld;
};

template <bool ROPE, bool FIN>
__global__ void __launch_bounds__(kAttnWaves * 64)
attn_mfma_kernel(const uint16_t *q, uint16_t *k_layer, uint16_t *v_layer,
                 const int32_t *meta, float *part_out, float scale_log2e, int M, int n_heads,
                 int n_kv, int G, int slots, int sigma, int parts, const RopeIn rope, const FinOut fin) {
    __shared__ unsigned fin_last;
    __shared__ float fin_max[kPairTile];
    __shared__ __attribute__((aligned(16))) unsigned char v_lds[kChunk * kVPitch];
    __shared__ __attribute__((aligned(16))) uint16_t q_new[ROPE ? kPairTile : 1][kHd];
    __shared__ __attribute__((aligned(16))) uint16_t k_new[ROPE ? BONSAI_MAX_WIDTH : 1][kHd];
    __shared__ __attribute__((aligned(16))) uint16_t v_new[ROPE ? BONSAI_MAX_WIDTH : 1][kHd];
    __shared__ __attribute__((aligned(16))) unsigned char p_lds[kPairTile * kPPitch];
    __shared__ __attribute__((aligned(16))) float st_max[kAttnWaves][kPairTile];
    __shared__ __attribute__((aligned(16))) float st_sum[kAttnWaves][kPairTile];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = lane & 15, kb = lane >> 4;
    int id = blockIdx.x;
    const int kvh = id % n_kv;
    id /= n_kv;
    const int part = id % parts;
    const int pt = id / parts;

    // a descriptor that does not fit the segment is clamped, never followed out of bounds
    const int cache_len = min(max(meta[0], 0), sigma);
    const int hide = meta[1];
    const int total = cache_len + M;
    const int live_chunks = (total + kChunk - 1) / kChunk;
    const int cpw = attn_chunks_per_part(live_chunks, parts);
    const int c_begin = part * cpw;
    if (c_begin >= live_chunks) return;  // whole workgroup; the combine step counts the same parts
    const int c_end = min(c_begin + cpw, live_chunks);
    const int pairs_total = M * G;

    // the four pairs whose results this lane holds (D layout: tile rows 4 kb + r)
    bool valid[4];
    int row_of[4], head_of[4];
    uint32_t wmask[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int pd = pt * kPairTile + 4 * kb + r;
        valid[r] = pd < pairs_total;
        const int pc = valid[r] ? pd : pairs_total - 1;
        row_of[r] = pc / G;
        head_of[r] = kvh * G + (pc - row_of[r] * G);
        wmask[r] = (uint32_t)meta[2 + row_of[r]];
    }

    float m_run[4], l_run[4];
    attn_f32x4_t acc_o[2];  // dims 32 w + 16 x + col
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.0f;
    }
    acc_o[0] = acc_o[1] = attn_f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    const uint16_t *kbase = k_layer + (size_t)kvh * slots * kHd;
    const uint16_t *vbase = v_layer + (size_t)kvh * slots * kHd;
    // One chunk's operands of this wave, as named registers (arrays of them end up in
    // scratch memory): K of slot t0 + col, dims 32 j + 8 kb .. + 8 (the B operand of S; dead
    // slots repeat the last live one and are masked), and the V rows of the same 16 slots,
    // coalesced: lane = (row 4 i + kb, dims 8 col .. + 8).
    struct ChunkRegs {
        uint4 k0, k1, k2, k3, v0, v1, v2, v3;
    };
    auto load_chunk = [&](int c) {
        const int t0 = c * kChunk + 16 * w;
        ChunkRegs cr;
        {
            const int t = min(t0 + col, total - 1);
            const int slot = t < cache_len ? t : sigma + (t - cache_len);
            const uint4 *krow = reinterpret_cast<const uint4 *>(kbase + (size_t)slot * kHd);
            cr.k0 = krow[kb];
            cr.k1 = krow[4 + kb];
            cr.k2 = krow[8 + kb];
            cr.k3 = krow[12 + kb];
        }
        auto v_row = [&](int i) {
            const int t = min(t0 + 4 * i + kb, total - 1);
            const int slot = t < cache_len ? t : sigma + (t - cache_len);
            return reinterpret_cast<const uint4 *>(vbase + (size_t)slot * kHd)[col];
        };
        cr.v0 = v_row(0);
        cr.v1 = v_row(1);
        cr.v2 = v_row(2);
        cr.v3 = v_row(3);
        return cr;
    };
    // ROPE: the block's own rows come from LDS (uniform branch), whatever the cache slot held
    auto own_chunk_rows = [&](ChunkRegs &cr, int c) {
        const int t0 = c * kChunk + 16 * w;
        if (ROPE && (c + 1) * kChunk > cache_len) {
            {
                const int t = min(t0 + col, total - 1);
                const uint4 *kn = reinterpret_cast<const uint4 *>(k_new[min(max(t - cache_len, 0), M - 1)]);
                const uint4 n0 = kn[kb], n1 = kn[4 + kb], n2 = kn[8 + kb], n3 = kn[12 + kb];
                if (t >= cache_len) {
                    cr.k0 = n0;
                    cr.k1 = n1;
                    cr.k2 = n2;
                    cr.k3 = n3;
                }
            }
            auto v_own = [&](int i, uint4 &dst) {
                const int t = min(t0 + 4 * i + kb, total - 1);
                const uint4 n = reinterpret_cast<const uint4 *>(v_new[min(max(t - cache_len, 0), M - 1)])[col];
                if (t >= cache_len) dst = n;
            };
            v_own(0, cr.v0);
            v_own(1, cr.v1);
            v_own(2, cr.v2);
            v_own(3, cr.v3);
        }
    };

    // the first chunk's loads travel while the q rows are fetched or derived
    ChunkRegs cur = load_chunk(c_begin);
    // ROPE: `q` is the merged projection [M][n_heads + 2 n_kv][128]
    if constexpr (ROPE) {
        const bool own_rows = c_end * kChunk > cache_len;  // this workgroup reaches the block's rows
        const int total_heads = n_heads + 2 * n_kv;
        const int n_q = min(kPairTile, pairs_total - pt * kPairTile);
        const int n_jobs = n_q + (own_rows ? M : 0);
        // a job is one row: q row `job` of the tile, then K row (with its V row) job - n_q of the
        // block.  A wave takes kRowsInFlight jobs at a time and issues all their loads first.
        constexpr int kRowsInFlight = 4;
        const int wu = __builtin_amdgcn_readfirstlane(w);
        for (int base = 0; base < n_jobs; base += kRowsInFlight * kAttnWaves) {
            RopeRowIn in[kRowsInFlight];
            uint16_t v0[kRowsInFlight], v1[kRowsInFlight];
            int jm[kRowsInFlight];
#pragma unroll
            for (int j = 0; j < kRowsInFlight; ++j) {
                const int job = min(base + wu + j * kAttnWaves, n_jobs - 1);  // past the end: a repeat, unused
                const bool is_q = job < n_q;
                const int qp = pt * kPairTile + job;
                jm[j] = is_q ? qp / G : job - n_q;
                const int src_head = is_q ? kvh * G + (qp - jm[j] * G) : n_heads + kvh;
                in[j] = rope_row_load(q + ((size_t)jm[j] * total_heads + src_head) * kHd,
                                      is_q ? rope.qw : rope.kw, rope.cos_t, rope.sin_t,
                                      rope.positions[jm[j]], rope.max_pos, lane);
                const uint16_t *xv = q + ((size_t)jm[j] * total_heads + n_heads + n_kv + kvh) * kHd;
                v0[j] = xv[lane];
                v1[j] = xv[lane + 64];
            }
#pragma unroll
            for (int j = 0; j < kRowsInFlight; ++j) {
                const int job = base + wu + j * kAttnWaves;
                if (job >= n_jobs) break;  // uniform
                const bool is_q = job < n_q;
                const int m = jm[j];
                uint32_t o0, o1;
                rope_row_math(in[j], rope.eps, o0, o1);
                uint16_t *dst = is_q ? q_new[job] : k_new[m];
                dst[lane] = (uint16_t)o0;
                dst[lane + 64] = (uint16_t)o1;
                if (!is_q) {
                    v_new[m][lane] = v0[j];
                    v_new[m][lane + 64] = v1[j];
                    // the cache row, once: by the workgroup of pair tile 0 that owns the row's chunk
                    const int c_row = (cache_len + m) / kChunk;
                    if (pt == 0 && c_row >= c_begin && c_row < c_end) {
                        uint16_t *kd = k_layer + ((size_t)kvh * slots + sigma + m) * kHd;
                        uint16_t *vd = v_layer + ((size_t)kvh * slots + sigma + m) * kHd;
                        kd[lane] = (uint16_t)o0;
                        kd[lane + 64] = (uint16_t)o1;
                        vd[lane] = v0[j];
                        vd[lane + 64] = v1[j];
                    }
                }
            }
        }
        __syncthreads();
    }
    // A operand of S: this lane's pair (tile row `col`), dims 32 j + 8 kb .. + 8
    uint4 qreg[4];
    if constexpr (ROPE) {
        const int n_q = min(kPairTile, pairs_total - pt * kPairTile);
        const uint4 *qrow = reinterpret_cast<const uint4 *>(q_new[min(col, n_q - 1)]);
#pragma unroll
        for (int j = 0; j < 4; ++j) qreg[j] = qrow[4 * j + kb];
    } else {
        const int qp = min(pt * kPairTile + col, pairs_total - 1);
        const int qm = qp / G, qg = qp - qm * G;
        const uint4 *qrow =
            reinterpret_cast<const uint4 *>(q + ((size_t)qm * n_heads + kvh * G + qg) * kHd);
#pragma unroll
        for (int j = 0; j < 4; ++j) qreg[j] = qrow[4 * j + kb];
    }
    own_chunk_rows(cur, c_begin);
    for (int c = c_begin; c < c_end; ++c) {
        const int t0 = c * kChunk + 16 * w;  // this wave's 16 slots
        // the next chunk's loads go out before this one is worked on (uniform branch)
        ChunkRegs nxt = cur;
        if (c + 1 < c_end) {
            nxt = load_chunk(c + 1);
            own_chunk_rows(nxt, c + 1);
        }
        const uint4 kreg[4] = {cur.k0, cur.k1, cur.k2, cur.k3};
        const uint4 vreg0 = cur.v0, vreg1 = cur.v1, vreg2 = cur.v2, vreg3 = cur.v3;

        attn_f32x4_t s = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(attn_as_bf16x8(qreg[j]),
                                                        attn_as_bf16x8(kreg[j]), s, 0, 0, 0);
        // s[r]: pair 4 kb + r against slot t0 + col.  Visibility without branches: history
        // slots but the hidden one, workspace slots by the row's bit.
        float sc[4];
        {
            const int t = t0 + col;
            const uint32_t hist_ok = (uint32_t)(t < cache_len) & (uint32_t)(t != hide);
            const uint32_t in_ws = (uint32_t)(t >= cache_len) & (uint32_t)(t < total);
            const int sh = (t - cache_len) & 31;
            float mx[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t vis = (uint32_t)valid[r] & (hist_ok | (in_ws & (wmask[r] >> sh)));
                sc[r] = (vis & 1u) ? s[r] * scale_log2e : -INFINITY;
                mx[r] = bonsai_wave::max16(sc[r]);
            }
            if (col == 0)
                *reinterpret_cast<float4 *>(&st_max[w][4 * kb]) = make_float4(mx[0], mx[1], mx[2], mx[3]);
        }
        __syncthreads();

        float alpha[4], m_new[4];
        {
            const int tl = 16 * w + col;  // slot of the chunk
            // P in A-operand order: slot 32 js + 4 e + kb' sits at index 32 js + 8 kb' + e
            const int idx = (tl & 32) + 8 * (tl & 3) + ((tl & 31) >> 2);
            const float4 x0 = *reinterpret_cast<const float4 *>(&st_max[0][4 * kb]);
            const float4 x1 = *reinterpret_cast<const float4 *>(&st_max[1][4 * kb]);
            const float4 x2 = *reinterpret_cast<const float4 *>(&st_max[2][4 * kb]);
            const float4 x3 = *reinterpret_cast<const float4 *>(&st_max[3][4 * kb]);
            const float mc[4] = {fmaxf(fmaxf(x0.x, x1.x), fmaxf(x2.x, x3.x)),
                                 fmaxf(fmaxf(x0.y, x1.y), fmaxf(x2.y, x3.y)),
                                 fmaxf(fmaxf(x0.z, x1.z), fmaxf(x2.z, x3.z)),
                                 fmaxf(fmaxf(x0.w, x1.w), fmaxf(x2.w, x3.w))};
            float sum[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                m_new[r] = fmaxf(m_run[r], mc[r]);
                // nothing visible so far: the differences below are NaN and are replaced
                const bool none = m_new[r] == -INFINITY;
                const float a_raw = __builtin_amdgcn_exp2f(m_run[r] - m_new[r]);  // 0 at the first live chunk
                const float p_raw = __builtin_amdgcn_exp2f(sc[r] - m_new[r]);
                alpha[r] = none ? 1.0f : a_raw;
                // p in [0, 1]: round to nearest even on the bits, no NaN case
                uint32_t pu = __float_as_uint(none ? 0.0f : p_raw);
                pu = (pu + 0x7fffu + ((pu >> 16) & 1u)) & 0xffff0000u;
                *reinterpret_cast<uint16_t *>(p_lds + (4 * kb + r) * kPPitch + 2 * idx) =
                    (uint16_t)(pu >> 16);
                sum[r] = bonsai_wave::sum16(__uint_as_float(pu));
            }
            if (col == 0)
                *reinterpret_cast<float4 *>(&st_sum[w][4 * kb]) =
                    make_float4(sum[0], sum[1], sum[2], sum[3]);
        }
        {
            unsigned char *vdst = v_lds + (16 * w + kb) * kVPitch + 16 * col;
            *reinterpret_cast<uint4 *>(vdst) = vreg0;
            *reinterpret_cast<uint4 *>(vdst + 4 * kVPitch) = vreg1;
            *reinterpret_cast<uint4 *>(vdst + 8 * kVPitch) = vreg2;
            *reinterpret_cast<uint4 *>(vdst + 12 * kVPitch) = vreg3;
        }
        __syncthreads();

        {
            const float4 y0 = *reinterpret_cast<const float4 *>(&st_sum[0][4 * kb]);
            const float4 y1 = *reinterpret_cast<const float4 *>(&st_sum[1][4 * kb]);
            const float4 y2 = *reinterpret_cast<const float4 *>(&st_sum[2][4 * kb]);
            const float4 y3 = *reinterpret_cast<const float4 *>(&st_sum[3][4 * kb]);
            const float tot[4] = {((y0.x + y1.x) + y2.x) + y3.x, ((y0.y + y1.y) + y2.y) + y3.y,
                                  ((y0.z + y1.z) + y2.z) + y3.z, ((y0.w + y1.w) + y2.w) + y3.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                l_run[r] = l_run[r] * alpha[r] + tot[r];
                m_run[r] = m_new[r];
                acc_o[0][r] *= alpha[r];
                acc_o[1][r] *= alpha[r];
            }
        }
        uint4 pop[2];
#pragma unroll
        for (int js = 0; js < 2; ++js)
            pop[js] = *reinterpret_cast<const uint4 *>(p_lds + col * kPPitch + 2 * (32 * js + 8 * kb));
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            const int d = 32 * w + 16 * x + col;
#pragma unroll
            for (int js = 0; js < 2; ++js) {
                uint32_t wd[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int sl = 32 * js + 4 * e + kb;
                    const uint32_t val =
                        *reinterpret_cast<const uint16_t *>(v_lds + sl * kVPitch + 2 * d);
                    wd[e >> 1] |= val << (16 * (e & 1));
                }
                const uint4 vop = make_uint4(wd[0], wd[1], wd[2], wd[3]);
                acc_o[x] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    attn_as_bf16x8(pop[js]), attn_as_bf16x8(vop), acc_o[x], 0, 0, 0);
            }
        }
        __syncthreads();  // the next chunk overwrites the staging areas
        cur = nxt;
    }

    // acc_o[x][r]: pair 4 kb + r, dim 32 w + 16 x + col, unnormalised against m_run
    const int part_bytes = M * n_heads * parts * kPartStride * 4;  // (the launcher keeps it below 2^31)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (valid[r]) {
            const int rec = ((row_of[r] * n_heads + head_of[r]) * parts + part) * kPartStride;
            float *dst = part_out + rec;
            if constexpr (FIN) {  // device-scope stores: written through to where every XCD reads
                const __amdgpu_buffer_rsrc_t rsrc =
                    __builtin_amdgcn_make_buffer_rsrc(part_out, 0, part_bytes, kBufferWord3);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc_o[0][r]), rsrc,
                                                      (rec + 32 * w + col) * 4, 0, kDeviceScope);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc_o[1][r]), rsrc,
                                                      (rec + 32 * w + 16 + col) * 4, 0, kDeviceScope);
                if (w == 0 && col == 0) {
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(m_run[r]), rsrc, (rec + kHd) * 4, 0,
                                                          kDeviceScope);
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(l_run[r]), rsrc,
                                                          (rec + kHd + 1) * 4, 0, kDeviceScope);
                }
            } else {
                dst[32 * w + col] = acc_o[0][r];
                dst[32 * w + 16 + col] = acc_o[1][r];
                if (w == 0 && col == 0) {
                    dst[kHd] = m_run[r];
                    dst[kHd + 1] = l_run[r];
                }
            }
        }
    }
    if constexpr (FIN) {
        // The partials went out as device-scope stores, and a wave's store counter reaches zero
        // when they have arrived: that wait stands for the release fence, whose write-back of
        // the whole L2 costs each of the launch's waves its turn at it (tens of ns apiece, one
        // after the other).  The arrival itself and the finisher's loads carry the device scope
        // as well, so nothing else needs to be written back or invalidated.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const int live = (live_chunks + cpw - 1) / cpw;  // workgroups of this kv head that got here
        if (threadIdx.x == 0) {
            const unsigned old = __hip_atomic_fetch_add(&fin.arrivals[kvh], 1u, __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT);
            fin_last = old == (unsigned)(live - 1) ? 1u : 0u;
        }
        __syncthreads();
        if (!fin_last) return;
        // thread = (pair of the tile, 8 dims); the pairs of a row are neighbours
        const int pr = threadIdx.x >> 4, j = threadIdx.x & 15;
        const bool mine = pr < pairs_total;
        const int pc = mine ? pr : pairs_total - 1;
        const int row = pc / G, head = kvh * G + (pc - row * G);
        float num[8];
        combine_head_slice<true>(part_out, part_bytes, (row * n_heads + head) * parts * kPartStride, live, j, num);
        uint32_t ob[8];
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float o = bf16_round(num[i]);
            ob[i] = f32_to_bf16_bits(o);
            amax = fmaxf(amax, fabsf(o));
        }
        if (mine)
            reinterpret_cast<uint4 *>(fin.out + ((size_t)row * n_heads + head) * kHd)[j] =
                make_uint4(ob[0] | (ob[1] << 16), ob[2] | (ob[3] << 16), ob[4] | (ob[5] << 16),
                           ob[6] | (ob[7] << 16));
        amax = bonsai_wave::max16(amax);
        if (j == 0) fin_max[pr] = mine ? amax : 0.0f;
        __syncthreads();
        if ((int)threadIdx.x < M) {  // one thread per row: the maximum over the row's heads of this kv head
            float top = 0.0f;
            for (int g = 0; g < G; ++g) top = fmaxf(top, fin_max[threadIdx.x * G + g]);
            uint16_t *arow = fin.amax + (size_t)threadIdx.x * fin.amax_ld;
            arow[kvh] = (uint16_t)f32_to_bf16_bits(top);  // exact: one of the bf16 values stored
            if (kvh == n_kv - 1)
                for (int x = n_kv; x < fin.amax_ld; ++x) arow[x] = 0;
        }
        if (threadIdx.x == 0)
            __hip_atomic_store(&fin.arrivals[kvh], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// One workgroup per token: merge the chunk partials of every head, round to bf16,
// then quantise the whole row (all heads) per token like `quant_input`.
struct CombineArgs {
    const float *part;
    const int32_t *meta;
    uint16_t *out_bf16;
    int8_t *out_q;
    float *out_s;
    int M, n_heads, n_chunks, sigma;
    int parts;  // 0: one partial per 64-slot chunk; > 0: the live chunks in that many even runs
};

constexpr int kCombineThreads = 256;
constexpr int kCombineMaxVec = 2;      // 8-element vectors per thread: up to 32 heads
constexpr int kCombineMaxHeads = kCombineThreads * kCombineMaxVec / (kHd / 8);
constexpr int kCombineMaxChunks = 136;  // sigma + M up to 8704 slots

__global__ void __launch_bounds__(kCombineThreads)
attn_combine_kernel(const float *ppart, const int32_t *pmeta, uint16_t *pout, int8_t *pq, float *ps,
                    int pM, int pheads, int pchunks, int psigma, int pparts) {
    const CombineArgs a{ppart, pmeta, pout, pq, ps, pM, pheads, pchunks, psigma, pparts};
    __shared__ float wgt[kCombineMaxHeads * kCombineMaxChunks];  // becomes the chunk weights
    __shared__ float lsum[kCombineMaxHeads * kCombineMaxChunks];
    __shared__ float max_scratch[kCombineThreads / 64];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int total = min(max(a.meta[0], 0), a.sigma) + a.M;
    int live_chunks = (total + kChunk - 1) / kChunk;
    if (a.parts > 0) {  // partials are runs of chunks: count the runs that hold live chunks
        const int cpw = attn_chunks_per_part(live_chunks, a.parts);
        live_chunks = (live_chunks + cpw - 1) / cpw;
    }
    const int nvec = a.n_heads * (kHd / 8);
    const float *row = a.part + (size_t)m * a.n_heads * a.n_chunks * kPartStride;

    // (max, sum) of every (head, chunk): one load per thread and pass
    const int pairs = a.n_heads * live_chunks;
    for (int idx = tid; idx < pairs; idx += kCombineThreads) {
        const int head = idx / live_chunks, c = idx % live_chunks;
        const float2 ml = *reinterpret_cast<const float2 *>(
            row + ((size_t)head * a.n_chunks + c) * kPartStride + kHd);
        wgt[idx] = ml.x;
        lsum[idx] = ml.y;
    }
    __syncthreads();
    if (tid < a.n_heads) {  // one thread per head turns them into normalised chunk weights
        float *wh = wgt + tid * live_chunks;
        const float *lh = lsum + tid * live_chunks;
        float mx = -INFINITY;
        for (int c = 0; c < live_chunks; ++c) mx = fmaxf(mx, wh[c]);
        float den = 0.0f;
        for (int c = 0; c < live_chunks; ++c) {
            const float e = (wh[c] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(wh[c] - mx);
            wh[c] = e;
            den = fmaf(e, lh[c], den);
        }
        const float inv = den > 0.0f ? 1.0f / den : 0.0f;
        for (int c = 0; c < live_chunks; ++c) wh[c] *= inv;
    }
    __syncthreads();

    float o[kCombineMaxVec][8];
    float amax = 0.0f;
#pragma unroll
    for (int it = 0; it < kCombineMaxVec; ++it) {
        const int v = tid + it * kCombineThreads;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[it][i] = 0.0f;
        if (v >= nvec) continue;
        const int head = v / (kHd / 8);
        const int d0 = (v % (kHd / 8)) * 8;
        const float *base = row + (size_t)head * a.n_chunks * kPartStride + d0;
        const float *wh = wgt + head * live_chunks;
        float num[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) num[i] = 0.0f;
#pragma unroll 4
        for (int c = 0; c < live_chunks; ++c) {
            const float4 x0 = reinterpret_cast<const float4 *>(base + (size_t)c * kPartStride)[0];
            const float4 x1 = reinterpret_cast<const float4 *>(base + (size_t)c * kPartStride)[1];
            const float w = wh[c];
            num[0] = fmaf(w, x0.x, num[0]); num[1] = fmaf(w, x0.y, num[1]);
            num[2] = fmaf(w, x0.z, num[2]); num[3] = fmaf(w, x0.w, num[3]);
            num[4] = fmaf(w, x1.x, num[4]); num[5] = fmaf(w, x1.y, num[5]);
            num[6] = fmaf(w, x1.z, num[6]); num[7] = fmaf(w, x1.w, num[7]);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            o[it][i] = bf16_round(num[i]);
            amax = fmaxf(amax, fabsf(o[it][i]));
        }
        if (a.out_bf16 != nullptr) {
            uint4 w;
            w.x = f32_to_bf16_bits(o[it][0]) | (f32_to_bf16_bits(o[it][1]) << 16);
            w.y = f32_to_bf16_bits(o[it][2]) | (f32_to_bf16_bits(o[it][3]) << 16);
            w.z = f32_to_bf16_bits(o[it][4]) | (f32_to_bf16_bits(o[it][5]) << 16);
            w.w = f32_to_bf16_bits(o[it][6]) | (f32_to_bf16_bits(o[it][7]) << 16);
            reinterpret_cast<uint4 *>(a.out_bf16 + (size_t)m * nvec * 8)[v] = w;
        }
    }
    if (a.out_q == nullptr) return;  // uniform over the grid
    amax = wave_max(amax);
    if ((tid & 63) == 0) max_scratch[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(max_scratch[0], max_scratch[1]), fmaxf(max_scratch[2], max_scratch[3]));
    const float sval = (1.0f / fmaxf(amax, 1e-5f)) * 127.0f;
    if (tid == 0) a.out_s[m] = sval;
#pragma unroll
    for (int it = 0; it < kCombineMaxVec; ++it) {
        const int v = tid + it * kCombineThreads;
        if (v >= nvec) continue;
        uint32_t b[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float r = __builtin_rintf(o[it][i] * sval);
            r = fminf(fmaxf(r, -128.0f), 127.0f);
            b[i] = (uint32_t)((int)r) & 0xffu;
        }
        uint2 w;
        w.x = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
        w.y = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
        reinterpret_cast<uint2 *>(a.out_q + (size_t)m * nvec * 8)[v] = w;
    }
}

// The same merge for the matrix-core chunk pass, whose partial count per (row, head) is at
// most kMaxParts = 16: one workgroup of 512 threads per token, thread = (head, 8 dims).  The
// 16 lanes of a head are one DPP row: lane j turns part j's (max, sum) into its normalised
// weight with two row reductions, the weights travel by row_share, and every thread has
// already requested its slice of all live partials, so the kernel is one memory round trip
// long.  Accumulation runs over the parts in ascending order.
constexpr int kCombinePartsThreads = 512;

__global__ void __launch_bounds__(kCombinePartsThreads)
attn_combine_parts_kernel(const float *part, const int32_t *meta, uint16_t *out_bf16, int8_t *out_q,
                          float *out_s, int M, int n_heads, int parts, int sigma) {
    __shared__ float max_scratch[kCombinePartsThreads / 64];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int total = min(max(meta[0], 0), sigma) + M;
    const int live_chunks = (total + kChunk - 1) / kChunk;
    const int cpw = attn_chunks_per_part(live_chunks, parts);
    const int live = (live_chunks + cpw - 1) / cpw;  // <= parts <= kMaxParts
    const int nvec = n_heads * (kHd / 8);
    const bool mine = tid < nvec;
    const int v = mine ? tid : nvec - 1;
    const int head = v >> 4, j = v & 15;
    float num[8];
    combine_head_slice<false>(part, 0, (m * n_heads + head) * parts * kPartStride, live, j, num);

    float o[8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        o[i] = bf16_round(num[i]);
        if (mine) amax = fmaxf(amax, fabsf(o[i]));
    }
    if (mine && out_bf16 != nullptr) {
        uint4 wv;
        wv.x = f32_to_bf16_bits(o[0]) | (f32_to_bf16_bits(o[1]) << 16);
        wv.y = f32_to_bf16_bits(o[2]) | (f32_to_bf16_bits(o[3]) << 16);
        wv.z = f32_to_bf16_bits(o[4]) | (f32_to_bf16_bits(o[5]) << 16);
        wv.w = f32_to_bf16_bits(o[6]) | (f32_to_bf16_bits(o[7]) << 16);
        reinterpret_cast<uint4 *>(out_bf16 + (size_t)m * nvec * 8)[v] = wv;
    }
    if (out_q == nullptr) return;  // uniform over the grid
    amax = wave_max(amax);
    if ((tid & 63) == 0) max_scratch[tid >> 6] = amax;
    __syncthreads();
    amax = max_scratch[0];
#pragma unroll
    for (int wv = 1; wv < kCombinePartsThreads / 64; ++wv) amax = fmaxf(amax, max_scratch[wv]);
    const float sval = (1.0f / fmaxf(amax, 1e-5f)) * 127.0f;
    if (tid == 0) out_s[m] = sval;
    if (mine) {
        uint32_t b[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float r = __builtin_rintf(o[i] * sval);
            r = fminf(fmaxf(r, -128.0f), 127.0f);
            b[i] = (uint32_t)((int)r) & 0xffu;
        }
        uint2 wq;
        wq.x = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
        wq.y = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
        reinterpret_cast<uint2 *>(out_q + (size_t)m * nvec * 8)[v] = wq;
    }
}

// ---------------------------------------------------------------------------
// KV commit: rows [src, src+n) -> [dst, dst+n) for every (k|v, layer, kv head).
// One thread per 16 bytes.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) kv_commit_kernel(uint4 *kv, int planes, int slots, int src,
                                                        int dst, int n) {
    const int per_plane = n * (kHd * 2 / 16);
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= planes * per_plane) return;
    const int plane = idx / per_plane;
    const int off = idx % per_plane;
    uint4 *base = kv + (size_t)plane * slots * (kHd * 2 / 16);
    base[(size_t)dst * (kHd * 2 / 16) + off] = base[(size_t)src * (kHd * 2 / 16) + off];
}

// ---------------------------------------------------------------------------
// Draft chain.  One workgroup of 1024 threads per logits row: running (max, index)
// and the sum of exp(x - max) in one pass with 16-byte loads; conf = 1 / sum.
// ---------------------------------------------------------------------------
constexpr int kDraftThreads = 1024;

struct RowStat {
    float mx;
    int idx;
    float sum;
};

__device__ __forceinline__ RowStat merge(RowStat a, RowStat b) {
    // larger max wins; equal maxima keep the lower index
    const bool take_b = (b.mx > a.mx) || (b.mx == a.mx && b.idx < a.idx);
    const float mx = fmaxf(a.mx, b.mx);
    RowStat r;
    r.mx = mx;
    r.idx = take_b ? b.idx : a.idx;
    const float sa = (a.mx == -INFINITY) ? 0.0f : a.sum * __builtin_amdgcn_exp2f((a.mx - mx) * 1.44269504f);
    const float sb = (b.mx == -INFINITY) ? 0.0f : b.sum * __builtin_amdgcn_exp2f((b.mx - mx) * 1.44269504f);
    r.sum = sa + sb;
    return r;
}

__global__ void __launch_bounds__(kDraftThreads)
draft_rows_kernel(const uint16_t *logits, int ld, int vocab, int32_t *tokens, float *conf) {
    __shared__ RowStat wave_stat[kDraftThreads / 64];
    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const uint16_t *x = logits + (size_t)row * ld;
    RowStat st;
    st.mx = -INFINITY;
    st.idx = 0x7fffffff;
    st.sum = 0.0f;
    const int nvec = vocab / 8;
    for (int v = tid; v < nvec; v += kDraftThreads) {
        const uint4 raw = reinterpret_cast<const uint4 *>(x)[v];
        const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
        float e[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            e[2 * i] = bf16_bits_to_f32(d[i] & 0xffffu);
            e[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
        }
        float vm = e[0];
        int vi = 0;
#pragma unroll
        for (int i = 1; i < 8; ++i) {
            if (e[i] > vm) {
                vm = e[i];
                vi = i;
            }
        }
        if (!(vm == vm)) continue;  // a NaN vector contributes nothing
        const float nm = fmaxf(st.mx, vm);
        float s = (st.mx == -INFINITY) ? 0.0f : st.sum * __builtin_amdgcn_exp2f((st.mx - nm) * 1.44269504f);
#pragma unroll
        for (int i = 0; i < 8; ++i) s += __builtin_amdgcn_exp2f((e[i] - nm) * 1.44269504f);
        if (vm > st.mx) st.idx = v * 8 + vi;
        st.mx = nm;
        st.sum = s;
    }
    for (int c = nvec * 8 + tid; c < vocab; c += kDraftThreads) {  // ragged tail
        RowStat one;
        one.mx = bf16_bits_to_f32(x[c]);
        one.idx = c;
        one.sum = 1.0f;
        if (one.mx == one.mx) st = merge(st, one);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        RowStat o;
        o.mx = __shfl_xor(st.mx, off);
        o.idx = __shfl_xor(st.idx, off);
        o.sum = __shfl_xor(st.sum, off);
        st = merge(st, o);
    }
    if ((tid & 63) == 0) wave_stat[tid >> 6] = st;
    __syncthreads();
    if (tid == 0) {
        RowStat t = wave_stat[0];
        for (int w = 1; w < kDraftThreads / 64; ++w) t = merge(t, wave_stat[w]);
        tokens[row] = t.idx == 0x7fffffff ? 0 : t.idx;
        conf[row] = t.sum > 0.0f ? 1.0f / t.sum : 0.0f;
    }
}

__global__ void draft_accept_kernel(const float *conf, int rows, float threshold, int32_t *accept) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    int n = 1;
    for (int r = 1; r < rows; ++r) {
        if (!(conf[r] > threshold)) break;
        ++n;
    }
    accept[0] = n;
    accept[1] = rows;
}

// The same statistics with a row split over `splits` workgroups (one workgroup per row is a
// single CU evaluating 150k exponentials): partial (max, index, sum) per split into a
// scratch buffer, then one small workgroup merges them per row and walks the chain.
constexpr int kDraftSplitThreads = 256;
constexpr int kDraftSplits = 32;

__device__ __forceinline__ RowStat wave_merge(RowStat st) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        RowStat o;
        o.mx = __shfl_xor(st.mx, off);
        o.idx = __shfl_xor(st.idx, off);
        o.sum = __shfl_xor(st.sum, off);
        st = merge(st, o);
    }
    return st;
}

__global__ void __launch_bounds__(kDraftSplitThreads)
draft_rows_split_kernel(const uint16_t *logits, int ld, int vocab, int splits, float *scratch) {
    __shared__ RowStat wave_stat[kDraftSplitThreads / 64];
    const int row = blockIdx.x / splits, sp = blockIdx.x % splits;
    const int tid = threadIdx.x;
    const uint16_t *x = logits + (size_t)row * ld;
    RowStat st;
    st.mx = -INFINITY;
    st.idx = 0x7fffffff;
    st.sum = 0.0f;
    const int nvec = vocab / 8;
    const int per = (nvec + splits - 1) / splits;
    const int v_end = min(nvec, (sp + 1) * per);
    for (int v = sp * per + tid; v < v_end; v += kDraftSplitThreads) {
        const uint4 raw = reinterpret_cast<const uint4 *>(x)[v];
        const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
        float e[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            e[2 * i] = bf16_bits_to_f32(d[i] & 0xffffu);
            e[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
        }
        float vm = e[0];
        int vi = 0;
#pragma unroll
        for (int i = 1; i < 8; ++i) {
            if (e[i] > vm) {
                vm = e[i];
                vi = i;
            }
        }
        if (!(vm == vm)) continue;  // a NaN vector contributes nothing
        const float nm = fmaxf(st.mx, vm);
        float s = (st.mx == -INFINITY) ? 0.0f : st.sum * __builtin_amdgcn_exp2f((st.mx - nm) * 1.44269504f);
#pragma unroll
        for (int i = 0; i < 8; ++i) s += __builtin_amdgcn_exp2f((e[i] - nm) * 1.44269504f);
        if (vm > st.mx) st.idx = v * 8 + vi;
        st.mx = nm;
        st.sum = s;
    }
    if (sp == splits - 1) {
        for (int c = nvec * 8 + tid; c < vocab; c += kDraftSplitThreads) {  // ragged tail
            RowStat one;
            one.mx = bf16_bits_to_f32(x[c]);
            one.idx = c;
            one.sum = 1.0f;
            if (one.mx == one.mx) st = merge(st, one);
        }
    }
    st = wave_merge(st);
    if ((tid & 63) == 0) wave_stat[tid >> 6] = st;
    __syncthreads();
    if (tid == 0) {
        RowStat t = wave_stat[0];
        for (int w = 1; w < kDraftSplitThreads / 64; ++w) t = merge(t, wave_stat[w]);
        float *dst = scratch + (size_t)blockIdx.x * 4;
        dst[0] = t.mx;
        dst[1] = __int_as_float(t.idx);
        dst[2] = t.sum;
    }
}

__global__ void __launch_bounds__(1024)
draft_merge_accept_kernel(const float *scratch, int rows, int splits, float threshold,
                          int32_t *tokens, float *conf, int32_t *accept) {
    __shared__ float conf_lds[BONSAI_MAX_WIDTH];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int row = w; row < rows; row += 16) {  // rows <= 32: every wave runs the same two rounds at most
        RowStat st;
        st.mx = -INFINITY;
        st.idx = 0x7fffffff;
        st.sum = 0.0f;
        if (lane < splits) {
            const float *src = scratch + ((size_t)row * splits + lane) * 4;
            st.mx = src[0];
            st.idx = __float_as_int(src[1]);
            st.sum = src[2];
        }
        st = wave_merge(st);
        if (lane == 0) {
            const float c = st.sum > 0.0f ? 1.0f / st.sum : 0.0f;
            tokens[row] = st.idx == 0x7fffffff ? 0 : st.idx;
            conf[row] = c;
            conf_lds[row] = c;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int n = 1;
        for (int r = 1; r < rows; ++r) {
            if (!(conf_lds[r] > threshold)) break;
            ++n;
        }
        accept[0] = n;
        accept[1] = rows;
    }
}

// ---------------------------------------------------------------------------
// bf16 output projection: out[m][n] = sum_k x[m][k] * w[n][k], the lm_head of a sign-weight
// backbone (`_lm_head`, precision "bf16": F.linear(h, W), src/bonsai_sft/gpu/model.py:1296).
// HBM-bound on w (2 N K bytes, read once).  The M <= 16 token rows sit in LDS; the waves of
// a workgroup split K, each streams its slice of 16 weight rows straight into the B operand
// of v_mfma_f32_16x16x32_bf16 (lane = (row, k-block): 32 contiguous bytes per pair of
// MFMAs, so the four lanes of a row cover one 128-byte line) and the workgroup adds the
// slices' partial tiles in wave order.  Workgroups stride over the 16-row tiles.
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
constexpr int kLinMaxWaves = 8;
constexpr int kLinTokens = 16;
constexpr int kLinUnroll = 4;  // pairs of 16-byte loads in flight per lane

__device__ __forceinline__ bf16x8_t as_bf16x8(const uint4 v) {
    bf16x8_t r;
    __builtin_memcpy(&r, &v, 16);
    return r;
}

__host__ __device__ inline size_t lin_lds_bytes(int M, int K, int nwaves) {
    return (size_t)M * (2 * K + 16) + (size_t)2 * nwaves * 256 * sizeof(float);
}

__global__ void __launch_bounds__(kLinMaxWaves * 64)
bf16_linear_kernel(const uint16_t *x, const uint16_t *w, uint16_t *out, int M, int N, int K,
                   int nwaves, int ntiles, int grid) {
    extern __shared__ __align__(16) unsigned char lin_smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pitch = 2 * K + 16;  // +16 bytes: consecutive tokens start four banks apart
    float *part = reinterpret_cast<float *>(lin_smem + (size_t)M * pitch);  // [2][nwaves][4][64]

    const int vec_per_row = K / 8;
    for (int v = tid; v < M * vec_per_row; v += nwaves * 64) {
        const int m = v / vec_per_row, c = v - m * vec_per_row;
        *reinterpret_cast<uint4 *>(lin_smem + (size_t)m * pitch + (size_t)c * 16) =
            reinterpret_cast<const uint4 *>(x + (size_t)m * K)[c];
    }
    __syncthreads();

    const int row_l = lane & 15, kb = lane >> 4;
    const int ksl = K / nwaves;    // elements of K per wave, a multiple of 64
    const int npairs = ksl / 64;
    const int k_base = wave * ksl + 16 * kb;
    // operand rows past M alias the last token; their products are never stored
    const int tok = row_l < M ? row_l : M - 1;
    const unsigned char *xl = lin_smem + (size_t)tok * pitch + (size_t)k_base * 2;
    int buf = 0;
    for (int tile = blockIdx.x; tile < ntiles; tile += grid) {
        int row = tile * 16 + row_l;
        row = row < N ? row : N - 1;
        const uint4 *wl = reinterpret_cast<const uint4 *>(w + (size_t)row * K + k_base);
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int p0 = 0; p0 < npairs; p0 += kLinUnroll) {
            uint4 wr[kLinUnroll][2];
#pragma unroll
            for (int u = 0; u < kLinUnroll; ++u)
                if (p0 + u < npairs) {
                    wr[u][0] = wl[(p0 + u) * 8];
                    wr[u][1] = wl[(p0 + u) * 8 + 1];
                }
#pragma unroll
            for (int u = 0; u < kLinUnroll; ++u)
                if (p0 + u < npairs) {
                    const uint4 x0 = *reinterpret_cast<const uint4 *>(xl + (size_t)(p0 + u) * 128);
                    const uint4 x1 = *reinterpret_cast<const uint4 *>(xl + (size_t)(p0 + u) * 128 + 16);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(x0), as_bf16x8(wr[u][0]),
                                                                  acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(x1), as_bf16x8(wr[u][1]),
                                                                  acc, 0, 0, 0);
                }
        }
        // acc[r]: token 4*kb + r, weight row row_l of this tile, over this wave's slice of K
        float *mine = part + ((size_t)buf * nwaves + wave) * 256;
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[r * 64 + lane] = acc[r];
        __syncthreads();
        if (wave == 0) {
            float t[4];
            const float *p = part + (size_t)buf * nwaves * 256;
#pragma unroll
            for (int r = 0; r < 4; ++r) t[r] = p[r * 64 + lane];
            for (int w2 = 1; w2 < nwaves; ++w2)
#pragma unroll
                for (int r = 0; r < 4; ++r) t[r] += p[w2 * 256 + r * 64 + lane];
            const int orow = tile * 16 + row_l;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * kb + r;
                if (m < M && orow < N) out[(size_t)m * N + orow] = (uint16_t)f32_to_bf16_bits(t[r]);
            }
        }
        // the other half of `part` takes the next tile: wave 0 reaches that tile's barrier
        // only after it has read this half
        buf ^= 1;
    }
}

constexpr int kMaxDevices = 16;
std::atomic<bool> g_lin_ready[kMaxDevices];  // set last, under g_lin_mutex
std::mutex g_lin_mutex;
int g_lin_cus[kMaxDevices];
int g_lin_lds[kMaxDevices];

// ---------------------------------------------------------------------------
// FP8 (E4M3, OCP "fn") draft projection of the reference (`prepare_fp8_lm_head` and
// `_lm_head` with precision "fp8", src/bonsai_sft/gpu/model.py:1168-1194,1268-1275): the
// rows are quantised with ONE scale for all of them, amax / 448 evaluated in bf16 like the
// reference's tensor expression, and multiplied with a per-tensor-scaled E4M3 weight matrix.
// ---------------------------------------------------------------------------
constexpr int kFp8Threads = 1024;

// fp32 -> E4M3 (bias 7, no infinities, 0x7f = NaN), round to nearest even, subnormals kept;
// magnitudes that round above 448 give NaN like torch's cast (they cannot occur after the
// division by the row scale)
__device__ __forceinline__ uint32_t f32_to_e4m3fn(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t au = u & 0x7fffffffu;
    if (au > 0x7f800000u) return sign | 0x7fu;  // NaN
    const float af = __uint_as_float(au);
    if (af > 464.0f) return sign | 0x7fu;        // beyond the rounding range of 448 (464 ties to 448)
    if (af < 0.015625f) {                        // below 2^-6: multiples of 2^-9
        const float q = rintf(af * 512.0f);      // round half to even
        return sign | (uint32_t)q;               // q == 8 is the smallest normal, same code
    }
    // normal: keep 3 mantissa bits, RNE on the 20 dropped ones
    uint32_t r = au + 0x7ffffu + ((au >> 20) & 1u);
    const uint32_t exp = (r >> 23) - 127u + 7u;
    const uint32_t man = (r >> 20) & 7u;
    return sign | (exp << 3) | man;
}

// x bf16 [M, K] -> q E4M3 [M, K], scale[0] = fp32(bf16(max(bf16(amax / 448), 1e-12)));
// q = e4m3(bf16(fp32(x) / scale)).  One workgroup: M * K is a few rows of the hidden size.
__global__ void __launch_bounds__(kFp8Threads)
fp8_quant_rows_kernel(const uint16_t *x, uint8_t *q, float *scale, int total) {
    __shared__ float wave_max[kFp8Threads / 64];
    const int tid = threadIdx.x;
    const int nvec = total / 8;
    float amax = 0.0f;
    for (int v = tid; v < nvec; v += kFp8Threads) {
        const uint4 raw = reinterpret_cast<const uint4 *>(x)[v];
        const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            amax = fmaxf(amax, fabsf(bf16_bits_to_f32(d[i] & 0xffffu)));
            amax = fmaxf(amax, fabsf(__uint_as_float(d[i] & 0xffff0000u)));
        }
    }
    amax = bonsai_wave::max64(amax);
    if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
    __syncthreads();
    float t = wave_max[0];
    for (int w = 1; w < kFp8Threads / 64; ++w) t = fmaxf(t, wave_max[w]);
    // bf16 arithmetic of the reference expression: (amax / 448).clamp_min(1e-12).float()
    float sc = bf16_round(t / 448.0f);
    sc = fmaxf(sc, bf16_round(1e-12f));
    if (tid == 0) scale[0] = sc;
    for (int v = tid; v < nvec; v += kFp8Threads) {
        const uint4 raw = reinterpret_cast<const uint4 *>(x)[v];
        const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
        uint32_t o[2] = {0u, 0u};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = bf16_round(bf16_bits_to_f32(d[i] & 0xffffu) / sc);
            const float hi = bf16_round(__uint_as_float(d[i] & 0xffff0000u) / sc);
            o[i >> 1] |= (f32_to_e4m3fn(lo) | (f32_to_e4m3fn(hi) << 8)) << (16 * (i & 1));
        }
        reinterpret_cast<uint2 *>(q)[v] = make_uint2(o[0], o[1]);
    }
}

__host__ __device__ inline size_t fp8_lin_lds_bytes(int M, int K, int nwaves) {
    return (size_t)M * (K + 16) + (size_t)2 * nwaves * 256 * sizeof(float);
}

// out[m][n] = bf16( (sum_k x[m][k] * w[n][k]) * x_scale * w_scale ), E4M3 operands, fp32
// accumulation.  Same structure as bf16_linear_kernel: tokens in LDS, the waves split K,
// a lane streams 32 contiguous bytes (four K-blocks of 8) of its weight row per group of
// four v_mfma_f32_16x16x32_fp8_fp8.
__global__ void __launch_bounds__(kLinMaxWaves * 64)
fp8_linear_kernel(const uint8_t *x, const float *x_scale, const uint8_t *w, float w_scale,
                  uint16_t *out, int M, int N, int K, int nwaves, int ntiles, int grid) {
    extern __shared__ __align__(16) unsigned char lin_smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pitch = K + 16;
    float *part = reinterpret_cast<float *>(lin_smem + (size_t)M * pitch);

    const int vec_per_row = K / 16;
    for (int v = tid; v < M * vec_per_row; v += nwaves * 64) {
        const int m = v / vec_per_row, c = v - m * vec_per_row;
        *reinterpret_cast<uint4 *>(lin_smem + (size_t)m * pitch + (size_t)c * 16) =
            reinterpret_cast<const uint4 *>(x + (size_t)m * K)[c];
    }
    __syncthreads();
    const float scale = x_scale[0] * w_scale;

    const int row_l = lane & 15, kb = lane >> 4;
    const int ksl = K / nwaves;     // a multiple of 128
    const int nblk = ksl / 128;
    const int k_base = wave * ksl + 32 * kb;
    const int tok = row_l < M ? row_l : M - 1;
    const unsigned char *xl = lin_smem + (size_t)tok * pitch + k_base;
    int buf = 0;
    for (int tile = blockIdx.x; tile < ntiles; tile += grid) {
        int row = tile * 16 + row_l;
        row = row < N ? row : N - 1;
        const uint4 *wl = reinterpret_cast<const uint4 *>(w + (size_t)row * K + k_base);
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int p0 = 0; p0 < nblk; p0 += kLinUnroll) {
            uint4 wr[kLinUnroll][2];
#pragma unroll
            for (int u = 0; u < kLinUnroll; ++u)
                if (p0 + u < nblk) {
                    wr[u][0] = wl[(p0 + u) * 8];
                    wr[u][1] = wl[(p0 + u) * 8 + 1];
                }
#pragma unroll
            for (int u = 0; u < kLinUnroll; ++u)
                if (p0 + u < nblk) {
                    const uint4 x0 = *reinterpret_cast<const uint4 *>(xl + (size_t)(p0 + u) * 128);
                    const uint4 x1 = *reinterpret_cast<const uint4 *>(xl + (size_t)(p0 + u) * 128 + 16);
                    const uint32_t xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                    const uint32_t ws[8] = {wr[u][0].x, wr[u][0].y, wr[u][0].z, wr[u][0].w,
                                            wr[u][1].x, wr[u][1].y, wr[u][1].z, wr[u][1].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const long xa = (long)(((uint64_t)xs[2 * j + 1] << 32) | xs[2 * j]);
                        const long wb = (long)(((uint64_t)ws[2 * j + 1] << 32) | ws[2 * j]);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(xa, wb, acc, 0, 0, 0);
                    }
                }
        }
        float *mine = part + ((size_t)buf * nwaves + wave) * 256;
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[r * 64 + lane] = acc[r];
        __syncthreads();
        if (wave == 0) {
            float t[4];
            const float *p = part + (size_t)buf * nwaves * 256;
#pragma unroll
            for (int r = 0; r < 4; ++r) t[r] = p[r * 64 + lane];
            for (int w2 = 1; w2 < nwaves; ++w2)
#pragma unroll
                for (int r = 0; r < 4; ++r) t[r] += p[w2 * 256 + r * 64 + lane];
            const int orow = tile * 16 + row_l;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * kb + r;
                if (m < M && orow < N)
                    out[(size_t)m * N + orow] = (uint16_t)f32_to_bf16_bits(t[r] * scale);
            }
        }
        buf ^= 1;
    }
}

std::atomic<bool> g_fp8_ready[kMaxDevices];  // set last, under g_lin_mutex

int g_rows_per_wave = 0;  // 0 = heuristic; set through bonsai_decode_set_tuning
int g_attn_engine = 0;    // 0 = matrix-core chunk pass, 1 = VALU chunk pass

int rows_per_wave(int M) {
    if (g_rows_per_wave >= 1 && g_rows_per_wave <= 4) return g_rows_per_wave < M ? g_rows_per_wave : (M < 4 ? M : 4);
    // few rows per wave keep the waves short; more row groups re-read K/V from L2 (measured:
    // two rows per wave up to a dozen rows, four above)
    if (M <= 2) return M;
    if (M <= 12) return 2;
    return 4;
}

}  // namespace

extern "C" int bonsai_qk_norm_rope_kv_write(const void *xqkv, const void *q_norm_w,
                                            const void *k_norm_w, float eps, const void *cos_table,
                                            const void *sin_table, const int32_t *positions,
                                            void *q_out, void *k_layer, void *v_layer, int M,
                                            int n_heads, int n_kv, int slots, int write_slot,
                                            int max_pos, void *stream) {
    if (!xqkv || !q_norm_w || !k_norm_w || !cos_table || !sin_table || !positions || !q_out ||
        !k_layer || !v_layer)
        return BONSAI_DECODE_ERR_ARG;
    if (M < 1 || M > BONSAI_MAX_WIDTH || n_heads < 1 || n_kv < 1 || max_pos < 1 || write_slot < 0 ||
        write_slot + M > slots)
        return BONSAI_DECODE_ERR_ARG;
    RopeArgs a;
    a.xqkv = static_cast<const uint16_t *>(xqkv);
    a.qw = static_cast<const uint16_t *>(q_norm_w);
    a.kw = static_cast<const uint16_t *>(k_norm_w);
    a.cos_t = static_cast<const uint16_t *>(cos_table);
    a.sin_t = static_cast<const uint16_t *>(sin_table);
    a.positions = positions;
    a.q_out = static_cast<uint16_t *>(q_out);
    a.k_layer = static_cast<uint16_t *>(k_layer);
    a.v_layer = static_cast<uint16_t *>(v_layer);
    a.eps = eps;
    a.M = M;
    a.n_heads = n_heads;
    a.n_kv = n_kv;
    a.slots = slots;
    a.write_slot = write_slot;
    a.max_pos = max_pos;
    const int total_heads = n_heads + 2 * n_kv;
    hipLaunchKernelGGL(qk_norm_rope_kernel, dim3((total_heads + 3) / 4, M), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a.xqkv, a.qw, a.kw, a.cos_t, a.sin_t,
                       a.positions, a.q_out, a.k_layer, a.v_layer, a.eps, a.M, a.n_heads, a.n_kv,
                       a.slots, a.write_slot, a.max_pos);
    return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
}

extern "C" void bonsai_decode_set_attention_engine(int engine) {
    g_attn_engine = engine == 1 ? 1 : 0;
}

extern "C" void bonsai_decode_set_tuning(int rows_per_wave_override) {
    g_rows_per_wave = rows_per_wave_override;
}

extern "C" int64_t bonsai_decode_attention_scratch_bytes(int M, int n_heads, int slots) {
    if (M < 1 || n_heads < 1 || slots < 1) return 0;
    const int64_t n_chunks = (slots + kChunk - 1) / kChunk;
    return (int64_t)M * n_heads * n_chunks * kPartStride * (int64_t)sizeof(float);
}

// Shared body of the two attention entry points.  `rope` non-null: `q` is the merged q|k|v
// projection and the chunk pass does the work of bonsai_qk_norm_rope_kv_write as well.
static int launch_attention(const void *q, void *k_layer, void *v_layer, const int32_t *meta,
                            void *scratch, void *out_bf16, int8_t *out_q, float *out_s, float scale,
                            int M, int n_heads, int n_kv, int slots, int sigma, const RopeIn *rope,
                            const FinOut *fin, hipStream_t st) {
    if (!q || !k_layer || !v_layer || !meta || !scratch) return BONSAI_DECODE_ERR_ARG;
    if ((out_q == nullptr) != (out_s == nullptr)) return BONSAI_DECODE_ERR_ARG;
    if (!fin && !out_bf16 && !out_q) return BONSAI_DECODE_ERR_ARG;
    if (M < 1 || M > BONSAI_MAX_WIDTH || n_kv < 1 || n_heads < n_kv || n_heads % n_kv != 0 ||
        n_heads > kCombineMaxHeads || sigma < 0 || sigma + M > slots ||
        (sigma + M + kChunk - 1) / kChunk > kCombineMaxChunks)
        return BONSAI_DECODE_ERR_ARG;
    AttnArgs a;
    a.q = static_cast<const uint32_t *>(q);
    a.k_layer = static_cast<const uint32_t *>(k_layer);
    a.v_layer = static_cast<const uint32_t *>(v_layer);
    a.meta = meta;
    a.part = static_cast<float *>(scratch);
    a.scale_log2e = scale * 1.44269504088896340736f;
    a.M = M;
    a.n_heads = n_heads;
    a.n_kv = n_kv;
    a.hpg = n_heads / n_kv;
    a.slots = slots;
    a.sigma = sigma;
    // the live length is cache_len + M <= sigma + M: chunks beyond it are never launched
    a.n_chunks = (sigma + M + kChunk - 1) / kChunk;
    int parts = 0;  // partials per (row, head): chunks for the VALU pass, runs of chunks otherwise
    if (g_attn_engine == 0 || rope != nullptr) {
        parts = a.n_chunks < kMaxParts ? a.n_chunks : kMaxParts;
        const int tiles = (M * a.hpg + kPairTile - 1) / kPairTile;
        const dim3 grid(n_kv * parts * tiles), block(kAttnWaves * 64);
        if (fin != nullptr) {  // the one launch that also merges its partials (rope != nullptr, one tile)
            hipLaunchKernelGGL((attn_mfma_kernel<true, true>), grid, block, 0, st,
                               static_cast<const uint16_t *>(q), static_cast<uint16_t *>(k_layer),
                               static_cast<uint16_t *>(v_layer), meta, a.part, a.scale_log2e, M,
                               n_heads, n_kv, a.hpg, slots, sigma, parts, *rope, *fin);
            return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
        }
        if (rope != nullptr)
            hipLaunchKernelGGL((attn_mfma_kernel<true, false>), grid, block, 0, st,
                               static_cast<const uint16_t *>(q), static_cast<uint16_t *>(k_layer),
                               static_cast<uint16_t *>(v_layer), meta, a.part, a.scale_log2e, M,
                               n_heads, n_kv, a.hpg, slots, sigma, parts, *rope, FinOut{});
        else
            hipLaunchKernelGGL((attn_mfma_kernel<false, false>), grid, block, 0, st,
                               static_cast<const uint16_t *>(q), static_cast<uint16_t *>(k_layer),
                               static_cast<uint16_t *>(v_layer), meta, a.part, a.scale_log2e, M,
                               n_heads, n_kv, a.hpg, slots, sigma, parts, RopeIn{}, FinOut{});
    } else {
    const int rw = rows_per_wave(M);
    a.row_groups = (M + rw - 1) / rw;
    const AttnArgs &launch = a;
    const int blocks = n_kv * a.n_chunks * a.hpg * a.row_groups;
#define ATTN_ARGS                                                                             \
    launch.q, launch.k_layer, launch.v_layer, launch.meta, launch.part, launch.scale_log2e,      \
        launch.M, launch.n_heads, launch.n_kv, launch.hpg, launch.slots, launch.sigma,           \
        launch.n_chunks, launch.row_groups
    switch (rw) {
        case 1: hipLaunchKernelGGL(attn_partial_kernel<1>, dim3(blocks), dim3(64), 0, st, ATTN_ARGS); break;
        case 2: hipLaunchKernelGGL(attn_partial_kernel<2>, dim3(blocks), dim3(64), 0, st, ATTN_ARGS); break;
        case 3: hipLaunchKernelGGL(attn_partial_kernel<3>, dim3(blocks), dim3(64), 0, st, ATTN_ARGS); break;
        default: hipLaunchKernelGGL(attn_partial_kernel<4>, dim3(blocks), dim3(64), 0, st, ATTN_ARGS); break;
    }
#undef ATTN_ARGS
    }
    if (hipGetLastError() != hipSuccess) return BONSAI_DECODE_ERR_LAUNCH;
    CombineArgs c;
    c.part = a.part;
    c.meta = meta;
    c.out_bf16 = static_cast<uint16_t *>(out_bf16);
    c.out_q = out_q;
    c.out_s = out_s;
    c.M = M;
    c.n_heads = n_heads;
    c.n_chunks = parts > 0 ? parts : a.n_chunks;  // partial slots per (row, head)
    c.sigma = sigma;
    c.parts = parts;
    if (parts > 0)
        hipLaunchKernelGGL(attn_combine_parts_kernel, dim3(M), dim3(kCombinePartsThreads), 0, st,
                           c.part, c.meta, c.out_bf16, c.out_q, c.out_s, c.M, c.n_heads, parts,
                           c.sigma);
    else
        hipLaunchKernelGGL(attn_combine_kernel, dim3(M), dim3(kCombineThreads), 0, st, c.part,
                           c.meta, c.out_bf16, c.out_q, c.out_s, c.M, c.n_heads, c.n_chunks,
                           c.sigma, c.parts);
    return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
}

extern "C" int bonsai_decode_attention(const void *q, const void *k_layer, const void *v_layer,
                                       const int32_t *meta, void *scratch, void *out_bf16,
                                       int8_t *out_q, float *out_s, float scale, int M, int n_heads,
                                       int n_kv, int slots, int sigma, void *stream) {
    return launch_attention(q, const_cast<void *>(k_layer), const_cast<void *>(v_layer), meta, scratch,
                            out_bf16, out_q, out_s, scale, M, n_heads, n_kv, slots, sigma, nullptr, nullptr,
                            static_cast<hipStream_t>(stream));
}

extern "C" int bonsai_decode_attention_rope(const void *xqkv, const void *q_norm_w, const void *k_norm_w,
                                            float eps, const void *cos_table, const void *sin_table,
                                            const int32_t *positions, int max_pos, void *k_layer,
                                            void *v_layer, const int32_t *meta, void *scratch,
                                            void *out_bf16, int8_t *out_q, float *out_s, float scale,
                                            int M, int n_heads, int n_kv, int slots, int sigma,
                                            void *stream) {
    if (!q_norm_w || !k_norm_w || !cos_table || !sin_table || !positions || max_pos < 1)
        return BONSAI_DECODE_ERR_ARG;
    const RopeIn rope{static_cast<const uint16_t *>(q_norm_w), static_cast<const uint16_t *>(k_norm_w),
                      static_cast<const uint16_t *>(cos_table), static_cast<const uint16_t *>(sin_table),
                      positions, eps, max_pos};
    return launch_attention(xqkv, k_layer, v_layer, meta, scratch, out_bf16, out_q, out_s, scale, M,
                            n_heads, n_kv, slots, sigma, &rope, nullptr, static_cast<hipStream_t>(stream));
}

extern "C" int bonsai_decode_attention_rope_parts(const void *xqkv, const void *q_norm_w,
                                                  const void *k_norm_w, float eps, const void *cos_table,
                                                  const void *sin_table, const int32_t *positions,
                                                  int max_pos, void *k_layer, void *v_layer,
                                                  const int32_t *meta, void *scratch, void *arrivals,
                                                  void *out_bf16, void *out_amax, float scale, int M,
                                                  int n_heads, int n_kv, int slots, int sigma,
                                                  void *stream) {
    if (!q_norm_w || !k_norm_w || !cos_table || !sin_table || !positions || max_pos < 1 || !arrivals ||
        !out_bf16 || !out_amax)
        return BONSAI_DECODE_ERR_ARG;
    if (M < 1 || n_kv < 1 || n_heads < n_kv || n_heads % n_kv != 0 || M * (n_heads / n_kv) > kPairTile ||
        n_kv > BONSAI_ATTN_MAX_KV_HEADS)
        return BONSAI_DECODE_ERR_ARG;
    const RopeIn rope{static_cast<const uint16_t *>(q_norm_w), static_cast<const uint16_t *>(k_norm_w),
                      static_cast<const uint16_t *>(cos_table), static_cast<const uint16_t *>(sin_table),
                      positions, eps, max_pos};
    const FinOut fin{static_cast<unsigned *>(arrivals), static_cast<uint16_t *>(out_bf16),
                     static_cast<uint16_t *>(out_amax), (n_kv + 7) & ~7};
    return launch_attention(xqkv, k_layer, v_layer, meta, scratch, nullptr, nullptr, nullptr, scale, M,
                            n_heads, n_kv, slots, sigma, &rope, &fin, static_cast<hipStream_t>(stream));
}

extern "C" int bonsai_kv_commit(void *kv, int n_layers, int n_kv, int slots, int src_slot,
                                int dst_slot, int n, void *stream) {
    if (!kv || n_layers < 1 || n_kv < 1 || slots < 1 || n < 0 || src_slot < 0 || dst_slot < 0 ||
        src_slot + n > slots || dst_slot + n > slots)
        return BONSAI_DECODE_ERR_ARG;
    if (n == 0) return BONSAI_DECODE_OK;
    if (src_slot < dst_slot + n && dst_slot < src_slot + n) return BONSAI_DECODE_ERR_ARG;  // overlap
    const int planes = 2 * n_layers * n_kv;
    const long long work = (long long)planes * n * (kHd * 2 / 16);
    if (work > 0x7fffffffLL) return BONSAI_DECODE_ERR_ARG;
    hipLaunchKernelGGL(kv_commit_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<uint4 *>(kv), planes, slots,
                       src_slot, dst_slot, n);
    return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
}

extern "C" int bonsai_draft_chain(const void *logits, int rows, int ld, int vocab, float threshold,
                                  int32_t *tokens, float *conf, int32_t *accept, void *stream) {
    if (!logits || !tokens || !conf || !accept) return BONSAI_DECODE_ERR_ARG;
    if (rows < 1 || vocab < 1 || ld < vocab || ld % 8 != 0) return BONSAI_DECODE_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(draft_rows_kernel, dim3(rows), dim3(kDraftThreads), 0, st,
                       static_cast<const uint16_t *>(logits), ld, vocab, tokens, conf);
    if (hipGetLastError() != hipSuccess) return BONSAI_DECODE_ERR_LAUNCH;
    hipLaunchKernelGGL(draft_accept_kernel, dim3(1), dim3(64), 0, st, conf, rows, threshold, accept);
    return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
}

extern "C" int64_t bonsai_draft_chain_scratch_bytes(int rows) {
    return rows < 1 ? 0 : (int64_t)rows * kDraftSplits * 4 * (int64_t)sizeof(float);
}

extern "C" int bonsai_draft_chain_ws(const void *logits, int rows, int ld, int vocab, float threshold,
                                     int32_t *tokens, float *conf, int32_t *accept, void *scratch,
                                     void *stream) {
    if (!logits || !tokens || !conf || !accept || !scratch) return BONSAI_DECODE_ERR_ARG;
    if (rows < 1 || rows > BONSAI_MAX_WIDTH || vocab < 1 || ld < vocab || ld % 8 != 0)
        return BONSAI_DECODE_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(draft_rows_split_kernel, dim3(rows * kDraftSplits), dim3(kDraftSplitThreads), 0,
                       st, static_cast<const uint16_t *>(logits), ld, vocab, kDraftSplits,
                       static_cast<float *>(scratch));
    if (hipGetLastError() != hipSuccess) return BONSAI_DECODE_ERR_LAUNCH;
    hipLaunchKernelGGL(draft_merge_accept_kernel, dim3(1), dim3(1024), 0, st,
                       static_cast<const float *>(scratch), rows, kDraftSplits, threshold, tokens,
                       conf, accept);
    return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
}

// ---------------------------------------------------------------------------
// The split draft chain for callers that cannot allocate: the partial statistics go through
// a library-owned device array instead of a caller-supplied workspace.  The array's name is
// only a host-side handle; its device address is looked up once per device and kept.
// ---------------------------------------------------------------------------
constexpr int kStaticScratchFloats = BONSAI_MAX_WIDTH * kDraftSplits * 4;  // 16 KiB
static __device__ __align__(256) float scratch[kStaticScratchFloats];
std::atomic<float *> g_static_scratch[kMaxDevices];  // the array's address on each device (every thread resolves the same value)

// Looks the array's device address up for the current device `dev` and keeps it.
static int resolve_static_scratch(int dev) {
    float *ptr = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess ||
        ptr == nullptr)
        return BONSAI_DECODE_ERR_LAUNCH;
    g_static_scratch[dev].store(ptr, std::memory_order_release);
    return BONSAI_DECODE_OK;
}

extern "C" int bonsai_decode_init(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return BONSAI_DECODE_ERR_LAUNCH;
    if (g_static_scratch[dev].load(std::memory_order_acquire) != nullptr) return BONSAI_DECODE_OK;
    return resolve_static_scratch(dev);
}

extern "C" int bonsai_draft_chain_static(const void *logits, int rows, int ld, int vocab,
                                         float threshold, int32_t *tokens, float *conf,
                                         int32_t *accept, void *stream) {
    if (!logits || !tokens || !conf || !accept) return BONSAI_DECODE_ERR_ARG;
    // rows beyond what the static array holds are refused, never truncated
    if (rows < 1 || rows > BONSAI_MAX_WIDTH || vocab < 1 || ld < vocab || ld % 8 != 0)
        return BONSAI_DECODE_ERR_ARG;
    if ((size_t)rows * kDraftSplits * 4 > (size_t)kStaticScratchFloats) return BONSAI_DECODE_ERR_ARG;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return BONSAI_DECODE_ERR_LAUNCH;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (g_static_scratch[dev].load(std::memory_order_acquire) == nullptr) {
        // the one-time address lookup is not made on a capturing stream: call bonsai_decode_init
        // (or this entry point once) before the capture
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
            return BONSAI_DECODE_ERR_NOT_INIT;
        const int rc = resolve_static_scratch(dev);
        if (rc != BONSAI_DECODE_OK) return rc;
    }
    float *ws = g_static_scratch[dev].load(std::memory_order_acquire);
    // every slot the merge reads is written by the split pass of the same call: nothing to clear
    hipLaunchKernelGGL(draft_rows_split_kernel, dim3(rows * kDraftSplits), dim3(kDraftSplitThreads), 0,
                       st, static_cast<const uint16_t *>(logits), ld, vocab, kDraftSplits, ws);
    if (hipGetLastError() != hipSuccess) return BONSAI_DECODE_ERR_LAUNCH;
    hipLaunchKernelGGL(draft_merge_accept_kernel, dim3(1), dim3(1024), 0, st,
                       static_cast<const float *>(ws), rows, kDraftSplits, threshold, tokens, conf,
                       accept);
    return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
}

// One-time set-up shared by the bf16 and the FP8 projection: device properties and the LDS limit
// of `kernel`, under the lock, with the flag checked again inside it (a second thread that
// waited for the lock finds the work done) and written last.
static int lin_setup_once(int dev, std::atomic<bool> &ready, const void *kernel) {
    if (ready.load(std::memory_order_acquire)) return BONSAI_DECODE_OK;
    std::lock_guard<std::mutex> lock(g_lin_mutex);
    if (ready.load(std::memory_order_acquire)) return BONSAI_DECODE_OK;
    int cus = 0, lds = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess)
        return BONSAI_DECODE_ERR_LAUNCH;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return BONSAI_DECODE_ERR_LAUNCH;
    g_lin_cus[dev] = cus > 0 ? cus : 1;
    g_lin_lds[dev] = lds;
    ready.store(true, std::memory_order_release);
    return BONSAI_DECODE_OK;
}

extern "C" int bonsai_bf16_linear(const void *x, const void *w, void *out, int M, int N, int K,
                                  void *stream) {
    if (!x || !w || !out) return BONSAI_DECODE_ERR_ARG;
    if (M < 1 || M > BONSAI_MAX_WIDTH || N < 1 || K < 64 || K % 64 != 0) return BONSAI_DECODE_ERR_ARG;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return BONSAI_DECODE_ERR_LAUNCH;
    {   // one-time set-up: call once before capturing
        const int rc = lin_setup_once(dev, g_lin_ready[dev], reinterpret_cast<const void *>(bf16_linear_kernel));
        if (rc != BONSAI_DECODE_OK) return rc;
    }
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return BONSAI_DECODE_ERR_ARG;
    const int nwaves = K % 512 == 0 ? 8 : (K % 256 == 0 ? 4 : (K % 128 == 0 ? 2 : 1));
    const int ntiles = (N + 15) / 16;
    // token rows per launch: up to 16, fewer when that many rows of K do not fit in LDS
    const size_t fixed = lin_lds_bytes(0, K, nwaves);
    if (fixed + (size_t)(2 * K + 16) > (size_t)g_lin_lds[dev]) return BONSAI_DECODE_ERR_ARG;
    int mt_max = (int)(((size_t)g_lin_lds[dev] - fixed) / (size_t)(2 * K + 16));
    mt_max = mt_max < kLinTokens ? mt_max : kLinTokens;
    hipStream_t st = static_cast<hipStream_t>(stream);
    for (int m0 = 0; m0 < M; m0 += mt_max) {
        const int mt = M - m0 < mt_max ? M - m0 : mt_max;
        const size_t lds = lin_lds_bytes(mt, K, nwaves);
        int per_cu = (int)((size_t)g_lin_lds[dev] / lds);
        const int by_waves = 32 / nwaves;
        per_cu = per_cu < by_waves ? per_cu : by_waves;
        per_cu = per_cu < 1 ? 1 : per_cu;
        const long want = (long)g_lin_cus[dev] * per_cu;
        const int grid = (int)(ntiles < want ? ntiles : want);
        hipLaunchKernelGGL(bf16_linear_kernel, dim3(grid), dim3(nwaves * 64), lds, st,
                           static_cast<const uint16_t *>(x) + (size_t)m0 * K,
                           static_cast<const uint16_t *>(w),
                           static_cast<uint16_t *>(out) + (size_t)m0 * N, mt, N, K, nwaves, ntiles,
                           grid);
        if (hipGetLastError() != hipSuccess) return BONSAI_DECODE_ERR_LAUNCH;
    }
    return BONSAI_DECODE_OK;
}

extern "C" int bonsai_fp8_quant_rows(const void *x, void *q, float *scale, int M, int K,
                                     void *stream) {
    if (!x || !q || !scale) return BONSAI_DECODE_ERR_ARG;
    if (M < 1 || M > BONSAI_MAX_WIDTH || K < 8 || K % 8 != 0) return BONSAI_DECODE_ERR_ARG;
    hipLaunchKernelGGL(fp8_quant_rows_kernel, dim3(1), dim3(kFp8Threads), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(x),
                       static_cast<uint8_t *>(q), scale, M * K);
    return hipGetLastError() == hipSuccess ? BONSAI_DECODE_OK : BONSAI_DECODE_ERR_LAUNCH;
}

extern "C" int bonsai_fp8_linear(const void *x, const float *x_scale, const void *w, float w_scale,
                                 void *out, int M, int N, int K, void *stream) {
    if (!x || !x_scale || !w || !out) return BONSAI_DECODE_ERR_ARG;
    if (M < 1 || M > BONSAI_MAX_WIDTH || N < 1 || K < 128 || K % 128 != 0) return BONSAI_DECODE_ERR_ARG;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return BONSAI_DECODE_ERR_ARG;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return BONSAI_DECODE_ERR_LAUNCH;
    {
        const int rc = lin_setup_once(dev, g_fp8_ready[dev], reinterpret_cast<const void *>(fp8_linear_kernel));
        if (rc != BONSAI_DECODE_OK) return rc;
    }
    const int nwaves = K % 1024 == 0 ? 8 : (K % 512 == 0 ? 4 : (K % 256 == 0 ? 2 : 1));
    const int ntiles = (N + 15) / 16;
    const size_t fixed = fp8_lin_lds_bytes(0, K, nwaves);
    if (fixed + (size_t)(K + 16) > (size_t)g_lin_lds[dev]) return BONSAI_DECODE_ERR_ARG;
    int mt_max = (int)(((size_t)g_lin_lds[dev] - fixed) / (size_t)(K + 16));
    mt_max = mt_max < kLinTokens ? mt_max : kLinTokens;
    hipStream_t st = static_cast<hipStream_t>(stream);
    for (int m0 = 0; m0 < M; m0 += mt_max) {
        const int mt = M - m0 < mt_max ? M - m0 : mt_max;
        const size_t lds = fp8_lin_lds_bytes(mt, K, nwaves);
        int per_cu = (int)((size_t)g_lin_lds[dev] / lds);
        const int by_waves = 32 / nwaves;
        per_cu = per_cu < by_waves ? per_cu : by_waves;
        per_cu = per_cu < 1 ? 1 : per_cu;
        const long want = (long)g_lin_cus[dev] * per_cu;
        const int grid = (int)(ntiles < want ? ntiles : want);
        hipLaunchKernelGGL(fp8_linear_kernel, dim3(grid), dim3(nwaves * 64), lds, st,
                           static_cast<const uint8_t *>(x) + (size_t)m0 * K, x_scale,
                           static_cast<const uint8_t *>(w), w_scale,
                           static_cast<uint16_t *>(out) + (size_t)m0 * N, mt, N, K, nwaves, ntiles,
                           grid);
        if (hipGetLastError() != hipSuccess) return BONSAI_DECODE_ERR_LAUNCH;
    }
    return BONSAI_DECODE_OK;
}
