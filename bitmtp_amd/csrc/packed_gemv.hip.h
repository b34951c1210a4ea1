// gfx950 kernels and launcher for the packed low-bit GEMV
//     C[m][n] = bf16( (sum_g fp32(G[m][n][g]) * ws[n][g]) / s[m] ),
//     G[m][n][g] = sum_{k in group g} A[m][k] * w[n][k]        (exact int32)
// for T2-g128 (BITS = 2) and Q1-g128 (BITS = 1) weights.  Replaces the CUDA
// kernels src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:29-92 and
// src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels.h:356-423 of the reference.
//
// Kernel `gemv_dot4_kernel` (one launch per GEMV, any M, N, K % 128 == 0):
//   * a wave covers 64/LPR weight rows; LPR lanes share one row and each lane
//     streams 16-byte chunks of it with global_load_dwordx4 (a full 128-byte
//     line per 8 lanes), several loads in flight per lane;
//   * the MT tokens of the block's token tile are staged once per workgroup in
//     LDS, pre-permuted to the order the in-register unpack produces, together
//     with the per-chunk activation sums (see gemv_core.h);
//   * group dot products are v_dot4_i32_i8 chains with int32 accumulation; each
//     chunk's exact int32 sum is converted to fp32, multiplied by the group's
//     scale and accumulated in fp32 (the product is exact for bf16 scales);
//   * the LPR partial sums of a row are combined with DPP adds, divided by the
//     token's activation multiplier and rounded to bf16 (round to nearest even).
// HBM traffic per launch is the packed weights plus scales, read exactly once;
// the activations (M*K bytes) come from L2.
#ifndef BONSAI_PACKED_GEMV_HIP_H
#define BONSAI_PACKED_GEMV_HIP_H

#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <stdint.h>
#include <stdio.h>

#include "gemv_core.h"
#include "wave_reduce.h"

namespace bonsai {

constexpr int kGroup = 128;
constexpr int kMaxTile = 8;       // tokens per tile (template MT is 1..kMaxTile)
constexpr int kMaxThreads = 512;  // workgroup size limit of the kernels
#ifndef BONSAI_PLANE_MAX_TILE
#define BONSAI_PLANE_MAX_TILE 2
#endif
constexpr int kPlaneMaxTile = BONSAI_PLANE_MAX_TILE;  // widest T2 token tile that takes the 4-bit-plane form

enum : int { OUT_BF16 = 0, OUT_F32 = 1, OUT_G32 = 2 };

// Which kernel the calling thread's last launch went to: the family and its template
// arguments, kept as numbers and formatted on request.  Tests and benchmarks read it to
// state (and assert) which kernel a shape reached; nothing in a launch depends on it.
struct LastKernel {
    const char *family = "none";
    int bits = 0;
    int t[6] = {0, 0, 0, 0, 0, 0};  // template arguments after BITS, -1 = unused
    int launches = 0;               // launches recorded by this thread so far
};
inline LastKernel &last_kernel() {
    static thread_local LastKernel k;
    return k;
}
inline void note_kernel(const char *family, int bits, int t0 = -1, int t1 = -1, int t2 = -1,
                        int t3 = -1, int t4 = -1, int t5 = -1) {
    LastKernel &k = last_kernel();
    k.family = family;
    k.bits = bits;
    k.t[0] = t0;
    k.t[1] = t1;
    k.t[2] = t2;
    k.t[3] = t3;
    k.t[4] = t4;
    k.t[5] = t5;
    ++k.launches;
}
// "family<bits,t0,...>" into a thread-local buffer
inline const char *last_kernel_name() {
    static thread_local char buf[128];
    const LastKernel &k = last_kernel();
    int n = snprintf(buf, sizeof buf, "%s<%d", k.family, k.bits);
    for (int i = 0; i < 6 && k.t[i] >= 0 && n < (int)sizeof buf; ++i)
        n += snprintf(buf + n, sizeof buf - n, ",%d", k.t[i]);
    if (n < (int)sizeof buf) snprintf(buf + n, sizeof buf - n, ">");
    return buf;
}

struct GemvArgs {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int M, N, K;
    int lpr_log2;        // log2(lanes per weight row)
    int passes;          // row passes per wave
    int out_f32;         // 1: store the fp32 value, 0: round to bf16
    uint32_t div_magic;  // floor(2^32 / (4*C)) + 1, for task -> token in the staging loop
    // fused forms only (see below)
    const void *in_parts = nullptr;       // PRO_BF16_AMAX: bf16 maxima, PRO_BF16_NORM: fp64 sums of squares
    int in_count = 0;                     // parts per token in in_parts
    const uint16_t *norm_w = nullptr;     // PRO_BF16_NORM: bf16 [K]
    float eps = 0.0f;
    const uint16_t *residual = nullptr;   // EPI_ADD_SUMSQ: bf16 [M, N]
    void *out_parts = nullptr;            // EPI_SILU_PAIR: bf16 maxima, EPI_ADD_SUMSQ: fp64 sums of squares
    int out_count = 0;                    // parts per token this launch writes: its workgroup count
    float *s_out = nullptr;               // PRO_BF16_*: receives the multipliers (may be null)
};

// ---- decode steps of one or two tokens without their element-wise launches -----------------
// Between two projections the reference runs a fused Python helper: residual add + RMSNorm +
// quantisation (src/bonsai_sft/gpu/model.py:307-336) or SiLU(gate) * up + quantisation
// (model.py:1059-1061).  For blocks of one or two tokens such a launch costs as much as a
// projection.  What keeps it from being folded into its neighbours is that the quantisation (and
// the norm) needs a value of the whole row -- max |x|, sum x^2 -- before the first element can be
// used.  The fused forms of the dot4 kernel split that: the projection that PRODUCES a row leaves,
// per workgroup and token, the maximum or the sum over the columns it stored (plain stores, one
// part per workgroup: its waves meet in LDS behind a barrier at the end); the projection that
// CONSUMES the row has every wave add up the parts (a few hundred values) and then derives the
// multiplier and quantises while it stages.
//   epilogues  EPI_SILU_PAIR   rows [gate; up] visited as gate 0, up 0, gate 1, up 1, ... so that the
//                              two results of a column meet in neighbouring lane sets; stores
//                              inner = bf16(bf16(silu(gate)) * up) [M, N/2] and max |inner| parts
//              EPI_ADD_SUMSQ   stores h = bf16(residual + bf16(y)) [M, N] and parts of sum h^2
//                              (fp64 sums of exact fp32 squares, in a fixed order)
//   prologues  PRO_BF16_AMAX   x = bf16 [M, K] with max |x| parts: s = fl(fl(1 / max(amax, 1e-5)) * 127),
//                              q = clamp(rne(fl(x * s)), -128, 127)
//              PRO_BF16_NORM   h = bf16 [M, K] with sum h^2 parts and norm weights w:
//                              var = fp32(sum) / K, rs = 1 / sqrt(var + eps), x = bf16(w * bf16(h * rs)),
//                              max |x| over the workgroup (one more barrier), then as PRO_BF16_AMAX
// The operations and their rounding points are those of the stand-alone producers (act_quant.hip),
// so q, s and the results are the same bits as the separate launches give; the one difference is
// the order in which the fp64 sum of squares is added up, which shows only where two fp64 roundings
// differ and the fp32 conversion of the sum lands on the other side of a rounding boundary.
// (Atomic maxima in memory instead of parts: 1536 of them over 32 cache lines cost 0.9 us on a
// 3.5 us launch, over two lines 13 us.)
constexpr int PRO_INT8 = 0, PRO_BF16_AMAX = 1, PRO_BF16_NORM = 2;
constexpr int EPI_PLAIN = 0, EPI_SILU_PAIR = 1, EPI_ADD_SUMSQ = 2;
constexpr int fuse_code(int pro, int epi) { return pro | (epi << 2); }
constexpr int FUSE_NONE = 0;
// Maxima are bf16 (max |x| is one of the bf16 values stored): up to 1024 of them are two 16-byte
// loads per lane of a wave; sums are fp64: up to 256 of them are four 8-byte loads per lane.
constexpr int kAmaxMaxParts = 1024;
constexpr int kSumsqMaxParts = 256;
// elements per token of the maxima array: parts rounded up to whole 16-byte words (the pad holds 0)
__host__ __device__ constexpr int amax_ld(int parts) { return (parts + 7) & ~7; }
constexpr int kFusedMeetBytes = 64 + 2 * (kMaxThreads / 64) * 8;  // LDS behind the staged activations

__device__ __forceinline__ float bf16_round_f32(float f) {
    const __bf16 b = static_cast<__bf16>(f);  // round to nearest even (v_cvt_pk_bf16_f32)
    uint16_t u;
    __builtin_memcpy(&u, &b, 2);
    return __uint_as_float((uint32_t)u << 16);
}

// bf16(bf16(silu(g)) * u) with silu through the hardware exp2 and reciprocal, exactly as
// silu_mul_quant_kernel (act_quant.hip) evaluates it.
__device__ __forceinline__ float silu_mul_bf16(float g, float u) {
    const float ex = __builtin_amdgcn_exp2f(g * -1.44269504088896341f);
    const float sg = bf16_round_f32(g * __builtin_amdgcn_rcpf(1.0f + ex));
    return bf16_round_f32(sg * u);
}

// Sixteen bf16 values (two 16-byte words) -> sixteen int8 in natural order.
__device__ __forceinline__ u32x4 quant16_bf16(const u32x4 lo, const u32x4 hi, float s) {
    const auto q1 = [s](uint32_t bits) {
        float r = __builtin_rintf(__uint_as_float(bits) * s);
        r = fminf(fmaxf(r, -128.0f), 127.0f);
        return (uint32_t)((int)r) & 0xffu;
    };
    const auto q4 = [&q1](uint32_t d0, uint32_t d1) {
        return q1(d0 << 16) | (q1(d0 & 0xffff0000u) << 8) | (q1(d1 << 16) << 16) |
               (q1(d1 & 0xffff0000u) << 24);
    };
    return u32x4{q4(lo.x, lo.y), q4(lo.z, lo.w), q4(hi.x, hi.y), q4(hi.z, hi.w)};
}

// Sixteen fp32 values -> sixteen int8 in natural order.
__device__ __forceinline__ u32x4 quant16_f32(const float *v, float s) {
    const auto q1 = [s](float x) {
        float r = __builtin_rintf(x * s);
        r = fminf(fmaxf(r, -128.0f), 127.0f);
        return (uint32_t)((int)r) & 0xffu;
    };
    const auto q4 = [&q1](const float *x) { return q1(x[0]) | (q1(x[1]) << 8) | (q1(x[2]) << 16) | (q1(x[3]) << 24); };
    return u32x4{q4(v), q4(v + 4), q4(v + 8), q4(v + 12)};
}

// Eight bf16 values h and their norm weights w (one 16-byte word each) -> bf16(w * bf16(h * rs)),
// as rmsnorm_quant_kernel (act_quant.hip) evaluates it; returns max |.| of the eight.
__device__ __forceinline__ float normalise8(const u32x4 h, const u32x4 w, float rs, float *out) {
    const uint32_t hd[4] = {h.x, h.y, h.z, h.w}, wd[4] = {w.x, w.y, w.z, w.w};
    float top = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i] = bf16_round_f32(__uint_as_float(wd[i] << 16) * bf16_round_f32(__uint_as_float(hd[i] << 16) * rs));
        out[2 * i + 1] = bf16_round_f32(__uint_as_float(wd[i] & 0xffff0000u) *
                                        bf16_round_f32(__uint_as_float(hd[i] & 0xffff0000u) * rs));
        top = fmaxf(top, fmaxf(fabsf(out[2 * i]), fabsf(out[2 * i + 1])));
    }
    return top;
}

template <bool SF16>
__device__ __forceinline__ float scale_to_f32(uint16_t raw) {
    if (SF16) {
        _Float16 h;
        __builtin_memcpy(&h, &raw, 2);
        return (float)h;
    }
    return __uint_as_float((uint32_t)raw << 16);
}

// fp32 -> bf16 bits, round to nearest even, quiet NaN preserved.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}

constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7-i inside each 8 lanes
constexpr int kDppMirror = 0x140;      // lane i <-> 15-i inside each 16 lanes

// Sum over the 2^lpr_log2 consecutive lanes that share a weight row; every lane
// of the set ends up with the total.
__device__ __forceinline__ float row_lanes_sum(float v, int lpr_log2) {
    v += __int_as_float(dpp_i32<kDppXor1>(__float_as_int(v)));
    v += __int_as_float(dpp_i32<kDppXor2>(__float_as_int(v)));
    if (lpr_log2 >= 3) v += __int_as_float(dpp_i32<kDppHalfMirror>(__float_as_int(v)));
    if (lpr_log2 >= 4) v += __int_as_float(dpp_i32<kDppMirror>(__float_as_int(v)));
    if (lpr_log2 >= 5) v += __shfl_xor(v, 16);
    if (lpr_log2 >= 6) v += __shfl_xor(v, 32);
    return v;
}

// U 16-byte weight chunks of one lane plus the raw 16-bit scales of their groups.
template <int U>
struct WeightBatch {
    u32x4 w[U];
    uint16_t sraw[U];
};

// ---- 4-bit planes (T2, narrow token tiles) -------------------------------------------------
// For one or two tokens the dot4 body is bound by its vector instructions (seven to unpack a
// packed dword into byte vectors, four v_dot4 per token).  With the activations staged as 4-bit
// planes, a = 16 hi + lo (hi signed, lo unsigned; even and odd positions apart), the codes are
// only masked to nibbles -- e = p & 0x33333333, o = (p >> 2) & 0x33333333: three operations --
// and meet the planes in four v_dot8 per token: 28 operations per 16-byte chunk against 44.
// raw = 16 H + L is the same integer sum of a * code the byte form gives.

// Sixteen natural-order activations (four dwords) -> {even hi, even lo, odd hi, odd lo}: nibble
// n of an "even" word belongs to activation 2 n, of an "odd" word to activation 2 n + 1.
__device__ __forceinline__ u32x4 nibble_planes16(const u32x4 in) {
    const uint32_t e0 = __builtin_amdgcn_perm(in.y, in.x, 0x06040200u);
    const uint32_t e1 = __builtin_amdgcn_perm(in.w, in.z, 0x06040200u);
    const uint32_t o0 = __builtin_amdgcn_perm(in.y, in.x, 0x07050301u);
    const uint32_t o1 = __builtin_amdgcn_perm(in.w, in.z, 0x07050301u);
    const auto lo = [](uint32_t x) { return x & 0x0f0f0f0fu; };
    const auto hi = [](uint32_t x) { return (x >> 4) & 0x0f0f0f0fu; };
    const auto pk = [](uint32_t x) { return x | (x >> 4); };  // bytes 0 and 2: two nibbles each
    u32x4 r;
    r.x = __builtin_amdgcn_perm(pk(hi(e1)), pk(hi(e0)), 0x06040200u);
    r.y = __builtin_amdgcn_perm(pk(lo(e1)), pk(lo(e0)), 0x06040200u);
    r.z = __builtin_amdgcn_perm(pk(hi(o1)), pk(hi(o0)), 0x06040200u);
    r.w = __builtin_amdgcn_perm(pk(lo(o1)), pk(lo(o0)), 0x06040200u);
    return r;
}

// Plane form of stage_quarter<2, MT>: the same LDS slot receives the four plane words of the
// quarter's sixteen activations; returns their sum.
template <int MT>
__device__ __forceinline__ int stage_quarter_planes(const u32x4 *src, u32x4 *act, int m, int chunk, int sub) {
    const u32x4 in = src[0];
    act[act_index<2, MT>(m, sub, chunk)] = nibble_planes16(in);
    return sum4_i8(in.x) + sum4_i8(in.y) + sum4_i8(in.z) + sum4_i8(in.w);
}

// Plane form of chunk_dot_raw<2, MT>: raw[m] += sum a[m][k] * code[k] over the chunk.
template <int MT>
__device__ __forceinline__ void chunk_dot_raw_planes(const u32x4 w, const u32x4 *act, int chunk, int raw[MT]) {
    const uint32_t p[4] = {w.x, w.y, w.z, w.w};
    int ah[MT];
    uint32_t al[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        ah[m] = 0;
        al[m] = 0;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const uint32_t e = p[t] & 0x33333333u, o = (p[t] >> 2) & 0x33333333u;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const u32x4 a = act[act_index<2, MT>(m, t, chunk)];
            ah[m] = __builtin_amdgcn_sdot8((int)a.x, (int)e, ah[m], false);
            al[m] = __builtin_amdgcn_udot8(a.y, e, al[m], false);
            ah[m] = __builtin_amdgcn_sdot8((int)a.z, (int)o, ah[m], false);
            al[m] = __builtin_amdgcn_udot8(a.w, o, al[m], false);
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) raw[m] += (ah[m] << 4) + (int)al[m];
}

// BITS: 2 = T2, 1 = Q1.  MT: tokens in the tile.  U: 16-byte weight loads a lane
// issues back to back (one batch).  G32: write the int32 group sums instead of
// the scaled result.  SF16: group scales are fp16 instead of bf16.
// The kernel proper: workgroup `bx` of the GEMV `a`, token tile `by`, `pthreads` threads.
template <int BITS, int MT, int U, bool G32, bool SF16, int FUSE = FUSE_NONE>
__device__ __forceinline__ void gemv_dot4_body(const GemvArgs &a, int bx, int by, int pthreads,
                                               unsigned char *smem) {
    using F = Fmt<BITS>;
    constexpr int PRO = FUSE & 3, EPI = FUSE >> 2;
    constexpr bool BF16_IN = PRO != PRO_INT8;
    static_assert(FUSE == FUSE_NONE || (!G32 && MT <= 2), "fused forms: one or two tokens, scaled output");
    // 4-bit planes and v_dot8 for T2 tiles of one or two tokens (see above)
    constexpr bool P4 = BITS == 2 && MT <= kPlaneMaxTile;

    const int K = a.K, N = a.N, M = a.M;
    const int C = K / F::kChunkWeights;  // 16-byte chunks per weight row
    const int ng = K / kGroup;

    u32x4 *act = reinterpret_cast<u32x4 *>(smem);  // C blocks, see gemv_core.h
    int *asum = reinterpret_cast<int *>(smem);

    const int tid = threadIdx.x;
    const int nthreads = pthreads;  // the workgroup size, as a parameter: blockDim is a load
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int nwaves = nthreads >> 6;
    const int lpr_log2 = a.lpr_log2;
    const int lpr = 1 << lpr_log2;
    const int c = lane & (lpr - 1);  // position of the lane along K
    const int r = lane >> lpr_log2;  // row of the lane inside the wave
    const int rpw = 64 >> lpr_log2;  // rows per wave and pass
    const int IT = (C + lpr - 1) >> lpr_log2;
    const int nb = (IT + U - 1) / U;
    const int m0 = by * MT;
    const int row0 = (bx * a.passes * nwaves + wave) * rpw + r;
    const int row_step = nwaves * rpw;  // rows between two passes of a wave

    // All loads of a batch are unconditional (indices clamped into the row) and
    // issued back to back; lanes past the end of a row are masked when used.
    // EPI_SILU_PAIR: visiting order gate 0, up 0, gate 1, up 1, ... over the rows [gate; up]
    const int half_n = N >> 1;
    auto stored_row = [&](int row) {
        return EPI == EPI_SILU_PAIR ? (row & 1) * half_n + (row >> 1) : row;
    };
    auto load_batch = [&](WeightBatch<U> &wb, int row, int it0) {
        const int row_c = stored_row(row < N ? row : N - 1);
        const u32x4 *wrow = reinterpret_cast<const u32x4 *>(a.B) + (size_t)row_c * C;
        const uint16_t *srow = a.ws + (size_t)row_c * ng;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int chunk = (it0 + u) * lpr + c;
            const int chunk_c = chunk < C ? chunk : C - 1;
            wb.w[u] = wrow[chunk_c];
            if (!G32) wb.sraw[u] = srow[chunk_c >> F::kGroupShift];
        }
    };

    // ---- prologue: first staging loads, then the first weight batch, so that the
    // staging data (an L2 hit) is back before the weights (HBM) are.
    const int ntasks = MT * C * 4;  // quarter chunks to stage
    constexpr int kQ = F::kUnits / 4;  // 16-byte words per quarter
    // (bf16 activations: twice the bytes per quarter)
    constexpr int kSrcWords = BF16_IN ? 2 * kQ : kQ;
    constexpr int kW = kMaxThreads / 64;
    auto task_src = [&](int task, int &m, int &chunk, int &sub) {
        if constexpr (FUSE != FUSE_NONE)
            m = (MT > 1 && task >= 4 * C) ? 1 : 0;  // at most two tokens: no division
        else
            m = (int)__umulhi((uint32_t)task, a.div_magic);  // task / (4*C)
        const int rest = task - m * 4 * C;
        chunk = rest >> 2;
        sub = rest & 3;
        const int msrc = (m0 + m) < M ? (m0 + m) : M - 1;
        return reinterpret_cast<const u32x4 *>(a.A + (size_t)msrc * K * (BF16_IN ? 2 : 1)) +
               ((size_t)chunk * 4 + sub) * kSrcWords;
    };
    // PRO_BF16_NORM: the norm weights of the same elements
    auto task_w = [&](int chunk, int sub) {
        return reinterpret_cast<const u32x4 *>(a.norm_w) + ((size_t)chunk * 4 + sub) * kSrcWords;
    };
    u32x4 first_q[kSrcWords];
    u32x4 first_w[PRO == PRO_BF16_NORM ? kSrcWords : 1];
    int fm = 0, fchunk = 0, fsub = 0;
    const bool has_first = tid < ntasks;
    if (has_first) {
        const u32x4 *src = task_src(tid, fm, fchunk, fsub);
#pragma unroll
        for (int i = 0; i < kSrcWords; ++i) first_q[i] = src[i];
        if constexpr (PRO == PRO_BF16_NORM) {
            const u32x4 *wsrc = task_w(fchunk, fsub);
#pragma unroll
            for (int i = 0; i < kSrcWords; ++i) first_w[i] = wsrc[i];
        }
    }
    // Every wave reads the parts of a token itself (a workgroup barrier for them costs more than
    // the repeated reads): maxima as one or two 16-byte words per lane, sums as up to four doubles
    // per lane, added in that order
    // (nothing below may wait for these loads before the weight loads are issued)
    u32x4 part_bits[MT][2];
    double part_raw[MT][4];
    if (PRO == PRO_BF16_AMAX) {
        const int words = amax_ld(a.in_count) >> 3;  // at most 128
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const u32x4 *prow = reinterpret_cast<const u32x4 *>(
                static_cast<const uint16_t *>(a.in_parts) + (size_t)((m0 + m) < M ? (m0 + m) : M - 1) * (words * 8));
            part_bits[m][0] = prow[lane < words ? lane : words - 1];  // past the end: a repeat
            part_bits[m][1] = prow[lane + 64 < words ? lane + 64 : words - 1];
        }
    }
    if (PRO == PRO_BF16_NORM) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const double *prow = static_cast<const double *>(a.in_parts) +
                                 (size_t)((m0 + m) < M ? (m0 + m) : M - 1) * a.in_count;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int idx = lane + 64 * j;
                part_raw[m][j] = 0.0;
                if (64 * j < a.in_count)  // uniform: no load for a run of 64 parts that does not exist
                    part_raw[m][j] = prow[idx < a.in_count ? idx : 0];  // past the end: not added below
            }
        }
    }

    WeightBatch<U> cur, nxt;
    load_batch(cur, row0, 0);
    // (arguments that only the end of the kernel needs are fetched now)
    if (EPI != EPI_PLAIN) asm volatile("" ::"s"(a.out_parts), "s"(a.out_count));
    // EPI_ADD_SUMSQ: the residual values of the first pass travel with the weights
    // (raw, from a clamped address and untouched until the epilogue: an operation on it here would
    // wait for the weight loads issued before it)
    uint16_t res0[MT];
    if constexpr (EPI == EPI_ADD_SUMSQ) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            res0[m] = a.residual[(size_t)((m0 + m) < M ? (m0 + m) : M - 1) * N + (row0 < N ? row0 : N - 1)];
    }

    // the multiplier of a token picked by a run-time index (at most two tokens)
    auto of_token = [](const float *v, int m) {
        float x = v[0];
#pragma unroll
        for (int t = 1; t < MT; ++t) x = (m == t) ? v[t] : x;
        return x;
    };
    float sdiv[MT];
    float rs[MT];                                             // PRO_BF16_NORM: 1 / sqrt(var + eps)
    float first_n[PRO == PRO_BF16_NORM ? kSrcWords * 8 : 1];  // the first task's normalised values
    if constexpr (PRO == PRO_BF16_AMAX) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            // non-negative bf16 values order as unsigned 16-bit integers
            typedef unsigned short us2 __attribute__((ext_vector_type(2)));
            const auto pk = [](uint32_t x) { us2 r; __builtin_memcpy(&r, &x, 4); return r; };
            const u32x4 v = part_bits[m][0], v1 = part_bits[m][1];
            const us2 p2 = __builtin_elementwise_max(
                __builtin_elementwise_max(__builtin_elementwise_max(pk(v.x), pk(v.y)),
                                          __builtin_elementwise_max(pk(v.z), pk(v.w))),
                __builtin_elementwise_max(__builtin_elementwise_max(pk(v1.x), pk(v1.y)),
                                          __builtin_elementwise_max(pk(v1.z), pk(v1.w))));
            const uint32_t top = p2.x > p2.y ? p2.x : p2.y;
            const float amax = bonsai_wave::max64(__uint_as_float(top << 16));
            const float recip = 1.0f / fmaxf(amax, 1e-5f);  // IEEE division, rounded on its own
            sdiv[m] = recip * 127.0f;
        }
    } else if constexpr (PRO == PRO_BF16_NORM) {
        float lmax[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            double mine = part_raw[m][0];
            mine = lane < a.in_count ? mine : 0.0;
#pragma unroll
            for (int j = 1; j < 4; ++j) mine += (lane + 64 * j) < a.in_count ? part_raw[m][j] : 0.0;
            const double total = bonsai_wave::sum64(mine);
            const float var = (float)total / (float)K;
            rs[m] = 1.0f / sqrtf(var + a.eps);
            lmax[m] = 0.0f;
        }
        // first pass over this thread's quarters: normalise, maxima per token
        if (has_first) {
            float top = 0.0f;
#pragma unroll
            for (int i = 0; i < kSrcWords; ++i)
                top = fmaxf(top, normalise8(first_q[i], first_w[i], of_token(rs, fm), first_n + 8 * i));
#pragma unroll
            for (int m = 0; m < MT; ++m) lmax[m] = (m == fm) ? top : lmax[m];
        }
        for (int task = tid + nthreads; task < ntasks; task += nthreads) {
            int m, chunk, sub;
            const u32x4 *src = task_src(task, m, chunk, sub);
            const u32x4 *wsrc = task_w(chunk, sub);
            float tmp[8], top = 0.0f;
#pragma unroll
            for (int i = 0; i < kSrcWords; ++i) top = fmaxf(top, normalise8(src[i], wsrc[i], of_token(rs, m), tmp));
#pragma unroll
            for (int t = 0; t < MT; ++t) lmax[t] = (t == m) ? fmaxf(lmax[t], top) : lmax[t];
        }
        float *pro_meet = reinterpret_cast<float *>(smem + (size_t)C * block_words<BITS, MT>() * 16);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float wm = bonsai_wave::max64(lmax[m]);
            if (lane == 0) pro_meet[m * kW + wave] = wm;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float amax = 0.0f;
#pragma unroll
            for (int w = 0; w < kW; ++w) amax = fmaxf(amax, pro_meet[m * kW + (w < nwaves ? w : nwaves - 1)]);
            const float recip = 1.0f / fmaxf(amax, 1e-5f);
            sdiv[m] = recip * 127.0f;
        }
    } else if (!G32) {
#pragma unroll
        for (int m = 0; m < MT; ++m) sdiv[m] = a.s[(m0 + m) < M ? (m0 + m) : M - 1];
    }
    if (BF16_IN && bx == 0 && tid == 0 && a.s_out != nullptr) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if ((m0 + m) < M) a.s_out[m0 + m] = sdiv[m];
    }
    // bf16 activations: a quarter as int8, quantised with its token's multiplier
    auto quantised = [&](const u32x4 *raw, int m, u32x4 *q) {
        const float sm = of_token(sdiv, m);
#pragma unroll
        for (int i = 0; i < kQ; ++i) q[i] = quant16_bf16(raw[2 * i], raw[2 * i + 1], sm);
    };

    // ---- stage the token tile: permuted activations and per-chunk sums into LDS
    if (has_first) {
        u32x4 fq[kQ];
        const u32x4 *fsrc = first_q;
        if constexpr (PRO == PRO_BF16_AMAX) {
            quantised(first_q, fm, fq);
            fsrc = fq;
        }
        if constexpr (PRO == PRO_BF16_NORM) {
#pragma unroll
            for (int i = 0; i < kQ; ++i) fq[i] = quant16_f32(first_n + 16 * i, of_token(sdiv, fm));
            fsrc = fq;
        }
        int qs;
        if constexpr (P4)
            qs = stage_quarter_planes<MT>(fsrc, act, fm, fchunk, fsub);
        else
            qs = stage_quarter<BITS, MT>(fsrc, act, fm, fchunk, fsub);
        qs += dpp_i32<kDppXor1>(qs);
        qs += dpp_i32<kDppXor2>(qs);
        if (fsub == 0) asum[asum_index<BITS, MT>(fm, fchunk)] = qs;
    }
    for (int task = tid + nthreads; task < ntasks; task += nthreads) {
        int m, chunk, sub;
        const u32x4 *src = task_src(task, m, chunk, sub);
        u32x4 tq[kQ];
        if constexpr (PRO == PRO_BF16_AMAX) {
            u32x4 raw[kSrcWords];
#pragma unroll
            for (int i = 0; i < kSrcWords; ++i) raw[i] = src[i];
            quantised(raw, m, tq);
            src = tq;
        }
        if constexpr (PRO == PRO_BF16_NORM) {
            // (second pass: the values are normalised again rather than kept)
            const u32x4 *wsrc = task_w(chunk, sub);
            float tmp[kSrcWords * 8];
#pragma unroll
            for (int i = 0; i < kSrcWords; ++i) (void)normalise8(src[i], wsrc[i], of_token(rs, m), tmp + 8 * i);
#pragma unroll
            for (int i = 0; i < kQ; ++i) tq[i] = quant16_f32(tmp + 16 * i, of_token(sdiv, m));
            src = tq;
        }
        int qs;
        if constexpr (P4)
            qs = stage_quarter_planes<MT>(src, act, m, chunk, sub);
        else
            qs = stage_quarter<BITS, MT>(src, act, m, chunk, sub);
        qs += dpp_i32<kDppXor1>(qs);
        qs += dpp_i32<kDppXor2>(qs);
        if (sub == 0) asum[asum_index<BITS, MT>(m, chunk)] = qs;
    }
    // where the waves of the workgroup meet at the end of an epilogue that leaves parts
    unsigned char *epi_meet = smem + (size_t)C * block_words<BITS, MT>() * 16 + 64;
    __syncthreads();

    float accf[MT];
    float inner_max[MT];  // EPI_SILU_PAIR: max |inner| this lane has stored
    double sumsq[MT];     // EPI_ADD_SUMSQ: sum of the squares this lane has stored
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        accf[m] = 0.0f;
        inner_max[m] = 0.0f;
        sumsq[m] = 0.0;
    }

    // One batch of one pass: unpack, dot, scale, and after the last batch of the
    // pass reduce over the row's lanes and store.
    auto compute_batch = [&](const WeightBatch<U> &wb, int pass, int b) {
        const int row = row0 + pass * row_step;
        const bool row_ok = row < N;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int chunk = (b * U + u) * lpr + c;
            const bool ok = row_ok && chunk < C;
            const int chunk_c = chunk < C ? chunk : C - 1;
            int raw[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) raw[m] = 0;
            if constexpr (P4)
                chunk_dot_raw_planes<MT>(wb.w[u], act, chunk_c, raw);
            else
                chunk_dot_raw<BITS, MT>(wb.w[u], act, chunk_c, raw);
            float wsf = 0.0f;
            if (!G32) wsf = scale_to_f32<SF16>(wb.sraw[u]);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                int g = chunk_dot_signed<BITS>(raw[m], asum[asum_index<BITS, MT>(m, chunk_c)]);
                g = ok ? g : 0;
                if (G32) {
                    // T2: two neighbouring lanes hold the halves of one group.
                    if (BITS == 2) g += dpp_i32<kDppXor1>(g);
                    const bool writer = (BITS == 2) ? ((c & 1) == 0) : true;
                    if (writer && ok && (m0 + m) < M) {
                        int32_t *G = reinterpret_cast<int32_t *>(a.out);
                        G[((size_t)(m0 + m) * N + row) * ng + (chunk >> F::kGroupShift)] = g;
                    }
                } else {
                    accf[m] += (float)g * wsf;
                }
            }
        }
        if (b == nb - 1 && !G32) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const float sum = row_lanes_sum(accf[m], lpr_log2);
                accf[m] = 0.0f;
                if constexpr (EPI == EPI_ADD_SUMSQ) {
                    if (c == 0 && row_ok && (m0 + m) < M) {
                        const size_t o = (size_t)(m0 + m) * N + row;
                        const float res = __uint_as_float((uint32_t)(pass == 0 ? res0[m] : a.residual[o]) << 16);
                        const float hv = bf16_round_f32(bf16_round_f32(sum / sdiv[m]) + res);
                        reinterpret_cast<uint16_t *>(a.out)[o] = (uint16_t)(__float_as_uint(hv) >> 16);
                        const float sq = hv * hv;  // exact: two 8-bit significands
                        sumsq[m] += (double)sq;
                    }
                    continue;
                }
                if constexpr (EPI == EPI_SILU_PAIR) {
                    // every lane of a row's set holds the row's value; the next set (row ^ 1)
                    // holds the other half of the column
                    const float mine = bf16_round_f32(sum / sdiv[m]);
                    const float other = __shfl_xor(mine, lpr);
                    if (c == 0 && (row & 1) == 0 && row_ok && (m0 + m) < M) {
                        const float inner = silu_mul_bf16(mine, other);
                        reinterpret_cast<uint16_t *>(a.out)[(size_t)(m0 + m) * half_n + (row >> 1)] =
                            (uint16_t)(__float_as_uint(inner) >> 16);
                        inner_max[m] = fmaxf(inner_max[m], fabsf(inner));
                    }
                    continue;
                }
                if (c == 0 && row_ok && (m0 + m) < M) {
                    const float y = sum / sdiv[m];
                    if (a.out_f32)
                        reinterpret_cast<float *>(a.out)[(size_t)(m0 + m) * N + row] = y;
                    else
                        reinterpret_cast<uint16_t *>(a.out)[(size_t)(m0 + m) * N + row] =
                            f32_to_bf16_rne(y);
                }
            }
        }
    };

    // Batches of all passes form one sequence; two register buffers alternate so
    // that the loads of batch i+1 are in flight while batch i is consumed.  The
    // steady-state loop has no conditional loads, which lets the compiler wait
    // for exactly the loads it needs.
    const int total = a.passes * nb;
    auto advance = [&](int &pass, int &b) {
        if (++b == nb) {
            b = 0;
            ++pass;
        }
    };
    int pa = 0, ba = 0;  // position of the batch in `cur`
    int i = 0;
    while (i + 2 < total) {
        int pb = pa, bb = ba;
        advance(pb, bb);
        load_batch(nxt, row0 + pb * row_step, bb * U);
        compute_batch(cur, pa, ba);
        pa = pb;
        ba = bb;
        advance(pa, ba);
        load_batch(cur, row0 + pa * row_step, ba * U);
        compute_batch(nxt, pb, bb);
        i += 2;
    }
    if (i + 1 < total) {
        int pb = pa, bb = ba;
        advance(pb, bb);
        load_batch(nxt, row0 + pb * row_step, bb * U);
        compute_batch(cur, pa, ba);
        compute_batch(nxt, pb, bb);
    } else {
        compute_batch(cur, pa, ba);
    }
    if constexpr (EPI == EPI_SILU_PAIR) {
        // the waves' maxima meet in LDS behind a barrier (every wave is at its end by then) and
        // thread 0 stores the workgroup's part.  Measured on 12288 x 2048 at one token (3.45 us as
        // a plain GEMV, 3.70 us with the pairing and SiLU alone): this barrier 3.97 us, a count in
        // LDS whose last arriver stores 4.14 us, one part per wave 3.83 us (but four times the
        // parts for every wave of the consumer to read)
        uint32_t *meet = reinterpret_cast<uint32_t *>(epi_meet);
        float wmax[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) wmax[m] = bonsai_wave::max64(inner_max[m]);
        if (lane == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) meet[m * kW + wave] = __float_as_uint(wmax[m]);
        }
        __syncthreads();
        if (tid == 0) {
            const int parts = a.out_count, ld = amax_ld(parts);  // (the grid size, as a parameter)
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if ((m0 + m) >= M) continue;
                uint32_t top = 0u;  // non-negative floats order as their bits
#pragma unroll
                for (int w = 0; w < kW; ++w) {
                    const uint32_t v = meet[m * kW + (w < nwaves ? w : nwaves - 1)];
                    top = v > top ? v : top;
                }
                uint16_t *prow = static_cast<uint16_t *>(a.out_parts) + (size_t)(m0 + m) * ld;
                prow[bx] = (uint16_t)(top >> 16);  // exact: one of the bf16 values stored
                if (bx == parts - 1)
                    for (int w = parts; w < ld; ++w) prow[w] = 0;
            }
        }
    }
    if constexpr (EPI == EPI_ADD_SUMSQ) {
        // the same meeting for the sums: a wave's lanes on the DPP butterfly, the waves left to right
        double *meet = reinterpret_cast<double *>(epi_meet);
        double wsum[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) wsum[m] = bonsai_wave::sum64(sumsq[m]);
        if (lane == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) meet[m * kW + wave] = wsum[m];
        }
        __syncthreads();
        if (tid == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if ((m0 + m) >= M) continue;
                double v[kW];  // all slots read at once (those past nwaves hold stale words: not added)
#pragma unroll
                for (int w = 0; w < kW; ++w) v[w] = meet[m * kW + w];
                double t = v[0];
#pragma unroll
                for (int w = 1; w < kW; ++w) t += w < nwaves ? v[w] : 0.0;
                static_cast<double *>(a.out_parts)[(size_t)(m0 + m) * a.out_count + bx] = t;
            }
        }
    }
}

template <int BITS, int MT, int U, bool G32, bool SF16>
__global__ void __launch_bounds__(kMaxThreads)
gemv_dot4_kernel(const int8_t *pA, const uint8_t *pB, void *pout, const float *ps,
                 const uint16_t *pws, int pM, int pN, int pK, int plpr_log2, int ppasses,
                 int pout_f32, uint32_t pdiv_magic, int pthreads) {
    // scalar parameters (instead of one struct) so that they can be preloaded into SGPRs
    const GemvArgs a{pA, pB, pout, ps, pws, pM, pN, pK, plpr_log2, ppasses, pout_f32, pdiv_magic};
    extern __shared__ __align__(16) unsigned char smem[];
    gemv_dot4_body<BITS, MT, U, G32, SF16>(a, (int)blockIdx.x, (int)blockIdx.y, pthreads, smem);
}

// The fused forms of the same body; bf16 scales.
// Sixteen dwords of arguments arrive in SGPRs with the wave; a later one is a scalar load that
// the compiler places where the value is first needed (0.3 us when that is the end of the last
// wave of a workgroup).  So the first sixteen are what the prologue needs -- `px` the multipliers
// (PRO_INT8) or the parts to read, `pw` the norm weights -- and the body asks for what only the
// end of the kernel needs once its first loads are on their way.
// pgeom = lpr_log2 | passes << 4 | out_f32 << 9 | waves << 10 | parts to read << 14.
template <int BITS, int MT, int U, int FUSE>
__global__ void __launch_bounds__(kMaxThreads)
gemv_dot4_fused_kernel(const int8_t *pA, const uint8_t *pB, void *pout, const uint16_t *pws,
                       const void *px, const uint16_t *pw, int pM, int pN, int pK, int pgeom,
                       float peps, void *py, const uint16_t *pr, int pout_count, float *ps_out) {
    GemvArgs a{pA, pB, pout, nullptr, pws, pM, pN, pK, pgeom & 0xf, (pgeom >> 4) & 0x1f, (pgeom >> 9) & 1, 0u};
    if ((FUSE & 3) == PRO_INT8)
        a.s = static_cast<const float *>(px);
    else
        a.in_parts = px;
    a.in_count = (pgeom >> 14) & 0x7ff;
    a.norm_w = pw;
    a.eps = peps;
    a.residual = pr;
    a.out_parts = py;
    a.out_count = pout_count;
    a.s_out = ps_out;
    extern __shared__ __align__(16) unsigned char smem[];
    gemv_dot4_body<BITS, MT, U, false, false, FUSE>(a, (int)blockIdx.x, (int)blockIdx.y,
                                                    ((pgeom >> 10) & 0xf) * 64, smem);
}

// ---- several GEMVs in one launch -------------------------------------------------------
// The same kernel over a table of up to twelve GEMVs: a workgroup finds its GEMV by comparing
// its number with the range ends, which arrive in SGPRs with the wave (preloaded kernel
// arguments), reads that GEMV's 64-byte descriptor with one scalar load and runs the body.
// For narrow blocks (one or two tokens) this is the fastest grouped form: no cross-wave
// reduction, a row's lanes add up on the DPP network, and a wave's critical path after its
// weights arrive is one batch of dot products.  Launches of one kernel per projection are what
// it replaces (src/bonsai_sft/gpu/model.py:977-1062).
constexpr int kDot4GroupMax = 12;

struct Dot4GroupDesc {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int M, N, K;
    int wg_begin;         // first workgroup of this GEMV
    int lpr_log2_passes;  // lpr_log2 | passes << 8
    uint32_t div_magic;
};
static_assert(sizeof(Dot4GroupDesc) == 64, "one descriptor is one 64-byte scalar load");

struct Dot4GroupTable {
    Dot4GroupDesc d[kDot4GroupMax];
};

template <int BITS, int MT, int U, bool SF16, bool G32 = false>
__global__ void __launch_bounds__(kMaxThreads)
gemv_dot4_grouped_kernel(int e0, int e1, int e2, int e3, int e4, int e5, int e6, int e7, int e8,
                         int e9, int e10, int e11, int pout_f32, int pthreads,
                         const Dot4GroupTable tbl) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int wg = (int)blockIdx.x;
    // (wg >= e) as the sign bit of e - 1 - wg: stays in scalar registers
    const auto ge = [wg](int e) { return (int)((uint32_t)(e - 1 - wg) >> 31); };
    const int di = ge(e0) + ge(e1) + ge(e2) + ge(e3) + ge(e4) + ge(e5) + ge(e6) + ge(e7) + ge(e8) +
                   ge(e9) + ge(e10) + ge(e11);
    const Dot4GroupDesc d = tbl.d[di];
    const GemvArgs a{d.A, d.B, d.out, d.s, d.ws, d.M, d.N, d.K, d.lpr_log2_passes & 0xff,
                     d.lpr_log2_passes >> 8, pout_f32, d.div_magic};
    gemv_dot4_body<BITS, MT, U, G32, SF16>(a, wg - d.wg_begin, 0, pthreads, smem);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
struct Tuning {
    int lanes_per_row = 0;
    int waves_per_wg = 0;
    int passes = 0;
};

using KernelFn = void (*)(const int8_t *, const uint8_t *, void *, const float *, const uint16_t *,
                          int, int, int, int, int, int, uint32_t, int);
constexpr int kBatchKinds = 3;  // U = 1, 2, 4
constexpr int kVariants = 3;    // 0: bf16 scales, 1: fp16 scales, 2: int32 group sums

template <int BITS>
struct KernelTable {
    KernelFn fn[kMaxTile][kBatchKinds][kVariants];
};

template <int BITS, int MT, int U, int UI>
void fill_table_cell(KernelTable<BITS> &t) {
    t.fn[MT - 1][UI][0] = gemv_dot4_kernel<BITS, MT, U, false, false>;
    t.fn[MT - 1][UI][1] = gemv_dot4_kernel<BITS, MT, U, false, true>;
    t.fn[MT - 1][UI][2] = gemv_dot4_kernel<BITS, MT, U, true, false>;
}

// Register use grows with MT*U (the compiler keeps a whole batch unpacked), so
// wide token tiles get shorter batches: U <= 4 for one token, U <= 2 for MT <= 4,
// U = 1 above (two tokens with four loads per batch need 172 VGPRs: two waves per SIMD,
// 21 us instead of 12 us on an 8B-shaped layer launch).  Cells that are not instantiated stay
// null.
constexpr int max_batch_index(int mt) { return mt <= 1 ? 2 : (mt <= 4 ? 1 : 0); }

template <int BITS, int MT>
void fill_table_row(KernelTable<BITS> &t) {
    fill_table_cell<BITS, MT, 1, 0>(t);
    if constexpr (max_batch_index(MT) >= 1) fill_table_cell<BITS, MT, 2, 1>(t);
    if constexpr (max_batch_index(MT) >= 2) fill_table_cell<BITS, MT, 4, 2>(t);
}

template <int BITS>
const KernelTable<BITS> &kernel_table() {
    static const KernelTable<BITS> table = [] {
        KernelTable<BITS> t{};
        fill_table_row<BITS, 1>(t);
        fill_table_row<BITS, 2>(t);
        fill_table_row<BITS, 3>(t);
        fill_table_row<BITS, 4>(t);
        fill_table_row<BITS, 5>(t);
        fill_table_row<BITS, 6>(t);
        fill_table_row<BITS, 7>(t);
        fill_table_row<BITS, 8>(t);
        return t;
    }();
    return table;
}

constexpr int kMaxDevices = 16;

template <int BITS>
struct LibState {
    Tuning tuning;
    int lds_limit[kMaxDevices] = {};  // 0 = device not initialised yet
    std::atomic<bool> mfma_ready[kMaxDevices] = {};  // set last, under init_mutex
    std::mutex init_mutex;
    int n_cus[kMaxDevices] = {};
};

template <int BITS>
LibState<BITS> &lib_state() {
    static LibState<BITS> st;
    return st;
}

template <int BITS>
int init_fused_kernels(int max_lds);

// Raises the dynamic-LDS limit of every kernel instantiation on the current
// device to what the device offers (160 KB per workgroup on gfx950).
template <int BITS>
int init_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 2;
    LibState<BITS> &st = lib_state<BITS>();
    if (st.lds_limit[dev] != 0) return 0;
    int max_lds = 0;
    if (hipDeviceGetAttribute(&max_lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) !=
            hipSuccess || max_lds <= 0)
        return 2;
    const KernelTable<BITS> &t = kernel_table<BITS>();
    for (int mt = 0; mt < kMaxTile; ++mt)
        for (int u = 0; u < kBatchKinds; ++u)
            for (int k = 0; k < kVariants; ++k)
                if (t.fn[mt][u][k] != nullptr &&
                    hipFuncSetAttribute(reinterpret_cast<const void *>(t.fn[mt][u][k]),
                                        hipFuncAttributeMaxDynamicSharedMemorySize,
                                        max_lds) != hipSuccess)
                    return 2;
    if (init_fused_kernels<BITS>(max_lds) != 0) return 2;
    st.lds_limit[dev] = max_lds;
    return 0;
}

struct Geometry {
    int lpr_log2, waves, passes, mt, ntiles, grid_x, batch_index;
    size_t lds;
};

inline int ilog2(int v) {
    int l = 0;
    while ((1 << (l + 1)) <= v) ++l;
    return l;
}

template <int BITS>
size_t lds_bytes(int mt, int C) {
    static const int words[kMaxTile] = {
        block_words<BITS, 1>(), block_words<BITS, 2>(), block_words<BITS, 3>(),
        block_words<BITS, 4>(), block_words<BITS, 5>(), block_words<BITS, 6>(),
        block_words<BITS, 7>(), block_words<BITS, 8>()};
    return (size_t)C * words[mt - 1] * 16;
}

// Picks lanes-per-row, workgroup size and passes for a shape.  The aim is to
// have every lane issue a few 16-byte loads at once and enough waves (a few per
// SIMD over 256 CUs) for the launch to cover the chip, without leaving more
// than about a quarter of the lanes past the end of short rows.  The constants
// come from sweeps over the decode shapes of the 1.7B- and 4B-shaped models.
template <int BITS>
Geometry pick_geometry(int M, int N, int K, int lds_limit, const Tuning &tu) {
    using F = Fmt<BITS>;
    Geometry g{};
    const int C = K / F::kChunkWeights;
    // largest token tile whose staged blocks fit in LDS
    int mt_cap = kMaxTile;
    while (mt_cap >= 1 && lds_bytes<BITS>(mt_cap, C) > (size_t)lds_limit) --mt_cap;
    if (mt_cap < 1) {
        g.mt = 0;
        return g;
    }
    g.ntiles = (M + mt_cap - 1) / mt_cap;
    g.mt = (M + g.ntiles - 1) / g.ntiles;
    g.lds = lds_bytes<BITS>(g.mt, C);

    int lpr = tu.lanes_per_row;
    if (lpr == 0) {
        const int min_lpr = BITS == 1 ? 4 : 8;
        int best = 0;
        for (int cand = min_lpr; cand <= 64; cand *= 2) {
            const int it = (C + cand - 1) / cand;
            // idle lanes: up to 27 % of a row's slots; a whole wave per row (two extra
            // cross-lane steps in the row reduction) only where that leaves each lane
            // exactly two loads, then up to 34 %
            const bool low_waste = cand < 64 ? (long)it * cand * 100 <= (long)C * 127
                                             : (it == 2 && (long)it * cand * 100 <= (long)C * 134);
            if (!low_waste && best != 0) continue;
            best = cand;
            const long waves = ((long)N * cand + 63) / 64;
            if (low_waste && waves >= 2048) break;
        }
        lpr = best;
        // 1-bit chunks carry 128 weights each, a long serial chain per lane: while the launch
        // is short of waves anyway, more lanes per row (up to 32) until a lane has at most
        // two chunks, idle lanes or not
        if (BITS == 1 && ((long)N * lpr + 63) / 64 < 2048)
            while (lpr < 32 && (C + lpr - 1) / lpr > 2) lpr *= 2;
    }
    g.lpr_log2 = ilog2(lpr);
    // loads per batch: the largest of 4, 2, 1 that wastes no load slot, 4 for long rows
    const int it = (C + lpr - 1) / lpr;
    // (one token of 2-bit weights: two at a time also for odd counts, the spare slot re-reads
    // the last chunk)
    const bool pair_odd = BITS == 2 && g.mt == 1 && it >= 3;
    g.batch_index = (it % 4 == 0 || it >= 8) ? 2 : ((it % 2 == 0 || pair_odd) ? 1 : 0);
    if (g.batch_index > max_batch_index(g.mt)) g.batch_index = max_batch_index(g.mt);
    const int rpw = 64 >> g.lpr_log2;
    const long wave_passes = ((long)N + rpw - 1) / rpw;

    // eight waves share one staging of the token tile where the rows are few, as long as
    // that leaves at least 128 workgroups
    g.waves = tu.waves_per_wg ? tu.waves_per_wg
                              : ((N <= 6144 && wave_passes >= 8 * 128) ? 8 : 4);
    if (g.waves * 64 > kMaxThreads) g.waves = kMaxThreads / 64;
    g.passes = tu.passes;
    if (g.passes == 0) {
        g.passes = (int)((wave_passes + 8191) / 8192);
        if (g.passes > 16) g.passes = 16;
    }
    if (g.passes < 1) g.passes = 1;
    const long rows_per_wg = (long)rpw * g.waves * g.passes;
    g.grid_x = (int)(((long)N + rows_per_wg - 1) / rows_per_wg);
    return g;
}

// Launches the dot4 kernel for a validated shape on an initialised device.
template <int BITS>
int launch_gemv_dot4(const int8_t *A, const uint8_t *B, void *out, const float *s, const void *ws,
                     int M, int N, int K, int out_kind, int scale_kind, int lds_limit,
                     hipStream_t stream) {
    const Geometry g = pick_geometry<BITS>(M, N, K, lds_limit, lib_state<BITS>().tuning);
    if (g.mt == 0) return 1;  // one token of K activations does not fit in LDS

    GemvArgs args;
    args.A = A;
    args.B = B;
    args.out = out;
    args.s = s;
    args.ws = reinterpret_cast<const uint16_t *>(ws);
    args.M = M;
    args.N = N;
    args.K = K;
    args.lpr_log2 = g.lpr_log2;
    args.passes = g.passes;
    args.out_f32 = out_kind == OUT_F32 ? 1 : 0;
    args.div_magic = (uint32_t)(0x100000000ull / (uint64_t)(4 * (K / Fmt<BITS>::kChunkWeights))) + 1u;

    const int variant = out_kind == OUT_G32 ? 2 : scale_kind;
    const KernelFn fn = kernel_table<BITS>().fn[g.mt - 1][g.batch_index][variant];
    hipLaunchKernelGGL(fn, dim3(g.grid_x, g.ntiles, 1), dim3(g.waves * 64, 1, 1), g.lds, stream,
                       args.A, args.B, args.out, args.s, args.ws, args.M, args.N, args.K,
                       args.lpr_log2, args.passes, args.out_f32, args.div_magic, g.waves * 64);
    note_kernel("gemv_dot4_kernel", BITS, g.mt, 1 << g.batch_index, scale_kind == 1 && out_kind != OUT_G32, out_kind == OUT_G32);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

// ---- fused forms: table, set-up, launch ------------------------------------------------
using FusedKernelFn = void (*)(const int8_t *, const uint8_t *, void *, const uint16_t *, const void *,
                               const uint16_t *, int, int, int, int, float, void *, const uint16_t *, int,
                               float *);
constexpr int kFusedMaxTile = 2;

// One fused GEMV (host side; the C structure of the entry point carries the same fields).
struct FusedGemv {
    int pro, epi;
    const void *act;      // int8 [M, K] (PRO_INT8) or bf16 [M, K]
    const void *act_aux;  // PRO_INT8: fp32 s[M]; PRO_BF16_AMAX: bf16 maxima; PRO_BF16_NORM: fp64 sums
    int act_parts;        // parts per token in act_aux
    const uint16_t *norm_w;
    float eps;
    const uint8_t *B;
    const void *ws;
    void *out;            // EPI_PLAIN: bf16 / fp32 [M, N]; EPI_SILU_PAIR: bf16 [M, N/2]; EPI_ADD_SUMSQ: bf16 [M, N]
    const uint16_t *residual;
    void *out_aux;        // EPI_SILU_PAIR: bf16 maxima [M, amax_ld(parts)]; EPI_ADD_SUMSQ: fp64 sums [M, parts]
    float *s_out;
    int M, N, K, out_kind;
};

template <int BITS>
struct FusedKernelTable {
    FusedKernelFn fn[3][3][kFusedMaxTile][kBatchKinds];  // [prologue][epilogue][MT - 1][batch index]
};

template <int BITS, int PRO, int EPI>
void fill_fused_cells(FusedKernelTable<BITS> &t) {
    constexpr int F = fuse_code(PRO, EPI);
    t.fn[PRO][EPI][0][0] = gemv_dot4_fused_kernel<BITS, 1, 1, F>;
    t.fn[PRO][EPI][0][1] = gemv_dot4_fused_kernel<BITS, 1, 2, F>;
    t.fn[PRO][EPI][0][2] = gemv_dot4_fused_kernel<BITS, 1, 4, F>;
    t.fn[PRO][EPI][1][0] = gemv_dot4_fused_kernel<BITS, 2, 1, F>;
    t.fn[PRO][EPI][1][1] = gemv_dot4_fused_kernel<BITS, 2, 2, F>;
}

// The combinations a decode layer uses (q|k|v: norm in; o: residual out; gate|up: norm in, SiLU
// pair out; down: maxima in, residual out) and the two of the MLP tail on its own.
template <int BITS>
const FusedKernelTable<BITS> &fused_kernel_table() {
    static const FusedKernelTable<BITS> table = [] {
        FusedKernelTable<BITS> t{};
        fill_fused_cells<BITS, PRO_INT8, EPI_SILU_PAIR>(t);
        fill_fused_cells<BITS, PRO_INT8, EPI_ADD_SUMSQ>(t);
        fill_fused_cells<BITS, PRO_BF16_AMAX, EPI_PLAIN>(t);
        fill_fused_cells<BITS, PRO_BF16_AMAX, EPI_ADD_SUMSQ>(t);
        fill_fused_cells<BITS, PRO_BF16_NORM, EPI_PLAIN>(t);
        fill_fused_cells<BITS, PRO_BF16_NORM, EPI_SILU_PAIR>(t);
        return t;
    }();
    return table;
}

template <int BITS>
int init_fused_kernels(int max_lds) {
    const FusedKernelTable<BITS> &t = fused_kernel_table<BITS>();
    for (int p = 0; p < 3; ++p)
        for (int e = 0; e < 3; ++e)
            for (int mt = 0; mt < kFusedMaxTile; ++mt)
                for (int u = 0; u < kBatchKinds; ++u)
                    if (t.fn[p][e][mt][u] != nullptr &&
                        hipFuncSetAttribute(reinterpret_cast<const void *>(t.fn[p][e][mt][u]),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, max_lds) != hipSuccess)
                        return 2;
    return 0;
}

// Geometry of a fused form; mt == 0 when the shape is not taken.  The number of parts a launch
// writes depends on its epilogue alone (`pro` only matters for launches that write none).
// A norm prologue is work every workgroup repeats for the whole row (normalise, maximum,
// quantise: about as many vector instructions as the workgroup's share of the projection), so
// such a launch wants few, fat workgroups: eight waves and at most one workgroup per CU -- the
// fewest lanes per row that get there, then more row passes.  Measured at one token: gate|up
// 12288 x 2048 with norm in and SiLU out 5.86 us on the plain launch's geometry (768 workgroups of
// four waves), 4.88 us on 192 of eight; 19456 x 2560 7.95 -> 7.25 us (152 workgroups, two passes);
// q|k|v already has 256 / 192 workgroups of eight waves.  The SiLU-pair epilogue takes the same
// geometry whatever it reads, so that its parts count depends on the shape only.
template <int BITS>
Geometry fused_geometry(int pro, int epi, int M, int N, int K, int lds_limit, int n_cus) {
    const int lds_left = lds_limit - kFusedMeetBytes;
    Tuning base = lib_state<BITS>().tuning;
    if ((pro == PRO_BF16_NORM || epi == EPI_SILU_PAIR) && base.lanes_per_row == 0 &&
        base.waves_per_wg == 0 && base.passes == 0) {
        const int cus = n_cus > 0 ? n_cus : 256;
        const int min_lpr = BITS == 1 ? 4 : 8;
        const int C = K / Fmt<BITS>::kChunkWeights;
        int lpr = 32;
        while (lpr > min_lpr && lpr / 2 >= C) lpr /= 2;  // no more lanes than a row has chunks
        const int waves = kMaxThreads / 64;
        auto grid_for = [&](int l) { return (N + waves * (64 / l) - 1) / (waves * (64 / l)); };
        while (lpr > min_lpr && grid_for(lpr) > cus) lpr /= 2;
        base.lanes_per_row = lpr;
        base.waves_per_wg = waves;
        base.passes = (grid_for(lpr) + cus - 1) / cus;
    }
    Geometry g = pick_geometry<BITS>(M, N, K, lds_left, base);
    if (g.mt != 0 && epi == EPI_SILU_PAIR && g.lpr_log2 > 5) {
        // the halves of a column meet in neighbouring lane sets of one wave: at most 32 lanes a row
        Tuning tu = base;
        tu.lanes_per_row = 32;
        g = pick_geometry<BITS>(M, N, K, lds_left, tu);
    }
    const int max_parts = epi == EPI_SILU_PAIR ? kAmaxMaxParts : (epi == EPI_ADD_SUMSQ ? kSumsqMaxParts : 1 << 30);
    if (g.mt != 0 && g.grid_x > max_parts) {
        // few enough workgroups for the consumer's waves to read every part with a few loads
        Tuning tu = base;
        tu.lanes_per_row = 1 << g.lpr_log2;
        tu.waves_per_wg = kMaxThreads / 64;
        const long rows_per_pass = (long)(64 >> g.lpr_log2) * tu.waves_per_wg;
        tu.passes = (int)((((long)N + rows_per_pass - 1) / rows_per_pass + max_parts - 1) / max_parts);
        g = pick_geometry<BITS>(M, N, K, lds_left, tu);
    }
    if (g.mt > kFusedMaxTile || g.ntiles != 1 || g.grid_x > max_parts || g.passes > 31) g.mt = 0;
    g.lds += kFusedMeetBytes;
    return g;
}

// Launches a fused form for validated operands (M <= 2) on an initialised device.
template <int BITS>
int launch_gemv_dot4_fused(const FusedGemv &d, int lds_limit, int n_cus, hipStream_t stream) {
    const Geometry g = fused_geometry<BITS>(d.pro, d.epi, d.M, d.N, d.K, lds_limit, n_cus);
    if (g.mt == 0) return 1;
    const FusedKernelFn fn = fused_kernel_table<BITS>().fn[d.pro][d.epi][g.mt - 1][g.batch_index];
    if (fn == nullptr) return 1;
    const int geom = g.lpr_log2 | (g.passes << 4) | ((d.out_kind == OUT_F32 ? 1 : 0) << 9) | (g.waves << 10) |
                     (d.act_parts << 14);
    hipLaunchKernelGGL(fn, dim3(g.grid_x, 1, 1), dim3(g.waves * 64, 1, 1), g.lds, stream,
                       reinterpret_cast<const int8_t *>(d.act), d.B, d.out,
                       reinterpret_cast<const uint16_t *>(d.ws), d.act_aux, d.norm_w, d.M, d.N, d.K, geom,
                       d.eps, d.out_aux, d.residual, g.grid_x, d.s_out);
    note_kernel("gemv_dot4_fused_kernel", BITS, g.mt, 1 << g.batch_index, fuse_code(d.pro, d.epi));
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // namespace bonsai
#endif  // BONSAI_PACKED_GEMV_HIP_H
