// Single-token streaming kernel of the T2 GEMV for matrices with very many rows (the 151936-row
// output projection of an autoregressive step, src/bonsai_sft/gpu/model.py:1058-1062 applied to
// the packed lm_head; one launch of t2g128_kernels.cu:94-100 in the reference).
//
// An 83 MB matrix streams at HBM speed only if the arithmetic per byte is small and nothing but
// the weights moves: on this part a pure read of that size takes 13.9 us, and every VALU
// instruction per KB of weights that does not overlap costs the launch about 0.13 us.  So
//   * a lane owns ONE 128-wide scale group of K for the whole launch (K = 128 x lanes per row)
//     and keeps its 128 activations in registers: no LDS traffic in the loop (the dot4 kernel
//     reads 64 activation bytes from LDS per 16 weight bytes);
//   * the activations are held as 4-bit planes, a = 16 hi + lo with hi signed and lo unsigned,
//     and the packed codes are masked to nibbles, c_even = p & 0x33333333, c_odd = (p >> 2) &
//     0x33333333: three operations per packed dword instead of seven for the byte vectors of
//     v_dot4, and 16 weights meet their activations in four v_dot8 (two signed for the hi plane,
//     two unsigned for the lo plane): 28 operations per 16-byte chunk against 44;
//   * the two chunks of a group are summed as integers, G = 16 H + L - 2 sum(a) (the offset of
//     the codes goes in as the initial value of L), so there is one conversion and one multiply
//     by the group scale per row and lane;
//   * workgroups are persistent; a wave has two batches of two row sets (four 16-byte loads per
//     lane and batch) in flight; all addresses are a per-lane offset plus a scalar, through
//     buffer resources whose range check makes rows past the matrix read as zero.
// The 4-bit planes are built once per workgroup (bytes -> planes through LDS).  Integer group
// sums are exact; fp32: the lanes of a row are added in tree order on the DPP network.
#ifndef BONSAI_GEMV_ROWREG_HIP_H
#define BONSAI_GEMV_ROWREG_HIP_H

#include "gemv_mx.hip.h"

namespace bonsai {

constexpr int kRowregThreads = 256;
constexpr int kRowregU = 2;  // row sets per batch

struct RowregParams {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int N, K;
    int out_f32;
};

constexpr int kRowregBufferWord3 = 0x00020000;  // raw buffer, 32-bit format, range check on

// G32: store the exact int32 group sums G[0][n][g] instead of the scaled result.
template <int LPR_LOG2, bool SF16, bool G32 = false>
__global__ void __launch_bounds__(kRowregThreads) __attribute__((amdgpu_waves_per_eu(4)))
gemv_rowreg_kernel(const RowregParams p) {
    constexpr int LPR = 1 << LPR_LOG2;   // lanes per row = scale groups per row
    constexpr int RPW = 64 / LPR;        // rows per row set (one pair of loads of a wave)
    constexpr int BR = RPW * kRowregU;   // rows per batch
    constexpr int K = LPR * 128;
    constexpr int G = LPR;
    constexpr int row_bytes = K / 4;
    __shared__ __align__(16) u32x4 planes[K / 16];  // one unit per 16 activations
    __shared__ int qsum[K / 16];                    // their sums

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane >> LPR_LOG2, lc = lane & (LPR - 1);
    const int N = p.N;

    const __amdgpu_buffer_rsrc_t rB = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(p.B), 0, N * row_bytes, kRowregBufferWord3);
    const __amdgpu_buffer_rsrc_t rS = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.ws), 0, G32 ? 0 : N * G * 2, kRowregBufferWord3);

    struct Batch {
        u32x4 w[kRowregU][2];
        uint16_t sc[kRowregU];
    };
    const uint32_t voff = (uint32_t)lr * row_bytes + (uint32_t)lc * 32u;
    const uint32_t vsoff = ((uint32_t)lr * G + (uint32_t)lc) * 2u;
    typedef unsigned int v4u __attribute__((ext_vector_type(4)));
    auto load = [&](Batch &t, int b) {
        // the batch offset travels in the vector offset: that is what the range check sees
        const uint32_t vb = voff + (uint32_t)b * (uint32_t)(BR * row_bytes);
        const uint32_t vs = vsoff + (uint32_t)b * (uint32_t)(BR * G * 2);
#pragma unroll
        for (int u = 0; u < kRowregU; ++u) {
            const v4u x0 = __builtin_amdgcn_raw_buffer_load_b128(rB, (int)(vb + u * RPW * row_bytes), 0, 0);
            const v4u x1 = __builtin_amdgcn_raw_buffer_load_b128(rB, (int)(vb + u * RPW * row_bytes + 16), 0, 0);
            t.w[u][0] = u32x4{x0.x, x0.y, x0.z, x0.w};
            t.w[u][1] = u32x4{x1.x, x1.y, x1.z, x1.w};
            t.sc[u] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rS, (int)(vs + u * RPW * G * 2), 0, 0);
        }
    };

    // ---- the first batches go out, then the activations are brought into plane form
    const int n_batch = (N + BR - 1) / BR;
    const int stride = (int)gridDim.x * (kRowregThreads / 64);
    int b = (int)blockIdx.x * (kRowregThreads / 64) + wave;
    Batch x, y;
    load(x, b);
    if (tid < K / 16) {
        const u32x4 in = reinterpret_cast<const u32x4 *>(p.A)[tid];
        planes[tid] = nibble_planes16(in);
        qsum[tid] = sum4_i8(in.x) + sum4_i8(in.y) + sum4_i8(in.z) + sum4_i8(in.w);
    }
    const float rinv = G32 ? 1.0f : __builtin_amdgcn_rcpf(p.s[0]);
    __syncthreads();
    uint32_t act[2][16];
    int asum = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const u32x4 v = planes[lc * 8 + q];
        act[q >> 2][4 * (q & 3)] = v.x;
        act[q >> 2][4 * (q & 3) + 1] = v.y;
        act[q >> 2][4 * (q & 3) + 2] = v.z;
        act[q >> 2][4 * (q & 3) + 3] = v.w;
        asum += qsum[lc * 8 + q];
    }
    const uint32_t l_init = (uint32_t)(-2 * asum);

    auto compute = [&](const Batch &t, int bb) {
        float res[kRowregU];
#pragma unroll
        for (int u = 0; u < kRowregU; ++u) {
            int ah = 0;
            uint32_t al = l_init;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint32_t pw[4] = {t.w[u][i].x, t.w[u][i].y, t.w[u][i].z, t.w[u][i].w};
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t e = pw[d] & 0x33333333u, o = (pw[d] >> 2) & 0x33333333u;
                    ah = __builtin_amdgcn_sdot8((int)act[i][4 * d], (int)e, ah, false);
                    al = __builtin_amdgcn_udot8(act[i][4 * d + 1], e, al, false);
                    ah = __builtin_amdgcn_sdot8((int)act[i][4 * d + 2], (int)o, ah, false);
                    al = __builtin_amdgcn_udot8(act[i][4 * d + 3], o, al, false);
                }
            }
            const int g = (ah << 4) + (int)al;  // the exact group sum
            if (G32) {
                const int row = bb * BR + u * RPW + lr;
                if (row < N) reinterpret_cast<int32_t *>(p.out)[(size_t)row * G + lc] = g;
                res[u] = 0.0f;
                continue;
            }
            res[u] = row_lanes_sum((float)g * scale_to_f32<SF16>(t.sc[u]), LPR_LOG2);
        }
#pragma unroll
        for (int u = 0; u < kRowregU; ++u) {
            const int row = bb * BR + u * RPW + lr;
            if (!G32 && lc == 0 && row < N) {
                const float yv = res[u] * rinv;
                if (p.out_f32)
                    reinterpret_cast<float *>(p.out)[row] = yv;
                else
                    reinterpret_cast<uint16_t *>(p.out)[row] = f32_to_bf16_rne_nobranch(yv);
            }
        }
    };

    // two register buffers alternate; a batch past the end reads zeros and is not computed
    while (b < n_batch) {
        load(y, b + stride);
        compute(x, b);
        b += stride;
        if (b >= n_batch) break;
        load(x, b + stride);
        compute(y, b);
        b += stride;
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
using RowregKernelFn = void (*)(const RowregParams);

inline RowregKernelFn rowreg_kernel(int K, int scale_kind) {
    const bool f16 = scale_kind == 1;
    if (scale_kind == 2) {  // int32 group sums
        switch (K) {
        case 1024: return gemv_rowreg_kernel<3, false, true>;
        case 2048: return gemv_rowreg_kernel<4, false, true>;
        case 4096: return gemv_rowreg_kernel<5, false, true>;
        default: return nullptr;
        }
    }
    switch (K) {
    case 1024: return f16 ? gemv_rowreg_kernel<3, true> : gemv_rowreg_kernel<3, false>;
    case 2048: return f16 ? gemv_rowreg_kernel<4, true> : gemv_rowreg_kernel<4, false>;
    case 4096: return f16 ? gemv_rowreg_kernel<5, true> : gemv_rowreg_kernel<5, false>;
    default: return nullptr;
    }
}

// True when the kernel takes the problem: one token, T2, K = 1024, 2048 or 4096 (128 x a power
// of two lanes per row), operands aligned and within the 32-bit buffer range, and (unless
// `forced`) a matrix long enough for persistent workgroups to pay.
inline bool rowreg_problem_ok(const GemvProblem &q, int out_kind, bool forced) {
    const auto al = [](const void *ptr, uintptr_t a) {
        return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) == 0;
    };
    (void)out_kind;  // every output kind, the int32 group sums included
    if (q.M != 1 || rowreg_kernel(q.K, 0) == nullptr) return false;
    if (!al(q.A, 16) || !al(q.B, 16) || !al(q.ws, 2)) return false;
    if ((long)q.N * (q.K / 4) >= (1L << 31)) return false;
    return forced || (long)q.N * (q.K / 4) >= (32L << 20);
}

inline int launch_rowreg(const GemvProblem &q, int out_kind, int scale_kind, int n_cus, int wgs_per_cu,
                         hipStream_t stream) {
    RowregParams prm{};
    prm.A = q.A;
    prm.B = q.B;
    prm.out = q.out;
    prm.s = q.s;
    prm.ws = reinterpret_cast<const uint16_t *>(q.ws);
    prm.N = q.N;
    prm.K = q.K;
    prm.out_f32 = out_kind == OUT_F32 ? 1 : 0;
    const int lpr = q.K / 128;
    const int rows_per_batch = (64 / lpr) * kRowregU;
    const int n_batch = (q.N + rows_per_batch - 1) / rows_per_batch;
    int wgs = n_cus * (wgs_per_cu > 0 ? wgs_per_cu : 4);
    const int need = (n_batch + 3) / 4;
    if (wgs > need) wgs = need;
    const int variant = out_kind == OUT_G32 ? 2 : scale_kind;
    hipLaunchKernelGGL(rowreg_kernel(q.K, variant), dim3(wgs, 1, 1), dim3(kRowregThreads, 1, 1), 0,
                       stream, prm);
    note_kernel("gemv_rowreg_kernel", 2, lpr == 8 ? 3 : (lpr == 16 ? 4 : 5), variant == 1, variant == 2);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_ROWREG_HIP_H
