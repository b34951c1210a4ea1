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
#include <stdint.h>
#include <stdio.h>

#include "gemv_core.h"

namespace bonsai {

constexpr int kGroup = 128;
constexpr int kMaxTile = 8;      // tokens per tile (template MT is 1..kMaxTile)
constexpr int kBatch = 4;        // 16-byte weight loads in flight per lane and batch
constexpr int kMaxThreads = 512; // workgroup size limit of the kernels

enum : int { OUT_BF16 = 0, OUT_F32 = 1, OUT_G32 = 2 };

struct GemvArgs {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int M, N, K;
    int lpr_log2;  // log2(lanes per weight row)
    int passes;    // row passes per wave
};

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

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8 lanes
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each 16 lanes

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

struct WeightBatch {
    u32x4 w[kBatch];
    float sc[kBatch];  // group scale, 0 for lanes past the end of the row
};

template <int BITS, int MT, int OUT, bool SF16>
__global__ void __launch_bounds__(kMaxThreads) gemv_dot4_kernel(const GemvArgs a) {
    using F = Fmt<BITS>;
    extern __shared__ __align__(16) unsigned char smem[];

    const int K = a.K, N = a.N, M = a.M;
    const int C = K / F::kChunkWeights;  // 16-byte chunks per weight row
    const int ng = K / kGroup;
    const size_t row_bytes = (size_t)C * 16;

    u32x4 *act = reinterpret_cast<u32x4 *>(smem);                 // [MT][kUnits][C]
    int *asum = reinterpret_cast<int *>(smem + (size_t)MT * K);   // [MT][C]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int nwaves = blockDim.x >> 6;
    const int lpr_log2 = a.lpr_log2;
    const int lpr = 1 << lpr_log2;
    const int c = lane & (lpr - 1);        // position of the lane along K
    const int r = lane >> lpr_log2;        // row of the lane inside the wave
    const int rpw = 64 >> lpr_log2;        // rows per wave and pass
    const int IT = (C + lpr - 1) >> lpr_log2;
    const int nb = (IT + kBatch - 1) / kBatch;
    const int m0 = blockIdx.y * MT;

    auto row_of = [&](int pass) {
        return (((int)blockIdx.x * a.passes + pass) * nwaves + wave) * rpw + r;
    };

    auto load_batch = [&](WeightBatch &wb, int row, int it0) {
        const int row_c = row < N ? row : N - 1;
        const u32x4 *wrow = reinterpret_cast<const u32x4 *>(a.B + (size_t)row_c * row_bytes);
        const uint16_t *srow = a.ws + (size_t)row_c * ng;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (it0 + u >= IT) break;  // wave-uniform: the row has no such chunk column
            const int chunk = (it0 + u) * lpr + c;
            const int chunk_c = chunk < C ? chunk : C - 1;
            wb.w[u] = wrow[chunk_c];
            if (OUT != OUT_G32) {
                const float f = scale_to_f32<SF16>(srow[chunk_c >> F::kGroupShift]);
                wb.sc[u] = (chunk < C && row < N) ? f : 0.0f;
            }
        }
    };

    // Weight loads for the first batch go out before the activations are
    // staged, so that their HBM latency overlaps the staging.
    WeightBatch cur, nxt;
    load_batch(cur, row_of(0), 0);

    for (int task = tid; task < MT * C; task += blockDim.x) {
        const int m = task / C;
        const int chunk = task - m * C;
        const int msrc = (m0 + m) < M ? (m0 + m) : M - 1;
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.A + (size_t)msrc * K) +
                           (size_t)chunk * F::kUnits;
        asum[m * C + chunk] = stage_chunk<BITS>(src, act, m, chunk, C);
    }
    __syncthreads();

    float accf[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) accf[m] = 0.0f;

    const int total = a.passes * nb;
    int pass = 0, b = 0;
    for (int i = 0; i < total; ++i) {
        int npass = pass, nbt = b + 1;
        if (nbt == nb) {
            nbt = 0;
            npass = pass + 1;
        }
        const bool more = i + 1 < total;
        if (more) load_batch(nxt, row_of(npass), nbt * kBatch);

        const int row = row_of(pass);
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (b * kBatch + u >= IT) break;  // wave-uniform
            const int chunk = (b * kBatch + u) * lpr + c;
            const int chunk_c = chunk < C ? chunk : C - 1;
            int raw[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) raw[m] = 0;
            chunk_dot_raw<BITS, MT>(cur.w[u], act, chunk_c, C, raw);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                int g = chunk_dot_signed<BITS>(raw[m], asum[m * C + chunk_c]);
                if (OUT == OUT_G32) {
                    // T2: two neighbouring lanes hold the halves of one group.
                    if (BITS == 2) g += dpp_i32<kDppXor1>(g);
                    const bool writer = (BITS == 2) ? ((c & 1) == 0) : true;
                    if (writer && chunk < C && row < N && (m0 + m) < M) {
                        int32_t *G = reinterpret_cast<int32_t *>(a.out);
                        G[((size_t)(m0 + m) * N + row) * ng + (chunk >> F::kGroupShift)] = g;
                    }
                } else {
                    accf[m] += (float)g * cur.sc[u];
                }
            }
        }

        if (b == nb - 1 && OUT != OUT_G32) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const float sum = row_lanes_sum(accf[m], lpr_log2);
                accf[m] = 0.0f;
                if (c == 0 && row < N && (m0 + m) < M) {
                    const float y = sum / a.s[m0 + m];
                    if (OUT == OUT_F32)
                        reinterpret_cast<float *>(a.out)[(size_t)(m0 + m) * N + row] = y;
                    else
                        reinterpret_cast<uint16_t *>(a.out)[(size_t)(m0 + m) * N + row] =
                            f32_to_bf16_rne(y);
                }
            }
        }
        if (more) cur = nxt;
        pass = npass;
        b = nbt;
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
struct Tuning {
    int lanes_per_row = 0;
    int waves_per_wg = 0;
    int passes = 0;
};

using KernelFn = void (*)(const GemvArgs);

template <int BITS>
struct KernelTable {
    // [MT-1][out_kind][scale_kind]
    KernelFn fn[kMaxTile][3][2];
};

template <int BITS, int MT>
void fill_table_row(KernelTable<BITS> &t) {
    t.fn[MT - 1][OUT_BF16][0] = gemv_dot4_kernel<BITS, MT, OUT_BF16, false>;
    t.fn[MT - 1][OUT_BF16][1] = gemv_dot4_kernel<BITS, MT, OUT_BF16, true>;
    t.fn[MT - 1][OUT_F32][0] = gemv_dot4_kernel<BITS, MT, OUT_F32, false>;
    t.fn[MT - 1][OUT_F32][1] = gemv_dot4_kernel<BITS, MT, OUT_F32, true>;
    // group sums do not read the scales: one instantiation serves both kinds
    t.fn[MT - 1][OUT_G32][0] = gemv_dot4_kernel<BITS, MT, OUT_G32, false>;
    t.fn[MT - 1][OUT_G32][1] = gemv_dot4_kernel<BITS, MT, OUT_G32, false>;
}

template <int BITS>
const KernelTable<BITS> &kernel_table() {
    static const KernelTable<BITS> table = [] {
        KernelTable<BITS> t;
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
};

template <int BITS>
LibState<BITS> &lib_state() {
    static LibState<BITS> st;
    return st;
}

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
        for (int o = 0; o < 3; ++o)
            for (int k = 0; k < 2; ++k)
                if (hipFuncSetAttribute(reinterpret_cast<const void *>(t.fn[mt][o][k]),
                                        hipFuncAttributeMaxDynamicSharedMemorySize,
                                        max_lds) != hipSuccess)
                    return 2;
    st.lds_limit[dev] = max_lds;
    return 0;
}

struct Geometry {
    int lpr_log2, waves, passes, mt, ntiles, grid_x;
    size_t lds;
};

inline int ilog2(int v) {
    int l = 0;
    while ((1 << (l + 1)) <= v) ++l;
    return l;
}

// Picks lanes-per-row, workgroup size and passes for a shape.  The aim is to
// have every lane issue a few 16-byte loads at once and enough waves (a few per
// SIMD over 256 CUs) for the launch to cover the chip, without leaving more
// than a quarter of the lanes past the end of short rows.
template <int BITS>
Geometry pick_geometry(int M, int N, int K, int lds_limit, const Tuning &tu) {
    using F = Fmt<BITS>;
    Geometry g{};
    const int C = K / F::kChunkWeights;
    const size_t per_token = (size_t)K + (size_t)C * 4;
    int mt_cap = (int)((size_t)lds_limit / per_token);
    if (mt_cap > kMaxTile) mt_cap = kMaxTile;
    if (mt_cap < 1) {
        g.mt = 0;
        return g;
    }
    g.ntiles = (M + mt_cap - 1) / mt_cap;
    g.mt = (M + g.ntiles - 1) / g.ntiles;
    g.lds = (size_t)g.mt * per_token;

    int lpr = tu.lanes_per_row;
    if (lpr == 0) {
        const int min_lpr = BITS == 1 ? 4 : 8;
        int best = 0;
        for (int cand = min_lpr; cand <= 64; cand *= 2) {
            const int it = (C + cand - 1) / cand;
            const bool low_waste = (long)it * cand * 4 <= (long)C * 5;  // <= 25 % idle lanes
            if (!low_waste && best != 0) continue;
            best = cand;
            const long waves = ((long)N * cand + 63) / 64;
            if (low_waste && waves >= 2048) break;
        }
        lpr = best;
    }
    g.lpr_log2 = ilog2(lpr);
    const int rpw = 64 >> g.lpr_log2;
    const long wave_passes = ((long)N + rpw - 1) / rpw;

    g.waves = tu.waves_per_wg ? tu.waves_per_wg : 4;
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

template <int BITS>
int launch_gemv(const int8_t *A, const uint8_t *B, void *out, const float *s, const void *ws,
                int M, int N, int K, int out_kind, int scale_kind, hipStream_t stream) {
    if (A == nullptr || B == nullptr || out == nullptr) return 1;
    if (out_kind < 0 || out_kind > 2 || scale_kind < 0 || scale_kind > 1) return 1;
    if (out_kind != OUT_G32 && (s == nullptr || ws == nullptr)) return 1;
    if (M < 1 || N < 1 || K < kGroup || K % kGroup != 0) return 1;
    if ((long)M * N > 0x7fffffffL / 2) return 1;  // row indices are 32-bit

    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 2;
    LibState<BITS> &st = lib_state<BITS>();
    if (st.lds_limit[dev] == 0) {
        const int rc = init_device<BITS>();
        if (rc != 0) return rc;
    }
    const Geometry g = pick_geometry<BITS>(M, N, K, st.lds_limit[dev], st.tuning);
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

    const KernelFn fn = kernel_table<BITS>().fn[g.mt - 1][out_kind][scale_kind];
    hipLaunchKernelGGL(fn, dim3(g.grid_x, g.ntiles, 1), dim3(g.waves * 64, 1, 1), g.lds, stream,
                       args);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // namespace bonsai
#endif  // BONSAI_PACKED_GEMV_HIP_H
