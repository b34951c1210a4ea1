// Streaming matrix-core kernel of the packed low-bit GEMV for matrices with very many rows (the
// 151936-row output projection, src/bonsai_sft/gpu/model.py:1058-1062 applied to the packed
// lm_head; in the reference one launch of t2g128_kernels.cu:94-100 like any other projection).
//
// Such a matrix (83 MB) is long enough to stream at HBM speed if enough bytes are in flight:
// at 8 TB/s and about 1.5 us of loaded memory latency that is 12 MB, 3 KB for each of the 4096
// waves a launch keeps resident.  The grouped kernel (gemv_mx.hip.h) has one 2 KB tile per wave in
// flight and a workgroup barrier per 16 rows; here
//   * a wave owns whole rows: 16 weight rows over all of K, so there is no cross-wave
//     reduction and no barrier after the set-up;
//   * a ring of four weight tiles (16 rows x 512 K) per wave is kept in flight: a ring slot is
//     refilled the moment its tile has been parked in LDS, with a statically known number of
//     loads behind it, so every wait is for exactly one tile;
//   * the activations of the whole block (up to 16 tokens x K) are staged once per workgroup
//     in operand order and stay in LDS; workgroups are persistent (grid = what is resident) and
//     walk the row tiles with the stride of the launch.
// Arithmetic, operand layouts and the parking of weight tiles are those of gemv_mx.hip.h.
#ifndef BONSAI_GEMV_MXS_HIP_H
#define BONSAI_GEMV_MXS_HIP_H

#include "gemv_mx.hip.h"

namespace bonsai {

constexpr int kMxsRing = 4;  // weight tiles in flight per wave

struct MxsParams {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int M, N, K;
    int out_f32;
};

// LDS bytes of one workgroup: the staged tokens of all K tiles, the per-(group, token) offset
// terms and one parked weight tile per wave.
template <int BITS>
__host__ __device__ constexpr size_t mxs_lds_bytes(int M, int K) {
    return (size_t)(K / kMxTileK) * M * kMxTokenUnits * 16 + (size_t)(K / kGroup) * 16 * 4 +
           (size_t)kMxWaves * mfma_wave_tile_bytes<BITS, 1>();
}

// MR: result columns kept per lane.  A lane's MFMA result holds tokens 4 (lane / 16) + r,
// r = 0..3; a single-token block needs only r = 0 (MR = 1), which saves three of the four
// convert / multiply-add pairs per group.
// G32: store the exact int32 group sums G[m][n][g] instead of the scaled result (scales and
// multipliers are not read).
template <int BITS, bool SF16, int MR, bool G32 = false>
__global__ void __launch_bounds__(kMxThreads) __attribute__((amdgpu_waves_per_eu(4)))
gemv_mxs_kernel(const MxsParams p) {
    using MF = MfmaFmt<BITS>;
    extern __shared__ __align__(16) unsigned char smem[];

    const int K = p.K, N = p.N, M = p.M;  // M <= 16 (M == 1 when MR == 1)
    const int G = K >> 7;
    const int KT = K >> 9;  // K % 512 == 0, K >= 2048
    const int row_bytes = K * BITS / 8;
    const uint8_t *const pB = p.B;
    const unsigned char *const pws = reinterpret_cast<const unsigned char *>(p.ws);
    const int8_t *const pA = p.A;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_rt = (N + 15) >> 4;
    const int wave_stride = (int)gridDim.x * kMxWaves;
    const int first_rt = (int)blockIdx.x * kMxWaves + wave;

    // LDS: [KT][M][33] staged units, [G][16] offset terms, one parked weight tile per wave
    u32x4 *act = reinterpret_cast<u32x4 *>(smem);
    const uint32_t tile_units = (uint32_t)M * kMxTokenUnits;
    int32_t *corr = reinterpret_cast<int32_t *>(smem + (size_t)KT * tile_units * 16);
    unsigned char *wt = reinterpret_cast<unsigned char *>(corr + G * 16) +
                        (uint32_t)wave * mfma_wave_tile_bytes<BITS, 1>();

    const int ld_row = lane / MF::kLanesPerRow;
    const int ld_col = lane % MF::kLanesPerRow;
    const int op_row = lane & 15;
    const int kb = lane >> 4;

    // Per-lane byte offsets inside a row tile, computed once: a load is base + scalar(row tile,
    // K tile) + one of these.  The second set is for the last row tile, whose rows past the matrix
    // alias row N - 1.
    const int last_n0 = (n_rt - 1) << 4;
    uint32_t voff_w[MF::kLoads], voff_w_last[MF::kLoads];
#pragma unroll
    for (int h = 0; h < MF::kLoads; ++h) {
        const int rr = h * MF::kRowsPerLoad + ld_row;
        const int rl = last_n0 + rr < N ? rr : N - 1 - last_n0;
        voff_w[h] = __umul24((uint32_t)rr, (uint32_t)row_bytes) + (uint32_t)(ld_col * 16);
        voff_w_last[h] = __umul24((uint32_t)rl, (uint32_t)row_bytes) + (uint32_t)(ld_col * 16);
    }
    const uint32_t voff_sc = __umul24((uint32_t)op_row, (uint32_t)G) * 2u;
    const uint32_t voff_sc_last =
        __umul24((uint32_t)(last_n0 + op_row < N ? op_row : N - 1 - last_n0), (uint32_t)G) * 2u;

    struct TileRegs {
        u32x4 w[MF::kLoads];
        uint2 sc;
    };
    // Unconditional loads (so that the number of loads behind any ring slot is a constant); a
    // position past the wave's last row tile re-reads row tile 0.
    auto load_tile = [&](TileRegs &tr, int rt, int kt) {
        const int rte = rt < n_rt ? rt : 0;
        const bool last = rte == n_rt - 1;
        const uint32_t soff_w = (uint32_t)rte * (uint32_t)(16 * row_bytes) + (uint32_t)(kt * MF::kTileBytes);
        const uint32_t soff_sc = ((uint32_t)rte * (uint32_t)(16 * G) + (uint32_t)(kt * kMxTileGroups)) * 2u;
        const uint8_t *bw = pB + soff_w;
        const unsigned char *bs = pws + soff_sc;
#pragma unroll
        for (int h = 0; h < MF::kLoads; ++h)
            tr.w[h] = *reinterpret_cast<const u32x4 *>(bw + (last ? voff_w_last[h] : voff_w[h]));
        if (!G32) tr.sc = *reinterpret_cast<const uint2 *>(bs + (last ? voff_sc_last : voff_sc));
    };
    auto park_tile = [&](const TileRegs &tr) {
#pragma unroll
        for (int h = 0; h < MF::kLoads; ++h) {
            unsigned char *dst = wt + (h * MF::kRowsPerLoad + ld_row) * MF::kPitch + ld_col * 16;
            uint2 *d2 = reinterpret_cast<uint2 *>(dst);
            d2[0] = make_uint2(tr.w[h].x, tr.w[h].y);
            d2[1] = make_uint2(tr.w[h].z, tr.w[h].w);
        }
    };

    // ---- activation staging, as in gemv_mx.hip.h, but once: wave w stages K tiles w, w + 4, ...
    constexpr int QB = mfma_quarter_bytes<BITS>();
    constexpr int QW = QB / 16;
    constexpr int QPT = kMxTileK / QB;
    constexpr int TSTEP = 64 / QPT;
    constexpr int kSt = 8 / TSTEP;
    const int sq = lane & (QPT - 1);
    const int st0 = lane / QPT;
    const int nbatch = (M + 7) >> 3;
    struct ActRegs {
        u32x4 v[kSt][QW];
    };
    auto act_load = [&](ActRegs &ar, int kt, int batch) {
#pragma unroll
        for (int i = 0; i < kSt; ++i) {
            if (TSTEP * i + 8 * batch >= M) break;
            int tok = st0 + TSTEP * i + 8 * batch;
            tok = tok < M ? tok : M - 1;
            const uint32_t off = (uint32_t)tok * (uint32_t)K + (uint32_t)(kt * kMxTileK + sq * QB);
            const u32x4 *src = reinterpret_cast<const u32x4 *>(pA + off);
#pragma unroll
            for (int w = 0; w < QW; ++w) ar.v[i][w] = src[w];
        }
    };
    auto act_store = [&](const ActRegs &ar, int kt, int batch) {
        u32x4 *dst = act + (uint32_t)kt * tile_units + (st0 + 8 * batch) * kMxTokenUnits;
#pragma unroll
        for (int i = 0; i < kSt; ++i) {
            if (TSTEP * i + 8 * batch >= M) break;
            if (st0 + TSTEP * i + 8 * batch < M)
                (void)mfma_stage_quarter<BITS>(ar.v[i], dst + TSTEP * i * kMxTokenUnits, sq);
        }
    };

    // ---- prologue: first activation loads (L2), multipliers, then the ring of weight tiles
    ActRegs a_first;
    act_load(a_first, wave, 0);  // KT >= 4: every wave has a tile
    float rinv[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        const int m = 4 * kb + r;
        rinv[r] = G32 ? 1.0f : p.s[m < M ? m : M - 1];
    }
    __builtin_amdgcn_sched_barrier(0);
    TileRegs ring[kMxsRing];
    int l_rt = first_rt, l_kt = 0;  // position of the next load in this wave's tile stream
    auto advance_load = [&]() {
        if (++l_kt == KT) {
            l_kt = 0;
            l_rt += wave_stride;
        }
    };
#pragma unroll
    for (int j = 0; j < kMxsRing; ++j) {
        load_tile(ring[j], l_rt, l_kt);
        advance_load();
    }
    __builtin_amdgcn_sched_barrier(0);
    act_store(a_first, wave, 0);
    for (int kt = wave; kt < KT; kt += kMxWaves)
        for (int b = (kt == wave ? 1 : 0); b < nbatch; ++b) {
            ActRegs more;
            act_load(more, kt, b);
            act_store(more, kt, b);
        }
#pragma unroll
    for (int r = 0; r < MR; ++r) rinv[r] = __builtin_amdgcn_rcpf(rinv[r]);
    __syncthreads();

    const int a_tok = op_row < M ? op_row : M - 1;
    const u32x4 *act_lane = act + a_tok * kMxTokenUnits + 2 * kb;
    // Offset term of the packed codes per (group, token): -2 sum(a) (T2) / -sum(a) (Q1), from the
    // matrix cores (-2 / -1 in every slot of the weight operand), once per workgroup.
    {
        constexpr int kNegs = BITS == 2 ? (int)0xFEFEFEFEu : (int)0xFFFFFFFFu;
        const v4i negs = {kNegs, kNegs, kNegs, kNegs};
        const v4i zero4 = {0, 0, 0, 0};
        for (int g = wave; g < G; g += kMxWaves) {
            const u32x4 *a_grp = act_lane + (uint32_t)(g >> 2) * tile_units + (g & 3) * 8;
            const u32x4 a0 = a_grp[0];
            const u32x4 a1 = a_grp[1];
            const v4i va0 = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w};
            const v4i va1 = {(int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
            v4i vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, negs, zero4, 0, 0, 0);
            vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, negs, vcr, 0, 0, 0);
            if (op_row == 0) *reinterpret_cast<v4i *>(corr + g * 16 + 4 * kb) = vcr;
        }
    }
    __syncthreads();
    const int32_t *corr_lane = corr + 4 * kb;
    const unsigned char *wsrc = wt + op_row * MF::kPitch;

    float acc[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r) acc[r] = 0.0f;
    int c_rt = first_rt, c_kt = 0;  // position of the tile being consumed
    // Four tiles per trip with no exit in between: when the wave's stream ends inside a trip
    // (K / 512 no multiple of four) the remaining positions are row tiles past the matrix, whose
    // results are not stored.
    while (c_rt < n_rt) {
#pragma unroll
        for (int j = 0; j < kMxsRing; ++j) {
            park_tile(ring[j]);
            // (the copy is pinned to its own registers here: otherwise the compiler lets the
            // reload below land in temporaries and moves them at the end of the trip, behind a
            // wait for every load in flight)
            uint2 sc = G32 ? make_uint2(0u, 0u) : ring[j].sc;
            asm volatile("" : "+v"(sc.x), "+v"(sc.y));
            load_tile(ring[j], l_rt, l_kt);
            advance_load();
            const u32x4 *a_tile = act_lane + (uint32_t)c_kt * tile_units;
            const int32_t *c_tile = corr_lane + c_kt * (kMxTileGroups * 16);
#pragma unroll
            for (int gi = 0; gi < kMxTileGroups; ++gi) {
                const u32x4 a0 = a_tile[gi * 8];
                const u32x4 a1 = a_tile[gi * 8 + 1];
                const v4i va0 = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w};
                const v4i va1 = {(int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                const v4i vcr = *reinterpret_cast<const v4i *>(c_tile + gi * 16);
                uint32_t p0, p1;
                if (BITS == 2) {
                    const uint2 pp = *reinterpret_cast<const uint2 *>(wsrc + gi * 32 + kb * 8);
                    p0 = pp.x;
                    p1 = pp.y;
                } else {
                    p0 = *reinterpret_cast<const uint32_t *>(wsrc + gi * 16 + kb * 4);
                    p1 = 0;
                }
                uint32_t b0[4], b1[4];
                mfma_unpack<BITS>(p0, p1, b0, b1);
                const v4i vb0 = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3]};
                const v4i vb1 = {(int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
                v4i dd = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, vb0, vcr, 0, 0, 0);
                dd = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, vb1, dd, 0, 0, 0);
                if (G32) {
                    const int row = (c_rt << 4) + op_row;
#pragma unroll
                    for (int r = 0; r < MR; ++r) {
                        const int tk = 4 * kb + r;
                        if (row < N && tk < M)
                            reinterpret_cast<int32_t *>(p.out)[((size_t)tk * N + row) * G + (c_kt * kMxTileGroups + gi)] = dd[r];
                    }
                    continue;
                }
                const uint32_t raw = (gi & 2) ? sc.y : sc.x;
                const float wsf =
                    scale_to_f32<SF16>((uint16_t)((gi & 1) ? (raw >> 16) : (raw & 0xffffu)));
#pragma unroll
                for (int r = 0; r < MR; ++r) acc[r] += (float)dd[r] * wsf;
            }
            if (++c_kt == KT) {  // uniform: the row tile is complete
                const int row = (c_rt << 4) + op_row;
                const bool row_ok = row < N && !G32;
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    const int tk = 4 * kb + r;
                    const float y = acc[r] * rinv[r];
                    const uint32_t o = (uint32_t)tk * (uint32_t)N + (uint32_t)row;
                    if (row_ok && tk < M) {
                        if (p.out_f32)
                            reinterpret_cast<float *>(p.out)[o] = y;
                        else
                            reinterpret_cast<uint16_t *>(p.out)[o] = f32_to_bf16_rne_nobranch(y);
                    }
                    acc[r] = 0.0f;
                }
                c_kt = 0;
                c_rt += wave_stride;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
using MxsKernelFn = void (*)(const MxsParams);

template <int BITS>
MxsKernelFn mxs_kernel(int scale_kind, bool one_token) {
    if (scale_kind == 2)  // int32 group sums
        return one_token ? gemv_mxs_kernel<BITS, false, 1, true> : gemv_mxs_kernel<BITS, false, 4, true>;
    if (one_token)
        return scale_kind == 1 ? gemv_mxs_kernel<BITS, true, 1> : gemv_mxs_kernel<BITS, false, 1>;
    return scale_kind == 1 ? gemv_mxs_kernel<BITS, true, 4> : gemv_mxs_kernel<BITS, false, 4>;
}

template <int BITS>
int mxs_init_device(int max_lds) {
    for (int sk = 0; sk < 3; ++sk)
        for (int one = 0; one < 2; ++one)
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(mxs_kernel<BITS>(sk, one != 0)),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    max_lds) != hipSuccess)
                return 2;
    return 0;
}

struct MxsTuning {
    int min_bytes = 0;  // smallest matrix (packed bytes) sent here; 0 = built-in, < 0 = never
    int wgs_per_cu = 0; // persistent workgroups per CU; 0 = built-in
};

template <int BITS>
MxsTuning &mxs_tuning() {
    static MxsTuning t;
    return t;
}

// Persistent workgroups per CU: three (measured on the 151936 x 2048 head at 4 / 8 / 9 / 16 tokens:
// 21.1 / 21.5 / 21.6 / 23.4 us against 21.9 / 22.5 / 22.1 / 22.9 us with four and no better with
// five to eight), fewer when the staged activations are large.
template <int BITS>
int mxs_wgs_per_cu(const GemvProblem &q, int lds_limit) {
    const MxsTuning &tu = mxs_tuning<BITS>();
    int per_cu = tu.wgs_per_cu > 0 ? tu.wgs_per_cu : 3;
    const int fit = (int)((size_t)lds_limit / mxs_lds_bytes<BITS>(q.M, q.K));
    return per_cu < fit ? per_cu : fit;
}

// True when the streaming kernel takes the problem: a block of at most 16 tokens whose staged
// activations leave room for at least two workgroups per CU, whole K tiles, and (unless
// `forced`) a matrix long enough that every resident wave gets at least two row tiles.
template <int BITS>
bool mxs_problem_ok(const GemvProblem &q, int out_kind, int lds_limit, int n_cus, bool forced) {
    (void)out_kind;  // every output kind, the int32 group sums included
    if (q.M > 16 || !mx_problem_ok(q, false)) return false;
    // tile offsets are 32-bit: the packed matrix and its scale table stay below 4 GiB
    if ((long)q.N * (q.K * BITS / 8) >= (1L << 32) || (long)q.N * (q.K / kGroup) * 2 >= (1L << 32)) return false;
    if (mxs_wgs_per_cu<BITS>(q, lds_limit) < 2) return false;
    if (forced) return true;
    const MxsTuning &tu = mxs_tuning<BITS>();
    if (tu.min_bytes < 0) return false;
    const long bytes = (long)q.N * (q.K * BITS / 8);
    const long min_bytes = tu.min_bytes > 0 ? tu.min_bytes : (32L << 20);
    if (bytes < min_bytes) return false;
    return (long)((q.N + 15) / 16) >= 2L * n_cus * 16;
}

template <int BITS>
int launch_mxs(const GemvProblem &q, int out_kind, int scale_kind, int lds_limit, int n_cus,
               hipStream_t stream) {
    MxsParams prm{};
    prm.A = q.A;
    prm.B = q.B;
    prm.out = q.out;
    prm.s = q.s;
    prm.ws = reinterpret_cast<const uint16_t *>(q.ws);
    prm.M = q.M;
    prm.N = q.N;
    prm.K = q.K;
    prm.out_f32 = out_kind == OUT_F32 ? 1 : 0;
    const int n_rt = (q.N + 15) / 16;
    int wgs = n_cus * mxs_wgs_per_cu<BITS>(q, lds_limit);
    if (wgs * kMxWaves > n_rt) wgs = (n_rt + kMxWaves - 1) / kMxWaves;
    const int variant = out_kind == OUT_G32 ? 2 : scale_kind;
    hipLaunchKernelGGL(mxs_kernel<BITS>(variant, q.M == 1), dim3(wgs, 1, 1), dim3(kMxThreads, 1, 1),
                       mxs_lds_bytes<BITS>(q.M, q.K), stream, prm);
    note_kernel("gemv_mxs_kernel", BITS, variant == 1, q.M == 1 ? 1 : 4, variant == 2);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_MXS_HIP_H
