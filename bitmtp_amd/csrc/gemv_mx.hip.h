// Grouped matrix-core kernel of the packed low-bit GEMV: ONE launch walks the row tiles of
// several GEMVs (a descriptor table in the kernel arguments), for any block width.
//
// Why one launch for many matrices: a decoder layer's projections are 0.5-3.3 MB each, and a
// launch costs about 1.7 us before its first byte arrives, so a launch per matrix cannot
// stream faster than a fraction of HBM speed whatever the kernel does.  The reference
// launches one kernel per projection (src/bonsai_sft/gpu/model.py:977-1062,
// src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:94-100); projections that do not
// depend on each other (q|k|v, gate|up, or all seven in a throughput measurement) share one
// launch here.
//
// Arithmetic: the same as gemv_mfma.hip.h.  Per 128-wide scale group and 16 weight rows, two
// v_mfma_i32_16x16x64_i8 produce the exact int32 group sums of up to 16 tokens (tokens are the
// A rows, weight rows the B columns); the code offset of the packed weights (T2 codes 0..3
// stand for -2..1, Q1 bits for -1/+1) goes in through the accumulator input as -2*sum(a) /
// -sum(a), so the MFMA result IS the group sum G.  fp32(G) * scale is accumulated per row in
// fp32, multiplied by the reciprocal of the token's activation multiplier (an IEEE division
// done once per token and lane, off the critical path) and rounded to bf16 (RNE).
//
// Data movement:
//   * weights: coalesced 16-byte loads (8 lanes read one 128-byte segment of a T2 row, 4 lanes a
//     64-byte segment of a Q1 row), parked in a wave-private LDS tile whose row pitch (tile bytes
//     + 8) keeps both directions free of bank conflicts, and read back in operand layout (lane =
//     weight row l % 16, K block l / 16).  Loading straight in operand layout would put every
//     lane of a load on a different cache line (neighbouring lanes are neighbouring rows).
//   * activations: every wave stages, per K tile (512 activations of up to 16 tokens), exactly
//     the slice it multiplies -- in operand order (4x4 byte transposes, see gemv_core.h), with the
//     per-(group, token) offset terms -- into its own LDS region.  Nothing is shared between
//     waves, so there is no workgroup barrier in front of the arithmetic and the LDS footprint
//     does not depend on K (a launch reserves the same LDS for all its workgroups: staging whole
//     rows would let one long-K matrix of a group cut the residency of every workgroup).  The
//     activation loads of the next tile travel with its weight loads.
//   * a workgroup is four waves: one block of 16 R rows, K cut into four slices; the slices are
//     added in slice order through LDS (deterministic), then stored.
//   * a workgroup walks row-block iterations with stride wg_count (one iteration per
//     workgroup for layer-sized matrices, a few for the 151936-row head), always with the
//     next K tile's loads in flight while the current one is consumed.
#ifndef BONSAI_GEMV_MX_HIP_H
#define BONSAI_GEMV_MX_HIP_H

#include "gemv_mfma.hip.h"

namespace bonsai {

constexpr int kMxMaxDesc = 24;      // descriptors per launch
constexpr int kMxWaves = 4;         // waves per workgroup: one block of 16 R rows, four K slices
constexpr int kMxThreads = kMxWaves * 64;
constexpr int kMxTileGroups = 4;    // scale groups per K tile
constexpr int kMxTileK = 512;       // activations per K tile
constexpr int kMxTokenUnits = 33;   // 16-byte units per staged token and tile (32 + 1: conflict-free)
constexpr int kMxBlockShift = 3;    // workgroup ranges of descriptors start at multiples of 8
constexpr int kMxMaxBlocks = 1024;  // entries of the workgroup-block -> descriptor table

struct MxDesc {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int M, N, K;
    int wg_begin;  // first workgroup of this descriptor
    int wg_count;  // its workgroups (iteration stride)
    int n_iter;    // row-block iterations: ceil(N / (16 R))
};
static_assert(sizeof(MxDesc) == 64, "one descriptor is one 64-byte scalar load");

struct MxParams {
    int out_f32;  // 1: fp32 value, 0: bf16
    int mmax;     // largest M of the launch (sizes the per-wave LDS regions)
    int pad[2];
    MxDesc d[kMxMaxDesc];
    uint32_t desc_of_block[kMxMaxBlocks / 4];  // one byte per block b: descriptor of workgroups [8b, 8b + 8)
};

// LDS bytes of one wave: the staged tokens of one K tile and one weight tile.
template <int BITS, int R>
__host__ __device__ constexpr size_t mx_wave_lds_bytes(int mmax) {
    return (size_t)mmax * kMxTokenUnits * 16 + mfma_wave_tile_bytes<BITS, R>();
}
// LDS bytes of one workgroup: the wave regions and the K-slice partials (two halves used in turn).
template <int BITS, int R>
__host__ __device__ constexpr size_t mx_lds_bytes(int mmax) {
    return kMxWaves * mx_wave_lds_bytes<BITS, R>(mmax) + (size_t)2 * kMxWaves * R * 4 * 64 * 4;
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne_nobranch(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    const bool is_nan = (u & 0x7fffffffu) > 0x7f800000u;
    return (uint16_t)(is_nan ? ((u >> 16) | 0x0040u) : r);
}

template <int BITS, int R, bool G32, bool SF16>
__global__ void __launch_bounds__(kMxThreads) __attribute__((amdgpu_waves_per_eu(4)))
gemv_mx_kernel(const MxParams p) {
    using MF = MfmaFmt<BITS>;
    extern __shared__ __align__(16) unsigned char smem[];

    // ---- which descriptor this workgroup serves: one table byte per block of 8 workgroups
    const int wg = (int)blockIdx.x;
    const int blk = wg >> kMxBlockShift;
    const int di = (int)((p.desc_of_block[blk >> 2] >> (8 * (blk & 3))) & 0xffu);  // a scalar load
    const MxDesc &d = p.d[di];
    const int lwg = wg - d.wg_begin;
    const int stride = d.wg_count;
    if (lwg >= stride) return;  // padding workgroups at the end of a descriptor's range

    const int K = d.K, N = d.N, M = d.M;  // M <= 16 (the host splits wider blocks)
    const int G = K >> 7;
    const int row_bytes = K * BITS / 8;
    const uint8_t *const pB = d.B;
    const uint16_t *const pws = d.ws;
    const int8_t *const pA = d.A;
    void *const pout = d.out;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: loop control stays scalar
    const int n_iter = d.n_iter;
    const int ntiles = K >> 9;  // K % 512 == 0 and K >= 2048 are checked on the host

    // ---- LDS: per wave [tokens][33] staged units and the weight tile; after the four wave
    // regions the K-slice partials
    const uint32_t wave_bytes = (uint32_t)mx_wave_lds_bytes<BITS, R>(p.mmax);
    unsigned char *wbase = smem + (uint32_t)wave * wave_bytes;
    u32x4 *act = reinterpret_cast<u32x4 *>(wbase);  // [M][33]
    unsigned char *wt = wbase + (uint32_t)p.mmax * (kMxTokenUnits * 16);
    float *red = reinterpret_cast<float *>(smem + kMxWaves * wave_bytes);

    const int ld_row = lane / MF::kLanesPerRow;  // row inside one coalesced load
    const int ld_col = lane % MF::kLanesPerRow;  // 16-byte chunk inside the tile row
    const int op_row = lane & 15;                // operand row: weight row / token
    const int kb = lane >> 4;                    // operand K block, also the token quad of the result

    // K tiles [tb, te) of this wave: the wave-th quarter of the row's tiles (never empty)
    const int tb = (ntiles * wave) >> 2;
    const int te = (ntiles * (wave + 1)) >> 2;

    struct TileRegs {
        u32x4 w[R][MF::kLoads];
        uint2 sc[R];
    };
    // Every load is unconditional (rows clamped into the matrix), so that the compiler can
    // count outstanding loads exactly.
    // (32-bit byte offsets from the uniform base pointers: every operand is far below 4 GB)
    auto load_tile = [&](TileRegs &tr, int n0, int kt) {
#pragma unroll
        for (int rt = 0; rt < R; ++rt) {
#pragma unroll
            for (int h = 0; h < MF::kLoads; ++h) {
                int row = n0 + rt * 16 + h * MF::kRowsPerLoad + ld_row;
                row = row < N ? row : N - 1;
                const uint32_t off = (uint32_t)row * (uint32_t)row_bytes +
                                     (uint32_t)(kt * MF::kTileBytes + ld_col * 16);
                tr.w[rt][h] = *reinterpret_cast<const u32x4 *>(pB + off);
            }
            if (!G32) {
                int row = n0 + rt * 16 + op_row;
                row = row < N ? row : N - 1;
                const uint32_t off = ((uint32_t)row * (uint32_t)G + (uint32_t)(kt * kMxTileGroups)) * 2u;
                tr.sc[rt] = *reinterpret_cast<const uint2 *>(
                    reinterpret_cast<const unsigned char *>(pws) + off);
            }
        }
    };
    auto park_tile = [&](const TileRegs &tr) {
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
#pragma unroll
            for (int h = 0; h < MF::kLoads; ++h) {
                unsigned char *dst = wt + (rt * 16 + h * MF::kRowsPerLoad + ld_row) * MF::kPitch +
                                     ld_col * 16;
                uint2 *d2 = reinterpret_cast<uint2 *>(dst);  // the pitch is 8- not 16-byte aligned
                d2[0] = make_uint2(tr.w[rt][h].x, tr.w[rt][h].y);
                d2[1] = make_uint2(tr.w[rt][h].z, tr.w[rt][h].w);
            }
    };

    // ---- staging of one K tile of activations by one wave: 4x4 byte transposes into operand
    // order, nothing else (the per-group activation sums come from the matrix cores, below).
    // A lane owns one quarter of the tile (16 natural-order bytes for T2, 32 for Q1: quarter
    // lane % QPT) and every (64 / QPT)-th token starting at lane / QPT; a batch is 8 tokens.
    constexpr int QB = mfma_quarter_bytes<BITS>();
    constexpr int QW = QB / 16;
    constexpr int QPT = kMxTileK / QB;       // quarters per token and tile: 32 (T2) or 16 (Q1)
    constexpr int TSTEP = 64 / QPT;          // tokens between two tasks of a lane: 2 (T2) or 4 (Q1)
    constexpr int kSt = 8 / TSTEP;           // tasks per batch: 4 (T2) or 2 (Q1), 16 VGPRs of loads
    const int sq = lane & (QPT - 1);
    const int st0 = lane / QPT;
    const int nbatch = (M + 7) >> 3;
    struct ActRegs {
        u32x4 v[kSt][QW];
    };
    auto act_load = [&](ActRegs &ar, int kt, int batch) {
#pragma unroll
        for (int i = 0; i < kSt; ++i) {
            if (TSTEP * i + 8 * batch >= M) break;  // uniform: no lane of this task has a token
            int tok = st0 + TSTEP * i + 8 * batch;
            tok = tok < M ? tok : M - 1;  // clamped duplicates are not written
            const uint32_t off = (uint32_t)tok * (uint32_t)K + (uint32_t)(kt * kMxTileK + sq * QB);
            const u32x4 *src = reinterpret_cast<const u32x4 *>(pA + off);
#pragma unroll
            for (int w = 0; w < QW; ++w) ar.v[i][w] = src[w];
        }
    };
    auto act_store = [&](const ActRegs &ar, int batch) {
        u32x4 *dst = act + (st0 + 8 * batch) * kMxTokenUnits;
#pragma unroll
        for (int i = 0; i < kSt; ++i) {
            if (TSTEP * i + 8 * batch >= M) break;
            if (st0 + TSTEP * i + 8 * batch < M)
                (void)mfma_stage_quarter<BITS>(ar.v[i], dst + TSTEP * i * kMxTokenUnits, sq);
        }
    };

    // ---- prologue: the activation loads of the first tile (an L2 hit), the activation
    // multipliers, then the first weight tile (HBM).  Loads return in order: the activations are
    // back first and are staged while the weights are on their way.
    ActRegs acur;
    act_load(acur, tb, 0);
    float rinv[4] = {1.0f, 1.0f, 1.0f, 1.0f};  // activation multipliers: wave 0 stores the rows
    if (!G32 && wave == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = 4 * kb + r;
            rinv[r] = d.s[m < M ? m : M - 1];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    TileRegs cur;
    load_tile(cur, lwg * (R * 16), tb);
    __builtin_amdgcn_sched_barrier(0);
    float acc[R][4];
#pragma unroll
    for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[rt][r] = 0.0f;

    // tokens past M alias the last valid one: their result columns are never stored
    const int a_tok = op_row < M ? op_row : M - 1;
    const u32x4 *act_lane = act + a_tok * kMxTokenUnits + 2 * kb;
    // -2 (T2) / -1 (Q1) in every slot of the weight operand gives -2 sum(a) / -sum(a) per token
    // in the accumulator layout: the offset term of the packed codes, straight from the matrix cores
    constexpr int kNegs = BITS == 2 ? (int)0xFEFEFEFEu : (int)0xFFFFFFFFu;
    const v4i negs = {kNegs, kNegs, kNegs, kNegs};
    const v4i zero4 = {0, 0, 0, 0};

    int staged = -1;  // the K tile whose activations sit in this wave's LDS region
    int par = 0;      // which half of `red` this iteration uses
    for (int iter = lwg; iter < n_iter; iter += stride) {
        const int n0 = iter * (R * 16);
        for (int kt = tb; kt < te; ++kt) {
            if (staged != kt) {
                act_store(acur, 0);
                for (int b = 1; b < nbatch; ++b) {  // blocks of more than 8 tokens
                    ActRegs more;
                    act_load(more, kt, b);
                    act_store(more, b);
                }
                staged = kt;
            }
            park_tile(cur);
            uint2 sc[R];
#pragma unroll
            for (int rt = 0; rt < R; ++rt) sc[rt] = cur.sc[rt];
            // next: the following tile of this slice, else the slice's first tile for the next
            // iteration's rows (a uniform branch: nothing is requested past the last tile)
            {
                int nkt = kt + 1, nn = n0;
                if (nkt == te) {
                    nkt = tb;
                    nn = (iter + stride) * (R * 16);
                }
                if (nn < N) {
                    if (nkt != kt) act_load(acur, nkt, 0);
                    load_tile(cur, nn, nkt);
                }
            }
#pragma unroll
            for (int gi = 0; gi < kMxTileGroups; ++gi) {
                const int g = kt * kMxTileGroups + gi;
                const u32x4 a0 = act_lane[gi * 8];
                const u32x4 a1 = act_lane[gi * 8 + 1];
                const v4i va0 = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w};
                const v4i va1 = {(int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                v4i vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, negs, zero4, 0, 0, 0);
                vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, negs, vcr, 0, 0, 0);
#pragma unroll
                for (int rt = 0; rt < R; ++rt) {
                    const unsigned char *src = wt + (rt * 16 + op_row) * MF::kPitch;
                    uint32_t p0, p1;
                    if (BITS == 2) {
                        const uint2 pp = *reinterpret_cast<const uint2 *>(src + gi * 32 + kb * 8);
                        p0 = pp.x;
                        p1 = pp.y;
                    } else {
                        p0 = *reinterpret_cast<const uint32_t *>(src + gi * 16 + kb * 4);
                        p1 = 0;
                    }
                    uint32_t b0[4], b1[4];
                    mfma_unpack<BITS>(p0, p1, b0, b1);
                    const v4i vb0 = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3]};
                    const v4i vb1 = {(int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
                    v4i dd = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, vb0, vcr, 0, 0, 0);
                    dd = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, vb1, dd, 0, 0, 0);
                    if (G32) {
                        const int row = n0 + rt * 16 + op_row;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int tk = 4 * kb + r;
                            if (row < N && tk < M)
                                reinterpret_cast<int32_t *>(
                                    pout)[((size_t)tk * N + row) * G + g] = dd[r];
                        }
                    } else {
                        const uint32_t raw = (gi & 2) ? sc[rt].y : sc[rt].x;
                        const float wsf = scale_to_f32<SF16>(
                            (uint16_t)((gi & 1) ? (raw >> 16) : (raw & 0xffffu)));
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[rt][r] += (float)dd[r] * wsf;
                    }
                }
            }
        }
        if (G32) continue;

        // ---- add the four K slices in slice order (every wave of the workgroup reaches the
        // barrier the same number of times: n_iter and the stride are uniform over the workgroup)
        {
            float *mine = red + ((size_t)par * kMxWaves + wave) * (R * 4 * 64);
            if (wave != 0) {
#pragma unroll
                for (int rt = 0; rt < R; ++rt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) mine[(rt * 4 + r) * 64 + lane] = acc[rt][r];
            }
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int k2 = 1; k2 < kMxWaves; ++k2) {
                    const float *other = mine + (size_t)k2 * (R * 4 * 64);
#pragma unroll
                    for (int rt = 0; rt < R; ++rt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[rt][r] += other[(rt * 4 + r) * 64 + lane];
                }
#pragma unroll
                for (int rt = 0; rt < R; ++rt) {
                    const int row = n0 + rt * 16 + op_row;
                    const bool row_ok = row < N;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int tk = 4 * kb + r;
                        // (reciprocal to 1 ulp instead of an IEEE division: the reference's own
                        // kernels are built with fast-math division)
                        const float y = acc[rt][r] * __builtin_amdgcn_rcpf(rinv[r]);
                        const uint32_t o = (uint32_t)tk * (uint32_t)N + (uint32_t)row;
                        if (row_ok && tk < M) {
                            if (p.out_f32)
                                reinterpret_cast<float *>(pout)[o] = y;
                            else
                                reinterpret_cast<uint16_t *>(pout)[o] = f32_to_bf16_rne_nobranch(y);
                        }
                    }
                }
            }
            par ^= 1;
        }
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[rt][r] = 0.0f;
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
// One GEMV of a grouped call, as the caller states it (host memory; the pointers inside are
// device pointers).  Mirrors bonsai_gemv_desc of include/bonsai_gemv.h.
struct GemvProblem {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const void *ws;
    int M, N, K;
};

struct MxTuning {
    int row_tiles = 0;   // R: 1 or 2; 0 = heuristic
    int max_wgs = 0;     // cap on the workgroups of one launch; 0 = heuristic
    int min_width = 0;   // smallest M the grouped entry sends here (below: the single-GEMV path); 0 = 1
};

template <int BITS>
MxTuning &mx_tuning() {
    static MxTuning t;
    return t;
}

using MxKernelFn = void (*)(const MxParams);

template <int BITS>
struct MxTable {
    MxKernelFn fn[2][3];  // [R index: 1, 2][variant: bf16 scales, fp16 scales, G32]
};

template <int BITS>
const MxTable<BITS> &mx_table() {
    static const MxTable<BITS> t = [] {
        MxTable<BITS> x{};
        x.fn[0][0] = gemv_mx_kernel<BITS, 1, false, false>;
        x.fn[0][1] = gemv_mx_kernel<BITS, 1, false, true>;
        x.fn[0][2] = gemv_mx_kernel<BITS, 1, true, false>;
        x.fn[1][0] = gemv_mx_kernel<BITS, 2, false, false>;
        x.fn[1][1] = gemv_mx_kernel<BITS, 2, false, true>;
        x.fn[1][2] = gemv_mx_kernel<BITS, 2, true, false>;
        return x;
    }();
    return t;
}

template <int BITS>
int mx_init_device(int max_lds) {
    const MxTable<BITS> &t = mx_table<BITS>();
    for (int r = 0; r < 2; ++r)
        for (int v = 0; v < 3; ++v)
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(t.fn[r][v]),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    max_lds) != hipSuccess)
                return 2;
    return 0;
}

// True when this kernel takes the problem: whole K tiles and at least four of them (one per
// wave), token block of at most 16 (wider blocks are split by the caller), operands aligned for
// the vector loads.
inline bool mx_problem_ok(const GemvProblem &q, bool g32) {
    const auto al = [](const void *ptr, uintptr_t a) {
        return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) == 0;
    };
    return q.K % 512 == 0 && q.K >= 2048 && al(q.A, 16) && al(q.B, 16) && (g32 || al(q.ws, 8));
}

// Launches the grouped kernel for up to kMxMaxDesc problems of at most 16 tokens each.
// Returns 0, -1 when a problem does not fit (the caller falls back), 2 on a launch error.
template <int BITS>
int launch_mx(const GemvProblem *probs, int count, int out_kind, int scale_kind, int lds_limit,
              int n_cus, hipStream_t stream) {
    if (count < 1 || count > kMxMaxDesc) return 1;
    const MxTuning &tu = mx_tuning<BITS>();
    long total_bytes = 0;
    for (int i = 0; i < count; ++i)
        total_bytes += (long)probs[i].N * (probs[i].K * BITS / 8 + probs[i].K / kGroup * 2);

    // row tiles per wave for the whole launch
    const int R = tu.row_tiles == 1 || tu.row_tiles == 2 ? tu.row_tiles
                                                         : (total_bytes >= (48L << 20) ? 2 : 1);
    const int ri = R - 1;

    MxParams prm{};
    prm.out_f32 = out_kind == OUT_F32 ? 1 : 0;
    int mmax = 1;
    long iters_total = 0;
    // Descriptors with the most K tiles per wave first: their workgroups run longest, so they
    // take the lowest workgroup numbers and start first.
    int order[kMxMaxDesc];
    for (int i = 0; i < count; ++i) order[i] = i;
    for (int i = 1; i < count; ++i)
        for (int j = i; j > 0 && probs[order[j]].K > probs[order[j - 1]].K; --j) {
            const int t = order[j];
            order[j] = order[j - 1];
            order[j - 1] = t;
        }
    for (int i = 0; i < count; ++i) {
        const GemvProblem &q = probs[order[i]];
        MxDesc &d = prm.d[i];
        d.A = q.A;
        d.B = q.B;
        d.out = q.out;
        d.s = q.s;
        d.ws = reinterpret_cast<const uint16_t *>(q.ws);
        d.M = q.M;
        d.N = q.N;
        d.K = q.K;
        mmax = q.M > mmax ? q.M : mmax;
        d.n_iter = (q.N + R * 16 - 1) / (R * 16);
        iters_total += d.n_iter;
    }
    // Workgroups: one per iteration while the launch stays within the cap (everything in
    // flight at once); above it every descriptor gets a share of the cap in proportion to
    // its iterations and its workgroups stride over them.  Every descriptor's range starts at
    // a multiple of 8 workgroups (the table has one entry per 8); the few workgroups past its
    // count return at once.
    long cap = tu.max_wgs > 0 ? tu.max_wgs : (long)n_cus * 24;
    if (cap < count) cap = count;
    if (cap > (long)(kMxMaxBlocks - kMxMaxDesc) << kMxBlockShift)
        cap = (long)(kMxMaxBlocks - kMxMaxDesc) << kMxBlockShift;
    int wg = 0;
    for (int i = 0; i < count; ++i) {
        MxDesc &d = prm.d[i];
        long share = iters_total <= cap ? d.n_iter : (long)d.n_iter * cap / iters_total;
        if (share < 1) share = 1;
        if (share > d.n_iter) share = d.n_iter;
        d.wg_begin = wg;
        d.wg_count = (int)share;
        const int blocks = ((int)share + (1 << kMxBlockShift) - 1) >> kMxBlockShift;
        if ((wg >> kMxBlockShift) + blocks > kMxMaxBlocks) return -1;
        for (int b = 0; b < blocks; ++b) {
            const int blk = (wg >> kMxBlockShift) + b;
            prm.desc_of_block[blk >> 2] |= (uint32_t)i << (8 * (blk & 3));
        }
        wg += blocks << kMxBlockShift;
    }

    prm.mmax = mmax;
    const size_t lds = R == 1 ? mx_lds_bytes<BITS, 1>(mmax) : mx_lds_bytes<BITS, 2>(mmax);
    if (lds > (size_t)lds_limit) return -1;
    const int variant = out_kind == OUT_G32 ? 2 : scale_kind;
    const MxKernelFn fn = mx_table<BITS>().fn[ri][variant];
    hipLaunchKernelGGL(fn, dim3(wg, 1, 1), dim3(kMxThreads, 1, 1), lds, stream, prm);
    note_kernel("gemv_mx_kernel", BITS, R, variant == 1, variant == 2);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_MX_HIP_H
