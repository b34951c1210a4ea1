// Lean form of the grouped matrix-core kernel (gemv_mx.hip.h) for launches of up to twelve
// GEMVs whose row tiles all fit one workgroup each: the same data movement and arithmetic --
// per wave one K slice of 16 rows, activations of the slice staged by the wave itself in operand
// order, weight tile parked in LDS, exact int32 group sums from v_mfma_i32_16x16x64_i8 with the
// code offset fed through the accumulator, K slices added in slice order -- with the
// bookkeeping cut down.  Measured with ablated builds and in-kernel time stamps on MI355X: a
// layer-sized launch (13 MB, 5120 waves) spends as long issuing VALU instructions as it spends
// receiving its bytes, and more than half of the instructions of gemv_mx.hip.h are not the
// tile arithmetic.  Here
//   * the descriptor of a workgroup is found by comparing the workgroup number with up to
//     twelve range ends that arrive in SGPRs with the wave (preloaded kernel arguments): one
//     scalar load (the descriptor) instead of three dependent ones before the first vector load;
//   * weights, scales and activations are read through buffer resources: rows past N and
//     tokens past M read as zero by the range check, so there are no clamps or selects in the
//     address arithmetic, and a load is one per-lane offset plus a scalar;
//   * one workgroup per 16 rows and no striding loop, and a register budget that lets every
//     workgroup of a layer-sized launch be resident at once (template parameters NB and OCC
//     below; a build that spills the staged-activation registers puts a memory round trip in
//     front of every tile and costs 40 % at eight tokens);
//   * after the K-slice exchange wave r finishes result column r of every token quad, so the
//     epilogue (division, rounding, store) is spread over the four waves.
// Same summation order as gemv_mx.hip.h; the final division by the activation multiplier is an
// IEEE division here (a reciprocal multiply there).
// Reference being replaced: one launch per projection, src/bonsai_sft/gpu/model.py:977-1062
// through src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:94-100.
#ifndef BONSAI_GEMV_MXL_HIP_H
#define BONSAI_GEMV_MXL_HIP_H

#include "gemv_mx.hip.h"

namespace bonsai {

constexpr int kMxlMaxDesc = 12;

struct MxlDesc {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int M, N, K;
    int wg_begin;
    int pad[2];
};
static_assert(sizeof(MxlDesc) == 64, "one descriptor is one 64-byte scalar load");

struct MxlTable {
    MxlDesc d[kMxlMaxDesc];
};

constexpr int kMxlBufferWord3 = 0x00020000;  // raw buffer, 32-bit format, range check on

__device__ __forceinline__ u32x4 mxl_load_b128(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
    typedef unsigned int v4u __attribute__((ext_vector_type(4)));
    const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, (int)soff, 0);
    return u32x4{v.x, v.y, v.z, v.w};
}

// LDS bytes of one workgroup: per wave the staged tokens of one K tile and one weight tile, then
// the K-slice partials.
template <int BITS>
__host__ __device__ constexpr size_t mxl_lds_bytes(int mmax, int waves) {
    return waves * mx_wave_lds_bytes<BITS, 1>(mmax) + (size_t)waves * 4 * 64 * 4;
}

// MR: result columns kept per lane (1 when every block of the launch has one token, else 4).
// W: waves per workgroup = K slices per row tile: four, or twelve for a single matrix with long
// rows (K = 6144: one tile per wave instead of three in sequence, each of which would wait for its
// own memory round trip).
// NB: token batches of eight a block can have (2 only when some block has more than eight tokens):
// without the registers of a second batch the four-wave form fits five waves per SIMD, so the
// 1280 workgroups of a layer-sized launch are all resident at once instead of 1024 of them.
// OCC: waves per SIMD the register allocation aims at.  With two batches five waves fit only
// at exactly 96 registers, which costs about 0.1 us on launches that have no fifth workgroup per
// CU to place, and saves a microsecond on those that do (19456 x 2560 at nine tokens 8.6 ->
// 7.6 us), so the host picks per launch.
// G32: store the exact int32 group sums G[m][n][g] (what the matrix cores return, before any
// scale) instead of the scaled result; the scales and multipliers are not read.
template <int BITS, int MR, bool SF16, int W, int NB, int OCC, bool G32 = false>
__global__ void __launch_bounds__(W * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
gemv_mxl_kernel(int e0, int e1, int e2, int e3, int e4, int e5, int e6, int e7, int e8, int e9,
                int e10, int e11, int out_f32, int mmax, const MxlTable tbl) {
    using MF = MfmaFmt<BITS>;
    extern __shared__ __align__(16) unsigned char smem[];

    // ---- descriptor of this workgroup: (wg >= e) is the sign bit of e - 1 - wg (scalar)
    const int wg = (int)blockIdx.x;
    const auto ge = [wg](int e) { return (int)((uint32_t)(e - 1 - wg) >> 31); };
    const int di = ge(e0) + ge(e1) + ge(e2) + ge(e3) + ge(e4) + ge(e5) + ge(e6) + ge(e7) + ge(e8) +
                   ge(e9) + ge(e10) + ge(e11);
    const MxlDesc d = tbl.d[di];
    const int K = d.K, N = d.N, M = d.M;
    const int G = K >> 7;
    const int KT = K >> 9;  // K % 512 == 0 and K >= 2048 (host)
    const int row_bytes = K * BITS / 8;
    const int n0 = (wg - d.wg_begin) << 4;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ld_row = lane / MF::kLanesPerRow, ld_col = lane % MF::kLanesPerRow;
    const int op_row = lane & 15, kb = lane >> 4;
    const int tb = (KT * wave) / W, te = (KT * (wave + 1)) / W;  // empty for some waves when KT < W

    const uint32_t wave_bytes = (uint32_t)mx_wave_lds_bytes<BITS, 1>(mmax);
    unsigned char *wbase = smem + (uint32_t)wave * wave_bytes;
    u32x4 *act = reinterpret_cast<u32x4 *>(wbase);  // [mmax][33]
    unsigned char *wt = wbase + (uint32_t)mmax * (kMxTokenUnits * 16);
    float *red = reinterpret_cast<float *>(smem + W * wave_bytes);

    const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(d.A), 0, M * K, kMxlBufferWord3);
    const __amdgpu_buffer_rsrc_t rB = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(d.B), 0, N * row_bytes, kMxlBufferWord3);
    // (no records when the group sums are wanted: every scale reads as zero, no access is made)
    const __amdgpu_buffer_rsrc_t rS = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(d.ws), 0, G32 ? 0 : N * G * 2, kMxlBufferWord3);

    // ---- weight tile: kLoads coalesced 16-byte loads per lane, one 8-byte scale load
    uint32_t w_off[MF::kLoads];
#pragma unroll
    for (int h = 0; h < MF::kLoads; ++h)
        w_off[h] = (uint32_t)(n0 + h * MF::kRowsPerLoad + ld_row) * (uint32_t)row_bytes +
                   (uint32_t)(ld_col * 16);
    const uint32_t s_off = (uint32_t)(n0 + op_row) * (uint32_t)(G * 2);
    u32x4 w[MF::kLoads];
    uint2 scr;
    auto load_w = [&](int kt) {
#pragma unroll
        for (int h = 0; h < MF::kLoads; ++h) w[h] = mxl_load_b128(rB, w_off[h], (uint32_t)(kt * MF::kTileBytes));
        typedef unsigned int v2u __attribute__((ext_vector_type(2)));
        const v2u sv = __builtin_amdgcn_raw_buffer_load_b64(rS, (int)s_off, kt * 8, 0);
        scr = make_uint2(sv.x, sv.y);
    };

    // ---- activation staging by the wave itself, as in gemv_mx.hip.h: a lane owns one quarter
    // of the tile (16 natural-order bytes for T2, 32 for Q1) of every TSTEP-th token; a batch
    // is 8 tokens.  Tokens past M read zeros and are not stored.
    constexpr int QB = mfma_quarter_bytes<BITS>();
    constexpr int QW = QB / 16;
    constexpr int QPT = kMxTileK / QB;
    constexpr int TSTEP = 64 / QPT;
    constexpr int kSt = 8 / TSTEP;
    const int sq = lane & (QPT - 1);
    const int st0 = lane / QPT;
    const int nbatch = (M + 7) >> 3;
    const uint32_t a_off = (uint32_t)st0 * (uint32_t)K + (uint32_t)(sq * QB);
    struct ActRegs {
        u32x4 v[kSt][QW];
    };
    auto act_load = [&](ActRegs &ar, int kt, int batch) {
#pragma unroll
        for (int i = 0; i < kSt; ++i) {
            if (TSTEP * i + 8 * batch >= M) break;  // uniform: no lane of this task has a token
#pragma unroll
            for (int q = 0; q < QW; ++q)
                ar.v[i][q] = mxl_load_b128(rA, a_off + (uint32_t)((TSTEP * i + 8 * batch) * K + q * 16),
                                           (uint32_t)(kt * kMxTileK));
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

    // ---- prologue: activation loads (L2), then the weight tile (HBM), then the multiplier of
    // the token this lane will finish
    ActRegs acur, amore;  // tokens 0-7 and 8-15 of the tile (amore unused when NB == 1)
    act_load(acur, tb, 0);
    if (NB > 1 && nbatch > 1) act_load(amore, tb, 1);
    load_w(tb);
    float s_tok = 1.0f;
    if (!G32 && wave < MR) {
        const int tkc = 4 * kb + wave;
        s_tok = d.s[tkc < M ? tkc : M - 1];
    }

    float acc[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r) acc[r] = 0.0f;
    const int a_tok = op_row < M ? op_row : M - 1;  // token rows past M alias the last one (never stored)
    const u32x4 *act_lane = act + a_tok * kMxTokenUnits + 2 * kb;
    constexpr int kNegs = BITS == 2 ? (int)0xFEFEFEFEu : (int)0xFFFFFFFFu;
    const v4i negs = {kNegs, kNegs, kNegs, kNegs};
    const v4i zero4 = {0, 0, 0, 0};
    unsigned char *park = wt + ld_row * MF::kPitch + ld_col * 16;
    const unsigned char *wsrc = wt + op_row * MF::kPitch;

    for (int kt = tb; kt < te; ++kt) {
        act_store(acur, 0);
        if (NB > 1 && nbatch > 1) act_store(amore, 1);
#pragma unroll
        for (int h = 0; h < MF::kLoads; ++h) {
            uint2 *d2 = reinterpret_cast<uint2 *>(park + h * MF::kRowsPerLoad * MF::kPitch);
            d2[0] = make_uint2(w[h].x, w[h].y);
            d2[1] = make_uint2(w[h].z, w[h].w);
        }
        const uint2 sc = scr;
        if (kt + 1 < te) {  // uniform: the next tile of this slice travels during the arithmetic
            act_load(acur, kt + 1, 0);
            if (NB > 1 && nbatch > 1) act_load(amore, kt + 1, 1);
            load_w(kt + 1);
        }
#pragma unroll
        for (int gi = 0; gi < kMxTileGroups; ++gi) {
            const u32x4 a0 = act_lane[gi * 8];
            const u32x4 a1 = act_lane[gi * 8 + 1];
            const v4i va0 = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w};
            const v4i va1 = {(int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
            v4i vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, negs, zero4, 0, 0, 0);
            vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, negs, vcr, 0, 0, 0);
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
                const int row = n0 + op_row;
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    const int tk = 4 * kb + r;
                    if (row < N && tk < M)
                        reinterpret_cast<int32_t *>(d.out)[((size_t)tk * N + row) * G + (kt * kMxTileGroups + gi)] = dd[r];
                }
                continue;
            }
            const uint32_t raw = (gi & 2) ? sc.y : sc.x;
            const float wsf = scale_to_f32<SF16>((uint16_t)((gi & 1) ? (raw >> 16) : (raw & 0xffffu)));
#pragma unroll
            for (int r = 0; r < MR; ++r) acc[r] += (float)dd[r] * wsf;
        }
    }
    if (G32) return;

    // ---- K slices added in slice order; wave r finishes column r of every token quad
#pragma unroll
    for (int r = 0; r < MR; ++r) red[(r * W + wave) * 64 + lane] = acc[r];
    __syncthreads();
    if (wave >= MR) return;
    const float *mine = red + (wave * W) * 64 + lane;
    float y = mine[0];
#pragma unroll
    for (int k2 = 1; k2 < W; ++k2) y += mine[k2 * 64];
    const int tk = 4 * kb + wave;
    const int row = n0 + op_row;
    if (row < N && tk < M) {
        y /= s_tok;  // IEEE division, as the single-GEMV kernels this one stands in for
        const uint32_t o = (uint32_t)tk * (uint32_t)N + (uint32_t)row;
        if (out_f32)
            reinterpret_cast<float *>(d.out)[o] = y;
        else
            reinterpret_cast<uint16_t *>(d.out)[o] = f32_to_bf16_rne_nobranch(y);
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
using MxlKernelFn = void (*)(int, int, int, int, int, int, int, int, int, int, int, int, int, int,
                             const MxlTable);

constexpr int kMxlWideWaves = 12;

// width class: 0 = every block has one token, 1 = at most eight tokens, 2 = up to sixteen;
// dense: more than four workgroups per CU to place (only matters for width class 2)
template <int BITS, int W, int OCC1, int OCC2>
MxlKernelFn mxl_kernel_w(int scale_kind, int width_class) {
    if (scale_kind == 2) {  // int32 group sums from the same builds
        if (width_class == 0) return gemv_mxl_kernel<BITS, 1, false, W, 1, OCC1, true>;
        if (width_class == 1) return gemv_mxl_kernel<BITS, 4, false, W, 1, OCC1, true>;
        return gemv_mxl_kernel<BITS, 4, false, W, 2, OCC2, true>;
    }
    if (width_class == 0)
        return scale_kind == 1 ? gemv_mxl_kernel<BITS, 1, true, W, 1, OCC1> : gemv_mxl_kernel<BITS, 1, false, W, 1, OCC1>;
    if (width_class == 1)
        return scale_kind == 1 ? gemv_mxl_kernel<BITS, 4, true, W, 1, OCC1> : gemv_mxl_kernel<BITS, 4, false, W, 1, OCC1>;
    return scale_kind == 1 ? gemv_mxl_kernel<BITS, 4, true, W, 2, OCC2> : gemv_mxl_kernel<BITS, 4, false, W, 2, OCC2>;
}
template <int BITS>
MxlKernelFn mxl_kernel(int scale_kind, int width_class, bool wide, bool dense) {
    if (wide) return mxl_kernel_w<BITS, kMxlWideWaves, 3, 3>(scale_kind, width_class);
    return dense ? mxl_kernel_w<BITS, kMxWaves, 5, 5>(scale_kind, width_class)
                 : mxl_kernel_w<BITS, kMxWaves, 5, 4>(scale_kind, width_class);
}

template <int BITS>
int mxl_init_device(int max_lds) {
    for (int sk = 0; sk < 3; ++sk)
        for (int wc = 0; wc < 3; ++wc)
            for (int wide = 0; wide < 2; ++wide)
                for (int dense = 0; dense < 2; ++dense)
                    if (hipFuncSetAttribute(
                            reinterpret_cast<const void *>(mxl_kernel<BITS>(sk, wc, wide != 0, dense != 0)),
                            hipFuncAttributeMaxDynamicSharedMemorySize, max_lds) != hipSuccess)
                        return 2;
    return 0;
}

// True when this kernel takes the problem: what gemv_mx.hip.h takes, with at most 16 tokens and
// operand sizes within the 32-bit buffer range (q.ws may be null when group sums are wanted).
template <int BITS>
bool mxl_problem_ok(const GemvProblem &q) {
    return mx_problem_ok(q, false) && q.M <= 16 && (long)q.N * (q.K * BITS / 8) < (1L << 31) &&
           (long)q.M * q.K < (1L << 31);
}

// Launches up to kMxlMaxDesc problems, one workgroup per 16 rows.  Returns 0, -1 when the launch
// is too long or does not fit the LDS (the caller takes gemv_mx.hip.h), 2 on a launch error.
template <int BITS>
int launch_mxl(const GemvProblem *probs, int count, int out_kind, int scale_kind, int lds_limit,
               int n_cus, hipStream_t stream) {
    if (count < 1 || count > kMxlMaxDesc) return -1;
    long wgs = 0;
    int mmax = 1;
    bool one_token = true;
    for (int i = 0; i < count; ++i) {
        wgs += (probs[i].N + 15) / 16;
        mmax = probs[i].M > mmax ? probs[i].M : mmax;
        one_token = one_token && probs[i].M == 1;
    }
    // twelve waves per workgroup: one matrix with rows of at least six K tiles whose workgroups
    // find a CU each (the LDS of twelve staged tiles leaves one workgroup per CU)
    const bool wide = count == 1 && probs[0].K >= 6 * kMxTileK && wgs <= n_cus &&
                      mxl_lds_bytes<BITS>(mmax, kMxlWideWaves) <= (size_t)lds_limit;
    const int waves = wide ? kMxlWideWaves : kMxWaves;
    const size_t lds = mxl_lds_bytes<BITS>(mmax, waves);
    if (lds > (size_t)lds_limit) return -1;
    // layer-sized launches only: a few rounds of workgroups at most (longer matrices go to the
    // striding kernel, whose workgroups restage nothing they do not have to)
    if (wgs > 8L * n_cus) return -1;
    // longest K first: those workgroups run longest and should start first
    int order[kMxlMaxDesc];
    for (int i = 0; i < count; ++i) order[i] = i;
    for (int i = 1; i < count; ++i)
        for (int j = i; j > 0 && probs[order[j]].K > probs[order[j - 1]].K; --j) {
            const int t = order[j];
            order[j] = order[j - 1];
            order[j - 1] = t;
        }
    // a fifth workgroup per CU: only when the launch has one to place and the LDS holds it
    const bool dense = !wide && wgs > 4L * n_cus && 5 * lds <= (size_t)lds_limit;
    MxlTable tbl{};
    int ends[kMxlMaxDesc];
    int wg = 0;
    for (int i = 0; i < count; ++i) {
        const GemvProblem &q = probs[order[i]];
        MxlDesc &d = tbl.d[i];
        d.A = q.A;
        d.B = q.B;
        d.out = q.out;
        d.s = q.s;
        d.ws = reinterpret_cast<const uint16_t *>(q.ws);
        d.M = q.M;
        d.N = q.N;
        d.K = q.K;
        d.wg_begin = wg;
        wg += (q.N + 15) / 16;
        ends[i] = wg;
    }
    for (int i = count; i < kMxlMaxDesc; ++i) ends[i] = 0x7fffffff;
    const int width_class = one_token ? 0 : (mmax <= 8 ? 1 : 2);
    const int variant = out_kind == OUT_G32 ? 2 : scale_kind;
    hipLaunchKernelGGL(mxl_kernel<BITS>(variant, width_class, wide, dense), dim3(wg, 1, 1), dim3(waves * 64, 1, 1),
                       lds, stream, ends[0], ends[1], ends[2], ends[3], ends[4], ends[5], ends[6],
                       ends[7], ends[8], ends[9], ends[10], ends[11], out_kind == OUT_F32 ? 1 : 0,
                       mmax, tbl);
    // <BITS, MR, SF16, W, NB, OCC, G32> as instantiated by mxl_kernel
    note_kernel("gemv_mxl_kernel", BITS, width_class == 0 ? 1 : 4, scale_kind == 1 && variant != 2, waves,
                width_class == 2 ? 2 : 1, wide ? 3 : (width_class == 2 && !dense ? 4 : 5), variant == 2);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_MXL_HIP_H
