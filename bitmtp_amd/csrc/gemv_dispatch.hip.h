// Entry-point logic shared by libbonsai_t2.so and libbonsai_q1.so: argument
// checks, one-time device set-up and the choice among the kernels.  Measured on
// MI355X: the dot4 kernel (packed_gemv.hip.h) is fastest for one and two tokens
// on layer-sized matrices; from three tokens on (from two for very long matrices,
// the lm_head) the int8 matrix-core kernels (gemv_mfma.hip.h) win: the one that
// loads the activations straight as operands up to 16384 rows, the one that
// stages them in LDS once per workgroup above; one token against a very long matrix
// has a kernel of its own (gemv_rowreg.hip.h), wider blocks there take the streaming
// matrix-core kernel (gemv_mxs.hip.h).  Shapes the matrix-core kernels do not take (K not a multiple of
// 512, unaligned operands, token tiles that do not fit in LDS) go to the dot4
// kernel.  Replaces the if-chain over registered (M, N, K) of the reference
// (src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:94-148).
#ifndef BONSAI_GEMV_DISPATCH_HIP_H
#define BONSAI_GEMV_DISPATCH_HIP_H

#include "gemv_mfma.hip.h"
#include "gemv_mx.hip.h"
#include "gemv_mxl.hip.h"
#include "gemv_mxs.hip.h"
#include "gemv_rowreg.hip.h"
#include "packed_gemv.hip.h"

namespace bonsai {

constexpr int kDefaultMfmaMinWidth = 3;       // layer-sized matrices (dot4 wins at 1 and 2 tokens)
constexpr int kDirectMaxRows = 16384;         // up to here the staging-free matrix-core kernel
constexpr int kLongMatrixRows = 32768;        // from here on the matrix cores pay off at M >= 2

// Every kernel reads A and B with 16-byte vector loads and the scales as 16-bit words.
inline bool operands_aligned(const void *A, const void *B, const void *out, const void *s,
                             const void *ws, int out_kind) {
    const auto mis = [](const void *p, uintptr_t a) {
        return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0;
    };
    return !(mis(A, 16) || mis(B, 16) || mis(out, out_kind == OUT_BF16 ? 2 : 4) ||
             (s != nullptr && mis(s, 4)) || (ws != nullptr && mis(ws, 2)));
}

// ---- grouped dot4 launch (narrow blocks) -------------------------------------------------
constexpr int kDot4GroupMaxWidth = 2;  // widest block the grouped dot4 kernel takes

using Dot4GroupFn = void (*)(int, int, int, int, int, int, int, int, int, int, int, int, int, int,
                             const Dot4GroupTable);

template <int BITS>
struct Dot4GroupKernels {
    Dot4GroupFn fn[kDot4GroupMaxWidth][kBatchKinds][kVariants];  // [MT - 1][U index][bf16 / fp16 scales / group sums]
};

template <int BITS, int MT, int U, int UI>
void fill_dot4_group_cell(Dot4GroupKernels<BITS> &x) {
    x.fn[MT - 1][UI][0] = gemv_dot4_grouped_kernel<BITS, MT, U, false, false>;
    x.fn[MT - 1][UI][1] = gemv_dot4_grouped_kernel<BITS, MT, U, true, false>;
    x.fn[MT - 1][UI][2] = gemv_dot4_grouped_kernel<BITS, MT, U, false, true>;
}

template <int BITS>
const Dot4GroupKernels<BITS> &dot4_group_kernels() {
    static const Dot4GroupKernels<BITS> t = [] {
        Dot4GroupKernels<BITS> x{};
        fill_dot4_group_cell<BITS, 1, 1, 0>(x);
        fill_dot4_group_cell<BITS, 1, 2, 1>(x);
        fill_dot4_group_cell<BITS, 1, 4, 2>(x);
        fill_dot4_group_cell<BITS, 2, 1, 0>(x);
        fill_dot4_group_cell<BITS, 2, 2, 1>(x);
        fill_dot4_group_cell<BITS, 2, 2, 2>(x);  // (never picked: two tokens take at most two loads per batch)
        return x;
    }();
    return t;
}

template <int BITS>
int dot4_group_init_device(int max_lds) {
    const Dot4GroupKernels<BITS> &t = dot4_group_kernels<BITS>();
    for (int mt = 0; mt < kDot4GroupMaxWidth; ++mt)
        for (int u = 0; u < kBatchKinds; ++u)
            for (int sk = 0; sk < kVariants; ++sk)
                if (hipFuncSetAttribute(reinterpret_cast<const void *>(t.fn[mt][u][sk]),
                                        hipFuncAttributeMaxDynamicSharedMemorySize,
                                        max_lds) != hipSuccess)
                    return 2;
    return 0;
}

// Launches up to kDot4GroupMax problems of at most kDot4GroupMaxWidth tokens each with the
// grouped dot4 kernel.  Lanes per row and passes are each problem's own (pick_geometry); the
// token tile, the loads per batch and the workgroup size are common to the launch (the widest
// block, the shortest batch and the smaller workgroup any problem asks for).  Returns 0, -1
// when a problem does not fit (the caller falls back), 2 on a launch error.
template <int BITS>
int launch_dot4_grouped(const GemvProblem *probs, int count, int out_kind, int scale_kind,
                        int lds_limit, hipStream_t stream) {
    if (count < 1 || count > kDot4GroupMax) return -1;
    int mt = 1;
    for (int i = 0; i < count; ++i) mt = probs[i].M > mt ? probs[i].M : mt;
    if (mt > kDot4GroupMaxWidth) return -1;
    // longest rows first: their workgroups run longest and should start first
    int order[kDot4GroupMax];
    for (int i = 0; i < count; ++i) order[i] = i;
    for (int i = 1; i < count; ++i)
        for (int j = i; j > 0 && probs[order[j]].K > probs[order[j - 1]].K; --j) {
            const int t = order[j];
            order[j] = order[j - 1];
            order[j - 1] = t;
        }
    Geometry geo[kDot4GroupMax];
    int waves = 8, batch_index = kBatchKinds - 1;
    size_t lds = 0;
    // A launch of several matrices has waves enough without spreading every row over many
    // lanes: eight lanes per row (four for 1-bit rows), sixteen once that leaves a lane eight
    // chunks or more, four waves per workgroup.  Sweeps over the seven projections of a layer at
    // one token: 1.7B-shaped 5.04 us (8 lanes for K = 2048, 16 for K = 6144) against 5.4 us with
    // 16 / 16, 5.2-5.3 us with 16 / 32 or 16 / 64 and 6.4 us with each matrix's own
    // single-launch geometry; 4B-shaped 8.4 against 8.8 us, Q1 7.3 against 7.4 us.
    Tuning tu = lib_state<BITS>().tuning;
    const bool own_rule = tu.lanes_per_row == 0 && tu.waves_per_wg == 0 && count > 1;
    for (int i = 0; i < count; ++i) {
        const GemvProblem &q = probs[order[i]];
        Tuning t = tu;
        if (own_rule) {
            const int C = q.K / Fmt<BITS>::kChunkWeights;
            int lpr = BITS == 1 ? 4 : 8;
            while (lpr < 16 && 4 * lpr * 2 <= C) lpr *= 2;
            t.lanes_per_row = lpr;
            t.waves_per_wg = 4;
        }
        geo[i] = pick_geometry<BITS>(mt, q.N, q.K, lds_limit, t);
        if (geo[i].mt != mt) return -1;  // the token tile does not fit the LDS
        waves = geo[i].waves < waves ? geo[i].waves : waves;
        batch_index = geo[i].batch_index < batch_index ? geo[i].batch_index : batch_index;
        lds = geo[i].lds > lds ? geo[i].lds : lds;
    }
    Dot4GroupTable tbl{};
    int ends[kDot4GroupMax];
    int wg = 0;
    for (int i = 0; i < count; ++i) {
        const GemvProblem &q = probs[order[i]];
        Dot4GroupDesc &d = tbl.d[i];
        d.A = q.A;
        d.B = q.B;
        d.out = q.out;
        d.s = q.s;
        d.ws = reinterpret_cast<const uint16_t *>(q.ws);
        d.M = q.M;
        d.N = q.N;
        d.K = q.K;
        d.wg_begin = wg;
        d.lpr_log2_passes = geo[i].lpr_log2 | (geo[i].passes << 8);
        d.div_magic = (uint32_t)(0x100000000ull / (uint64_t)(4 * (q.K / Fmt<BITS>::kChunkWeights))) + 1u;
        const long rows_per_wg = (long)(64 >> geo[i].lpr_log2) * waves * geo[i].passes;
        wg += (int)(((long)q.N + rows_per_wg - 1) / rows_per_wg);
        ends[i] = wg;
    }
    for (int i = count; i < kDot4GroupMax; ++i) ends[i] = 0x7fffffff;
    const Dot4GroupFn fn = dot4_group_kernels<BITS>().fn[mt - 1][batch_index][out_kind == OUT_G32 ? 2 : scale_kind];
    hipLaunchKernelGGL(fn, dim3(wg, 1, 1), dim3(waves * 64, 1, 1), lds, stream, ends[0], ends[1],
                       ends[2], ends[3], ends[4], ends[5], ends[6], ends[7], ends[8], ends[9],
                       ends[10], ends[11], out_kind == OUT_F32 ? 1 : 0, waves * 64, tbl);
    note_kernel("gemv_dot4_grouped_kernel", BITS, mt, batch_index == 2 && mt == 1 ? 4 : (batch_index >= 1 ? 2 : 1),
                scale_kind == 1 && out_kind != OUT_G32, out_kind == OUT_G32);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

// One-time set-up of every kernel on the current device, under a lock: two host threads that
// launch at the same moment initialise once.  The ready flag is written last.
template <int BITS>
int init_all_kernels() {
    LibState<BITS> &st = lib_state<BITS>();
    std::lock_guard<std::mutex> guard(st.init_mutex);
    const int rc = init_device<BITS>();
    if (rc != 0) return rc;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 2;
    if (!st.mfma_ready[dev].load(std::memory_order_acquire)) {
        const int rc2 = mfma_init_device<BITS>(st.lds_limit[dev]);
        if (rc2 != 0) return rc2;
        const int rc4 = mx_init_device<BITS>(st.lds_limit[dev]);
        if (rc4 != 0) return rc4;
        const int rc5 = mxs_init_device<BITS>(st.lds_limit[dev]);
        if (rc5 != 0) return rc5;
        const int rc6 = dot4_group_init_device<BITS>(st.lds_limit[dev]);
        if (rc6 != 0) return rc6;
        const int rc7 = mxl_init_device<BITS>(st.lds_limit[dev]);
        if (rc7 != 0) return rc7;
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cus <= 0)
            return 2;
        st.n_cus[dev] = cus;
        st.mfma_ready[dev].store(true, std::memory_order_release);
    }
    return 0;
}

// Set-up on first use.  A first launch on a capturing stream is refused (status 3) instead of
// changing kernel attributes under capture: call *_init before capturing.
template <int BITS>
int ensure_ready(int dev, hipStream_t stream) {
    LibState<BITS> &st = lib_state<BITS>();
    if (st.mfma_ready[dev].load(std::memory_order_acquire)) return 0;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) return 3;
    return init_all_kernels<BITS>();
}

// Launches one of the matrix-core kernels (engine 1 staged int8, 3 direct int8).  Returns -1 when the shape does not
// fit (the caller falls back), 0 on success, 2 on a launch error.  `single_tile`
// refuses shapes whose tokens would need more than ceil(M/16) token tiles, i.e.
// a second pass over the weights.
template <int BITS>
int launch_matrix_core(int engine, bool single_tile, const int8_t *A, const uint8_t *B, void *out,
                       const float *s, const void *ws, int M, int N, int K, int out_kind,
                       int scale_kind, int lds_limit, hipStream_t stream) {
    const MfmaTuning &tu = mfma_tuning<BITS>();
    const bool direct = engine == 3;
    int nw = 4;  // waves per workgroup; eight only for the direct kernel on long rows
    auto lds_for = [&](int ri, int mt) {
        return direct ? mfma_direct_lds_for<BITS>(ri, nw) : mfma_lds_for<BITS>(ri, mt, K);
    };
    int ntok_tiles = (M + kMfmaTokens - 1) / kMfmaTokens;
    int mt = (M + ntok_tiles - 1) / ntok_tiles;
    while (lds_for(0, mt) > (size_t)lds_limit) {
        if (single_tile || mt == 1) return -1;
        ++ntok_tiles;
        mt = (M + ntok_tiles - 1) / ntok_tiles;
    }

    // K split among the waves of a workgroup for short matrices, more row tiles per
    // wave and several row blocks per workgroup for long ones.
    int ks = tu.k_split;
    int R = tu.row_tiles;
    const int ntiles = K / 512;
    if (ks == 0) {
        if (direct)  // no staging to amortise: split K as far as it goes; eight waves per
                     // workgroup only while that leaves at most about one workgroup per CU
            ks = (ntiles >= 8 && N <= 4096) ? 8 : (ntiles >= 4 ? 4 : (ntiles >= 2 ? 2 : 1));
        else
            ks = (N <= 4096 && ntiles >= 4) ? 4 : ((N <= 16384 && ntiles >= 2) ? 2 : 1);
    }
    // Tile counts that are no power of two (K = 2560, 6144, 9728 ...) on matrices of at most
    // 4096 rows (about one workgroup per CU: with more workgroups this form measured slower
    // than a split of four): the direct kernel in its one-slice-per-wave form, one tile per
    // wave up to twelve waves.  A tuning override of the split in 3..12 other than 4 and 8
    // selects this form as well.
    bool flex = false;
    if (direct && (tu.row_tiles == 0 || tu.row_tiles == 1)) {
        if (tu.k_split == 0 && (ntiles & (ntiles - 1)) != 0 && ntiles >= 3) {
            if (N <= 4096) {
                flex = true;
                ks = ntiles < kMfmaFlexMaxWaves ? ntiles : kMfmaFlexMaxWaves;
            }
        } else if (tu.k_split >= 3 && tu.k_split <= kMfmaFlexMaxWaves && tu.k_split != 4 &&
                   tu.k_split != 8 && tu.k_split <= ntiles) {
            flex = true;
            ks = tu.k_split;
        }
    }
    if (!flex && ks != 1 && ks != 2 && ks != 4 && !(ks == 8 && direct)) ks = 1;
    // slices may be uneven (tile t goes to slice floor-partition): every wave still reaches the
    // single barrier after its K loop; an empty slice is never scheduled
    if (ks > ntiles) ks = 1;
    if (ks == 8) nw = 8;
    if (flex) {
        nw = ks;
        R = 1;
    }
    if (R == 0) {
        const long wgs1 = ((long)N + 16 * (nw / ks) - 1) / (16 * (nw / ks));  // workgroups at R = 1
        R = wgs1 >= 8192 ? 4 : (wgs1 >= 2048 ? 2 : 1);
        // long rows walked tile after tile: two row tiles per wave double the bytes in flight
        if (direct && R == 1 && ntiles / ks >= 4 && wgs1 >= 512) R = 2;
    }
    int ri = R >= 4 ? 2 : (R >= 2 ? 1 : 0);
    while (ri > 0 && lds_for(ri, mt) > (size_t)lds_limit) --ri;
    R = 1 << ri;

    int passes = 1;
    if (ks == 1) {
        passes = tu.passes;
        if (passes == 0) {
            const long blocks = ((long)N + 64 * R - 1) / (64 * R);
            passes = blocks >= 4096 ? 4 : (blocks >= 2048 ? 2 : 1);
        }
        if (passes < 1) passes = 1;
    }

    MfmaArgs args;
    args.A = A;
    args.B = B;
    args.out = out;
    args.s = s;
    args.ws = reinterpret_cast<const uint16_t *>(ws);
    args.M = M;
    args.N = N;
    args.K = K;
    args.mt = mt;
    args.ks_log2 = flex ? ks : (ks == 8 ? 3 : (ks == 4 ? 2 : (ks == 2 ? 1 : 0)));
    args.out_f32 = out_kind == OUT_F32 ? 1 : 0;
    args.passes = passes;
    const int per_token = K / mfma_quarter_bytes<BITS>();  // staging tasks per token
    args.div_magic = (uint32_t)(0x100000000ull / (uint64_t)per_token) + 1u;

    const int rows_per_wg = 16 * R * (nw / ks) * passes;
    const int grid_x = (N + rows_per_wg - 1) / rows_per_wg;
    const int variant = out_kind == OUT_G32 ? 2 : scale_kind;
    const MfmaKernelFn fn = flex ? mfma_direct_flex_table<BITS>().fn[0][variant]
                            : direct ? (nw == 8 ? mfma_direct8_table<BITS>().fn[ri][variant]
                                                : mfma_direct_table<BITS>().fn[ri][variant])
                                     : mfma_table<BITS>().fn[ri][variant];
    hipLaunchKernelGGL(fn, dim3(grid_x, ntok_tiles, 1), dim3(nw * 64, 1, 1), lds_for(ri, mt),
                       stream, args.A, args.B, args.out, args.s, args.ws, args.M, args.N, args.K,
                       args.mt, args.ks_log2, args.out_f32, args.passes, args.div_magic);
    note_kernel(flex ? "gemv_mfma_direct_flex_kernel" : (direct ? (nw == 8 ? "gemv_mfma_direct8_kernel" : "gemv_mfma_direct_kernel")
                                                                : "gemv_mfma_kernel"),
                BITS, 1 << ri, variant == 1, variant == 2);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

// One problem through the grouped kernel (token tiles of at most 16 as separate descriptors).
// Returns -1 when it does not fit.
template <int BITS>
int launch_grouped_mx_only(const GemvProblem &q, int out_kind, int scale_kind, int lds_limit,
                           int n_cus, hipStream_t stream) {
    // (the staged activations are chunked along K, so any block of up to 16 tokens fits in LDS)
    const int cap = q.M < kMfmaTokens ? q.M : kMfmaTokens;
    const int ntt = (q.M + cap - 1) / cap;
    if (ntt > kMxMaxDesc) return -1;
    const int mt = (q.M + ntt - 1) / ntt;
    const size_t out_elt = out_kind == OUT_BF16 ? 2 : 4;
    GemvProblem batch[kMxMaxDesc];
    int nb = 0;
    for (int m0 = 0; m0 < q.M; m0 += mt) {
        GemvProblem sub = q;
        sub.M = (q.M - m0) < mt ? (q.M - m0) : mt;
        sub.A = q.A + (size_t)m0 * q.K;
        sub.s = q.s == nullptr ? nullptr : q.s + m0;
        const size_t per_tok = out_kind == OUT_G32 ? (size_t)q.N * (q.K / kGroup) : (size_t)q.N;
        sub.out = static_cast<unsigned char *>(q.out) + (size_t)m0 * per_tok * out_elt;
        batch[nb++] = sub;
    }
    // the lean form where it applies (every token tile of at most 16, a layer-sized matrix)
    const MxTuning &gtu = mx_tuning<BITS>();
    if (nb <= kMxlMaxDesc && gtu.row_tiles == 0 && gtu.max_wgs == 0) {
        bool ok = true;
        for (int i = 0; i < nb; ++i) ok = ok && mxl_problem_ok<BITS>(batch[i]);
        if (ok) {
            const int rc = launch_mxl<BITS>(batch, nb, out_kind, scale_kind, lds_limit, n_cus, stream);
            if (rc != -1) return rc;
        }
    }
    return launch_mx<BITS>(batch, nb, out_kind, scale_kind, lds_limit, n_cus, stream);
}

template <int BITS>
int launch_gemv(const int8_t *A, const uint8_t *B, void *out, const float *s, const void *ws,
                int M, int N, int K, int out_kind, int scale_kind, hipStream_t stream) {
    if (A == nullptr || B == nullptr || out == nullptr) return 1;
    if (out_kind < 0 || out_kind > 2 || scale_kind < 0 || scale_kind > 1) return 1;
    if (out_kind != OUT_G32 && (s == nullptr || ws == nullptr)) return 1;
    if (M < 1 || N < 1 || K < kGroup || K % kGroup != 0) return 1;
    if ((long)M * N > 0x7fffffffL / 2) return 1;  // row indices are 32-bit
    if (!operands_aligned(A, B, out, s, ws, out_kind)) return 1;

    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 2;
    LibState<BITS> &st = lib_state<BITS>();
    {
        const int rc = ensure_ready<BITS>(dev, stream);
        if (rc != 0) return rc;
    }
    const int lds_limit = st.lds_limit[dev];

    const MfmaTuning &mtu = mfma_tuning<BITS>();
    // two tokens go to the matrix cores for very long matrices and for long rows (K >= 4096: at
    // two tokens 2048 x 6144 takes 3.74 us there against 4.23 us on the dot4 kernel, 2560 x 9728
    // 4.77 against 5.91; K = 2048 and 2560 are level or slower)
    const int min_width = mtu.min_width > 0 ? mtu.min_width
                                            : (N >= kLongMatrixRows || K >= 4096 ? 2 : kDefaultMfmaMinWidth);
    if constexpr (BITS == 2) {
        if (mtu.engine == 6 || mtu.engine == 0) {
            // one token against a very long matrix: activations in registers, v_dot8
            const GemvProblem q{A, B, out, s, ws, M, N, K};
            if (rowreg_problem_ok(q, out_kind, mtu.engine == 6))
                return launch_rowreg(q, out_kind, scale_kind, st.n_cus[dev],
                                     mxs_tuning<BITS>().wgs_per_cu, stream);
        }
    }
    if (mtu.engine == 5 || mtu.engine == 0) {
        // very long matrices: the streaming kernel, at every width up to 16
        const GemvProblem q{A, B, out, s, ws, M, N, K};
        if (mxs_problem_ok<BITS>(q, out_kind, lds_limit, st.n_cus[dev], mtu.engine == 5))
            return launch_mxs<BITS>(q, out_kind, scale_kind, lds_limit, st.n_cus[dev], stream);
    }
    // Layer-sized matrices at three or more tokens: the lean grouped kernel with one descriptor per
    // tile of up to 16 tokens, as long as its grid stays within eight workgroups per CU.  Measured
    // against the operand-loading and the staged kernel at widths 3-16: 8-15 % faster on the
    // K = 2048 / 2560 decode shapes of the 1.7B- and 4B-shaped models, 15-25 % on 12288 x 4096,
    // 9728 x 9728, 24576 x 4096 and 27648 x 5120, level on 4096 x 12288 (where the twelve-wave
    // form of the same kernel already ran).
    const long lean_tiles = (long)((M + kMfmaTokens - 1) / kMfmaTokens) * ((N + 15) / 16);
    const bool lean_default = mtu.engine == 0 && M >= min_width && N <= kLongMatrixRows &&
                              lean_tiles <= 8L * st.n_cus[dev];
    if ((mtu.engine == 4 || lean_default) && M >= min_width) {
        // the grouped kernel with a single descriptor
        const GemvProblem q{A, B, out, s, ws, M, N, K};
        if (mx_problem_ok(q, out_kind == OUT_G32)) {
            const int rc = launch_grouped_mx_only<BITS>(q, out_kind, scale_kind, lds_limit, st.n_cus[dev],
                                                        stream);
            if (rc >= 0) return rc;
        }
    }
    if (M >= min_width && mfma_shape_ok(B, out_kind == OUT_G32 ? nullptr : ws, K)) {
        int rc = -1;
        // operand-loaded activations win up to about 16k rows, staged ones above (measured)
        const int engine = mtu.engine != 0 ? mtu.engine : (N <= kDirectMaxRows ? 3 : 1);
        if (engine == 3)
            rc = launch_matrix_core<BITS>(engine, false, A, B, out, s, ws, M, N, K, out_kind,
                                          scale_kind, lds_limit, stream);
        if (rc < 0)
            rc = launch_matrix_core<BITS>(1, false, A, B, out, s, ws, M, N, K, out_kind,
                                          scale_kind, lds_limit, stream);
        if (rc >= 0) return rc;
    }
    return launch_gemv_dot4<BITS>(A, B, out, s, ws, M, N, K, out_kind, scale_kind, lds_limit,
                                  stream);
}

// ---- fused forms for blocks of one or two tokens (see packed_gemv.hip.h) ----------------------
constexpr int kFusedMaxWidth = kFusedMaxTile;

template <int BITS>
int fused_ready(int M, int N, int K, hipStream_t stream, int *lds_limit, int *n_cus) {
    if (M < 1 || M > kFusedMaxWidth || N < 1 || K < kGroup || K % kGroup != 0) return 1;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 2;
    const int rc = ensure_ready<BITS>(dev, stream);
    if (rc != 0) return rc;
    *lds_limit = lib_state<BITS>().lds_limit[dev];
    *n_cus = lib_state<BITS>().n_cus[dev];
    return 0;
}

// Parts per token that a fused launch with this epilogue writes for this shape (its workgroup
// count), or a negative status: -1 the shape is not taken, -2 / -3 as the launch statuses 2 / 3.
template <int BITS>
int fused_parts(int epi, int M, int N, int K) {
    if (epi != EPI_SILU_PAIR && epi != EPI_ADD_SUMSQ) return -1;
    if (epi == EPI_SILU_PAIR && (N < 2 || (N & 1))) return -1;
    int lds_limit = 0, n_cus = 0;
    const int rc = fused_ready<BITS>(M, N, K, nullptr, &lds_limit, &n_cus);
    if (rc != 0) return -rc;
    const Geometry g = fused_geometry<BITS>(PRO_INT8, epi, M, N, K, lds_limit, n_cus);
    return g.mt == 0 ? -1 : g.grid_x;
}

// Validates and launches one fused GEMV.
template <int BITS>
int launch_gemv_fused(const FusedGemv &d, hipStream_t stream) {
    const auto mis = [](const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; };
    if (d.pro < PRO_INT8 || d.pro > PRO_BF16_NORM || d.epi < EPI_PLAIN || d.epi > EPI_ADD_SUMSQ) return 1;
    if (d.pro == PRO_INT8 && d.epi == EPI_PLAIN) return 1;  // that is *_gemv_ex
    if (d.act == nullptr || d.B == nullptr || d.ws == nullptr || d.out == nullptr || d.act_aux == nullptr) return 1;
    if (mis(d.act, 16) || mis(d.B, 16) || mis(d.ws, 2)) return 1;
    if (d.pro == PRO_INT8) {
        if (mis(d.act_aux, 4)) return 1;
    } else if (d.pro == PRO_BF16_AMAX) {
        if (mis(d.act_aux, 16) || d.act_parts < 1 || d.act_parts > kAmaxMaxParts) return 1;
    } else {
        if (mis(d.act_aux, 8) || d.act_parts < 1 || d.act_parts > kSumsqMaxParts) return 1;
        if (d.norm_w == nullptr || mis(d.norm_w, 16) || !(d.eps >= 0.0f)) return 1;
    }
    if (d.s_out != nullptr && (d.pro == PRO_INT8 || mis(d.s_out, 4))) return 1;
    if (d.epi == EPI_PLAIN) {
        if ((d.out_kind != OUT_BF16 && d.out_kind != OUT_F32) || mis(d.out, d.out_kind == OUT_BF16 ? 2 : 4)) return 1;
    } else {
        if (d.out_kind != OUT_BF16 || mis(d.out, 2) || d.out_aux == nullptr) return 1;
        if (d.epi == EPI_SILU_PAIR && (d.N < 2 || (d.N & 1) || mis(d.out_aux, 16))) return 1;
        if (d.epi == EPI_ADD_SUMSQ && (d.residual == nullptr || mis(d.residual, 2) || mis(d.out_aux, 8))) return 1;
    }
    int lds_limit = 0, n_cus = 0;
    const int rc = fused_ready<BITS>(d.M, d.N, d.K, stream, &lds_limit, &n_cus);
    if (rc != 0) return rc;
    return launch_gemv_dot4_fused<BITS>(d, lds_limit, n_cus, stream);
}

// Several GEMVs in one call (descriptors in host memory, read before the call returns).
// Problems the grouped kernel takes (K % 512 == 0, aligned operands) share launches of up to
// kMxMaxDesc descriptors each, blocks wider than 16 tokens as several token tiles; the rest
// go through launch_gemv one by one.  The arithmetic of every problem is that of the
// single-GEMV entry points: identical int32 group sums; the fp32 value has the same bits where
// the same kernel and geometry serve both, and differs by summation order only elsewhere.
template <int BITS>
int launch_grouped(const GemvProblem *probs, int count, int out_kind, int scale_kind,
                   hipStream_t stream) {
    if (probs == nullptr || count < 1) return 1;
    if (out_kind < 0 || out_kind > 2 || scale_kind < 0 || scale_kind > 1) return 1;
    for (int i = 0; i < count; ++i) {
        const GemvProblem &q = probs[i];
        if (q.A == nullptr || q.B == nullptr || q.out == nullptr) return 1;
        if (out_kind != OUT_G32 && (q.s == nullptr || q.ws == nullptr)) return 1;
        if (q.M < 1 || q.N < 1 || q.K < kGroup || q.K % kGroup != 0) return 1;
        if ((long)q.M * q.N > 0x7fffffffL / 2) return 1;
        if (!operands_aligned(q.A, q.B, q.out, q.s, q.ws, out_kind)) return 1;
    }
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 2;
    LibState<BITS> &st = lib_state<BITS>();
    {
        const int rc = ensure_ready<BITS>(dev, stream);
        if (rc != 0) return rc;
    }
    const int lds_limit = st.lds_limit[dev];
    const MxTuning &tu = mx_tuning<BITS>();
    const int min_width = tu.min_width > 0 ? tu.min_width : 1;

    GemvProblem batch[kMxMaxDesc];
    int nb = 0;
    auto flush = [&]() -> int {
        if (nb == 0) return 0;
        int rc = -1;
        // the lean form where the launch is resident at once (tu.row_tiles or tu.max_wgs set:
        // the striding kernel is being steered by hand)
        if (nb <= kMxlMaxDesc && tu.row_tiles == 0 && tu.max_wgs == 0) {
            bool ok = true;
            for (int i = 0; i < nb; ++i) ok = ok && mxl_problem_ok<BITS>(batch[i]);
            if (ok) rc = launch_mxl<BITS>(batch, nb, out_kind, scale_kind, lds_limit, st.n_cus[dev], stream);
        }
        if (rc == -1)
            rc = launch_mx<BITS>(batch, nb, out_kind, scale_kind, lds_limit, st.n_cus[dev], stream);
        if (rc == -1) {  // no grouped kernel takes the batch: its problems one by one
            rc = 0;
            for (int i = 0; i < nb && rc == 0; ++i)
                rc = launch_gemv<BITS>(batch[i].A, batch[i].B, batch[i].out, batch[i].s, batch[i].ws,
                                       batch[i].M, batch[i].N, batch[i].K, out_kind, scale_kind, stream);
        }
        nb = 0;
        return rc;
    };
    // Blocks of one or two tokens: the grouped dot4 kernel, twelve problems per launch
    // (a forced smallest width of the matrix-core kernel, tu.min_width > 0, keeps them there)
    GemvProblem nbatch[kDot4GroupMax];
    int nnb = 0;
    const bool narrow_on = tu.min_width <= 0;
    auto flush_n = [&]() -> int {
        if (nnb == 0) return 0;
        int rc = launch_dot4_grouped<BITS>(nbatch, nnb, out_kind, scale_kind, lds_limit, stream);
        if (rc == -1) {  // did not fit: one by one
            rc = 0;
            for (int i = 0; i < nnb && rc == 0; ++i)
                rc = launch_gemv<BITS>(nbatch[i].A, nbatch[i].B, nbatch[i].out, nbatch[i].s, nbatch[i].ws,
                                       nbatch[i].M, nbatch[i].N, nbatch[i].K, out_kind, scale_kind, stream);
        }
        nnb = 0;
        return rc;
    };
    const size_t out_elt = out_kind == OUT_BF16 ? 2 : 4;
    for (int i = 0; i < count; ++i) {
        const GemvProblem &q = probs[i];
        if (narrow_on && q.M <= kDot4GroupMaxWidth) {
            nbatch[nnb++] = q;
            if (nnb == kDot4GroupMax) {
                const int rc = flush_n();
                if (rc != 0) return rc;
            }
            continue;
        }
        // token tiles of at most 16 (the staged activations are chunked along K: they always fit)
        const int cap = q.M < kMfmaTokens ? q.M : kMfmaTokens;
        if (q.M < min_width || !mx_problem_ok(q, out_kind == OUT_G32)) {
            const int rc = launch_gemv<BITS>(q.A, q.B, q.out, q.s, q.ws, q.M, q.N, q.K, out_kind,
                                             scale_kind, stream);
            if (rc != 0) return rc;
            continue;
        }
        const int ntt = (q.M + cap - 1) / cap;
        const int mt = (q.M + ntt - 1) / ntt;
        for (int m0 = 0; m0 < q.M; m0 += mt) {
            GemvProblem sub = q;
            sub.M = (q.M - m0) < mt ? (q.M - m0) : mt;
            sub.A = q.A + (size_t)m0 * q.K;
            sub.s = q.s == nullptr ? nullptr : q.s + m0;
            const size_t per_tok = out_kind == OUT_G32 ? (size_t)q.N * (q.K / kGroup) : (size_t)q.N;
            sub.out = static_cast<unsigned char *>(q.out) + (size_t)m0 * per_tok * out_elt;
            batch[nb++] = sub;
            if (nb == kMxMaxDesc) {
                const int rc = flush();
                if (rc != 0) return rc < 0 ? 2 : rc;
            }
        }
    }
    const int rcn = flush_n();
    if (rcn != 0) return rcn;
    const int rc = flush();
    return rc < 0 ? 2 : rc;
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_DISPATCH_HIP_H
