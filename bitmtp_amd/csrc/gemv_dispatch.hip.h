// Entry-point logic shared by libbonsai_t2.so and libbonsai_q1.so: argument
// checks, one-time device set-up and the choice among the kernels.  Measured on
// MI355X: the dot4 kernel (packed_gemv.hip.h) is fastest for one and two tokens
// on layer-sized matrices; from three tokens on (from two for very long matrices,
// the lm_head) the int8 matrix-core kernels (gemv_mfma.hip.h) win: the one that
// loads the activations straight as operands up to 16384 rows, the one that
// stages them in LDS once per workgroup above.  The FP4 x FP8 matrix-core kernel
// (gemv_fp4.hip.h) needs fewer VALU operations per byte but its FP8 staging and
// deeper register use make it no faster yet; it runs only when selected with the
// tuning call.  Shapes the matrix-core kernels do not take (K not a multiple of
// 512, unaligned operands, token tiles that do not fit in LDS) go to the dot4
// kernel.  Replaces the if-chain over registered (M, N, K) of the reference
// (src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:94-148).
#ifndef BONSAI_GEMV_DISPATCH_HIP_H
#define BONSAI_GEMV_DISPATCH_HIP_H

#include "gemv_fp4.hip.h"
#include "gemv_mfma.hip.h"
#include "gemv_mx.hip.h"
#include "gemv_mxs.hip.h"
#include "packed_gemv.hip.h"

namespace bonsai {

constexpr int kDefaultMfmaMinWidth = 3;       // layer-sized matrices (dot4 wins at 1 and 2 tokens)
constexpr int kDirectMaxRows = 16384;         // up to here the staging-free matrix-core kernel
constexpr int kLongMatrixRows = 32768;        // from here on the matrix cores pay off at M >= 2

template <int BITS>
int init_all_kernels() {
    const int rc = init_device<BITS>();
    if (rc != 0) return rc;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 2;
    LibState<BITS> &st = lib_state<BITS>();
    if (!st.mfma_ready[dev]) {
        const int rc2 = mfma_init_device<BITS>(st.lds_limit[dev]);
        if (rc2 != 0) return rc2;
        const int rc3 = fp4_init_device<BITS>(st.lds_limit[dev]);
        if (rc3 != 0) return rc3;
        const int rc4 = mx_init_device<BITS>(st.lds_limit[dev]);
        if (rc4 != 0) return rc4;
        const int rc5 = mxs_init_device<BITS>(st.lds_limit[dev]);
        if (rc5 != 0) return rc5;
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cus <= 0)
            return 2;
        st.n_cus[dev] = cus;
        st.mfma_ready[dev] = true;
    }
    return 0;
}

// Launches one of the matrix-core kernels (engine 1 staged int8, 2 FP4 x FP8, 3 direct int8).  Returns -1 when the shape does not
// fit (the caller falls back), 0 on success, 2 on a launch error.  `single_tile`
// refuses shapes whose tokens would need more than ceil(M/16) token tiles, i.e.
// a second pass over the weights.
template <int BITS>
int launch_matrix_core(int engine, bool single_tile, const int8_t *A, const uint8_t *B, void *out,
                       const float *s, const void *ws, int M, int N, int K, int out_kind,
                       int scale_kind, int lds_limit, hipStream_t stream) {
    const MfmaTuning &tu = mfma_tuning<BITS>();
    const bool fp4 = engine == 2, direct = engine == 3;
    int nw = 4;  // waves per workgroup; eight only for the direct kernel on long rows
    auto lds_for = [&](int ri, int mt) {
        return fp4 ? fp4_lds_for<BITS>(ri, mt, K)
                   : (direct ? mfma_direct_lds_for<BITS>(ri, nw) : mfma_lds_for<BITS>(ri, mt, K));
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
    const int per_token = fp4 ? K / 32 : K / mfma_quarter_bytes<BITS>();  // staging tasks per token
    args.div_magic = (uint32_t)(0x100000000ull / (uint64_t)per_token) + 1u;

    const int rows_per_wg = 16 * R * (nw / ks) * passes;
    const int grid_x = (N + rows_per_wg - 1) / rows_per_wg;
    const int variant = out_kind == OUT_G32 ? 2 : scale_kind;
    const MfmaKernelFn fn = fp4 ? fp4_table<BITS>().fn[ri][variant]
                                : (flex ? mfma_direct_flex_table<BITS>().fn[0][variant]
                                   : direct ? (nw == 8 ? mfma_direct8_table<BITS>().fn[ri][variant]
                                                       : mfma_direct_table<BITS>().fn[ri][variant])
                                            : mfma_table<BITS>().fn[ri][variant]);
    hipLaunchKernelGGL(fn, dim3(grid_x, ntok_tiles, 1), dim3(nw * 64, 1, 1), lds_for(ri, mt),
                       stream, args.A, args.B, args.out, args.s, args.ws, args.M, args.N, args.K,
                       args.mt, args.ks_log2, args.out_f32, args.passes, args.div_magic);
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

    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 2;
    LibState<BITS> &st = lib_state<BITS>();
    if (st.lds_limit[dev] == 0 || !st.mfma_ready[dev]) {
        const int rc = init_all_kernels<BITS>();
        if (rc != 0) return rc;
    }
    const int lds_limit = st.lds_limit[dev];

    const MfmaTuning &mtu = mfma_tuning<BITS>();
    const int min_width = mtu.min_width > 0 ? mtu.min_width
                                            : (N >= kLongMatrixRows ? 2 : kDefaultMfmaMinWidth);
    if (mtu.engine == 5 || mtu.engine == 0) {
        // very long matrices: the streaming kernel, at every width up to 16
        const GemvProblem q{A, B, out, s, ws, M, N, K};
        if (mxs_problem_ok<BITS>(q, out_kind, lds_limit, st.n_cus[dev], mtu.engine == 5))
            return launch_mxs<BITS>(q, out_kind, scale_kind, lds_limit, st.n_cus[dev], stream);
    }
    if (mtu.engine == 4 && M >= min_width) {
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
        if (engine == 2 || engine == 3)
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

// Several GEMVs in one call (descriptors in host memory, read before the call returns).
// Problems the grouped kernel takes (K % 512 == 0, aligned operands) share launches of up to
// kMxMaxDesc descriptors each, blocks wider than 16 tokens as several token tiles; the rest
// go through launch_gemv one by one.  The arithmetic of every problem is that of the
// single-GEMV entry points.
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
    }
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 2;
    LibState<BITS> &st = lib_state<BITS>();
    if (st.lds_limit[dev] == 0 || !st.mfma_ready[dev]) {
        const int rc = init_all_kernels<BITS>();
        if (rc != 0) return rc;
    }
    const int lds_limit = st.lds_limit[dev];
    const MxTuning &tu = mx_tuning<BITS>();
    const int min_width = tu.min_width > 0 ? tu.min_width : 1;

    GemvProblem batch[kMxMaxDesc];
    int nb = 0;
    auto flush = [&]() -> int {
        if (nb == 0) return 0;
        const int rc = launch_mx<BITS>(batch, nb, out_kind, scale_kind, lds_limit, st.n_cus[dev], stream);
        nb = 0;
        return rc;
    };
    const size_t out_elt = out_kind == OUT_BF16 ? 2 : 4;
    for (int i = 0; i < count; ++i) {
        const GemvProblem &q = probs[i];
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
    const int rc = flush();
    return rc < 0 ? 2 : rc;
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_DISPATCH_HIP_H
