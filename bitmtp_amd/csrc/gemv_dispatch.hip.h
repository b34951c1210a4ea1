// Entry-point logic shared by libbonsai_t2.so and libbonsai_q1.so: argument
// checks, one-time device set-up and the choice between the two kernels --
// the dot4 kernel (packed_gemv.hip.h) for a single token and for shapes the
// matrix-core kernel does not take, the MFMA kernel (gemv_mfma.hip.h) from
// `min_width` tokens on.  Replaces the if-chain over registered (M, N, K) of the
// reference (src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:94-148).
#ifndef BONSAI_GEMV_DISPATCH_HIP_H
#define BONSAI_GEMV_DISPATCH_HIP_H

#include "gemv_mfma.hip.h"
#include "packed_gemv.hip.h"

namespace bonsai {

constexpr int kDefaultMfmaMinWidth = 2;

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
        st.mfma_ready[dev] = true;
    }
    return 0;
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
    const int min_width = mtu.min_width > 0 ? mtu.min_width : kDefaultMfmaMinWidth;
    if (M >= min_width && mfma_shape_ok(B, out_kind == OUT_G32 ? nullptr : ws, K)) {
        const int rc = launch_gemv_mfma<BITS>(A, B, out, s, ws, M, N, K, out_kind, scale_kind,
                                              lds_limit, stream);
        if (rc >= 0) return rc;
    }
    return launch_gemv_dot4<BITS>(A, B, out, s, ws, M, N, K, out_kind, scale_kind, lds_limit,
                                  stream);
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_DISPATCH_HIP_H
