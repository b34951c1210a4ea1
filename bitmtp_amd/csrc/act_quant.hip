// libbonsai_actq.so: per-token absmax INT8 activation quantisation for gfx950,
// the native form of `quant_input` (src/bonsai_sft/gpu/model.py:632-636):
//   s = fl(fl(1 / max(max_k |x_k|, 1e-5)) * 127)     two fp32 roundings: PyTorch
//                                                    evaluates `127.0 / tensor` as
//                                                    `tensor.reciprocal() * 127.0`
//   q_k = clamp(round_half_even(fp32(x_k) * s), -128, 127)
// One workgroup per token; the row is read twice (the second read hits L2) with
// 16-byte loads and written with 8-byte stores.  HBM-bound: K * (sizeof(x) + 1)
// bytes per token.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/bonsai_gemv.h"

namespace {

constexpr int kThreads = 256;

template <int XK>
struct Elem;
template <>
struct Elem<BONSAI_X_BF16> {
    static constexpr int kBytes = 2;
    static __device__ __forceinline__ float get(uint16_t raw) {
        return __uint_as_float((uint32_t)raw << 16);
    }
};
template <>
struct Elem<BONSAI_X_F16> {
    static constexpr int kBytes = 2;
    static __device__ __forceinline__ float get(uint16_t raw) {
        _Float16 h;
        __builtin_memcpy(&h, &raw, 2);
        return (float)h;
    }
};

// Loads 8 consecutive elements starting at element index 8*v of the row.
template <int XK>
__device__ __forceinline__ void load8(const void *row, int v, float out[8]) {
    if (XK == BONSAI_X_F32) {
        const float4 *p = reinterpret_cast<const float4 *>(row) + 2 * (size_t)v;
        const float4 a = p[0], b = p[1];
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
    } else {
        const uint4 raw = reinterpret_cast<const uint4 *>(row)[v];
        const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (XK == BONSAI_X_BF16) {
                out[2 * i] = Elem<BONSAI_X_BF16>::get((uint16_t)(d[i] & 0xffffu));
                out[2 * i + 1] = Elem<BONSAI_X_BF16>::get((uint16_t)(d[i] >> 16));
            } else {
                out[2 * i] = Elem<BONSAI_X_F16>::get((uint16_t)(d[i] & 0xffffu));
                out[2 * i + 1] = Elem<BONSAI_X_F16>::get((uint16_t)(d[i] >> 16));
            }
        }
    }
}

__device__ __forceinline__ uint32_t quant1(float x, float s) {
    float r = __builtin_rintf(x * s);
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (uint32_t)((int)r) & 0xffu;
}

template <int XK>
__global__ void __launch_bounds__(kThreads) act_quant_kernel(const void *x, int8_t *q, float *s,
                                                             int K) {
    __shared__ float wave_max[kThreads / 64];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const size_t elem_bytes = XK == BONSAI_X_F32 ? 4 : 2;
    const unsigned char *row = reinterpret_cast<const unsigned char *>(x) + (size_t)m * K * elem_bytes;
    const int nvec = K / 8;

    float amax = 0.0f;
    for (int v = tid; v < nvec; v += kThreads) {
        float e[8];
        load8<XK>(row, v, e);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(e[i]));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
    __syncthreads();
    amax = wave_max[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) amax = fmaxf(amax, wave_max[w]);

    const float recip = 1.0f / fmaxf(amax, 1e-5f);  // IEEE division, rounded on its own
    const float sval = recip * 127.0f;
    if (tid == 0) s[m] = sval;

    uint2 *qrow = reinterpret_cast<uint2 *>(q + (size_t)m * K);
    for (int v = tid; v < nvec; v += kThreads) {
        float e[8];
        load8<XK>(row, v, e);
        uint2 o;
        o.x = quant1(e[0], sval) | (quant1(e[1], sval) << 8) | (quant1(e[2], sval) << 16) |
              (quant1(e[3], sval) << 24);
        o.y = quant1(e[4], sval) | (quant1(e[5], sval) << 8) | (quant1(e[6], sval) << 16) |
              (quant1(e[7], sval) << 24);
        qrow[v] = o;
    }
}

}  // namespace

extern "C" int bonsai_act_quant_int8(const void *x, int x_kind, int8_t *q, float *s, int M, int K,
                                     void *stream) {
    if (x == nullptr || q == nullptr || s == nullptr) return BONSAI_ERR_ARG;
    if (M < 1 || K < 8 || K % 8 != 0) return BONSAI_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (x_kind) {
        case BONSAI_X_BF16:
            hipLaunchKernelGGL(act_quant_kernel<BONSAI_X_BF16>, dim3(M), dim3(kThreads), 0, st, x, q, s, K);
            break;
        case BONSAI_X_F16:
            hipLaunchKernelGGL(act_quant_kernel<BONSAI_X_F16>, dim3(M), dim3(kThreads), 0, st, x, q, s, K);
            break;
        case BONSAI_X_F32:
            hipLaunchKernelGGL(act_quant_kernel<BONSAI_X_F32>, dim3(M), dim3(kThreads), 0, st, x, q, s, K);
            break;
        default:
            return BONSAI_ERR_ARG;
    }
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}
