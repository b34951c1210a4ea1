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


// ---------------------------------------------------------------------------
// Fused producers of the GEMV input: RMSNorm (+ residual add) + quantisation and
// SiLU(gate) * up + quantisation.  They replace the torch.compile'd Python
// helpers of the reference (src/bonsai_sft/gpu/model.py:307-336 and :1059-1061)
// and keep their rounding points:
//   h      = bf16(x + residual)                       (add variant only)
//   var    = fp32(sum of fp32 squares) / K ; rs = 1 / sqrt(var + eps)     (fp32, IEEE)
//   normed = bf16( w * bf16(fp32(h) * rs) )           (two bf16 roundings)
//   s, q   = per-token absmax quantisation of fp32(normed)
// The sum of squares is accumulated in fp64 in a fixed order (thread-strided, then
// an xor butterfly per wave, then the four waves left to right), which the CPU
// oracle replays, so q and s are reproducible bit for bit.
// One workgroup per token; the row is re-read from L2 instead of being kept in
// registers (M is at most a few dozen tokens).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ float bf16_round(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ __forceinline__ void load8_bf16(const uint16_t *row, int v, float out[8]) {
    const uint4 raw = reinterpret_cast<const uint4 *>(row)[v];
    const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i] = bf16_bits_to_f32(d[i] & 0xffffu);
        out[2 * i + 1] = bf16_bits_to_f32(d[i] >> 16);
    }
}

__device__ __forceinline__ double block_sum_f64(double v, double *scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    double t = scratch[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) t += scratch[w];
    __syncthreads();
    return t;
}

__device__ __forceinline__ float block_max_f32(float v, float *scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = scratch[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) t = fmaxf(t, scratch[w]);
    __syncthreads();
    return t;
}

__device__ __forceinline__ void store_q8(int8_t *qrow, int v, const float nf[8], float sval) {
    uint2 o;
    o.x = quant1(nf[0], sval) | (quant1(nf[1], sval) << 8) | (quant1(nf[2], sval) << 16) |
          (quant1(nf[3], sval) << 24);
    o.y = quant1(nf[4], sval) | (quant1(nf[5], sval) << 8) | (quant1(nf[6], sval) << 16) |
          (quant1(nf[7], sval) << 24);
    reinterpret_cast<uint2 *>(qrow)[v] = o;
}

template <bool ADD>
__global__ void __launch_bounds__(kThreads)
rmsnorm_quant_kernel(const uint16_t *x, const uint16_t *residual, const uint16_t *w, float eps,
                     uint16_t *h_out, int8_t *q, float *s, int K) {
    __shared__ double sum_scratch[kThreads / 64];
    __shared__ float max_scratch[kThreads / 64];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int nvec = K / 8;
    const uint16_t *xrow = x + (size_t)m * K;
    const uint16_t *rrow = ADD ? residual + (size_t)m * K : nullptr;

    auto load_h = [&](int v, float h[8]) {
        load8_bf16(xrow, v, h);
        if (ADD) {
            float r[8];
            load8_bf16(rrow, v, r);
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] = bf16_round(h[i] + r[i]);
        }
    };

    double ss = 0.0;
    for (int v = tid; v < nvec; v += kThreads) {
        float h[8];
        load_h(v, h);
        if (ADD) {
            uint4 o;
            o.x = f32_to_bf16_bits(h[0]) | (f32_to_bf16_bits(h[1]) << 16);
            o.y = f32_to_bf16_bits(h[2]) | (f32_to_bf16_bits(h[3]) << 16);
            o.z = f32_to_bf16_bits(h[4]) | (f32_to_bf16_bits(h[5]) << 16);
            o.w = f32_to_bf16_bits(h[6]) | (f32_to_bf16_bits(h[7]) << 16);
            reinterpret_cast<uint4 *>(h_out + (size_t)m * K)[v] = o;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float sq = h[i] * h[i];
            ss += (double)sq;
        }
    }
    const double total = block_sum_f64(ss, sum_scratch);
    const float var = (float)total / (float)K;
    const float rs = 1.0f / sqrtf(var + eps);

    auto normed = [&](int v, float nf[8]) {
        float h[8], wv[8];
        load_h(v, h);
        load8_bf16(w, v, wv);
#pragma unroll
        for (int i = 0; i < 8; ++i) nf[i] = bf16_round(wv[i] * bf16_round(h[i] * rs));
    };

    float amax = 0.0f;
    for (int v = tid; v < nvec; v += kThreads) {
        float nf[8];
        normed(v, nf);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(nf[i]));
    }
    amax = block_max_f32(amax, max_scratch);
    const float recip = 1.0f / fmaxf(amax, 1e-5f);
    const float sval = recip * 127.0f;
    if (tid == 0) s[m] = sval;

    int8_t *qrow = q + (size_t)m * K;
    for (int v = tid; v < nvec; v += kThreads) {
        float nf[8];
        normed(v, nf);
        store_q8(qrow, v, nf, sval);
    }
}

// inner = bf16( fp32(bf16(silu(gate))) * up ), gate = gu[m][0..F), up = gu[m][F..2F)
__global__ void __launch_bounds__(kThreads)
silu_mul_quant_kernel(const uint16_t *gu, int8_t *q, float *s, int F) {
    __shared__ float max_scratch[kThreads / 64];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int nvec = F / 8;
    const uint16_t *grow = gu + (size_t)m * 2 * F;
    const uint16_t *urow = grow + F;

    auto inner = [&](int v, float nf[8]) {
        float g[8], u[8];
        load8_bf16(grow, v, g);
        load8_bf16(urow, v, u);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float sg = bf16_round(g[i] / (1.0f + expf(-g[i])));
            nf[i] = bf16_round(sg * u[i]);
        }
    };
    float amax = 0.0f;
    for (int v = tid; v < nvec; v += kThreads) {
        float nf[8];
        inner(v, nf);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(nf[i]));
    }
    amax = block_max_f32(amax, max_scratch);
    const float recip = 1.0f / fmaxf(amax, 1e-5f);
    const float sval = recip * 127.0f;
    if (tid == 0) s[m] = sval;
    int8_t *qrow = q + (size_t)m * F;
    for (int v = tid; v < nvec; v += kThreads) {
        float nf[8];
        inner(v, nf);
        store_q8(qrow, v, nf, sval);
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

extern "C" int bonsai_rmsnorm_quant_int8(const void *x, const void *w, float eps, int8_t *q, float *s,
                                         int M, int K, void *stream) {
    if (x == nullptr || w == nullptr || q == nullptr || s == nullptr) return BONSAI_ERR_ARG;
    if (M < 1 || K < 8 || K % 8 != 0) return BONSAI_ERR_ARG;
    hipLaunchKernelGGL(rmsnorm_quant_kernel<false>, dim3(M), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t *>(x),
                       nullptr, reinterpret_cast<const uint16_t *>(w), eps, nullptr, q, s, K);
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}

extern "C" int bonsai_add_rmsnorm_quant_int8(const void *x, const void *residual, const void *w,
                                             float eps, void *h_out, int8_t *q, float *s, int M,
                                             int K, void *stream) {
    if (x == nullptr || residual == nullptr || w == nullptr || h_out == nullptr || q == nullptr ||
        s == nullptr)
        return BONSAI_ERR_ARG;
    if (M < 1 || K < 8 || K % 8 != 0) return BONSAI_ERR_ARG;
    hipLaunchKernelGGL(rmsnorm_quant_kernel<true>, dim3(M), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), reinterpret_cast<const uint16_t *>(x),
                       reinterpret_cast<const uint16_t *>(residual),
                       reinterpret_cast<const uint16_t *>(w), eps,
                       reinterpret_cast<uint16_t *>(h_out), q, s, K);
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}

extern "C" int bonsai_silu_mul_quant_int8(const void *gate_up, int8_t *q, float *s, int M, int F,
                                          void *stream) {
    if (gate_up == nullptr || q == nullptr || s == nullptr) return BONSAI_ERR_ARG;
    if (M < 1 || F < 8 || F % 8 != 0) return BONSAI_ERR_ARG;
    hipLaunchKernelGGL(silu_mul_quant_kernel, dim3(M), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const uint16_t *>(gate_up), q, s, F);
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}
