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
#include "wave_reduce.h"

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
// an xor butterfly per wave, then the waves left to right), which the CPU
// oracle replays, so q and s are reproducible bit for bit.
// One workgroup per token; the row is read once and kept in registers, so the kernel
// is one memory round trip plus two workgroup reductions long.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
// round to nearest even through the hardware conversion (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    const __bf16 b = static_cast<__bf16>(f);
    uint16_t u;
    __builtin_memcpy(&u, &b, 2);
    return u;
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

// Block geometry of the fused producers: one workgroup per token, one 8-element vector
// per thread and pass, `producer_threads(K/8)` threads, so that a row of up to 8192
// elements is read from memory exactly once and kept in registers across the two
// reductions.  Longer rows take several vectors per thread (VPT, a power of two).
constexpr int kMaxProducerThreads = 1024;
constexpr int kMaxProducerWaves = kMaxProducerThreads / 64;

__host__ __device__ inline int producer_threads(int nvec) {
    const int t = ((nvec < kMaxProducerThreads ? nvec : kMaxProducerThreads) + 63) / 64 * 64;
    return t < 64 ? 64 : t;
}

// Fixed reduction order (the CPU oracle replays it): thread t accumulates its vectors
// t, t+T, ... in turn, an xor butterfly (1,2,...,32) inside each wave, then the wave
// totals left to right.
__device__ __forceinline__ double block_sum_f64(double v, double *scratch, int waves) {
    v = bonsai_wave::sum64(v);  // the xor butterfly 1, 2, ..., 32 on the DPP network
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    double t = scratch[0];
    for (int w = 1; w < waves; ++w) t += scratch[w];
    return t;
}

__device__ __forceinline__ float block_max_f32(float v, float *scratch, int waves) {
    v = bonsai_wave::max64(v);
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = scratch[0];
    for (int w = 1; w < waves; ++w) t = fmaxf(t, scratch[w]);
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

__device__ __forceinline__ void unpack8_bf16(const uint4 raw, float out[8]) {
    const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i] = bf16_bits_to_f32(d[i] & 0xffffu);
        out[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
    }
}

template <bool ADD, int VPT>
__global__ void __launch_bounds__(kMaxProducerThreads)
rmsnorm_quant_kernel(const uint16_t *x, const uint16_t *residual, const uint16_t *w, float eps,
                     uint16_t *h_out, uint16_t *n_out, int8_t *q, float *s, int K, int T) {
    // n_out (optional): the normalised row in bf16; q / s (optional): its quantisation.
    // T = workgroup size, passed explicitly: reading blockDim costs a load at kernel start
    __shared__ double sum_scratch[kMaxProducerWaves];
    __shared__ float max_scratch[kMaxProducerWaves];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int nvec = K / 8;
    const uint4 *xrow = reinterpret_cast<const uint4 *>(x + (size_t)m * K);
    const uint4 *rrow = ADD ? reinterpret_cast<const uint4 *>(residual + (size_t)m * K) : nullptr;
    const uint4 *wrow = reinterpret_cast<const uint4 *>(w);

    // every load of the row is issued before anything waits on one
    uint4 xr[VPT], rr[VPT], wr[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * T;
        const int vc = v < nvec ? v : 0;
        xr[i] = xrow[vc];
        if (ADD) rr[i] = rrow[vc];
        wr[i] = wrow[vc];
    }
    float h[VPT][8];
    double ss = 0.0;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * T;
        unpack8_bf16(xr[i], h[i]);
        if (ADD) {
            float r[8];
            unpack8_bf16(rr[i], r);
#pragma unroll
            for (int e = 0; e < 8; ++e) h[i][e] = bf16_round(h[i][e] + r[e]);
            if (v < nvec && h_out != nullptr) {
                uint4 o;
                o.x = f32_to_bf16_bits(h[i][0]) | (f32_to_bf16_bits(h[i][1]) << 16);
                o.y = f32_to_bf16_bits(h[i][2]) | (f32_to_bf16_bits(h[i][3]) << 16);
                o.z = f32_to_bf16_bits(h[i][4]) | (f32_to_bf16_bits(h[i][5]) << 16);
                o.w = f32_to_bf16_bits(h[i][6]) | (f32_to_bf16_bits(h[i][7]) << 16);
                reinterpret_cast<uint4 *>(h_out + (size_t)m * K)[v] = o;
            }
        }
        if (v < nvec) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float sq = h[i][e] * h[i][e];
                ss += (double)sq;
            }
        }
    }
    const double total = block_sum_f64(ss, sum_scratch, T >> 6);
    const float var = (float)total / (float)K;
    const float rs = 1.0f / sqrtf(var + eps);

    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * T;
        float wv[8];
        unpack8_bf16(wr[i], wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            h[i][e] = bf16_round(wv[e] * bf16_round(h[i][e] * rs));
            if (v < nvec) amax = fmaxf(amax, fabsf(h[i][e]));
        }
        if (n_out != nullptr && v < nvec) {
            uint4 o;
            o.x = f32_to_bf16_bits(h[i][0]) | (f32_to_bf16_bits(h[i][1]) << 16);
            o.y = f32_to_bf16_bits(h[i][2]) | (f32_to_bf16_bits(h[i][3]) << 16);
            o.z = f32_to_bf16_bits(h[i][4]) | (f32_to_bf16_bits(h[i][5]) << 16);
            o.w = f32_to_bf16_bits(h[i][6]) | (f32_to_bf16_bits(h[i][7]) << 16);
            reinterpret_cast<uint4 *>(n_out + (size_t)m * K)[v] = o;
        }
    }
    if (q == nullptr) return;  // norm only (uniform over the grid)
    amax = block_max_f32(amax, max_scratch, T >> 6);
    const float recip = 1.0f / fmaxf(amax, 1e-5f);
    const float sval = recip * 127.0f;
    if (tid == 0) s[m] = sval;
    int8_t *qrow = q + (size_t)m * K;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * T;
        if (v < nvec) store_q8(qrow, v, h[i], sval);
    }
}

// inner = bf16( fp32(bf16(silu(gate))) * up ), gate = gu[m][0..F), up = gu[m][F..2F)
template <int VPT>
__global__ void __launch_bounds__(kMaxProducerThreads)
silu_mul_quant_kernel(const uint16_t *gu, int8_t *q, float *s, int F, int T) {
    __shared__ float max_scratch[kMaxProducerWaves];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int nvec = F / 8;
    const uint4 *grow = reinterpret_cast<const uint4 *>(gu + (size_t)m * 2 * F);
    const uint4 *urow = reinterpret_cast<const uint4 *>(gu + (size_t)m * 2 * F + F);
    uint4 gr[VPT], ur[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * T;
        const int vc = v < nvec ? v : 0;
        gr[i] = grow[vc];
        ur[i] = urow[vc];
    }
    float nf[VPT][8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * T;
        float g[8], u[8];
        unpack8_bf16(gr[i], g);
        unpack8_bf16(ur[i], u);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            // silu through the hardware exp2 and reciprocal (about 1e-6 relative error, far
            // below the bf16 rounding that follows): one CU evaluates a whole token row, and
            // libm's expf and the IEEE division made this kernel compute-bound
            const float ex = __builtin_amdgcn_exp2f(g[e] * -1.44269504088896341f);
            const float sg = bf16_round(g[e] * __builtin_amdgcn_rcpf(1.0f + ex));
            nf[i][e] = bf16_round(sg * u[e]);
            if (v < nvec) amax = fmaxf(amax, fabsf(nf[i][e]));
        }
    }
    amax = block_max_f32(amax, max_scratch, T >> 6);
    const float recip = 1.0f / fmaxf(amax, 1e-5f);
    const float sval = recip * 127.0f;
    if (tid == 0) s[m] = sval;
    int8_t *qrow = q + (size_t)m * F;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * T;
        if (v < nvec) store_q8(qrow, v, nf[i], sval);
    }
}

// vectors per thread for a row of nvec 8-element vectors: 1, 2, 4 or 8
inline int producer_vpt(int nvec) {
    const int t = producer_threads(nvec);
    const int need = (nvec + t - 1) / t;
    int vpt = 1;
    while (vpt < need) vpt *= 2;
    return vpt;
}

constexpr int kMaxProducerK = 8 * kMaxProducerThreads * 8;  // VPT <= 8

template <bool ADD>
void launch_rmsnorm(const uint16_t *x, const uint16_t *r, const uint16_t *w, float eps,
                    uint16_t *h_out, uint16_t *n_out, int8_t *q, float *s, int M, int K,
                    hipStream_t st) {
    const int nvec = K / 8;
    const dim3 grid(M), block(producer_threads(nvec));
    switch (producer_vpt(nvec)) {
        case 1: hipLaunchKernelGGL((rmsnorm_quant_kernel<ADD, 1>), grid, block, 0, st, x, r, w, eps, h_out, n_out, q, s, K, (int)block.x); break;
        case 2: hipLaunchKernelGGL((rmsnorm_quant_kernel<ADD, 2>), grid, block, 0, st, x, r, w, eps, h_out, n_out, q, s, K, (int)block.x); break;
        case 4: hipLaunchKernelGGL((rmsnorm_quant_kernel<ADD, 4>), grid, block, 0, st, x, r, w, eps, h_out, n_out, q, s, K, (int)block.x); break;
        default: hipLaunchKernelGGL((rmsnorm_quant_kernel<ADD, 8>), grid, block, 0, st, x, r, w, eps, h_out, n_out, q, s, K, (int)block.x); break;
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
    if (M < 1 || K < 8 || K % 8 != 0 || K > kMaxProducerK) return BONSAI_ERR_ARG;
    launch_rmsnorm<false>(reinterpret_cast<const uint16_t *>(x), nullptr,
                          reinterpret_cast<const uint16_t *>(w), eps, nullptr, nullptr, q, s, M, K,
                          static_cast<hipStream_t>(stream));
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}

extern "C" int bonsai_add_rmsnorm_quant_int8(const void *x, const void *residual, const void *w,
                                             float eps, void *h_out, int8_t *q, float *s, int M,
                                             int K, void *stream) {
    if (x == nullptr || residual == nullptr || w == nullptr || h_out == nullptr || q == nullptr ||
        s == nullptr)
        return BONSAI_ERR_ARG;
    if (M < 1 || K < 8 || K % 8 != 0 || K > kMaxProducerK) return BONSAI_ERR_ARG;
    launch_rmsnorm<true>(reinterpret_cast<const uint16_t *>(x),
                         reinterpret_cast<const uint16_t *>(residual),
                         reinterpret_cast<const uint16_t *>(w), eps,
                         reinterpret_cast<uint16_t *>(h_out), nullptr, q, s, M, K,
                         static_cast<hipStream_t>(stream));
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}

extern "C" int bonsai_add_rmsnorm_bf16(const void *x, const void *residual, const void *w, float eps,
                                       void *h_out, void *n_out, int M, int K, void *stream) {
    if (x == nullptr || w == nullptr || n_out == nullptr) return BONSAI_ERR_ARG;
    if (M < 1 || K < 8 || K % 8 != 0 || K > kMaxProducerK) return BONSAI_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (residual != nullptr)
        launch_rmsnorm<true>(reinterpret_cast<const uint16_t *>(x),
                             reinterpret_cast<const uint16_t *>(residual),
                             reinterpret_cast<const uint16_t *>(w), eps,
                             reinterpret_cast<uint16_t *>(h_out),
                             reinterpret_cast<uint16_t *>(n_out), nullptr, nullptr, M, K, st);
    else
        launch_rmsnorm<false>(reinterpret_cast<const uint16_t *>(x), nullptr,
                              reinterpret_cast<const uint16_t *>(w), eps, nullptr,
                              reinterpret_cast<uint16_t *>(n_out), nullptr, nullptr, M, K, st);
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}

extern "C" int bonsai_silu_mul_quant_int8(const void *gate_up, int8_t *q, float *s, int M, int F,
                                          void *stream) {
    if (gate_up == nullptr || q == nullptr || s == nullptr) return BONSAI_ERR_ARG;
    if (M < 1 || F < 8 || F % 8 != 0 || F > kMaxProducerK) return BONSAI_ERR_ARG;
    const int nvec = F / 8;
    const dim3 grid(M), block(producer_threads(nvec));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t *gu = reinterpret_cast<const uint16_t *>(gate_up);
    switch (producer_vpt(nvec)) {
        case 1: hipLaunchKernelGGL(silu_mul_quant_kernel<1>, grid, block, 0, st, gu, q, s, F, (int)block.x); break;
        case 2: hipLaunchKernelGGL(silu_mul_quant_kernel<2>, grid, block, 0, st, gu, q, s, F, (int)block.x); break;
        case 4: hipLaunchKernelGGL(silu_mul_quant_kernel<4>, grid, block, 0, st, gu, q, s, F, (int)block.x); break;
        default: hipLaunchKernelGGL(silu_mul_quant_kernel<8>, grid, block, 0, st, gu, q, s, F, (int)block.x); break;
    }
    return hipGetLastError() == hipSuccess ? BONSAI_OK : BONSAI_ERR_LAUNCH;
}
