/*
 * CPU oracle for the packed low-bit GEMV path (T2-g128 ternary W2A8 and
 * Q1-g128 sign W1A8).  TEST INFRASTRUCTURE ONLY: this file is the checker the
 * HIP kernels are compared against and the CPU baseline that gets timed.  The
 * shipped library never links or calls it.
 *
 * It restates, in plain C, the arithmetic of the reference CUDA kernels and
 * Python helpers (paths relative to the reference tree):
 *   - weight decode     src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:21-27
 *                       src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels.h:21-24
 *   - group dot + scale src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:62-81
 *                       src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels.h:388-410
 *   - epilogue          src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:83-91
 *   - activation quant  src/bonsai_sft/gpu/model.py:632-636
 *   - packers           src/bonsai_sft/gpu/convert_bonsai_mtp_to_gpu.py:87-144
 *
 * The reference's path is CUDA only and cannot be built in this image, so no
 * function here is validated against a reference binary.  Each one is pinned
 * instead by known answers, brute force and library cross-checks in
 * tests/test_oracle.py (none is "parity unpinned").
 *
 * Numerical definition (the canonical one both the tests and the kernels use):
 *   G[m,n,g] = sum_{k in group g} int32(A[m,k]) * int32(w[n,k])        exact
 *   y32[m,n] = ( sum_{g ascending} float(G[m,n,g]) * float(ws[n,g]) ) / s[m]
 *   y[m,n]   = bf16_round_to_nearest_even(y32[m,n])
 * The reference sums lane partials in tree order and divides with an
 * approximate reciprocal; both differ from this only by fp32 rounding.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define ORACLE_GROUP 128

/* ---- scalar conversions ------------------------------------------------ */

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float oracle_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* Round-to-nearest-even fp32 -> bf16, NaN kept quiet. */
uint16_t oracle_f32_to_bf16(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_f32(sign | 0x7f800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline float scale_to_f32(uint16_t raw, int scale_is_f16) {
    return scale_is_f16 ? oracle_f16_to_f32(raw) : oracle_bf16_to_f32(raw);
}

/* ---- weight decode (t2g128_kernels.cu:21-27, q1g128_kernels.h:21-24) ---- */

/* T2: weight k of row n = ((byte[k/4] >> 2*(k%4)) & 3) - 2.  Code 0 decodes to
 * -2; the packer never emits it but the decode is defined for it. */
void oracle_unpack_t2(const uint8_t *B, int8_t *W, int N, int K) {
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) {
            uint8_t byte = B[(size_t)n * (K / 4) + k / 4];
            W[(size_t)n * K + k] = (int8_t)(((byte >> (2 * (k % 4))) & 3) - 2);
        }
}

/* Q1: weight k of row n = 2*bit(k%8 of byte[k/8]) - 1, LSB first. */
void oracle_unpack_q1(const uint8_t *B, int8_t *W, int N, int K) {
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) {
            uint8_t byte = B[(size_t)n * (K / 8) + k / 8];
            W[(size_t)n * K + k] = (int8_t)(2 * ((byte >> (k % 8)) & 1) - 1);
        }
}

/* ---- packers (convert_bonsai_mtp_to_gpu.py:87-144) --------------------- */

/* Pack ternary values q in {-1,0,+1} as codes q+2, four per byte, LSB first. */
void oracle_pack_t2_codes(const int8_t *Q, uint8_t *B, int N, int K) {
    for (int n = 0; n < N; ++n)
        for (int j = 0; j < K / 4; ++j) {
            unsigned byte = 0;
            for (int i = 0; i < 4; ++i)
                byte |= (unsigned)((Q[(size_t)n * K + 4 * j + i] + 2) & 3) << (2 * i);
            B[(size_t)n * (K / 4) + j] = (uint8_t)byte;
        }
}

/* Pack signs (value >= 0 -> bit 1) eight per byte, LSB first. */
void oracle_pack_q1_signs(const int8_t *Q, uint8_t *B, int N, int K) {
    for (int n = 0; n < N; ++n)
        for (int j = 0; j < K / 8; ++j) {
            unsigned byte = 0;
            for (int i = 0; i < 8; ++i)
                byte |= (unsigned)(Q[(size_t)n * K + 8 * j + i] >= 0) << i;
            B[(size_t)n * (K / 8) + j] = (uint8_t)byte;
        }
}

/* _pack_t2_g128 (convert_bonsai_mtp_to_gpu.py:127-144): latent weights given
 * as bf16 bit patterns.  scale = bf16(max|w|) per group;
 * q = clamp(round_half_even(w / max(float(scale), 1e-30)), -1, 1). */
void oracle_pack_t2_g128(const uint16_t *Wlat, uint8_t *B, uint16_t *scales, int N, int K) {
    int ng = K / ORACLE_GROUP;
    for (int n = 0; n < N; ++n)
        for (int g = 0; g < ng; ++g) {
            const uint16_t *w = Wlat + (size_t)n * K + (size_t)g * ORACLE_GROUP;
            float amax = 0.0f;
            for (int i = 0; i < ORACLE_GROUP; ++i) {
                float a = fabsf(oracle_bf16_to_f32(w[i]));
                if (a > amax) amax = a;
            }
            uint16_t sc = oracle_f32_to_bf16(amax);
            scales[(size_t)n * ng + g] = sc;
            float d = oracle_bf16_to_f32(sc);
            if (d < 1e-30f) d = 1e-30f;
            for (int j = 0; j < ORACLE_GROUP / 4; ++j) {
                unsigned byte = 0;
                for (int i = 0; i < 4; ++i) {
                    float r = rintf(oracle_bf16_to_f32(w[4 * j + i]) / d);
                    if (r < -1.0f) r = -1.0f;
                    if (r > 1.0f) r = 1.0f;
                    byte |= (unsigned)(((int)r + 2) & 3) << (2 * i);
                }
                B[(size_t)n * (K / 4) + (size_t)g * (ORACLE_GROUP / 4) + j] = (uint8_t)byte;
            }
        }
}

/* _pack_q1_0_g128 (convert_bonsai_mtp_to_gpu.py:87-124): scale = bf16(mean|w|)
 * per group (fp32 mean), bit = (w > 0) | (w == 0). */
void oracle_pack_q1_g128(const uint16_t *Wlat, uint8_t *B, uint16_t *scales, int N, int K) {
    int ng = K / ORACLE_GROUP;
    for (int n = 0; n < N; ++n)
        for (int g = 0; g < ng; ++g) {
            const uint16_t *w = Wlat + (size_t)n * K + (size_t)g * ORACLE_GROUP;
            /* The converter only ever packs frozen-grid weights (every |w| in a
             * group equals the same bf16 d_g), for which the mean is d_g exactly
             * in any summation order.  For other inputs this is the correctly
             * rounded mean (double sum, exact /128), which torch's fp32 sum can
             * miss by one fp32 ulp before the bf16 rounding. */
            double acc = 0.0;
            for (int i = 0; i < ORACLE_GROUP; ++i) acc += fabs((double)oracle_bf16_to_f32(w[i]));
            scales[(size_t)n * ng + g] = oracle_f32_to_bf16((float)(acc / ORACLE_GROUP));
            for (int j = 0; j < ORACLE_GROUP / 8; ++j) {
                unsigned byte = 0;
                for (int i = 0; i < 8; ++i)
                    byte |= (unsigned)(oracle_bf16_to_f32(w[8 * j + i]) >= 0.0f) << i;
                B[(size_t)n * (K / 8) + (size_t)g * (ORACLE_GROUP / 8) + j] = (uint8_t)byte;
            }
        }
}

/* ---- activation quant (model.py:632-636) ------------------------------- */

/* x is the activation already widened to fp32 (x.float() is exact for fp16 and
 * bf16).  The reference writes `127.0 / absmax.clamp_(min=1e-5)`; PyTorch evaluates
 * a Python scalar divided by a tensor as `tensor.reciprocal() * scalar`
 * (Tensor.__rtruediv__), i.e. TWO fp32 roundings, so
 *     s = fl( fl(1 / max(absmax, 1e-5)) * 127 ),   q = clamp(rint(fl(x*s)), -128, 127). */
void oracle_act_quant(const float *X, int8_t *Q, float *S, int M, int K) {
    for (int m = 0; m < M; ++m) {
        const float *x = X + (size_t)m * K;
        float amax = 0.0f;
        for (int k = 0; k < K; ++k) {
            float a = fabsf(x[k]);
            if (a > amax) amax = a;
        }
        if (amax < 1e-5f) amax = 1e-5f;
        volatile float recip = 1.0f / amax; /* kept as its own rounding step */
        float s = recip * 127.0f;
        S[m] = s;
        for (int k = 0; k < K; ++k) {
            float r = rintf(x[k] * s); /* default rounding mode: half to even */
            if (r < -128.0f) r = -128.0f;
            if (r > 127.0f) r = 127.0f;
            Q[(size_t)m * K + k] = (int8_t)r;
        }
    }
}

/* ---- group sums and GEMV (t2g128_kernels.cu:54-91) ---------------------- */

static inline void decode_row_group(const uint8_t *brow, int g, int bits, int8_t *w) {
    if (bits == 2) {
        const uint8_t *p = brow + (size_t)g * (ORACLE_GROUP / 4);
        for (int k = 0; k < ORACLE_GROUP; ++k) w[k] = (int8_t)(((p[k / 4] >> (2 * (k % 4))) & 3) - 2);
    } else {
        const uint8_t *p = brow + (size_t)g * (ORACLE_GROUP / 8);
        for (int k = 0; k < ORACLE_GROUP; ++k) w[k] = (int8_t)(2 * ((p[k / 8] >> (k % 8)) & 1) - 1);
    }
}

/* G[m,n,g], int32, exact.  bits = 2 (T2) or 1 (Q1). */
void oracle_group_sums(const int8_t *A, const uint8_t *B, int32_t *G, int M, int N, int K, int bits) {
    int ng = K / ORACLE_GROUP;
    size_t rowbytes = (size_t)K * bits / 8;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        int8_t w[ORACLE_GROUP];
        for (int g = 0; g < ng; ++g) {
            decode_row_group(B + (size_t)n * rowbytes, g, bits, w);
            for (int m = 0; m < M; ++m) {
                const int8_t *a = A + (size_t)m * K + (size_t)g * ORACLE_GROUP;
                int32_t acc = 0;
                for (int k = 0; k < ORACLE_GROUP; ++k) acc += (int32_t)a[k] * (int32_t)w[k];
                G[((size_t)m * N + n) * ng + g] = acc;
            }
        }
    }
}

/* y32[m,n] (fp32, before the bf16 rounding) and, if Y16 != NULL, y as bf16 bits. */
void oracle_gemv(const int8_t *A, const uint8_t *B, const float *S, const uint16_t *WS,
                 float *Y32, uint16_t *Y16, int M, int N, int K, int bits, int scale_is_f16) {
    int ng = K / ORACLE_GROUP;
    size_t rowbytes = (size_t)K * bits / 8;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        int8_t w[ORACLE_GROUP];
        float acc[64];
        for (int m0 = 0; m0 < M; m0 += 64) {
            int mt = M - m0 < 64 ? M - m0 : 64;
            for (int m = 0; m < mt; ++m) acc[m] = 0.0f;
            for (int g = 0; g < ng; ++g) {
                decode_row_group(B + (size_t)n * rowbytes, g, bits, w);
                float wsf = scale_to_f32(WS[(size_t)n * ng + g], scale_is_f16);
                for (int m = 0; m < mt; ++m) {
                    const int8_t *a = A + (size_t)(m0 + m) * K + (size_t)g * ORACLE_GROUP;
                    int32_t dot = 0;
                    for (int k = 0; k < ORACLE_GROUP; ++k) dot += (int32_t)a[k] * (int32_t)w[k];
                    /* float(dot)*wsf is exact (|dot| < 2^15, 8- or 11-bit scale
                     * significand); only the running sum rounds.  Written with an
                     * explicit temporary so no fused multiply-add can change that. */
                    volatile float term = (float)dot * wsf;
                    acc[m] = acc[m] + term;
                }
            }
            for (int m = 0; m < mt; ++m) {
                float y = acc[m] / S[m0 + m];
                if (Y32) Y32[(size_t)(m0 + m) * N + n] = y;
                if (Y16) Y16[(size_t)(m0 + m) * N + n] = oracle_f32_to_bf16(y);
            }
        }
    }
}

/* ---- fused norm / activation producers (model.py:307-336, 1058-1061) ---- */

static inline float bf16_round_f(float f) { return oracle_bf16_to_f32(oracle_f32_to_bf16(f)); }

/* Sum of fp32 squares in fp64, in the order the HIP kernel uses: T threads with
 * T = min(1024, K/8 rounded up to a multiple of 64); thread t takes the 8-element
 * vectors t, t+T, ... in turn; xor butterfly (1,2,..,32) inside each 64-thread wave;
 * the wave totals added left to right. */
static double sumsq_kernel_order(const float *h, int K) {
    static double lane[1024];
    int nvec = K / 8;
    int T = ((nvec < 1024 ? nvec : 1024) + 63) / 64 * 64;
    if (T < 64) T = 64;
    for (int t = 0; t < T; ++t) {
        double acc = 0.0;
        for (int v = t; v < nvec; v += T)
            for (int i = 0; i < 8; ++i) {
                volatile float sq = h[8 * v + i] * h[8 * v + i];
                acc += (double)sq;
            }
        lane[t] = acc;
    }
    double total = 0.0;
    for (int w = 0; w < T / 64; ++w) {
        double a[64], b[64];
        for (int i = 0; i < 64; ++i) a[i] = lane[64 * w + i];
        for (int off = 1; off < 64; off <<= 1) {
            for (int i = 0; i < 64; ++i) b[i] = a[i] + a[i ^ off];
            for (int i = 0; i < 64; ++i) a[i] = b[i];
        }
        total = (w == 0) ? a[0] : total + a[0];
    }
    return total;
}

static void quant_row(const float *nf, int8_t *q, float *s, int K) {
    float amax = 0.0f;
    for (int k = 0; k < K; ++k) {
        float a = fabsf(nf[k]);
        if (a > amax) amax = a;
    }
    if (amax < 1e-5f) amax = 1e-5f;
    volatile float recip = 1.0f / amax;
    float sv = recip * 127.0f;
    *s = sv;
    for (int k = 0; k < K; ++k) {
        float r = rintf(nf[k] * sv);
        if (r < -128.0f) r = -128.0f;
        if (r > 127.0f) r = 127.0f;
        q[k] = (int8_t)r;
    }
}

/* _fused_norm_quant / _fused_add_norm_quant.  X, RES (may be NULL), W are bf16 bit
 * patterns; H (may be NULL) receives bf16(x + residual).  K <= 65536. */
static void rmsnorm_row(const uint16_t *x, const uint16_t *res, const uint16_t *W, float eps,
                        uint16_t *hrow, float *nf, int K) {
    static float h[65536];
    for (int k = 0; k < K; ++k) {
        float v = oracle_bf16_to_f32(x[k]);
        if (res) {
            volatile float sum = v + oracle_bf16_to_f32(res[k]);
            v = bf16_round_f(sum);
            if (hrow) hrow[k] = oracle_f32_to_bf16(v);
        }
        h[k] = v;
    }
    float var = (float)sumsq_kernel_order(h, K) / (float)K;
    volatile float root = sqrtf(var + eps);
    float rs = 1.0f / root;
    for (int k = 0; k < K; ++k) {
        volatile float t = h[k] * rs;
        volatile float u = oracle_bf16_to_f32(W[k]) * bf16_round_f(t);
        nf[k] = bf16_round_f(u);
    }
}

void oracle_rmsnorm_quant(const uint16_t *X, const uint16_t *RES, const uint16_t *W, float eps,
                          uint16_t *H, int8_t *Q, float *S, int M, int K) {
    static float nf[65536];
    for (int m = 0; m < M; ++m) {
        rmsnorm_row(X + (size_t)m * K, RES ? RES + (size_t)m * K : NULL, W, eps,
                    H ? H + (size_t)m * K : NULL, nf, K);
        quant_row(nf, Q + (size_t)m * K, S + m, K);
    }
}

/* The same norm without the quantisation: RMSNorm.forward on h = x (+ residual)
 * (src/bonsai_sft/gpu/model.py:290-295, 1401-1402).  NOUT receives bf16(w * bf16(h * rs)). */
void oracle_rmsnorm_bf16(const uint16_t *X, const uint16_t *RES, const uint16_t *W, float eps,
                         uint16_t *H, uint16_t *NOUT, int M, int K) {
    static float nf[65536];
    for (int m = 0; m < M; ++m) {
        rmsnorm_row(X + (size_t)m * K, RES ? RES + (size_t)m * K : NULL, W, eps,
                    H ? H + (size_t)m * K : NULL, nf, K);
        for (int k = 0; k < K; ++k) NOUT[(size_t)m * K + k] = oracle_f32_to_bf16(nf[k]);
    }
}

/* SiLU(gate) * up + quant: GU bf16 [M, 2F]; inner = bf16(bf16(g / (1 + exp(-g))) * u). */
void oracle_silu_mul_quant(const uint16_t *GU, int8_t *Q, float *S, int M, int F) {
    static float nf[65536];
    for (int m = 0; m < M; ++m) {
        const uint16_t *g = GU + (size_t)m * 2 * F, *u = g + F;
        for (int k = 0; k < F; ++k) {
            float gv = oracle_bf16_to_f32(g[k]);
            volatile float sg = gv / (1.0f + expf(-gv));
            volatile float pr = bf16_round_f(sg) * oracle_bf16_to_f32(u[k]);
            nf[k] = bf16_round_f(pr);
        }
        quant_row(nf, Q + (size_t)m * F, S + m, F);
    }
}

int oracle_abi_version(void) { return 3; }
