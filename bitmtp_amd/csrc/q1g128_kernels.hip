// libbonsai_q1.so: C ABI of the Q1-g128 (sign, 1 bit) W1A8 GEMV for gfx950.
// Entry points are declared in include/bonsai_gemv.h; the drop-in one replaces
// src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels_block8.cu:118-241.
#include "gemv_dispatch.hip.h"

#include "../../include/bonsai_gemv.h"

using namespace bonsai;

namespace {

// 1-bit weights x bf16 activations with fp32 accumulation (no activation
// quantisation), the lm_head variant of the reference
// (src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels_block8.cu:31-84).
// 8 lanes share a weight row, a lane owns whole 128-weight groups:
//     p = sum_{k in g} (+-1) * fp32(A[m][k]);  acc[m] += p * ws[n][g]
// A plain streaming kernel: weights are read once per token tile of 4, the
// bf16 activations come from L2.
constexpr int kW16Tile = 4;

__global__ void __launch_bounds__(256) w1a16_kernel(const uint16_t *A, const uint8_t *B,
                                                    uint16_t *C, const uint16_t *ws, int M, int N,
                                                    int K) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int c = lane & 7;
    const int row = ((int)blockIdx.x * 4 + wave) * 8 + (lane >> 3);
    const int row_c = row < N ? row : N - 1;
    const int ng = K / kGroup;
    const int m0 = blockIdx.y * kW16Tile;
    const u32x4 *wrow = reinterpret_cast<const u32x4 *>(B + (size_t)row_c * (K / 8));
    float acc[kW16Tile] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int g = c; g < ng; g += 8) {
        const u32x4 w = wrow[g];
        const float wsf = __uint_as_float((uint32_t)ws[(size_t)row_c * ng + g] << 16);
        const uint32_t p[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int m = 0; m < kW16Tile; ++m) {
            const int msrc = (m0 + m) < M ? (m0 + m) : M - 1;
            const uint32_t *a = reinterpret_cast<const uint32_t *>(A + (size_t)msrc * K + (size_t)g * kGroup);
            float part = 0.0f;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll 4
                for (int j = 0; j < 16; ++j) {
                    const uint32_t pair = a[t * 16 + j];  // activations 32t+2j, 32t+2j+1
                    const float a0 = __uint_as_float(pair << 16);
                    const float a1 = __uint_as_float(pair & 0xffff0000u);
                    part += ((p[t] >> (2 * j)) & 1u) ? a0 : -a0;
                    part += ((p[t] >> (2 * j + 1)) & 1u) ? a1 : -a1;
                }
            }
            acc[m] += part * wsf;
        }
    }
#pragma unroll
    for (int m = 0; m < kW16Tile; ++m) {
        const float sum = row_lanes_sum(acc[m], 3);
        if (c == 0 && row < N && (m0 + m) < M) C[(size_t)(m0 + m) * N + row] = f32_to_bf16_rne(sum);
    }
}

}  // namespace

extern "C" {

void q1g128_w1a16_linear(const void *A, const int8_t *B, void *C, const void *ws, int M, int N,
                         int K, void *stream) {
    if (A == nullptr || B == nullptr || C == nullptr || ws == nullptr || M < 1 || N < 1 ||
        K < kGroup || K % kGroup != 0) {
        fprintf(stderr, "[q1g128_w1a16_linear] unsupported (M=%d, N=%d, K=%d)\n", M, N, K);
        return;
    }
    hipLaunchKernelGGL(w1a16_kernel, dim3((N + 31) / 32, (M + kW16Tile - 1) / kW16Tile, 1),
                       dim3(256, 1, 1), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<const uint16_t *>(A), reinterpret_cast<const uint8_t *>(B),
                       reinterpret_cast<uint16_t *>(C), reinterpret_cast<const uint16_t *>(ws), M, N,
                       K);
}

int q1g128_init(void) { return init_all_kernels<1>(); }

const char *q1g128_last_kernel(void) { return last_kernel_name(); }

int q1g128_launch_count(void) { return last_kernel().launches; }

void q1g128_set_tuning(int lanes_per_row, int waves_per_wg, int passes) {
    Tuning &t = lib_state<1>().tuning;
    t.lanes_per_row = lanes_per_row;
    t.waves_per_wg = waves_per_wg;
    t.passes = passes;
}

void q1g128_set_mfma_tuning(int min_width, int row_tiles, int k_split, int passes, int engine) {
    MfmaTuning &t = mfma_tuning<1>();
    t.min_width = min_width;
    t.row_tiles = row_tiles;
    t.k_split = k_split;
    t.passes = passes;
    t.engine = engine;
}

int q1g128_gemv_grouped(const bonsai_gemv_desc *descs, int count, int out_kind, int scale_kind,
                        void *stream) {
    if (descs == nullptr || count < 1 || count > BONSAI_GROUPED_MAX) return BONSAI_ERR_ARG;
    GemvProblem probs[BONSAI_GROUPED_MAX];
    for (int i = 0; i < count; ++i)
        probs[i] = GemvProblem{descs[i].A, descs[i].B, descs[i].out, descs[i].s, descs[i].ws,
                               descs[i].M, descs[i].N, descs[i].K};
    return launch_grouped<1>(probs, count, out_kind, scale_kind, static_cast<hipStream_t>(stream));
}

void q1g128_set_grouped_tuning(int row_tiles, int max_wgs, int min_width) {
    MxTuning &t = mx_tuning<1>();
    t.row_tiles = row_tiles;
    t.max_wgs = max_wgs;
    t.min_width = min_width;
}

void q1g128_set_stream_tuning(int min_bytes, int wgs_per_cu) {
    MxsTuning &t = mxs_tuning<1>();
    t.min_bytes = min_bytes;
    t.wgs_per_cu = wgs_per_cu;
}

int q1g128_gemv_ex(const int8_t *A, const uint8_t *B, void *out, const float *s, const void *ws,
                   int M, int N, int K, int out_kind, int scale_kind, void *stream) {
    return launch_gemv<1>(A, B, out, s, ws, M, N, K, out_kind, scale_kind,
                          static_cast<hipStream_t>(stream));
}

void q1g128_int8xint1_linear(int8_t *A, int8_t *B, void *C, float *s, void *ws, int M, int N,
                             int K, void *stream) {
    const int rc = launch_gemv<1>(A, reinterpret_cast<const uint8_t *>(B), C, s, ws, M, N, K,
                                  BONSAI_OUT_BF16, BONSAI_SCALE_BF16,
                                  static_cast<hipStream_t>(stream));
    if (rc != 0)
        fprintf(stderr, "[q1g128] unsupported shape M=%d N=%d K=%d (status %d)\n", M, N, K, rc);
}

static FusedGemv fused_from(const bonsai_fused_gemv *d) {
    return FusedGemv{d->act_kind, d->epi_kind, d->act, d->act_aux, d->act_parts,
                     static_cast<const uint16_t *>(d->norm_weight), d->eps, d->B, d->ws, d->out,
                     static_cast<const uint16_t *>(d->residual), d->out_aux, d->s_out, d->M, d->N, d->K,
                     d->out_kind};
}

int q1g128_fused_parts(int epi_kind, int M, int N, int K) { return fused_parts<1>(epi_kind, M, N, K); }

int q1g128_gemv_fused(const bonsai_fused_gemv *d, void *stream) {
    if (d == nullptr) return BONSAI_ERR_ARG;
    return launch_gemv_fused<1>(fused_from(d), static_cast<hipStream_t>(stream));
}

}  // extern "C"
