// libbonsai_t2.so: C ABI of the T2-g128 (ternary, 2-bit codes) W2A8 GEMV for
// gfx950.  Entry points are declared in include/bonsai_gemv.h; the drop-in one
// replaces src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:123-148.
#include "gemv_dispatch.hip.h"

#include "../../include/bonsai_gemv.h"

using namespace bonsai;

extern "C" {

int t2g128_init(void) { return init_all_kernels<2>(); }

const char *t2g128_last_kernel(void) { return last_kernel_name(); }

int t2g128_launch_count(void) { return last_kernel().launches; }

void t2g128_set_tuning(int lanes_per_row, int waves_per_wg, int passes) {
    Tuning &t = lib_state<2>().tuning;
    t.lanes_per_row = lanes_per_row;
    t.waves_per_wg = waves_per_wg;
    t.passes = passes;
}

void t2g128_set_mfma_tuning(int min_width, int row_tiles, int k_split, int passes, int engine) {
    MfmaTuning &t = mfma_tuning<2>();
    t.min_width = min_width;
    t.row_tiles = row_tiles;
    t.k_split = k_split;
    t.passes = passes;
    t.engine = engine;
}

int t2g128_gemv_grouped(const bonsai_gemv_desc *descs, int count, int out_kind, int scale_kind,
                        void *stream) {
    if (descs == nullptr || count < 1 || count > BONSAI_GROUPED_MAX) return BONSAI_ERR_ARG;
    GemvProblem probs[BONSAI_GROUPED_MAX];
    for (int i = 0; i < count; ++i)
        probs[i] = GemvProblem{descs[i].A, descs[i].B, descs[i].out, descs[i].s, descs[i].ws,
                               descs[i].M, descs[i].N, descs[i].K};
    return launch_grouped<2>(probs, count, out_kind, scale_kind, static_cast<hipStream_t>(stream));
}

void t2g128_set_grouped_tuning(int row_tiles, int max_wgs, int min_width) {
    MxTuning &t = mx_tuning<2>();
    t.row_tiles = row_tiles;
    t.max_wgs = max_wgs;
    t.min_width = min_width;
}

void t2g128_set_stream_tuning(int min_bytes, int wgs_per_cu) {
    MxsTuning &t = mxs_tuning<2>();
    t.min_bytes = min_bytes;
    t.wgs_per_cu = wgs_per_cu;
}

int t2g128_gemv_ex(const int8_t *A, const uint8_t *B, void *out, const float *s, const void *ws,
                   int M, int N, int K, int out_kind, int scale_kind, void *stream) {
    return launch_gemv<2>(A, B, out, s, ws, M, N, K, out_kind, scale_kind,
                          static_cast<hipStream_t>(stream));
}

void t2g128_int8xint2_linear(int8_t *A, int8_t *B, void *C, float *s, void *ws, int M, int N,
                             int K, void *stream) {
    const int rc = launch_gemv<2>(A, reinterpret_cast<const uint8_t *>(B), C, s, ws, M, N, K,
                                  BONSAI_OUT_BF16, BONSAI_SCALE_BF16,
                                  static_cast<hipStream_t>(stream));
    if (rc != 0)
        fprintf(stderr, "[t2g128] unsupported shape M=%d N=%d K=%d (status %d)\n", M, N, K, rc);
}

static FusedGemv fused_from(const bonsai_fused_gemv *d) {
    return FusedGemv{d->act_kind, d->epi_kind, d->act, d->act_aux, d->act_parts,
                     static_cast<const uint16_t *>(d->norm_weight), d->eps, d->B, d->ws, d->out,
                     static_cast<const uint16_t *>(d->residual), d->out_aux, d->s_out, d->M, d->N, d->K,
                     d->out_kind};
}

int t2g128_fused_parts(int epi_kind, int M, int N, int K) { return fused_parts<2>(epi_kind, M, N, K); }

int t2g128_gemv_fused(const bonsai_fused_gemv *d, void *stream) {
    if (d == nullptr) return BONSAI_ERR_ARG;
    return launch_gemv_fused<2>(fused_from(d), static_cast<hipStream_t>(stream));
}

}  // extern "C"
