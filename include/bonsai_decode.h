/* C ABI of libbonsai_decode.so: the per-layer ops that sit between the packed GEMVs
 * of one captured decode step on gfx950 (MI355X).
 *
 * The reference runs these steps as torch.compile'd Python inside its CUDA graphs:
 *   - split + per-head q/k RMSNorm + RoPE + in-place KV write at a fixed offset
 *     (`_fused_qkv_qknorm_rope_kv_write`, src/bonsai_sft/gpu/model.py:388-436);
 *   - attention of the M new rows over the shared KV buffer
 *     (`Attention.forward_sdlm_graph_kernel`, src/bonsai_sft/gpu/model.py:996-1003)
 *     under the additive mask that `GraphAtlas.prepare_step` rebuilds every step
 *     (src/bonsai_sft/gpu/fast_runtime.py:391-421,443-465), followed by the per-token
 *     quantisation of the o_proj input (src/bonsai_sft/gpu/model.py:1004-1005);
 *   - the argmax/confidence chain over the draft logits (`_fused_draft_chain`,
 *     src/bonsai_sft/gpu/fast_generate.py:111-130) and the verifier's row argmax
 *     (src/bonsai_sft/gpu/fast_generate.py:1073).
 *
 * Every entry point only enqueues kernels on `stream`: no allocation, no
 * synchronisation, no memset, so all of them may be captured into a HIP graph.
 * They return BONSAI_DECODE_OK or an error code and never print.
 *
 * KV layout (one layer): K and V are separate bf16 arrays [n_kv][slots][128];
 * slot t < sigma holds history position t, slots sigma .. sigma+M-1 are the
 * workspace the current step writes (src/bonsai_sft/gpu/fast_runtime.py:130-138).
 *
 * Step descriptor `meta` (int32, device memory, written by the host before each
 * replay; it replaces the reference's dense [1,1,M,sigma+M] additive mask):
 *   meta[0]      cache_len   history slots [0, cache_len) are visible to every row
 *   meta[1]      hide        one history slot hidden from every row, or -1
 *   meta[2 + r]  bit j set   row r sees workspace slot sigma + j      (r, j < M <= 32)
 * A row that sees nothing at all yields zeros (the reference lets such padding rows
 * look at slot 0 instead; their output is discarded either way).
 */
#ifndef BONSAI_DECODE_H
#define BONSAI_DECODE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BONSAI_DECODE_OK 0
#define BONSAI_DECODE_ERR_ARG 1
#define BONSAI_DECODE_ERR_LAUNCH 2
#define BONSAI_DECODE_ERR_NOT_INIT 3 /* a one-time set-up would have run on a capturing stream:
                                        call bonsai_decode_init before the capture */

#define BONSAI_HEAD_DIM 128     /* the only head size of the Bonsai/Qwen3 family */
#define BONSAI_MAX_WIDTH 32     /* rows per step (the reference uses at most 17) */
#define BONSAI_ATTN_CHUNK 64    /* KV slots per attention work item */

/* Replaces `_fused_qkv_qknorm_rope_kv_write` (src/bonsai_sft/gpu/model.py:388-436).
 *   xqkv      bf16 [M, (n_heads + 2 n_kv) * 128]   merged q|k|v GEMV output
 *   q_norm_w, k_norm_w  bf16 [128]
 *   cos, sin  bf16 [max_pos, 128]                  RoPE tables (model.py:950-955)
 *   positions int32 [M] (device)                   clamped into [0, max_pos)
 *   q_out     bf16 [M, n_heads, 128]
 *   k_layer, v_layer  bf16 [n_kv, slots, 128]      rows written at slot write_slot + m
 * Rounding points are the eager ones of the reference expression:
 *   n = bf16(w * bf16(fp32(x) * rs)),  rs = 1/sqrt(mean(fp32(x)^2) + eps)
 *   out = bf16( bf16(n * cos) + bf16(rotate_half(n) * sin) );  V is copied. */
int bonsai_qk_norm_rope_kv_write(const void *xqkv, const void *q_norm_w, const void *k_norm_w,
                                 float eps, const void *cos_table, const void *sin_table,
                                 const int32_t *positions, void *q_out, void *k_layer,
                                 void *v_layer, int M, int n_heads, int n_kv, int slots,
                                 int write_slot, int max_pos, void *stream);

/* Process-wide tuning of the attention launch geometry: query rows per wave (1..4), 0 =
 * built-in heuristic.  No counterpart in the reference; results do not depend on it. */
void bonsai_decode_set_tuning(int rows_per_wave);

/* Chunk pass of the attention: 0 = matrix cores (default), 1 = the VALU form (one wave per
 * query head and row group).  Process-wide; no counterpart in the reference; results agree
 * to the tolerance stated below. */
void bonsai_decode_set_attention_engine(int engine);

/* Bytes of scratch `bonsai_decode_attention` needs for the given shape. */
int64_t bonsai_decode_attention_scratch_bytes(int M, int n_heads, int slots);

/* Replaces the attention of `forward_sdlm_graph_kernel` (src/bonsai_sft/gpu/model.py:996-1003)
 * and the quantisation of its output (model.py:1004).
 *   q        bf16 [M, n_heads, 128]
 *   k_layer, v_layer  bf16 [n_kv, slots, 128]
 *   meta     int32 [2 + M] (device), see above; sigma = first workspace slot
 *   scratch  at least bonsai_decode_attention_scratch_bytes(M, n_heads, slots) bytes
 *   out_bf16 bf16 [M, n_heads*128] or NULL
 *   out_q    int8 [M, n_heads*128] and out_s fp32 [M] (multiplier 127/absmax), or both NULL
 * softmax(q k^T * scale + mask) v per head with fp32 accumulation (the probabilities enter
 * the P V product rounded to bf16, as in the reference, model.py:1001); the KV read is
 * bounded by cache_len + M, not by the buffer size.  Compared with a float64 reference
 * within rtol 2e-2 / atol 2e-3 on the bf16 output. */
int bonsai_decode_attention(const void *q, const void *k_layer, const void *v_layer,
                            const int32_t *meta, void *scratch, void *out_bf16, int8_t *out_q,
                            float *out_s, float scale, int M, int n_heads, int n_kv, int slots,
                            int sigma, void *stream);

/* bonsai_qk_norm_rope_kv_write and bonsai_decode_attention as one call (two launches instead of
 * three): the chunk pass of the attention derives its q rows and
 * the block's own K / V rows from the merged projection itself, with the arithmetic and rounding
 * points stated for bonsai_qk_norm_rope_kv_write (same bits), uses them without a round trip
 * through the cache, and writes the K / V rows to slots sigma .. sigma + M - 1 for later steps.
 * No counterpart in the reference beyond the two functions this stands for (model.py:388-436
 * and :996-1004); a one-token decode step spends as long on the separate RoPE launch as on the
 * attention itself, while for blocks of nine rows the two calls are the faster form (every
 * workgroup of the chunk pass repeats the q rows of its tile).  Operands as for those two
 * functions; always the matrix-core chunk pass. */
int bonsai_decode_attention_rope(const void *xqkv, const void *q_norm_w, const void *k_norm_w,
                                 float eps, const void *cos_table, const void *sin_table,
                                 const int32_t *positions, int max_pos, void *k_layer, void *v_layer,
                                 const int32_t *meta, void *scratch, void *out_bf16, int8_t *out_q,
                                 float *out_s, float scale, int M, int n_heads, int n_kv, int slots,
                                 int sigma, void *stream);

/* bonsai_decode_attention_rope in ONE launch, for a projection that quantises from bf16 rows
 * and per-part maxima (t2g128_gemv_fused / q1g128_gemv_fused with BONSAI_ACT_BF16_AMAX, act_parts
 * = n_kv; include/bonsai_gemv.h): the workgroup of a kv head that finishes last merges that kv
 * head's partials itself (the arithmetic of the second launch) and stores
 *   out_bf16 [M, n_heads x 128]            the attention rows, the bits of
 *                                          bonsai_decode_attention(_rope)'s out_bf16;
 *   out_amax bf16 [M, (n_kv + 7) & ~7]     entry [m, h]: max |out_bf16| over the heads of kv head h
 *                                          (the rest zero), so that the projection's multiplier
 *                                          is the out_s of the two-launch form, bit for bit.
 * arrivals: n_kv 32-bit counters (BONSAI_ATTN_MAX_KV_HEADS at most) that are ZERO before the first
 * call; every call leaves them zero.  Calls that share `arrivals` or `scratch` must not overlap.
 * One pair tile only: M x (n_heads / n_kv) <= 16 (BONSAI_DECODE_ERR_ARG otherwise).  No
 * counterpart in the reference, as for bonsai_decode_attention_rope. */
#define BONSAI_ATTN_MAX_KV_HEADS 64
int bonsai_decode_attention_rope_parts(const void *xqkv, const void *q_norm_w, const void *k_norm_w,
                                       float eps, const void *cos_table, const void *sin_table,
                                       const int32_t *positions, int max_pos, void *k_layer,
                                       void *v_layer, const int32_t *meta, void *scratch,
                                       void *arrivals, void *out_bf16, void *out_amax, float scale,
                                       int M, int n_heads, int n_kv, int slots, int sigma,
                                       void *stream);

/* Copies n KV rows of every layer and kv head from slot src to slot dst inside one
 * shared buffer [2, n_layers, n_kv, slots, 128] bf16 (commit_kv / commit_kv_from_verify,
 * src/bonsai_sft/gpu/fast_runtime.py:467-508).  Source and destination ranges must
 * not overlap. */
int bonsai_kv_commit(void *kv, int n_layers, int n_kv, int slots, int src_slot, int dst_slot,
                     int n, void *stream);

/* Row argmax + confidence of the draft logits (`_fused_draft_chain`,
 * src/bonsai_sft/gpu/fast_generate.py:111-130):
 *   logits bf16 [rows, ld], the first `vocab` columns of each row are used
 *   tokens int32 [rows]   argmax (lowest index among equal maxima)
 *   conf   fp32 [rows]    exp(max - logsumexp(row)) in fp32
 *   accept int32 [2]      accept[0] = 1 + longest prefix of rows 1.. with conf > threshold
 *                         (NaN compares false); accept[1] = rows
 * One launch for all rows. */
int bonsai_draft_chain(const void *logits, int rows, int ld, int vocab, float threshold,
                       int32_t *tokens, float *conf, int32_t *accept, void *stream);

/* The same chain with every row split over several workgroups (one workgroup per row is a
 * single CU working through the whole vocabulary): partial statistics go through `scratch`
 * (at least bonsai_draft_chain_scratch_bytes(rows) bytes of device memory, contents
 * undefined afterwards; rows <= BONSAI_MAX_WIDTH).  Same outputs; the confidence may differ
 * from the one-workgroup form in the last place (another summation order). */
int64_t bonsai_draft_chain_scratch_bytes(int rows);
int bonsai_draft_chain_ws(const void *logits, int rows, int ld, int vocab, float threshold,
                          int32_t *tokens, float *conf, int32_t *accept, void *scratch,
                          void *stream);

/* The split chain for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same kernels and outputs as bonsai_draft_chain_ws, but the partial statistics go
 * through a 16 KiB device array owned by the library (one copy per GPU, held until the
 * process ends) instead of a caller workspace; the call allocates and frees nothing.
 * rows <= BONSAI_MAX_WIDTH, larger inputs are refused with BONSAI_DECODE_ERR_ARG.  All calls
 * on one GPU share that array: calls that overlap in time on one GPU (different streams) race.
 * The array's address is looked up once per device, by bonsai_decode_init or by the first
 * call; a first call that arrives on a capturing stream is refused with
 * BONSAI_DECODE_ERR_NOT_INIT and launches nothing. */
int bonsai_draft_chain_static(const void *logits, int rows, int ld, int vocab, float threshold,
                              int32_t *tokens, float *conf, int32_t *accept, void *stream);

/* One-time set-up for the current device of what bonsai_draft_chain_static needs (the device
 * address of the library's scratch array).  Allocates nothing; call it before capturing a graph
 * whose first launch would be that entry point.  No reference counterpart. */
int bonsai_decode_init(void);

/* bf16 output projection of a sign-weight (Q1) backbone, whose graphs keep the tied lm_head
 * in bf16: logits = F.linear(h, W) (`_lm_head`, precision "bf16",
 * src/bonsai_sft/gpu/model.py:1296; chosen in src/bonsai_sft/gpu/fast_runtime.py:175-178).
 *   x bf16 [M, K], w bf16 [N, K] row-major, out bf16 [M, N]; M <= BONSAI_MAX_WIDTH, K % 64 == 0
 * fp32 accumulation in a fixed order (k ascending inside a slice of K, slices left to
 * right), one RNE rounding to bf16.  The reference's library GEMM fixes no order, so the
 * result is compared with an fp32 matmul to one bf16 step.  The first call on a device sets
 * a function attribute: make it outside stream capture. */
int bonsai_bf16_linear(const void *x, const void *w, void *out, int M, int N, int K, void *stream);

/* FP8 draft projection (the acceptance-tolerant `draft_fp8` role): the run-time half of
 * `_lm_head` with precision "fp8" (src/bonsai_sft/gpu/model.py:1268-1275).
 *   h_scale = fp32( max( bf16(amax(|x|) / 448), bf16(1e-12) ) )   one scale for all M rows,
 *                                                     evaluated in bf16 like the tensor expression
 *   q       = e4m3fn( bf16( fp32(x) / h_scale ) )       OCP E4M3, round to nearest even
 * x bf16 [M, K] (M <= BONSAI_MAX_WIDTH, K % 8 == 0), q uint8 [M, K], scale fp32 [1] (device). */
int bonsai_fp8_quant_rows(const void *x, void *q, float *scale, int M, int K, void *stream);

/* out = bf16( (x_fp8 @ w_fp8^T) * x_scale[0] * w_scale ): `torch._scaled_mm(h_fp8, W.T,
 * scale_a, scale_b, out_dtype=bf16)` of model.py:1271-1275, with the weight matrix
 * prepared as in `prepare_fp8_lm_head` (model.py:1168-1194: w_scale = amax(|W|)/448,
 * W_fp8 = e4m3fn(W / w_scale), rows padded to a multiple of 16).
 *   x uint8 [M, K] E4M3, x_scale fp32 [1] (device), w uint8 [N, K] E4M3, out bf16 [M, N];
 *   K % 128 == 0.  fp32 accumulation in a fixed order; compared with a float64 product of the
 * same FP8 operands to one bf16 step.  First call per device outside stream capture. */
int bonsai_fp8_linear(const void *x, const float *x_scale, const void *w, float w_scale, void *out,
                      int M, int N, int K, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BONSAI_DECODE_H */
