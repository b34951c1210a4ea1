/*
 * C ABI of the MI355X (gfx950) packed low-bit GEMV libraries.
 *
 *   libbonsai_t2.so      T2-g128 ternary weights (2-bit codes), int8 activations
 *   libbonsai_q1.so      Q1-g128 sign weights   (1 bit),       int8 activations
 *   libbonsai_actq.so    per-token absmax INT8 activation quantisation
 *
 * Plain pointers and sizes only; every pointer is DEVICE memory unless stated.
 * Nothing here synchronises the host, allocates, frees or retains a pointer;
 * all work is enqueued on `stream` (a hipStream_t passed as void*), so every
 * entry point may be called while that stream is being captured into a graph.
 *
 * Operand layout (identical to the reference kernels,
 * src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:3-8 and
 * src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels.h:14-24):
 *   A   int8  [M, K]        row-major, per-token quantised activations
 *   B   uint8 [N, K/4]      T2: weight k of row n = ((B[n][k/4] >> 2(k%4)) & 3) - 2
 *       uint8 [N, K/8]      Q1: weight k of row n = 2*((B[n][k/8] >> (k%8)) & 1) - 1
 *   ws  16-bit [N, K/128]   one scale per row and 128-wide K group (bf16; the
 *                           *_gemv_ex entry points also read IEEE fp16)
 *   s   fp32  [M]           activation MULTIPLIER 127/absmax (the result is divided by it)
 *   C   bf16  [M, N]        C[m][n] = bf16( (sum_g fp32(G[m][n][g]) * ws[n][g]) / s[m] )
 *   G   int32 [M, N, K/128] exact group sums G[m][n][g] = sum_{k in g} A[m][k] * w[n][k]
 *
 * Preconditions: M >= 1, N >= 1, K >= 128 and K % 128 == 0; A and B 16-byte
 * aligned (every row then is, for K % 128 == 0), s 4-byte, ws 2-byte, C / out
 * aligned to its element: anything else is refused with BONSAI_ERR_ARG.  Any M is
 * accepted: wide blocks are processed as several token tiles.
 */
#ifndef BONSAI_GEMV_H
#define BONSAI_GEMV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes of the int-returning entry points. */
#define BONSAI_OK 0
#define BONSAI_ERR_ARG 1    /* null pointer, M/N/K out of range, K % 128 != 0, misaligned operand */
#define BONSAI_ERR_LAUNCH 2 /* hipLaunchKernel / attribute call failed */
#define BONSAI_ERR_NOT_INIT 3 /* first launch on this device happened on a capturing stream:
                                 call *_init before the capture */

/* ---- drop-in entry points ------------------------------------------------ */

/* Replaces `t2g128_int8xint2_linear`
 * (src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:123-148), bound by ctypes
 * at src/bonsai_sft/gpu/model.py:206-219 with argtypes 5 x void*, 3 x int, void*.
 * Like the reference it returns nothing: on a violated precondition it prints
 * one line to stderr and leaves C untouched.  Unlike the reference it has no
 * table of registered (M,N,K): every shape meeting the preconditions runs. */
void t2g128_int8xint2_linear(int8_t *A, int8_t *B, void *C /* bf16 */, float *s,
                             void *ws /* bf16 */, int M, int N, int K, void *stream);

/* Replaces `q1g128_int8xint1_linear`
 * (src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels_block8.cu:118-241), bound at
 * src/bonsai_sft/gpu/model.py:70-93.  Same contract as above with 1-bit weights. */
void q1g128_int8xint1_linear(int8_t *A, int8_t *B, void *C /* bf16 */, float *s,
                             void *ws /* bf16 */, int M, int N, int K, void *stream);

/* Replaces `q1g128_w1a16_linear`
 * (src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels_block8.cu:93-112): 1-bit
 * weights times bf16 activations with fp32 accumulation and no activation
 * scale, C[m][n] = bf16( sum_g ws[n][g] * sum_{k in g} fp32(A[m][k]) * w[n][k] ).
 * Exported because the reference loader binds it together with the symbol
 * above (model.py:86-91). */
void q1g128_w1a16_linear(const void *A /* bf16 [M,K] */, const int8_t *B, void *C /* bf16 */,
                         const void *ws /* bf16 */, int M, int N, int K, void *stream);

/* ---- checked variants of the same kernels -------------------------------- */
/* Same kernels as the drop-in entry points, selected by `out_kind`, with a
 * status code instead of a message.  They exist so that tests and callers can
 * read the exact int32 group sums and the fp32 value before the bf16 rounding
 * (the reference has no counterpart; its CUDA kernels keep both in registers,
 * t2g128_kernels.cu:74-90). */
#define BONSAI_OUT_BF16 0 /* out = bf16 [M,N]                                  */
#define BONSAI_OUT_F32 1  /* out = fp32 [M,N], value before rounding to bf16  */
#define BONSAI_OUT_G32 2  /* out = int32 [M,N,K/128]; s and ws are not read    */

#define BONSAI_SCALE_BF16 0
#define BONSAI_SCALE_F16 1

int t2g128_gemv_ex(const int8_t *A, const uint8_t *B, void *out, const float *s, const void *ws,
                   int M, int N, int K, int out_kind, int scale_kind, void *stream);
int q1g128_gemv_ex(const int8_t *A, const uint8_t *B, void *out, const float *s, const void *ws,
                   int M, int N, int K, int out_kind, int scale_kind, void *stream);

/* ---- several GEMVs in one launch ------------------------------------------ */
/* No counterpart in the reference, which launches one kernel per projection
 * (src/bonsai_sft/gpu/model.py:977,1006,1058,1062 through t2g128_kernels.cu:94-100).  A
 * layer-sized matrix (0.5-3.3 MB) is far too small to amortise a kernel launch, so GEMVs
 * that do not depend on each other -- q|k|v, gate|up, or a whole layer in a throughput
 * measurement -- can be handed over together: one grid walks the row tiles of all of them.
 * Every descriptor is an independent GEMV with the operands and the result of the
 * single-GEMV entry points above (same arithmetic: exact int32 group sums, fp32 scale
 * accumulation, division by s[m], bf16 RNE; bit-identical to the single call only where both
 * reach the same kernel with the same geometry, otherwise equal within the stated tolerance);
 * widths, row counts and K may differ between descriptors.  `descs` is HOST memory and is read before the call returns; the pointers
 * inside are device pointers.  out_kind / scale_kind apply to all descriptors. */
typedef struct bonsai_gemv_desc {
    const int8_t *A;   /* int8 [M, K] */
    const uint8_t *B;  /* packed weights [N, K/4] (T2) or [N, K/8] (Q1) */
    void *out;         /* bf16 / fp32 [M, N] or int32 [M, N, K/128], see out_kind */
    const float *s;    /* fp32 [M] */
    const void *ws;    /* 16-bit [N, K/128] */
    int32_t M, N, K;
    int32_t reserved;  /* set to 0 */
} bonsai_gemv_desc;
#define BONSAI_GROUPED_MAX 64 /* descriptors per call */
int t2g128_gemv_grouped(const bonsai_gemv_desc *descs, int count, int out_kind, int scale_kind,
                        void *stream);
int q1g128_gemv_grouped(const bonsai_gemv_desc *descs, int count, int out_kind, int scale_kind,
                        void *stream);

/* ---- decode steps of one or two tokens without their element-wise launches ------------ */
/* No counterpart in the reference, which runs a torch.compile'd helper between two projections:
 * residual add + RMSNorm + `quant_input` (src/bonsai_sft/gpu/model.py:307-336, called at
 * :977,1006,1058) or silu(gate) * up + `quant_input` (model.py:1058-1061).  For one or two tokens
 * every launch of a decode step costs about as much as a projection, so these helpers are folded
 * into the projections on either side.  A row-wide value the helper needs (max |x| for the
 * quantisation, sum x^2 for the norm) is left by the projection that produces the row as one
 * PART per workgroup and token, and added up by every wave of the projection that consumes it.
 *
 * epi_kind (what the launch stores):
 *   BONSAI_EPI_PLAIN      out = bf16 / fp32 [M, N] as *_gemv_ex (out_kind BONSAI_OUT_BF16 / _F32)
 *   BONSAI_EPI_SILU_PAIR  B holds the merged rows [gate (N/2 rows); up (N/2 rows)]:
 *                         out = bf16(bf16(silu(gate)) * up) as bf16 [M, N/2]; out_aux = bf16
 *                         [M, ld], ld = parts rounded up to a multiple of 8, 16-byte aligned:
 *                         max |out[m]| over the columns of each workgroup; all of [M, ld] is written
 *   BONSAI_EPI_ADD_SUMSQ  out = bf16(residual + bf16(y)) as bf16 [M, N] (residual bf16 [M, N], may
 *                         be the buffer a later launch overwrites but not `out`); out_aux = fp64
 *                         [M, parts]: sum of out[m]^2 over the columns of each workgroup
 *   parts = *_fused_parts(epi_kind, M, N, K): the workgroups of that launch; depends on the shape only.
 * act_kind (what the launch reads):
 *   BONSAI_ACT_INT8       act int8 [M, K], act_aux = fp32 s[M], as *_gemv_ex
 *   BONSAI_ACT_BF16_AMAX  act bf16 [M, K], act_aux = the bf16 maxima an EPI_SILU_PAIR launch left
 *                         (act_parts of them per token): s[m] = fl(fl(1 / max(amax, 1e-5)) * 127),
 *                         q = clamp(rne(fl(act * s)), -128, 127), as bonsai_act_quant_int8
 *   BONSAI_ACT_BF16_NORM  act = h bf16 [M, K], act_aux = the fp64 sums an EPI_ADD_SUMSQ launch left
 *                         (act_parts per token), norm_weight bf16 [K], eps:
 *                         var = fp32(sum) / K, x = bf16(w * bf16(h * rsqrt(var + eps))), then as
 *                         BONSAI_ACT_BF16_AMAX on max |x|: bonsai_rmsnorm_quant_int8 without its launch
 *   s_out (fp32 [M], may be NULL; BF16 kinds only) receives the multipliers.
 * The operations and rounding points are those of the stand-alone producers between *_gemv_ex
 * calls on the dot4 kernels, so the results are the same bits; the fp64 sum of squares alone is
 * added up in another order (per workgroup, then over the parts), which can show only where two
 * fp64 roundings differ AND the fp32 conversion of the sum straddles a rounding boundary.
 * M <= 2, bf16 weight scales, operands aligned as for *_gemv_ex (act_aux / out_aux: 16 bytes for
 * maxima, 8 for sums).  *_fused_parts returns -1 for a shape these kernels do not take (use the
 * separate launches), -2 / -3 for the set-up failures BONSAI_ERR_LAUNCH / BONSAI_ERR_NOT_INIT. */
#define BONSAI_ACT_INT8 0
#define BONSAI_ACT_BF16_AMAX 1
#define BONSAI_ACT_BF16_NORM 2
#define BONSAI_EPI_PLAIN 0
#define BONSAI_EPI_SILU_PAIR 1
#define BONSAI_EPI_ADD_SUMSQ 2
typedef struct bonsai_fused_gemv {
    const void *act;
    const void *act_aux;
    const void *norm_weight; /* BONSAI_ACT_BF16_NORM only */
    const uint8_t *B;        /* packed weights [N, K/4] (T2) or [N, K/8] (Q1) */
    const void *ws;          /* bf16 [N, K/128] */
    void *out;
    const void *residual;    /* BONSAI_EPI_ADD_SUMSQ only */
    void *out_aux;           /* BONSAI_EPI_SILU_PAIR / _ADD_SUMSQ */
    float *s_out;
    float eps;
    int32_t M, N, K;
    int32_t act_kind, act_parts, epi_kind, out_kind;
} bonsai_fused_gemv;
int t2g128_fused_parts(int epi_kind, int M, int N, int K);
int q1g128_fused_parts(int epi_kind, int M, int N, int K);
int t2g128_gemv_fused(const bonsai_fused_gemv *d, void *stream);
int q1g128_gemv_fused(const bonsai_fused_gemv *d, void *stream);

/* One-time set-up for the current device (raises the kernels' dynamic-LDS
 * limit).  Called implicitly by the first launch; call it explicitly before
 * capturing a graph if the first launch would otherwise happen under capture.
 * No reference counterpart (the CUDA kernels use no shared memory). */
int t2g128_init(void);
int q1g128_init(void);

/* ---- activation quantisation (libbonsai_actq.so) ------------------------- */
/* Per-token symmetric INT8 quantisation, the native form of `quant_input`
 * (src/bonsai_sft/gpu/model.py:632-636, identical copy at :571-575):
 *   s[m] = fl( fl(1 / max(max_k |x[m][k]|, 1e-5)) * 127 )   (fp32; the reference's
 *          `127.0 / tensor` is evaluated by PyTorch as `tensor.reciprocal() * 127.0`)
 *   q[m][k] = clamp(round_half_even(fp32(x[m][k]) * s[m]), -128, 127)
 * x_kind selects the element type of x. */
#define BONSAI_X_BF16 0
#define BONSAI_X_F16 1
#define BONSAI_X_F32 2
int bonsai_act_quant_int8(const void *x, int x_kind, int8_t *q, float *s, int M, int K,
                          void *stream);

/* ---- fused producers of the GEMV input (libbonsai_actq.so) ------------------ */
/* RMSNorm + per-token INT8 quantisation, the native form of `_fused_norm_quant`
 * (src/bonsai_sft/gpu/model.py:307-319): x, w bf16; q int8 [M,K]; s fp32 [M].
 *   var = mean(fp32(x)^2); normed = bf16(w * bf16(fp32(x) * rsqrt(var + eps)));
 *   (q, s) = quantisation of fp32(normed) as in bonsai_act_quant_int8. */
int bonsai_rmsnorm_quant_int8(const void *x, const void *w, float eps, int8_t *q, float *s, int M,
                              int K, void *stream);

/* Residual add + RMSNorm + quantisation, `_fused_add_norm_quant`
 * (src/bonsai_sft/gpu/model.py:322-336): h_out = bf16(x + residual) [M,K] is also
 * returned, then as above on h_out. */
int bonsai_add_rmsnorm_quant_int8(const void *x, const void *residual, const void *w, float eps,
                                  void *h_out, int8_t *q, float *s, int M, int K, void *stream);

/* Residual add + RMSNorm without quantisation: the final `h = h + ffn_out; norm(h[rows])`
 * in front of a bf16 output projection (src/bonsai_sft/gpu/model.py:1401-1402 with
 * `RMSNorm.forward`, model.py:290-295).  n_out = bf16(w * bf16(fp32(h) * rsqrt(var + eps)))
 * [M,K], h = bf16(x + residual), or h = x when residual is NULL; h_out [M,K] receives h
 * when it and residual are not NULL. */
int bonsai_add_rmsnorm_bf16(const void *x, const void *residual, const void *w, float eps,
                            void *h_out, void *n_out, int M, int K, void *stream);

/* SiLU(gate) * up + quantisation of the merged gate/up GEMV output
 * (src/bonsai_sft/gpu/model.py:1058-1061): gate_up bf16 [M, 2F] with the gate in
 * columns [0,F) and up in [F,2F); inner = bf16(bf16(silu(gate)) * up); q int8
 * [M,F], s fp32 [M]. */
int bonsai_silu_mul_quant_int8(const void *gate_up, int8_t *q, float *s, int M, int F, void *stream);

/* ---- development hooks --------------------------------------------------------- */
/* Overrides of the built-in kernel choice and launch geometry, for measurements and for the
 * tests that force every kernel onto small shapes.  Not part of the drop-in surface: no
 * reference counterpart, process-wide, not thread-safe, and a value of zero always restores
 * the built-in choice for that field.  Every kernel computes the arithmetic stated at the top
 * of this file: the int32 group sums are identical whatever is chosen, while the fp32 value
 * may differ in its last bits between kernels and geometries (the order of the fp32 additions
 * over the groups follows the lanes that share a row, and the streaming kernels multiply by
 * an approximate reciprocal of s[m] where the others divide), always within the stated
 * tolerance; the same kernel and geometry give the same bits.
 *
 * set_tuning: the dot4 kernel -- lanes per weight row (4..64, power of two), waves per
 *   workgroup (1..16), row passes per wave (>= 1).
 * set_mfma_tuning: the single-GEMV matrix-core kernels -- smallest width they take (a value
 *   above any M disables them); 16-row tiles per wave (1, 2 or 4); waves of a workgroup that
 *   split K (1, 2, 4, 8, or 3..12 for the one-tile-per-wave form); row blocks a workgroup walks
 *   when K is not split; engine: 1 = int8 MFMA with activations staged in LDS, 3 = int8 MFMA
 *   with activations loaded as operands, 4 = the grouped kernels with one descriptor (the lean
 *   form where it applies), 5 = the streaming kernel on any shape it can run (otherwise only on
 *   very long matrices), 6 = the single-token register kernel on any T2 matrix with K of 1024,
 *   2048 or 4096 (otherwise only on very long ones).
 * set_grouped_tuning: the grouped kernels -- 16-row tiles per wave (1 or 2) and a cap on the
 *   workgroups of one launch (either one set selects the general grouped kernel instead of
 *   its lean form), smallest width sent to the matrix cores (a value above zero also keeps
 *   one- and two-token blocks off the grouped dot4 kernel).
 * set_stream_tuning: the streaming kernels for very long matrices -- smallest packed size in
 *   bytes that is sent to them (negative: never), persistent workgroups per CU. */
void t2g128_set_tuning(int lanes_per_row, int waves_per_wg, int passes);
void q1g128_set_tuning(int lanes_per_row, int waves_per_wg, int passes);
void t2g128_set_mfma_tuning(int min_width, int row_tiles, int k_split, int passes, int engine);
void q1g128_set_mfma_tuning(int min_width, int row_tiles, int k_split, int passes, int engine);
void t2g128_set_grouped_tuning(int row_tiles, int max_wgs, int min_width);
void q1g128_set_grouped_tuning(int row_tiles, int max_wgs, int min_width);
void t2g128_set_stream_tuning(int min_bytes, int wgs_per_cu);
void q1g128_set_stream_tuning(int min_bytes, int wgs_per_cu);

/* Which kernel the calling thread's last launch through this library went to, as
 * "family<template arguments>" (a pointer into thread-local storage, valid until the thread's
 * next call of the same function), and how many kernel launches the thread has made through
 * the library so far.  Read-only diagnostics for tests and benchmarks, which state and assert
 * the kernel a shape reaches; no reference counterpart. */
const char *t2g128_last_kernel(void);
const char *q1g128_last_kernel(void);
int t2g128_launch_count(void);
int q1g128_launch_count(void);

#ifdef __cplusplus
}
#endif
#endif /* BONSAI_GEMV_H */
