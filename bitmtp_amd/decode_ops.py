"""ctypes binding of ``decode_ops/libbonsai_decode.so``: the ops between the packed GEMVs
of one captured decode step (include/bonsai_decode.h).  They take pre-allocated
tensors and launch on the current stream, so all of them can be captured in a graph.

No fallback: a missing library raises.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
HEAD_DIM = 128
MAX_WIDTH = 32
ATTN_CHUNK = 64

_lib = None


def decode_lib_path() -> str:
    return os.path.join(_HERE, "decode_ops", "libbonsai_decode.so")


def load_decode_kernel() -> None:
    global _lib
    so = decode_lib_path()
    if not os.path.exists(so):
        raise RuntimeError(
            f"{so} is missing: build the gfx950 libraries with `python -m bitmtp_amd.build` "
            "(there is no fallback implementation)")
    lib = ctypes.CDLL(so)
    vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    lib.bonsai_qk_norm_rope_kv_write.argtypes = [vp, vp, vp, cf, vp, vp, vp, vp, vp, vp,
                                                 ci, ci, ci, ci, ci, ci, vp]
    lib.bonsai_qk_norm_rope_kv_write.restype = ci
    lib.bonsai_decode_attention_scratch_bytes.argtypes = [ci, ci, ci]
    lib.bonsai_decode_attention_scratch_bytes.restype = ctypes.c_int64
    lib.bonsai_decode_attention.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, cf,
                                            ci, ci, ci, ci, ci, vp]
    lib.bonsai_decode_attention.restype = ci
    lib.bonsai_decode_attention_rope.argtypes = [vp, vp, vp, cf, vp, vp, vp, ci, vp, vp, vp, vp, vp, vp, vp,
                                                 cf, ci, ci, ci, ci, ci, vp]
    lib.bonsai_decode_attention_rope.restype = ci
    lib.bonsai_decode_attention_rope_parts.argtypes = [vp, vp, vp, cf, vp, vp, vp, ci, vp, vp, vp, vp, vp,
                                                       vp, vp, cf, ci, ci, ci, ci, ci, vp]
    lib.bonsai_decode_attention_rope_parts.restype = ci
    lib.bonsai_decode_set_tuning.argtypes = [ci]
    lib.bonsai_decode_set_tuning.restype = None
    lib.bonsai_decode_set_attention_engine.argtypes = [ci]
    lib.bonsai_decode_set_attention_engine.restype = None
    lib.bonsai_kv_commit.argtypes = [vp, ci, ci, ci, ci, ci, ci, vp]
    lib.bonsai_kv_commit.restype = ci
    lib.bonsai_draft_chain.argtypes = [vp, ci, ci, ci, cf, vp, vp, vp, vp]
    lib.bonsai_draft_chain.restype = ci
    lib.bonsai_draft_chain_ws.argtypes = [vp, ci, ci, ci, cf, vp, vp, vp, vp, vp]
    lib.bonsai_draft_chain_ws.restype = ci
    lib.bonsai_draft_chain_static.argtypes = [vp, ci, ci, ci, cf, vp, vp, vp, vp]
    lib.bonsai_draft_chain_static.restype = ci
    lib.bonsai_decode_init.argtypes = []
    lib.bonsai_decode_init.restype = ci
    lib.bonsai_draft_chain_scratch_bytes.argtypes = [ci]
    lib.bonsai_draft_chain_scratch_bytes.restype = ctypes.c_int64
    lib.bonsai_bf16_linear.argtypes = [vp, vp, vp, ci, ci, ci, vp]
    lib.bonsai_bf16_linear.restype = ci
    lib.bonsai_fp8_quant_rows.argtypes = [vp, vp, vp, ci, ci, vp]
    lib.bonsai_fp8_quant_rows.restype = ci
    lib.bonsai_fp8_linear.argtypes = [vp, vp, vp, cf, vp, ci, ci, ci, vp]
    lib.bonsai_fp8_linear.restype = ci
    _lib = lib


def decode_lib() -> ctypes.CDLL:
    if _lib is None:
        load_decode_kernel()
    return _lib


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream(device: torch.device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _need(cond: bool, what: str) -> None:
    if not cond:
        raise RuntimeError(what)


def _check(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    _need(t.is_cuda and t.is_contiguous() and t.dtype == dtype,
          f"{name} must be a contiguous {dtype} CUDA tensor")


def qk_norm_rope_kv_write(xqkv: torch.Tensor, q_norm_w: torch.Tensor, k_norm_w: torch.Tensor,
                          eps: float, cos: torch.Tensor, sin: torch.Tensor,
                          positions: torch.Tensor, q_out: torch.Tensor, k_layer: torch.Tensor,
                          v_layer: torch.Tensor, n_heads: int, n_kv: int, write_slot: int) -> None:
    """Per-head q/k RMSNorm + RoPE + KV write (reference: model.py:388-436).

    ``xqkv`` bf16 ``[M, (n_heads+2 n_kv)*128]``; ``k_layer``/``v_layer`` bf16
    ``[n_kv, slots, 128]``; ``q_out`` bf16 ``[M, n_heads, 128]``; ``positions`` int32 ``[M]``.
    """
    m = xqkv.shape[0]
    for t, name in ((xqkv, "xqkv"), (q_norm_w, "q_norm_w"), (k_norm_w, "k_norm_w"), (cos, "cos"),
                    (sin, "sin"), (q_out, "q_out"), (k_layer, "k_layer"), (v_layer, "v_layer")):
        _check(t, torch.bfloat16, name)
    _check(positions, torch.int32, "positions")
    _need(xqkv.shape == (m, (n_heads + 2 * n_kv) * HEAD_DIM), "xqkv shape mismatch")
    _need(q_out.shape == (m, n_heads, HEAD_DIM), "q_out shape mismatch")
    _need(k_layer.shape == v_layer.shape and k_layer.dim() == 3 and k_layer.shape[0] == n_kv
          and k_layer.shape[2] == HEAD_DIM, "KV layer shape mismatch")
    _need(cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == HEAD_DIM,
          "RoPE table shape mismatch")
    _need(positions.numel() == m and q_norm_w.numel() == HEAD_DIM and k_norm_w.numel() == HEAD_DIM,
          "positions / norm weight size mismatch")
    slots = k_layer.shape[1]
    with torch.cuda.device(xqkv.device):
        rc = decode_lib().bonsai_qk_norm_rope_kv_write(
            _ptr(xqkv), _ptr(q_norm_w), _ptr(k_norm_w), float(eps), _ptr(cos), _ptr(sin),
            _ptr(positions), _ptr(q_out), _ptr(k_layer), _ptr(v_layer), m, n_heads, n_kv, slots,
            int(write_slot), cos.shape[0], _stream(xqkv.device))
    _need(rc == 0, f"bonsai_qk_norm_rope_kv_write failed with status {rc}")


def attention_scratch_bytes(m: int, n_heads: int, slots: int) -> int:
    return int(decode_lib().bonsai_decode_attention_scratch_bytes(m, n_heads, slots))


def decode_attention(q: torch.Tensor, k_layer: torch.Tensor, v_layer: torch.Tensor,
                     meta: torch.Tensor, scratch: torch.Tensor, sigma: int,
                     out_bf16: Optional[torch.Tensor] = None,
                     out_q: Optional[torch.Tensor] = None, out_s: Optional[torch.Tensor] = None,
                     scale: Optional[float] = None) -> None:
    """Attention of the M new rows over the shared KV under the step descriptor ``meta``
    (int32 ``[2+M]``: cache_len, hidden slot or -1, one workspace-visibility word per row),
    optionally followed by the per-token quantisation of the result
    (reference: model.py:996-1005, fast_runtime.py:391-465)."""
    _check(q, torch.bfloat16, "q")
    _check(k_layer, torch.bfloat16, "k_layer")
    _check(v_layer, torch.bfloat16, "v_layer")
    _check(meta, torch.int32, "meta")
    m, n_heads = q.shape[0], q.shape[1]
    n_kv, slots = k_layer.shape[0], k_layer.shape[1]
    _need(q.dim() == 3 and q.shape[2] == HEAD_DIM, "q must be [M, n_heads, 128]")
    _need(k_layer.shape == v_layer.shape and k_layer.shape[2] == HEAD_DIM, "KV layer shape mismatch")
    _need(meta.numel() >= 2 + m, "meta needs 2 + M entries")
    _need(scratch.is_cuda and scratch.is_contiguous()
          and scratch.numel() * scratch.element_size() >= attention_scratch_bytes(m, n_heads, slots),
          "attention scratch too small")
    if out_bf16 is not None:
        _check(out_bf16, torch.bfloat16, "out_bf16")
        _need(out_bf16.numel() == m * n_heads * HEAD_DIM, "out_bf16 size mismatch")
    if out_q is not None or out_s is not None:
        _need(out_q is not None and out_s is not None, "out_q and out_s come together")
        _check(out_q, torch.int8, "out_q")
        _check(out_s, torch.float32, "out_s")
        _need(out_q.numel() == m * n_heads * HEAD_DIM and out_s.numel() == m, "out_q/out_s size mismatch")
    if scale is None:
        scale = 1.0 / math.sqrt(HEAD_DIM)
    with torch.cuda.device(q.device):
        rc = decode_lib().bonsai_decode_attention(
            _ptr(q), _ptr(k_layer), _ptr(v_layer), _ptr(meta), _ptr(scratch), _ptr(out_bf16),
            _ptr(out_q), _ptr(out_s), float(scale), m, n_heads, n_kv, slots, int(sigma),
            _stream(q.device))
    _need(rc == 0, f"bonsai_decode_attention failed with status {rc}")


ROPE_FUSED_MAX_WIDTH = MAX_WIDTH


def decode_attention_rope(xqkv: torch.Tensor, q_norm_w: torch.Tensor, k_norm_w: torch.Tensor, eps: float,
                          cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                          k_layer: torch.Tensor, v_layer: torch.Tensor, meta: torch.Tensor,
                          scratch: torch.Tensor, sigma: int, n_heads: int,
                          out_bf16: Optional[torch.Tensor] = None, out_q: Optional[torch.Tensor] = None,
                          out_s: Optional[torch.Tensor] = None, scale: Optional[float] = None) -> None:
    """:func:`qk_norm_rope_kv_write` and :func:`decode_attention` in two launches instead of three,
    the attention derives q and the block's own K / V rows from the
    merged projection ``xqkv`` itself (same bits) and writes the K / V rows to slots ``sigma ..``
    (reference: model.py:388-436 and :996-1005)."""
    m = xqkv.shape[0]
    n_kv, slots = k_layer.shape[0], k_layer.shape[1]
    for t, name in ((xqkv, "xqkv"), (q_norm_w, "q_norm_w"), (k_norm_w, "k_norm_w"), (cos, "cos"),
                    (sin, "sin"), (k_layer, "k_layer"), (v_layer, "v_layer")):
        _check(t, torch.bfloat16, name)
    _check(positions, torch.int32, "positions")
    _check(meta, torch.int32, "meta")
    _need(1 <= m <= ROPE_FUSED_MAX_WIDTH, f"1..{ROPE_FUSED_MAX_WIDTH} rows")
    _need(xqkv.shape == (m, (n_heads + 2 * n_kv) * HEAD_DIM), "xqkv shape mismatch")
    _need(k_layer.shape == v_layer.shape and k_layer.dim() == 3 and k_layer.shape[2] == HEAD_DIM,
          "KV layer shape mismatch")
    _need(cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == HEAD_DIM,
          "RoPE table shape mismatch")
    _need(positions.numel() == m and q_norm_w.numel() == HEAD_DIM and k_norm_w.numel() == HEAD_DIM,
          "positions / norm weight size mismatch")
    _need(meta.numel() >= 2 + m, "meta needs 2 + M entries")
    _need(scratch.is_cuda and scratch.is_contiguous()
          and scratch.numel() * scratch.element_size() >= attention_scratch_bytes(m, n_heads, slots),
          "attention scratch too small")
    if out_bf16 is not None:
        _check(out_bf16, torch.bfloat16, "out_bf16")
        _need(out_bf16.numel() == m * n_heads * HEAD_DIM, "out_bf16 size mismatch")
    if out_q is not None or out_s is not None:
        _need(out_q is not None and out_s is not None, "out_q and out_s come together")
        _check(out_q, torch.int8, "out_q")
        _check(out_s, torch.float32, "out_s")
        _need(out_q.numel() == m * n_heads * HEAD_DIM and out_s.numel() == m, "out_q/out_s size mismatch")
    if scale is None:
        scale = 1.0 / math.sqrt(HEAD_DIM)
    with torch.cuda.device(xqkv.device):
        rc = decode_lib().bonsai_decode_attention_rope(
            _ptr(xqkv), _ptr(q_norm_w), _ptr(k_norm_w), float(eps), _ptr(cos), _ptr(sin), _ptr(positions),
            cos.shape[0], _ptr(k_layer), _ptr(v_layer), _ptr(meta), _ptr(scratch), _ptr(out_bf16),
            _ptr(out_q), _ptr(out_s), float(scale), m, n_heads, n_kv, slots, int(sigma),
            _stream(xqkv.device))
    _need(rc == 0, f"bonsai_decode_attention_rope failed with status {rc}")


ATTN_MAX_KV_HEADS = 64


def attention_amax_ld(n_kv: int) -> int:
    """Row pitch of the maxima :func:`decode_attention_rope_parts` leaves (one per kv head)."""
    return (n_kv + 7) & ~7


def decode_attention_rope_parts(xqkv: torch.Tensor, q_norm_w: torch.Tensor, k_norm_w: torch.Tensor,
                                eps: float, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                                k_layer: torch.Tensor, v_layer: torch.Tensor, meta: torch.Tensor,
                                scratch: torch.Tensor, arrivals: torch.Tensor, sigma: int, n_heads: int,
                                out_bf16: torch.Tensor, out_amax: torch.Tensor,
                                scale: Optional[float] = None) -> None:
    """:func:`decode_attention_rope` in one launch: the last workgroup of every kv head merges the
    partials itself and leaves the rows as bf16 plus one maximum per (row, kv head) in
    ``out_amax [M, attention_amax_ld(n_kv)]`` -- what ``packed_gemv_fused(..., amax=out_amax,
    parts=n_kv)`` quantises from, to the bits of the two-launch form.  ``arrivals``: int32
    counters, one per kv head, zero before the first call (every call leaves them zero)."""
    m = xqkv.shape[0]
    n_kv, slots = k_layer.shape[0], k_layer.shape[1]
    for t, name in ((xqkv, "xqkv"), (q_norm_w, "q_norm_w"), (k_norm_w, "k_norm_w"), (cos, "cos"),
                    (sin, "sin"), (k_layer, "k_layer"), (v_layer, "v_layer"), (out_bf16, "out_bf16"),
                    (out_amax, "out_amax")):
        _check(t, torch.bfloat16, name)
    _check(positions, torch.int32, "positions")
    _check(meta, torch.int32, "meta")
    _check(arrivals, torch.int32, "arrivals")
    _need(n_heads % n_kv == 0 and 1 <= m and m * (n_heads // n_kv) <= 16,
          "one pair tile only: rows x heads per kv head <= 16")
    _need(n_kv <= ATTN_MAX_KV_HEADS and arrivals.numel() >= n_kv, "one arrival counter per kv head")
    _need(xqkv.shape == (m, (n_heads + 2 * n_kv) * HEAD_DIM), "xqkv shape mismatch")
    _need(k_layer.shape == v_layer.shape and k_layer.dim() == 3 and k_layer.shape[2] == HEAD_DIM,
          "KV layer shape mismatch")
    _need(cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == HEAD_DIM,
          "RoPE table shape mismatch")
    _need(positions.numel() == m and q_norm_w.numel() == HEAD_DIM and k_norm_w.numel() == HEAD_DIM,
          "positions / norm weight size mismatch")
    _need(meta.numel() >= 2 + m, "meta needs 2 + M entries")
    _need(scratch.is_cuda and scratch.is_contiguous()
          and scratch.numel() * scratch.element_size() >= attention_scratch_bytes(m, n_heads, slots),
          "attention scratch too small")
    _need(out_bf16.numel() == m * n_heads * HEAD_DIM, "out_bf16 size mismatch")
    _need(out_amax.numel() >= m * attention_amax_ld(n_kv), "out_amax too small")
    if scale is None:
        scale = 1.0 / math.sqrt(HEAD_DIM)
    with torch.cuda.device(xqkv.device):
        rc = decode_lib().bonsai_decode_attention_rope_parts(
            _ptr(xqkv), _ptr(q_norm_w), _ptr(k_norm_w), float(eps), _ptr(cos), _ptr(sin), _ptr(positions),
            cos.shape[0], _ptr(k_layer), _ptr(v_layer), _ptr(meta), _ptr(scratch), _ptr(arrivals),
            _ptr(out_bf16), _ptr(out_amax), float(scale), m, n_heads, n_kv, slots, int(sigma),
            _stream(xqkv.device))
    _need(rc == 0, f"bonsai_decode_attention_rope_parts failed with status {rc}")


def kv_commit(kv: torch.Tensor, src_slot: int, dst_slot: int, n: int) -> None:
    """Copy ``n`` rows of every layer / kv head from slot ``src_slot`` to ``dst_slot`` of a
    shared buffer ``[2, n_layers, n_kv, slots, 128]`` (reference: fast_runtime.py:467-508)."""
    _check(kv, torch.bfloat16, "kv")
    _need(kv.dim() == 5 and kv.shape[0] == 2 and kv.shape[4] == HEAD_DIM,
          "kv must be [2, n_layers, n_kv, slots, 128]")
    if n <= 0:
        return
    with torch.cuda.device(kv.device):
        rc = decode_lib().bonsai_kv_commit(_ptr(kv), kv.shape[1], kv.shape[2], kv.shape[3],
                                           int(src_slot), int(dst_slot), int(n), _stream(kv.device))
    _need(rc == 0, f"bonsai_kv_commit failed with status {rc}")


def draft_chain(logits: torch.Tensor, vocab: int, threshold: float, tokens: torch.Tensor,
                conf: torch.Tensor, accept: torch.Tensor,
                scratch: Optional[torch.Tensor] = None) -> None:
    """Row argmax, confidence ``exp(max - logsumexp)`` and the accepted-prefix length
    ``1 + longest prefix of rows 1.. with conf > threshold`` (reference:
    fast_generate.py:111-130).  ``logits`` bf16 ``[rows, ld]``; outputs are pre-allocated
    int32 ``[rows]``, fp32 ``[rows]`` and int32 ``[2]``."""
    _check(logits, torch.bfloat16, "logits")
    _check(tokens, torch.int32, "tokens")
    _check(conf, torch.float32, "conf")
    _check(accept, torch.int32, "accept")
    rows, ld = logits.shape
    _need(tokens.numel() >= rows and conf.numel() >= rows and accept.numel() >= 2,
          "draft_chain output buffers too small")
    with torch.cuda.device(logits.device):
        if scratch is not None:
            # rows split over several workgroups, partial statistics through `scratch`
            need = int(decode_lib().bonsai_draft_chain_scratch_bytes(rows))
            _need(scratch.is_cuda and scratch.is_contiguous()
                  and scratch.numel() * scratch.element_size() >= need, "draft_chain scratch too small")
            rc = decode_lib().bonsai_draft_chain_ws(_ptr(logits), rows, ld, int(vocab),
                                                    float(threshold), _ptr(tokens), _ptr(conf),
                                                    _ptr(accept), _ptr(scratch), _stream(logits.device))
        else:
            rc = decode_lib().bonsai_draft_chain(_ptr(logits), rows, ld, int(vocab), float(threshold),
                                                 _ptr(tokens), _ptr(conf), _ptr(accept),
                                                 _stream(logits.device))
    _need(rc == 0, f"bonsai_draft_chain failed with status {rc}")


def bf16_linear(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out = x @ w.T`` for a few bf16 rows ``x [M, K]`` and a bf16 matrix ``w [N, K]`` with
    fp32 accumulation: the bf16 lm_head of a sign-weight backbone (reference: ``_lm_head``
    with precision "bf16", model.py:1296).  ``out`` bf16 ``[M, N]`` is allocated when absent."""
    _check(x, torch.bfloat16, "x")
    _check(w, torch.bfloat16, "w")
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], "x [M, K] and w [N, K] must share K")
    m, k = x.shape
    n = w.shape[0]
    _need(1 <= m <= MAX_WIDTH, f"bf16_linear takes 1..{MAX_WIDTH} rows")
    _need(k % 64 == 0 and k >= 64, "K must be a multiple of 64")
    if out is None:
        out = torch.empty(m, n, dtype=torch.bfloat16, device=x.device)
    else:
        _check(out, torch.bfloat16, "out")
        _need(out.numel() >= m * n, "out too small")
    with torch.cuda.device(x.device):
        rc = decode_lib().bonsai_bf16_linear(_ptr(x), _ptr(w), _ptr(out), m, n, k, _stream(x.device))
    _need(rc == 0, f"bonsai_bf16_linear failed with status {rc}")
    return out


FP8_MAX = 448.0


def prepare_fp8_weight(w: torch.Tensor):
    """``(w_fp8 uint8 [ceil16(N), K], w_scale float)``: per-tensor scale ``amax|w| / 448`` and
    E4M3 codes of ``w / w_scale`` with the rows padded to a multiple of 16 (reference:
    ``prepare_fp8_lm_head``, model.py:1168-1194).  Done once at load time with torch's own cast."""
    _need(w.dtype == torch.bfloat16 and w.dim() == 2, "w must be bf16 [N, K]")
    n, k = w.shape
    n_pad = -(-n // 16) * 16
    wp = w
    if n_pad != n:
        wp = torch.zeros(n_pad, k, dtype=w.dtype, device=w.device)
        wp[:n].copy_(w)
    w_scale = (wp.abs().amax() / FP8_MAX).clamp_min(1e-12).to(torch.float32)
    codes = (wp / w_scale).to(torch.float8_e4m3fn).view(torch.uint8).contiguous()
    return codes, float(w_scale.item())


def fp8_quant_rows(x: torch.Tensor, q: Optional[torch.Tensor] = None,
                   scale: Optional[torch.Tensor] = None):
    """Per-tensor E4M3 quantisation of a few bf16 rows: ``(q uint8 [M, K], scale fp32 [1])``
    with ``scale = bf16(amax|x| / 448)`` and ``q = e4m3(bf16(x / scale))`` (reference:
    model.py:1269-1270)."""
    _check(x, torch.bfloat16, "x")
    _need(x.dim() == 2 and 1 <= x.shape[0] <= MAX_WIDTH and x.shape[1] % 8 == 0,
          f"x must be [1..{MAX_WIDTH}, K] with K a multiple of 8")
    m, k = x.shape
    if q is None:
        q = torch.empty(m, k, dtype=torch.uint8, device=x.device)
    if scale is None:
        scale = torch.empty(1, dtype=torch.float32, device=x.device)
    _check(q, torch.uint8, "q")
    _check(scale, torch.float32, "scale")
    _need(q.numel() >= m * k and scale.numel() >= 1, "fp8 output buffers too small")
    with torch.cuda.device(x.device):
        rc = decode_lib().bonsai_fp8_quant_rows(_ptr(x), _ptr(q), _ptr(scale), m, k, _stream(x.device))
    _need(rc == 0, f"bonsai_fp8_quant_rows failed with status {rc}")
    return q, scale


def fp8_linear(x_q: torch.Tensor, x_scale: torch.Tensor, w_q: torch.Tensor, w_scale: float,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``bf16((x_q @ w_q.T) * x_scale * w_scale)`` for E4M3 codes ``x_q uint8 [M, K]`` and
    ``w_q uint8 [N, K]`` (reference: ``torch._scaled_mm`` call of model.py:1271-1275)."""
    _check(x_q, torch.uint8, "x_q")
    _check(w_q, torch.uint8, "w_q")
    _check(x_scale, torch.float32, "x_scale")
    _need(x_q.dim() == 2 and w_q.dim() == 2 and x_q.shape[1] == w_q.shape[1], "x_q and w_q must share K")
    m, k = x_q.shape
    n = w_q.shape[0]
    _need(1 <= m <= MAX_WIDTH and k % 128 == 0 and k >= 128, "fp8_linear: 1..32 rows, K a multiple of 128")
    if out is None:
        out = torch.empty(m, n, dtype=torch.bfloat16, device=x_q.device)
    else:
        _check(out, torch.bfloat16, "out")
        _need(out.numel() >= m * n, "out too small")
    with torch.cuda.device(x_q.device):
        rc = decode_lib().bonsai_fp8_linear(_ptr(x_q), _ptr(x_scale), _ptr(w_q), float(w_scale),
                                            _ptr(out), m, n, k, _stream(x_q.device))
    _need(rc == 0, f"bonsai_fp8_linear failed with status {rc}")
    return out
