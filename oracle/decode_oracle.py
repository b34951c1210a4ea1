"""CPU restatement of the decode-step ops around the packed GEMV -- TEST INFRASTRUCTURE ONLY.

Only ``tests/`` and ``__graft_entry__.smoke()`` may import this module; the product
(``bitmtp_amd``) never does.  NumPy only; bf16 values travel as uint16 bit patterns.

What each function follows in the reference, and what pins it (tests/test_decode_host.py):

* ``dense_mask_draft`` / ``dense_mask_causal``: the additive-mask templates and per-step
  patches of ``GraphAtlas`` (src/bonsai_sft/gpu/fast_runtime.py:316-372,391-465), as
  booleans (True = 0.0, False = -inf).  Pinned by the assertions of the reference's own
  mask tests (tests/test_bonsai_cpu.py:13-42) and by the row-by-row specification in the
  template docstring (fast_runtime.py:316-332).
* ``qk_norm_rope``: ``_fused_qkv_qknorm_rope_kv_write`` (src/bonsai_sft/gpu/model.py:388-436)
  with the eager bf16 rounding points.  Pinned against the same expression evaluated by
  PyTorch's CPU bf16 ops.
* ``attention``: masked softmax attention with GQA (src/bonsai_sft/gpu/model.py:996-1003)
  in float64.  Pinned against ``torch.nn.functional.scaled_dot_product_attention``.
* ``draft_chain`` / ``verify_accept``: fast_generate.py:111-146.  Pinned by the reference's
  known answers (tests/test_orin_runtime.py:146-154, tests/test_bonsai_strict_verifier.py:18-36).
* ``decode_step``: the whole graph forward (model.py:1386-1403) composed from the above and
  the C GEMV / producer oracle; no reference fixture exists for it (random-init weights),
  so it is checked through its parts and used with a tolerance: parity of the end-to-end
  logits is "unpinned" beyond that.
"""
from __future__ import annotations

import numpy as np

from . import oracle as O

HEAD_DIM = 128


# --------------------------------------------------------------------------
# masks
# --------------------------------------------------------------------------
def dense_mask_draft(M: int, sigma: int, D: int, n_pend: int, cache_len: int) -> np.ndarray:
    """Boolean [M, sigma+M] visibility of a draft replay: template
    (fast_runtime.py:345-372) followed by the per-step patch (fast_runtime.py:411-421)."""
    P = M - D
    n_pend = max(0, min(n_pend, P))
    vis = np.zeros((M, sigma + M), dtype=bool)
    for r in range(n_pend):                      # pending-causal
        for c in range(r + 1):
            vis[r, sigma + c] = True
    if n_pend < P:                               # padding rows look at slot 0
        vis[n_pend:P, 0] = True
    for r in range(P, M):                        # block-causal triangle
        for c in range(r - P + 1):
            vis[r, sigma + P + c] = True
    if n_pend > 1:                               # earlier pending rows, not the anchor's twin
        vis[P:, sigma:sigma + n_pend - 1] = True
    if cache_len > 0:
        vis[:, :cache_len] = True
        if n_pend == 0:
            vis[:, cache_len - 1] = False
    return vis


def dense_mask_causal(M: int, sigma: int, cache_len: int, role: str) -> np.ndarray:
    """Boolean [M, sigma+M] visibility of a verify / AR replay
    (fast_runtime.py:423-465)."""
    vis = np.zeros((M, sigma + M), dtype=bool)
    for r in range(M):
        vis[r, sigma:sigma + r + 1] = True
    if cache_len > 0:
        vis[:, :cache_len] = True
    if role != "ar":
        if cache_len <= 0:
            raise RuntimeError("batched verifier requires a committed anchor")
        vis[:, cache_len - 1] = False
    return vis


# --------------------------------------------------------------------------
# q/k norm + RoPE
# --------------------------------------------------------------------------
def _bf(x: np.ndarray) -> np.ndarray:
    """Round fp32 to bf16 and back."""
    return O.bf16_bits_to_f32(O.f32_to_bf16_bits(np.asarray(x, dtype=np.float32)))


def qk_norm_rope(xqkv_bits, qw_bits, kw_bits, eps, cos_bits, sin_bits, positions,
                 n_heads: int, n_kv: int):
    """Returns bf16 bit patterns ``(q [M,n_heads,128], k [M,n_kv,128], v [M,n_kv,128])``.

    n   = bf16(w * bf16(fp32(x) * rs)),  rs = 1/sqrt(mean(x^2) + eps)   (mean via float64)
    out = bf16(bf16(n*cos) + bf16(rotate_half(n)*sin)),  rotate_half(n) = [-n_hi, n_lo]
    """
    X = O.bf16_bits_to_f32(np.asarray(xqkv_bits, dtype=np.uint16))
    M = X.shape[0]
    H = n_heads + 2 * n_kv
    X = X.reshape(M, H, HEAD_DIM)
    cos = O.bf16_bits_to_f32(np.asarray(cos_bits, dtype=np.uint16))[np.asarray(positions)]
    sin = O.bf16_bits_to_f32(np.asarray(sin_bits, dtype=np.uint16))[np.asarray(positions)]

    def norm_rope(x, w_bits):
        w = O.bf16_bits_to_f32(np.asarray(w_bits, dtype=np.uint16))
        sq = (x * x).astype(np.float32).astype(np.float64)
        var = (sq.sum(axis=-1, keepdims=True).astype(np.float32) / np.float32(HEAD_DIM)).astype(np.float32)
        rs = (np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)).astype(np.float32)
        n = _bf(w * _bf(x * rs))
        rot = np.concatenate([-n[..., HEAD_DIM // 2:], n[..., : HEAD_DIM // 2]], axis=-1)
        c = cos[:, None, :]
        s = sin[:, None, :]
        return O.f32_to_bf16_bits(_bf(n * c) + _bf(rot * s))

    q = norm_rope(X[:, :n_heads], qw_bits)
    k = norm_rope(X[:, n_heads:n_heads + n_kv], kw_bits)
    v = O.f32_to_bf16_bits(X[:, n_heads + n_kv:])
    return q, k, v


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------
def attention(q_bits, k_bits, v_bits, vis: np.ndarray, scale: float) -> np.ndarray:
    """float64 ``softmax(q k^T * scale + mask) v`` with grouped KV heads.

    q bf16 bits [M, n_heads, 128]; k, v bf16 bits [n_kv, slots, 128]; vis bool [M, slots'].
    Only the first ``vis.shape[1]`` slots take part.  A row that sees nothing gives zeros.
    Returns float64 [M, n_heads*128]."""
    q = O.bf16_bits_to_f32(np.asarray(q_bits, dtype=np.uint16)).astype(np.float64)
    k = O.bf16_bits_to_f32(np.asarray(k_bits, dtype=np.uint16)).astype(np.float64)
    v = O.bf16_bits_to_f32(np.asarray(v_bits, dtype=np.uint16)).astype(np.float64)
    M, n_heads, _ = q.shape
    n_kv = k.shape[0]
    hpg = n_heads // n_kv
    L = vis.shape[1]
    out = np.zeros((M, n_heads, HEAD_DIM), dtype=np.float64)
    for h in range(n_heads):
        kh = k[h // hpg, :L]
        vh = v[h // hpg, :L]
        s = q[:, h] @ kh.T * scale
        s = np.where(vis, s, -np.inf)
        for r in range(M):
            if not vis[r].any():
                continue
            e = np.exp(s[r] - s[r].max())
            out[r, h] = (e / e.sum()) @ vh
    return out.reshape(M, n_heads * HEAD_DIM)


# --------------------------------------------------------------------------
# draft chain / verifier
# --------------------------------------------------------------------------
def draft_chain(logits: np.ndarray, threshold: float):
    """(argmax tokens, conf, 1 + longest prefix of conf[1:] > threshold)
    (fast_generate.py:111-130); lowest index among equal maxima."""
    x = np.asarray(logits, dtype=np.float32).astype(np.float64)
    tokens = x.argmax(axis=-1)
    mx = x.max(axis=-1)
    lse = mx + np.log(np.exp(x - mx[:, None]).sum(axis=-1))
    conf = np.exp(mx - lse).astype(np.float32)
    n = 1
    for c in conf[1:]:
        if not (c > np.float32(threshold)):
            break
        n += 1
    return tokens.astype(np.int64), conf, n


def verify_accept(draft_tokens, verify_tokens, D: int) -> int:
    """Longest prefix of identical ids (fast_generate.py:133-146)."""
    d = np.asarray(draft_tokens)[:D]
    v = np.asarray(verify_tokens)[:D]
    eq = (d == v).astype(np.int64)
    return int(np.cumprod(eq).sum())


# --------------------------------------------------------------------------
# the whole step (small shapes)
# --------------------------------------------------------------------------
def decode_step(weights: dict, kv_k: np.ndarray, kv_v: np.ndarray, tokens, positions,
                vis: np.ndarray, sigma: int, logits_start: int, logits_end: int):
    """One graph forward (model.py:1386-1403) on the CPU.

    ``weights``: ``embed`` (bf16 bits [vocab, dim]), ``norm``, ``head`` = (packed uint8, scale
    bits) with ``head_bits`` (default ``bits``) or, for the bf16 projection of a sign-weight
    backbone (model.py:1296), ``head_bf16`` = bf16 bits [rows, dim]; ``bits`` = 2 (ternary,
    default) or 1 (sign) for the layers; ``cos``/``sin`` bits, ``eps``, ``n_heads``, ``n_kv``,
    and ``layers`` = list of dicts
    with ``wqkv``/``wo``/``w_gu``/``w_down`` (packed, scale bits), ``input_layernorm``,
    ``post_attention_layernorm``, ``q_norm``, ``k_norm`` (bf16 bits).
    ``kv_k``/``kv_v``: bf16 bits [n_layers, n_kv, slots, 128], updated in place at
    slots sigma..sigma+M-1.  Returns bf16 bits of the logits rows [rows, head_rows].
    """
    eps = weights["eps"]
    n_heads, n_kv = weights["n_heads"], weights["n_kv"]
    M = len(tokens)
    scale = 1.0 / np.sqrt(HEAD_DIM)

    bits = weights.get("bits", 2)

    def gemv(q8, s, w, b=bits):
        _, y_bits = O.c_gemv(q8, w[0], s, w[1], b)
        return y_bits

    h = weights["embed"][np.asarray(tokens)]
    ffn_out = None
    for i, lw in enumerate(weights["layers"]):
        if i == 0:
            a_q, a_s, _ = O.c_rmsnorm_quant(h, lw["input_layernorm"], eps)
        else:
            a_q, a_s, h = O.c_rmsnorm_quant(ffn_out, lw["input_layernorm"], eps, residual_bits=h)
        xqkv = gemv(a_q, a_s, lw["wqkv"])
        q, k, v = qk_norm_rope(xqkv, lw["q_norm"], lw["k_norm"], eps, weights["cos"],
                               weights["sin"], positions, n_heads, n_kv)
        kv_k[i][:, sigma:sigma + M] = k.transpose(1, 0, 2)
        kv_v[i][:, sigma:sigma + M] = v.transpose(1, 0, 2)
        att = attention(q, kv_k[i], kv_v[i], vis, scale)
        att_bits = O.f32_to_bf16_bits(att.astype(np.float32))
        o_q, o_s = O.c_act_quant(O.bf16_bits_to_f32(att_bits))
        attn_out = gemv(o_q, o_s, lw["wo"])
        f_q, f_s, h = O.c_rmsnorm_quant(h, lw["post_attention_layernorm"], eps,
                                        residual_bits=attn_out)
        gu = gemv(f_q, f_s, lw["w_gu"])
        i_q, i_s = O.c_silu_mul_quant(gu)
        ffn_out = gemv(i_q, i_s, lw["w_down"])
    if weights.get("head_bf16") is not None:
        n_bits, _ = O.c_rmsnorm(ffn_out[logits_start:logits_end], weights["norm"], eps,
                                residual_bits=h[logits_start:logits_end])
        # fp32 accumulation of exact bf16 products; float64 here, the order is the library's
        # in the reference, so callers compare with a tolerance of one bf16 step
        y = O.bf16_bits_to_f32(n_bits).astype(np.float64) @ \
            O.bf16_bits_to_f32(weights["head_bf16"]).astype(np.float64).T
        return O.f32_to_bf16_bits(y.astype(np.float32))
    l_q, l_s, _ = O.c_rmsnorm_quant(ffn_out[logits_start:logits_end], weights["norm"], eps,
                                    residual_bits=h[logits_start:logits_end])
    return gemv(l_q, l_s, weights["head"], weights.get("head_bits", bits))
