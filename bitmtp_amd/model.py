"""Packed-ternary Bonsai (Qwen3-shaped) decoder for MI355X: weights and the one
fixed-shape decode step that the graph atlas captures.

The step is the reference's fully kernelised graph forward
(``Transformer.forward_sdlm_decode_graph_kernel``, src/bonsai_sft/gpu/model.py:1386-1403,
with ``TransformerBlock.forward_sdlm_graph_kernel`` :1112-1137,
``Attention.forward_sdlm_graph_kernel`` :958-1009 and
``FeedForward.forward_merged_kernel`` :1053-1064), laid out MI355X-first: every op is
one native launch on pre-allocated buffers,

    embed gather -> [norm+quant | add+norm+quant] -> qkv GEMV -> qk-norm+RoPE+KV write
    -> attention (+quant) -> o GEMV -> add+norm+quant -> gate|up GEMV -> SiLU*up+quant
    -> down GEMV ... -> add+norm+quant (logit rows only) -> packed head GEMV
    -> argmax / confidence chain

so a replayed graph is 10 launches per layer and reads each packed weight once.
PyTorch supplies device memory, the embedding gather and graph capture only.
"""
from __future__ import annotations

import ctypes
import os
import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from . import decode_ops, ops
from .packing import GROUP_SIZE, _pack_fields

HEAD_DIM = decode_ops.HEAD_DIM


@dataclass
class ModelArgs:
    """Same fields and defaults as the reference ``ModelArgs`` (model.py:690-713)."""
    dim: int = 2048
    n_layers: int = 28
    n_heads: int = 16
    n_kv_heads: int = 8
    head_dim: int = 128
    ffn_dim: int = 6144
    vocab_size: int = 151669
    norm_eps: float = 1.0e-6
    rope_theta: float = 1.0e6
    rope_original_max: int = 8192
    rope_factor: float = 4.0
    rope_mscale: float = 1.0
    rope_mscale_all_dim: float = 0.0
    rope_beta_fast: float = 32.0
    rope_beta_slow: float = 1.0
    tie_word_embeddings: bool = True
    use_kernel: bool = True
    kernel_kind: str = "t2g128"
    block_size: int = 8
    causal_attn: bool = True
    mask_token_id: int = 151654

    @property
    def q_dim(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.n_kv_heads * self.head_dim


def qwen3_1p7b_args(**over) -> ModelArgs:
    """Qwen3-1.7B shape: 28 layers, hidden 2048, 16 q / 8 kv heads x 128, ffn 6144."""
    return ModelArgs(**{**dict(vocab_size=151936), **over})


def qwen3_4b_args(**over) -> ModelArgs:
    """Qwen3-4B shape: 36 layers, hidden 2560, 32 q / 8 kv heads x 128, ffn 9728."""
    return ModelArgs(**{**dict(dim=2560, n_layers=36, n_heads=32, n_kv_heads=8, ffn_dim=9728,
                               vocab_size=151936), **over})


# ---------------------------------------------------------------------------
# RoPE tables (reference: `_yarn_inv_freq`, `_yarn_attention_factor`, model.py:342-379,
# and the lookup tables of `prepare_merged_weights`, model.py:950-955)
# ---------------------------------------------------------------------------
def yarn_inv_freq(head_dim: int, base: float, factor: float, original_max: int,
                  beta_fast: float = 32.0, beta_slow: float = 1.0, device=None) -> torch.Tensor:
    dim = head_dim
    idx = torch.arange(0, dim, 2, device=device).float()
    pos_freqs = base ** (idx / dim)
    extrap = 1.0 / pos_freqs
    interp = 1.0 / (factor * pos_freqs)

    def correction_dim(rotations: float) -> float:
        return (dim * math.log(original_max / (rotations * 2 * math.pi))) / (2 * math.log(base))

    low = max(math.floor(correction_dim(beta_fast)), 0)
    high = min(math.ceil(correction_dim(beta_slow)), dim - 1)
    if low == high:
        high += 0.001
    ramp = ((torch.arange(dim // 2, device=device, dtype=torch.float32) - low) / (high - low)).clamp(0.0, 1.0)
    keep = 1.0 - ramp
    return interp * (1.0 - keep) + extrap * keep


def yarn_attention_factor(scale: float, mscale: float = 1.0, mscale_all_dim: float = 0.0) -> float:
    if scale <= 1.0:
        return 1.0

    def g(s, m):
        return 0.1 * m * math.log(s) + 1.0
    if mscale and mscale_all_dim:
        return g(scale, mscale) / g(scale, mscale_all_dim)
    return g(scale, mscale)


def rope_tables(args: ModelArgs, max_positions: int, device) -> Tuple[torch.Tensor, torch.Tensor]:
    inv_freq = yarn_inv_freq(args.head_dim, args.rope_theta, args.rope_factor,
                             args.rope_original_max, args.rope_beta_fast, args.rope_beta_slow,
                             device=device)
    mscale = yarn_attention_factor(args.rope_factor, args.rope_mscale, args.rope_mscale_all_dim)
    pos = torch.arange(max_positions, device=device, dtype=torch.float32)
    freqs = torch.outer(pos, inv_freq.float())
    emb = torch.cat((freqs, freqs), dim=-1)
    return ((emb.cos() * mscale).to(torch.bfloat16).contiguous(),
            (emb.sin() * mscale).to(torch.bfloat16).contiguous())


# ---------------------------------------------------------------------------
# Weights
# ---------------------------------------------------------------------------
@dataclass
class PackedLinear:
    weight: torch.Tensor        # int8 [N, K/4] (ternary, bits = 2) or [N, K/8] (sign, bits = 1)
    weight_scale: torch.Tensor  # bf16 [N, K/128]
    bits: int = 2

    @property
    def out_features(self) -> int:
        return self.weight.shape[0]

    @property
    def in_features(self) -> int:
        return self.weight.shape[1] * (8 // self.bits)


def kind_bits(kernel_kind: str) -> int:
    """Weight bits of a backbone kind: the reference's ``kernel_kind`` is "t2g128" (ternary)
    or "q1" (sign weights), model.py:709."""
    if kernel_kind == "t2g128":
        return 2
    if kernel_kind == "q1":
        return 1
    raise ValueError(f"unknown kernel_kind {kernel_kind!r} (expected 't2g128' or 'q1')")


@dataclass
class LayerWeights:
    """One block with q|k|v and gate|up already merged along the output rows
    (reference: ``prepare_merged_weights``, model.py:931-956 and :1042-1051)."""
    wqkv: PackedLinear
    wo: PackedLinear
    w_gu: PackedLinear
    w_down: PackedLinear
    input_layernorm: torch.Tensor           # bf16 [dim]
    post_attention_layernorm: torch.Tensor  # bf16 [dim]
    q_norm: torch.Tensor                    # bf16 [128]
    k_norm: torch.Tensor                    # bf16 [128]


def _random_packed(n: int, k: int, gen: torch.Generator, device, bits: int = 2) -> PackedLinear:
    """i.i.d. ternary codes (p = 1/3 each) or sign bits (p = 1/2) and log-normal(-4, 0.5)
    group scales."""
    if bits == 2:
        codes = torch.randint(1, 4, (n, k), generator=gen, device=device, dtype=torch.uint8)
    else:
        codes = torch.randint(0, 2, (n, k), generator=gen, device=device, dtype=torch.uint8)
    packed = _pack_fields(codes, bits)
    scale = torch.exp(torch.randn((n, k // GROUP_SIZE), generator=gen, device=device) * 0.5 - 4.0)
    return PackedLinear(packed, scale.to(torch.bfloat16).contiguous(), bits)


def head_rows_for(vocab: int) -> int:
    """The packed head is padded to whole 128-row tiles (the reference pads 151669 to
    151936, model.py:1227); pad rows carry zero scales and are never selected."""
    return -(-vocab // 128) * 128


class BonsaiDecoder:
    """Weights of a packed low-bit decoder plus its step enqueue function.

    ``head`` is the packed output projection (ternary for a "t2g128" backbone, as the
    reference's graphs use, fast_runtime.py:115-118; sign-packed W1A8 for "q1" when asked for,
    model.py:1262-1267), or None: then the logits come from the bf16 matrix ``head_bf16``
    ``[vocab, dim]`` (the tied embedding unless given), which is what the reference's graphs
    do for a "q1" backbone (fast_runtime.py:175-178)."""

    def __init__(self, args: ModelArgs, layers: List[LayerWeights], embed: torch.Tensor,
                 norm: torch.Tensor, head: Optional[PackedLinear],
                 head_bf16: Optional[torch.Tensor] = None):
        if args.head_dim != HEAD_DIM:
            raise ValueError("only head_dim 128 is supported")
        bits = kind_bits(args.kernel_kind)
        if args.dim % GROUP_SIZE or args.ffn_dim % GROUP_SIZE or args.q_dim % GROUP_SIZE:
            raise ValueError("dim, ffn_dim and n_heads*head_dim must be multiples of 128")
        for lw in layers:
            for p in (lw.wqkv, lw.wo, lw.w_gu, lw.w_down):
                if p.bits != bits:
                    raise ValueError(f"a {args.kernel_kind!r} backbone takes {bits}-bit layers")
        self.args = args
        self.layers = layers
        self.embed = embed          # bf16 [vocab, dim]
        self.norm = norm            # bf16 [dim]
        self.head = head            # packed [head_rows, dim*bits/8] or None
        self.device = embed.device
        if head is None:
            w = embed if head_bf16 is None else head_bf16
            if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != args.dim \
                    or w.shape[0] < args.vocab_size:
                raise ValueError("the bf16 head must be bf16 [>= vocab, dim]")
            if w.shape[0] % 8:  # the logits' leading dimension must be a multiple of 8
                padded = torch.zeros(-(-w.shape[0] // 8) * 8, args.dim, dtype=w.dtype, device=w.device)
                padded[: w.shape[0]].copy_(w)
                w = padded
            self.head_bf16 = w.contiguous()
            self.head_rows = self.head_bf16.shape[0]
        else:
            self.head_bf16 = None
            self.head_rows = head.out_features

        self.head_fp8 = None        # (E4M3 codes uint8 [ceil16(vocab), dim], w_scale): draft_fp8
        self.head_raw_bf16 = None   # bf16 [ceil8(vocab), dim]: draft_bf16

    @property
    def head_kind(self) -> str:
        if self.head is None:
            return "bf16"
        return "t2" if self.head.bits == 2 else "q1"

    def _lm_head_weight(self) -> torch.Tensor:
        """The bf16 output matrix ``[vocab, dim]``: the tied embedding (which a packed head
        dequantises to) or the untied matrix (reference: model.py:1160-1166)."""
        w = self.embed if self.head_bf16 is None else self.head_bf16
        return w[: self.args.vocab_size]

    def prepare_fp8_lm_head(self) -> None:
        """E4M3 copy of the output matrix for the ``draft_fp8`` role (reference:
        ``prepare_fp8_lm_head``, model.py:1168-1194)."""
        if self.head_fp8 is None:
            self.head_fp8 = decode_ops.prepare_fp8_weight(self._lm_head_weight())

    def prepare_raw_bf16_head(self) -> None:
        """The raw bf16 output matrix for the ``draft_bf16`` role (reference: precision
        "bf16_raw", model.py:1276-1282), rows padded to a multiple of 8."""
        if self.head_raw_bf16 is None:
            if self.head_bf16 is not None:
                self.head_raw_bf16 = self.head_bf16
                return
            w = self._lm_head_weight()
            if w.shape[0] % 8:
                padded = torch.zeros(-(-w.shape[0] // 8) * 8, w.shape[1], dtype=w.dtype, device=w.device)
                padded[: w.shape[0]].copy_(w)
                w = padded
            self.head_raw_bf16 = w.contiguous()

    def max_logits_ld(self) -> int:
        """Largest leading dimension any prepared output projection writes."""
        ld = self.head_rows
        if self.head_fp8 is not None:
            ld = max(ld, self.head_fp8[0].shape[0])
        if self.head_raw_bf16 is not None:
            ld = max(ld, self.head_raw_bf16.shape[0])
        return ld

    # -- construction --------------------------------------------------------
    @classmethod
    def random_init(cls, args: ModelArgs, seed: int = 0, device="cuda",
                    head_kind: Optional[str] = None) -> "BonsaiDecoder":
        """Random low-bit weights; the embedding is the dequantised tied head, as in a
        converted checkpoint whose tied projection sits on the weight grid (reference:
        ``prepare_t2_lm_head`` / ``prepare_q1_lm_head``, model.py:1196-1243).  ``head_kind``
        "t2", "q1" or "bf16"; by default what the reference's graphs use for the backbone:
        the packed ternary head for "t2g128", the bf16 matrix for "q1"."""
        device = torch.device(device)
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        bits = kind_bits(args.kernel_kind)
        if head_kind is None:
            head_kind = "t2" if bits == 2 else "bf16"
        if head_kind not in ("t2", "q1", "bf16"):
            raise ValueError(f"unknown head_kind {head_kind!r}")
        layers = []
        for _ in range(args.n_layers):
            def ln(n):
                return (1.0 + 0.1 * torch.randn(n, generator=gen, device=device)).to(torch.bfloat16)
            layers.append(LayerWeights(
                wqkv=_random_packed(args.q_dim + 2 * args.kv_dim, args.dim, gen, device, bits),
                wo=_random_packed(args.dim, args.q_dim, gen, device, bits),
                w_gu=_random_packed(2 * args.ffn_dim, args.dim, gen, device, bits),
                w_down=_random_packed(args.dim, args.ffn_dim, gen, device, bits),
                input_layernorm=ln(args.dim), post_attention_layernorm=ln(args.dim),
                q_norm=ln(HEAD_DIM), k_norm=ln(HEAD_DIM)))
        rows = head_rows_for(args.vocab_size)
        head = _random_packed(rows, args.dim, gen, device, 1 if head_kind == "q1" else
                              (2 if head_kind == "t2" else bits))
        if rows > args.vocab_size:
            head.weight_scale[args.vocab_size:] = 0
        embed = dequantize_packed(head)[: args.vocab_size].contiguous()
        norm = (1.0 + 0.1 * torch.randn(args.dim, generator=gen, device=device)).to(torch.bfloat16)
        return cls(args, layers, embed, norm, None if head_kind == "bf16" else head)

    def weight_bytes_per_step(self) -> int:
        """Packed weight + scale bytes one replay streams (head included)."""
        total = 0
        for lw in self.layers:
            for p in (lw.wqkv, lw.wo, lw.w_gu, lw.w_down):
                total += p.weight.numel() + 2 * p.weight_scale.numel()
        if self.head is None:
            return total + 2 * self.head_bf16.numel()
        return total + self.head.weight.numel() + 2 * self.head.weight_scale.numel()


def dequantize_packed(p: PackedLinear) -> torch.Tensor:
    """bf16 [N, K]: ``(code - 2) * scale`` for ternary weights, ``(2 bit - 1) * scale`` for
    sign weights (reference: ``_unpack_to_bf16``, model.py:641-647 and :585-593)."""
    b = p.weight.view(torch.uint8)
    if p.bits == 2:
        shifts = torch.arange(0, 8, 2, device=b.device, dtype=torch.uint8)
        q = ((b.unsqueeze(-1) >> shifts) & 3).to(torch.int8) - 2
    else:
        shifts = torch.arange(0, 8, 1, device=b.device, dtype=torch.uint8)
        q = ((b.unsqueeze(-1) >> shifts) & 1).to(torch.int8) * 2 - 1
    n = b.shape[0]
    q = q.view(n, -1, GROUP_SIZE).to(torch.bfloat16)
    return (q * p.weight_scale.unsqueeze(-1)).view(n, -1)


def dequantize_t2(p: PackedLinear) -> torch.Tensor:
    return dequantize_packed(p)


# ---------------------------------------------------------------------------
# The step
# ---------------------------------------------------------------------------
class Workspace:
    """Intermediate buffers of one step, sized for the widest graph and shared by all
    graphs (they replay one after another on one stream)."""

    def __init__(self, args: ModelArgs, m_max: int, max_slots: int, head_rows: int, device,
                 logits_ld_max: int = 0):
        bf, i8, f32 = torch.bfloat16, torch.int8, torch.float32

        def buf(shape, dtype):
            return torch.zeros(shape, dtype=dtype, device=device)
        self.m_max = m_max
        self.h = [buf((m_max, args.dim), bf), buf((m_max, args.dim), bf)]
        self.a_q = buf((m_max, args.dim), i8)
        self.a_s = buf((m_max,), f32)
        self.xqkv = buf((m_max, args.q_dim + 2 * args.kv_dim), bf)
        self.q = buf((m_max, args.n_heads, HEAD_DIM), bf)
        nbytes = decode_ops.attention_scratch_bytes(m_max, args.n_heads, max_slots)
        self.attn_scratch = buf((nbytes // 4,), f32)
        self.o_q = buf((m_max, args.q_dim), i8)
        self.o_s = buf((m_max,), f32)
        self.attn_out = buf((m_max, args.dim), bf)
        self.f_q = buf((m_max, args.dim), i8)
        self.f_s = buf((m_max,), f32)
        self.gu = buf((m_max, 2 * args.ffn_dim), bf)
        # fused layers (blocks of one or two tokens): SiLU(gate) * up in bf16, the per-workgroup
        # maxima its quantisation needs (at most 1024 per token) and the per-workgroup sums of
        # squares of the residual stream (at most 256 per token)
        self.inner = buf((m_max, args.ffn_dim), bf)
        self.inner_amax = buf((min(m_max, 2), 1024), bf)
        self.sumsq = buf((min(m_max, 2), 256), torch.float64)
        # the attention that merges its own partials: rows as bf16, one maximum per kv head, and the
        # arrival counters of its workgroups (zero between launches)
        self.attn_rows = buf((min(m_max, 2), args.q_dim), bf)
        self.attn_amax = buf((min(m_max, 2), decode_ops.attention_amax_ld(args.n_kv_heads)), bf)
        self.attn_arrivals = buf((decode_ops.ATTN_MAX_KV_HEADS,), torch.int32)
        self.i_q = buf((m_max, args.ffn_dim), i8)
        self.i_s = buf((m_max,), f32)
        self.ffn_out = buf((m_max, args.dim), bf)
        self.h_last = buf((m_max, args.dim), bf)
        self.l_q = buf((m_max, args.dim), i8)
        self.l_s = buf((m_max,), f32)
        self.l_n = buf((m_max, args.dim), bf)
        self.l_f8 = buf((m_max, args.dim), torch.uint8)
        self.l_f8_scale = buf((1,), f32)
        # one buffer for the logits of every output projection; `logits` is its view with
        # the native projection's leading dimension
        self.logits_buf = buf((m_max * max(head_rows, logits_ld_max),), bf)
        self.logits = self.logits_buf[: m_max * head_rows].view(m_max, head_rows)

    def logits_view(self, rows: int, ld: int) -> torch.Tensor:
        return self.logits_buf[: rows * ld].view(rows, ld)


@dataclass
class StepIO:
    """Per-graph inputs and outputs.  ``step_in`` is one int32 vector
    ``[meta (2+M) | positions (M) | tokens (M)]`` so a replay needs a single
    host-to-device copy; ``out`` is ``[argmax tokens (M) | accept (2) | conf bits (M)]``
    so the results come back in a single device-to-host copy."""
    M: int
    step_in: torch.Tensor        # int32 [3M+2] device
    step_in_host: torch.Tensor   # pinned mirror
    out: torch.Tensor            # int32 [2M+2] device
    out_host: torch.Tensor       # pinned mirror
    uploaded: "torch.cuda.Event"  # recorded once step_in_host has been consumed: after the
                                  # eager upload, or after the replay of a graph that carries it
    downloaded: bool = False      # the last replay already copied `out` into `out_host`

    @property
    def meta(self) -> torch.Tensor:
        return self.step_in[: 2 + self.M]

    @property
    def positions(self) -> torch.Tensor:
        return self.step_in[2 + self.M: 2 + 2 * self.M]

    @property
    def tokens(self) -> torch.Tensor:
        return self.step_in[2 + 2 * self.M:]

    @property
    def tokens_out(self) -> torch.Tensor:
        return self.out[: self.M]

    @property
    def accept(self) -> torch.Tensor:
        return self.out[self.M: self.M + 2]

    @property
    def conf(self) -> torch.Tensor:
        return self.out[self.M + 2:].view(torch.float32)

    @classmethod
    def allocate(cls, M: int, device) -> "StepIO":
        return cls(M=M,
                   step_in=torch.zeros(3 * M + 2, dtype=torch.int32, device=device),
                   step_in_host=torch.zeros(3 * M + 2, dtype=torch.int32).pin_memory(),
                   out=torch.zeros(2 * M + 2, dtype=torch.int32, device=device),
                   out_host=torch.zeros(2 * M + 2, dtype=torch.int32).pin_memory(),
                   uploaded=torch.cuda.Event())


def _vp(t: torch.Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr())


def _gemv(a_q: torch.Tensor, a_s: torch.Tensor, w: PackedLinear, out: torch.Tensor, m: int,
          stream: ctypes.c_void_p) -> None:
    fn = ops.t2_lib().t2g128_gemv_ex if w.bits == 2 else ops.q1_lib().q1g128_gemv_ex
    rc = fn(_vp(a_q), _vp(w.weight), _vp(out), _vp(a_s), _vp(w.weight_scale), m, w.out_features,
            w.in_features, ops.OUT_BF16, ops.SCALE_BF16, stream)
    if rc != 0:
        raise RuntimeError(f"{'t2g128' if w.bits == 2 else 'q1g128'}_gemv_ex failed with status {rc}")


@dataclass
class FusedPlan:
    """Parts per token that the three part-writing launches of a fused layer leave
    (``*_fused_parts`` of include/bonsai_gemv.h)."""
    o: int      # o projection: sums of squares
    gu: int     # gate|up projection: maxima
    down: int   # down projection: sums of squares
    attn: int = 0   # attention: maxima, one per kv head, when it merges its own partials (else 0)


def fused_plan(model: "BonsaiDecoder", m: int) -> Optional[FusedPlan]:
    """How a step of width ``m`` runs its layers: with the residual add + RMSNorm + quantisation
    and the SiLU * up + quantisation folded into the projections, q / k norm + RoPE into the
    attention and -- ``attn`` > 0 -- the merge of the attention's partials as well (five launches a
    layer instead of ten; blocks of one or two tokens), or -- ``None`` -- with the separate
    producers (wider blocks, shapes the fused kernels do not take, BONSAI_FUSED_STEP=0)."""
    if m > ops.FUSED_MAX_TOKENS or os.environ.get("BONSAI_FUSED_STEP", "1") == "0":
        return None
    lw = model.layers[0]
    packed = (lw.wqkv, lw.wo, lw.w_gu, lw.w_down)
    if len({p.bits for p in packed}) != 1 or any(p.weight_scale.dtype != torch.bfloat16 for p in packed):
        return None
    bits = lw.wo.bits
    plan = FusedPlan(
        o=ops.fused_parts(ops.EPI_ADD_SUMSQ, m, lw.wo.out_features, lw.wo.in_features, bits=bits),
        gu=ops.fused_parts(ops.EPI_SILU_PAIR, m, lw.w_gu.out_features, lw.w_gu.in_features, bits=bits),
        down=ops.fused_parts(ops.EPI_ADD_SUMSQ, m, lw.w_down.out_features, lw.w_down.in_features, bits=bits))
    if min(plan.o, plan.gu, plan.down) < 1 or max(plan.o, plan.down) > 256 or plan.gu > 1024:
        return None
    a = model.args
    if (m * (a.n_heads // a.n_kv_heads) <= 16 and a.n_kv_heads <= decode_ops.ATTN_MAX_KV_HEADS
            and os.environ.get("BONSAI_ATTENTION_ONE_LAUNCH", "1") != "0"):
        plan.attn = a.n_kv_heads
    return plan


def _fused(w: PackedLinear, m: int, stream: ctypes.c_void_p, *, act, act_aux, act_kind: int, out,
           epi: int, act_parts: int = 0, norm_w=None, eps: float = 0.0, residual=None, out_aux=None) -> None:
    d = ops.FusedGemvDesc(act=act.data_ptr(), act_aux=act_aux.data_ptr(),
                          norm_weight=norm_w.data_ptr() if norm_w is not None else None,
                          B=w.weight.data_ptr(), ws=w.weight_scale.data_ptr(), out=out.data_ptr(),
                          residual=residual.data_ptr() if residual is not None else None,
                          out_aux=out_aux.data_ptr() if out_aux is not None else None, s_out=None,
                          eps=eps, M=m, N=w.out_features, K=w.in_features, act_kind=act_kind,
                          act_parts=act_parts, epi_kind=epi, out_kind=ops.OUT_BF16)
    fn = ops.t2_lib().t2g128_gemv_fused if w.bits == 2 else ops.q1_lib().q1g128_gemv_fused
    rc = fn(ctypes.byref(d), stream)
    if rc != 0:
        raise RuntimeError(f"{'t2g128' if w.bits == 2 else 'q1g128'}_gemv_fused failed with status {rc} "
                           f"(act {act_kind}, epilogue {epi}, M={m}, N={w.out_features}, K={w.in_features})")


def enqueue_step(model: BonsaiDecoder, ws: Workspace, io: StepIO, kv: torch.Tensor, sigma: int,
                 rope: Tuple[torch.Tensor, torch.Tensor], logits_start: int, logits_end: int,
                 threshold: float, head_mode: str = "native") -> None:
    """Enqueue one width-``io.M`` step on the current stream.

    ``kv`` is the shared buffer ``[2, n_layers, n_kv, slots, 128]``; the new rows go to
    slots ``sigma .. sigma+M-1``.  Logit rows ``[logits_start, logits_end)`` are projected
    through the packed head; their argmax, confidence and accepted-prefix length land in
    ``io.tokens_out / io.conf / io.accept`` (rows counted from ``logits_start``).
    ``head_mode``: "native" (the backbone's own projection), "fp8" or "bf16_raw" (the
    approximate draft projections, model.py:1268-1282; prepared beforehand).
    """
    args = model.args
    M = io.M
    dim = args.dim
    eps = float(args.norm_eps)
    actq = ops.actq_lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream(model.device).cuda_stream)
    cos, sin = rope

    def check(rc: int, what: str) -> None:
        if rc != 0:
            raise RuntimeError(f"{what} failed with status {rc}")

    plan = fused_plan(model, M)
    # wider blocks keep the ten-launch layer; BONSAI_ROPE_IN_ATTENTION=1 drops its q / k norm + RoPE
    # launch (same bits; measured slower at nine rows, where every workgroup of the attention
    # repeats sixteen q rows)
    rope_in_attention = (M <= decode_ops.ROPE_FUSED_MAX_WIDTH
                         and os.environ.get("BONSAI_ROPE_IN_ATTENTION", "0") == "1")
    h_cur, h_nxt = ws.h[0][:M], ws.h[1][:M]
    torch.index_select(model.embed, 0, io.tokens, out=h_cur)
    for i, lw in enumerate(model.layers):
        if plan is not None:
            # five launches (six when the attention's merge is a launch of its own): the
            # element-wise producers ride in the projections on either side, the q / k norm +
            # RoPE in the attention;
            # h_cur already holds the residual stream including the previous layer's MLP
            if i == 0:
                check(actq.bonsai_rmsnorm_quant_int8(_vp(h_cur), _vp(lw.input_layernorm), eps,
                                                     _vp(ws.a_q), _vp(ws.a_s), M, dim, stream),
                      "bonsai_rmsnorm_quant_int8")
                _gemv(ws.a_q, ws.a_s, lw.wqkv, ws.xqkv, M, stream)
            else:
                _fused(lw.wqkv, M, stream, act=h_cur, act_aux=ws.sumsq, act_kind=ops.ACT_BF16_NORM,
                       act_parts=plan.down, norm_w=lw.input_layernorm, eps=eps, out=ws.xqkv,
                       epi=ops.EPI_PLAIN)
            if plan.attn:
                decode_ops.decode_attention_rope_parts(ws.xqkv[:M], lw.q_norm, lw.k_norm, eps, cos, sin,
                                                       io.positions, kv[0, i], kv[1, i], io.meta,
                                                       ws.attn_scratch, ws.attn_arrivals, sigma,
                                                       args.n_heads, ws.attn_rows[:M], ws.attn_amax)
                _fused(lw.wo, M, stream, act=ws.attn_rows, act_aux=ws.attn_amax,
                       act_kind=ops.ACT_BF16_AMAX, act_parts=plan.attn, out=h_nxt,
                       epi=ops.EPI_ADD_SUMSQ, residual=h_cur, out_aux=ws.sumsq)
            else:
                decode_ops.decode_attention_rope(ws.xqkv[:M], lw.q_norm, lw.k_norm, eps, cos, sin,
                                                 io.positions, kv[0, i], kv[1, i], io.meta,
                                                 ws.attn_scratch, sigma, args.n_heads,
                                                 out_q=ws.o_q[:M], out_s=ws.o_s[:M])
                _fused(lw.wo, M, stream, act=ws.o_q, act_aux=ws.o_s,
                       act_kind=ops.ACT_INT8, out=h_nxt, epi=ops.EPI_ADD_SUMSQ, residual=h_cur,
                       out_aux=ws.sumsq)
            h_cur, h_nxt = h_nxt, h_cur
            _fused(lw.w_gu, M, stream, act=h_cur, act_aux=ws.sumsq, act_kind=ops.ACT_BF16_NORM,
                   act_parts=plan.o, norm_w=lw.post_attention_layernorm, eps=eps, out=ws.inner,
                   epi=ops.EPI_SILU_PAIR, out_aux=ws.inner_amax)
            _fused(lw.w_down, M, stream, act=ws.inner, act_aux=ws.inner_amax, act_kind=ops.ACT_BF16_AMAX,
                   act_parts=plan.gu, out=h_nxt, epi=ops.EPI_ADD_SUMSQ, residual=h_cur, out_aux=ws.sumsq)
            h_cur, h_nxt = h_nxt, h_cur
            continue
        if i == 0:
            check(actq.bonsai_rmsnorm_quant_int8(_vp(h_cur), _vp(lw.input_layernorm), eps,
                                                 _vp(ws.a_q), _vp(ws.a_s), M, dim, stream),
                  "bonsai_rmsnorm_quant_int8")
        else:
            check(actq.bonsai_add_rmsnorm_quant_int8(_vp(ws.ffn_out), _vp(h_cur),
                                                     _vp(lw.input_layernorm), eps, _vp(h_nxt),
                                                     _vp(ws.a_q), _vp(ws.a_s), M, dim, stream),
                  "bonsai_add_rmsnorm_quant_int8")
            h_cur, h_nxt = h_nxt, h_cur
        _gemv(ws.a_q, ws.a_s, lw.wqkv, ws.xqkv, M, stream)
        if rope_in_attention:
            decode_ops.decode_attention_rope(ws.xqkv[:M], lw.q_norm, lw.k_norm, eps, cos, sin,
                                             io.positions, kv[0, i], kv[1, i], io.meta,
                                             ws.attn_scratch, sigma, args.n_heads,
                                             out_q=ws.o_q[:M], out_s=ws.o_s[:M])
        else:
            decode_ops.qk_norm_rope_kv_write(ws.xqkv[:M], lw.q_norm, lw.k_norm, eps, cos, sin,
                                             io.positions, ws.q[:M], kv[0, i], kv[1, i],
                                             args.n_heads, args.n_kv_heads, sigma)
            decode_ops.decode_attention(ws.q[:M], kv[0, i], kv[1, i], io.meta, ws.attn_scratch, sigma,
                                        out_q=ws.o_q[:M], out_s=ws.o_s[:M])
        _gemv(ws.o_q, ws.o_s, lw.wo, ws.attn_out, M, stream)
        check(actq.bonsai_add_rmsnorm_quant_int8(_vp(h_cur), _vp(ws.attn_out),
                                                 _vp(lw.post_attention_layernorm), eps, _vp(h_nxt),
                                                 _vp(ws.f_q), _vp(ws.f_s), M, dim, stream),
              "bonsai_add_rmsnorm_quant_int8")
        h_cur, h_nxt = h_nxt, h_cur
        _gemv(ws.f_q, ws.f_s, lw.w_gu, ws.gu, M, stream)
        check(actq.bonsai_silu_mul_quant_int8(_vp(ws.gu), _vp(ws.i_q), _vp(ws.i_s), M,
                                              args.ffn_dim, stream),
              "bonsai_silu_mul_quant_int8")
        _gemv(ws.i_q, ws.i_s, lw.w_down, ws.ffn_out, M, stream)

    # the last MLP's result: still to be added (ffn_out + h_cur), or already in the stream (fused layers)
    last_x = ws.ffn_out[logits_start:] if plan is None else h_cur[logits_start:]
    last_res = _vp(h_cur[logits_start:]) if plan is None else None

    rows = logits_end - logits_start
    if head_mode not in ("native", "fp8", "bf16_raw"):
        raise ValueError(f"unknown head_mode {head_mode!r}")
    if head_mode != "native" or model.head is None:
        # projections of the normalised bf16 rows (reference: model.py:1401-1403)
        check(actq.bonsai_add_rmsnorm_bf16(_vp(last_x), last_res, _vp(model.norm), eps, _vp(ws.h_last),
                                           _vp(ws.l_n), rows, dim, stream),
              "bonsai_add_rmsnorm_bf16")
        if head_mode == "fp8":
            if model.head_fp8 is None:
                raise RuntimeError("the FP8 draft projection was not prepared")
            w_q, w_scale = model.head_fp8
            logits = ws.logits_view(rows, w_q.shape[0])
            decode_ops.fp8_quant_rows(ws.l_n[:rows], ws.l_f8, ws.l_f8_scale)
            decode_ops.fp8_linear(ws.l_f8[:rows], ws.l_f8_scale, w_q, w_scale, logits)
        else:
            w = model.head_bf16 if head_mode == "native" else model.head_raw_bf16
            if w is None:
                raise RuntimeError("the raw bf16 draft projection was not prepared")
            logits = ws.logits_view(rows, w.shape[0])
            decode_ops.bf16_linear(ws.l_n[:rows], w, logits)
    else:
        if plan is None:
            check(actq.bonsai_add_rmsnorm_quant_int8(_vp(last_x), last_res, _vp(model.norm), eps,
                                                     _vp(ws.h_last), _vp(ws.l_q), _vp(ws.l_s), rows,
                                                     dim, stream),
                  "bonsai_add_rmsnorm_quant_int8")
        else:
            check(actq.bonsai_rmsnorm_quant_int8(_vp(last_x), _vp(model.norm), eps, _vp(ws.l_q),
                                                 _vp(ws.l_s), rows, dim, stream),
                  "bonsai_rmsnorm_quant_int8")
        logits = ws.logits_view(rows, model.head_rows)
        _gemv(ws.l_q, ws.l_s, model.head, logits, rows, stream)
    # (the attention scratch is free again by now and far larger than the chain needs)
    decode_ops.draft_chain(logits, args.vocab_size, threshold, io.tokens_out, io.conf, io.accept,
                           scratch=ws.attn_scratch)
