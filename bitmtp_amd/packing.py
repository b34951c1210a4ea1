"""Producers of the packed weight layouts the GEMV kernels stream.

Layouts (identical to the reference converter,
src/bonsai_sft/gpu/convert_bonsai_mtp_to_gpu.py:87-144, and to its on-GPU head
packers, src/bonsai_sft/gpu/model.py:1196-1243):

T2-g128  ``weight int8 [N, K/4]``: weight ``k`` is the 2-bit field ``k % 4`` (LSB
         first) of byte ``k // 4`` and holds ``q + 2`` for ``q`` in {-1, 0, +1};
         ``weight_scale bf16 [N, K/128]`` is the group's absmax.
Q1-g128  ``weight int8 [N, K/8]``: weight ``k`` is bit ``k % 8`` (LSB first) of byte
         ``k // 8``, 1 for ``w >= 0``; ``weight_scale bf16 [N, K/128]`` is the group's
         mean magnitude.

These are offline, one-shot tensor programs (any device); they are not on the
decode path.
"""
from __future__ import annotations

from typing import Tuple

import torch

GROUP_SIZE = 128


def _check(w: torch.Tensor) -> Tuple[int, int]:
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise ValueError("expected a rank-2 bfloat16 weight")
    n, k = w.shape
    if k % GROUP_SIZE != 0:
        raise ValueError(f"in_features={k} is not a multiple of {GROUP_SIZE}")
    return n, k


def _pack_fields(values: torch.Tensor, bits: int) -> torch.Tensor:
    """values uint8 [N, K] with entries < 2**bits -> int8 [N, K*bits/8], LSB first."""
    per = 8 // bits
    n, k = values.shape
    fields = values.view(n, k // per, per).to(torch.int32)
    weights = (1 << (bits * torch.arange(per, device=values.device, dtype=torch.int32)))
    packed = (fields * weights).sum(dim=-1).to(torch.uint8)
    return packed.view(torch.int8).contiguous()


@torch.no_grad()
def pack_t2_g128(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 ``[N, K]`` weights on (or near) the ternary grid -> ``(packed, scales)``."""
    n, k = _check(w)
    groups = w.float().view(n, k // GROUP_SIZE, GROUP_SIZE)
    scale = groups.abs().amax(dim=-1).to(torch.bfloat16)
    step = scale.float().clamp_min(1e-30).unsqueeze(-1)
    q = torch.round(groups / step).clamp_(-1, 1)
    codes = (q + 2).to(torch.uint8).view(n, k)
    return _pack_fields(codes, 2), scale.contiguous()


@torch.no_grad()
def pack_q1_g128(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 ``[N, K]`` weights on the sign grid -> ``(packed, scales)``; zero counts as +."""
    n, k = _check(w)
    groups = w.float().view(n, k // GROUP_SIZE, GROUP_SIZE)
    scale = groups.abs().mean(dim=-1).to(torch.bfloat16)
    bits = (w >= 0).to(torch.uint8)
    return _pack_fields(bits, 1), scale.contiguous()


@torch.no_grad()
def unpack_t2_g128(packed: torch.Tensor) -> torch.Tensor:
    """int8 ``[N, K/4]`` -> int8 ``[N, K]`` ternary values (code - 2)."""
    p = packed.view(torch.uint8).to(torch.int32)
    shifts = 2 * torch.arange(4, device=packed.device, dtype=torch.int32)
    return (((p.unsqueeze(-1) >> shifts) & 3) - 2).to(torch.int8).view(packed.shape[0], -1)


@torch.no_grad()
def unpack_q1_g128(packed: torch.Tensor) -> torch.Tensor:
    """int8 ``[N, K/8]`` -> int8 ``[N, K]`` signs (2*bit - 1)."""
    p = packed.view(torch.uint8).to(torch.int32)
    shifts = torch.arange(8, device=packed.device, dtype=torch.int32)
    return (2 * ((p.unsqueeze(-1) >> shifts) & 1) - 1).to(torch.int8).view(packed.shape[0], -1)


def merge_packed_rows(parts):
    """Concatenate packed projections that share their input along the output-row axis,
    weights and group scales alike, so that one GEMV serves q/k/v or gate/up (reference:
    ``prepare_merged_weights``, src/bonsai_sft/gpu/model.py:931-946,1042-1051).

    ``parts`` is a sequence of ``(packed int8 [N_i, bytes], scales [N_i, K/128])``.
    Returns ``(packed [sum N_i, bytes], scales [sum N_i, K/128], [N_i...])``."""
    parts = list(parts)
    cols = {p.shape[1] for p, _ in parts}
    if len(cols) != 1:
        raise ValueError("merged projections must share K")
    packed = torch.cat([p for p, _ in parts], dim=0).contiguous()
    scales = torch.cat([s for _, s in parts], dim=0).contiguous()
    return packed, scales, [p.shape[0] for p, _ in parts]
