"""Packed low-bit GEMV operators for MI355X, mirroring the reference's operator
boundary (src/bonsai_sft/gpu/model.py:66-268): the same function names, argument
meaning, output shape/dtype and error behaviour, bound with ctypes to the gfx950
libraries built by ``bitmtp_amd.build``.

There is no CPU or PyTorch fallback: if a library is missing the loaders raise.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional, Sequence, Tuple

import torch

from .contracts import require_kernel_shape

_HERE = os.path.dirname(os.path.abspath(__file__))

OUT_BF16, OUT_F32, OUT_G32 = 0, 1, 2
SCALE_BF16, SCALE_F16 = 0, 1
_X_KIND = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

_t2_lib = None
_q1_lib = None
_actq_lib = None

_GEMV_ARGTYPES = [
    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
    ctypes.c_void_p, ctypes.c_void_p,
    ctypes.c_int, ctypes.c_int, ctypes.c_int,
    ctypes.c_void_p,
]
_GEMV_EX_ARGTYPES = [
    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
    ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
]
ACT_INT8, ACT_BF16_AMAX, ACT_BF16_NORM = 0, 1, 2
EPI_PLAIN, EPI_SILU_PAIR, EPI_ADD_SUMSQ = 0, 1, 2


class FusedGemvDesc(ctypes.Structure):
    """``bonsai_fused_gemv`` of include/bonsai_gemv.h."""
    _fields_ = [("act", ctypes.c_void_p), ("act_aux", ctypes.c_void_p), ("norm_weight", ctypes.c_void_p),
                ("B", ctypes.c_void_p), ("ws", ctypes.c_void_p), ("out", ctypes.c_void_p),
                ("residual", ctypes.c_void_p), ("out_aux", ctypes.c_void_p), ("s_out", ctypes.c_void_p),
                ("eps", ctypes.c_float), ("M", ctypes.c_int32), ("N", ctypes.c_int32), ("K", ctypes.c_int32),
                ("act_kind", ctypes.c_int32), ("act_parts", ctypes.c_int32), ("epi_kind", ctypes.c_int32),
                ("out_kind", ctypes.c_int32)]


class GemvDesc(ctypes.Structure):
    """``bonsai_gemv_desc`` of include/bonsai_gemv.h: one GEMV of a grouped call."""
    _fields_ = [("A", ctypes.c_void_p), ("B", ctypes.c_void_p), ("out", ctypes.c_void_p),
                ("s", ctypes.c_void_p), ("ws", ctypes.c_void_p),
                ("M", ctypes.c_int32), ("N", ctypes.c_int32), ("K", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


GROUPED_MAX = 64
_GROUPED_ARGTYPES = [ctypes.POINTER(GemvDesc), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                     ctypes.c_void_p]


def _open(relpath: str) -> ctypes.CDLL:
    so = os.path.join(_HERE, relpath)
    if not os.path.exists(so):
        raise RuntimeError(
            f"{so} is missing: build the gfx950 libraries with `python -m bitmtp_amd.build` "
            "(there is no fallback implementation)")
    return ctypes.CDLL(so)


def t2_lib_path() -> str:
    return os.path.join(_HERE, "t2g128_kernels", "libbonsai_t2.so")


def q1_lib_path() -> str:
    return os.path.join(_HERE, "q1g128_kernels", "libbonsai_q1.so")


def actq_lib_path() -> str:
    return os.path.join(_HERE, "act_quant", "libbonsai_actq.so")


def load_t2_kernel() -> None:
    """Load the T2-g128 INT8 x packed-INT2 library (reference: model.py:206-219)."""
    global _t2_lib
    lib = _open(os.path.join("t2g128_kernels", "libbonsai_t2.so"))
    lib.t2g128_int8xint2_linear.argtypes = _GEMV_ARGTYPES
    lib.t2g128_int8xint2_linear.restype = None
    lib.t2g128_gemv_ex.argtypes = _GEMV_EX_ARGTYPES
    lib.t2g128_gemv_ex.restype = ctypes.c_int
    lib.t2g128_init.argtypes = []
    lib.t2g128_init.restype = ctypes.c_int
    lib.t2g128_set_tuning.argtypes = [ctypes.c_int] * 3
    lib.t2g128_set_tuning.restype = None
    lib.t2g128_set_mfma_tuning.argtypes = [ctypes.c_int] * 5
    lib.t2g128_set_mfma_tuning.restype = None
    lib.t2g128_gemv_grouped.argtypes = _GROUPED_ARGTYPES
    lib.t2g128_gemv_grouped.restype = ctypes.c_int
    lib.t2g128_set_grouped_tuning.argtypes = [ctypes.c_int] * 3
    lib.t2g128_set_grouped_tuning.restype = None
    lib.t2g128_set_stream_tuning.argtypes = [ctypes.c_int] * 2
    lib.t2g128_set_stream_tuning.restype = None
    lib.t2g128_last_kernel.argtypes = []
    lib.t2g128_last_kernel.restype = ctypes.c_char_p
    lib.t2g128_launch_count.argtypes = []
    lib.t2g128_launch_count.restype = ctypes.c_int
    lib.t2g128_fused_parts.argtypes = [ctypes.c_int] * 4
    lib.t2g128_fused_parts.restype = ctypes.c_int
    lib.t2g128_gemv_fused.argtypes = [ctypes.POINTER(FusedGemvDesc), ctypes.c_void_p]
    lib.t2g128_gemv_fused.restype = ctypes.c_int
    _t2_lib = lib


def load_q1_kernel() -> None:
    """Load the Q1-g128 INT8 x packed-INT1 library (reference: model.py:70-93)."""
    global _q1_lib
    lib = _open(os.path.join("q1g128_kernels", "libbonsai_q1.so"))
    lib.q1g128_int8xint1_linear.argtypes = _GEMV_ARGTYPES
    lib.q1g128_int8xint1_linear.restype = None
    lib.q1g128_w1a16_linear.argtypes = [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
    ]
    lib.q1g128_w1a16_linear.restype = None
    lib.q1g128_gemv_ex.argtypes = _GEMV_EX_ARGTYPES
    lib.q1g128_gemv_ex.restype = ctypes.c_int
    lib.q1g128_init.argtypes = []
    lib.q1g128_init.restype = ctypes.c_int
    lib.q1g128_set_tuning.argtypes = [ctypes.c_int] * 3
    lib.q1g128_set_tuning.restype = None
    lib.q1g128_set_mfma_tuning.argtypes = [ctypes.c_int] * 5
    lib.q1g128_set_mfma_tuning.restype = None
    lib.q1g128_gemv_grouped.argtypes = _GROUPED_ARGTYPES
    lib.q1g128_gemv_grouped.restype = ctypes.c_int
    lib.q1g128_set_grouped_tuning.argtypes = [ctypes.c_int] * 3
    lib.q1g128_set_grouped_tuning.restype = None
    lib.q1g128_set_stream_tuning.argtypes = [ctypes.c_int] * 2
    lib.q1g128_set_stream_tuning.restype = None
    lib.q1g128_last_kernel.argtypes = []
    lib.q1g128_last_kernel.restype = ctypes.c_char_p
    lib.q1g128_launch_count.argtypes = []
    lib.q1g128_launch_count.restype = ctypes.c_int
    lib.q1g128_fused_parts.argtypes = [ctypes.c_int] * 4
    lib.q1g128_fused_parts.restype = ctypes.c_int
    lib.q1g128_gemv_fused.argtypes = [ctypes.POINTER(FusedGemvDesc), ctypes.c_void_p]
    lib.q1g128_gemv_fused.restype = ctypes.c_int
    _q1_lib = lib


def load_actq_kernel() -> None:
    global _actq_lib
    lib = _open(os.path.join("act_quant", "libbonsai_actq.so"))
    lib.bonsai_act_quant_int8.argtypes = [
        ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
    ]
    lib.bonsai_act_quant_int8.restype = ctypes.c_int
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.bonsai_rmsnorm_quant_int8.argtypes = [vp, vp, ctypes.c_float, vp, vp, ci, ci, vp]
    lib.bonsai_rmsnorm_quant_int8.restype = ci
    lib.bonsai_add_rmsnorm_quant_int8.argtypes = [vp, vp, vp, ctypes.c_float, vp, vp, vp, ci, ci, vp]
    lib.bonsai_add_rmsnorm_quant_int8.restype = ci
    lib.bonsai_add_rmsnorm_bf16.argtypes = [vp, vp, vp, ctypes.c_float, vp, vp, ci, ci, vp]
    lib.bonsai_add_rmsnorm_bf16.restype = ci
    lib.bonsai_silu_mul_quant_int8.argtypes = [vp, vp, vp, ci, ci, vp]
    lib.bonsai_silu_mul_quant_int8.restype = ci
    _actq_lib = lib


_torch_ops_loaded = False


def torch_ops_lib_path() -> str:
    return os.path.join(_HERE, "torch_ops", "libbonsai_torch.so")


def load_torch_ops():
    """Registers the dispatcher operators ``torch.ops.bonsai.t2g128_int8xint2_linear``,
    ``q1g128_int8xint1_linear``, ``quant_input``, ``fused_norm_quant``, ``fused_add_norm_quant``
    and ``silu_mul_quant`` (CUDA and Meta kernels; csrc/torch_ops.cpp)
    and returns the ``torch.ops.bonsai`` namespace.  Same tensors in and out as the functions of
    this module (reference: model.py:118-268,632-636); a missing library raises."""
    global _torch_ops_loaded
    if not _torch_ops_loaded:
        so = torch_ops_lib_path()
        if not os.path.exists(so):
            raise RuntimeError(
                f"{so} is missing: build it with `python -m bitmtp_amd.build` "
                "(there is no fallback implementation)")
        torch.ops.load_library(so)
        _torch_ops_loaded = True
    return torch.ops.bonsai


def t2_lib() -> ctypes.CDLL:
    if _t2_lib is None:
        load_t2_kernel()
    return _t2_lib


def q1_lib() -> ctypes.CDLL:
    if _q1_lib is None:
        load_q1_kernel()
    return _q1_lib


def actq_lib() -> ctypes.CDLL:
    if _actq_lib is None:
        load_actq_kernel()
    return _actq_lib


def last_kernel(bits: int) -> str:
    """``family<template arguments>`` of the kernel this thread's last launch through the T2
    (``bits=2``) or Q1 (``bits=1``) library went to (diagnostics for tests and benchmarks)."""
    lib = t2_lib() if bits == 2 else q1_lib()
    fn = lib.t2g128_last_kernel if bits == 2 else lib.q1g128_last_kernel
    return fn().decode()


def launch_count(bits: int) -> int:
    """Kernel launches this thread has made through the T2 / Q1 library so far."""
    lib = t2_lib() if bits == 2 else q1_lib()
    return int((lib.t2g128_launch_count if bits == 2 else lib.q1g128_launch_count)())


def init_kernels() -> None:
    """One-time per-device set-up of both GEMV libraries; call before graph capture."""
    if t2_lib().t2g128_init() != 0 or q1_lib().q1g128_init() != 0:
        raise RuntimeError("bonsai GEMV kernel initialisation failed on the current device")


def _validate_packed_inputs(a, b, s, ws, *, kind, bits, activation_dtype,
                            scale_dtypes=(torch.bfloat16,)):
    """Tensor metadata checks before a native call, in the reference's order and
    with its messages (model.py:96-115)."""
    if a.dim() not in (2, 3) or b.dim() != 2:
        raise ValueError(f"{kind}: expected rank-2/3 activation and rank-2 weight")
    m = a.numel() // a.shape[-1] if a.shape[-1] else 0
    n, k = b.shape[0], b.shape[1] * (8 // bits)
    require_kernel_shape(kind, m, n, k)
    if a.shape[-1] != k:
        raise RuntimeError(f"{kind}: activation width mismatch: {a.shape[-1]} != {k}")
    if tuple(ws.shape) != (n, k // 128):
        raise RuntimeError(f"{kind}: invalid weight scale shape {tuple(ws.shape)}")
    if a.dtype != activation_dtype or b.dtype != torch.int8 or ws.dtype not in scale_dtypes:
        raise RuntimeError(f"{kind}: invalid activation, packed-weight, or scale dtype")
    tensors = (a, b, ws) if s is None else (a, b, s, ws)
    if s is not None and (s.dtype != torch.float32 or s.shape[-1:] != (1,) or s.numel() != m):
        raise RuntimeError(f"{kind}: activation scales must be float32 with one value per row")
    if not all(t.is_cuda and t.is_contiguous() for t in tensors):
        raise RuntimeError(f"{kind}: inputs and scales must be contiguous CUDA tensors")
    if not all(t.device == a.device for t in tensors):
        raise RuntimeError(f"{kind}: inputs and scales must share one CUDA device")


def _validate_group_sum_inputs(a, b, *, kind, bits, device=None):
    """Checks for a call that returns the int32 group sums (no scales are read): the operand
    checks of ``_validate_packed_inputs`` that concern the activations and the packed weights.
    Raw pointers of these tensors go to the kernel, so width, dtype, device and contiguity are
    all checked before any native call."""
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError(f"{kind}: expected rank-2 activation and rank-2 weight")
    n, k = b.shape[0], b.shape[1] * (8 // bits)
    require_kernel_shape(kind, a.shape[0], n, k)
    if a.shape[-1] != k:
        raise RuntimeError(f"{kind}: activation width mismatch: {a.shape[-1]} != {k}")
    if a.dtype != torch.int8 or b.dtype != torch.int8:
        raise RuntimeError(f"{kind}: invalid activation or packed-weight dtype")
    if not (a.is_cuda and b.is_cuda and a.is_contiguous() and b.is_contiguous()):
        raise RuntimeError(f"{kind}: inputs must be contiguous CUDA tensors")
    if b.device != a.device or (device is not None and a.device != device):
        raise RuntimeError(f"{kind}: inputs must share one CUDA device")


def _out_shape(a: torch.Tensor, n: int, kind: str) -> Tuple[int, Tuple[int, ...]]:
    if a.dim() == 2:
        return a.shape[0], (a.shape[0], n)
    if a.dim() == 3:
        bsz, slen, _ = a.shape
        return bsz * slen, (bsz, slen, n)
    raise ValueError(f"{kind} wrapper: bad input shape {a.shape}")


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(None if t is None else t.data_ptr())


def _stream(device: torch.device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def t2g128_int8xint2_linear(a_int8: torch.Tensor, b_packed: torch.Tensor, s: torch.Tensor,
                            ws: torch.Tensor) -> torch.Tensor:
    """``[..., K] int8 x [N, K/4] packed ternary -> [..., N] bf16`` on the current
    stream (reference: model.py:222-256)."""
    _validate_packed_inputs(a_int8, b_packed, s, ws, kind="t2g128", bits=2,
                            activation_dtype=torch.int8)
    n, k = b_packed.shape[0], b_packed.shape[1] * 4
    m, out_shape = _out_shape(a_int8, n, "t2g128")
    lib = t2_lib()
    out = torch.empty(*out_shape, dtype=torch.bfloat16, device=a_int8.device)
    # the checked form of the same entry point: the drop-in symbol returns nothing, and a
    # refused launch would hand back the uninitialised tensor
    with torch.cuda.device(a_int8.device):
        rc = lib.t2g128_gemv_ex(_ptr(a_int8), _ptr(b_packed), _ptr(out), _ptr(s), _ptr(ws),
                                m, n, k, OUT_BF16, SCALE_BF16, _stream(a_int8.device))
    if rc != 0:
        raise RuntimeError(f"t2g128: native launch failed with status {rc} (M={m}, N={n}, K={k})")
    return out


def q1g128_int8xint1_linear(a_int8: torch.Tensor, b_packed: torch.Tensor, s: torch.Tensor,
                            ws: torch.Tensor) -> torch.Tensor:
    """``[..., K] int8 x [N, K/8] packed signs -> [..., N] bf16`` (reference:
    model.py:118-153)."""
    _validate_packed_inputs(a_int8, b_packed, s, ws, kind="q1", bits=1,
                            activation_dtype=torch.int8)
    n, k = b_packed.shape[0], b_packed.shape[1] * 8
    m, out_shape = _out_shape(a_int8, n, "q1g128")
    lib = q1_lib()
    out = torch.empty(*out_shape, dtype=torch.bfloat16, device=a_int8.device)
    with torch.cuda.device(a_int8.device):
        rc = lib.q1g128_gemv_ex(_ptr(a_int8), _ptr(b_packed), _ptr(out), _ptr(s), _ptr(ws),
                                m, n, k, OUT_BF16, SCALE_BF16, _stream(a_int8.device))
    if rc != 0:
        raise RuntimeError(f"q1: native launch failed with status {rc} (M={m}, N={n}, K={k})")
    return out


def q1g128_w1a16_linear(a_bf16: torch.Tensor, b_packed: torch.Tensor,
                        ws: torch.Tensor) -> torch.Tensor:
    """1-bit weights x bf16 activations, fp32 accumulation (reference: model.py:159-197).
    The output is a fresh tensor from the caching allocator, which graph capture
    tracks like any other allocation."""
    if a_bf16.dim() != 2:
        raise ValueError("w1a16 requires a rank-2 activation")
    _validate_packed_inputs(a_bf16, b_packed, None, ws, kind="w1a16", bits=1,
                            activation_dtype=torch.bfloat16)
    m, n, k = a_bf16.shape[0], b_packed.shape[0], b_packed.shape[1] * 8
    lib = q1_lib()
    out = torch.empty(m, n, dtype=torch.bfloat16, device=a_bf16.device)
    with torch.cuda.device(a_bf16.device):
        lib.q1g128_w1a16_linear(_ptr(a_bf16), _ptr(b_packed), _ptr(out), _ptr(ws), m, n, k,
                                _stream(a_bf16.device))
    return out


def packed_int8_linear(a_int8, b_packed, s, ws):
    """Dispatch by packed width: Q1 has K/8 bytes per row, T2 has K/4
    (reference: model.py:259-268)."""
    K = a_int8.shape[-1]
    if b_packed.shape[-1] * 8 == K:
        return q1g128_int8xint1_linear(a_int8, b_packed, s, ws)
    if b_packed.shape[-1] * 4 == K:
        return t2g128_int8xint2_linear(a_int8, b_packed, s, ws)
    raise ValueError(
        f"unknown packed weight layout A.K={K}, B.shape={tuple(b_packed.shape)}"
    )


def packed_gemv_ex(a_int8: torch.Tensor, b_packed: torch.Tensor, s: Optional[torch.Tensor],
                   ws: Optional[torch.Tensor], *, bits: int, out_kind: int = OUT_BF16,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same kernels with a selectable result: bf16 ``[M,N]``, the fp32 value
    before the bf16 rounding, or the exact int32 group sums ``[M,N,K/128]``.
    ``ws`` may be bf16 or fp16.  Rank-2 activations only.  ``out`` supplies a preallocated
    result (so that a captured graph allocates nothing)."""
    if bits not in (1, 2):
        raise ValueError("bits must be 1 (Q1) or 2 (T2)")
    kind = "t2g128" if bits == 2 else "q1"
    if out_kind == OUT_G32:
        _validate_group_sum_inputs(a_int8, b_packed, kind=kind, bits=bits)
    else:
        if a_int8.dim() != 2:
            raise ValueError(f"{kind}: expected rank-2 activation")
        _validate_packed_inputs(a_int8, b_packed, s, ws, kind=kind, bits=bits,
                                activation_dtype=torch.int8,
                                scale_dtypes=(torch.bfloat16, torch.float16))
    m, n, k = a_int8.shape[0], b_packed.shape[0], b_packed.shape[1] * (8 // bits)
    dev = a_int8.device
    if out_kind == OUT_BF16:
        shape, dtype = (m, n), torch.bfloat16
    elif out_kind == OUT_F32:
        shape, dtype = (m, n), torch.float32
    elif out_kind == OUT_G32:
        shape, dtype = (m, n, k // 128), torch.int32
    else:
        raise ValueError("bad out_kind")
    if out is None:
        out = torch.empty(*shape, dtype=dtype, device=dev)
    elif (tuple(out.shape) != shape or out.dtype != dtype or out.device != dev
          or not out.is_contiguous()):
        raise RuntimeError(f"{kind}: out must be a contiguous {dtype} tensor of shape {shape} on {dev}")
    scale_kind = SCALE_F16 if (ws is not None and ws.dtype == torch.float16) else SCALE_BF16
    fn = t2_lib().t2g128_gemv_ex if bits == 2 else q1_lib().q1g128_gemv_ex
    with torch.cuda.device(dev):
        rc = fn(_ptr(a_int8), _ptr(b_packed), _ptr(out), _ptr(s), _ptr(ws), m, n, k, out_kind,
                scale_kind, _stream(dev))
    if rc != 0:
        raise RuntimeError(f"{kind}: native launch failed with status {rc} (M={m}, N={n}, K={k})")
    return out


FUSED_MAX_TOKENS = 2


def fused_parts(epi: int, m: int, n: int, k: int, *, bits: int) -> int:
    """Parts per token that a fused launch with epilogue ``epi`` writes for this shape (the
    number of workgroups of that launch); 0 when the shape is not taken."""
    fn = t2_lib().t2g128_fused_parts if bits == 2 else q1_lib().q1g128_fused_parts
    parts = fn(epi, m, n, k)
    if parts < -1:
        raise RuntimeError(f"fused_parts: native set-up failed with status {-parts}")
    return max(parts, 0)


def _amax_ld(parts: int) -> int:
    return (parts + 7) // 8 * 8


def packed_gemv_fused(act: torch.Tensor, b_packed: torch.Tensor, ws: torch.Tensor, *, bits: int,
                      s: Optional[torch.Tensor] = None, amax: Optional[torch.Tensor] = None,
                      sumsq: Optional[torch.Tensor] = None, parts: int = 0,
                      norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                      epi: int = EPI_PLAIN, residual: Optional[torch.Tensor] = None,
                      out: Optional[torch.Tensor] = None, out_aux: Optional[torch.Tensor] = None,
                      s_out: Optional[torch.Tensor] = None, out_kind: int = OUT_BF16):
    """One projection of a one- or two-token decode step with the element-wise work of its
    neighbours folded in (``*_gemv_fused`` of include/bonsai_gemv.h).

    What it reads: ``s`` given -- int8 ``act`` with its multipliers, as :func:`packed_gemv_ex`;
    ``amax`` given -- bf16 ``act`` quantised on the fly from the ``parts`` maxima per token a
    SiLU-pair launch left; ``sumsq`` given -- bf16 ``act`` = residual stream, RMS-normalised with
    ``norm_weight`` / ``eps`` from the ``parts`` sums of squares an add launch left, then quantised.
    What it stores (``epi``): the plain result; ``EPI_SILU_PAIR`` -- ``bf16(bf16(silu(gate)) *
    up)`` of merged rows ``[gate; up]`` plus maxima; ``EPI_ADD_SUMSQ`` -- ``bf16(residual +
    bf16(y))`` plus sums of squares.  Returns ``(out, out_aux, out_parts)``.
    Reference: the helpers between the projections, model.py:307-336 and :1058-1061."""
    kind = "t2g128" if bits == 2 else "q1"
    given = [x is not None for x in (s, amax, sumsq)]
    if sum(given) != 1:
        raise ValueError(f"{kind}: exactly one of s, amax, sumsq selects what the launch reads")
    act_kind = ACT_INT8 if s is not None else (ACT_BF16_AMAX if amax is not None else ACT_BF16_NORM)
    if epi not in (EPI_PLAIN, EPI_SILU_PAIR, EPI_ADD_SUMSQ):
        raise ValueError("bad epi")
    if act.dim() != 2 or b_packed.dim() != 2:
        raise ValueError(f"{kind}: expected rank-2 activation and rank-2 weight")
    m, n, k = act.shape[0], b_packed.shape[0], b_packed.shape[1] * (8 // bits)
    dev = act.device
    want_act = torch.int8 if act_kind == ACT_INT8 else torch.bfloat16
    if act.dtype != want_act or act.shape[1] != k or b_packed.dtype != torch.int8:
        raise RuntimeError(f"{kind}: activations must be {want_act} [M, {k}] and the weights packed int8")
    if m < 1 or m > FUSED_MAX_TOKENS:
        raise RuntimeError(f"{kind}: the fused forms take one or two tokens")
    if ws.dtype != torch.bfloat16 or tuple(ws.shape) != (n, k // 128):
        raise RuntimeError(f"{kind}: weight scales must be bf16 [{n}, {k // 128}]")
    aux = s if s is not None else (amax if amax is not None else sumsq)
    if act_kind == ACT_INT8:
        if s.dtype != torch.float32 or s.numel() != m:
            raise RuntimeError(f"{kind}: activation scales must be float32 with one value per row")
    elif act_kind == ACT_BF16_AMAX:
        if amax.dtype != torch.bfloat16 or parts < 1 or amax.numel() < m * _amax_ld(parts):
            raise RuntimeError(f"{kind}: amax must be bf16 with at least {m * _amax_ld(parts)} elements")
    else:
        if sumsq.dtype != torch.float64 or parts < 1 or sumsq.numel() < m * parts:
            raise RuntimeError(f"{kind}: sumsq must be float64 with at least {m * parts} elements")
        if norm_weight is None or norm_weight.dtype != torch.bfloat16 or norm_weight.numel() != k:
            raise RuntimeError(f"{kind}: norm_weight must be bf16 [{k}]")
    out_parts = 0
    with torch.cuda.device(dev):
        if epi != EPI_PLAIN:
            if out_kind != OUT_BF16:
                raise ValueError(f"{kind}: this epilogue stores bf16")
            if epi == EPI_SILU_PAIR and n % 2:
                raise RuntimeError(f"{kind}: merged gate|up rows must be even in number")
            out_parts = fused_parts(epi, m, n, k, bits=bits)
            if out_parts == 0:
                raise RuntimeError(f"{kind}: shape not taken by the fused forms (M={m}, N={n}, K={k})")
        n_out = n // 2 if epi == EPI_SILU_PAIR else n
        dtype = torch.float32 if (epi == EPI_PLAIN and out_kind == OUT_F32) else torch.bfloat16
        if epi == EPI_PLAIN and out_kind not in (OUT_BF16, OUT_F32):
            raise ValueError("bad out_kind")
        if out is None:
            out = torch.empty(m, n_out, dtype=dtype, device=dev)
        elif tuple(out.shape) != (m, n_out) or out.dtype != dtype or not out.is_contiguous():
            raise RuntimeError(f"{kind}: out must be a contiguous {dtype} tensor of shape {(m, n_out)}")
        if epi == EPI_SILU_PAIR:
            need, adt = m * _amax_ld(out_parts), torch.bfloat16
        elif epi == EPI_ADD_SUMSQ:
            need, adt = m * out_parts, torch.float64
            if residual is None or residual.dtype != torch.bfloat16 or tuple(residual.shape) != (m, n):
                raise RuntimeError(f"{kind}: residual must be bf16 [{m}, {n}]")
        else:
            need, adt = 0, None
        if need:
            if out_aux is None:
                out_aux = torch.empty(need, dtype=adt, device=dev)
            elif out_aux.dtype != adt or out_aux.numel() < need or not out_aux.is_contiguous():
                raise RuntimeError(f"{kind}: out_aux must be contiguous {adt} with at least {need} elements")
        if s_out is not None and (act_kind == ACT_INT8 or s_out.dtype != torch.float32 or s_out.numel() < m):
            raise RuntimeError(f"{kind}: s_out is fp32 [M] and only for bf16 activations")
        tensors = [t for t in (act, b_packed, ws, aux, norm_weight, residual, out, out_aux, s_out) if t is not None]
        if not all(t.is_cuda and t.is_contiguous() and t.device == dev for t in tensors):
            raise RuntimeError(f"{kind}: operands must be contiguous tensors on {dev}")
        d = FusedGemvDesc(act=act.data_ptr(), act_aux=aux.data_ptr(),
                          norm_weight=norm_weight.data_ptr() if norm_weight is not None else None,
                          B=b_packed.data_ptr(), ws=ws.data_ptr(), out=out.data_ptr(),
                          residual=residual.data_ptr() if residual is not None else None,
                          out_aux=out_aux.data_ptr() if out_aux is not None else None,
                          s_out=s_out.data_ptr() if s_out is not None else None,
                          eps=float(eps), M=m, N=n, K=k, act_kind=act_kind, act_parts=int(parts),
                          epi_kind=epi, out_kind=out_kind)
        fn = t2_lib().t2g128_gemv_fused if bits == 2 else q1_lib().q1g128_gemv_fused
        rc = fn(ctypes.byref(d), _stream(dev))
    if rc != 0:
        raise RuntimeError(f"{kind}: native launch failed with status {rc} (M={m}, N={n}, K={k})")
    return out, out_aux, out_parts


def packed_gemv_grouped(problems: Sequence[Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor],
                                                 Optional[torch.Tensor]]],
                        *, bits: int, out_kind: int = OUT_BF16,
                        outs: Optional[Sequence[torch.Tensor]] = None) -> List[torch.Tensor]:
    """Several independent GEMVs ``(a_int8 [M,K], b_packed, s, ws)`` in one native call
    (``*_gemv_grouped``): one launch walks the row tiles of all of them.  Widths, row counts
    and K may differ between the problems; every result is what ``packed_gemv_ex`` gives for
    that problem alone: the same int32 group sums, and the same fp32 / bf16 bits wherever both
    calls reach the same kernel with the same geometry (otherwise equal within the tolerance
    of the fp32 summation order).  ``outs`` supplies preallocated outputs (so that a captured graph
    allocates nothing); otherwise fresh tensors are returned."""
    if bits not in (1, 2):
        raise ValueError("bits must be 1 (Q1) or 2 (T2)")
    if not 1 <= len(problems) <= GROUPED_MAX:
        raise ValueError(f"a grouped call takes 1..{GROUPED_MAX} problems")
    if out_kind not in (OUT_BF16, OUT_F32, OUT_G32):
        raise ValueError("bad out_kind")
    if outs is not None and len(outs) != len(problems):
        raise ValueError("one output per problem")
    kind = "t2g128" if bits == 2 else "q1"
    descs = (GemvDesc * len(problems))()
    results: List[torch.Tensor] = []
    dev = problems[0][0].device
    scale_kinds = set()
    for i, (a, b, s, ws) in enumerate(problems):
        if a.dim() != 2:
            raise ValueError(f"{kind}: expected rank-2 activation")
        if out_kind == OUT_G32:
            _validate_group_sum_inputs(a, b, kind=kind, bits=bits, device=dev)
        else:
            _validate_packed_inputs(a, b, s, ws, kind=kind, bits=bits, activation_dtype=torch.int8,
                                    scale_dtypes=(torch.bfloat16, torch.float16))
            scale_kinds.add(SCALE_F16 if ws.dtype == torch.float16 else SCALE_BF16)
        if a.device != dev:
            raise RuntimeError(f"{kind}: all problems of a grouped call must share one CUDA device")
        m, n, k = a.shape[0], b.shape[0], b.shape[1] * (8 // bits)
        shape = (m, n, k // 128) if out_kind == OUT_G32 else (m, n)
        dtype = {OUT_BF16: torch.bfloat16, OUT_F32: torch.float32, OUT_G32: torch.int32}[out_kind]
        if outs is None:
            out = torch.empty(*shape, dtype=dtype, device=dev)
        else:
            out = outs[i]
            if tuple(out.shape) != shape or out.dtype != dtype or out.device != dev or \
                    not out.is_contiguous():
                raise RuntimeError(f"{kind}: output {i} must be a contiguous {dtype} tensor {shape}")
        results.append(out)
        descs[i] = GemvDesc(a.data_ptr(), b.data_ptr(), out.data_ptr(),
                            None if s is None else s.data_ptr(),
                            None if ws is None else ws.data_ptr(), m, n, k, 0)
    if len(scale_kinds) > 1:
        raise RuntimeError(f"{kind}: the scales of a grouped call must share one dtype")
    scale_kind = scale_kinds.pop() if scale_kinds else SCALE_BF16
    fn = t2_lib().t2g128_gemv_grouped if bits == 2 else q1_lib().q1g128_gemv_grouped
    with torch.cuda.device(dev):
        rc = fn(descs, len(problems), out_kind, scale_kind, _stream(dev))
    if rc != 0:
        raise RuntimeError(f"{kind}: grouped native launch failed with status {rc}")
    return results


def quant_input(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token absmax INT8 quantisation on the GPU: returns ``(q int8 [..., K],
    s fp32 [..., 1])`` with ``s = reciprocal(clamp_min(absmax, 1e-5)) * 127`` -- what
    PyTorch computes for the reference's ``127.0 / absmax.clamp_(min=1e-5)``
    (model.py:632-636)."""
    if x.dtype not in _X_KIND:
        raise RuntimeError("quant_input: activation must be bfloat16, float16 or float32")
    if not (x.is_cuda and x.is_contiguous()) or x.dim() < 1:
        raise RuntimeError("quant_input: activation must be a contiguous CUDA tensor")
    k = x.shape[-1]
    if k == 0 or k % 8 != 0:
        raise RuntimeError("quant_input: last dimension must be a positive multiple of 8")
    m = x.numel() // k
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(*x.shape[:-1], 1, dtype=torch.float32, device=x.device)
    if m == 0:
        return q, s
    with torch.cuda.device(x.device):
        rc = actq_lib().bonsai_act_quant_int8(_ptr(x), _X_KIND[x.dtype], _ptr(q), _ptr(s), m, k,
                                              _stream(x.device))
    if rc != 0:
        raise RuntimeError(f"quant_input: native launch failed with status {rc}")
    return q, s


def _check_bf16_rows(name: str, *tensors: torch.Tensor) -> None:
    for t in tensors:
        if t.dtype != torch.bfloat16 or not (t.is_cuda and t.is_contiguous()):
            raise RuntimeError(f"{name}: operands must be contiguous CUDA bfloat16 tensors")


def fused_norm_quant(x: torch.Tensor, w: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """RMSNorm then per-token INT8 quantisation: ``(q int8 [..., K], s fp32 [..., 1])``
    (reference: ``_fused_norm_quant``, model.py:307-319)."""
    _check_bf16_rows("fused_norm_quant", x, w)
    k = x.shape[-1]
    if w.shape != (k,) or k % 8 != 0:
        raise RuntimeError("fused_norm_quant: weight must be [K] and K a multiple of 8")
    m = x.numel() // k
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(*x.shape[:-1], 1, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = actq_lib().bonsai_rmsnorm_quant_int8(_ptr(x), _ptr(w), float(eps), _ptr(q), _ptr(s), m, k,
                                                  _stream(x.device))
    if rc != 0:
        raise RuntimeError(f"fused_norm_quant: native launch failed with status {rc}")
    return q, s


def fused_add_norm_quant(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor,
                         eps: float) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``h = x + residual``; returns ``(h, q, s)`` with ``(q, s)`` the quantised RMSNorm of h
    (reference: ``_fused_add_norm_quant``, model.py:322-336)."""
    _check_bf16_rows("fused_add_norm_quant", x, residual, w)
    k = x.shape[-1]
    if residual.shape != x.shape or w.shape != (k,) or k % 8 != 0:
        raise RuntimeError("fused_add_norm_quant: shape mismatch or K not a multiple of 8")
    m = x.numel() // k
    h = torch.empty_like(x)
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(*x.shape[:-1], 1, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = actq_lib().bonsai_add_rmsnorm_quant_int8(_ptr(x), _ptr(residual), _ptr(w), float(eps),
                                                      _ptr(h), _ptr(q), _ptr(s), m, k,
                                                      _stream(x.device))
    if rc != 0:
        raise RuntimeError(f"fused_add_norm_quant: native launch failed with status {rc}")
    return h, q, s


def add_rmsnorm(x: torch.Tensor, residual: Optional[torch.Tensor], w: torch.Tensor,
                eps: float) -> torch.Tensor:
    """``RMSNorm(x + residual) * w`` in bf16 without quantisation (``residual`` may be None):
    the final norm in front of a bf16 output projection (reference: model.py:1401-1402,
    ``RMSNorm.forward`` model.py:290-295)."""
    ts = (x, w) if residual is None else (x, residual, w)
    _check_bf16_rows("add_rmsnorm", *ts)
    k = x.shape[-1]
    if (residual is not None and residual.shape != x.shape) or w.shape != (k,) or k % 8 != 0:
        raise RuntimeError("add_rmsnorm: shape mismatch or K not a multiple of 8")
    m = x.numel() // k
    n = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = actq_lib().bonsai_add_rmsnorm_bf16(_ptr(x), _ptr(residual) if residual is not None
                                                else ctypes.c_void_p(0), _ptr(w), float(eps),
                                                ctypes.c_void_p(0), _ptr(n), m, k, _stream(x.device))
    if rc != 0:
        raise RuntimeError(f"add_rmsnorm: native launch failed with status {rc}")
    return n


def silu_mul_quant(gate_up: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``inner = silu(gate) * up`` of a merged gate/up projection ``[..., 2F]`` followed by
    per-token quantisation: ``(q int8 [..., F], s fp32 [..., 1])`` (reference:
    model.py:1058-1061)."""
    _check_bf16_rows("silu_mul_quant", gate_up)
    f2 = gate_up.shape[-1]
    if f2 % 16 != 0:
        raise RuntimeError("silu_mul_quant: last dimension must be 2F with F a multiple of 8")
    f = f2 // 2
    m = gate_up.numel() // f2
    q = torch.empty(*gate_up.shape[:-1], f, dtype=torch.int8, device=gate_up.device)
    s = torch.empty(*gate_up.shape[:-1], 1, dtype=torch.float32, device=gate_up.device)
    with torch.cuda.device(gate_up.device):
        rc = actq_lib().bonsai_silu_mul_quant_int8(_ptr(gate_up), _ptr(q), _ptr(s), m, f,
                                                   _stream(gate_up.device))
    if rc != 0:
        raise RuntimeError(f"silu_mul_quant: native launch failed with status {rc}")
    return q, s
