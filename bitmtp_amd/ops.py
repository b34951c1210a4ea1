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
# (A, B, inner, s, ws, M, N2, K, amax, stream) and
# (inner, B, out, ws, M, N, K, amax, parts, s_out, out_kind, stream)
_SILU_PAIR_ARGTYPES = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 3 + [ctypes.c_void_p] * 2
_BF16_ACT_ARGTYPES = ([ctypes.c_void_p] * 4 + [ctypes.c_int] * 3 +
                      [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p])


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
    lib.t2g128_silu_pair_parts.argtypes = [ctypes.c_int] * 3
    lib.t2g128_silu_pair_parts.restype = ctypes.c_int
    lib.t2g128_gemv_silu_pair.argtypes = _SILU_PAIR_ARGTYPES
    lib.t2g128_gemv_silu_pair.restype = ctypes.c_int
    lib.t2g128_gemv_bf16_act.argtypes = _BF16_ACT_ARGTYPES
    lib.t2g128_gemv_bf16_act.restype = ctypes.c_int
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
    lib.q1g128_silu_pair_parts.argtypes = [ctypes.c_int] * 3
    lib.q1g128_silu_pair_parts.restype = ctypes.c_int
    lib.q1g128_gemv_silu_pair.argtypes = _SILU_PAIR_ARGTYPES
    lib.q1g128_gemv_silu_pair.restype = ctypes.c_int
    lib.q1g128_gemv_bf16_act.argtypes = _BF16_ACT_ARGTYPES
    lib.q1g128_gemv_bf16_act.restype = ctypes.c_int
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


FUSED_MLP_MAX_TOKENS = 2


def silu_pair_parts(m: int, n2: int, k: int, *, bits: int) -> int:
    """Maxima per token that :func:`packed_gemv_silu_pair` writes for this shape (the number
    of workgroups of its launch); 0 when the shape is not taken."""
    fn = t2_lib().t2g128_silu_pair_parts if bits == 2 else q1_lib().q1g128_silu_pair_parts
    parts = fn(m, n2, k)
    if parts < -1:
        raise RuntimeError(f"silu_pair_parts: native set-up failed with status {-parts}")
    return max(parts, 0)


def packed_gemv_silu_pair(a_int8: torch.Tensor, b_gate_up: torch.Tensor, s: torch.Tensor,
                          ws: torch.Tensor, *, bits: int, inner: Optional[torch.Tensor] = None,
                          amax: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, int]:
    """The merged gate|up projection (rows ``[gate; up]``) of one or two quantised tokens with
    ``inner = bf16(bf16(silu(gate)) * up)`` computed in its epilogue: returns ``(inner bf16
    [M, F], amax bf16 [M, ld], parts)`` where ``amax[m, :parts]`` holds max ``|inner[m]|`` of
    each workgroup of the launch.  Together with :func:`packed_gemv_bf16_act` it stands for
    projection, SiLU * up + quantisation (reference: model.py:1059-1061) and projection, with
    the same bits."""
    kind = "t2g128" if bits == 2 else "q1"
    if a_int8.dim() != 2:
        raise ValueError(f"{kind}: expected rank-2 activation")
    _validate_packed_inputs(a_int8, b_gate_up, s, ws, kind=kind, bits=bits,
                            activation_dtype=torch.int8, scale_dtypes=(torch.bfloat16,))
    m, n2, k = a_int8.shape[0], b_gate_up.shape[0], b_gate_up.shape[1] * (8 // bits)
    if m > FUSED_MLP_MAX_TOKENS or n2 % 2:
        raise RuntimeError(f"{kind}: the fused MLP tail takes one or two tokens and an even row count")
    dev = a_int8.device
    with torch.cuda.device(dev):
        parts = silu_pair_parts(m, n2, k, bits=bits)
        if parts == 0:
            raise RuntimeError(f"{kind}: shape not taken by the fused MLP tail (M={m}, N={n2}, K={k})")
        ld = (parts + 7) // 8 * 8
        if inner is None:
            inner = torch.empty(m, n2 // 2, dtype=torch.bfloat16, device=dev)
        if amax is None:
            amax = torch.empty(m, ld, dtype=torch.bfloat16, device=dev)
        if (tuple(inner.shape) != (m, n2 // 2) or inner.dtype != torch.bfloat16 or not inner.is_contiguous()
                or amax.dtype != torch.bfloat16 or amax.numel() < m * ld or not amax.is_contiguous()
                or inner.device != dev or amax.device != dev):
            raise RuntimeError(f"{kind}: inner must be bf16 [{m}, {n2 // 2}] and amax bf16 with at least "
                               f"{m * ld} elements, contiguous, on {dev}")
        fn = t2_lib().t2g128_gemv_silu_pair if bits == 2 else q1_lib().q1g128_gemv_silu_pair
        rc = fn(_ptr(a_int8), _ptr(b_gate_up), _ptr(inner), _ptr(s), _ptr(ws), m, n2, k, _ptr(amax),
                _stream(dev))
    if rc != 0:
        raise RuntimeError(f"{kind}: native launch failed with status {rc} (M={m}, N={n2}, K={k})")
    return inner, amax, parts


def packed_gemv_bf16_act(inner: torch.Tensor, b_packed: torch.Tensor, ws: torch.Tensor,
                         amax: torch.Tensor, parts: int, *, bits: int, out_kind: int = OUT_BF16,
                         out: Optional[torch.Tensor] = None,
                         s_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Projection of bf16 activations ``inner [M, K]`` (one or two tokens) that are quantised
    per token while they are staged, with ``s = fl(fl(1 / max(amax, 1e-5)) * 127)`` taken from
    the ``parts`` maxima per token that :func:`packed_gemv_silu_pair` left in ``amax``; ``s_out``
    (fp32 [M]) receives the multipliers when given."""
    kind = "t2g128" if bits == 2 else "q1"
    if inner.dim() != 2 or inner.dtype != torch.bfloat16 or not inner.is_contiguous() or not inner.is_cuda:
        raise RuntimeError(f"{kind}: expected contiguous rank-2 bf16 CUDA activations")
    m, n, k = inner.shape[0], b_packed.shape[0], b_packed.shape[1] * (8 // bits)
    if inner.shape[1] != k or m > FUSED_MLP_MAX_TOKENS:
        raise RuntimeError(f"{kind}: inner must be [M <= {FUSED_MLP_MAX_TOKENS}, {k}]")
    if ws.dtype != torch.bfloat16 or tuple(ws.shape) != (n, k // 128):
        raise RuntimeError(f"{kind}: weight scales must be bf16 [{n}, {k // 128}]")
    if out_kind not in (OUT_BF16, OUT_F32):
        raise ValueError("bad out_kind")
    ld = (parts + 7) // 8 * 8
    if amax.dtype != torch.bfloat16 or amax.numel() < m * ld or parts < 1 or not amax.is_contiguous():
        raise RuntimeError(f"{kind}: amax must be contiguous bf16 with at least {m * ld} elements")
    dev = inner.device
    dtype = torch.bfloat16 if out_kind == OUT_BF16 else torch.float32
    if out is None:
        out = torch.empty(m, n, dtype=dtype, device=dev)
    elif tuple(out.shape) != (m, n) or out.dtype != dtype or out.device != dev or not out.is_contiguous():
        raise RuntimeError(f"{kind}: out must be a contiguous {dtype} tensor of shape {(m, n)} on {dev}")
    if s_out is not None and (s_out.dtype != torch.float32 or s_out.numel() < m or s_out.device != dev):
        raise RuntimeError(f"{kind}: s_out must be fp32 with at least {m} elements on {dev}")
    for t in (b_packed, ws, amax):
        if t.device != dev:
            raise RuntimeError(f"{kind}: all operands must be on {dev}")
    fn = t2_lib().t2g128_gemv_bf16_act if bits == 2 else q1_lib().q1g128_gemv_bf16_act
    with torch.cuda.device(dev):
        rc = fn(_ptr(inner), _ptr(b_packed), _ptr(out), _ptr(ws), m, n, k, _ptr(amax), parts,
                _ptr(s_out), out_kind, _stream(dev))
    if rc != 0:
        raise RuntimeError(f"{kind}: native launch failed with status {rc} (M={m}, N={n}, K={k})")
    return out


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
