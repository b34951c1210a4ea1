"""CPU oracle for the packed low-bit GEMV path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  The product (``bitmtp_amd``) never does.

Two independent statements of the same arithmetic live here:

* ``c_*`` functions call ``oracle/_build/libbonsai_oracle.so`` (plain C,
  ``bonsai_oracle.c``) -- fast enough for the full benchmark shapes;
* ``np_*`` functions are a vectorised NumPy restatement written separately, used
  to cross-check the C code at small sizes.

Both follow the reference files cited in ``bonsai_oracle.c``:
``src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:21-27,54-91``,
``src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels.h:21-24,388-422``,
``src/bonsai_sft/gpu/model.py:632-636`` and
``src/bonsai_sft/gpu/convert_bonsai_mtp_to_gpu.py:87-144``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

GROUP = 128
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libbonsai_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with the committed Makefile; returns the .so path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        L.oracle_unpack_t2.argtypes = [vp, vp, ci, ci]
        L.oracle_unpack_q1.argtypes = [vp, vp, ci, ci]
        L.oracle_pack_t2_codes.argtypes = [vp, vp, ci, ci]
        L.oracle_pack_q1_signs.argtypes = [vp, vp, ci, ci]
        L.oracle_pack_t2_g128.argtypes = [vp, vp, vp, ci, ci]
        L.oracle_pack_q1_g128.argtypes = [vp, vp, vp, ci, ci]
        L.oracle_act_quant.argtypes = [vp, vp, vp, ci, ci]
        L.oracle_group_sums.argtypes = [vp, vp, vp, ci, ci, ci, ci]
        L.oracle_gemv.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
        L.oracle_rmsnorm_quant.argtypes = [vp, vp, vp, ctypes.c_float, vp, vp, vp, ci, ci]
        L.oracle_rmsnorm_quant.restype = None
        L.oracle_rmsnorm_bf16.argtypes = [vp, vp, vp, ctypes.c_float, vp, vp, ci, ci]
        L.oracle_rmsnorm_bf16.restype = None
        L.oracle_silu_mul_quant.argtypes = [vp, vp, vp, ci, ci]
        L.oracle_silu_mul_quant.restype = None
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_f32.restype = ctypes.c_float
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = ctypes.c_float
        for name in ("oracle_unpack_t2", "oracle_unpack_q1", "oracle_pack_t2_codes",
                     "oracle_pack_q1_signs", "oracle_pack_t2_g128", "oracle_pack_q1_g128",
                     "oracle_act_quant", "oracle_group_sums", "oracle_gemv"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------
# bf16 helpers (NumPy has no bf16: carried as uint16 bit patterns)
# --------------------------------------------------------------------------
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 bit patterns (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


# --------------------------------------------------------------------------
# C oracle wrappers
# --------------------------------------------------------------------------
def c_unpack(B: np.ndarray, bits: int) -> np.ndarray:
    B = _c(B.view(np.uint8), np.uint8)
    N, K = B.shape[0], B.shape[1] * (8 // bits)
    W = np.empty((N, K), dtype=np.int8)
    (lib().oracle_unpack_t2 if bits == 2 else lib().oracle_unpack_q1)(_p(B), _p(W), N, K)
    return W


def c_pack_values(Q: np.ndarray, bits: int) -> np.ndarray:
    """Q int8 [N,K]: ternary values for bits=2, signs (>=0 -> +1) for bits=1."""
    Q = _c(Q, np.int8)
    N, K = Q.shape
    B = np.empty((N, K * bits // 8), dtype=np.uint8)
    (lib().oracle_pack_t2_codes if bits == 2 else lib().oracle_pack_q1_signs)(_p(Q), _p(B), N, K)
    return B


def c_pack_latent(W_bf16_bits: np.ndarray, bits: int):
    W = _c(W_bf16_bits, np.uint16)
    N, K = W.shape
    B = np.empty((N, K * bits // 8), dtype=np.uint8)
    S = np.empty((N, K // GROUP), dtype=np.uint16)
    (lib().oracle_pack_t2_g128 if bits == 2 else lib().oracle_pack_q1_g128)(_p(W), _p(B), _p(S), N, K)
    return B, S


def c_act_quant(X: np.ndarray):
    """X: any float array [M,K] (fp16 values widened exactly).  Returns (q int8, s fp32[M])."""
    X = _c(X, np.float32)
    M, K = X.shape
    Q = np.empty((M, K), dtype=np.int8)
    S = np.empty((M,), dtype=np.float32)
    lib().oracle_act_quant(_p(X), _p(Q), _p(S), M, K)
    return Q, S


def c_rmsnorm_quant(x_bits, w_bits, eps: float, residual_bits=None):
    """bf16 bit patterns in; returns (q int8 [M,K], s fp32 [M], h bf16 bits or None)."""
    X = _c(x_bits, np.uint16)
    W = _c(w_bits, np.uint16)
    M, K = X.shape
    Q = np.empty((M, K), dtype=np.int8)
    S = np.empty((M,), dtype=np.float32)
    if residual_bits is None:
        lib().oracle_rmsnorm_quant(_p(X), None, _p(W), eps, None, _p(Q), _p(S), M, K)
        return Q, S, None
    R = _c(residual_bits, np.uint16)
    H = np.empty((M, K), dtype=np.uint16)
    lib().oracle_rmsnorm_quant(_p(X), _p(R), _p(W), eps, _p(H), _p(Q), _p(S), M, K)
    return Q, S, H


def c_rmsnorm(x_bits, w_bits, eps: float, residual_bits=None):
    """RMSNorm without quantisation: returns (normed bf16 bits [M,K], h bf16 bits or None)."""
    X = _c(x_bits, np.uint16)
    W = _c(w_bits, np.uint16)
    M, K = X.shape
    N = np.empty((M, K), dtype=np.uint16)
    if residual_bits is None:
        lib().oracle_rmsnorm_bf16(_p(X), None, _p(W), eps, None, _p(N), M, K)
        return N, None
    R = _c(residual_bits, np.uint16)
    H = np.empty((M, K), dtype=np.uint16)
    lib().oracle_rmsnorm_bf16(_p(X), _p(R), _p(W), eps, _p(H), _p(N), M, K)
    return N, H


def c_silu_mul_quant(gu_bits):
    GU = _c(gu_bits, np.uint16)
    M, F2 = GU.shape
    F = F2 // 2
    Q = np.empty((M, F), dtype=np.int8)
    S = np.empty((M,), dtype=np.float32)
    lib().oracle_silu_mul_quant(_p(GU), _p(Q), _p(S), M, F)
    return Q, S


def c_group_sums(A: np.ndarray, B: np.ndarray, bits: int) -> np.ndarray:
    A = _c(A, np.int8)
    B = _c(B.view(np.uint8), np.uint8)
    M, K = A.shape
    N = B.shape[0]
    assert B.shape[1] * (8 // bits) == K
    G = np.empty((M, N, K // GROUP), dtype=np.int32)
    lib().oracle_group_sums(_p(A), _p(B), _p(G), M, N, K, bits)
    return G


def c_gemv(A, B, s, ws_bits, bits: int, scale_is_f16: bool = False):
    """Returns (y32 fp32 [M,N], y bf16 bits uint16 [M,N])."""
    A = _c(A, np.int8)
    B = _c(B.view(np.uint8), np.uint8)
    s = _c(np.asarray(s).reshape(-1), np.float32)
    ws_bits = _c(ws_bits, np.uint16)
    M, K = A.shape
    N = B.shape[0]
    assert B.shape[1] * (8 // bits) == K and ws_bits.shape == (N, K // GROUP) and s.shape == (M,)
    Y32 = np.empty((M, N), dtype=np.float32)
    Y16 = np.empty((M, N), dtype=np.uint16)
    lib().oracle_gemv(_p(A), _p(B), _p(s), _p(ws_bits), _p(Y32), _p(Y16), M, N, K, bits,
                      1 if scale_is_f16 else 0)
    return Y32, Y16


# --------------------------------------------------------------------------
# NumPy restatement (independent of the C code)
# --------------------------------------------------------------------------
def np_unpack(B: np.ndarray, bits: int) -> np.ndarray:
    B = np.asarray(B).view(np.uint8)
    per = 8 // bits
    shifts = (np.arange(per, dtype=np.uint8) * bits)
    codes = (B[:, :, None] >> shifts[None, None, :]) & ((1 << bits) - 1)
    codes = codes.reshape(B.shape[0], -1).astype(np.int16)
    return (codes - 2 if bits == 2 else 2 * codes - 1).astype(np.int8)


def np_act_quant(X: np.ndarray):
    Xf = np.asarray(X, dtype=np.float32)
    amax = np.maximum(np.abs(Xf).max(axis=-1, keepdims=True), np.float32(1e-5))
    recip = (np.float32(1.0) / amax).astype(np.float32)  # torch: scalar / tensor = reciprocal * scalar
    s = (recip * np.float32(127.0)).astype(np.float32)
    q = np.clip(np.rint((Xf * s).astype(np.float32)), -128, 127).astype(np.int8)
    return q, s.reshape(-1)


def np_group_sums(A: np.ndarray, B: np.ndarray, bits: int) -> np.ndarray:
    W = np_unpack(B, bits).astype(np.int64)
    A = np.asarray(A, dtype=np.int64)
    M, K = A.shape
    N = W.shape[0]
    Ag = A.reshape(M, K // GROUP, GROUP)
    Wg = W.reshape(N, K // GROUP, GROUP)
    return np.einsum("mgk,ngk->mng", Ag, Wg).astype(np.int32)


def np_gemv_f32(A, B, s, ws_bits, bits: int) -> np.ndarray:
    """fp32 result with the canonical ascending-group summation order."""
    G = np_group_sums(A, B, bits).astype(np.float32)
    ws = bf16_bits_to_f32(ws_bits)
    acc = np.zeros(G.shape[:2], dtype=np.float32)
    for g in range(G.shape[2]):
        acc = (acc + (G[:, :, g] * ws[None, :, g]).astype(np.float32)).astype(np.float32)
    return (acc / np.asarray(s, dtype=np.float32).reshape(-1, 1)).astype(np.float32)


# --------------------------------------------------------------------------
# Seeded synthetic inputs with the benchmark distributions
# --------------------------------------------------------------------------
def synth_problem(seed: int, M: int, N: int, K: int, bits: int):
    """Weights i.i.d. ternary (p=1/3) or sign (p=1/2); scales exp(N(-4, 0.5^2))
    rounded to bf16; activations fp16 N(0,1) quantised per token.

    Returns dict with A int8[M,K], s fp32[M], B uint8[N,K*bits/8], ws uint16[N,K/128]
    (bf16 bits), x fp16[M,K].
    """
    rng = np.random.default_rng(seed)
    if bits == 2:
        q = rng.integers(-1, 2, size=(N, K), dtype=np.int8)
    else:
        q = (2 * rng.integers(0, 2, size=(N, K), dtype=np.int8) - 1).astype(np.int8)
    B = c_pack_values(q, bits)
    ws = f32_to_bf16_bits(np.exp(rng.normal(-4.0, 0.5, size=(N, K // GROUP))).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float16)
    A, s = c_act_quant(x.astype(np.float32))
    return {"A": A, "s": s, "B": B, "ws": ws, "x": x, "q": q}
