"""CPU check of the kernels' per-lane arithmetic (bitmtp_amd/csrc/gemv_core.h): the
staging permutation, the shift/mask unpack, the dot4 chains and the activation-sum
correction are replayed lane by lane on the host and must reproduce the oracle's
int32 group sums bit for bit."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "host_sim", "sim_gemv.cpp")
OUT = os.path.join(HERE, "host_sim", "_build", "libsim_gemv.so")


@pytest.fixture(scope="module")
def sim():
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    deps = [SRC, os.path.join(HERE, "..", "bitmtp_amd", "csrc", "gemv_core.h")]
    if not os.path.exists(OUT) or any(os.path.getmtime(d) > os.path.getmtime(OUT) for d in deps):
        subprocess.run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", SRC, "-o", OUT], check=True)
    L = ctypes.CDLL(OUT)
    L.sim_group_sums.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 5
    L.sim_group_sums.restype = ctypes.c_int
    L.sim_group_sums_mfma.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4
    L.sim_group_sums_mfma.restype = ctypes.c_int
    return L


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M,N,K,mt", [(1, 8, 128, 1), (1, 6, 2048, 1), (3, 5, 384, 2),
                                       (5, 16, 2560, 3), (4, 3, 9728, 2), (7, 2, 640, 3)])
def test_lane_arithmetic_matches_oracle(oracle, sim, bits, M, N, K, mt):
    rng = np.random.default_rng(M * 131 + N * 17 + K + bits)
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)       # all of int8, -128 included
    B = rng.integers(0, 256, size=(N, K * bits // 8), dtype=np.uint8)  # every code, T2 code 0 too
    G = np.zeros((M, N, K // 128), dtype=np.int32)
    rc = sim.sim_group_sums(A.ctypes.data, B.ctypes.data, G.ctypes.data, M, N, K, bits, mt)
    assert rc == 0
    assert np.array_equal(G, oracle.c_group_sums(A, B, bits))


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M,N,K", [(1, 4, 128), (3, 5, 512), (16, 3, 2560), (9, 2, 1024)])
def test_mfma_slot_mapping_matches_oracle(oracle, sim, bits, M, N, K):
    """Matrix-core path: staged operand order, per-MFMA dword choice and correction
    terms reproduce the exact group sums (the MFMA itself is modelled slot by slot)."""
    rng = np.random.default_rng(M * 7 + N * 3 + K + bits)
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(0, 256, size=(N, K * bits // 8), dtype=np.uint8)
    G = np.zeros((M, N, K // 128), dtype=np.int32)
    assert sim.sim_group_sums_mfma(A.ctypes.data, B.ctypes.data, G.ctypes.data, M, N, K, bits) == 0
    assert np.array_equal(G, oracle.c_group_sums(A, B, bits))
