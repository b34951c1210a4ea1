"""Integer arithmetic of the kernels the default dispatch picks for layer- and head-sized work
-- ``gemv_mxl_kernel`` (three tokens and more, single and grouped, in every build the host can
choose), ``gemv_dot4_grouped_kernel`` (one- and two-token grouped launches),
``gemv_mxs_kernel`` and ``gemv_rowreg_kernel`` (very long matrices) -- pinned on their own,
through the C ABI, at the K of the real layers (2048, 2560, 6144, 9728):

* the int32 group sums ``G`` come from the very kernel that produces the bf16 result
  (asserted through the library's last-kernel record) and are bit-exact against the oracle on
  every byte value (T2 code 0 = -2 included, rows of 0x00 and 0xFF) and activations over all of
  int8 with an all -128 and an all 127 row;
* with every scale 1 the fp32 output equals the integer product ``unpack(B) @ A`` exactly (all
  partial sums stay below 2**24), so a wrong group sum cannot hide behind a tolerance;
* with one-hot scales (``ws[:, g] = 1``, the rest 0) each group sum is pinned on its own.

Reference contract: src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:62-81 (exact int32 dot
per group, fp32 scale accumulation).
"""
import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def extreme_problem(O, seed, M, N, K, bits):
    """Arbitrary bytes and activations over all of int8; rows 0 / 1 of the weights are 0x00 /
    0xFF, tokens 0 / 1 (where present) are all -128 / all 127."""
    rng = np.random.default_rng(seed)
    p = O.synth_problem(seed, M, N, K, bits)
    p["A"] = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    p["A"][0, :] = -128
    if M > 1:
        p["A"][1, :] = 127
    p["B"] = rng.integers(0, 256, size=p["B"].shape, dtype=np.uint8)
    p["B"][0, :] = 0x00
    if N > 1:
        p["B"][1, :] = 0xFF
    return p


def dev_tensors(p):
    A = torch.from_numpy(p["A"]).to(DEV)
    B = torch.from_numpy(p["B"].view(np.int8)).to(DEV)
    s = torch.from_numpy(p["s"].reshape(-1, 1).copy()).to(DEV)
    ws = torch.from_numpy(p["ws"].view(np.int16).copy()).view(torch.bfloat16).to(DEV)
    return A, B, s, ws


def same_build(a: str, b: str) -> bool:
    """Kernel names agree in everything but their last template argument (the output kind)."""
    return a.rsplit(",", 1)[0] == b.rsplit(",", 1)[0]


def integer_product(O, p, bits):
    """unpack(B) @ A as integers [M, N]: a float64 matrix product of the unpacked weights (exact:
    every partial sum is an integer far below 2**53) for matrices up to 2**25 weights, the sum of
    the oracle's int32 group sums above (the oracle is pinned against that product elsewhere)."""
    if p["B"].shape[0] * p["A"].shape[1] <= (1 << 25):
        w = O.np_unpack(p["B"], bits).astype(np.float64)
        return np.rint(p["A"].astype(np.float64) @ w.T).astype(np.int64)
    return O.c_group_sums(p["A"], p["B"], bits).astype(np.int64).sum(-1)


def check_exact(O, ops, problems, bits, family, grouped, label):
    """G from the named kernel family, bit-exact; unit scales give the integer product exactly;
    one-hot scales give single group sums exactly; the ordinary result within tolerance."""
    devs = [dev_tensors(p) for p in problems]
    shapes = [(p["A"].shape[0], p["B"].shape[0], p["A"].shape[1]) for p in problems]
    print(f"[case] headline {label} bits={bits} grouped={grouped} (M,N,K)={shapes}", flush=True)

    def run(quads, out_kind):
        if grouped:
            outs = ops.packed_gemv_grouped(quads, bits=bits, out_kind=out_kind)
        else:
            outs = [ops.packed_gemv_ex(*q, bits=bits, out_kind=out_kind) for q in quads]
        torch.cuda.synchronize()
        return outs, ops.last_kernel(bits)

    G, k_g = run([(A, B, None, None) for A, B, s, ws in devs], ops.OUT_G32)
    y16, k_16 = run(devs, ops.OUT_BF16)
    y32, k_32 = run(devs, ops.OUT_F32)
    assert k_16.startswith(family + "<"), f"{label}: bf16 result came from {k_16}, not {family}"
    assert same_build(k_g, k_16) and same_build(k_32, k_16), \
        f"{label}: group sums from {k_g}, fp32 from {k_32}, bf16 from {k_16}"
    ones = [(A, B, torch.ones_like(s), torch.ones_like(ws)) for A, B, s, ws in devs]
    y_unit, k_u = run(ones, ops.OUT_F32)
    assert same_build(k_u, k_16)
    for i, p in enumerate(problems):
        G_ref = O.c_group_sums(p["A"], p["B"], bits)
        assert np.array_equal(G[i].cpu().numpy(), G_ref), f"{label}[{i}]: int32 group sums differ"
        want = integer_product(O, p, bits)
        assert np.abs(want).max() < 2 ** 24
        assert np.array_equal(y_unit[i].cpu().numpy(), want.astype(np.float32)), \
            f"{label}[{i}]: unit-scale fp32 result is not the integer product"
        y32_ref, y16_ref = O.c_gemv(p["A"], p["B"], p["s"], p["ws"], bits)
        got = y32[i].cpu().numpy()
        assert np.all(np.abs(got - y32_ref) <= 1e-3 + 1e-3 * np.abs(y32_ref)), f"{label}[{i}]: fp32"
        d = np.abs(bf16_ordinal(bf16_bits(y16[i])) - bf16_ordinal(y16_ref))
        assert d.max() <= 1, f"{label}[{i}]: bf16 more than one representable value away"
        assert np.array_equal(bf16_bits(y16[i]), O.f32_to_bf16_bits(got)), f"{label}[{i}]: bf16 != rne(fp32)"
    # one-hot scales: first, a middle and the last group of every problem
    ngs = [p["A"].shape[1] // 128 for p in problems]
    for pick in (0, 1, 2):
        hot = []
        for (A, B, s, ws), ng in zip(devs, ngs):
            g = (0, ng // 2, ng - 1)[pick]
            w1 = torch.zeros_like(ws)
            w1[:, g] = 1.0
            hot.append((A, B, torch.ones_like(s), w1))
        y_hot, k_h = run(hot, ops.OUT_F32)
        assert same_build(k_h, k_16)
        for i, (p, ng) in enumerate(zip(problems, ngs)):
            g = (0, ng // 2, ng - 1)[pick]
            G_ref = O.c_group_sums(p["A"], p["B"], bits)[:, :, g].astype(np.float32)
            assert np.array_equal(y_hot[i].cpu().numpy(), G_ref), f"{label}[{i}]: group {g} alone"
    return k_16


# ---- the lean matrix-core kernel, single launches: every build the host picks --------------
# (M, N, K) -> the build it reaches: MR 4 / NB 1 (3..8 tokens), NB 2 (9..16), W = 12 (one matrix
# with K >= 3072 and at most one row tile per CU), dense (more than four workgroups per CU)
MXL_SINGLE = [
    (3, 2048, 2048), (8, 4096, 2048), (9, 2048, 2048), (16, 1024, 2048),
    (4, 4096, 2560), (8, 6144, 2560), (9, 1024, 2560), (16, 2560, 2560),
    (3, 2048, 6144), (8, 2048, 6144), (9, 2048, 6144), (16, 2048, 6144),   # W = 12
    (4, 2560, 9728), (8, 2560, 9728), (16, 2560, 9728),                    # W = 12
    (8, 8192, 6144),                                                        # W = 4, K = 6144
    (4, 19456, 2560), (9, 19456, 2560), (16, 19456, 2560),                  # dense
    (2, 2560, 9728),                                                        # two tokens, long rows
]


@pytest.mark.parametrize("M,N,K", MXL_SINGLE)
def test_lean_kernel_single_t2(oracle, M, N, K):
    import bitmtp_amd as ops
    name = check_exact(oracle, ops, [extreme_problem(oracle, M * 7 + N + K, M, N, K, 2)], 2,
                       "gemv_mxl_kernel", False, "lean single")
    # <BITS, MR, SF16, W, NB, OCC, G32>
    args = [int(x) for x in name[name.index("<") + 1:-1].split(",")]
    assert args[3] == (12 if K >= 3072 and N <= 4096 else 4), name
    assert args[4] == (2 if M > 8 else 1), name


@pytest.mark.parametrize("M,N,K", [(3, 2560, 2560), (8, 9728, 2560), (9, 1024, 9728), (16, 2560, 9728),
                                   (8, 19456, 2560)])
def test_lean_kernel_single_q1(oracle, M, N, K):
    import bitmtp_amd as ops
    check_exact(oracle, ops, [extreme_problem(oracle, M + N + K, M, N, K, 1)], 1,
                "gemv_mxl_kernel", False, "lean single q1")


# ---- grouped launches ---------------------------------------------------------------------
LAYER_17B = [(2048, 2048), (1024, 2048), (1024, 2048), (2048, 2048), (6144, 2048), (6144, 2048),
             (2048, 6144)]
LAYER_4B = [(4096, 2560), (1024, 2560), (1024, 2560), (2560, 4096), (9728, 2560), (9728, 2560),
            (2560, 9728)]


@pytest.mark.parametrize("M", [3, 4, 8, 9, 16])
@pytest.mark.parametrize("layer", ["1.7b", "4b"])
def test_lean_kernel_grouped_layer_t2(oracle, layer, M):
    """The seven projections of a layer in one launch: the headline workload's own kernel on
    extreme bytes, unit scales and one-hot scales (1.7B: 1280 workgroups, the dense build)."""
    import bitmtp_amd as ops
    shapes = LAYER_17B if layer == "1.7b" else LAYER_4B
    probs = [extreme_problem(oracle, 100 * M + i, M, n, k, 2) for i, (n, k) in enumerate(shapes)]
    check_exact(oracle, ops, probs, 2, "gemv_mxl_kernel", True, f"lean grouped {layer}")


def test_lean_kernel_grouped_one_token_blocks_forced(oracle):
    """The MR = 1 build (every block one token) is reachable only with the narrow grouped kernel
    switched off: forced through the grouped tuning hook."""
    import bitmtp_amd as ops
    from bitmtp_amd import ops as O2
    lib = O2.t2_lib()
    try:
        lib.t2g128_set_grouped_tuning(0, 0, 1)
        probs = [extreme_problem(oracle, 900 + i, 1, n, k, 2) for i, (n, k) in enumerate(LAYER_17B)]
        name = check_exact(oracle, ops, probs, 2, "gemv_mxl_kernel", True, "lean grouped MR=1")
        assert name.startswith("gemv_mxl_kernel<2,1,"), name
    finally:
        lib.t2g128_set_grouped_tuning(0, 0, 0)


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("layer", ["1.7b", "4b"])
def test_narrow_grouped_kernel(oracle, bits, M, layer):
    """One- and two-token grouped launches: the grouped dot4 kernel, K = 2048 / 6144 and
    2560 / 4096 / 9728."""
    import bitmtp_amd as ops
    shapes = LAYER_17B if layer == "1.7b" else LAYER_4B
    probs = [extreme_problem(oracle, 300 * M + i + bits, M, n, k, bits) for i, (n, k) in enumerate(shapes)]
    check_exact(oracle, ops, probs, bits, "gemv_dot4_grouped_kernel", True, f"narrow grouped {layer}")


# ---- the kernels for very long matrices, forced onto shapes the oracle finishes quickly ----
@pytest.fixture
def forced_engine():
    from bitmtp_amd import ops as O2
    t2, q1 = O2.t2_lib(), O2.q1_lib()

    def force(engine):
        t2.t2g128_set_mfma_tuning(0, 0, 0, 0, engine)
        q1.q1g128_set_mfma_tuning(0, 0, 0, 0, engine)

    yield force
    force(0)


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M,N,K", [(1, 3000, 2048), (4, 4099, 2048), (8, 2000, 2560), (9, 1500, 6144),
                                   (16, 700, 4096), (4, 700, 9728), (2, 1030, 2048)])
def test_streaming_kernel(oracle, forced_engine, bits, M, N, K):
    import bitmtp_amd as ops
    forced_engine(5)
    check_exact(oracle, ops, [extreme_problem(oracle, 50 + M + N + K + bits, M, N, K, bits)], bits,
                "gemv_mxs_kernel", False, "streaming")


@pytest.mark.parametrize("N,K", [(3000, 1024), (3001, 2048), (1500, 4096)])
def test_single_token_register_kernel(oracle, forced_engine, N, K):
    import bitmtp_amd as ops
    forced_engine(6)
    check_exact(oracle, ops, [extreme_problem(oracle, 70 + N + K, 1, N, K, 2)], 2,
                "gemv_rowreg_kernel", False, "single token")


def test_head_shape_group_sums_from_the_head_kernels(oracle):
    """At the real head shape the default dispatch's own kernels return the group sums: a sample
    of rows against the oracle (the full product at 151936 rows is left to the float checks)."""
    import bitmtp_amd as ops
    N, K = 151936, 2048
    rng = np.random.default_rng(5)
    Bp = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    rows = np.concatenate([np.arange(0, 64), rng.integers(0, N, 512), np.arange(N - 64, N)])
    B = torch.from_numpy(Bp.view(np.int8)).to(DEV)
    for M, family in ((1, "gemv_rowreg_kernel"), (8, "gemv_mxs_kernel"), (16, "gemv_mxs_kernel")):
        A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
        A[0, :] = -128
        print(f"[case] headline head M={M}", flush=True)
        G = ops.packed_gemv_ex(torch.from_numpy(A).to(DEV), B, None, None, bits=2, out_kind=ops.OUT_G32)
        torch.cuda.synchronize()
        assert ops.last_kernel(2).startswith(family + "<"), ops.last_kernel(2)
        G_ref = oracle.c_group_sums(A, Bp[rows], 2)
        assert np.array_equal(G[:, torch.from_numpy(rows).to(DEV), :].cpu().numpy(), G_ref)
