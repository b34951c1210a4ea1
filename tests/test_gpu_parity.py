"""GPU parity of the HIP packed GEMV against the CPU oracle, through the C ABI.

Bars: int32 group sums bit-exact; fp32 value (before the bf16 rounding) within
rtol 1e-3 / atol 1e-3; bf16 output equal to, or the representable neighbour of,
the oracle's bf16; activation quantisation bit-exact.
"""
import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal, to_dev

pytestmark = pytest.mark.gpu

RTOL = 1e-3
ATOL = 1e-3


def _ops():
    import bitmtp_amd
    return bitmtp_amd


def check_problem(O, p, bits, label):
    ops = _ops()
    A, B, s, ws = to_dev(p)
    print(f"[case] {label} bits={bits} M={A.shape[0]} N={B.shape[0]} K={A.shape[1]}", flush=True)
    G = ops.packed_gemv_ex(A, B, None, None, bits=bits, out_kind=ops.OUT_G32)
    k_g = ops.last_kernel(bits)
    y32 = ops.packed_gemv_ex(A, B, s, ws, bits=bits, out_kind=ops.OUT_F32)
    y16 = ops.packed_int8_linear(A, B, s, ws)
    k_16 = ops.last_kernel(bits)
    torch.cuda.synchronize()
    # the group sums come from the same kernel build that produces the bf16 result (the names
    # differ in their last template argument, the output kind, only)
    assert k_g.rsplit(",", 1)[0] == k_16.rsplit(",", 1)[0], f"{label}: G from {k_g}, bf16 from {k_16}"
    G_ref = O.c_group_sums(p["A"], p["B"], bits)
    y32_ref, y16_ref = O.c_gemv(p["A"], p["B"], p["s"], p["ws"], bits)
    assert np.array_equal(G.cpu().numpy(), G_ref), f"{label}: int32 group sums differ"
    got = y32.cpu().numpy()
    err = np.abs(got - y32_ref)
    assert np.all(err <= ATOL + RTOL * np.abs(y32_ref)), f"{label}: fp32 max err {err.max()}"
    d = np.abs(bf16_ordinal(bf16_bits(y16)) - bf16_ordinal(y16_ref))
    assert d.max() <= 1, f"{label}: bf16 output more than one representable value away"
    # the bf16 entry point rounds the same fp32 value the F32 entry point returns
    assert np.array_equal(bf16_bits(y16), O.f32_to_bf16_bits(got)), f"{label}: bf16 != rne(fp32)"


SMALL_SHAPES = [
    # M, N, K
    (1, 1, 128), (1, 8, 256), (2, 5, 384), (3, 37, 512), (1, 64, 2048), (4, 100, 2560),
    (8, 33, 1024), (5, 130, 4096), (7, 17, 6144), (1, 24, 9728), (8, 24, 9728),
    (9, 40, 2048), (17, 19, 2560), (16, 8, 9728), (33, 9, 640),
]


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M,N,K", SMALL_SHAPES)
def test_small_shapes(oracle, bits, M, N, K):
    p = oracle.synth_problem(100 + M + N + K, M, N, K, bits)
    check_problem(oracle, p, bits, "small")


@pytest.mark.parametrize("bits", [2, 1])
def test_random_shapes(oracle, bits):
    """Forty seeded random (M, N, K): every width 1..17, ragged N, every K that is a multiple
    of 128 up to 9728 -- whatever kernel and geometry the dispatcher picks for them."""
    rng = np.random.default_rng(2024 + bits)
    for i in range(40):
        M = int(rng.integers(1, 18))
        N = int(rng.integers(1, 600))
        K = 128 * int(rng.integers(1, 77))
        p = oracle.synth_problem(5000 + i, M, N, K, bits)
        check_problem(oracle, p, bits, f"random {i}")


@pytest.mark.parametrize("bits", [2, 1])
def test_arbitrary_bytes_and_extreme_activations(oracle, bits):
    """Every byte value (T2 code 0 -> -2 included) and activations over all of int8."""
    rng = np.random.default_rng(7)
    for M, N, K in ((6, 96, 1536), (6, 96, 2048), (2, 300, 2048), (1, 300, 6144)):
        p = oracle.synth_problem(7, M, N, K, bits)
        p["A"] = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
        p["A"][0, :] = -128
        if M > 1:
            p["A"][1, :] = 127
        p["B"] = rng.integers(0, 256, size=p["B"].shape, dtype=np.uint8)
        p["B"][0, :] = 0x00
        p["B"][1, :] = 0xFF
        check_problem(oracle, p, bits, "extreme")


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("lpr,waves,passes", [
    (4, 1, 1), (8, 4, 1), (8, 8, 3), (16, 2, 2), (32, 4, 1), (64, 8, 2), (64, 1, 5),
])
def test_launch_geometries(oracle, bits, lpr, waves, passes):
    """Every lanes-per-row / workgroup / pass combination computes the same thing."""
    ops = _ops()
    from bitmtp_amd import ops as O2
    lib = O2.t2_lib() if bits == 2 else O2.q1_lib()
    setter = lib.t2g128_set_tuning if bits == 2 else lib.q1g128_set_tuning
    try:
        setter(lpr, waves, passes)
        for (M, N, K) in [(1, 70, 2048), (3, 257, 2560), (8, 50, 9728), (2, 9, 128)]:
            p = oracle.synth_problem(lpr * 1000 + waves * 10 + passes + K, M, N, K, bits)
            check_problem(oracle, p, bits, f"geom lpr={lpr} waves={waves} passes={passes}")
    finally:
        setter(0, 0, 0)


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("engine", [1, 3])
@pytest.mark.parametrize("min_width,row_tiles,k_split,passes", [
    (1, 1, 1, 1), (1, 2, 2, 0), (1, 4, 4, 0), (2, 1, 4, 0), (2, 4, 1, 3), (2, 2, 1, 2),
    (1, 1, 1, 5), (1, 1, 8, 0), (2, 2, 8, 0), (1000, 0, 0, 0),
    (1, 1, 3, 0), (1, 1, 5, 0), (2, 0, 12, 0),
])
def test_mfma_geometries(oracle, bits, engine, min_width, row_tiles, k_split, passes):
    """The matrix-core kernels (1 = int8 MFMA with staged activations,
    3 = int8 MFMA with activations loaded as operands): every row-tile /
    K-split / pass combination (a split of eight is the eight-wave form of engine 3, taken
    for K >= 4096, splits of 3, 5 and 12 its one-slice-per-wave form; engine 1 and
    shorter rows fall back to no split), including a
    single token sent through them, and the dot4 kernel forced for every width
    (min_width 1000)."""
    from bitmtp_amd import ops as O2
    lib = O2.t2_lib() if bits == 2 else O2.q1_lib()
    setter = lib.t2g128_set_mfma_tuning if bits == 2 else lib.q1g128_set_mfma_tuning
    try:
        setter(min_width, row_tiles, k_split, passes, engine)
        for (M, N, K) in [(1, 70, 2048), (3, 257, 2560), (8, 50, 9728), (16, 33, 512),
                          (17, 130, 1024), (5, 16, 6144)]:
            p = oracle.synth_problem(min_width * 100 + row_tiles * 10 + k_split + K, M, N, K, bits)
            check_problem(oracle, p, bits,
                          f"mfma engine={engine} min={min_width} R={row_tiles} ks={k_split} "
                          f"passes={passes}")
    finally:
        setter(0, 0, 0, 0, 0)


LAYER_17B = [(2048, 2048), (1024, 2048), (6144, 2048), (2048, 6144)]
LAYER_4B_Q1 = [(1024, 2560), (2560, 2560), (9728, 2560), (1024, 9728), (2560, 9728), (9728, 9728)]


@pytest.mark.parametrize("M", [1, 4, 8])
@pytest.mark.parametrize("N,K", LAYER_17B)
def test_t2_layer_shapes_full_size(oracle, M, N, K):
    """Benchmark configs 0/1: the 1.7B-shaped layer projections at widths 1, 4, 8."""
    p = oracle.synth_problem(1, M, N, K, 2)
    check_problem(oracle, p, 2, "t2-1.7B-layer")


@pytest.mark.parametrize("M", [1, 3, 8])
@pytest.mark.parametrize("N,K", LAYER_4B_Q1)
def test_q1_4b_shapes_full_size(oracle, M, N, K):
    """Benchmark config 4: Q1 on the 4B-shaped layer set."""
    p = oracle.synth_problem(4, M, N, K, 1)
    check_problem(oracle, p, 1, "q1-4B")


@pytest.mark.parametrize("M,N,K", [(1, 4096, 2048), (9, 12288, 2048), (17, 2560, 9728),
                                    (16, 19456, 2560), (12, 6144, 2560), (10, 2560, 4096),
                                    (9, 2048, 6144), (16, 4096, 2560), (9, 1024, 2560)])
def test_t2_decode_widths_merged_shapes(oracle, M, N, K):
    """Merged decode shapes at the widths a D8 schedule replays (9..17)."""
    p = oracle.synth_problem(2, M, N, K, 2)
    check_problem(oracle, p, 2, "t2-merged")


@pytest.mark.parametrize("bits,M,N,K", [(2, 3, 12288, 4096), (2, 16, 9728, 9728), (2, 17, 12288, 4096),
                                         (2, 8, 24576, 4096), (2, 2, 2048, 6144), (2, 2, 2560, 9728),
                                         (1, 2, 9728, 9728), (1, 16, 12288, 4096), (2, 32, 19456, 2560),
                                         (2, 33, 4100, 5120),
                                         (2, 9, 19456, 2560), (2, 9, 24576, 4096), (1, 9, 19456, 2560)])
def test_larger_single_matrices_and_two_token_long_rows(oracle, bits, M, N, K):
    """Single matrices with more 16-row tiles than CUs and long rows (several K tiles per wave of
    the lean matrix-core kernel, two and three token tiles), the two-token blocks that go to the
    matrix cores for K >= 4096, the 32-row prefill width on the widest merged matrix, and nine tokens
    on matrices with more than four row tiles per CU (the 96-register build of the lean kernel)."""
    p = oracle.synth_problem(300 + M + N // 7, M, N, K, bits)
    check_problem(oracle, p, bits, "large-single")


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M,N,K", [(1, 2049, 2048), (2, 4100, 2048), (1, 2050, 6144),
                                    (9, 2050, 6144), (9, 4090, 2560), (16, 1030, 9728)])
def test_ragged_rows_at_layer_size(oracle, bits, M, N, K):
    """Row counts that are no multiple of a workgroup's rows, at sizes where the launcher
    picks its eight-wave and one-slice-per-wave geometries."""
    p = oracle.synth_problem(77 + M + N, M, N, K, bits)
    check_problem(oracle, p, bits, "ragged")


def test_t2_head_shape(oracle):
    """The packed lm_head: N = 151936, width D+1 = 9."""
    p = oracle.synth_problem(3, 9, 151936, 2048, 2)
    check_problem(oracle, p, 2, "t2-head")


def test_known_answers():
    """Hand-derived results: K=128 all +1 weights, scale 0.5, x = 1 -> 64.0; alternating
    +1/-1 -> 0; two groups with scales 1 and 0.25 -> 160.0."""
    ops = _ops()
    dev = "cuda:0"
    one = torch.ones(1, 128, device=dev, dtype=torch.bfloat16)
    q, s = ops.quant_input(one)
    assert float(s.item()) == 127.0 and int(q.min()) == 127 and int(q.max()) == 127
    B = torch.full((1, 32), -1, dtype=torch.int8, device=dev)  # 0xFF: four +1 codes
    ws = torch.tensor([[0.5]], dtype=torch.bfloat16, device=dev)
    y = ops.t2g128_int8xint2_linear(q, B, s, ws)
    G = ops.packed_gemv_ex(q, B, None, None, bits=2, out_kind=ops.OUT_G32)
    assert int(G.item()) == 127 * 128 and float(y.item()) == 64.0
    B_alt = torch.full((1, 32), 0x77, dtype=torch.int8, device=dev)  # codes 3,1,3,1
    assert float(ops.t2g128_int8xint2_linear(q, B_alt, s, ws).item()) == 0.0
    two = torch.ones(1, 256, device=dev, dtype=torch.bfloat16)
    q2, s2 = ops.quant_input(two)
    B2 = torch.full((1, 64), -1, dtype=torch.int8, device=dev)
    ws2 = torch.tensor([[1.0, 0.25]], dtype=torch.bfloat16, device=dev)
    assert float(ops.t2g128_int8xint2_linear(q2, B2, s2, ws2).item()) == 160.0
    # Q1: all bits set -> +1 weights
    Bq = torch.full((1, 16), -1, dtype=torch.int8, device=dev)
    assert float(ops.q1g128_int8xint1_linear(q, Bq, s, ws).item()) == 64.0
    Bq0 = torch.zeros((1, 16), dtype=torch.int8, device=dev)  # all -1
    assert float(ops.q1g128_int8xint1_linear(q, Bq0, s, ws).item()) == -64.0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,K", [(1, 128), (3, 2048), (8, 2560), (17, 9728), (5, 6144)])
def test_act_quant_bit_exact(oracle, dtype, M, K):
    ops = _ops()
    g = torch.Generator().manual_seed(M * 10000 + K)
    x = (torch.randn(M, K, generator=g) * 3.0).to(dtype)
    if M >= 3:
        x[1].zero_()                      # all-zero row: absmax clamps to 1e-5
        x[2] = x[2] * 1e-7                # tiny row
    print(f"[case] act_quant {dtype} M={M} K={K}", flush=True)
    q, s = ops.quant_input(x.to("cuda:0"))
    torch.cuda.synchronize()
    q_ref, s_ref = oracle.c_act_quant(x.float().numpy())
    assert s.shape == (M, 1) and s.dtype == torch.float32 and q.dtype == torch.int8
    assert np.array_equal(s.cpu().numpy().reshape(-1), s_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)


def test_act_quant_half_even_known_answer():
    """x*s lands exactly on .5: [127, 0.5, 1.5, 2.5, -1.5] -> [127, 0, 2, 2, -2]."""
    ops = _ops()
    x = torch.zeros(1, 128, dtype=torch.float16)
    x[0, :5] = torch.tensor([127 / 64, 1 / 128, 3 / 128, 5 / 128, -3 / 128], dtype=torch.float16)
    q, s = ops.quant_input(x.to("cuda:0"))
    assert float(s.item()) == 64.0
    assert q[0, :6].tolist() == [127, 0, 2, 2, -2, 0]


@pytest.mark.parametrize("bits", [2, 1])
def test_rank3_and_dequant_cross_check(oracle, bits):
    """Rank-3 activations keep their batch shape, and the op agrees with the
    dequantise-then-matmul statement of the same linear (fp64 here)."""
    ops = _ops()
    Bsz, S, N, K = 2, 3, 48, 1024
    p = oracle.synth_problem(11, Bsz * S, N, K, bits)
    A, B, s, ws = to_dev(p)
    y = ops.packed_int8_linear(A.view(Bsz, S, K), B, s.view(Bsz, S, 1), ws)
    assert y.shape == (Bsz, S, N) and y.dtype == torch.bfloat16
    W = oracle.np_unpack(p["B"], bits).astype(np.float64) * np.repeat(
        oracle.bf16_bits_to_f32(p["ws"]).astype(np.float64), 128, axis=1)
    ref = (p["A"].astype(np.float64) / p["s"].astype(np.float64)[:, None]) @ W.T
    got = y.float().cpu().numpy().reshape(Bsz * S, N)
    assert np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-3)  # bf16 output: 2^-8 relative


def test_fp16_scales(oracle):
    ops = _ops()
    p = oracle.synth_problem(12, 4, 64, 2048, 2)
    ws16 = oracle.bf16_bits_to_f32(p["ws"]).astype(np.float16)
    A, B, s, _ = to_dev(p)
    ws = torch.from_numpy(ws16).to("cuda:0")
    y32 = ops.packed_gemv_ex(A, B, s, ws, bits=2, out_kind=ops.OUT_F32).cpu().numpy()
    ref, _ = oracle.c_gemv(p["A"], p["B"], p["s"], ws16.view(np.uint16), 2, scale_is_f16=True)
    assert np.all(np.abs(y32 - ref) <= ATOL + RTOL * np.abs(ref))


def test_linearity_in_scales_full_size(oracle):
    """Size-independent property at a full benchmark shape: doubling every group
    scale doubles the fp32 result exactly; zeroing all but one group isolates it."""
    ops = _ops()
    p = oracle.synth_problem(13, 8, 6144, 2048, 2)
    A, B, s, ws = to_dev(p)
    y1 = ops.packed_gemv_ex(A, B, s, ws, bits=2, out_kind=ops.OUT_F32)
    y2 = ops.packed_gemv_ex(A, B, s, (ws.float() * 2).to(torch.bfloat16), bits=2, out_kind=ops.OUT_F32)
    assert torch.equal(y2, y1 * 2)
    ws_one = torch.zeros_like(ws)
    ws_one[:, 5] = ws[:, 5]
    y5 = ops.packed_gemv_ex(A, B, s, ws_one, bits=2, out_kind=ops.OUT_F32)
    G = ops.packed_gemv_ex(A, B, None, None, bits=2, out_kind=ops.OUT_G32)
    expect = (G[:, :, 5].float() * ws[:, 5].float()[None, :]) / s
    assert torch.equal(y5, expect)


def test_stream_and_graph_replay(oracle):
    """The entry point enqueues on the current stream only and can be captured; three
    replays with eager work in between reproduce the eager result."""
    ops = _ops()
    ops.init_kernels()
    p = oracle.synth_problem(14, 8, 2048, 2048, 2)
    A, B, s, ws = to_dev(p)
    eager = ops.packed_int8_linear(A, B, s, ws).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            out = ops.packed_int8_linear(A, B, s, ws)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert torch.equal(out, eager)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        cap = ops.packed_int8_linear(A, B, s, ws)
    for i in range(3):
        cap.zero_()
        _ = ops.packed_int8_linear(A, B, s, ws)  # eager work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(cap, eager), f"replay {i} differs"
