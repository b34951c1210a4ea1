"""GPU parity of the grouped GEMV entry points (`t2g128_gemv_grouped`, `q1g128_gemv_grouped`)
against the CPU oracle, through the C ABI: every descriptor of a call is checked as a GEMV of
its own -- int32 group sums bit-exact, fp32 value within rtol 1e-3 / atol 1e-3, bf16 output the
oracle's or the neighbouring representable value, and equal to the RNE rounding of the fp32
value the same call returns.
"""
import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal, to_dev

pytestmark = pytest.mark.gpu

RTOL = 1e-3
ATOL = 1e-3

LAYER_17B = [(2048, 2048), (1024, 2048), (1024, 2048), (2048, 2048), (6144, 2048), (6144, 2048),
             (2048, 6144)]
LAYER_4B = [(4096, 2560), (1024, 2560), (1024, 2560), (2560, 4096), (9728, 2560), (9728, 2560),
            (2560, 9728)]


def check_group(O, probs, bits, label):
    import bitmtp_amd as ops
    dev = [to_dev(p) for p in probs]
    shapes = [(p["A"].shape[0], p["B"].shape[0], p["A"].shape[1]) for p in probs]
    print(f"[case] grouped {label} bits={bits} (M,N,K)={shapes}", flush=True)
    n0 = ops.launch_count(bits)
    G = ops.packed_gemv_grouped([(A, B, None, None) for A, B, s, ws in dev], bits=bits,
                                out_kind=ops.OUT_G32)
    k_g, n1 = ops.last_kernel(bits), ops.launch_count(bits)
    y32 = ops.packed_gemv_grouped(dev, bits=bits, out_kind=ops.OUT_F32)
    n2 = ops.launch_count(bits)
    y16 = ops.packed_gemv_grouped(dev, bits=bits, out_kind=ops.OUT_BF16)
    k_16 = ops.last_kernel(bits)
    torch.cuda.synchronize()
    # the group sums take the same launches as the results (same kernel builds, same count)
    assert k_g.rsplit(",", 1)[0] == k_16.rsplit(",", 1)[0], f"{label}: G from {k_g}, bf16 from {k_16}"
    assert n1 - n0 == n2 - n1, f"{label}: {n1 - n0} launches for G, {n2 - n1} for the fp32 result"
    for i, p in enumerate(probs):
        G_ref = O.c_group_sums(p["A"], p["B"], bits)
        y32_ref, y16_ref = O.c_gemv(p["A"], p["B"], p["s"], p["ws"], bits)
        assert np.array_equal(G[i].cpu().numpy(), G_ref), f"{label}[{i}]: int32 group sums differ"
        got = y32[i].cpu().numpy()
        err = np.abs(got - y32_ref)
        assert np.all(err <= ATOL + RTOL * np.abs(y32_ref)), f"{label}[{i}]: fp32 max err {err.max()}"
        d = np.abs(bf16_ordinal(bf16_bits(y16[i])) - bf16_ordinal(y16_ref))
        assert d.max() <= 1, f"{label}[{i}]: bf16 output more than one representable value away"
        assert np.array_equal(bf16_bits(y16[i]), O.f32_to_bf16_bits(got)), f"{label}[{i}]: bf16 != rne(fp32)"


@pytest.mark.parametrize("M", [1, 4, 8, 9, 17])
def test_t2_17b_layer_in_one_call(oracle, M):
    """All seven projections of the 1.7B-shaped layer (K = 2048 and 6144 mixed) in one call."""
    probs = [oracle.synth_problem(10 * M + i, M, n, k, 2) for i, (n, k) in enumerate(LAYER_17B)]
    check_group(oracle, probs, 2, f"1.7B layer M={M}")


@pytest.mark.parametrize("M", [1, 8, 16])
def test_t2_4b_layer_in_one_call(oracle, M):
    """The 4B-shaped layer: K in {2560, 4096, 9728} (5, 8 and 19 K tiles over four waves)."""
    probs = [oracle.synth_problem(20 * M + i, M, n, k, 2) for i, (n, k) in enumerate(LAYER_4B)]
    check_group(oracle, probs, 2, f"4B layer M={M}")


@pytest.mark.parametrize("M", [1, 3, 8])
def test_q1_4b_set_in_one_call(oracle, M):
    shapes = [(1024, 2560), (2560, 2560), (9728, 2560), (1024, 9728), (2560, 9728)]
    probs = [oracle.synth_problem(30 * M + i, M, n, k, 1) for i, (n, k) in enumerate(shapes)]
    check_group(oracle, probs, 1, f"Q1 4B set M={M}")


@pytest.mark.parametrize("bits", [2, 1])
def test_mixed_widths_ragged_rows_and_odd_k(oracle, bits):
    """Different M, N, K per descriptor; row counts that are no multiple of 16; K values the
    grouped kernel does not take (below 2048 or no multiple of 512: they run through the
    single-GEMV path inside the same call); blocks wider than 16 tokens."""
    shapes = [(1, 2049, 2048), (9, 17, 512), (17, 130, 1024), (4, 1, 2560), (8, 1030, 6144),
              (2, 33, 384), (33, 9, 640), (16, 50, 9728), (5, 255, 1536), (3, 100, 128)]
    probs = [oracle.synth_problem(400 + i, m, n, k, bits) for i, (m, n, k) in enumerate(shapes)]
    check_group(oracle, probs, bits, "mixed")


def test_more_descriptors_than_one_launch_holds(oracle):
    """40 small problems: more than the 24 descriptors of one launch."""
    rng = np.random.default_rng(5)
    probs = []
    for i in range(40):
        m, n, k = int(rng.integers(1, 18)), int(rng.integers(1, 200)), 512 * int(rng.integers(4, 9))
        probs.append(oracle.synth_problem(600 + i, m, n, k, 2))
    check_group(oracle, probs, 2, "many")


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("row_tiles,max_wgs", [(1, 0), (2, 0), (1, 7), (2, 5), (1, 16), (2, 64)])
def test_grouped_geometries(oracle, bits, row_tiles, max_wgs):
    """One or two row tiles per wave compute the same thing, also when a small cap on the
    workgroups makes every workgroup stride over several row-block iterations (the path the
    151936-row head takes), restaging its activation tiles as it goes."""
    from bitmtp_amd import ops as O2
    lib = O2.t2_lib() if bits == 2 else O2.q1_lib()
    setter = lib.t2g128_set_grouped_tuning if bits == 2 else lib.q1g128_set_grouped_tuning
    shapes = [(1, 300, 2048), (8, 77, 2560), (16, 200, 4096), (5, 129, 6144), (3, 64, 3072), (16, 40, 9728),
              (9, 33, 2048)]
    try:
        setter(row_tiles, max_wgs, 0)
        probs = [oracle.synth_problem(700 + 10 * row_tiles + i, m, n, k, bits)
                 for i, (m, n, k) in enumerate(shapes)]
        check_group(oracle, probs, bits, f"geom R={row_tiles} cap={max_wgs}")
    finally:
        setter(0, 0, 0)


@pytest.mark.parametrize("bits", [2, 1])
def test_grouped_arbitrary_bytes_and_extreme_activations(oracle, bits):
    rng = np.random.default_rng(9)
    probs = []
    for i, (M, N, K) in enumerate([(6, 96, 1536), (1, 40, 512), (5, 96, 2048), (2, 80, 2048), (1, 50, 6144), (9, 33, 2560)]):
        p = oracle.synth_problem(800 + i, M, N, K, bits)
        p["A"] = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
        p["A"][0, :] = -128
        p["B"] = rng.integers(0, 256, size=p["B"].shape, dtype=np.uint8)
        p["B"][0, :] = 0x00
        p["B"][1, :] = 0xFF
        probs.append(p)
    check_group(oracle, probs, bits, "extreme")


def test_grouped_head_and_single_descriptor(oracle):
    """One descriptor is a valid group: the packed lm_head at width 9."""
    check_group(oracle, [oracle.synth_problem(3, 9, 151936, 2048, 2)], 2, "head")


def test_grouped_equals_single_calls_bit_for_bit_per_kernel(oracle):
    """The grouped kernel through the single-GEMV entry point (engine 4) returns exactly what
    the grouped call returns for the same problem: the result does not depend on what else
    shares the launch."""
    import bitmtp_amd as ops
    from bitmtp_amd import ops as O2
    probs = [oracle.synth_problem(900 + i, 8, n, k, 2) for i, (n, k) in enumerate(LAYER_17B[3:])]
    dev = [to_dev(p) for p in probs]
    grouped = ops.packed_gemv_grouped(dev, bits=2, out_kind=ops.OUT_F32)
    lib = O2.t2_lib()
    try:
        lib.t2g128_set_mfma_tuning(1, 0, 0, 0, 4)
        for i, (A, B, s, ws) in enumerate(dev):
            alone = ops.packed_gemv_ex(A, B, s, ws, bits=2, out_kind=ops.OUT_F32)
            assert torch.equal(alone, grouped[i])
    finally:
        lib.t2g128_set_mfma_tuning(0, 0, 0, 0, 0)


def test_grouped_graph_replay_and_argument_errors(oracle):
    import bitmtp_amd as ops
    ops.init_kernels()
    probs = [oracle.synth_problem(950 + i, 8, n, k, 2) for i, (n, k) in enumerate(LAYER_17B)]
    dev = [to_dev(p) for p in probs]
    eager = [t.clone() for t in ops.packed_gemv_grouped(dev, bits=2)]
    outs = [torch.empty_like(t) for t in eager]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        ops.packed_gemv_grouped(dev, bits=2, outs=outs)
    for rep in range(3):
        for t in outs:
            t.zero_()
        _ = ops.packed_gemv_grouped(dev, bits=2)   # eager work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, eager):
            assert torch.equal(a, b), f"replay {rep} differs"
    with pytest.raises(ValueError):
        ops.packed_gemv_grouped([], bits=2)
    with pytest.raises(RuntimeError):
        ops.packed_gemv_grouped(dev, bits=2, outs=[torch.empty(1, 1, device="cuda:0")] * len(dev))
    A, B, s, ws = dev[0]
    with pytest.raises(RuntimeError):
        ops.packed_gemv_grouped([(A, B[:, :-32].contiguous(), s, ws)], bits=2)


@pytest.mark.parametrize("bits", [2, 1])
def test_narrow_blocks_share_a_dot4_launch(oracle, bits):
    """Blocks of one and two tokens go through the grouped form of the dot4 kernel: mixed widths,
    ragged row counts, K from 128 to 9728 (rows shorter than the lanes that share them and rows
    of many loads per lane), more problems than one launch holds."""
    shapes = [(1, 2048, 2048), (2, 1024, 2048), (1, 2048, 6144), (2, 33, 128), (1, 1, 384),
              (1, 1030, 2560), (2, 77, 9728), (1, 129, 4096), (2, 6144, 2048), (1, 17, 1536),
              (1, 300, 640), (2, 255, 3072), (1, 64, 512), (2, 9, 1024)]
    probs = [oracle.synth_problem(1100 + i, m, n, k, bits) for i, (m, n, k) in enumerate(shapes)]
    check_group(oracle, probs, bits, "narrow")


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M", [1, 2])
def test_narrow_grouped_equals_single_calls_bit_for_bit(oracle, bits, M):
    """The grouped dot4 launch runs the body of the single-GEMV dot4 kernel: whatever lanes per
    row and workgroup size the grouped launch picks, each row's lanes are added in the same tree
    order only if the geometry matches, so the check forces one geometry for both calls."""
    import bitmtp_amd as ops
    from bitmtp_amd import ops as O2
    lib = O2.t2_lib() if bits == 2 else O2.q1_lib()
    set_tuning = lib.t2g128_set_tuning if bits == 2 else lib.q1g128_set_tuning
    set_mfma = lib.t2g128_set_mfma_tuning if bits == 2 else lib.q1g128_set_mfma_tuning
    probs = [oracle.synth_problem(1200 + i, M, n, k, bits) for i, (n, k) in enumerate(LAYER_17B)]
    dev = [to_dev(p) for p in probs]
    try:
        set_tuning(16, 4, 0)
        set_mfma(100, 0, 0, 0, 0)  # the single calls stay on the dot4 kernel at width 2 as well
        grouped = ops.packed_gemv_grouped(dev, bits=bits, out_kind=ops.OUT_F32)
        for i, (A, B, s, ws) in enumerate(dev):
            alone = ops.packed_gemv_ex(A, B, s, ws, bits=bits, out_kind=ops.OUT_F32)
            assert torch.equal(alone, grouped[i]), f"problem {i}"
    finally:
        set_tuning(0, 0, 0)
        set_mfma(0, 0, 0, 0, 0)


def test_narrow_grouped_fp16_scales_and_graph_replay(oracle):
    import bitmtp_amd as ops
    probs = [oracle.synth_problem(1300 + i, 1, n, k, 2) for i, (n, k) in enumerate(LAYER_17B)]
    dev, ws16s = [], []
    for p in probs:
        A, B, s, _ = to_dev(p)
        ws16 = oracle.bf16_bits_to_f32(p["ws"]).astype(np.float16)
        ws16s.append(ws16)
        dev.append((A, B, s, torch.from_numpy(ws16).to("cuda:0")))
    y32 = ops.packed_gemv_grouped(dev, bits=2, out_kind=ops.OUT_F32)
    for i, p in enumerate(probs):
        ref, _ = oracle.c_gemv(p["A"], p["B"], p["s"], ws16s[i].view(np.uint16), 2, scale_is_f16=True)
        got = y32[i].cpu().numpy()
        assert np.all(np.abs(got - ref) <= ATOL + RTOL * np.abs(ref)), f"fp16 scales, problem {i}"
    eager = [t.clone() for t in ops.packed_gemv_grouped(dev, bits=2)]
    outs = [torch.empty_like(t) for t in eager]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        ops.packed_gemv_grouped(dev, bits=2, outs=outs)
    for rep in range(3):
        for t in outs:
            t.zero_()
        _ = ops.packed_gemv_grouped(dev, bits=2)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, eager):
            assert torch.equal(a, b), f"replay {rep} differs"


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_descriptor_sets(oracle, bits, seed):
    """Seeded random calls: 1 to 20 descriptors with any mix of widths 1..17, ragged row counts
    and K from 128 to 6144 -- narrow and wide blocks in one call, token tiling, more descriptors
    than one launch of either grouped kernel holds, shapes that fall back to the single-GEMV
    path -- each descriptor checked against the oracle as a GEMV of its own."""
    rng = np.random.default_rng(seed * 10 + bits)
    count = int(rng.integers(1, 21))
    ks = [128, 384, 512, 1024, 1536, 2048, 2560, 4096, 6144]
    probs = []
    for i in range(count):
        m = int(rng.choice([1, 1, 2, 3, 4, 8, 9, 16, 17]))
        n = int(rng.integers(1, 700))
        k = int(rng.choice(ks))
        probs.append(oracle.synth_problem(seed * 1000 + i, m, n, k, bits))
    check_group(oracle, probs, bits, f"random set seed={seed}")
