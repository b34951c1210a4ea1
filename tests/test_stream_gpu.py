"""GPU parity of the streaming matrix-core kernel (the one very long matrices such as the packed
lm_head take) against the CPU oracle, through the C ABI.  The kernel is forced on shapes the
oracle finishes in seconds (engine 5 of the tuning call) and checked at the full head shape through
the ordinary entry point: fp32 value within rtol 1e-3 / atol 1e-3, bf16 output the oracle's or the
neighbouring representable value and equal to the RNE rounding of the fp32 value.
"""
import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal, to_dev

pytestmark = pytest.mark.gpu

RTOL = 1e-3
ATOL = 1e-3


def check_one(O, p, bits, label, scale_kind=0):
    import bitmtp_amd as ops
    A, B, s, ws = to_dev(p)
    print(f"[case] stream {label} bits={bits} M={p['A'].shape[0]} N={p['B'].shape[0]} K={p['A'].shape[1]}",
          flush=True)
    y32 = ops.packed_gemv_ex(A, B, s, ws, bits=bits, out_kind=ops.OUT_F32)
    y16 = ops.packed_gemv_ex(A, B, s, ws, bits=bits, out_kind=ops.OUT_BF16)
    torch.cuda.synchronize()
    y32_ref, y16_ref = O.c_gemv(p["A"], p["B"], p["s"], p["ws"], bits)
    got = y32.cpu().numpy()
    err = np.abs(got - y32_ref)
    assert np.all(err <= ATOL + RTOL * np.abs(y32_ref)), f"{label}: fp32 max err {err.max()}"
    d = np.abs(bf16_ordinal(bf16_bits(y16)) - bf16_ordinal(y16_ref))
    assert d.max() <= 1, f"{label}: bf16 output more than one representable value away"
    assert np.array_equal(bf16_bits(y16), O.f32_to_bf16_bits(got)), f"{label}: bf16 != rne(fp32)"


@pytest.fixture
def forced_stream():
    from bitmtp_amd import ops as O2
    t2, q1 = O2.t2_lib(), O2.q1_lib()
    t2.t2g128_set_mfma_tuning(0, 0, 0, 0, 5)
    q1.q1g128_set_mfma_tuning(0, 0, 0, 0, 5)
    yield (t2, q1)
    t2.t2g128_set_mfma_tuning(0, 0, 0, 0, 0)
    q1.q1g128_set_mfma_tuning(0, 0, 0, 0, 0)
    t2.t2g128_set_stream_tuning(0, 0)
    q1.q1g128_set_stream_tuning(0, 0)


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M,N,K", [
    (1, 4096, 2048), (8, 4099, 2048), (9, 1000, 2048), (16, 257, 2048), (5, 33, 2560), (3, 8200, 2560),
    (2, 15, 4096), (16, 700, 3072), (7, 1, 2048), (12, 20000, 2048),
])
def test_forced_stream_kernel(oracle, forced_stream, bits, M, N, K):
    """Ragged row counts, K / 512 that is no multiple of the ring depth (the stream then ends
    inside a trip), fewer row tiles than waves, blocks of up to 16 tokens."""
    check_one(oracle, oracle.synth_problem(1000 + M + N, M, N, K, bits), bits, "forced")


@pytest.mark.parametrize("wgs_per_cu", [1, 2, 3])
def test_forced_stream_kernel_other_residency(oracle, forced_stream, wgs_per_cu):
    forced_stream[0].t2g128_set_stream_tuning(0, wgs_per_cu)
    check_one(oracle, oracle.synth_problem(1100 + wgs_per_cu, 8, 40000, 2048, 2), 2, f"wgs/cu {wgs_per_cu}")


def test_forced_stream_kernel_extreme_bytes(oracle, forced_stream):
    rng = np.random.default_rng(11)
    p = oracle.synth_problem(1200, 6, 600, 2048, 2)
    p["A"] = rng.integers(-128, 128, size=p["A"].shape, dtype=np.int8)
    p["A"][0, :] = -128
    p["B"] = rng.integers(0, 256, size=p["B"].shape, dtype=np.uint8)
    p["B"][0, :] = 0x00
    p["B"][1, :] = 0xFF
    check_one(oracle, p, 2, "extreme")


@pytest.mark.parametrize("M", [1, 4, 9, 16])
def test_head_shape_default_dispatch(oracle, M):
    """The 151936 x 2048 packed lm_head through the ordinary entry point."""
    check_one(oracle, oracle.synth_problem(1300 + M, M, 151936, 2048, 2), 2, "head")


def test_head_shape_4b(oracle):
    check_one(oracle, oracle.synth_problem(1400, 8, 151936, 2560, 2), 2, "head 4B")


def test_stream_kernel_graph_replay(oracle):
    import bitmtp_amd as ops
    ops.init_kernels()
    A, B, s, ws = to_dev(oracle.synth_problem(1500, 8, 151936, 2048, 2))
    eager = ops.packed_gemv_ex(A, B, s, ws, bits=2).clone()
    out = torch.empty_like(eager)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        ops.packed_gemv_ex(A, B, s, ws, bits=2, out=out)
    for rep in range(3):
        out.zero_()
        _ = ops.packed_gemv_ex(A, B, s, ws, bits=2)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs"


# ---- the single-token streaming kernel (activations in registers, v_dot8) -------------------
@pytest.fixture
def forced_rowreg():
    from bitmtp_amd import ops as O2
    t2 = O2.t2_lib()
    t2.t2g128_set_mfma_tuning(0, 0, 0, 0, 6)
    yield t2
    t2.t2g128_set_mfma_tuning(0, 0, 0, 0, 0)
    t2.t2g128_set_stream_tuning(0, 0)


@pytest.mark.parametrize("N,K", [
    (4096, 2048), (4099, 2048), (1, 2048), (7, 2048), (9, 1024), (1000, 1024), (33, 4096),
    (5001, 4096), (40000, 2048), (20003, 1024),
])
def test_forced_single_token_kernel(oracle, forced_rowreg, N, K):
    """8, 16 and 32 lanes per row (K = 1024, 2048, 4096); row counts that end inside a row
    set, inside a batch, and matrices shorter than one batch of one wave."""
    check_one(oracle, oracle.synth_problem(1600 + N, 1, N, K, 2), 2, "single token")


@pytest.mark.parametrize("wgs_per_cu", [1, 2, 6])
def test_forced_single_token_kernel_other_residency(oracle, forced_rowreg, wgs_per_cu):
    forced_rowreg.t2g128_set_stream_tuning(0, wgs_per_cu)
    check_one(oracle, oracle.synth_problem(1700 + wgs_per_cu, 1, 70001, 2048, 2), 2,
              f"single token wgs/cu {wgs_per_cu}")


def test_forced_single_token_kernel_extreme_bytes_and_fp16_scales(oracle, forced_rowreg):
    """Every code value including 0 (-2), activations of -128 in every slot (the planes hold
    hi = -8, lo = 0), fp16 group scales."""
    import bitmtp_amd as ops
    rng = np.random.default_rng(12)
    p = oracle.synth_problem(1800, 1, 600, 2048, 2)
    p["B"] = rng.integers(0, 256, size=p["B"].shape, dtype=np.uint8)
    p["B"][0, :] = 0x00
    p["B"][1, :] = 0xFF
    for fill in (None, -128, 127):
        p["A"] = rng.integers(-128, 128, size=p["A"].shape, dtype=np.int8)
        if fill is not None:
            p["A"][:] = fill
        check_one(oracle, p, 2, f"extreme fill={fill}")
        A, B, s, ws = to_dev(p)
        G = ops.packed_gemv_ex(A, B, None, None, bits=2, out_kind=ops.OUT_G32)  # dot4 kernel: exact sums
        assert np.array_equal(G.cpu().numpy(), oracle.c_group_sums(p["A"], p["B"], 2))
    ws16 = oracle.bf16_bits_to_f32(p["ws"]).astype(np.float16)
    A, B, s, _ = to_dev(p)
    y32 = ops.packed_gemv_ex(A, B, s, torch.from_numpy(ws16).to("cuda:0"), bits=2,
                             out_kind=ops.OUT_F32).cpu().numpy()
    ref, _ = oracle.c_gemv(p["A"], p["B"], p["s"], ws16.view(np.uint16), 2, scale_is_f16=True)
    assert np.all(np.abs(y32 - ref) <= ATOL + RTOL * np.abs(ref))


def test_single_token_kernel_is_exact_for_unit_scales(oracle, forced_rowreg):
    """With every group scale 1 and s = 1 the fp32 result is the integer dot product, exactly
    (|sum| < 2^24): pins the plane arithmetic G = 16 H + L - 2 sum(a) bit for bit."""
    import bitmtp_amd as ops
    rng = np.random.default_rng(13)
    N, K = 3000, 2048
    A = rng.integers(-128, 128, size=(1, K), dtype=np.int8)
    Bp = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    w = oracle.np_unpack(Bp, 2).astype(np.int64)
    want = (w @ A[0].astype(np.int64)).astype(np.float32)
    ws = torch.ones(N, K // 128, dtype=torch.bfloat16, device="cuda:0")
    s = torch.ones(1, 1, dtype=torch.float32, device="cuda:0")
    y = ops.packed_gemv_ex(torch.from_numpy(A).cuda(), torch.from_numpy(Bp.view(np.int8)).cuda(), s, ws,
                           bits=2, out_kind=ops.OUT_F32).cpu().numpy()[0]
    assert np.array_equal(y, want)


def test_single_token_kernel_graph_replay(oracle):
    import bitmtp_amd as ops
    ops.init_kernels()
    A, B, s, ws = to_dev(oracle.synth_problem(1900, 1, 151936, 2048, 2))
    eager = ops.packed_gemv_ex(A, B, s, ws, bits=2).clone()
    out = torch.empty_like(eager)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        ops.packed_gemv_ex(A, B, s, ws, bits=2, out=out)
    for rep in range(3):
        out.zero_()
        _ = ops.packed_gemv_ex(A, B, s, ws, bits=2)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs"


@pytest.mark.parametrize("persistent", [0, 1])
@pytest.mark.parametrize("nbytes, workgroups", [(16, 1), (4096 * 3 + 16, 2), (1 << 20, 64), (13369344, 1280)])
def test_read_probe_runs_and_writes_nothing(nbytes, workgroups, persistent):
    """The measurement aid reads its buffer (including a ragged tail) and leaves the sink and the
    buffer as they were."""
    import ctypes
    from bitmtp_amd import probe
    buf = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda")
    before = buf.clone()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = probe.probe_lib().bonsai_read_probe(buf.data_ptr(), nbytes, workgroups, persistent, sink.data_ptr(), sp)
    assert rc == 0
    torch.cuda.synchronize()
    assert int(sink.item()) == 0 and torch.equal(buf, before)


def test_first_launch_on_a_capturing_stream_is_refused():
    """In a fresh process whose first GEMV launch arrives while the stream is being captured,
    the entry points return status 3 and enqueue nothing (the one-time set-up changes kernel
    attributes, which must not happen under capture); after `t2g128_init` outside capture the
    same call is captured and replays with the eager result."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = r'''
import ctypes, sys, torch
sys.path.insert(0, %r)
from bitmtp_amd import ops
lib = ops.t2_lib()
M, N, K = 4, 256, 2048
g0 = torch.Generator().manual_seed(1)
a = torch.randint(-128, 128, (M, K), generator=g0, dtype=torch.int8).cuda()
b = torch.randint(-128, 128, (N, K // 4), generator=g0, dtype=torch.int8).cuda()
s = torch.full((M, 1), 3.0, dtype=torch.float32).cuda()
ws = torch.full((N, K // 128), 0.02, dtype=torch.bfloat16).cuda()
out = torch.zeros(M, N, dtype=torch.bfloat16).cuda()
def call():
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return lib.t2g128_gemv_ex(a.data_ptr(), b.data_ptr(), out.data_ptr(), s.data_ptr(), ws.data_ptr(),
                              M, N, K, 0, 0, sp)
torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):
    rc_captured = call()
assert rc_captured == 3, rc_captured
graph.replay(); torch.cuda.synchronize()
assert not out.any()                      # nothing was enqueued
assert lib.t2g128_init() == 0
assert call() == 0
torch.cuda.synchronize()
eager = out.clone(); out.zero_()
graph2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph2):
    assert call() == 0
graph2.replay(); torch.cuda.synchronize()
assert eager.any() and torch.equal(out.view(torch.int16), eager.view(torch.int16))
print("REFUSED-THEN-OK")
''' % root
    proc = subprocess.run([sys.executable, "-c", script], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=110)
    assert proc.returncode == 0 and "REFUSED-THEN-OK" in proc.stdout, proc.stderr[-1500:]


def test_first_launches_from_two_threads():
    """Two host threads make the library's first launches at the same moment (ctypes releases
    the interpreter lock during the call): the one-time set-up runs under a lock, both calls
    succeed and both results equal a later single-threaded call."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = r'''
import ctypes, sys, threading, torch
sys.path.insert(0, %r)
from bitmtp_amd import ops
lib = ops.t2_lib()
M, N, K = 9, 512, 2048
g0 = torch.Generator().manual_seed(2)
a = torch.randint(-128, 128, (M, K), generator=g0, dtype=torch.int8).cuda()
b = torch.randint(-128, 128, (N, K // 4), generator=g0, dtype=torch.int8).cuda()
s = torch.full((M, 1), 5.0, dtype=torch.float32).cuda()
ws = torch.full((N, K // 128), 0.03, dtype=torch.bfloat16).cuda()
outs = [torch.zeros(M, N, dtype=torch.bfloat16).cuda() for _ in range(3)]
streams = [torch.cuda.Stream(), torch.cuda.Stream()]
torch.cuda.synchronize()
rcs = [None, None]
barrier = threading.Barrier(2)
def work(i):
    barrier.wait()
    rcs[i] = lib.t2g128_gemv_ex(a.data_ptr(), b.data_ptr(), outs[i].data_ptr(), s.data_ptr(), ws.data_ptr(),
                                M, N, K, 0, 0, ctypes.c_void_p(streams[i].cuda_stream))
ts = [threading.Thread(target=work, args=(i,)) for i in range(2)]
[t.start() for t in ts]; [t.join() for t in ts]
torch.cuda.synchronize()
assert rcs == [0, 0], rcs
sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
assert lib.t2g128_gemv_ex(a.data_ptr(), b.data_ptr(), outs[2].data_ptr(), s.data_ptr(), ws.data_ptr(), M, N, K, 0, 0, sp) == 0
torch.cuda.synchronize()
assert outs[2].any()
assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))
assert torch.equal(outs[1].view(torch.int16), outs[2].view(torch.int16))
print("TWO-THREADS-OK")
''' % root
    proc = subprocess.run([sys.executable, "-c", script], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=110)
    assert proc.returncode == 0 and "TWO-THREADS-OK" in proc.stdout, proc.stderr[-1500:]
