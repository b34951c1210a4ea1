"""Guard on the dispatcher's measured thresholds (which kernel a shape gets: the dot4 kernel up to
two tokens, the lean matrix-core kernel from three, from two for long rows and very long matrices,
the streaming kernels for the head).  The constants came from sweeps on two model shapes; this
test re-times the built-in choice against each kernel forced through the development hooks on a
handful of shapes around the thresholds and fails when the built-in choice is grossly wrong (more
than 1.5 x the best alternative) -- wide enough for box-to-box noise, narrow enough to catch a
threshold that sends a shape to the wrong family (the dot4 kernel at eight tokens is 2.3 x the
matrix-core kernel).  Collected late on purpose: it is the only timing assertion in the suite.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

# (M, N, K, forced alternatives): kernels of bitmtp_amd.gemv_bench.KERNELS that can run the shape
CASES = [
    (1, 12288, 2048, ("dot4", "lean")),
    (2, 2048, 6144, ("dot4", "lean")),
    (3, 4096, 2048, ("dot4", "lean", "operand")),
    (8, 12288, 2048, ("dot4", "lean", "operand", "staged")),
    (8, 2560, 9728, ("lean", "operand")),
    (1, 151936, 2048, ("dot4", "single-token", "stream")),
    (8, 151936, 2048, ("stream", "staged")),
]


def _time_us(fn_ptr, tensors, m, n, k, count):
    """Best of 3 replays of a graph of `count` launches over distinct matrices, per launch."""
    q, s, out, mats = tensors
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for packed, scales in mats[:2]:
        fn_ptr(q.data_ptr(), packed.data_ptr(), out.data_ptr(), s.data_ptr(), scales.data_ptr(), m, n, k, sp)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        spc = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for packed, scales in mats:
            fn_ptr(q.data_ptr(), packed.data_ptr(), out.data_ptr(), s.data_ptr(), scales.data_ptr(), m, n, k, spc)
    g.replay()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / count)
    return best


@pytest.mark.parametrize("M,N,K,alternatives", CASES)
def test_built_in_choice_is_not_grossly_wrong(M, N, K, alternatives):
    import bitmtp_amd as ops
    from bitmtp_amd import gemv_bench, ops as ops_mod
    dev = torch.device("cuda:0")
    ops.init_kernels()
    lib = ops_mod.t2_lib()
    fn = lib.t2g128_int8xint2_linear
    gen = torch.Generator(device=dev)
    gen.manual_seed(M + N + K)
    nbytes = gemv_bench.gemv_bytes("t2", N, K)
    count = max(4, min(96, (320 << 20) // nbytes + 1))   # beyond the Infinity Cache
    mats = []
    for _ in range(count):
        packed = torch.randint(-128, 128, (N, K // 4), generator=gen, device=dev, dtype=torch.int8)
        scales = torch.exp(torch.randn(N, K // 128, generator=gen, device=dev) * 0.5 - 4.0).to(torch.bfloat16)
        mats.append((packed, scales))
    q, s = ops.quant_input(torch.randn(M, K, generator=gen, device=dev).to(torch.float16))
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    tensors = (q, s, out, mats)
    times = {}
    try:
        for kern in ("auto",) + tuple(alternatives):
            min_width, engine = gemv_bench.KERNELS[kern]
            lib.t2g128_set_mfma_tuning(min_width, 0, 0, 0, engine)
            times[kern] = _time_us(fn, tensors, M, N, K, count)
            times[kern + ":kernel"] = ops.last_kernel(2)
    finally:
        lib.t2g128_set_mfma_tuning(0, 0, 0, 0, 0)
    print(f"[case] dispatch guard M={M} N={N} K={K}: {times}", flush=True)
    best_alt = min(times[k] for k in alternatives)
    assert times["auto"] <= 1.5 * best_alt, times
