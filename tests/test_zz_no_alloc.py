"""GPU test of the allocation-free entry point `bonsai_draft_chain_static`: called through the
C ABI, its outputs must equal those of `bonsai_draft_chain_ws` (same kernels, caller-supplied
workspace) exactly -- tokens and accepted length as integers, confidences bit for bit -- on two
calls in a row, the second on a smaller input, so that contents the library's own scratch
array keeps from the first call cannot leak into the second.  Sizes beyond the array are
refused.  The file is named so that it is collected after every other test.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _logits(rng, rows, vocab, ld):
    x = torch.from_numpy(rng.normal(0, 2.0, (rows, ld)).astype(np.float32)).to(torch.bfloat16)
    for r in range(1, rows, 2):
        x[r, (r * 7919) % vocab] = 30.0       # confident rows
    x[:, vocab:] = 100.0                       # padding columns must not be read
    return x.to(DEV)


def _run(lib, name, logits, rows, ld, vocab, thr, scratch=None):
    tokens = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    conf = torch.full((rows,), float("nan"), dtype=torch.float32, device=DEV)
    accept = torch.full((2,), -7, dtype=torch.int32, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [_ptr(logits), rows, ld, vocab, ctypes.c_float(thr), _ptr(tokens), _ptr(conf), _ptr(accept)]
    if scratch is not None:
        args.append(_ptr(scratch))
    rc = getattr(lib, name)(*args, stream)
    torch.cuda.synchronize()
    return rc, tokens.cpu().numpy(), conf.cpu().numpy(), accept.cpu().numpy()


def test_static_scratch_draft_chain_matches_workspace_form():
    from bitmtp_amd import decode_ops
    lib = decode_ops.decode_lib()
    rng = np.random.default_rng(11)
    # first a wide call on the full vocabulary, then a narrower, shorter one
    for rows, vocab, ld in ((17, 151669, 151936), (5, 1000, 1024)):
        print(f"[case] draft_chain_static rows={rows} vocab={vocab}", flush=True)
        logits = _logits(rng, rows, vocab, ld)
        nbytes = int(lib.bonsai_draft_chain_scratch_bytes(rows))
        ws = torch.full((nbytes // 4,), float("nan"), device=DEV)
        rc0, t0, c0, a0 = _run(lib, "bonsai_draft_chain_ws", logits, rows, ld, vocab, 0.9, ws)
        rc1, t1, c1, a1 = _run(lib, "bonsai_draft_chain_static", logits, rows, ld, vocab, 0.9)
        assert rc0 == 0 and rc1 == 0
        assert np.array_equal(t0, t1) and np.array_equal(a0, a1)
        assert np.array_equal(c0.view(np.uint32), c1.view(np.uint32))
        assert a1[1] == rows and 1 <= a1[0] <= rows and (t1 >= 0).all() and (t1 < vocab).all()


def test_static_scratch_draft_chain_refuses_oversize():
    from bitmtp_amd import decode_ops
    lib = decode_ops.decode_lib()
    rows, vocab, ld = 33, 64, 64          # one row more than the array holds
    logits = torch.zeros(rows, ld, dtype=torch.bfloat16, device=DEV)
    rc, tokens, _, accept = _run(lib, "bonsai_draft_chain_static", logits, rows, ld, vocab, 0.9)
    assert rc == 1
    assert (tokens == -7).all() and (accept == -7).all()   # nothing was launched


def test_static_scratch_draft_chain_first_call_under_capture_is_refused_then_captured():
    """In a fresh process the first call arrives on a capturing stream: status 3, nothing
    launched, the capture stays valid.  After bonsai_decode_init the same call is captured, and
    every replay (with eager work and synchronisations in between) gives the workspace form's
    result while the device's free memory does not move: the entry point allocates nothing."""
    import subprocess
    import sys
    import textwrap
    code = textwrap.dedent("""
        import ctypes, numpy as np, torch
        from bitmtp_amd import decode_ops
        lib = decode_ops.decode_lib()
        lib.bonsai_decode_init.restype = ctypes.c_int
        dev = "cuda:0"
        rows, vocab, ld = 9, 5000, 5120
        rng = np.random.default_rng(3)
        def P(t): return ctypes.c_void_p(t.data_ptr())
        logits = torch.from_numpy(rng.normal(0, 2, (rows, ld)).astype(np.float32)).to(torch.bfloat16).to(dev)
        tokens = torch.zeros(rows, dtype=torch.int32, device=dev)
        conf = torch.zeros(rows, dtype=torch.float32, device=dev)
        accept = torch.zeros(2, dtype=torch.int32, device=dev)
        ws = torch.zeros(int(lib.bonsai_draft_chain_scratch_bytes(rows)) // 4, device=dev)
        t0 = torch.zeros_like(tokens); c0 = torch.zeros_like(conf); a0 = torch.zeros_like(accept)
        def static_call():
            sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            return lib.bonsai_draft_chain_static(P(logits), rows, ld, vocab, ctypes.c_float(0.9), P(tokens), P(conf), P(accept), sp)
        def ws_call():
            sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            return lib.bonsai_draft_chain_ws(P(logits), rows, ld, vocab, ctypes.c_float(0.9), P(t0), P(c0), P(a0), P(ws), sp)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            rc_first = static_call()
        assert rc_first == 3, rc_first
        assert lib.bonsai_decode_init() == 0
        g2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g2):
            rc = static_call()
        assert rc == 0, rc
        for rep in range(4):
            logits.copy_(torch.from_numpy(rng.normal(0, 2, (rows, ld)).astype(np.float32)).to(torch.bfloat16))
            assert ws_call() == 0
            torch.cuda.synchronize()
            tokens.fill_(-1); conf.fill_(-1); accept.fill_(-1)
            g2.replay()
            torch.cuda.synchronize()
            assert torch.equal(tokens, t0) and torch.equal(accept, a0), rep
            assert torch.equal(conf.view(torch.int32), c0.view(torch.int32)), rep
        free_before = torch.cuda.mem_get_info()[0]
        for _ in range(3):
            assert static_call() == 0
        g2.replay()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, (torch.cuda.mem_get_info()[0], free_before)
        print("ok")
    """)
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=170)
    assert proc.returncode == 0 and "ok" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-2000:]
