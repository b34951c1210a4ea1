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
