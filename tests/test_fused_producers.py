"""Fused producers of the GEMV input: RMSNorm(+residual)+quant and SiLU*up+quant.

CPU: the C oracle against the same expressions evaluated by this build's own PyTorch
(the library routine; they are the reference's eager statements,
src/bonsai_sft/gpu/model.py:307-336 and :1058-1061) and against hand-derived cases.
GPU: the HIP kernels against the oracle, bit for bit (the sum of squares uses one
fixed fp64 order in both).
"""
import numpy as np
import pytest
import torch


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def torch_norm_quant(x, w, eps):
    h = x.float()
    var = h.pow(2).mean(-1, keepdim=True)
    h = h * torch.rsqrt(var + eps)
    nf = (w * h.to(x.dtype)).float()
    s = 127.0 / nf.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
    return (nf * s).round().clamp(-128, 127).to(torch.int8), s


def torch_silu_quant(gu):
    f = gu.shape[-1] // 2
    g, u = gu.split([f, f], dim=-1)
    xf = (torch.nn.functional.silu(g) * u).float()
    s = 127.0 / xf.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
    return (xf * s).round().clamp(-128, 127).to(torch.int8), s


def make_inputs(seed, M, K):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(M, K, generator=g) * 1.7).to(torch.bfloat16)
    r = (torch.randn(M, K, generator=g) * 0.8).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16)
    return x, r, w


@pytest.mark.parametrize("M,K", [(1, 128), (4, 2048), (9, 2560), (3, 6144), (2, 9728)])
def test_oracle_norm_quant_matches_torch(oracle, M, K):
    x, r, w = make_inputs(K + M, M, K)
    eps = 1e-6
    q, s, _ = oracle.c_rmsnorm_quant(bits(x), bits(w), eps)
    qt, st = torch_norm_quant(x, w, eps)
    assert np.array_equal(s, st.numpy().reshape(-1)) and np.array_equal(q, qt.numpy())
    q, s, h = oracle.c_rmsnorm_quant(bits(x), bits(w), eps, bits(r))
    hh = x + r
    qt, st = torch_norm_quant(hh, w, eps)
    assert np.array_equal(h, bits(hh))
    assert np.array_equal(s, st.numpy().reshape(-1)) and np.array_equal(q, qt.numpy())


@pytest.mark.parametrize("M,K", [(1, 128), (3, 2048), (9, 2560)])
def test_oracle_norm_without_quant_matches_torch(oracle, M, K):
    """The norm-only form is RMSNorm.forward (model.py:290-295) on x or on x + residual."""
    x, r, w = make_inputs(7 * K + M, M, K)
    eps = 1e-6

    def torch_norm(h):
        hf = h.float()
        return w * (hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + eps)).to(h.dtype)
    n, h = oracle.c_rmsnorm(bits(x), bits(w), eps)
    assert h is None and np.array_equal(n, bits(torch_norm(x)))
    n, h = oracle.c_rmsnorm(bits(x), bits(w), eps, bits(r))
    assert np.array_equal(h, bits(x + r)) and np.array_equal(n, bits(torch_norm(x + r)))
    # known answer: x = 2, w = 0.5, eps = 0 -> rms 2, normed 0.5 everywhere
    n, _ = oracle.c_rmsnorm(bits(torch.full((1, 256), 2.0, dtype=torch.bfloat16)),
                            bits(torch.full((256,), 0.5, dtype=torch.bfloat16)), 0.0)
    assert np.all(n == 0x3F00)


def test_oracle_norm_quant_known_answer(oracle):
    """x = 2 everywhere, w = 0.5, eps = 0: rms = 2, normed = 0.5, s = 254, q = 127."""
    x = torch.full((1, 256), 2.0, dtype=torch.bfloat16)
    w = torch.full((256,), 0.5, dtype=torch.bfloat16)
    q, s, _ = oracle.c_rmsnorm_quant(bits(x), bits(w), 0.0)
    assert s[0] == 254.0 and np.all(q == 127)
    # alternating sign, one element doubled: that element alone reaches 127
    x[0, ::2] = -2.0
    q, s, _ = oracle.c_rmsnorm_quant(bits(x), bits(w), 0.0)
    assert set(q[0].tolist()) == {-127, 127}


@pytest.mark.parametrize("M,F", [(1, 128), (5, 6144), (2, 9728)])
def test_oracle_silu_mul_quant_matches_torch(oracle, M, F):
    g = torch.Generator().manual_seed(F + M)
    gu = (torch.randn(M, 2 * F, generator=g) * 2).to(torch.bfloat16)
    q, s = oracle.c_silu_mul_quant(bits(gu))
    qt, st = torch_silu_quant(gu)
    assert np.array_equal(s, st.numpy().reshape(-1)) and np.array_equal(q, qt.numpy())


def test_oracle_silu_known_answer(oracle):
    """gate = 0 -> silu = 0 -> everything quantises to 0 with the clamped scale."""
    gu = torch.zeros(1, 256, dtype=torch.bfloat16)
    gu[0, 128:] = 3.0
    q, s = oracle.c_silu_mul_quant(bits(gu))
    assert np.all(q == 0) and s[0] == (np.float32(1.0) / np.float32(1e-5)) * np.float32(127.0)


def test_merge_packed_rows():
    import bitmtp_amd
    parts = [(torch.full((n, 64), i, dtype=torch.int8), torch.full((n, 2), float(i), dtype=torch.bfloat16))
             for i, n in enumerate((4, 2, 2))]
    packed, scales, split = bitmtp_amd.merge_packed_rows(parts)
    assert packed.shape == (8, 64) and scales.shape == (8, 2) and split == [4, 2, 2]
    assert packed[:4].eq(0).all() and packed[4:6].eq(1).all() and scales[6:].eq(2).all()
    with pytest.raises(ValueError, match="share K"):
        bitmtp_amd.merge_packed_rows([parts[0], (torch.zeros(2, 32, dtype=torch.int8), parts[1][1])])


# ---------------------------------------------------------------------------- GPU
@pytest.mark.gpu
@pytest.mark.parametrize("M,K", [(1, 128), (1, 2048), (8, 2048), (17, 2560), (4, 6144), (9, 9728)])
def test_hip_norm_quant_bit_exact(oracle, M, K):
    import bitmtp_amd as ops
    x, r, w = make_inputs(K * 3 + M, M, K)
    eps = 1e-6
    dev = "cuda:0"
    print(f"[case] fused_norm_quant M={M} K={K}", flush=True)
    q, s = ops.fused_norm_quant(x.to(dev), w.to(dev), eps)
    q_ref, s_ref, _ = oracle.c_rmsnorm_quant(bits(x), bits(w), eps)
    assert s.shape == (M, 1)
    assert np.array_equal(s.cpu().numpy().reshape(-1), s_ref) and np.array_equal(q.cpu().numpy(), q_ref)
    h, q, s = ops.fused_add_norm_quant(x.to(dev), r.to(dev), w.to(dev), eps)
    q_ref, s_ref, h_ref = oracle.c_rmsnorm_quant(bits(x), bits(w), eps, bits(r))
    assert np.array_equal(bits(h.cpu()), h_ref)
    assert np.array_equal(s.cpu().numpy().reshape(-1), s_ref) and np.array_equal(q.cpu().numpy(), q_ref)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K", [(1, 128), (1, 2048), (9, 2048), (17, 2560), (2, 9728)])
def test_hip_norm_without_quant_bit_exact(oracle, M, K):
    import bitmtp_amd as ops
    x, r, w = make_inputs(K * 5 + M, M, K)
    eps = 1e-6
    dev = "cuda:0"
    print(f"[case] add_rmsnorm M={M} K={K}", flush=True)
    n = ops.add_rmsnorm(x.to(dev), None, w.to(dev), eps)
    n_ref, _ = oracle.c_rmsnorm(bits(x), bits(w), eps)
    assert n.shape == x.shape and np.array_equal(bits(n.cpu()), n_ref)
    n = ops.add_rmsnorm(x.to(dev), r.to(dev), w.to(dev), eps)
    n_ref, _ = oracle.c_rmsnorm(bits(x), bits(w), eps, bits(r))
    assert np.array_equal(bits(n.cpu()), n_ref)
    with pytest.raises(RuntimeError):
        ops.add_rmsnorm(x.to(dev), r[:, :-8].contiguous().to(dev), w.to(dev), eps)


@pytest.mark.gpu
@pytest.mark.parametrize("M,F", [(1, 128), (1, 6144), (8, 6144), (16, 9728)])
def test_hip_silu_mul_quant(oracle, M, F):
    """expf on the GPU and in libm may differ in the last place, which can move a value
    across a bf16 rounding boundary: q may differ by one in a handful of positions, and s
    by one fp32 ulp only if that happens to the row's largest element."""
    import bitmtp_amd as ops
    g = torch.Generator().manual_seed(F * 5 + M)
    gu = (torch.randn(M, 2 * F, generator=g) * 2).to(torch.bfloat16)
    print(f"[case] silu_mul_quant M={M} F={F}", flush=True)
    q, s = ops.silu_mul_quant(gu.to("cuda:0"))
    q_ref, s_ref = oracle.c_silu_mul_quant(bits(gu))
    got_s = s.cpu().numpy().reshape(-1)
    assert np.all(np.abs(got_s - s_ref) <= np.abs(s_ref) * 1e-2)
    same_scale = got_s == s_ref
    dq = np.abs(q.cpu().numpy().astype(int) - q_ref.astype(int))
    assert dq.max() <= 1
    assert (dq[same_scale] != 0).mean() <= 1e-3 if same_scale.any() else True
