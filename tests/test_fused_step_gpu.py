"""Decode steps of one or two tokens with the element-wise producers folded into the projections
(``*_gemv_fused``), against the separate launches they stand for, through the C ABI:

* MLP tail: gate|up projection with ``inner = silu(gate) * up`` in its epilogue + down projection
  that quantises ``inner`` while staging, against projection, ``bonsai_silu_mul_quant_int8``
  (src/bonsai_sft/gpu/model.py:1058-1061), projection;
* residual add + RMSNorm + quantisation (model.py:322-336): a projection that stores
  ``h = residual + y`` and parts of ``sum h^2`` + a projection that normalises and quantises ``h``
  while staging, against projection, ``bonsai_add_rmsnorm_quant_int8``, projection;
* a whole layer chained the fused way against the ten-launch way.

In each case the intermediate rows, the multipliers the consuming launch derives and the fp32 and
bf16 results are the SAME BITS as the separate launches give (these are forced onto the dot4
kernels, whose arithmetic the fused forms share).  The parts arrays are checked on their own
(all written, pad zero, maxima / sums of what was stored), the pieces are anchored on the CPU
oracle directly, and the decode loop produces the same tokens with and without the fused layers.
"""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
EPS = 1e-6

# (dim, ffn): the 1.7B- and 4B-shaped MLPs, the tiny test model, odd chunk counts
SHAPES = [(2048, 6144), (2560, 9728), (512, 1024), (384, 1408), (128, 128)]


@pytest.fixture
def dot4_only():
    """Keeps two-token projections of the separate-launch path on the dot4 kernels (the built-in
    choice sends K >= 4096 to the matrix cores, whose fp32 summation order differs)."""
    from bitmtp_amd import ops
    ops.init_kernels()
    ops.t2_lib().t2g128_set_mfma_tuning(3, 0, 0, 0, 0)
    ops.q1_lib().q1g128_set_mfma_tuning(3, 0, 0, 0, 0)
    yield
    ops.t2_lib().t2g128_set_mfma_tuning(0, 0, 0, 0, 0)
    ops.q1_lib().q1g128_set_mfma_tuning(0, 0, 0, 0, 0)


def _gen(seed):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    return g


def _packed(gen, n, k, bits, scale_mul=1.0):
    from bitmtp_amd import model as mdl
    p = mdl._random_packed(n, k, gen, DEV, bits)
    if scale_mul != 1.0:
        p.weight_scale.mul_(scale_mul)   # a power of two: exact in bf16
    return p


def _rows(gen, m, k, std=1.0):
    return (torch.randn(m, k, generator=gen, device=DEV) * std).to(torch.bfloat16)


def _same_bits(a, b):
    view = {torch.float32: torch.int32, torch.bfloat16: torch.int16}[a.dtype]
    return a.dtype == b.dtype and torch.equal(a.view(view), b.view(view))


@pytest.mark.parametrize("dim,ffn", SHAPES)
@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("bits", [2, 1])
def test_mlp_tail_two_launches_give_the_bits_of_three(dot4_only, bits, M, dim, ffn):
    from bitmtp_amd import ops
    print(f"[case] fused MLP tail bits={bits} M={M} dim={dim} ffn={ffn}", flush=True)
    gen = _gen(1000 * bits + 10 * M + dim)
    # (scales large enough for the gate to leave the linear part of the sigmoid)
    w_gu, w_dn = _packed(gen, 2 * ffn, dim, bits, 8.0), _packed(gen, dim, ffn, bits)
    x_q, x_s = ops.quant_input(_rows(gen, M, dim))

    gu = ops.packed_gemv_ex(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=bits)
    assert ops.last_kernel(bits).startswith("gemv_dot4_kernel")
    i_q, i_s = ops.silu_mul_quant(gu)
    want = {k: ops.packed_gemv_ex(i_q, w_dn.weight, i_s, w_dn.weight_scale, bits=bits, out_kind=k)
            for k in (ops.OUT_F32, ops.OUT_BF16)}
    assert ops.last_kernel(bits).startswith("gemv_dot4_kernel")

    poison = torch.full((M * 1024,), 7e9, dtype=torch.bfloat16, device=DEV)
    inner, amax, parts = ops.packed_gemv_fused(x_q, w_gu.weight, w_gu.weight_scale, bits=bits, s=x_s,
                                               epi=ops.EPI_SILU_PAIR, out_aux=poison)
    assert ops.last_kernel(bits).startswith("gemv_dot4_fused_kernel")
    assert 0 < parts <= 1024 and parts == ops.fused_parts(ops.EPI_SILU_PAIR, M, 2 * ffn, dim, bits=bits)
    q2, s2 = ops.quant_input(inner)
    assert torch.equal(q2, i_q) and torch.equal(s2.reshape(-1), i_s.reshape(-1))

    ld = (parts + 7) // 8 * 8
    am = amax[: M * ld].view(M, ld).float()
    assert torch.all(am[:, parts:] == 0) and torch.all(am >= 0)
    assert torch.equal(am.max(dim=1).values, inner.float().abs().max(dim=1).values)

    for kind, ref in want.items():
        s_out = torch.empty(M, dtype=torch.float32, device=DEV)
        got, _, _ = ops.packed_gemv_fused(inner, w_dn.weight, w_dn.weight_scale, bits=bits, amax=amax,
                                          parts=parts, out_kind=kind, s_out=s_out)
        assert ops.last_kernel(bits).startswith("gemv_dot4_fused_kernel")
        assert torch.equal(s_out, i_s.reshape(-1))
        assert _same_bits(got, ref), f"out_kind {kind}"


# (5120 and 8192 columns at two tokens: more quarters than a workgroup has threads, so the staging
# loops past each thread's first quarter run too)
@pytest.mark.parametrize("n_prod,k_prod,n_cons", [(2048, 2048, 4096), (2048, 6144, 12288), (2560, 9728, 6144),
                                                  (512, 512, 1024), (384, 1408, 256), (128, 128, 128),
                                                  (5120, 1024, 640), (8192, 512, 20480)])
@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("bits", [2, 1])
def test_add_norm_quant_rides_in_the_projections(dot4_only, bits, M, n_prod, k_prod, n_cons):
    """Producer (o or down projection, K = k_prod) -> residual stream of n_prod columns -> consumer
    (q|k|v or gate|up projection with n_cons rows)."""
    from bitmtp_amd import ops
    print(f"[case] fused add+norm+quant bits={bits} M={M} producer {n_prod}x{k_prod} consumer rows {n_cons}",
          flush=True)
    gen = _gen(7 * bits + M + n_prod + k_prod)
    w_p, w_c = _packed(gen, n_prod, k_prod, bits, 4.0), _packed(gen, n_cons, n_prod, bits)
    norm_w = (1.0 + 0.1 * torch.randn(n_prod, generator=gen, device=DEV)).to(torch.bfloat16)
    h = _rows(gen, M, n_prod)
    x_q, x_s = ops.quant_input(_rows(gen, M, k_prod))

    y = ops.packed_gemv_ex(x_q, w_p.weight, x_s, w_p.weight_scale, bits=bits)
    assert ops.last_kernel(bits).startswith("gemv_dot4_kernel")
    h_ref, q_ref, s_ref = ops.fused_add_norm_quant(y, h, norm_w, EPS)
    want = {k: ops.packed_gemv_ex(q_ref, w_c.weight, s_ref, w_c.weight_scale, bits=bits, out_kind=k)
            for k in (ops.OUT_F32, ops.OUT_BF16)}

    poison = torch.full((M * 256,), float("nan"), dtype=torch.float64, device=DEV)
    h_new, sumsq, parts = ops.packed_gemv_fused(x_q, w_p.weight, w_p.weight_scale, bits=bits, s=x_s,
                                                epi=ops.EPI_ADD_SUMSQ, residual=h, out_aux=poison)
    assert ops.last_kernel(bits).startswith("gemv_dot4_fused_kernel")
    assert 0 < parts <= 256 and parts == ops.fused_parts(ops.EPI_ADD_SUMSQ, M, n_prod, k_prod, bits=bits)
    assert _same_bits(h_new, h_ref)
    # the parts add up to the sum of the squares stored (squares of bf16 values are exact in fp32)
    total = sumsq[: M * parts].view(M, parts).sum(dim=1)
    exact = (h_new.float() ** 2).double().sum(dim=1)
    assert torch.all(torch.isfinite(total)) and torch.all((total - exact).abs() <= 1e-12 * exact)
    assert torch.all(torch.isnan(sumsq[M * parts:]))      # nothing written past the parts

    for kind, ref in want.items():
        s_out = torch.empty(M, dtype=torch.float32, device=DEV)
        got, _, _ = ops.packed_gemv_fused(h_new, w_c.weight, w_c.weight_scale, bits=bits, sumsq=sumsq,
                                          parts=parts, norm_weight=norm_w, eps=EPS, out_kind=kind, s_out=s_out)
        assert ops.last_kernel(bits).startswith("gemv_dot4_fused_kernel")
        assert torch.equal(s_out, s_ref.reshape(-1))
        assert _same_bits(got, ref), f"out_kind {kind}"


@pytest.mark.parametrize("bits,M,dim,q_dim,ffn", [(2, 1, 2048, 2048, 6144), (2, 2, 2560, 4096, 9728),
                                                  (1, 1, 512, 512, 1024), (1, 2, 384, 256, 1408)])
def test_a_layer_chained_the_fused_way(dot4_only, bits, M, dim, q_dim, ffn):
    """o -> (add, norm) -> gate|up -> (SiLU * up) -> down -> (add, norm) -> next q|k|v: the four
    fused launches in a row, every stage feeding on the previous one's rows and parts, against the
    seven separate launches."""
    from bitmtp_amd import ops
    print(f"[case] fused layer chain bits={bits} M={M} dim={dim} q_dim={q_dim} ffn={ffn}", flush=True)
    gen = _gen(31 * bits + M + dim)
    w_o, w_gu = _packed(gen, dim, q_dim, bits, 4.0), _packed(gen, 2 * ffn, dim, bits, 8.0)
    w_dn, w_qkv = _packed(gen, dim, ffn, bits, 4.0), _packed(gen, q_dim + 512, dim, bits)
    n1 = (1.0 + 0.1 * torch.randn(dim, generator=gen, device=DEV)).to(torch.bfloat16)
    n2 = (1.0 + 0.1 * torch.randn(dim, generator=gen, device=DEV)).to(torch.bfloat16)
    h0 = _rows(gen, M, dim)
    o_q, o_s = ops.quant_input(_rows(gen, M, q_dim))

    def ex(q, s, w):
        return ops.packed_gemv_ex(q, w.weight, s, w.weight_scale, bits=bits)
    attn = ex(o_q, o_s, w_o)
    h1, f_q, f_s = ops.fused_add_norm_quant(attn, h0, n1, EPS)
    i_q, i_s = ops.silu_mul_quant(ex(f_q, f_s, w_gu))
    h2, a_q, a_s = ops.fused_add_norm_quant(ex(i_q, i_s, w_dn), h1, n2, EPS)
    want = ex(a_q, a_s, w_qkv)

    def fused(act, w, **kw):
        return ops.packed_gemv_fused(act, w.weight, w.weight_scale, bits=bits, **kw)
    g1, ss, p_o = fused(o_q, w_o, s=o_s, epi=ops.EPI_ADD_SUMSQ, residual=h0)
    inner, am, p_gu = fused(g1, w_gu, sumsq=ss, parts=p_o, norm_weight=n1, eps=EPS, epi=ops.EPI_SILU_PAIR)
    g2, ss2, p_dn = fused(inner, w_dn, amax=am, parts=p_gu, epi=ops.EPI_ADD_SUMSQ, residual=g1)
    got, _, _ = fused(g2, w_qkv, sumsq=ss2, parts=p_dn, norm_weight=n2, eps=EPS)
    assert _same_bits(g1, h1) and _same_bits(g2, h2) and _same_bits(got, want)


@pytest.mark.parametrize("bits,M,dim,ffn", [(2, 1, 2048, 6144), (2, 2, 512, 1024), (1, 2, 2560, 9728),
                                            (1, 1, 384, 1408)])
def test_fused_forms_against_the_oracle(bits, M, dim, ffn):
    from oracle import oracle as O
    from bitmtp_amd import ops
    O.build()
    print(f"[case] fused forms vs oracle bits={bits} M={M} dim={dim} ffn={ffn}", flush=True)
    gen = _gen(77 + bits + M + ffn)
    w_gu, w_dn = _packed(gen, 2 * ffn, dim, bits, 8.0), _packed(gen, dim, ffn, bits, 4.0)
    x_q, x_s = ops.quant_input(_rows(gen, M, dim))
    h = _rows(gen, M, dim)

    def host(p):
        return p.weight.cpu().numpy().view(np.uint8), bf16_bits(p.weight_scale)

    inner, amax, parts = ops.packed_gemv_fused(x_q, w_gu.weight, w_gu.weight_scale, bits=bits, s=x_s,
                                               epi=ops.EPI_SILU_PAIR)
    s_out = torch.empty(M, dtype=torch.float32, device=DEV)
    h_new, sumsq, p2 = ops.packed_gemv_fused(inner, w_dn.weight, w_dn.weight_scale, bits=bits, amax=amax,
                                             parts=parts, s_out=s_out, epi=ops.EPI_ADD_SUMSQ, residual=h)

    # first launch: the oracle's projection, then the oracle's SiLU * up + quantisation
    _, gu_ref = O.c_gemv(x_q.cpu().numpy(), host(w_gu)[0], x_s.cpu().numpy().reshape(-1), host(w_gu)[1], bits)
    q_ref, s_ref = O.c_silu_mul_quant(gu_ref)
    q_gpu, s_gpu = ops.quant_input(inner)
    s_gpu = s_gpu.cpu().numpy().reshape(-1)
    assert np.array_equal(s_gpu, s_out.cpu().numpy())
    # (a projection value one bf16 step from the oracle's, or a sigmoid on the other side of a
    # rounding boundary, moves a product by a step; the multiplier moves with the row maximum)
    assert np.all(np.abs(s_gpu - s_ref) <= 2e-2 * np.abs(s_ref))
    dq = np.abs(q_gpu.cpu().numpy().astype(np.int32) - q_ref.astype(np.int32))
    assert dq.max() <= 2
    same = s_gpu == s_ref
    assert not same.any() or (dq[same].max() <= 1 and (dq[same] != 0).mean() <= 0.05), \
        (dq[same].max(), (dq[same] != 0).mean())

    # second launch: the oracle's GEMV on the GPU's own quantised input, then the residual add
    y32, _ = O.c_gemv(q_gpu.cpu().numpy(), host(w_dn)[0], s_gpu, host(w_dn)[1], bits)
    yb = O.bf16_bits_to_f32(O.f32_to_bf16_bits(y32))
    want_h = O.f32_to_bf16_bits((yb + O.bf16_bits_to_f32(bf16_bits(h))).astype(np.float32))
    d = np.abs(bf16_ordinal(bf16_bits(h_new)) - bf16_ordinal(want_h))
    assert d.max() <= 1 and (d != 0).mean() <= 0.02, (d.max(), (d != 0).mean())

    # third: the oracle's RMSNorm + quantisation of the GPU's own stream against the norm prologue
    norm_w = (1.0 + 0.1 * torch.randn(dim, generator=gen, device=DEV)).to(torch.bfloat16)
    w_c = _packed(gen, 256, dim, bits)
    s3 = torch.empty(M, dtype=torch.float32, device=DEV)
    out, _, _ = ops.packed_gemv_fused(h_new, w_c.weight, w_c.weight_scale, bits=bits, sumsq=sumsq, parts=p2,
                                      norm_weight=norm_w, eps=EPS, s_out=s3)
    nq, ns, _ = O.c_rmsnorm_quant(bf16_bits(h_new), bf16_bits(norm_w), EPS)
    assert np.array_equal(ns, s3.cpu().numpy())
    _, ref = O.c_gemv(nq, host(w_c)[0], ns, host(w_c)[1], bits)
    d = np.abs(bf16_ordinal(bf16_bits(out)) - bf16_ordinal(ref))
    assert d.max() <= 1, f"normalising projection: {d.max()} bf16 steps from the oracle"


def test_zero_and_large_rows(dot4_only):
    """A token whose products are all zero takes the clamped multiplier fl(fl(1 / 1e-5) * 127);
    a token with large values and a small one side by side keep their own multipliers."""
    from bitmtp_amd import ops
    dim, ffn, bits, M = 512, 1024, 2, 2
    print("[case] fused MLP tail: zero row, large row", flush=True)
    gen = _gen(5)
    w_gu, w_dn = _packed(gen, 2 * ffn, dim, bits, 8.0), _packed(gen, dim, ffn, bits)
    x_q, x_s = ops.quant_input(_rows(gen, M, dim, 30.0))
    x_q[0].zero_()
    gu = ops.packed_gemv_ex(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=bits)
    i_q, i_s = ops.silu_mul_quant(gu)
    ref = ops.packed_gemv_ex(i_q, w_dn.weight, i_s, w_dn.weight_scale, bits=bits, out_kind=ops.OUT_F32)
    inner, amax, parts = ops.packed_gemv_fused(x_q, w_gu.weight, w_gu.weight_scale, bits=bits, s=x_s,
                                               epi=ops.EPI_SILU_PAIR)
    s_out = torch.empty(M, dtype=torch.float32, device=DEV)
    got, _, _ = ops.packed_gemv_fused(inner, w_dn.weight, w_dn.weight_scale, bits=bits, amax=amax, parts=parts,
                                      out_kind=ops.OUT_F32, s_out=s_out)
    clamped = float(np.float32(np.float32(1.0) / np.float32(1e-5)) * np.float32(127.0))
    assert torch.all(inner[0] == 0) and float(s_out[0]) == clamped
    assert torch.equal(s_out, i_s.reshape(-1)) and _same_bits(got, ref)
    # an all-zero residual stream: var = 0, every normalised value 0, the clamped multiplier again
    w_c = _packed(gen, 256, dim, bits)
    zeros = torch.zeros(M, dim, dtype=torch.bfloat16, device=DEV)
    ss = torch.zeros(M * 4, dtype=torch.float64, device=DEV)
    norm_w = torch.ones(dim, dtype=torch.bfloat16, device=DEV)
    out, _, _ = ops.packed_gemv_fused(zeros, w_c.weight, w_c.weight_scale, bits=bits, sumsq=ss, parts=4,
                                      norm_weight=norm_w, eps=EPS, s_out=s_out)
    assert torch.all(out == 0) and float(s_out[0]) == clamped and float(s_out[1]) == clamped


def test_argument_checks():
    from bitmtp_amd import ops
    ops.init_kernels()
    gen = _gen(9)
    bits, M, dim, ffn = 2, 2, 512, 1024
    w_gu, w_dn = _packed(gen, 2 * ffn, dim, bits), _packed(gen, dim, ffn, bits)
    x_q, x_s = ops.quant_input(_rows(gen, M, dim))
    h = _rows(gen, M, dim)
    t2 = ops.t2_lib()
    # three tokens, an odd row count, a bad K, an epilogue without parts: not taken
    assert t2.t2g128_fused_parts(ops.EPI_SILU_PAIR, 3, 2048, 512) == -1
    assert t2.t2g128_fused_parts(ops.EPI_SILU_PAIR, 1, 2047, 512) == -1
    assert t2.t2g128_fused_parts(ops.EPI_ADD_SUMSQ, 1, 2048, 500) == -1
    assert t2.t2g128_fused_parts(ops.EPI_PLAIN, 1, 2048, 512) == -1
    inner, amax, parts = ops.packed_gemv_fused(x_q, w_gu.weight, w_gu.weight_scale, bits=bits, s=x_s,
                                               epi=ops.EPI_SILU_PAIR)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.empty(M, dim, dtype=torch.bfloat16, device=DEV)
    ss = torch.empty(M * 256, dtype=torch.float64, device=DEV)

    def desc(**over):
        f = dict(act=inner.data_ptr(), act_aux=amax.data_ptr(), norm_weight=None, B=w_dn.weight.data_ptr(),
                 ws=w_dn.weight_scale.data_ptr(), out=out.data_ptr(), residual=h.data_ptr(),
                 out_aux=ss.data_ptr(), s_out=None, eps=EPS, M=M, N=dim, K=ffn,
                 act_kind=ops.ACT_BF16_AMAX, act_parts=parts, epi_kind=ops.EPI_ADD_SUMSQ, out_kind=ops.OUT_BF16)
        f.update(over)
        return ops.FusedGemvDesc(**f)

    assert t2.t2g128_gemv_fused(ctypes.byref(desc()), st) == 0
    assert t2.t2g128_gemv_fused(None, st) == 1
    for over in (dict(act=None), dict(act_aux=None), dict(act_aux=amax.data_ptr() + 2), dict(act_parts=0),
                 dict(act_parts=1025), dict(out_kind=ops.OUT_F32), dict(out_kind=ops.OUT_G32), dict(M=3),
                 dict(residual=None), dict(out_aux=None), dict(out_aux=ss.data_ptr() + 4), dict(act_kind=3),
                 dict(epi_kind=3), dict(K=ffn + 64), dict(act_kind=ops.ACT_INT8, epi_kind=ops.EPI_PLAIN),
                 dict(act_kind=ops.ACT_BF16_NORM), dict(act_kind=ops.ACT_BF16_NORM, act_aux=ss.data_ptr(),
                                                        norm_weight=h.data_ptr(), act_parts=257),
                 dict(s_out=x_s.data_ptr() + 2)):
        assert t2.t2g128_gemv_fused(ctypes.byref(desc(**over)), st) == 1, over
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):       # four tokens
        ops.packed_gemv_fused(x_q.repeat(2, 1), w_gu.weight, w_gu.weight_scale, bits=bits, s=x_s.repeat(2, 1),
                              epi=ops.EPI_SILU_PAIR)
    with pytest.raises(RuntimeError):       # fp16 weight scales
        ops.packed_gemv_fused(inner, w_dn.weight, w_dn.weight_scale.to(torch.float16), bits=bits, amax=amax,
                              parts=parts)
    with pytest.raises(ValueError):         # two descriptions of the activations
        ops.packed_gemv_fused(inner, w_dn.weight, w_dn.weight_scale, bits=bits, amax=amax, s=x_s, parts=parts)


ROPE_CASES = [
    # M, n_heads, n_kv, sigma, cache_len, role, pending rows (draft roles)
    (1, 16, 8, 1024, 500, "ar", 0),
    (1, 16, 8, 1024, 0, "ar", 0),        # nothing but the row itself
    (1, 16, 8, 1024, 63, "ar", 0),       # the row is the last slot of a chunk
    (1, 16, 8, 1024, 64, "ar", 0),       # ... the first slot of the next
    (2, 16, 8, 1024, 63, "ar", 0),       # the two rows sit in two chunks (and two workgroups)
    (2, 32, 8, 4096, 1531, "ar", 0),     # four query heads per kv head
    (1, 32, 8, 4096, 4095, "ar", 0),
    (2, 4, 2, 256, 255, "verify", 0),
    (1, 6, 2, 64, 17, "ar", 0),
    # wide blocks: several pair tiles per kv head, more rows than a wave takes at a time
    (9, 16, 8, 1024, 500, "verify", 0),
    (9, 16, 8, 1024, 500, "draft", 1),
    (9, 32, 8, 4096, 2000, "draft", 0),
    (9, 16, 8, 1024, 60, "verify", 0),   # the block's rows straddle two chunks
    (8, 16, 8, 1024, 0, "draft", 0),     # no history at all
    (17, 16, 8, 1024, 1007, "draft", 9),
    (17, 32, 8, 4096, 4079, "ar", 0),
    (16, 6, 2, 64, 48, "draft", 3),
    (5, 4, 2, 256, 100, "ar", 0),
    (3, 16, 8, 1024, 126, "ar", 0),
    (32, 16, 8, 1024, 300, "ar", 0),     # the widest block the library takes
]


@pytest.mark.parametrize("M,n_heads,n_kv,sigma,cache_len,role,n_pend", ROPE_CASES)
def test_attention_with_rope_inside_gives_the_bits_of_the_two_calls(M, n_heads, n_kv, sigma, cache_len, role,
                                                                    n_pend):
    """bonsai_decode_attention_rope against bonsai_qk_norm_rope_kv_write + bonsai_decode_attention:
    the bf16 and the quantised attention output and the K / V rows it leaves in the cache are the
    same bits; no other cache row is touched."""
    from bitmtp_amd import decode_ops, runtime
    print(f"[case] attention with rope inside M={M} heads={n_heads}/{n_kv} sigma={sigma} "
          f"cache_len={cache_len} {role} pending={n_pend}", flush=True)
    gen = _gen(M + n_heads + sigma + cache_len)
    slots = sigma + 32
    hd = 128
    xqkv = _rows(gen, M, (n_heads + 2 * n_kv) * hd, 1.5)
    qw = (1.0 + 0.1 * torch.randn(hd, generator=gen, device=DEV)).to(torch.bfloat16)
    kw = (1.0 + 0.1 * torch.randn(hd, generator=gen, device=DEV)).to(torch.bfloat16)
    max_pos = 8192
    ang = torch.rand(max_pos, hd, generator=gen, device=DEV) * 6.28
    cos, sin = torch.cos(ang).to(torch.bfloat16), torch.sin(ang).to(torch.bfloat16)
    # a verify block replays the anchor at cache_len - 1; the other roles start at cache_len
    first = cache_len - 1 if role == "verify" else cache_len
    positions = torch.tensor([first + i for i in range(M)], dtype=torch.int32, device=DEV)
    kv0 = (torch.randn(2, n_kv, slots, hd, generator=gen, device=DEV) * 1.2).to(torch.bfloat16)
    meta = torch.tensor(runtime.step_descriptor(role, M, 8, cache_len, n_pend), dtype=torch.int32, device=DEV)
    scratch = torch.empty(decode_ops.attention_scratch_bytes(M, n_heads, slots) // 4, dtype=torch.float32,
                          device=DEV)

    def outs():
        return (torch.zeros(M, n_heads * hd, dtype=torch.bfloat16, device=DEV),
                torch.zeros(M, n_heads * hd, dtype=torch.int8, device=DEV),
                torch.zeros(M, dtype=torch.float32, device=DEV))

    kv_a = kv0.clone()
    q = torch.empty(M, n_heads, hd, dtype=torch.bfloat16, device=DEV)
    decode_ops.qk_norm_rope_kv_write(xqkv, qw, kw, EPS, cos, sin, positions, q, kv_a[0], kv_a[1], n_heads,
                                     n_kv, sigma)
    o_a, q_a, s_a = outs()
    decode_ops.decode_attention(q, kv_a[0], kv_a[1], meta, scratch, sigma, out_bf16=o_a, out_q=q_a, out_s=s_a)
    torch.cuda.synchronize()

    kv_b = kv0.clone()
    o_b, q_b, s_b = outs()
    scratch.fill_(float("nan"))
    decode_ops.decode_attention_rope(xqkv, qw, kw, EPS, cos, sin, positions, kv_b[0], kv_b[1], meta, scratch,
                                     sigma, n_heads, out_bf16=o_b, out_q=q_b, out_s=s_b)
    torch.cuda.synchronize()
    assert _same_bits(o_a, o_b) and torch.equal(q_a, q_b) and torch.equal(s_a, s_b)
    assert torch.equal(kv_a.view(torch.int16), kv_b.view(torch.int16))
    changed = (kv_b.view(torch.int16) != kv0.view(torch.int16)).any(dim=-1)   # [2, n_kv, slots]
    assert not changed[:, :, :sigma].any() and not changed[:, :, sigma + M:].any()


def test_attention_with_rope_inside_refuses_blocks_beyond_the_widest():
    from bitmtp_amd import decode_ops
    m = decode_ops.ROPE_FUSED_MAX_WIDTH + 1
    xqkv = torch.zeros(m, (4 + 4) * 128, dtype=torch.bfloat16, device=DEV)
    w = torch.ones(128, dtype=torch.bfloat16, device=DEV)
    tab = torch.ones(16, 128, dtype=torch.bfloat16, device=DEV)
    kv = torch.zeros(2, 2, 128, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        decode_ops.decode_attention_rope(xqkv, w, w, EPS, tab, tab, torch.zeros(m, dtype=torch.int32, device=DEV),
                                         kv[0], kv[1], torch.zeros(2 + m, dtype=torch.int32, device=DEV),
                                         torch.zeros(1 << 18, dtype=torch.float32, device=DEV), 64, 4,
                                         out_bf16=torch.zeros(m, 512, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("kind", ["t2g128", "q1"])
def test_decode_loop_tokens_do_not_depend_on_the_fused_layers(kind, monkeypatch):
    """Greedy AR decoding (width-1 steps) through graphs captured with and without the fused
    layers gives the same tokens and the same logits bits."""
    from bitmtp_amd import generate
    from bitmtp_amd.model import BonsaiDecoder, ModelArgs, fused_plan
    from bitmtp_amd.runtime import GraphAtlas
    args = ModelArgs(dim=512, n_layers=3, n_heads=4, n_kv_heads=2, ffn_dim=1024, vocab_size=1000,
                     mask_token_id=999, kernel_kind=kind)
    model = BonsaiDecoder.random_init(args, seed=17, device=DEV)
    prompt = np.random.default_rng(4).integers(0, 1000, 21).tolist()
    runs = {}
    for flag in ("1", "0"):
        monkeypatch.setenv("BONSAI_FUSED_STEP", flag)
        assert (fused_plan(model, 1) is not None) == (flag == "1")
        assert fused_plan(model, 3) is None
        atlas = GraphAtlas(model, segment_ladder=(64,), threshold=0.9)
        print(f"[case] AR decode kind={kind} BONSAI_FUSED_STEP={flag}", flush=True)
        toks, _ = generate.ar_generate(atlas, prompt, max_gen_len=24)
        runs[flag] = (toks, atlas.workspace.logits[:1].clone())
        del atlas
    assert runs["1"][0] == runs["0"][0]
    assert _same_bits(runs["1"][1], runs["0"][1])


@pytest.mark.parametrize("threshold,hybrid_m", [(0.9, None), (0.0, 1)])
def test_hybrid_decode_tokens_do_not_depend_on_where_the_rope_runs(threshold, hybrid_m, monkeypatch):
    """Hybrid decoding (draft and verify blocks of nine and more rows) through graphs whose
    attention derives q / k itself and through graphs with the separate q / k launch commits the
    same tokens, and the last step leaves the same logits bits."""
    from bitmtp_amd import generate
    from bitmtp_amd.model import BonsaiDecoder, ModelArgs
    from bitmtp_amd.runtime import GraphAtlas
    args = ModelArgs(dim=512, n_layers=3, n_heads=4, n_kv_heads=2, ffn_dim=1024, vocab_size=1000,
                     mask_token_id=999)
    model = BonsaiDecoder.random_init(args, seed=23, device=DEV)
    prompt = np.random.default_rng(9).integers(0, 999, 19).tolist()
    runs = {}
    for flag in ("1", "0"):
        monkeypatch.setenv("BONSAI_ROPE_IN_ATTENTION", flag)
        atlas = GraphAtlas(model, segment_ladder=(128,), threshold=0.9)
        print(f"[case] hybrid decode threshold={threshold} BONSAI_ROPE_IN_ATTENTION={flag}", flush=True)
        toks, st = generate.hybrid_generate(atlas, prompt, threshold=threshold, hybrid_m=hybrid_m,
                                            max_gen_len=40)
        runs[flag] = (toks, st["n_iters"], atlas.workspace.logits.clone())
        del atlas
    assert runs["1"][0] == runs["0"][0] and runs["1"][1] == runs["0"][1]
    assert _same_bits(runs["1"][2], runs["0"][2])


MERGE_CASES = [
    # M, n_heads, n_kv, sigma, cache_len, role
    (1, 16, 8, 1024, 500, "ar"),
    (1, 16, 8, 1024, 0, "ar"),         # one live part
    (1, 16, 8, 1024, 63, "ar"),
    (1, 16, 8, 1024, 64, "ar"),
    (2, 16, 8, 1024, 1022, "ar"),      # every part live
    (2, 32, 8, 4096, 1531, "ar"),
    (1, 32, 8, 4096, 4095, "ar"),      # runs of several chunks per part
    (2, 4, 2, 256, 255, "verify"),
    (1, 6, 2, 64, 17, "ar"),           # three heads per kv head
    (2, 16, 16, 128, 100, "ar"),       # one head per kv head, sixteen counters
    (8, 16, 8, 1024, 300, "draft"),    # a full pair tile
    (4, 32, 8, 4096, 77, "ar"),
]


@pytest.mark.parametrize("M,n_heads,n_kv,sigma,cache_len,role", MERGE_CASES)
def test_attention_that_merges_its_own_partials(M, n_heads, n_kv, sigma, cache_len, role):
    """bonsai_decode_attention_rope_parts (one launch) against bonsai_decode_attention_rope (two):
    the same bf16 rows, maxima whose largest gives the same multiplier, counters back at zero --
    twice in a row on the same counters, the second time with a shorter history."""
    from bitmtp_amd import decode_ops, runtime
    print(f"[case] self-merging attention M={M} heads={n_heads}/{n_kv} sigma={sigma} "
          f"cache_len={cache_len} {role}", flush=True)
    gen = _gen(3 * M + n_heads + sigma + cache_len)
    slots, hd = sigma + 32, 128
    qw = (1.0 + 0.1 * torch.randn(hd, generator=gen, device=DEV)).to(torch.bfloat16)
    kw = (1.0 + 0.1 * torch.randn(hd, generator=gen, device=DEV)).to(torch.bfloat16)
    max_pos = 8192
    ang = torch.rand(max_pos, hd, generator=gen, device=DEV) * 6.28
    cos, sin = torch.cos(ang).to(torch.bfloat16), torch.sin(ang).to(torch.bfloat16)
    scratch = torch.empty(decode_ops.attention_scratch_bytes(M, n_heads, slots) // 4, dtype=torch.float32,
                          device=DEV)
    arrivals = torch.zeros(decode_ops.ATTN_MAX_KV_HEADS, dtype=torch.int32, device=DEV)
    ld = decode_ops.attention_amax_ld(n_kv)
    for clen in (cache_len, cache_len // 3 + (1 if role == "verify" else 0)):
        xqkv = _rows(gen, M, (n_heads + 2 * n_kv) * hd, 1.5)
        first = clen - 1 if role == "verify" else clen
        positions = torch.tensor([first + i for i in range(M)], dtype=torch.int32, device=DEV)
        kv0 = (torch.randn(2, n_kv, slots, hd, generator=gen, device=DEV) * 1.2).to(torch.bfloat16)
        meta = torch.tensor(runtime.step_descriptor(role, M, 8, clen, 0), dtype=torch.int32, device=DEV)
        kv_a = kv0.clone()
        o_a = torch.zeros(M, n_heads * hd, dtype=torch.bfloat16, device=DEV)
        q_a = torch.zeros(M, n_heads * hd, dtype=torch.int8, device=DEV)
        s_a = torch.zeros(M, dtype=torch.float32, device=DEV)
        decode_ops.decode_attention_rope(xqkv, qw, kw, EPS, cos, sin, positions, kv_a[0], kv_a[1], meta,
                                         scratch, sigma, n_heads, out_bf16=o_a, out_q=q_a, out_s=s_a)
        torch.cuda.synchronize()
        kv_b = kv0.clone()
        o_b = torch.zeros_like(o_a)
        amax = torch.full((M, ld), 7.0, dtype=torch.bfloat16, device=DEV)
        scratch.fill_(float("nan"))
        decode_ops.decode_attention_rope_parts(xqkv, qw, kw, EPS, cos, sin, positions, kv_b[0], kv_b[1],
                                               meta, scratch, arrivals, sigma, n_heads, o_b, amax)
        torch.cuda.synchronize()
        assert _same_bits(o_a, o_b)
        assert torch.equal(kv_a.view(torch.int16), kv_b.view(torch.int16))
        assert int(arrivals.abs().sum()) == 0
        assert float(amax[:, n_kv:].float().abs().sum()) == 0.0
        per_kv = o_b.float().abs().view(M, n_kv, -1).amax(dim=2)
        assert torch.equal(amax[:, :n_kv].float(), per_kv)
        top = amax.float().amax(dim=1).clamp_min(1e-5)
        assert torch.equal((1.0 / top) * 127.0, s_a)


@pytest.mark.parametrize("bits", [2, 1])
@pytest.mark.parametrize("M", [1, 2])
def test_o_projection_from_the_self_merging_attention(M, bits):
    """attention (one launch) -> o projection that quantises from its rows and maxima, against
    attention (two launches, int8 rows out) -> o projection: the residual stream and the sums of
    squares that come out are the same bits."""
    from bitmtp_amd import decode_ops, ops, runtime
    n_heads, n_kv, sigma, cache_len, hd = 16, 8, 1024, 700, 128
    print(f"[case] o projection behind the self-merging attention M={M} bits={bits}", flush=True)
    gen = _gen(50 + M + bits)
    slots = sigma + 32
    w_o = _packed(gen, n_heads * hd, n_heads * hd, bits)
    xqkv = _rows(gen, M, (n_heads + 2 * n_kv) * hd, 1.5)
    h = _rows(gen, M, n_heads * hd, 1.0)
    qw = (1.0 + 0.1 * torch.randn(hd, generator=gen, device=DEV)).to(torch.bfloat16)
    kw = (1.0 + 0.1 * torch.randn(hd, generator=gen, device=DEV)).to(torch.bfloat16)
    ang = torch.rand(4096, hd, generator=gen, device=DEV) * 6.28
    cos, sin = torch.cos(ang).to(torch.bfloat16), torch.sin(ang).to(torch.bfloat16)
    positions = torch.tensor([cache_len + i for i in range(M)], dtype=torch.int32, device=DEV)
    kv0 = (torch.randn(2, n_kv, slots, hd, generator=gen, device=DEV) * 1.2).to(torch.bfloat16)
    meta = torch.tensor(runtime.step_descriptor("ar", M, 8, cache_len, 0), dtype=torch.int32, device=DEV)
    scratch = torch.empty(decode_ops.attention_scratch_bytes(M, n_heads, slots) // 4, dtype=torch.float32,
                          device=DEV)
    kv_a = kv0.clone()
    q_a = torch.zeros(M, n_heads * hd, dtype=torch.int8, device=DEV)
    s_a = torch.zeros(M, dtype=torch.float32, device=DEV)
    decode_ops.decode_attention_rope(xqkv, qw, kw, EPS, cos, sin, positions, kv_a[0], kv_a[1], meta, scratch,
                                     sigma, n_heads, out_q=q_a, out_s=s_a)
    h_a, ss_a, parts_a = ops.packed_gemv_fused(q_a, w_o.weight, w_o.weight_scale, bits=bits, s=s_a,
                                               epi=ops.EPI_ADD_SUMSQ, residual=h)
    kv_b = kv0.clone()
    rows = torch.zeros(M, n_heads * hd, dtype=torch.bfloat16, device=DEV)
    amax = torch.zeros(M, decode_ops.attention_amax_ld(n_kv), dtype=torch.bfloat16, device=DEV)
    arrivals = torch.zeros(decode_ops.ATTN_MAX_KV_HEADS, dtype=torch.int32, device=DEV)
    decode_ops.decode_attention_rope_parts(xqkv, qw, kw, EPS, cos, sin, positions, kv_b[0], kv_b[1], meta,
                                           scratch, arrivals, sigma, n_heads, rows, amax)
    s_b = torch.zeros(M, dtype=torch.float32, device=DEV)
    h_b, ss_b, parts_b = ops.packed_gemv_fused(rows, w_o.weight, w_o.weight_scale, bits=bits, amax=amax,
                                               parts=n_kv, epi=ops.EPI_ADD_SUMSQ, residual=h, s_out=s_b)
    torch.cuda.synchronize()
    assert parts_a == parts_b and torch.equal(s_a, s_b)
    assert _same_bits(h_a, h_b)
    assert torch.equal(ss_a[:M * parts_a].view(torch.int64), ss_b[:M * parts_b].view(torch.int64))


def test_self_merging_attention_refuses_more_than_one_pair_tile():
    from bitmtp_amd import decode_ops
    m, n_heads, n_kv = 9, 4, 2     # 18 pairs
    xqkv = torch.zeros(m, (n_heads + 2 * n_kv) * 128, dtype=torch.bfloat16, device=DEV)
    w = torch.ones(128, dtype=torch.bfloat16, device=DEV)
    tab = torch.ones(16, 128, dtype=torch.bfloat16, device=DEV)
    kv = torch.zeros(2, n_kv, 128, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        decode_ops.decode_attention_rope_parts(
            xqkv, w, w, EPS, tab, tab, torch.zeros(m, dtype=torch.int32, device=DEV), kv[0], kv[1],
            torch.zeros(2 + m, dtype=torch.int32, device=DEV), torch.zeros(1 << 18, dtype=torch.float32, device=DEV),
            torch.zeros(64, dtype=torch.int32, device=DEV), 64, n_heads,
            torch.zeros(m, n_heads * 128, dtype=torch.bfloat16, device=DEV),
            torch.zeros(m, 8, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("kind", ["t2g128", "q1"])
def test_decode_loop_tokens_do_not_depend_on_the_self_merging_attention(kind, monkeypatch):
    """Greedy AR decoding through graphs whose attention merges its own partials (five launches a
    layer) and through graphs with the separate merge gives the same tokens and logits bits."""
    from bitmtp_amd import generate
    from bitmtp_amd.model import BonsaiDecoder, ModelArgs, fused_plan
    from bitmtp_amd.runtime import GraphAtlas
    args = ModelArgs(dim=512, n_layers=3, n_heads=4, n_kv_heads=2, ffn_dim=1024, vocab_size=1000,
                     mask_token_id=999, kernel_kind=kind)
    model = BonsaiDecoder.random_init(args, seed=31, device=DEV)
    prompt = np.random.default_rng(6).integers(0, 1000, 70).tolist()
    runs = {}
    for flag in ("1", "0"):
        monkeypatch.setenv("BONSAI_ATTENTION_ONE_LAUNCH", flag)
        assert (fused_plan(model, 1).attn > 0) == (flag == "1")
        atlas = GraphAtlas(model, segment_ladder=(128,), threshold=0.9)
        print(f"[case] AR decode kind={kind} BONSAI_ATTENTION_ONE_LAUNCH={flag}", flush=True)
        toks, _ = generate.ar_generate(atlas, prompt, max_gen_len=40)
        runs[flag] = (toks, atlas.workspace.logits[:1].clone())
        del atlas
    assert runs["1"][0] == runs["0"][0]
    assert _same_bits(runs["1"][1], runs["0"][1])
