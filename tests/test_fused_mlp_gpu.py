"""The MLP tail as two launches (``*_gemv_silu_pair`` + ``*_gemv_bf16_act``, blocks of one or two
tokens) against the three launches it stands for -- gate|up projection, SiLU * up +
quantisation (src/bonsai_sft/gpu/model.py:1058-1061), down projection -- through the C ABI:

* the bf16 product ``inner`` quantises (``bonsai_act_quant_int8``) to exactly the ``q`` and ``s``
  of ``bonsai_silu_mul_quant_int8`` on the three-launch path's gate|up result, the multipliers
  the second launch derives are those ``s``, and its fp32 and bf16 results are the same bits
  as the third launch's (the three-launch path is forced onto the dot4 kernels, whose
  arithmetic the fused forms share);
* against the CPU oracle directly: the projection inside the first launch within one bf16
  step, its SiLU * up within the tolerance of the hardware exp2 (as for the stand-alone
  producer), the second launch within one bf16 step of the oracle's GEMV on the GPU's own
  quantised input;
* the maxima array: every element written, the pad zero, the row maximum equal to max |inner|;
* the decode loop produces the same tokens with and without the fused tail.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

# (dim, ffn): the 1.7B- and 4B-shaped MLPs, the tiny test model, odd chunk counts
SHAPES = [(2048, 6144), (2560, 9728), (512, 1024), (384, 1408), (128, 128)]


def _lib(ops, bits):
    return ops.t2_lib() if bits == 2 else ops.q1_lib()


@pytest.fixture
def dot4_only():
    """Keeps two-token projections of the three-launch path on the dot4 kernels (the built-in
    choice sends K >= 4096 to the matrix cores, whose fp32 summation order differs)."""
    from bitmtp_amd import ops
    ops.init_kernels()
    ops.t2_lib().t2g128_set_mfma_tuning(3, 0, 0, 0, 0)
    ops.q1_lib().q1g128_set_mfma_tuning(3, 0, 0, 0, 0)
    yield
    ops.t2_lib().t2g128_set_mfma_tuning(0, 0, 0, 0, 0)
    ops.q1_lib().q1g128_set_mfma_tuning(0, 0, 0, 0, 0)


def _problem(seed, M, dim, ffn, bits, x_scale=1.0):
    from bitmtp_amd import model as mdl
    from bitmtp_amd import ops
    gen = torch.Generator(device=DEV)
    gen.manual_seed(seed)
    w_gu = mdl._random_packed(2 * ffn, dim, gen, DEV, bits)
    w_dn = mdl._random_packed(dim, ffn, gen, DEV, bits)
    # scales large enough for the gate to leave the linear part of the sigmoid
    w_gu.weight_scale.mul_(8.0)
    x = (torch.randn(M, dim, generator=gen, device=DEV) * x_scale).to(torch.bfloat16)
    x_q, x_s = ops.quant_input(x)
    return w_gu, w_dn, x_q, x_s


@pytest.mark.parametrize("dim,ffn", SHAPES)
@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("bits", [2, 1])
def test_two_launches_give_the_bits_of_three(dot4_only, bits, M, dim, ffn):
    from bitmtp_amd import ops
    print(f"[case] fused MLP tail bits={bits} M={M} dim={dim} ffn={ffn}", flush=True)
    w_gu, w_dn, x_q, x_s = _problem(1000 * bits + 10 * M + dim, M, dim, ffn, bits)

    gu = ops.packed_gemv_ex(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=bits)
    assert ops.last_kernel(bits).startswith("gemv_dot4_kernel")
    i_q, i_s = ops.silu_mul_quant(gu)
    want = {k: ops.packed_gemv_ex(i_q, w_dn.weight, i_s, w_dn.weight_scale, bits=bits, out_kind=k)
            for k in (ops.OUT_F32, ops.OUT_BF16)}
    assert ops.last_kernel(bits).startswith("gemv_dot4_kernel")

    inner, amax, parts = ops.packed_gemv_silu_pair(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=bits,
                                                   amax=torch.full((M, 1024), 7e9, dtype=torch.bfloat16,
                                                                   device=DEV))
    assert ops.last_kernel(bits).startswith("gemv_dot4_fused_kernel")
    assert 0 < parts <= 1024 and parts == ops.silu_pair_parts(M, 2 * ffn, dim, bits=bits)
    q2, s2 = ops.quant_input(inner)
    assert torch.equal(q2, i_q) and torch.equal(s2.reshape(-1), i_s.reshape(-1))

    ld = (parts + 7) // 8 * 8
    am = amax.reshape(-1)[: M * ld].view(M, ld).float()
    assert torch.all(am[:, parts:] == 0) and torch.all(am >= 0)
    assert torch.equal(am.max(dim=1).values, inner.float().abs().max(dim=1).values)

    for kind, ref in want.items():
        s_out = torch.empty(M, dtype=torch.float32, device=DEV)
        got = ops.packed_gemv_bf16_act(inner, w_dn.weight, w_dn.weight_scale, amax, parts, bits=bits,
                                       out_kind=kind, s_out=s_out)
        assert ops.last_kernel(bits).startswith("gemv_dot4_fused_kernel")
        assert torch.equal(s_out, i_s.reshape(-1))
        as_int = torch.int32 if kind == ops.OUT_F32 else torch.int16
        assert torch.equal(got.view(as_int), ref.view(as_int)), f"out_kind {kind}"


@pytest.mark.parametrize("bits,M,dim,ffn", [(2, 1, 2048, 6144), (2, 2, 512, 1024), (1, 2, 2560, 9728),
                                            (1, 1, 384, 1408)])
def test_two_launches_against_the_oracle(bits, M, dim, ffn):
    from oracle import oracle as O
    from bitmtp_amd import ops
    O.build()
    print(f"[case] fused MLP tail vs oracle bits={bits} M={M} dim={dim} ffn={ffn}", flush=True)
    w_gu, w_dn, x_q, x_s = _problem(77 + bits + M + ffn, M, dim, ffn, bits)
    inner, amax, parts = ops.packed_gemv_silu_pair(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=bits)
    s_out = torch.empty(M, dtype=torch.float32, device=DEV)
    out = ops.packed_gemv_bf16_act(inner, w_dn.weight, w_dn.weight_scale, amax, parts, bits=bits, s_out=s_out)

    def host(p):
        return p.weight.cpu().numpy().view(np.uint8), bf16_bits(p.weight_scale)

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

    # second launch: the oracle's GEMV on the GPU's own quantised input
    _, ref = O.c_gemv(q_gpu.cpu().numpy(), host(w_dn)[0], s_gpu, host(w_dn)[1], bits)
    d = np.abs(bf16_ordinal(bf16_bits(out)) - bf16_ordinal(ref))
    assert d.max() <= 1, f"down projection: {d.max()} bf16 steps from the oracle"


def test_zero_and_large_rows(dot4_only):
    """A token whose products are all zero takes the clamped multiplier fl(fl(1 / 1e-5) * 127);
    a token with large values and a small one side by side keep their own multipliers."""
    from bitmtp_amd import ops
    dim, ffn, bits, M = 512, 1024, 2, 2
    print("[case] fused MLP tail: zero row, large row", flush=True)
    w_gu, w_dn, x_q, x_s = _problem(5, M, dim, ffn, bits, x_scale=30.0)
    x_q[0].zero_()
    gu = ops.packed_gemv_ex(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=bits)
    i_q, i_s = ops.silu_mul_quant(gu)
    ref = ops.packed_gemv_ex(i_q, w_dn.weight, i_s, w_dn.weight_scale, bits=bits, out_kind=ops.OUT_F32)
    inner, amax, parts = ops.packed_gemv_silu_pair(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=bits)
    s_out = torch.empty(M, dtype=torch.float32, device=DEV)
    got = ops.packed_gemv_bf16_act(inner, w_dn.weight, w_dn.weight_scale, amax, parts, bits=bits,
                                   out_kind=ops.OUT_F32, s_out=s_out)
    assert torch.all(inner[0] == 0) and float(s_out[0]) == float(np.float32(np.float32(1.0) / np.float32(1e-5)) * np.float32(127.0))
    assert torch.equal(s_out, i_s.reshape(-1))
    assert torch.equal(got.view(torch.int32), ref.view(torch.int32))


def test_argument_checks():
    from bitmtp_amd import ops
    ops.init_kernels()
    w_gu, w_dn, x_q, x_s = _problem(9, 2, 512, 1024, 2)
    t2 = ops.t2_lib()
    # three tokens, an odd row count: not taken
    assert t2.t2g128_silu_pair_parts(3, 2048, 512) == -1
    assert t2.t2g128_silu_pair_parts(1, 2047, 512) == -1
    assert t2.t2g128_silu_pair_parts(1, 2048, 500) == -1
    inner, amax, parts = ops.packed_gemv_silu_pair(x_q, w_gu.weight, x_s, w_gu.weight_scale, bits=2)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.empty(2, 512, dtype=torch.bfloat16, device=DEV)
    args = [vp(inner), vp(w_dn.weight), vp(out), vp(w_dn.weight_scale), 2, 512, 1024, vp(amax), parts, None,
            ops.OUT_BF16, st]
    assert t2.t2g128_gemv_bf16_act(*args) == 0
    for pos, bad in ((0, None), (7, None), (7, ctypes.c_void_p(amax.data_ptr() + 2)), (8, 0), (8, 1025),
                     (10, ops.OUT_G32), (4, 3)):
        a = list(args)
        a[pos] = bad
        assert t2.t2g128_gemv_bf16_act(*a) == 1, (pos, bad)
    pargs = [vp(x_q), vp(w_gu.weight), vp(inner), vp(x_s), vp(w_gu.weight_scale), 2, 2048, 512, vp(amax), st]
    assert t2.t2g128_gemv_silu_pair(*pargs) == 0
    for pos, bad in ((8, None), (8, ctypes.c_void_p(amax.data_ptr() + 4)), (5, 3), (6, 2047), (3, None)):
        a = list(pargs)
        a[pos] = bad
        assert t2.t2g128_gemv_silu_pair(*a) == 1, (pos, bad)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):
        ops.packed_gemv_silu_pair(x_q.repeat(2, 1), w_gu.weight, x_s.repeat(2, 1), w_gu.weight_scale, bits=2)
    with pytest.raises(RuntimeError):
        ops.packed_gemv_bf16_act(inner, w_dn.weight, w_dn.weight_scale.to(torch.float16), amax, parts, bits=2)


@pytest.mark.parametrize("kind", ["t2g128", "q1"])
def test_decode_loop_tokens_do_not_depend_on_the_fused_tail(kind, monkeypatch):
    """Greedy AR decoding (width-1 steps) through graphs captured with and without the fused
    tail gives the same tokens and the same logits bits."""
    from bitmtp_amd import generate
    from bitmtp_amd.model import BonsaiDecoder, ModelArgs, mlp_tail_parts
    from bitmtp_amd.runtime import GraphAtlas
    args = ModelArgs(dim=512, n_layers=3, n_heads=4, n_kv_heads=2, ffn_dim=1024, vocab_size=1000,
                     mask_token_id=999, kernel_kind=kind)
    model = BonsaiDecoder.random_init(args, seed=17, device=DEV)
    prompt = np.random.default_rng(4).integers(0, 1000, 21).tolist()
    runs = {}
    for flag in ("1", "0"):
        monkeypatch.setenv("BONSAI_FUSED_MLP", flag)
        assert (mlp_tail_parts(model, 1) > 0) == (flag == "1")
        atlas = GraphAtlas(model, segment_ladder=(64,), threshold=0.9)
        print(f"[case] AR decode kind={kind} BONSAI_FUSED_MLP={flag}", flush=True)
        toks, _ = generate.ar_generate(atlas, prompt, max_gen_len=24)
        runs[flag] = (toks, atlas.workspace.logits[:1].clone())
        del atlas
    assert runs["1"][0] == runs["0"][0]
    assert torch.equal(runs["1"][1].view(torch.int16), runs["0"][1].view(torch.int16))
