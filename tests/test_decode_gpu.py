"""GPU tests of the decode harness: the ops between the GEMVs against the decode oracle,
one whole captured step against the CPU composition of the oracles, and the system
invariants of the generation loops (fast_generate.py:611-657,1151-1162).

Tolerances: q/k-norm + RoPE, KV commit and the quantisation after attention are bit-exact;
attention (bf16 inputs, fp32 online softmax with the probabilities rounded to bf16 for the
P V product as in the reference, model.py:1001; float64 throughout in the oracle) is compared
on its bf16 output with rtol 2e-2 / atol 2e-3; whole-step logits with atol 6e-2 * max|logit|.
Both chunk passes of the attention (matrix cores, the default, and the VALU form) are run.
"""
import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bf16_from_bits(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def _rand_bf16(rng, shape, std=1.0):
    return torch.from_numpy(rng.normal(0, std, shape).astype(np.float32)).to(torch.bfloat16)


@pytest.fixture(scope="module")
def DO():
    from oracle import decode_oracle
    from oracle import oracle as O
    O.build()
    return decode_oracle


# ---------------------------------------------------------------- qk norm + rope
@pytest.mark.parametrize("M,n_heads,n_kv", [(1, 16, 8), (9, 16, 8), (17, 32, 8), (5, 3, 1)])
def test_qk_norm_rope_bit_exact(DO, M, n_heads, n_kv):
    from bitmtp_amd import decode_ops
    from bitmtp_amd.model import ModelArgs, rope_tables
    rng = np.random.default_rng(M * 100 + n_heads)
    slots, write = 64, 40
    xqkv = _rand_bf16(rng, (M, (n_heads + 2 * n_kv) * 128), 2.0)
    qw = (1 + 0.1 * _rand_bf16(rng, (128,)).float()).to(torch.bfloat16)
    kw = (1 + 0.1 * _rand_bf16(rng, (128,)).float()).to(torch.bfloat16)
    cos_t, sin_t = rope_tables(ModelArgs(), 512, "cpu")
    positions = torch.from_numpy(rng.integers(0, 512, M).astype(np.int32))
    k_layer = _rand_bf16(rng, (n_kv, slots, 128))
    v_layer = _rand_bf16(rng, (n_kv, slots, 128))
    q_out = torch.zeros(M, n_heads, 128, dtype=torch.bfloat16)

    d = [t.to(DEV) for t in (xqkv, qw, kw, cos_t, sin_t, positions, q_out, k_layer, v_layer)]
    decode_ops.qk_norm_rope_kv_write(d[0], d[1], d[2], 1e-6, d[3], d[4], d[5], d[6], d[7], d[8],
                                     n_heads, n_kv, write)
    torch.cuda.synchronize()
    q, k, v = DO.qk_norm_rope(bf16_bits(xqkv), bf16_bits(qw), bf16_bits(kw), 1e-6, bf16_bits(cos_t),
                              bf16_bits(sin_t), positions.numpy(), n_heads, n_kv)
    assert np.array_equal(bf16_bits(d[6]), q)
    want_k = bf16_bits(k_layer).copy()
    want_v = bf16_bits(v_layer).copy()
    want_k[:, write:write + M] = k.transpose(1, 0, 2)
    want_v[:, write:write + M] = v.transpose(1, 0, 2)
    assert np.array_equal(bf16_bits(d[7]), want_k)      # also: no other slot was touched
    assert np.array_equal(bf16_bits(d[8]), want_v)


# ---------------------------------------------------------------- attention
ATTN_CASES = [
    # M, n_heads, n_kv, sigma, cache_len, role, n_pend
    (1, 16, 8, 256, 0, "ar", 0),
    (1, 16, 8, 256, 1, "ar", 0),
    (1, 16, 8, 256, 200, "ar", 0),
    (1, 32, 8, 1024, 777, "ar", 0),
    (9, 16, 8, 256, 63, "verify", 0),
    (9, 16, 8, 256, 64, "verify", 0),
    (9, 32, 8, 1024, 1000, "verify", 0),
    (9, 16, 8, 256, 100, "draft", 1),
    (10, 16, 8, 256, 129, "draft", 2),
    (12, 16, 8, 256, 55, "draft", 3),
    (16, 16, 8, 1024, 500, "draft", 8),
    (17, 32, 8, 256, 239, "draft", 9),
    (16, 16, 8, 256, 0, "ar", 0),
    (16, 16, 8, 256, 240, "ar", 0),
    (5, 3, 1, 64, 30, "verify", 0),
    (8, 16, 8, 256, 77, "draft", 0),
    (32, 16, 8, 256, 100, "ar", 0),
    # long segments: several chunks per workgroup of the matrix-core pass
    (9, 16, 8, 4096, 3000, "verify", 0),
    (1, 32, 8, 4096, 4095, "ar", 0),
    (17, 32, 8, 4096, 1531, "draft", 9),
    (3, 6, 2, 2048, 1100, "ar", 0),
]


@pytest.mark.parametrize("engine", [0, 1])
@pytest.mark.parametrize("M,n_heads,n_kv,sigma,cache_len,role,n_pend", ATTN_CASES)
def test_attention_against_oracle(DO, oracle, M, n_heads, n_kv, sigma, cache_len, role, n_pend,
                                  engine):
    from bitmtp_amd import decode_ops, runtime
    rng = np.random.default_rng(hash((M, n_heads, sigma, cache_len)) % (2 ** 31))
    slots = sigma + max(17, M)
    q = _rand_bf16(rng, (M, n_heads, 128), 1.5)
    k = _rand_bf16(rng, (n_kv, slots, 128), 1.5)
    v = _rand_bf16(rng, (n_kv, slots, 128), 1.0)
    desc = runtime.step_descriptor(role, M, 8, cache_len, n_pend)
    meta = torch.tensor(desc, dtype=torch.int32, device=DEV)
    scratch = torch.empty(decode_ops.attention_scratch_bytes(M, n_heads, slots) // 4,
                          dtype=torch.float32, device=DEV)
    out = torch.zeros(M, n_heads * 128, dtype=torch.bfloat16, device=DEV)
    out_q = torch.zeros(M, n_heads * 128, dtype=torch.int8, device=DEV)
    out_s = torch.zeros(M, dtype=torch.float32, device=DEV)
    print(f"attention case M={M} heads={n_heads}/{n_kv} sigma={sigma} cache_len={cache_len} {role} "
          f"engine={engine}", flush=True)
    decode_ops.decode_lib().bonsai_decode_set_attention_engine(engine)
    try:
        decode_ops.decode_attention(q.to(DEV), k.to(DEV), v.to(DEV), meta, scratch, sigma,
                                    out_bf16=out, out_q=out_q, out_s=out_s)
        torch.cuda.synchronize()
    finally:
        decode_ops.decode_lib().bonsai_decode_set_attention_engine(0)
    vis = runtime.dense_visibility(desc, M, sigma)
    # the oracle reads workspace rows where the kernel does: slots sigma..sigma+M-1
    want = DO.attention(bf16_bits(q), bf16_bits(k), bf16_bits(v), vis, 1 / np.sqrt(128))
    got = out.float().cpu().numpy().astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=2e-2, atol=2e-3)
    # quantisation of the kernel's own bf16 result is exact
    wq, wsc = oracle.c_act_quant(out.float().cpu().numpy())
    assert np.array_equal(out_q.cpu().numpy(), wq)
    assert np.array_equal(out_s.cpu().numpy(), wsc)


def test_attention_row_without_visible_slot_is_zero(DO):
    from bitmtp_amd import decode_ops
    M, n_heads, n_kv, sigma = 4, 2, 1, 64
    rng = np.random.default_rng(0)
    q = _rand_bf16(rng, (M, n_heads, 128)).to(DEV)
    k = _rand_bf16(rng, (n_kv, sigma + M, 128)).to(DEV)
    v = _rand_bf16(rng, (n_kv, sigma + M, 128)).to(DEV)
    meta = torch.tensor([0, -1, 1, 0, 0b101, 0], dtype=torch.int32, device=DEV)
    scratch = torch.empty(decode_ops.attention_scratch_bytes(M, n_heads, sigma + M) // 4,
                          dtype=torch.float32, device=DEV)
    out = torch.full((M, n_heads * 128), 7.0, dtype=torch.bfloat16, device=DEV)
    decode_ops.decode_attention(q, k, v, meta, scratch, sigma, out_bf16=out)
    torch.cuda.synchronize()
    o = out.float().cpu()
    assert torch.all(o[1] == 0) and torch.all(o[3] == 0)
    # row 0 sees only workspace row 0: its output is that V row
    assert torch.equal(out[0].view(n_heads, 128)[0].cpu(), v[0, sigma].cpu())
    assert torch.any(o[2] != 0)


def test_kv_commit_moves_exactly_the_rows():
    from bitmtp_amd import decode_ops
    rng = np.random.default_rng(1)
    kv = _rand_bf16(rng, (2, 3, 2, 40, 128)).to(DEV)
    want = kv.clone()
    want[:, :, :, 5:9] = want[:, :, :, 31:35]
    decode_ops.kv_commit(kv, 31, 5, 4)
    torch.cuda.synchronize()
    assert torch.equal(kv, want)
    with pytest.raises(RuntimeError):
        decode_ops.kv_commit(kv, 5, 7, 4)      # overlapping ranges
    decode_ops.kv_commit(kv, 5, 7, 0)          # nothing to do


@pytest.mark.parametrize("rows,vocab,ld", [(1, 151936, 151936), (8, 151669, 151936), (9, 1000, 1024),
                                           (3, 37, 40)])
def test_draft_chain_kernel(DO, rows, vocab, ld):
    from bitmtp_amd import decode_ops
    rng = np.random.default_rng(rows + vocab)
    logits = _rand_bf16(rng, (rows, ld), 2.0)
    # make some rows confident, plant a tie and poison the padding columns
    for r in range(1, rows, 2):
        logits[r, (r * 7919) % vocab] = 30.0
    if rows > 2 and vocab > 20:
        logits[2, 5] = 25.0
        logits[2, 17] = 25.0
    logits[:, vocab:] = 100.0
    wt, wc, wn = DO.draft_chain(logits[:, :vocab].float().numpy(), 0.9)
    # one workgroup per row, and the rows split over several workgroups through a scratch buffer
    nbytes = int(decode_ops.decode_lib().bonsai_draft_chain_scratch_bytes(rows))
    assert nbytes == rows * 32 * 16
    for scratch in (None, torch.full((nbytes // 4,), float("nan"), device=DEV)):
        tokens = torch.zeros(rows, dtype=torch.int32, device=DEV)
        conf = torch.zeros(rows, dtype=torch.float32, device=DEV)
        accept = torch.zeros(2, dtype=torch.int32, device=DEV)
        print(f"[case] draft_chain rows={rows} vocab={vocab} split={scratch is not None}", flush=True)
        decode_ops.draft_chain(logits.to(DEV), vocab, 0.9, tokens, conf, accept, scratch=scratch)
        torch.cuda.synchronize()
        assert tokens.cpu().tolist() == wt.tolist()
        np.testing.assert_allclose(conf.cpu().numpy(), wc, rtol=2e-3, atol=1e-6)
        assert accept.cpu().tolist() == [wn, rows]
    with pytest.raises(RuntimeError):
        decode_ops.draft_chain(logits.to(DEV), vocab, 0.9, tokens, conf, accept,
                               scratch=torch.zeros(4, device=DEV))


# ---------------------------------------------------------------- bf16 output projection
def _assert_one_bf16_step(got: torch.Tensor, want64: torch.Tensor) -> None:
    """fp32 accumulation against a float64 product: the same or the adjacent bf16 value
    wherever the result is not a cancellation (>= 2 % of the largest), a small absolute
    error elsewhere (there the fp32 summation order shows in the last places)."""
    want_b = want64.to(torch.bfloat16)
    d = np.abs(bf16_ordinal(bf16_bits(got)) - bf16_ordinal(bf16_bits(want_b)))
    top = want64.abs().max().item()
    big = (want64.abs() >= 0.02 * top).cpu().numpy()
    assert d[big].max() <= 1 and (d[big] != 0).mean() < 0.05
    assert (got.double() - want64).abs().max().item() <= 2.0 ** -8 * top


@pytest.mark.parametrize("M,N,K", [(1, 1000, 512), (9, 4099, 2048), (16, 1536, 2560), (17, 300, 64),
                                   (32, 129, 128), (3, 7, 320), (5, 151936, 2048)])
def test_bf16_linear_against_fp32_matmul(M, N, K):
    """fp32 accumulation of exact bf16 products, one rounding: the bf16 result is within one
    bf16 step of the rounded float64 product (the reference's library GEMM fixes no order)."""
    from bitmtp_amd import decode_ops
    rng = np.random.default_rng(M * 131 + N + K)
    x = _rand_bf16(rng, (M, K), 1.0).to(DEV)
    w = _rand_bf16(rng, (N, K), 0.05).to(DEV)
    print(f"[case] bf16_linear M={M} N={N} K={K}", flush=True)
    got = decode_ops.bf16_linear(x, w)
    torch.cuda.synchronize()
    _assert_one_bf16_step(got, x.double() @ w.double().T)
    # a preallocated output with a wider leading dimension is rejected, wrong K as well
    with pytest.raises(RuntimeError):
        decode_ops.bf16_linear(x, w[:, : K - 64].contiguous() if K > 64 else w[:, :32].contiguous())


# ---------------------------------------------------------------- FP8 draft projection
@pytest.mark.parametrize("M,K", [(1, 128), (8, 2048), (17, 2560), (3, 264)])
def test_fp8_row_quantiser_matches_torch_cast(M, K):
    """scale and codes are the reference's tensor expression (model.py:1269-1270) evaluated
    by this build's own PyTorch on the CPU, bit for bit."""
    from bitmtp_amd import decode_ops
    rng = np.random.default_rng(M + K)
    x = _rand_bf16(rng, (M, K), 3.0)
    x[0, :8] = torch.tensor([0.0, -0.0, 1e-4, -1e-4, 2e-3, 7.0, -7.0, 0.013], dtype=torch.bfloat16)
    print(f"[case] fp8_quant_rows M={M} K={K}", flush=True)
    q, s = decode_ops.fp8_quant_rows(x.to(DEV))
    torch.cuda.synchronize()
    h_scale = (x.abs().amax() / 448.0).clamp_min(1e-12).to(torch.float32)
    want = (x / h_scale).to(torch.float8_e4m3fn).view(torch.uint8)
    assert s.cpu().item() == h_scale.item()
    got = q.cpu()
    # -0 and +0 results are the same value; everything else is the same code
    same = (got == want) | (((got | want) & 0x7F) == 0)
    assert bool(same.all())
    # an all-zero tensor takes the clamp: scale bf16(1e-12), codes zero
    q0, s0 = decode_ops.fp8_quant_rows(torch.zeros(2, 128, dtype=torch.bfloat16, device=DEV))
    assert s0.cpu().item() == torch.tensor(1e-12).to(torch.bfloat16).float().item()
    assert int(q0.cpu().max()) == 0


@pytest.mark.parametrize("M,N,K", [(1, 1008, 512), (8, 4112, 2048), (16, 1536, 2560), (17, 304, 128),
                                   (9, 151936, 2048)])
def test_fp8_linear_against_float64_product(M, N, K):
    from bitmtp_amd import decode_ops
    rng = np.random.default_rng(M * 7 + N + K)
    w = _rand_bf16(rng, (N - 5, K), 0.03).to(DEV)
    x = _rand_bf16(rng, (M, K), 2.0).to(DEV)
    w_q, w_scale = decode_ops.prepare_fp8_weight(w)
    assert tuple(w_q.shape) == (N, K) and w_q.dtype == torch.uint8      # rows padded to 16
    assert bool((w_q[N - 5:] == 0).all())
    x_q, x_scale = decode_ops.fp8_quant_rows(x)
    print(f"[case] fp8_linear M={M} N={N} K={K}", flush=True)
    got = decode_ops.fp8_linear(x_q, x_scale, w_q, w_scale)
    torch.cuda.synchronize()
    xf = x_q.view(torch.float8_e4m3fn).double()
    wf = w_q.view(torch.float8_e4m3fn).double()
    want = (xf @ wf.T) * float(x_scale.item()) * w_scale
    _assert_one_bf16_step(got, want)
    # and the FP8 projection approximates the bf16 one it stands in for
    exact = x.double() @ torch.cat([w, torch.zeros(5, K, dtype=w.dtype, device=DEV)]).double().T
    assert (got.double() - exact).abs().max().item() <= 0.08 * exact.abs().max().item()


# ---------------------------------------------------------------- whole step and loops
def _tiny_args(**over):
    from bitmtp_amd.model import ModelArgs
    base = dict(dim=512, n_layers=2, n_heads=4, n_kv_heads=2, ffn_dim=1024, vocab_size=1000,
                mask_token_id=999)
    base.update(over)
    return ModelArgs(**base)


@pytest.fixture(scope="module")
def tiny():
    from bitmtp_amd.model import BonsaiDecoder
    from bitmtp_amd.runtime import GraphAtlas
    model = BonsaiDecoder.random_init(_tiny_args(), seed=11, device=DEV)
    atlas = GraphAtlas(model, segment_ladder=(64, 256), threshold=0.9)
    return model, atlas


def _oracle_weights(model, atlas):
    def pl(p):
        return (p.weight.cpu().numpy().view(np.uint8), bf16_bits(p.weight_scale))
    a = model.args
    head = {"head": pl(model.head), "head_bits": model.head.bits} if model.head is not None \
        else {"head_bf16": bf16_bits(model.head_bf16)}
    return {
        "embed": bf16_bits(model.embed), "norm": bf16_bits(model.norm), **head,
        "bits": model.layers[0].wqkv.bits,
        "cos": bf16_bits(atlas.rope[0]), "sin": bf16_bits(atlas.rope[1]), "eps": a.norm_eps,
        "n_heads": a.n_heads, "n_kv": a.n_kv_heads,
        "layers": [{
            "wqkv": pl(l.wqkv), "wo": pl(l.wo), "w_gu": pl(l.w_gu), "w_down": pl(l.w_down),
            "input_layernorm": bf16_bits(l.input_layernorm),
            "post_attention_layernorm": bf16_bits(l.post_attention_layernorm),
            "q_norm": bf16_bits(l.q_norm), "k_norm": bf16_bits(l.k_norm)} for l in model.layers],
    }


@pytest.mark.parametrize("role,M,n_pend", [("ar", 1, 0), ("verify", 9, 0), ("draft", 12, 3),
                                           ("ar", 16, 0)])
def test_captured_step_against_cpu_composition(DO, tiny, role, M, n_pend):
    from bitmtp_amd import runtime
    model, atlas = tiny
    sigma, cache_len = 64, 21
    rng = np.random.default_rng(M)
    kv = atlas.kv(sigma)
    kv.copy_(_rand_bf16(rng, tuple(kv.shape), 0.5).to(DEV))
    kv_bits = bf16_bits(kv)
    tokens = rng.integers(0, model.args.vocab_size, M).tolist()
    positions = [cache_len + i for i in range(M)]
    g = atlas.get_graph(M, sigma, role)
    print(f"step case {role} M={M}", flush=True)
    atlas.replay(g, tokens, positions, cache_len, n_pend=n_pend)
    toks, conf, accept = atlas.read_outputs(g)
    rows = g.logits_end - g.logits_start
    got = atlas.workspace.logits[:rows, : model.args.vocab_size].float().cpu().numpy()

    desc = runtime.step_descriptor(role, M, atlas.D, cache_len, n_pend)
    vis = runtime.dense_visibility(desc, M, sigma)
    kk, vv = kv_bits[0].copy(), kv_bits[1].copy()
    want_bits = DO.decode_step(_oracle_weights(model, atlas), kk, vv, tokens, positions, vis, sigma,
                               g.logits_start, g.logits_end)
    from oracle import oracle as O
    want = O.bf16_bits_to_f32(want_bits)[:, : model.args.vocab_size]
    tol = 6e-2 * np.abs(want).max()
    assert np.abs(got - want).max() <= tol
    # the K rows the step wrote: those of layer 0 do not pass through attention and agree with
    # the oracle's to the last place or two; deeper layers carry the bf16 rounding of the
    # attention probabilities (the reference rounds them too, the float64 oracle does not)
    new_k = bf16_bits(atlas.kv(sigma))[0][:, :, sigma:sigma + M]
    ref_k = kk[:, :, sigma:sigma + M]
    d = np.abs(bf16_ordinal(new_k[0]) - bf16_ordinal(ref_k[0]))
    assert np.quantile(d, 0.99) <= 2
    from oracle import oracle as O2
    dk = np.abs(O2.bf16_bits_to_f32(new_k) - O2.bf16_bits_to_f32(ref_k))
    assert dk.max() <= 6e-2 * np.abs(O2.bf16_bits_to_f32(ref_k)).max()
    # argmax / confidence outputs describe the logits the step produced
    wt, wc, wn = DO.draft_chain(got, atlas.threshold)
    assert toks.tolist() == wt.tolist()
    np.testing.assert_allclose(conf, wc, rtol=2e-3, atol=1e-6)
    assert accept == wn


def test_graph_replay_equals_eager_and_is_repeatable(tiny):
    from bitmtp_amd.runtime import GraphAtlas
    model, atlas = tiny
    eager = GraphAtlas(model, segment_ladder=(64, 256), use_graphs=False)
    rng = np.random.default_rng(5)
    sigma, cache_len, M = 64, 30, 9
    hist = _rand_bf16(rng, tuple(atlas.kv(sigma).shape), 0.5).to(DEV)
    tokens = rng.integers(0, 1000, M).tolist()
    positions = [cache_len - 1 + i for i in range(M)]
    outs = []
    for a in (atlas, eager, atlas, atlas):
        a.kv(sigma).copy_(hist)
        g = a.get_graph(M, sigma, "verify")
        a.replay(g, tokens, positions, cache_len)
        a.read_outputs(g)
        outs.append(a.workspace.logits[:M].clone())
        torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


def test_wide_causal_replay_matches_sequential_width_one(tiny):
    """Width-M AR-causal replay == M width-1 replays on the same tokens, within the
    accumulation-order differences of the two GEMV kernels."""
    model, atlas = tiny
    sigma, M = 64, 16
    rng = np.random.default_rng(9)
    tokens = rng.integers(0, 1000, M).tolist()
    atlas.kv(sigma).zero_()
    gw = atlas.get_graph(M, sigma, "ar")
    atlas.replay(gw, tokens, list(range(M)), 0)
    atlas.read_outputs(gw)
    wide = atlas.workspace.logits[:M, :1000].float().cpu().numpy()
    atlas.kv(sigma).zero_()
    g1 = atlas.get_graph(1, sigma, "ar")
    seq = []
    for i, t in enumerate(tokens):
        atlas.replay(g1, [t], [i], i)
        atlas.commit_kv(sigma, i, 1)
        atlas.read_outputs(g1)
        seq.append(atlas.workspace.logits[0, :1000].float().cpu().numpy())
    seq = np.stack(seq)
    assert np.abs(wide - seq).max() <= 6e-2 * np.abs(seq).max()


def test_hybrid_with_exact_verification_reproduces_ar(tiny):
    from bitmtp_amd import generate
    model, atlas = tiny
    rng = np.random.default_rng(21)
    prompt = rng.integers(0, 1000, 37).tolist()
    ar, st_ar = generate.ar_generate(atlas, prompt, max_gen_len=40)
    hy, st = generate.hybrid_generate(atlas, prompt, max_gen_len=40, exact_m1_verify=True)
    assert len(ar) == 40 and st_ar["timed_decode_tokens"] == 39
    assert hy == ar
    assert st["draft_iters"] == st["n_conf_path"] + st["n_verify_path"]
    assert st["decode_tokens"] == 1 + st["accepted_drafts"] + st["verifier_bonus_tokens"]


def test_prefill_width_does_not_change_the_tokens(tiny):
    """The prompt may be prefilled 16 or 32 rows at a time (AR-causal replays of the same
    kernels): the greedy continuation is the same."""
    from bitmtp_amd import generate
    from bitmtp_amd.runtime import GraphAtlas
    model, atlas = tiny
    assert atlas.prefill_width == 32
    narrow = GraphAtlas(model, segment_ladder=(64, 256), prefill_width=16)
    rng = np.random.default_rng(53)
    prompt = rng.integers(0, 1000, 45).tolist()
    a, _ = generate.ar_generate(atlas, prompt, max_gen_len=12)
    b, _ = generate.ar_generate(narrow, prompt, max_gen_len=12)
    assert a == b


def test_speculative_decode_always_verifies(tiny):
    """fast_generate.py:664-899: draft + verify every iteration; with the exact width-1
    verifier the tokens are the AR ones, with the width-(D+1) verifier every committed
    token is a verifier-approved draft or a verifier bonus."""
    from bitmtp_amd import generate
    model, atlas = tiny
    rng = np.random.default_rng(29)
    prompt = rng.integers(0, 1000, 23).tolist()
    ar, _ = generate.ar_generate(atlas, prompt, max_gen_len=30)
    sp, st = generate.speculative_generate(atlas, prompt, max_gen_len=30, exact_m1_verify=True)
    assert sp == ar
    assert st["n_conf_path"] == 0 and st["conf_path_frac"] == 0.0
    assert st["n_verify_path"] == st["draft_iters"] and st["drafted_tokens"] == 8 * st["draft_iters"]
    sp2, st2 = generate.speculative_generate(atlas, prompt, max_gen_len=30)
    assert len(sp2) == 30 and st2["n_conf_path"] == 0
    assert st2["decode_tokens"] == 1 + st2["accepted_drafts"] + st2["verifier_bonus_tokens"]
    assert sp2[0] == ar[0]


def test_confidence_decode(tiny):
    """fast_generate.py:393-572: blocks are committed on confidence alone.  Threshold 0
    commits whole blocks, an infinite threshold one token per iteration; the first block is
    drafted from the last prompt token, so its first token is the AR one."""
    from bitmtp_amd import generate
    model, atlas = tiny
    rng = np.random.default_rng(41)
    prompt = rng.integers(0, 1000, 27).tolist()
    ar, _ = generate.ar_generate(atlas, prompt, max_gen_len=4)
    full, st = generate.confidence_generate(atlas, prompt, threshold=0.0, max_gen_len=50)
    assert len(full) == 50 and full[0] == ar[0]
    assert st["n_iters"] == 7 and st["untimed_output_tokens"] == 8       # 6 x 8 + 2
    assert st["timed_decode_tokens"] == 42 and st["n_verify_path"] == 0 and st["conf_path_frac"] == 1.0
    assert st["drafted_tokens"] == 8 * st["n_iters"] and st["accepted_drafts"] == 50
    again, _ = generate.confidence_generate(atlas, prompt, threshold=0.0, max_gen_len=50)
    assert again == full
    one, st1 = generate.confidence_generate(atlas, prompt, threshold=float("inf"), max_gen_len=12)
    assert len(one) == 12 and st1["n_iters"] == 12 and st1["untimed_output_tokens"] == 1
    assert one[0] == full[0]
    # an EOS inside the first block ends the run in front of it
    cut, stc = generate.confidence_generate(atlas, prompt, threshold=0.0, max_gen_len=50,
                                            eos_ids=[full[3]])
    assert cut == full[:full.index(full[3])] and stc["n_iters"] == 1


@pytest.mark.parametrize("threshold,hybrid_m", [(0.9, None), (0.0, 1), (0.0, 8)])
def test_hybrid_accounting_and_width_schedule(tiny, threshold, hybrid_m):
    from bitmtp_amd import generate
    model, atlas = tiny
    rng = np.random.default_rng(22)
    prompt = rng.integers(0, 1000, 50).tolist()
    before = set(atlas.graphs)
    out, st = generate.hybrid_generate(atlas, prompt, threshold=threshold, hybrid_m=hybrid_m,
                                       max_gen_len=64)
    assert len(out) == 64 and all(0 <= t < 1000 for t in out)
    assert st["n_iters"] == st["draft_iters"] + 1
    assert st["drafted_tokens"] == 8 * st["draft_iters"]
    assert st["committed_tokens"] == 63 == st["timed_decode_tokens"]
    if threshold == 0.0:
        # every confidence passes: whole blocks are committed and re-forwarded as 8 pending rows
        assert st["n_verify_path"] == 0 and st["committed_per_iter"] > 7
        assert (16, 64, "draft") in atlas.graphs or (16, 256, "draft") in atlas.graphs
    else:
        # near-uniform random logits never pass 0.9: draft(9) + verify(9) every iteration
        # (the last bonus may be clipped by max_gen_len)
        assert st["n_conf_path"] == 0
        assert st["n_verify_path"] - 1 <= st["verifier_bonus_tokens"] <= st["n_verify_path"]


def test_eos_stops_generation(tiny):
    from bitmtp_amd import generate
    model, atlas = tiny
    prompt = list(range(3, 30))
    ar, _ = generate.ar_generate(atlas, prompt, max_gen_len=24)
    eos = ar[10]
    first = ar.index(eos)
    cut, st = generate.ar_generate(atlas, prompt, max_gen_len=24, eos_ids=[eos])
    assert cut == ar[:first]
    hy, _ = generate.hybrid_generate(atlas, prompt, max_gen_len=24, eos_ids=[eos],
                                     exact_m1_verify=True)
    assert hy == ar[:first]


def test_segment_migration_keeps_the_sequence(tiny):
    """Moving the live history to a larger segment's buffer (fast_runtime.py:510-521) and
    decoding on from there gives the same tokens as staying put."""
    from bitmtp_amd import generate
    model, atlas = tiny
    prompt = list(range(11, 29))
    ar, _ = generate.ar_generate(atlas, prompt, max_gen_len=12)       # lives in segment 64
    assert atlas.select_segment(len(prompt) + 12 + atlas.M_max) == 64
    # replay the same decode by hand, migrating 64 -> 256 after four tokens
    sigma = 64
    tok = generate.prefill(atlas, prompt, sigma)
    cache_len = len(prompt)
    out = [tok]
    for step in range(11):
        if step == 4:
            atlas.migrate_segment(sigma, 256, cache_len)
            sigma = 256
        g = atlas.get_graph(1, sigma, "ar")
        atlas.replay(g, [tok], [cache_len], cache_len)
        atlas.commit_kv(sigma, cache_len, 1)
        cache_len += 1
        toks, _, _ = atlas.read_outputs(g)
        tok = int(toks[0])
        out.append(tok)
    assert out == ar


def test_replay_argument_checks(tiny):
    model, atlas = tiny
    g = atlas.get_graph(9, 64, "verify")
    with pytest.raises(ValueError):
        atlas.replay(g, [1, 2, 3], [0, 1, 2], 5)
    with pytest.raises(RuntimeError, match="committed anchor"):
        atlas.replay(g, [1] * 9, list(range(9)), 0)
    with pytest.raises(RuntimeError):
        atlas.replay(g, [1] * 9, list(range(9)), 65)
    with pytest.raises(RuntimeError):
        atlas.commit_kv(64, 60, 9)
    with pytest.raises(ValueError):
        atlas.get_graph(4, 64, "draft")
    with pytest.raises(KeyError):
        atlas.kv(100)


# ---------------------------------------------------------------- sign-weight (Q1) backbone
@pytest.fixture(scope="module", params=["bf16", "q1"])
def tiny_q1(request):
    """A "q1" backbone with the bf16 output projection the reference's graphs use for it
    (fast_runtime.py:175-178) and with the sign-packed W1A8 projection (model.py:1262-1267)."""
    from bitmtp_amd.model import BonsaiDecoder
    from bitmtp_amd.runtime import GraphAtlas
    model = BonsaiDecoder.random_init(_tiny_args(kernel_kind="q1"), seed=13, device=DEV,
                                      head_kind=request.param)
    assert model.head_kind == request.param and model.layers[0].wo.bits == 1
    atlas = GraphAtlas(model, segment_ladder=(64, 256), threshold=0.9)
    return model, atlas


@pytest.mark.parametrize("role,M,n_pend", [("ar", 1, 0), ("verify", 9, 0), ("draft", 12, 3)])
def test_q1_step_against_cpu_composition(DO, tiny_q1, role, M, n_pend):
    from bitmtp_amd import runtime
    from oracle import oracle as O
    model, atlas = tiny_q1
    sigma, cache_len = 64, 17
    rng = np.random.default_rng(100 + M)
    kv = atlas.kv(sigma)
    kv.copy_(_rand_bf16(rng, tuple(kv.shape), 0.5).to(DEV))
    kv_bits = bf16_bits(kv)
    tokens = rng.integers(0, model.args.vocab_size, M).tolist()
    positions = [cache_len + i for i in range(M)]
    g = atlas.get_graph(M, sigma, role)
    print(f"q1 step case head={model.head_kind} {role} M={M}", flush=True)
    atlas.replay(g, tokens, positions, cache_len, n_pend=n_pend)
    toks, conf, accept = atlas.read_outputs(g)
    rows = g.logits_end - g.logits_start
    got = atlas.workspace.logits[:rows, : model.args.vocab_size].float().cpu().numpy()
    desc = runtime.step_descriptor(role, M, atlas.D, cache_len, n_pend)
    vis = runtime.dense_visibility(desc, M, sigma)
    kk, vv = kv_bits[0].copy(), kv_bits[1].copy()
    want_bits = DO.decode_step(_oracle_weights(model, atlas), kk, vv, tokens, positions, vis, sigma,
                               g.logits_start, g.logits_end)
    want = O.bf16_bits_to_f32(want_bits)[:, : model.args.vocab_size]
    assert np.abs(got - want).max() <= 6e-2 * np.abs(want).max()
    wt, wc, wn = DO.draft_chain(got, atlas.threshold)
    assert toks.tolist() == wt.tolist() and accept == wn
    np.testing.assert_allclose(conf, wc, rtol=2e-3, atol=1e-6)


def test_q1_hybrid_with_exact_verification_reproduces_ar(tiny_q1):
    from bitmtp_amd import generate
    model, atlas = tiny_q1
    rng = np.random.default_rng(23)
    prompt = rng.integers(0, 1000, 29).tolist()
    ar, _ = generate.ar_generate(atlas, prompt, max_gen_len=32)
    hy, st = generate.hybrid_generate(atlas, prompt, max_gen_len=32, exact_m1_verify=True)
    assert len(ar) == 32 and hy == ar
    assert st["draft_iters"] == st["n_conf_path"] + st["n_verify_path"]
    # replays of a captured bf16-head graph are repeatable (no stale state in the graph)
    again, _ = generate.ar_generate(atlas, prompt, max_gen_len=32)
    assert again == ar


def test_decoder_rejects_mixed_weight_kinds():
    from bitmtp_amd.model import BonsaiDecoder
    model = BonsaiDecoder.random_init(_tiny_args(), seed=3, device=DEV)
    with pytest.raises(ValueError):
        BonsaiDecoder(_tiny_args(kernel_kind="q1"), model.layers, model.embed, model.norm, None)
    with pytest.raises(ValueError):
        BonsaiDecoder.random_init(_tiny_args(kernel_kind="w4"), seed=3, device=DEV)


# ---------------------------------------------------------------- approximate draft roles
@pytest.mark.parametrize("kind", ["t2g128", "q1"])
def test_fp8_and_bf16_draft_roles(kind):
    """The acceptance-tolerant draft projections (fast_runtime.py:188-199): their logits stay
    close to the native ones, verification stays native, so hybrid decode with exact width-1
    verification still reproduces AR token for token, and a role that was not requested for
    the atlas is refused."""
    from bitmtp_amd import generate
    from bitmtp_amd.model import BonsaiDecoder
    from bitmtp_amd.runtime import GraphAtlas
    model = BonsaiDecoder.random_init(_tiny_args(kernel_kind=kind), seed=17, device=DEV)
    atlas = GraphAtlas(model, segment_ladder=(64, 256), threshold=0.9,
                       roles=("ar", "draft", "draft_fp8", "draft_bf16", "verify"))
    assert model.head_fp8[0].shape == (1008, 512) and model.head_raw_bf16.shape == (1000, 512)
    rng = np.random.default_rng(31)
    sigma, cache_len, M = 64, 19, 9
    hist = _rand_bf16(rng, tuple(atlas.kv(sigma).shape), 0.5).to(DEV)
    tokens = rng.integers(0, 1000, M).tolist()
    positions = [cache_len + i for i in range(M)]
    logits = {}
    for role in ("draft", "draft_fp8", "draft_bf16"):
        atlas.kv(sigma).copy_(hist)
        g = atlas.get_graph(M, sigma, role)
        print(f"[case] {kind} role {role}", flush=True)
        for _ in range(2):   # a replay after the first gives the same result
            atlas.replay(g, tokens, positions, cache_len, n_pend=1)
            toks, conf, accept = atlas.read_outputs(g)
            rows = g.logits_end - g.logits_start
            ld = {"draft": model.head_rows, "draft_fp8": 1008, "draft_bf16": 1000}[role]
            cur = atlas.workspace.logits_view(rows, ld)[:, :1000].float().cpu().numpy()
            if role in logits:
                assert np.array_equal(cur, logits[role])
            logits[role] = cur
            assert toks.tolist() == cur.argmax(-1).tolist()
    ref = logits["draft"]
    scale = np.abs(ref).max()
    assert np.abs(logits["draft_bf16"] - ref).max() <= 0.05 * scale
    assert np.abs(logits["draft_fp8"] - ref).max() <= 0.12 * scale
    prompt = rng.integers(0, 1000, 21).tolist()
    ar, _ = generate.ar_generate(atlas, prompt, max_gen_len=24)
    for kw in ({"use_fp8_draft": True}, {"use_bf16_draft": True}):
        hy, st = generate.hybrid_generate(atlas, prompt, max_gen_len=24, exact_m1_verify=True, **kw)
        assert hy == ar
    plain = GraphAtlas(model, segment_ladder=(64,))
    with pytest.raises(RuntimeError, match="not captured"):
        generate.hybrid_generate(plain, prompt, max_gen_len=4, use_fp8_draft=True)
