"""GPU tests at the real model sizes of the end-to-end benchmark configurations: the
1.7B-shaped (28 layers, hidden 2048, sigma 1024) and the 4B-shaped (36 layers, hidden 2560,
32 query heads, sigma 4096) random-init ternary decoders, block 8.

What the reference checks by hand on a GPU (docs/testing.md:11-15, fast_generate.py:611-657):
speculation with the exact width-1 verifier reproduces greedy AR token for token; the
accounting identities of fast_generate.py:1151-1162 hold.  Added here: a captured width-9
step equals the same step enqueued eagerly, bit for bit, and one step of a two-layer model at
the real dimensions against the CPU composition of the oracles, where everything in front of
the first attention (merged q|k|v GEMV output through q/k norm, RoPE and the KV write) must
agree with the oracle to the last place and the logits to a tolerance far tighter than the
tiny-model test needs.  Also: the block-4 schedule (widths {1,4,5,6,7,8,9},
src/bonsai_sft/gpu/run_generation.py:74-75) on the small model, the W1A16 entry point against
a float64 product, and the sign-weight layer set at the widths the other tests leave out.
"""
import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, bf16_ordinal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _args(name, **over):
    from bitmtp_amd.model import qwen3_1p7b_args, qwen3_4b_args
    return (qwen3_1p7b_args if name == "1.7b" else qwen3_4b_args)(**over)


@pytest.fixture(scope="module", params=["1.7b", "4b"])
def full(request):
    from bitmtp_amd.model import BonsaiDecoder
    from bitmtp_amd.runtime import GraphAtlas
    name = request.param
    sigma = 1024 if name == "1.7b" else 4096
    print(f"[case] building the {name}-shaped decoder, sigma={sigma}", flush=True)
    model = BonsaiDecoder.random_init(_args(name), seed=3, device=DEV)
    atlas = GraphAtlas(model, segment_ladder=(sigma,), threshold=0.9)
    yield name, sigma, model, atlas
    del atlas, model
    torch.cuda.empty_cache()


def test_exact_verification_reproduces_ar_at_full_size(full):
    from bitmtp_amd import generate
    name, sigma, model, atlas = full
    n_prompt, n_new = (256, 72) if name == "1.7b" else (512, 64)
    rng = np.random.default_rng(17)
    prompt = rng.integers(0, model.args.vocab_size, n_prompt).tolist()
    print(f"[case] {name}: AR {n_new} tokens from a {n_prompt}-token prompt", flush=True)
    ar, st_ar = generate.ar_generate(atlas, prompt, max_gen_len=n_new)
    assert len(ar) == n_new and st_ar["timed_decode_tokens"] == n_new - 1
    print(f"[case] {name}: hybrid with exact width-1 verification", flush=True)
    hy, st = generate.hybrid_generate(atlas, prompt, max_gen_len=n_new, exact_m1_verify=True)
    assert hy == ar
    assert st["draft_iters"] == st["n_conf_path"] + st["n_verify_path"]
    assert st["decode_tokens"] == 1 + st["accepted_drafts"] + st["verifier_bonus_tokens"]
    assert st["drafted_tokens"] == 8 * st["draft_iters"]
    # the production schedule (width-9 verifier): every identity still holds
    print(f"[case] {name}: hybrid, threshold 0.9", flush=True)
    out, st2 = generate.hybrid_generate(atlas, prompt, threshold=0.9, max_gen_len=n_new)
    assert len(out) == n_new and out[0] == ar[0]
    assert st2["n_iters"] == st2["draft_iters"] + 1
    assert st2["committed_tokens"] == n_new - 1 == st2["timed_decode_tokens"]
    assert st2["decode_tokens"] == 1 + st2["accepted_drafts"] + st2["verifier_bonus_tokens"]


def test_ar_tokens_do_not_depend_on_the_layer_form_at_full_size(full, monkeypatch):
    """Greedy AR decoding at full size through the ten-launch layer, the fused layer with the
    attention's merge as a launch of its own and the fused layer with the self-merging attention:
    the same tokens and the same logits bits after the last step."""
    from bitmtp_amd import generate
    from bitmtp_amd.runtime import GraphAtlas
    name, sigma, model, _ = full
    n_prompt, n_new = (256, 200) if name == "1.7b" else (1000, 120)
    prompt = np.random.default_rng(29).integers(0, model.args.vocab_size, n_prompt).tolist()
    runs = []
    for fused, one_launch in (("0", "1"), ("1", "0"), ("1", "1")):
        monkeypatch.setenv("BONSAI_FUSED_STEP", fused)
        monkeypatch.setenv("BONSAI_ATTENTION_ONE_LAUNCH", one_launch)
        atlas = GraphAtlas(model, segment_ladder=(sigma,), threshold=0.9, roles=("ar",))
        print(f"[case] {name}: AR {n_new} tokens, BONSAI_FUSED_STEP={fused} "
              f"BONSAI_ATTENTION_ONE_LAUNCH={one_launch}", flush=True)
        toks, _ = generate.ar_generate(atlas, prompt, max_gen_len=n_new)
        runs.append((toks, atlas.workspace.logits[:1].clone()))
        del atlas
    for toks, logits in runs[1:]:
        assert toks == runs[0][0]
        assert torch.equal(logits.view(torch.int16), runs[0][1].view(torch.int16))


def test_graph_replay_equals_eager_at_full_size(full):
    from bitmtp_amd.runtime import GraphAtlas
    name, sigma, model, atlas = full
    eager = GraphAtlas(model, segment_ladder=(sigma,), use_graphs=False)
    rng = np.random.default_rng(5)
    M, cache_len = 9, sigma // 2 + 3
    hist = (torch.randn(tuple(atlas.kv(sigma).shape), device=DEV) * 0.5).to(torch.bfloat16)
    tokens = rng.integers(0, model.args.vocab_size, M).tolist()
    positions = [cache_len - 1 + i for i in range(M)]
    outs = []
    for a in (atlas, eager, atlas):
        print(f"[case] {name}: width-9 verify step, graphs={a.use_graphs}", flush=True)
        a.kv(sigma).copy_(hist)
        g = a.get_graph(M, sigma, "verify")
        a.replay(g, tokens, positions, cache_len)
        toks, conf, accept = a.read_outputs(g)
        outs.append((a.workspace.logits[:M].clone(), toks.copy(), conf.copy()))
        torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o[0], outs[0][0])
        assert np.array_equal(o[1], outs[0][1]) and np.array_equal(o[2], outs[0][2])
    del eager


def _oracle_weights(model, atlas):
    def pl(p):
        return (p.weight.cpu().numpy().view(np.uint8), bf16_bits(p.weight_scale))
    a = model.args
    return {
        "embed": bf16_bits(model.embed), "norm": bf16_bits(model.norm), "head": pl(model.head),
        "head_bits": model.head.bits, "bits": model.layers[0].wqkv.bits,
        "cos": bf16_bits(atlas.rope[0]), "sin": bf16_bits(atlas.rope[1]), "eps": a.norm_eps,
        "n_heads": a.n_heads, "n_kv": a.n_kv_heads,
        "layers": [{
            "wqkv": pl(l.wqkv), "wo": pl(l.wo), "w_gu": pl(l.w_gu), "w_down": pl(l.w_down),
            "input_layernorm": bf16_bits(l.input_layernorm),
            "post_attention_layernorm": bf16_bits(l.post_attention_layernorm),
            "q_norm": bf16_bits(l.q_norm), "k_norm": bf16_bits(l.k_norm)} for l in model.layers],
    }


@pytest.mark.parametrize("name", ["1.7b", "4b"])
def test_two_layer_step_at_real_dims_stage_by_stage(name):
    """Two layers of the real width and the real head.  The whole step is compared with the
    CPU composition of the oracles, and -- much sharper -- every stage of the LAST layer and of
    the head with the oracle applied to the GPU's own input of that stage, which the step's
    workspace still holds.  A wiring mistake (a swapped norm weight, a missing residual, the
    wrong rows into the head) shows at its stage in full size, while the unavoidable
    differences stay what they are at their source: the GEMVs' fp32 summation order (the
    neighbouring bf16 value at most) and the attention (bf16 probabilities and fp32 sums here,
    float64 in the oracle: one quantisation step on a few elements)."""
    from oracle import decode_oracle as DO
    from oracle import oracle as O
    from bitmtp_amd import runtime
    from bitmtp_amd.model import BonsaiDecoder
    from bitmtp_amd.runtime import GraphAtlas
    O.build()
    sigma, cache_len, M, role = 256, 131, 9, "verify"
    model = BonsaiDecoder.random_init(_args(name, n_layers=2), seed=5, device=DEV)
    atlas = GraphAtlas(model, segment_ladder=(sigma,), threshold=0.9)
    a = model.args
    rng = np.random.default_rng(3)
    kv = atlas.kv(sigma)
    kv.copy_((torch.randn(tuple(kv.shape), device=DEV) * 0.5).to(torch.bfloat16))
    kv_bits = bf16_bits(kv)
    tokens = rng.integers(0, a.vocab_size, M).tolist()
    positions = [cache_len + i for i in range(M)]
    g = atlas.get_graph(M, sigma, role)
    print(f"[case] {name} two-layer step M={M}", flush=True)
    atlas.replay(g, tokens, positions, cache_len)
    toks, conf, accept = atlas.read_outputs(g)
    rows = g.logits_end - g.logits_start
    V = a.vocab_size
    ws = atlas.workspace
    got_bits = bf16_bits(ws.logits[:rows])
    got = O.bf16_bits_to_f32(got_bits)[:, :V]

    # ---- the whole step against the composition of the oracles
    desc = runtime.step_descriptor(role, M, atlas.D, cache_len, 0)
    vis = runtime.dense_visibility(desc, M, sigma)
    kk, vv = kv_bits[0].copy(), kv_bits[1].copy()
    W = _oracle_weights(model, atlas)
    want_bits = DO.decode_step(W, kk, vv, tokens, positions, vis, sigma, g.logits_start, g.logits_end)
    want = O.bf16_bits_to_f32(want_bits)[:, :V]
    new = bf16_bits(atlas.kv(sigma))
    for plane, ref in ((0, kk), (1, vv)):
        # layer 0's new K and V rows have not passed through attention: the oracle's, or the
        # neighbouring bf16 value where the GEMV's fp32 summation order shows
        d = np.abs(bf16_ordinal(new[plane][0][:, sigma:sigma + M]) -
                   bf16_ordinal(ref[0][:, sigma:sigma + M]))
        assert d.max() <= 1 and (d != 0).mean() < 0.02, (plane, d.max(), (d != 0).mean())
    err = np.abs(got - want).max() / np.abs(want).max()
    rms = np.sqrt(np.mean((got - want) ** 2)) / np.sqrt(np.mean(want ** 2))
    print(f"[info] {name}: whole step max err / max = {err:.3e}, rms err / rms = {rms:.3e}", flush=True)
    assert err <= 1e-1 and rms <= 1e-1

    # ---- the last layer and the head, stage by stage, on the GPU's own stage inputs
    def gemv_ok(label, out_t, q_t, s_t, w):
        _, ref = O.c_gemv(q_t[:M].cpu().numpy(), w[0], s_t[:M].cpu().numpy(), w[1], 2)
        d = np.abs(bf16_ordinal(bf16_bits(out_t[:M])) - bf16_ordinal(ref))
        assert d.max() <= 1, f"{label}: {d.max()} bf16 steps from the oracle"

    def quant_ok(label, q_t, s_t, q_ref, s_ref, n=M, flips=0.0):
        q, s_ = q_t[:n].cpu().numpy(), s_t[:n].cpu().numpy()
        assert np.array_equal(s_, s_ref), f"{label}: activation multipliers differ"
        dq = np.abs(q.astype(np.int32) - q_ref.astype(np.int32))
        assert dq.max() <= (1 if flips else 0) and (dq != 0).mean() <= flips, \
            f"{label}: max |dq| {dq.max()}, {(dq != 0).mean():.2e} of the elements"

    lw = W["layers"][1]
    eps = a.norm_eps
    h_in = bf16_bits(ws.h[0][:M])          # residual stream entering layer 1's attention
    h_mid = bf16_bits(ws.h[1][:M])         # ... after the attention block
    a_q, a_s, _ = O.c_rmsnorm_quant(h_in, lw["input_layernorm"], eps)
    quant_ok("input norm", ws.a_q, ws.a_s, a_q, a_s)
    gemv_ok("q|k|v", ws.xqkv, ws.a_q, ws.a_s, lw["wqkv"])
    xqkv = bf16_bits(ws.xqkv[:M])
    q, k, v = DO.qk_norm_rope(xqkv, lw["q_norm"], lw["k_norm"], eps, W["cos"], W["sin"], positions,
                              a.n_heads, a.n_kv_heads)
    assert np.array_equal(bf16_bits(ws.q[:M]), q)
    assert np.array_equal(new[0][1][:, sigma:sigma + M], k.transpose(1, 0, 2))
    assert np.array_equal(new[1][1][:, sigma:sigma + M], v.transpose(1, 0, 2))
    att = DO.attention(q, new[0][1], new[1][1], vis, 1.0 / np.sqrt(128))
    o_q, o_s = O.c_act_quant(O.bf16_bits_to_f32(O.f32_to_bf16_bits(att.astype(np.float32))))
    gq, gs = ws.o_q[:M].cpu().numpy().astype(np.int32), ws.o_s[:M].cpu().numpy()
    assert np.allclose(gs, o_s, rtol=1e-2)
    dq = np.abs(gq - np.rint(att * gs[:, None]).clip(-128, 127))
    assert dq.max() <= 1 and (dq != 0).mean() < 0.05, (dq.max(), (dq != 0).mean())
    gemv_ok("o_proj", ws.attn_out, ws.o_q, ws.o_s, lw["wo"])
    f_q, f_s, h_ref = O.c_rmsnorm_quant(h_in, lw["post_attention_layernorm"], eps,
                                        residual_bits=bf16_bits(ws.attn_out[:M]))
    assert np.array_equal(h_mid, h_ref), "residual add after attention"
    quant_ok("post-attention norm", ws.f_q, ws.f_s, f_q, f_s)
    gemv_ok("gate|up", ws.gu, ws.f_q, ws.f_s, lw["w_gu"])
    i_q, i_s = O.c_silu_mul_quant(bf16_bits(ws.gu[:M]))
    # (the sigmoid runs on the transcendental unit: a value may cross a bf16 rounding boundary,
    # one quantisation step on a handful of elements; the multiplier moves only if that
    # happens to a row's largest element)
    gi_s = ws.i_s[:M].cpu().numpy()
    assert np.all(np.abs(gi_s - i_s) <= 1e-2 * np.abs(i_s))
    same = gi_s == i_s
    dq = np.abs(ws.i_q[:M].cpu().numpy().astype(np.int32) - i_q.astype(np.int32))
    assert dq.max() <= 1 and (not same.any() or (dq[same] != 0).mean() <= 1e-3)
    gemv_ok("down", ws.ffn_out, ws.i_q, ws.i_s, lw["w_down"])
    ls, le = g.logits_start, g.logits_end
    l_q, l_s, _ = O.c_rmsnorm_quant(bf16_bits(ws.ffn_out[ls:le]), W["norm"], eps, residual_bits=h_mid[ls:le])
    quant_ok("final norm", ws.l_q, ws.l_s, l_q, l_s, n=rows)
    _, ref_logits = O.c_gemv(ws.l_q[:rows].cpu().numpy(), W["head"][0], ws.l_s[:rows].cpu().numpy(),
                             W["head"][1], 2)
    d = np.abs(bf16_ordinal(got_bits) - bf16_ordinal(ref_logits))
    assert d.max() <= 1, f"head: {d.max()} bf16 steps from the oracle"
    # argmax / confidence describe the logits the step produced
    wt, wc, wn = DO.draft_chain(got, atlas.threshold)
    assert np.asarray(toks)[:rows].tolist() == wt.tolist()
    np.testing.assert_allclose(conf[:rows], wc, rtol=2e-3, atol=1e-6)
    assert accept == wn
    del atlas, model
    torch.cuda.empty_cache()


def test_block4_hybrid_with_exact_verification_reproduces_ar():
    """D4: block 4, captured widths {1,4,5,6,7,8,9} (run_generation.py:74-75)."""
    from bitmtp_amd import generate
    from bitmtp_amd.model import BonsaiDecoder, ModelArgs
    from bitmtp_amd.runtime import GraphAtlas
    args = ModelArgs(dim=512, n_layers=2, n_heads=4, n_kv_heads=2, ffn_dim=1024, vocab_size=1000,
                     mask_token_id=999, block_size=4)
    model = BonsaiDecoder.random_init(args, seed=11, device=DEV)
    atlas = GraphAtlas(model, segment_ladder=(64, 256), m_set=(1, 4, 5, 6, 7, 8, 9), threshold=0.9)
    assert atlas.D == 4
    rng = np.random.default_rng(21)
    prompt = rng.integers(0, 1000, 37).tolist()
    print("[case] block-4 AR / hybrid exact / hybrid thr 0.9 / thr 0", flush=True)
    ar, _ = generate.ar_generate(atlas, prompt, max_gen_len=40)
    hy, st = generate.hybrid_generate(atlas, prompt, max_gen_len=40, exact_m1_verify=True)
    assert hy == ar
    assert st["drafted_tokens"] == 4 * st["draft_iters"]
    assert st["draft_iters"] == st["n_conf_path"] + st["n_verify_path"]
    assert st["decode_tokens"] == 1 + st["accepted_drafts"] + st["verifier_bonus_tokens"]
    out, st2 = generate.hybrid_generate(atlas, prompt, threshold=0.9, max_gen_len=40)
    assert len(out) == 40 and st2["committed_tokens"] == 39
    assert all(k[0] in (1, 4, 5, 6, 7, 8, 9, 32) for k in atlas.graphs)   # 32 = prefill width
    full, st3 = generate.hybrid_generate(atlas, prompt, threshold=0.0, hybrid_m=1, max_gen_len=40)
    assert len(full) == 40 and st3["n_verify_path"] == 0 and st3["committed_per_iter"] > 3
    sp, _ = generate.speculative_generate(atlas, prompt, max_gen_len=40, exact_m1_verify=True)
    assert sp == ar


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (3, 1000, 2560), (4, 2560, 2560), (9, 333, 9728),
                                   (17, 16, 1024)])
def test_w1a16_against_float64_product(oracle, M, N, K):
    """`q1g128_w1a16_linear`: sign weights times bf16 activations, fp32 accumulation, no
    activation scale.  Against sum_g ws[n][g] * sum_k a[m][k] * w[n][k] in float64; fp32
    accumulation over K = 9728 terms: a relative error of a few 1e-4 of the row's scale
    before the bf16 rounding (2^-9 relative)."""
    import bitmtp_amd as ops
    rng = np.random.default_rng(M * 7 + N + K)
    p = oracle.synth_problem(31 + M + N, M, N, K, 1)
    x = torch.from_numpy(rng.normal(0, 1.0, (M, K)).astype(np.float32)).to(torch.bfloat16)
    B = torch.from_numpy(p["B"].view(np.int8)).to(DEV)
    ws = torch.from_numpy(p["ws"].view(np.int16).copy()).view(torch.bfloat16).to(DEV)
    print(f"[case] w1a16 M={M} N={N} K={K}", flush=True)
    y = ops.q1g128_w1a16_linear(x.to(DEV), B, ws)
    torch.cuda.synchronize()
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    W = oracle.np_unpack(p["B"], 1).astype(np.float64) * np.repeat(
        oracle.bf16_bits_to_f32(p["ws"]).astype(np.float64), 128, axis=1)
    ref = x.double().numpy() @ W.T
    got = y.float().cpu().numpy()
    mag = np.abs(x.double().numpy()) @ np.abs(W).T          # bound on any partial sum
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-5 * mag)


@pytest.mark.parametrize("M", [2, 4, 5, 6, 7])
@pytest.mark.parametrize("N,K", [(1024, 2560), (2560, 2560), (9728, 2560), (1024, 9728),
                                 (2560, 9728), (9728, 9728)])
def test_q1_4b_shapes_full_size_other_widths(oracle, M, N, K):
    """The sign-weight layer set at the widths 2, 4, 5, 6, 7 (1, 3 and 8 are covered beside
    the ternary layer shapes)."""
    from test_gpu_parity import check_problem
    p = oracle.synth_problem(40 + M, M, N, K, 1)
    check_problem(oracle, p, 1, "q1-4B")
