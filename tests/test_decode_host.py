"""Host logic of the decode harness and the decode oracle, on the CPU.

* the visibility descriptor that replaces the reference's additive mask expands to exactly
  the mask the reference builds (restated in oracle/decode_oracle.py from
  src/bonsai_sft/gpu/fast_runtime.py:316-372,391-465), for every (M, n_pend, cache_len);
* the oracle's masks satisfy the assertions of the reference's own mask tests
  (tests/test_bonsai_cpu.py:13-42);
* width selection, accept predicates and the draft chain reproduce the reference's known
  answers (tests/test_generation_artifact_preflight.py:118-126, tests/test_bonsai_d4.py:37-41,
  tests/test_bonsai_strict_verifier.py:18-36, tests/test_orin_runtime.py:146-154);
* the oracle's q/k-norm + RoPE and attention equal the same expressions evaluated by
  PyTorch on the CPU.
"""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import decode_oracle as DO
from oracle import oracle as O

from bitmtp_amd import generate as G
from bitmtp_amd import runtime as R


# ---------------------------------------------------------------- masks
@pytest.mark.parametrize("M", [8, 9, 10, 12, 16, 17])
def test_draft_descriptor_equals_reference_mask(M):
    D, sigma = 8, 40
    P = M - D
    for n_pend in range(0, P + 1):
        for cache_len in (1, 5, 23, sigma - 1):
            if n_pend == 0 and P != 0:
                # the reference only uses n_pend == 0 with M == D (fast_runtime.py:418-421);
                # with P > 0 its padding rows and hidden anchor are the same as here
                pass
            desc = R.step_descriptor("draft", M, D, cache_len, n_pend)
            got = R.dense_visibility(desc, M, sigma)
            want = DO.dense_mask_draft(M, sigma, D, n_pend, cache_len)
            assert np.array_equal(got, want), (M, n_pend, cache_len)


def test_draft_descriptor_empty_history_differs_only_on_padding_rows():
    # with no history the reference lets padding rows look at (empty) slot 0 so that their
    # softmax is finite; the descriptor gives such rows nothing and the kernel returns zeros
    M, D, sigma, n_pend = 12, 8, 16, 2
    got = R.dense_visibility(R.step_descriptor("draft", M, D, 0, n_pend), M, sigma)
    want = DO.dense_mask_draft(M, sigma, D, n_pend, 0)
    diff = np.argwhere(got != want)
    assert set(diff[:, 0]) == {2, 3} and set(diff[:, 1]) == {0}


@pytest.mark.parametrize("role,M", [("ar", 1), ("ar", 16), ("verify", 9), ("verify", 5)])
def test_causal_descriptor_equals_reference_mask(role, M):
    sigma = 24
    for cache_len in ([0] if role == "ar" else []) + [1, 7, sigma]:
        desc = R.step_descriptor(role, M, 8, cache_len)
        got = R.dense_visibility(desc, M, sigma)
        want = DO.dense_mask_causal(M, sigma, cache_len, role)
        assert np.array_equal(got, want)


def test_verifier_anchor_is_not_counted_twice():
    # assertions of the reference's tests/test_bonsai_cpu.py:13-30
    sigma, m, cache_len = 12, 9, 5
    for vis in (DO.dense_mask_causal(m, sigma, cache_len, "verify"),
                R.dense_visibility(R.step_descriptor("verify", m, 8, cache_len), m, sigma)):
        assert not vis[:, cache_len - 1].any()
        assert vis[:, :cache_len - 1].all()
        assert vis[:, sigma].all()
        assert not vis[0, sigma + 1:].any()
    with pytest.raises(RuntimeError, match="committed anchor"):
        DO.dense_mask_causal(m, sigma, 0, "verify")
    with pytest.raises(RuntimeError, match="committed anchor"):
        R.step_descriptor("verify", m, 8, 0)


def test_ar_keeps_last_history_slot():
    # tests/test_bonsai_cpu.py:32-42
    sigma, cache_len = 12, 5
    for vis in (DO.dense_mask_causal(1, sigma, cache_len, "ar"),
                R.dense_visibility(R.step_descriptor("ar", 1, 8, cache_len), 1, sigma)):
        assert vis[0, cache_len - 1]
        assert vis[0, sigma]


def test_draft_template_rows_follow_the_specification():
    # fast_runtime.py:316-332, spelled out for M=12 (P=4), n_pend=3
    M, D, sigma, n_pend, cache_len = 12, 8, 20, 3, 6
    vis = DO.dense_mask_draft(M, sigma, D, n_pend, cache_len)
    ws = vis[:, sigma:]
    assert ws[0].tolist() == [True] + [False] * 11            # pending row 0: itself
    assert ws[2].tolist() == [True] * 3 + [False] * 9         # pending row 2: rows 0..2
    assert not ws[3].any()                                    # padding row
    assert ws[4].tolist() == [True, True, False, False, True] + [False] * 7   # anchor
    assert ws[11].tolist() == [True, True, False, False] + [True] * 8          # last mask row
    assert vis[:, :cache_len].all() and not vis[:, cache_len:sigma].any()


def test_widest_step_fits_the_32_bit_row_words():
    """32 rows use bit 31 of the visibility word: the descriptor stays an int32 vector."""
    for role, n_pend in (("ar", 0), ("draft", 24), ("verify", 0)):
        desc = R.step_descriptor(role, 32, 8, 40, n_pend)
        arr = np.array(desc, dtype=np.int32)          # raises if a word does not fit
        assert arr.shape == (34,)
        vis = R.dense_visibility(desc, 32, 64)
        assert vis[31, 64 + 31] and vis.shape == (32, 96)
    causal = R.dense_visibility(R.step_descriptor("ar", 32, 8, 40), 32, 64)
    assert np.array_equal(causal[:, 64:], np.tril(np.ones((32, 32), dtype=bool)))
    assert np.array_equal(causal, DO.dense_mask_causal(32, 64, 40, "ar"))


def test_unknown_role_and_bad_pending_are_rejected():
    with pytest.raises(ValueError, match="unsupported graph role"):
        R.step_descriptor("verify_q1", 9, 8, 3, 1)
    with pytest.raises(ValueError, match="unsupported graph role"):
        R.logits_rows("draft_int4", 9, 8)
    with pytest.raises(ValueError):
        R.draft_row_masks(9, 8, 2)
    assert R.logits_rows("ar", 1, 8) == (0, 1)
    assert R.logits_rows("draft", 12, 8) == (4, 12)
    assert R.logits_rows("verify", 9, 8) == (0, 9)


# ---------------------------------------------------------------- selectors and predicates
def test_width_selector_tables():
    d8 = SimpleNamespace(D=8, m_set=(1, 8, 9, 10, 12, 16, 17))
    assert [G.select_M_for_pending(d8, n) for n in range(1, 10)] == [9, 10, 12, 12, 16, 16, 16, 16, 17]
    d4 = SimpleNamespace(D=4, m_set=(1, 4, 5, 6, 7, 8, 9))
    assert [G.select_M_for_pending(d4, n) for n in range(1, 6)] == [5, 6, 7, 8, 9]
    assert G.default_hybrid_m(8) == 6 and G.default_hybrid_m(4) == 3


def test_verify_accept_known_answers():
    verify = list(range(9))
    for prefix in range(9):
        draft = list(range(8))
        if prefix < 8:
            draft[prefix] = 99
        assert G.verify_accept(draft, verify, 8) == prefix
        assert DO.verify_accept(draft, verify, 8) == prefix
    # tied logits: only identical ids count (argmax of a tie is the lowest index)
    tied = np.array([[3.0, 3.0], [0.0, 0.0], [2.0, 2.0]], dtype=np.float32)
    verifier = DO.draft_chain(tied, 0.5)[0]
    assert verifier.tolist() == [0, 0, 0]
    assert G.verify_accept([1, 0], verifier, 2) == 0
    assert G.verify_accept([0, 1], verifier, 2) == 1
    assert G.verify_accept([0, 0], verifier, 2) == 2


def test_margins_and_foreign_verifiers_are_rejected_before_gpu_use():
    """tests/test_bonsai_strict_verifier.py:38-52 of the reference: every nonzero margin and
    every non-native verifier flag raises before the atlas is touched."""
    from bitmtp_amd import contracts
    for generate in (G.speculative_generate, G.hybrid_generate):
        for margin in (-0.5, 1e-20, 0.5, float("inf"), float("nan")):
            with pytest.raises(ValueError, match="requires rabv_margin=0"):
                generate(None, None, rabv_margin=margin)
        for flag in ("use_fp8_verify", "use_q1_verify", "use_w1a16_verify"):
            with pytest.raises(ValueError, match="native verifier projection"):
                generate(None, None, **{flag: True})
    contracts.validate_verification_options(0.0)
    contracts.validate_verification_options(-0.0, exact_m1_verify=True)
    with pytest.raises(ValueError):
        contracts.validate_verification_options("0.1")


def test_draft_and_verifier_role_selection():
    """tests/test_bonsai_strict_verifier.py:54-68 and :103-110 of the reference."""
    from bitmtp_amd import contracts
    atlas = SimpleNamespace(roles=("draft", "draft_fp8", "draft_bf16", "verify"))
    assert G.draft_role(atlas, False) == "draft"
    assert G.draft_role(atlas, False, True) == "draft_bf16"
    assert G.draft_role(atlas, True) == "draft_fp8"
    assert G.verify_role(atlas, False) == "verify"
    with pytest.raises(ValueError, match="native verifier"):
        G.verify_role(atlas, False, True)
    with pytest.raises(RuntimeError, match="mutually exclusive"):
        G.draft_role(atlas, True, True)
    with pytest.raises(ValueError, match="native verifier"):
        G.verify_role(atlas, True, True)
    with pytest.raises(RuntimeError, match="not captured"):
        G.draft_role(SimpleNamespace(roles=("draft", "verify")), True)
    with pytest.raises(RuntimeError, match="not captured"):
        G.verify_role(SimpleNamespace(roles=("draft",)))
    contracts.validate_graph_roles(("ar", "draft_bf16", "verify"), (8, 6))
    contracts.validate_graph_roles(("ar", "draft", "verify"), (8, 6))
    contracts.validate_graph_roles(("ar", "draft_fp8", "verify"), (9, 5))
    with pytest.raises(ValueError, match="FP8 draft"):
        contracts.validate_graph_roles(("ar", "draft_fp8", "verify"), (8, 6))
    with pytest.raises(ValueError, match="unsupported strict graph roles"):
        contracts.validate_graph_roles(("ar", "verify_q1"))
    # the approximate draft roles share the draft mask and logit rows
    for role in ("draft_fp8", "draft_bf16"):
        assert R.step_descriptor(role, 12, 8, 30, 3) == R.step_descriptor("draft", 12, 8, 30, 3)
        assert R.logits_rows(role, 12, 8) == (4, 12)
        assert R.HEAD_MODE_OF_ROLE[role] in ("fp8", "bf16_raw")
    assert {R.HEAD_MODE_OF_ROLE[r] for r in ("ar", "draft", "verify")} == {"native"}


def test_confidence_accept_known_answers():
    """``_confidence_accept`` (fast_generate.py:354-386): streak after the first token, cut in
    front of an EOS, at least the anchor's prediction."""
    toks = [5, 6, 7, 8, 9, 10, 11, 12]
    conf = [0.1, 0.95, 0.97, 0.5, 0.99, 0.99, 0.99, 0.99]
    assert G.confidence_accept(toks, conf, 0.9, set(), 8) == ([5, 6, 7], 3, False)
    assert G.confidence_accept(toks, [0.0] + [1.0] * 7, 0.9, set(), 8) == (toks, 8, False)
    assert G.confidence_accept(toks, [1.0] + [0.0] * 7, 0.9, set(), 8) == ([5], 1, False)
    assert G.confidence_accept(toks, conf, 0.9, {6}, 8) == ([5], 1, True)
    assert G.confidence_accept(toks, conf, 0.9, {5}, 8) == ([], 0, True)
    assert G.confidence_accept(toks, conf, 0.9, {8}, 8) == ([5, 6, 7], 3, False)   # beyond the streak
    # NaN never passes the gate
    assert G.confidence_accept(toks, [0.5, float("nan"), 1.0], 0.9, set(), 8)[1] == 1


def test_draft_chain_known_answer():
    logits = np.array([[0., 0.], [20., 0.], [0., 0.], [20., 0.]], dtype=np.float32)
    tokens, conf, length = DO.draft_chain(logits, 0.9)
    assert tokens.tolist() == [0, 0, 0, 0] and length == 2
    assert G.draft_chain_accept(conf, 0.9) == 2
    assert conf[0] == np.float32(0.5) and conf[1] > 0.999
    # row 0 never gates; NaN confidence stops the chain
    assert G.draft_chain_accept([0.0, 1.0, 1.0], 0.9) == 3
    assert G.draft_chain_accept([1.0, float("nan"), 1.0], 0.9) == 1
    # equal to the threshold is not above it (fp32 comparison)
    assert G.draft_chain_accept([1.0, np.float32(0.9)], 0.9) == 1


def test_draft_chain_matches_torch_expression():
    rng = np.random.default_rng(3)
    logits = torch.from_numpy(rng.normal(0, 3, (8, 4096)).astype(np.float32)).to(torch.bfloat16)
    mx, idx = logits.max(dim=-1)
    conf = torch.exp(mx.float() - torch.logsumexp(logits.float(), dim=-1))
    tokens, c, n = DO.draft_chain(logits.float().numpy(), 0.01)
    assert tokens.tolist() == idx.tolist()
    np.testing.assert_allclose(c, conf.numpy(), rtol=1e-5)
    assert n == 1 + int((conf[1:] > 0.01).int().cumprod(0).sum())


# ---------------------------------------------------------------- oracle vs PyTorch
def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _torch_qk_norm_rope(xqkv, qw, kw, eps, cos_t, sin_t, positions, n_heads, n_kv):
    """The reference expression (src/bonsai_sft/gpu/model.py:388-436) in eager PyTorch."""
    hd = 128
    M = xqkv.shape[0]
    dt = xqkv.dtype
    q_dim, k_dim = n_heads * hd, n_kv * hd
    xq = xqkv[:, :q_dim].view(M, n_heads, hd)
    xk = xqkv[:, q_dim:q_dim + k_dim].view(M, n_kv, hd)
    xv = xqkv[:, q_dim + k_dim:].view(M, n_kv, hd)

    def norm(x, w):
        xf = x.float()
        var = xf.pow(2).mean(-1, keepdim=True)
        return w * (xf * torch.rsqrt(var + eps)).to(dt)

    def rot(x):
        return torch.cat((-x[..., hd // 2:], x[..., : hd // 2]), dim=-1)
    xq, xk = norm(xq, qw), norm(xk, kw)
    cos = cos_t[positions].unsqueeze(1)
    sin = sin_t[positions].unsqueeze(1)
    return (xq * cos) + (rot(xq) * sin), (xk * cos) + (rot(xk) * sin), xv


def test_qk_norm_rope_oracle_equals_torch_eager():
    from bitmtp_amd.model import ModelArgs, rope_tables
    torch.manual_seed(0)
    M, n_heads, n_kv = 9, 4, 2
    xqkv = (torch.randn(M, (n_heads + 2 * n_kv) * 128) * 2).to(torch.bfloat16)
    qw = (1 + 0.1 * torch.randn(128)).to(torch.bfloat16)
    kw = (1 + 0.1 * torch.randn(128)).to(torch.bfloat16)
    cos_t, sin_t = rope_tables(ModelArgs(), 300, "cpu")
    positions = torch.tensor([0, 1, 2, 17, 100, 101, 255, 299, 5])
    tq, tk, tv = _torch_qk_norm_rope(xqkv, qw, kw, 1e-6, cos_t, sin_t, positions, n_heads, n_kv)
    q, k, v = DO.qk_norm_rope(_bits(xqkv), _bits(qw), _bits(kw), 1e-6, _bits(cos_t), _bits(sin_t),
                              positions.numpy(), n_heads, n_kv)
    assert np.array_equal(v, _bits(tv))
    for got, want in ((q, _bits(tq)), (k, _bits(tk))):
        # identical up to the last-place effects of rsqrt / the order of the mean
        from gpu_util import bf16_ordinal
        d = np.abs(bf16_ordinal(got) - bf16_ordinal(want))
        assert d.max() <= 1 and (d != 0).mean() < 0.01


def test_rope_table_known_values():
    from bitmtp_amd.model import ModelArgs, rope_tables, yarn_attention_factor
    cos_t, sin_t = rope_tables(ModelArgs(), 4, "cpu")
    m = yarn_attention_factor(4.0)
    assert abs(m - (0.1 * np.log(4.0) + 1.0)) < 1e-12
    # position 0: cos = mscale, sin = 0; halves of the table repeat
    assert torch.all(cos_t[0].float() == torch.tensor(m).to(torch.bfloat16).float())
    assert torch.all(sin_t[0] == 0)
    assert torch.equal(cos_t[:, :64], cos_t[:, 64:]) and torch.equal(sin_t[:, :64], sin_t[:, 64:])
    # highest frequency (pair 0) is not interpolated: angle = position
    assert abs(float(sin_t[1, 0]) - m * np.sin(1.0)) < 1e-2


def test_attention_oracle_equals_torch_sdpa():
    rng = np.random.default_rng(5)
    M, n_heads, n_kv, sigma, cache_len = 9, 4, 2, 20, 11
    q = torch.from_numpy(rng.normal(0, 1, (M, n_heads, 128)).astype(np.float32)).to(torch.bfloat16)
    k = torch.from_numpy(rng.normal(0, 1, (n_kv, sigma + M, 128)).astype(np.float32)).to(torch.bfloat16)
    v = torch.from_numpy(rng.normal(0, 1, (n_kv, sigma + M, 128)).astype(np.float32)).to(torch.bfloat16)
    vis = DO.dense_mask_causal(M, sigma, cache_len, "verify")
    got = DO.attention(_bits(q), _bits(k), _bits(v), vis, 1 / np.sqrt(128))
    qq = q.double().permute(1, 0, 2).unsqueeze(0)
    kk = k.double().repeat_interleave(n_heads // n_kv, dim=0).unsqueeze(0)
    vv = v.double().repeat_interleave(n_heads // n_kv, dim=0).unsqueeze(0)
    want = torch.nn.functional.scaled_dot_product_attention(
        qq, kk, vv, attn_mask=torch.from_numpy(vis)[None, None])
    want = want[0].permute(1, 0, 2).reshape(M, -1).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-12)


def test_graph_capture_runs_with_the_garbage_collector_off():
    """A collector run inside a stream capture can destroy another atlas's graphs and abort
    the process: `_capture_one` collects first and keeps the collector off until the capture
    has ended, also when the capture raises."""
    import gc
    atlas = R.GraphAtlas.__new__(R.GraphAtlas)
    seen = []

    def fake_impl(M, sigma, role):
        seen.append((gc.isenabled(), torch.is_inference_mode_enabled()))
        if role == "boom":
            raise RuntimeError("capture failed")
        return "graph"
    atlas._capture_one_impl = fake_impl
    assert gc.isenabled()
    with torch.inference_mode():
        assert atlas._capture_one(1, 64, "ar") == "graph"
    assert seen == [(False, False)] and gc.isenabled()
    with pytest.raises(RuntimeError, match="capture failed"):
        atlas._capture_one(1, 64, "boom")
    assert gc.isenabled()
    gc.disable()
    try:
        atlas._capture_one(1, 64, "ar")
        assert not gc.isenabled()      # a caller's own setting is left alone
    finally:
        gc.enable()
