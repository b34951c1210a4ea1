"""The generation loops on a symbolic atlas (tests/symbolic_atlas.py): every replay predicts
from exactly the KV slots the real step descriptor makes visible, so the loops' bookkeeping
(pending rows, commits from draft and verify workspaces, anchors, segment migration) is
checked on the CPU against the toy model's greedy continuation.  The invariants are the
reference's: speculation with a strict verifier reproduces greedy AR token for token
(docs/testing.md:13, fast_generate.py:611-657), accounting identities
(fast_generate.py:1151-1162), confidence decoding commits the drafter's confident prefix
(fast_generate.py:354-386)."""
import pytest

from bitmtp_amd import generate as G
from symbolic_atlas import MASK, VOCAB, SymbolicAtlas, greedy

PROMPTS = [list(range(5, 5 + n)) for n in (1, 7, 31, 32, 33, 70)]


@pytest.mark.parametrize("prompt", PROMPTS, ids=lambda p: f"prompt{len(p)}")
def test_ar_loop_reproduces_the_greedy_continuation(prompt):
    atlas = SymbolicAtlas()
    out, st = G.ar_generate(atlas, prompt, max_gen_len=40)
    assert out == greedy(prompt, 40)
    assert st["decode_tokens"] == 40 and st["timed_decode_tokens"] == 39 and st["n_iters"] == 40


@pytest.mark.parametrize("wrong_every", [0, 2, 3, 5])
@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("prompt", PROMPTS[1:5], ids=lambda p: f"prompt{len(p)}")
def test_speculative_and_hybrid_loops_reproduce_greedy(prompt, exact, wrong_every):
    want = greedy(prompt, 57)
    for fn, kw in ((G.speculative_generate, {}), (G.hybrid_generate, {"threshold": 0.9}),
                   (G.hybrid_generate, {"threshold": 0.9, "hybrid_m": 2})):
        atlas = SymbolicAtlas(wrong_every=wrong_every)
        out, st = fn(atlas, prompt, max_gen_len=57, exact_m1_verify=exact, **kw)
        if fn is G.speculative_generate or wrong_every == 0:
            assert out == want, (fn.__name__, kw)
        else:
            # the confidence path commits unverified drafts: with a drafter that is wrong
            # only where its confidence is low they are still the greedy tokens
            assert out == want, (fn.__name__, kw)
        assert st["draft_iters"] == st["n_conf_path"] + st["n_verify_path"]
        assert st["decode_tokens"] == 1 + st["accepted_drafts"] + st["verifier_bonus_tokens"] == 57
        assert st["drafted_tokens"] == 8 * st["draft_iters"]
        if fn is G.speculative_generate:
            assert st["n_conf_path"] == 0
        if wrong_every == 0 and not exact:
            # a perfect drafter: every verified iteration commits D drafts + 1 bonus
            assert st["committed_per_iter"] > 7.0


def test_hybrid_takes_the_confidence_path_when_the_chain_is_long_enough():
    prompt = list(range(3, 20))
    atlas = SymbolicAtlas(wrong_every=0)
    out, st = G.hybrid_generate(atlas, prompt, threshold=0.9, max_gen_len=64)
    assert out == greedy(prompt, 64)
    assert st["n_conf_path"] > 0 and st["n_verify_path"] == 0 and st["verifier_bonus_tokens"] == 0
    # pending rows of a confidence iteration: the whole committed block is re-forwarded
    widths = {m for role, m in atlas.log if role == "draft"}
    assert 16 in widths
    # a drafter that misses every second position never builds a chain of six
    atlas = SymbolicAtlas(wrong_every=2)
    out, st = G.hybrid_generate(atlas, prompt, threshold=0.9, max_gen_len=40)
    assert out == greedy(prompt, 40) and st["n_conf_path"] == 0


@pytest.mark.parametrize("wrong_every", [0, 3])
def test_confidence_loop(wrong_every):
    prompt = list(range(9, 30))
    atlas = SymbolicAtlas(wrong_every=wrong_every)
    out, st = G.confidence_generate(atlas, prompt, threshold=0.9, max_gen_len=50)
    # the drafter is wrong only where its confidence is low, so the committed prefix of every
    # block is the greedy continuation
    assert out == greedy(prompt, 50)
    assert st["n_verify_path"] == 0 and st["conf_path_frac"] == 1.0
    assert st["decode_tokens"] == 50 and st["timed_decode_tokens"] == 50 - st["untimed_output_tokens"]
    if wrong_every == 0:
        assert st["n_iters"] == 7 and st["untimed_output_tokens"] == 8
    else:
        assert st["n_iters"] > 7


def test_eos_and_length_limits():
    prompt = list(range(2, 25))
    want = greedy(prompt, 64)
    eos = want[20]
    cut = want.index(eos)
    for fn, kw in ((G.ar_generate, {}), (G.speculative_generate, {}), (G.hybrid_generate, {}),
                   (G.confidence_generate, {})):
        atlas = SymbolicAtlas(wrong_every=0)
        out, st = fn(atlas, prompt, max_gen_len=64, eos_ids=[eos], **kw)
        assert out == want[:cut], fn.__name__
        out, st = fn(SymbolicAtlas(wrong_every=3), prompt, max_gen_len=13, **kw)
        assert out == want[:13] and st["decode_tokens"] == 13, fn.__name__


def test_long_generation_migrates_between_segments():
    prompt = list(range(1, 41))
    want = greedy(prompt, 300)
    for fn in (G.ar_generate, G.speculative_generate, G.hybrid_generate, G.confidence_generate):
        atlas = SymbolicAtlas(segment_ladder=(64, 128, 512), wrong_every=4)
        # start in a segment the run outgrows: force it by asking for few tokens first
        out, st = fn(atlas, prompt, max_gen_len=300)
        assert out == want, fn.__name__
    # a run that starts in the smallest segment and has to move twice
    for fn in (G.ar_generate, G.speculative_generate, G.hybrid_generate, G.confidence_generate):
        atlas = SymbolicAtlas(segment_ladder=(64, 128, 512), wrong_every=4)
        real_select, calls = atlas.select_segment, []

        def select(needed):
            calls.append(needed)
            # the first placement pretends that the run is short; later ones ask for little
            # more than the live history, as after an under-estimated generation length
            return 64 if len(calls) == 1 else real_select(needed - 60)
        atlas.select_segment = select
        out, _ = fn(atlas, prompt, max_gen_len=300)
        assert out == want, fn.__name__
        assert len(calls) >= 3, fn.__name__
    assert MASK > VOCAB
