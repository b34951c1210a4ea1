"""Greedy AR and hybrid multi-token decode loops over the graph atlas, the
counterparts of ``fast_ar_generate`` and ``fast_hybrid_generate``
(src/bonsai_sft/gpu/fast_generate.py:179-292 and :903-1187).

Semantics kept from the reference:

* AR: one width-1 replay per token; the new KV row is committed after each replay.
* Hybrid: a draft replay of width ``M = select_M_for_pending(n_pend)`` carries the
  pending committed tokens, the anchor (a repeat of the last pending token) and D-1 mask
  tokens.  Row 0 of the D draft predictions is always committed; the confidence chain
  ``1 + longest prefix of conf[1:] > threshold`` decides between a pure confidence commit
  (chain >= hybrid_m) and verification.  Verification replays width D+1 over
  ``[anchor, draft tokens]``, accepts the longest prefix of identical token ids, appends
  the verifier's own next token, and promotes the accepted rows' KV
  (``exact_m1_verify`` replays width-1 AR steps instead and reproduces AR output
  token for token).
* Accounting and the returned statistics keys follow fast_generate.py:1151-1186; decode
  throughput is ``timed_decode_tokens / decode_time`` with prefill and the first token
  excluded (fast_generate.py:1001,1147-1148,1171).

The prompt is prefilled with the same packed kernels: AR-causal replays of width
``atlas.prefill_width`` over consecutive chunks (the reference uses a bf16 dequantised
variable-shape forward, fast_generate.py:949-953).
"""
from __future__ import annotations

import time
from typing import Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import contracts
from .runtime import GraphAtlas


def select_M_for_pending(atlas: GraphAtlas, n_pend: int) -> int:
    """Smallest captured M with P = M - D >= n_pend (fast_generate.py:574-583).
    For D=8 and m_set {9,10,12,16,17}: n_pend 1 -> 9, 2 -> 10, 3-4 -> 12, 5-8 -> 16, >=9 -> 17."""
    target = n_pend + atlas.D
    for M in atlas.m_set:
        if M >= target and M - atlas.D >= n_pend:
            return M
    return atlas.m_set[-1]


def draft_chain_accept(conf: Sequence[float], threshold: float) -> int:
    """``1 + longest_true_prefix(conf[1:] > threshold)`` in fp32 (fast_generate.py:126-129)."""
    thr = np.float32(threshold)
    n = 1
    for c in conf[1:]:
        if not (np.float32(c) > thr):
            break
        n += 1
    return n


def verify_accept(draft_tokens: Sequence[int], verify_tokens: Sequence[int], D: int) -> int:
    """Longest prefix of identical token ids (fast_generate.py:133-146)."""
    n = 0
    for a, b in zip(draft_tokens[:D], verify_tokens[:D]):
        if int(a) != int(b):
            break
        n += 1
    return n


def draft_role(atlas: GraphAtlas, use_fp8: bool, use_bf16: bool = False) -> str:
    """The draft output-projection role: the exact native one, or one of the two
    acceptance-tolerant approximations (``_draft_role``, fast_generate.py:586-599)."""
    if use_fp8 and use_bf16:
        raise RuntimeError("FP8 and BF16 draft roles are mutually exclusive")
    role = "draft_fp8" if use_fp8 else ("draft_bf16" if use_bf16 else "draft")
    if role not in atlas.roles:
        raise RuntimeError(f"requested draft role was not captured: {role}")
    return role


def verify_role(atlas: GraphAtlas, use_fp8: bool = False, use_q1: bool = False,
                use_w1a16: bool = False) -> str:
    """Native verification only (``_verify_role``, fast_generate.py:602-608)."""
    contracts.validate_native_verifier(use_fp8, use_q1, use_w1a16)
    if "verify" not in atlas.roles:
        raise RuntimeError("requested native verify role was not captured")
    return "verify"


def default_hybrid_m(D: int) -> int:
    """Confidence-streak gate: 6 for D=8, 3 for D=4 (fast_generate.py:938-939)."""
    return 6 if D == 8 else (3 if D == 4 else max(1, (3 * D) // 4))


def _scan_eos(toks: List[int], eos_set) -> Tuple[bool, int]:
    """(eos_hit, tokens kept before the EOS) (fast_generate.py:149-172)."""
    if not eos_set:
        return False, len(toks)
    for i, t in enumerate(toks):
        if t in eos_set:
            return True, i
    return False, len(toks)


def prefill(atlas: GraphAtlas, prompt: Sequence[int], sigma: int) -> int:
    """Materialise the prompt's KV in segment sigma and return the first generated token."""
    W = atlas.prefill_width
    n = len(prompt)
    if n < 1:
        raise ValueError("empty prompt")
    g = atlas.get_graph(W, sigma, "ar")
    cache_len = 0
    first = None
    while cache_len < n:
        take = min(W, n - cache_len)
        toks = list(prompt[cache_len:cache_len + take]) + [0] * (W - take)
        pos = [cache_len + i for i in range(W)]
        atlas.replay(g, toks, pos, cache_len)
        atlas.commit_kv(sigma, cache_len, take)
        cache_len += take
        if cache_len == n:
            out, _, _ = atlas.read_outputs(g)
            first = int(out[take - 1])
    return first


def _stats_common(prefill_time, decode_time, total_time, seq_len, out_len):
    return {
        "prefill_time": prefill_time, "decode_time": decode_time, "total_time": total_time,
        "prefill_tokens": seq_len, "decode_tokens": out_len,
        "timed_decode_tokens": max(0, out_len - 1),
        "untimed_output_tokens": min(1, out_len),
        "ttft": prefill_time,
    }


def ar_generate(atlas: GraphAtlas, input_ids: Sequence[int], max_gen_len: int = 512,
                eos_ids: Iterable[int] = ()) -> Tuple[List[int], dict]:
    """Greedy AR decode with the width-1 graph (fast_generate.py:179-292)."""
    eos_set = set(int(e) for e in eos_ids)
    prompt = [int(t) for t in input_ids]
    seq_len = len(prompt)
    t0 = time.time()
    sigma = atlas.select_segment(seq_len + max_gen_len + atlas.M_max)
    next_tok = prefill(atlas, prompt, sigma)
    cache_len = seq_len
    atlas.synchronize()
    prefill_time = time.time() - t0
    if eos_set and next_tok in eos_set:
        st = _stats_common(prefill_time, 1e-9, prefill_time, seq_len, 0)
        st.update({"n_iters": 0, "avg_accept": None})
        return [], st
    gen = [next_tok]
    g = atlas.get_graph(1, sigma, "ar")
    t1 = time.time()
    while len(gen) < max_gen_len:
        if cache_len + atlas.M_max > sigma:
            new_sigma = atlas.select_segment(cache_len + atlas.M_max + 64)
            if new_sigma != sigma:
                atlas.migrate_segment(sigma, new_sigma, cache_len)
                sigma = new_sigma
                g = atlas.get_graph(1, sigma, "ar")
        atlas.replay(g, [next_tok], [cache_len], cache_len)
        atlas.commit_kv(sigma, cache_len, 1)
        cache_len += 1
        out, _, _ = atlas.read_outputs(g)
        next_tok = int(out[0])
        if eos_set and next_tok in eos_set:
            break
        gen.append(next_tok)
        if cache_len + 1 > atlas.segment_ladder[-1]:
            break
    atlas.synchronize()
    decode_time = max(time.time() - t1, 1e-9)
    st = _stats_common(prefill_time, decode_time, time.time() - t0, seq_len, len(gen))
    st.update({"n_iters": len(gen), "avg_accept": 1.0})
    return gen, st


def _exact_m1_verify(atlas: GraphAtlas, sigma: int, cache_len: int, pending: List[int],
                     draft_tokens: Sequence[int]) -> Tuple[int, int, int]:
    """Verify with the width-1 AR graph (fast_generate.py:611-657): recompute the pending
    tail at width 1, then walk the proposals until the first mismatch.  Returns
    ``(accept_count, new_cache_len, correction_or_bonus)``."""
    g = atlas.get_graph(1, sigma, "ar")
    n_pend = len(pending)
    base_len = cache_len - n_pend
    for j, tok in enumerate(pending):
        pos = base_len + j
        atlas.replay(g, [int(tok)], [pos], pos)
        atlas.commit_kv(sigma, pos, 1)
    out, _, _ = atlas.read_outputs(g)
    pred = int(out[0])
    accept = 0
    for j, tok in enumerate(draft_tokens):
        if int(tok) != pred:
            break
        accept += 1
        pos = cache_len + j
        atlas.replay(g, [int(tok)], [pos], pos)
        atlas.commit_kv(sigma, pos, 1)
        out, _, _ = atlas.read_outputs(g)
        pred = int(out[0])
    return accept, cache_len + accept, pred


def hybrid_generate(atlas: GraphAtlas, input_ids: Sequence[int], threshold: float = 0.9,
                    hybrid_m: Optional[int] = None, max_gen_len: int = 512,
                    eos_ids: Iterable[int] = (), exact_m1_verify: bool = False,
                    use_fp8_draft: bool = False, use_bf16_draft: bool = False,
                    use_fp8_verify: bool = False, use_q1_verify: bool = False,
                    use_w1a16_verify: bool = False, rabv_margin: float = 0.0
                    ) -> Tuple[List[int], dict]:
    """Hybrid decode: the confidence streak switches between draft-only commits and
    verification (fast_generate.py:903-1187).  Nonzero margins and non-native verifier
    projections are rejected before anything touches the GPU (fast_generate.py:934-935);
    ``use_fp8_draft`` / ``use_bf16_draft`` pick the approximate draft projection."""
    contracts.validate_verification_options(rabv_margin, exact_m1_verify)
    contracts.validate_native_verifier(use_fp8_verify, use_q1_verify, use_w1a16_verify)
    if hybrid_m is not None and hybrid_m < 1:
        raise ValueError("hybrid_m must be at least 1")
    role_d = draft_role(atlas, use_fp8_draft, use_bf16_draft)
    role_v = verify_role(atlas)
    args = atlas.args
    D = args.block_size
    MASK = args.mask_token_id
    if hybrid_m is None:
        hybrid_m = default_hybrid_m(D)
    eos_set = set(int(e) for e in eos_ids)
    prompt = [int(t) for t in input_ids]
    seq_len = len(prompt)
    M_verify = D + 1

    t0 = time.time()
    sigma = atlas.select_segment(seq_len + max_gen_len + atlas.M_max)
    next_tok = prefill(atlas, prompt, sigma)
    cache_len = seq_len
    atlas.synchronize()
    prefill_time = time.time() - t0
    if eos_set and next_tok in eos_set:
        st = _stats_common(prefill_time, 1e-9, prefill_time, seq_len, 0)
        st.update({"n_iters": 0, "avg_accept": None, "draft_iters": 0, "drafted_tokens": 0,
                   "accepted_drafts": 0, "accept_rate": None, "verifier_bonus_tokens": 0,
                   "committed_tokens": 0, "committed_per_iter": None, "conf_path_frac": None,
                   "n_conf_path": 0, "n_verify_path": 0})
        return [], st

    gen = [next_tok]
    pending = [next_tok]
    n_iters = 1
    eos_found = False
    n_conf_path = n_verify_path = 0
    draft_iters = drafted_total = accepted_draft_total = verifier_bonus_total = 0

    t1 = time.time()
    while len(gen) < max_gen_len and not eos_found:
        n_iters += 1
        draft_iters += 1
        drafted_total += D
        n_pend = len(pending)
        M_draft = select_M_for_pending(atlas, n_pend)
        P = M_draft - D
        if n_pend > P:
            raise RuntimeError(f"{n_pend} pending tokens do not fit the widest draft graph")

        if cache_len + atlas.M_max > sigma:
            new_sigma = atlas.select_segment(cache_len + atlas.M_max + 64)
            if new_sigma != sigma:
                atlas.migrate_segment(sigma, new_sigma, cache_len)
                sigma = new_sigma

        # ---- draft replay: [pending | pad | anchor | MASK x (D-1)]
        gd = atlas.get_graph(M_draft, sigma, role_d)
        toks = pending + [0] * (P - n_pend) + [pending[-1]] + [MASK] * (D - 1)
        pos = [cache_len + i for i in range(n_pend)] + [0] * (P - n_pend) + \
              [cache_len + n_pend - 1 + i for i in range(D)]
        atlas.replay(gd, toks, pos, cache_len, n_pend=n_pend)
        atlas.commit_kv(sigma, cache_len, n_pend)
        cache_len += n_pend
        d_tokens, d_conf, _ = atlas.read_outputs(gd)
        draft_tokens = [int(t) for t in d_tokens[:D]]
        iter_accept = draft_chain_accept(d_conf[:D], threshold)

        use_verify = iter_accept < hybrid_m
        if not use_verify:
            commit = draft_tokens[:iter_accept]
            accepted_this_iter, bonus_this_iter = iter_accept, 0
            n_conf_path += 1
        else:
            if exact_m1_verify:
                accept_count, cache_len, bonus = _exact_m1_verify(
                    atlas, sigma, cache_len, pending, draft_tokens)
            else:
                gv = atlas.get_graph(M_verify, sigma, role_v)
                vt = [pending[-1]] + draft_tokens
                vp = [cache_len - 1 + i for i in range(M_verify)]
                atlas.replay(gv, vt, vp, cache_len)
                v_tokens, _, _ = atlas.read_outputs(gv)
                accept_count = verify_accept(draft_tokens, v_tokens, D)
                bonus = int(v_tokens[accept_count])
                if accept_count > 0:
                    # rows 1..accept_count of the verify workspace are AR-correct
                    atlas.commit_kv(sigma, cache_len, accept_count, first_row=1)
                    cache_len += accept_count
            commit = draft_tokens[:accept_count] + [bonus]
            accepted_this_iter, bonus_this_iter = accept_count, 1
            n_verify_path += 1

        n_commit = len(commit)
        eos_hit, n_kept = _scan_eos(commit, eos_set)
        if eos_hit:
            eos_found = True
            n_commit = n_kept
        if len(gen) + n_commit > max_gen_len:
            n_commit = max(0, max_gen_len - len(gen))

        accepted_emitted = min(accepted_this_iter, n_commit)
        bonus_emitted = int(bool(bonus_this_iter) and n_commit > accepted_this_iter)
        if accepted_emitted + bonus_emitted != n_commit:
            raise RuntimeError("hybrid emitted-token accounting mismatch: "
                               f"accepted={accepted_emitted} bonus={bonus_emitted} "
                               f"committed={n_commit}")
        accepted_draft_total += accepted_emitted
        verifier_bonus_total += bonus_emitted

        if n_commit > 0:
            gen.extend(commit[:n_commit])
        else:
            eos_found = True
        if eos_found or len(gen) >= max_gen_len:
            break

        # verify path reused KV: only the bonus is pending; confidence path re-forwards
        # the whole committed block as pending rows
        pending = [commit[n_commit - 1]] if use_verify else list(commit[:n_commit])
        if cache_len + len(pending) + D > atlas.segment_ladder[-1]:
            break

    atlas.synchronize()
    decode_time = max(time.time() - t1, 1e-9)
    n_out = len(gen)
    if drafted_total != D * draft_iters:
        raise RuntimeError("hybrid drafted-token accounting mismatch")
    if draft_iters != n_conf_path + n_verify_path:
        raise RuntimeError("hybrid path/iteration accounting mismatch")
    if n_iters != draft_iters + 1:
        raise RuntimeError("hybrid n_iters accounting mismatch")
    if n_out != 1 + accepted_draft_total + verifier_bonus_total:
        raise RuntimeError("hybrid output-origin accounting mismatch")
    if verifier_bonus_total > n_verify_path:
        raise RuntimeError("hybrid verifier bonus count exceeds verify paths")
    if accepted_draft_total > drafted_total:
        raise RuntimeError("hybrid accepted draft count exceeds drafted count")
    committed_per_iter = (n_out - 1) / draft_iters if draft_iters > 0 else 0.0
    st = _stats_common(prefill_time, decode_time, time.time() - t0, seq_len, n_out)
    st.update({
        "n_iters": n_iters, "avg_accept": committed_per_iter, "draft_iters": draft_iters,
        "drafted_tokens": drafted_total, "accepted_drafts": accepted_draft_total,
        "accept_rate": accepted_draft_total / drafted_total if drafted_total > 0 else 0.0,
        "verifier_bonus_tokens": verifier_bonus_total, "committed_tokens": n_out - 1,
        "committed_per_iter": committed_per_iter,
        "conf_path_frac": n_conf_path / max(1, n_conf_path + n_verify_path),
        "n_conf_path": n_conf_path, "n_verify_path": n_verify_path,
    })
    return gen, st


def speculative_generate(atlas: GraphAtlas, input_ids: Sequence[int], max_gen_len: int = 512,
                         eos_ids: Iterable[int] = (), exact_m1_verify: bool = False,
                         use_fp8_draft: bool = False, use_bf16_draft: bool = False,
                         use_fp8_verify: bool = False, use_q1_verify: bool = False,
                         use_w1a16_verify: bool = False, rabv_margin: float = 0.0
                         ) -> Tuple[List[int], dict]:
    """Self-speculative decode (fast_generate.py:664-899): every iteration drafts D tokens,
    verifies them with the width-(D+1) graph (or the exact width-1 path) and commits the
    matching prefix plus the verifier's bonus token.  It is the hybrid loop with the
    confidence path switched off: a chain length never reaches D + 1."""
    gen, st = hybrid_generate(atlas, input_ids, threshold=float("inf"),
                              hybrid_m=atlas.args.block_size + 1 if atlas is not None else None,
                              max_gen_len=max_gen_len, eos_ids=eos_ids,
                              exact_m1_verify=exact_m1_verify, use_fp8_draft=use_fp8_draft,
                              use_bf16_draft=use_bf16_draft, use_fp8_verify=use_fp8_verify,
                              use_q1_verify=use_q1_verify, use_w1a16_verify=use_w1a16_verify,
                              rabv_margin=rabv_margin)
    if st["n_conf_path"] != 0:
        raise RuntimeError("speculative decode took a confidence path")
    return gen, st


def confidence_accept(tokens: Sequence[int], conf: Sequence[float], threshold: float, eos_set,
                      D: int) -> Tuple[List[int], int, bool]:
    """Confidence-streak acceptance of one block (``_confidence_accept``,
    fast_generate.py:354-386): ``1 + longest streak of conf[1:] > threshold`` tokens, cut in
    front of the first EOS among them; returns ``(accepted, count, eos_hit)``."""
    n = min(draft_chain_accept(conf[:D], threshold), D)
    accepted: List[int] = []
    for t in tokens[:n]:
        if int(t) in eos_set:
            return accepted, len(accepted), True
        accepted.append(int(t))
    return accepted, n, False


def confidence_generate(atlas: GraphAtlas, input_ids: Sequence[int], threshold: float = 0.9,
                        max_gen_len: int = 512, eos_ids: Iterable[int] = (),
                        use_fp8_draft: bool = False, use_bf16_draft: bool = False
                        ) -> Tuple[List[int], dict]:
    """Confidence-chain decode (fast_generate.py:393-572): every iteration commits the
    confident prefix of a drafted block and re-forwards it as pending rows of the next; no
    verifier.  The first block is drafted straight after the prompt from the last prompt
    token as anchor (positions seq_len-1 .. seq_len+D-2, its history copy hidden), which the
    reference runs as a variable-shape forward (fast_generate.py:322-352) and this harness as
    the width-D draft graph with no pending rows: the same mask
    (``create_sdlm_attention_mask``, model.py:462-505)."""
    role = draft_role(atlas, use_fp8_draft, use_bf16_draft)
    args = atlas.args
    D, MASK = args.block_size, args.mask_token_id
    eos_set = set(int(e) for e in eos_ids)
    prompt = [int(t) for t in input_ids]
    seq_len = len(prompt)

    t0 = time.time()
    sigma = atlas.select_segment(seq_len + max_gen_len + atlas.M_max)
    prefill(atlas, prompt, sigma)
    cache_len = seq_len
    g1 = atlas.get_graph(D, sigma, role)
    atlas.replay(g1, [prompt[-1]] + [MASK] * (D - 1),
                 [seq_len - 1 + i for i in range(D)], cache_len, n_pend=0)
    toks, conf, _ = atlas.read_outputs(g1)
    accepted, _, eos_found = confidence_accept(toks, conf, threshold, eos_set, D)
    atlas.synchronize()
    prefill_time = time.time() - t0

    gen: List[int] = list(accepted[:max_gen_len])
    untimed = len(gen)
    n_iters = 1
    accept_total = len(gen)
    pending = list(gen)
    t1 = time.time()
    while len(gen) < max_gen_len and not eos_found and pending:
        n_iters += 1
        n_pend = len(pending)
        M = select_M_for_pending(atlas, n_pend)
        P = M - D
        if n_pend > P:
            raise RuntimeError(f"{n_pend} pending tokens do not fit the widest draft graph")
        if cache_len + atlas.M_max > sigma:
            new_sigma = atlas.select_segment(cache_len + atlas.M_max + 64)
            if new_sigma != sigma:
                atlas.migrate_segment(sigma, new_sigma, cache_len)
                sigma = new_sigma
        g = atlas.get_graph(M, sigma, role)
        toks_in = pending + [0] * (P - n_pend) + [pending[-1]] + [MASK] * (D - 1)
        pos = [cache_len + i for i in range(n_pend)] + [0] * (P - n_pend) + \
              [cache_len + n_pend - 1 + i for i in range(D)]
        atlas.replay(g, toks_in, pos, cache_len, n_pend=n_pend)
        atlas.commit_kv(sigma, cache_len, n_pend)
        cache_len += n_pend
        toks, conf, _ = atlas.read_outputs(g)
        accepted, n_acc, eos_hit = confidence_accept(toks, conf, threshold, eos_set, D)
        remaining = max(0, max_gen_len - len(gen))
        if n_acc > remaining:
            accepted = accepted[:remaining]
            n_acc = len(accepted)
        accept_total += n_acc
        pending = accepted
        if n_acc == 0:
            break
        gen.extend(accepted)
        eos_found = eos_hit
        if cache_len + n_pend + D > atlas.segment_ladder[-1]:
            break
    atlas.synchronize()
    decode_time = max(time.time() - t1, 1e-9)
    n_out = len(gen)
    st = {
        "prefill_time": prefill_time, "decode_time": decode_time if n_iters > 1 else 1e-9,
        "total_time": time.time() - t0, "prefill_tokens": seq_len, "decode_tokens": n_out,
        "timed_decode_tokens": max(0, n_out - untimed), "untimed_output_tokens": untimed,
        "n_iters": n_iters, "avg_accept": accept_total / max(1, n_iters), "ttft": prefill_time,
        "draft_iters": n_iters, "drafted_tokens": D * n_iters, "accepted_drafts": n_out,
        "accept_rate": n_out / max(1, D * n_iters), "verifier_bonus_tokens": 0,
        "committed_tokens": n_out, "committed_per_iter": n_out / max(1, n_iters),
        "conf_path_frac": 1.0, "n_conf_path": n_iters, "n_verify_path": 0,
    }
    return gen, st
