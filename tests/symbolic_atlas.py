"""A symbolic stand-in for ``GraphAtlas`` that runs on the CPU.

Every KV slot remembers which (position, token) was written to it; a replay writes its rows
into the workspace slots, expands the real step descriptor (``runtime.step_descriptor`` /
``dense_visibility``) and lets each logit row "predict" from exactly the slots it can see.
The toy language model is a hash of the visible sequence, so a row predicts the true greedy
continuation if and only if it sees every earlier position exactly once and nothing else:
a wrong mask, a missed or doubled KV commit, a stale segment after migration or a wrong
position all change the tokens.  Draft rows (MASK tokens) are answered by an oracle drafter
whose proposals are deliberately wrong at some positions, with a confidence that says so.
"""
from types import SimpleNamespace
from typing import Dict, List, Sequence, Tuple

import numpy as np

from bitmtp_amd import runtime as R

VOCAB = 997
MASK = VOCAB + 1


def next_token(seq: Sequence[int]) -> int:
    """The toy model's greedy continuation of a token sequence."""
    h = 1469598103934665603
    for i, t in enumerate(seq):
        h = ((h ^ (t + 31 * i)) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h % VOCAB


def greedy(prompt: Sequence[int], n: int) -> List[int]:
    seq = list(prompt)
    for _ in range(n):
        seq.append(next_token(seq))
    return seq[len(prompt):]


class SymbolicAtlas:
    def __init__(self, D: int = 8, segment_ladder=(64, 256, 1024), m_set=(1, 8, 9, 10, 12, 16, 17),
                 roles=("draft", "verify", "ar"), prefill_width: int = 32, wrong_every: int = 3):
        self.args = SimpleNamespace(block_size=D, mask_token_id=MASK, vocab_size=VOCAB)
        self.D = D
        self.segment_ladder = tuple(segment_ladder)
        self.m_set = tuple(m_set)
        self.roles = tuple(roles)
        self.prefill_width = prefill_width
        self.M_max = max(max(m_set), prefill_width)
        self.device = "cpu"
        self.wrong_every = wrong_every       # the drafter misses every n-th position (0: never)
        self.kv: Dict[int, List] = {s: [None] * (s + self.M_max) for s in segment_ladder}
        self.replays = 0
        self.log: List[Tuple[str, int]] = []

    # -- the GraphAtlas surface the loops use -----------------------------------
    def synchronize(self) -> None:
        pass

    def select_segment(self, needed: int) -> int:
        for s in self.segment_ladder:
            if needed <= s:
                return s
        return self.segment_ladder[-1]

    def get_graph(self, M: int, sigma: int, role: str):
        if role not in self.roles:
            raise RuntimeError(f"graph role {role!r} was not requested for this atlas")
        ls, le = R.logits_rows(role, M, self.D)
        return SimpleNamespace(M=M, sigma=sigma, role=role, logits_start=ls, logits_end=le, out=None)

    def commit_kv(self, sigma: int, cache_len: int, n: int, first_row: int = 0) -> None:
        if n <= 0:
            return
        assert cache_len + n <= sigma, "KV commit would run past the history segment"
        buf = self.kv[sigma]
        for i in range(n):
            buf[cache_len + i] = buf[sigma + first_row + i]

    def migrate_segment(self, src: int, dst: int, cache_len: int) -> None:
        if src != dst:
            self.kv[dst][:cache_len] = self.kv[src][:cache_len]

    def replay(self, g, tokens, positions, cache_len: int, n_pend: int = 0) -> None:
        M = g.M
        assert len(tokens) == M and len(positions) == M and cache_len <= g.sigma
        buf = self.kv[g.sigma]
        for j in range(M):
            buf[g.sigma + j] = (int(positions[j]), int(tokens[j]))
        desc = R.step_descriptor(g.role, M, self.D, cache_len, n_pend)
        vis = R.dense_visibility(desc, M, g.sigma)
        toks, conf = [], []
        for r in range(g.logits_start, g.logits_end):
            seen = [buf[s] for s in np.nonzero(vis[r])[0]]
            assert all(x is not None for x in seen), "a row sees a slot nobody wrote"
            seen.sort()
            pos = [p for p, _ in seen]
            ctx = [t for _, t in seen]
            masks = sum(1 for t in ctx if t == MASK)
            real = [t for t in ctx if t != MASK]
            # a sound context holds positions 0..n-1 once each, the masks at the end
            sound = pos == list(range(len(pos))) and all(t != MASK for t in ctx[: len(ctx) - masks])
            if not sound:
                toks.append(VOCAB - 1 - (len(toks) % 7))     # garbage, never the right token
                conf.append(0.0)
                continue
            # a MASK row at block offset i stands for the token i+1 places after the anchor:
            # the oracle drafter continues the real context greedily and misses some positions
            seq = list(real)
            for _ in range(masks):
                seq.append(next_token(seq))
            tok = next_token(seq)
            position = len(seq)
            if masks and self.wrong_every and position % self.wrong_every == 0:
                toks.append((tok + 1) % VOCAB)
                conf.append(0.3)
            else:
                toks.append(tok)
                conf.append(0.99 if masks else 0.5)
        g.out = (np.array(toks, dtype=np.int32), np.array(conf, dtype=np.float32))
        self.replays += 1
        self.log.append((g.role, M))

    def read_outputs(self, g):
        toks, conf = g.out
        n = 1
        for c in conf[1:]:
            if not (c > 0.9):
                break
            n += 1
        return toks, conf, n
