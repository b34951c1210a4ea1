"""HIP-graph atlas with shared per-segment KV history and workspace, the MI355X
counterpart of the reference ``GraphAtlas`` (src/bonsai_sft/gpu/fast_runtime.py:76-521).

Graphs are keyed by ``(M, sigma, role)``.  Each segment sigma owns one KV buffer
``[2, n_layers, n_kv, sigma + M_max, 128]``: slots ``[0, sigma)`` are history, the
captured step always writes its M new rows at slot ``sigma`` (so the graph does not
depend on ``cache_len``), and accepted rows are copied down into history afterwards.

Differences from the reference, by design:

* the additive mask tensor ``[1, 1, M, sigma+M]`` and its per-step rebuild
  (fast_runtime.py:391-465) are replaced by a ``2 + M`` word descriptor
  (``cache_len``, one hidden history slot, one workspace-visibility word per row) that
  the attention kernel evaluates, so attention reads ``cache_len + M`` slots instead
  of ``sigma + M``;
* tokens, positions and the descriptor travel in one host-to-device copy per replay and
  argmax / confidence come back in one device-to-host copy;
* intermediate buffers are shared by all graphs; graphs are captured on first use.
"""
from __future__ import annotations

import gc
import time
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

import torch

from . import contracts, decode_ops, ops
from .model import BonsaiDecoder, StepIO, Workspace, enqueue_step, rope_tables

DEFAULT_SEGMENT_LADDER = (256, 1024, 4096)
DEFAULT_M_SET = (1, 8, 9, 10, 12, 16, 17)
ROLES = ("draft", "verify", "ar")


# ---------------------------------------------------------------------------
# Visibility descriptors (host side, pure Python: unit-tested without a GPU)
# ---------------------------------------------------------------------------
def _as_int32(mask: int) -> int:
    """A 32-bit visibility word as the signed value an int32 buffer holds (bit 31 = row 31)."""
    mask &= 0xFFFFFFFF
    return mask - (1 << 32) if mask >= (1 << 31) else mask


def draft_row_masks(M: int, D: int, n_pend: int) -> List[int]:
    """Workspace visibility of a draft step (reference template:
    ``_build_mask_template``, fast_runtime.py:345-372).

    Rows ``[0, n_pend)`` are the pending committed tokens (row r sees workspace rows
    0..r); rows ``[n_pend, P)`` are padding; rows ``[P, M)`` are the block (anchor +
    D-1 masks): block-causal among themselves, and they see the pending rows except
    the last one, which the anchor repeats.
    """
    P = M - D
    if P < 0 or not 0 <= n_pend <= P:
        raise ValueError(f"draft width {M} cannot carry {n_pend} pending rows with D={D}")
    masks = [0] * M
    for r in range(n_pend):
        masks[r] = (1 << (r + 1)) - 1
    earlier = (1 << (n_pend - 1)) - 1 if n_pend > 1 else 0
    for r in range(P, M):
        block = ((1 << (r - P + 1)) - 1) << P
        masks[r] = block | earlier
    return [_as_int32(m) for m in masks]


def causal_row_masks(M: int) -> List[int]:
    """AR-causal workspace visibility of verify / AR steps: row r sees rows 0..r
    (reference: ``_build_verify_templates``, fast_runtime.py:423-441)."""
    return [_as_int32((1 << (r + 1)) - 1) for r in range(M)]


# output projection of each role: the backbone's own ("native"), the FP8 or the raw bf16
# approximation for the acceptance-tolerant draft roles (fast_runtime.py:179-203)
DRAFT_ROLES = ("draft", "draft_fp8", "draft_bf16")
HEAD_MODE_OF_ROLE = {"ar": "native", "verify": "native", "draft": "native",
                     "draft_fp8": "fp8", "draft_bf16": "bf16_raw"}


def step_descriptor(role: str, M: int, D: int, cache_len: int, n_pend: int = 0) -> List[int]:
    """``[cache_len, hide, rowmask_0 .. rowmask_{M-1}]`` for one replay
    (reference: ``prepare_step`` / ``_prepare_verify``, fast_runtime.py:391-421,443-465)."""
    if role in DRAFT_ROLES:  # the three draft roles share the mask
        P = M - D
        n_clamp = max(0, min(n_pend, P))
        hide = cache_len - 1 if (n_clamp == 0 and cache_len > 0) else -1
        return [cache_len, hide] + draft_row_masks(M, D, n_clamp)
    if role == "ar":
        return [cache_len, -1] + causal_row_masks(M)
    if role == "verify":
        if cache_len <= 0:
            raise RuntimeError("batched verifier requires a committed anchor")
        # row 0 replays the anchor that already sits at history slot cache_len-1
        return [cache_len, cache_len - 1] + causal_row_masks(M)
    raise ValueError(f"unsupported graph role: {role!r}")


def dense_visibility(desc: Sequence[int], M: int, sigma: int) -> np.ndarray:
    """Boolean ``[M, sigma+M]`` form of a descriptor (what the reference keeps as an
    additive 0 / -inf mask); used by tests and debugging only."""
    cache_len, hide = desc[0], desc[1]
    vis = np.zeros((M, sigma + M), dtype=bool)
    vis[:, :cache_len] = True
    if hide >= 0:
        vis[:, hide] = False
    for r in range(M):
        for j in range(M):
            if (desc[2 + r] >> j) & 1:
                vis[r, sigma + j] = True
    return vis


def logits_rows(role: str, M: int, D: int) -> Tuple[int, int]:
    """Rows projected through the head (reference: ``_capture_one``, fast_runtime.py:179-203)."""
    if role == "ar":
        return 0, M
    if role in DRAFT_ROLES:
        return M - D, M
    if role == "verify":
        return 0, min(D + 1, M)
    raise ValueError(f"unsupported graph role: {role!r}")


# ---------------------------------------------------------------------------
@dataclass
class CapturedGraph:
    graph: "torch.cuda.CUDAGraph"
    io: StepIO
    M: int
    sigma: int
    role: str
    P: int
    logits_start: int
    logits_end: int


class GraphAtlas:
    """Captured decode steps keyed by ``(M, sigma, role)`` over shared KV."""

    def __init__(self, model: BonsaiDecoder,
                 segment_ladder: Tuple[int, ...] = DEFAULT_SEGMENT_LADDER,
                 m_set: Tuple[int, ...] = DEFAULT_M_SET,
                 roles: Tuple[str, ...] = ROLES,
                 threshold: float = 0.9,
                 prefill_width: int = 32,
                 use_graphs: bool = True):
        contracts.validate_graph_roles(roles)
        self.model = model
        self.args = model.args
        self.device = model.device
        self.segment_ladder = tuple(sorted(set(segment_ladder)))
        self.m_set = tuple(sorted(set(m_set)))
        self.roles = tuple(roles)
        self.D = self.args.block_size
        self.prefill_width = int(prefill_width)
        self.M_max = max(max(self.m_set), self.prefill_width)
        if self.M_max > decode_ops.MAX_WIDTH:
            raise ValueError(f"widths above {decode_ops.MAX_WIDTH} are not supported")
        self.threshold = float(threshold)
        self.use_graphs = bool(use_graphs)
        ops.init_kernels()
        self.kv_buffers: Dict[int, torch.Tensor] = {}
        max_slots = self.segment_ladder[-1] + self.M_max
        # the approximate draft projections are prepared once, like the reference does in
        # GraphAtlas.__init__ (fast_runtime.py:112-118)
        if "draft_fp8" in self.roles:
            contracts.validate_graph_roles(self.roles, torch.cuda.get_device_capability(self.device))
            model.prepare_fp8_lm_head()
        if "draft_bf16" in self.roles:
            model.prepare_raw_bf16_head()
        self.workspace = Workspace(self.args, self.M_max, max_slots, model.head_rows, self.device,
                                   logits_ld_max=model.max_logits_ld())
        self.rope = rope_tables(self.args, max_slots, self.device)
        self.graphs: Dict[Tuple[int, int, str], CapturedGraph] = {}
        self.replays = 0

    def synchronize(self) -> None:
        """Wait for everything queued on the atlas's device (the loops' timing fences)."""
        torch.cuda.synchronize(self.device)

    # -- KV ------------------------------------------------------------------
    def kv(self, sigma: int) -> torch.Tensor:
        """Shared buffer of segment sigma, allocated on first use
        (reference: ``_allocate_shared_kv``, fast_runtime.py:130-138)."""
        buf = self.kv_buffers.get(sigma)
        if buf is None:
            if sigma not in self.segment_ladder:
                raise KeyError(f"segment {sigma} is not in the ladder {self.segment_ladder}")
            buf = torch.zeros(2, self.args.n_layers, self.args.n_kv_heads, sigma + self.M_max,
                              self.args.head_dim, device=self.device, dtype=torch.bfloat16)
            self.kv_buffers[sigma] = buf
        return buf

    def select_segment(self, needed_kv_len: int) -> int:
        """Smallest sigma >= needed_kv_len, else the largest (fast_runtime.py:377-386)."""
        for sigma in self.segment_ladder:
            if needed_kv_len <= sigma:
                return sigma
        return self.segment_ladder[-1]

    def commit_kv(self, sigma: int, cache_len: int, n_accept: int, first_row: int = 0) -> None:
        """Workspace rows ``first_row .. first_row+n_accept-1`` become history rows
        ``cache_len ..`` (``commit_kv`` with first_row 0, ``commit_kv_from_verify`` with
        first_row 1; fast_runtime.py:467-508)."""
        if n_accept <= 0:
            return
        if cache_len + n_accept > sigma:
            raise RuntimeError("KV commit would run past the history segment")
        decode_ops.kv_commit(self.kv(sigma), sigma + first_row, cache_len, n_accept)

    def migrate_segment(self, src_sigma: int, dst_sigma: int, cache_len: int) -> None:
        """Copy live history to another segment's buffer (fast_runtime.py:510-521)."""
        if src_sigma == dst_sigma:
            return
        self.kv(dst_sigma)[:, :, :, :cache_len].copy_(self.kv(src_sigma)[:, :, :, :cache_len])

    # -- graphs --------------------------------------------------------------
    def get_graph(self, M: int, sigma: int, role: str) -> CapturedGraph:
        key = (M, sigma, role)
        g = self.graphs.get(key)
        if g is None:
            g = self._capture_one(M, sigma, role)
            self.graphs[key] = g
        return g

    def capture_all(self) -> None:
        """Capture every (M, sigma, role) the reference captures up front
        (``_capture_all``, fast_runtime.py:154-169)."""
        for sigma in self.segment_ladder:
            for M in self.m_set:
                if M == 1:
                    if "ar" in self.roles:
                        self.get_graph(1, sigma, "ar")
                    continue
                for role in self.roles:
                    if role == "ar" or (role in DRAFT_ROLES and M < self.D) or \
                            (role == "verify" and M != self.D + 1):
                        continue
                    self.get_graph(M, sigma, role)

    def _capture_one(self, M: int, sigma: int, role: str) -> CapturedGraph:
        # The cyclic garbage collector must not run while a stream is capturing: if it finds
        # an unreachable atlas, it destroys that atlas's graphs in the middle of this capture,
        # which aborts the process.  Collect first, then keep the collector off until the
        # capture has ended.  (Capture keeps process-wide state tensors; they must not become
        # inference tensors, hence inference_mode(False).)
        gc.collect()
        gc_was_enabled = gc.isenabled()
        gc.disable()
        try:
            with torch.inference_mode(False):
                return self._capture_one_impl(M, sigma, role)
        finally:
            if gc_was_enabled:
                gc.enable()

    def _capture_one_impl(self, M: int, sigma: int, role: str) -> CapturedGraph:
        if role not in contracts.GRAPH_ROLES:
            raise ValueError(f"unsupported graph role: {role!r}")
        if role not in self.roles:
            raise RuntimeError(f"graph role {role!r} was not requested for this atlas")
        if role in DRAFT_ROLES and M < self.D:
            raise ValueError(f"a draft graph needs M >= D = {self.D}")
        if M > self.M_max:
            raise ValueError(f"width {M} exceeds the atlas maximum {self.M_max}")
        ls, le = logits_rows(role, M, self.D)
        io = StepIO.allocate(M, self.device)
        kv = self.kv(sigma)
        # a harmless valid descriptor for the warm-up / capture launches
        desc = step_descriptor("ar", M, self.D, 0)
        io.step_in_host[: 2 + M] = torch.tensor(desc, dtype=torch.int32)
        io.step_in.copy_(io.step_in_host)

        # the closure holds the pieces, not the atlas: no reference cycle through the graphs
        model, workspace, rope, threshold = self.model, self.workspace, self.rope, self.threshold
        head_mode = HEAD_MODE_OF_ROLE[role]

        def run():
            enqueue_step(model, workspace, io, kv, sigma, rope, ls, le, threshold,
                         head_mode=head_mode)

        graph = None
        if self.use_graphs:
            side = torch.cuda.Stream(device=self.device)
            side.wait_stream(torch.cuda.current_stream(self.device))
            with torch.cuda.stream(side):
                run()  # warm-up outside capture: lazy library set-up happens here
            torch.cuda.current_stream(self.device).wait_stream(side)
            torch.cuda.synchronize(self.device)
            # the graph carries its own upload of the step inputs and download of the results
            # (copy nodes between the pinned mirrors and the device vectors): a replay is one
            # launch call on the host
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                io.step_in.copy_(io.step_in_host, non_blocking=True)
                run()
                io.out_host.copy_(io.out, non_blocking=True)
        cg = CapturedGraph(graph=graph, io=io, M=M, sigma=sigma, role=role, P=M - self.D,
                           logits_start=ls, logits_end=le)
        cg._eager = run
        return cg

    # -- one replay ----------------------------------------------------------
    def replay(self, g: CapturedGraph, tokens: Sequence[int], positions: Sequence[int],
               cache_len: int, n_pend: int = 0) -> None:
        """Upload tokens, positions and the visibility descriptor, then replay."""
        M = g.M
        if len(tokens) != M or len(positions) != M:
            raise ValueError("tokens / positions must have exactly M entries")
        if cache_len + M > g.sigma + M or cache_len > g.sigma:
            raise RuntimeError("history does not fit the segment")
        desc = step_descriptor(g.role, M, self.D, cache_len, n_pend)
        # the previous upload from this pinned buffer must have left the host first
        g.io.uploaded.synchronize()
        host = g.io.step_in_host.numpy()
        host[: 2 + M] = desc
        host[2 + M: 2 + 2 * M] = positions
        host[2 + 2 * M:] = tokens
        stream = torch.cuda.current_stream(self.device)
        if g.graph is not None:
            g.graph.replay()          # uploads, runs the step, downloads the results
            g.io.uploaded.record(stream)
            g.io.downloaded = True
        else:
            g.io.step_in.copy_(g.io.step_in_host, non_blocking=True)
            g.io.uploaded.record(stream)
            g._eager()
            g.io.downloaded = False
        self.replays += 1

    def read_outputs(self, g: CapturedGraph) -> Tuple[np.ndarray, np.ndarray, int]:
        """One device-to-host copy + synchronisation: (argmax tokens, confidences,
        device-side accepted-prefix length) of the projected rows."""
        if g.io.downloaded:
            # the event after the replay: polling it returns sooner than a blocking
            # synchronisation wakes the thread up
            ev = g.io.uploaded
            deadline = time.perf_counter() + 0.05
            while not ev.query():
                if time.perf_counter() > deadline:  # a replay is a millisecond: stop spinning
                    ev.synchronize()
                    break
        else:
            g.io.out_host.copy_(g.io.out, non_blocking=True)
            torch.cuda.current_stream(self.device).synchronize()
        rows = g.logits_end - g.logits_start
        out = g.io.out_host.numpy()
        toks = out[:rows].copy()
        accept = int(out[g.M])
        conf = out[g.M + 2: g.M + 2 + rows].view(np.float32).copy()
        return toks, conf, accept
