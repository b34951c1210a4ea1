#!/usr/bin/env python3
"""Benchmark of the packed T2-g128 GEMV hot path on one MI355X.

Workload (BASELINE.json configs[1]): all seven linear projections of one
Qwen3-1.7B-shaped decoder layer in T2-g128 -- q/o 2048x2048, k/v 1024x2048,
gate/up 6144x2048, down 2048x6144 -- at widths 1, 4 and 8.  One STEP is that set
once.  It is measured two ways:

* grouped (the headline `value`): the seven projections of a width handed to
  ``t2g128_gemv_grouped`` together, one launch per width, 3 launches per step;
* drop-in: one launch per projection through ``t2g128_int8xint2_linear``, the
  reference's own launch structure, 21 launches per step (``config.drop_in``).

Every launch reads a different layer of a pool of distinct random layers larger than
the 256 MB Infinity Cache, so the weights come from HBM; every timed graph walks at
least 512 MB of distinct weights whatever --steps is; the steps are replayed from one
HIP graph so that the Python launch cost is outside the measurement, as in the
reference's graph-replayed decode.

Beside the headline, `config` carries the rest of the target range on the same timing (one
graph per figure over >= 512 MB of distinct weights): BASELINE.json configs[0] (one 6144 x 2048 GEMV
at width 1), the 4B-shaped layer (K = 2560, 4096, 9728) grouped and as its four merged
matrices, the Q1-g128 set of configs[4], both packed lm_heads, and the end-to-end decode runs.
Every figure names the kernel that was launched (read back from the library, not written here).

Prints ONE JSON line: the driver's fields (metric, value, unit, ...), `config`, `roofline` of the
dominant kernel and `cpu_baseline`.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MIN_DISTINCT_BYTES = 512 << 20   # every timed graph walks at least this much distinct weight data


def kernel_sources_digest() -> str:
    """sha256 over the GEMV kernel sources (csrc/*.h, *.hip of the GEMV libraries), the key under
    which profiles/traffic.json records what its counters were measured on."""
    import hashlib
    csrc = os.path.join(ROOT, "bitmtp_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(csrc)):
        if name.startswith("gemv_") or name in ("packed_gemv.hip.h", "wave_reduce.h", "t2g128_kernels.hip"):
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def measured_traffic(width: int):
    """HBM bytes per launch of the grouped kernel at `width` (FETCH_SIZE + WRITE_SIZE of two
    rocprofv3 --pmc runs, each scaled by a 256 MiB copy), read from profiles/traffic.json --
    the file the counter summaries under profiles/ are condensed into.  The file records the
    digest of the kernel sources it was measured on: when the sources have changed since, the
    figure is stale and is NOT reported (None, with a message on stderr)."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            table = json.load(f)
        if table.get("kernel_sources_sha256_16") != kernel_sources_digest():
            print("bench.py: profiles/traffic.json was measured on other kernel sources "
                  f"({table.get('kernel_sources_sha256_16')} != {kernel_sources_digest()}): "
                  "roofline.traffic is not reported; regenerate the counter summaries",
                  file=sys.stderr)
            return None
        return table["grouped_t2_layer_1p7b"][str(width)]["hbm_bytes_per_launch"]
    except (OSError, KeyError, ValueError):
        return None


WIDTHS = (1, 4, 8)
# name, N, K  (Qwen3-1.7B: hidden 2048, 16 q / 8 kv heads x 128, ffn 6144)
PROJECTIONS = (
    ("q_proj", 2048, 2048), ("k_proj", 1024, 2048), ("v_proj", 1024, 2048),
    ("o_proj", 2048, 2048), ("gate_proj", 6144, 2048), ("up_proj", 6144, 2048),
    ("down_proj", 2048, 6144),
)


# Qwen3-4B: hidden 2560, 32 q / 8 kv heads x 128, ffn 9728 (reference shape table,
# src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:113-121)
PROJECTIONS_4B = (
    ("q_proj", 4096, 2560), ("k_proj", 1024, 2560), ("v_proj", 1024, 2560),
    ("o_proj", 2560, 4096), ("gate_proj", 9728, 2560), ("up_proj", 9728, 2560),
    ("down_proj", 2560, 9728),
)
# merged decode matrices as (N, K, indices of the projections concatenated along N)
MERGED_17B = ((4096, 2048, (0, 1, 2)), (2048, 2048, (3,)), (12288, 2048, (4, 5)), (2048, 6144, (6,)))
MERGED_4B = ((6144, 2560, (0, 1, 2)), (2560, 4096, (3,)), (19456, 2560, (4, 5)), (2560, 9728, (6,)))


def t2_bytes(n: int, k: int) -> int:
    """Algorithmic bytes of one T2 GEMV: packed weights + group scales."""
    return n * k // 4 + n * (k // 128) * 2


LAYER_BYTES = sum(t2_bytes(n, k) for _, n, k in PROJECTIONS)  # 13,369,344
LAYER_BYTES_4B = sum(t2_bytes(n, k) for _, n, k in PROJECTIONS_4B)  # 26,808,320


def make_pool(torch, n_layers: int, seed: int, dev, projections=None):
    """Seeded i.i.d. ternary weights (p = 1/3 each, codes 1..3 packed four per byte)
    and log-normal(-4, 0.5) group scales rounded to bf16."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    shifts = torch.tensor([1, 4, 16, 64], device=dev, dtype=torch.int32)
    projections = PROJECTIONS if projections is None else projections
    pool = []
    for _ in range(n_layers):
        layer = []
        for _, n, k in projections:
            codes = torch.randint(1, 4, (n, k // 4, 4), generator=gen, device=dev, dtype=torch.int32)
            packed = (codes * shifts).sum(-1).to(torch.uint8).view(torch.int8).contiguous()
            scales = torch.exp(torch.randn(n, k // 128, generator=gen, device=dev) * 0.5 - 4.0)
            layer.append((packed, scales.to(torch.bfloat16).contiguous()))
        pool.append(layer)
    return pool


def make_pool_matrix(torch, count: int, n: int, k: int, seed: int, dev):
    """`count` distinct packed T2 matrices of one shape (same distributions as make_pool)."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    shifts = torch.tensor([1, 4, 16, 64], device=dev, dtype=torch.int32)
    out = []
    for _ in range(count):
        codes = torch.randint(1, 4, (n, k // 4, 4), generator=gen, device=dev, dtype=torch.int32)
        packed = (codes * shifts).sum(-1).to(torch.uint8).view(torch.int8).contiguous()
        del codes
        scales = torch.exp(torch.randn(n, k // 128, generator=gen, device=dev) * 0.5 - 4.0)
        out.append((packed, scales.to(torch.bfloat16).contiguous()))
    return out


def make_activations(torch, ops, seed: int, dev, ks=None):
    """fp16 N(0,1) activations per width and K, quantised per token on the GPU."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed + 1)
    acts = {}
    for m in WIDTHS:
        for k in sorted({k for _, _, k in PROJECTIONS} if ks is None else set(ks)):
            x = torch.randn(m, k, generator=gen, device=dev).to(torch.float16)
            q, s = ops.quant_input(x)
            acts[(m, k)] = (q, s)
    return acts


class Runner:
    def __init__(self, torch, ops_mod, pool, acts, dev, projections=None):
        self.torch = torch
        self.pool = pool
        self.acts = acts
        self.ops_mod = ops_mod
        self.projections = PROJECTIONS if projections is None else projections
        self.fn = ops_mod.t2_lib().t2g128_int8xint2_linear
        self.grouped = ops_mod.t2_lib().t2g128_gemv_grouped
        self.desc_type = ops_mod.GemvDesc
        self.outs = {(m, i): torch.empty(m, n, dtype=torch.bfloat16, device=dev)
                     for m in WIDTHS for i, (_, n, _) in enumerate(self.projections)}
        self.cursor = 0  # next pool layer

    def launch_layer(self, m: int, stream_ptr):
        layer = self.pool[self.cursor % len(self.pool)]
        self.cursor += 1
        for i, (_, n, k) in enumerate(self.projections):
            q, s = self.acts[(m, k)]
            packed, scales = layer[i]
            self.fn(q.data_ptr(), packed.data_ptr(), self.outs[(m, i)].data_ptr(), s.data_ptr(),
                    scales.data_ptr(), m, n, k, stream_ptr)

    def launch_layer_grouped(self, m: int, stream_ptr):
        """The seven projections of one layer in ONE launch (t2g128_gemv_grouped)."""
        layer = self.pool[self.cursor % len(self.pool)]
        self.cursor += 1
        descs = (self.desc_type * len(self.projections))()
        for i, (_, n, k) in enumerate(self.projections):
            q, s = self.acts[(m, k)]
            packed, scales = layer[i]
            descs[i] = self.desc_type(q.data_ptr(), packed.data_ptr(), self.outs[(m, i)].data_ptr(),
                                      s.data_ptr(), scales.data_ptr(), m, n, k, 0)
        rc = self.grouped(descs, len(self.projections), 0, 0, stream_ptr)
        if rc != 0:
            raise RuntimeError(f"t2g128_gemv_grouped failed with status {rc}")

    def step(self, widths, stream_ptr, grouped=False):
        for m in widths:
            if grouped:
                self.launch_layer_grouped(m, stream_ptr)
            else:
                self.launch_layer(m, stream_ptr)

    def capture(self, n_steps: int, widths, grouped=False):
        torch = self.torch
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for _ in range(n_steps):
                self.step(widths, sp, grouped)
        return g

    def time_graph(self, g) -> float:
        torch = self.torch
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3  # seconds

    def time_stats(self, g, replays: int = 5):
        """(best, median) seconds over `replays` timed replays of one graph."""
        ts = sorted(self.time_graph(g) for _ in range(replays))
        return ts[0], ts[len(ts) // 2]



def read_probe_us(torch, ops_mod, run, nbytes: int, workgroups: int, persistent: bool, dev) -> float:
    """Microseconds per launch of the read probe of the bench-only probe library (the same bytes
    read once from HBM with the GEMV's launch shape and no arithmetic), timed like every other
    figure here: one graph of launches over >= 512 MB of distinct buffers, best of 5 replays."""
    from bitmtp_amd import probe
    return probe.read_probe_us(torch, nbytes, workgroups, persistent, dev, MIN_DISTINCT_BYTES)


def cpu_baseline(budget_s: float):
    """Times the C oracle (OpenMP over output rows) on one layer at widths 1, 4, 8 --
    the same 21 GEMVs as one step -- repeating it until about `budget_s` seconds."""
    import numpy as np
    from oracle import oracle as O
    O.build()
    problems = []
    for m in WIDTHS:
        for _, n, k in PROJECTIONS:
            problems.append(O.synth_problem(1, m, n, k, 2))
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    reps, t_used = 0, 0.0
    while t_used < budget_s and reps < 1000:
        t0 = time.perf_counter()
        for p in problems:
            O.c_gemv(p["A"], p["B"], p["s"], p["ws"], 2)
        t_used += time.perf_counter() - t0
        reps += 1
    total_bytes = reps * len(WIDTHS) * LAYER_BYTES
    res = {
        "value": round(total_bytes / t_used / 1e9, 3), "unit": "GB/s", "cores": threads,
        "kind": "port",
        "sample": f"{reps} x (one 1.7B-shaped layer, 7 T2 projections at widths 1,4,8) in "
                  f"{t_used:.1f} s with the C oracle, OpenMP over rows",
    }
    # Second figure: the only statement of the op the reference can run on a CPU,
    # F.linear(dequantised activations, dequantised weights) in bf16
    # (src/bonsai_sft/gpu/model.py:646-656), with this build's own PyTorch.
    import torch
    import torch.nn.functional as F
    dense = []
    for p in problems:
        w = O.np_unpack(p["B"], 2).astype(np.float32).reshape(p["B"].shape[0], -1, O.GROUP)
        w = (w * O.bf16_bits_to_f32(p["ws"])[:, :, None]).reshape(p["B"].shape[0], -1)
        x = p["A"].astype(np.float32) / p["s"].reshape(-1, 1)
        dense.append((torch.from_numpy(x).to(torch.bfloat16), torch.from_numpy(w).to(torch.bfloat16)))
    reps2, t2 = 0, 0.0
    with torch.no_grad():
        for x, w in dense:   # untimed first pass
            F.linear(x, w)
        while t2 < budget_s / 3 and reps2 < 200:
            t0 = time.perf_counter()
            for x, w in dense:
                F.linear(x, w)
            t2 += time.perf_counter() - t0
            reps2 += 1
    res["torch_cpu_f_linear"] = {
        "value": round(reps2 * len(WIDTHS) * LAYER_BYTES / t2 / 1e9, 3), "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "sample": f"{reps2} x the same 21 products as bf16 F.linear on dequantised operands in "
                  f"{t2:.1f} s (same algorithmic bytes counted)",
    }
    return res


def graph_steps(bytes_per_step: int, steps: int = 0) -> int:
    """Steps per timed graph: at least `steps`, and enough of them to walk >= 512 MB of distinct
    weights (the pools are at least that large)."""
    need = -(-MIN_DISTINCT_BYTES // bytes_per_step)
    return max(steps, need)


def width_table(run, layer_bytes: int, grouped: bool, torch):
    """Per width: one graph of layer launches (grouped: one launch per layer, else one per
    projection) over >= 512 MB of distinct layers; best and median of 5 replays; the kernel the
    last launch of the graph went to."""
    table = {}
    launches_per_layer = 1 if grouped else len(run.projections)
    n = min(graph_steps(layer_bytes), len(run.pool))
    for m in WIDTHS:
        run.cursor = 0
        g = run.capture(n, (m,), grouped=grouped)
        launched = run.ops_mod.last_kernel(2)
        g.replay()
        torch.cuda.synchronize()
        t, t_med = run.time_stats(g)
        table[m] = {
            "gbps": round(layer_bytes * n / t / 1e9, 1),
            "pct_hbm_peak": round(layer_bytes * n / t / 1e9 / HBM_PEAK_GBPS * 100, 2),
            "median_pct_hbm_peak": round(layer_bytes * n / t_med / 1e9 / HBM_PEAK_GBPS * 100, 2),
            "us_per_layer": round(t / n * 1e6, 3),
            "us_per_launch": round(t / (n * launches_per_layer) * 1e6, 3),
            "layers_timed": n,
            "launched": launched,
        }
        del g
    return table


def merged_table(run, merged_shapes, layer_bytes: int, torch, dev):
    """The same layer bytes as the merged matrices a decode step launches (q|k|v and gate|up
    concatenated along N, as the reference's prepare_merged_weights, model.py:931-956,
    1042-1051): one drop-in launch per merged matrix."""
    mpool = [[(torch.cat([layer[i][0] for i in idx]).contiguous(),
               torch.cat([layer[i][1] for i in idx]).contiguous())
              for _, _, idx in merged_shapes] for layer in run.pool]
    mouts = {(m, j): torch.empty(m, n, dtype=torch.bfloat16, device=dev)
             for m in WIDTHS for j, (n, _, _) in enumerate(merged_shapes)}
    n_m = min(graph_steps(layer_bytes), len(mpool))
    merged = {}
    for m in WIDTHS:
        launched = []
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            spc = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for st in range(n_m):
                layer = mpool[st % len(mpool)]
                for j, (n, k, _) in enumerate(merged_shapes):
                    q, s_ = run.acts[(m, k)]
                    run.fn(q.data_ptr(), layer[j][0].data_ptr(), mouts[(m, j)].data_ptr(),
                           s_.data_ptr(), layer[j][1].data_ptr(), m, n, k, spc)
                    if st == 0:
                        launched.append(run.ops_mod.last_kernel(2))
        g.replay()
        torch.cuda.synchronize()
        t, _ = run.time_stats(g)
        merged[str(m)] = {
            "gbps": round(layer_bytes * n_m / t / 1e9, 1),
            "pct_hbm_peak": round(layer_bytes * n_m / t / 1e9 / HBM_PEAK_GBPS * 100, 2),
            "us_per_layer": round(t / n_m * 1e6, 3),
            "us_per_launch": round(t / (n_m * len(merged_shapes)) * 1e6, 3),
            "launched": launched,
        }
        del g
    del mpool
    return merged


def head_table(run, torch, ops_mod, hn: int, hk: int, acts, dev, n_cus: int):
    """One packed lm_head (hn x hk) at every width through the drop-in symbol, HBM-cold over a
    small pool, with the persistent read probe of the same bytes beside it."""
    hbytes = t2_bytes(hn, hk)
    hpool = make_pool_matrix(torch, max(4, -(-MIN_DISTINCT_BYTES // hbytes)), hn, hk, seed=2, dev=dev)
    hout = torch.empty(max(WIDTHS), hn, dtype=torch.bfloat16, device=dev)
    head = {}
    for m in WIDTHS:
        q, s_ = acts[(m, hk)]
        sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        run.fn(q.data_ptr(), hpool[0][0].data_ptr(), hout.data_ptr(), s_.data_ptr(),
               hpool[0][1].data_ptr(), m, hn, hk, sp)
        launched = ops_mod.last_kernel(2)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            spc = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for packed, scales in hpool:
                run.fn(q.data_ptr(), packed.data_ptr(), hout.data_ptr(), s_.data_ptr(),
                       scales.data_ptr(), m, hn, hk, spc)
        g.replay()
        torch.cuda.synchronize()
        t = min(run.time_graph(g) for _ in range(3)) / len(hpool)
        head[str(m)] = {"us_per_launch": round(t * 1e6, 2), "gbps": round(hbytes / t / 1e9, 1),
                        "pct_hbm_peak": round(hbytes / t / 1e9 / HBM_PEAK_GBPS * 100, 1),
                        "launched": launched}
        del g
    del hpool
    probe_us = read_probe_us(torch, ops_mod, run, hbytes, 2 * n_cus, True, dev)
    for m in WIDTHS:
        head[str(m)]["read_probe_us"] = round(probe_us, 2)
        head[str(m)]["pct_of_read_probe"] = round(probe_us / head[str(m)]["us_per_launch"] * 100, 1)
    return head


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=48, help="distinct layers in the weight pool")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget; 0 skips it")
    ap.add_argument("--no-decode", action="store_true",
                    help="skip the end-to-end decode tokens/s section")
    ap.add_argument("--no-head", action="store_true", help="skip the lm_head-sized extra measurements")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip configs[0], the 4B-shaped layer and the Q1 set (profiling runs)")
    ap.add_argument("--widths", default=None,
                    help="comma list restricting the widths measured (profiling runs); default 1,4,8")
    ap.add_argument("--no-drop-in", action="store_true",
                    help="skip the one-launch-per-projection and merged-matrix figures (profiling runs)")
    ap.add_argument("--kernel-digest", action="store_true",
                    help="print the digest of the GEMV kernel sources (the key profiles/traffic.json "
                         "is stored under) and exit; needs no GPU")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device copy (for scaling rocprofv3 PMC byte counters)")
    args = ap.parse_args()
    if args.kernel_digest:
        print(kernel_sources_digest())
        return 0
    global WIDTHS
    if args.widths:
        WIDTHS = tuple(int(w) for w in args.widths.split(","))
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (--gpus must be 1)",
              file=sys.stderr)
        return 2

    import torch
    import bitmtp_amd as ops
    from bitmtp_amd import ops as ops_mod

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ops.init_kernels()
    n_cus = torch.cuda.get_device_properties(dev).multi_processor_count

    pool = make_pool(torch, args.layers, seed=1, dev=dev)
    acts = make_activations(torch, ops, seed=1, dev=dev, ks=(2048, 2560, 4096, 6144, 9728))
    run = Runner(torch, ops_mod, pool, acts, dev)

    # warm-up: eager steps of both launch structures (loads code objects)
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(max(args.warmup, 1)):
        run.step(WIDTHS, sp, grouped=True)
    run.step(WIDTHS, sp, grouped=False)
    torch.cuda.synchronize()

    step_bytes = len(WIDTHS) * LAYER_BYTES

    # ---- headline: grouped, one launch per width, exactly args.steps steps timed; when that
    # is too few to leave the Infinity Cache behind, the graph holds more steps and the time
    # of args.steps of them is reported
    n_g = graph_steps(step_bytes, args.steps)
    run.cursor = 0
    graph = run.capture(n_g, WIDTHS, grouped=True)
    graph.replay()
    torch.cuda.synchronize()
    best, med = run.time_stats(graph)
    elapsed = best * args.steps / n_g
    gbps = step_bytes * n_g / best / 1e9
    ms_per_step = best / n_g * 1e3
    headline_median_gbps = step_bytes * n_g / med / 1e9
    del graph

    per_width = width_table(run, LAYER_BYTES, True, torch)   # 1 launch per layer and width
    # what the machine needs for the bytes of one layer alone: 1280 workgroups (one per 16 rows,
    # as the grouped launch), every thread's loads requested up front
    probe_layer_us = read_probe_us(torch, ops_mod, run, LAYER_BYTES, sum(n for _, n, _ in PROJECTIONS) // 16,
                                   False, dev)
    for m in WIDTHS:
        per_width[m]["read_probe_us"] = round(probe_layer_us, 3)
        per_width[m]["pct_of_read_probe"] = round(probe_layer_us / per_width[m]["us_per_launch"] * 100, 1)
    skip_drop_in = args.no_drop_in
    per_width_dropin = {} if skip_drop_in else width_table(run, LAYER_BYTES, False, torch)  # 7 launches per layer

    # drop-in, all three widths (the reference's launch structure: 21 launches per step)
    drop_in, merged = None, {}
    if not skip_drop_in:
        n_d = graph_steps(step_bytes, args.steps)
        run.cursor = 0
        gd = run.capture(n_d, WIDTHS, grouped=False)
        gd.replay()
        torch.cuda.synchronize()
        t_d, t_d_med = run.time_stats(gd)
        drop_in = {
            "gbps": round(step_bytes * n_d / t_d / 1e9, 1),
            "pct_hbm_peak": round(step_bytes * n_d / t_d / 1e9 / HBM_PEAK_GBPS * 100, 2),
            "ms_per_step": round(t_d / n_d * 1e3, 5),
            "launches_per_step": len(WIDTHS) * len(PROJECTIONS),
            "per_width": {str(m): per_width_dropin[m] for m in WIDTHS},
        }
        del gd
        merged = merged_table(run, MERGED_17B, LAYER_BYTES, torch, dev)

    # roofline of the dominant kernel: the grouped kernel at the width whose launches take the
    # most time; one launch streams one layer (13,369,344 algorithmic bytes).  The kernel's name
    # is what the library reports for that launch.
    dom = max(WIDTHS, key=lambda m: per_width[m]["us_per_launch"])
    bytes_per_launch = LAYER_BYTES
    achieved = bytes_per_launch / (per_width[dom]["us_per_launch"] * 1e-6) / 1e9
    traffic = measured_traffic(dom)
    roofline = {
        "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": None if traffic is None else round(traffic),
        "kernel": f"{per_width[dom]['launched']} (grouped, {len(PROJECTIONS)} descriptors, width {dom})",
        "bytes_per_launch": bytes_per_launch,
        "us_per_launch": per_width[dom]["us_per_launch"],
        "read_probe_us": per_width[dom]["read_probe_us"],
    }

    # ---- the rest of the target range (BASELINE.json: T2 K = 2048..9728, Q1 configs[4])
    config0 = layer_4b = q1_set = None
    if not args.no_extra:
        from bitmtp_amd import gemv_bench
        # configs[0]: a single 6144 x 2048 GEMV at width 1 through the drop-in symbol
        r0 = gemv_bench.sweep("t2", [(6144, 2048)], [1], pool_bytes=MIN_DISTINCT_BYTES, max_pool=512,
                              quiet=True)[0]
        config0 = {k: r0[k] for k in ("N", "K", "width", "bytes", "pool", "us_per_launch", "gbps",
                                      "pct_hbm_peak", "launched")}
        # the 4B-shaped layer: grouped (one launch per layer and width) and as the four merged
        # matrices of a decode step (one drop-in launch each)
        del run, pool
        torch.cuda.empty_cache()
        pool4 = make_pool(torch, max(4, -(-MIN_DISTINCT_BYTES // LAYER_BYTES_4B)), seed=3, dev=dev,
                          projections=PROJECTIONS_4B)
        run4 = Runner(torch, ops_mod, pool4, acts, dev, projections=PROJECTIONS_4B)
        run4.step(WIDTHS, sp, grouped=True)
        torch.cuda.synchronize()
        g4 = width_table(run4, LAYER_BYTES_4B, True, torch)
        probe4 = read_probe_us(torch, ops_mod, run4, LAYER_BYTES_4B,
                               sum(n for _, n, _ in PROJECTIONS_4B) // 16, False, dev)
        for m in WIDTHS:
            g4[m]["read_probe_us"] = round(probe4, 3)
            g4[m]["pct_of_read_probe"] = round(probe4 / g4[m]["us_per_launch"] * 100, 1)
        layer_4b = {
            "bytes_per_layer": LAYER_BYTES_4B,
            "grouped_1_launch_per_layer": {str(m): g4[m] for m in WIDTHS},
            "merged_decode_shapes_4_launches_per_layer": merged_table(run4, MERGED_4B, LAYER_BYTES_4B,
                                                                      torch, dev),
        }
        run = run4
        del pool4
        # configs[4]: Q1-g128, K in {2560, 9728} x N in {1024, 2560, 9728}, drop-in symbol
        q1_rows = gemv_bench.sweep("q1", gemv_bench.PRESETS["config4"], list(WIDTHS),
                                   pool_bytes=MIN_DISTINCT_BYTES, quiet=True)
        q1_set = {}
        for r in q1_rows:
            q1_set.setdefault(f"{r['N']}x{r['K']}", {})[str(r["width"])] = {
                "us_per_launch": r["us_per_launch"], "gbps": r["gbps"],
                "pct_hbm_peak": r["pct_hbm_peak"], "launched": r["launched"]}

    # The bandwidth-bound GEMVs of the models, for scale: the packed lm_heads
    # (151936 x 2048, 82.7 MB; 151936 x 2560, 103.3 MB) at the same widths.
    head, head_4b = {}, {}
    if not args.no_head:
        head = head_table(run, torch, ops_mod, 151936, 2048, acts, dev, n_cus)
        if not args.no_extra:
            head_4b = head_table(run, torch, ops_mod, 151936, 2560, acts, dev, n_cus)

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    # The other half of the headline metric: end-to-end decode tokens/s of the random-init
    # 1.7B-shaped model (configs[2]), AR and D8 hybrid, by the reference's timing contract.
    decode = decode_bf16 = decode_4b = None
    if not args.no_decode:
        del run
        torch.cuda.empty_cache()
        from bitmtp_amd.decode_bench import run_decode_bench
        decode = run_decode_bench("1.7b", prompt_len=256, new_tokens=512, repeats=1)
        torch.cuda.empty_cache()
        # the same model with the output projection kept in bf16 (622 MB per step instead of
        # the 83 MB packed head the reference's graphs use for a ternary backbone)
        decode_bf16 = run_decode_bench("1.7b", prompt_len=256, new_tokens=512, repeats=1,
                                       head_kind="bf16")
        torch.cuda.empty_cache()
        # configs[3]: the 4B-shaped model, 512-token prompt, 1024 new tokens
        decode_4b = run_decode_bench("4b", prompt_len=512, new_tokens=1024, repeats=1)

    cpu = cpu_baseline(args.cpu_seconds) if args.cpu_seconds > 0 else None

    line = {
        "metric": "t2g128_packed_gemv_hbm_throughput", "value": round(gbps, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {
            "workload": "configs[1]: 7 T2-g128 projections of one Qwen3-1.7B-shaped layer at "
                        "widths 1,4,8, grouped: one t2g128_gemv_grouped launch per width "
                        "(3 launches/step), HBM-cold over a pool of distinct layers",
            "pool_layers": args.layers, "pool_bytes": args.layers * LAYER_BYTES,
            "bytes_per_step": step_bytes, "launches_per_step": len(WIDTHS),
            "steps_in_timed_graph": n_g, "seconds_for_steps": round(elapsed, 6),
            "pct_hbm_peak": round(gbps / HBM_PEAK_GBPS * 100, 2),
            "median_pct_hbm_peak": round(headline_median_gbps / HBM_PEAK_GBPS * 100, 2),
            "per_width": {str(m): per_width[m] for m in WIDTHS},
            "timing": "one HIP graph per figure holding >= 512 MB of distinct weights, HIP events "
                      "on the launch stream, best and median of 5 replays",
            "drop_in": drop_in,
            "merged_decode_shapes_4_launches_per_layer": merged,
            "config0_single_6144x2048_width1": config0,
            "layer_4b": layer_4b,
            "q1_config4": q1_set,
            "lm_head_151936x2048": head,
            "lm_head_151936x2560": head_4b,
            "decode_1p7b_d8": decode,
            "decode_1p7b_d8_bf16_lm_head": decode_bf16,
            "decode_4b_d8": decode_4b,
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
