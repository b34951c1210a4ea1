#!/usr/bin/env python3
"""Benchmark of the packed T2-g128 GEMV hot path on one MI355X.

Workload (BASELINE.json configs[1]): all seven linear projections of one
Qwen3-1.7B-shaped decoder layer in T2-g128 -- q/o 2048x2048, k/v 1024x2048,
gate/up 6144x2048, down 2048x6144 -- at widths 1, 4 and 8, through the drop-in
C entry point ``t2g128_int8xint2_linear``.  One STEP is that set once: 3 widths x
7 projections = 21 launches.  Every launch reads a different layer of a pool of
distinct random layers larger than the 256 MB Infinity Cache, so the weights come
from HBM, and the steps are replayed from one HIP graph so that the Python launch
cost is outside the measurement, as in the reference's graph-replayed decode.

Prints ONE JSON line: the driver's fields (metric, value, unit, ...), `config` with the
per-width, merged-shape, lm_head and end-to-end decode figures, `roofline` of the slowest
layer kernel and `cpu_baseline`.
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
# HBM bytes per launch (FETCH_SIZE + WRITE_SIZE, each scaled by a 256 MiB copy), from the
# two rocprofv3 --pmc runs summarised under profiles/: mean over the seven launches of a
# width.  Not measured live.
MEASURED_TRAFFIC_BYTES = {1: (1971.3 + 6.9) * 1024, 4: (2031.1 + 22.9) * 1024,
                          8: (2115.2 + 45.7) * 1024}
WIDTHS = (1, 4, 8)
# name, N, K  (Qwen3-1.7B: hidden 2048, 16 q / 8 kv heads x 128, ffn 6144)
PROJECTIONS = (
    ("q_proj", 2048, 2048), ("k_proj", 1024, 2048), ("v_proj", 1024, 2048),
    ("o_proj", 2048, 2048), ("gate_proj", 6144, 2048), ("up_proj", 6144, 2048),
    ("down_proj", 2048, 6144),
)


def t2_bytes(n: int, k: int) -> int:
    """Algorithmic bytes of one T2 GEMV: packed weights + group scales."""
    return n * k // 4 + n * (k // 128) * 2


LAYER_BYTES = sum(t2_bytes(n, k) for _, n, k in PROJECTIONS)  # 13,369,344


def make_pool(torch, n_layers: int, seed: int, dev):
    """Seeded i.i.d. ternary weights (p = 1/3 each, codes 1..3 packed four per byte)
    and log-normal(-4, 0.5) group scales rounded to bf16."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    shifts = torch.tensor([1, 4, 16, 64], device=dev, dtype=torch.int32)
    pool = []
    for _ in range(n_layers):
        layer = []
        for _, n, k in PROJECTIONS:
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


def make_activations(torch, ops, seed: int, dev):
    """fp16 N(0,1) activations per width and K, quantised per token on the GPU."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed + 1)
    acts = {}
    for m in WIDTHS:
        for k in sorted({k for _, _, k in PROJECTIONS}):
            x = torch.randn(m, k, generator=gen, device=dev).to(torch.float16)
            q, s = ops.quant_input(x)
            acts[(m, k)] = (q, s)
    return acts


class Runner:
    def __init__(self, torch, ops_mod, pool, acts, dev):
        self.torch = torch
        self.pool = pool
        self.acts = acts
        self.fn = ops_mod.t2_lib().t2g128_int8xint2_linear
        self.outs = {(m, i): torch.empty(m, n, dtype=torch.bfloat16, device=dev)
                     for m in WIDTHS for i, (_, n, _) in enumerate(PROJECTIONS)}
        self.cursor = 0  # next pool layer

    def launch_layer(self, m: int, stream_ptr):
        layer = self.pool[self.cursor % len(self.pool)]
        self.cursor += 1
        for i, (_, n, k) in enumerate(PROJECTIONS):
            q, s = self.acts[(m, k)]
            packed, scales = layer[i]
            self.fn(q.data_ptr(), packed.data_ptr(), self.outs[(m, i)].data_ptr(), s.data_ptr(),
                    scales.data_ptr(), m, n, k, stream_ptr)

    def step(self, widths, stream_ptr):
        for m in widths:
            self.launch_layer(m, stream_ptr)

    def capture(self, n_steps: int, widths):
        torch = self.torch
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for _ in range(n_steps):
                self.step(widths, sp)
        return g

    def capture_concurrent(self, n_steps: int, widths, n_streams: int):
        """The same launches spread round-robin over `n_streams` forked streams inside one
        graph: the projections of a step do not depend on each other, so this shows what the
        kernels stream when a launch does not wait for its predecessor."""
        torch = self.torch
        g = torch.cuda.CUDAGraph()
        sides = [torch.cuda.Stream() for _ in range(n_streams)]
        with torch.cuda.graph(g):
            main = torch.cuda.current_stream()
            for s in sides:
                s.wait_stream(main)
            k = 0
            for _ in range(n_steps):
                for m in widths:
                    layer = self.pool[self.cursor % len(self.pool)]
                    self.cursor += 1
                    for i, (_, n, kk) in enumerate(PROJECTIONS):
                        q, s_ = self.acts[(m, kk)]
                        packed, scales = layer[i]
                        st = sides[k % n_streams]
                        k += 1
                        self.fn(q.data_ptr(), packed.data_ptr(), self.outs[(m, i)].data_ptr(),
                                s_.data_ptr(), scales.data_ptr(), m, n, kk,
                                ctypes.c_void_p(st.cuda_stream))
            for s in sides:
                main.wait_stream(s)
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


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=192)
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--layers", type=int, default=48, help="distinct layers in the weight pool")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget; 0 skips it")
    ap.add_argument("--no-decode", action="store_true",
                    help="skip the end-to-end decode tokens/s section")
    ap.add_argument("--no-head", action="store_true", help="skip the lm_head-sized extra measurement")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device copy (for scaling rocprofv3 PMC byte counters)")
    args = ap.parse_args()
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

    pool = make_pool(torch, args.layers, seed=1, dev=dev)
    acts = make_activations(torch, ops, seed=1, dev=dev)
    run = Runner(torch, ops_mod, pool, acts, dev)

    # warm-up: eager steps (loads code objects), then one untimed replay of the timed graph
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(max(args.warmup, 1)):
        run.step(WIDTHS, sp)
    torch.cuda.synchronize()

    run.cursor = 0
    graph = run.capture(args.steps, WIDTHS)
    graph.replay()
    torch.cuda.synchronize()
    elapsed = min(run.time_graph(graph) for _ in range(3))

    step_bytes = len(WIDTHS) * LAYER_BYTES
    gbps = step_bytes * args.steps / elapsed / 1e9
    ms_per_step = elapsed / args.steps * 1e3

    # per-width: the same stream with one width only (7 launches per step)
    per_width = {}
    for m in WIDTHS:
        run.cursor = 0
        g = run.capture(args.steps, (m,))
        g.replay()
        torch.cuda.synchronize()
        t = min(run.time_graph(g) for _ in range(3))
        launches = args.steps * len(PROJECTIONS)
        per_width[m] = {
            "gbps": round(LAYER_BYTES * args.steps / t / 1e9, 1),
            "pct_hbm_peak": round(LAYER_BYTES * args.steps / t / 1e9 / HBM_PEAK_GBPS * 100, 2),
            "us_per_layer": round(t / args.steps * 1e6, 3),
            "us_per_launch": round(t / launches * 1e6, 3),
        }
        del g

    # the same layer bytes in the four merged matrices the decode step launches
    # (q|k|v and gate|up concatenated along N, as the reference's prepare_merged_weights,
    # model.py:931-956,1042-1051): 4 launches per layer instead of 7
    merged_shapes = ((4096, 2048, (0, 1, 2)), (2048, 2048, (3,)), (12288, 2048, (4, 5)),
                     (2048, 6144, (6,)))
    mpool = [[(torch.cat([layer[i][0] for i in idx]).contiguous(),
               torch.cat([layer[i][1] for i in idx]).contiguous())
              for _, _, idx in merged_shapes] for layer in pool]
    mouts = {(m, j): torch.empty(m, n, dtype=torch.bfloat16, device=dev)
             for m in WIDTHS for j, (n, _, _) in enumerate(merged_shapes)}
    merged = {}
    for m in WIDTHS:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            spc = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for st in range(args.steps):
                layer = mpool[st % len(mpool)]
                for j, (n, k, _) in enumerate(merged_shapes):
                    q, s_ = acts[(m, k)]
                    run.fn(q.data_ptr(), layer[j][0].data_ptr(), mouts[(m, j)].data_ptr(),
                           s_.data_ptr(), layer[j][1].data_ptr(), m, n, k, spc)
        g.replay()
        torch.cuda.synchronize()
        t = min(run.time_graph(g) for _ in range(3))
        merged[str(m)] = {
            "gbps": round(LAYER_BYTES * args.steps / t / 1e9, 1),
            "pct_hbm_peak": round(LAYER_BYTES * args.steps / t / 1e9 / HBM_PEAK_GBPS * 100, 2),
            "us_per_layer": round(t / args.steps * 1e6, 3),
            "us_per_launch": round(t / (args.steps * len(merged_shapes)) * 1e6, 3),
        }
        del g
    del mpool

    # secondary figure: the same 21 launches per step on four forked streams of one graph
    # (two launches may write the same output buffer at once: the values are not used)
    run.cursor = 0
    gc_ = run.capture_concurrent(args.steps, WIDTHS, 4)
    gc_.replay()
    torch.cuda.synchronize()
    t_conc = min(run.time_graph(gc_) for _ in range(3))
    concurrent = {
        "streams": 4, "gbps": round(step_bytes * args.steps / t_conc / 1e9, 1),
        "pct_hbm_peak": round(step_bytes * args.steps / t_conc / 1e9 / HBM_PEAK_GBPS * 100, 2),
        "us_per_launch": round(t_conc / (args.steps * len(WIDTHS) * len(PROJECTIONS)) * 1e6, 3),
        "note": "independent projections overlapped; `value` is the serial figure",
    }
    del gc_

    # roofline of the dominant kernel: the width whose launches take the most time
    dom = max(WIDTHS, key=lambda m: per_width[m]["us_per_launch"])
    bytes_per_launch = LAYER_BYTES / len(PROJECTIONS)
    achieved = bytes_per_launch / (per_width[dom]["us_per_launch"] * 1e-6) / 1e9
    roofline = {
        "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": round(MEASURED_TRAFFIC_BYTES[dom]),
        "kernel": (f"gemv_mfma_direct_kernel<BITS=2> (width {dom})" if dom >= 3
                   else f"gemv_dot4_kernel<BITS=2, MT={dom}> (width {dom})"),
        "bytes_per_launch": round(bytes_per_launch),
        "us_per_launch": per_width[dom]["us_per_launch"],
    }

    # The one bandwidth-bound GEMV of the model, for scale: the packed lm_head
    # (151936 x 2048, 82.7 MB) at the same widths, HBM-cold over a small pool.
    head = {}
    if not args.no_head:
        hn, hk = 151936, 2048
        hbytes = t2_bytes(hn, hk)
        hpool = make_pool_matrix(torch, 8, hn, hk, seed=2, dev=dev)
        hout = torch.empty(max(WIDTHS), hn, dtype=torch.bfloat16, device=dev)
        for m in WIDTHS:
            q, s_ = acts[(m, hk)]
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
                            "pct_hbm_peak": round(hbytes / t / 1e9 / HBM_PEAK_GBPS * 100, 1)}
            del g
        del hpool

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    # The other half of the headline metric: end-to-end decode tokens/s of the random-init
    # 1.7B-shaped model (configs[2]), AR and D8 hybrid, by the reference's timing contract.
    decode = decode_bf16 = decode_4b = None
    if not args.no_decode:
        del run, pool, graph
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
                        "widths 1,4,8 (21 launches/step), HBM-cold over a pool of distinct layers",
            "pool_layers": args.layers, "pool_bytes": args.layers * LAYER_BYTES,
            "bytes_per_step": step_bytes, "launches_per_step": len(WIDTHS) * len(PROJECTIONS),
            "pct_hbm_peak": round(gbps / HBM_PEAK_GBPS * 100, 2),
            "per_width": {str(m): per_width[m] for m in WIDTHS},
            "timing": "one HIP graph of all steps, HIP events on the launch stream, best of 3 replays",
            "merged_decode_shapes_4_launches_per_layer": merged,
            "concurrent_streams": concurrent,
            "lm_head_151936x2048": head,
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
