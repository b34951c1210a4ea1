"""Sweep of the packed GEMV over shapes and block widths on one GPU.

``python -m bitmtp_amd.gemv_bench --kind q1 --preset config4 --widths 1-8`` times the drop-in
entry points (``t2g128_int8xint2_linear`` / ``q1g128_int8xint1_linear``) the way ``bench.py``
does: every launch of a HIP graph reads a different matrix of a pool larger than the 256 MB
Infinity Cache, HIP events bracket the replay on the launch stream, the best of three replays
counts.  One JSON line per (shape, width): microseconds per launch, GB/s and percent of the
8 TB/s HBM peak over the algorithmic bytes (packed weights + group scales).

Presets follow the reference's registered decode shapes (``contracts.py:11-20``):
``layer-1.7b`` / ``layer-4b`` are the seven projections of one decoder layer,
``merged-1.7b`` / ``merged-4b`` the four merged matrices a decode step launches, ``config4``
the 1-bit sweep K in {2560, 9728} x N in {1024, 2560, 9728}, ``head`` the 151936-row output
projection.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import sys

HBM_PEAK_GBPS = 8000.0

PRESETS = {
    "layer-1.7b": [(2048, 2048), (1024, 2048), (6144, 2048), (2048, 6144)],
    "merged-1.7b": [(4096, 2048), (2048, 2048), (12288, 2048), (2048, 6144)],
    "layer-4b": [(4096, 2560), (1024, 2560), (2560, 4096), (9728, 2560), (2560, 9728)],
    "merged-4b": [(6144, 2560), (2560, 4096), (19456, 2560), (2560, 9728)],
    "config4": [(n, k) for k in (2560, 9728) for n in (1024, 2560, 9728)],
    "head": [(151936, 2048), (151936, 2560)],
}


def gemv_bytes(kind: str, n: int, k: int) -> int:
    """Algorithmic bytes of one GEMV: packed weights plus bf16 group scales."""
    per_byte = 4 if kind == "t2" else 8
    return n * k // per_byte + n * (k // 128) * 2


def parse_widths(text: str):
    out = []
    for part in text.split(","):
        if "-" in part:
            lo, hi = part.split("-")
            out.extend(range(int(lo), int(hi) + 1))
        else:
            out.append(int(part))
    if not out or min(out) < 1:
        raise ValueError(f"bad width list {text!r}")
    return out


def parse_shapes(text: str):
    shapes = []
    for part in text.split(","):
        n, k = part.lower().split("x")
        shapes.append((int(n), int(k)))
    return shapes


# --kernel: which kernel the single-GEMV entry point is steered to (development hooks of the
# libraries); "auto" is the built-in choice
KERNELS = {"auto": (0, 0), "dot4": (1000, 0), "staged": (1, 1), "operand": (1, 3), "lean": (1, 4),
           "stream": (0, 5), "single-token": (0, 6)}


def sweep(kind: str, shapes, widths, pool_bytes: int = 640 << 20, max_pool: int = 256, seed: int = 4,
          kernel: str = "auto", quiet: bool = False):
    import torch
    import bitmtp_amd as ops
    from bitmtp_amd import ops as ops_mod

    if not torch.cuda.is_available():
        raise RuntimeError("gemv_bench needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ops.init_kernels()
    lib = ops_mod.t2_lib() if kind == "t2" else ops_mod.q1_lib()
    fn = lib.t2g128_int8xint2_linear if kind == "t2" else lib.q1g128_int8xint1_linear
    min_width, engine = KERNELS[kernel]
    (lib.t2g128_set_mfma_tuning if kind == "t2" else lib.q1g128_set_mfma_tuning)(min_width, 0, 0, 0, engine)
    per_byte = 4 if kind == "t2" else 8
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    results = []
    for n, k in shapes:
        if k % 128:
            raise ValueError(f"K = {k} is not a multiple of the group size 128")
        nbytes = gemv_bytes(kind, n, k)
        count = max(4, min(max_pool, pool_bytes // nbytes + 1))
        mats = []
        for _ in range(count):
            if kind == "t2":  # codes 1..3, four per byte, least significant first
                codes = torch.randint(1, 4, (n, k // 4, 4), generator=gen, device=dev, dtype=torch.int32)
                shifts = torch.tensor([1, 4, 16, 64], device=dev, dtype=torch.int32)
                packed = (codes * shifts).sum(-1).to(torch.uint8).view(torch.int8).contiguous()
                del codes
            else:  # i.i.d. sign bits
                packed = torch.randint(-128, 128, (n, k // per_byte), generator=gen, device=dev,
                                       dtype=torch.int8)
            scales = torch.exp(torch.randn(n, k // 128, generator=gen, device=dev) * 0.5 - 4.0)
            mats.append((packed, scales.to(torch.bfloat16).contiguous()))
        for m in widths:
            x = torch.randn(m, k, generator=gen, device=dev).to(torch.float16)
            q, s = ops.quant_input(x)
            out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
            sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for packed, scales in mats[:3]:  # loads the code objects before the capture
                fn(q.data_ptr(), packed.data_ptr(), out.data_ptr(), s.data_ptr(),
                   scales.data_ptr(), m, n, k, sp)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                spc = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for packed, scales in mats:
                    fn(q.data_ptr(), packed.data_ptr(), out.data_ptr(), s.data_ptr(),
                       scales.data_ptr(), m, n, k, spc)
            g.replay()
            torch.cuda.synchronize()
            best = float("inf")
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                g.replay()
                e1.record()
                torch.cuda.synchronize()
                best = min(best, e0.elapsed_time(e1) * 1e-3 / count)
            del g
            results.append({
                "kind": kind, "kernel": kernel, "N": n, "K": k, "width": m, "bytes": nbytes, "pool": count,
                "us_per_launch": round(best * 1e6, 3),
                "gbps": round(nbytes / best / 1e9, 1),
                "pct_hbm_peak": round(nbytes / best / 1e9 / HBM_PEAK_GBPS * 100, 2),
                "launched": ops_mod.last_kernel(2 if kind == "t2" else 1),
            })
            if not quiet:
                print(json.dumps(results[-1]), flush=True)
        del mats
        torch.cuda.empty_cache()
    (lib.t2g128_set_mfma_tuning if kind == "t2" else lib.q1g128_set_mfma_tuning)(0, 0, 0, 0, 0)
    return results


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--kind", choices=("t2", "q1"), default="t2")
    ap.add_argument("--preset", choices=sorted(PRESETS), default=None)
    ap.add_argument("--shapes", default=None, help="comma list of NxK, e.g. 9728x2560,2560x9728")
    ap.add_argument("--widths", default="1,4,8", help="comma list and ranges, e.g. 1-8 or 1,4,8")
    ap.add_argument("--pool-mb", type=int, default=640, help="bytes of distinct matrices per shape")
    ap.add_argument("--kernel", choices=sorted(KERNELS), default="auto",
                    help="steer the entry point to one kernel (profiling runs)")
    args = ap.parse_args()
    if (args.preset is None) == (args.shapes is None):
        print("give exactly one of --preset and --shapes", file=sys.stderr)
        return 2
    shapes = PRESETS[args.preset] if args.preset else parse_shapes(args.shapes)
    sweep(args.kind, shapes, parse_widths(args.widths), pool_bytes=args.pool_mb << 20, kernel=args.kernel)
    return 0


if __name__ == "__main__":
    sys.exit(main())
