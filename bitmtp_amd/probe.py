"""Measurement aids of the benchmarks (``bench_probe/libbonsai_probe.so``, declared in
include/bonsai_probe.h): what the machine charges for the bytes alone, for a launch, for a
dependent launch and for a hand-over between resident workgroups.  Nothing here is on the
operator path; the reference has no counterpart.

    python -m bitmtp_amd.probe            # prints the machine-cost table as JSON lines

Every figure is taken like the GEMV figures of bench.py: the launches are captured in one HIP
graph (or enqueued on a plain stream where stated), timed with events on the launch stream, best
of five.
"""
from __future__ import annotations

import ctypes
import json
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def probe_lib_path() -> str:
    return os.path.join(_HERE, "bench_probe", "libbonsai_probe.so")


def probe_lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        so = probe_lib_path()
        if not os.path.exists(so):
            raise RuntimeError(f"{so} is missing: build it with `python -m bitmtp_amd.build`")
        lib = ctypes.CDLL(so)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        lib.bonsai_read_probe.argtypes = [vp, ctypes.c_size_t, ci, ci, vp, vp]
        lib.bonsai_read_probe.restype = ci
        lib.bonsai_probe_empty_launches.argtypes = [ci, ci, ci, ci, vp, vp]
        lib.bonsai_probe_empty_launches.restype = ci
        lib.bonsai_probe_chain_launches.argtypes = [ci, vp, vp]
        lib.bonsai_probe_chain_launches.restype = ci
        lib.bonsai_probe_grid_barrier.argtypes = [ci, ci, vp, vp]
        lib.bonsai_probe_grid_barrier.restype = ci
        lib.bonsai_probe_last_arriver.argtypes = [ci, ci, ci, ci, vp, vp, vp]
        lib.bonsai_probe_last_arriver.restype = ci
        _lib = lib
    return _lib


def _stream_ptr(torch):
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _time_us(torch, fn, replays: int = 5) -> float:
    """Best of `replays` event-timed runs of fn() on the current stream, in microseconds."""
    best = float("inf")
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3)
    return best


def _graph_of(torch, enqueue):
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        enqueue(_stream_ptr(torch))
    g.replay()
    torch.cuda.synchronize()
    return g


def read_probe_us(torch, nbytes: int, workgroups: int, persistent: bool, dev,
                  min_distinct_bytes: int = 512 << 20) -> float:
    """Microseconds per launch of ``bonsai_read_probe``: `nbytes` read once from HBM with no
    arithmetic, one graph of launches over at least `min_distinct_bytes` of distinct buffers."""
    lib = probe_lib()
    n = max(2, -(-min_distinct_bytes // nbytes))
    bufs = torch.empty(n, nbytes, dtype=torch.uint8, device=dev).random_(0, 256)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)

    def enqueue(sp):
        for i in range(n):
            rc = lib.bonsai_read_probe(bufs[i].data_ptr(), nbytes, workgroups, int(persistent),
                                       sink.data_ptr(), sp)
            if rc != 0:
                raise RuntimeError(f"bonsai_read_probe returned {rc}")

    enqueue(_stream_ptr(torch))
    torch.cuda.synchronize()
    g = _graph_of(torch, enqueue)
    t = _time_us(torch, g.replay) / n
    del g, bufs
    return t


def launch_cost_us(torch, dev, launches: int = 2000, workgroups: int = 1280, threads: int = 256,
                   lds_bytes: int = 0, dependent: bool = False, graph: bool = True) -> float:
    """Microseconds per launch of a kernel that does nothing (`dependent`: a one-wave kernel
    that increments the word the previous launch wrote), `launches` of them back to back in one
    HIP graph, or enqueued by one native call on a plain stream when `graph` is false."""
    lib = probe_lib()
    word = torch.zeros(4, dtype=torch.int32, device=dev)

    def enqueue(sp):
        if dependent:
            rc = lib.bonsai_probe_chain_launches(launches, word.data_ptr(), sp)
        else:
            rc = lib.bonsai_probe_empty_launches(launches, workgroups, threads, lds_bytes,
                                                 word.data_ptr(), sp)
        if rc != 0:
            raise RuntimeError(f"launch probe returned {rc}")

    enqueue(_stream_ptr(torch))
    torch.cuda.synchronize()
    if graph:
        g = _graph_of(torch, enqueue)
        return _time_us(torch, g.replay) / launches
    return _time_us(torch, lambda: enqueue(_stream_ptr(torch))) / launches


def grid_barrier_us(torch, dev, workgroups: int, barriers: int = 101) -> float:
    """Microseconds per device-wide barrier among `workgroups` resident workgroups through one
    counter: (time of a launch with `barriers` barriers - time with one) / (barriers - 1).
    Raises if a wait ran into its spin limit."""
    lib = probe_lib()
    state = torch.zeros(2, dtype=torch.int32, device=dev)

    def run(nbar):
        def once():
            state.zero_()
            rc = lib.bonsai_probe_grid_barrier(workgroups, nbar, state.data_ptr(), _stream_ptr(torch))
            if rc != 0:
                raise RuntimeError(f"bonsai_probe_grid_barrier returned {rc}")
        t = _time_us(torch, once, replays=4)
        if int(state[1].item()) != 0:
            raise RuntimeError("grid barrier probe: a wait ran into its spin limit")
        return t

    return (run(barriers) - run(1)) / (barriers - 1)


def last_arriver_us(torch, dev, workgroups: int, words: int, launches: int = 500) -> dict:
    """Microseconds per launch, in one HIP graph of `launches` dependent launches each: producers
    only, producers with the arrival counter and the finishing stage fused behind it, and the
    pair (producers, then the finishing stage as a launch of its own)."""
    lib = probe_lib()
    records = torch.zeros(workgroups * 64, dtype=torch.int32, device=dev)
    state = torch.zeros(2, dtype=torch.int32, device=dev)
    out = {}
    for name, modes in (("producers_only", (0,)), ("fused_last_arriver", (1,)), ("two_launches", (0, 2))):
        def enqueue(sp, modes=modes):
            for _ in range(launches):
                for mode in modes:
                    rc = lib.bonsai_probe_last_arriver(1, workgroups, words, mode, records.data_ptr(),
                                                       state.data_ptr(), sp)
                    if rc != 0:
                        raise RuntimeError(f"bonsai_probe_last_arriver returned {rc}")
        state.zero_()
        enqueue(_stream_ptr(torch))
        torch.cuda.synchronize()
        state.zero_()
        g = _graph_of(torch, enqueue)
        out[name] = _time_us(torch, g.replay) / launches
        del g
    return out


def main() -> int:
    import torch
    if not torch.cuda.is_available():
        print("bitmtp_amd.probe needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    out = []

    def emit(name, **kw):
        rec = {"probe": name, **{k: (round(v, 3) if isinstance(v, float) else v) for k, v in kw.items()}}
        out.append(rec)
        print(json.dumps(rec), flush=True)

    for wgs, thr, lds in ((1, 64, 0), (1280, 256, 0), (1280, 256, 32768), (4096, 256, 0), (256, 1024, 0)):
        emit("empty_launch", workgroups=wgs, threads=thr, lds_bytes=lds,
             graph_us=launch_cost_us(torch, dev, workgroups=wgs, threads=thr, lds_bytes=lds),
             stream_us=launch_cost_us(torch, dev, workgroups=wgs, threads=thr, lds_bytes=lds, graph=False))
    emit("dependent_launch", graph_us=launch_cost_us(torch, dev, dependent=True),
         stream_us=launch_cost_us(torch, dev, dependent=True, graph=False))
    layer = 13369344
    emit("read_once", bytes=layer, workgroups=1280, us=read_probe_us(torch, layer, 1280, False, dev))
    emit("read_once", bytes=26808320, workgroups=2560, us=read_probe_us(torch, 26808320, 2560, False, dev))
    head = 82653184
    emit("read_stream", bytes=head, workgroups=512, us=read_probe_us(torch, head, 512, True, dev))
    for wgs in (256, 512, 1024):
        emit("grid_barrier", workgroups=wgs, us_per_barrier=grid_barrier_us(torch, dev, wgs))
    # o / down projection of the 1.7B layer: 128 row tiles of 16 rows; one token is 8 words (16
    # bf16) per workgroup, nine tokens 64+ (capped)
    for wgs, words in ((128, 8), (128, 64), (768, 8)):
        emit("last_arriver", workgroups=wgs, words_per_record=words, **last_arriver_us(torch, dev, wgs, words))
    return 0


if __name__ == "__main__":
    sys.exit(main())
