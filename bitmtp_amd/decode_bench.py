"""End-to-end decode throughput of a random-init packed low-bit model on one MI355X.

    python -m bitmtp_amd.decode_bench --model 1.7b            # 256-token prompt, 512 new
    python -m bitmtp_amd.decode_bench --model 4b --prompt 512 --new 1024
    python -m bitmtp_amd.decode_bench --model 4b --kind q1    # sign weights, bf16 lm_head
    python -m bitmtp_amd.decode_bench --slot-costs            # what each operator costs inside the captured step
    python -m bitmtp_amd.decode_bench --attention-sweep       # attention time against the history length

Reports tokens/s by the reference's timing contract (``timed_decode_tokens /
decode_time``, prefill and the first token excluded; src/bonsai_sft/gpu/fast_generate.py:
1001,1147-1148,1171) for greedy AR, for D8 hybrid decode with the default gate
(threshold 0.9, chain 6) and for a forced-confidence run (threshold 0, chain 1) that
exercises the wide draft graphs.  With random weights the logits are near-uniform, so the
default gate verifies every iteration (draft width 9 + verify width 9, about one token per
iteration); the forced run commits whole blocks.  Prompt ids are uniform random.
"""
from __future__ import annotations

import argparse
import os
import json
import time

import numpy as np
import torch

from .generate import ar_generate, hybrid_generate
from .model import BonsaiDecoder, qwen3_1p7b_args, qwen3_4b_args
from .runtime import GraphAtlas

MODELS = {"1.7b": qwen3_1p7b_args, "4b": qwen3_4b_args}


def run_decode_bench(model_name: str = "1.7b", prompt_len: int = 256, new_tokens: int = 512,
                     seed: int = 2, repeats: int = 2, device: str = "cuda:0",
                     n_layers: int = 0, kernel_kind: str = "t2g128", head_kind=None,
                     draft_precision: str = "native") -> dict:
    over = {"n_layers": n_layers} if n_layers else {}
    over["kernel_kind"] = kernel_kind
    args = MODELS[model_name](**over)
    t0 = time.time()
    model = BonsaiDecoder.random_init(args, seed=seed, device=device, head_kind=head_kind)
    draft_kw = {"fp8": {"use_fp8_draft": True}, "bf16": {"use_bf16_draft": True},
                "native": {}}[draft_precision]
    roles = ("ar", "draft", "verify") + {"fp8": ("draft_fp8",), "bf16": ("draft_bf16",),
                                         "native": ()}[draft_precision]
    atlas = GraphAtlas(model, threshold=0.9, roles=roles)
    torch.cuda.synchronize()
    init_s = time.time() - t0
    rng = np.random.default_rng(seed)
    prompt = rng.integers(0, args.vocab_size, prompt_len).tolist()

    def best(fn):
        res, prefill = None, None
        for _ in range(repeats + 1):   # the first pass also captures the graphs it needs
            out, st = fn()
            prefill = st["prefill_time"] if prefill is None else min(prefill, st["prefill_time"])
            if res is None or st["decode_time"] < res[1]["decode_time"]:
                res = (out, st)
        res[1]["prefill_time"] = prefill   # the fastest prefill seen (capture excluded)
        return res

    out_ar, st_ar = best(lambda: ar_generate(atlas, prompt, max_gen_len=new_tokens))
    out_hy, st_hy = best(lambda: hybrid_generate(atlas, prompt, threshold=0.9,
                                                 max_gen_len=new_tokens, **draft_kw))
    out_fc, st_fc = best(lambda: hybrid_generate(atlas, prompt, threshold=0.0, hybrid_m=1,
                                                 max_gen_len=new_tokens, **draft_kw))

    def line(st, extra=()):
        d = {"tokens_per_s": round(st["timed_decode_tokens"] / st["decode_time"], 1),
             "decode_tokens": st["decode_tokens"], "decode_time_s": round(st["decode_time"], 4),
             "prefill_time_s": round(st["prefill_time"], 4), "n_iters": st["n_iters"]}
        for k in extra:
            d[k] = st[k] if not isinstance(st[k], float) else round(st[k], 3)
        return d

    hy_keys = ("committed_per_iter", "n_conf_path", "n_verify_path", "accept_rate")
    res = {
        "model": f"random-init Qwen3-{model_name}-shaped "
                 f"{'T2-g128' if kernel_kind == 't2g128' else 'Q1-g128'}, {args.n_layers} layers, "
                 f"dim {args.dim}, vocab {args.vocab_size}, "
                 f"{ {'t2': 'packed T2', 'q1': 'packed Q1', 'bf16': 'bf16'}[model.head_kind] } head",
        "draft_projection": draft_precision,
        "prompt_tokens": prompt_len, "new_tokens": new_tokens, "block_size": args.block_size,
        "weight_bytes_per_step": model.weight_bytes_per_step(),
        "init_s": round(init_s, 1),
        "ar": line(st_ar),
        "hybrid_d8_thr0.9_m6": line(st_hy, hy_keys),
        "hybrid_d8_forced_confidence": line(st_fc, hy_keys),
        "graphs_captured": sorted(f"{m}/{s}/{r}" for (m, s, r) in atlas.graphs),
    }
    ar_step_us = 1e6 * st_ar["decode_time"] / max(1, st_ar["timed_decode_tokens"])
    res["ar"]["us_per_step"] = round(ar_step_us, 1)
    res["ar"]["weight_stream_gbps"] = round(res["weight_bytes_per_step"] / ar_step_us / 1e3, 1)
    return res


def run_slot_costs(model_name: str = "1.7b", cache_len: int = 500, device: str = "cuda:0",
                   replays: int = 30) -> dict:
    """What each operator type costs INSIDE the captured step: the step is captured again with
    one operator type left out (its launches are simply not enqueued; the results are garbage,
    only the time counts) and the difference to the complete graph is divided by the launches
    left out.  Width 1 (role ar) and width 9 (role verify).  Measurement only: the operators
    are swapped out through this module's own references, nothing in the libraries changes."""
    from . import decode_ops, model as mdl, ops
    args = MODELS[model_name]()
    model = BonsaiDecoder.random_init(args, seed=0, device=device)
    actq = ops.actq_lib()
    n_layers = args.n_layers

    class WithoutEntryPoints:
        """The activation-producer library with chosen entry points turned into no-ops."""
        def __init__(self, skip):
            self.skip = skip

        def __getattr__(self, name):
            return (lambda *a: 0) if name in self.skip else getattr(actq, name)

    def graph_us(M, role):
        atlas = GraphAtlas(model)
        sigma = atlas.select_segment(1024)
        g = atlas.get_graph(M, sigma, role)
        atlas.replay(g, [1] * M, list(range(cache_len, cache_len + M)), cache_len, 0)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(replays):
            g.graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / replays * 1e3

    saved = (mdl._gemv, decode_ops.qk_norm_rope_kv_write, decode_ops.decode_attention, ops.actq_lib,
             mdl._fused, os.environ.get("BONSAI_FUSED_STEP"))
    out = {"model": model_name, "cache_len": cache_len, "widths": {}}
    try:
        for M, role in ((1, "ar"), (9, "verify")):
            # the ten-launch layer (what widths above two always run)
            os.environ["BONSAI_FUSED_STEP"] = "0"
            base = graph_us(M, role)
            row = {"graph_us": round(base, 1), "launches": 10 * n_layers + 4}
            mdl._gemv = lambda *a, **k: None
            row["gemv_us_per_launch"] = round((base - graph_us(M, role)) / (4 * n_layers + 1), 2)
            mdl._gemv = saved[0]
            decode_ops.qk_norm_rope_kv_write = lambda *a, **k: None
            row["qk_norm_rope_kv_write_us_per_launch"] = round((base - graph_us(M, role)) / n_layers, 2)
            decode_ops.qk_norm_rope_kv_write = saved[1]
            decode_ops.decode_attention = lambda *a, **k: None
            row["attention_us_per_layer_2_launches"] = round((base - graph_us(M, role)) / n_layers, 2)
            decode_ops.decode_attention = saved[2]
            ops.actq_lib = lambda: WithoutEntryPoints({"bonsai_silu_mul_quant_int8"})
            row["silu_mul_quant_us_per_launch"] = round((base - graph_us(M, role)) / n_layers, 2)
            ops.actq_lib = lambda: WithoutEntryPoints({"bonsai_add_rmsnorm_quant_int8",
                                                       "bonsai_rmsnorm_quant_int8"})
            row["add_norm_quant_us_per_launch"] = round((base - graph_us(M, role)) / (2 * n_layers + 1), 2)
            ops.actq_lib = saved[3]
            if M <= ops.FUSED_MAX_TOKENS:
                # the fused layer: each projection by what it reads and stores, and the attention
                # that derives q / k itself and merges its own partials (one launch; two when the
                # merge is a launch of its own)
                os.environ["BONSAI_FUSED_STEP"] = "1"
                plan = mdl.fused_plan(model, M)
                per_layer = 5 if plan.attn else 6
                fbase = graph_us(M, role)
                frow = {"graph_us": round(fbase, 1), "launches": per_layer * n_layers + 5,
                        "attention_launches_per_layer": 1 if plan.attn else 2}
                rope_attn = (decode_ops.decode_attention_rope, decode_ops.decode_attention_rope_parts)
                decode_ops.decode_attention_rope = lambda *a, **k: None
                decode_ops.decode_attention_rope_parts = lambda *a, **k: None
                frow["attention_with_rope_us_per_layer"] = round((fbase - graph_us(M, role)) / n_layers, 2)
                decode_ops.decode_attention_rope, decode_ops.decode_attention_rope_parts = rope_attn
                lw0 = model.layers[0]
                for label, which in (("qkv_norm_in", "wqkv"), ("o_add_out", "wo"),
                                     ("gate_up_norm_in_silu_out", "w_gu"), ("down_amax_in_add_out", "w_down")):
                    shape = (getattr(lw0, which).out_features, getattr(lw0, which).in_features)

                    def without(w, m, stream, _skip=shape, **kw):
                        if (w.out_features, w.in_features) != _skip:
                            saved[4](w, m, stream, **kw)
                    mdl._fused = without
                    n = n_layers - 1 if label == "qkv_norm_in" else n_layers
                    frow[label + "_us_per_launch"] = round((fbase - graph_us(M, role)) / n, 2)
                    mdl._fused = saved[4]
                row["fused_layers"] = frow
            out["widths"][str(M)] = row
    finally:
        (mdl._gemv, decode_ops.qk_norm_rope_kv_write, decode_ops.decode_attention, ops.actq_lib,
         mdl._fused) = saved[:5]
        if saved[5] is None:
            os.environ.pop("BONSAI_FUSED_STEP", None)
        else:
            os.environ["BONSAI_FUSED_STEP"] = saved[5]
    return out


def run_attention_sweep(model_name: str = "1.7b", device: str = "cuda:0", replays: int = 20) -> dict:
    """Time of the attention (chunk pass + merge, two launches) per layer against the length of
    the history, for blocks of one and nine rows: a graph of one call per layer over distinct KV
    buffers (nothing is served from a cache), segment sizes 1024, 4096 and 8192 slots."""
    from . import decode_ops, runtime
    args = MODELS[model_name]()
    n_heads, n_kv, n_layers = args.n_heads, args.n_kv_heads, args.n_layers
    gen = torch.Generator(device=device)
    gen.manual_seed(1)
    rows = []
    for sigma in (1024, 4096, 8192):
        slots = sigma + decode_ops.MAX_WIDTH
        kv = torch.randn(n_layers, 2, n_kv, slots, decode_ops.HEAD_DIM, generator=gen,
                         device=device).to(torch.bfloat16)
        for m, role in ((1, "ar"), (9, "verify")):
            q = torch.randn(m, n_heads, decode_ops.HEAD_DIM, generator=gen, device=device).to(torch.bfloat16)
            scratch = torch.empty(decode_ops.attention_scratch_bytes(m, n_heads, slots) // 4,
                                  dtype=torch.float32, device=device)
            o_q = torch.zeros(m, n_heads * decode_ops.HEAD_DIM, dtype=torch.int8, device=device)
            o_s = torch.zeros(m, dtype=torch.float32, device=device)
            for frac in (0.12, 0.45, 0.95):
                cache_len = int(sigma * frac)
                meta = torch.tensor(runtime.step_descriptor(role, m, args.block_size, cache_len, 0),
                                    dtype=torch.int32, device=device)

                def layers():
                    for layer in range(n_layers):
                        decode_ops.decode_attention(q, kv[layer, 0], kv[layer, 1], meta, scratch, sigma,
                                                    out_q=o_q, out_s=o_s)
                layers()
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    layers()
                graph.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(replays):
                    graph.replay()
                e1.record()
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) / replays / n_layers * 1e3
                kv_bytes = 2 * n_kv * (cache_len + m) * decode_ops.HEAD_DIM * 2
                rows.append({"segment": sigma, "rows": m, "cache_len": cache_len,
                             "us_per_layer": round(us, 2), "kv_gbps": round(kv_bytes / us / 1e3, 1)})
        del kv
    return {"model": model_name, "n_heads": n_heads, "n_kv_heads": n_kv, "attention": rows}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", choices=sorted(MODELS), default="1.7b")
    ap.add_argument("--prompt", type=int, default=256)
    ap.add_argument("--new", type=int, default=512)
    ap.add_argument("--seed", type=int, default=2)
    ap.add_argument("--repeats", type=int, default=2)
    ap.add_argument("--layers", type=int, default=0, help="override the layer count (0 = model's)")
    ap.add_argument("--kind", choices=("t2g128", "q1"), default="t2g128",
                    help="backbone weights: ternary T2-g128 or sign Q1-g128")
    ap.add_argument("--head", choices=("t2", "q1", "bf16"), default=None,
                    help="output projection (default: packed T2 for t2g128, bf16 for q1)")
    ap.add_argument("--draft", choices=("native", "fp8", "bf16"), default="native",
                    help="draft output projection: the backbone's own, or the FP8 / raw bf16 "
                         "approximation (verification always uses the backbone's own)")
    ap.add_argument("--slot-costs", action="store_true",
                    help="instead of tokens/s: the cost of each operator type inside the captured "
                         "step (graphs captured with that operator left out)")
    ap.add_argument("--attention-sweep", action="store_true",
                    help="instead of tokens/s: the attention's time per layer against the history length")
    a = ap.parse_args()
    if a.slot_costs:
        print(json.dumps(run_slot_costs(a.model)))
        return
    if a.attention_sweep:
        print(json.dumps(run_attention_sweep(a.model)))
        return
    print(json.dumps(run_decode_bench(a.model, a.prompt, a.new, a.seed, a.repeats,
                                      n_layers=a.layers, kernel_kind=a.kind, head_kind=a.head,
                                      draft_precision=a.draft)))


if __name__ == "__main__":
    main()
