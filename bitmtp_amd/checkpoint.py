"""Packed checkpoint format: conversion from Hugging Face safetensors and loading into
the MI355X decoder.

The on-disk format is the reference's, byte for byte, so files written by either side load
on the other (src/bonsai_sft/gpu/convert_bonsai_mtp_to_gpu.py:37-66,150-278,
src/bonsai_sft/gpu/checkpoint_validation.py, src/bonsai_sft/gpu/generate.py:30-68):

``model_state_t2g128.pt`` / ``model_state_q1g128.pt``
    a ``torch.save``d dict: ``layers.{i}.attention.{q,k,v,o}_proj.weight`` int8 packed
    ``[N, K/4]`` (T2) or ``[N, K/8]`` (Q1) with ``.weight_scale`` bf16 ``[N, K/128]``;
    ``layers.{i}.feed_forward.{gate,up,down}_proj`` likewise; norm weights,
    ``attention.{q,k}_norm.weight`` and ``embed_tokens.weight`` (frozen onto the grid) bf16.
``model_state_fp16.pt``
    the same keys with frozen-grid bf16 matrices instead of packed ones.
``bonsai_gpu_config.json``
    the ModelArgs fields.

Everything here is offline host code (PyTorch on the CPU); files are read with
``weights_only=True`` / safetensors, which execute nothing from the file.
"""
from __future__ import annotations

import json
import math
import os
from pathlib import Path
from typing import Dict, List, Optional, Tuple

import torch

from .packing import GROUP_SIZE, merge_packed_rows, pack_q1_g128, pack_t2_g128

_LIN_SUFFIXES = (
    ".q_proj.weight", ".k_proj.weight", ".v_proj.weight", ".o_proj.weight",
    ".gate_proj.weight", ".up_proj.weight", ".down_proj.weight",
)
_EMBED_KEY = "embed_tokens.weight"


# ---------------------------------------------------------------------------
# key mapping and grids
# ---------------------------------------------------------------------------
def hf_to_gpu_key(hf_key: str) -> str:
    """HF Qwen3 state-dict key -> packed-checkpoint key
    (``_hf_to_gpu_key``, convert_bonsai_mtp_to_gpu.py:37-66)."""
    if hf_key == "model.embed_tokens.weight":
        return "embed_tokens.weight"
    if hf_key == "model.norm.weight":
        return "norm.weight"
    if hf_key.startswith("model.layers."):
        k = "layers." + hf_key[len("model.layers."):]
        k = k.replace(".self_attn.", ".attention.")
        for proj in ("gate_proj", "up_proj", "down_proj"):
            k = k.replace(f".mlp.{proj}.", f".feed_forward.{proj}.")
        return k
    return hf_key


def is_quantised(gpu_key: str, *, quantize_embedding: bool = True) -> bool:
    if gpu_key == _EMBED_KEY:
        return quantize_embedding
    return gpu_key.endswith(_LIN_SUFFIXES)


@torch.no_grad()
def freeze_ternary_g128(w: torch.Tensor) -> torch.Tensor:
    """Latent weights -> {-s, 0, +s} per group of 128, s = max(absmax, 1e-8), computed in
    fp32 and cast back (``_ternary_quantize``, src/bonsai_sft/ternary_modules.py:22-34)."""
    n, k = w.shape
    if k % GROUP_SIZE:
        raise ValueError(f"ternary quant: in_features={k} not divisible by group={GROUP_SIZE}")
    g = w.detach().float().view(n, k // GROUP_SIZE, GROUP_SIZE)
    s = g.abs().amax(dim=-1, keepdim=True).clamp_min(1e-8)
    return (torch.round(g / s).clamp_(-1, 1) * s).view(n, k).to(w.dtype)


@torch.no_grad()
def freeze_q1_g128(w: torch.Tensor) -> torch.Tensor:
    """Latent weights -> +-d per group of 128, d = max(mean|w|, 1e-5); zero counts as +
    (``freeze_quantize_to_q1_0_g128``, src/bonsai_sft/binary_modules.py:152-170)."""
    n, k = w.shape
    if k % GROUP_SIZE:
        raise ValueError(f"q1 quant: in_features={k} not divisible by group={GROUP_SIZE}")
    g = w.detach().float().view(n, k // GROUP_SIZE, GROUP_SIZE)
    d = g.abs().mean(dim=-1, keepdim=True).clamp_min(1e-5)
    q = torch.where(g < 0, -d, d.expand_as(g))
    return q.reshape(n, k).to(w.dtype)


# ---------------------------------------------------------------------------
# source validation (read-only)
# ---------------------------------------------------------------------------
def _positive_number(value, name: str, *, integer: bool = False) -> None:
    ok_type = type(value) is int if integer else type(value) in (int, float)
    if not ok_type or not math.isfinite(value) or value <= 0:
        kind = "integer" if integer else "number"
        raise ValueError(f"config.json: {name} must be a positive {kind}")


def expected_tensor_shapes(config: dict) -> Dict[str, Tuple[int, ...]]:
    """Core tensors the decoder consumes, all layers
    (checkpoint_validation.py:17-45)."""
    dim, vocab, head = config["hidden_size"], config["vocab_size"], config["head_dim"]
    query = config["num_attention_heads"] * head
    kv = config["num_key_value_heads"] * head
    ffn = config["intermediate_size"]
    shapes: Dict[str, Tuple[int, ...]] = {
        "model.embed_tokens.weight": (vocab, dim), "model.norm.weight": (dim,)}
    if not config["tie_word_embeddings"]:
        shapes["lm_head.weight"] = (vocab, dim)
    per_layer = {
        "input_layernorm.weight": (dim,), "post_attention_layernorm.weight": (dim,),
        "self_attn.q_proj.weight": (query, dim), "self_attn.k_proj.weight": (kv, dim),
        "self_attn.v_proj.weight": (kv, dim), "self_attn.o_proj.weight": (dim, query),
        "self_attn.q_norm.weight": (head,), "self_attn.k_norm.weight": (head,),
        "mlp.gate_proj.weight": (ffn, dim), "mlp.up_proj.weight": (ffn, dim),
        "mlp.down_proj.weight": (dim, ffn),
    }
    for layer in range(config["num_hidden_layers"]):
        for key, shape in per_layer.items():
            shapes[f"model.layers.{layer}.{key}"] = shape
    return shapes


def validate_hf_checkpoint(src_ckpt_dir) -> Tuple[dict, List[str]]:
    """Config and shard names after checking container / key / shape metadata; tensor
    values are not read and nothing is written (checkpoint_validation.py:48-126)."""
    from safetensors import safe_open

    source = Path(src_ckpt_dir)
    config_path = source / "config.json"
    if not config_path.is_file():
        raise ValueError(f"missing HF config.json: {config_path}")
    try:
        config = json.loads(config_path.read_text())
    except (OSError, ValueError) as error:
        raise ValueError(f"cannot read valid HF config.json: {config_path}") from error
    if not isinstance(config, dict):
        raise ValueError("config.json must contain a JSON object")
    for key in ("hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                "head_dim", "intermediate_size", "vocab_size"):
        _positive_number(config.get(key), key, integer=True)
    for key in ("rms_norm_eps", "rope_theta"):
        _positive_number(config.get(key), key)
    if type(config.get("tie_word_embeddings")) is not bool:
        raise ValueError("config.json: tie_word_embeddings must be an explicit boolean")
    rope = config.get("rope_scaling")
    if not isinstance(rope, dict):
        raise ValueError("config.json: Bonsai rope_scaling metadata is required")
    _positive_number(rope.get("original_max_position_embeddings"),
                     "rope_scaling.original_max_position_embeddings", integer=True)
    _positive_number(rope.get("factor"), "rope_scaling.factor")
    if config["num_attention_heads"] % config["num_key_value_heads"]:
        raise ValueError("config.json: attention heads must be divisible by key/value heads")
    if config["head_dim"] % 2:
        raise ValueError("config.json: head_dim must be even for rotary embedding")
    for name, width in (("hidden_size", config["hidden_size"]),
                        ("intermediate_size", config["intermediate_size"]),
                        ("query projection width",
                         config["num_attention_heads"] * config["head_dim"])):
        if width % GROUP_SIZE:
            raise ValueError(f"config.json: {name} must be divisible by group size 128")
    _positive_number(config.get("block_size", 8), "block_size", integer=True)
    if type(config.get("causal_attn", True)) is not bool:
        raise ValueError("config.json: causal_attn must be a boolean")
    mask = config.get("text_mask_token_id", 151654)
    if type(mask) is not int or not 0 <= mask < config["vocab_size"]:
        raise ValueError("config.json: text_mask_token_id must index the checkpoint vocabulary")

    shards = sorted(p for p in source.glob("*.safetensors") if p.is_file())
    if not shards:
        raise ValueError(
            "No HF safetensors weight shards found. A config/card or .bin-only checkpoint is not "
            "sufficient; export the complete HF model with "
            "save_pretrained(..., safe_serialization=True) before conversion.")
    expected = expected_tensor_shapes(config)
    allowed = dict(expected)
    if config["tie_word_embeddings"]:
        allowed["lm_head.weight"] = (config["vocab_size"], config["hidden_size"])
    seen = set()
    for shard in shards:
        try:
            with safe_open(str(shard), framework="pt", device="cpu") as reader:
                keys = list(reader.keys())
                if not keys:
                    raise ValueError(f"empty safetensors shard: {shard.name}")
                for key in keys:
                    if key in seen:
                        raise ValueError(f"duplicate tensor key across shards: {key}")
                    if key not in allowed:
                        raise ValueError(f"unsupported tensor key for Bonsai GPU conversion: {key}")
                    meta = reader.get_slice(key)
                    shape = tuple(meta.get_shape())
                    if shape != allowed[key]:
                        raise ValueError(f"tensor shape mismatch for {key}: {shape} != {allowed[key]}")
                    if meta.get_dtype() not in ("F16", "BF16", "F32", "F64"):
                        raise ValueError(f"{key} must contain floating-point HF weights, "
                                         "not packed/integer weights")
                    seen.add(key)
        except Exception as error:
            raise ValueError(f"invalid HF safetensors shard {shard.name}: {error}") from error
    missing = sorted(set(expected) - seen)
    if missing:
        raise ValueError(f"incomplete HF checkpoint: missing {len(missing)} core tensors: {missing[:5]}")
    return config, [p.name for p in shards]


def validate_sdlm_config(ckpt_dir, config: dict):
    """Optional ``sdlm_config.json`` sidecar must agree with config.json
    (src/bonsai_sft/export_ternary.py:32-54)."""
    path = os.path.join(ckpt_dir, "sdlm_config.json")
    if not os.path.isfile(path):
        return None
    with open(path, encoding="utf-8") as source:
        saved = json.load(source)
    if not isinstance(saved, dict):
        raise ValueError("sdlm_config.json must contain a JSON object")
    for key, kind in (("block_size", int), ("causal_attn", bool), ("text_mask_token_id", int)):
        value = saved.get(key)
        if type(value) is not kind:
            raise ValueError(f"sdlm_config.json: invalid or missing {key}")
        hf_value = config.get(key)
        if type(hf_value) is not kind or hf_value != value:
            raise ValueError(f"sdlm_config.json conflicts with config.json: {key}")
    if saved["block_size"] <= 0:
        raise ValueError("sdlm_config.json: block_size must be positive")
    if not 0 <= saved["text_mask_token_id"] < config["vocab_size"]:
        raise ValueError("sdlm_config.json: text_mask_token_id is outside the vocabulary")
    return saved


# ---------------------------------------------------------------------------
# convert
# ---------------------------------------------------------------------------
@torch.no_grad()
def convert(src_ckpt_dir: str, out_dir: str, pack_kernel: bool = True, pack_fp16: bool = True,
            quant: str = "q1", quantize_embedding: bool = True) -> None:
    """Freeze HF weights onto the requested grid and pack them
    (``convert``, convert_bonsai_mtp_to_gpu.py:150-278): same options, same checks in the
    same order, same output files.  Nothing is written unless the whole source converted."""
    from safetensors import safe_open

    if quant not in ("q1", "ternary"):
        raise ValueError("quant must be 'q1' or 'ternary'")
    if os.path.lexists(out_dir):
        raise ValueError("conversion output already exists; use a new output directory")
    if not pack_kernel and not pack_fp16:
        raise ValueError("at least one output format must be enabled")
    if quant == "ternary" and not quantize_embedding:
        raise ValueError("ternary requires quantized embedding/head; --keep-embedding-fp is Q1-only")
    hf_config, shards = validate_hf_checkpoint(src_ckpt_dir)
    validate_sdlm_config(src_ckpt_dir, hf_config)
    freeze = freeze_ternary_g128 if quant == "ternary" else freeze_q1_g128
    pack = pack_t2_g128 if quant == "ternary" else pack_q1_g128

    state_fp16: Dict[str, torch.Tensor] = {}
    state_packed: Dict[str, torch.Tensor] = {}
    for shard in shards:
        with safe_open(os.path.join(src_ckpt_dir, shard), framework="pt", device="cpu") as reader:
            for hf_key in reader.keys():
                if hf_key.startswith("lm_head.") and hf_config["tie_word_embeddings"]:
                    continue  # tied to embed_tokens at run time
                t = reader.get_tensor(hf_key).to(torch.bfloat16)
                gpu_key = hf_to_gpu_key(hf_key)
                if not is_quantised(gpu_key, quantize_embedding=quantize_embedding):
                    if pack_fp16:
                        state_fp16[gpu_key] = t
                    if pack_kernel:
                        state_packed[gpu_key] = t
                    continue
                if t.dim() != 2:
                    raise ValueError(f"unexpected non-2D quantised tensor {hf_key}: {tuple(t.shape)}")
                if t.shape[1] % GROUP_SIZE:
                    # not groupable: kept as bf16 in both files, as the reference does
                    if pack_fp16:
                        state_fp16[gpu_key] = t
                    if pack_kernel:
                        state_packed[gpu_key] = t
                    continue
                frozen = freeze(t)
                if pack_fp16:
                    state_fp16[gpu_key] = frozen
                if pack_kernel:
                    if gpu_key == _EMBED_KEY:
                        state_packed[gpu_key] = frozen  # a lookup table, not a GEMV operand
                    else:
                        packed, scales = pack(frozen)
                        state_packed[gpu_key] = packed
                        state_packed[gpu_key[: -len(".weight")] + ".weight_scale"] = scales

    os.makedirs(out_dir, exist_ok=False)
    if pack_fp16:
        torch.save(state_fp16, os.path.join(out_dir, "model_state_fp16.pt"))
    if pack_kernel:
        name = "model_state_t2g128.pt" if quant == "ternary" else "model_state_q1g128.pt"
        torch.save(state_packed, os.path.join(out_dir, name))
    cfg = {
        "dim": hf_config["hidden_size"],
        "n_layers": hf_config["num_hidden_layers"],
        "n_heads": hf_config["num_attention_heads"],
        "n_kv_heads": hf_config["num_key_value_heads"],
        "head_dim": hf_config["head_dim"],
        "ffn_dim": hf_config["intermediate_size"],
        "vocab_size": hf_config["vocab_size"],
        "norm_eps": hf_config["rms_norm_eps"],
        "rope_theta": hf_config["rope_theta"],
        "rope_original_max": hf_config["rope_scaling"]["original_max_position_embeddings"],
        "rope_factor": hf_config["rope_scaling"]["factor"],
        "tie_word_embeddings": bool(hf_config["tie_word_embeddings"]),
        "block_size": int(hf_config.get("block_size", 8)),
        "causal_attn": bool(hf_config.get("causal_attn", True)),
        "mask_token_id": int(hf_config.get("text_mask_token_id", 151654)),
        "kernel_kind": "t2g128" if quant == "ternary" else "q1",
        "quantize_embedding": bool(quantize_embedding),
    }
    with open(os.path.join(out_dir, "bonsai_gpu_config.json"), "w") as f:
        json.dump(cfg, f, indent=2)


# ---------------------------------------------------------------------------
# load
# ---------------------------------------------------------------------------
def load_args_from_ckpt(ckpt_dir: str, use_kernel: bool = True):
    """``bonsai_gpu_config.json`` -> ModelArgs (``load_args_from_ckpt``, generate.py:30-46)."""
    from .model import ModelArgs
    with open(os.path.join(ckpt_dir, "bonsai_gpu_config.json"), "r") as f:
        cfg = json.load(f)
    return ModelArgs(
        dim=cfg["dim"], n_layers=cfg["n_layers"], n_heads=cfg["n_heads"],
        n_kv_heads=cfg["n_kv_heads"], head_dim=cfg["head_dim"], ffn_dim=cfg["ffn_dim"],
        vocab_size=cfg["vocab_size"], norm_eps=cfg["norm_eps"], rope_theta=cfg["rope_theta"],
        rope_original_max=cfg["rope_original_max"], rope_factor=cfg["rope_factor"],
        tie_word_embeddings=cfg["tie_word_embeddings"], block_size=cfg["block_size"],
        causal_attn=cfg["causal_attn"], mask_token_id=cfg["mask_token_id"],
        use_kernel=use_kernel, kernel_kind=cfg.get("kernel_kind", "q1"))


def expected_packed_keys(args) -> Dict[str, Tuple[torch.dtype, Tuple[int, ...]]]:
    """Every key of ``model_state_t2g128.pt`` with its dtype and shape."""
    per = 4 if args.kernel_kind == "t2g128" else 8
    bf, i8 = torch.bfloat16, torch.int8
    out: Dict[str, Tuple[torch.dtype, Tuple[int, ...]]] = {
        "embed_tokens.weight": (bf, (args.vocab_size, args.dim)),
        "norm.weight": (bf, (args.dim,)),
    }
    lin = {
        "attention.q_proj": (args.q_dim, args.dim), "attention.k_proj": (args.kv_dim, args.dim),
        "attention.v_proj": (args.kv_dim, args.dim), "attention.o_proj": (args.dim, args.q_dim),
        "feed_forward.gate_proj": (args.ffn_dim, args.dim),
        "feed_forward.up_proj": (args.ffn_dim, args.dim),
        "feed_forward.down_proj": (args.dim, args.ffn_dim),
    }
    for i in range(args.n_layers):
        p = f"layers.{i}."
        out[p + "input_layernorm.weight"] = (bf, (args.dim,))
        out[p + "post_attention_layernorm.weight"] = (bf, (args.dim,))
        out[p + "attention.q_norm.weight"] = (bf, (args.head_dim,))
        out[p + "attention.k_norm.weight"] = (bf, (args.head_dim,))
        for name, (n, k) in lin.items():
            out[p + name + ".weight"] = (i8, (n, k // per))
            out[p + name + ".weight_scale"] = (bf, (n, k // GROUP_SIZE))
    return out


def load_packed_state(ckpt_dir: str) -> Tuple[object, Dict[str, torch.Tensor]]:
    """Read and validate ``model_state_t2g128.pt`` (``model_state_q1g128.pt`` for a sign-weight
    checkpoint; CPU tensors).  Missing or unexpected keys
    and wrong dtypes / shapes raise, like ``build_model`` (generate.py:49-68)."""
    args = load_args_from_ckpt(ckpt_dir, use_kernel=True)
    if args.kernel_kind not in ("t2g128", "q1"):
        raise ValueError(f"unknown kernel_kind {args.kernel_kind!r} in bonsai_gpu_config.json")
    if args.kernel_kind == "t2g128" and not args.tie_word_embeddings:
        raise ValueError("the packed T2 head is the tied embedding; untied checkpoints are not supported")
    path = os.path.join(ckpt_dir, "model_state_t2g128.pt" if args.kernel_kind == "t2g128"
                        else "model_state_q1g128.pt")
    sd = torch.load(path, map_location="cpu", weights_only=True)
    want = expected_packed_keys(args)
    missing = [k for k in want if k not in sd]
    if missing:
        raise RuntimeError(f"Missing weights: {missing[:5]}")
    unexpected = [k for k in sd if k not in want and "lm_head" not in k]
    if unexpected:
        raise RuntimeError(f"Unexpected weights: {unexpected[:5]}")
    for k, (dtype, shape) in want.items():
        if sd[k].dtype != dtype or tuple(sd[k].shape) != shape:
            raise RuntimeError(f"{k}: expected {dtype} {shape}, got {sd[k].dtype} {tuple(sd[k].shape)}")
    return args, sd


def load_decoder(ckpt_dir: str, device="cuda", head_kind: Optional[str] = None):
    """Packed checkpoint -> ``BonsaiDecoder`` with q|k|v and gate|up merged along the output
    rows (``prepare_merged_weights``, model.py:931-956,1042-1051).  A ternary checkpoint gets
    the tied head packed on its ternary grid, padded to whole 128-row tiles
    (``prepare_t2_lm_head``, model.py:1222-1243); a sign-weight ("q1") checkpoint keeps the
    output projection in bf16 (the tied embedding, or ``lm_head.weight`` when untied), as the
    reference's graphs do (fast_runtime.py:175-178); ``head_kind="q1"`` packs it to sign bits
    instead (``prepare_q1_lm_head``, model.py:1196-1220)."""
    from .model import BonsaiDecoder, LayerWeights, PackedLinear, head_rows_for, kind_bits
    args, sd = load_packed_state(ckpt_dir)
    dev = torch.device(device)
    bits = kind_bits(args.kernel_kind)

    def lin(prefix: str) -> Tuple[torch.Tensor, torch.Tensor]:
        return sd[prefix + ".weight"], sd[prefix + ".weight_scale"]

    def to_dev(pair) -> PackedLinear:
        return PackedLinear(pair[0].contiguous().to(dev), pair[1].contiguous().to(dev), bits)

    layers = []
    for i in range(args.n_layers):
        a, f = f"layers.{i}.attention.", f"layers.{i}.feed_forward."
        layers.append(LayerWeights(
            wqkv=to_dev(merge_packed_rows([lin(a + "q_proj"), lin(a + "k_proj"), lin(a + "v_proj")])),
            wo=to_dev(lin(a + "o_proj")),
            w_gu=to_dev(merge_packed_rows([lin(f + "gate_proj"), lin(f + "up_proj")])),
            w_down=to_dev(lin(f + "down_proj")),
            input_layernorm=sd[f"layers.{i}.input_layernorm.weight"].to(dev),
            post_attention_layernorm=sd[f"layers.{i}.post_attention_layernorm.weight"].to(dev),
            q_norm=sd[a + "q_norm.weight"].to(dev), k_norm=sd[a + "k_norm.weight"].to(dev)))
    embed = sd["embed_tokens.weight"].to(dev).contiguous()
    if head_kind not in (None, "t2", "q1", "bf16") or (bits == 2 and head_kind not in (None, "t2")):
        raise ValueError(f"head_kind {head_kind!r} does not fit a {args.kernel_kind!r} checkpoint")
    if bits == 1 and head_kind == "q1":
        src = embed if args.tie_word_embeddings else sd["lm_head.weight"].to(dev)
        rows = head_rows_for(args.vocab_size)
        padded = torch.zeros(rows, args.dim, dtype=torch.bfloat16, device=dev)
        padded[: args.vocab_size].copy_(src)
        head_w, head_s = pack_q1_g128(padded)
        return BonsaiDecoder(args, layers, embed, sd["norm.weight"].to(dev),
                             PackedLinear(head_w, head_s, 1))
    if bits == 1:
        if head_kind == "t2":
            raise ValueError("a 'q1' checkpoint takes head_kind 'bf16' or 'q1'")
        head_bf16 = None
        if not args.tie_word_embeddings:
            if "lm_head.weight" not in sd:
                raise RuntimeError("Missing weights: ['lm_head.weight']")
            head_bf16 = sd["lm_head.weight"].to(dev).contiguous()
        return BonsaiDecoder(args, layers, embed, sd["norm.weight"].to(dev), None, head_bf16)
    rows = head_rows_for(args.vocab_size)
    padded = torch.zeros(rows, args.dim, dtype=torch.bfloat16, device=dev)
    padded[: args.vocab_size].copy_(embed)
    head_w, head_s = pack_t2_g128(padded)
    return BonsaiDecoder(args, layers, embed, sd["norm.weight"].to(dev), PackedLinear(head_w, head_s))


def main(argv=None) -> None:
    import argparse
    ap = argparse.ArgumentParser(description="Convert a Bonsai HF safetensors checkpoint to the "
                                             "packed T2-g128 inference files.")
    ap.add_argument("--src", required=True, help="HF safetensors directory")
    ap.add_argument("--out", required=True, help="output directory (must not exist)")
    ap.add_argument("--no-kernel", action="store_true", help="skip the packed dump")
    ap.add_argument("--no-fp16", action="store_true", help="skip the frozen bf16 dump")
    ap.add_argument("--quant", choices=("ternary", "q1"), default="ternary")
    a = ap.parse_args(argv)
    try:
        convert(a.src, a.out, pack_kernel=not a.no_kernel, pack_fp16=not a.no_fp16, quant=a.quant)
    except ValueError as error:
        ap.error(str(error))


if __name__ == "__main__":
    main()
