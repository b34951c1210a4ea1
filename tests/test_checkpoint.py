"""Packed checkpoint format: converter guards, file contents and loading.

The cases and expected messages are the ones the reference's own converter tests hold
(tests/test_bonsai_converter.py, tests/test_export_input_guards.py:104-126): tiny synthetic
shapes, every rejection leaves no output behind.  The converted bytes are pinned by known
answers: an all-ones 128x128 matrix packs to T2 bytes 0xFF with scale 1.0 (Q1: 0xFF, 1.0),
and unpack(pack(freeze(w))) * scale == freeze(w) for random latent weights.
"""
import copy
import json

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from bitmtp_amd import checkpoint as C
from bitmtp_amd.packing import unpack_q1_g128, unpack_t2_g128

BASE_CONFIG = {
    "hidden_size": 128, "num_hidden_layers": 1, "num_attention_heads": 1,
    "num_key_value_heads": 1, "head_dim": 128, "intermediate_size": 128,
    "vocab_size": 16, "rms_norm_eps": 1e-6, "rope_theta": 1e6,
    "rope_scaling": {"original_max_position_embeddings": 32, "factor": 4.0},
    "tie_word_embeddings": True, "block_size": 4, "causal_attn": True,
    "text_mask_token_id": 15,
}


def ones_weights(config=BASE_CONFIG, fill=None):
    """Stand-in tensors of the right shapes (ones, or `fill(shape)`)."""
    make = fill or (lambda shape: torch.ones(*shape))
    return {k: make(shape) for k, shape in C.expected_tensor_shapes(config).items()}


@pytest.fixture
def dirs(tmp_path):
    src = tmp_path / "hf"
    src.mkdir()
    (src / "config.json").write_text(json.dumps(BASE_CONFIG))
    return src, tmp_path / "converted"


def rejected(src, out, pattern, **options):
    with pytest.raises(ValueError, match=pattern):
        C.convert(str(src), str(out), **options)
    assert not out.exists(), "invalid source created conversion artifacts"


# ---------------------------------------------------------------- guards
def test_missing_config(dirs):
    src, out = dirs
    (src / "config.json").unlink()
    rejected(src, out, "missing HF config.json")


def test_bin_only_checkpoint(dirs):
    src, out = dirs
    (src / "pytorch_model.bin").write_bytes(b"not model weights")
    rejected(src, out, "safe_serialization=True")


def test_invalid_and_empty_containers(dirs):
    src, out = dirs
    (src / "model.safetensors").write_bytes(b"not safetensors")
    rejected(src, out, "invalid HF safetensors shard")
    save_file({}, str(src / "model.safetensors"))
    rejected(src, out, "empty safetensors shard")


def test_missing_tensor_and_missing_layer(dirs):
    src, out = dirs
    w = ones_weights()
    del w["model.layers.0.self_attn.k_proj.weight"]
    save_file(w, str(src / "model.safetensors"))
    rejected(src, out, "incomplete HF checkpoint.*missing 1 core")
    save_file(ones_weights(), str(src / "model.safetensors"))
    (src / "config.json").write_text(json.dumps(dict(BASE_CONFIG, num_hidden_layers=2)))
    rejected(src, out, "incomplete HF checkpoint.*missing 11 core")


def test_wrong_shape_integer_input_duplicates_and_unknown_keys(dirs):
    src, out = dirs
    w = ones_weights()
    w["model.layers.0.self_attn.q_proj.weight"] = torch.ones(127, 128)
    save_file(w, str(src / "model.safetensors"))
    rejected(src, out, "tensor shape mismatch")
    w = ones_weights()
    w["model.embed_tokens.weight"] = torch.ones(16, 128, dtype=torch.int8)
    save_file(w, str(src / "model.safetensors"))
    rejected(src, out, "floating-point HF weights")
    w = ones_weights()
    w["unrecognized.weight"] = torch.ones(1)
    save_file(w, str(src / "model.safetensors"))
    rejected(src, out, "unsupported tensor key")
    (src / "model.safetensors").unlink()
    save_file(ones_weights(), str(src / "model-1.safetensors"))
    save_file({"model.norm.weight": torch.ones(128)}, str(src / "model-2.safetensors"))
    rejected(src, out, "duplicate tensor key across shards")


def test_untied_model_requires_lm_head(dirs):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    (src / "config.json").write_text(json.dumps(dict(BASE_CONFIG, tie_word_embeddings=False)))
    rejected(src, out, "incomplete HF checkpoint.*lm_head")


@pytest.mark.parametrize("key,bad", [("rope_scaling", None), ("hidden_size", 127),
                                     ("tie_word_embeddings", "true"), ("text_mask_token_id", 100),
                                     ("num_attention_heads", 0), ("rms_norm_eps", float("nan"))])
def test_bad_config_rejected_before_output(dirs, key, bad):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    cfg = copy.deepcopy(BASE_CONFIG)
    cfg[key] = bad
    (src / "config.json").write_text(json.dumps(cfg))
    rejected(src, out, "config.json")


def test_existing_output_is_never_touched(dirs):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    out.mkdir()
    with pytest.raises(ValueError, match="output already exists"):
        C.convert(str(src), str(out), quant="ternary")
    assert list(out.iterdir()) == []
    sentinel = out / "model_state_t2g128.pt"
    sentinel.write_bytes(b"previous checkpoint")
    with pytest.raises(ValueError, match="output already exists"):
        C.convert(str(src), str(out), quant="ternary")
    assert sentinel.read_bytes() == b"previous checkpoint"
    sentinel.unlink()
    out.rmdir()
    out.symlink_to(out.parent / "missing")          # dangling symlink
    with pytest.raises(ValueError, match="output already exists"):
        C.convert(str(src), str(out), quant="ternary")
    assert out.is_symlink()


def test_invalid_options(dirs):
    src, out = dirs
    rejected(src, out, "at least one output", pack_kernel=False, pack_fp16=False)
    rejected(src, out, "Q1-only", quant="ternary", quantize_embedding=False)
    rejected(src, out, "quant must be", quant="not-a-grid")


@pytest.mark.parametrize("saved", [[], {"block_size": True, "causal_attn": True, "text_mask_token_id": 15},
                                   {"block_size": 4},
                                   {"block_size": 8, "causal_attn": True, "text_mask_token_id": 15}])
def test_invalid_or_conflicting_sidecar(dirs, saved):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    (src / "sdlm_config.json").write_text(json.dumps(saved))
    with pytest.raises(ValueError):
        C.convert(str(src), str(out), quant="ternary")
    assert not out.exists()


def test_matching_sidecar_changes_nothing(dirs, tmp_path):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    plain = tmp_path / "plain"
    C.convert(str(src), str(plain), quant="ternary")
    (src / "sdlm_config.json").write_text(json.dumps(
        {"block_size": 4, "causal_attn": True, "text_mask_token_id": 15}))
    C.convert(str(src), str(out), quant="ternary")
    for name in ("model_state_t2g128.pt", "model_state_fp16.pt"):
        a = torch.load(plain / name, weights_only=True)
        b = torch.load(out / name, weights_only=True)
        assert set(a) == set(b) and all(torch.equal(a[k], b[k]) for k in a)
    assert (plain / "bonsai_gpu_config.json").read_bytes() == (out / "bonsai_gpu_config.json").read_bytes()


def test_4b_metadata_uses_query_width():
    cfg = dict(BASE_CONFIG, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
               intermediate_size=9728)
    shapes = C.expected_tensor_shapes(cfg)
    assert shapes["model.layers.0.self_attn.q_proj.weight"] == (4096, 2560)
    assert shapes["model.layers.0.self_attn.k_proj.weight"] == (1024, 2560)
    assert shapes["model.layers.0.self_attn.o_proj.weight"] == (2560, 4096)
    assert shapes["model.layers.0.mlp.down_proj.weight"] == (2560, 9728)


def test_key_mapping():
    m = C.hf_to_gpu_key
    assert m("model.embed_tokens.weight") == "embed_tokens.weight"
    assert m("model.norm.weight") == "norm.weight"
    assert m("model.layers.3.self_attn.q_norm.weight") == "layers.3.attention.q_norm.weight"
    assert m("model.layers.12.mlp.down_proj.weight") == "layers.12.feed_forward.down_proj.weight"
    assert m("model.layers.0.input_layernorm.weight") == "layers.0.input_layernorm.weight"
    assert m("lm_head.weight") == "lm_head.weight"


# ---------------------------------------------------------------- contents
def test_ternary_conversion_known_answers(dirs):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    C.convert(str(src), str(out), quant="ternary")
    packed = torch.load(out / "model_state_t2g128.pt", weights_only=True)
    key = "layers.0.attention.q_proj"
    assert packed[key + ".weight"].dtype == torch.int8
    assert tuple(packed[key + ".weight"].shape) == (128, 32)
    assert torch.all(packed[key + ".weight"] == -1)                  # byte 0xFF: four codes 3 (+1)
    assert packed[key + ".weight_scale"].dtype == torch.bfloat16
    assert tuple(packed[key + ".weight_scale"].shape) == (128, 1)
    assert torch.all(packed[key + ".weight_scale"] == 1.0)
    assert packed["norm.weight"].dtype == torch.bfloat16
    assert packed["embed_tokens.weight"].dtype == torch.bfloat16
    cfg = json.loads((out / "bonsai_gpu_config.json").read_text())
    assert cfg["kernel_kind"] == "t2g128" and cfg["block_size"] == 4
    assert cfg["mask_token_id"] == 15 and cfg["rope_original_max"] == 32 and cfg["rope_factor"] == 4.0
    assert set(packed) == set(C.expected_packed_keys(C.load_args_from_ckpt(str(out))))


def test_q1_conversion_known_answers(dirs):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    C.convert(str(src), str(out), quant="q1", quantize_embedding=False)
    packed = torch.load(out / "model_state_q1g128.pt", weights_only=True)
    frozen = torch.load(out / "model_state_fp16.pt", weights_only=True)
    key = "layers.0.attention.q_proj"
    assert packed[key + ".weight"].dtype == torch.int8
    assert tuple(packed[key + ".weight"].shape) == (128, 16)
    assert torch.all(packed[key + ".weight"] == -1) and torch.all(packed[key + ".weight_scale"] == 1.0)
    assert packed["embed_tokens.weight"].dtype == torch.bfloat16
    assert frozen[key + ".weight"].dtype == torch.bfloat16
    cfg = json.loads((out / "bonsai_gpu_config.json").read_text())
    assert cfg["kernel_kind"] == "q1" and cfg["quantize_embedding"] is False


def test_freeze_grids_known_answers():
    w = torch.zeros(1, 128, dtype=torch.bfloat16)
    w[0, :4] = torch.tensor([0.5, -0.26, 0.24, -0.5], dtype=torch.bfloat16)
    t = C.freeze_ternary_g128(w)
    assert t[0, :4].tolist() == [0.5, -0.5, 0.0, -0.5] and torch.all(t[0, 4:] == 0)
    q = C.freeze_q1_g128(w)
    d = float(w.float().abs().mean())
    assert torch.all(q[0].abs().float() == torch.tensor(d).to(torch.bfloat16).float())
    assert q[0, 1] < 0 and q[0, 3] < 0 and q[0, 5] > 0            # zero counts as +
    z = C.freeze_ternary_g128(torch.zeros(2, 128, dtype=torch.bfloat16))
    assert torch.all(z == 0)


def test_random_latent_round_trip(dirs):
    src, out = dirs
    gen = torch.Generator().manual_seed(4)
    cfg = dict(BASE_CONFIG, hidden_size=256, intermediate_size=384, num_attention_heads=2,
               vocab_size=40)
    (src / "config.json").write_text(json.dumps(cfg))
    w = ones_weights(cfg, fill=lambda shape: torch.randn(*shape, generator=gen) * 0.02)
    save_file(w, str(src / "model.safetensors"))
    C.convert(str(src), str(out), quant="ternary")
    packed = torch.load(out / "model_state_t2g128.pt", weights_only=True)
    frozen = torch.load(out / "model_state_fp16.pt", weights_only=True)
    for name in ("attention.q_proj", "attention.o_proj", "feed_forward.gate_proj",
                 "feed_forward.down_proj"):
        key = f"layers.0.{name}"
        f = frozen[key + ".weight"]
        q = unpack_t2_g128(packed[key + ".weight"])
        assert set(np.unique(q.numpy()).tolist()) <= {-1, 0, 1}        # code 0 never appears
        n, k = q.shape
        deq = (q.view(n, k // 128, 128).to(torch.bfloat16) * packed[key + ".weight_scale"].unsqueeze(-1))
        assert torch.equal(deq.view(n, k), f)
        # the frozen grid is the latent weight rounded per group
        lat = w["model.layers.0." + name.replace("attention", "self_attn")
                .replace("feed_forward", "mlp") + ".weight"].to(torch.bfloat16)
        assert torch.equal(f, C.freeze_ternary_g128(lat))
    assert torch.equal(packed["embed_tokens.weight"], frozen["embed_tokens.weight"])
    assert torch.equal(unpack_q1_g128(C.pack_q1_g128(C.freeze_q1_g128(lat))[0]).float(),
                       torch.where(lat < 0, -1.0, 1.0))


def test_loader_rejects_missing_unexpected_and_misshapen(dirs):
    src, out = dirs
    save_file(ones_weights(), str(src / "model.safetensors"))
    C.convert(str(src), str(out), quant="ternary")
    path = out / "model_state_t2g128.pt"
    good = torch.load(path, weights_only=True)
    args, sd = C.load_packed_state(str(out))
    assert args.kernel_kind == "t2g128" and args.block_size == 4 and set(sd) == set(good)
    bad = dict(good)
    del bad["layers.0.attention.k_proj.weight_scale"]
    torch.save(bad, path)
    with pytest.raises(RuntimeError, match="Missing weights"):
        C.load_packed_state(str(out))
    bad = dict(good, extra=torch.ones(1))
    torch.save(bad, path)
    with pytest.raises(RuntimeError, match="Unexpected weights"):
        C.load_packed_state(str(out))
    bad = dict(good)
    bad["layers.0.attention.q_proj.weight"] = good["layers.0.attention.q_proj.weight"].to(torch.int16)
    torch.save(bad, path)
    with pytest.raises(RuntimeError, match="expected torch.int8"):
        C.load_packed_state(str(out))


# ---------------------------------------------------------------- GPU: a converted checkpoint decodes
@pytest.mark.gpu
def test_converted_checkpoint_loads_and_decodes(tmp_path):
    from bitmtp_amd.generate import ar_generate, hybrid_generate
    from bitmtp_amd.model import dequantize_t2
    from bitmtp_amd.runtime import GraphAtlas
    src, out = tmp_path / "hf", tmp_path / "converted"
    src.mkdir()
    cfg = dict(BASE_CONFIG, hidden_size=512, intermediate_size=1024, num_attention_heads=4,
               num_key_value_heads=2, num_hidden_layers=2, vocab_size=1000, block_size=8,
               text_mask_token_id=999)
    (src / "config.json").write_text(json.dumps(cfg))
    gen = torch.Generator().manual_seed(8)

    def fill(shape):
        if len(shape) == 1:
            return 1.0 + 0.1 * torch.randn(*shape, generator=gen)
        return torch.randn(*shape, generator=gen) * 0.02
    save_file(ones_weights(cfg, fill=fill), str(src / "model.safetensors"))
    C.convert(str(src), str(out), quant="ternary")
    model = C.load_decoder(str(out), device="cuda:0")
    frozen = torch.load(out / "model_state_fp16.pt", weights_only=True)
    # merged rows are q | k | v and gate | up of the frozen grid; the head is the tied embedding
    lw = model.layers[1]
    want = torch.cat([frozen[f"layers.1.attention.{p}_proj.weight"] for p in "qkv"], dim=0)
    assert torch.equal(dequantize_t2(lw.wqkv).cpu(), want)
    want = torch.cat([frozen[f"layers.1.feed_forward.{p}_proj.weight"] for p in ("gate", "up")], dim=0)
    assert torch.equal(dequantize_t2(lw.w_gu).cpu(), want)
    assert model.head_rows == 1024
    assert torch.equal(dequantize_t2(model.head)[:1000].cpu(), frozen["embed_tokens.weight"])
    assert torch.all(dequantize_t2(model.head)[1000:] == 0)
    atlas = GraphAtlas(model, segment_ladder=(128,))
    prompt = list(range(7, 40))
    ar, _ = ar_generate(atlas, prompt, max_gen_len=20)
    hy, st = hybrid_generate(atlas, prompt, max_gen_len=20, exact_m1_verify=True)
    assert len(ar) == 20 and hy == ar


@pytest.mark.gpu
def test_converted_q1_checkpoint_loads_and_decodes(tmp_path):
    """A sign-weight checkpoint decodes with 1-bit layers and the bf16 tied output projection
    (fast_runtime.py:175-178); exact verification reproduces the AR tokens."""
    from bitmtp_amd.generate import ar_generate, hybrid_generate
    from bitmtp_amd.model import dequantize_packed
    from bitmtp_amd.runtime import GraphAtlas
    src, out = tmp_path / "hf", tmp_path / "converted"
    src.mkdir()
    cfg = dict(BASE_CONFIG, hidden_size=512, intermediate_size=1024, num_attention_heads=4,
               num_key_value_heads=2, num_hidden_layers=2, vocab_size=1000, block_size=8,
               text_mask_token_id=999)
    (src / "config.json").write_text(json.dumps(cfg))
    gen = torch.Generator().manual_seed(9)

    def fill(shape):
        if len(shape) == 1:
            return 1.0 + 0.1 * torch.randn(*shape, generator=gen)
        return torch.randn(*shape, generator=gen) * 0.02
    save_file(ones_weights(cfg, fill=fill), str(src / "model.safetensors"))
    C.convert(str(src), str(out), quant="q1")
    model = C.load_decoder(str(out), device="cuda:0")
    frozen = torch.load(out / "model_state_fp16.pt", weights_only=True)
    assert model.head_kind == "bf16" and model.head_rows == 1000
    lw = model.layers[0]
    assert lw.wqkv.bits == 1 and lw.wqkv.in_features == 512
    want = torch.cat([frozen[f"layers.0.attention.{p}_proj.weight"] for p in "qkv"], dim=0)
    assert torch.equal(dequantize_packed(lw.wqkv).cpu(), want)
    assert torch.equal(model.head_bf16.cpu(), frozen["embed_tokens.weight"])
    atlas = GraphAtlas(model, segment_ladder=(128,))
    prompt = list(range(5, 31))
    ar, _ = ar_generate(atlas, prompt, max_gen_len=16)
    hy, _ = hybrid_generate(atlas, prompt, max_gen_len=16, exact_m1_verify=True)
    assert len(ar) == 16 and hy == ar
    # the sign-packed head: scale = bf16(mean |w|) per group, bit = (w >= 0), 24 zero pad rows
    packed = C.load_decoder(str(out), device="cuda:0", head_kind="q1")
    assert packed.head_kind == "q1" and packed.head_rows == 1024
    w = frozen["embed_tokens.weight"].float().view(1000, 4, 128)
    assert torch.equal(packed.head.weight_scale[:1000].cpu(), w.abs().mean(-1).to(torch.bfloat16))
    assert torch.all(packed.head.weight_scale[1000:] == 0)
    with pytest.raises(ValueError):
        C.load_decoder(str(out), device="cuda:0", head_kind="t2")
