"""Golden fixtures (tests/golden): the oracle reproduces the hand-derived known
answers and the committed seeded vectors (CPU); the HIP path reproduces both (GPU)."""
import glob
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")
KNOWN = json.load(open(os.path.join(GOLD, "known_answers.json")))
NPZ = sorted(glob.glob(os.path.join(GOLD, "gemv_*.npz")))


def test_fixture_files_present():
    assert len(NPZ) == 4


def test_oracle_known_answers(oracle):
    for case in KNOWN["t2_decode"]:
        assert oracle.c_unpack(np.array([[case["byte"]]], dtype=np.uint8), 2)[0].tolist() == case["weights"]
    for case in KNOWN["q1_decode"]:
        assert oracle.c_unpack(np.array([[case["byte"]]], dtype=np.uint8), 1)[0].tolist() == case["weights"]
    for case in KNOWN["act_quant"]:
        x = np.full((1, case["K"]), case["x_fill"], dtype=np.float32)
        x[0, :len(case["x_head"])] = case["x_head"]
        q, s = oracle.c_act_quant(x)
        assert s[0] == case["s"] and q[0, :len(case["q_head"])].tolist() == case["q_head"]
    for case in KNOWN["gemv"]:
        K, bits = case["K"], case["bits"]
        A = np.full((1, K), 127, dtype=np.int8)
        B = np.full((1, K * bits // 8), case["weight_byte"], dtype=np.uint8)
        ws = oracle.f32_to_bf16_bits(np.array([case["ws"]], dtype=np.float32))
        s = np.array([127.0], dtype=np.float32)
        assert oracle.c_group_sums(A, B, bits)[0, 0].tolist() == case["G"]
        assert oracle.c_gemv(A, B, s, ws, bits)[0][0, 0] == case["y"]
    ones = np.full((128, 128), 0x3F80, dtype=np.uint16)
    for key, bits in (("t2", 2), ("q1", 1)):
        fx = KNOWN["converter_all_ones_128x128"][key]
        B, S = oracle.c_pack_latent(ones, bits)
        assert list(B.shape) == fx["shape"] and np.all(B == fx["byte"])
        assert list(S.shape) == fx["scale_shape"] and np.all(S == fx["scale_bf16_bits"])


@pytest.mark.parametrize("path", NPZ, ids=[os.path.basename(p) for p in NPZ])
def test_oracle_reproduces_golden_vectors(oracle, path):
    z = np.load(path)
    bits = int(z["bits"])
    q, s = oracle.c_act_quant(z["x"].astype(np.float32))
    assert np.array_equal(q, z["A"]) and np.array_equal(s, z["s"])
    assert np.array_equal(oracle.c_group_sums(z["A"], z["B"], bits), z["G"])
    y32, y16 = oracle.c_gemv(z["A"], z["B"], z["s"], z["ws"], bits)
    assert np.array_equal(y32, z["y32"]) and np.array_equal(y16, z["y16"])
    assert np.array_equal(oracle.np_group_sums(z["A"], z["B"], bits), z["G"])


@pytest.mark.gpu
@pytest.mark.parametrize("path", NPZ, ids=[os.path.basename(p) for p in NPZ])
def test_hip_path_reproduces_golden_vectors(path):
    import torch
    import bitmtp_amd as ops
    from gpu_util import bf16_bits, bf16_ordinal
    z = np.load(path)
    bits = int(z["bits"])
    dev = "cuda:0"
    print(f"[case] golden {os.path.basename(path)}", flush=True)
    q, s = ops.quant_input(torch.from_numpy(z["x"]).to(dev))
    assert np.array_equal(q.cpu().numpy(), z["A"]) and np.array_equal(s.cpu().numpy().reshape(-1), z["s"])
    B = torch.from_numpy(z["B"].view(np.int8)).to(dev)
    ws = torch.from_numpy(z["ws"].view(np.int16)).view(torch.bfloat16).to(dev)
    G = ops.packed_gemv_ex(q, B, None, None, bits=bits, out_kind=ops.OUT_G32)
    assert np.array_equal(G.cpu().numpy(), z["G"])
    y32 = ops.packed_gemv_ex(q, B, s, ws, bits=bits, out_kind=ops.OUT_F32).cpu().numpy()
    assert np.all(np.abs(y32 - z["y32"]) <= 1e-3 + 1e-3 * np.abs(z["y32"]))
    y16 = ops.packed_int8_linear(q, B, s, ws)
    assert np.abs(bf16_ordinal(bf16_bits(y16)) - bf16_ordinal(z["y16"])).max() <= 1


@pytest.mark.gpu
def test_hip_path_known_answers():
    import torch
    import bitmtp_amd as ops
    dev = "cuda:0"
    for case in KNOWN["act_quant"]:
        x = torch.full((1, case["K"]), case["x_fill"], dtype=torch.float16)
        x[0, :len(case["x_head"])] = torch.tensor(case["x_head"], dtype=torch.float16)
        q, s = ops.quant_input(x.to(dev))
        assert float(s.item()) == case["s"] and q[0, :len(case["q_head"])].tolist() == case["q_head"]
    for case in KNOWN["gemv"]:
        K, bits = case["K"], case["bits"]
        A = torch.full((1, K), 127, dtype=torch.int8, device=dev)
        byte = case["weight_byte"] - 256 if case["weight_byte"] > 127 else case["weight_byte"]
        B = torch.full((1, K * bits // 8), byte, dtype=torch.int8, device=dev)
        ws = torch.tensor([case["ws"]], dtype=torch.bfloat16, device=dev)
        s = torch.tensor([[127.0]], dtype=torch.float32, device=dev)
        G = ops.packed_gemv_ex(A, B, None, None, bits=bits, out_kind=ops.OUT_G32)
        assert G[0, 0].tolist() == case["G"]
        assert float(ops.packed_int8_linear(A, B, s, ws).item()) == case["y"]
