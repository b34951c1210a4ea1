"""Pins the CPU oracle (oracle/bonsai_oracle.c and the NumPy restatement) without
any GPU: hand-derived known answers, brute force over every byte value, closed
forms, invariants and library routines -- chosen so that a dropped term, a wrong
sign, bit order or index fails at least one of them.  None of these tests retypes
the oracle's own formula."""
import numpy as np
import pytest
import torch


# ---- weight decode ---------------------------------------------------------
def test_t2_decode_known_bytes(oracle):
    # 0x1B = 0b00_01_10_11 -> fields LSB first 3,2,1,0 -> +1, 0, -1, -2
    B = np.array([[0x1B, 0xFF, 0xAA, 0x55]], dtype=np.uint8)
    expect = [1, 0, -1, -2, 1, 1, 1, 1, 0, 0, 0, 0, -1, -1, -1, -1]
    assert oracle.c_unpack(B, 2)[0].tolist() == expect
    assert oracle.np_unpack(B, 2)[0].tolist() == expect


def test_q1_decode_known_byte(oracle):
    # 0xA5 = 0b10100101 -> bits LSB first 1,0,1,0,0,1,0,1
    B = np.array([[0xA5]], dtype=np.uint8)
    expect = [1, -1, 1, -1, -1, 1, -1, 1]
    assert oracle.c_unpack(B, 1)[0].tolist() == expect
    assert oracle.np_unpack(B, 1)[0].tolist() == expect


@pytest.mark.parametrize("bits", [2, 1])
def test_decode_all_byte_values_against_bit_strings(oracle, bits):
    """Brute force: every byte value, decoded independently from its binary text."""
    per = 8 // bits
    B = np.arange(256, dtype=np.uint8).reshape(1, 256)
    # pad each byte to its own K-slot: row of 256 bytes -> 256*per weights
    got = oracle.c_unpack(B, bits)[0].reshape(256, per)
    for byte in range(256):
        text = format(byte, "08b")[::-1]  # LSB first
        fields = [int(text[i * bits:(i + 1) * bits][::-1], 2) for i in range(per)]
        want = [f - 2 for f in fields] if bits == 2 else [2 * f - 1 for f in fields]
        assert got[byte].tolist() == want, byte


# ---- packers ---------------------------------------------------------------
@pytest.mark.parametrize("bits", [2, 1])
def test_pack_values_round_trip(oracle, bits):
    rng = np.random.default_rng(3)
    if bits == 2:
        q = rng.integers(-1, 2, size=(7, 384), dtype=np.int8)
    else:
        q = (2 * rng.integers(0, 2, size=(7, 384), dtype=np.int8) - 1).astype(np.int8)
    B = oracle.c_pack_values(q, bits)
    assert B.shape == (7, 384 * bits // 8)
    assert np.array_equal(oracle.c_unpack(B, bits), q)
    if bits == 2:  # the packer never emits code 0
        fields = [(B >> s) & 3 for s in (0, 2, 4, 6)]
        assert all(f.min() >= 1 for f in fields)


def test_converter_fixture_all_ones(oracle):
    """The reference converter's own synthetic fixture (tests/test_bonsai_converter.py:37-48,
    169-196): all-ones 128x128 weights -> T2 bytes 0xFF with shape (128, 32), Q1 bytes
    0xFF with shape (128, 16), every scale bf16 1.0 with shape (128, 1)."""
    ones_bf16 = np.full((128, 128), 0x3F80, dtype=np.uint16)
    for bits, cols in ((2, 32), (1, 16)):
        B, S = oracle.c_pack_latent(ones_bf16, bits)
        assert B.shape == (128, cols) and S.shape == (128, 1)
        assert np.all(B == 0xFF) and np.all(S == 0x3F80)


def test_pack_latent_t2_grid_and_rounding(oracle):
    """Latent weights d*{-1,0,+1} come back exactly; 0.5*d rounds half-to-even to 0 and
    0.51*d to 1; the scale is the group's absmax as bf16."""
    d = np.float32(0.0625)
    w = np.zeros((1, 128), dtype=np.float32)
    w[0, :6] = [d, -d, 0.0, 0.5 * d, 0.51 * d, -0.75 * d]
    wb = oracle.f32_to_bf16_bits(w)
    B, S = oracle.c_pack_latent(wb, 2)
    assert oracle.bf16_bits_to_f32(S)[0, 0] == d
    back = oracle.c_unpack(B, 2)[0, :6].tolist()
    assert back == [1, -1, 0, 0, 1, -1]


def test_pack_latent_q1_sign_and_mean(oracle):
    d = np.float32(0.25)
    w = np.full((1, 128), d, dtype=np.float32)
    w[0, ::3] = -d
    w[0, 5] = 0.0  # zero counts as positive; mean magnitude drops by d/128
    B, S = oracle.c_pack_latent(oracle.f32_to_bf16_bits(w), 1)
    back = oracle.c_unpack(B, 1)[0]
    want = np.where(w[0] >= 0, 1, -1)
    assert np.array_equal(back, want)
    mean = np.float32(127 * 0.25 / 128)
    assert S[0, 0] == oracle.f32_to_bf16_bits(np.array([mean]))[0]


@pytest.mark.parametrize("bits", [2, 1])
def test_product_packers_match_oracle(oracle, bits):
    """The package's torch packers produce the oracle's bytes and scales."""
    import bitmtp_amd
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(16, 512, generator=g) * 0.02).to(torch.bfloat16)
    if bits == 2:  # put the weights on the ternary grid first, as the converter does
        grp = w.float().view(16, 4, 128)
        s = grp.abs().amax(-1, keepdim=True).clamp_min(1e-8)
        w = (torch.round(grp / s).clamp(-1, 1) * s).view(16, 512).to(torch.bfloat16)
        packed, scale = bitmtp_amd.pack_t2_g128(w)
    else:
        grp = w.float().view(16, 4, 128)
        dgrp = grp.abs().mean(-1, keepdim=True)
        w = (torch.where(grp >= 0, 1.0, -1.0) * dgrp).view(16, 512).to(torch.bfloat16)
        packed, scale = bitmtp_amd.pack_q1_g128(w)
    B, S = oracle.c_pack_latent(w.view(torch.int16).numpy().view(np.uint16), bits)
    assert np.array_equal(packed.numpy().view(np.uint8), B)
    assert np.array_equal(scale.view(torch.int16).numpy().view(np.uint16), S)
    unpack = bitmtp_amd.unpack_t2_g128 if bits == 2 else bitmtp_amd.unpack_q1_g128
    assert np.array_equal(unpack(packed).numpy(), oracle.c_unpack(B, bits))


# ---- activation quantisation -------------------------------------------------
def test_act_quant_known_answers(oracle):
    q, s = oracle.c_act_quant(np.ones((1, 128), dtype=np.float32))
    assert s[0] == 127.0 and np.all(q == 127)
    q, s = oracle.c_act_quant(np.zeros((1, 128), dtype=np.float32))
    assert s[0] == (np.float32(1.0) / np.float32(1e-5)) * np.float32(127.0) and np.all(q == 0)
    # x*s exactly on .5 -> round half to even (all values exact in fp16)
    x = np.zeros((1, 128), dtype=np.float32)
    x[0, :5] = [127 / 64, 1 / 128, 3 / 128, 5 / 128, -3 / 128]
    q, s = oracle.c_act_quant(x)
    assert s[0] == 64.0 and q[0, :6].tolist() == [127, 0, 2, 2, -2, 0]


def test_act_quant_properties_and_torch_cross_check(oracle):
    g = torch.Generator().manual_seed(9)
    x16 = (torch.randn(6, 2048, generator=g) * 2.5).to(torch.float16)
    x16[3] = -x16[3].abs()  # the extreme element is negative in this row
    q, s = oracle.c_act_quant(x16.float().numpy())
    qn, sn = oracle.np_act_quant(x16.float().numpy())
    assert np.array_equal(q, qn) and np.array_equal(s, sn)
    # library routine: torch's own amax / division / round / clamp on the same values
    xf = x16.float()
    st = 127.0 / xf.abs().amax(dim=-1, keepdim=True).clamp_min(1e-5)
    qt = (xf * st).round().clamp(-128, 127).to(torch.int8)
    assert np.array_equal(q, qt.numpy()) and np.array_equal(s, st.numpy().reshape(-1))
    # the absmax element maps to +-127 and nothing exceeds it
    idx = np.abs(x16.float().numpy()).argmax(axis=1)
    assert np.all(np.abs(q[np.arange(6), idx].astype(int)) == 127)
    assert np.abs(q.astype(int)).max() == 127


# ---- group sums ----------------------------------------------------------------
@pytest.mark.parametrize("bits", [2, 1])
def test_group_sums_against_integer_matmul(oracle, bits):
    """Library routine: per group, an int64 matrix product of the decoded weights."""
    rng = np.random.default_rng(11)
    M, N, K = 5, 23, 640
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(0, 256, size=(N, K * bits // 8), dtype=np.uint8)
    W = oracle.c_unpack(B, bits).astype(np.int64)
    G = oracle.c_group_sums(A, B, bits)
    for g in range(K // 128):
        sl = slice(128 * g, 128 * (g + 1))
        assert np.array_equal(G[:, :, g], A[:, sl].astype(np.int64) @ W[:, sl].T)
    assert np.array_equal(G, oracle.np_group_sums(A, B, bits))
    assert np.abs(G).max() <= 128 * 128 * (2 if bits == 2 else 1)


def test_group_sums_brute_force_tiny(oracle):
    rng = np.random.default_rng(12)
    A = rng.integers(-128, 128, size=(2, 256), dtype=np.int8)
    B = rng.integers(0, 256, size=(3, 64), dtype=np.uint8)
    G = oracle.c_group_sums(A, B, 2)
    for m in range(2):
        for n in range(3):
            for g in range(2):
                acc = 0
                for k in range(128 * g, 128 * g + 128):
                    code = (int(B[n, k // 4]) >> (2 * (k % 4))) & 3
                    acc += int(A[m, k]) * (code - 2)
                assert G[m, n, g] == acc


# ---- fp32 epilogue ---------------------------------------------------------------
def test_gemv_hand_derived(oracle):
    one = 0x3F80
    A = np.full((1, 128), 127, dtype=np.int8)
    s = np.array([127.0], dtype=np.float32)
    B = np.full((1, 32), 0xFF, dtype=np.uint8)          # all +1
    y32, y16 = oracle.c_gemv(A, B, s, np.array([[0x3F00]], dtype=np.uint16), 2)  # ws = 0.5
    assert y32[0, 0] == 64.0 and y16[0, 0] == 0x4280      # 127*128*0.5/127
    B_alt = np.full((1, 32), 0x77, dtype=np.uint8)       # +1,-1,+1,-1
    assert oracle.c_gemv(A, B_alt, s, np.array([[0x3F00]], dtype=np.uint16), 2)[0][0, 0] == 0.0
    A2 = np.full((1, 256), 127, dtype=np.int8)
    B2 = np.full((1, 64), 0xFF, dtype=np.uint8)
    ws2 = np.array([[one, 0x3E80]], dtype=np.uint16)     # 1.0, 0.25
    assert oracle.c_gemv(A2, B2, s, ws2, 2)[0][0, 0] == 160.0   # (16256 + 4064)/127
    Bq = np.full((1, 16), 0x00, dtype=np.uint8)          # Q1 all -1
    assert oracle.c_gemv(A, Bq, s, np.array([[0x3F00]], dtype=np.uint16), 1)[0][0, 0] == -64.0


@pytest.mark.parametrize("bits", [2, 1])
def test_gemv_unit_scales_is_integer_gemm(oracle, bits):
    """ws = 1, s = 1: the op is a textbook integer GEMM (exact in fp32 at this size)."""
    rng = np.random.default_rng(13)
    M, N, K = 3, 17, 512
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(0, 256, size=(N, K * bits // 8), dtype=np.uint8)
    ws = np.full((N, K // 128), 0x3F80, dtype=np.uint16)
    y32, _ = oracle.c_gemv(A, B, np.ones(M, dtype=np.float32), ws, bits)
    W = oracle.c_unpack(B, bits).astype(np.int64)
    assert np.array_equal(y32.astype(np.int64), A.astype(np.int64) @ W.T)


@pytest.mark.parametrize("bits", [2, 1])
def test_gemv_against_float64_and_linearity(oracle, bits):
    p = oracle.synth_problem(21, 4, 64, 2048, bits)
    y32, y16 = oracle.c_gemv(p["A"], p["B"], p["s"], p["ws"], bits)
    W = oracle.c_unpack(p["B"], bits).astype(np.float64)
    wsf = np.repeat(oracle.bf16_bits_to_f32(p["ws"]).astype(np.float64), 128, axis=1)
    ref = (p["A"].astype(np.float64) @ (W * wsf).T) / p["s"].astype(np.float64)[:, None]
    assert np.all(np.abs(y32 - ref) <= 1e-5 * np.abs(ref) + 1e-6)
    assert np.array_equal(y32, oracle.np_gemv_f32(p["A"], p["B"], p["s"], p["ws"], bits))
    assert np.array_equal(y16, oracle.f32_to_bf16_bits(y32))
    # doubling every scale (exact in bf16) doubles the result exactly
    ws2 = oracle.f32_to_bf16_bits(oracle.bf16_bits_to_f32(p["ws"]) * 2)
    assert np.array_equal(oracle.c_gemv(p["A"], p["B"], p["s"], ws2, bits)[0], 2 * y32)
    # a single non-zero group isolates that group's sum and scale
    ws1 = np.zeros_like(p["ws"])
    ws1[:, 3] = p["ws"][:, 3]
    G = oracle.c_group_sums(p["A"], p["B"], bits)
    want = (G[:, :, 3].astype(np.float32) * oracle.bf16_bits_to_f32(p["ws"])[None, :, 3]) / p["s"][:, None]
    assert np.array_equal(oracle.c_gemv(p["A"], p["B"], p["s"], ws1, bits)[0], want.astype(np.float32))


def test_gemv_matches_dequantised_linear(oracle):
    """The only CPU-runnable statement of the op in the reference is dequantise-then-
    F.linear (src/bonsai_sft/gpu/model.py:646-656); the oracle agrees with that
    composition in this build's own PyTorch within bf16 resolution."""
    p = oracle.synth_problem(22, 3, 96, 1024, 2)
    _, y16 = oracle.c_gemv(p["A"], p["B"], p["s"], p["ws"], 2)
    y = torch.from_numpy(y16.view(np.int16)).view(torch.bfloat16).float()
    w = torch.from_numpy(oracle.c_unpack(p["B"], 2)).to(torch.bfloat16)
    scales = torch.from_numpy(p["ws"].view(np.int16)).view(torch.bfloat16).repeat_interleave(128, dim=1)
    x = torch.from_numpy(p["x"]).float()
    st = 127.0 / x.abs().amax(-1, keepdim=True).clamp_min(1e-5)
    xq = ((x * st).round().clamp(-128, 127) / st).to(torch.bfloat16)
    ref = torch.nn.functional.linear(xq, w * scales).float()
    assert torch.all((y - ref).abs() <= 2e-2 * ref.abs() + 2e-3)


def test_bf16_rounding_helpers(oracle):
    L = oracle.lib()
    assert L.oracle_f32_to_bf16(1.0) == 0x3F80
    # 1 + 2^-8 is a tie between 0x3F80 and 0x3F81 -> even; 1 + 3*2^-8 ties to 0x3F82
    assert L.oracle_f32_to_bf16(1.00390625) == 0x3F80
    assert L.oracle_f32_to_bf16(1.01171875) == 0x3F82
    assert L.oracle_f32_to_bf16(-2.5) == 0xC020
    x = np.random.default_rng(1).standard_normal(4096).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_bits(x), want)
    assert all(L.oracle_f32_to_bf16(float(v)) == w for v, w in zip(x[:256], want[:256]))
    h = np.array([0x3C00, 0x0001, 0xC000, 0x7BFF, 0x0400], dtype=np.uint16)
    assert [L.oracle_f16_to_f32(int(v)) for v in h] == h.view(np.float16).astype(np.float32).tolist()
