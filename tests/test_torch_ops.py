"""The registered PyTorch operators (torch.ops.bonsai.*): schema, shape inference on meta
tensors and argument checks without a GPU; on the GPU the same results as the ctypes operators,
eagerly and from a captured graph."""
import pytest
import torch

from bitmtp_amd import ops


@pytest.fixture(scope="module")
def bonsai():
    from bitmtp_amd import build
    build.build_torch_ops(verbose=False)  # compiles only when missing or out of date
    return ops.load_torch_ops()


def _meta_problem(m_shape, n, k, bits, scale_dtype=torch.bfloat16):
    a = torch.empty(*m_shape, k, dtype=torch.int8, device="meta")
    b = torch.empty(n, k * bits // 8, dtype=torch.int8, device="meta")
    s = torch.empty(*m_shape, 1, dtype=torch.float32, device="meta")
    ws = torch.empty(n, k // 128, dtype=scale_dtype, device="meta")
    return a, b, s, ws


def test_schemas(bonsai):
    assert str(bonsai.t2g128_int8xint2_linear.default._schema) == \
        "bonsai::t2g128_int8xint2_linear(Tensor a_int8, Tensor b_packed, Tensor s, Tensor ws) -> Tensor"
    assert str(bonsai.q1g128_int8xint1_linear.default._schema) == \
        "bonsai::q1g128_int8xint1_linear(Tensor a_int8, Tensor b_packed, Tensor s, Tensor ws) -> Tensor"
    assert str(bonsai.quant_input.default._schema) == "bonsai::quant_input(Tensor x) -> (Tensor, Tensor)"
    assert str(bonsai.fused_norm_quant.default._schema) == \
        "bonsai::fused_norm_quant(Tensor x, Tensor w, float eps) -> (Tensor, Tensor)"
    assert str(bonsai.fused_add_norm_quant.default._schema) == \
        "bonsai::fused_add_norm_quant(Tensor x, Tensor residual, Tensor w, float eps) -> (Tensor, Tensor, Tensor)"
    assert str(bonsai.silu_mul_quant.default._schema) == "bonsai::silu_mul_quant(Tensor gate_up) -> (Tensor, Tensor)"


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("m_shape", [(1,), (9,), (2, 5)])
def test_meta_shapes_follow_the_reference_wrappers(bonsai, bits, m_shape):
    """Rank-2 and rank-3 activations give [.., N] bf16, as model.py:231-240 derives out_shape
    (the reference's own meta-tensor checks: tests/test_bonsai_cpu.py:44-54)."""
    op = bonsai.t2g128_int8xint2_linear if bits == 2 else bonsai.q1g128_int8xint1_linear
    out = op(*_meta_problem(m_shape, 384, 2560, bits))
    assert out.shape == (*m_shape, 384) and out.dtype == torch.bfloat16 and out.device.type == "meta"
    out = op(*_meta_problem(m_shape, 384, 2560, bits, torch.float16))
    assert out.shape == (*m_shape, 384)


def test_meta_argument_checks(bonsai):
    a, b, s, ws = _meta_problem((3,), 256, 2048, 2)
    op = bonsai.t2g128_int8xint2_linear
    with pytest.raises(RuntimeError, match="activation width mismatch"):
        op(a[:, :1024], b, s, ws)
    with pytest.raises(RuntimeError, match="invalid weight scale shape"):
        op(a, b, s, ws[:, :8])
    with pytest.raises(RuntimeError, match="dtype"):
        op(a.to(torch.uint8), b, s, ws)
    with pytest.raises(RuntimeError, match="one value per row"):
        op(a, b, s[:2], ws)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        op(torch.empty(3, 192, dtype=torch.int8, device="meta"),
           torch.empty(256, 48, dtype=torch.int8, device="meta"), s,
           torch.empty(256, 1, dtype=torch.bfloat16, device="meta"))


def test_quant_input_meta(bonsai):
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        q, s = bonsai.quant_input(torch.empty(2, 7, 384, dtype=dt, device="meta"))
        assert q.shape == (2, 7, 384) and q.dtype == torch.int8
        assert s.shape == (2, 7, 1) and s.dtype == torch.float32
    with pytest.raises(RuntimeError, match="bf16, fp16 or fp32"):
        bonsai.quant_input(torch.empty(2, 128, dtype=torch.int32, device="meta"))


def test_fused_producers_meta(bonsai):
    """Shapes and dtypes of the fused producers as the reference's helpers return them
    (model.py:307-336, 1058-1061), and their argument checks."""
    x = torch.empty(2, 3, 2048, dtype=torch.bfloat16, device="meta")
    w = torch.empty(2048, dtype=torch.bfloat16, device="meta")
    q, s = bonsai.fused_norm_quant(x, w, 1e-6)
    assert q.shape == x.shape and q.dtype == torch.int8 and s.shape == (2, 3, 1) and s.dtype == torch.float32
    h, q, s = bonsai.fused_add_norm_quant(x, x, w, 1e-6)
    assert h.shape == x.shape and h.dtype == torch.bfloat16 and q.dtype == torch.int8 and s.shape == (2, 3, 1)
    gu = torch.empty(5, 2 * 6144, dtype=torch.bfloat16, device="meta")
    q, s = bonsai.silu_mul_quant(gu)
    assert q.shape == (5, 6144) and q.dtype == torch.int8 and s.shape == (5, 1)
    with pytest.raises(RuntimeError, match="weight must be bf16"):
        bonsai.fused_norm_quant(x, w[:1024], 1e-6)
    with pytest.raises(RuntimeError, match="residual must match"):
        bonsai.fused_add_norm_quant(x, x[:1], w, 1e-6)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        bonsai.silu_mul_quant(torch.empty(5, 24, dtype=torch.bfloat16, device="meta"))
    with pytest.raises(RuntimeError, match="bf16"):
        bonsai.silu_mul_quant(torch.empty(5, 32, dtype=torch.float32, device="meta"))


def test_cpu_tensors_have_no_kernel(bonsai):
    """There is no CPU implementation behind the operators: a CPU tensor is refused by the
    dispatcher rather than computed somewhere else."""
    with pytest.raises((RuntimeError, NotImplementedError)):
        bonsai.quant_input(torch.zeros(2, 128))


@pytest.mark.gpu
@pytest.mark.parametrize("bits, M, N, K", [(2, 1, 2048, 2048), (2, 9, 4096, 2048), (2, 3, 2048, 6144),
                                           (1, 1, 1024, 2560), (1, 8, 2560, 9728), (2, 17, 512, 1024)])
def test_registered_ops_equal_the_ctypes_operators(bonsai, bits, M, N, K):
    g = torch.Generator(device="cpu").manual_seed(bits * 1000 + M)
    x = torch.randn(M, K, generator=g).to("cuda", torch.bfloat16)
    b = torch.randint(-128, 128, (N, K * bits // 8), generator=g, dtype=torch.int8).cuda()
    ws = (torch.rand(N, K // 128, generator=g) * 0.05 + 0.01).to("cuda", torch.bfloat16)
    q_ref, s_ref = ops.quant_input(x)
    q, s = bonsai.quant_input(x)
    assert torch.equal(q, q_ref) and torch.equal(s, s_ref)
    ref_fn = ops.t2g128_int8xint2_linear if bits == 2 else ops.q1g128_int8xint1_linear
    op = bonsai.t2g128_int8xint2_linear if bits == 2 else bonsai.q1g128_int8xint1_linear
    y_ref = ref_fn(q, b, s, ws)
    y = op(q, b, s, ws)
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    assert torch.equal(y.view(torch.int16), y_ref.view(torch.int16))
    # rank-3 activations
    if M % 3 == 0:
        y3 = op(q.view(3, M // 3, K), b, s.view(3, M // 3, 1), ws)
        assert y3.shape == (3, M // 3, N) and torch.equal(y3.view(M, N).view(torch.int16), y.view(torch.int16))


@pytest.mark.gpu
def test_registered_ops_under_graph_capture(bonsai):
    """The operators allocate through PyTorch's allocator and launch on the current stream, so a
    captured graph replays them; every replay is compared with the eager result."""
    ops.init_kernels()
    M, N, K = 9, 4096, 2048
    g = torch.Generator(device="cpu").manual_seed(5)
    x = torch.randn(M, K, generator=g).to("cuda", torch.bfloat16)
    b = torch.randint(-128, 128, (N, K // 4), generator=g, dtype=torch.int8).cuda()
    ws = (torch.rand(N, K // 128, generator=g) * 0.05 + 0.01).to("cuda", torch.bfloat16)
    q, s = bonsai.quant_input(x)
    eager = bonsai.t2g128_int8xint2_linear(q, b, s, ws).clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        q2, s2 = bonsai.quant_input(x)
        y = bonsai.t2g128_int8xint2_linear(q2, b, s2, ws)
    for rep in range(3):
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), eager.view(torch.int16)), rep


@pytest.mark.gpu
@pytest.mark.parametrize("M, K", [(1, 2048), (9, 2560), (4, 6144)])
def test_registered_producers_equal_the_ctypes_operators(bonsai, M, K):
    g = torch.Generator(device="cpu").manual_seed(M * 7 + K)
    x = torch.randn(M, K, generator=g).to("cuda", torch.bfloat16)
    r = torch.randn(M, K, generator=g).to("cuda", torch.bfloat16)
    w = (torch.rand(K, generator=g) + 0.5).to("cuda", torch.bfloat16)
    q0, s0 = ops.fused_norm_quant(x, w, 1e-6)
    q1, s1 = bonsai.fused_norm_quant(x, w, 1e-6)
    assert torch.equal(q0, q1) and torch.equal(s0, s1)
    h0, q0, s0 = ops.fused_add_norm_quant(x, r, w, 1e-6)
    h1, q1, s1 = bonsai.fused_add_norm_quant(x, r, w, 1e-6)
    assert torch.equal(h0.view(torch.int16), h1.view(torch.int16)) and torch.equal(q0, q1) and torch.equal(s0, s1)
    gu = torch.randn(M, 2 * K, generator=g).to("cuda", torch.bfloat16)
    q0, s0 = ops.silu_mul_quant(gu)
    q1, s1 = bonsai.silu_mul_quant(gu)
    assert q1.shape == (M, K) and torch.equal(q0, q1) and torch.equal(s0, s1)
