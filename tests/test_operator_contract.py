"""Host-side behaviour of the operator layer, checked the way the reference checks
its own wrappers: on the allocation-free meta device and on CPU tensors, never
reaching native code (reference tests: tests/test_bonsai_cpu.py:44-54,
tests/test_bonsai_contracts.py:15-51)."""
import pytest
import torch

from bitmtp_amd import contracts, ops


@pytest.fixture
def strict():
    contracts.set_strict_reference_shapes(True)
    yield
    contracts.set_strict_reference_shapes(False)


def meta(shape, dtype):
    return torch.empty(shape, dtype=dtype, device="meta")


def test_strict_registry_matches_the_reference_sets(strict):
    for kind in ("q1", "t2g128"):
        for m in contracts.Q1_M:
            for n, k in contracts.BONSAI_17B_NK:
                assert contracts.supports_kernel_shape(kind, m, n, k)
    for n, k in contracts.T2_4B_NK:
        for m in contracts.T2_4B_M:
            assert contracts.supports_kernel_shape("t2g128", m, n, k)
        for m in (0, 2, 3, 4, 5, 6, 7, 11, 13, 18):
            with pytest.raises(RuntimeError, match="unsupported t2g128"):
                contracts.require_kernel_shape("t2g128", m, n, k)
        assert not contracts.supports_kernel_shape("q1", 1, n, k)
    for n, k in ((4096, 2560), (9728, 2560)):
        for m in contracts.Q1_M:
            assert not contracts.supports_kernel_shape("t2g128", m, n, k)
    for n, k in contracts.T2_4B_NK:
        assert contracts.supports_layer_kernel_shape("t2g128", 1, n, k)
        assert not contracts.supports_layer_kernel_shape("t2g128", 8, n, k)
    assert contracts.supports_kernel_shape("w1a16", 9, 151936, 2048)
    assert not contracts.supports_kernel_shape("w1a16", 9, 2048, 2048)
    with pytest.raises(ValueError, match="unknown kernel kind"):
        contracts.supports_kernel_shape("fp8", 1, 1, 128)


def test_strict_guard_precedes_library_load(strict, monkeypatch):
    """The reference's 4B guard test: widths 4..7 on the 4B head shape raise before
    any native library is touched."""
    monkeypatch.setattr(ops, "_t2_lib", None)
    for m in (4, 5, 6, 7):
        a = meta((m, 2560), torch.int8)
        b = meta((151936, 640), torch.int8)
        s = meta((m, 1), torch.float32)
        ws = meta((151936, 20), torch.bfloat16)
        with pytest.raises(RuntimeError, match="unsupported t2g128 kernel shape"):
            ops.t2g128_int8xint2_linear(a, b, s, ws)
    assert ops._t2_lib is None


def test_generic_mode_accepts_every_aligned_shape():
    assert not contracts.strict_reference_shapes()
    assert contracts.supports_kernel_shape("t2g128", 5, 151936, 2560)
    assert contracts.supports_kernel_shape("q1", 3, 9728, 9728)
    assert contracts.supports_kernel_shape("t2g128", 33, 7, 128)
    for m, n, k in ((0, 8, 128), (1, 0, 128), (1, 8, 0), (1, 8, 192)):
        with pytest.raises(RuntimeError, match="unsupported t2g128 kernel shape"):
            contracts.require_kernel_shape("t2g128", m, n, k)


def test_shapes_past_the_launcher_limits_raise_before_the_native_call():
    """The void drop-in symbol cannot report an error, so the wrapper must refuse what the
    launcher would refuse: more than 2^30 output elements, rows longer than 65536."""
    assert contracts.supports_kernel_shape("t2g128", 7067, 151936, 2048)       # just below 2^30
    assert not contracts.supports_kernel_shape("t2g128", 7068, 151936, 2048)
    assert not contracts.supports_kernel_shape("q1", 1, 8, 65536 + 128)
    a = torch.empty(7068, 2048, dtype=torch.int8, device="meta")
    b = torch.empty(151936, 512, dtype=torch.int8, device="meta")
    s = torch.empty(7068, 1, dtype=torch.float32, device="meta")
    ws = torch.empty(151936, 16, dtype=torch.bfloat16, device="meta")
    with pytest.raises(RuntimeError, match="unsupported t2g128 kernel shape"):
        ops.t2g128_int8xint2_linear(a, b, s, ws)


@pytest.mark.parametrize("fn,bits,kind", [(ops.t2g128_int8xint2_linear, 2, "t2g128"),
                                          (ops.q1g128_int8xint1_linear, 1, "q1")])
def test_validation_messages(fn, bits, kind, monkeypatch):
    monkeypatch.setattr(ops, "_t2_lib", None)
    monkeypatch.setattr(ops, "_q1_lib", None)
    K, N, M = 256, 8, 2
    cols = K * bits // 8
    a, b = meta((M, K), torch.int8), meta((N, cols), torch.int8)
    s, ws = meta((M, 1), torch.float32), meta((N, K // 128), torch.bfloat16)
    with pytest.raises(ValueError, match="expected rank-2/3 activation and rank-2 weight"):
        fn(meta((K,), torch.int8), b, s, ws)
    with pytest.raises(ValueError, match="expected rank-2/3"):
        fn(a, meta((1, N, cols), torch.int8), s, ws)
    with pytest.raises(RuntimeError, match="activation width mismatch"):
        fn(meta((M, K + 128), torch.int8), b, s, ws)
    with pytest.raises(RuntimeError, match="invalid weight scale shape"):
        fn(a, b, s, meta((N, K // 128 + 1), torch.bfloat16))
    with pytest.raises(RuntimeError, match="invalid activation, packed-weight, or scale dtype"):
        fn(a, b, s, meta((N, K // 128), torch.float16))
    with pytest.raises(RuntimeError, match="invalid activation, packed-weight, or scale dtype"):
        fn(meta((M, K), torch.uint8), b, s, ws)
    with pytest.raises(RuntimeError, match="activation scales must be float32 with one value per row"):
        fn(a, b, meta((M,), torch.float32), ws)
    with pytest.raises(RuntimeError, match="activation scales must be float32"):
        fn(a, b, meta((M, 1), torch.float16), ws)
    with pytest.raises(RuntimeError, match="must be contiguous CUDA tensors"):
        fn(a, b, s, ws)  # meta tensors are not CUDA tensors
    cpu = [torch.zeros(t.shape, dtype=t.dtype) for t in (a, b, s, ws)]
    with pytest.raises(RuntimeError, match="must be contiguous CUDA tensors"):
        fn(*cpu)
    assert ops._t2_lib is None and ops._q1_lib is None  # nothing native was loaded


@pytest.mark.parametrize("bits,kind", [(2, "t2g128"), (1, "q1")])
def test_group_sum_calls_check_their_operands_before_any_native_call(bits, kind, monkeypatch):
    """A call for the int32 group sums reads no scales, but its activations and weights are
    checked like any other call -- single and grouped alike: raw pointers of these tensors go
    to the kernel, so a wrong width, dtype, device or stride must raise here."""
    monkeypatch.setattr(ops, "_t2_lib", None)
    monkeypatch.setattr(ops, "_q1_lib", None)
    K, N, M = 2048, 32, 3
    cols = K * bits // 8
    a, b = meta((M, K), torch.int8), meta((N, cols), torch.int8)

    def single(a_, b_):
        return ops.packed_gemv_ex(a_, b_, None, None, bits=bits, out_kind=ops.OUT_G32)

    def grouped(a_, b_):
        return ops.packed_gemv_grouped([(a_, b_, None, None)], bits=bits, out_kind=ops.OUT_G32)

    for call in (single, grouped):
        with pytest.raises(RuntimeError, match="activation width mismatch"):
            call(meta((M, K + 128), torch.int8), b)
        with pytest.raises(RuntimeError, match="invalid activation or packed-weight dtype"):
            call(meta((M, K), torch.uint8), b)
        with pytest.raises(RuntimeError, match="invalid activation or packed-weight dtype"):
            call(a, meta((N, cols), torch.uint8))
        with pytest.raises(ValueError, match="rank-2"):
            call(meta((1, M, K), torch.int8), b)
        with pytest.raises(RuntimeError, match="must be contiguous CUDA tensors"):
            call(a, b)  # meta tensors are not CUDA tensors
        with pytest.raises(RuntimeError, match="must be contiguous CUDA tensors"):
            call(torch.zeros(M, K, dtype=torch.int8), torch.zeros(N, cols, dtype=torch.int8))
        with pytest.raises(RuntimeError, match="must be contiguous CUDA tensors"):
            call(torch.zeros(M, 2 * K, dtype=torch.int8)[:, ::2], torch.zeros(N, cols, dtype=torch.int8))
    assert ops._t2_lib is None and ops._q1_lib is None  # nothing native was loaded


def test_dispatcher_by_packed_width():
    a = meta((1, 256), torch.int8)
    with pytest.raises(ValueError, match="unknown packed weight layout"):
        ops.packed_int8_linear(a, meta((8, 100), torch.int8), None, None)
    s, ws = meta((1, 1), torch.float32), meta((8, 2), torch.bfloat16)
    # K/8 columns routes to q1, K/4 to t2: seen through the kind named in the message
    with pytest.raises(RuntimeError, match="^q1: inputs and scales must be contiguous CUDA"):
        ops.packed_int8_linear(a, meta((8, 32), torch.int8), s, ws)
    with pytest.raises(RuntimeError, match="^t2g128: inputs and scales must be contiguous CUDA"):
        ops.packed_int8_linear(a, meta((8, 64), torch.int8), s, ws)


def test_w1a16_requires_rank2_bf16():
    with pytest.raises(ValueError, match="rank-2 activation"):
        ops.q1g128_w1a16_linear(meta((1, 2, 256), torch.bfloat16), meta((8, 32), torch.int8),
                                meta((8, 2), torch.bfloat16))
    with pytest.raises(RuntimeError, match="invalid activation"):
        ops.q1g128_w1a16_linear(meta((2, 256), torch.float16), meta((8, 32), torch.int8),
                                meta((8, 2), torch.bfloat16))


def test_quant_input_rejects_bad_inputs():
    with pytest.raises(RuntimeError, match="bfloat16, float16 or float32"):
        ops.quant_input(torch.zeros(2, 128, dtype=torch.int8))
    with pytest.raises(RuntimeError, match="contiguous CUDA tensor"):
        ops.quant_input(torch.zeros(2, 128, dtype=torch.float16))


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    """No fallback: an absent library raises instead of computing anything."""
    monkeypatch.setattr(ops, "_HERE", str(tmp_path))
    monkeypatch.setattr(ops, "_t2_lib", None)
    with pytest.raises(RuntimeError, match="there is no fallback implementation"):
        ops.load_t2_kernel()
