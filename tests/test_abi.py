"""The C-ABI libraries load without a GPU and export every entry point that the headers
under include/ declare (no compute call is made here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("bonsai_gemv.h", "bonsai_decode.h", "bonsai_probe.h")]


def declared_functions():
    names = set()
    for header in HEADERS:
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(?:int|void|int64_t|const char \*)\s*([a-z0-9_]+)\s*\(", text))
    return sorted(names)


@pytest.fixture(scope="module")
def libs():
    from bitmtp_amd import build, ops
    build.build_all(verbose=False)  # compiles only what is missing or out of date
    from bitmtp_amd import decode_ops
    from bitmtp_amd import probe
    paths = [ops.t2_lib_path(), ops.q1_lib_path(), ops.actq_lib_path(),
             decode_ops.decode_lib_path(), probe.probe_lib_path()]
    assert all(os.path.exists(p) for p in paths)
    return [ctypes.CDLL(p) for p in paths]


def test_header_declares_the_drop_in_symbols():
    names = declared_functions()
    for required in ("t2g128_int8xint2_linear", "q1g128_int8xint1_linear", "q1g128_w1a16_linear"):
        assert required in names


def test_every_declared_symbol_is_exported(libs):
    for name in declared_functions():
        owners = [lib for lib in libs if hasattr(lib, name)]
        assert len(owners) == 1, f"{name} exported by {len(owners)} libraries"


def test_reference_loader_view_of_the_libraries(libs):
    """What the reference's ctypes loaders touch (src/bonsai_sft/gpu/model.py:70-93,
    206-219): both Q1 symbols in libbonsai_q1.so, the T2 symbol in libbonsai_t2.so."""
    t2, q1 = libs[0], libs[1]
    assert hasattr(t2, "t2g128_int8xint2_linear")
    assert hasattr(q1, "q1g128_int8xint1_linear") and hasattr(q1, "q1g128_w1a16_linear")
    from bitmtp_amd import ops
    assert ops.t2_lib_path().endswith(os.path.join("t2g128_kernels", "libbonsai_t2.so"))
    assert ops.q1_lib_path().endswith(os.path.join("q1g128_kernels", "libbonsai_q1.so"))


def test_python_binding_sets_argtypes():
    from bitmtp_amd import ops
    ops.load_t2_kernel()
    ops.load_q1_kernel()
    ops.load_actq_kernel()
    assert len(ops.t2_lib().t2g128_int8xint2_linear.argtypes) == 9
    assert ops.t2_lib().t2g128_int8xint2_linear.restype is None
    assert len(ops.q1_lib().q1g128_w1a16_linear.argtypes) == 8
    assert len(ops.t2_lib().t2g128_gemv_ex.argtypes) == 11


def test_decode_library_exports_and_binding(libs):
    assert sorted(os.listdir(os.path.join(ROOT, "include"))) == ["bonsai_decode.h", "bonsai_gemv.h",
                                                                  "bonsai_probe.h"]
    dec = libs[3]
    for name in ("bonsai_qk_norm_rope_kv_write", "bonsai_decode_attention",
                 "bonsai_decode_attention_scratch_bytes", "bonsai_kv_commit", "bonsai_draft_chain",
                 "bonsai_bf16_linear", "bonsai_fp8_quant_rows", "bonsai_fp8_linear",
                 "bonsai_decode_set_tuning", "bonsai_decode_set_attention_engine",
                 "bonsai_draft_chain_ws", "bonsai_draft_chain_scratch_bytes",
                 "bonsai_draft_chain_static", "bonsai_decode_init"):
        assert name in declared_functions() and hasattr(dec, name)
    from bitmtp_amd import decode_ops
    decode_ops.load_decode_kernel()
    assert len(decode_ops.decode_lib().bonsai_decode_attention.argtypes) == 15
    # host-only query: partials are [M][heads][chunks][132] fp32
    assert decode_ops.attention_scratch_bytes(9, 16, 1024 + 17) == 9 * 16 * 17 * 132 * 4
    assert decode_ops.attention_scratch_bytes(0, 16, 64) == 0


def test_argument_checks_need_no_gpu():
    """The entry points refuse bad arguments before they touch the device: null pointers, a K
    that is no multiple of 128, and operands that are not aligned for the 16-byte vector loads
    (the pointers here are never dereferenced)."""
    from bitmtp_amd import ops
    t2, q1 = ops.t2_lib(), ops.q1_lib()
    VP = ctypes.c_void_p
    ok = dict(A=0x10000, B=0x20000, out=0x30000, s=0x40000, ws=0x50000)

    def call(lib_fn, M=1, N=16, K=128, **over):
        a = dict(ok, **over)
        return lib_fn(VP(a["A"]), VP(a["B"]), VP(a["out"]), VP(a["s"]), VP(a["ws"]), M, N, K, 0, 0, None)

    for fn in (t2.t2g128_gemv_ex, q1.q1g128_gemv_ex):
        assert call(fn, A=None) == 1 and call(fn, B=None) == 1 and call(fn, out=None) == 1
        assert call(fn, K=64) == 1 and call(fn, K=192) == 1 and call(fn, M=0) == 1 and call(fn, N=0) == 1
        assert call(fn, A=0x10008) == 1 and call(fn, B=0x20004) == 1    # 16-byte loads
        assert call(fn, ws=0x50001) == 1 and call(fn, s=0x40002) == 1 and call(fn, out=0x30001) == 1
        assert call(fn, M=70000, N=151936) == 1                          # M * N beyond the index range
    d = (ops.GemvDesc * 1)(ops.GemvDesc(0x10008, 0x20000, 0x30000, 0x40000, 0x50000, 1, 16, 2048, 0))
    assert t2.t2g128_gemv_grouped(d, 1, 0, 0, None) == 1
    assert t2.t2g128_gemv_grouped(d, 0, 0, 0, None) == 1
    # the read probe: null or misaligned pointers, and a one-shot launch of more than eight loads
    # per thread (256 threads x 16 bytes x 8 per workgroup)
    from bitmtp_amd import probe as probe_mod
    assert not hasattr(t2, "bonsai_read_probe")  # measurement aids live in their own library
    probe = probe_mod.probe_lib().bonsai_read_probe
    assert probe(None, 4096, 1, 0, VP(0x40000), None) == 1
    assert probe(VP(0x10000), 4096, 1, 0, None, None) == 1
    assert probe(VP(0x10008), 4096, 1, 0, VP(0x40000), None) == 1
    assert probe(VP(0x10000), 4096, 0, 0, VP(0x40000), None) == 1
    assert probe(VP(0x10000), 256 * 16 * 8 + 16, 1, 0, VP(0x40000), None) == 1
