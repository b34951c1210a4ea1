"""Builds the gfx950 shared libraries of this package with hipcc, in-tree, and the PyTorch
operator library on top of them with g++.

    python -m bitmtp_amd.build            # build what is missing or out of date
    python -m bitmtp_amd.build --force    # rebuild everything

The libraries keep the file names the reference loader expects
(``t2g128_kernels/libbonsai_t2.so`` and ``q1g128_kernels/libbonsai_q1.so`` next
to the operator module, src/bonsai_sft/gpu/model.py:77-78,209-210; its build
script is src/bonsai_sft/gpu/t2g128_kernels/compile.sh:12-18).  hipcc
cross-compiles for gfx950 without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")

# source (under csrc/, or a path relative to the package) -> library (under the package)
TARGETS = {
    "t2g128_kernels.hip": os.path.join("t2g128_kernels", "libbonsai_t2.so"),
    "q1g128_kernels.hip": os.path.join("q1g128_kernels", "libbonsai_q1.so"),
    "act_quant.hip": os.path.join("act_quant", "libbonsai_actq.so"),
    "decode_ops.hip": os.path.join("decode_ops", "libbonsai_decode.so"),
    # measurement aids of the benchmarks, apart from the drop-in libraries
    os.path.join("..", "bench_probe", "bench_probe.hip"): os.path.join("bench_probe", "libbonsai_probe.so"),
}

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed fp32 VALU forms are kept out of generated code on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results go to ordinary VGPRs: the scale-accumulate epilogue consumes them
    # at once and v_accvgpr_read copies would cost four VALU slots per tile
    "-mllvm", "--amdgpu-mfma-vgpr-form",
    # scalar kernel arguments arrive in SGPRs with the wave instead of through a load
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def lib_path(source: str) -> str:
    return os.path.join(HERE, TARGETS[source])


def _deps() -> list[str]:
    probe = os.path.join(HERE, "bench_probe")
    return [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [
        os.path.join(probe, f) for f in os.listdir(probe) if f.endswith((".hip", ".h"))] + [
        os.path.join(HERE, "..", "include", h) for h in ("bonsai_gemv.h", "bonsai_decode.h", "bonsai_probe.h")]


def _stale(out: str) -> bool:
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(d) > t for d in _deps() if os.path.exists(d))


def _build_one(source: str) -> str:
    out = lib_path(source)
    os.makedirs(os.path.dirname(out), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + [os.path.join(CSRC, source), "-o", out]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {source}:\n{proc.stdout}")
    return out


def build_all(force: bool = False, verbose: bool = True) -> list[str]:
    todo = [s for s in TARGETS if os.path.exists(os.path.join(CSRC, s))
            and (force or _stale(lib_path(s)))]
    with ThreadPoolExecutor(max_workers=max(1, len(todo))) as pool:
        built = list(pool.map(_build_one, todo))
    if verbose:
        for b in built:
            print(f"[bitmtp_amd.build] built {os.path.relpath(b, HERE)}")
    return [lib_path(s) for s in TARGETS if os.path.exists(lib_path(s))]


# ---- the PyTorch operator library (host code only, g++) ---------------------------------
TORCH_OPS_SOURCE = "torch_ops.cpp"
TORCH_OPS_LIB = os.path.join("torch_ops", "libbonsai_torch.so")


def torch_ops_path() -> str:
    return os.path.join(HERE, TORCH_OPS_LIB)


def build_torch_ops(force: bool = False, verbose: bool = True) -> str:
    """Compiles csrc/torch_ops.cpp against the installed PyTorch and links it to the three C-ABI
    libraries it calls (found at run time next to it through $ORIGIN).  No device code."""
    out = torch_ops_path()
    if not force and not _stale(out):
        return out
    build_all(verbose=verbose)  # the libraries it links to
    import torch
    tdir = os.path.dirname(torch.__file__)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    os.makedirs(os.path.dirname(out), exist_ok=True)
    libdirs = [os.path.dirname(lib_path(s)) for s in ("t2g128_kernels.hip", "q1g128_kernels.hip", "act_quant.hip")]
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{tdir}/include", f"-I{tdir}/include/torch/csrc/api/include", f"-I{rocm}/include",
           os.path.join(CSRC, TORCH_OPS_SOURCE), "-o", out,
           f"-L{tdir}/lib", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip"]
    cmd += [f"-L{d}" for d in libdirs] + ["-lbonsai_t2", "-lbonsai_q1", "-lbonsai_actq",
            "-Wl,-rpath,$ORIGIN/../t2g128_kernels:$ORIGIN/../q1g128_kernels:$ORIGIN/../act_quant"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"g++ failed for {TORCH_OPS_SOURCE}:\n{proc.stdout}")
    if verbose:
        print(f"[bitmtp_amd.build] built {os.path.relpath(out, HERE)}")
    return out


if __name__ == "__main__":
    build_all(force="--force" in sys.argv[1:])
    build_torch_ops(force="--force" in sys.argv[1:])
