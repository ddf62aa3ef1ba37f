"""Builds the native libraries in-tree with hipcc / g++ (no JIT cache: the .so files travel with the tree)."""
from __future__ import annotations

import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(PKG, "build")
NATIVE_LIB = os.path.join(LIBDIR, "libm40llm_native.so")
HOST_LIB = os.path.join(LIBDIR, "libm40llm_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    # hipcc fuses float pairs into packed-FP32 instructions by itself; keep those out.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
HIP_SOURCES = ["context.hip", "elementwise.hip", "gemm.hip", "kvcache.hip", "attention.hip", "block_select.hip",
               "decode_fused.hip", "skinny_mfma.hip", "attention_mfma.hip", "rows_gemv.hip", "rows_mfma.hip", "rows_khalf_mfma.hip", "prefill_attention.hip", "gemm_tiled.hip", "q80_i8.hip"]
CPP_SOURCES = ["unavailable.cpp"]
# per-file additions: matrix-instruction results straight into vector registers (the default form writes them to
# accumulation registers and copies every element out again)
HIP_FILE_FLAGS = {"prefill_attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_native(verbose: bool = False) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    jobs = []
    for src in HIP_SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(OBJDIR, src + ".o")
        jobs.append(([HIPCC, *HIP_FLAGS, *HIP_FILE_FLAGS.get(src, []), "-c", path, "-o", obj], obj))
    for src in CPP_SOURCES:
        obj = os.path.join(OBJDIR, src + ".o")
        jobs.append((["g++", "-O2", "-std=c++17", "-fPIC", "-c", os.path.join(CSRC, src), "-o", obj], obj))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        outs = list(ex.map(lambda j: _run(j[0]), jobs))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    objs = [j[1] for j in jobs]
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", NATIVE_LIB, *objs])
    return NATIVE_LIB


def build_host(verbose: bool = False) -> str:
    """C++ host layer above the C ABI (decode loop, batch plan, KV config, selection telemetry, model step)."""
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp")) if os.path.isdir(HOST) else []
    if not srcs:
        return ""
    out = _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", os.path.join(PKG, "..", "include"),
                "-o", HOST_LIB, *srcs, "-L", LIBDIR, "-lm40llm_native", "-Wl,-rpath,$ORIGIN", "-lpthread"])
    if verbose and out.strip():
        print(out)
    return HOST_LIB


def build_all(verbose: bool = False):
    return build_native(verbose), build_host(verbose)


if __name__ == "__main__":
    print(build_all(verbose=True))
