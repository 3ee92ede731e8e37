"""Builds libapt_hip.so (the C-ABI HIP library) for gfx950 with hipcc, libnpc.so (its torch
operator binding) and libapt_bench.so (synthetic inputs and measurement helpers of the benchmark
and the tests: a library of its own, so that libapt_hip.so exports the product ABI only).

Run it as a script (`python apt_amd/build.py`): importing it as `apt_amd.build`
would first import the package, which needs the libraries this file produces.

The library has no dependency on torch or Python: it is plain HIP.  hipcc
cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is
installed.  The result is written next to this file and loaded by capi.py.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libapt_hip.so")
NPC_LIB = os.path.join(HERE, "libnpc.so")
BENCH_LIB = os.path.join(HERE, "libapt_bench.so")
SOURCES = ["lib.hip", "sample.hip", "relabel.hip", "gather.hip", "bucket.hip", "minibatch.hip", "spmm.hip", "cache.hip", "block.hip", "epoch.hip"]
BENCH_SOURCES = ["synth.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Wall", "-Wno-unused-function",
    # packed-FP32 code generation is kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _obj(src):
    return os.path.join(CSRC, os.path.splitext(src)[0] + ".o")


def build(force=True, verbose=False):
    """Compile every source and link libapt_hip.so.  Returns its path."""
    procs = []
    headers = [os.path.join(CSRC, h) for h in sorted(os.listdir(CSRC)) if h.endswith(".hpp")]
    headers += [os.path.join(HERE, "..", "include", "apt_amd.h"), os.path.join(HERE, "..", "include", "apt_synth.h")]
    newest_hdr = max(os.path.getmtime(h) for h in headers)
    objs, bench_objs = [], []
    for s in SOURCES + BENCH_SOURCES:
        src = os.path.join(CSRC, s)
        obj = _obj(s)
        (bench_objs if s in BENCH_SOURCES else objs).append(obj)
        stale = (force or not os.path.exists(obj)
                 or os.path.getmtime(obj) < max(os.path.getmtime(src), newest_hdr))
        if stale:
            cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
            if verbose:
                print(" ".join(cmd), file=sys.stderr)
            procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    for s, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        # hipcc's host pass does not know the packed-fp32 feature name; harmless
        text = "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {s}:\n{text}")
        if verbose and text.strip():
            print(text, file=sys.stderr)
    # -Bsymbolic: each library binds its own helpers (both define apt::last_error_buf)
    for lib, parts in ((LIB, objs), (BENCH_LIB, bench_objs)):
        subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", lib, *parts])
    build_torch_binding(verbose=verbose)
    build_c_consumer(verbose=verbose)
    return LIB


C_CONSUMER_SRC = os.path.join(HERE, "..", "tests", "c_abi", "epoch_consumer.c")
C_CONSUMER = os.path.join(HERE, "..", "tests", "c_abi", "epoch_consumer")


def build_c_consumer(verbose=False):
    """Compile the plain-C program that drives the library through include/apt_amd.h alone (gcc, C11; the GPU
    tests run it).  Skipped when the source is not there (an installed copy of the package without the tests)."""
    if not os.path.exists(C_CONSUMER_SRC):
        return None
    cmd = [os.environ.get("CC", "gcc"), "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror",
           f"-I{os.path.join(HERE, '..', 'include')}", "-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__",
           C_CONSUMER_SRC, f"-L{HERE}", "-lapt_hip", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../apt_amd", "-Wl,-rpath,/opt/rocm/lib", "-o", C_CONSUMER]
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    subprocess.check_call(cmd)
    return C_CONSUMER


def build_torch_binding(verbose=False):
    """Compile libnpc.so: TORCH_LIBRARY(npc) over the C ABI (host code only)."""
    import torch
    from torch.utils import cpp_extension as ce

    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           os.path.join(CSRC, "torch_bind.cc"), "-o", NPC_LIB,
           *[f"-I{p}" for p in ce.include_paths()], "-I/opt/rocm/include",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-L{tlib}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
           f"-L{HERE}", "-lapt_hip", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"]
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    subprocess.check_call(cmd)
    return NPC_LIB


if __name__ == "__main__":
    print(build(force="--incremental" not in sys.argv, verbose=True))
