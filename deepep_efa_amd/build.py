"""Builds the gfx950 HIP library (csrc/*.hip -> libdeepep_hip.so) with hipcc.

hipcc cross-compiles without a GPU.  The flag pair
``-Xclang -target-feature -Xclang -packed-fp32-ops`` keeps the compiler from
forming packed-FP32 instructions; the host pass prints that it does not know
the feature, which is harmless and filtered from the output here.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libdeepep_hip.so")
SOURCES = ["lib.cpp", "ll_dispatch.hip", "ll_combine.hip", "ll_exchange_meta.hip", "ll_recv_by_source.hip", "layout.hip", "normal_meta.hip", "cast.hip", "loopback.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
         "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_hip_library(verbose: bool = True) -> str:
    cmd = ["hipcc"] + FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if verbose and out.strip():
        print(out, file=sys.stderr)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return LIB


BENCH_PROBE_SRC = os.path.join(os.path.dirname(HERE), "bench_probe.hip")
BENCH_PROBE = os.path.join(os.path.dirname(HERE), "bench_probe.so")


def build_bench_probe(verbose: bool = True) -> str:
    """Builds the measuring-stick kernels bench.py times beside the library's own (bench_probe.hip beside
    bench.py -> bench_probe.so).  They are not part of libdeepep_hip.so."""
    cmd = ["hipcc"] + FLAGS + [f"-I{os.path.dirname(HERE)}", BENCH_PROBE_SRC, "-o", BENCH_PROBE]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if verbose and out.strip():
        print(out, file=sys.stderr)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return BENCH_PROBE


BENCH_PHASE_SRC = os.path.join(os.path.dirname(HERE), "bench_phase.hip")
BENCH_PHASE = os.path.join(os.path.dirname(HERE), "bench_phase.so")


def build_bench_phase(verbose: bool = True) -> str:
    """Builds the timing build for `bench.py --phase-marks` (bench_phase.hip beside bench.py -> bench_phase.so):
    the whole C ABI again, with the two low-latency kernel files compiled with their phase marks switched on."""
    rest = [s for s in SOURCES if s not in ("ll_dispatch.hip", "ll_combine.hip")]
    cmd = (["hipcc"] + FLAGS + [f"-I{os.path.dirname(HERE)}", BENCH_PHASE_SRC] + [os.path.join(CSRC, s) for s in rest]
           + ["-o", BENCH_PHASE])
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if verbose and out.strip():
        print(out, file=sys.stderr)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return BENCH_PHASE


HOST_MODULE = os.path.join(HERE, "deep_ep_cpp.so")


def build_host_module(verbose: bool = True) -> str:
    """Builds the pybind11 host module deep_ep_cpp (C++ only, no device code) with g++
    against the installed PyTorch-ROCm and links it to libdeepep_hip.so."""
    import sysconfig

    import torch
    tdir = os.path.dirname(torch.__file__)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function", "-Wno-sign-compare",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=deep_ep_cpp",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{tdir}/include", f"-I{tdir}/include/torch/csrc/api/include", f"-I{sysconfig.get_paths()['include']}",
           "-I/opt/rocm/include", os.path.join(CSRC, "deep_ep_cpp.cpp"), "-o", HOST_MODULE,
           f"-L{HERE}", "-ldeepep_hip", f"-L{tdir}/lib", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
           "-ltorch_python", "-lamdhip64", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tdir}/lib"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose and proc.stdout.strip():
        print(proc.stdout, file=sys.stderr)
    if proc.returncode != 0:
        raise RuntimeError("g++ failed:\n" + proc.stdout)
    return HOST_MODULE


if __name__ == "__main__":
    print(build_hip_library())
    print(build_host_module())
    print(build_bench_probe())
    print(build_bench_phase())
