"""Builds the C checker (oracle_kernels.c -> _build/liboracle.so) with gcc.

There is no reference build here: the reference's path is CUDA (nvcc, cuda_fp8.h,
libfabric, GDRCopy) and cannot be compiled in this image, so no oracle/_ref exists.
"""
import ctypes
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "_build", "liboracle.so")


def build() -> str:
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    cmd = ["gcc", "-O2", "-std=c11", "-shared", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
           os.path.join(HERE, "oracle_kernels.c"), "-o", LIB, "-lm"]
    subprocess.run(cmd, check=True)
    return LIB


def load() -> ctypes.CDLL:
    """Loads the built checker; builds it first if it is missing."""
    if not os.path.exists(LIB):
        build()
    lib = ctypes.CDLL(LIB)
    c = ctypes
    lib.oracle_e4m3_encode.restype = c.c_uint8
    lib.oracle_e4m3_encode.argtypes = [c.c_float]
    lib.oracle_e4m3_decode.restype = c.c_float
    lib.oracle_e4m3_decode.argtypes = [c.c_uint8]
    lib.oracle_e4m3_encode_many.argtypes = [c.c_void_p, c.c_void_p, c.c_int64]
    lib.oracle_per_token_cast.argtypes = [c.c_void_p, c.c_int64, c.c_int, c.c_int, c.c_void_p, c.c_void_p]
    lib.oracle_combine_chain.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_int64, c.c_int, c.c_int, c.c_void_p]
    lib.oracle_mix32.restype = c.c_uint32
    lib.oracle_mix32.argtypes = [c.c_uint32]
    lib.oracle_synth_bf16_rows.argtypes = [c.c_void_p, c.c_int64, c.c_int, c.c_uint32, c.c_int, c.c_void_p]
    lib.oracle_synth_topk_idx.argtypes = [c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_int, c.c_uint32,
                                          c.c_void_p]
    return lib


if __name__ == "__main__":
    print(build())
