"""Compile the oracle's C restatement (``oracle/fp8_e4m3fn.c``) with gcc into ``oracle/_build/``.

TEST INFRASTRUCTURE ONLY.  The reference's device code is TileLang-generated CUDA (tilelang >=0.1.9,<0.2.0,
absent here), so there is no reference source that compiles with gcc: ``oracle/_ref`` is not built.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT_DIR = HERE / "_build"
LIB = OUT_DIR / "liboracle_fp8.so"


def build() -> Path:
    OUT_DIR.mkdir(exist_ok=True)
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-std=c99", "-o", str(LIB), str(HERE / "fp8_e4m3fn.c"), "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"gcc failed on the oracle:\n{res.stderr}")
    return LIB


def load() -> ctypes.CDLL:
    if not LIB.exists():
        build()
    lib = ctypes.CDLL(str(LIB))
    u8p, f32p, i64 = ctypes.POINTER(ctypes.c_uint8), ctypes.POINTER(ctypes.c_float), ctypes.c_int64
    lib.fp8_e4m3fn_decode.restype = ctypes.c_float
    lib.fp8_e4m3fn_decode.argtypes = [ctypes.c_uint8]
    lib.fp8_e4m3fn_encode.restype = ctypes.c_uint8
    lib.fp8_e4m3fn_encode.argtypes = [ctypes.c_float]
    lib.fp8_e4m3fn_decode_n.argtypes = [u8p, f32p, i64]
    lib.fp8_e4m3fn_encode_n.argtypes = [f32p, u8p, i64]
    lib.fp8_quant_per_token.argtypes = [f32p, u8p, f32p, i64, i64]
    return lib


if __name__ == "__main__":
    print(build())
