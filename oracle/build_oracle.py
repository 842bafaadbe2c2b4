"""Compile and load oracle.c (test infrastructure, not part of the product)."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle.so")


def build() -> str:
    subprocess.run(["make", "-C", HERE, "-B", "liboracle.so"], check=True, stdout=subprocess.DEVNULL)
    return LIB


def load():
    if not os.path.exists(LIB):
        build()
    lib = C.CDLL(LIB)
    i64, p, i = C.c_int64, C.c_void_p, C.c_int
    lib.orc_pack_sign_f32.argtypes = [p, p, i64]
    lib.orc_pack_sign_f32.restype = None
    lib.orc_hamming_score.argtypes = [p, p, p, i, i64, i, i, i, i]
    lib.orc_hamming_score.restype = None
    lib.orc_topk_select.argtypes = [p, p, i, i64, i, i, i]
    lib.orc_topk_select.restype = i
    lib.orc_sparse_attention_f32.argtypes = [p, p, p, p, p, i, i, i, i, i64, i]
    lib.orc_sparse_attention_f32.restype = None
    return lib
