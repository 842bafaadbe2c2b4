"""ctypes binding of libspotlight_hip.so (the C ABI in include/spotlight_hip.h).

The library is the only compute path of this package: if it is missing the
import of any op fails loudly, there is no eager or CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# SPOTLIGHT_HIP_LIB points at another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("SPOTLIGHT_HIP_LIB") or os.path.join(_HERE, "libspotlight_hip.so")

SL_F32, SL_BF16, SL_F16 = 0, 1, 2
SL_HEADMAP_INTERLEAVED, SL_HEADMAP_BLOCKED = 0, 1
STAMP_WGS, STAMP_SLOTS = 4096, 24
STAGE_HASH, STAGE_SCORE, STAGE_SELECT, STAGE_LRU, STAGE_ATTN, STAGE_ALL = 1, 2, 4, 8, 16, 31

c_void_p, c_int, c_int64, c_size_t, c_float, c_uint32 = (
    C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float, C.c_uint32)


class DecodeParams(C.Structure):
    """Mirror of sl_decode_params."""
    _fields_ = [
        ("dtype", c_int), ("B", c_int), ("QH", c_int), ("KH", c_int), ("d", c_int),
        ("nbits", c_int), ("k", c_int), ("head_map", c_int),
        ("n_cap", c_int64), ("n_max", c_int64),
        ("q", c_void_p), ("k_new", c_void_p), ("v_new", c_void_p),
        ("rope_inv_freq", c_void_p), ("q_rot", c_void_p),
        ("n_layers", c_int), ("d_hid", c_int), ("residue", c_int),
        ("w1_q", c_void_p), ("b1_q", c_void_p), ("w2_q", c_void_p), ("b2_q", c_void_p),
        ("w1_k", c_void_p), ("b1_k", c_void_p), ("w2_k", c_void_p), ("b2_k", c_void_p),
        ("codes_head_major", c_int), ("codes", c_void_p), ("keys", c_void_p), ("vals", c_void_p), ("seq_lens", c_void_p),
        ("out", c_void_p), ("idx", c_void_p),
        ("lru_C", c_int), ("lru_map_cap", c_int64),
        ("slot_token", c_void_p), ("slot_stamp", c_void_p), ("token_slot", c_void_p),
        ("k_res", c_void_p), ("v_res", c_void_p), ("slots_out", c_void_p),
        ("lru_stats", c_void_p), ("step_counter", c_void_p),
        ("ws", c_void_p), ("ws_bytes", c_size_t),
        ("budget_on", c_int), ("budget_min_remain", c_int), ("budget_mask_out", C.c_double),
    ]


# name -> (restype, argtypes); every symbol include/spotlight_hip.h declares
SIGNATURES = {
    "sl_strerror": (C.c_char_p, [c_int]),
    "sl_version": (c_int, []),
    "sl_tune": (c_int, [C.c_char_p, c_int]),
    "sl_host_device_pointer": (c_int, [c_void_p, C.POINTER(c_void_p)]),
    "sl_pack_sign_u32": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p]),
    "sl_pack_sign_u8": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p]),
    "sl_hash_mlp_pack": (c_int, [c_void_p] * 6 + [c_int] * 8 + [c_int64] * 4 + [c_void_p, c_void_p]),
    "sl_hash_rows_pack": (c_int, [c_void_p] * 6 + [c_int, c_int, c_int, c_int64] + [c_int] * 5 + [c_int64] * 5 + [c_void_p]),
    "sl_hamming_score": (c_int, [c_void_p] * 3 + [c_int, c_int64, c_int, c_int, c_int] + [c_int64] * 3 + [c_int, c_void_p, c_void_p]),
    "sl_hamming_score_u8": (c_int, [c_void_p] * 3 + [c_int, c_int64, c_int, c_void_p]),
    "sl_topk_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int64]),
    "sl_topk_select": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_int, c_int, c_int,
                               c_void_p, c_void_p, c_size_t, c_void_p]),
    "sl_topk_select_static": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_int, c_int, c_int,
                                      c_void_p, c_void_p]),
    "sl_gather_kv": (c_int, [c_void_p] * 5 + [c_int] * 5 + [c_int64, c_void_p]),
    "sl_cache_append": (c_int, [c_void_p, c_void_p, c_int] + [c_int64] * 5 + [c_void_p, c_void_p]),
    "sl_lru_update": (c_int, [c_void_p] * 11 + [c_int] * 6 + [c_int64, c_int64, c_uint32, c_void_p, c_void_p]),
    "sl_attn_workspace_bytes": (c_size_t, [c_int] * 5),
    "sl_sparse_gqa_attn": (c_int, [c_void_p] * 5 + [c_int] * 6 + [c_int64] * 4 + [c_float, c_void_p, c_size_t, c_void_p]),
    "sl_decode_workspace_bytes": (c_size_t, [C.POINTER(DecodeParams)]),
    "sl_decode_error_offset": (c_size_t, [C.POINTER(DecodeParams)]),
    "sl_decode_head_major_fits": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int64, c_int, c_int]),
    "sl_decode_step": (c_int, [C.POINTER(DecodeParams), c_void_p]),
    "sl_decode_stages": (c_int, [C.POINTER(DecodeParams), c_int, c_void_p]),
    "sl_probe_launch": (c_int, [c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "sl_workspace_init": (c_int, [c_void_p, c_size_t, c_void_p]),
    "sl_phase_stamps": (c_int, [C.c_char_p, c_void_p, c_size_t, c_int]),
}

_lib = None


def load():
    """Load the shared library once and attach the C signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it first with `python -m spotlight_amd.build` "
            "(there is no fallback path)")
    import torch  # noqa: F401  -- makes torch's HIP runtime the one the library binds to
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class SpotlightHipError(RuntimeError):
    pass


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().sl_strerror(status).decode()
        raise SpotlightHipError(f"{what}: {msg} (status {status})")
