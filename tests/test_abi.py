"""The C ABI: the library loads, exports every symbol include/spotlight_hip.h
declares, the Python binding covers them all, and argument validation answers
with the documented status codes before anything touches a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "spotlight_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sl_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from spotlight_amd import _lib
    return _lib.load()


def test_header_declares_the_expected_surface():
    syms = declared_symbols()
    for name in ("sl_pack_sign_u32", "sl_pack_sign_u8", "sl_hash_mlp_pack", "sl_hamming_score", "sl_hamming_score_u8",
                 "sl_topk_select", "sl_gather_kv", "sl_cache_append", "sl_lru_update", "sl_sparse_gqa_attn",
                 "sl_decode_step", "sl_decode_stages", "sl_workspace_init", "sl_strerror"):
        assert name in syms


def test_library_exports_every_declared_symbol(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"


def test_binding_covers_every_declared_symbol():
    from spotlight_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_decode_params_struct_matches_header():
    from spotlight_amd import _lib
    text = open(HEADER).read()
    body = text[text.index("typedef struct {"):text.index("} sl_decode_params;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.replace("typedef struct {", "").strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.findall(r"([A-Za-z_0-9]+)\s*$", part.strip())[0])
    assert names == [f[0] for f in _lib.DecodeParams._fields_]


def test_status_strings(lib):
    assert lib.sl_strerror(0) == b"ok"
    for code in range(-6, 0):
        assert lib.sl_strerror(code) not in (b"ok", b"unknown status")
    assert lib.sl_strerror(-99) == b"unknown status"
    assert lib.sl_version() >= 100


def test_argument_validation_needs_no_gpu(lib):
    # every call below is rejected (or is a no-op) before any kernel launch
    assert lib.sl_pack_sign_u32(None, 0, None, -1, None) == -2           # shape
    assert lib.sl_pack_sign_u32(None, 0, None, 0, None) == 0             # nothing to do
    assert lib.sl_pack_sign_u32(None, 0, None, 4, None) == -1            # null
    assert lib.sl_pack_sign_u32(8, 0, 16, 4, None) == -4                 # misaligned input
    assert lib.sl_pack_sign_u32(16, 7, 16, 4, None) == -3                # unknown dtype
    assert lib.sl_hamming_score(16, 16, 16, 1, 10, 3, 4, 4, 0, 0, 0, 0, None, None) == -3   # 256 % KH != 0
    assert lib.sl_hamming_score(16, 16, 16, 1, 10, 8, 4, 3, 0, 0, 0, 0, None, None) == -3   # W not in {1,2,4,8}
    assert lib.sl_hamming_score(16, 16, 16, 1, 10, 8, 4, 4, 0, 0, 0, 5, None, None) == -3   # head map
    assert lib.sl_hamming_score_u8(16, 16, 16, 2, 10, 5, None) == -3
    assert lib.sl_topk_select(16, 1, 1, 1, 16, 1, 10, 2, 3, 5000, None, 16, 1 << 30, None) == -3   # too many bins
    assert lib.sl_topk_select(16, 1, 1, 1, 16, 1, 10, 2, 3, 128, None, 16, 8, None) == -5          # workspace too small
    assert lib.sl_sparse_gqa_attn(16, 16, 16, 16, 16, 1, 1, 32, 8, 64, 10, 0, 0, 0, 0, 0.0, None, 0, None) == -3  # d != 128
    assert lib.sl_sparse_gqa_attn(16, 16, 16, 16, 16, 1, 1, 30, 8, 128, 10, 0, 0, 0, 0, 0.0, None, 0, None) == -2  # QH % KH
    assert lib.sl_hash_mlp_pack(16, 16, None, 16, None, 16, 1, 2, 1, 4, 64, 256, 128, 0, 64, 16, 4, 0, None, None) == -3  # d_in
    assert lib.sl_hash_mlp_pack(16, 16, None, 16, None, 16, 1, 2, 1, 4, 128, 200, 128, 0, 128, 16, 4, 0, None, None) == -3  # d_hid
    assert lib.sl_cache_append(16, 16, 1, 1, 24, 0, 0, 0, None, None) == -4      # row bytes not a multiple of 16
    assert lib.sl_lru_update(*([16] * 11), 1, 1, 8, 128, 20, 16, 100, 0, 1, None, None) == -3   # k + 1 > C
    assert lib.sl_decode_step(None, None) == -1
    assert lib.sl_workspace_init(None, 0, None) == 0
    assert lib.sl_tune(b"no_such_key", 1) == -3


def test_workspace_sizes(lib):
    assert lib.sl_attn_workspace_bytes(1, 32, 8, 128, 655) >= 64 * 1024
    assert lib.sl_attn_workspace_bytes(1, 32, 8, 64, 655) == 0
    small = lib.sl_topk_workspace_bytes(1, 8, 512, 1000)
    big = lib.sl_topk_workspace_bytes(1, 8, 512, 100000)
    assert 0 < small < big


def test_host_budget_formula():
    from spotlight_amd import kernel as K
    # spotlight_generation.py:162-164
    for n, mask_out, k in [(4096, 0.9, 410), (16384, 0.98, 328), (32768, 0.98, 656), (131072, 0.98, 2622), (7, 0.98, 7)]:
        assert K.num_remain(n, mask_out) == k


def test_product_library_carries_no_phase_stamps(lib):
    """sl_phase_stamps only answers in the measurement build (-DSL_PHASE_STAMPS); the product library says
    SL_ERR_UNSUPPORTED without touching its arguments' memory or a GPU."""
    buf = (C.c_ulonglong * 4)()
    assert lib.sl_phase_stamps(b"fused", buf, 4, 0) == -3
    assert lib.sl_phase_stamps(None, None, 0, 0) == -3
