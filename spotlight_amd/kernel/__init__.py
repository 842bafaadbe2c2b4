"""Operator surface of the retrieval path, backed by libspotlight_hip.so.

The first block keeps the names, argument meaning and error behaviour of the
reference's ``spotlight/kernel/__init__.py`` (lines 1-40) so that code written
against it runs unchanged; the second block exposes the steps the reference
leaves to torch (top-k, gather, attention, hashing, cache/LRU updates).

All ops launch on torch's current stream and return tensors from torch's
allocator; none of them synchronises.  Importing this module without the
built library raises ImportError, as the reference does for its ``.so`` files
(``spotlight/kernel/__init__.py:7-11``).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from .. import _lib
from .._lib import SL_HEADMAP_BLOCKED, SL_HEADMAP_INTERLEAVED

try:
    _L = _lib.load()
except OSError as exc:  # pragma: no cover
    raise ImportError(f"cannot load {_lib.LIB_PATH}: {exc}") from exc

_DTYPES = {torch.float32: _lib.SL_F32, torch.bfloat16: _lib.SL_BF16, torch.float16: _lib.SL_F16}
_HEAD_MAPS = {"interleaved": SL_HEADMAP_INTERLEAVED, "blocked": SL_HEADMAP_BLOCKED}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dtype(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {t.dtype}: expected float32, bfloat16 or float16") from None


def _need_gpu(*ts: torch.Tensor) -> None:
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError("Input must be on the GPU")


def device_ptr(t: torch.Tensor) -> int:
    """Address a kernel may use for ``t``: its data pointer for a GPU tensor, the
    device-side address of the mapping for a PINNED host tensor (the host-memory
    tier; the kernels then read and write host memory in place).  Pageable host
    memory is refused."""
    if t.is_cuda:
        return t.data_ptr()
    if not t.is_pinned():
        raise RuntimeError("Input must be on the GPU or in pinned host memory")
    import ctypes
    dev = ctypes.c_void_p()
    _lib.check(_L.sl_host_device_pointer(t.data_ptr(), ctypes.byref(dev)), "sl_host_device_pointer")
    return dev.value


def _need_gpu_or_pinned(*ts: torch.Tensor) -> None:
    for t in ts:
        if not t.is_cuda and not t.is_pinned():
            raise RuntimeError("Input must be on the GPU or in pinned host memory")


class Workspace:
    """A zero-initialised scratch buffer the kernels leave zeroed again.
    One per concurrent caller; grown on demand."""

    def __init__(self):
        self.buf: Optional[torch.Tensor] = None

    def get(self, nbytes: int, device) -> torch.Tensor:
        if self.buf is None or self.buf.numel() < nbytes or self.buf.device != torch.device(device):
            with torch.cuda.device(device):
                self.buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
                _lib.check(_L.sl_workspace_init(self.buf.data_ptr(), self.buf.numel(), _stream()),
                           "sl_workspace_init")
        return self.buf


_default_ws = {}


def _ws(kind, nbytes: int, device) -> torch.Tensor:
    """Default workspace of one op and one shape family on one device (parts of a
    workspace must stay zero between calls, and where they lie depends on the shapes)."""
    key = (kind, torch.device(device))
    return _default_ws.setdefault(key, Workspace()).get(nbytes, device)


# ---------------------------------------------------------------------------
# reference-compatible ops  (spotlight/kernel/__init__.py)
# ---------------------------------------------------------------------------

def pack_cuda_func(x: torch.Tensor) -> torch.Tensor:
    """x[..., 32m] -> uint32[..., m], bit j of word w = (x[..., 32w+j] > 0).

    Same contract as ``packbits`` (spotlight/kernel/packbits.cu:28-63); also
    accepts float32 and float16, which the reference rejects."""
    _need_gpu(x)
    if x.shape[-1] % 32 != 0:
        raise RuntimeError("Last dimension must be divisible by 32")
    xc = x.contiguous()
    out = torch.empty((*x.shape[:-1], x.shape[-1] // 32), dtype=torch.uint32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_L.sl_pack_sign_u32(xc.data_ptr(), _dtype(xc), out.data_ptr(), out.numel(), _stream()),
                   "sl_pack_sign_u32")
    return out


def pack_dx_u32_func(x: torch.Tensor) -> torch.Tensor:
    """spotlight/kernel/pack_dx_u32.py:35-59 (asserts instead of raising)."""
    assert x.shape[-1] % 32 == 0, "suppose `last_dim % 32 == 0`"
    assert x.is_contiguous()
    return pack_cuda_func(x)


def pack_triton_func(x: torch.Tensor) -> torch.Tensor:
    return pack_dx_u32_func(x)


def pack_dx_u8_func(x: torch.Tensor) -> torch.Tensor:
    """x[..., 8m] -> uint8[..., m]  (spotlight/kernel/pack_dx_u8.py:34-56)."""
    _need_gpu(x)
    assert x.shape[-1] % 8 == 0, "suppose `last_dim % 8 == 0`"
    xc = x.contiguous()
    out = torch.empty((*x.shape[:-1], x.shape[-1] // 8), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_L.sl_pack_sign_u8(xc.data_ptr(), _dtype(xc), out.data_ptr(), out.numel(), _stream()),
                   "sl_pack_sign_u8")
    return out


def hamming_score(q_hash: torch.Tensor, k_hash: torch.Tensor, head_map: str = "interleaved",
                  seq_lens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q_hash u32[B,1,QH,W], k_hash u32[B,n,KH,W] -> int16[B,n,KH] matching bits
    summed over the G = QH/KH query heads of each kv head."""
    _need_gpu(q_hash, k_hash)
    if q_hash.dtype != torch.uint32 or k_hash.dtype != torch.uint32:
        raise RuntimeError("Inputs must be uint32")
    if q_hash.dim() != 4 or k_hash.dim() != 4:
        raise RuntimeError("Inputs must be 4D tensors")
    B, QN, QH, W = q_hash.shape
    Bk, n, KH, Wk = k_hash.shape
    if QN != 1:
        raise RuntimeError("Only support single query")
    if B != Bk or W != Wk or QH % KH != 0:
        raise RuntimeError("Head dimension mismatch")
    if k_hash.device != q_hash.device:
        raise RuntimeError("k_hash must be on the same device as q_hash")
    assert q_hash.is_contiguous()
    if not (k_hash.stride(3) == 1 and k_hash.stride(2) == W and k_hash.stride(1) == KH * W):
        raise AssertionError("k_hash rows must be contiguous [n, KH, W]")
    out = torch.zeros((B, n, KH), dtype=torch.int16, device=q_hash.device)
    with torch.cuda.device(q_hash.device):
        _lib.check(_L.sl_hamming_score(
            q_hash.data_ptr(), k_hash.data_ptr(), out.data_ptr(), B, n, KH, QH // KH, W,
            q_hash.stride(0), k_hash.stride(0), out.stride(0), _HEAD_MAPS[head_map],
            seq_lens.data_ptr() if seq_lens is not None else None, _stream()), "sl_hamming_score")
    return out


def attn_dx_u32_func(q_hash: torch.Tensor, k_hash: torch.Tensor) -> torch.Tensor:
    """spotlight/kernel/attn_dx_u32.py:131-161 (interleaved head mapping)."""
    assert q_hash.shape[1] == 1, "only support single query"
    assert q_hash.shape[2] % k_hash.shape[2] == 0, "query head must be multiple of key head"
    assert q_hash.is_contiguous()
    assert k_hash.is_contiguous()
    return hamming_score(q_hash, k_hash, "interleaved")


def attn_triton_func(q_hash, k_hash):
    return attn_dx_u32_func(q_hash, k_hash)


def attn_cuda_func(q_hash, k_hash):
    """spotlight/kernel/__init__.py:31-40.  The reference only ships the
    (KH, QH) = (4, 28), W = 4 instance; here any QH = G*KH with KH dividing
    256 and W in {1, 2, 4, 8} runs."""
    return hamming_score(q_hash, k_hash, "interleaved")


def attn_dx_u8_func(q_hash: torch.Tensor, k_hash: torch.Tensor) -> torch.Tensor:
    """q u8[B,H,1,D], k u8[B,H,n,D] -> u8[B,H,n]  (spotlight/kernel/attn_dx_u8.py:46-74)."""
    _need_gpu(q_hash, k_hash)
    batch_size, num_heads, q_len, dim = q_hash.shape
    k_len = k_hash.shape[2]
    assert q_len == 1, "only support single query"
    q = q_hash.reshape(-1, dim).contiguous()
    k = k_hash.reshape(-1, k_len, dim).contiguous()
    out = torch.zeros((q.shape[0], k_len), dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        _lib.check(_L.sl_hamming_score_u8(q.data_ptr(), k.data_ptr(), out.data_ptr(), q.shape[0], k_len, dim,
                                          _stream()), "sl_hamming_score_u8")
    return out.view(batch_size, num_heads, k_len)


# ---------------------------------------------------------------------------
# the steps the reference leaves to torch
# ---------------------------------------------------------------------------

def topk_select(score: torch.Tensor, k: int, max_score: int,
                seq_lens: Optional[torch.Tensor] = None, layout: str = "bnh") -> torch.Tensor:
    """Indices of the k largest scores per (b, kv head); ties go to the lower
    token index; each row comes out in ascending token order.

    score int16 [B,n,KH] (layout 'bnh', what the scorer returns) or [B,KH,n]
    ('bhn'), 0 <= score <= max_score.  Returns int32 [B,KH,k]; when fewer than
    k tokens exist the tail is -1.  Replaces ``attn.topk(k, dim=1,
    sorted=False).indices`` (spotlight/modifiers/gpu_cache.py:50)."""
    _need_gpu(score)
    if score.dtype != torch.int16 or score.dim() != 3:
        raise RuntimeError("score must be a 3-D int16 tensor")
    if layout == "bnh":
        B, n, KH = score.shape
        sb, sn, sh = score.stride()
    elif layout == "bhn":
        B, KH, n = score.shape
        sb, sh, sn = score.stride()
    else:
        raise ValueError(layout)
    idx = torch.empty((B, KH, k), dtype=torch.int32, device=score.device)
    with torch.cuda.device(score.device):
        nbytes = _L.sl_topk_workspace_bytes(B, KH, max_score, n)
        ws = _ws(("topk", B, KH, max_score), nbytes, score.device)
        _lib.check(_L.sl_topk_select(
            score.data_ptr(), sb, sn, sh, idx.data_ptr(), B, n, KH, k, max_score,
            seq_lens.data_ptr() if seq_lens is not None else None, ws.data_ptr(), ws.numel(), _stream()),
            "sl_topk_select")
    return idx


def gather_kv(keys: torch.Tensor, vals: torch.Tensor, idx: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """keys/vals [B,L,KH,d] (rows contiguous), idx int32 [B,KH,k] ->
    (K_sel, V_sel) [B,k,KH,d]; the two torch.gather calls of
    spotlight/modifiers/gpu_cache.py:51-53."""
    _need_gpu(idx)
    _need_gpu_or_pinned(keys, vals)      # a pinned host store is gathered from in place
    B, L, KH, d = keys.shape
    k = idx.shape[2]
    assert keys.shape == vals.shape and keys.stride() == vals.stride()
    assert keys.stride(3) == 1 and keys.stride(2) == d and keys.stride(1) == KH * d
    assert idx.dtype == torch.int32 and idx.is_contiguous()
    k_out = torch.empty((B, k, KH, d), dtype=keys.dtype, device=idx.device)
    v_out = torch.empty_like(k_out)
    with torch.cuda.device(idx.device):
        _lib.check(_L.sl_gather_kv(device_ptr(keys), device_ptr(vals), idx.data_ptr(), k_out.data_ptr(),
                                   v_out.data_ptr(), _dtype(keys), B, KH, d, k, keys.stride(0), _stream()),
                   "sl_gather_kv")
    return k_out, v_out


def sparse_gqa_attn(q: torch.Tensor, keys: torch.Tensor, vals: torch.Tensor, idx: torch.Tensor,
                    layout: str = "bnhd", scale: Optional[float] = None) -> torch.Tensor:
    """softmax(q K_sel^T * scale) V_sel over the rows idx selects, without
    materialising K_sel / V_sel.

    q [B,QH,d]; keys/vals [B,L,KH,d] ('bnhd', the cache layout of
    spotlight/modifiers/gpu_cache.py:27-36) or [B,KH,L,d] ('bhnd'); idx int32
    [B,KH,k], negative entries skipped.  kv head of q head qh is qh // G.
    Returns [B,QH,d] in q's dtype."""
    _need_gpu(q, keys, vals, idx)
    B, QH, d = q.shape
    if layout == "bnhd":
        _, L, KH, _ = keys.shape
        sb, sn, sh, sd = keys.stride()
    elif layout == "bhnd":
        _, KH, L, _ = keys.shape
        sb, sh, sn, sd = keys.stride()
    else:
        raise ValueError(layout)
    assert sd == 1 and keys.stride() == vals.stride() and keys.dtype == q.dtype == vals.dtype
    assert idx.dtype == torch.int32 and idx.is_contiguous() and idx.shape[:2] == (B, KH)
    assert q.stride(2) == 1 and q.stride(1) == d
    k = idx.shape[2]
    out = torch.empty((B, QH, d), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        nbytes = _L.sl_attn_workspace_bytes(B, QH, KH, d, k)
        ws = _ws("attn", nbytes, q.device)
        _lib.check(_L.sl_sparse_gqa_attn(
            q.data_ptr(), keys.data_ptr(), vals.data_ptr(), idx.data_ptr(), out.data_ptr(), _dtype(q),
            B, QH, KH, d, k, q.stride(0), sb, sn, sh, float(scale) if scale else 0.0,
            ws.data_ptr(), ws.numel(), _stream()), "sl_sparse_gqa_attn")
    return out


def hash_mlp_pack(x: torch.Tensor, w1: torch.Tensor, b1: Optional[torch.Tensor],
                  w2: Optional[torch.Tensor] = None, b2: Optional[torch.Tensor] = None,
                  residue: bool = False) -> torch.Tensor:
    """Fused per-head hash -> sign -> pack for one new vector per (b, head).

    x [B,H,d_in]; w1 [H,d_in,d_hid]; b1 [H,d_hid]|None; w2 [H,d_hid,nbits]|None;
    b2 [H,nbits]|None.  With w2: codes of silu(x@w1+b1)(+x) @ w2 + b2 (+h)
    (spotlight_generation.py:229-255); without: codes of x@w1 (+b1)
    (linearhashing_generation.py:224-231).  Returns uint32 [B,H,nbits/32]."""
    _need_gpu(x, w1)
    B, H, d_in = x.shape
    d_hid = w1.shape[2]
    n_layers = 2 if w2 is not None else 1
    nbits = w2.shape[2] if w2 is not None else d_hid
    xc = x.contiguous()
    for t in (w1, b1, w2, b2):
        assert t is None or (t.is_contiguous() and t.dtype == x.dtype)
    codes = torch.empty((B, H, nbits // 32), dtype=torch.uint32, device=x.device)
    ptr = lambda t: t.data_ptr() if t is not None else None
    with torch.cuda.device(x.device):
        _lib.check(_L.sl_hash_mlp_pack(
            xc.data_ptr(), w1.data_ptr(), ptr(b1), ptr(w2), ptr(b2), codes.data_ptr(), _dtype(x), n_layers,
            B, H, d_in, d_hid, nbits, int(residue), xc.stride(0), codes.stride(0), codes.stride(1), 0, None,
            _stream()), "sl_hash_mlp_pack")
    return codes


def hash_rows_pack(x: torch.Tensor, w1: torch.Tensor, b1: Optional[torch.Tensor],
                   w2: Optional[torch.Tensor] = None, b2: Optional[torch.Tensor] = None,
                   residue: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same hash for many rows per head: x [B,n,H,d_in] -> uint32 [B,n,H,nbits/32] (or into
    ``out``, any tensor of that shape whose last dimension is contiguous, e.g. a slice of a cache).
    Bit-identical to ``hash_mlp_pack`` row by row: both sum the projections in one order."""
    _need_gpu(x, w1)
    B, n, H, d_in = x.shape
    d_hid = w1.shape[2]
    n_layers = 2 if w2 is not None else 1
    nbits = w2.shape[2] if w2 is not None else d_hid
    assert x.stride(3) == 1 and x.stride(2) == d_in, "rows of a head must be contiguous, heads adjacent"
    for t in (w1, b1, w2, b2):
        assert t is None or (t.is_contiguous() and t.dtype == x.dtype)
    if out is None:
        out = torch.empty((B, n, H, nbits // 32), dtype=torch.uint32, device=x.device)
    assert out.shape == (B, n, H, nbits // 32) and out.dtype == torch.uint32 and out.stride(3) == 1
    ptr = lambda t: t.data_ptr() if t is not None else None
    with torch.cuda.device(x.device):
        _lib.check(_L.sl_hash_rows_pack(
            x.data_ptr(), w1.data_ptr(), ptr(b1), ptr(w2), ptr(b2), out.data_ptr(), _dtype(x), n_layers,
            B, n, H, d_in, d_hid, nbits, int(residue), x.stride(0), x.stride(1),
            out.stride(0), out.stride(1), out.stride(2), _stream()), "sl_hash_rows_pack")
    return out


def cache_append(dst: torch.Tensor, src: torch.Tensor, start: int = 0,
                 seq_lens: Optional[torch.Tensor] = None) -> None:
    """dst[b, start + seq_lens[b] : ... + t] = src[b]  for dst [B,L,...] and
    src [B,t,...] with contiguous rows (gpu_cache.py:42,112-113)."""
    _need_gpu(src)
    _need_gpu_or_pinned(dst)             # a pinned host store is appended to in place
    B, t = src.shape[0], src.shape[1]
    row_bytes = src[0, 0].numel() * src.element_size()
    assert dst.dtype == src.dtype and dst[0, 0].numel() == src[0, 0].numel()
    assert src[0].is_contiguous() and dst[0].is_contiguous()
    if seq_lens is None and start + t > dst.shape[1]:
        raise RuntimeError("append exceeds the cache capacity")
    with torch.cuda.device(src.device):
        _lib.check(_L.sl_cache_append(
            src.data_ptr(), device_ptr(dst), B, t, row_bytes, src.stride(0) * src.element_size(),
            dst.stride(0) * dst.element_size(), start,
            seq_lens.data_ptr() if seq_lens is not None else None, _stream()), "sl_cache_append")


def num_remain(n: int, mask_out: float, min_remain: int = 20) -> int:
    """Tokens kept out of n (spotlight_generation.py:162-164)."""
    return max(min(n, min_remain), n - int(n * mask_out))
