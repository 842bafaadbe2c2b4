"""Per-layer decode state driving the fused HIP decode step.

One ``LayerDecodeState`` owns what one attention layer needs between decode
steps: packed key codes, K and V (token-major ``[B, n_cap, KH, .]`` like the
reference's ``KVHash`` / ``KVCache`` buffers, spotlight/modifiers/gpu_cache.py:
27-36,77-95), the per-sequence lengths on the device, the hash weights of both
sides and the scratch workspace.  ``step`` is the kernel-path composition of
the reference's decode branch (spotlight/modifiers/spotlight_generation.py:
143-215): hash -> pack -> score -> top-k -> (LRU) -> sparse attention.

All lengths live on the device, so a captured HIP graph of ``step`` can be
replayed while the cache grows (``capture`` / ``replay``).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from . import kernel as K

_L = _lib.load()


class PeerWaitError(RuntimeError):
    """A workgroup of the one-launch scorer + tail gave up waiting for the other blocks of its
    (b, kv head): the indices and the attention output of that step are invalid."""


@dataclass
class HashWeights:
    """Per-head hash weights of one side (query or key).

    Two layers: ``w1 [H,d,d_hid]``, ``b1 [H,d_hid]``, ``w2 [H,d_hid,nbits]``,
    ``b2 [H,nbits]`` -- the ``proj`` / ``bias`` of MLPLayer squeezed of their
    unit dimensions (spotlight_generation.py:232-234).  One layer (linear
    hashing, linearhashing_generation.py:227): ``w1 [H,d,nbits]`` only."""
    w1: torch.Tensor
    b1: Optional[torch.Tensor] = None
    w2: Optional[torch.Tensor] = None
    b2: Optional[torch.Tensor] = None
    residue: bool = False

    @property
    def n_layers(self) -> int:
        return 2 if self.w2 is not None else 1

    @property
    def d_hid(self) -> int:
        return self.w1.shape[2]

    @property
    def nbits(self) -> int:
        return self.w2.shape[2] if self.w2 is not None else self.w1.shape[2]

    @staticmethod
    def random_mlp(H, dims, dtype, device, generator=None, scale=0.001, residue=False):
        """The reference's init: proj ~ N(0,1)*0.001, bias = 0 (spotlight_generation.py:232-234)."""
        assert len(dims) == 3
        w = [(torch.randn(H, dims[i], dims[i + 1], generator=generator) * scale).to(dtype).to(device)
             for i in range(2)]
        b = [torch.zeros(H, dims[i + 1], dtype=dtype, device=device) for i in range(2)]
        return HashWeights(w[0], b[0], w[1], b[1], residue)

    @staticmethod
    def random_linear(H, d, nbits, dtype, device, generator=None):
        """Gaussian projection, not orthogonalised (linearhashing_generation.py:227)."""
        return HashWeights(torch.randn(H, d, nbits, generator=generator).to(dtype).to(device))

    def hash_rows(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Codes of many rows per head (prefill): x [B,n,H,d] -> uint32 [B,n,H,nbits/32].

        The HIP kernel for many rows; it sums exactly as the decode step's hash does, so a key
        gets the same code whether it arrives with the prompt or as a decoded token."""
        return K.hash_rows_pack(x, self.w1, self.b1, self.w2, self.b2, self.residue, out=out)


class LayerDecodeState:
    def __init__(self, batch_size: int, num_heads: int, num_kv_heads: int, head_dim: int, n_cap: int, k: int,
                 hash_q: HashWeights, hash_k: HashWeights, dtype=torch.bfloat16, device="cuda",
                 head_map: str = "blocked", lru_slots: int = 0, inputs=None, host_store: bool = False,
                 rope_theta: Optional[float] = None, rope_inv_freq: Optional[torch.Tensor] = None,
                 codes_layout: str = "auto", exclusive_device: bool = True):
        assert head_dim == 128, "the attention kernel covers head_dim 128"
        assert n_cap % 8 == 0, "n_cap must be a multiple of 8"
        assert hash_q.nbits == hash_k.nbits and hash_q.n_layers == hash_k.n_layers
        assert hash_q.d_hid == hash_k.d_hid and hash_q.residue == hash_k.residue
        self.B, self.QH, self.KH, self.d = batch_size, num_heads, num_kv_heads, head_dim
        self.n_cap, self.k, self.dtype, self.device = n_cap, k, dtype, torch.device(device)
        self.nbits = hash_q.nbits
        self.W = self.nbits // 32
        self.hash_q, self.hash_k = hash_q, hash_k
        self.head_map = head_map
        dev = self.device
        B, QH, KH, d, W = self.B, self.QH, self.KH, self.d, self.W
        # Key codes: token-major [B, n_cap, KH, W] (the reference's layout, attn_k4_q28.cu:55) for the
        # three-launch step, or head-major [B, KH, n_cap, W] for the step whose scorer, selection and
        # attention are ONE launch (a workgroup then owns 4096 or 8192 contiguous rows of one kv head;
        # with an LRU table the launch ends at the selection).  "auto"
        # takes head-major whenever that launch covers the shape.  ``codes`` is always indexed
        # [b, row, kv head, word]; with head-major storage it is a strided view.
        # The head-major step's workgroups wait for each other (bounded), which assumes that this launch
        # has the device to itself: a caller whose other streams keep kernels running at the same time
        # says so with exclusive_device=False and gets token-major codes, whose kernels never wait.
        if codes_layout == "auto" and not exclusive_device:
            codes_layout = "token"
        if codes_layout == "auto":
            # without an LRU table the launch also attends, one run per block of rows (up to 16 blocks per head,
            # 32 beyond 64k rows): keep <= 128 rows per block on average
            most_blocks = min(32 if n_cap > 65536 else 16, (n_cap + 511) // 512)
            rows_ok = bool(lru_slots) or k <= 128 * most_blocks
            fits = 0
            if rows_ok and W == 4:
                # all blocks of a launch must be resident at once; the library knows what the device holds
                with torch.cuda.device(dev):
                    fits = _lib.load().sl_decode_head_major_fits(K._DTYPES[self.dtype], B, QH, KH, self.nbits, n_cap, k,
                                                                 int(bool(lru_slots)))
            codes_layout = "head" if fits > 0 else "token"
        assert codes_layout in ("token", "head")
        self.codes_layout = codes_layout
        if codes_layout == "head":
            self._codes = torch.zeros((B, KH, n_cap, W), dtype=torch.uint32, device=dev)
            self.codes = self._codes.permute(0, 2, 1, 3)
        else:
            self._codes = torch.zeros((B, n_cap, KH, W), dtype=torch.uint32, device=dev)
            self.codes = self._codes
        # host_store: the full K / V store lives in pinned host memory, which the step's
        # kernels append to and fetch missed rows from in place; the GPU then only
        # holds the codes and the LRU resident table the attention reads
        self.host_store = host_store
        if host_store:
            assert lru_slots, "a host-memory store needs the LRU resident table in front of it"
            self.keys = torch.zeros((B, n_cap, KH, d), dtype=dtype, pin_memory=True)
            self.vals = torch.zeros((B, n_cap, KH, d), dtype=dtype, pin_memory=True)
        else:
            self.keys = torch.zeros((B, n_cap, KH, d), dtype=dtype, device=dev)
            self.vals = torch.zeros((B, n_cap, KH, d), dtype=dtype, device=dev)
        self.seq_lens = torch.zeros((B,), dtype=torch.int32, device=dev)
        self.step_counter = torch.zeros((1,), dtype=torch.int32, device=dev)
        if inputs is None:  # the step's inputs are read from these buffers
            inputs = (torch.zeros((B, QH, d), dtype=dtype, device=dev),
                      torch.zeros((B, KH, d), dtype=dtype, device=dev),
                      torch.zeros((B, KH, d), dtype=dtype, device=dev))
        self.q_in, self.k_in, self.v_in = inputs
        assert self.q_in.shape == (B, QH, d) and self.k_in.shape == (B, KH, d) and self.v_in.shape == (B, KH, d)
        assert all(t.is_contiguous() and t.dtype == dtype for t in inputs)
        self.out = torch.zeros((B, QH, d), dtype=dtype, device=dev)
        # rotary embedding inside the step: q and k_new are handed over UN-rotated and the hash launch
        # rotates them at position seq_lens[b] (the reference re-rotates the whole cache every step,
        # spotlight_generation.py:139-141; here a key is rotated once, when it is appended)
        if rope_inv_freq is None and rope_theta is not None:
            rope_inv_freq = 1.0 / (rope_theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        self.rope_inv_freq = None
        if rope_inv_freq is not None:
            self.rope_inv_freq = rope_inv_freq.to(device=dev, dtype=torch.float32).contiguous()
            assert self.rope_inv_freq.shape == (d // 2,)
            self.q_rot = torch.zeros((B, QH, d), dtype=dtype, device=dev)
        self.idx = torch.full((B, KH, k), -1, dtype=torch.int32, device=dev)
        self.host_len = 0  # upper bound of seq_lens, tracked on the host for grid sizing
        self.lru_slots = lru_slots
        if lru_slots:
            assert k + 1 <= lru_slots <= 4096
            self.slot_token = torch.full((B, KH, lru_slots), -1, dtype=torch.int32, device=dev)
            self.slot_stamp = torch.zeros((B, KH, lru_slots), dtype=torch.int32, device=dev)
            self.token_slot = torch.full((B, KH, n_cap), -1, dtype=torch.int32, device=dev)
            self.k_res = torch.zeros((B, KH, lru_slots, d), dtype=dtype, device=dev)
            self.v_res = torch.zeros((B, KH, lru_slots, d), dtype=dtype, device=dev)
            self.slots_out = torch.full((B, KH, k), -1, dtype=torch.int32, device=dev)
            self.lru_stats = torch.zeros((B, KH, 2), dtype=torch.int32, device=dev)
        self.params = self._make_params()
        nbytes = _L.sl_decode_workspace_bytes(C.byref(self.params))
        assert nbytes > 0
        self.ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            _lib.check(_L.sl_workspace_init(self.ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream),
                       "sl_workspace_init")
        self.params.ws = self.ws.data_ptr()
        self.params.ws_bytes = nbytes
        self._graph = None

    def _make_params(self) -> _lib.DecodeParams:
        p = _lib.DecodeParams()
        p.dtype = K._DTYPES[self.dtype]
        p.B, p.QH, p.KH, p.d = self.B, self.QH, self.KH, self.d
        p.nbits, p.k = self.nbits, self.k
        p.head_map = K._HEAD_MAPS[self.head_map]
        p.n_cap, p.n_max = self.n_cap, 1
        p.q, p.k_new, p.v_new = self.q_in.data_ptr(), self.k_in.data_ptr(), self.v_in.data_ptr()
        if self.rope_inv_freq is not None:
            p.rope_inv_freq, p.q_rot = self.rope_inv_freq.data_ptr(), self.q_rot.data_ptr()
        hq, hk = self.hash_q, self.hash_k
        p.n_layers, p.d_hid, p.residue = hq.n_layers, hq.d_hid, int(hq.residue)
        ptr = lambda t: t.data_ptr() if t is not None else None
        p.w1_q, p.b1_q, p.w2_q, p.b2_q = ptr(hq.w1), ptr(hq.b1), ptr(hq.w2), ptr(hq.b2)
        p.w1_k, p.b1_k, p.w2_k, p.b2_k = ptr(hk.w1), ptr(hk.b1), ptr(hk.w2), ptr(hk.b2)
        p.codes_head_major = int(self.codes_layout == "head")
        p.codes, p.keys, p.vals = self._codes.data_ptr(), K.device_ptr(self.keys), K.device_ptr(self.vals)
        p.seq_lens, p.out, p.idx = self.seq_lens.data_ptr(), self.out.data_ptr(), self.idx.data_ptr()
        p.step_counter = self.step_counter.data_ptr()
        p.lru_C = self.lru_slots
        if self.lru_slots:
            p.lru_map_cap = self.n_cap
            p.slot_token, p.slot_stamp = self.slot_token.data_ptr(), self.slot_stamp.data_ptr()
            p.token_slot = self.token_slot.data_ptr()
            p.k_res, p.v_res = self.k_res.data_ptr(), self.v_res.data_ptr()
            p.slots_out, p.lru_stats = self.slots_out.data_ptr(), self.lru_stats.data_ptr()
        return p

    # -- prefill ---------------------------------------------------------------
    def prefill(self, keys: torch.Tensor, vals: torch.Tensor, codes: Optional[torch.Tensor] = None) -> None:
        """Store n0 post-RoPE rows per sequence: keys/vals [B,n0,KH,d]; codes
        [B,n0,KH,W] are hashed from the keys when not given."""
        n0 = keys.shape[1]
        assert self.host_len == 0 and n0 < self.n_cap
        self.load_rows(keys, vals, 0, codes)
        self.seq_lens.fill_(n0)
        self.host_len = n0

    def load_rows(self, keys: torch.Tensor, vals: torch.Tensor, start: int,
                  codes: Optional[torch.Tensor] = None) -> None:
        """Prefill in slabs: rows [start, start + t) of every sequence; lengths are set
        afterwards with ``set_length``.  Bounds the transient memory of hashing."""
        t = keys.shape[1]
        assert start + t < self.n_cap
        K.cache_append(self.keys, keys.contiguous(), start=start)
        K.cache_append(self.vals, vals.contiguous(), start=start)
        dst = self.codes[:, start:start + t]
        if codes is None:
            self.hash_k.hash_rows(keys.contiguous(), out=dst)      # hashed straight into the cache, whatever its layout
        else:
            dst.view(torch.int32).copy_(codes.view(torch.int32))

    def set_length(self, n: int) -> None:
        assert 0 <= n < self.n_cap
        self.seq_lens.fill_(n)
        self.host_len = n
        self._graph = None

    # -- decode ------------------------------------------------------------------
    def _launch(self, n_max: int, stages: int = _lib.STAGE_ALL) -> None:
        if n_max > self.n_cap:
            raise RuntimeError(f"cache capacity {self.n_cap} exceeded")
        self.params.n_max = n_max
        _lib.check(_L.sl_decode_stages(C.byref(self.params), stages, torch.cuda.current_stream().cuda_stream),
                   "sl_decode_stages")

    def launch_stages(self, stages: int) -> None:
        """Enqueue a subset of the step's kernels on the current inputs (profiling
        aid; lengths do not advance).  After SCORE without SELECT call
        ``reset_workspace`` before the next real step."""
        with torch.cuda.device(self.device):
            self._launch(self.host_len + 1, stages)

    def reset_workspace(self) -> None:
        with torch.cuda.device(self.device):
            _lib.check(_L.sl_workspace_init(self.ws.data_ptr(), self.ws.numel(),
                                            torch.cuda.current_stream().cuda_stream), "sl_workspace_init")

    def error_word(self) -> Optional[torch.Tensor]:
        """The device word (int32, shape [1]) a workgroup of the one-launch scorer + tail sets when it
        gives up waiting for its peers; None with token-major codes, whose kernels never wait."""
        off = _L.sl_decode_error_offset(C.byref(self.params))
        if off == C.c_size_t(-1).value:
            return None
        return self.ws[off:off + 4].view(torch.int32)

    def peer_wait_failed(self) -> bool:
        """True if a workgroup of the one-launch scorer + tail ever gave up waiting for its peers (one
        device read; always False with token-major codes)."""
        w = self.error_word()
        return False if w is None else bool(w.item())

    def check_peer_wait(self, fallback: bool = True) -> None:
        """Raises PeerWaitError if a bounded wait ran out since the last check (one device read, so
        call it where the host synchronises anyway).  The word is cleared, and with ``fallback`` the
        state moves to token-major codes first -- whose kernels never wait for each other -- so the
        steps after the failed one are right whatever else keeps the device busy."""
        if not self.peer_wait_failed():
            return
        self.error_word().zero_()
        if fallback:
            self.use_token_major()
        raise PeerWaitError(
            "a workgroup gave up waiting for the other blocks of its (batch entry, kv head): the last step's "
            "indices and output are invalid (the device was probably shared with another stream's kernels)"
            + ("; the state now uses token-major codes" if fallback else ""))

    def use_token_major(self) -> None:
        """Re-lay the key codes token-major and rebuild parameters and workspace for the three-launch
        step.  Lengths, K/V, LRU table and the current budget are kept; a captured graph is dropped."""
        if self.codes_layout == "token":
            return
        with torch.cuda.device(self.device):
            torch.cuda.synchronize()
            k_now, old = self.params.k, self.params
            self._codes = self.codes.view(torch.int32).contiguous().view(torch.uint32)
            self.codes = self._codes
            self.codes_layout = "token"
            self.params = self._make_params()
            self.params.k = k_now
            self.params.budget_on, self.params.budget_min_remain = old.budget_on, old.budget_min_remain
            self.params.budget_mask_out = old.budget_mask_out
            nbytes = _L.sl_decode_workspace_bytes(C.byref(self.params))
            self.ws = torch.empty((nbytes,), dtype=torch.uint8, device=self.device)
            _lib.check(_L.sl_workspace_init(self.ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream),
                       "sl_workspace_init")
            self.params.ws, self.params.ws_bytes = self.ws.data_ptr(), nbytes
            self._graph = None

    def set_k(self, k: int) -> None:
        """Tokens kept per (b, kv head) from the next step on (at most the k given at
        construction, which sized the index buffers; rows of ``idx`` become k long).
        The reference recomputes its budget from the cache length every step
        (spotlight_generation.py:162-164)."""
        if not 1 <= k <= self.k:
            raise ValueError(f"k must be in [1, {self.k}]")
        if self.lru_slots and k + 1 > self.lru_slots:
            raise ValueError("k + 1 must not exceed the LRU slots")
        self.params.k = k
        self._graph = None

    def set_budget(self, mask_out: Optional[float], min_remain: int = 0) -> None:
        """Let the DEVICE evaluate the reference's budget rule every step
        (spotlight_generation.py:162-164): a sequence that holds n rows after the append keeps
        max(min(n, min_remain), n - int(n * mask_out)) of them, capped at ``current_k`` (the row
        length of ``idx``; entries beyond the budget are -1).  Nothing on the host changes when the
        budget does, so one captured graph serves a growing cache.  ``None`` switches the rule off."""
        p = self.params
        if mask_out is None:
            p.budget_on = 0
        else:
            if not 0.0 <= mask_out <= 1.0 or min_remain < 0:
                raise ValueError("mask_out must be in [0, 1] and min_remain >= 0")
            p.budget_on, p.budget_min_remain, p.budget_mask_out = 1, int(min_remain), float(mask_out)
        self._graph = None

    @property
    def current_k(self) -> int:
        return self.params.k

    def selected(self) -> torch.Tensor:
        """int32 [B, KH, current_k]: the tokens the last step attended to, ascending; -1 beyond the
        rows a sequence has, or beyond its budget.  Reads the device, so it also checks that no
        bounded wait ran out (PeerWaitError)."""
        self.check_peer_wait()
        k = self.params.k
        return self.idx.view(-1)[: self.B * self.KH * k].view(self.B, self.KH, k)

    def step(self, q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, check: bool = False) -> torch.Tensor:
        """One decode step: q [B,QH,d], k_new/v_new [B,KH,d] (post-RoPE, or un-rotated when the
        state was built with ``rope_theta`` / ``rope_inv_freq``).
        Returns the attention output [B,QH,d] (a buffer reused by the next step).  ``check``
        synchronises and raises PeerWaitError if a bounded wait of this step ran out (debugging aid;
        ``Spotlight.generate`` and ``selected`` check where they read the device anyway)."""
        with torch.cuda.device(self.device):
            if q is not self.q_in:
                self.q_in.copy_(q)
            if k_new is not self.k_in:
                self.k_in.copy_(k_new)
            if v_new is not self.v_in:
                self.v_in.copy_(v_new)
            self._launch(self.host_len + 1)
        self.host_len += 1
        if check:
            self.check_peer_wait()
        return self.out

    def capture(self, steps_ahead: int) -> None:
        """Capture one step as a HIP graph valid for the next ``steps_ahead``
        replays (grids are sized for the longest length in that window).
        Inputs are read from ``q_in`` / ``k_in`` / ``v_in``."""
        n_max = min(self.host_len + steps_ahead, self.n_cap)
        self._graph_budget = n_max - self.host_len
        with torch.cuda.device(self.device):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._launch(n_max)
        self._graph = g

    def replay(self) -> torch.Tensor:
        if self._graph is None or self._graph_budget <= 0:
            raise RuntimeError("capture() a graph that covers this step first")
        self._graph.replay()
        self._graph_budget -= 1
        self.host_len += 1
        return self.out


def any_peer_wait_failed(states) -> bool:
    """One device read for many layer states: True if any of them has its error word set."""
    words = [w for w in (st.error_word() for st in states) if w is not None]
    if not words:
        return False
    return bool(torch.cat(words).any().item())
