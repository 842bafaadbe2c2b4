"""Writes tests/golden/retrieval_small.npz: seeded inputs and the outputs the CPU
oracle (oracle/spotlight_oracle.py) gives for every stage of the retrieval path.

The reference holds no golden vectors for this path and cannot be run here
(its kernels need CUDA, its modifiers need packages this image lacks), so the
fixture pins the oracle against drift and gives the GPU tests a second,
file-based target.  Run from the repository root:
    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import spotlight_oracle as orc  # noqa: E402


def main():
    r = np.random.default_rng(20240607)
    B, QH, KH, n, k, d = 2, 4, 2, 120, 12, 128
    x_pack = r.standard_normal((5, 3, 128)).astype(np.float32)
    x_pack[0, 0, :6] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-38]
    q_code = r.integers(0, 2 ** 32, size=(B, 1, QH, 4), dtype=np.uint64).astype(np.uint32)
    k_code = r.integers(0, 2 ** 32, size=(B, n, KH, 4), dtype=np.uint64).astype(np.uint32)
    # clustered codes so that scores tie heavily, as real sign codes do
    k_code[:, ::3] = k_code[:, 1::3][:, : k_code[:, ::3].shape[1]]
    score_i = orc.hamming_score_u32(q_code, k_code, "interleaved")
    score_b = orc.hamming_score_u32(q_code, k_code, "blocked")
    idx = orc.topk_stable(score_b, k)
    q = r.standard_normal((B, QH, d)).astype(np.float32)
    keys = r.standard_normal((B, n, KH, d)).astype(np.float32)
    vals = r.standard_normal((B, n, KH, d)).astype(np.float32)
    k_sel, v_sel = orc.gather_kv(keys, vals, idx)
    attn = orc.sparse_attention(q, keys, vals, idx)
    HH = 2
    x_hash = r.standard_normal((B, HH, 128)).astype(np.float32)
    w1 = (r.standard_normal((HH, 128, 128)) * 0.05).astype(np.float32)
    b1 = (r.standard_normal((HH, 128)) * 0.05).astype(np.float32)
    w2 = (r.standard_normal((HH, 128, 128)) * 0.05).astype(np.float32)
    b2 = (r.standard_normal((HH, 128)) * 0.05).astype(np.float32)
    pre = orc.mlp_hash(x_hash, [(w1, b1), (w2, b2)], residue=False)
    lin = r.standard_normal((HH, 128, 128)).astype(np.float32)
    pre_lin = orc.linear_hash(x_hash, lin)
    lru = orc.LruModel(8)
    lru_trace = []
    for t, (sel, new) in enumerate([([0, 1, 2], 3), ([1, 2, 9], 10), ([0, 9, 10], 11), ([4, 5, 6], 12)], 1):
        slots = lru.step(t, sel, new)
        lru_trace.append(np.array(slots + lru.token + lru.stamp, dtype=np.int64))
    np.savez_compressed(
        os.path.join(ROOT, "tests", "golden", "retrieval_small.npz"),
        x_pack=x_pack, packed_u32=orc.pack_sign_u32(x_pack), packed_u8=orc.pack_sign_u8(x_pack),
        q_code=q_code, k_code=k_code, score_interleaved=score_i, score_blocked=score_b, k=np.int64(k), idx=idx,
        q=q, keys=keys, vals=vals, k_sel=k_sel, v_sel=v_sel, attn=attn,
        x_hash=x_hash, w1=w1, b1=b1, w2=w2, b2=b2, pre_mlp=pre, code_mlp=orc.pack_sign_u32(pre),
        lin=lin, pre_lin=pre_lin, code_lin=orc.pack_sign_u32(pre_lin), lru_trace=np.stack(lru_trace))


if __name__ == "__main__":
    main()
