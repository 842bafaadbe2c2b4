"""Where the time of a decode step goes inside its kernels: per-phase wall-clock stamps.

Needs the measurement build of the library (``python -m spotlight_amd.build --stamps``), selected
with ``SPOTLIGHT_HIP_LIB``::

    SPOTLIGHT_HIP_LIB=spotlight_amd/libspotlight_hip_stamps.so \\
        python -m spotlight_amd.phase_stamps --config c2 [--batch B] [--layers L] [--codes-layout head]

Runs a few decode tokens over L independent layer states (so that a layer finds nothing of its own
in the caches), then reads the stamps of the LAST launch of each instrumented kernel
(csrc/phase_stamps.h) and prints, per numbered point: how many workgroups reached it, and the mean /
min / max time since the launch's first workgroup started, in microseconds.
"""
from __future__ import annotations

import argparse
import ctypes as C

POINTS = {
    "hash": {0: "start", 1: "inputs arrived (rotated)", 2: "inputs in LDS", 3: "projection 1 partial sums in LDS (its weights arrived)",
             4: "projection 1 folded", 5: "hidden row in LDS", 6: "projection 2 partial sums in LDS", 7: "projection 2 folded",
             8: "codes stored"},
    "fused": {0: "start", 1: "row count known, histogram cleared", 2: "codes arrived, scores counted",
              3: "own histogram published and acknowledged", 4: "every peer's flag seen", 5: "peers' bins read and summed",
              6: "threshold known", 7: "kept rows listed in LDS",
              8: "table update: list acknowledged, ticket won", 9: "table update: wanted rows classified, misses listed",
              21: "table update: threshold stamp known", 22: "table update: victims listed", 23: "table update: table updated",
              10: "attention: query slices requested", 11: "chunk 0: K / V loads issued", 12: "chunk 0: scores done (K rows arrived)",
              13: "chunk 0: probabilities in LDS", 14: "all chunks accumulated", 15: "wave tiles in LDS", 16: "partials stored",
              17: "partials acknowledged", 18: "ticket taken", 19: "merge: loads of all runs issued", 20: "merged output stored"},
    "lru": {0: "start", 1: "wanted rows classified, misses listed", 2: "threshold stamp known", 3: "victims listed", 4: "table updated"},
}
POINTS["attn"] = {k: v for k, v in POINTS["fused"].items() if 10 <= k <= 20}
POINTS["select_attend"] = POINTS["attn"]


def read(lib, name):
    import numpy as np
    from . import _lib
    buf = np.zeros((_lib.STAMP_WGS, _lib.STAMP_SLOTS), dtype=np.uint64)
    rc = lib.sl_phase_stamps(name.encode(), buf.ctypes.data_as(C.c_void_p), buf.size, 1)
    if rc != 0:
        return None
    return buf


def report(name, buf):
    import numpy as np
    t = buf.astype(np.int64)
    live = t[:, 0] > 0 if name not in ("attn", "select_attend") else t[:, 10] > 0
    first = 0 if name not in ("attn", "select_attend") else 10
    if not live.any():
        return
    t = t[live]
    base = t[:, first].min()
    print(f"== {name}: {live.sum()} workgroups; per point: workgroups that reached it, mean / min / max us since the "
          "launch's first workgroup started, mean us since the workgroup's own start")
    for i in range(t.shape[1]):
        ok = t[:, i] >= t[:, first]
        if not ok.any() or not (t[:, i] > 0).any():
            continue
        rel = (t[ok, i] - base) / 100.0
        own = (t[ok, i] - t[ok, first]) / 100.0
        print(f"  {i:2d} {POINTS.get(name, {}).get(i, ''):55s} n={ok.sum():5d}  mean {rel.mean():6.2f}  min {rel.min():6.2f}  "
              f"max {rel.max():6.2f}  own {own.mean():6.2f}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="c2")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--layers", type=int, default=8)
    ap.add_argument("--tokens", type=int, default=4)
    ap.add_argument("--codes-layout", default="auto")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE")
    ap.add_argument("--cold", action="store_true",
                    help="fill 1 GiB before the stamped token, so that its data (with --layers 1 also its code) come from HBM")
    args = ap.parse_args()
    import torch

    from . import _lib
    from .workloads import CONFIGS, build_layers
    lib = _lib.load()
    for kv in args.tune:
        key, val = kv.split("=")
        _lib.check(lib.sl_tune(key.encode(), int(val)), f"sl_tune({kv})")
    c = dict(CONFIGS[args.config])
    if args.batch:
        c["B"] = args.batch
    dev = torch.device("cuda:0")
    dtype = torch.float32 if c["dtype"] == "f32" else torch.bfloat16
    L = args.layers
    layers = build_layers(c, L, (c["n0"] + 64 + 7) // 8 * 8, dev, codes_layout=args.codes_layout)
    probe = (C.c_ulonglong * 1)()
    if lib.sl_phase_stamps(b"hash", probe, 1, 0) == -3:
        raise SystemExit("this library carries no stamps: build it with `python -m spotlight_amd.build --stamps` "
                         "and point SPOTLIGHT_HIP_LIB at libspotlight_hip_stamps.so")
    g = torch.Generator(device=dev)
    g.manual_seed(7)
    B, QH, KH = c["B"], c["QH"], c["KH"]
    # the tokens run as one captured graph, as in the benchmark: launches follow each other without host gaps
    ins = [[torch.randn((B, h, 128), generator=g, device=dev, dtype=torch.float32).to(dtype) for h in (QH, KH, KH)]
           for _ in range(L)]
    for st, (q, k, v) in zip(layers, ins):
        st.step(q, k, v)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    n_max = c["n0"] + 64
    with torch.cuda.graph(graph):
        for st, (q, k, v) in zip(layers, ins):
            st.q_in.copy_(q); st.k_in.copy_(k); st.v_in.copy_(v)
            st._launch(n_max)
    for i in range(args.tokens):
        if args.cold and i == args.tokens - 1:
            torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        graph.replay()
    torch.cuda.synchronize()
    print(f"config {args.config}: batch {B}, {c['n0']} rows, k = {c['k']}, codes {layers[0].codes_layout}-major, "
          f"{L} layers rotated; stamps of the last layer's launches of the last token" + (", caches flushed before it" if args.cold else ""))
    for name in ("hash", "fused", "lru", "attn", "select_attend"):
        buf = read(lib, name)
        if buf is not None:
            report(name, buf)
    assert not any(st.peer_wait_failed() for st in layers)


if __name__ == "__main__":
    main()
