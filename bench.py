#!/usr/bin/env python3
"""Decode-time retrieval benchmark: sparse-decode us/step/layer and achieved HBM GB/s.

A *step* is one decode step of ONE attention layer: hash the new query and key,
append code + K + V, score every cached code, select the top k per (batch, kv
head), optionally update the LRU resident table, and attend over the selected
rows.  Consecutive steps walk round-robin over ``--layers`` independent layer
states (a real decode token visits every layer once), so no layer finds its
codes or K/V in L2 from its previous visit.  One HIP graph holds one token
(= ``layers`` steps plus the delivery of that token's fresh q/k/v from a
pre-generated pool); replays are timed with the inputs resident in HBM.

Prints ONE JSON line.  ``value`` is microseconds per step (lower is better);
``roofline`` prices the dominant kernel against the 8 TB/s HBM peak of MI355X
on its algorithmic bytes; ``cpu_baseline`` is the CPU oracle's cached-codes
decode step timed on this host on a bounded sample of the same workload, and
``cpu_baseline_reference_form`` the reference's literal decode branch (every key
re-hashed per step, dense masked attention) on the same host.  ``latency_floor``
is what the step's launches cost when their kernels do nothing.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

from spotlight_amd.workloads import CONFIGS, E2EModel, algorithmic_bytes, build_layers  # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS) + ["c5"])
    ap.add_argument("--layers", type=int, default=None)
    ap.add_argument("--batch", type=int, default=None, help="override the configuration's batch size (c1-c4)")
    ap.add_argument("--context", type=int, default=None,
                    help="override the configuration's context length (c1-c4); k follows as 2 %% of it unless --keep is given")
    ap.add_argument("--keep", type=int, default=None, help="override k, the rows kept per (batch entry, kv head)")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="launch heuristic passed to sl_tune (e.g. attn_target_wgs=128)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (reference point for HBM byte counters)")
    ap.add_argument("--host-store", action="store_true",
                    help="keep the full K/V store in pinned host memory behind the LRU table (configs with LRU slots)")
    ap.add_argument("--reuse", type=float, default=None, metavar="P",
                    help="each token's queries repeat the previous token's with probability P (fresh new keys and values "
                         "every token): the access pattern an LRU resident table is for; reports its hit rate")
    ap.add_argument("--floor-only", action="store_true",
                    help="only measure what the step's launches cost by themselves (near-empty kernels on the step's grids)")
    ap.add_argument("--codes-layout", default="auto", choices=["auto", "token", "head"],
                    help="key-code layout: head-major runs scorer, selection and attention as one launch")
    ap.add_argument("--via-modifier", action="store_true",
                    help="c5 only: drive a Llama-3-8B-shaped nn.Module through get_modifier('spotlight-generation-hip') "
                         "and Spotlight.generate (the drop-in path) instead of the hand-written decode token")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-breakdown", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path shards over (batch, kv head) without any exchange, "
              "so this build has no multi-GPU figure; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from spotlight_amd import _lib, decode, kernel

    if args.config == "c5":
        return run_e2e_modifier(args) if args.via_modifier else run_e2e(args)
    for kv in args.tune:
        key, val = kv.split("=")
        _lib.check(_lib.load().sl_tune(key.encode(), int(val)), f"sl_tune({kv})")
    c = dict(CONFIGS[args.config])
    if args.batch:
        c["B"] = args.batch
        c["desc"] += f", batch overridden to {args.batch}"
    if args.context:
        c["n0"] = args.context
        c["k"] = max(1, args.context - int(args.context * 0.98))
        c["desc"] += f", context overridden to {args.context} (k = {c['k']})"
    if args.keep:
        c["k"] = args.keep
        c["desc"] += f", k overridden to {args.keep}"
    L = args.layers or c["layers"]
    steps = args.steps if args.steps is not None else (256 if args.config == "c3" else 1000)
    warmup = args.warmup if args.warmup is not None else 64
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    dtype = torch.float32 if c["dtype"] == "f32" else torch.bfloat16
    B, QH, KH, n0, k, d = c["B"], c["QH"], c["KH"], c["n0"], c["k"], 128

    # the timed region is whole tokens (one graph replay = one token = L steps): the number of steps asked
    # for is rounded to whole tokens, at least one, and the warm-up covers every layer at least once
    # (at least 8 tokens whatever --steps says: one replay alone is a sub-millisecond sample)
    tokens_timed = max(8, round(steps / L))
    tokens_warm = max(1, math.ceil(warmup / L))
    steps_timed, steps_warm = tokens_timed * L, tokens_warm * L
    tokens = tokens_warm + tokens_timed + 4 + 64 + 8   # cache growth incl. the cold tokens and the breakdown passes
    n_cap = (n0 + tokens + 7) // 8 * 8
    if args.floor_only:
        blocks = (n_cap + 4095) // 4096
        head = args.codes_layout == "head" or (args.codes_layout == "auto" and not c["lru"] and QH // KH in (1, 2, 4)
                                               and n_cap <= 65536 and B * KH * blocks <= 256 and k <= 128 * blocks)
        print(json.dumps({"config": args.config, "latency_floor": latency_floor(dev, c, L, n0 + tokens, reps=64, one_launch_tail=head,
                                                                                   lru_inside=lru_inside_selection_launch(c, args.tune, head))}), flush=True)
        return

    gpu_gen = torch.Generator(device=dev)
    gpu_gen.manual_seed(0)

    # per-token inputs for every layer, drawn once; a token's slice is copied in by the graph
    P = 16 if args.reuse is None else 64
    pool = [torch.randn((P, L, B, h, d), generator=gpu_gen, device=dev, dtype=torch.float32).to(dtype)
            for h in (QH, KH, KH)]
    if args.reuse is not None:
        # a token keeps the previous token's queries with probability --reuse (decided per token, seeded)
        coin = torch.rand(P, generator=torch.Generator().manual_seed(3))
        for i in range(1, P):
            if coin[i].item() < args.reuse:
                pool[0][i].copy_(pool[0][i - 1])
    cur = [torch.empty((1, L, B, h, d), device=dev, dtype=dtype) for h in (QH, KH, KH)]
    tok = torch.zeros((1,), dtype=torch.int64, device=dev)

    layers = build_layers(c, L, n_cap, dev, codes_layout=args.codes_layout, host_store=args.host_store,
                          inputs=[tuple(t[0, li] for t in cur) for li in range(L)])

    def token_body(n_max):
        for i in range(3):
            torch.index_select(pool[i], 0, tok, out=cur[i])
        tok.add_(1).remainder_(P)
        for st in layers:
            st._launch(n_max)

    def capture(fn):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g

    n_max = n0 + tokens
    token_graph = capture(lambda: token_body(n_max))

    # cold figure: the very first replay on freshly built layer states (kernel code, weights, codes and
    # translation entries all come from memory for the first time); it is also the first warm-up token
    torch.cuda.synchronize()
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    token_graph.replay()
    c1.record()
    torch.cuda.synchronize()
    cold_first_token_us = c0.elapsed_time(c1) * 1e3 / L
    for _ in range(tokens_warm - 1):
        token_graph.replay()
    torch.cuda.synchronize()
    lru_before = [st.lru_stats.sum(dim=(0, 1)).cpu() for st in layers] if c["lru"] else None
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(tokens_timed + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(tokens_timed):
        token_graph.replay()
        marks[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = marks[0].elapsed_time(marks[-1])
    per_token_us = sorted(marks[i].elapsed_time(marks[i + 1]) * 1e3 / L for i in range(tokens_timed))
    ms_per_step = wall_ms / steps_timed
    us_per_step = ms_per_step * 1e3
    lru_hit_rate = link_gbps = None
    if c["lru"]:
        delta = sum((st.lru_stats.sum(dim=(0, 1)).cpu() - b0).to(torch.int64) for st, b0 in zip(layers, lru_before))
        hits, misses = int(delta[0]), int(delta[1])
        lru_hit_rate = hits / max(1, hits + misses)
        # every miss moves one K and one V row from the full store into the resident table
        link_gbps = misses * 2 * d * (4 if c["dtype"] == "f32" else 2) / (wall_ms * 1e-3) / 1e9
    # a bounded wait that ran out would have produced wrong rows silently: no figure is reported then
    failed = [i for i, st in enumerate(layers) if st.peer_wait_failed()]
    if failed:
        raise RuntimeError(f"bounded peer wait ran out in layers {failed}: the timed steps are invalid")
    # cold figure per token: a 1 GiB fill before each replay pushes the step's weights, codes and rows out
    # of the L2s and the 256 MB memory-side cache -- what the model's own layers do between two decode
    # steps of a layer (Llama-3-8B streams 0.4 GB of weights per layer); the timed replays above revisit
    # each layer's data after only L - 1 other layers of this path
    flush = torch.empty(1 << 28, dtype=torch.float32, device=dev)
    cold = []
    for i in range(8):
        flush.fill_(float(i))
        c0.record()
        token_graph.replay()
        c1.record()
        torch.cuda.synchronize()
        cold.append(c0.elapsed_time(c1) * 1e3 / L)
    del flush
    cold.sort()
    cold_token_us = cold[len(cold) // 2]
    n_mid = n0 + tokens_warm + tokens_timed / 2
    ab = algorithmic_bytes(c, n_mid)
    for st in layers:   # the graph advanced the lengths on the device; keep the host-side bound in step
        st.host_len = n0 + tokens_warm + tokens_timed + 8

    if args.calibration_copy:
        src = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)   # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # ---- per-kernel durations: HIP events around a graph of M launches of one stage, rotating layers
    kernels = {}
    dominant = None
    if not args.no_kernel_breakdown:
        # equalise lengths (a partial token may have advanced only some layers)
        M = 4 * L
        one_launch_tail = layers[0].codes_layout == "head"   # scorer + selection + attention as ONE launch
        if one_launch_tail and c["lru"]:    # the launch ends at the selection: table update and attention follow
            stage_sets = [("hash", _lib.STAGE_HASH), ("score+select", _lib.STAGE_SCORE | _lib.STAGE_SELECT), ("attn", _lib.STAGE_ATTN)]
        elif one_launch_tail:
            stage_sets = [("hash", _lib.STAGE_HASH), ("score+select+attn", _lib.STAGE_SCORE | _lib.STAGE_SELECT | _lib.STAGE_ATTN)]
        else:
            stage_sets = [("hash", _lib.STAGE_HASH), ("score", _lib.STAGE_SCORE),
                          ("score+select", _lib.STAGE_SCORE | _lib.STAGE_SELECT), ("attn", _lib.STAGE_ATTN),
                          ("select+attn", _lib.STAGE_SELECT | _lib.STAGE_ATTN)]
        if c["lru"]:
            stage_sets.insert(2 if one_launch_tail else 3, ("lru", _lib.STAGE_LRU))
        raw = {}
        for name, mask in stage_sets:
            def body(mask=mask):
                for j in range(M):
                    layers[j % L]._launch(n_max, mask)
            g = capture(body)
            g.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            raw[name] = e0.elapsed_time(e1) * 1e3 / M
            del g
        if not one_launch_tail:
            raw["select"] = max(raw["score+select"] - raw["score"], 0.0)
        ab["select+attn"] = ab["attn"]
        ab["score+select+attn"] = ab["score"] + ab["attn"]
        ab["score+select"] = ab["score"]
        # the step runs selection and attention as one launch when it can (no LRU, <= 64k rows):
        # then "select+attn" is that launch and "select" / "attn" are the two-launch alternative
        # (same rule as the library: the shape allows it and a 4096-token block keeps <= 128 rows on average)
        fused_tail = (not c["lru"] and n_cap <= 65536 and QH // KH in (1, 2, 4)
                      and k <= 128 * ((n_max + 4095) // 4096))
        names = ("hash", "score", "select+attn") if fused_tail else ("hash", "score", "select", "lru", "attn")
        if one_launch_tail:
            names = ("hash", "score+select", "lru", "attn") if c["lru"] else ("hash", "score+select+attn")
        for name in ("hash", "score", "select", "score+select", "lru", "attn", "select+attn", "score+select+attn"):
            if name == "score+select" and not (one_launch_tail and c["lru"]):
                continue
            if name in raw:
                us = raw[name]
                kernels[name] = {"us": round(us, 3), "algorithmic_bytes": ab[name],
                                 "gbps": round(ab[name] / us / 1e3, 1) if us > 0 else None,
                                 "in_step": name in names}
        dominant = max((n for n in kernels if kernels[n]["in_step"] and kernels[n]["algorithmic_bytes"] > 0),
                       key=lambda n: kernels[n]["us"])

    traffic = profiled_traffic(args.config, dominant) if dominant else None
    roofline = None
    if dominant:
        ach = kernels[dominant]["gbps"]
        roofline = {"kernel": dominant, "bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": traffic,
                    "algorithmic_bytes_per_launch": kernels[dominant]["algorithmic_bytes"],
                    "us_per_launch": kernels[dominant]["us"]}

    lru_inside = lru_inside_selection_launch(c, args.tune, layers[0].codes_layout == "head")
    floor = latency_floor(dev, c, L, n_max, one_launch_tail=layers[0].codes_layout == "head", lru_inside=lru_inside)

    cpu_baseline = cpu_reference_form = None
    if not args.no_cpu_baseline:
        cpu_baseline = cpu_leg(layers[0], c, budget_s=12.0)
        cpu_reference_form = cpu_leg_reference_form(layers[0], c, budget_s=12.0)

    failed = [i for i, st in enumerate(layers) if st.peer_wait_failed()]
    if failed:
        raise RuntimeError(f"bounded peer wait ran out in layers {failed} during the per-kernel passes")
    step_gbps = ab["step"] / us_per_step / 1e3
    out = {
        "metric": "sparse-decode us/step/layer (Llama-3-8B GQA, 32k ctx)" if args.config == "c2"
                  else f"sparse-decode us/step/layer ({args.config})",
        "value": round(us_per_step, 3), "unit": "us/step/layer", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "steps_timed": steps_timed, "warmup_timed": steps_warm,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": c["dtype"], "data": "synthetic",
        "config": {"workload": f"{args.config}: {c['desc']}", "batch": B, "q_heads": QH, "kv_heads": KH,
                   "head_dim": d, "context": n0, "k": k, "code_bits": 128, "hash": c["hash"],
                   "lru_slots": c["lru"], "codes_layout": layers[0].codes_layout,
                   "launches_per_step": floor["launches_per_step"] if floor else None, "kv_store": "pinned host memory" if args.host_store else "hbm",
                   "layers_rotated": L,
                   "graph": f"one HIP graph per token ({L} steps); {tokens_timed} replays timed after {tokens_warm} warm-up replays"},
        "gpu_event_ms_per_step": round(gpu_ms / steps_timed, 6),
        "us_per_step_median_token": round(per_token_us[len(per_token_us) // 2], 3),
        "us_per_step_min_token": round(per_token_us[0], 3), "us_per_step_max_token": round(per_token_us[-1], 3),
        "cold_first_token_us": round(cold_first_token_us, 3), "cold_token_us": round(cold_token_us, 3),
        "lru_hit_rate": round(lru_hit_rate, 4) if lru_hit_rate is not None else None,
        "lru_miss_row_gbps": round(link_gbps, 1) if link_gbps is not None else None,
        "query_reuse": args.reuse,
        "hbm_gbps": round(step_gbps, 1), "hbm_frac": round(step_gbps / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_step": int(ab["step"]),
        "tokens_per_s": round(B / (ms_per_step * 1e-3 * L), 2), "tokens_per_s_layers": L,
        "kernels": kernels, "lru_inside_selection_launch": lru_inside, "roofline": roofline, "cpu_baseline": cpu_baseline,
        "cpu_baseline_reference_form": cpu_reference_form,
        "latency_floor": floor,
        "value_over_floor": round(us_per_step / floor["launches_with_one_load_us"], 2) if floor else None,
    }
    print(json.dumps(out), flush=True)


def run_e2e(args):
    """c5: a random-init Llama-3-8B, batch 4, 32768-token prompt prefilled densely, then greedy decoding
    with layers 0-1 dense and layers 2.. on the sparse step (k = 655).  One decoded token for the
    whole batch and all layers is ONE captured HIP graph; `value` is decoded tokens per second over
    the timed replays."""
    import torch

    L = args.layers or 32
    steps = args.steps if args.steps is not None else 512
    warmup = args.warmup if args.warmup is not None else 8
    B, n0, k = 4, 32768, 655
    m = E2EModel(L=L, B=B, n0=n0, n_cap=(n0 + steps + warmup + 16 + 7) // 8 * 8, k=k)
    prefill_s = m.prefill()
    with torch.no_grad():
        m.step_body()                                                          # eager once (lazy initialisations)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            m.step_body()
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        gpu_ms = e0.elapsed_time(e1)
        # the sparse attention's share: a graph with only the sparse layers' launches
        ga = torch.cuda.CUDAGraph()
        with torch.cuda.graph(ga):
            for st in m.sparse:
                st._launch(m.n_cap, _STAGES_NO_ADVANCE)
        ga.replay()
        torch.cuda.synchronize()
        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a0.record()
        for _ in range(32):
            ga.replay()
        a1.record()
        torch.cuda.synchronize()
        attn_ms = a0.elapsed_time(a1) / 32
    ms_per_step = max(wall_ms, gpu_ms) / steps
    lens = [int(st.seq_lens[0]) for st in m.sparse]
    assert all(v == lens[0] for v in lens), "sparse layers disagree on the cache length"
    out = {
        "metric": "e2e greedy decode tokens/s (random-init Llama-3-8B, batch 4, 32k prompt)",
        "value": round(B / (ms_per_step * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "c5: random-init Llama-3-8B end to end, batch 4, 32768-token dense prefill, greedy decode, "
                               "layers 0-1 dense, k=655", "layers": L, "batch": B, "context": n0, "k": k,
                   "graph": "one HIP graph per decoded token (all layers)"},
        "prefill_s": round(prefill_s, 2), "cache_len_after": lens[0] if lens else None,
        "sparse_attention_ms_per_step": round(attn_ms, 4),
        "sparse_attention_us_per_layer": round(attn_ms * 1e3 / max(1, len(m.sparse)), 2),
        "sparse_attention_share": round(attn_ms / ms_per_step, 4),
        "roofline": None, "cpu_baseline": None,
    }
    print(json.dumps(out), flush=True)


def run_e2e_modifier(args):
    """c5 through the drop-in path: a random-init Llama-3-8B-shaped nn.Module patched by
    get_modifier('spotlight-generation-hip') (layers 0-1 dense, per-kv-head key hash, MLP 128-256-128, 98 %
    pruned with the budget rule evaluated on the device), batch 4, 32768-token prompt prefilled densely by the
    patched forward, then ``Spotlight.generate``: first decoded token eagerly, the rest as replays of the one
    HIP graph ``generate`` captures.  `value` is decoded tokens per second over the decode part of ``generate``
    (its own clock, bracketed by device synchronisation)."""
    import torch

    from spotlight_amd.modifiers import get_modifier
    from spotlight_amd.workloads import llama_shaped

    L = args.layers or 32
    steps = args.steps if args.steps is not None else 64
    B, n0 = args.batch or 4, args.context or 32768
    conf = {"draft_kwargs": {"enable": True, "fix_layers": [0, 1], "mask_out": 0.98, "bench_mark": False, "min_remain": 20,
                             "num_mlp_layers": 2, "mlp_dims": "[128,256,128]", "mlp_residue": False, "gqa_key_hash": True,
                             "record_timing": True}}
    base = llama_shaped(L=L)
    _, cls = get_modifier("spotlight-generation-hip")
    m = cls(base, None, None, conf).eval()
    ids = torch.randint(0, base.config.vocab_size, (B, n0), generator=torch.Generator().manual_seed(0))
    out = m.generate(ids, max_new_tokens=steps, eos_token_id=[-1])
    assert out.shape == (B, n0 + steps)
    t = m.timing
    ms_per_token = t["graph_decode_s"] * 1e3 / max(1, t["graph_tokens"]) if t["graph_tokens"] else t["decode_s"] * 1e3 / steps
    res = {
        "metric": "e2e greedy decode tokens/s through the patched modifier (random-init Llama-3-8B, batch 4, 32k prompt)",
        "value": round(B / (ms_per_token * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 1,
        "ms_per_step": round(ms_per_token, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "c5 via the modifier: get_modifier('spotlight-generation-hip') -> Spotlight.generate on a "
                               "random-init Llama-3-8B-shaped nn.Module, batch 4, 32768-token dense prefill, greedy decode, "
                               "layers 0-1 dense, 98 % pruned (budget rule on the device)",
                   "layers": L, "batch": B, "context": n0,
                   "graph": "generate() captures the decode token once and replays it"},
        "prefill_s": round(t["prefill_s"], 2), "first_decode_token_ms": round(t["eager_decode_s"] * 1e3 / max(1, t["eager_tokens"]), 3),
        "graph_tokens": t["graph_tokens"], "eager_tokens": t["eager_tokens"], "capture_s": round(t["capture_s"], 3),
        "roofline": None, "cpu_baseline": None,
    }
    print(json.dumps(res), flush=True)


_STAGES_NO_ADVANCE = 1 | 2 | 4 | 16     # hash, score, select, attention launched as stages: lengths do not advance


STAGE_KERNEL = {"score+select+attn": "score_select_attend_kernel", "score+select": "score_select_attend_kernel", "hash": "hash_kernel", "score": "hamming_kernel", "select": "select_fused_kernel",
                "lru": "lru_kernel", "attn": "sparse_attn_kernel", "select+attn": "select_attend_kernel"}


def profiled_traffic(config, stage):
    """HBM bytes per launch of the stage's kernel as counted by rocprofv3 (FETCH_SIZE and
    WRITE_SIZE, calibrated on a device copy): read from the committed summary of that
    profile, profiles/decode_step_<config>_*.txt; None when there is no such summary."""
    import glob
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", f"decode_step_{config}_*.txt"))):
        in_table = False
        with open(path) as f:
            for line in f:
                if line.startswith("HBM traffic per launch"):
                    in_table = True
                elif in_table and line.startswith(STAGE_KERNEL.get(stage, "?")):
                    cols = line.split()
                    try:
                        return int(round((float(cols[-2]) + float(cols[-1])) * 1e6))
                    except ValueError:
                        return None
    return None


def lru_inside_selection_launch(c, tunes, one_launch_tail):
    """Whether the step's scorer + selection launch also runs the table update (the library's rule:
    head-major codes, a table of at most 2048 slots, not switched off with --tune fused_lru=0)."""
    return bool(one_launch_tail and c["lru"] and c["lru"] <= 2048 and "fused_lru=0" not in tunes)


def latency_floor(dev, c, L, n_max, reps=8, one_launch_tail=False, lru_inside=False):
    """What the step's launches cost by themselves on this machine: a HIP graph of L x (as many dependent
    launches as the step has, with the step's grids) of a kernel that does nothing, and of one whose lanes do a
    single dependent load.  us per step-equivalent."""
    import torch

    from spotlight_amd import _lib
    lib = _lib.load()
    B, QH, KH = c["B"], c["QH"], c["KH"]
    # the library's rule: the fewest batch rows per hash workgroup (1, 2, 3, 4, 6, 8) that give one round of
    # workgroups over the 256 compute units, else 4
    hash_rows = next((r for r in (1, 2, 3, 4, 6, 8) if (QH + KH) * ((B + r - 1) // r) <= 256), 4)
    blocks4k = (n_max + 4095) // 4096
    grids = [((QH + KH) * ((B + hash_rows - 1) // hash_rows), 512),
             (((n_max * KH + 2047) // 2048) * B, 512)]
    if one_launch_tail:
        # the library picks the rows per block by shape and by what the device holds at once
        dt = {"f32": 0, "bf16": 1, "f16": 2}[c["dtype"]]
        rows = lib.sl_decode_head_major_fits(dt, B, QH, KH, 128, n_max, c["k"], int(bool(c["lru"])))
        blocks = (n_max + rows - 1) // rows if rows > 0 else blocks4k
        grids = [grids[0], (blocks * KH * B, 512)]
        if c["lru"]:
            grids += ([] if lru_inside else [(B * KH, 1024)]) + [(min(32, max(1, -(-512 // (B * KH)))) * B * KH, 256)]
    elif c["lru"]:
        grids += [(((n_max + 8191) // 8192) * B * KH, 1024), (B * KH, 1024), (min(32, max(1, -(-512 // (B * KH)))) * B * KH, 256)]
    elif QH // KH in (1, 2, 4) and n_max <= 65536 and c["k"] <= 128 * blocks4k:
        grids += [(blocks4k * KH * B, 512)]
    else:
        grids += [(((n_max + 8191) // 8192) * B * KH, 1024), (min(32, max(1, -(-512 // (B * KH)))) * B * KH, 256)]
    table = torch.zeros(1024, dtype=torch.int32, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    res = {"launches_per_step": len(grids), "grids": grids}
    for name, chain in (("empty_launches_us", 0), ("launches_with_one_load_us", 1)):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            s = torch.cuda.current_stream().cuda_stream
            for _ in range(L):
                for blocks, threads in grids:
                    _lib.check(lib.sl_probe_launch(blocks, threads, table.data_ptr(), sink.data_ptr(), chain, s), "sl_probe_launch")
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        res[name] = round(e0.elapsed_time(e1) * 1e3 / (reps * L), 3)
        del g
    return res


def cpu_leg_reference_form(st, c, budget_s):
    """The reference's literal decode branch (spotlight_generation.py:149-215) on this host: hash the query
    AND every cached key with the per-query-head weights (keys repeat_kv'd), +-1 matmul, per-query-head
    topk, finfo.min mask, dense SDPA -- one sequence at a time, as the reference asserts batch 1."""
    import torch

    from oracle import spotlight_oracle as orc

    n = int(st.seq_lens.max().item())
    B, QH, KH = st.B, st.QH, st.KH
    G = QH // KH
    hq = st.hash_q
    bias = lambda b, width: (b.cpu() if b is not None else torch.zeros(QH, width, dtype=hq.w1.dtype))[None, :, None]
    ws = [(hq.w1.cpu()[None], bias(hq.b1, hq.d_hid))]
    if hq.w2 is not None:
        ws.append((hq.w2.cpu()[None], bias(hq.b2, hq.nbits)))
    keys = [st.keys[b:b + 1, :n].cpu().permute(0, 2, 1, 3).repeat_interleave(G, dim=1) for b in range(min(B, 2))]
    vals = [st.vals[b:b + 1, :n].cpu().permute(0, 2, 1, 3).repeat_interleave(G, dim=1) for b in range(min(B, 2))]
    mask_out = 1.0 - c["k"] / n
    g = torch.Generator()
    g.manual_seed(2)
    times = []
    t_start = time.perf_counter()
    while len(times) < 1 or (time.perf_counter() - t_start < budget_s and len(times) < 20):
        q = torch.randn(1, QH, 1, 128, generator=g).to(st.dtype)
        b = len(times) % len(keys)
        t0 = time.perf_counter()
        orc.decode_step_reference_form(q, keys[b], vals[b], ws, hq.residue, mask_out)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(med * B * 1e6, 1), "unit": "us/step/layer", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": os.cpu_count(),
            "sample": f"{len(times)} decode steps of one layer and ONE sequence at n={n} (median"
                      + (f", multiplied by the batch of {B}" if B > 1 else "") + "), torch CPU restatement of the "
                      "reference's own decode branch: every cached key re-hashed per step, +-1 matmul, torch.topk, "
                      "masked dense SDPA"}


def cpu_leg(st, c, budget_s):
    """The oracle's cached-codes decode step (hash q -> pack -> XOR/popcount -> stable
    top-k -> gather -> softmax attention) on this host, on layer 0's real cache."""
    import numpy as np
    import torch

    from oracle import spotlight_oracle as orc

    n = int(st.seq_lens.max().item())
    B, QH, KH, k = st.B, st.QH, st.KH, st.k
    codes = st.codes[:, :n].cpu().numpy()
    keys, vals = st.keys[:, :n].cpu(), st.vals[:, :n].cpu()
    hq = st.hash_q
    ws = [(hq.w1.cpu()[None], (hq.b1.cpu() if hq.b1 is not None else torch.zeros(QH, hq.d_hid, dtype=hq.w1.dtype))[None, :, None])]
    if hq.w2 is not None:
        ws.append((hq.w2.cpu()[None], hq.b2.cpu()[None, :, None]))
    g = torch.Generator()
    g.manual_seed(1)
    bidx = torch.arange(B)[:, None, None]
    hidx = torch.arange(KH)[None, :, None]
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        q = torch.randn(B, QH, 128, generator=g).to(st.dtype)
        t0 = time.perf_counter()
        pre = orc.mlp_hash_torch(q.unsqueeze(2), ws, hq.residue).squeeze(2)
        q_code = orc.pack_sign_u32(pre.float().numpy())[:, None]
        score = orc.hamming_score_u32(q_code, codes, st.head_map)
        idx = orc.topk_stable(score, k)
        ti = torch.from_numpy(idx).long()
        ks = keys[bidx, ti, hidx].float()            # [B,KH,k,d]
        vs = vals[bidx, ti, hidx].float()
        qg = q.float().view(B, KH, QH // KH, 128)
        p = torch.softmax(torch.einsum("bhgd,bhkd->bhgk", qg, ks) / math.sqrt(128), dim=-1)
        _ = torch.einsum("bhgk,bhkd->bhgd", p, vs)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(med * 1e6, 1), "unit": "us/step/layer", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": os.cpu_count(),
            "sample": f"{len(times)} decode steps of one layer at n={n} (median), numpy/torch CPU restatement "
                      "with cached key codes"}


if __name__ == "__main__":
    main()
