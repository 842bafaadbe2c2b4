"""The synthetic workloads the benchmark, the profiling aids and the end-to-end tests share: the
four per-layer decode configurations (shapes of BASELINE's configs 1-4), their algorithmic bytes,
layer states prefilled with seeded random rows, and two random-init Llama-shaped models for the
end-to-end configuration -- ``E2EModel`` (the decode token written out by hand, one HIP graph per
token) and ``LlamaShaped`` (an ``nn.Module`` with the attribute names the reference's modifier
patches, spotlight/modifiers/spotlight_generation.py:298-330, to be driven through
``get_modifier('spotlight-generation-hip')``)."""
from __future__ import annotations

import time
import types

CONFIGS = {
    # name: B, QH, KH, n0, k, dtype, hash, lru slots, default layers, description
    "c1": dict(B=1, QH=32, KH=32, n0=4096, k=410, dtype="f32", hash="linear", lru=0, layers=32,
               desc="Llama-2-7B shape, fp32, linear 128x128 Gaussian hash, 90% pruned"),
    "c2": dict(B=1, QH=32, KH=8, n0=32768, k=655, dtype="bf16", hash="mlp", lru=0, layers=32,
               desc="Llama-3-8B GQA, bf16, 32k ctx, MLP 128-256-128 hash, 98% pruned"),
    "c3": dict(B=16, QH=32, KH=8, n0=16384, k=328, dtype="bf16", hash="mlp", lru=1024, layers=32,
               desc="Llama-3-8B GQA, bf16, batch 16 x 16k ctx, LRU resident buffer 1024, 98% pruned"),
    "c4": dict(B=1, QH=40, KH=8, n0=131072, k=2622, dtype="bf16", hash="mlp", lru=0, layers=16,
               desc="Qwen2.5-14B shape, bf16, 128k ctx, 98% pruned"),
}


def algorithmic_bytes(c, n):
    """Bytes one step of one layer has to move, intermediates excluded."""
    s = 4 if c["dtype"] == "f32" else 2
    B, QH, KH, k, d, nbits = c["B"], c["QH"], c["KH"], c["k"], 128, 128
    if c["hash"] == "mlp":
        per_head = (128 * 256 + 256 + 256 * 128 + 128) * s
        w = per_head * (QH + KH)
    else:
        w = 128 * 128 * s * (QH if KH == QH else QH + KH)
    io_new = B * (QH + 2 * KH) * d * s                       # q, k_new, v_new read
    append = B * KH * (nbits // 8 + 2 * d * s)               # code + K + V written
    hash_b = w + io_new + append + B * QH * nbits // 8
    score_b = B * n * KH * nbits // 8 + B * QH * nbits // 8  # codes streamed + q codes
    attn_b = 2 * B * k * KH * d * s + 2 * B * QH * d * s     # selected K and V rows, q, out
    lru_b = 0
    return {"hash": hash_b, "score": score_b, "select": 0, "lru": lru_b, "attn": attn_b,
            "step": w + B * QH * d * s + B * n * KH * nbits // 8 + 2 * B * k * KH * d * s + B * QH * d * s + append}



def build_layers(c, L, n_cap, dev, codes_layout="auto", host_store=False, inputs=None, seed=0):
    """L independent layer states of configuration ``c`` (a CONFIGS entry), each prefilled with
    c["n0"] seeded N(0,1) rows per sequence whose codes come from the many-rows hash kernel.
    ``inputs``: per layer a (q, k, v) tuple of buffers the step reads its inputs from."""
    import torch

    from . import decode
    dtype = torch.float32 if c["dtype"] == "f32" else torch.bfloat16
    B, QH, KH, n0, k, d = c["B"], c["QH"], c["KH"], c["n0"], c["k"], 128
    cpu_gen = torch.Generator()
    cpu_gen.manual_seed(seed)
    gpu_gen = torch.Generator(device=dev)
    gpu_gen.manual_seed(seed + 1)
    layers = []
    for li in range(L):
        if c["hash"] == "mlp":
            hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dtype, dev, cpu_gen)
            hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dtype, dev, cpu_gen)
        else:
            hq = decode.HashWeights.random_linear(QH, 128, 128, dtype, dev, cpu_gen)
            hk = hq if KH == QH else decode.HashWeights.random_linear(KH, 128, 128, dtype, dev, cpu_gen)
        st = decode.LayerDecodeState(B, QH, KH, d, n_cap, k, hq, hk, dtype=dtype, device=dev,
                                     lru_slots=c["lru"], inputs=inputs[li] if inputs is not None else None,
                                     host_store=host_store, codes_layout=codes_layout)
        # prefill in slabs to bound the transient memory of hashing
        st.seq_lens.zero_()
        slab = max(1, (1 << 22) // (B * KH))
        for s0 in range(0, n0, slab):
            s1 = min(n0, s0 + slab)
            kk = torch.randn((B, s1 - s0, KH, d), generator=gpu_gen, device=dev, dtype=torch.float32).to(dtype)
            vv = torch.randn((B, s1 - s0, KH, d), generator=gpu_gen, device=dev, dtype=torch.float32).to(dtype)
            st.keys[:, s0:s1] = kk      # (a device-to-host copy with a host-memory store)
            st.vals[:, s0:s1] = vv
            st.hash_k.hash_rows(kk, out=st.codes[:, s0:s1])
        st.seq_lens.fill_(n0)
        st.host_len = n0
        layers.append(st)
    torch.cuda.synchronize()
    return layers


class E2EModel:
    """Random-init Llama-shaped decoder (RMSNorm, rotary GQA attention, SiLU-gated MLP; defaults are
    Llama-3-8B's dims: hidden 4096, 32 q / 8 kv heads of 128, MLP 14336, vocab 128256, rope theta 5e5)
    whose layers in ``fix_layers`` attend densely and whose other layers run the sparse HIP step
    (k rows kept, MLP hash 128-256-128 per query head and per kv head).  It stands for the loop of
    the reference's ``generate`` (spotlight_generation.py:470-495) with dense layers 0-1
    (config/llama3-8b-spotlight-generation.json).  ``step_body`` is one decoded token for the
    whole batch and is capturable as one HIP graph: positions and lengths live on the device, and
    the sparse step rotates q and the new key itself."""

    def __init__(self, L=32, B=4, n0=32768, n_cap=None, k=655, fix_layers=(0, 1), hidden=4096, inter=14336,
                 vocab=128256, QH=32, KH=8, theta=5e5, seed=0):
        import torch

        from spotlight_amd import decode
        self.dev = dev = torch.device("cuda:0")
        self.dt = dt = torch.bfloat16
        self.L, self.B, self.n0, self.k, self.QH, self.KH, self.d = L, B, n0, k, QH, KH, 128
        self.hidden, self.vocab, self.theta = hidden, vocab, theta
        self.n_cap = n_cap or (n0 + 1024 + 7) // 8 * 8
        d = self.d
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        cg = torch.Generator()
        cg.manual_seed(seed)
        self.g = g
        rnd = lambda *shape: (torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * 0.02).to(dt)
        self.embed, self.lm_head = rnd(vocab, hidden), rnd(vocab, hidden)
        self.layers = []
        for li in range(L):
            w = dict(wq=rnd(QH * d, hidden), wk=rnd(KH * d, hidden), wv=rnd(KH * d, hidden), wo=rnd(hidden, QH * d),
                     wg=rnd(inter, hidden), wu=rnd(inter, hidden), wd=rnd(hidden, inter),
                     n1=torch.ones(hidden, device=dev, dtype=dt), n2=torch.ones(hidden, device=dev, dtype=dt))
            if li in fix_layers:
                w["kc"] = torch.zeros((B, KH, self.n_cap, d), device=dev, dtype=dt)   # head-major: read in place
                w["vc"] = torch.zeros((B, KH, self.n_cap, d), device=dev, dtype=dt)
            else:
                hq = decode.HashWeights.random_mlp(QH, [128, 256, 128], dt, dev, cg)
                hk = decode.HashWeights.random_mlp(KH, [128, 256, 128], dt, dev, cg)
                w["st"] = decode.LayerDecodeState(B, QH, KH, d, self.n_cap, k, hq, hk, dtype=dt, device=dev,
                                                  rope_theta=theta)
            self.layers.append(w)
        self.norm_f = torch.ones(hidden, device=dev, dtype=dt)
        self.inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, device=dev, dtype=torch.float32) / d))
        self.tok = torch.zeros((B,), dtype=torch.int64, device=dev)
        self.logits = torch.zeros((B, vocab), dtype=torch.float32, device=dev)   # of the last decoded token
        self.pos = torch.full((1,), n0, dtype=torch.int64, device=dev)
        self.col = torch.arange(self.n_cap, device=dev)
        self.sparse = [w["st"] for w in self.layers if "st" in w]

    def rms(self, x, w):
        import torch
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).to(self.dt) * w

    def rope(self, x, pos):   # x [..., t, H, d], pos [t] (device)
        import torch
        d = self.d
        ang = pos.float()[:, None] * self.inv_freq[None, :]
        emb = torch.cat((ang, ang), dim=-1)
        cos, sin = emb.cos().to(self.dt)[:, None, :], emb.sin().to(self.dt)[:, None, :]
        rot = torch.cat((-x[..., d // 2:], x[..., : d // 2]), dim=-1)
        return x * cos + rot * sin

    def mlp(self, w, h):
        import torch.nn.functional as F
        return (F.silu(h @ w["wg"].T) * (h @ w["wu"].T)) @ w["wd"].T

    def prefill(self):
        """Dense causal attention in every layer (the draft is not used there), one sequence at a
        time; sparse layers also get the codes of their keys.  Returns the seconds it took."""
        import torch
        import torch.nn.functional as F

        from spotlight_amd import kernel
        B, n0, QH, KH, d, dev = self.B, self.n0, self.QH, self.KH, self.d, self.dev
        t_pre = time.perf_counter()
        pos0 = torch.arange(n0, device=dev)
        with torch.no_grad():
            for b in range(B):
                ids = torch.randint(0, self.vocab, (n0,), generator=self.g, device=dev)
                x = self.embed[ids]                                                   # [n0, hidden]
                for w in self.layers:
                    h = self.rms(x, w["n1"])
                    q = self.rope((h @ w["wq"].T).view(n0, QH, d), pos0)
                    kk = self.rope((h @ w["wk"].T).view(n0, KH, d), pos0)
                    vv = (h @ w["wv"].T).view(n0, KH, d)
                    o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None],
                                                       vv.transpose(0, 1)[None], is_causal=True, enable_gqa=True)
                    x = x + o[0].transpose(0, 1).reshape(n0, QH * d) @ w["wo"].T
                    x = x + self.mlp(w, self.rms(x, w["n2"]))
                    if "st" in w:
                        st = w["st"]
                        st.keys[b, :n0] = kk
                        st.vals[b, :n0] = vv
                        st.hash_k.hash_rows(kk[None], out=st.codes[b:b + 1, :n0])
                    else:
                        w["kc"][b, :, :n0] = kk.transpose(0, 1)
                        w["vc"][b, :, :n0] = vv.transpose(0, 1)
                self.tok[b] = (self.rms(x[-1:], self.norm_f) @ self.lm_head.T).float().argmax(dim=-1)[0]
                del x, h, q, kk, vv, o
            for st in self.sparse:
                st.set_length(n0)
        torch.cuda.synchronize()
        return time.perf_counter() - t_pre

    def step_body(self):
        import torch
        B, QH, KH, d, dt = self.B, self.QH, self.KH, self.d, self.dt
        x = self.embed[self.tok]                                                       # [B, hidden]
        for w in self.layers:
            h = self.rms(x, w["n1"])
            q = (h @ w["wq"].T).view(B, QH, d)
            kk = (h @ w["wk"].T).view(B, KH, d)
            vv = (h @ w["wv"].T).view(B, KH, d)
            if "st" in w:
                st = w["st"]          # un-rotated q and k: the step rotates them at its own position
                st.q_in.copy_(q)
                st.k_in.copy_(kk)
                st.v_in.copy_(vv)
                st._launch(self.n_cap)
                o = st.out.reshape(B, QH * d)
            else:
                q = self.rope(q[:, None], self.pos)[:, 0]
                kk = self.rope(kk[:, None], self.pos)[:, 0]
                w["kc"].index_copy_(2, self.pos, kk[:, :, None])
                w["vc"].index_copy_(2, self.pos, vv[:, :, None])
                # dense decode attention as two batched GEMMs per kv head group (the G query heads of
                # a kv head are the G rows of the left operand: no K/V expansion, K and V read once)
                sc = torch.matmul(q.view(B, KH, QH // KH, d), w["kc"].transpose(2, 3)).float() * (d ** -0.5)
                sc = sc.masked_fill((self.col > self.pos)[None, None, None, :], float("-inf"))
                o = torch.matmul(torch.softmax(sc, dim=-1).to(dt), w["vc"]).reshape(B, QH * d)
            x = x + o @ w["wo"].T
            x = x + self.mlp(w, self.rms(x, w["n2"]))
        self.logits.copy_((self.rms(x, self.norm_f) @ self.lm_head.T).float())
        self.tok.copy_(self.logits.argmax(dim=-1))
        self.pos.add_(1)

    def rewind(self, tokens, tok):
        """Undo the last ``tokens`` decoded tokens: positions and lengths go back, the input token is
        restored.  Rows beyond the lengths are simply overwritten by the next steps."""
        self.pos.sub_(tokens)
        self.tok.copy_(tok)
        for st in self.sparse:
            st.seq_lens.sub_(tokens)




def llama_shaped(L=32, hidden=4096, inter=14336, vocab=128256, QH=32, KH=8, theta=5e5, device="cuda:0", seed=0):
    """A random-init bf16 ``nn.Module`` with Llama's module tree and the attribute names the reference's
    modifier reads and patches (spotlight_generation.py:109-126, 298-330): ``config`` (num_attention_heads,
    hidden_size, num_key_value_heads, rope_theta, vocab_size), ``model.embed_tokens``, ``model.layers[i]``
    with ``self_attn.{q,k,v,o}_proj`` + ``self_attn.config``, ``input_layernorm``,
    ``post_attention_layernorm``, ``mlp``; ``model.norm``; ``lm_head``.  Defaults are Llama-3-8B's sizes."""
    import torch
    nn = torch.nn
    dt = torch.bfloat16
    d = hidden // QH
    cfg = types.SimpleNamespace(num_attention_heads=QH, hidden_size=hidden, num_key_value_heads=KH,
                                rope_theta=theta, vocab_size=vocab)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)

    def linear(n_in, n_out):
        lin = nn.Linear(n_in, n_out, bias=False, device="meta", dtype=dt)
        lin.weight = nn.Parameter((torch.randn((n_out, n_in), generator=gen, device=device, dtype=torch.float32) * 0.02).to(dt),
                                  requires_grad=False)
        return lin

    class RMSNorm(nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = nn.Parameter(torch.ones(hidden, device=device, dtype=dt), requires_grad=False)

        def forward(self, x):
            xf = x.float()
            return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).to(dt) * self.weight

    class Attention(nn.Module):
        def __init__(self):
            super().__init__()
            self.config = cfg
            self.q_proj, self.k_proj = linear(hidden, QH * d), linear(hidden, KH * d)
            self.v_proj, self.o_proj = linear(hidden, KH * d), linear(QH * d, hidden)

    class MLP(nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj, self.up_proj, self.down_proj = linear(hidden, inter), linear(hidden, inter), linear(inter, hidden)

        def forward(self, x):
            return self.down_proj(nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))

    class Layer(nn.Module):
        def __init__(self):
            super().__init__()
            self.self_attn, self.mlp = Attention(), MLP()
            self.input_layernorm, self.post_attention_layernorm = RMSNorm(), RMSNorm()

    class Inner(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed_tokens = nn.Embedding(vocab, hidden, device="meta", dtype=dt)
            self.embed_tokens.weight = nn.Parameter(
                (torch.randn((vocab, hidden), generator=gen, device=device, dtype=torch.float32) * 0.02).to(dt), requires_grad=False)
            self.layers = nn.ModuleList([Layer() for _ in range(L)])
            self.norm = RMSNorm()

    class LM(nn.Module):
        def __init__(self):
            super().__init__()
            self.config = cfg
            self.model = Inner()
            self.lm_head = linear(hidden, vocab)

    return LM().eval()
