"""`bench.py --hybrid`: prefill and decode throughput of the hybrid decoder family at layer sizes of real models (random weights), beside
the Qwen2 / Llama engine at equal width, depth, head geometry, FFN width and vocabulary (bf16, 16-bit weights), and the kernels of both
against their rooflines (HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, fp32 vector FMA 157 TFLOP/s).

`--hybrid-design pokepel` measures the Pokepel member (latent attention, retention, PolyNorm MLP, routed experts) beside the family's
Nufalorn member at equal width, depth, heads, FFN width (active per token) and vocabulary, and Pokepel's kernels beside the like
Nufalorn kernels against their rooflines.

`--hybrid-design nepudra` does the same for the Nepudra member (delta-rule recurrence, capped causal and sliding-window attention with gated
heads, bigram embedding, depth-averaged sequential layers).

`--hybrid-design nudorax` measures the Nudorax member (windowed sink attention beside lightning attention in every layer, layer norms on the
sublayers' outputs, sigmoid-routed clamped experts with a gated shared expert) beside the Pokepel member, the family's closest (routed experts
with a shared expert, fixed-decay recurrence, sink attention), at equal width, depth, heads, expert sizes and vocabulary, and its kernels beside
the like Pokepel kernels against their rooflines.

Output: one JSON line {"hybrid_bench": {size: {"hybrid": {...}, "qwen2": {...}, "kernels": [...]}}} (with --hybrid-design pokepel:
{"pokepel": {...}, "nufalorn": {...}, "kernels": [...]})."""
import json
import math
import sys
import time

import torch

HBM, MFMA_BF16, VALU_F32 = 8.0e12, 2.5e15, 157.0e12

SIZES = {
    "w1024": dict(width=1024, layers=8, heads=8, kv=2, hd=128, ff=2816, vocab=32000),
    "w2048": dict(width=2048, layers=16, heads=16, kv=4, hd=128, ff=5632, vocab=32000),
    "w4096": dict(width=4096, layers=8, heads=32, kv=8, hd=128, ff=11008, vocab=32000),
}
PATTERN = ["gla", "attention", "hgrn2", "gla", "gla", "shared", "hgrn2", "gla"]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def hybrid_config(s, chunk=1024):
    layers, owner = [], None
    for i in range(s["layers"]):
        kind = PATTERN[i % len(PATTERN)]
        mlp = {"kind": "dense", "ff": s["ff"]}
        if kind in ("attention", "shared"):
            mx = {"heads": s["heads"], "kv_heads": s["kv"], "dim": s["hd"], "vdim": s["hd"], "scale": s["hd"] ** -0.5, "mask": {"size": chunk},
                  "rot": {"base": 1e6, "dims": s["hd"]}}
            if kind == "shared":
                mx["kv_from"] = owner
            else:
                owner = i
            layers.append({"type": "attention", "mixer": mx, "mlp": mlp})
        elif kind == "gla":
            layers.append({"type": "gla", "mixer": {"heads": s["heads"], "dim": s["hd"] // 2, "vdim": s["hd"], "tau": 16.0}, "mlp": mlp})
        else:
            layers.append({"type": "hgrn2", "mixer": {"heads": s["heads"], "dim": s["hd"] // 2, "vdim": s["hd"]}, "mlp": mlp})
    return {"architecture": "Nufalorn", "layers": layers, "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-5},
            "residual_mult": 0.3, "logit_softcap": 30.0}


def hybrid_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    W = cfg["width"]
    lin = lambda o, i: (torch.randn(o, i, device=dev, generator=g) * i ** -0.5).bfloat16()
    vec = lambda n, k=0.1, off=0.0: (torch.randn(n, device=dev, generator=g) * k + off).bfloat16()
    w = {"embed": (torch.randn(cfg["vocab"], W, device=dev, generator=g)).bfloat16(), "head": lin(cfg["vocab"], W), "final.norm": vec(W)}
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        w[p + "norm1"], w[p + "norm2"] = vec(W), vec(W)
        if L["type"] == "attention":
            w[p + "mix.q"], w[p + "mix.o"] = lin(H * d, W), lin(W, H * dv)
            if "kv_from" not in mx:
                w[p + "mix.k"], w[p + "mix.v"] = lin(mx["kv_heads"] * d, W), lin(mx["kv_heads"] * dv, W)
        elif L["type"] == "hgrn2":
            for n, o in (("q", H * d), ("f", H * d), ("v", H * dv)):
                w[p + "mix." + n] = lin(o, W)
            w[p + "mix.f.b"], w[p + "mix.lower"], w[p + "mix.norm"] = vec(H * d, 0.5), torch.sigmoid(vec(H * d, 1.0).float()).bfloat16(), vec(dv, 0.1, 1.0)
            w[p + "mix.o"] = lin(W, H * dv)
        else:
            for n, o in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv), ("a1", 16)):
                w[p + "mix." + n] = lin(o, W)
            w[p + "mix.a2"], w[p + "mix.a2.b"], w[p + "mix.norm"], w[p + "mix.o"] = lin(H * d, 16), vec(H * d, 1.0, 2.0), vec(dv, 0.1, 1.0), lin(W, H * dv)
        ff = L["mlp"]["ff"]
        w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
    return w


POKEPEL_PATTERN = ["retention", "latent", "latent", "retention", "latent", "latent", "retention", "latent"]


def pokepel_config(s, experts=16, top=4, groups=4, keep=2):
    """Width, depth, heads and vocabulary of `s`; latent attention with a 192-channel latent + 64 rotated channels (one 256-channel cached row
    per token), retention with the recurrent sizes of the GLA layers; the first layer has a PolyNorm MLP of the full FFN width, the others
    `experts` experts of a quarter of it (`top` of them + one shared expert per token: 1.25 x the dense FFN's work)."""
    layers, hd = [], s["hd"]
    for i in range(s["layers"]):
        kind = POKEPEL_PATTERN[i % len(POKEPEL_PATTERN)]
        fe = s["ff"] // 4 // 32 * 32
        mlp = {"kind": "dense", "ff": s["ff"]} if i == 0 else {"kind": "moe", "expert": {"ff": fe}, "shared": {"ff": fe},
                                                               "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
        if kind == "latent":
            mx = {"heads": s["heads"], "dim": hd, "rot_dim": hd // 2, "vdim": hd, "kv_rank": 3 * hd // 2, "scale": (hd + hd // 2) ** -0.5,
                  "rot": {"base": 1e6, "dims": hd // 2, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
            layers.append({"type": "latent_attention", "mixer": mx, "mlp": mlp})
        else:
            mx = {"heads": s["heads"], "dim": hd // 2, "vdim": hd, "decay": [1.0 - 2.0 ** -(5 + h % 8) for h in range(s["heads"])], "rot": {"base": 1e6, "dims": hd // 2}}
            layers.append({"type": "retention", "mixer": mx, "mlp": mlp})
    return {"architecture": "Pokepel", "layers": layers, "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}}


def pokepel_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    W = cfg["width"]
    lin = lambda o, i: (torch.randn(o, i, device=dev, generator=g) * i ** -0.5).bfloat16()
    vec = lambda n, k=0.1, off=0.0: (torch.randn(n, device=dev, generator=g) * k + off).bfloat16()
    w = {"embed": (torch.randn(cfg["vocab"], W, device=dev, generator=g)).bfloat16(), "head": lin(cfg["vocab"], W), "final.norm": vec(W, 0.1, 1.0)}
    for i, L in enumerate(cfg["layers"]):
        p, mx, mlp = f"l{i}.", L["mixer"], L["mlp"]
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        w[p + "norm1"] = vec(W, 0.1, 1.0)
        if L["type"] == "latent_attention":
            dr, R = mx["rot_dim"], mx["kv_rank"]
            for n, (o, k) in {"q": (H * (d + dr), W), "dkv": (R + dr, W), "uk": (H * d, R), "uv": (H * dv, R), "g": (H * dv, W), "o": (W, H * dv)}.items():
                w[p + "mix." + n] = lin(o, k)
            w[p + "mix.dkv.norm"], w[p + "mix.sink"] = vec(R, 0.1, 1.0), vec(H, 1.0)
        else:
            for n, (o, k) in {"q": (H * d, W), "k": (H * d, W), "v": (H * dv, W), "g": (H * dv, W), "o": (W, H * dv)}.items():
                w[p + "mix." + n] = lin(o, k)
        for n in ("rg1", "rg2"):
            w[p + n], w[p + n + ".b"] = lin(W, W), vec(W, 0.5)
        if mlp["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"], w[p + "mlp.act"] = lin(mlp["ff"], W), lin(W, mlp["ff"]), torch.tensor([0.6, 0.3, 0.1, 0.0]).bfloat16()
        else:
            w[p + "mlp.router"] = lin(mlp["router"]["experts"], W)
            for n in [f"e{j}" for j in range(mlp["router"]["experts"])] + ["shared"]:
                f = mlp["expert"]["ff"]
                w[p + f"mlp.{n}.gate"], w[p + f"mlp.{n}.up"], w[p + f"mlp.{n}.down"] = lin(f, W), lin(f, W), lin(W, f)
    return w


NEPUDRA_PATTERN = ["delta", "capped", "delta", "delta", "window", "shared", "delta", "delta"]


def nepudra_config(s, window=1024):
    """Width, depth, attention heads, FFN width and vocabulary of `s`; delta-rule layers with width / 64 heads of 64 key and value channels,
    capped causal attention (one layer in eight reads the keys and values of the capped layer before it) and sliding-window attention
    with normed, YaRN-rotated queries and keys over `window` positions; gelu-gated MLPs; a bigram table of 65521 buckets."""
    layers, owner, hd = [], None, s["hd"]
    for i in range(s["layers"]):
        kind = NEPUDRA_PATTERN[i % len(NEPUDRA_PATTERN)]
        mlp = {"kind": "dense", "ff": s["ff"]}
        if kind == "delta":
            layers.append({"type": "general_delta", "mixer": {"heads": s["width"] // 64, "dim": 64}, "mlp": mlp})
        elif kind in ("capped", "shared"):
            mx = {"heads": s["heads"], "kv_heads": s["kv"], "dim": hd, "vdim": hd, "scale": hd ** -0.5, "softcap": 30.0, "q_temp": {"coef": 0.2, "every": 128}}
            if kind == "shared":
                mx["kv_from"] = owner
            else:
                owner = i
            layers.append({"type": "attention", "mixer": mx, "mlp": mlp})
        else:
            mx = {"heads": s["heads"], "kv_heads": s["kv"], "dim": hd, "vdim": hd, "scale": hd ** -0.5, "mask": {"size": window},
                  "rot": {"base": 1e6, "dims": hd, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
            layers.append({"type": "attention_2", "mixer": mx, "mlp": mlp})
    return {"architecture": "Nepudra", "layers": layers, "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6},
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 8191, "mul_cur": 131}}}


def nepudra_weights(cfg, dev, seed=0, rank=64):
    g = torch.Generator(device=dev).manual_seed(seed)
    W = cfg["width"]
    lin = lambda o, i: (torch.randn(o, i, device=dev, generator=g) * i ** -0.5).bfloat16()
    vec = lambda n, k=0.1, off=0.0: (torch.randn(n, device=dev, generator=g) * k + off).bfloat16()
    one = lambda: torch.tensor(1.0, device=dev).bfloat16()
    w = {"embed": torch.randn(cfg["vocab"], W, device=dev, generator=g).bfloat16(), "head": lin(cfg["vocab"], W), "final.norm": one(),
         "bigram": (torch.randn(cfg["embedding"]["bigram"]["buckets"] + 1, W, device=dev, generator=g) * 0.5).bfloat16()}
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        H, d = mx["heads"], mx["dim"]
        w[p + "norm1"], w[p + "norm2"] = one(), one()
        c = torch.full((i + 2,), 0.2 / (i + 1), device=dev)
        c[-1] = 0.8
        w[p + "dwa"] = c.bfloat16()
        if L["type"] == "general_delta":
            for n in ("r", "k", "v", "a", "g"):
                w[p + "mix." + n] = lin(H * d, W)
            w[p + "mix.a.b"], w[p + "mix.w1"], w[p + "mix.w2"], w[p + "mix.w0"] = vec(H * d, 0.5), lin(rank, W), lin(H * d, rank), vec(H * d, 1.0)
            w[p + "mix.norm"], w[p + "mix.o"] = vec(H * d, 0.1, 1.0), lin(W, H * d)
        else:
            G, dv = mx["kv_heads"], mx["vdim"]
            w[p + "mix.q"], w[p + "mix.q.b"], w[p + "mix.g"], w[p + "mix.o"] = lin(H * d, W), vec(H * d), lin(H, W), lin(W, H * dv)
            if "kv_from" not in mx:
                w[p + "mix.k"], w[p + "mix.k.b"], w[p + "mix.v"], w[p + "mix.v.b"] = lin(G * d, W), vec(G * d), lin(G * dv, W), vec(G * dv)
            if L["type"] == "attention":
                w[p + "mix.o.b"] = vec(W)
            else:
                w[p + "mix.q.norm"], w[p + "mix.k.norm"] = vec(d, 0.1, 1.0), vec(d, 0.1, 1.0)
        ff = L["mlp"]["ff"]
        w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
    return w


def nudorax_config(s, experts=16, top=4, groups=4, keep=2, window=1024):
    """Width, depth, heads and vocabulary of `s`; every layer runs grouped-query attention over a sliding window (learned sinks, queries and keys
    normed over all heads, wavelength-scaled rotary steps) beside lightning attention with the recurrent sizes of Pokepel's retention layers,
    and a mixture of `experts` clamped gated experts of a quarter of the FFN width (`top` of them + one gated shared expert per token)."""
    layers, hd = [], s["hd"]
    fe = s["ff"] // 4 // 32 * 32
    for i in range(s["layers"]):
        left = {"heads": s["heads"], "kv_heads": s["kv"], "dim": hd, "vdim": hd, "scale": hd ** -0.5, "mask": {"size": window},
                "rot": {"base": 1e6, "dims": hd, "scaling": {"factor": 16.0, "low": 1.0, "high": 4.0, "original": 8192}}}
        right = {"heads": s["heads"], "dim": hd // 2, "vdim": hd, "decay": [1.0 - 2.0 ** -(5 + h % 8) for h in range(s["heads"])]}
        mlp = {"kind": "moe", "expert": {"ff": fe, "limit": 7.0}, "shared": {"ff": fe, "limit": 7.0},
               "router": {"experts": experts, "top": top, "scale": 2.5, "groups": {"count": groups, "keep": keep}}}
        layers.append({"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 1.0, "right_scale": 1.0}, "mlp": mlp})
    return {"architecture": "Nudorax", "layers": layers, "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}, "embedding": {"scale": s["width"] ** 0.5},
            "logit_softcap": 30.0}


def nudorax_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    W = cfg["width"]
    lin = lambda o, i: (torch.randn(o, i, device=dev, generator=g) * i ** -0.5).bfloat16()
    vec = lambda n, k=0.1, off=0.0: (torch.randn(n, device=dev, generator=g) * k + off).bfloat16()
    w = {"embed": (torch.randn(cfg["vocab"], W, device=dev, generator=g) * W ** -0.5).bfloat16(), "final.norm": vec(W, 0.1, 1.0)}
    for i, L in enumerate(cfg["layers"]):
        p, a, b, mlp = f"l{i}.", L["mixer"]["left"], L["mixer"]["right"], L["mlp"]
        w[p + "norm1"], w[p + "norm2"] = vec(W, 0.1, 1.0), vec(W, 0.1, 1.0)
        H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        q = p + "mix.left."
        for n, (o, k) in {"q": (H * d, W), "k": (G * d, W), "v": (G * dv, W), "o": (W, H * dv)}.items():
            w[q + n] = lin(o, k)
        w[q + "q.norm"], w[q + "k.norm"], w[q + "sink"] = vec(H * d, 0.1, 1.0), vec(G * d, 0.1, 1.0), vec(H, 1.0)
        H, d, dv = b["heads"], b["dim"], b["vdim"]
        q = p + "mix.right."
        for n, (o, k) in {"q": (H * d, W), "k": (H * d, W), "v": (H * dv, W), "g": (H * dv, W), "o": (W, H * dv)}.items():
            w[q + n] = lin(o, k)
        w[q + "norm"] = vec(H * dv, 0.1, 1.0)
        w[p + "mlp.router"], w[p + "mlp.shared.sg"] = lin(mlp["router"]["experts"], W), lin(1, W)
        for n in [f"e{j}" for j in range(mlp["router"]["experts"])] + ["shared"]:
            f = mlp["expert"]["ff"]
            w[p + f"mlp.{n}.gate"], w[p + f"mlp.{n}.up"], w[p + f"mlp.{n}.down"] = lin(f, W), lin(f, W), lin(W, f)
    return w


def timed(fn, reps=5, warm=2, graph=False):
    """Seconds per call.  graph: the calls are captured into one HIP graph and the replay is timed, so the figure is the kernels' own
    time and not the host's launch path (what a graph-replayed step pays)."""
    for _ in range(warm):
        fn()
    if graph:
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(reps):
                fn()
        inner, fn, reps = reps, g.replay, 3
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * inner) * 1e-3
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e-3


def bench_hybrid_engine(s, dev, prompt, batch, steps, design="nufalorn"):
    from .hybrid import HybridConfig, HybridModel
    from .scheduler import ServingEngine
    make_cfg, make_w = {"pokepel": (pokepel_config, pokepel_weights), "nepudra": (nepudra_config, nepudra_weights),
                        "nudorax": (nudorax_config, nudorax_weights)}.get(design, (hybrid_config, hybrid_weights))
    cfg = make_cfg(s)
    model = HybridModel(HybridConfig.from_json(cfg), make_w(cfg, dev), torch.bfloat16, dev)
    eng = ServingEngine(model, max_tokens=batch * (prompt + 8 * (steps + 3) + 128), max_seqs=batch, max_step_tokens=1 << 20)
    g = torch.Generator().manual_seed(1)
    toks = lambda n: torch.randint(0, s["vocab"], (n,), generator=g).tolist()
    out = {}
    # prefill: one sequence of `prompt` tokens per step (released afterwards), then `batch` sequences in one step
    def one():
        eng.run_step([("p", toks(prompt), [prompt - 1])]); eng.release("p")
    t = timed(one, reps=3, warm=1)
    out["prefill_1x%d_tok_s" % prompt] = round(prompt / t)
    ids = [f"s{i}" for i in range(batch)]
    torch.cuda.synchronize(); t0 = time.time()
    eng.run_step([(i, toks(prompt), [prompt - 1]) for i in ids])
    torch.cuda.synchronize()
    out["prefill_%dx%d_tok_s" % (batch, prompt)] = round(batch * prompt / (time.time() - t0))
    # decode: `batch` live sequences, one token each per step
    for b in sorted({1, min(8, batch), batch}):
        step = lambda: eng.run_step([(i, [7], [0]) for i in ids[:b]])
        for graph in (False, True):
            eng.use_graphs = graph
            t = timed(step, reps=steps, warm=3)
            out["decode_b%d_%s_tok_s" % (b, "graph" if graph else "eager")] = round(b / t)
            out["decode_b%d_%s_ms" % (b, "graph" if graph else "eager")] = round(t * 1e3, 3)
    for i in ids:
        eng.release(i)
    return out, model, eng


def bench_qwen2_engine(s, dev, prompt, batch, steps):
    from . import model as M
    cfg = M.ModelConfig("qwen2-like", s["layers"], s["width"], s["heads"], s["kv"], s["hd"], s["ff"], s["vocab"], max_pos=prompt + 8 * steps + 256)
    w = M.synth_model(cfg, "fp16", dev, seed=0)
    page = 64
    per = (prompt + 8 * steps + 128 + page - 1) // page
    eng = M.DecoderEngine(cfg, w, kv_int8=False, page=page, num_blocks=per * batch, max_batch=max(batch, 1), max_seq_len=per * page, device=dev,
                          dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(1)
    toks = lambda n: torch.randint(0, s["vocab"], (n,), generator=g).tolist()
    bt = torch.arange(per * batch, dtype=torch.int32).reshape(batch, per)
    out = {}
    t = timed(lambda: eng.prefill([toks(prompt)], bt[:1], chunk=512), reps=3, warm=1)
    out["prefill_1x%d_tok_s" % prompt] = round(prompt / t)
    torch.cuda.synchronize(); t0 = time.time()
    eng.prefill([toks(prompt) for _ in range(batch)], bt, chunk=512)
    torch.cuda.synchronize()
    out["prefill_%dx%d_tok_s" % (batch, prompt)] = round(batch * prompt / (time.time() - t0))
    for b in sorted({1, min(8, batch), batch}):
        eng.set_inputs([7] * b, [prompt] * b, bt[:b])
        eng.capture(b)
        t = timed(lambda: eng.replay(b, 1), reps=steps, warm=3)
        out["decode_b%d_graph_tok_s" % b] = round(b / t)
        out["decode_b%d_graph_ms" % b] = round(t * 1e3, 3)
    return out, eng


def kernel_table(s, dev, prompt):
    """Time the kernels of both families at this size; roofline time = max(bytes / HBM, flops / peak of the unit that does them)."""
    from . import hybrid_ops as hops, ops, quant
    rows = []
    timed_k = lambda fn: timed(fn, reps=10, warm=2, graph=True)
    g = torch.Generator(device=dev).manual_seed(3)
    bf = lambda *sh: torch.randn(*sh, device=dev, generator=g).bfloat16()
    W, H, G, hd, ff = s["width"], s["heads"], s["kv"], s["hd"], s["ff"]

    def add(family, name, shape, t, nbytes, flops, peak):
        roof = max(nbytes / HBM, flops / peak)
        rows.append({"family": family, "kernel": name, "shape": shape, "us": round(t * 1e6, 1), "roofline_us": round(roof * 1e6, 2),
                     "x_roofline": round(t / roof, 1)})

    # linears: the FFN up projection (N = 2 ff gated) and the attention output projection
    for M_ in (prompt, 8, 1):
        x = bf(M_, W)
        wgu = hops.group_gate_up(bf(ff, W), bf(ff, W))
        t = timed_k(lambda: hops.dense_linear(x, wgu, gated=True, act=hops.ACT_RELU))
        add("hybrid", "dense_linear gated", f"M={M_} N={2 * ff} K={W}", t, 2 * ff * W * 2 + M_ * (W + ff) * 2, 2.0 * M_ * 2 * ff * W, MFMA_BF16)
        pw = quant.pack_fp16(quant.interleave_gate_up(bf(W, 2 * ff), -1))
        t = timed_k(lambda: ops.linear(x, pw, None, epilogue=1))
        add("qwen2", "linear W16 silu_mul", f"M={M_} N={2 * ff} K={W}", t, 2 * ff * W * 2 + M_ * (W + ff) * 2, 2.0 * M_ * 2 * ff * W, MFMA_BF16)
        xo, wo = bf(M_, H * hd), bf(W, H * hd)
        t = timed_k(lambda: hops.dense_linear(xo, wo, out_dtype=torch.float32))
        add("hybrid", "dense_linear", f"M={M_} N={W} K={H * hd}", t, W * H * hd * 2 + M_ * (H * hd * 2 + W * 4), 2.0 * M_ * W * H * hd, MFMA_BF16)
        pwo = quant.pack_fp16(bf(H * hd, W))
        t = timed_k(lambda: ops.linear(xo, pwo))
        add("qwen2", "linear W16", f"M={M_} N={W} K={H * hd}", t, W * H * hd * 2 + M_ * (H * hd + W) * 2, 2.0 * M_ * W * H * hd, MFMA_BF16)
    # norms
    for M_ in (prompt, 8):
        x, a, b = [torch.randn(M_, W, device=dev, generator=g) for _ in range(3)]
        w1, w2 = bf(W), bf(W)
        t = timed_k(lambda: hops.residual_norm(x, a, b, 0.3, w1, w2, 1e-5, weight_offset=1.0))
        add("hybrid", "residual + 2 norms (fp32 stream)", f"M={M_} W={W}", t, M_ * W * (4 * 4 + 2 * 2), 0, VALU_F32)
        xh, rh, wh = bf(M_, W).to(torch.bfloat16), bf(M_, W), bf(W)
        t = timed_k(lambda: ops.add_rmsnorm(xh, rh, wh, 1e-6))
        add("qwen2", "add + rmsnorm (16-bit stream)", f"M={M_} W={W}", t, M_ * W * 2 * 4, 0, VALU_F32)
    # attention: prefill rows over a chunk-local mask vs plain causal rows; decode at a context of `prompt`
    page, chunk = 64, 1024
    nblk = (prompt + page - 1) // page + 1
    geom = hops.attn_geometry(H, G, hd, hd, hd, 0, 0, page, nblk, nblk)
    kc, vc = bf(nblk, G, page, hd), bf(nblk, G, page, hd)
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).reshape(1, nblk)
    vf = torch.ones(hd // 2, device=dev) * 1e-3
    sink0 = torch.zeros(H, device=dev)
    for T_, name in ((prompt, "prefill"), (1, "decode")):
        pos = (torch.arange(T_, dtype=torch.int32, device=dev) if T_ > 1 else torch.tensor([prompt - 1], dtype=torch.int32, device=dev))
        seq = torch.zeros(T_, dtype=torch.int32, device=dev)
        q = torch.randn(T_, H * hd, device=dev, generator=g)
        t = timed_k(lambda: hops.attn_rows(q, hd ** -0.5, geom, chunk, sink0, vf, pos, seq, bt, kc, vc, H, hd))
        keys = float(sum(min(int(p) % chunk + 1, chunk) for p in pos.tolist()))
        add("hybrid", f"attn_rows {name} (chunk {chunk})", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t,
            min(prompt, chunk if T_ == 1 else prompt) * G * hd * 2 * 2 + T_ * H * hd * 6, 4.0 * keys * H * hd, MFMA_BF16)
        if T_ > 1:
            t0 = torch.arange(0, T_, 16, dtype=torch.int32, device=dev)
            tn = torch.full_like(t0, 16)
            t = timed_k(lambda: hops.attn_tiles(q, hd ** -0.5, geom, chunk, sink0, vf, pos, seq, bt, t0, tn, kc, vc, H, hd))
            add("hybrid", f"attn_tiles {name} (chunk {chunk}, MFMA)", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t,
                prompt * G * hd * 2 * 2 + T_ * H * hd * 6, 4.0 * keys * H * hd, MFMA_BF16)
        kvb = torch.randn(nblk, 2, G, page, hd, device=dev, generator=g).bfloat16()
        qh = bf(T_, H, hd)
        if T_ > 1:
            q_len = 512
            posr = torch.arange(q_len, dtype=torch.int32, device=dev) + (prompt - q_len)
            qh = bf(q_len, H, hd)
            t = timed_k(lambda: ops.paged_attention_rows(qh, kvb, None, bt, posr, G, page, q_len, nblk * page))
            keysq = float(sum(int(p) + 1 for p in posr.tolist()))
            add("qwen2", "paged_attn_rows prefill (last 512 rows, causal)", f"T={q_len} H={H} G={G} hd={hd} ctx={prompt}", t,
                prompt * G * hd * 2 * 2 + q_len * H * hd * 4, 4.0 * keysq * H * hd, MFMA_BF16)
        else:
            sl = torch.tensor([prompt], dtype=torch.int32, device=dev)
            t = timed_k(lambda: ops.paged_decode_attention(qh, kvb, None, bt, sl, G, page, nblk * page))
            add("qwen2", "paged_decode_attn", f"B=1 H={H} G={G} hd={hd} ctx={prompt}", t, prompt * G * hd * 2 * 2, 4.0 * prompt * H * hd, MFMA_BF16)
    # recurrence: no counterpart in the Qwen2 family
    d = hd // 2
    for T_, name in ((prompt, "prefill"), (8, "decode b=8")):
        nseq = 1 if T_ > 8 else 8
        proj = torch.randn(T_, 2 * H * d + 2 * H * hd, device=dev, generator=g)
        z = torch.randn(T_, H * d, device=dev, generator=g)
        rs = torch.arange(0, T_ + 1, T_ // nseq, dtype=torch.int32, device=dev)
        slot = torch.arange(nseq, dtype=torch.int32, device=dev)
        fp = torch.ones(nseq, dtype=torch.int32, device=dev)
        state = torch.zeros(nseq, H, d, hd, device=dev)
        t = timed_k(lambda: hops.scan(hops.SCAN_GLA, proj, 0, H * d, 2 * H * d, z, None, None, 16.0, d ** -0.5, H, d, hd, rs, slot, fp, state, torch.bfloat16))
        add("hybrid", f"scan GLA {name}", f"T={T_} H={H} dim={d} vdim={hd}", t, T_ * (3 * H * d + 2 * H * hd) * 4 + 2 * nseq * H * d * hd * 4,
            4.0 * T_ * H * d * hd, VALU_F32)
    return rows


def kernel_table_pokepel(s, dev, prompt):
    """Pokepel's kernels at this size beside the like kernels of the Nufalorn member, against max(bytes / HBM, flops / peak of the unit)."""
    from . import hybrid_ops as hops
    rows = []
    timed_k = lambda fn: timed(fn, reps=10, warm=2, graph=True)
    g = torch.Generator(device=dev).manual_seed(3)
    bf = lambda *sh: torch.randn(*sh, device=dev, generator=g).bfloat16()
    f32 = lambda *sh: torch.randn(*sh, device=dev, generator=g)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    W, H, G, hd, ff = s["width"], s["heads"], s["kv"], s["hd"], s["ff"]
    cfg = pokepel_config(s)
    lat = next(L["mixer"] for L in cfg["layers"] if L["type"] == "latent_attention")
    moe = next(L["mlp"] for L in cfg["layers"] if L["mlp"]["kind"] == "moe")
    R, dr, fe, E, top = lat["kv_rank"], lat["rot_dim"], moe["expert"]["ff"], moe["router"]["experts"], moe["router"]["top"]
    dpad = -(-(R + dr) // 32) * 32

    def add(family, name, shape, t, nbytes, flops, peak):
        roof = max(nbytes / HBM, flops / peak)
        rows.append({"family": family, "kernel": name, "shape": shape, "us": round(t * 1e6, 1), "roofline_us": round(roof * 1e6, 2),
                     "x_roofline": round(t / roof, 1)})

    page = 64
    nblk = (prompt + page - 1) // page + 1
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).reshape(1, nblk)
    sink = f32(H)
    # attention: one cached row of dpad channels per token for all heads (values = its first R channels) against grouped-query pages
    geom = hops.attn_geometry(H, 1, dpad, R, 0, 0, 0, page, nblk, nblk, v_ld=dpad)
    ngeom = hops.attn_geometry(H, G, hd, hd, hd, 0, 0, page, nblk, nblk)
    kc = bf(nblk, 1, page, dpad)
    nk, nv = bf(nblk, G, page, hd), bf(nblk, G, page, hd)
    vf = torch.ones(hd // 2, device=dev) * 1e-3
    for T_, name in ((prompt, "prefill"), (1, "decode")):
        pos = torch.arange(T_, dtype=torch.int32, device=dev) if T_ > 1 else i32([prompt - 1])
        seq = torch.zeros(T_, dtype=torch.int32, device=dev)
        q, nq = f32(T_, H * dpad), f32(T_, H * hd)
        keys = float(sum(int(p) + 1 for p in pos.tolist()))
        ctx = prompt
        if T_ > 1:
            t0 = torch.arange(0, T_, 16, dtype=torch.int32, device=dev)
            tn = torch.full_like(t0, 16)
            t = timed_k(lambda: hops.attn_tiles(q, 0.07, geom, 0, sink, None, pos, seq, bt, t0, tn, kc, kc, H, R))
            add("pokepel", "attn_tiles latent prefill (causal, MFMA)", f"T={T_} H={H} row={dpad} rank={R} ctx={ctx}", t, ctx * dpad * 2 + T_ * H * (dpad * 4 + R * 2),
                2.0 * keys * H * (dpad + R), MFMA_BF16)
            t = timed_k(lambda: hops.attn_tiles(nq, hd ** -0.5, ngeom, 0, sink, vf, pos, seq, bt, t0, tn, nk, nv, H, hd))
            add("nufalorn", "attn_tiles prefill (causal, MFMA)", f"T={T_} H={H} G={G} hd={hd} ctx={ctx}", t, ctx * G * hd * 2 * 2 + T_ * H * hd * 6, 4.0 * keys * H * hd, MFMA_BF16)
        else:
            t = timed_k(lambda: hops.attn_rows(q, 0.07, geom, 0, sink, None, pos, seq, bt, kc, kc, H, R))
            add("pokepel", "attn_rows latent decode", f"T=1 H={H} row={dpad} rank={R} ctx={ctx}", t, ctx * dpad * 2, 2.0 * keys * H * (dpad + R), MFMA_BF16)
            t = timed_k(lambda: hops.attn_rows(nq, hd ** -0.5, ngeom, 0, sink, vf, pos, seq, bt, nk, nv, H, hd))
            add("nufalorn", "attn_rows decode", f"T=1 H={H} G={G} hd={hd} ctx={ctx}", t, ctx * G * hd * 2 * 2, 4.0 * keys * H * hd, MFMA_BF16)
    # before the scores: norm + turn + page write + query split, against turn + value norm + page write
    lgeom = hops.latent_geometry(H, hd, dr, R, dpad, dr, page, nblk, nblk)
    freq = torch.ones(dr // 2, device=dev) * 1e-3
    for T_ in (prompt, 8):
        pos, seq = torch.arange(T_, dtype=torch.int32, device=dev), torch.zeros(T_, dtype=torch.int32, device=dev)
        proj, qn, qabs, cw = f32(T_, H * (hd + dr) + R + dr), bf(T_, H * hd), f32(T_, H * dpad), bf(R)
        t = timed_k(lambda: hops.latent_prep(proj, H * (hd + dr), lgeom, freq, 1.2, cw, 1e-6, pos, seq, bt, qn, qabs, kc.view(nblk, page, dpad)))
        add("pokepel", "latent_prep", f"T={T_} H={H}", t, T_ * (H * (hd + dr) * 4 + H * hd * 2 + H * (dpad - R) * 4 + dpad * 2), 0, VALU_F32)
        qkv = f32(T_, (H + 2 * G) * hd)
        t = timed_k(lambda: hops.attn_prep(qkv, H * hd, (H + G) * hd, ngeom, freq.repeat(2)[: hd // 2], vf, True, 1e-5, pos, seq, bt, nk, nv))
        add("nufalorn", "attn_prep", f"T={T_} H={H} G={G}", t, T_ * ((H + 2 * G) * hd * 4 + H * hd * 4 + 2 * G * hd * 2), 0, VALU_F32)
    # per-head products around the attention (key up-projection on the query side, value up-projection) against a dense linear of the same work
    for T_ in (prompt, 8):
        qn, wuk = bf(T_, H * hd), bf(H, R, hd)
        out = f32(T_, H * dpad)
        t = timed_k(lambda: hops.dense_grouped(qn, wuk, x_step=hd, y_step=dpad, out_dtype=torch.float32, out=out))
        add("pokepel", "dense_grouped heads (absorb)", f"M={T_} G={H} N={R} K={hd}", t, H * R * hd * 2 + T_ * H * (hd * 2 + R * 4), 2.0 * T_ * H * R * hd, MFMA_BF16)
        ol, wuv = bf(T_, H * R), bf(H, hd, R)
        t = timed_k(lambda: hops.dense_grouped(ol, wuv, x_step=R, y_step=hd, out_dtype=torch.float32))
        add("pokepel", "dense_grouped heads (values)", f"M={T_} G={H} N={hd} K={R}", t, H * R * hd * 2 + T_ * H * (R * 2 + hd * 4), 2.0 * T_ * H * R * hd, MFMA_BF16)
        x, wd = bf(T_, H * hd), bf(R, H * hd)
        t = timed_k(lambda: hops.dense_linear(x, wd, out_dtype=torch.float32))
        add("nufalorn", "dense_linear", f"M={T_} N={R} K={H * hd}", t, H * R * hd * 2 + T_ * (H * hd * 2 + R * 4), 2.0 * T_ * H * R * hd, MFMA_BF16)
    # experts: routing + sorting, both grouped linears, weighted sum, against the dense gated MLP of the same active width
    for T_ in (prompt, 8, 1):
        h = bf(T_, W)
        z = f32(T_, E) * 2
        gr = moe["router"]["groups"]
        t = timed_k(lambda: hops.moe_route_sorted(z, E, gr["count"], gr["keep"], top))
        add("pokepel", "moe route + sort", f"T={T_} E={E} top={top}", t, T_ * (E * 4 + top * 16), 0, VALU_F32)
        ids, wts = hops.moe_route(z, gr["count"], gr["keep"], top)
        offs, src, place, tiles = hops.moe_align(ids, E)
        n = T_ * top
        used = len(set(ids.flatten().tolist()))
        wgu = torch.stack([hops.group_gate_up(bf(fe, W), bf(fe, W)) for _ in range(E)]).contiguous()
        t = timed_k(lambda: hops.dense_grouped(h, wgu, offs=offs, gather=src, tiles=tiles, rows=n, gated=True, act=hops.ACT_SILU))
        add("pokepel", "dense_grouped experts gated", f"M={T_}x{top} E={E} ({used} used) N={2 * fe} K={W}", t, used * 2 * fe * W * 2 + n * (W + fe) * 2, 2.0 * n * 2 * fe * W, MFMA_BF16)
        a, wdn = bf(n, fe), bf(E, W, fe)
        t = timed_k(lambda: hops.dense_grouped(a, wdn, offs=offs, tiles=tiles, rows=n, out_dtype=torch.float32))
        add("pokepel", "dense_grouped experts down", f"M={T_}x{top} E={E} ({used} used) N={W} K={fe}", t, used * fe * W * 2 + n * (fe * 2 + W * 4), 2.0 * n * fe * W, MFMA_BF16)
        y, extra = f32(n, W), f32(T_, W)
        xs_, as_, gt_, w1_ = f32(T_, W), f32(T_, W), f32(T_, 2 * W), bf(W)
        t = timed_k(lambda: hops.residual_norm(xs_, as_, hops.MoeSum(y, place, wts, extra), 1.0, w1_, None, 1e-6, gate=gt_))
        add("pokepel", "gated residual + mixture sum + norm", f"T={T_} top={top} W={W}", t, (n + 7 * T_) * W * 4 + T_ * W * 2, 0, VALU_F32)
        ffa = fe * top
        wd_gu = hops.group_gate_up(bf(ffa, W), bf(ffa, W))
        t = timed_k(lambda: hops.dense_linear(h, wd_gu, gated=True, act=hops.ACT_RELU))
        add("nufalorn", "dense_linear gated", f"M={T_} N={2 * ffa} K={W}", t, 2 * ffa * W * 2 + T_ * (W + ffa) * 2, 2.0 * T_ * 2 * ffa * W, MFMA_BF16)
        wdd, aa = bf(W, ffa), bf(T_, ffa)
        t = timed_k(lambda: hops.dense_linear(aa, wdd, out_dtype=torch.float32))
        add("nufalorn", "dense_linear down", f"M={T_} N={W} K={ffa}", t, ffa * W * 2 + T_ * (ffa * 2 + W * 4), 2.0 * T_ * ffa * W, MFMA_BF16)
    # PolyNorm, gated residual + norm
    for T_ in (prompt, 8):
        z = f32(T_, ff)
        t = timed_k(lambda: hops.polynorm(z, (0.6, 0.3, 0.1, 0.0), 1e-6, torch.bfloat16))
        add("pokepel", "polynorm", f"M={T_} ff={ff}", t, T_ * ff * 6, 0, VALU_F32)
        x, a, b, gt = f32(T_, W), f32(T_, W), f32(T_, W), f32(T_, 2 * W)
        w1, w2 = bf(W), bf(W)
        t = timed_k(lambda: hops.residual_norm(x, a, b, 1.0, w1, None, 1e-6, gate=gt))
        add("pokepel", "gated residual + norm (fp32 stream)", f"M={T_} W={W}", t, stream_bytes(T_, W, 6, 1), 0, VALU_F32)
        t = timed_k(lambda: hops.residual_norm(x, a, b, 0.3, w1, w2, 1e-5, weight_offset=1.0))
        add("nufalorn", "residual + 2 norms (fp32 stream)", f"M={T_} W={W}", t, stream_bytes(T_, W, 4, 2), 0, VALU_F32)
    # recurrence: fixed decay (after the separate turn of q and k) against the gated-linear-attention scan
    d = hd // 2
    for T_, name in ((prompt, "prefill"), (8, "decode b=8")):
        nseq = 1 if T_ > 8 else 8
        proj = f32(T_, 2 * H * d + 2 * H * hd)
        z = f32(T_, H * d)
        rs = torch.arange(0, T_ + 1, T_ // nseq, dtype=torch.int32, device=dev)
        slot, fp = torch.arange(nseq, dtype=torch.int32, device=dev), torch.ones(nseq, dtype=torch.int32, device=dev)
        state = torch.zeros(nseq, H, d, hd, device=dev)
        decay = torch.full((H,), 0.97, device=dev)
        nb, fl = T_ * (2 * H * d + 2 * H * hd) * 4 + 2 * nseq * H * d * hd * 4, 4.0 * T_ * H * d * hd
        t = timed_k(lambda: hops.scan(hops.SCAN_FIXED, proj, 0, H * d, 2 * H * d, None, decay, None, 1.0, 1.0, H, d, hd, rs, slot, fp, state, torch.bfloat16))
        add("pokepel", f"scan retention {name}", f"T={T_} H={H} dim={d} vdim={hd}", t, nb, fl, VALU_F32)
        t = timed_k(lambda: hops.scan(hops.SCAN_GLA, proj, 0, H * d, 2 * H * d, z, None, None, 16.0, d ** -0.5, H, d, hd, rs, slot, fp, state, torch.bfloat16))
        add("nufalorn", f"scan GLA {name}", f"T={T_} H={H} dim={d} vdim={hd}", t, nb + T_ * H * d * 4, fl, VALU_F32)
        pos = torch.arange(T_, dtype=torch.int32, device=dev)
        fr = torch.ones(d // 2, device=dev) * 1e-3
        t = timed_k(lambda: hops.rotary(proj, [(0, H, d, 1.0), (H * d, H, d, d ** -0.5)], d, 1, fr, 1.0, pos))
        add("pokepel", f"rotary q, k {name}", f"T={T_} H={H} dim={d}", t, T_ * 2 * H * d * 8, 0, VALU_F32)
    return rows


def kernel_table_nepudra(s, dev, prompt):
    """Nepudra's kernels at this size beside the like kernels of the Nufalorn member, against max(bytes / HBM, flops / peak of the unit)."""
    from . import hybrid_ops as hops
    rows = []
    timed_k = lambda fn: timed(fn, reps=10, warm=2, graph=True)
    g = torch.Generator(device=dev).manual_seed(3)
    bf = lambda *sh: torch.randn(*sh, device=dev, generator=g).bfloat16()
    f32 = lambda *sh: torch.randn(*sh, device=dev, generator=g)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    W, H, G, hd, ff, L = s["width"], s["heads"], s["kv"], s["hd"], s["ff"], s["layers"]

    def add(family, name, shape, t, nbytes, flops, peak):
        roof = max(nbytes / HBM, flops / peak)
        rows.append({"family": family, "kernel": name, "shape": shape, "us": round(t * 1e6, 1), "roofline_us": round(roof * 1e6, 2),
                     "x_roofline": round(t / roof, 1)})

    page, window = 64, 1024
    nblk = (prompt + page - 1) // page + 1
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).reshape(1, nblk)
    geom = hops.attn_geometry(H, G, hd, hd, hd, 1, 0, page, nblk, nblk)
    ngeom = hops.attn_geometry(H, G, hd, hd, hd, 0, 0, page, nblk, nblk)
    kc, vc = bf(nblk, G, page, hd), bf(nblk, G, page, hd)
    vf = torch.ones(hd // 2, device=dev) * 1e-3
    sink0 = torch.zeros(H, device=dev)
    # attention: sliding window with gated heads against the block mask with sink and turned values; capped causal against plain causal
    for T_, name in ((prompt, "prefill"), (1, "decode")):
        pos = torch.arange(T_, dtype=torch.int32, device=dev) if T_ > 1 else i32([prompt - 1])
        seq = torch.zeros(T_, dtype=torch.int32, device=dev)
        q = f32(T_, H * hd + H)
        og = q[:, H * hd:]
        kw = float(sum(min(int(p) + 1, window) for p in pos.tolist()))
        kb = float(sum(int(p) % window + 1 for p in pos.tolist()))
        kc_ = float(sum(int(p) + 1 for p in pos.tolist()))
        byt = lambda keys: min(prompt, keys) * G * hd * 2 * 2 + T_ * H * hd * 6
        if T_ > 1:
            t0 = torch.arange(0, T_, 16, dtype=torch.int32, device=dev)
            tn = torch.full_like(t0, 16)
            t = timed_k(lambda: hops.attn_tiles(q, hd ** -0.5, geom, 0, None, None, pos, seq, bt, t0, tn, kc, vc, H, hd, window=window, out_gate=og))
            add("nepudra", f"attn_tiles prefill (window {window}, gated heads)", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t, byt(prompt), 4.0 * kw * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_tiles(q, hd ** -0.5, ngeom, window, sink0, vf, pos, seq, bt, t0, tn, kc, vc, H, hd))
            add("nufalorn", f"attn_tiles prefill (block mask {window}, sink, turned values)", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t, byt(prompt), 4.0 * kb * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_tiles(q, hd ** -0.5, geom, 0, None, None, pos, seq, bt, t0, tn, kc, vc, H, hd, softcap=30.0, out_gate=og))
            add("nepudra", "attn_tiles prefill (causal, capped scores, gated heads)", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t, byt(prompt), 4.0 * kc_ * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_tiles(q, hd ** -0.5, ngeom, 0, sink0, vf, pos, seq, bt, t0, tn, kc, vc, H, hd))
            add("nufalorn", "attn_tiles prefill (causal, sink, turned values)", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t, byt(prompt), 4.0 * kc_ * H * hd, MFMA_BF16)
        else:
            t = timed_k(lambda: hops.attn_rows(q, hd ** -0.5, geom, 0, None, None, pos, seq, bt, kc, vc, H, hd, window=window, out_gate=og))
            add("nepudra", f"attn_rows decode (window {window}, gated heads)", f"T=1 H={H} G={G} hd={hd} ctx={prompt}", t, byt(window), 4.0 * kw * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_rows(q, hd ** -0.5, ngeom, window, sink0, vf, pos, seq, bt, kc, vc, H, hd))
            add("nufalorn", f"attn_rows decode (block mask {window})", f"T=1 H={H} G={G} hd={hd} ctx={prompt}", t, byt(window), 4.0 * kb * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_rows(q, hd ** -0.5, geom, 0, None, None, pos, seq, bt, kc, vc, H, hd, softcap=30.0, out_gate=og))
            add("nepudra", "attn_rows decode (causal, capped scores, gated heads)", f"T=1 H={H} G={G} hd={hd} ctx={prompt}", t, byt(prompt), 4.0 * kc_ * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_rows(q, hd ** -0.5, ngeom, 0, sink0, vf, pos, seq, bt, kc, vc, H, hd))
            add("nufalorn", "attn_rows decode (causal)", f"T=1 H={H} G={G} hd={hd} ctx={prompt}", t, byt(prompt), 4.0 * kc_ * H * hd, MFMA_BF16)
    # before the scores: head norms + scaled turn + page write, and temperature + page write, against turn + value norm + page write
    freq = torch.ones(hd // 2, device=dev) * 1e-3
    qn, kn = bf(hd), bf(hd)
    for T_ in (prompt, 8):
        pos, seq = torch.arange(T_, dtype=torch.int32, device=dev), torch.zeros(T_, dtype=torch.int32, device=dev)
        qkv = f32(T_, (H + 2 * G) * hd + H)
        nb = T_ * ((H + 2 * G) * hd * 4 + H * hd * 4 + 2 * G * hd * 2)
        t = timed_k(lambda: hops.attn_prep(qkv, H * hd, (H + G) * hd, geom, freq, None, False, 1e-6, pos, seq, bt, kc, vc, q_norm=qn, k_norm=kn, mag=1.2))
        add("nepudra", "attn_prep (head norms, scaled turn)", f"T={T_} H={H} G={G}", t, nb, 0, VALU_F32)
        g0 = hops.attn_geometry(H, G, hd, hd, 0, 0, 0, page, nblk, nblk)
        t = timed_k(lambda: hops.attn_prep(qkv, H * hd, (H + G) * hd, g0, None, None, False, 1e-6, pos, seq, bt, kc, vc, q_temp=(0.2, 128)))
        add("nepudra", "attn_prep (query temperature)", f"T={T_} H={H} G={G}", t, nb, 0, VALU_F32)
        t = timed_k(lambda: hops.attn_prep(qkv, H * hd, (H + G) * hd, ngeom, freq, vf, True, 1e-5, pos, seq, bt, kc, vc))
        add("nufalorn", "attn_prep (turn, value norm + turn)", f"T={T_} H={H} G={G}", t, nb, 0, VALU_F32)
    # recurrence: the delta rule (width / 64 heads of 64 x 64) against the gated-linear-attention scan (heads of 64 x 128), and their head norms
    Hd, d = W // 64, 64
    for T_, name in ((prompt, "prefill"), (8, "decode b=8")):
        nseq = 1 if T_ > 8 else 8
        rs = torch.arange(0, T_ + 1, T_ // nseq, dtype=torch.int32, device=dev)
        slot, fp = torch.arange(nseq, dtype=torch.int32, device=dev), torch.ones(nseq, dtype=torch.int32, device=dev)
        proj, z = f32(T_, 5 * Hd * d), f32(T_, Hd * d)
        state = torch.zeros(nseq, Hd, d, d, device=dev)
        t = timed_k(lambda: hops.delta_scan(proj, 0, Hd * d, 2 * Hd * d, 3 * Hd * d, z, 0.6, 1e-6, Hd, d, d, rs, slot, fp, state))
        add("nepudra", f"delta scan {name}", f"T={T_} H={Hd} dim={d} vdim={d}", t, T_ * 6 * Hd * d * 4 + 2 * nseq * Hd * d * d * 4, 8.0 * T_ * Hd * d * d, VALU_F32)
        dg = hd // 2
        pg, zg = f32(T_, 2 * H * dg + 2 * H * hd), f32(T_, H * dg)
        sg = torch.zeros(nseq, H, dg, hd, device=dev)
        t = timed_k(lambda: hops.scan(hops.SCAN_GLA, pg, 0, H * dg, 2 * H * dg, zg, None, None, 16.0, dg ** -0.5, H, dg, hd, rs, slot, fp, sg, torch.bfloat16))
        add("nufalorn", f"scan GLA {name}", f"T={T_} H={H} dim={dg} vdim={hd}", t, T_ * (3 * H * dg + 2 * H * hd) * 4 + 2 * nseq * H * dg * hd * 4, 4.0 * T_ * H * dg * hd, VALU_F32)
        o, wn = f32(T_, Hd * d), bf(Hd * d)
        t = timed_k(lambda: hops.head_norm(o, Hd, d, wn, 1e-6, proj, 4 * Hd * d, gate_act="sigmoid"))
        add("nepudra", f"head norm (weight per channel, sigmoid gate) {name}", f"T={T_} H={Hd} vdim={d}", t, T_ * Hd * d * 10, 0, VALU_F32)
        og_, wg = f32(T_, H * hd), bf(hd)
        t = timed_k(lambda: hops.head_norm(og_, H, hd, wg, 1e-5, pg, 2 * H * dg + H * hd))
        add("nufalorn", f"head norm (shared weight, silu gate) {name}", f"T={T_} H={H} vdim={hd}", t, T_ * H * hd * 10, 0, VALU_F32)
    # the layer's end: residual update + average over the stack's depth + norm, against residual update + two norms; embedding rows
    for T_ in (prompt, 8):
        x, a, b = f32(T_, W), f32(T_, W), f32(T_, W)
        w1, w2 = bf(W), bf(W)
        for n in (1, L // 2, L):
            stack, coef = f32(n + 1, T_, W), f32(n + 1)
            t = timed_k(lambda: hops.depth_mix_norm(x, a, stack, n, coef, w1, 1e-6))
            add("nepudra", f"residual + depth average over {n + 1} + norm", f"M={T_} W={W}", t, stream_bytes(T_, W, n + 4, 1), 2.0 * T_ * W * (n + 1), VALU_F32)
        t = timed_k(lambda: hops.residual_norm(x, a, None, 1.0, w1, None, 1e-6))
        add("nepudra", "residual + norm (between the sublayers)", f"M={T_} W={W}", t, stream_bytes(T_, W, 3, 1), 0, VALU_F32)
        t = timed_k(lambda: hops.residual_norm(x, a, b, 0.3, w1, w2, 1e-5, weight_offset=1.0))
        add("nufalorn", "residual + 2 norms (fp32 stream)", f"M={T_} W={W}", t, stream_bytes(T_, W, 4, 2), 0, VALU_F32)
        ids, prev = torch.randint(0, s["vocab"], (T_,), device=dev, dtype=torch.int32), torch.randint(0, s["vocab"], (T_,), device=dev, dtype=torch.int32)
        table, bg, copy = bf(s["vocab"], W), bf(65522, W), f32(T_, W)
        t = timed_k(lambda: hops.embed(ids, table, prev=prev, bigram=bg, mul_prev=8191, mul_cur=131, copy=copy))
        add("nepudra", "embedding + bigram row (two copies)", f"M={T_} W={W}", t, T_ * W * (2 * 2 + 2 * 4), 0, VALU_F32)
        t = timed_k(lambda: hops.embed(ids, table))
        add("nufalorn", "embedding", f"M={T_} W={W}", t, T_ * W * (2 + 4), 0, VALU_F32)
    # linears: the one input linear of a delta layer (r | k | v | a | g, biased, fp32 out), the gelu-gated MLP against the relu-gated one
    for M_ in (prompt, 8, 1):
        x = bf(M_, W)
        w5, b5 = bf(5 * W, W), bf(5 * W)
        t = timed_k(lambda: hops.dense_linear(x, w5, b5, out_dtype=torch.float32))
        add("nepudra", "dense_linear r|k|v|a|g (bias, fp32 out)", f"M={M_} N={5 * W} K={W}", t, 5 * W * W * 2 + M_ * (W * 2 + 5 * W * 4), 2.0 * M_ * 5 * W * W, MFMA_BF16)
        wq = bf((H + 2 * G) * hd, W)
        t = timed_k(lambda: hops.dense_linear(x, wq, out_dtype=torch.float32))
        add("nufalorn", "dense_linear q|k|v (fp32 out)", f"M={M_} N={(H + 2 * G) * hd} K={W}", t, (H + 2 * G) * hd * W * 2 + M_ * (W * 2 + (H + 2 * G) * hd * 4),
            2.0 * M_ * (H + 2 * G) * hd * W, MFMA_BF16)
        wgu = hops.group_gate_up(bf(ff, W), bf(ff, W))
        for fam, act in (("nepudra", hops.ACT_GELU_TANH), ("nufalorn", hops.ACT_RELU)):
            t = timed_k(lambda: hops.dense_linear(x, wgu, gated=True, act=act))
            add(fam, "dense_linear gated (%s)" % ("gelu" if fam == "nepudra" else "relu"), f"M={M_} N={2 * ff} K={W}", t, 2 * ff * W * 2 + M_ * (W + ff) * 2,
                2.0 * M_ * 2 * ff * W, MFMA_BF16)
    return rows


def kernel_table_nudorax(s, dev, prompt):
    """Nudorax's kernels at this size beside the like kernels of the Pokepel member, against max(bytes / HBM, flops / peak of the unit)."""
    from . import hybrid_ops as hops
    rows = []
    timed_k = lambda fn: timed(fn, reps=10, warm=2, graph=True)
    g = torch.Generator(device=dev).manual_seed(3)
    bf = lambda *sh: torch.randn(*sh, device=dev, generator=g).bfloat16()
    f32 = lambda *sh: torch.randn(*sh, device=dev, generator=g)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    W, H, G, hd = s["width"], s["heads"], s["kv"], s["hd"]
    cfg, pcfg = nudorax_config(s), pokepel_config(s)
    moe = cfg["layers"][0]["mlp"]
    lat = next(L["mixer"] for L in pcfg["layers"] if L["type"] == "latent_attention")
    R, dr = lat["kv_rank"], lat["rot_dim"]
    dpad = -(-(R + dr) // 32) * 32
    fe, E, top, gr, lim = moe["expert"]["ff"], moe["router"]["experts"], moe["router"]["top"], moe["router"]["groups"], moe["expert"]["limit"]
    window = cfg["layers"][0]["mixer"]["left"]["mask"]["size"]

    def add(family, name, shape, t, nbytes, flops, peak):
        roof = max(nbytes / HBM, flops / peak)
        rows.append({"family": family, "kernel": name, "shape": shape, "us": round(t * 1e6, 1), "roofline_us": round(roof * 1e6, 2),
                     "x_roofline": round(t / roof, 1)})

    page = 64
    nblk = (prompt + page - 1) // page + 1
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).reshape(1, nblk)
    sink = f32(H)
    # attention: grouped-query pages under a sliding window with learned sinks, against one cached latent row per token for all heads (causal)
    geom = hops.attn_geometry(H, G, hd, hd, hd, 1, 0, page, nblk, nblk)
    lgeo = hops.attn_geometry(H, 1, dpad, R, 0, 0, 0, page, nblk, nblk, v_ld=dpad)
    kc, vc, lc = bf(nblk, G, page, hd), bf(nblk, G, page, hd), bf(nblk, 1, page, dpad)
    for T_, name in ((prompt, "prefill"), (1, "decode")):
        pos = torch.arange(T_, dtype=torch.int32, device=dev) if T_ > 1 else i32([prompt - 1])
        seq = torch.zeros(T_, dtype=torch.int32, device=dev)
        q, lq = f32(T_, H * hd), f32(T_, H * dpad)
        kw = float(sum(min(int(p) + 1, window) for p in pos.tolist()))
        kall = float(sum(int(p) + 1 for p in pos.tolist()))
        byt = lambda keys: min(prompt, keys) * G * hd * 2 * 2 + T_ * H * hd * 6
        if T_ > 1:
            t0 = torch.arange(0, T_, 16, dtype=torch.int32, device=dev)
            tn = torch.full_like(t0, 16)
            t = timed_k(lambda: hops.attn_tiles(q, hd ** -0.5, geom, 0, sink, None, pos, seq, bt, t0, tn, kc, vc, H, hd, window=window))
            add("nudorax", f"attn_tiles prefill (window {window}, learned sinks)", f"T={T_} H={H} G={G} hd={hd} ctx={prompt}", t, byt(prompt), 4.0 * kw * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_tiles(lq, 0.07, lgeo, 0, sink, None, pos, seq, bt, t0, tn, lc, lc, H, R))
            add("pokepel", "attn_tiles latent prefill (causal, learned sinks)", f"T={T_} H={H} row={dpad} rank={R} ctx={prompt}", t, prompt * dpad * 2 + T_ * H * (dpad * 4 + R * 2),
                2.0 * kall * H * (dpad + R), MFMA_BF16)
        else:
            t = timed_k(lambda: hops.attn_rows(q, hd ** -0.5, geom, 0, sink, None, pos, seq, bt, kc, vc, H, hd, window=window))
            add("nudorax", f"attn_rows decode (window {window}, learned sinks)", f"T=1 H={H} G={G} hd={hd} ctx={prompt}", t, byt(window), 4.0 * kw * H * hd, MFMA_BF16)
            t = timed_k(lambda: hops.attn_rows(lq, 0.07, lgeo, 0, sink, None, pos, seq, bt, lc, lc, H, R))
            add("pokepel", "attn_rows latent decode (learned sinks)", f"T=1 H={H} row={dpad} rank={R} ctx={prompt}", t, prompt * dpad * 2, 2.0 * kall * H * (dpad + R), MFMA_BF16)
    # before the scores: norm over all heads + turn + page write, against latent norm + turn + page write + query split
    freq = torch.ones(hd // 2, device=dev) * 1e-3
    lgeom = hops.latent_geometry(H, hd, dr, R, dpad, dr, page, nblk, nblk)
    for T_ in (prompt, 8):
        pos, seq = torch.arange(T_, dtype=torch.int32, device=dev), torch.zeros(T_, dtype=torch.int32, device=dev)
        qkv, qn_, kn_ = f32(T_, (H + 2 * G) * hd), bf(H * hd), bf(G * hd)
        t = timed_k(lambda: hops.attn_prep(qkv, H * hd, (H + G) * hd, geom, freq, None, False, 1e-6, pos, seq, bt, kc, vc, q_norm=qn_, k_norm=kn_, norm_whole=True))
        add("nudorax", "attn_prep (norm over all heads, turn, page write)", f"T={T_} H={H} G={G}", t, T_ * ((H + 2 * G) * hd * 4 + H * hd * 4 + 2 * G * hd * 2), 0, VALU_F32)
        proj, qn, qabs, cw = f32(T_, H * (hd + dr) + R + dr), bf(T_, H * hd), f32(T_, H * dpad), bf(R)
        t = timed_k(lambda: hops.latent_prep(proj, H * (hd + dr), lgeom, freq[: dr // 2], 1.2, cw, 1e-6, pos, seq, bt, qn, qabs, lc.view(nblk, page, dpad)))
        add("pokepel", "latent_prep", f"T={T_} H={H}", t, T_ * (H * (hd + dr) * 4 + H * hd * 2 + H * (dpad - R) * 4 + dpad * 2), 0, VALU_F32)
    # recurrence: fixed decay with silu on q, k, v inside the scan, against fixed decay after a separate turn of q and k; then the norm + gate
    d = hd // 2
    for T_, name in ((prompt, "prefill"), (8, "decode b=8")):
        nseq = 1 if T_ > 8 else 8
        proj = f32(T_, 2 * H * d + 2 * H * hd)
        rs = torch.arange(0, T_ + 1, T_ // nseq, dtype=torch.int32, device=dev)
        slot, fp = torch.arange(nseq, dtype=torch.int32, device=dev), torch.ones(nseq, dtype=torch.int32, device=dev)
        state = torch.zeros(nseq, H, d, hd, device=dev)
        decay = torch.full((H,), 0.97, device=dev)
        nb, fl = T_ * (2 * H * d + 2 * H * hd) * 4 + 2 * nseq * H * d * hd * 4, 4.0 * T_ * H * d * hd
        t = timed_k(lambda: hops.scan(hops.SCAN_FIXED_SILU, proj, 0, H * d, 2 * H * d, None, decay, None, 1.0, 1.0, H, d, hd, rs, slot, fp, state, torch.bfloat16))
        add("nudorax", f"scan lightning (silu inside) {name}", f"T={T_} H={H} dim={d} vdim={hd}", t, nb, fl, VALU_F32)
        t = timed_k(lambda: hops.scan(hops.SCAN_FIXED, proj, 0, H * d, 2 * H * d, None, decay, None, 1.0, 1.0, H, d, hd, rs, slot, fp, state, torch.bfloat16))
        add("pokepel", f"scan retention {name}", f"T={T_} H={H} dim={d} vdim={hd}", t, nb, fl, VALU_F32)
        o, wn = f32(T_, H * hd), bf(H * hd)
        t = timed_k(lambda: hops.head_norm(o, 1, H * hd, wn, 1e-6, proj, 2 * H * d + H * hd, gate_act="sigmoid"))
        add("nudorax", f"norm over all heads (weight, sigmoid gate) {name}", f"T={T_} H={H} vdim={hd}", t, T_ * H * hd * 10, 0, VALU_F32)
        t = timed_k(lambda: hops.head_norm(o, H, hd, None, 1e-6, proj, 2 * H * d + H * hd, out_dtype=torch.bfloat16))
        add("pokepel", f"norm per head (silu gate) {name}", f"T={T_} H={H} vdim={hd}", t, T_ * H * hd * 10, 0, VALU_F32)
    # experts: routing + sorting, both grouped linears with the clamped gate, and the sublayer's end (mixture sum + gated shared expert + layer norm +
    # residual + rounded copy) against Pokepel's (gated residual + mixture sum + RMS norm)
    for T_ in (prompt, 8, 1):
        h = bf(T_, W)
        z = f32(T_, E + 4) * 2
        t = timed_k(lambda: hops.moe_route_sorted(z[:, :E], E, gr["count"], gr["keep"], top, sigmoid=True, group_top=2, scale=2.5))
        add("nudorax", "moe route + sort (sigmoid, groups by two best)", f"T={T_} E={E} top={top}", t, T_ * (E * 4 + top * 16), 0, VALU_F32)
        t = timed_k(lambda: hops.moe_route_sorted(z[:, :E], E, gr["count"], gr["keep"], top))
        add("pokepel", "moe route + sort (softmax, groups by best)", f"T={T_} E={E} top={top}", t, T_ * (E * 4 + top * 16), 0, VALU_F32)
        ids, wts = hops.moe_route(z[:, :E], gr["count"], gr["keep"], top, sigmoid=True, group_top=2, scale=2.5)
        offs, src, place, tiles = hops.moe_align(ids, E)
        n = T_ * top
        used = len(set(ids.flatten().tolist()))
        wgu = torch.stack([hops.group_gate_up(bf(fe, W), bf(fe, W)) for _ in range(E)]).contiguous()
        for fam, act, par in (("nudorax", hops.ACT_SWIGLU_CLAMP, lim), ("pokepel", hops.ACT_SILU, 0.0)):
            t = timed_k(lambda: hops.dense_grouped(h, wgu, offs=offs, gather=src, tiles=tiles, rows=n, gated=True, act=act, act_param=par))
            add(fam, "dense_grouped experts gated (%s)" % ("clamped" if par else "silu"), f"M={T_}x{top} E={E} ({used} used) N={2 * fe} K={W}", t,
                used * 2 * fe * W * 2 + n * (W + fe) * 2, 2.0 * n * 2 * fe * W, MFMA_BF16)
        y, extra = f32(n, W), f32(T_, W)
        xs_, as_, gt_, w1_ = f32(T_, W), f32(T_, W), f32(T_, 2 * W), bf(W)
        t = timed_k(lambda: hops.branch_norm(xs_, w1_, 1e-6, moe=hops.MoeSum(y, place, wts, extra, z[:, E]), rounded=True))
        add("nudorax", "mixture sum + gated shared + layer norm + residual", f"T={T_} top={top} W={W}", t, (n + 3 * T_) * W * 4 + T_ * W * 2, 0, VALU_F32)
        t = timed_k(lambda: hops.residual_norm(xs_, as_, hops.MoeSum(y, place, wts, extra), 1.0, w1_, None, 1e-6, gate=gt_))
        add("pokepel", "gated residual + mixture sum + norm", f"T={T_} top={top} W={W}", t, (n + 7 * T_) * W * 4 + T_ * W * 2, 0, VALU_F32)
    # the mixer sublayer's end (two weighted branches + layer norm + residual + rounded copy), the last norm on gathered rows, the embedding
    for T_ in (prompt, 8):
        x, a, b, gt = f32(T_, W), f32(T_, W), f32(T_, W), f32(T_, 2 * W)
        w1 = bf(W)
        t = timed_k(lambda: hops.branch_norm(x, w1, 1e-6, a=a, ca=1.5, b=b, cb=0.75, rounded=True))
        add("nudorax", "two branches + layer norm + residual (fp32 stream)", f"M={T_} W={W}", t, stream_bytes(T_, W, 4, 1), 0, VALU_F32)
        t = timed_k(lambda: hops.residual_norm(x, a, b, 1.0, w1, None, 1e-6, gate=gt))
        add("pokepel", "gated residual + norm (fp32 stream)", f"M={T_} W={W}", t, stream_bytes(T_, W, 6, 1), 0, VALU_F32)
        ids = torch.randint(0, s["vocab"], (T_,), device=dev, dtype=torch.int32)
        table = bf(s["vocab"], W)
        t = timed_k(lambda: hops.embed_scaled(ids, table, 8.0, rounded=True))
        add("nudorax", "embedding x scale (stream + rounded copy)", f"M={T_} W={W}", t, T_ * W * (2 + 4 + 2), 0, VALU_F32)
        t = timed_k(lambda: hops.embed(ids, table))
        add("pokepel", "embedding", f"M={T_} W={W}", t, T_ * W * (2 + 4), 0, VALU_F32)
    rows_ = torch.arange(8, dtype=torch.int32, device=dev)
    x8, w1 = f32(8, W), bf(W)
    t = timed_k(lambda: hops.norm_rows(x8, rows_, w1, 1e-6))
    add("nudorax", "last layer norm on gathered rows", f"M=8 W={W}", t, 8 * W * 6, 0, VALU_F32)
    t = timed_k(lambda: hops.residual_norm(x8, None, None, 1.0, w1, None, 1e-6, rows=rows_))
    add("pokepel", "last norm on gathered rows", f"M=8 W={W}", t, 8 * W * 6, 0, VALU_F32)
    # linears: ONE input linear per layer for both sides (left q | k | v, right q | k | v | g) against Pokepel's (mixer inputs | gates | router)
    nl, nr = (H + 2 * G) * hd, 2 * H * d + 2 * H * hd
    npk = H * (hd + dr) + R + dr + H * hd + 2 * W + E
    for M_ in (prompt, 8, 1):
        x = bf(M_, W)
        for fam, N_ in (("nudorax", nl + nr), ("pokepel", npk // 4 * 4)):
            wi = bf(N_, W)
            t = timed_k(lambda: hops.dense_linear(x, wi, out_dtype=torch.float32))
            add(fam, "dense_linear all projections of the input (fp32 out)", f"M={M_} N={N_} K={W}", t, N_ * W * 2 + M_ * (W * 2 + N_ * 4), 2.0 * M_ * N_ * W, MFMA_BF16)
    return rows


def stream_bytes(T_, W, f32_streams, bf16_streams):
    return T_ * W * (4 * f32_streams + 2 * bf16_streams)


KERNEL_TABLES = {"pokepel": (kernel_table_pokepel, "nufalorn"), "nepudra": (kernel_table_nepudra, "nufalorn"), "nudorax": (kernel_table_nudorax, "pokepel")}


def run_pokepel(args, dev, sizes, member="pokepel"):
    """A member beside the member of the family that is closest to it (KERNEL_TABLES), engines and kernels."""
    table, beside = KERNEL_TABLES[member]
    prompt, batch, steps = args.hybrid_prompt, args.hybrid_batch, args.steps
    out = {}
    for name in sizes:
        s = SIZES[name]
        log(f"[hybrid bench] {name}: {s}")
        rec = {"config": s, "prompt": prompt, "batch": batch}
        for design in (member, beside):
            rec[design], model, eng = bench_hybrid_engine(s, dev, prompt, batch, steps, design)
            del model, eng
            torch.cuda.empty_cache()
            log(f"[hybrid bench] {name} {design}: {rec[design]}")
        rec["kernels"] = table(s, dev, prompt)
        for r in rec["kernels"]:
            log(f"    {r['family']:8s} {r['kernel']:64s} {r['shape']:48s} {r['us']:10.1f} us  roofline {r['roofline_us']:9.2f} us  x{r['x_roofline']}")
        out[name] = rec
    print(json.dumps({"hybrid_bench": out, "design": member, "dtype": "bf16", "data": "synthetic (random weights and tokens)"}))
    return 0


def run(args):
    from . import _C
    _C.lib(); _C.hybrid_lib()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    sizes = [x for x in (args.hybrid_sizes.split(",") if args.hybrid_sizes else SIZES)]
    if getattr(args, "hybrid_design", "nufalorn") in KERNEL_TABLES:
        return run_pokepel(args, dev, sizes, args.hybrid_design)
    prompt, batch, steps = args.hybrid_prompt, args.hybrid_batch, args.steps
    out = {}
    for name in sizes:
        s = SIZES[name]
        log(f"[hybrid bench] {name}: {s}")
        rec = {"config": s, "prompt": prompt, "batch": batch}
        rec["hybrid"], model, eng = bench_hybrid_engine(s, dev, prompt, batch, steps)
        del model, eng
        torch.cuda.empty_cache()
        log(f"[hybrid bench] {name} hybrid: {rec['hybrid']}")
        rec["qwen2"], q = bench_qwen2_engine(s, dev, prompt, batch, steps)
        del q
        torch.cuda.empty_cache()
        log(f"[hybrid bench] {name} qwen2 : {rec['qwen2']}")
        rec["kernels"] = kernel_table(s, dev, prompt)
        for r in rec["kernels"]:
            log(f"    {r['family']:7s} {r['kernel']:48s} {r['shape']:44s} {r['us']:10.1f} us  roofline {r['roofline_us']:9.2f} us  x{r['x_roofline']}")
        out[name] = rec
    print(json.dumps({"hybrid_bench": out, "dtype": "bf16", "data": "synthetic (random weights and tokens)"}))
    return 0
