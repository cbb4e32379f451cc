"""Small random configurations and checkpoints of the Nepudra decoder for the tests (config.json dicts + name -> tensor)."""
import torch

YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def delta_layer(heads=2, dim=16, mlp=None):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


def capped_layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=None, softcap=20.0, coef=0.25, every=8, kv_from=None, mlp=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale, "softcap": softcap,
          "q_temp": {"coef": coef, "every": every}}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def window_layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=None, window=24, rot_dims=None, base=10000.0, scaling=None, mlp=None):
    rot = {"base": base, "dims": dim if rot_dims is None else rot_dims}
    if scaling:
        rot["scaling"] = dict(scaling)
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale, "mask": {"size": window}, "rot": rot}
    return {"type": "attention_2", "mixer": mx, "mlp": mlp}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def make_config(layers, vocab=96, width=64, eps=1e-5, buckets=53, mul_prev=31, mul_cur=7):
    return {"architecture": "Nepudra", "layers": layers, "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}


def make_weights(cfg, seed=0, rank=8):
    """Random float32 tensors under the checkpoint names (values exactly representable in bfloat16)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    rn = lambda *s, k=1.0: (torch.randn(*s, generator=g) * k).bfloat16().float()
    lin = lambda o, i: rn(o, i, k=i ** -0.5)
    gain = lambda: (1.0 + rn(1, k=0.1)).bfloat16().float().reshape(())
    w = {"embed": rn(cfg["vocab"], W), "bigram": rn(cfg["embedding"]["bigram"]["buckets"] + 1, W, k=0.5), "head": lin(cfg["vocab"], W),
         "final.norm": gain()}
    for i, L in enumerate(cfg["layers"]):
        p, mx, mlp = f"l{i}.", L["mixer"], L.get("mlp")
        w[p + "norm1"] = gain()
        # weights over the embedding output and the results of layers 0 .. i: mostly the newest, a little of everything older
        c = torch.full((i + 2,), 0.3 / (i + 1)) + rn(i + 2, k=0.05)
        c[-1] = 0.8
        w[p + "dwa"] = c.bfloat16().float()
        H, d = mx["heads"], mx["dim"]
        if L["type"] == "general_delta":
            for n in ("r", "k", "v", "a", "g"):
                w[p + "mix." + n] = lin(H * d, W)
            w[p + "mix.a.b"] = rn(H * d, k=0.5)
            w[p + "mix.w1"], w[p + "mix.w2"], w[p + "mix.w0"] = lin(rank, W), lin(H * d, rank), rn(H * d, k=1.0)
            w[p + "mix.norm"] = (1.0 + rn(H * d, k=0.2)).bfloat16().float()
            w[p + "mix.o"] = lin(W, H * d)
        else:
            G, dv = mx.get("kv_heads", H), mx["vdim"]
            w[p + "mix.q"], w[p + "mix.q.b"] = lin(H * d, W), rn(H * d, k=0.2)
            if mx.get("kv_from") is None:
                w[p + "mix.k"], w[p + "mix.k.b"] = lin(G * d, W), rn(G * d, k=0.2)
                w[p + "mix.v"], w[p + "mix.v.b"] = lin(G * dv, W), rn(G * dv, k=0.2)
            w[p + "mix.g"], w[p + "mix.o"] = lin(H, W), lin(W, H * dv)
            if L["type"] == "attention":
                w[p + "mix.o.b"] = rn(W, k=0.2)
            else:
                w[p + "mix.q.norm"] = (1.0 + rn(d, k=0.2)).bfloat16().float()
                if mx.get("kv_from") is None:
                    w[p + "mix.k.norm"] = (1.0 + rn(d, k=0.2)).bfloat16().float()
        if mlp is not None:
            w[p + "norm2"] = gain()
            w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = lin(mlp["ff"], W), lin(mlp["ff"], W), lin(W, mlp["ff"])
    return w


def oracle_logits(cfg, w, tokens, collect=None):
    """float64 logits [T, vocab] of the plain implementation."""
    import nepudra_oracle
    return nepudra_oracle.forward(cfg, {k: v.double() for k, v in w.items()}, tokens, collect)
