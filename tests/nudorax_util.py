"""Small random configurations and checkpoints of the Nudorax decoder for the tests (config.json dicts + name -> tensor)."""
import torch

SCALING = {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 48}


def window_side(heads=4, kv_heads=2, dim=16, vdim=24, scale=None, window=24, rot_dims=None, base=1000.0, scaling=None):
    rot = {"base": base, "dims": dim if rot_dims is None else rot_dims}
    if scaling:
        rot["scaling"] = dict(scaling)
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale, "mask": {"size": window}, "rot": rot}


def lightning_side(heads=2, dim=16, vdim=24, decay=None):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": [0.5 + 0.49 * h / max(1, heads - 1) for h in range(heads)] if decay is None else list(decay)}


def moe(experts=6, top=2, count=3, keep=2, ff=40, limit=1.25, scale=1.5, shared_ff=24, shared_limit=2.5):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return m


def layer(left=None, right=None, left_scale=1.3, right_scale=0.7, mlp=None):
    return {"type": "parallel", "mixer": {"left": left or window_side(), "right": right or lightning_side(), "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp}


def make_config(layers, vocab=96, width=64, eps=1e-5, embed_scale=6.0, softcap=20.0):
    return {"architecture": "Nudorax", "layers": layers, "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
            "logit_softcap": softcap}


def make_weights(cfg, seed=0):
    """Random float32 tensors under the checkpoint names (values exactly representable in bfloat16)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    rn = lambda *s, k=1.0: (torch.randn(*s, generator=g) * k).bfloat16().float()
    lin = lambda o, i: rn(o, i, k=i ** -0.5)
    gain = lambda n: (1.0 + rn(n, k=0.2)).bfloat16().float()
    w = {"embed": rn(cfg["vocab"], W, k=0.3), "final.norm": gain(W)}
    for i, L in enumerate(cfg["layers"]):
        p, mx, mlp = f"l{i}.", L["mixer"], L.get("mlp")
        w[p + "norm1"] = gain(W)
        a, q = mx["left"], p + "mix.left."
        H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        w[q + "q"], w[q + "k"], w[q + "v"], w[q + "o"] = lin(H * d, W), lin(G * d, W), lin(G * dv, W), lin(W, H * dv)
        w[q + "q.norm"], w[q + "k.norm"], w[q + "sink"] = gain(H * d), gain(G * d), rn(H, k=1.0)
        b, q = mx["right"], p + "mix.right."
        H, d, dv = b["heads"], b["dim"], b["vdim"]
        w[q + "q"], w[q + "k"], w[q + "v"], w[q + "g"], w[q + "o"] = lin(H * d, W), lin(H * d, W), lin(H * dv, W), lin(H * dv, W), lin(W, H * dv)
        w[q + "norm"] = gain(H * dv)
        if mlp is not None:
            w[p + "norm2"] = gain(W)
            w[p + "mlp.router"] = rn(mlp["router"]["experts"], W, k=0.1)
            names = [(f"e{j}.", mlp["expert"]["ff"]) for j in range(mlp["router"]["experts"])] + ([("shared.", mlp["shared"]["ff"])] if mlp.get("shared") else [])
            for n, ff in names:
                w[p + "mlp." + n + "gate"], w[p + "mlp." + n + "up"], w[p + "mlp." + n + "down"] = rn(ff, W, k=0.25), rn(ff, W, k=0.25), lin(W, ff)
            if mlp.get("shared"):
                w[p + "mlp.shared.sg"] = rn(1, W, k=0.2)
    return w


def oracle_logits(cfg, w, tokens, collect=None):
    """float64 logits [T, vocab] of the plain implementation."""
    import nudorax_oracle
    return nudorax_oracle.forward(cfg, {k: v.double() for k, v in w.items()}, tokens, collect)
