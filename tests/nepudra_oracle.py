"""Plain, slow restatement of the Nepudra decoder: sequential pre-norm layers with scalar-gain RMS norms and a learned weighted average
over the outputs of all earlier layers, a hashed bigram embedding beside the token embedding, and three token mixers: a generalized
delta-rule recurrence, causal grouped-query attention with a position-dependent query temperature and a tanh cap on the scores, and
sliding-window grouped-query attention with normed, partly rotated queries and keys.  Both attentions gate every head's output by a
sigmoid.  One function per mechanism, token by token where it is recurrent.  Pure torch on the CPU; shares nothing with the package.

Notation: h [T, W] normed activations of ONE sequence at positions 0..T-1, weights as a dict name -> tensor ([out, in] for linears),
`pre` the layer's tensor prefix.  Everything runs in the dtype of the tensors handed in."""
import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def embedding(wts, tokens, bg):
    """Token rows plus the bigram table's row of (previous token, token); the first token of a sequence takes the table's last row."""
    rows = []
    for t, tok in enumerate(tokens):
        if t == 0:
            r = int(bg["buckets"])
        else:
            r = (int(tokens[t - 1]) * int(bg["mul_prev"]) + int(tok) * int(bg["mul_cur"])) % int(bg["buckets"])
        rows.append(wts["embed"][int(tok)] + wts["bigram"][r])
    return torch.stack(rows)


def rotary_table(rot):
    """(angular step per pair [dims / 2] in float64, magnitude of cos and sin).  scaling {factor, original, fast, slow}: pairs that turn
    fewer than `slow` times over `original` positions are slowed by `factor`, pairs that turn more than `fast` times keep their step,
    with a linear ramp over the pair index between."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    idx = lambda turns: dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(idx(sc["fast"])), 0)
    hi = min(math.ceil(idx(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_halves(t, rot):
    """Turn the first rot.dims channels of t [T, heads, d] by position * step; channel i pairs with channel i + dims / 2."""
    dims = int(rot["dims"])
    if dims == 0:
        return t
    f, mag = rotary_table(rot)
    pos = torch.arange(t.shape[0], dtype=torch.float64)
    a = (pos[:, None] * f[None, :]).to(t.dtype)
    c, s = (torch.cos(a) * mag)[:, None, :], (torch.sin(a) * mag)[:, None, :]
    hf = dims // 2
    out = t.clone()
    u, v = t[..., :hf], t[..., hf:dims]
    out[..., :hf] = u * c - v * s
    out[..., hf:dims] = v * c + u * s
    return out


def softmax_attention(q, k, v, scale, softcap=0.0, window=0):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; row i sees keys j <= i, and with a window only those with i - j < window."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for i in range(T):
        lo = max(0, i - window + 1) if window else 0
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            p = torch.softmax(s, 0)
            out[i, h] = p @ v[lo:i + 1, g]
    return out


def capped_attention(h, wts, pre, mx, kv=None):
    """Mixer "attention": biased projections, no rotation, queries multiplied by 1 + coef ln(floor((p + 1) / every) + 1), scores capped by
    cap tanh(s / cap), causal softmax, a sigmoid gate per head, biased output projection.  kv: (k, v) of the layer named by kv_from.
    -> (output [T, W], (k, v))"""
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    q = (h @ wts[pre + "q"].T + wts[pre + "q.b"]).view(T, H, d)
    if kv is None:
        k = (h @ wts[pre + "k"].T + wts[pre + "k.b"]).view(T, G, d)
        v = (h @ wts[pre + "v"].T + wts[pre + "v.b"]).view(T, G, dv)
    else:
        k, v = kv
    qt = mx.get("q_temp")
    if qt:
        pos = torch.arange(T, dtype=torch.float64)
        temp = 1.0 + float(qt["coef"]) * torch.log(torch.floor((pos + 1.0) / int(qt["every"])) + 1.0)
        q = q * temp.to(q.dtype)[:, None, None]
    o = softmax_attention(q, k, v, float(mx["scale"]), float(mx.get("softcap") or 0.0))
    o = o * torch.sigmoid(h @ wts[pre + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ wts[pre + "o"].T + wts[pre + "o.b"], (k, v)


def window_attention(h, wts, pre, mx, eps, kv=None):
    """Mixer "attention_2": biased q / k / v projections, per-head RMS norm of queries and keys under a weight shared by the heads, partial
    rotary (halves layout, optional frequency scaling), sliding window, softmax, a sigmoid gate per head, output projection without bias."""
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    rot = mx.get("rot") or {"dims": 0, "base": 1.0}
    q = (h @ wts[pre + "q"].T + wts[pre + "q.b"]).view(T, H, d)
    q = rotate_halves(rms_unit(q, eps) * wts[pre + "q.norm"], rot)
    if kv is None:
        k = (h @ wts[pre + "k"].T + wts[pre + "k.b"]).view(T, G, d)
        k = rotate_halves(rms_unit(k, eps) * wts[pre + "k.norm"], rot)
        v = (h @ wts[pre + "v"].T + wts[pre + "v.b"]).view(T, G, dv)
    else:
        k, v = kv
    o = softmax_attention(q, k, v, float(mx["scale"]), 0.0, int((mx.get("mask") or {}).get("size", 0) or 0))
    o = o * torch.sigmoid(h @ wts[pre + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ wts[pre + "o"].T, (k, v)


def delta_rule(h, wts, pre, mx, eps, state=None):
    """Mixer "general_delta": per head a state S [d, d] (key channel x value channel), S <- diag(w) S - (a * u)(u^T S) + k v^T with both
    subtracted and decayed terms taken from the OLD state, o = S^T r.  w = exp(-e^(-1/2) sigmoid(low-rank(h) + w0)), a = sigmoid(W_a h + b),
    u = k / sqrt(|k|^2 + 1e-6) per head.  Heads are brought to unit RMS, multiplied by a per-channel weight and by sigmoid(W_g h)."""
    T = h.shape[0]
    H, d = mx["heads"], mx["dim"]
    r = (h @ wts[pre + "r"].T).view(T, H, d)
    k = (h @ wts[pre + "k"].T).view(T, H, d)
    v = (h @ wts[pre + "v"].T).view(T, H, d)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ wts[pre + "w1"].T) @ wts[pre + "w2"].T + wts[pre + "w0"])).view(T, H, d)
    a = torch.sigmoid(h @ wts[pre + "a"].T + wts[pre + "a.b"]).view(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, d, d, dtype=h.dtype) if state is None else state.clone()
    out = torch.zeros(T, H, d, dtype=h.dtype)
    for t in range(T):
        for j in range(H):
            old = S[j]
            S[j] = w[t, j][:, None] * old - torch.outer(a[t, j] * u[t, j], u[t, j] @ old) + torch.outer(k[t, j], v[t, j])
            out[t, j] = S[j].T @ r[t, j]
    o = (rms_unit(out, eps).reshape(T, H * d) * wts[pre + "norm"]) * torch.sigmoid(h @ wts[pre + "g"].T)
    return o @ wts[pre + "o"].T, S


def gated_mlp(h, wts, pre):
    return (gelu_tanh(h @ wts[pre + "gate"].T) * (h @ wts[pre + "up"].T)) @ wts[pre + "down"].T


def forward(cfg, wts, tokens, collect=None):
    """Logits [T, vocab] of one sequence.  collect: receives the stream after every layer (after the depth average)."""
    eps = float(cfg["norm"]["eps"])
    x = embedding(wts, tokens, cfg["embedding"]["bigram"])
    outs = [x]                                        # X_0 .. X_i: the embedding output and every layer's own result
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        pre, mx = f"l{i}.", L["mixer"]
        h = rms_unit(x, eps) * wts[pre + "norm1"]
        src = mx.get("kv_from")
        kv = kvs[int(src)] if src is not None else None
        if L["type"] == "general_delta":
            a, _ = delta_rule(h, wts, pre + "mix.", mx, eps)
        elif L["type"] == "attention":
            a, kvs[i] = capped_attention(h, wts, pre + "mix.", mx, kv)
        elif L["type"] == "attention_2":
            a, kvs[i] = window_attention(h, wts, pre + "mix.", mx, eps, kv)
        else:
            raise NotImplementedError(L["type"])
        x = x + a
        if L.get("mlp") is not None:
            x = x + gated_mlp(rms_unit(x, eps) * wts[pre + "norm2"], wts, pre + "mlp.")
        outs.append(x)
        c = wts[pre + "dwa"]
        x = sum(c[j] * outs[j] for j in range(i + 2))
        if collect is not None:
            collect.append(x.clone())
    return (rms_unit(x, eps) * wts["final.norm"]) @ wts["head"].T
