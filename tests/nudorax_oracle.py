"""Plain, slow implementation of the Nudorax decoder for the tests: one function per mechanism, written from the model's equations in
float64 (or whatever dtype the weights come in), token by token where the model is sequential.  It shares no code with the package.

Model.  x_0 = embed[token] * embedding.scale.  Every layer adds its sublayers' NORMED outputs to the stream, and the sublayers read the
stream itself:  x <- x + LN_1(mixer(x)),  x <- x + LN_2(ff(x)),  LN(y) = (y - mean y) / sqrt(var y + eps) * w.  The mixer is two mixers side by
side on the same input, a_l * window_attention(x) + a_r * lightning(x).  The feed-forward is a mixture of clamped gated experts with a
sigmoid router, group-limited choice and a gated shared expert.  Logits: embed @ LN_final(x), then cap * tanh(. / cap)."""
import math

import torch


# ------------------------------------------------------------------------------------------------ norms and activations
def layer_norm(y, w, eps):
    """(y - mean) / sqrt(mean of squared deviations + eps) * w over the last axis."""
    mu = y.mean(-1, keepdim=True)
    d = y - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def rms_norm(y, w, eps):
    """y / sqrt(mean(y^2) + eps) * w over the last axis."""
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------------------------------ rotary positions
def rotary_steps(rot):
    """Angular step per pair i = 0 .. dims / 2 - 1: base^(-2 i / dims), then per-wavelength scaling: steps whose wavelength is under
    original / high stay, those over original / low are divided by factor, between the two a linear blend in original / wavelength."""
    n = int(rot["dims"])
    out = []
    sc = rot.get("scaling")
    for i in range(n // 2):
        f = float(rot["base"]) ** (-2.0 * i / n)
        if sc:
            lam = 2.0 * math.pi / f
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            if lam < orig / high:
                pass
            elif lam > orig / low:
                f = f / factor
            else:
                s = (orig / lam - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(vec, position, steps):
    """Turn the first 2 len(steps) channels of one head's vector: channel i is paired with channel i + len(steps)."""
    n = len(steps)
    out = vec.clone()
    for i, f in enumerate(steps):
        a = position * f
        c, s = math.cos(a), math.sin(a)
        u, v = vec[i], vec[i + n]
        out[i] = u * c - v * s
        out[i + n] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------------ left mixer: windowed attention with a sink
def window_attention(x, w, p, mx, eps):
    """x [T, W] -> [T, W].  q / k are RMS-normed over the WHOLE projection (all heads at once), split into heads, rotated; query head h reads
    key/value head h // (H / G); position i sees j with 0 <= i - j < window; the softmax denominator also holds exp(sink_h)."""
    H, G, d, dv = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    T = x.shape[0]
    q = rms_norm(x @ w[p + "q"].T, w[p + "q.norm"], eps).view(T, H, d)
    k = rms_norm(x @ w[p + "k"].T, w[p + "k.norm"], eps).view(T, G, d)
    v = (x @ w[p + "v"].T).view(T, G, dv)
    rot = mx.get("rot")
    steps = rotary_steps(rot) if rot and int(rot.get("dims", 0)) else []
    if steps:
        q = torch.stack([torch.stack([rotate(q[t, h], t, steps) for h in range(H)]) for t in range(T)])
        k = torch.stack([torch.stack([rotate(k[t, g], t, steps) for g in range(G)]) for t in range(T)])
    window = int((mx.get("mask") or {}).get("size") or 0)
    scale = float(mx["scale"])
    out = torch.zeros(T, H, dv, dtype=x.dtype)
    for h in range(H):
        g = h // (H // G)
        sink = float(w[p + "sink"][h])
        for i in range(T):
            lo = max(0, i - window + 1) if window > 0 else 0
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            m = max(float(s.max()), sink)
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * v[lo:i + 1, g]).sum(0) / (e.sum() + math.exp(sink - m))
    return out.reshape(T, H * dv) @ w[p + "o"].T


# ------------------------------------------------------------------------------------------------ right mixer: lightning attention
def lightning(x, w, p, mx, eps, state=None):
    """x [T, W] -> [T, W].  Per head S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q, k, v = silu of their projections; the heads
    together are RMS-normed under `norm`, multiplied by sigmoid(W_g x) and projected.  state: list of per-head [dim, vdim] matrices that is
    continued and updated in place (None: start from zero)."""
    H, d, dv = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    T = x.shape[0]
    q = silu(x @ w[p + "q"].T).view(T, H, d)
    k = silu(x @ w[p + "k"].T).view(T, H, d)
    v = silu(x @ w[p + "v"].T).view(T, H, dv)
    if state is None:
        state = [torch.zeros(d, dv, dtype=x.dtype) for _ in range(H)]
    o = torch.zeros(T, H, dv, dtype=x.dtype)
    for h in range(H):
        a = float(mx["decay"][h])
        S = state[h]
        for t in range(T):
            S = a * S + torch.outer(k[t, h], v[t, h])
            o[t, h] = S.T @ q[t, h]
        state[h] = S
    y = rms_norm(o.reshape(T, H * dv), w[p + "norm"], eps) * torch.sigmoid(x @ w[p + "g"].T)
    return y @ w[p + "o"].T


def parallel_mixer(x, w, p, mx, eps, state=None):
    return float(mx["left_scale"]) * window_attention(x, w, p + "left.", mx["left"], eps) + \
        float(mx["right_scale"]) * lightning(x, w, p + "right.", mx["right"], eps, state)


# ------------------------------------------------------------------------------------------------ feed-forward: mixture of clamped gated experts
def expert(x, gate, up, down, limit):
    """g = min(gate x, limit), u = clamp(up x, -limit, limit), y = g sigmoid(1.702 g) (u + 1), output down y."""
    g = torch.clamp(x @ gate.T, max=limit)
    u = torch.clamp(x @ up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(z, router):
    """Router logits [E] of one token -> (chosen experts, their weights).  Scores are sigmoids; the experts form `count` groups of neighbours,
    a group scores as the sum of its two largest scores, only the `keep` best groups stay eligible, the `top` best eligible experts are
    chosen (ties to the lower index) and weigh score * scale, not renormalised."""
    E, top = int(router["experts"]), int(router["top"])
    grp = router.get("groups") or {}
    count = int(grp.get("count", 1))
    keep = int(grp.get("keep", count))
    s = torch.sigmoid(z)
    per = E // count
    gscore = [float(torch.sort(s[g * per:(g + 1) * per], descending=True).values[:2].sum()) for g in range(count)]
    kept = sorted(range(count), key=lambda g: (-gscore[g], g))[:keep]
    eligible = [e for e in range(E) if e // per in kept]
    chosen = sorted(eligible, key=lambda e: (-float(s[e]), e))[:top]
    return chosen, [float(s[e]) * float(router.get("scale", 1.0)) for e in chosen]


def moe(x, w, p, mlp):
    T = x.shape[0]
    z = x @ w[p + "router"].T
    out = torch.zeros_like(x)
    lim = float(mlp["expert"]["limit"])
    for t in range(T):
        ids, wts = route(z[t], mlp["router"])
        for e, a in zip(ids, wts):
            q = p + f"e{e}."
            out[t] += a * expert(x[t:t + 1], w[q + "gate"], w[q + "up"], w[q + "down"], lim)[0]
    sh = mlp.get("shared")
    if sh:
        q = p + "shared."
        out = out + torch.sigmoid(x @ w[q + "sg"].T) * expert(x, w[q + "gate"], w[q + "up"], w[q + "down"], float(sh["limit"]))
    return out


# ------------------------------------------------------------------------------------------------ the model
def forward(cfg, w, tokens, collect=None, states=None):
    """Logits [T, vocab] of one sequence run from its start (states: per-layer lightning states to continue, for tests of the recurrence
    alone; positions then still count from 0).  collect: receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        if L["type"] != "parallel":
            raise NotImplementedError(L["type"])
        x = x + layer_norm(parallel_mixer(x, w, p + "mix.", L["mixer"], eps, None if states is None else states[i]), w[p + "norm1"], eps)
        if L.get("mlp") is not None:
            x = x + layer_norm(moe(x, w, p + "mlp.", L["mlp"]), w[p + "norm2"], eps)
        if collect is not None:
            collect.append(x.clone())
    logits = layer_norm(x, w["final.norm"], eps) @ w["embed"].T
    cap = float(cfg.get("logit_softcap") or 0.0)
    return cap * torch.tanh(logits / cap) if cap > 0 else logits
