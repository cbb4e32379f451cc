"""The hybrid decoder family: a stack of parallel-residual layers  x <- x + m * (g1 * mixer(norm1 x) + g2 * mlp(norm2 x))  over an fp32
residual stream, every layer with its own mixer (mixers.PagedChunkAttention, GatedLinearRecurrence, LatentAttention or Retention) and an
optional feed-forward (gated dense, PolyNorm dense, or routed experts), a final norm, the output head and an optional tanh soft cap of the
logits.  Per member of the family: norm weights stored as offsets from one or plain; one norm per branch or one for both; branch gates
g = sigmoid(W h + b) per channel or none.

``HybridConfig.from_json`` reads the family's config.json (keys: architecture, vocab, width, residual_mult, logit_softcap, norm.eps and
layers[i].{type, mixer, mlp}); ``HybridModel`` holds the device weights (checkpoint tensors embed, l<i>.norm1/2, l<i>.mix.*, l<i>.mlp.*,
final.norm, head) and runs one ragged step against the cache tensors an engine allocated from ``cache_layout()``.

Members: Nufalorn (chunk-masked sink attention with unit-normed, rotated values and shared-KV layers, HGRN2 and GLA recurrences,
relu-gated MLPs, two offset norms per layer) and Pokepel (latent attention and retention, PolyNorm MLPs and group-limited mixtures of
silu-gated experts with a shared expert, one plain norm per layer, sigmoid-gated branches; checkpoint tensors l<i>.rg1 / rg2 (+ .b),
l<i>.mlp.{up, down, act} or l<i>.mlp.{router, e<j>.{gate, up, down}, shared.{gate, up, down}}) and Nepudra (sequential pre-norm layers
x <- x + mixer(norm1 x), x <- x + mlp(norm2 x) whose norms have ONE gain for all channels, every layer reading a learned weighted average
of the embedding output and the results of all layers before it (l<i>.dwa); a hashed bigram table beside the token embedding (bigram);
mixers: a generalized delta-rule recurrence, causal attention with a query temperature, a score cap, biases and per-head output gates, and
sliding-window attention with normed, YaRN-rotated queries and keys; gelu-gated MLPs) and Nudorax (layers x <- x + LN(mixer(x)),
x <- x + LN(mlp(x)): the sublayers read the stream itself and a layer norm follows each; every mixer is two side by side, windowed attention
with a learned sink and queries / keys normed over all heads at once beside lightning attention; mixtures of clamped gated experts under a
sigmoid router whose groups rank by their two best, with a gated shared expert; the embedding is scaled on entry and is the output head;
checkpoint tensors l<i>.mix.left.{q, k, v, q.norm, k.norm, sink, o}, l<i>.mix.right.{q, k, v, g, norm, o}, l<i>.mlp.{router, e<j>.*, shared.{gate, up,
down, sg}})."""
import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Union

import torch

from . import hybrid_ops as hops
from .mixers import (AttentionSpec, DeltaRuleSpec, GatedLinearRecurrence, GatedMLP, GeneralizedDeltaRule, LatentAttention, LatentAttentionSpec,
                     LightningAttention, LightningSpec, PagedChunkAttention, ParallelMixer, PolyNormMLP, RecurrenceSpec, Retention, RetentionSpec,
                     RotarySpec, RoutedExperts, RouterSpec, StepBatch)


@dataclass
class ParallelSpec:
    """Two mixers on the same input, added as left_scale * left + right_scale * right; their checkpoint tensors sit under mix.left. / mix.right."""
    left: Union[AttentionSpec, LightningSpec]
    right: Union[AttentionSpec, LightningSpec]
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass
class HybridLayerSpec:
    kind: str                                        # "attention" | "hgrn2" | "gla" | "latent_attention" | "retention" | "delta_rule" | "lightning" | "parallel"
    mixer: Union[AttentionSpec, RecurrenceSpec, LatentAttentionSpec, RetentionSpec, DeltaRuleSpec, LightningSpec, ParallelSpec]
    ff: Optional[int] = None                         # None: the layer has no MLP; hidden size of the dense MLP or of one routed expert
    mlp_act: str = "relu"
    mlp_kind: str = "gated"                          # "gated" | "polynorm" | "experts"
    router: Optional[RouterSpec] = None              # experts: the router ...
    shared_ff: Optional[int] = None                  # ... and the hidden size of the expert every token runs (None: no such expert)
    act_param: float = 0.0                           # parameter of mlp_act (the limit of "swiglu_clamp") ...
    shared_act_param: float = 0.0                    # ... and the shared expert's own
    shared_gate: bool = False                        # the shared expert's output is multiplied by sigmoid(w . h), one number per token (mlp.shared.sg)


@dataclass
class BigramSpec:
    """A second embedding table indexed by a hash of (previous token, token): row (prev * mul_prev + token * mul_cur) mod buckets, and row
    `buckets` (the table's last) for the first token of a sequence."""
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class HybridConfig:
    name: str
    vocab: int
    width: int
    layers: List[HybridLayerSpec]
    eps: float = 1e-5
    residual_mult: float = 1.0
    logit_softcap: float = 0.0
    norm_offset: float = 1.0                         # stored norm weights are offsets from this value
    shared_norm: bool = False                        # one norm per layer feeds the mixer and the MLP
    branch_gates: bool = False                       # each branch is multiplied by sigmoid(W h + b) of its input before it joins the stream
    sequential: bool = False                         # x <- x + mixer(norm1 x), then x <- x + mlp(norm2 x) (instead of both branches from one x)
    scalar_norm: bool = False                        # every norm's weight is ONE number for all channels
    depth_mix: bool = False                          # a layer reads sum_j dwa[j] X_j over the embedding output X_0 and all earlier layers' results
    bigram: Optional[BigramSpec] = None              # hashed (previous token, token) rows added to the token embedding
    embed_scale: float = 1.0                         # the embedding rows are multiplied by this as they enter the stream
    tied_head: bool = False                          # the output head is the embedding table itself (without embed_scale); no `head` tensor
    out_norm: bool = False                           # sequential layers whose sublayers read the stream ITSELF and whose OUTPUT is normed: x <- x + norm(f(x))
    norm_kind: str = "rms"                           # "rms" | "layer" (mean removed, variance of the deviations, a weight and no bias)

    @staticmethod
    def from_json(cfg: dict) -> "HybridConfig":
        """config.json -> the configuration of the member its "architecture" names."""
        reader = _READERS.get(str(cfg.get("architecture", "")).lower())
        if reader is None:
            raise NotImplementedError(f"hybrid family: architecture {cfg.get('architecture')!r} (known: {', '.join(sorted(_READERS))})")
        return reader(cfg)

    @staticmethod
    def nufalorn_from_json(cfg: dict) -> "HybridConfig":
        """The Nufalorn reading of config.json: attention layers have the softmax sink, unit-normed values and values rotated in the key
        layout (interleaved pairs); MLPs are relu-gated; norm weights are stored around zero."""
        layers = []
        for i, L in enumerate(cfg["layers"]):
            kind, mx, mlp = L["type"], L["mixer"], L.get("mlp")
            if kind == "attention":
                rot = mx.get("rot")
                rs = RotarySpec(int(rot["dims"]), float(rot["base"]), "interleaved") if rot and int(rot.get("dims", 0)) else None
                mask = mx.get("mask") or {}
                spec = AttentionSpec(heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]), vdim=int(mx["vdim"]),
                                     scale=float(mx["scale"]), rot=rs, chunk=int(mask.get("size", 0) or 0), sink=True, value_norm=True,
                                     value_rot=rs is not None, value_layout="interleaved",
                                     kv_from=None if mx.get("kv_from") is None else int(mx["kv_from"]))
            elif kind in ("hgrn2", "gla"):
                spec = RecurrenceSpec(kind, heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx["vdim"]), tau=float(mx.get("tau", 1.0)))
            else:
                raise NotImplementedError(f"layer {i}: mixer type {kind!r}")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise NotImplementedError(f"layer {i}: mlp kind {mlp.get('kind')!r}")
            layers.append(HybridLayerSpec(kind, spec, None if mlp is None else int(mlp["ff"]), "relu"))
        _check_kv_from(layers)
        return HybridConfig(name=str(cfg.get("architecture", "hybrid")), vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=layers,
                            eps=float(cfg["norm"]["eps"]), residual_mult=float(cfg.get("residual_mult", 1.0)),
                            logit_softcap=float(cfg.get("logit_softcap") or 0.0))

    @staticmethod
    def pokepel_from_json(cfg: dict) -> "HybridConfig":
        """The Pokepel reading of config.json: latent attention (interleaved rotary pairs on the rotated part, optional YaRN scaling, learned
        sink, output gate) and retention (rotary pairs half a span apart, one decay per head); dense MLPs use PolyNorm, mixtures have silu-gated
        experts; one plain norm per layer, gated branches, no residual multiplier or soft cap."""
        layers = []
        for i, L in enumerate(cfg["layers"]):
            kind, mx, mlp = L["type"], L["mixer"], L.get("mlp")
            if kind == "latent_attention":
                rot = dict(mx.get("rot") or {})
                rot.setdefault("dims", mx["rot_dim"])
                spec = LatentAttentionSpec(heads=int(mx["heads"]), dim=int(mx["dim"]), rot_dim=int(mx["rot_dim"]), vdim=int(mx["vdim"]),
                                           kv_rank=int(mx["kv_rank"]), scale=float(mx["scale"]),
                                           rot=RotarySpec.from_json(rot if "base" in rot else None, "interleaved"))
            elif kind == "retention":
                if len(mx["decay"]) != int(mx["heads"]):
                    raise ValueError(f"layer {i}: {len(mx['decay'])} decays for {mx['heads']} heads")
                spec = RetentionSpec(heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx["vdim"]), decay=tuple(float(a) for a in mx["decay"]),
                                     rot=RotarySpec.from_json(mx.get("rot"), "halves"))
            else:
                raise NotImplementedError(f"layer {i}: mixer type {kind!r}")
            if mlp is None:
                layers.append(HybridLayerSpec(kind, spec))
            elif mlp.get("kind", "dense") == "dense":
                layers.append(HybridLayerSpec(kind, spec, int(mlp["ff"]), "polynorm", "polynorm"))
            elif mlp["kind"] == "moe":
                r, grp, sh = mlp["router"], mlp["router"].get("groups") or {}, mlp.get("shared")
                layers.append(HybridLayerSpec(kind, spec, int(mlp["expert"]["ff"]), "silu", "experts",
                                              RouterSpec(int(r["experts"]), int(r["top"]), int(grp.get("count", 1)), int(grp.get("keep", grp.get("count", 1)))),
                                              None if not sh else int(sh["ff"])))
            else:
                raise NotImplementedError(f"layer {i}: mlp kind {mlp.get('kind')!r}")
        return HybridConfig(name=str(cfg["architecture"]), vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=layers, eps=float(cfg["norm"]["eps"]),
                            residual_mult=1.0, logit_softcap=0.0, norm_offset=0.0, shared_norm=True, branch_gates=True)


def _check_kv_from(layers):
    for i, L in enumerate(layers):
        src = getattr(L.mixer, "kv_from", None)
        if src is not None:
            o = layers[src].mixer if 0 <= src < i else None
            if not isinstance(o, AttentionSpec) or o.kv_from is not None or (o.kv_heads, o.dim, o.vdim) != (L.mixer.kv_heads, L.mixer.dim, L.mixer.vdim):
                raise ValueError(f"layer {i}: kv_from {src} must name an earlier attention layer with its own keys and values of the same shape")


def nepudra_from_json(cfg: dict) -> HybridConfig:
    """The Nepudra reading of config.json.  Layer types: "general_delta" (mixer.{heads, dim}: key and value size are both dim),
    "attention" (mixer.{heads, kv_heads, dim, vdim, scale, softcap, q_temp.{coef, every}, kv_from}: biased projections, no rotation, causal)
    and "attention_2" (mixer.{heads, kv_heads, dim, vdim, scale, mask.size, rot.{dims, base, scaling}}: biased q / k / v, normed queries and
    keys, rotary pairs half a span apart, sliding window); both attentions gate every head's output.  mlp: null or {kind: dense, ff}."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        kind, mx, mlp = L["type"], L["mixer"], L.get("mlp")
        src = None if mx.get("kv_from") is None else int(mx["kv_from"])
        if kind == "general_delta":
            spec, kind = DeltaRuleSpec(heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx["dim"])), "delta_rule"
        elif kind == "attention":
            qt = mx.get("q_temp")
            spec = AttentionSpec(heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                                 scale=float(mx.get("scale", int(mx["dim"]) ** -0.5)), kv_from=src, softcap=float(mx.get("softcap") or 0.0),
                                 q_temp=(float(qt["coef"]), int(qt["every"])) if qt else None, bias=True, out_bias=True, out_gate=True)
        elif kind == "attention_2":
            mask = mx.get("mask") or {}
            spec = AttentionSpec(heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                                 scale=float(mx.get("scale", int(mx["dim"]) ** -0.5)), rot=RotarySpec.from_json(mx.get("rot"), "halves"), kv_from=src,
                                 window=int(mask.get("size", 0) or 0), qk_norm=True, bias=True, out_gate=True)
            kind = "attention"
        else:
            raise NotImplementedError(f"layer {i}: mixer type {kind!r}")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise NotImplementedError(f"layer {i}: mlp kind {mlp.get('kind')!r}")
        layers.append(HybridLayerSpec(kind, spec, None if mlp is None else int(mlp["ff"]), "gelu_tanh"))
    _check_kv_from(layers)
    bg = (cfg.get("embedding") or {}).get("bigram")
    return HybridConfig(name=str(cfg["architecture"]), vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=layers, eps=float(cfg["norm"]["eps"]),
                        norm_offset=0.0, sequential=True, scalar_norm=True, depth_mix=True,
                        bigram=BigramSpec(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None)


def nudorax_from_json(cfg: dict) -> HybridConfig:
    """The Nudorax reading of config.json.  Layer type "parallel": mixer.{left, right, left_scale, right_scale} with left = windowed attention
    {heads, kv_heads, dim, vdim, scale, mask.size, rot.{dims, base, scaling.{factor, low, high, original}}} (queries and keys normed over all heads
    at once, rotary pairs half a span apart with wavelength-scaled steps, a learned sink logit per head) and right = lightning attention
    {heads, dim, vdim, decay[heads]}.  mlp: null or {kind: moe, expert.{ff, limit}, router.{experts, top, scale, groups.{count, keep}},
    shared.{ff, limit}} with a sigmoid router whose groups rank by their two best experts, clamped gated experts and a gated shared expert.
    Layer norms on the sublayers' outputs, the embedding scaled on entry and reused as the output head, a tanh cap on the logits."""
    def attention(mx):
        mask = mx.get("mask") or {}
        return AttentionSpec(heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads") or mx["heads"]), dim=int(mx["dim"]), vdim=int(mx.get("vdim") or mx["dim"]),
                             scale=float(mx["scale"]), rot=RotarySpec.from_json(mx.get("rot"), "halves", scaling="wavelength"),
                             window=int(mask.get("size") or 0), sink=True, learned_sink=True, qk_norm=True, qk_norm_whole=True)

    def lightning(mx):
        return LightningSpec(heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx.get("vdim") or mx["dim"]), decay=tuple(float(a) for a in mx["decay"]))

    layers = []
    for i, L in enumerate(cfg["layers"]):
        kind, mx, mlp = L["type"], L["mixer"], L.get("mlp")
        if kind != "parallel":
            raise NotImplementedError(f"layer {i}: mixer type {kind!r}")
        if len(mx["right"]["decay"]) != int(mx["right"]["heads"]):
            raise ValueError(f"layer {i}: {len(mx['right']['decay'])} decays for {mx['right']['heads']} heads")
        spec = ParallelSpec(attention(mx["left"]), lightning(mx["right"]), float(mx.get("left_scale", 1.0)), float(mx.get("right_scale", 1.0)))
        if mlp is None:
            layers.append(HybridLayerSpec(kind, spec))
        elif mlp.get("kind") == "moe":
            r, sh = mlp["router"], mlp.get("shared")
            grp = r.get("groups") or {}
            count = int(grp.get("count", 1))
            router = RouterSpec(int(r["experts"]), int(r["top"]), count, int(grp.get("keep", count)), score="sigmoid", group_top=2, scale=float(r.get("scale", 1.0)))
            layers.append(HybridLayerSpec(kind, spec, int(mlp["expert"]["ff"]), "swiglu_clamp", "experts", router, None if not sh else int(sh["ff"]),
                                          act_param=float(mlp["expert"]["limit"]), shared_act_param=float(sh["limit"]) if sh else 0.0, shared_gate=bool(sh)))
        else:
            raise NotImplementedError(f"layer {i}: mlp kind {mlp.get('kind')!r}")
    return HybridConfig(name=str(cfg["architecture"]), vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=layers, eps=float(cfg["norm"]["eps"]),
                        logit_softcap=float(cfg.get("logit_softcap") or 0.0), norm_offset=0.0, sequential=True, out_norm=True, norm_kind="layer",
                        embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)), tied_head=True)


_READERS = {"nufalorn": HybridConfig.nufalorn_from_json, "pokepel": HybridConfig.pokepel_from_json, "nepudra": nepudra_from_json, "nudorax": nudorax_from_json}


class HybridModel:
    """Device weights + the step function.  dtype: torch.bfloat16 (16-bit weights and activations, fp32 accumulation and fp32 for everything
    the family keeps in 32-bit) or torch.float32 (everything in true fp32)."""

    def __init__(self, cfg: HybridConfig, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device, page: int = 64):
        hops.act_code(dtype)
        self.cfg, self.dtype, self.device, self.page = cfg, dtype, torch.device(device), page

        def get(name):
            if name not in tensors:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            return tensors[name].to(device=self.device, dtype=dtype).contiguous()

        def sub(prefix, names):
            return {n: get(prefix + n) for n in names}

        def norm_w(name):                             # a norm with one gain is run as a norm whose weight repeats it over the channels
            t = get(name)
            return t.reshape(1).expand(cfg.width).contiguous() if cfg.scalar_norm else t

        self.embed = get("embed")
        self.head = self.embed if cfg.tied_head else get("head")
        self.final_norm = norm_w("final.norm")
        self.bigram = None
        if cfg.bigram is not None:
            self.bigram = get("bigram")
            if self.bigram.shape != (cfg.bigram.buckets + 1, cfg.width):
                raise ValueError(f"bigram table {tuple(self.bigram.shape)} for {cfg.bigram.buckets} buckets of width {cfg.width}")
        self.depth_coef = []                             # layer i: fp32 [i + 2] weights over X_0 .. X_(i+1)
        if cfg.depth_mix:
            for i in range(len(cfg.layers)):
                c = tensors[f"l{i}.dwa"].to(device=self.device, dtype=torch.float32).contiguous()
                if c.numel() != i + 2:
                    raise ValueError(f"l{i}.dwa has {c.numel()} weights for {i + 2} results")
                self.depth_coef.append(c)
        if self.embed.shape != (cfg.vocab, cfg.width) or self.head.shape != (cfg.vocab, cfg.width):
            raise ValueError(f"embed {tuple(self.embed.shape)} / head {tuple(self.head.shape)} against vocab {cfg.vocab} width {cfg.width}")
        self.layers = []
        self.n_mix = {}                                  # layer -> (columns, padded columns) of the mixer's inputs inside the layer's shared linear
        for i, L in enumerate(cfg.layers):
            p = f"l{i}."
            def attention(a, q):
                own = a.kv_from is None
                names = ["q", "o"] + (["k", "v"] if own else []) + (["g"] if a.out_gate else []) + (["o.b"] if a.out_bias else [])
                names += (["q.b"] + (["k.b", "v.b"] if own else [])) if a.bias else []
                names += (["q.norm"] + (["k.norm"] if own else [])) if a.qk_norm else []
                names += ["sink"] if a.sink and a.learned_sink else []
                return PagedChunkAttention(a, sub(q, names), cfg.eps, page, self.device)

            def lightning(a, q):
                return LightningAttention(a, sub(q, ["q", "k", "v", "g", "norm", "o"]), cfg.eps, self.device)

            def side(a, q):
                if isinstance(a, AttentionSpec):
                    if a.kv_from is not None:
                        raise NotImplementedError("a side of a parallel mixer keeps its own keys and values")
                    return attention(a, q)
                return lightning(a, q)

            if L.kind == "attention":
                mixer = attention(L.mixer, p + "mix.")
            elif L.kind == "lightning":
                mixer = lightning(L.mixer, p + "mix.")
            elif L.kind == "parallel":
                mixer = ParallelMixer(side(L.mixer.left, p + "mix.left."), side(L.mixer.right, p + "mix.right."), L.mixer.left_scale, L.mixer.right_scale)
            elif L.kind == "delta_rule":
                mixer = GeneralizedDeltaRule(L.mixer, sub(p + "mix.", ["r", "k", "v", "a", "a.b", "g", "w1", "w2", "w0", "norm", "o"]), cfg.eps)
            elif L.kind == "latent_attention":
                mixer = LatentAttention(L.mixer, sub(p + "mix.", ["q", "dkv", "dkv.norm", "uk", "uv", "sink", "g", "o"]), cfg.eps, page, self.device)
            elif L.kind == "retention":
                mixer = Retention(L.mixer, sub(p + "mix.", ["q", "k", "v", "g", "o"]), cfg.eps, self.device)
            elif L.kind == "hgrn2":
                mixer = GatedLinearRecurrence(L.mixer, sub(p + "mix.", ["q", "f", "f.b", "lower", "v", "norm", "o"]), cfg.eps)
            else:
                mixer = GatedLinearRecurrence(L.mixer, sub(p + "mix.", ["q", "k", "v", "g", "a1", "a2", "a2.b", "norm", "o"]), cfg.eps)
            mlp = None
            if L.ff is not None:
                gated = lambda q, act, par=0.0: GatedMLP(get(q + "gate"), get(q + "up"), get(q + "down"), act, par)
                if L.mlp_kind == "gated":
                    mlp = gated(p + "mlp.", L.mlp_act)
                elif L.mlp_kind == "polynorm":
                    mlp = PolyNormMLP(get(p + "mlp.up"), get(p + "mlp.down"), tensors[p + "mlp.act"], cfg.eps)
                else:
                    ex = [p + f"mlp.e{j}." for j in range(L.router.experts)]
                    mlp = RoutedExperts(L.router, get(p + "mlp.router"), [get(q + "gate") for q in ex], [get(q + "up") for q in ex],
                                        [get(q + "down") for q in ex],
                                        gated(p + "mlp.shared.", L.mlp_act, L.shared_act_param or L.act_param) if L.shared_ff is not None else None, L.mlp_act,
                                        act_param=L.act_param, shared_gate=get(p + "mlp.shared.sg") if L.shared_gate else None)
            gate_w = gate_b = None
            if cfg.branch_gates:                       # both gates in one linear: columns [0, W) scale the mixer, [W, 2W) the MLP
                names = ["rg1"] + (["rg2"] if mlp is not None else [])
                gate_w = torch.cat([get(p + n) for n in names], 0).contiguous()
                gate_b = torch.cat([get(p + n + ".b") for n in names], 0).contiguous()
                if mlp is None:                        # the kernel reads two gates per row: keep the row stride at 2 W
                    gate_w = torch.cat([gate_w, torch.zeros_like(gate_w)], 0).contiguous()
                    gate_b = torch.cat([gate_b, torch.zeros_like(gate_b)], 0).contiguous()
                if isinstance(mlp, RoutedExperts):     # the router's logits come out of the same linear: columns [2W, 2W + experts), padded to 4
                    E = L.router.experts
                    rw = torch.cat([mlp.w_router, torch.zeros((-E) % 4, cfg.width, dtype=dtype, device=self.device)], 0)
                    gate_w = torch.cat([gate_w, rw], 0).contiguous()
                    gate_b = torch.cat([gate_b, torch.zeros(rw.shape[0], dtype=dtype, device=self.device)], 0).contiguous()
            n2 = norm_w(p + "norm2") if mlp is not None and not cfg.shared_norm else None
            if gate_w is not None and cfg.shared_norm and isinstance(mixer, (LatentAttention, Retention)):
                # every projection of the layer's one normed input in ONE linear: [mixer inputs (padded to 4 columns) | gates | router]
                pad = (-mixer.w_in.shape[0]) % 4
                zrow = torch.zeros(pad, cfg.width, dtype=dtype, device=self.device)
                self.n_mix[i] = (mixer.w_in.shape[0], mixer.w_in.shape[0] + pad)
                gate_b = torch.cat([torch.zeros(mixer.w_in.shape[0] + pad, dtype=dtype, device=self.device), gate_b], 0).contiguous()
                gate_w = torch.cat([mixer.w_in, zrow, gate_w], 0).contiguous()
                mixer.w_in = None                      # lives on as the leading rows of the shared weight
            self.layers.append((L, mixer, mlp, norm_w(p + "norm1"), n2, gate_w, gate_b))
        self.has_state = any(L.kind not in ("attention", "latent_attention") for L in cfg.layers)
        self.norm_center = cfg.norm_kind == "layer"
        if cfg.norm_kind not in ("rms", "layer") or (cfg.norm_kind == "layer" and not cfg.out_norm):
            raise NotImplementedError(f"norm kind {cfg.norm_kind!r} (layer norms are built for stacks that norm the sublayers' outputs)")

    # ---- what an engine has to allocate
    def cache_layout(self):
        """Per layer: ("kv", K page shape, V page shape) | ("kv_from", layer) | ("latent", page shape) | ("state", per-slot shape) |
        ("sides", [entries of the two sides of a parallel mixer, each "kv" or "state"])."""
        out = []
        for L, mixer, *_ in self.layers:
            if L.kind == "parallel":
                out.append(("sides", [(("kv",) + m.cache_shapes()) if m.cache_kind() == "kv" else ("state", m.state_shape()) for m in (mixer.left, mixer.right)]))
            elif L.kind == "attention":
                out.append((("kv",) + mixer.cache_shapes()) if mixer.owns_cache else ("kv_from", L.mixer.kv_from))
            elif L.kind == "latent_attention":
                out.append(("latent", mixer.cache_shape()))
            else:
                out.append(("state", mixer.state_shape()))
        return out

    def alloc_cache(self, num_pages: int, num_slots: int):
        """Cache tensors for `num_pages` pages and `num_slots` state slots: per layer (kcache, vcache) or a state tensor; for a parallel mixer
        the tuple of its sides' tensors in order."""
        caches = []
        pages = lambda shape: torch.zeros(num_pages, *shape, dtype=self.dtype, device=self.device)
        slots = lambda shape: torch.zeros(num_slots, *shape, dtype=torch.float32, device=self.device)
        for ent in self.cache_layout():
            if ent[0] == "sides":
                flat = []
                for e in ent[1]:
                    flat += [pages(e[1]), pages(e[2])] if e[0] == "kv" else [slots(e[1])]
                caches.append(tuple(flat))
            elif ent[0] == "kv":
                caches.append((torch.zeros(num_pages, *ent[1], dtype=self.dtype, device=self.device),
                               torch.zeros(num_pages, *ent[2], dtype=self.dtype, device=self.device)))
            elif ent[0] == "kv_from":
                caches.append(caches[ent[1]])
            elif ent[0] == "latent":                   # one row per token serves as key and (its leading channels) as value
                caches.append((torch.zeros(num_pages, *ent[1], dtype=self.dtype, device=self.device), None))
            else:
                caches.append(torch.zeros(num_slots, *ent[1], dtype=torch.float32, device=self.device))
        return caches

    # ---- one step
    def forward(self, batch: StepBatch, caches, collect: Optional[list] = None) -> torch.Tensor:
        """fp32 logits [len(batch.want), vocab] of the wanted rows; the caches of every row's sequence are advanced.  collect: receives
        the residual stream after every layer (debugging / tests; costs one extra norm launch per layer)."""
        cfg = self.cfg
        if cfg.out_norm:
            return self._forward_out_norm(batch, caches, collect)
        if cfg.sequential:
            return self._forward_sequential(batch, caches, collect)
        x = hops.embed(batch.tokens, self.embed)
        a = b = g = None
        shared = self.n_mix
        for i, ((L, mixer, mlp, n1, n2, gate_w, gate_b), cache) in enumerate(zip(self.layers, caches)):
            h1, h2 = hops.residual_norm(x, a, b, cfg.residual_mult, n1, n2, cfg.eps, weight_offset=cfg.norm_offset, gate=g)
            if collect is not None and a is not None:
                collect.append(x.clone())
            if cfg.shared_norm:
                h2 = h1
            if i in shared:                            # the mixer's projections are the leading rows of the gates' weight
                n_in, n_pad = shared[i]
                if h1.shape[0] <= 16:                  # decode-sized steps: one launch streams the whole weight
                    g = hops.dense_linear(h1, gate_w, gate_b, out_dtype=torch.float32)
                    proj, g = g[:, :n_in], g[:, n_pad:]
                else:                                  # prompt portions: the tile kernel is faster on the two halves (measured: 0.6 ms of a 2048-token prefill)
                    proj = hops.dense_linear(h1, gate_w[:n_in], out_dtype=torch.float32)
                    g = hops.dense_linear(h1, gate_w[n_pad:], gate_b[n_pad:], out_dtype=torch.float32)
                a = mixer.forward(h1, batch, *cache, proj=proj) if isinstance(cache, tuple) else mixer.forward(h1, batch, cache, proj=proj)
            else:
                g = hops.dense_linear(h1, gate_w, gate_b, out_dtype=torch.float32) if gate_w is not None else None
                a = mixer.forward(h1, batch, *cache) if isinstance(cache, tuple) else mixer.forward(h1, batch, cache)
            if mlp is None:
                b = None
            elif g is not None and isinstance(mlp, RoutedExperts):
                b = mlp.forward(h2, g[:, 2 * cfg.width: 2 * cfg.width + L.router.experts], defer=True)   # summed by the next residual kernel
            else:
                b = mlp.forward(h2)
        if collect is not None:
            hops.residual_norm(x, a, b, cfg.residual_mult, self.final_norm, None, cfg.eps, weight_offset=cfg.norm_offset, gate=g)
            collect.append(x.clone())
            a = b = g = None
        hf, _ = hops.residual_norm(x, a, b, cfg.residual_mult, self.final_norm, None, cfg.eps, weight_offset=cfg.norm_offset, rows=batch.want, gate=g)
        return hops.dense_linear(hf, self.head, out_dtype=torch.float32, softcap=cfg.logit_softcap)


    def _forward_sequential(self, batch: StepBatch, caches, collect: Optional[list]) -> torch.Tensor:
        """The step of a member whose two sublayers follow each other: x <- x + mixer(norm1 x), x <- x + mlp(norm2 x).  With depth_mix the
        results X_1 .. of all layers and the embedding output X_0 are kept for the step, and the end of layer i replaces the stream by
        sum_j dwa_i[j] X_j, fused with the last residual update and the next norm."""
        cfg, T = self.cfg, batch.tokens.numel()
        n_layers = len(self.layers)
        stack = torch.empty(n_layers + 1 if cfg.depth_mix else 0, T, cfg.width, dtype=torch.float32, device=self.device)
        bg = cfg.bigram
        x = hops.embed(batch.tokens, self.embed, prev=batch.prev if bg else None, bigram=self.bigram, mul_prev=bg.mul_prev if bg else 0,
                       mul_cur=bg.mul_cur if bg else 0, copy=stack[0] if cfg.depth_mix else None)
        h1, _ = hops.residual_norm(x, None, None, 1.0, self.layers[0][3], None, cfg.eps, weight_offset=cfg.norm_offset)
        for i, ((L, mixer, mlp, n1, n2, _gw, _gb), cache) in enumerate(zip(self.layers, caches)):
            a = mixer.forward(h1, batch, *cache) if isinstance(cache, tuple) else mixer.forward(h1, batch, cache)
            if mlp is not None:
                h2, _ = hops.residual_norm(x, a, None, 1.0, n2, None, cfg.eps, weight_offset=cfg.norm_offset)
                a = mlp.forward(h2)
            last = i + 1 == n_layers
            nw = self.final_norm if last else self.layers[i + 1][3]
            rows = batch.want if last and collect is None else None
            if cfg.depth_mix:
                h1 = hops.depth_mix_norm(x, a, stack, i + 1, self.depth_coef[i], nw, cfg.eps, weight_offset=cfg.norm_offset, rows=rows)
            else:
                h1, _ = hops.residual_norm(x, a, None, 1.0, nw, None, cfg.eps, weight_offset=cfg.norm_offset, rows=rows)
            if collect is not None:
                collect.append(x.clone())
        if collect is not None:
            h1, _ = hops.residual_norm(x, None, None, 1.0, self.final_norm, None, cfg.eps, weight_offset=cfg.norm_offset, rows=batch.want)
        return hops.dense_linear(h1, self.head, out_dtype=torch.float32, softcap=cfg.logit_softcap)


    def _forward_out_norm(self, batch: StepBatch, caches, collect: Optional[list]) -> torch.Tensor:
        """The step of a member whose sublayers read the stream itself and whose outputs are normed: x <- x + N(mixer(x)), x <- x + N(mlp(x)).  The
        stream stays fp32; the sublayers' input is its rounding to the activation type, written by the kernel that ends the sublayer before.  A
        parallel mixer's two outputs and a mixture's parts (chosen experts, gated shared expert) are summed inside that kernel."""
        cfg = self.cfg
        lowp = self.dtype != torch.float32
        x, h = hops.embed_scaled(batch.tokens, self.embed, cfg.embed_scale, rounded=lowp)
        for (L, mixer, mlp, n1, n2, _gw, _gb), cache in zip(self.layers, caches):
            src = h if lowp else x
            out = mixer.forward(src, batch, *cache) if isinstance(cache, tuple) else mixer.forward(src, batch, cache)
            a, ca, b, cb = out if isinstance(out, tuple) else (out, 1.0, None, 1.0)
            h = hops.branch_norm(x, n1, cfg.eps, a=a, ca=ca, b=b, cb=cb, center=self.norm_center, rounded=lowp)
            if mlp is not None:
                src = h if lowp else x
                y = mlp.forward(src, defer=True) if isinstance(mlp, RoutedExperts) else mlp.forward(src)
                h = hops.branch_norm(x, n2, cfg.eps, center=self.norm_center, rounded=lowp, **({"moe": y} if isinstance(y, hops.MoeSum) else {"a": y}))
            if collect is not None:
                collect.append(x.clone())
        hf = hops.norm_rows(x, batch.want, self.final_norm, cfg.eps, center=self.norm_center)
        return hops.dense_linear(hf, self.head, out_dtype=torch.float32, softcap=cfg.logit_softcap)


def load_hybrid_checkpoint(path: str, dtype: torch.dtype, device, page: int = 64) -> HybridModel:
    """A folder with config.json and *.safetensors of the family -> HybridModel on `device`."""
    from .loader import _Shards
    cfg = HybridConfig.from_json(json.load(open(os.path.join(path, "config.json"))))
    sh = _Shards(path)
    return HybridModel(cfg, {k: sh.get(k) for k in sh.map}, dtype, device, page)
