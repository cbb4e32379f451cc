"""Token mixers of the hybrid decoder family, each a mechanism with its constants as parameters:

  * ``PagedChunkAttention`` -- grouped-query attention over the paged cache with a partial rotary embedding of either pair layout, a
    mask that is causal inside blocks of `chunk` positions (0: plain causal), an optional softmax sink (one added to the denominator),
    optional unit-normed values and optional value rotation (values are turned by their own position when cached and the head output
    is turned back by the query's position, so a value enters the sum turned by the distance).  A layer may read the cache that an
    earlier layer with the same geometry wrote (`kv_from`) and then has no key / value projections.  Further options, each off by default:
    a sliding window instead of the block mask, a tanh cap on the scaled scores, a temperature on the queries that grows with the
    logarithm of the position, RMS-normed queries and keys under weights shared by the heads, YaRN-scaled rotary steps, biases on the
    projections, and a sigmoid gate per head on the output.
  * ``GeneralizedDeltaRule`` -- S_t = diag(w_t) S_(t-1) - (a_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T r_t per head with the state in an
    fp32 slot: a per-channel decay w from a low-rank projection, a per-channel removal rate a along the unit key u, heads brought to unit
    RMS under a per-channel weight and gated by a sigmoid.
  * ``GatedLinearRecurrence`` -- S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head with the state in an fp32 slot, in the
    HGRN2 parametrisation (a = f, k = 1 - f with a lower-bounded forget gate f, q = silu) or the gated-linear-attention one
    (a = sigmoid(low-rank z)^(1/tau), q scaled by dim^-1/2, output gate silu(g)); per-head RMS norm of o, then the output projection.

  * ``LatentAttention`` -- attention whose keys and values are linear images of ONE low-rank latent vector per token, plus a rotated key
    part shared by all heads.  Only the normed latent and that key part are cached (one row per token for all heads); the key
    up-projection is moved to the query side and the value up-projection behind the weighted sum, so the paged kernels see multi-query
    attention over the cached rows.  Rotary with optional YaRN frequency scaling, a learned per-head softmax sink, a sigmoid output gate.
  * ``Retention`` -- the same recurrence with one constant decay per head, rotated q and k, unit-RMS heads and a silu output gate.
  * ``LightningAttention`` -- that recurrence with silu on q, k and v, one RMS norm over all heads together and a sigmoid output gate.
  * ``ParallelMixer`` -- two of the mixers side by side on one input, their outputs added with a constant each.
  * ``GatedMLP``, ``PolyNormMLP``, ``RoutedExperts`` -- feed-forward branches: gated dense, dense with the PolyNorm activation, and a
    mixture of gated experts (softmax or sigmoid router, group-limited top-k, optional shared expert with an optional gate of its own) over
    one grouped linear per projection.  The gated activations include the clamped form min(g, L) sigmoid(1.702 min(g, L)) (clamp(u) + 1).

All take the normed activations of a ragged batch (``StepBatch``) and return the fp32 branch output [T, width]."""
import math
from dataclasses import dataclass, field
from typing import Dict, Optional

import torch

from . import hybrid_ops as hops


@dataclass
class RotaryScaling:
    """YaRN: pairs that turn fewer than `slow` times over `original` positions are slowed by `factor`, pairs that turn more than `fast`
    times keep their step, with a linear ramp over the pair index between; cos and sin are multiplied by 0.1 ln(factor) + 1."""
    factor: float
    original: float
    fast: float
    slow: float


@dataclass
class WavelengthScaling:
    """Scaling by wavelength (the Llama 3.1 rule): with l = 2 pi / step, steps with l < original / high stay, steps with l > original / low are divided
    by `factor`, and between the two the step is (1 - s) step / factor + s step with s = (original / l - low) / (high - low).  cos and sin keep
    their magnitude."""
    factor: float
    original: float
    low: float
    high: float


@dataclass
class RotarySpec:
    dims: int
    base: float
    layout: str = "interleaved"          # "interleaved": pairs (2i, 2i+1); "halves": (i, i + dims / 2)
    scaling: Optional[object] = None     # RotaryScaling (YaRN) | WavelengthScaling | None

    @staticmethod
    def from_json(rot: Optional[dict], layout: str, scaling: str = "yarn") -> Optional["RotarySpec"]:
        """scaling: how rot.scaling is read: "yarn" {factor, original, fast, slow} or "wavelength" {factor, original, low, high}."""
        if not rot or not int(rot.get("dims", 0)):
            return None
        sc = rot.get("scaling")
        if not sc:
            spec = None
        elif scaling == "yarn":
            spec = RotaryScaling(float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"]))
        elif scaling == "wavelength":
            spec = WavelengthScaling(float(sc["factor"]), float(sc["original"]), float(sc["low"]), float(sc["high"]))
        else:
            raise ValueError(f"rotary scaling {scaling!r}")
        return RotarySpec(int(rot["dims"]), float(rot["base"]), layout, spec)


@dataclass
class AttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotarySpec] = None
    chunk: int = 0                       # 0: every earlier position is visible
    sink: bool = False                   # exp(0) joins the softmax denominator
    value_norm: bool = False
    value_rot: bool = False
    value_layout: str = "interleaved"
    kv_from: Optional[int] = None
    window: int = 0                      # > 0 (chunk must be 0): position i sees the keys j with 0 <= i - j < window
    softcap: float = 0.0                 # > 0: scaled scores become softcap * tanh(score / softcap)
    q_temp: Optional[tuple] = None       # (coef, every): queries at position p are multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)
    qk_norm: bool = False                # queries and keys are RMS-normed per head under weights [dim] shared by the heads, before the rotation
    bias: bool = False                   # the q, k, v projections have biases
    out_bias: bool = False               # the output projection has a bias
    out_gate: bool = False               # head h's output is multiplied by sigmoid(W_g x)_h, one number per head
    learned_sink: bool = False           # with sink: head h's sink logit is the checkpoint's `sink`[h] instead of 0
    qk_norm_whole: bool = False          # with qk_norm: ONE RMS norm over all query heads (and one over all key heads) under weights [heads * dim]


@dataclass
class RecurrenceSpec:
    kind: str                            # "hgrn2" | "gla"
    heads: int
    dim: int
    vdim: int
    tau: float = 1.0


@dataclass
class DeltaRuleSpec:
    heads: int
    dim: int                             # key channels per head
    vdim: int                            # value channels per head
    decay_mult: float = math.exp(-0.5)   # w = exp(-decay_mult * sigmoid(.)): the decay of a channel stays above exp(-decay_mult)
    unit_eps: float = 1e-6               # u = k / sqrt(|k|^2 + unit_eps)


@dataclass
class StepBatch:
    """One ragged step on the device.  Row r is a token at position pos[r] of sequence seq[r]; sequence s owns rows
    row_start[s] .. row_start[s + 1] - 1 (in position order), the block-table row s and state slot slot[s]; first_pos[s] is the
    position of its first row in this step (0: the sequence starts here and recurrent states start from zero)."""
    tokens: torch.Tensor
    pos: torch.Tensor
    seq: torch.Tensor
    row_start: torch.Tensor
    slot: torch.Tensor
    first_pos: torch.Tensor
    block_table: torch.Tensor
    want: torch.Tensor                   # rows whose logits are computed
    tile_row0: Optional[torch.Tensor] = None   # tiles of at most 16 consecutive rows of one sequence covering every row: first row ...
    tile_n: Optional[torch.Tensor] = None      # ... and row count (the matrix-core attention for prompt portions works on them)
    prev: Optional[torch.Tensor] = None        # the token before each row in its sequence (-1 for a sequence's first token): bigram embeddings
    host: Optional[torch.Tensor] = None        # the pinned buffer all index fields were uploaded from (one copy per step)
    plans: dict = field(default_factory=dict)  # what the step's layers share beyond the index arrays (the chunk plan of the fixed-decay recurrences)
    max_rows: int = 0                          # rows of the step's longest sequence when the host knows them (0: unknown)


def rotary_table(rot: RotarySpec, device):
    """(fp32 angular steps [dims / 2] on the device, magnitude of cos and sin) of a rotary description; evaluated in float64, rounded once."""
    i = torch.arange(rot.dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(rot.base), dtype=torch.float64), -2.0 * i / rot.dims)
    mag, sc = 1.0, rot.scaling
    if isinstance(sc, WavelengthScaling):
        if sc.high <= sc.low or sc.factor <= 0:
            raise ValueError(f"rotary scaling: low {sc.low} high {sc.high} factor {sc.factor}")
        lam = 2.0 * math.pi / f
        blend = (sc.original / lam - sc.low) / (sc.high - sc.low)
        mid = (1.0 - blend) * f / sc.factor + blend * f
        f = torch.where(lam < sc.original / sc.high, f, torch.where(lam > sc.original / sc.low, f / sc.factor, mid))
    elif sc is not None:
        at = lambda turns: rot.dims * math.log(sc.original / (2.0 * math.pi * turns)) / (2.0 * math.log(rot.base))
        lo, hi = max(math.floor(at(sc.fast)), 0), min(math.ceil(at(sc.slow)), rot.dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / sc.factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(sc.factor) + 1.0
    return f.to(torch.float32).to(device), mag


def rotary_steps(n_pairs: int, span: int, base: float, device) -> torch.Tensor:
    """fp32 angular step of pair i: base^(-2 i / span), evaluated in float64 and rounded once."""
    i = torch.arange(n_pairs, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / span).to(torch.float32).to(device)


class PagedChunkAttention:
    """weights: q [H dim, W], k [G dim, W], v [G vdim, W] (absent with kv_from), o [W, H vdim]; by option q.b / k.b / v.b / o.b, q.norm / k.norm [dim]
    (or [H dim] / [G dim] when the norm runs over all heads at once), g [H, W], sink [H].  Every projection of the input (q | k | v | gate) is one
    linear."""

    def __init__(self, spec: AttentionSpec, weights: Dict[str, torch.Tensor], eps: float, page: int, device):
        s = self.spec = spec
        self.eps, self.page = eps, page
        if s.heads % s.kv_heads:
            raise ValueError(f"attention: {s.heads} query heads over {s.kv_heads} key/value heads")
        if s.window and s.chunk:
            raise ValueError("attention: a sliding window and a block mask exclude each other")
        self.owns_cache = s.kv_from is None
        names = ["q"] + (["k", "v"] if self.owns_cache else [])
        parts = [weights[n] for n in names] + ([weights["g"]] if s.out_gate else [])
        self.w_in = torch.cat(parts, 0).contiguous()
        self.b_in = None
        if s.bias:
            zero = [torch.zeros(s.heads, dtype=self.w_in.dtype, device=self.w_in.device)] if s.out_gate else []
            self.b_in = torch.cat([weights[n + ".b"] for n in names] + zero, 0).contiguous()
        self.w_o = weights["o"].contiguous()
        self.b_o = weights["o.b"].contiguous() if s.out_bias else None
        self.koff, self.voff = s.heads * s.dim, (s.heads + s.kv_heads) * s.dim
        self.goff = s.heads * s.dim + ((s.kv_heads * (s.dim + s.vdim)) if self.owns_cache else 0)
        self.q_norm = weights["q.norm"].contiguous() if s.qk_norm else None
        self.k_norm = weights["k.norm"].contiguous() if s.qk_norm and self.owns_cache else None
        rot = s.rot
        self.kfreq, self.mag = rotary_table(rot, device) if rot and rot.dims else (None, 1.0)
        self.vfreq = rotary_steps(s.vdim // 2, s.vdim, rot.base, device) if s.value_rot and rot else None
        self._geom = None
        self.use_tiles = True
        self.sink = None
        if s.sink:
            self.sink = weights["sink"].to(torch.float32).contiguous() if s.learned_sink else torch.zeros(s.heads, dtype=torch.float32, device=device)
            if self.sink.numel() != s.heads:
                raise ValueError(f"attention: {self.sink.numel()} sink logits for {s.heads} heads")
        for t, n in ((self.q_norm, s.heads), (self.k_norm, s.kv_heads)):
            if t is not None and t.numel() != s.dim * (n if s.qk_norm_whole else 1):
                raise ValueError(f"attention: norm weight of {t.numel()} channels for {n} heads of {s.dim} ({'all heads at once' if s.qk_norm_whole else 'per head'})")

    def cache_kind(self):
        return "kv" if self.owns_cache else "kv_from"

    def cache_shapes(self):
        """(K page tensor shape, V page tensor shape) without the leading page count."""
        s = self.spec
        return (s.kv_heads, self.page, s.dim), (s.kv_heads, self.page, s.vdim)

    def geometry(self, max_blocks: int, num_pages: int):
        s = self.spec
        key = (max_blocks, num_pages)
        if self._geom is None or self._geom[0] != key:
            rot = s.rot
            self._geom = (key, hops.attn_geometry(s.heads, s.kv_heads, s.dim, s.vdim, rot.dims if rot else 0,
                                                  hops.LAYOUTS[rot.layout] if rot else 0, hops.LAYOUTS[s.value_layout], self.page, max_blocks,
                                                  num_pages))
        return self._geom[1]

    def forward(self, h: torch.Tensor, batch: StepBatch, kcache: torch.Tensor, vcache: torch.Tensor, proj: Optional[torch.Tensor] = None,
                out_proj: bool = True) -> torch.Tensor:
        """proj: h w_in^T (+ b_in) in fp32 when the caller has computed it (as columns of a linear shared with other projections of h; the query
        columns are turned in place).  out_proj False: the heads' outputs [T, H vdim] come back without the output projection."""
        s = self.spec
        geom = self.geometry(batch.block_table.shape[1], kcache.shape[0])
        qkv = hops.dense_linear(h, self.w_in, self.b_in, out_dtype=torch.float32) if proj is None else proj
        write = self.owns_cache
        hops.attn_prep(qkv, self.koff, self.voff, geom, self.kfreq, self.vfreq, s.value_norm, self.eps, batch.pos, batch.seq, batch.block_table,
                       kcache if write else None, vcache if write else None, q_norm=self.q_norm, k_norm=self.k_norm, mag=self.mag, q_temp=s.q_temp,
                       cache_dtype=kcache.dtype, norm_whole=s.qk_norm_whole)
        T = qkv.shape[0]
        extra = dict(window=s.window, softcap=s.softcap, out_gate=qkv[:, self.goff:self.goff + s.heads] if s.out_gate else None)
        # prompt portions (tiles mostly full) go to the matrix-core kernel, decode rows to the one that spreads a row's keys over four waves
        if (self.use_tiles and batch.tile_row0 is not None and batch.tile_row0.numel() * 4 <= T
                and hops.attn_tiles_supported(kcache.dtype, s.dim, s.vdim, self.vfreq is not None, hops.LAYOUTS[s.value_layout])):
            o = hops.attn_tiles(qkv, s.scale, geom, s.chunk, self.sink, self.vfreq, batch.pos, batch.seq, batch.block_table, batch.tile_row0, batch.tile_n,
                                kcache, vcache, s.heads, s.vdim, **extra)
        else:
            o = hops.attn_rows(qkv, s.scale, geom, s.chunk, self.sink, self.vfreq, batch.pos, batch.seq, batch.block_table, kcache, vcache, s.heads, s.vdim,
                               **extra)
        return hops.dense_linear(o, self.w_o, self.b_o, out_dtype=torch.float32) if out_proj else o


class GeneralizedDeltaRule:
    """weights: r, k, a [H dim, W], v, g [H vdim, W], a.b [H dim], w1 [rank, W], w2 [H dim, rank], w0 [H dim], norm [H vdim], o [W, H vdim].
    One linear gives r | k | v | a (+ bias) | g in fp32; the decay's pre-activation is the low-rank pair w2 tanh(w1 x) + w0.  Decay, removal
    rate, unit key, state and update are fp32 (hybrid_ops.delta_scan); the heads are brought to unit RMS, multiplied by `norm` and by
    sigmoid(g), then projected."""

    def __init__(self, spec: DeltaRuleSpec, weights: Dict[str, torch.Tensor], eps: float):
        s = self.spec = spec
        self.eps = eps
        hd, hv = s.heads * s.dim, s.heads * s.vdim
        for n, shape in (("r", hd), ("k", hd), ("a", hd), ("v", hv), ("g", hv), ("w2", hd)):
            if weights[n].shape[0] != shape:
                raise ValueError(f"delta rule: weight {n} {tuple(weights[n].shape)} for {s.heads} heads of {s.dim} x {s.vdim}")
        self.w_in = torch.cat([weights[n] for n in ("r", "k", "v", "a", "g")], 0).contiguous()
        z = lambda n: torch.zeros(n, dtype=self.w_in.dtype, device=self.w_in.device)
        self.b_in = torch.cat([z(2 * hd + hv), weights["a.b"], z(hv)], 0).contiguous()
        self.ro, self.ko, self.vo, self.ao, self.go = 0, hd, 2 * hd, 2 * hd + hv, 3 * hd + hv
        self.w_w1, self.w_w2, self.b_w = weights["w1"].contiguous(), weights["w2"].contiguous(), weights["w0"].contiguous()
        self.norm, self.w_o = weights["norm"].contiguous(), weights["o"].contiguous()

    def state_shape(self):
        s = self.spec
        return (s.heads, s.dim, s.vdim)

    def forward(self, h: torch.Tensor, batch: StepBatch, state: torch.Tensor) -> torch.Tensor:
        s = self.spec
        proj = hops.dense_linear(h, self.w_in, self.b_in, out_dtype=torch.float32)
        z = hops.dense_linear(hops.dense_linear(h, self.w_w1, act=hops.ACT_TANH), self.w_w2, self.b_w, out_dtype=torch.float32)
        o = hops.delta_scan(proj, self.ro, self.ko, self.vo, self.ao, z, s.decay_mult, s.unit_eps, s.heads, s.dim, s.vdim,
                            batch.row_start, batch.slot, batch.first_pos, state)
        o = hops.head_norm(o, s.heads, s.vdim, self.norm, self.eps, proj, self.go, gate_act="sigmoid")
        return hops.dense_linear(o, self.w_o, out_dtype=torch.float32)


class GatedLinearRecurrence:
    def __init__(self, spec: RecurrenceSpec, weights: Dict[str, torch.Tensor], eps: float):
        s = self.spec = spec
        self.eps = eps
        hd = s.heads * s.dim
        if s.kind == "hgrn2":
            self.w_in = torch.cat([weights["q"], weights["f"], weights["v"]], 0).contiguous()
            self.lower, self.fbias = weights["lower"].contiguous(), weights["f.b"].contiguous()
            self.qo, self.ko, self.vo, self.go = 0, hd, 2 * hd, None
            self.mode = hops.SCAN_HGRN2
        elif s.kind == "gla":
            self.w_in = torch.cat([weights["q"], weights["k"], weights["v"], weights["g"]], 0).contiguous()
            self.w_a1, self.w_a2, self.b_a2 = weights["a1"].contiguous(), weights["a2"].contiguous(), weights["a2.b"].contiguous()
            self.qo, self.ko, self.vo, self.go = 0, hd, 2 * hd, 2 * hd + s.heads * s.vdim
            self.lower = self.fbias = None
            self.mode = hops.SCAN_GLA
        else:
            raise ValueError(f"recurrence kind {s.kind!r}")
        self.norm, self.w_o = weights["norm"].contiguous(), weights["o"].contiguous()
        self.act = self.w_o.dtype

    def state_shape(self):
        s = self.spec
        return (s.heads, s.dim, s.vdim)

    def forward(self, h: torch.Tensor, batch: StepBatch, state: torch.Tensor) -> torch.Tensor:
        s = self.spec
        proj = hops.dense_linear(h, self.w_in, out_dtype=torch.float32)
        z = None
        if self.mode == hops.SCAN_GLA:
            z = hops.dense_linear(hops.dense_linear(h, self.w_a1), self.w_a2, self.b_a2, out_dtype=torch.float32)
        o = hops.scan(self.mode, proj, self.qo, self.ko, self.vo, z, self.lower, self.fbias, s.tau, 1.0 / math.sqrt(s.dim), s.heads, s.dim, s.vdim,
                      batch.row_start, batch.slot, batch.first_pos, state, self.act)
        o = hops.head_norm(o, s.heads, s.vdim, self.norm, self.eps, proj if self.go is not None else None, self.go or 0)
        return hops.dense_linear(o, self.w_o, out_dtype=torch.float32)


@dataclass
class LatentAttentionSpec:
    heads: int
    dim: int                             # un-rotated query / key channels per head
    rot_dim: int                         # rotated channels per head (the key's are shared by all heads)
    vdim: int
    kv_rank: int                         # size of the cached latent
    scale: float
    rot: Optional[RotarySpec] = None     # turns the first rot.dims of the rot_dim channels
    sink: bool = True                    # learned per-head sink logit in the softmax denominator
    out_gate: bool = True                # heads multiplied by sigmoid(W_g h) before the output projection


class LatentAttention:
    """weights: q [H (dim + rot_dim), W], dkv [kv_rank + rot_dim, W], dkv.norm [kv_rank], uk [H dim, kv_rank], uv [H vdim, kv_rank], sink [H],
    g [H vdim, W], o [W, H vdim].  Cached per token: [normed latent | turned shared key part | zeros] in `padded` channels (a multiple of 32,
    so that the matrix-core attention takes the rows); the values are the first kv_rank channels of the same row."""

    def __init__(self, spec: LatentAttentionSpec, weights: Dict[str, torch.Tensor], eps: float, page: int, device):
        s = self.spec = spec
        self.eps, self.page = eps, page
        H, d, dr, R = s.heads, s.dim, s.rot_dim, s.kv_rank
        self.padded = -(-(R + dr) // 32) * 32
        if s.rot is not None and (s.rot.dims > dr or s.rot.layout != "interleaved"):
            raise ValueError(f"latent attention: rotary span {s.rot.dims} of {dr} channels ({s.rot.layout})")
        parts = [weights["q"], weights["dkv"]] + ([weights["g"]] if s.out_gate else [])
        self.w_in = torch.cat(parts, 0).contiguous()
        self.doff, self.goff = H * (d + dr), H * (d + dr) + R + dr
        self.c_norm = weights["dkv.norm"].contiguous()
        # key up-projection on the query side: per head [kv_rank, dim] (q_abs = W_uk,h^T q_h); value up-projection per head [vdim, kv_rank]
        self.w_uk_t = weights["uk"].view(H, d, R).transpose(1, 2).contiguous()
        self.w_uv = weights["uv"].view(H, s.vdim, R).contiguous()
        self.w_o = weights["o"].contiguous()
        self.sink = weights["sink"].to(torch.float32).contiguous() if s.sink else None
        self.freq, self.mag = rotary_table(s.rot, device) if s.rot is not None else (None, 1.0)
        self.act = self.w_o.dtype
        self._geom = None
        self.use_tiles = True

    def cache_shape(self):
        return (self.page, self.padded)

    def geometry(self, max_blocks: int, num_pages: int):
        s = self.spec
        key = (max_blocks, num_pages)
        if self._geom is None or self._geom[0] != key:
            self._geom = (key, hops.attn_geometry(s.heads, 1, self.padded, s.kv_rank, 0, 0, 0, self.page, max_blocks, num_pages, v_ld=self.padded),
                          hops.latent_geometry(s.heads, s.dim, s.rot_dim, s.kv_rank, self.padded, s.rot.dims if s.rot else 0, self.page, max_blocks,
                                               num_pages))
        return self._geom[1], self._geom[2]

    def forward(self, h: torch.Tensor, batch: StepBatch, cache: torch.Tensor, _values=None, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        """proj: h w_in^T in fp32 when the caller has computed it (as columns of a linear shared with other projections of h)."""
        s = self.spec
        H, R = s.heads, s.kv_rank
        ageom, lgeom = self.geometry(batch.block_table.shape[1], cache.shape[0])
        T = h.shape[0]
        if proj is None:
            proj = hops.dense_linear(h, self.w_in, out_dtype=torch.float32)
        qn = torch.empty(T, H * s.dim, dtype=self.act, device=h.device)
        qabs = torch.empty(T, H * self.padded, dtype=torch.float32, device=h.device)
        hops.latent_prep(proj, self.doff, lgeom, self.freq, self.mag, self.c_norm, self.eps, batch.pos, batch.seq, batch.block_table, qn, qabs, cache)
        hops.dense_grouped(qn, self.w_uk_t, x_step=s.dim, y_step=self.padded, out_dtype=torch.float32, out=qabs)
        kc = cache.view(cache.shape[0], 1, self.page, self.padded)
        if (self.use_tiles and batch.tile_row0 is not None and batch.tile_row0.numel() * 4 <= T
                and hops.attn_tiles_supported(cache.dtype, self.padded, R, False, 0)):
            ol = hops.attn_tiles(qabs, s.scale, ageom, 0, self.sink, None, batch.pos, batch.seq, batch.block_table, batch.tile_row0, batch.tile_n, kc, kc, H, R)
        else:
            ol = hops.attn_rows(qabs, s.scale, ageom, 0, self.sink, None, batch.pos, batch.seq, batch.block_table, kc, kc, H, R)
        # value up-projection per head; the output gate sigmoid(W_g h) is applied in its epilogue
        o = hops.dense_grouped(ol, self.w_uv, x_step=R, y_step=s.vdim, mul_sigmoid=proj[:, self.goff:self.goff + H * s.vdim] if s.out_gate else None)
        return hops.dense_linear(o, self.w_o, out_dtype=torch.float32)


@dataclass
class RetentionSpec:
    heads: int
    dim: int
    vdim: int
    decay: tuple                         # one constant decay per head
    rot: Optional[RotarySpec] = None


class Retention:
    """weights: q, k [H dim, W], v, g [H vdim, W], o [W, H vdim].  S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q and k turned by the
    position and k multiplied by dim^-1/2 after the turn; every head's o is brought to unit RMS, the heads are multiplied by silu(W_g h)."""

    def __init__(self, spec: RetentionSpec, weights: Dict[str, torch.Tensor], eps: float, device):
        s = self.spec = spec
        self.eps = eps
        if len(s.decay) != s.heads:
            raise ValueError(f"retention: {len(s.decay)} decays for {s.heads} heads")
        hd = s.heads * s.dim
        self.w_in = torch.cat([weights["q"], weights["k"], weights["v"], weights["g"]], 0).contiguous()
        self.b_in = None
        self.qo, self.ko, self.vo, self.go = 0, hd, 2 * hd, 2 * hd + s.heads * s.vdim
        self.decay = torch.tensor([float(a) for a in s.decay], dtype=torch.float32, device=device)
        self.w_o = weights["o"].contiguous()
        self.act = self.w_o.dtype
        self.freq, self.mag = rotary_table(s.rot, device) if s.rot is not None else (None, 1.0)

    def cache_kind(self):
        return "state"

    def state_shape(self):
        s = self.spec
        return (s.heads, s.dim, s.vdim)

    def forward(self, h: torch.Tensor, batch: StepBatch, state: torch.Tensor, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        """proj: h w_in^T in fp32 when the caller has computed it (as columns of a linear shared with other projections of h)."""
        s = self.spec
        if proj is None:
            proj = hops.dense_linear(h, self.w_in, out_dtype=torch.float32)
        rot = s.rot
        hops.rotary(proj, [(self.qo, s.heads, s.dim, 1.0), (self.ko, s.heads, s.dim, 1.0 / math.sqrt(s.dim))], rot.dims if rot else 0,
                    hops.LAYOUTS[rot.layout] if rot else 0, self.freq, self.mag, batch.pos)
        o = hops.scan(hops.SCAN_FIXED, proj, self.qo, self.ko, self.vo, None, self.decay, None, 1.0, 1.0, s.heads, s.dim, s.vdim,
                      batch.row_start, batch.slot, batch.first_pos, state, self.act, plans=batch.plans, max_rows=batch.max_rows)
        o = hops.head_norm(o, s.heads, s.vdim, None, self.eps, proj, self.go, out_dtype=self.act)
        return hops.dense_linear(o, self.w_o, out_dtype=torch.float32)


@dataclass
class LightningSpec:
    heads: int
    dim: int
    vdim: int
    decay: tuple                         # one constant decay per head


class LightningAttention:
    """weights: q, k [H dim, W], v, g [H vdim, W], norm [H vdim], o [W, H vdim].  Linear attention with a constant decay per head:
    S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q, k, v = silu of their projections and the state in an fp32 slot.  The heads TOGETHER
    are brought to unit RMS under `norm`, multiplied by sigmoid(W_g h) and projected."""

    def __init__(self, spec: LightningSpec, weights: Dict[str, torch.Tensor], eps: float, device):
        s = self.spec = spec
        self.eps = eps
        if len(s.decay) != s.heads:
            raise ValueError(f"lightning attention: {len(s.decay)} decays for {s.heads} heads")
        hd, hv = s.heads * s.dim, s.heads * s.vdim
        for n, rows in (("q", hd), ("k", hd), ("v", hv), ("g", hv)):
            if weights[n].shape[0] != rows:
                raise ValueError(f"lightning attention: weight {n} {tuple(weights[n].shape)} for {s.heads} heads of {s.dim} x {s.vdim}")
        self.w_in = torch.cat([weights["q"], weights["k"], weights["v"], weights["g"]], 0).contiguous()
        self.b_in = None
        self.qo, self.ko, self.vo, self.go = 0, hd, 2 * hd, 2 * hd + hv
        self.decay = torch.tensor([float(a) for a in s.decay], dtype=torch.float32, device=device)
        self.norm = weights["norm"].contiguous()
        if self.norm.numel() != hv:
            raise ValueError(f"lightning attention: norm weight of {self.norm.numel()} channels for {hv}")
        self.w_o = weights["o"].contiguous()
        self.act = self.w_o.dtype

    def cache_kind(self):
        return "state"

    def state_shape(self):
        s = self.spec
        return (s.heads, s.dim, s.vdim)

    def forward(self, h: torch.Tensor, batch: StepBatch, state: torch.Tensor, proj: Optional[torch.Tensor] = None, out_proj: bool = True) -> torch.Tensor:
        """proj: h w_in^T in fp32 when the caller has computed it.  out_proj False: the normed, gated heads [T, H vdim] come back unprojected."""
        s = self.spec
        if proj is None:
            proj = hops.dense_linear(h, self.w_in, out_dtype=torch.float32)
        o = hops.scan(hops.SCAN_FIXED_SILU, proj, self.qo, self.ko, self.vo, None, self.decay, None, 1.0, 1.0, s.heads, s.dim, s.vdim,
                      batch.row_start, batch.slot, batch.first_pos, state, self.act, plans=batch.plans, max_rows=batch.max_rows)
        o = hops.head_norm(o, 1, s.heads * s.vdim, self.norm, self.eps, proj, self.go, gate_act="sigmoid")
        return hops.dense_linear(o, self.w_o, out_dtype=torch.float32) if out_proj else o


class ParallelMixer:
    """Two mixers side by side on the same input: left_scale * left(h) + right_scale * right(h).  Each side is any mixer of this module whose
    forward takes `proj` (its input projections as columns of a shared linear): all projections of h, of both sides, are ONE linear.  The
    layer's cache is the sides' caches one after the other (pages for an attention side, a state slot for a recurrent side).  forward returns
    the two sides' outputs with their scales, (left, left_scale, right, right_scale): the sum is formed by the kernel that ends the sublayer."""

    def __init__(self, left, right, left_scale: float, right_scale: float):
        self.left, self.right, self.left_scale, self.right_scale = left, right, float(left_scale), float(right_scale)
        for m in (left, right):
            if getattr(m, "w_in", None) is None or not hasattr(m, "cache_kind"):
                raise ValueError(f"parallel mixer: {type(m).__name__} cannot run beside another mixer")
        nl = left.w_in.shape[0]
        self.n_left, self.off_right = nl, nl + (-nl) % 4                     # the right side's columns start 16-byte aligned
        wl, wr = left.w_in, right.w_in
        zrow = torch.zeros(self.off_right - nl, wl.shape[1], dtype=wl.dtype, device=wl.device)
        self.w_in = torch.cat([wl, zrow, wr], 0).contiguous()
        self.b_in = None
        if left.b_in is not None or right.b_in is not None:
            zb = lambda n: torch.zeros(n, dtype=wl.dtype, device=wl.device)
            self.b_in = torch.cat([left.b_in if left.b_in is not None else zb(nl), zb(self.off_right - nl),
                                   right.b_in if right.b_in is not None else zb(wr.shape[0])]).contiguous()
        left.w_in = right.w_in = None                                            # live on as rows of the shared weight

    def cache_parts(self):
        """Per side: how many cache tensors its forward takes (2: key and value pages; 1: a state)."""
        return [2 if m.cache_kind() in ("kv", "kv_from") else 1 for m in (self.left, self.right)]

    def forward(self, h: torch.Tensor, batch: StepBatch, *cache):
        nl_c, _ = self.cache_parts()
        proj = hops.dense_linear(h, self.w_in, self.b_in, out_dtype=torch.float32)
        a = self.left.forward(h, batch, *cache[:nl_c], proj=proj[:, :self.n_left])
        b = self.right.forward(h, batch, *cache[nl_c:], proj=proj[:, self.off_right:])
        return a, self.left_scale, b, self.right_scale


class PolyNormMLP:
    """down(a N(z) + b N(z^2) + c N(z^3) + e), z = up h, N = unit RMS over a token's hidden channels; coef = the four numbers (a, b, c, e)."""

    def __init__(self, up: torch.Tensor, down: torch.Tensor, coef: torch.Tensor, eps: float):
        self.w_up, self.w_down = up.contiguous(), down.contiguous()
        self.coef = tuple(float(v) for v in coef.detach().to("cpu", torch.float32).flatten())
        if len(self.coef) != 4:
            raise ValueError(f"PolyNorm takes four coefficients, got {len(self.coef)}")
        self.eps = eps

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        z = hops.dense_linear(h, self.w_up, out_dtype=torch.float32)
        return hops.dense_linear(hops.polynorm(z, self.coef, self.eps, self.w_down.dtype), self.w_down, out_dtype=torch.float32)


@dataclass
class RouterSpec:
    experts: int
    top: int
    groups: int = 1                      # experts form `groups` runs of neighbours ...
    keep: int = 1                        # ... and only those of the `keep` best runs can be chosen
    score: str = "softmax"               # "softmax" over the logits | "sigmoid" of each logit
    group_top: int = 1                   # a run scores as its best expert (1) or as the sum of its two best (2)
    scale: float = 1.0                   # the chosen experts weigh score * scale


class RoutedExperts:
    """Mixture of gated experts down_e(act(gate_e h) * up_e h): fp32 softmax router, group-limited top-k, the chosen experts' outputs weighted
    by their softmax scores (not renormalised), plus an optional shared expert that every token runs.  The (token, choice) pairs are sorted
    by expert on the device and each projection of all experts is one grouped linear; nothing returns to the host."""

    def __init__(self, router: RouterSpec, w_router: torch.Tensor, gates, ups, downs, shared: Optional["GatedMLP"] = None, act: str = "silu",
                 act_param: float = 0.0, shared_gate: Optional[torch.Tensor] = None):
        """act_param: the activation's parameter (the limit of "swiglu_clamp").  shared_gate [1, W]: the shared expert's output is multiplied by
        sigmoid(shared_gate . h), one number per token; its row rides behind the router's in one linear."""
        r = self.router = router
        if r.score not in ("softmax", "sigmoid") or r.group_top not in (1, 2):
            raise ValueError(f"experts: router score {r.score!r}, groups ranked by their best {r.group_top}")
        if len(gates) != r.experts or w_router.shape[0] != r.experts:
            raise ValueError(f"experts: router of {w_router.shape[0]}, {len(gates)} experts, config says {r.experts}")
        if r.experts % r.groups or not 1 <= r.keep <= r.groups or not 1 <= r.top <= (r.experts // r.groups) * r.keep:
            raise ValueError(f"experts: {r.experts} experts in {r.groups} groups, keep {r.keep}, top {r.top}")
        self.w_router = w_router.contiguous()
        self.n_router = r.experts
        if shared_gate is not None:
            if shared is None or shared_gate.numel() != w_router.shape[1]:
                raise ValueError("experts: a gate for the shared expert needs that expert and one weight per input channel")
            pad = torch.zeros((-(r.experts + 1)) % 4, w_router.shape[1], dtype=w_router.dtype, device=w_router.device)
            self.w_router = torch.cat([w_router, shared_gate.reshape(1, -1), pad], 0).contiguous()
        self.shared_gated = shared_gate is not None
        ff, K = gates[0].shape
        pad = (-ff) % 32
        gu, dn = [], []
        for g, u, d in zip(gates, ups, downs):
            if pad:
                z = torch.zeros(pad, K, dtype=g.dtype, device=g.device)
                g, u = torch.cat([g, z]), torch.cat([u, z])
                d = torch.cat([d, torch.zeros(d.shape[0], pad, dtype=d.dtype, device=d.device)], 1)
            gu.append(hops.group_gate_up(g, u)); dn.append(d)
        self.w_gate_up, self.w_down = torch.stack(gu).contiguous(), torch.stack(dn).contiguous()
        self.shared, self.act, self.act_param = shared, hops.ACTIVATIONS[act], float(act_param)

    def forward(self, h: torch.Tensor, logits: Optional[torch.Tensor] = None, defer: bool = False):
        """logits: the router's fp32 logits [T, experts] when the caller has computed them (in a linear shared with other projections of h).
        defer: return the parts of the weighted sum (hybrid_ops.MoeSum) for a residual kernel that forms it, instead of the summed tensor
        (a gated shared expert is always left to that kernel)."""
        r = self.router
        sgate = None
        if logits is None:
            logits = hops.dense_linear(h, self.w_router, out_dtype=torch.float32)
            if self.shared_gated:
                logits, sgate = logits[:, :self.n_router], logits[:, self.n_router]
        ids, wts, offs, src, place, tiles = hops.moe_route_sorted(logits, r.experts, r.groups, r.keep, r.top, sigmoid=r.score == "sigmoid",
                                                                  group_top=r.group_top, scale=r.scale)
        n = ids.numel()
        a = hops.dense_grouped(h, self.w_gate_up, offs=offs, gather=src, tiles=tiles, rows=n, gated=True, act=self.act, act_param=self.act_param)
        y = hops.dense_grouped(a, self.w_down, offs=offs, tiles=tiles, rows=n, out_dtype=torch.float32)
        parts = hops.MoeSum(y, place, wts, self.shared.forward(h) if self.shared is not None else None, sgate)
        if self.shared_gated and not defer:
            raise ValueError("experts: a gated shared expert joins the sum in the kernel that ends the sublayer (defer=True)")
        return parts if defer else hops.moe_combine(parts)


class GatedMLP:
    """down(act(gate h) * up h) with the gate and up weights grouped for the fused epilogue of the dense linear.  Channel counts that are
    not a multiple of 32 are padded with zero channels (zero gate and up rows, zero down columns)."""

    def __init__(self, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, act: str = "relu", act_param: float = 0.0):
        ff, K = gate.shape
        pad = (-ff) % 32
        if pad:
            z = torch.zeros(pad, K, dtype=gate.dtype, device=gate.device)
            gate, up = torch.cat([gate, z]), torch.cat([up, z])
            down = torch.cat([down, torch.zeros(down.shape[0], pad, dtype=down.dtype, device=down.device)], 1)
        self.w_gate_up = hops.group_gate_up(gate, up)
        self.w_down = down.contiguous()
        self.act, self.act_param = hops.ACTIVATIONS[act], float(act_param)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return hops.dense_linear(hops.dense_linear(h, self.w_gate_up, gated=True, act=self.act, act_param=self.act_param), self.w_down, out_dtype=torch.float32)
