"""Tensor-level wrappers over libmi355_hybrid.so: dense linears on checkpoint-layout weights and the kernels of the hybrid decoder
family (csrc/gemm_dense.hip, csrc/hybrid_ops.hip).  As in ``ops``: PyTorch supplies device memory and the current stream, every
function enqueues hand-written HIP kernels and never falls back.  Activations and weights are bfloat16 or float32 (`act`); what the
family keeps in 32-bit (residual stream, projections that feed gates and rotations, recurrent state, logits) is float32 in both."""
import ctypes as C
from typing import Optional

import torch

from . import _C

ACT_NONE, ACT_RELU, ACT_SILU, ACT_GELU_TANH, ACT_TANH, ACT_SWIGLU_CLAMP = 0, 1, 2, 3, 4, 5
ACTIVATIONS = {"none": ACT_NONE, "relu": ACT_RELU, "silu": ACT_SILU, "gelu_tanh": ACT_GELU_TANH, "tanh": ACT_TANH, "swiglu_clamp": ACT_SWIGLU_CLAMP}
SCAN_HGRN2, SCAN_GLA, SCAN_FIXED, SCAN_FIXED_SILU = 0, 1, 2, 3
LAYOUTS = {"interleaved": 0, "halves": 1}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def act_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return _C.ACT_BF16
    if dtype == torch.float32:
        return _C.ACT_F32
    raise _C.Mi355Error(f"hybrid ops run in bfloat16 or float32, not {dtype}")


def _dev(t: torch.Tensor, dtype, name: str):
    if not t.is_cuda:
        raise _C.Mi355Error(f"{name}: tensor must live on the GPU (no CPU path exists)")
    if t.dtype != dtype:
        raise _C.Mi355Error(f"{name}: expected {dtype}, got {t.dtype}")


def _rows(t: torch.Tensor, name: str) -> int:
    """Leading dimension of a 2-D tensor whose rows are contiguous (a column slice of a wider buffer is fine)."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise _C.Mi355Error(f"{name}: expected a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0)


def dense_linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, *, out_dtype: Optional[torch.dtype] = None,
                 gated: bool = False, act: int = ACT_NONE, softcap: float = 0.0, out: Optional[torch.Tensor] = None, act_param: float = 0.0) -> torch.Tensor:
    """y = x @ w.T (+ bias) for w [N, K] in checkpoint layout.  gated: w holds groups of 32 gate rows followed by the 32 up rows of the
    same channels and y [M, N / 2] = act(gate) * up; without `gated`, act applies to the plain output.  out_dtype float32 keeps the accumulator;
    softcap > 0 applies cap * tanh(y / cap).  ACT_SWIGLU_CLAMP (gated only) with L = act_param: g = min(gate, L), u = clamp(up, -L, L),
    y = g sigmoid(1.702 g) (u + 1)."""
    _dev(x, w.dtype, "dense_linear.x"); _dev(w, w.dtype, "dense_linear.w")
    ldx = _rows(x, "dense_linear.x")
    M, K = x.shape
    N = w.shape[0]
    if w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise _C.Mi355Error(f"dense_linear: x {tuple(x.shape)} against w {tuple(w.shape)}")
    if bias is not None:
        _dev(bias, w.dtype, "dense_linear.bias")
        if bias.numel() != N or not bias.is_contiguous():
            raise _C.Mi355Error(f"dense_linear: bias {tuple(bias.shape)} for N={N}")
    if gated and N % 64:
        raise _C.Mi355Error(f"dense_linear: a gated weight has whole groups of 64 rows, N={N}")
    od = out_dtype or w.dtype
    if w.dtype == torch.float32:
        od = torch.float32
    if od not in (torch.float32, w.dtype):
        raise _C.Mi355Error(f"dense_linear: output {od} from {w.dtype} operands")
    n_out = N // 2 if gated else N
    if out is None:
        out = torch.empty(M, n_out, dtype=od, device=x.device)
    else:
        _dev(out, od, "dense_linear.out")
        if out.shape != (M, n_out):
            raise _C.Mi355Error(f"dense_linear: out {tuple(out.shape)} for [{M}, {n_out}]")
    ldy = _rows(out, "dense_linear.out")
    if M == 0:
        return out
    _C.check_hybrid(_C.hybrid_lib().mi355_dense_linear_ex(x.data_ptr(), ldx, M, w.data_ptr(), N, K, _p(bias), out.data_ptr(), ldy,
                                                          1 if od == torch.float32 else 0, 1 if gated else 0, act, float(act_param), float(softcap),
                                                          act_code(w.dtype), _stream()), "dense_linear")
    return out


def group_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[ff, K] gate and up weights -> the [2 ff, K] weight of a gated dense_linear: per 32 channels, 32 gate rows then 32 up rows
    (ff % 32 == 0)."""
    ff, K = gate.shape
    if ff % 32 or up.shape != gate.shape:
        raise ValueError(f"group_gate_up: gate {tuple(gate.shape)} up {tuple(up.shape)} (channels in whole groups of 32)")
    return torch.stack([gate.view(ff // 32, 32, K), up.view(ff // 32, 32, K)], dim=1).reshape(2 * ff, K).contiguous()


def embed(ids: torch.Tensor, table: torch.Tensor, *, prev: Optional[torch.Tensor] = None, bigram: Optional[torch.Tensor] = None, mul_prev: int = 0,
          mul_cur: int = 0, copy: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 stream rows [T, W] of the token ids.  bigram [buckets + 1, W] with prev (int32 [T]: the token before each row in its sequence, -1 for
    a sequence's first token): the row (prev * mul_prev + id * mul_cur) mod buckets of the table is added (its last row for a first token).
    copy: an fp32 [T, W] tensor that receives the same rows."""
    _dev(ids, torch.int32, "embed.ids")
    T, W = ids.numel(), table.shape[1]
    out = torch.empty(T, W, dtype=torch.float32, device=table.device)
    buckets = 0
    if bigram is not None:
        _dev(bigram, table.dtype, "embed.bigram"); _dev(prev, torch.int32, "embed.prev")
        buckets = bigram.shape[0] - 1
        if bigram.dim() != 2 or bigram.shape[1] != W or buckets < 1 or prev.numel() != T or not bigram.is_contiguous():
            raise _C.Mi355Error(f"embed: bigram table {tuple(bigram.shape)} / prev {tuple(prev.shape)} for {T} rows of {W}")
    if copy is not None:
        _dev(copy, torch.float32, "embed.copy")
        if copy.shape != (T, W) or not copy.is_contiguous():
            raise _C.Mi355Error(f"embed: copy {tuple(copy.shape)} for [{T}, {W}]")
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_embed_bigram(ids.data_ptr(), T, table.data_ptr(), W, table.shape[0], out.data_ptr(), _p(prev), _p(bigram),
                                                              buckets, int(mul_prev), int(mul_cur), _p(copy), act_code(table.dtype), _stream()), "hy_embed")
    return out


def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float, *, rounded: bool = False):
    """(fp32 stream rows [T, W] = table[ids] * scale, the same rows in the table's dtype or None): `rounded` asks for the second tensor, the input
    of the first sublayer of a stack whose sublayers read the stream itself."""
    _dev(ids, torch.int32, "embed_scaled.ids")
    T, W = ids.numel(), table.shape[1]
    out = torch.empty(T, W, dtype=torch.float32, device=table.device)
    outh = torch.empty(T, W, dtype=table.dtype, device=table.device) if rounded else None
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_embed_scaled(ids.data_ptr(), T, table.data_ptr(), W, table.shape[0], float(scale), out.data_ptr(), _p(outh),
                                                              act_code(table.dtype), _stream()), "hy_embed_scaled")
    return out, outh


def branch_norm(x: torch.Tensor, w: torch.Tensor, eps: float, *, a: Optional[torch.Tensor] = None, ca: float = 1.0, b: Optional[torch.Tensor] = None,
                cb: float = 1.0, moe: Optional["MoeSum"] = None, center: bool = True, rounded: bool = False) -> Optional[torch.Tensor]:
    """The end of a sublayer whose OUTPUT is normed: x <- x + N(y) * w in place on the fp32 stream, y = ca * a + cb * b + the mixture sum `moe`
    (its `extra` is the shared expert's output, multiplied by sigmoid(moe.extra_gate) per row when that is given).  N: layer norm (center) or RMS
    norm.  -> the new rows in w's dtype when `rounded`, else None."""
    _dev(x, torch.float32, "branch_norm.x")
    T, W = x.shape
    if not x.is_contiguous() or w.numel() != W or not w.is_contiguous():
        raise _C.Mi355Error(f"branch_norm: stream {tuple(x.shape)} (contiguous) against a weight {tuple(w.shape)}")
    sh = sg = None
    ldsg = 0
    if moe is not None:
        _dev(moe.y, torch.float32, "branch_norm.moe.y"); _dev(moe.wts, torch.float32, "branch_norm.moe.wts"); _dev(moe.place_of, torch.int32, "branch_norm.moe.place")
        if moe.wts.shape[0] != T or moe.y.shape != (moe.wts.numel(), W) or moe.place_of.numel() != moe.wts.numel() or not (moe.y.is_contiguous() and moe.wts.is_contiguous()):
            raise _C.Mi355Error(f"branch_norm: mixture sum y {tuple(moe.y.shape)} wts {tuple(moe.wts.shape)} against the stream {tuple(x.shape)}")
        sh, sg = moe.extra, getattr(moe, "extra_gate", None)
        if sg is not None:
            _dev(sg, torch.float32, "branch_norm.moe.extra_gate")
            if sh is None or sg.dim() != 1 or sg.numel() != T:
                raise _C.Mi355Error(f"branch_norm: gate {tuple(sg.shape)} of the shared branch for {T} rows")
            ldsg = sg.stride(0)
    for t, nm in ((a, "a"), (b, "b"), (sh, "shared")):
        if t is not None:
            _dev(t, torch.float32, "branch_norm." + nm)
            if t.shape != x.shape or not t.is_contiguous():
                raise _C.Mi355Error(f"branch_norm.{nm}: {tuple(t.shape)} against the stream {tuple(x.shape)}")
    if a is None and b is None and moe is None:
        raise _C.Mi355Error("branch_norm: no branch")
    h = torch.empty(T, W, dtype=w.dtype, device=x.device) if rounded else None
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_branch_norm(x.data_ptr(), _p(a), float(ca), _p(b), float(cb), _p(sh), _p(sg), ldsg,
                                                             _p(moe.y) if moe else None, _p(moe.place_of) if moe else None, _p(moe.wts) if moe else None,
                                                             moe.wts.shape[1] if moe else 0, None, T, W, w.data_ptr(), 1 if center else 0, float(eps), _p(h),
                                                             act_code(w.dtype), _stream()), "hy_branch_norm")
    return h


def norm_rows(x: torch.Tensor, rows: torch.Tensor, w: torch.Tensor, eps: float, *, center: bool = True) -> torch.Tensor:
    """N(x[rows]) * w in w's dtype for the fp32 stream x (layer norm with `center`, else RMS norm); x is left as it is."""
    _dev(x, torch.float32, "norm_rows.x"); _dev(rows, torch.int32, "norm_rows.rows")
    W = x.shape[1]
    if not x.is_contiguous() or w.numel() != W or not w.is_contiguous():
        raise _C.Mi355Error(f"norm_rows: stream {tuple(x.shape)} (contiguous) against a weight {tuple(w.shape)}")
    n = rows.numel()
    h = torch.empty(n, W, dtype=w.dtype, device=x.device)
    if n:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_branch_norm(x.data_ptr(), None, 1.0, None, 1.0, None, None, 0, None, None, None, 0, rows.data_ptr(), n, W,
                                                             w.data_ptr(), 1 if center else 0, float(eps), h.data_ptr(), act_code(w.dtype), _stream()),
                        "hy_norm_rows")
    return h


def depth_mix_norm(x: torch.Tensor, a: Optional[torch.Tensor], stack: torch.Tensor, n: int, coef: torch.Tensor, w1: Optional[torch.Tensor], eps: float, *,
                   weight_offset: float = 0.0, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """The end of layer n - 1 of a stack whose layers read a weighted average of ALL earlier results: stack[n] <- x + a (the layer's own result; a may
    be None), x <- sum_{j <= n} coef[j] * stack[j] (fp32, in the order of j), then the RMS norm of the new rows under w1 -> h1 in the weight's dtype
    (None without w1).  stack fp32 [>= n + 1, T, W] holds the embedding output and the results of the layers before; coef fp32 [n + 1] on the device.
    rows (int32): only these rows are formed and nothing is written back (the final norm of the rows whose logits are wanted)."""
    _dev(x, torch.float32, "depth_mix_norm.x"); _dev(stack, torch.float32, "depth_mix_norm.stack"); _dev(coef, torch.float32, "depth_mix_norm.coef")
    T, W = x.shape
    if stack.dim() != 3 or stack.shape[1:] != (T, W) or stack.shape[0] < n + 1 or not stack.is_contiguous() or not x.is_contiguous() or coef.numel() != n + 1:
        raise _C.Mi355Error(f"depth_mix_norm: stack {tuple(stack.shape)} coef {tuple(coef.shape)} for entry {n} of a stream {tuple(x.shape)}")
    if a is not None:
        _dev(a, torch.float32, "depth_mix_norm.a")
        if a.shape != x.shape or not a.is_contiguous():
            raise _C.Mi355Error(f"depth_mix_norm.a: {tuple(a.shape)} against the stream {tuple(x.shape)}")
    if rows is not None:
        _dev(rows, torch.int32, "depth_mix_norm.rows")
    if w1 is not None and w1.numel() != W:
        raise _C.Mi355Error(f"depth_mix_norm: weight {tuple(w1.shape)} for width {W}")
    cnt = T if rows is None else rows.numel()
    h1 = torch.empty(cnt, W, dtype=w1.dtype, device=x.device) if w1 is not None else None
    if cnt:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_depth_mix_norm(x.data_ptr(), _p(a), stack.data_ptr(), T * W, n, coef.data_ptr(), _p(rows), cnt, W, _p(w1),
                                                                float(weight_offset), float(eps), _p(h1), act_code(w1.dtype if w1 is not None else torch.float32),
                                                                _stream()), "hy_depth_mix_norm")
    return h1


class MoeSum:
    """A mixture's weighted sum still to be formed: sum_k wts[t, k] * y[place_of[t, k]] (+ extra[t]).  residual_norm takes it as a branch and
    forms it while it updates the stream; moe_combine forms it on its own.  extra_gate (fp32 [T], any stride): extra[t] is multiplied by
    sigmoid(extra_gate[t]) (branch_norm forms that)."""

    def __init__(self, y: torch.Tensor, place_of: torch.Tensor, wts: torch.Tensor, extra: Optional[torch.Tensor] = None,
                 extra_gate: Optional[torch.Tensor] = None):
        self.y, self.place_of, self.wts, self.extra, self.extra_gate = y, place_of, wts, extra, extra_gate


def residual_norm(x: torch.Tensor, a: Optional[torch.Tensor], b, mult: float, w1: torch.Tensor,
                  w2: Optional[torch.Tensor], eps: float, *, weight_offset: float = 0.0, rows: Optional[torch.Tensor] = None,
                  gate: Optional[torch.Tensor] = None):
    """x <- x + mult * (a + b) on the fp32 stream (in place; skipped for absent branches, and x is only read when `rows` gathers), then
    RMS norms of the new rows under w1 and w2 (stored weight + weight_offset).  -> (h1, h2) in the weights' dtype.
    gate: fp32 [T, >= 2 W] pre-activations; a is multiplied by sigmoid(gate[:, :W]) and b by sigmoid(gate[:, W:2W]) before they are added."""
    _dev(x, torch.float32, "residual_norm.x")
    W = x.shape[1]
    n = x.shape[0] if rows is None else rows.numel()
    ms = None
    if isinstance(b, MoeSum):                 # b: a tensor, or the parts of a mixture's sum
        ms, b = b, b.extra
        _dev(ms.y, torch.float32, "residual_norm.moe.y"); _dev(ms.wts, torch.float32, "residual_norm.moe.wts"); _dev(ms.place_of, torch.int32, "residual_norm.moe.place")
        if ms.wts.shape[0] != x.shape[0] or ms.y.shape != (ms.wts.numel(), W) or ms.place_of.numel() != ms.wts.numel() or not (ms.y.is_contiguous() and ms.wts.is_contiguous()):
            raise _C.Mi355Error(f"residual_norm: mixture sum y {tuple(ms.y.shape)} wts {tuple(ms.wts.shape)} against the stream {tuple(x.shape)}")
    for t, nm in ((a, "a"), (b, "b")):
        if t is not None:
            _dev(t, torch.float32, "residual_norm." + nm)
            if t.shape != x.shape or not t.is_contiguous():
                raise _C.Mi355Error(f"residual_norm.{nm}: {tuple(t.shape)} against the stream {tuple(x.shape)}")
    if rows is not None:
        _dev(rows, torch.int32, "residual_norm.rows")
    ldg = 0
    if gate is not None:
        _dev(gate, torch.float32, "residual_norm.gate")
        ldg = _rows(gate, "residual_norm.gate")
        if gate.shape[0] != x.shape[0] or gate.shape[1] < 2 * W:
            raise _C.Mi355Error(f"residual_norm.gate: {tuple(gate.shape)} for two gates of the stream {tuple(x.shape)}")
    if not x.is_contiguous() or w1.numel() != W or (w2 is not None and (w2.numel() != W or w2.dtype != w1.dtype)):
        raise _C.Mi355Error("residual_norm: stream must be contiguous and the weights [W] of one dtype")
    h1 = torch.empty(n, W, dtype=w1.dtype, device=x.device)
    h2 = torch.empty(n, W, dtype=w1.dtype, device=x.device) if w2 is not None else None
    if n:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_gated_residual_norm(x.data_ptr(), _p(a), _p(b), _p(gate), ldg, float(mult), _p(rows), n, W,
                                                                     w1.data_ptr(), _p(w2), float(weight_offset), float(eps), h1.data_ptr(), _p(h2),
                                                                     _p(ms.y) if ms else None, _p(ms.place_of) if ms else None, _p(ms.wts) if ms else None,
                                                                     ms.wts.shape[1] if ms else 0, act_code(w1.dtype), _stream()), "hy_residual_norm")
    return h1, h2


def attn_geometry(heads, kv_heads, dim, vdim, rot_dims, rot_layout, v_layout, page, max_blocks, num_pages, v_ld=0):
    """v_ld: row stride of the value cache in elements (0: vdim; wider when the value rows are a leading part of wider cached rows)."""
    return (C.c_int32 * 11)(heads, kv_heads, dim, vdim, rot_dims, rot_layout, v_layout, page, max_blocks, num_pages, v_ld)


def attn_prep(qkv: torch.Tensor, koff: int, voff: int, geom, kfreq, vfreq, v_norm: bool, eps: float, pos, seq, block_table,
              kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor], *, q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
              mag: float = 1.0, q_temp=None, cache_dtype: Optional[torch.dtype] = None, norm_whole: bool = False):
    """Rotate the query heads of qkv (fp32 [T, ld], in place); with caches: rotate the keys, unit-norm and rotate the values, and write both
    to their pages.  q_norm / k_norm ([dim] in the cache dtype): queries / keys are brought to unit RMS per head and multiplied by the weight
    before the rotation; mag multiplies cos and sin; q_temp = (coef, every): queries are multiplied by 1 + coef ln(floor((p + 1) / every) + 1).
    norm_whole: q_norm is [heads * dim] and k_norm [kv_heads * dim], and the unit RMS is taken over all heads of the row at once."""
    _dev(qkv, torch.float32, "attn_prep.qkv")
    ld = _rows(qkv, "attn_prep.qkv")
    T = qkv.shape[0]
    if not T:
        return
    dt = kcache.dtype if kcache is not None else (cache_dtype or torch.float32)
    for t, nm in ((q_norm, "q_norm"), (k_norm, "k_norm")):
        if t is not None:
            _dev(t, dt, "attn_prep." + nm)
            want = geom[2] * ((geom[0] if nm == "q_norm" else geom[1]) if norm_whole else 1)
            if t.numel() != want or not t.is_contiguous():
                raise _C.Mi355Error(f"attn_prep.{nm}: {tuple(t.shape)} for {want} channels")
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp else (0.0, 1)
    _C.check_hybrid(_C.hybrid_lib().mi355_hy_attn_prep_ex2(qkv.data_ptr(), ld, koff, voff, geom, _p(kfreq), _p(vfreq), 1 if v_norm else 0, float(eps),
                                                           pos.data_ptr(), seq.data_ptr(), _p(block_table), T, _p(kcache), _p(vcache), _p(q_norm), _p(k_norm),
                                                           1 if norm_whole else 0, float(mag), coef, every, act_code(dt), _stream()), "hy_attn_prep")


def _sink(sink: Optional[torch.Tensor], heads: int):
    if sink is not None:
        _dev(sink, torch.float32, "attention.sink")
        if sink.numel() != heads or not sink.is_contiguous():
            raise _C.Mi355Error(f"attention.sink: {tuple(sink.shape)} for {heads} heads")
    return _p(sink)


def _ogate(gate: Optional[torch.Tensor], T: int, heads: int, name: str):
    if gate is None:
        return None, 0
    _dev(gate, torch.float32, name)
    ld = _rows(gate, name)
    if gate.shape != (T, heads):
        raise _C.Mi355Error(f"{name}: {tuple(gate.shape)} for {T} rows of {heads} heads")
    return gate.data_ptr(), ld


def attn_rows(q: torch.Tensor, scale: float, geom, chunk: int, sink: Optional[torch.Tensor], vfreq, pos, seq, block_table, kcache, vcache,
              heads: int, vdim: int, *, window: int = 0, softcap: float = 0.0, out_gate: Optional[torch.Tensor] = None):
    """Attention of every row over its sequence's pages -> [T, heads * vdim] in the cache dtype.  sink: fp32 [heads] or None; exp(sink[h])
    joins head h's softmax denominator.  Few rows over long block tables (decode steps) are dealt over several blocks per (row, head) whose
    partial sums a second launch merges; the count depends on the rows and the table's width only.  window > 0: a row at position i sees
    the keys j with 0 <= i - j < window; softcap > 0: cap * tanh(score / cap) on the scaled scores; out_gate fp32 [T, heads] (a column slice is
    fine): head h of a row is multiplied by the sigmoid of its entry."""
    _dev(q, torch.float32, "attn_rows.q")
    T = q.shape[0]
    out = torch.empty(T, heads * vdim, dtype=kcache.dtype, device=q.device)
    splits, parts = 1, None
    gp, ldg = _ogate(out_gate, T, heads, "attn_rows.out_gate")
    if chunk == 0 and T * heads <= 2048:                   # sixteen waves per block: one 64-key tile per wave and block where the chip has room
        tiles = (block_table.shape[1] * geom[7] + 63) // 64
        if window > 0:
            tiles = min(tiles, (window + 63) // 64 + 1)
        splits = max(1, min(16, (tiles + 15) // 16, 1024 // (T * heads)))
        if splits > 1:
            parts = torch.empty(T * heads * splits * (vdim + 2), dtype=torch.float32, device=q.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_attn_rows_ex(q.data_ptr(), _rows(q, "attn_rows.q"), float(scale), geom, int(chunk), _sink(sink, heads), _p(vfreq),
                                                              pos.data_ptr(), seq.data_ptr(), block_table.data_ptr(), T, kcache.data_ptr(), vcache.data_ptr(),
                                                              out.data_ptr(), splits, _p(parts), int(window), float(softcap), gp, ldg, act_code(kcache.dtype),
                                                              _stream()), "hy_attn_rows")
    return out


def attn_tiles_supported(dtype: torch.dtype, dim: int, vdim: int, value_rot: bool, v_layout: int) -> bool:
    """Shapes the MFMA kernel for prompt portions takes (attn_rows serves every other)."""
    return dtype == torch.bfloat16 and dim % 32 == 0 and dim <= 256 and vdim % 16 == 0 and vdim <= 256 and not (value_rot and v_layout and vdim % 32)


def attn_tiles(q: torch.Tensor, scale: float, geom, chunk: int, sink: Optional[torch.Tensor], vfreq, pos, seq, block_table, tile_row0, tile_n, kcache, vcache,
               heads: int, vdim: int, *, window: int = 0, softcap: float = 0.0, out_gate: Optional[torch.Tensor] = None):
    """attn_rows for prompt portions on the matrix cores: tile t = rows tile_row0[t] .. + tile_n[t] - 1 (at most 16 consecutive rows of one
    sequence); every row of the batch must lie in exactly one tile."""
    _dev(q, torch.float32, "attn_tiles.q"); _dev(tile_row0, torch.int32, "attn_tiles.tile_row0"); _dev(tile_n, torch.int32, "attn_tiles.tile_n")
    T = q.shape[0]
    out = torch.empty(T, heads * vdim, dtype=kcache.dtype, device=q.device)
    gp, ldg = _ogate(out_gate, T, heads, "attn_tiles.out_gate")
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_attn_tiles_ex(q.data_ptr(), _rows(q, "attn_tiles.q"), float(scale), geom, int(chunk), _sink(sink, heads), _p(vfreq),
                                                               pos.data_ptr(), seq.data_ptr(), block_table.data_ptr(), tile_row0.data_ptr(), tile_n.data_ptr(),
                                                               tile_row0.numel(), kcache.data_ptr(), vcache.data_ptr(), out.data_ptr(), int(window),
                                                               float(softcap), gp, ldg, act_code(kcache.dtype), _stream()), "hy_attn_tiles")
    return out


SCAN_CHUNK = 64            # tokens per chunk of the chunked form of the fixed-decay recurrence ...
SCAN_CHUNKED_FROM = 256    # ... which a step takes when its longest sequence has at least this many rows and the walk would leave the chip idle
SCAN_CHUNK_BYTES = 512 << 20
SCAN_BLOCKS_AT_ONCE = 512  # blocks of the scan kernel the chip runs side by side (two per compute unit)


def scan_prefers_chunks(T: int, nseq: int, max_rows: int, heads: int, vdim: int, C: int) -> bool:
    """Whether the chunked form is expected to be faster: the token-by-token walk takes (rounds of blocks) x (rows of the longest sequence)
    token steps, the chunked form two passes of (rounds of blocks over all chunks) x (chunk size)."""
    longest = max_rows if max_rows > 0 else T - (nseq - 1)
    if longest < SCAN_CHUNKED_FROM:
        return False
    per = heads * ((vdim + 63) // 64)
    rounds = lambda blocks: -(-blocks // SCAN_BLOCKS_AT_ONCE)
    return 2 * rounds((T // C + nseq + 1) * per) * C < rounds(nseq * per) * longest


class ChunkPlan:
    """Chunks of a step's sequences for the chunked recurrence: device index arrays (see mi355_hy_chunk_plan) for one (row_start, chunk size)."""

    def __init__(self, row_start: torch.Tensor, T: int, nseq: int, C: int):
        self.C, self.max_chunks = C, T // C + nseq + 1
        n = self.max_chunks
        buf = torch.empty(4 * n + 1 + nseq + 1, dtype=torch.int32, device=row_start.device)
        self.cs, self.sc, self.ids, self.zeros, self.ones = buf[:n + 1], buf[n + 1:n + 2 + nseq], buf[n + 2 + nseq:2 * n + 2 + nseq], \
            buf[2 * n + 2 + nseq:3 * n + 2 + nseq], buf[3 * n + 2 + nseq:4 * n + 2 + nseq]
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_chunk_plan(row_start.data_ptr(), nseq, C, n, self.cs.data_ptr(), self.sc.data_ptr(), self.ids.data_ptr(),
                                                            self.zeros.data_ptr(), self.ones.data_ptr(), _stream()), "hy_chunk_plan")


def scan(mode: int, proj: torch.Tensor, qo: int, ko: int, vo: int, z: Optional[torch.Tensor], lower, fbias, tau: float, qscale: float,
         heads: int, dim: int, vdim: int, row_start, slot, first_pos, state: torch.Tensor, act: torch.dtype, *, plans: Optional[dict] = None,
         chunked: Optional[bool] = None, max_rows: int = 0) -> torch.Tensor:
    """Gated linear recurrence over the rows of every sequence, continuing (and leaving) the fp32 state of its slot -> fp32 [T, heads * vdim].
    The modes with a constant decay per head (SCAN_FIXED, SCAN_FIXED_SILU) run long prompt portions in chunks that are walked side by side
    (every chunk from a zero state, a prefix over each sequence's chunks, then the chunk-start states' share of the outputs): the same sums in
    another order.  They do so when that is expected to be faster (scan_prefers_chunks: few long sequences; max_rows = the rows of the step's
    longest sequence when the caller knows it).  plans: a dict that keeps the step's chunk plan between calls (the layers of one step share
    it); chunked forces the choice."""
    _dev(proj, torch.float32, "scan.proj"); _dev(state, torch.float32, "scan.state")
    T = proj.shape[0]
    out = torch.empty(T, heads * vdim, dtype=torch.float32, device=proj.device)
    nseq = slot.numel()
    if not (T and nseq):
        return out
    lib, ld = _C.hybrid_lib(), _rows(proj, "scan.proj")

    def run(m, rs, sl, fp, n, st):
        _C.check_hybrid(lib.mi355_hy_scan(m, proj.data_ptr(), ld, qo, ko, vo, _p(z), 0 if z is None else _rows(z, "scan.z"), _p(lower), _p(fbias), float(tau),
                                          float(qscale), heads, dim, vdim, rs.data_ptr(), sl.data_ptr(), fp.data_ptr(), n, st.data_ptr(), out.data_ptr(),
                                          act_code(act), _stream()), "hy_scan")

    fixed = mode in (SCAN_FIXED, SCAN_FIXED_SILU)
    if chunked is None:
        chunked = fixed and scan_prefers_chunks(T, nseq, max_rows, heads, vdim, SCAN_CHUNK)
    if not chunked:
        run(mode, row_start, slot, first_pos, nseq, state)
        return out
    if not fixed or not state.is_contiguous() or state.shape[1:] != (heads, dim, vdim):
        raise _C.Mi355Error(f"scan: the chunked form takes a constant decay per head and a contiguous state [slots, {heads}, {dim}, {vdim}]")
    _dev(lower, torch.float32, "scan.decay")
    C = SCAN_CHUNK
    while (T // C + nseq + 1) * heads * dim * vdim * 4 > SCAN_CHUNK_BYTES and C < T:
        C *= 2
    key = (row_start.data_ptr(), T, nseq, C)
    plan = plans.get(key) if plans is not None else None
    if plan is None:
        plan = ChunkPlan(row_start, T, nseq, C)
        if plans is not None:
            plans.clear()
            plans[key] = plan
    cstate = torch.empty(plan.max_chunks, heads, dim, vdim, dtype=torch.float32, device=proj.device)
    run(mode, plan.cs, plan.ids, plan.zeros, plan.max_chunks, cstate)                       # 1: every chunk from a zero state
    _C.check_hybrid(lib.mi355_hy_chunk_prefix(plan.cs.data_ptr(), plan.sc.data_ptr(), slot.data_ptr(), first_pos.data_ptr(), nseq, lower.data_ptr(), heads,
                                              dim * vdim, cstate.data_ptr(), state.data_ptr(), _stream()), "hy_chunk_prefix")        # 2: states at the chunks' starts
    run(mode + 4, plan.cs, plan.ids, plan.ones, plan.max_chunks, cstate)                    # 3: their share of the outputs
    return out


def delta_scan(proj: torch.Tensor, ro: int, ko: int, vo: int, ao: int, z: torch.Tensor, decay_mult: float, unit_eps: float, heads: int, dim: int,
               vdim: int, row_start, slot, first_pos, state: torch.Tensor) -> torch.Tensor:
    """Generalized delta rule over the rows of every sequence: S <- diag(w) S - (a * u)(u^T S) + k v^T (both terms from the old state), o = S^T r,
    with w = exp(-decay_mult * sigmoid(z)), a = sigmoid(proj[:, ao:]), u = k / sqrt(|k|^2 + unit_eps) per head; r, k (heads x dim) and v (heads x
    vdim) are fp32 columns ro, ko, vo of proj, z fp32 [T, heads * dim].  Continues and leaves the fp32 state [slots, heads, dim, vdim] of each
    sequence's slot -> fp32 [T, heads * vdim]."""
    _dev(proj, torch.float32, "delta_scan.proj"); _dev(state, torch.float32, "delta_scan.state"); _dev(z, torch.float32, "delta_scan.z")
    T = proj.shape[0]
    ld, ldz = _rows(proj, "delta_scan.proj"), _rows(z, "delta_scan.z")
    hd = heads * dim
    if max(ro, ko, ao) + hd > proj.shape[1] or vo + heads * vdim > proj.shape[1] or z.shape != (T, hd) or state.shape[1:] != (heads, dim, vdim) or not state.is_contiguous():
        raise _C.Mi355Error(f"delta_scan: proj {tuple(proj.shape)} z {tuple(z.shape)} state {tuple(state.shape)} for {heads} heads of {dim} x {vdim}")
    out = torch.empty(T, heads * vdim, dtype=torch.float32, device=proj.device)
    nseq = slot.numel()
    if T and nseq:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_delta_scan(proj.data_ptr(), ld, ro, ko, vo, ao, z.data_ptr(), ldz, float(decay_mult), float(unit_eps), heads, dim,
                                                            vdim, row_start.data_ptr(), slot.data_ptr(), first_pos.data_ptr(), nseq, state.data_ptr(),
                                                            out.data_ptr(), _stream()), "hy_delta_scan")
    return out


def head_norm(o: torch.Tensor, heads: int, vdim: int, w: Optional[torch.Tensor], eps: float, gate: Optional[torch.Tensor] = None, goff: int = 0,
              out_dtype: Optional[torch.dtype] = None, gate_act: str = "silu") -> torch.Tensor:
    """Per-head RMS norm of o (fp32 [T, heads * vdim]) under the weight w ([vdim] shared by the heads, or [heads * vdim]; None: unit RMS only,
    output in `out_dtype`), times gate_act(gate[:, goff:]) ("silu" or "sigmoid") when a gate is given."""
    _dev(o, torch.float32, "head_norm.o")
    T = o.shape[0]
    dt = w.dtype if w is not None else out_dtype
    out = torch.empty(T, heads * vdim, dtype=dt, device=o.device)
    per_head = 0
    if w is not None:
        if w.numel() not in (vdim, heads * vdim) or not w.is_contiguous():
            raise _C.Mi355Error(f"head_norm: weight {tuple(w.shape)} for {heads} heads of {vdim}")
        per_head = 1 if w.numel() == heads * vdim and heads > 1 else 0
    if gate_act not in ("silu", "sigmoid"):
        raise _C.Mi355Error(f"head_norm: gate activation {gate_act!r}")
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_head_norm_ex(o.data_ptr(), T, heads, vdim, _p(w), float(eps), _p(gate),
                                                              0 if gate is None else _rows(gate, "head_norm.gate"), goff, out.data_ptr(), per_head,
                                                              1 if gate_act == "sigmoid" else 0, act_code(dt), _stream()), "hy_head_norm")
    return out


def dense_grouped(x: torch.Tensor, w: torch.Tensor, *, x_step: int = 0, y_step: int = 0, offs: Optional[torch.Tensor] = None,
                  gather: Optional[torch.Tensor] = None, tiles: Optional[torch.Tensor] = None, rows: Optional[int] = None, out_dtype: Optional[torch.dtype] = None, gated: bool = False,
                  act: int = ACT_NONE, out: Optional[torch.Tensor] = None, mul_sigmoid: Optional[torch.Tensor] = None, act_param: float = 0.0) -> torch.Tensor:
    """One launch of G = w.shape[0] linears with the weights w [G, N, K].  mul_sigmoid: fp32 [M, width of the output] pre-activations (a column
    slice of a wider buffer is fine); every output is multiplied by the sigmoid of its entry before it is stored.
    Without offs every group takes all rows of x, reads its K inputs from column g * x_step and writes its outputs from column g * y_step
    (per-head projections).  With offs (int32 [G + 1] on the device) the `rows` rows of the output are sorted by group, group g owns rows
    offs[g] .. offs[g + 1] - 1, and sorted row r reads x[gather[r]] (x[r] without gather): the experts of a mixture.  tiles: the list of
    64-row tiles that hold rows, as moe_align writes it (without it every group is launched over all row tiles)."""
    _dev(x, w.dtype, "dense_grouped.x"); _dev(w, w.dtype, "dense_grouped.w")
    if w.dim() != 3 or not w.is_contiguous():
        raise _C.Mi355Error(f"dense_grouped: weights {tuple(w.shape)} must be contiguous [G, N, K]")
    G, N, K = w.shape
    ldx = _rows(x, "dense_grouped.x")
    M = x.shape[0] if rows is None else int(rows)
    if gated and N % 64:
        raise _C.Mi355Error(f"dense_grouped: a gated weight has whole groups of 64 rows, N={N}")
    n_out = N // 2 if gated else N
    od = torch.float32 if w.dtype == torch.float32 else (out_dtype or w.dtype)
    width = y_step * (G - 1) + n_out if offs is None else n_out
    if out is None:
        out = torch.empty(M, width, dtype=od, device=x.device)
    else:
        _dev(out, od, "dense_grouped.out")
        if out.shape[0] != M or out.shape[1] < width:
            raise _C.Mi355Error(f"dense_grouped: out {tuple(out.shape)} for [{M}, {width}]")
    if x.shape[1] < x_step * (G - 1) + K:
        raise _C.Mi355Error(f"dense_grouped: x {tuple(x.shape)} for {G} groups of K={K} at step {x_step}")
    for t, nm in ((offs, "offs"), (gather, "gather"), (tiles, "tiles")):
        if t is not None:
            _dev(t, torch.int32, "dense_grouped." + nm)
    if offs is not None and offs.numel() != G + 1:
        raise _C.Mi355Error(f"dense_grouped: offs has {offs.numel()} entries for {G} groups")
    if gather is not None and gather.numel() < M:
        raise _C.Mi355Error(f"dense_grouped: gather has {gather.numel()} entries for {M} rows")
    ldg = 0
    if mul_sigmoid is not None:
        _dev(mul_sigmoid, torch.float32, "dense_grouped.mul_sigmoid")
        ldg = _rows(mul_sigmoid, "dense_grouped.mul_sigmoid")
        if mul_sigmoid.shape != (M, width):
            raise _C.Mi355Error(f"dense_grouped: gate {tuple(mul_sigmoid.shape)} for outputs [{M}, {width}]")
    if M:
        _C.check_hybrid(_C.hybrid_lib().mi355_dense_grouped_ex(x.data_ptr(), ldx, M, w.data_ptr(), N, K, None, out.data_ptr(), _rows(out, "dense_grouped.out"),
                                                               1 if od == torch.float32 else 0, 1 if gated else 0, act, float(act_param), act_code(w.dtype), G, x_step,
                                                               y_step, _p(offs), _p(gather), _p(tiles), 0 if tiles is None else (tiles.numel() - 1) // 2,
                                                               _p(mul_sigmoid), ldg, 0, _stream()),
                        "dense_grouped")
    return out


def latent_geometry(heads, dim, rot_dim, rank, padded, rot_span, page, max_blocks, num_pages):
    return (C.c_int32 * 9)(heads, dim, rot_dim, rank, padded, rot_span, page, max_blocks, num_pages)


def latent_prep(proj: torch.Tensor, doff: int, geom, freq, mag: float, cw: torch.Tensor, eps: float, pos, seq, block_table, qn: torch.Tensor,
                qabs: torch.Tensor, cache: torch.Tensor):
    """Latent attention, before the scores: from the fp32 projections [T, ld] (query heads from column 0, down projection from column doff) write
    the token's cached row [normed latent | turned shared key part | zeros], the un-rotated query parts (qn, activation dtype) and the turned
    query parts + padding into columns rank.. of every head's absorbed query row (qabs fp32)."""
    _dev(proj, torch.float32, "latent_prep.proj"); _dev(qabs, torch.float32, "latent_prep.qabs")
    _dev(qn, cache.dtype, "latent_prep.qn"); _dev(cw, cache.dtype, "latent_prep.norm")
    T = proj.shape[0]
    H, dim, dr, R, dpad = geom[0], geom[1], geom[2], geom[3], geom[4]
    if qn.shape != (T, H * dim) or qabs.shape != (T, H * dpad) or not qn.is_contiguous() or not qabs.is_contiguous() or cw.numel() != R:
        raise _C.Mi355Error(f"latent_prep: qn {tuple(qn.shape)} qabs {tuple(qabs.shape)} norm {tuple(cw.shape)}")
    if cache.dim() != 3 or cache.shape[1:] != (geom[6], dpad) or cache.shape[0] != geom[8] or not cache.is_contiguous():
        raise _C.Mi355Error(f"latent_prep: cache {tuple(cache.shape)} against pages of {geom[6]} rows of {dpad}")
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_latent_prep(proj.data_ptr(), _rows(proj, "latent_prep.proj"), doff, geom, _p(freq), float(mag), cw.data_ptr(),
                                                             float(eps), pos.data_ptr(), seq.data_ptr(), block_table.data_ptr(), T, qn.data_ptr(),
                                                             qabs.data_ptr(), cache.data_ptr(), act_code(cache.dtype), _stream()), "hy_latent_prep")


def rotary(buf: torch.Tensor, segments, rot_dims: int, layout: int, freq: torch.Tensor, mag: float, pos: torch.Tensor):
    """Turn, in place, the first rot_dims channels of every head of up to two segments (column, heads, head size, scale) of the fp32 rows of buf
    by position * freq (cos and sin times mag); a segment's heads are multiplied by its scale afterwards."""
    _dev(buf, torch.float32, "rotary.buf")
    segs = list(segments) + [(0, 0, 0, 1.0)] * (2 - len(segments))
    if len(segs) != 2:
        raise _C.Mi355Error("rotary: one or two segments")
    if buf.shape[0]:
        (o0, h0, d0, s0), (o1, h1, d1, s1) = segs
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_rotary(buf.data_ptr(), _rows(buf, "rotary.buf"), buf.shape[0], o0, h0, d0, float(s0), o1, h1, d1, float(s1),
                                                        rot_dims, layout, _p(freq), float(mag), pos.data_ptr(), _stream()), "hy_rotary")


def polynorm(z: torch.Tensor, coef, eps: float, dtype: torch.dtype) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e per row of the fp32 z, N = unit RMS over the row; coef = (a, b, c, e) -> `dtype`."""
    _dev(z, torch.float32, "polynorm.z")
    T, n = z.shape
    out = torch.empty(T, n, dtype=dtype, device=z.device)
    if T:
        a, b, c, e = [float(v) for v in coef]
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_polynorm(z.data_ptr(), _rows(z, "polynorm.z"), T, n, a, b, c, e, float(eps), out.data_ptr(), n,
                                                          act_code(dtype), _stream()), "hy_polynorm")
    return out


def moe_route(z: torch.Tensor, groups: int, keep: int, top: int, *, sigmoid: bool = False, group_top: int = 1, scale: float = 1.0):
    """Router logits fp32 [T, E] -> (expert ids int32 [T, top], weights fp32 [T, top]): softmax scores (sigmoid: a sigmoid of every logit), only
    experts of the `keep` best of `groups` runs of neighbouring experts (a run scores as its best member, or with group_top = 2 as the sum of its
    two best) are eligible, the `top` best eligible are chosen; their weights are score * scale."""
    _dev(z, torch.float32, "moe_route.z")
    T, E = z.shape
    ids = torch.empty(T, top, dtype=torch.int32, device=z.device)
    wts = torch.empty(T, top, dtype=torch.float32, device=z.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_moe_route_ex(z.data_ptr(), _rows(z, "moe_route.z"), T, E, groups, keep, top, ids.data_ptr(), wts.data_ptr(),
                                                              1 if sigmoid else 0, int(group_top), float(scale), _stream()), "hy_moe_route")
    return ids, wts


def moe_align(ids: torch.Tensor, experts: int):
    """ids int32 [T, top] -> (offs int32 [E + 1], src_row int32 [T * top], place_of int32 [T * top], tiles): the (token, choice) pairs sorted
    by expert; sorted place p belongs to token src_row[p], pair i sits at place_of[i]; tiles = {count, (expert, first row) x count} lists the
    64-row tiles of the sorted rows for dense_grouped."""
    _dev(ids, torch.int32, "moe_align.ids")
    T, top = ids.shape
    offs = torch.empty(experts + 1, dtype=torch.int32, device=ids.device)
    src = torch.empty(T * top, dtype=torch.int32, device=ids.device)
    place = torch.empty(T * top, dtype=torch.int32, device=ids.device)
    tiles = torch.empty(1 + 2 * (T * top // 64 + experts), dtype=torch.int32, device=ids.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_moe_align(ids.data_ptr(), T * top, top, experts, offs.data_ptr(), src.data_ptr(), place.data_ptr(),
                                                           tiles.data_ptr(), _stream()), "hy_moe_align")
    return offs, src, place, tiles


def moe_route_sorted(z: torch.Tensor, experts: int, groups: int, keep: int, top: int, *, sigmoid: bool = False, group_top: int = 1, scale: float = 1.0):
    """moe_route followed by moe_align -> (ids, wts, offs, src_row, place_of, tiles); a few tokens (a decode step) take one launch for both."""
    _dev(z, torch.float32, "moe_route_sorted.z")
    T = z.shape[0]
    if z.shape[1] != experts:
        raise _C.Mi355Error(f"moe_route_sorted: logits {tuple(z.shape)} for {experts} experts")
    if not 0 < T <= 64 or 16 * (experts + groups) * 4 + experts * 8 > 48 * 1024:
        ids, wts = moe_route(z, groups, keep, top, sigmoid=sigmoid, group_top=group_top, scale=scale)
        return (ids, wts) + moe_align(ids, experts)
    dev = z.device
    ids, wts = torch.empty(T, top, dtype=torch.int32, device=dev), torch.empty(T, top, dtype=torch.float32, device=dev)
    offs, src, place = torch.empty(experts + 1, dtype=torch.int32, device=dev), torch.empty(T * top, dtype=torch.int32, device=dev), torch.empty(T * top, dtype=torch.int32, device=dev)
    tiles = torch.empty(1 + 2 * (T * top // 64 + experts), dtype=torch.int32, device=dev)
    _C.check_hybrid(_C.hybrid_lib().mi355_hy_moe_route_align_ex(z.data_ptr(), _rows(z, "moe_route_sorted.z"), T, experts, groups, keep, top, ids.data_ptr(),
                                                                wts.data_ptr(), offs.data_ptr(), src.data_ptr(), place.data_ptr(), tiles.data_ptr(),
                                                                1 if sigmoid else 0, int(group_top), float(scale), _stream()), "hy_moe_route_align")
    return ids, wts, offs, src, place, tiles


def moe_combine(y, place_of: Optional[torch.Tensor] = None, wts: Optional[torch.Tensor] = None, extra: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = sum_k wts[t, k] * y[place_of[t, k]] (+ extra[t]) -> fp32 [T, W]; y may be a MoeSum holding all four."""
    if isinstance(y, MoeSum):
        y, place_of, wts, extra = y.y, y.place_of, y.wts, y.extra
    _dev(y, torch.float32, "moe_combine.y"); _dev(wts, torch.float32, "moe_combine.wts")
    T, top = wts.shape
    W = y.shape[1]
    if not y.is_contiguous() or y.shape[0] != T * top or (extra is not None and (extra.shape != (T, W) or extra.dtype != torch.float32 or not extra.is_contiguous())):
        raise _C.Mi355Error(f"moe_combine: y {tuple(y.shape)} for {T} tokens x {top}")
    out = torch.empty(T, W, dtype=torch.float32, device=y.device)
    if T:
        _C.check_hybrid(_C.hybrid_lib().mi355_hy_moe_combine(y.data_ptr(), T, W, place_of.data_ptr(), wts.data_ptr(), top, _p(extra), out.data_ptr(), _stream()),
                        "hy_moe_combine")
    return out
