"""The Nudorax member of the hybrid family on the GPU against the plain implementation in nudorax_oracle (float64, CPU): single operations,
every mechanism alone in many shapes, whole prompts against token-by-token decoding, portions down to two tokens, unequal batches, reused
pages and slots, a key just inside / just outside the sliding window and at page borders with weights built so that it dominates, a sink
that takes most of the weight, a token carried for hundreds of steps by the slow head of the lightning state, long decoding, graph replay,
and greedy generation through the scheduler and the command line."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import nudorax_oracle as O  # noqa: E402
import nudorax_util as U  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def engine(cfg, w, dtype=torch.float32, max_tokens=1024, max_seqs=4, **kw):
    from rtp_llm_amd.hybrid import HybridConfig, HybridModel
    from rtp_llm_amd.scheduler import ServingEngine
    return ServingEngine(HybridModel(HybridConfig.from_json(cfg), w, dtype, DEV), max_tokens=max_tokens, max_seqs=max_seqs, **kw)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def close(got, ref, tol):
    err = float((got.double().cpu() - ref).abs().max())
    assert err <= tol, f"max |error| {err} > {tol}"


def bf16_close(got, ref, median=0.03, tail=0.06):
    """Row by row: rounding to 16 bits moves a row's logits by a few per cent of their size."""
    d = got.double().cpu() - ref
    rel = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt()
    assert float(rel.median()) < median and float(rel.quantile(0.9)) < tail, f"bf16 step is off by more than rounding: median {float(rel.median())}, 90% {float(rel.quantile(0.9))}"


def whole(eng, t, sid="s"):
    out = eng.run_step([(sid, t, range(len(t)))])
    eng.release(sid)
    return out


FULL = [U.layer(mlp=U.moe()),
        U.layer(U.window_side(heads=2, kv_heads=1, dim=32, vdim=16, rot_dims=16, window=70, scaling=U.SCALING), U.lightning_side(heads=3, dim=8, vdim=40), mlp=None),
        U.layer(U.window_side(heads=3, kv_heads=3, dim=12, vdim=20, window=9), U.lightning_side(heads=1, dim=24, vdim=8, decay=[0.97]),
                left_scale=0.5, right_scale=1.5, mlp=U.moe(experts=4, top=1, count=1, keep=1, ff=32, shared_ff=0)),
        U.layer(mlp=U.moe(experts=8, top=3, count=4, keep=4, ff=33, limit=0.4, shared_ff=50, shared_limit=0.7))]


# ------------------------------------------------------------------------------------------------ single operations
def test_scaled_embedding_rows():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(1)
    for W in (8, 50, 257):
        table = torch.randn(120, W, generator=g)
        ids = torch.randint(0, 120, (33,), generator=g).to(torch.int32)
        for dt in (torch.float32, torch.bfloat16):
            tb = table.to(dt).to(DEV)
            x, h = hops.embed_scaled(ids.to(DEV), tb, 7.5, rounded=True)
            want = tb.double().cpu()[ids.long()] * 7.5
            close(x, want, 1e-6)
            assert h.dtype == dt and torch.equal(h, x.to(dt))
            assert hops.embed_scaled(ids.to(DEV), tb, 1.0)[1] is None


@pytest.mark.parametrize("center", [True, False])
def test_norm_of_a_branch_joins_the_stream(center):
    """x <- x + N(ca a + cb b + mixture sum + sigmoid(gate) shared) * w for the layer norm and the RMS norm, every term alone and together."""
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(2)
    norm = (lambda y, w: O.layer_norm(y, w, 1e-5)) if center else (lambda y, w: O.rms_norm(y, w, 1e-5))
    for W in (8, 50, 64, 1000):
        T, top = 7, 3
        x, a, b, sh = (torch.randn(T, W, generator=g) for _ in range(4))
        a = a + 3.0                                                   # a mean far from zero: the two norms differ by a lot
        w = 1.0 + 0.3 * torch.randn(W, generator=g)
        y = torch.randn(T * top, W, generator=g)
        place = torch.randperm(T * top, generator=g).to(torch.int32).reshape(T, top)
        wts = torch.rand(T, top, generator=g)
        gate = torch.randn(T, 5, generator=g)                         # the gate is column 2 of a wider buffer
        mix = (wts.double()[:, :, None] * y.double()[place.long()]).sum(1)
        d = lambda t: t.to(DEV)
        for dt in (torch.float32, torch.bfloat16):
            wd = w.to(dt).to(DEV)
            wr = wd.double().cpu()
            cases = {
                "a": (dict(a=d(a), ca=1.0), a.double()),
                "a and b": (dict(a=d(a), ca=1.3, b=d(b), cb=-0.7), 1.3 * a.double() - 0.7 * b.double()),
                "mixture": (dict(moe=hops.MoeSum(d(y), d(place), d(wts))), mix),
                "mixture and shared": (dict(moe=hops.MoeSum(d(y), d(place), d(wts), d(sh))), mix + sh.double()),
                "mixture and gated shared": (dict(moe=hops.MoeSum(d(y), d(place), d(wts), d(sh), d(gate)[:, 2])), mix + torch.sigmoid(gate[:, 2:3].double()) * sh.double()),
            }
            for name, (kw, branch) in cases.items():
                xd = d(x)
                h = hops.branch_norm(xd, wd, 1e-5, center=center, rounded=True, **kw)
                want = x.double() + norm(branch, wr)
                close(xd, want, 2e-5)
                assert h.dtype == dt and torch.equal(h, xd.to(dt)), name
                assert hops.branch_norm(d(x), wd, 1e-5, center=center, **kw) is None
            rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
            xd = d(x)
            hn = hops.norm_rows(xd, rows, wd, 1e-5, center=center)
            close(hn, norm(x.double(), wr)[[5, 0, 5]], 2e-5 if dt == torch.float32 else 0.03)
            assert torch.equal(xd.cpu(), x)


def test_clamped_gated_activation_in_the_linears():
    """Dense, skinny, row and grouped kernels with the clamped form, inputs large enough that all three clamps bite."""
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(3)
    K, ff, lim = 48, 64, 0.8
    gate, up, down = torch.randn(ff, K, generator=g) * 0.4, torch.randn(ff, K, generator=g) * 0.4, torch.randn(K, ff, generator=g) * 0.1
    for M in (1, 5, 16, 70):
        x = torch.randn(M, K, generator=g)
        gg, uu = x.double() @ gate.double().T, x.double() @ up.double().T
        assert float(gg.max()) > lim and float(uu.max()) > lim and float(uu.min()) < -lim
        ref_mid = torch.clamp(gg, max=lim) * torch.sigmoid(1.702 * torch.clamp(gg, max=lim)) * (torch.clamp(uu, -lim, lim) + 1.0)
        close(ref_mid @ down.double().T, O.expert(x.double(), gate.double(), up.double(), down.double(), lim), 1e-12)
        wgu = hops.group_gate_up(gate.to(DEV), up.to(DEV))
        close(hops.dense_linear(x.to(DEV), wgu, gated=True, act=hops.ACT_SWIGLU_CLAMP, act_param=lim), ref_mid, 1e-5)
        got = hops.dense_linear(x.bfloat16().to(DEV), wgu.bfloat16(), gated=True, act=hops.ACT_SWIGLU_CLAMP, act_param=lim)
        assert float((got.double().cpu() - ref_mid).abs().max()) < 0.06
        # grouped: three experts, the rows dealt over them
        w3 = torch.stack([wgu, wgu * 0.5, -wgu])
        ids = (torch.arange(M) % 3).to(torch.int32).reshape(M, 1).to(DEV)
        offs, src, place, tiles = hops.moe_align(ids, 3)
        out = hops.dense_grouped(x.to(DEV), w3, offs=offs, gather=src, tiles=tiles, rows=M, gated=True, act=hops.ACT_SWIGLU_CLAMP, act_param=lim)
        for r in range(M):
            e = r % 3
            f = (1.0, 0.5, -1.0)[e]
            want = O.expert(x[r:r + 1].double(), f * gate.double(), f * up.double(), torch.eye(ff, dtype=torch.float64), lim)
            close(out[place[r].long()].reshape(1, -1), want, 1e-5)
    with pytest.raises(Exception):
        hops.dense_linear(x.to(DEV), wgu, gated=True, act=hops.ACT_SWIGLU_CLAMP, act_param=0.0)       # the limit is part of the activation


@pytest.mark.parametrize("E,count,keep,top", [(10, 5, 3, 4), (8, 4, 2, 2), (6, 3, 1, 2), (12, 3, 2, 5), (4, 1, 1, 1), (16, 16, 5, 3), (9, 3, 3, 9), (130, 10, 4, 7)])
def test_sigmoid_router_with_groups_ranked_by_their_two_best(E, count, keep, top):
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(E * 100 + top)
    router = {"experts": E, "top": top, "scale": 2.5, "groups": {"count": count, "keep": keep}}
    differs = 0
    for T in (5, 100):
        z = torch.randn(T, E + 3, generator=g) * 1.5
        zl = z[:, 1:1 + E]                                           # the logits are columns of a wider buffer
        ids, wts, offs, src, place, tiles = hops.moe_route_sorted(z.to(DEV)[:, 1:1 + E], E, count, keep, top, sigmoid=True, group_top=2, scale=2.5)
        per = E // count
        for t in range(T):
            want_ids, want_w = O.route(zl[t].double(), router)
            assert ids[t].tolist() == want_ids, f"token {t}"
            close(wts[t], torch.tensor(want_w, dtype=torch.float64), 1e-6)
            s = torch.sigmoid(zl[t].double()).view(count, per)
            by_max = sorted(range(count), key=lambda q: (-float(s[q].max()), q))[:keep]
            by_two = sorted(range(count), key=lambda q: (-float(s[q].sort(descending=True).values[:2].sum()), q))[:keep]
            differs += sorted(by_max) != sorted(by_two)
        n = T * top
        assert int(offs[-1]) == n and sorted(src.tolist()) == sorted([t for t in range(T) for _ in range(top)])
        assert all(int(offs[e]) <= int(place.reshape(-1)[i]) < int(offs[e + 1]) for i, e in enumerate(ids.reshape(-1).tolist()))
    if per >= 2 and 1 < count and keep < count:
        assert differs > 0, "no token tells a ranking by two best from a ranking by the best"


def test_sigmoid_router_ranks_by_logit_where_the_sigmoid_rounds_to_one():
    """Logits beyond 17 all have an fp32 sigmoid of exactly one; the order of the logits still decides (one group, so no group sums tie)."""
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(77)
    z = torch.randn(40, 12, generator=g) * 3 + 30.0
    assert float(torch.sigmoid(z).min()) == 1.0
    ids, wts = hops.moe_route(z.to(DEV), 1, 1, 5, sigmoid=True, group_top=2, scale=2.0)
    assert ids.cpu().tolist() == z.topk(5, dim=1).indices.tolist()
    assert float((wts - 2.0).abs().max()) == 0.0


@pytest.mark.parametrize("H,G,dim", [(4, 1, 16), (3, 3, 20), (2, 1, 64), (5, 5, 8), (8, 2, 128)])
def test_query_and_key_norm_over_all_heads_at_once(H, G, dim):
    """attn_prep with the norm over the whole projection: the queries come back normed and turned, the keys land in their pages."""
    from rtp_llm_amd import hybrid_ops as hops
    from rtp_llm_amd.mixers import RotarySpec, WavelengthScaling, rotary_table
    g = torch.Generator().manual_seed(dim)
    vdim, page, T = 8, 64, 70
    rot = {"dims": dim // 2, "base": 500.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 48}}
    freq, mag = rotary_table(RotarySpec(dim // 2, 500.0, "halves", WavelengthScaling(4.0, 48.0, 1.0, 3.0)), DEV)
    steps = O.rotary_steps(rot)
    close(freq, torch.tensor(steps, dtype=torch.float64), 1e-7)
    assert mag == 1.0
    qkv = torch.randn(T, (H + G) * dim + G * vdim + 4, generator=g)
    qw, kw = 1.0 + 0.3 * torch.randn(H * dim, generator=g), 1.0 + 0.3 * torch.randn(G * dim, generator=g)
    pos = torch.arange(100, 100 + T)
    geom = hops.attn_geometry(H, G, dim, vdim, dim // 2, 1, 0, page, 4, 4)
    kc, vc = torch.zeros(4, G, page, dim, device=DEV), torch.zeros(4, G, page, vdim, device=DEV)
    bt = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32, device=DEV)
    qd = qkv.to(DEV)
    hops.attn_prep(qd, H * dim, (H + G) * dim, geom, freq, None, False, 1e-5, pos.to(torch.int32).to(DEV), torch.zeros(T, dtype=torch.int32, device=DEV), bt,
                   kc, vc, q_norm=qw.to(DEV), k_norm=kw.to(DEV), norm_whole=True)
    q = O.rms_norm(qkv[:, :H * dim].double(), qw.double(), 1e-5).view(T, H, dim)
    k = O.rms_norm(qkv[:, H * dim:(H + G) * dim].double(), kw.double(), 1e-5).view(T, G, dim)
    pages = bt[0].tolist()
    for t in range(T):
        p = int(pos[t])
        for h in range(H):
            close(qd[t, h * dim:(h + 1) * dim], O.rotate(q[t, h], p, steps), 6e-5)      # angles near 170 rad in fp32
        for j in range(G):
            close(kc[pages[p // page], j, p % page], O.rotate(k[t, j], p, steps), 6e-5)
            close(vc[pages[p // page], j, p % page], qkv[t, (H + G) * dim + j * vdim:(H + G) * dim + (j + 1) * vdim].double(), 1e-6)


@pytest.mark.parametrize("H,dim,vdim", [(2, 16, 24), (1, 8, 8), (3, 20, 12), (2, 64, 64), (1, 130, 72), (2, 96, 100)])
def test_lightning_scan_states_and_outputs(H, dim, vdim):
    """The recurrence alone: three sequences of unequal length in one launch, continued from the states an earlier launch left."""
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(dim + vdim)
    lens, slots, cut = [37, 1, 18], [3, 0, 4], [20, 1, 5]
    T, hd, hv = sum(lens), H * dim, H * vdim
    proj = torch.randn(T, 2 * hd + hv + 7, generator=g)
    qo, ko, vo = 3, 3 + hd, 5 + 2 * hd
    decay = torch.tensor([0.998, 0.6, 0.9][:H])
    sd = torch.zeros(5, H, dim, vdim, device=DEV)
    S = [torch.zeros(H, dim, vdim, dtype=torch.float64) for _ in lens]
    starts = [0, lens[0], lens[0] + lens[1], T]

    def ref(rows, St):
        out = torch.zeros(len(rows), H, vdim, dtype=torch.float64)
        for n, t in enumerate(rows):
            p = proj[t].double()
            for j in range(H):
                q, k = (O.silu(p[o + j * dim:o + (j + 1) * dim]) for o in (qo, ko))
                v = O.silu(p[vo + j * vdim:vo + (j + 1) * vdim])
                St[j] = float(decay[j]) * St[j] + torch.outer(k, v)
                out[n, j] = St[j].T @ q
        return out.reshape(len(rows), hv)

    for part in (0, 1):
        rows = [list(range(starts[i] + (0 if part == 0 else cut[i]), starts[i] + (cut[i] if part == 0 else lens[i]))) for i in range(3)]
        keep = [i for i in range(3) if rows[i]]
        flat = [t for i in keep for t in rows[i]]
        rs = [0]
        for i in keep:
            rs.append(rs[-1] + len(rows[i]))
        I = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        out = hops.scan(hops.SCAN_FIXED_SILU, proj[flat].to(DEV), qo, ko, vo, None, decay.to(DEV), None, 1.0, 1.0, H, dim, vdim, I(rs),
                        I([slots[i] for i in keep]), I([0 if part == 0 else cut[i] for i in keep]), sd, torch.float32)
        close(out, torch.cat([ref(rows[i], S[i]) for i in keep]), 2e-4)
    for i in range(3):
        close(sd[slots[i]], S[i], 2e-4)
    assert float(sd[1].abs().max()) == 0.0 and float(sd[2].abs().max()) == 0.0


@pytest.mark.parametrize("mode_silu,H,dim,vdim,chunk", [(True, 2, 16, 24, 64), (False, 1, 64, 64, 64), (True, 3, 20, 12, 128), (True, 2, 136, 72, 64), (False, 2, 8, 100, 64)])
def test_chunked_form_of_the_fixed_decay_scan(mode_silu, H, dim, vdim, chunk):
    """Long prompt portions walk their chunks side by side: against the token-by-token walk of the same kernel and against the definition, with
    sequences that start fresh or continue a state, lengths on both sides of chunk borders, single rows between long ones, decays of 0 and 1."""
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(dim * 7 + vdim)
    lens, slots, first = [200, 1, 64, 65, 330, 2, 127], [6, 0, 3, 1, 5, 2, 4], [0, 9, 0, 40, 7, 0, 1]
    T, hd, hv = sum(lens), H * dim, H * vdim
    proj = torch.randn(T, 2 * hd + hv + 4, generator=g) * 0.7
    qo, ko, vo = 0, hd, 2 * hd + 4
    decay = torch.tensor([0.998, 0.5, 1.0][:H]) if H > 1 else torch.tensor([0.97])
    if not mode_silu and H > 1:
        decay[1] = 0.0
    start = torch.randn(7, H, dim, vdim, generator=g)
    act = O.silu if mode_silu else (lambda t: t)
    rs = [0]
    for n in lens:
        rs.append(rs[-1] + n)
    want, S_end = torch.zeros(T, hv, dtype=torch.float64), {}
    for i, n in enumerate(lens):
        S = [torch.zeros(dim, vdim, dtype=torch.float64) if first[i] == 0 else start[slots[i], j].double() for j in range(H)]
        for t in range(rs[i], rs[i + 1]):
            p = proj[t].double()
            for j in range(H):
                q, k = act(p[qo + j * dim:qo + (j + 1) * dim]), act(p[ko + j * dim:ko + (j + 1) * dim])
                v = act(p[vo + j * vdim:vo + (j + 1) * vdim])
                S[j] = float(decay[j]) * S[j] + torch.outer(k, v)
                want[t, j * vdim:(j + 1) * vdim] = S[j].T @ q
        S_end[i] = torch.stack(S)
    I = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    mode = hops.SCAN_FIXED_SILU if mode_silu else hops.SCAN_FIXED
    old = hops.SCAN_CHUNK
    hops.SCAN_CHUNK = chunk
    try:
        for chunked in (True, False):
            sd = start.clone().to(DEV)
            plans = {}
            out = hops.scan(mode, proj.to(DEV), qo, ko, vo, None, decay.to(DEV), None, 1.0, 1.0, H, dim, vdim, I(rs), I(slots), I(first), sd, torch.float32,
                            plans=plans, chunked=chunked)
            assert (len(plans) == 1) == chunked
            scale = float(want.abs().max())
            close(out, want, 2e-5 * scale)
            for i in range(len(lens)):
                close(sd[slots[i]], S_end[i], 2e-5 * float(S_end[i].abs().max()) + 1e-6)
    finally:
        hops.SCAN_CHUNK = old


# ------------------------------------------------------------------------------------------------ mechanisms alone
ALONE = {
    "plain": U.layer(),
    "with_experts": U.layer(mlp=U.moe()),
    "one_kv_head_odd_sizes": U.layer(U.window_side(heads=3, kv_heads=1, dim=20, vdim=12, rot_dims=10, window=17), U.lightning_side(heads=1, dim=20, vdim=12)),
    "mha_no_rotary": U.layer(U.window_side(heads=2, kv_heads=2, dim=12, vdim=20, rot_dims=0, window=33), U.lightning_side(heads=2, dim=8, vdim=8)),
    "window_of_one": U.layer(U.window_side(window=1)),
    "window_wider_than_the_prompt": U.layer(U.window_side(window=500, scaling=U.SCALING)),
    "no_window_scaled_partial_rotary": U.layer(U.window_side(heads=2, kv_heads=1, dim=24, vdim=16, rot_dims=8, scaling=U.SCALING, base=300.0, window=0)),
    "matrix_core_sizes": U.layer(U.window_side(heads=4, kv_heads=2, dim=64, vdim=32, rot_dims=32, window=64), U.lightning_side(heads=2, dim=64, vdim=64), mlp=U.moe()),
    "wide_heads": U.layer(U.window_side(heads=2, kv_heads=1, dim=160, vdim=136, window=40), U.lightning_side(heads=1, dim=136, vdim=72)),
    "left_only_weighs": U.layer(left_scale=1.0, right_scale=0.0),
    "right_only_weighs": U.layer(left_scale=0.0, right_scale=1.0),
    "experts_one_group_top_one_no_shared": U.layer(mlp=U.moe(experts=5, top=1, count=1, keep=1, ff=32, shared_ff=0)),
    "experts_every_group_kept": U.layer(mlp=U.moe(experts=8, top=8, count=2, keep=2, ff=17, limit=0.3, shared_ff=64, shared_limit=0.5)),
    "experts_groups_of_one": U.layer(mlp=U.moe(experts=7, top=2, count=7, keep=3, ff=80, scale=1.0)),
}


@pytest.mark.parametrize("name", sorted(ALONE))
def test_one_layer_models(name):
    cfg = U.make_config([ALONE[name]], vocab=80, width=48)
    w = U.make_weights(cfg, seed=3)
    t = toks(70, 80, 4)
    col, ocol = [], []
    ref = U.oracle_logits(cfg, w, t, ocol)
    eng = engine(cfg, w)
    got = eng.run_step([("x", t, range(len(t)))], collect=col)
    close(col[0], ocol[0], 3e-4)
    close(got, ref, 3e-4)
    eng.release("x")
    one = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[:30]])       # and token by token from the first token on
    close(one, ref[:30], 3e-4)


def test_other_widths_and_constants():
    """Widths that are no multiple of four or eight, no cap on the logits, an embedding multiplier of one, another eps."""
    for width, softcap, scale in ((50, 0.0, 1.0), (36, 5.0, 11.0), (130, 30.0, 0.5)):
        cfg = U.make_config([U.layer(mlp=U.moe(ff=40)), U.layer(U.window_side(window=11), mlp=None), U.layer(mlp=U.moe(ff=33, shared_ff=31))], vocab=61, width=width,
                            eps=1e-3, embed_scale=scale, softcap=softcap)
        w = U.make_weights(cfg, seed=width)
        t = toks(40, 61, width)
        ref = U.oracle_logits(cfg, w, t)
        eng = engine(cfg, w)
        close(whole(eng, t), ref, 3e-4)
        eng.run_step([("d", t[:25], [])])
        close(torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[25:]]), ref[25:], 3e-4)


def test_all_mechanisms_together_residual_stream_and_bf16():
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=5)
    t = toks(90, cfg["vocab"], 6)
    ocol = []
    ref = U.oracle_logits(cfg, w, t, ocol)
    col = []
    got = engine(cfg, w).run_step([("x", t, range(len(t)))], collect=col)
    assert len(col) == len(FULL)
    for a, b in zip(col, ocol):
        close(a, b, 3e-4)
    close(got, ref, 3e-4)
    for tiles in (True, False):                                    # prompt attention on the matrix cores and on the row kernel
        eng = engine(cfg, w, torch.bfloat16)
        for _, mixer, *_ in eng.model.layers:
            mixer.left.use_tiles = tiles
        bf16_close(whole(eng, t), ref)


def test_every_constant_of_the_model_matters():
    """The oracle itself: dropping the sink, the embedding multiplier, a side's weight, the router's scale, a limit or the shared expert's gate
    moves the logits, so a part the engine lost would show in the comparisons above."""
    cfg = U.make_config(FULL[:1])
    w = U.make_weights(cfg, seed=7)
    t = toks(30, cfg["vocab"], 8)
    ref = U.oracle_logits(cfg, w, t)
    moved = lambda c, ww: float((U.oracle_logits(c, ww, t) - ref).abs().max())
    w2 = dict(w); w2["l0.mix.left.sink"] = w["l0.mix.left.sink"] - 30.0
    assert moved(cfg, w2) > 0.02
    w2 = dict(w); w2["l0.mlp.shared.sg"] = w["l0.mlp.shared.sg"] * 0.0 + 1.0
    assert moved(cfg, w2) > 0.02
    for path, val in ((("embedding", "scale"), 1.0), (("logit_softcap",), 0.0), (("layers", 0, "mixer", "left_scale"), 0.0), (("layers", 0, "mixer", "right_scale"), 0.0),
                      (("layers", 0, "mlp", "router", "scale"), 1.0), (("layers", 0, "mlp", "expert", "limit"), 100.0), (("layers", 0, "mlp", "shared", "limit"), 100.0),
                      (("layers", 0, "mlp", "router", "groups", "keep"), 3), (("layers", 0, "mixer", "left", "mask", "size"), 5),
                      (("layers", 0, "mixer", "right", "decay"), [0.9, 0.9])):
        c2 = json.loads(json.dumps(cfg))
        node = c2
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = val
        assert moved(c2, w) > 0.02, path


# ------------------------------------------------------------------------------------------------ schedules
def test_prefill_against_token_by_token_and_first_tokens():
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=9)
    t = toks(100, cfg["vocab"], 10)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    close(whole(eng, t), ref, 3e-4)
    one = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t])
    eng.release("d")
    close(one, ref, 3e-4)
    for n in (1, 2, 3):                                            # the shortest sequences
        close(whole(eng, t[:n]), ref[:n], 3e-4)


@pytest.mark.parametrize("sizes", [[2] * 40, [33, 2, 31, 5, 64, 1, 1, 2, 60], [63, 1, 64, 65, 6], [1, 198], [23, 1, 24, 25, 47, 70]])
def test_portions(sizes):
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=11)
    n = sum(sizes)
    t = toks(n, cfg["vocab"], 12)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    at, outs = 0, []
    for s in sizes:
        outs.append(eng.run_step([("p", t[at:at + s], range(s))]))
        at += s
    close(torch.cat(outs), ref, 3e-4)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-4), (torch.bfloat16, None)])
def test_unequal_batches_reused_pages_and_slots(dtype, tol):
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=13)
    lens = {"a": 150, "b": 9, "c": 70, "d": 131, "e": 64, "f": 40}
    seqs = {k: toks(n, cfg["vocab"], 20 + i) for i, (k, n) in enumerate(lens.items())}
    ref = {k: U.oracle_logits(cfg, w, v) for k, v in seqs.items()}
    # pool: 7 pages of 64 and 3 slots -- less than the requests need together, so pages and slots come back and go out again
    eng = engine(cfg, w, dtype, max_tokens=7 * 64, max_seqs=3)
    plan = [
        [("a", 100), ("b", 4)],
        [("a", 1), ("b", 1), ("c", 30)],
        [("b", 4), ("c", 40), ("a", 49)],            # a, b, c complete -> released
        [("d", 2), ("e", 64)],
        [("d", 129), ("f", 3)],                      # d, e complete
        [("f", 1)], [("f", 36)],
    ]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries = [(k, seqs[k][at[k]:at[k] + n], range(n)) for k, n in step]
        out = eng.run_step(entries)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n]); o += n; at[k] += n
            if at[k] == lens[k]:
                eng.release(k)
    assert eng.cache.pages.free == 7 and eng.cache.slots.free == 3
    for k in seqs:
        if tol is not None:
            close(torch.cat(got[k]), ref[k], tol)
        else:
            bf16_close(torch.cat(got[k]), ref[k])
    with pytest.raises(MemoryError):
        eng.run_step([("big", toks(8 * 64, cfg["vocab"], 1), [])])


def test_a_state_slot_that_comes_back_starts_from_zero():
    """One slot, two requests after each other: the second must not see what the first left in the lightning state or in the pages."""
    cfg = U.make_config([U.layer(right=U.lightning_side(decay=[1.0, 0.998]), mlp=U.moe())], vocab=50, width=32)
    w = U.make_weights(cfg, seed=15)
    a, b = toks(70, 50, 16), toks(66, 50, 17)
    eng = engine(cfg, w, max_tokens=128, max_seqs=1)
    close(whole(eng, a, "a"), U.oracle_logits(cfg, w, a), 3e-4)
    eng.run_step([("b", b[:3], [])])
    out = torch.cat([eng.run_step([("b", b[3:40], range(37))])] + [eng.run_step([("b", [tk], [0])]) for tk in b[40:]])
    close(out, U.oracle_logits(cfg, w, b)[3:], 3e-4)


# ------------------------------------------------------------------------------------------------ one key that dominates: page borders, window edges, the sink
def _beacon_model(window=40, width=32, vocab=40, heads=2, kv_heads=1, dim=16, vdim=16, sink=-2.0, right_scale=0.0):
    """One layer whose left side lets the key of token 1 (the beacon) and the query of token 2 (the asker) meet in one un-rotated channel that
    every other token leaves empty: after the norm over the whole projection the asker scores the beacon near sqrt(H dim) sqrt(G dim) * scale
    and every other key near zero, and the beacon's value is far from the others'.  Whether the asker sees the beacon moves its logits."""
    c = dim - 1                                          # the channel: beyond the rotary span
    L = U.layer(U.window_side(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot_dims=8, window=window, scale=0.5), U.lightning_side(heads=2, dim=8, vdim=8),
                left_scale=1.0, right_scale=right_scale)
    cfg = U.make_config([L], vocab=vocab, width=width, embed_scale=4.0)
    w = U.make_weights(cfg, seed=17)
    p = "l0.mix.left."
    for n in ("q", "k"):
        w[p + n] *= 0.05
    w["l0.norm1"].fill_(1.0)
    w[p + "q.norm"].fill_(1.0); w[p + "k.norm"].fill_(1.0)
    w[p + "sink"].fill_(sink)
    e = torch.randn(vocab, width, generator=torch.Generator().manual_seed(18)) * 0.05
    e[:, :2] = 0.0                                       # only the beacon and the asker live on the first two axes
    e[1], e[2] = 0.0, 0.0
    e[1, 0], e[2, 1] = 1.0, 1.0
    w["embed"] = e
    for g in range(kv_heads):
        w[p + "k"][g * dim + c] = 0.0
        w[p + "k"][g * dim + c, 0] = 4.0
    for h in range(heads):
        w[p + "q"][h * dim + c] = 0.0
        w[p + "q"][h * dim + c, 1] = 4.0
    w[p + "v"][:, 0] = 3.0
    return cfg, {k: v.bfloat16().float() for k, v in w.items()}


def _ask(cfg, w, t, asker, ref, beacon):
    for dtype, tol in ((torch.float32, 3e-4), (torch.bfloat16, 0.05 * float(ref[asker].abs().max()) + 0.05)):
        eng = engine(cfg, w, dtype)
        close(eng.run_step([("w", t, [asker])]), ref[asker:asker + 1], tol)              # in a prompt
        eng.release("w")
        eng.run_step([("d", t[:asker], [])])
        close(eng.run_step([("d", [t[asker]], [0])]), ref[asker:asker + 1], tol)         # decoded alone
        eng.release("d")
        cut = max(1, beacon)                                                              # a portion that starts at the beacon
        eng.run_step([("p", t[:cut], [])])
        close(eng.run_step([("p", t[cut:], [asker - cut])]), ref[asker:asker + 1], tol)
        eng.release("p")
        if asker - beacon > 3:                                                            # decoding from just after the beacon to the asker
            eng.run_step([("q", t[:beacon + 2], [])])
            for tk in t[beacon + 2:asker]:
                eng.run_step([("q", [tk], [])])
            close(eng.run_step([("q", [t[asker]], [0])]), ref[asker:asker + 1], tol)


@pytest.mark.parametrize("window,asker", [(40, 100), (40, 39), (40, 40), (64, 127), (64, 128), (65, 200), (16, 70), (1, 9), (97, 230), (130, 320)])
def test_dominant_key_just_inside_and_just_outside_the_window(window, asker):
    """The beacon as the oldest key the asker still sees (distance window - 1), and one further back (not seen any more): the oracle confirms
    that the first moves the asker's logits and the second does not, and the engine matches it in a prompt, decoded, and in portions."""
    cfg, w = _beacon_model(window=window)
    for dist, seen in ((window - 1, True), (window, False)):
        beacon = asker - dist
        if beacon < 0:
            continue
        t = [3 + (i % 30) for i in range(asker + 1)]
        t[beacon], t[asker] = 1, 2
        ref = U.oracle_logits(cfg, w, t)
        if beacon != asker:
            t2 = list(t)
            t2[beacon] = 5
            moved = float((U.oracle_logits(cfg, w, t2)[asker] - ref[asker]).abs().max())
            assert (moved > 0.05) == seen, f"distance {dist}: the oracle's logits moved by {moved}"
        _ask(cfg, w, t, asker, ref, beacon)


@pytest.mark.parametrize("beacon,asker", [(0, 250), (3, 299), (63, 290), (64, 290), (127, 128), (128, 191), (190, 191), (1, 2)])
def test_dominant_key_far_back_and_at_page_borders(beacon, asker):
    """A window wider than the sequence: the beacon at the first positions and on both sides of page borders, hundreds of keys back."""
    cfg, w = _beacon_model(window=1000)
    t = [3 + (i % 30) for i in range(asker + 1)]
    t[beacon], t[asker] = 1, 2
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[beacon] = 5
    assert float((U.oracle_logits(cfg, w, t2)[asker] - ref[asker]).abs().max()) > 0.05, "the beacon must move the asker's logits"
    _ask(cfg, w, t, asker, ref, beacon)


def test_a_sink_that_takes_most_of_the_weight():
    """A sink logit above the beacon's score in one head and far below in the other: the first head's output nearly vanishes.  The sink is
    not scaled by the attention scale and counts once, whatever the number of keys.  (The right side weighs in as well: the layer norm behind
    the mixer would undo a shrinking of the left side alone.)"""
    cfg, w = _beacon_model(window=50, right_scale=0.6)
    t = [3 + (i % 30) for i in range(120)]
    t[100], t[119] = 1, 2
    refs = []
    for sinks in ((14.0, -30.0), (-30.0, -30.0), (9.0, 9.0)):
        w2 = dict(w); w2["l0.mix.left.sink"] = torch.tensor(sinks)
        ref = U.oracle_logits(cfg, w2, t)
        refs.append(ref)
        for dtype, tol in ((torch.float32, 3e-4), (torch.bfloat16, 0.05 * float(ref.abs().max()) + 0.05)):
            eng = engine(cfg, w2, dtype)
            close(eng.run_step([("w", t, [0, 1, 60, 119])]), ref[[0, 1, 60, 119]], tol)
            eng.release("w")
            eng.run_step([("d", t[:119], [])])
            close(eng.run_step([("d", [t[119]], [0])]), ref[119:], tol)
    assert float((refs[0][119] - refs[1][119]).abs().max()) > 0.05 and float((refs[2][119] - refs[1][119]).abs().max()) > 0.05


def test_lightning_state_carries_a_far_token():
    """A beacon at position 2 writes its value into a key channel that no other token touches; the slow head (decay 0.998) keeps it for hundreds
    of tokens, the fast head (decay 0.5) forgets it.  The asker reads that channel; the window of the left side has long passed."""
    W, d = 32, 16
    cfg = U.make_config([U.layer(U.window_side(window=8), U.lightning_side(heads=2, dim=d, vdim=12, decay=[0.998, 0.5]), left_scale=0.3, right_scale=1.0)],
                        vocab=40, width=W, embed_scale=4.0)
    w = U.make_weights(cfg, seed=19)
    e = torch.randn(40, W, generator=torch.Generator().manual_seed(20)) * 0.05
    e[:, :2] = 0.0
    e[1], e[2] = 0.0, 0.0
    e[1, 0], e[2, 1] = 1.0, 1.0
    w["embed"] = e
    p = "l0.mix.right."
    w[p + "k"] *= 0.2; w[p + "q"] *= 0.2
    for hh in range(2):
        c = hh * d + d - 1
        w[p + "k"][c] = 0.0
        w[p + "q"][c] = 0.0
        w[p + "k"][c, 0] = 2.0                            # other tokens leave silu(0) = 0 in this key channel
        w[p + "q"][c, 1] = 2.0
        w[p + "k"][c, 1] = -8.0                           # the asker itself writes (nearly) nothing there
    w = {k: v.bfloat16().float() for k, v in w.items()}
    t = [3 + (i % 30) for i in range(400)]
    t[2], t[399] = 1, 2
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[2] = 7
    assert float((U.oracle_logits(cfg, w, t2)[-1] - ref[-1]).abs().max()) > 0.05
    c2 = json.loads(json.dumps(cfg)); c2["layers"][0]["mixer"]["right"]["decay"] = [0.5, 0.5]
    assert float((U.oracle_logits(c2, w, t2)[-1] - U.oracle_logits(c2, w, t)[-1]).abs().max()) < 1e-6      # only the slow head remembers
    eng = engine(cfg, w)
    close(whole(eng, t)[-1:], ref[-1:], 3e-4)
    eng.run_step([("d", t[:350], [])])
    out = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[350:]])
    close(out, ref[350:], 3e-4)
    eng.release("d")
    eng.run_step([("p", t[:2], [])])                                    # a portion that starts at the beacon, then two-token portions
    eng.run_step([("p", t[2:395], [])])
    out = torch.cat([eng.run_step([("p", t[395:397], [0, 1])]), eng.run_step([("p", t[397:399], [0, 1])]), eng.run_step([("p", t[399:], [0])])])
    close(out, ref[395:], 3e-4)
    bf16_close(whole(engine(cfg, w, torch.bfloat16), t), ref)


def test_long_decoding():
    cfg = U.make_config([U.layer(U.window_side(scaling=U.SCALING, window=50), mlp=U.moe()), U.layer(U.window_side(heads=2, kv_heads=1, window=130), mlp=None),
                         U.layer(right=U.lightning_side(heads=2, decay=[1.0, 0.95]), mlp=U.moe(top=3, keep=3))])
    w = U.make_weights(cfg, seed=23)
    t = toks(330, cfg["vocab"], 24)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    eng.run_step([("d", t[:10], [])])
    out = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[10:]])
    close(out, ref[10:], 5e-4)


def test_contexts_beyond_a_thousand_tokens_split_decode_rows():
    """Past 1024 cached tokens a decode row's keys are dealt over several blocks and merged by a second launch: the learned sink and the
    window's start must survive that path (a window wide enough to be split, and none)."""
    cfg = U.make_config([U.layer(U.window_side(heads=2, kv_heads=1, window=1100, scaling=U.SCALING), U.lightning_side(decay=[0.998, 0.9])),
                         U.layer(U.window_side(heads=2, kv_heads=2, window=0))], vocab=50, width=32)
    w = U.make_weights(cfg, seed=41)
    t = toks(1180, 50, 42)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w, max_tokens=1280)
    close(eng.run_step([("d", t[:1140], [0, 700, 1139])]), ref[[0, 700, 1139]], 5e-4)
    out = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[1140:]])
    close(out, ref[1140:], 5e-4)
    eng = engine(cfg, w, torch.bfloat16, max_tokens=1280)
    eng.run_step([("d", t[:1140], [])])
    bf16_close(torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[1140:]]), ref[1140:])


# ------------------------------------------------------------------------------------------------ generation
def _oracle_greedy(cfg, w, prompt, n):
    seq, margins = list(prompt), []
    for _ in range(n):
        lg = U.oracle_logits(cfg, w, seq)[-1]
        top = lg.topk(2).values
        margins.append(float(top[0] - top[1]))
        seq.append(int(lg.argmax()))
    return seq[len(prompt):], margins


def test_greedy_generation_through_the_scheduler():
    cfg = U.make_config([U.layer(mlp=U.moe()), U.layer(U.window_side(window=20), mlp=None), U.layer(mlp=U.moe(top=1, keep=1))], vocab=64, width=48)
    w = U.make_weights(cfg, seed=29)
    prompts = [toks(n, 64, 30 + n) for n in (5, 40, 1, 70, 18, 33)]            # six requests over three slots: some wait their turn
    eng = engine(cfg, w, max_tokens=5 * 64, max_seqs=3, max_step_tokens=48)     # prompts are cut into portions of the step budget
    outs = eng.generate(prompts, 12)
    assert eng.cache.pages.free == 5 and eng.cache.slots.free == 3 and not eng.running and not eng.waiting
    for p, o in zip(prompts, outs):
        ref, margins = _oracle_greedy(cfg, w, p, 12)
        for i, (a, b) in enumerate(zip(o, ref)):
            if a != b:
                assert margins[i] < 1e-3, f"token {i}: {a} != {b} with a top-2 margin of {margins[i]}"
                break
    eng.use_graphs = True                                                        # decode-only steps as replayed graphs give the same tokens
    assert eng.generate(prompts[:3], 12) == outs[:3]
    sampled = eng.generate(prompts[:2], 6, top_k=5, top_p=0.9, temperature=0.8, seed=3)
    assert sampled == eng.generate(prompts[:2], 6, top_k=5, top_p=0.9, temperature=0.8, seed=3)
    assert all(len(o) == 6 and all(0 <= x < 64 for x in o) for o in sampled)


def test_command_line_generate_and_trace(tmp_path):
    from safetensors.torch import save_file
    cfg = U.make_config([U.layer(mlp=None), U.layer(U.window_side(window=7), mlp=U.moe())], vocab=64, width=48)
    w = U.make_weights(cfg, seed=31)
    d = tmp_path / "model"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = toks(21, 64, 32)
    r = subprocess.run([sys.executable, "-m", "rtp_llm_amd.cli", "generate", "--model", str(d), "--dtype", "float32", "--max-new-tokens", "5",
                        "--prompt-ids", ",".join(map(str, p))], cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    gen = json.loads(r.stdout.strip().splitlines()[-1])["generated"]
    ref, margins = _oracle_greedy(cfg, w, p, 5)
    assert gen == ref or min(margins) < 1e-3
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": p[:9], "want": [8]}, {"id": "b", "tokens": p[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": p[9:], "want": [0, 11]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(d), "--dtype", "float32", "--out", str(out), "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "done 0" in r.stdout and "done 1" in r.stdout, r.stderr[-2000:]
    import numpy as np
    full = U.oracle_logits(cfg, w, p)
    close(torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(1, -1)), full[8:9], 3e-4)
    close(torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(2, -1)), full[[9, 20]], 3e-4)


def test_graph_replayed_decode_steps_match_eager_and_oracle():
    """Decode steps through the captured graph with eager prompt portions and eager decode steps between the replays."""
    cfg = U.make_config(FULL)
    w = U.make_weights(cfg, seed=37)
    seqs = {k: toks(n, cfg["vocab"], 40 + i) for i, (k, n) in enumerate({"a": 90, "b": 61, "c": 75}.items())}
    ref = {k: U.oracle_logits(cfg, w, v) for k, v in seqs.items()}
    eng = engine(cfg, w)
    eng.run_step([("a", seqs["a"][:50], []), ("b", seqs["b"][:30], [])])
    at = {"a": 50, "b": 30, "c": 0}
    for i in range(30):
        eng.use_graphs = i % 3 != 2                                   # every third decode step runs eagerly
        out = eng.run_step([(k, [seqs[k][at[k]]], [0]) for k in ("a", "b")])
        for j, k in enumerate(("a", "b")):
            close(out[j:j + 1], ref[k][at[k]:at[k] + 1], 3e-4)
            at[k] += 1
        if i == 10:                                                   # an eager prefill step between replays
            eng.use_graphs = True
            eng.run_step([("c", seqs["c"][:70], [])]); at["c"] = 70
    eng.use_graphs = True
    out = eng.run_step([(k, [seqs[k][at[k]]], [0]) for k in ("a", "b", "c")])     # another shape: a second graph
    for j, k in enumerate(("a", "b", "c")):
        close(out[j:j + 1], ref[k][at[k]:at[k] + 1], 3e-4)
    assert len(eng._graphs) == 2
