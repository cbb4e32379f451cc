"""The Nepudra member of the hybrid family on the GPU against the plain implementation in nepudra_oracle (float64, CPU): single operations,
every mechanism alone in many shapes, whole prompts against token-by-token decoding, portions, unequal batches, reused pages and slots,
keys far back, at page borders and just inside / just outside the sliding window with weights built so that one key dominates, a token
carried by the delta rule's state, long decoding, graph replay, and greedy generation through the scheduler and the command line."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import nepudra_oracle as O  # noqa: E402
import nepudra_util as U  # noqa: E402

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


def bf16_close(got, ref):
    """Row by row: rounding moves a row's logits by a few per cent of their size.  A few rows may move more where the model itself is
    unstable: a delta-rule head's very first output is sign(k . r) * v / rms(v) after its norm, so rounding a small k . r can turn a head over."""
    d = got.double().cpu() - ref
    rel = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt()
    assert float(rel.median()) < 0.03 and float(rel.quantile(0.9)) < 0.06, f"bf16 step is off by more than rounding: median {float(rel.median())}"


def whole(eng, t, sid="s"):
    out = eng.run_step([(sid, t, range(len(t)))])
    eng.release(sid)
    return out


FULL = [U.delta_layer(mlp=None), U.capped_layer(mlp=U.dense()), U.capped_layer(kv_from=1, mlp=U.dense(ff=40)),
        U.window_layer(scaling=U.YARN, rot_dims=8, mlp=U.dense()), U.delta_layer(heads=3, dim=24, mlp=U.dense(ff=72)), U.window_layer(window=70, mlp=None)]


# ------------------------------------------------------------------------------------------------ single operations
def test_embedding_with_hashed_bigram_rows():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(1)
    for W, buckets, mp, mc in ((8, 5, 3, 2), (50, 97, 1, 1), (64, 1, 7, 11), (33, 1000, 2 ** 33 + 9, 2 ** 31 - 1)):      # also products beyond 32 bits
        vocab = 300
        table, bg = torch.randn(vocab, W, generator=g), torch.randn(buckets + 1, W, generator=g)
        ids = torch.randint(0, vocab, (40,), generator=g).to(torch.int32)
        prev = torch.randint(0, vocab, (40,), generator=g).to(torch.int32)
        prev[[0, 17, 39]] = -1
        rows = [buckets if p < 0 else (int(p) * mp + int(t) * mc) % buckets for p, t in zip(prev.tolist(), ids.tolist())]
        ref = table.double()[ids.long()] + bg.double()[rows]
        for dt, tol in ((torch.float32, 1e-6), (torch.bfloat16, 0.0)):
            tb, bb = table.to(dt).to(DEV), bg.to(dt).to(DEV)
            want = ref if dt == torch.float32 else tb.double().cpu()[ids.long()] + bb.double().cpu()[rows]
            copy = torch.zeros(40, W, device=DEV)
            out = hops.embed(ids.to(DEV), tb, prev=prev.to(DEV), bigram=bb, mul_prev=mp, mul_cur=mc, copy=copy)
            close(out, want, max(tol, 1e-6))
            assert torch.equal(out, copy)
        close(hops.embed(ids.to(DEV), table.to(DEV)), table.double()[ids.long()], 0.0)


def test_depth_average_joins_residual_update_and_norm():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(2)
    for W in (8, 50, 64, 1000):
        for n in (1, 2, 5):
            T = 7
            stack = torch.randn(n + 1, T, W, generator=g)
            x, a = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g)
            coef = torch.randn(n + 1, generator=g)
            w1 = torch.full((W,), 1.25)
            xn = x.double() + a.double()
            mixed = sum(coef[j].double() * stack[j].double() for j in range(n)) + coef[n].double() * xn
            sd, xd = stack.to(DEV), x.to(DEV)
            h = hops.depth_mix_norm(xd, a.to(DEV), sd, n, coef.to(DEV), w1.to(DEV), 1e-6)
            close(sd[n], xn, 1e-6)
            close(xd, mixed, 1e-5)
            close(h, O.rms_unit(mixed, 1e-6) * 1.25, 1e-4)
            sd, xd = stack.to(DEV), x.to(DEV)                       # only some rows, nothing written back; and without a branch
            rows = torch.tensor([6, 2], dtype=torch.int32, device=DEV)
            h = hops.depth_mix_norm(xd, a.to(DEV), sd, n, coef.to(DEV), w1.to(DEV), 1e-6, rows=rows)
            close(h, (O.rms_unit(mixed, 1e-6) * 1.25)[[6, 2]], 1e-4)
            close(xd, x.double(), 0.0)
            close(sd[n], stack[n].double(), 0.0)
            hops.depth_mix_norm(xd, None, sd, n, coef.to(DEV), None, 1e-6)
            close(sd[n], x.double(), 0.0)


@pytest.mark.parametrize("H,dim,vdim", [(2, 16, 16), (1, 8, 8), (3, 20, 20), (2, 64, 64), (2, 96, 40), (1, 130, 72), (1, 256, 16), (2, 12, 100)])
def test_delta_rule_scan_states_and_outputs(H, dim, vdim):
    """The recurrence alone: three sequences of unequal length in one launch, continued from states left by an earlier launch, against the
    update written out with outer products."""
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(dim)
    lens = [37, 1, 18]
    T, hd, hv = sum(lens), H * dim, H * vdim
    proj = torch.randn(T, 3 * hd + hv + 5, generator=g)
    ro, ko, ao, vo = 0, hd, 2 * hd, 3 * hd + 3
    z = torch.randn(T, hd, generator=g) * 2
    mult, ueps = math.exp(-0.5), 1e-6
    state = torch.zeros(5, H, dim, vdim)
    slots = [3, 0, 4]

    def ref(rows, S):
        out = torch.zeros(len(rows), H, vdim, dtype=torch.float64)
        for n, t in enumerate(rows):
            p, zz = proj[t].double(), z[t].double()
            for j in range(H):
                r, k, a = (p[o + j * dim:o + (j + 1) * dim] for o in (ro, ko, ao))
                v = p[vo + j * vdim:vo + (j + 1) * vdim]
                w = torch.exp(-mult * torch.sigmoid(zz[j * dim:(j + 1) * dim]))
                u = k / torch.sqrt((k * k).sum() + ueps)
                old = S[j]
                S[j] = w[:, None] * old - torch.outer(torch.sigmoid(a) * u, u @ old) + torch.outer(k, v)
                out[n, j] = S[j].T @ r
        return out.reshape(len(rows), hv)

    sd = state.to(DEV)
    starts = [0, lens[0], lens[0] + lens[1], T]
    S = [torch.zeros(H, dim, vdim, dtype=torch.float64) for _ in lens]
    cut = [20, 1, 5]                                                 # first launch: the first `cut` tokens of every sequence; second: the rest
    for part in (0, 1):
        rows = [list(range(starts[i] + (0 if part == 0 else cut[i]), starts[i] + (cut[i] if part == 0 else lens[i]))) for i in range(3)]
        keep = [i for i in range(3) if rows[i]]
        flat = [t for i in keep for t in rows[i]]
        rs = [0]
        for i in keep:
            rs.append(rs[-1] + len(rows[i]))
        out = hops.delta_scan(proj[flat].to(DEV), ro, ko, vo, ao, z[flat].to(DEV), mult, ueps, H, dim, vdim,
                              torch.tensor(rs, dtype=torch.int32, device=DEV), torch.tensor([slots[i] for i in keep], dtype=torch.int32, device=DEV),
                              torch.tensor([0 if part == 0 else cut[i] for i in keep], dtype=torch.int32, device=DEV), sd)
        want = torch.cat([ref(rows[i], S[i]) for i in keep])
        close(out, want, 2e-4)
    for i in range(3):
        close(sd[slots[i]], S[i], 2e-4)
    assert float(sd[1].abs().max()) == 0.0 and float(sd[2].abs().max()) == 0.0


def test_head_norm_with_a_weight_per_head_and_a_sigmoid_gate():
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(3)
    for H, vd in ((3, 20), (1, 64), (4, 100)):
        o = torch.randn(9, H * vd, generator=g)
        w = 1.0 + 0.3 * torch.randn(H * vd, generator=g)
        gate = torch.randn(9, H * vd + 6, generator=g)
        ref = O.rms_unit(o.double().view(9, H, vd), 1e-5).reshape(9, H * vd) * w.double() * torch.sigmoid(gate[:, 4:4 + H * vd].double())
        close(hops.head_norm(o.to(DEV), H, vd, w.to(DEV), 1e-5, gate.to(DEV), 4, gate_act="sigmoid"), ref, 1e-5)


@pytest.mark.parametrize("window,softcap,gate", [(0, 0.0, False), (40, 0.0, True), (0, 7.0, True), (1, 0.0, False), (64, 3.0, False), (200, 0.0, True)])
def test_matrix_core_attention_against_the_row_kernel_with_window_cap_and_gate(window, softcap, gate):
    """Both attention kernels on identical bf16 pages: ragged tiles of 1-16 rows, scattered pages, two sequences."""
    from rtp_llm_amd import hybrid_ops as hops
    g = torch.Generator().manual_seed(5)
    H, G, dim, vdim, page, pages = 4, 2, 32, 48, 64, 12
    lens, first = [150, 75], [37, 0]                                 # sequence 0 continues at position 37, sequence 1 starts
    kc = torch.randn(pages, G, page, dim, generator=g).bfloat16().to(DEV)
    vc = torch.randn(pages, G, page, vdim, generator=g).bfloat16().to(DEV)
    bt = torch.tensor([[7, 2, 9, 0, 0, 0, 0, 0], [4, 11, 1, 0, 0, 0, 0, 0]], dtype=torch.int32, device=DEV)
    pos, seq, t0, tn = [], [], [], []
    for s_, (n, f) in enumerate(zip(lens, first)):
        base = len(pos)
        pos += list(range(f, n)); seq += [s_] * (n - f)
        for a in range(base, len(pos), 16):
            t0.append(a); tn.append(min(16, len(pos) - a))
    T = len(pos)
    q = torch.randn(T, H * dim + H, generator=g).to(DEV) * 1.5
    I = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    geom = hops.attn_geometry(H, G, dim, vdim, 0, 0, 0, page, 8, pages)
    og = q[:, H * dim:] if gate else None
    a = hops.attn_tiles(q, 0.2, geom, 0, None, None, I(pos), I(seq), bt, I(t0), I(tn), kc, vc, H, vdim, window=window, softcap=softcap, out_gate=og)
    b = hops.attn_rows(q, 0.2, geom, 0, None, None, I(pos), I(seq), bt, kc, vc, H, vdim, window=window, softcap=softcap, out_gate=og)
    assert float((a.float() - b.float()).abs().max()) < 0.03
    # and the row kernel against the definition, from the same pages
    ref = torch.zeros(T, H, vdim, dtype=torch.float64)
    for r in range(T):
        p, s_ = pos[r], seq[r]
        lo = max(0, p - window + 1) if window else 0
        pg = bt[s_].cpu().long()
        for h in range(H):
            kk = torch.stack([kc[pg[j // page], h // (H // G), j % page] for j in range(lo, p + 1)]).double().cpu()
            vv = torch.stack([vc[pg[j // page], h // (H // G), j % page] for j in range(lo, p + 1)]).double().cpu()
            sc = (kk @ q[r, h * dim:(h + 1) * dim].double().cpu()) * 0.2
            if softcap:
                sc = softcap * torch.tanh(sc / softcap)
            o = torch.softmax(sc, 0) @ vv
            ref[r, h] = o * (torch.sigmoid(q[r, H * dim + h].double().cpu()) if gate else 1.0)
    assert float((b.double().cpu() - ref.reshape(T, H * vdim)).abs().max()) < 0.02


# ------------------------------------------------------------------------------------------------ mechanisms alone
ALONE = {
    "delta": U.delta_layer(),
    "delta_one_head_odd_size": U.delta_layer(heads=1, dim=20),
    "delta_head_of_64": U.delta_layer(heads=2, dim=64),
    "delta_head_of_96_with_mlp": U.delta_layer(heads=1, dim=96, mlp=U.dense(ff=100)),
    "delta_head_of_136": U.delta_layer(heads=1, dim=136),
    "capped": U.capped_layer(),
    "capped_one_kv_head_every_position": U.capped_layer(heads=3, kv_heads=1, dim=8, vdim=40, every=1, coef=1.0, softcap=5.0),
    "capped_mha_sizes_not_of_8": U.capped_layer(heads=2, kv_heads=2, dim=20, vdim=12, softcap=100.0, every=1000),
    "capped_matrix_core_sizes": U.capped_layer(heads=4, kv_heads=1, dim=32, vdim=32, mlp=U.dense(ff=40)),
    "capped_wide_heads": U.capped_layer(heads=2, kv_heads=1, dim=160, vdim=136, softcap=2.0),
    "window": U.window_layer(),
    "window_of_one": U.window_layer(window=1),
    "window_wider_than_the_prompt": U.window_layer(window=500, scaling=U.YARN),
    "window_partial_rotary_scaled": U.window_layer(heads=2, kv_heads=1, dim=24, vdim=16, rot_dims=8, scaling=U.YARN, base=300.0, window=17),
    "window_no_rotary_mha": U.window_layer(heads=2, kv_heads=2, dim=12, vdim=20, rot_dims=0, window=33),
    "window_matrix_core_sizes": U.window_layer(heads=4, kv_heads=2, dim=64, vdim=32, rot_dims=32, window=64, mlp=U.dense()),
}


@pytest.mark.parametrize("name", sorted(ALONE))
def test_one_layer_models(name):
    cfg = U.make_config([ALONE[name]], vocab=80, width=48)
    w = U.make_weights(cfg, seed=3, rank=4 if "odd" in name else 8)
    t = toks(70, 80, 4)
    col, ocol = [], []
    ref = U.oracle_logits(cfg, w, t, ocol)
    eng = engine(cfg, w)
    got = eng.run_step([("x", t, range(len(t)))], collect=col)
    close(col[0], ocol[0], 2e-4)
    close(got, ref, 2e-4)
    eng.release("x")
    one = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[:30]])       # and token by token from the first token on
    close(one, ref[:30], 2e-4)


def test_other_widths_and_constants():
    """Widths that are no multiple of four, a bigram table of one bucket, multipliers of one, a vocabulary smaller than the table."""
    for width, buckets, mp, mc in ((50, 1, 1, 1), (36, 300, 1, 1000003), (130, 7, 5, 0)):
        cfg = U.make_config([U.delta_layer(mlp=U.dense(ff=40)), U.window_layer(mlp=None), U.capped_layer(mlp=U.dense(ff=33))], vocab=61, width=width,
                            buckets=buckets, mul_prev=mp, mul_cur=mc, eps=1e-3)
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
            mixer.use_tiles = tiles
        bf16_close(whole(eng, t), ref)


def test_the_bigram_row_and_the_depth_average_matter():
    """The oracle itself: another previous token and other depth weights move the logits, so a lost one would show."""
    cfg = U.make_config(FULL[:3])
    w = U.make_weights(cfg, seed=7)
    t = toks(12, cfg["vocab"], 8)
    ref = U.oracle_logits(cfg, w, t)
    w2 = dict(w); w2["bigram"] = torch.zeros_like(w["bigram"])
    assert float((U.oracle_logits(cfg, w2, t) - ref).abs().max()) > 0.05
    w3 = dict(w); w3["l2.dwa"] = torch.tensor([0.0, 0.0, 0.0, 1.0])
    assert float((U.oracle_logits(cfg, w3, t) - ref).abs().max()) > 0.05


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


# ------------------------------------------------------------------------------------------------ one key that dominates: far back, page borders, window edges
def _beacon_attention(kind, window=40, width=32, vocab=40, heads=2, kv_heads=1, dim=16, vdim=16):
    """One attention layer in which the key of token 1 (the beacon) and the query of token 2 (the asker) meet in one un-rotated channel that
    every other token leaves empty, so that the asker scores the beacon far above all other keys; the beacon's value is far from the
    others'.  Whether the asker sees the beacon moves its logits by a lot."""
    c = dim - 1                                          # the channel: beyond the rotary span
    if kind == "window":
        L = U.window_layer(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot_dims=8, window=window, scale=1.0)
    else:
        L = U.capped_layer(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=1.0, softcap=30.0, coef=0.1, every=16)
    cfg = U.make_config([L], vocab=vocab, width=width)
    w = U.make_weights(cfg, seed=17)
    for n in ("q", "k"):
        w[f"l0.mix.{n}"] *= 0.05
        w[f"l0.mix.{n}.b"].zero_()
    w["l0.norm1"].fill_(1.0)
    w["l0.mix.g"].zero_()                                # every head's gate one half
    w["bigram"].zero_()                                  # a neighbour's identity reaches a token through attention only
    e = torch.randn(vocab, width, generator=torch.Generator().manual_seed(18)) * 0.05
    e[:, :2] = 0.0                                       # only the beacon and the asker live on the first two axes
    e[1], e[2] = 0.0, 0.0
    e[1, 0], e[2, 1] = 1.0, 1.0
    w["embed"] = e
    big = 4.0 if kind == "window" else 15.0 ** 0.5 / width ** 0.5        # normed heads need no size; plain ones give a score of about 15
    for g in range(kv_heads):
        w["l0.mix.k"][g * dim + c] = 0.0
        w["l0.mix.k"][g * dim + c, 0] = big
    for h in range(heads):
        w["l0.mix.q"][h * dim + c] = 0.0
        w["l0.mix.q"][h * dim + c, 1] = big
    w["l0.mix.v"][:, 0] = 3.0
    if kind == "window":
        w["l0.mix.q.norm"].fill_(1.0); w["l0.mix.k.norm"].fill_(1.0)
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


@pytest.mark.parametrize("beacon,asker", [(0, 250), (3, 299), (63, 290), (64, 290), (127, 128), (128, 191), (190, 191), (1, 2)])
def test_dominant_key_far_back_and_at_page_borders(beacon, asker):
    cfg, w = _beacon_attention("capped")
    t = [3 + (i % 30) for i in range(asker + 1)]
    t[beacon], t[asker] = 1, 2
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[beacon] = 5
    assert float((U.oracle_logits(cfg, w, t2)[asker] - ref[asker]).abs().max()) > 0.05, "the beacon must move the asker's logits"
    _ask(cfg, w, t, asker, ref, beacon)


@pytest.mark.parametrize("window,asker", [(40, 100), (40, 39), (40, 40), (64, 127), (64, 128), (65, 200), (16, 70), (1, 9), (97, 230)])
def test_dominant_key_just_inside_and_just_outside_the_window(window, asker):
    """The beacon as the oldest key the asker still sees (distance window - 1), and one further back (not seen any more): the oracle confirms
    that the first moves the asker's logits and the second does not, and the engine matches it in a prompt, decoded, and in portions."""
    cfg, w = _beacon_attention("window", window=window)
    for dist, seen in ((window - 1, True), (window, False)):
        beacon = asker - dist
        if beacon < 0:
            continue
        t = [3 + (i % 30) for i in range(asker + 1)]
        t[beacon], t[asker] = 1, 2
        if beacon == asker:                                        # a window of one: the asker sees only itself
            t[asker] = 2
        ref = U.oracle_logits(cfg, w, t)
        t2 = list(t)
        if beacon != asker:
            t2[beacon] = 5
            moved = float((U.oracle_logits(cfg, w, t2)[asker] - ref[asker]).abs().max())
            assert (moved > 0.05) == seen, f"distance {dist}: the oracle's logits moved by {moved}"
        _ask(cfg, w, t, asker, ref, beacon)


def test_delta_rule_state_carries_a_far_token():
    """A beacon at position 2 writes its value into a key channel that no other token touches; the slow head keeps it for hundreds of tokens
    (decay near one), the fast head forgets it (decay near exp(-exp(-1/2)) a step).  The asker reads that channel."""
    W, d = 32, 16
    cfg = U.make_config([U.delta_layer(heads=2, dim=d)], vocab=40, width=W)
    w = U.make_weights(cfg, seed=19)
    w["l0.norm1"].fill_(1.0)
    w["bigram"].zero_()
    e = torch.randn(40, W, generator=torch.Generator().manual_seed(20)) * 0.05
    e[:, :2] = 0.0
    e[1], e[2] = 0.0, 0.0
    e[1, 0], e[2, 1] = 1.0, 1.0
    w["embed"] = e
    for hh in range(2):
        c = hh * d + d - 1
        w["l0.mix.k"][c] = 0.0
        w["l0.mix.r"][c] = 0.0
        w["l0.mix.k"][c, 0] = 2.0
        w["l0.mix.r"][c, 1] = 2.0
        w["l0.mix.w2"][c] = 0.0
        w["l0.mix.w0"][c] = -14.0 if hh == 0 else 14.0
    w = {k: v.bfloat16().float() for k, v in w.items()}
    t = [3 + (i % 30) for i in range(400)]
    t[2], t[399] = 1, 2
    ref = U.oracle_logits(cfg, w, t)
    t2 = list(t); t2[2] = 7
    assert float((U.oracle_logits(cfg, w, t2)[-1] - ref[-1]).abs().max()) > 0.05
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
    cfg = U.make_config([U.window_layer(scaling=U.YARN, window=50, mlp=U.dense()), U.delta_layer(mlp=U.dense()), U.capped_layer(heads=2, mlp=None),
                         U.capped_layer(heads=2, kv_from=2, mlp=U.dense())])
    w = U.make_weights(cfg, seed=23)
    t = toks(330, cfg["vocab"], 24)
    ref = U.oracle_logits(cfg, w, t)
    eng = engine(cfg, w)
    eng.run_step([("d", t[:10], [])])
    out = torch.cat([eng.run_step([("d", [tk], [0])]) for tk in t[10:]])
    close(out, ref[10:], 5e-4)


def test_contexts_beyond_a_thousand_tokens_split_decode_rows():
    """Past 1024 cached tokens a decode row's keys are dealt over several blocks and merged by a second launch: cap, window start and head gate
    must survive that path (causal layer, and a window wide enough to be split as well)."""
    cfg = U.make_config([U.capped_layer(heads=2, kv_heads=1, softcap=6.0), U.window_layer(heads=2, kv_heads=1, window=1100, scaling=U.YARN)], vocab=50, width=32)
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
    cfg = U.make_config([U.delta_layer(mlp=U.dense()), U.capped_layer(mlp=U.dense()), U.window_layer(mlp=None)], vocab=64, width=48)
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
    cfg = U.make_config([U.delta_layer(mlp=None), U.capped_layer(mlp=U.dense()), U.capped_layer(kv_from=1, mlp=None), U.window_layer(mlp=U.dense())], vocab=64, width=48)
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
    """Decode steps through the captured graph with eager prompt portions and eager decode steps between the replays; the previous token of
    every sequence travels with the step's index arrays."""
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
