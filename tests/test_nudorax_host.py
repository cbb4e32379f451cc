"""Host-side pieces of the Nudorax member (CPU): configuration reading and its errors, the registry, the scaled rotary steps, and the plain
implementation against closed forms."""
import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import nudorax_oracle as O  # noqa: E402
import nudorax_util as U  # noqa: E402


def test_config_reading():
    from rtp_llm_amd.hybrid import HybridConfig, ParallelSpec
    from rtp_llm_amd.mixers import AttentionSpec, LightningSpec, WavelengthScaling
    cfg = U.make_config([U.layer(U.window_side(heads=6, kv_heads=3, dim=20, vdim=12, rot_dims=10, window=33, scaling=U.SCALING), U.lightning_side(heads=3, dim=8, vdim=40),
                                 left_scale=0.25, right_scale=2.0, mlp=U.moe(experts=12, top=5, count=3, keep=2, ff=72, limit=0.9, scale=3.0, shared_ff=56, shared_limit=1.7)),
                         U.layer(U.window_side(window=0), mlp=None), U.layer(mlp=U.moe(shared_ff=0))], width=80, vocab=77, eps=1e-4, embed_scale=9.0, softcap=12.0)
    c = HybridConfig.from_json(cfg)
    assert c.sequential and c.out_norm and c.norm_kind == "layer" and c.tied_head and c.embed_scale == 9.0 and c.logit_softcap == 12.0 and c.eps == 1e-4
    assert not c.depth_mix and not c.branch_gates and c.bigram is None and c.norm_offset == 0.0
    L0, L1, L2 = c.layers
    assert L0.kind == "parallel" and isinstance(L0.mixer, ParallelSpec) and (L0.mixer.left_scale, L0.mixer.right_scale) == (0.25, 2.0)
    a, b = L0.mixer.left, L0.mixer.right
    assert isinstance(a, AttentionSpec) and (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.chunk) == (6, 3, 20, 12, 33, 0)
    assert a.sink and a.learned_sink and a.qk_norm and a.qk_norm_whole and not a.bias and not a.out_gate and a.softcap == 0.0
    assert a.rot.layout == "halves" and a.rot.dims == 10 and isinstance(a.rot.scaling, WavelengthScaling) and (a.rot.scaling.low, a.rot.scaling.high) == (1.0, 3.0)
    assert isinstance(b, LightningSpec) and (b.heads, b.dim, b.vdim) == (3, 8, 40) and len(b.decay) == 3
    r = L0.router
    assert (r.experts, r.top, r.groups, r.keep, r.score, r.group_top, r.scale) == (12, 5, 3, 2, "sigmoid", 2, 3.0)
    assert (L0.ff, L0.mlp_kind, L0.mlp_act, L0.act_param, L0.shared_ff, L0.shared_act_param, L0.shared_gate) == (72, "experts", "swiglu_clamp", 0.9, 56, 1.7, True)
    assert L1.ff is None and L1.mixer.left.window == 0 and L1.mixer.left.rot.scaling is None
    assert L2.shared_ff is None and not L2.shared_gate
    bad = json.loads(json.dumps(cfg)); bad["layers"][0]["type"] = "conv"
    with pytest.raises(NotImplementedError):
        HybridConfig.from_json(bad)
    bad = json.loads(json.dumps(cfg)); bad["layers"][0]["mlp"]["kind"] = "dense"
    with pytest.raises(NotImplementedError):
        HybridConfig.from_json(bad)
    bad = json.loads(json.dumps(cfg)); bad["layers"][0]["mixer"]["right"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)


def test_registry_names_the_member():
    from rtp_llm_amd import registry
    assert "nudorax" in registry.families()
    assert registry.architecture_of({"architecture": "Nudorax"}) == "Nudorax"


def test_wavelength_scaled_rotary_steps():
    """The package's table against the plain implementation, and the three regimes by hand."""
    from rtp_llm_amd.mixers import RotarySpec, WavelengthScaling, rotary_table
    kinds = set()
    for dims, base, (factor, low, high, orig) in ((64, 5000.0, (6.0, 1.0, 4.0, 512)), (16, 100.0, (2.0, 2.0, 5.0, 64)), (32, 1e6, (32.0, 1.0, 4.0, 8192)), (8, 10.0, (4.0, 1.0, 3.0, 48))):
        rot = {"dims": dims, "base": base, "scaling": {"factor": factor, "low": low, "high": high, "original": orig}}
        want = O.rotary_steps(rot)
        f, mag = rotary_table(RotarySpec(dims, base, "halves", WavelengthScaling(factor, float(orig), low, high)), "cpu")
        assert mag == 1.0 and f.dtype == torch.float32
        assert float((f.double() - torch.tensor(want, dtype=torch.float64)).abs().max() / max(want)) < 1e-7
        for i, got in enumerate(want):
            plain = base ** (-2.0 * i / dims)
            lam = 2 * math.pi / plain
            if lam < orig / high:
                assert got == plain; kinds.add("kept")
            elif lam > orig / low:
                assert abs(got - plain / factor) < 1e-15; kinds.add("slowed")
            else:
                assert plain / factor <= got <= plain; kinds.add("between")
    assert kinds == {"kept", "slowed", "between"}
    plain, _ = rotary_table(RotarySpec(16, 100.0, "halves", None), "cpu")
    assert abs(float(plain[3]) - 100.0 ** (-6.0 / 16)) < 1e-7


def test_plain_implementation_against_closed_forms():
    g = torch.Generator().manual_seed(1)
    y = torch.randn(5, 12, generator=g, dtype=torch.float64) + 2.0
    w = torch.rand(12, generator=g, dtype=torch.float64)
    assert torch.allclose(O.layer_norm(y, w, 1e-5), torch.nn.functional.layer_norm(y, (12,), w, None, 1e-5))
    assert torch.allclose(O.rms_norm(y, w, 0.0).pow(2).div(w * w).mean(-1), torch.ones(5, dtype=torch.float64))
    # rotation: position 0 leaves the vector, a pair turns by position * step, channels beyond the span pass
    v = torch.randn(10, generator=g, dtype=torch.float64)
    assert torch.equal(O.rotate(v, 0, [1.0, 0.5, 0.25]), v)
    r = O.rotate(v, 7, [1.0, 0.5, 0.25])
    assert torch.equal(r[6:], v[6:]) and abs(float(r[1] ** 2 + r[4] ** 2 - v[1] ** 2 - v[4] ** 2)) < 1e-12
    assert abs(float(r[1]) - float(v[1] * math.cos(3.5) - v[4] * math.sin(3.5))) < 1e-12
    # the router: the group of the single best expert loses to a group whose two best sum higher
    z = torch.tensor([4.0, -4.0, 1.5, 1.4, -1.0, 0.1], dtype=torch.float64)
    ids, wts = O.route(z, {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 1}})
    assert ids == [2, 3] and abs(wts[0] - 2.0 / (1 + math.exp(-1.5))) < 1e-12
    ids, _ = O.route(z, {"experts": 6, "top": 2, "scale": 1.0, "groups": {"count": 3, "keep": 2}})
    assert ids == [0, 2]
    ids, _ = O.route(z, {"experts": 6, "top": 3, "scale": 1.0})
    assert ids == [0, 2, 3]
    # the expert: limits on the gate (from above only) and on the up value (both sides)
    one = torch.eye(1, dtype=torch.float64)
    for gate, up, want in ((5.0, 0.0, 2.0 / (1 + math.exp(-3.404))), (-5.0, 9.0, -5.0 / (1 + math.exp(8.51)) * 3.0), (1.0, -9.0, -1.0 / (1 + math.exp(-1.702)))):
        got = O.expert(torch.ones(1, 1, dtype=torch.float64), one * gate, one * up, one, 2.0)
        assert abs(float(got) - want) < 1e-12
    # lightning attention: with decay 1, one head and identity-like projections the state is the running sum of outer products
    W = 4
    wts_ = {"q": torch.eye(W, dtype=torch.float64), "k": torch.eye(W, dtype=torch.float64), "v": torch.eye(W, dtype=torch.float64), "g": torch.zeros(W, W, dtype=torch.float64),
            "norm": torch.ones(W, dtype=torch.float64), "o": torch.eye(W, dtype=torch.float64)}
    x = torch.randn(6, W, generator=g, dtype=torch.float64)
    st = [torch.zeros(W, W, dtype=torch.float64)]
    out = O.lightning(x, {"p." + k: v for k, v in wts_.items()}, "p.", {"heads": 1, "dim": W, "vdim": W, "decay": [1.0]}, 0.0, st)
    s = O.silu(x)
    assert torch.allclose(st[0], s.T @ s)
    o5 = (s[:6].T @ s[:6]).T @ s[5]
    assert torch.allclose(out[5], 0.5 * o5 / torch.sqrt((o5 * o5).mean()))
    # the window and the sink: a window of one and a sink far below leave every token its own value
    cfg = U.make_config([U.layer(U.window_side(heads=2, kv_heads=1, dim=8, vdim=8, window=1))], vocab=20, width=16)
    wd = {k: v.double() for k, v in U.make_weights(cfg, seed=2).items()}
    wd["l0.mix.left.sink"].fill_(-50.0)
    xx = torch.randn(9, 16, generator=g, dtype=torch.float64)
    got = O.window_attention(xx, wd, "l0.mix.left.", cfg["layers"][0]["mixer"]["left"], 1e-5)
    v = (xx @ wd["l0.mix.left.v"].T)
    assert torch.allclose(got, torch.cat([v, v], 1) @ wd["l0.mix.left.o"].T)
    wd["l0.mix.left.sink"].fill_(50.0)                                   # and a sink far above leaves nothing
    assert float(O.window_attention(xx, wd, "l0.mix.left.", cfg["layers"][0]["mixer"]["left"], 1e-5).abs().max()) < 1e-12


def test_cache_layout_of_a_layer_with_pages_and_a_state():
    """A parallel mixer holds pages for its attention side and a state slot for its recurrent side (built on the CPU: no kernel runs)."""
    from rtp_llm_amd.hybrid import HybridConfig, HybridModel
    cfg = U.make_config([U.layer(U.window_side(heads=4, kv_heads=2, dim=16, vdim=24), U.lightning_side(heads=3, dim=8, vdim=40), mlp=U.moe()), U.layer()], width=32, vocab=30)
    m = HybridModel(HybridConfig.from_json(cfg), U.make_weights(cfg), torch.float32, "cpu")
    lay = m.cache_layout()
    assert lay[0] == ("sides", [("kv", (2, 64, 16), (2, 64, 24)), ("state", (3, 8, 40))])
    k, v, s = m.alloc_cache(5, 3)[0]
    assert k.shape == (5, 2, 64, 16) and v.shape == (5, 2, 64, 24) and s.shape == (3, 3, 8, 40) and s.dtype == torch.float32
    assert m.has_state and m.head is m.embed
    mixer = m.layers[0][1]
    assert mixer.w_in.shape[0] == mixer.off_right + 3 * (8 + 8 + 40 + 40) and mixer.off_right % 4 == 0 and mixer.n_left == 4 * 16 + 2 * 16 + 2 * 24
    assert m.layers[0][2].w_router.shape[0] % 4 == 0 and m.layers[0][2].shared_gated
