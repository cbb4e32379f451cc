"""Host-side pieces of the Nepudra member (CPU): configuration reading and its errors, the registry, the previous token in the step builder and
the cache manager, and the plain implementation against closed forms."""
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import nepudra_oracle as O  # noqa: E402
import nepudra_util as U  # noqa: E402


def test_config_reading():
    from rtp_llm_amd.hybrid import HybridConfig
    from rtp_llm_amd.mixers import AttentionSpec, DeltaRuleSpec
    cfg = U.make_config([U.delta_layer(heads=3, dim=24), U.capped_layer(mlp=U.dense(ff=72)), U.capped_layer(kv_from=1),
                         U.window_layer(window=33, rot_dims=8, scaling=U.YARN, mlp=U.dense())], width=80, buckets=11, mul_prev=5, mul_cur=3)
    c = HybridConfig.from_json(cfg)
    assert c.sequential and c.scalar_norm and c.depth_mix and c.norm_offset == 0.0 and not c.branch_gates
    assert (c.bigram.buckets, c.bigram.mul_prev, c.bigram.mul_cur) == (11, 5, 3)
    d, a, s, w = [L.mixer for L in c.layers]
    assert isinstance(d, DeltaRuleSpec) and (d.heads, d.dim, d.vdim) == (3, 24, 24) and abs(d.decay_mult - math.exp(-0.5)) < 1e-12 and d.unit_eps == 1e-6
    assert isinstance(a, AttentionSpec) and a.softcap == 20.0 and a.q_temp == (0.25, 8) and a.bias and a.out_bias and a.out_gate and not a.qk_norm and a.window == 0 and a.rot is None
    assert s.kv_from == 1 and a.kv_from is None
    assert w.window == 33 and w.qk_norm and w.bias and not w.out_bias and w.out_gate and w.rot.layout == "halves" and w.rot.dims == 8 and w.rot.scaling.factor == 4.0
    assert [L.ff for L in c.layers] == [None, 72, None, 48] and all(L.mlp_act == "gelu_tanh" for L in c.layers)
    bad = U.make_config([U.capped_layer(), U.capped_layer(kv_from=1)])
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)                                           # a layer cannot read its own cache
    bad = U.make_config([U.delta_layer(), U.capped_layer(kv_from=0)])
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)                                           # nor a recurrent layer's
    bad = U.make_config([U.capped_layer(), U.capped_layer(kv_from=0, dim=8)])
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)
    bad = U.make_config([{"type": "conv", "mixer": {}, "mlp": None}])
    with pytest.raises(NotImplementedError):
        HybridConfig.from_json(bad)


def test_registry_names_the_family():
    from rtp_llm_amd import registry
    assert "nepudra" in registry.families()
    assert registry.architecture_of({"architecture": "Nepudra"}) == "Nepudra"


def test_previous_tokens_travel_with_the_step_and_stay_with_the_sequence():
    from rtp_llm_amd.kvcache import CacheManager
    from rtp_llm_amd.scheduler import ServingEngine

    class Stub:
        page, device = 64, torch.device("cpu")

        def alloc_cache(self, pages, slots):
            return []

        def forward(self, batch, tensors, collect=None):
            self.seen = batch
            return torch.zeros(batch.want.numel(), 3)

    m = Stub()
    eng = ServingEngine(m, max_tokens=256, max_seqs=2)
    eng.run_step([("a", [5, 6, 7], [2]), ("b", [9], [])])
    assert m.seen.prev.tolist() == [-1, 5, 6, -1]
    eng.run_step([("b", [4, 3], [1]), ("a", [8], [0])])
    assert m.seen.prev.tolist() == [9, 4, 7] and m.seen.tokens.tolist() == [4, 3, 8]
    eng.release("a")
    eng.run_step([("c", [1], [0])])                                           # the slot of a, used again: no previous token
    assert m.seen.prev.tolist() == [-1] and eng.cache.live["c"].last_token == 1
    cm = CacheManager(4, 64, 2)
    cm.admit("s"); cm.grow("s", 3); cm.advance("s", 3, 17)
    assert cm.live["s"].last_token == 17 and cm.live["s"].length == 3


def test_rotary_table_matches_the_oracle():
    from rtp_llm_amd.mixers import RotarySpec, rotary_table
    for rot in ({"dims": 16, "base": 10000.0}, {"dims": 8, "base": 300.0, "scaling": U.YARN},
                {"dims": 64, "base": 1e6, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}):
        f, mag = rotary_table(RotarySpec.from_json(rot, "halves"), "cpu")
        fo, mo = O.rotary_table(rot)
        assert float((f.double() - fo).abs().max()) <= 1e-7 * float(fo.max()) and abs(mag - mo) < 1e-12


def test_oracle_closed_forms():
    # delta rule with full removal along an axis-aligned unit key: the state's row is replaced by the new value
    W, d = 4, 4
    eye = torch.eye(W, dtype=torch.float64)
    wts = {"m.r": eye.clone(), "m.k": eye.clone(), "m.v": 2 * eye, "m.a": torch.zeros(d, W, dtype=torch.float64), "m.a.b": torch.full((d,), 40.0, dtype=torch.float64),
           "m.w1": torch.zeros(2, W, dtype=torch.float64), "m.w2": torch.zeros(d, 2, dtype=torch.float64), "m.w0": torch.full((d,), -40.0, dtype=torch.float64),
           "m.g": torch.zeros(d, W, dtype=torch.float64), "m.norm": torch.ones(d, dtype=torch.float64), "m.o": eye.clone()}
    h = torch.tensor([[1.0, 0, 0, 0], [1.0, 0, 0, 0], [0, 1.0, 0, 0]], dtype=torch.float64)
    _, S = O.delta_rule(h, wts, "m.", {"heads": 1, "dim": d}, 0.0)
    # token 0 writes row 0 = (2,0,0,0); token 1 removes row 0 (a = 1, u = e0, no decay) and writes it again; token 2 writes row 1
    want = torch.zeros(1, d, d, dtype=torch.float64)
    want[0, 0, 0], want[0, 1, 1] = 2.0, 2.0
    assert float((S - want).abs().max()) < 1e-5                               # the 1e-6 under the unit key's root leaves that much
    # attention: a window of one returns the own value; the cap bounds every score
    q, k, v = torch.randn(5, 2, 4, dtype=torch.float64), torch.randn(5, 1, 4, dtype=torch.float64), torch.randn(5, 1, 3, dtype=torch.float64)
    o = O.softmax_attention(q, k, v, 1.0, 0.0, 1)
    assert float((o - v.expand(5, 2, 3)).abs().max()) < 1e-12
    big = O.softmax_attention(q * 1e6, k, v, 1.0, 1e-9, 0)                    # a vanishing cap: every visible key weighs the same
    assert float((big[4, 0] - v[:, 0].mean(0)).abs().max()) < 1e-6
    # embedding: first token takes the table's last row
    e = O.embedding({"embed": torch.zeros(5, 2, dtype=torch.float64), "bigram": torch.arange(8, dtype=torch.float64).view(4, 2)}, [3, 4, 1],
                    {"buckets": 3, "mul_prev": 2, "mul_cur": 5})
    assert e.tolist() == [[6.0, 7.0], [4.0, 5.0], [2.0, 3.0]]               # rows 3, (3*2+4*5)%3 = 2, (4*2+1*5)%3 = 1
    assert abs(float(O.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12
