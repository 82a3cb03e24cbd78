"""Mutirax's configuration, plan, cache needs and model folder, and the plain implementation on cases worked by hand:
what runs without a GPU."""
import copy
import math

import pytest
import torch

import plain_mutirax as pm
from mutirax_cases import CONFIGS, write_folder

F64 = torch.float64


def test_configuration_round_trip_plan_and_schedule():
    from bitnet_c_amd.config import MutiraxConfig, architecture_for
    from bitnet_c_amd.config.mutirax import build_mutirax_plan
    for name, raw in CONFIGS.items():
        assert architecture_for(raw).name == "Mutirax"
        c = MutiraxConfig.from_dict(raw)
        assert MutiraxConfig.from_dict(c.to_dict()) == c
        plan = build_mutirax_plan(c)
        assert [e.layer for e in plan.schedule] == pm.layer_runs(raw) and all(e.kv_from is None for e in plan.schedule)
        assert plan.residual_streams == raw.get("streams", 1)
        D, S = raw["width"], raw.get("streams")
        t = plan.expected_tensors()
        assert t["embed"].shape == (raw["vocab"], D) == t["head"].shape
        assert t["final.norm"].shape == t["final.norm.b"].shape == (D,) and t["final.norm.alpha"].shape == ()
        for i, L in enumerate(raw["layers"]):
            p, m = f"l{i}.", L["mixer"]
            assert t[p + "norm1"].shape == t[p + "norm1.b"].shape == (D,) and t[p + "norm1.alpha"].shape == ()
            assert (p + "hc1.in" in t) == (S is not None)
            if S is not None:
                assert t[p + "hc1.in"].shape == t[p + "hc1.out"].shape == (S,) and t[p + "hc1.mix"].shape == (S, S)
                assert (p + "hc2.mix" in t) == (L["mlp"] is not None)
            if L["type"] == "gla":
                A, B = m["heads"] * m["dim"], m["heads"] * m["vdim"]
                assert t[p + "mix.q"].shape == t[p + "mix.k"].shape == (A, D) and t[p + "mix.v"].shape == t[p + "mix.g"].shape == (B, D)
                assert t[p + "mix.a1"].shape == (m["decay_rank"], D) and t[p + "mix.a2"].shape == (A, m["decay_rank"])
                assert t[p + "mix.a2.b"].shape == (A,) and t[p + "mix.norm"].shape == (m["vdim"],) and t[p + "mix.o"].shape == (D, B)
            elif L["type"] == "latent_attention":
                H, d, r = m["heads"], m["dim"], m["rot_dim"]
                assert t[p + "mix.dq"].shape == (m["q_rank"], D) and t[p + "mix.uq"].shape == (H * (d + r), m["q_rank"])
                assert t[p + "mix.dkv"].shape == (m["kv_rank"] + r, D) and t[p + "mix.dkv.norm"].shape == (m["kv_rank"],)
                assert t[p + "mix.uk"].shape == (H * d, m["kv_rank"]) and t[p + "mix.uv"].shape == (H * m["vdim"], m["kv_rank"])
                assert t[p + "mix.g"].shape == (H, D) and t[p + "mix.o"].shape == (D, H * m["vdim"])
            else:
                l, r = m["left"], m["right"]
                Q, K, W = l["heads"] * l["dim"], l["kv_heads"] * l["dim"], r["width"]
                assert t[p + "mix.left.q"].shape == (Q, D) and t[p + "mix.left.k"].shape == (K, D) and p + "mix.left.v" not in t
                assert t[p + "mix.left.q.conv"].shape == (Q, l["conv"]) and t[p + "mix.left.k.conv"].shape == (K, l["conv"])
                assert t[p + "mix.left.q.norm"].shape == (Q,) and t[p + "mix.left.k.norm"].shape == (K,)
                assert t[p + "mix.left.sink"].shape == (l["heads"],) and t[p + "mix.left.out"].shape == t[p + "mix.right.out"].shape == (D,)
                assert t[p + "mix.right.y"].shape == t[p + "mix.right.x"].shape == (W, D) and t[p + "mix.right.conv"].shape == (W, r["conv"])
                assert t[p + "mix.right.ra"].shape == t[p + "mix.right.ri"].shape == (r["blocks"], W // r["blocks"], W // r["blocks"])
                assert t[p + "mix.right.ra.b"].shape == (r["blocks"], W // r["blocks"]) and t[p + "mix.right.lam"].shape == (W,)
            mlp = L["mlp"]
            assert (p + "norm2" in t) == (mlp is not None)
            if mlp is None:
                assert not [n for n in t if n.startswith(p + "mlp.")]
            elif mlp["kind"] == "dense":
                assert t[p + "mlp.gate"].shape == t[p + "mlp.up"].shape == (mlp["ff"], D) and t[p + "mlp.down"].shape == (D, mlp["ff"])
            else:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                assert t[p + "mlp.router"].shape == (E, D) and t[p + "mlp.router.b"].shape == (E,)
                assert t[f"{p}mlp.e{E - 1}.gate"].shape == (F, D) and t[f"{p}mlp.e0.down"].shape == (D, F)


def test_the_decay_rank_comes_from_the_folder(tmp_path):
    from bitnet_c_amd.config import load_config
    raw = copy.deepcopy(CONFIGS["B"])
    folder = write_folder(tmp_path / "m", raw, 1)
    stripped = copy.deepcopy(raw)
    del stripped["layers"][0]["mixer"]["decay_rank"]          # config.json does not say it; the tensor a1 does
    import json, os
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(stripped, f)
    arch, c = load_config(folder)
    assert arch.name == "Mutirax" and c.layers[0].mixer.decay_rank == 3


def test_every_run_of_a_looped_layer_has_storage_of_its_own():
    from bitnet_c_amd.cache import PagedCache
    from bitnet_c_amd.config import MutiraxConfig
    from bitnet_c_amd.config.mutirax import build_mutirax_plan
    from bitnet_c_amd.parts import BLOCKS
    raw = CONFIGS["A"]
    plan = build_mutirax_plan(MutiraxConfig.from_dict(raw))
    blocks = [BLOCKS.build(lp.block) for lp in plan.layers]
    needs = [blocks[e.layer].cache_need() for e in plan.schedule]
    runs = pm.layer_runs(raw)
    assert runs == [0, 1, 2, 1, 2, 3] and len(needs) == 6
    l0, r0 = raw["layers"][0]["mixer"]["left"], raw["layers"][0]["mixer"]["right"]
    conv_l = (l0["conv"] - 1) * (l0["heads"] + l0["kv_heads"]) * l0["dim"]
    assert needs[0].state.shape == (conv_l + r0["width"] * r0["conv"],) and needs[0].kv.n_kv_heads == l0["kv_heads"]
    g = raw["layers"][1]["mixer"]
    assert needs[1].kv is None and needs[1].state.shape == (g["heads"] * g["dim"] * g["vdim"],) and needs[3].state == needs[1].state
    lat = raw["layers"][2]["mixer"]
    assert needs[2].state is None and needs[2].kv.head_dim == lat["kv_rank"] + lat["rot_dim"] and needs[2].kv.v_dim == lat["kv_rank"]
    cache = PagedCache(needs, [None] * 6, 256, dtype=torch.float32, device=None)
    assert cache.group_of(2) == cache.group_of(4) and cache.group_of(0) != cache.group_of(2) and cache.group_of(1) is None
    assert sorted(cache._state_needs) == [0, 1, 3, 5]


def _bad(raw, change, match):
    from bitnet_c_amd.config import ConfigError, MutiraxConfig
    raw = copy.deepcopy(raw)
    change(raw)
    with pytest.raises(ConfigError, match=match):
        MutiraxConfig.from_dict(raw)


def test_configurations_that_cannot_be_are_refused():
    A = CONFIGS["A"]
    _bad(A, lambda r: r["layers"][0].update(type="conv"), "type")
    _bad(A, lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3), "kv_heads")
    _bad(A, lambda r: r["layers"][0]["mixer"]["left"].update(vdim=8), "vdim")
    _bad(A, lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "dims")
    _bad(A, lambda r: r["layers"][0]["mixer"]["right"].update(blocks=5), "equal parts")
    _bad(A, lambda r: r["layers"][1]["mixer"].update(tau=0), "tau")
    _bad(A, lambda r: r["layers"][2]["mixer"].pop("rot"), "rot")
    _bad(A, lambda r: r["layers"][0]["mlp"]["router"].update(top=7), "top")
    _bad(A, lambda r: r["layers"][1]["mlp"].pop("limit"), "limit")
    _bad(A, lambda r: r.update(loop=dict(start=2, stop=2, times=2)), "loop")
    _bad(A, lambda r: r.update(loop=dict(start=0, stop=5, times=2)), "loop")
    _bad(A, lambda r: r.update(streams=0), "streams")


def test_the_plain_pieces_on_cases_worked_by_hand():
    # the convolution: the last column meets the current token, zeros before the start
    u = torch.tensor([[1.0], [2.0], [4.0]], dtype=F64)
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=F64)
    assert pm.short_convolution(u, w).reshape(-1).tolist() == [1.0, 12.0, 124.0]
    # streams: two copies, the read sums them with `in`, the write mixes [from, to]
    cfg = dict(norm=dict(eps=1e-5), residual_mult=0.5, streams=2, vocab=2, width=1, layers=[])
    W = {"embed": torch.tensor([[1.0], [3.0]], dtype=F64), "head": torch.tensor([[1.0], [0.0]], dtype=F64),
         "final.norm": torch.ones(1, dtype=F64), "final.norm.b": torch.zeros(1, dtype=F64), "final.norm.alpha": torch.tensor(1.0, dtype=F64)}
    assert abs(float(pm.forward(cfg, W, [1])[0, 0]) - math.tanh(6.0)) < 1e-12          # the end is the streams' sum
    # the rescaled frequencies: one factor for cosine and sine, the ramp's ends
    f, mult = pm.rotary_table(dict(base=100.0, dims=8, scaling=dict(factor=4.0, original=16, fast=8.0, slow=0.5)))
    assert abs(mult - (0.1 * math.log(4.0) + 1.0)) < 1e-15 and abs(float(f[0]) - 1.0) < 1e-15 and abs(float(f[-1]) - 100.0 ** -0.75 / 4.0) < 1e-15
    # the loop runs its layers as a block
    assert pm.layer_runs(dict(layers=[0] * 5, loop=dict(start=1, stop=3, times=3))) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    # a sink that takes half: one key of score 0 beside a sink of 0
    W = {"q": torch.zeros(2, 2, dtype=F64), "k": torch.eye(2, dtype=F64), "q.conv": torch.ones(2, 1, dtype=F64), "k.conv": torch.ones(2, 1, dtype=F64),
         "q.norm": torch.ones(2, dtype=F64), "k.norm": torch.ones(2, dtype=F64), "sink": torch.zeros(1, dtype=F64), "o": torch.eye(2, dtype=F64)}
    y = pm.sink_attention(torch.tensor([[2.0, 4.0]], dtype=F64), W, "", dict(heads=1, kv_heads=1, dim=2, scale=1.0), 1e-5)
    assert torch.allclose(y, torch.tensor([[1.0, 2.0]], dtype=F64))
