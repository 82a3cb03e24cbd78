"""Fazopel's configuration, plan, cache needs and model folder, and the plain implementation on cases worked by hand:
what runs without a GPU."""
import copy
import math
import os

import pytest
import torch

import plain_fazopel as pf
from fazopel_cases import CONFIGS, settled_tokens, write_folder

F64 = torch.float64


def test_configuration_round_trip_and_plan():
    from bitnet_c_amd.config import FazopelConfig, architecture_for
    from bitnet_c_amd.config.fazopel import build_fazopel_plan
    for name, raw in CONFIGS.items():
        assert architecture_for(raw).name == "Fazopel"
        c = FazopelConfig.from_dict(raw)
        assert FazopelConfig.from_dict(c.to_dict()) == c
        assert c.to_dict()["layers"] == raw["layers"]
        plan = build_fazopel_plan(c)
        own = [i for i, L in enumerate(raw["layers"]) if "weights_of" not in L]
        assert len(plan.layers) == len(own) and len(plan.schedule) == len(raw["layers"])
        D = raw["width"]
        t = plan.expected_tensors()
        assert t["embed"].shape == (raw["vocab"], D) == t["head"].shape and t["final.norm"].shape == (D,)
        for i, (e, L) in enumerate(zip(plan.schedule, raw["layers"])):
            assert e.layer == own.index(L.get("weights_of", i)) and e.kv_from is None
            p, m = f"l{i}.", L["mixer"]
            if "weights_of" in L:
                assert not [n for n in t if n.startswith(p)]
                continue
            assert t[p + "norm1"].shape == (D,)
            if L["type"] == "attention":
                assert t[p + "mix.q"].shape == (m["heads"] * m["dim"], D) and t[p + "mix.k"].shape == (m["kv_heads"] * m["dim"], D)
                assert t[p + "mix.o"].shape == (D, m["heads"] * m["dim"]) and p + "mix.v" not in t
                assert t[p + "mix.q.norm"].shape == t[p + "mix.k.norm"].shape == (m["dim"],)
            else:
                assert t[p + "mix.q"].shape == t[p + "mix.k"].shape == (m["heads"] * m["dim"], D)
                assert t[p + "mix.v"].shape == t[p + "mix.g"].shape == (m["heads"] * m["vdim"], D)
                assert t[p + "mix.o"].shape == (D, m["heads"] * m["vdim"]) and t[p + "mix.norm"].shape == (m["heads"] * m["vdim"],)
            mlp = L["mlp"]
            assert (p + "norm2" in t) == (mlp is not None)
            if mlp is None:
                assert not [n for n in t if n.startswith(p + "mlp.")]
            elif mlp["kind"] == "dense":
                assert t[p + "mlp.up"].shape == (mlp["ff"], D) and t[p + "mlp.down"].shape == (D, mlp["ff"])
            else:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                assert t[p + "mlp.router"].shape == (E, D) and t[p + "mlp.correction"].shape == (E,)
                assert sorted(n for n in t if n.startswith(p + "mlp.e")) == sorted(
                    f"{p}mlp.e{e}.{w}" for e in range(E) for w in ("gate", "up", "down"))
                assert t[f"{p}mlp.e{E - 1}.gate"].shape == (F, D) and t[f"{p}mlp.e0.down"].shape == (D, F)
                assert (p + "mlp.shared.sg" in t) == ("shared" in mlp)
                if "shared" in mlp:
                    Fs = mlp["shared"]["ff"]
                    assert t[p + "mlp.shared.gate"].shape == t[p + "mlp.shared.up"].shape == (Fs, D)
                    assert t[p + "mlp.shared.down"].shape == (D, Fs) and t[p + "mlp.shared.sg"].shape == (1, D)


def _bad(raw, change, match):
    from bitnet_c_amd.config import ConfigError, FazopelConfig
    raw = copy.deepcopy(raw)
    change(raw)
    with pytest.raises(ConfigError, match=match):
        FazopelConfig.from_dict(raw)


def test_configurations_that_cannot_be_are_refused():
    A = CONFIGS["A"]
    _bad(A, lambda r: r["layers"][0].update(type="conv"), "type")
    _bad(A, lambda r: r["layers"][0]["mixer"].update(decay=[0.5]), "decay")
    _bad(A, lambda r: r["layers"][0]["mixer"].update(decay=[0.5, 0.5, 0.5, 1.5]), "decay")
    _bad(A, lambda r: r["layers"][1]["mixer"].update(kv_heads=3), "kv_heads")
    _bad(A, lambda r: r["layers"][1]["mixer"].update(vdim=8), "vdim")
    _bad(A, lambda r: r["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims")
    _bad(A, lambda r: r["layers"][1]["mixer"]["rot"].update(dims=18), "rot.dims")
    _bad(A, lambda r: r["layers"][1]["mixer"]["rot"]["scaling"].pop("factor"), "factor")
    _bad(A, lambda r: r["layers"][1]["mixer"].pop("scale"), "scale")
    _bad(A, lambda r: r["layers"][0]["mlp"].update(kind="glu"), "kind")
    _bad(A, lambda r: r["layers"][1]["mlp"]["router"].update(top=7), "top")
    _bad(A, lambda r: r["layers"][1]["mlp"]["expert"].pop("limit"), "limit")
    _bad(A, lambda r: r["layers"][2].update(weights_of=2), "weights_of")
    _bad(A, lambda r: r["layers"][2].update(weights_of=1), "differs")
    _bad(A, lambda r: r["layers"][4].update(weights_of=2), "none of its own|differs")
    _bad(A, lambda r: r.pop("norm"), "norm")
    _bad(A, lambda r: r.update(layers=[]), "layers")


def test_cache_needs_states_pages_and_shared_weights():
    """A lightning layer keeps a float32 matrix per head and no pages, an attention layer keeps keys and values as wide as
    its keys; layers that run one layer's weights have a state or pages each."""
    from bitnet_c_amd.cache import PAGE, PagedCache
    from bitnet_c_amd.config import FazopelConfig
    from bitnet_c_amd.config.fazopel import build_fazopel_plan
    from bitnet_c_amd.parts import BLOCKS
    raw = CONFIGS["A"]
    plan = build_fazopel_plan(FazopelConfig.from_dict(raw))
    needs = [BLOCKS.build(plan.layers[e.layer].block).cache_need() for e in plan.schedule]
    for need, L in zip(needs, raw["layers"]):
        m = L["mixer"]
        if L["type"] == "attention":
            assert need.state is None
            assert (need.kv.n_kv_heads, need.kv.head_dim, need.kv.v_dim, need.kv.window) == (m["kv_heads"], m["dim"], m["dim"], 0)
        else:
            assert need.kv is None and need.state.shape == (m["heads"] * m["dim"] * m["vdim"],)
            assert need.state.dtype == torch.float32 and need.state.device_addressed
    cache = PagedCache(needs, [e.kv_from for e in plan.schedule], 16 * PAGE)
    assert len(cache.groups) == 2 and cache.group_of(1) == cache.group_of(4) != cache.group_of(3)
    assert cache.group_of(0) is None and sorted(cache._state_needs) == [0, 2]
    tables = {g: None for g in range(2)}
    assert cache.view(1, tables, 0).writes and cache.view(4, tables, 0).writes
    s = cache.alloc_slot()
    cache.reserve([s], [3 * PAGE + 1])
    cache.commit([s], [3 * PAGE + 1])
    assert [len(cache.pages_of(g, s)) for g in range(2)] == [4, 4]
    cache.free_slot(s)
    cache.check()


def test_random_weights_folder_and_plain_reading(tmp_path):
    """The library writes a folder from a configuration alone; the plain implementation reads it and runs."""
    from bitnet_c_amd.config import FazopelConfig, load_config
    from bitnet_c_amd.weights import write_model_folder
    folder = write_model_folder(str(tmp_path / "made"), FazopelConfig.from_dict(CONFIGS["B"]), 5, torch.bfloat16)
    arch, cfg = load_config(folder)
    assert arch.name == "Fazopel" and cfg == FazopelConfig.from_dict(CONFIGS["B"])
    logits = pf.forward(pf.read_config(folder), pf.read_weights(folder), [1, 2, 3, 4])
    assert logits.shape == (4, 77) and bool(torch.isfinite(logits).all())


def test_a_folder_with_a_tensor_missing_or_left_over_is_refused(tmp_path):
    from safetensors.torch import load_file
    from bitnet_c_amd.config import FazopelConfig
    from bitnet_c_amd.config.fazopel import build_fazopel_plan
    from bitnet_c_amd.weights import WeightError, open_tensors, write_file
    folder = write_folder(tmp_path / "m", CONFIGS["A"], 1)
    plan = build_fazopel_plan(FazopelConfig.from_dict(CONFIGS["A"]))
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    tensors["l1.mix.v"] = tensors.pop("l1.mix.k")                   # an attention layer has no value matrix
    tensors["l1.mlp.e5.gate"] = tensors["l1.mlp.e5.gate"][:-1].contiguous()
    tensors["l2.norm1"] = tensors["l0.norm1"].clone()               # a layer that runs another's weights has no tensors
    write_file(os.path.join(folder, "model.safetensors"), tensors)
    with pytest.raises(WeightError) as err:
        open_tensors(folder, plan.expected_tensors())
    assert err.value.missing == ["l1.mix.k"] and err.value.unexpected == ["l1.mix.v", "l2.norm1"]
    assert [n for n, _, _ in err.value.wrong_shape] == ["l1.mlp.e5.gate"]


def test_the_plain_mechanisms_on_cases_worked_by_hand():
    """The oracle itself, where a result can be written down."""
    g = torch.Generator().manual_seed(0)
    T, D = 6, 8
    h = torch.randn(T, D, generator=g, dtype=F64)
    # decayed sums: decay 0 keeps the current token alone, decay 1 sums everything; one token is (q . k) v
    q, k, v = (torch.randn(T, 2, 3, generator=g, dtype=F64), torch.randn(T, 2, 3, generator=g, dtype=F64),
               torch.randn(T, 2, 5, generator=g, dtype=F64))
    o, S = pf.decayed_sums(q, k, v, torch.tensor([0.0, 1.0], dtype=F64))
    assert torch.allclose(o[:, 0], (q[:, 0] * k[:, 0]).sum(-1, keepdim=True) * v[:, 0])
    scores = torch.tril(q[:, 1] @ k[:, 1].T)
    assert torch.allclose(o[:, 1], scores @ v[:, 1]) and torch.allclose(S[1], k[:, 1].T @ v[:, 1])
    o2, _ = pf.decayed_sums(q[4:], k[4:], v[4:], torch.tensor([0.0, 1.0], dtype=F64), pf.decayed_sums(q[:4], k[:4], v[:4], torch.tensor([0.0, 1.0], dtype=F64))[1])
    assert torch.allclose(o2, o[4:])
    half = 0.5 ** torch.arange(T - 1, -1, -1, dtype=F64)                       # decay 1/2: the weights of the last token's sum
    o3, _ = pf.decayed_sums(q[:, :1], k[:, :1], v[:, :1], torch.tensor([0.5], dtype=F64))
    assert torch.allclose(o3[-1, 0], ((k[:, 0] @ q[-1, 0]) * half) @ v[:, 0])
    # attention: one token sees itself and the sink; its value is its key projection as projected
    W = {"q": torch.randn(4, D, generator=g, dtype=F64), "k": torch.randn(4, D, generator=g, dtype=F64), "o": torch.eye(4, dtype=F64),
         "q.norm": torch.ones(4, dtype=F64), "k.norm": torch.ones(4, dtype=F64)}
    m = dict(heads=1, kv_heads=1, dim=4, vdim=4, scale=0.5, rot=dict(base=10.0, dims=4))
    y, (keys, values) = pf.sink_attention(h[:1], W, "", m, 1e-6)
    s = float((pf.unit_rms(h[:1] @ W["q"].T, 1e-6) * pf.unit_rms(h[:1] @ W["k"].T, 1e-6)).sum()) * 0.5
    assert torch.allclose(y[0], math.exp(s) / (1.0 + math.exp(s)) * (h[0] @ W["k"].T))
    assert torch.equal(values[0, 0], h[0] @ W["k"].T)
    whole, _ = pf.sink_attention(h, W, "", m, 1e-6)
    first, past = pf.sink_attention(h[:4], W, "", m, 1e-6)
    rest, _ = pf.sink_attention(h[4:], W, "", m, 1e-6, pos0=4, past=past)
    assert torch.allclose(torch.cat([first, rest]), whole)
    # rotation: position 0 changes nothing, lengths stay, dimensions beyond rot.dims pass, the pair is (i, i + dims / 2)
    x = torch.randn(3, 2, 6, generator=g, dtype=F64)
    r = pf.rotate_halves(x, [0, 3, 11], dict(base=100.0, dims=4))
    assert torch.equal(r[0], x[0]) and torch.equal(r[..., 4:], x[..., 4:])
    assert torch.allclose(r[..., :4].pow(2).sum(-1), x[..., :4].pow(2).sum(-1))
    assert torch.allclose(r[1, 0, 0], x[1, 0, 0] * math.cos(3.0) - x[1, 0, 2] * math.sin(3.0))
    assert torch.allclose(r[1, 0, 3], x[1, 0, 3] * math.cos(0.3) + x[1, 0, 1] * math.sin(0.3))
    # stretched wavelengths: the three bands
    f = pf.rotary_frequencies(dict(base=10000.0, dims=8, scaling=dict(factor=4.0, low=1.0, high=4.0, original=64)))
    assert f[0] == 1.0 and torch.allclose(f[2:], torch.tensor([1e-2 / 4, 1e-3 / 4], dtype=F64))
    s1 = (64 / (2 * math.pi / 0.1) - 1.0) / 3.0
    assert abs(float(f[1]) - ((1 - s1) * 0.1 / 4 + s1 * 0.1)) < 1e-15
    # the expert unit: both clamps, and a limit that never bites leaves g sigmoid(1.702 g) (u + 1)
    We = {"gate": torch.tensor([[3.0], [-5.0], [0.5]], dtype=F64), "up": torch.tensor([[4.0], [-4.0], [0.25]], dtype=F64),
          "down": torch.eye(3, dtype=F64)}
    y = pf.expert_unit(torch.ones(1, 1, dtype=F64), We, "", 2.0)[0]
    sg = lambda z: 1.0 / (1.0 + math.exp(-z))
    assert torch.allclose(y, torch.tensor([2.0 * sg(3.404) * 3.0, -5.0 * sg(-8.51) * -1.0, 0.5 * sg(0.851) * 1.25], dtype=F64))
    # the router: the correction changes the choice and not the weights; one expert gets the constant itself
    Wr = {"router": torch.tensor([[1.0], [0.9], [-1.0]], dtype=F64), "correction": torch.tensor([0.0, 0.0, 5.0], dtype=F64)}
    chosen, w = pf.route(torch.ones(1, 1, dtype=F64), Wr, "", dict(router=dict(experts=3, top=2, scale=3.0)))
    sc = torch.softmax(torch.tensor([1.0, 0.9, -1.0], dtype=F64), 0)
    assert sorted(chosen[0].tolist()) == [0, 2] and abs(float(w.sum()) - 3.0) < 1e-12
    assert torch.allclose(w[0].sort().values, (3.0 * sc[[2, 0]] / (sc[0] + sc[2])))
    _, w1 = pf.route(torch.ones(1, 1, dtype=F64), Wr, "", dict(router=dict(experts=3, top=1, scale=3.0)))
    assert abs(float(w1) - 3.0) < 1e-12


def test_settled_sequences_have_no_close_expert_choice(tmp_path):
    folder = write_folder(tmp_path / "m", CONFIGS["A"], 2)
    toks = settled_tokens(folder, 60, 4)
    assert settled_tokens(folder, 40, 4) == toks[:40]
    margins = []
    pf.forward(pf.read_config(folder), pf.read_weights(folder), toks, margins=margins)
    assert len(margins) == 60 and min(margins) >= 0.05
