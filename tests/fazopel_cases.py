"""Configurations and model folders of the Fazopel tests: sizes of this file's own choosing and weights of its own making."""
import json
import math
import os

import torch


def _decays(heads, slowest=0.999):
    """One decay per head, from a fast one to a slow one."""
    return [round(math.exp(-0.5 / (3.0 ** i)), 12) if i < heads - 1 else slowest for i in range(heads)]


def _lin(heads, dim, vdim, mlp, decay=None, weights_of=None):
    L = dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=decay or _decays(heads)), mlp=mlp)
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def _att(heads, kv, dim, scale, rot, mlp, weights_of=None):
    m = dict(heads=heads, kv_heads=kv, dim=dim, vdim=dim, scale=scale)
    if rot:
        m["rot"] = dict(base=rot[0], dims=rot[1])
        if len(rot) > 2:
            m["rot"]["scaling"] = dict(factor=rot[2], low=rot[3], high=rot[4], original=rot[5])
    L = dict(type="attention", mixer=m, mlp=mlp)
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def _dense(ff):
    return dict(kind="dense", ff=ff)


def _moe(experts, top, scale, ff, limit, shared=None):
    m = dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top, scale=scale))
    if shared:
        m["shared"] = dict(ff=shared[0], limit=shared[1])
    return m


# Sizes that differ from layer to layer and between the configurations: key and value widths that differ, value widths
# of more than one column block of the recurrence's kernel, several kv heads and one, rotations over part of a head, over
# the whole head and none, frequency scalings whose three bands are all met and none, experts with and without a shared
# one, all experts per token, a single expert, layers without a feed-forward, layers that run another layer's weights
# (both kinds of mixers), either kind of layer first and last.
CONFIGS = {
    "A": dict(architecture="Fazopel", vocab=97, width=64, norm=dict(eps=1e-5), layers=[
        _lin(4, 16, 24, _dense(72)),
        _att(4, 2, 16, 0.3, (10000.0, 8, 4.0, 1.0, 4.0, 64), _moe(6, 2, 1.5, 32, 1.0, (40, 1.5))),
        _lin(4, 16, 24, _dense(72), weights_of=0),
        _att(4, 4, 16, 0.25, (300.0, 16), _moe(5, 1, 1.0, 40, 2.0)),
        _att(4, 2, 16, 0.3, (10000.0, 8, 4.0, 1.0, 4.0, 64), _moe(6, 2, 1.5, 32, 1.0, (40, 1.5)), weights_of=1)]),
    # sizes that fit no kernel's favourite shape: a width that is no multiple of 8, value heads of 70 (two column blocks),
    # key heads of 10 and 40, six query heads on one kv head, no rotation, all of three experts
    "B": dict(architecture="Fazopel", vocab=77, width=50, norm=dict(eps=1e-6), layers=[
        _att(6, 1, 8, 0.5, None, _moe(3, 3, 0.7, 16, 0.8, (10, 0.5))),
        _lin(3, 10, 70, None),
        _lin(2, 40, 12, _moe(9, 4, 2.5, 8, 1.2)),
        _att(2, 2, 30, 0.2, (50.0, 2), _dense(44))]),
    # the head sizes of real models: the matrix-core attention kernels and the grouped products take every layer
    "C": dict(architecture="Fazopel", vocab=211, width=128, norm=dict(eps=1e-6), layers=[
        _lin(2, 64, 64, _moe(8, 2, 2.0, 64, 1.0, (128, 1.5))),
        _att(4, 2, 64, 0.125, (500000.0, 32, 8.0, 1.0, 4.0, 2048), _dense(256)),
        _lin(1, 128, 128, _moe(16, 3, 1.0, 32, 3.0)),
        _att(2, 1, 128, 0.09, (10000.0, 128), _moe(8, 2, 2.0, 64, 1.0, (128, 1.5))),
        _lin(2, 64, 64, _moe(8, 2, 2.0, 64, 1.0, (128, 1.5)), weights_of=0)]),
    # ones everywhere: one head, one expert, decays of exactly 1 (nothing fades) and 0 (nothing is kept), one kv head
    "D": dict(architecture="Fazopel", vocab=40, width=32, norm=dict(eps=1e-5), layers=[
        _lin(1, 8, 8, _moe(1, 1, 1.0, 8, 1.0), decay=[1.0]),
        _att(1, 1, 8, 0.35, (100.0, 8), _moe(2, 1, 3.0, 4, 1.0, (8, 1.0))),
        _lin(2, 6, 10, _dense(20), decay=[0.0, 0.5])]),
}


def write_folder(path, cfg, seed, dtype=torch.bfloat16, overrides=None):
    """A model folder with weights of this file's own making: matrices N(0, 1/in) (those of the experts twice as large,
    so that the units' limits are met), norm weights near 1, router rows three times larger and small corrections (the
    scores are spread and the corrections change some choices), the embedding N(0, 1).  overrides: name -> tensor, put in
    place of what is drawn."""
    from bitnet_c_amd.config import FazopelConfig
    from bitnet_c_amd.config.fazopel import build_fazopel_plan
    from bitnet_c_amd.weights import write_file
    plan = build_fazopel_plan(FazopelConfig.from_dict(cfg))
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, spec in plan.expected_tensors().items():
        shape = tuple(spec.shape)
        if name.endswith(".correction"):
            t = 0.05 * torch.randn(shape, generator=g)
        elif len(shape) == 1:
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif name.endswith(".router"):
            t = 3.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        elif ".mlp.e" in name or ".mlp.shared." in name:
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        tensors[name] = t.to(dtype)
    for name, t in (overrides or {}).items():
        assert tuple(t.shape) == tuple(tensors[name].shape), name
        tensors[name] = t.to(dtype)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_file(os.path.join(path, "model.safetensors"), tensors)
    return str(path)


_settled = {}


def settled_tokens(folder, n, seed, margin=0.05):
    """n token ids for which no expert choice of the model in `folder` is a close call: built from left to right, a few
    tokens at a time; whatever follows the first token whose smallest routing margin (plain implementation, float64) is
    below `margin` is drawn again.  Routing is causal, so a sequence's beginning stays settled however it goes on, and one
    sequence per (folder, seed) serves every length.  A model that rounds its activations to 8 bits (its router's logits
    are then off by well under a hundredth of their size) chooses as the plain implementation does, and a difference
    between the two is a fault and not a coin that fell the other way."""
    import plain_fazopel as pf
    key = (folder, seed)
    if key not in _settled:
        _settled[key] = ([], torch.Generator().manual_seed(seed))
    toks, g = _settled[key]
    if len(toks) < n:
        cfg, W = pf.read_config(folder), pf.read_weights(folder)
        if not any(L.get("mlp") and L["mlp"]["kind"] == "moe" for L in cfg["layers"]):
            toks += torch.randint(0, cfg["vocab"], (n - len(toks),), generator=g).tolist()
        tries = 0
        while len(toks) < n:
            tries += 1
            assert tries < 100 * n, "no sequence without a close expert choice was found"
            more = torch.randint(0, cfg["vocab"], (min(16, n - len(toks)),), generator=g).tolist()
            margins = []
            pf.forward(cfg, W, toks + more, margins=margins)
            good = 0
            while good < len(more) and margins[len(toks) + good] >= margin:
                good += 1
            toks += more[:good]
    return list(toks[:n])
