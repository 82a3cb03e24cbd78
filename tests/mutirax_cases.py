"""Configurations and model folders of the Mutirax tests: sizes of this file's own choosing and weights of its own making."""
import json
import math
import os

import torch


def _par(heads, kv, dim, conv_l, scale, rot, width, blocks, conv_r, mlp):
    left = dict(heads=heads, kv_heads=kv, dim=dim, vdim=dim, conv=conv_l, scale=scale)
    if rot:
        left["rot"] = dict(base=rot[0], dims=rot[1])
    return dict(type="parallel", mixer=dict(left=left, right=dict(width=width, blocks=blocks, conv=conv_r)), mlp=mlp)


def _gla(heads, dim, vdim, tau, mlp, rank=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, tau=tau)
    if rank is not None:
        m["decay_rank"] = rank
    return dict(type="gla", mixer=m, mlp=mlp)


def _lat(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot, mlp):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale)
    if rot_dim:
        m["rot"] = dict(base=rot[0], dims=rot_dim)
        if len(rot) > 1:
            m["rot"]["scaling"] = dict(factor=rot[1], original=rot[2], fast=rot[3], slow=rot[4])
    return dict(type="latent_attention", mixer=m, mlp=mlp)


def _dense(ff, limit):
    return dict(kind="dense", ff=ff, limit=limit)


def _moe(experts, top, ff):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


def _model(vocab, width, eps, mult, layers, streams=None, loop=None):
    c = dict(architecture="Mutirax", vocab=vocab, width=width, norm=dict(eps=eps), residual_mult=mult, layers=layers)
    if streams is not None:
        c["streams"] = streams
    if loop is not None:
        c["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return c


# Sizes that differ from layer to layer and between the configurations: every kind of mixer first and last and inside
# a loop, three streams, two, one and none, loops of one layer and of all, key and value widths that differ, one kv head
# and as many as heads, rotations over part of a head, the whole head and none, convolutions of one tap (none at all) to
# seven, gate matrices in one block and in many, frequency scalings whose ramp is met inside the rotated part, all
# experts per token and a single expert, layers without a feed-forward.
CONFIGS = {
    "A": _model(131, 64, 1e-5, 0.4, [
        _par(4, 2, 16, 3, 0.3, (10000.0, 8), 48, 3, 5, _moe(6, 2, 24)),
        _gla(3, 8, 24, 12.0, _dense(72, 1.2), rank=6),
        _lat(4, 12, 8, 20, 40, 24, 0.2, (5000.0, 4.0, 64, 8.0, 1.0), _moe(5, 3, 16)),
        _par(2, 2, 32, 4, 0.2, (500.0, 32), 64, 1, 2, None)], streams=3, loop=(1, 3, 2)),
    # sizes that fit no kernel's favourite shape: a width that is no multiple of 8, six query heads on one kv head, heads of
    # 10 and 70 value columns, no rotation on the left, a loop of one layer at the end, two streams
    "B": _model(77, 50, 1e-6, 1.0, [
        _gla(2, 10, 70, 4.0, None, rank=3),
        _lat(3, 6, 2, 10, 14, 9, 0.5, (50.0,), _dense(44, 0.7)),
        _par(6, 1, 8, 1, 0.5, None, 35, 5, 7, _moe(3, 3, 12))], streams=2, loop=(2, 3, 3)),
    # the head sizes of real models: the matrix-core attention kernels and the grouped products take every layer
    "C": _model(211, 128, 1e-6, 0.5, [
        _lat(4, 32, 32, 32, 96, 48, 0.11, (100000.0, 4.0, 2048, 16.0, 2.0), _moe(6, 2, 64)),
        _par(4, 1, 64, 3, 0.11, (10000.0, 32), 128, 2, 5, _dense(256, 2.0)),
        _gla(2, 64, 64, 8.0, _moe(16, 3, 32), rank=16),
        _par(2, 1, 128, 4, 0.09, (10000.0, 64), 256, 2, 4, _moe(6, 2, 64))], streams=4, loop=(0, 2, 2)),
    # ones everywhere and no streams at all: the plain residual, one head, one expert, one block, no loop
    "D": _model(40, 32, 1e-5, 1.0, [
        _gla(1, 8, 8, 1.0, _moe(1, 1, 8), rank=1),
        _par(1, 1, 8, 2, 0.35, (100.0, 8), 16, 1, 1, _moe(2, 1, 4)),
        _lat(1, 8, 0, 8, 8, 4, 0.3, None, _dense(20, 3.0))]),
    # one stream with connection tensors, every layer in a loop
    "E": _model(53, 48, 1e-5, 0.7, [
        _lat(2, 8, 4, 12, 16, 8, 0.3, (100.0, 2.0, 16, 4.0, 1.0), _dense(40, 1.0)),
        _gla(2, 16, 8, 2.0, _moe(4, 2, 8), rank=4)], streams=1, loop=(0, 2, 2)),
}


def write_folder(path, cfg, seed, dtype=torch.bfloat16, overrides=None):
    """A model folder with weights of this file's own making: matrices N(0, 1/in) (those of the experts and the dense
    units twice as large, so that the units' limits are met), norm weights near 1 with small biases and alpha near 0.7,
    reading coefficients near 1 / streams, writing coefficients near 1 and mixing matrices near the identity, router rows three times larger with a bias
    that changes some choices, decay biases that put most decays near 1, sinks of either sign.  overrides: name -> tensor."""
    from bitnet_c_amd.config import MutiraxConfig
    from bitnet_c_amd.config.mutirax import build_mutirax_plan
    from bitnet_c_amd.weights import write_file
    plan = build_mutirax_plan(MutiraxConfig.from_dict(cfg))
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, spec in plan.expected_tensors().items():
        shape = tuple(spec.shape)
        n = lambda *s: torch.randn(s or shape, generator=g)
        if name.endswith(".alpha"):
            t = 0.7 + 0.2 * n()
        elif name.endswith(".mix") and ".hc" in name:
            t = torch.eye(shape[0]) + 0.15 * n()
        elif name.endswith(".in") and ".hc" in name:
            t = (1.0 + 0.3 * n()) / shape[0]
        elif name.endswith(".conv"):
            t = n() / math.sqrt(shape[-1]) + (torch.arange(shape[1]) == shape[1] - 1).float()
        elif name.endswith((".sink", ".lam", ".router.b")):
            t = n()
        elif name.endswith(".a2.b"):
            t = 2.0 + 2.0 * n()
        elif name.endswith(".b"):
            t = 0.2 * n()
        elif len(shape) == 1:
            t = 1.0 + 0.2 * n()
        elif name == "embed":
            t = n()
        elif name.endswith(".router"):
            t = 3.0 * n() / math.sqrt(shape[-1])
        elif ".mlp." in name:
            t = 2.0 * n() / math.sqrt(shape[-1])
        else:
            t = n() / math.sqrt(shape[-1])
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
    below `margin` is drawn again.  Routing is causal, so a sequence's beginning stays settled however it goes on."""
    import plain_mutirax as pm
    key = (folder, seed)
    if key not in _settled:
        _settled[key] = ([], torch.Generator().manual_seed(seed))
    toks, g = _settled[key]
    if len(toks) < n:
        cfg, W = pm.read_config(folder), pm.read_weights(folder)
        tries = 0
        while len(toks) < n:
            tries += 1
            assert tries < 100 * n, "no sequence without a close expert choice was found"
            more = torch.randint(0, cfg["vocab"], (min(16, n - len(toks)),), generator=g).tolist()
            margins = []
            pm.forward(cfg, W, toks + more, margins=margins)
            good = 0
            while good < len(more) and margins[len(toks) + good] >= margin:
                good += 1
            toks += more[:good]
    return list(toks[:n])
