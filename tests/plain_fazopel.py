"""Plain, slow implementation of the Fazopel decoder, for tests only.

Whole sequences, no cache, nothing carried between calls unless a caller asks for a state, one function per mechanism,
CPU tensors in float64.  It shares no code with the package under test: its own reading of config.json, its own
safetensors reading (through the `safetensors` library), its own greedy loop.  Notation: h is a sublayer's input
[T, D]; positions count from 0; linear weights are [out, in]; the recurrence and the attention are written token by
token, the way their definitions read.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64
GATE_SLOPE = 1.702          # the expert unit's gate is g * sigmoid(GATE_SLOPE * g)
WEIGHT_FLOOR = 1e-20        # joins the sum that the chosen scores are divided by


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def read_weights(folder: str) -> dict:
    from safetensors.torch import load_file
    return {k: v.to(F64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


# ---- small pieces ----------------------------------------------------------------------------------------------

def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis; eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rotary_frequencies(rot: dict) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims / 2; with rot.scaling the long wavelengths are stretched: a wavelength below
    original/high keeps its frequency, one above original/low gets f / factor, and between the two the frequency goes
    linearly (in original / wavelength) from the one to the other."""
    dims = rot["dims"]
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if sc:
        out = []
        for fi in f.tolist():
            wave = 2.0 * math.pi / fi
            if wave < sc["original"] / sc["high"]:
                out.append(fi)
            elif wave > sc["original"] / sc["low"]:
                out.append(fi / sc["factor"])
            else:
                s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
                out.append((1.0 - s) * fi / sc["factor"] + s * fi)
        f = torch.tensor(out, dtype=F64)
    return f


def rotate_halves(x: torch.Tensor, positions, rot: dict, angle_dtype=F64) -> torch.Tensor:
    """x [T, heads, d] at the given positions [T]: dimension i is turned together with dimension i + dims / 2
    (i < dims / 2) by the angle position * f_i; dimensions from dims on pass.  angle_dtype float32: frequency and angle
    rounded as an engine that keeps them in 32 bits forms them."""
    dims = rot["dims"]
    half = dims // 2
    f = rotary_frequencies(rot).to(angle_dtype)
    pos = torch.as_tensor(list(positions), dtype=F64).to(angle_dtype)
    a = (pos[:, None] * f[None, :]).to(F64)[:, None, :]             # [T, 1, half]
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * torch.cos(a) - v * torch.sin(a)
    out[..., half:dims] = v * torch.cos(a) + u * torch.sin(a)
    return out


# ---- mixers ----------------------------------------------------------------------------------------------------

def decayed_sums(q, k, v, decay, state=None):
    """q, k [T, H, d], v [T, H, vd], decay [H]: token by token S <- decay S + k v^T, o = S^T q.  Returns (o [T, H, vd],
    the state after the last token [H, d, vd])."""
    T, H, d = q.shape
    S = torch.zeros((H, d, v.shape[-1]), dtype=F64) if state is None else state.clone()
    o = torch.zeros((T, H, v.shape[-1]), dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def lightning(h, W, p, m, eps, state=None):
    """Linear attention with a fixed decay per head.  q, k = silu of their projections [heads, dim], v = silu of its
    projection [heads, vdim]; per head S <- decay S + k v^T, o = S^T q; the heads' outputs side by side are divided by
    their common root mean square, times the weight `norm`, times sigmoid of the gate projection; then W_o.
    state: [heads, dim, vdim] carried in from earlier tokens (None: zeros).  Returns (output [T, D], state after)."""
    T = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = silu(h @ W[p + "q"].T).reshape(T, H, d)
    k = silu(h @ W[p + "k"].T).reshape(T, H, d)
    v = silu(h @ W[p + "v"].T).reshape(T, H, vd)
    o, S = decayed_sums(q, k, v, torch.tensor([float(x) for x in m["decay"]], dtype=F64), state)
    y = unit_rms(o.reshape(T, H * vd), eps) * W[p + "norm"] * sigmoid(h @ W[p + "g"].T)
    return y @ W[p + "o"].T, S


def sink_attention(h, W, p, m, eps, angle_dtype=F64, pos0: int = 0, past=None):
    """Grouped-query causal attention whose values are the key projections themselves (as projected: before the key norm
    and before the rotation).  Query and key heads are normed one by one (weights q.norm, k.norm [dim], the same for all
    heads), then their first rot.dims dimensions are rotated.  The softmax has one more term of score 0 without a value:
    p_j = exp(s_j) / (1 + sum_j exp(s_j)).  past: (keys [P, G, d], values [P, G, d]) of earlier positions.
    Returns (output, (keys, values) of all positions so far)."""
    T = h.shape[0]
    H, G, d = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    q = (h @ W[p + "q"].T).reshape(T, H, d)
    kraw = (h @ W[p + "k"].T).reshape(T, G, d)
    v = kraw.clone()
    q = unit_rms(q, eps) * W[p + "q.norm"]
    k = unit_rms(kraw, eps) * W[p + "k.norm"]
    rot = m.get("rot")
    if rot:
        q = rotate_halves(q, range(pos0, pos0 + T), rot, angle_dtype)
        k = rotate_halves(k, range(pos0, pos0 + T), rot, angle_dtype)
    if past is not None:
        k, v = torch.cat([past[0], k]), torch.cat([past[1], v])
    out = torch.zeros((T, H, d), dtype=F64)
    for t in range(T):
        n = pos0 + t + 1
        for hd in range(H):
            g = hd // (H // G)
            s = (k[:n, g] @ q[t, hd]) * m["scale"]
            top = max(float(s.max()), 0.0)
            e = torch.exp(s - top)
            w = e / (math.exp(-top) + e.sum())
            out[t, hd] = w @ v[:n, g]
    return out.reshape(T, H * d) @ W[p + "o"].T, (k, v)


# ---- feed-forwards ---------------------------------------------------------------------------------------------

def dense_ff(h, W, p):
    """W_down relu(W_up h)^2"""
    a = torch.clamp(h @ W[p + "up"].T, min=0.0)
    return (a * a) @ W[p + "down"].T


def expert_unit(h, W, p, limit: float):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))"""
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, min=-limit, max=limit)
    return (g * sigmoid(GATE_SLOPE * g) * (u + 1.0)) @ W[p + "down"].T


def route(h, W, p, mlp, margins=None):
    """(chosen experts [T, top], their weights [T, top]).  Scores are the softmax of the router's logits over all
    experts; the choice goes by score + correction, the weights are the plain scores of the chosen, divided by their sum
    and multiplied by router.scale.  margins: a list that receives, per token, how far the last chosen expert's choice
    score lies above the first one left out, in units of what a small relative change of the logits does to a score
    (score times the logits' root mean square): a small number is a close call."""
    r = mlp["router"]
    z = h @ W[p + "router"].T
    e = torch.exp(z - z.max(dim=-1, keepdim=True).values)
    s = e / e.sum(dim=-1, keepdim=True)
    c = s + W[p + "correction"]
    chosen = torch.topk(c, r["top"], dim=-1).indices
    if margins is not None:
        if r["top"] < r["experts"]:
            order = torch.argsort(c, dim=-1, descending=True)
            last, nxt = order[:, r["top"] - 1:r["top"]], order[:, r["top"]:r["top"] + 1]
            gap = (torch.gather(c, 1, last) - torch.gather(c, 1, nxt))[:, 0]
            size = torch.maximum(torch.gather(s, 1, last), torch.gather(s, 1, nxt))[:, 0] * z.pow(2).mean(dim=-1).sqrt()
            margins.append(gap / size.clamp_min(1e-300))
        else:
            margins.append(torch.full((h.shape[0],), float("inf"), dtype=F64))
    w = torch.gather(s, 1, chosen)
    w = w / (w.sum(dim=-1, keepdim=True) + WEIGHT_FLOOR) * r.get("scale", 1.0)
    return chosen, w


def moe_ff(h, W, p, mlp, margins=None):
    """The weighted sum of the chosen experts, plus (when the layer has one) a shared expert that every token runs,
    times sigmoid(W_sg h)."""
    chosen, w = route(h, W, p, mlp, margins)
    out = torch.zeros_like(h)
    for e in range(mlp["router"]["experts"]):               # expert by expert: the tokens that chose it, with their weights
        share = (w * (chosen == e)).sum(dim=-1)
        rows = torch.nonzero((chosen == e).any(dim=-1))[:, 0]
        if rows.numel():
            out[rows] += share[rows, None] * expert_unit(h[rows], W, f"{p}e{e}.", mlp["expert"]["limit"])
    if mlp.get("shared"):
        out = out + sigmoid(h @ W[p + "shared.sg"].T) * expert_unit(h, W, p + "shared.", mlp["shared"]["limit"])
    return out


# ---- the model -------------------------------------------------------------------------------------------------

def weights_prefix(c: dict, i: int) -> str:
    """A layer that names another layer under weights_of runs that layer's tensors."""
    return f"l{c['layers'][i].get('weights_of', i)}."


def layer_forward(c, W, i, x, angle_dtype=F64, round_to=None, carry=None, pos0: int = 0, margins=None):
    """x <- x + norm1(mixer(x)); x <- x + norm2(ff(x)): the sublayers read x itself, the norms sit on their outputs.
    carry: what the layer keeps from earlier tokens (a state or keys and values).  Returns (x, carry after)."""
    L, eps, p = c["layers"][i], c["norm"]["eps"], weights_prefix(c, i)
    rd = (lambda t: t.to(round_to).to(F64)) if round_to is not None else (lambda t: t)
    h = rd(x)
    if L["type"] == "lightning":
        y, carry = lightning(h, W, p + "mix.", L["mixer"], eps, carry)
    elif L["type"] == "attention":
        y, carry = sink_attention(h, W, p + "mix.", L["mixer"], eps, angle_dtype, pos0, carry)
    else:
        raise ValueError(f"unknown mixer {L['type']!r}")
    x = x + unit_rms(y, eps) * W[p + "norm1"]
    mlp = L.get("mlp")
    if mlp is not None:
        h = rd(x)
        y = dense_ff(h, W, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(h, W, p + "mlp.", mlp, margins)
        x = x + unit_rms(y, eps) * W[p + "norm2"]
    return x, carry


def forward(c: dict, W: dict, tokens, layers_out=None, angle_dtype=F64, round_to=None, margins=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  round_to: the stream is rounded to this type where a sublayer reads it
    (what an engine with activations of that type does); layers_out: a list that receives the stream after every layer;
    margins: a list that receives, per token, the smallest routing margin over all layers (see route)."""
    x = W["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    per_layer = [] if margins is not None else None
    for i in range(len(c["layers"])):
        x, _ = layer_forward(c, W, i, x, angle_dtype, round_to, margins=per_layer)
        if layers_out is not None:
            layers_out.append(x.clone())
    if margins is not None:
        low = torch.stack(per_layer).min(dim=0).values if per_layer else torch.full((len(tokens),), float("inf"), dtype=F64)
        margins.extend(low.tolist())
    h = unit_rms(x, c["norm"]["eps"]) * W["final.norm"]
    if round_to is not None:
        h = h.to(round_to).to(F64)
    return h @ W["head"].T


def generate(c: dict, W: dict, prompt, n_new: int, angle_dtype=F64, round_to=None):
    """Greedy continuation, the whole sequence run again for every token."""
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(int(forward(c, W, seq, angle_dtype=angle_dtype, round_to=round_to)[-1].argmax()))
    return seq[len(prompt):]
