"""Plain, slow implementation of the Mutirax decoder, for tests only.

Whole sequences, no cache, nothing carried between calls, one function per mechanism, CPU tensors in float64.  It shares
no code with the package under test: its own reading of config.json, its own safetensors reading (through the
`safetensors` library), its own greedy loop.  Notation: h is a sublayer's input [T, D]; positions count from 0; linear
weights are [out, in]; recurrences and attention are written token by token, the way their definitions read.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64
GATE_SLOPE = 1.702          # the dense unit's gate is g * sigmoid(GATE_SLOPE * g)
LRU_SHARPNESS = 8.0         # log a = -LRU_SHARPNESS * r * softplus(lam)


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def read_weights(folder: str) -> dict:
    from safetensors.torch import load_file
    return {k: v.to(F64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


# ---- small pieces ----------------------------------------------------------------------------------------------

def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis; eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def tanh_norm(x, W, name):
    """No mean, no variance: tanh(alpha x) * w + b with one number alpha."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


def rotary_table(rot: dict):
    """(frequencies f_i for i < dims / 2, the factor that multiplies every cosine and sine).  Without rot.scaling
    f_i = base^(-2i/dims) and the factor is 1.  With it, let d(t) = dims ln(original / (2 pi t)) / (2 ln base),
    lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1):
    the frequency is f_i / factor where r_i = 1, f_i where r_i = 0 and the mix of both between, and the factor is
    0.1 ln(factor) + 1."""
    dims, base = rot["dims"], float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0

    def d(t):
        return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo, hi = max(math.floor(d(sc["fast"])), 0), min(math.ceil(d(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / sc["factor"] * r + fi * (1.0 - r))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_halves(x, positions, rot: dict):
    """x [T, heads, d] at positions [T]: dimension i turns with dimension i + dims / 2 by the angle position * f_i;
    dimensions from dims on pass unchanged."""
    dims = rot["dims"]
    half = dims // 2
    f, mult = rotary_table(rot)
    a = (torch.as_tensor(list(positions), dtype=F64)[:, None] * f[None, :])[:, None, :]
    c, s = torch.cos(a) * mult, torch.sin(a) * mult
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def short_convolution(u, w, bias=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first token; the last column
    of w meets the current token."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros((T, C), dtype=F64)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y if bias is None else y + bias


# ---- mixers ----------------------------------------------------------------------------------------------------

def gated_linear_attention(h, W, p, m, eps):
    """q = W_q h / sqrt(dim), k = W_k h [heads, dim], v = W_v h [heads, vdim]; a decay per key channel,
    alpha = sigmoid(W_a2 W_a1 h + b)^(1 / tau); per head S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t; every head's o
    divided by its root mean square, times `norm` [vdim]; heads side by side times silu(W_g h); W_o."""
    T = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).reshape(T, H, d)
    v = (h @ W[p + "v"].T).reshape(T, H, vd)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, d)
    S = torch.zeros((H, d, vd), dtype=F64)
    o = torch.zeros((T, H, vd), dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    y = (unit_rms(o, eps) * W[p + "norm"]).reshape(T, H * vd) * silu(h @ W[p + "g"].T)
    return y @ W[p + "o"].T


def latent_attention(h, W, p, m, eps):
    """Queries through a normed latent; keys and values from a normed latent c of kv_rank numbers per token plus one
    rotated key part of rot_dim numbers that all heads share.  Head i's query is [dim plain, rot_dim rotated]; its score
    against position j is (q_plain . W_uk,i c_j + q_rot . k_rot,j) * scale; causal softmax; values W_uv,i c_j; head i's
    output times sigmoid of the i-th of `heads` gate numbers; W_o."""
    T = h.shape[0]
    H, d, r, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = unit_rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).reshape(T, H, d + r)
    dkv = h @ W[p + "dkv"].T
    c = unit_rms(dkv[:, :R], eps) * W[p + "dkv.norm"]
    if r:
        rot = dict(m["rot"], dims=r)
        k_rot = rotate_halves(dkv[:, R:].reshape(T, 1, r), range(T), rot)[:, 0]
        q_rot = rotate_halves(q[..., d:], range(T), rot)
    else:                                                 # no rotated part: the plain scores alone
        k_rot, q_rot = torch.zeros((T, 0), dtype=F64), torch.zeros((T, H, 0), dtype=F64)
    k = (c @ W[p + "uk"].T).reshape(T, H, d)
    v = (c @ W[p + "uv"].T).reshape(T, H, vd)
    gate = sigmoid(h @ W[p + "g"].T)                      # [T, H]
    out = torch.zeros((T, H, vd), dtype=F64)
    for t in range(T):
        s = (torch.einsum("hd,jhd->hj", q[t, :, :d], k[:t + 1]) + q_rot[t] @ k_rot[:t + 1].T) * m["scale"]
        w = torch.softmax(s, dim=-1)
        out[t] = torch.einsum("hj,jhv->hv", w, v[:t + 1]) * gate[t][:, None]
    return out.reshape(T, H * vd) @ W[p + "o"].T


def sink_attention(h, W, p, m, eps):
    """Grouped-query causal attention without a value matrix.  q, k = projections, then a short convolution over time on
    every channel; the values are the keys as they leave the convolution; q and k are then divided by the root mean
    square of their whole rows (weights q.norm, k.norm), split into heads and rotated.  The softmax's denominator holds
    one more term exp(sink_head)."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = short_convolution(h @ W[p + "q"].T, W[p + "q.conv"])
    k = short_convolution(h @ W[p + "k"].T, W[p + "k.conv"])
    v = k.reshape(T, G, d)
    q = (unit_rms(q, eps) * W[p + "q.norm"]).reshape(T, H, d)
    k = (unit_rms(k, eps) * W[p + "k.norm"]).reshape(T, G, d)
    if m.get("rot"):
        q, k = rotate_halves(q, range(T), m["rot"]), rotate_halves(k, range(T), m["rot"])
    out = torch.zeros((T, H, d), dtype=F64)
    for t in range(T):
        for i in range(H):
            g = i // (H // G)
            s = (k[:t + 1, g] @ q[t, i]) * m["scale"]
            top = torch.maximum(s.max(), W[p + "sink"][i])
            e = torch.exp(s - top)
            out[t, i] = (e[:, None] * v[:t + 1, g]).sum(0) / (e.sum() + torch.exp(W[p + "sink"][i] - top))
    return out.reshape(T, H * d) @ W[p + "o"].T


def gated_recurrent_unit(h, W, p, m):
    """Two branches `width` wide: y = gelu_tanh(W_y h + b), u = convolution(W_x h + b) with a bias.  u in `blocks` equal
    parts; in part b, r = sigmoid(ra[b] u_b + b) and i = sigmoid(ri[b] u_b + b).  log a = -8 r softplus(lam);
    S <- a S + sqrt(1 - a^2) i u from S = 0; output W_o (S * y)."""
    T = h.shape[0]
    Wd, B = m["width"], m["blocks"]
    y = gelu_tanh(h @ W[p + "y"].T + W[p + "y.b"])
    u = short_convolution(h @ W[p + "x"].T + W[p + "x.b"], W[p + "conv"], W[p + "conv.b"])
    ub = u.reshape(T, B, Wd // B)
    r = sigmoid(torch.einsum("boi,tbi->tbo", W[p + "ra"], ub) + W[p + "ra.b"]).reshape(T, Wd)
    i = sigmoid(torch.einsum("boi,tbi->tbo", W[p + "ri"], ub) + W[p + "ri.b"]).reshape(T, Wd)
    a = torch.exp(-LRU_SHARPNESS * r * softplus(W[p + "lam"]))
    S = torch.zeros(Wd, dtype=F64)
    out = torch.zeros((T, Wd), dtype=F64)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ W[p + "o"].T


def side_by_side(h, W, p, m, eps):
    """Both mixers read h; each output is divided by its root mean square over the width, times its weight; half the sum."""
    a = sink_attention(h, W, p + "left.", m["left"], eps)
    b = gated_recurrent_unit(h, W, p + "right.", m["right"])
    return 0.5 * (unit_rms(a, eps) * W[p + "left.out"] + unit_rms(b, eps) * W[p + "right.out"])


MIXERS = {"gla": gated_linear_attention, "latent_attention": latent_attention, "parallel": side_by_side}


# ---- feed-forwards ---------------------------------------------------------------------------------------------

def dense_unit(h, W, p, mlp):
    g = (h @ W[p + "gate"].T).clamp(max=mlp["limit"])
    u = (h @ W[p + "up"].T).clamp(min=-mlp["limit"], max=mlp["limit"])
    return (g * sigmoid(GATE_SLOPE * g) * (u + 1.0)) @ W[p + "down"].T


def expert_mixture(h, W, p, mlp, margins=None):
    """Router logits W_router h + b; the `top` largest are chosen and weighted by the softmax over the chosen alone; an
    expert is W_down (silu(W_gate h) * (W_up h)).  margins: a list of one number per token, lowered to the distance
    between the last chosen logit and the first one left out."""
    z = h @ W[p + "router"].T + W[p + "router.b"]
    top = mlp["router"]["top"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        val, idx = torch.topk(z[t], top)
        if margins is not None and top < z.shape[1]:
            rest = torch.topk(z[t], top + 1)[0]
            margins[t] = min(margins[t], float(rest[top - 1] - rest[top]))
        w = torch.softmax(val, dim=-1)
        for wt, e in zip(w.tolist(), idx.tolist()):
            q = f"{p}e{e}."
            out[t] += wt * ((silu(W[q + "gate"] @ h[t]) * (W[q + "up"] @ h[t])) @ W[q + "down"].T)
    return out


def feed_forward(h, W, p, mlp, margins=None):
    return dense_unit(h, W, p, mlp) if mlp["kind"] == "dense" else expert_mixture(h, W, p, mlp, margins)


# ---- the model -------------------------------------------------------------------------------------------------

def layer_runs(cfg: dict):
    """The layers in the order they run: those of the loop `times` times in a row, as a block."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b = loop["start"], loop["stop"]
    return list(range(a)) + list(range(a, b)) * loop["times"] + list(range(b, n))


def forward(cfg: dict, W: dict, tokens, collect=None, margins=None):
    """Logits [T, vocab] of one whole sequence.  collect: a list that receives the sum of the streams after every layer
    run.  The residual is `streams` copies of the embedding; a sublayer reads their sum weighted by `in`, and all copies
    are rebuilt at once from the old ones: x_t <- sum_s mix[s, t] x_s + m out[t] y.  Without `streams` in the configuration
    there is one residual and x <- x + m y."""
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    S = cfg.get("streams")
    x0 = W["embed"][torch.as_tensor(list(tokens))]
    if margins is not None:
        margins[:] = [float("inf")] * len(tokens)          # margins: every token's smallest routing margin over the layers
    X = torch.stack([x0] * (S or 1))

    def sublayer(X, name, fn, q):
        if S is None:
            return X + m * fn(tanh_norm(X[0], W, name))[None]
        u = torch.einsum("s,std->td", W[q + ".in"], X)
        y = fn(tanh_norm(u, W, name))
        return torch.einsum("sr,std->rtd", W[q + ".mix"], X) + m * W[q + ".out"][:, None, None] * y[None]

    for i in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        X = sublayer(X, p + "norm1", lambda hh: MIXERS[L["type"]](hh, W, p + "mix.", L["mixer"], eps), p + "hc1")
        if L.get("mlp") is not None:
            X = sublayer(X, p + "norm2", lambda hh: feed_forward(hh, W, p + "mlp.", L["mlp"], margins), p + "hc2")
        if collect is not None:
            collect.append(X.sum(0))
    return tanh_norm(X.sum(0), W, "final.norm") @ W["head"].T


def greedy(cfg, W, prompt, n_new):
    """The prompt's continuation, token by token, every time from the whole sequence."""
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(int(forward(cfg, W, seq)[-1].argmax()))
    return seq[len(prompt):]
