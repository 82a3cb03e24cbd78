"""The Mutirax architecture against the plain implementation of tests/plain_mutirax.py: every mechanism alone (the
kernels through their checked wrappers), then whole models built from folders that this file writes (its own small
configurations and weights), stepped through the engine in every way a request can arrive."""
import json
import math
import os

import pytest
import torch

import plain_mutirax as pm
from conftest import rel_err
from mutirax_cases import CONFIGS, _dense, _gla, _lat, _model, _moe, _par, settled_tokens, write_folder

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
# Bounds on the distance from the plain implementation (float64 from the same stored weights).  float32: the largest
# difference of any element over the reference's root mean square: summation order and the float32 functions.
# bfloat16: the design's norm has no statistics, so nothing brings a layer's input back to a fixed size and a rounding
# early in the model is carried, mixed between the streams and multiplied by slow decays to its end: measured layer by layer
# on these configurations, rows are 0.5 to 1.5 % of their root mean square off after the first layers and 3 to 7 % after the
# last, 17 % in the logits.  So a row's root-mean-square difference is bounded by 25 % and any element by the row's
# size; float32 is what pins the formulas.  A wrong key, a lost state, a sink left out or another expert moves rows by
# their own size.
TOL = {torch.float32: 3e-4, torch.bfloat16: 0.25}
BF16_ELEMENT = 1.0
DEV = "cuda:0"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = write_folder(tmp_path_factory.mktemp(f"mutirax{name}"), CONFIGS[name], 31 + len(made))
        return made[name]
    return get


_plain_cache = {}


def plain(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        _plain_cache[key] = pm.forward(pm.read_config(folder), pm.read_weights(folder), tokens)
    return _plain_cache[key]


def engine(folder, dtype, max_tokens=1024, **kw):
    import bitnet_c_amd as bn
    return bn.Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, **kw)


def close(got, want, dtype, bf16_rows=None):
    e = rel_err(got, want)
    if dtype == torch.float32:
        assert e < TOL[dtype], f"relative error {e}"
        return
    g, w = got.detach().double().cpu().reshape(-1, got.shape[-1]), want.detach().double().cpu().reshape(-1, want.shape[-1])
    rms = float(w.pow(2).mean().sqrt())
    rows = float((g - w).pow(2).mean(dim=-1).sqrt().max()) / max(rms, 1e-30)
    assert rows < (bf16_rows or TOL[dtype]) and e < (10 * bf16_rows if bf16_rows else BF16_ELEMENT), \
        f"a row is {rows} rms off, an element {e}"


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def f32(v):
    return v.to(torch.float32).to(DEV).contiguous()


def cut_steps(lens_per_seq):
    """Steps of a schedule: lens_per_seq[b] lists how many tokens sequence b brings in each step (0: none)."""
    return list(zip(*lens_per_seq))


# ------------------------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,D", [(1, 24), (2, 50), (3, 256), (8, 1100)])
def test_streams_are_read_rebuilt_and_normed_in_one_pass(dtype, n, D):
    """The residual as n streams: the first read takes the embedding's rows as every stream; a write is held back and
    rebuilds all streams at once from the old ones when the next read comes; the end sums the streams at chosen rows.  The
    output of a sublayer arrives in the activations' type or as float32 slabs."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.parts import NORMS, PartSpec
    from bitnet_c_amd.parts.hyper import HyperStream
    g = torch.Generator().manual_seed(n * 1000 + D)
    T, mult = 7, 0.3
    x0 = torch.randn(T, D, generator=g)
    norm = NORMS.build(PartSpec.of("dyt", dim=D))
    w, b, alpha = 1 + 0.3 * torch.randn(D, generator=g), 0.2 * torch.randn(D, generator=g), torch.tensor(0.6)
    norm.load({"weight": w, "bias": b, "alpha": alpha}, DEV, dtype)

    def tn(u):
        return torch.tanh(0.6 * u.double()) * w.double() + b.double()
    coef = [(torch.randn(n, generator=g), torch.randn(n, generator=g), torch.eye(n) + 0.5 * torch.randn(n, n, generator=g))
            for _ in range(3)]
    y1 = (2.0 * torch.randn(T, D, generator=g)).to(dtype)
    slabs = torch.randn(3, T, D, generator=g)
    stream = HyperStream(x0.to(DEV), n)
    X = torch.stack([x0.double()] * n)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    h = stream.read(f32(coef[0][0]), norm, dtype)
    assert h.dtype == dtype and rel_err(h, tn(torch.einsum("s,std->td", coef[0][0].double(), X))) < tol
    stream.write(y1.to(DEV), f32(coef[0][2]), f32(coef[0][1]), mult)
    X = torch.einsum("sr,std->rtd", coef[0][2].double(), X) + mult * coef[0][1].double()[:, None, None] * y1.double()[None]
    h = stream.read(f32(coef[1][0]), norm, dtype)
    assert stream.pending is None and rel_err(stream.lanes, X) < 1e-5
    assert rel_err(h, tn(torch.einsum("s,std->td", coef[1][0].double(), X))) < tol
    stream.write(ops.PartialSums(slabs.to(DEV)), f32(coef[1][2]), f32(coef[1][1]), mult)
    X = torch.einsum("sr,std->rtd", coef[1][2].double(), X) + mult * coef[1][1].double()[:, None, None] * slabs.double().sum(0)[None]
    rows = stream.normed(norm, dtype, rows=i32([5, 0, 5]))              # the model's end: pending still, a choice of rows
    assert rel_err(rows, tn(X.sum(0))[[5, 0, 5]]) < tol
    assert rel_err(stream.flush(), X.sum(0)) < 1e-5 and rel_err(stream.lanes, X) < 1e-5
    # the norm alone, on a residual of one stream that other code holds
    x = x0.to(DEV).clone()
    h = norm.apply(x, y1.to(DEV), dtype)
    assert rel_err(x, x0.double() + y1.double()) < 1e-6 and rel_err(h, tn(x0.double() + y1.double())) < tol
    assert rel_err(norm.apply(x, None, dtype, rows=i32([3])), tn(x0.double() + y1.double())[[3]]) < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,taps,bias", [(37, 4, True), (5, 1, False), (300, 2, False), (64, 7, True), (16, 16, False)])
def test_a_short_convolution_over_prompts_portions_and_single_tokens(dtype, C, taps, bias):
    """Three sequences through the same slots' state in steps of unequal portions (one token, two, more than the taps,
    fewer), then token by token, beside a padding row; against the convolution of each whole sequence.  The channels are
    a run of columns of a wider tensor; a slot's state row holds other values in front of the convolution's."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(C * 31 + taps)
    w = torch.randn(C, taps, generator=g)
    b = torch.randn(C, generator=g) if bias else None
    plan = [[5, 1, 2, 9, 1, 1], [1, 1, 1, 0, 3, 1], [0, 12, 0, 2, 0, 1]]       # tokens of sequence b in step i
    lens = [sum(p) for p in plan]
    col, width, lead = 3, C + 8, 6
    xs = [(torch.randn(n, width, generator=g)).to(dtype) for n in lens]
    want = [pm.short_convolution(x[:, col:col + C].double(), w.double(), None if b is None else b.double()) for x in xs]
    slots = [4, 0, 2]
    state = torch.full((6, lead + max(taps - 1, 1) * C), 9.0)                 # what former owners left
    for s in slots:
        state[s] = 0.0                                                        # a slot is handed out zeroed
    st = state.to(DEV)
    conv_state = st[:, lead:]
    done = [0, 0, 0]
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for step in cut_steps(plan):
        live = [bq for bq in range(3) if step[bq]]
        rows, pos, seq, tiles, r = [], [], [], [], 0
        for k, bq in enumerate(live):
            n = step[bq]
            rows.append(xs[bq][done[bq]:done[bq] + n])
            pos += list(range(done[bq], done[bq] + n))
            seq += [k] * n
            tiles.append([k, r, n, done[bq]])
            r += n
        x = torch.cat(rows).to(DEV)
        decode = all(step[bq] == 1 for bq in live)
        if decode:                                         # with a padding row at the end
            x = torch.cat([x, torch.zeros(1, width, dtype=dtype, device=DEV)])
            y = ops.short_conv(x, col, f32(w), None if b is None else f32(b), conv_state, i32(pos + [-1]), i32(seq + [0]),
                               i32([slots[bq] for bq in live] + [5]), seq_lens=i32([done[bq] + 1 for bq in live] + [0]))
            assert float(y[-1].abs().max()) == 0.0
            y = y[:-1]
        else:
            y = ops.short_conv(x, col, f32(w), None if b is None else f32(b), conv_state, i32(pos), i32(seq),
                               i32([slots[bq] for bq in live]), tiles=i32(tiles + [[0, 0, 0, 0]]))
        r = 0
        for bq in live:
            n = step[bq]
            assert rel_err(y[r:r + n], want[bq][done[bq]:done[bq] + n]) < tol, (step, bq)
            r += n
            done[bq] += n
    assert torch.equal(st[:, :lead].cpu(), state[:, :lead]) and torch.equal(st[[1, 3, 5]].cpu(), state[[1, 3, 5]])
    for bq in range(3):                                    # the state: the last taps - 1 inputs, oldest first
        if taps > 1:
            last = xs[bq][-(taps - 1):, col:col + C].float()
            have = conv_state[slots[bq], :(taps - 1) * C].view(taps - 1, C)[-last.shape[0]:]
            assert torch.equal(have.cpu(), last)


@pytest.mark.parametrize("W,blocks", [(48, 3), (35, 5), (64, 1), (320, 4), (600, 2)])
def test_the_gates_and_the_chain_of_the_recurrent_unit(W, blocks):
    """r, i, a and the unit's input in float32 from a float32 u, then S <- a S + b over a prompt step of three sequences
    (one continuing from a state), and one token each; channels whose decay is next to 1 and next to 0."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(W)
    bw = W // blocks
    ra, ri = torch.randn(blocks, bw, bw, generator=g) / math.sqrt(bw), torch.randn(blocks, bw, bw, generator=g) / math.sqrt(bw)
    ba, bi = torch.randn(W, generator=g), torch.randn(W, generator=g)
    lam = 2.0 * torch.randn(W, generator=g)
    lam[0], lam[1] = -12.0, 6.0                                # a next to 1 whatever r is, and a next to 0
    lens, first = [30 if W != 64 else 300, 1, 13], [4, 0, 0]      # one case with many rows
    slots = [3, 1, 0]
    state = torch.zeros(5, W + 2)
    state[1] = 5.0                                            # a former owner's: ignored at position 0
    us, ys, want = [], [], []
    c_neg = (-8.0 * pm.softplus(lam.double())).float()

    def gates(u):
        ub = u.double().view(-1, blocks, bw)
        r = pm.sigmoid(torch.einsum("boi,tbi->tbo", ra.double(), ub).reshape(-1, W) + ba.double())
        i = pm.sigmoid(torch.einsum("boi,tbi->tbo", ri.double(), ub).reshape(-1, W) + bi.double())
        a = torch.exp(-8.0 * r * pm.softplus(lam.double()))
        return a, torch.sqrt(1.0 - a * a) * i * u.double()
    for bq, (n, p0) in enumerate(zip(lens, first)):
        S = torch.zeros(W, dtype=torch.float64)
        if p0:
            S = torch.randn(W, generator=g).double()
            state[slots[bq], :W] = S.float()
            S = state[slots[bq], :W].double()
        u, y = torch.randn(n + 1, W, generator=g), torch.randn(n + 1, W, generator=g)
        a, b = gates(u)
        out = torch.zeros(n + 1, W, dtype=torch.float64)
        for t in range(n + 1):
            S = a[t] * S + b[t]
            out[t] = S * pm.gelu_tanh(y[t].double())
        us.append(u)
        ys.append(y)
        want.append(out)
    wa_t, wi_t = f32(ra.transpose(1, 2)), f32(ri.transpose(1, 2))
    u = torch.cat([x[:-1] for x in us])
    a_dev, b_dev = ops.lru_gates(f32(u), wa_t, f32(ba), wi_t, f32(bi), f32(c_neg))
    a_ref, b_ref = gates(u)
    assert rel_err(a_dev, a_ref) < 1e-5 and rel_err(b_dev, b_ref) < 1e-5
    assert float((1 - a_ref[:, 0]).max()) < 1e-3 and float(a_ref[:, 1].median()) < 1e-2       # both ends of the decay are met
    tiles, r = [], 0
    for bq, n in enumerate(lens):
        tiles.append([bq, r, n, first[bq]])
        r += n
    wide = torch.cat([torch.cat([x[:-1] for x in ys]), torch.zeros(r, 3)], dim=1).to(DEV)     # y: columns of a wider tensor
    for pieces in (True, False):                       # long prompts' form (pieces side by side), then the plain walk
        st = state.to(DEV)
        out = ops.lru_scan(a_dev, b_dev, wide[:, :W], st, i32(slots), tiles=i32(tiles), pieces=pieces)
        assert rel_err(out, torch.cat([x[:-1] for x in want])) < 2e-5, pieces
    ud = torch.stack([us[2][-1], us[0][-1], us[1][-1]])
    a_dev, b_dev = ops.lru_gates(f32(ud), wa_t, f32(ba), wi_t, f32(bi), f32(c_neg))
    yd = torch.stack([ys[2][-1], ys[0][-1], ys[1][-1]]).to(DEV)
    od = ops.lru_scan(a_dev, b_dev, yd, st, i32([slots[2], slots[0], slots[1]]), seq_lens=i32([lens[2] + 1, first[0] + lens[0] + 1, 2]))
    assert rel_err(od, torch.stack([want[2][-1], want[0][-1], want[1][-1]])) < 2e-5
    assert torch.equal(st[:, W:].cpu(), state[:, W:]) and torch.equal(st[[2, 4]].cpu(), state[[2, 4]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk,dv", [(3, 16, 24), (2, 10, 70), (1, 64, 64), (2, 130, 20), (1, 256, 16), (5, 1, 1), (6, 32, 64)])
def test_gated_linear_attention_over_prompts_portions_and_single_tokens(dtype, H, dk, dv):
    """The recurrence with a decay per key channel and token over a step of three sequences of unequal lengths (one
    continues from a state, one starts in a row that a former sequence left its state in), then one token each beside a
    padding row, against the recurrence written token by token; the projections are runs of columns of one tensor."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(dk * 7 + dv)
    tau = 3.0
    lens, first = ([37, 1, 70], [5, 0, 0]) if dk != 32 else ([201, 64, 130], [9, 0, 0])    # pieces: two; four, one whole, three
    qc, kc, vc, Wd = 3, 3 + H * dk + 2, 3 + 2 * H * dk + 4, 3 + 2 * H * dk + 4 + H * dv + 1
    slots = [4, 1, 2]
    state = torch.zeros(6, H * dk * dv + 3)
    state[1] = 7.0
    xs, zs, want, S_after = [], [], [], []

    def chain(x, z, S):
        x = x.double()
        q = x[:, qc:qc + H * dk].view(-1, H, dk) * dk ** -0.5
        k, v = x[:, kc:kc + H * dk].view(-1, H, dk), x[:, vc:vc + H * dv].view(-1, H, dv)
        al = (pm.sigmoid(z.double()) ** (1.0 / tau)).view(-1, H, dk)
        o = torch.zeros(x.shape[0], H, dv, dtype=torch.float64)
        for t in range(x.shape[0]):
            S = al[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        return o, S
    for bq, (n, p0) in enumerate(zip(lens, first)):
        S0 = torch.zeros(H, dk, dv, dtype=torch.float64)
        if p0:
            S0 = torch.randn(H, dk, dv, generator=g).float().double()
            state[slots[bq], :H * dk * dv] = S0.reshape(-1).float()
        x = (0.7 * torch.randn(n + 1, Wd, generator=g)).to(dtype)
        z = 3.0 * torch.randn(n + 1, H * dk, generator=g) + 2.0
        o, _ = chain(x, z, S0)
        _, S = chain(x[:-1], z[:-1], S0)
        xs.append(x)
        zs.append(z)
        want.append(o)
        S_after.append(S)
    st = state.to(DEV)
    tiles, r = [], 0
    for bq, n in enumerate(lens):
        tiles.append([bq, r, n, first[bq]])
        r += n
    tiles.append([0, 0, 0, 0])
    x, z = torch.cat([t[:-1] for t in xs]).to(DEV), f32(torch.cat([t[:-1] for t in zs]))
    tol = 2e-5
    for pieces in (True, False):                       # long prompts' form (pieces of 64 tokens side by side), then the plain walk
        st = state.to(DEV)
        o = ops.gla_scan(x, qc, kc, vc, z, st, i32(slots), H, dk, dv, dk ** -0.5, 1.0 / tau, tiles=i32(tiles), pieces=pieces)
        assert rel_err(o, torch.cat([w[:-1] for w in want]).reshape(sum(lens), -1)) < tol, pieces
        for bq in range(3):
            assert rel_err(st[slots[bq], :H * dk * dv], S_after[bq].reshape(-1)) < tol, pieces
        assert torch.equal(st[[0, 3, 5]].cpu(), state[[0, 3, 5]]) and torch.equal(st[:, H * dk * dv:].cpu(), state[:, H * dk * dv:])
    xd = torch.stack([xs[2][-1], xs[0][-1], torch.zeros(Wd, dtype=dtype), xs[1][-1]]).to(DEV)
    zd = f32(torch.stack([zs[2][-1], zs[0][-1], torch.zeros(H * dk), zs[1][-1]]))
    before = st.clone()
    od = ops.gla_scan(xd, qc, kc, vc, zd, st, i32([slots[2], slots[0], 5, slots[1]]), H, dk, dv, dk ** -0.5, 1.0 / tau,
                      seq_lens=i32([lens[2] + 1, first[0] + lens[0] + 1, 0, 2]))
    assert rel_err(od[[0, 1, 3]], torch.stack([want[2][-1], want[0][-1], want[1][-1]]).reshape(3, -1)) < tol
    assert torch.equal(st[5], before[5]) and torch.equal(st[0], before[0]) and torch.equal(st[:, H * dk * dv:], before[:, H * dk * dv:])


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_key_far_back_carries_the_result_where_its_channels_do_not_decay(dtype):
    """One key far back is made to stand out along one channel whose decay stays next to 1 in head 0 and falls fast in head
    1: 900 tokens later its value is what comes out of head 0 and is gone from head 1.  As a prompt, in portions, decoded."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(5)
    H, dk, dv, T, far, tau = 2, 32, 32, 1000, 100, 4.0
    x = 0.3 * torch.randn(T, 2 * H * dk + H * dv, generator=g)
    z = torch.randn(T, H * dk, generator=g)
    z[:, 0], z[:, dk] = 40.0, -1.0                            # channel 0 of head 0 keeps everything, of head 1 forgets
    for h in range(H):
        x[far, H * dk + h * dk] = 30.0
        x[T - 1, h * dk] = 30.0
    x[far, 2 * H * dk:] = 3.0
    x = x.to(dtype)
    xd = x.double()
    q, k, v = xd[:, :H * dk].view(T, H, dk) * dk ** -0.5, xd[:, H * dk:2 * H * dk].view(T, H, dk), xd[:, 2 * H * dk:].view(T, H, dv)
    al = (pm.sigmoid(z.double()) ** (1.0 / tau)).view(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=torch.float64)
    want = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        S = al[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        want[t] = torch.einsum("hdv,hd->hv", S, q[t])
    share = 900.0 * dk ** -0.5 * v[far, 0]
    assert float((want[-1, 0] - share).norm() / want[-1, 0].norm()) < 0.2
    assert float(want[-1, 1].norm()) < 0.05 * float(want[-1, 0].norm())
    for cut in (T, T - 1, 700):
        st = torch.zeros(2, H * dk * dv, dtype=torch.float32, device=DEV)
        o = ops.gla_scan(x[:cut].to(DEV), 0, H * dk, 2 * H * dk, f32(z[:cut]), st, i32([1]), H, dk, dv, dk ** -0.5, 1 / tau,
                         tiles=i32([[0, 0, cut, 0]]))
        parts = [o]
        for t in range(cut, T):
            parts.append(ops.gla_scan(x[t:t + 1].to(DEV), 0, H * dk, 2 * H * dk, f32(z[t:t + 1]), st, i32([1]), H, dk, dv,
                                      dk ** -0.5, 1 / tau, seq_lens=i32([t + 1])))
        got = torch.cat(parts)
        assert rel_err(got[-1], want[-1].reshape(-1)) < 1e-4 and rel_err(got[:-1], want[:-1].reshape(T - 1, -1)) < 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,hs", [(4, 2, 16), (6, 1, 8), (2, 2, 64), (4, 1, 128), (3, 3, 34)])
def test_a_learned_sink_in_the_softmax(dtype, H, G, hs):
    """Attention over pages with one more term exp(sink_h) in every head's denominator: sinks far below every score change
    nothing, a sink far above takes all the weight, and between the two the plain formula holds; in a prompt step (on the
    matrix cores where the sizes allow, else on the vector kernel) and decoded, with the keys in one run and split."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    g = torch.Generator().manual_seed(H * 10 + hs)
    T, scale = 150, 0.3
    q = torch.randn(T, H, hs, generator=g).to(dtype)
    k = torch.randn(T, G, hs, generator=g).to(dtype)
    sink = torch.randn(H, generator=g) * 2.0
    sink[0], sink[-1] = -80.0, 60.0
    want = torch.zeros(T, H, hs, dtype=torch.float64)
    for i in range(H):
        s = (q[:, i].double() @ k[:, i // (H // G)].double().T) * scale
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), -float("inf"))
        top = torch.maximum(s.max(dim=1).values, sink[i].double())
        e = torch.exp(s - top[:, None])
        want[:, i] = (e @ k[:, i // (H // G)].double()) / (e.sum(1) + torch.exp(sink[i].double() - top))[:, None]
    assert H == 1 or float(want[:, -1].abs().max()) < 1e-10           # the large sink takes everything
    n_pages = (T + PAGE - 1) // PAGE
    kp = torch.zeros(8, G, PAGE, hs, dtype=dtype, device=DEV)
    vp = torch.zeros(8, G, hs, PAGE, dtype=dtype, device=DEV)
    table = [5, 2, 7][:n_pages]
    for p in range(T):
        kp[table[p // PAGE], :, p % PAGE] = k[p].to(DEV)
        vp[table[p // PAGE], :, :, p % PAGE] = k[p].to(DEV)
    bt = i32([table + [0] * (4 - n_pages)])
    qd = q.reshape(T, H * hs).to(DEV)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    from bitnet_c_amd.engine.step import _query_tiles
    forms = [False] + ([True] if ops.attention_general_supported(dtype, hs, hs) else [])
    for mfma in forms:
        out = torch.empty(T, H * hs, dtype=dtype, device=DEV)
        if mfma:
            tiles = i32(_query_tiles([T], [0], ops.GENERAL_PROMPT_TILE)).reshape(-1, 4)
            ops.attention_general_prompt(qd, out, kp, vp, bt, H, G, hs, hs, scale, tiles, sink=f32(sink))
        else:
            _, _, qt = ops.attention_row_shape(H, G, False)
            tiles = i32(_query_tiles([T], [0], qt)).reshape(-1, 4)
            ops.attention(qd, out, kp, vp, bt, H, G, hs, scale, tiles=tiles, qt=qt, v_transposed=True, blocked=False, v_dim=hs,
                          sink=f32(sink))
        assert rel_err(out, want.reshape(T, -1)) < tol, mfma
        for n_splits in ((1, 2) if dtype == torch.bfloat16 else (1,)):       # a float32 cache's keys are cut in fixed runs
            chunk = 2 * PAGE if n_splits > 1 else 0
            out = torch.empty(1, H * hs, dtype=dtype, device=DEV)
            if mfma:
                ops.attention_general_decode(qd[-1:], out, kp, vp, bt, i32([T]), H, G, hs, hs, scale, n_splits=n_splits, chunk=chunk,
                                             sink=f32(sink))
            else:
                ops.attention(qd[-1:], out, kp, vp, bt, H, G, hs, scale, seq_lens=i32([T]), n_splits=n_splits, chunk=chunk,
                              v_transposed=True, blocked=False, v_dim=hs, sink=f32(sink))
            assert rel_err(out, want[-1:].reshape(1, -1)) < tol, (mfma, n_splits)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,rot,scaled", [(40, 8, True), (14, 2, False), (96, 32, True), (8, 0, False), (64, 64, True)])
def test_the_latent_and_its_rotated_part_in_the_pages(dtype, R, rot, scaled):
    """The latent under its norm as a key row and in the transposed value page; behind it in the key row the rotated part,
    not normed, turned by frequencies whose rescaling meets both ends of its ramp; the same rotation in place on the tail of
    every query head."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    from bitnet_c_amd.parts.position import rope_frequencies, rope_magnitude
    g = torch.Generator().manual_seed(R + rot)
    eps, col = 1e-5, 5
    rd = dict(base=5000.0, dims=rot)
    scaling = None
    if scaled:
        rd["scaling"] = dict(factor=4.0, original=64, fast=8.0, slow=1.0)
        scaling = dict(rope_type="yarn", **rd["scaling"])
    pos = [0, 1, 63, 64, 300, -1, 2047]
    T = len(pos)
    x = torch.randn(T, col + R + rot + 2, generator=g).to(dtype)
    w = 1 + 0.2 * torch.randn(R, generator=g)
    inv, mult = None, 1.0
    if rot:
        inv, mult = rope_frequencies(rot, rd["base"], scaling).to(DEV), rope_magnitude(scaling)
        f_ref, m_ref = pm.rotary_table(rd)
        assert rel_err(inv, f_ref) < 1e-6 and abs(mult - m_ref) < 1e-12
        if scaled and rot >= 32:
            plain_f = torch.tensor([rd["base"] ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64)
            ratio = f_ref / plain_f
            assert float(ratio.max()) == 1.0 and abs(float(ratio.min()) - 0.25) < 1e-12 and bool(((ratio > 0.26) & (ratio < 0.99)).any())
    kp = torch.zeros(40, 1, PAGE, R + rot, dtype=dtype, device=DEV)
    vp = torch.zeros(40, 1, R, PAGE, dtype=dtype, device=DEV)
    table = i32([[(7 * j + 3) % 40 for j in range(33)]])
    ops.latent_store(x.to(DEV), col, R, f32(w), eps, i32(pos), i32([0] * T), table, kp, vp, rot_dims=rot, inv_freq=inv, rot_mult=mult)
    live = [t for t, p in enumerate(pos) if p >= 0]
    c = pm.unit_rms(x[:, col:col + R].double(), eps) * w.double()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    kr = None
    if rot:
        kr = pm.rotate_halves(x[live, col + R:col + R + rot].double().view(len(live), 1, rot), [pos[t] for t in live], rd)[:, 0]
    for n, t in enumerate(live):
        page, at = int(table[0, pos[t] // PAGE]), pos[t] % PAGE
        assert rel_err(kp[page, 0, at, :R], c[t]) < tol and rel_err(vp[page, 0, :, at], c[t]) < tol
        if rot:
            assert rel_err(kp[page, 0, at, R:], kr[n]) < (5e-4 if dtype == torch.float32 else tol)     # angles are float32
    if rot:
        H, off = 3, R
        q = torch.randn(T, H * (R + rot) + 1, generator=g).to(dtype)
        qd = q.to(DEV).clone()
        ops.rope_heads(qd, i32(pos), inv, H, R + rot, off, rot, mult)
        heads = q[:, :H * (R + rot)].double().view(T, H, R + rot)
        turned = pm.rotate_halves(heads[live][..., off:], [pos[t] for t in live], rd)
        got = qd[:, :H * (R + rot)].view(T, H, R + rot)
        assert rel_err(got[live][..., off:], turned) < (5e-4 if dtype == torch.float32 else tol)
        assert torch.equal(got[..., :off].cpu(), heads[..., :off].to(dtype)) and torch.equal(qd[5].cpu(), q[5])


@pytest.mark.parametrize("H,G,hs", [(6, 1, 8), (16, 4, 64), (5, 5, 34)])
def test_a_norm_over_the_whole_projection_reads_it_before_any_head_is_rewritten(H, G, hs):
    """The queries are rewritten in place, and the norm over the whole query projection needs all of them as they arrived:
    with more heads than one workgroup's waves take at once, many rows, again and again, every result is the plain one; the
    values are the keys as they arrived."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    g = torch.Generator().manual_seed(H + hs)
    T, eps = 128, 1e-5
    qk = torch.randn(T, (H + G) * hs, generator=g)
    wq, wk = 1 + 0.2 * torch.randn(H * hs, generator=g), 1 + 0.2 * torch.randn(G * hs, generator=g)
    rot = dict(base=100.0, dims=hs // 2 * 2)
    from bitnet_c_amd.parts.position import rope_frequencies
    inv = rope_frequencies(rot["dims"], rot["base"]).to(DEV)
    q = pm.rotate_halves((pm.unit_rms(qk[:, :H * hs].double(), eps) * wq.double()).view(T, H, hs), range(T), rot)
    kp = torch.zeros(2, G, PAGE, hs, device=DEV)
    vp = torch.zeros(2, G, hs, PAGE, device=DEV)
    for _ in range(30):
        x = qk.to(DEV).clone()
        ops.qk_norm_store(x, i32(list(range(T))), H, G, hs, q_weight=f32(wq), k_weight=f32(wk), eps=eps, seq_index=i32([0] * T),
                          block_table=i32([[1, 0]]), k_pages=kp, v_pages=vp, v_transposed=True, inv_freq=inv, rope_dims=rot["dims"],
                          norm_projection=True, v_from_k=True)
        assert rel_err(x[:, :H * hs], q.reshape(T, -1)) < 2e-4
        assert torch.equal(vp[0, :, :, 5].cpu(), qk[PAGE + 5, H * hs:].view(G, hs))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [1, 5, 40])
def test_a_product_per_head_with_one_gate_number_per_head(dtype, T):
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(T)
    H, I, O = 3, 20, 24
    x = torch.randn(T, H * I, generator=g).to(dtype)
    w = (torch.randn(H, I, O, generator=g) / math.sqrt(I)).to(dtype)
    wide = torch.randn(T, 7 + H, generator=g).to(dtype)
    want = torch.einsum("thi,hio->tho", x.double().view(T, H, I), w.double()) * pm.sigmoid(wide[:, 7:].double())[:, :, None]
    got = ops.head_linear(x.to(DEV), w.to(DEV), wide.to(DEV)[:, 7:], gate_per_head=True)
    assert rel_err(got, want.reshape(T, -1)) < (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,K,D,T", [(6, 2, 64, 5), (3, 3, 48, 40), (1, 1, 32, 3), (70, 5, 40, 20)])
def test_a_router_with_a_bias_weighs_by_the_chosen_logits_alone(dtype, E, K, D, T):
    """The logits with their bias choose; the weights are the softmax over the chosen logits alone.  Then the experts as
    silu-gated units without bounds, a pair at a time and (many rows, bfloat16) as grouped products."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(E * 100 + D)
    F = 24
    h = torch.randn(T, D, generator=g).to(dtype)
    router, bias = 3.0 * torch.randn(E, D, generator=g) / math.sqrt(D), 2.0 * torch.randn(E, generator=g)
    z = h.double() @ router.double().T + bias.double()
    ids, wts = ops.moe_route(h.to(DEV), f32(router), K, "softmax", True, logit_bias=f32(bias))
    plain_pick = torch.topk(z - bias.double(), K).indices
    changed = 0
    for t in range(T):
        val, idx = torch.topk(z[t], K)
        gap = float(val[-1] - torch.topk(z[t], min(K + 1, E)).values[-1]) if K < E else 1.0
        if gap < 1e-3:
            continue
        assert ids[t].tolist() == idx.tolist()
        assert rel_err(wts[t], torch.softmax(val, dim=-1)) < 1e-5
        changed += set(idx.tolist()) != set(plain_pick[t].tolist())
    assert changed > 0 or E == K                             # the bias changes some choices
    w_gate, w_up = (2.0 * torch.randn(E, F, D, generator=g) / math.sqrt(D)).to(dtype), (torch.randn(E, F, D, generator=g) / math.sqrt(D)).to(dtype)
    w_down = (torch.randn(E, D, F, generator=g) / math.sqrt(F)).to(dtype)
    want = torch.zeros(T, D, dtype=torch.float64)
    for t in range(T):
        for j in range(K):
            e = int(ids[t, j])
            hid = pm.silu(w_gate[e].double() @ h[t].double()) * (w_up[e].double() @ h[t].double())
            want[t] += float(wts[t, j]) * (w_down[e].double() @ hid)
    unit = ops.ClampedUnit(float("inf"), 1.0, 0.0)
    stacked = torch.cat([w_gate, w_up], dim=1).contiguous().to(DEV)
    y = ops.moe_experts(h.to(DEV), stacked, w_down.to(DEV), ids, wts, "silu", False, gated=unit)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert rel_err(y.slabs.sum(0), want) < tol
    if ops.moe_grouped_supported(T, D, F, dtype):
        y = ops.moe_experts_grouped(h.to(DEV), stacked, w_down.to(DEV), ids, wts, "silu", False, gated=unit)
        assert rel_err(y.slabs.sum(0), want) < tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_dense_unit_bounds_its_arguments(dtype):
    from bitnet_c_amd.parts import FEED_FORWARDS, PartSpec
    g = torch.Generator().manual_seed(8)
    D, F, T, limit = 48, 72, 9, 0.8
    W = {"gate": (3.0 * torch.randn(F, D, generator=g) / math.sqrt(D)).to(dtype).double(),
         "up": (3.0 * torch.randn(F, D, generator=g) / math.sqrt(D)).to(dtype).double(),
         "down": (torch.randn(D, F, generator=g) / math.sqrt(F)).to(dtype).double()}
    h = torch.randn(T, D, generator=g).to(dtype)
    assert float((h.double() @ W["gate"].T).abs().max()) > 2 * limit            # the bounds are met
    ff = FEED_FORWARDS.build(PartSpec.of("gated_clamped", hidden=D, intermediate=F, limit=limit))
    ff.load({"w_gate": W["gate"], "w_up": W["up"], "w_down": W["down"]}, DEV, dtype)
    got = ff.forward(h.to(DEV), None)
    assert rel_err(got, pm.dense_unit(h.double(), W, "", dict(limit=limit))) < (1e-5 if dtype == torch.float32 else 3e-2)


# ------------------------------------------------------------------------------------------------------------------
# whole models through the engine
# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts_and_decoding_follow_the_plain_implementation(folders, name, dtype):
    """Every position of a prompt in one step; then the same sequence as a shorter prompt and token by token, across a
    page's border; the first tokens of a sequence are among them."""
    import bitnet_c_amd as bn
    folder = folders(name)
    toks = settled_tokens(folder, 75, 1)
    want = plain(folder, toks)
    eng = engine(folder, dtype)
    s = eng.new_sequence()
    whole = eng.step([bn.StepEntry(s, toks, list(range(75)))])
    close(whole, want, dtype)
    eng.release(s)
    s = eng.new_sequence()                               # the slot that was just given back
    first = eng.step([bn.StepEntry(s, toks[:58], list(range(58)))])
    dec = torch.cat([eng.step([bn.StepEntry(s, [t], [0])]) for t in toks[58:]])
    got = torch.cat([first, dec])
    close(got, want, dtype)
    if dtype == torch.float32:
        assert rel_err(got, whole) < 2e-5
    one = eng.new_sequence()                             # a sequence of one token, and one decoded from its first token on
    close(eng.step([bn.StepEntry(one, toks[:1], [0])]), want[:1], dtype)
    close(torch.cat([eng.step([bn.StepEntry(one, [t], [0])]) for t in toks[1:6]]), want[1:6], dtype)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,portions", [("A", (2, 3, 5, 2, 17, 1, 40, 2)), ("B", (1, 2, 2, 2, 64, 1)), ("C", (63, 2, 64, 3)),
                                           ("E", (2,) * 12)])
def test_prompts_in_portions_down_to_two_tokens(folders, name, portions, dtype):
    import bitnet_c_amd as bn
    folder = folders(name)
    n = sum(portions)
    toks = settled_tokens(folder, n, 2)
    want = plain(folder, toks)
    eng = engine(folder, dtype)
    s, at, parts = eng.new_sequence(), 0, []
    for p in portions:
        parts.append(eng.step([bn.StepEntry(s, toks[at:at + p], list(range(p)))]))
        at += p
    close(torch.cat(parts), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_batches_of_unequal_requests_and_slots_used_again(folders, name, dtype):
    """Requests of unequal lengths start together and are decoded together; the shorter ones end, their slots and pages
    go to new requests while a neighbour lives on; every request against itself alone (the plain implementation)."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype, max_tokens=768)
    keep = eng.new_sequence()
    eng.step([bn.StepEntry(keep, settled_tokens(folder, 9, 1), [])])
    for i in range(4):
        reqs = [settled_tokens(folder, n, 2 + (i + k) % 4) for k, n in enumerate((70 + i, 20 - i, 1 + 2 * i))]
        slots = [eng.new_sequence() for _ in reqs]
        out = eng.step([bn.StepEntry(s, r[:max(1, len(r) - 3)], [0, max(1, len(r) - 3) - 1]) for s, r in zip(slots, reqs)])
        for k, r in enumerate(reqs):
            want = plain(folder, r)
            head = max(1, len(r) - 3)
            close(out[2 * k:2 * k + 2], want[[0, head - 1]], dtype)
        live = [(s, r, max(1, len(r) - 3)) for s, r in zip(slots, reqs)]
        while any(at < len(r) for _, r, at in live):
            now = [(s, r, at) for s, r, at in live if at < len(r)]
            o = eng.step([bn.StepEntry(s, [r[at]], [0]) for s, r, at in now])
            for k, (s, r, at) in enumerate(now):
                close(o[k:k + 1], plain(folder, r)[at:at + 1], dtype)
            live = [(s, r, at + 1 if at < len(r) else at) for s, r, at in live]
        for s in slots[i % 2:]:
            eng.release(s)
    close(eng.step([bn.StepEntry(keep, [3], [0])]), plain(folder, settled_tokens(folder, 9, 1) + [3])[-1:], dtype)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_that_mixes_single_tokens_and_portions(folders, dtype):
    import bitnet_c_amd as bn
    folder = folders("A")
    eng = engine(folder, dtype)
    a, b, c = (settled_tokens(folder, n, 2 + i) for i, n in enumerate((30, 90, 12)))
    sa, sb, sc = (eng.new_sequence() for _ in range(3))
    eng.step([bn.StepEntry(sa, a[:29], []), bn.StepEntry(sb, b[:10], [])])
    out = eng.step([bn.StepEntry(sa, a[29:], [0]), bn.StepEntry(sb, b[10:], [0, 79]), bn.StepEntry(sc, c, [11])])
    want = torch.stack([plain(folder, a)[29], plain(folder, b)[10], plain(folder, b)[89], plain(folder, c)[11]])
    close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_with_far_keys_and_slow_decays(tmp_path, dtype):
    """A model whose attention is peaked (large scales: single far keys carry a query's result, and where none does the
    sink takes the weight) and whose decays stay next to 1: a prompt of many pages in portions, then 70 decoded tokens."""
    import bitnet_c_amd as bn
    cfg = _model(61, 32, 1e-5, 0.5, [
        _par(2, 1, 8, 3, 1.5, (10000.0, 4), 16, 2, 3, _dense(48, 1.0)),
        _gla(2, 8, 8, 32.0, None, rank=2),
        _lat(2, 8, 4, 8, 12, 6, 1.2, (1000.0, 4.0, 256, 16.0, 1.0), None)], streams=2, loop=(0, 2, 2))
    folder = write_folder(tmp_path / "peaked", cfg, 9)
    toks = torch.randint(0, 61, (700,), generator=torch.Generator().manual_seed(2)).tolist()     # no experts: no close calls
    want = plain(folder, toks)
    eng = engine(folder, dtype, max_tokens=2048)
    s, at, parts = eng.new_sequence(), 0, []
    check = [0, 1, 2, 3, 15, 16, 17, 63, 64, 65, 299, 300, 301, 511, 512, 629]
    for n in (300, 257, 73):
        w = [p - at for p in check if at <= p < at + n]
        parts.append(eng.step([bn.StepEntry(s, toks[at:at + n], w)]))
        at += n
    close(torch.cat(parts), want[check], dtype, bf16_rows=0.2)
    dec = torch.cat([eng.step([bn.StepEntry(s, [toks[t]], [0])]) for t in range(at, 700)])
    close(dec, want[at:], dtype, bf16_rows=0.2)
    s2 = eng.new_sequence()
    whole = eng.step([bn.StepEntry(s2, toks, list(range(at, 700)))])
    assert rel_err(dec, whole) < (1e-4 if dtype == torch.float32 else 1.0)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_convolution_sees_exactly_its_taps(tmp_path, dtype):
    """Convolutions whose oldest tap carries all the weight: a token's query, key and recurrent input are the projections
    of the token taps - 1 places back and nothing nearer or further.  Prompts, portions that end inside the taps, decoding."""
    import bitnet_c_amd as bn
    cfg = _model(47, 32, 1e-5, 1.0, [_par(2, 1, 8, 4, 0.4, (100.0, 8), 16, 2, 3, None)], streams=2)
    ov = {}
    for name, C, taps in (("l0.mix.left.q.conv", 16, 4), ("l0.mix.left.k.conv", 8, 4), ("l0.mix.right.conv", 16, 3)):
        w = torch.zeros(C, taps)
        w[:, 0] = 1.5
        ov[name] = w
    folder = write_folder(tmp_path / "taps", cfg, 3, overrides=ov)
    toks = torch.randint(0, 47, (40,), generator=torch.Generator().manual_seed(1)).tolist()
    want = plain(folder, toks)
    eng = engine(folder, dtype)
    s, at, parts = eng.new_sequence(), 0, []
    for p in (1, 1, 2, 1, 3, 5, 2, 25):
        parts.append(eng.step([bn.StepEntry(s, toks[at:at + p], list(range(p)))]))
        at += p
    close(torch.cat(parts), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_wide_latent_beside_its_rotated_part(tmp_path, dtype):
    """A latent of 192 numbers beside 64 rotated ones: key rows of 256, values of 192, the widths at which the prompt and
    decode steps of the latent mixer run on the matrix cores in bfloat16.  A prompt across a page's border, then decoded."""
    import bitnet_c_amd as bn
    cfg = _model(59, 64, 1e-5, 0.5, [_lat(3, 16, 64, 24, 192, 40, 0.11, (100000.0, 4.0, 2048, 16.0, 2.0), None)], streams=2)
    folder = write_folder(tmp_path / "wide", cfg, 6)
    toks = torch.randint(0, 59, (90,), generator=torch.Generator().manual_seed(4)).tolist()
    want = plain(folder, toks)
    eng = engine(folder, dtype)
    s = eng.new_sequence()
    got = eng.step([bn.StepEntry(s, toks[:70], list(range(70)))])
    dec = torch.cat([eng.step([bn.StepEntry(s, [t], [0])]) for t in toks[70:]])
    close(torch.cat([got, dec]), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_do_not_depend_on_the_cut_or_the_batch(folders, dtype):
    """Whole, in portions, one by one and beside other requests: float32 logits agree to the last bits, bfloat16 within
    its rounding (steps of few rows and of many take different kernels for the products and the experts)."""
    import bitnet_c_amd as bn
    folder = folders("C")
    eng = engine(folder, dtype)
    toks, other = settled_tokens(folder, 100, 1), settled_tokens(folder, 37, 3)
    s = eng.new_sequence()
    whole = eng.step([bn.StepEntry(s, toks, list(range(100)))])
    eng.release(s)
    s, o = eng.new_sequence(), eng.new_sequence()
    a = eng.step([bn.StepEntry(o, other, []), bn.StepEntry(s, toks[:37], list(range(37)))])
    b = eng.step([bn.StepEntry(s, toks[37:99], list(range(62)))])
    c = eng.step([bn.StepEntry(s, toks[99:], [0]), bn.StepEntry(o, [5], [])])
    got = torch.cat([a, b, c])
    if dtype == torch.float32:
        assert rel_err(got, whole) < 2e-5
    else:
        close(got, whole.double(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    """Greedy generation through load() and generate(), the scheduler batching three prompts two at a time.  Every token
    that was chosen holds, where it was chosen, the plain implementation's largest logit within rounding (up to the first
    close expert choice of the sequence that the engine itself wrote)."""
    import bitnet_c_amd as bn
    folder = folders(name)
    llm = bn.load(folder, dtype="float32" if dtype == torch.float32 else "bfloat16", max_tokens=1024)
    prompts = [settled_tokens(folder, n, 2 + i) for i, n in enumerate((5, 66, 1))]
    got = llm.generate(prompts, max_new_tokens=12, temperature=0.0, stop_ids=(), batch_size=2)
    cfg, W = pm.read_config(folder), pm.read_weights(folder)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        margins = []
        logits = pm.forward(cfg, W, p + g, margins=margins)[len(p) - 1:-1]
        settled = 0
        while settled < 12 and margins[len(p) + settled - 1] >= (1e-3 if dtype == torch.float32 else 0.05):
            settled += 1
        rms = float(logits.pow(2).mean().sqrt())
        for i, tok in enumerate(g[:settled]):
            gap = float(logits[i].max() - logits[i, tok])
            # bfloat16: an element of a row may be off by as much as BF16_ELEMENT of the rows' size (see TOL), on either token
            assert gap <= (1e-4 if dtype == torch.float32 else BF16_ELEMENT) * rms, (i, gap / rms)
    llm.engine.cache.check()
    assert llm.engine.cache.live_slots() == []


def test_command_line_and_trace_replay(folders, tmp_path):
    """The command line generates from a Mutirax folder (also one that it writes itself from a configuration file, with
    random weights), and the trace replay program steps one through a batch of prompts and single tokens."""
    import subprocess
    import sys
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = folders("D")
    cfg, W = pm.read_config(folder), pm.read_weights(folder)
    prompt = settled_tokens(folder, 8, 1)
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "bitnet"), folder, "--prompt-token-ids", ",".join(map(str, prompt)),
                        "-n", "6", "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--quiet"], capture_output=True, text=True,
                       timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    ids = [int(x) for x in [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0].split(",")]
    margins = []
    logits = pm.forward(cfg, W, prompt + ids, margins=margins)[len(prompt) - 1:-1]
    for i, tok in enumerate(ids):
        if min(margins[:len(prompt) + i]) < 1e-3:
            break
        assert float(logits[i].max() - logits[i, tok]) <= 1e-4 * float(logits.pow(2).mean().sqrt())
    conf = tmp_path / "conf.json"
    conf.write_text(json.dumps(CONFIGS["B"]))
    made = str(tmp_path / "made")
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "bitnet"), made, "--random", str(conf), "--seed", "4",
                        "--prompt-token-ids", "1,2,3", "-n", "4", "--fp32", "--token-ids", "--quiet", "--repeat-penalty", "1.0"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    assert len([l for l in p.stderr.splitlines() if l and l[0].isdigit()][0].split(",")) == 4
    assert pm.read_config(made)["loop"] == CONFIGS["B"]["loop"] and pm.read_config(made)["streams"] == CONFIGS["B"]["streams"]
    folder = folders("A")
    a, b = settled_tokens(folder, 40, 2), settled_tokens(folder, 7, 3)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:37], "want": [0, 29, 36]}, {"id": "b", "tokens": b[:5], "want": [4]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[37:38], "want": [0]}, {"id": "b", "tokens": b[5:6], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[38:39], "want": []}, {"id": "b", "tokens": b[6:], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[39:], "want": [0]}], "end": ["a"]}]
    for dtype, name in ((torch.float32, "float32"), (torch.bfloat16, "bfloat16")):
        out = tmp_path / ("out_" + name)
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", name,
                            "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                           capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-1500:]
        assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
        assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "2.f32", "3.f32"]
        la, lb = plain(folder, a), plain(folder, b)
        want_rows = {0: torch.stack([la[0], la[29], la[36], lb[4]]), 1: la[37:38], 2: lb[6:7], 3: la[39:40]}
        for i, w in want_rows.items():
            got = torch.from_numpy(np.fromfile(str(out / f"{i}.f32"), dtype="<f4").reshape(-1, CONFIGS["A"]["vocab"]))
            close(got, w, dtype)
