"""The Fazopel architecture against the plain implementation of tests/plain_fazopel.py: every mechanism alone (the
kernels through their checked wrappers), then whole models built from folders that this file writes (its own small
configurations and weights), stepped through the engine in every way a request can arrive."""
import json
import math
import os

import pytest
import torch

import plain_fazopel as pf
from conftest import rel_err
from fazopel_cases import CONFIGS, _att, _dense, _lin, _moe, settled_tokens, write_folder

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
# Bounds on the distance from the plain implementation (float64 from the same stored weights).  float32: the largest
# difference of any element over the reference's root mean square: summation order and the float32 functions.
# bfloat16: every half of a layer is normed behind itself, so its relative error joins the stream at full size, whatever
# the half's own size was; rounding nothing but the inputs of the halves to 8 bits (the plain implementation with
# round_to) already leaves rows 2.4 to 4.5 % of their root mean square off in these configurations, and an engine that
# also rounds every product's result measures 2.6 to 10.5 % (the small head sizes most).  So a row's root-mean-square
# difference is bounded by 15 % and any element by 60 %; float32 is what pins the formulas.  A wrong key, a lost state,
# a sink left out or another expert moves rows by their own size.
TOL = {torch.float32: 2e-4, torch.bfloat16: 0.15}
BF16_ELEMENT = 0.6
DEV = "cuda:0"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """One folder a configuration, weights stored in bfloat16: engines of both types and the plain implementation read
    the same numbers."""
    made = {}

    def get(name):
        if name not in made:
            made[name] = write_folder(tmp_path_factory.mktemp(f"fazopel{name}"), CONFIGS[name], 21 + len(made))
        return made[name]
    return get


_plain_cache = {}


def plain(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        _plain_cache[key] = pf.forward(pf.read_config(folder), pf.read_weights(folder), tokens)
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


# ------------------------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [24, 256, 2500])
def test_a_part_reads_the_stream_itself(dtype, D):
    """No norm in front of a part: the stream's rows in the activations' type, alone, behind a plain output, and in one
    pass with a held-back output that has a norm of its own (a tensor or float32 slabs)."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.parts import NORMS, NormedDelta, PartSpec, ResidualStream
    g = torch.Generator().manual_seed(D)
    T, eps_b = 7, 1e-5
    x0 = torch.randn(T, D, generator=g)
    d = (3.0 * torch.randn(T, D, generator=g)).to(dtype)
    slabs = torch.randn(3, T, D, generator=g)
    wb = 1 + 0.3 * torch.randn(D, generator=g)
    none = NORMS.build(PartSpec.of("none", dim=D))
    out_norm = NORMS.build(PartSpec.of("rmsnorm", dim=D, eps=eps_b))
    out_norm.load({"weight": wb}, DEV, dtype)
    h = ops.stream_rows(x0.to(DEV), dtype)
    assert h.dtype == dtype and torch.equal(h.cpu(), x0.to(dtype))
    stream = ResidualStream(x0.to(DEV).clone())
    stream.add(d.to(DEV))
    h = stream.normed(none, dtype)
    assert stream.pending is None and rel_err(stream.x, x0.double() + d.double()) < 1e-6
    assert torch.equal(h.float(), stream.x.to(dtype).float())
    rows = stream.normed(none, dtype, rows=i32([5, 0]))
    assert torch.equal(rows, h[[5, 0]])
    for delta, dd in ((d.to(DEV), d.double()), (ops.PartialSums(slabs.to(DEV)), slabs.double().sum(0))):
        want_x = x0.double() + pf.unit_rms(dd, eps_b) * wb.double()
        stream = ResidualStream(x0.to(DEV).clone())
        stream.add(NormedDelta(delta, out_norm))
        h = stream.normed(none, dtype)
        assert stream.pending is None and h.dtype == dtype and rel_err(stream.x, want_x) < 1e-5
        assert torch.equal(h.float(), stream.x.to(dtype).float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,hs,rd,scaled", [(4, 2, 16, 8, True), (6, 1, 8, 2, False), (2, 2, 64, 64, True), (3, 1, 130, 128, False),
                                              (1, 1, 256, 0, False)])
def test_head_norms_rotation_and_values_that_are_the_keys(dtype, H, G, hs, rd, scaled):
    """An RMSNorm over every query and key head, the rotation in split-half pairs with stretched long wavelengths, the
    keys at their places in the pages, and the values: the key projections as they arrived, before norm and rotation."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    from bitnet_c_amd.parts.position import rope_frequencies
    g = torch.Generator().manual_seed(H * 100 + hs)
    eps = 1e-5
    rot = dict(base=700.0, dims=rd)
    if scaled:
        rot["scaling"] = dict(factor=4.0, low=1.0, high=4.0, original=40)
    pos = [0, 1, 63, 64, 300, -1, 2047]
    T = len(pos)
    qk = torch.randn(T, (H + G) * hs, generator=g).to(dtype)
    wq, wk = 1 + 0.2 * torch.randn(hs, generator=g), 1 + 0.2 * torch.randn(hs, generator=g)
    inv = None
    if rd:
        sc = rot.get("scaling")
        inv = rope_frequencies(rd, rot["base"], dict(rope_type="llama3", factor=sc["factor"], low_freq_factor=sc["low"],
                                                     high_freq_factor=sc["high"], original_max_position_embeddings=sc["original"])
                               if sc else None).to(DEV)
        assert rel_err(inv, pf.rotary_frequencies(rot)) < 1e-6
        if scaled and rd >= 8:            # all three bands are met: kept, in between, stretched
            plain_f = torch.tensor([rot["base"] ** (-2.0 * i / rd) for i in range(rd // 2)], dtype=torch.float64)
            ratio = pf.rotary_frequencies(rot) / plain_f
            assert float(ratio.max()) == 1.0 and abs(float(ratio.min()) - 0.25) < 1e-12 and bool(((ratio > 0.26) & (ratio < 0.99)).any())
    live = [t for t, p in enumerate(pos) if p >= 0]
    q = (pf.unit_rms(qk[:, :H * hs].double().view(T, H, hs), eps) * wq.double())[live]
    kraw = qk[:, H * hs:].double().view(T, G, hs)[live]
    k = pf.unit_rms(kraw, eps) * wk.double()
    if rd:
        q = pf.rotate_halves(q, [pos[t] for t in live], rot, angle_dtype=torch.float32)
        k = pf.rotate_halves(k, [pos[t] for t in live], rot, angle_dtype=torch.float32)
    kp = torch.zeros(40, G, PAGE, hs, dtype=dtype, device=DEV)
    vp = torch.zeros(40, G, hs, PAGE, dtype=dtype, device=DEV)
    table = i32([[(7 * j + 3) % 40 for j in range(33)]])
    x = qk.to(DEV).clone()
    ops.qk_norm_store(x, i32(pos), H, G, hs, q_weight=wq.to(DEV), k_weight=wk.to(DEV), eps=eps, seq_index=i32([0] * T),
                      block_table=table, k_pages=kp, v_pages=vp, v_transposed=True, inv_freq=inv, rope_dims=rd, v_from_k=True)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert rel_err(x[live, :H * hs], q.reshape(len(live), -1)) < tol
    assert torch.equal(x[:, H * hs:].cpu(), qk[:, H * hs:])                  # the key columns are left as they arrived
    assert torch.equal(x[5].cpu(), qk[5])                                    # and so is a padding row
    for n, t in enumerate(live):
        page, at = int(table[0, pos[t] // PAGE]), pos[t] % PAGE
        assert rel_err(kp[page, :, at], k[n]) < tol
        assert torch.equal(vp[page, :, :, at].cpu(), qk[t, H * hs:].view(G, hs))       # the values: the keys as projected


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chain", [False, True])
@pytest.mark.parametrize("H,dk,dv", [(3, 16, 24), (2, 10, 70), (1, 64, 64), (2, 128, 130), (1, 200, 8), (5, 1, 1)])
def test_the_decayed_sums_over_prompts_portions_and_single_tokens(dtype, H, dk, dv, chain):
    """The recurrence over a step of three sequences of unequal lengths (one continues from a state, one starts in a row
    that a former sequence left its state in), then one token each, against the recurrence written token by token; the
    projections lie side by side in one tensor with other columns between and around them.  The prompt step in the form
    the sizes choose (chunks on the matrix cores where the key width allows) and in the token-by-token form."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(dk * 7 + dv)
    decay = torch.tensor([0.0, 1.0, 0.9, 0.999, 0.5][:H] if H <= 5 else [0.9] * H, dtype=torch.float64)
    lens, first = [37, 1, 70], [5, 0, 0]                      # sequence 0 has 5 earlier tokens
    qc, kc, vc, W = 3, 3 + H * dk + 2, 3 + 2 * H * dk + 4, 3 + 2 * H * dk + 4 + H * dv + 1
    slots = [4, 1, 2]
    state = torch.zeros(6, H * dk * dv + 3, dtype=torch.float32)
    state[1] = 7.0                                            # what an earlier owner of slot 1 left: a sequence at position 0 ignores it
    xs, want, S_after = [], [], []

    def halves(x):
        x = x.double()
        return (pf.silu(x[:, qc:qc + H * dk]).view(-1, H, dk), pf.silu(x[:, kc:kc + H * dk]).view(-1, H, dk),
                pf.silu(x[:, vc:vc + H * dv]).view(-1, H, dv))
    for b, (n, p0) in enumerate(zip(lens, first)):
        S0 = None
        if p0:
            x0 = (0.7 * torch.randn(p0, W, generator=g)).to(dtype)
            _, S0 = pf.decayed_sums(*halves(x0), decay)
            state[slots[b], :H * dk * dv] = S0.reshape(-1).float()
        x = (0.7 * torch.randn(n + 1, W, generator=g)).to(dtype)          # the last row is decoded afterwards
        o, S = pf.decayed_sums(*halves(x), decay, S0)
        xs.append(x)
        want.append(o)
        S_after.append(S)
    st = state.to(DEV)
    tiles, r = [], 0
    for b, n in enumerate(lens):
        tiles.append([b, r, n, first[b]])
        r += n
    tiles.append([0, 0, 0, 0])                                 # a tile of no rows
    x = torch.cat([t[:-1] for t in xs]).to(DEV)
    o = ops.lightning_scan(x, qc, kc, vc, decay.float().to(DEV), st, i32(slots), H, dk, dv, tiles=i32(tiles), chain=chain)
    tol = 2e-5 if dtype == torch.float32 else 1e-4            # the inputs are the same rounded numbers on both sides
    close_ = lambda a, b: rel_err(a, b) < tol
    assert close_(o, torch.cat([w[:-1] for w in want]).reshape(sum(lens), -1))
    # one token each, with a padding row between them; slots in another order than the rows
    xd = torch.stack([xs[2][-1], xs[0][-1], torch.zeros(W, dtype=dtype), xs[1][-1]]).to(DEV)
    before = st.clone()
    od = ops.lightning_scan(xd, qc, kc, vc, decay.float().to(DEV), st, i32([slots[2], slots[0], 5, slots[1]]), H, dk, dv,
                            seq_lens=i32([lens[2] + 1, first[0] + lens[0] + 1, 0, 2]))
    assert close_(od[[0, 1, 3]], torch.stack([want[2][-1], want[0][-1], want[1][-1]]).reshape(3, -1))
    for b in range(3):
        assert close_(st[slots[b], :H * dk * dv], S_after[b].reshape(-1))
    assert torch.equal(st[5], before[5]) and torch.equal(st[0], before[0]) and torch.equal(st[:, H * dk * dv:], before[:, H * dk * dv:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk,dv,seqs", [(2, 64, 64, 1), (2, 128, 128, 1), (3, 96, 40, 1), (1, 32, 16, 1), (20, 48, 64, 1),
                                          (40, 64, 72, 1)])
def test_the_chunked_form_at_the_edges_of_its_chunks(dtype, H, dk, dv, seqs):
    """Prompt steps whose sequences end just before, at and just behind a chunk of 64 tokens and a block of 16, some
    continuing from a state at a position that is no multiple of either; few heads and many, widths that are no multiple
    of a tile's 16.  Against the recurrence written token by token, and the state left behind against both; then the same
    step on the token-by-token kernel."""
    from bitnet_c_amd import ops
    assert ops.lightning_chunked(dk, dv)
    g = torch.Generator().manual_seed(H * 1000 + dk + dv)
    decay = torch.tensor([0.97, 0.5, 0.9995, 0.0, 1.0], dtype=torch.float64).repeat(H // 5 + 1)[:H]
    lens = [63, 64, 65, 128, 129, 2, 200, 15, 16, 17, 1] * seqs
    first = [0, 7, 0, 0, 70, 3, 0, 64, 0, 1, 9] * seqs
    W = 2 * H * dk + H * dv + 8
    qc, kc, vc = 0, H * dk, 2 * H * dk + 8
    n_slots = len(lens) + 2
    state = torch.zeros(n_slots, H * dk * dv, dtype=torch.float32)
    slots = list(range(n_slots - 1, 1, -1))[:len(lens)]
    xs, want, S_after = [], [], []

    def halves(x):
        x = x.double()
        return (pf.silu(x[:, qc:qc + H * dk]).view(-1, H, dk), pf.silu(x[:, kc:kc + H * dk]).view(-1, H, dk),
                pf.silu(x[:, vc:vc + H * dv]).view(-1, H, dv))
    for b, (n, p0) in enumerate(zip(lens, first)):
        S0 = None
        if p0:
            S0 = 0.5 * torch.randn(H, dk, dv, generator=g).float().double()
            state[slots[b]] = S0.reshape(-1).float()
        else:
            state[slots[b]] = 3.0                              # a former owner's state: ignored at position 0
        x = (0.7 * torch.randn(n, W, generator=g)).to(dtype)
        o, S = pf.decayed_sums(*halves(x), decay, S0)
        xs.append(x)
        want.append(o.reshape(n, -1))
        S_after.append(S.reshape(-1))
    tiles, r = [], 0
    for b, n in enumerate(lens):
        tiles.append([b, r, n, first[b]])
        r += n
    x = torch.cat(xs).to(DEV)
    want, S_after = torch.cat(want), torch.stack(S_after)
    tol = 2e-5 if dtype == torch.float32 else 1e-4            # the inputs are the same rounded numbers on both sides
    outs = []
    for chain in (False, True):
        st = state.to(DEV)
        o = ops.lightning_scan(x, qc, kc, vc, decay.float().to(DEV), st, i32(slots), H, dk, dv, tiles=i32(tiles), chain=chain)
        # sequence by sequence and head by head (each against its own size: a head that never decays grows far beyond
        # the others): a short sequence is not hidden by a long one
        for b in range(len(lens)):
            rows = slice(tiles[b][1], tiles[b][1] + lens[b])
            for h in range(H):
                assert rel_err(o[rows, h * dv:(h + 1) * dv], want[rows, h * dv:(h + 1) * dv]) < tol, (chain, b, h)
                assert rel_err(st[slots[b]].view(H, -1)[h], S_after[b].view(H, -1)[h]) < tol, (chain, b, h)
        assert torch.equal(st[:2].cpu(), state[:2])            # rows of no sequence of the step
        outs.append(o)
    assert rel_err(outs[0], outs[1]) < 2 * tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_key_far_back_carries_the_result_under_a_slow_decay(dtype):
    """One key far back is made to stand out (it and the last query are scaled along one direction): under decay 0.9995
    its value is what comes out, 900 tokens later; under decay 0.9 it has faded away.  In a prompt and decoded."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(5)
    H, dk, dv, T, far = 2, 32, 32, 1000, 100
    decay = torch.tensor([0.9995, 0.9], dtype=torch.float64)
    x = (0.3 * torch.randn(T, 2 * H * dk + H * dv, generator=g))
    for h in range(H):
        x[far, H * dk + h * dk] = 30.0                        # the far key, and the last query along it
        x[T - 1, h * dk] = 30.0
    x[far, 2 * H * dk:] = 3.0                                 # and a value that is seen
    x = x.to(dtype)
    xd = x.double()
    q, k, v = (pf.silu(xd[:, :H * dk]).view(T, H, dk), pf.silu(xd[:, H * dk:2 * H * dk]).view(T, H, dk),
               pf.silu(xd[:, 2 * H * dk:]).view(T, H, dv))
    want, _ = pf.decayed_sums(q, k, v, decay)
    share = (0.9995 ** (T - 1 - far)) * 900.0 * v[far, 0]
    assert float((want[-1, 0] - share).norm() / want[-1, 0].norm()) < 0.2      # the far key carries head 0's last output
    assert float(want[-1, 1].norm()) < 0.05 * float(want[-1, 0].norm())          # and is gone from head 1's
    tol = 1e-4              # the far key's share has been multiplied by its decay 900 times, each product rounded to float32
    for cut in (T, T - 1, 700):
        st = torch.zeros(2, H * dk * dv, dtype=torch.float32, device=DEV)
        o = ops.lightning_scan(x[:cut].to(DEV), 0, H * dk, 2 * H * dk, decay.float().to(DEV), st, i32([1]), H, dk, dv,
                               tiles=i32([[0, 0, cut, 0]]))
        parts = [o]
        for t in range(cut, T):
            parts.append(ops.lightning_scan(x[t:t + 1].to(DEV), 0, H * dk, 2 * H * dk, decay.float().to(DEV), st, i32([1]), H,
                                            dk, dv, seq_lens=i32([t + 1])))
        got = torch.cat(parts)
        assert rel_err(got[-1], want[-1].reshape(-1)) < tol and rel_err(got[:-1], want[:-1].reshape(T - 1, -1)) < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [24, 96, 2500])
def test_heads_normed_together_and_gated(dtype, W):
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(W)
    T, eps = 9, 1e-5
    o = 5.0 * torch.randn(T, W, generator=g)
    wide = torch.randn(T, W + 11, generator=g).to(dtype)       # the gate is a run of columns of a wider tensor
    w = 1 + 0.3 * torch.randn(W, generator=g)
    want = pf.unit_rms(o.double(), eps) * w.double() * pf.sigmoid(wide[:, 11:].double())
    got = ops.row_norm_gate(o.to(DEV), wide.to(DEV)[:, 11:], w.to(DEV), eps, "sigmoid")
    assert got.dtype == dtype and rel_err(got, want) < (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,K,D,shared", [(6, 2, 64, True), (3, 3, 48, False), (1, 1, 32, True), (70, 5, 40, False), (16, 1, 256, True)])
def test_the_router_chooses_by_corrected_scores_and_weighs_by_plain_ones(dtype, E, K, D, shared):
    """Softmax scores, the choice by score + correction (a correction large enough to change choices), the weights from
    the plain scores of the chosen over their sum, times a constant; and the shared expert's gate beside them."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(E * 10 + K)
    T, scale = 50, 2.5
    h = torch.randn(T, D, generator=g).to(dtype)
    W = {"r.router": (3.0 * torch.randn(E, D, generator=g) / math.sqrt(D)).to(torch.bfloat16).double(),
         "r.correction": (0.3 * torch.randn(E, generator=g)).to(torch.bfloat16).double(),
         "r.sg": torch.randn(1, D, generator=g).to(torch.bfloat16).double() / math.sqrt(D)}
    mlp = dict(router=dict(experts=E, top=K, scale=scale))
    margins = []
    chosen, w = pf.route(h.double(), W, "r.", mlp, margins)
    plain_choice = torch.topk(torch.softmax(h.double() @ W["r.router"].T, -1), K, dim=-1).indices
    if 1 < K < E or (K == 1 and E > 1):
        assert not torch.equal(chosen.sort(-1).values, plain_choice.sort(-1).values)        # the correction matters
    out = ops.moe_route(h.to(DEV), W["r.router"].float().to(DEV), K, "softmax", True, choice_bias=W["r.correction"].float().to(DEV),
                        weight_floor=1e-20, weight_scale=scale, gate=W["r.sg"].float().reshape(-1).to(DEV) if shared else None)
    ids, wts = out[0].cpu(), out[1].cpu()
    sure = margins[0] > 0.02
    assert int(sure.sum()) > T // 2
    for t in range(T):
        if not sure[t]:
            continue
        assert sorted(ids[t].tolist()) == sorted(chosen[t].tolist())
        by_id = {int(e): float(x) for e, x in zip(chosen[t], w[t])}
        for e, x in zip(ids[t].tolist(), wts[t].tolist()):
            assert abs(x - by_id[e]) <= 2e-5 * scale
        assert abs(float(wts[t].sum()) - scale) < 1e-4 * scale
    if shared:
        assert rel_err(out[2], pf.sigmoid(h.double() @ W["r.sg"].T)[:, 0]) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,K,D,F,T,limit", [(6, 2, 64, 32, 40, 1.0), (3, 3, 48, 16, 9, 0.5), (1, 1, 32, 8, 20, 2.0), (9, 4, 96, 64, 70, 1.0),
                                             (16, 1, 128, 64, 300, 1.5), (4, 2, 72, 40, 700, 1.0), (5, 1, 36, 20, 30, 50.0)])
def test_gated_experts_with_clamped_arguments(dtype, E, K, D, F, T, limit):
    """Every (token, choice) pair against the unit written out: steps of few rows (a pair at a time) and of many (grouped
    products on the matrix cores); the weights are large enough for both clamps to bite, and a limit that never does."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(E * 100 + T)
    h = torch.randn(T, D, generator=g).to(dtype)
    W = {}
    for e in range(E):
        W[f"x.e{e}.gate"] = (2.0 * torch.randn(F, D, generator=g) / math.sqrt(D)).to(dtype).double()
        W[f"x.e{e}.up"] = (2.0 * torch.randn(F, D, generator=g) / math.sqrt(D)).to(dtype).double()
        W[f"x.e{e}.down"] = (torch.randn(D, F, generator=g) / math.sqrt(F)).to(dtype).double()
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    wts = torch.rand(T, K, generator=g) + 0.1
    w_up = torch.stack([torch.cat([W[f"x.e{e}.gate"], W[f"x.e{e}.up"]]) for e in range(E)]).to(dtype).to(DEV)
    w_down = torch.stack([W[f"x.e{e}.down"] for e in range(E)]).to(dtype).to(DEV)
    want = torch.zeros(K, T, D, dtype=torch.float64)
    hit = 0
    for j in range(K):
        for e in range(E):
            rows = torch.nonzero(ids[:, j] == e)[:, 0]
            if rows.numel():
                want[j, rows] = wts[rows, j, None].double() * pf.expert_unit(h[rows].double(), W, f"x.e{e}.", limit)
                hit += int(((h[rows].double() @ W[f"x.e{e}.gate"].T) > limit).sum())
    assert (hit > 0) == (limit < 50.0)
    unit = ops.ClampedUnit(limit)
    paths = [ops.moe_experts]
    if ops.moe_grouped_supported(T, D, F, dtype):
        paths.append(ops.moe_experts_grouped)
    for path in paths:
        y = path(h.to(DEV), w_up, w_down, ids.to(DEV), wts.to(DEV), weight_on_input=False, gated=unit, extra_slabs=1)
        assert tuple(y.slabs.shape) == (K + 1, T, D)
        assert rel_err(y.slabs[:K], want) < (1e-5 if dtype == torch.float32 else 2.5e-2)
    gu = torch.randn(T, 2 * F, generator=g).to(dtype)
    rs = torch.rand(T, generator=g)
    wanted = (lambda gg, u: torch.clamp(gg, max=limit) * pf.sigmoid(pf.GATE_SLOPE * torch.clamp(gg, max=limit))
              * (torch.clamp(u, -limit, limit) + 1.0))(2 * gu[:, :F].double(), 2 * gu[:, F:].double()) * rs[:, None].double()
    got = ops.gated_unit((2 * gu).to(DEV), unit, rs.to(DEV)).double().cpu()
    if dtype == torch.float32:
        assert rel_err(got, wanted) < 1e-5
    else:                                  # one rounding of every element
        assert bool(((got - wanted).abs() <= 2.0 ** -8 * wanted.abs() + 1e-6).all())


# ------------------------------------------------------------------------------------------------------------------
# whole models through the engine
# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts_and_the_stream_after_every_layer(folders, name, dtype):
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype)
    for n in (1, 2, 77, 150):
        toks = settled_tokens(folder, n, 1)
        streams, got = [], []
        want = pf.forward(pf.read_config(folder), pf.read_weights(folder), toks, streams)
        eng.tap = lambda point, entry, stream, ctx: got.append(stream.flush().clone()) if point == "layer_out" else None
        s = eng.new_sequence()
        logits = eng.step([bn.StepEntry(s, toks, list(range(n)))])
        eng.release(s)
        eng.tap = None
        assert len(got) == len(streams) == len(CONFIGS[name]["layers"])
        for a, b in zip(got, streams):
            close(a, b, dtype)
        close(logits, want, dtype)
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prefill_against_decoding_token_by_token(folders, name, dtype, graphs):
    """A prompt, then 100 tokens one by one (across page borders), against the plain implementation of the whole
    sequence; and the same sequence from its very first token one by one."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype, use_graphs=graphs)
    toks = settled_tokens(folder, 150, 1)
    want = plain(folder, toks)
    for first in (50, 1):
        s = eng.new_sequence()
        parts = [eng.step([bn.StepEntry(s, toks[:first], list(range(first)))])]
        for t in range(first, len(toks) if first == 50 else 40):
            parts.append(eng.step([bn.StepEntry(s, [toks[t]], [0])]))
        eng.release(s)
        got = torch.cat(parts)
        close(got, want[:got.shape[0]], dtype)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_of_several_sizes(folders, name, dtype):
    """A prompt cut into portions of 2, 3, 1, 64, 5, 2, ... tokens gives what the whole prompt gives."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype)
    toks = settled_tokens(folder, 150, 1)
    want = plain(folder, toks)
    for cuts in ([2, 3, 1, 64, 5, 2, 40, 2, 31], [2] * 75, [149, 1], [63, 1, 1, 85], [15, 1, 16, 17, 101]):
        assert sum(cuts) == len(toks)
        s, at, parts = eng.new_sequence(), 0, []
        for n in cuts:
            parts.append(eng.step([bn.StepEntry(s, toks[at:at + n], list(range(n)))]))
            at += n
        eng.release(s)
        close(torch.cat(parts), want, dtype)
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_unequal_batches_and_slots_used_again(folders, name, dtype, graphs):
    """Requests of 1, 70, 9 and 130 tokens as one batch, decoded together while the shorter ones end; then other
    requests in the slots, pages and state rows that were given back; every request against itself alone (the plain
    implementation)."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype, max_tokens=1024, use_graphs=graphs)
    for round_, lens in enumerate(([1, 70, 9, 130], [64, 3, 128], [5])):
        reqs = [settled_tokens(folder, n + 6 + 3 * i, 2 + (round_ + i) % 4) for i, n in enumerate(lens)]
        slots = [eng.new_sequence() for _ in reqs]
        got = [[] for _ in reqs]
        out = eng.step([bn.StepEntry(s, r[:n], [n - 1]) for s, r, n in zip(slots, reqs, lens)])
        for i in range(len(reqs)):
            got[i].append(out[i:i + 1])
        at = list(lens)
        live = list(range(len(reqs)))
        while live:
            out = eng.step([bn.StepEntry(slots[i], [reqs[i][at[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                got[i].append(out[j:j + 1])
                at[i] += 1
            for i in [i for i in live if at[i] == len(reqs[i])]:
                eng.release(slots[i])
                live.remove(i)
        for i, r in enumerate(reqs):
            close(torch.cat(got[i]), plain(folder, r)[lens[i] - 1:], dtype)
        eng.cache.check()
    assert eng.cache.live_slots() == []


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_steps_replayed_from_graphs(folders, name, dtype):
    """Prompt steps of one size run eagerly the first time, are recorded the second time and replayed afterwards, with
    other sequences in other slots each time: every one of them against the plain implementation, and what a recorded step
    left in the cache and in the states is what the tokens decoded behind it go on from."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype)
    assert eng.prompt_graphs and eng.use_graphs
    keep = eng.new_sequence()                      # a live neighbour, so that later sequences get other slots
    eng.step([bn.StepEntry(keep, settled_tokens(folder, 9, 1), [])])
    for i in range(5):
        reqs = [settled_tokens(folder, n, 2 + (i + k) % 4) for k, n in enumerate((70 + i, 20 - i))]
        slots = [eng.new_sequence() for _ in reqs]
        out = eng.step([bn.StepEntry(s, r[:-3], [0, len(r) - 4]) for s, r in zip(slots, reqs)])
        tail = [eng.step([bn.StepEntry(s, [r[t]], [0]) for s, r in zip(slots, reqs)]) for t in (-3, -2, -1)]
        for k, r in enumerate(reqs):
            want = plain(folder, r)
            close(out[2 * k:2 * k + 2], want[[0, len(r) - 4]], dtype)
            close(torch.cat([t[k:k + 1] for t in tail]), want[-3:], dtype)
        eng.release(slots[i % 2])
    assert eng.graphs_built >= 2                   # a prompt step and the decode steps were recorded
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


def _peaked_folder(tmp_path):
    """A model whose attention is peaked (a large scale: single far keys carry a query's result, and where none does the
    sink takes the weight) and whose recurrences keep what is far back (decays next to 1) beside heads that forget."""
    cfg = dict(architecture="Fazopel", vocab=61, width=32, norm=dict(eps=1e-5), layers=[
        _att(2, 1, 8, 1.5, (10000.0, 4, 8.0, 1.0, 4.0, 256), _dense(48)),
        _lin(2, 8, 8, None, decay=[0.9995, 0.8]),
        _att(2, 2, 8, 1.0, None, None),
        _lin(3, 4, 8, _dense(40), decay=[1.0, 0.999, 0.3])])
    return write_folder(tmp_path / "peaked", cfg, 9)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_with_far_keys_and_slow_decays(tmp_path, dtype):
    """A long sequence (past a run of a float32 cache's keys, many pages, states that have summed thousands of tokens), as
    a prompt in portions and then decoded for 80 tokens."""
    import bitnet_c_amd as bn
    folder = _peaked_folder(tmp_path)
    toks = torch.randint(0, 61, (2200,), generator=torch.Generator().manual_seed(2)).tolist()     # no experts: no close calls
    # positions and angles are float32 in the engine; at 2,000 tokens and under a peaked softmax that alone is seen in
    # float32 logits, so the plain implementation rounds them alike here
    want = pf.forward(pf.read_config(folder), pf.read_weights(folder), toks, angle_dtype=torch.float32)
    eng = engine(folder, dtype, max_tokens=4608)
    s, at, parts = eng.new_sequence(), 0, []
    check = [0, 1, 15, 16, 17, 63, 64, 65, 299, 300, 301, 2047, 2048, 2049, 2119]
    for n in (1000, 1047, 73):
        w = [p - at for p in check if at <= p < at + n]
        parts.append(eng.step([bn.StepEntry(s, toks[at:at + n], w)]))
        at += n
    # bfloat16: scores reach 12 here, so the rounding of queries and keys to 8 bits moves a score by up to 0.1 and a
    # weight of the softmax by a tenth; a wrong or a lost key moves a row by its own size
    close(torch.cat(parts), want[check], dtype, bf16_rows=0.2)
    dec = torch.cat([eng.step([bn.StepEntry(s, [toks[t]], [0])]) for t in range(at, 2200)])
    close(dec, want[at:], dtype, bf16_rows=0.2)
    s2 = eng.new_sequence()                              # and the same positions from one step over the whole sequence
    whole = eng.step([bn.StepEntry(s2, toks, list(range(at, 2200)))])
    assert rel_err(dec, whole) < (1e-4 if dtype == torch.float32 else 1.0)
    if dtype == torch.bfloat16:
        close(dec, whole.double(), dtype, bf16_rows=0.2)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_sink_takes_the_weight_that_no_key_claims(tmp_path, dtype):
    """Queries made to score far below zero against every key (the query norm's weight negated and the scale raised): the
    sink then holds nearly all of the softmax and the attention's output nearly vanishes; a softmax without the sink would
    hand the values on in full.  The model's logits follow the plain implementation either way."""
    import bitnet_c_amd as bn
    cfg = dict(architecture="Fazopel", vocab=50, width=32, norm=dict(eps=1e-5), layers=[_att(2, 1, 8, 4.0, None, None)])
    g = torch.Generator().manual_seed(3)
    wk = torch.randn(8, 32, generator=g) / math.sqrt(32)
    folder = write_folder(tmp_path / "sink", cfg, 4, overrides={"l0.mix.q": torch.cat([wk, wk]), "l0.mix.k": wk,
                                                                "l0.mix.q.norm": -torch.ones(8), "l0.mix.k.norm": torch.ones(8)})
    toks = torch.randint(0, 50, (70,), generator=g).tolist()
    c, W = pf.read_config(folder), pf.read_weights(folder)
    h = W["embed"][toks]
    y, _ = pf.sink_attention(h, W, "l0.mix.", c["layers"][0]["mixer"], 1e-5)
    kv = (h @ W["l0.mix.k"].T)
    assert float(y[0].norm()) < 1e-3 * float((kv[0:1].repeat(1, 2) @ W["l0.mix.o"].T).norm())      # q = -k: score -32, all in the sink
    eng = engine(folder, dtype)
    s = eng.new_sequence()
    got = eng.step([bn.StepEntry(s, toks[:60], list(range(60)))])
    dec = torch.cat([eng.step([bn.StepEntry(s, [t], [0])]) for t in toks[60:]])
    close(torch.cat([got, dec]), pf.forward(c, W, toks), dtype)


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
    """Greedy generation through load() and generate(), the scheduler batching three prompts two at a time.  float32: the
    plain implementation's tokens, as far as no expert choice along the way is a close call; bfloat16: every token that was
    chosen holds, where it was chosen, the plain implementation's largest logit within rounding (up to the first close
    expert choice of the sequence that the engine itself wrote)."""
    import bitnet_c_amd as bn
    folder = folders(name)
    llm = bn.load(folder, dtype="float32" if dtype == torch.float32 else "bfloat16", max_tokens=1024)
    prompts = [settled_tokens(folder, n, 2 + i) for i, n in enumerate((5, 66, 1))]
    got = llm.generate(prompts, max_new_tokens=12, temperature=0.0, stop_ids=(), batch_size=2)
    cfg, W = pf.read_config(folder), pf.read_weights(folder)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        margins = []
        logits = pf.forward(cfg, W, p + g, margins=margins)[len(p) - 1:-1]
        settled = 0                                        # generated tokens before the first close call
        while settled < 12 and margins[len(p) + settled - 1] >= (1e-3 if dtype == torch.float32 else 0.05):
            settled += 1
        rms = float(logits.pow(2).mean().sqrt())
        for i, tok in enumerate(g[:settled]):
            gap = float(logits[i].max() - logits[i, tok])
            assert gap <= (1e-4 if dtype == torch.float32 else 4e-2) * rms, (i, gap / rms)
    llm.engine.cache.check()
    assert llm.engine.cache.live_slots() == []


def test_command_line_and_trace_replay(folders, tmp_path):
    """The command line generates from a Fazopel folder (also one that it writes itself from a configuration file, with
    random weights), and the trace replay program steps one through a batch of prompts and single tokens."""
    import subprocess
    import sys
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = folders("D")
    cfg, W = pf.read_config(folder), pf.read_weights(folder)
    prompt = settled_tokens(folder, 8, 1)
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "bitnet"), folder, "--prompt-token-ids", ",".join(map(str, prompt)),
                        "-n", "6", "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--quiet"], capture_output=True, text=True,
                       timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    ids = [int(x) for x in [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0].split(",")]
    margins = []
    logits = pf.forward(cfg, W, prompt + ids, margins=margins)[len(prompt) - 1:-1]
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
    assert pf.read_config(made)["layers"] == CONFIGS["B"]["layers"]
    # trace replay: two requests that start together, then go on token by token; the shorter one ends earlier
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
