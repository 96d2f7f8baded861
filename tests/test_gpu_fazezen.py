"""Fazezen on the GPU against the plain implementation: each kernel alone, each mixer alone with its own cache (whole,
token by token, in portions, in unequal batches, with pages and slots used again), whole models replayed in the four
ways of cutting, and greedy generation through the session and its scheduler.

Where random weights would hide a fault, the inputs are made so that it shows: one key is scaled so that its score
stands out, and it is put far back, on a page's first and last row, and just inside and just outside a run of positions;
one key and query of the fading state are made to meet hundreds of tokens apart.
"""
import math

import numpy as np
import pytest
import torch

import plain_fazezen as P
import replay as R
from tiny import random_ids
from tiny_fazezen import CONFIGS, STD, write_tiny

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def gen(seed):
    return torch.Generator().manual_seed(seed)


def tol(dtype, ref, f32=2e-5, bf16=1e-2):
    return (f32 if dtype == torch.float32 else bf16) * max(1.0, float(ref.abs().max()))


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


@pytest.fixture(scope="module")
def ops():
    from gesso_amd.kernels import ops
    ops.lib()
    return ops


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return str(tmp_path_factory.mktemp("fazezen"))


# ------------------------------------------------------------------ kernels alone

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [100, 256, 1030])
def test_two_adds_and_two_norms_of_one_row(ops, dtype, H):
    res = torch.randn(5, H, generator=gen(0))
    d1, d2 = (torch.randn(5, H, generator=gen(1)) * 2).to(dtype), torch.randn(5, H, generator=gen(2)).to(dtype)
    w1, w2 = 1 + 0.2 * torch.randn(H, generator=gen(3)), 1 + 0.2 * torch.randn(H, generator=gen(4))
    for deltas in ((d1, d2), (d1, None), (None, None)):
        r = res.clone().to(DEV)
        a, b = ops.add_rmsnorm_pair(r, *(None if d is None else d.to(DEV) for d in deltas), w1.to(DEV), w2.to(DEV), 1e-4, dtype)
        x = res.double() + sum(d.double() for d in deltas if d is not None)
        assert float((r.cpu().double() - x).abs().max()) <= 1e-6 * float(x.abs().max())
        for got, w in ((a, w1), (b, w2)):
            want = P.rms(x, 1e-4) * w.double()
            assert float((got.cpu().double() - want).abs().max()) <= tol(dtype, want)
    only, none = ops.add_rmsnorm_pair(res.clone().to(DEV), d1.to(DEV), None, w1.to(DEV), None, 1e-4, dtype)
    assert none is None and only.shape == (5, H)
    # a vector added to every row on the way (a last product's bias)
    bias = torch.randn(H, generator=gen(5))
    r = res.clone().to(DEV)
    a, _ = ops.add_rmsnorm_pair(r, d1.to(DEV), d2.to(DEV), w1.to(DEV), w2.to(DEV), 1e-4, dtype, bias=bias.to(DEV))
    x = res.double() + d1.double() + d2.double() + bias.double()
    assert float((r.cpu().double() - x).abs().max()) <= 1e-6 * float(x.abs().max())
    want = P.rms(x, 1e-4) * w1.double()
    assert float((a.cpu().double() - want).abs().max()) <= tol(dtype, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["gelu_tanh", "silu"])
def test_gated_activation_with_and_without_biases(ops, dtype, act):
    x = (torch.randn(7, 2 * 52, generator=gen(5)) * 2).to(dtype)
    b = torch.randn(104, generator=gen(6))
    f = P.gelu_tanh if act == "gelu_tanh" else P.silu
    for bias in (b, None):
        got = ops.gated_act(x.to(DEV), None if bias is None else bias.to(DEV), act, dtype).cpu().double()
        xb = x.double() + (0 if bias is None else bias.double())
        want = f(xb[:, :52]) * xb[:, 52:]
        assert float((got - want).abs().max()) <= tol(dtype, want)
    wide = ops.gated_act(x.float().to(DEV), b.to(DEV), act, dtype).cpu().double()       # a product's float32 sums
    xb = x.double() + b.double()
    assert float((wide - f(xb[:, :52]) * xb[:, 52:]).abs().max()) <= tol(dtype, xb)


def test_weighted_sum_of_two_results(ops):
    a, b = torch.randn(9, 33, generator=gen(7)), torch.randn(9, 33, generator=gen(8))
    got = ops.scaled_sum(a.to(DEV), 1.25, b.to(DEV), -0.5, torch.bfloat16).cpu()
    assert torch.equal(got, (1.25 * a - 0.5 * b).to(torch.bfloat16))
    assert torch.allclose(ops.scaled_sum(a.to(DEV), 0.3, b.to(DEV), 2.0, torch.float32).cpu(), 0.3 * a + 2.0 * b, atol=1e-6)


def scan_case(ops, dtype, H, n, m, lens, rd=0, act=None, scale=1.0, decay=None, seed=0, base=1e3, pos0=None, boost=None,
              runs_from=0, segment=0):
    """Rows of q | junk | k | v for sequences of ``lens`` tokens, states in shuffled slots: the kernel's outputs and
    states, and the plain implementation's.  ``pos0``: the first position of each sequence (its state then starts from
    a random one).  ``boost``: ``(sequence, far token, near token)``: that key and that query are made to meet."""
    g = gen(seed)
    T = sum(lens)
    junk = 5
    ld = 2 * H * n + junk + H * m
    x = (torch.randn(T, ld, generator=g) * 0.7)
    if boost is not None:
        s, far, near = boost
        a0 = sum(lens[:s])
        for h in range(H):
            x[a0 + far, H * n + junk + h * n:H * n + junk + (h + 1) * n] = 200.0 * x[a0 + near, h * n:(h + 1) * n]
    x = x.to(dtype)
    decay = decay or [0.3 + 0.69 * i / max(1, H - 1) for i in range(H)]
    pos0 = pos0 or [0] * len(lens)
    slots = torch.randperm(len(lens) + 2, generator=g)[:len(lens)].tolist()
    state = torch.full((len(lens) + 3, H, n, m), float("nan"))
    start = {}
    for s_, sl in enumerate(slots):
        start[s_] = torch.randn(H, n, m, generator=g) if pos0[s_] else torch.zeros(H, n, m)
        state[sl] = start[s_]
    q_start = [0]
    for L in lens:
        q_start.append(q_start[-1] + L)
    positions = [pos0[s_] + t for s_, L in enumerate(lens) for t in range(L)]
    cos = sin = None
    f = P.frequencies(rd, base) if rd else []
    if rd:
        ang = torch.arange(max(positions) + 1, dtype=torch.float64)[:, None] * torch.tensor(f, dtype=torch.float64)[None]
        cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    st = state.to(DEV)
    args = (x.to(DEV), 0, H * n + junk, 2 * H * n + junk, H, n, m, torch.tensor(decay, dtype=torch.float32, device=DEV), st,
            i32(q_start), i32(slots), i32(positions), len(lens))
    kw = dict(activation=act, cos=cos, sin=sin, rotary_dim=rd, key_scale=scale)
    if runs_from:
        # sequences of at least that many tokens on the matrix cores, the others token by token, into one result
        out = torch.full((T, H * m), float("nan"), device=DEV)
        ops.linear_attention_scan(*args, chunks_from=runs_from, out=out, segment=segment, longest=max(lens), **kw)
        ops.linear_attention_scan(*args, below=runs_from, out=out, **kw)
    else:
        out = ops.linear_attention_scan(*args, **kw)
    xd = x.double()
    fa = P.silu if act == "silu" else (lambda z: z)
    want, want_state = [], {}
    for s_, L in enumerate(lens):
        a0 = q_start[s_]
        rows = xd[a0:a0 + L]
        q = fa(rows[:, :H * n]).reshape(L, H, n)
        k = fa(rows[:, H * n + junk:2 * H * n + junk]).reshape(L, H, n)
        v = fa(rows[:, 2 * H * n + junk:]).reshape(L, H, m)
        pos = positions[a0:a0 + L]
        q, k = P.turn(q, pos, f), P.turn(k, pos, f) * scale
        o = torch.zeros(L, H, m, dtype=torch.float64)
        S = start[s_].double().clone()
        for t in range(L):
            for h in range(H):
                S[h] = float(torch.tensor(decay[h], dtype=torch.float32)) * S[h] + torch.outer(k[t, h], v[t, h])
                o[t, h] = S[h].t() @ q[t, h]
        want.append(o.reshape(L, H * m))
        want_state[slots[s_]] = S
    return out.cpu().double(), torch.cat(want), st.cpu().double(), want_state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,n,m,rd,act,scale", [(3, 24, 16, 0, "silu", 1.0), (2, 16, 24, 8, None, 0.25), (1, 40, 48, 40, None, 0.5),
                                                (2, 64, 64, 0, "silu", 1.0), (1, 128, 130, 64, None, 0.1), (5, 6, 10, 2, None, 1.0),
                                                (1, 200, 70, 0, None, 0.3), (2, 32, 64, 32, None, 32 ** -0.5), (1, 300, 40, 300, None, 0.05),
                                                (1, 512, 8, 0, "silu", 0.1)])
def test_fading_state_kernel_over_unequal_sequences(ops, dtype, H, n, m, rd, act, scale):
    got, want, state, want_state = scan_case(ops, dtype, H, n, m, [1, 19, 2, 33], rd, act, scale, seed=n + m)
    assert float((got - want).abs().max()) <= 5e-5 * max(1.0, float(want.abs().max()))     # float32 arithmetic in both types
    for slot, S in want_state.items():
        assert float((state[slot] - S).abs().max()) <= 5e-5 * max(1.0, float(S.abs().max()))
    untouched = [s for s in range(state.shape[0]) if s not in want_state]
    assert all(torch.isnan(state[s]).all() for s in untouched)


@pytest.mark.parametrize("H,n,m,rd,act,scale,decay", [
    (3, 24, 16, 0, "silu", 1.0, None), (2, 16, 24, 8, None, 0.25, None), (1, 40, 48, 40, None, 0.5, None),
    (2, 64, 64, 0, "silu", 1.0, (0.97, 0.999)), (1, 128, 130, 64, None, 0.1, (0.99,)), (5, 6, 10, 2, None, 1.0, (0.0, 0.5, 0.9, 1.0, 0.999)),
    (2, 128, 128, 0, "silu", 1.0, (1.0, 0.9)), (2, 32, 64, 32, None, 32 ** -0.5, None), (1, 96, 300, 10, None, 0.2, None)])
def test_fading_state_kernel_on_the_matrix_cores(ops, H, n, m, rd, act, scale, decay):
    """Prompt portions 32 tokens at a time: whole runs, a last run of one token, sequences below the kernel's least
    length beside it, states that go on from earlier steps (positions deep in a sequence)."""
    lens, pos0 = [1, 70, 9, 33, 8, 140, 32, 7], [5, 0, 100, 0, 31, 12, 0, 0]
    got, want, state, want_state = scan_case(ops, torch.bfloat16, H, n, m, lens, rd, act, scale, decay=decay and list(decay),
                                             seed=n + m, pos0=pos0, runs_from=8)
    bound = 1e-4
    assert float((got - want).abs().max()) <= bound * max(1.0, float(want.abs().max()))
    for slot, S in want_state.items():
        assert float((state[slot] - S).abs().max()) <= bound * max(1.0, float(S.abs().max()))
    untouched = [s for s in range(state.shape[0]) if s not in want_state]
    assert all(torch.isnan(state[s]).all() for s in untouched)


@pytest.mark.parametrize("H,n,m,rd,act,scale,decay,segment", [
    (2, 64, 64, 0, "silu", 1.0, (0.97, 0.999), 64), (1, 128, 130, 64, None, 0.1, (0.99,), 128), (3, 24, 16, 0, None, 1.0, (1.0, 0.0, 0.9), 32),
    (2, 32, 64, 32, None, 32 ** -0.5, (0.9, 0.995), 96), (2, 16, 24, 8, None, 0.25, None, 64)])
def test_fading_state_kernel_with_long_portions_cut_into_segments(ops, H, n, m, rd, act, scale, decay, segment):
    """Segments side by side, their first states made by a pass between: a last segment of one token, of a whole
    segment, sequences of one segment only, states that go on from earlier steps."""
    lens, pos0 = [300, 1, 2 * segment, 40, 2 * segment + 1, 9], [0, 3, 77, 0, 10, 200]
    got, want, state, want_state = scan_case(ops, torch.bfloat16, H, n, m, lens, rd, act, scale, decay=decay and list(decay),
                                             seed=n + m + segment, pos0=pos0, runs_from=8, segment=segment)
    bound = 1e-4
    assert float((got - want).abs().max()) <= bound * max(1.0, float(want.abs().max()))
    for slot, S in want_state.items():
        assert float((state[slot] - S).abs().max()) <= bound * max(1.0, float(S.abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
def test_fading_state_kernel_goes_on_from_a_state_and_is_the_same_however_cut(ops, dtype):
    H, n, m = 2, 16, 24
    got, want, _, _ = scan_case(ops, dtype, H, n, m, [7, 1, 12], rd=8, scale=0.25, pos0=[100, 0, 31], seed=3)
    assert float((got - want).abs().max()) <= 5e-5 * max(1.0, float(want.abs().max()))
    # one sequence whole, and the same rows in cuts of 1, 2 and 9 tokens: the same bits
    g = gen(9)
    T, ld = 40, 2 * H * n + H * m
    x = torch.randn(T, ld, generator=g).to(dtype).to(DEV)
    decay = torch.tensor([0.9, 0.999], dtype=torch.float32, device=DEV)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * torch.tensor(P.frequencies(8, 1e4), dtype=torch.float64)[None]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)

    def run(cuts):
        state = torch.zeros(2, H, n, m, device=DEV)
        outs, at = [], 0
        for c in cuts:
            outs.append(ops.linear_attention_scan(x[at:at + c], 0, H * n, 2 * H * n, H, n, m, decay, state, i32([0, c]), i32([1]),
                                                  i32(list(range(at, at + c))), 1, cos=cos, sin=sin, rotary_dim=8, key_scale=0.25))
            at += c
        return torch.cat(outs), state

    whole, s0 = run([T])
    cut, s1 = run([1, 2, 9, 1, 1, 8, 2, 16])
    assert torch.equal(whole, cut) and torch.equal(s0, s1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_key_and_a_query_of_the_fading_state_meet_hundreds_of_tokens_apart(ops, dtype):
    """With a decay of one (and one close to it) the key of token 3 still answers the query of token 603."""
    got, want, _, _ = scan_case(ops, dtype, 2, 16, 8, [610], decay=[1.0, 0.9995], seed=11, boost=(0, 3, 603))
    assert float(want[603].abs().max()) > 2 * float(want[600].abs().max())              # the meeting shows
    assert float((got - want).abs().max()) <= 1e-4 * float(want.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("joint,gate", [(True, "sigmoid"), (False, "silu"), (True, "silu"), (False, "sigmoid")])
def test_norm_and_gate_of_the_heads(ops, dtype, joint, gate):
    H, m, T = 3, 20, 6
    o = torch.randn(T, H * m, generator=gen(12)) * 4
    rows = torch.randn(T, 7 + H * m, generator=gen(13)).to(dtype)
    w = 1 + 0.3 * torch.randn(H * m, generator=gen(14))
    got = ops.gated_outnorm(o.to(DEV), rows.to(DEV), 7, w.to(DEV) if joint else None, 1e-5, H, m, joint, gate, dtype).cpu().double()
    od, z = o.double(), rows.double()[:, 7:]
    y = P.rms(od, 1e-5) * w.double() if joint else P.rms(od.reshape(T, H, m), 1e-5).reshape(T, H * m)
    want = y * (torch.sigmoid(z) if gate == "sigmoid" else P.silu(z))
    assert float((got - want).abs().max()) <= tol(dtype, want)


def tables(dims, base, P_max, freqs=None):
    f = freqs or P.frequencies(dims, base)
    ang = torch.arange(P_max, dtype=torch.float64)[:, None] * torch.tensor(f, dtype=torch.float64)[None]
    return torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV), f


def attention_case(ops, dtype, nh, nkv, d, vd, rd, chunk, T, page_size, seed, sink=True, turned=True, boost=None,
                   single_from=None, norm=True, cores=False):
    """Random q | k | v rows of one sequence through the cache write (head norms, turns, turned values) and attention
    over shuffled pages; the plain implementation's result beside it.  ``boost = (query position, key position)``: that
    key is made to stand out for that query.  ``single_from``: the rows from there on go one token a launch."""
    g = gen(seed)
    width = (nh + nkv) * d + nkv * vd
    x = torch.randn(T, width, generator=g)
    qw, kw = 1 + 0.2 * torch.randn(d, generator=g), 1 + 0.2 * torch.randn(d, generator=g)
    dev = (lambda w: w.to(DEV)) if norm else (lambda w: None)
    normed = (lambda z, w: P.rms(z, 1e-5) * w.double()) if norm else (lambda z, w: z)
    cos, sin, f = tables(rd, 1e4, T) if rd else (None, None, [])
    vcos, vsin, vf = tables(vd, 1e4, T) if turned else (None, None, [])
    pos = list(range(T))
    if boost is not None:
        # the key that, after its turn, points along the turned query of head 0 (no head norms: they would undo the scaling)
        assert not norm
        qi, kj = boost
        qn = P.turn(x[qi:qi + 1, :d].double(), [qi], f)
        x[kj, nh * d:nh * d + d] = P.turn(qn, [kj], f, sign=-1.0)[0].float() * 6.0
    x = x.to(dtype)
    blocks = -(-T // page_size)
    order = torch.randperm(blocks + 3, generator=g)[:blocks].to(torch.int32)
    kc = torch.full((blocks + 4, nkv, page_size, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((blocks + 4, nkv, page_size, vd), float("nan"), dtype=dtype, device=DEV)
    bt = order.reshape(1, blocks).to(DEV)
    rows = x.clone().to(DEV)
    cuts = [(0, T)] if single_from is None else [(0, single_from)] + [(t, t + 1) for t in range(single_from, T)]
    outs = []
    for a, b in cuts:
        part = rows[a:b].contiguous()
        seq = torch.zeros(b - a, dtype=torch.int32, device=DEV)
        ops.qknorm_rope_kv(part, dev(qw), dev(kw), 1e-5, cos, sin, rd, i32(pos[a:b]), seq, bt, page_size, kc, vc, nh, nkv, d,
                           vd=vd, vcos=vcos, vsin=vsin)
        if cores is True and b - a > 1:
            # the kernel on the matrix cores, in tiles of 16 queries, and the heads' sums turned back afterwards
            tiles = torch.tensor([[0] * len(range(0, b - a, 16)), list(range(0, b - a, 16)),
                                  [min(16, b - a - r) for r in range(0, b - a, 16)]], dtype=torch.int32, device=DEV)
            o = ops.attention_prefill(part, width, kc, vc, i32(pos[a:b]), tiles, bt, page_size, None, 0.3, nh, nkv, d, b - a,
                                      chunk=chunk, sink=sink)
            outs.append(ops.turn_heads(o, vcos, vsin, i32(pos[a:b]), nh, vd, sign=-1.0) if turned else o)
            continue
        if cores and b - a == 1:
            # a single token: the kernel for single queries, its keys in one part and in three
            o = ops.attention_decode(part, width, kc, vc, i32(pos[a:b]), bt, page_size, None, 0.3, nh, nkv, d, 1, 1 + 2 * (a % 2),
                                     chunk=chunk, sink=sink)
            outs.append(ops.turn_heads(o, vcos, vsin, i32(pos[a:b]), nh, vd, sign=-1.0) if turned else o)
            continue
        outs.append(ops.attention_generic(part, width, kc, vc, i32(pos[a:b]), seq, bt, page_size, None, 0.3, nh, nkv, d, b - a,
                                          vd=vd, chunk=chunk, sink=sink, vcos=vcos, vsin=vsin))
    got = torch.cat(outs).cpu().double()
    xd = x.double()
    q = P.turn(normed(xd[:, :nh * d].reshape(T, nh, d), qw), pos, f)
    k = P.turn(normed(xd[:, nh * d:(nh + nkv) * d].reshape(T, nkv, d), kw), pos, f)
    v = xd[:, (nh + nkv) * d:].reshape(T, nkv, vd)
    if turned:
        v = P.turn(v, pos, vf)
    if dtype == torch.bfloat16:
        q, k, v = P.to_bfloat16(q), P.to_bfloat16(k), P.to_bfloat16(v)
    if sink:
        o = P.chunked_sink_attention(q, k, v, 0.3, chunk)
    else:
        o = torch.zeros(T, nh, vd, dtype=torch.float64)
        for i in range(T):
            lo = 0 if not chunk else i - i % chunk
            for h in range(nh):
                o[i, h] = torch.softmax(0.3 * (k[lo:i + 1, h // (nh // nkv)] @ q[i, h]), 0) @ v[lo:i + 1, h // (nh // nkv)]
    if turned:
        o = P.turn(o, pos, vf, sign=-1.0)
    return got, o.reshape(T, nh * vd), v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,vd,rd,chunk,ps", [(4, 2, 24, 16, 16, 24, 8), (2, 2, 16, 8, 16, 7, 16), (3, 1, 12, 20, 0, 1, 4),
                                                     (6, 3, 10, 14, 6, 17, 16), (2, 1, 64, 64, 64, 64, 16), (1, 1, 8, 4, 4, None, 8),
                                                     (6, 1, 96, 40, 96, 32, 16)])
def test_attention_within_runs_with_a_sink_and_turned_values(ops, dtype, nh, nkv, d, vd, rd, chunk, ps):
    got, want, _ = attention_case(ops, dtype, nh, nkv, d, vd, rd, chunk, 75, ps, seed=d + vd)
    assert float((got - want).abs().max()) <= tol(dtype, want, 2e-5, 2e-2)
    got, want, _ = attention_case(ops, dtype, nh, nkv, d, vd, rd, chunk, 40, ps, seed=d, sink=False, turned=False)
    assert float((got - want).abs().max()) <= tol(dtype, want, 2e-5, 2e-2)
    got, want, _ = attention_case(ops, dtype, nh, nkv, d, vd, rd, chunk, 40, ps, seed=vd, sink=True, turned=False)
    assert float((got - want).abs().max()) <= tol(dtype, want, 2e-5, 2e-2)


@pytest.mark.parametrize("nh,nkv,d,rd,chunk,ps", [(4, 2, 64, 64, 64, 16), (2, 1, 128, 128, 128, 16), (8, 2, 32, 16, 24, 8),
                                                  (3, 3, 64, 0, 7, 4), (2, 1, 64, 64, None, 16), (6, 1, 32, 32, 100, 16)])
def test_attention_within_runs_on_the_matrix_cores(ops, nh, nkv, d, rd, chunk, ps):
    got, want, _ = attention_case(ops, torch.bfloat16, nh, nkv, d, d, rd, chunk, 150, ps, seed=d + nh, cores=True)
    assert float((got - want).abs().max()) <= tol(torch.bfloat16, want, 2e-5, 2e-2)
    got, want, _ = attention_case(ops, torch.bfloat16, nh, nkv, d, d, rd, chunk, 70, ps, seed=d, sink=False, turned=False, cores=True)
    assert float((got - want).abs().max()) <= tol(torch.bfloat16, want, 2e-5, 2e-2)
    # the last tokens one by one through the kernel for single queries
    got, want, _ = attention_case(ops, torch.bfloat16, nh, nkv, d, d, rd, chunk, 150, ps, seed=d + 1, cores=True, single_from=105)
    assert float((got - want).abs().max()) <= tol(torch.bfloat16, want, 2e-5, 2e-2)


@pytest.mark.parametrize("nh,nkv,d,rd,chunk,ps", [(4, 2, 16, 16, 24, 8), (2, 1, 16, 8, None, 16), (8, 1, 32, 32, 5, 4)])
def test_single_tokens_through_the_kernel_for_single_queries_at_narrow_heads(ops, nh, nkv, d, rd, chunk, ps):
    """Heads of 16 (and 32) in bfloat16: the prompt through the general kernel, the last 60 tokens one by one through
    the kernel for single queries, with runs, the sink and turned values."""
    got, want, _ = attention_case(ops, torch.bfloat16, nh, nkv, d, d, rd, chunk, 130, ps, seed=7 * d + nh, cores="single", single_from=70)
    assert float((got - want).abs().max()) <= tol(torch.bfloat16, want, 2e-5, 2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk,ps", [(24, 8), (21, 8), (32, 16), (None, 16)])
def test_a_key_that_stands_out_is_found_at_the_edges_of_runs_and_pages_and_far_back(ops, dtype, chunk, ps):
    """The key is put at the first position of the query's run (seen: the head's output is that value, turned back),
    at the last position of the run before (not seen), on a page's last and first row, and, without runs, 300 tokens
    back; the query in a launch of many and in a launch of its own."""
    T = 340
    qi = 333
    start = qi - qi % chunk if chunk else 0
    places = {start: True, qi: True, (qi // ps) * ps: None, (qi // ps) * ps - 1: None}
    if chunk:
        places[start - 1] = False
        places[start - chunk] = False
    else:
        places[qi - 300] = True
        places[3] = True
    for kj, seen in places.items():
        if kj < 0 or kj > qi:
            continue
        if seen is None:
            seen = kj >= start
        for single_from in (None, qi - 2):
            got, want, v = attention_case(ops, dtype, 2, 1, 16, 12, 8, chunk, T, ps, seed=kj, boost=(qi, kj),
                                          single_from=single_from, norm=False)
            assert float((got - want).abs().max()) <= tol(dtype, want, 3e-5, 3e-2), (kj, single_from)
            # what the head would put out if that key took all the weight
            alone = P.turn(v[kj:kj + 1, 0], [qi], P.frequencies(12, 1e4), sign=-1.0)[0]
            near = float((got[qi, :12] - alone).abs().max()) <= 0.05 * float(alone.abs().max())
            assert near == seen, (kj, single_from)
        if dtype == torch.bfloat16:
            # the same through the kernel on the matrix cores (keys and values 32 wide)
            for single_from in (None, qi - 2):
                got, want, v = attention_case(ops, dtype, 2, 1, 32, 32, 16, chunk, T, ps, seed=kj, boost=(qi, kj), norm=False,
                                              cores=True, single_from=single_from)
                assert float((got - want).abs().max()) <= tol(dtype, want, 3e-5, 3e-2), (kj, single_from)
                alone = P.turn(v[kj:kj + 1, 0], [qi], P.frequencies(32, 1e4), sign=-1.0)[0]
                assert (float((got[qi, :32] - alone).abs().max()) <= 0.05 * float(alone.abs().max())) == seen, (kj, single_from)


# ------------------------------------------------------------------ the mixers alone, with their own caches

def linear_spec(kind, W, H, n, m, decay, rd=0, base=1e4, max_position=512):
    from gesso_amd.config import LinearAttentionSpec, NoPositionSpec, RopeSpec
    pos = RopeSpec(head_dim=n, rotary_dim=rd, theta=base, max_position=max_position) if rd else NoPositionSpec()
    if kind == "lightning":
        return LinearAttentionSpec(hidden=W, n_heads=H, key_dim=n, value_dim=m, decay=tuple(decay), eps=1e-5,
                                   activation="silu", out_norm="joint", gate="sigmoid")
    return LinearAttentionSpec(hidden=W, n_heads=H, key_dim=n, value_dim=m, decay=tuple(decay), eps=1e-5, position=pos,
                               key_scale=n ** -0.5, out_norm="head", gate="silu")


def left_spec(W, nh, nkv, d, vd, rd, chunk, stretch=True, base=1e4, max_position=512):
    from gesso_amd.config import AttentionSpec, NoPositionSpec, RMSNormSpec, RopeSpec, StretchedRopeSpec
    if not rd:
        pos = NoPositionSpec()
    elif stretch:
        pos = StretchedRopeSpec(head_dim=d, rotary_dim=rd, theta=base, max_position=max_position, factor=4.0, original=64.0,
                                low=1.0, high=4.0)
    else:
        pos = RopeSpec(head_dim=d, rotary_dim=rd, theta=base, max_position=max_position)
    return AttentionSpec(hidden=W, n_heads=nh, n_kv_heads=nkv, head_dim=d, position=pos, qk_norm=RMSNormSpec(size=d, eps=1e-5),
                         scale=0.2, value_dim=vd, chunk=chunk, sink=True,
                         value_position=RopeSpec(head_dim=vd, rotary_dim=vd, theta=base, max_position=max_position) if rd else None)


_LOCAL = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate_proj.weight": "g", "out_proj.weight": "o",
          "out_norm.weight": "norm", "q_norm.weight": "q.norm", "k_norm.weight": "k.norm"}


def stored(tensors, prefix="m"):
    out = {}
    for k, v in tensors.items():
        if k.startswith(("left.", "right.")):
            side, local = k.split(".", 1)
            out[f"{prefix}.{side}.{_LOCAL[local]}"] = v
        else:
            out[f"{prefix}.{_LOCAL[k]}"] = v
    return out


def harness(kind, dtype, page_size=8, num_pages=64, **kw):
    """A mixer with its own cache, and the plain implementation of it on whole sequences."""
    from gesso_amd.config import MixerPairSpec
    from test_gpu_parts import Harness
    W = kw.get("W", 96)
    if kind in ("lightning", "retention"):
        H, n, m, decay, rd = kw.get("H", 3), kw.get("n", 24), kw.get("m", 16), kw.get("decay", (0.5, 0.9, 0.99)), kw.get("rd", 0)
        spec = linear_spec(kind, W, H, n, m, decay, rd)
        mx = {"heads": H, "dim": n, "vdim": m, "decay": list(decay), "rot": {"base": 1e4, "dims": rd} if rd else None}
        h = Harness("mixer", spec, dtype, seed=kw.get("seed", 5), page_size=page_size, num_pages=num_pages, std=0.25)
        w = stored(h.tensors)
        if kind == "lightning":
            return h, lambda x: P.lightning(x.double(), w, "m", mx, 1e-5)
        return h, lambda x: P.right_branch(x.double(), w, "m", mx, 1e-5, list(range(x.shape[0])))
    nh, nkv, d, vd, rd, chunk = (kw.get(k, v) for k, v in (("nh", 4), ("nkv", 2), ("d", 24), ("vd", 16), ("rd", 16), ("chunk", 24)))
    left = left_spec(W, nh, nkv, d, vd, rd, chunk)
    lmx = {"heads": nh, "kv_heads": nkv, "dim": d, "vdim": vd, "scale": 0.2, "mask": {"size": chunk} if chunk else None,
           "rot": {"base": 1e4, "dims": rd, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64.0}} if rd else None}
    if kind == "left":
        h = Harness("mixer", left, dtype, seed=kw.get("seed", 6), page_size=page_size, num_pages=num_pages, std=0.25)
        w = stored(h.tensors)
        return h, lambda x: P.left_branch(x.double(), w, "m", lmx, 1e-5, list(range(x.shape[0])))
    right = linear_spec("retention", W, 2, 16, 24, (0.9, 0.97), 8)
    rmx = {"heads": 2, "dim": 16, "vdim": 24, "decay": [0.9, 0.97], "rot": {"base": 1e4, "dims": 8}}
    spec = MixerPairSpec(left=left, right=right, left_scale=1.3, right_scale=0.8)
    h = Harness("mixer", spec, dtype, seed=kw.get("seed", 7), page_size=page_size, num_pages=num_pages, std=0.25)
    w = stored(h.tensors)
    mx = {"left": lmx, "right": rmx, "left_scale": 1.3, "right_scale": 0.8}
    return h, lambda x: P.parallel(x.double(), w, "m", mx, 1e-5, list(range(x.shape[0])))


CASES = [("lightning", dict()), ("lightning", dict(H=1, n=40, m=48, decay=(0.95,), W=64)),
         ("lightning", dict(H=2, n=64, m=64, decay=(0.97, 0.999), W=128)),
         ("retention", dict(H=2, n=16, m=24, decay=(0.9, 0.97), rd=8)), ("retention", dict(H=5, n=6, m=10, decay=(0.5, 0.8, 0.9, 0.95, 1.0), rd=2, W=100)),
         ("retention", dict(H=1, n=24, m=8, decay=(0.0,), rd=0, W=64)),
         ("left", dict()), ("left", dict(nh=2, nkv=2, d=16, vd=8, rd=16, chunk=7, W=64)), ("left", dict(nh=3, nkv=1, d=12, vd=20, rd=0, chunk=1, W=64)),
         ("left", dict(nh=6, nkv=3, d=10, vd=14, rd=6, chunk=17, W=100, page_size=16)), ("left", dict(nh=2, nkv=1, d=18, vd=6, rd=18, chunk=None, W=100)),
         ("left", dict(nh=2, nkv=1, d=64, vd=64, rd=64, chunk=32, W=128, page_size=16)),
         ("pair", dict()), ("pair", dict(chunk=16, page_size=16))]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,kw", CASES)
def test_mixers_whole_token_by_token_in_portions_and_in_batches(dtype, kind, kw):
    kw = dict(kw)
    ps = kw.pop("page_size", 8)
    h, plain = harness(kind, dtype, page_size=ps, **kw)
    W = kw.get("W", 96)
    T = 90
    x = torch.randn(T, W, generator=gen(40)).to(dtype)
    want = plain(x)
    bound = tol(dtype, want, 5e-5, 3e-2)
    whole = h.mixer(x, [("whole", T)])
    assert float((whole - want).abs().max()) <= bound
    # most of it at once, the rest token by token (runs end and begin among the decoded tokens)
    head = 40
    got = [h.mixer(x[:head], [("tail", head)])] + [h.mixer(x[i:i + 1], [("tail", 1)]) for i in range(head, T)]
    assert float((torch.cat(got) - want).abs().max()) <= bound
    # the first tokens one by one from an empty cache
    got = [h.mixer(x[i:i + 1], [("first", 1)]) for i in range(6)]
    assert float((torch.cat(got) - want[:6]).abs().max()) <= bound
    # portions of several sizes, down to two tokens
    at, got = 0, []
    for size in (2, 7, 2, 13, 3, 16, 5, 2, 31, 9):
        size = min(size, T - at)
        if size:
            got.append(h.mixer(x[at:at + size], [("cut", size)]))
            at += size
    assert at == T and float((torch.cat(got) - want).abs().max()) <= bound
    for rid in ("whole", "tail", "first", "cut"):
        h.manager.release(rid)
    # unequal requests side by side: a single token of one, a portion of another, a whole short one
    y = torch.randn(30, W, generator=gen(41)).to(dtype)
    u = torch.randn(5, W, generator=gen(42)).to(dtype)
    h.mixer(y[:29], [("b", 29)])
    h.mixer(x[:50], [("a", 50)])
    out = h.mixer(torch.cat([y[29:30], x[50:70], u]), [("b", 1), ("a", 20), ("c", 5)])
    assert float((out[0] - plain(y)[29]).abs().max()) <= bound
    assert float((out[1:21] - want[50:70]).abs().max()) <= bound
    assert float((out[21:] - plain(u)).abs().max()) <= bound


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["lightning", "left", "pair"])
def test_mixers_with_pages_and_slots_freed_and_used_again(dtype, kind):
    """A pool that holds little more than one request's run, and four slots: requests come and go, every later one
    writes pages and a slot that an earlier one gave back (filled with NaN in between)."""
    h, plain = harness(kind, dtype, page_size=8, num_pages=6)
    for i, T in enumerate((60, 35, 64, 9, 50, 20)):
        x = torch.randn(T, 96, generator=gen(50 + i)).to(dtype)
        want = plain(x)
        at, got = 0, []
        while at < T:
            size = min((11, 2, 1, 16)[(at + i) % 4], T - at)
            got.append(h.mixer(x[at:at + size], [(i, size)]))
            at += size
        assert float((torch.cat(got) - want).abs().max()) <= tol(dtype, want, 5e-5, 3e-2), i
        h.manager.release(i)
        for pool in h.storage.keys + h.storage.values:
            pool[:, :-1].fill_(float("nan"))
        for pool, _ in h.storage.state_pools:
            pool[:, :-1].fill_(float("nan"))


@pytest.mark.parametrize("dtype", DTYPES)
def test_dense_feed_forward_with_biases(dtype):
    from gesso_amd.config import GatedMLPSpec
    from test_gpu_parts import Harness
    for W, F, M in ((96, 80, 7), (100, 36, 70), (128, 256, 200)):
        h = Harness("ffn", GatedMLPSpec(hidden=W, intermediate=F), dtype, seed=F, std=0.2)
        t = h.tensors
        w = {"f.gate": t["gate.weight"], "f.gate.b": t["gate.bias"], "f.up": t["up.weight"], "f.up.b": t["up.bias"],
             "f.down": t["down.weight"], "f.down.b": t["down.bias"]}
        x = torch.randn(M, W, generator=gen(60)).to(dtype)
        got = h.part.forward(x.to(DEV), None).double().cpu()
        want = P.dense_ff(x.double(), w, "f")
        assert float((got - want).abs().max()) <= tol(dtype, want, 3e-5, 2e-2)
        one = h.part.forward(x[3:4].to(DEV), None).double().cpu()
        assert float((one - want[3:4]).abs().max()) <= tol(dtype, want, 3e-5, 2e-2)


# ------------------------------------------------------------------ whole models

LENGTHS = {"A": (1, 23, 70, 130), "B": (2, 40, 77), "C": (5, 64, 150, 300), "D": (3, 52, 110)}


def sequences(name):
    cfg, seed = CONFIGS[name]
    return {f"s{i}": random_ids(n, cfg.vocab, 100 * seed + i) for i, n in enumerate(LENGTHS[name])}


def four_ways(seqs, seed, tail=48):
    ways = {"whole": R.trace_whole, "tail": lambda s: R.trace_tail(s, tail=tail), "portions": R.trace_portions,
            "mixed": lambda s: R.trace_mixed(s, seed=seed)}
    big = R.Trace()
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            big.steps.append(dict(rec, step=len(big.steps)))
            big.rows.append(rows)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    return ways, big


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_replay_four_ways(name, dtype, folders, tmp_path):
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences(name)
    plain = R.Plain(model_dir, seqs, dtype)
    ways, big = four_ways(seqs, 5)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab)
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        plain.check(mine, f"Fazezen {name} {way}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_token_by_token(name, dtype, folders, tmp_path):
    """A short prompt, then three hundred tokens one by one: states carried and runs begun and ended many times over."""
    cfg, seed = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = {"long": random_ids(330, cfg.vocab, 7000 + seed), "other": random_ids(301, cfg.vocab, 7100 + seed)}
    plain = R.Plain(model_dir, seqs, dtype)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), R.trace_tail(seqs, tail=300), cfg.vocab)
    assert rc == 0 and {k: len(v) for k, v in got.items()} == {"long": 330, "other": 301}
    plain.check(got, f"Fazezen {name}, 300 tokens one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_with_pages_of_eight_given_back_poisoned(dtype, folders, tmp_path):
    cfg, _ = CONFIGS["A"]
    model_dir = write_tiny(folders, "A", torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences("A")
    plain = R.Plain(model_dir, seqs, dtype)
    for way, make in (("portions", lambda s: R.trace_portions(s, sizes=(13, 2, 8, 3))), ("mixed", lambda s: R.trace_mixed(s, seed=9))):
        got, rc = R.run_trace(model_dir, dtype, str(tmp_path / way), make(seqs), cfg.vocab, page_size=8, extra=["--poison"])
        assert rc == 0
        plain.check(got, f"Fazezen A, pages of 8, poisoned, {way}")


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_session(name, folders):
    """Prompts of unequal length generated together through the scheduler (prefill in portions, then the decode loop),
    far enough for runs to end and begin among generated tokens; float32 must give the plain model's tokens."""
    from gesso_amd import Session
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32)
    pc, pw = P.read_config(model_dir), P.read_weights(model_dir)
    prompts = [random_ids(n, cfg.vocab, 900 + n) for n in (3, 41, 18)]
    new = 70
    want = [P.greedy(pc, pw, p, new) for p in prompts]
    session = Session(model_dir, dtype="float32", device=DEV, context_length=256, chunk_size=16)
    try:
        assert session.generate(prompts, max_new_tokens=new) == want
        assert session.generate([prompts[1]], max_new_tokens=new)[0] == want[1]
    finally:
        session.close()
    session = Session(write_tiny(folders, name, torch.bfloat16), dtype="bfloat16", device=DEV, context_length=256)
    try:
        got = session.generate(prompts, max_new_tokens=new)
        assert [len(g) for g in got] == [len(w) for w in want]
        # every token bfloat16 chose is one the plain model ranks close to its best at that place
        from noise import supported
        pw16 = P.read_weights(write_tiny(folders, name, torch.bfloat16))
        for g, p in zip(got, prompts):
            lg = P.forward(pc, pw16, g).numpy()
            assert all(supported(lg[i - 1], g[i], 0.5) for i in range(len(p), len(g)))
    finally:
        session.close()


def test_the_command_line_serves_a_fazezen_folder(folders):
    import json
    import os
    import subprocess
    import sys
    cfg, _ = CONFIGS["D"]
    model_dir = write_tiny(folders, "D", torch.float32)
    prompt = random_ids(19, cfg.vocab, 77)
    want = P.greedy(P.read_config(model_dir), P.read_weights(model_dir), prompt, 24)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "gesso_amd", "--model", model_dir, "--dtype", "float32", "--prompt-ids",
                        ",".join(str(t) for t in prompt), "--max-new-tokens", "24", "--n-ctx", "128"],
                       capture_output=True, text=True, cwd=root, timeout=240, env=dict(os.environ, PYTHONPATH=root))
    assert r.returncode == 0, r.stderr[-2000:]
    assert json.loads(r.stdout.strip().splitlines()[-1])["ids"] == [want]


def test_seventy_requests_at_once_decode_through_the_loop_for_many_rows(folders):
    """More requests than the weight-streaming products take rows: the recorded loop over the many-row kernels, seventy
    states and block tables side by side.  Every token chosen is one the plain model ranks near its best at that place,
    and so is every token the first request gets when it runs alone."""
    from gesso_amd import Session
    from noise import supported
    cfg, _ = CONFIGS["C"]
    model_dir = write_tiny(folders, "C", torch.bfloat16)
    pc, pw = P.read_config(model_dir), P.read_weights(model_dir)
    prompts = [random_ids(3 + (7 * i) % 40, cfg.vocab, 2000 + i) for i in range(70)]
    session = Session(model_dir, dtype="bfloat16", device=DEV, context_length=128, max_num_seqs=128)
    try:
        got = session.generate(prompts, max_new_tokens=12)
        alone = session.generate([prompts[0]], max_new_tokens=12)[0]
    finally:
        session.close()
    assert [len(g) for g in got] == [len(p) + 12 for p in prompts]
    for i in (0, 33, 69):
        lg = P.forward(pc, pw, got[i]).numpy()
        assert all(supported(lg[j - 1], got[i][j], 0.5) for j in range(len(prompts[i]), len(got[i]))), i
    lg = P.forward(pc, pw, alone).numpy()
    assert all(supported(lg[j - 1], alone[j], 0.5) for j in range(len(prompts[0]), len(alone)))


def random_fazezen(seed: int):
    """A configuration drawn from a seed: two to four layers of either kind in any order, sizes with and without whole
    tiles, runs shorter and longer than the sequences or none, turns over a part of a head, all of it or none, layers
    without a feed-forward."""
    import random
    from gesso_amd.config import (ChunkedAttentionConfig, DenseConfig, FazezenConfig, FazezenLayer, LightningConfig,
                                  ParallelConfig, RetentionConfig, Rotation, Stretch)
    rng = random.Random(seed)

    def decays(n):
        # no decay of 0 here: such a head puts out (q . k) v, and the norm that follows turns a q . k near zero into a
        # sign, which one rounding flips; the bound made from another set of roundings then says nothing (the tiny
        # configuration B keeps such a head, with keys wide enough)
        return tuple(rng.choice([0.5, 0.9, 0.97, 0.99, 0.999, 1.0]) for _ in range(n))

    def rot(dim, stretch):
        if rng.random() < 0.15:
            return None
        dims = rng.choice([d for d in (2, 4, 8, 16, 32, 64) if d <= dim] + [dim - dim % 2])
        s = Stretch(rng.choice([2.0, 4.0, 8.0]), rng.choice([1.0, 2.0]), rng.choice([4.0, 6.0]), rng.choice([16.0, 64.0, 256.0]))
        return Rotation(rng.choice([1e2, 1e4, 1e6]), dims, s if stretch and rng.random() < 0.6 else None)

    layers = []
    for _ in range(rng.randint(2, 4)):
        ff = None if rng.random() < 0.2 else DenseConfig(rng.choice([8, 24, 40, 64, 130]))
        if rng.random() < 0.5:
            H = rng.choice([1, 2, 3, 4])
            layers.append(FazezenLayer("lightning", LightningConfig(H, rng.choice([4, 12, 16, 32, 64]),
                                                                    rng.choice([4, 10, 16, 32, 64, 80]), decays(H)), ff))
        else:
            nkv = rng.choice([1, 2, 3])
            d, vd = rng.choice([4, 8, 12, 16, 32, 64]), rng.choice([2, 4, 8, 16, 20, 32, 64])
            left = ChunkedAttentionConfig(nkv * rng.choice([1, 2, 3]), nkv, d, vd, rng.choice([0.08, 0.15, 0.3]), rot(d, True),
                                          rng.choice([None, 1, 3, 16, 33, 64, 150]))
            H, rd = rng.choice([1, 2, 4]), rng.choice([4, 8, 16, 32])
            right = RetentionConfig(H, rd, rng.choice([4, 8, 16, 24, 64, 72]), decays(H), rot(rd, False))
            layers.append(FazezenLayer("parallel", ParallelConfig(left, right, rng.choice([0.5, 1.0, 1.2]), rng.choice([0.7, 1.0, 1.5])), ff))
    return FazezenConfig(vocab=rng.choice([97, 200, 333, 512]), width=rng.choice([64, 72, 96, 128, 160]), layers=tuple(layers),
                         norm_eps=rng.choice([1e-5, 1e-6, 1e-4]), max_position=512)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [51, 52, 53, 54, 55, 56])
def test_replay_of_configurations_drawn_at_random(seed, dtype, tmp_path):
    import random
    from gesso_amd.weights import write_model_folder
    cfg = random_fazezen(seed)
    rng = random.Random(seed)
    model_dir = write_model_folder(str(tmp_path / "m"), cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16,
                                   std=STD)
    lens = [rng.randint(1, 4), rng.randint(20, 60), rng.randint(70, 120), rng.randint(130, 210)]
    seqs = {f"s{i}": random_ids(n, cfg.vocab, seed * 10 + i) for i, n in enumerate(lens)}
    plain = R.Plain(model_dir, seqs, dtype)
    ways, big = four_ways(seqs, seed, tail=40)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab, extra=["--poison"])
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        plain.check(mine, f"Fazezen drawn from {seed}, {way}")
