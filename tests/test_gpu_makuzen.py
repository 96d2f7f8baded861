"""Makuzen on the GPU against the plain implementation: each kernel alone, the mixer and the feed-forward alone with
their own cache (whole, token by token, in portions, in unequal batches, with pages used again), whole models replayed
in the four ways of cutting, and greedy generation through the session and its scheduler.

Where random weights would hide a fault, the inputs are made so that it shows: one cached row is scaled so that its
score stands out, and it is put far back, on a page's first and last row, and just inside and just outside the window.
"""
import math

import numpy as np
import pytest
import torch

import plain_makuzen as P
import replay as R
from tiny import random_ids
from tiny_makuzen import CONFIGS, STD, write_tiny

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def gen(seed):
    return torch.Generator().manual_seed(seed)


def tol(dtype, ref, f32=2e-5, bf16=1e-2):
    return (f32 if dtype == torch.float32 else bf16) * max(1.0, float(ref.abs().max()))


@pytest.fixture(scope="module")
def ops():
    from gesso_amd.kernels import ops
    ops.lib()
    return ops


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return str(tmp_path_factory.mktemp("makuzen"))


# ------------------------------------------------------------------ kernels alone

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [100, 256, 1030])
def test_norm_scaled_add(ops, dtype, H):
    res = torch.randn(5, H, generator=gen(0))
    y = (torch.randn(5, H, generator=gen(1)) * 3).to(dtype)
    w = 1 + 0.2 * torch.randn(H, generator=gen(2))
    r = res.clone().to(DEV)
    rows = ops.norm_scaled_add(r, y.to(DEV), w.to(DEV), 1e-4, 0.6, None if dtype == torch.float32 else dtype)
    want = res.double() + 0.6 * P.rmsnorm(y.double(), w.double(), 1e-4)
    assert float((r.cpu().double() - want).abs().max()) <= 2e-6 * float(want.abs().max())
    if dtype == torch.float32:
        assert rows is None
    else:
        assert torch.equal(rows.cpu(), r.cpu().to(dtype))
        only = ops.norm_scaled_add(r, None, None, 0.0, 0.0, dtype)
        assert torch.equal(only.cpu(), r.cpu().to(dtype))


def paged(rows, page_size, num_pages, seed, dtype):
    """Rows ``(T, D)`` of one sequence scattered over pages in a random order: the pool and the block table."""
    T, D = rows.shape
    blocks = -(-T // page_size)
    order = torch.randperm(num_pages, generator=gen(seed))[:blocks].to(torch.int32)
    pool = torch.full((num_pages + 1, 1, page_size, D), float("nan"), dtype=dtype)
    for t in range(T):
        pool[int(order[t // page_size]), 0, t % page_size] = rows[t].to(dtype)
    return pool, order.reshape(1, blocks)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("qr,c,r", [(40, 48, 8), (28, 36, 6), (64, 128, 32), (20, 40, 0)])
def test_latent_prep_norms_rotates_and_writes_the_cache_row(ops, dtype, qr, c, r):
    T, ps, extra = 21, 8, 5
    down = (torch.randn(T, qr + c + r + extra, generator=gen(3)) * 2).to(dtype)
    qw, kw = 1 + 0.1 * torch.randn(qr, generator=gen(4)), 1 + 0.1 * torch.randn(c, generator=gen(5))
    freqs, mult = P.yarn_frequencies(r, 1e4, {"factor": 2.0, "original": 16.0, "fast": 4.0, "slow": 1.0}) if r else ([], 1.0)
    start = 37                                                # the rows stand at positions 37.. of their sequence
    pos = torch.arange(start, start + T, dtype=torch.int32)
    ang = torch.arange(start + T, dtype=torch.float64)[:, None] * torch.tensor(freqs, dtype=torch.float64)[None, :]
    cos, sin = (torch.cos(ang) * mult).float(), (torch.sin(ang) * mult).float()
    pool, table = paged(torch.zeros(start + T, c + r), ps, 12, 6, dtype)
    pool_d = pool.to(DEV)
    a = ops.latent_prep(down.to(DEV), 0, qr, qr, c, r, qw.to(DEV), kw.to(DEV), 1e-5, cos.to(DEV) if r else None,
                        sin.to(DEV) if r else None, pos.to(DEV), torch.zeros(T, dtype=torch.int32, device=DEV),
                        table.to(DEV), ps, pool_d)
    d = down.double()
    want_a = P.rmsnorm(d[:, :qr], qw.double(), 1e-5)
    want_z = P.rmsnorm(d[:, qr:qr + c], kw.double(), 1e-5)
    want_k = P.rotate(d[:, qr + c:qr + c + r], pos.tolist(), freqs, mult) if r else d[:, :0]
    assert float((a.cpu().double() - want_a).abs().max()) <= tol(dtype, want_a, 2e-6, 4e-3)
    got = torch.stack([pool_d[int(table[0, p // ps]), 0, p % ps] for p in pos.tolist()]).cpu().double()
    want = torch.cat([want_z, want_k], 1)
    assert float((got - want).abs().max()) <= tol(dtype, want, 4e-6, 4e-3)
    # nothing else was written: rows before the step's first position keep what they held
    before = torch.stack([pool_d[int(table[0, p // ps]), 0, p % ps] for p in range(start)]).cpu()
    assert torch.equal(before, torch.zeros_like(before))


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_q_rot_puts_the_rotated_part_behind_the_absorbed_one(ops, dtype):
    T, H, n, r, c = 9, 3, 12, 6, 20
    q = torch.randn(T, H * (n + r), generator=gen(7)).to(dtype)
    freqs, mult = P.yarn_frequencies(r, 500.0, None)
    pos = torch.tensor([0, 1, 2, 50, 51, 7, 300, 301, 302], dtype=torch.int32)
    ang = torch.arange(320, dtype=torch.float64)[:, None] * torch.tensor(freqs, dtype=torch.float64)[None, :]
    qa = torch.zeros(T, H * (c + r), dtype=dtype, device=DEV)
    ops.latent_q_rot(q.to(DEV), H, n, r, c, torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV), pos.to(DEV), qa)
    got = qa.cpu().double().reshape(T, H, c + r)
    want = P.rotate(q.double().reshape(T, H, n + r)[:, :, n:], pos.tolist(), freqs, mult)
    assert float(got[:, :, :c].abs().max()) == 0.0
    assert float((got[:, :, c:] - want).abs().max()) <= tol(dtype, want, 2e-6, 4e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,H,N,K", [(1, 3, 48, 24), (70, 5, 20, 36), (130, 2, 64, 130), (9, 1, 7, 3), (8, 4, 64, 32),
                                     (200, 3, 40, 72), (33, 2, 16, 8), (64, 16, 512, 128), (65, 2, 128, 512)])
def test_heads_product_with_and_without_gate(ops, dtype, M, H, N, K):
    x = torch.randn(M, H * K + 8, generator=gen(8)).to(dtype)      # (rows of whole 16-byte pieces where H K allows)
    w = (torch.randn(H, N, K, generator=gen(9)) / math.sqrt(K)).to(dtype)
    g = torch.randn(M, H + 2, generator=gen(10)).to(dtype)
    for gate in (None, g):
        y = torch.zeros(M, H * N + 5, dtype=dtype, device=DEV)
        ops.heads_product(x.to(DEV), K, w.to(DEV), y, N, K, gate=None if gate is None else gate.to(DEV)[:, 1:])
        want = torch.einsum("mhk,hnk->mhn", x.double()[:, :H * K].reshape(M, H, K), w.double())
        if gate is not None:
            want = want * torch.sigmoid(gate.double()[:, 1:1 + H])[:, :, None]
        got = y.cpu().double()
        assert float(got[:, H * N:].abs().max()) == 0.0
        assert float((got[:, :H * N].reshape(M, H, N) - want).abs().max()) <= tol(dtype, want, 2e-6, 4e-3)


def latent_case(T, H, n, r, dv, c, seed, dtype):
    """Cached rows, queries and the up-projections of a single sequence, as float64 (rounded to ``dtype``)."""
    g = gen(seed)
    rnd = lambda *s: torch.randn(*s, generator=g).to(dtype).double()
    return dict(z=rnd(T, c), k_rot=rnd(T, r), q_plain=rnd(T, H, n), q_rot=rnd(T, H, r),
                uk=(rnd(H, n, c) / math.sqrt(c)), uv=(rnd(H, dv, c) / math.sqrt(c)))


def attend_both(ops, case, scale, window, dtype, page_size, rows, seed=0, cores=False):
    """``rows``: the positions whose queries are run (one launch).  Returns the kernel's latent output mapped through
    W_uv, and the plain attention's, ``(len(rows), H, dv)`` each."""
    z, k_rot, qp, qr, uk, uv = (case[k] for k in ("z", "k_rot", "q_plain", "q_rot", "uk", "uv"))
    T, c = z.shape
    H, r = qp.shape[1], k_rot.shape[1]
    k_plain = torch.einsum("hnc,tc->thn", uk, z)
    v = torch.einsum("hdc,tc->thd", uv, z)
    want = P.windowed_attention(qp, qr, k_plain, k_rot, v, scale, window)[rows]
    qa = torch.cat([torch.einsum("thn,hnc->thc", qp, uk), qr], 2)[rows].reshape(len(rows), H * (c + r))
    pool, table = paged(torch.cat([z, k_rot], 1), page_size, -(-T // page_size) + 3, seed, dtype)
    positions = torch.tensor(rows, dtype=torch.int32, device=DEV)
    if cores:
        # consecutive positions form tiles of as many tokens as a block takes; the rest are tiles of one token
        most, tiles, at = ops.attention_latent_mfma_tokens(H), [], 0
        while at < len(rows):
            n = 1
            while at + n < len(rows) and n < most and rows[at + n] == rows[at + n - 1] + 1:
                n += 1
            tiles.append((0, at, n))
            at += n
        tiles = torch.tensor(tiles, dtype=torch.int32).T.contiguous().to(DEV)
        o = ops.attention_latent_mfma(qa.to(dtype).to(DEV), pool.to(DEV), positions, tiles, table.to(DEV), page_size,
                                      window, scale, H, c, r, len(rows))
    else:
        o = ops.attention_latent(qa.to(dtype).to(DEV), pool.to(DEV), positions,
                                 torch.zeros(len(rows), dtype=torch.int32, device=DEV), table.to(DEV), page_size, window,
                                 scale, H, c, r, len(rows))
    got = torch.einsum("thc,hdc->thd", o.cpu().double().reshape(len(rows), H, c), uv)
    return got, want


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,n,r,dv,c,window,ps", [(3, 24, 8, 16, 48, 24, 8), (5, 12, 6, 20, 36, 17, 16), (2, 16, 0, 8, 32, None, 4),
                                                  (4, 32, 32, 32, 64, 40, 16), (1, 8, 2, 4, 200, 1, 8)])
def test_attention_over_latent_rows_equals_attention_over_keys_and_values(ops, dtype, H, n, r, dv, c, window, ps):
    T = 150
    case = latent_case(T, H, n, r, dv, c, 11, dtype)
    rows = list(range(T))
    got, want = attend_both(ops, case, 0.3 / math.sqrt(n + r), window, dtype, ps, rows)
    assert float((got - want).abs().max()) <= tol(dtype, want, 1e-5, 2e-2)
    single, _ = attend_both(ops, case, 0.3 / math.sqrt(n + r), window, dtype, ps, [T - 1])
    assert float((single[0] - want[-1]).abs().max()) <= tol(dtype, want, 1e-5, 2e-2)
    if dtype == torch.bfloat16 and ops.attention_latent_mfma_supports(H, c, r):
        got, _ = attend_both(ops, case, 0.3 / math.sqrt(n + r), window, dtype, ps, rows, cores=True)
        assert float((got - want).abs().max()) <= tol(dtype, want, 1e-5, 2e-2)
        some = [0, 1, 2, 40, 41, 97, T - 2, T - 1]
        got, _ = attend_both(ops, case, 0.3 / math.sqrt(n + r), window, dtype, ps, some, cores=True)
        assert float((got - want[some]).abs().max()) <= tol(dtype, want, 1e-5, 2e-2)


@pytest.mark.parametrize("H,n,r,dv,c,window,ps", [(70, 8, 8, 8, 16, 30, 16), (16, 64, 64, 32, 512, 100, 16), (6, 32, 16, 32, 256, None, 8),
                                                  (3, 16, 24, 8, 112, 7, 32)])
def test_attention_over_latent_rows_on_the_matrix_cores_at_other_sizes(ops, H, n, r, dv, c, window, ps):
    """More heads than a block takes, the widest latent, values in seven tiles, pages longer than the window."""
    T, dtype = 200, torch.bfloat16
    assert ops.attention_latent_mfma_supports(H, c, r)
    case = latent_case(T, H, n, r, dv, c, 13, dtype)
    scale = 0.3 / math.sqrt(n + r)
    got, want = attend_both(ops, case, scale, window, dtype, ps, list(range(T)), cores=True)
    assert float((got - want).abs().max()) <= tol(dtype, want, 1e-5, 2e-2)
    got, _ = attend_both(ops, case, scale, window, dtype, ps, [T - 1], cores=True)
    assert float((got[0] - want[-1]).abs().max()) <= tol(dtype, want, 1e-5, 2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,ps", [(24, 8), (21, 8), (33, 16), (None, 16)])
def test_a_row_that_stands_out_is_found_far_back_at_page_borders_and_just_inside_the_window(ops, dtype, window, ps):
    """One cached row is made to take nearly all of a query's weight when it is seen (its latent is the query's absorbed
    form, scaled up).  Seen: the output is that row's value.  Just outside the window: it is not.  The place is put on a
    page's last and first row, at the window's oldest place, one older than that, and (without a window) 300 back."""
    T, H, n, r, dv, c = 340, 2, 16, 8, 8, 32
    query = T - 1
    edge = query - window + 1 if window else None
    places = [query, query - 1, (query // ps) * ps, (query // ps) * ps - 1]
    places += [edge, edge + 1, edge - 1, edge - 2] if window else [query - 300, 0, ps - 1, ps]
    for place in places:
        case = latent_case(T, H, n, r, dv, c, 12, dtype)
        absorbed = torch.einsum("hn,hnc->hc", case["q_plain"][query], case["uk"])       # (H, c)
        case["z"][place] = (absorbed[0] * 40.0 / float(absorbed[0].norm())).to(dtype).double()
        seen = window is None or place >= edge
        value = torch.einsum("dc,c->d", case["uv"][0], case["z"][place])
        for cores in ([False, True] if dtype == torch.bfloat16 else [False]):
            got, want = attend_both(ops, case, 1.0, window, dtype, ps, [query - 5, query - 1, query], seed=place, cores=cores)
            near = float((want[2, 0] - value).abs().max()) < 1e-3 * float(value.abs().max())
            assert near == seen, (place, seen)
            assert float((got - want).abs().max()) <= tol(dtype, want, 2e-5, 2e-2), (place, seen, cores)


class Tokens:
    """A step's context for a feed-forward alone: the only field it reads is the token ids."""

    def __init__(self, ids):
        self.token_ids = torch.tensor(ids, dtype=torch.int32, device=DEV)
        self.T = len(ids)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,F,shared,H", [(5, 2, 40, 56, 96), (3, 1, 24, None, 96), (4, 4, 8, 8, 64), (7, 3, 20, 36, 100),
                                              (6, 2, 96, 160, 384)])
def test_table_routed_experts_alone(dtype, E, top, F, shared, H):
    from gesso_amd.config import TableMoESpec
    from test_gpu_parts import Harness
    vocab = 50
    spec = TableMoESpec(hidden=H, vocab=vocab, n_experts=E, top=top, expert_ff=F, shared_ff=shared)
    h = Harness("ffn", spec, dtype, seed=30 + E, std=0.3)
    w = {"m.table": h.tensors["table"].long()}
    for e in range(E):
        w[f"m.e{e}.up"], w[f"m.e{e}.down"] = h.tensors[f"experts.{e}.up.weight"], h.tensors[f"experts.{e}.down.weight"]
    if shared:
        w.update({"m.shared.up": h.tensors["shared.up.weight"], "m.shared.down": h.tensors["shared.down.weight"],
                  "m.shared.sg": h.tensors["shared.gate.weight"]})
    mlp = {"router": {"top": top}, "shared": {"ff": shared} if shared else None}
    for T in (1, 7, 70, 200):                                  # few rows, and more than the streaming products take
        ids = random_ids(T, vocab, T)
        x = torch.randn(T, H, generator=gen(T)).to(dtype)
        got = h.part.forward(x.to(DEV), Tokens(ids)).double().cpu()
        want = P.table_moe(x.double(), ids, w, "m", mlp)
        assert float((got - want).abs().max()) <= tol(dtype, want, 2e-5, 2e-2), T
        # a token's row does not depend on its neighbours in the batch
        alone = h.part.forward(x[T // 2:T // 2 + 1].to(DEV), Tokens(ids[T // 2:T // 2 + 1])).double().cpu()
        assert float((alone[0] - got[T // 2]).abs().max()) <= tol(dtype, want, 1e-6, 1e-2)


# ------------------------------------------------------------------ the mixer alone, with its own cache

def mixer_harness(dtype, H=3, n=24, r=8, dv=16, qr=40, c=48, window=24, W=96, scaling=True, page_size=8, num_pages=96, seed=5):
    from gesso_amd.config import LatentAttentionSpec, ScaledRopeSpec
    from test_gpu_parts import Harness
    sc = dict(factor=4.0, original=64.0, fast=8.0, slow=2.0) if scaling else dict(factor=None)
    pos = ScaledRopeSpec(head_dim=r, rotary_dim=r, theta=1e4, max_position=512, **sc)
    spec = LatentAttentionSpec(hidden=W, n_heads=H, plain_dim=n, rot_dim=r, value_dim=dv, q_rank=qr, kv_rank=c, scale=0.2,
                               eps=1e-5, position=pos, window=window)
    h = Harness("mixer", spec, dtype, seed=seed, page_size=page_size, num_pages=num_pages, std=0.25)
    t = h.tensors
    w = {"m.dq": t["q_down.weight"], "m.dq.norm": t["q_norm.weight"], "m.uq": t["q_up.weight"], "m.dkv": t["kv_down.weight"],
         "m.dkv.norm": t["kv_norm.weight"], "m.uk": t["k_up.weight"], "m.uv": t["v_up.weight"], "m.g": t["gate.weight"],
         "m.o": t["out.weight"]}
    mx = {"heads": H, "dim": n, "rot_dim": r, "vdim": dv, "kv_rank": c, "scale": 0.2, "mask": {"size": window} if window else None,
          "rot": {"base": 1e4, "dims": r, "scaling": {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 2.0} if scaling else None}}

    def plain(x):
        return P.latent_attention(x.double(), w, "m", mx, 1e-5, list(range(x.shape[0])))

    return h, plain


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kw", [dict(), dict(H=5, n=12, r=6, dv=20, qr=28, c=36, window=17, W=100, scaling=False),
                                dict(H=4, n=32, r=32, dv=32, qr=64, c=64, window=40, W=128, page_size=16),
                                dict(H=1, n=16, r=8, dv=24, qr=20, c=40, window=None, W=64)])
def test_latent_mixer_whole_token_by_token_in_portions_and_in_batches(dtype, kw):
    h, plain = mixer_harness(dtype, **kw)
    W = kw.get("W", 96)
    T = 90
    x = torch.randn(T, W, generator=gen(40)).to(dtype)
    want = plain(x)
    bound = tol(dtype, want, 3e-5, 3e-2)
    whole = h.mixer(x, [("whole", T)])
    assert float((whole - want).abs().max()) <= bound
    # most of it at once, the rest token by token (the window passes over decoded tokens)
    head = 40
    got = [h.mixer(x[:head], [("tail", head)])] + [h.mixer(x[i:i + 1], [("tail", 1)]) for i in range(head, T)]
    assert float((torch.cat(got) - want).abs().max()) <= bound
    # portions of several sizes, down to two tokens
    at, got = 0, []
    for size in (2, 7, 2, 13, 3, 16, 5, 2, 31, 9):
        size = min(size, T - at)
        if size:
            got.append(h.mixer(x[at:at + size], [("cut", size)]))
            at += size
    assert at == T and float((torch.cat(got) - want).abs().max()) <= bound
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
def test_latent_mixer_with_pages_freed_and_used_again(dtype):
    """A pool that holds little more than one request's window: requests come and go, every later one writes pages that
    an earlier one gave back (poisoned with NaN in between)."""
    h, plain = mixer_harness(dtype, window=24, page_size=8, num_pages=9)
    for i, T in enumerate((60, 35, 64, 9)):
        x = torch.randn(T, 96, generator=gen(50 + i)).to(dtype)
        want = plain(x)
        at, got = 0, []
        while at < T:
            size = min((11, 2, 1, 16)[(at + i) % 4], T - at)
            got.append(h.mixer(x[at:at + size], [(i, size)]))
            at += size
        assert float((torch.cat(got) - want).abs().max()) <= tol(dtype, want, 3e-5, 3e-2), i
        released = h.manager.release(i)
        for pool in h.storage.keys:
            pool[:, :-1].fill_(float("nan"))


# ------------------------------------------------------------------ whole models

LENGTHS = {"A": (1, 23, 70, 130), "B": (2, 40, 77), "C": (5, 64, 150, 260), "D": (3, 52, 110)}


def sequences(name):
    cfg, seed = CONFIGS[name]
    return {f"s{i}": random_ids(n, cfg.vocab, 100 * seed + i) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_replay_four_ways(name, dtype, folders, tmp_path):
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences(name)
    plain = R.Plain(model_dir, seqs, dtype)
    ways = {"whole": R.trace_whole, "tail": lambda s: R.trace_tail(s, tail=48), "portions": R.trace_portions,
            "mixed": lambda s: R.trace_mixed(s, seed=5)}
    big = R.Trace()
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            big.steps.append(dict(rec, step=len(big.steps)))
            big.rows.append(rows)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab)
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        plain.check(mine, f"Makuzen {name} {way}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_with_pages_of_eight_given_back_poisoned(dtype, folders, tmp_path):
    cfg, _ = CONFIGS["A"]
    model_dir = write_tiny(folders, "A", torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences("A")
    plain = R.Plain(model_dir, seqs, dtype)
    for way, make in (("portions", lambda s: R.trace_portions(s, sizes=(13, 2, 8, 3))), ("mixed", lambda s: R.trace_mixed(s, seed=9))):
        got, rc = R.run_trace(model_dir, dtype, str(tmp_path / way), make(seqs), cfg.vocab, page_size=8, extra=["--poison"])
        assert rc == 0
        plain.check(got, f"Makuzen A, pages of 8, poisoned, {way}")


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_session(name, folders):
    """Prompts of unequal length generated together through the scheduler (prefill in portions, then the decode loop),
    far enough for every window to pass over generated tokens; float32 must give the plain model's tokens."""
    from gesso_amd import Session
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32)
    pc, pw = P.read_config(model_dir), P.read_weights(model_dir)
    prompts = [random_ids(n, cfg.vocab, 900 + n) for n in (3, 41, 18)]
    new = 56
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


def test_the_command_line_serves_a_makuzen_folder(folders):
    """``python -m gesso_amd --model DIR`` picks the model class by the folder's config.json; float32 gives the plain
    model's tokens, also for a sampled request's first tokens being among the plain model's likely ones."""
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
    """More requests than the weight-streaming products take rows: the recorded loop over the many-row kernels, with
    the experts grouped and the tokens' keys not shared out.  Every token chosen is one the plain model ranks near its
    best at that place, and so is every token the first request gets when it runs alone."""
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


def random_makuzen(seed: int):
    """A configuration drawn from a seed: two to four layers that differ from one another, sizes with and without
    whole tiles, windows shorter and longer than the sequences or none, one to all experts used, layers without a
    feed-forward or without a shared expert, rotation with and without slowed pairs."""
    import random
    from gesso_amd.config import LatentAttentionConfig, MakuzenConfig, MakuzenLayer, TableMoEConfig, YarnScaling
    rng = random.Random(seed)
    width = rng.choice([64, 72, 96, 128, 160, 256])
    layers = []
    for _ in range(rng.randint(2, 4)):
        rot = rng.choice([2, 4, 8, 16, 32])
        experts = rng.randint(1, 12)
        mixer = LatentAttentionConfig(
            heads=rng.choice([1, 2, 3, 4, 6, 8]), dim=rng.choice([8, 12, 16, 24, 32, 64]), rot_dim=rot,
            vdim=rng.choice([8, 16, 20, 32, 64]), q_rank=rng.choice([16, 24, 40, 64, 96]),
            kv_rank=rng.choice([16, 32, 36, 48, 64, 80, 128]), scale=rng.choice([0.08, 0.15, 0.25]),
            rot_base=rng.choice([1e3, 1e4, 5e5]),
            scaling=None if rng.random() < 0.4 else YarnScaling(rng.choice([2.0, 4.0, 8.0]), rng.choice([16.0, 64.0, 256.0]),
                                                                rng.choice([4.0, 8.0, 32.0]), rng.choice([1.0, 2.0])),
            window=rng.choice([None, 3, 16, 33, 64, 72, 150]))
        mlp = None if rng.random() < 0.2 else TableMoEConfig(experts=experts, top=rng.randint(1, min(3, experts)),
                                                             ff=rng.choice([8, 24, 32, 64]),
                                                             shared_ff=rng.choice([None, 16, 40, 128]))
        layers.append(MakuzenLayer(mixer, mlp))
    return MakuzenConfig(vocab=rng.choice([97, 200, 333, 512]), width=width, layers=tuple(layers),
                         embedding_scale=rng.choice([0.5, 1.0, 3.0]), norm_eps=rng.choice([1e-5, 1e-6, 1e-4]),
                         residual_mult=rng.choice([0.25, 0.5, 1.0]), max_position=512)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [31, 32, 33, 34, 35, 36])
def test_replay_of_configurations_drawn_at_random(seed, dtype, tmp_path):
    import random
    from gesso_amd.weights import write_model_folder
    cfg = random_makuzen(seed)
    rng = random.Random(seed)
    model_dir = write_model_folder(str(tmp_path / "m"), cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16,
                                   std=STD)
    lens = [rng.randint(1, 4), rng.randint(20, 60), rng.randint(70, 120), rng.randint(130, 210)]
    seqs = {f"s{i}": random_ids(n, cfg.vocab, seed * 10 + i) for i, n in enumerate(lens)}
    plain = R.Plain(model_dir, seqs, dtype)
    ways = {"whole": R.trace_whole, "tail": lambda s: R.trace_tail(s, tail=40), "portions": R.trace_portions,
            "mixed": lambda s: R.trace_mixed(s, seed=seed)}
    big = R.Trace()
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            big.steps.append(dict(rec, step=len(big.steps)))
            big.rows.append(rows)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab, extra=["--poison"])
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        plain.check(mine, f"seed {seed} {way}")
