"""Fazezen without a GPU: the configuration through its file and back, the model as data, the cache's bookkeeping for
a call with two caches and for runs of positions that have passed, and the plain implementation's own mechanisms."""
import json
import math

import pytest
import torch

import plain_fazezen as P
from tiny_fazezen import CONFIGS, FZ_A, FZ_B, FZ_D

from gesso_amd.cache.manager import RELEASED, CacheLayout, CacheManager
from gesso_amd.config import FazezenConfig, architecture_of
from gesso_amd.errors import ConfigError
from gesso_amd.models.model import tensor_table
from gesso_amd.parts.base import PagedKV, SlotState
from gesso_amd.parts.registry import part_class


def gen(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------ configuration

@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configuration_through_its_file_and_back(name):
    cfg, _ = CONFIGS[name]
    raw = json.loads(json.dumps(cfg.to_json()))
    assert architecture_of(raw).name == "Fazezen"
    assert FazezenConfig.from_dict(raw) == cfg
    assert FazezenConfig.from_dict(raw).to_json() == raw


def test_errors_name_the_key():
    raw = FZ_A.to_json()
    bad = json.loads(json.dumps(raw))
    bad["layers"][1]["mixer"]["left"]["window"] = 5
    with pytest.raises(ConfigError, match="window"):
        FazezenConfig.from_dict(bad)
    bad = json.loads(json.dumps(raw))
    bad["layers"][0]["mixer"]["decay"] = [0.5, 0.9]
    with pytest.raises(ConfigError, match="decay"):
        FazezenConfig.from_dict(bad)
    bad = json.loads(json.dumps(raw))
    bad["layers"][1]["type"] = "lightning"
    with pytest.raises(ConfigError):
        FazezenConfig.from_dict(bad)
    bad = json.loads(json.dumps(raw))
    bad["layers"][1]["mixer"]["left"]["rot"]["dims"] = 26
    with pytest.raises(ConfigError, match="dims"):
        FazezenConfig.from_dict(bad)
    bad = json.loads(json.dumps(raw))
    del bad["layers"][2]["mlp"]["ff"]
    with pytest.raises(ConfigError, match="ff"):
        FazezenConfig.from_dict(bad)
    bad = json.loads(json.dumps(raw))
    bad["layers"][1]["mixer"]["left"]["kv_heads"] = 3
    with pytest.raises(ConfigError):
        FazezenConfig.from_dict(bad)
    # null counts as left out
    ok = json.loads(json.dumps(raw))
    ok["layers"][1]["mixer"]["left"]["mask"] = None
    assert FazezenConfig.from_dict(ok).layers[1].mixer.left.chunk is None


def test_the_model_as_data():
    spec = architecture_of(FZ_A.to_json()).to_spec(FZ_A)
    table = tensor_table(spec)
    assert table["embed"].shape == (211, 96) and table["embed.norm"].shape == (96,) and "head" not in table
    assert table["l0.mix.q"].shape == (72, 96) and table["l0.mix.v"].shape == (48, 96) and table["l0.mix.norm"].shape == (48,)
    assert table["l0.mlp.gate.b"].shape == (80,) and table["l0.mlp.down.b"].shape == (96,)
    assert table["l1.mix.left.q"].shape == (96, 96) and table["l1.mix.left.k"].shape == (48, 96)
    assert table["l1.mix.left.v"].shape == (32, 96) and table["l1.mix.left.o"].shape == (96, 64)
    assert table["l1.mix.left.q.norm"].shape == (24,)
    assert table["l1.mix.right.v"].shape == (48, 96) and table["l1.mix.right.g"].shape == (48, 96)
    assert "l1.norm2" not in table and "l1.mlp.gate" not in table and "l1.mix.right.norm" not in table
    assert spec.tie_embeddings and spec.embed_norm.offset == 1.0 and spec.final_norm.offset == 1.0
    needs = [part_class("block", b).cache_need(b) for b in spec.blocks]
    assert needs[0] == SlotState((("state", (3, 24, 16), "float32"),))
    assert needs[1] == (PagedKV(2, 24, None, value_dim=16, chunk=24), SlotState((("state", (2, 16, 24), "float32"),)))
    left = spec.blocks[1].mixer.left
    assert left.sink and left.chunk == 24 and left.value_position.rotary_dim == 16 and left.position.rotary_dim == 16
    assert spec.blocks[1].mixer.right.key_scale == 0.25 and spec.blocks[1].mixer.right.position.rotary_dim == 8
    # a left side without any turn caches its values as they are
    spec_b = architecture_of(FZ_B.to_json()).to_spec(FZ_B)
    assert spec_b.blocks[2].mixer.left.value_position is None and spec_b.blocks[2].mixer.left.position.kind == "none"


# ------------------------------------------------------------------ the cache's bookkeeping

def test_a_call_with_two_caches_and_runs_that_have_passed():
    spec = architecture_of(FZ_D.to_json()).to_spec(FZ_D)
    needs = [part_class("block", b).cache_need(b) for b in spec.blocks]
    layout = CacheLayout.plan(needs, [None] * len(needs))
    assert layout.parts_of_call == {1: 2, 2: 2}
    assert [g.members for g in layout.paged] == [((1, 0),), ((2, 0),)]
    assert [m.call for m in layout.slots] == [0, (1, 1), (2, 1)]
    mgr = CacheManager(layout, 4, 24, 2, 400)
    mgr.admit("a")
    at = 0
    for n in (5, 11, 1, 1, 20, 2, 30):
        mgr.reserve("a", n)
        mgr.commit("a", n)
        at += n
        chunked, whole = mgr.get("a").tables
        first = at - at % 17                       # the oldest position the next token reads
        for b, page in enumerate(chunked):
            assert (page == RELEASED) == ((b + 1) * 4 <= first), (at, b)
        assert RELEASED not in whole
        mgr.check()
    mgr.release("a")
    assert mgr.pools[0].n_free == 24 and mgr.pools[1].n_free == 24 and mgr.slot_pool.n_free == 2


def test_first_needed_of_windows_and_runs():
    assert PagedKV(1, 8).first_needed(100) == 0
    assert PagedKV(1, 8, window=10).first_needed(100) == 91
    assert [PagedKV(1, 8, chunk=16).first_needed(n) for n in (0, 15, 16, 17, 31, 32)] == [0, 0, 16, 16, 16, 32]
    assert PagedKV(1, 8, window=4, chunk=16).first_needed(30) == 27 and PagedKV(1, 8, window=40, chunk=16).first_needed(33) == 32


# ------------------------------------------------------------------ the plain implementation's mechanisms

def test_stretched_frequencies_keep_divide_and_blend():
    plain = P.frequencies(16, 100.0)
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64.0}
    got = P.stretched_frequencies(16, 100.0, sc)
    for f, g in zip(plain, got):
        wl = 2 * math.pi / f
        if wl < 16.0:
            assert g == f
        elif wl > 64.0:
            assert g == f / 4.0
        else:
            s = (64.0 / wl - 1.0) / 3.0
            assert g == pytest.approx((1 - s) * f / 4.0 + s * f) and f / 4.0 <= g <= f
    assert any(g == f for f, g in zip(plain, got)) and any(g == f / 4.0 for f, g in zip(plain, got))
    assert any(f / 4.0 < g < f for f, g in zip(plain, got))
    assert P.stretched_frequencies(16, 100.0, None) == plain


def test_turn_pairs_halves_and_scores_depend_on_distance_alone():
    f = P.frequencies(8, 50.0)
    x = torch.randn(1, 12, generator=gen(0), dtype=torch.float64)
    y = P.turn(x, [3], f)
    a = 3 * f[1]
    assert float(y[0, 1]) == pytest.approx(float(x[0, 1] * math.cos(a) - x[0, 5] * math.sin(a)))
    assert float(y[0, 5]) == pytest.approx(float(x[0, 5] * math.cos(a) + x[0, 1] * math.sin(a)))
    assert torch.equal(y[0, 8:], x[0, 8:])
    q, k = torch.randn(1, 8, generator=gen(1), dtype=torch.float64), torch.randn(1, 8, generator=gen(2), dtype=torch.float64)
    s1 = float(P.turn(q, [9], f) @ P.turn(k, [4], f).t())
    s2 = float(P.turn(q, [105], f) @ P.turn(k, [100], f).t())
    assert s1 == pytest.approx(s2, abs=1e-12)
    assert torch.allclose(P.turn(P.turn(x, [7], f), [7], f, sign=-1.0), x, atol=1e-14)


def test_fading_state_equals_the_sum_over_the_past():
    T, H, n, m = 9, 2, 3, 4
    q, k = torch.randn(T, H, n, generator=gen(3), dtype=torch.float64), torch.randn(T, H, n, generator=gen(4), dtype=torch.float64)
    v = torch.randn(T, H, m, generator=gen(5), dtype=torch.float64)
    decay = [0.5, 1.0]
    got = P.decayed_state_attention(q, k, v, decay)
    for h in range(H):
        for t in range(T):
            want = sum(decay[h] ** (t - j) * float(q[t, h] @ k[j, h]) * v[j, h] for j in range(t + 1))
            assert torch.allclose(got[t, h], want, atol=1e-12)
    zero = P.decayed_state_attention(q, k, v, [0.0, 0.0])
    assert torch.allclose(zero[5, 0], float(q[5, 0] @ k[5, 0]) * v[5, 0], atol=1e-12)


def test_runs_and_the_sink():
    T, H, G, n, m = 11, 2, 1, 4, 3
    q = torch.randn(T, H, n, generator=gen(6), dtype=torch.float64)
    k = torch.randn(T, G, n, generator=gen(7), dtype=torch.float64)
    v = torch.randn(T, G, m, generator=gen(8), dtype=torch.float64)
    got = P.chunked_sink_attention(q, k, v, 0.7, 4)
    for i in (0, 3, 4, 6, 8, 10):
        lo = i - i % 4
        for h in range(H):
            e = torch.exp(0.7 * (k[lo:i + 1, 0] @ q[i, h]))
            assert torch.allclose(got[i, h], (e / (1.0 + e.sum())) @ v[lo:i + 1, 0], atol=1e-12)
    # a key just behind a run's edge counts for nothing, however large; the first key of the run counts
    k2 = k.clone()
    k2[3] *= 1e3
    assert torch.allclose(P.chunked_sink_attention(q, k2, v, 0.7, 4)[4:], got[4:], atol=1e-12)
    k2 = k.clone()
    k2[4] = 50.0 * q[7, 0] / float(q[7, 0] @ q[7, 0])
    assert torch.allclose(P.chunked_sink_attention(q, k2, v, 0.7, 4)[7, 0], v[4, 0], atol=1e-9)
    # with every score far below zero the sink takes all the weight and the output vanishes
    far = P.chunked_sink_attention(q, k, v, 0.7, 1)
    e = torch.exp(0.7 * (k[5, 0] @ q[5, 1]))
    assert torch.allclose(far[5, 1], e / (1 + e) * v[5, 0], atol=1e-12)
    no_runs = P.chunked_sink_attention(q, k, v, 0.7, None)
    e = torch.exp(0.7 * (k[:, 0] @ q[10, 0]))
    assert torch.allclose(no_runs[10, 0], (e / (1.0 + e.sum())) @ v[:, 0], atol=1e-12)


def test_turned_values_give_sums_that_depend_on_distance():
    """Values turned by their own position and a sum turned back by the query's: value ``j`` enters output ``i`` turned
    by ``j - i``."""
    f = P.frequencies(6, 30.0)
    v = torch.randn(5, 1, 6, generator=gen(9), dtype=torch.float64)
    p = torch.rand(5, generator=gen(10), dtype=torch.float64)
    turned = P.turn(v, list(range(5)), f)
    out = P.turn((p[:, None, None] * turned).sum(0, keepdim=True), [4], f, sign=-1.0)
    want = sum(p[j] * P.turn(v[j:j + 1], [j - 4], f) for j in range(5))
    assert torch.allclose(out, want, atol=1e-12)


def test_a_layer_by_hand():
    """One lightning layer and one pair, written out once more from the equations with explicit loops over heads."""
    cfg = {"norm": {"eps": 1e-5}, "layers": FZ_A.to_json()["layers"]}
    W = 96
    g = gen(11)
    spec = architecture_of(FZ_A.to_json()).to_spec(FZ_A)
    w = {name: 0.2 * torch.randn(ts.shape, generator=g, dtype=torch.float64) for name, ts in tensor_table(spec).items()}
    x = torch.randn(6, W, generator=g, dtype=torch.float64)
    # layer 0
    y = P.layer(x, w, 0, cfg, list(range(6)))
    h1 = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5)
    h2 = h1 * (1 + w["l0.norm2"])
    h1 = h1 * (1 + w["l0.norm1"])
    silu = lambda z: z * torch.sigmoid(z)
    q, k, v = silu(h1 @ w["l0.mix.q"].t()), silu(h1 @ w["l0.mix.k"].t()), silu(h1 @ w["l0.mix.v"].t())
    o = torch.zeros(6, 48, dtype=torch.float64)
    for h, d in enumerate((0.5, 0.9, 0.99)):
        for t in range(6):
            for j in range(t + 1):
                o[t, 16 * h:16 * h + 16] += d ** (t - j) * float(q[t, 24 * h:24 * h + 24] @ k[j, 24 * h:24 * h + 24]) * v[j, 16 * h:16 * h + 16]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5) * w["l0.mix.norm"] * torch.sigmoid(h1 @ w["l0.mix.g"].t())
    a = h2 @ w["l0.mlp.gate"].t() + w["l0.mlp.gate.b"]
    gelu = 0.5 * a * (1 + torch.tanh(math.sqrt(2 / math.pi) * (a + 0.044715 * a ** 3)))
    ff = (gelu * (h2 @ w["l0.mlp.up"].t() + w["l0.mlp.up.b"])) @ w["l0.mlp.down"].t() + w["l0.mlp.down.b"]
    assert torch.allclose(y, x + o @ w["l0.mix.o"].t() + ff, atol=1e-10)
    # layer 1 has no feed-forward: the stream moves by the pair's weighted sum alone
    y = P.layer(x, w, 1, cfg, list(range(6)))
    h = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * (1 + w["l1.norm1"])
    mx = cfg["layers"][1]["mixer"]
    left = P.left_branch(h, w, "l1.mix.left", mx["left"], 1e-5, list(range(6)))
    right = P.right_branch(h, w, "l1.mix.right", mx["right"], 1e-5, list(range(6)))
    assert torch.allclose(y, x + 1.3 * left + 0.8 * right, atol=1e-12)
    # the right side's heads are normed one by one, without a weight
    qr, kr = h @ w["l1.mix.right.q"].t(), h @ w["l1.mix.right.k"].t()
    vr = (h @ w["l1.mix.right.v"].t()).reshape(6, 2, 24)
    f = P.frequencies(8, 1e4)
    qr, kr = P.turn(qr.reshape(6, 2, 16), range(6), f), P.turn(kr.reshape(6, 2, 16), range(6), f) / 4.0
    o = P.decayed_state_attention(qr, kr, vr, (0.9, 0.97))
    o = (o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5)).reshape(6, 48) * silu(h @ w["l1.mix.right.g"].t())
    assert torch.allclose(right, o @ w["l1.mix.right.o"].t(), atol=1e-12)
