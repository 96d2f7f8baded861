"""Makuzen without a GPU: the configuration reader, the model as data, and the plain implementation's own mechanisms."""
import json
import math

import pytest
import torch

import plain_makuzen as P
from tiny_makuzen import CONFIGS, MK_A, MK_B, STD, write_tiny

from gesso_amd.config import MakuzenConfig, load_config
from gesso_amd.config.registry import architecture_of
from gesso_amd.errors import ConfigError
from gesso_amd.models.model import tensor_table


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return str(tmp_path_factory.mktemp("makuzen"))


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configuration_survives_its_file(name, folders):
    cfg, _ = CONFIGS[name]
    d = write_tiny(folders, name)
    arch, back = load_config(d)
    assert arch.name == "Makuzen" and back == cfg
    assert MakuzenConfig.from_dict(json.loads(json.dumps(cfg.to_json()))) == cfg


def test_unknown_and_missing_keys_are_named():
    raw = MK_A.to_json()
    raw["layers"][0]["mixer"]["softcap"] = 30.0
    with pytest.raises(ConfigError, match="softcap"):
        MakuzenConfig.from_dict(raw)
    raw = MK_A.to_json()
    del raw["layers"][2]["mixer"]["kv_rank"]
    with pytest.raises(ConfigError, match="kv_rank"):
        MakuzenConfig.from_dict(raw)
    raw = MK_A.to_json()
    raw["layers"][1]["type"] = "recurrent"
    with pytest.raises(ConfigError, match="recurrent"):
        MakuzenConfig.from_dict(raw)
    raw = MK_A.to_json()
    raw["layers"][0]["mlp"]["router"]["top"] = 9
    with pytest.raises(ConfigError):
        MakuzenConfig.from_dict(raw)


def test_the_model_as_data_names_every_tensor_with_its_shape():
    spec = architecture_of(MK_A.to_json()).to_spec(MK_A)
    table = tensor_table(spec)
    assert table["embed"].shape == (211, 96) and table["head"].shape == (211, 96) and table["final.norm"].shape == (96,)
    assert table["l0.mix.dq"].shape == (40, 96) and table["l0.mix.uq"].shape == (3 * 32, 40)
    assert table["l0.mix.dkv"].shape == (48 + 8, 96) and table["l0.mix.dkv.norm"].shape == (48,)
    assert table["l0.mix.uk"].shape == (3 * 24, 48) and table["l0.mix.uv"].shape == (3 * 16, 48)
    assert table["l0.mix.g"].shape == (3, 96) and table["l0.mix.o"].shape == (96, 3 * 16)
    assert table["l0.mlp.table"].shape == (211, 2) and table["l0.mlp.e4.up"].shape == (40, 96)
    assert table["l0.mlp.shared.sg"].shape == (1, 96) and table["l0.mlp.shared.down"].shape == (96, 56)
    assert not any(k.startswith("l1.mlp") or k == "l1.norm2" for k in table)
    assert "l2.mlp.shared.up" not in table and table["l2.mlp.table"].shape == (211, 1)
    # the cache: one row of latent + rotated features a token, no value rows, the layer's own window
    from gesso_amd.parts import part_class
    needs = [part_class("block", b).cache_need(b) for b in spec.blocks]
    assert [(n.n_kv_heads, n.head_dim, n.window, n.value_width) for n in needs] == \
        [(1, 56, 24, 0), (1, 80, None, 0), (1, 36, 9, 0)]


def test_written_tables_hold_different_experts_in_a_row(folders):
    w = P.read_weights(write_tiny(folders, "B"))
    t = w["l0.mlp.table"]
    assert t.shape == (150, 3) and int(t.min()) >= 0 and int(t.max()) < 4
    assert all(len(set(row)) == 3 for row in t.tolist())


# ------------------------------------------------------------------ the plain mechanisms

def test_frequencies_without_and_with_scaling():
    f, mult = P.yarn_frequencies(8, 100.0, None)
    assert mult == 1.0 and f == pytest.approx([100.0 ** (-2 * i / 8) for i in range(4)])
    sc = {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 2.0}
    g, mult = P.yarn_frequencies(8, 100.0, sc)
    assert mult == pytest.approx(0.1 * math.log(4.0) + 1.0)
    # dim(8) = 8 ln(64 / (16 pi)) / (2 ln 100) = 0.21 -> lo = 0; dim(2) = 8 ln(64 / (4 pi)) / (2 ln 100) = 1.41 -> hi = 2
    ramps = [0.0, 0.5, 1.0, 1.0]
    assert g == pytest.approx([f[i] / 4.0 * ramps[i] + f[i] * (1 - ramps[i]) for i in range(4)])
    # lo == hi: the step from "kept" to "slowed" falls between two pairs
    h, _ = P.yarn_frequencies(8, 100.0, {"factor": 2.0, "original": 64.0, "fast": 4.0, "slow": 4.0})
    lo = max(math.floor(8 * math.log(64 / (8 * math.pi)) / (2 * math.log(100.0))), 0)
    assert h[lo] == pytest.approx(f[lo]) and h[3] == pytest.approx(f[3] / 2.0)


def test_rotation_pairs_halves_and_keeps_differences_of_positions():
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 6, generator=g, dtype=torch.float64), torch.randn(1, 6, generator=g, dtype=torch.float64)
    f = [1.0, 0.3, 0.01]
    assert torch.equal(P.rotate(q, [0], f, 1.0), q)
    one = P.rotate(torch.tensor([[1.0, 0, 0, 0, 0, 0]], dtype=torch.float64), [2], f, 1.5)
    assert one[0].tolist() == pytest.approx([1.5 * math.cos(2.0), 0, 0, 1.5 * math.sin(2.0), 0, 0])
    a = float(P.rotate(q, [17], f, 1.0)[0] @ P.rotate(k, [11], f, 1.0)[0])
    b = float(P.rotate(q, [106], f, 1.0)[0] @ P.rotate(k, [100], f, 1.0)[0])
    assert a == pytest.approx(b, abs=1e-12)
    assert float(P.rotate(q, [5], f, 1.3).norm()) == pytest.approx(1.3 * float(q.norm()))


def test_window_sees_itself_and_the_tokens_before_it_and_no_more():
    g = torch.Generator().manual_seed(1)
    T, H, n, r, dv = 12, 2, 4, 2, 3
    qp, kp = torch.randn(T, H, n, generator=g, dtype=torch.float64), torch.randn(T, H, n, generator=g, dtype=torch.float64)
    qr, kr = torch.randn(T, H, r, generator=g, dtype=torch.float64), torch.randn(T, r, generator=g, dtype=torch.float64)
    v = torch.randn(T, H, dv, generator=g, dtype=torch.float64)
    base = P.windowed_attention(qp, qr, kp, kr, v, 0.5, 4)
    v2 = v.clone()
    v2[5] += 10.0                    # token 5 is seen by 5, 6, 7, 8 and by nobody else
    moved = (P.windowed_attention(qp, qr, kp, kr, v2, 0.5, 4) - base).abs().amax(dim=(1, 2)) > 1e-9
    assert moved.tolist() == [i in (5, 6, 7, 8) for i in range(T)]
    assert torch.allclose(P.windowed_attention(qp, qr, kp, kr, v, 0.5, 1), v)
    assert torch.allclose(P.windowed_attention(qp, qr, kp, kr, v, 0.5, None), P.windowed_attention(qp, qr, kp, kr, v, 0.5, T))


def test_a_token_uses_the_experts_of_its_row_and_no_others(folders):
    d = write_tiny(folders, "A")
    cfg, w = P.read_config(d), P.read_weights(d)
    mlp = cfg["layers"][0]["mlp"]
    x = torch.randn(3, cfg["width"], generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    ids = [7, 7, 100]
    base = P.table_moe(x, ids, w, "l0.mlp", mlp)
    used = set(w["l0.mlp.table"][7].tolist())
    other = next(e for e in range(5) if e not in used)
    w2 = dict(w)
    w2[f"l0.mlp.e{other}.down"] = w[f"l0.mlp.e{other}.down"] * 3.0
    again = P.table_moe(x, ids, w2, "l0.mlp", mlp)
    assert torch.equal(again[:2], base[:2])
    mine = next(iter(used))
    w2 = dict(w)
    w2[f"l0.mlp.e{mine}.down"] = w[f"l0.mlp.e{mine}.down"] * 3.0
    assert not torch.allclose(P.table_moe(x, ids, w2, "l0.mlp", mlp)[:2], base[:2])
    # by hand for one token: half of each of its two experts plus the gated shared one
    e0, e1 = w["l0.mlp.table"][100].tolist()
    want = sum(torch.relu(x[2] @ w[f"l0.mlp.e{e}.up"].T) ** 2 @ w[f"l0.mlp.e{e}.down"].T for e in (e0, e1)) / 2
    want = want + torch.sigmoid(x[2] @ w["l0.mlp.shared.sg"].reshape(-1)) * (
        torch.relu(x[2] @ w["l0.mlp.shared.up"].T) ** 2 @ w["l0.mlp.shared.down"].T)
    assert torch.allclose(base[2], want)


def test_a_layer_adds_the_normed_outputs_of_sublayers_that_read_the_stream_itself(folders):
    d = write_tiny(folders, "B")
    cfg, w = P.read_config(d), P.read_weights(d)
    ids = [3, 9, 27, 81]
    x = P.embedding(w["embed"], ids, 1.0)
    y = P.latent_attention(x, w, "l0.mix", cfg["layers"][0]["mixer"], 1e-6, [0, 1, 2, 3])
    x1 = x + P.rmsnorm(y, w["l0.norm1"], 1e-6)
    x2 = x1 + P.rmsnorm(P.table_moe(x1, ids, w, "l0.mlp", cfg["layers"][0]["mlp"]), w["l0.norm2"], 1e-6)
    assert torch.allclose(P.layer(x, ids, w, 0, cfg, [0, 1, 2, 3]), x2)
    # a window of one: the mixer of layer 0 is a function of the token alone
    lone = P.latent_attention(x[2:3], w, "l0.mix", cfg["layers"][0]["mixer"], 1e-6, [0])
    # (its rotated parts turn by the same angle in query and key, which leaves their product as it was)
    assert torch.allclose(lone[0], y[2])
