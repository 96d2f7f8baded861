"""Plain Makuzen: a slow, whole-sequence, cache-free implementation used as the oracle.

Nothing is imported from ``gesso_amd``: a model folder is read with ``json`` and the ``safetensors``
package, the arithmetic is explicit torch on the CPU in float64 (or another type on request).  One
function per mechanism:

    embedding  rmsnorm  yarn_frequencies  rotate  windowed_attention  latent_attention  expert  table_moe  layer  forward

Notation.  Rows are tokens: activations are ``(T, features)``, a linear weight ``W`` is ``(out, in)``
and acts as ``y = x @ W.T``.  ``rms(x) = x / sqrt(mean(x^2) + eps)`` with eps under the root.

The model.  ``x_0 = E[token] * s_e``.  A layer adds its sub-layers' *normed outputs*:
``x <- x + m * rms(mixer(x)) * g_1``, then (when the layer has a feed-forward)
``x <- x + m * rms(ffn(x)) * g_2``; the sub-layers read ``x`` itself.  Logits are ``W_head (rms(x) * g_f)``.

The mixer attends through two low-rank bottlenecks.  With ``a = rms(W_dq x) * g_q`` the queries are
``q = W_uq a``, head ``h`` holding ``n`` plain features followed by ``r`` rotated ones.  ``W_dkv x`` has
``c + r`` features: the first ``c``, normed (``z = rms(.) * g_kv``), are the token's latent row; the last
``r``, not normed, are a rotated key part that all heads share.  Head ``h`` has plain keys ``W_uk[h] z`` and
values ``W_uv[h] z``; its score against token ``j`` is ``(q_plain . k_plain_j + q_rot . k_rot_j) * scale``
over the tokens ``j`` with ``0 <= i - j < window``, softmax over them, and its output is multiplied by
``sigmoid(W_g x)[h]`` before ``W_o`` mixes the heads.

The feed-forward is a table-routed mixture: token id ``v`` uses the experts ``table[v, :]``, each with weight
``1 / top``; an expert is ``W_down relu(W_up x)^2``.  A shared expert of the same form runs for every token,
scaled by ``sigmoid(w_sg . x)``.
"""
from __future__ import annotations

import json
import math
import os

import torch


def _keep(x):
    return x


def to_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 and widen back: what a pipeline with bfloat16 activations does where it stores one."""
    return x.to(torch.bfloat16).to(x.dtype)


# --------------------------------------------------------------------------- mechanisms

def embedding(table: torch.Tensor, ids, scale: float) -> torch.Tensor:
    rows = []
    for tok in ids:
        tok = int(tok)
        if not 0 <= tok < table.shape[0]:
            raise ValueError(f"token id {tok} outside the vocabulary of {table.shape[0]}")
        rows.append(table[tok] * scale)
    return torch.stack(rows, 0)


def rmsnorm(x: torch.Tensor, weight, eps: float) -> torch.Tensor:
    r = torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    y = x / r
    return y if weight is None else y * weight


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    return x @ w.t()


def yarn_frequencies(dims: int, base: float, scaling):
    """``(frequencies of the dims/2 pairs, factor on cos and sin)``.

    Pair ``i`` turns by ``f_i = base^(-2i/dims)`` a position.  With a scaling ``(factor, original, fast, slow)``:
    ``dim(t) = dims ln(original / (2 pi t)) / (2 ln base)`` is the (real-valued) pair that makes ``t`` turns over
    the original length; pairs below ``lo = max(floor(dim(fast)), 0)`` keep their frequency, pairs above
    ``hi = min(ceil(dim(slow)), dims - 1)`` are slowed by ``factor``, and those between are blended linearly;
    cos and sin are both multiplied by ``0.1 ln(factor) + 1``."""
    half = dims // 2
    f = [float(base) ** (-2.0 * i / dims) for i in range(half)]
    if scaling is None:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001)))
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions, freqs, mult: float) -> torch.Tensor:
    """``x (T, ..., dims)``: feature ``i`` is paired with ``i + dims/2``; the pair ``(u, v)`` at position ``p``
    becomes ``(u cos a - v sin a, v cos a + u sin a)``, ``a = p f_i``, with cos and sin both times ``mult``."""
    half = len(freqs)
    assert x.shape[-1] == 2 * half
    out = x.clone()
    for t in range(x.shape[0]):
        p = float(positions[t])
        for i in range(half):
            a = p * freqs[i]
            c, s = math.cos(a) * mult, math.sin(a) * mult
            u, v = x[t, ..., i], x[t, ..., i + half]
            out[t, ..., i] = u * c - v * s
            out[t, ..., i + half] = v * c + u * s
    return out


def windowed_attention(q_plain, q_rot, k_plain, k_rot, v, scale: float, window=None) -> torch.Tensor:
    """Softmax attention of token ``i`` over the tokens ``j`` with ``0 <= i - j < window`` (all ``j <= i`` without a
    window).  ``q_plain, k_plain (T, H, n)``, ``q_rot (T, H, r)``, ``k_rot (T, r)`` shared by the heads,
    ``v (T, H, dv)``; the score is ``(q_plain . k_plain + q_rot . k_rot) * scale``.  Returns ``(T, H, dv)``."""
    T, H = q_plain.shape[0], q_plain.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=v.dtype)
    for i in range(T):
        lo = 0 if not window else max(0, i - int(window) + 1)
        for h in range(H):
            s = (k_plain[lo:i + 1, h] @ q_plain[i, h] + k_rot[lo:i + 1] @ q_rot[i, h]) * scale
            pr = torch.softmax(s, dim=0)
            out[i, h] = pr @ v[lo:i + 1, h]
    return out


def latent_attention(x, w, p, mx, eps, positions, store=_keep):
    """The mixer on ``x (T, width)``, the whole sequence from position 0; ``w``: name -> tensor, ``p``: the tensors'
    prefix (``l3.mix``), ``mx``: the layer's ``mixer`` entry of the configuration."""
    T = x.shape[0]
    H, n, r, dv, c = int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]), int(mx["kv_rank"])
    rot = mx.get("rot") or {}
    assert int(rot.get("dims", r)) == r
    freqs, mult = yarn_frequencies(r, float(rot["base"]), rot.get("scaling")) if r else ([], 1.0)
    window = (mx.get("mask") or {}).get("size")
    scale = float(mx["scale"])

    a = store(rmsnorm(store(linear(x, w[p + ".dq"])), w[p + ".dq.norm"], eps))
    q = store(linear(a, w[p + ".uq"])).reshape(T, H, n + r)
    down = store(linear(x, w[p + ".dkv"]))
    z = store(rmsnorm(down[:, :c], w[p + ".dkv.norm"], eps))
    k_rot = store(rotate(down[:, c:], positions, freqs, mult)) if r else down[:, c:]
    q_plain = q[:, :, :n]
    q_rot = store(rotate(q[:, :, n:], positions, freqs, mult)) if r else q[:, :, n:]
    k_plain = store(linear(z, w[p + ".uk"])).reshape(T, H, n)
    v = store(linear(z, w[p + ".uv"])).reshape(T, H, dv)
    gate = torch.sigmoid(linear(x, w[p + ".g"]))                       # (T, H)
    out = windowed_attention(q_plain, q_rot, k_plain, k_rot, v, scale, window)
    out = store(out * gate[:, :, None])
    return store(linear(out.reshape(T, H * dv), w[p + ".o"]))


def expert(x, up, down, store=_keep):
    """``W_down relu(W_up x)^2``."""
    h = torch.relu(store(linear(x, up)))
    return linear(store(h * h), down)


def table_moe(x, ids, w, p, mlp, store=_keep):
    """The feed-forward on ``x (T, width)`` for the token ids ``ids``; ``p``: the tensors' prefix (``l3.mlp``)."""
    top = int(mlp["router"]["top"])
    table = w[p + ".table"]
    out = torch.zeros_like(x)
    for t, tok in enumerate(ids):
        chosen = [int(e) for e in table[int(tok)].tolist()]
        assert len(chosen) == top and len(set(chosen)) == top
        for e in chosen:
            out[t] += expert(x[t:t + 1], w[f"{p}.e{e}.up"], w[f"{p}.e{e}.down"], store)[0] / top
    if mlp.get("shared") is not None:
        g = torch.sigmoid(linear(x, w[p + ".shared.sg"].reshape(1, -1)))    # (T, 1)
        out = out + g * expert(x, w[p + ".shared.up"], w[p + ".shared.down"], store)
    return store(out)


def layer(x, ids, w, i, cfg, positions, store=_keep):
    """Layer ``i``: each sub-layer reads ``x`` and adds ``m`` times its normed output."""
    L = cfg["layers"][i]
    eps, m = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    if L["type"] != "latent_attention":
        raise ValueError(f"unknown layer type {L['type']!r}")
    y = latent_attention(store(x), w, f"l{i}.mix", L["mixer"], eps, positions, store)
    x = x + m * rmsnorm(y, w[f"l{i}.norm1"], eps)
    if L.get("mlp") is not None:
        if L["mlp"]["kind"] != "moe":
            raise ValueError(f"unknown feed-forward kind {L['mlp']['kind']!r}")
        y = table_moe(store(x), ids, w, f"l{i}.mlp", L["mlp"], store)
        x = x + m * rmsnorm(y, w[f"l{i}.norm2"], eps)
    return x


# --------------------------------------------------------------------------- whole model

def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json"), encoding="utf-8") as f:
        return json.load(f)


def read_weights(model_dir: str, dtype=torch.float64) -> dict:
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            out[name] = t.to(dtype) if t.is_floating_point() else t.to(torch.int64)
    return out


def forward(cfg: dict, w: dict, ids, store=_keep, layers_out=None) -> torch.Tensor:
    """Logits ``(T, vocab)`` of the whole sequence ``ids``, positions from 0.  ``layers_out``: a list that receives
    the residual stream after every layer."""
    ids = [int(t) for t in ids]
    positions = list(range(len(ids)))
    x = embedding(w["embed"], ids, float(cfg["embedding"]["scale"]))
    for i in range(len(cfg["layers"])):
        x = layer(x, ids, w, i, cfg, positions, store)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = store(rmsnorm(x, w["final.norm"], float(cfg["norm"]["eps"])))
    return linear(x, w["head"])


def greedy(cfg: dict, w: dict, prompt, max_new_tokens: int):
    ids = [int(t) for t in prompt]
    for _ in range(max_new_tokens):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids
