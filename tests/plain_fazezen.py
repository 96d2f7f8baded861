"""Plain Fazezen: a slow, whole-sequence, cache-free implementation used as the oracle.

Nothing is imported from ``gesso_amd``: a model folder is read with ``json`` and the ``safetensors``
package, the arithmetic is explicit torch on the CPU in float64 (or another type on request).  One
function per mechanism:

    embedding  rms  offset_norm  gelu_tanh  dense_ff  frequencies  stretched_frequencies  turn
    decayed_state_attention  lightning  chunked_sink_attention  left_branch  right_branch  parallel  layer  forward

Notation.  Rows are tokens: activations are ``(T, features)``, a linear weight ``W`` is ``(out, in)`` and acts as
``y = x @ W.T``.  ``rms(x) = x / sqrt(mean(x^2) + eps)``, eps under the root.

The model.  ``x_0 = offset_norm(E[token], g_e)`` with ``offset_norm(x, g) = rms(x) * (1 + g)``.  A layer reads one
``x`` twice and adds both results at once: ``x <- x + mixer(offset_norm(x, g_1)) + ff(offset_norm(x, g_2))`` (a layer
without a feed-forward adds the mixer alone).  Logits are ``E offset_norm(x, g_f)``: the embedding table is the head.

Mixer ``lightning``: ``q, k, v = silu(W_q h), silu(W_k h), silu(W_v h)`` split into heads; per head a matrix state
``S_t = d_h S_(t-1) + k_t v_t^T`` from ``S = 0`` and ``o_t = S_t^T q_t``; all heads' outputs side by side are normed as
one row (``rms(.) * g_n``), multiplied by ``sigmoid(W_g h)`` and projected by ``W_o``.

Mixer ``parallel``: two branches read the same ``h``; the result is ``a_l left(h) + a_r right(h)``.

* left: grouped-query softmax attention.  ``q, k`` are normed per head (``rms(.) * g`` with one weight of the head's
  width for all heads), then turned by the position (the first ``dims`` features of a head, feature ``i`` paired with
  ``i + dims/2``, with the frequencies stretched for long contexts).  The *values* are turned as well, over their
  whole width, by their own position ``j`` with unstretched frequencies, and a head's weighted sum at position ``i``
  is turned back by ``-i``.  Position ``i`` sees ``j <= i`` within its own block of ``size`` positions
  (``i // size == j // size``).  The softmax has one more term in its denominator, ``exp(0)``, which has no value:
  ``p_j = exp(s_j) / (1 + sum_j' exp(s_j'))``, ``s_j = scale (q_i . k_j)``.
* right: retention.  ``q, k`` turned by the position (plain frequencies), ``k`` then times ``dim^(-1/2)``; the same
  decayed matrix state as above with a fixed decay per head and no softmax; each head's output is divided by its root
  mean square (no weight), the heads side by side are multiplied by ``silu(W_g h)`` and projected by ``W_o``.

Feed-forward ``dense``: ``W_d (gelu_tanh(W_g h + b_g) * (W_u h + b_u)) + b_d``.
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


# --------------------------------------------------------------------------- small mechanisms

def embedding(table: torch.Tensor, ids) -> torch.Tensor:
    rows = []
    for tok in ids:
        tok = int(tok)
        if not 0 <= tok < table.shape[0]:
            raise ValueError(f"token id {tok} outside the vocabulary of {table.shape[0]}")
        rows.append(table[tok])
    return torch.stack(rows, 0)


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """The model's norm: the weight is stored around zero and one is added to it."""
    return rms(x, eps) * (1.0 + g)


def linear(x, w, b=None):
    y = x @ w.t()
    return y if b is None else y + b


def silu(z):
    return z / (1.0 + torch.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_ff(h, w, p, store=_keep):
    a = store(linear(h, w[p + ".gate"], w[p + ".gate.b"]))
    b = store(linear(h, w[p + ".up"], w[p + ".up.b"]))
    return store(linear(store(gelu_tanh(a) * b), w[p + ".down"], w[p + ".down.b"]))


# --------------------------------------------------------------------------- positions

def frequencies(dims: int, base: float):
    return [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]


def stretched_frequencies(dims: int, base: float, scaling):
    """Frequencies for contexts longer than ``original``: a pair whose wavelength ``2 pi / f`` is shorter than
    ``original / high`` keeps ``f``; one longer than ``original / low`` gets ``f / factor``; between the two, with
    ``s = (original / wavelength - low) / (high - low)``, the blend ``(1 - s) f / factor + s f``."""
    f = frequencies(dims, base)
    if scaling is None:
        return f
    factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
    original = float(scaling["original"])
    out = []
    for fi in f:
        wavelength = 2.0 * math.pi / fi
        if wavelength < original / high:
            out.append(fi)
        elif wavelength > original / low:
            out.append(fi / factor)
        else:
            s = (original / wavelength - low) / (high - low)
            out.append((1.0 - s) * fi / factor + s * fi)
    return out


def turn(x: torch.Tensor, positions, freqs, sign: float = 1.0) -> torch.Tensor:
    """``x (T, ..., width)``: the first ``2 len(freqs)`` features of the last axis are turned, feature ``i`` with
    ``i + len(freqs)``: ``(u, v) -> (u cos a - v sin a, v cos a + u sin a)``, ``a = sign p f_i``; the rest passes."""
    half = len(freqs)
    assert x.shape[-1] >= 2 * half
    out = x.clone()
    for t in range(x.shape[0]):
        p = float(positions[t])
        for i in range(half):
            a = sign * p * freqs[i]
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, ..., i], x[t, ..., i + half]
            out[t, ..., i] = u * c - v * s
            out[t, ..., i + half] = v * c + u * s
    return out


# --------------------------------------------------------------------------- the two kinds of token mixing

def decayed_state_attention(q, k, v, decay) -> torch.Tensor:
    """``q, k (T, H, n)``, ``v (T, H, m)``, ``decay`` one number per head.  Per head ``S_t = d S_(t-1) + k_t v_t^T``
    (``S`` is ``n x m``, zero before the first token) and ``o_t = S_t^T q_t``.  Returns ``(T, H, m)``."""
    T, H, n = q.shape
    m = v.shape[2]
    out = torch.zeros(T, H, m, dtype=v.dtype)
    for h in range(H):
        S = torch.zeros(n, m, dtype=v.dtype)
        d = float(decay[h])
        for t in range(T):
            S = d * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.t() @ q[t, h]
    return out


def chunked_sink_attention(q, k, v, scale: float, size=None) -> torch.Tensor:
    """``q (T, H, n)``, ``k (T, G, n)``, ``v (T, G, m)``; query head ``h`` reads key head ``h // (H / G)``.  Position
    ``i`` sees ``j <= i`` with ``i // size == j // size`` (every ``j <= i`` without a size); the weights are
    ``exp(s_j) / (1 + sum exp(s))``.  Returns ``(T, H, m)``."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=v.dtype)
    for i in range(T):
        lo = 0 if not size else (i // int(size)) * int(size)
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            top = max(float(s.max()), 0.0)
            e = torch.exp(s - top)
            out[i, h] = (e / (math.exp(-top) + e.sum())) @ v[lo:i + 1, g]
    return out


def lightning(h, w, p, mx, eps, store=_keep):
    T = h.shape[0]
    H, n, m = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    q = store(silu(linear(h, w[p + ".q"]))).reshape(T, H, n)
    k = store(silu(linear(h, w[p + ".k"]))).reshape(T, H, n)
    v = store(silu(linear(h, w[p + ".v"]))).reshape(T, H, m)
    o = decayed_state_attention(q, k, v, mx["decay"]).reshape(T, H * m)
    o = rms(o, eps) * w[p + ".norm"]
    o = store(o * torch.sigmoid(linear(h, w[p + ".g"])))
    return store(linear(o, w[p + ".o"]))


def left_branch(h, w, p, mx, eps, positions, store=_keep):
    T = h.shape[0]
    H, G, n, m = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    rot = mx.get("rot")
    q = store(linear(h, w[p + ".q"])).reshape(T, H, n)
    k = store(linear(h, w[p + ".k"])).reshape(T, G, n)
    v = store(linear(h, w[p + ".v"])).reshape(T, G, m)
    q = rms(q, eps) * w[p + ".q.norm"]
    k = rms(k, eps) * w[p + ".k.norm"]
    if rot is not None:
        f = stretched_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = turn(q, positions, f), turn(k, positions, f)
        v = turn(v, positions, frequencies(m, float(rot["base"])))
    q, k, v = store(q), store(k), store(v)
    size = (mx.get("mask") or {}).get("size")
    o = chunked_sink_attention(q, k, v, float(mx["scale"]), size)
    if rot is not None:
        o = turn(o, positions, frequencies(m, float(rot["base"])), sign=-1.0)
    return store(linear(store(o.reshape(T, H * m)), w[p + ".o"]))


def right_branch(h, w, p, mx, eps, positions, store=_keep):
    T = h.shape[0]
    H, n, m = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    rot = mx.get("rot")
    q = store(linear(h, w[p + ".q"])).reshape(T, H, n)
    k = store(linear(h, w[p + ".k"])).reshape(T, H, n)
    v = store(linear(h, w[p + ".v"])).reshape(T, H, m)
    if rot is not None:
        f = stretched_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = turn(q, positions, f), turn(k, positions, f)
    k = k * float(n) ** -0.5
    o = rms(decayed_state_attention(q, k, v, mx["decay"]), eps).reshape(T, H * m)
    o = store(o * silu(linear(h, w[p + ".g"])))
    return store(linear(o, w[p + ".o"]))


def parallel(h, w, p, mx, eps, positions, store=_keep):
    a = left_branch(h, w, p + ".left", mx["left"], eps, positions, store)
    b = right_branch(h, w, p + ".right", mx["right"], eps, positions, store)
    return float(mx["left_scale"]) * a + float(mx["right_scale"]) * b


def layer(x, w, i, cfg, positions, store=_keep):
    """Layer ``i``: mixer and feed-forward both read the ``x`` that enters; their sum is added."""
    L = cfg["layers"][i]
    eps = float(cfg["norm"]["eps"])
    h = store(offset_norm(x, w[f"l{i}.norm1"], eps))
    if L["type"] == "lightning":
        y = lightning(h, w, f"l{i}.mix", L["mixer"], eps, store)
    elif L["type"] == "parallel":
        y = parallel(h, w, f"l{i}.mix", L["mixer"], eps, positions, store)
    else:
        raise ValueError(f"unknown layer type {L['type']!r}")
    if L.get("mlp") is not None:
        if L["mlp"]["kind"] != "dense":
            raise ValueError(f"unknown feed-forward kind {L['mlp']['kind']!r}")
        y = y + dense_ff(store(offset_norm(x, w[f"l{i}.norm2"], eps)), w, f"l{i}.mlp", store)
    return x + y


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
    eps = float(cfg["norm"]["eps"])
    x = offset_norm(embedding(w["embed"], ids), w["embed.norm"], eps)
    for i in range(len(cfg["layers"])):
        x = layer(x, w, i, cfg, positions, store)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = store(offset_norm(x, w["final.norm"], eps))
    return linear(x, w["embed"])


def greedy(cfg: dict, w: dict, prompt, max_new_tokens: int):
    ids = [int(t) for t in prompt]
    for _ in range(max_new_tokens):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids
