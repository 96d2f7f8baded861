"""Fazezen as a composition of parts: configuration -> model as data.

A decoder whose blocks feed one stream to a mixer and a feed-forward at once, each through its own norm, and add both
results (``ParallelBlockSpec``).  A block's mixer is either linear attention through a fading matrix state with
activated projections, a joint output norm and a sigmoid gate (``lightning``), or a pair of mixers side by side
(``parallel``, ``MixerPairSpec``): grouped-query softmax attention within runs of positions, with a sink term, head
norms, stretched rotation and values that are cached turned (``AttentionSpec``), beside retention, the same fading
state with turned queries and keys, a norm per head and a silu gate (``LinearAttentionSpec``).  The feed-forward is a
gated one with the tanh form of gelu and biases (``GatedMLPSpec``).  Every norm of the stream stores its weight
around zero; the embedding rows are normed before the first block; the embedding table is the head.

This file holds what is Fazezen's own: the tensor names and the way the typed configuration fills the parts'
sizes.  Layers may differ from one another in every size.
"""
from __future__ import annotations

from ..config.fazezen import ARCHITECTURE, LIGHTNING, FazezenConfig
from ..config.registry import register_architecture
from ..config.spec import (AttentionSpec, GatedMLPSpec, LayerCall, LinearAttentionSpec, MixerPairSpec, ModelSpec,
                           NoPositionSpec, ParallelBlockSpec, RMSNormSpec, RopeSpec, StretchedRopeSpec)


def _rotation(rot, head_dim: int, max_position: int):
    if rot is None or rot.dims == 0:
        return NoPositionSpec()
    s = rot.scaling
    if s is None:
        return RopeSpec(head_dim=head_dim, rotary_dim=rot.dims, theta=rot.base, max_position=max_position)
    return StretchedRopeSpec(head_dim=head_dim, rotary_dim=rot.dims, theta=rot.base, max_position=max_position,
                             factor=s.factor, original=s.original, low=s.low, high=s.high)


def _lightning(mx, W, eps, p):
    spec = LinearAttentionSpec(hidden=W, n_heads=mx.heads, key_dim=mx.dim, value_dim=mx.vdim, decay=mx.decay, eps=eps,
                               activation="silu", out_norm="joint", gate="sigmoid")
    names = {local: p + stored for local, stored in (
        ("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("gate_proj.weight", "g"),
        ("out_proj.weight", "o"), ("out_norm.weight", "norm"))}
    return spec, names


def _pair(mx, W, eps, p, max_position):
    le, ri = mx.left, mx.right
    turned = le.rot is not None
    left = AttentionSpec(hidden=W, n_heads=le.heads, n_kv_heads=le.kv_heads, head_dim=le.dim,
                         position=_rotation(le.rot, le.dim, max_position), qk_norm=RMSNormSpec(size=le.dim, eps=eps),
                         scale=le.scale, value_dim=le.vdim, chunk=le.chunk, sink=True,
                         value_position=RopeSpec(head_dim=le.vdim, rotary_dim=le.vdim, theta=le.rot.base,
                                                 max_position=max_position) if turned else None)
    right = LinearAttentionSpec(hidden=W, n_heads=ri.heads, key_dim=ri.dim, value_dim=ri.vdim, decay=ri.decay, eps=eps,
                                position=_rotation(ri.rot, ri.dim, max_position), activation=None,
                                key_scale=float(ri.dim) ** -0.5, out_norm="head", gate="silu")
    names = {"left." + local: p + "left." + stored for local, stored in (
        ("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("q_norm.weight", "q.norm"),
        ("k_norm.weight", "k.norm"), ("out_proj.weight", "o"))}
    names.update({"right." + local: p + "right." + stored for local, stored in (
        ("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("gate_proj.weight", "g"),
        ("out_proj.weight", "o"))})
    return MixerPairSpec(left=left, right=right, left_scale=mx.left_scale, right_scale=mx.right_scale), names


def fazezen_spec(cfg: FazezenConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps
    norm = RMSNormSpec(size=W, eps=eps, offset=1.0)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        if layer.type == LIGHTNING:
            mixer, local = _lightning(layer.mixer, W, eps, p + "mix.")
        else:
            mixer, local = _pair(layer.mixer, W, eps, p + "mix.", cfg.max_position)
        names = {"mixer_norm.weight": p + "norm1"}
        names.update({"mixer." + k: v for k, v in local.items()})
        ffn = None
        if layer.mlp is not None:
            ffn = GatedMLPSpec(hidden=W, intermediate=layer.mlp.ff, activation="gelu_tanh", bias=True)
            names["ffn_norm.weight"] = p + "norm2"
            for local_name, stored in (("gate", "gate"), ("up", "up"), ("down", "down")):
                names[f"ffn.{local_name}.weight"] = p + "mlp." + stored
                names[f"ffn.{local_name}.bias"] = p + "mlp." + stored + ".b"
        blocks.append(ParallelBlockSpec(mixer=mixer, mixer_norm=norm, ffn=ffn, ffn_norm=norm if ffn is not None else None,
                                        names=names))
    names = {"embed": "embed", "embed_norm.weight": "embed.norm", "final_norm.weight": "final.norm"}
    # a file may hold the second norm of a layer without a feed-forward; nobody reads it
    return ModelSpec(architecture=ARCHITECTURE, hidden=W, vocab=cfg.vocab, blocks=tuple(blocks),
                     schedule=tuple(LayerCall(i) for i in range(len(blocks))), final_norm=norm, tie_embeddings=True,
                     max_position=cfg.max_position, names=names, embed_norm=norm, ignored_tensors=(".norm2",))


register_architecture(ARCHITECTURE, FazezenConfig.from_dict, fazezen_spec, FazezenConfig.to_json)
