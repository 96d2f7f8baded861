"""Makuzen as a composition of parts: configuration -> model as data.

A decoder whose blocks add the *normed outputs* of their sub-layers to the residual stream, each scaled by one
constant (``OutNormBlockSpec``); every block's mixer is attention through low-rank latents with a shared rotated
key part, a sliding window and a per-head output gate (``LatentAttentionSpec``, rotation with slowed pairs:
``ScaledRopeSpec``); its feed-forward, where it has one, is a mixture of experts routed by a table over token ids
with a gated shared expert (``TableMoESpec``).  The embedding rows are scaled; the head is untied.

This file holds what is Makuzen's own: the tensor names and the way the typed configuration fills the parts'
sizes.  Layers may differ from one another in every size.
"""
from __future__ import annotations

from ..config.makuzen import ARCHITECTURE, MakuzenConfig
from ..config.registry import register_architecture
from ..config.spec import (LatentAttentionSpec, LayerCall, ModelSpec, OutNormBlockSpec, RMSNormSpec, ScaledRopeSpec,
                           TableMoESpec)


def makuzen_spec(cfg: MakuzenConfig) -> ModelSpec:
    W = cfg.width
    norm = RMSNormSpec(size=W, eps=cfg.norm_eps)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mx = layer.mixer
        sc = mx.scaling
        position = ScaledRopeSpec(head_dim=mx.rot_dim, rotary_dim=mx.rot_dim, theta=mx.rot_base,
                                  max_position=cfg.max_position, factor=None if sc is None else sc.factor,
                                  original=0.0 if sc is None else sc.original, fast=32.0 if sc is None else sc.fast,
                                  slow=1.0 if sc is None else sc.slow)
        mixer = LatentAttentionSpec(hidden=W, n_heads=mx.heads, plain_dim=mx.dim, rot_dim=mx.rot_dim, value_dim=mx.vdim,
                                    q_rank=mx.q_rank, kv_rank=mx.kv_rank, scale=mx.scale, eps=cfg.norm_eps,
                                    position=position, window=mx.window, gated=True)
        names = {"mixer_norm.weight": p + "norm1"}
        names.update({"mixer." + local: p + "mix." + stored for local, stored in (
            ("q_down.weight", "dq"), ("q_norm.weight", "dq.norm"), ("q_up.weight", "uq"), ("kv_down.weight", "dkv"),
            ("kv_norm.weight", "dkv.norm"), ("k_up.weight", "uk"), ("v_up.weight", "uv"), ("gate.weight", "g"),
            ("out.weight", "o"))})
        ffn = None
        if layer.mlp is not None:
            m = layer.mlp
            ffn = TableMoESpec(hidden=W, vocab=cfg.vocab, n_experts=m.experts, top=m.top, expert_ff=m.ff,
                               shared_ff=m.shared_ff, shared_gate=True)
            names["ffn_norm.weight"] = p + "norm2"
            names["ffn.table"] = p + "mlp.table"
            for e in range(m.experts):
                names[f"ffn.experts.{e}.up.weight"] = p + f"mlp.e{e}.up"
                names[f"ffn.experts.{e}.down.weight"] = p + f"mlp.e{e}.down"
            if m.shared_ff is not None:
                names.update({"ffn.shared.up.weight": p + "mlp.shared.up", "ffn.shared.down.weight": p + "mlp.shared.down",
                              "ffn.shared.gate.weight": p + "mlp.shared.sg"})
        blocks.append(OutNormBlockSpec(mixer=mixer, mixer_norm=norm, ffn=ffn, ffn_norm=norm if ffn is not None else None,
                                       mult=cfg.residual_mult, names=names))
    names = {"embed": "embed", "final_norm.weight": "final.norm", "head": "head"}
    return ModelSpec(architecture=ARCHITECTURE, hidden=W, vocab=cfg.vocab, blocks=tuple(blocks),
                     schedule=tuple(LayerCall(i) for i in range(len(blocks))), final_norm=norm, tie_embeddings=False,
                     max_position=cfg.max_position, names=names, embed_scale=cfg.embedding_scale)


register_architecture(ARCHITECTURE, MakuzenConfig.from_dict, makuzen_spec, MakuzenConfig.to_json)
