"""A mixture of small feed-forwards routed by a table over token ids.

Token ``t`` with id ``v`` uses the experts ``table[v, :]`` (``top`` different ones), each with weight ``1 / top``:

    y_t = (1 / top) sum_k W_down[e_k] relu(W_up[e_k] x_t)^2        e_k = table[v, k]
        + sigmoid(w_g . x_t) * W_down^s relu(W_up^s x_t)^2         (the shared expert, when the spec has one)

There is no router to compute: which experts a token uses is known from its id alone (the step's token ids are part
of every step's context).  The experts' weights are stacked at load, ``(E, F, H)`` and ``(E, H, F)``; the shared
expert's gate row is laid under its up-projection, so one product gives both.
"""
from __future__ import annotations

import torch

from .base import INDEX, MATRIX, Part, TensorSpec
from .latent_attention import _pad_rows
from .registry import register


class TableMoE(Part):
    graph_safe = True
    stage, out_stage = "moe_ffn", "ffn_down"

    @staticmethod
    def tensor_specs(spec):
        H, F = spec.hidden, spec.expert_ff
        out = {"table": TensorSpec((spec.vocab, spec.top), INDEX, "distinct", high=spec.n_experts)}
        for e in range(spec.n_experts):
            out[f"experts.{e}.up.weight"] = TensorSpec((F, H), MATRIX)
            out[f"experts.{e}.down.weight"] = TensorSpec((H, F), MATRIX)
        if spec.shared_ff is not None:
            out["shared.up.weight"] = TensorSpec((spec.shared_ff, H), MATRIX)
            out["shared.down.weight"] = TensorSpec((H, spec.shared_ff), MATRIX)
            if spec.shared_gate:
                out["shared.gate.weight"] = TensorSpec((1, H), MATRIX)
        return out

    def bind(self, tensors):
        s, rt = self.spec, self.rt
        self.table = tensors["table"].to(torch.int32).contiguous()
        if int(self.table.min()) < 0 or int(self.table.max()) >= s.n_experts:
            raise ValueError(f"the routing table names experts outside 0..{s.n_experts - 1}")
        ups = [tensors[f"experts.{e}.up.weight"] for e in range(s.n_experts)]
        downs = [tensors[f"experts.{e}.down.weight"] for e in range(s.n_experts)]
        if len({w.dtype for w in ups + downs}) > 1:
            ups, downs = [w.float() for w in ups], [w.float() for w in downs]
        self.up = torch.stack(ups, 0).contiguous()
        self.down = torch.stack(downs, 0).contiguous()
        self.w_sup = self.w_sdown = None
        if s.shared_ff is not None:
            ws = [tensors["shared.up.weight"]] + ([tensors["shared.gate.weight"].reshape(1, s.hidden)] if s.shared_gate else [])
            if len({w.dtype for w in ws}) > 1:
                ws = [w.float() for w in ws]
            self.w_sup = rt.prepare(_pad_rows(torch.cat(ws, 0)))
            self.w_sdown = rt.prepare(tensors["shared.down.weight"])

    def forward(self, x, ctx):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        x = rt.dense(x)
        shared = gate = None
        if self.w_sup is not None:
            with rt.stage("ffn_shared"):
                inner = rt.linear(x, self.w_sup)                       # [shared up | gate]
                shared = rt.linear(ops.relu_squared(inner, s.shared_ff), self.w_sdown)
                gate = inner[:, s.shared_ff:] if s.shared_gate else None
        if shared is not None and gate is None:
            # an ungated shared expert: sigmoid(large) = 1
            gate = torch.full((x.shape[0], 1), 80.0, dtype=x.dtype, device=x.device)
        # once the pairs outnumber the experts twice over, sorting them by expert reads less: each expert's weights
        # once, instead of once a pair (the option "token" keeps the token-by-token kernels for every step)
        if (x.shape[0] * s.top >= 2 * s.n_experts and rt.options.routed_experts != "token"
                and ops.moe_grouped_ok(x, self.up, self.down)):
            return ops.moe_table_grouped(x, ctx.token_ids, self.table, self.up, self.down, shared=shared, gate=gate)
        return ops.moe_table(x, ctx.token_ids, self.table, self.up, self.down, shared=shared, gate=gate)


register("ffn", "table_moe", TableMoE)
