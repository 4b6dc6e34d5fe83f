"""Feed-forwards of which a token takes a few: a router scores the experts, the token takes the best ``top`` of them, and
what they give is summed with weights that follow from the scores; an expert that every token takes may stand beside them.

Router: z = x W_r^T in float32; the score is sigmoid(z); the ``top`` largest are taken (the lower index among equals);
the weights are the taken scores (made to sum to one first where the design says so) times ``weight_scale``.
Expert ("clamped_glu"): a = min(gate(x), limit), b = clamp(up(x), -limit, limit); down(a sigmoid(slope a) (b + 1)).

The experts' matrices lie side by side in one tensor each (gate and up by rows, down by columns, the shared expert's
last), so that every expert is a slice of them."""
from __future__ import annotations

import os

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import FeedForward, register_part


SPARSE_EXPERTS = os.environ.get("ALOFA_SPARSE_EXPERTS", "1") != "0"      # 0 (for measurements): every expert against every row


class RoutedExperts(FeedForward):
    """params: prefix, hidden, experts, top, score ("sigmoid"), weight_scale, renormalize, expert {intermediate, limit},
    shared (the same, or None), activation ("clamped_glu"), slope, names (after the prefix: router; expert, a pattern with {}
    for the expert's number; shared; gate, up, down after an expert's name and a dot).
    ``forward(..., scale=)`` with a float32 vector: what is added to the stream is multiplied by it channel by channel."""
    capturable = True
    takes_channel_scale = True

    @staticmethod
    def _expert_names(p, e) -> dict:
        n = p["names"]
        stem = p["prefix"] + (n["shared"] if e is None else n["expert"].format(e)) + "."
        return {k: stem + n[k] for k in ("gate", "up", "down")}

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        h = p["hidden"]
        out = {}
        for e in range(p["experts"]):
            names, i = cls._expert_names(p, e), p["expert"]["intermediate"]
            out.update({names["gate"]: TensorRule((i, h), "fan_in"), names["up"]: TensorRule((i, h), "fan_in"), names["down"]: TensorRule((h, i), "fan_in")})
        out[p["prefix"] + p["names"]["router"]] = TensorRule((p["experts"], h), "fan_in")
        if p.get("shared") is not None:
            names, i = cls._expert_names(p, None), p["shared"]["intermediate"]
            out.update({names["gate"]: TensorRule((i, h), "fan_in"), names["up"]: TensorRule((i, h), "fan_in"), names["down"]: TensorRule((h, i), "fan_in")})
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        if p.get("score", "sigmoid") != "sigmoid" or p.get("activation", "clamped_glu") != "clamped_glu":
            raise AlofaError("unsupported", "no such router score or expert activation is built", f"score={p.get('score')} activation={p.get('activation')}")
        self.hidden, self.experts, self.top = int(p["hidden"]), int(p["experts"]), int(p["top"])
        if not 0 < self.top <= self.experts <= ops.MAX_EXPERTS:
            raise AlofaError("unsupported", f"a token takes 1..experts experts of at most {ops.MAX_EXPERTS}", f"experts={self.experts} top={self.top}")
        self.weight_scale, self.renormalize, self.slope = float(p.get("weight_scale", 1.0)), bool(p.get("renormalize", False)), float(p.get("slope", 1.0))
        self.ff, self.limit = int(p["expert"]["intermediate"]), float(p["expert"]["limit"])
        shared = p.get("shared")
        self.shared_ff, self.shared_limit = (int(shared["intermediate"]), float(shared["limit"])) if shared is not None else (0, 0.0)
        who = list(range(self.experts)) + ([None] if shared is not None else [])
        names = [self._expert_names(p, e) for e in who]
        self.w_gate = rt.matrix(torch.cat([weights[n["gate"]] for n in names], dim=0))
        self.w_up = rt.matrix(torch.cat([weights[n["up"]] for n in names], dim=0))
        self.w_down = rt.matrix(torch.cat([weights[n["down"]] for n in names], dim=1))
        self.w_router = rt.matrix(weights[p["prefix"] + p["names"]["router"]])
        self.channels = self.experts * self.ff + self.shared_ff

    def route(self, ctx, x):
        """(dense [T, E], chosen [T, top], weights [T, top]) of the step's rows."""
        T = x.shape[0]
        z = ctx.scratch("router_z", (T, self.experts), torch.float32)
        ops.gemm(z, x, self.w_router, exact=self.rt.exact)
        dense = ctx.scratch("router_dense", (T, self.experts), torch.float32)
        chosen, weights = ctx.scratch("router_chosen", (T, self.top), torch.int32), ctx.scratch("router_weights", (T, self.top), torch.float32)
        ops.route_top(z, dense, chosen, weights, self.top, self.weight_scale, self.renormalize, self.rt.exact)
        return dense, chosen, weights

    def sparse(self, x) -> bool:
        """Whether the experts run slot by slot (every row against the experts it takes only) rather than all of them against
        every row with weights of zero: where a token leaves at least half of the experts out, and the kernel takes the sizes."""
        return (SPARSE_EXPERTS and not self.rt.exact and 2 * self.top <= self.experts
                and ops.can_group_experts(x, self.w_gate, self.ff, self.shared_ff))

    def forward(self, ctx, x, residual, scale=None):
        T, exact = residual.shape[0], self.rt.exact
        dense, chosen, weights = self.route(ctx, x)
        if self.sparse(x):
            rows = ops.ExpertRows(T, self.top, self.experts, self.shared_ff > 0, ctx.scratch)
            ops.expert_rows(rows, chosen, weights)
            act = ctx.scratch("experts_act", (rows.slots, (max(self.ff, self.shared_ff) + 7) // 8 * 8), torch.bfloat16)
            ops.experts_gate_up(act, x, self.w_gate, self.w_up, rows, self.ff, self.shared_ff, self.limit, self.shared_limit, self.slope)
            y = ctx.scratch("experts_out", (rows.slots, self.hidden), torch.float32)
            ops.experts_down(y, act, self.w_down, rows, self.ff, self.shared_ff)
            ops.experts_sum(residual, y, rows, scale)
            return
        # every expert's gate and up for every row, the rows an expert is not taken by weighted with zero
        g, u = ctx.scratch("experts_gate", (T, self.channels), self.rt.dtype), ctx.scratch("experts_up", (T, self.channels), self.rt.dtype)
        ops.gemm(g, x, self.w_gate, exact=exact)
        ops.gemm(u, x, self.w_up, exact=exact)
        act = ctx.scratch("ff_act", (T, self.channels), self.rt.dtype)
        ops.clamped_glu(act, g, u, dense, self.experts, self.ff, self.shared_ff, self.limit, self.shared_limit, self.slope, exact)
        if scale is None:
            ops.gemm(residual, act, self.w_down, add_to_out=True, exact=exact)
        else:
            ops.gemm_channel_scaled(residual, act, self.w_down, scale, ctx.scratch("sub_out", tuple(residual.shape), torch.float32), exact)


register_part("feed_forward", "routed_experts", RoutedExperts)
