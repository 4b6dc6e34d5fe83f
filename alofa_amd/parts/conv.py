"""A short causal convolution over time in front of a sub-layer: what the sub-layer reads, h, becomes
h + conv(h) with conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j) on every channel by itself, zeros before a
request's first token. The last taps - 1 rows of h are the part's state per request, so a request's rows may
arrive in any portions."""
from __future__ import annotations

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import StateNeed, TimeConv, register_part
from .rows import rows_of_requests


class ShortCausalConv(TimeConv):
    """params: name (tensor [width, taps], no bias), width, taps."""
    capturable = True   # native kernels on the current stream only

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        return {p["name"]: TensorRule((p["width"], p["taps"]), "filter")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.width, self.taps = int(spec.params["width"]), int(spec.params["taps"])
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise AlofaError("unsupported", f"the convolution kernel takes 1 to {ops.CONV_MAX_TAPS} taps", f"taps={self.taps}")
        self.weight = rt.vector(weights[spec.params["name"]])

    def state_need(self):
        return StateNeed((self.taps - 1, self.width), torch.float32) if self.taps > 1 else None

    def fuses_norm(self, ctx, norm):
        # single rows (decoding): norm, filter and the state's step are one launch
        return ctx.max_q_len == 1 and self.taps > 1 and norm.as_layernorm() is not None

    def forward(self, ctx, where, out, x, norm=None):
        """out = x + conv(x) for float32 rows x (with ``norm``: for the norm of the rows x); the state moves on by this step's rows."""
        if norm is not None:
            weight, bias, eps = norm.as_layernorm()
            ops.norm_conv_step(out, x, weight, bias, eps, self.weight, ctx.state(where), rows_of_requests(ctx), self.rt.exact)
            return
        if self.taps == 1:      # a filter of one tap sees the row itself only
            state = ctx.scratch("conv_no_state", (ctx.fn.cache.max_requests, 0, self.width), torch.float32)
            ops.short_conv(out, x, self.weight, state, rows_of_requests(ctx), self.rt.exact)
            return
        state = ctx.state(where)
        rows = rows_of_requests(ctx)
        ops.short_conv(out, x, self.weight, state, rows, self.rt.exact)
        ops.keep_last_rows(state, x, rows)


register_part("conv", "short_causal", ShortCausalConv)
