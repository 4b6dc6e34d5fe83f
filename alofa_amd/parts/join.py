"""Joins: what a run entry may ask for in front of it, on the stream and the embedding's output.

concat_projection: x <- W [x | x0], W [h, 2h] with the stream's half first, x0 the embedding's output. Both halves are
one product's operand (rounded to the activation dtype, float32 accumulation); the result replaces the stream."""
from __future__ import annotations

import torch

from .. import ops
from ..weights.loader import TensorRule
from .base import Join, register_part


class ConcatProjection(Join):
    """params: name (the tensor, [width, 2 width]), width."""
    capturable = True

    @classmethod
    def tensors(cls, spec):
        h = spec.params["width"]
        return {spec.params["name"]: TensorRule((h, 2 * h), "fan_in")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.width = int(spec.params["width"])
        self.weight = rt.matrix(weights[spec.params["name"]])

    def forward(self, ctx, hidden, first):
        both = ctx.scratch("joined", (hidden.shape[0], 2 * self.width), self.rt.dtype)
        ops.concat_rows(both, hidden, first)
        ops.gemm(hidden, both, self.weight, exact=self.rt.exact)


register_part("join", "concat_projection", ConcatProjection)
