"""Token embedding and output head.

hidden[t] = E[id_t], no scaling (src/alofa/model/arch/qwen.mojo:1391-1413).
logits = y W^T without bias or scaling, W = the head's own matrix if the file
has it, else the embedding when tied, else an error (qwen.mojo:1080-1089)."""
from __future__ import annotations

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import Part, StateNeed, build_part, register_part, tensors_of


class TokenEmbedding(Part):
    """params: name, vocab, width; optional: norm (PartSpec of a norm applied to the looked-up rows), scale (the looked-up rows
    are multiplied by it; the table itself, which a tied head reads, is not), init."""
    family = "embedding"

    @classmethod
    def tensors(cls, spec):
        out = {spec.params["name"]: TensorRule((spec.params["vocab"], spec.params["width"]), spec.params.get("init", "matrix"))}
        if spec.params.get("norm") is not None:
            out.update(tensors_of("norm", spec.params["norm"]))
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.vocab, self.width = int(spec.params["vocab"]), int(spec.params["width"])
        self.table = rt.matrix(weights[spec.params["name"]])
        self.norm = build_part("norm", spec.params["norm"], weights, rt) if spec.params.get("norm") is not None else None
        self.scale = float(spec.params.get("scale", 1.0))

    def forward(self, ctx, ids):
        hidden = ctx.scratch("hidden", (ids.shape[0], self.width), torch.float32)
        if self.scale != 1.0:
            ops.pair_embed(hidden, self.table, ids, self.scale, getattr(ctx, "token_store", None))
        else:
            ops.embed_gather(hidden, self.table, ids, getattr(ctx, "token_store", None))
        if self.norm is not None:      # (float32 rows, normed where they lie)
            self.norm.forward(hidden, hidden)
        return hidden


class PairHashEmbedding(TokenEmbedding):
    """A token's row (times ``scale``) plus a row of a second table that a hash of the token before and the token names:
    row (before * mul_prev + token * mul_cur) mod buckets, and the table's last row (number ``buckets``) for a sequence's first
    token. The token before a step's first row of a request is state of that request (one int32 per slot).
    params: as ``token_embedding``, and pairs (tensor name, [buckets + 1, width]), buckets, mul_prev, mul_cur."""
    capturable = True

    @classmethod
    def tensors(cls, spec):
        out = super().tensors(spec)
        out[spec.params["pairs"]] = TensorRule((spec.params["buckets"] + 1, spec.params["width"]), spec.params.get("init", "matrix"))
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.buckets, self.mul_prev, self.mul_cur = int(p["buckets"]), int(p["mul_prev"]), int(p["mul_cur"])
        pairs = weights[p["pairs"]]
        if pairs.dtype is not weights[p["name"]].dtype:
            raise AlofaError("invalid_argument", "the two embedding tables must share a dtype", f"{p['name']}={weights[p['name']].dtype} {p['pairs']}={pairs.dtype}")
        self.pairs = rt.matrix(pairs)

    def state_need(self):
        return StateNeed((1,), torch.int32)

    def forward(self, ctx, ids):
        from .rows import rows_of_requests
        hidden = ctx.scratch("hidden", (ids.shape[0], self.width), torch.float32)
        ops.pair_embed(hidden, self.table, ids, self.scale, getattr(ctx, "token_store", None), self.pairs, ctx.positions, ctx.state(("embedding", 0)),
                       rows_of_requests(ctx), self.buckets, self.mul_prev, self.mul_cur)
        if self.norm is not None:
            self.norm.forward(hidden, hidden)
        return hidden


class LMHead(Part):
    """params: name, tied_to (embedding tensor name or None), vocab, width; optional: scale (the logits are multiplied
    by it), softcap (then passed through cap * tanh(z / cap)), init."""
    family = "head"

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        return {p["name"]: TensorRule((p["vocab"], p["width"]), p.get("init", "matrix"), optional=p.get("tied_to") is not None)}

    def __init__(self, spec, weights, rt, embedding=None):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.vocab = int(p["vocab"])
        self.scale = float(p.get("scale", 1.0))
        self.softcap = float(p["softcap"]) if p.get("softcap") is not None else None
        if self.softcap is not None and not self.softcap > 0:
            raise AlofaError("invalid_argument", "a cap of the logits is positive", f"softcap={self.softcap}")
        if p["name"] in weights:
            self.weight = rt.matrix(weights[p["name"]])
        elif p.get("tied_to") is not None and embedding is not None:
            self.weight = embedding.table  # shared, not copied
        else:
            raise AlofaError("invalid_argument", "no output matrix: the head's tensor is absent and the embedding is not tied", f"name={p['name']}")

    def forward(self, ctx, y):
        logits = ctx.scratch("logits", (y.shape[0], self.vocab), torch.float32)
        ops.gemm(logits, y, self.weight, exact=self.rt.exact)
        if self.scale != 1.0:
            ops.scale_(logits, self.scale)
        if self.softcap is not None:
            ops.softcap_(logits, self.softcap, self.rt.exact)
        return logits

    def greedy(self, ctx, y, out, store=None, store_index=None):
        """out[r] = the first index of row r's highest logit (and store[store_index[r]], when
        given), without the logits where the product can take the argmax with it."""
        # (a positive scale moves no maximum, and neither does the cap, which rises with its argument)
        if not self.rt.exact and self.scale > 0 and ops.can_gemm_argmax(y.shape[0], self.weight):      # (a positive scale moves no maximum)
            ops.gemm_argmax(out, y, self.weight, store=store, store_index=store_index)
        else:
            ops.argmax(out, self.forward(ctx, y), store=store, store_index=store_index)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("embedding", "pair_hash_embedding", PairHashEmbedding)
register_part("head", "lm_head", LMHead)
