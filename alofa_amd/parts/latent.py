"""Attention over one small latent vector per token.

With x the mixer's input: q = x Wq^T (H heads of dk channels); c = norm(x Wd^T), r channels, the only thing kept per
token; per head a, k_a = Uk_a c and v_a = Uv_a c; softmax over the visible keys of scale * (q_a . k_a); the heads' outputs
side by side, multiplied by sigmoid(x Wg^T) where the design has such a gate; then the output projection. No positions.

The keys and values of a head are never formed. Since q_a . (Uk_a c) = (Uk_a^T q_a) . c and sum_j p_j Uv_a c_j =
Uv_a (sum_j p_j c_j), every head asks the same keys and values, the latents themselves, with a query of its own of r
channels, and its result is taken through Uv_a afterwards: attention with H query heads over ONE key/value head of size r,
which is what the paged attention kernels of this package do best (all heads of a key head share the keys a block reads).
The cache holds c twice, as keys [page, 1, slot, d] and as transposed values [page, 1, d, slot] (d: r widened to a size
the kernels are built for, with zeros), the layouts those kernels read."""
from __future__ import annotations

import torch

from .. import ops
from ..errors import AlofaError
from ..config.base import PartSpec
from ..weights.loader import TensorRule
from .attention import GQAAttention, _padded_heads, paged_attend
from .base import CacheNeed, Mixer, build_part, register_part, tensors_of

NAMES = {"q": "q", "down": "down", "up_k": "up_k", "up_v": "up_v", "gate": "gate", "o": "o"}


class LatentAttention(Mixer):
    """params: prefix, hidden, heads, head_dim, v_head_dim, latent (r), scale (None: 1/sqrt(head_dim)), latent_norm (PartSpec of
    the norm of the latent, an RMSNorm), gate ("sigmoid" or None), window (None or a count of keys), names (tensor names after the
    prefix for q, down, up_k, up_v, gate, o). ``forward(..., scale=)`` with a float32 vector: what is added to the stream is
    multiplied by it channel by channel."""
    capturable = True
    takes_channel_scale = True

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        n, pre, h, H, dk, dv, r = {**NAMES, **p.get("names", {})}, p["prefix"], p["hidden"], p["heads"], p["head_dim"], p["v_head_dim"], p["latent"]
        out = {pre + n["q"]: TensorRule((H * dk, h), "fan_in"), pre + n["down"]: TensorRule((r, h), "fan_in")}
        out.update(tensors_of("norm", p["latent_norm"]))
        out.update({pre + n["up_k"]: TensorRule((H * dk, r), "fan_in"), pre + n["up_v"]: TensorRule((H * dv, r), "fan_in")})
        if p.get("gate") is not None:
            out[pre + n["gate"]] = TensorRule((H * dv, h), "fan_in")
        out[pre + n["o"]] = TensorRule((h, H * dv), "fan_in")
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        n, pre = {**NAMES, **p.get("names", {})}, p["prefix"]
        self.hidden, self.heads, self.dk, self.dv, self.r = int(p["hidden"]), int(p["heads"]), int(p["head_dim"]), int(p["v_head_dim"]), int(p["latent"])
        self.window = p.get("window")
        if p.get("gate") not in (None, "sigmoid"):
            raise AlofaError("unsupported", "no such gate is built", f"gate={p['gate']}")
        # the one head size of the attention kernels: the latent's, widened to a size they are built for
        self.d = GQAAttention.common_head_size(self.r, self.r)
        if self.d not in ops.PREFILL_HEAD_DIMS:
            self.d = next((s for s in ops.PREFILL_HEAD_DIMS if s >= self.d), self.d)
        if self.d > ops.MAX_HEAD_DIM:
            raise AlofaError("unsupported", f"the attention kernels take latents of up to {ops.MAX_HEAD_DIM} channels", f"latent={self.r}")
        H, dk, dv, r, d = self.heads, self.dk, self.dv, self.r, self.d
        self.scale = float(p["scale"]) if p.get("scale") is not None else dk ** -0.5
        mats = [weights[pre + n["q"]]] + ([weights[pre + n["gate"]]] if p.get("gate") is not None else [])
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.gated = p.get("gate") is not None
        self.w_in = rt.matrix(torch.cat(mats, dim=0))          # queries and gates in one product
        self.w_down = rt.matrix(weights[pre + n["down"]])
        norm = p.get("latent_norm")
        self.norm = build_part("norm", norm, weights, rt).as_rmsnorm() if norm is not None else None
        if self.norm is None:
            raise AlofaError("unsupported", "the latent's norm is an RMSNorm", f"norm={norm.kind if norm is not None else None}")
        # per head [out, in]: a query into the latent's channels (Uk_a^T, [d, dk], zero rows beyond r) and a result out of them (Uv_a, [dv, d], zero columns beyond r)
        uk = weights[pre + n["up_k"]].reshape(H, dk, r).transpose(1, 2)
        self.w_query = rt.matrix(torch.cat([uk, torch.zeros(H, d - r, dk, dtype=uk.dtype)], dim=1).contiguous())
        uv = weights[pre + n["up_v"]].reshape(H, dv, r)
        self.w_result = rt.matrix(torch.cat([uv, torch.zeros(H, dv, d - r, dtype=uv.dtype)], dim=2).contiguous())
        self.w_o = rt.matrix(weights[pre + n["o"]])
        self.position = build_part("position", PartSpec("none", {"head_dim": d}), weights, rt)

    def cache_need(self):
        return CacheNeed.keys_and_values(1, self.d, self.window)

    def prepare(self, n_positions):
        self.position.table(n_positions)

    def forward(self, ctx, where, x, residual, scale=None, out=None):
        T, exact, H, d = residual.shape[0], self.rt.exact, self.heads, self.d
        qg = ctx.scratch("latent_in", (T, self.w_in.shape[0]), self.rt.dtype)
        ops.gemm(qg, x, self.w_in, exact=exact)
        down = ctx.scratch("latent_down", (T, self.r), torch.float32)
        ops.gemm(down, x, self.w_down, exact=exact)
        # [a query per head | the latent as key | the latent as value]
        qkv = ctx.scratch("qkv", (T, (H + 2) * d), self.rt.dtype)
        w, eps = self.norm
        ops.rmsnorm_spread(qkv[:, H * d:], down, w, eps, d, 2, exact)
        ops.head_project(qkv[:, :H * d], qg[:, :H * self.dk], self.w_query, exact)
        attn = ctx.scratch("attn", (T, H * d), self.rt.dtype)
        paged_attend(ctx, where, qkv, attn, H, 1, d, self.window, self.scale, self.position, self.rt)
        heads_out = ctx.scratch("latent_out", (T, H * self.dv), self.rt.dtype)
        ops.head_project(heads_out, attn, self.w_result, exact, gate=qg[:, H * self.dk:] if self.gated else None)
        if out is not None:
            ops.gemm(out, heads_out, self.w_o, exact=exact)
        elif scale is None:
            ops.gemm(residual, heads_out, self.w_o, add_to_out=True, exact=exact)
        else:
            ops.gemm_channel_scaled(residual, heads_out, self.w_o, scale, ctx.scratch("sub_out", tuple(residual.shape), torch.float32), exact)


register_part("mixer", "latent_attention", LatentAttention)
