"""Attention over one small latent vector per token.

With x the mixer's input: q = x Wq^T (H heads of dk channels); c = norm(x Wd^T), r channels, the only thing kept per
token; per head a, k_a = Uk_a c and v_a = Uv_a c; softmax over the visible keys of scale * (q_a . k_a); the heads' outputs
side by side, multiplied by sigmoid(x Wg^T) where the design has such a gate; then the output projection. No positions.

The keys and values of a head are never formed. Since q_a . (Uk_a c) = (Uk_a^T q_a) . c and sum_j p_j Uv_a c_j =
Uv_a (sum_j p_j c_j), every head asks the same keys and values, the latents themselves, with a query of its own of r
channels, and its result is taken through Uv_a afterwards: attention with H query heads over ONE key/value head of size r,
which is what the paged attention kernels of this package do best (all heads of a key head share the keys a block reads).
The cache holds c twice, as keys [page, 1, slot, d] and as transposed values [page, 1, d, slot] (d: r widened to a size
the kernels are built for, with zeros), the layouts those kernels read.

A latent wider than the largest head the kernels take cannot be a head: there the keys and values of every head are formed
from c when it is made (k_a = Uk_a c, v_a = Uv_a c) and kept per head in the pages, as for any attention with H key heads."""
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
    prefix for q, down, up_k, up_v, gate, o); optional: keep ("latent", the default: the pages hold the latent where the kernels take
    its size; "heads": they hold every head's keys and values). ``forward(..., scale=)`` with a float32 vector: what is added to the stream is
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
        H, dk, dv, r = self.heads, self.dk, self.dv, self.r
        self.scale = float(p["scale"]) if p.get("scale") is not None else dk ** -0.5
        self.gated = p.get("gate") is not None
        norm = p.get("latent_norm")
        self.norm = build_part("norm", norm, weights, rt).as_rmsnorm() if norm is not None else None
        if self.norm is None:
            raise AlofaError("unsupported", "the latent's norm is an RMSNorm", f"norm={norm.kind if norm is not None else None}")
        self.w_down = rt.matrix(weights[pre + n["down"]])
        # the one head size of the attention kernels: the latent's, widened to a size they are built for
        d = GQAAttention.common_head_size(r, r)
        if d not in ops.PREFILL_HEAD_DIMS:
            d = next((s for s in ops.PREFILL_HEAD_DIMS if s >= d), d)
        self.latent_heads = d <= ops.MAX_HEAD_DIM and p.get("keep", "latent") == "latent"
        w_q, w_g, w_o = weights[pre + n["q"]], weights[pre + n["gate"]] if self.gated else None, weights[pre + n["o"]]
        if self.latent_heads:
            # per head [out, in]: a query into the latent's channels (Uk_a^T, [d, dk], zero rows beyond r) and a result out of them (Uv_a, [dv, d], zero columns beyond r)
            uk = weights[pre + n["up_k"]].reshape(H, dk, r).transpose(1, 2)
            self.w_query = rt.matrix(torch.cat([uk, torch.zeros(H, d - r, dk, dtype=uk.dtype, device=uk.device)], dim=1).contiguous())
            uv = weights[pre + n["up_v"]].reshape(H, dv, r)
            self.w_result = rt.matrix(torch.cat([uv, torch.zeros(H, dv, d - r, dtype=uv.dtype, device=uv.device)], dim=2).contiguous())
            self.kv_heads = 1
        else:
            # keys and values per head, every head widened to one size with zero rows (zero columns of the output matrix)
            d = GQAAttention.common_head_size(dk, dv)
            if d > ops.MAX_HEAD_DIM:
                raise AlofaError("unsupported", f"the attention kernels take heads of up to {ops.MAX_HEAD_DIM} channels", f"head_dim={dk} v_head_dim={dv}")
            w_q = _padded_heads(w_q, H, dk, d)
            self.w_kv = rt.matrix(torch.cat([_padded_heads(weights[pre + n["up_k"]], H, dk, d), _padded_heads(weights[pre + n["up_v"]], H, dv, d)], dim=0))
            if d != dv:
                w_g = _padded_heads(w_g, H, dv, d) if self.gated else None
                w_o = _padded_heads(w_o.t(), H, dv, d).t()
            self.kv_heads = H
        self.d = d
        self.w_q = rt.matrix(w_q)
        self.w_gate = rt.matrix(w_g) if self.gated else None
        w_d = weights[pre + n["down"]]
        if self.latent_heads and w_q.dtype is w_d.dtype and (not self.gated or w_g.dtype is w_q.dtype):      # queries, gates and the latent in one product
            self.w_in = rt.matrix(torch.cat([w_q] + ([w_g] if self.gated else []) + [w_d], dim=0))
        else:
            self.w_in = None
        self.w_o = rt.matrix(w_o)
        self.position = build_part("position", PartSpec("none", {"head_dim": d}), weights, rt)

    def cache_need(self):
        return CacheNeed.keys_and_values(self.kv_heads, self.d, self.window)

    def prepare(self, n_positions):
        self.position.table(n_positions)

    def _latent(self, ctx, x, out, pad, copies, down=None):
        """The step's latents, normed, ``copies`` times side by side in ``out`` (each widened to ``pad`` channels with zeros)."""
        if down is None:
            down = ctx.scratch("latent_down", (x.shape[0], self.r), torch.float32)
            ops.gemm(down, x, self.w_down, exact=self.rt.exact)
        w, eps = self.norm
        ops.rmsnorm_spread(out, down, w, eps, pad, copies, self.rt.exact)

    def fuses_norm(self, norm, rows):
        return (self.w_in is not None and not self.rt.exact and norm.as_rmsnorm() is not None and ops.can_fuse_norm(rows, self.w_in, self.rt.dtype))

    def forward(self, ctx, where, x, residual, scale=None, out=None, norm=None, then=None):
        """``norm``: x is None and the mixer's input is this norm of the residual's rows, applied by the first product. ``then`` =
        (weight, eps, rows): the RMSNorm of the residual's new rows is left in ``rows`` (with ``scale``)."""
        T, exact, H, d = residual.shape[0], self.rt.exact, self.heads, self.d
        attn = ctx.scratch("attn", (T, H * d), self.rt.dtype)
        down = None
        if self.latent_heads:
            if self.w_in is not None:
                qg = ctx.scratch("latent_in", (T, self.w_in.shape[0]), self.rt.dtype)
                if norm is not None:
                    ops.gemm(qg, residual, self.w_in, norm=norm.as_rmsnorm())
                else:
                    ops.gemm(qg, x, self.w_in, exact=exact)
                q, gate = qg[:, :H * self.dk], (qg[:, H * self.dk:H * (self.dk + self.dv)] if self.gated else None)
                down = qg[:, qg.shape[1] - self.r:]
            else:
                q, gate = ctx.scratch("latent_q", (T, H * self.dk), self.rt.dtype), None
                ops.gemm(q, x, self.w_q, exact=exact)
                if self.gated:
                    gate = ctx.scratch("latent_gate", (T, H * self.dv), self.rt.dtype)
                    ops.gemm(gate, x, self.w_gate, exact=exact)
            # [a query per head | the latent as key | the latent as value]
            qkv = ctx.scratch("qkv", (T, (H + 2) * d), self.rt.dtype)
            self._latent(ctx, x, qkv[:, H * d:], d, 2, down)
            ops.head_project(qkv[:, :H * d], q, self.w_query, exact)
            paged_attend(ctx, where, qkv, attn, H, 1, d, self.window, self.scale, self.position, self.rt)
            heads_out = ctx.scratch("latent_out", (T, H * self.dv), self.rt.dtype)
            ops.head_project(heads_out, attn, self.w_result, exact, gate=gate)
        else:
            qkv = ctx.scratch("qkv", (T, 3 * H * d), self.rt.dtype)
            ops.gemm(qkv[:, :H * d], x, self.w_q, exact=exact)
            c = ctx.scratch("latent", (T, self.r), self.rt.dtype)
            self._latent(ctx, x, c, self.r, 1)
            ops.gemm(qkv[:, H * d:], c, self.w_kv, exact=exact)
            paged_attend(ctx, where, qkv, attn, H, H, d, self.window, self.scale, self.position, self.rt)
            if self.gated:
                gate = ctx.scratch("latent_gate", (T, H * d), self.rt.dtype)
                ops.gemm(gate, x, self.w_gate, exact=exact)
                ops.sigmoid_gate(attn, gate, exact)
            heads_out = attn
        if out is not None:
            ops.gemm(out, heads_out, self.w_o, exact=exact)
        elif scale is None:
            ops.gemm(residual, heads_out, self.w_o, add_to_out=True, exact=exact)
        else:
            ops.gemm_channel_scaled(residual, heads_out, self.w_o, scale, ctx.scratch("sub_out", tuple(residual.shape), torch.float32), exact, then_norm=then)


register_part("mixer", "latent_attention", LatentAttention)
