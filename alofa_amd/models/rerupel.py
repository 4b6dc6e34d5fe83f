"""Rerupel: a decoder whose layers are listed one by one in config.json; attention over one small latent vector per
token, dense or routed feed-forwards, a run of layers that is passed through several times.

config.json: ``architecture`` "Rerupel"; ``vocab``, ``width``; ``norm.eps``; ``residual_mult``; ``logit_softcap``;
``embedding``: {``scale``, ``bigram``: {``buckets``, ``mul_prev``, ``mul_cur``}}; ``loop``: {``start``, ``stop``, ``times``};
``layers``: a list of {``type``, ``mixer``, ``mlp``}. Tensor names: ``embed``, ``bigram``, ``loop.in``, ``l<i>.`` +
``norm1``/``norm2``, ``ls1``/``ls2``, ``mix.*``, ``mlp.*``; ``final.norm``.

The model: a token's row of ``embed`` times ``embedding.scale``, plus the row of ``bigram`` that a hash of (token
before, token) names (the table's last row for a sequence's first token). A layer is pre-norm (RMSNorm); what a
sub-layer gives is multiplied channel by channel by the layer's ``ls1`` / ``ls2`` and by ``residual_mult`` before it is
added to the stream. The layers ``loop.start`` .. ``loop.stop`` - 1 run ``loop.times`` times one after the other with the same
weights (every pass keeps a cache of its own); what a pass starts from is ``loop.in`` [width, 2 width] applied to the
stream beside the embedding's output. The logits are the embedding table's product with the final norm's rows, passed
through cap * tanh(z / cap).

Mixer by ``type``:
  latent_attention  ``heads`` x (``dim``, ``vdim``), a latent of ``kv_rank`` channels (RMSNorm with a weight of its own), scores times
                    ``scale``, no positions; the heads' outputs gated by a sigmoid of a projection of the mixer's input.
Feed-forward by ``mlp.kind`` (``mlp`` null: none):
  dense  two matrices, ``ff`` wide, the square of relu between them.
  moe    ``router.experts`` gated feed-forwards of ``expert.ff`` channels with values clamped at ``expert.limit``, of which a
         token takes the ``router.top`` with the largest sigmoid scores, weighted by score times ``router.scale``; and
         optionally one of the same form that every token takes (``shared``: ``ff``, ``limit``)."""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional

from ..config.base import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry
from ..errors import AlofaError
from .tugalix import _get, _positive

MIXERS = ("latent_attention",)


def _mixer(kind: str, m: dict, where: str) -> dict:
    out = {k: _get(m, k, int, where) for k in ("heads", "dim", "vdim", "kv_rank")}
    _positive(where, **out)
    out["scale"] = _get(m, "scale", float, where)
    return out


def _gated(m: dict, where: str) -> dict:
    out = {"ff": _get(m, "ff", int, where), "limit": _get(m, "limit", float, where)}
    _positive(where, **out)
    return out


def _mlp(mlp, where: str):
    if mlp is None:
        return None
    kind = _get(mlp, "kind", str, where)
    if kind == "dense":
        out = {"kind": "dense", "ff": _get(mlp, "ff", int, where)}
        _positive(where, ff=out["ff"])
        return out
    if kind != "moe":
        raise AlofaError("unsupported", "no such feed-forward in this design", f"kind={kind} config={where}")
    r = _get(mlp, "router", dict, where)
    router = {"experts": _get(r, "experts", int, where), "top": _get(r, "top", int, where), "scale": _get(r, "scale", float, where)}
    _positive(where, experts=router["experts"], top=router["top"])
    if router["top"] > router["experts"]:
        raise AlofaError("parse", "a token cannot take more experts than there are", f"top={router['top']} experts={router['experts']} config={where}")
    shared = mlp.get("shared")
    return {"kind": "moe", "router": router, "expert": _gated(_get(mlp, "expert", dict, where), where),
            "shared": None if shared is None else _gated(shared, where)}


@dataclass(frozen=True)
class RerupelConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    residual_mult: float
    logit_softcap: float
    embed_scale: float
    bigram: Optional[tuple]      # (buckets, mul_prev, mul_cur), or None: no pair table
    loop: Optional[tuple]        # (start, stop, times), or None: every layer once
    layers: tuple                # per layer a dict {type, mixer, mlp}, checked

    architecture = "Rerupel"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "<dict>") -> "RerupelConfig":
        layers = []
        for i, l in enumerate(_get(raw, "layers", list, where)):
            at = f"{where} layers[{i}]"
            kind = _get(l, "type", str, at)
            if kind not in MIXERS:
                raise AlofaError("unsupported", "no such mixer in this design", f"type={kind} known={','.join(MIXERS)} config={at}")
            layers.append({"type": kind, "mixer": _mixer(kind, _get(l, "mixer", dict, at), at), "mlp": _mlp(l.get("mlp"), at)})
        if not layers:
            raise AlofaError("parse", "a model has at least one layer", f"config={where}")
        emb = _get(raw, "embedding", dict, where)
        bigram = emb.get("bigram")
        if bigram is not None:
            bigram = (_get(bigram, "buckets", int, where), _get(bigram, "mul_prev", int, where), _get(bigram, "mul_cur", int, where))
            _positive(where, buckets=bigram[0])
        loop = raw.get("loop")
        if loop is not None:
            loop = (_get(loop, "start", int, where), _get(loop, "stop", int, where), _get(loop, "times", int, where))
            if not (0 <= loop[0] < loop[1] <= len(layers) and loop[2] >= 1):
                raise AlofaError("parse", "loop names a run of existing layers and a positive count", f"loop={loop} layers={len(layers)} config={where}")
        cfg = cls(vocab=_get(raw, "vocab", int, where), width=_get(raw, "width", int, where), eps=_get(_get(raw, "norm", dict, where), "eps", float, where),
                  residual_mult=_get(raw, "residual_mult", float, where), logit_softcap=_get(raw, "logit_softcap", float, where),
                  embed_scale=_get(emb, "scale", float, where), bigram=bigram, loop=loop, layers=tuple(layers))
        _positive(where, vocab=cfg.vocab, width=cfg.width, eps=cfg.eps, logit_softcap=cfg.logit_softcap)
        return cfg

    def to_dict(self) -> dict:
        emb = {"scale": self.embed_scale}
        if self.bigram is not None:
            emb["bigram"] = dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps}, "residual_mult": self.residual_mult,
               "logit_softcap": self.logit_softcap, "embedding": emb, "layers": copy.deepcopy(list(self.layers))}
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return out

    # ---- the model as data
    def _norm(self, name: str, width: Optional[int] = None) -> PartSpec:
        return PartSpec("rmsnorm", {"name": name, "width": width or self.width, "eps": self.eps})

    def _feed_forward(self, mlp, pre: str) -> Optional[PartSpec]:
        h = self.width
        if mlp is None:
            return None
        if mlp["kind"] == "dense":
            return PartSpec("dense_activated", {"prefix": pre, "hidden": h, "intermediate": mlp["ff"], "activation": "relu_squared", "names": {"up": "up", "down": "down"}})

        def gated(m):
            return {"intermediate": m["ff"], "limit": m["limit"]}
        r = mlp["router"]
        return PartSpec("routed_experts", {
            "prefix": pre, "hidden": h, "experts": r["experts"], "top": r["top"], "score": "sigmoid", "weight_scale": r["scale"], "renormalize": False,
            "expert": gated(mlp["expert"]), "shared": None if mlp["shared"] is None else gated(mlp["shared"]), "activation": "clamped_glu", "slope": 1.702,
            "names": {"router": "router", "expert": "e{}", "shared": "shared", "gate": "gate", "up": "up", "down": "down"}})

    def run_order(self) -> tuple:
        """(layer, whether a pass starts here) per run."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, False) for i in range(n))
        a, b, times = self.loop
        return (tuple((i, False) for i in range(a)) + tuple((i, i == a) for _ in range(times) for i in range(a, b))
                + tuple((i, False) for i in range(b, n)))

    def spec(self) -> ModelSpec:
        h = self.width
        layers = []
        for i, l in enumerate(self.layers):
            p, m = f"l{i}.", l["mixer"]
            mixer = PartSpec("latent_attention", {
                "prefix": p + "mix.", "hidden": h, "heads": m["heads"], "head_dim": m["dim"], "v_head_dim": m["vdim"], "latent": m["kv_rank"], "scale": m["scale"],
                "latent_norm": self._norm(p + "mix.dkv.norm", m["kv_rank"]), "gate": "sigmoid", "window": None,
                "names": {"q": "q", "down": "dkv", "up_k": "uk", "up_v": "uv", "gate": "g", "o": "o"}})
            ff = self._feed_forward(l["mlp"], p + "mlp.")
            layers.append(LayerSpec(prefix=p, block=PartSpec("scaled_prenorm", {"hidden": h, "residual_scale": self.residual_mult,
                                                                                 "channel_scales": (p + "ls1", p + "ls2")[:1 if ff is None else 2]}),
                                    parts=dict(mixer=mixer, feed_forward=ff, norms=tuple(self._norm(p + f"norm{s + 1}") for s in range(1 if ff is None else 2)))))
        joins = () if self.loop is None else (PartSpec("concat_projection", {"name": "loop.in", "width": h}),)
        embedding = PartSpec("token_embedding", {"name": "embed", "vocab": self.vocab, "width": h, "scale": self.embed_scale, "init": "unit"})
        if self.bigram is not None:
            embedding = PartSpec("pair_hash_embedding", {**embedding.params, "pairs": "bigram", "buckets": self.bigram[0], "mul_prev": self.bigram[1], "mul_cur": self.bigram[2]})
        return ModelSpec(
            hidden_size=h, vocab_size=self.vocab, max_positions=1 << 30, embedding=embedding,
            layers=tuple(layers), order=tuple(RunEntry(i, join=0 if starts else None) for i, starts in self.run_order()), joins=joins,
            final_norm=self._norm("final.norm"),
            head=PartSpec("lm_head", {"name": "head", "tied_to": "embed", "tied_only": True, "vocab": self.vocab, "width": h, "softcap": self.logit_softcap}))
