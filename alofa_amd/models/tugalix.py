"""Tugalix: a decoder whose layers are listed one by one in config.json, each with one of three mixers and an
optional feed-forward.

config.json: ``architecture`` "Tugalix"; ``vocab``, ``width``; ``norm.eps``; ``canon.taps``; ``logit_scale``;
``layers``: a list of {``type``, ``mixer``, ``mlp``}. Tensor names: ``embed``, ``embed.norm`` (+ ``.b``), ``l<i>.`` +
``norm1``/``norm2`` (+ ``.b``), ``canon1``/``canon2``, ``mix.*``, ``mlp.*``, ``dwa``; ``final.norm`` (+ ``.b``), ``head``.

The model: the embedding's rows pass a layer norm. A layer is pre-norm (layer norm with bias), and what each
sub-layer reads passes a short causal convolution over time first (h + conv(h), ``canon.taps`` taps per channel). A
layer whose ``mlp`` is null has the mixer's sub-layer only. What a layer hands on is a weighted sum over the outputs
of all layers so far (the embedding's first), with the layer's own weights ``dwa``. The logits are the head's
product of the final layer norm, times ``logit_scale``.

Mixers by ``type``:
  retention  heads x (dim, vdim), one ``decay`` per head, rotary positions on ``rot.dims`` channels with ``rot.base``.
  gla        heads x (dim, vdim), decays sigmoid(z)^(1/``tau``) per key channel from a two-step projection.
  parallel   ``left`` (softmax attention with ``heads`` query and ``kv_heads`` key/value heads of sizes ``dim`` and ``vdim``,
             rotary positions, scores times ``scale``) beside ``right`` (RWKV-style time mixing, heads x dim), summed with
             ``left_scale`` and ``right_scale``.
The feed-forward (``mlp.kind`` "dense", ``mlp.ff`` wide) is two matrices with xIELU between them.

The ranks of the two-step decay projections are no keys of config.json: they are the first dimension of the
tensors ``a1`` and ``w1`` (``sized_by``). A configuration written by this engine names them as ``rank``."""
from __future__ import annotations

import copy
from dataclasses import dataclass

from ..config.base import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry
from ..errors import AlofaError

MIXERS = ("retention", "gla", "parallel")


def _get(raw: dict, key: str, kind, where: str):
    if not isinstance(raw, dict) or key not in raw:
        raise AlofaError("invalid_argument", "config.json lacks a required key", f"key={key} config={where}")
    v = raw[key]
    if kind in (int, float):
        if isinstance(v, bool) or not isinstance(v, (int, float)) or (kind is int and int(v) != v):
            raise AlofaError("parse", "config value must be a number" if kind is float else "config value must be a whole number", f"key={key} config={where}")
        return kind(v)
    if not isinstance(v, kind):
        raise AlofaError("parse", "config value has the wrong kind", f"key={key} config={where}")
    return v


def _positive(where: str, **values) -> None:
    for k, v in values.items():
        if not v > 0:
            raise AlofaError("parse", "config value must be positive", f"key={k} value={v} config={where}")


def _rot(raw: dict, dim: int, where: str) -> dict:
    rot = _get(raw, "rot", dict, where)
    out = {"base": _get(rot, "base", float, where), "dims": _get(rot, "dims", int, where)}
    _positive(where, base=out["base"], dims=out["dims"])
    if out["dims"] % 2 or out["dims"] > dim:
        raise AlofaError("parse", "rot.dims is even and at most the head's size", f"dims={out['dims']} dim={dim} config={where}")
    return out


def _recurrent_sizes(m: dict, where: str, vdim: bool = True) -> dict:
    out = {"heads": _get(m, "heads", int, where), "dim": _get(m, "dim", int, where)}
    if vdim:
        out["vdim"] = _get(m, "vdim", int, where)
    _positive(where, **out)
    if "rank" in m:
        out["rank"] = _get(m, "rank", int, where)
        _positive(where, rank=out["rank"])
    return out


def _mixer(kind: str, m: dict, where: str) -> dict:
    """The mixer's keys, checked and in a fixed form."""
    if kind == "retention":
        out = _recurrent_sizes(m, where)
        out.pop("rank", None)
        out["decay"] = [float(x) for x in _get(m, "decay", list, where)]
        if len(out["decay"]) != out["heads"]:
            raise AlofaError("parse", "one decay per head", f"heads={out['heads']} decay={len(out['decay'])} config={where}")
        out["rot"] = _rot(m, out["dim"], where)
        return out
    if kind == "gla":
        out = _recurrent_sizes(m, where)
        out["tau"] = _get(m, "tau", float, where)
        _positive(where, tau=out["tau"])
        return out
    left, right = _get(m, "left", dict, where), _get(m, "right", dict, where)
    lo = {"heads": _get(left, "heads", int, where), "kv_heads": _get(left, "kv_heads", int, where), "dim": _get(left, "dim", int, where),
          "vdim": _get(left, "vdim", int, where), "scale": _get(left, "scale", float, where)}
    _positive(where, **{k: v for k, v in lo.items() if k != "scale"})
    if lo["heads"] % lo["kv_heads"]:
        raise AlofaError("parse", "kv_heads must divide heads", f"heads={lo['heads']} kv_heads={lo['kv_heads']} config={where}")
    lo["rot"] = _rot(left, lo["dim"], where)
    return {"left": lo, "right": _recurrent_sizes(right, where, vdim=False),
            "left_scale": _get(m, "left_scale", float, where), "right_scale": _get(m, "right_scale", float, where)}


@dataclass(frozen=True)
class TugalixConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    taps: int
    logit_scale: float
    layers: tuple      # per layer a dict {type, mixer, mlp}, checked

    architecture = "Tugalix"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "<dict>") -> "TugalixConfig":
        layers = []
        for i, l in enumerate(_get(raw, "layers", list, where)):
            at = f"{where} layers[{i}]"
            kind = _get(l, "type", str, at)
            if kind not in MIXERS:
                raise AlofaError("unsupported", "no such mixer in this design", f"type={kind} known={','.join(MIXERS)} config={at}")
            mlp = l.get("mlp") if isinstance(l, dict) else None
            if mlp is not None:
                if _get(mlp, "kind", str, at) != "dense":
                    raise AlofaError("unsupported", "no such feed-forward in this design", f"kind={mlp['kind']} config={at}")
                mlp = {"kind": "dense", "ff": _get(mlp, "ff", int, at)}
                _positive(at, ff=mlp["ff"])
            layers.append({"type": kind, "mixer": _mixer(kind, _get(l, "mixer", dict, at), at), "mlp": mlp})
        cfg = cls(vocab=_get(raw, "vocab", int, where), width=_get(raw, "width", int, where),
                  eps=_get(_get(raw, "norm", dict, where), "eps", float, where), taps=_get(_get(raw, "canon", dict, where), "taps", int, where),
                  logit_scale=_get(raw, "logit_scale", float, where), layers=tuple(layers))
        _positive(where, vocab=cfg.vocab, width=cfg.width, eps=cfg.eps, taps=cfg.taps)
        if not layers:
            raise AlofaError("parse", "a model has at least one layer", f"config={where}")
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps}, "canon": {"taps": self.taps},
                "logit_scale": self.logit_scale, "layers": copy.deepcopy(list(self.layers))}

    # ---- sizes that only the tensors give
    @staticmethod
    def _rank_tensors(i: int, layer: dict) -> list:
        """(the dict that lacks its rank, the tensor whose first dimension is that rank)"""
        if layer["type"] == "gla":
            return [(layer["mixer"], f"l{i}.mix.a1")]
        if layer["type"] == "parallel":
            return [(layer["mixer"]["right"], f"l{i}.mix.right.w1")]
        return []

    def wants_shapes(self) -> bool:
        return any("rank" not in m for i, l in enumerate(self.layers) for m, _ in self._rank_tensors(i, l))

    def sized_by(self, shapes: dict) -> "TugalixConfig":
        layers = copy.deepcopy(list(self.layers))
        for i, l in enumerate(layers):
            for m, name in self._rank_tensors(i, l):
                if "rank" not in m:
                    if name not in shapes or len(shapes[name]) != 2:
                        raise AlofaError("invalid_argument", "the tensor that gives a projection's rank is missing", f"tensor={name}")
                    m["rank"] = int(shapes[name][0])
        return TugalixConfig(self.vocab, self.width, self.eps, self.taps, self.logit_scale, tuple(layers))

    # ---- the model as data
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("layernorm", {"name": name, "bias": name + ".b", "width": self.width, "eps": self.eps})

    def _rotary(self, rot: dict, dim: int) -> PartSpec:
        return PartSpec("rotary", {"theta": rot["base"], "head_dim": dim, "dims": rot["dims"], "pairing": "half"})

    def _mixer_spec(self, kind: str, m: dict, pre: str) -> PartSpec:
        h = self.width
        if kind == "retention":
            return PartSpec("retention", {"prefix": pre, "hidden": h, "heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                                          "decay": tuple(m["decay"]), "position": self._rotary(m["rot"], m["dim"]), "eps": self.eps})
        if kind == "gla":
            return PartSpec("gated_linear", {"prefix": pre, "hidden": h, "heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                                             "tau": m["tau"], "rank": m["rank"], "eps": self.eps})
        left, right = m["left"], m["right"]
        attention = PartSpec("gqa_attention", {
            "prefix": pre + "left.", "hidden": h, "heads": left["heads"], "kv_heads": left["kv_heads"], "head_dim": left["dim"],
            "v_head_dim": left["vdim"], "scale": left["scale"], "qkv_bias": False, "out_bias": False, "window": None,
            "position": self._rotary(left["rot"], left["dim"]), "names": {"q": "q", "k": "k", "v": "v", "o": "o"}, "init": "fan_in"})
        time_mix = PartSpec("time_mix", {"prefix": pre + "right.", "hidden": h, "heads": right["heads"], "key_dim": right["dim"],
                                         "rank": right["rank"], "eps": self.eps})
        return PartSpec("parallel", {"branches": (attention, time_mix), "scales": (m["left_scale"], m["right_scale"]), "hidden": h})

    def spec(self) -> ModelSpec:
        if self.wants_shapes():
            raise AlofaError("invalid_argument", "the ranks of the decay projections are not known yet: they come from the tensors' shapes (sized_by) or the key rank")
        h, n = self.width, len(self.layers)
        layers = []
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            subs = 1 if l["mlp"] is None else 2
            ff = None if l["mlp"] is None else PartSpec("dense_activated", {
                "prefix": p + "mlp.", "hidden": h, "intermediate": l["mlp"]["ff"], "activation": "xielu", "names": {"up": "up", "down": "down", "act": "act"}})
            layers.append(LayerSpec(prefix=p, block=PartSpec("filtered_prenorm", {"depth_average": p + "dwa", "level": i + 1, "levels": n + 1, "hidden": h}), parts=dict(
                mixer=self._mixer_spec(l["type"], l["mixer"], p + "mix."), feed_forward=ff,
                norms=tuple(self._norm(p + f"norm{s + 1}") for s in range(subs)),
                convs=tuple(PartSpec("short_causal", {"name": p + f"canon{s + 1}", "width": h, "taps": self.taps}) for s in range(subs)))))
        return ModelSpec(
            hidden_size=h, vocab_size=self.vocab, max_positions=1 << 30,
            embedding=PartSpec("token_embedding", {"name": "embed", "vocab": self.vocab, "width": h, "norm": self._norm("embed.norm"), "init": "unit"}),
            layers=tuple(layers), order=tuple(RunEntry(i) for i in range(n)),
            final_norm=self._norm("final.norm"),
            head=PartSpec("lm_head", {"name": "head", "tied_to": None, "vocab": self.vocab, "width": h, "scale": self.logit_scale, "init": "fan_in"}))
