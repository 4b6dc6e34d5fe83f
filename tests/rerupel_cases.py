"""Small Rerupel configurations for the tests, different in every size and option, and their plain logits."""
import functools

import numpy as np

from helpers import Reference
from plain import rerupel as pr


def _latent(heads, dim, vdim, rank, scale):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}


def _moe(experts, top, scale, ff, limit, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff, "limit": limit},
            "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _config(vocab, width, eps, mult, cap, scale, bigram, loop, layers):
    out = {"architecture": "Rerupel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult, "logit_softcap": cap,
           "embedding": {"scale": scale}, "layers": [{"type": "latent_attention", "mixer": m, "mlp": mlp} for m, mlp in layers]}
    if bigram is not None:
        out["embedding"]["bigram"] = dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


RERUPEL = {
    # every feed-forward once; values wider than keys and narrower; the last two layers run twice
    "A": _config(200, 64, 1e-6, 0.7, 20.0, 3.0, (101, 13, 5), (1, 3, 2), [
        (_latent(2, 16, 24, 32, 0.25), _dense(96)),
        (_latent(4, 16, 16, 16, 0.2), _moe(4, 2, 1.5, 32, 1.0, (48, 2.0))),
        (_latent(3, 32, 8, 48, 0.15), None)]),
    # sizes no kernel tiles evenly; one head; a latent of 24 channels (widened to 32); every expert taken (top = experts), no shared
    # expert; the first layer alone runs three times; factors of one
    "B": _config(131, 72, 1e-5, 1.0, 50.0, 1.0, (37, 1, 1), (0, 1, 3), [
        (_latent(1, 40, 72, 24, 0.16), _moe(3, 3, 1.0, 20, 0.5)),
        (_latent(3, 24, 40, 72, 0.2), _dense(100))]),
    # no pair table and no loop; one expert per token
    "C": _config(96, 48, 1e-6, 0.5, 8.0, 6.0, None, None, [
        (_latent(3, 16, 16, 16, 0.25), _moe(5, 1, 2.5, 24, 3.0, (16, 0.75))),
        (_latent(2, 8, 24, 40, 0.35), _dense(64))]),
    # wider: twenty heads (more than a block of the decode kernel takes), latents of 128 and 100 channels, sixteen experts; all layers loop
    "D": _config(500, 256, 1e-6, 0.4, 30.0, 10.0, (997, 29, 3), (0, 3, 2), [
        (_latent(8, 32, 64, 128, 0.18), _moe(16, 4, 1.2, 64, 1.5, (128, 1.5))),
        (_latent(20, 16, 16, 64, 0.25), _dense(512)),
        (_latent(4, 64, 32, 100, 0.125), None)]),
    # nothing a multiple of eight: width 100, heads of 15 and 9 channels, latents of 10 and 18 channels, experts of 14 channels; the
    # loop is the last layer, once
    "E": _config(301, 100, 1e-4, 1.3, 12.0, 0.5, (64, 7, 300), (2, 3, 1), [
        (_latent(5, 15, 9, 10, 0.3), _dense(30)),
        (_latent(1, 30, 50, 18, 0.2), _moe(5, 2, 0.8, 14, 1.25, (6, 4.0))),
        (_latent(10, 6, 10, 34, 0.4), _moe(2, 1, 3.0, 22, 0.9))]),
    # latents wider than any head the attention kernels take (the pages then hold every head's keys and values), values wider
    # and narrower than keys
    "F": _config(150, 64, 1e-6, 0.6, 25.0, 4.0, (89, 3, 11), (0, 2, 2), [
        (_latent(2, 16, 24, 264, 0.25), _dense(48)),
        (_latent(3, 32, 16, 320, 0.18), _moe(4, 2, 1.0, 16, 2.0, (16, 2.0)))]),
    # five heads of 48 and 80 channels over a latent of 96; three layers passed through three times between two others; twelve experts of
    # which a token takes three (slot by slot) or five (every expert against every row)
    "G": _config(777, 320, 1e-5, 0.35, 15.0, 8.0, (1021, 17, 3), (1, 4, 3), [
        (_latent(5, 48, 80, 96, 0.14), _dense(384)),
        (_latent(5, 48, 80, 96, 0.14), _moe(12, 3, 1.7, 72, 1.2, (40, 1.2))),
        (_latent(10, 32, 32, 160, 0.18), _moe(12, 5, 0.6, 72, 2.5, (72, 2.5))),
        (_latent(5, 64, 64, 64, 0.125), _moe(12, 3, 1.7, 64, 1.2, (40, 1.2))),
        (_latent(2, 128, 128, 192, 0.09), _dense(200))]),
}


@functools.lru_cache(maxsize=None)
def plain_model(model_dir):
    return pr.read_config(model_dir), pr.read_weights(model_dir)


@functools.lru_cache(maxsize=64)
def _logits(model_dir, ids, rounded):
    cfg, w = plain_model(model_dir)
    return pr.forward_logits(w, cfg, list(ids), store=pr.to_bfloat16 if rounded else (lambda x: x)).astype(np.float32)


def plain_logits(model_dir, ids):
    ref = _logits(str(model_dir), tuple(ids), False).view(Reference)
    ref._rounded = lambda: _logits(str(model_dir), tuple(ids), True)
    return ref


@functools.lru_cache(maxsize=64)
def _margins(model_dir, ids):
    cfg, w = plain_model(model_dir)
    return pr.router_margins(w, cfg, list(ids))


def clear_calls(model_dir, ids, dtype, threshold=0.04):
    """The positions to compare: all of them in float32; in bfloat16 those at which no router's call is so close that rounding
    the activations may change which experts the token takes (such a change is no fault, and moves logits by far more than
    the bound measured from rounding allows)."""
    if dtype == "float32":
        return np.arange(len(ids))
    return np.flatnonzero(_margins(str(model_dir), tuple(ids)) >= threshold)
