"""Small Tugalix configurations for the tests, different in every size and option, and their plain logits."""
import functools

import numpy as np

from helpers import Reference
from plain import tugalix as pt


def _retention(heads, dim, vdim, dims, base, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"dims": dims, "base": base}, "decay": decay}


def _parallel(heads, kv_heads, dim, vdim, dims, base, scale, r_heads, r_dim, rank, ls, rs):
    return {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"dims": dims, "base": base}},
            "right": {"heads": r_heads, "dim": r_dim, "rank": rank}, "left_scale": ls, "right_scale": rs}


def _config(vocab, width, eps, taps, logit_scale, layers):
    return {"architecture": "Tugalix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "logit_scale": logit_scale, "layers": [{"type": t, "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}} for t, m, ff in layers]}


TUGALIX = {
    # every mixer once; value heads wider than key heads, part of a head rotated, groups of two query heads
    "A": _config(200, 64, 1e-6, 3, 1.5, [
        ("retention", _retention(2, 16, 24, 8, 10000.0, [0.9, 0.99]), 96),
        ("parallel", _parallel(4, 2, 16, 16, 16, 500000.0, 0.25, 2, 32, 8, 0.7, 1.3), None),
        ("gla", {"heads": 2, "dim": 24, "vdim": 16, "tau": 8.0, "rank": 4}, 80)]),
    # sizes no kernel tiles evenly: one head, ranks 5 and 3, four taps, a head of 40 with 12 channels rotated, values wider than keys
    "B": _config(131, 72, 1e-5, 4, 0.5, [
        ("gla", {"heads": 1, "dim": 40, "vdim": 72, "tau": 4.0, "rank": 5}, None),
        ("parallel", _parallel(3, 3, 24, 40, 12, 10000.0, 0.3, 3, 24, 3, 1.0, -0.5), 100),
        ("retention", _retention(3, 24, 8, 24, 1000000.0, [0.5, 0.97, 0.999]), None)]),
    # no layer keeps pages; two taps
    "C": _config(96, 48, 1e-6, 2, 1.0, [
        ("retention", _retention(3, 16, 16, 16, 10000.0, [0.8, 0.95, 0.99]), 64),
        ("gla", {"heads": 2, "dim": 8, "vdim": 24, "tau": 16.0, "rank": 8}, None)]),
    # wider: value heads of 128 (two slices of lanes), keys of 64 and 128, two attention layers, one tap
    "D": _config(500, 256, 1e-6, 1, 2.0, [
        ("parallel", _parallel(4, 1, 64, 32, 32, 10000.0, 0.125, 2, 128, 16, 1.1, 0.9), 512),
        ("retention", _retention(2, 64, 128, 64, 10000.0, [0.96, 0.995]), None),
        ("parallel", _parallel(2, 2, 128, 128, 128, 1000000.0, 0.09, 4, 64, 16, 0.5, 0.5), None),
        ("gla", {"heads": 2, "dim": 128, "vdim": 128, "tau": 16.0, "rank": 16}, 256)]),
    # nothing a multiple of eight: width 100, odd head sizes (15 with 6 channels rotated, 9, 7), ranks 7 and 1, five taps, two kv heads of five
    "E": _config(301, 100, 1e-4, 5, 0.75, [
        ("retention", _retention(5, 15, 9, 6, 20000.0, [0.7, 0.9, 0.95, 0.99, 1.0]), 150),
        ("parallel", _parallel(10, 2, 20, 12, 10, 300.0, 0.4, 5, 7, 1, 0.3, 2.0), None),
        ("parallel", _parallel(1, 1, 30, 50, 30, 10000.0, 0.2, 1, 33, 7, 1.0, 1.0), 66),
        ("gla", {"heads": 3, "dim": 9, "vdim": 15, "tau": 2.5, "rank": 7}, None),
        ("gla", {"heads": 1, "dim": 21, "vdim": 100, "tau": 30.0, "rank": 2}, 30)]),
}


@functools.lru_cache(maxsize=None)
def plain_model(model_dir):
    return pt.read_config(model_dir), pt.read_weights(model_dir)


@functools.lru_cache(maxsize=64)
def _logits(model_dir, ids, rounded):
    cfg, w = plain_model(model_dir)
    return pt.forward_logits(w, cfg, list(ids), store=pt.to_bfloat16 if rounded else (lambda x: x)).astype(np.float32)


def plain_logits(model_dir, ids):
    ref = _logits(str(model_dir), tuple(ids), False).view(Reference)
    ref._rounded = lambda: _logits(str(model_dir), tuple(ids), True)
    return ref
