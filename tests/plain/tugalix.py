"""Plain Tugalix: whole sequences, no cache and no state carried between calls, float64 throughout, one function per
mechanism, written from the design's equations. It shares nothing with the engine.

Notation: T tokens, h the width; a sub-layer reads r = n + filter(n) with n the layer norm of the stream.
``store`` is applied wherever the engine keeps a bfloat16 tensor between kernels (the identity by default;
``to_bfloat16`` to measure what that rounding alone does)."""
from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np


def read_config(model_dir) -> dict:
    return json.loads((Path(model_dir) / "config.json").read_text())


def read_weights(model_dir) -> dict:
    """name -> float64 array, read with the safetensors library (the engine has a reader of its own)."""
    import torch
    from safetensors.torch import load_file
    return {name: t.to(torch.float64).numpy() for name, t in load_file(str(Path(model_dir) / "model.safetensors")).items()}


def to_bfloat16(x: np.ndarray) -> np.ndarray:
    """Round to nearest even at 8 bits of mantissa, through float32."""
    bits = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32).astype(np.float64)


def _keep(x):
    return x


# ------------------------------------------------------------------ mechanisms

def layer_norm(x, w, b, eps):
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def causal_filter(n, w):
    """f_t = sum_j w[:, j] * n_(t - taps + 1 + j), nothing before the first row."""
    taps = w.shape[1]
    f = np.zeros_like(n)
    for t in range(n.shape[0]):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                f[t] += w[:, j] * n[s]
    return f


def rotate(x, dims, base):
    """x [T, heads, d]: the pairs (i, i + dims/2), i < dims/2, turned by t * base^(-2i/dims); the rest unchanged."""
    out = x.copy()
    half = dims // 2
    for t in range(x.shape[0]):
        for i in range(half):
            a = t * base ** (-2.0 * i / dims)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * math.cos(a) - v * math.sin(a)
            out[t, :, i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def silu(z):
    return z / (1.0 + np.exp(-z))


def softplus(z):
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def xielu(z, p, q):
    pos = softplus(p) * z * z + z / 2
    neg = (0.5 + softplus(q)) * (np.expm1(np.minimum(z, 0.0)) - z) + z / 2
    return np.where(z > 0, pos, neg)


def decayed_outer_sum(q, k, v, w, bonus=None):
    """One head. q, k, w [T, dk], v [T, dv]. S_t = diag(w_t) S_(t-1) + k_t v_t^T from S = 0.
    Without bonus: o_t = S_t^T q_t. With bonus u [dk]: o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t, the update after it."""
    S = np.zeros((k.shape[1], v.shape[1]))
    o = np.zeros((q.shape[0], v.shape[1]))
    for t in range(q.shape[0]):
        kv = np.outer(k[t], v[t])
        if bonus is not None:
            o[t] = (S + bonus[:, None] * kv).T @ q[t]
            S = w[t][:, None] * S + kv
        else:
            S = w[t][:, None] * S + kv
            o[t] = S.T @ q[t]
    return o


def retention(r, W, pre, m, eps, store=_keep):
    T, H, dk, dv = r.shape[0], m["heads"], m["dim"], m["vdim"]
    q = store(r @ W[pre + "q"].T).reshape(T, H, dk)
    k = store(r @ W[pre + "k"].T).reshape(T, H, dk)
    v = store(r @ W[pre + "v"].T).reshape(T, H, dv)
    gate = store(r @ W[pre + "g"].T)
    q = store(rotate(q, m["rot"]["dims"], m["rot"]["base"]))
    k = store(rotate(k, m["rot"]["dims"], m["rot"]["base"])) * dk ** -0.5
    o = np.stack([decayed_outer_sum(q[:, i], k[:, i], v[:, i], np.full((T, dk), m["decay"][i])) for i in range(H)], axis=1)
    y = store(unit_rms(o, eps).reshape(T, H * dv) * silu(gate))
    return y @ W[pre + "o"].T


def gated_linear_attention(r, W, pre, m, eps, store=_keep):
    T, H, dk, dv = r.shape[0], m["heads"], m["dim"], m["vdim"]
    q = store(r @ W[pre + "q"].T).reshape(T, H, dk) * dk ** -0.5
    k = store(r @ W[pre + "k"].T).reshape(T, H, dk)
    v = store(r @ W[pre + "v"].T).reshape(T, H, dv)
    gate = store(r @ W[pre + "g"].T)
    z = store(r @ W[pre + "a1"].T) @ W[pre + "a2"].T + W[pre + "a2.b"]
    alpha = (1.0 / (1.0 + np.exp(-z))) ** (1.0 / m["tau"])
    alpha = alpha.reshape(T, H, dk)
    o = np.stack([decayed_outer_sum(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], axis=1)
    y = store((unit_rms(o, eps) * W[pre + "norm"]).reshape(T, H * dv) * silu(gate))
    return y @ W[pre + "o"].T


def softmax_attention(r, W, pre, m, store=_keep):
    T, H, G, dk, dv = r.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(rotate(store(r @ W[pre + "q"].T).reshape(T, H, dk), m["rot"]["dims"], m["rot"]["base"]))
    k = store(rotate(store(r @ W[pre + "k"].T).reshape(T, G, dk), m["rot"]["dims"], m["rot"]["base"]))
    v = store(r @ W[pre + "v"].T).reshape(T, G, dv)
    o = np.zeros((T, H, dv))
    for i in range(H):
        g = i // (H // G)
        for t in range(T):
            s = (k[:t + 1, g] @ q[t, i]) * m["scale"]
            e = np.exp(s - s.max())
            o[t, i] = (e / e.sum()) @ v[:t + 1, g]
    return store(o.reshape(T, H * dv)) @ W[pre + "o"].T


def time_mix(r, W, pre, m, eps, store=_keep):
    T, H, d = r.shape[0], m["heads"], m["dim"]
    before = np.vstack([np.zeros((1, r.shape[1])), r[:-1]])
    mix = {s: store(r + (before - r) * W[pre + "mu." + s]) for s in "rkvgw"}
    rr = store(mix["r"] @ W[pre + "r"].T).reshape(T, H, d)
    k = store(mix["k"] @ W[pre + "k"].T).reshape(T, H, d)
    v = store(mix["v"] @ W[pre + "v"].T).reshape(T, H, d)
    gate = store(mix["g"] @ W[pre + "g"].T)
    low = store(np.tanh(store(mix["w"] @ W[pre + "w1"].T)))
    w = np.exp(-np.exp(low @ W[pre + "w2"].T + W[pre + "w0"])).reshape(T, H, d)
    o = np.stack([decayed_outer_sum(rr[:, i], k[:, i], v[:, i], w[:, i], bonus=W[pre + "u"][i]) for i in range(H)], axis=1)
    y = store(unit_rms(o, eps).reshape(T, H * d) * W[pre + "norm"] * silu(gate))
    return y @ W[pre + "o"].T


def feed_forward(r, W, pre, store=_keep):
    p, q = W[pre + "act"]
    return store(xielu(store(r @ W[pre + "up"].T), p, q)) @ W[pre + "down"].T


# ------------------------------------------------------------------ the model

def mixer(kind, r, W, pre, m, eps, store=_keep):
    if kind == "retention":
        return retention(r, W, pre, m, eps, store)
    if kind == "gla":
        return gated_linear_attention(r, W, pre, m, eps, store)
    if kind == "parallel":
        return (m["left_scale"] * softmax_attention(r, W, pre + "left.", m["left"], store)
                + m["right_scale"] * time_mix(r, W, pre + "right.", m["right"], eps, store))
    raise ValueError(kind)


def forward_hidden(W, cfg, ids, store=_keep):
    """The stream after every layer (after its average over depth): a list of [T, h]."""
    eps, taps = cfg["norm"]["eps"], cfg["canon"]["taps"]
    x = layer_norm(W["embed"][np.asarray(ids, dtype=np.int64)], W["embed.norm"], W["embed.norm.b"], eps)
    outputs, streams = [x], []
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        n = layer_norm(x, W[pre + "norm1"], W[pre + "norm1.b"], eps)
        assert W[pre + "canon1"].shape[1] == taps
        x = x + mixer(layer["type"], store(n + causal_filter(n, W[pre + "canon1"])), W, pre + "mix.", layer["mixer"], eps, store)
        if layer.get("mlp") is not None:
            n = layer_norm(x, W[pre + "norm2"], W[pre + "norm2.b"], eps)
            x = x + feed_forward(store(n + causal_filter(n, W[pre + "canon2"])), W, pre + "mlp.", store)
        outputs.append(x)
        x = sum(W[pre + "dwa"][j] * outputs[j] for j in range(i + 2))
        streams.append(x)
    return streams


def forward_logits(W, cfg, ids, store=_keep):
    x = forward_hidden(W, cfg, ids, store)[-1]
    y = store(layer_norm(x, W["final.norm"], W["final.norm.b"], cfg["norm"]["eps"]))
    return y @ W["head"].T * cfg["logit_scale"]


def greedy(W, cfg, prompt, n_new):
    ids, out = list(prompt), []
    for _ in range(n_new):
        row = forward_logits(W, cfg, ids)[-1]
        out.append(int(np.argmax(row)))      # the first of equal maxima
        ids.append(out[-1])
    return out
