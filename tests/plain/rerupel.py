"""Plain Rerupel: whole sequences, no cache and no state carried between calls, float64 throughout, one function per
mechanism, written from the design's equations. It shares nothing with the engine.

Notation: T tokens, h the width, H heads of dk query/key and dv value channels, r the latent's size.
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
    """name -> float64 array (integer tables stay integers), read with the safetensors library (the engine has a
    reader of its own)."""
    import torch
    from safetensors.torch import load_file
    return {name: (t.numpy() if not t.is_floating_point() else t.to(torch.float64).numpy())
            for name, t in load_file(str(Path(model_dir) / "model.safetensors")).items()}


def to_bfloat16(x: np.ndarray) -> np.ndarray:
    """Round to nearest even at 8 bits of mantissa, through float32."""
    bits = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32).astype(np.float64)


def _keep(x):
    return x


# ------------------------------------------------------------------ mechanisms

def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def bigram_rows(ids, buckets, mul_prev, mul_cur):
    """The row of the pair table for every token: a hash of (token before, token); the last row for the first token."""
    rows = []
    for t, tok in enumerate(ids):
        rows.append(buckets if t == 0 else (int(ids[t - 1]) * mul_prev + int(tok) * mul_cur) % buckets)
    return rows


def embed(ids, table, scale, pair_table, buckets, mul_prev, mul_cur):
    x = table[np.asarray(ids)] * scale
    return x + pair_table[np.asarray(bigram_rows(ids, buckets, mul_prev, mul_cur))]


def join_streams(x, x0, w):
    """What a pass starts from: w [h, 2h] on the stream beside the embedding's output, the stream first."""
    return np.concatenate([x, x0], axis=-1) @ w.T


def latent_attention(hn, wq, wdkv, latent_w, wuk, wuv, wg, wo, heads, dk, dv, scale, eps, store=_keep):
    """Softmax attention whose keys and values are projections of one small vector per token (the only thing a cache would
    have to hold), no positions, every earlier token visible, the heads' outputs gated by sigmoid(wg hn)."""
    T = hn.shape[0]
    q = store(hn @ wq.T).reshape(T, heads, dk)
    c = store(rms_norm(hn @ wdkv.T, latent_w, eps))
    k = store(c @ wuk.T).reshape(T, heads, dk)
    v = store(c @ wuv.T).reshape(T, heads, dv)
    gate = sigmoid(store(hn @ wg.T))
    out = np.zeros((T, heads, dv))
    for a in range(heads):
        s = (q[:, a] @ k[:, a].T) * scale
        for t in range(T):
            row = s[t, :t + 1]
            p = np.exp(row - row.max())
            out[t, a] = (p / p.sum()) @ v[:t + 1, a]
    return store(store(out.reshape(T, heads * dv)) * gate) @ wo.T


def squared_relu_ff(hn, w_up, w_down, store=_keep):
    z = np.maximum(store(hn @ w_up.T), 0.0)
    return store(z * z) @ w_down.T


def clamped_expert(hn, w_gate, w_up, w_down, limit, store=_keep):
    """g = min(gate, limit), u = clamp(up, -limit, limit); down((g sigmoid(1.702 g)) (u + 1))."""
    g = np.minimum(store(hn @ w_gate.T), limit)
    u = np.clip(store(hn @ w_up.T), -limit, limit)
    return store(g * sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def route(hn, w_router, top, scale):
    """Per token the ``top`` experts of the largest sigmoid scores (the lower index wins a tie) and their weights:
    the scores themselves times ``scale``, not made to sum to one."""
    s = sigmoid(hn @ w_router.T)
    chosen = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return chosen, np.take_along_axis(s, chosen, axis=-1) * scale


def routed_experts(hn, w_router, experts, shared, top, scale, limit, shared_limit, store=_keep):
    """experts: a list of (gate, up, down); shared: one such triple, or None."""
    chosen, weights = route(hn, w_router, top, scale)
    out = np.zeros((hn.shape[0], experts[0][2].shape[0]))
    for t in range(hn.shape[0]):
        for e, wt in zip(chosen[t], weights[t]):
            out[t] += wt * clamped_expert(hn[t:t + 1], *experts[e], limit, store)[0]
    if shared is not None:
        out += clamped_expert(hn, *shared, shared_limit, store)
    return out


def soft_cap(z, cap):
    return cap * np.tanh(z / cap)


# ------------------------------------------------------------------ the model

def run_order(cfg) -> list:
    """Layer indices in the order they run, and the runs a pass starts with."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n)), set()
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order, starts = list(range(a)), set()
    for _ in range(times):
        starts.add(len(order))
        order += list(range(a, b))
    return order + list(range(b, n)), starts


def layer(x, w, cfg, i, store=_keep):
    l, p, eps, m = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"], cfg["residual_mult"]
    mx = l["mixer"]
    y = latent_attention(store(rms_norm(x, w[p + "norm1"], eps)), w[p + "mix.q"], w[p + "mix.dkv"], w[p + "mix.dkv.norm"], w[p + "mix.uk"],
                         w[p + "mix.uv"], w[p + "mix.g"], w[p + "mix.o"], mx["heads"], mx["dim"], mx["vdim"], mx["scale"], eps, store)
    x = x + m * (y * w[p + "ls1"])
    mlp = l["mlp"]
    if mlp is None:
        return x
    hn = store(rms_norm(x, w[p + "norm2"], eps))
    if mlp["kind"] == "dense":
        y = squared_relu_ff(hn, w[p + "mlp.up"], w[p + "mlp.down"], store)
    else:
        def triple(q):
            return w[q + ".gate"], w[q + ".up"], w[q + ".down"]
        r = mlp["router"]
        sh = mlp.get("shared")
        y = routed_experts(hn, w[p + "mlp.router"], [triple(p + f"mlp.e{e}") for e in range(r["experts"])],
                           triple(p + "mlp.shared") if sh else None, r["top"], r["scale"], mlp["expert"]["limit"], sh["limit"] if sh else None, store)
    return x + m * (y * w[p + "ls2"])


def forward_hidden(w, cfg, ids, store=_keep) -> list:
    """The stream after every layer run, [T, h] each."""
    e = cfg["embedding"]
    b = e.get("bigram")
    if b is None:      # (a model without the pair table)
        x0 = w["embed"][np.asarray(ids)] * e["scale"]
    else:
        x0 = embed(ids, w["embed"], e["scale"], w["bigram"], b["buckets"], b["mul_prev"], b["mul_cur"])
    x, out = x0, []
    order, starts = run_order(cfg)
    for n, i in enumerate(order):
        if n in starts:
            x = join_streams(store(x), store(x0), w["loop.in"])
        x = layer(x, w, cfg, i, store)
        out.append(x)
    return out


def forward_logits(w, cfg, ids, store=_keep) -> np.ndarray:
    x = forward_hidden(w, cfg, ids, store)[-1]
    z = store(rms_norm(x, w["final.norm"], cfg["norm"]["eps"])) @ w["embed"].T
    return soft_cap(z, cfg["logit_softcap"])


def greedy(w, cfg, prompt, n_new) -> list:
    """n_new tokens, each the first index of the highest logit after everything before it."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        out.append(int(np.argmax(forward_logits(w, cfg, ids)[-1])))
        ids.append(out[-1])
    return out


def router_margins(w, cfg, ids) -> np.ndarray:
    """Per position the smallest gap, over all runs of layers with a router, between the last router product that is taken
    and the first that is not, in units of the products' spread at that position (infinite where nothing is left out).
    Positions with a small gap are the ones where rounding may change which experts a token takes."""
    T = len(ids)
    out = np.full(T, np.inf)
    e = cfg["embedding"]
    b = e.get("bigram")
    x0 = w["embed"][np.asarray(ids)] * e["scale"] if b is None else embed(ids, w["embed"], e["scale"], w["bigram"], b["buckets"], b["mul_prev"], b["mul_cur"])
    x = x0
    order, starts = run_order(cfg)
    for n, i in enumerate(order):
        if n in starts:
            x = join_streams(x, x0, w["loop.in"])
        l, p = cfg["layers"][i], f"l{i}."
        if l["mlp"] is not None and l["mlp"]["kind"] == "moe" and l["mlp"]["router"]["top"] < l["mlp"]["router"]["experts"]:
            mx = l["mixer"]
            y = latent_attention(rms_norm(x, w[p + "norm1"], cfg["norm"]["eps"]), w[p + "mix.q"], w[p + "mix.dkv"], w[p + "mix.dkv.norm"], w[p + "mix.uk"],
                                 w[p + "mix.uv"], w[p + "mix.g"], w[p + "mix.o"], mx["heads"], mx["dim"], mx["vdim"], mx["scale"], cfg["norm"]["eps"])
            mid = x + cfg["residual_mult"] * (y * w[p + "ls1"])
            z = np.sort(rms_norm(mid, w[p + "norm2"], cfg["norm"]["eps"]) @ w[p + "mlp.router"].T, axis=-1)[:, ::-1]
            top = l["mlp"]["router"]["top"]
            out = np.minimum(out, (z[:, top - 1] - z[:, top]) / (z.std(axis=-1) + 1e-30))
        x = layer(x, w, cfg, i)
    return out
