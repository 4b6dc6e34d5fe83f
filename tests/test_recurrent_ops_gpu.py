"""Each mechanism of the layers with state alone: the kernel against the plain function of the same equation, with
rows of several requests in one call, state carried from call to call, and sizes that no tile divides."""
import numpy as np
import pytest
import torch

from plain import tugalix as pt

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def rows_of(spans, n_slots):
    """spans: [(slot, rows)] in the order of the step's rows."""
    from alofa_amd import ops
    slots = torch.tensor([s for s, _ in spans], dtype=torch.int32, device=DEV)
    total = sum(n for _, n in spans)
    if all(n == 1 for _, n in spans):
        return ops.RowsOfRequests(slots, None, None, len(spans), total, n_slots)
    offsets = torch.tensor(np.concatenate([[0], np.cumsum([n for _, n in spans])]), dtype=torch.int32, device=DEV)
    req = torch.tensor([i for i, (_, n) in enumerate(spans) for _ in range(n)], dtype=torch.int32, device=DEV)
    return ops.RowsOfRequests(slots, offsets, req, len(spans), total, n_slots)


def dev(x, dtype=torch.float32):
    return torch.tensor(np.asarray(x), dtype=dtype, device=DEV).contiguous()


def cuts(n, sizes):
    out, at, k = [], 0, 0
    while at < n:
        m = min(sizes[k % len(sizes)], n - at)
        out.append((at, at + m))
        at, k = at + m, k + 1
    return out


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("width", [48, 1000])
def test_layer_norm(width, exact):
    from alofa_amd import ops
    rng = np.random.default_rng(0)
    x, w, b = rng.normal(2.0, 3.0, (9, width)), rng.normal(1, 0.2, width), rng.normal(0, 0.5, width)
    want = pt.layer_norm(x.astype(np.float32).astype(np.float64), w.astype(np.float32), b.astype(np.float32), 1e-5)
    out = torch.empty(9, width, device=DEV)
    ops.layernorm(out, dev(x), dev(w), dev(b), 1e-5, exact)
    assert np.abs(out.cpu().numpy() - want).max() <= (2e-6 if exact else 2e-5)
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    some = torch.empty(3, width, device=DEV)
    ops.layernorm(some, dev(x), dev(w), dev(b), 1e-5, exact, rows)
    assert torch.equal(some, out[[8, 0, 3]])
    inplace = dev(x)
    ops.layernorm(inplace, inplace, dev(w), dev(b), 1e-5, exact)
    assert torch.equal(inplace, out)


@pytest.mark.parametrize("taps", [1, 2, 3, 4, 9, 16])
def test_short_convolution_in_portions_of_two_requests(taps):
    """Two requests whose rows arrive in unequal portions within the same calls; the state carries the last rows."""
    from alofa_amd import ops
    rng = np.random.default_rng(taps)
    width, n_slots = 40, 5
    h = {5: rng.normal(0, 1, (23, width)), 2: rng.normal(0, 1, (17, width))}      # by slot
    w = rng.normal(0, 0.5, (width, taps))
    want = {s: x + pt.causal_filter(x, w) for s, x in h.items()}
    n_slots = 6
    state = torch.zeros(n_slots, taps - 1, width, device=DEV)
    state[1] = 7.0      # another request's slot: must stay as it is
    parts = {5: cuts(23, (1, 4, 2, 1, 1, 9)), 2: cuts(17, (3, 1, 1, 2, 8))}
    got = {5: [], 2: []}
    for step in range(max(len(p) for p in parts.values())):
        live = [(s, parts[s][step]) for s in (5, 2) if step < len(parts[s])]
        x = np.concatenate([h[s][a:b] for s, (a, b) in live])
        rows = rows_of([(s, b - a) for s, (a, b) in live], n_slots)
        out = torch.empty(x.shape[0], width, device=DEV)
        ops.short_conv(out, dev(x), dev(w), state, rows, exact=True)
        if taps > 1:
            ops.keep_last_rows(state, dev(x), rows)
        at = 0
        for s, (a, b) in live:
            got[s].append(out[at:at + b - a].cpu().numpy())
            at += b - a
    for s in (5, 2):
        assert np.abs(np.concatenate(got[s]) - want[s]).max() <= 1e-5
    if taps > 1:
        assert bool((state[1] == 7.0).all())


def test_mix_with_the_token_before():
    from alofa_amd import ops
    rng = np.random.default_rng(1)
    width = 24
    x, mu = rng.normal(0, 1, (11, width)).astype(np.float32), rng.uniform(0, 1, (5, width)).astype(np.float32)
    before = np.vstack([np.zeros((1, width)), x[:-1]])
    want = np.stack([x + (before - x) * m for m in mu])
    state = torch.zeros(3, 1, width, device=DEV)
    got = []
    for a, b in cuts(11, (1, 1, 4, 2, 1, 1, 1)):
        rows = rows_of([(2, b - a)], 3)
        out = torch.empty(5, b - a, width, device=DEV)
        if b - a == 1 and a % 2:      # a single row: the state may move on in the same launch
            ops.shift_mix(out, dev(x[a:b]), dev(mu), state, rows, keep=True)
        else:
            ops.shift_mix(out, dev(x[a:b]), dev(mu), state, rows)
            ops.keep_last_rows(state, dev(x[a:b]), rows)
        got.append(out.cpu().numpy())
    assert np.abs(np.concatenate(got, axis=1) - want).max() <= 1e-6


DECAYS = ["per_head", "sigmoid_root", "exp_neg_exp"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", DECAYS)
@pytest.mark.parametrize("heads,dk,dv", [(2, 16, 16), (1, 40, 72), (3, 24, 8), (2, 128, 128), (1, 130, 66), (1, 300, 20)])
def test_linear_recurrence(heads, dk, dv, kind, dtype):
    """Two requests side by side in unequal portions (single rows among them) against the plain recurrence of each."""
    from alofa_amd import ops
    rng = np.random.default_rng(dk + dv)
    n_slots, T = 4, {3: 141, 0: 29}      # (steps of more than 64 rows make their decays in a launch of their own)
    data = {}
    for s, n in T.items():
        q, k, v = rng.normal(0, 1, (n, heads * dk)), rng.normal(0, 1, (n, heads * dk)), rng.normal(0, 1, (n, heads * dv))
        if dtype is torch.bfloat16:
            q, k, v = (pt.to_bfloat16(a) for a in (q, k, v))
        data[s] = (q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), rng.normal(0.5, 1.5, (n, heads * dk)).astype(np.float32))
    per_head = rng.uniform(0.8, 1.0, heads).astype(np.float32)
    bonus = rng.normal(0, 1, (heads, dk)).astype(np.float32) if kind == "exp_neg_exp" else None
    tau, qs, ks = 7.0, 0.37, 1.9

    def weights(z):
        if kind == "per_head":
            return np.repeat(per_head.astype(np.float64), dk)[None, :].repeat(z.shape[0], 0)
        z = z.astype(np.float64)
        return (1 / (1 + np.exp(-z))) ** (1 / tau) if kind == "sigmoid_root" else np.exp(-np.exp(z - 2.0))
    want = {}
    for s, (q, k, v, z) in data.items():
        w = weights(z)
        want[s] = np.concatenate([pt.decayed_outer_sum(q[:, i * dk:(i + 1) * dk].astype(np.float64) * np.float32(qs), k[:, i * dk:(i + 1) * dk].astype(np.float64) * np.float32(ks),
                                                       v[:, i * dv:(i + 1) * dv].astype(np.float64), w[:, i * dk:(i + 1) * dk], None if bonus is None else bonus[i].astype(np.float64))
                                  for i in range(heads)], axis=1)
    state = torch.zeros(n_slots, heads, dk, dv, device=DEV)
    state[1] = 3.0
    parts = {3: cuts(141, (1, 17, 1, 2, 100, 5, 15)), 0: cuts(29, (6, 1, 1, 16, 2, 9))}
    got = {3: [], 0: []}
    code = {"per_head": ops.DECAY_PER_HEAD, "sigmoid_root": ops.DECAY_SIGMOID_ROOT, "exp_neg_exp": ops.DECAY_EXP_NEG_EXP}[kind]
    for step in range(max(len(p) for p in parts.values())):
        live = [(s, parts[s][step]) for s in (3, 0) if step < len(parts[s])]
        q, k, v, z = (np.concatenate([data[s][j][a:b] for s, (a, b) in live]) for j in range(4))
        rows = rows_of([(s, b - a) for s, (a, b) in live], n_slots)
        # (room for the read-outs in parts: the step of 100 rows deals the key channels out over blocks where the key size allows)
        room = torch.full((ops.recurrence_max_parts(dk), q.shape[0], heads * dv), float("nan"), device=DEV)
        decay = dev(per_head) if kind == "per_head" else dev(z - 2.0 if kind == "exp_neg_exp" else z)
        used = ops.linear_recurrence(room, dev(q, dtype), dev(k, dtype), dev(v, dtype), state, rows, heads, dk, dv, code, decay, tau=tau,
                                     bonus=None if bonus is None else dev(bonus), q_scale=qs, k_scale=ks, before_update=bonus is not None)
        assert 1 <= used <= room.shape[0] and (used > 1) == (q.shape[0] > 64 and dk >= 32)
        out = room[:used].sum(0)
        at = 0
        for s, (a, b) in live:
            got[s].append(out[at:at + b - a].cpu().numpy())
            at += b - a
    for s in (3, 0):
        g = np.concatenate(got[s])
        assert np.abs(g - want[s]).max() <= 2e-5 * max(1.0, np.abs(want[s]).max()), f"slot {s}"
    assert bool((state[1] == 3.0).all()) and bool((state[2] == 0.0).all())


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("heads,dv", [(3, 8), (2, 72), (1, 200)])
def test_head_norm_and_gate(heads, dv, weighted):
    from alofa_amd import ops
    rng = np.random.default_rng(heads)
    T = 7
    o, g = rng.normal(0, 2, (T, heads, dv)).astype(np.float32), rng.normal(0, 2, (T, heads * dv)).astype(np.float32)
    w = rng.normal(1, 0.3, heads * dv).astype(np.float32) if weighted else None
    want = pt.unit_rms(o.astype(np.float64), 1e-6).reshape(T, -1) * (1.0 if w is None else w) * pt.silu(g.astype(np.float64))
    wide = torch.zeros(T, heads * dv + 8, device=DEV)      # the gate as columns of a wider matrix
    wide[:, 8:] = dev(g)
    out = torch.empty(T, heads * dv, device=DEV)
    ops.headnorm_gate(out, dev(o.reshape(T, -1)), wide[:, 8:], None if w is None else dev(w), heads, dv, 1e-6, True)
    assert np.abs(out.cpu().numpy() - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
    # the same read-outs in three parts, with room for four
    shares = rng.normal(0, 1, (4, T, heads * dv)).astype(np.float32)
    shares[2] = o.reshape(T, -1) - shares[0] - shares[1]
    ops.headnorm_gate(out, dev(shares), wide[:, 8:], None if w is None else dev(w), heads, dv, 1e-6, True, parts=3)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-5 * max(1.0, np.abs(want).max())


def test_activations():
    from alofa_amd import ops
    z = np.linspace(-9, 9, 1001).astype(np.float32).reshape(7, 143)
    out = torch.empty(7, 143, device=DEV)
    ops.activation(out, dev(z), ops.XIELU, pt.softplus(0.3), 0.5 + pt.softplus(-1.2), exact=True)
    assert np.abs(out.cpu().numpy() - pt.xielu(z.astype(np.float64), 0.3, -1.2)).max() <= 1e-5
    ops.activation(out, dev(z), ops.TANH, exact=True)
    assert np.abs(out.cpu().numpy() - np.tanh(z.astype(np.float64))).max() <= 1e-6
    half = dev(z, torch.bfloat16)
    ops.activation(half, half, ops.XIELU, pt.softplus(0.3), 0.5 + pt.softplus(-1.2))
    want = pt.xielu(pt.to_bfloat16(z), 0.3, -1.2)
    assert np.abs(half.float().cpu().numpy() - want).max() <= 2 ** -8 * np.abs(want).max()


def test_average_over_depth_and_sum_of_branches():
    from alofa_amd import ops
    rng = np.random.default_rng(3)
    levels, shape = 4, (5, 12)
    outs = [rng.normal(0, 1, shape).astype(np.float32) for _ in range(levels)]
    weights = [rng.normal(0.4, 0.3, n + 1).astype(np.float32) for n in range(levels)]
    stack = torch.zeros(levels, *shape, device=DEV)
    x = dev(outs[0])
    ops.depth_average(x, stack, None, 1)
    assert torch.equal(x, dev(outs[0])) and torch.equal(stack[0], x)
    for n in range(1, levels):
        x = dev(outs[n])
        ops.depth_average(x, stack, dev(weights[n]), n + 1, exact=True)
        want = sum(weights[n][j].astype(np.float64) * outs[j] for j in range(n + 1))
        assert np.abs(x.cpu().numpy() - want).max() <= 1e-6
    r, a, b = (rng.normal(0, 1, shape).astype(np.float32) for _ in range(3))
    res = dev(r)
    ops.add_scaled(res, dev(a), 1.25, dev(b), -0.5, exact=True)
    assert np.abs(res.cpu().numpy() - (r + 1.25 * a.astype(np.float64) - 0.5 * b)).max() <= 1e-6
    ops.scale_(res, 3.0)
    assert np.abs(res.cpu().numpy() - 3.0 * (r + 1.25 * a.astype(np.float64) - 0.5 * b)).max() <= 3e-6


def test_part_of_a_head_rotated():
    """Rotary positions on the first channels of a head only: the position part's table and channel order against the
    plain rotation, through the products q . k, which are what the order of channels must not change."""
    from alofa_amd import ops
    from alofa_amd.config.base import PartSpec
    from alofa_amd.parts.base import Runtime, build_part
    rng = np.random.default_rng(5)
    T, heads, d, dims, base = 19, 3, 40, 12, 10000.0
    q, k = rng.normal(0, 1, (T, heads, d)).astype(np.float32), rng.normal(0, 1, (T, heads, d)).astype(np.float32)
    want = np.einsum("thd,shd->hts", pt.rotate(q.astype(np.float64), dims, base), pt.rotate(k.astype(np.float64), dims, base))
    part = build_part("position", PartSpec("rotary", {"theta": base, "head_dim": d, "dims": dims}), {}, Runtime(torch.device(DEV), torch.float32))
    order = part.channel_order()
    assert sorted(order) == list(range(d))
    both = dev(np.concatenate([q[:, :, order].reshape(T, -1), k[:, :, order].reshape(T, -1)], axis=1))
    cos, sin = part.table(T)
    ops.rope_kv_write(both, cos, sin, torch.arange(T, dtype=torch.int32, device=DEV), 2 * heads, 0, d)
    got = both.cpu().numpy().astype(np.float64).reshape(T, 2, heads, d)
    assert np.abs(np.einsum("thd,shd->hts", got[:, 0], got[:, 1]) - want).max() <= 1e-4


@pytest.mark.parametrize("taps", [2, 4, 16])
@pytest.mark.parametrize("exact", [True, False])
def test_norm_filter_and_state_in_one_launch(taps, exact):
    """Single rows of three requests: the fused kernel against norm, filter and state update one after the other."""
    from alofa_amd import ops
    rng = np.random.default_rng(taps)
    width, n_slots = 200, 5
    w, nw, nb = dev(rng.normal(0, 0.5, (width, taps))), dev(rng.normal(1, 0.2, width)), dev(rng.normal(0, 0.3, width))
    fused, apart = torch.zeros(n_slots, taps - 1, width, device=DEV), torch.zeros(n_slots, taps - 1, width, device=DEV)
    rows = rows_of([(4, 1), (0, 1), (2, 1)], n_slots)
    for _ in range(6):
        x = dev(rng.normal(1.0, 2.0, (3, width)))
        normed, want, got = torch.empty(3, width, device=DEV), torch.empty(3, width, device=DEV), torch.empty(3, width, device=DEV)
        ops.layernorm(normed, x, nw, nb, 1e-5, exact)
        ops.short_conv(want, normed, w, apart, rows, exact)
        ops.keep_last_rows(apart, normed, rows)
        ops.norm_conv_step(got, x, nw, nb, 1e-5, w, fused, rows, exact)
        assert torch.equal(got, want) and torch.equal(fused, apart)
