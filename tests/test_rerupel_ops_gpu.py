"""Each mechanism of Rerupel's layers alone: the kernel against the plain function of the same equation, with rows of several
requests in one call, state carried from call to call, and sizes that no tile divides."""
import numpy as np
import pytest
import torch

from plain import rerupel as pr
from test_recurrent_ops_gpu import cuts, dev, rows_of

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def b16(x):
    return pr.to_bfloat16(np.asarray(x, dtype=np.float64))


@pytest.mark.parametrize("table_dtype", [torch.float32, torch.bfloat16])
def test_pair_embedding_in_portions_of_two_requests(table_dtype):
    """Two requests whose tokens arrive in unequal portions within the same calls; the token before a portion's first row is
    state; one step brings its token through the token store."""
    from alofa_amd import ops
    rng = np.random.default_rng(0)
    vocab, width, buckets, mp, mc, scale = 50, 72, 23, 31, 7, 2.5
    table, pairs = b16(rng.normal(0, 1, (vocab, width))), b16(rng.normal(0, 1, (buckets + 1, width)))
    ids = {4: [int(t) for t in rng.integers(0, vocab, 19)], 1: [int(t) for t in rng.integers(0, vocab, 11)]}
    want = {s: pr.embed(seq, table, scale, pairs, buckets, mp, mc) for s, seq in ids.items()}
    state = torch.full((6, 1), 7, dtype=torch.int32, device=DEV)
    store = torch.zeros(6, dtype=torch.int32, device=DEV)
    parts = {4: cuts(19, (1, 4, 2, 1, 1, 9)), 1: cuts(11, (3, 1, 1, 2, 8))}
    for k in range(max(len(p) for p in parts.values())):
        spans, toks, pos = [], [], []
        for s in (4, 1):
            if k < len(parts[s]):
                a, b = parts[s][k]
                spans.append((s, b - a))
                seq = list(ids[s][a:b])
                if b - a == 1 and k % 2:      # the one token comes from the device's store
                    store[s] = seq[0]
                    seq = [-(s + 1)]
                toks += seq
                pos += list(range(a, b))
        out = torch.empty(len(toks), width, device=DEV)
        ops.pair_embed(out, dev(table, table_dtype), dev(toks, torch.int32), scale, store, dev(pairs, table_dtype), dev(pos, torch.int32), state,
                       rows_of(spans, 6), buckets, mp, mc)
        row = 0
        for s, n in spans:
            a = parts[s][k][0]
            assert np.abs(out[row:row + n].cpu().numpy() - want[s][a:a + n]).max() <= 1e-5, (k, s)
            row += n
    assert state[4, 0].item() == ids[4][-1] and state[1, 0].item() == ids[1][-1] and state[0, 0].item() == 7
    plain_rows = torch.empty(3, width, device=DEV)      # without the pair table: the row times the factor
    ops.pair_embed(plain_rows, dev(table, table_dtype), dev([3, 0, 49], torch.int32), scale)
    assert np.abs(plain_rows.cpu().numpy() - table[[3, 0, 49]] * scale).max() <= 1e-5


def test_big_factors_of_the_pair_hash_do_not_overflow():
    from alofa_amd import ops
    vocab, width, buckets, mp, mc = 70000, 8, 65521, 2 ** 31 - 1, 99991
    rng = np.random.default_rng(1)
    table, pairs = rng.normal(0, 1, (vocab, width)).astype(np.float32), rng.normal(0, 1, (buckets + 1, width)).astype(np.float32)
    ids = [69999, 69998, 12345, 69999]
    out = torch.empty(4, width, device=DEV)
    state = torch.zeros((1, 1), dtype=torch.int32, device=DEV)
    ops.pair_embed(out, dev(table), dev(ids, torch.int32), 1.0, None, dev(pairs), dev([0, 1, 2, 3], torch.int32), state, rows_of([(0, 4)], 1), buckets, mp, mc)
    assert np.abs(out.cpu().numpy() - pr.embed(ids, table.astype(np.float64), 1.0, pairs.astype(np.float64), buckets, mp, mc)).max() <= 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_join_of_two_streams(dtype):
    from alofa_amd import ops
    rng = np.random.default_rng(2)
    x, x0, w = rng.normal(0, 1, (13, 40)), rng.normal(0, 3, (13, 40)), b16(rng.normal(0, 0.2, (40, 80)))
    both = torch.empty(13, 80, dtype=dtype, device=DEV)
    ops.concat_rows(both, dev(x), dev(x0))
    out = torch.empty(13, 40, device=DEV)
    ops.gemm(out, both, dev(w, dtype), exact=dtype is torch.float32)
    if dtype is torch.float32:
        want = pr.join_streams(x.astype(np.float32).astype(np.float64), x0.astype(np.float32).astype(np.float64), w)
        assert np.abs(out.cpu().numpy() - want).max() <= 1e-5
    else:
        assert np.abs(out.cpu().numpy() - pr.join_streams(b16(x), b16(x0), w)).max() <= 1e-4


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("width, pad", [(10, 16), (64, 64), (100, 128), (200, 256)])
def test_norm_of_the_latent_left_as_keys_and_values(width, pad, exact):
    from alofa_amd import ops
    rng = np.random.default_rng(width)
    x, w = rng.normal(0.5, 2.0, (7, width)).astype(np.float32), rng.normal(1, 0.3, width).astype(np.float32)
    out = torch.full((7, 3 + 2 * pad), 9.0, device=DEV)
    ops.rmsnorm_spread(out[:, 3:], dev(x), dev(w), 1e-5, pad, 2, exact)
    got = out.cpu().numpy()
    want = pr.rms_norm(x.astype(np.float64), w.astype(np.float64), 1e-5)
    for k in range(2):
        assert np.abs(got[:, 3 + k * pad:3 + k * pad + width] - want).max() <= (1e-6 if exact else 1e-5) * np.abs(want).max()
        assert (got[:, 3 + k * pad + width:3 + (k + 1) * pad] == 0).all()
    assert (got[:, :3] == 9.0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_channel_scale_cap_and_squared_relu(dtype):
    from alofa_amd import ops
    rng = np.random.default_rng(3)
    exact = dtype is torch.float32
    x, g = b16(rng.normal(0, 2, (9, 50))), b16(rng.normal(0, 3, (9, 70)))
    xs = dev(x, dtype)
    ops.sigmoid_gate(xs, dev(g, dtype)[:, 20:], exact)
    want = x * pr.sigmoid(g[:, 20:])
    assert np.abs(xs.float().cpu().numpy() - want).max() <= (1e-6 if exact else 2e-2)
    stream, add, scale = rng.normal(0, 1, (9, 50)).astype(np.float32), rng.normal(0, 1, (9, 50)).astype(np.float32), rng.normal(1, 0.5, 50).astype(np.float32)
    s = dev(stream)
    ops.add_channel_scaled(s, dev(add), dev(scale), exact)
    assert np.abs(s.cpu().numpy() - (stream + scale.astype(np.float64) * add)).max() <= 1e-6
    z = rng.normal(0, 40, (5, 33)).astype(np.float32)
    zs = dev(z)
    ops.softcap_(zs, 30.0, exact)
    assert np.abs(zs.cpu().numpy() - pr.soft_cap(z.astype(np.float64), 30.0)).max() <= 1e-5
    r = dev(x, dtype)
    ops.relu_squared(r, r)
    sq = np.maximum(x, 0) ** 2
    assert (np.abs(r.float().cpu().numpy() - sq) <= (1e-6 if exact else 2.0 ** -8) * np.maximum(sq, 1.0)).all()


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("experts, top", [(8, 3), (5, 5), (3, 1), (64, 6), (100, 7), (300, 2)])
def test_the_choice_of_experts(experts, top, exact):
    from alofa_amd import ops
    rng = np.random.default_rng(experts)
    z = rng.normal(0, 2, (37, experts)).astype(np.float32)
    z[3, :] = 0.25                      # all equal: the lowest indices win
    if experts > 3:
        z[5, [1, 3]] = z[5].max() + 1   # a tie at the top
    dense, chosen, weights = torch.empty(37, experts, device=DEV), torch.empty(37, top, dtype=torch.int32, device=DEV), torch.empty(37, top, device=DEV)
    ops.route_top(dev(z), dense, chosen, weights, top, 2.0, False, exact)
    # (the plain choice from products whose sigmoid is the score: the identity as input, the products as router rows)
    want_e, want_w = pr.route(z.astype(np.float64), np.eye(experts), top, 2.0)
    order = np.argsort(-z.astype(np.float64), axis=-1, kind="stable")[:, :top]
    assert (chosen.cpu().numpy() == order).all()
    assert np.abs(weights.cpu().numpy() - 2.0 * pr.sigmoid(np.take_along_axis(z.astype(np.float64), order, -1))).max() <= 1e-6
    assert chosen[3].tolist() == list(range(top))
    d = np.zeros((37, experts))
    np.put_along_axis(d, order, weights.cpu().numpy().astype(np.float64), -1)
    assert (dense.cpu().numpy() == d.astype(np.float32)).all()
    if top < experts:      # where the scores do not saturate the plain choice by score is the same
        clear = np.abs(z).max(axis=1) < 8
        assert (want_e[clear] == order[clear]).all() and np.allclose(want_w[clear], 2.0 * pr.sigmoid(np.take_along_axis(z.astype(np.float64), order, -1))[clear])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_experts_as_one_product(dtype):
    """The experts' activations side by side, weighted by the choice, against the plain sum over the experts a token takes."""
    from alofa_amd import ops
    rng = np.random.default_rng(4)
    exact = dtype is torch.float32
    T, h, E, top, ff, sff = 21, 40, 5, 2, 12, 20
    hn = b16(rng.normal(0, 1, (T, h)))
    experts = [tuple(b16(rng.normal(0, s, shape)) for s, shape in ((0.3, (ff, h)), (0.3, (ff, h)), (0.3, (h, ff)))) for _ in range(E)]
    shared = tuple(b16(rng.normal(0, s, shape)) for s, shape in ((0.3, (sff, h)), (0.3, (sff, h)), (0.3, (h, sff))))
    w_router = b16(rng.normal(0, 0.5, (E, h)))
    want = pr.routed_experts(hn, w_router, experts, shared, top, 1.5, 1.0, 0.6)
    x = dev(hn, dtype)
    z = torch.empty(T, E, device=DEV)
    ops.gemm(z, x, dev(w_router, dtype), exact=exact)
    dense, chosen, weights = torch.empty(T, E, device=DEV), torch.empty(T, top, dtype=torch.int32, device=DEV), torch.empty(T, top, device=DEV)
    ops.route_top(z, dense, chosen, weights, top, 1.5, False, exact)
    F = E * ff + sff
    w_gate, w_up = (dev(np.concatenate([e[k] for e in experts] + [shared[k]], axis=0), dtype) for k in (0, 1))
    w_down = dev(np.concatenate([e[2] for e in experts] + [shared[2]], axis=1), dtype)
    g, u, act = (torch.empty(T, F, dtype=dtype, device=DEV) for _ in range(3))
    ops.gemm(g, x, w_gate, exact=exact)
    ops.gemm(u, x, w_up, exact=exact)
    ops.clamped_glu(act, g, u, dense, E, ff, sff, 1.0, 0.6, 1.702, exact)
    out = torch.zeros(T, h, device=DEV)
    ops.gemm(out, act, w_down, add_to_out=True, exact=exact)
    assert np.abs(out.cpu().numpy() - want).max() <= (1e-5 if exact else 3e-2) * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, din, dout, rows", [(6, 64, 64, 5), (3, 40, 16, 1), (5, 15, 9, 70), (20, 16, 64, 130), (2, 128, 256, 33), (4, 32, 48, 300), (3, 96, 40, 1000)])
def test_a_projection_per_head(heads, din, dout, rows, dtype):
    from alofa_amd import ops
    rng = np.random.default_rng(heads)
    exact = dtype is torch.float32
    x, w = b16(rng.normal(0, 1, (rows, heads * din + 8))), b16(rng.normal(0, din ** -0.5, (heads, dout, din)))
    out = torch.full((rows, heads * dout + 8), 5.0, dtype=dtype, device=DEV)
    ops.head_project(out[:, 8:], dev(x, dtype)[:, :heads * din], dev(w, dtype), exact)
    want = np.einsum("tai,aoi->tao", x[:, :heads * din].reshape(rows, heads, din), w).reshape(rows, heads * dout)
    got = out.float().cpu().numpy()
    assert np.abs(got[:, 8:] - want).max() <= (1e-5 if exact else 2e-2) * max(1.0, np.abs(want).max())
    assert (got[:, :8] == 5.0).all()


@pytest.mark.parametrize("T, h, E, top, ff, sff", [(21, 40, 5, 2, 16, 24), (1, 64, 8, 3, 96, 96), (150, 72, 16, 4, 8, 0), (64, 48, 4, 1, 40, 8), (5, 200, 3, 1, 24, 48),
                                                  (300, 64, 4, 2, 72, 40), (700, 40, 6, 3, 16, 0)])
def test_routed_experts_slot_by_slot(T, h, E, top, ff, sff):
    """The rows sorted by expert and every expert against its own rows only, against the plain sum over the experts a token
    takes; every row lands in exactly one slot per choice."""
    from alofa_amd import ops
    rng = np.random.default_rng(T)
    bf = torch.bfloat16
    hn = b16(rng.normal(0, 1, (T, h)))
    experts = [tuple(b16(rng.normal(0, s, shape)) for s, shape in ((0.3, (ff, h)), (0.3, (ff, h)), (0.3, (h, ff)))) for _ in range(E)]
    shared = tuple(b16(rng.normal(0, s, shape)) for s, shape in ((0.3, (sff, h)), (0.3, (sff, h)), (0.3, (h, sff)))) if sff else None
    w_router = b16(rng.normal(0, 0.5, (E, h)))
    want = pr.routed_experts(hn, w_router, experts, shared, top, 1.5, 1.0, 0.6)
    x = dev(hn, bf)
    z = torch.empty(T, E, device=DEV)
    ops.gemm(z, x, dev(w_router, bf))
    dense, chosen, weights = torch.empty(T, E, device=DEV), torch.empty(T, top, dtype=torch.int32, device=DEV), torch.empty(T, top, device=DEV)
    ops.route_top(z, dense, chosen, weights, top, 1.5, False, False)
    both = experts + ([shared] if sff else [])
    w_gate, w_up = (dev(np.concatenate([e[k] for e in both], axis=0), bf) for k in (0, 1))
    w_down = dev(np.concatenate([e[2] for e in both], axis=1), bf)
    assert ops.can_group_experts(x, w_gate, ff, sff)
    rows = ops.ExpertRows(T, top, E, sff > 0, lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device=DEV))
    ops.expert_rows(rows, chosen, weights)
    row_in, slot_of, tile_batch = rows.row_in.cpu().numpy(), rows.slot_of.cpu().numpy(), rows.tile_batch.cpu().numpy()
    picks = chosen.cpu().numpy()
    for t in range(T):
        for k in range(top):
            slot = slot_of[t * top + k]
            assert row_in[slot] == t and tile_batch[slot // rows.tile_rows] == picks[t, k]
        if sff:
            assert row_in[slot_of[T * top + t]] == t and tile_batch[slot_of[T * top + t] // rows.tile_rows] == E
    assert (row_in >= 0).sum() == T * (top + (1 if sff else 0))
    act = torch.zeros(rows.slots, (max(ff, sff) + 7) // 8 * 8, dtype=bf, device=DEV)
    ops.experts_gate_up(act, x, w_gate, w_up, rows, ff, sff, 1.0, 0.6, 1.702)
    y = torch.empty(rows.slots, h, device=DEV)
    ops.experts_down(y, act, w_down, rows, ff, sff)
    stream = rng.normal(0, 1, (T, h)).astype(np.float32)
    scale = rng.normal(1, 0.3, h).astype(np.float32)
    out = dev(stream)
    ops.experts_sum(out, y, rows, dev(scale))
    got = (out.cpu().numpy().astype(np.float64) - stream) / scale
    assert np.abs(got - want).max() <= 3e-2 * max(1.0, np.abs(want).max())
    again = dev(stream)      # the same rows in another order of arrival give the same bits
    ops.expert_rows(rows, chosen, weights)
    ops.experts_gate_up(act, x, w_gate, w_up, rows, ff, sff, 1.0, 0.6, 1.702)
    ops.experts_down(y, act, w_down, rows, ff, sff)
    ops.experts_sum(again, y, rows, dev(scale))
    assert torch.equal(again, out)
