"""Rerupel without a GPU: the configuration's keys and checks, the tensor list, the order of runs, and the plain
implementation's own consistency."""
import copy
import json

import numpy as np
import pytest

from alofa_amd.config.registry import config_from_dict, load_config
from alofa_amd.errors import AlofaError
from alofa_amd.model import check_spec, expected_tensors
from alofa_amd.weights import write_random_model
from plain import rerupel as pr
from rerupel_cases import RERUPEL


@pytest.mark.parametrize("name", list(RERUPEL))
def test_config_round_trip_and_tensor_list(name, tmp_path):
    cfg = config_from_dict(RERUPEL[name])
    assert config_from_dict(cfg.to_dict()) == cfg
    spec = cfg.spec()
    check_spec(spec)
    write_random_model(RERUPEL[name], tmp_path, seed=1)
    assert load_config(tmp_path) == cfg
    w = pr.read_weights(tmp_path)
    expected = expected_tensors(spec)
    assert set(w) == {n for n, r in expected.items() if not r.optional}
    assert all(tuple(w[n].shape) == tuple(expected[n].shape) for n in w)
    raw = RERUPEL[name]
    assert ("bigram" in w) == ("bigram" in raw["embedding"]) and ("loop.in" in w) == ("loop" in raw)
    for i, l in enumerate(raw["layers"]):
        m = l["mixer"]
        assert w[f"l{i}.mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"]) and w[f"l{i}.mix.uv"].shape == (m["heads"] * m["vdim"], m["kv_rank"])
        assert (f"l{i}.ls2" in w) == (l["mlp"] is not None)


def test_the_order_of_runs():
    cfg = config_from_dict(RERUPEL["A"])      # layers 1 and 2 twice
    spec = cfg.spec()
    assert [(e.layer, e.join) for e in spec.order] == [(0, None), (1, 0), (2, None), (1, 0), (2, None)]
    assert all(e.cache_of is None for e in spec.order)      # every pass keeps a cache of its own
    assert pr.run_order(RERUPEL["A"]) == ([0, 1, 2, 1, 2], {1, 3})
    spec = config_from_dict(RERUPEL["B"]).spec()             # the first layer three times, then the second
    assert [(e.layer, e.join) for e in spec.order] == [(0, 0), (0, 0), (0, 0), (1, None)]
    spec = config_from_dict(RERUPEL["C"]).spec()             # no loop: no join, and no tensor for one
    assert [(e.layer, e.join) for e in spec.order] == [(0, None), (1, None)] and spec.joins == ()


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="windowed"), "no such mixer"),
    (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "no such feed-forward"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "more experts than there are"),
    (lambda c: c["loop"].update(stop=7), "loop names a run of existing layers"),
    (lambda c: c["loop"].update(times=0), "loop names a run of existing layers"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "lacks a required key"),
    (lambda c: c.update(logit_softcap=0.0), "must be positive"),
    (lambda c: c["embedding"]["bigram"].update(buckets=0), "must be positive"),
])
def test_what_the_configuration_refuses(change, message):
    raw = copy.deepcopy(RERUPEL["A"])
    change(raw)
    with pytest.raises(AlofaError, match=message):
        config_from_dict(raw)


def test_weights_that_do_not_fit_are_named(tmp_path):
    from alofa_amd.weights.loader import load_weights
    write_random_model(RERUPEL["A"], tmp_path, seed=1)
    raw = json.loads((tmp_path / "config.json").read_text())
    raw["layers"][1]["mlp"]["router"]["experts"] = 5
    (tmp_path / "config.json").write_text(json.dumps(raw))
    with pytest.raises(AlofaError, match=r"l1\.mlp\.e4\.gate"):
        load_weights(tmp_path, expected_tensors(load_config(tmp_path).spec()))


# ---- the plain implementation against itself

@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    d = tmp_path_factory.mktemp("plain_a")
    write_random_model(RERUPEL["A"], d, seed=5)
    return pr.read_config(d), pr.read_weights(d)


def test_a_position_depends_on_nothing_after_it(model_a):
    cfg, w = model_a
    ids = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 40)]
    full = pr.forward_logits(w, cfg, ids)
    assert np.abs(pr.forward_logits(w, cfg, ids[:17]) - full[:17]).max() < 1e-9
    other = ids[:30] + [(ids[30] + 1) % cfg["vocab"]] + ids[31:]
    moved = np.abs(pr.forward_logits(w, cfg, other) - full).max(axis=1)
    assert moved[:30].max() < 1e-9 and moved[30:].min() > 1e-6


def test_the_pair_rows():
    assert pr.bigram_rows([5, 7, 7, 0], 11, 3, 2) == [11, (15 + 14) % 11, (21 + 14) % 11, 21 % 11]
    assert pr.bigram_rows([4], 11, 3, 2) == [11]


def test_the_choice_of_experts():
    hn = np.array([[1.0, 0.0], [0.0, 1.0]])
    w_router = np.array([[0.5, 2.0], [3.0, 2.0], [0.5, -1.0], [3.0, 0.0]])      # the first row ties experts 1 and 3, the second 0 and 1
    chosen, weights = pr.route(hn, w_router, 2, 10.0)
    assert chosen.tolist() == [[1, 3], [0, 1]]
    assert np.allclose(weights[0], 10.0 * pr.sigmoid(3.0)) and np.allclose(weights[1], 10.0 * pr.sigmoid(2.0))


def test_the_expert_clamps_before_it_gates():
    one = np.eye(1)
    for g, u, want in [(5.0, 0.0, 2.0 * pr.sigmoid(1.702 * 2.0)), (-5.0, 9.0, -5.0 * pr.sigmoid(1.702 * -5.0) * 3.0), (1.0, -9.0, pr.sigmoid(1.702) * -1.0)]:
        assert np.isclose(pr.clamped_expert(np.array([[1.0]]), one * g, one * u, one, 2.0)[0, 0], want)


def test_the_cap_and_the_norm():
    assert np.allclose(pr.soft_cap(np.array([0.0, 1e-3, 1e6, -1e6]), 30.0), [0.0, 1e-3, 30.0, -30.0], atol=1e-6)
    x = np.array([[3.0, 4.0]])
    assert np.allclose(pr.rms_norm(x, np.array([1.0, 2.0]), 0.5), x / np.sqrt(12.5 + 0.5) * [1.0, 2.0])
