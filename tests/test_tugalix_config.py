"""Tugalix without a GPU: its configuration (keys, checks, sizes that only the tensors give), the list of tensors its
parts read, the random-weights mode, and the plain implementation's own consistency."""
import copy
import json

import numpy as np
import pytest

from alofa_amd.config.registry import architectures, config_from_dict, load_config
from alofa_amd.errors import AlofaError
from alofa_amd.model import check_spec, expected_tensors
from alofa_amd.weights import write_random_model
from plain import tugalix as pt
from tugalix_cases import TUGALIX


def test_registered_by_its_plain_architecture_key():
    assert "Tugalix" in architectures()
    cfg = config_from_dict(TUGALIX["A"])
    assert type(cfg).__name__ == "TugalixConfig" and cfg.width == 64 and len(cfg.layers) == 3
    assert config_from_dict(cfg.to_dict()) == cfg


@pytest.mark.parametrize("name", list(TUGALIX))
def test_spec_and_tensor_list(name):
    raw = TUGALIX[name]
    spec = config_from_dict(raw).spec()
    check_spec(spec)
    names = expected_tensors(spec)
    assert {"embed", "embed.norm", "embed.norm.b", "final.norm", "final.norm.b", "head"} <= set(names)
    for i, layer in enumerate(raw["layers"]):
        assert tuple(names[f"l{i}.dwa"].shape) == (i + 2,)
        assert tuple(names[f"l{i}.canon1"].shape) == (raw["width"], raw["canon"]["taps"])
        assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None) == (f"l{i}.canon2" in names) == (f"l{i}.mlp.act" in names)
        m = layer["mixer"]
        if layer["type"] == "parallel":
            assert tuple(names[f"l{i}.mix.left.k"].shape) == (m["left"]["kv_heads"] * m["left"]["dim"], raw["width"])
            assert tuple(names[f"l{i}.mix.left.o"].shape) == (raw["width"], m["left"]["heads"] * m["left"]["vdim"])
            assert tuple(names[f"l{i}.mix.right.u"].shape) == (m["right"]["heads"], m["right"]["dim"])
            assert tuple(names[f"l{i}.mix.right.w2"].shape) == (m["right"]["heads"] * m["right"]["dim"], m["right"]["rank"])
        elif layer["type"] == "gla":
            assert tuple(names[f"l{i}.mix.norm"].shape) == (m["vdim"],)
            assert tuple(names[f"l{i}.mix.a1"].shape) == (m["rank"], raw["width"])
        else:
            assert tuple(names[f"l{i}.mix.g"].shape) == (m["heads"] * m["vdim"], raw["width"])


def test_ranks_come_from_the_tensors_when_the_keys_are_absent(tmp_path):
    d = write_random_model(TUGALIX["A"], tmp_path / "m", seed=1)
    raw = json.loads((d / "config.json").read_text())
    del raw["layers"][1]["mixer"]["right"]["rank"], raw["layers"][2]["mixer"]["rank"]
    (d / "config.json").write_text(json.dumps(raw))
    bare = config_from_dict(raw)
    assert bare.wants_shapes()
    with pytest.raises(AlofaError):
        bare.spec()
    cfg = load_config(d)
    assert not cfg.wants_shapes() and cfg == config_from_dict(TUGALIX["A"])


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="mamba"), "no such mixer"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "one decay per head"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "kv_heads must divide"),
    (lambda c: c["layers"][2]["mixer"].pop("tau"), "lacks a required key"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "no such feed-forward"),
    (lambda c: c.pop("logit_scale"), "lacks a required key"),
    (lambda c: c["canon"].update(taps=0), "must be positive"),
])
def test_bad_configurations_are_refused_by_name(change, word):
    raw = copy.deepcopy(TUGALIX["A"])
    change(raw)
    with pytest.raises(AlofaError) as e:
        config_from_dict(raw)
    assert word in str(e.value)


def test_random_model_has_what_the_plain_model_reads(tmp_path):
    d = write_random_model(TUGALIX["B"], tmp_path / "m", seed=3)
    cfg, w = pt.read_config(d), pt.read_weights(d)
    ids = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 30)]
    logits = pt.forward_logits(w, cfg, ids)
    assert logits.shape == (30, cfg["vocab"]) and np.isfinite(logits).all() and logits.std() > 0.05
    # causal: a position's logits do not move when tokens are added behind it
    more = pt.forward_logits(w, cfg, ids + [5, 6, 7])
    assert np.abs(more[:30] - logits).max() <= 1e-9
    # and every mechanism is felt: without the filters, the averages or a mixer the logits differ
    for name in ("l0.canon1", "l1.mix.right.u", "l1.mix.left.v", "l2.mix.g", "l1.mlp.act"):
        changed = dict(w)
        changed[name] = w[name] * 0.0 + (1.0 if name.endswith("act") else 0.0)
        assert np.abs(pt.forward_logits(changed, cfg, ids) - logits).max() > 1e-4, name


def test_plain_recurrence_matches_its_closed_form():
    """o_t = sum_{s <= t} (q_t . (prod_{s < r <= t} w_r) * k_s) v_s for the read-out after the update."""
    rng = np.random.default_rng(1)
    T, dk, dv = 9, 5, 3
    q, k, v, w = rng.normal(size=(T, dk)), rng.normal(size=(T, dk)), rng.normal(size=(T, dv)), rng.uniform(0.5, 1, (T, dk))
    got = pt.decayed_outer_sum(q, k, v, w)
    for t in range(T):
        want = np.zeros(dv)
        for s in range(t + 1):
            want += (q[t] * np.prod(w[s + 1:t + 1], axis=0) * k[s]).sum() * v[s]
        assert np.abs(got[t] - want).max() <= 1e-12
    u = rng.normal(size=dk)
    with_bonus = pt.decayed_outer_sum(q, k, v, w, bonus=u)
    for t in range(T):
        want = (q[t] * u * k[t]).sum() * v[t]
        for s in range(t):
            want = want + (q[t] * np.prod(w[s + 1:t], axis=0) * k[s]).sum() * v[s]
        assert np.abs(with_bonus[t] - want).max() <= 1e-12
