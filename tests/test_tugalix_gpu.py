"""Tugalix through the engine against the plain implementation, in float32 and bfloat16: whole prompts, decoding token
by token, portions down to two tokens, unequal requests in one batch, slots and pages that are used again, weights
made so that one far key or one old token decides, and greedy generation through the engine's own loop."""
import json

import numpy as np
import pytest

from helpers import assert_close, bulk_and_tail, collect, mixed, portions, random_ids, whole
from plain import tugalix as pt
from tugalix_cases import TUGALIX, plain_logits, plain_model

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
LENGTHS = {"A": 90, "B": 75, "C": 120, "D": 150, "E": 100}


@pytest.fixture(scope="module")
def replayers(tugalix_dirs):
    from alofa_amd.replay import Replayer
    made = {}

    def get(name, dtype, max_tokens=512):
        key = (name, dtype, max_tokens)
        if key not in made:
            made[key] = Replayer(tugalix_dirs[name], dtype, max_tokens, max_requests=4)
        r = made[key]
        assert not r.cache.requests, "a test left requests behind"
        return r
    return get


def ids_of(name, seed=7, n=None):
    return random_ids(seed, n or LENGTHS[name], TUGALIX[name]["vocab"])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TUGALIX))
def test_whole_prompt(replayers, tugalix_dirs, name, dtype):
    ids = ids_of(name)
    got = collect(replayers(name, dtype), whole("w", ids))["w"]
    assert_close(got, plain_logits(tugalix_dirs[name], tuple(ids)), dtype, f"{name} whole")


def test_the_stream_after_every_layer(replayers, tugalix_dirs):
    """float32, layer by layer: the engine keeps every layer's output in a stack for its average over depth."""
    import torch
    name = "A"
    ids = ids_of(name, n=33)
    r = replayers(name, "float32")
    collect(r, whole("w", ids))
    cfg, w = plain_model(str(tugalix_dirs[name]))
    want = pt.forward_hidden(w, cfg, ids)
    L = len(cfg["layers"])
    stack = r.fn.scratch("depth_stack", (L + 1, len(ids), cfg["width"]), torch.float32).cpu().numpy().astype(np.float64)
    for i in range(L):
        got = sum(w[f"l{i}.dwa"][j] * stack[j] for j in range(i + 2))
        assert np.abs(got - want[i]).max() <= 1e-5 * max(1.0, np.abs(want[i]).max()), f"layer {i}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TUGALIX))
def test_prompt_then_token_by_token(replayers, tugalix_dirs, name, dtype):
    ids = ids_of(name)
    got = collect(replayers(name, dtype), bulk_and_tail("t", ids, tail=40))["t"]
    assert_close(got, plain_logits(tugalix_dirs[name], tuple(ids)), dtype, f"{name} bulk+tail")


@pytest.mark.parametrize("dtype", DTYPES)
def test_from_the_first_token_one_by_one(replayers, tugalix_dirs, dtype):
    """Long decoding from an empty state: nothing but single tokens, the first tokens of the sequence included."""
    name = "B"
    ids = ids_of(name, seed=3, n=70)
    got = collect(replayers(name, dtype), bulk_and_tail("t", ids, tail=69))["t"]
    assert_close(got, plain_logits(tugalix_dirs[name], tuple(ids)), dtype, f"{name} one by one")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TUGALIX))
def test_portions_of_changing_size(replayers, tugalix_dirs, name, dtype):
    ids = ids_of(name)
    steps = portions("p", ids)
    assert min(len(s["entries"][0]["tokens"]) for s in steps) == 2
    got = collect(replayers(name, dtype), steps)["p"]
    assert_close(got, plain_logits(tugalix_dirs[name], tuple(ids)), dtype, f"{name} portions")
    other = collect(replayers(name, dtype), portions("q", ids, sizes=(2, 19, 2, 2, 33, 3, 17)))["q"]
    assert_close(other, plain_logits(tugalix_dirs[name], tuple(ids)), dtype, f"{name} other portions")
    if dtype == "float32":      # the cut changes nothing beyond rounding
        assert np.abs(other - got).max() <= 2e-6 * max(1.0, np.abs(got).max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C", "E"])
def test_unequal_requests_together_with_slots_and_pages_used_again(tugalix_dirs, name, dtype):
    """Up to four live requests, seven in all: portions beside single tokens, a request left out now and then; a slot and
    its pages go to the next request as soon as one ends. Every request must come out as it does alone."""
    from alofa_amd.replay import Replayer
    vocab, top = TUGALIX[name]["vocab"], LENGTHS[name]
    requests = {f"r{i}": random_ids(200 + i, n, vocab) for i, n in enumerate([top, 37, top - 23, 64, 35, top - 9, 50])}
    steps, peak = mixed(requests, seed=9, tail=20)
    assert max(len(s["entries"]) for s in steps) >= 3
    r = Replayer(tugalix_dirs[name], dtype, peak, max_requests=4)
    got = collect(r, steps)
    r.cache.check()
    assert not r.cache.requests
    for req, ids in requests.items():
        assert_close(got[req], plain_logits(tugalix_dirs[name], tuple(ids)), dtype, f"{name} mixed {req}")


def test_a_slot_used_again_starts_from_nothing(replayers, tugalix_dirs):
    """The same request twice in the same slot, a different one between them: state of an earlier owner must not show."""
    name = "C"
    r = replayers(name, "float32")
    a, b = ids_of(name, seed=1, n=40), ids_of(name, seed=2, n=55)
    first = collect(r, whole("a", a))["a"]
    assert r.cache.slot is not None
    collect(r, whole("b", b))
    again = collect(r, portions("a", a, sizes=(3, 2, 9)))["a"]
    assert np.abs(again - first).max() <= 2e-6 * max(1.0, np.abs(first).max())
    assert_close(again, plain_logits(tugalix_dirs[name], tuple(a)), "float32", "slot used again")


def _rewrite(model_dir, out_dir, change):
    """A copy of a model folder with some tensors changed by ``change(name -> float32 tensor)``."""
    import torch
    from safetensors.torch import load_file, save_file
    out_dir.mkdir(parents=True, exist_ok=True)
    (out_dir / "config.json").write_text((model_dir / "config.json").read_text())
    w = {k: v.float() for k, v in load_file(str(model_dir / "model.safetensors")).items()}
    change(w)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, str(out_dir / "model.safetensors"))
    return out_dir


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_that_decides(tugalix_dirs, tmp_path, dtype):
    """Attention with queries and keys scaled up, so that single keys carry nearly all the weight, hundreds of tokens
    back and across page borders, in a prompt's portions and in decoding."""
    from alofa_amd.replay import Replayer
    name = "A"

    def sharpen(w):
        w["l1.mix.left.q"] *= 6.0
        w["l1.mix.left.k"] *= 6.0
    d = _rewrite(tugalix_dirs[name], tmp_path / "sharp", sharpen)
    ids = ids_of(name, seed=21, n=330)
    cfg, w = plain_model(str(d))
    # the weights do concentrate: in the plain model the largest softmax weight of late queries is large
    ref = plain_logits(d, tuple(ids))
    r = Replayer(d, dtype, 384, max_requests=4)
    got = collect(r, portions("p", ids, sizes=(150, 2, 61, 17, 3)))["p"]
    assert_close(got, ref, dtype, "far key, portions")
    got = collect(r, bulk_and_tail("t", ids, tail=40))["t"]
    assert_close(got, ref, dtype, "far key, decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_an_old_token_that_the_state_must_keep(tugalix_dirs, tmp_path, dtype):
    """Decays pushed towards one and values scaled up: what a recurrent layer reads out late in the sequence comes from
    tokens hundreds of steps back, so a state that is lost or mixed up between steps shows."""
    from alofa_amd.replay import Replayer
    name = "C"
    d = tmp_path / "slow"

    def slow(w):
        w["l1.mix.a2.b"] += 6.0
        w["l1.mix.v"] *= 4.0
        w["l0.mix.v"] *= 4.0
    _rewrite(tugalix_dirs[name], d, slow)
    raw = json.loads((d / "config.json").read_text())
    raw["layers"][0]["mixer"]["decay"] = [0.999, 0.9995, 1.0]
    (d / "config.json").write_text(json.dumps(raw))
    ids = ids_of(name, seed=4, n=300)
    ref = plain_logits(d, tuple(ids))
    r = Replayer(d, dtype, 320, max_requests=4)
    got = collect(r, portions("p", ids, sizes=(2, 131, 5, 64, 16, 3)))["p"]
    assert_close(got, ref, dtype, "old token, portions")
    got = collect(r, bulk_and_tail("t", ids, tail=45))["t"]
    assert_close(got, ref, dtype, "old token, decoding")


def test_greedy_generation_through_the_engine(tugalix_dirs):
    """The engine's own loop and scheduler: prompts of unequal length, more than a batch holds at once."""
    from alofa_amd import Engine
    for name in ("A", "C"):
        cfg, w = plain_model(str(tugalix_dirs[name]))
        prompts = [random_ids(300 + i, n, cfg["vocab"]) for i, n in enumerate((5, 23, 2, 41, 17, 9))]
        want = [pt.greedy(w, cfg, p, 8) for p in prompts]
        engine = Engine(tugalix_dirs[name], dtype="float32", max_tokens=64, max_batch=4, token_budget=48, max_chunk=16)
        assert engine.generate(prompts, max_new=8) == want, name
        engine.cache.check()
        got = Engine(tugalix_dirs[name], dtype="bfloat16", max_tokens=64, max_batch=4).generate(prompts, max_new=8)
        agree = sum(a == b for g, r in zip(got, want) for a, b in zip(g, r))
        assert agree >= 40, f"{name}: {agree}/48 greedy tokens agree with the plain model in bfloat16"


def test_decode_steps_replay_a_captured_graph(replayers, tugalix_dirs):
    """Single-token steps of a model that carries state run as a captured graph; every replay must move the state on."""
    name = "A"
    r = replayers(name, "bfloat16")
    if not r.fn.use_graphs:
        pytest.skip("graphs are switched off")
    ids = ids_of(name, seed=5, n=60)
    before = r.fn.graph_replays
    got = collect(r, bulk_and_tail("t", ids, tail=30))["t"]
    assert r.fn.graph_replays > before
    assert_close(got, plain_logits(tugalix_dirs[name], tuple(ids)), "bfloat16", "graph decode")


def test_the_programs_take_the_design_by_its_config(tugalix_dirs, tmp_path):
    """bin/generate and bin/trace_run on a folder whose config.json names the architecture plainly and leaves the ranks of
    the decay projections to the tensors' shapes."""
    import os
    import subprocess
    from conftest import ROOT
    name = "A"
    d = tmp_path / "bare"
    d.mkdir()
    raw = json.loads((tugalix_dirs[name] / "config.json").read_text())
    del raw["layers"][1]["mixer"]["right"]["rank"], raw["layers"][2]["mixer"]["rank"]
    (d / "config.json").write_text(json.dumps(raw))
    (d / "model.safetensors").write_bytes((tugalix_dirs[name] / "model.safetensors").read_bytes())
    cfg, w = plain_model(str(tugalix_dirs[name]))
    prompts = [random_ids(1, 5, cfg["vocab"]), random_ids(2, 19, cfg["vocab"])]
    want = [pt.greedy(w, cfg, p, 5) for p in prompts]
    env = dict(os.environ, ALOFA_WEIGHTS=str(d), ALOFA_DTYPE="float32", ALOFA_MAX_NEW="5", ALOFA_MAX_TOKENS="64",
               ALOFA_PROMPT_IDS=";".join(",".join(map(str, p)) for p in prompts))
    p = subprocess.run([str(ROOT / "bin" / "generate")], env=env, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [[int(t) for t in line.split(",")] for line in p.stdout.strip().splitlines()] == want
    ids = ids_of(name, seed=12, n=70)
    steps = portions("a", ids, sizes=(33, 2, 1, 1, 20, 1))
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", "bfloat16", "--out", str(tmp_path / "out"), "--max-tokens", "128"],
                       input=text, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    got = np.concatenate([np.fromfile(tmp_path / "out" / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab"]) for s in steps])
    assert_close(got, plain_logits(tugalix_dirs[name], tuple(ids)), "bfloat16", "program")
