"""The Roravik decoder in the engine against the plain implementation: whole requests, tails fed one by one,
portions of prompts down to two tokens, batches of unequal requests against each alone, slots, pages and
states used again, windows passed in prompts and in decoding, long decoding, greedy generation through the
Python entry point, the command line and the replay program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests import roravik_models as rm
from tests.plain import roravik_plain as plain

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# 32-bit: the worst position's largest difference over that position's largest logit.
TOL = {"float32": 3e-4}
# bfloat16: these models turn small differences into large ones (attention scales far above 1/sqrt(dim), a single
# chosen expert, recurrences that keep what a position wrote), so a rounding now and then flips a choice of experts
# and reaches every later position: the 32-bit runs pin every position, the bfloat16 runs pin the bulk of them against
# the plain implementation and against each other.
BF16_MOST = {"A": (0.5, 6e-2), "B": (0.5, 5e-2), "C": (0.5, 1e-1), "D": (0.5, 6e-2)}
BF16_SAME = {"A": (0.8, 6e-2), "B": (0.8, 6e-2), "C": (0.8, 1e-1), "D": (0.8, 6e-2)}
LENGTHS = {"A": [1, 2, 21, 66, 150, 211], "B": [3, 64, 65, 131, 262], "C": [1, 8, 30, 77], "D": [5, 40, 129]}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("roravik")
    out = {}
    for name, (cfg, seed) in rm.CONFIGS.items():
        tensors = rm.random_tensors(cfg, seed)
        out[name] = (rm.write_model(str(root / name), cfg, tensors), cfg, rm.as_double(tensors))
    return out


def _engine(path, dtype, **kw):
    from rocml_amd.engine import Engine
    from rocml_amd.weights import load_model
    kw.setdefault("max_tokens", 4096)
    return Engine(load_model(path, dtype=dtype, device="cuda:0"), **kw)


def _prompts(name, cfg):
    return [helpers.random_tokens(n, cfg["vocab"], 300 + i) for i, n in enumerate(LENGTHS[name])]


def _ref(cfg, tensors, p):
    return plain.forward(cfg, tensors, p).float()


def _errors(got, ref):
    ref = ref.to(torch.float64)
    return (got.to(torch.float64) - ref).abs().amax(dim=-1) / ref.abs().amax(dim=-1)


def _fits(got, ref, dtype, name) -> bool:
    """Whether a run agrees with the plain implementation: every position in 32-bit, most in bfloat16."""
    if dtype == "float32":
        return float(_errors(got, ref).max()) < TOL["float32"]
    q, tol = BF16_MOST[name]
    return float(torch.quantile(_errors(got, ref), q)) < tol


def _same(got, other, name) -> bool:
    """Whether two bfloat16 runs of the same tokens agree."""
    q, tol = BF16_SAME[name]
    return float(torch.quantile(_errors(got, other), q)) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_tail_and_batches(models, name, dtype):
    path, cfg, tensors = models[name]
    engine = _engine(path, dtype)
    prompts = _prompts(name, cfg)
    refs = [_ref(cfg, tensors, p) for p in prompts]
    whole = [helpers.run_whole(engine, p) for p in prompts]
    for i, p in enumerate(prompts):
        assert _fits(whole[i], refs[i], dtype, name), f"whole, length {len(p)}"
    for i, p in enumerate(prompts):
        # the last 100 tokens one by one: the states, the convolution's kept rows, the previous token's input and the
        # keys all come from the cache, and every window of these models passes over decoded tokens
        tail = helpers.run_tail_by_one(engine, p, 100)
        assert _fits(tail, refs[i], dtype, name), f"tail, length {len(p)}"
        assert dtype == "float32" or _same(tail, whole[i], name), f"tail against whole, length {len(p)}"
    # batches of unequal requests, twice, so that slots, pages and states are used again; the second time in another order
    for order in (list(range(len(prompts))), list(reversed(range(len(prompts))))):
        batch = [prompts[i] for i in order]
        n_prefill = [max(1, len(p) - 9 - 3 * j) for j, p in enumerate(batch)]
        got = helpers.run_batch(engine, batch, n_prefill)
        for j, i in enumerate(order):
            assert _fits(got[j], refs[i], dtype, name), f"batch, request of length {len(prompts[i])}"
            assert dtype == "float32" or _same(got[j], whole[i], name), f"batch against alone, length {len(prompts[i])}"
    engine.cache.check()
    assert not engine.cache.lengths


@pytest.mark.parametrize("name", ["A", "B"])
def test_batched_logits_equal_those_of_each_request_alone(models, name):
    """32-bit: what else is in the batch changes nothing beyond rounding."""
    path, cfg, tensors = models[name]
    engine = _engine(path, "float32")
    prompts = _prompts(name, cfg)
    alone = [helpers.run_tail_by_one(engine, p, 12) for p in prompts]
    got = helpers.run_batch(engine, prompts, [max(1, len(p) - 12) for p in prompts])
    for a, g, p in zip(alone, got, prompts):
        assert helpers.per_position(g, a) < 2e-5, f"length {len(p)}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("piece", [2, 7, 64])
def test_prompts_cut_into_portions(models, piece, dtype):
    """The engine cuts a long step into pieces itself; the states, the convolution's kept rows, the previous token's
    input and the windows' keys pass from piece to piece (a piece of two tokens is shorter than every window and
    than two of the convolutions)."""
    path, cfg, tensors = models["A"]
    engine = _engine(path, dtype, max_step_tokens=piece)
    prompts = _prompts("A", cfg)[2:5]
    refs = [_ref(cfg, tensors, p) for p in prompts]
    uncut = _engine(path, dtype)
    for p, ref in zip(prompts, refs):
        got = helpers.run_whole(engine, p)
        assert _fits(got, ref, dtype, "A"), f"pieces of {piece}, length {len(p)}"
        assert dtype == "float32" or _same(got, helpers.run_whole(uncut, p), "A"), f"pieces of {piece} against the whole, length {len(p)}"
    # three unequal requests in one step that is cut across them
    got = helpers.run_batch(engine, prompts, [len(p) for p in prompts])
    for g, ref in zip(got, refs):
        assert _fits(g, ref, dtype, "A")
    engine.cache.check()


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_portions_given_by_the_caller(models, name):
    """Steps of several tokens on top of a cache: portions of 2, 5, 64 and 3 tokens, then the rest."""
    from rocml_amd.engine import StepEntry
    path, cfg, tensors = models[name]
    engine = _engine(path, "float32")
    p = _prompts(name, cfg)[-1]
    ref = _ref(cfg, tensors, p)
    slot = engine.new_sequence()
    out, at = [], 0
    for n in [2, 5, 64, 3, len(p)]:
        part = p[at:at + n]
        if not part:
            break
        out.append(engine.step([StepEntry(slot, part, list(range(len(part))))]).cpu())
        at += len(part)
    engine.release(slot)
    assert helpers.per_position(torch.cat(out), ref) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_portions_on_top_of_a_cache_with_unequal_starts(models, dtype):
    """Prompt steps of several hundred tokens on top of cached positions, and two sequences with different first
    positions in one step; the windows of 64, 65 and 130 are passed many times over."""
    from rocml_amd.engine import StepEntry
    path, cfg, tensors = models["B"]
    engine = _engine(path, dtype)
    a, b = helpers.random_tokens(760, cfg["vocab"], 61), helpers.random_tokens(300, cfg["vocab"], 62)
    ref_a, ref_b = _ref(cfg, tensors, a), _ref(cfg, tensors, b)
    sa, sb = engine.new_sequence(), engine.new_sequence()
    out_a = [engine.step([StepEntry(sa, a[:90], list(range(90)))]).cpu()]
    out_a.append(engine.step([StepEntry(sa, a[90:390], list(range(300)))]).cpu())
    both = engine.step([StepEntry(sa, a[390:], list(range(370))), StepEntry(sb, b[:280], list(range(280)))]).cpu()
    out_a.append(both[:370])
    out_b = [both[370:], engine.step([StepEntry(sb, b[280:], list(range(20)))]).cpu()]
    engine.release(sa)
    engine.release(sb)
    assert _fits(torch.cat(out_a), ref_a, dtype, "B")
    assert _fits(torch.cat(out_b), ref_b, dtype, "B")
    if dtype == "bfloat16":
        assert _same(torch.cat(out_a), helpers.run_whole(engine, a), "B")
        assert _same(torch.cat(out_b), helpers.run_whole(engine, b), "B")
    engine.cache.check()


def test_slots_pages_and_states_are_used_again(models):
    """One slot and few pages for many requests in turn: a request must find the states of its slot at zero,
    whatever the request before it left there, and the windows give their pages back as they move on."""
    path, cfg, tensors = models["A"]
    engine = _engine(path, "float32", max_tokens=5 * 64, max_seqs=1, max_step_tokens=64)
    prompts = [helpers.random_tokens(n, cfg["vocab"], 500 + i) for i, n in enumerate([300, 130, 2, 65, 200, 1])]
    for round_ in range(2):
        for p in prompts:
            ref = _ref(cfg, tensors, p)
            assert helpers.per_position(helpers.run_tail_by_one(engine, p, 40), ref) < TOL["float32"], f"length {len(p)}"
            engine.cache.check()
    assert all(g.n_free_pages == g.n_pages for g in engine.cache.kv_groups)


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(models, name):
    from rocml_amd.api import Model
    path, cfg, tensors = models[name]
    model = Model.load(path, dtype="float32", ctx=256, max_batch=3)
    lengths = [5, 1, 30, 2, 70, 9, 24]
    prompts = [helpers.random_tokens(n, cfg["vocab"], 700 + i) for i, n in enumerate(lengths)]
    want = [plain.greedy(cfg, tensors, p, 10) for p in prompts]
    got = model.generate(prompts, max_new_tokens=10)          # seven requests in three slots
    assert [r.tokens for r in got] == want
    assert model.last_stats.batches == 3
    model.engine.cache.check()
    assert not model.engine.cache.lengths
    # in bfloat16 the same entry point runs: every token it draws is the largest logit of the same model's whole-prompt
    # step over the prompt and the tokens drawn before it (or all but ties with it)
    model16 = Model.load(path, dtype="bfloat16", ctx=256, max_batch=3)
    got16 = model16.generate(prompts, max_new_tokens=10)
    check = _engine(path, "bfloat16")
    for r, p in zip(got16, prompts):
        assert len(r.tokens) == 10
        logits = helpers.run_whole(check, list(p) + list(r.tokens[:-1]))[len(p) - 1:]
        for k, tok in enumerate(r.tokens):
            row = logits[k]
            assert float(row.max() - row[tok]) <= 0.05 * float(row.abs().max()), f"token {k} of the request of length {len(p)}"


def test_long_decoding(models):
    """300 tokens decoded one by one after a prompt of three: every state is carried 300 times, every window is
    passed, and the decode steps run from a recorded graph."""
    path, cfg, tensors = models["B"]
    p = helpers.random_tokens(303, cfg["vocab"], 900)
    ref = _ref(cfg, tensors, p)
    for dtype in ("float32", "bfloat16"):
        engine = _engine(path, dtype)
        assert engine.use_graphs
        assert _fits(helpers.run_tail_by_one(engine, p, 300), ref, dtype, "B")


def test_replay_program(models, tmp_path):
    path, cfg, tensors = models["A"]
    vocab = cfg["vocab"]
    prompts = {"a": helpers.random_tokens(90, vocab, 41), "b": helpers.random_tokens(7, vocab, 42)}
    refs = {k: _ref(cfg, tensors, p) for k, p in prompts.items()}
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompts["a"][:80], "want": [0, 79]},
                                     {"id": "b", "tokens": prompts["b"][:5], "want": [4]}], "end": []}]
    expect = [[("a", 0), ("a", 79), ("b", 4)]]
    for k in range(10):
        entries = [{"id": "a", "tokens": [prompts["a"][80 + k]], "want": [0]}]
        rows = [("a", 80 + k)]
        if k < 2:
            entries.append({"id": "b", "tokens": [prompts["b"][5 + k]], "want": [0]})
            rows.append(("b", 5 + k))
        steps.append({"step": k + 1, "entries": entries, "end": (["b"] if k == 1 else []) + (["a"] if k == 9 else [])})
        expect.append(rows)
    for dtype in ("float32", "bfloat16"):
        out_dir = str(tmp_path / dtype)
        cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", dtype,
               "--out", out_dir, "--max-tokens", "128"]
        proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
        got, want = [], []
        for step, rows in zip(steps, expect):
            got.append(torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step['step']}.f32"), dtype="<f4").reshape(-1, vocab)))
            want.append(torch.stack([refs[r][i] for r, i in rows]))
            assert got[-1].shape == want[-1].shape, f"step {step['step']} in {dtype}"
        assert _fits(torch.cat(got), torch.cat(want), dtype, "A"), dtype


def test_command_line_runs_the_design(models, capsys):
    from rocml_amd.cli import main
    path, cfg, tensors = models["D"]
    prompt = helpers.random_tokens(9, cfg["vocab"], 77)
    rc = main(["generate", "--model", path, "--dtype", "float32", "--prompt-ids", " ".join(map(str, prompt)),
               "-n", "6", "--ctx", "128", "--batch", "2"])
    out = capsys.readouterr().out.strip().splitlines()
    assert rc == 0 and [int(t) for t in out[-1].split()] == plain.greedy(cfg, tensors, prompt, 6)
    # a catalog name: random weights, no file
    assert main(["generate", "--model", "roravik-tiny", "--prompt-ids", "1 2 3", "-n", "4", "--ctx", "64", "--batch", "1"]) == 0
    assert len(capsys.readouterr().out.strip().splitlines()[-1].split()) == 4
    assert main(["models"]) == 0 and "roravik-tiny" in capsys.readouterr().out


def test_prompt_steps_of_one_shape_are_replayed(models):
    """The second prompt step of a shape is recorded as a graph and later ones replayed: four different prompts of
    one length, each against the plain implementation, with decode steps between them."""
    path, cfg, tensors = models["B"]
    engine = _engine(path, "bfloat16")
    assert engine.model.prompt_graph_safe and engine.use_graphs
    for k in range(4):
        p = helpers.random_tokens(153, cfg["vocab"], 1000 + k)
        ref = _ref(cfg, tensors, p)
        got = helpers.run_tail_by_one(engine, p, 3)
        assert _fits(got, ref, "bfloat16", "B"), f"prompt {k}"
        assert _same(got, helpers.run_whole(_engine(path, "bfloat16", use_graphs=False), p), "B"), f"prompt {k} against a run without graphs"
    assert any(key[0] == "prompt" and entry[1] is not None for key, entry in engine._graphs.items()), "a prompt shape was recorded"
