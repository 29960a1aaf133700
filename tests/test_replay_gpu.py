"""The step function on the GPU against the plain implementation, under every way of
cutting the same requests into steps, in 32-bit and in bfloat16."""
import json
import os
import subprocess
from pathlib import Path

import numpy as np
import pytest

import scenarios
import tiny_models

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent

LENGTHS = {"A": [70, 33, 97, 5, 120, 64], "B": [40, 129, 9, 64, 200, 1 + 32], "C": [150, 61, 33, 90, 47, 128],
           "D": [260, 77, 140, 33, 200, 64], "E": [90, 35, 120, 7, 64, 50],
           "F": [8, 3, 7, 8, 5, 2], "G": [150, 40, 97, 300, 18, 64]}
TOL = {"float32": scenarios.FP32_TOL, "bfloat16": scenarios.BF16_TOL}


def _run_in_process(folder, dtype, steps, page_size, max_tokens, max_requests=4, poison=False):
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import load_model, make_runner

    _, model = load_model(folder, dtype)
    runner = make_runner(model, page_size=page_size, num_pages=-(-max_tokens // page_size) + 1, max_requests=max_requests)
    if poison:      # every page but the sentinel (page 0), which nothing ever writes and released entries point to
        for group in runner.cache.groups:
            for plane in group.tensors:
                plane[:, 1:].fill_(float("nan"))                     # [runs, pages, heads, page, head size]
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.cpu().numpy()
        for r in s["end"]:
            runner.release(r)
    runner.cache.check()
    assert runner.cache.live_requests() == []
    if poison:
        for group in runner.cache.groups:
            assert not any(bool(plane[:, 0].any()) for plane in group.tensors), "the sentinel page was written"
    return out


@pytest.fixture(scope="module")
def expected(model_folders):
    cache = {}

    def get(name):
        if name not in cache:
            cfg = json.loads((model_folders[name] / "config.json").read_text())
            reqs = scenarios.make_requests(cfg["vocab_size"], LENGTHS[name], seed=11)
            cache[name] = (reqs, scenarios.expected_logits(model_folders[name], reqs))
        return cache[name]
    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F", "G"])
@pytest.mark.parametrize("mode", ["whole", "tail_singles", "portions", "mixed"])
def test_split(model_folders, expected, name, dtype, mode):
    reqs, exp = expected(name)
    build = getattr(scenarios, mode)
    steps = scenarios.number(build(reqs))
    page = tiny_models.PAGE_SIZES[name]
    # the pool holds exactly what the live requests need, so that freed pages are used again
    out = _run_in_process(model_folders[name], dtype, steps, page, scenarios.max_tokens_needed(steps))
    scenarios.check(steps, out, exp, TOL[dtype], f"{name}/{dtype}/{mode}")


def test_trace_run_program(model_folders, expected, tmp_path):
    """The replay program itself, as a user starts it: a mixed trace, both dtypes."""
    reqs, exp = expected("B")
    steps = scenarios.number(scenarios.mixed(reqs, seed=3))
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / dtype
        proc = subprocess.Popen(
            [str(ROOT / "bin" / "trace_run"), "--model", str(model_folders["B"]), "--dtype", dtype, "--out", str(out_dir),
             "--max-tokens", str(scenarios.max_tokens_needed(steps))],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=dict(os.environ, PYTHONUNBUFFERED="1"))
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", f"expected 'done {s['step']}', got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
        vocab = len(next(iter(exp.values()))[0])
        out = {int(p.stem): np.fromfile(p, dtype="<f4").reshape(-1, vocab) for p in out_dir.glob("*.f32")}
        scenarios.check(steps, out, exp, TOL[dtype], f"trace_run/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_decode_steps_replayed_as_graphs(model_folders, expected, name, dtype):
    """Decode-only steps under captured HIP graphs: every replay is checked against the plain
    implementation, with eager steps (prompt portions, other batch widths) and synchronizations
    between the replays, requests joining and leaving, and pages reused."""
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import load_model, make_runner
    reqs, exp = expected(name)
    steps = scenarios.number(scenarios.mixed(reqs, seed=5, prompt_fraction=0.3))
    page = tiny_models.PAGE_SIZES[name]
    _, model = load_model(model_folders[name], dtype)
    runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps) // page) + 1,
                         max_requests=4, use_graphs=True)
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        out[s["step"]] = logits.cpu().numpy()
        for r in s["end"]:
            runner.release(r)
    assert runner.graph_replays >= 20 and len(runner._graphs) >= 2
    scenarios.check(steps, out, exp, TOL[dtype], f"graphs/{name}/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F", "G"])
def test_pages_that_hold_nan_where_nothing_is_written_yet(model_folders, expected, name, dtype):
    """The pool starts out full of NaN instead of zeros, as if earlier requests had left the worst
    behind: no kernel may let a place that its request has not written reach a result."""
    reqs, exp = expected(name)
    steps = scenarios.number(scenarios.mixed(reqs))
    out = _run_in_process(model_folders[name], dtype, steps, tiny_models.PAGE_SIZES[name], scenarios.max_tokens_needed(steps), poison=True)
    scenarios.check(steps, out, exp, TOL[dtype], f"poisoned pool/{name}/{dtype}")


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["portions", "mixed"])
def test_prompt_portion_attention_kernel_in_the_engine(model_folders, expected, monkeypatch, name, mode):
    """The shared-memory attention kernel for prompt portions is used from 4096-token contexts
    on; here it is switched on for every step so that the tiny models exercise it, together
    with the split of a step's requests between the two attention kernels."""
    from torchlet_amd.parts import attention
    monkeypatch.setattr(attention, "_PORTION_MIN_CONTEXT", 0)
    monkeypatch.setattr(attention, "_PORTION_MIN_TOKENS", 3)
    reqs, exp = expected(name)
    steps = scenarios.number(getattr(scenarios, mode)(reqs))
    out = _run_in_process(model_folders[name], "bfloat16", steps, tiny_models.PAGE_SIZES[name], scenarios.max_tokens_needed(steps))
    scenarios.check(steps, out, exp, TOL["bfloat16"], f"portion kernel/{name}/{mode}")
