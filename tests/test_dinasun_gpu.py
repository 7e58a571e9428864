"""Dinasun models through the engine against the plain implementation (``plain_dinasun``):
whole prompts, prompts with their last tokens one by one, portions down to two tokens, mixed
batches in pools so small that pages and state slots are used again, long decoding through
recorded steps, and greedy generation through the engine's own entry point and scheduler.
Seven configurations that differ in every size and constant (``dinasun_tiny``)."""
import io
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_dinasun as P
import traces
from dinasun_tiny import CONFIGS, make_model
from plain_llama import load_folder
from tiny import logit_error, prompt_ids

pytestmark = pytest.mark.gpu

# fraction of the mean logit range: (max, mean)
# (bfloat16: the matrix-core attention rounds its probabilities to 8 bits for the value product, and a
# looped span passes every rounding on several times)
TOL = {"float32": (2e-5, 2e-6), "bfloat16": (5e-2, 6e-3)}
# prompt lengths (the rest of every request is given "decoded" tokens) and how many of those
WORKLOAD = {
    "D1": ([1, 4, 23, 64, 150], 30),        # 64: ends on a page of 64 and 16; the temperature steps every 5 positions
    "D2": ([2, 9, 31, 100], 26),
    "D3": ([3, 63, 129, 200], 40),          # the temperature's step of 64 is a page of 64: 63 and 129 end beside it
    "D4": ([2, 65, 99, 330], 80),           # position 99 is the first with the higher temperature: as the last of a prompt, and decoded
    "D5": ([1, 30, 90], 50),
    "D6": ([1, 2, 17, 40], 12),
    "D7": ([2, 33, 70], 20),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for which in WORKLOAD:
        d = make_model(which, str(tmp_path_factory.mktemp("dinasun" + which)))
        cfg, w = load_folder(d)
        lens, extra = WORKLOAD[which]
        reqs = {f"r{i}": prompt_ids(n + extra, cfg["vocab"], 900 + i) for i, n in enumerate(lens)}
        plens = {f"r{i}": n for i, n in enumerate(lens)}
        want = {rid: P.forward(cfg, w, toks) for rid, toks in reqs.items()}
        out[which] = (d, cfg, w, reqs, plens, want)
    return out


def poison(runner):
    """Old keys, old state and old shifted rows must never show: they start as NaN."""
    for lc in runner.storage.layers:
        for st in lc.states.values():
            st.fill_(float("nan"))
        if lc.owns and lc.k is not None:
            lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))


def run_replay(model_dir, dtype, steps, tmp_path, page_size, max_requests=4, max_tokens=None, use_graphs=True):
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    mt = max_tokens or traces.max_live_tokens(steps, max(64, page_size))
    runner = ModelRunner.from_folder(model_dir, dtype=dtype, max_tokens=mt, page_size=page_size, max_requests=max_requests,
                                     use_graphs=use_graphs)
    poison(runner)
    out = str(tmp_path / "out")
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    runner.manager.check()
    assert not runner.manager.requests and runner.manager.all_free()
    return out, runner


def check(got, want, dtype, what):
    assert set(got) == set(want)
    for rid in want:
        assert np.isfinite(got[rid]).all(), f"{what} {rid}: a logit is not finite"
        mx, mean = logit_error(got[rid], want[rid])
        assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], f"{what} {rid} ({dtype}): max {mx:.3g} mean {mean:.3g}"


SCHEDULES = ["whole", "tail", "portions", "mixed"]


def steps_for(schedule, reqs, plens, extra):
    if schedule == "whole":
        return traces.whole(reqs)
    if schedule == "tail":
        return traces.tail_one_by_one(reqs, tail=extra)
    if schedule == "portions":
        return traces.portions(reqs)
    return traces.mixed(reqs, plens, max_live=min(3, len(reqs)), seed=5)


@pytest.mark.parametrize("schedule", SCHEDULES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,page_size", [("D1", 16), ("D2", 8), ("D3", 64), ("D4", 64), ("D5", 32), ("D6", 4),
                                              ("D7", 16)])
def test_every_way_of_cutting_gives_the_plain_logits(models, tmp_path, which, page_size, dtype, schedule):
    d, cfg, w, reqs, plens, want = models[which]
    steps = steps_for(schedule, reqs, plens, WORKLOAD[which][1])
    out, runner = run_replay(d, dtype, steps, tmp_path, page_size, max_requests=3)
    check(traces.collect(steps, out, cfg["vocab"]), want, dtype, f"{which} {schedule}")
    if schedule == "tail":
        assert runner.graphs.replays > 0, "single tokens went through no recorded step"


def test_mixed_batch_equals_each_request_alone(models, tmp_path):
    """What a request's logits are does not depend on its neighbours in the batch beyond rounding:
    the mixed schedule against the same requests alone, engine against engine, in 32-bit."""
    d, cfg, w, reqs, plens, want = models["D4"]
    alone, _ = run_replay(d, "float32", traces.portions(reqs), tmp_path / "a", 64)
    steps = traces.mixed(reqs, plens, max_live=4, seed=9)
    mixed, _ = run_replay(d, "float32", steps, tmp_path / "m", 64)
    a = traces.collect(traces.portions(reqs), alone, cfg["vocab"])
    m = traces.collect(steps, mixed, cfg["vocab"])
    for rid in reqs:
        mx, _ = logit_error(m[rid], a[rid])
        assert mx <= 1e-5, f"{rid}: {mx:.3g}"      # (the 32-bit products sum in another order from 17 rows on)


def test_slots_and_pages_are_used_again(models, tmp_path):
    """Two state slots and pools for the two longest requests: every request after the first two runs
    in a slot and in pages that another has used, which hold its state, its shifted row and its keys,
    for every pass of the looped span."""
    d, cfg, w, reqs, plens, want = models["D1"]
    steps = traces.mixed(reqs, plens, max_live=2, seed=3)
    out, runner = run_replay(d, "float32", steps, tmp_path, 8, max_requests=2)
    assert runner.manager.slots.size == 2
    check(traces.collect(steps, out, cfg["vocab"]), want, "float32", "reuse")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["D4", "D2"])
def test_long_decoding_through_recorded_steps(models, tmp_path, dtype, which):
    """A short prompt and 300 tokens one by one: several pages of every attention layer and several
    steps of the query temperature pass over decoded tokens, and the state is carried 300 times."""
    d, cfg, w, reqs, plens, want = models[which]
    toks = prompt_ids(310, cfg["vocab"], 77)
    wanted = P.forward(cfg, w, toks)
    steps = traces.tail_one_by_one({"long": toks}, tail=300)
    out, runner = run_replay(d, dtype, steps, tmp_path, 16)
    assert runner.graphs.replays >= 290
    check(traces.collect(steps, out, cfg["vocab"]), {"long": wanted}, dtype, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whole_and_in_portions(models, tmp_path, dtype):
    """1,300 tokens in one step (time mixing then runs its rows as chunks side by side, attention in whole
    tiles), the same in two long portions around a short one, and 20 more one by one behind either."""
    d, cfg, w, *_ = models["D1"]
    toks = prompt_ids(1320, cfg["vocab"], 78)
    wanted = {"long": P.forward(cfg, w, toks)}
    whole = traces.tail_one_by_one({"long": toks}, tail=20)
    out, _ = run_replay(d, dtype, whole, tmp_path / "w", 64)
    check(traces.collect(whole, out, cfg["vocab"]), wanted, dtype, "long prompt")
    cut = traces.portions({"long": toks}, sizes=(1100, 2, 198, 1, 1, 18))
    out, _ = run_replay(d, dtype, cut, tmp_path / "c", 16)
    check(traces.collect(cut, out, cfg["vocab"]), wanted, dtype, "long prompt in portions")


def test_eager_and_recorded_steps_agree(models, tmp_path):
    d, cfg, w, reqs, plens, want = models["D1"]
    steps = traces.tail_one_by_one(reqs, tail=30)
    a, _ = run_replay(d, "float32", steps, tmp_path / "g", 8, use_graphs=True)
    b, _ = run_replay(d, "float32", steps, tmp_path / "e", 8, use_graphs=False)
    ga, gb = traces.collect(steps, a, cfg["vocab"]), traces.collect(steps, b, cfg["vocab"])
    for rid in reqs:
        assert np.array_equal(ga[rid], gb[rid]), rid


def test_every_pass_of_the_span_has_a_cache_of_its_own(models):
    """Three passes over (wkv, attention): six entries behind the first layer, each with pages or a
    state slot of its own, and the residual stream after every entry is the plain one."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, w, reqs, plens, want = models["D1"]
    toks = reqs["r2"]
    plain_layers = []
    P.forward(cfg, w, toks, layers_out=plain_layers)
    r = ModelRunner.from_folder(d, dtype="float32", max_tokens=128, page_size=16, max_requests=2, use_graphs=False)
    assert len(r.storage.layers) == 8 and all(lc.owns for lc in r.storage.layers)
    taps = []
    r.model.tap = lambda i, x: taps.append(x.detach().float().cpu().numpy().copy())
    cut = 11            # a portion, then the rest: the taps of both steps side by side are the whole sequence's
    r.step([StepEntry("a", toks[:cut], [])])
    r.step([StepEntry("a", toks[cut:], [])])
    r.finish("a")
    assert len(taps) == 16
    for i in range(8):
        got = np.concatenate([taps[i], taps[8 + i]], axis=0)
        assert np.abs(got - plain_layers[i]).max() <= 2e-5 * max(1.0, np.abs(plain_layers[i]).max()), f"entry {i}"


def greedy(cfg, w, prompt, n_new):
    toks, out = list(prompt), []
    for _ in range(n_new):
        t = int(np.argmax(P.forward(cfg, w, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out


@pytest.mark.parametrize("which", ["D1", "D2", "D5"])
def test_greedy_generation_through_the_entry_point(models, which):
    """``LLM.generate``: scheduler, portions under a token budget, sampling on the device."""
    from xyntetik_runner_amd import LLM, SamplingParams
    d, cfg, w, reqs, plens, want = models[which]
    prompts = [prompt_ids(n, cfg["vocab"], 500 + n) for n in (3, 21, 40)]
    wanted = [greedy(cfg, w, p, 8) for p in prompts]
    llm = LLM(d, dtype="float32", max_tokens=512, page_size=16, max_batched_tokens=16, max_running=2)
    got = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=8))
    assert got == wanted
    assert llm.runner.manager.all_free()


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_command_line(models):
    d, cfg, w, *_ = models["D3"]
    prompt = prompt_ids(9, cfg["vocab"], 21)
    wanted = greedy(cfg, w, prompt, 5)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "runner"), "-m", d, "--ids", ",".join(map(str, prompt)), "-n", "5",
           "--temp", "0", "--dtype", "float32", "-c", "128", "-b", "4"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr
    assert p.stdout.strip() == ",".join(map(str, prompt + wanted))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, tmp_path, dtype):
    """bin/trace_run as a user runs it: a child process, steps on stdin, 'done <step>' lines back,
    four state slots and pools for the tokens that are live."""
    d, cfg, w, reqs, plens, want = models["D3"]
    steps = traces.mixed(reqs, plens, max_live=4, seed=2)
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                          "--out", out, "--max-tokens", str(traces.max_live_tokens(steps, 64))],
                         stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        assert p.stdout.readline().strip() == f"done {st['step']}"
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    check(traces.collect(steps, out, cfg["vocab"]), want, dtype, "trace_run")
