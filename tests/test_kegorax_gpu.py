"""Kegorax models through the engine against the plain implementation (``plain_kegorax``):
whole prompts, prompts with their last tokens one by one, portions down to two tokens, mixed
batches in pools so small that pages and state slots are used again, long decoding through
recorded steps, and greedy generation through the engine's own entry point and scheduler.
Seven configurations that differ in every size and constant (``kegorax_tiny``)."""
import io
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_kegorax as P
import traces
from kegorax_tiny import CONFIGS, make_model
from plain_llama import load_folder
from tiny import logit_error, prompt_ids

pytestmark = pytest.mark.gpu

# fraction of the mean logit range: (max, mean)
# (bfloat16: the matrix-core attention rounds its probabilities to 8 bits for the value product, and a
# looped span passes every rounding on several times)
TOL = {"float32": (2e-5, 2e-6), "bfloat16": (5e-2, 6e-3)}
# In bfloat16 a token whose last chosen expert (or last kept group) and the next one score within rounding of each
# other may take the other one: that token's row then differs by what the two experts differ, which no tolerance
# on rounding covers, and the layers behind carry the difference on in their states to every later row of the
# request.  The plain implementation says by how much every choice is decided (``route_margin``): in bfloat16 the
# bounds hold for a request's rows before its first choice that is decided by less than CLOSE_CALL, and among
# those a few rows (8 in 100, or one) may still lie over the bound on the largest difference, none far over it
# (a close call in the last layer changes its own row alone); the rows behind are only asked to be numbers.
# In 32 bits every row of every request is held to the bounds.
BF16_ROWS_OVER, BF16_FAR, CLOSE_CALL = 0.08, 0.5, 0.02
# prompt lengths (the rest of every request is given "decoded" tokens) and how many of those
WORKLOAD = {
    "K1": ([1, 4, 23, 64, 150], 30),        # chunks of 24 and windows of 20 end inside prompts and among decoded tokens
    "K2": ([2, 9, 31, 100], 26),
    "K3": ([3, 63, 129, 200], 40),          # the chunk of 64 is a page of 64: 63 and 129 end beside its edge
    "K4": ([2, 65, 99], 30),
    "K5": ([2, 90, 128, 330], 60),          # the chunk of 130 and the window of 100 pass over pages of 64, in prompts and decoded
    "K6": ([1, 30, 90], 50),
    "K7": ([3, 420], 40),                   # the chunk of 200 and the window of 150 end inside the prompt and among decoded tokens
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for which in WORKLOAD:
        d = make_model(which, str(tmp_path_factory.mktemp("kegorax" + which)))
        cfg, w = load_folder(d)
        lens, extra = WORKLOAD[which]
        reqs = {f"r{i}": prompt_ids(n + extra, cfg["vocab"], 1100 + i) for i, n in enumerate(lens)}
        plens = {f"r{i}": n for i, n in enumerate(lens)}
        want = {}
        for rid, toks in reqs.items():
            calls = []
            want[rid] = P.forward(cfg, w, toks, choices=calls)
            FIRST_CLOSE[(which, rid)] = first_close_call(cfg, calls, len(toks))
        out[which] = (d, cfg, w, reqs, plens, want)
    return out


FIRST_CLOSE = {}        # (configuration, request) -> the first row whose choice of experts a rounding may change


def first_close_call(cfg, calls, n_tokens):
    """``calls``: what ``forward`` recorded of every routed token, layer run by layer run, each over all tokens.
    A close call in the model's last layer run changes its own row only and is left to the bound on single rows."""
    if not calls:
        return n_tokens
    runs = len(calls) // n_tokens
    last_is_final = cfg["layers"][-1].get("mlp") is not None and cfg["layers"][-1]["mlp"]["kind"] == "moe"
    first = n_tokens
    for run in range(runs - 1 if last_is_final else runs):
        for t in range(n_tokens):
            if calls[run * n_tokens + t][2] < CLOSE_CALL:
                first = min(first, t)
                break
    return first


def poison(runner):
    """Old keys and old state must never show: they start as NaN."""
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


def check(got, want, dtype, what, which=None, upto=None):
    """``which``: the configuration whose requests' first close calls bound the rows that are compared in bfloat16
    (``upto``: the same as a mapping request -> row)."""
    assert set(got) == set(want)
    for rid in want:
        assert np.isfinite(got[rid]).all(), f"{what} {rid}: a logit is not finite"
        rng = float(np.mean(want[rid].max(axis=-1) - want[rid].min(axis=-1)))
        n = len(want[rid])
        if dtype == "bfloat16":
            n = upto[rid] if upto is not None else FIRST_CLOSE.get((which, rid), n)
        if n == 0:
            continue
        d = np.abs(np.asarray(got[rid][:n], dtype=np.float64) - want[rid][:n]) / rng
        mx, mean = float(d.max()), float(d.mean())
        if dtype == "bfloat16" and mx > TOL[dtype][0]:
            rows = d.max(axis=-1)
            over = int((rows > TOL[dtype][0]).sum())
            assert over <= max(1, BF16_ROWS_OVER * len(rows)) and mx <= BF16_FAR and mean <= TOL[dtype][1], \
                f"{what} {rid} ({dtype}): {over} of {len(rows)} rows over, max {mx:.3g} mean {mean:.3g}"
            continue
        assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], f"{what} {rid} ({dtype}): max {mx:.3g} mean {mean:.3g} ({n} rows)"


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
@pytest.mark.parametrize("which,page_size", [("K1", 16), ("K2", 8), ("K3", 64), ("K4", 16), ("K5", 64), ("K6", 4),
                                              ("K7", 64)])
def test_every_way_of_cutting_gives_the_plain_logits(models, tmp_path, which, page_size, dtype, schedule):
    d, cfg, w, reqs, plens, want = models[which]
    steps = steps_for(schedule, reqs, plens, WORKLOAD[which][1])
    out, runner = run_replay(d, dtype, steps, tmp_path, page_size, max_requests=3)
    check(traces.collect(steps, out, cfg["vocab"]), want, dtype, f"{which} {schedule}", which)
    if schedule == "tail":
        assert runner.graphs.replays > 0, "single tokens went through no recorded step"


def test_mixed_batch_equals_each_request_alone(models, tmp_path):
    """What a request's logits are does not depend on its neighbours in the batch beyond rounding:
    the mixed schedule against the same requests alone, engine against engine, in 32-bit."""
    d, cfg, w, reqs, plens, want = models["K5"]
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
    in a slot and in pages that another has used, which hold its state, its convolution's inputs and its
    keys, for every pass of the looped span."""
    d, cfg, w, reqs, plens, want = models["K1"]
    steps = traces.mixed(reqs, plens, max_live=2, seed=3)
    out, runner = run_replay(d, "float32", steps, tmp_path, 8, max_requests=2)
    assert runner.manager.slots.size == 2
    check(traces.collect(steps, out, cfg["vocab"]), want, "float32", "reuse")


def test_a_window_gives_pages_back_but_for_the_kept_ones(models, tmp_path):
    """With pages of 4 and a window of 20 that keeps 3 tokens, a request of 180 tokens holds the window's
    pages and the first page of the windowed group, not its 45 pages."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, w, reqs, plens, want = models["K1"]
    r = ModelRunner.from_folder(d, dtype="float32", max_tokens=256, page_size=4, max_requests=2, use_graphs=False)
    toks = reqs["r4"]
    r.step([StepEntry("a", toks[:150], [])])
    gi = [i for i, g in enumerate(r.manager.groups) if g.spec.keep_first == 3][0]
    table = r.manager.get("a").tables[gi]
    assert table[0] >= 0 and all(p < 0 for p in table[1:32]) and all(p >= 0 for p in table[33:38])
    r.manager.check()
    r.finish("a")
    assert r.manager.all_free()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["K6", "K2"])
def test_long_decoding_through_recorded_steps(models, tmp_path, dtype, which):
    """A short prompt and 300 tokens one by one: chunks, windows and pages of every attention layer pass over
    decoded tokens, and the states are carried 300 times."""
    d, cfg, w, reqs, plens, want = models[which]
    toks = prompt_ids(310, cfg["vocab"], 77)
    calls = []
    wanted = P.forward(cfg, w, toks, choices=calls)
    steps = traces.tail_one_by_one({"long": toks}, tail=300)
    out, runner = run_replay(d, dtype, steps, tmp_path, 16)
    assert runner.graphs.replays >= 290
    check(traces.collect(steps, out, cfg["vocab"]), {"long": wanted}, dtype, "long decoding",
          upto={"long": first_close_call(cfg, calls, len(toks))})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whole_and_in_portions(models, tmp_path, dtype):
    """1,300 tokens in one step (gated linear attention and retention then run their rows as chunks side by
    side, attention in whole tiles), the same in two long portions around a short one, and 20 more one by one."""
    d, cfg, w, *_ = models["K5"]
    toks = prompt_ids(1320, cfg["vocab"], 78)
    calls = []
    wanted = {"long": P.forward(cfg, w, toks, choices=calls)}
    upto = {"long": first_close_call(cfg, calls, len(toks))}
    whole = traces.tail_one_by_one({"long": toks}, tail=20)
    out, _ = run_replay(d, dtype, whole, tmp_path / "w", 64)
    check(traces.collect(whole, out, cfg["vocab"]), wanted, dtype, "long prompt", upto=upto)
    cut = traces.portions({"long": toks}, sizes=(1100, 2, 198, 1, 1, 18))
    out, _ = run_replay(d, dtype, cut, tmp_path / "c", 16)
    check(traces.collect(cut, out, cfg["vocab"]), wanted, dtype, "long prompt in portions", upto=upto)


def test_eager_and_recorded_steps_agree(models, tmp_path):
    d, cfg, w, reqs, plens, want = models["K1"]
    steps = traces.tail_one_by_one(reqs, tail=30)
    a, _ = run_replay(d, "float32", steps, tmp_path / "g", 8, use_graphs=True)
    b, _ = run_replay(d, "float32", steps, tmp_path / "e", 8, use_graphs=False)
    ga, gb = traces.collect(steps, a, cfg["vocab"]), traces.collect(steps, b, cfg["vocab"])
    for rid in reqs:
        assert np.array_equal(ga[rid], gb[rid]), rid


def test_every_pass_of_the_span_has_a_cache_of_its_own(models):
    """Three passes over two layers behind the first and before the last: eight entries, each with pages and
    state of its own, and the residual stream after every entry is the plain one."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, w, reqs, plens, want = models["K1"]
    toks = reqs["r2"]
    plain_layers = []
    P.forward(cfg, w, toks, taps=plain_layers)
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


@pytest.mark.parametrize("which", ["K1", "K2", "K6"])
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
    d, cfg, w, *_ = models["K3"]
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
    d, cfg, w, reqs, plens, want = models["K3"]
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
    check(traces.collect(steps, out, cfg["vocab"]), want, dtype, "trace_run", "K3")
