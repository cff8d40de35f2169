"""Sugosun models through the engine against the plain implementation (``plain_sugosun``):
whole prompts, prompts with their last tokens one by one, portions down to two tokens, mixed
batches in pools so small that pages and state slots are used again, long decoding through
recorded steps, and greedy generation through the engine's own entry point and scheduler.
Six configurations that differ in every size and constant (``sugosun_tiny``)."""
import io
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_sugosun as G
import traces
from plain_llama import load_folder
from sugosun_tiny import CONFIGS, make_model
from tiny import logit_error, prompt_ids

pytestmark = pytest.mark.gpu

# fraction of the mean logit range: (max, mean)
# (bfloat16: the matrix-core attention rounds its probabilities to 8 bits for the value product, the
# queries pass two products between their projection and the scores, and a looped span passes every
# rounding on several times; the largest of some 100,000 logits strays further than their mean)
TOL = {"float32": (2e-5, 2e-6), "bfloat16": (5e-2, 6e-3)}
# In bfloat16 a token whose last chosen expert and the next one score within rounding of each other may
# take the other one: that token's row then differs by what the two experts differ (times the smallest of
# its weights), which no tolerance on rounding covers.  So a few rows may lie over the bound on the
# largest difference (8 in 100, or one), none far over it; the mean bound holds for every request.
BF16_ROWS_OVER, BF16_FAR = 0.08, 0.5
# prompt lengths (the rest of every request is given "decoded" tokens) and how many of those
WORKLOAD = {
    "G1": ([1, 4, 23, 64, 150], 30),        # 64: ends on a page of 64 and 16; the window of 21 passes over decoded tokens
    "G2": ([2, 9, 31, 100], 26),
    "G3": ([3, 63, 129, 200], 40),          # the window of 64 is a page of 64
    "G4": ([2, 65, 140, 330], 80),          # windows of 70 and 130 pass over pages of 64 in prompts and decoded tokens
    "G5": ([1, 30, 90], 50),
    "G6": ([1, 2, 17, 40], 12),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for which in WORKLOAD:
        d = make_model(which, str(tmp_path_factory.mktemp("sugosun" + which)))
        cfg, w = load_folder(d)
        lens, extra = WORKLOAD[which]
        reqs = {f"r{i}": prompt_ids(n + extra, cfg["vocab"], 700 + i) for i, n in enumerate(lens)}
        plens = {f"r{i}": n for i, n in enumerate(lens)}
        want = {rid: G.forward(cfg, w, toks) for rid, toks in reqs.items()}
        out[which] = (d, cfg, w, reqs, plens, want)
    return out


def poison(runner):
    """Old latents, old state and old last tokens must never show: floats start as NaN, tokens as a wrong id."""
    for lc in runner.storage.layers:
        for st in lc.states.values():
            st.fill_(float("nan"))
        if lc.owns and lc.k is not None:
            lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
    for st in runner.storage.model_states.values():
        st.fill_(12345)


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
        if dtype == "bfloat16" and mx > TOL[dtype][0]:
            rng = float(np.mean(want[rid].max(axis=-1) - want[rid].min(axis=-1)))
            rows = np.abs(got[rid] - want[rid]).max(axis=-1) / rng
            over = int((rows > TOL[dtype][0]).sum())
            assert over <= max(1, BF16_ROWS_OVER * len(rows)) and mx <= BF16_FAR and mean <= TOL[dtype][1], \
                f"{what} {rid} ({dtype}): {over} of {len(rows)} rows over, max {mx:.3g} mean {mean:.3g}"
            continue
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
@pytest.mark.parametrize("which,page_size", [("G1", 16), ("G2", 8), ("G3", 64), ("G4", 64), ("G5", 32), ("G6", 4)])
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
    d, cfg, w, reqs, plens, want = models["G4"]
    alone, _ = run_replay(d, "float32", traces.portions(reqs), tmp_path / "a", 64)
    steps = traces.mixed(reqs, plens, max_live=4, seed=9)
    mixed, _ = run_replay(d, "float32", steps, tmp_path / "m", 64)
    a = traces.collect(traces.portions(reqs), alone, cfg["vocab"])
    m = traces.collect(steps, mixed, cfg["vocab"])
    for rid in reqs:
        mx, _ = logit_error(m[rid], a[rid])
        assert mx <= 1e-5, f"{rid}: {mx:.3g}"      # (the 32-bit products sum in another order from 17 rows on)


def test_slots_and_pages_are_used_again(models, tmp_path):
    """Two state slots and pools for the two longest requests: every request after the first two
    runs in a slot and in pages that another has used, which hold its state, latents and last token."""
    d, cfg, w, reqs, plens, want = models["G1"]
    steps = traces.mixed(reqs, plens, max_live=2, seed=3)
    out, runner = run_replay(d, "float32", steps, tmp_path, 8, max_requests=2)
    assert runner.manager.slots.size == 2
    check(traces.collect(steps, out, cfg["vocab"]), want, "float32", "reuse")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(models, tmp_path, dtype):
    """A short prompt and 300 tokens one by one: both windows and several pages of every attention
    layer pass over decoded tokens, and the recurrent state is carried 300 times."""
    d, cfg, w, reqs, plens, want = models["G4"]
    toks = prompt_ids(310, cfg["vocab"], 77)
    wanted = G.forward(cfg, w, toks)
    steps = traces.tail_one_by_one({"long": toks}, tail=300)
    out, runner = run_replay(d, dtype, steps, tmp_path, 16)
    assert runner.graphs.replays >= 290
    check(traces.collect(steps, out, cfg["vocab"]), {"long": wanted}, dtype, "long decoding")


def test_eager_and_recorded_steps_agree(models, tmp_path):
    d, cfg, w, reqs, plens, want = models["G1"]
    steps = traces.tail_one_by_one(reqs, tail=30)
    a, _ = run_replay(d, "float32", steps, tmp_path / "g", 8, use_graphs=True)
    b, _ = run_replay(d, "float32", steps, tmp_path / "e", 8, use_graphs=False)
    ga, gb = traces.collect(steps, a, cfg["vocab"]), traces.collect(steps, b, cfg["vocab"])
    for rid in reqs:
        assert np.array_equal(ga[rid], gb[rid]), rid


def greedy(cfg, w, prompt, n_new):
    toks, out = list(prompt), []
    for _ in range(n_new):
        t = int(np.argmax(G.forward(cfg, w, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out


@pytest.mark.parametrize("which", ["G1", "G2"])
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
    d, cfg, w, *_ = models["G3"]
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
    d, cfg, w, reqs, plens, want = models["G3"]
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


def test_model_is_built_from_its_config(models):
    from xyntetik_runner_amd.config import load_config
    from xyntetik_runner_amd.engine.model import Model
    d, cfg, w, *_ = models["G1"]
    arch, c = load_config(d)
    assert arch.name == "Sugosun"
    spec = arch.build_spec(c)
    exp = Model.expected_tensors(spec)
    assert sorted(exp) == sorted(w)                                 # (the random-weights mode writes optional tensors too)
    assert sorted(n for n, ps in exp.items() if ps.optional) == ["l2.hc2.in", "l2.hc2.mix", "l2.hc2.out", "l2.norm2"]
    assert [st.layer for st in spec.order] == [0, 1, 2, 1, 2, 1, 2, 3]      # every pass an entry with a cache of its own
    model = Model(spec)
    kv, st, of = model.cache_needs()
    assert of == [None] * 8
    assert kv[0].num_kv_heads == 1 and kv[0].head_dim == 64 and kv[0].window == 21 and kv[1] is None
    assert st[0] is None and st[1] is not None and st[3] is not None
    assert set(model.model_states()) == {"embedding"}
    # without streams and a pair table: the plain arrangement, and no state outside the layers
    arch2, c2 = load_config(models["G2"][0])
    spec2 = arch2.build_spec(c2)
    assert spec2.streams is None and {ls.block for ls in spec2.layers} == {"prenorm_optional"}
    assert Model(spec2).model_states() == {}
