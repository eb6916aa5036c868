"""The engine against the plain implementation, in every way of cutting the work:
whole, tail one by one, changing portions, mixed with page reuse; both tiny
configurations; 32-bit and bfloat16; through the step function in-process and
through bin/trace_run as a separate program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as plain
import traces
from util import CONFIGS, make_folder, random_tokens, read_weights, rel_err

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# 32-bit: the target is 1e-4 of the row scale; bfloat16: the plain model rounds activations where
# the serving path stores bfloat16, so what is left is the order of float32 sums flipping roundings.
TOL = {"float32": 1e-4, "bfloat16": 2e-2}

LENGTHS = {"A": [70, 133, 33, 200, 97, 64], "B": [1, 9, 40, 100, 150, 57], "C": [40, 130, 75, 200, 64, 9],
           "D": [24, 121, 48, 190, 5, 73]}


def requests_for(name, cfg):
    return {f"r{i}": random_tokens(n, cfg["vocab_size"], 100 * i + len(name)) for i, n in enumerate(LENGTHS[name])}


_cache = {}


def material(name, dtype, tmp_path_factory):
    """Model folder, plain logits of every request, built once per (configuration, dtype)."""
    key = (name, dtype)
    if key not in _cache:
        cfg, eng, init = CONFIGS[name]
        folder = make_folder(tmp_path_factory.mktemp(f"model_{name}_{dtype}"), cfg, seed=7, **init)
        rounded = torch.bfloat16 if dtype == "bfloat16" else None
        w, c = read_weights(folder, round_to=rounded)
        reqs = requests_for(name, cfg)
        ref = {rid: plain.llama_forward(w, c, toks, act_dtype=rounded) for rid, toks in reqs.items()}
        _cache[key] = (folder, reqs, ref, eng)
    return _cache[key]


def make_runner(folder, dtype, block_size, max_tokens, poison=True):
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, load_model
    engine = EngineConfig(dtype=dtype, kv_block_size=block_size, max_cache_tokens=max_tokens, max_num_seqs=8,
                          max_num_batched_tokens=1 << 16, use_graphs=False)
    _, dec = load_model(folder, engine)
    runner = build_runner(dec, engine)
    if poison:                      # stale or unwritten cache contents must never reach a result
        for g in runner.cache.groups:
            for t in g.tensors.values():
                t.fill_(float("nan"))
    return runner


def replay(runner, steps, use_graph=False):
    from tiny_llm_amd.engine.step import StepEntry
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]], use_graph=use_graph)
        if logits.shape[0]:
            out[s["step"]] = logits.cpu()
        for rid in s["end"]:
            runner.finish(rid)
        runner.cache.audit()
    return out


def check(out, steps, ref, tol):
    rows = traces.rows_of(steps)
    assert set(rows) == set(out)
    worst = 0.0
    for step, where in rows.items():
        got = out[step]
        assert got.shape[0] == len(where)
        for i, (rid, pos) in enumerate(where):
            assert torch.isfinite(got[i]).all(), (step, rid, pos)
            e = rel_err(got[i], ref[rid][pos])
            worst = max(worst, e)
            assert e < tol, f"step {step}: request {rid} position {pos}: rel err {e:.3e}"
    return worst


def r64(n):
    return -(-n // 64) * 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_tail_portions(name, dtype, tmp_path_factory):
    folder, reqs, ref, eng = material(name, dtype, tmp_path_factory)
    biggest = max(r64(len(t)) for t in reqs.values())
    for build in (traces.whole, traces.tail_one_by_one, traces.portions):
        steps = build(reqs)
        runner = make_runner(folder, dtype, eng["kv_block_size"], biggest)
        out = replay(runner, steps)
        worst = check(out, steps, ref, TOL[dtype])
        print(f"{name} {dtype} {build.__name__}: worst rel err {worst:.2e}")
        assert runner.cache.free_blocks() == [g.pool.num_blocks for g in runner.cache.groups]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_mixed_with_page_reuse(name, dtype, tmp_path_factory):
    folder, reqs, ref, eng = material(name, dtype, tmp_path_factory)
    for seed in (0, 1):
        steps, peak = traces.mixed(reqs, seed=seed)
        total = sum(r64(len(t)) for t in reqs.values())
        assert peak < total          # the pool is smaller than all requests together: pages are used again
        runner = make_runner(folder, dtype, eng["kv_block_size"], peak)
        out = replay(runner, steps)
        worst = check(out, steps, ref, TOL[dtype])
        print(f"{name} {dtype} mixed seed {seed}: worst rel err {worst:.2e}, pool {peak} tokens")
        assert runner.cache.free_blocks() == [g.pool.num_blocks for g in runner.cache.groups]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_cuttings_as_captured_steps(name, dtype, tmp_path_factory):
    """The same traces with every step run as a HIP graph of its shape (sizes rounded up, padding
    tokens, tiles and rows): twice over on one runner, so that the second pass replays what the
    first captured, with other shapes between the replays."""
    folder, reqs, ref, eng = material(name, dtype, tmp_path_factory)
    steps, peak = traces.mixed(reqs, seed=2)
    runner = make_runner(folder, dtype, eng["kv_block_size"], max(peak, max(r64(len(t)) for t in reqs.values())))
    for build in (lambda: steps, lambda: traces.portions(reqs), lambda: traces.tail_one_by_one(reqs)):
        st = build()
        for again in range(2):
            out = replay(runner, st, use_graph=True)
            worst = check(out, st, ref, TOL[dtype])
            assert runner.cache.free_blocks() == [g.pool.num_blocks for g in runner.cache.groups]
    captured = [k for k, g in runner._graphs.items() if g.graph is not None]
    print(f"{name} {dtype}: {len(runner._graphs)} shapes, {len(captured)} captured, "
          f"{runner.graph_steps} graph steps, {runner.eager_steps} eager, worst {worst:.2e}")
    assert runner.graph_steps > runner.eager_steps
    assert not any(g.capture_failed for g in runner._graphs.values())


def test_first_tokens_and_single_token_request(tmp_path_factory):
    """The first positions of a sequence, alone: a one-key context returns v itself."""
    folder, reqs, ref, eng = material("B", "float32", tmp_path_factory)
    runner = make_runner(folder, "float32", eng["kv_block_size"], 64)
    from tiny_llm_amd.engine.step import StepEntry
    toks = reqs["r3"]
    for n in (1, 2, 3):
        logits = runner.step([StepEntry("x", toks[:n], list(range(n)))]).cpu()
        runner.finish("x")
        for i in range(n):
            assert rel_err(logits[i], ref["r3"][i]) < TOL["float32"]


def test_permuting_requests_permutes_rows(tmp_path_factory):
    folder, reqs, ref, eng = material("A", "float32", tmp_path_factory)
    from tiny_llm_amd.engine.step import StepEntry
    a, b, c = reqs["r0"][:20], reqs["r1"][:31], reqs["r2"][:5]
    runner = make_runner(folder, "float32", 16, 256)
    l1 = runner.step([StepEntry("a", a, [19]), StepEntry("b", b, [30]), StepEntry("c", c, [4])]).cpu()
    for r in "abc":
        runner.finish(r)
    l2 = runner.step([StepEntry("c", c, [4]), StepEntry("a", a, [19]), StepEntry("b", b, [30])]).cpu()
    assert rel_err(l2[0], l1[2]) < 1e-6 and rel_err(l2[1], l1[0]) < 1e-6 and rel_err(l2[2], l1[1]) < 1e-6


def test_long_decoding(tmp_path_factory):
    """Several hundred single-token steps: every page edge of a long request is crossed."""
    cfg, eng, init = CONFIGS["A"]
    folder, _, _, _ = material("A", "float32", tmp_path_factory)
    w, c = read_weights(folder)
    toks = random_tokens(420, cfg["vocab_size"], 4242)
    ref = plain.llama_forward(w, c, toks)
    runner = make_runner(folder, "float32", 16, r64(420))
    from tiny_llm_amd.engine.step import StepEntry
    got = [runner.step([StepEntry("long", toks[:8], list(range(8)))]).cpu()]
    for i in range(8, 420):
        got.append(runner.step([StepEntry("long", [toks[i]], [0])]).cpu())
    got = torch.cat(got)
    worst = max(rel_err(got[i], ref[i]) for i in range(420))
    print(f"long decoding: worst rel err {worst:.2e}")
    assert worst < TOL["float32"]


@pytest.mark.parametrize("dtype,graphs", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
def test_trace_run_program(dtype, graphs, tmp_path_factory, tmp_path):
    """bin/trace_run as a user runs it: JSON steps on stdin, <step>.f32 files, `done <step>` lines;
    with --graphs the shapes of step that come again (the decoded tokens' steps) replay captured graphs."""
    folder, reqs, ref, eng = material("A", dtype, tmp_path_factory)
    steps, peak = traces.mixed(reqs, seed=3)
    out_dir = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(peak)] + (["--graphs", "--npy"] if graphs else []),
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    vocab = CONFIGS["A"][0]["vocab_size"]
    out = {}
    for step, where in traces.rows_of(steps).items():
        arr = np.fromfile(out_dir / f"{step}.f32", dtype="<f4")
        assert arr.size == len(where) * vocab
        out[step] = torch.from_numpy(arr.reshape(len(where), vocab))
        if graphs:
            assert np.array_equal(np.load(out_dir / f"{step}.npy"), arr.reshape(len(where), vocab))
    check(out, steps, ref, TOL[dtype])
