"""Contexts of several thousand tokens through the engine, against the plain implementation:
what the measurements run at 4,224 and 8,192 tokens and the short tests never reach.  A whole
prompt of more rows than the step workspace is first made for; the same prompt in portions of
512 as captured steps (the prefill attention shares a portion's keys out over workgroups);
decoding across the 4,096 bound beside a short request (the decode attention splits a request's
keys 8 and 16 ways; the float32 attention merges up to 32 chunks).  That these paths were
taken is read off the calls the run itself made."""
import pytest
import torch

import plain_llama as plain
from util import TINY_A, TINY_C, make_folder, random_tokens, read_weights, rel_err

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 2e-2}
CONFIGS = {
    "A": (dict(TINY_A, max_position_embeddings=8192), 16, {"std": 0.02, "norm_std": 0.0}),
    "C": (dict(TINY_C, max_position_embeddings=8192), 32, {"std": 0.03, "norm_std": 0.05}),
}
LONG, NEAR_BOUND, SHORT, DECODED, MID = 5000, 4072, 50, 40, 1030
_made = {}


def material(name, dtype, tmp_path_factory):
    key = (name, dtype)
    if key not in _made:
        cfg, _, init = CONFIGS[name]
        if ("folder", name) not in _made:
            _made[("folder", name)] = make_folder(tmp_path_factory.mktemp(f"long_{name}"), cfg, seed=17, **init)
        folder = _made[("folder", name)]
        act = torch.bfloat16 if dtype == "bfloat16" else None
        w, c = read_weights(folder, round_to=act)
        V = cfg["vocab_size"]
        reqs = {"long": random_tokens(LONG, V, 1), "near": random_tokens(NEAR_BOUND + DECODED, V, 2),
                "short": random_tokens(SHORT + DECODED, V, 3), "mid": random_tokens(MID + 6, V, 4)}
        ref = {r: plain.llama_forward(w, c, t, act_dtype=act) for r, t in reqs.items()}
        _made[key] = (folder, reqs, ref)
    return _made[key]


class Calls:
    """Records how the attention kernels were called during a run."""

    def __init__(self, monkeypatch):
        from tiny_llm_amd.kernels import ops
        self.decode_splits, self.prefill_splits, self.f32_chunks, self.rows = [], [], [], []
        flash, prefill, f32 = ops.flash_attention, ops.flash_prefill, ops.attention_f32

        def spy_flash(*a, **k):
            self.decode_splits.append(k.get("n_splits", a[12] if len(a) > 12 else 1))
            return flash(*a, **k)

        def spy_prefill(*a, **k):
            self.prefill_splits.append(k.get("n_splits", a[13] if len(a) > 13 else 1))
            self.rows.append(a[0].shape[0])
            return prefill(*a, **k)

        def spy_f32(*a, **k):
            self.f32_chunks.append(k.get("n_chunks", a[12] if len(a) > 12 else 1))
            self.rows.append(a[0].shape[0])
            return f32(*a, **k)
        monkeypatch.setattr(ops, "flash_attention", spy_flash)
        monkeypatch.setattr(ops, "flash_prefill", spy_prefill)
        monkeypatch.setattr(ops, "attention_f32", spy_f32)


def make_runner(folder, dtype, block_size, budget):
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, load_model
    engine = EngineConfig(dtype=dtype, kv_block_size=block_size, max_cache_tokens=LONG + 64 + 4224 + 128, max_num_seqs=4,
                          max_num_batched_tokens=budget, use_graphs=True)
    _, dec = load_model(folder, engine)
    runner = build_runner(dec, engine)
    for g in runner.cache.groups:
        for t in g.tensors.values():
            t.fill_(float("nan"))
    return runner


def compare(got, ref, positions, tol, what):
    got = got.cpu()
    assert got.shape[0] == len(positions)
    worst = 0.0
    for i, p in enumerate(positions):
        assert torch.isfinite(got[i]).all(), (what, p)
        e = rel_err(got[i], ref[p])
        worst = max(worst, e)
        assert e < tol, f"{what}: position {p}: rel err {e:.3e}"
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_contexts_of_thousands_of_tokens(name, dtype, tmp_path_factory, monkeypatch):
    from tiny_llm_amd.engine.step import StepEntry
    from tiny_llm_amd.kernels import ops
    folder, reqs, ref = material(name, dtype, tmp_path_factory)
    _, block_size, _ = CONFIGS[name]
    tol = TOL[dtype]
    calls = Calls(monkeypatch)
    runner = make_runner(folder, dtype, block_size, budget=LONG)
    assert runner.workspace.max_rows == ops.Workspace.FIRST_ROWS < LONG
    # 1. a whole prompt of more rows than the workspace was first made for (by a small step)
    runner.step([StepEntry("first", reqs["short"][:SHORT], [])])
    runner.finish("first")
    some = sorted(set(list(range(0, LONG, 61)) + list(range(LONG - 40, LONG)) + [4095, 4096, 4097]))
    long = reqs["long"]
    w1 = compare(runner.step([StepEntry("long", long, some)]), ref["long"], some, tol, "whole prompt")
    assert max(calls.rows) == LONG and runner.workspace._retired      # its buffers were made again, larger
    runner.finish("long")
    # 2. the same prompt in portions of 512 as captured steps: twice, so that portions replay graphs
    w2 = 0.0
    for again in range(2):
        for at in range(0, LONG, 512):
            n = min(512, LONG - at)
            want = sorted({0, 1, n // 2, n - 2, n - 1})
            got = runner.step([StepEntry("long", long[at:at + n], want)], use_graph=True)
            w2 = max(w2, compare(got, ref["long"], [at + p for p in want], tol, f"portion at {at}"))
        runner.finish("long")
    bounds = sorted({k[4] for k, g in runner._graphs.items() if k[0] == "mixed" and g.graph is not None})
    assert bounds and bounds[-1] == 8192 and 4096 in bounds and 2048 in bounds
    if dtype == "bfloat16":
        assert max(calls.prefill_splits) == 4           # late portions: few query rows over many keys
    # 3. decoding across the 4,096 bound beside a short request, as captured steps
    near, short = reqs["near"], reqs["short"]
    for at in range(0, NEAR_BOUND, 512):
        runner.step([StepEntry("near", near[at:min(at + 512, NEAR_BOUND)], [])], use_graph=True)
    runner.step([StepEntry("short", short[:SHORT], [])], use_graph=True)
    calls.decode_splits.clear(), calls.f32_chunks.clear()
    w3 = 0.0
    mid = reqs["mid"]
    runner.step([StepEntry("mid", mid[:MID], [])], use_graph=True)
    for k in range(6):          # a context between 1,024 and 2,048: half as many splits
        got = runner.step([StepEntry("mid", [mid[MID + k]], [0])], use_graph=True)
        w3 = max(w3, compare(got, ref["mid"], [MID + k], tol, f"decoding at {MID + k}"))
    runner.finish("mid")
    for k in range(DECODED):
        got = runner.step([StepEntry("near", [near[NEAR_BOUND + k]], [0]), StepEntry("short", [short[SHORT + k]], [0])],
                          use_graph=True).cpu()
        w3 = max(w3, compare(got[:1], ref["near"], [NEAR_BOUND + k], tol, f"decoding at {NEAR_BOUND + k}"))
        w3 = max(w3, compare(got[1:], ref["short"], [SHORT + k], tol, f"the short request at {SHORT + k}"))
    assert runner.cache.num_tokens("near") == NEAR_BOUND + DECODED > 4096
    decode_bounds = sorted(k[2] for k, g in runner._graphs.items() if k[0] == "decode" and g.graph is not None)
    assert decode_bounds == [2048, 4096, 8192]
    if dtype == "bfloat16":
        assert {8, 16} <= set(calls.decode_splits)
    else:
        assert {8, 16, 32} <= set(calls.f32_chunks)
    print(f"{name} {dtype}: whole {w1:.2e}, portions of 512 {w2:.2e}, decoding across 4096 {w3:.2e}", flush=True)
    runner.cache.audit()
