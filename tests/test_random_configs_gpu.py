"""Configurations drawn at random (head sizes with and without a matrix-core kernel, any number of
heads and groups, widths and vocabularies that are no power of two, pages of any size), each
replayed in three cuttings in both precisions against the plain model.  The four fixed tiny
configurations cannot hold every combination; this holds a sample of them and a seed names each."""
import random
import tempfile

import pytest
import torch

import plain_llama as plain
import traces
from test_replay_gpu import TOL, check, make_runner, r64, replay
from util import make_folder, random_tokens, read_weights

pytestmark = pytest.mark.gpu

HEAD_SIZES = [16, 32, 48, 64, 80, 96, 112, 128, 24, 40, 72, 144, 160, 256]
PAGE_SIZES = [1, 2, 4, 8, 16, 32, 64, 3, 5, 12]


def random_config(rng: random.Random) -> dict:
    hd = rng.choice(HEAD_SIZES)
    kv = rng.choice([1, 1, 2, 2, 3, 4, 5, 8])
    group = rng.choice([1, 1, 2, 3, 4, 4, 5, 6, 8, 12, 16, 17, 20])
    if kv * group * hd > 4096:
        group = max(1, 2048 // (kv * hd))
    return {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "num_hidden_layers": rng.randint(1, 3), "hidden_size": rng.choice([8, 16, 24]) * rng.randint(2, 40),
        "num_attention_heads": kv * group, "num_key_value_heads": kv, "head_dim": hd,
        "intermediate_size": 8 * rng.randint(3, 90), "vocab_size": rng.randint(17, 3000),
        "rope_theta": rng.choice([10000.0, 500000.0, 1e6, 777.0]), "rms_norm_eps": rng.choice([1e-5, 1e-6, 3e-4]),
        "max_position_embeddings": 512, "tie_word_embeddings": rng.random() < 0.4, "hidden_act": "silu",
        "attention_bias": False, "rope_scaling": None, "initializer_range": 0.03, "eos_token_id": 2,
        "torch_dtype": "float32",
    }


def test_the_sample_covers_what_it_is_for():
    """The seeds below reach every head size (those with a matrix-core kernel and those without),
    more than sixteen query heads a kv head, and pages that do not divide 64."""
    seen_hd, seen_pages, wide_group = set(), set(), False
    for seed in SEEDS:
        rng = random.Random(seed)
        cfg = random_config(rng)
        seen_hd.add(cfg["head_dim"])
        seen_pages.add(rng.choice(PAGE_SIZES))
        wide_group |= cfg["num_attention_heads"] // cfg["num_key_value_heads"] > 16
    assert seen_hd == set(HEAD_SIZES) and {3, 5, 12} <= seen_pages and wide_group


def _pick_seeds(count):
    """The first seeds that add a head size not seen before, then the next ones up to `count`."""
    chosen, seen = [], set()
    for seed in range(400):
        hd = random_config(random.Random(seed))["head_dim"]
        if hd not in seen:
            seen.add(hd)
            chosen.append(seed)
    for seed in range(400):
        if len(chosen) >= count:
            break
        if seed not in chosen:
            chosen.append(seed)
    return sorted(chosen)


SEEDS = sorted(set(_pick_seeds(28)) | {41, 44, 65})      # the three: heads of 112, decoded tokens


@pytest.mark.parametrize("seed", SEEDS)
def test_random_configuration(seed):
    rng = random.Random(seed)
    cfg = random_config(rng)
    page = rng.choice(PAGE_SIZES)
    lens = [rng.randint(1, 260) for _ in range(5)]
    print(f"seed {seed}: {cfg['num_hidden_layers']} layers, hidden {cfg['hidden_size']}, "
          f"{cfg['num_attention_heads']}/{cfg['num_key_value_heads']} heads of {cfg['head_dim']}, "
          f"intermediate {cfg['intermediate_size']}, vocabulary {cfg['vocab_size']}, page {page}, lengths {lens}", flush=True)
    with tempfile.TemporaryDirectory() as tmp:
        folder = make_folder(tmp, cfg, seed=seed, std=0.03, norm_std=0.1, sharpen=2.0)
        reqs = {f"r{i}": random_tokens(n, cfg["vocab_size"], 100 * i + seed) for i, n in enumerate(lens)}
        for dtype in ("float32", "bfloat16"):
            rounded = torch.bfloat16 if dtype == "bfloat16" else None
            w, c = read_weights(folder, round_to=rounded)
            ref = {rid: plain.llama_forward(w, c, toks, act_dtype=rounded) for rid, toks in reqs.items()}
            biggest = max(r64(len(t)) for t in reqs.values())
            mixed_steps, peak = traces.mixed(reqs, seed=seed)
            for steps, tokens in ((mixed_steps, peak), (traces.portions(reqs), biggest),
                                  (traces.tail_one_by_one(reqs), biggest)):
                if 64 % page:
                    tokens += 8 * page          # a request's last page may reach beyond its multiple of 64
                runner = make_runner(folder, dtype, page, tokens)
                check(replay(runner, steps), steps, ref, TOL[dtype])
                assert runner.cache.free_blocks() == [g.pool.num_blocks for g in runner.cache.groups]


@pytest.mark.parametrize("seed", range(24))
def test_random_schedule(seed):
    """Generation through the entry point with everything about the schedule drawn at random (how
    many requests and how long, pages so few that requests are preempted, token budgets from 4 to
    2,048, one to sixteen live requests, captured steps or not, runs of chained decode steps or
    not): every token is the plain model's choice or within rounding of it, every page comes back."""
    from tiny_llm_amd import Engine, SamplingParams
    rng = random.Random(9000 + seed)
    cfg = random_config(rng)
    cfg["num_hidden_layers"] = rng.randint(1, 2)
    page = rng.choice(PAGE_SIZES)
    n = rng.randint(1, 12)
    lens = [rng.randint(1, 120) for _ in range(n)]
    news = [rng.randint(1, 70) for _ in range(n)]
    budget = rng.choice([4, 8, 16, 33, 64, 256, 2048])
    seqs = rng.choice([1, 2, 3, 4, 8, 16])
    biggest = max(-(-(l + m) // page) for l, m in zip(lens, news))
    total = sum(-(-(l + m) // page) for l, m in zip(lens, news))
    blocks = rng.randint(biggest, max(biggest, total))
    graphs = rng.random() < 0.7
    burst = rng.choice([1, 4, 32])
    dtype = rng.choice(["float32", "float32", "bfloat16"])
    print(f"seed {seed}: hidden {cfg['hidden_size']}, {cfg['num_attention_heads']}/{cfg['num_key_value_heads']} heads of "
          f"{cfg['head_dim']}, page {page}, {blocks} of {total} blocks, budget {budget}, {seqs} live, graphs {graphs}, "
          f"burst {burst}, {dtype}, (prompt, new) {list(zip(lens, news))}", flush=True)
    with tempfile.TemporaryDirectory() as tmp:
        folder = make_folder(tmp, cfg, seed=seed, std=0.03, norm_std=0.1, sharpen=2.0)
        prompts = [random_tokens(n_tok, cfg["vocab_size"], 100 * i + seed) for i, n_tok in enumerate(lens)]
        eng = Engine(folder, dtype=dtype, kv_block_size=page, num_kv_blocks=blocks, max_num_seqs=seqs,
                     max_num_batched_tokens=budget, use_graphs=graphs, decode_burst=burst)
        for g in eng.runner.cache.groups:
            for t in g.tensors.values():
                t.fill_(float("nan"))
        out = eng.generate(prompts, [SamplingParams.greedy(m, ignore_eos=True) for m in news])
        eng.runner.cache.audit()
        assert eng.runner.cache.free_blocks() == [g.pool.num_blocks for g in eng.runner.cache.groups]
        rounded = torch.bfloat16 if dtype == "bfloat16" else None
        w, c = read_weights(folder, round_to=rounded)
        tol = 2 * TOL[dtype]
        for i, (p, o) in enumerate(zip(prompts, out)):
            assert len(o) == news[i], i
            ref = plain.llama_forward(w, c, p + o, act_dtype=rounded)
            for k, tok in enumerate(o):
                row = ref[len(p) + k - 1]
                assert float(row.max() - row[tok]) <= tol * float(row.abs().max()), (i, k)


@pytest.mark.parametrize("seed", range(16))
def test_random_windowed_architecture(seed):
    """A toy architecture registered here: two to four attention layers, each with a window drawn at
    random (0: every key) and so with cache groups and pools of their own, either rotary pairing.
    Generation under a random schedule (as `test_random_schedule`) against the same model run over
    each finished request whole, in one eager step with a pool that is never short."""
    from tiny_llm_amd import Engine, SamplingParams
    from tiny_llm_amd.config import (EngineConfig, ModelSpec, PartSpec, PlanEntry, pre_norm_layer, register_architecture,
                                     unregister_architecture)
    from tiny_llm_amd.engine.loading import build_runner, random_model
    from tiny_llm_amd.engine.step import StepEntry
    rng = random.Random(seed)
    hd = rng.choice([16, 32, 48, 64, 40, 128])
    kv, group = rng.choice([1, 2, 3]), rng.choice([1, 2, 4])
    hidden = 8 * rng.randint(4, 40)
    windows = [rng.choice([0, 1, 2, 5, 16, 20, 33, 64, 100]) for _ in range(rng.randint(2, 4))]
    pairing = rng.choice(["half", "half", "interleaved"])
    vocab = rng.randint(50, 900)
    inter = 8 * rng.randint(4, 40)

    def build(cfg):
        norm = PartSpec("rmsnorm", {"hidden_size": hidden, "eps": 1e-5})
        ffn = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter})
        rope = {"kind": "rotary", "head_dim": hd, "theta": 1000.0, "max_position": 1024, "pairing": pairing}
        layers = tuple(pre_norm_layer(f"model.layers.{i}", norm, PartSpec("attention", {
            "hidden_size": hidden, "num_heads": kv * group, "num_kv_heads": kv, "head_dim": hd, "window": w,
            "position": rope}), norm, ffn) for i, w in enumerate(windows))
        sizes = {"vocab_size": vocab, "hidden_size": hidden}
        return ModelSpec("ToyWindowsForCausalLM", vocab, hidden, 1024, PartSpec("token_embedding", sizes, "model.embed_tokens"),
                         layers, tuple(PlanEntry(i) for i in range(len(windows))), norm.named("model.norm"),
                         PartSpec("lm_head", dict(sizes, tied_to="model.embed_tokens"), "lm_head"))

    register_architecture("ToyWindowsForCausalLM", dict, build)
    try:
        raw = {"architectures": ["ToyWindowsForCausalLM"], "hidden_size": hidden, "vocab_size": vocab}
        page = rng.choice([1, 2, 4, 8, 16, 32, 3, 12])
        n = rng.randint(1, 8)
        lens = [rng.randint(1, 150) for _ in range(n)]
        news = [rng.randint(1, 80) for _ in range(n)]
        budget = rng.choice([4, 8, 16, 33, 64, 256, 2048])
        seqs = rng.choice([1, 2, 3, 4, 8])
        graphs = rng.random() < 0.7
        burst = rng.choice([1, 4, 32])
        dtype = rng.choice(["float32", "float32", "bfloat16"])
        biggest = r64(max(l + m for l, m in zip(lens, news))) + 64
        total = sum(r64(l + m) for l, m in zip(lens, news))
        cache_tokens = rng.randint(biggest, max(total, biggest) + 64)
        print(f"seed {seed}: hidden {hidden}, {kv * group}/{kv} heads of {hd}, windows {windows}, {pairing}, page {page}, "
              f"{cache_tokens} cache tokens, budget {budget}, {seqs} live, graphs {graphs}, burst {burst}, {dtype}, "
              f"(prompt, new) {list(zip(lens, news))}", flush=True)
        eng = Engine(config=raw, dtype=dtype, weights_seed=seed, init_std=0.2, kv_block_size=page, max_num_seqs=seqs,
                     max_num_batched_tokens=budget, max_cache_tokens=cache_tokens, use_graphs=graphs, decode_burst=burst)
        cm = eng.runner.cache
        assert len(cm.groups) == len(set(windows))
        for g in cm.groups:
            for t in g.tensors.values():
                t.fill_(float("nan"))
        prompts = [random_tokens(n_tok, vocab, 100 * i + seed) for i, n_tok in enumerate(lens)]
        out = eng.generate(prompts, [SamplingParams.greedy(m, ignore_eos=True) for m in news])
        cm.audit()
        assert cm.free_blocks() == cm.group_blocks
        whole = EngineConfig(dtype=dtype, kv_block_size=16, max_cache_tokens=biggest, max_num_seqs=2,
                             max_num_batched_tokens=4096, use_graphs=False)
        _, dec = random_model(raw, whole, seed=seed, std=0.2)
        runner = build_runner(dec, whole)
        tol = 2 * TOL[dtype]
        for i, (p, o) in enumerate(zip(prompts, out)):
            assert len(o) == news[i], i
            toks = p + o
            ref = runner.step([StepEntry("w", toks, list(range(len(p) - 1, len(toks) - 1)))]).float().cpu()
            runner.finish("w")
            for k, tok in enumerate(o):
                assert float(ref[k].max() - ref[k][tok]) <= tol * float(ref[k].abs().max()), (i, k)
    finally:
        unregister_architecture("ToyWindowsForCausalLM")


@pytest.mark.parametrize("seed", range(12))
def test_random_seeded_sampling_is_the_same_under_any_schedule(seed):
    """float32, requests with sampling settings and seeds drawn at random (some greedy, some ended
    by an end-of-sequence token): each request alone in whole-prompt steps, then the batch under two
    random schedules (the second in another order of arrival) give the same tokens, token for token:
    a row's logits have the same bits whatever surrounds it, and the random numbers follow the
    request's seed and position, not the step."""
    from tiny_llm_amd import Engine, SamplingParams
    rng = random.Random(31000 + seed)
    cfg = random_config(rng)
    cfg["num_hidden_layers"] = rng.randint(1, 2)
    n = rng.randint(1, 10)
    lens = [rng.randint(1, 100) for _ in range(n)]
    news = [rng.randint(1, 60) for _ in range(n)]
    sps = []
    for i in range(n):
        if rng.random() < 0.25:
            sps.append(SamplingParams.greedy(news[i], ignore_eos=True))
        else:
            sps.append(SamplingParams(max_new_tokens=news[i], temperature=rng.choice([0.3, 0.7, 1.0, 1.5]),
                                      top_k=rng.choice([0, 1, 5, 50]), top_p=rng.choice([0.5, 0.9, 0.95, 1.0]),
                                      seed=rng.getrandbits(40), ignore_eos=rng.random() < 0.7))
    with tempfile.TemporaryDirectory() as tmp:
        folder = make_folder(tmp, cfg, seed=seed, std=0.03, norm_std=0.1, sharpen=2.0)
        prompts = [random_tokens(n_tok, cfg["vocab_size"], 100 * i + seed) for i, n_tok in enumerate(lens)]
        outs = []
        for variant in range(3):
            page = rng.choice(PAGE_SIZES)
            budget = rng.choice([4, 8, 16, 33, 64, 256, 2048])
            seqs = rng.choice([1, 2, 3, 4, 8, 16])
            biggest = max(-(-(l + m) // page) for l, m in zip(lens, news))
            total = sum(-(-(l + m) // page) for l, m in zip(lens, news))
            blocks = rng.randint(biggest, max(biggest, total))
            graphs = rng.random() < 0.7
            burst = rng.choice([1, 4, 32])
            if variant == 0:        # each request alone, whole prompts, eagerly
                page, budget, seqs, graphs, burst = 16, 4096, 1, False, 1
                blocks = -(-max(l + m for l, m in zip(lens, news)) // 16) + 1
            print(f"seed {seed} variant {variant}: page {page}, budget {budget}, {seqs} live, {blocks} of {total} blocks, "
                  f"graphs {graphs}, burst {burst}", flush=True)
            eng = Engine(folder, dtype="float32", kv_block_size=page, num_kv_blocks=blocks, max_num_seqs=seqs,
                         max_num_batched_tokens=budget, use_graphs=graphs, decode_burst=burst)
            order = list(range(n))
            if variant == 2:
                rng.shuffle(order)
            got = eng.generate([prompts[i] for i in order], [sps[i] for i in order])
            back = [None] * n
            for j, i in enumerate(order):
                back[i] = got[j]
            outs.append(back)
            eng.runner.cache.audit()
        assert outs[1] == outs[0] and outs[2] == outs[0]
