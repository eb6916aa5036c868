"""The engine at the layer sizes of TinyLlama 1.1B (hidden 2048, 32 heads over 4 kv heads of 64,
intermediate 5632, vocabulary 32000; 2 of its 22 layers) with seeded random weights made on the
device, against the plain implementation run on the same weights made on the host: the four
cuttings in 32-bit and bfloat16, and generation with graphs across the 512-token context bound."""
import pytest
import torch

import plain_llama as plain
import traces
from test_replay_gpu import check, r64, replay
from util import random_tokens, rel_err

pytestmark = pytest.mark.gpu

SHAPE = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 2048,
    "num_attention_heads": 32, "num_key_value_heads": 4, "intermediate_size": 5632, "vocab_size": 32000,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 2048, "tie_word_embeddings": False,
    "hidden_act": "silu", "attention_bias": False, "rope_scaling": None, "initializer_range": 0.02, "eos_token_id": 2,
}
LAYERS_FULL = 22
SEED, STD = 5, 0.02
SHARPEN = 2.0       # q and k projections times this: attention far from uniform, so a misplaced key shows
TOL = {"float32": 1e-4, "bfloat16": 2e-2}
LENGTHS = [330, 137, 540, 64]

_made = {}


def host_weights(round_to=None):
    """The weights `Engine(config=SHAPE, weights_seed=SEED)` makes on the device, made on the host."""
    key = str(round_to)
    if key not in _made:
        from tiny_llm_amd.config import resolve
        from tiny_llm_amd.models.decoder import Decoder
        from tiny_llm_amd.weights.loader import random_tensor
        _, spec = resolve(SHAPE)
        w = {}
        for s in Decoder(spec, "float32", "cpu").weight_specs():
            t = random_tensor(s, SEED, STD, 0.0)
            if s.name.endswith(("q_proj.weight", "k_proj.weight")):
                t = t * SHARPEN
            if round_to is not None and t.dim() >= 2:
                t = t.to(round_to)
            w[s.name] = t.double()
        _made[key] = w
    return _made[key]


def requests():
    return {f"r{i}": random_tokens(n, SHAPE["vocab_size"], 31 * i + 7) for i, n in enumerate(LENGTHS)}


def references(dtype):
    key = ("ref", dtype)
    if key not in _made:
        act = torch.bfloat16 if dtype == "bfloat16" else None
        w = host_weights(act)
        _made[key] = {rid: plain.llama_forward(w, SHAPE, toks, act_dtype=act) for rid, toks in requests().items()}
    return _made[key]


def sharpen(decoder):
    for layer in decoder.layers:
        m = layer.mixer
        m.w_qkv[: m.q_size + m.kv_size] *= SHARPEN       # a power of two: exact in both element types


def make_runner(dtype, max_tokens):
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, random_model
    engine = EngineConfig(dtype=dtype, kv_block_size=16, max_cache_tokens=max_tokens, max_num_seqs=8,
                          max_num_batched_tokens=4096, use_graphs=False)
    _, dec = random_model(SHAPE, engine, seed=SEED, std=STD)
    sharpen(dec)
    runner = build_runner(dec, engine)
    for g in runner.cache.groups:
        for t in g.tensors.values():
            t.fill_(float("nan"))
    return runner


def test_device_made_weights_equal_host_made_weights():
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import random_model
    _, dec = random_model(SHAPE, EngineConfig(dtype="float32"), seed=SEED, std=STD)
    w = host_weights()
    m = dec.layers[1].mixer
    q = w["model.layers.1.self_attn.q_proj.weight"] / SHARPEN
    assert torch.equal(m.w_qkv[: m.q_size].cpu().double(), q)
    assert torch.equal(dec.lm_head.weight.cpu().double(), w["lm_head.weight"])
    assert torch.equal(dec.layers[0].by_role["ffn"].w_down.cpu().double(), w["model.layers.0.mlp.down_proj.weight"])
    assert torch.equal(dec.final_norm.weight.cpu().double(), w["model.norm.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_cuttings_at_the_real_layer_sizes(dtype):
    reqs, ref = requests(), references(dtype)
    biggest = max(r64(len(t)) for t in reqs.values())
    mixed, peak = traces.mixed(reqs, seed=4)
    assert peak < sum(r64(len(t)) for t in reqs.values())        # pages are used again
    runner = make_runner(dtype, max(biggest, peak))
    for name, steps in (("whole", traces.whole(reqs)), ("tail", traces.tail_one_by_one(reqs)),
                        ("portions", traces.portions(reqs, sizes=(7, 2, 190, 3, 2, 33, 64, 2, 300, 1, 129))),
                        ("mixed", mixed)):
        out = replay(runner, steps)
        worst = check(out, steps, ref, TOL[dtype])
        print(f"TinyLlama layer sizes (2 of {LAYERS_FULL} layers) {dtype} {name}: worst rel err {worst:.2e}", flush=True)
        assert runner.cache.free_blocks() == [g.pool.num_blocks for g in runner.cache.groups]


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_across_the_512_bound_at_the_real_layer_sizes(dtype, graphs):
    """What the throughput measurement runs: prompts of about 500 tokens, decode steps as graphs,
    the graph of the next bound on the context taking over once the context passes 512."""
    from tiny_llm_amd import Engine, SamplingParams
    from test_engine_gpu import check_logged_logits, poison, spy_on_steps
    act = torch.bfloat16 if dtype == "bfloat16" else None
    w = host_weights(act)
    prompts = [random_tokens(n, SHAPE["vocab_size"], 900 + n) for n in (500, 481, 507, 470)]
    eng = Engine(config=SHAPE, dtype=dtype, weights_seed=SEED, init_std=STD, kv_block_size=16, max_num_seqs=4,
                 max_num_batched_tokens=1024, max_cache_tokens=4 * 576, use_graphs=graphs, decode_burst=1)
    sharpen(eng.decoder)
    poison(eng)
    log = spy_on_steps(eng)
    out = eng.generate(prompts, SamplingParams.greedy(24, ignore_eos=True))
    tokens_of = {i: p + o for i, (p, o) in enumerate(zip(prompts, out))}
    worst, n = check_logged_logits(log, tokens_of, w, SHAPE, act, TOL[dtype])
    print(f"TinyLlama layer sizes {dtype} graphs={graphs}: {n} rows across 512, worst rel err {worst:.2e}", flush=True)
    assert n == 4 * 24
    if graphs:
        assert sorted({k[2] for k, g in eng.runner._graphs.items() if k[0] == "decode" and g.graph is not None}) == [512, 1024]


@pytest.mark.parametrize("n_requests", [20, 40])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_many_requests_at_the_real_layer_sizes(dtype, n_requests):
    """Decode steps of 20 and 40 rows as graphs: the products take other kernels there than up to 16
    rows (two row tiles; from 33 rows a split inner size with a second kernel, also for the output
    head, which gets every row without a gather) and the attention other workgroups.  Every step's
    logits of every request against the plain implementation."""
    from tiny_llm_amd import Engine, SamplingParams
    from test_engine_gpu import check_logged_logits, poison, spy_on_steps
    act = torch.bfloat16 if dtype == "bfloat16" else None
    w = host_weights(act)
    prompts = [random_tokens(9 + (7 * i) % 23, SHAPE["vocab_size"], 400 + i) for i in range(n_requests)]
    new = 6
    eng = Engine(config=SHAPE, dtype=dtype, weights_seed=SEED, init_std=STD, kv_block_size=16, max_num_seqs=n_requests,
                 max_num_batched_tokens=1024, max_cache_tokens=n_requests * 64, use_graphs=True, decode_burst=1)
    sharpen(eng.decoder)
    poison(eng)
    log = spy_on_steps(eng)
    out = eng.generate(prompts, SamplingParams.greedy(new, ignore_eos=True))
    tokens_of = {i: p + o for i, (p, o) in enumerate(zip(prompts, out))}
    worst, n = check_logged_logits(log, tokens_of, w, SHAPE, act, TOL[dtype])
    print(f"TinyLlama layer sizes {dtype}, {n_requests} requests: {n} rows, worst rel err {worst:.2e}", flush=True)
    assert n == n_requests * new
    decode_graphs = [k for k, g in eng.runner._graphs.items() if k[0] == "decode" and g.graph is not None]
    assert any(k[1] == n_requests for k in decode_graphs)
    # the same requests with runs of steps chained on the device: the same kernels, so the same tokens
    del eng
    chained = Engine(config=SHAPE, dtype=dtype, weights_seed=SEED, init_std=STD, kv_block_size=16,
                     max_num_seqs=n_requests, max_num_batched_tokens=1024, max_cache_tokens=n_requests * 64,
                     use_graphs=True)
    sharpen(chained.decoder)
    assert chained.generate(prompts, SamplingParams.greedy(new, ignore_eos=True)) == out


# ------------------------------------------------- the larger shapes the measurements run
# Two layers at the layer sizes of Llama-3-8B and Llama-2-13B: the products and the attention take
# other kernels there than at TinyLlama's sizes (inner sizes beyond 4096, heads of 128 with four and
# with one query head per kv head, a vocabulary of 128256).  The weights are made on the device by
# name (the same bits as on the host, see above) and copied to the host for the plain model.
LARGE = {
    "llama3_8b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 4096,
        "num_attention_heads": 32, "num_key_value_heads": 8, "intermediate_size": 14336, "vocab_size": 128256,
        "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192, "tie_word_embeddings": False,
        "hidden_act": "silu", "attention_bias": False, "rope_scaling": None, "initializer_range": 0.02},
    "llama2_13b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 5120,
        "num_attention_heads": 40, "num_key_value_heads": 40, "intermediate_size": 13824, "vocab_size": 32000,
        "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 4096, "tie_word_embeddings": False,
        "hidden_act": "silu", "attention_bias": False, "rope_scaling": None, "initializer_range": 0.02},
}
_large = {}


def large_weights(name):
    """float32 weights by checkpoint name, on the host (q and k sharpened); made once per shape."""
    if _large.get("name") != name:
        from tiny_llm_amd.config import resolve
        from tiny_llm_amd.models.decoder import Decoder
        from tiny_llm_amd.weights.loader import random_tensor
        _large.clear()
        _, spec = resolve(LARGE[name])
        w = {}
        for s in Decoder(spec, "float32", "cpu").weight_specs():
            t = random_tensor(s, SEED, STD, 0.0, device="cuda:0").cpu()
            if s.name.endswith(("q_proj.weight", "k_proj.weight")):
                t = t * SHARPEN
            w[s.name] = t
        _large.update(name=name, weights=w)
    return _large["weights"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["llama3_8b", "llama2_13b"])
def test_the_larger_layer_sizes(name, dtype):
    """A prompt of 520 tokens whole and in portions of 512 + 8, forty short requests whose prompts
    run as one step, then decode steps of 40, 16 and 1 rows (eagerly, captured and replayed): every
    wanted row against the plain implementation."""
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, random_model
    from tiny_llm_amd.engine.step import StepEntry
    cfg = LARGE[name]
    V = cfg["vocab_size"]
    act = torch.bfloat16 if dtype == "bfloat16" else None
    w = large_weights(name)
    if act is not None:
        w = {k: (t.to(act).float() if t.dim() >= 2 else t) for k, t in w.items()}
    long = random_tokens(520, V, 77)
    n_short, n_decode = 40, 9
    prompt_len = [6 + (5 * i) % 11 for i in range(n_short)]
    short = [random_tokens(prompt_len[i] + n_decode, V, 500 + i) for i in range(n_short)]
    long_rows = [0, 1, 63, 64, 255, 511, 512, 513, 514, 515, 516, 517, 518, 519]
    # one pass of the plain model over all requests: the weights stream once
    segments = [520] + [len(s) for s in short]
    starts = [sum(segments[:i]) for i in range(len(segments))]
    wanted = [(0, p) for p in long_rows] + [(1 + i, p) for i in range(n_short) for p in range(prompt_len[i] - 1, len(short[i]))]
    ref_rows = plain.llama_forward(w, cfg, long + [t for s in short for t in s], act_dtype=act, segments=segments,
                                   rows=[starts[s] + p for s, p in wanted])
    ref = {sp: ref_rows[i] for i, sp in enumerate(wanted)}
    del ref_rows, w

    engine = EngineConfig(dtype=dtype, kv_block_size=16, max_cache_tokens=n_short * 64 + 576, max_num_seqs=n_short + 1,
                          max_num_batched_tokens=1024, use_graphs=True)
    _, dec = random_model(cfg, engine, seed=SEED, std=STD)
    sharpen(dec)
    runner = build_runner(dec, engine)
    for g in runner.cache.groups:
        for t in g.tensors.values():
            t.fill_(float("nan"))
    worst = 0.0

    def compare(got, where, what):
        nonlocal worst
        got = got.cpu()
        assert got.shape[0] == len(where)
        for i, sp in enumerate(where):
            assert torch.isfinite(got[i]).all(), (what, sp)
            e = rel_err(got[i], ref[sp])
            worst = max(worst, e)
            assert e < TOL[dtype], f"{name} {dtype} {what}: request {sp[0]} position {sp[1]}: rel err {e:.3e}"

    compare(runner.step([StepEntry("long", long, long_rows)]), [(0, p) for p in long_rows], "whole")
    runner.finish("long")
    for graph in (False, True, True):
        compare(runner.step([StepEntry("long", long[:512], [0, 1, 63, 64, 255, 511])], use_graph=graph),
                [(0, p) for p in (0, 1, 63, 64, 255, 511)], "portion of 512")
        compare(runner.step([StepEntry("long", long[512:], list(range(8)))], use_graph=graph),
                [(0, p) for p in range(512, 520)], "the last 8 tokens")
        runner.finish("long")
    compare(runner.step([StepEntry(i, short[i][:prompt_len[i]], [prompt_len[i] - 1]) for i in range(n_short)], use_graph=True),
            [(1 + i, prompt_len[i] - 1) for i in range(n_short)], "forty prompts")
    at = 0
    for live in (40, 16, 1):
        for i in range(live, n_short):
            runner.finish(i)
        for _ in range(3):          # eagerly on the static buffers, captured, replayed
            ents = [StepEntry(i, [short[i][prompt_len[i] + at]], [0]) for i in range(live)]
            compare(runner.step(ents, use_graph=True), [(1 + i, prompt_len[i] + at) for i in range(live)],
                    f"decode step of {live} rows")
            at += 1
    assert at == n_decode
    assert sorted(k[1] for k, g in runner._graphs.items() if k[0] == "decode" and g.graph is not None) == [1, 16, 40]
    print(f"{name} layer sizes (2 layers) {dtype}: worst rel err {worst:.2e}", flush=True)
    runner.cache.audit()
