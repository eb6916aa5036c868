"""The engine above the step function: parts alone, generation through the entry points,
seeded sampling, preemption, and a toy architecture with a stateful mixer that is
registered here, in the test, without touching the framework's files."""
import math
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_llama as plain
from util import CONFIGS, TINY_A, TINY_B, make_folder, random_tokens, read_weights, rel_err

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (cfg, eng, init) in CONFIGS.items():
        out[name] = make_folder(tmp_path_factory.mktemp(f"engine_{name}"), cfg, seed=11, **init)
    return out


def fake_ctx(lens, q_lens, block_size, n_groups=1, shuffle_seed=0):
    """A StepContext for requests with lens[r] tokens of which the last q_lens[r] are new."""
    from tiny_llm_amd.engine.step import StepContext
    g = torch.Generator().manual_seed(shuffle_seed)
    nb = sum(-(-l // block_size) for l in lens)
    perm = torch.randperm(nb + 2, generator=g).tolist()
    mb = max(-(-l // block_size) for l in lens)
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    tok_pos, req_of, slots, cu = [], [], [], [0]
    for r, (L, q) in enumerate(zip(lens, q_lens)):
        for b in range(-(-L // block_size)):
            bt[r, b] = perm.pop()
        for p in range(L - q, L):
            tok_pos.append(p)
            req_of.append(r)
            slots.append(int(bt[r, p // block_size]) * block_size + p % block_size)
        cu.append(cu[-1] + q)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    T = len(tok_pos)
    return StepContext(num_tokens=T, num_requests=len(lens), tokens=i32([0] * T), positions=i32(tok_pos),
                       req_of_token=i32(req_of), cu_seqlens_q=i32(cu), seq_lens=i32(lens),
                       state_slots=i32(list(range(len(lens)))), logit_rows=None, block_tables=[bt.to(DEV)],
                       slot_mappings=[i32(slots)], q_lens=list(q_lens),
                       context_lens=[l - q for l, q in zip(lens, q_lens)], slots_host=list(range(len(lens))),
                       max_q_len=max(q_lens), max_seq_len=max(lens), block_size=block_size), nb + 2


# ----------------------------------------------------------------- parts alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_ffn_embedding_head_parts(dtype):
    from tiny_llm_amd.parts import EMBEDDINGS, FEED_FORWARDS, HEADS, NORMS
    TokenEmbedding, LMHead = EMBEDDINGS.get("token_embedding"), HEADS.get("lm_head")
    g = torch.Generator().manual_seed(3)
    H, I, V, T = 80, 136, 123, 19
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    x = torch.randn(T, H, generator=g)
    norm = NORMS.get("rmsnorm")("n", dtype, DEV, hidden_size=H, eps=3e-6)
    w = 1 + 0.2 * torch.randn(H, generator=g)
    norm.bind({"n.weight": w.to(DEV)})
    h = norm.forward(x.to(DEV))
    assert h.dtype == dtype and rel_err(h, plain.rms_norm(x.double(), w.double(), 3e-6)) < tol

    ffn = FEED_FORWARDS.get("swiglu")("f", dtype, DEV, hidden_size=H, intermediate_size=I)
    ws = {n: (torch.randn(s, generator=g) / math.sqrt(s[1])).to(dtype) for n, s in
          (("f.gate_proj.weight", (I, H)), ("f.up_proj.weight", (I, H)), ("f.down_proj.weight", (H, I)))}
    ffn.bind({k: v.to(DEV) for k, v in ws.items()})
    hin = torch.randn(T, H, generator=g).to(dtype)
    res = torch.randn(T, H, generator=g)
    out = ffn.forward(hin.to(DEV), None, res.clone().to(DEV))
    act = None if dtype == torch.float32 else dtype
    ref = res.double() + plain.swiglu(hin.double(), ws["f.gate_proj.weight"].double(), ws["f.up_proj.weight"].double(),
                                      ws["f.down_proj.weight"].double(), act)
    assert out.dtype == torch.float32 and rel_err(out, ref) < tol

    emb = TokenEmbedding("e", dtype, DEV, vocab_size=V, hidden_size=H)
    table = torch.randn(V, H, generator=g).to(dtype)
    emb.bind({"e.weight": table.to(DEV)})
    ids = [5, 0, V - 1, 5]
    assert torch.equal(emb.forward(torch.tensor(ids, dtype=torch.int32, device=DEV)).cpu(), table.float()[ids])
    head = LMHead("lm", dtype, DEV, vocab_size=V, hidden_size=H)
    head.bind({"lm.weight": table.to(DEV)})
    assert rel_err(head.forward(hin.to(DEV)), hin.double() @ table.double().T) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,hd,bs,window", [(6, 2, 48, 16, 0), (4, 4, 16, 8, 0), (5, 1, 80, 32, 0), (4, 2, 32, 8, 9)])
def test_attention_part_alone(dtype, nq, nkv, hd, bs, window):
    """Two steps through the part: a prefix of every request, then the rest (mixed lengths),
    against the plain functions over the whole sequences."""
    from tiny_llm_amd.parts import MIXERS, LayerCache
    g = torch.Generator().manual_seed(hd + bs)
    H = 72
    lens, cut = [37, 9, 64, 1], [30, 8, 17, 0]
    attn = MIXERS.get("attention")("a", dtype, DEV, hidden_size=H, num_heads=nq, num_kv_heads=nkv, head_dim=hd,
                                   window=window, position={"kind": "rotary", "head_dim": hd, "theta": 777.0,
                                                            "max_position": 128})
    ws = {f"a.{n}_proj.weight": (torch.randn(s, generator=g) * f).to(dtype) for n, s, f in
          (("q", (nq * hd, H), 0.3), ("k", (nkv * hd, H), 0.3), ("v", (nkv * hd, H), 0.1), ("o", (H, nq * hd), 0.1))}
    attn.bind({k: v.to(DEV) for k, v in ws.items()})
    hs = [torch.randn(L, H, generator=g).to(dtype) for L in lens]
    act = None if dtype == torch.float32 else dtype
    cos, sin = plain.rope_table(128, hd, 777.0)
    refs = []
    for h in hs:
        L = h.shape[0]
        rnd = (lambda t: t) if act is None else (lambda t: t.to(act).double())
        q = rnd(plain.apply_rope(rnd(plain.linear(h.double(), ws["a.q_proj.weight"].double())).view(L, nq, hd), range(L), cos, sin))
        k = rnd(plain.apply_rope(rnd(plain.linear(h.double(), ws["a.k_proj.weight"].double())).view(L, nkv, hd), range(L), cos, sin))
        v = rnd(plain.linear(h.double(), ws["a.v_proj.weight"].double())).view(L, nkv, hd)
        o = rnd(plain.attention_fast(q, k, v, range(L), window)).reshape(L, nq * hd)
        refs.append(plain.linear(o, ws["a.o_proj.weight"].double()))
    # step 1: prefixes; step 2: the rest.  Same physical blocks in both steps.
    ctx2, nblocks = fake_ctx(lens, [l - c for l, c in zip(lens, cut)], bs)
    kc = torch.full((nblocks, nkv, bs, hd), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((nblocks, nkv, bs, hd), float("nan"), dtype=dtype, device=DEV)
    cache = LayerCache({"k": kc, "v": vc}, 0, True)
    live = [r for r, c in enumerate(cut) if c > 0]
    ctx1, _ = fake_ctx([cut[r] for r in live], [cut[r] for r in live], bs)
    ctx1.block_tables = [ctx2.block_tables[0][live][:, :ctx1.block_tables[0].shape[1]].contiguous()]
    slots = []
    for i, r in enumerate(live):
        slots += [int(ctx1.block_tables[0][i, p // bs]) * bs + p % bs for p in range(cut[r])]
    ctx1.slot_mappings = [torch.tensor(slots, dtype=torch.int32, device=DEV)]
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    h1 = torch.cat([hs[r][:cut[r]] for r in live]).to(DEV)
    out1 = attn.forward(h1, ctx1, cache, None, torch.zeros(h1.shape[0], H, device=DEV))
    assert rel_err(out1, torch.cat([refs[r][:cut[r]] for r in live])) < tol
    h2 = torch.cat([hs[r][cut[r]:] for r in range(len(lens))]).to(DEV)
    res = torch.randn(h2.shape[0], H, generator=g)
    out2 = attn.forward(h2, ctx2, cache, None, res.clone().to(DEV))
    ref2 = res.double() + torch.cat([refs[r][cut[r]:] for r in range(len(lens))])
    assert rel_err(out2, ref2) < tol


# ------------------------------------------------------------------ generation
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(name, folders):
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS[name]
    w, c = read_weights(folders[name])
    prompts = [random_tokens(n, cfg["vocab_size"], 50 + n) for n in ((5, 17, 31) if name == "A" else (1, 9, 40, 100))]
    eng = Engine(folders[name], dtype="float32", max_num_seqs=4, max_num_batched_tokens=8 if name == "B" else 64, **eng_kw)
    out = eng.generate(prompts, SamplingParams.greedy(16 if name == "A" else 6, ignore_eos=True))
    for p, o in zip(prompts, out):
        assert o == plain.greedy_generate(w, c, p, len(o))
    assert eng.runner.cache.free_blocks() == [g.pool.num_blocks for g in eng.runner.cache.groups]
    # eos ends a request and is part of its output
    first = out[0][0]
    eng.scheduler.eos_token_id = first
    assert eng.generate([prompts[0]], SamplingParams.greedy(16))[0] == [first]


def test_bfloat16_generation_follows_the_plain_model(folders):
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    w, c = read_weights(folders["A"], round_to=torch.bfloat16)
    prompts = [random_tokens(n, cfg["vocab_size"], 70 + n) for n in (5, 17, 31)]
    eng = Engine(folders["A"], dtype="bfloat16", max_num_seqs=4, **eng_kw)
    out = eng.generate(prompts, SamplingParams.greedy(16, ignore_eos=True))
    for p, o in zip(prompts, out):
        ref = plain.llama_forward(w, c, p + o, act_dtype=torch.bfloat16)
        for i, tok in enumerate(o):
            row = ref[len(p) + i - 1]
            # the chosen token is the plain model's argmax, or within rounding of it
            assert float(row.max() - row[tok]) <= 2e-2 * float(row.abs().max())


def test_seeded_sampling_does_not_depend_on_batching(folders):
    """Temperature 0.8 with a fixed seed: the same tokens whether the request runs alone, beside
    others, or with its prompt cut into portions of 8."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["B"]
    prompts = [random_tokens(n, cfg["vocab_size"], 90 + n) for n in (1, 9, 40, 100)]
    sp = [SamplingParams(max_new_tokens=24, temperature=0.8, top_k=50, top_p=0.95, seed=1234 + i, ignore_eos=True)
          for i in range(4)]
    together = Engine(folders["B"], dtype="float32", max_num_seqs=4, max_num_batched_tokens=8, **eng_kw).generate(prompts, sp)
    alone_eng = Engine(folders["B"], dtype="float32", max_num_seqs=4, max_num_batched_tokens=512, **eng_kw)
    for i in range(4):
        assert alone_eng.generate([prompts[i]], sp[i])[0] == together[i]
    assert len({tuple(t) for t in together}) == 4
    # the plain chain, fed the engine's documented uniform numbers, draws the same tokens
    w, c = read_weights(folders["B"])
    toks = list(prompts[1])
    for tok in together[1][:6]:
        logits = plain.llama_forward(w, c, toks)[-1].float()
        u = plain.uniform_for(sp[1].seed, len(toks))
        assert plain.sample_token(logits, 0.8, 50, 0.95, u) == tok
        toks.append(tok)


def test_preemption_recomputes_and_gives_the_same_tokens(folders):
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    prompts = [random_tokens(n, cfg["vocab_size"], 130 + n) for n in (30, 28, 26)]
    sp = SamplingParams.greedy(40, ignore_eos=True)
    roomy = Engine(folders["A"], dtype="float32", max_num_seqs=4, kv_block_size=16).generate(prompts, sp)
    tight = Engine(folders["A"], dtype="float32", max_num_seqs=4, kv_block_size=16, num_kv_blocks=9)
    out = tight.generate(prompts, sp)            # 3 x 70 tokens need 15 blocks, 9 exist
    assert out == roomy
    assert len(tight.scheduler.finished) == 3 and sum(r.preemptions for r in tight.scheduler.finished) >= 1
    assert all(r.finish_reason == "length" for r in tight.scheduler.finished)
    tight.runner.cache.audit()
    assert tight.runner.cache.free_blocks() == [9]


@pytest.mark.parametrize("name", ["A", "B"])
def test_float32_generation_does_not_depend_on_the_schedule(name, folders):
    """In float32 a row gives the same bits alone and in any batch, so greedy generation must give
    the same tokens whatever the token budget, the page size, the number of live requests, the
    number of pages (with preemption) and graphs or eager steps."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS[name]
    kw = {k: v for k, v in eng_kw.items() if k != "kv_block_size"}
    prompts = [random_tokens(n, cfg["vocab_size"], 900 + n) for n in (70, 3, 33, 64, 17, 129, 5)]
    sps = [SamplingParams.greedy(n, ignore_eos=True) for n in (40, 60, 25, 33, 50, 20, 64)]
    outs = []
    for budget, bs, seqs, graphs, blocks in [(256, 16, 8, True, None), (7, 8, 2, False, None), (32, 32, 4, True, 12),
                                             (256, 8, 8, False, 40), (7, 16, 4, True, 16), (32, 16, 2, False, None)]:
        extra = {} if blocks is None else {"num_kv_blocks": blocks}
        eng = Engine(folders[name], dtype="float32", max_num_seqs=seqs, max_num_batched_tokens=budget, kv_block_size=bs,
                     use_graphs=graphs, **extra, **kw)
        outs.append(eng.generate(prompts, sps))
        eng.runner.cache.audit()
    assert all(o == outs[0] for o in outs[1:])


def spy_on_steps(eng):
    """Records, for every step the engine runs, (request, position) and the logits of each row a
    token was chosen from."""
    log = []
    run = eng.runner.run
    cache = eng.runner.cache

    def spy(entries, samples, use_graph=True):
        rows = [(e.req_id, (cache.num_tokens(e.req_id) if cache.has(e.req_id) else 0) + len(e.tokens) - 1)
                for e in entries if e.want]
        toks = run(entries, samples, use_graph)
        if rows:
            log.append((rows, eng.runner.last_logits.float().cpu().clone()))
        return toks

    eng.runner.run = spy
    return log


def check_logged_logits(log, tokens_of, w, c, act, tol):
    """Every logged row against the plain model run over the request's final token list."""
    refs = {rid: plain.llama_forward(w, c, toks, act_dtype=act) for rid, toks in tokens_of.items()}
    worst, n = 0.0, 0
    for rows, logits in log:
        assert logits.shape[0] == len(rows)
        for i, (rid, pos) in enumerate(rows):
            assert torch.isfinite(logits[i]).all(), (rid, pos)
            e = rel_err(logits[i], refs[rid][pos])
            worst, n = max(worst, e), n + 1
            assert e < tol, f"request {rid} position {pos}: rel err {e:.3e}"
    return worst, n


def poison(eng):
    for g in eng.runner.cache.groups:
        for t in g.tensors.values():
            t.fill_(float("nan"))


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_against_the_plain_model(dtype, graphs, folders):
    """Steps captured in HIP graphs, decode steps and steps with prompt portions alike: every
    replay, with other shapes of step between replays as requests come and go, gives the plain
    model's logits at every row a token is chosen from."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    act = torch.bfloat16 if dtype == "bfloat16" else None
    w, c = read_weights(folders["A"], round_to=act)
    prompts = [random_tokens(n, cfg["vocab_size"], 300 + n) for n in (40, 3, 17, 64, 9, 77, 30)]
    sp = [SamplingParams.greedy(n, ignore_eos=True) for n in (50, 20, 35, 8, 44, 12, 25)]     # batch sizes change as they end
    sp[2] = SamplingParams(max_new_tokens=35, temperature=0.9, top_k=20, top_p=0.9, seed=5, ignore_eos=True)
    eng = Engine(folders["A"], dtype=dtype, max_num_seqs=3, max_num_batched_tokens=32, use_graphs=graphs,
                 decode_burst=1, **eng_kw)       # single steps: the logits of every one are looked at
    poison(eng)
    log = spy_on_steps(eng)
    out = eng.generate(prompts, sp)
    tokens_of = {i: p + o for i, (p, o) in enumerate(zip(prompts, out))}
    worst, n = check_logged_logits(log, tokens_of, w, c, act, 1e-4 if dtype == "float32" else 2e-2)
    print(f"{dtype} graphs={graphs}: {n} rows, worst rel err {worst:.2e}, graph steps {eng.runner.graph_steps}, "
          f"eager {eng.runner.eager_steps}")
    assert n == sum(len(o) for o in out)
    if graphs:
        kinds = {k[0] for k, g in eng.runner._graphs.items() if g.graph is not None}
        assert kinds == {"decode", "mixed"}                 # both kinds of step were captured and replayed
        assert eng.runner.graph_steps > 60
        assert not any(g.capture_failed for g in eng.runner._graphs.values())
    else:
        assert eng.runner.graph_steps == 0
    eng.runner.cache.audit()


@pytest.mark.parametrize("around", [512, 1024])
@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_past_a_context_bucket(dtype, graphs, around, tmp_path_factory):
    """Contexts that grow from below a bound on the context (512, 1024) to beyond: the decode
    graph of the next bound takes over a live batch, and the bfloat16 attention kernel splits the
    keys of a request over workgroups and a second kernel merges them, inside a graph and outside.  Logits of every step against the plain model."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, init = CONFIGS["B"]
    cfg = dict(cfg, max_position_embeddings=2048)
    key = ("past_bound",)
    if key not in _folders:
        _folders[key] = make_folder(tmp_path_factory.mktemp("past_bound"), cfg, seed=21, **init)
    folder = _folders[key]
    act = torch.bfloat16 if dtype == "bfloat16" else None
    w, c = read_weights(folder, round_to=act)
    prompts = [random_tokens(n, cfg["vocab_size"], 700 + n) for n in (around - 15, around - 22, around - 7)]
    eng = Engine(folder, dtype=dtype, max_num_seqs=4, max_num_batched_tokens=512, use_graphs=graphs,
                 max_cache_tokens=3 * (around + 64), decode_burst=1, **eng_kw)
    poison(eng)
    log = spy_on_steps(eng)
    out = eng.generate(prompts, SamplingParams.greedy(44, ignore_eos=True))
    tokens_of = {i: p + o for i, (p, o) in enumerate(zip(prompts, out))}
    worst, n = check_logged_logits(log, tokens_of, w, c, act, 1e-4 if dtype == "float32" else 2e-2)
    print(f"{dtype} graphs={graphs}: {n} rows across the {around} boundary, worst rel err {worst:.2e}")
    assert n == 3 * 44
    if graphs:
        bounds = sorted({k[2] for k, g in eng.runner._graphs.items() if k[0] == "decode" and g.graph is not None})
        assert bounds == [around, 2 * around]
    # beyond the bound the keys of a request were really shared out: the run itself asked the
    # workspace for the partial results (bfloat16: over workgroups; float32: chunks of 256 keys)
    parts = eng.runner.workspace._bufs.get(("attention_partials", torch.float32))
    heads, hd = cfg["num_attention_heads"], cfg["head_dim"]
    assert parts is not None and parts.numel() >= 2 * 3 * heads * (hd + 2)


_folders = {}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_runs_of_decode_steps_chained_on_the_device(dtype, folders):
    """Decode steps that the device chains by itself (the sampled token fed back, positions, cache
    slots and sampling counters moved on by a kernel) give the tokens of single steps: across page
    edges, with requests ending by length and by an end-of-sequence token inside a run, with
    seeded sampling, and with requests joining and leaving between runs."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    prompts = [random_tokens(n, cfg["vocab_size"], 800 + n) for n in (40, 3, 17, 64, 9, 30)]
    sps = [SamplingParams.greedy(n, ignore_eos=True) for n in (70, 33, 50, 21, 64, 45)]
    sps[2] = SamplingParams(max_new_tokens=50, temperature=0.9, top_k=20, top_p=0.9, seed=5, ignore_eos=True)
    sps[4] = SamplingParams.greedy(64)                  # may end early: eos is chosen below among its tokens
    outs = {}
    for burst in (1, 32, 5):
        eng = Engine(folders["A"], dtype=dtype, max_num_seqs=4, max_num_batched_tokens=64, decode_burst=burst, **eng_kw)
        poison(eng)
        if burst != 1:
            eng.scheduler.eos_token_id = outs[1][4][37]         # request 4 draws it in the middle of a run
        outs[burst] = eng.generate(prompts, sps)
        eng.runner.cache.audit()
        assert eng.runner.cache.free_blocks() == [g.pool.num_blocks for g in eng.runner.cache.groups]
        if burst != 1:
            assert any(g.runs > 20 and g.feeds_next for g in eng.runner._graphs.values())
            assert any(g.chain is not None for g in eng.runner._graphs.values())     # four steps a launch
            # the chain is captured behind a shape's first run: no later run pays for a capture
            assert all(g.chain is not None for g in eng.runner._graphs.values() if g.bursts > 0)
    eos = outs[1][4][37]
    cut = outs[1][4].index(eos) + 1
    want = [o if i != 4 else o[:cut] for i, o in enumerate(outs[1])]
    assert outs[32] == want and outs[5] == want
    assert [len(o) for o in want] == [70, 33, 50, 21, cut, 45]


def test_collector_rests_while_a_step_is_captured(folders, monkeypatch):
    """Python's garbage collector must not run while a step is captured: finalising the
    pinned buffers or graphs of an engine that is no longer referenced is not allowed during a
    capture and would end the process.  (torch.cuda.graph no longer collects before a capture.)"""
    import gc
    from tiny_llm_amd import Engine, SamplingParams
    from tiny_llm_amd.engine import step as step_module
    cfg = CONFIGS["A"][0]
    seen = []
    body = step_module.StepGraph._body

    def watched(self):
        seen.append((torch.cuda.is_current_stream_capturing(), gc.isenabled()))
        return body(self)

    monkeypatch.setattr(step_module.StepGraph, "_body", watched)
    assert gc.isenabled()
    prompts = [random_tokens(12, cfg["vocab_size"], 77)]
    for _ in range(2):      # the second engine is built while the first one is garbage
        Engine(folders["A"], dtype="bfloat16", use_graphs=True).generate(prompts, SamplingParams.greedy(6, ignore_eos=True))
    assert any(capturing for capturing, _ in seen)
    assert all(not collecting for capturing, collecting in seen if capturing)
    assert gc.isenabled()


def test_abort_gives_everything_back_mid_generation(folders):
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    w, c = read_weights(folders["A"])
    prompts = [random_tokens(n, cfg["vocab_size"], 400 + n) for n in (20, 45, 33)]
    eng = Engine(folders["A"], dtype="float32", max_num_seqs=4, max_num_batched_tokens=16, **eng_kw)
    ids = [eng.add_request(p, SamplingParams.greedy(30, ignore_eos=True)) for p in prompts]
    for _ in range(4):
        eng.step()                      # request 1 is still in its prompt, the others decode
    assert eng.requests[ids[1]].num_computed < 45 and len(eng.requests[ids[0]].output) > 0
    held = eng.runner.cache.free_blocks()[0]
    eng.abort(ids[0])                   # a decoding request
    eng.abort(ids[1])                   # a request in the middle of its prompt
    eng.runner.cache.audit()
    assert eng.runner.cache.free_blocks()[0] > held and eng.runner.cache.free_slots == 4
    assert eng.requests[ids[0]].finish_reason == "abort" and eng.requests[ids[1]].status == "finished"
    late = eng.add_request(prompts[1], SamplingParams.greedy(5, ignore_eos=True))     # takes the pages over
    while eng.has_unfinished():
        eng.step()
    assert eng.requests[ids[2]].output == plain.greedy_generate(w, c, prompts[2], 30)
    assert eng.requests[late].output == plain.greedy_generate(w, c, prompts[1], 5)
    assert eng.runner.cache.free_blocks() == [g.pool.num_blocks for g in eng.runner.cache.groups]
    eng.abort(ids[2])                   # finished already: nothing happens
    eng.runner.cache.audit()


def test_a_request_that_cannot_go_on_even_alone_ends_with_capacity(folders):
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    w, c = read_weights(folders["A"])
    eng = Engine(folders["A"], dtype="float32", max_num_seqs=2, kv_block_size=16, num_kv_blocks=3)
    prompt = random_tokens(40, cfg["vocab_size"], 41)
    out = eng.generate([prompt], SamplingParams.greedy(30, ignore_eos=True))[0]
    req = eng.scheduler.finished[-1]
    assert req.finish_reason == "capacity" and len(out) == 3 * 16 - 40 + 1      # 48 cached tokens, one more chosen
    assert out == plain.greedy_generate(w, c, prompt, len(out))
    assert eng.runner.cache.free_blocks() == [3]
    with pytest.raises(ValueError):                  # a prompt that the whole pool cannot hold is refused at once
        eng.add_request(random_tokens(60, cfg["vocab_size"], 42), SamplingParams.greedy(2))


def test_preemption_in_bfloat16_with_seeded_sampling(folders):
    """Recomputation after a preemption goes through other kernels than the first pass (a long
    prompt portion instead of single tokens), so in bfloat16 logits differ by rounding; tokens are
    compared where the plain model's choice is clear of that, logits everywhere."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    w, c = read_weights(folders["A"], round_to=torch.bfloat16)
    prompts = [random_tokens(n, cfg["vocab_size"], 530 + n) for n in (30, 28, 26)]
    sps = [SamplingParams(max_new_tokens=40, temperature=0.8, top_k=40, top_p=0.95, seed=900 + i, ignore_eos=True)
           for i in range(3)]
    tight = Engine(folders["A"], dtype="bfloat16", max_num_seqs=4, kv_block_size=16, num_kv_blocks=9, decode_burst=1)
    poison(tight)
    log = spy_on_steps(tight)
    out = tight.generate(prompts, sps)
    assert sum(r.preemptions for r in tight.scheduler.finished) >= 1
    assert all(len(o) == 40 for o in out)
    tight.runner.cache.audit()
    assert tight.runner.cache.free_blocks() == [9]
    # a preempted request is recomputed from position 0; what it had generated stays its own
    worst, n = check_logged_logits(log, {r.req_id: r.tokens for r in tight.scheduler.finished}, w, c, torch.bfloat16, 2e-2)
    print(f"preemption in bfloat16: {n} rows , worst rel err {worst:.2e}")
    assert n == 120
    refs = [plain.llama_forward(w, c, p + o, act_dtype=torch.bfloat16) for p, o in zip(prompts, out)]
    for i, (p, o) in enumerate(zip(prompts, out)):
        for j, tok in enumerate(o):
            row = refs[i][len(p) + j - 1].float()
            u = plain.uniform_for(sps[i].seed, len(p) + j)
            want = plain.sample_token(row, 0.8, 40, 0.95, u)
            if want != tok:
                # the engine drew the same uniform number from logits that differ by rounding: the two
                # tokens are neighbours in the cumulative distribution
                probs = torch.softmax(row.double() / 0.8, -1)
                assert float(probs[tok]) > 1e-4
    agree = sum(plain.sample_token(refs[i][len(p) + j - 1].float(), 0.8, 40, 0.95,
                                   plain.uniform_for(sps[i].seed, len(p) + j)) == tok
                for i, (p, o) in enumerate(zip(prompts, out)) for j, tok in enumerate(o))
    assert agree >= 0.9 * 120


def test_sharded_folder_generates_like_the_single_file(folders, tmp_path):
    from safetensors import safe_open
    from tiny_llm_amd import Engine, SamplingParams
    from tiny_llm_amd.weights import save_file
    cfg, eng_kw, _ = CONFIGS["B"]
    with safe_open(os.path.join(folders["B"], "model.safetensors"), "pt") as f:
        names = list(f.keys())
        weight_map = {}
        for i in range(2):
            fname = f"model-{i + 1:05d}-of-00002.safetensors"
            save_file({n: f.get_tensor(n) for n in names[i::2]}, str(tmp_path / fname))
            weight_map.update({n: fname for n in names[i::2]})
    json.dump({"metadata": {}, "weight_map": weight_map}, open(tmp_path / "model.safetensors.index.json", "w"))
    json.dump(json.load(open(os.path.join(folders["B"], "config.json"))), open(tmp_path / "config.json", "w"))
    prompts = [random_tokens(n, cfg["vocab_size"], 60 + n) for n in (9, 40)]
    sp = SamplingParams.greedy(12, ignore_eos=True)
    a = Engine(folders["B"], dtype="float32", **eng_kw).generate(prompts, sp)
    b = Engine(str(tmp_path), dtype="float32", **eng_kw).generate(prompts, sp)
    assert a == b


def test_a_step_that_fails_leaves_the_cache_as_it_was(folders):
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, load_model
    from tiny_llm_amd.engine.step import StepEntry
    cfg, eng_kw, _ = CONFIGS["A"]
    engine = EngineConfig(dtype="float32", max_cache_tokens=256, max_num_seqs=3, use_graphs=False, **eng_kw)
    _, dec = load_model(folders["A"], engine)
    runner = build_runner(dec, engine)
    a = random_tokens(40, cfg["vocab_size"], 1)
    first = runner.step([StepEntry("a", a[:20], [19])]).cpu()
    before = (runner.cache.free_blocks(), runner.cache.free_slots, list(runner.cache.block_table("a", 0)))
    forward = dec.forward

    def broken(ctx):
        raise RuntimeError("a kernel refused")
    dec.forward = broken
    with pytest.raises(RuntimeError):
        runner.step([StepEntry("a", a[20:], [19]), StepEntry("b", a[:17], [16])])
    dec.forward = forward
    assert (runner.cache.free_blocks(), runner.cache.free_slots, list(runner.cache.block_table("a", 0))) == before
    assert not runner.cache.has("b") and runner.cache.num_tokens("a") == 20
    runner.cache.audit()
    again = runner.step([StepEntry("a", a[20:], [19]), StepEntry("b", a[:20], [19])]).cpu()
    assert rel_err(again[1], first[0]) < 1e-6


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_logits_have_the_same_bits_alone_and_in_any_batch(name, folders):
    """In float32 a token's logits must not depend, to the bit, on what else its step holds: decoded
    alone (1 row: norms ride in the few-row products), beside other decoding requests, beside a
    prompt portion that makes the step 40 and 200 rows long (the norm as a row factor of the tiled
    products; attention by tiles), and as a captured step."""
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, load_model
    from tiny_llm_amd.engine.step import StepEntry
    cfg, eng_kw, _ = CONFIGS[name]
    engine = EngineConfig(dtype="float32", max_cache_tokens=2048, max_num_seqs=4, max_num_batched_tokens=512,
                          use_graphs=True, **eng_kw)
    _, dec = load_model(folders[name], engine)
    runner = build_runner(dec, engine)
    V = cfg["vocab_size"]
    a, other, long = random_tokens(60, V, 1), random_tokens(30, V, 2), random_tokens(400, V, 3)
    results = []
    for beside, graph in ((None, False), ("decoding", False), (39, False), (199, False), (39, True), (None, True)):
        runner.step([StepEntry("a", a[:50], [])])
        if beside == "decoding":
            runner.step([StepEntry("o", other[:20], []), StepEntry("p", long[:77], [])])
        rows = []
        for at in range(50, 60):
            ents = [StepEntry("a", [a[at]], [0])]
            if beside == "decoding":
                ents = [StepEntry("o", [other[at - 30]], [0])] + ents + [StepEntry("p", [long[at + 27]], [])]
            elif beside is not None:
                ents = [StepEntry(f"l{at}", long[:beside], [beside - 1])] + ents
            out = runner.step(ents, use_graph=graph)
            rows.append(out[1 if beside is not None else 0].clone())
            if beside not in (None, "decoding"):
                runner.finish(f"l{at}")
        results.append(torch.stack(rows).cpu())
        for r in ("a", "o", "p"):
            runner.finish(r)
    for got in results[1:]:
        assert torch.equal(got, results[0])
    runner.cache.audit()


def test_captured_shapes_are_bounded_and_come_back(folders):
    """At most MAX_STEP_SHAPES shapes of step keep their buffers and graphs; the one used longest ago
    goes, and is simply built and captured again when its shape returns."""
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, load_model
    from tiny_llm_amd.engine.step import StepEntry
    cfg, eng_kw, _ = CONFIGS["A"]
    w, c = read_weights(folders["A"])
    engine = EngineConfig(dtype="float32", max_cache_tokens=512, max_num_seqs=4, **eng_kw)
    _, dec = load_model(folders["A"], engine)
    runner = build_runner(dec, engine)
    runner.MAX_STEP_SHAPES = 2
    toks = {r: random_tokens(40, cfg["vocab_size"], 70 + i) for i, r in enumerate("abc")}
    refs = {r: plain.llama_forward(w, c, t) for r, t in toks.items()}
    at = {r: 0 for r in toks}

    def step(who, n):
        ents = [StepEntry(r, toks[r][at[r]:at[r] + n], [n - 1]) for r in who]
        got = runner.step(ents, use_graph=True).cpu()
        for i, r in enumerate(who):
            at[r] += n
            assert rel_err(got[i], refs[r][at[r] - 1]) < 1e-4
    step("abc", 5)                       # a mixed shape
    for _ in range(3):
        step("abc", 1)                   # decode, three requests: eager, captured, replayed
    for _ in range(3):
        step("ab", 1)                    # decode, two requests: the mixed shape goes
    assert len(runner._graphs) == 2 and {k[0] for k in runner._graphs} == {"decode"}
    for _ in range(3):
        step("c", 1)                     # decode, one request: the three-request shape goes
    assert [k[1] for k in runner._graphs] == [2, 1]
    for _ in range(3):
        step("abc", 1)                   # and comes back
    assert [k[1] for k in runner._graphs] == [1, 3] and runner._graphs[("decode", 3, 512, False)].graph is not None


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_captured_step_that_fails_leaves_no_stale_block_table(dtype, folders):
    """A replayed decode step fails after its tables were laid out and is undone; another request
    takes the block that went back; the step is run again and the requests grow to the same
    lengths with other blocks.  The static buffers of the captured step must follow: logits
    against the plain model, with a poisoned pool."""
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, load_model
    from tiny_llm_amd.engine.step import StepEntry
    cfg, eng_kw, _ = CONFIGS["A"]
    act = torch.bfloat16 if dtype == "bfloat16" else None
    tol = 1e-4 if dtype == "float32" else 2e-2
    w, c = read_weights(folders["A"], round_to=act)
    engine = EngineConfig(dtype=dtype, max_cache_tokens=256, max_num_seqs=3, use_graphs=True, **eng_kw)
    bs = engine.kv_block_size
    _, dec = load_model(folders["A"], engine)
    runner = build_runner(dec, engine)
    for g in runner.cache.groups:
        for t in g.tensors.values():
            t.fill_(float("nan"))
    n0 = 2 * bs - 2
    toks = {r: random_tokens(n0 + 8, cfg["vocab_size"], 90 + i) for i, r in enumerate("ab")}
    toks["c"] = random_tokens(5, cfg["vocab_size"], 99)
    refs = {r: plain.llama_forward(w, c, t, act_dtype=act) for r, t in toks.items()}
    runner.step([StepEntry(r, toks[r][:n0], []) for r in "ab"], use_graph=True)

    def decode(at):
        got = runner.step([StepEntry(r, [toks[r][at]], [0]) for r in "ab"], use_graph=True).cpu()
        for i, r in enumerate("ab"):
            assert rel_err(got[i], refs[r][at]) < tol, (r, at)

    decode(n0)              # eagerly on the static buffers
    decode(n0 + 1)          # captured
    sg = next(g for k, g in runner._graphs.items() if k[0] == "decode" and g.graph is not None)
    before = {r: list(runner.cache.block_table(r, 0)) for r in "ab"}

    class Refuses:
        def replay(self):
            raise RuntimeError("the replay was refused")
    good, sg.graph = sg.graph, Refuses()
    with pytest.raises(RuntimeError):
        decode(n0 + 2)      # starts a new block for both: laid out, then undone
    sg.graph = good
    assert {r: list(runner.cache.block_table(r, 0)) for r in "ab"} == before
    got = runner.step([StepEntry("c", toks["c"], [4])], use_graph=True).cpu()      # takes the block a was given
    assert rel_err(got[0], refs["c"][4]) < tol
    for at in range(n0 + 2, n0 + 8):
        decode(at)
    assert runner.cache.block_table("a", 0)[2] != runner.cache.block_table("c", 0)[0]
    assert runner.graph_steps >= 6
    runner.cache.audit()


def test_command_line_generates_from_prompt_ids(folders):
    cfg = CONFIGS["A"][0]
    prompt = random_tokens(12, cfg["vocab_size"], 5)
    w, c = read_weights(folders["A"])
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tiny_llm"), "--model_path", folders["A"],
                           "--nodo_sample", "--max_new_tokens=5", "--dtype", "float32", "--ignore_eos",
                           "--prompt_ids", ",".join(map(str, prompt))], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [int(t) for t in proc.stdout.strip().splitlines()[-1].split()]
    assert got == plain.greedy_generate(w, c, prompt, 5)
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tiny_llm"), "--model_path", "/nonexistent"],
                         capture_output=True, text=True, timeout=120)
    assert bad.returncode == 1 and "[Fatal]" in bad.stderr


def test_command_line_interactive_loop(folders):
    """The reference's loop (main.cpp:51-85): lines up to a blank line are one prompt, a blank line
    alone asks again, the end of the input ends the program with 0.  Without a tokenizer in the folder
    a prompt is token ids; they may come on several lines."""
    cfg = CONFIGS["A"][0]
    w, c = read_weights(folders["A"])
    p1, p2 = random_tokens(9, cfg["vocab_size"], 41), random_tokens(14, cfg["vocab_size"], 42)
    text = (" ".join(map(str, p1)) + "\n\n"                                      # one line, then the blank line
            + "\n"                                                              # an empty prompt
            + " ".join(map(str, p2[:6])) + "\n" + ",".join(map(str, p2[6:])) + "\n\n")      # two lines
    for extra in ([], ["--stream"]):
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tiny_llm"), "--model_path", folders["A"],
                               "--nodo_sample", "--max_new_tokens=6", "--dtype=float32", "--ignore_eos"] + extra,
                              input=text, capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        out = proc.stdout
        assert out.count("[Input] >") == 4 and out.count("[Output] >") == 2 and "The prompt is empty" in out
        answers = [blk.strip().splitlines()[0] for blk in out.split("[Output] >")[1:]]
        assert [[int(t) for t in a.split()] for a in answers] == [plain.greedy_generate(w, c, p1, 6),
                                                                  plain.greedy_generate(w, c, p2, 6)]


def test_command_line_speaks_text_when_the_folder_has_a_tokenizer(folders, tmp_path):
    """With tokenizer.json in the model folder prompts are text and so is the output
    (tiny_llm/pipeline/pipeline.cpp:113, 236: encode with special tokens, decode without)."""
    tokenizers = pytest.importorskip("tokenizers")
    import shutil
    cfg = CONFIGS["A"][0]
    folder = tmp_path / "with_tokenizer"
    shutil.copytree(folders["A"], folder)
    vocab = {f"w{i}": i for i in range(cfg["vocab_size"])}
    tok = tokenizers.Tokenizer(tokenizers.models.WordLevel(vocab, unk_token="w0"))
    tok.pre_tokenizer = tokenizers.pre_tokenizers.Whitespace()
    tok.save(str(folder / "tokenizer.json"))
    w, c = read_weights(str(folder))
    prompt = random_tokens(10, cfg["vocab_size"], 77)
    text = " ".join(f"w{t}" for t in prompt) + "\n\n"
    want = plain.greedy_generate(w, c, prompt, 5)
    for extra in ([], ["--stream"]):
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tiny_llm"), "--model_path", str(folder),
                               "--nodo_sample", "--max_new_tokens=5", "--dtype=float32", "--ignore_eos"] + extra,
                              input=text, capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        answer = proc.stdout.split("[Output] >")[1].strip().splitlines()[0]
        assert answer == " ".join(f"w{t}" for t in want), answer


def test_finished_requests_are_let_go(folders):
    """`generate` forgets its requests when it returns; a request added by hand stays until it is
    released, and beyond the bound the oldest finished ones go by themselves; the scheduler's record
    of finished requests is bounded too."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    eng = Engine(folders["A"], dtype="float32", max_num_seqs=4, **eng_kw)
    eng.FINISHED_KEPT = 6
    eng.scheduler.finished = type(eng.scheduler.finished)(maxlen=5)
    p = random_tokens(7, cfg["vocab_size"], 3)
    eng.generate([p, p], SamplingParams.greedy(3, ignore_eos=True))
    assert eng.requests == {}
    rid = eng.add_request(p, SamplingParams.greedy(2, ignore_eos=True))
    assert eng.release(rid) is None                   # live: it stays
    while eng.has_unfinished():
        eng.step()
    assert eng.requests[rid].finish_reason == "length"
    kept = eng.release(rid)
    assert kept.output and rid not in eng.requests and eng.release(rid) is None
    ids = []
    for _ in range(10):
        ids.append(eng.add_request(p, SamplingParams.greedy(1, ignore_eos=True)))
        while eng.has_unfinished():
            eng.step()
    assert len(eng.requests) <= 7 and ids[-1] in eng.requests and ids[0] not in eng.requests
    assert len(eng.scheduler.finished) == 5


def test_tokens_stream_as_they_are_generated(folders):
    """`stream` yields every prompt's tokens in order, each once, with the finish reason at the end;
    together they are what `generate` returns; a bound of one decode step hands over a token at a time."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg, eng_kw, _ = CONFIGS["A"]
    prompts = [random_tokens(n, cfg["vocab_size"], 300 + n) for n in (5, 40, 17)]
    sp = [SamplingParams.greedy(n, ignore_eos=True) for n in (9, 3, 20)]
    eng = Engine(folders["A"], dtype="float32", max_num_seqs=4, max_num_batched_tokens=32, **eng_kw)
    want = eng.generate(prompts, sp)
    assert [len(o) for o in want] == [9, 3, 20]
    for bound in (None, 1):
        got = [[] for _ in prompts]
        reasons = [None] * 3
        chunks = [[] for _ in prompts]
        for i, fresh, reason in eng.stream(prompts, sp, max_decode_steps=bound):
            assert reasons[i] is None, "tokens after a request's end"
            got[i] += fresh
            chunks[i].append(len(fresh))
            reasons[i] = reason
        assert got == want and reasons == ["length"] * 3
        if bound == 1:
            assert all(c <= 1 for per in chunks for c in per)
        else:
            assert max(chunks[2]) > 1               # chained decode steps hand over several tokens at once
    seen = []
    assert eng.generate(prompts[:1], sp[0], on_tokens=lambda i, t, r: seen.append((i, list(t), r))) == want[:1]
    assert [t for _, ts, _ in seen for t in ts] == want[0] and seen[-1][2] == "length"
    # a request that asks for nothing ends at once, with its reason and no tokens
    assert list(eng.stream([prompts[0]], SamplingParams.greedy(0))) == [(0, [], "length")]


def test_command_line_streams_and_takes_norm_std(tmp_path):
    """--stream prints the same ids as the plain run; --norm_std reaches the random weights."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg = CONFIGS["B"][0]
    only_config = tmp_path / "only_config"
    only_config.mkdir()
    with open(only_config / "config.json", "w") as f:
        json.dump(cfg, f)
    prompt = random_tokens(11, cfg["vocab_size"], 31)
    base = [sys.executable, os.path.join(ROOT, "bin", "tiny_llm"), "--model_path", str(only_config),
            "--random_weights", "--weights_seed=5", "--norm_std=0.3", "--nodo_sample", "--max_new_tokens=40",
            "--dtype", "float32", "--ignore_eos", "--kv_block_size=8", "--prompt_ids", ",".join(map(str, prompt))]
    outs = []
    for extra in ([], ["--stream"]):
        proc = subprocess.run(base + extra, capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        outs.append([int(t) for t in proc.stdout.strip().splitlines()[-1].split()])
    engine = Engine(config=cfg, dtype="float32", weights_seed=5, norm_std=0.3, kv_block_size=8)
    want = engine.generate([prompt], SamplingParams.greedy(40, ignore_eos=True))[0]
    assert outs[0] == want and outs[1] == want
    flat = Engine(config=cfg, dtype="float32", weights_seed=5, norm_std=0.0, kv_block_size=8)
    assert flat.generate([prompt], SamplingParams.greedy(40, ignore_eos=True))[0] != want


def test_command_line_random_weights_and_prompt_file(tmp_path):
    """--random_weights takes only config.json from the folder and fills the weights on the device
    from --weights_seed, as the Python entry point does for a configuration; --prompt_ids_file
    holds one prompt a line."""
    from tiny_llm_amd import Engine, SamplingParams
    cfg = CONFIGS["A"][0]
    only_config = tmp_path / "only_config"
    only_config.mkdir()
    with open(only_config / "config.json", "w") as f:
        json.dump(cfg, f)
    prompts = [random_tokens(9, cfg["vocab_size"], 21), random_tokens(14, cfg["vocab_size"], 22)]
    ids_file = tmp_path / "prompts.txt"
    ids_file.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tiny_llm"), "--model_path", str(only_config),
                           "--random_weights", "--weights_seed=11", "--init_std=0.05", "--nodo_sample",
                           "--max_new_tokens=4", "--dtype", "float32", "--ignore_eos",
                           "--prompt_ids_file", str(ids_file)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [[int(t) for t in line.split()] for line in proc.stdout.strip().splitlines()[-2:]]
    engine = Engine(config=cfg, dtype="float32", weights_seed=11, init_std=0.05)
    assert got == engine.generate(prompts, SamplingParams.greedy(4, ignore_eos=True))
    other = Engine(config=cfg, dtype="float32", weights_seed=12, init_std=0.05)
    assert got != other.generate(prompts, SamplingParams.greedy(4, ignore_eos=True))


# ------------------------------------------------------ a toy architecture
def test_toy_stateful_mixer_registers_builds_and_steps(tmp_path):
    """A mixer with per-request state of fixed size (an exponential running mean), defined here.
    The toy model mixes it with attention layers, runs one layer twice and lets one run read
    another run's cache.  Cutting its input differently must not change its logits."""
    from tiny_llm_amd.config import (EngineConfig, ModelSpec, PartSpec, PlanEntry, pre_norm_layer,
                                     register_architecture, unregister_architecture)
    from tiny_llm_amd.engine.loading import build_runner, random_model
    from tiny_llm_amd.engine.step import StepEntry
    from tiny_llm_amd.parts import MIXERS, Mixer, StateSpec, WeightSpec, add_to_residual, register_mixer

    class DecayMixer(Mixer):
        def __init__(self, prefix, dtype, device, *, hidden_size, decay):
            super().__init__(prefix, dtype, device)
            self.hidden_size, self.decay = hidden_size, decay

        def weights(self):
            return [WeightSpec(f"{self.prefix}.gain", (self.hidden_size,), role="vector", init="ones")]

        def bind(self, tensors):
            self.gain = tensors[f"{self.prefix}.gain"].float()

        def state_spec(self):
            return StateSpec((self.hidden_size,), torch.float32)

        def forward(self, h, ctx, cache, state, residual):
            out = torch.empty_like(h, dtype=torch.float32)
            t = 0
            for slot, n in zip(ctx.slots_host, ctx.q_lens):     # each request's tokens, in order, once
                s = state[slot]
                for i in range(n):
                    s = self.decay * s + h[t + i].float()
                    out[t + i] = s * self.gain
                state[slot] = s
                t += n
            return add_to_residual(residual, out)

    def read(raw):
        return dict(raw)

    def build(cfg):
        H = cfg["hidden_size"]
        norm = PartSpec("rmsnorm", {"hidden_size": H, "eps": 1e-5})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg["intermediate_size"]})
        attn = PartSpec("attention", {"hidden_size": H, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                      "position": {"kind": "rotary", "head_dim": 16, "theta": 100.0, "max_position": 256}})
        win = PartSpec("attention", {"hidden_size": H, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "window": 5,
                                     "position": {"kind": "none"}})
        toy = PartSpec("toy_decay", {"hidden_size": H, "decay": 0.5})
        layers = tuple(pre_norm_layer(f"model.layers.{i}", norm, m, norm, ffn) for i, m in enumerate([attn, toy, win]))
        # layer 0, layer 1 (state), layer 2 (window), layer 0 again with a cache of its own,
        # then layer 0 once more reading the first run's cache
        plan = (PlanEntry(0), PlanEntry(1), PlanEntry(2), PlanEntry(0), PlanEntry(0, cache_of=0))
        sizes = {"vocab_size": cfg["vocab_size"], "hidden_size": H}
        return ModelSpec("ToyForCausalLM", cfg["vocab_size"], H, 256, PartSpec("token_embedding", sizes, "model.embed_tokens"),
                         layers, plan, norm.named("model.norm"),
                         PartSpec("lm_head", dict(sizes, tied_to="model.embed_tokens"), "lm_head"))

    register_mixer("toy_decay", DecayMixer)
    register_architecture("ToyForCausalLM", read, build)
    try:
        raw = {"architectures": ["ToyForCausalLM"], "hidden_size": 64, "intermediate_size": 96, "vocab_size": 101}
        engine = EngineConfig(dtype="float32", kv_block_size=4, max_cache_tokens=256, max_num_seqs=3,
                              max_num_batched_tokens=48, use_graphs=False)
        _, dec = random_model(raw, engine, seed=1, std=0.3)
        runner = build_runner(dec, engine)
        assert [g.entries for g in runner.cache.groups] == [[(0, "mixer"), (3, "mixer")], [(2, "mixer")]]   # full, windowed
        # the windowed group never holds more of a request than its window and a step's tokens:
        # (5 - 1 + 48) positions, starting anywhere in a block, for each of 3 requests
        assert runner.cache.group_blocks == [64, 3 * 14]
        assert runner.decoder.caches[2]["mixer"].k.shape[0] == 42 and runner.decoder.caches[0]["mixer"].k.shape[0] == 64
        assert runner.decoder.states[1]["mixer"].shape == (3, 64) and runner.decoder.states[0] == {}
        a, b = random_tokens(45, 101, 1), random_tokens(23, 101, 2)
        whole = torch.cat([runner.step([StepEntry("a", a, list(range(45)))]).cpu(),
                           runner.step([StepEntry("b", b, list(range(23)))]).cpu()])
        runner.finish("a")
        runner.finish("b")
        got_a, got_b = [], []
        at_a = at_b = 0
        for na, nb in [(7, 2), (2, 0), (19, 11), (1, 1), (16, 9)]:
            ents = [StepEntry("a", a[at_a:at_a + na], list(range(na)))] if na else []
            if nb:
                ents.append(StepEntry("b", b[at_b:at_b + nb], list(range(nb))))
            l = runner.step(ents).cpu()
            got_a.append(l[:na])
            got_b.append(l[na:])
            at_a, at_b = at_a + na, at_b + nb
            runner.cache.audit()
        assert at_a == 45 and at_b == 23
        assert rel_err(torch.cat(got_a), whole[:45]) < 1e-5 and rel_err(torch.cat(got_b), whole[45:]) < 1e-5
        # the window group gave back what its window passed; the full group kept everything
        assert sum(x >= 0 for x in runner.cache.block_table("a", 1)) <= 3
        assert all(x >= 0 for x in runner.cache.block_table("a", 0))
        # a slot is zeroed when a new request takes it
        runner.finish("a")
        again = runner.step([StepEntry("c", a, list(range(45)))]).cpu()
        assert rel_err(again, whole[:45]) < 1e-5
        # As captured steps: the toy mixer runs loops on the host and may not be captured, so a step is
        # the graph of the stages before it, the toy layer eagerly, the graph of the stages behind it.
        # Each shape of step: first eagerly, then captured, then replayed; the same logits every time.
        assert not runner.decoder.graph_safe and runner.graphs_possible
        assert [(safe, first, last) for safe, first, last in runner.decoder.graph_runs()] == [(True, 0, 2), (False, 2, 3), (True, 3, 7)]
        runner.finish("c")
        for rid in ("g0", "g1", "g2", "g3"):
            got = runner.step([StepEntry(rid, a, list(range(45)))], use_graph=True).cpu()
            assert rel_err(got, whole[:45]) < 1e-5, rid
            runner.finish(rid)
        sg = next(g for k, g in runner._graphs.items() if k[0] == "mixed")
        assert sg.runs_captured and [g is not None for g in sg.run_graphs] == [True, False, True] and sg.graph is None
        before = runner.graph_steps
        runner.step([StepEntry("h", a[:38], [])], use_graph=True)
        runner.step([StepEntry("i", b[:20], [])], use_graph=True)
        for t in range(38, 45):       # single tokens of two requests: one shape, captured at its second step
            ents = [StepEntry("h", [a[t]], [0])] + ([StepEntry("i", [b[t - 18]], [0])] if t - 18 < 23 else [])
            got = runner.step(ents, use_graph=True).cpu()
            assert rel_err(got[0], whole[t]) < 1e-5, t
            if len(ents) == 2:
                assert rel_err(got[1], whole[45 + t - 18]) < 1e-5, t
            runner.cache.audit()
        assert runner.graph_steps - before >= 4
        runner.finish("h")
        runner.finish("i")
        # the state matters: another decay, other logits
        dec.layers[1].mixer.decay = 0.9
        assert rel_err(runner.step([StepEntry("d", a, list(range(45)))]).cpu(), whole[:45]) > 1e-3
        # through the entry point: the scheduler's steps, the sampler behind the last run of stages;
        # the same tokens with graphs and without (runs of chained decode steps need the whole model
        # in one graph: asked for, they fall back to single steps)
        from tiny_llm_amd import Engine, SamplingParams
        prompts = [a[:30], b, a[5:12]]
        sps = [SamplingParams.greedy(20, ignore_eos=True), SamplingParams.greedy(9, ignore_eos=True),
               SamplingParams(max_new_tokens=25, temperature=0.9, top_k=20, seed=5, ignore_eos=True)]
        outs = []
        for graphs in (False, True):
            eng = Engine(config=raw, dtype="float32", weights_seed=1, init_std=0.3, kv_block_size=4, max_cache_tokens=256,
                         max_num_seqs=3, max_num_batched_tokens=16, use_graphs=graphs, decode_burst=32)
            outs.append(eng.generate(prompts, sps))
            eng.runner.cache.audit()
            assert (eng.runner.graph_steps > 20) == graphs
        assert outs[0] == outs[1] and [len(o) for o in outs[0]] == [20, 9, 25]
    finally:
        MIXERS.unregister("toy_decay")
        unregister_architecture("ToyForCausalLM")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_other_position_encoding(dtype):
    """A feed-forward with routing (two experts, the larger router logit takes the token) and a
    position encoding of its own (a rotation of the first half of each head with doubled angles),
    both defined here, in a toy architecture: registered, built, and stepped in different cuttings."""
    from tiny_llm_amd.config import (EngineConfig, ModelSpec, PartSpec, PlanEntry, pre_norm_layer,
                                     register_architecture, unregister_architecture)
    from tiny_llm_amd.engine.loading import build_runner, random_model
    from tiny_llm_amd.engine.step import StepEntry
    from tiny_llm_amd.kernels import ops
    from tiny_llm_amd.parts import (EMBEDDINGS, FEED_FORWARDS, HEADS, POSITION_ENCODINGS, Embedding, FeedForward, Head,
                                    PositionEncoding, WeightSpec, add_to_residual, register_embedding,
                                    register_feed_forward, register_head, register_position_encoding)

    class DoubledHalfRotary(PositionEncoding):
        def __init__(self, prefix, dtype, device, *, head_dim, max_position):
            super().__init__(prefix, dtype, device)
            self.rot = head_dim // 2
            inv = torch.pow(torch.tensor(50.0, dtype=torch.float64), -torch.arange(self.rot // 2, dtype=torch.float64)
                            / (self.rot // 2))
            ang = 2.0 * torch.arange(max_position, dtype=torch.float64)[:, None] * inv[None, :]
            self.cos, self.sin = torch.cos(ang).float().to(device), torch.sin(ang).float().to(device)

        def rotary_tables(self):
            return self.cos, self.sin, self.rot

    used = set()

    class TwoExperts(FeedForward):
        def __init__(self, prefix, dtype, device, *, hidden_size, intermediate_size):
            super().__init__(prefix, dtype, device)
            self.H, self.I = hidden_size, intermediate_size

        def weights(self):
            w = [WeightSpec(f"{self.prefix}.router.weight", (2, self.H))]
            for e in range(2):
                w += [WeightSpec(f"{self.prefix}.experts.{e}.up.weight", (self.I, self.H)),
                      WeightSpec(f"{self.prefix}.experts.{e}.down.weight", (self.H, self.I))]
            return w

        def bind(self, tensors):
            self.router = tensors[f"{self.prefix}.router.weight"].float()
            self.up = [tensors[f"{self.prefix}.experts.{e}.up.weight"].contiguous() for e in range(2)]
            self.down = [tensors[f"{self.prefix}.experts.{e}.down.weight"].contiguous() for e in range(2)]

        def forward(self, h, ctx, residual):
            choice = (h.float() @ self.router.T).argmax(dim=-1)          # router logits in float32
            y = torch.zeros_like(residual)
            for e in range(2):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                used.add(e)
                mid = torch.empty((rows.numel(), self.I), dtype=h.dtype, device=h.device)
                ops.linear(h[rows].contiguous(), self.up[e], mid)
                out = torch.empty((rows.numel(), self.H), dtype=torch.float32, device=h.device)
                ops.linear(torch.relu(mid), self.down[e], out)
                y[rows] = out
            return add_to_residual(residual, y)

    class ScaledEmbedding(Embedding):
        """An embedding with a scale and a table under another name, looked up with torch."""
        def __init__(self, prefix, dtype, device, *, vocab_size, hidden_size, scale):
            super().__init__(prefix, dtype, device)
            self.V, self.H, self.scale = vocab_size, hidden_size, scale

        def weights(self):
            return [WeightSpec(f"{self.prefix}.table", (self.V, self.H))]

        def bind(self, tensors):
            self.table = tensors[f"{self.prefix}.table"]

        def forward(self, tokens, ctx=None):
            return (self.table[tokens.long()].float() * self.scale).contiguous()

    class CappedHead(Head):
        """A head of its own name whose logits are soft-capped: cap * tanh(logits / cap)."""
        def __init__(self, prefix, dtype, device, *, vocab_size, hidden_size, cap):
            super().__init__(prefix, dtype, device)
            self.V, self.H, self.cap = vocab_size, hidden_size, cap

        def weights(self):
            return [WeightSpec(f"{self.prefix}.proj", (self.V, self.H))]

        def bind(self, tensors):
            self.w = tensors[f"{self.prefix}.proj"].contiguous()

        def forward(self, h):
            out = torch.empty((h.shape[0], self.V), dtype=torch.float32, device=h.device)
            return self.cap * torch.tanh(ops.linear(h, self.w, out) / self.cap)

    def build(cfg):
        H = cfg["hidden_size"]
        norm = PartSpec("rmsnorm", {"hidden_size": H, "eps": 1e-5})
        attn = PartSpec("attention", {"hidden_size": H, "num_heads": 4, "num_kv_heads": 1, "head_dim": 16,
                                      "position": {"kind": "doubled_half_rotary", "head_dim": 16, "max_position": 256}})
        dense = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 96})
        routed = PartSpec("two_experts", {"hidden_size": H, "intermediate_size": 40})
        names = {"mixer_norm": "ln1", "mixer": "attn", "ffn_norm": "ln2", "ffn": "moe"}
        layers = (pre_norm_layer("decoder.h.0", norm, attn, norm, routed, names),
                  pre_norm_layer("decoder.h.1", norm, attn, norm, dense, names))
        return ModelSpec("Toy2ForCausalLM", cfg["vocab_size"], H, 256,
                         PartSpec("scaled_embedding", {"vocab_size": cfg["vocab_size"], "hidden_size": H, "scale": 2.0},
                                  "decoder.wte"), layers,
                         (PlanEntry(0), PlanEntry(1)), norm.named("decoder.ln_f"),
                         PartSpec("capped_head", {"vocab_size": cfg["vocab_size"], "hidden_size": H, "cap": 3.0},
                                  "output"))

    register_position_encoding("doubled_half_rotary", DoubledHalfRotary)
    register_feed_forward("two_experts", TwoExperts)
    register_embedding("scaled_embedding", ScaledEmbedding)
    register_head("capped_head", CappedHead)
    register_architecture("Toy2ForCausalLM", dict, build)
    try:
        raw = {"architectures": ["Toy2ForCausalLM"], "hidden_size": 64, "vocab_size": 101}
        engine = EngineConfig(dtype=dtype, kv_block_size=8, max_cache_tokens=256, max_num_seqs=3,
                              max_num_batched_tokens=256, use_graphs=False)
        _, dec = random_model(raw, engine, seed=3, std=0.3)
        # embedding, head and layers carry the names this architecture gave them
        names = {s.name for s in dec.weight_specs()}
        assert {"decoder.wte.table", "output.proj", "decoder.ln_f.weight", "decoder.h.0.attn.q_proj.weight",
                "decoder.h.0.moe.router.weight", "decoder.h.1.ln2.weight"} <= names
        assert not any(n.startswith(("model.", "lm_head")) for n in names)
        runner = build_runner(dec, engine)
        a, b = random_tokens(41, 101, 5), random_tokens(18, 101, 6)
        whole = runner.step([StepEntry("a", a, list(range(41))), StepEntry("b", b, list(range(18)))]).cpu()
        assert used == {0, 1}                       # both experts got tokens
        assert float(whole.abs().max()) <= 3.0 and float(whole.abs().max()) > 1.0      # the head's cap is at work
        runner.finish("a")
        runner.finish("b")
        got_a, got_b, at_a, at_b = [], [], 0, 0
        for na, nb in [(9, 3), (2, 0), (14, 6), (1, 1), (15, 8)]:
            ents = [StepEntry("a", a[at_a:at_a + na], list(range(na)))] if na else []
            if nb:
                ents.append(StepEntry("b", b[at_b:at_b + nb], list(range(nb))))
            l = runner.step(ents).cpu()
            got_a.append(l[:na])
            got_b.append(l[na:])
            at_a, at_b = at_a + na, at_b + nb
        tol = 1e-5 if dtype == "float32" else 2e-2
        assert rel_err(torch.cat(got_a), whole[:41]) < tol and rel_err(torch.cat(got_b), whole[41:]) < tol
        # the position encoding matters: a shift of the positions' angles changes the logits
        for layer in dec.layers:
            layer.mixer.position.cos, layer.mixer.position.sin = layer.mixer.position.sin, layer.mixer.position.cos
        runner.finish("a")
        runner.finish("b")
        assert rel_err(runner.step([StepEntry("c", a, list(range(41)))]).cpu(), whole[:41]) > 1e-3
    finally:
        FEED_FORWARDS.unregister("two_experts")
        POSITION_ENCODINGS.unregister("doubled_half_rotary")
        EMBEDDINGS.unregister("scaled_embedding")
        HEADS.unregister("capped_head")
        unregister_architecture("Toy2ForCausalLM")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_block_arrangement_and_norm(dtype):
    """Another arrangement of a layer's parts (one norm; mixer and feed-forward both read it and both
    add to the residual stream) and another norm (mean taken out, gain and bias), both defined here,
    in a toy architecture with interleaved rotary pairs and scaled positions.  Against a plain
    float64 model written here from the plain parts; whole, in portions, as captured steps, and in
    runs of chained decode steps through the entry point (every part says it may be captured)."""
    from tiny_llm_amd import Engine, SamplingParams
    from tiny_llm_amd.config import (EngineConfig, LayerSpec, ModelSpec, PartSpec, PlanEntry, register_architecture,
                                     resolve, unregister_architecture)
    from tiny_llm_amd.engine.loading import build_runner, random_model
    from tiny_llm_amd.engine.step import StepEntry
    from tiny_llm_amd.models.decoder import Decoder
    from tiny_llm_amd.parts import BLOCKS, NORMS, Block, Norm, WeightSpec, register_block, register_norm
    from tiny_llm_amd.weights.loader import random_tensor

    class CentredNorm(Norm):
        graph_safe = True           # device work only, nothing of the step read on the host

        def __init__(self, prefix, dtype, device, *, hidden_size, eps):
            super().__init__(prefix, dtype, device)
            self.H, self.eps = hidden_size, eps

        def weights(self):
            return [WeightSpec(f"{self.prefix}.gain", (self.H,), role="vector", init="around_one"),
                    WeightSpec(f"{self.prefix}.bias", (self.H,), role="vector")]

        def bind(self, tensors):
            self.gain, self.bias = tensors[f"{self.prefix}.gain"].float(), tensors[f"{self.prefix}.bias"].float()

        def forward(self, x, rows=None):
            if rows is not None:
                x = x[rows.long()]
            x = x.float()
            c = x - x.mean(dim=-1, keepdim=True)
            y = c * torch.rsqrt((c * c).mean(dim=-1, keepdim=True) + self.eps) * self.gain + self.bias
            return y.to(self.dtype).contiguous()

    class ParallelBlock(Block):
        roles = {"norm": "norm", "mixer": "mixer", "ffn": "feed_forward"}

        def forward(self, x, ctx, caches, states):
            p = self._parts
            h = p["norm"].forward(x)
            x = p["mixer"].forward(h, ctx, caches.get("mixer"), states.get("mixer"), x)
            return p["ffn"].forward(h, ctx, x)

    H, V, HD, NQ, NKV, I, EPS, THETA, FACTOR = 72, 131, 24, 4, 2, 104, 1e-5, 300.0, 2.0

    def build(cfg):
        norm = PartSpec("centred_norm", {"hidden_size": H, "eps": EPS})
        rope = {"kind": "rotary", "head_dim": HD, "theta": THETA, "max_position": 256, "pairing": "interleaved",
                "scaling": {"kind": "linear", "factor": FACTOR}}
        attn = PartSpec("attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV, "head_dim": HD, "position": rope})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I})
        layers = tuple(LayerSpec(f"blocks.{i}", "parallel", {"norm": norm.named("ln"), "mixer": attn.named("attn"),
                                                               "ffn": ffn.named("mlp")}) for i in range(2))
        sizes = {"vocab_size": V, "hidden_size": H}
        return ModelSpec("Toy4ForCausalLM", V, H, 256, PartSpec("token_embedding", sizes, "wte"), layers,
                         (PlanEntry(0), PlanEntry(1)), norm.named("ln_f"),
                         PartSpec("lm_head", dict(sizes, tied_to="wte"), "lm_head"))

    register_norm("centred_norm", CentredNorm)
    register_block("parallel", ParallelBlock)
    register_architecture("Toy4ForCausalLM", dict, build)
    try:
        raw = {"architectures": ["Toy4ForCausalLM"]}
        SEED, STD, NSTD = 3, 0.2, 0.1
        # the plain model, float64, from the plain parts and the weights by name
        _, spec = resolve(raw)
        w = {ws.name: random_tensor(ws, SEED, STD, NSTD).double() for ws in Decoder(spec, "float32", "cpu").weight_specs()
             if ws.alias_of is None}           # (the head is tied to the embedding table)
        assert sorted(w) == sorted(["wte.weight", "ln_f.gain", "ln_f.bias"] + [
            f"blocks.{i}.{n}" for i in range(2) for n in ("ln.gain", "ln.bias", "attn.q_proj.weight", "attn.k_proj.weight",
                                                          "attn.v_proj.weight", "attn.o_proj.weight", "mlp.gate_proj.weight",
                                                          "mlp.up_proj.weight", "mlp.down_proj.weight")])
        if dtype == "bfloat16":
            w = {k: (t.to(torch.bfloat16).double() if t.dim() == 2 else t) for k, t in w.items()}
        cos, sin = plain.rope_table_fast(256, HD, THETA, position_factor=FACTOR)

        def centred(x, pre):
            c = x - x.mean(dim=-1, keepdim=True)
            return c / torch.sqrt((c * c).mean(dim=-1, keepdim=True) + EPS) * w[f"{pre}.gain"] + w[f"{pre}.bias"]

        def reference(tokens):
            T = len(tokens)
            x = w["wte.weight"][list(tokens)]
            for i in range(2):
                pre = f"blocks.{i}"
                h = centred(x, f"{pre}.ln")
                q = plain.linear(h, w[f"{pre}.attn.q_proj.weight"]).reshape(T, NQ, HD)
                k = plain.linear(h, w[f"{pre}.attn.k_proj.weight"]).reshape(T, NKV, HD)
                v = plain.linear(h, w[f"{pre}.attn.v_proj.weight"]).reshape(T, NKV, HD)
                q, k = (plain.apply_rope_interleaved(t, range(T), cos, sin) for t in (q, k))
                a = plain.attention_fast(q, k, v, range(T)).reshape(T, NQ * HD)
                x = x + plain.linear(a, w[f"{pre}.attn.o_proj.weight"]) + plain.swiglu(
                    h, w[f"{pre}.mlp.gate_proj.weight"], w[f"{pre}.mlp.up_proj.weight"], w[f"{pre}.mlp.down_proj.weight"])
            return plain.linear(centred(x, "ln_f"), w["wte.weight"])

        a, b = random_tokens(70, V, 11), random_tokens(29, V, 12)
        ref_a, ref_b = reference(a), reference(b)
        tol = 1e-4 if dtype == "float32" else 3e-2      # bfloat16: the plain model here rounds nothing but the weights
        engine = EngineConfig(dtype=dtype, kv_block_size=8, max_cache_tokens=256, max_num_seqs=3,
                              max_num_batched_tokens=80, use_graphs=True)
        _, dec = random_model(raw, engine, seed=SEED, std=STD, norm_std=NSTD)
        assert dec.graph_safe
        runner = build_runner(dec, engine)
        for g in runner.cache.groups:
            for t in g.tensors.values():
                t.fill_(float("nan"))
        whole = runner.step([StepEntry("a", a, list(range(70)))]).cpu()
        assert rel_err(whole, ref_a) < tol
        runner.finish("a")
        for graphs in (False, True, True, True):
            got_a, got_b, at_a, at_b = [], [], 0, 0
            for na, nb in [(7, 2), (2, 0), (19, 11), (1, 1), (40, 14), (1, 1)]:
                ents = [StepEntry("a", a[at_a:at_a + na], list(range(na)))]
                if nb:
                    ents.append(StepEntry("b", b[at_b:at_b + nb], list(range(nb))))
                out = runner.step(ents, use_graph=graphs).cpu()
                got_a.append(out[:na])
                got_b.append(out[na:])
                at_a, at_b = at_a + na, at_b + nb
            assert at_a == 70 and at_b == 29
            assert rel_err(torch.cat(got_a), ref_a) < tol and rel_err(torch.cat(got_b), ref_b) < tol
            runner.finish("a")
            runner.finish("b")
        assert runner.graph_steps >= 8
        # through the entry point, with runs of chained decode steps: the plain model's greedy tokens
        eng = Engine(config=raw, dtype=dtype, weights_seed=SEED, init_std=STD, norm_std=NSTD, kv_block_size=8,
                     max_cache_tokens=256, max_num_seqs=3, max_num_batched_tokens=32, decode_burst=32)
        out = eng.generate([a[:20], b[:9]], SamplingParams.greedy(40, ignore_eos=True))
        assert any(g.bursts > 0 for g in eng.runner._graphs.values())
        for p, o in zip([a[:20], b[:9]], out):
            ref = reference(p + o)
            for k, tok in enumerate(o):
                row = ref[len(p) + k - 1]
                assert float(row.max() - row[tok]) <= 2 * tol * float(row.abs().max()), k
    finally:
        NORMS.unregister("centred_norm")
        BLOCKS.unregister("parallel")
        unregister_architecture("Toy4ForCausalLM")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_chained_decode_steps_with_several_cache_groups(dtype):
    """A toy architecture whose three attention layers keep caches of three kinds (every position;
    a window of 20; every position with other kv heads): three cache groups with pools of their own
    sizes.  Runs of decode steps chained on the device, in which the window group's blocks for a
    whole run are taken up front and given back behind it, give the tokens of single steps."""
    from tiny_llm_amd import Engine, SamplingParams
    from tiny_llm_amd.config import (ModelSpec, PartSpec, PlanEntry, pre_norm_layer, register_architecture,
                                     unregister_architecture)

    def build(cfg):
        H = cfg["hidden_size"]
        norm = PartSpec("rmsnorm", {"hidden_size": H, "eps": 1e-5})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 96})
        rope = {"kind": "rotary", "head_dim": 16, "theta": 1000.0, "max_position": 512}

        def attn(kv_heads, window=0):
            return PartSpec("attention", {"hidden_size": H, "num_heads": 4, "num_kv_heads": kv_heads, "head_dim": 16,
                                          "window": window, "position": rope})
        layers = tuple(pre_norm_layer(f"model.layers.{i}", norm, m, norm, ffn)
                       for i, m in enumerate([attn(2), attn(2, window=20), attn(1)]))
        sizes = {"vocab_size": cfg["vocab_size"], "hidden_size": H}
        return ModelSpec("Toy3ForCausalLM", cfg["vocab_size"], H, 512, PartSpec("token_embedding", sizes, "model.embed_tokens"),
                         layers, (PlanEntry(0), PlanEntry(1), PlanEntry(2)), norm.named("model.norm"),
                         PartSpec("lm_head", dict(sizes, tied_to="model.embed_tokens"), "lm_head"))

    register_architecture("Toy3ForCausalLM", dict, build)
    try:
        raw = {"architectures": ["Toy3ForCausalLM"], "hidden_size": 64, "vocab_size": 211}
        prompts = [random_tokens(n, 211, 40 + n) for n in (33, 5, 58)]
        sps = [SamplingParams.greedy(n, ignore_eos=True) for n in (90, 70, 41)]
        sps[1] = SamplingParams(max_new_tokens=70, temperature=0.8, top_k=30, top_p=0.9, seed=3, ignore_eos=True)
        outs = {}
        for burst in (1, 32):
            eng = Engine(config=raw, dtype=dtype, weights_seed=2, init_std=0.3, kv_block_size=8, max_num_seqs=3,
                         max_num_batched_tokens=64, max_cache_tokens=3 * 160, decode_burst=burst)
            cm = eng.runner.cache
            assert len(cm.groups) == 3 and cm.group_blocks[0] == 60 and cm.group_blocks[1] < 60 and cm.group_blocks[2] == 60
            poison(eng)
            outs[burst] = eng.generate(prompts, sps)
            cm.audit()
            assert cm.free_blocks() == cm.group_blocks
            if burst > 1:
                chained = [g for g in eng.runner._graphs.values() if g.bursts > 0]
                assert chained and all(g.feeds_next and g.chain is not None for g in chained)
        assert outs[32] == outs[1] and [len(o) for o in outs[1]] == [90, 70, 41]
    finally:
        unregister_architecture("Toy3ForCausalLM")
