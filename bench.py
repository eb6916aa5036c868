"""Decode and prefill throughput with random weights, on one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole serving path (scheduler, step function, sampling).  The
headline is the TinyLlama-1.1B shape in bfloat16 at batch 8 with 512-token prompts.  ONE JSON line is
printed: decoded tokens per second, the 2,048-token prefill (whole and in portions of 512), the HBM
roofline of the decode step, decode at batch 1 and 64, the time of a decode step and of the prefill by
kernel; the same in true float32; the machine's peaks
as measured on the spot (a streaming kernel, a loop of matrix instructions); and two soak workloads
at larger shapes (a mixed batch of 16 requests with prompts cut into portions of 512 at the
Llama-3-8B shape; 64 requests of 1,024 tokens that nearly fill the cache at the Llama-2-13B shape).
`--only` picks a part (for profiling), or one of the measurements that are not part of the line:
`attention` (the attention kernels alone at contexts up to 131,072 tokens), `long_context` (the Llama-3-8B
shape with 8 requests of 32,000 tokens and one of 131,000), `decode_shapes` (decode steps at the two larger
shapes by batch), `host` (a step's wall time against its time on the GPU).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}


def llama(layers, hidden, heads, kv_heads, inter, vocab, theta, max_pos):
    return {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": layers,
            "hidden_size": hidden, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
            "intermediate_size": inter, "vocab_size": vocab, "rope_theta": theta, "rms_norm_eps": 1e-5,
            "max_position_embeddings": max_pos, "tie_word_embeddings": False, "hidden_act": "silu",
            "attention_bias": False, "rope_scaling": None, "initializer_range": 0.02, "eos_token_id": 2}


TINYLLAMA = llama(22, 2048, 32, 4, 5632, 32000, 10000.0, 2048)       # the TinyLlama 1.1B shape
LLAMA3_8B = llama(32, 4096, 32, 8, 14336, 128256, 500000.0, 8192)
LLAMA2_13B = llama(40, 5120, 40, 40, 13824, 32000, 10000.0, 4096)
PROMPT_LEN = 512
PREFILL_TOKENS = 2048
ELT = {"bf16": 2, "fp32": 4}
TORCH_NAME = {"bf16": "bfloat16", "fp32": "float32"}


def model_numbers(cfg, elt_bytes):
    L, H, I, V = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = H // nq
    per_layer = (nq + 2 * nkv) * hd * H + H * nq * hd + 3 * I * H
    matmul_params = L * per_layer
    weight_bytes = (matmul_params + V * H + (2 * L + 1) * H) * elt_bytes      # every weight a step uses, once
    kv_bytes_per_token = L * 2 * nkv * hd * elt_bytes
    return matmul_params, weight_bytes, kv_bytes_per_token, (L, H, I, V, nq, nkv, hd)


def prefill_flops(cfg, tokens):
    matmul_params, _, _, (L, H, I, V, nq, nkv, hd) = model_numbers(cfg, 2)
    return 2.0 * tokens * matmul_params + L * nq * 2.0 * tokens * tokens * hd + 2.0 * V * H


def gen_tokens(n, vocab, seed):
    import torch
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# --------------------------------------------------------------- measured peaks
def measure_peaks():
    """GB/s of a streaming read and of a copy over 2 GiB, TFLOP/s of matrix-instruction loops."""
    import torch
    from tiny_llm_amd.kernels import ops
    dev = "cuda:0"
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    src = torch.ones(1 << 29, dtype=torch.float32, device=dev)       # 2 GiB: far beyond every cache
    dst = torch.empty_like(src)
    nbytes = src.numel() * 4

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    read = max(nbytes / timed(lambda: ops.peak_stream(src, None, sink, blocks), 5) for blocks in (2048, 4096, 8192))
    copy = max(2 * nbytes / timed(lambda: ops.peak_stream(src, dst, sink, blocks), 5) for blocks in (2048, 4096, 8192))
    del src, dst
    out = {"hbm_read_GBs": round(read / 1e9, 1), "hbm_copy_GBs": round(copy / 1e9, 1)}
    for name, dt in (("bf16", torch.bfloat16), ("fp32", torch.float32)):
        flops = ops.peak_mfma(sink, dt, 20000, 2048)
        t = timed(lambda: ops.peak_mfma(sink, dt, 20000, 2048), 3)
        out[f"mfma_{name}_TFLOPs"] = round(flops / t / 1e12, 1)
    # one all-to-all hand-over of a few floats among 256 resident workgroups inside a launch, and the
    # time of an empty launch that depends on the one before it in a graph: a decode layer has five
    # dependent phases, and either way a phase costs microseconds whatever it computes
    out["handover_in_kernel_us"] = round(ops.peak_handover(256, 2000, 16), 2)
    out["dependent_launch_us"] = round(dependent_launch_us(), 2)
    return out


def dependent_launch_us(n=200):
    """Microseconds per kernel of a captured chain of `n` tiny kernels, each depending on the one before."""
    import torch
    x = torch.zeros(64, device="cuda:0")
    for _ in range(3):
        x.add_(1.0)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(n):
            x.add_(1.0)
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (5 * n)


# ------------------------------------------------------------------- one model
class Bench:
    def __init__(self, cfg, dtype, max_batch, total_new, block_size, budget=4096, extra_tokens=PREFILL_TOKENS,
                 prompt_len=PROMPT_LEN, max_cache_tokens=None):
        import torch
        from tiny_llm_amd import Engine
        self.torch = torch
        self.cfg, self.dtype = cfg, dtype
        self.V = cfg["vocab_size"]
        blocks = (max_batch * (prompt_len + total_new) + extra_tokens) // block_size + max_batch + 8
        if max_cache_tokens is not None:
            blocks = max_cache_tokens // block_size
        self.engine = Engine(config=cfg, dtype=TORCH_NAME[dtype], kv_block_size=block_size, max_num_seqs=max_batch,
                             max_num_batched_tokens=budget, weights_seed=0, num_kv_blocks=blocks)
        self.sync = torch.cuda.synchronize

    def close(self):
        self.engine = None
        import gc
        gc.collect()
        self.torch.cuda.empty_cache()

    def decode(self, batch, steps, warmup, prompt_len=PROMPT_LEN):
        """Prefills `batch` prompts (untimed), then times `steps` decode steps.
        Returns (seconds, cached tokens read per step summed over the batch)."""
        from tiny_llm_amd import SamplingParams
        eng = self.engine
        # nobody ends inside the run: requests whose prompt is done decode while the others' prompts are
        # still computed, a token per step of that phase
        ahead = -(-batch * prompt_len // eng.scheduler.budget)
        params = SamplingParams.greedy(warmup + steps + 64 + ahead, ignore_eos=True)
        ids = [eng.add_request(gen_tokens(prompt_len, self.V, 1000 + i), params) for i in range(batch)]
        reqs = [eng.requests[i] for i in ids]
        while any(r.num_computed < prompt_len for r in reqs):
            eng.step()
        run0 = eng.steps_run
        while eng.steps_run - run0 < warmup:
            eng.step(max_decode_steps=warmup - (eng.steps_run - run0))
        ctx0 = sum(r.num_tokens for r in reqs)
        run0, out0 = eng.steps_run, sum(len(r.output) for r in reqs)
        self.sync()
        t0 = time.perf_counter()
        # exactly `steps` decode steps (the engine chains several of them on the device per call)
        while eng.steps_run - run0 < steps:
            eng.step(max_decode_steps=steps - (eng.steps_run - run0))
        self.sync()
        dt = time.perf_counter() - t0
        assert eng.steps_run - run0 == steps and sum(len(r.output) for r in reqs) - out0 == steps * batch
        ctx1 = sum(r.num_tokens for r in reqs)
        for i in ids:
            eng.abort(i)
        return dt, (ctx0 + ctx1) / 2.0

    def prefill(self, reps, tokens=PREFILL_TOKENS, budget=None):
        """Best of `reps` prefills of one prompt (after one untimed), its last logits sampled; with
        `budget` the prompt is cut into portions of that many tokens (one step each)."""
        from tiny_llm_amd import SamplingParams
        eng = self.engine
        old = eng.scheduler.budget
        if budget is not None:
            eng.scheduler.budget = budget
        times = []
        for r in range(reps + 1):
            rid = eng.add_request(gen_tokens(tokens, self.V, 77 + r), SamplingParams.greedy(1, ignore_eos=True))
            self.sync()
            t0 = time.perf_counter()
            while eng.requests[rid].status != "finished":
                eng.step()
            self.sync()
            times.append(time.perf_counter() - t0)
        eng.scheduler.budget = old
        return min(times[1:])

    def profile_decode(self, batch, prompt_len=PROMPT_LEN, steps=32):
        """Per-kernel times of a decode step (see kernel_breakdown): `steps` chained steps behind a warm-up."""
        from tiny_llm_amd import SamplingParams
        eng = self.engine
        params = SamplingParams.greedy(3 * steps + 64, ignore_eos=True)
        ids = [eng.add_request(gen_tokens(prompt_len, self.V, 1000 + i), params) for i in range(batch)]
        reqs = [eng.requests[i] for i in ids]
        while any(r.num_computed < prompt_len for r in reqs):
            eng.step()
        run0 = eng.steps_run
        while eng.steps_run - run0 < 2 * steps:             # the shape is captured, its chain of steps too
            eng.step()

        def run():
            at = eng.steps_run
            while eng.steps_run - at < steps:
                eng.step(max_decode_steps=steps - (eng.steps_run - at))
        out = kernel_breakdown(run, self.cfg["num_hidden_layers"])
        for i in ids:
            eng.abort(i)
        return out

    def profile_prefill(self, tokens=PREFILL_TOKENS):
        """Per-kernel times of one whole-prompt prefill step."""
        from tiny_llm_amd import SamplingParams
        eng = self.engine

        def once(seed):
            rid = eng.add_request(gen_tokens(tokens, self.V, seed), SamplingParams.greedy(1, ignore_eos=True))
            while eng.requests[rid].status != "finished":
                eng.step()
        once(91)
        once(92)
        return kernel_breakdown(lambda: once(93), self.cfg["num_hidden_layers"])

    def soak(self, prompt_lens, new_tokens, budget):
        """All requests at once through the scheduler: prompts in portions under `budget` tokens a
        step beside decoded tokens.  Returns (seconds, steps, preemptions)."""
        from tiny_llm_amd import SamplingParams
        eng = self.engine
        eng.scheduler.budget = budget
        ids = [eng.add_request(gen_tokens(n, self.V, 5000 + i), SamplingParams.greedy(new_tokens, ignore_eos=True))
               for i, n in enumerate(prompt_lens)]
        self.sync()
        steps = 0
        t0 = time.perf_counter()
        while eng.has_unfinished():
            eng.step()
            steps += 1
        self.sync()
        dt = time.perf_counter() - t0
        assert all(len(eng.requests[i].output) == new_tokens for i in ids)
        return dt, steps, sum(eng.requests[i].preemptions for i in ids)


def kernel_breakdown(run, layers):
    """Where a step's time goes, kernel by kernel: `run` executes steps of one kind (decode steps of one
    batch, or one prefill) under torch's profiler, which also sees the kernels of replayed graphs; what it
    reports for a kernel reaches from the end of the kernel before it to its own end, so the figures add up
    to the step.  The kernels of a step are told apart by their order around each layer's attention
    kernel: before the first one the q/k/v product; between two of them the o product, the gate/up
    product(s), the down product and the next layer's q/k/v product; behind the last one o, gate/up and
    down; rotation, the merge of attention's key splits and norms by their names; a product's second
    kernel (partial sums added up) counts with the product; then the output head, the sampler and, in
    chained decode steps, the kernel that prepares the next step.  Returns microseconds per step by part,
    summed over the layers."""
    import torch
    from torch.autograd import DeviceType
    from torch.profiler import ProfilerActivity, profile
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        run()
        torch.cuda.synchronize()
    evs = [e for e in prof.events() if e.device_type == DeviceType.CUDA and "emcpy" not in e.name and "emset" not in e.name]
    evs.sort(key=lambda e: e.time_range.start)
    starts = [i for i, e in enumerate(evs) if "embedding_kernel" in e.name]
    is_attention = lambda n: ("attn" in n or "attention" in n or "flash_prefill" in n) and "combine" not in n
    parts, n_steps = {}, 0
    for a, z in zip(starts, starts[1:] + [len(evs)]):
        step = evs[a:z]
        names = [e.name for e in step]
        dur = [e.time_range.end - e.time_range.start for e in step]
        # behind the layers: the head (a product, perhaps with a second kernel), sampler, the next step's metadata
        tail = len(step)
        while tail > 0 and ("sample_kernel" in names[tail - 1] or "decode_advance" in names[tail - 1]):
            tail -= 1
        head = tail - 1
        while head > 0 and "splitk_reduce" in names[head]:
            head -= 1
        body = list(range(1, head))
        att = [i for i in body if is_attention(names[i])]
        if layers <= 0 or len(att) != layers or head <= 0 or "gemm" not in names[head]:
            continue                                    # not a whole step (the profile began or ended inside one)
        n_steps += 1
        add = lambda k, v: parts.__setitem__(k, parts.get(k, 0.0) + v)
        add("embedding", dur[0])
        is_product = lambda i: "gemm" in names[i] and "splitk_reduce" not in names[i]
        last = None
        for i in body:
            n = names[i]
            if "splitk_reduce" in n and last is not None:
                add(last, dur[i])
            elif "rope_store" in n:
                add("rotation", dur[i])
            elif "combine" in n:
                add("attention_merge", dur[i])
            elif is_attention(n):
                add("attention", dur[i])
            elif is_product(i):
                seg = sum(1 for x in att if x < i)                  # attention kernels before this product
                lo = att[seg - 1] if seg else 0
                hi = att[seg] if seg < layers else head
                group = [x for x in body if lo < x < hi and is_product(x)]
                k = group.index(i)
                if seg == 0:
                    last = "qkv"
                elif seg < layers:
                    last = "o" if k == 0 else "qkv" if k == len(group) - 1 else "down" if k == len(group) - 2 else "gate_up"
                else:
                    last = "o" if k == 0 else "down" if k == len(group) - 1 else "gate_up"
                add(last, dur[i])
            elif "norm" in n:
                add("norm", dur[i])
            else:
                add("other", dur[i])
        for i in range(head, tail):
            add("lm_head", dur[i])
        for i in range(tail, len(step)):
            add("sample" if "sample_kernel" in names[i] else "next_step", dur[i])
    if not n_steps:
        return None
    out = {k: round(v / n_steps, 1) for k, v in parts.items()}
    out["sum"] = round(sum(parts.values()) / n_steps, 1)
    out["steps_seen"] = n_steps
    return out


def decode_rooflines(cfg, dtype, batch, seconds, ctx_tokens):
    """A decode step against both of its bounds: the bytes it has to read (every weight once, the cache of
    the live requests) over the published memory bandwidth, and its flops (two per weight and row, and the
    attention over the cached keys) over the published matrix peak of its element type.  `bound` names the
    one that allows less (float32 at batch 64 is bound by the float32 matrix peak, not by memory)."""
    matmul_params, weight_bytes, kv_per_tok, (L, H, I, V, nq, nkv, hd) = model_numbers(cfg, ELT[dtype])
    nbytes = weight_bytes + ctx_tokens * kv_per_tok
    flops = 2.0 * batch * (matmul_params + V * H) + 4.0 * L * nq * hd * ctx_tokens
    t_mem, t_flop = nbytes / (HBM_GBS * 1e9), flops / (PEAK_TFLOPS[dtype] * 1e12)
    return {"ms": round(seconds * 1e3, 4), "bound": "hbm" if t_mem >= t_flop else f"{dtype} matrix peak",
            "hbm_frac": round(t_mem / seconds, 4), "flops_frac": round(t_flop / seconds, 4),
            "GBs": round(nbytes / seconds / 1e9, 1), "TFLOPs": round(flops / seconds / 1e12, 2)}


def tinyllama_figures(args, dtype, peaks):
    """Decode at batch 8 / 1 / 64 and the 2,048-token prefill at the TinyLlama shape in `dtype`."""
    elt = ELT[dtype]
    cfg = dict(TINYLLAMA)
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    matmul_params, weight_bytes, kv_per_tok, (L, H, I, V, nq, nkv, hd) = model_numbers(cfg, elt)
    steps, warmup = args.steps, args.warmup
    if dtype == "fp32":
        steps, warmup = min(steps, 64), min(warmup, 8)       # the 32-bit path is for checking: a shorter run
    ahead = -(-max(args.batch, 64) * args.prompt_len // 4096)        # tokens decoded while other prompts are computed
    b = Bench(cfg, dtype, max(args.batch, 64), warmup + steps + 80 + ahead, args.block_size, prompt_len=args.prompt_len)
    out = {}
    if args.only in ("all", "headline", "fp32", "prefill"):
        pf = b.prefill(3)
        flops = prefill_flops(cfg, PREFILL_TOKENS)
        out["prefill"] = {"value": round(PREFILL_TOKENS / pf, 1), "tokens": PREFILL_TOKENS, "ms": round(pf * 1e3, 3),
                          "frac": round(flops / pf / (PEAK_TFLOPS[dtype] * 1e12), 4)}
        if peaks:
            out["prefill"]["frac_measured"] = round(flops / pf / (peaks[f"mfma_{dtype}_TFLOPs"] * 1e12), 4)
        pc = b.prefill(2, budget=512)
        out["prefill_chunked_512"] = {"value": round(PREFILL_TOKENS / pc, 1), "ms": round(pc * 1e3, 3), "steps": 4}
    if args.only != "prefill":
        dt, ctx_tokens = b.decode(args.batch, steps, warmup, prompt_len=args.prompt_len)
        out["ms_per_step"] = dt / steps * 1e3
        out["value"] = args.batch * steps / dt
        achieved = (weight_bytes + ctx_tokens * kv_per_tok) / (dt / steps) / 1e9
        out["roofline"] = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                           "frac": round(achieved / HBM_GBS, 4)}
        if peaks:
            out["roofline"]["frac_measured"] = round(achieved / peaks["hbm_read_GBs"], 4)
        if args.only in ("all", "headline", "fp32", "kernels"):
            out["kernels_us"] = {"decode": b.profile_decode(args.batch, prompt_len=args.prompt_len),
                                 "prefill": b.profile_prefill()}
        out["points"] = {}
        if args.only in ("all", "headline", "fp32"):
            for n in (1, 64):
                d, ctx_n = b.decode(n, steps, warmup, prompt_len=args.prompt_len)
                out["points"][f"decode_b{n}"] = round(n * steps / d, 1)
                out[f"roofline_b{n}"] = decode_rooflines(cfg, dtype, n, d / steps, ctx_n)
    out["sizes"] = (L, H, I, V, nq, nkv, hd)
    out["steps"], out["warmup"] = steps, warmup
    b.close()
    return out


def soak_llama3_8b(args, dtype="bf16"):
    """16 requests, seeded prompt lengths 128..4096, prompts in portions of 512, 128 tokens each.
    bfloat16: three passes, the third counts; float32 (the checking path): one pass."""
    import random
    cfg = dict(LLAMA3_8B)
    layers_full = cfg["num_hidden_layers"]
    if args.soak_layers:
        cfg["num_hidden_layers"] = min(layers_full, args.soak_layers)
    rng = random.Random(8)
    lens = [rng.randint(128, 4096) for _ in range(16)]
    new = 128
    b = Bench(cfg, dtype, 16, new, 16, budget=512, max_cache_tokens=sum(-(-(n + new) // 16) * 16 for n in lens) + 1024)
    b.soak(lens[:2], 4, 512)                                  # warm-up: kernels configure themselves
    # The workload three times over: the first pass meets every shape of step for the first time (a
    # shape's first step runs eagerly, its second is captured as a graph), the third replays graphs
    # only and is the one that counts; the first is reported beside it.
    cold, steps, pre = b.soak(lens, new, 512)
    dt, passes = cold, 1
    if dtype == "bf16":
        b.soak(lens, new, 512)
        dt, steps, pre = b.soak(lens, new, 512)
        passes = 3
    b.close()
    total = sum(lens) + 16 * new
    return {"model": "Llama-3-8B shape", "dtype": dtype, "layers": cfg["num_hidden_layers"], "layers_full": layers_full,
            "requests": 16, "prompt_tokens": sum(lens), "decode_tokens": 16 * new, "chunk": 512, "steps": steps,
            "seconds": round(dt, 3), "tokens_per_s": round(total / dt, 1), "decode_tokens_per_s": round(16 * new / dt, 1),
            "preemptions": pre, "pass": passes, "first_pass_seconds": round(cold, 3)}


def long_context_llama3_8b(args):
    """The Llama-3-8B shape far beyond its own context: 8 requests of 32,000 tokens and one of 131,000,
    prompts in portions of 2,048, then decode steps; what a step reads (weights and the live
    requests' keys and values) over its time."""
    import torch
    from tiny_llm_amd import SamplingParams
    cfg = dict(LLAMA3_8B, max_position_embeddings=140000)
    layers_full = cfg["num_hidden_layers"]
    if args.soak_layers:
        cfg["num_hidden_layers"] = min(layers_full, args.soak_layers)
    out = {"model": "Llama-3-8B shape", "dtype": "bf16", "layers": cfg["num_hidden_layers"], "layers_full": layers_full,
           "chunk": 2048}
    for batch, prompt in ((8, 32000), (1, 131000)):
        b = Bench(cfg, "bf16", batch, 512, 16, budget=2048, prompt_len=prompt)
        eng = b.engine
        params = SamplingParams.greedy(400, ignore_eos=True)            # nobody ends inside the run
        b.sync()
        t0 = time.perf_counter()
        ids = [eng.add_request(gen_tokens(prompt, b.V, 1000 + i), params) for i in range(batch)]
        reqs = [eng.requests[i] for i in ids]
        steps = 0
        while any(r.num_computed < prompt for r in reqs):
            eng.step()
            steps += 1
        b.sync()
        t1 = time.perf_counter()
        run0 = eng.steps_run
        while eng.steps_run - run0 < 8:
            eng.step(max_decode_steps=8)
        b.sync()
        t2, run0 = time.perf_counter(), eng.steps_run
        while eng.steps_run - run0 < 32:
            eng.step(max_decode_steps=32 - (eng.steps_run - run0))
        b.sync()
        ms = (time.perf_counter() - t2) / 32 * 1e3
        assert len(eng.scheduler.running) == batch
        _, weight_bytes, kv_per_token, _ = model_numbers(cfg, ELT["bf16"])
        nbytes = weight_bytes + sum(r.num_tokens for r in reqs) * kv_per_token
        out[f"batch{batch}_context{prompt}"] = {
            "prefill_steps": steps, "prefill_tok_s": round(batch * prompt / (t1 - t0), 1), "decode_ms": round(ms, 3),
            "decode_tok_s": round(batch / ms * 1e3, 1), "GB_a_step": round(nbytes / 1e9, 1),
            "GBs": round(nbytes / ms / 1e6, 1), "hbm_frac": round(nbytes / ms / 1e6 / HBM_GBS, 3)}
        for i in ids:
            eng.abort(i)
        b.close()
    return out


def decode_larger_shapes(args):
    """Decode steps at the Llama-3-8B and Llama-2-13B shapes, 512-token prompts, by batch: a step's time
    against the bytes it has to read."""
    out = {}
    for name, shape in (("llama3_8b", LLAMA3_8B), ("llama2_13b", LLAMA2_13B)):
        cfg = dict(shape)
        if args.soak_layers:
            cfg["num_hidden_layers"] = min(cfg["num_hidden_layers"], args.soak_layers)
        b = Bench(cfg, "bf16", 64, 160, 16, budget=4096)
        out[name] = {"layers": cfg["num_hidden_layers"], "layers_full": shape["num_hidden_layers"]}
        for batch in (1, 8, 16, 32, 64):
            dt, ctx = b.decode(batch, 64, 8)
            r = decode_rooflines(cfg, "bf16", batch, dt / 64, ctx)
            out[name][f"batch{batch}"] = {"ms": r["ms"], "tok_s": round(batch * 64 / dt, 1), "GBs": r["GBs"],
                                         "hbm_frac": r["hbm_frac"]}
            print(f"# {name} batch {batch:2d}: {dt / 64 * 1e3:7.3f} ms a step, {r['GBs']:7.1f} GB/s ({r['hbm_frac']:.3f} of "
                  f"{HBM_GBS / 1e3:.0f} TB/s)", file=sys.stderr, flush=True)
        b.close()
    return out


def prefill_llama3_8b(args):
    """Whole prompts of 4,096 and 8,192 tokens at the Llama-3-8B shape, one step each."""
    cfg = dict(LLAMA3_8B)
    layers_full = cfg["num_hidden_layers"]
    if args.soak_layers:
        cfg["num_hidden_layers"] = min(layers_full, args.soak_layers)
    b = Bench(cfg, "bf16", 1, 1, 16, budget=8192, max_cache_tokens=8192 + 256)
    out = {"model": "Llama-3-8B shape", "dtype": "bf16", "layers": cfg["num_hidden_layers"], "layers_full": layers_full}
    for tokens in (4096, 8192):
        dt = b.prefill(2, tokens=tokens, budget=tokens)
        out[f"tokens_{tokens}"] = {"ms": round(dt * 1e3, 2), "value": round(tokens / dt, 1),
                                   "frac": round(prefill_flops(cfg, tokens) / dt / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    b.close()
    return out


def soak_llama2_13b(args, dtype="bf16"):
    """64 requests of 1,024 prompt tokens, 256 greedy tokens each; the cache pool holds them with little to spare.
    bfloat16: three passes, the third counts; float32 (the checking path): one pass."""
    cfg = dict(LLAMA2_13B)
    layers_full = cfg["num_hidden_layers"]
    if args.soak_layers:
        cfg["num_hidden_layers"] = min(layers_full, args.soak_layers)
    n_req, prompt, new = 64, 1024, 256
    pool_tokens = n_req * (prompt + new) + 64 * 16           # one spare page a request
    b = Bench(cfg, dtype, n_req, new, 16, budget=2048, max_cache_tokens=pool_tokens)
    b.soak([prompt] * 2, 4, 2048)
    cold, steps, pre = b.soak([prompt] * n_req, new, 2048)    # three passes, as above
    dt, passes = cold, 1
    if dtype == "bf16":
        b.soak([prompt] * n_req, new, 2048)
        dt, steps, pre = b.soak([prompt] * n_req, new, 2048)
        passes = 3
    _, _, kv_per_tok, _ = model_numbers(cfg, ELT[dtype])
    b.close()
    return {"model": "Llama-2-13B shape", "dtype": dtype, "layers": cfg["num_hidden_layers"], "layers_full": layers_full,
            "requests": n_req, "prompt_tokens": n_req * prompt, "decode_tokens": n_req * new, "steps": steps,
            "seconds": round(dt, 3), "tokens_per_s": round(n_req * (prompt + new) / dt, 1),
            "decode_tokens_per_s": round(n_req * new / dt, 1), "preemptions": pre, "pass": passes,
            "first_pass_seconds": round(cold, 3),
            "cache_pool_GB": round(pool_tokens * kv_per_tok / 1e9, 1), "cache_pool_fill": round(n_req * (prompt + new) / pool_tokens, 3)}


def host_time(args):
    """Wall time of a step against the time its captured graph takes on the GPU (events around every
    replay): decode at batch 64, 8 and 1, and mixed steps of 64 tokens (8 decoded tokens beside 56 of a
    prompt).  What is left is the host's share: scheduling, metadata, upload, download."""
    import torch
    from tiny_llm_amd import SamplingParams
    spans = []
    replay = torch.cuda.CUDAGraph.replay

    def timed(self):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        replay(self)
        e1.record()
        spans.append((e0, e1))

    torch.cuda.CUDAGraph.replay = timed
    out = {}
    try:
        b = Bench(dict(TINYLLAMA), "bf16", 64, 400, args.block_size, budget=4096)
        eng = b.engine
        for batch in (64, 8, 1):
            ids = [eng.add_request(gen_tokens(PROMPT_LEN, b.V, 1000 + i), SamplingParams.greedy(300, ignore_eos=True))
                   for i in range(batch)]
            reqs = [eng.requests[i] for i in ids]
            while any(r.num_computed < PROMPT_LEN for r in reqs):
                eng.step()
            for _ in range(4):
                eng.step()
            spans.clear()
            run0 = eng.steps_run
            b.sync()
            t0 = time.perf_counter()
            while eng.steps_run - run0 < 128:
                eng.step(max_decode_steps=128 - (eng.steps_run - run0))
            b.sync()
            wall = (time.perf_counter() - t0) / 128 * 1e3
            gpu = sum(a.elapsed_time(c) for a, c in spans) / 128        # a replay may hold several steps
            out[f"decode_b{batch}"] = {"wall_ms": round(wall, 4), "gpu_ms": round(gpu, 4), "host_ms": round(wall - gpu, 4),
                                       "steps_per_call": eng.engine_config.decode_burst}
            for i in ids:
                eng.abort(i)
        eng.scheduler.budget = 64
        ids = [eng.add_request(gen_tokens(100, b.V, 2000 + i), SamplingParams.greedy(400, ignore_eos=True)) for i in range(8)]
        while any(eng.requests[i].num_computed < 100 for i in ids):
            eng.step()
        for trial in range(2):          # the first pass captures the graphs of these shapes of step, the second is timed
            long_id = eng.add_request(gen_tokens(1800, b.V, 77 + trial), SamplingParams.greedy(2, ignore_eos=True))
            for _ in range(4):
                eng.step()
            spans.clear()
            b.sync()
            t0 = time.perf_counter()
            n = 0
            while eng.requests[long_id].num_computed < 1700:
                eng.step()
                n += 1
            b.sync()
            wall = (time.perf_counter() - t0) / n * 1e3
            gpu = sum(a.elapsed_time(c) for a, c in spans) / max(1, len(spans))
            eng.abort(long_id)
        out["mixed_64_tokens"] = {"wall_ms": round(wall, 4), "gpu_ms": round(gpu, 4), "ratio": round(wall / gpu, 3), "steps": n}
        b.close()
    finally:
        torch.cuda.CUDAGraph.replay = replay
    return out


def attention_sweep():
    """The attention kernels alone at contexts and batches the model runs do not reach, with the key
    splits the engine would choose.  Decode (rotation and cache write inside, merge kernel included):
    microseconds a call and the bytes of the keys and values it reads per second.  Prompts, whole and
    512 tokens at the end of a long context: microseconds and the flops of the two products per second."""
    import torch
    from tiny_llm_amd.kernels import ops
    dev, page = "cuda:0", 16
    rows = []
    for name, nq, nkv, hd in (("tinyllama", 32, 4, 64), ("llama3_8b", 32, 8, 128), ("llama2_13b", 40, 40, 128)):
        for batch in (1, 8, 64):
            for ctx in (2048, 8192, 32768, 131072):
                pages = -(-ctx // page)
                nbytes = batch * ctx * nkv * hd * 2 * 2
                if nbytes > 48e9:
                    continue
                kc = torch.randn(batch * pages + 1, nkv, page, hd, device=dev, dtype=torch.bfloat16)
                vc = torch.randn_like(kc)
                table = (torch.randperm(batch * pages, device=dev).to(torch.int32) + 1).view(batch, pages).contiguous()
                pos = torch.full((batch,), ctx - 1, device=dev, dtype=torch.int32)
                qkv = torch.randn(batch, (nq + 2 * nkv) * hd, device=dev, dtype=torch.bfloat16)
                out = torch.empty(batch, nq * hd, device=dev, dtype=torch.bfloat16)
                cos, sin = torch.randn(ctx + 8, hd // 2, device=dev), torch.randn(ctx + 8, hd // 2, device=dev)
                splits = ops.decode_key_splits(batch, ctx, nkv, hd)
                scratch = torch.empty(splits * batch * nq * (hd + 2), device=dev) if splits > 1 else None

                def call():
                    ops.flash_attention(qkv[:, :nq * hd], kc, vc, table, None, pos, out, nq, nkv, hd, hd ** -0.5, 0, splits,
                                        scratch, fused_rope=(cos, sin))
                for _ in range(2):
                    call()
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for _ in range(8):
                        call()
                g.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(3):
                    g.replay()
                e1.record()
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / 24
                rows.append({"heads": name, "batch": batch, "context": ctx, "splits": splits, "us": round(us, 1),
                             "GBs": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_GBS, 3)})
                print(f"# {name:10s} batch {batch:3d} context {ctx:6d}: {splits:2d} splits {us:8.1f} us "
                      f"{nbytes / us / 1e6:6.2f} TB/s", file=sys.stderr, flush=True)
                del kc, vc
    # prompt portions: whole prompts, and 512 tokens at the end of a long context
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for name, nq, nkv, hd in (("tinyllama", 32, 4, 64), ("llama3_8b", 32, 8, 128)):
        for ctx, new in ((8192, 8192), (32768, 32768), (8192, 512), (32768, 512), (131072, 512)):
            pages = -(-ctx // page)
            kc = torch.randn(pages + 1, nkv, page, hd, device=dev, dtype=torch.bfloat16)
            vc = torch.randn_like(kc)
            table = (torch.randperm(pages, device=dev).to(torch.int32) + 1).view(1, pages).contiguous()
            q = torch.randn(new, nq * hd, device=dev, dtype=torch.bfloat16)
            out = torch.empty_like(q)
            pos = torch.arange(ctx - new, ctx, device=dev, dtype=torch.int32)
            waves = ops.prefill_tile_waves(new, nq, nkv)
            per = (16 // (nq // nkv)) * waves                       # tokens of a query tile group
            starts = list(range(0, new, per))
            tiles = (i32([0] * len(starts)), i32(starts), i32([min(per, new - t) for t in starts]))
            splits = ops.prefill_key_splits(new, ctx, nq, nkv, waves)
            scratch = torch.empty(max(1, splits * new * nq * (hd + 2)), device=dev)

            def call():
                ops.flash_prefill(q, kc, vc, table, tiles, pos, out, nq, nkv, hd, hd ** -0.5, 0, waves, splits, scratch)
            call()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                call()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 3
            flops = 4.0 * sum(range(ctx - new + 1, ctx + 1)) * nq * hd      # row p sees p + 1 keys; two products
            rows.append({"heads": name, "prompt_rows": new, "context": ctx, "splits": splits, "us": round(us, 1),
                         "TFLOPs": round(flops / us / 1e6, 1), "frac": round(flops / us / 1e6 / PEAK_TFLOPS["bf16"], 3)})
            print(f"# {name:10s} {new:5d} prompt tokens ending at {ctx:6d}: {splits} splits {us:9.1f} us "
                  f"{flops / us / 1e6:6.1f} TFLOP/s", file=sys.stderr, flush=True)
            del kc, vc
    return rows


def run(args):
    if args.only == "attention":
        print(json.dumps({"decode_attention": attention_sweep()}), flush=True)
        return
    if args.only == "host":
        print(json.dumps({"host_time": host_time(args)}), flush=True)
        return
    peaks = measure_peaks() if args.only in ("all", "peaks", "headline", "fp32") else None
    if args.only == "peaks":
        print(json.dumps({"measured_peaks": peaks}), flush=True)
        return
    if args.only == "decode_shapes":
        print(json.dumps({"decode_larger_shapes": decode_larger_shapes(args)}), flush=True)
        return
    if args.only == "long_context":
        print(json.dumps({"llama3_8b_long_context": long_context_llama3_8b(args)}), flush=True)
        return
    if args.only in ("llama3_8b", "llama2_13b", "llama3_8b_prefill"):
        fn = {"llama3_8b": soak_llama3_8b, "llama2_13b": soak_llama2_13b, "llama3_8b_prefill": prefill_llama3_8b}[args.only]
        res = fn(args) if args.only == "llama3_8b_prefill" else fn(args, args.dtype)
        print(json.dumps({args.only: res}), flush=True)
        return
    main_dtype = "fp32" if args.only == "fp32" else args.dtype
    fig = tinyllama_figures(args, main_dtype, peaks)
    if args.only == "prefill":
        print(json.dumps({"prefill_tok_s": fig["prefill"]["value"], "ms": fig["prefill"]["ms"],
                          "chunked_512": fig["prefill_chunked_512"]}), flush=True)
        return
    L, H, I, V, nq, nkv, hd = fig["sizes"]
    line = {
        "metric": "decode tok/s at batch 8, TinyLlama 1.1B shape (prefill tok/s at 2,048 tokens and batch 1/64 beside it)",
        "value": round(fig["value"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": fig["steps"], "warmup": fig["warmup"],
        "ms_per_step": round(fig["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_dtype, "data": "synthetic: uniform-random token ids, random weights N(0, 0.02)",
        "config": {"model": "TinyLlama-1.1B shape", "layers": L, "layers_full": TINYLLAMA["num_hidden_layers"], "hidden": H,
                   "heads": nq, "kv_heads": nkv, "head_dim": hd, "intermediate": I, "vocab": V,
                   "context": TINYLLAMA["max_position_embeddings"], "global_batch": args.batch, "seq_len": args.prompt_len,
                   "decode_tokens": fig["steps"], "kv_block_size": args.block_size, "parallelism": "single GPU"},
        "prefill": fig.get("prefill"), "roofline": fig["roofline"], "points": fig["points"],
    }
    for n in (1, 64):
        if f"roofline_b{n}" in fig:
            line[f"roofline_b{n}"] = fig[f"roofline_b{n}"]
    if "prefill_chunked_512" in fig:
        line["prefill_chunked_512"] = fig["prefill_chunked_512"]
    if "kernels_us" in fig:
        line["kernels_us"] = fig["kernels_us"]
    if peaks:
        line["measured_peaks"] = peaks
    if args.only == "all":
        f32 = tinyllama_figures(args, "fp32", peaks)
        line["fp32"] = {"decode_b8": round(f32["value"], 1), "ms_per_step_b8": round(f32["ms_per_step"], 4),
                        "decode_b1": f32["points"]["decode_b1"], "decode_b64": f32["points"]["decode_b64"],
                        "steps": f32["steps"], "prefill": f32["prefill"], "prefill_chunked_512": f32["prefill_chunked_512"],
                        "roofline_b8": f32["roofline"], "roofline_b1": f32["roofline_b1"], "roofline_b64": f32["roofline_b64"],
                        "kernels_us": f32.get("kernels_us")}
        line["workloads"] = {"llama3_8b_mixed16": soak_llama3_8b(args), "llama3_8b_prefill": prefill_llama3_8b(args),
                             "llama2_13b_64x1024": soak_llama2_13b(args),
                             "llama3_8b_mixed16_fp32": soak_llama3_8b(args, "fp32"),
                             "llama2_13b_64x1024_fp32": soak_llama2_13b(args, "fp32")}
    print(json.dumps(line), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)      # with the warm-up: 256 generated tokens a request
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN, help="prompt tokens of the decode runs (the context they begin at)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the TinyLlama shape has (0: all)")
    ap.add_argument("--soak-layers", type=int, default=0, help="fewer layers for the two larger shapes (0: all)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--only", default="all",
                    choices=["all", "headline", "decode", "prefill", "fp32", "kernels", "peaks", "llama3_8b", "llama3_8b_prefill", "llama2_13b", "host",
                             "attention", "long_context", "decode_shapes"],
                    help="all: everything in one line; headline: the bfloat16 TinyLlama figures only; decode / prefill: "
                         "one of them (profiling); fp32: the float32 figures as the headline; kernels: decode with the time of "
                         "a step by kernel (torch's profiler); peaks / llama3_8b / "
                         "llama2_13b: that part alone; host: a step's wall time against its time on the GPU; attention: the "
                         "attention kernels alone at contexts up to 131,072 tokens; long_context: the Llama-3-8B shape with "
                         "8 requests of 32,000 tokens and one of 131,000; decode_shapes: decode steps at the two larger shapes by batch")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for {args.gpus})")
        return 2
    run(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
