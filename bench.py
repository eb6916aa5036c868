"""Decode and prefill throughput of the TinyLlama-1.1B shape with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole serving path (scheduler, step function, sampling)
at batch 8 with 512-token prompts.  One JSON line is printed: decoded tokens per second,
the 2,048-token prefill, the HBM roofline of the decode step, and decode at batch 1 and 64.
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

# the TinyLlama 1.1B shape
TINYLLAMA = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 22, "hidden_size": 2048,
    "num_attention_heads": 32, "num_key_value_heads": 4, "intermediate_size": 5632, "vocab_size": 32000,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 2048, "tie_word_embeddings": False,
    "hidden_act": "silu", "attention_bias": False, "rope_scaling": None, "initializer_range": 0.02,
    "eos_token_id": 2,
}
PROMPT_LEN = 512
PREFILL_TOKENS = 2048


def model_numbers(cfg, elt_bytes):
    L, H, I, V = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = H // nq
    per_layer = (nq + 2 * nkv) * hd * H + H * nq * hd + 3 * I * H
    matmul_params = L * per_layer
    weight_bytes = (matmul_params + V * H + (2 * L + 1) * H) * elt_bytes      # every weight a step uses, once
    kv_bytes_per_token = L * 2 * nkv * hd * elt_bytes
    return matmul_params, weight_bytes, kv_bytes_per_token, (L, H, I, V, nq, nkv, hd)


def run(args):
    import torch
    from tiny_llm_amd import Engine, SamplingParams

    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    elt = 2 if args.dtype == "bf16" else 4
    cfg = dict(TINYLLAMA)
    layers_full = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    matmul_params, weight_bytes, kv_per_tok, (L, H, I, V, nq, nkv, hd) = model_numbers(cfg, elt)

    def gen_tokens(n, seed):
        g = torch.Generator().manual_seed(seed)
        return torch.randint(0, V, (n,), generator=g).tolist()

    total_new = args.warmup + args.steps + 1
    max_batch = max(args.batch, 64)
    engine = Engine(config=cfg, dtype=dtype, kv_block_size=args.block_size, max_num_seqs=max_batch,
                    max_num_batched_tokens=max(PREFILL_TOKENS, 4096), weights_seed=0,
                    num_kv_blocks=(max_batch * (PROMPT_LEN + total_new) + PREFILL_TOKENS) // args.block_size + max_batch + 8)
    sync = torch.cuda.synchronize

    def decode_run(batch, steps, warmup):
        """Prefills `batch` prompts (untimed), then times `steps` decode steps."""
        params = SamplingParams.greedy(warmup + steps + 1, ignore_eos=True)
        ids = [engine.add_request(gen_tokens(PROMPT_LEN, 1000 + i), params) for i in range(batch)]
        while any(engine.requests[i].num_computed < PROMPT_LEN for i in ids):
            engine.step()
        for _ in range(warmup):
            engine.step()
        ctx0 = sum(engine.requests[i].num_tokens for i in ids)
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            engine.step()
        sync()
        dt = time.perf_counter() - t0
        ctx1 = sum(engine.requests[i].num_tokens for i in ids)
        for i in ids:
            engine.abort(i)
        avg_ctx_tokens = (ctx0 + ctx1) / 2.0          # cached tokens read per step, summed over the batch
        return dt, avg_ctx_tokens

    def prefill_run(reps):
        times = []
        for r in range(reps + 1):
            rid = engine.add_request(gen_tokens(PREFILL_TOKENS, 77 + r), SamplingParams.greedy(1, ignore_eos=True))
            sync()
            t0 = time.perf_counter()
            engine.step()
            sync()
            times.append(time.perf_counter() - t0)
            assert engine.requests[rid].status == "finished"
        return min(times[1:])

    # prefill of one 2,048-token prompt in one step, its last logits sampled
    pf_tokens = PREFILL_TOKENS
    pf_s = prefill_run(3) if args.only in ("all", "prefill") else float("nan")
    if args.only == "prefill":
        print(json.dumps({"prefill_tok_s": round(pf_tokens / pf_s, 1), "ms": round(pf_s * 1e3, 3)}), flush=True)
        return
    pf_flops = 2.0 * pf_tokens * matmul_params + L * nq * 2.0 * pf_tokens * pf_tokens * hd + 2.0 * V * H
    pf_frac = pf_flops / pf_s / (PEAK_TFLOPS[args.dtype] * 1e12)

    dt, ctx_tokens = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    bytes_per_step = weight_bytes + ctx_tokens * kv_per_tok
    achieved = bytes_per_step / (dt / args.steps) / 1e9

    points = {}
    for b in ((1, 64) if args.only == "all" else ()):
        d, _ = decode_run(b, args.steps, args.warmup)
        points[f"decode_b{b}"] = round(b * args.steps / d, 1)

    line = {
        "metric": "decode tok/s at batch 8, TinyLlama 1.1B shape (prefill tok/s at 2,048 tokens and batch 1/64 beside it)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: uniform-random token ids, random weights N(0, 0.02)",
        "config": {"model": "TinyLlama-1.1B shape", "layers": L, "layers_full": layers_full, "hidden": H,
                   "heads": nq, "kv_heads": nkv, "head_dim": hd, "intermediate": I, "vocab": V,
                   "context": cfg["max_position_embeddings"], "global_batch": args.batch, "seq_len": PROMPT_LEN,
                   "decode_tokens": args.steps, "kv_block_size": args.block_size, "parallelism": "single GPU"},
        "prefill": {"value": round(pf_tokens / pf_s, 1), "tokens": pf_tokens, "ms": round(pf_s * 1e3, 3),
                    "frac": round(pf_frac, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": points,
    }
    print(json.dumps(line), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)      # with the warm-up: 256 generated tokens a request
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0: all)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--only", default="all", choices=["all", "decode", "prefill"],
                    help="profiling aid: time only the decode batch or only the prefill")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for {args.gpus})")
        return 2
    run(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
