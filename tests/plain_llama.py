"""A plain, slow Llama: whole sequences, no cache, one function per part.

Written from the reference's formulas (each function cites file:line, relative to the
reference's checkout); it shares no code with the engine.  Everything is computed in
float64 by default so that it can serve as the truth for the float32 engine;
`act_dtype=torch.bfloat16` rounds activations at the places where the serving
path stores bfloat16, which makes the comparison with that path tight.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


def _rnd(x: torch.Tensor, act_dtype) -> torch.Tensor:
    return x if act_dtype is None else x.to(act_dtype).to(x.dtype)


# ------------------------------------------------------------------------- parts
def embedding(tokens: Sequence[int], table: torch.Tensor) -> torch.Tensor:
    """x[t, :] = E[token_ids[t], :], a pure gather without scale
    (tiny_llm/ops/cuda/embedding.cu:10-29)."""
    return torch.stack([table[int(t)] for t in tokens]).to(F64)


def rope_table(max_len: int, dim: int, base: float):
    """theta = p * base^(-i / (dim/2)) in double, cos/sin rounded to float
    (tiny_llm/ops/cuda/rope.cu:12-24).  Returns float64 copies of the float32 tables
    [max_len, dim/2]."""
    half = dim // 2
    cos = torch.empty(max_len, half, dtype=F64)
    sin = torch.empty(max_len, half, dtype=F64)
    for p in range(max_len):
        for i in range(half):
            th = float(p) * math.pow(base, -float(i) / float(half))
            cos[p, i] = math.cos(th)
            sin[p, i] = math.sin(th)
    return cos.to(torch.float32).to(F64), sin.to(torch.float32).to(F64)


def rope_table_fast(max_len: int, dim: int, base: float, position_factor: float = 1.0):
    """Same table as `rope_table`, vectorised (used for long sequences).  `position_factor`
    divides the positions first (linear scaling of positions; the reference has none: 1)."""
    half = dim // 2
    inv = torch.tensor([math.pow(base, -float(i) / float(half)) for i in range(half)], dtype=F64)
    ang = (torch.arange(max_len, dtype=F64) / position_factor)[:, None] * inv[None, :]
    return torch.cos(ang).to(torch.float32).to(F64), torch.sin(ang).to(torch.float32).to(F64)


def apply_rope(x: torch.Tensor, positions: Sequence[int], cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x: [T, heads, hd].  Rotate-half pairing: a = x[i], b = x[i + hd/2];
    x[i] = cos*a - sin*b; x[i + hd/2] = sin*a + cos*b (tiny_llm/ops/cuda/rope.cu:46-54)."""
    T, nh, hd = x.shape
    half = hd // 2
    out = x.clone()
    for t in range(T):
        c, s = cos[int(positions[t])], sin[int(positions[t])]
        a, b = x[t, :, :half], x[t, :, half:]
        out[t, :, :half] = c * a - s * b
        out[t, :, half:] = s * a + c * b
    return out


def apply_rope_interleaved(x: torch.Tensor, positions: Sequence[int], cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """The other usual pairing, which the reference does not have: pair i is (x[2i], x[2i + 1]),
    rotated by the same angles as pair i of `apply_rope`.  Equal to `apply_rope` on a head whose
    dims are permuted so that the even ones come first (tested)."""
    T, nh, hd = x.shape
    out = x.clone()
    for t in range(T):
        c, s = cos[int(positions[t])], sin[int(positions[t])]
        a, b = x[t, :, 0::2], x[t, :, 1::2]
        out[t, :, 0::2] = c * a - s * b
        out[t, :, 1::2] = s * a + c * b
    return out


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """s = sum_j x_j^2 / H; r = sqrt(s + eps); y_j = (w_j * x_j) / r
    (tiny_llm/ops/cuda/norm.cu:29-48)."""
    H = x.shape[-1]
    s = (x * x / H).sum(dim=-1, keepdim=True)
    r = torch.sqrt(s + eps)
    return (w.to(x.dtype) * x) / r


def linear(x: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
    """dst[m, n] = sum_k in[m, k] * W[n, k] (tiny_llm/ops/cuda/gemm.cu:86-100)."""
    return x @ W.to(x.dtype).T


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)) (tiny_llm/ops/cuda/silu.cu:10)."""
    return x / (1.0 + torch.exp(-x))


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: Sequence[int],
              window: int = 0, scale: Optional[float] = None, causal: bool = True) -> torch.Tensor:
    """q: [T, nq, hd], k, v: [T, nkv, hd] of ONE request, token t at positions[t].
    Scores (q * hd^-0.5) . k (tiny_llm/ops/cuda/flash_attention.cu:149-152, 69-74), kv head
    h / (nq / nkv) (:158), a key is masked when it lies after the query (:63-68; by absolute
    position here) or, with a window, `window` or more positions before it; softmax;
    weighted sum of v (:90-117, written without the running rescale)."""
    T, nq, hd = q.shape
    nkv = k.shape[1]
    g = nq // nkv
    sc = (1.0 / math.sqrt(hd)) if scale is None else scale
    out = torch.zeros_like(q)
    for h in range(nq):
        kh = h // g
        for t in range(T):
            qs = q[t, h] * sc
            scores = torch.full((T,), float("-inf"), dtype=q.dtype)
            for j in range(T):
                if causal and positions[j] > positions[t]:
                    continue
                if window and positions[j] <= positions[t] - window:
                    continue
                scores[j] = (qs * k[j, kh]).sum()
            m = scores.max()
            p = torch.exp(scores - m)
            out[t, h] = (p[:, None] * v[:, kh]).sum(dim=0) / p.sum()
    return out


def attention_fast(q, k, v, positions, window: int = 0, scale: Optional[float] = None) -> torch.Tensor:
    """The same function as `attention`, with the loops over keys vectorised."""
    T, nq, hd = q.shape
    nkv = k.shape[1]
    g = nq // nkv
    sc = (1.0 / math.sqrt(hd)) if scale is None else scale
    pos = torch.as_tensor(list(positions))
    mask = pos[None, :] > pos[:, None]
    if window:
        mask |= pos[None, :] <= pos[:, None] - window
    out = torch.empty_like(q)
    for h in range(nq):
        s = (q[:, h] * sc) @ k[:, h // g].T
        s = s.masked_fill(mask, float("-inf"))
        p = torch.exp(s - s.max(dim=-1, keepdim=True).values)
        out[:, h] = (p @ v[:, h // g]) / p.sum(dim=-1, keepdim=True)
    return out


def swiglu(h: torch.Tensor, Wg, Wu, Wd, act_dtype=None, row_scale=None) -> torch.Tensor:
    """g = h Wg^T; g <- silu(g); u = h Wu^T; z = g * u; m = z Wd^T
    (tiny_llm/parser/llama_parser.cpp:225-249).  `row_scale` multiplies g and u (see normed_linear)."""
    g = linear(h, Wg)
    u = linear(h, Wu)
    if row_scale is not None:
        g, u = g * row_scale, u * row_scale
    z = _rnd(silu(g) * u, act_dtype)      # the serving path stores only the gated product
    return linear(z, Wd)


def norm_operand(x: torch.Tensor, w: torch.Tensor, eps: float, act_dtype):
    """(h, row_scale) with rms_norm(x) W^T == (h W^T) * row_scale.  In float64 h is the norm itself.
    With act_dtype the serving path's rounding is followed: it feeds bf16(w * x) to the product and
    applies 1 / rms to the result."""
    if act_dtype is None:
        return rms_norm(x, w, eps), None
    H = x.shape[-1]
    r = torch.sqrt((x * x / H).sum(dim=-1, keepdim=True) + eps)
    return _rnd(w.to(x.dtype) * x, act_dtype), 1.0 / r


# ------------------------------------------------------------------------- model
def llama_forward(w: Dict[str, torch.Tensor], cfg: dict, tokens: Sequence[int],
                  positions: Optional[Sequence[int]] = None, act_dtype=None, window: int = 0,
                  segments: Optional[Sequence[int]] = None, rows: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one request's whole token list
    (layer order: tiny_llm/parser/llama_parser.cpp:181-271).

    segments: `tokens` holds several requests one after the other, of these lengths: every part
    but attention works token by token, and attention runs on each request by itself (positions
    start at 0 in each).  rows: logits of these token rows only (the reference computes the last
    row of each request only, tiny_llm/ops/cuda/gemm_q1_helper.cu:99-124)."""
    H = cfg["hidden_size"]
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nq)
    hd = cfg.get("head_dim") or H // nq
    eps = cfg.get("rms_norm_eps", 1e-6)
    T = len(tokens)
    segments = [T] if segments is None else list(segments)
    assert sum(segments) == T
    if positions is None:
        positions = [p for n in segments for p in range(n)]
    positions = list(positions)
    starts = [sum(segments[:i]) for i in range(len(segments))]
    cos, sin = rope_table_fast(max(positions) + 1, hd, cfg.get("rope_theta", 10000.0))
    x = embedding(tokens, w["model.embed_tokens.weight"])
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        h, rs = norm_operand(x, w[f"{p}.input_layernorm.weight"], eps, act_dtype)
        sc = (lambda t: t) if rs is None else (lambda t: t * rs)
        q = _rnd(sc(linear(h, w[f"{p}.self_attn.q_proj.weight"])), act_dtype).view(T, nq, hd)
        k = _rnd(sc(linear(h, w[f"{p}.self_attn.k_proj.weight"])), act_dtype).view(T, nkv, hd)
        v = _rnd(sc(linear(h, w[f"{p}.self_attn.v_proj.weight"])), act_dtype).view(T, nkv, hd)
        q = _rnd(apply_rope(q, positions, cos, sin), act_dtype)
        k = _rnd(apply_rope(k, positions, cos, sin), act_dtype)
        o = torch.cat([attention_fast(q[a:a + n], k[a:a + n], v[a:a + n], positions[a:a + n], window)
                       for a, n in zip(starts, segments)])
        o = _rnd(o, act_dtype).reshape(T, nq * hd)
        x = x + linear(o, w[f"{p}.self_attn.o_proj.weight"])
        h2, rs2 = norm_operand(x, w[f"{p}.post_attention_layernorm.weight"], eps, act_dtype)
        x = x + swiglu(h2, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                       w[f"{p}.mlp.down_proj.weight"], act_dtype, rs2)
    if rows is not None:
        x = x[list(rows)]
    xn, rsn = norm_operand(x, w["model.norm.weight"], eps, act_dtype)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    logits = linear(xn, head)
    return logits if rsn is None else logits * rsn


def greedy_generate(w, cfg, prompt: Sequence[int], n_new: int, act_dtype=None) -> List[int]:
    """Argmax of the last position, appended, again (tiny_llm/pipeline/pipeline.cpp:181-226)."""
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        logits = llama_forward(w, cfg, toks, act_dtype=act_dtype)[-1]
        nxt = argmax_first(logits)
        out.append(nxt)
        toks.append(nxt)
    return out


# ---------------------------------------------------------------------- sampling
def argmax_first(logits: torch.Tensor) -> int:
    """First maximum, strict > (tiny_llm/logit_processors/argmax_processor.cpp:24-29)."""
    best = 0
    for j in range(1, logits.numel()):
        if logits[j] > logits[best]:
            best = j
    return best


def temperature(logits: torch.Tensor, t: float) -> torch.Tensor:
    """All logits times 1/t in float32 (tiny_llm/logit_processors/temperature_processor.hpp:12-19,
    tiny_llm/ops/cpu/arithmetic.cpp:75-78)."""
    return logits.to(torch.float32) * torch.tensor(1.0 / t, dtype=torch.float32)


def sorted_ids(logits: torch.Tensor) -> List[int]:
    """Token ids by descending logit, ties by ascending id."""
    return sorted(range(logits.numel()), key=lambda i: (-float(logits[i]), i))


def top_k_top_p_ids(logits: torch.Tensor, k: int, p: float, min_keep: int = 1) -> List[int]:
    """Ids kept by TopK then TopP (tiny_llm/logit_processors/sort_processors.cpp:54-142):
    the k largest; then, sorted descending, prob_i = exp(l_i - l_0) / sum, remain = 1 - p,
    walking from the tail remain -= prob_i and stopping at the first remain < 0."""
    order = sorted_ids(logits)
    if 0 < k < len(order):
        order = order[:k]
    vals = torch.tensor([float(logits[i]) for i in order], dtype=F64)
    probs = torch.exp(vals - vals[0])
    probs = probs / probs.sum()
    remain = 1.0 - p
    idx = len(order) - 1
    while idx >= min_keep:
        remain -= float(probs[idx])
        if remain < 0:
            break
        idx -= 1
    return order[:idx + 1]


def multinomial(logits: torch.Tensor, ids: List[int], u: float) -> int:
    """Softmax over the kept ids, subtract probabilities in order from u until it is
    negative (tiny_llm/logit_processors/sample_processors.cpp:26-49)."""
    vals = torch.tensor([float(logits[i]) for i in ids], dtype=F64)
    probs = torch.exp(vals - vals.max())
    probs = probs / probs.sum()
    for j, i in enumerate(ids):
        u -= float(probs[j])
        if u < 0:
            return i
    return ids[-1]


def splitmix64(z: int) -> int:
    M = (1 << 64) - 1
    z = (z + 0x9E3779B97F4A7C15) & M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
    return z ^ (z >> 31)


def uniform_for(seed: int, counter: int) -> float:
    """The engine's documented uniform number for (seed, counter): 24 bits of
    splitmix64(splitmix64(seed) ^ counter * 0xD1B54A32D192ED03)."""
    M = (1 << 64) - 1
    bits = splitmix64(splitmix64(seed & M) ^ ((counter * 0xD1B54A32D192ED03) & M))
    return (bits >> 40) / 16777216.0


def sample_token(logits: torch.Tensor, t: float, k: int, p: float, u: float) -> int:
    """Temperature -> TopK -> TopP -> Multinomial (tiny_llm/pipeline/pipeline.cpp:156-164)."""
    x = temperature(logits, t)
    ids = top_k_top_p_ids(x, k, p)
    return multinomial(x, ids, u)
