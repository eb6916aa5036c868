"""What fixes the plain implementation beside the reference's text: the golden tensors the
reference's own tests compare against (read from its checkout with the safetensors reader,
inputs rebuilt from the ramps its tests use), special cases that reduce to library
routines, and invariants.  Each is chosen so that a plausible mistake fails it: a wrong
sign or pairing in the rotation, a wrong head grouping, a mask off by one, a norm that
divides before it sums."""
import math
import os

import pytest
import torch

import plain_llama as plain
from util import REFERENCE_DATA as DATA

needs_reference = pytest.mark.skipif(not os.path.isdir(DATA), reason="reference checkout not mounted")


def golden(name):
    from safetensors import safe_open
    with safe_open(os.path.join(DATA, name), "pt") as f:
        return {k: f.get_tensor(k).double() for k in f.keys()}


def ramp(n, shift=0, scale=100.0):
    return ((torch.arange(n) + shift) % 100).double() / scale


# ------------------------------------------------------------------ goldens
@needs_reference
def test_linear_golden():
    # tests/ops/cuda/test_gemm.cpp:160-199: input and weight are i % 100
    a = ramp(127 * 255, scale=1.0).reshape(127, 255)
    w = ramp(353 * 255, scale=1.0).reshape(353, 255)
    assert torch.equal(plain.linear(a, w), golden("gemm_m127d255n353.safetensors")["res"])


@needs_reference
def test_rms_norm_golden():
    # tests/ops/cuda/test_norm.cpp:8-47
    x = ramp(2 * 107 * 241).reshape(2 * 107, 241)
    w = ramp(241)
    ref = golden("rms_norm_b2l107d241.safetensors")["res"].reshape(2 * 107, 241)
    assert (plain.rms_norm(x, w, 1.192e-7) - ref).abs().max() < 1e-5


@needs_reference
def test_rope_table_golden_fixes_the_half_split_convention():
    # tests/ops/cuda/test_rope.cpp:8-37: both halves of the full-width golden equal the [2, 48] table
    g = golden("rope_s2_d96.safetensors")
    cos, sin = plain.rope_table(2, 96, 10000.0)
    for half in (slice(0, 48), slice(48, 96)):
        assert (cos - g["cos"][0][:, half]).abs().max() < 1e-6
        assert (sin - g["sin"][0][:, half]).abs().max() < 1e-6
    assert torch.equal(plain.rope_table_fast(37, 96, 10000.0)[0], plain.rope_table(37, 96, 10000.0)[0])
    assert torch.equal(plain.rope_table_fast(37, 96, 10000.0)[1], plain.rope_table(37, 96, 10000.0)[1])


@needs_reference
def test_apply_rope_golden_fixes_sign_and_pairing():
    # tests/ops/cuda/test_rope.cpp:40-98: [b3, h4, q_end5, d96], rows 1..2 are ramps rotated at
    # positions 0, 1; all other rows stay 1.0
    b, h, q, d, qs, qe = 3, 4, 2, 96, 1, 5
    cos, sin = plain.rope_table(2, d, 10000.0)
    want = golden("apply_rope_b3_h4_q2_d96_qs1qe5.safetensors")["res"]
    vals = ramp(b * h * q * d).reshape(b, h, q, d)
    got = torch.ones(b, h, qe, d, dtype=torch.float64)
    for bi in range(b):
        x = vals[bi].transpose(0, 1)                 # [q, h, d], token t at position t & 1
        got[bi, :, qs:qs + q] = plain.apply_rope(x, [0, 1], cos, sin).transpose(0, 1)
    assert (got - want).abs().max() < 1e-4


@needs_reference
def test_causal_attention_golden_fixes_grouping_scale_and_mask():
    # tests/ops/cuda/test_flash_attention.cpp:90-170: b2, q = kv = 107, heads 4:2, hd 61
    B, L, nq, nkv, hd = 2, 107, 4, 2, 61
    q = ramp(B * nq * L * hd).reshape(B, nq, L, hd)
    k = ramp(B * nkv * L * hd, 1).reshape(B, nkv, L, hd)
    v = ramp(B * nkv * L * hd, 2).reshape(B, nkv, L, hd)
    want = golden("causal_attn_res_b2l107q4k2d61.safetensors")["res"]      # [B, nq, L, hd]
    for b in range(B):
        got = plain.attention_fast(q[b].transpose(0, 1), k[b].transpose(0, 1), v[b].transpose(0, 1), range(L))
        assert (got.transpose(0, 1) - want[b]).abs().max() < 1e-5
    slow = plain.attention(q[0].transpose(0, 1)[:9], k[0].transpose(0, 1)[:9], v[0].transpose(0, 1)[:9], range(9))
    fast = plain.attention_fast(q[0].transpose(0, 1)[:9], k[0].transpose(0, 1)[:9], v[0].transpose(0, 1)[:9], range(9))
    assert (slow - fast).abs().max() < 1e-12


@needs_reference
def test_unmasked_attention_golden():
    # tests/ops/cuda/test_flash_attention.cpp:8-88: q 107 rows against kv 123 rows, no mask
    B, Lq, Lk, nq, nkv, hd = 2, 107, 123, 4, 2, 61
    q = ramp(B * nq * Lq * hd).reshape(B, nq, Lq, hd)
    k = ramp(B * nkv * Lk * hd, 1).reshape(B, nkv, Lk, hd)
    v = ramp(B * nkv * Lk * hd, 2).reshape(B, nkv, Lk, hd)
    want = golden("attn_res_b2q107h4k123h2d61.safetensors")["res"]
    for b in range(B):
        for h in range(nq):
            s = (q[b, h] / math.sqrt(hd)) @ k[b, h // 2].T
            p = torch.softmax(s, dim=-1)
            assert ((p @ v[b, h // 2]) - want[b, h]).abs().max() < 1e-5
    # the plain function with every query placed after all keys computes the same thing
    one = plain.attention_fast(torch.cat([torch.zeros(Lk - 1, nq, hd, dtype=torch.float64), q[0].transpose(0, 1)[:1]]),
                               k[0].transpose(0, 1), v[0].transpose(0, 1), range(Lk))
    assert (one[-1] - want[0, :, 0]).abs().max() < 1e-5


@needs_reference
def test_attention_block_golden_whole_five_tokens():
    # tests/runtime/cuda/test_attention_runtime.cpp:474-530: TinyLlama-size block, hidden and weights
    # are (i % 100) / 1e4 ramps, 5 tokens; the golden is the whole-sequence result
    g = golden("llama_attn_res_b1q5h2048.safetensors")
    H, nq, nkv, hd, T = 2048, 32, 4, 64, 5
    x = ramp(T * H, scale=10000.0).reshape(T, H)
    wqo = ramp(H * H, scale=10000.0).reshape(H, H)
    wkv = ramp(nkv * hd * H, scale=10000.0).reshape(nkv * hd, H)
    cos, sin = plain.rope_table(T, hd, 10000.0)
    assert (cos - g["cos"][0]).abs().max() < 1e-6 and (sin - g["sin"][0]).abs().max() < 1e-6
    q = plain.apply_rope(plain.linear(x, wqo).view(T, nq, hd), range(T), cos, sin)
    k = plain.apply_rope(plain.linear(x, wkv).view(T, nkv, hd), range(T), cos, sin)
    v = plain.linear(x, wkv).view(T, nkv, hd)
    o = plain.attention(q, k, v, range(T)).reshape(T, nq * hd)
    out = plain.linear(o, wqo)
    want = g["res"][0]
    assert (out - want).abs().max() < 1e-5 * max(1.0, float(want.abs().max()))
    # prefill of 3 tokens then 2 decoded ones equals rows 0..4 of the whole (test_attention_runtime.cpp:240-316)
    o3 = plain.attention(q[:3], k[:3], v[:3], range(3)).reshape(3, nq * hd)
    assert (plain.linear(o3, wqo) - want[:3]).abs().max() < 1e-5 * max(1.0, float(want.abs().max()))


# --------------------------------------------------- library routines, invariants
def test_parts_reduce_to_library_routines():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 48, generator=g, dtype=torch.float64)
    w = torch.randn(48, generator=g, dtype=torch.float64)
    assert torch.allclose(plain.rms_norm(x, torch.ones(48), 1e-6), torch.nn.functional.rms_norm(x, (48,), eps=1e-6))
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), torch.nn.functional.rms_norm(x, (48,), w, eps=1e-5))
    assert torch.allclose(plain.silu(x), torch.nn.functional.silu(x))
    W = torch.randn(5, 48, generator=g, dtype=torch.float64)
    assert torch.allclose(plain.linear(x, W), torch.nn.functional.linear(x, W))
    E = torch.randn(11, 6, generator=g, dtype=torch.float64)
    assert torch.equal(plain.embedding([3, 0, 10], E), torch.nn.functional.embedding(torch.tensor([3, 0, 10]), E))
    # one head, no rotation: plain causal attention
    q, k, v = (torch.randn(9, 1, 16, generator=g, dtype=torch.float64) for _ in range(3))
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                                           is_causal=True).transpose(0, 1)
    assert torch.allclose(plain.attention(q, k, v, range(9)), ref)
    # grouped heads equal full heads with keys and values repeated
    q = torch.randn(9, 6, 16, generator=g, dtype=torch.float64)
    k, v = (torch.randn(9, 2, 16, generator=g, dtype=torch.float64) for _ in range(2))
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.repeat_interleave(3, 1).transpose(0, 1), v.repeat_interleave(3, 1).transpose(0, 1),
        is_causal=True).transpose(0, 1)
    assert torch.allclose(plain.attention_fast(q, k, v, range(9)), ref)
    # silu vectors of tests/ops/cuda/test_silu.cpp:8-28
    assert plain.silu(torch.tensor([0.0, 1.0], dtype=torch.float64)).tolist() == [0.0, 1 / (1 + math.exp(-1))]


def test_rotation_invariants():
    cos, sin = plain.rope_table(400, 32, 500000.0)
    g = torch.Generator().manual_seed(1)
    q = torch.randn(1, 2, 32, generator=g, dtype=torch.float64)
    k = torch.randn(1, 2, 32, generator=g, dtype=torch.float64)
    assert torch.equal(plain.apply_rope(q, [0], cos, sin), q)                  # position 0: identity
    r = plain.apply_rope(q, [17], cos, sin)
    assert torch.allclose(r[..., :16] ** 2 + r[..., 16:] ** 2, q[..., :16] ** 2 + q[..., 16:] ** 2)
    dot = lambda m, n: (plain.apply_rope(q, [m], cos, sin) * plain.apply_rope(k, [n], cos, sin)).sum()
    assert abs(dot(5, 2) - dot(305, 302)) < 1e-5                               # only the distance counts
    assert abs(dot(5, 2) - dot(2, 5)) > 1e-3                                   # and its sign


def test_window_and_shift_of_all_positions():
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(12, 2, 8, generator=g, dtype=torch.float64) for _ in range(3))
    full = plain.attention(q, k, v, range(12))
    assert torch.allclose(plain.attention(q, k, v, range(12), window=12), full)
    w1 = plain.attention(q, k, v, range(12), window=1)
    assert torch.allclose(w1, v)                                               # each token sees itself only
    w3 = plain.attention(q, k, v, range(12), window=3)
    assert torch.allclose(w3[:3], full[:3]) and not torch.allclose(w3[3], full[3])
    assert torch.allclose(plain.attention_fast(q, k, v, range(12), window=3), w3)
    # without rotation only the order of positions counts
    assert torch.allclose(plain.attention(q, k, v, range(100, 112), window=3), w3)


def _tiny_weights(cfg, seed=3, std=0.05, norm_std=0.1):
    from tiny_llm_amd.weights.loader import random_tensor
    from tiny_llm_amd.config import resolve
    from tiny_llm_amd.models.decoder import Decoder
    _, spec = resolve(cfg)
    dec = Decoder(spec, "float32", "cpu")
    return {s.name: random_tensor(s, seed, std, norm_std).double() for s in dec.weight_specs() if not s.alias_of}


def _library_model(w, cfg, tokens, causal):
    """The whole model from torch's own routines only, for the cases in which the rotation is the
    identity (every token at position 0): embedding, rms_norm, linear, scaled_dot_product_attention
    with keys and values repeated per group, silu.  Layer order as tiny_llm/parser/llama_parser.cpp:194-271."""
    F = torch.nn.functional
    H, nq = cfg["hidden_size"], cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nq)
    hd = cfg.get("head_dim") or H // nq
    eps = cfg["rms_norm_eps"]
    T = len(tokens)
    x = F.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"])
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        h = F.rms_norm(x, (H,), w[f"{p}.input_layernorm.weight"], eps)
        q = F.linear(h, w[f"{p}.self_attn.q_proj.weight"]).view(T, nq, hd).transpose(0, 1)
        k = F.linear(h, w[f"{p}.self_attn.k_proj.weight"]).view(T, nkv, hd).transpose(0, 1)
        v = F.linear(h, w[f"{p}.self_attn.v_proj.weight"]).view(T, nkv, hd).transpose(0, 1)
        k, v = k.repeat_interleave(nq // nkv, 0), v.repeat_interleave(nq // nkv, 0)
        o = F.scaled_dot_product_attention(q, k, v, is_causal=causal).transpose(0, 1).reshape(T, nq * hd)
        x = x + F.linear(o, w[f"{p}.self_attn.o_proj.weight"])
        h = F.rms_norm(x, (H,), w[f"{p}.post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(h, w[f"{p}.mlp.up_proj.weight"]),
                         w[f"{p}.mlp.down_proj.weight"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return F.linear(F.rms_norm(x, (H,), w["model.norm.weight"], eps), head)


@pytest.mark.parametrize("name", ["A", "B"])
def test_whole_model_reduces_to_library_routines_where_the_rotation_is_the_identity(name):
    """With every token at position 0 nothing is rotated and (the mask comparing positions) every
    token sees every other: the model is embedding, rms_norm, linear, unmasked attention and silu
    of the library, in the reference's layer order.  A norm in another place, gate and up swapped,
    the residual taken before instead of after, a missing final norm or another head-to-group
    mapping all fail this.  One token alone is the causal case of it."""
    from util import CONFIGS, random_tokens
    cfg, _, init = CONFIGS[name]
    w = _tiny_weights(cfg, 3, init["std"] * 3, max(init["norm_std"], 0.1))
    toks = random_tokens(13, cfg["vocab_size"], 4)
    got = plain.llama_forward(w, cfg, toks, positions=[0] * 13)
    want = _library_model(w, cfg, toks, causal=False)
    assert (got - want).abs().max() < 1e-9 * max(1.0, float(want.abs().max()))
    one = plain.llama_forward(w, cfg, toks[:1])
    assert (one - _library_model(w, cfg, toks[:1], causal=True)).abs().max() < 1e-9
    # and the causal model agrees with the library on its FIRST row whatever follows (position 0)
    assert (plain.llama_forward(w, cfg, toks)[0] - one[0]).abs().max() < 1e-9


def test_whole_model_invariants_that_plausible_mistakes_break():
    from util import TINY_A, random_tokens
    cfg = TINY_A
    w = _tiny_weights(cfg, 5, 0.08, 0.1)
    toks = random_tokens(17, cfg["vocab_size"], 6)
    base = plain.llama_forward(w, cfg, toks)
    scaled = lambda key, c: {**w, **{k: v * c for k, v in w.items() if key in k}}
    # the feed-forward is linear in `up` and in `down` but not in `gate` (SiLU sits on gate only)
    up2, down2, gate2 = (plain.llama_forward(scaled(k, 2.0), cfg, toks) for k in ("up_proj", "down_proj", "gate_proj"))
    assert (up2 - down2).abs().max() < 1e-9 and (up2 - base).abs().max() > 1e-3
    assert (gate2 - up2).abs().max() > 1e-3
    # attention is linear in `v` and in `o` alike, and only distances between positions count
    v2, o2 = (plain.llama_forward(scaled(k, 2.0), cfg, toks) for k in ("v_proj", "o_proj"))
    assert (v2 - o2).abs().max() < 1e-9 and (v2 - base).abs().max() > 1e-3
    shifted = plain.llama_forward(w, cfg, toks, positions=range(300, 317))
    assert (shifted - base).abs().max() < 1e-6       # the angle table is rounded to float32, as the reference's
    # pre-norm: a norm's weight times c is its consumers' weights times c (the residual stream itself
    # is not normed: scaling the embedding changes the logits, scaling after the final norm does not exist)
    n2 = plain.llama_forward(scaled("input_layernorm", 3.0), cfg, toks)
    qkv3 = plain.llama_forward({**w, **{k: v * 3.0 for k, v in w.items() if any(
        p in k for p in ("q_proj", "k_proj", "v_proj"))}}, cfg, toks)
    assert (n2 - qkv3).abs().max() < 1e-8 and (n2 - base).abs().max() > 1e-3
    f2 = plain.llama_forward(scaled("model.norm", 3.0), cfg, toks)
    assert (f2 - 3.0 * base).abs().max() < 1e-8                              # the final norm feeds the head alone
    # zeroed o and down projections: the layers add nothing and the logits are head(norm(embedding))
    z = scaled("down_proj", 0.0)
    z = {k: (v * 0.0 if "o_proj" in k else v) for k, v in z.items()}
    F = torch.nn.functional
    x = F.embedding(torch.tensor(toks), w["model.embed_tokens.weight"])
    want = F.linear(F.rms_norm(x, (cfg["hidden_size"],), w["model.norm.weight"], cfg["rms_norm_eps"]), w["lm_head.weight"])
    assert (plain.llama_forward(z, cfg, toks) - want).abs().max() < 1e-9


def test_model_invariants():
    from util import TINY_B, random_tokens
    w = _tiny_weights(TINY_B)
    toks = random_tokens(24, TINY_B["vocab_size"], 9)
    logits = plain.llama_forward(w, TINY_B, toks)
    assert logits.shape == (24, TINY_B["vocab_size"])
    # causality: a later token does not change earlier logits
    other = list(toks)
    other[20] = (other[20] + 1) % TINY_B["vocab_size"]
    l2 = plain.llama_forward(w, TINY_B, other)
    assert torch.equal(logits[:20], l2[:20]) and not torch.allclose(logits[20:], l2[20:])
    # a one-token sequence: attention returns v itself, so the first logits need no other token
    assert torch.allclose(plain.llama_forward(w, TINY_B, toks[:1])[0], logits[0])
    # tied head: logits are xn E^T
    assert "lm_head.weight" not in w
    # greedy generation is the step-wise argmax of the model
    out = plain.greedy_generate(w, TINY_B, toks[:5], 3)
    assert out[0] == int(plain.llama_forward(w, TINY_B, toks[:5])[-1].argmax())
    assert out[1] == int(plain.llama_forward(w, TINY_B, toks[:5] + out[:1])[-1].argmax())
    # several requests in one call (what tests of large shapes use to stream the weights once) are
    # the requests one by one; `rows` picks rows of the result
    a, b, c = toks[:9], toks[9:10], toks[10:]
    both = plain.llama_forward(w, TINY_B, a + b + c, segments=[9, 1, 14], act_dtype=torch.bfloat16)
    for got, one in ((both[:9], a), (both[9:10], b), (both[10:], c)):
        assert torch.equal(got, plain.llama_forward(w, TINY_B, one, act_dtype=torch.bfloat16))
    picked = plain.llama_forward(w, TINY_B, a + b + c, segments=[9, 1, 14], rows=[8, 9, 23, 0])
    assert torch.allclose(picked, plain.llama_forward(w, TINY_B, a + b + c, segments=[9, 1, 14])[[8, 9, 23, 0]], atol=1e-12)


# ------------------------------------------------------------------- sampling
def test_sampling_reference_vectors():
    # argmax on ramps -> 19 (tests/logit_processors/test_argmax_processor.cpp:19-31)
    assert plain.argmax_first(torch.arange(20.0)) == 19
    assert plain.argmax_first(torch.tensor([1.0, 3.0, 3.0, 2.0])) == 1          # first maximum
    # temperature 0.5 doubles (tests/logit_processors/test_temperature_processor.cpp:22-26)
    assert plain.temperature(torch.tensor([1.0, -2.0]), 0.5).tolist() == [2.0, -4.0]
    # top-k 5 of ramps keeps 15..19 (tests/logit_processors/test_sort_processors.cpp:45-99)
    assert sorted(plain.top_k_top_p_ids(torch.arange(20.0), 5, 1.0)) == [15, 16, 17, 18, 19]
    assert plain.top_k_top_p_ids(torch.arange(20.0), 1, 1.0) == [19]
    # top-p (test_sort_processors.cpp:103-201): p = 1 keeps 20; p = 0 with min 3 keeps the top 3;
    # p = 0.2 keeps 4 and 2 after logit[0] is raised
    l = torch.arange(20.0) / 40
    assert len(plain.top_k_top_p_ids(l, 0, 1.0)) == 20
    assert plain.top_k_top_p_ids(l, 0, 0.0, min_keep=3) == [19, 18, 17]
    a = l.clone()
    a[0] = 0.5
    assert plain.top_k_top_p_ids(a, 0, 0.2) == [0, 19, 18, 17]
    b = l + 0.5
    b[0] = 2.0
    assert plain.top_k_top_p_ids(b, 0, 0.2) == [0, 19]
    # multinomial with one finite logit returns it (tests/logit_processors/test_sample_processors.cpp:20-34)
    one = torch.full((8,), -1e30)
    one[5] = 0.0
    assert plain.multinomial(one, list(range(8)), 0.77) == 5
    probs = [0.5, 0.25, 0.25]
    lg = torch.log(torch.tensor(probs))
    assert [plain.multinomial(lg, [0, 1, 2], u) for u in (0.0, 0.49, 0.51, 0.74, 0.76, 0.999)] == [0, 0, 1, 1, 2, 2]


def test_uniform_generator_is_uniform_and_keyed():
    us = [plain.uniform_for(42, c) for c in range(4000)]
    assert all(0.0 <= u < 1.0 for u in us)
    assert abs(sum(us) / len(us) - 0.5) < 0.02
    assert plain.uniform_for(42, 7) == plain.uniform_for(42, 7) != plain.uniform_for(43, 7)
