"""Grouped-query causal attention over the paged cache (the Llama mixer).

Per token: q, k, v = h Wq^T, h Wk^T, h Wv^T (tiny_llm/ops/cuda/gemm.cu:86-100,
head-major columns gemm.cu:119-123); q and k rotated by the token's position
(rope.cu:46-54); k (rotated) and v written to the cache (gemm.cu:400-407);
scores q.k * hd^-0.5 against the request's cached keys with a causal mask, online
softmax, weighted sum of values (flash_attention.cu:374-405); output projection
with the residual add folded in (gemm.cu:171-190, arithmetic.cu:13).

Q, K and V weights are concatenated on load into one [(nq + 2 nkv) * hd, H]
matrix: row concatenation leaves every dot product as it was.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .norm import LazyNorm
from .base import (CacheSpec, LayerCache, Mixer, POSITION_ENCODINGS, WeightSpec, project_into_residual,
                   register_mixer)


class Attention(Mixer):
    graph_safe = True
    accepts_lazy_norm = True
    prepares_next_norm = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, position: dict = None, window: int = 0, scale: float = None,
                 max_position: int = 0):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        if self.num_kv_heads <= 0 or self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        # sizes a kernel refuses are refused here, when the model is built, not at its first step
        ops.check_attention_sizes(dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.num_heads * self.head_dim, f"{prefix}: num_heads * head_dim")
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        pos = dict(position or {"kind": "none"})
        kind = pos.pop("kind")
        self.position = POSITION_ENCODINGS.get(kind)(f"{prefix}.position", dtype, device, **pos)
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    # ---------------------------------------------------------------- declarations
    def weights(self) -> List[WeightSpec]:
        p, H = self.prefix, self.hidden_size
        return [WeightSpec(f"{p}.q_proj.weight", (self.q_size, H)),
                WeightSpec(f"{p}.k_proj.weight", (self.kv_size, H)),
                WeightSpec(f"{p}.v_proj.weight", (self.kv_size, H)),
                WeightSpec(f"{p}.o_proj.weight", (H, self.q_size))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        self.w_qkv = torch.cat([tensors[f"{p}.q_proj.weight"], tensors[f"{p}.k_proj.weight"],
                                tensors[f"{p}.v_proj.weight"]], dim=0).contiguous()
        self.w_o = tensors[f"{p}.o_proj.weight"].contiguous()

    def cache_spec(self) -> CacheSpec:
        return CacheSpec.keys_and_values(self.num_kv_heads, self.head_dim, "window" if self.window else "full",
                                         self.window)

    # --------------------------------------------------------------------- compute
    def forward(self, h, ctx, cache: LayerCache, state, residual, next_norm=None):
        T = residual.shape[0]
        qkv = ops.scratch("qkv", (T, self.q_size + 2 * self.kv_size), self.dtype, residual.device)
        if isinstance(h, LazyNorm):
            h.linear(self.w_qkv, qkv)
        else:
            ops.linear(h, self.w_qkv, qkv)
        tables = self.position.rotary_tables()
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        pairing = getattr(self.position, "pairing", "half")     # an encoding that says nothing pairs (i, i + rot/2)
        attn = ops.scratch("attention_out", (T, self.q_size), self.dtype, residual.device)
        q = qkv[:, :self.q_size]
        flash = ops.flash_attention_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        group = self.num_heads // self.num_kv_heads
        # decode steps: rotation and cache write ride in the attention kernel
        fuse = flash and ctx.max_q_len == 1 and cache.write and rot == self.head_dim and pairing == "half"
        if not fuse:
            slots = ctx.slot_mappings[cache.group] if cache.write else None
            ops.rope_store(qkv, ctx.positions, cos, sin, slots, cache.k if cache.write else None,
                           cache.v if cache.write else None, self.num_heads, self.num_kv_heads, self.head_dim, rot,
                           pairing)
        if flash and ctx.max_q_len > 1:
            # prompt portions: many query rows share each staged key tile
            waves = ops.prefill_tile_waves(T, self.num_heads, self.num_kv_heads)
            tiles = ctx.attention_tiles(waves * (16 // group))
            # a portion late in a long prompt: few query rows, many keys; the keys are shared out
            n_splits = ops.prefill_key_splits(T, ctx.max_seq_len, self.num_heads, self.num_kv_heads, waves)
            scratch = None
            if n_splits > 1:
                scratch = ops.scratch("attention_partials", (n_splits * T * self.num_heads * (self.head_dim + 2),),
                                      torch.float32, residual.device)
            ops.flash_prefill(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                              self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window, waves,
                              n_splits, scratch)
        elif flash:
            # decoding: one token per request, its keys split over the waves of a workgroup (and over
            # workgroups when the context is long)
            # (no tile arrays when every request brings exactly one token: row i is request i)
            tiles = None if T == ctx.num_requests else ctx.attention_tiles(16 // group)
            n_splits, scratch = self._splits(ctx, T, residual.device)
            ops.flash_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                                self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window,
                                n_splits, scratch, fused_rope=(cos, sin) if fuse else None)
        elif ops.attention_f32_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim) \
                and q.stride(0) % 4 == 0:
            # true float32 on the matrix cores; one fixed merge tree, so the same bits whatever the batch
            decode = ctx.max_q_len == 1 and T == ctx.num_requests
            tiles = None if decode else ctx.attention_tiles(16 // group)
            n_chunks = -(-ctx.max_seq_len // ops.F32_CHUNK_KEYS) if ctx.max_q_len == 1 else 1
            scratch = None
            if n_chunks > 1:
                scratch = ops.scratch("attention_partials", (n_chunks * T * self.num_heads * (self.head_dim + 2),),
                                      torch.float32, residual.device)
            ops.attention_f32(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                              self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window, n_chunks,
                              scratch)
        else:
            ops.paged_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.req_of_token,
                                ctx.positions, attn, self.num_heads, self.num_kv_heads, self.head_dim,
                                self.scale, self.window)
        out, prepared = project_into_residual(attn, self.w_o, residual, next_norm)
        return out if next_norm is None else (out, prepared)

    def _splits(self, ctx, T: int, device):
        """How many workgroups share one query tile's keys (`ops.decode_key_splits`), and the scratch
        for their partial results."""
        n_splits = ops.decode_key_splits(T, ctx.max_seq_len, self.num_kv_heads, self.head_dim)
        if n_splits == 1:
            return 1, None
        return n_splits, ops.scratch("attention_partials", (n_splits * T * self.num_heads * (self.head_dim + 2),),
                                     torch.float32, device)


register_mixer("attention", Attention)
