"""The step function: one batch of (request, its next tokens) through the model.

A step runs only the tokens it is given, against the cache that earlier steps
left, and returns the logits at the wanted places.  Entries may be portions of
prompts beside single decoded tokens, cut anywhere.  The reference's runtime needs
five calls and allows either whole prompts from position 0 or exactly one token per
request (tiny_llm/pipeline/pipeline.cpp:132-140, 184-190,
tiny_llm/runtime/cuda/cuda_runtime.cpp:673, 690); here it is one call for any mix.

Step metadata is built on the host in one pinned int32 buffer and uploaded with
one copy (the reference uploads a block table per layer with a stream sync each,
cuda_runtime.cpp:758-773).  Token rows map to requests through `req_of_token`, so
kernels need no search over sequence separators (tiny_llm/ops/details.hpp:19-36).
"""
from __future__ import annotations

import gc
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import CacheManager


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()        # places among `tokens` whose logits are asked for


@dataclass
class StepContext:
    """Who is in the batch and where each token sits; device tensors are int32."""
    num_tokens: int
    num_requests: int
    tokens: torch.Tensor            # [T]
    positions: torch.Tensor         # [T] absolute position of each token in its request
    req_of_token: torch.Tensor      # [T] row of the block tables
    cu_seqlens_q: torch.Tensor      # [R+1]
    seq_lens: torch.Tensor          # [R] cached length after this step
    state_slots: torch.Tensor       # [R] per-request state slot
    logit_rows: Optional[torch.Tensor]      # [n_out] token rows whose logits are wanted
    block_tables: List[torch.Tensor]        # per cache group [R, max_blocks]
    slot_mappings: List[torch.Tensor]       # per cache group [T] flat slot = block * block_size + offset
    # host copies
    q_lens: List[int] = field(default_factory=list)
    context_lens: List[int] = field(default_factory=list)
    slots_host: List[int] = field(default_factory=list)
    max_q_len: int = 0
    max_seq_len: int = 0
    block_size: int = 0

    _tiles: Dict[int, tuple] = field(default_factory=dict)

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1

    def attention_tiles(self, tokens_per_tile: int):
        """(tile_req, tile_tok0, tile_ntok) int32 device tensors: every request's tokens of this
        step cut into groups of at most `tokens_per_tile` (the query tiles of the MFMA attention
        kernel).  Built once per width and step."""
        if tokens_per_tile not in self._tiles:
            req, tok0, ntok = [], [], []
            t = 0
            for r, n in enumerate(self.q_lens):
                for s in range(0, n, tokens_per_tile):
                    req.append(r)
                    tok0.append(t + s)
                    ntok.append(min(tokens_per_tile, n - s))
                t += n
            dev = self.tokens.device
            packed = torch.tensor([req, tok0, ntok], dtype=torch.int32).to(dev, non_blocking=True)
            self._tiles[tokens_per_tile] = (packed[0], packed[1], packed[2])
        return self._tiles[tokens_per_tile]


class StepError(ValueError):
    pass


class ModelRunner:
    """Owns the decoder's cache views and turns step entries into one forward pass."""

    def __init__(self, decoder, cache: CacheManager, max_num_batched_tokens: int, max_model_len: int):
        self.decoder = decoder
        self.cache = cache
        self.device = decoder.device
        self.max_tokens = int(max_num_batched_tokens)
        self.max_model_len = int(max_model_len)
        self.vocab_size = decoder.spec.vocab_size
        readers = decoder.cache_readers()
        for (i, role) in list(decoder.cache_specs()) + list(readers):
            decoder.caches[i][role] = cache.layer_cache((i, role), readers.get((i, role)))
        for (i, role) in decoder.state_specs():
            decoder.states[i][role] = cache.states[(i, role)]
        self._pinned: Optional[torch.Tensor] = None
        self._uploaded: Optional[torch.cuda.Event] = None
        self._graphs: Dict[Tuple[int, int], "DecodeGraph"] = {}

    # ----------------------------------------------------------------- metadata
    def _host_buffer(self, n: int) -> torch.Tensor:
        if self._pinned is None or self._pinned.numel() < n:
            self._pinned = torch.empty(max(n, 1 << 16), dtype=torch.int32, pin_memory=True)
        return self._pinned[:n]

    def prepare(self, entries: Sequence[StepEntry]) -> StepContext:
        """Checks the entries, takes the cache blocks they need (all or nothing) and
        builds the step metadata on the device."""
        cm = self.cache
        bs = cm.block_size
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        T = 0
        for e in entries:
            if e.req_id in seen:
                raise StepError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.req_id!r} brings no tokens")
            for t in e.tokens:
                if not (0 <= int(t) < self.vocab_size):
                    raise StepError(f"token id {t} of request {e.req_id!r} is outside the vocabulary")
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise StepError(f"wanted place {w} of request {e.req_id!r} is outside its {n} tokens")
            T += n
        if T > self.max_tokens:
            raise StepError(f"step brings {T} tokens, the budget is {self.max_tokens}")

        for e in entries:
            c = cm.num_tokens(e.req_id) if cm.has(e.req_id) else 0
            if c + len(e.tokens) > self.max_model_len:
                raise StepError(f"request {e.req_id!r} would reach {c + len(e.tokens)} tokens, "
                                f"the limit is {self.max_model_len}")
        ctx_lens = cm.reserve_step([(e.req_id, len(e.tokens)) for e in entries])
        new_lens = [c + len(e.tokens) for c, e in zip(ctx_lens, entries)]

        R, G = len(entries), len(cm.groups)
        max_blocks = max(1, max(-(-n // bs) for n in new_lens))
        n_out = sum(len(e.want) for e in entries)
        sizes = [T, T, T, R + 1, R, R, n_out] + [T] * G + [R * max_blocks] * G
        offs = [0]
        for s in sizes:
            offs.append(offs[-1] + ((s + 3) // 4) * 4)   # 16-byte aligned sections
        if self._uploaded is not None:
            self._uploaded.synchronize()      # the last step's upload has left the pinned buffer
        buf = self._host_buffer(offs[-1])
        host = buf.numpy()
        host[:offs[-1]] = 0
        tok, pos, rot = host[offs[0]:], host[offs[1]:], host[offs[2]:]
        cu, sl, ss, lr = host[offs[3]:], host[offs[4]:], host[offs[5]:], host[offs[6]:]
        t = 0
        k = 0
        q_lens, slots = [], []
        for r, e in enumerate(entries):
            n = len(e.tokens)
            c = ctx_lens[r]
            tok[t:t + n] = e.tokens
            pos[t:t + n] = range(c, c + n)
            rot[t:t + n] = r
            cu[r] = t
            sl[r] = new_lens[r]
            ss[r] = cm.slot(e.req_id)
            slots.append(cm.slot(e.req_id))
            for w in e.want:
                lr[k] = t + int(w)
                k += 1
            for g in range(G):
                table = cm.block_table(e.req_id, g)
                sm = host[offs[7 + g]:]
                bt = host[offs[7 + G + g]:]
                tb = np.maximum(np.asarray(table, dtype=np.int32), 0)   # released blocks are never read
                bt[r * max_blocks: r * max_blocks + len(table)] = tb
                p = np.arange(c, c + n, dtype=np.int32)
                sm[t:t + n] = tb[p // bs] * bs + p % bs
            q_lens.append(n)
            t += n
        cu[R] = T
        dev = buf.to(self.device, non_blocking=True)
        self._uploaded = torch.cuda.Event()
        self._uploaded.record()
        sec = lambda i, n: dev[offs[i]:offs[i] + n]
        return StepContext(
            num_tokens=T, num_requests=R,
            tokens=sec(0, T), positions=sec(1, T), req_of_token=sec(2, T), cu_seqlens_q=sec(3, R + 1),
            seq_lens=sec(4, R), state_slots=sec(5, R), logit_rows=sec(6, n_out) if n_out else None,
            block_tables=[sec(7 + G + g, R * max_blocks).view(R, max_blocks) for g in range(G)],
            slot_mappings=[sec(7 + g, T) for g in range(G)],
            q_lens=q_lens, context_lens=ctx_lens, slots_host=slots, max_q_len=max(q_lens),
            max_seq_len=max(new_lens), block_size=bs)

    # --------------------------------------------------------------------- step
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs the entries as one batch.  Returns float32 logits [wanted, vocab] on the
        device, in the order of the entries and of each entry's `want`."""
        ctx = self.prepare(entries)
        logits = self.decoder.forward(ctx)
        for e, c, n in zip(entries, ctx.context_lens, ctx.q_lens):
            self.cache.commit(e.req_id, c + n)
        return logits

    # ------------------------------------------------------------ decode graphs
    def decode_step(self, req_ids: Sequence[Hashable], tokens: Sequence[int], params, seeds: Sequence[int],
                    counters: Sequence[int], use_graph: bool = True) -> List[int]:
        """One decoded token for each request (its next input token given), sampled on the device.
        With `use_graph` the whole step (model and sampler) is one HIP graph per batch size,
        replayed on static buffers; only the metadata upload and the token download remain."""
        R = len(req_ids)
        cm = self.cache
        for rid, t in zip(req_ids, tokens):
            if not (0 <= int(t) < self.vocab_size):
                raise StepError(f"token id {t} of request {rid!r} is outside the vocabulary")
            if (cm.num_tokens(rid) if cm.has(rid) else 0) + 1 > self.max_model_len:
                raise StepError(f"request {rid!r} would exceed {self.max_model_len} tokens")
        ctx_lens = cm.reserve_step([(rid, 1) for rid in req_ids])
        # One graph per batch size and context bound: the bound (a power of two, at least 512) decides
        # into how many workgroups the attention kernel splits a request's keys, which is fixed at capture.
        bound = 512
        while bound < max(ctx_lens) + 1:
            bound *= 2
        bound = min(bound, self.max_model_len)
        dg = self._graphs.get((R, bound))
        if dg is None:
            dg = self._graphs[(R, bound)] = DecodeGraph(self, R, bound)
        toks = dg.run(req_ids, tokens, ctx_lens, params, seeds, counters,
                      capture=use_graph and self.decoder.graph_safe)
        for rid, c in zip(req_ids, ctx_lens):
            cm.commit(rid, c + 1)
        return toks

    def finish(self, req_id) -> None:
        """The request is done: its blocks and its state slot are given back."""
        if self.cache.has(req_id):
            self.cache.free_request(req_id)


class DecodeGraph:
    """Static buffers and the captured HIP graph of a decode-only step of `R` requests whose
    contexts stay within `max_seq_len` tokens.

    The block-table width is fixed at its maximum and the key splits of the attention kernel follow
    `max_seq_len`, so one capture serves every step of that batch size and context bound.  The
    first run of a size executes eagerly (kernels configure themselves, the allocator warms up);
    the second is captured; later ones are replayed.  No memset node is recorded: buffers are
    written by kernels and by the upload only."""

    def __init__(self, runner: ModelRunner, R: int, max_seq_len: int):
        self.runner, self.R = runner, R
        cm = runner.cache
        dev = runner.device
        bs = cm.block_size
        self.G = len(cm.groups)
        self.MB = -(-runner.max_model_len // bs)
        G, MB = self.G, self.MB
        # int32 sections: tokens, positions, req_of_token, cu_seqlens, seq_lens, state_slots, logit_rows,
        # slot mappings, block tables, then sampling: temperature(f32) top_p(f32) top_k counters seeds(i64)
        sizes = [R, R, R, R + 1, R, R, R] + [R] * G + [R * MB] * G + [R, R, R, R, 2 * R]
        offs = [0]
        for n in sizes:
            offs.append(offs[-1] + ((n + 3) // 4) * 4)
        self.offs = offs
        self.host = torch.zeros(offs[-1], dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(offs[-1], dtype=torch.int32, device=dev)
        self.np = self.host.numpy()
        sec = lambda i, n: self.dev[offs[i]:offs[i] + n]
        self.np[offs[2]:offs[2] + R] = np.arange(R)
        self.np[offs[3]:offs[3] + R + 1] = np.arange(R + 1)
        self.np[offs[6]:offs[6] + R] = np.arange(R)
        self.ctx = StepContext(
            num_tokens=R, num_requests=R, tokens=sec(0, R), positions=sec(1, R), req_of_token=sec(2, R),
            cu_seqlens_q=sec(3, R + 1), seq_lens=sec(4, R), state_slots=sec(5, R), logit_rows=sec(6, R),
            block_tables=[sec(7 + G + g, R * MB).view(R, MB) for g in range(G)],
            slot_mappings=[sec(7 + g, R) for g in range(G)],
            q_lens=[1] * R, context_lens=[0] * R, slots_host=[0] * R, max_q_len=1,
            max_seq_len=max_seq_len, block_size=bs)
        s0 = 7 + 2 * G
        self.temperature = sec(s0, R).view(torch.float32)
        self.top_p = sec(s0 + 1, R).view(torch.float32)
        self.top_k = sec(s0 + 2, R)
        self.counters = sec(s0 + 3, R)
        self.seeds = sec(s0 + 4, 2 * R).view(torch.int64)
        self.s0 = s0
        self.out = torch.zeros(R, dtype=torch.int32, device=dev)
        self.out_host = torch.zeros(R, dtype=torch.int32, pin_memory=True)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.runs = 0
        self._tables = [[None] * R for _ in range(G)]     # (table, its length) last written per row
        # the attention kernel's query tiles of a decode step never change: one token per request
        ar = torch.arange(R, dtype=torch.int32, device=dev)
        one = torch.ones(R, dtype=torch.int32, device=dev)
        for width in range(1, 17):
            self.ctx._tiles[width] = (ar, ar, one)

    def _body(self):
        from ..kernels import ops
        logits = self.runner.decoder.forward(self.ctx)
        ops.sample(logits, self.out, self.temperature, self.top_k, self.top_p, self.seeds, self.counters)

    def run(self, req_ids, tokens, ctx_lens, params, seeds, counters, capture: bool) -> List[int]:
        R, G, MB, offs, h = self.R, self.G, self.MB, self.offs, self.np
        cm = self.runner.cache
        bs = cm.block_size
        h[offs[0]:offs[0] + R] = tokens
        h[offs[1]:offs[1] + R] = ctx_lens
        h[offs[4]:offs[4] + R] = np.asarray(ctx_lens, dtype=np.int32) + 1
        slots = [cm.slot(rid) for rid in req_ids]
        h[offs[5]:offs[5] + R] = slots
        for g in range(G):
            bt = h[offs[7 + G + g]:offs[7 + G + g] + R * MB].reshape(R, MB)
            sm = h[offs[7 + g]:offs[7 + g] + R]
            seen = self._tables[g]
            for r, (rid, c) in enumerate(zip(req_ids, ctx_lens)):
                table = cm.block_table(rid, g)
                # a row is rewritten only when it belongs to another admission than last time (the
                # table object is made when a request is admitted) or has changed length (released
                # blocks turn into -1 without a change of length, but a decode step never reads
                # them: they lie before the window)
                last = seen[r]
                if last is None or last[0] is not table or last[1] != len(table):
                    bt[r, :len(table)] = np.maximum(np.asarray(table, dtype=np.int32), 0)
                    seen[r] = (table, len(table))
                sm[r] = max(table[c // bs], 0) * bs + c % bs
        s0 = self.s0
        fview = self.host.view(torch.float32).numpy()
        fview[offs[s0]:offs[s0] + R] = [p.temperature if p.do_sample else 0.0 for p in params]
        fview[offs[s0 + 1]:offs[s0 + 1] + R] = [p.top_p for p in params]
        h[offs[s0 + 2]:offs[s0 + 2] + R] = [p.top_k for p in params]
        h[offs[s0 + 3]:offs[s0 + 3] + R] = counters
        self.host.view(torch.int64).numpy()[offs[s0 + 4] // 2:offs[s0 + 4] // 2 + R] = \
            [s & 0x7FFFFFFFFFFFFFFF for s in seeds]
        self.ctx.context_lens = list(ctx_lens)
        self.ctx.slots_host = slots
        self.dev.copy_(self.host, non_blocking=True)
        if not capture or self.runs == 0:
            self._body()
        elif self.graph is None:
            torch.cuda.synchronize()
            # Nothing may be finalised while the stream is capturing: the release of pinned buffers,
            # graphs or events of an engine that is no longer referenced is not allowed then and
            # ends the process.  So dead objects are collected now, and the collector rests until
            # the capture is over (torch.cuda.graph does not collect by itself any more).
            gc.collect()
            collecting = gc.isenabled()
            gc.disable()
            try:
                self.graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self.graph):
                    self._body()
            finally:
                if collecting:
                    gc.enable()
            self.graph.replay()
        else:
            self.graph.replay()
        self.runs += 1
        self.out_host.copy_(self.out, non_blocking=True)
        torch.cuda.current_stream().synchronize()
        return self.out_host.tolist()
