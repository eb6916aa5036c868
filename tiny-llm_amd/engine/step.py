"""The step function: one batch of (request, its next tokens) through the model.

A step runs only the tokens it is given, against the cache that earlier steps
left, and returns the logits at the wanted places (`step`) or the tokens sampled
from them on the device (`run`).  Entries may be portions of prompts beside single
decoded tokens, cut anywhere.  The reference's runtime needs five calls and allows
either whole prompts from position 0 or exactly one token per request
(tiny_llm/pipeline/pipeline.cpp:132-140, 184-190,
tiny_llm/runtime/cuda/cuda_runtime.cpp:673, 690); here it is one call for any mix.

Step metadata is laid out by ONE routine (`Layout`, `fill_metadata`) in one pinned
int32 buffer and uploaded with one copy (the reference uploads a block table per
layer with a stream sync each, cuda_runtime.cpp:758-773).  Token rows map to
requests through `req_of_token`, so kernels need no search over sequence
separators (tiny_llm/ops/details.hpp:19-36).

A step runs eagerly or as a HIP graph.  A graph is captured per shape of step:
decode-only steps by (requests, bound on the context), other steps by capacities
(tokens, requests, wanted rows) to which the step is padded: padding tokens write
no cache slot, padding query tiles hold no token, padding rows of the output are
dropped.  Eager and captured steps share the layout routine, the model code and
the sampler; a captured step only has its sizes rounded up and its buffers static.
A model that holds a part which may not be captured still runs as graphs: one for each
run of stages that may be, the other stages eagerly between them on the same buffers.
"""
from __future__ import annotations

import gc
from collections import OrderedDict
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import CacheManager
from ..kernels import ops


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()        # places among `tokens` whose logits are asked for


@dataclass
class SampleSpec:
    """How the token of one wanted row is chosen on the device: temperature <= 0 is the first
    maximum; else temperature -> top-k -> top-p -> multinomial with the uniform number of
    (seed, counter)."""
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int = 0
    counter: int = 0


@dataclass
class StepContext:
    """Who is in the batch and where each token sits; device tensors are int32.
    In a captured step the sizes are capacities, and the host copies are this step's only while a
    part runs eagerly (a step's first run, or a part that may not be captured)."""
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
    static: bool = False            # a captured step: nothing may be built on the host any more
    logits_all_rows: bool = False   # logit_rows is 0, 1, 2, ...: every token's logits, in order (no gather needed)
    _tiles: Dict[int, tuple] = field(default_factory=dict)
    _on_new_width = None            # told when a tile width is asked for the first time

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1

    def attention_tiles(self, tokens_per_tile: int):
        """(tile_req, tile_tok0, tile_ntok) int32 device tensors: every request's tokens of this
        step cut into groups of at most `tokens_per_tile` (the query tiles of the MFMA attention
        kernels).  Widths that earlier steps asked for came with the step's upload; a new width is
        built here, once, and remembered for the steps to come."""
        if tokens_per_tile not in self._tiles:
            if self.static:
                raise StepError(f"query tiles of {tokens_per_tile} tokens were not laid out for this captured step")
            req, tok0, ntok = tile_lists(self.q_lens, tokens_per_tile)
            packed = torch.tensor([req, tok0, ntok], dtype=torch.int32).to(self.tokens.device, non_blocking=True)
            self._tiles[tokens_per_tile] = (packed[0], packed[1], packed[2])
            if self._on_new_width is not None:
                self._on_new_width(tokens_per_tile)
        return self._tiles[tokens_per_tile]


class StepError(ValueError):
    pass


def tile_lists(q_lens: Sequence[int], width: int):
    """Every request's tokens cut into groups of at most `width`: (request, first token row, count)."""
    req, tok0, ntok = [], [], []
    t = 0
    for r, n in enumerate(q_lens):
        for s in range(0, n, width):
            req.append(r)
            tok0.append(t + s)
            ntok.append(min(width, n - s))
        t += n
    return req, tok0, ntok


# ----------------------------------------------------------------------- layout
class Layout:
    """Where every section of a step's metadata lies in its int32 buffer, for given capacities:
    T tokens, R requests, n_out wanted rows, G cache groups with block tables MB wide, query-tile
    lists by width, and (optionally) the sampler's per-row arguments.  Sections start on 16 bytes."""

    def __init__(self, T: int, R: int, n_out: int, G: int, MB: int, tile_caps: Dict[int, int], sampling: bool):
        self.T, self.R, self.n_out, self.G, self.MB = T, R, n_out, G, MB
        self.tile_caps = dict(tile_caps)
        self.sampling = sampling
        self.off: Dict[str, Tuple[int, int]] = {}
        at = 0

        def add(name, n):
            nonlocal at
            self.off[name] = (at, n)
            at += ((n + 3) // 4) * 4

        for name, n in (("tokens", T), ("positions", T), ("req_of_token", T), ("cu_seqlens", R + 1), ("seq_lens", R),
                        ("state_slots", R), ("logit_rows", n_out)):
            add(name, n)
        for g in range(G):
            add(f"slots{g}", T)
        for g in range(G):
            add(f"tables{g}", R * MB)
        for w, cap in self.tile_caps.items():
            add(f"tiles{w}", 3 * cap)
        if sampling:
            for name in ("temperature", "top_p", "top_k", "counters"):
                add(name, n_out)
            add("seeds", 2 * n_out)         # int64
            add("burst_step", 1)            # decode steps run on the device since this upload
        self.total = at

    def sec(self, buf, name: str):
        o, n = self.off[name]
        return buf[o:o + n]

    def context(self, dev: torch.Tensor, block_size: int, **host) -> StepContext:
        """The device views of an uploaded buffer as a StepContext."""
        T, R, G, MB = self.T, self.R, self.G, self.MB
        ctx = StepContext(
            num_tokens=T, num_requests=R, tokens=self.sec(dev, "tokens"), positions=self.sec(dev, "positions"),
            req_of_token=self.sec(dev, "req_of_token"), cu_seqlens_q=self.sec(dev, "cu_seqlens"),
            seq_lens=self.sec(dev, "seq_lens"), state_slots=self.sec(dev, "state_slots"),
            logit_rows=self.sec(dev, "logit_rows") if self.n_out else None,
            block_tables=[self.sec(dev, f"tables{g}").view(R, MB) for g in range(G)],
            slot_mappings=[self.sec(dev, f"slots{g}") for g in range(G)], block_size=block_size, **host)
        for w, cap in self.tile_caps.items():
            t = self.sec(dev, f"tiles{w}")
            ctx._tiles[w] = (t[:cap], t[cap:2 * cap], t[2 * cap:3 * cap])
        return ctx

    def sampler_args(self, dev: torch.Tensor):
        n = self.n_out
        return (self.sec(dev, "temperature").view(torch.float32), self.sec(dev, "top_k"),
                self.sec(dev, "top_p").view(torch.float32), self.sec(dev, "seeds").view(torch.int64),
                self.sec(dev, "counters"))


@dataclass
class _Row:
    """One entry of a step, resolved against the cache."""
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int]
    context_len: int            # tokens cached before the step
    slot: int
    tables: List[List[int]]     # per cache group


class SeenTables:
    """What a static step buffer already holds of the requests' block tables: per cache group and
    request row the table object and the length that were written last.  A table only ever grows
    between two admissions, except when a step that did not run is undone: the cache manager's
    `table_epoch` goes up then, and everything remembered under an older epoch is forgotten (a
    table cut back and grown again has its old length with other blocks)."""

    def __init__(self, groups: int, rows: int, epoch: int = 0):
        self.groups, self.rows_per_group = groups, rows
        self.epoch = epoch
        self.rows: List[list] = [[None] * rows for _ in range(groups)]

    def at_epoch(self, epoch: int) -> List[list]:
        if epoch != self.epoch:
            self.rows = [[None] * self.rows_per_group for _ in range(self.groups)]
            self.epoch = epoch
        return self.rows


def fill_metadata(host: np.ndarray, lay: Layout, rows: Sequence[_Row], block_size: int,
                  samples: Optional[Sequence[SampleSpec]] = None, seen: Optional[SeenTables] = None,
                  table_epoch: int = 0) -> None:
    """Writes the metadata of a step into `host` (int32, at least lay.total long): the ONE routine
    behind eager steps, captured decode steps and captured mixed steps.

    Capacities beyond the step's own sizes are padded so that the same kernels run unchanged:
    padding tokens are token 0 at position 0 of request row 0 with cache slot -1 (nothing is
    stored); padding requests have no tokens (cu_seqlens stays at T); padding query tiles hold no
    token; padding output rows point at row 0 and are dropped by the caller.
    `seen`: the block-table rows a static buffer already holds, valid for the cache manager's
    `table_epoch` under which they were written."""
    T_cap, R_cap, G, MB, bs = lay.T, lay.R, lay.G, lay.MB, block_size
    seen = seen.at_epoch(table_epoch) if seen is not None else None
    R = len(rows)
    tok, pos, rot = lay.sec(host, "tokens"), lay.sec(host, "positions"), lay.sec(host, "req_of_token")
    cu, sl, ss, lr = (lay.sec(host, n) for n in ("cu_seqlens", "seq_lens", "state_slots", "logit_rows"))
    sms = [lay.sec(host, f"slots{g}") for g in range(G)]
    bts = [lay.sec(host, f"tables{g}").reshape(R_cap, MB) for g in range(G)]
    t = k = 0
    q_lens = []
    for r, row in enumerate(rows):
        n, c = len(row.tokens), row.context_len
        tok[t:t + n] = row.tokens
        cu[r] = t
        sl[r] = c + n
        ss[r] = row.slot
        for w in row.want:
            lr[k] = t + int(w)
            k += 1
        if n == 1:
            pos[t] = c
            rot[t] = r
        else:
            pos[t:t + n] = np.arange(c, c + n, dtype=np.int32)
            rot[t:t + n] = r
        for g in range(G):
            table = row.tables[g]
            if len(table) > MB:
                raise StepError(f"request {row.req_id!r} holds {len(table)} blocks, the table has room for {MB}")
            last = seen[g][r] if seen is not None else None
            # a row is rewritten only when it belongs to another admission than last time (the table
            # object is made when a request is admitted) or has changed length (within one epoch a
            # table only grows); blocks that a window has released turn into -1 without a change of
            # length, but they lie before the window and are never read
            if last is None or last[0] is not table or last[1] != len(table):
                bts[g][r, :len(table)] = np.maximum(np.asarray(table, dtype=np.int32), 0)
                if seen is not None:
                    seen[g][r] = (table, len(table))
            if n == 1:
                sms[g][t] = max(table[c // bs], 0) * bs + c % bs
            else:
                p = np.arange(c, c + n, dtype=np.int32)
                sms[g][t:t + n] = np.maximum(np.asarray(table, dtype=np.int32), 0)[p // bs] * bs + p % bs
        q_lens.append(n)
        t += n
    T = t
    if T < T_cap:
        tok[T:T_cap] = 0
        pos[T:T_cap] = 0
        rot[T:T_cap] = 0
        for g in range(G):
            sms[g][T:T_cap] = -1
    cu[R:R_cap + 1] = T
    if R < R_cap:
        sl[R:R_cap] = 0
        ss[R:R_cap] = 0
    if k < lay.n_out:
        lr[k:lay.n_out] = 0
    for w, cap in lay.tile_caps.items():
        req, tok0, ntok = tile_lists(q_lens, w)
        m = len(req)
        if m > cap:
            raise StepError(f"{m} query tiles of {w} tokens, the layout has room for {cap}")
        sec = lay.sec(host, f"tiles{w}")
        sec[0:m], sec[cap:cap + m], sec[2 * cap:2 * cap + m] = req, tok0, ntok
        sec[m:cap], sec[cap + m:2 * cap], sec[2 * cap + m:3 * cap] = 0, 0, 0
    if lay.sampling:
        n_out = lay.n_out
        fl = host.view(np.float32)
        o_t, o_p = lay.off["temperature"][0], lay.off["top_p"][0]
        tk, ct = lay.sec(host, "top_k"), lay.sec(host, "counters")
        sd = host.view(np.int64)[lay.off["seeds"][0] // 2: lay.off["seeds"][0] // 2 + n_out]
        m = len(samples) if samples is not None else 0
        if m:
            fl[o_t:o_t + m] = [s.temperature for s in samples]
            fl[o_p:o_p + m] = [s.top_p for s in samples]
            tk[:m] = [s.top_k for s in samples]
            ct[:m] = [s.counter for s in samples]
            sd[:m] = [s.seed & 0x7FFFFFFFFFFFFFFF for s in samples]
        if m < n_out:
            fl[o_t + m:o_t + n_out] = 0.0
            fl[o_p + m:o_p + n_out] = 1.0
            tk[m:], ct[m:], sd[m:] = 0, 0, 0
        lay.sec(host, "burst_step")[0] = 0


def token_capacity(n: int, limit: int) -> int:
    """The token count a captured step is padded to: steps of 16 up to 64 (the few-row products'
    own steps), of 64 up to 1024, of 256 beyond."""
    step = 16 if n <= 64 else (64 if n <= 1024 else 256)
    return min(-(-n // step) * step, max(limit, n))


def power_of_two_at_least(n: int) -> int:
    p = 1
    while p < n:
        p *= 2
    return p


# ----------------------------------------------------------------------- runner
class ModelRunner:
    """Owns the decoder's cache views and turns step entries into one forward pass."""

    # Shapes of step whose static buffers and graphs are kept.  A serving run meets a few dozen
    # (batch sizes while requests end one after the other, portions, bounds on the context); each
    # holds a pinned and a device copy of its metadata and up to two graphs.  The shape used
    # longest ago goes when a new one would exceed the number.
    MAX_STEP_SHAPES = 64

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
        self.workspace = ops.Workspace(self.device, self.max_tokens)
        self._pinned: Optional[torch.Tensor] = None
        self._uploaded: Optional[torch.cuda.Event] = None
        # captured steps by shape, least recently used first; at most MAX_STEP_SHAPES are kept
        self._graphs: "OrderedDict[tuple, StepGraph]" = OrderedDict()
        self._graph_pool = None
        self._tile_widths: set = set()          # query-tile widths the model's kernels have asked for
        self.last_logits: Optional[torch.Tensor] = None     # of the last `run` (tests look at it)
        self.graph_steps = 0
        self.eager_steps = 0

    # ---------------------------------------------------------------- validation
    def _resolve(self, entries: Sequence[StepEntry], reserve: int = 0) -> Tuple[List[_Row], int]:
        """Checks the entries, takes the cache blocks they need (all or nothing); `reserve`: blocks
        for that many positions per request instead of for the tokens it brings."""
        cm = self.cache
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
            c = cm.num_tokens(e.req_id) if cm.has(e.req_id) else 0
            if c + max(n, reserve) > self.max_model_len:
                raise StepError(f"request {e.req_id!r} would reach {c + max(n, reserve)} tokens, "
                                f"the limit is {self.max_model_len}")
            T += n
        if T > self.max_tokens:
            raise StepError(f"step brings {T} tokens, the budget is {self.max_tokens}")
        ctx_lens = cm.reserve_step([(e.req_id, max(len(e.tokens), reserve)) for e in entries])
        G = len(cm.groups)
        rows = [_Row(e.req_id, e.tokens, e.want, c, cm.slot(e.req_id), [cm.block_table(e.req_id, g) for g in range(G)])
                for e, c in zip(entries, ctx_lens)]
        return rows, T

    def _host_buffer(self, n: int) -> torch.Tensor:
        if self._pinned is None or self._pinned.numel() < n:
            self._pinned = torch.empty(max(n, 1 << 16), dtype=torch.int32, pin_memory=True)
        return self._pinned[:n]

    def _new_width(self, w: int) -> None:
        self._tile_widths.add(w)

    def _tile_caps(self, T: int, R: int, decode_only: bool) -> Dict[int, int]:
        """Room for the query tiles of every width the kernels use (none in decode-only steps,
        where row i is request i)."""
        if decode_only:
            return {}
        return {w: -(-T // w) + R for w in sorted(self._tile_widths)}

    # ------------------------------------------------------------------- eager
    def prepare(self, entries: Sequence[StepEntry], samples: Optional[Sequence[SampleSpec]] = None):
        """Reserves cache, lays the step out at its exact sizes and uploads it.
        Returns (context, layout, device buffer, rows)."""
        rows, T = self._resolve(entries)
        try:
            bs = self.cache.block_size
            R, G = len(rows), len(self.cache.groups)
            max_blocks = max(1, max(len(tb) for row in rows for tb in row.tables) if G else 1)
            n_out = sum(len(r.want) for r in rows)
            q_lens = [len(r.tokens) for r in rows]
            decode_only = max(q_lens) == 1
            tile_caps = {} if decode_only else {w: len(tile_lists(q_lens, w)[0]) for w in sorted(self._tile_widths)}
            lay = Layout(T, R, n_out, G, max_blocks, tile_caps, samples is not None)
            if self._uploaded is not None:
                self._uploaded.synchronize()      # the last step's upload has left the pinned buffer
            buf = self._host_buffer(lay.total)
            host = buf.numpy()
            host[:lay.total] = 0
            fill_metadata(host, lay, rows, bs, samples)
            dev = buf.to(self.device, non_blocking=True)
            self._uploaded = torch.cuda.Event()
            self._uploaded.record()
            ctx_lens = [r.context_len for r in rows]
            ctx = lay.context(dev, bs, q_lens=q_lens, context_lens=ctx_lens, slots_host=[r.slot for r in rows],
                              max_q_len=max(q_lens), max_seq_len=max(c + n for c, n in zip(ctx_lens, q_lens)))
            ctx._on_new_width = self._new_width
            return ctx, lay, dev, rows
        except BaseException:
            self.cache.undo_reservation()
            raise

    def _forward(self, ctx: StepContext) -> torch.Tensor:
        with ops.use_workspace(self.workspace):
            return self.decoder.forward(ctx)

    @property
    def graphs_possible(self) -> bool:
        """Whether a step can run as HIP graphs: as one, if every part may be captured, or as the
        capturable runs of its stages with the others eagerly between them."""
        return any(safe for safe, _, _ in self.decoder.graph_runs())

    def _commit(self, rows: Sequence[_Row]) -> None:
        for r in rows:
            self.cache.commit(r.req_id, r.context_len + len(r.tokens))
        self.cache.forget_reservation()

    def step(self, entries: Sequence[StepEntry], use_graph: bool = False) -> torch.Tensor:
        """Runs the entries as one batch.  Returns float32 logits [wanted, vocab] on the
        device, in the order of the entries and of each entry's `want`.  If the forward pass
        raises, the cache is as it was before the call."""
        if use_graph and self.graphs_possible:
            return self._graph_step(entries, None)[0]
        ctx, _, _, rows = self.prepare(entries)
        try:
            logits = self._forward(ctx)
        except BaseException:
            self.cache.undo_reservation()
            raise
        self._commit(rows)
        self.eager_steps += 1
        return logits

    def run(self, entries: Sequence[StepEntry], samples: Sequence[SampleSpec], use_graph: bool = True) -> List[int]:
        """Runs the entries and chooses a token for every wanted row on the device (`samples` has
        one SampleSpec per wanted row, in order).  Returns the tokens.  With `use_graph` the whole
        step, model and sampler, is a HIP graph per shape of step, replayed on static buffers: only
        the metadata upload and the token download remain on the host."""
        n_out = sum(len(e.want) for e in entries)
        if len(samples) != n_out:
            raise StepError(f"{n_out} rows are wanted, {len(samples)} sampling settings were given")
        if use_graph and self.graphs_possible:
            return self._graph_step(entries, samples)[1]
        ctx, lay, dev, rows = self.prepare(entries, samples)
        try:
            logits = self._forward(ctx)
            out = torch.empty(n_out, dtype=torch.int32, device=self.device)
            if n_out:
                ops.sample(logits, out, *lay.sampler_args(dev))
        except BaseException:
            self.cache.undo_reservation()
            raise
        self._commit(rows)
        self.eager_steps += 1
        self.last_logits = logits
        return out.cpu().tolist()

    def run_burst(self, entries: Sequence[StepEntry], samples: Sequence[SampleSpec], steps: int):
        """`steps` decode steps back to back without the host in between: every entry is one
        decoded token whose logits are wanted; after each step the device turns the step's metadata
        into the next one's (`ops.decode_advance`: sampled token in, position and counter up, cache
        slot looked up), so only the first step's metadata is uploaded and only the tokens of all
        steps come back, once.  Cache blocks for all `steps` positions are taken up front.
        Returns the tokens by step, [steps][entries], or None if these steps cannot run as a burst
        (no captured graph of this shape yet, too many cache groups): the caller then runs one step."""
        if steps < 2 or not self.decoder.graph_safe or len(self.cache.groups) > ops.MAX_CACHE_GROUPS:
            return None
        if not all(len(e.tokens) == 1 and len(e.want) == 1 for e in entries) or len(samples) != len(entries):
            return None
        cm = self.cache
        new_max = max((cm.num_tokens(e.req_id) if cm.has(e.req_id) else 0) for e in entries) + steps
        R = len(entries)
        bound = min(max(512, power_of_two_at_least(new_max)), max(self.max_model_len, 1))
        sg = self._step_graph(("decode", R, bound, True))
        if sg is None or sg.graph is None or new_max > bound or steps > sg.history_steps:
            return None
        rows, _ = self._resolve(entries, reserve=steps)
        try:
            toks = sg.burst(rows, samples, steps)
        except BaseException:
            self.cache.undo_reservation()
            raise
        for r in rows:
            self.cache.commit(r.req_id, r.context_len + steps)
        self.cache.forget_reservation()
        self.graph_steps += steps
        return toks

    # ------------------------------------------------------------------ graphs
    def _graph_step(self, entries: Sequence[StepEntry], samples: Optional[Sequence[SampleSpec]]):
        rows, T = self._resolve(entries)
        try:
            R = len(rows)
            n_out = sum(len(r.want) for r in rows)
            decode_only = all(len(r.tokens) == 1 for r in rows)
            new_lens = [r.context_len + len(r.tokens) for r in rows]
            if decode_only and all(len(r.want) == 1 for r in rows):      # row i of the logits is request i
                # exact sizes; the bound on the context (a power of two, at least 512) decides into how
                # many workgroups the attention kernel splits a request's keys, which is fixed at capture
                bound = min(max(512, power_of_two_at_least(max(new_lens))), max(self.max_model_len, 1))
                bound = max(bound, max(new_lens))
                key = ("decode", R, bound, samples is not None)
                caps = (R, R, R, 1, bound)
            else:
                T_cap = token_capacity(T, self.max_tokens)
                R_cap = min(power_of_two_at_least(R), max(self.cache.max_seqs, R))
                # every row may be wanted (replay), or at most one per request (serving)
                n_cap = R_cap if n_out <= R_cap and samples is not None else T_cap
                # the bound on the context decides whether attention shares a tile's keys out
                bound = max(min(max(512, power_of_two_at_least(max(new_lens))), max(self.max_model_len, 1)), max(new_lens))
                key = ("mixed", T_cap, R_cap, n_cap, bound, samples is not None)
                caps = (T_cap, R_cap, n_cap, T_cap, bound)
            sg = self._step_graph(key)
            if sg is None:
                sg = self._graphs[key] = StepGraph(self, *caps, sampling=samples is not None)
                while len(self._graphs) > self.MAX_STEP_SHAPES:
                    self._graphs.popitem(last=False)        # no capture is under way here: it may be released
            logits, toks = sg.run(rows, samples, n_out)
        except BaseException:
            self.cache.undo_reservation()
            raise
        self._commit(rows)
        return logits, toks

    def _step_graph(self, key) -> Optional["StepGraph"]:
        sg = self._graphs.get(key)
        if sg is not None:
            self._graphs.move_to_end(key)
        return sg

    def finish(self, req_id) -> None:
        """The request is done: its blocks and its state slot are given back."""
        if self.cache.has(req_id):
            self.cache.free_request(req_id)


class StepGraph:
    """Static buffers and the captured HIP graph of steps of one shape: capacities of T tokens,
    R requests and n_out wanted rows, `max_q_len` 1 (decode: row i is request i) or more, contexts
    within `max_seq_len`.

    The block-table width is fixed at its maximum.  The first run of a shape executes eagerly on the
    static buffers (kernels configure themselves, the workspace grows, the tile widths the kernels
    ask for become known); the second is captured; later ones are replayed.  No memset node is
    recorded: buffers are written by kernels and by the upload only.  A shape whose capture fails
    (a part asks for something that was not laid out) keeps running eagerly."""

    def __init__(self, runner: ModelRunner, T: int, R: int, n_out: int, max_q_len: int, max_seq_len: int,
                 sampling: bool):
        self.runner = runner
        self.T, self.R, self.n_out = T, R, n_out
        self.max_q_len, self.max_seq_len, self.sampling = max_q_len, max_seq_len, sampling
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.chain: Optional[torch.cuda.CUDAGraph] = None      # CHAIN steps of a burst as one graph
        self.capture_failed = False
        self.chain_failed = False
        self.runs = 0
        self.logits: Optional[torch.Tensor] = None
        self._build()

    def _build(self) -> None:
        """(Re)lays the static buffers out for the tile widths known by now."""
        runner = self.runner
        cm = runner.cache
        G = len(cm.groups)
        MB = -(-runner.max_model_len // cm.block_size)
        self.layout = Layout(self.T, self.R, self.n_out, G, MB,
                             runner._tile_caps(self.T, self.R, self.max_q_len == 1), self.sampling)
        self.widths = set(self.layout.tile_caps)
        self.host = torch.zeros(self.layout.total, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(self.layout.total, dtype=torch.int32, device=runner.device)
        self.np = self.host.numpy()
        self.ctx = self.layout.context(self.dev, cm.block_size, q_lens=[], context_lens=[], slots_host=[],
                                       max_q_len=self.max_q_len, max_seq_len=self.max_seq_len)
        # decode with a wanted row per request: row i of the logits is token i (padding rows, which would
        # point at row 0, are dropped by the caller either way), so the head needs no gather of rows
        self.ctx.logits_all_rows = self.max_q_len == 1 and self.n_out == self.R == self.T
        self.seen = SeenTables(G, self.R, cm.table_epoch)
        self.out = torch.zeros(max(self.n_out, 1), dtype=torch.int32, device=runner.device)
        self.out_host = torch.zeros(max(self.n_out, 1), dtype=torch.int32, pin_memory=True)
        # a decode step with its sampler ends by preparing the next one on the device (bursts)
        self.feeds_next = (self.max_q_len == 1 and self.sampling and self.n_out == self.R == self.T
                           and G <= ops.MAX_CACHE_GROUPS and runner.decoder.graph_safe)
        self.history_steps = self.BURST_STEPS if self.feeds_next else 0
        if self.feeds_next:
            self.history = torch.zeros(self.history_steps * self.R, dtype=torch.int32, device=runner.device)
            self.history_host = torch.zeros(self.history_steps * self.R, dtype=torch.int32, pin_memory=True)
        self.graph = None
        self.chain = None
        self.bursts = 0         # runs of steps this shape has served
        self._uploaded: Optional[torch.cuda.Event] = None
        # A model with a part that may not be captured: the runs of its stages, one graph for each
        # capturable run and the place where each run leaves the residual stream for the next.
        runs = runner.decoder.graph_runs()
        self.stage_runs = None if len(runs) == 1 and runs[0][0] else runs
        self.run_graphs: List[Optional[torch.cuda.CUDAGraph]] = [None] * len(runs)
        self.run_out: List[Optional[torch.Tensor]] = [None] * len(runs)
        self.runs_captured = False

    BURST_STEPS = 32        # most decode steps a burst may hold

    def _body(self):
        self.logits = self.runner._forward(self.ctx)
        self._tail()

    def _tail(self):
        """Behind the logits: the sampler and, in a decode step that may be chained, the next step's metadata."""
        if self.sampling and self.n_out:
            ops.sample(self.logits, self.out[:self.n_out], *self.layout.sampler_args(self.dev))
        if self.feeds_next:
            lay, ctx = self.layout, self.ctx
            ops.decode_advance(ctx.tokens, ctx.positions, ctx.seq_lens, lay.sec(self.dev, "counters"), self.out,
                               self.history, lay.sec(self.dev, "burst_step"), ctx.slot_mappings,
                               ctx.block_tables, ctx.block_size)

    def _stage_run(self, first: int, last: int, x):
        """Stages first .. last - 1 on the static buffers; the last run ends with the sampler."""
        runner = self.runner
        with ops.use_workspace(runner.workspace):
            y = runner.decoder.run_stages(self.ctx, first, last, x)
        if last == runner.decoder.num_stages:
            self.logits = y
            self._tail()
        return y

    def _body_in_runs(self, capture: bool) -> None:
        """The step of a model that holds a part which may not be captured: every capturable run of
        stages replays its graph (or is captured now and then replayed), the others run eagerly on the
        same static buffers.  What an eager run leaves has a new address every time, so it is copied
        to a fixed place, from which the graph behind it reads."""
        runner = self.runner
        x = None
        for k, (safe, first, last) in enumerate(self.stage_runs):
            if safe and self.run_graphs[k] is None and capture:
                self.ctx.static = True
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, pool=runner._graph_pool):
                    self.run_out[k] = self._stage_run(first, last, x)
                self.run_graphs[k] = graph
            if safe and self.run_graphs[k] is not None:
                self.run_graphs[k].replay()
                x = self.run_out[k]
                continue
            self.ctx.static = False
            y = self._stage_run(first, last, x)
            if last < runner.decoder.num_stages:
                if self.run_out[k] is None or self.run_out[k].shape != y.shape or self.run_out[k].dtype != y.dtype:
                    self.run_out[k] = torch.empty_like(y)
                self.run_out[k].copy_(y)
                y = self.run_out[k]
            x = y

    def burst(self, rows: Sequence[_Row], samples, steps: int) -> List[List[int]]:
        """Uploads the first step's metadata and replays the captured step `steps` times; each
        replay leaves the next step's metadata behind.  Returns the tokens by step."""
        runner = self.runner
        if self._uploaded is not None:
            self._uploaded.synchronize()
        fill_metadata(self.np, self.layout, rows, runner.cache.block_size, samples, self.seen,
                      runner.cache.table_epoch)
        self.dev.copy_(self.host, non_blocking=True)
        left = steps
        if self.chain is not None:
            while left >= self.CHAIN:       # several steps a launch: the gap between two launches is paid once for them
                self.chain.replay()
                left -= self.CHAIN
        for _ in range(left):
            self.graph.replay()
        n = steps * self.R
        self.history_host[:n].copy_(self.history[:n], non_blocking=True)
        torch.cuda.current_stream().synchronize()
        self._uploaded = None
        self.runs += steps
        self.bursts += 1
        flat = self.history_host[:n].tolist()
        if self.chain is None and not self.chain_failed:
            self._capture_chain()       # behind the shape's first run, of whatever length: see there
        return [flat[k * self.R:(k + 1) * self.R] for k in range(steps)]

    def run(self, rows: Sequence[_Row], samples, n_out: int):
        runner = self.runner
        if self.graph is None and not self.runs_captured and self.max_q_len > 1 and self.widths != runner._tile_widths:
            self._build()                       # a kernel asked for a tile width this layout lacks
        if self._uploaded is not None:
            self._uploaded.synchronize()        # the last upload has left the pinned buffer
        fill_metadata(self.np, self.layout, rows, runner.cache.block_size, samples, self.seen,
                      runner.cache.table_epoch)
        self.dev.copy_(self.host, non_blocking=True)
        self._uploaded = torch.cuda.Event()
        self._uploaded.record()
        if self.graph is not None:
            self.graph.replay()
            runner.graph_steps += 1
        elif self.runs == 0 or self.capture_failed:
            # eager on the static buffers; the host copies a part may look at are those of this step
            self.ctx.static = False
            self._host_copies(rows)
            self.ctx._on_new_width = runner._new_width
            if self.max_q_len > 1:
                for w in runner._tile_widths - self.widths:
                    self.ctx._tiles.pop(w, None)
            known = set(self.ctx._tiles)
            self._body()
            for w in set(self.ctx._tiles) - known:      # built for this step only: not part of the layout
                del self.ctx._tiles[w]
            runner.eager_steps += 1
        elif self.stage_runs is not None:
            # graphs for the capturable runs of stages (captured at this shape's second step), the
            # other runs eagerly between them with this step's host copies
            self._host_copies(rows)
            known = set(self.ctx._tiles)
            if self.runs_captured:
                self._body_in_runs(capture=False)
            else:
                self._capture_runs()
            for w in set(self.ctx._tiles) - known:
                del self.ctx._tiles[w]
            runner.graph_steps += 1
        else:
            self._capture()
            runner.graph_steps += 1
        self.runs += 1
        toks: List[int] = []
        if self.sampling and n_out:
            self.out_host.copy_(self.out, non_blocking=True)
            torch.cuda.current_stream().synchronize()
            toks = self.out_host[:n_out].tolist()
            runner.last_logits = self.logits[:n_out]
            return None, toks
        # the logits live in memory the next replay overwrites: the caller gets a copy
        return self.logits[:n_out].clone(), toks

    def _host_copies(self, rows: Sequence[_Row]) -> None:
        """What a part that runs eagerly may read on the host: this step's lengths and slots."""
        pad = [0] * (self.R - len(rows))
        self.ctx.q_lens = [len(r.tokens) for r in rows] + pad
        self.ctx.context_lens = [r.context_len for r in rows] + pad
        self.ctx.slots_host = [r.slot for r in rows] + pad

    def _capture_runs(self) -> None:
        """Captures the capturable runs of stages, one graph each, while the step runs."""
        runner = self.runner
        torch.cuda.synchronize()
        collecting = gc.isenabled()
        gc.disable()                        # as in _capture: nothing may be finalised during a capture
        self.ctx._on_new_width = None
        if runner._graph_pool is None:
            runner._graph_pool = torch.cuda.graph_pool_handle()
        try:
            self._body_in_runs(capture=True)
            self.runs_captured = True
        except StepError:
            # a part asked for something that was not laid out: this shape keeps running eagerly
            self.capture_failed = True
            self.run_graphs = [None] * len(self.run_graphs)
            self.ctx.static = False
            torch.cuda.synchronize()
            self._body()
        finally:
            if collecting:
                gc.enable()

    CHAIN = 4               # decode steps captured as ONE graph for bursts

    def _capture_chain(self) -> None:
        """Captures CHAIN decode steps as one graph for runs of steps (each step's last kernel
        prepares the next step's metadata, so the body simply repeats).  Nothing runs.  It is
        captured behind the first run of steps of this shape, however short: a shape that is
        replayed in runs stays, and its later runs pay for no capture; a shape that a batch passes
        through once (requests ending one after the other) never pays for this one."""
        runner = self.runner
        torch.cuda.synchronize()
        collecting = gc.isenabled()
        gc.disable()                        # as in _capture: nothing may be finalised during a capture
        graph = torch.cuda.CUDAGraph()
        try:
            with torch.cuda.graph(graph, pool=runner._graph_pool):
                for _ in range(self.CHAIN):
                    self._body()
        except StepError:
            self.chain_failed = True
            torch.cuda.synchronize()
            return
        finally:
            if collecting:
                gc.enable()
        self.chain = graph

    def _capture(self) -> None:
        runner = self.runner
        torch.cuda.synchronize()
        # Nothing may be finalised while the stream is capturing: the release of pinned buffers,
        # graphs or events of an engine that is no longer referenced is not allowed then and
        # ends the process.  So the collector rests until the capture is over; what is dead waits
        # for its next turn.  (A collection here, ahead of every capture, took 20 to 50 ms, more
        # than the capture itself.)
        collecting = gc.isenabled()
        gc.disable()
        self.ctx.static = True
        self.ctx._on_new_width = None
        graph = torch.cuda.CUDAGraph()
        if runner._graph_pool is None:
            runner._graph_pool = torch.cuda.graph_pool_handle()
        try:
            # all graphs of a runner share one memory pool: one runs at a time, and what a step
            # returns has left the pool (tokens on the host, logits copied) before the next replay
            with torch.cuda.graph(graph, pool=runner._graph_pool):
                self._body()
        except StepError:
            self.capture_failed = True
            self.ctx.static = False
            torch.cuda.synchronize()
            self._body()
            return
        finally:
            if collecting:
                gc.enable()
        self.graph = graph
        graph.replay()
