"""The cache manager: paged keys and values with a block table per request, in
groups of layers with the same needs, and slots for per-request state of fixed size.

Differences from the reference, which keeps one pool per layer sized so that it can
never run out and frees everything when the whole batch is done
(tiny_llm/runtime/cuda/cuda_runtime.cpp:505-526, 683-709, 804-819):

* Layers whose mixers declare the same CacheSpec form a group.  A group has ONE
  block-id space and one block table per request that serves all its layers; each
  layer has its own tensors, the ones its CacheSpec describes (keys and values
  [blocks, kv_heads, block_size, head_dim] for attention), indexed by those ids.
* A "window" group gives a request's blocks back as soon as every position in them
  is more than `window` behind the next query; a "full" group when the request ends.
* Blocks that are given back are used again by later growth, most recently freed first.
* `grow` is all-or-nothing over all groups, so a step that cannot be held changes nothing.
* Every group has a pool of its own size: a window group never holds more of a request than
  its window and the portion in hand, so its pool may be much smaller than a full group's.
* A step that did not run is undone: tables are cut back, admitted requests leave, and the
  per-request state that the step's parts may already have written is put back.

Everything here is host bookkeeping; device tensors are only allocated (by
`allocate_tensors`) and handed to the mixers as views.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Mapping, Optional, Sequence, Tuple

import torch

from ..parts.base import CacheSpec, LayerCache, StateSpec
from .block_pool import BlockPool, CacheError, OutOfBlocks

RELEASED = -1


class NoFreeSlot(CacheError):
    pass


@dataclass
class CacheGroup:
    spec: CacheSpec
    entries: List[Hashable]            # owners (runs of layers) that keep a cache in this group
    pool: BlockPool
    # by tensor name: [len(entries), blocks, *page_shape]
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)

    def elements_per_block(self, block_size: int) -> int:
        """Elements one block takes over all owners and tensors of the group."""
        per_token = sum(math.prod(t.shape) for t in self.spec.tensors)
        return len(self.entries) * per_token * block_size


@dataclass
class RequestCache:
    slot: int
    num_tokens: int = 0
    blocks: List[List[int]] = field(default_factory=list)   # per group: logical block -> id or RELEASED


def group_specs(cache_specs) -> Tuple[List[CacheSpec], List[List[Hashable]]]:
    """The groups that owners with these cache specs form, in order of first appearance:
    (spec of each group, owners of each group)."""
    if not isinstance(cache_specs, Mapping):
        cache_specs = {i: c for i, c in enumerate(cache_specs) if c is not None}
    specs: List[CacheSpec] = []
    owners: List[List[Hashable]] = []
    by_key: Dict[Tuple, int] = {}
    for i, cs in cache_specs.items():
        key = cs.group_key()
        if key not in by_key:
            by_key[key] = len(specs)
            specs.append(cs)
            owners.append([])
        owners[by_key[key]].append(i)
    return specs, owners


def blocks_held_at_most(spec: CacheSpec, block_size: int, total_len: int, portion: int) -> int:
    """The most blocks a request of `total_len` tokens holds in a group at any time when it is
    fed in portions of at most `portion` tokens.  A full group keeps every position.  A window
    group keeps, while a portion runs, the window behind its first token and the portion itself:
    at most window - 1 + portion positions, which may start anywhere in a block."""
    whole = -(-max(0, int(total_len)) // block_size)
    if spec.kind != "window" or spec.window <= 0:
        return whole
    span = spec.window - 1 + max(1, int(portion))
    return min(whole, (span + block_size - 2) // block_size + 1)


class CacheManager:
    def __init__(self, cache_specs, state_specs, block_size: int, num_blocks, max_seqs: int):
        """cache_specs / state_specs: {owner: spec} for the runs of layers that keep a cache or a
        state (any hashable owner), or a sequence indexed by owner with None where there is none.
        num_blocks: blocks of every group's pool, or one number per group (in the order of
        `group_specs`)."""
        if not isinstance(cache_specs, Mapping):
            cache_specs = {i: c for i, c in enumerate(cache_specs) if c is not None}
        if not isinstance(state_specs, Mapping):
            state_specs = {i: c for i, c in enumerate(state_specs) if c is not None}
        if block_size <= 0:
            raise ValueError("block_size must be positive")
        self.block_size = int(block_size)
        self.max_seqs = int(max_seqs)
        specs, owners = group_specs(cache_specs)
        if isinstance(num_blocks, (list, tuple)):
            if len(num_blocks) != len(specs):
                raise ValueError(f"{len(num_blocks)} pool sizes for {len(specs)} cache groups")
            counts = [int(n) for n in num_blocks]
        else:
            counts = [int(num_blocks)] * len(specs)
        self.groups: List[CacheGroup] = []
        self.group_of_entry: Dict[Hashable, int] = {}
        self.index_in_group: Dict[Hashable, int] = {}
        for g, (cs, own, n) in enumerate(zip(specs, owners, counts)):
            self.groups.append(CacheGroup(cs, list(own), BlockPool(n)))
            for j, i in enumerate(own):
                self.group_of_entry[i] = g
                self.index_in_group[i] = j
        # the largest pool (what a model with one group calls "the" number of blocks)
        self.num_blocks = max(counts) if counts else (int(num_blocks) if not isinstance(num_blocks, (list, tuple)) else 0)
        # goes up whenever a request's block table is cut back: what a step buffer remembers of
        # the tables it holds is worthless then (the same length may come back with other blocks)
        self.table_epoch = 0
        self.state_specs: Dict[Hashable, StateSpec] = dict(state_specs)
        self.states: Dict[Hashable, torch.Tensor] = {}
        self._free_slots: List[int] = list(range(self.max_seqs - 1, -1, -1))
        self.requests: Dict[Hashable, RequestCache] = {}
        # what the last `reserve_step` changed, until the step commits:
        # (new requests, table lengths before, order of growth, saved state of the step's requests)
        self._reservation: Optional[tuple] = None

    # ------------------------------------------------------------------- tensors
    def elements_per_block(self) -> List[int]:
        """Cache elements one more block costs in each group (all its owners and tensors)."""
        return [g.elements_per_block(self.block_size) for g in self.groups]

    @property
    def group_blocks(self) -> List[int]:
        """Blocks of each group's pool."""
        return [g.pool.num_blocks for g in self.groups]

    def blocks_held_at_most(self, total_len: int, portion: int) -> List[int]:
        """Per group: the most blocks a request of `total_len` tokens holds at any time when fed
        in portions of at most `portion` tokens."""
        return [blocks_held_at_most(g.spec, self.block_size, total_len, portion) for g in self.groups]

    def allocate_tensors(self, dtype: torch.dtype, device) -> None:
        for g in self.groups:
            for t in g.spec.tensors:
                shape = (len(g.entries), g.pool.num_blocks, *t.page_shape(self.block_size))
                g.tensors[t.name] = torch.zeros(shape, dtype=dtype, device=device)
        for owner, ss in self.state_specs.items():
            self.states[owner] = torch.zeros((self.max_seqs, *ss.shape), dtype=ss.dtype, device=device)

    def layer_cache(self, owner: Hashable, cache_of: Optional[Hashable] = None) -> Optional[LayerCache]:
        """The view a run's part gets: its own cache, or (read-only) the cache that `cache_of` owns."""
        owner = owner if cache_of is None else cache_of
        if owner not in self.group_of_entry:
            return None
        g = self.group_of_entry[owner]
        grp = self.groups[g]
        j = self.index_in_group[owner]
        return LayerCache({name: t[j] for name, t in grp.tensors.items()}, group=g, write=cache_of is None)

    # ------------------------------------------------------------------ requests
    def has(self, req_id) -> bool:
        return req_id in self.requests

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def add_request(self, req_id) -> int:
        if req_id in self.requests:
            raise CacheError(f"request {req_id!r} is already live")
        if not self._free_slots:
            raise NoFreeSlot(f"all {self.max_seqs} request slots are taken")
        slot = self._free_slots.pop()
        self.requests[req_id] = RequestCache(slot, 0, [[] for _ in self.groups])
        for st in self.states.values():
            st[slot].zero_()
        return slot

    def num_tokens(self, req_id) -> int:
        return self.requests[req_id].num_tokens

    def slot(self, req_id) -> int:
        return self.requests[req_id].slot

    def block_table(self, req_id, group: int) -> List[int]:
        return self.requests[req_id].blocks[group]

    def _first_needed_block(self, g: CacheGroup, context_len: int) -> int:
        """Lowest logical block a query at position >= context_len can still read."""
        if g.spec.kind != "window" or g.spec.window <= 0:
            return 0
        first_pos = max(0, context_len - g.spec.window + 1)
        return first_pos // self.block_size

    def has_room(self, req_id, new_len: int) -> bool:
        """True if the request is live and holds blocks for positions < new_len in every group
        (the common case of a decoded token that does not start a new block)."""
        rc = self.requests.get(req_id)
        if rc is None:
            return False
        want = -(-new_len // self.block_size)
        for b in rc.blocks:
            if len(b) < want:
                return False
        return True

    def blocks_needed(self, req_id, new_len: int) -> List[int]:
        """New blocks per group to hold positions up to new_len - 1."""
        rc = self.requests.get(req_id)
        have = [len(b) for b in rc.blocks] if rc else [0] * len(self.groups)
        want = -(-new_len // self.block_size)
        return [max(0, want - h) for h in have]

    def can_grow(self, needs: Sequence[Sequence[int]]) -> bool:
        """needs: for several requests, their `blocks_needed`; true if all fit together."""
        for gi, g in enumerate(self.groups):
            if sum(n[gi] for n in needs) > g.pool.free_count:
                return False
        return True

    def grow(self, req_id, new_len: int) -> None:
        """Blocks for positions < new_len in every group, or none at all."""
        rc = self.requests[req_id]
        if new_len < rc.num_tokens:
            raise CacheError("a request's cache cannot shrink")
        need = self.blocks_needed(req_id, new_len)
        for g, n in zip(self.groups, need):
            if n > g.pool.free_count:
                raise OutOfBlocks(f"request {req_id!r} needs {n} more blocks, {g.pool.free_count} are free")
        for gi, (g, n) in enumerate(zip(self.groups, need)):
            rc.blocks[gi].extend(g.pool.allocate(n))

    def reserve_step(self, entries: Sequence[Tuple[Hashable, int]]) -> List[int]:
        """entries: (request, number of new tokens) of one step.  Admits the requests that are
        new (a state slot each) and takes the blocks every entry needs, or changes nothing and
        raises.  Returns each request's cached length before the step."""
        new = [rid for rid, _ in entries if rid not in self.requests]
        if len(new) > len(self._free_slots):
            raise NoFreeSlot(f"{len(new)} new requests, {len(self._free_slots)} request slots are free")
        before, needs, growing = [], [], []
        for rid, n in entries:
            rc = self.requests.get(rid)
            c = rc.num_tokens if rc is not None else 0
            before.append(c)
            if rc is not None and self.has_room(rid, c + n):
                continue                      # nothing to take for this one
            needs.append(self.blocks_needed(rid, c + n))
            growing.append((rid, c + n))
        if not self.can_grow(needs):
            raise OutOfBlocks("the step needs more cache blocks than are free: needs "
                              f"{[sum(n[g] for n in needs) for g in range(len(self.groups))]}, "
                              f"free {self.free_blocks()}")
        lengths = {rid: [len(b) for b in self.requests[rid].blocks] for rid, _ in growing if rid in self.requests}
        # the state of the requests that are live already, as it is before the step: a part may
        # have written a request's state by the time the step fails
        saved = None
        if self.states:
            slots = [self.requests[rid].slot for rid, _ in entries if rid in self.requests]
            if slots:
                idx = torch.tensor(slots, dtype=torch.long, device=next(iter(self.states.values())).device)
                saved = (idx, {owner: st.index_select(0, idx) for owner, st in self.states.items()})
        self._reservation = (list(new), lengths, [rid for rid, _ in growing], saved)
        for rid in new:
            self.add_request(rid)
        for rid, new_len in growing:
            self.grow(rid, new_len)
        return before

    def undo_reservation(self) -> None:
        """The step that the last `reserve_step` was for did not run: requests it admitted leave
        again and tables it lengthened are cut back, in the reverse of the order in which they were
        served, so that the cache and its free lists are as they were before; the per-request
        state of the step's requests is put back as it was.  Does nothing when no reservation is open."""
        if self._reservation is None:
            return
        new, lengths, order, saved = self._reservation
        self._reservation = None
        if saved is not None:
            idx, by_owner = saved
            for owner, values in by_owner.items():
                self.states[owner].index_copy_(0, idx, values)
        if order:
            self.table_epoch += 1
        for rid in reversed(order):
            rc = self.requests.get(rid)
            if rc is None:
                continue
            lens = lengths.get(rid, [0] * len(self.groups))
            for gi, (g, n) in enumerate(zip(self.groups, lens)):
                extra = [b for b in rc.blocks[gi][n:] if b != RELEASED]
                if extra:
                    g.pool.free(list(reversed(extra)))
                del rc.blocks[gi][n:]
        for rid in reversed(new):
            rc = self.requests.pop(rid, None)
            if rc is not None:
                self._free_slots.append(rc.slot)

    def forget_reservation(self) -> None:
        """The step ran and was committed."""
        self._reservation = None

    def commit(self, req_id, new_len: int) -> None:
        """The step has written positions < new_len.  Gives back what a window has passed."""
        rc = self.requests[req_id]
        if new_len < rc.num_tokens:
            raise CacheError("a request's cache cannot shrink")
        want = -(-new_len // self.block_size)
        for gi, g in enumerate(self.groups):
            if len(rc.blocks[gi]) < want:
                raise CacheError(f"request {req_id!r} commits {new_len} tokens without blocks for them")
        rc.num_tokens = new_len
        for gi, g in enumerate(self.groups):
            first = self._first_needed_block(g, new_len)
            gone = [b for b in rc.blocks[gi][:first] if b != RELEASED]
            if gone:
                g.pool.free(gone)
                for i in range(first):
                    rc.blocks[gi][i] = RELEASED

    def free_request(self, req_id) -> None:
        rc = self.requests.pop(req_id, None)
        if rc is None:
            raise CacheError(f"request {req_id!r} is not live")
        for gi, g in enumerate(self.groups):
            g.pool.free([b for b in rc.blocks[gi] if b != RELEASED])
        self._free_slots.append(rc.slot)

    # -------------------------------------------------------------------- checks
    def free_blocks(self) -> List[int]:
        return [g.pool.free_count for g in self.groups]

    def audit(self) -> None:
        """Every block is either free or held by exactly one request; every slot likewise."""
        for gi, g in enumerate(self.groups):
            held: Dict[int, Hashable] = {}
            for rid, rc in self.requests.items():
                for b in rc.blocks[gi]:
                    if b == RELEASED:
                        continue
                    if b in held:
                        raise CacheError(f"group {gi}: block {b} is held by {held[b]!r} and {rid!r}")
                    if g.pool.is_free(b):
                        raise CacheError(f"group {gi}: block {b} of {rid!r} is on the free list")
                    held[b] = rid
            if len(held) + g.pool.free_count != g.pool.num_blocks:
                raise CacheError(f"group {gi}: {g.pool.num_blocks - len(held) - g.pool.free_count} blocks are lost")
        slots = [rc.slot for rc in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise CacheError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.max_seqs:
            raise CacheError("a state slot is lost")
