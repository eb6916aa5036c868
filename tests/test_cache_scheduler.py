"""The cache manager and the scheduler's decisions, on the host only."""
import random

import pytest

from tiny_llm_amd.cache import BlockPool, CacheError, CacheManager, NoFreeSlot, OutOfBlocks, RELEASED
from tiny_llm_amd.engine.scheduler import Request, Scheduler
from tiny_llm_amd.parts.base import CacheSpec, StateSpec
from tiny_llm_amd.sampling import SamplingParams


# ------------------------------------------------------------------ block pool
def test_pool_reference_vectors():
    # (ref) tests/runtime/test_page_pool.cpp:5-23: 10 pages, allocate(10) = 0..9, allocate(12) throws,
    # freeing a free page throws
    pool = BlockPool(10)
    with pytest.raises(OutOfBlocks):
        pool.allocate(12)
    assert pool.free_count == 10            # a refused request takes nothing
    assert pool.allocate(10) == list(range(10))
    assert pool.free_count == 0
    pool.free([3, 7])
    with pytest.raises(CacheError):
        pool.free([3])
    with pytest.raises(CacheError):
        pool.free([5, 5])
    assert pool.allocate(2) == [7, 3]       # most recently freed first
    with pytest.raises(CacheError):
        pool.free([11])


def full(n=1):
    return [CacheSpec.keys_and_values(2, 16)] * n


def test_groups_by_need():
    kv = CacheSpec.keys_and_values
    specs = [kv(2, 16), kv(2, 16, "window", 8), None, kv(2, 16), kv(2, 16, "window", 8), kv(4, 16)]
    cm = CacheManager(specs, [None] * 6, block_size=4, num_blocks=10, max_seqs=2)
    assert [g.entries for g in cm.groups] == [[0, 3], [1, 4], [5]]
    assert cm.group_of_entry == {0: 0, 3: 0, 1: 1, 4: 1, 5: 2}
    assert cm.layer_cache(2) is None


def test_grow_commit_free_and_reuse():
    cm = CacheManager(full(2), [None, None], block_size=4, num_blocks=6, max_seqs=3)
    assert cm.reserve_step([("a", 5)]) == [0]
    assert cm.block_table("a", 0) == [0, 1]
    cm.commit("a", 5)
    assert cm.reserve_step([("a", 3), ("b", 9)]) == [5, 0]     # a: 5 -> 8 needs nothing new; b: 3 blocks
    assert cm.block_table("a", 0) == [0, 1] and cm.block_table("b", 0) == [2, 3, 4]
    cm.commit("a", 8)
    cm.commit("b", 9)
    with pytest.raises(OutOfBlocks):
        cm.reserve_step([("a", 1), ("c", 5)])                  # needs 1 + 2, one is free
    assert not cm.has("c") and cm.free_blocks() == [1] and cm.free_slots == 1   # nothing changed
    cm.free_request("b")
    assert cm.free_blocks() == [4]
    cm.reserve_step([("c", 13)])
    assert cm.block_table("c", 0) == [4, 3, 2, 5]              # b's pages are used again
    cm.audit()
    with pytest.raises(CacheError):
        cm.free_request("b")
    with pytest.raises(CacheError):
        cm.commit("a", 3)                                       # cannot shrink
    with pytest.raises(CacheError):
        cm.commit("c", 99)                                      # no blocks for that


def test_slots_run_out_and_come_back():
    cm = CacheManager(full(), [StateSpec((3,))], block_size=4, num_blocks=50, max_seqs=2)
    assert cm.add_request("a") == 0 and cm.add_request("b") == 1
    with pytest.raises(NoFreeSlot):
        cm.add_request("c")
    with pytest.raises(NoFreeSlot):
        cm.reserve_step([("c", 1)])
    cm.free_request("a")
    assert cm.add_request("c") == 0
    with pytest.raises(CacheError):
        cm.add_request("c")


def test_window_gives_blocks_back_as_it_passes():
    spec = [CacheSpec.keys_and_values(1, 8), CacheSpec.keys_and_values(1, 8, "window", 6)]
    cm = CacheManager(spec, [None, None], block_size=4, num_blocks=8, max_seqs=2)
    cm.reserve_step([("a", 10)])
    cm.commit("a", 10)        # next query at >= 10 reads keys >= 5: block 0 (0..3) of the window group is done
    assert cm.block_table("a", 0) == [0, 1, 2]
    assert cm.block_table("a", 1) == [RELEASED, 1, 2]
    assert cm.free_blocks() == [5, 6]
    for n in range(11, 22):
        cm.reserve_step([("a", 1)])
        cm.commit("a", n)
        cm.audit()
    # at 21 tokens the window group holds keys 16.. only: logical blocks 4 and 5
    assert [b != RELEASED for b in cm.block_table("a", 1)] == [False, False, False, False, True, True]
    assert cm.free_blocks() == [8 - 6, 8 - 2]
    cm.free_request("a")
    assert cm.free_blocks() == [8, 8]


@pytest.mark.parametrize("seed", range(6))
def test_no_page_lost_held_twice_or_freed_twice_under_random_orders(seed):
    rng = random.Random(seed)
    spec = [CacheSpec.keys_and_values(2, 16), CacheSpec.keys_and_values(2, 16, "window", 11), CacheSpec.keys_and_values(2, 16)]
    cm = CacheManager(spec, [None, StateSpec((2,)), None], block_size=4, num_blocks=40, max_seqs=5)
    live = {}
    n_new = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.55 and (live or True):
            batch = []
            ids = list(live)
            rng.shuffle(ids)
            for rid in ids[:rng.randint(0, 3)]:
                batch.append((rid, rng.choice([1, 1, 1, 2, 5, 9])))
            if rng.random() < 0.4:
                batch.append((f"n{n_new}", rng.randint(1, 30)))
            if not batch:
                continue
            free_before, slots_before = cm.free_blocks(), cm.free_slots
            try:
                before = cm.reserve_step(batch)
            except (OutOfBlocks, NoFreeSlot):
                assert cm.free_blocks() == free_before and cm.free_slots == slots_before
                continue
            for (rid, n), c in zip(batch, before):
                assert c == live.get(rid, 0)
                live[rid] = c + n
                cm.commit(rid, c + n)
                for g in range(2):
                    assert len(cm.block_table(rid, g)) == -(-live[rid] // 4)
            if batch[-1][0].startswith("n") and batch[-1][0] == f"n{n_new}":
                n_new += 1
        elif live:
            rid = rng.choice(list(live))
            cm.free_request(rid)
            del live[rid]
        cm.audit()
    for rid in list(live):
        cm.free_request(rid)
    assert cm.free_blocks() == [40, 40] and cm.free_slots == 5
    cm.audit()


# ------------------------------------------------------------------- scheduler
def make_sched(num_blocks=64, block_size=4, max_seqs=4, budget=16, max_len=256, eos=None):
    cm = CacheManager(full(), [None], block_size=block_size, num_blocks=num_blocks, max_seqs=max_seqs)
    return cm, Scheduler(cm, max_seqs, budget, max_len, eos)


def run_plan(cm, sched, plan, token=7):
    """What the engine does with a plan, without a model: reserve, commit, 'sample' `token`."""
    cm.reserve_step([(e.request.req_id, e.count) for e in plan.entries])
    for e in plan.entries:
        cm.commit(e.request.req_id, e.start + e.count)
    tok = token if not callable(token) else None
    sampled = {e.request.req_id: (token(e.request) if callable(token) else tok) for e in plan.entries if e.samples}
    done = sched.update(plan, sampled)
    cm.audit()
    return done


def req(rid, n_prompt, max_new=4, **kw):
    return Request(rid, list(range(1, n_prompt + 1)), SamplingParams.greedy(max_new, **kw))


def test_prompts_are_cut_under_the_token_budget():
    cm, s = make_sched(budget=16)
    s.add(req("a", 40))
    s.add(req("b", 5))
    p = s.schedule()
    assert [(e.request.req_id, e.start, e.count, e.samples) for e in p.entries] == [("a", 0, 16, False)]
    run_plan(cm, s, p)
    p = s.schedule()
    assert [(e.request.req_id, e.start, e.count) for e in p.entries] == [("a", 16, 16)]
    run_plan(cm, s, p)
    p = s.schedule()        # a's last 8 tokens, then b is admitted with what is left of the budget
    assert [(e.request.req_id, e.start, e.count, e.samples) for e in p.entries] == [("a", 32, 8, True), ("b", 0, 5, True)]
    assert p.num_tokens <= 16
    run_plan(cm, s, p)
    p = s.schedule()        # both decode: one token each, at position prompt_len + generated - 1
    assert [(e.request.req_id, e.start, e.count, e.samples) for e in p.entries] == [("a", 40, 1, True), ("b", 5, 1, True)]


def test_decoding_goes_before_prompt_portions():
    cm, s = make_sched(budget=8)
    s.add(req("a", 3))
    run_plan(cm, s, s.schedule())
    s.add(req("b", 20))
    p = s.schedule()
    assert [(e.request.req_id, e.count) for e in p.entries] == [("a", 1), ("b", 7)]
    run_plan(cm, s, p)
    p = s.schedule()
    assert [(e.request.req_id, e.count) for e in p.entries] == [("a", 1), ("b", 7)]


def test_finish_on_eos_length_and_model_len():
    cm, s = make_sched(eos=9, max_len=12)
    s.add(req("stop", 3, max_new=10))
    s.add(req("len", 3, max_new=2))
    s.add(req("ctx", 10, max_new=10))
    s.add(req("ign", 3, max_new=3, ignore_eos=True))
    run_plan(cm, s, s.schedule(), token=lambda r: 9 if r.req_id in ("stop", "ign") else 7)
    by = {r.req_id: r for r in s.finished}
    assert by["stop"].finish_reason == "stop" and by["stop"].output == [9]     # eos is part of the output
    assert not cm.has("stop")                                                   # freed at once
    run_plan(cm, s, s.schedule())
    by = {r.req_id: r for r in s.finished}
    assert by["len"].finish_reason == "length" and by["len"].output == [7, 7]
    assert by["ctx"].finish_reason == "length" and len(by["ctx"].prompt) + len(by["ctx"].output) == 12
    while s.has_work():     # "ign" was admitted a step later (the first step's budget was spent)
        run_plan(cm, s, s.schedule(), token=lambda r: 9)
    by = {r.req_id: r for r in s.finished}
    assert by["ign"].finish_reason == "length" and by["ign"].output == [7, 9, 9]
    assert {r.req_id for r in s.finished} == {"stop", "len", "ctx", "ign"}
    assert cm.free_blocks() == [64] and cm.free_slots == 4 and not s.has_work()


def test_admission_waits_for_slots_and_blocks():
    cm, s = make_sched(num_blocks=6, block_size=4, max_seqs=2, budget=64)
    for rid in "abc":
        s.add(req(rid, 8, max_new=3))
    p = s.schedule()
    assert [e.request.req_id for e in p.entries] == ["a", "b"]      # two slots
    run_plan(cm, s, p)
    assert [r.req_id for r in s.waiting] == ["c"]
    admitted_c_with_finished = None
    while s.has_work():
        p = s.schedule()
        if admitted_c_with_finished is None and any(e.request.req_id == "c" for e in p.entries):
            admitted_c_with_finished = sorted(r.req_id for r in s.finished)
        assert len(s.running) <= 2
        run_plan(cm, s, p)
    assert admitted_c_with_finished == ["a", "b"]                   # c got a slot only when one was given back
    assert sorted(r.req_id for r in s.finished) == ["a", "b", "c"]
    assert all(len(r.output) == 3 for r in s.finished)


def test_when_pages_run_out_the_newest_request_is_preempted_and_recomputed():
    cm, s = make_sched(num_blocks=5, block_size=4, max_seqs=3, budget=64)
    s.add(req("old", 8, max_new=12))
    s.add(req("new", 8, max_new=12))
    run_plan(cm, s, s.schedule())                 # 2 + 2 blocks, both sampled their first token
    p = s.schedule()                              # both need a third block, one is free
    assert [e.request.req_id for e in p.entries] == ["old"]
    assert [r.req_id for r in p.preempted] == ["new"]
    assert not cm.has("new") and s.waiting[0].req_id == "new" and s.waiting[0].num_computed == 0
    assert s.waiting[0].output == [7]             # what it generated is kept and recomputed later
    run_plan(cm, s, p)
    steps = 0
    while s.has_work():
        plan = s.schedule()
        assert plan.entries or plan.finished
        run_plan(cm, s, plan)
        steps += 1
        assert steps < 200
    by = {r.req_id: r for r in s.finished}
    assert by["old"].finish_reason == "length" and len(by["old"].output) == 12
    assert by["new"].finish_reason == "length" and len(by["new"].output) == 12 and by["new"].preemptions >= 1
    assert cm.free_blocks() == [5] and cm.free_slots == 3


def test_a_request_that_cannot_fit_alone_ends_with_capacity():
    cm, s = make_sched(num_blocks=3, block_size=4, max_seqs=2, budget=64)
    with pytest.raises(ValueError):
        s.add(req("huge", 13))                    # the prompt alone needs 4 blocks of 3
    s.add(req("grows", 10, max_new=50))
    steps = 0
    while s.has_work():
        run_plan(cm, s, s.schedule())
        steps += 1
        assert steps < 100
    r = s.finished[0]
    assert r.finish_reason == "capacity" and len(r.prompt) + len(r.output) == 13   # 12 cached + the one in hand
    assert cm.free_blocks() == [3]


@pytest.mark.parametrize("seed", range(5))
def test_scheduler_invariants_under_random_load(seed):
    rng = random.Random(seed)
    cm, s = make_sched(num_blocks=30, block_size=4, max_seqs=4, budget=24, max_len=80, eos=3)
    added = 0
    steps = 0
    while added < 25 or s.has_work():
        if added < 25 and rng.random() < 0.5:
            s.add(req(f"r{added}", rng.randint(1, 40), max_new=rng.randint(1, 30)))
            added += 1
        if not s.has_work():
            continue
        plan = s.schedule()
        assert plan.num_tokens <= 24
        assert len(s.running) <= 4
        ids = [e.request.req_id for e in plan.entries]
        assert len(ids) == len(set(ids))
        for e in plan.entries:
            assert e.start == e.request.num_computed and e.count >= 1
            assert e.samples == (e.start + e.count == e.request.num_tokens)
        run_plan(cm, s, plan, token=lambda r: rng.choice([3, 5, 6, 8, 11, 12]))
        steps += 1
        assert steps < 3000
    assert len(s.finished) == 25 and cm.free_blocks() == [30] and cm.free_slots == 4
    for r in s.finished:
        assert r.finish_reason in ("stop", "length", "capacity")
        if r.finish_reason == "stop":
            assert r.output[-1] == 3


# ------------------------------------------------------------- step metadata
def _rows(specs, bs):
    """specs: (context_len, new tokens, wanted places) per request, with made-up block tables."""
    from tiny_llm_amd.engine.step import _Row
    rows, nxt = [], 3
    for i, (c, toks, want) in enumerate(specs):
        nb = -(-(c + len(toks)) // bs)
        rows.append(_Row(f"r{i}", toks, want, c, slot=10 + i, tables=[list(range(nxt, nxt + nb))]))
        nxt += nb + 1
    return rows


def test_step_metadata_layout_and_padding():
    """One routine lays out eager steps (exact sizes) and captured steps (capacities): the padded
    layout holds the exact one in its first entries, and what is padding can do no harm."""
    import numpy as np
    from tiny_llm_amd.engine.step import Layout, SampleSpec, fill_metadata, tile_lists
    bs = 4
    rows = _rows([(5, [7, 8, 9], [2]), (0, [1, 2, 3, 4, 5, 6], []), (9, [4], [0])], bs)
    exact = Layout(10, 3, 2, 1, 3, {2: 6, 16: 3}, True)
    a = np.full(exact.total, -7, dtype=np.int32)
    samples = [SampleSpec(0.8, 5, 0.9, 123456789012345, 8), SampleSpec()]
    fill_metadata(a, exact, rows, bs, samples)
    assert exact.sec(a, "tokens").tolist() == [7, 8, 9, 1, 2, 3, 4, 5, 6, 4]
    assert exact.sec(a, "positions").tolist() == [5, 6, 7, 0, 1, 2, 3, 4, 5, 9]
    assert exact.sec(a, "req_of_token").tolist() == [0, 0, 0, 1, 1, 1, 1, 1, 1, 2]
    assert exact.sec(a, "cu_seqlens").tolist() == [0, 3, 9, 10] and exact.sec(a, "seq_lens").tolist() == [8, 6, 10]
    assert exact.sec(a, "state_slots").tolist() == [10, 11, 12] and exact.sec(a, "logit_rows").tolist() == [2, 9]
    # slots: request 0 holds blocks 3, 4 (positions 5..7 -> block 4), request 1 blocks 6, 7, request 2 blocks 9, 10, 11
    assert exact.sec(a, "slots0").tolist() == [17, 18, 19, 24, 25, 26, 27, 28, 29, 11 * 4 + 1]
    assert exact.sec(a, "tables0").reshape(3, 3).tolist() == [[3, 4, -7], [6, 7, -7], [9, 10, 11]]
    t2 = exact.sec(a, "tiles2").reshape(3, 6)
    assert t2.tolist() == [[0, 0, 1, 1, 1, 2], [0, 2, 3, 5, 7, 9], [2, 1, 2, 2, 2, 1]]
    assert exact.sec(a, "tiles16").reshape(3, 3).tolist() == [[0, 1, 2], [0, 3, 9], [3, 6, 1]]
    assert exact.sec(a, "temperature").view(np.float32).tolist() == [np.float32(0.8), 0.0]
    assert exact.sec(a, "top_k").tolist() == [5, 0] and exact.sec(a, "counters").tolist() == [8, 0]
    assert exact.sec(a, "seeds").view(np.int64).tolist() == [123456789012345, 0]

    padded = Layout(16, 4, 4, 1, 5, {2: 12, 16: 5}, True)
    b = np.full(padded.total, -7, dtype=np.int32)
    fill_metadata(b, padded, rows, bs, samples)
    for name in ("tokens", "positions", "req_of_token", "slots0"):
        n = exact.off[name][1]
        assert padded.sec(b, name)[:n].tolist() == exact.sec(a, name).tolist()
    assert padded.sec(b, "tokens")[10:].tolist() == [0] * 6 and padded.sec(b, "positions")[10:].tolist() == [0] * 6
    assert padded.sec(b, "slots0")[10:].tolist() == [-1] * 6            # a padding token stores nothing
    assert padded.sec(b, "cu_seqlens").tolist() == [0, 3, 9, 10, 10]    # the padding request has no tokens
    assert padded.sec(b, "logit_rows").tolist() == [2, 9, 0, 0]
    assert padded.sec(b, "tables0").reshape(4, 5)[:3, :3].tolist() == [[3, 4, -7], [6, 7, -7], [9, 10, 11]]
    p2 = padded.sec(b, "tiles2").reshape(3, 12)
    assert p2[:, :6].tolist() == t2.tolist() and p2[2, 6:].tolist() == [0] * 6     # padding tiles hold no token
    assert padded.sec(b, "top_p").view(np.float32).tolist() == [np.float32(0.9), 1.0, 1.0, 1.0]
    # too many tiles for the layout is an error, not an overrun
    small = Layout(10, 3, 2, 1, 3, {2: 5}, False)
    with pytest.raises(ValueError):
        fill_metadata(np.zeros(small.total, dtype=np.int32), small, rows, bs)
    assert tile_lists([3, 0, 5], 2) == ([0, 0, 2, 2, 2], [0, 2, 3, 5, 7], [2, 1, 2, 2, 1])


def test_static_block_table_rows_are_rewritten_when_they_change():
    import numpy as np
    from tiny_llm_amd.engine.step import Layout, SeenTables, fill_metadata
    bs = 4
    lay = Layout(2, 2, 2, 1, 4, {}, False)
    buf = np.zeros(lay.total, dtype=np.int32)
    seen = SeenTables(1, 2)
    rows = _rows([(5, [1], [0]), (2, [1], [0])], bs)
    fill_metadata(buf, lay, rows, bs, None, seen)
    assert lay.sec(buf, "tables0").reshape(2, 4).tolist() == [[3, 4, 0, 0], [6, 0, 0, 0]]
    assert lay.sec(buf, "slots0").tolist() == [4 * 4 + 1, 6 * 4 + 2]
    rows[0].tables[0].append(20)                      # the same request grew by a block
    rows[0].context_len = 8
    rows[1] = _rows([(0, [5], [0])], bs)[0]           # another request took row 1
    fill_metadata(buf, lay, rows, bs, None, seen)
    assert lay.sec(buf, "tables0").reshape(2, 4).tolist() == [[3, 4, 20, 0], [3, 0, 0, 0]]
    assert lay.sec(buf, "slots0").tolist() == [20 * 4, 3 * 4]


def test_static_rows_after_a_step_that_did_not_run():
    """A captured step fails and is undone; another request takes the block that was given back;
    the first request grows again to the SAME length with ANOTHER block.  The static buffer must
    then hold the real table: the request would otherwise write its new key to one page and read
    another request's page."""
    import numpy as np
    from tiny_llm_amd.engine.step import Layout, SeenTables, _Row, fill_metadata
    bs = 4
    cm = CacheManager(full(1), [None], block_size=bs, num_blocks=8, max_seqs=3)
    cm.reserve_step([("a", 8), ("b", 8)])
    cm.commit("a", 8), cm.commit("b", 8)
    cm.forget_reservation()
    lay = Layout(2, 2, 2, 1, 4, {}, False)
    buf = np.zeros(lay.total, dtype=np.int32)
    seen = SeenTables(1, 2, cm.table_epoch)

    def rows_of(ids):
        before = cm.reserve_step([(r, 1) for r in ids])
        return [_Row(r, [1], [0], c, cm.slot(r), [cm.block_table(r, 0)]) for r, c in zip(ids, before)]

    rows = rows_of(["a", "b"])                                  # a: [0, 1, 4], b: [2, 3, 5]
    fill_metadata(buf, lay, rows, bs, None, seen, cm.table_epoch)
    assert lay.sec(buf, "tables0").reshape(2, 4).tolist() == [[0, 1, 4, 0], [2, 3, 5, 0]]
    cm.undo_reservation()                                       # the step did not run
    assert cm.block_table("a", 0) == [0, 1] and cm.free_blocks() == [4]
    cm.reserve_step([("c", 3)])                                 # somebody else takes block 4
    cm.commit("c", 3)
    cm.forget_reservation()
    assert cm.block_table("c", 0) == [4]
    rows = rows_of(["a", "b"])                                  # the same lengths, other blocks
    assert cm.block_table("a", 0) == [0, 1, 5] and cm.block_table("b", 0) == [2, 3, 6]
    fill_metadata(buf, lay, rows, bs, None, seen, cm.table_epoch)
    tables = lay.sec(buf, "tables0").reshape(2, 4)
    assert tables[0, :3].tolist() == cm.block_table("a", 0) and tables[1, :3].tolist() == cm.block_table("b", 0)
    assert lay.sec(buf, "slots0").tolist() == [5 * bs, 6 * bs]  # and the new keys go where the table says
    # without an undo in between nothing is forgotten: rows of unchanged tables are not rewritten
    for r in ("a", "b"):
        cm.commit(r, 9)
    cm.forget_reservation()
    tables[:] = -5
    rows = rows_of(["a", "b"])
    fill_metadata(buf, lay, rows, bs, None, seen, cm.table_epoch)
    assert (lay.sec(buf, "tables0") == -5).all()


def test_a_step_that_did_not_run_leaves_the_state_slots_as_they_were():
    import torch
    cm = CacheManager(full(1), [StateSpec((3,))], block_size=4, num_blocks=8, max_seqs=3)
    cm.allocate_tensors(torch.float32, "cpu")
    cm.reserve_step([("a", 2), ("b", 2)])
    st = cm.states[0]
    st[cm.slot("a")] = torch.tensor([1.0, 2.0, 3.0])
    st[cm.slot("b")] = torch.tensor([4.0, 5.0, 6.0])
    cm.commit("a", 2), cm.commit("b", 2)
    cm.forget_reservation()
    cm.reserve_step([("b", 1), ("c", 4)])
    st[cm.slot("b")] += 10.0                # the failing step's parts had already written
    st[cm.slot("c")] += 7.0
    cm.undo_reservation()
    assert st[cm.slot("a")].tolist() == [1.0, 2.0, 3.0] and st[cm.slot("b")].tolist() == [4.0, 5.0, 6.0]
    assert not cm.has("c")
    cm.reserve_step([("c", 4)])             # a request admitted later starts from zero as ever
    assert st[cm.slot("c")].tolist() == [0.0, 0.0, 0.0]
    cm.audit()


def test_every_group_has_a_pool_of_its_own_size():
    """A window group holds, per request, its window and one portion at most: its pool may be much
    smaller than the full group's, and a long request is still admitted and served."""
    from tiny_llm_amd.cache.manager import blocks_held_at_most
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import plan_cache_blocks
    bs, window, budget, max_len = 4, 6, 8, 200
    kv = CacheSpec.keys_and_values
    specs = [kv(1, 8), kv(1, 8, "window", window)]
    assert blocks_held_at_most(specs[0], bs, 100, budget) == 25
    assert blocks_held_at_most(specs[1], bs, 100, budget) == 4      # 5 + 8 = 13 positions, starting anywhere
    assert blocks_held_at_most(specs[1], bs, 9, budget) == 3        # a short request holds all it has
    probe = CacheManager(specs, [None, None], bs, 1, 1)
    held = probe.blocks_held_at_most(max_len, budget)
    e = EngineConfig(kv_block_size=bs, max_num_seqs=2, max_num_batched_tokens=budget)
    assert plan_cache_blocks(e, max_len, [100, 100], None, held) == [2 * 50, 2 * 4]
    assert plan_cache_blocks(e, max_len, [100, 100], 5500, held) == [45, 3]     # one factor for all groups
    e2 = EngineConfig(kv_block_size=bs, max_num_seqs=2, max_num_batched_tokens=budget, num_kv_blocks=30)
    assert plan_cache_blocks(e2, max_len, [100, 100], None, held) == [30, 8]    # given: for a full group
    cm = CacheManager(specs, [None, None], bs, [30, 4], 2)
    assert cm.group_blocks == [30, 4] and cm.num_blocks == 30
    cm.allocate_tensors(__import__("torch").float32, "cpu")
    assert cm.groups[0].tensors["k"].shape[1] == 30 and cm.groups[1].tensors["k"].shape[1] == 4
    s = Scheduler(cm, 2, budget, max_len, None)
    s.add(req("long", 90, max_new=6))      # 23 blocks in the full group, 4 at most in the window group
    steps = 0
    while s.has_work():
        p = s.schedule()
        assert p.entries and not p.preempted and not p.finished
        run_plan(cm, s, p)
        assert cm.groups[1].pool.used_count <= 4
        steps += 1
        assert steps < 100
    assert s.finished[0].finish_reason == "length" and len(s.finished[0].output) == 6
    assert cm.free_blocks() == [30, 4]
    # what can never be held is refused when it is added, per group
    cm2 = CacheManager(specs, [None, None], bs, [30, 3], 2)
    s2 = Scheduler(cm2, 2, budget, max_len, None)
    with pytest.raises(ValueError):
        s2.add(req("too long for the window pool", 90))
    s2.add(req("short", 9))                # holds 3 blocks in either group


def test_reservation_of_a_step_that_did_not_run_is_undone():
    cm = CacheManager(full(1), [None], block_size=4, num_blocks=8, max_seqs=2)
    cm.reserve_step([("a", 6)])
    cm.commit("a", 6)
    cm.forget_reservation()
    before = (cm.free_blocks(), cm.free_slots, list(cm.block_table("a", 0)))
    cm.reserve_step([("a", 5), ("b", 9)])              # a: one more block; b: admitted with three
    assert cm.free_blocks() == [2] and cm.has("b")
    cm.undo_reservation()
    assert (cm.free_blocks(), cm.free_slots, list(cm.block_table("a", 0))) == before and not cm.has("b")
    cm.audit()
    assert cm.reserve_step([("a", 5), ("b", 9)]) == [6, 0]
    assert cm.block_table("a", 0) == [0, 1, 2] and cm.block_table("b", 0) == [3, 4, 5]    # the same pages again
    cm.undo_reservation()
    cm.undo_reservation()                               # nothing open: nothing happens
    cm.audit()


def test_a_run_of_steps_is_applied_as_the_steps_one_by_one_would_be():
    """`update_burst` against `update` called once per step, on random tokens: ends by an
    end-of-sequence token, by `max_new_tokens` and by the model's length, anywhere in the run."""
    import copy
    from tiny_llm_amd.engine.scheduler import Scheduled, StepPlan, RUNNING
    rng = random.Random(3)
    for trial in range(60):
        steps = rng.randint(2, 12)
        n = rng.randint(1, 5)
        by_step = [[rng.randint(0, 6) for _ in range(n)] for _ in range(steps)]
        results = []
        for burst in (False, True):
            cm, s = make_sched(num_blocks=200, block_size=4, max_seqs=8, budget=64, max_len=30, eos=(5, 6))
            r2 = random.Random(trial)
            for i in range(n):
                s.add(req(f"r{i}", r2.randint(1, 12), max_new=r2.randint(2, 14), ignore_eos=r2.random() < 0.3))
            run_plan(cm, s, s.schedule(), token=1)               # prompts; one token each (no eos)
            p = s.schedule()
            cm.reserve_step([(e.request.req_id, steps) for e in p.entries])
            for e in p.entries:
                cm.commit(e.request.req_id, e.start + steps)
            if burst:
                done = s.update_burst(p, by_step)
            else:
                done, live = [], list(range(len(p.entries)))
                for k, toks in enumerate(by_step):
                    sp = StepPlan([Scheduled(p.entries[i].request, p.entries[i].start + k, 1, True) for i in live], [], [])
                    done += s.update(sp, {p.entries[i].request.req_id: toks[i] for i in live})
                    live = [i for i in live if p.entries[i].request.status == RUNNING]
            results.append(([r.req_id for r in done],
                            [(e.request.output, e.request.num_computed, e.request.status, e.request.finish_reason)
                             for e in p.entries]))
        assert results[0] == results[1], trial


def test_runs_of_decode_steps_end_where_a_decision_is_due():
    """How long a run of chained decode steps may be: up to the first request's end by length, never
    beside a prompt portion or while somebody waits, never beyond the free cache blocks."""
    cm, s = make_sched(num_blocks=12, block_size=4, max_seqs=2, budget=64, max_len=40, eos=9)
    s.add(req("a", 6, max_new=20))
    s.add(req("b", 3, max_new=7))
    run_plan(cm, s, s.schedule())                          # prompts; one token each
    p = s.schedule()
    assert all(e.count == 1 and e.samples for e in p.entries)
    assert s.burst_length(p, 16) == 6                      # b has 6 of its 7 tokens to go
    assert s.burst_length(p, 4) == 4 and s.burst_length(p, 1) == 1
    s.add(req("c", 5))
    assert s.burst_length(p, 16) == 1                      # somebody waits: decide step by step
    s.waiting.clear()
    # the run's blocks are taken at once; its tokens are applied step by step: b ends by eos at step 3
    k = 6
    cm.reserve_step([(e.request.req_id, k) for e in p.entries])
    for e in p.entries:
        cm.commit(e.request.req_id, e.start + k)
    by_step = [[7, 7], [7, 7], [7, 9], [7, 1], [7, 2], [7, 3]]
    done = s.update_burst(p, by_step)
    a, b = p.entries[0].request, p.entries[1].request
    assert [r.req_id for r in done] == ["b"] and b.finish_reason == "stop" and b.output == [7, 7, 7, 9]
    assert a.output == [7] * 7 and a.num_computed == 6 + 6 and a.status == "running"
    assert not cm.has("b") and cm.num_tokens("a") == 12
    cm.audit()
    # not more steps than blocks: a holds 3 blocks (12 tokens), 9 are free
    p = s.schedule()
    assert s.burst_length(p, 32) == 13                     # 13 more tokens end its 20
    cm2, s2 = make_sched(num_blocks=4, block_size=4, max_seqs=2, budget=64, max_len=400)
    s2.add(req("x", 6, max_new=200))
    run_plan(cm2, s2, s2.schedule())
    p2 = s2.schedule()
    assert s2.burst_length(p2, 10) == 10                   # 6 + 10 = 16 tokens: the pool's 4 blocks
    assert s2.burst_length(p2, 11) == 10                   # one more does not fit: the run ends where the blocks end
    # a running request that the plan leaves out (the budget is below the number of decoding
    # requests) would sit idle for a whole run: step by step then
    cm3, s3 = make_sched(num_blocks=40, block_size=4, max_seqs=3, budget=8, max_len=100)
    for rid in "abc":
        s3.add(req(rid, 2, max_new=30))
    run_plan(cm3, s3, s3.schedule())
    assert s3.burst_length(s3.schedule(), 8) == 8
    s3.budget = 2
    p3 = s3.schedule()
    assert [e.request.req_id for e in p3.entries] == ["a", "b"] and s3.burst_length(p3, 8) == 1


def test_runs_of_decode_steps_in_a_window_group():
    """The blocks of a whole run are taken up front in every group; what the window has passed
    goes back when the run is committed."""
    bs, window = 4, 6
    specs = [CacheSpec.keys_and_values(1, 8), CacheSpec.keys_and_values(1, 8, "window", window)]
    cm = CacheManager(specs, [None, None], bs, [20, 6], 2)
    s = Scheduler(cm, 2, 16, 60, None)
    s.add(req("a", 10, max_new=30))
    run_plan(cm, s, s.schedule())
    p = s.schedule()
    # the window pool has 6 blocks: a holds 2 (positions 5.. of its 10), 4 are free: 16 more positions
    k = s.burst_length(p, 32)
    assert k == 18                                          # 10 + 18 = 28 positions: 7 logical blocks, 3 were given
    cm.reserve_step([(e.request.req_id, k) for e in p.entries])
    assert cm.free_blocks() == [20 - 7, 0]
    for e in p.entries:
        cm.commit(e.request.req_id, e.start + k)
    cm.forget_reservation()
    cm.audit()
    done = s.update_burst(p, [[7]] * k)
    assert not done and cm.num_tokens("a") == 28
    # after the commit only the window's blocks are held: positions 23.. -> logical blocks 5 and 6
    assert [b != RELEASED for b in cm.block_table("a", 1)] == [False] * 5 + [True] * 2
    assert cm.free_blocks() == [20 - 7, 6 - 2]
