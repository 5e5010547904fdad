"""Host-side slot indexing of the product package against the list-based oracle model (bit-exact integers)."""
import random

import numpy as np
import pytest

from oracle.ref_context import RefContext, RefPoolError, RefRecyclePool, ref_iteration_tables, ref_shared_context_len
from parrotserve_amd.attn_func import (BuiltinConfig, HipGroupedPrefixAttn, HipSharedPrefixAttn,
                                       build_iteration_tables, get_attn_func, get_shared_context_len)
from parrotserve_amd.context import BlockContext, ParrotError, RecyclePool
from parrotserve_amd.primitive_job import Fill, Generate


def test_pool_random_trace_matches_oracle():
    rng = random.Random(0)
    a, b = RecyclePool(pool_size=64), RefRecyclePool(pool_size=64)
    live = []
    for _ in range(3000):
        if live and rng.random() < 0.45:
            i = live.pop(rng.randrange(len(live)))
            a.free(i)
            b.free(i)
        else:
            try:
                x = a.allocate()
            except ParrotError:
                with pytest.raises(RefPoolError):
                    b.allocate()
                a.allocated_num -= 1  # the reference counts the failed attempt too; keep both models aligned
                b.allocated_num -= 1
                continue
            assert x == b.allocate()
            live.append(x)
        assert a.get_allocated_num() == b.allocated_num
    with pytest.raises(ValueError):
        i = live.pop()
        a.free(i)
        a.free(i)


def test_pool_never_issues_last_id():
    p = RecyclePool(pool_size=3)
    assert [p.allocate(), p.allocate()] == [0, 1]
    with pytest.raises(ParrotError):
        p.allocate()


def _random_forest(seed, n_ctx=40):
    """The same random fork/allocate/destroy script applied to the product and the oracle models."""
    rng = random.Random(seed)
    pa, pb = RecyclePool(pool_size=100000), RefRecyclePool(pool_size=100000)
    A, B = {}, {}
    next_id = 0
    for _ in range(n_ctx * 3):
        r = rng.random()
        if r < 0.5 or not A:
            parent = rng.choice(list(A)) if A and rng.random() < 0.8 else None
            A[next_id] = BlockContext(next_id, A.get(parent), pa, 1)
            B[next_id] = RefContext(next_id, B.get(parent), pb)
            n = rng.randrange(0, 9)
            A[next_id].allocate(n)
            B[next_id].allocate(n)
            next_id += 1
        elif r < 0.85:
            c = rng.choice(list(A))
            n = rng.randrange(1, 5)
            A[c].allocate(n)
            B[c].allocate(n)
        else:
            leaves = [c for c in A if not A[c].sub_context_ids]
            c = rng.choice(leaves)
            A.pop(c).destruction()
            B.pop(c).destroy()
    return A, B


@pytest.mark.parametrize("seed", range(5))
def test_context_tree_matches_oracle(seed):
    A, B = _random_forest(seed)
    assert A.keys() == B.keys()
    for c in A:
        assert A[c].get_context_slot_ids() == B[c].context_slot_ids()
        assert A[c].get_context_block_ids() == B[c].context_slot_ids()
        assert A[c].get_context_len() == B[c].context_len()
        assert A[c].get_this_context_len() == B[c].this_len()
        assert A[c].depth == B[c].depth
    root = next(iter(A.values()))
    if root.sub_context_ids:
        with pytest.raises(AssertionError):
            root.destruction()


def _jobs_for(A, B, seed):
    rng = random.Random(seed)
    ids = [c for c in A if A[c].get_this_context_len() > 0]
    rng.shuffle(ids)
    ids = ids[: max(2, len(ids) // 2)]
    fills = ids[: len(ids) // 3]
    gens = ids[len(ids) // 3 :]
    ja, jb = [], []
    for c in fills:  # Fill jobs first (builtin_runner.py:76)
        n = rng.randrange(1, A[c].get_this_context_len() + 1)
        f = Fill(0, 0, c, -1, token_ids=list(range(n)))
        f.context = A[c]
        ja.append(f)
        jb.append(dict(kind="fill", context=B[c], num_tokens=n))
    for c in gens:
        g = Generate(0, 0, c, -1, sampling_config=None)
        g.context = A[c]
        ja.append(g)
        jb.append(dict(kind="generate", context=B[c], num_tokens=1))
    return ja, jb


@pytest.mark.parametrize("seed", range(6))
def test_iteration_tables_match_oracle(seed):
    A, B = _random_forest(seed + 10)
    ja, jb = _jobs_for(A, B, seed)
    t = build_iteration_tables(ja, "lca")
    ref = ref_iteration_tables(jb)
    assert get_shared_context_len(ja) == ref_shared_context_len([j["context"] for j in jb])
    for key in ("flash_context_len", "flash_block_table", "paged_block_tables", "paged_context_lens", "slot_mapping",
                "fill_q_lens", "fill_kv_lens", "fill_slots"):
        assert getattr(t, key) == ref[key], key


def test_shared_prefix_scenario_tables():
    """The reference's shared-prefix scenario: one parent Fill context, children fork and generate
    (tests/engine/builtin/test_shared_prefix.py:7-54 in the reference drives this shape)."""
    pool = RecyclePool(pool_size=10000)
    parent = BlockContext(0, None, pool, 1)
    parent.allocate(100)
    kids = []
    for i in range(8):
        c = BlockContext(1 + i, parent, pool, 1)
        c.allocate(3 + i)
        g = Generate(0, i, 1 + i, 0)
        g.context = c
        kids.append(g)
    t = build_iteration_tables(kids, "lca")
    assert t.flash_context_len == 100 and t.flash_block_table == list(range(100))
    assert t.paged_context_lens == [3 + i for i in range(8)]
    assert t.slot_mapping == [k.context.token_kv_slot_ids[-1] for k in kids]
    assert t.groups == [(list(range(100)), list(range(8)))]
    tp = build_iteration_tables(kids, "parent")
    assert tp.groups == t.groups and tp.paged_block_tables == t.paged_block_tables


def test_parent_grouping_two_prompt_groups_and_a_loner():
    pool = RecyclePool(pool_size=10000)
    p1 = BlockContext(0, None, pool, 1); p1.allocate(10)
    p2 = BlockContext(1, None, pool, 1); p2.allocate(20)
    jobs = []
    for i, par in enumerate([p1, p2, p1, None, p2]):
        c = BlockContext(10 + i, par, pool, 1)
        c.allocate(2)
        g = Generate(0, i, 10 + i, -1)
        g.context = c
        jobs.append(g)
    lca = build_iteration_tables(jobs, "lca")
    assert lca.flash_context_len == 0 and lca.groups == []  # the reference's single-LCA rule finds nothing shared
    assert [len(x) for x in lca.paged_block_tables] == [12, 22, 12, 2, 22]
    par = build_iteration_tables(jobs, "parent")
    assert par.groups == [(p1.token_kv_slot_ids, [0, 2]), (p2.token_kv_slot_ids, [1, 4])]
    assert par.paged_context_lens == [2, 2, 2, 2, 2]


def test_selector_and_config():
    for name in ("xformers_with_buffer", "xformers_fill_vllm_paged_attention_generate",
                 "xformers_fill_shared_prompts_generate"):
        assert get_attn_func(name) is HipSharedPrefixAttn
    assert get_attn_func("hip_shared_prefix") is HipGroupedPrefixAttn
    with pytest.raises(ValueError):
        get_attn_func("flash_attn_3")
    cfg = BuiltinConfig(num_kv_cache_blocks=16, attn_func="hip_shared_prefix", dtype="float16", device="cpu")
    assert cfg.attn_func is HipGroupedPrefixAttn and cfg.attn_func_name == "hip_shared_prefix"
    with pytest.raises(ValueError):
        BuiltinConfig(num_kv_cache_blocks=16, block_size=16)
    with pytest.raises(ValueError):
        BlockContext(0, None, RecyclePool(), block_size=16)


@pytest.mark.parametrize("seed", range(4))
def test_suffix_plan_covers_every_token_once_and_balances(seed):
    import numpy as np

    from parrotserve_amd.kernels import plan_suffix_items

    rng = random.Random(seed)
    lens = [rng.choice([0, 1, 3, 17, 64, 500, 2000]) for _ in range(rng.randrange(1, 60))]
    lanes = rng.choice([1, 7, 64, 384])
    items, lane_cu, req_cu = plan_suffix_items(lens, lanes)
    total = sum(lens)
    if total == 0:
        assert items.shape[0] == 0
        return
    # every request's tokens are covered exactly once, in order, by consecutive items
    for b, n in enumerate(lens):
        mine = items[req_cu[b] : req_cu[b + 1]]
        assert (mine[:, 0] == b).all()
        pos = 0
        for _, t0, cnt, _z in mine.tolist():
            assert t0 == pos and cnt > 0
            pos += cnt
        assert pos == n
    assert req_cu[-1] == items.shape[0] == lane_cu[-1]
    # pieces differ by at most one token
    per_lane = [int(items[lane_cu[j] : lane_cu[j + 1], 2].sum()) for j in range(len(lane_cu) - 1)]
    assert sum(per_lane) == total and max(per_lane) - min(per_lane) <= 1


def _decode_batch(pool, branches=5, prefix=40):
    parent = BlockContext(0, None, pool, 1)
    parent.allocate(prefix)
    jobs = []
    for b in range(branches):
        child = BlockContext(1 + b, parent, pool, 1)
        child.allocate(3 + b)
        job = Generate(0, b, child.context_id, parent.context_id, sampling_config=None)
        job.context = child
        jobs.append(job)
    return parent, jobs


def test_table_cache_host_side_hits_only_on_the_same_batch_one_token_later():
    """Host half of the incremental tables: a hit returns exactly the slots the contexts gained (what the
    from-scratch build reports as slot_mapping) and moves the cached lengths; every way a batch can differ
    from 'same jobs, one token later' is a miss that leaves the cache untouched."""
    from parrotserve_amd.table_cache import DecodeTableCache, _Cached

    pool = RecyclePool(pool_size=4096)
    parent, jobs = _decode_batch(pool)
    cache = DecodeTableCache()
    assert cache.advance_host(jobs) is None  # nothing cached yet

    def remember():
        ctxs = [j.context for j in jobs]
        lens = np.array([len(c.token_kv_block_ids) for c in ctxs], dtype=np.int64)
        cache.state = _Cached(ctxs, [c.parent_context for c in ctxs], [len(c.token_kv_block_ids) for c in ctxs],
                              [parent.get_context_len()] * len(jobs), None, lens, None, None, 0, 8, 128)

    remember()
    assert cache.advance_host(jobs) is None  # same lengths: not one token later
    for it in range(3):
        for j in jobs:
            j.context.allocate(1)
        got = cache.advance_host(jobs)
        assert got == build_iteration_tables(jobs).slot_mapping  # the from-scratch path, itself pinned to the oracle
        assert cache.state.lens_host.tolist() == [len(j.context.token_kv_block_ids) for j in jobs]
    before = (list(cache.state.own_lens), cache.state.lens_host.copy())

    def unchanged():
        return cache.state.own_lens == before[0] and np.array_equal(cache.state.lens_host, before[1])

    # two tokens at once
    for j in jobs:
        j.context.allocate(2)
    assert cache.advance_host(jobs) is None and unchanged()
    remember()
    before = (list(cache.state.own_lens), cache.state.lens_host.copy())
    for j in jobs:
        j.context.allocate(1)
    # a job left; the order changed
    assert cache.advance_host(jobs[:-1]) is None and unchanged()
    assert cache.advance_host(jobs[::-1]) is None and unchanged()
    # a Fill on one of the contexts
    f = Fill(0, 99, jobs[0].context_id, parent.context_id, token_ids=[1])
    f.context = jobs[0].context
    assert cache.advance_host([f] + jobs[1:]) is None and unchanged()
    # the parent grew (the shared prefix changed)
    parent.allocate(1)
    assert cache.advance_host(jobs) is None and unchanged()
    parent.token_kv_block_ids.pop()
    # a different context object with the right length
    other = BlockContext(50, parent, pool, 1)
    other.allocate(len(jobs[0].context.token_kv_block_ids))
    g = Generate(0, 98, 50, parent.context_id)
    g.context = other
    assert cache.advance_host([g] + jobs[1:]) is None and unchanged()
    # and the unchanged batch still qualifies
    assert cache.advance_host(jobs) == [j.context.token_kv_block_ids[-1] for j in jobs]


def test_forked_fill_tables_grouping_rules():
    """Forked Fills as a shared-prefix decode problem: groups by neighbouring common parent, per-token suffix lists
    = the own context up to the token; refused for lone chunks, short parents, long own contexts, parentless Fills."""
    from parrotserve_amd.attn_func import forked_fill_tables
    from parrotserve_amd.context import BlockContext, RecyclePool
    from parrotserve_amd.primitive_job import Fill, Generate

    pool = RecyclePool(pool_size=4096)

    def fork(parent, own_prev, n, cid):
        c = BlockContext(cid, parent, pool, 1)
        c.allocate(own_prev + n)
        j = Fill(0, cid, cid, parent.context_id if parent is not None else -1, token_ids=list(range(n)))
        j.context = c
        return j

    pa = BlockContext(100, None, pool, 1)
    pa.allocate(80)
    pb = BlockContext(101, None, pool, 1)
    pb.allocate(60)
    jobs = [fork(pa, 0, 3, 1), fork(pa, 2, 2, 2), fork(pb, 0, 1, 3), fork(pb, 0, 4, 4)]
    prefix, gcu, suffix = forked_fill_tables(jobs, 32, 16)
    assert prefix == [pa.get_context_slot_ids(), pb.get_context_slot_ids()] and gcu == [0, 5, 10]
    own1 = jobs[1].context.token_kv_block_ids
    assert suffix[0] == jobs[0].context.token_kv_block_ids[:1] and suffix[2] == jobs[0].context.token_kv_block_ids[:3]
    assert suffix[3] == own1[:3] and suffix[4] == own1[:4]  # two older own tokens are visible to the chunk's first token
    assert [len(x) for x in suffix[5:]] == [1, 1, 2, 3, 4]
    assert forked_fill_tables(jobs, 70, 16) is None            # parent b is shorter than 70
    assert forked_fill_tables(jobs, 32, 3) is None             # an own context of 4 tokens
    assert forked_fill_tables(jobs[:3], 32, 16) is None        # the last parent has a single chunk
    assert forked_fill_tables([jobs[0], jobs[2], jobs[1], jobs[3]], 32, 16) is None  # same parent, not neighbours
    assert forked_fill_tables([jobs[0]], 32, 16) is None
    # it has to pay: two 12-token chunks read 2 x 78 own pairs for the 80 parent rows they save
    assert forked_fill_tables([fork(pa, 0, 12, 20), fork(pa, 0, 12, 21)], 32, 16) is None
    assert forked_fill_tables([fork(None, 0, 5, 7), fork(None, 0, 5, 8)], 0, 16) is None  # no parent


def test_grouping_by_the_deepest_shared_ancestor():
    """Jobs under contexts of their own share the grandparent chain (the reference's two-level scenario); nested
    forks group at the lower level; a job nothing is shared with keeps its whole context as its own list."""
    pool = RecyclePool(pool_size=10000)

    def ctx(cid, parent, n):
        c = BlockContext(cid, parent, pool, 1)
        c.allocate(n)
        return c

    def gen(c):
        j = Generate(0, c.context_id, c.context_id, -1)
        j.context = c
        return j

    top = ctx(0, None, 20)
    mid = ctx(1, top, 10)
    fills = [ctx(2 + i, mid, 3 + i) for i in range(4)]
    jobs = [gen(ctx(10 + i, fills[i], 1)) for i in range(4)]
    t = build_iteration_tables(jobs, "parent")
    lca = build_iteration_tables(jobs, "lca")
    assert lca.flash_context_len == 30
    assert t.groups == [(lca.flash_block_table, [0, 1, 2, 3])]
    assert t.paged_block_tables == lca.paged_block_tables
    assert t.paged_block_tables[2] == fills[2].token_kv_slot_ids + jobs[2].context.token_kv_slot_ids
    # nested forks: two jobs under fills[0], one under fills[1] -> the pair groups at fills[0] (33 tokens); the
    # third job would anchor at mid, alone there (its cousins found a deeper anchor), so it shares nothing
    a, b = gen(ctx(20, fills[0], 2)), gen(ctx(21, fills[0], 1))
    c = gen(ctx(22, fills[1], 1))
    t = build_iteration_tables([a, c, b], "parent")
    assert [len(p) for p, _ in t.groups] == [33] and [m for _, m in t.groups] == [[0, 2]]
    assert t.paged_context_lens == [2, 30 + 4 + 1, 1]
    assert t.paged_block_tables[1] == c.context.get_context_slot_ids()
    # unrelated roots: nothing shared, no group, whole contexts
    x, y = gen(ctx(30, ctx(31, None, 7), 2)), gen(ctx(32, ctx(33, None, 5), 1))
    t = build_iteration_tables([x, y], "parent")
    assert t.groups == [] and t.paged_context_lens == [9, 6]


def test_model_cache_storage_takes_the_reference_call_form():
    """init_model_cache_storage(hf_config, builtin_config), as parrot/engine/builtin/mem.py:179-184 is called."""
    import types

    import torch

    from parrotserve_amd import mem
    from parrotserve_amd.attn_func import BuiltinConfig

    hf = types.SimpleNamespace(num_hidden_layers=2, num_attention_heads=4, hidden_size=64, max_position_embeddings=32,
                               rope_theta=10000.0)
    cfg = BuiltinConfig(num_kv_cache_blocks=10, attn_func="hip_shared_prefix", dtype="float32", device="cpu")
    store = mem.init_model_cache_storage(hf, cfg)
    assert store.k_cache.shape == (2, 10, 4, 16) and store.v_cache.dtype == torch.float32
    assert mem.get_k_cache(1).shape == (10, 4, 16) and mem.get_cos_sin_cache().shape == (32, 16)
    same = mem.init_model_cache_storage(2, 10, 4, 16, torch.float32, "cpu", max_seq_len=32)
    assert torch.equal(same.cos_sin_cache, store.cos_sin_cache)
    mem.Model_Cache = None
