"""Pins for the slot-indexing oracle: hand-computed traces read off the
reference's allocator and context-tree source."""
import pytest

from oracle.ref_context import (RefContext, RefPoolError, RefRecyclePool, ref_iteration_tables, ref_lca,
                                ref_shared_context_len)


def test_pool_fresh_ids_ascend_then_fifo_reuse():
    p = RefRecyclePool(pool_size=10)
    assert [p.allocate() for _ in range(4)] == [0, 1, 2, 3]
    p.free(2)
    p.free(0)
    # freed ids come back oldest-freed first (deque.popleft), before any fresh id
    assert p.allocate() == 2
    assert p.allocate() == 0
    assert p.allocate() == 4
    assert p.allocated_num == 5


def test_pool_never_issues_last_id_and_double_free_raises():
    p = RefRecyclePool(pool_size=3)
    assert p.allocate() == 0 and p.allocate() == 1
    with pytest.raises(RefPoolError):
        p.allocate()  # cur_max_id becomes 3 >= pool_size: id 2 is never handed out
    q = RefRecyclePool(pool_size=8)
    a = q.allocate()
    q.free(a)
    with pytest.raises(ValueError):
        q.free(a)


def test_context_tree_slots_and_lengths():
    pool = RefRecyclePool(100)
    root = RefContext(0, None, pool)
    root.allocate(3)  # slots 0,1,2
    a = RefContext(1, root, pool)
    a.allocate(2)  # 3,4
    b = RefContext(2, root, pool)
    b.allocate(1)  # 5
    a.allocate(1)  # 6
    assert root.context_slot_ids() == [0, 1, 2]
    assert a.context_slot_ids() == [0, 1, 2, 3, 4, 6]
    assert b.context_slot_ids() == [0, 1, 2, 5]
    assert (a.context_len(), b.context_len(), a.this_len(), a.depth) == (6, 4, 3, 1)
    with pytest.raises(AssertionError):
        root.destroy()  # children first
    b.destroy()
    assert root.children == [1]
    c = RefContext(3, a, pool)
    c.allocate(2)  # reuses 5 first, then fresh 7
    assert c.context_slot_ids() == [0, 1, 2, 3, 4, 6, 5, 7]


def test_lca_and_shared_len():
    pool = RefRecyclePool(1000)
    root = RefContext(0, None, pool); root.allocate(10)
    mid = RefContext(1, root, pool); mid.allocate(5)
    x = RefContext(2, mid, pool); x.allocate(2)
    y = RefContext(3, mid, pool); y.allocate(7)
    z = RefContext(4, root, pool); z.allocate(1)
    other = RefContext(5, None, pool); other.allocate(4)
    assert ref_lca(x, y) is mid and ref_lca(x, z) is root and ref_lca(x, mid) is mid
    assert ref_lca(x, other) is None and ref_lca(x, x) is x
    assert ref_shared_context_len([x, y]) == 15
    assert ref_shared_context_len([x, y, z]) == 10
    assert ref_shared_context_len([x, other, y]) == 0
    assert ref_shared_context_len([y]) == 22  # a single job shares its whole context


def test_iteration_tables_mixed_fill_and_generate():
    pool = RefRecyclePool(1000)
    root = RefContext(0, None, pool); root.allocate(4)          # 0..3
    f = RefContext(1, root, pool); f.allocate(3)               # 4,5,6  (a Fill of 3 tokens)
    g1 = RefContext(2, root, pool); g1.allocate(2)             # 7,8    (Generate: last slot is the new token)
    g2 = RefContext(3, root, pool); g2.allocate(1)             # 9
    jobs = [dict(kind="fill", context=f, num_tokens=3), dict(kind="generate", context=g1, num_tokens=1),
            dict(kind="generate", context=g2, num_tokens=1)]
    t = ref_iteration_tables(jobs)
    assert t["flash_context_len"] == 4 and t["flash_block_table"] == [0, 1, 2, 3]
    assert t["paged_block_tables"] == [[7, 8], [9]] and t["paged_context_lens"] == [2, 1]
    assert t["slot_mapping"] == [4, 5, 6, 8, 9]
    assert t["fill_q_lens"] == [3] and t["fill_kv_lens"] == [7] and t["fill_slots"] == [0, 1, 2, 3, 4, 5, 6]
