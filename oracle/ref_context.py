"""CPU oracle for slot indexing: a list-based model of the reference's slot
allocator, context tree and per-iteration index tables.

TEST INFRASTRUCTURE ONLY -- the product package never imports this module.

Restates, for ``block_size == 1`` (token-granular slots):
  * ``RecyclePool``  (parrot/utils/recycle_pool.py:11-65)
  * ``BlockContext`` (parrot/engine/context/block_context.py:13-135) and the
    tree bookkeeping of ``LowLevelContext`` (low_level_context.py:15-52)
  * ``xFormersFill_SharedPromptsGenerate._lca / get_shared_context_len /
    init_iteration_state`` (parrot/engine/builtin/attn_func.py:412-599)

Pinned by hand-computed allocation traces in tests/test_oracle_context.py
(fresh ids ascend, freed ids come back oldest-first, the last id of the pool
is never issued, double free raises) -- integer facts read off the reference
source, not recomputed with this model.
"""
from __future__ import annotations

from collections import deque
from typing import Dict, List, Optional, Sequence


class RefPoolError(RuntimeError):
    pass


class RefRecyclePool:
    """recycle_pool.py:30-55: a fresh ascending id unless a freed id exists, in
    which case the oldest freed id; ``cur_max_id >= pool_size`` raises *after*
    the increment, so only ids ``0 .. pool_size-2`` are ever issued."""

    def __init__(self, pool_size: Optional[int] = None):
        self.pool_size = pool_size
        self.cur_max_id = 0
        self.free_ids: deque = deque()
        self.allocated_num = 0

    def allocate(self) -> int:
        self.allocated_num += 1
        if len(self.free_ids) == 0:
            self.cur_max_id += 1
            if self.pool_size is not None and self.cur_max_id >= self.pool_size:
                raise RefPoolError("no free ids")
            return self.cur_max_id - 1
        return self.free_ids.popleft()

    def free(self, i: int) -> None:
        self.allocated_num -= 1
        if i in self.free_ids:
            raise ValueError("The id is already free.")
        self.free_ids.append(i)


class RefContext:
    """block_context.py with block_size 1: one pool id per token; a child
    indexes its ancestors' slots by recursion (:110-124); destruction frees own
    slots and requires children gone first (low_level_context.py:32-40)."""

    def __init__(self, context_id: int, parent: Optional["RefContext"], pool: RefRecyclePool):
        self.context_id = context_id
        self.parent = parent
        self.pool = pool
        self.children: List[int] = []
        self.depth = 0
        if parent is not None:
            parent.children.append(context_id)
            self.depth = parent.depth + 1
        self.slots: List[int] = []

    def allocate(self, n: int) -> None:
        for _ in range(n):
            self.slots.append(self.pool.allocate())

    def this_len(self) -> int:
        return len(self.slots)

    def context_len(self) -> int:
        return (self.parent.context_len() if self.parent else 0) + len(self.slots)

    def context_slot_ids(self) -> List[int]:
        return (self.parent.context_slot_ids() if self.parent else []) + self.slots

    def destroy(self) -> None:
        if self.parent is not None:
            self.parent.children.remove(self.context_id)
        assert len(self.children) == 0
        for s in self.slots:
            self.pool.free(s)


def ref_lca(a: Optional[RefContext], b: Optional[RefContext]) -> Optional[RefContext]:
    """attn_func.py:412-439."""
    if a is b:
        return a
    if a is None or b is None:
        return None
    while a is not None:
        if a is b:
            return a
        if a.depth > b.depth:
            a = a.parent
        elif a.depth < b.depth:
            b = b.parent
        else:
            a = a.parent
            b = b.parent
    return None


def ref_shared_context_len(contexts: Sequence[RefContext]) -> int:
    """attn_func.py:441-459: whole context for one job; LCA length else, 0 when
    no common ancestor exists."""
    assert len(contexts) > 0
    if len(contexts) == 1:
        return contexts[0].context_len()
    lca = ref_lca(contexts[0], contexts[1])
    for c in contexts[2:]:
        if lca is None:
            break
        lca = ref_lca(lca, c)
    return lca.context_len() if lca is not None else 0


def ref_iteration_tables(jobs: Sequence[dict]) -> Dict[str, object]:
    """Index tables of one iteration, attn_func.py:462-599 at block_size 1.

    ``jobs``: dicts ``{"kind": "fill"|"generate", "context": RefContext,
    "num_tokens": int}`` (Generate has num_tokens 1), Fill jobs first
    (builtin_runner.py:76).  Returns python lists:
      flash_context_len, flash_block_table (= first P slots of job 0),
      paged_block_tables (per Generate: slots[P:], ragged), paged_context_lens,
      slot_mapping (flat, the last num_tokens slots per job -- the reference
      pads this to 2-D and then consumes it flat, which is only right when all
      jobs add the same token count; the flat list is what it means),
      fill_q_lens, fill_kv_lens, fill_slots (whole context incl. ancestors).
    """
    ctxs = [j["context"] for j in jobs]
    P = ref_shared_context_len(ctxs)
    out: Dict[str, object] = {
        "flash_context_len": P,
        "flash_block_table": ctxs[0].context_slot_ids()[:P],
        "paged_block_tables": [],
        "paged_context_lens": [],
        "slot_mapping": [],
        "fill_q_lens": [],
        "fill_kv_lens": [],
        "fill_slots": [],
    }
    for j in jobs:
        slots = j["context"].context_slot_ids()
        n = j["num_tokens"]
        out["slot_mapping"].extend(slots[-n:])
        if j["kind"] == "generate":
            out["paged_block_tables"].append(slots[P:])
            out["paged_context_lens"].append(len(slots) - P)
        else:
            out["fill_q_lens"].append(n)
            out["fill_kv_lens"].append(len(slots))
            out["fill_slots"].extend(slots)
    return out
