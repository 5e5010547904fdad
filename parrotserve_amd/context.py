"""Slot allocator and context tree of the engine, token-granular (block_size 1).

Mirrors ``RecyclePool`` (parrot/utils/recycle_pool.py:11-65), ``LowLevelContext``
(parrot/engine/context/low_level_context.py:15-52) and ``BlockContext``
(parrot/engine/context/block_context.py:13-135): same method names, same id
order (fresh ids ascend, freed ids are reused oldest-first, the last id of a
bounded pool is never issued), same errors.  A child context owns only its own
slots and reads its ancestors' through ``get_context_slot_ids()``; forking
copies no KV.
"""
from __future__ import annotations

from collections import deque
from typing import Deque, List, Optional


class ParrotError(Exception):
    """parrot/exceptions.py: engine-level error (pool exhausted, ...)."""


class RecyclePool:
    """Ids 0, 1, 2, ... with recycling.  The pool's state is the recycled ids -- a queue in the order they came
    back and a set for membership -- plus the number of fresh ids issued so far; everything else is derived or
    bookkeeping.  Behaviour kept from the reference because callers and tests can see it: recycled ids go out
    oldest first and before any fresh id (unless ``debug_mode``, which only ever issues fresh ones); a bounded
    pool never issues its last id (``pool_size - 1``); the allocation count moves before the failure checks (an
    exhausted ``allocate`` and a double ``free`` both leave it changed); the high-water mark is only sampled when a
    recycled id goes out."""

    def __init__(self, pool_name: str = "pool", pool_size: Optional[int] = None, debug_mode: bool = False) -> None:
        self.pool_name = pool_name
        self.pool_size = pool_size
        self.debug_mode = debug_mode
        self.free_ids: Deque[int] = deque()   # recycled ids, oldest first
        self._recycled = set()                # the same ids, for the double-free check
        self.cur_max_id = 0                   # fresh ids issued so far (the next fresh id)
        self.allocated_num = 0
        self.history_max = 0

    def _fresh(self) -> int:
        issued = self.cur_max_id
        self.cur_max_id = issued + 1
        if self.pool_size is not None and issued + 1 >= self.pool_size:
            raise ParrotError(f"No free ids in Pool: {self.pool_name} (pool_size={self.pool_size}).")
        return issued

    def allocate(self) -> int:
        self.allocated_num += 1
        if self.debug_mode or not self.free_ids:
            return self._fresh()
        reused = self.free_ids.popleft()
        self._recycled.remove(reused)
        if self.allocated_num > self.history_max:
            self.history_max = self.allocated_num
        return reused

    def free(self, id: int) -> None:
        self.allocated_num -= 1
        if id in self._recycled:
            raise ValueError("The id is already free.")
        self._recycled.add(id)
        self.free_ids.append(id)

    def get_allocated_num(self) -> int:
        return self.allocated_num

    def get_history_max_allocated_num(self) -> int:
        return self.history_max


class BlockContext:
    """One node of the context tree; ``block_size`` must be 1 (token-granular pool)."""

    def __init__(self, context_id: int, parent_context: Optional["BlockContext"], kv_cache_manager: RecyclePool,
                 block_size: int = 1):
        if block_size != 1:
            raise ValueError("this build uses the token-granular KV layout: block_size must be 1")
        self.context_id = context_id
        self.sub_context_ids: List[int] = []
        self.depth = 0
        self.parent_context = parent_context
        if parent_context is not None:
            parent_context.sub_context_ids.append(context_id)
            self.depth = parent_context.depth + 1
            parent_context.padded = True  # pad-on-fork of the reference; zero tokens at block_size 1
        self.block_size = 1
        self.padded = False
        self.padded_len = 0
        self.token_kv_block_ids: List[int] = []  # == slot ids at block_size 1 (same list object)
        self.token_kv_slot_ids: List[int] = self.token_kv_block_ids
        self.token_ids: List[int] = []
        self.kv_cache_manager = kv_cache_manager
        self.last_hidden_state = None

    # -- allocation ------------------------------------------------------- #
    def allocate(self, length: int) -> None:
        alloc = self.kv_cache_manager.allocate
        for _ in range(length):
            self.token_kv_block_ids.append(alloc())

    def destruction(self) -> None:
        if self.parent_context is not None:
            self.parent_context.sub_context_ids.remove(self.context_id)
        assert len(self.sub_context_ids) == 0, f"Sub-contexts {self.sub_context_ids[0]} should be deleted first."
        for slot in self.token_kv_block_ids:
            self.kv_cache_manager.free(slot)

    # -- lengths ---------------------------------------------------------- #
    def get_this_context_len(self) -> int:
        return len(self.token_kv_block_ids)

    def get_context_len(self) -> int:
        n, c = 0, self
        while c is not None:
            n += len(c.token_kv_block_ids)
            c = c.parent_context
        return n

    # -- slot tables ------------------------------------------------------ #
    def get_context_slot_ids(self) -> List[int]:
        chain, c = [], self
        while c is not None:
            chain.append(c.token_kv_block_ids)
            c = c.parent_context
        out: List[int] = []
        for part in reversed(chain):
            out.extend(part)
        return out

    def get_context_block_ids(self) -> List[int]:
        return self.get_context_slot_ids()

    # -- tokens ----------------------------------------------------------- #
    def get_last_token_id(self) -> int:
        return self.token_ids[-1]

    def push_token_id(self, token_id: int) -> None:
        self.token_ids.append(token_id)

    def get_last_hidden_state(self):
        if len(self.token_ids) == 0:
            assert self.parent_context is not None, "The parent context should not be None if this is an empty context."
            return self.parent_context.get_last_hidden_state()
        return self.last_hidden_state
