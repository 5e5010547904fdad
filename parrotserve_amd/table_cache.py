"""Slot tables of a decode batch kept across iterations.

The reference rebuilds every index tensor from Python lists at each iteration
(parrot/engine/builtin/attn_func.py:462-599): O(sum of context lengths) list
work plus several uploads per iteration.  Between two decode iterations of the
same batch nothing changes except that every Generate job's context gained the
one slot of the token being generated, so the device tables of the previous
iteration are patched instead: O(batch) host work, one upload of the new slots,
one tiny kernel (``ph_suffix_tables_append``), and a fresh balanced suffix plan
(its cut points move with the lengths) that a second tiny kernel writes from
the device length vector (``ph_suffix_plan_build``).

A batch qualifies when it consists of Generate jobs only, bound to the same
context objects in the same order as the cached iteration, each context exactly
one token longer and hanging under the same parent of unchanged length.
Anything else (a Fill in the batch, a job that joined or left, a context that
was rewound) falls back to the full build, which then becomes the cached state.
"""
from __future__ import annotations

import dataclasses
from typing import Any, List, Optional, Sequence

import numpy as np
import torch

from . import kernels
from .primitive_job import Generate


@dataclasses.dataclass
class _Cached:
    contexts: List[Any]            # job order
    parents: List[Any]
    own_lens: List[int]            # len(context.token_kv_block_ids) at the cached iteration
    parent_lens: List[int]         # get_context_len() of each parent (0 without parent)
    rows: Optional[torch.Tensor]   # device int32: table row of job i (None = identity)
    lens_host: np.ndarray          # int64, table-row order
    tables: Any                    # kernels.DecodeTables (patched in place)
    decode_perm: Any
    flash_context_len: int
    num_heads: int
    head_dim: int
    dtype: Any = torch.float16     # element type of the caches (the library's launch choice depends on it)
    slot_mapping: Any = None       # device int32 [B], job order: this iteration's new slots


class DecodeTableCache:
    """One cached decode batch per plug-in class (the engine runs one batch at a time)."""

    def __init__(self) -> None:
        self.state: Optional[_Cached] = None
        self.hits = 0
        self.rebuilds = 0

    def clear(self) -> None:
        self.state = None

    def advance_host(self, jobs: Sequence[Any]) -> Optional[List[int]]:
        """If ``jobs`` is the cached batch one token later, return the new slot of every job (job
        order) and move the cached host-side lengths forward; otherwise ``None`` (cache untouched)."""
        c = self.state
        if c is None or len(jobs) != len(c.contexts):
            return None
        new_slots: List[int] = []
        for i, job in enumerate(jobs):
            ctx = getattr(job, "context", None)
            if not isinstance(job, Generate) or ctx is not c.contexts[i] or ctx.parent_context is not c.parents[i]:
                return None
            own = ctx.token_kv_block_ids
            if len(own) != c.own_lens[i] + 1:
                return None
            p = c.parents[i]
            if (p.get_context_len() if p is not None else 0) != c.parent_lens[i]:
                return None
            new_slots.append(own[-1])
        for i in range(len(jobs)):
            c.own_lens[i] += 1
        c.lens_host += 1
        return new_slots

    def advance(self, jobs: Sequence[Any], device) -> Optional[_Cached]:
        """Patch the cached device tables for the next iteration; ``None`` when the batch does not qualify."""
        new_slots = self.advance_host(jobs)
        if new_slots is None:
            return None
        c = self.state
        t = c.tables
        need = int(c.lens_host.max())
        if t.suffix_slots is None or need > t.suffix_table_stride:
            _widen(t, need, device)
        c.slot_mapping = torch.from_numpy(np.asarray(new_slots, dtype=np.int32)).to(device)
        kernels.suffix_tables_append(t.suffix_slots, t.suffix_lens, c.rows, c.slot_mapping)
        t.max_suffix_len = need
        shape = dict(num_reqs=t.num_reqs, num_groups=t.num_groups, max_prefix_len=t.max_prefix_len,
                     max_suffix_len=need, dtype=c.dtype)
        if t.num_reqs <= kernels.PLAN_MAX_REQS:  # the cut points move with the lengths: a fresh plan, built on the device
            # (the lane count follows the library's launch choice for the batch's shape: it moves at a few thresholds
            # of the growing lengths, and the plan's arrays are laid out anew when it does)
            lanes = kernels.suffix_lane_capacity(device, c.num_heads, c.head_dim, **shape)
            t.plan_on_device(lanes, device)
        else:
            total = int(c.lens_host.sum())
            t.set_plan(c.lens_host, kernels.suffix_lanes(device, c.num_heads, c.head_dim, total, **shape), device)
        self.hits += 1
        return c

    def store(self, jobs: Sequence[Any], order: List[int], suffix_lens: Sequence[int], tables, decode_perm,
              flash_context_len: int, num_heads: int, head_dim: int, device, dtype=torch.float16) -> None:
        """Remember a batch that was just built from scratch.  ``order[r]`` = job whose suffix is table
        row r; ``suffix_lens`` in table-row order."""
        self.rebuilds += 1
        if not jobs or not all(isinstance(j, Generate) for j in jobs):
            self.state = None
            return
        ctxs = [j.context for j in jobs]
        parents = [c.parent_context for c in ctxs]
        B = len(jobs)
        rows = None
        if order != list(range(B)):
            rows_host = np.empty(B, dtype=np.int32)
            rows_host[np.asarray(order)] = np.arange(B, dtype=np.int32)  # job i sits in table row rows_host[i]
            rows = torch.from_numpy(rows_host).to(device)
        self.state = _Cached(ctxs, parents, [len(c.token_kv_block_ids) for c in ctxs],
                             [p.get_context_len() if p is not None else 0 for p in parents], rows,
                             np.asarray(list(suffix_lens), dtype=np.int64), tables, decode_perm, flash_context_len,
                             num_heads, head_dim, dtype)


def _widen(t, need: int, device) -> None:
    """Give the padded suffix table room for ``need`` tokens per row (doubling, multiples of 64)."""
    old = t.suffix_slots
    width = max(64, (max(need, 2 * t.suffix_table_stride) + 63) // 64 * 64)
    new = torch.zeros((t.num_reqs, width), dtype=torch.int32, device=device)
    if old is not None:
        new[:, : old.shape[1]] = old
    else:
        t.suffix_lens = torch.zeros(t.num_reqs, dtype=torch.int32, device=device)
        t.suffix_offsets = None
    t.suffix_slots = new
    t.suffix_table_stride = width
