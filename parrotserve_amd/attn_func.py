"""Attention plug-in of the builtin engine on the HIP kernels.

Same contract as the reference's ``AttnFunc`` classes
(parrot/engine/builtin/attn_func.py:31-55): ``__init__(layer_idx, scaling,
num_heads, head_dim)``, a static ``init_iteration_state(iteration_state,
builtin_config, jobs, num_heads, head_size)`` that turns the jobs' context trees
into index tensors once per iteration, and ``forward(q, k, v, iteration_state)
-> [T, H*D]`` with Fill tokens first, then one token per Generate job.

``forward`` = KV append by slot, prefill-with-parent-context for the Fill
tokens, shared-prefix decode (prefix phase + suffix phase + merge) for the
Generate tokens.  The three reference selector strings all resolve to this
class (the KV layout is token-granular for all of them here).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
from torch import nn

from . import kernels
from .table_cache import DecodeTableCache
from .mem import get_k_cache, get_v_cache
from .primitive_job import Fill, Generate

ATTN_FUNCS = [
    "xformers_with_buffer",
    "xformers_fill_vllm_paged_attention_generate",
    "xformers_fill_shared_prompts_generate",
    "hip_shared_prefix",
]


# --------------------------------------------------------------------------- #
# host-side index tables (pure python, no device)
# --------------------------------------------------------------------------- #
def _lca(context1, context2):
    """Lowest common ancestor of two context nodes, ``None`` if they sit in different trees (what
    attn_func.py:412-439 computes).  The deeper node is lifted to the other's depth, then both climb together."""
    a, b = context1, context2
    if a is None or b is None:
        return None
    if a.depth < b.depth:
        a, b = b, a
    for _ in range(a.depth - b.depth):
        a = a.parent_context
    while a is not b:
        if a is None or b is None:
            return None
        a, b = a.parent_context, b.parent_context
    return a


def get_shared_context_len(jobs: Sequence[Any]) -> int:
    """Tokens of context shared by ALL jobs: the context length of the lowest common ancestor of every job's
    context, 0 when there is none (attn_func.py:441-459)."""
    assert len(jobs) > 0
    common = jobs[0].context
    for job in jobs[1:]:
        common = _lca(common, job.context)
        if common is None:
            return 0
    return common.get_context_len()


@dataclasses.dataclass
class IterationTables:
    """Index tables of one iteration as python lists (what the reference uploads
    as tensors, attn_func.py:462-599, at block_size 1)."""

    flash_context_len: int
    flash_block_table: List[int]
    paged_block_tables: List[List[int]]  # ragged; the reference pads with 0
    paged_context_lens: List[int]
    slot_mapping: List[int]  # flat [T]
    fill_q_lens: List[int]
    fill_kv_lens: List[int]
    fill_slots: List[int]
    fill_slot_lists: List[List[int]]
    # prefix groups over the Generate jobs: (prefix slot list, generate indices)
    groups: List[Tuple[List[int], List[int]]]
    num_fill_tokens: List[int]
    num_generates: int


def build_iteration_tables(jobs: Sequence[Any], grouping: str = "lca") -> IterationTables:
    """``grouping="lca"``: one prefix shared by every job of the iteration, the
    reference's rule.  ``grouping="parent"``: Generate jobs that descend from a common
    context form a group whose prefix is that context's whole chain -- the deepest
    such context per job, so several prompt groups can share the iteration and a
    batch the reference's rule covers gets the same prefix from it."""
    assert grouping in ("lca", "parent")
    P = get_shared_context_len(jobs) if grouping == "lca" else 0
    slots0 = jobs[0].context.get_context_slot_ids() if P > 0 else []
    t = IterationTables(P, slots0[:P], [], [], [], [], [], [], [], [], [], 0)
    gen_full: List[List[int]] = []    # "lca": every Generate job's whole context
    gen_own: List[Any] = []           # "parent": every Generate job's context ...
    gen_parent: List[Any] = []        # ... and its fork parent
    for job in jobs:
        if isinstance(job, Fill):
            slots = job.context.get_context_slot_ids()
            n = len(job.token_ids)
            t.num_fill_tokens.append(n)
            t.fill_q_lens.append(n)
            t.fill_kv_lens.append(len(slots))
            t.fill_slots.extend(slots)
            t.fill_slot_lists.append(slots)
            t.slot_mapping.extend(slots[-n:])
        elif isinstance(job, Generate):
            t.num_generates += 1
            if grouping == "lca":
                slots = job.context.get_context_slot_ids()
                gen_full.append(slots)
                t.slot_mapping.append(slots[-1])
            else:
                # an ancestor's list is taken once per group below, not copied into every job's list
                gen_own.append(job.context)
                gen_parent.append(job.context.parent_context)
                t.slot_mapping.append(job.context.token_kv_block_ids[-1])
        else:
            raise TypeError(f"unknown job type {type(job)}")
    if grouping == "lca":
        for slots in gen_full:
            t.paged_block_tables.append(slots[P:])
            t.paged_context_lens.append(len(slots) - P)
        if P > 0 and gen_full:
            t.groups.append((t.flash_block_table, list(range(len(gen_full)))))
    else:
        # A job's group is the deepest ancestor context that at least two Generate jobs of the iteration descend
        # from (its fork parent when siblings decode together; a grandparent when every job sits under a
        # context of its own, as in tests/engine/builtin/test_shared_prefix.py:57-115 of the reference); the
        # group's prefix is that ancestor's whole context, a job's own list everything below it.
        below: Dict[int, int] = {}
        for parent in gen_parent:
            c = parent
            while c is not None:
                below[id(c)] = below.get(id(c), 0) + 1
                c = c.parent_context
        by_anchor: Dict[int, int] = {}
        for i, (ctx, parent) in enumerate(zip(gen_own, gen_parent)):
            own = [ctx.token_kv_block_ids]
            anchor = parent
            while anchor is not None and below[id(anchor)] < 2:
                own.append(anchor.token_kv_block_ids)
                anchor = anchor.parent_context
            g = None
            if anchor is not None:
                g = by_anchor.get(id(anchor))
                if g is None:
                    prefix = anchor.get_context_slot_ids()
                    if prefix:
                        g = by_anchor[id(anchor)] = len(t.groups)
                        t.groups.append((prefix, []))
                    else:
                        by_anchor[id(anchor)] = g = -1
                if g < 0:
                    g = None
            if g is None:  # nothing shared: the whole context is the job's own list
                slots = ctx.get_context_slot_ids()
            else:
                t.groups[g][1].append(i)
                slots = [s for part in reversed(own) for s in part]
            t.paged_block_tables.append(slots)
            t.paged_context_lens.append(len(slots))
        # a group that ended up with a single member (its siblings found a deeper anchor) shares nothing
        for prefix, members in t.groups:
            if len(members) == 1:
                i = members[0]
                t.paged_block_tables[i] = prefix + t.paged_block_tables[i]
                t.paged_context_lens[i] = len(t.paged_block_tables[i])
        t.groups = [gm for gm in t.groups if len(gm[1]) > 1]
    return t


def forked_fill_tables(jobs: Sequence[Any], min_parent_len: int, max_own_len: int, pay_ratio: int = 4):
    """Fill jobs forked from common parents, as a shared-prefix *decode* problem: every new token is a request,
    the parent's whole context is the prefix its group shares, and its suffix is its own context up to itself
    (the causal part).  The parent's K/V is then read once per group of up to 256 new tokens instead of once per
    chunk, which is what the prefix phase exists for.  Worth it for short chunks over long shared parents (the
    forked prompts of the reference's experiments: tens of tokens over thousands); returns None otherwise, i.e.
    unless every Fill of the iteration has a parent of at least ``min_parent_len`` tokens that it shares with a
    neighbouring Fill, and an own context of at most ``max_own_len`` tokens -- and unless it pays: the suffix phase
    reads a token's own context once per *token* (no reuse across the chunk's queries), so the (query, own key)
    pairs it adds must stay well under the parent rows it saves (``1 / pay_ratio`` of them: chunks of about
    sqrt(P / 2) tokens over a P-token parent at the most).
    Returns (prefix slot lists, token offsets of the groups, per-token suffix slot lists)."""
    fills = [j for j in jobs if isinstance(j, Fill)]
    if len(fills) < 2:
        return None
    prefix_lists: List[List[int]] = []
    gcu = [0]
    suffix_lists: List[List[int]] = []
    last_parent = None
    members = 0
    own_pairs = 0      # (query, own key) pairs the suffix phase would read
    parent_rows = 0    # parent rows read chunk by chunk
    for job in fills:
        parent = job.context.parent_context
        plen = parent.get_context_len() if parent is not None else 0
        slots = job.context.get_context_slot_ids()
        own = slots[plen:]
        n = len(job.token_ids)
        if parent is None or plen < min_parent_len or len(own) > max_own_len:
            return None
        if parent is not last_parent:
            if last_parent is not None:
                if members < 2:
                    return None
                gcu.append(len(suffix_lists))
            prefix_lists.append(slots[:plen])
            last_parent = parent
            members = 0
        members += 1
        first = len(own) - n
        for r in range(n):
            suffix_lists.append(own[: first + r + 1])
        own_pairs += n * first + n * (n + 1) // 2
        parent_rows += plen
    if members < 2:
        return None
    gcu.append(len(suffix_lists))
    # parent rows read as a shared prefix: once per 256 new tokens of a group
    shared_rows = sum(len(p) * ((gcu[g + 1] - gcu[g] + 255) // 256) for g, p in enumerate(prefix_lists))
    if pay_ratio * own_pairs > parent_rows - shared_rows:
        return None
    return prefix_lists, gcu, suffix_lists


# --------------------------------------------------------------------------- #
# the plug-in
# --------------------------------------------------------------------------- #
class AttnFunc(nn.Module):
    """Base class (attn_func.py:31-55)."""

    def __init__(self, layer_idx: int, scaling: float, num_heads: int, head_dim: int):
        super().__init__()
        self.layer_idx = layer_idx
        self.scaling = scaling
        self.num_heads = num_heads
        self.head_dim = head_dim

    @staticmethod
    def init_iteration_state(iteration_state, builtin_config, jobs, num_heads: int, head_size: int):
        raise NotImplementedError


class HipSharedPrefixAttn(AttnFunc):
    """Fill: prefill with parent context.  Generate: shared-prefix decode."""

    grouping = "lca"
    # device tables of the last decode-only batch, patched in place while the same batch keeps generating
    table_cache = DecodeTableCache()
    incremental = True
    # Fill jobs forked from a shared parent run as a shared-prefix decode over their new tokens when the parent is
    # at least this long and every chunk's own context at most that long (see forked_fill_tables); 0 switches it off
    forked_fill_min_parent = 256
    forked_fill_max_own = 64
    forked_fill_pay_ratio = 4

    @classmethod
    def init_iteration_state(cls, iteration_state, builtin_config, jobs, num_heads: int, head_size: int):
        device = builtin_config.device
        dtype = getattr(builtin_config, "dtype", torch.float16)
        if not isinstance(dtype, torch.dtype):
            dtype = torch.float16
        st = iteration_state
        cached = cls.table_cache.advance(jobs, device) if cls.incremental else None
        if cached is not None:
            st.generation_sampling_config.extend(j.sampling_config for j in jobs)
            st.tables = None  # the python-list form is not rebuilt on this path
            st.flash_context_len = cached.flash_context_len
            st.slot_mapping = cached.slot_mapping
            st.fill_tables = None
            st.fill_decode_tables = None
            st.decode_tables = cached.tables
            st.decode_perm = cached.decode_perm
            return
        tabs = build_iteration_tables(jobs, cls.grouping)
        st.num_fill_tokens.extend(tabs.num_fill_tokens)
        st.generation_sampling_config.extend(j.sampling_config for j in jobs if isinstance(j, Generate))
        st.tables = tabs
        # names the reference attaches (attn_func.py:571-599)
        st.flash_context_len = tabs.flash_context_len
        st.slot_mapping = torch.from_numpy(np.asarray(tabs.slot_mapping, dtype=np.int32)).to(device)
        st.fill_tables = None
        st.fill_decode_tables = None
        if tabs.fill_q_lens:
            forked = None
            if cls.forked_fill_min_parent > 0 and head_size == 128:
                forked = forked_fill_tables(jobs, cls.forked_fill_min_parent, cls.forked_fill_max_own,
                                            cls.forked_fill_pay_ratio)
            if forked is not None:
                st.fill_decode_tables = kernels.DecodeTables.build(*forked, device, num_heads=num_heads,
                                                                   head_dim=head_size, dtype=dtype)
            else:
                st.fill_tables = kernels.PrefillTables.build(tabs.fill_q_lens, tabs.fill_slot_lists, device)
        st.decode_tables = None
        st.decode_perm = None
        if tabs.num_generates:
            # requests of one prefix group must be adjacent: order = groups first, ungrouped last
            order: List[int] = []
            gcu = [0]
            for _, members in tabs.groups:
                order.extend(members)
                gcu.append(len(order))
            grouped = set(order)
            order.extend(i for i in range(tabs.num_generates) if i not in grouped)
            suffix = [tabs.paged_block_tables[i] for i in order]
            st.decode_tables = kernels.DecodeTables.build([p for p, _ in tabs.groups], gcu if tabs.groups else [],
                                                          suffix, device, num_heads=num_heads, head_dim=head_size,
                                                          dtype=dtype)
            if order != list(range(tabs.num_generates)):
                perm = torch.tensor(order, dtype=torch.int64, device=device)
                inv = torch.empty_like(perm)
                inv[perm] = torch.arange(len(order), dtype=torch.int64, device=device)
                st.decode_perm = (perm, inv)
            if cls.incremental:
                cls.table_cache.store(jobs, order, [len(x) for x in suffix], st.decode_tables, st.decode_perm,
                                      tabs.flash_context_len, num_heads, head_size, device, dtype)
        elif cls.incremental:
            cls.table_cache.clear()

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, iteration_state,
                kv_appended: bool = False) -> torch.Tensor:
        """``kv_appended``: the caller has already written this iteration's k, v rows to their slots (the fused
        rotary + append kernel does); the reference's four-argument call appends here."""
        st = iteration_state
        k_cache = get_k_cache(self.layer_idx)
        v_cache = get_v_cache(self.layer_idx)
        if not kv_appended:
            kernels.kv_append(k, v, k_cache, v_cache, st.slot_mapping)
        T = q.shape[0]
        if q.stride(1) != self.head_dim or q.stride(2) != 1:
            q = q.contiguous()
        output = torch.empty((T, self.num_heads, self.head_dim), dtype=q.dtype, device=q.device)
        nf = st.num_total_fill_tokens
        if nf > 0 and st.fill_decode_tables is not None:  # forked Fills: the parent is a shared prefix of their tokens
            kernels.decode_attention(q[:nf], k_cache, v_cache, st.fill_decode_tables, scale=self.scaling,
                                     out=output[:nf])
        elif nf > 0:
            kernels.prefill_attention(q[:nf], k_cache, v_cache, st.fill_tables, scale=self.scaling, out=output[:nf])
        if st.num_generation_jobs > 0:
            q_gen = q[nf:]
            if st.decode_perm is None:
                kernels.decode_attention(q_gen, k_cache, v_cache, st.decode_tables, scale=self.scaling, out=output[nf:])
            else:
                perm, inv = st.decode_perm
                o = kernels.decode_attention(q_gen.index_select(0, perm), k_cache, v_cache, st.decode_tables,
                                             scale=self.scaling)
                output[nf:] = o.index_select(0, inv)
        return output.view(-1, self.num_heads * self.head_dim)


class HipGroupedPrefixAttn(HipSharedPrefixAttn):
    """Same kernels; prefix groups are detected per fork parent, so several prompt
    groups in one batch each keep their shared-prefix phase."""

    grouping = "parent"
    table_cache = DecodeTableCache()


def get_attn_func(attn_func_name: str):
    """Selector of ``instance.attn_func`` (attn_func.py:711-737): unknown names raise ValueError."""
    if attn_func_name in ("xformers_with_buffer", "xformers_fill_vllm_paged_attention_generate",
                          "xformers_fill_shared_prompts_generate"):
        return HipSharedPrefixAttn
    if attn_func_name == "hip_shared_prefix":
        return HipGroupedPrefixAttn
    raise ValueError(f"Unknown attention function name: {attn_func_name}. Supported attetion functions: {ATTN_FUNCS}")


@dataclasses.dataclass
class BuiltinConfig:
    """The fields of ``BuiltinConfig`` the attention path reads (parrot/engine/config.py:28-60)."""

    num_kv_cache_blocks: int
    attn_func: Any = "xformers_fill_shared_prompts_generate"
    dtype: Any = torch.float16
    device: Any = "cuda"
    block_size: int = 1
    max_seq_len: Optional[int] = None

    def __post_init__(self):
        if isinstance(self.dtype, str):
            # float16 / float32 are the reference's choices (parrot/engine/config.py:22-25); bfloat16 its kernels' third
            table = {"float16": torch.float16, "float32": torch.float32, "bfloat16": torch.bfloat16}
            if self.dtype not in table:
                raise ValueError(f"Unknown dtype {self.dtype}")
            self.dtype = table[self.dtype]
        if self.block_size != 1:
            raise ValueError("block_size must be 1: the KV pool is token-granular")
        self.attn_func_name = self.attn_func if isinstance(self.attn_func, str) else self.attn_func.__name__
        if isinstance(self.attn_func, str):
            self.attn_func = get_attn_func(self.attn_func)
