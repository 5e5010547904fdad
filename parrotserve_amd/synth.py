"""Seeded synthetic workloads of the five benchmark configurations.

Everything is generated on the CPU with ``torch.Generator().manual_seed(seed)``
and then cast / moved, so a CPU checker and the GPU kernels see identical bits.
A case is held in *compact* form: only the KV rows that some request references
exist (``k_rows[i]`` lives at pool slot ``used_slots[i]``); ``to_device``
scatters them into a zero-filled ``[pool_slots, H, D]`` pool.  Slot lists in a
case are compact row indices; ``used_slots`` maps them to pool slot ids.
"""
from __future__ import annotations

import dataclasses
import math
from typing import List, Optional, Sequence

import torch


@dataclasses.dataclass
class DecodeCase:
    """Decode requests over a scattered slot pool; optional shared prefix groups."""

    name: str
    dtype: torch.dtype
    q: torch.Tensor  # [B, H, D]
    k_rows: torch.Tensor  # [n_used, H, D]
    v_rows: torch.Tensor
    used_slots: torch.Tensor  # int64 [n_used] pool slot of each compact row
    pool_slots: int
    prefix_lists: List[torch.Tensor]  # per group, compact indices
    group_req_cu: List[int]
    suffix_lists: List[torch.Tensor]  # per request, compact indices

    @property
    def num_reqs(self) -> int:
        return self.q.shape[0]

    def full_lists(self) -> List[torch.Tensor]:
        """prefix(group(b)) || suffix(b) per request, compact indices."""
        out = []
        for b in range(self.num_reqs):
            pre = None
            for g in range(len(self.prefix_lists)):
                if self.group_req_cu[g] <= b < self.group_req_cu[g + 1]:
                    pre = self.prefix_lists[g]
            out.append(self.suffix_lists[b] if pre is None else torch.cat([pre, self.suffix_lists[b]]))
        return out

    def pool_lists(self, lists: Sequence[torch.Tensor]) -> List[List[int]]:
        return [self.used_slots[l].tolist() for l in lists]


def _randn(gen, shape, dtype):
    return torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype)


def make_decode_case(name: str, seed: int, dtype: torch.dtype, groups: int, reqs_per_group: int, prefix_len: int,
                     suffix_lens: Sequence[int], num_heads: int, head_dim: int, pool_slots: int,
                     group_sizes: Sequence[int] = ()) -> DecodeCase:
    """``groups`` prefix groups of ``reqs_per_group`` requests each, or of ``group_sizes[g]`` requests when given
    (``reqs_per_group`` is then ignored)."""
    gen = torch.Generator().manual_seed(seed)
    if group_sizes:
        assert len(group_sizes) == groups
    B = int(sum(group_sizes)) if group_sizes else groups * reqs_per_group
    assert len(suffix_lens) == B
    n_used = groups * prefix_len + int(sum(suffix_lens))
    assert n_used <= pool_slots
    perm = torch.randperm(pool_slots, generator=gen)
    used = perm[:n_used].clone()
    pos = 0
    prefix_lists = []
    for _ in range(groups):
        prefix_lists.append(torch.arange(pos, pos + prefix_len))
        pos += prefix_len
    suffix_lists = []
    for s in suffix_lens:
        suffix_lists.append(torch.arange(pos, pos + int(s)))
        pos += int(s)
    q = _randn(gen, (B, num_heads, head_dim), dtype)
    k = _randn(gen, (n_used, num_heads, head_dim), dtype)
    v = _randn(gen, (n_used, num_heads, head_dim), dtype)
    if group_sizes:
        gcu = [0]
        for n in group_sizes:
            gcu.append(gcu[-1] + int(n))
    else:
        gcu = [g * reqs_per_group for g in range(groups + 1)]
    if prefix_len <= 0:
        gcu = []
    return DecodeCase(name, dtype, q, k, v, used, pool_slots, prefix_lists if prefix_len > 0 else [], gcu,
                      suffix_lists)


def _randint(gen, lo, hi, n):
    return torch.randint(lo, hi + 1, (n,), generator=gen).tolist()


def config1(scale: float = 1.0) -> DecodeCase:
    """C1: fp32 CPU plumbing -- B 8, prefix 512, suffix U[32,128], 32x128, seed 0."""
    gen = torch.Generator().manual_seed(0)
    s = _randint(gen, 32, 128, 8)
    P = max(1, int(512 * scale))
    return make_decode_case("C1", 0, torch.float32, 1, 8, P, s, 32, 128, P + sum(s))


def config2(batch: int = 64, prefix: int = 4096, pool_slots: int = 1 << 20, dtype=torch.float16) -> DecodeCase:
    """C2: fp16, B 64 share one 4096-token prefix, suffix U[16,512], 32x128, 1M-slot pool, seed 1."""
    gen = torch.Generator().manual_seed(1)
    s = _randint(gen, 16, 512, batch)
    return make_decode_case("C2", 1, dtype, 1, batch, prefix, s, 32, 128, pool_slots)


def config3(batch: int = 256, lo: int = 128, hi: int = 8192, pool_slots: int = 1 << 22) -> DecodeCase:
    """C3: fp16 ragged non-shared decode, ctx log-uniform[128,8192], 4M-slot pool, seed 2."""
    gen = torch.Generator().manual_seed(2)
    u = torch.rand(batch, generator=gen, dtype=torch.float64)
    ctx = torch.round(torch.exp(math.log(lo) + u * (math.log(hi) - math.log(lo)))).long().tolist()
    return make_decode_case("C3", 2, torch.float16, 1, batch, 0, ctx, 32, 128, pool_slots)


def config3_move(n: int = 65536, pool_slots: int = 1 << 22, index_dtype=torch.int64):
    """C3 token move: n random src -> n unique dst slots (disjoint from src)."""
    gen = torch.Generator().manual_seed(2)
    src = torch.randperm(pool_slots, generator=gen)[:n]
    mask = torch.ones(pool_slots, dtype=torch.bool)
    mask[src] = False
    free = torch.nonzero(mask).flatten()
    dst = free[torch.randperm(free.numel(), generator=gen)[:n]]
    return src.to(index_dtype), dst.to(index_dtype)


@dataclasses.dataclass
class PrefillCase:
    name: str
    dtype: torch.dtype
    q: torch.Tensor  # [T, H, D] pre-RoPE
    k_new: torch.Tensor  # [T, H, D] pre-RoPE
    v_new: torch.Tensor
    positions: torch.Tensor  # int64 [T]
    q_lens: List[int]
    k_rows: torch.Tensor  # compact parent rows (already rotated keys, as a cache holds them)
    v_rows: torch.Tensor
    used_slots: torch.Tensor  # pool slots: parents first, then the new tokens' slots
    pool_slots: int
    parent_lists: List[torch.Tensor]  # compact indices of each chunk's parent context
    new_lists: List[torch.Tensor]  # compact indices (into used_slots) of each chunk's new tokens
    theta: float


def make_prefill_case(name: str, seed: int, dtype, q_lens: Sequence[int], parent_len: int, num_heads: int,
                      head_dim: int, pool_slots: int, theta: float = 10000.0) -> PrefillCase:
    gen = torch.Generator().manual_seed(seed)
    C = len(q_lens)
    T = int(sum(q_lens))
    n_par = C * parent_len
    perm = torch.randperm(pool_slots, generator=gen)
    used = perm[: n_par + T].clone()
    parent_lists, new_lists, pos_list = [], [], []
    p = n_par
    for c, n in enumerate(q_lens):
        parent_lists.append(torch.arange(c * parent_len, (c + 1) * parent_len))
        new_lists.append(torch.arange(p, p + n))
        pos_list.append(torch.arange(parent_len, parent_len + n))
        p += n
    q = _randn(gen, (T, num_heads, head_dim), dtype)
    k_new = _randn(gen, (T, num_heads, head_dim), dtype)
    v_new = _randn(gen, (T, num_heads, head_dim), dtype)
    k_rows = _randn(gen, (n_par, num_heads, head_dim), dtype)
    v_rows = _randn(gen, (n_par, num_heads, head_dim), dtype)
    return PrefillCase(name, dtype, q, k_new, v_new, torch.cat(pos_list).long(), list(q_lens), k_rows, v_rows, used,
                       pool_slots, parent_lists, new_lists, theta)


def config4(chunks: int = 16, lo: int = 64, hi: int = 1024, parent: int = 2048, pool_slots: int = 1 << 18) -> PrefillCase:
    """C4: bf16 prefill, 16 ragged chunks U[64,1024] over 2048-token parents, 40x128, RoPE theta 1e4, seed 3."""
    gen = torch.Generator().manual_seed(3)
    n = _randint(gen, lo, hi, chunks)
    return make_prefill_case("C4", 3, torch.bfloat16, n, parent, 40, 128, pool_slots)


@dataclasses.dataclass
class LayerCase:
    """C5: one LLaMA-13B decoder layer over a mixed batch of prefix groups."""

    decode: DecodeCase  # q unused; KV rows are the cached context
    x: torch.Tensor  # [B, hidden]
    positions: torch.Tensor  # int64 [B] = context length before this token
    new_slots: torch.Tensor  # int64 [B] pool slot of each request's new token
    weights: dict
    eps: float
    theta: float


def config5(groups: int = 4, branches: int = 32, prefix: int = 6000, s_lo: int = 32, s_hi: int = 1024,
            hidden: int = 5120, heads: int = 40, ffn: int = 13824, pool_slots: int = 1 << 18) -> LayerCase:
    """C5: fp16 LLaMA-13B layer, weights N(0, 0.02), 4 groups x 32 branches, prefix 6000, suffix U[32,1024], seed 4."""
    gen = torch.Generator().manual_seed(4)
    B = groups * branches
    s = _randint(gen, s_lo, s_hi, B)
    head_dim = hidden // heads
    # the new token of each request takes the last slot of its suffix list: its K/V rows are
    # overwritten by the layer's own append
    dec = make_decode_case("C5", 4, torch.float16, groups, branches, prefix, s, heads, head_dim, pool_slots)

    def w(*shape):
        return (torch.randn(shape, generator=gen, dtype=torch.float32) * 0.02).to(torch.float16)

    weights = {
        "qkv_proj": w(3 * hidden, hidden),
        "o_proj": w(hidden, hidden),
        "gate_proj": w(ffn, hidden),
        "up_proj": w(ffn, hidden),
        "down_proj": w(hidden, ffn),
        "input_layernorm": torch.ones(hidden, dtype=torch.float16),
        "post_attention_layernorm": torch.ones(hidden, dtype=torch.float16),
    }
    x = _randn(gen, (B, hidden), torch.float16)
    positions = torch.tensor([prefix + n - 1 for n in s], dtype=torch.int64)
    new_slots = torch.stack([dec.used_slots[l[-1]] for l in dec.suffix_lists]).long()
    return LayerCase(dec, x, positions, new_slots, weights, 1e-6, 10000.0)


# --------------------------------------------------------------------------- #
# device placement
# --------------------------------------------------------------------------- #
def pool_to_device(rows_k: torch.Tensor, rows_v: torch.Tensor, used_slots: torch.Tensor, pool_slots: int, device,
                   extra_slots: int = 0):
    """Zero-filled [pool_slots, H, D] K and V pools with the compact rows scattered to their slots."""
    H, D = rows_k.shape[1:]
    kc = torch.zeros((pool_slots + extra_slots, H, D), dtype=rows_k.dtype, device=device)
    vc = torch.zeros_like(kc)
    n = rows_k.shape[0]
    idx = used_slots[:n].to(device)
    step = 1 << 16
    for i in range(0, n, step):  # bounded staging copies
        kc[idx[i : i + step]] = rows_k[i : i + step].to(device)
        vc[idx[i : i + step]] = rows_v[i : i + step].to(device)
    return kc, vc
