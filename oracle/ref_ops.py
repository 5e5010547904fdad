"""CPU oracle: restatement of the reference's attention hot path in plain PyTorch.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this module;
it is used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
bench.py as the checker, never as the thing shipped or measured as the product.

Every function restates a reference function (path:line relative to the
reference checkout) on the token-granular KV layout ``[slots, H, D]`` (the
reference's ``MemLayout.NORMAL``, parrot/engine/builtin/mem.py:43-56), which is
the blocked layouts with ``block_size == 1``: a block table is then a slot list
and a context length is its row count.

All arithmetic is fp32 on inputs that are already rounded to the tensor dtype.

Pinning status (what independent check fails if this file has a plausible bug):
  * ref_decode_attention        -- pinned: brute-force python loops on tiny
                                   inputs, torch SDPA (library routine).
  * ref_partial / ref_lse_merge -- pinned: merge(prefix, suffix) == one-shot
                                   softmax over prefix||suffix; split invariance.
  * ref_prefill_with_parent     -- pinned: brute force, SDPA with explicit mask
                                   (the mask of 3rdparty/vllm/tests/kernels/
                                   test_attention.py:127-130), q_len==1 reduces
                                   to decode, parent==0 reduces to causal.
  * ref_move_tokens/ref_kv_append -- pinned: python-loop copy, untouched rows.
  * ref_move_from_blocked_k / ref_move_from_blocked_v -- pinned: element-wise
                                   python loops over the flat cache buffer with the
                                   layout's offset formula; the permuted view that
                                   turns a blocked cache into token-granular rows;
                                   block_size 1 reduces to ref_move_tokens.
  * ref_rope_neox / ref_rotary_embedding -- pinned: HF rotate_half form
                                   (3rdparty/vllm/tests/kernels/test_pos_encoding.py:10-24),
                                   norm preservation, position 0 identity,
                                   inverse rotation.
  * ref_rms_norm                -- pinned: torch.nn.functional.rms_norm (library),
                                   unit-weight mean-square == 1, scale invariance.
The reference ships no stored golden vectors for any of these ops (its checks
are kernel-vs-in-file-formula), so the formula checks above are the pins.
"""
from __future__ import annotations

import math
from typing import List, Sequence, Tuple

import torch

LOG2E = 1.4426950408889634


def _f32(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32)


# --------------------------------------------------------------------------- #
# decode attention
# --------------------------------------------------------------------------- #
def ref_decode_attention(
    query: torch.Tensor,  # [B, H, D]
    key_cache: torch.Tensor,  # [slots, H, D]
    value_cache: torch.Tensor,  # [slots, H, D]
    slot_lists: Sequence[torch.Tensor],  # B index tensors
    scale: float | None = None,
) -> torch.Tensor:
    """One-shot softmax attention of each query over its own slot list.

    Follows ``paged_flash_attention_reference``
    (parrot/engine/builtin/kernels/shared_flash_decoding.py:382-404, twin at
    kernels/vllm/paged_attention.py:44-66) and
    ``ref_single_query_cached_kv_attention``
    (3rdparty/vllm/tests/kernels/test_attention.py:30-66) with block_size 1;
    scale defaults to ``head_size ** -0.5`` (models/llama.py:90).
    An empty slot list yields a zero row.
    """
    B, H, D = query.shape
    scale = D ** -0.5 if scale is None else scale
    out = torch.zeros((B, H, D), dtype=torch.float32)
    for i in range(B):
        slots = slot_lists[i].long()
        if slots.numel() == 0:
            continue
        k = _f32(key_cache[slots])  # [n, H, D]
        v = _f32(value_cache[slots])
        q = _f32(query[i]) * scale  # [H, D]
        p = torch.einsum("hd,nhd->hn", q, k)
        s = torch.softmax(p, dim=-1)
        out[i] = torch.einsum("hn,nhd->hd", s, v)
    return out.to(query.dtype)


def ref_partial(
    query: torch.Tensor,  # [B, H, D]
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_lists: Sequence[torch.Tensor],
    scale: float | None = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Partial attention in the exp2 domain: returns (O, m, l), all fp32.

    ``y = q.k * scale * log2(e)``; ``m = max_j y_j``; ``l = sum_j 2^(y_j-m)``;
    ``O = sum_j 2^(y_j-m) v_j / l``
    (shared_flash_decoding.py:98,118-133; the suffix kernel stores the same
    pair, csrc/attention/attention_prev_kernels.cu:147,223,332-337).
    An empty list yields ``m=-inf, l=0, O=0``.
    """
    B, H, D = query.shape
    scale = D ** -0.5 if scale is None else scale
    O = torch.zeros((B, H, D), dtype=torch.float32)
    m = torch.full((B, H), -math.inf, dtype=torch.float32)
    l = torch.zeros((B, H), dtype=torch.float32)
    for i in range(B):
        slots = slot_lists[i].long()
        if slots.numel() == 0:
            continue
        k = _f32(key_cache[slots])
        v = _f32(value_cache[slots])
        y = torch.einsum("hd,nhd->hn", _f32(query[i]), k) * (scale * LOG2E)
        mi = y.max(dim=-1).values
        p = torch.exp2(y - mi[:, None])
        li = p.sum(dim=-1)
        O[i] = torch.einsum("hn,nhd->hd", p, v) / li[:, None]
        m[i] = mi
        l[i] = li
    return O, m, l


def ref_lse_merge(
    a: Tuple[torch.Tensor, torch.Tensor, torch.Tensor],
    b: Tuple[torch.Tensor, torch.Tensor, torch.Tensor],
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Log-sum-exp merge of two partials (exp2 domain).

    ``M=max(m_a,m_b)``, ``L=2^(m_a-M) l_a + 2^(m_b-M) l_b``,
    ``O=(2^(m_a-M) l_a O_a + 2^(m_b-M) l_b O_b)/L``
    (csrc/attention/attention_post_kernels.cu:321-340; n-way form in
    shared_flash_decoding.py:181-199).  An empty side (m=-inf, l=0) passes the
    other side through; two empty sides give zeros.
    """
    Oa, ma, la = a
    Ob, mb, lb = b
    M = torch.maximum(ma, mb)
    Msafe = torch.where(torch.isinf(M), torch.zeros_like(M), M)
    wa = torch.exp2(ma - Msafe) * la
    wb = torch.exp2(mb - Msafe) * lb
    L = wa + wb
    Ls = torch.where(L > 0, L, torch.ones_like(L))
    O = (wa[..., None] * Oa + wb[..., None] * Ob) / Ls[..., None]
    return O, M, L


def ref_shared_prefix_decode(
    query: torch.Tensor,  # [B, H, D]
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    prefix_slots: torch.Tensor,  # [P] shared by all B queries
    suffix_slot_lists: Sequence[torch.Tensor],
    scale: float | None = None,
) -> torch.Tensor:
    """``flash_paged_attention`` (shared_flash_decoding.py:285-329): prefix
    phase over the shared slots, suffix phase per request, LSE merge."""
    B = query.shape[0]
    pre = ref_partial(query, key_cache, value_cache, [prefix_slots] * B, scale)
    suf = ref_partial(query, key_cache, value_cache, suffix_slot_lists, scale)
    O, _, _ = ref_lse_merge(pre, suf)
    return O.to(query.dtype)


# --------------------------------------------------------------------------- #
# prefill with parent context
# --------------------------------------------------------------------------- #
def ref_prefill_with_parent(
    query: torch.Tensor,  # [T, H, D] packed chunks
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    q_lens: Sequence[int],
    ctx_slot_lists: Sequence[torch.Tensor],  # per chunk: ALL context slots (ancestors || own)
    scale: float | None = None,
) -> torch.Tensor:
    """Block-diagonal, bottom-right-aligned causal attention.

    Chunk c has ``n_c`` packed queries and ``kv_c = len(ctx_slot_lists[c])``
    keys (``fill_slots`` = the whole context including ancestors, in order,
    parrot/engine/builtin/attn_func.py:532-535).  Query r may see key j iff
    ``j <= r + (kv_c - n_c)`` -- xformers'
    ``BlockDiagonalCausalFromBottomRightMask.from_seqlens(q_seqlen, kv_seqlen)``
    built at attn_func.py:541-546 and consumed at :666-674; the same mask is
    written out explicitly as ``triu(ones(q_len, ctx_len), diagonal=ctx_len -
    q_len + 1)`` in 3rdparty/vllm/tests/kernels/test_attention.py:127-130.
    """
    T, H, D = query.shape
    scale = D ** -0.5 if scale is None else scale
    out = torch.zeros((T, H, D), dtype=torch.float32)
    start = 0
    for n, slots in zip(q_lens, ctx_slot_lists):
        slots = slots.long()
        kv = slots.numel()
        assert kv >= n
        q = _f32(query[start : start + n]) * scale  # [n, H, D]
        k = _f32(key_cache[slots])
        v = _f32(value_cache[slots])
        att = torch.einsum("qhd,khd->hqk", q, k)
        r = torch.arange(n)[:, None]
        j = torch.arange(kv)[None, :]
        att = att.masked_fill(~(j <= r + (kv - n))[None], -math.inf)
        att = torch.softmax(att, dim=-1)
        out[start : start + n] = torch.einsum("hqk,khd->qhd", att, v)
        start += n
    assert start == T
    return out.to(query.dtype)


# --------------------------------------------------------------------------- #
# token move / KV append (bit copies)
# --------------------------------------------------------------------------- #
def ref_move_tokens(
    src_storage: torch.Tensor,
    dest_storage: torch.Tensor,
    src_indices: torch.Tensor,
    dest_indices: torch.Tensor,
) -> None:
    """``dest[dest_idx[i], :, :] = src[src_idx[i], :, :]`` in place
    (parrot/engine/builtin/kernels/tokens_moving.py:47-64).  Destination
    indices must be unique, as in the reference (no atomics there either)."""
    assert src_indices.shape == dest_indices.shape
    assert dest_storage.shape[1:] == src_storage.shape[1:]
    rows = src_storage.index_select(0, src_indices.long())
    dest_storage.index_copy_(0, dest_indices.long(), rows)


def ref_move_from_blocked_k(
    blocked_k_cache: torch.Tensor,  # [num_blocks, H, D/x, block_size, x]
    dest_storage: torch.Tensor,  # [rows, H, D]
    src_slot_indices: torch.Tensor,  # [n]
    dest_indices: torch.Tensor,  # [n]
) -> None:
    """``dest[dest_idx[i], h, c*x + e] = K[slot // bs, h, c, slot % bs, e]`` in place
    (parrot/engine/builtin/kernels/tokens_moving.py:135-160: ``block_id = src_index // block_size``,
    ``block_offset = src_index % block_size``, the head row viewed as ``[D/x, x]``, :177-181)."""
    assert src_slot_indices.shape == dest_indices.shape
    num_heads, cols, block_size, x = blocked_k_cache.shape[1:]
    assert dest_storage.shape[1] == num_heads and dest_storage.shape[2] == cols * x
    slots = src_slot_indices.long()
    blk = torch.div(slots, block_size, rounding_mode="floor")
    off = slots - blk * block_size
    rows = blocked_k_cache[blk, :, :, off, :]  # [n, H, D/x, x]
    dest_storage.index_copy_(0, dest_indices.long(), rows.reshape(rows.shape[0], num_heads, cols * x))


def ref_move_from_blocked_v(
    blocked_v_cache: torch.Tensor,  # [num_blocks, H, D, block_size]
    dest_storage: torch.Tensor,  # [rows, H, D]
    src_slot_indices: torch.Tensor,
    dest_indices: torch.Tensor,
) -> None:
    """``dest[dest_idx[i], h, d] = V[slot // bs, h, d, slot % bs]`` in place
    (parrot/engine/builtin/kernels/tokens_moving.py:248-270)."""
    assert src_slot_indices.shape == dest_indices.shape
    block_size = blocked_v_cache.shape[3]
    assert dest_storage.shape[1:] == blocked_v_cache.shape[1:3]
    slots = src_slot_indices.long()
    blk = torch.div(slots, block_size, rounding_mode="floor")
    off = slots - blk * block_size
    dest_storage.index_copy_(0, dest_indices.long(), blocked_v_cache[blk, :, :, off])


def ref_kv_append(
    key: torch.Tensor,  # [T, H, D] (row stride free)
    value: torch.Tensor,
    key_cache: torch.Tensor,  # [slots, H, D]
    value_cache: torch.Tensor,
    slot_mapping: torch.Tensor,  # [T]
) -> None:
    """``K[slot[t]] = k[t]``, ``V[slot[t]] = v[t]``
    (3rdparty/vllm/csrc/cache_kernels.cu:155-180 with block_size 1; twin:
    attn_func.py:143-155 via discontinuous_move_tokens with src=arange)."""
    idx = slot_mapping.long()
    key_cache.index_copy_(0, idx, key.contiguous())
    value_cache.index_copy_(0, idx, value.contiguous())


# --------------------------------------------------------------------------- #
# RoPE
# --------------------------------------------------------------------------- #
def ref_cos_sin_cache(max_seq_len: int, rotary_dim: int, theta: float, dtype: torch.dtype) -> torch.Tensor:
    """``cat(cos(freqs), sin(freqs))`` of shape [max_seq_len, rotary_dim],
    computed in fp32 then cast (parrot/engine/builtin/mem.py:125-143)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2).float() / rotary_dim))
    t = torch.arange(max_seq_len, dtype=inv_freq.dtype)
    freqs = torch.outer(t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(dtype)


def ref_rotary_embedding(state: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, elem_rounding: bool = False) -> torch.Tensor:
    """NeoX rotation with per-token cos/sin ``[T, 1, D/2]``; returns the rotated
    copy: ``x' = x cos - y sin``, ``y' = x sin + y cos`` with x / y the first /
    second half of D (``torch_rotary_embedding``,
    parrot/engine/builtin/kernels/rotary_embedding.py:146-152).

    ``elem_rounding=True`` restates the CUDA kernel's arithmetic, where every
    product and the sum are rounded to the element type
    (3rdparty/vllm/csrc/pos_encoding_kernels.cu:36-42); otherwise fp32 math and
    one final rounding.
    """
    D = state.shape[-1]
    dt = state.dtype
    if elem_rounding:
        x, y = state[..., : D // 2], state[..., D // 2 :]
        c, s = cos.to(dt), sin.to(dt)
        ox = (x * c).to(dt) - (y * s).to(dt)
        oy = (y * c).to(dt) + (x * s).to(dt)
        return torch.cat((ox.to(dt), oy.to(dt)), dim=-1)
    x, y = _f32(state[..., : D // 2]), _f32(state[..., D // 2 :])
    c, s = _f32(cos), _f32(sin)
    return torch.cat((x * c - y * s, x * s + y * c), dim=-1).to(dt)


def ref_rope_neox(
    positions: torch.Tensor,  # [T] int64
    query: torch.Tensor,  # [T, Hq*D] or [T, Hq, D]
    key: torch.Tensor,
    cos_sin_cache: torch.Tensor,  # [max_pos, rot_dim]
    head_size: int,
    elem_rounding: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``rotary_embedding_neox(positions, q, k, head_size, cos_sin_cache)``
    (3rdparty/vllm/csrc/pos_encoding_kernels.cu:6-104 via
    parrot/engine/builtin/kernels/vllm/rotary_embed.py:10-25): cos/sin rows are
    looked up by position; the first ``rot_dim`` dims of every head rotate.
    Returns rotated copies (the reference mutates in place)."""
    rot = cos_sin_cache.shape[-1]
    T = positions.shape[0]
    cs = cos_sin_cache[positions.long()]  # [T, rot]
    cos = cs[:, None, : rot // 2]
    sin = cs[:, None, rot // 2 :]
    outs = []
    for t in (query, key):
        shp = t.shape
        h = t.reshape(T, -1, head_size)
        rotated = ref_rotary_embedding(h[..., :rot], cos, sin, elem_rounding)
        outs.append(torch.cat((rotated, h[..., rot:]), dim=-1).reshape(shp))
    return outs[0], outs[1]


# --------------------------------------------------------------------------- #
# RMSNorm
# --------------------------------------------------------------------------- #
def ref_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, round_before_weight: bool = True) -> torch.Tensor:
    """``y = w * t(x * rsqrt(mean(x^2) + eps))``.

    ``round_before_weight=True`` is the CUDA kernel's order: the normalised
    value is rounded to the element type, then multiplied by the weight in the
    element type (3rdparty/vllm/csrc/layernorm_kernels.cu:24-33, ``RefRMSNorm``
    in 3rdparty/vllm/tests/kernels/test_layernorm.py:7-23).  False is the
    Triton twin: all fp32, one rounding
    (parrot/engine/builtin/kernels/rms_norm.py:15-46, ``torch_rms_norm`` :81-82).
    """
    dt = x.dtype
    xf = _f32(x)
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if round_before_weight:
        return ((xf * rstd).to(dt) * weight.to(dt)).to(dt)
    return (xf * rstd * _f32(weight)).to(dt)


# --------------------------------------------------------------------------- #
# fused per-layer ops (compositions of the above, kept as the unfused sequences)
# --------------------------------------------------------------------------- #
def ref_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                     round_before_weight: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """``h = residual + x`` as a tensor of the element type (the torch add of
    parrot/engine/builtin/models/llama.py:160-178), then ``ref_rms_norm(h)``.
    Returns ``(y, h)``: the norm runs on the rounded, stored ``h``."""
    h = (_f32(residual) + _f32(x)).to(x.dtype)
    return ref_rms_norm(h, weight, eps, round_before_weight), h


def ref_silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``t(t(g / (1 + exp(-g))) * u)``: silu in fp32 rounded to the element type, then the product rounded
    (3rdparty/vllm/csrc/activation_kernels.cu:6-24; the same two roundings as ``act_fn(gate) * up`` of the
    Hugging Face LlamaMLP the reference imports, parrot/engine/builtin/models/llama.py:36-39)."""
    dt = gate.dtype
    g = _f32(gate)
    s = (g / (1.0 + torch.exp(-g))).to(dt)
    return (_f32(s) * _f32(up)).to(dt)
