"""Kernel surface of Parrot's builtin engine, backed by libparrot_hip.so.

Same names, argument order and in-place behaviour as
``parrot/engine/builtin/kernels/__init__.py:7-16`` of the reference, on the
token-granular KV layout ``[slots, H, D]`` (``MemLayout.NORMAL`` with
``block_size == 1``, parrot/engine/builtin/mem.py:43-56): a block table is a
list of slot ids and a context length is its row count.

Every function launches hand-written HIP kernels through the C ABI on the
current torch stream.  torch is used for device memory and streams only; there
is no PyTorch fallback.
"""
from __future__ import annotations

import collections
import ctypes
import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from ._lib import PH_BF16, PH_F16, PH_IDX_I32, PH_IDX_I64, check

__all__ = [
    "discontinuous_move_tokens",
    "move_tokens_from_blocked_k_cache",
    "move_tokens_from_blocked_v_cache",
    "rotary_embedding",
    "rmsnorm_forward",
    "vllm_paged_attention",
    "vllm_reshape_and_cache",
    "vllm_rms_norm",
    "vllm_rotary_emb",
    "flash_paged_attention",
    "paged_flash_attention",
    "DecodeTables",
    "PrefillTables",
    "decode_attention",
    "decode_attention_static",
    "prefill_attention",
    "kv_append",
]


# --------------------------------------------------------------------------- #
# plumbing
# --------------------------------------------------------------------------- #
def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return PH_F16
    if t.dtype == torch.bfloat16:
        return PH_BF16
    if t.dtype == torch.float32:
        return _lib.PH_F32
    # TORCH_CHECK(false, "Unsupported data type") in the reference's launcher
    raise RuntimeError(f"Unsupported data type: {t.dtype}")


def _index_code(t: torch.Tensor) -> int:
    if t.dtype == torch.int32:
        return PH_IDX_I32
    if t.dtype == torch.int64:
        return PH_IDX_I64
    raise ValueError(f"index tensor must be int32 or int64, got {t.dtype}")


def _require_gpu(*ts: torch.Tensor) -> torch.device:
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("parrotserve_amd kernels run on the GPU only; got a CPU tensor (no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError("all tensors must live on the same device")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of torch's current stream on the current device (the raw getter costs a fraction of a
    microsecond; building a torch.cuda.Stream object per launch costs several)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}
_captured_keys: set = set()               # (device, stream) whose current buffer a captured graph points at
_pinned_workspaces: List[torch.Tensor] = []  # outgrown buffers that recorded graphs still use


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """Grow-only scratch buffer per (device, stream); reuse is ordered by the stream.

    A buffer handed out while the stream is being captured into a graph is recorded by address in that graph, so
    it is pinned for the life of the process: growing never frees it (an eager call that needs more gets a new
    buffer, the recorded graph keeps the old one), and a request made under capture that does not fit the
    stream's buffer is refused instead of allocating inside the capture."""
    key = (device.index or 0, _stream())
    buf = _workspaces.get(key)
    capturing = torch.cuda.is_current_stream_capturing()
    if buf is None or buf.numel() < nbytes:
        if capturing and buf is not None:
            raise RuntimeError(
                f"decode workspace of {buf.numel()} bytes is too small for {nbytes} bytes and the stream is being "
                "captured: run the step once eagerly at its largest shape before capturing it")
        if buf is not None and key in _captured_keys:
            _pinned_workspaces.append(buf)  # a recorded graph still points at it
            _captured_keys.discard(key)
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    if capturing:
        _captured_keys.add(key)
    return buf


# --------------------------------------------------------------------------- #
# token move / KV append
# --------------------------------------------------------------------------- #
def discontinuous_move_tokens(src_storage, dest_storage, src_indices, dest_indices):
    """``dest_storage[dest_indices[i]] = src_storage[src_indices[i]]``
    (parrot/engine/builtin/kernels/tokens_moving.py:67-100).  Storages are
    ``[tokens, H, D]`` with free strides; indices are int64 or int32 ``[n]``."""
    assert src_indices.shape == dest_indices.shape, "src_indices and dest_indices must have the same shape"
    assert dest_storage.shape[1:] == src_storage.shape[1:], "storage shape mismatch"
    assert src_storage.dtype == dest_storage.dtype, "storage dtype mismatch"
    assert src_indices.dtype == dest_indices.dtype, "index dtype mismatch"
    _require_gpu(src_storage, dest_storage, src_indices, dest_indices)
    src_indices = src_indices.contiguous()
    dest_indices = dest_indices.contiguous()
    n = src_indices.shape[0]
    num_heads, head_dim = src_storage.shape[1:]
    rc = _lib.load().ph_move_tokens(
        _ptr(src_storage), _ptr(dest_storage), _ptr(src_indices), _ptr(dest_indices), _index_code(src_indices),
        n, num_heads, head_dim, src_storage.element_size(),
        src_storage.stride(0), src_storage.stride(1), src_storage.stride(2),
        dest_storage.stride(0), dest_storage.stride(1), dest_storage.stride(2), _stream())
    check(rc, "discontinuous_move_tokens")


def _gather_checks(cache, dest_storage, src_slot_indices, dest_indices):
    assert src_slot_indices.shape == dest_indices.shape, "src_indices and dest_indices must have the same shape"
    assert dest_storage.shape[0] >= dest_indices.shape[0], "dest_storage is too small"
    assert cache.dtype == dest_storage.dtype, "storage dtype mismatch"
    assert src_slot_indices.dtype == dest_indices.dtype, "index dtype mismatch"
    _require_gpu(cache, dest_storage, src_slot_indices, dest_indices)


def move_tokens_from_blocked_k_cache(blocked_k_cache, dest_storage, src_slot_indices, dest_indices):
    """Gather token rows of a blocked K cache ``[num_blocks, H, D/x, block_size, x]`` by slot id
    (``slot = block * block_size + offset``) into ``dest_storage [n, H, D]``
    (parrot/engine/builtin/kernels/tokens_moving.py:104-218).  A 3-d cache is the token-granular layout
    ``[slots, H, D]`` (the blocked layout at ``block_size == 1``) and takes the plain token move."""
    if blocked_k_cache.dim() == 3:
        return discontinuous_move_tokens(blocked_k_cache, dest_storage, src_slot_indices, dest_indices)
    if blocked_k_cache.dim() != 5:
        raise ValueError(f"move_tokens_from_blocked_k_cache: expected a 5-d or 3-d cache, got {blocked_k_cache.dim()}-d")
    _gather_checks(blocked_k_cache, dest_storage, src_slot_indices, dest_indices)
    num_heads, cols, block_size, x = blocked_k_cache.shape[1:]
    assert dest_storage.dim() == 3 and dest_storage.shape[1] == num_heads and dest_storage.shape[2] == cols * x, \
        "storage shape mismatch"
    src_slot_indices = src_slot_indices.contiguous()
    dest_indices = dest_indices.contiguous()
    c = blocked_k_cache
    rc = _lib.load().ph_gather_blocked_k(
        _ptr(c), _ptr(dest_storage), _ptr(src_slot_indices), _ptr(dest_indices), _index_code(src_slot_indices),
        src_slot_indices.shape[0], num_heads, cols * x, block_size, x, c.element_size(),
        c.stride(0), c.stride(1), c.stride(2), c.stride(3), c.stride(4),
        dest_storage.stride(0), dest_storage.stride(1), dest_storage.stride(2), _stream())
    check(rc, "move_tokens_from_blocked_k_cache")


def move_tokens_from_blocked_v_cache(blocked_v_cache, dest_storage, src_slot_indices, dest_indices):
    """V twin of the above for ``[num_blocks, H, D, block_size]`` (tokens_moving.py:222-313)."""
    if blocked_v_cache.dim() == 3:
        return discontinuous_move_tokens(blocked_v_cache, dest_storage, src_slot_indices, dest_indices)
    if blocked_v_cache.dim() != 4:
        raise ValueError(f"move_tokens_from_blocked_v_cache: expected a 4-d or 3-d cache, got {blocked_v_cache.dim()}-d")
    _gather_checks(blocked_v_cache, dest_storage, src_slot_indices, dest_indices)
    num_heads, head_dim, block_size = blocked_v_cache.shape[1:]
    assert tuple(dest_storage.shape[1:]) == (num_heads, head_dim), "storage shape mismatch"
    src_slot_indices = src_slot_indices.contiguous()
    dest_indices = dest_indices.contiguous()
    c = blocked_v_cache
    rc = _lib.load().ph_gather_blocked_v(
        _ptr(c), _ptr(dest_storage), _ptr(src_slot_indices), _ptr(dest_indices), _index_code(src_slot_indices),
        src_slot_indices.shape[0], num_heads, head_dim, block_size, c.element_size(),
        c.stride(0), c.stride(1), c.stride(2), c.stride(3),
        dest_storage.stride(0), dest_storage.stride(1), dest_storage.stride(2), _stream())
    check(rc, "move_tokens_from_blocked_v_cache")


def kv_append(key, value, key_cache, value_cache, slot_mapping):
    """``key_cache[slot[t]] = key[t]`` and the same for V, one launch."""
    assert key.shape == value.shape and key.dim() == 3
    assert key_cache.shape == value_cache.shape and key_cache.dim() == 3
    assert key.shape[1:] == key_cache.shape[1:], "head shape mismatch"
    assert key.dtype == value.dtype == key_cache.dtype == value_cache.dtype
    _require_gpu(key, value, key_cache, value_cache, slot_mapping)
    slot_mapping = slot_mapping.reshape(-1).contiguous()
    T, H, D = key.shape
    assert slot_mapping.shape[0] == T, "slot_mapping must hold one slot per token"
    for t in (key, value, key_cache, value_cache):
        assert t.stride(2) == 1 and t.stride(1) == D, "heads of a token must be contiguous"
    assert key_cache.stride(0) == value_cache.stride(0)
    rc = _lib.load().ph_kv_append(
        _ptr(key), _ptr(value), _ptr(key_cache), _ptr(value_cache), _ptr(slot_mapping), _index_code(slot_mapping),
        T, H, D, _dtype_code(key), key.stride(0), value.stride(0), key_cache.stride(0), _stream())
    check(rc, "kv_append")


def vllm_reshape_and_cache(key_to_cache, value_to_cache, key_cache, value_cache, slot_mapping):
    """``cache_ops.reshape_and_cache`` on the token-granular layout
    (parrot/engine/builtin/kernels/vllm/reshape_and_cache.py:9-22)."""
    kv_append(key_to_cache, value_to_cache, key_cache, value_cache, slot_mapping)


# --------------------------------------------------------------------------- #
# RMSNorm / RoPE
# --------------------------------------------------------------------------- #
def _rms(x, weight, eps, round_first, name):
    _require_gpu(x, weight)
    assert x.shape[-1] == weight.shape[0], "weight size mismatch"
    assert x.dtype == weight.dtype, "weight dtype mismatch"
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    out = torch.empty((x2.shape[0], x2.shape[1]), dtype=x.dtype, device=x.device)
    rc = _lib.load().ph_rms_norm(_ptr(out), _ptr(x2), _ptr(weight.contiguous()), float(eps), x2.shape[0], x2.shape[1],
                                 x2.stride(0), out.stride(0), _dtype_code(x), int(round_first), _stream())
    check(rc, name)
    return out.view(x.shape)


def vllm_rms_norm(input, weight, eps):
    """``layernorm_ops.rms_norm`` (parrot/engine/builtin/kernels/vllm/rms_norm.py:9-16):
    the normalised value is rounded to the element type before the weight multiply."""
    return _rms(input, weight, eps, True, "vllm_rms_norm")


def rmsnorm_forward(x, weight, eps):
    """Triton twin (parrot/engine/builtin/kernels/rms_norm.py:49-78): fp32 math, one rounding."""
    return _rms(x, weight, eps, False, "rmsnorm_forward")


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                       round_before_weight: bool = True) -> torch.Tensor:
    """``residual += x`` in place, returns ``RMSNorm(residual) * weight`` (one launch for the residual add of
    the decoder layer and the norm that follows it)."""
    _require_gpu(x, residual, weight)
    n = x.shape[-1]
    assert x.shape == residual.shape and weight.shape == (n,) and x.dtype == residual.dtype == weight.dtype
    x2, r2 = x.reshape(-1, n), residual.view(-1, n)
    assert x2.stride(1) == 1 and r2.stride(1) == 1
    out = torch.empty(x2.shape, dtype=x.dtype, device=x.device)
    check(_lib.load().ph_add_rms_norm(_ptr(out), _ptr(r2), _ptr(x2), _ptr(weight), float(eps), x2.shape[0], n,
                                      x2.stride(0), r2.stride(0), out.stride(0), _dtype_code(x),
                                      1 if round_before_weight else 0, _stream()), "fused_add_rms_norm")
    return out.view(x.shape)


def silu_mul(gate: torch.Tensor, up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` in one launch; ``gate`` / ``up`` may be column slices of one fused projection."""
    _require_gpu(gate, up)
    d = gate.shape[-1]
    assert gate.shape == up.shape and gate.dtype == up.dtype
    g2 = gate if gate.dim() == 2 else gate.reshape(-1, d)
    u2 = up if up.dim() == 2 else up.reshape(-1, d)
    assert g2.stride(1) == 1 and u2.stride(1) == 1
    if out is None:
        out = torch.empty(g2.shape, dtype=gate.dtype, device=gate.device)
    o2 = out.view(-1, d)
    check(_lib.load().ph_silu_mul(_ptr(o2), _ptr(g2), _ptr(u2), g2.shape[0], d, g2.stride(0), u2.stride(0),
                                  o2.stride(0), _dtype_code(gate), _stream()), "silu_mul")
    return out.view(gate.shape)


def sample_top_p(logits: torch.Tensor, temperature: Optional[torch.Tensor], top_p: Optional[torch.Tensor],
                 uniform: torch.Tensor) -> torch.Tensor:
    """Temperature, top-p filter and one draw per row of ``logits [B, V]`` (fp16, bf16 or fp32) in one launch: the
    body of the reference's ``Sampler.forward`` after the logits GEMM (models/sampler.py:33-64), with the filter
    found by bisection instead of two sorts and the draw taken from ``uniform [B]`` (float32 in [0, 1), from the
    caller's generator) by inverse CDF over ascending token ids.  ``temperature`` / ``top_p``: float32 ``[B]`` on the
    device, or ``None`` for 1.  Returns int64 ``[B]``."""
    _require_gpu(logits, temperature, top_p, uniform)
    assert logits.dim() == 2 and logits.stride(1) == 1
    B, V = logits.shape
    if logits.dtype == torch.float32:
        code = _lib.PH_F32
    else:
        code = _dtype_code(logits)
    for name, v in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
        if v is not None and (v.dtype != torch.float32 or v.numel() != B or not v.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous float32 tensor of {B} elements")
    out = torch.empty(B, dtype=torch.int64, device=logits.device)
    check(_lib.load().ph_sample_top_p(_ptr(logits), logits.stride(0) if B > 1 else max(logits.stride(0), V),
                                      _ptr(temperature) if temperature is not None else None,
                                      _ptr(top_p) if top_p is not None else None, _ptr(uniform), _ptr(out), B, V, code,
                                      _stream()), "sample_top_p")
    return out


def top_p_probs(logits: torch.Tensor, temperature: Optional[torch.Tensor], top_p: Optional[torch.Tensor]) -> torch.Tensor:
    """The distribution the reference's sampler draws from (models/sampler.py:33-64 up to the ``torch.multinomial``
    call): temperature in the element type, top-p filter, soft-max of the survivors in fp32; dropped tokens get 0.
    ``torch.multinomial(top_p_probs(...), 1, replacement=True)`` is then the reference's own draw."""
    _require_gpu(logits, temperature, top_p)
    assert logits.dim() == 2 and logits.stride(1) == 1
    B, V = logits.shape
    code = _dtype_code(logits)
    for name, v in (("temperature", temperature), ("top_p", top_p)):
        if v is not None and (v.dtype != torch.float32 or v.numel() != B or not v.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous float32 tensor of {B} elements")
    probs = torch.empty((B, V), dtype=torch.float32, device=logits.device)
    check(_lib.load().ph_top_p_probs(_ptr(logits), logits.stride(0) if B > 1 else max(logits.stride(0), V),
                                     _ptr(temperature), _ptr(top_p), _ptr(probs), probs.stride(0), B, V, code,
                                     _stream()), "top_p_probs")
    return probs


def silu_and_mul(out: torch.Tensor, input: torch.Tensor) -> None:
    """vLLM's form (3rdparty/vllm/csrc/activation.cpp:3-6): ``input`` is ``[T, 2d]`` = gate | up."""
    d = input.shape[-1] // 2
    silu_mul(input[..., :d], input[..., d:], out=out)


def rope_and_cache(positions, query, key, value, cos_sin_cache, head_size, key_cache, value_cache, slot_mapping,
                   key_in_place=True):
    """``vllm_rotary_emb(positions, query, key, ...)`` followed by ``vllm_reshape_and_cache(key, value, ...)``
    in one launch: q and k rotated in place, rotated k rows and v rows written to their slots.
    ``key_in_place=False``: the caller reads K from the cache from here on, so ``key`` is not written back
    (its contents afterwards are unspecified) and the pass is a quarter shorter."""
    _require_gpu(query, key, value, key_cache, value_cache, cos_sin_cache, positions, slot_mapping)
    assert positions.dtype == torch.int64 and positions.dim() == 1
    T = positions.shape[0]
    q2, k2, v2 = query.view(T, -1) if query.dim() == 3 else query, key.view(T, -1) if key.dim() == 3 else key, \
        value.view(T, -1) if value.dim() == 3 else value
    assert q2.stride(1) == 1 and k2.stride(1) == 1 and v2.stride(1) == 1
    hq, hk = q2.shape[1] // head_size, k2.shape[1] // head_size
    assert v2.shape[1] == hk * head_size and key_cache.shape[1:] == (hk, head_size)
    assert key_cache.stride() == value_cache.stride() and key_cache.stride(2) == 1 and key_cache.stride(1) == head_size
    assert query.dtype == key.dtype == value.dtype == key_cache.dtype == cos_sin_cache.dtype
    assert slot_mapping.numel() == T and cos_sin_cache.is_contiguous()
    check(_lib.load().ph_rope_append(_ptr(positions), _ptr(q2), _ptr(k2), _ptr(v2), _ptr(cos_sin_cache),
                                     _ptr(key_cache), _ptr(value_cache), _ptr(slot_mapping), _index_code(slot_mapping),
                                     T, hq, hk, head_size, cos_sin_cache.shape[-1], q2.stride(0), k2.stride(0),
                                     v2.stride(0), key_cache.stride(0), _dtype_code(query), 1 if key_in_place else 0,
                                     _stream()),
          "rope_and_cache")


def vllm_rotary_emb(positions, query, key, cos_sin_cache, head_size):
    """NeoX rotary embedding of ``query`` and ``key`` in place
    (parrot/engine/builtin/kernels/vllm/rotary_embed.py:10-25).  query / key are
    ``[T, heads*head_size]`` and may be row-strided chunk views of a fused qkv."""
    _require_gpu(positions, query, key, cos_sin_cache)
    assert positions.dtype == torch.int64, "positions must be int64"
    assert query.dim() == 2 and key.dim() == 2 and query.stride(1) == 1 and key.stride(1) == 1
    assert query.dtype == key.dtype == cos_sin_cache.dtype
    T = positions.shape[0]
    assert query.shape[0] == T and key.shape[0] == T
    assert cos_sin_cache.is_contiguous()
    rc = _lib.load().ph_rope_neox(
        _ptr(positions.contiguous()), _ptr(query), _ptr(key), _ptr(cos_sin_cache), T,
        query.shape[1] // head_size, key.shape[1] // head_size, head_size, cos_sin_cache.shape[1],
        query.stride(0), key.stride(0), _dtype_code(query), _stream())
    check(rc, "vllm_rotary_emb")


def rotary_embedding(state, cos, sin):
    """In-place NeoX rotation of ``state [T, H, D]`` with per-token ``cos``,
    ``sin`` of shape ``[T, 1, D/2]`` (parrot/engine/builtin/kernels/rotary_embedding.py:107-143)."""
    _require_gpu(state, cos, sin)
    assert state.dim() == 3 and state.stride(2) == 1
    T, H, D = state.shape
    assert cos.shape == sin.shape == (T, 1, D // 2), "cos/sin must be [T, 1, D/2]"
    assert cos.dtype == sin.dtype == state.dtype
    assert cos.stride(2) == 1 and sin.stride(2) == 1 and cos.stride(0) == sin.stride(0)
    rc = _lib.load().ph_rotary_embedding(_ptr(state), _ptr(cos), _ptr(sin), T, H, D, state.stride(0), state.stride(1),
                                         cos.stride(0), _dtype_code(state), _stream())
    check(rc, "rotary_embedding")


# --------------------------------------------------------------------------- #
# decode attention
# --------------------------------------------------------------------------- #
@dataclasses.dataclass
class DecodeTables:
    """Per-iteration slot tables of the decode requests (built once, used by
    every layer).  Device tensors are int32 unless noted."""

    num_reqs: int
    # prefix groups
    num_groups: int = 0
    prefix_slots: Optional[torch.Tensor] = None  # all groups back to back
    prefix_cu: Optional[torch.Tensor] = None  # [G+1] device
    group_req_cu: Optional[torch.Tensor] = None  # [G+1] device
    group_req_cu_host: Optional[torch.Tensor] = None  # [G+1] CPU int32
    max_prefix_len: int = 0
    # per-request suffix
    suffix_slots: Optional[torch.Tensor] = None  # ragged (with offsets) or [B, max] padded
    suffix_offsets: Optional[torch.Tensor] = None  # int64 [B] device, None for a padded table
    suffix_table_stride: int = 0
    suffix_lens: Optional[torch.Tensor] = None  # [B] device
    max_suffix_len: int = 0
    chunk_tokens: int = 0  # 0 = let the library choose
    # balanced suffix plan (needs the lengths on the host): device int32 arrays + the host struct
    plan_buffer: Optional[torch.Tensor] = None  # the three arrays below, back to back
    plan_items: Optional[torch.Tensor] = None  # [lanes + B, 4], the first rows in use
    plan_lane_item_cu: Optional[torch.Tensor] = None  # lane records [num_lanes, 8]
    plan_req_item_cu: Optional[torch.Tensor] = None  # [B + 1]
    plan: Optional[_lib.SuffixPlan] = None

    def suffix_slots_count(self) -> int:
        """Entries readable behind ``suffix_slots`` (bound for the kernel's early slot fetch)."""
        if self.suffix_slots is None:
            return 0
        if self.suffix_offsets is None:
            return (self.num_reqs - 1) * self.suffix_table_stride + self.suffix_slots.shape[-1]
        return self.suffix_slots.numel()

    def set_plan(self, lens: Sequence[int], num_lanes: int, device) -> None:
        """Cut the batch's suffix token stream into ``num_lanes`` near-equal pieces (see ph_suffix_plan).

        The device arrays have a fixed layout for a given (lanes, batch) -- the item array is sized for the most
        items a cut can produce, lanes + batch -- and are rewritten in place when the lengths change, so the
        plan's pointers and counts (and with them the workspace layout) stay what a captured graph recorded."""
        items, lane_cu, req_cu = plan_suffix_items(lens, num_lanes)
        if items.shape[0] == 0:
            return
        lanes = lane_cu.shape[0] - 1
        n_items = items.shape[0]
        cap = lanes + req_cu.shape[0] - 1
        # one host buffer, one upload: items | lane records | per-request item offsets
        o_rec = cap * 4
        o_cu = o_rec + lanes * 8
        buf = np.zeros(o_cu + req_cu.shape[0], dtype=np.int32)
        buf[: n_items * 4] = items.reshape(-1)
        rec = buf[o_rec:o_cu].reshape(lanes, 8)
        rec[:, 0] = lane_cu[:-1]
        rec[:, 1] = lane_cu[1:] - lane_cu[:-1]
        first = np.minimum(lane_cu[:-1], n_items - 1)
        rec[:, 2:5] = items[first, 0:3]
        buf[o_cu:] = req_cu
        old = self.plan_buffer
        if old is not None and old.numel() == buf.shape[0] and old.device == torch.device(device) and \
                self.plan is not None and self.plan.num_lanes == lanes:
            old.copy_(torch.from_numpy(buf))  # ordered on the current stream behind the kernels still reading it
            return
        dev_buf = torch.from_numpy(buf).to(device)
        self.plan_buffer = dev_buf
        self.plan_items = dev_buf[:o_rec].view(cap, 4)
        self.plan_lane_item_cu = dev_buf[o_rec:o_cu].view(lanes, 8)
        self.plan_req_item_cu = dev_buf[o_cu:]
        self.plan = _lib.SuffixPlan(self.plan_items.data_ptr(), cap, self.plan_lane_item_cu.data_ptr(),
                                    lanes, self.plan_req_item_cu.data_ptr())

    def plan_on_device(self, num_lanes: int, device) -> None:
        """The balanced plan written by the library from the device length vector (``ph_suffix_plan_build``): no
        host-side list work, no upload.  ``num_lanes`` is the lane capacity (``suffix_lane_capacity``); the planner
        uses as many of them as the token count warrants.  The arrays keep their place from call to call."""
        B = self.num_reqs
        cap = num_lanes + B
        o_rec = cap * 4
        o_cu = o_rec + num_lanes * 8
        n = o_cu + B + 1
        buf = self.plan_buffer
        if buf is None or buf.numel() != n or self.plan is None or self.plan.num_lanes != num_lanes or \
                self.plan.num_items != cap:
            buf = torch.zeros(n, dtype=torch.int32, device=device)
            self.plan_buffer = buf
            self.plan_items = buf[:o_rec].view(cap, 4)
            self.plan_lane_item_cu = buf[o_rec:o_cu].view(num_lanes, 8)
            self.plan_req_item_cu = buf[o_cu:]
            self.plan = _lib.SuffixPlan(self.plan_items.data_ptr(), cap, self.plan_lane_item_cu.data_ptr(),
                                        num_lanes, self.plan_req_item_cu.data_ptr())
        suffix_plan_build(self.suffix_lens, num_lanes, self.plan_items, self.plan_lane_item_cu, self.plan_req_item_cu,
                          max_len=self.max_suffix_len)

    @staticmethod
    def build(prefix_lists: Sequence[Sequence[int]], group_req_cu: Sequence[int],
              suffix_lists: Sequence[Sequence[int]], device, num_heads: int = 32, head_dim: int = 128,
              balanced: bool = True, dtype: torch.dtype = torch.float16, kv_group: int = 1) -> "DecodeTables":
        """From python lists: ``prefix_lists[g]`` is group g's slot list shared by
        requests ``group_req_cu[g] .. group_req_cu[g+1]-1``; ``suffix_lists[b]`` is
        request b's own slot list.  ``balanced`` adds the item list of the
        suffix phase, cut for ``num_heads x head_dim`` heads of ``dtype`` elements (``kv_group = G``: for calls
        whose query heads share KV heads as ``h // G``)."""
        B = len(suffix_lists)
        t = DecodeTables(num_reqs=B)
        G = len(prefix_lists)
        if G > 0:
            assert len(group_req_cu) == G + 1
            cu = [0]
            flat: List[int] = []
            for p in prefix_lists:
                flat.extend(p)
                cu.append(len(flat))
            t.num_groups = G
            t.max_prefix_len = max(len(p) for p in prefix_lists)
            t.prefix_slots = torch.from_numpy(np.asarray(flat if flat else [0], dtype=np.int32)).to(device)
            t.prefix_cu = torch.tensor(cu, dtype=torch.int32, device=device)
            t.group_req_cu_host = torch.tensor(list(group_req_cu), dtype=torch.int32)
            t.group_req_cu = t.group_req_cu_host.to(device)
        lens = [len(s) for s in suffix_lists]
        t.max_suffix_len = max(lens) if lens else 0
        total = sum(lens)
        if t.max_suffix_len > 0:
            # padded [B, max] table: a request's list start needs no lookup, so the kernel can fetch
            # slot ids and the length at the same time
            width = (t.max_suffix_len + 15) // 16 * 16
            # one conversion of all lists back to back, then a scatter into the padded rows
            flat_suffix: List[int] = []
            for sl in suffix_lists:
                flat_suffix.extend(sl)
            lens_a = np.asarray(lens, dtype=np.int64)
            starts = np.zeros(B, dtype=np.int64)
            np.cumsum(lens_a[:-1], out=starts[1:])
            pos = np.arange(total, dtype=np.int64) - np.repeat(starts, lens_a)
            table = np.zeros((B, width), dtype=np.int32)
            table[np.repeat(np.arange(B, dtype=np.int64), lens_a), pos] = np.asarray(flat_suffix, dtype=np.int32)
            t.suffix_slots = torch.from_numpy(table).to(device)
            t.suffix_offsets = None
            t.suffix_table_stride = width
            t.suffix_lens = torch.tensor(lens, dtype=torch.int32, device=device)
            # parts of about 1/2048 of the batch's tokens, 32 .. 1024 tokens each
            chunk = 32
            while chunk < total // 2048 and chunk < 1024:
                chunk *= 2
            t.chunk_tokens = chunk
            if balanced:
                shape = dict(num_reqs=B, num_groups=t.num_groups, max_prefix_len=t.max_prefix_len,
                             max_suffix_len=t.max_suffix_len, dtype=dtype, kv_group=kv_group)
                if B <= PLAN_MAX_REQS and t.suffix_offsets is None:
                    t.plan_on_device(suffix_lane_capacity(device, num_heads, head_dim, **shape), device)
                else:
                    t.set_plan(lens, suffix_lanes(device, num_heads, head_dim, total, **shape), device)
        return t


_cu_counts: Dict[str, int] = {}


def _cu_count(device) -> int:
    key = str(device)
    n = _cu_counts.get(key)
    if n is None:
        n = 256
        if torch.cuda.is_available() and key != "cpu":
            n = torch.cuda.get_device_properties(device).multi_processor_count
        _cu_counts[key] = n
    return n


def suffix_tables_append(table: torch.Tensor, lens: torch.Tensor, rows: Optional[torch.Tensor],
                         new_slots: torch.Tensor) -> None:
    """``table[rows[i], lens[rows[i]]] = new_slots[i]; lens[rows[i]] += 1`` on the device (int32 tensors; the
    per-iteration patch of the padded suffix table, in place of rebuilding it from lists)."""
    _require_gpu(table, lens, new_slots)
    assert table.dtype == lens.dtype == new_slots.dtype == torch.int32 and table.dim() == 2 and table.stride(1) == 1
    assert rows is None or (rows.dtype == torch.int32 and rows.numel() == new_slots.numel())
    check(_lib.load().ph_suffix_tables_append(_ptr(table), table.stride(0), _ptr(lens), _ptr(rows), _ptr(new_slots),
                                              new_slots.numel(), _stream()), "suffix_tables_append")


def suffix_plan_build(lens: torch.Tensor, num_lanes: int, items: torch.Tensor, lane_rec: torch.Tensor,
                      req_item_cu: torch.Tensor, max_len: int = 2 ** 31 - 1) -> None:
    """The balanced suffix plan written on the device from the device length vector (``ph_suffix_plan_build``):
    ``items [num_lanes + B, 4]``, ``lane_rec [num_lanes, 8]``, ``req_item_cu [B + 1]``, all int32.  Lengths are
    read clamped to ``[0, max_len]`` (the width of the slot table), as the attention kernels read them."""
    _require_gpu(lens, items, lane_rec, req_item_cu)
    B = lens.numel()
    assert lens.dtype == items.dtype == lane_rec.dtype == req_item_cu.dtype == torch.int32
    assert items.numel() >= (num_lanes + B) * 4 and lane_rec.numel() >= num_lanes * 8 and req_item_cu.numel() >= B + 1
    check(_lib.load().ph_suffix_plan_build(_ptr(lens), B, int(max_len), num_lanes, _ptr(items), _ptr(lane_rec),
                                           _ptr(req_item_cu), _stream()), "suffix_plan_build")


PLAN_MAX_REQS = 8192  # batch size up to which the library plans on the device


def _heads_per_wave(head_dim: int) -> int:
    """A head's elements sit on head_dim / 8 lanes, rounded up to a power of two (80, 96, 112 take 16 like 128)."""
    lanes = 1
    while lanes * 8 < head_dim:
        lanes *= 2
    return max(1, 64 // lanes)


def suffix_lane_capacity(device, num_heads: int, head_dim: int, num_reqs: int = 0, num_groups: int = 0,
                         max_prefix_len: int = 0, max_suffix_len: int = 0, dtype: torch.dtype = torch.float16,
                         kv_group: int = 1) -> int:
    """Lanes the balanced suffix plan should be cut into (``ph_decode_suffix_lanes``): one launch-wide round of waves
    at two waves per SIMD on the compute units the suffix phase runs on -- all of them, or, for a batch whose
    prefix and suffix phases get workgroups of their own inside one launch, the ones the prefix leaves.
    ``kv_group = G > 1``: the call will name a head mapping ``h // G`` (``decode_attention(..., kv_group=G)``), where
    the suffix waves may divide the KV heads instead of the query heads."""
    if num_reqs <= 0 or str(device) == "cpu" or not torch.cuda.is_available():
        heads_per_wave = _heads_per_wave(head_dim)
        hgroups = (num_heads + heads_per_wave - 1) // heads_per_wave
        return max(1, _cu_count(device) * 4 * 2 // hgroups)
    code = {torch.float16: _lib.PH_F16, torch.bfloat16: _lib.PH_BF16, torch.float32: _lib.PH_F32}[dtype]
    with torch.cuda.device(device):
        return int(_lib.load().ph_decode_suffix_lanes(num_reqs, num_heads, head_dim, code, num_groups, max_prefix_len,
                                                      max_suffix_len, max(1, int(kv_group))))


def suffix_lanes(device, num_heads: int, head_dim: int, total_tokens: int, **shape) -> int:
    """Pieces of the host-planned balanced suffix phase: ``suffix_lane_capacity`` (a piece is streamed by one wave
    per `_heads_per_wave(head_dim)` heads; measured: one to three waves per SIMD stream at the same rate, and fewer,
    longer pieces pay the start-up chain less often), and no piece under 4 tokens (one round of the streaming body's
    register pipeline)."""
    lanes = suffix_lane_capacity(device, num_heads, head_dim, **shape)
    return max(1, min(lanes, (total_tokens + 3) // 4))


def plan_suffix_items(lens: Sequence[int], num_lanes: int):
    """(items [n, 4] int32, lane_item_cu [lanes+1] int32, req_item_cu [B+1] int32): the token stream of
    all requests back to back is cut at the request boundaries and at ``num_lanes`` near-equal marks."""
    lens_a = np.asarray(lens, dtype=np.int64)
    B = lens_a.shape[0]
    cu = np.zeros(B + 1, dtype=np.int64)
    np.cumsum(lens_a, out=cu[1:])
    total = int(cu[-1])
    if total == 0:
        return np.zeros((0, 4), np.int32), np.zeros(1, np.int32), np.zeros(B + 1, np.int32)
    num_lanes = max(1, min(num_lanes, total))
    cuts = (np.arange(num_lanes + 1, dtype=np.int64) * total) // num_lanes
    pts = np.unique(np.concatenate([cu, cuts]))
    a, b = pts[:-1], pts[1:]
    req = np.searchsorted(cu, a, side="right") - 1
    lane = np.searchsorted(cuts, a, side="right") - 1
    items = np.zeros((a.shape[0], 4), dtype=np.int32)
    items[:, 0] = req
    items[:, 1] = a - cu[req]
    items[:, 2] = b - a
    lane_cu = np.zeros(num_lanes + 1, dtype=np.int32)
    np.cumsum(np.bincount(lane, minlength=num_lanes), out=lane_cu[1:])
    req_cu = np.zeros(B + 1, dtype=np.int32)
    np.cumsum(np.bincount(req, minlength=B), out=req_cu[1:])
    return items, lane_cu, req_cu


def decode_attention(query: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor, tables: DecodeTables,
                     scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                     events6=None, head_mapping: Optional[torch.Tensor] = None, kv_group: int = 0) -> torch.Tensor:
    """Shared-prefix (or plain ragged) decode attention: prefix phase on the
    matrix cores, per-request suffix phase, log-sum-exp merge.  ``events6``: optional array of six
    ``hipEvent_t`` handles that receive the begin / end timestamps of the call's prefix, suffix and merge
    kernels (``ph_decode_attention_timed``).  ``head_mapping`` (int32 device ``[H]``): query head h reads KV head
    ``head_mapping[h]`` of caches ``[slots, H_kv, D]``; ``kv_group = G > 0`` states that it is ``h // G``
    (``ph_decode_attention_gqa``)."""
    _require_gpu(query, key_cache, value_cache)
    assert query.dim() == 3 and key_cache.dim() == 3 and value_cache.shape == key_cache.shape
    B, H, D = query.shape
    assert B == tables.num_reqs
    if head_mapping is None:
        assert key_cache.shape[1:] == (H, D), "cache head shape mismatch"
    else:
        assert events6 is None, "the timed call has no head mapping"
        assert key_cache.shape[2] == D and head_mapping.dtype == torch.int32 and head_mapping.numel() == H
        assert head_mapping.is_contiguous() and head_mapping.device == query.device
    assert query.dtype == key_cache.dtype == value_cache.dtype
    assert query.stride(2) == 1 and query.stride(1) == D
    assert key_cache.stride(2) == 1 and key_cache.stride(1) == D and key_cache.stride() == value_cache.stride()
    if out is None:
        out = torch.empty((B, H, D), dtype=query.dtype, device=query.device)
    if B == 0:
        return out
    scale = D ** -0.5 if scale is None else scale
    lib = _lib.load()
    plan = tables.plan
    nbytes = lib.ph_decode_workspace_bytes(B, H, D, tables.num_groups, tables.max_prefix_len, tables.max_suffix_len,
                                           tables.chunk_tokens, 0 if plan is None else plan.num_items)
    ws = _workspace(nbytes, query.device)
    args = (
        _ptr(out), _ptr(query), _ptr(key_cache), _ptr(value_cache), B, H, D, _dtype_code(query),
        query.stride(0), out.stride(0), key_cache.stride(0), float(scale),
        tables.num_groups, _ptr(tables.prefix_slots), _ptr(tables.prefix_cu), _ptr(tables.group_req_cu),
        _ptr(tables.group_req_cu_host), tables.max_prefix_len,
        _ptr(tables.suffix_slots), _ptr(tables.suffix_offsets), tables.suffix_table_stride,
        tables.suffix_slots_count(), _ptr(tables.suffix_lens),
        tables.max_suffix_len, tables.chunk_tokens, None if plan is None else ctypes.byref(plan),
        _ptr(ws), ws.numel(), _stream())
    if head_mapping is not None:
        rc = lib.ph_decode_attention_gqa(*args[:6], key_cache.shape[1], _ptr(head_mapping), int(kv_group), *args[6:])
    elif events6 is None:
        rc = lib.ph_decode_attention(*args)
    else:
        rc = lib.ph_decode_attention_timed(*args, events6)
    check(rc, "decode_attention")
    return out


def decode_attention_static(query: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                            tables: DecodeTables, out: torch.Tensor, scale: Optional[float] = None) -> torch.Tensor:
    """``decode_attention`` on the library's own fixed scratch array (``ph_decode_attention_static``): nothing is
    allocated, here or in the library, so ``out`` must be given.  Shapes whose partials exceed the array raise
    ``RuntimeError``; calls that overlap on one device share the array and must be serialised by the caller."""
    _require_gpu(query, key_cache, value_cache, out)
    B, H, D = query.shape
    assert B == tables.num_reqs and out.shape == query.shape and out.dtype == query.dtype
    assert key_cache.shape[1:] == (H, D) and value_cache.shape == key_cache.shape
    assert query.dtype == key_cache.dtype == value_cache.dtype
    assert query.stride(2) == 1 and query.stride(1) == D and out.stride(2) == 1 and out.stride(1) == D
    assert key_cache.stride(2) == 1 and key_cache.stride(1) == D and key_cache.stride() == value_cache.stride()
    if B == 0:
        return out
    scale = D ** -0.5 if scale is None else scale
    plan = tables.plan
    rc = _lib.load().ph_decode_attention_static(
        _ptr(out), _ptr(query), _ptr(key_cache), _ptr(value_cache), B, H, D, _dtype_code(query),
        query.stride(0), out.stride(0), key_cache.stride(0), float(scale),
        tables.num_groups, _ptr(tables.prefix_slots), _ptr(tables.prefix_cu), _ptr(tables.group_req_cu),
        _ptr(tables.group_req_cu_host), tables.max_prefix_len,
        _ptr(tables.suffix_slots), _ptr(tables.suffix_offsets), tables.suffix_table_stride,
        tables.suffix_slots_count(), _ptr(tables.suffix_lens),
        tables.max_suffix_len, tables.chunk_tokens, None if plan is None else ctypes.byref(plan), _stream())
    check(rc, "decode_attention_static")
    return out


_small_cache: Dict[Tuple, Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = {}


def _single_group_cu(P: int, B: int, device) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    key = (P, B, str(device))
    hit = _small_cache.get(key)
    if hit is None:
        if len(_small_cache) > 256:
            _small_cache.clear()
        host = torch.tensor([0, B], dtype=torch.int32)
        hit = (torch.tensor([0, P], dtype=torch.int32, device=device), host.to(device), host)
        _small_cache[key] = hit
    return hit


# head mappings seen before: id of the tensor -> (the tensor itself, its version, what it was found to be).  The
# entry holds the tensor, so its id and address cannot pass to another tensor while the entry lives.
_head_maps: "collections.OrderedDict[int, Tuple[torch.Tensor, int, int, Tuple[Optional[torch.Tensor], int]]]" = \
    collections.OrderedDict()


def _head_mapping_info(head_mapping: torch.Tensor, num_heads: int, num_kv_heads: int) -> Tuple[Optional[torch.Tensor], int]:
    """``head_mapping[h]`` names the KV head of query head h (3rdparty/vllm/csrc/attention/attention_kernels.cu:
    ``kv_head_idx = head_mapping[head_idx]``).  Returns ``(None, 0)`` for the identity over as many KV heads as query
    heads (what the reference's models pass, models/llama.py:95-97: the plain kernels), else ``(int32 mapping on
    the device, G)`` with ``G > 0`` when the mapping is ``h // G`` and 0 for any other.  The contents are read
    once per tensor and version (one small copy to the host)."""
    assert head_mapping.shape[0] == num_heads, "head_mapping must have one entry per head"
    hit = _head_maps.get(id(head_mapping))
    if hit is not None and hit[0] is head_mapping and hit[1] == head_mapping._version and hit[2] == num_kv_heads:
        return hit[3]
    host = head_mapping.detach().cpu().to(torch.int64)
    if int(host.min()) < 0 or int(host.max()) >= num_kv_heads:
        raise ValueError("head_mapping names a KV head outside the cache")
    if num_kv_heads == num_heads and torch.equal(host, torch.arange(num_heads)):
        info: Tuple[Optional[torch.Tensor], int] = (None, 0)
    else:
        group = num_heads // num_kv_heads if num_heads % num_kv_heads == 0 else 0
        if group and not torch.equal(host, torch.arange(num_heads) // group):
            group = 0
        info = (head_mapping.to(torch.int32).contiguous(), group)
    _head_maps[id(head_mapping)] = (head_mapping, head_mapping._version, num_kv_heads, info)
    while len(_head_maps) > 16:
        _head_maps.popitem(last=False)
    return info


def _check_paged_args(query, key_cache, value_cache, head_mapping, context_lens, block_tables):
    """Argument checks of the reference-named ops; returns the head mapping as ``decode_attention`` takes it."""
    if key_cache.dim() != 3 or value_cache.dim() != 3:
        raise ValueError("key_cache / value_cache must be token-granular [slots, H, D] (block_size 1)")
    assert block_tables.dim() == 2 and block_tables.dtype == torch.int32
    assert context_lens.dtype == torch.int32 and context_lens.shape[0] == query.shape[0]
    assert block_tables.shape[0] == query.shape[0]
    mapping, group = _head_mapping_info(head_mapping, query.shape[1], key_cache.shape[1])
    return dict(head_mapping=mapping, kv_group=group)


# Device tables (with the balanced suffix plan) of recent calls of the reference-named ops.  Unchanged model code
# calls these once per layer with the same tensors, and the plan depends on the lengths only: layer 1 of an
# iteration builds it, layers 2..L find it here.  An entry is keyed by the tensors' addresses and torch's version
# counter of the length tensor, and holds references to the tensors, so an address cannot come back for another
# tensor while its entry lives; a length tensor rewritten in place through torch bumps the version and misses.
# (Writes torch does not see -- a kernel of the caller's own -- are not detected: such a caller passes a new tensor.)
_paged_tables_cache: "collections.OrderedDict[Tuple, Tuple[Tuple, DecodeTables]]" = collections.OrderedDict()
_PAGED_TABLES_CACHE_ENTRIES = 8


def _paged_tables(query, context_lens, block_tables, flash_context_len: int = 0, flash_block_table=None,
                  kv_group: int = 0) -> DecodeTables:
    B, H, D = query.shape
    P = int(flash_context_len)
    key = (context_lens.data_ptr(), context_lens._version, B, block_tables.data_ptr(), block_tables.stride(0),
           block_tables.shape[1], H, D, query.dtype, P, 0 if flash_block_table is None else flash_block_table.data_ptr(),
           str(query.device), kv_group)
    hit = _paged_tables_cache.get(key)
    if hit is not None:
        _paged_tables_cache.move_to_end(key)
        return hit[1]
    table = block_tables if block_tables.stride(1) == 1 else block_tables.contiguous()
    lens = context_lens.contiguous()
    t = DecodeTables(num_reqs=B, suffix_slots=table, suffix_offsets=None, suffix_table_stride=table.stride(0),
                     suffix_lens=lens, max_suffix_len=table.shape[1])
    if P > 0:
        assert flash_block_table.dtype == torch.int32 and flash_block_table.numel() >= P
        cu, gcu, gcu_host = _single_group_cu(P, B, query.device)
        t.num_groups = 1
        t.prefix_slots = flash_block_table.contiguous()
        t.prefix_cu, t.group_req_cu, t.group_req_cu_host = cu, gcu, gcu_host
        t.max_prefix_len = P
    if 0 < B <= PLAN_MAX_REQS and t.max_suffix_len > 0:
        t.plan_on_device(suffix_lane_capacity(query.device, H, D, num_reqs=B, num_groups=t.num_groups,
                                              max_prefix_len=t.max_prefix_len, max_suffix_len=t.max_suffix_len,
                                              dtype=query.dtype, kv_group=kv_group), query.device)
    _paged_tables_cache[key] = ((context_lens, block_tables, flash_block_table), t)
    while len(_paged_tables_cache) > _PAGED_TABLES_CACHE_ENTRIES:
        _paged_tables_cache.popitem(last=False)
    return t


def vllm_paged_attention(query, key_cache, value_cache, head_mapping, context_lens, block_tables):
    """Non-shared ragged decode (parrot/engine/builtin/kernels/vllm/paged_attention.py:12-38):
    request i attends over ``block_tables[i, :context_lens[i]]``."""
    heads = _check_paged_args(query, key_cache, value_cache, head_mapping, context_lens, block_tables)
    tables = _paged_tables(query, context_lens, block_tables, kv_group=heads["kv_group"])
    return decode_attention(query, key_cache, value_cache, tables, **heads)


def flash_paged_attention(query, key_cache, value_cache, head_mapping, flash_context_len, flash_block_table,
                          paged_context_lens, paged_block_tables):
    """Shared-prefix decode (parrot/engine/builtin/kernels/shared_flash_decoding.py:285-329):
    all requests attend over ``flash_block_table[:flash_context_len]`` plus their
    own ``paged_block_tables[i, :paged_context_lens[i]]``."""
    heads = _check_paged_args(query, key_cache, value_cache, head_mapping, paged_context_lens, paged_block_tables)
    t = _paged_tables(query, paged_context_lens, paged_block_tables, flash_context_len, flash_block_table,
                      kv_group=heads["kv_group"])
    return decode_attention(query, key_cache, value_cache, t, **heads)


def paged_flash_attention(query, key_cache, value_cache, head_mapping, flash_context_len, flash_block_table,
                          paged_context_lens, paged_block_tables):
    """The phases in the other order, as in the reference (shared_flash_decoding.py:332-376): the suffix phase
    first, exporting its row maxima and denominators (``single_query_cached_kv_prev_attention``), then the prefix
    phase merged on top of it in place (the Triton kernel with ``load_mid_results``) -- two calls of the library,
    ``ph_suffix_prev_attention`` and ``ph_prefix_post_attention``.  Same result as ``flash_paged_attention``."""
    heads = _check_paged_args(query, key_cache, value_cache, head_mapping, paged_context_lens, paged_block_tables)
    if heads["head_mapping"] is not None:
        raise ValueError("paged_flash_attention (the split entry points) takes the identity head_mapping only; "
                         "flash_paged_attention serves grouped KV heads")
    _require_gpu(query, key_cache, value_cache, paged_context_lens, paged_block_tables)
    B, H, D = query.shape
    assert key_cache.shape[1:] == (H, D) and value_cache.shape == key_cache.shape
    assert query.dtype == key_cache.dtype == value_cache.dtype
    assert query.stride(2) == 1 and query.stride(1) == D
    assert key_cache.stride(2) == 1 and key_cache.stride(1) == D and key_cache.stride() == value_cache.stride()
    out = torch.empty((B, H, D), dtype=query.dtype, device=query.device)
    if B == 0:
        return out
    P = int(flash_context_len)
    table = paged_block_tables if paged_block_tables.stride(1) == 1 else paged_block_tables.contiguous()
    lens = paged_context_lens.contiguous()
    width = table.shape[1]
    lib = _lib.load()
    scale = D ** -0.5
    m = torch.empty((B, H), dtype=torch.float32, device=query.device)
    l = torch.empty((B, H), dtype=torch.float32, device=query.device)
    nbytes = max(lib.ph_decode_workspace_bytes(B, H, D, 0, 0, width, 0, 0),
                 lib.ph_decode_workspace_bytes(B, H, D, 1 if P > 0 else 0, P, 0, 0, 0))
    ws = _workspace(nbytes, query.device)
    code, st = _dtype_code(query), _stream()
    check(lib.ph_suffix_prev_attention(
        _ptr(out), _ptr(m), _ptr(l), _ptr(query), _ptr(key_cache), _ptr(value_cache), B, H, D, code,
        query.stride(0), out.stride(0), key_cache.stride(0), float(scale), _ptr(table), None, table.stride(0),
        (B - 1) * table.stride(0) + width, _ptr(lens), width, 0, _ptr(ws), ws.numel(), st), "paged_flash_attention")
    if P > 0:
        assert flash_block_table.dtype == torch.int32 and flash_block_table.numel() >= P
        check(lib.ph_prefix_post_attention(
            _ptr(out), _ptr(m), _ptr(l), _ptr(query), _ptr(key_cache), _ptr(value_cache), B, H, D, code,
            query.stride(0), out.stride(0), key_cache.stride(0), float(scale), _ptr(flash_block_table.contiguous()), P,
            _ptr(ws), ws.numel(), st), "paged_flash_attention")
    return out


# --------------------------------------------------------------------------- #
# prefill with parent context
# --------------------------------------------------------------------------- #
@dataclasses.dataclass
class PrefillTables:
    num_tokens: int
    num_chunks: int
    q_cu: torch.Tensor  # int32 [C+1] device
    kv_cu: torch.Tensor  # int32 [C+1] device
    ctx_slots: torch.Tensor  # int32 device
    max_kv_len: int

    @staticmethod
    def build(q_lens: Sequence[int], ctx_slot_lists: Sequence[Sequence[int]], device) -> "PrefillTables":
        q_cu, kv_cu, flat = [0], [0], []
        for n, s in zip(q_lens, ctx_slot_lists):
            assert len(s) >= n, "a chunk's context must include its own tokens"
            q_cu.append(q_cu[-1] + n)
            flat.extend(s)
            kv_cu.append(len(flat))
        return PrefillTables(
            num_tokens=q_cu[-1], num_chunks=len(q_lens),
            q_cu=torch.tensor(q_cu, dtype=torch.int32, device=device),
            kv_cu=torch.tensor(kv_cu, dtype=torch.int32, device=device),
            ctx_slots=torch.tensor(flat if flat else [0], dtype=torch.int32, device=device),
            max_kv_len=max((len(s) for s in ctx_slot_lists), default=0))


def prefill_attention(query, key_cache, value_cache, tables: PrefillTables, scale: Optional[float] = None,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Packed ragged prefill, each chunk causal (bottom-right aligned) over its
    ancestors' and its own KV read through the slot table -- the op the
    reference assembles from a gather plus xformers' block-diagonal FMHA
    (parrot/engine/builtin/attn_func.py:635-674)."""
    _require_gpu(query, key_cache, value_cache)
    T, H, D = query.shape
    assert T == tables.num_tokens
    assert key_cache.shape[1:] == (H, D) and value_cache.shape == key_cache.shape
    assert query.dtype == key_cache.dtype == value_cache.dtype
    assert query.stride(2) == 1 and query.stride(1) == D
    assert key_cache.stride(2) == 1 and key_cache.stride(1) == D and key_cache.stride() == value_cache.stride()
    if out is None:
        out = torch.empty((T, H, D), dtype=query.dtype, device=query.device)
    if T == 0:
        return out
    scale = D ** -0.5 if scale is None else scale
    lib = _lib.load()
    nbytes = lib.ph_prefill_workspace_bytes(T, H, D, _dtype_code(query), tables.max_kv_len)
    ws = _workspace(nbytes, query.device)
    rc = lib.ph_prefill_attention(
        _ptr(out), _ptr(query), _ptr(key_cache), _ptr(value_cache), T, tables.num_chunks, H, D, _dtype_code(query),
        query.stride(0), out.stride(0), key_cache.stride(0), float(scale), _ptr(tables.q_cu), _ptr(tables.kv_cu),
        _ptr(tables.ctx_slots), tables.ctx_slots.numel(), tables.max_kv_len, _ptr(ws), ws.numel(), _stream())
    check(rc, "prefill_attention")
    return out
