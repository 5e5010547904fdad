"""CPU restatement of the builtin engine's LLaMA forward over ONE flat token sequence.

TEST INFRASTRUCTURE ONLY (imported by tests/): composes the already pinned
oracle ops in the order of parrot/engine/builtin/models/llama.py:102-226 --
embedding, per layer RMSNorm -> qkv -> NeoX RoPE -> causal attention -> o_proj
-> residual -> RMSNorm -> SiLU MLP -> residual, final RMSNorm -- with no slots,
contexts or iteration state, so it is independent of everything the engine loop
adds.  fp32 math on the given (dtype-rounded) weights; intermediate activations
are NOT re-rounded, so comparisons against the fp16 engine need a tolerance that
covers per-layer rounding.
Pins: the ops it calls are pinned in tests/test_oracle_*.py; the composition is
pinned in tests/test_oracle_llama.py against torch's own scaled_dot_product_attention
/ rms_norm / silu on the same weights and by the prefix property (the hidden
state of token t does not depend on tokens after t).
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .ref_ops import ref_cos_sin_cache, ref_prefill_with_parent, ref_rms_norm, ref_rope_neox


def ref_llama_hidden(w: Dict[str, torch.Tensor], token_ids: Sequence[int], num_heads: int, eps: float,
                     theta: float = 10000.0, cache_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``w``: embed [V, N]; per layer i: ``l{i}.ln1``, ``l{i}.qkv`` [3N, N], ``l{i}.o`` [N, N], ``l{i}.ln2``,
    ``l{i}.gate`` / ``l{i}.up`` [F, N], ``l{i}.down`` [N, F]; ``norm`` [N].  ``cache_dtype``: element type the engine keeps its cos/sin table in (mem.py:125-143 casts it).
    Returns fp32 [T, N] after the final norm."""
    ids = torch.as_tensor(list(token_ids), dtype=torch.long)
    T = ids.numel()
    x = w["embed"].float()[ids]
    N = x.shape[1]
    D = N // num_heads
    pos = torch.arange(T)
    cache = ref_cos_sin_cache(T, D, theta, cache_dtype).float()
    n_layers = sum(1 for k in w if k.endswith(".qkv"))
    for i in range(n_layers):
        h = ref_rms_norm(x, w[f"l{i}.ln1"].float(), eps, round_before_weight=False).float()
        qkv = h @ w[f"l{i}.qkv"].float().t()
        q, k, v = qkv.chunk(3, dim=-1)
        q, k = ref_rope_neox(pos, q.contiguous(), k.contiguous(), cache, D, elem_rounding=False)
        q, k, v = (t.reshape(T, num_heads, D).float() for t in (q, k, v))
        a = ref_prefill_with_parent(q, k, v, [T], [torch.arange(T)]).float()  # plain causal attention
        x = x + a.reshape(T, N) @ w[f"l{i}.o"].float().t()
        h = ref_rms_norm(x, w[f"l{i}.ln2"].float(), eps, round_before_weight=False).float()
        g = torch.nn.functional.silu(h @ w[f"l{i}.gate"].float().t()) * (h @ w[f"l{i}.up"].float().t())
        x = x + g @ w[f"l{i}.down"].float().t()
    return ref_rms_norm(x, w["norm"].float(), eps, round_before_weight=False).float()
