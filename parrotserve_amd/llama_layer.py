"""LLaMA decoder-layer wiring around the attention plug-in
(parrot/engine/builtin/models/llama.py:54-178): RMSNorm -> qkv_proj -> RoPE (in
place on strided chunk views of the fused qkv) -> AttnFunc -> o_proj -> RMSNorm
-> MLP, with the two residual adds.  GEMMs are plain ``nn.Linear`` (library
GEMMs); norms, RoPE and attention are the HIP kernels.

``fused_ops=True`` keeps the same arithmetic with fewer launches: RoPE and the KV
append in one kernel, silu(gate) * up in one kernel, and each residual add folded
into the norm that follows it (the layer then hands ``(mlp_out, residual)`` to the
next layer, whose first norm performs the add)."""
from __future__ import annotations

import torch
from torch import nn

from .kernels import fused_add_rms_norm, rope_and_cache, silu_mul, vllm_rms_norm, vllm_rotary_emb
from .mem import get_cos_sin_cache, get_k_cache, get_v_cache


class LlamaRMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        return vllm_rms_norm(x, self.weight, self.eps)

    def forward_add(self, x, residual):
        """``residual += x`` in place; returns the norm of the sum."""
        return fused_add_rms_norm(x, residual, self.weight, self.eps)


class LlamaMLP(nn.Module):
    """down(silu(gate(x)) * up(x)) -- the HF module the reference imports (models/llama.py:36-39)."""

    def __init__(self, hidden_size: int, intermediate_size: int, fused_ops: bool = False):
        super().__init__()
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=False)
        self.fused_ops = fused_ops

    def forward(self, x):
        if self.fused_ops:
            return self.down_proj(silu_mul(self.gate_proj(x), self.up_proj(x)))
        return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))


class LlamaAttention(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, layer_idx: int, attn_func_cls, fused_ops: bool = False):
        super().__init__()
        self.fused_ops = fused_ops
        self.layer_idx = layer_idx
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.head_dim = hidden_size // num_heads
        if self.head_dim * num_heads != hidden_size:
            raise ValueError("hidden_size must be divisible by num_heads")
        self.scaling = self.head_dim ** -0.5
        self.qkv_proj = nn.Linear(hidden_size, 3 * hidden_size, bias=False)
        self.o_proj = nn.Linear(hidden_size, hidden_size, bias=False)
        self.attn_func = attn_func_cls(layer_idx=layer_idx, scaling=self.scaling, num_heads=num_heads,
                                       head_dim=self.head_dim)

    def forward(self, hidden_states, positions, iteration_state):
        qkv = self.qkv_proj(hidden_states)
        q, k, v = torch.chunk(qkv, 3, dim=-1)
        if self.fused_ops:
            # attention reads K from the cache only (kv_appended below), so k need not be rotated in place
            rope_and_cache(positions, q, k, v, get_cos_sin_cache(), self.head_dim, get_k_cache(self.layer_idx),
                           get_v_cache(self.layer_idx), iteration_state.slot_mapping, key_in_place=False)
        else:
            vllm_rotary_emb(positions, q, k, get_cos_sin_cache(), head_size=self.head_dim)
        q = q.view(-1, self.num_heads, self.head_dim)
        k = k.view(-1, self.num_heads, self.head_dim)
        v = v.view(-1, self.num_heads, self.head_dim)
        if self.fused_ops:
            return self.o_proj(self.attn_func(q, k, v, iteration_state, kv_appended=True))
        return self.o_proj(self.attn_func(q, k, v, iteration_state))


class LlamaDecoderLayer(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, intermediate_size: int, rms_norm_eps: float, layer_idx: int,
                 attn_func_cls, fused_ops: bool = False):
        super().__init__()
        self.self_attn = LlamaAttention(hidden_size, num_heads, layer_idx, attn_func_cls, fused_ops)
        self.mlp = LlamaMLP(hidden_size, intermediate_size, fused_ops)
        self.input_layernorm = LlamaRMSNorm(hidden_size, eps=rms_norm_eps)
        self.post_attention_layernorm = LlamaRMSNorm(hidden_size, eps=rms_norm_eps)

    def forward(self, hidden_states, positions, iteration_state):
        residual = hidden_states
        hidden_states = self.input_layernorm(hidden_states)
        hidden_states = self.self_attn(hidden_states, positions, iteration_state)
        hidden_states = residual + hidden_states
        residual = hidden_states
        hidden_states = self.post_attention_layernorm(hidden_states)
        hidden_states = self.mlp(hidden_states)
        return residual + hidden_states

    def forward_fused(self, hidden_states, residual, positions, iteration_state):
        """Same layer with the residual adds folded into the norms: takes the previous layer's MLP output and
        running residual (``residual is None`` for the first layer: ``hidden_states`` is the embedding), returns
        this layer's MLP output and the residual it must still be added to."""
        if residual is None:
            residual = hidden_states
            hidden_states = self.input_layernorm(hidden_states)
        else:
            hidden_states = self.input_layernorm.forward_add(hidden_states, residual)
        hidden_states = self.self_attn(hidden_states, positions, iteration_state)
        hidden_states = self.post_attention_layernorm.forward_add(hidden_states, residual)
        return self.mlp(hidden_states), residual
