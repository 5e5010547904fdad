"""KV pools and cos/sin cache (parrot/engine/builtin/mem.py:22-206), token-granular layout only:
``k_cache`` / ``v_cache`` are ``[layers, slots, H, D]``."""
from __future__ import annotations

from typing import Optional

import torch


class ModelCacheStorage:
    def __init__(self, num_layers: int, num_slots: int, num_heads: int, head_size: int, dtype: torch.dtype, device,
                 max_seq_len: int = 0, rope_theta: float = 10000.0) -> None:
        self.k_cache = torch.empty([num_layers, num_slots, num_heads, head_size], dtype=dtype, device=device)
        self.v_cache = torch.empty([num_layers, num_slots, num_heads, head_size], dtype=dtype, device=device)
        self.cos_sin_cache: Optional[torch.Tensor] = None
        if max_seq_len > 0:
            self.cos_sin_cache = make_cos_sin_cache(max_seq_len, head_size, rope_theta, dtype, device)


def make_cos_sin_cache(max_seq_len: int, rotary_size: int, rope_theta: float, dtype: torch.dtype, device) -> torch.Tensor:
    """``cat(cos(t*inv_freq), sin(t*inv_freq))`` in fp32, then cast (mem.py:125-143)."""
    inv_freq = 1.0 / (rope_theta ** (torch.arange(0, rotary_size, 2, device=device).float() / rotary_size))
    t = torch.arange(max_seq_len, dtype=inv_freq.dtype, device=device)
    freqs = torch.outer(t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(dtype)


Model_Cache: Optional[ModelCacheStorage] = None


def init_model_cache_storage(*args, **kwargs) -> ModelCacheStorage:
    """Two call forms.  The reference's (parrot/engine/builtin/mem.py:179-184):
    ``init_model_cache_storage(hf_config, builtin_config)`` -- layers, heads, head size, maximum positions and rope
    base are read from the model configuration, slot count, dtype and device from the engine configuration.  And the
    explicit one: ``init_model_cache_storage(num_layers, num_slots, num_heads, head_size, dtype, device,
    max_seq_len=0, rope_theta=10000.0)``."""
    global Model_Cache
    if args and hasattr(args[0], "num_hidden_layers"):
        hf_config, builtin_config = args[0], (args[1] if len(args) > 1 else kwargs["builtin_config"])
        heads = hf_config.num_attention_heads
        Model_Cache = ModelCacheStorage(
            hf_config.num_hidden_layers, builtin_config.num_kv_cache_blocks, heads, hf_config.hidden_size // heads,
            builtin_config.dtype, builtin_config.device,
            max_seq_len=getattr(hf_config, "max_position_embeddings", 0) or 0,
            rope_theta=float(getattr(hf_config, "rope_theta", 10000.0) or 10000.0))
    else:
        Model_Cache = ModelCacheStorage(*args, **kwargs)
    return Model_Cache


def get_k_cache(layer_idx: int) -> torch.Tensor:
    assert Model_Cache is not None
    return Model_Cache.k_cache[layer_idx]


def get_v_cache(layer_idx: int) -> torch.Tensor:
    assert Model_Cache is not None
    return Model_Cache.v_cache[layer_idx]


def get_cos_sin_cache() -> torch.Tensor:
    assert Model_Cache is not None and Model_Cache.cos_sin_cache is not None
    return Model_Cache.cos_sin_cache
