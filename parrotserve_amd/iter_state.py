"""Per-iteration carrier (parrot/engine/builtin/iter_state.py:15-60): built once per
iteration, shared by every layer's attention call.

Token rows of an iteration are packed job after job: first every Fill job's new tokens
(``num_fill_tokens[j]`` rows for Fill job j, in job order), then one row per Generate job.
The attention plug-in attaches its index tables to this object in ``init_iteration_state``.
"""
from __future__ import annotations

from typing import Any, List


class IterationState:
    def __init__(self, jobs: List[Any], model_config: Any, builtin_config: Any):
        self.num_fill_tokens: List[int] = []
        self.generation_sampling_config: List[Any] = []
        num_heads = model_config.num_attention_heads
        head_size = model_config.hidden_size // num_heads
        builtin_config.attn_func.init_iteration_state(self, builtin_config, jobs, num_heads, head_size)

    @property
    def num_fill_jobs(self) -> int:
        return len(self.num_fill_tokens)

    @property
    def num_generation_jobs(self) -> int:
        return len(self.generation_sampling_config)

    @property
    def num_total_fill_tokens(self) -> int:
        return sum(self.num_fill_tokens)
