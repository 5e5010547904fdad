"""Iteration loop of the builtin engine around the HIP attention path
(parrot/engine/builtin/builtin_runner.py:36-199, models/llama.py:181-226,
models/sampler.py:13-66, engine/context/context_manager.py:13-62): jobs are
sorted Fill-first, contexts are bound and grown, the index tables are built once
per iteration, the model runs, contexts take the sampled tokens.

Weights are random (``initialize_dummy_weights``, models/weight_utils.py:52-65)
or set by the caller; nothing is downloaded.  The model configuration is a plain
object with the Hugging Face LLaMA field names the reference reads.
"""
from __future__ import annotations

import dataclasses
import time
from typing import Dict, List, Optional, Tuple

import torch
from torch import nn

from . import kernels, mem
from .attn_func import BuiltinConfig
from .context import BlockContext, RecyclePool
from .iter_state import IterationState
from .llama_layer import LlamaDecoderLayer, LlamaRMSNorm
from .primitive_job import Fill, Generate, PrimitiveJob

NONE_CONTEXT_ID = -1


@dataclasses.dataclass
class SamplingConfig:
    """parrot/sampling_config.py: the fields the engine reads."""

    temperature: float = 1.0
    top_p: float = 1.0
    max_gen_length: int = 512
    ignore_tokenizer_eos: bool = False
    stop_token_ids: List[int] = dataclasses.field(default_factory=list)


@dataclasses.dataclass
class LlamaConfig:
    vocab_size: int = 32000
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    rms_norm_eps: float = 1e-6
    max_position_embeddings: int = 4096
    rope_theta: float = 10000.0
    pad_token_id: Optional[int] = None
    fused_ops: bool = False  # fewer launches, same arithmetic (see llama_layer)


class EngineContextManager:
    """context id -> context; a job's context is created on first sight under its parent."""

    def __init__(self) -> None:
        self.map: Dict[int, BlockContext] = {}

    def free_context(self, context_id: int) -> int:
        if context_id not in self.map:
            return 0
        context = self.map.pop(context_id)
        n = context.get_this_context_len()
        context.destruction()
        return n

    def bind_job_context(self, job: PrimitiveJob, ctx_cls, **ctx_kwargs) -> None:
        if job.context_id not in self.map:
            parent = None if job.parent_context_id == NONE_CONTEXT_ID else self.map[job.parent_context_id]
            self.map[job.context_id] = ctx_cls(job.context_id, parent, **ctx_kwargs)
        job.context = self.map[job.context_id]

    def get_num_cached_tokens(self) -> int:
        return sum(c.get_this_context_len() for c in self.map.values())


class Sampler(nn.Module):
    """Temperature, top-p, one draw per row over ``hidden @ lm_head.T`` (models/sampler.py:19-66).  Everything
    after the logits GEMM is one kernel (``ph_sample_top_p``): the reference's two sorts become a threshold search
    and its ``torch.multinomial`` an inverse-CDF draw from ``torch.rand`` numbers: the tokens are deterministic
    in torch's generator (same seed, same tokens from run to run) and follow the reference's distribution, but for a
    given seed they are NOT the ids the reference's ``torch.multinomial`` call would draw."""

    # True: the draw is the reference's own call, ``torch.multinomial`` on the filtered probabilities (the library's
    # random stream; one more launch and a [B, V] fp32 tensor), instead of the kernel's inverse-CDF draw
    reference_draw = False

    def __init__(self, config: LlamaConfig, embd_weight: torch.Tensor):
        super().__init__()
        self.embd_weight = embd_weight
        self.vocab_size = config.vocab_size

    def forward(self, hidden_states: torch.Tensor, sampling_config: List[SamplingConfig]) -> torch.Tensor:
        if hidden_states.shape[0] == 0:
            return torch.zeros(0, dtype=torch.int64, device=hidden_states.device)
        assert hidden_states.shape[0] == len(sampling_config)
        logits = torch.matmul(hidden_states, self.embd_weight.t())
        dev = logits.device
        temperature = [sc.temperature for sc in sampling_config]
        top_ps = [sc.top_p for sc in sampling_config]
        t_dev = torch.tensor(temperature, dtype=torch.float, device=dev) if any(t != 1.0 for t in temperature) else None
        p_dev = torch.tensor(top_ps, dtype=torch.float, device=dev) if any(p < 1.0 for p in top_ps) else None
        if self.reference_draw:
            probs = kernels.top_p_probs(logits, t_dev, p_dev)
            return torch.multinomial(probs, num_samples=1, replacement=True).squeeze(-1)
        uniform = torch.rand(logits.shape[0], dtype=torch.float, device=dev)
        return kernels.sample_top_p(logits, t_dev, p_dev, uniform)


def hidden_states_postprocess(hidden_states: torch.Tensor, iteration_state) -> Tuple[torch.Tensor, torch.Tensor]:
    """Last row of every Fill, and the Generate rows (models/model_utils.py:10-21)."""
    idx = 0
    last: List[int] = []
    for n in iteration_state.num_fill_tokens:
        idx += n
        last.append(idx - 1)
    return hidden_states[last], hidden_states[idx:]


class LlamaModel(nn.Module):
    def __init__(self, config: LlamaConfig, builtin_config: BuiltinConfig):
        super().__init__()
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size, config.pad_token_id)
        self.layers = nn.ModuleList([
            LlamaDecoderLayer(config.hidden_size, config.num_attention_heads, config.intermediate_size,
                              config.rms_norm_eps, i, builtin_config.attn_func, config.fused_ops)
            for i in range(config.num_hidden_layers)])
        self.norm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.fused_ops = config.fused_ops

    def forward(self, input_ids, positions, iteration_state):
        hidden_states = self.embed_tokens(input_ids)
        if self.fused_ops:
            residual = None
            for layer in self.layers:
                hidden_states, residual = layer.forward_fused(hidden_states, residual, positions, iteration_state)
            return self.norm.forward_add(hidden_states, residual)
        for layer in self.layers:
            hidden_states = layer(hidden_states, positions, iteration_state)
        return self.norm(hidden_states)


class LlamaForCausalLM(nn.Module):
    def __init__(self, config: LlamaConfig, builtin_config: BuiltinConfig):
        super().__init__()
        self.config = config
        self.model = LlamaModel(config, builtin_config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.sampler = Sampler(config, self.lm_head.weight)

    def forward(self, input_ids, positions, iteration_state):
        hidden_states = self.model(input_ids, positions, iteration_state)
        fill_hidden_states, gen_hidden_states = hidden_states_postprocess(hidden_states, iteration_state)
        next_tokens = self.sampler(gen_hidden_states, iteration_state.generation_sampling_config)
        return fill_hidden_states, next_tokens


def initialize_dummy_weights(model: nn.Module, low: float = -1e-3, high: float = 1e-3) -> None:
    for param in model.state_dict().values():
        param.data.uniform_(low, high)


class BuiltinRunner:
    """One model, one KV pool, one context tree; ``run_iter(jobs)`` is one engine iteration."""

    def __init__(self, model_config: LlamaConfig, config: BuiltinConfig, dummy_weights: bool = True):
        self.builtin_config = config
        self.context_manager = EngineContextManager()
        self.kv_cache_manager = RecyclePool("KVCache pool", pool_size=config.num_kv_cache_blocks)
        self.hf_model_config = model_config
        if config.max_seq_len is not None:
            model_config.max_position_embeddings = config.max_seq_len
        # parameters are created on the device in the target dtype (a 13B model would spend minutes in
        # host-side initialisation otherwise)
        prev = torch.get_default_dtype()
        torch.set_default_dtype(config.dtype)
        try:
            with torch.device(config.device):
                self.model = LlamaForCausalLM(model_config, config)
        finally:
            torch.set_default_dtype(prev)
        if dummy_weights:
            initialize_dummy_weights(self.model)
        heads = model_config.num_attention_heads
        mem.init_model_cache_storage(model_config.num_hidden_layers, config.num_kv_cache_blocks, heads,
                                     model_config.hidden_size // heads, config.dtype, config.device,
                                     max_seq_len=model_config.max_position_embeddings,
                                     rope_theta=model_config.rope_theta)

    @torch.inference_mode()
    def run_iter(self, jobs: List[PrimitiveJob]) -> Tuple[int, int]:
        """Returns (whole-iteration time, model time) in nanoseconds."""
        st = time.perf_counter_ns()
        jobs.sort(key=lambda job: isinstance(job, Generate))  # Fill jobs first
        first_states, first_configs, first_jobs = [], [], []
        for job in jobs:
            if job.context is None:
                self.context_manager.bind_job_context(job, BlockContext, block_size=self.builtin_config.block_size,
                                                      kv_cache_manager=self.kv_cache_manager)
            if isinstance(job, Fill):
                job.context.token_ids.extend(job.token_ids)
                job.context.allocate(len(job.token_ids))
            elif isinstance(job, Generate):
                job.context.allocate(1)
                last_hidden_state = job.context.get_last_hidden_state()
                if last_hidden_state is not None:  # the first token of a generation comes from the last Fill
                    first_states.append(last_hidden_state)
                    first_configs.append(job.sampling_config)
                    first_jobs.append(job)
                    job.context.last_hidden_state = None
        if first_states:
            tokens = self.model.sampler(torch.stack(first_states), first_configs).cpu().tolist()
            for job, tok in zip(first_jobs, tokens):
                job.put_token(tok)

        iteration_state = IterationState(jobs, self.hf_model_config, self.builtin_config)

        input_ids: List[int] = []
        input_positions: List[int] = []
        for job in jobs:
            context_len = job.context.get_context_len()
            if isinstance(job, Fill):
                input_ids.extend(job.token_ids)
                input_positions.extend(range(context_len - len(job.token_ids), context_len))
            else:
                input_ids.append(job.context.get_last_token_id())
                input_positions.append(context_len - 1)
        device = self.builtin_config.device
        input_ids_t = torch.tensor(input_ids, dtype=torch.int64, device=device)
        input_positions_t = torch.tensor(input_positions, dtype=torch.int64, device=device)

        torch.cuda.synchronize()
        st_model = time.perf_counter_ns()
        fill_hidden_states, next_tokens = self.model(input_ids_t, input_positions_t, iteration_state)
        next_tokens = next_tokens.cpu().tolist()
        torch.cuda.synchronize()
        ed_model = time.perf_counter_ns()
        assert fill_hidden_states.shape[0] + len(next_tokens) == len(jobs)

        for i, job in enumerate(jobs):
            if isinstance(job, Fill):
                job.context.last_hidden_state = fill_hidden_states[i]
                job.finish_event.set()
            else:
                job.put_token(next_tokens[i - iteration_state.num_fill_jobs])
                if job.check_stop():
                    job.finish_event.set()
        return time.perf_counter_ns() - st, ed_model - st_model
