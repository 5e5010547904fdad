"""End-to-end: the engine's iteration loop (shared Fill -> forked Fills -> Generate iterations) on the HIP
attention path against the flat-sequence CPU oracle of the same model."""
import pytest
import torch

from oracle.ref_llama import ref_llama_hidden

pytestmark = pytest.mark.gpu


def _set_weights(model, seed):
    """Random weights with O(1) activations (the dummy U(-1e-3, 1e-3) weights give near-uniform attention);
    returns them as the oracle's dict, rounded to fp16 like the model's."""
    g = torch.Generator().manual_seed(seed)
    w = {}

    def put(param, value, key):
        param.data.copy_(value.to(param.dtype))
        w[key] = param.data.detach().cpu().float()

    m = model.model
    put(m.embed_tokens.weight, torch.randn(m.embed_tokens.weight.shape, generator=g), "embed")
    put(m.norm.weight, 1 + 0.1 * torch.randn(m.norm.weight.shape, generator=g), "norm")
    for i, layer in enumerate(m.layers):
        put(layer.input_layernorm.weight, 1 + 0.1 * torch.randn(m.norm.weight.shape, generator=g), f"l{i}.ln1")
        put(layer.post_attention_layernorm.weight, 1 + 0.1 * torch.randn(m.norm.weight.shape, generator=g), f"l{i}.ln2")
        for name, lin in (("qkv", layer.self_attn.qkv_proj), ("o", layer.self_attn.o_proj),
                          ("gate", layer.mlp.gate_proj), ("up", layer.mlp.up_proj), ("down", layer.mlp.down_proj)):
            put(lin.weight, 0.08 * torch.randn(lin.weight.shape, generator=g), f"l{i}.{name}")
    put(model.lm_head.weight, 0.5 * torch.randn(model.lm_head.weight.shape, generator=g), "lm_head")
    return w


@pytest.mark.parametrize("attn_func,fused,forked", [("xformers_fill_shared_prompts_generate", False, False),
                                                    ("hip_shared_prefix", False, False),
                                                    ("hip_shared_prefix", True, False),
                                                    ("hip_shared_prefix", True, True)])
def test_shared_prompt_generation_loop_matches_flat_oracle(dev, attn_func, fused, forked, monkeypatch):
    """The scenario of the reference's decode benchmark (benchmark/bench_kernel.py:11-66), small: one shared
    Fill, B forked Fills, then Generate iterations on the forked contexts.  Every hidden state handed to the
    sampler must equal the oracle's hidden state of the same token in the branch's flat sequence, and every
    sampled token the oracle's arg-max wherever its margin is clear of fp16 noise.  ``forked``: the B forked Fills run
    as a shared-prefix decode over their new tokens instead of through the prefill kernel."""
    from parrotserve_amd.attn_func import BuiltinConfig
    from parrotserve_amd.primitive_job import Fill, Generate
    from parrotserve_amd.runner import BuiltinRunner, LlamaConfig, SamplingConfig

    V, N, H, L, Fdim = 211, 256, 2, 2, 384
    B, shared_len, diverged_len, output_len = 6, 40, 5, 7
    mc = LlamaConfig(vocab_size=V, hidden_size=N, intermediate_size=Fdim, num_hidden_layers=L, num_attention_heads=H,
                     rms_norm_eps=1e-6, max_position_embeddings=256, fused_ops=fused)
    cfg = BuiltinConfig(num_kv_cache_blocks=2048, attn_func=attn_func, dtype=torch.float16, device=dev)
    if forked:  # the forked Fills of this scenario (5-7 tokens over the 40-token parent) take the shared-prefix path
        monkeypatch.setattr(cfg.attn_func, "forked_fill_min_parent", 16)
        monkeypatch.setattr(cfg.attn_func, "forked_fill_pay_ratio", 0)  # taken whatever it saves
    cfg.attn_func.table_cache.clear()
    hits0 = cfg.attn_func.table_cache.hits
    runner = BuiltinRunner(mc, cfg, dummy_weights=False)
    w = _set_weights(runner.model, 7)
    seen = []
    runner.model.sampler.register_forward_pre_hook(lambda mod, args: seen.append(args[0].detach().float().cpu()))

    g = torch.Generator().manual_seed(11)
    shared = torch.randint(0, V, (shared_len,), generator=g).tolist()
    diverged = [torch.randint(0, V, (diverged_len + b % 3,), generator=g).tolist() for b in range(B)]
    sc = SamplingConfig(top_p=1e-6, max_gen_length=output_len)  # only the most likely token survives top-p
    runner.run_iter([Fill(0, 0, 0, -1, token_ids=shared)])
    runner.run_iter([Fill(0, 0, b + 1, 0, token_ids=diverged[b]) for b in range(B)])
    gens = [Generate(0, 0, b + 1, 0, sampling_config=sc) for b in range(B)]
    for _ in range(output_len - 1):  # the first token comes from the Fill's last hidden state
        runner.run_iter(gens)
    assert all(j.finish_event.is_set() and j.gen_length == output_len for j in gens)
    hits = cfg.attn_func.table_cache.hits - hits0
    assert hits == output_len - 2  # every Generate iteration after the first reused the cached tables

    # seen: [first sampling (B rows)], then per iteration B rows; empty calls (Fill-only iterations) have 0 rows
    rows = [s for s in seen if s.shape[0] > 0]
    assert len(rows) == output_len and all(r.shape == (B, N) for r in rows)
    clear = 0
    for b, job in enumerate(gens):
        produced = list(job.output_queue)
        assert produced == job.context.token_ids[len(diverged[b]):] and len(produced) == output_len
        seq = shared + diverged[b] + produced
        hid = ref_llama_hidden(w, seq[:-1], H, 1e-6, cache_dtype=torch.float16)
        first = shared_len + len(diverged[b]) - 1
        for s in range(output_len):
            torch.testing.assert_close(rows[s][b], hid[first + s], atol=3e-2, rtol=3e-2)
            logits = hid[first + s] @ w["lm_head"].t()
            top2 = logits.topk(2)
            if top2.values[0] - top2.values[1] > 0.25:
                clear += 1
                assert produced[s] == int(top2.indices[0])
    assert clear >= B * output_len // 2  # the margin filter must not hollow out the token check
    cfg.attn_func.table_cache.clear()


@pytest.mark.parametrize("attn_func", ["xformers_fill_shared_prompts_generate", "hip_shared_prefix"])
def test_two_level_shared_prompts_match_flat_oracle(dev, attn_func):
    """The reference's two-level scenario (tests/engine/builtin/test_shared_prefix.py:57-115), small: a context, a child
    of it, B Fills of different lengths forked from the child, and every Generate job in a fresh context under its own
    Fill's context -- so no two jobs share a fork parent, and what they share is the grandparent chain.  Hidden
    states and tokens against the flat-sequence oracle; the grouped plug-in must find the same shared prefix as the
    reference's rule (the chain of the two upper contexts)."""
    from parrotserve_amd.attn_func import BuiltinConfig, build_iteration_tables
    from parrotserve_amd.primitive_job import Fill, Generate
    from parrotserve_amd.runner import BuiltinRunner, LlamaConfig, SamplingConfig

    V, N, H, L, Fdim = 211, 256, 2, 2, 384
    B, len1, len2, output_len = 5, 20, 10, 6
    mc = LlamaConfig(vocab_size=V, hidden_size=N, intermediate_size=Fdim, num_hidden_layers=L, num_attention_heads=H,
                     rms_norm_eps=1e-6, max_position_embeddings=256)
    cfg = BuiltinConfig(num_kv_cache_blocks=2048, attn_func=attn_func, dtype=torch.float16, device=dev)
    cfg.attn_func.table_cache.clear()
    runner = BuiltinRunner(mc, cfg, dummy_weights=False)
    w = _set_weights(runner.model, 9)
    seen = []
    runner.model.sampler.register_forward_pre_hook(lambda mod, args: seen.append(args[0].detach().float().cpu()))

    g = torch.Generator().manual_seed(13)
    top = torch.randint(0, V, (len1,), generator=g).tolist()
    mid = torch.randint(0, V, (len2,), generator=g).tolist()
    diverged = [torch.randint(0, V, (3 * (b + 1),), generator=g).tolist() for b in range(B)]
    sc = SamplingConfig(top_p=1e-6, max_gen_length=output_len)
    runner.run_iter([Fill(0, 0, 0, -1, token_ids=top)])
    runner.run_iter([Fill(0, 0, 1, 0, token_ids=mid)])
    runner.run_iter([Fill(0, 0, b + 2, 1, token_ids=diverged[b]) for b in range(B)])
    gens = [Generate(0, 0, b + 2 + B, b + 2, sampling_config=sc) for b in range(B)]
    for it in range(output_len - 1):
        runner.run_iter(gens)
        if it == 0:  # both rules see the same 30 shared tokens; the grouped rule puts every job into that one group
            lca = build_iteration_tables(gens, "lca")
            par = build_iteration_tables(gens, "parent")
            assert lca.flash_context_len == len1 + len2
            assert len(par.groups) == 1 and par.groups[0][0] == lca.flash_block_table
            assert sorted(par.groups[0][1]) == list(range(B)) and par.paged_block_tables == lca.paged_block_tables
    assert all(j.finish_event.is_set() and j.gen_length == output_len for j in gens)

    rows = [s for s in seen if s.shape[0] > 0]
    assert len(rows) == output_len and all(r.shape == (B, N) for r in rows)
    clear = 0
    for b, job in enumerate(gens):
        produced = list(job.output_queue)
        assert produced == job.context.token_ids and len(produced) == output_len
        seq = top + mid + diverged[b] + produced
        hid = ref_llama_hidden(w, seq[:-1], H, 1e-6, cache_dtype=torch.float16)
        first = len1 + len2 + len(diverged[b]) - 1
        for s in range(output_len):
            torch.testing.assert_close(rows[s][b], hid[first + s], atol=3e-2, rtol=3e-2)
            logits = hid[first + s] @ w["lm_head"].t()
            top2 = logits.topk(2)
            if top2.values[0] - top2.values[1] > 0.25:
                clear += 1
                assert produced[s] == int(top2.indices[0])
    assert clear >= B * output_len // 2
    cfg.attn_func.table_cache.clear()


@pytest.mark.parametrize("attn_func", ["xformers_with_buffer", "hip_shared_prefix"])
def test_staggered_fills_and_generates_match_flat_oracle(dev, attn_func):
    """The reference's mixed scenario (parrot/testing/model_runner_test_template.py:148-190): three unrelated
    requests arrive one iteration apart, so iterations hold a Fill next to running Generate jobs and the batch
    changes from one iteration to the next (the cached slot tables must be rebuilt each time it does)."""
    from parrotserve_amd.attn_func import BuiltinConfig
    from parrotserve_amd.primitive_job import Fill, Generate
    from parrotserve_amd.runner import BuiltinRunner, LlamaConfig, SamplingConfig

    V, N, H, L, Fdim = 211, 256, 2, 2, 384
    mc = LlamaConfig(vocab_size=V, hidden_size=N, intermediate_size=Fdim, num_hidden_layers=L, num_attention_heads=H,
                     rms_norm_eps=1e-6, max_position_embeddings=256)
    cfg = BuiltinConfig(num_kv_cache_blocks=2048, attn_func=attn_func, dtype=torch.float16, device=dev)
    cfg.attn_func.table_cache.clear()
    runner = BuiltinRunner(mc, cfg, dummy_weights=False)
    w = _set_weights(runner.model, 5)
    g = torch.Generator().manual_seed(17)
    prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (9, 33, 17)]
    sc = SamplingConfig(top_p=1e-6, max_gen_length=8)
    fills = [Fill(0, i, i, -1, token_ids=prompts[i]) for i in range(3)]
    gens = [Generate(0, i, i, -1, sampling_config=sc) for i in range(3)]
    runner.run_iter([fills[0]])
    runner.run_iter([gens[0], fills[1]])
    runner.run_iter([gens[0], gens[1], fills[2]])
    for _ in range(4):
        runner.run_iter([gens[0], gens[1], gens[2]])
    for i, job in enumerate(gens):
        produced = list(job.output_queue)
        assert len(produced) == [7, 6, 5][i] and job.context.token_ids == prompts[i] + produced
        seq = prompts[i] + produced
        hid = ref_llama_hidden(w, seq[:-1], H, 1e-6, cache_dtype=torch.float16)
        clear = 0
        for s, tok in enumerate(produced):
            logits = hid[len(prompts[i]) - 1 + s] @ w["lm_head"].t()
            top2 = logits.topk(2)
            if top2.values[0] - top2.values[1] > 0.25:
                clear += 1
                assert tok == int(top2.indices[0]), (i, s)
        assert clear >= len(produced) // 2
    cfg.attn_func.table_cache.clear()
