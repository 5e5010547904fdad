"""GPU parity of the AttnFunc plug-in and the decoder-layer wiring against the CPU oracle."""
import pytest
import torch

from oracle.ref_ops import (ref_cos_sin_cache, ref_decode_attention, ref_prefill_with_parent, ref_rms_norm,
                            ref_rope_neox)

pytestmark = pytest.mark.gpu

TOL = dict(atol=2e-3, rtol=1e-2)


class _Cfg:
    def __init__(self, heads, hidden):
        self.num_attention_heads = heads
        self.hidden_size = hidden


def _build_forest(pool, rng_seed, n_groups, branches, prefix, with_fills):
    """parents (already filled) -> forked children; returns jobs in engine order (Fill first)."""
    from parrotserve_amd.context import BlockContext
    from parrotserve_amd.primitive_job import Fill, Generate

    g = torch.Generator().manual_seed(rng_seed)
    cid = 0
    fills, gens = [], []
    for gi in range(n_groups):
        parent = BlockContext(cid, None, pool, 1)
        cid += 1
        parent.allocate(prefix + 7 * gi)
        for b in range(branches):
            child = BlockContext(cid, parent, pool, 1)
            cid += 1
            child.allocate(int(torch.randint(1, 30, (1,), generator=g)))
            job = Generate(0, cid, child.context_id, parent.context_id, sampling_config=None)
            job.context = child
            gens.append(job)
        if with_fills:
            child = BlockContext(cid, parent, pool, 1)
            cid += 1
            n = int(torch.randint(1, 50, (1,), generator=g))
            child.allocate(n)
            job = Fill(0, cid, child.context_id, parent.context_id, token_ids=list(range(n)))
            job.context = child
            fills.append(job)
    # interleave groups among the generates so that grouping has to reorder them
    perm = torch.randperm(len(gens), generator=g).tolist()
    return fills + [gens[i] for i in perm]


@pytest.mark.parametrize("name", ["xformers_fill_shared_prompts_generate", "hip_shared_prefix"])
@pytest.mark.parametrize("n_groups,with_fills", [(1, False), (1, True), (3, True)])
def test_attn_func_forward_matches_oracle(dev, name, n_groups, with_fills):
    from parrotserve_amd import mem
    from parrotserve_amd.attn_func import BuiltinConfig
    from parrotserve_amd.context import RecyclePool
    from parrotserve_amd.iter_state import IterationState
    from parrotserve_amd.primitive_job import Fill

    H, D, slots = 8, 128, 4096
    pool = RecyclePool(pool_size=slots)
    jobs = _build_forest(pool, 5 + n_groups, n_groups, 6, 150, with_fills)
    cfg = BuiltinConfig(num_kv_cache_blocks=slots, attn_func=name, dtype=torch.float16, device=dev)
    store = mem.init_model_cache_storage(2, slots, H, D, torch.float16, dev)
    g = torch.Generator().manual_seed(3)
    kc_cpu = torch.randn(slots, H, D, generator=g).half()
    vc_cpu = torch.randn(slots, H, D, generator=g).half()
    store.k_cache[1].copy_(kc_cpu)
    store.v_cache[1].copy_(vc_cpu)

    st = IterationState(jobs, _Cfg(H, H * D), cfg)
    n_new = [len(j.token_ids) if isinstance(j, Fill) else 1 for j in jobs]
    T = sum(n_new)
    assert st.num_total_fill_tokens + st.num_generation_jobs == T
    qkv = torch.randn(T, 3 * H * D, generator=g).half()
    q, k, v = (t.view(T, H, D) for t in qkv.chunk(3, dim=-1))  # strided views, as the model passes them

    # oracle: append, then per job attention over its whole context
    kc_ref, vc_ref = kc_cpu.clone(), vc_cpu.clone()
    pos = 0
    ref = torch.zeros(T, H, D, dtype=torch.float16)
    for j, n in zip(jobs, n_new):
        sl = torch.tensor(j.context.get_context_slot_ids())
        kc_ref[sl[-n:]] = k[pos : pos + n]
        vc_ref[sl[-n:]] = v[pos : pos + n]
        pos += n
    pos = 0
    for j, n in zip(jobs, n_new):
        sl = torch.tensor(j.context.get_context_slot_ids())
        if isinstance(j, Fill):
            ref[pos : pos + n] = ref_prefill_with_parent(q[pos : pos + n], kc_ref, vc_ref, [n], [sl])
        else:
            ref[pos : pos + 1] = ref_decode_attention(q[pos : pos + 1], kc_ref, vc_ref, [sl])
        pos += n

    attn = cfg.attn_func(layer_idx=1, scaling=D ** -0.5, num_heads=H, head_dim=D)
    dq = qkv.to(dev)
    q_d, k_d, v_d = (t.view(T, H, D) for t in dq.chunk(3, dim=-1))
    out = attn(q_d, k_d, v_d, st)
    assert out.shape == (T, H * D)
    torch.testing.assert_close(out.cpu().view(T, H, D).float(), ref.float(), **TOL)
    # the append really happened, bit-exact, and only at the new tokens' slots
    assert torch.equal(store.k_cache[1].cpu().view(torch.int16), kc_ref.view(torch.int16))
    assert torch.equal(store.v_cache[1].cpu().view(torch.int16), vc_ref.view(torch.int16))


def _check_config5_layer(dev, case, groups, branches, prefix, hidden, H, ffn, fused_ops, oracle_reqs=None,
                         gemm_rows=None):
    """One decoder layer of config 5's recipe on the GPU, stage by stage, each HIP op checked on the inputs it
    really saw: RMSNorm, RoPE (bit-exact), append (bit-exact) and attention against the oracle; the stages behind
    the library GEMMs against an fp32 CPU evaluation that takes the checked attention output.  ``oracle_reqs`` /
    ``gemm_rows``: the requests (rows) the attention oracle / the CPU GEMMs are evaluated on (default: all)."""
    from parrotserve_amd import mem
    from parrotserve_amd.attn_func import BuiltinConfig
    from parrotserve_amd.context import BlockContext, RecyclePool
    from parrotserve_amd.iter_state import IterationState
    from parrotserve_amd.kernels import rope_and_cache, vllm_rotary_emb
    from parrotserve_amd import synth
    from parrotserve_amd.llama_layer import LlamaDecoderLayer
    from parrotserve_amd.primitive_job import Generate

    dec = case.decode
    B, D = dec.num_reqs, 128
    slots = dec.pool_slots
    max_pos = int(case.positions.max()) + 1
    store = mem.init_model_cache_storage(1, slots, H, D, torch.float16, dev, max_seq_len=max_pos, rope_theta=case.theta)
    kc, vc = synth.pool_to_device(dec.k_rows, dec.v_rows, dec.used_slots, slots, dev)
    store.k_cache[0].copy_(kc)
    store.v_cache[0].copy_(vc)

    # contexts whose slot lists are exactly the synthetic case's (ids handed out through a scripted pool)
    class _Scripted(RecyclePool):
        def __init__(self, ids):
            super().__init__(pool_size=None)
            self._ids = list(ids)
            self._next = 0

        def allocate(self):
            self._next += 1
            return self._ids[self._next - 1]

    jobs = []
    for gi in range(groups):
        parent = BlockContext(gi, None, _Scripted(dec.used_slots[dec.prefix_lists[gi]].tolist()), 1)
        parent.allocate(prefix)
        for b in range(branches):
            r = gi * branches + b
            ids = dec.used_slots[dec.suffix_lists[r]].tolist()
            child = BlockContext(1000 + r, parent, _Scripted(ids), 1)
            child.allocate(len(ids))
            j = Generate(0, r, child.context_id, parent.context_id)
            j.context = child
            jobs.append(j)
    cfg = BuiltinConfig(num_kv_cache_blocks=slots, attn_func="hip_shared_prefix", dtype=torch.float16, device=dev)
    st = IterationState(jobs, type("C", (), dict(num_attention_heads=H, hidden_size=hidden))(), cfg)
    assert st.decode_tables.num_groups == groups and st.decode_perm is None

    layer = LlamaDecoderLayer(hidden, H, ffn, case.eps, 0, cfg.attn_func, fused_ops=fused_ops).half().to(dev)
    w = case.weights
    with torch.no_grad():
        layer.self_attn.qkv_proj.weight.copy_(w["qkv_proj"])
        layer.self_attn.o_proj.weight.copy_(w["o_proj"])
        layer.mlp.gate_proj.weight.copy_(w["gate_proj"])
        layer.mlp.up_proj.weight.copy_(w["up_proj"])
        layer.mlp.down_proj.weight.copy_(w["down_proj"])
    x = case.x.to(dev)
    pos = case.positions.to(dev)

    # GPU, stage by stage (the calls LlamaAttention.forward makes for this setting of fused_ops)
    with torch.inference_mode():
        h1 = layer.input_layernorm(x)
        qkv = layer.self_attn.qkv_proj(h1)
        qkv_before = qkv.clone()
        q, k, v = torch.chunk(qkv, 3, dim=-1)
        if fused_ops:
            rope_and_cache(pos, q, k, v, mem.get_cos_sin_cache(), D, mem.get_k_cache(0), mem.get_v_cache(0),
                           st.slot_mapping, key_in_place=False)
            attn_out = layer.self_attn.attn_func(q.view(B, H, D), k.view(B, H, D), v.view(B, H, D), st,
                                                 kv_appended=True)
        else:
            vllm_rotary_emb(pos, q, k, mem.get_cos_sin_cache(), head_size=D)
            attn_out = layer.self_attn.attn_func(q.view(B, H, D), k.view(B, H, D), v.view(B, H, D), st)
        k_cache_after = mem.Model_Cache.k_cache[0].clone()
        v_cache_after = mem.Model_Cache.v_cache[0].clone()
        mem.Model_Cache.k_cache[0].copy_(kc)  # undo the append, then run the whole layer in one go
        mem.Model_Cache.v_cache[0].copy_(vc)
        y = layer(x, pos, st)

    # 1. RMSNorm
    ref_h1 = ref_rms_norm(case.x, w["input_layernorm"], case.eps)
    torch.testing.assert_close(h1.cpu().float(), ref_h1.float(), **TOL)
    # 2. RoPE on the GPU's own qkv (bit-exact with the reference kernel's arithmetic)
    cache = ref_cos_sin_cache(max_pos, D, case.theta, torch.float16)
    torch.testing.assert_close(mem.get_cos_sin_cache().cpu().float(), cache.float(), atol=1e-3, rtol=0)
    qb, kb, vb = qkv_before.cpu().chunk(3, dim=-1)
    rq, rk = ref_rope_neox(case.positions, qb, kb, mem.get_cos_sin_cache().cpu(), D, elem_rounding=True)
    assert torch.equal(q.cpu().view(torch.int16), rq.contiguous().view(torch.int16))
    if not fused_ops:  # the fused pass writes the rotated k rows to the cache only
        assert torch.equal(k.cpu().view(torch.int16), rk.contiguous().view(torch.int16))
    # 3. append (bit-exact, only at the new tokens' slots) + shared-prefix attention on those q/k/v
    k_rows, v_rows = dec.k_rows.clone(), dec.v_rows.clone()
    for r in range(B):
        last = int(dec.suffix_lists[r][-1])
        k_rows[last] = rk.view(B, H, D)[r]
        v_rows[last] = vb.reshape(B, H, D)[r]
    used = dec.used_slots[: k_rows.shape[0]].to(dev)
    assert torch.equal(k_cache_after[used].cpu().view(torch.int16), k_rows.view(torch.int16))
    assert torch.equal(v_cache_after[used].cpu().view(torch.int16), v_rows.view(torch.int16))
    untouched = torch.ones(slots, dtype=torch.bool, device=dev)
    untouched[used] = False
    assert not k_cache_after[untouched].any() and not v_cache_after[untouched].any()
    pick = list(range(B)) if oracle_reqs is None else list(oracle_reqs)
    full = dec.full_lists()
    ref_attn = ref_decode_attention(rq.view(B, H, D)[pick], k_rows, v_rows, [full[i] for i in pick])
    torch.testing.assert_close(attn_out.cpu().view(B, H, D)[pick].float(), ref_attn.float(), **TOL)
    # 4. whole layer vs an fp32 CPU evaluation that takes the checked attention output
    rows = list(range(B)) if gemm_rows is None else list(gemm_rows)
    a = attn_out.cpu().float()[rows]
    hcpu = case.x.float()[rows] + (a @ w["o_proj"].float().t()).half().float()
    hcpu = hcpu.half()
    h2 = ref_rms_norm(hcpu, w["post_attention_layernorm"], case.eps).float()
    gate = (h2 @ w["gate_proj"].float().t()).half().float()
    up = (h2 @ w["up_proj"].float().t()).half().float()
    act = (torch.nn.functional.silu(gate).half().float() * up).half().float()
    mlp = (act @ w["down_proj"].float().t()).half().float()
    ref_y = (hcpu.float() + mlp).half()
    torch.testing.assert_close(y.cpu()[rows].float(), ref_y.float(), atol=2e-2, rtol=2e-2)
    mem.Model_Cache = None


@pytest.mark.parametrize("fused_ops", [False, True])
def test_decoder_layer_config5_scaled(dev, fused_ops):
    """Config 5's recipe scaled down (fp16, weights N(0, 0.02), RMSNorm -> QKV -> RoPE -> prefix groups x
    branches -> shared-prefix + suffix attention -> O-proj -> MLP): hidden 640, 5 heads x 128, FFN 1728,
    2 groups x 8 branches, prefix 300, suffix U[4,40], seed 4."""
    from parrotserve_amd import synth

    case = synth.config5(groups=2, branches=8, prefix=300, s_lo=4, s_hi=40, hidden=640, heads=5, ffn=1728,
                         pool_slots=1 << 12)
    _check_config5_layer(dev, case, 2, 8, 300, 640, 5, 1728, fused_ops)


_C5_FULL = {}


@pytest.mark.parametrize("fused_ops", [False, True])
def test_decoder_layer_config5_full_size(dev, fused_ops):
    """Config 5 at full size: hidden 5120, 40 heads x 128, FFN 13824, 4 groups x 32 branches over 6000-token
    prefixes, suffix U[32,1024], seed 4.  RMSNorm, RoPE and the append on all 128 rows; the attention oracle on
    twelve requests (three per group, the shortest and longest suffix among them); the stages behind the GEMMs on
    16 sampled rows."""
    from parrotserve_amd import synth

    if "case" not in _C5_FULL:
        _C5_FULL["case"] = synth.config5()
    case = _C5_FULL["case"]
    lens = [l.numel() for l in case.decode.suffix_lists]
    pick = sorted({min(range(128), key=lens.__getitem__), max(range(128), key=lens.__getitem__),
                   0, 17, 31, 32, 50, 63, 64, 95, 100, 127})
    rows = [0, 5, 13, 31, 32, 40, 47, 63, 64, 70, 77, 95, 96, 101, 120, 127]
    _check_config5_layer(dev, case, 4, 32, 6000, 5120, 40, 13824, fused_ops, oracle_reqs=pick, gemm_rows=rows)
    if fused_ops:
        _C5_FULL.clear()


@pytest.mark.parametrize("name,n_groups", [("xformers_fill_shared_prompts_generate", 1), ("hip_shared_prefix", 3)])
def test_incremental_tables_match_full_rebuild_over_a_decode_loop(dev, name, n_groups):
    """A decode loop of 40 iterations: the tables the plug-in patches in place each iteration (one appended slot
    per request, fresh plan) are bit-identical to the ones built from the context trees from scratch, through
    the widening of the padded table, and the attention outputs agree."""
    from parrotserve_amd import mem
    from parrotserve_amd.attn_func import BuiltinConfig, get_attn_func
    from parrotserve_amd.context import RecyclePool
    from parrotserve_amd.iter_state import IterationState
    from parrotserve_amd.table_cache import DecodeTableCache

    H, D, slots = 8, 128, 8192
    pool = RecyclePool(pool_size=slots)
    jobs = _build_forest(pool, 17 + n_groups, n_groups, 5, 200, with_fills=False)
    base = get_attn_func(name)

    class Inc(base):  # own cache, so other tests' batches do not interfere
        table_cache = DecodeTableCache()

    class Fresh(base):  # the cache switched off: rebuilds everything every iteration
        incremental = False

    cfg_inc = BuiltinConfig(num_kv_cache_blocks=slots, attn_func=Inc, dtype=torch.float16, device=dev)
    cfg_full = BuiltinConfig(num_kv_cache_blocks=slots, attn_func=Fresh, dtype=torch.float16, device=dev)
    store = mem.init_model_cache_storage(1, slots, H, D, torch.float16, dev)
    g = torch.Generator(device=dev).manual_seed(9)
    store.k_cache[0].normal_(generator=g)
    store.v_cache[0].normal_(generator=g)
    attn_inc = Inc(layer_idx=0, scaling=D ** -0.5, num_heads=H, head_dim=D)
    attn_full = Fresh(layer_idx=0, scaling=D ** -0.5, num_heads=H, head_dim=D)
    B = len(jobs)
    for it in range(40):
        for j in jobs:
            j.context.allocate(1)
        st_i = IterationState(jobs, _Cfg(H, H * D), cfg_inc)
        st_f = IterationState(jobs, _Cfg(H, H * D), cfg_full)
        assert (st_i.tables is None) == (it > 0)  # every iteration after the first came from the cache
        assert st_f.tables is not None
        ti, tf = st_i.decode_tables, st_f.decode_tables
        assert torch.equal(st_i.slot_mapping, st_f.slot_mapping)
        assert torch.equal(ti.suffix_lens, tf.suffix_lens) and ti.max_suffix_len == tf.max_suffix_len
        w = tf.suffix_slots.shape[1]
        assert ti.suffix_slots.shape[1] >= w
        cols = torch.arange(w, device=dev)[None, :] < tf.suffix_lens[:, None]
        assert torch.equal(torch.where(cols, ti.suffix_slots[:, :w], 0), torch.where(cols, tf.suffix_slots, 0))
        assert torch.equal(ti.plan_req_item_cu, tf.plan_req_item_cu)
        n_items = int(tf.plan_req_item_cu[-1])  # rows of the item array in use (the rest keeps older contents)
        assert torch.equal(ti.plan_items[:n_items], tf.plan_items[:n_items])
        assert torch.equal(ti.plan_lane_item_cu, tf.plan_lane_item_cu)
        assert (st_i.decode_perm is None) == (st_f.decode_perm is None)
        if st_i.decode_perm is not None:
            assert torch.equal(st_i.decode_perm[0], st_f.decode_perm[0])
        if it % 13 == 0 or it == 39:
            qkv = torch.randn(B, 3 * H * D, generator=g, device=dev, dtype=torch.float16)
            q, k, v = (t.view(B, H, D) for t in qkv.chunk(3, dim=-1))
            o_i = attn_inc(q, k, v, st_i)
            o_f = attn_full(q, k, v, st_f)  # appends the same rows again: idempotent
            assert torch.equal(o_i, o_f)
    assert Inc.table_cache.hits == 39 and Inc.table_cache.rebuilds == 1


@pytest.mark.parametrize("seed", range(10))
def test_device_suffix_plan_equals_the_host_plan(dev, seed):
    """ph_suffix_plan_build against the numpy planner: same items, lane records and per-request offsets, for ragged
    batches with empty requests, fewer tokens than lanes, one request, and lengths that are multiples of the cut."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(50 + seed)
    B = [1, 2, 7, 64, 64, 200, 333, 1000, 5, 8192][seed]
    hi = [5000, 40, 3, 512, 16, 2000, 100, 64, 8192, 30][seed]
    lens = torch.randint(0, hi + 1, (B,), generator=g)
    if seed in (2, 6):
        lens[torch.rand(B, generator=g) < 0.4] = 0
    if seed == 4:
        lens[:] = 16
    lanes_cap = [256, 256, 256, 256, 512, 128, 2048, 37, 256, 256][seed]
    total = int(lens.sum())
    items = torch.full(((lanes_cap + B), 4), -1, dtype=torch.int32, device=dev)
    rec = torch.full((lanes_cap, 8), -1, dtype=torch.int32, device=dev)
    rcu = torch.full((B + 1,), -1, dtype=torch.int32, device=dev)
    kernels.suffix_plan_build(lens.to(torch.int32).to(dev), lanes_cap, items, rec, rcu)
    lanes = max(1, min(lanes_cap, (total + 3) // 4))
    h_items, h_lane_cu, h_rcu = kernels.plan_suffix_items(lens.tolist(), lanes)
    n = h_items.shape[0]
    assert torch.equal(rcu.cpu(), torch.from_numpy(h_rcu))
    assert torch.equal(items[:n].cpu(), torch.from_numpy(h_items))
    rec = rec.cpu()
    eff = h_lane_cu.shape[0] - 1
    if n:
        assert torch.equal(rec[:eff, 0], torch.from_numpy(h_lane_cu[:-1]))
        assert torch.equal(rec[:eff, 1], torch.from_numpy(h_lane_cu[1:] - h_lane_cu[:-1]))
        assert torch.equal(rec[:eff, 2:5], torch.from_numpy(h_items[h_lane_cu[:-1], 0:3]))
    assert (rec[eff:, 1] == 0).all()  # lanes beyond the cut count own nothing


@pytest.mark.parametrize("name", ["xformers_fill_shared_prompts_generate", "hip_shared_prefix"])
@pytest.mark.parametrize("n_parents,chunks,own_prev", [(1, 9, 0), (3, 4, 0), (2, 70, 5)])
def test_forked_fills_run_as_shared_prefix_decode(dev, name, n_parents, chunks, own_prev):
    """Fill jobs forked from shared parents (short chunks over long parents): the plug-in hands their new tokens to
    the shared-prefix decode path; results against the oracle's prefill with parent context, for one and several
    parents, for more than 256 new tokens under one parent (two query tiles), for chunks that continue an own
    context, and mixed with Generate jobs in the same iteration."""
    from parrotserve_amd import mem
    from parrotserve_amd.attn_func import BuiltinConfig
    from parrotserve_amd.context import BlockContext, RecyclePool
    from parrotserve_amd.iter_state import IterationState
    from parrotserve_amd.primitive_job import Fill, Generate

    H, D, slots = 4, 128, 8192
    pool = RecyclePool(pool_size=slots)
    g = torch.Generator().manual_seed(70 + chunks)
    fills, gens, cid = [], [], 0
    for pi in range(n_parents):
        parent = BlockContext(cid, None, pool, 1)
        cid += 1
        parent.allocate(300 + 41 * pi)
        for c in range(chunks):
            child = BlockContext(cid, parent, pool, 1)
            cid += 1
            n = int(torch.randint(1, 12, (1,), generator=g))
            child.allocate(own_prev + n)  # an own context of own_prev older tokens, then the chunk
            job = Fill(0, cid, child.context_id, parent.context_id, token_ids=list(range(n)))
            job.context = child
            fills.append(job)
        child = BlockContext(cid, parent, pool, 1)
        cid += 1
        child.allocate(7)
        job = Generate(0, cid, child.context_id, parent.context_id, sampling_config=None)
        job.context = child
        gens.append(job)
    jobs = fills + gens
    cfg = BuiltinConfig(num_kv_cache_blocks=slots, attn_func=name, dtype=torch.float16, device=dev)
    cfg.attn_func.table_cache.clear()
    store = mem.init_model_cache_storage(1, slots, H, D, torch.float16, dev)
    kc_cpu = torch.randn(slots, H, D, generator=g).half()
    vc_cpu = torch.randn(slots, H, D, generator=g).half()
    store.k_cache[0].copy_(kc_cpu)
    store.v_cache[0].copy_(vc_cpu)
    st = IterationState(jobs, _Cfg(H, H * D), cfg)
    assert st.fill_decode_tables is not None and st.fill_tables is None  # the forked form was chosen
    n_new = [len(j.token_ids) if isinstance(j, Fill) else 1 for j in jobs]
    T = sum(n_new)
    qkv = torch.randn(T, 3 * H * D, generator=g).half()
    q, k, v = (t.view(T, H, D) for t in qkv.chunk(3, dim=-1))
    kc_ref, vc_ref = kc_cpu.clone(), vc_cpu.clone()
    pos = 0
    for j, n in zip(jobs, n_new):
        sl = torch.tensor(j.context.get_context_slot_ids())
        kc_ref[sl[-n:]] = k[pos:pos + n]
        vc_ref[sl[-n:]] = v[pos:pos + n]
        pos += n
    ref = torch.zeros(T, H, D, dtype=torch.float16)
    pos = 0
    for j, n in zip(jobs, n_new):
        sl = torch.tensor(j.context.get_context_slot_ids())
        if isinstance(j, Fill):
            ref[pos:pos + n] = ref_prefill_with_parent(q[pos:pos + n], kc_ref, vc_ref, [n], [sl])
        else:
            ref[pos:pos + 1] = ref_decode_attention(q[pos:pos + 1], kc_ref, vc_ref, [sl])
        pos += n
    attn = cfg.attn_func(layer_idx=0, scaling=D ** -0.5, num_heads=H, head_dim=D)
    q_d, k_d, v_d = (t.view(T, H, D) for t in qkv.to(dev).chunk(3, dim=-1))
    out = attn(q_d, k_d, v_d, st)
    torch.testing.assert_close(out.cpu().view(T, H, D).float(), ref.float(), **TOL)
    # the same iteration with the forked form switched off takes the prefill kernel and agrees
    class Plain(cfg.attn_func):
        forked_fill_min_parent = 0
    cfg2 = BuiltinConfig(num_kv_cache_blocks=slots, attn_func=Plain, dtype=torch.float16, device=dev)
    st2 = IterationState(jobs, _Cfg(H, H * D), cfg2)
    assert st2.fill_decode_tables is None and st2.fill_tables is not None
    out2 = Plain(layer_idx=0, scaling=D ** -0.5, num_heads=H, head_dim=D)(q_d, k_d, v_d, st2)
    torch.testing.assert_close(out2.cpu().view(T, H, D).float(), ref.float(), **TOL)
    cfg.attn_func.table_cache.clear()
    mem.Model_Cache = None
