"""GPU parity in float32, the second element type the reference's configuration offers
(parrot/engine/config.py:22-25): BASELINE config 1 at its own precision, the reference-named entry points, the two
orders of the split prefix / suffix pair, prefill with parent context, token move / KV append (bit-exact), rotary
embedding and RMSNorm, each against the CPU oracle on identical seeded inputs.

Tolerance: atol 2e-5, rtol 1e-4 for attention and RMSNorm (fp32 sums of a few hundred to a few thousand terms in a
different order than the oracle's, hardware exp2), bit-exact for copies and for the rotary products."""
import pytest
import torch

from oracle.ref_ops import (ref_cos_sin_cache, ref_decode_attention, ref_kv_append, ref_move_tokens,
                            ref_prefill_with_parent, ref_rms_norm, ref_rope_neox, ref_rotary_embedding)

pytestmark = pytest.mark.gpu

TOL32 = dict(atol=2e-5, rtol=1e-4)


def test_config1_in_fp32(dev):
    """Config 1 as BASELINE states it: fp32, batch 8 forked from one parent, prefix 512, suffix U[32,128], 32 x 128,
    seed 0 -- the shared-prefix path (prefix phase per request on the 32-bit kernel, suffix phase, merge)."""
    from parrotserve_amd import kernels, synth

    c = synth.config1()
    assert c.dtype == torch.float32 and c.q.dtype == torch.float32 and c.num_reqs == 8
    assert c.prefix_lists[0].numel() == 512
    c.pool_slots = 4096
    c.used_slots = torch.randperm(4096, generator=torch.Generator().manual_seed(0))[: c.k_rows.shape[0]]
    kc, vc = synth.pool_to_device(c.k_rows, c.v_rows, c.used_slots, c.pool_slots, dev)
    assert kc.dtype == torch.float32
    ref = ref_decode_attention(c.q, c.k_rows, c.v_rows, c.full_lists())
    for balanced in (True, False):
        t = kernels.DecodeTables.build(c.pool_lists(c.prefix_lists), c.group_req_cu, c.pool_lists(c.suffix_lists), dev,
                                       balanced=balanced)
        out = kernels.decode_attention(c.q.to(dev), kc, vc, t)
        torch.testing.assert_close(out.cpu(), ref, **TOL32)
    # the same requests as plain ragged decode over their whole contexts
    full = [c.used_slots[l].tolist() for l in c.full_lists()]
    t = kernels.DecodeTables.build([], [], full, dev)
    torch.testing.assert_close(kernels.decode_attention(c.q.to(dev), kc, vc, t).cpu(), ref, **TOL32)


@pytest.mark.parametrize("B,P,H,D", [(70, 300, 4, 128), (9, 129, 6, 64), (5, 77, 3, 80), (3, 40, 2, 256)])
def test_reference_named_entry_points_fp32(dev, B, P, H, D):
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(B + D)
    s = torch.randint(0, 70, (B,), generator=g).tolist()
    case = synth.make_decode_case("f32", 50 + B, torch.float32, 1, B, P, s, H, D, 1 << 13)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    suf = case.pool_lists(case.suffix_lists)
    mx = max(1, max(len(x) for x in suf))
    table = torch.tensor([x + [0] * (mx - len(x)) for x in suf], dtype=torch.int32, device=dev)
    lens = torch.tensor([len(x) for x in suf], dtype=torch.int32, device=dev)
    flash = torch.tensor(case.pool_lists(case.prefix_lists)[0], dtype=torch.int32, device=dev)
    hm = torch.arange(H, dtype=torch.int32, device=dev)
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    for fn in (kernels.flash_paged_attention, kernels.paged_flash_attention):
        out = fn(case.q.to(dev), kc, vc, hm, P, flash, lens, table)
        assert out.dtype == torch.float32
        torch.testing.assert_close(out.cpu(), ref, **TOL32)
    full = [case.used_slots[l].tolist() for l in case.full_lists()]
    mx = max(len(x) for x in full)
    ftable = torch.tensor([x + [0] * (mx - len(x)) for x in full], dtype=torch.int32, device=dev)
    flens = torch.tensor([len(x) for x in full], dtype=torch.int32, device=dev)
    out = kernels.vllm_paged_attention(case.q.to(dev), kc, vc, hm, flens, ftable)
    torch.testing.assert_close(out.cpu(), ref, **TOL32)


@pytest.mark.parametrize("q_lens,parent,H,D", [([5, 1, 70, 33], 100, 4, 128), ([64, 17], 0, 3, 64), ([9], 333, 2, 96)])
def test_prefill_with_parent_fp32(dev, q_lens, parent, H, D):
    """Rotary embedding on the new q / k, append, attention over parents || own, all in fp32."""
    from parrotserve_amd import kernels, synth

    case = synth.make_prefill_case("p32", 60 + parent, torch.float32, q_lens, parent, H, D, 1 << 12)
    T = case.q.shape[0]
    cache = ref_cos_sin_cache(int(case.positions.max()) + 1, D, case.theta, torch.float32)
    rq, rk = ref_rope_neox(case.positions, case.q.reshape(T, -1), case.k_new.reshape(T, -1), cache, D, elem_rounding=True)
    rq, rk = rq.view(T, H, D), rk.view(T, H, D)
    k_all, v_all = torch.cat([case.k_rows, rk]), torch.cat([case.v_rows, case.v_new])
    ctx = [torch.cat([p, n]) for p, n in zip(case.parent_lists, case.new_lists)]
    ref = ref_prefill_with_parent(rq, k_all, v_all, case.q_lens, ctx)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    q, k, v = case.q.to(dev), case.k_new.to(dev), case.v_new.to(dev)
    kernels.vllm_rotary_emb(case.positions.to(dev), q.view(T, -1), k.view(T, -1), cache.to(dev), D)
    assert torch.equal(q.cpu().view(torch.int32), rq.view(torch.int32))  # fp32 products and sums, no contraction
    assert torch.equal(k.cpu().view(torch.int32), rk.view(torch.int32))
    new_slots = torch.cat([case.used_slots[n] for n in case.new_lists]).to(torch.int32).to(dev)
    kernels.vllm_reshape_and_cache(k, v, kc, vc, new_slots)
    assert torch.equal(kc[new_slots.long()].cpu().view(torch.int32), rk.view(torch.int32))
    tables = kernels.PrefillTables.build(case.q_lens, [case.used_slots[c].tolist() for c in ctx], dev)
    out = kernels.prefill_attention(q, kc, vc, tables)
    torch.testing.assert_close(out.cpu(), ref, **TOL32)


def test_move_append_rotary_rmsnorm_fp32(dev):
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(77)
    H, D = 5, 128
    src = torch.randn(300, H, D, generator=g)
    dst0 = torch.randn(400, H, D, generator=g)
    si = torch.randint(0, 300, (123,), generator=g)
    di = torch.randperm(400, generator=g)[:123]
    want = dst0.clone()
    ref_move_tokens(src, want, si, di)
    d = dst0.to(dev)
    kernels.discontinuous_move_tokens(src.to(dev), d, si.to(dev), di.to(dev))
    assert torch.equal(d.cpu().view(torch.int32), want.view(torch.int32))
    # append from strided views of a fused projection
    T = 31
    qkv = torch.randn(T, 3 * H * D, generator=g)
    _, k, v = qkv.chunk(3, dim=-1)
    kc0, vc0 = torch.randn(64, H, D, generator=g), torch.randn(64, H, D, generator=g)
    sm = torch.randperm(64, generator=g)[:T]
    kc, vc = kc0.clone(), vc0.clone()
    ref_kv_append(k.view(T, H, D), v.view(T, H, D), kc, vc, sm)
    dq = qkv.to(dev)
    _, dk, dv = dq.chunk(3, dim=-1)
    dkc, dvc = kc0.to(dev), vc0.to(dev)
    kernels.vllm_reshape_and_cache(dk.view(T, H, D), dv.view(T, H, D), dkc, dvc, sm.to(dev))
    assert torch.equal(dkc.cpu().view(torch.int32), kc.view(torch.int32))
    assert torch.equal(dvc.cpu().view(torch.int32), vc.view(torch.int32))
    # rotary_embedding(state, cos, sin) with per-token rows
    state = torch.randn(T, H, D, generator=g)
    ang = torch.rand(T, 1, D // 2, generator=g) * 6.0
    cos, sin = ang.cos(), ang.sin()
    want = ref_rotary_embedding(state, cos, sin, elem_rounding=True)
    st = state.to(dev)
    kernels.rotary_embedding(st, cos.to(dev), sin.to(dev))
    assert torch.equal(st.cpu().view(torch.int32), want.view(torch.int32))
    # RMSNorm: both entry points coincide in fp32
    for rows, n in ((33, 5120), (5, 1000), (2100, 512)):
        x = torch.randn(rows, n, generator=g) * 2 - 0.5
        w = torch.rand(n, generator=g) + 0.5
        ref = ref_rms_norm(x, w, 1e-6, round_before_weight=True)
        for fn in (kernels.vllm_rms_norm, kernels.rmsnorm_forward):
            torch.testing.assert_close(fn(x.to(dev), w.to(dev), 1e-6).cpu(), ref, **TOL32)


def test_fp32_through_the_plug_in_config(dev):
    """``BuiltinConfig(dtype="float32")`` is accepted as in the reference, and the matrix-core-only / fused ops refuse
    fp32 loudly instead of computing in another type."""
    from parrotserve_amd import kernels
    from parrotserve_amd.attn_func import BuiltinConfig

    cfg = BuiltinConfig(num_kv_cache_blocks=64, attn_func="hip_shared_prefix", dtype="float32", device=dev)
    assert cfg.dtype == torch.float32
    x = torch.randn(4, 64, device=dev)
    with pytest.raises(RuntimeError, match="data type"):
        kernels.fused_add_rms_norm(x, x.clone(), torch.ones(64, device=dev), 1e-6)
