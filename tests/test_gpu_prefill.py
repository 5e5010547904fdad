"""GPU parity of prefill-with-parent-context (packed ragged chunks, bottom-right
causal over scattered parent slots) against the CPU oracle."""
import pytest
import torch

from oracle.ref_ops import ref_cos_sin_cache, ref_prefill_with_parent, ref_rope_neox

pytestmark = pytest.mark.gpu

TOL = {torch.float16: dict(atol=2e-3, rtol=1e-2), torch.bfloat16: dict(atol=1e-2, rtol=2e-2)}


def run_prefill_case(case, dev, fused_path=True):
    """RoPE on new q/k -> append -> attention, on the GPU; returns (out, oracle_out)."""
    from parrotserve_amd import kernels, synth

    T, H, D = case.q.shape
    cache = ref_cos_sin_cache(int(case.positions.max()) + 1, D, case.theta, case.dtype)
    # oracle: rotate with the reference kernel's arithmetic, then attention over parents || own
    rq, rk = ref_rope_neox(case.positions, case.q.reshape(T, -1), case.k_new.reshape(T, -1), cache, D,
                           elem_rounding=True)
    rq, rk = rq.view(T, H, D), rk.view(T, H, D)
    k_all = torch.cat([case.k_rows, rk])
    v_all = torch.cat([case.v_rows, case.v_new])
    ctx = [torch.cat([p, n]) for p, n in zip(case.parent_lists, case.new_lists)]
    ref = ref_prefill_with_parent(rq, k_all, v_all, case.q_lens, ctx)

    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    q, k, v = case.q.to(dev), case.k_new.to(dev), case.v_new.to(dev)
    kernels.vllm_rotary_emb(case.positions.to(dev), q.view(T, -1), k.view(T, -1), cache.to(dev), D)
    new_slots = torch.cat([case.used_slots[n] for n in case.new_lists]).to(torch.int32).to(dev)
    kernels.vllm_reshape_and_cache(k, v, kc, vc, new_slots)
    tables = kernels.PrefillTables.build(case.q_lens, [case.used_slots[c].tolist() for c in ctx], dev)
    out = kernels.prefill_attention(q, kc, vc, tables)
    torch.cuda.synchronize()
    return out.cpu(), ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("q_lens,parent,H", [([5, 1, 70, 33], 100, 4), ([64, 128, 17], 0, 8), ([200], 333, 2),
                                             ([1, 1, 1], 50, 40)])
def test_prefill_small(dev, dtype, q_lens, parent, H):
    from parrotserve_amd import synth

    case = synth.make_prefill_case("p", 21 + parent, dtype, q_lens, parent, H, 128, 1 << 13)
    out, ref = run_prefill_case(case, dev)
    torch.testing.assert_close(out.float(), ref.float(), **TOL[dtype])


def test_config4_scaled(dev):
    """Config 4's recipe (bf16, 40x128, ragged chunks over 2048-token parents, RoPE theta 1e4, seed 3)
    on 4 of the 16 chunks with chunk lengths U[64,256]."""
    from parrotserve_amd import synth

    case = synth.config4(chunks=4, lo=64, hi=256, parent=2048, pool_slots=1 << 15)
    assert case.dtype == torch.bfloat16 and case.q.shape[1:] == (40, 128)
    out, ref = run_prefill_case(case, dev)
    torch.testing.assert_close(out.float(), ref.float(), **TOL[torch.bfloat16])
