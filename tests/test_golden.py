"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the CPU oracle must keep
reproducing them, and the GPU kernels must match them through the same ops the other parity tests use."""
import os

import numpy as np
import pytest
import torch

from oracle.ref_ops import (ref_add_rms_norm, ref_decode_attention, ref_kv_append, ref_move_tokens,
                            ref_prefill_with_parent, ref_rms_norm, ref_rope_neox, ref_silu_mul)

from oracle import ref_sampler

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = {torch.float16: dict(atol=2e-3, rtol=1e-2), torch.bfloat16: dict(atol=1e-2, rtol=2e-2)}
# oracle against its own frozen output: reductions and exp may round differently on another host CPU, so
# floating-point results are held to about one unit in the last place; bit copies and the element-wise
# rotary arithmetic are held bit-exact
ULP = {torch.float16: dict(atol=1e-3, rtol=2e-3), torch.bfloat16: dict(atol=8e-3, rtol=1.6e-2)}


def _close(got, want, dtype):
    torch.testing.assert_close(got.float(), want.float(), **ULP[dtype])


def _load(name):
    return np.load(os.path.join(GOLD, name))  # allow_pickle stays False


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t.view(dtype) if dtype is not None else t


def _decode_inputs(f, dtype):
    q, kc, vc = _t(f["q"], dtype), _t(f["k_cache"], dtype), _t(f["v_cache"], dtype)
    prefix = _t(f["prefix_slots"]).long()
    lens = f["suffix_lens"].tolist()
    suffix = [_t(f["suffix_table"][i, :n]).long() for i, n in enumerate(lens)]
    return q, kc, vc, prefix, suffix, _t(f["out"], dtype)


@pytest.mark.parametrize("name,dtype", [("decode_fp16.npz", torch.float16), ("decode_bf16.npz", torch.bfloat16)])
def test_oracle_reproduces_decode_fixture(name, dtype):
    q, kc, vc, prefix, suffix, want = _decode_inputs(_load(name), dtype)
    got = ref_decode_attention(q, kc, vc, [torch.cat([prefix, s]) for s in suffix])
    _close(got, want, dtype)


def test_oracle_reproduces_prefill_and_elementwise_fixtures():
    f = _load("prefill_bf16.npz")
    dt = torch.bfloat16
    kv = f["kv_lens"].tolist()
    off = np.concatenate([[0], np.cumsum(kv)])
    ctx = [_t(f["ctx_slots"][off[i]:off[i + 1]]).long() for i in range(len(kv))]
    got = ref_prefill_with_parent(_t(f["q"], dt), _t(f["k_cache"], dt), _t(f["v_cache"], dt), f["q_lens"].tolist(), ctx)
    _close(got, _t(f["out"], dt), dt)
    e = _load("elementwise_fp16.npz")
    h = torch.float16
    dst = _t(e["move_dst"], h).clone()
    ref_move_tokens(_t(e["move_src"], h), dst, _t(e["move_sidx"]), _t(e["move_didx"]))
    assert torch.equal(dst.view(torch.int16), _t(e["move_out"], h).view(torch.int16))
    kc, vc = _t(e["app_kc"], h).clone(), _t(e["app_vc"], h).clone()
    ref_kv_append(_t(e["app_k"], h), _t(e["app_v"], h), kc, vc, _t(e["app_slots"]))
    assert torch.equal(kc.view(torch.int16), _t(e["app_kc_out"], h).view(torch.int16))
    assert torch.equal(vc.view(torch.int16), _t(e["app_vc_out"], h).view(torch.int16))
    oq, ok = ref_rope_neox(_t(e["rope_pos"]), _t(e["rope_q"], h), _t(e["rope_k"], h), _t(e["rope_cache"], h), 128, True)
    assert torch.equal(oq.view(torch.int16), _t(e["rope_q_out"], h).view(torch.int16))
    assert torch.equal(ok.view(torch.int16), _t(e["rope_k_out"], h).view(torch.int16))
    x, r, w = _t(e["norm_x"], h), _t(e["norm_r"], h), _t(e["norm_w"], h)
    _close(ref_rms_norm(x, w, 1e-6, True), _t(e["norm_round_first"], h), h)
    _close(ref_rms_norm(x, w, 1e-6, False), _t(e["norm_round_once"], h), h)
    y, hh = ref_add_rms_norm(x, r, w, 1e-6, True)
    _close(y, _t(e["addnorm_y"], h), h)
    assert torch.equal(hh.view(torch.int16), _t(e["addnorm_h"], h).view(torch.int16))
    _close(ref_silu_mul(x, r), _t(e["silu_mul"], h), h)


@pytest.mark.gpu
@pytest.mark.parametrize("name,dtype", [("decode_fp16.npz", torch.float16), ("decode_bf16.npz", torch.bfloat16)])
def test_gpu_decode_matches_fixture(dev, name, dtype):
    from parrotserve_amd import kernels

    q, kc, vc, prefix, suffix, want = _decode_inputs(_load(name), dtype)
    tabs = kernels.DecodeTables.build([prefix.tolist()], [0, q.shape[0]], [s.tolist() for s in suffix], dev,
                                      num_heads=q.shape[1], head_dim=q.shape[2])
    out = kernels.decode_attention(q.to(dev), kc.to(dev), vc.to(dev), tabs)
    torch.testing.assert_close(out.cpu().float(), want.float(), **TOL[dtype])
    # the reference-named entry point on the same tables
    f = _load(name)
    out2 = kernels.flash_paged_attention(q.to(dev), kc.to(dev), vc.to(dev), torch.arange(q.shape[1], device=dev),
                                         prefix.numel(), _t(f["prefix_slots"]).to(dev), _t(f["suffix_lens"]).to(dev),
                                         _t(f["suffix_table"]).to(dev))
    torch.testing.assert_close(out2.cpu().float(), want.float(), **TOL[dtype])


@pytest.mark.gpu
def test_gpu_prefill_and_elementwise_match_fixtures(dev):
    from parrotserve_amd import kernels

    f = _load("prefill_bf16.npz")
    dt = torch.bfloat16
    kv = f["kv_lens"].tolist()
    off = np.concatenate([[0], np.cumsum(kv)])
    ctx = [f["ctx_slots"][off[i]:off[i + 1]].tolist() for i in range(len(kv))]
    tabs = kernels.PrefillTables.build(f["q_lens"].tolist(), ctx, dev)
    out = kernels.prefill_attention(_t(f["q"], dt).to(dev), _t(f["k_cache"], dt).to(dev), _t(f["v_cache"], dt).to(dev), tabs)
    torch.testing.assert_close(out.cpu().float(), _t(f["out"], dt).float(), **TOL[dt])

    e = _load("elementwise_fp16.npz")
    h = torch.float16
    bits = lambda t: t.cpu().contiguous().view(torch.int16)  # noqa: E731
    dst = _t(e["move_dst"], h).to(dev)
    kernels.discontinuous_move_tokens(_t(e["move_src"], h).to(dev), dst, _t(e["move_sidx"]).to(dev), _t(e["move_didx"]).to(dev))
    assert torch.equal(bits(dst), _t(e["move_out"], h).view(torch.int16))
    kc, vc = _t(e["app_kc"], h).to(dev), _t(e["app_vc"], h).to(dev)
    kernels.vllm_reshape_and_cache(_t(e["app_k"], h).to(dev), _t(e["app_v"], h).to(dev), kc, vc, _t(e["app_slots"]).to(dev))
    assert torch.equal(bits(kc), _t(e["app_kc_out"], h).view(torch.int16))
    assert torch.equal(bits(vc), _t(e["app_vc_out"], h).view(torch.int16))
    rq, rk = _t(e["rope_q"], h).to(dev), _t(e["rope_k"], h).to(dev)
    kernels.vllm_rotary_emb(_t(e["rope_pos"]).to(dev), rq, rk, _t(e["rope_cache"], h).to(dev), 128)
    assert torch.equal(bits(rq), _t(e["rope_q_out"], h).view(torch.int16))
    assert torch.equal(bits(rk), _t(e["rope_k_out"], h).view(torch.int16))
    x, r, w = _t(e["norm_x"], h).to(dev), _t(e["norm_r"], h).to(dev), _t(e["norm_w"], h).to(dev)
    torch.testing.assert_close(kernels.vllm_rms_norm(x, w, 1e-6).cpu().float(), _t(e["norm_round_first"], h).float(), **TOL[h])
    torch.testing.assert_close(kernels.rmsnorm_forward(x, w, 1e-6).cpu().float(), _t(e["norm_round_once"], h).float(), **TOL[h])
    rr = r.clone()
    y = kernels.fused_add_rms_norm(x, rr, w, 1e-6)
    assert torch.equal(bits(rr), _t(e["addnorm_h"], h).view(torch.int16))
    torch.testing.assert_close(y.cpu().float(), _t(e["addnorm_y"], h).float(), **TOL[h])
    torch.testing.assert_close(kernels.silu_mul(x, r).cpu().float(), _t(e["silu_mul"], h).float(), **TOL[h])


def test_oracle_reproduces_sampler_fixture():
    f = _load("sampler_fp16.npz")
    x = _t(f["logits"], torch.float16)
    ids, margins = ref_sampler.ref_sample(x.double().numpy(), f["temperature"], f["top_p"], f["uniform"], "f16")
    assert (ids == f["ids"]).all() and (margins >= 1e-4).all()


@pytest.mark.gpu
def test_gpu_sampler_matches_fixture(dev):
    from parrotserve_amd import kernels

    f = _load("sampler_fp16.npz")
    ids = kernels.sample_top_p(_t(f["logits"], torch.float16).to(dev), _t(f["temperature"]).to(dev), _t(f["top_p"]).to(dev),
                               _t(f["uniform"]).to(dev))
    assert ids.cpu().tolist() == f["ids"].tolist()
