"""Pins for the token move / KV append / RoPE / RMSNorm parts of the CPU oracle."""
import math

import pytest
import torch

from oracle.ref_ops import (ref_cos_sin_cache, ref_kv_append, ref_move_from_blocked_k, ref_move_from_blocked_v,
                            ref_move_tokens, ref_rms_norm, ref_rope_neox, ref_rotary_embedding)


def test_move_tokens_python_loop():
    g = torch.Generator().manual_seed(0)
    src = torch.randn(20, 3, 4, generator=g).half()
    dst0 = torch.randn(30, 3, 4, generator=g).half()
    si = torch.randint(0, 20, (9,), generator=g)  # repeats allowed on the source side
    di = torch.randperm(30, generator=g)[:9]
    dst = dst0.clone()
    ref_move_tokens(src, dst, si, di)
    want = dst0.clone()
    for i in range(9):
        for h in range(3):
            for d in range(4):
                want[int(di[i]), h, d] = src[int(si[i]), h, d]
    assert torch.equal(dst.view(torch.int16), want.view(torch.int16))
    untouched = [r for r in range(30) if r not in set(di.tolist())]
    assert torch.equal(dst[untouched].view(torch.int16), dst0[untouched].view(torch.int16))


def test_move_tokens_strided_dest_like_reference_selftest():
    # tokens_moving.py:316-362 moves random src rows to every second dest row
    g = torch.Generator().manual_seed(1)
    src = torch.randn(64, 2, 8, generator=g).half()
    dst = torch.zeros(128, 2, 8).half()
    si = torch.randperm(64, generator=g)
    di = torch.arange(0, 128, 2)
    ref_move_tokens(src, dst, si, di)
    assert torch.equal(dst[::2], src[si]) and (dst[1::2] == 0).all()


def _blocked_case(seed, nblk=5, H=3, D=8, bs=4, x=2, n=11, rows=30):
    g = torch.Generator().manual_seed(seed)
    kc = torch.randn(nblk, H, D // x, bs, x, generator=g).half()
    vc = torch.randn(nblk, H, D, bs, generator=g).half()
    slots = torch.randint(0, nblk * bs, (n,), generator=g)
    di = torch.randperm(rows, generator=g)[:n]
    dst0 = torch.randn(rows, H, D, generator=g).half()
    return kc, vc, slots, di, dst0


def test_move_from_blocked_flat_offset_loops():
    """Element-wise loops over the flat buffers with each layout's offset formula (K [nb,H,D/x,bs,x], V [nb,H,D,bs])."""
    nblk, H, D, bs, x = 5, 3, 8, 4, 2
    kc, vc, slots, di, dst0 = _blocked_case(3, nblk, H, D, bs, x)
    kflat, vflat = kc.reshape(-1), vc.reshape(-1)
    want_k, want_v = dst0.clone(), dst0.clone()
    for i in range(slots.numel()):
        b, o = divmod(int(slots[i]), bs)
        for h in range(H):
            for d in range(D):
                want_k[int(di[i]), h, d] = kflat[(((b * H + h) * (D // x) + d // x) * bs + o) * x + d % x]
                want_v[int(di[i]), h, d] = vflat[((b * H + h) * D + d) * bs + o]
    got_k, got_v = dst0.clone(), dst0.clone()
    ref_move_from_blocked_k(kc, got_k, slots, di)
    ref_move_from_blocked_v(vc, got_v, slots, di)
    assert torch.equal(got_k.view(torch.int16), want_k.view(torch.int16))
    assert torch.equal(got_v.view(torch.int16), want_v.view(torch.int16))
    untouched = [r for r in range(dst0.shape[0]) if r not in set(di.tolist())]
    assert torch.equal(got_k[untouched], dst0[untouched]) and torch.equal(got_v[untouched], dst0[untouched])


def test_move_from_blocked_equals_move_on_the_token_granular_view():
    """Permuting a blocked cache to [num_blocks * block_size, H, D] makes the gather an ordinary token move."""
    kc, vc, slots, di, dst0 = _blocked_case(4, nblk=6, H=2, D=16, bs=8, x=4, n=20, rows=40)
    nblk, H, cols, bs, x = kc.shape
    k_rows = kc.permute(0, 3, 1, 2, 4).reshape(nblk * bs, H, cols * x)
    v_rows = vc.permute(0, 3, 1, 2).reshape(nblk * bs, H, cols * x)
    for blocked, rows, fn in ((kc, k_rows, ref_move_from_blocked_k), (vc, v_rows, ref_move_from_blocked_v)):
        got, want = dst0.clone(), dst0.clone()
        fn(blocked, got, slots, di)
        ref_move_tokens(rows, want, slots, di)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_move_from_blocked_block_size_one_is_the_token_move():
    g = torch.Generator().manual_seed(5)
    rows = torch.randn(12, 2, 8, generator=g).half()
    slots = torch.randint(0, 12, (7,), generator=g)
    di = torch.randperm(9, generator=g)[:7]
    want = torch.zeros(9, 2, 8).half()
    ref_move_tokens(rows, want, slots, di)
    got_k, got_v = torch.zeros(9, 2, 8).half(), torch.zeros(9, 2, 8).half()
    ref_move_from_blocked_k(rows.view(12, 2, 2, 1, 4), got_k, slots, di)
    ref_move_from_blocked_v(rows.view(12, 2, 8, 1), got_v, slots, di)
    assert torch.equal(got_k, want) and torch.equal(got_v, want)


def test_kv_append_roundtrip_and_noncontiguous_source():
    g = torch.Generator().manual_seed(2)
    qkv = torch.randn(5, 3 * 2 * 4, generator=g).bfloat16()
    _, k, v = qkv.chunk(3, dim=-1)  # strided views, as in models/llama.py:111-112
    k, v = k.view(5, 2, 4), v.view(5, 2, 4)
    kc = torch.zeros(16, 2, 4).bfloat16()
    vc = torch.zeros(16, 2, 4).bfloat16()
    slots = torch.tensor([3, 0, 15, 7, 8], dtype=torch.int32)
    ref_kv_append(k, v, kc, vc, slots)
    for t in range(5):
        assert torch.equal(kc[int(slots[t])], k[t]) and torch.equal(vc[int(slots[t])], v[t])
    assert (kc[[1, 2, 4, 5, 6, 9]] == 0).all()


def test_cos_sin_cache_closed_form():
    c = ref_cos_sin_cache(64, 8, 10000.0, torch.float32)
    assert c.shape == (64, 8)
    for p in (0, 1, 17, 63):
        for i in range(4):
            f = 10000.0 ** (-2 * i / 8)
            assert abs(float(c[p, i]) - math.cos(p * f)) < 1e-5
            assert abs(float(c[p, 4 + i]) - math.sin(p * f)) < 1e-5
    assert ref_cos_sin_cache(4, 8, 10000.0, torch.float16).dtype == torch.float16


def _rotate_half(x):
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2 :]
    return torch.cat((-x2, x1), dim=-1)


def test_rope_matches_hf_rotate_half_form():
    # 3rdparty/vllm/tests/kernels/test_pos_encoding.py:10-24,27-75
    g = torch.Generator().manual_seed(3)
    T, H, D = 6, 3, 16
    q = torch.randn(T, H * D, generator=g)
    k = torch.randn(T, H * D, generator=g)
    pos = torch.tensor([0, 5, 1, 31, 7, 7])
    cache = ref_cos_sin_cache(32, D, 10000.0, torch.float32)
    rq, rk = ref_rope_neox(pos, q, k, cache, D)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))
    emb = torch.cat([torch.outer(pos.float(), inv)] * 2, dim=-1)  # [T, D]
    cos, sin = emb.cos()[:, None, :], emb.sin()[:, None, :]
    for x, r in ((q, rq), (k, rk)):
        x3 = x.view(T, H, D)
        want = x3 * cos + _rotate_half(x3) * sin
        torch.testing.assert_close(r.view(T, H, D), want, atol=1e-5, rtol=1e-5)


def test_rope_invariants():
    g = torch.Generator().manual_seed(4)
    T, H, D = 5, 2, 8
    x = torch.randn(T, H, D, generator=g)
    pos = torch.tensor([0, 3, 9, 2, 0])
    cache = ref_cos_sin_cache(16, D, 10000.0, torch.float32)
    cs = cache[pos]
    cos, sin = cs[:, None, : D // 2], cs[:, None, D // 2 :]
    r = ref_rotary_embedding(x, cos, sin)
    # position 0 is the identity
    torch.testing.assert_close(r[0], x[0])
    torch.testing.assert_close(r[4], x[4])
    # each (x_i, y_i) pair keeps its norm
    n0 = x[..., : D // 2] ** 2 + x[..., D // 2 :] ** 2
    n1 = r[..., : D // 2] ** 2 + r[..., D // 2 :] ** 2
    torch.testing.assert_close(n0, n1, atol=1e-5, rtol=1e-5)
    # rotating back by -angle restores the input
    back = ref_rotary_embedding(r, cos, -sin)
    torch.testing.assert_close(back, x, atol=1e-5, rtol=1e-5)
    # dot products depend on the position difference only
    a = torch.randn(1, 1, D, generator=g)
    b = torch.randn(1, 1, D, generator=g)

    def rot(v, p):
        c = cache[p][None, None]
        return ref_rotary_embedding(v, c[..., : D // 2], c[..., D // 2 :])

    d1 = (rot(a, 7) * rot(b, 4)).sum()
    d2 = (rot(a, 10) * rot(b, 7)).sum()
    torch.testing.assert_close(d1, d2, atol=1e-5, rtol=1e-5)


def test_rope_partial_rotary_dim_passes_tail_through():
    g = torch.Generator().manual_seed(5)
    T, H, D, rot = 3, 2, 16, 8
    q = torch.randn(T, H * D, generator=g)
    cache = ref_cos_sin_cache(8, rot, 10000.0, torch.float32)
    rq, _ = ref_rope_neox(torch.tensor([1, 2, 3]), q, q.clone(), cache, D)
    torch.testing.assert_close(rq.view(T, H, D)[..., rot:], q.view(T, H, D)[..., rot:])
    assert not torch.allclose(rq.view(T, H, D)[..., :rot], q.view(T, H, D)[..., :rot])


def test_rope_elem_rounding_mode_rounds_each_product():
    # a case where rounding each product to fp16 differs from fp32 math
    x = torch.tensor([[[1.0 + 2 ** -10, 1.0]]]).half()  # D=2: x=first, y=second
    cos = torch.tensor([[[1.0 + 2 ** -10]]]).half()
    sin = torch.tensor([[[2.0 ** -11]]]).half()
    exact = ref_rotary_embedding(x, cos, sin, elem_rounding=False)
    elem = ref_rotary_embedding(x, cos, sin, elem_rounding=True)
    xf, cf, sf = float(x[0, 0, 0]), float(cos[0, 0, 0]), float(sin[0, 0, 0])
    want_elem = (torch.tensor(xf * cf).half() - torch.tensor(1.0 * sf).half()).half()
    assert float(elem[0, 0, 0]) == float(want_elem)
    assert float(exact[0, 0, 0]) == float(torch.tensor(xf * cf - sf).half())


def test_rms_norm_library_and_invariants():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(7, 48, generator=g) * 3 - 1
    w = torch.rand(48, generator=g)
    y = ref_rms_norm(x, w, 1e-6)
    lib = torch.nn.functional.rms_norm(x, (48,), weight=w, eps=1e-6)
    torch.testing.assert_close(y, lib, atol=1e-6, rtol=1e-6)
    # unit weight: mean square of the output is 1
    y1 = ref_rms_norm(x, torch.ones(48), 0.0)
    torch.testing.assert_close(y1.pow(2).mean(-1), torch.ones(7), atol=1e-5, rtol=1e-5)
    # scale invariance for eps -> 0
    torch.testing.assert_close(ref_rms_norm(5 * x, w, 0.0), ref_rms_norm(x, w, 0.0), atol=1e-5, rtol=1e-5)
    # eps matters when x is tiny
    tiny = torch.full((1, 4), 1e-4)
    assert float(ref_rms_norm(tiny, torch.ones(4), 1e-2)[0, 0]) == pytest.approx(1e-4 / math.sqrt(1e-8 + 1e-2), rel=1e-5)


def test_rms_norm_rounding_order_half():
    # layernorm_kernels.cu:32 rounds x*rstd to fp16 BEFORE the weight multiply
    x = torch.tensor([[3.0, 4.0, 0.0, 0.0]]).half()
    w = torch.tensor([1.0 + 2 ** -10, 3.0, 1.0, 1.0]).half()
    rstd = 1.0 / math.sqrt(25.0 / 4 + 0.0)
    first = ref_rms_norm(x, w, 0.0, round_before_weight=True)
    once = ref_rms_norm(x, w, 0.0, round_before_weight=False)
    n0 = torch.tensor(3.0 * rstd).half()
    assert float(first[0, 0]) == float((n0.float() * w[0].float()).half())
    assert float(once[0, 0]) == float(torch.tensor(3.0 * rstd * float(w[0])).half())
    # the reference's own self-test distribution (kernels/rms_norm.py:85-99): both orders agree within its atol
    g = torch.Generator().manual_seed(7)
    xx = (-2.3 + 0.5 * torch.randn(16, 256, generator=g)).half()
    ww = torch.rand(256, generator=g).half()
    assert torch.allclose(ref_rms_norm(xx, ww, 1e-5, True).float(), ref_rms_norm(xx, ww, 1e-5, False).float(), atol=1e-2, rtol=0)


# --------------------------------------------------------------------------- #
# fused per-layer ops
# --------------------------------------------------------------------------- #
def test_add_rms_norm_is_torch_add_then_norm_on_the_stored_sum():
    from oracle.ref_ops import ref_add_rms_norm

    g = torch.Generator().manual_seed(31)
    for dt in (torch.float16, torch.bfloat16):
        x = (torch.randn(7, 96, generator=g) * 3).to(dt)
        r = (torch.randn(7, 96, generator=g) * 3).to(dt)
        w = (torch.rand(96, generator=g) + 0.5).to(dt)
        y, h = ref_add_rms_norm(x, r, w, 1e-6, round_before_weight=False)
        h_t = r + x                                   # torch's own add in the element type
        assert torch.equal(h.view(torch.int16), h_t.view(torch.int16))
        y_t = torch.nn.functional.rms_norm(h_t.float(), (96,), w.float(), 1e-6).to(dt)
        torch.testing.assert_close(y.float(), y_t.float(), atol=1e-2, rtol=1e-2)
    # the norm sees the ROUNDED sum: 2048 + 1 is not representable in fp16 (spacing 2), so h = 2048, not 2049
    x = torch.tensor([[2048.0, 0.0]], dtype=torch.float16)
    r = torch.tensor([[1.0, 0.0]], dtype=torch.float16)
    y, h = ref_add_rms_norm(x, r, torch.ones(2, dtype=torch.float16), 0.0, round_before_weight=False)
    assert h[0, 0].item() == 2048.0
    assert abs(y[0, 0].item() - 2 ** 0.5) < 1e-3      # 2048 / sqrt((2048^2 + 0) / 2)


def test_silu_mul_closed_forms_and_torch():
    from oracle.ref_ops import ref_silu_mul

    one = torch.ones(5, dtype=torch.float16)
    gate = torch.tensor([0.0, 20.0, -20.0, 1.0, -1.0], dtype=torch.float16)
    got = ref_silu_mul(gate, one).float()
    want = torch.tensor([0.0, 20.0, 0.0, 1 / (1 + math.exp(-1.0)), -1 / (1 + math.exp(1.0))])
    torch.testing.assert_close(got, want, atol=1e-3, rtol=1e-3)
    g = torch.Generator().manual_seed(32)
    for dt in (torch.float16, torch.bfloat16):
        a = (torch.randn(4, 64, generator=g) * 3).to(dt)
        b = (torch.randn(4, 64, generator=g) * 3).to(dt)
        ref = torch.nn.functional.silu(a) * b         # torch rounds silu, then the product, in the element type
        assert torch.equal(ref_silu_mul(a, b).view(torch.int16), ref.view(torch.int16))
    # linear in `up`, and the two roundings are visible: silu(1) rounds before the product
    a = torch.tensor([1.0], dtype=torch.float16)
    s = torch.nn.functional.silu(a.float()).half()
    assert ref_silu_mul(a, torch.tensor([3.0], dtype=torch.float16)).item() == (s.float() * 3).half().item()
