"""GPU parity: token move / KV append (bit-exact), RoPE, RMSNorm vs the CPU oracle."""
import pytest
import torch

from oracle.ref_ops import (ref_cos_sin_cache, ref_kv_append, ref_move_from_blocked_k, ref_move_from_blocked_v,
                            ref_move_tokens, ref_rms_norm, ref_rope_neox, ref_rotary_embedding)

pytestmark = pytest.mark.gpu

TOL = {torch.float16: dict(atol=2e-3, rtol=1e-2), torch.bfloat16: dict(atol=1e-2, rtol=2e-2)}


def _bits(t):
    return t.contiguous().view(torch.int16) if t.element_size() == 2 else t.contiguous().view(torch.int32)


@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("H,D,dtype", [(32, 128, torch.float16), (40, 128, torch.bfloat16), (3, 20, torch.float16),
                                        (2, 8, torch.float32)])
def test_move_tokens_bit_exact(dev, idx_dtype, H, D, dtype):
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(11)
    n_src, n_dst, n = 300, 500, 257
    src = torch.randn(n_src, H, D, generator=g).to(dtype)
    dst0 = torch.randn(n_dst, H, D, generator=g).to(dtype)
    si = torch.randint(0, n_src, (n,), generator=g).to(idx_dtype)
    di = torch.randperm(n_dst, generator=g)[:n].to(idx_dtype)
    want = dst0.clone()
    ref_move_tokens(src, want, si, di)
    d = dst0.to(dev)
    kernels.discontinuous_move_tokens(src.to(dev), d, si.to(dev), di.to(dev))
    assert torch.equal(_bits(d.cpu()), _bits(want))


def test_move_tokens_strided_storages(dev):
    """Free strides on all three axes (tokens_moving.py:88-93): a head-sliced, dim-strided view."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(12)
    big_src = torch.randn(64, 6, 32, generator=g).half()
    big_dst = torch.randn(80, 4, 48, generator=g).half()
    src_view = lambda t: t[:, 1:5, ::2]  # [64, 4, 16], strides (192, 32, 2)
    dst_view = lambda t: t[:, :, 16:32]  # [80, 4, 16], strides (192, 48, 1)
    si = torch.randperm(64, generator=g)[:40]
    di = torch.randperm(80, generator=g)[:40]
    want = big_dst.clone()
    ref_move_tokens(src_view(big_src), dst_view(want), si, di)
    s, d = big_src.to(dev), big_dst.to(dev)
    kernels.discontinuous_move_tokens(src_view(s), dst_view(d), si.to(dev), di.to(dev))
    assert torch.equal(_bits(d.cpu()), _bits(want))


def _blocked_inputs(seed, nblk, H, D, bs, x, n, rows, dtype, idx_dtype, runs):
    g = torch.Generator().manual_seed(seed)
    kc = torch.randn(nblk, H, D // x, bs, x, generator=g).to(dtype)
    vc = torch.randn(nblk, H, D, bs, generator=g).to(dtype)
    if runs:  # whole blocks in order (a context that owns its blocks), then a random tail
        blocks = torch.randperm(nblk, generator=g)[: n // bs]
        slots = (blocks[:, None] * bs + torch.arange(bs)[None, :]).reshape(-1)
        slots = torch.cat([slots, torch.randint(0, nblk * bs, (n - slots.numel(),), generator=g)])
    else:
        slots = torch.randint(0, nblk * bs, (n,), generator=g)
    di = torch.randperm(rows, generator=g)[:n]
    dst0 = torch.randn(rows, H, D, generator=g).to(dtype)
    return kc, vc, slots.to(idx_dtype), di.to(idx_dtype), dst0


@pytest.mark.parametrize("runs", [True, False])
@pytest.mark.parametrize("H,D,bs,x,dtype,idx_dtype", [
    (32, 128, 16, 8, torch.float16, torch.int64),   # the vLLM layout at 16-bit elements
    (40, 128, 16, 8, torch.bfloat16, torch.int32),
    (96, 128, 16, 8, torch.float16, torch.int64),   # tokens_moving.py:365-420 (H 96, block 16, x 8)
    (5, 64, 8, 4, torch.float32, torch.int64),      # 16-byte units of 4-byte elements, head count not a multiple of 4
    (3, 256, 32, 8, torch.float16, torch.int32),    # 512-byte head rows
    (2, 512, 4, 8, torch.float16, torch.int64),     # 1 KB head rows: one head per LDS round
    (3, 24, 4, 2, torch.float16, torch.int64),      # 3-unit... head rows of 48 bytes, not a power of two: element path
    (2, 20, 3, 5, torch.float16, torch.int32),      # odd everything: element path
])
def test_move_from_blocked_caches_bit_exact(dev, H, D, bs, x, dtype, idx_dtype, runs):
    from parrotserve_amd import kernels

    nblk, n, rows = 24, 203, 300
    kc, vc, slots, di, dst0 = _blocked_inputs(21, nblk, H, D, bs, x, n, rows, dtype, idx_dtype, runs)
    want_k, want_v = dst0.clone(), dst0.clone()
    ref_move_from_blocked_k(kc, want_k, slots, di)
    ref_move_from_blocked_v(vc, want_v, slots, di)
    dk, dv = dst0.to(dev), dst0.to(dev)
    kernels.move_tokens_from_blocked_k_cache(kc.to(dev), dk, slots.to(dev), di.to(dev))
    kernels.move_tokens_from_blocked_v_cache(vc.to(dev), dv, slots.to(dev), di.to(dev))
    assert torch.equal(_bits(dk.cpu()), _bits(want_k))
    assert torch.equal(_bits(dv.cpu()), _bits(want_v))


def test_move_from_blocked_strided_views_and_empty(dev):
    """Free strides (tokens_moving.py:182-200 passes every stride): a head slice of a larger cache, a strided
    destination; and an empty index list is a no-op."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(22)
    big_k = torch.randn(10, 6, 4, 8, 8, generator=g).half()
    big_v = torch.randn(10, 6, 32, 8, generator=g).half()
    kc, vc = big_k[:, 1:5], big_v[:, 1:5]               # heads 1..4 of 6
    big_dst = torch.randn(50, 4, 64, generator=g).half()
    dview = lambda t: t[:, :, 16:48]                    # [50, 4, 32], head stride 64
    slots = torch.randint(0, 80, (33,), generator=g)
    di = torch.randperm(50, generator=g)[:33]
    want_k, want_v = big_dst.clone(), big_dst.clone()
    ref_move_from_blocked_k(kc, dview(want_k), slots, di)
    ref_move_from_blocked_v(vc, dview(want_v), slots, di)
    dk, dv = big_dst.to(dev), big_dst.to(dev)
    kernels.move_tokens_from_blocked_k_cache(big_k.to(dev)[:, 1:5], dview(dk), slots.to(dev), di.to(dev))
    kernels.move_tokens_from_blocked_v_cache(big_v.to(dev)[:, 1:5], dview(dv), slots.to(dev), di.to(dev))
    assert torch.equal(_bits(dk.cpu()), _bits(want_k))
    assert torch.equal(_bits(dv.cpu()), _bits(want_v))
    empty = torch.zeros(0, dtype=torch.int64, device=dev)
    before = dk.clone()
    kernels.move_tokens_from_blocked_k_cache(big_k.to(dev)[:, 1:5], dview(dk), empty, empty)
    assert torch.equal(dk, before)


def test_move_from_blocked_equals_token_move_at_scale(dev):
    """65,536 tokens at 32 x 128: the blocked gathers against the plain token move on the permuted caches."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(23)
    nblk, H, D, bs, x, n = 8192, 32, 128, 16, 8, 65536
    rows = torch.randn(nblk * bs, H, D, generator=g).half().to(dev)   # token-granular truth
    kc = rows.view(nblk, bs, H, D // x, x).permute(0, 2, 3, 1, 4).contiguous()
    vc = rows.view(nblk, bs, H, D).permute(0, 2, 3, 1).contiguous()
    slots = torch.randint(0, nblk * bs, (n,), generator=g).to(dev)
    di = torch.randperm(n, generator=g).to(dev)
    want = torch.zeros(n, H, D, dtype=torch.float16, device=dev)
    kernels.discontinuous_move_tokens(rows, want, slots, di)
    for cache, fn in ((kc, kernels.move_tokens_from_blocked_k_cache), (vc, kernels.move_tokens_from_blocked_v_cache)):
        got = torch.zeros_like(want)
        fn(cache, got, slots, di)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
def test_config3_token_move_full_size(dev, idx_dtype):
    """Config 3's move at its own size: 65,536 random source rows to 65,536 other rows of one 4M-slot pool
    (32 x 128 fp16, 8 KB rows), bit-exact against the oracle on the touched rows, and every other row of the pool
    unchanged.  The oracle runs on the compacted rows (source rows first, then the destinations' old contents)
    with the indices renumbered to match; the pool itself only exists on the device (34 GB)."""
    from parrotserve_amd import kernels, synth

    pool, H, D = 1 << 22, 32, 128
    src, dst = synth.config3_move(index_dtype=idx_dtype)
    n = src.numel()
    assert n == 65536 and src.dtype == idx_dtype and torch.unique(dst).numel() == n
    assert not torch.isin(dst.long(), src.long()).any()
    gen = torch.Generator(device=dev).manual_seed(5)
    kc = torch.randn((pool, H, D), generator=gen, device=dev, dtype=torch.float16)
    before = kc.clone()
    sd, dd = src.to(dev), dst.to(dev)
    compact = torch.cat([before[sd.long()], before[dd.long()]]).cpu()  # [2n, H, D]
    ref_move_tokens(compact, compact, torch.arange(n), n + torch.arange(n))
    kernels.discontinuous_move_tokens(kc, kc, sd, dd)
    torch.cuda.synchronize()
    assert torch.equal(_bits(kc[dd.long()].cpu()), _bits(compact[n:]))
    # everything but the destination rows is what it was (compared as bits, in slices of 256K rows)
    before[dd.long()] = kc[dd.long()]
    a, b = kc.view(torch.int16), before.view(torch.int16)
    step = 1 << 18
    for r in range(0, pool, step):
        assert torch.equal(a[r:r + step], b[r:r + step]), f"rows {r}..{r + step} changed"
    del kc, before, a, b
    torch.cuda.empty_cache()


def test_move_tokens_reference_selftest_shape(dev):
    """tokens_moving.py:316-362: H 96 x D 128 fp16, random src rows to every second dest row (scaled-down count)."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(13)
    n = 4096
    src = torch.randn(n, 96, 128, generator=g).half()
    si = torch.randperm(n, generator=g)
    di = torch.arange(0, 2 * n, 2)
    d = torch.zeros(2 * n, 96, 128, dtype=torch.float16, device=dev)
    kernels.discontinuous_move_tokens(src.to(dev), d, si.to(dev), di.to(dev))
    out = d.cpu()
    assert torch.equal(_bits(out[::2]), _bits(src[si])) and (out[1::2] == 0).all()


def test_move_empty_and_blocked_names(dev):
    from parrotserve_amd import kernels

    src = torch.randn(8, 2, 16).half().to(dev)
    dst = torch.zeros(8, 2, 16).half().to(dev)
    e = torch.empty(0, dtype=torch.int64, device=dev)
    kernels.discontinuous_move_tokens(src, dst, e, e)
    assert (dst == 0).all()
    idx = torch.arange(8, device=dev)
    kernels.move_tokens_from_blocked_k_cache(src, dst, idx.flip(0), idx)
    assert torch.equal(dst.cpu(), src.cpu().flip(0))
    kernels.move_tokens_from_blocked_v_cache(src, dst, idx, idx)
    assert torch.equal(dst.cpu(), src.cpu())
    with pytest.raises(ValueError):  # neither the 5-d blocked K layout nor token-granular rows
        kernels.move_tokens_from_blocked_k_cache(torch.zeros(2, 2, 16, 4, device=dev).half(), dst, idx, idx)
    with pytest.raises(AssertionError):  # head shape of the cache and of the destination differ
        kernels.move_tokens_from_blocked_k_cache(torch.zeros(2, 2, 4, 4, 8, device=dev).half(), dst, idx, idx)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("idx_dtype", [torch.int32, torch.int64])
def test_kv_append_bit_exact_from_qkv_views(dev, dtype, idx_dtype):
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(14)
    T, H, D, slots = 77, 40, 128, 1000
    qkv = torch.randn(T, 3 * H * D, generator=g).to(dtype)
    kc0 = torch.randn(slots, H, D, generator=g).to(dtype)
    vc0 = torch.randn(slots, H, D, generator=g).to(dtype)
    sm = torch.randperm(slots, generator=g)[:T].to(idx_dtype)
    _, k, v = qkv.chunk(3, dim=-1)
    kc, vc = kc0.clone(), vc0.clone()
    ref_kv_append(k.view(T, H, D), v.view(T, H, D), kc, vc, sm)
    dq = qkv.to(dev)
    _, dk, dv = dq.chunk(3, dim=-1)
    dkc, dvc = kc0.to(dev), vc0.to(dev)
    kernels.vllm_reshape_and_cache(dk.view(T, H, D), dv.view(T, H, D), dkc, dvc, sm.to(dev))
    assert torch.equal(_bits(dkc.cpu()), _bits(kc)) and torch.equal(_bits(dvc.cpu()), _bits(vc))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,n", [(128, 5120), (33, 4096), (5, 8192), (7, 1000), (3, 130),
                                    (2049, 5120), (2051, 8192), (2048, 512), (2050, 1320), (2500, 16384)])
def test_rms_norm(dev, dtype, rows, n):
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(15)
    x = (torch.randn(rows, n, generator=g) * 2 - 0.5).to(dtype)
    w = (torch.rand(n, generator=g) + 0.5).to(dtype)
    for fn, first in ((kernels.vllm_rms_norm, True), (kernels.rmsnorm_forward, False)):
        y = fn(x.to(dev), w.to(dev), 1e-6).cpu()
        ref = ref_rms_norm(x, w, 1e-6, round_before_weight=first)
        torch.testing.assert_close(y.float(), ref.float(), **TOL[dtype])


def test_rms_norm_reference_selftest_distribution(dev):
    """kernels/rms_norm.py:85-99: x ~ -2.3 + 0.5 N(0,1), w ~ U[0,1), atol 1e-2 rtol 0."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(16)
    x = (-2.3 + 0.5 * torch.randn(1151, 8192, generator=g)).half()
    w = torch.rand(8192, generator=g).half()
    y = kernels.rmsnorm_forward(x.to(dev), w.to(dev), 1e-5).cpu()
    ref = ref_rms_norm(x, w, 1e-5, round_before_weight=False)
    assert torch.allclose(y.float(), ref.float(), atol=1e-2, rtol=0)
    torch.testing.assert_close(y.float(), ref.float(), **TOL[torch.float16])


def test_rms_norm_3d_input_keeps_shape(dev):
    from parrotserve_amd import kernels

    x = torch.randn(2, 5, 256).half()
    w = torch.ones(256).half()
    y = kernels.vllm_rms_norm(x.to(dev), w.to(dev), 1e-6)
    assert y.shape == x.shape
    torch.testing.assert_close(y.cpu().float(), ref_rms_norm(x, w, 1e-6).float(), **TOL[torch.float16])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,H,D", [(129, 40, 128), (17, 32, 64), (5, 3, 80)])
def test_rope_neox_on_qkv_views(dev, dtype, T, H, D):
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(17)
    qkv = torch.randn(T, 3 * H * D, generator=g).to(dtype)
    pos = torch.randint(0, 4096, (T,), generator=g)
    cache = ref_cos_sin_cache(4096, D, 10000.0, dtype)
    q, k, v = qkv.chunk(3, dim=-1)
    rq, rk = ref_rope_neox(pos, q, k, cache, D, elem_rounding=True)
    rq32, rk32 = ref_rope_neox(pos, q, k, cache, D, elem_rounding=False)
    d = qkv.to(dev)
    dq, dk, dv = d.chunk(3, dim=-1)
    kernels.vllm_rotary_emb(pos.to(dev), dq, dk, cache.to(dev), D)
    out = d.cpu()
    oq, ok, ov = out.chunk(3, dim=-1)
    assert torch.equal(_bits(ov), _bits(v)), "v must be untouched"
    # same arithmetic as the reference kernel (every product rounded to the element type): bit-exact
    assert torch.equal(_bits(oq), _bits(rq)) and torch.equal(_bits(ok), _bits(rk))
    torch.testing.assert_close(oq.float(), rq32.float(), **TOL[dtype])
    torch.testing.assert_close(ok.float(), rk32.float(), **TOL[dtype])


def test_rotary_embedding_reference_selftest(dev):
    """kernels/rotary_embedding.py:155-174: T 256, H 96, D 128, cos ~ -1.2+0.5N, sin ~ -2.0+0.5N, atol 1e-2."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(18)
    T, H, D = 256, 96, 128
    state = torch.randn(T, H, D, generator=g).half()
    cos = (-1.2 + 0.5 * torch.randn(T, 1, D // 2, generator=g)).half()
    sin = (-2.0 + 0.5 * torch.randn(T, 1, D // 2, generator=g)).half()
    ref = ref_rotary_embedding(state, cos, sin)
    d = state.to(dev)
    kernels.rotary_embedding(d, cos.to(dev), sin.to(dev))
    assert torch.allclose(d.cpu().float(), ref.float(), atol=1e-2, rtol=0)
    assert torch.equal(_bits(d.cpu()), _bits(ref_rotary_embedding(state, cos, sin, elem_rounding=True)))


def test_rope_round_trip_property(dev):
    """rotate by +angle then -angle restores the input (within two roundings)."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(19)
    T, H, D = 64, 8, 128
    x = torch.randn(T, H, D, generator=g).half()
    cache = ref_cos_sin_cache(512, D, 10000.0, torch.float16)
    pos = torch.randint(0, 512, (T,), generator=g)
    cs = cache[pos]
    cos, sin = cs[:, None, : D // 2].contiguous(), cs[:, None, D // 2 :].contiguous()
    d = x.to(dev)
    kernels.rotary_embedding(d, cos.to(dev), sin.to(dev))
    kernels.rotary_embedding(d, cos.to(dev), (-sin).to(dev))
    torch.testing.assert_close(d.cpu().float(), x.float(), atol=8e-3, rtol=1e-2)


# --------------------------------------------------------------------------- #
# fused per-layer ops
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,n", [(128, 5120), (64, 4096), (5, 8192), (7, 1000), (3, 130)])
def test_fused_add_rms_norm(dev, dtype, rows, n):
    """residual += x is bit-exact (it is a rounded fp add); the norm matches the oracle, and equals the library's
    own unfused norm of the stored sum bit for bit."""
    from oracle.ref_ops import ref_add_rms_norm
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(16)
    x = (torch.randn(rows, n, generator=g) * 2).to(dtype)
    r = (torch.randn(rows, n, generator=g) * 2 - 0.5).to(dtype)
    w = (torch.rand(n, generator=g) + 0.5).to(dtype)
    for first in (True, False):
        rd = r.to(dev)
        y = kernels.fused_add_rms_norm(x.to(dev), rd, w.to(dev), 1e-6, round_before_weight=first)
        y_ref, h_ref = ref_add_rms_norm(x, r, w, 1e-6, round_before_weight=first)
        assert torch.equal(_bits(rd.cpu()), _bits(h_ref))
        torch.testing.assert_close(y.cpu().float(), y_ref.float(), **TOL[dtype])
        unfused = (kernels.vllm_rms_norm if first else kernels.rmsnorm_forward)(rd, w.to(dev), 1e-6)
        assert torch.equal(_bits(y.cpu()), _bits(unfused.cpu()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,d", [(128, 13824), (9, 11008), (3, 100), (1, 7)])
def test_silu_mul(dev, dtype, rows, d):
    from oracle.ref_ops import ref_silu_mul
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(17)
    gu = (torch.randn(rows, 2 * d, generator=g) * 2).to(dtype)
    ref = ref_silu_mul(gu[:, :d], gu[:, d:])
    dgu = gu.to(dev)
    out = kernels.silu_mul(dgu[:, :d], dgu[:, d:])          # strided column views of one fused projection
    torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[dtype])
    out2 = torch.empty(rows, d, dtype=dtype, device=dev)
    kernels.silu_and_mul(out2, dgu)                          # vLLM's [T, 2d] form
    assert torch.equal(_bits(out2.cpu()), _bits(out.cpu()))
    sep = kernels.silu_mul(dgu[:, :d].contiguous(), dgu[:, d:].contiguous())
    assert torch.equal(_bits(sep.cpu()), _bits(out.cpu()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,H,D,idx", [(77, 8, 128, torch.int32), (5, 40, 128, torch.int64), (33, 3, 64, torch.int32),
                                       (9, 2, 72, torch.int32)])
def test_rope_and_cache_equals_rope_then_append(dev, dtype, T, H, D, idx):
    """The fused op leaves q, k and both pools bit-identical to the two separate kernels, which are themselves
    checked against the oracle (rotation in the element type, append by slot); D = 72 takes the unfused path."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(18)
    slots = 512
    qkv = torch.randn(T, 3 * H * D, generator=g).to(dtype)
    pos = torch.randint(0, 300, (T,), generator=g)
    sm = torch.randperm(slots, generator=g)[:T].to(idx)
    cache = ref_cos_sin_cache(300, D, 10000.0, dtype)
    kc0 = torch.randn(slots, H, D, generator=g).to(dtype)
    vc0 = torch.randn(slots, H, D, generator=g).to(dtype)
    # oracle
    rq, rk = ref_rope_neox(pos, qkv[:, : H * D], qkv[:, H * D : 2 * H * D], cache, D, elem_rounding=True)
    kc_ref, vc_ref = kc0.clone(), vc0.clone()
    ref_kv_append(rk.reshape(T, H, D), qkv[:, 2 * H * D :].reshape(T, H, D), kc_ref, vc_ref, sm)
    # fused
    d1 = qkv.to(dev)
    q1, k1, v1 = d1.chunk(3, dim=-1)
    kc1, vc1 = kc0.to(dev), vc0.to(dev)
    kernels.rope_and_cache(pos.to(dev), q1, k1, v1, cache.to(dev), D, kc1, vc1, sm.to(dev))
    # separate
    d2 = qkv.to(dev)
    q2, k2, v2 = d2.chunk(3, dim=-1)
    kc2, vc2 = kc0.to(dev), vc0.to(dev)
    kernels.vllm_rotary_emb(pos.to(dev), q2, k2, cache.to(dev), D)
    kernels.vllm_reshape_and_cache(k2.view(T, H, D), v2.view(T, H, D), kc2, vc2, sm.to(dev))
    assert torch.equal(_bits(d1.cpu()), _bits(d2.cpu()))
    assert torch.equal(_bits(kc1.cpu()), _bits(kc2.cpu())) and torch.equal(_bits(vc1.cpu()), _bits(vc2.cpu()))
    assert torch.equal(_bits(q1.cpu()), _bits(rq)) and torch.equal(_bits(k1.cpu()), _bits(rk))
    assert torch.equal(_bits(kc1.cpu()), _bits(kc_ref)) and torch.equal(_bits(vc1.cpu()), _bits(vc_ref))
    # without the write-back of k: q, v and both pools as before (k itself is left to the op)
    d3 = qkv.to(dev)
    q3, k3, v3 = d3.chunk(3, dim=-1)
    kc3, vc3 = kc0.to(dev), vc0.to(dev)
    kernels.rope_and_cache(pos.to(dev), q3, k3, v3, cache.to(dev), D, kc3, vc3, sm.to(dev), key_in_place=False)
    assert torch.equal(_bits(q3.cpu()), _bits(rq)) and torch.equal(_bits(v3.cpu()), _bits(qkv[:, 2 * H * D :]))
    assert torch.equal(_bits(kc3.cpu()), _bits(kc_ref)) and torch.equal(_bits(vc3.cpu()), _bits(vc_ref))
