"""GPU parity of decode attention (shared prefix on MFMA, per-request suffix,
LSE merge, plain ragged decode) against the CPU oracle on identical seeded inputs."""
import pytest
import torch

from oracle.ref_ops import ref_decode_attention, ref_partial, ref_shared_prefix_decode

pytestmark = pytest.mark.gpu

TOL = {torch.float16: dict(atol=2e-3, rtol=1e-2), torch.bfloat16: dict(atol=1e-2, rtol=2e-2)}


def _run_case(case, dev, chunk_tokens=None):
    from parrotserve_amd import kernels, synth

    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    tables = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                        case.pool_lists(case.suffix_lists), dev, num_heads=case.q.shape[1],
                                        head_dim=case.q.shape[2], dtype=case.dtype)
    if chunk_tokens is not None:
        tables.chunk_tokens = chunk_tokens
    out = kernels.decode_attention(case.q.to(dev), kc, vc, tables)
    torch.cuda.synchronize()
    return out.cpu()


def _check(case, dev, **kw):
    out = _run_case(case, dev, **kw)
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(out.float(), ref.float(), **TOL[case.dtype])
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,P,H", [(64, 1000, 8), (8, 512, 32), (33, 130, 4), (1, 64, 2), (100, 257, 4)])
def test_shared_prefix_decode(dev, dtype, B, P, H):
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(B * 7 + P)
    s = torch.randint(1, 200, (B,), generator=g).tolist()
    case = synth.make_decode_case("t", 100 + B, dtype, 1, B, P, s, H, 128, 1 << 14)
    _check(case, dev)


def test_config1_shape_in_fp16(dev):
    """Config 1's shape (B 8, P 512, S U[32,128], 32x128, seed 0) cast to fp16 for the GPU."""
    from parrotserve_amd import synth

    c = synth.config1()
    c.q, c.k_rows, c.v_rows, c.dtype = c.q.half(), c.k_rows.half(), c.v_rows.half(), torch.float16
    c.pool_slots = 4096
    c.used_slots = torch.randperm(4096, generator=torch.Generator().manual_seed(0))[: c.k_rows.shape[0]]
    _check(c, dev)


def test_config2_full_size(dev):
    """Config 2: fp16, B 64, one 4096-token prefix, suffix U[16,512], 32x128, 1M-slot pool, seed 1."""
    from parrotserve_amd import synth

    case = synth.config2()
    assert case.num_reqs == 64 and case.prefix_lists[0].numel() == 4096 and case.pool_slots == 1 << 20
    _check(case, dev)


def test_config5_full_size_attention(dev):
    """Config 5's attention at full size (4 groups x 32 branches, prefix 6000, suffix U[32,1024], 40x128, seed 4):
    the grouped shared-prefix path equals the non-shared ragged path over every request's whole context (two
    independent kernel paths on the GPU), and eight sampled requests equal the oracle."""
    from parrotserve_amd import kernels, synth

    gen = torch.Generator().manual_seed(4)
    s = torch.randint(32, 1025, (128,), generator=gen).tolist()  # the draw of synth.config5
    case = synth.make_decode_case("C5", 4, torch.float16, 4, 32, 6000, s, 40, 128, 1 << 18)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    q = case.q.to(dev)
    shared = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                        case.pool_lists(case.suffix_lists), dev, num_heads=40, head_dim=128)
    out = kernels.decode_attention(q, kc, vc, shared)
    full = case.full_lists()
    plain = kernels.DecodeTables.build([], [], [case.used_slots[l].tolist() for l in full], dev, num_heads=40,
                                       head_dim=128)
    out_plain = kernels.decode_attention(q, kc, vc, plain)
    torch.testing.assert_close(out.float(), out_plain.float(), **TOL[torch.float16])
    pick = [0, 31, 32, 50, 64, 95, 100, 127]
    ref = ref_decode_attention(case.q[pick], case.k_rows, case.v_rows, [full[i] for i in pick])
    torch.testing.assert_close(out[pick].cpu().float(), ref.float(), **TOL[torch.float16])


def _role_split(dev, case):
    """(prefix-only workgroups, compute units) the library gives a batch of this shape, read off the lane count it
    asks a plan to be cut into: lanes = 8 waves x (compute units - prefix workgroups) / head groups."""
    from parrotserve_amd import kernels

    B, H, D = case.q.shape
    P = max(len(p) for p in case.prefix_lists)
    S = max(len(x) for x in case.suffix_lists)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    lanes = kernels.suffix_lane_capacity(dev, H, D, num_reqs=B, num_groups=len(case.prefix_lists), max_prefix_len=P,
                                         max_suffix_len=S, dtype=case.dtype)
    heads_per_wave = 4 if D > 64 else 8  # a head takes D / 8 lanes of a wave, rounded up to a power of two
    hgroups = (H + heads_per_wave - 1) // heads_per_wave
    return cus - (lanes * hgroups + 7) // 8, cus


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_prefix_and_suffix_workgroups_of_their_own(dev, dtype):
    """A suffix-heavy batch (config 2's proportions at a quarter of its heads): the library gives the prefix phase
    workgroups of its own inside the one launch, the plan is cut for the rest, and the result equals the oracle --
    also with a plan cut for the whole device (more pieces than suffix waves: further rounds) and for a handful of
    lanes (fewer pieces than suffix workgroups)."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(21)
    s = torch.randint(300, 1100, (64,), generator=g).tolist()
    case = synth.make_decode_case("roles", 21, dtype, 1, 64, 2048, s, 8, 128, 1 << 17)
    np_, cus = _role_split(dev, case)
    assert 0 < np_ < cus, "this shape is meant to take the two-role launch"
    out = _check(case, dev)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    for lanes in (kernels.suffix_lane_capacity(dev, 8, 128), 5):
        tables = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                            case.pool_lists(case.suffix_lists), dev, num_heads=8, head_dim=128,
                                            dtype=dtype)
        tables.plan_on_device(lanes, dev)
        other = kernels.decode_attention(case.q.to(dev), kc, vc, tables).cpu()
        torch.testing.assert_close(other.float(), out.float(), **TOL[dtype])


@pytest.mark.parametrize("dtype,H,D", [(torch.float16, 8, 128), (torch.bfloat16, 8, 128), (torch.float16, 16, 64)])
def test_every_workgroup_runs_both_phases_when_the_launch_is_all_prefix(dev, dtype, H, D):
    """A long prefix under a handful of own tokens per request: the prefix wants every compute unit, so the library
    keeps the launch in which each workgroup streams its suffix pieces and then runs a prefix unit (no prefix-only
    workgroups: the lane count it asks for is the whole device's)."""
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(25)
    s = torch.randint(0, 9, (64,), generator=g).tolist()
    s[5] = 8
    case = synth.make_decode_case("allprefix", 25, dtype, 1, 64, 8192, s, H, D, 1 << 15)
    np_, cus = _role_split(dev, case)
    assert np_ == 0, "this shape is meant to take the launch whose workgroups run both phases"
    _check(case, dev)


def test_prefix_workgroups_walk_several_units_each(dev):
    """Eight groups x 32 heads are 256 prefix units per split -- more than the prefix-only workgroups of a device
    with that many compute units or fewer -- so every prefix workgroup walks several units back to back (the fold
    scratch of one is the staging ring of the next).  Groups of eight requests: the 64-query tile mostly empty."""
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(22)
    s = torch.randint(120, 400, (64,), generator=g).tolist()
    case = synth.make_decode_case("units", 22, torch.float16, 8, 8, 520, s, 32, 128, 1 << 16)
    np_, cus = _role_split(dev, case)
    assert 0 < np_ < 8 * 32, "prefix workgroups must be fewer than the prefix units"
    _check(case, dev)


def test_two_role_launch_with_empty_suffixes(dev):
    """Requests whose own list is empty inside a batch that takes the two-role launch (their output is the prefix
    part alone), and, with every list empty, the prefix phase on its own."""
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(23)
    s = torch.randint(500, 1200, (48,), generator=g).tolist()
    for b in (0, 7, 8, 30, 47):
        s[b] = 0
    case = synth.make_decode_case("empty", 23, torch.float16, 1, 48, 1500, s, 8, 128, 1 << 17)
    np_, cus = _role_split(dev, case)
    assert 0 < np_ < cus
    _check(case, dev)
    none = synth.make_decode_case("none", 24, torch.float16, 1, 48, 1500, [0] * 48, 8, 128, 1 << 17)
    _check(none, dev)


def test_multi_group_prefixes(dev):
    """Config-5 style: several prefix groups in one batch (scaled down)."""
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(5)
    s = torch.randint(32, 300, (4 * 32,), generator=g).tolist()
    case = synth.make_decode_case("g", 5, torch.float16, 4, 32, 700, s, 40, 128, 1 << 15)
    _check(case, dev)


def test_groups_of_different_prefix_length_and_ungrouped_requests(dev):
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(6)
    H, D, B = 8, 128, 50
    n_rows = 3000
    q = torch.randn(B, H, D, generator=g).half()
    k = torch.randn(n_rows, H, D, generator=g).half()
    v = torch.randn(n_rows, H, D, generator=g).half()
    perm = torch.randperm(n_rows, generator=g)
    pre = [perm[:900], perm[900:1000]]  # group 0: 900 tokens, group 1: 100 tokens
    gcu = [0, 20, 45]  # requests 45..49 have no prefix at all
    pos = 1000
    suf = []
    for b in range(B):
        n = int(torch.randint(0, 40, (1,), generator=g))  # some empty suffixes
        if b >= 45:
            n = max(n, 1)
        suf.append(perm[pos : pos + n])
        pos += n
    full = []
    for b in range(B):
        p = pre[0] if b < 20 else pre[1] if b < 45 else perm[:0]
        full.append(torch.cat([p, suf[b]]))
    ref = ref_decode_attention(q, k, v, full)
    tables = kernels.DecodeTables.build([p.tolist() for p in pre], gcu, [s.tolist() for s in suf], dev)
    out = kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), tables).cpu()
    torch.testing.assert_close(out.float(), ref.float(), **TOL[torch.float16])


@pytest.mark.parametrize("chunk", [16, 64, 1024])
def test_suffix_chunking_is_invisible(dev, chunk):
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(7)
    s = torch.randint(1, 700, (16,), generator=g).tolist()
    case = synth.make_decode_case("c", 7, torch.float16, 1, 16, 0, s, 8, 128, 1 << 14)
    _check(case, dev, chunk_tokens=chunk)


@pytest.mark.parametrize("D,H", [(64, 12), (256, 3), (128, 5), (80, 32), (80, 5), (96, 7), (112, 3)])
def test_other_head_sizes_and_odd_head_counts(dev, D, H):
    """Every head size the reference's kernels dispatch (csrc/attention/attention_post_kernels.cu:420-446:
    64, 80, 96, 112, 128, 256); 80 x 32 is OPT-2.7B's shape."""
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(8)
    s = torch.randint(1, 150, (9,), generator=g).tolist()
    case = synth.make_decode_case("d", 8 + D, torch.float16, 1, 9, 200, s, H, D, 1 << 12)
    _check(case, dev)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [80, 96, 112])
def test_short_heads_on_the_wide_prefix_tile(dev, D, dtype):
    """Head sizes 80 / 96 / 112: the prefix phase on the matrix cores as short heads on the 128-wide tile (their
    padding lanes re-read the row's first chunk, the query's padding dims are zero, the partial rows are D floats
    long), in every query-tile form (groups of 20, 70, 150 and 300 requests), several groups, a prefix longer than
    one split; the suffix phase per request at the head's own size."""
    from parrotserve_amd import synth

    for sizes, P, H in (([20], 300, 5), ([70, 33], 700, 3), ([150], 1300, 2), ([300, 9], 520, 2)):
        g = torch.Generator().manual_seed(600 + D + sizes[0])
        s = torch.randint(0, 60, (sum(sizes),), generator=g).tolist()
        case = synth.make_decode_case("sh", 600 + D + sizes[0], dtype, len(sizes), 0, P, s, H, D, 1 << 15,
                                      group_sizes=sizes)
        _check(case, dev)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 80, 96, 112, 128, 256])
def test_vllm_test_distribution_over_head_sizes(dev, D, dtype):
    """The vendored vLLM kernel test's inputs (3rdparty/vllm/tests/kernels/test_attention.py:159-246): q, k, v uniform
    in [-1e-3, 1e-3], 7 sequences of random length, every head size its kernels take.  Outputs are of the order of
    1e-5, so the comparison is relative with a floor two orders below them instead of that test's atol of 1e-3."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(D)
    B, H = 7, 12
    lens = torch.randint(1, 300, (B,), generator=g).tolist()
    total = sum(lens)
    uni = lambda *shape: ((torch.rand(*shape, generator=g) * 2 - 1) * 1e-3).to(dtype)  # noqa: E731
    q, k, v = uni(B, H, D), uni(total + 5, H, D), uni(total + 5, H, D)
    perm = torch.randperm(total + 5, generator=g)
    lists, pos = [], 0
    for n in lens:
        lists.append(perm[pos:pos + n])
        pos += n
    ref = ref_decode_attention(q, k, v, lists)
    width = max(lens)
    table = torch.zeros((B, width), dtype=torch.int32)
    for i, x in enumerate(lists):
        table[i, : len(x)] = x.to(torch.int32)
    hm = torch.arange(H, dtype=torch.int32, device=dev)
    out = kernels.vllm_paged_attention(q.to(dev), k.to(dev), v.to(dev), hm, torch.tensor(lens, dtype=torch.int32, device=dev),
                                       table.to(dev)).cpu()
    rel = 1e-2 if dtype == torch.float16 else 2e-2
    torch.testing.assert_close(out.float(), ref.float(), atol=2e-7 if dtype == torch.float16 else 1e-6, rtol=rel)


def test_config3_ragged_decode_scaled(dev):
    """Config 3's distribution (ctx log-uniform[128,8192], 32x128) on 32 of the 256 requests."""
    from parrotserve_amd import synth

    case = synth.config3(batch=32, pool_slots=1 << 18)
    assert all(128 <= l.numel() <= 8192 for l in case.suffix_lists)
    _check(case, dev)


def test_config3_full_size_properties(dev):
    """Config 3 at full size (B 256, ctx log-uniform[128,8192], 32x128, 4M-slot pool of device-generated rows):
    the balanced form and the plain grid form agree, a value cache of ones gives ones (softmax weights sum to one
    over every ragged list), and the four shortest requests equal the oracle on their own rows."""
    from parrotserve_amd import kernels, synth

    pool = 1 << 22
    case = synth.config3(batch=256, pool_slots=pool)
    lists = case.pool_lists(case.suffix_lists)
    assert len(lists) == 256 and sum(len(l) for l in lists) > 300000
    gen = torch.Generator(device=dev).manual_seed(3)
    kc = torch.randn((pool, 32, 128), generator=gen, device=dev, dtype=torch.float16)
    vc = torch.randn((pool, 32, 128), generator=gen, device=dev, dtype=torch.float16)
    q = case.q.to(dev)
    balanced = kernels.DecodeTables.build([], [], lists, dev)
    grid = kernels.DecodeTables.build([], [], lists, dev, balanced=False)
    out = kernels.decode_attention(q, kc, vc, balanced)
    out_grid = kernels.decode_attention(q, kc, vc, grid)
    torch.testing.assert_close(out.float(), out_grid.float(), **TOL[torch.float16])
    short = sorted(range(256), key=lambda i: len(lists[i]))[:4]
    for i in short:
        rows = torch.tensor(lists[i], device=dev)
        ref = ref_decode_attention(case.q[i:i + 1], kc[rows].cpu(), vc[rows].cpu(), [torch.arange(len(lists[i]))])
        torch.testing.assert_close(out[i:i + 1].cpu().float(), ref.float(), **TOL[torch.float16])
    vc.fill_(1.0)
    ones = kernels.decode_attention(q, kc, vc, balanced)
    torch.testing.assert_close(ones.float(), torch.ones_like(ones).float(), atol=2e-3, rtol=0)
    del kc, vc
    torch.cuda.empty_cache()  # 69 GB of pool rows


def test_reference_named_entry_points(dev):
    """flash_paged_attention / paged_flash_attention / vllm_paged_attention with the
    reference's argument lists (padded 2-D tables, int32 lens)."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(9)
    B, P, H, D = 16, 300, 8, 128
    s = torch.randint(1, 90, (B,), generator=g).tolist()
    case = synth.make_decode_case("r", 9, torch.float16, 1, B, P, s, H, D, 1 << 12)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    suf = case.pool_lists(case.suffix_lists)
    mx = max(len(x) for x in suf)
    table = torch.tensor([x + [0] * (mx - len(x)) for x in suf], dtype=torch.int32, device=dev)
    lens = torch.tensor([len(x) for x in suf], dtype=torch.int32, device=dev)
    flash = torch.tensor(case.pool_lists(case.prefix_lists)[0], dtype=torch.int32, device=dev)
    hm = torch.arange(H, dtype=torch.int32, device=dev)
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    for fn in (kernels.flash_paged_attention, kernels.paged_flash_attention):
        out = fn(case.q.to(dev), kc, vc, hm, P, flash, lens, table).cpu()
        torch.testing.assert_close(out.float(), ref.float(), **TOL[torch.float16])
    # no shared prefix (P = 0): suffix only -- the reference is fragile here, this build defines it
    out0 = kernels.flash_paged_attention(case.q.to(dev), kc, vc, hm, 0, flash[:0], lens, table).cpu()
    ref0 = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.suffix_lists)
    torch.testing.assert_close(out0.float(), ref0.float(), **TOL[torch.float16])
    # non-shared path over the full context
    full = [case.used_slots[l].tolist() for l in case.full_lists()]
    mx = max(len(x) for x in full)
    ftable = torch.tensor([x + [0] * (mx - len(x)) for x in full], dtype=torch.int32, device=dev)
    flens = torch.tensor([len(x) for x in full], dtype=torch.int32, device=dev)
    out1 = kernels.vllm_paged_attention(case.q.to(dev), kc, vc, hm, flens, ftable).cpu()
    torch.testing.assert_close(out1.float(), ref.float(), **TOL[torch.float16])


def test_reference_named_ops_reuse_the_plan_across_layers_and_notice_new_lengths(dev):
    """The reference-named ops keep the device tables and suffix plan of a call for the next call with the same
    tensors (the next layer of the iteration).  Lengths rewritten in place through torch must not find the old
    plan: the second result is checked against the oracle on the new lengths."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(10)
    B, P, H, D = 24, 260, 8, 128
    s = torch.randint(20, 90, (B,), generator=g).tolist()
    case = synth.make_decode_case("rc", 10, torch.float16, 1, B, P, s, H, D, 1 << 12)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    suf = case.pool_lists(case.suffix_lists)
    mx = max(len(x) for x in suf)
    table = torch.tensor([x + [0] * (mx - len(x)) for x in suf], dtype=torch.int32, device=dev)
    lens = torch.tensor([len(x) for x in suf], dtype=torch.int32, device=dev)
    flash = torch.tensor(case.pool_lists(case.prefix_lists)[0], dtype=torch.int32, device=dev)
    hm = torch.arange(H, dtype=torch.int32, device=dev)
    q = case.q.to(dev)
    kernels._paged_tables_cache.clear()
    out_a = kernels.flash_paged_attention(q, kc, vc, hm, P, flash, lens, table)
    assert len(kernels._paged_tables_cache) == 1
    tables_a = next(iter(kernels._paged_tables_cache.values()))[1]
    out_b = kernels.flash_paged_attention(q, kc, vc, hm, P, flash, lens, table)  # "layer 2": same tensors
    assert len(kernels._paged_tables_cache) == 1
    assert next(iter(kernels._paged_tables_cache.values()))[1] is tables_a
    assert torch.equal(out_a, out_b)
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(out_a.cpu().float(), ref.float(), **TOL[torch.float16])
    # the next iteration, written into the same tensor: every list one to nineteen tokens shorter
    cut = torch.randint(1, 20, (B,), generator=g)
    lens.sub_(cut.to(torch.int32).to(dev))
    out_c = kernels.flash_paged_attention(q, kc, vc, hm, P, flash, lens, table)
    assert len(kernels._paged_tables_cache) == 2
    short = [torch.cat([case.prefix_lists[0], l[: l.numel() - int(c)]]) for l, c in zip(case.suffix_lists, cut)]
    ref_c = ref_decode_attention(case.q, case.k_rows, case.v_rows, short)
    torch.testing.assert_close(out_c.cpu().float(), ref_c.float(), **TOL[torch.float16])


def _gqa_case(dtype, B, P, Hq, Hkv, D, seed, smax=90, pool=1 << 13):
    """A shared-prefix decode case with Hq query heads over Hkv KV heads: the case is drawn with Hkv heads and the
    query widened to Hq."""
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(seed)
    s = torch.randint(1, smax, (B,), generator=g).tolist()
    case = synth.make_decode_case("gqa", seed, dtype, 1, B, P, s, Hkv, D, pool)
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    return case, q


def _paged_inputs(case, dev):
    suf = case.pool_lists(case.suffix_lists)
    mx = max(len(x) for x in suf)
    table = torch.tensor([x + [0] * (mx - len(x)) for x in suf], dtype=torch.int32, device=dev)
    lens = torch.tensor([len(x) for x in suf], dtype=torch.int32, device=dev)
    flash = torch.tensor(case.pool_lists(case.prefix_lists)[0], dtype=torch.int32, device=dev)
    return flash, lens, table


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,P", [(48, 700), (7, 150)])
def test_grouped_kv_heads(dev, dtype, D, B, P):
    """head_mapping = repeat_interleave(arange(H / 4), 4): four query heads share each KV head
    (csrc/attention/attention_post_kernels.cu:79,101).  flash_paged_attention and vllm_paged_attention against an
    oracle that gathers KV head h // 4 for query head h."""
    from parrotserve_amd import kernels, synth

    Hq, Hkv = 16, 4
    case, q = _gqa_case(dtype, B, P, Hq, Hkv, D, 300 + B + D)
    hm = torch.arange(Hkv, dtype=torch.int32).repeat_interleave(Hq // Hkv)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    flash, lens, table = _paged_inputs(case, dev)
    ref = ref_decode_attention(q, case.k_rows[:, hm.long()], case.v_rows[:, hm.long()], case.full_lists())
    out = kernels.flash_paged_attention(q.to(dev), kc, vc, hm.to(dev), P, flash, lens, table)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[dtype])
    full = [case.used_slots[l].tolist() for l in case.full_lists()]
    mx = max(len(x) for x in full)
    ftable = torch.tensor([x + [0] * (mx - len(x)) for x in full], dtype=torch.int32, device=dev)
    flens = torch.tensor([len(x) for x in full], dtype=torch.int32, device=dev)
    out1 = kernels.vllm_paged_attention(q.to(dev), kc, vc, hm.to(dev), flens, ftable)
    torch.testing.assert_close(out1.cpu().float(), ref.float(), **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv", [(16, 2), (12, 3), (40, 5), (8, 2), (32, 2)])
def test_query_heads_of_a_kv_head_streamed_together(dev, dtype, Hq, Hkv):
    """Groups of 16, 8 and 4 query heads per KV head at head size 128: the suffix waves divide runs of four query heads
    that share a KV head and meet every token row with the run's queries at once (run counts that fill a wave's four
    head slots, leave some empty, and need further waves).  Through the reference-named ops (plan cut for the grouped form), with a plan
    cut for the plain form (fewer pieces than the grouped launch has room for), and without a prefix."""
    from parrotserve_amd import kernels, synth

    B, P, D, G = 70, 420, 128, Hq // Hkv
    case, q = _gqa_case(dtype, B, P, Hq, Hkv, D, 600 + Hq, smax=260, pool=1 << 15)  # lists long enough for the form
    hm = torch.arange(Hkv, dtype=torch.int32).repeat_interleave(G)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    flash, lens, table = _paged_inputs(case, dev)
    ref = ref_decode_attention(q, case.k_rows[:, hm.long()], case.v_rows[:, hm.long()], case.full_lists())
    out = kernels.flash_paged_attention(q.to(dev), kc, vc, hm.to(dev), P, flash, lens, table)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[dtype])
    plain = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                       case.pool_lists(case.suffix_lists), dev, num_heads=Hq, head_dim=D, dtype=dtype)
    out2 = kernels.decode_attention(q.to(dev), kc, vc, plain, head_mapping=hm.to(dev), kv_group=G)
    torch.testing.assert_close(out2.cpu().float(), ref.float(), **TOL[dtype])
    full = [case.used_slots[l].tolist() for l in case.full_lists()]
    mx = max(len(x) for x in full)
    ftable = torch.tensor([x + [0] * (mx - len(x)) for x in full], dtype=torch.int32, device=dev)
    flens = torch.tensor([len(x) for x in full], dtype=torch.int32, device=dev)
    out3 = kernels.vllm_paged_attention(q.to(dev), kc, vc, hm.to(dev), flens, ftable)
    torch.testing.assert_close(out3.cpu().float(), ref.float(), **TOL[dtype])


def test_any_head_mapping_and_the_identity(dev):
    """A mapping that is not h // G (here a permutation with repeats) runs per request; multi-query attention (one
    KV head); and the identity mapping over equal head counts is the plain call, bit for bit.  The split entry
    points (paged_flash_attention) take the identity only and say so."""
    from parrotserve_amd import kernels, synth

    dtype, D, B, P = torch.float16, 128, 20, 333
    for Hq, Hkv, hm in ((6, 3, [2, 0, 0, 1, 2, 1]), (8, 1, [0] * 8), (12, 4, [0, 0, 0, 1, 1, 1, 2, 2, 2, 3, 3, 3])):
        case, q = _gqa_case(dtype, B, P, Hq, Hkv, D, 400 + Hq)
        hm_t = torch.tensor(hm, dtype=torch.int32)
        kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
        flash, lens, table = _paged_inputs(case, dev)
        ref = ref_decode_attention(q, case.k_rows[:, hm_t.long()], case.v_rows[:, hm_t.long()], case.full_lists())
        out = kernels.flash_paged_attention(q.to(dev), kc, vc, hm_t.to(dev), P, flash, lens, table)
        torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[dtype])
        with pytest.raises(ValueError, match="head_mapping"):
            kernels.paged_flash_attention(q.to(dev), kc, vc, hm_t.to(dev), P, flash, lens, table)
    # identity: the same kernels as a call without any mapping
    case, q = _gqa_case(dtype, B, P, 8, 8, D, 77)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    flash, lens, table = _paged_inputs(case, dev)
    ident = torch.arange(8, dtype=torch.int32, device=dev)
    a = kernels.flash_paged_attention(q.to(dev), kc, vc, ident, P, flash, lens, table)
    tabs = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                      case.pool_lists(case.suffix_lists), dev, num_heads=8, head_dim=D)
    b = kernels.decode_attention(q.to(dev), kc, vc, tabs)
    assert torch.equal(a, b)
    with pytest.raises(ValueError, match="head_mapping"):  # a KV head the cache does not have
        kernels.flash_paged_attention(q.to(dev), kc, vc, ident + 1, P, flash, lens, table)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_grouped_kv_heads_on_the_matrix_cores_at_config2_proportions(dev, dtype):
    """Grouped KV heads where the call runs the prefix and suffix phases in one launch with workgroups of their own:
    64 requests x 32 query heads over 8 KV heads (G = 4: 256 query rows per KV head and tile), and two groups of
    40 over 16 -> 8 heads (G = 2)."""
    from parrotserve_amd import kernels, synth

    for B, groups, P, Hq, Hkv, lo, hi in ((64, 1, 1536, 32, 8, 200, 700), (80, 2, 600, 16, 8, 100, 500)):
        g = torch.Generator().manual_seed(500 + B)
        s = torch.randint(lo, hi, (B,), generator=g).tolist()
        case = synth.make_decode_case("gqa2", 500 + B, dtype, groups, B // groups, P, s, Hkv, 128, 1 << 17)
        q = torch.randn(B, Hq, 128, generator=g).to(dtype)
        hm = torch.arange(Hkv, dtype=torch.int32).repeat_interleave(Hq // Hkv)
        kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
        tabs = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                          case.pool_lists(case.suffix_lists), dev, num_heads=Hq, head_dim=128,
                                          dtype=dtype)
        out = kernels.decode_attention(q.to(dev), kc, vc, tabs, head_mapping=hm.to(dev), kv_group=Hq // Hkv)
        ref = ref_decode_attention(q, case.k_rows[:, hm.long()], case.v_rows[:, hm.long()], case.full_lists())
        torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[dtype])


def test_timed_call_is_the_same_call_with_timestamps(dev):
    """``ph_decode_attention_timed`` launches what ``ph_decode_attention`` launches (same bits out) and stamps the
    caller's events with its own dispatches: three begin / end pairs, each end after its begin, the merge after
    the kernel that feeds it; a pair whose kernel the call does not launch (no separate prefix kernel when both
    phases share one launch) stays unrecorded."""
    import ctypes

    from parrotserve_amd import kernels, synth

    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
    hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
    hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]

    def elapsed(a, b):
        ms = ctypes.c_float()
        rc = hip.hipEventElapsedTime(ctypes.byref(ms), a, b)
        if rc != 0:
            hip.hipGetLastError()
            return None
        return ms.value

    g = torch.Generator().manual_seed(77)
    # head size 128: one launch for both phases; 96 (a short head on the wide tile): a prefix launch of its own
    for B, D, expect_prefix_pair in ((64, 128, False), (16, 128, False), (16, 96, True)):
        s = torch.randint(1, 150, (B,), generator=g).tolist()
        case = synth.make_decode_case("t", 500 + B, torch.float16, 1, B, 700, s, 8, D, 1 << 14)
        kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
        tables = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                            case.pool_lists(case.suffix_lists), dev, num_heads=8, head_dim=D)
        q = case.q.to(dev)
        plain = kernels.decode_attention(q, kc, vc, tables)
        evs = (ctypes.c_void_p * 6)()
        for i in range(6):
            e = ctypes.c_void_p()
            assert hip.hipEventCreate(ctypes.byref(e)) == 0
            evs[i] = e
        timed = kernels.decode_attention(q, kc, vc, tables, events6=evs)
        torch.cuda.synchronize()
        assert torch.equal(plain.view(torch.int16), timed.view(torch.int16))
        t_prefix, t_suffix, t_merge = elapsed(evs[0], evs[1]), elapsed(evs[2], evs[3]), elapsed(evs[4], evs[5])
        assert t_suffix is not None and 0 < t_suffix < 50 and t_merge is not None and 0 < t_merge < 50
        assert elapsed(evs[3], evs[4]) >= 0  # the merge begins after the suffix kernel ended
        assert (t_prefix is not None) == expect_prefix_pair
        if expect_prefix_pair:
            assert 0 < t_prefix < 50
        for i in range(6):
            hip.hipEventDestroy(evs[i])
        ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
        torch.testing.assert_close(timed.cpu().float(), ref.float(), **TOL[torch.float16])


@pytest.mark.parametrize("balanced", [True, False])
def test_lengths_beyond_the_table_are_clamped(dev, balanced):
    """A context length larger than the table's width must not walk into the next request's row (or past the
    table): the kernels read it clamped to the width, so the result is that of the full row."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(31)
    B, H, D, W = 6, 4, 128, 24
    k = torch.randn(B * W, H, D, generator=g).half()
    v = torch.randn(B * W, H, D, generator=g).half()
    q = torch.randn(B, H, D, generator=g).half()
    rows = torch.randperm(B * W, generator=g).view(B, W)
    good = torch.tensor([W, 5, W, 1, 17, W], dtype=torch.int32)
    bad = good.clone()
    bad[0], bad[2], bad[5] = W + 9, 100000, 2 ** 31 - 1
    ref = ref_decode_attention(q, k, v, [rows[b, : int(good[b])] for b in range(B)])
    table = rows.to(torch.int32).to(dev)
    hm = torch.arange(H, dtype=torch.int32, device=dev)
    if balanced:
        out = kernels.vllm_paged_attention(q.to(dev), k.to(dev), v.to(dev), hm, bad.to(dev), table)
    else:
        t = kernels.DecodeTables(num_reqs=B, suffix_slots=table, suffix_table_stride=W, suffix_lens=bad.to(dev),
                                 max_suffix_len=W, chunk_tokens=16)
        out = kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), t)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[torch.float16])


@pytest.mark.parametrize("B,grouped", [(8192, True), (8193, False), (9000, True)])
def test_batches_around_the_device_planner_limit(dev, B, grouped):
    """The suffix plan is written on the device for up to 8192 requests and on the host beyond; thousands of
    requests with one to three tokens each (and a 40-token prefix every request shares) against the oracle."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(5 + B)
    H, D = 2, 128
    lens = torch.randint(1, 4, (B,), generator=g).tolist()
    total, P = sum(lens), (40 if grouped else 0)
    perm = torch.randperm(total + P + 16, generator=g)
    k = torch.randn(total + P + 16, H, D, generator=g).half()
    v = torch.randn(total + P + 16, H, D, generator=g).half()
    q = torch.randn(B, H, D, generator=g).half()
    pre, pos, suf = perm[:P], P, []
    for n in lens:
        suf.append(perm[pos:pos + n])
        pos += n
    t = kernels.DecodeTables.build([pre.tolist()] if grouped else [], [0, B] if grouped else [],
                                   [s.tolist() for s in suf], dev, num_heads=H, head_dim=D)
    assert t.plan is not None
    out = kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), t).cpu()
    ref = ref_decode_attention(q, k, v, [torch.cat([pre, s]) for s in suf])
    torch.testing.assert_close(out.float(), ref.float(), **TOL[torch.float16])


def test_reference_self_test_harness_shape(dev):
    """The reference's own kernel check (kernels/shared_flash_decoding.py:417-459 and kernels/vllm/paged_attention.py:
    81-134): 16 sequences of 1024 tokens, 48 heads of 64, contexts laid out back to back in the cache, inputs N(0, 1),
    seed 2023, compared with its in-file formula at atol = rtol = 1e-2 -- here on the token-granular layout (a block
    table is a slot list), against the oracle, at this build's tighter tolerance."""
    from parrotserve_amd import kernels

    torch.manual_seed(2023)
    B, H, D, L = 16, 48, 64, 1024
    q = torch.randn(B, H, D).half()
    k = torch.randn(B * L + 64, H, D).half()
    v = torch.randn(B * L + 64, H, D).half()
    tables = torch.arange(B * L, dtype=torch.int32).reshape(B, L)
    lens = torch.full((B,), L, dtype=torch.int32)
    ref = ref_decode_attention(q, k, v, [tables[b].long() for b in range(B)])
    hm = torch.arange(H, dtype=torch.int32, device=dev)
    out = kernels.vllm_paged_attention(q.to(dev), k.to(dev), v.to(dev), hm, lens.to(dev), tables.to(dev)).cpu()
    torch.testing.assert_close(out.float(), ref.float(), **TOL[torch.float16])
    # the same contexts with their first 768 tokens declared as a prefix every sequence shares (sequence 0's slots)
    P = 768
    shared = torch.cat([tables[:1, :P].expand(B, P), tables[:, P:]], dim=1)
    ref2 = ref_decode_attention(q, k, v, [shared[b].long() for b in range(B)])
    for fn in (kernels.flash_paged_attention, kernels.paged_flash_attention):
        out2 = fn(q.to(dev), k.to(dev), v.to(dev), hm, P, tables[0, :P].to(dev), (lens - P).to(dev),
                  tables[:, P:].contiguous().to(dev)).cpu()
        torch.testing.assert_close(out2.float(), ref2.float(), **TOL[torch.float16])


def test_shared_equals_non_shared_property(dev):
    """Size-independent property at config-2 scale: the shared-prefix path and the
    non-shared ragged path agree (both on the GPU), and softmax weights sum to one
    (all-ones V gives all-ones output)."""
    from parrotserve_amd import kernels, synth

    case = synth.config2(batch=64, prefix=4096, pool_slots=1 << 17)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    t_shared = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                          case.pool_lists(case.suffix_lists), dev)
    t_plain = kernels.DecodeTables.build([], [], case.pool_lists(case.full_lists()), dev)
    q = case.q.to(dev)
    a = kernels.decode_attention(q, kc, vc, t_shared)
    b = kernels.decode_attention(q, kc, vc, t_plain)
    torch.testing.assert_close(a.float(), b.float(), atol=2e-3, rtol=1e-2)
    ones = torch.ones_like(vc)
    c = kernels.decode_attention(q, kc, ones, t_shared)
    torch.testing.assert_close(c.float(), torch.ones_like(c).float(), atol=2e-3, rtol=0)


def test_unsupported_inputs_raise(dev):
    from parrotserve_amd import kernels

    q = torch.zeros(2, 2, 72, dtype=torch.float16, device=dev)
    kc = torch.zeros(8, 2, 72, dtype=torch.float16, device=dev)
    t = kernels.DecodeTables.build([], [], [[0, 1], [2]], dev)
    with pytest.raises(RuntimeError, match="head size"):
        kernels.decode_attention(q, kc, kc, t)
    q64 = torch.zeros(2, 2, 128, dtype=torch.float64, device=dev)  # float16 / bfloat16 / float32 are the element types
    with pytest.raises(RuntimeError, match="data type"):
        kernels.decode_attention(q64, q64.new_zeros(8, 2, 128), q64.new_zeros(8, 2, 128), t)


def test_balanced_and_grid_suffix_forms_agree(dev):
    """The host-planned balanced suffix phase and the grid-of-chunks form give the same result (and both
    match the oracle) on ragged lengths including empty and one-token suffixes."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(21)
    s = [0, 1, 2, 700, 33, 64, 65, 0, 511, 5] + torch.randint(1, 300, (40,), generator=g).tolist()
    case = synth.make_decode_case("bg", 21, torch.float16, 1, len(s), 300, s, 8, 128, 1 << 14)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    pre, suf = case.pool_lists(case.prefix_lists), case.pool_lists(case.suffix_lists)
    ta = kernels.DecodeTables.build(pre, case.group_req_cu, suf, dev, num_heads=8, balanced=True)
    tb = kernels.DecodeTables.build(pre, case.group_req_cu, suf, dev, num_heads=8, balanced=False)
    assert ta.plan is not None and tb.plan is None
    q = case.q.to(dev)
    a = kernels.decode_attention(q, kc, vc, ta).cpu()
    b = kernels.decode_attention(q, kc, vc, tb).cpu()
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(a.float(), ref.float(), **TOL[torch.float16])
    torch.testing.assert_close(b.float(), ref.float(), **TOL[torch.float16])
    torch.testing.assert_close(a.float(), b.float(), atol=1e-3, rtol=1e-2)


def test_prefix_longer_than_slot_window(dev):
    """Eight groups of 33 requests over 4200-token prefixes, 32 heads: enough workgroups that the planner
    leaves each prefix in one split, so a workgroup walks more than the 4096 slot ids it keeps on chip."""
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(11)
    s = torch.randint(1, 40, (8 * 33,), generator=g).tolist()
    case = synth.make_decode_case("w", 11, torch.float16, 8, 33, 4200, s, 32, 128, 1 << 16)
    _check(case, dev)


def _split_halves_case(dtype, B, P, H, seed, D=128):
    from parrotserve_amd import synth

    g = torch.Generator().manual_seed(seed)
    s = torch.randint(1, 150, (B,), generator=g).tolist()
    s[0] = 0 if B > 1 else s[0]  # one request without a suffix
    return synth.make_decode_case("halves", seed, dtype, 1, B, P, s, H, D, 1 << 14)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,P,H,D", [(64, 700, 8, 128), (20, 333, 4, 128), (40, 500, 6, 64), (7, 129, 3, 64)])
def test_prefix_and_post_entry_points(dev, dtype, B, P, H, D):
    """The two halves exported separately, called through the C ABI the way the reference calls its Triton
    prefix kernel (O, row max and denominator out) and then its post kernel (suffix + merge in place)."""
    import ctypes

    from parrotserve_amd import _lib, kernels, synth

    case = _split_halves_case(dtype, B, P, H, 40 + B, D)
    lib = _lib.load()
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    q = case.q.to(dev)
    out = torch.zeros_like(q)
    m = torch.empty((B, H), dtype=torch.float32, device=dev)
    l = torch.empty((B, H), dtype=torch.float32, device=dev)
    prefix = case.pool_lists(case.prefix_lists)[0]
    pslots = torch.tensor(prefix, dtype=torch.int32, device=dev)
    suffix = case.pool_lists(case.suffix_lists)
    width = max(1, max(len(x) for x in suffix))
    table = torch.zeros((B, width), dtype=torch.int32)
    for i, x in enumerate(suffix):
        table[i, : len(x)] = torch.tensor(x, dtype=torch.int32)
    table = table.to(dev)
    lens = torch.tensor([len(x) for x in suffix], dtype=torch.int32, device=dev)
    nbytes = lib.ph_decode_workspace_bytes(B, H, D, 1, P, width, 0, 0)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    scale = D ** -0.5
    st = torch.cuda.current_stream().cuda_stream
    code = 0 if dtype == torch.float16 else 1
    rc = lib.ph_prefix_attention(out.data_ptr(), m.data_ptr(), l.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                 B, H, D, code, q.stride(0), out.stride(0), kc.stride(0), scale,
                                 pslots.data_ptr(), P, ws.data_ptr(), nbytes, st)
    assert rc == 0
    torch.cuda.synchronize()
    # prefix half against the oracle's partial: normalised O, row max (exp2 domain) and denominator
    ridx = [case.prefix_lists[0]] * B
    o_ref, m_ref, l_ref = ref_partial(case.q, case.k_rows, case.v_rows, ridx, scale)
    torch.testing.assert_close(out.cpu().float(), o_ref.float(), **TOL[dtype])
    torch.testing.assert_close(m.cpu(), m_ref, atol=1e-3, rtol=1e-4)
    torch.testing.assert_close(l.cpu(), l_ref, atol=1e-3, rtol=2e-2 if dtype == torch.bfloat16 else 5e-3)
    rc = lib.ph_suffix_post_attention(out.data_ptr(), m.data_ptr(), l.data_ptr(), q.data_ptr(), kc.data_ptr(),
                                      vc.data_ptr(), B, H, D, code, q.stride(0), out.stride(0), kc.stride(0), scale,
                                      table.data_ptr(), None, table.stride(0), table.numel(), lens.data_ptr(),
                                      width, 0, ws.data_ptr(), nbytes, st)
    assert rc == 0
    torch.cuda.synchronize()
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[dtype])
    # the other order (shared_flash_decoding.py:332-376): suffix phase first with its (m, l) exported, then the
    # prefix phase merged on top
    out2 = torch.zeros_like(q)
    m2 = torch.empty_like(m)
    l2 = torch.empty_like(l)
    rc = lib.ph_suffix_prev_attention(out2.data_ptr(), m2.data_ptr(), l2.data_ptr(), q.data_ptr(), kc.data_ptr(),
                                      vc.data_ptr(), B, H, D, code, q.stride(0), out2.stride(0), kc.stride(0), scale,
                                      table.data_ptr(), None, table.stride(0), table.numel(), lens.data_ptr(),
                                      width, 0, ws.data_ptr(), nbytes, st)
    assert rc == 0
    torch.cuda.synchronize()
    so_ref, sm_ref, sl_ref = ref_partial(case.q, case.k_rows, case.v_rows, case.suffix_lists, scale)
    has = torch.tensor([len(x) > 0 for x in suffix])
    torch.testing.assert_close(out2.cpu().float()[has], so_ref.float()[has], **TOL[dtype])
    torch.testing.assert_close(m2.cpu()[has], sm_ref[has], atol=1e-3, rtol=1e-4)
    torch.testing.assert_close(l2.cpu()[has], sl_ref[has], atol=1e-3, rtol=2e-2 if dtype == torch.bfloat16 else 5e-3)
    assert (l2.cpu()[~has] == 0).all()  # no suffix: an empty partial
    rc = lib.ph_prefix_post_attention(out2.data_ptr(), m2.data_ptr(), l2.data_ptr(), q.data_ptr(), kc.data_ptr(),
                                      vc.data_ptr(), B, H, D, code, q.stride(0), out2.stride(0), kc.stride(0), scale,
                                      pslots.data_ptr(), P, ws.data_ptr(), nbytes, st)
    assert rc == 0
    torch.cuda.synchronize()
    torch.testing.assert_close(out2.cpu().float(), ref.float(), **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_single_launch_path_with_uneven_groups(dev, dtype):
    """Groups large enough for the path that runs the prefix and suffix phases in one launch, shaped to reach its
    corners: prefixes of very different lengths (the short groups' later splits are empty), a group of more than
    64 requests (two query tiles), more prefix units than workgroups (a workgroup runs several), requests with
    no prefix and requests with no suffix, and a batch whose suffix stream is shorter than the prefix work."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(21)
    H, D = 40, 128
    sizes = [40, 70, 33]
    plens = [90, 2600, 700]
    B = sum(sizes) + 4
    n_rows = 6000
    q = torch.randn(B, H, D, generator=g).to(dtype)
    k = torch.randn(n_rows, H, D, generator=g).to(dtype)
    v = torch.randn(n_rows, H, D, generator=g).to(dtype)
    perm = torch.randperm(n_rows, generator=g)
    pre, pos = [], 0
    for n in plens:
        pre.append(perm[pos:pos + n])
        pos += n
    gcu = [0]
    for n in sizes:
        gcu.append(gcu[-1] + n)
    suf = []
    for b in range(B):
        n = int(torch.randint(0, 12, (1,), generator=g))
        if b >= gcu[-1]:
            n = max(n, 1)  # ungrouped requests need something to attend to
        suf.append(perm[pos:pos + n])
        pos += n
    full = []
    for b in range(B):
        grp = next((i for i in range(len(sizes)) if gcu[i] <= b < gcu[i + 1]), None)
        full.append(torch.cat([pre[grp] if grp is not None else perm[:0], suf[b]]))
    ref = ref_decode_attention(q, k, v, full)
    tables = kernels.DecodeTables.build([p.tolist() for p in pre], gcu, [s.tolist() for s in suf], dev, num_heads=H,
                                        head_dim=D)
    assert tables.plan is not None
    out = kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), tables).cpu()
    torch.testing.assert_close(out.float(), ref.float(), **TOL[dtype])
    # the same batch as separate launches (no plan) must agree with the single launch
    grid = kernels.DecodeTables.build([p.tolist() for p in pre], gcu, [s.tolist() for s in suf], dev, num_heads=H,
                                      head_dim=D, balanced=False)
    out2 = kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), grid).cpu()
    torch.testing.assert_close(out2.float(), ref.float(), **TOL[dtype])
    torch.testing.assert_close(out.float(), out2.float(), **TOL[dtype])


def test_decode_attention_replays_from_a_captured_graph(dev):
    """The decode step (single-launch prefix + suffix, merge) recorded into a graph: every replay, with eager
    work and synchronisation between replays, must reproduce the eager result for the inputs then in place."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(23)
    s = torch.randint(1, 120, (48,), generator=g).tolist()
    case = synth.make_decode_case("graph", 23, torch.float16, 1, 48, 900, s, 8, 128, 1 << 14)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    tables = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                        case.pool_lists(case.suffix_lists), dev, num_heads=8, head_dim=128)
    q_static = case.q.to(dev)
    out_static = torch.empty_like(q_static)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream: workspace and lazy state exist before recording
        kernels.decode_attention(q_static, kc, vc, tables, out=out_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        kernels.decode_attention(q_static, kc, vc, tables, out=out_static)
    gq = torch.Generator(device=dev).manual_seed(5)
    for rep in range(4):
        q_new = torch.randn(q_static.shape, generator=gq, device=dev, dtype=torch.float16)
        eager = kernels.decode_attention(q_new, kc, vc, tables)  # eager work between the replays
        torch.cuda.synchronize()
        q_static.copy_(q_new)
        out_static.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager), f"replay {rep} differs from the eager result"
    ref = ref_decode_attention(q_static.cpu(), case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(out_static.cpu().float(), ref.float(), **TOL[torch.float16])


@pytest.mark.parametrize("sizes", [[100], [128], [129], [200, 40], [257], [300, 70, 3]])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_large_groups_take_wider_query_tiles(dev, sizes, dtype):
    """Groups of more than 64 requests share each prefix tile among 128 or 256 queries (one read of the prefix
    per group instead of one per 64 requests); mixed with smaller groups, partial last tiles, both element types."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(31 + sum(sizes))
    B = sum(sizes)
    lens = torch.randint(0, 40, (B,), generator=g).tolist()
    case = synth.make_decode_case("wide", 31, dtype, len(sizes), B, 333, lens, 3, 128, 1 << 14, group_sizes=sizes)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    tables = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                        case.pool_lists(case.suffix_lists), dev, num_heads=3, head_dim=128)
    out = kernels.decode_attention(case.q.to(dev), kc, vc, tables).cpu()
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(out.float(), ref.float(), **TOL[dtype])
    # the same batch without the balanced plan: prefix kernel on its own launch
    plain = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                       case.pool_lists(case.suffix_lists), dev, num_heads=3, head_dim=128, balanced=False)
    out2 = kernels.decode_attention(case.q.to(dev), kc, vc, plain).cpu()
    torch.testing.assert_close(out2.float(), ref.float(), **TOL[dtype])


@pytest.mark.parametrize("groups,B,P", [(1, 48, 600), (2, 20, 300), (0, 37, 0)])
def test_library_plans_for_callers_without_a_plan(dev, groups, B, P):
    """No plan from the caller and the chunk size left to the library (0): the library builds the balanced plan on
    the device inside the call (workspace from the same query) -- one large group (single-launch path), small
    groups (prefix kernel + balanced suffix) and a ragged batch without any prefix."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(41 + B)
    n = max(1, groups) * B
    lens = torch.randint(0, 300, (n,), generator=g).tolist()
    case = synth.make_decode_case("noplan", 41, torch.float16, max(1, groups), B, P if groups else 0, lens, 5, 128, 1 << 15)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    tables = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                        case.pool_lists(case.suffix_lists), dev, num_heads=5, head_dim=128, balanced=False)
    assert tables.plan is None
    tables.chunk_tokens = 0
    out = kernels.decode_attention(case.q.to(dev), kc, vc, tables).cpu()
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(out.float(), ref.float(), **TOL[torch.float16])


def test_captured_decode_step_replays_while_contexts_grow(dev):
    """One decode step recorded once, replayed over six iterations in which every request gains a token: the slot
    tables are patched and the suffix plan rebuilt in place (on the device) between replays (fixed pointers, counts and workspace
    layout), and each replay must equal the eager result on tables built from scratch for that iteration."""
    from parrotserve_amd import kernels, synth, table_cache

    g = torch.Generator().manual_seed(29)
    B, H, D, P = 40, 8, 128, 700
    lens = torch.randint(1, 100, (B,), generator=g).tolist()
    case = synth.make_decode_case("grow", 29, torch.float16, 1, B, P, lens, H, D, 1 << 14)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    prefix = case.pool_lists(case.prefix_lists)
    suffix = [list(l) for l in case.pool_lists(case.suffix_lists)]
    used = set(case.used_slots.tolist())
    spare = [s for s in range(case.pool_slots) if s not in used][: 6 * B]
    tables = kernels.DecodeTables.build(prefix, case.group_req_cu, suffix, dev, num_heads=H, head_dim=D)
    table_cache._widen(tables, max(lens) + 8, dev)          # room for the tokens to come
    lanes = tables.plan.num_lanes                           # the recorded launch is shaped for this many pieces
    q_static = case.q.to(dev)
    out_static = torch.empty_like(q_static)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        kernels.decode_attention(q_static, kc, vc, tables, out=out_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        kernels.decode_attention(q_static, kc, vc, tables, out=out_static)
    plan_ptrs = (tables.plan.items, tables.plan.num_items, tables.plan.lane_rec, tables.plan.num_lanes)
    gq = torch.Generator(device=dev).manual_seed(6)
    for it in range(6):
        new = spare[it * B:(it + 1) * B]
        new_dev = torch.tensor(new, dtype=torch.int32, device=dev)
        kc[new_dev.long()] = torch.randn((B, H, D), generator=gq, device=dev, dtype=torch.float16)
        vc[new_dev.long()] = torch.randn((B, H, D), generator=gq, device=dev, dtype=torch.float16)
        for b in range(B):
            suffix[b].append(new[b])
        kernels.suffix_tables_append(tables.suffix_slots, tables.suffix_lens, None, new_dev)
        tables.max_suffix_len += 1
        tables.plan_on_device(lanes, dev)
        assert (tables.plan.items, tables.plan.num_items, tables.plan.lane_rec, tables.plan.num_lanes) == plan_ptrs
        q_new = torch.randn(q_static.shape, generator=gq, device=dev, dtype=torch.float16)
        fresh = kernels.DecodeTables.build(prefix, case.group_req_cu, suffix, dev, num_heads=H, head_dim=D)
        eager = kernels.decode_attention(q_new, kc, vc, fresh)
        torch.cuda.synchronize()
        q_static.copy_(q_new)
        out_static.zero_()
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(out_static.float(), eager.float(), **TOL[torch.float16])
        assert torch.equal(out_static, eager), f"iteration {it}: the replay differs from the eager result"
    full = [prefix[0] + l for l in suffix]
    ref = ref_decode_attention(q_static.cpu(), kc.cpu(), vc.cpu(), [torch.tensor(l) for l in full])
    torch.testing.assert_close(out_static.cpu().float(), ref.float(), **TOL[torch.float16])


def test_captured_library_planned_step_replays_while_contexts_grow(dev):
    """A caller without a plan of its own: the library builds the suffix plan inside the call, so the plan launch
    and its length bound are part of what a graph records.  Captured with max_suffix_len = the table's width (the
    largest length a replay will see), the replays follow the growing lists; each equals the eager result on
    tables built from scratch."""
    from parrotserve_amd import kernels, synth, table_cache

    g = torch.Generator().manual_seed(30)
    B, H, D, P = 48, 8, 128, 600
    lens = torch.randint(1, 80, (B,), generator=g).tolist()
    case = synth.make_decode_case("growlib", 30, torch.float16, 1, B, P, lens, H, D, 1 << 14)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    prefix = case.pool_lists(case.prefix_lists)
    suffix = [list(l) for l in case.pool_lists(case.suffix_lists)]
    used = set(case.used_slots.tolist())
    spare = [s for s in range(case.pool_slots) if s not in used][: 5 * B]
    tables = kernels.DecodeTables.build(prefix, case.group_req_cu, suffix, dev, num_heads=H, head_dim=D,
                                        balanced=False)
    assert tables.plan is None
    tables.chunk_tokens = 0                                  # leave the decomposition to the library: it plans
    table_cache._widen(tables, max(lens) + 8, dev)
    tables.max_suffix_len = tables.suffix_table_stride       # what the captured call records as its bound
    q_static = case.q.to(dev)
    out_static = torch.empty_like(q_static)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        kernels.decode_attention(q_static, kc, vc, tables, out=out_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        kernels.decode_attention(q_static, kc, vc, tables, out=out_static)
    gq = torch.Generator(device=dev).manual_seed(7)
    for it in range(5):
        new = spare[it * B:(it + 1) * B]
        new_dev = torch.tensor(new, dtype=torch.int32, device=dev)
        kc[new_dev.long()] = torch.randn((B, H, D), generator=gq, device=dev, dtype=torch.float16)
        vc[new_dev.long()] = torch.randn((B, H, D), generator=gq, device=dev, dtype=torch.float16)
        for b in range(B):
            suffix[b].append(new[b])
        kernels.suffix_tables_append(tables.suffix_slots, tables.suffix_lens, None, new_dev)
        q_new = torch.randn(q_static.shape, generator=gq, device=dev, dtype=torch.float16)
        fresh = kernels.DecodeTables.build(prefix, case.group_req_cu, suffix, dev, num_heads=H, head_dim=D)
        eager = kernels.decode_attention(q_new, kc, vc, fresh)
        torch.cuda.synchronize()
        q_static.copy_(q_new)
        out_static.zero_()
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(out_static.float(), eager.float(), **TOL[torch.float16])
    full = [prefix[0] + l for l in suffix]
    ref = ref_decode_attention(q_static.cpu(), kc.cpu(), vc.cpu(), [torch.tensor(l) for l in full])
    torch.testing.assert_close(out_static.cpu().float(), ref.float(), **TOL[torch.float16])


def test_inconsistent_table_extents(dev):
    """A padded table that does not hold max_suffix_len entries in its last row is refused; a ragged table whose
    last list runs past the table's end is read up to the end by the kernel that writes the parts and by the one
    that merges them alike (the result is that of the truncated list)."""
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(33)
    B, H, D, W = 5, 4, 128, 40
    k = torch.randn(B * W, H, D, generator=g).half()
    v = torch.randn(B * W, H, D, generator=g).half()
    q = torch.randn(B, H, D, generator=g).half()
    rows = torch.randperm(B * W, generator=g).to(torch.int32)
    lens = torch.tensor([W, 7, W, 20, W], dtype=torch.int32)
    padded = kernels.DecodeTables(num_reqs=B, suffix_slots=rows[: B * W - 9].to(dev), suffix_table_stride=W,
                                  suffix_lens=lens.to(dev), max_suffix_len=W, chunk_tokens=16)
    padded.suffix_slots_count = lambda: B * W - 9  # the true extent: the last row is nine entries short
    with pytest.raises(ValueError):
        kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), padded)
    # ragged: lists back to back, the last one claims W tokens but only W - 9 lie inside the table
    offs = torch.tensor([0, W, W + 7, 2 * W + 7, 2 * W + 27], dtype=torch.int64)
    total = int(offs[-1]) + W - 9
    ragged = kernels.DecodeTables(num_reqs=B, suffix_slots=rows[:total].to(dev), suffix_offsets=offs.to(dev),
                                  suffix_lens=lens.to(dev), max_suffix_len=W, chunk_tokens=16)
    out = kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), ragged)
    true_lens = [W, 7, W, 20, W - 9]
    ref = ref_decode_attention(q, k, v, [rows[int(offs[b]): int(offs[b]) + true_lens[b]].long() for b in range(B)])
    torch.testing.assert_close(out.cpu().float(), ref.float(), **TOL[torch.float16])


@pytest.mark.parametrize("seed", range(12))
def test_randomized_grouped_decode_shapes(dev, seed):
    """Seeded random batches: 1-3 prefix groups of 1-140 requests, prefixes of 1-1500 tokens (not multiples of
    any tile size), suffixes of 0-90 tokens, odd head counts, a few ungrouped requests, both element types."""
    _random_grouped_case(dev, seed, 128)


@pytest.mark.parametrize("seed", range(12))
def test_randomized_grouped_decode_shapes_head_size_64(dev, seed):
    """The same batches with 64-wide heads: even head counts run the prefix phase on head pairs through the
    128-wide matrix-core kernel (twice the rows, so groups of up to 140 requests cover every tile size and more
    than one tile), odd head counts take the per-request kernel."""
    _random_grouped_case(dev, seed, 64)


def _random_grouped_case(dev, seed, D):
    from parrotserve_amd import kernels

    g = torch.Generator().manual_seed(1000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    dtype = torch.float16 if seed % 2 == 0 else torch.bfloat16
    H = ri(1, 9)
    n_groups = ri(1, 3)
    sizes = [ri(1, 140) if i == 0 else ri(1, 50) for i in range(n_groups)]
    plens = [ri(1, 1500) for _ in range(n_groups)]
    loners = ri(0, 3)
    B = sum(sizes) + loners
    n_rows = sum(plens) + 90 * B + 8
    q = torch.randn(B, H, D, generator=g).to(dtype)
    k = torch.randn(n_rows, H, D, generator=g).to(dtype)
    v = torch.randn(n_rows, H, D, generator=g).to(dtype)
    perm = torch.randperm(n_rows, generator=g)
    pre, pos = [], 0
    for n in plens:
        pre.append(perm[pos:pos + n])
        pos += n
    gcu = [0]
    for n in sizes:
        gcu.append(gcu[-1] + n)
    suf, full = [], []
    for b in range(B):
        grp = next((i for i in range(n_groups) if gcu[i] <= b < gcu[i + 1]), None)
        n = ri(0, 90) if grp is not None else ri(1, 90)
        suf.append(perm[pos:pos + n])
        pos += n
        full.append(torch.cat([pre[grp] if grp is not None else perm[:0], suf[-1]]))
    ref = ref_decode_attention(q, k, v, full)
    tables = kernels.DecodeTables.build([p.tolist() for p in pre], gcu, [s.tolist() for s in suf], dev, num_heads=H,
                                        head_dim=D)
    out = kernels.decode_attention(q.to(dev), k.to(dev), v.to(dev), tables).cpu()
    torch.testing.assert_close(out.float(), ref.float(), **TOL[dtype])
