"""The decode entry point that allocates nothing (ph_decode_attention_static: partials in the library's own fixed
device array) against ph_decode_attention on a caller's workspace, both through the C ABI: two calls in a row, the
second on a smaller input, then a shape beyond the array."""
import ctypes

import pytest
import torch

from oracle.ref_ops import ref_decode_attention

pytestmark = pytest.mark.gpu

TOL = {torch.float16: dict(atol=2e-3, rtol=1e-2), torch.bfloat16: dict(atol=1e-2, rtol=2e-2)}


def _call_both(dev, dtype, seed, groups, per_group, P, H, D, smax):
    """One case through both entry points (raw ctypes); returns (static result, workspace result, oracle)."""
    from parrotserve_amd import _lib, kernels, synth

    lib = _lib.load()
    g = torch.Generator().manual_seed(seed)
    B = groups * per_group
    s = torch.randint(0, smax, (B,), generator=g).tolist()
    case = synth.make_decode_case("na", seed, dtype, groups, per_group, P, s, H, D, 1 << 14)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    t = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                   case.pool_lists(case.suffix_lists), dev, num_heads=H, head_dim=D)
    q = case.q.to(dev)
    code = 0 if dtype == torch.float16 else 1
    plan = None if t.plan is None else ctypes.byref(t.plan)
    n_items = 0 if t.plan is None else t.plan.num_items
    common = (B, H, D, code, q.stride(0), q.stride(0), kc.stride(0), float(D ** -0.5),
              t.num_groups, t.prefix_slots.data_ptr(), t.prefix_cu.data_ptr(), t.group_req_cu.data_ptr(),
              t.group_req_cu_host.data_ptr(), t.max_prefix_len,
              None if t.suffix_slots is None else t.suffix_slots.data_ptr(), None, t.suffix_table_stride,
              t.suffix_slots_count(), None if t.suffix_lens is None else t.suffix_lens.data_ptr(),
              t.max_suffix_len, t.chunk_tokens, plan)
    st = torch.cuda.current_stream().cuda_stream
    nbytes = lib.ph_decode_workspace_bytes(B, H, D, t.num_groups, t.max_prefix_len, t.max_suffix_len, t.chunk_tokens,
                                           n_items)
    assert 0 < nbytes <= lib.ph_decode_static_scratch_bytes()
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    want = torch.zeros_like(q)
    assert lib.ph_decode_attention(want.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), *common,
                                   ws.data_ptr(), nbytes, st) == 0
    got = torch.zeros_like(q)
    # first call on the device outside the measured region: it looks the array's address up (hipGetSymbolAddress,
    # which may load the code object)
    assert lib.ph_decode_attention_static(got.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), *common, st) == 0
    torch.cuda.synchronize()
    got.zero_()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]  # the driver's own count: sees allocations torch's allocator does not
    assert lib.ph_decode_attention_static(got.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), *common, st) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    ref = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    return got.cpu(), want.cpu(), ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_static_scratch_entry_point_matches_workspace_entry_point(dev, dtype):
    # first call: one group of 64 requests (prefix and suffix phases in one launch), 8 heads
    # second call, smaller: two groups of 12 requests, 4 heads, shorter prefix -- on the array the first call left
    for seed, groups, per_group, P, H, smax in ((41, 1, 64, 700, 8, 90), (42, 2, 12, 130, 4, 40)):
        got, want, ref = _call_both(dev, dtype, seed, groups, per_group, P, H, 128, smax)
        torch.testing.assert_close(got.float(), want.float(), **TOL[dtype])
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))  # same kernels, same order of sums
        torch.testing.assert_close(got.float(), ref.float(), **TOL[dtype])


def test_static_scratch_entry_point_under_graph_capture(dev):
    """The entry point recorded into a graph (after one eager call on the device, which resolves the array's
    address) and replayed three times with eager work between the replays: every replay equals the workspace form."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(43)
    B, H, D, P = 64, 8, 128, 500
    s = torch.randint(0, 70, (B,), generator=g).tolist()
    case = synth.make_decode_case("nag", 43, torch.float16, 1, B, P, s, H, D, 1 << 14)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    t = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                   case.pool_lists(case.suffix_lists), dev, num_heads=H, head_dim=D)
    q = case.q.to(dev)
    out = torch.empty_like(q)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        kernels.decode_attention_static(q, kc, vc, t, out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        kernels.decode_attention_static(q, kc, vc, t, out)
    gq = torch.Generator(device=dev).manual_seed(8)
    for _ in range(3):
        q.copy_(torch.randn(q.shape, generator=gq, device=dev, dtype=torch.float16))
        want = kernels.decode_attention(q, kc, vc, t)       # eager work between the replays, on its own workspace
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_static_scratch_entry_point_refuses_what_does_not_fit(dev):
    from parrotserve_amd import _lib

    lib = _lib.load()
    # 4096 requests x 32 heads with 8192-token suffixes in 32-token chunks: gigabytes of partials
    assert lib.ph_decode_workspace_bytes(4096, 32, 128, 0, 0, 8192, 32, 0) > lib.ph_decode_static_scratch_bytes()
    rc = lib.ph_decode_attention_static(1, 1, 1, 1, 4096, 32, 128, 0, 4096, 4096, 4096, 1.0, 0, None, None, None, None,
                                        0, 1, None, 8192, 4096 * 8192, 1, 8192, 32, None, None)
    assert rc == _lib.PH_ERR_SCRATCH
    assert "scratch" in _lib.status_string(rc)
