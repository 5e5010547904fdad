"""Pins for the attention part of the CPU oracle: brute force, library routine
(SDPA), and the defining invariants of the partial/merge decomposition."""
import math

import pytest
import torch

from oracle.ref_ops import (ref_decode_attention, ref_lse_merge, ref_partial, ref_prefill_with_parent,
                            ref_shared_prefix_decode)


def brute_force_decode(q, kc, vc, slot_lists, scale):
    """Pure python loops, no tensor ops on more than scalars."""
    B, H, D = q.shape
    out = torch.zeros(B, H, D, dtype=torch.float64)
    for b in range(B):
        slots = [int(s) for s in slot_lists[b]]
        for h in range(H):
            logits = []
            for s in slots:
                acc = 0.0
                for d in range(D):
                    acc += float(q[b, h, d]) * float(kc[s, h, d])
                logits.append(acc * scale)
            mx = max(logits)
            ws = [math.exp(x - mx) for x in logits]
            tot = sum(ws)
            for d in range(D):
                out[b, h, d] = sum(w * float(vc[s, h, d]) for w, s in zip(ws, slots)) / tot
    return out


def _pool(seed, slots=40, H=2, D=8, B=3):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, D, generator=g)
    kc = torch.randn(slots, H, D, generator=g)
    vc = torch.randn(slots, H, D, generator=g)
    return q, kc, vc, g


def test_decode_matches_brute_force():
    q, kc, vc, g = _pool(0)
    lists = [torch.randperm(40, generator=g)[:n] for n in (5, 1, 17)]
    ref = ref_decode_attention(q, kc, vc, lists)
    bf = brute_force_decode(q, kc, vc, lists, 8 ** -0.5)
    torch.testing.assert_close(ref.double(), bf, atol=1e-5, rtol=1e-5)


def test_decode_matches_sdpa_library():
    q, kc, vc, g = _pool(1, slots=64, H=4, D=16, B=2)
    lists = [torch.randperm(64, generator=g)[:n] for n in (33, 64)]
    ref = ref_decode_attention(q, kc, vc, lists)
    for b, l in enumerate(lists):
        k = kc[l].permute(1, 0, 2)  # [H, n, D]
        v = vc[l].permute(1, 0, 2)
        o = torch.nn.functional.scaled_dot_product_attention(q[b][:, None, :], k, v)  # default scale D^-0.5
        torch.testing.assert_close(ref[b], o[:, 0, :], atol=1e-5, rtol=1e-5)


def test_explicit_scale_is_used():
    q, kc, vc, g = _pool(2)
    lists = [torch.arange(10)] * 3
    a = ref_decode_attention(q, kc, vc, lists, scale=0.0)  # uniform weights
    torch.testing.assert_close(a[0], vc[:10].mean(0), atol=1e-6, rtol=1e-6)


def test_slot_permutation_invariance_and_order_independence():
    q, kc, vc, g = _pool(3)
    l = torch.randperm(40, generator=g)[:12]
    a = ref_decode_attention(q, kc, vc, [l] * 3)
    b = ref_decode_attention(q, kc, vc, [l.flip(0)] * 3)
    torch.testing.assert_close(a, b, atol=1e-6, rtol=1e-6)
    perm = torch.randperm(40, generator=g)
    kc2, vc2 = torch.empty_like(kc), torch.empty_like(vc)
    kc2[perm] = kc
    vc2[perm] = vc
    c = ref_decode_attention(q, kc2, vc2, [perm[l]] * 3)
    torch.testing.assert_close(a, c, atol=1e-6, rtol=1e-6)


def test_partial_closed_form_single_key():
    # one key: m = q.k*scale*log2e, l = 1, O = v
    q, kc, vc, g = _pool(4)
    O, m, l = ref_partial(q, kc, vc, [torch.tensor([7])] * 3)
    torch.testing.assert_close(O, vc[7].expand(3, -1, -1))
    torch.testing.assert_close(l, torch.ones(3, 2))
    want = (q * kc[7]).sum(-1) * (8 ** -0.5) * math.log2(math.e)
    torch.testing.assert_close(m, want, atol=1e-6, rtol=1e-6)


def test_merge_equals_one_shot():
    q, kc, vc, g = _pool(5, slots=100, H=3, D=16, B=4)
    pre = torch.randperm(100, generator=g)[:37]
    rest = [x for x in range(100) if x not in set(pre.tolist())]
    sufs = [torch.tensor(rest[:n]) for n in (1, 9, 0, 40)]
    merged = ref_shared_prefix_decode(q, kc, vc, pre, sufs)
    oneshot = ref_decode_attention(q, kc, vc, [torch.cat([pre, s]) for s in sufs])
    torch.testing.assert_close(merged, oneshot, atol=1e-5, rtol=1e-5)


def test_split_invariance_nway():
    q, kc, vc, g = _pool(6, slots=90, H=2, D=8, B=2)
    l = torch.randperm(90, generator=g)[:61]
    whole = ref_partial(q, kc, vc, [l] * 2)
    for cuts in ([10, 30], [1, 2, 3, 60], [31]):
        bounds = [0] + cuts + [61]
        acc = None
        for a, b in zip(bounds[:-1], bounds[1:]):
            part = ref_partial(q, kc, vc, [l[a:b]] * 2)
            acc = part if acc is None else ref_lse_merge(acc, part)
        torch.testing.assert_close(acc[0], whole[0], atol=1e-5, rtol=1e-5)
        # log2-sum-exp is the split-invariant quantity
        torch.testing.assert_close(acc[1] + torch.log2(acc[2]), whole[1] + torch.log2(whole[2]), atol=1e-5, rtol=1e-5)


def test_merge_edge_cases_empty_sides():
    q, kc, vc, g = _pool(7)
    l = torch.arange(6)
    full = ref_partial(q, kc, vc, [l] * 3)
    empty = ref_partial(q, kc, vc, [torch.tensor([], dtype=torch.long)] * 3)
    assert torch.isinf(empty[1]).all() and (empty[2] == 0).all() and (empty[0] == 0).all()
    for a, b in ((full, empty), (empty, full)):
        O, m, ll = ref_lse_merge(a, b)
        torch.testing.assert_close(O, full[0])
        torch.testing.assert_close(m, full[1])
        torch.testing.assert_close(ll, full[2])
    O, m, ll = ref_lse_merge(empty, empty)
    assert (O == 0).all() and (ll == 0).all() and not torch.isnan(O).any()


def test_merge_is_commutative_and_handles_large_gap():
    O1 = torch.ones(1, 1, 4)
    O2 = 3 * torch.ones(1, 1, 4)
    a = (O1, torch.tensor([[100.0]]), torch.tensor([[2.0]]))
    b = (O2, torch.tensor([[-100.0]]), torch.tensor([[5.0]]))
    x = ref_lse_merge(a, b)
    y = ref_lse_merge(b, a)
    torch.testing.assert_close(x[0], y[0])
    torch.testing.assert_close(x[0], O1)  # b is 2^-200 of a
    # equal maxima: weights are l
    c = (O2, torch.tensor([[100.0]]), torch.tensor([[6.0]]))
    z = ref_lse_merge(a, c)
    torch.testing.assert_close(z[0], (2 * O1 + 6 * O2) / 8)
    torch.testing.assert_close(z[2], torch.tensor([[8.0]]))


def brute_force_prefill(q, kc, vc, q_lens, ctx_lists, scale):
    T, H, D = q.shape
    out = torch.zeros(T, H, D, dtype=torch.float64)
    start = 0
    for n, slots in zip(q_lens, ctx_lists):
        slots = [int(s) for s in slots]
        kv = len(slots)
        for r in range(n):
            visible = slots[: kv - n + r + 1]  # bottom-right aligned causal
            for h in range(H):
                logits = [sum(float(q[start + r, h, d]) * float(kc[s, h, d]) for d in range(D)) * scale for s in visible]
                mx = max(logits)
                ws = [math.exp(x - mx) for x in logits]
                tot = sum(ws)
                for d in range(D):
                    out[start + r, h, d] = sum(w * float(vc[s, h, d]) for w, s in zip(ws, visible)) / tot
        start += n
    return out


def test_prefill_matches_brute_force():
    g = torch.Generator().manual_seed(8)
    H, D = 2, 4
    kc = torch.randn(50, H, D, generator=g)
    vc = torch.randn(50, H, D, generator=g)
    q_lens = [3, 1, 5]
    ctx = [torch.randperm(50, generator=g)[:n] for n in (7, 4, 5)]  # parents 4, 3, 0
    q = torch.randn(sum(q_lens), H, D, generator=g)
    ref = ref_prefill_with_parent(q, kc, vc, q_lens, ctx)
    bf = brute_force_prefill(q, kc, vc, q_lens, ctx, D ** -0.5)
    torch.testing.assert_close(ref.double(), bf, atol=1e-5, rtol=1e-5)


def test_prefill_matches_sdpa_with_explicit_mask():
    # the mask written out in 3rdparty/vllm/tests/kernels/test_attention.py:127-130
    g = torch.Generator().manual_seed(9)
    H, D = 3, 8
    kc = torch.randn(80, H, D, generator=g)
    vc = torch.randn(80, H, D, generator=g)
    q_len, ctx_len = 6, 21
    ctx = torch.randperm(80, generator=g)[:ctx_len]
    q = torch.randn(q_len, H, D, generator=g)
    ref = ref_prefill_with_parent(q, kc, vc, [q_len], [ctx])
    blocked = torch.triu(torch.ones(q_len, ctx_len), diagonal=ctx_len - q_len + 1).bool()
    o = torch.nn.functional.scaled_dot_product_attention(
        q.permute(1, 0, 2), kc[ctx].permute(1, 0, 2), vc[ctx].permute(1, 0, 2), attn_mask=~blocked)
    torch.testing.assert_close(ref, o.permute(1, 0, 2), atol=1e-5, rtol=1e-5)


def test_prefill_reductions():
    g = torch.Generator().manual_seed(10)
    H, D = 2, 8
    kc = torch.randn(60, H, D, generator=g)
    vc = torch.randn(60, H, D, generator=g)
    # q_len == 1 is decode over the whole context
    ctx = [torch.randperm(60, generator=g)[:n] for n in (9, 30)]
    q = torch.randn(2, H, D, generator=g)
    a = ref_prefill_with_parent(q, kc, vc, [1, 1], ctx)
    b = ref_decode_attention(q, kc, vc, ctx)
    torch.testing.assert_close(a, b, atol=1e-6, rtol=1e-6)
    # parent == 0 is ordinary causal attention (library routine)
    n = 7
    c = torch.randperm(60, generator=g)[:n]
    q = torch.randn(n, H, D, generator=g)
    a = ref_prefill_with_parent(q, kc, vc, [n], [c])
    o = torch.nn.functional.scaled_dot_product_attention(
        q.permute(1, 0, 2), kc[c].permute(1, 0, 2), vc[c].permute(1, 0, 2), is_causal=True)
    torch.testing.assert_close(a, o.permute(1, 0, 2), atol=1e-5, rtol=1e-5)
    # the first query of a chunk with a parent sees exactly parent + 1 keys; chunks do not leak into each other
    two = ref_prefill_with_parent(torch.cat([q, q]), kc, vc, [n, n], [c, c.flip(0)])
    torch.testing.assert_close(two[:n], a, atol=1e-6, rtol=1e-6)


def test_config1_shared_prefix_plumbing():
    """BASELINE config 1 (fp32, B 8, P 512, S U[32,128], 32x128, seed 0): the
    prefix/suffix/merge decomposition equals one-shot attention."""
    from parrotserve_amd import synth

    case = synth.config1()
    assert case.q.shape == (8, 32, 128) and case.prefix_lists[0].numel() == 512
    assert all(32 <= s.numel() <= 128 for s in case.suffix_lists)
    split = ref_shared_prefix_decode(case.q, case.k_rows, case.v_rows, case.prefix_lists[0], case.suffix_lists)
    one = ref_decode_attention(case.q, case.k_rows, case.v_rows, case.full_lists())
    torch.testing.assert_close(split, one, atol=2e-5, rtol=1e-4)
