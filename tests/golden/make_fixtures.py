"""Writes the golden fixtures of tests/golden/: small seeded inputs and the outputs the CPU oracle
(oracle/ref_ops.py) gives for them, as .npz files of plain arrays (16-bit floats stored as their bit patterns).

Nothing of the reference is imported or run: the reference holds no stored vectors for this path, and its own
checks are kernel-vs-formula in the same file, so the fixtures freeze THIS build's oracle (itself pinned by the
closed forms and library routines of tests/test_oracle_*.py).  They guard against drift of the oracle and give
the GPU tests inputs and answers that do not depend on it at run time.

    python tests/golden/make_fixtures.py        # rewrites the files next to this script
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import ref_sampler  # noqa: E402
from oracle.ref_ops import (ref_add_rms_norm, ref_cos_sin_cache, ref_decode_attention, ref_kv_append,  # noqa: E402
                            ref_move_tokens, ref_prefill_with_parent, ref_rms_norm, ref_rope_neox, ref_silu_mul)


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy() if t.dtype in (torch.float16, torch.bfloat16) else t.numpy()


def decode_fixture(dtype, name):
    g = torch.Generator().manual_seed(101)
    H, D, B, P, slots = 2, 128, 5, 45, 112
    perm = torch.randperm(slots, generator=g)
    kc = torch.randn(slots, H, D, generator=g).to(dtype)
    vc = torch.randn(slots, H, D, generator=g).to(dtype)
    q = torch.randn(B, H, D, generator=g).to(dtype)
    prefix = perm[:P]
    lens = [7, 0, 33, 1, 18]
    suffix, p = [], P
    for n in lens:
        suffix.append(perm[p:p + n])
        p += n
    full = [torch.cat([prefix, s]) for s in suffix]
    out = ref_decode_attention(q, kc, vc, full)
    width = max(lens)
    table = np.zeros((B, width), np.int32)
    for i, s in enumerate(suffix):
        table[i, : len(s)] = s.numpy()
    np.savez(os.path.join(HERE, name), q=bits(q), k_cache=bits(kc), v_cache=bits(vc), prefix_slots=prefix.numpy().astype(np.int32),
             suffix_table=table, suffix_lens=np.asarray(lens, np.int32), out=bits(out))


def prefill_fixture():
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(102)
    H, D, slots = 2, 128, 272
    q_lens, parent = [37, 70, 1], 50
    perm = torch.randperm(slots, generator=g)
    kc = torch.randn(slots, H, D, generator=g).to(dtype)
    vc = torch.randn(slots, H, D, generator=g).to(dtype)
    T = sum(q_lens)
    q = torch.randn(T, H, D, generator=g).to(dtype)
    ctx, p = [], 0
    for n in q_lens:
        ctx.append(perm[p:p + parent + n])
        p += parent + n
    out = ref_prefill_with_parent(q, kc, vc, q_lens, ctx)
    np.savez(os.path.join(HERE, "prefill_bf16.npz"), q=bits(q), k_cache=bits(kc), v_cache=bits(vc),
             q_lens=np.asarray(q_lens, np.int32), ctx_slots=torch.cat(ctx).numpy().astype(np.int32),
             kv_lens=np.asarray([parent + n for n in q_lens], np.int32), out=bits(out))


def elementwise_fixture():
    g = torch.Generator().manual_seed(103)
    dt = torch.float16
    # token move + append (bit-exact ops)
    src = torch.randn(40, 2, 64, generator=g).to(dt)
    dst0 = torch.randn(64, 2, 64, generator=g).to(dt)
    sidx = torch.randperm(40, generator=g)[:17]
    didx = torch.randperm(64, generator=g)[:17]
    moved = dst0.clone()
    ref_move_tokens(src, moved, sidx, didx)
    k = torch.randn(9, 2, 64, generator=g).to(dt)
    v = torch.randn(9, 2, 64, generator=g).to(dt)
    kc, vc = dst0.clone(), dst0.flip(0).clone()
    sm = torch.randperm(64, generator=g)[:9]
    kc_out, vc_out = kc.clone(), vc.clone()
    ref_kv_append(k, v, kc_out, vc_out, sm)
    # rope (element-type arithmetic, bit-exact) and norms / activation (tolerance)
    T, H, D = 11, 3, 128
    pos = torch.randint(0, 90, (T,), generator=g)
    cache = ref_cos_sin_cache(90, D, 10000.0, dt)
    rq = torch.randn(T, H * D, generator=g).to(dt)
    rk = torch.randn(T, H * D, generator=g).to(dt)
    oq, ok = ref_rope_neox(pos, rq, rk, cache, D, elem_rounding=True)
    x = (torch.randn(6, 1024, generator=g) * 2).to(dt)
    r = (torch.randn(6, 1024, generator=g) * 2).to(dt)
    w = (torch.rand(1024, generator=g) + 0.5).to(dt)
    y_first = ref_rms_norm(x, w, 1e-6, round_before_weight=True)
    y_once = ref_rms_norm(x, w, 1e-6, round_before_weight=False)
    y_add, h_add = ref_add_rms_norm(x, r, w, 1e-6, round_before_weight=True)
    act = ref_silu_mul(x, r)
    np.savez(os.path.join(HERE, "elementwise_fp16.npz"), move_src=bits(src), move_dst=bits(dst0), move_sidx=sidx.numpy(),
             move_didx=didx.numpy(), move_out=bits(moved), app_k=bits(k), app_v=bits(v), app_kc=bits(kc), app_vc=bits(vc),
             app_slots=sm.numpy(), app_kc_out=bits(kc_out), app_vc_out=bits(vc_out), rope_pos=pos.numpy(),
             rope_cache=bits(cache), rope_q=bits(rq), rope_k=bits(rk), rope_q_out=bits(oq), rope_k_out=bits(ok),
             norm_x=bits(x), norm_r=bits(r), norm_w=bits(w), norm_round_first=bits(y_first), norm_round_once=bits(y_once),
             addnorm_y=bits(y_add), addnorm_h=bits(h_add), silu_mul=bits(act))


def sampler_fixture():
    """48 rows of 2000 fp16 logits with mixed temperatures and top-p values; only rows whose decisions are clear of
    every rounding boundary (relative margin >= 1e-4) are kept, so any correct fp32 implementation draws these ids."""
    g = torch.Generator().manual_seed(21)
    B, V = 48, 2000
    x = (torch.randn(B, V, generator=g) * 3).half()
    temps = torch.tensor([1.0, 0.7, 1.5])[torch.randint(0, 3, (B,), generator=g)]
    tops = torch.tensor([1.0, 0.9, 0.5, 1e-6])[torch.randint(0, 4, (B,), generator=g)]
    u = torch.rand(B, generator=g)
    ids, margins = ref_sampler.ref_sample(x.double().numpy(), temps.numpy(), tops.numpy(), u.numpy(), "f16")
    keep = margins >= 1e-4
    assert keep.sum() >= 40
    np.savez(os.path.join(HERE, "sampler_fp16.npz"), logits=bits(x[keep]), temperature=temps.numpy()[keep],
             top_p=tops.numpy()[keep], uniform=u.numpy()[keep], ids=ids[keep])


if __name__ == "__main__":
    sampler_fixture()
    decode_fixture(torch.float16, "decode_fp16.npz")
    decode_fixture(torch.bfloat16, "decode_bf16.npz")
    prefill_fixture()
    elementwise_fixture()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
