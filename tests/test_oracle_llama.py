"""Pins oracle/ref_llama.py (the flat-sequence LLaMA forward used to check the engine loop end to end)."""
import torch
import torch.nn.functional as F

from oracle.ref_llama import ref_llama_hidden


def _weights(seed, V=97, N=256, Fdim=384, layers=2):
    g = torch.Generator().manual_seed(seed)
    w = {"embed": torch.randn(V, N, generator=g), "norm": 1 + 0.1 * torch.randn(N, generator=g)}
    for i in range(layers):
        w[f"l{i}.ln1"] = 1 + 0.1 * torch.randn(N, generator=g)
        w[f"l{i}.ln2"] = 1 + 0.1 * torch.randn(N, generator=g)
        w[f"l{i}.qkv"] = 0.08 * torch.randn(3 * N, N, generator=g)
        w[f"l{i}.o"] = 0.08 * torch.randn(N, N, generator=g)
        w[f"l{i}.gate"] = 0.08 * torch.randn(Fdim, N, generator=g)
        w[f"l{i}.up"] = 0.08 * torch.randn(Fdim, N, generator=g)
        w[f"l{i}.down"] = 0.08 * torch.randn(N, Fdim, generator=g)
    return w


def _independent_forward(w, ids, H, eps, theta):
    """The same model written with torch's own building blocks and the Hugging Face rotate_half form of RoPE."""
    x = w["embed"][torch.tensor(ids)]
    T, N = x.shape
    D = N // H
    inv = 1.0 / (theta ** (torch.arange(0, D, 2).float() / D))
    ang = torch.outer(torch.arange(T).float(), inv)
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1)[:, None], torch.cat([ang.sin(), ang.sin()], -1)[:, None]

    def rot(t):
        t = t.view(T, H, D)
        half = torch.cat([-t[..., D // 2:], t[..., : D // 2]], -1)
        return t * cos + half * sin

    layers = sum(1 for k in w if k.endswith(".qkv"))
    for i in range(layers):
        h = F.rms_norm(x, (N,), w[f"l{i}.ln1"], eps)
        q, k, v = (h @ w[f"l{i}.qkv"].t()).chunk(3, -1)
        q, k, v = rot(q).transpose(0, 1), rot(k).transpose(0, 1), v.view(T, H, D).transpose(0, 1)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(0, 1).reshape(T, N)
        x = x + a @ w[f"l{i}.o"].t()
        h = F.rms_norm(x, (N,), w[f"l{i}.ln2"], eps)
        x = x + (F.silu(h @ w[f"l{i}.gate"].t()) * (h @ w[f"l{i}.up"].t())) @ w[f"l{i}.down"].t()
    return F.rms_norm(x, (N,), w["norm"], eps)


def test_matches_torch_building_blocks():
    w = _weights(0)
    ids = torch.randint(0, 97, (37,), generator=torch.Generator().manual_seed(1)).tolist()
    got = ref_llama_hidden(w, ids, num_heads=2, eps=1e-6)
    ref = _independent_forward(w, ids, 2, 1e-6, 10000.0)
    torch.testing.assert_close(got, ref, atol=2e-4, rtol=1e-4)


def test_prefix_property_and_token_sensitivity():
    """Causality of the composition: rows of a prefix do not change when tokens are appended; the row of a
    changed token and the rows after it do."""
    w = _weights(3)
    ids = torch.randint(0, 97, (20,), generator=torch.Generator().manual_seed(4)).tolist()
    full = ref_llama_hidden(w, ids, 2, 1e-6)
    part = ref_llama_hidden(w, ids[:11], 2, 1e-6)
    torch.testing.assert_close(full[:11], part, atol=1e-5, rtol=1e-5)
    ids2 = list(ids)
    ids2[11] = (ids2[11] + 1) % 97
    other = ref_llama_hidden(w, ids2, 2, 1e-6)
    torch.testing.assert_close(other[:11], full[:11], atol=1e-5, rtol=1e-5)
    assert (other[11:] - full[11:]).abs().max() > 1e-2
