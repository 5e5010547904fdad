"""Token sampler kernel (ph_sample_top_p through kernels.sample_top_p) against the float64 oracle
(oracle/ref_sampler.py, after parrot/engine/builtin/models/sampler.py:19-66).

Token ids are integers, so the comparison is exact -- on every row whose decision is not within rounding noise of
a boundary: the oracle reports, per row, how close top_p came to the mass-before of a token at the cut and how
close the uniform number came to an edge of the drawn token's interval.  fp32 sums over a row carry a relative
error of a few 1e-7, so rows with a margin under MARGIN are not compared (and must stay a small minority)."""
import numpy as np
import pytest
import torch

from oracle import ref_sampler as rs
from parrotserve_amd import kernels

pytestmark = pytest.mark.gpu
MARGIN = 5e-6

DT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}


def _case(seed, B, V, dtype, std=4.0, quantum=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, V, generator=g) * std
    if quantum:
        x = torch.round(x / quantum) * quantum  # many equal values
    x = x.to(DT[dtype])
    temps = torch.tensor([1.0, 0.7, 1.3, 0.25])[torch.randint(0, 4, (B,), generator=g)]
    tops = torch.tensor([1.0, 0.95, 0.9, 0.5, 0.1, 1e-6])[torch.randint(0, 6, (B,), generator=g)]
    u = torch.rand(B, generator=g)
    return x, temps, tops, u


def _check(x, temps, tops, u, dtype, min_compared=0.9, stride_pad=0):
    B, V = x.shape
    dev = torch.device("cuda:0")
    if stride_pad:
        buf = torch.full((B, V + stride_pad), 100.0, dtype=x.dtype, device=dev)  # a read past the row would win
        buf[:, :V] = x.to(dev)
        xd = buf[:, :V]
    else:
        xd = x.to(dev)
    ids = kernels.sample_top_p(xd, None if temps is None else temps.to(dev), None if tops is None else tops.to(dev),
                               u.to(dev)).cpu().numpy()
    want, margins = rs.ref_sample(x.double().numpy(), None if temps is None else temps.numpy(),
                                  None if tops is None else tops.numpy(), u.numpy(), dtype)
    assert ids.dtype == np.int64 and ((ids >= 0) & (ids < V)).all()
    clear = margins >= MARGIN
    assert clear.mean() >= min_compared, f"only {clear.sum()} of {B} rows are clear of a boundary"
    bad = np.nonzero(clear & (ids != want))[0]
    assert bad.size == 0, f"rows {bad[:8].tolist()}: got {ids[bad[:8]].tolist()}, want {want[bad[:8]].tolist()}"
    return ids


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("B,V", [(64, 32000), (3, 1000), (1, 7), (3, 1003), (5, 36864), (4, 50257), (6, 50272),
                                 (3, 57344), (2, 70001)])
def test_matches_oracle(dtype, B, V):
    """Row lengths on every path of the library: rows that fit the register file and start on 16-byte boundaries
    (32000, 1000, 36864, 50272, 57344: the largest), rows that do not start on such boundaries (7, 1003: kept in
    LDS; 50257: re-read) and rows too long for the registers (70001)."""
    x, temps, tops, u = _case(B * 131 + V, B, V, dtype)
    _check(x, temps, tops, u, dtype, min_compared=0.6 if B < 8 else 0.9)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_rows_full_of_equal_values(dtype):
    """Logits on a coarse grid: the cut falls inside a group of equal values, which survive in id order."""
    x, temps, tops, u = _case(5, 48, 4000, dtype, std=2.0, quantum=0.5)
    temps = torch.ones_like(temps)  # a division would spread the grid
    _check(x, temps, tops, u, dtype)


def test_no_filter_no_temperature_and_strided_rows():
    x, _, _, u = _case(9, 32, 32000, "f16")
    a = _check(x, None, None, u, "f16")
    b = _check(x, None, None, u, "f16", stride_pad=24)
    c = _check(x, None, None, u, "f16", stride_pad=3)  # rows off the 16-byte grid: another kernel, same tokens
    assert (a == b).all()
    assert (a == c)[rs.ref_sample(x.double().numpy(), None, None, u.numpy())[1] >= MARGIN].all()


def test_limits_select_the_most_likely_token():
    x, _, _, u = _case(11, 16, 32000, "f16")
    dev = torch.device("cuda:0")
    want = rs.ref_sample(x.double().numpy(), None, np.full(16, 1e-6, dtype=np.float32), u.numpy())[0]
    assert (want == x.double().numpy().argmax(1)).all()
    for temps, tops in [(None, torch.full((16,), 1e-6)), (None, torch.zeros(16)), (torch.zeros(16), None),
                        (torch.full((16,), -1.0), torch.ones(16))]:
        ids = kernels.sample_top_p(x.to(dev), None if temps is None else temps.to(dev),
                                   None if tops is None else tops.to(dev), u.to(dev)).cpu().numpy()
        assert (ids == want).all()


def test_uniform_logits_draw_floor_u_times_v():
    V, B = 64, 512
    g = torch.Generator().manual_seed(3)
    u = torch.rand(B, generator=g)
    dev = torch.device("cuda:0")
    ids = kernels.sample_top_p(torch.zeros(B, V, dtype=torch.float16, device=dev), None, None, u.to(dev)).cpu()
    assert (ids == torch.floor(u * V).long()).all()


def test_masked_tokens_are_never_drawn_and_edges_of_the_range():
    V, B = 1000, 256
    g = torch.Generator().manual_seed(4)
    x = torch.randn(B, V, generator=g).half()
    x[:, ::2] = float("-inf")
    x[0, 1] = 5.0  # certainly inside the filter
    u = torch.rand(B, generator=g)
    u[0], u[1] = 0.0, float(np.nextafter(np.float32(1.0), np.float32(0.0)))
    ids = _check(x, None, torch.full((B,), 0.99), u, "f16")
    assert (ids % 2 == 1).all()
    assert ids[0] == 1  # the first token that can be drawn


def test_draw_frequencies_match_the_probabilities():
    V, B = 16, 65536
    g = torch.Generator().manual_seed(6)
    row = (torch.randn(V, generator=g) * 1.5).half()
    top_p = 0.8
    p, _ = rs.kept_probs(row.double().numpy(), 1.0, top_p, "f16")
    dev = torch.device("cuda:0")
    u = torch.rand(B, generator=torch.Generator(device=dev).manual_seed(1), device=dev)
    ids = kernels.sample_top_p(row.to(dev).expand(B, V).contiguous(), None, torch.full((B,), top_p, device=dev), u)
    counts = torch.bincount(ids.cpu(), minlength=V).numpy()
    assert (counts[p == 0] == 0).all()
    np.testing.assert_allclose(counts / B, p, atol=4 * np.sqrt(0.25 / B))


def test_same_inputs_same_tokens():
    x, temps, tops, u = _case(13, 64, 32000, "bf16")
    dev = torch.device("cuda:0")
    args = (x.to(dev), temps.to(dev), tops.to(dev), u.to(dev))
    a = kernels.sample_top_p(*args)
    b = kernels.sample_top_p(*args)
    assert torch.equal(a, b)


def test_sampler_module_uses_the_kernel():
    """runner.Sampler: top_p -> 0 gives the arg-max of hidden @ W.T; a plain draw stays inside the vocabulary and
    follows torch's generator (same seed, same tokens)."""
    from parrotserve_amd.runner import LlamaConfig, Sampler, SamplingConfig

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(2)
    W = (torch.randn(4096, 256, generator=g) * 0.05).half().to(dev)
    h = torch.randn(8, 256, generator=g).half().to(dev)
    cfg = LlamaConfig(vocab_size=4096, hidden_size=256)
    s = Sampler(cfg, W)
    ids = s(h, [SamplingConfig(top_p=1e-6)] * 8)
    logits = (h @ W.t()).double().cpu().numpy()
    want = rs.ref_sample(logits, None, np.full(8, 1e-6, dtype=np.float32), np.zeros(8, dtype=np.float32))[0]
    assert ids.cpu().tolist() == want.tolist()
    torch.manual_seed(5)
    a = s(h, [SamplingConfig(temperature=0.8, top_p=0.9)] * 8)
    torch.manual_seed(5)
    b = s(h, [SamplingConfig(temperature=0.8, top_p=0.9)] * 8)
    assert torch.equal(a, b) and int(a.min()) >= 0 and int(a.max()) < 4096
    assert s(h[:0], []).shape == (0,)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("B,V", [(16, 32000), (3, 1003), (2, 50257)])
def test_filtered_probabilities_match_oracle(dtype, B, V):
    """ph_top_p_probs: the tensor the reference hands to torch.multinomial (models/sampler.py:58-64) -- soft-max of
    the tokens the top-p filter keeps, zero elsewhere -- against the float64 oracle, on rows whose cut is clear of
    rounding noise: same support, probabilities to fp32 accuracy."""
    x, temps, tops, _ = _case(31 + V, B, V, dtype)
    dev = torch.device("cuda:0")
    probs = kernels.top_p_probs(x.to(dev), temps.to(dev), tops.to(dev)).cpu().double().numpy()
    assert probs.shape == (B, V)
    compared = 0
    for b in range(B):
        want, margin = rs.kept_probs(x[b].double().numpy(), float(temps[b]), float(tops[b]), dtype)
        np.testing.assert_allclose(probs[b].sum(), 1.0, rtol=1e-5)
        if margin < MARGIN:
            continue
        compared += 1
        assert ((probs[b] > 0) == (want > 0)).all(), f"row {b}: support differs"
        np.testing.assert_allclose(probs[b], want, rtol=2e-5, atol=1e-9)
    assert compared >= 0.8 * B


def test_reference_draw_mode_of_the_sampler_module():
    """Sampler.reference_draw: torch.multinomial on the kernel's filtered probabilities -- the reference's own call
    sequence from there on (models/sampler.py:63-64), so for one seed the ids equal torch.multinomial's on the oracle
    path of torch ops (division, sort, cumulative sum, mask, soft-max) whenever the two probability tensors agree."""
    from parrotserve_amd.runner import LlamaConfig, Sampler, SamplingConfig

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(4)
    W = (torch.randn(4096, 256, generator=g) * 0.3).half().to(dev)  # logits of a few units: a nucleus of tens of tokens
    h = torch.randn(16, 256, generator=g).half().to(dev)
    s = Sampler(LlamaConfig(vocab_size=4096, hidden_size=256), W)
    s.reference_draw = True
    cfgs = [SamplingConfig(temperature=0.8, top_p=0.9)] * 16
    torch.manual_seed(11)
    ids = s(h, cfgs)
    assert ids.shape == (16,) and ids.dtype == torch.int64
    # the reference's sequence of torch calls on the same logits, same seed
    logits = torch.matmul(h, W.t())
    logits.div_(torch.full((16, 1), 0.8, dtype=logits.dtype, device=dev))
    sl, si = logits.sort(dim=-1, descending=True)
    pr = sl.softmax(dim=-1)
    mask = (pr.cumsum(dim=-1) - pr) > torch.full((16, 1), 0.9, dtype=logits.dtype, device=dev)
    sl[mask] = -float("inf")
    logits = torch.gather(sl, dim=-1, index=torch.argsort(si, dim=-1))
    probs = torch.softmax(logits, dim=-1, dtype=torch.float)
    torch.manual_seed(11)
    want = torch.multinomial(probs, num_samples=1, replacement=True).squeeze(-1)
    mine = kernels.top_p_probs(torch.matmul(h, W.t()), torch.full((16,), 0.8, device=dev), torch.full((16,), 0.9, device=dev))
    same_support = ((mine > 0) == (probs > 0)).all(dim=-1)
    # (the torch path rounds its probabilities and their running sums to fp16, which can move a cut by a token)
    assert same_support.float().mean() >= 0.75
    assert torch.equal(ids[same_support], want[same_support])
