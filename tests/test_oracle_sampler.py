"""Pins of the sampler oracle (oracle/ref_sampler.py): library softmax, brute-force nucleus, arg-max limits,
closed-form draws and empirical frequencies."""
import itertools

import numpy as np
import pytest
import scipy.special

from oracle import ref_sampler as rs


def test_unfiltered_probabilities_are_the_library_softmax():
    rng = np.random.default_rng(0)
    x = rs.round_to(rng.normal(0, 3, size=257), "f16")
    p, margin = rs.kept_probs(x, 1.0, 1.0, "f16")
    np.testing.assert_allclose(p, scipy.special.softmax(x), rtol=1e-12)
    assert margin == np.inf


@pytest.mark.parametrize("seed", range(6))
def test_kept_set_is_the_smallest_sorted_prefix_whose_mass_exceeds_top_p(seed):
    """Brute force over every subset of a 7-token row: among the subsets that are closed under 'more likely
    than a member' (top-k sets) the kept set is the smallest one whose mass is above top_p."""
    rng = np.random.default_rng(seed)
    x = rng.normal(0, 1.5, size=7)
    top_p = float(rng.uniform(0.05, 0.95))
    p_all = scipy.special.softmax(x)
    best = None
    for r in range(1, 8):
        for sub in itertools.combinations(range(7), r):
            rest = [i for i in range(7) if i not in sub]
            if rest and min(p_all[list(sub)]) < max(p_all[rest]):
                continue  # not a top-k set
            if p_all[list(sub)].sum() > np.float64(np.float32(top_p)):
                best = set(sub)
                break
        if best:
            break
    p, _ = rs.kept_probs(x, 1.0, top_p, "f32")
    assert set(np.nonzero(p)[0].tolist()) == best
    kept = sorted(best)
    np.testing.assert_allclose(p[kept], p_all[kept] / p_all[kept].sum(), rtol=1e-12)


def test_limits_reduce_to_arg_max():
    rng = np.random.default_rng(3)
    x = rs.round_to(rng.normal(0, 2, size=(5, 1000)), "f16")
    u = rng.uniform(0, 1, size=5)
    ids, _ = rs.ref_sample(x, None, np.full(5, 1e-6), u)
    assert ids.tolist() == x.argmax(1).tolist()
    ids, _ = rs.ref_sample(x, np.full(5, 1e-3), None, u)  # a tiny temperature puts all mass on the maximum
    assert ids.tolist() == x.argmax(1).tolist()


def test_most_likely_token_survives_any_top_p_and_ties_go_to_the_lower_id():
    x = np.array([0.0, 2.0, 2.0, 1.0])
    p, _ = rs.kept_probs(x, 1.0, 0.0, "f32")
    assert np.nonzero(p)[0].tolist() == [1]
    # mass before the second 2.0 is 0.3995: kept at 0.45, dropped at 0.35
    assert np.nonzero(rs.kept_probs(x, 1.0, 0.45, "f32")[0])[0].tolist() == [1, 2]
    assert np.nonzero(rs.kept_probs(x, 1.0, 0.35, "f32")[0])[0].tolist() == [1]


def test_temperature_quotient_is_rounded_to_the_element_type():
    x = np.array([1.0, 3.0, 0.333251953125])  # fp16 values
    t = 0.7
    p, _ = rs.kept_probs(x, t, 1.0, "f16")
    q = (x.astype(np.float32) / np.float32(t)).astype(np.float16).astype(np.float64)
    np.testing.assert_allclose(p, scipy.special.softmax(q), rtol=1e-12)
    pb, _ = rs.kept_probs(x, t, 1.0, "bf16")
    assert not np.allclose(p, pb, rtol=1e-6)  # the coarser type shows


def test_bf16_rounding_matches_torch():
    import torch

    rng = np.random.default_rng(5)
    x = rng.normal(0, 10, size=4096)
    want = torch.from_numpy(x).to(torch.float32).to(torch.bfloat16).to(torch.float64).numpy()
    np.testing.assert_array_equal(rs.round_to(x, "bf16"), want)


def test_uniform_logits_draw_floor_u_times_v():
    V = 64  # 1/64 and its multiples are exact, so the interval edges are too
    p, _ = rs.kept_probs(np.zeros(V), 1.0, 1.0, "f32")
    for u in [0.0, 0.0155, 0.0157, 0.5, 0.731, 0.99999]:
        assert rs.draw(p, u)[0] == int(np.float64(np.float32(u)) * V)


def test_draw_frequencies_match_the_probabilities():
    rng = np.random.default_rng(7)
    x = rng.normal(0, 1, size=8)
    p, _ = rs.kept_probs(x, 1.0, 0.9, "f32")
    n = 200_000
    us = rng.uniform(0, 1, size=n)
    counts = np.bincount([rs.draw(p, u)[0] for u in us], minlength=8)
    assert (counts[p == 0] == 0).all()
    np.testing.assert_allclose(counts / n, p, atol=4 * np.sqrt(0.25 / n))


def test_draw_never_returns_a_dropped_token_at_the_top_of_the_range():
    p = np.array([0.5, 0.5, 0.0, 0.0])
    assert rs.draw(p, np.nextafter(np.float32(1.0), np.float32(0.0)))[0] == 1
