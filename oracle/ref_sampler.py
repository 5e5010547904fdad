"""CPU oracle of the token sampler: temperature, top-p filter, one draw per row.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this module;
tests/ use it as the checker.

Restates parrot/engine/builtin/models/sampler.py:19-66 in numpy float64:
  * :33-40  logits are divided by the row's temperature, in place, so the
            quotient is rounded to the logits' element type;
  * :43-56  rows are sorted in descending order, soft-maxed, and a token is
            dropped when the probability mass sorted strictly before it
            exceeds top_p (so the most likely token always stays, and the
            token on which the running mass crosses top_p stays too);
  * :63-64  the surviving logits are soft-maxed again and one token is drawn
            from that distribution.
Two things the reference leaves to its libraries are fixed here so that the
result is a function of the inputs: ties sort by ascending token id (the
reference's sort is not stable), and the draw is the inverse-CDF draw over
ascending token ids from a uniform number u in [0, 1) that the caller passes
(the reference calls torch.multinomial, whose stream of random numbers is the
library's own: the drawn *distribution* is the same, the drawn token for a
given seed is not reproducible outside that library -- parity unpinned for
the seed-to-token mapping, pinned for the distribution).

Pinning status:
  * softmax / kept set  -- pinned: scipy.special.softmax; brute-force nucleus
                           on tiny rows (smallest sorted prefix whose mass
                           exceeds top_p); top_p -> 0 and temperature -> 0 both
                           reduce to arg-max; top_p = 1 keeps everything.
  * draw                -- pinned: uniform logits give floor(u * V); empirical
                           frequencies of many draws match the probabilities.
The reference's own check (tests/engine/builtin/test_sampler.py:13-40) needs
downloaded weights and the library's random stream and holds no vector that
can be used here.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    """float64 values rounded to the element type ('f16', 'bf16', 'f32'), returned as float64."""
    if dtype == "f32":
        return x.astype(np.float32).astype(np.float64)
    if dtype == "f16":
        return x.astype(np.float32).astype(np.float16).astype(np.float64)
    if dtype == "bf16":  # round to nearest even on the upper 16 bits of the fp32 pattern
        f = np.ascontiguousarray(x.astype(np.float32))
        b = f.view(np.uint32).astype(np.uint64)
        b = (b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000
        return b.astype(np.uint32).view(np.float32).astype(np.float64)
    raise ValueError(dtype)


def kept_probs(logits_row: np.ndarray, temperature: float, top_p: float, dtype: str) -> Tuple[np.ndarray, float]:
    """Probabilities of one row after temperature and the top-p filter (zeros for dropped tokens), and
    the filter's margin: the smallest relative distance between top_p and the mass-before of a token
    (sums of positive terms carry a relative error, so a row with a tiny relative margin is decided by
    rounding noise in any fp32 implementation; a mass-before of exactly zero is exact everywhere)."""
    x = logits_row.astype(np.float64)
    if temperature != 1.0:
        x = round_to(x / np.float64(np.float32(temperature)), dtype)
    e = np.exp(x - x.max())
    p = e / e.sum()
    margin = np.inf
    if top_p < 1.0:
        order = np.lexsort((np.arange(x.size), -x))  # descending value, ties by ascending id
        before = np.cumsum(p[order]) - p[order]
        keep_sorted = before <= np.float64(np.float32(top_p))
        tp = np.float64(np.float32(top_p))
        margin = float(np.min(np.abs(before - tp) / np.maximum(np.maximum(before, tp), 1e-300)))
        keep = np.zeros(x.size, dtype=bool)
        keep[order[keep_sorted]] = True
        e = np.where(keep, e, 0.0)
        p = e / e.sum()
    return p, margin


def draw(p: np.ndarray, u: float) -> Tuple[int, float]:
    """Inverse-CDF draw over ascending token ids: the first id whose inclusive cumulative probability
    exceeds u.  Also returns the relative distance from u to the nearest edge of that id's interval."""
    c = np.cumsum(p)
    u = np.float64(np.float32(u))
    idx = int(np.searchsorted(c, u, side="right"))
    nz = np.nonzero(p)[0]
    idx = min(idx, int(nz[-1]))
    lo = c[idx] - p[idx]
    rel = lambda a, b: abs(a - b) / max(a, b, 1e-300)
    return idx, float(min(rel(u, lo), rel(c[idx], u)))


def ref_sample(logits: np.ndarray, temperature: Optional[np.ndarray], top_p: Optional[np.ndarray],
               uniform: np.ndarray, dtype: str = "f16"):
    """ids [B] int64, and per row the smaller of the filter margin and the draw margin."""
    B = logits.shape[0]
    ids = np.zeros(B, dtype=np.int64)
    margins = np.zeros(B)
    for b in range(B):
        t = 1.0 if temperature is None else float(temperature[b])
        tp = 1.0 if top_p is None else float(top_p[b])
        p, m1 = kept_probs(logits[b], t, tp, dtype)
        ids[b], m2 = draw(p, float(uniform[b]))
        margins[b] = min(m1, m2)
    return ids, margins
