"""Statistics of the dropout hash, on the host model of it (tests/dropout_model.py): keep rate, independence of
the masks of neighbouring seeds, units and streams, and that no index permutation relates them."""
import numpy as np
import pytest

import dropout_model as dm

N = 256
P = 0.25


def _rate(m):
    return float(m.mean())


def test_keep_rate_and_byte_independence():
    m = dm.keep_mask(12345, 3, 0, N, P)
    assert abs(_rate(m) - (1 - P)) < 0.01
    # the four pairs of a 2x2 block come from the four bytes of one word: pairwise independent
    for a, b in (((0, 0), (0, 1)), ((0, 0), (1, 0)), ((0, 1), (1, 1))):
        ma, mb = m[a[0]::2, a[1]::2], m[b[0]::2, b[1]::2]
        assert abs(_rate(ma & mb) - (1 - P) ** 2) < 0.015


@pytest.mark.parametrize("delta", [1, 2, 5, N // 2, (N // 2) ** 2, 1 << 32, (1 << 32) + 1])
def test_neighbouring_seeds_give_unrelated_masks(delta):
    s = 0x1234_5678_9ABC
    a = dm.keep_mask(s, 0, 0, N, P)
    b = dm.keep_mask(s ^ delta, 0, 0, N, P)
    # equal positions: joint keep rate of two independent masks
    assert abs(_rate(a & b) - (1 - P) ** 2) < 0.01
    # no XOR permutation of the key-pair or query-pair index maps one word table onto the other: for
    # every constant c below the table size the permuted tables agree in about 2^-32 of the positions
    wa, wb = dm.words(s, 0, 0, N), dm.words(s ^ delta, 0, 0, N)
    idx = np.arange(N // 2)
    for c in list(range(1, 16)) + [N // 4, N // 2 - 1, delta % (N // 2)]:
        assert (wa[:, idx ^ c] == wb).mean() < 1e-3
        assert (wa[idx ^ c, :] == wb).mean() < 1e-3
    assert (wa == wb).mean() < 1e-3


def test_units_and_streams_are_independent_whatever_the_upper_seed_half():
    s1, s2 = 7, 7 | (0x85EBCA77 << 32)       # the second differs in its upper half only
    base = dm.keep_mask(s1, 0, 0, N, P)
    for seed, unit, stream in ((s1, 0, 1), (s1, 1, 0), (s1, 5, 1), (s2, 0, 0), (s2, 1, 0), (s2, 0, 1)):
        other = dm.keep_mask(seed, unit, stream, N, P)
        assert abs(_rate(base & other) - (1 - P) ** 2) < 0.01, (seed, unit, stream)
        assert (dm.words(s1, 0, 0, N) == dm.words(seed, unit, stream, N)).mean() < 1e-3


def test_threshold_steps():
    for p in (0.0, 1 / 256, 0.5, 255 / 256):
        m = dm.keep_mask(99, 2, 1, N, p)
        assert abs(_rate(m) - (1 - round(p * 256) / 256)) < 0.01
    assert dm.keep_mask(99, 2, 1, N, 0.0).all()
