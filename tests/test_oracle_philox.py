"""Pins oracle/philox.py: Random123 known-answer vectors, two independent
implementations against each other, and the mask layout."""
import numpy as np
import pytest

from oracle import philox

# Random123 kat_vectors, philox4x32 with 10 rounds: (counter, key, expected)
KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    (
        (0xFFFFFFFF,) * 4,
        (0xFFFFFFFF,) * 2,
        (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD),
    ),
    (
        (0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344),
        (0xA4093822, 0x299F31D0),
        (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1),
    ),
]


@pytest.mark.parametrize("ctr,key,want", KAT)
def test_known_answer_int(ctr, key, want):
    assert philox.philox4x32_10_int(ctr, key) == want


@pytest.mark.parametrize("ctr,key,want", KAT)
def test_known_answer_numpy(ctr, key, want):
    got = philox.philox4x32_10(*[np.array([c], dtype=np.uint64) for c in ctr], key[0], key[1])
    assert tuple(int(g[0]) for g in got) == want


def test_numpy_matches_int_on_random_counters():
    r = np.random.default_rng(0)
    c = r.integers(0, 2 ** 32, size=(4, 200), dtype=np.uint64)
    k0, k1 = 0x12345678, 0x9ABCDEF0
    got = philox.philox4x32_10(c[0], c[1], c[2], c[3], k0, k1)
    for i in range(200):
        want = philox.philox4x32_10_int([int(c[j, i]) for j in range(4)], (k0, k1))
        assert tuple(int(g[i]) for g in got) == want


def test_group_words_counter_layout():
    seed, offset = 0x0123456789ABCDEF, 0x00000002FFFFFFFF
    w = philox.group_words(2 ** 32 + 5, 3, seed, offset)
    for i in range(3):
        grp = 2 ** 32 + 5 + i
        want = philox.philox4x32_10_int(
            (offset & 0xFFFFFFFF, offset >> 32, grp & 0xFFFFFFFF, grp >> 32),
            (seed & 0xFFFFFFFF, seed >> 32),
        )
        assert tuple(int(v) for v in w[i]) == want


def test_keep_mask_layout_and_slicing():
    seed, offset, p = 1234, 0, 0.1
    m = philox.keep_mask(64, p, seed, offset)
    thr = philox.dropout_threshold(p)
    assert thr == 6554
    w = philox.group_words(0, 8, seed, offset)
    for i in range(64):
        word = int(w[i // 8, (i % 8) // 2])
        half = (word >> 16) if (i % 8) & 1 else (word & 0xFFFF)
        assert m[i] == (1 if half >= thr else 0)
    # any window of the stream equals the same window of a longer stream
    assert np.array_equal(philox.keep_mask(21, p, seed, offset, first_element=13), m[13:34])


def test_keep_mask_statistics_and_edge_probabilities():
    n = 1 << 20
    m = philox.keep_mask(n, 0.1, 1234, 0)
    rate = m.mean()
    sigma = np.sqrt(0.1 * 0.9 / n)
    assert abs(rate - (1 - 6554 / 65536)) < 5 * sigma
    assert philox.keep_mask(1000, 0.0, 7, 3).all()
    assert not philox.keep_mask(1000, 1.0, 7, 3).any()
    # different offsets / seeds give different masks, same arguments the same mask
    a = philox.keep_mask(4096, 0.5, 7, 0)
    assert np.array_equal(a, philox.keep_mask(4096, 0.5, 7, 0))
    assert not np.array_equal(a, philox.keep_mask(4096, 0.5, 7, 4))
    assert not np.array_equal(a, philox.keep_mask(4096, 0.5, 8, 0))
    assert abs(a.mean() - 0.5) < 0.05
