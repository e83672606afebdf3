"""Philox4x32-10 and the dropout keep-mask built on it.  Test infrastructure only.

Philox4x32-10 is the counter-based generator of Salmon, Moraes, Dror and Shaw
("Parallel random numbers: as easy as 1, 2, 3", SC'11) with the Random123
constants; torch uses the same round function (ATen/core/PhiloxRNGEngine.h).
The reference draws its dropout masks from torch
(oslo/torch/nn/modules/functional.py:295-298 -> F.dropout), whose CPU stream
is mt19937 and cannot be reproduced on a GPU; what is pinned here instead is
the generator itself (known-answer vectors) and the mask layout of
include/oslo_hip.h.

Two independent implementations: `philox4x32_10_int` (Python integers, one
counter) and `philox4x32_10` (numpy, vectorised).
"""
import numpy as np

M0 = 0xD2511F53
M1 = 0xCD9E8D57
W0 = 0x9E3779B9
W1 = 0xBB67AE85
MASK32 = 0xFFFFFFFF


def philox4x32_10_int(counter, key):
    """counter: 4 ints, key: 2 ints (32-bit each) -> 4 ints."""
    c0, c1, c2, c3 = (int(v) & MASK32 for v in counter)
    k0, k1 = (int(v) & MASK32 for v in key)
    for _ in range(10):
        p0 = M0 * c0
        p1 = M1 * c2
        c0, c1, c2, c3 = (
            ((p1 >> 32) ^ c1 ^ k0) & MASK32,
            p1 & MASK32,
            ((p0 >> 32) ^ c3 ^ k1) & MASK32,
            p0 & MASK32,
        )
        k0 = (k0 + W0) & MASK32
        k1 = (k1 + W1) & MASK32
    return c0, c1, c2, c3


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """Vectorised: c* are uint64 arrays holding 32-bit values, k* Python ints.
    Returns four uint32 arrays."""
    c0 = np.asarray(c0, dtype=np.uint64)
    c1 = np.asarray(c1, dtype=np.uint64)
    c2 = np.asarray(c2, dtype=np.uint64)
    c3 = np.asarray(c3, dtype=np.uint64)
    k0 = int(k0) & MASK32
    k1 = int(k1) & MASK32
    m32 = np.uint64(MASK32)
    s32 = np.uint64(32)
    for _ in range(10):
        p0 = np.uint64(M0) * c0
        p1 = np.uint64(M1) * c2
        n0 = (p1 >> s32) ^ c1 ^ np.uint64(k0)
        n1 = p1 & m32
        n2 = (p0 >> s32) ^ c3 ^ np.uint64(k1)
        n3 = p0 & m32
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0 = (k0 + W0) & MASK32
        k1 = (k1 + W1) & MASK32
    return tuple(c.astype(np.uint32) for c in (c0, c1, c2, c3))


def dropout_threshold(p):
    """16-bit keep threshold: an element is kept when its draw >= threshold."""
    t = float(np.float32(p)) * 65536.0 + 0.5
    return 65536 if t >= 65536.0 else int(t)


def group_words(first_group, ngroups, seed, offset):
    """Words of groups first_group .. first_group + ngroups - 1 as a
    [ngroups, 4] uint32 array; counter = (offset_lo, offset_hi, group_lo,
    group_hi), key = (seed_lo, seed_hi)."""
    grp = np.arange(first_group, first_group + ngroups, dtype=np.uint64)
    n = grp.shape[0]
    seed = int(seed)
    offset = int(offset)
    w = philox4x32_10(
        np.full(n, offset & MASK32, dtype=np.uint64),
        np.full(n, (offset >> 32) & MASK32, dtype=np.uint64),
        grp & np.uint64(MASK32),
        grp >> np.uint64(32),
        seed & MASK32,
        (seed >> 32) & MASK32,
    )
    return np.stack(w, axis=1)


def keep_mask(n, p, seed, offset, first_element=0):
    """uint8 keep mask (1 = kept) of elements first_element .. first_element + n - 1.

    Element i belongs to group i // 8 and takes the 16-bit half (i % 8) & 1 of
    word (i % 8) // 2 (low half first); kept when that value >= round(p * 65536).
    """
    first_group = first_element // 8
    last_group = (first_element + n + 7) // 8
    words = group_words(first_group, last_group - first_group, seed, offset)
    halves = np.empty((words.shape[0], 8), dtype=np.uint32)
    halves[:, 0::2] = words & np.uint32(0xFFFF)
    halves[:, 1::2] = words >> np.uint32(16)
    keep = (halves >= np.uint32(min(dropout_threshold(p), 0xFFFFFFFF))).astype(np.uint8)
    if dropout_threshold(p) >= 65536:
        keep[:] = 0
    flat = keep.reshape(-1)
    start = first_element - first_group * 8
    return flat[start:start + n].copy()
