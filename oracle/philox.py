"""Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
SC'11; the Random123 library) and the element-wise streams the device RNG derives from it.

TEST INFRASTRUCTURE: a numpy restatement used by tests/ and the CPU emulator to check
nabla_amd/csrc/random.hip; nothing in the product imports it.

Pinned by the known-answer vectors of Random123's kat_vectors for philox4x32 with 10 rounds
(tests/test_oracle_pins.py).  The reference framework draws its random numbers from MAX
(nabla/ops/creation.py:152-183, ops.random.uniform / gaussian), whose generator is not part
of the reference's sources: value parity with it is unpinned; what is pinned is the generator
itself, the distribution of the streams and their reproducibility.
"""
from __future__ import annotations

import numpy as np

M0, M1 = 0xD2511F53, 0xCD9E8D57
W0, W1 = 0x9E3779B9, 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter: np.ndarray, key: np.ndarray) -> np.ndarray:
    """``counter`` [..., 4] and ``key`` [..., 2] (uint32, broadcastable) -> [..., 4] uint32."""
    c = [np.asarray(counter[..., i], dtype=np.uint64) for i in range(4)]
    k0 = np.asarray(key[..., 0], dtype=np.uint64)
    k1 = np.asarray(key[..., 1], dtype=np.uint64)
    for r in range(10):
        if r:
            k0 = (k0 + np.uint64(W0)) & _MASK
            k1 = (k1 + np.uint64(W1)) & _MASK
        p0 = np.uint64(M0) * c[0]
        p1 = np.uint64(M1) * c[2]
        c = [(p1 >> np.uint64(32)) ^ c[1] ^ k0, p1 & _MASK, (p0 >> np.uint64(32)) ^ c[3] ^ k1, p0 & _MASK]
    return np.stack(c, axis=-1).astype(np.uint32)


def words(n: int, seed: int, run: int, stream: int) -> np.ndarray:
    """The first ``n`` 32-bit words of stream ``stream`` in run ``run`` under ``seed``: element i
    is word i % 4 of the block with counter (i // 4 low, i // 4 high, stream, run) and key
    (seed low, seed high)."""
    blocks = (n + 3) // 4
    idx = np.arange(blocks, dtype=np.uint64)
    ctr = np.stack([idx & _MASK, idx >> np.uint64(32), np.full(blocks, stream & 0xFFFFFFFF, np.uint64),
                    np.full(blocks, run & 0xFFFFFFFF, np.uint64)], axis=-1)
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint64)
    return philox4x32_10(ctr, key[None, :]).reshape(-1)[:n]


def unit_floats(w: np.ndarray) -> np.ndarray:
    """24 high bits of each word as a float32 in [0, 1)."""
    return ((w >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)).astype(np.float32)


def uniform(n: int, low: float, high: float, seed: int, run: int, stream: int) -> np.ndarray:
    u = unit_floats(words(n, seed, run, stream))
    return (np.float32(low) + np.float32(high - low) * u).astype(np.float32)


def keep_mask(n: int, p: float, seed: int, run: int, stream: int) -> np.ndarray:
    """``uniform[0, 1) > p`` (the keep mask of dropout with rate p)."""
    return unit_floats(words(n, seed, run, stream)) > np.float32(p)


def normal(n: int, mean: float, std: float, seed: int, run: int, stream: int) -> np.ndarray:
    """Box-Muller on the word pairs (0, 1) and (2, 3) of every block: the first word, moved into
    (0, 1], gives the radius, the second the angle; the pair yields the cosine and the sine."""
    w = words((n + 3) // 4 * 4, seed, run, stream).reshape(-1, 2)
    u1 = ((w[:, 0] >> np.uint32(8)).astype(np.float64) + 1.0) * 2.0 ** -24
    u2 = (w[:, 1] >> np.uint32(8)).astype(np.float64) * 2.0 ** -24
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.stack([r * np.cos(2.0 * np.pi * u2), r * np.sin(2.0 * np.pi * u2)], axis=-1).reshape(-1)[:n]
    return (mean + std * z).astype(np.float32)
