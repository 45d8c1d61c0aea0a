"""Counter-based noise for the KeyFormer score path (oracle side, numpy).

Philox4x32-10 as published by Salmon et al. (Random123): ten rounds of
    hi0:lo0 = M0 * c0 ; hi1:lo1 = M1 * c2
    c = (hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0)
with the key bumped by the Weyl constants between rounds.

Counter layout used by the kernels (one call yields the noise of four
consecutive keys of one query row):
    counter = (key_index // 4, query_index, head, 0)
    key     = (seed & 0xffffffff, seed >> 32)
    output word j -> key index 4 * (key_index // 4) + j
The reference takes its noise as an input tensor (convert_eval_rms.py:163);
the seeded form exists because a [heads, S, S] tensor is 1 GiB at S = 4096.
"""
import numpy as np

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = np.uint32(0x9E3779B9)
_W1 = np.uint32(0xBB67AE85)
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """Vectorised Philox4x32-10.  All arguments broadcastable uint32 arrays.

    Returns a tuple of four uint32 arrays.
    """
    c0, c1, c2, c3, k0, k1 = np.broadcast_arrays(
        *[np.asarray(a, dtype=np.uint32) for a in (c0, c1, c2, c3, k0, k1)]
    )
    c0, c1, c2, c3, k0, k1 = [a.copy() for a in (c0, c1, c2, c3, k0, k1)]
    with np.errstate(over="ignore"):
        for _ in range(10):
            p0 = _M0 * c0.astype(np.uint64)
            p1 = _M1 * c2.astype(np.uint64)
            hi0 = (p0 >> np.uint64(32)).astype(np.uint32)
            lo0 = (p0 & _MASK).astype(np.uint32)
            hi1 = (p1 >> np.uint64(32)).astype(np.uint32)
            lo1 = (p1 & _MASK).astype(np.uint32)
            c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
            k0 = k0 + _W0
            k1 = k1 + _W1
    return c0, c1, c2, c3


def uniform_from_bits(x):
    """uint32 -> float64 in (0, 1): the top 23 bits, centred in their bin
    (so that the value is exact in fp32 as well)."""
    return ((np.asarray(x, dtype=np.uint32) >> np.uint32(9)).astype(np.float64) + 0.5) * 2.0 ** -23


def gumbel_noise(seed, n_heads, n_queries, n_keys, heads=None):
    """Standard Gumbel noise g[h, q, k] = -log(-log(u)) as float32.

    `heads` optionally restricts the head axis to the given iterable (memory).
    """
    seed = int(seed)
    k0 = np.uint32(seed & 0xFFFFFFFF)
    k1 = np.uint32((seed >> 32) & 0xFFFFFFFF)
    hs = np.arange(n_heads, dtype=np.uint32) if heads is None else np.asarray(list(heads), dtype=np.uint32)
    nk4 = (n_keys + 3) // 4
    kb = np.arange(nk4, dtype=np.uint32)[None, None, :]
    q = np.arange(n_queries, dtype=np.uint32)[None, :, None]
    h = hs[:, None, None]
    words = philox4x32_10(kb, q, h, np.uint32(0), k0, k1)
    bits = np.stack(words, axis=-1).reshape(len(hs), n_queries, nk4 * 4)[:, :, :n_keys]
    u = uniform_from_bits(bits)
    return (-np.log(-np.log(u))).astype(np.float32)
