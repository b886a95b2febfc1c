"""Philox4x32-10 counter-based generator, numpy restatement.  TEST INFRASTRUCTURE ONLY.

The fused kernels draw `rand_like` values from this generator (the reference
draws them from cuRAND's Philox4_32_10 with a per-thread subsequence,
src/cuda/epilogue/threadblock/visitor_load.hpp:106-135, which ties the stream
to CUTLASS's thread layout; here the stream is tied to the element instead, so
the result does not depend on the tile configuration).

Definition used by the kernels (evt_ae_amd/csrc/evt_epilogue.hpp, rand_row):
    element e (row-major index in the rand_like tensor) takes word (e & 3) of
    Philox4x32-10(counter = (lo32(e >> 2), hi32(e >> 2), lo32(offset), salt),
                  key = (lo32(seed), hi32(seed)))
    and maps it to a float in [0, 1):  (word >> 8) * 2**-24.

The algorithm is the published one (Salmon et al., "Parallel Random Numbers: As
Easy as 1, 2, 3", SC'11): 10 rounds of
    (c0, c1, c2, c3) <- (hi(M1*c2) ^ c1 ^ k0, lo(M1*c2), hi(M0*c0) ^ c3 ^ k1, lo(M0*c0))
with M0 = 0xD2511F53, M1 = 0xCD9E8D57 and the key bumped by (0x9E3779B9,
0xBB67AE85) between rounds.  It is pinned in tests/test_oracle.py by the
known-answer vectors of the Random123 distribution (kat_vectors, philox4x32 10).
"""
import numpy as np

M0 = np.uint64(0xD2511F53)
M1 = np.uint64(0xCD9E8D57)
W0 = 0x9E3779B9
W1 = 0xBB67AE85
MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter: np.ndarray, key) -> np.ndarray:
    """counter: uint32 array [..., 4]; key: two 32-bit ints.  Returns uint32 [..., 4]."""
    c = [counter[..., i].astype(np.uint64) for i in range(4)]
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = M0 * c[0]
        p1 = M1 * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0 = (k0 + W0) & 0xFFFFFFFF
        k1 = (k1 + W1) & 0xFFFFFFFF
    return np.stack([x.astype(np.uint32) for x in c], axis=-1)


def uniform(seed: int, offset: int, salt: int, numel: int) -> np.ndarray:
    """float32 [numel]: the values the kernels generate for elements 0..numel-1."""
    groups = (numel + 3) // 4
    g = np.arange(groups, dtype=np.uint64)
    ctr = np.empty((groups, 4), dtype=np.uint32)
    ctr[:, 0] = (g & MASK).astype(np.uint32)
    ctr[:, 1] = (g >> np.uint64(32)).astype(np.uint32)
    ctr[:, 2] = np.uint32(offset & 0xFFFFFFFF)
    ctr[:, 3] = np.uint32(salt & 0xFFFFFFFF)
    words = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)).reshape(-1)[:numel]
    return ((words >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)).astype(np.float32)
