"""CPU restatement of the Philox4x32-10 counter-based generator (Salmon, Moraes, Dror, Shaw:
"Parallel random numbers: as easy as 1, 2, 3", SC'11) and of the mask rule of the library's
optional fast random stream. Test infrastructure only, like the rest of oracle/.

The reference has no such generator: its GPU handler draws masks with cuRAND's XORWOW
(pycuda_handler.py:37-39, 191-193), a stream that matches NumPy's no more than this one does.
Pinned by the generator's published known-answer vectors (tests/test_oracle_pinning.py).
"""
import numpy as np

M0, M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
W0, W1 = 0x9E3779B9, 0xBB67AE85
MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(counters, key):
    """counters: (n, 4) uint32; key: two uint32. Returns the (n, 4) uint32 outputs."""
    c = [np.asarray(counters)[:, i].astype(np.uint64) for i in range(4)]
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0, p1 = M0 * c[0], M1 * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK32
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK32
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0, k1 = (k0 + W0) & 0xFFFFFFFF, (k1 + W1) & 0xFFFFFFFF
    return np.stack(c, axis=1).astype(np.uint32)


def mask_threshold(probability):
    """A 32-bit draw u gives 1.0 when u < threshold: P(1) = floor(p * 2^32) / 2^32, clipped to [0, 1]."""
    return int(min(max(np.floor(float(probability) * 4294967296.0), 0.0), 4294967296.0))


def probability_mask(n, probability, seed, offset):
    """Elements 4b .. 4b+3 of the mask are the four words of block `offset + b` under key `seed`
    (both 64-bit, low word first). Returns (mask as float32 of n elements, blocks consumed)."""
    blocks = (n + 3) // 4
    ctr = np.zeros((blocks, 4), np.uint32)
    idx = np.uint64(offset) + np.arange(blocks, dtype=np.uint64)
    ctr[:, 0] = (idx & MASK32).astype(np.uint32)
    ctr[:, 1] = (idx >> np.uint64(32)).astype(np.uint32)
    words = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)).reshape(-1)[:n]
    return (words.astype(np.uint64) < np.uint64(mask_threshold(probability))).astype(np.float32), blocks
