"""Synthetic cohorts for the message kernels: random suffix words, keys, routing tags in every combination the kernels
branch on (suffix below ctx, below ctx / 2, retired recipients, pill receipts, retiring senders)."""
import numpy as np


def cohort(n, p, ctx, packed, seed):
    rng = np.random.default_rng(seed)
    suf = rng.integers(0, 4 * ctx + 1000, n).astype(np.uint64)
    suf[: min(n, 8)] = np.array([0, ctx - 1, ctx, ctx // 2, max(ctx // 2 - 1, 0), ctx + 1, 3 * ctx, 1], dtype=np.uint64)[: min(n, 8)]
    tag = rng.integers(0, 1 << 16, n).astype(np.uint64)
    sa = suf | (tag << np.uint64(48))                       # the forward tag rides in the top 16 bits of a word
    cur = rng.integers(0, p, n).astype(np.uint32) | (np.uint32(0x8000) * (rng.random(n) < 0.2))
    prev = rng.integers(0, p, n).astype(np.uint32) | (np.uint32(0x8000) * (rng.random(n) < 0.2))
    beta = (prev.astype(np.uint32) << np.uint32(16)) | cur.astype(np.uint32)
    if packed:
        primary = rng.integers(0, 1 << 31, n).astype(np.uint64)
        secondary = rng.integers(0, 1 << 31, n).astype(np.uint64)
        pill = (rng.random(n) < 0.3).astype(np.uint64)
        keys = (primary << np.uint64(31)) | secondary | (pill << np.uint64(62))
    else:
        keys = rng.integers(0, 1 << 31, n).astype(np.uint64)
    active_sz = int(rng.integers(0, n + 1))
    return sa, keys, beta.astype(np.uint32), active_sz


def groups(target, rank, end, p):
    """The messages of every destination as a sorted list, whatever their order inside the group."""
    start = 0
    out = []
    for q in range(p):
        e = int(end[q])
        out.append(sorted(zip(target[start:e].tolist(), rank[start:e].tolist())))
        start = e
    return out
