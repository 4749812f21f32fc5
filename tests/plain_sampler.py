"""A plain statement of the reference's sampler: the random generator and the rules by which a
token is drawn from logits.  Shares no code with the engine's sampler."""
from __future__ import annotations

import numpy as np

_MASK = (1 << 64) - 1


def splitmix64(x):
    """Seed spreading, src/sampler/sampler.cpp:16-21."""
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniforms(seed, count):
    """xorshift64* started at splitmix64(seed) (0 becomes 1); the high 32 bits of the product,
    of which the top 24 give u in [0, 1).  src/sampler/sampler.cpp:34-52."""
    state = splitmix64(seed) or 1
    out = np.empty(count, dtype=np.float32)
    for i in range(count):
        state ^= state >> 12
        state ^= (state << 25) & _MASK
        state ^= state >> 27
        u32 = ((state * 0x2545F4914F6CDD1D) & _MASK) >> 32
        out[i] = (u32 >> 8) / 16777216.0
    return out


def sample(logits, temperature, top_k, top_p, u):
    """One draw as src/sampler/sampler.cpp:54-129 makes it.

    Greedy for temperature <= 0 (lowest index among equal maxima).  Otherwise p = exp((l - max)/T)
    in float32, normalised by a float64 sum; candidates sorted by (p descending, index ascending)
    when top-k or top-p filter, else in index order; top-k keeps k, top-p the shortest prefix whose
    mass reaches top_p times the kept mass; the draw walks the kept tokens until r = u * total < cum."""
    logits = np.asarray(logits, dtype=np.float32)
    n = len(logits)
    if temperature <= 0:
        return int(np.argmax(logits))
    p = np.exp((logits - logits.max()) / np.float32(temperature)).astype(np.float32)
    total = float(np.sum(p.astype(np.float64)))
    p = (p * np.float32(1.0 / total)).astype(np.float32)
    order = np.arange(n)
    use_k = 0 < top_k < n
    use_p = top_p < 1.0
    if use_k or use_p:
        order = np.lexsort((np.arange(n), -p))
        if use_k:
            order = order[:top_k]
        if use_p:
            kept = p[order].astype(np.float64)
            threshold = float(np.float32(top_p)) * kept.sum()
            cum = np.cumsum(kept)
            reached = np.nonzero(cum >= threshold)[0]
            if len(reached):
                order = order[:reached[0] + 1]
    kept = p[order].astype(np.float64)
    cum = np.cumsum(kept)
    r = float(np.float32(u)) * cum[-1]
    hit = np.nonzero(r < cum)[0]
    return int(order[hit[0]] if len(hit) else order[-1])
