"""A slow, sort-everything transcription of the reference's sampler for one row, with the uniform number given.

Written from /root/reference/src/inference/sampler.hpp:258-378: keep = top_k when 0 < top_k < m else m; weight =
exp((score - best) / temp) in float32; sums in double; all kept and no top-p: walk ids in increasing order; top-k
without top-p: walk the kept ids in increasing order (weights below min_p count 0); top-p: the shortest ranked prefix
(best first; ties to the lower id, :76-82) whose weight reaches top_p of the kept weight, min_p cuts its tail, the draw
walks it best first; when no running sum exceeds r * sum the best token is returned.
"""

import math
import struct


def f32(x):
    return struct.unpack("f", struct.pack("f", x))[0]


def weight(score, best, temp):
    # float32 arithmetic as the reference: expf((score - best) / temp)
    return f32(math.exp(f32(f32(score - best) / f32(temp))))


def sample(scores, temp, top_k, top_p, min_p, r, skip=None):
    return prepare(scores, temp, top_k, top_p, min_p, skip)(r)


def prepare(scores, temp, top_k, top_p, min_p, skip=None):
    """draw(r) for one row and its settings: everything that does not depend on the uniform number r (the ranking, the
    weights and their sums, the nucleus) is formed once, so that many draws of one row stay affordable."""
    n = len(scores)
    ids = [i for i in range(n) if i != skip]
    m = len(ids)
    ranked = sorted(ids, key=lambda i: (-scores[i], i))
    if temp <= 0.0:
        return lambda r: ranked[0]
    keep = top_k if 0 < top_k < m else m
    best = scores[ranked[0]]
    cut = lambda w: 0.0 if w < f32(min_p) else w

    def walk(order, w, total):
        def draw(r):
            target = f32(r) * total
            acc = 0.0
            for i in order:
                acc += w[i]
                if target < acc:
                    return i
            return ranked[0]
        return draw

    if keep == m and top_p >= 1.0:
        w = {i: cut(weight(scores[i], best, temp)) for i in ids}
        total = 0.0
        for i in ids:
            total += w[i]
        return walk(ids, w, total)
    kept_ranked = ranked[:keep]
    kept = sorted(kept_ranked)
    w = {i: weight(scores[i], best, temp) for i in kept}
    total = 0.0
    for i in kept:
        total += w[i]
    if top_p >= 1.0:
        if min_p > 0.0:
            total = 0.0
            for i in kept:
                w[i] = cut(w[i])
                total += w[i]
        return walk(kept, w, total)
    goal = f32(top_p) * total
    nucleus_weight, nucleus = 0.0, 0
    while True:
        nucleus_weight += w[kept_ranked[nucleus]]
        nucleus += 1
        if not (nucleus < keep and nucleus_weight < goal):
            break
    if min_p > 0.0:
        last = nucleus
        while last > 1 and w[kept_ranked[last - 1]] < f32(min_p):
            last -= 1
        if last < nucleus:
            nucleus = last
            nucleus_weight = 0.0
            for i in range(nucleus):
                nucleus_weight += w[kept_ranked[i]]
    return walk(kept_ranked[:nucleus], w, nucleus_weight)
