#!/usr/bin/env python3
"""Writes tests/golden/tiny_pipeline.json: inputs and expected outputs of the PBS
pipeline on tiny shapes, computed by an INDEPENDENT pure-python implementation
(lists and math only: no torch, no numpy, none of the oracle's code).

The reference repository ships no golden vectors for this path, and the
reference itself is not executed; these vectors pin the oracle's indexing
(segment boundaries, stable tie order, candidate / own-segment masks, first
token block, the causal test on ORIGINAL key positions) against a second,
separately written statement of the algorithm in float64 arithmetic.

    python tests/golden/make_fixtures.py
"""
import json
import math
import os
import random

HERE = os.path.dirname(os.path.abspath(__file__))


def pipeline(q, k, v, bs, seg, thr, force_first):
    """q, k, v: [S][D] python floats of ONE head.  float64 everywhere (the fixture
    inputs are small dyadic numbers so nothing depends on rounding of the inputs)."""
    S, D = len(q), len(q[0])
    rt = math.sqrt(D)
    nseg = S // seg
    sc = nseg * seg
    # 1. key scores from the last `bs` queries over the complete segments
    idx = list(range(S))
    scores = None
    if not (nseg == 0 or (nseg == 1 and S == sc)):
        scores = [0.0] * sc
        for qi in range(S - bs, S):
            lg = [sum(a * b for a, b in zip(q[qi], k[j])) / rt for j in range(sc)]
            m = max(lg)
            ex = [math.exp(x - m) for x in lg]
            z = sum(ex)
            for j in range(sc):
                scores[j] += ex[j] / z / bs
        # 2. stable descending sort inside each segment
        for s in range(nseg):
            loc = sorted(range(s * seg, (s + 1) * seg), key=lambda j: (-scores[j], j))
            idx[s * seg:(s + 1) * seg] = loc
    pk = [k[i] for i in idx]
    pv = [v[i] for i in idx]
    # 3. block pooling on the zero-padded sequence
    nb = (S + bs - 1) // bs
    bps = seg // bs
    idx_pad = idx + list(range(S, nb * bs))

    def pool(x):
        out = []
        for b in range(nb):
            rows = [x[i] if i < S else [0.0] * D for i in range(b * bs, (b + 1) * bs)]
            out.append([sum(r[d] for r in rows) / bs for d in range(D)])
        return out
    Pq, Pk = pool(q), pool(pk)
    probs = [[0.0] * nb for _ in range(nb)]
    sel = [[False] * nb for _ in range(nb)]
    for qb in range(nb):
        cand = [kb for kb in range(nb) if kb // bps != qb // bps and kb <= qb]
        if cand:
            lg = {kb: sum(a * b for a, b in zip(Pq[qb], Pk[kb])) / rt for kb in cand}
            m = max(lg.values())
            z = sum(math.exp(x - m) for x in lg.values())
            for kb in cand:
                probs[qb][kb] = math.exp(lg[kb] - m) / z
        if isinstance(thr, int) and thr == 1:
            for kb in cand:
                sel[qb][kb] = True
        else:
            order = sorted(range(nb), key=lambda kb: (-probs[qb][kb], kb))
            c = 0.0
            for rank, kb in enumerate(order):
                c += probs[qb][kb]
                if c >= thr:
                    for kb2 in order[:rank + 1]:
                        sel[qb][kb2] = True
                    break
    if force_first:
        fb = idx_pad.index(0) // bs
        for qb in range(nb):
            sel[qb][fb] = True
    final = [[sel[qb][kb] or (qb // bps == kb // bps) for kb in range(nb)] for qb in range(nb)]
    # 4. attention over selected blocks, causal on ORIGINAL key positions
    out = []
    for qi in range(S):
        keys = [j for j in range(S) if final[qi // bs][j // bs] and idx[j] <= qi]
        lg = [sum(a * b for a, b in zip(q[qi], pk[j])) / rt for j in keys]
        m = max(lg)
        ex = [math.exp(x - m) for x in lg]
        z = sum(ex)
        out.append([sum(e / z * pv[j][d] for e, j in zip(ex, keys)) for d in range(D)])
    return dict(key_indices=idx, scores=scores, block_probs=probs, block_mask=sel, final_mask=final, out=out)


def dyadic(rng, n, d, scale=4):
    return [[rng.randint(-8, 8) / scale for _ in range(d)] for _ in range(n)]


def main():
    cases = []
    specs = [  # S, D, bs, seg, thr, force_first, seed
        (8, 4, 2, 4, 0.6, True, 1), (16, 4, 2, 4, 0.9, True, 2), (13, 4, 2, 4, 0.7, False, 3),
        (16, 8, 4, 8, 0.5, True, 4), (24, 4, 2, 8, 1, True, 5), (10, 4, 2, 6, 0.8, True, 6),
        (6, 4, 2, 8, 0.9, True, 7),
    ]
    for S, D, bs, seg, thr, ff, seed in specs:
        rng = random.Random(seed)
        q, k, v = dyadic(rng, S, D), dyadic(rng, S, D), dyadic(rng, S, D)
        if S > seg:
            k[3] = list(k[1])          # duplicated keys: exact score ties inside a segment
        res = pipeline(q, k, v, bs, seg, thr, ff)   # S <= seg degenerates to plain causal attention
        cases.append(dict(S=S, D=D, block_size=bs, segment_size=seg, threshold=thr, force_first=ff,
                          q=q, k=k, v=v, expected=res))
    with open(os.path.join(HERE, "tiny_pipeline.json"), "w") as f:
        json.dump(cases, f)
    print(f"wrote {len(cases)} cases")


if __name__ == "__main__":
    main()
