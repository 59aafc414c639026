"""Independent brute-force rulebook builders used to pin the oracle.

They do not follow the reference's loop structure: the active output set is
computed by scanning every output site's window, rows are numbered by sorting
on (smallest active key in the window, output key), and the background row is
appended when the output grid is not full.
"""
import itertools

import numpy as np


def decode(key, n, d):
    c = []
    for _ in range(d):
        c.append(key % n)
        key //= n
    return tuple(reversed(c))


def encode(c, n):
    k = 0
    for x in c:
        k = k * n + x
    return k


def tri_ord(s, d):
    ordv, S = [], 0
    for off in itertools.product(range(s), repeat=d):
        if sum(off) < s:
            ordv.append(S)
            S += 1
        else:
            ordv.append(-1)
    return ordv, S


def triangle_size(n, d):
    return sum(1 for j in itertools.product(range(n), repeat=d) if sum(j) < n)


def rules(samples, d, nIn, nOut, size, stride, minActive=1, triangular=False):
    """samples: list of (bg, dict key->row).  Returns (rules, nSites, outs)
    with outs = list of (bg, dict key->row)."""
    out_rules, n, outs = [], 0, []
    ordv, S = tri_ord(size, d) if triangular else (None, size ** d)
    full = triangle_size(nOut, d) if triangular else nOut ** d
    offs = list(itertools.product(range(size), repeat=d))
    for bg, mp in samples:
        cands = []
        for j in itertools.product(range(nOut), repeat=d):
            if triangular and sum(j) >= nOut:
                continue
            win = [encode(tuple(j[a] * stride + o[a] for a in range(d)), nIn) for o in offs]
            act_sq = [k for k in win if k in mp]
            if not act_sq:
                continue
            if triangular:
                row = [mp.get(win[q], bg) for q in range(len(offs)) if ordv[q] >= 0]
                count = sum(1 for q in range(len(offs)) if ordv[q] >= 0 and win[q] in mp)
            else:
                row = [mp.get(k, bg) for k in win]
                count = len(act_sq)
            if minActive == -1:
                centre = encode(tuple(x + 1 for x in j), nIn)
                if centre not in mp:
                    continue
                cands.append((encode(j, nOut), encode(j, nOut), row))
                continue
            if minActive > 1 and count < minActive:
                continue
            cands.append((min(act_sq), encode(j, nOut), row))
        cands.sort(key=lambda t: (t[0], t[1]))
        grid = {}
        for _, okey, row in cands:
            grid[okey] = n
            n += 1
            out_rules.extend(row)
        obg = -1
        if len(grid) < full:
            out_rules.extend([bg] * S)
            obg = n
            n += 1
        outs.append((obg, grid))
    return np.array(out_rules, np.int32), n, outs


def random_samples(rng, batch, d, nIn, density, with_bg=True, shuffle=True):
    """Layer-0 style grids: bg row first (if any), then sites in shuffled order."""
    samples, row = [], 0
    for _ in range(batch):
        vol = nIn ** d
        k = rng.random(vol) < density
        keys = np.flatnonzero(k)
        if shuffle:
            rng.shuffle(keys)
        bg = -1
        if with_bg and keys.size < vol:
            bg = row
            row += 1
        elif keys.size < vol:
            # a not-full grid always needs a background row
            bg = row
            row += 1
        mp = {}
        for kk in keys:
            mp[int(kk)] = row
            row += 1
        samples.append((bg, mp))
    return samples, row
