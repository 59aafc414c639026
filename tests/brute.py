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


def coords_of(key, side, d):
    c = []
    for _ in range(d):
        c.append(key % side)
        key = key // side
    return c[::-1]  # most significant axis first


def rules_vectorized(d, batch, sIn, sOut, size, stride, gin):
    """The square rule book with minActive 1 once more, in whole-array numpy, for inputs too large for rules():
    gridRules (Regions.cu:557-652) under ascending-key iteration.
    gin = (sample, key, row, background) of the input grids.  Returns (sample, key, row) of the output sites,
    background row per sample (-1: none), number of rows, and the rules [rows x size^d]."""
    s, k, r, bg = gin
    volIn, volOut = sIn ** d, sOut ** d
    dense = np.repeat(np.asarray(bg, np.int64)[:, None], volIn, 1)  # what a rule says for an empty cell
    dense[s, k] = r
    # owner of an output site: the smallest active input key in its window; a site exists iff it has one.
    # For one window offset, distinct input sites name distinct output sites, so a plain indexed update does.
    s64, k64 = np.asarray(s, np.int64), np.asarray(k, np.int64)
    ic = coords_of(k64, sIn, d)
    owner = np.full(batch * volOut, np.iinfo(np.int64).max, np.int64)
    offs = np.stack(np.meshgrid(*[np.arange(size)] * d, indexing="ij"), -1).reshape(-1, d)
    for off in offs:
        valid, okey = np.ones(len(k64), bool), np.zeros(len(k64), np.int64)
        for a in range(d):
            t = ic[a] - off[a]
            valid &= (t >= 0) & (t % stride == 0) & (t // stride < sOut)
            okey = okey * sOut + t // stride
        idx = s64[valid] * volOut + okey[valid]
        owner[idx] = np.minimum(owner[idx], k64[valid])
    owner = owner.reshape(batch, volOut)
    bs, ks = np.nonzero(owner != np.iinfo(np.int64).max)
    order = np.lexsort((ks, owner[bs, ks], bs))  # by sample, then owner key, then output key
    bs, ks = bs[order], ks[order]
    per = np.bincount(bs, minlength=batch)
    notFull = per < volOut
    # rows: a sample's sites, then its background row if the sample is not full
    before = np.concatenate([[0], np.cumsum(per + notFull)[:-1]])
    rows = before[bs] + (np.arange(len(bs)) - np.concatenate([[0], np.cumsum(per)[:-1]])[bs])
    bgOut = np.where(notFull, before + per, -1)
    nRows = int((per + notFull).sum())
    rules = np.empty((nRows, size ** d), np.int64)
    oc = coords_of(ks, sOut, d)
    for q, off in enumerate(offs):
        kin = np.zeros(len(ks), np.int64)
        for a in range(d):
            kin = kin * sIn + (oc[a] * stride + off[a])
        rules[rows, q] = dense[bs, kin]
    rules[bgOut[notFull]] = np.asarray(bg, np.int64)[notFull][:, None]
    return (bs, ks, rows), bgOut, nRows, rules


def rules_windows(samples, d, nIn, nOut, s, inL, inR, uniform):
    """Rule book over explicit per-sample windows (fractional max-pooling regions): output site j of sample b looks at
    the cells [inL[b][a][j_a], inR[b][a][j_a]) along every axis a.  Rows are s^d wide; `uniform` rows start as all
    background, others as -1 with the background row inside the window's extent.  Same return value as rules()."""
    out_rules, n, outs = [], 0, []
    S = s ** d
    for b, (bg, mp) in enumerate(samples):
        cands = []
        for j in itertools.product(range(nOut), repeat=d):
            ext = [int(inR[b][a][j[a]] - inL[b][a][j[a]]) for a in range(d)]
            row = [bg if uniform else -1] * S
            active = []
            for o in itertools.product(*[range(e) for e in ext]):
                cell = encode(tuple(int(inL[b][a][j[a]]) + o[a] for a in range(d)), nIn)
                k = 0
                for a in range(d):
                    k = k * s + o[a]
                row[k] = mp.get(cell, bg)
                if cell in mp:
                    active.append(cell)
            if active:
                cands.append((min(active), encode(j, nOut), row))
        cands.sort(key=lambda t: (t[0], t[1]))
        grid = {}
        for _, okey, row in cands:
            grid[okey] = n
            n += 1
            out_rules.extend(row)
        obg = -1
        if len(grid) < nOut ** d:
            out_rules.extend([bg] * S)
            obg = n
            n += 1
        outs.append((obg, grid))
    return np.array(out_rules, np.int32), n, outs
