"""Helpers shared by the GPU parity tests."""
import numpy as np

import oracle as orc


def flatten_samples(samples):
    """list of (bg, {key: row}) -> sample[], key[], row[], bg[] in insertion order."""
    s, k, r, bg = [], [], [], []
    for i, (b, mp) in enumerate(samples):
        bg.append(b)
        for kk, rr in mp.items():
            s.append(i)
            k.append(kk)
            r.append(rr)
    return (np.array(s, np.int32), np.array(k, np.int64), np.array(r, np.int32), np.array(bg, np.int32))


def oracle_grids(samples):
    g = orc.Grids(len(samples))
    for i, (bg, mp) in enumerate(samples):
        g.set(i, list(mp.keys()), list(mp.values()), bg)
    return g


def device_grids(scn, ctx, samples, d, n, nSites):
    s, k, r, bg = flatten_samples(samples)
    g = scn.Grids(ctx)
    g.build(len(samples), d, n, s, k, r, bg, nSites)
    return g


def assert_same_grids(dev, ora):
    s, k, r, bg = dev.download()
    os_, ok, or_, obg = ora.flat()
    assert np.array_equal(bg, obg)
    assert np.array_equal(s, os_)
    assert np.array_equal(k, ok)
    assert np.array_equal(r, or_)
