// Host harness for csrc/scn_pyr_dev.h: the per-lane bodies of the kernels that
// build a net's rule books from the output side, run here lane after lane with
// the barriers between the sweeps, on plain memory.  Built with the address and
// undefined-behaviour sanitizers by tests/test_chain_cpu.py, which compares
// what comes out with the oracle: every index the kernels compute is computed
// here first, on the CPU, with bounds checked.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include "scn_pyr_dev.h"

namespace {

unsigned magic(long long x) { return (unsigned)((1ull << 32) / (unsigned long long)(x > 0 ? x : 1) + 1); }
long long ipow(long long a, int d) {
  long long r = 1;
  for (int i = 0; i < d; ++i)
    r *= a;
  return r;
}

// k_pyr_masks for sample b with T lanes
template <int D> void pass_a(const PyrArgs &a, int b, int T, bool *gaveUp) {
  std::vector<pyr_u64> lds((size_t)a.pyrStride + 64, 0);
  pyr_u64 *masks = lds.data();
  unsigned short *pref = reinterpret_cast<unsigned short *>(lds.data() + a.maskWords);
  int cnt[PYR_MAX_LEVELS + 1] = {0};
  {
    const PyrLevel &L = a.lv[0];
    for (int t = 0; t < T; ++t)
      for (int w = t; w < L.words + 2; w += T)
        masks[w] = w < L.words ? pyr_source_word(a.bits, L.volOut, b, (unsigned)w) : 0ull;
  }
  for (int x = 1; x < a.nMasks; ++x) { // (the masks start as zero: the pieces are OR-ed in)
    const PyrLevel &L = a.lv[x];
    const pyr_u64 *in = masks + a.lv[x - 1].maskOff;
    pyr_u64 *out = masks + L.maskOff;
    for (int t = 0; t < T; ++t)
      pyr_sweep_dilate<D>(in, out, L.nIn, L.nOut, L.size, L.stride, L.magicN, L.seg, L.segs, L.magicSegs, t, T);
  }
  for (int x = 0; x < a.nMasks; ++x) {
    const PyrLevel &L = a.lv[x];
    unsigned carry = 0;
    for (int w = 0; w < L.words + 2; ++w) {
      pref[L.maskOff + w] = (unsigned short)carry;
      carry += (unsigned)pyr_popc64(masks[L.maskOff + w]);
    }
    cnt[x] = (int)carry;
  }
  memcpy(a.pyramid + (long long)b * a.pyrStride, lds.data(), 8ll * a.pyrStride);
  for (int x = 0; x < a.nMasks; ++x) {
    int *c = a.counts + ((long long)x * a.batch + b) * 2;
    c[0] = cnt[x];
    c[1] = (long long)cnt[x] < a.lv[x].fullSize;
  }
  bool fits = pyr_fits(a, cnt);
  for (int x = 0; x < a.nMasks; ++x)
    fits = fits && cnt[x] <= PYR_ROWS_MAX;
  if (!fits)
    *gaveUp = true;
}

// k_pyr_rules for sample b with T lanes; report: [nLevels + 1][4]
template <int D> void pass_b(const PyrArgs &a, int b, int T, bool gaveUp, long long *report, bool *overOut) {
  std::vector<unsigned char> ldsv((size_t)a.ldsBytesB);
  unsigned char *lds = ldsv.data();
  PyrHdr *h = reinterpret_cast<PyrHdr *>(lds);
  h->over = 0;
  memcpy(lds + PYR_HDR_BYTES, a.pyramid + (long long)b * a.pyrStride, 8ll * a.pyrStride);
  for (int x = 0; x < a.nMasks; ++x) {
    const int *cnt = a.counts + (long long)x * a.batch * 2;
    long long v0 = 0, v1 = 0, v2 = 0, v3 = 0;
    int mx = 0;
    for (int s = 0; s < a.batch; ++s) {
      const int n = cnt[2 * s], hb = cnt[2 * s + 1];
      if (s < b) {
        v0 += n;
        v1 += hb;
      }
      v2 += n;
      v3 += hb;
      mx = n > mx ? n : mx;
    }
    h->n[x] = cnt[2 * b];
    h->hasBg[x] = cnt[2 * b + 1];
    h->actBefore[x] = v0;
    h->bgBefore[x] = v1;
    h->actAll[x] = v2;
    h->bgAll[x] = v3;
    h->maxAct[x] = mx;
  }
  for (int t = 1; t <= a.nLevels; ++t)
    if (pyr_report(a, a.lv[t], h, t).over)
      h->over |= 1;
  if (!pyr_fits(a, h->n))
    h->over |= 2;
  const bool over = h->over != 0 || gaveUp;
  if (b == 0)
    for (int t = 1; t <= a.nLevels; ++t) {
      const PyrReport r = pyr_report(a, a.lv[t], h, t);
      report[4 * t + 0] = r.nSites;
      report[4 * t + 1] = r.nActive;
      report[4 * t + 2] = over;
      report[4 * t + 3] = r.extra;
    }
  if (over) {
    *overOut = true;
    return;
  }
  int windows = 0;
  for (int xa = 0;;) {
    const int xb = pyr_window_end(a, h->n, xa);
    const int la = xa + 1, lb = xb;
    const bool last = xb == a.nMasks - 1;
    ++windows;
    for (int t = 0; t <= a.nMasks; ++t)
      pyr_fill_offsets(h, xa, xb, t);
    for (int t = 0; t < a.nMasks; ++t)
      pyr_fill_en(a.lv[t], lds, t, h->siteOff[t]);
    const PyrLds s = pyr_lds_view(a, lds, h->total, h->n[xa]);
    // (the last array must end inside what pass B was launched with)
    if (s.kOf + h->total > lds + a.ldsBytesB || pyr_lds_window(a, h->n, xa, xb) > a.ldsBytesB) {
      fprintf(stderr, "a window takes more LDS than pass B was launched with\n");
      abort();
    }
    for (int t = 1; t <= a.nLevels; ++t)
      if ((t >= la && t <= lb) || (last && t == a.nLevels && t > lb))
        pyr_fill_level(a.lv[t], a.lv[t - 1].maskOff, a.bg[b], s, t, xa);
    for (int t = 0; t < T; ++t)
      pyr_sweep_clear(s, t, T);
    for (int t = 0; t < T; ++t)
      pyr_sweep_enumerate<D>(a, s, xa, xb, t, T);
    if (xa == 0) {
      const PyrLevel &L = a.lv[0];
      const long long p0 = (long long)b * L.volOut;
      for (int r = 0; r < h->n[0]; ++r) {
        int c[D];
        pyr_unpack<D>(s.key[r], c);
        s.srcRow[r] = (unsigned)a.dense[p0 + pyr_key<D>(c, L.nOut)];
      }
    }
    for (int t = 0; t < T; ++t)
      pyr_sweep_owners<D>(s, la, lb, t, T);
    for (int x = xa; x < xb; ++x) {
      unsigned carry = 0;
      for (int r = 0; r < h->n[x]; ++r) {
        s.base[h->siteOff[x] + r] = (unsigned short)carry;
        carry += (unsigned)pyr_popc32(pyr_own_mask(s, (unsigned)(h->siteOff[x] + r)));
      }
      if ((int)carry != h->n[x + 1]) {
        fprintf(stderr, "level %d: %u sites owned, %d sites exist\n", x + 1, carry, h->n[x + 1]);
        abort();
      }
    }
    for (int t = 0; t < T; ++t)
      pyr_sweep_rows<D>(s, la, lb, b, t, T);
    for (int t = 0; t < T; ++t)
      pyr_sweep_rules<D>(s, la, lb, t, T);
    for (int t = 0; t < T; ++t)
      pyr_sweep_tail(a, s, la, lb, b, t, T);
    if (last)
      break;
    for (int t = 0; t < T; ++t)
      pyr_sweep_carry(s, lds, a, xb, t, T);
    xa = xb;
  }
  if (windows > report[0])
    report[0] = windows; // (the most windows a sample took)
}

template <int D> int run(PyrArgs &a, int T, long long *report) {
  bool gaveUp = false, over = false;
  for (int b = 0; b < a.batch; ++b)
    pass_a<D>(a, b, T / 2 > 0 ? T / 2 : 1, &gaveUp);
  for (int b = 0; b < a.batch; ++b)
    pass_b<D>(a, b, T, gaveUp, report, &over);
  return (gaveUp ? 1 : 0) | (over ? 2 : 0);
}

} // namespace

// geo: per recorded layer {kind, nIn, nOut, size, stride}.  Source grids as
// scn_grids_build takes them.  Per layer l (1-based) rules[l - 1] (capacity
// rulesCap[l - 1] ints, may be null), ekey / erow / bgOut [l - 1]; bounds
// [l - 1][2] = {rows, active}.  report: [nLevels + 1][4] = sites, active sites,
// outgrew, terminal width or largest sample; report[0][0] = the most windows of
// levels a sample was built in.  Returns 0, or 1 | 2 when a sample
// outgrew the LDS or a layer its bounds (nothing is written then).
extern "C" int pyr_cpu_chain(int d, int batch, int n0, int nLevels, const int *geo, const int *sample,
                             const long long *key, const int *row, long long nActive, const int *bg,
                             int **rules, const long long *rulesCap, long long **ekey, int **erow, int **bgOut,
                             const long long *bounds, long long *report, int ldsBytesB, int T) {
  PyrArgs a;
  memset(&a, 0, sizeof(a));
  const long long vol0 = ipow(n0, d);
  std::vector<pyr_u64> bits((size_t)((batch * vol0 + 63) / 64 + 2), 0);
  std::vector<int> dense((size_t)(batch * vol0), -7);
  for (long long i = 0; i < nActive; ++i) {
    const long long p = (long long)sample[i] * vol0 + key[i];
    bits[p >> 6] |= 1ull << (p & 63);
    dense[p] = row[i];
  }
  a.nLevels = nLevels;
  a.batch = batch;
  a.d = d;
  a.dense = dense.data();
  a.bits = bits.data();
  a.bg = bg;
  long long maskWords = 0;
  {
    PyrLevel &L = a.lv[0];
    L.kind = PYR_REGIONS;
    L.nIn = L.nOut = n0;
    L.size = L.stride = L.width = 1;
    L.volOut = vol0;
    L.fullSize = vol0 + 1;
    L.words = (int)((vol0 + 63) / 64);
    L.maskOff = 0;
    L.magicN = magic(n0);
    L.magicS = magic(1);
    maskWords = L.words + 2;
  }
  a.nMasks = 1;
  for (int l = 1; l <= nLevels; ++l) {
    const int *g = geo + 5 * (l - 1);
    PyrLevel &L = a.lv[l];
    L.kind = g[0];
    L.nIn = g[1];
    L.nOut = g[2];
    L.size = g[3];
    L.stride = g[4];
    L.width = L.kind == PYR_TERMINAL ? 1 : (int)ipow(L.size, d);
    L.volOut = L.kind == PYR_TERMINAL ? 1 : ipow(L.nOut, d);
    L.fullSize = L.volOut;
    L.magicN = magic(L.nOut);
    L.magicS = magic(L.size);
    pyr_set_pieces(L);
    L.rules = rules[l - 1];
    L.capacity = rulesCap[l - 1];
    L.ekey = ekey[l - 1];
    L.erow = erow[l - 1];
    L.bg = bgOut[l - 1];
    L.boundRows = bounds[2 * (l - 1)];
    L.boundActive = bounds[2 * (l - 1) + 1];
    if (L.kind == PYR_REGIONS) {
      L.words = (int)((L.volOut + 63) / 64);
      L.maskOff = (int)maskWords;
      maskWords += L.words + 2;
      a.nMasks = l + 1;
    }
  }
  long long pyrStride = maskWords + (maskWords + 3) / 4;
  pyrStride = (pyrStride + 1) / 2 * 2;
  a.maskWords = (int)maskWords;
  a.pyrStride = (int)pyrStride;
  a.ldsBytesB = ldsBytesB;
  std::vector<pyr_u64> pyramid((size_t)(batch * pyrStride));
  std::vector<int> counts((size_t)a.nMasks * batch * 2);
  a.pyramid = pyramid.data();
  a.counts = counts.data();
  if (PYR_HDR_BYTES + 8 * pyrStride > ldsBytesB)
    return 4;
  switch (d) {
  case 1:
    return run<1>(a, T, report);
  case 2:
    return run<2>(a, T, report);
  default:
    return run<3>(a, T, report);
  }
}
