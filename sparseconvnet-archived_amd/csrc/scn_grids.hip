// Sparse grids in HBM and rule-book construction.
//
// A batch of SparseGrids (SparseGrid.h:26-37) is kept as
//   * an occupancy bit mask over the packed coordinates (packed coordinate =
//     sample * spatialSize^d + key), with an exclusive popcount prefix per
//     64-bit word, so that the position of a site in map iteration order
//     (sample, then ascending key) -- its rank -- is prefix + popcount;
//   * the rows by rank: the row of the site at every position of iteration
//     order.  "Which row has site p" is one mask word, one prefix word and one
//     element of this array, and sites that are neighbours along the innermost
//     axis are neighbours in it: a run of a rule row reads consecutive words;
//   * the list of entries (packed coordinate, row) in no particular order;
//   * for look-ups by coordinate (scn_grids_find, the source of a chain of
//     recorded plans) a dense table of rows, one int per site of the field and
//     valid where the mask is set, while the batch's fields are small enough;
//     else, on demand, an open-addressing hash table, linear probing, 16-byte
//     slots {int64 packed coordinate, int32 row}, load factor <= 1/2.
//
// Rule books (Regions.cu gridRules*) number output sites in first-touch order
// while the input map is iterated in ascending key.  An output site is first
// touched by the active input with the smallest key inside its window (its
// "owner"), and one input touches its outputs in ascending output key.  So
//   row(o) = #outputs owned by inputs that precede owner(o) in iteration order
//          + position of o among owner(o)'s outputs
//          + #background rows appended for earlier samples,
// which needs no sort: count owned outputs per input, scatter the counts to
// iteration order through the rank, prefix-sum, emit.
#include "scn_common.h"
#include <atomic>
#include "scn_scan_dev.h"

#include "scn_grids_dev.h"

__global__ void k_grid_build(GridView g, const int *sample,
                             const long long *key, const int *row, long long n,
                             long long *ekey, int *erow,
                             unsigned long long *badSites,
                             const int *bgIn, int *bgOut) {
  long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e < g.batch)
    bgOut[e] = bgIn[e];
  if (e >= n)
    return;
  const int b = sample[e];
  const long long k = key[e];
  if (b < 0 || b >= g.batch || k < 0 || k >= g.vol) {
    // outside the field: counted and reported by the next call that
    // synchronises; stored on the sample-0 origin so every list stays valid
    atomicAdd(badSites, 1ull);
    ekey[e] = 0;
    erow[e] = row[e];
    return;
  }
  long long p = (long long)b * g.vol + k;
  int r = row[e];
  if (g.dense)
    g.dense[p] = r;
  else if (g.table)
    hash_insert(g.table, g.shift, g.mask, p, r);
  atomicOr(&g.bits[p >> 6], 1ull << (p & 63));
  ekey[e] = p;
  erow[e] = r;
}

// pass 1: number of output sites owned by each input, stored at the input's
// position in iteration order
template <int D>
__global__ void k_plan_count(GridView in, Geom g, const long long *ekey,
                             Count nEntries, const long long *inMeta,
                             unsigned *cntByRank, unsigned long long *ownMask,
                             unsigned *rankOf) {
  long long e = xcd_contiguous_block((count_now(nEntries) + 255) / 256) * blockDim.x + threadIdx.x;
  if (e >= nEntries.bound)
    return;
  // an input whose own deferred plan outgrew its bounds holds no entries worth
  // reading (its emit pass wrote nothing): count nothing
  if (e >= count_now(nEntries) || (inMeta && inMeta[META_OVERFLOW])) {
    // past the real entries: the ranks of the real ones are below their
    // number, so these lanes zero exactly the rest of what the scan covers
    cntByRank[e] = 0;
    return;
  }
  long long p = ekey[e];
  int i[D];
  const int b = split_site<D>(p, g.volIn, g.nIn, i);
  unsigned n = 0;
  unsigned long long mask = 0;
  bool done = false;
  if constexpr (D >= 2) {
    // square windows of side 2 or 3 without a minimum: every mask word of the
    // site's neighbourhood is requested at once and the candidates are decided
    // in registers
    if (g.mode == MODE_SQ_NOMIN && (g.size == 2 || g.size == 3)) {
      int lo[D], hi[D];
      if (cand_box<D>(g, b, i, lo, hi)) {
        const long long sampleBase = (long long)b * g.volIn;
        auto none = [](const int *) {};
        mask = g.size == 2
                   ? owned_nomin<D, 2>(in.bits, sampleBase, i, lo, hi, g.nIn,
                                       g.stride, g.magicStride, none)
                   : owned_nomin<D, 3>(in.bits, sampleBase, i, lo, hi, g.nIn,
                                       g.stride, g.magicStride, none);
        n = (unsigned)__popcll(mask);
      }
      done = true;
    }
  }
  if (!done)
    for_each_owned<D>(in, g, b, i, [&](long long, int c) {
      ++n;
      mask |= 1ull << (c & 63);
    });
  unsigned r = rank_of(in, p);
  cntByRank[r] = n;
  if (ownMask) { // only when a box never has more than 64 candidates
    ownMask[e] = mask; // kept per entry, with the rank, so that the emit pass
    rankOf[e] = r;     // reads them without walking the mask again
  }
}

// where sample t starts and ends in iteration order: what the first round of
// plan_samples_body needs of the input grids (independent of the counts, so
// a caller that scans first can have these loads in flight meanwhile)
__device__ __forceinline__ void sample_ranks(const GridView &in, unsigned &rs,
                                             unsigned &re) {
  const int t = threadIdx.x;
  rs = re = 0;
  if (t < in.batch) {
    rs = rank_of(in, (long long)t * in.vol);
    re = rank_of(in, (long long)(t + 1) * in.vol);
  }
}

// per sample: does it need a background row, and how many were appended
// before it.  One block of SCAN1_THREADS lanes.
// OWNERS: `in` is the mask of the owning inputs with its prefix, so the rank
// of a position is already the number of outputs before it and base is unused.
template <bool OWNERS = false>
__device__ __forceinline__ void
plan_samples_body(const GridView &in, const unsigned *base, long long nEntries,
                  long long fullSize, int *outBg, int *bgBefore,
                  unsigned *sampleStart, volatile long long *scalars,
                  const long long *badSites, long long ticket,
                  long long *meta, const long long *inMeta, long long boundRows,
                  long long boundActive, int pinnedSlot, unsigned rs0,
                  unsigned re0) {
  __shared__ int waveSum[2 * SCAN1_WAVES];
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  int carry = 0, flip = 0; // the same in every lane
  for (int b0 = 0; b0 < in.batch; b0 += SCAN1_THREADS) {
    int b = b0 + t;
    int notFull = 0;
    unsigned re = 0;
    if (b < in.batch) {
      // (the first round's ranks were fetched by the caller, ahead of its scan)
      unsigned rs = b0 == 0 ? rs0 : rank_of(in, (long long)b * in.vol);
      re = b0 == 0 ? re0 : rank_of(in, (long long)(b + 1) * in.vol);
      sampleStart[b] = rs;
      if (!OWNERS) {
        rs = base[rs];
        re = base[re];
      }
      notFull = (long long)re - (long long)rs < fullSize;
    }
    // prefix of notFull over the lanes: shuffles inside a wavefront, the
    // wavefront totals through LDS (two sets of words: one barrier per round)
    int incl = notFull;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      int up = __shfl_up(incl, off, 64);
      if (lane >= off)
        incl += up;
    }
    int *ws = waveSum + flip * SCAN1_WAVES;
    if (lane == 63)
      ws[wave] = incl;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < SCAN1_WAVES; ++w) {
      const int x = ws[w];
      before += w < wave ? x : 0;
      total += x;
    }
    int excl = before + incl - notFull + carry;
    if (b < in.batch) {
      bgBefore[b] = excl;
      outBg[b] = notFull ? (int)re + excl : -1;
    }
    carry += total;
    flip ^= 1;
  }
  if (t == 0) {
    const long long nActive = // active output sites
        OWNERS ? (long long)rank_of(in, (long long)in.batch * in.vol) : (long long)base[nEntries];
    const long long nSites = nActive + carry; // nOutputSpatialSites
    const long long over = (inMeta && inMeta[META_OVERFLOW]) || nSites > boundRows ||
                           nActive > boundActive;
    meta[META_SITES] = nSites;
    meta[META_ACTIVE] = nActive;
    meta[META_OVERFLOW] = over;
    // scalars is host memory the device can write (the caller waits for the
    // stream and reads it, no copy kernel in between)
    if (pinnedSlot >= 0) { // deferred: read at settle time
      volatile long long *slot = scalars + 16 + 4 * pinnedSlot;
      slot[0] = nSites;
      slot[1] = nActive;
      slot[2] = over;
      scalars[15] = *badSites;
    } else {
      scalars[0] = nSites;
      scalars[1] = nActive;
      scalars[15] = *badSites; // sites scn_grids_build found outside the field
      __threadfence_system();
      scalars[14] = ticket; // last: the host spins on this word
    }
  }
}

template <bool OWNERS>
__global__ void __launch_bounds__(SCAN1_THREADS)
    k_plan_samples(GridView in, const unsigned *base, long long nEntries,
                   long long fullSize, int *outBg, int *bgBefore,
                   unsigned *sampleStart, long long *scalars,
                   const long long *badSites, long long ticket, long long *meta,
                   const long long *inMeta, long long boundRows,
                   long long boundActive, int pinnedSlot) {
  unsigned rs0, re0;
  sample_ranks(in, rs0, re0);
  plan_samples_body<OWNERS>(in, base, nEntries, fullSize, outBg, bgBefore, sampleStart,
                            scalars, badSites, ticket, meta, inMeta, boundRows,
                            boundActive, pinnedSlot, rs0, re0);
}

// small batches: prefix sum of the owned counts and the per-sample pass in
// one launch
__global__ void __launch_bounds__(SCAN1_THREADS)
    k_plan_scan_samples(GridView in, const unsigned *cnt, unsigned *base,
                        long long nEntries, long long fullSize, int *outBg,
                        int *bgBefore, unsigned *sampleStart,
                        long long *scalars, const long long *badSites,
                        long long ticket, long long *meta,
                        const long long *inMeta, long long boundRows,
                        long long boundActive, int pinnedSlot) {
  __shared__ uint32_t ldsScan[SCAN1_LDS_WORDS];
  unsigned rs0, re0;
  sample_ranks(in, rs0, re0);
  (void)block_scan_loop<false>(cnt, base, (size_t)nEntries, ldsScan);
  __syncthreads(); // the block's own writes to base[] are visible to it
  plan_samples_body(in, base, nEntries, fullSize, outBg, bgBefore, sampleStart,
                    scalars, badSites, ticket, meta, inMeta, boundRows,
                    boundActive, pinnedSlot, rs0, re0);
}

// pass 2: emit the owned outputs
template <int D>
__global__ void k_plan_emit(GridView in, GridView out, Geom g,
                            const long long *ekey, Count nEntries,
                            const long long *outMeta,
                            const unsigned *base, const int *bgBefore,
                            const int *outBg, long long *okey, int *orow,
                            long long *siteKey) {
  const long long live = count_now(nEntries) > in.batch ? count_now(nEntries) : in.batch;
  long long e = xcd_contiguous_block((live + 255) / 256) * blockDim.x + threadIdx.x;
  if (outMeta[META_OVERFLOW])
    return; // the bounds did not hold: nothing may be written
  if (e < in.batch) { // background rows
    int r = outBg[e];
    if (r >= 0)
      siteKey[r] = -1 - e;
  }
  if (e >= count_now(nEntries))
    return;
  long long p = ekey[e];
  int i[D];
  const int b = split_site<D>(p, g.volIn, g.nIn, i);
  unsigned idx = base[rank_of(in, p)];
  const int shiftRows = bgBefore[b];
  for_each_owned<D>(in, g, b, i, [&](long long outKey, int) {
    long long po = (long long)b * g.volOut + outKey;
    int row = (int)idx + shiftRows;
    int j[D];
    decode_key<D>(outKey, g.nOut, j);
    if (out.bits)
      atomicOr(&out.bits[po >> 6], 1ull << (po & 63));
    okey[idx] = po;
    orow[idx] = row;
    siteKey[row] = pack_row_site<D>(b, j);
    ++idx;
  });
}

// pass 2 when the ownership masks are available: one lane per (input,
// candidate), candidate index on blockIdx.y, so no lane walks a chain of
// dependent atomics.
template <int D>
__global__ void k_plan_emit_masked(GridView in, GridView out, Geom g,
                                   const long long *ekey, Count nEntries,
                                   const long long *outMeta,
                                   const unsigned *base,
                                   const unsigned long long *ownMask,
                                   const unsigned *rankOf,
                                   const int *bgBefore, const int *outBg,
                                   long long *okey, int *orow,
                                   long long *siteKey) {
  const long long live = count_now(nEntries) > in.batch ? count_now(nEntries) : in.batch;
  long long e = xcd_contiguous_block((live + 255) / 256) * blockDim.x + threadIdx.x;
  const int c = blockIdx.y;
  if (outMeta[META_OVERFLOW])
    return; // the bounds did not hold: nothing may be written
  if (c == 0 && e < in.batch) { // background rows
    int r = outBg[e];
    if (r >= 0)
      siteKey[r] = -1 - e;
  }
  if (e >= count_now(nEntries))
    return;
  // all three at once: one memory latency instead of two in a row
  const unsigned long long mask = ownMask[e];
  const long long p = ekey[e];
  const unsigned r = rankOf[e];
  if (!((mask >> c) & 1ull))
    return;
  int i[D], lo[D], hi[D], j[D];
  const int b = split_site<D>(p, g.volIn, g.nIn, i);
  (void)cand_box<D>(g, b, i, lo, hi);
  int rem = c;
#pragma unroll
  for (int a = D - 1; a >= 0; --a) {
    int ext = hi[a] - lo[a];
    j[a] = lo[a] + rem % ext;
    rem /= ext;
  }
  unsigned idx = base[r] + (unsigned)__popcll(mask & ((1ull << c) - 1ull));
  long long po = (long long)b * g.volOut + encode_key<D>(j, g.nOut);
  int row = (int)idx + bgBefore[b];
  if (out.bits)
    atomicOr(&out.bits[po >> 6], 1ull << (po & 63));
  okey[idx] = po;
  orow[idx] = row;
  siteKey[row] = pack_row_site<D>(b, j);
}

// position of the r-th (from 0) set bit of x, which has more than r
__device__ __forceinline__ int select_bit64(unsigned long long x, unsigned r) {
  int pos = 0;
  unsigned v = (unsigned)x;
  unsigned c = (unsigned)__popc(v);
  if (r >= c) {
    r -= c;
    v = (unsigned)(x >> 32);
    pos = 32;
  }
#pragma unroll
  for (int half = 16; half >= 2; half >>= 1) {
    c = (unsigned)__popc(v & ((1u << half) - 1u));
    if (r >= c) {
      r -= c;
      v >>= half;
      pos += half;
    }
  }
  return pos + (r >= (v & 1u) ? 1 : 0);
}

// The lanes of a wavefront hold counts; their exclusive prefix goes to
// before[0 .. 63] (LDS, this wavefront's part) and the total is returned.
__device__ __forceinline__ unsigned wave_deal_prefix(unsigned cnt, unsigned *before) {
  const int lane = threadIdx.x & 63;
  unsigned incl = cnt;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const unsigned up = __shfl_up(incl, off, 64);
    if (lane >= off)
      incl += up;
  }
  before[lane] = incl - cnt;
  return __shfl(incl, 63, 64);
}
// which lane's items hold item o of the wavefront (o < total): the last lane
// with at most o items before it
__device__ __forceinline__ int wave_deal_find(const unsigned *before, unsigned o) {
  int l = 0;
#pragma unroll
  for (int step = 32; step; step >>= 1)
    if (before[l + step] <= o)
      l += step;
  return l;
}

// The same for boxes of many candidates (3-D: 27) of which an input owns a
// few, where a lane per (input, candidate) would mostly read masks and leave,
// and a lane per input walking its own mask would leave most lanes idle.  A
// lane takes its input apart once (sample, box of candidates, where its
// outputs go) and leaves that in LDS; then the wavefront deals the set bits
// of its 64 ownership masks out to its lanes, one output each.
struct WalkItem {
  unsigned long long mask;
  int lo[3];
  unsigned ext[3], inv[3];
  unsigned idx;
  int b, shiftRows;
};
template <int D>
__global__ void __launch_bounds__(256)
    k_plan_emit_walk(GridView in, GridView out, Geom g,
                     const long long *ekey, Count nEntries,
                     const long long *outMeta, const unsigned *base,
                     const unsigned long long *ownMask,
                     const unsigned *rankOf, const int *bgBefore,
                     const int *outBg, long long *okey, int *orow,
                     long long *siteKey) {
  __shared__ WalkItem items[256];
  __shared__ unsigned before[256];
  const long long live = count_now(nEntries) > in.batch ? count_now(nEntries) : in.batch;
  long long e = xcd_contiguous_block((live + 255) / 256) * blockDim.x + threadIdx.x;
  if (outMeta[META_OVERFLOW])
    return; // the bounds did not hold: nothing may be written
  if (e < in.batch) { // background rows
    int r = outBg[e];
    if (r >= 0)
      siteKey[r] = -1 - e;
  }
  const int first = threadIdx.x & ~63;
  unsigned long long mask = 0;
  if (e < count_now(nEntries)) {
    // all three at once: one memory latency instead of two in a row
    mask = ownMask[e];
    const long long p = ekey[e];
    const unsigned r = rankOf[e];
    if (mask) {
      WalkItem &it = items[threadIdx.x];
      int i[D], lo[D], hi[D];
      const int b = split_site<D>(p, g.volIn, g.nIn, i);
      (void)cand_box<D>(g, b, i, lo, hi);
      // a box is at most 64 candidates, so its sides are small: x / ext by a
      // multiplication (exact for x < 64: the error of the factor stays below 1 / 64 ext)
#pragma unroll
      for (int a = 0; a < D; ++a) {
        it.lo[a] = lo[a];
        it.ext[a] = (unsigned)(hi[a] - lo[a]);
        it.inv[a] = 65536u / it.ext[a] + 1u;
      }
      it.mask = mask;
      it.idx = base[r];
      it.b = b;
      it.shiftRows = bgBefore[b];
    }
  }
  const unsigned total = wave_deal_prefix((unsigned)__popcll(mask), before + first);
  __syncthreads();
  for (unsigned o = threadIdx.x & 63; o < total; o += 64) {
    const int l = wave_deal_find(before + first, o);
    const WalkItem &it = items[first + l];
    const unsigned nth = o - before[first + l];
    // ascending candidate = ascending output key
    unsigned rem = (unsigned)select_bit64(it.mask, nth);
    int j[D];
#pragma unroll
    for (int a = D - 1; a >= 0; --a) {
      const unsigned up = (rem * it.inv[a]) >> 16;
      j[a] = it.lo[a] + (int)(rem - up * it.ext[a]);
      rem = up;
    }
    const unsigned idx = it.idx + nth;
    const long long po = (long long)it.b * g.volOut + encode_key<D>(j, g.nOut);
    const int row = (int)idx + it.shiftRows;
    if (out.bits)
      atomicOr(&out.bits[po >> 6], 1ull << (po & 63));
    okey[idx] = po;
    orow[idx] = row;
    siteKey[row] = pack_row_site<D>(it.b, j);
  }
}

// Square windows without a minimum: an output site is active when any site of
// its window is, so the output mask is the input mask OR-ed over the window
// and thinned by the stride -- whole words at a time, every word of the
// output mask written once (no atomics, no clearing).  One lane per output
// word; a word is cut into the pieces that lie in one row of the output field.
struct Bits128 {
  unsigned long long lo, hi;
};
// the L (at most 128) mask bits from position p on, and whatever follows them up to 128
__device__ __forceinline__ Bits128 get_bits128(const unsigned long long *bits,
                                               long long p, int L) {
  const long long w = p >> 6;
  const int sh = (int)(p & 63);
  Words2 ww; // one request; a third word only when the L bits reach into it
  __builtin_memcpy(&ww, bits + w, sizeof(ww));
  const unsigned long long a = ww.a, b = ww.b;
  unsigned long long c = 0;
  if (sh + L > 128)
    c = bits[w + 2];
  Bits128 r;
  r.lo = sh ? (a >> sh) | (b << (64 - sh)) : a;
  r.hi = sh ? (b >> sh) | (c << (64 - sh)) : b;
  return r;
}
// 96 mask bits from position p on, as three 32-bit words: one request at the
// 4-byte boundary below p and three funnel shifts
struct __attribute__((packed, aligned(4))) Dwords4 {
  unsigned d[4];
};
__device__ __forceinline__ void get_bits96(const unsigned long long *bits, long long p,
                                           unsigned &r0, unsigned &r1, unsigned &r2) {
  Dwords4 v;
  __builtin_memcpy(&v, reinterpret_cast<const unsigned *>(bits) + (p >> 5), sizeof(v));
  const unsigned s = (unsigned)p & 31u;
  r0 = __builtin_amdgcn_alignbit(v.d[1], v.d[0], s);
  r1 = __builtin_amdgcn_alignbit(v.d[2], v.d[1], s);
  r2 = __builtin_amdgcn_alignbit(v.d[3], v.d[2], s);
}
// 64 mask bits from position p on
__device__ __forceinline__ unsigned long long get_bits64(const unsigned long long *bits,
                                                         long long p) {
  const long long w = p >> 6;
  const int sh = (int)(p & 63);
  Words2 ww;
  __builtin_memcpy(&ww, bits + w, sizeof(ww));
  return sh ? (ww.a >> sh) | (ww.b << (64 - sh)) : ww.a;
}
// the even bits of x, packed
__device__ __forceinline__ unsigned long long even_bits(unsigned long long x) {
  x &= 0x5555555555555555ull;
  x = (x | (x >> 1)) & 0x3333333333333333ull;
  x = (x | (x >> 2)) & 0x0F0F0F0F0F0F0F0Full;
  x = (x | (x >> 4)) & 0x00FF00FF00FF00FFull;
  x = (x | (x >> 8)) & 0x0000FFFF0000FFFFull;
  x = (x | (x >> 16)) & 0x00000000FFFFFFFFull;
  return x;
}
// S: the window's side when it is 2 or 3 (the loops over a window's rows unroll and all its rows are requested at
// once), else 0 (read from g)
template <int D, int S>
__global__ void __launch_bounds__(256)
    k_mask_dilate(GridView in, Geom g, unsigned long long *outBits,
                  long long nWords, long long totalBits) {
  // (runs of blocks to one XCD: the rows and planes a word's windows reach into
  // are the ones its neighbours in the same L2 have just read)
  const long long w = xcd_contiguous_block((nWords + 255) / 256) * blockDim.x + threadIdx.x;
  if (w >= nWords)
    return;
  const int size = S ? S : g.size;
  constexpr int UN = S ? S : 1; // (no unrolling of loops whose length is not known here)
  unsigned long long res = 0;
  long long pos = 64 * w;
  const long long end = pos + 64 < totalBits ? pos + 64 : totalBits;
  // a piece reads (len - 1) stride + size input bits: at most 128
  const int lenMax = g.stride == 1 ? 64 : (128 - size) / g.stride + 1;
  int j[D];
  int b = split_site<D>(pos, g.volOut, g.nOut, j);
  while (pos < end) {
    long long len = g.nOut - j[D - 1];
    len = len < end - pos ? len : end - pos;
    len = len < lenMax ? len : lenMax;
    const int L = ((int)len - 1) * g.stride + size;
    const long long sampleBase = (long long)b * g.volIn;
    unsigned long long r;
    if (S && g.stride == 1) {
      // at most 66 bits a row: three 32-bit words, shifted as such (64-bit
      // shifts by a variable run at a quarter of the rate)
      unsigned x0 = 0, x1 = 0, x2 = 0;
      auto row = [&](long long p) {
        unsigned a0, a1, a2;
        get_bits96(in.bits, p, a0, a1, a2);
        x0 |= a0;
        x1 |= a1;
        x2 |= a2;
      };
      if constexpr (D == 1) {
        row(sampleBase + j[0]);
      } else if constexpr (D == 2) {
#pragma unroll
        for (int q0 = 0; q0 < S; ++q0)
          row(sampleBase + (long long)(j[0] + q0) * g.nIn + j[1]);
      } else {
#pragma unroll
        for (int q0 = 0; q0 < S; ++q0)
#pragma unroll
          for (int q1 = 0; q1 < S; ++q1)
            row(sampleBase + ((long long)(j[0] + q0) * g.nIn + (j[1] + q1)) * g.nIn + j[2]);
      }
      // bit t: any of the S sites from t on (t below 64)
      unsigned y0 = x0, y1 = x1;
#pragma unroll
      for (int q = 1; q < S; ++q) {
        y0 |= __builtin_amdgcn_alignbit(x1, x0, q);
        y1 |= __builtin_amdgcn_alignbit(x2, x1, q);
      }
      r = (unsigned long long)y0 | ((unsigned long long)y1 << 32);
    } else {
      unsigned long long lo = 0, hi = 0;
      if (D == 1) {
        const Bits128 x = get_bits128(in.bits, sampleBase + (long long)j[0] * g.stride, L);
        lo = x.lo;
        hi = x.hi;
      } else if (D == 2) {
#pragma unroll UN
        for (int q0 = 0; q0 < size; ++q0) {
          const Bits128 x = get_bits128(
              in.bits, sampleBase + (long long)(j[0] * g.stride + q0) * g.nIn +
                           (long long)j[1] * g.stride, L);
          lo |= x.lo;
          hi |= x.hi;
        }
      } else {
#pragma unroll UN
        for (int q0 = 0; q0 < size; ++q0)
#pragma unroll UN
          for (int q1 = 0; q1 < size; ++q1) {
            const Bits128 x = get_bits128(
                in.bits,
                sampleBase +
                    ((long long)(j[0] * g.stride + q0) * g.nIn +
                     (j[D > 1 ? 1 : 0] * g.stride + q1)) * g.nIn +
                    (long long)j[D - 1] * g.stride, L);
            lo |= x.lo;
            hi |= x.hi;
          }
      }
      // only the L bits of this piece's windows
      if (L < 64) {
        lo &= (1ull << L) - 1ull;
        hi = 0;
      } else if (L < 128) {
        hi &= L == 64 ? 0ull : (1ull << (L - 64)) - 1ull;
      }
      // bit t: any of the `size` sites from t on
      unsigned long long ylo = lo, yhi = hi;
#pragma unroll UN
      for (int q = 1; q < size; ++q) {
        lo = (lo >> 1) | (hi << 63);
        hi >>= 1;
        ylo |= lo;
        yhi |= hi;
      }
      if (g.stride == 1) {
        r = ylo;
      } else if (g.stride == 2) {
        r = even_bits(ylo) | (even_bits(yhi) << 32);
      } else {
        r = 0;
        for (int t = 0; t < (int)len; ++t) {
          const int at = t * g.stride;
          const unsigned long long bit = at < 64 ? (ylo >> at) : (yhi >> (at - 64));
          r |= (bit & 1ull) << t;
        }
      }
    }
    if (len < 64)
      r &= (1ull << len) - 1ull;
    res |= r << (pos - 64 * w);
    pos += len;
    // the next piece starts where this one ended: carry through the axes
    j[D - 1] += (int)len;
#pragma unroll
    for (int a = D - 1; a >= 0; --a)
      if (j[a] >= g.nOut) {
        j[a] = 0;
        if (a > 0)
          ++j[a - 1];
        else
          ++b;
      }
  }
  outBits[w] = res;
}

// Windows of side 2 that tile the field (stride 2, no minimum): every input
// lies in one window, a window's sites along the last axis are an even bit of
// the mask and its odd neighbour (fields have an even side, so rows start at
// even positions), and the owner of an output -- the first active site of its
// window in key order -- can be told from the input mask a word at a time.
// One lane per word of the input mask: a site owns its window's output when it
// is active, no earlier row of the window holds an active site in its pair of
// columns, and it is the first of its own pair.  The number of owners before
// a position (prefix of this mask) is the number of outputs before it in the
// reference's iteration order, so no per-input count is needed
// (Regions.cu:528-653 for the order).
template <int D>
__global__ void __launch_bounds__(256)
    k_tile2_owners(GridView in, Geom g, const long long *inMeta,
                   unsigned long long *ownBits, long long nWords,
                   long long totalBits) {
  const long long w = xcd_contiguous_block((nWords + 255) / 256) * blockDim.x + threadIdx.x;
  if (w >= nWords)
    return;
  unsigned long long res = 0;
  long long pos = 64 * w;
  const long long end = pos + 64 < totalBits ? pos + 64 : totalBits;
  // (an input whose own deferred plan outgrew its bounds counts for nothing)
  const unsigned long long X =
      pos < end && !(inMeta && inMeta[META_OVERFLOW]) ? in.bits[w] : 0ull;
  if (X) {
    const unsigned long long EVEN = 0x5555555555555555ull;
    int i[D];
    (void)split_site<D>(pos, g.volIn, g.nIn, i);
    const long long plane = (long long)g.nIn * g.nIn;
    while (pos < end) {
      long long len = g.nIn - i[D - 1];
      len = len < end - pos ? len : end - pos;
      const int at = (int)(pos - 64 * w); // even: rows and words start at even positions
      const unsigned long long m = (len >= 64 ? ~0ull : (1ull << len) - 1ull) << at;
      const unsigned long long x = X & m;
      if (x) {
        // the earlier rows of the windows, their bits under this piece's
        unsigned long long earlier = 0;
        if constexpr (D >= 2) {
          const int dy = i[D - 2] & 1;
          if (dy)
            earlier |= get_bits64(in.bits, pos - g.nIn);
          if constexpr (D == 3) {
            if (i[0] & 1) {
              earlier |= get_bits64(in.bits, pos - plane - (long long)dy * g.nIn);
              earlier |= get_bits64(in.bits, pos - plane + (long long)(1 - dy) * g.nIn);
            }
          }
        }
        earlier <<= at;
        const unsigned long long taken =
            earlier | ((earlier & EVEN) << 1) | ((earlier >> 1) & EVEN) | ((x & EVEN) << 1);
        res |= x & ~taken;
      }
      pos += len;
      i[D - 1] += (int)len;
#pragma unroll
      for (int a = D - 1; a > 0; --a)
        if (i[a] >= g.nIn) {
          i[a] = 0;
          ++i[a - 1];
        }
      if (i[0] >= g.nIn) // the next sample
        i[0] = 0;
    }
  }
  ownBits[w] = res;
}

// The outputs of such windows, in ascending position of their owners = the
// reference's order.  A wavefront takes 64 words of the owners' mask and deals
// their set bits out to its lanes one each (prefix of the words' counts, a
// search in it, the r-th set bit of the word found), so that the lanes write
// consecutive entries whatever the words hold.  The wavefront's first position
// is taken apart once; a site's coordinates follow from it by carries.
template <int D>
__global__ void __launch_bounds__(256)
    k_tile2_emit(GridView in, Geom g, const unsigned long long *ownBits,
                 const unsigned *ownPrefix, long long nWords,
                 const long long *outMeta, const int *bgBefore,
                 const int *outBg, long long *okey, int *orow,
                 long long *siteKey) {
  __shared__ unsigned long long sWord[256];
  __shared__ unsigned sBefore[256];
  const long long live = nWords > in.batch ? nWords : in.batch;
  const long long w = xcd_contiguous_block((live + 255) / 256) * blockDim.x + threadIdx.x;
  if (outMeta[META_OVERFLOW])
    return; // the bounds did not hold: nothing may be written
  if (w < in.batch) { // background rows
    const int r = outBg[w];
    if (r >= 0)
      siteKey[r] = -1 - w;
  }
  const int lane = threadIdx.x & 63, first = threadIdx.x & ~63;
  const unsigned long long word = w < nWords ? ownBits[w] : 0ull;
  const unsigned total = wave_deal_prefix((unsigned)__popcll(word), sBefore + first);
  sWord[threadIdx.x] = word;
  __syncthreads();
  if (total == 0)
    return;
  const long long w0 = w - lane; // the wavefront's first word, which exists as total > 0
  const unsigned idx0 = ownPrefix[w0];
  int i0[D];
  const int b0 = split_site<D>(64 * w0, g.volIn, g.nIn, i0);
  for (unsigned o = lane; o < total; o += 64) {
    const int l = wave_deal_find(sBefore + first, o);
    unsigned carry =
        64u * (unsigned)l + (unsigned)select_bit64(sWord[first + l], o - sBefore[first + l]);
    int j[D];
#pragma unroll
    for (int a = D - 1; a >= 0; --a) {
      unsigned t = (unsigned)i0[a] + carry;
      carry = 0;
      if (t >= (unsigned)g.nIn) {
        carry = t / (unsigned)g.nIn;
        t -= carry * (unsigned)g.nIn;
      }
      j[a] = (int)(t >> 1);
    }
    const int b = b0 + (int)carry;
    const unsigned idx = idx0 + o;
    const int row = (int)idx + bgBefore[b];
    okey[idx] = (long long)b * g.volOut + encode_key<D>(j, g.nOut);
    orow[idx] = row;
    siteKey[row] = pack_row_site<D>(b, j);
  }
}

// clears a hash table (all-ones = empty slots) and an occupancy mask at once
__global__ void k_clear_grid(uint4 *slots, size_t nSlots,
                             unsigned long long *bits, size_t nWords) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t k = i; k < nSlots; k += step)
    slots[k] = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
  for (size_t k = i; k < nWords; k += step)
    bits[k] = 0ull;
}

// inverse of RegularTriangularRegions::ord (Regions.cu:810-826)
__global__ void k_tri_table(int size, int d, int *invOrd) {
  if (blockIdx.x != 0 || threadIdx.x != 0)
    return;
  int cube = 1;
  for (int a = 0; a < d; ++a)
    cube *= size;
  int S = 0;
  for (int i = 0; i < cube; ++i) {
    int j = i, J = 0;
    while (j > 0) {
      J += j % size;
      j /= size;
    }
    if (J < size)
      invOrd[S++] = i;
  }
}

// The rank prefix of the output mask (which the next rule book needs of its
// input) depends on the emit pass only, as the rules do: with SCAN, workgroup 0
// of the fill launch computes it while the others fill, instead of a launch
// of its own later (masks of up to SCAN1_MAX_ELEMS words).
struct RankScan {
  const unsigned long long *bits;
  unsigned *prefix;
  size_t n;
};

// row of the active site at packed position p
__device__ __forceinline__ int row_at(const GridView &g, long long p) {
  return g.rankRow[rank_of(g, p)];
}

// one thread per rule: rules[row * width + q]
template <int D, bool SCAN>
__global__ void __launch_bounds__(256)
    k_rules_fill(GridView in, Geom g, const long long *siteKey, Count nSites,
                 const long long *outMeta, const int *invOrd, int *rules,
                 RankScan rs) {
  __shared__ uint32_t ldsScan[SCAN1_LDS_WORDS];
  long long blk = blockIdx.x;
  if (SCAN) {
    if (blk == 0) {
      (void)block_scan_loop<true>(rs.bits, rs.prefix, rs.n, ldsScan);
      return;
    }
    blk -= 1;
  }
  long long idx = blk * blockDim.x + threadIdx.x;
  if (outMeta[META_OVERFLOW])
    return;
  long long total = count_now(nSites) * g.width;
  if (idx >= total)
    return;
  long long r = idx / g.width;
  int q = (int)(idx - r * g.width);
  long long sk = siteKey[r];
  if (sk < 0) { // all-background row (Regions.cu:647-652)
    rules[idx] = in.bg[-1 - sk];
    return;
  }
  int j[D], c[D];
  const int b = unpack_row_site<D>(sk, j);
  int cubeOff = invOrd ? invOrd[q] : q;
  if (g.mode == MODE_SQ_FMP) {
    // offsets past a region's extent keep the -1 the reference's rule rows
    // start from (Regions.cu:177-178)
    bool outside = false;
#pragma unroll
    for (int a = D - 1; a >= 0; --a) {
      const int o = cubeOff % g.size;
      cubeOff /= g.size;
      const int l = fmp_inputL(g, b, a, j[a]);
      outside |= o >= fmp_inputR(g, b, a, j[a]) - l;
      c[a] = l + o;
    }
    if (outside) {
      rules[idx] = -1;
      return;
    }
  } else {
#pragma unroll
    for (int a = D - 1; a >= 0; --a) {
      c[a] = j[a] * g.stride + cubeOff % g.size;
      cubeOff /= g.size;
    }
  }
  long long p = (long long)b * g.volIn + encode_key<D>(c, g.nIn);
  int val;
  if ((in.bits[p >> 6] >> (p & 63)) & 1ull)
    val = row_at(in, p);
  else
    val = in.bg[b];
  rules[idx] = val;
}

// Square windows.  A workgroup takes `rowsPerBlock` consecutive rule rows -- a
// contiguous piece of the rule book -- one lane per row.  A lane decodes its
// output site once and walks the runs of `size` entries along the innermost
// axis: the input sites of a run are neighbours in the mask and in rank, so a
// run costs one mask word (two when it straddles), one prefix word and
// consecutive words of the rows by rank; and since consecutive rows are mostly
// neighbouring sites, the lanes of a wavefront read the same few lines in
// every step.  All runs of a row are in flight at once when the side is 2 or
// 3, else three at a time (all loads unconditional, results selected
// afterwards).  The rows are collected in LDS
// (odd pitch: no bank conflicts) and leave as whole 16-byte stores, lane after
// lane.  S: the window's side when it is 2 or 3, else 0 (read from g).
#define FILL_LDS_INTS 8192
struct __attribute__((packed, aligned(4))) Rows4 {
  int r[4];
};
template <int D, bool SCAN, int S>
__global__ void __launch_bounds__(256)
    k_rules_fill_runs(GridView in, Geom g, const long long *siteKey,
                      Count nSites, const long long *outMeta, int *rules,
                      RankScan rs, int rowsPerBlock, int pitch,
                      unsigned magicWidth, unsigned magicSize) {
  __shared__ uint32_t ldsScan[SCAN1_LDS_WORDS];
  // rowsPerBlock rows of `pitch` words (the launch says how many bytes: what the
  // rows need and no more, so that short rows leave room for more workgroups)
  extern __shared__ __attribute__((aligned(16))) int staged[];
  long long blk = blockIdx.x;
  if (SCAN) {
    if (blk == 0) {
      (void)block_scan_loop<true>(rs.bits, rs.prefix, rs.n, ldsScan);
      return;
    }
    blk -= 1;
  } else {
    blk = xcd_contiguous_block((count_now(nSites) + rowsPerBlock - 1) / rowsPerBlock);
  }
  if (outMeta[META_OVERFLOW])
    return;
  // runs in flight per lane: a whole row when the side is known
  constexpr int U = S == 0 ? 3 : (D == 1 ? 1 : (D == 2 ? S : S * S));
  const int t = threadIdx.x;
  const long long row0 = blk * rowsPerBlock;
  const long long left = count_now(nSites) - row0;
  if (left <= 0)
    return;
  const int nRows = left < rowsPerBlock ? (int)left : rowsPerBlock;
  const int size = S ? S : g.size;
  const int runsPerRow = g.width / size;
  if (t < nRows) {
    const long long sk = siteKey[row0 + t];
    int *dst = staged + t * pitch;
    if (sk < 0) { // all-background row (Regions.cu:647-652)
      const int v = in.bg[-1 - sk];
      for (int q = 0; q < g.width; ++q)
        dst[q] = v;
    } else {
      int j[D];
      const int b = unpack_row_site<D>(sk, j);
      const int bgRow = in.bg[b];
      // packed position of the window's origin
      long long origin = 0;
#pragma unroll
      for (int a = 0; a < D; ++a)
        origin = origin * g.nIn + (long long)j[a] * g.stride;
      origin += (long long)b * g.volIn;
      const long long plane = D == 3 ? (long long)g.nIn * g.nIn : 0;
      for (int k0 = 0; k0 < runsPerRow; k0 += U) {
        unsigned long long w0[U], w1[U];
        unsigned pre[U];
        int sh[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int k = k0 + u < runsPerRow ? k0 + u : runsPerRow - 1;
          long long p0 = origin;
          if (D == 2) {
            p0 += (long long)k * g.nIn;
          } else if (D == 3) {
            const int hiRun = (int)div_magic((unsigned)k, (unsigned)size, magicSize);
            p0 += hiRun * plane + (long long)(k - hiRun * size) * g.nIn;
          }
          const long long w = p0 >> 6;
          sh[u] = (int)(p0 & 63);
          // both words in one request (the mask has spare words at its end)
          Words2 ww;
          __builtin_memcpy(&ww, in.bits + w, sizeof(ww));
          w0[u] = ww.a;
          w1[u] = ww.b;
          pre[u] = in.prefix[w];
        }
        if (S) {
          Rows4 val[U];
          unsigned present[U];
#pragma unroll
          for (int u = 0; u < U; ++u) {
            // in 32-bit pieces: 64-bit shifts by a variable run at a quarter of the rate
            const unsigned d0 = (unsigned)w0[u], d1 = (unsigned)(w0[u] >> 32), d2 = (unsigned)w1[u];
            const bool upper = sh[u] >= 32;
            const unsigned s = (unsigned)sh[u] & 31u;
            present[u] = __builtin_amdgcn_alignbit(upper ? d2 : d1, upper ? d1 : d0, s) & ((1u << S) - 1u);
            const unsigned below = (1u << s) - 1u; // of the 32-bit word the run starts in
            const unsigned rank0 = pre[u] + (upper ? (unsigned)__popc(d0) + (unsigned)__popc(d1 & below)
                                                   : (unsigned)__popc(d0 & below));
            // the rows of the run's active sites are consecutive words: one
            // request (the array has spare words at its end)
            __builtin_memcpy(&val[u], in.rankRow + (present[u] ? rank0 : 0u), sizeof(Rows4));
          }
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (k0 + u < runsPerRow) {
#pragma unroll
              for (int q = 0; q < S; ++q) {
                const int at = __popc(present[u] & ((1u << q) - 1u));
                const int v = at == 0 ? val[u].r[0] : (at == 1 ? val[u].r[1] : val[u].r[2]);
                dst[(k0 + u) * S + q] = (present[u] >> q) & 1u ? v : bgRow;
              }
            }
        } else {
#pragma unroll
          for (int u = 0; u < U; ++u) {
            if (k0 + u >= runsPerRow)
              break;
            unsigned long long lo = w0[u] >> sh[u];
            if (sh[u])
              lo |= w1[u] << (64 - sh[u]);
            const unsigned present =
                (unsigned)lo & (size >= 32 ? 0xFFFFFFFFu : ((1u << size) - 1u));
            const unsigned rank0 =
                pre[u] + (unsigned)__popcll(sh[u] ? (w0[u] & ((1ull << sh[u]) - 1ull)) : 0ull);
            for (int q = 0; q < size; ++q)
              dst[(k0 + u) * size + q] =
                  (present >> q) & 1u
                      ? in.rankRow[rank0 + __popc(present & ((1u << q) - 1u))]
                      : bgRow;
          }
        }
      }
    }
  }
  __syncthreads();
  const unsigned total = (unsigned)nRows * (unsigned)g.width;
  int *out = rules + row0 * g.width;
  if (pitch == g.width && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    typedef int v4i __attribute__((ext_vector_type(4)));
    const v4i *src = reinterpret_cast<const v4i *>(staged);
    // (written once, read by a later kernel: streamed past the caches)
    for (unsigned v = t; 4 * v + 4 <= total; v += 256)
      __builtin_nontemporal_store(src[v], reinterpret_cast<v4i *>(out) + v);
    const unsigned tail = total & ~3u;
    if (t < (int)(total - tail))
      out[tail + t] = staged[tail + t];
  } else {
    for (unsigned v = t; v < total; v += 256) {
      const unsigned r = div_magic(v, (unsigned)g.width, magicWidth);
      out[v] = staged[r * pitch + (v - r * g.width)];
    }
  }
}

// terminal pooling: sample sizes and their maximum.  One block.
__global__ void __launch_bounds__(SCAN1_THREADS) k_terminal_plan(GridView in, unsigned *sampleStart,
                                volatile long long *scalars,
                                long long ticket, long long *meta,
                                const long long *inMeta, long long boundWidth,
                                int pinnedSlot) {
  __shared__ long long lds[SCAN1_THREADS];
  const int t = threadIdx.x;
  long long mx = 1; // TerminalPoolingLayer.cu:90
  for (int b = t; b < in.batch; b += SCAN1_THREADS) {
    unsigned rs = rank_of(in, (long long)b * in.vol);
    unsigned re = rank_of(in, (long long)(b + 1) * in.vol);
    sampleStart[b] = rs;
    if (b == in.batch - 1)
      sampleStart[in.batch] = re;
    long long c = (long long)re - rs;
    mx = c > mx ? c : mx;
  }
  lds[t] = mx;
  __syncthreads();
  for (int off = SCAN1_THREADS / 2; off > 0; off >>= 1) {
    if (t < off && lds[t + off] > lds[t])
      lds[t] = lds[t + off];
    __syncthreads();
  }
  if (t == 0) {
    const long long over = (inMeta && inMeta[META_OVERFLOW]) || lds[0] > boundWidth;
    meta[META_SITES] = in.batch;
    meta[META_ACTIVE] = in.batch;
    meta[META_OVERFLOW] = over;
    meta[META_WIDTH] = lds[0];
    if (pinnedSlot >= 0) { // deferred: read at settle time
      volatile long long *slot = scalars + 16 + 4 * pinnedSlot;
      slot[0] = in.batch;
      slot[1] = in.batch;
      slot[2] = over;
      slot[3] = lds[0];
    } else {
      scalars[0] = lds[0];
      __threadfence_system();
      scalars[14] = ticket;
    }
  }
}

// out grid of the terminal layer: key 0 of sample b -> row b
__global__ void k_terminal_out(GridView out, long long *okey, int *orow,
                               int *outBg) {
  int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= out.batch)
    return;
  long long p = (long long)b * out.vol;
  atomicOr(&out.bits[p >> 6], 1ull << (p & 63));
  okey[b] = p;
  orow[b] = b;
  outBg[b] = -1;
}

__global__ void k_terminal_init(GridView in, const unsigned *sampleStart,
                                Count width, const long long *outMeta,
                                int *rules) {
  long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (outMeta[META_OVERFLOW])
    return;
  const long long S = count_now(width);
  if (idx >= (long long)in.batch * S)
    return;
  int b = (int)(idx / S);
  long long s = idx - (long long)b * S;
  int v = -1;
  // a sample without active sites pools its background row
  // (TerminalPoolingLayer.cu:12-13)
  if (s == 0 && sampleStart[b + 1] == sampleStart[b])
    v = in.bg[b];
  rules[idx] = v;
}

__global__ void k_terminal_scatter(GridView in, const long long *ekey,
                                   const int *erow, Count nEntries,
                                   const unsigned *sampleStart, Count width,
                                   const long long *outMeta, int *rules) {
  long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (outMeta[META_OVERFLOW] || e >= count_now(nEntries))
    return;
  const long long S = count_now(width);
  long long p = ekey[e];
  int b = (int)(p / in.vol);
  unsigned r = rank_of(in, p) - sampleStart[b];
  rules[(long long)b * S + r] = erow[e];
}

__global__ void k_download(GridView g, const long long *ekey, const int *erow,
                           long long n, int *sample, long long *key, int *row) {
  long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n)
    return;
  long long p = ekey[e];
  unsigned r = rank_of(g, p);
  int b = (int)(p / g.vol);
  sample[r] = b;
  key[r] = p - (long long)b * g.vol;
  row[r] = erow[e];
}

__global__ void k_find(GridView g, const int *sample, const long long *key,
                       long long n, int *row) {
  long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n)
    return;
  long long k = key[e];
  int b = sample[e];
  int r = -1;
  if (b >= 0 && b < g.batch && k >= 0 && k < g.vol)
    r = grid_row(g, (long long)b * g.vol + k);
  row[e] = r;
}

// ------------------------------------------------------------------ host

static bool dense_rows(const scn_grids *g) {
  return (long long)(g->batch > 0 ? g->batch : 1) * g->vol <= SCN_DENSE_MAX_SITES;
}

GridView view_of(const scn_grids *g) {
  GridView v;
  v.table = g->tableValid && !dense_rows(g) ? g->table.p : nullptr;
  v.dense = g->tableValid && dense_rows(g) ? g->dense.p : nullptr;
  v.shift = 64 - g->log2cap;
  v.mask = (1u << g->log2cap) - 1u;
  v.bits = g->bits.p;
  v.prefix = g->prefix.p;
  v.rankRow = g->rankRow.p;
  v.bg = g->bg.p;
  v.vol = g->vol;
  v.n = g->n;
  v.d = g->d;
  v.batch = g->batch;
  return v;
}

static long long ipow_ll(long long b, int e) {
  long long r = 1;
  for (int i = 0; i < e; ++i)
    r *= b;
  return r;
}

// (re)shape a grids object for `batch` samples of an n^d field holding up to
// nActive sites; clears the mask, and the hash table when the caller is about
// to fill it (withTable)
static int grids_prepare(scn_ctx *ctx, scn_grids *g, int batch, int d, int n,
                         long long nActive, bool withTable = false) {
  SCN_REQUIRE(batch >= 0 && d >= 1 && d <= 3 && n >= 1, SCN_ERR_ARG,
              "grids: batch %d dimension %d spatialSize %d (dimension must be 1..3)",
              batch, d, n);
  long long vol = ipow_ll(n, d);
  SCN_REQUIRE((double)vol * (double)(batch > 0 ? batch : 1) < 6.0e10,
              SCN_ERR_CAPACITY,
              "grids: %d samples of %lld sites exceed the occupancy-mask limit",
              batch, vol);
  // (the rows of a rule-book plan carry their sample above 40 bits of coordinates)
  SCN_REQUIRE(batch < (1 << 22) && (d == 1 || n < (d == 3 ? (1 << 13) : (1 << 20))),
              SCN_ERR_CAPACITY, "grids: %d samples of side %d", batch, n);
  g->batch = batch;
  g->d = d;
  g->n = n;
  g->vol = vol;
  g->nActive = nActive;
  g->rankValid = false;
  g->rankRowValid = false;
  g->tableValid = withTable;
  g->indexValid = true;
  g->chained = false;
  g->planKind = PLAN_NONE;
  g->planIn = nullptr;
  g->pending = false;
  unsigned lg = 6;
  while ((1ll << lg) < 2 * nActive)
    ++lg;
  SCN_REQUIRE(lg <= 31, SCN_ERR_CAPACITY, "grids: %lld active sites", nActive);
  g->log2cap = lg;
  const size_t cap = (size_t)1 << lg;
  g->nWords = (size_t)(((long long)batch * vol + 63) / 64);
  const void *hadTable = g->table.p, *hadBits = g->bits.p;
  const bool dense = dense_rows(g);
  if (withTable && dense)
    SCN_TRY(g->dense.reserve((size_t)((long long)batch * vol) + 1));
  else if (withTable)
    SCN_TRY(g->table.reserve(cap));
  SCN_TRY(g->bits.reserve(g->nWords + 8)); // the scan reads whole 32-byte groups
  if (g->table.p != hadTable)
    g->cleanSlots = 0; // fresh memory
  if (g->bits.p != hadBits)
    g->cleanWords = 0;
  SCN_TRY(g->prefix.reserve(g->nWords + 2));
  SCN_TRY(g->ekey.reserve((size_t)nActive + 1));
  SCN_TRY(g->erow.reserve((size_t)nActive + 1));
  SCN_TRY(g->bg.reserve((size_t)batch + 1));
  // (a dense row table needs no clearing: it is read where the mask is set)
  const size_t clearSlots = withTable && !dense && cap > g->cleanSlots ? cap : 0;
  const size_t clearWords = g->nWords + 2 > g->cleanWords ? g->nWords + 2 : 0;
  if (withTable && !dense)
    g->cleanSlots = 0; // about to be written
  g->cleanWords = 0;
  if (clearSlots || clearWords) {
    size_t most = clearSlots > clearWords ? clearSlots : clearWords;
    size_t blocks = (most + 255) / 256;
    if (blocks > 16384)
      blocks = 16384;
    hipLaunchKernelGGL(k_clear_grid, dim3((unsigned)blocks), dim3(256), 0,
                       ctx->stream, (uint4 *)g->table.p, clearSlots, g->bits.p,
                       clearWords);
    SCN_HIP_CHECK(hipGetLastError());
  }
  return SCN_OK;
}

// One launch empties the tables and masks of up to CLEAR_MANY grids objects.
#define CLEAR_MANY 24
struct ClearList {
  uint4 *slots[CLEAR_MANY];
  unsigned long long *bits[CLEAR_MANY];
  size_t nSlots[CLEAR_MANY], nWords[CLEAR_MANY];
};
__global__ void k_clear_many(ClearList l) {
  const int g = blockIdx.y;
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  uint4 *slots = l.slots[g];
  for (size_t k = i; k < l.nSlots[g]; k += step)
    slots[k] = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
  unsigned long long *bits = l.bits[g];
  for (size_t k = i; k < l.nWords[g]; k += step)
    bits[k] = 0ull;
}

extern "C" int scn_grids_clear_many(scn_ctx *ctx, scn_grids **grids, int n) {
  SCN_REQUIRE(ctx && (grids || n == 0) && n >= 0, SCN_ERR_ARG,
              "scn_grids_clear_many: bad argument");
  SCN_TRY(scn_chain_flush(ctx));
  for (int first = 0; first < n; first += CLEAR_MANY) {
    ClearList l;
    int m = 0;
    size_t most = 0;
    for (int i = first; i < n && i < first + CLEAR_MANY; ++i) {
      scn_grids *g = grids[i];
      if (!g || (!g->table.p && !g->bits.p))
        continue;
      // nothing to do for grids whose table and mask are not in use (a chain
      // of recorded plans fills the entry list only) or are empty already
      if (!g->indexValid || ((!g->table.p || g->cleanSlots >= g->table.cap) &&
                             (!g->bits.p || g->cleanWords >= g->bits.cap)))
        continue;
      l.slots[m] = (uint4 *)g->table.p;
      l.nSlots[m] = g->table.p ? g->table.cap : 0;
      l.bits[m] = g->bits.p;
      l.nWords[m] = g->bits.p ? g->bits.cap : 0;
      most = l.nSlots[m] > most ? l.nSlots[m] : most;
      most = l.nWords[m] > most ? l.nWords[m] : most;
      g->cleanSlots = l.nSlots[m];
      g->cleanWords = l.nWords[m];
      g->rankValid = false;
      g->rankRowValid = false;
      g->tableValid = false;
      g->nActive = 0; // (the entry list goes with the mask: an emptied object holds no sites)
      ++m;
    }
    if (m == 0)
      continue;
    size_t blocks = (most + 1023) / 1024; // four elements per lane
    blocks = blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks);
    hipLaunchKernelGGL(k_clear_many, dim3((unsigned)blocks, (unsigned)m),
                       dim3(256), 0, ctx->stream, l);
    SCN_HIP_CHECK(hipGetLastError());
  }
  return SCN_OK;
}

// mask of grids that only hold their entry list
__global__ void k_grid_index(GridView g, const long long *ekey, const int *erow,
                             Count n, const long long *meta) {
  long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n.bound || (meta && meta[META_OVERFLOW]) || e >= count_now(n))
    return;
  const long long p = ekey[e];
  atomicOr(&g.bits[p >> 6], 1ull << (p & 63));
}
// the rows by rank from the entry list
__global__ void k_rank_rows(GridView g, const long long *ekey, const int *erow,
                            Count n, const long long *meta, int *rankRow) {
  long long e = xcd_contiguous_block((count_now(n) + 255) / 256) * blockDim.x + threadIdx.x;
  if (e >= n.bound || (meta && meta[META_OVERFLOW]) || e >= count_now(n))
    return;
  rankRow[rank_of(g, ekey[e])] = erow[e];
}
// the look-up table (dense rows or hash) from the entry list
__global__ void k_grid_table(GridView g, const long long *ekey, const int *erow,
                             Count n, const long long *meta) {
  long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n.bound || (meta && meta[META_OVERFLOW]) || e >= count_now(n))
    return;
  if (g.dense)
    g.dense[ekey[e]] = erow[e];
  else
    hash_insert(g.table, g.shift, g.mask, ekey[e], erow[e]);
}
static Count count_active(const scn_grids *g);
// the occupancy mask of grids that only hold their entry list
static int ensure_index(scn_ctx *ctx, scn_grids *g) {
  if (g->indexValid)
    return SCN_OK;
  SCN_TRY(scn_chain_flush(ctx));
  // (grids_prepare forgets the plan and the deferral: they are put back)
  const int planKind = g->planKind, nSites = g->nSites, pinnedSlot = g->pinnedSlot;
  const scn_grids *planIn = g->planIn;
  const bool pending = g->pending, chained = g->chained;
  const long long nActive = g->nActive;
  SCN_TRY(grids_prepare(ctx, g, g->batch, g->d, g->n, nActive));
  g->planKind = planKind;
  g->planIn = planIn;
  g->nSites = nSites;
  g->pending = pending;
  g->pinnedSlot = pinnedSlot;
  g->chained = chained;
  if (nActive > 0) {
    hipLaunchKernelGGL(k_grid_index, dim3(scn_ceil_div(nActive, 256)), dim3(256),
                       0, ctx->stream, view_of(g), g->ekey.p, g->erow.p,
                       count_active(g), pending ? g->meta.p : nullptr);
    SCN_HIP_CHECK(hipGetLastError());
  }
  return SCN_OK;
}

// mask, rank prefix and rows by rank: what a rule book needs of its input
static int ensure_rank(scn_ctx *ctx, scn_grids *g) {
  SCN_TRY(ensure_index(ctx, g));
  if (!g->rankValid) {
    SCN_TRY(g->scanTmp.reserve(scn_scan_tmp_elems(g->nWords + 1)));
    // one word past the mask so that the rank of the end position is defined
    SCN_TRY(scn_scan_exclusive_popc64(ctx->stream,
                                      (const uint64_t *)g->bits.p, g->prefix.p,
                                      g->nWords + 1, g->scanTmp.p));
    g->rankValid = true;
  }
  if (!g->rankRowValid) {
    SCN_TRY(g->rankRow.reserve((size_t)g->nActive + 4));
    if (g->nActive > 0) {
      hipLaunchKernelGGL(k_rank_rows, dim3(xcd_grid(scn_ceil_div(g->nActive, 256))),
                         dim3(256), 0, ctx->stream, view_of(g), g->ekey.p,
                         g->erow.p, count_active(g),
                         g->pending ? g->meta.p : nullptr, g->rankRow.p);
      SCN_HIP_CHECK(hipGetLastError());
    }
    g->rankRowValid = true;
  }
  return SCN_OK;
}

// the table for look-ups by coordinate
int scn_grids_ensure_table(scn_ctx *ctx, scn_grids *g) {
  SCN_TRY(ensure_index(ctx, g));
  if (g->tableValid)
    return SCN_OK;
  if (dense_rows(g)) {
    SCN_TRY(g->dense.reserve((size_t)((long long)g->batch * g->vol) + 1));
  } else {
    const size_t cap = (size_t)1 << g->log2cap;
    const void *had = g->table.p;
    SCN_TRY(g->table.reserve(cap));
    if (g->table.p != had)
      g->cleanSlots = 0;
    if (g->cleanSlots < cap) {
      size_t blocks = (cap + 255) / 256;
      if (blocks > 16384)
        blocks = 16384;
      hipLaunchKernelGGL(k_clear_grid, dim3((unsigned)blocks), dim3(256), 0,
                         ctx->stream, (uint4 *)g->table.p, cap,
                         (unsigned long long *)nullptr, (size_t)0);
      SCN_HIP_CHECK(hipGetLastError());
    }
    g->cleanSlots = 0;
  }
  g->tableValid = true; // (view_of hands the table out from here on)
  if (g->nActive > 0) {
    hipLaunchKernelGGL(k_grid_table, dim3(scn_ceil_div(g->nActive, 256)),
                       dim3(256), 0, ctx->stream, view_of(g), g->ekey.p,
                       g->erow.p, count_active(g),
                       g->pending ? g->meta.p : nullptr);
    SCN_HIP_CHECK(hipGetLastError());
  }
  return SCN_OK;
}

// Waits for the kernel that wrote the counts into the mapped host words.  The
// kernel writes its ticket last; watching that word costs a microsecond or two
// where a stream synchronisation costs ten, and this wait is on the critical
// path of every layer.  A kernel that does not deliver falls back to the
// stream (which also surfaces its error).
static int read_scalars(scn_ctx *ctx, long long ticket) {
  volatile int64_t *word = ctx->h_pinned + 14;
  bool seen = false;
  for (int spin = 0; spin < 400000; ++spin) {
    if (*word == ticket) {
      seen = true;
      break;
    }
    __builtin_ia32_pause();
  }
  std::atomic_thread_fence(std::memory_order_acquire);
  if (!seen) {
    SCN_HIP_CHECK(hipStreamSynchronize(ctx->stream));
    SCN_REQUIRE(*word == ticket, SCN_ERR_STATE,
                "rules: the planning kernel did not deliver its counts");
  }
  if (ctx->h_pinned[15] != 0) {
    long long bad = ctx->h_pinned[15];
    ctx->h_pinned[15] = 0;
    SCN_TRY(scn_fill32(ctx, ctx->d_scalars + 15, 0u, 2));
    SCN_REQUIRE(false, SCN_ERR_ARG,
                "scn_grids_build was given %lld sites outside the field", bad);
  }
  return SCN_OK;
}

static Count count_active(const scn_grids *g) {
  Count c;
  c.bound = g->nActive;
  c.live = g->pending ? g->meta.p + META_ACTIVE : nullptr;
  return c;
}
static Count count_sites(const scn_grids *g) {
  Count c;
  c.bound = g->nSites;
  c.live = g->pending ? g->meta.p + META_SITES : nullptr;
  return c;
}
static Count count_width(const scn_grids *g) {
  Count c;
  c.bound = g->termS;
  c.live = g->pending ? g->meta.p + META_WIDTH : nullptr;
  return c;
}
long long grow_bound(long long seen, long long slack, long long cap) {
  long long b = seen + seen / 4 + slack;
  return b < cap ? b : cap;
}

// Deferred counts.  With deferral on, a plan whose output object has held a
// plan before does not wait for its counts: it sizes everything by bounds
// derived from the largest counts the object has seen, its kernels read the
// real counts from device memory, and scn_rules_settle() collects them all
// with one synchronisation.
extern "C" int scn_ctx_defer_counts(scn_ctx *ctx, int on) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_ctx_defer_counts: null context");
  ctx->deferCounts = on != 0;
  return SCN_OK;
}
extern "C" int scn_rules_settle(scn_ctx *ctx) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_rules_settle: null context");
  SCN_TRY(scn_chain_flush(ctx));
  if (ctx->pendingGrids.empty())
    return SCN_OK;
  SCN_HIP_CHECK(hipStreamSynchronize(ctx->stream));
  std::atomic_thread_fence(std::memory_order_acquire);
  bool overflowed = false;
  for (scn_grids *g : ctx->pendingGrids) {
    const volatile int64_t *slot = ctx->h_pinned + 16 + 4 * g->pinnedSlot;
    if (g->chained)
      scn_chain_settled(ctx, g, slot[3], slot[2] != 0);
    if (slot[2]) {
      overflowed = true;
      g->planKind = PLAN_NONE; // nothing was emitted
      g->nSites = 0;
      g->nActive = 0;
    } else {
      g->nSites = (int)slot[0];
      g->nActive = slot[1];
      g->seenRows = slot[0] > g->seenRows ? slot[0] : g->seenRows;
      g->seenActive = slot[1] > g->seenActive ? slot[1] : g->seenActive;
      if (g->planKind == PLAN_TERMINAL) {
        g->termS = slot[3];
        g->seenWidth = slot[3] > g->seenWidth ? slot[3] : g->seenWidth;
      }
    }
    g->pending = false;
    g->pinnedSlot = -1;
  }
  ctx->pendingGrids.clear();
  if (ctx->h_pinned[15] != 0) {
    long long bad = ctx->h_pinned[15];
    ctx->h_pinned[15] = 0;
    SCN_TRY(scn_fill32(ctx, ctx->d_scalars + 15, 0u, 2));
    SCN_REQUIRE(false, SCN_ERR_ARG,
                "scn_grids_build was given %lld sites outside the field", bad);
  }
  SCN_REQUIRE(!overflowed, SCN_ERR_CAPACITY,
              "scn_rules_settle: a batch outgrew the bounds of its deferred "
              "plans; plan it again with deferral off");
  return SCN_OK;
}
void mark_pending(scn_ctx *ctx, scn_grids *g, int slot) {
  g->pending = true;
  g->pinnedSlot = slot;
  ctx->pendingGrids.push_back(g);
}

extern "C" int scn_grids_create(scn_ctx *ctx, scn_grids **out) {
  SCN_REQUIRE(ctx && out, SCN_ERR_ARG, "scn_grids_create: null argument");
  *out = new scn_grids();
  return SCN_OK;
}

extern "C" int scn_grids_destroy(scn_ctx *ctx, scn_grids *g) {
  if (!g)
    return SCN_OK;
  if (ctx) {
    (void)scn_chain_flush(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    auto &pl = ctx->pendingGrids;
    for (size_t i = 0; i < pl.size(); ++i)
      if (pl[i] == g) {
        pl.erase(pl.begin() + i);
        break;
      }
  }
  g->meta.release();
  g->table.release();
  g->dense.release();
  g->bits.release();
  g->prefix.release();
  g->rankRow.release();
  g->ekey.release();
  g->erow.release();
  g->bg.release();
  g->scanTmp.release();
  g->siteKey.release();
  g->cnt.release();
  g->ownMask.release();
  g->rankOf.release();
  g->base.release();
  g->bgBefore.release();
  g->sampleStart.release();
  g->invOrd.release();
  g->ticks.release();
  g->dlSample.release();
  g->dlRow.release();
  g->dlKey.release();
  delete g;
  return SCN_OK;
}

extern "C" int scn_grids_build(scn_ctx *ctx, scn_grids *g, int batch,
                               int dimension, int spatialSize,
                               const int32_t *d_sample, const int64_t *d_key,
                               const int32_t *d_row, int64_t n,
                               const int32_t *d_background,
                               int32_t nSpatialSites) {
  SCN_REQUIRE(ctx && g, SCN_ERR_ARG, "scn_grids_build: null argument");
  SCN_REQUIRE(n >= 0 && (n == 0 || (d_sample && d_key && d_row)), SCN_ERR_ARG,
              "scn_grids_build: null site arrays");
  SCN_REQUIRE(batch == 0 || d_background, SCN_ERR_ARG,
              "scn_grids_build: null background array");
  SCN_TRY(scn_chain_flush(ctx));
  ProfScope ps(ctx, SCN_K_GRID_BUILD);
  // batches small enough for a dense row table get it as they are built (a
  // chain of recorded plans reads its source through it); larger ones get
  // their hash table when somebody asks
  long long sites = batch > 0 ? batch : 1;
  for (int a = 0; a < dimension && a < 3; ++a)
    sites *= spatialSize > 0 ? spatialSize : 1;
  SCN_TRY(grids_prepare(ctx, g, batch, dimension, spatialSize, n,
                        sites <= SCN_DENSE_MAX_SITES));
  g->nSites = nSpatialSites;
  // (backgroundCol is copied by the same launch: lane e < batch takes entry e)
  const long long lanes = n > batch ? n : batch;
  if (lanes > 0) {
    hipLaunchKernelGGL(k_grid_build, dim3(scn_ceil_div(lanes, 256)), dim3(256), 0,
                       ctx->stream, view_of(g), d_sample,
                       (const long long *)d_key, d_row, (long long)n, g->ekey.p,
                       g->erow.p, (unsigned long long *)(ctx->d_scalars + 15),
                       d_background, g->bg.p);
    SCN_HIP_CHECK(hipGetLastError());
  }
  return SCN_OK;
}

extern "C" int scn_grids_info(const scn_grids *g, int *batch, int *dimension,
                              int *spatialSize, int64_t *nActive,
                              int32_t *nSpatialSites) {
  SCN_REQUIRE(g, SCN_ERR_ARG, "scn_grids_info: null grids");
  SCN_REQUIRE(!g->pending, SCN_ERR_STATE,
              "scn_grids_info: the counts of these grids are deferred; call "
              "scn_rules_settle first");
  if (batch)
    *batch = g->batch;
  if (dimension)
    *dimension = g->d;
  if (spatialSize)
    *spatialSize = g->n;
  if (nActive)
    *nActive = g->nActive;
  if (nSpatialSites)
    *nSpatialSites = g->nSites;
  return SCN_OK;
}

extern "C" int scn_grids_download(scn_ctx *ctx, const scn_grids *cg,
                                  int32_t *h_sample, int64_t *h_key,
                                  int32_t *h_row, int32_t *h_background) {
  scn_grids *g = const_cast<scn_grids *>(cg);
  SCN_REQUIRE(ctx && g, SCN_ERR_ARG, "scn_grids_download: null argument");
  SCN_REQUIRE(!g->pending, SCN_ERR_STATE,
              "scn_grids_download: the counts of these grids are deferred; "
              "call scn_rules_settle first");
  SCN_TRY(ensure_rank(ctx, g));
  long long n = g->nActive;
  if (n > 0) {
    SCN_TRY(g->dlSample.reserve((size_t)n));
    SCN_TRY(g->dlRow.reserve((size_t)n));
    SCN_TRY(g->dlKey.reserve((size_t)n));
    hipLaunchKernelGGL(k_download, dim3(scn_ceil_div(n, 256)), dim3(256), 0,
                       ctx->stream, view_of(g), g->ekey.p, g->erow.p, n,
                       g->dlSample.p, g->dlKey.p, g->dlRow.p);
    SCN_HIP_CHECK(hipGetLastError());
    SCN_TRY(scn_d2h(ctx, h_sample, g->dlSample.p, n * sizeof(int)));
    SCN_TRY(scn_d2h(ctx, h_key, g->dlKey.p, n * sizeof(long long)));
    SCN_TRY(scn_d2h(ctx, h_row, g->dlRow.p, n * sizeof(int)));
  }
  if (g->batch > 0)
    SCN_TRY(scn_d2h(ctx, h_background, g->bg.p, g->batch * sizeof(int)));
  return SCN_OK;
}

extern "C" int scn_grids_find(scn_ctx *ctx, const scn_grids *g,
                              const int32_t *d_sample, const int64_t *d_key,
                              int64_t n, int32_t *d_row) {
  SCN_REQUIRE(ctx && g, SCN_ERR_ARG, "scn_grids_find: null argument");
  if (n <= 0)
    return SCN_OK;
  SCN_TRY(scn_grids_ensure_table(ctx, const_cast<scn_grids *>(g)));
  hipLaunchKernelGGL(k_find, dim3(scn_ceil_div(n, 256)), dim3(256), 0,
                     ctx->stream, view_of(g), d_sample,
                     (const long long *)d_key, (long long)n, d_row);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

static int triangle_size(int n, int d) { // utilities.cu:27-32
  int fs = 1;
  for (int i = 1; i <= d; ++i)
    fs = fs * (n + d - i) / i;
  return fs;
}

// SCN_TILE2_WORDWISE=0 sends windows of side 2, stride 2 down the general path
static bool tile2_enabled() {
  static const bool on = [] {
    const char *e = getenv("SCN_TILE2_WORDWISE");
    return !(e && e[0] == '0');
  }();
  return on;
}

template <int D>
static int plan_regions_d(scn_ctx *ctx, scn_grids *in, scn_grids *out,
                          const Geom &g, long long fullSize,
                          int64_t *nOutSites, long long fmpCand = 0) {
  // deferred: size by bounds, leave the counts on the device (see scn_rules_settle)
  const bool deferred = ctx->deferCounts && out->seenRows > 0 &&
                        (int)ctx->pendingGrids.size() < SCN_MAX_PENDING;
  if (!deferred && in->pending)
    SCN_TRY(scn_rules_settle(ctx)); // the exact path needs the exact input count
  const long long nE = in->nActive; // a bound while `in` is pending
  const Count nEc = count_active(in);
  const long long *inMeta = in->pending ? in->meta.p : nullptr;
  const long long volOutAll = (long long)in->batch * g.volOut;
  const long long boundActive =
      deferred ? grow_bound(out->seenActive, 64, volOutAll) : 0x7FFFFFFFFFFFll;
  const long long boundRows =
      deferred ? grow_bound(out->seenRows, 64, boundActive + in->batch)
               : 0x7FFFFFFFFFFFll;
  const int slot = deferred ? (int)ctx->pendingGrids.size() : -1;
  SCN_TRY(out->meta.reserve(8));
  SCN_TRY(out->cnt.reserve((size_t)nE + 8)); // the scan reads whole 16-byte groups
  SCN_TRY(out->base.reserve((size_t)nE + 2));
  SCN_TRY(out->bgBefore.reserve((size_t)in->batch + 2));
  SCN_TRY(out->sampleStart.reserve((size_t)in->batch + 2));
  SCN_TRY(out->bg.reserve((size_t)in->batch + 1));
  SCN_TRY(out->scanTmp.reserve(scn_scan_tmp_elems((size_t)nE + 1)));
  GridView vin = view_of(in);
  // number of candidates of one input: (ceil(size / stride))^d at most
  long long maxCand = 1;
  for (int a = 0; a < D; ++a)
    maxCand *= g.mode == MODE_SQ_VALID ? 1 : (g.size + g.stride - 1) / g.stride;
  if (g.mode == MODE_SQ_FMP)
    maxCand = fmpCand; // from the tables themselves
  const bool masked = maxCand <= 64;
  // windows of side 2 that tile the field: owners and counts from the input
  // mask a word at a time (k_tile2_owners)
  const bool tiled = tile2_enabled() && g.mode == MODE_SQ_NOMIN && g.size == 2 &&
                     g.stride == 2 && in->batch > 0;
  const long long ownWords = (long long)in->nWords + 1; // one past: the rank of the end
  if (tiled) {
    SCN_TRY(out->ownMask.reserve((size_t)ownWords + 8)); // the scan reads whole 32-byte groups
    SCN_TRY(out->base.reserve((size_t)ownWords + 2));
    SCN_TRY(out->scanTmp.reserve(scn_scan_tmp_elems((size_t)ownWords)));
    hipLaunchKernelGGL(k_tile2_owners<D>, dim3(xcd_grid(scn_ceil_div(ownWords, 256))),
                       dim3(256), 0, ctx->stream, vin, g, inMeta, out->ownMask.p,
                       ownWords, (long long)in->batch * g.volIn);
    SCN_HIP_CHECK(hipGetLastError());
  } else if (masked) {
    SCN_TRY(out->ownMask.reserve((size_t)nE + 2));
    SCN_TRY(out->rankOf.reserve((size_t)nE + 2));
  }
  if (nE > 0 && !tiled) {
    hipLaunchKernelGGL(k_plan_count<D>, dim3(xcd_grid(scn_ceil_div(nE, 256))), dim3(256),
                       0, ctx->stream, vin, g, in->ekey.p, nEc, inMeta, out->cnt.p,
                       masked ? out->ownMask.p : nullptr, out->rankOf.p);
    SCN_HIP_CHECK(hipGetLastError());
  }
  const long long *bad = (const long long *)(ctx->d_scalars + 15);
  const long long ticket = ++ctx->ticket;
  if (tiled) {
    SCN_TRY(scn_scan_exclusive_popc64(ctx->stream, (const uint64_t *)out->ownMask.p,
                                      out->base.p, (size_t)ownWords, out->scanTmp.p));
    GridView owners = vin;
    owners.bits = out->ownMask.p;
    owners.prefix = out->base.p;
    hipLaunchKernelGGL(k_plan_samples<true>, dim3(1), dim3(SCAN1_THREADS), 0, ctx->stream,
                       owners, (const unsigned *)nullptr, 0ll, fullSize, out->bg.p,
                       out->bgBefore.p, out->sampleStart.p, (long long *)ctx->d_pinned, bad,
                       ticket, out->meta.p, inMeta, boundRows, boundActive, slot);
  } else if ((size_t)nE <= SCAN1_MAX_ELEMS) {
    hipLaunchKernelGGL(k_plan_scan_samples, dim3(1), dim3(SCAN1_THREADS), 0,
                       ctx->stream, vin, out->cnt.p, out->base.p, nE, fullSize,
                       out->bg.p, out->bgBefore.p, out->sampleStart.p,
                       (long long *)ctx->d_pinned, bad, ticket, out->meta.p,
                       inMeta, boundRows, boundActive, slot);
  } else {
    SCN_TRY(scn_scan_exclusive_u32(ctx->stream, out->cnt.p, out->base.p,
                                   (size_t)nE, out->scanTmp.p));
    hipLaunchKernelGGL(k_plan_samples<false>, dim3(1), dim3(SCAN1_THREADS), 0, ctx->stream, vin,
                       out->base.p, nE, fullSize, out->bg.p, out->bgBefore.p,
                       out->sampleStart.p, (long long *)ctx->d_pinned, bad, ticket, out->meta.p,
                         inMeta, boundRows, boundActive, slot);
  }
  SCN_HIP_CHECK(hipGetLastError());
  long long nSites = boundRows, nOutActive = boundActive;
  if (!deferred) {
    SCN_TRY(read_scalars(ctx, ticket));
    nSites = ctx->h_pinned[0];
    nOutActive = ctx->h_pinned[1];
    out->seenRows = nSites > out->seenRows ? nSites : out->seenRows;
    out->seenActive = nOutActive > out->seenActive ? nOutActive : out->seenActive;
  }
  SCN_REQUIRE(nSites < 2147483647ll, SCN_ERR_CAPACITY,
              "rules: %lld output rows do not fit 32-bit row numbers", nSites);
  // out->bg already holds what k_plan_samples wrote: grids_prepare only
  // reserves it (no reallocation at the same size) and clears table and mask
  SCN_TRY(grids_prepare(ctx, out, in->batch, g.d, g.nOut, nOutActive));
  out->nSites = (int)nSites;
  if (deferred)
    mark_pending(ctx, out, slot);
  SCN_TRY(out->siteKey.reserve((size_t)nSites + 1));
  long long nThreads = nE > in->batch ? nE : in->batch;
  // the output mask: word by word from the input mask where the mode allows
  // it, else bit by bit as the emit pass finds the sites
  GridView vout = view_of(out);
  if (g.mode == MODE_SQ_NOMIN && g.size <= 64) {
    const long long words = (long long)out->nWords + 2;
    const long long blocks = (scn_ceil_div(words, 256) + 7) / 8 * 8; // whole rounds of the 8 XCDs
    auto dilate = g.size == 2 ? k_mask_dilate<D, 2>
                              : (g.size == 3 ? k_mask_dilate<D, 3> : k_mask_dilate<D, 0>);
    hipLaunchKernelGGL(dilate, dim3((unsigned)blocks), dim3(256),
                       0, ctx->stream, vin, g, out->bits.p, words,
                       (long long)in->batch * g.volOut);
    SCN_HIP_CHECK(hipGetLastError());
    vout.bits = nullptr;
  }
  if (tiled) {
    const long long lanes = ownWords > in->batch ? ownWords : in->batch;
    hipLaunchKernelGGL(k_tile2_emit<D>, dim3(xcd_grid(scn_ceil_div(lanes, 256))), dim3(256),
                       0, ctx->stream, vin, g, out->ownMask.p, out->base.p, ownWords,
                       out->meta.p, out->bgBefore.p, out->bg.p, out->ekey.p, out->erow.p,
                       out->siteKey.p);
    SCN_HIP_CHECK(hipGetLastError());
  } else if (nThreads > 0 && masked && maxCand > 9) {
    hipLaunchKernelGGL(k_plan_emit_walk<D>, dim3(xcd_grid(scn_ceil_div(nThreads, 256))),
                       dim3(256), 0, ctx->stream, vin, vout, g,
                       in->ekey.p, nEc, out->meta.p, out->base.p, out->ownMask.p,
                       out->rankOf.p, out->bgBefore.p, out->bg.p, out->ekey.p,
                       out->erow.p, out->siteKey.p);
    SCN_HIP_CHECK(hipGetLastError());
  } else if (nThreads > 0 && masked) {
    hipLaunchKernelGGL(k_plan_emit_masked<D>,
                       dim3(xcd_grid(scn_ceil_div(nThreads, 256)), (unsigned)maxCand),
                       dim3(256), 0, ctx->stream, vin, vout, g,
                       in->ekey.p, nEc, out->meta.p, out->base.p, out->ownMask.p,
                       out->rankOf.p, out->bgBefore.p, out->bg.p, out->ekey.p,
                       out->erow.p, out->siteKey.p);
    SCN_HIP_CHECK(hipGetLastError());
  } else if (nThreads > 0) {
    hipLaunchKernelGGL(k_plan_emit<D>, dim3(xcd_grid(scn_ceil_div(nThreads, 256))),
                       dim3(256), 0, ctx->stream, vin, vout, g,
                       in->ekey.p, nEc, out->meta.p, out->base.p, out->bgBefore.p,
                       out->bg.p,
                       out->ekey.p, out->erow.p, out->siteKey.p);
    SCN_HIP_CHECK(hipGetLastError());
  }
  *nOutSites = nSites;
  return SCN_OK;
}

static int plan_regions(scn_ctx *ctx, const scn_grids *cin, scn_grids *out,
                        int nIn, int nOut, int size, int stride, int minActive,
                        bool tri, int64_t *nOutSites) {
  scn_grids *in = const_cast<scn_grids *>(cin);
  SCN_REQUIRE(ctx && in && out && nOutSites, SCN_ERR_ARG,
              "rules plan: null argument");
  SCN_REQUIRE(in != out, SCN_ERR_ARG, "rules plan: in and out are the same object");
  SCN_REQUIRE(size >= 1 && size <= 32 && stride >= 1 && nOut >= 1,
              SCN_ERR_ARG, "rules plan: size %d stride %d nOut %d", size,
              stride, nOut);
  // Regions.cu:17,823
  SCN_REQUIRE(nIn == size + (nOut - 1) * stride, SCN_ERR_ARG,
              "rules plan: nIn %d != size %d + (nOut %d - 1) * stride %d", nIn,
              size, nOut, stride);
  SCN_REQUIRE(in->n == nIn, SCN_ERR_ARG,
              "rules plan: input grids have spatialSize %d, regions say %d",
              in->n, nIn);
  Geom g;
  g.d = in->d;
  g.nIn = nIn;
  g.nOut = nOut;
  g.size = size;
  g.stride = stride;
  g.minActive = minActive;
  g.volIn = in->vol;
  g.volOut = ipow_ll(nOut, in->d);
  g.cube = (int)ipow_ll(size, in->d);
  g.magicStride = (unsigned)((1ull << 32) / (unsigned)stride + 1);
  g.ticks = nullptr;
  g.tInR = g.tOutL = g.tOutR = 0;
  SCN_REQUIRE(ipow_ll(size, in->d) <= 32768, SCN_ERR_ARG,
              "rules plan: window of %d^%d sites", size, in->d);
  long long fullSize;
  if (tri) {
    SCN_REQUIRE(minActive >= 1, SCN_ERR_ARG,
                "triangular rules: minActive %d", minActive);
    g.mode = minActive == 1 ? MODE_TRI_NOMIN : MODE_TRI_MIN;
    g.width = triangle_size(size, in->d);
    fullSize = triangle_size(nOut, in->d);
  } else {
    SCN_REQUIRE(minActive >= 1 || minActive == -1, SCN_ERR_ARG,
                "square rules: minActive %d", minActive);
    if (minActive == -1) {
      // Regions.cu:668,671,714,748: only the 2-D, size-3 case is live
      SCN_REQUIRE(size == 3 && in->d == 2, SCN_ERR_ARG,
                  "valid-mode rules need dimension 2 and size 3");
      g.mode = MODE_SQ_VALID;
    } else
      g.mode = minActive == 1 ? MODE_SQ_NOMIN : MODE_SQ_MIN;
    g.width = g.cube;
    fullSize = g.volOut;
  }
  {
    // a plan that can wait joins the chain of recorded plans
    long long maxCand = 1;
    for (int a = 0; a < in->d; ++a)
      maxCand *= g.mode == MODE_SQ_VALID ? 1 : (size + stride - 1) / stride;
    bool taken = false;
    SCN_TRY(scn_chain_record_regions(ctx, in, out, g, fullSize, maxCand,
                                     nOutSites, &taken));
    if (taken)
      return SCN_OK;
    SCN_TRY(scn_chain_flush(ctx));
  }
  ProfScope ps(ctx, SCN_K_RULES);
  SCN_TRY(ensure_rank(ctx, in));
  int rc;
  switch (in->d) {
  case 1:
    rc = plan_regions_d<1>(ctx, in, out, g, fullSize, nOutSites);
    break;
  case 2:
    rc = plan_regions_d<2>(ctx, in, out, g, fullSize, nOutSites);
    break;
  default:
    rc = plan_regions_d<3>(ctx, in, out, g, fullSize, nOutSites);
    break;
  }
  SCN_TRY(rc);
  if (tri) {
    SCN_TRY(out->invOrd.reserve((size_t)g.cube));
    hipLaunchKernelGGL(k_tri_table, dim3(1), dim3(64), 0, ctx->stream, size,
                       in->d, out->invOrd.p);
    SCN_HIP_CHECK(hipGetLastError());
  }
  out->geom = g;
  out->planKind = PLAN_REGIONS;
  out->planIn = in;
  return SCN_OK;
}

extern "C" int scn_rules_square_plan(scn_ctx *ctx, const scn_grids *in,
                                     scn_grids *out, int nIn, int nOut,
                                     int size, int stride, int minActive,
                                     int64_t *nOutSites) {
  return plan_regions(ctx, in, out, nIn, nOut, size, stride, minActive, false,
                      nOutSites);
}

extern "C" int scn_rules_triangular_plan(scn_ctx *ctx, const scn_grids *in,
                                         scn_grids *out, int nIn, int nOut,
                                         int size, int stride, int minActive,
                                         int64_t *nOutSites) {
  return plan_regions(ctx, in, out, nIn, nOut, size, stride, minActive, true,
                      nOutSites);
}

// gridRules over FractionalPoolingRegions (Regions.cu:121-156 and the tick
// constructors :31-119): the caller brings inputL / inputR of every sample and
// axis; outputL / outputR follow from them as in the tick constructors
// (:49-56).  The tables are checked on the host so that no kernel indexes
// outside a grid.
extern "C" int scn_rules_fmp_plan(scn_ctx *ctx, const scn_grids *cin,
                                  scn_grids *out, int nIn, int nOut,
                                  int poolSize, const int32_t *h_inputL,
                                  const int32_t *h_inputR,
                                  int64_t *nOutSites) {
  scn_grids *in = const_cast<scn_grids *>(cin);
  SCN_REQUIRE(ctx && in && out && nOutSites && h_inputL && h_inputR,
              SCN_ERR_ARG, "fmp rules plan: null argument");
  SCN_REQUIRE(in != out, SCN_ERR_ARG,
              "fmp rules plan: in and out are the same object");
  SCN_REQUIRE(poolSize >= 1 && poolSize <= 32 && nOut >= 1, SCN_ERR_ARG,
              "fmp rules plan: poolSize %d nOut %d", poolSize, nOut);
  SCN_REQUIRE(nIn >= nOut - 1 + poolSize, SCN_ERR_ARG, // Regions.cu:35,131
              "fmp rules plan: nIn %d < nOut %d - 1 + poolSize %d", nIn, nOut,
              poolSize);
  SCN_REQUIRE(in->n == nIn, SCN_ERR_ARG,
              "fmp rules plan: input grids have spatialSize %d, regions say %d",
              in->n, nIn);
  const int d = in->d, B = in->batch;
  SCN_REQUIRE(ipow_ll(poolSize, d) <= 32768, SCN_ERR_ARG,
              "fmp rules plan: window of %d^%d sites", poolSize, d);
  const size_t nT = (size_t)B * d * nOut, nI = (size_t)B * d * nIn;
  std::vector<int> t(2 * nT + 2 * nI);
  int *inL = t.data(), *inR = inL + nT, *outL = inR + nT, *outR = outL + nI;
  long long cand = 1;
  std::vector<int> widest(d, 0);
  for (int b = 0; b < B; ++b)
    for (int a = 0; a < d; ++a) {
      const size_t o = ((size_t)b * d + a) * nOut, oi = ((size_t)b * d + a) * nIn;
      for (int i = 0; i < nIn; ++i) {
        outL[oi + i] = nOut;
        outR[oi + i] = 0;
      }
      for (int j = 0; j < nOut; ++j) {
        const int l = h_inputL[o + j], r = h_inputR[o + j];
        SCN_REQUIRE(l >= 0 && r > l && r - l <= poolSize && r <= nIn &&
                        (j == 0 || (l >= h_inputL[o + j - 1] &&
                                    r >= h_inputR[o + j - 1])),
                    SCN_ERR_ARG,
                    "fmp rules plan: sample %d axis %d region %d = [%d, %d)", b,
                    a, j, l, r);
        inL[o + j] = l;
        inR[o + j] = r;
        for (int i = l; i < r; ++i) {
          outL[oi + i] = outL[oi + i] < j ? outL[oi + i] : j;
          outR[oi + i] = outR[oi + i] > j + 1 ? outR[oi + i] : j + 1;
        }
      }
      for (int i = 0; i < nIn; ++i)
        if (outR[oi + i] - outL[oi + i] > widest[a])
          widest[a] = outR[oi + i] - outL[oi + i];
    }
  for (int a = 0; a < d; ++a)
    cand *= widest[a] > 0 ? widest[a] : 1;
  Geom g;
  g.d = d;
  g.nIn = nIn;
  g.nOut = nOut;
  g.size = poolSize;
  g.stride = 1;
  g.minActive = 1;
  g.mode = MODE_SQ_FMP;
  g.volIn = in->vol;
  g.volOut = ipow_ll(nOut, d);
  g.cube = (int)ipow_ll(poolSize, d);
  g.magicStride = 0; // (stride 1: div_magic leaves x as it is)
  g.width = g.cube;
  g.tInR = (long long)nT;
  g.tOutL = (long long)(2 * nT);
  g.tOutR = (long long)(2 * nT + nI);
  SCN_TRY(scn_chain_flush(ctx));
  ProfScope ps(ctx, SCN_K_RULES);
  SCN_TRY(out->ticks.reserve(t.size() + 1));
  // (the copy returns when done: `t` may go out of scope)
  SCN_TRY(scn_h2d(ctx, out->ticks.p, t.data(), t.size() * sizeof(int)));
  g.ticks = out->ticks.p;
  SCN_TRY(ensure_rank(ctx, in));
  int rc;
  switch (d) {
  case 1:
    rc = plan_regions_d<1>(ctx, in, out, g, g.volOut, nOutSites, cand);
    break;
  case 2:
    rc = plan_regions_d<2>(ctx, in, out, g, g.volOut, nOutSites, cand);
    break;
  default:
    rc = plan_regions_d<3>(ctx, in, out, g, g.volOut, nOutSites, cand);
    break;
  }
  SCN_TRY(rc);
  out->geom = g;
  out->planKind = PLAN_REGIONS;
  out->planIn = in;
  return SCN_OK;
}

extern "C" int scn_rules_terminal_plan(scn_ctx *ctx, const scn_grids *cin,
                                       scn_grids *out, int64_t *ruleWidth) {
  scn_grids *in = const_cast<scn_grids *>(cin);
  SCN_REQUIRE(ctx && in && out && ruleWidth, SCN_ERR_ARG,
              "terminal rules plan: null argument");
  SCN_REQUIRE(in != out, SCN_ERR_ARG,
              "terminal rules plan: in and out are the same object");
  {
    bool taken = false;
    SCN_TRY(scn_chain_record_terminal(ctx, in, out, ruleWidth, &taken));
    if (taken)
      return SCN_OK;
    SCN_TRY(scn_chain_flush(ctx));
  }
  ProfScope ps(ctx, SCN_K_RULES);
  const bool deferred = ctx->deferCounts && out->seenWidth > 0 &&
                        (int)ctx->pendingGrids.size() < SCN_MAX_PENDING;
  SCN_TRY(ensure_rank(ctx, in));
  SCN_TRY(out->sampleStart.reserve((size_t)in->batch + 2));
  SCN_TRY(out->meta.reserve(8));
  const long long boundWidth =
      deferred ? grow_bound(out->seenWidth, 8, in->vol) : 0x7FFFFFFFFFFFll;
  const int slot = deferred ? (int)ctx->pendingGrids.size() : -1;
  const long long ticket = ++ctx->ticket;
  hipLaunchKernelGGL(k_terminal_plan, dim3(1), dim3(SCAN1_THREADS), 0, ctx->stream,
                     view_of(in), out->sampleStart.p,
                     (long long *)ctx->d_pinned, ticket, out->meta.p,
                     in->pending ? in->meta.p : nullptr, boundWidth, slot);
  SCN_HIP_CHECK(hipGetLastError());
  long long S = boundWidth;
  if (!deferred) {
    SCN_TRY(read_scalars(ctx, ticket));
    S = ctx->h_pinned[0];
    out->seenWidth = S > out->seenWidth ? S : out->seenWidth;
  }
  SCN_TRY(grids_prepare(ctx, out, in->batch, in->d, 1, in->batch));
  out->nSites = in->batch;
  if (deferred)
    mark_pending(ctx, out, slot);
  if (in->batch > 0) {
    hipLaunchKernelGGL(k_terminal_out, dim3(scn_ceil_div(in->batch, 256)),
                       dim3(256), 0, ctx->stream, view_of(out), out->ekey.p,
                       out->erow.p, out->bg.p);
    SCN_HIP_CHECK(hipGetLastError());
  }
  out->termS = S;
  out->planKind = PLAN_TERMINAL;
  out->planIn = in;
  *ruleWidth = S;
  return SCN_OK;
}

extern "C" int scn_rules_width(const scn_grids *out, int64_t *width) {
  SCN_REQUIRE(out && width, SCN_ERR_ARG, "scn_rules_width: null argument");
  SCN_REQUIRE(out->planKind != PLAN_NONE, SCN_ERR_STATE,
              "scn_rules_width: no plan on these grids");
  *width = out->planKind == PLAN_TERMINAL ? out->termS : out->geom.width;
  return SCN_OK;
}

extern "C" int scn_rules_fill(scn_ctx *ctx, const scn_grids *in,
                              scn_grids *out, int32_t *d_rules,
                              int64_t capacity) {
  SCN_REQUIRE(ctx && in && out, SCN_ERR_ARG, "scn_rules_fill: null argument");
  SCN_REQUIRE(out->planKind != PLAN_NONE && out->planIn == in, SCN_ERR_STATE,
              "scn_rules_fill: `out` does not hold a plan made from `in`");
  {
    bool taken = false;
    SCN_TRY(scn_chain_record_fill(ctx, in, out, d_rules, capacity, &taken));
    if (taken)
      return SCN_OK;
    SCN_TRY(scn_chain_flush(ctx));
  }
  SCN_REQUIRE(!out->chained, SCN_ERR_STATE,
              "scn_rules_fill: the rules of a recorded plan are written when "
              "the chain runs; plan again to fill another buffer");
  ProfScope ps(ctx, SCN_K_RULES);
  SCN_TRY(ensure_rank(ctx, const_cast<scn_grids *>(in)));
  GridView vin = view_of(in);
  if (out->planKind == PLAN_TERMINAL) {
    long long total = (long long)in->batch * out->termS;
    SCN_REQUIRE(capacity >= total, SCN_ERR_CAPACITY,
                "scn_rules_fill: %lld rules, capacity %lld", total,
                (long long)capacity);
    if (total == 0)
      return SCN_OK;
    SCN_REQUIRE(d_rules, SCN_ERR_ARG, "scn_rules_fill: null rules buffer");
    hipLaunchKernelGGL(k_terminal_init, dim3(scn_ceil_div(total, 256)),
                       dim3(256), 0, ctx->stream, vin, out->sampleStart.p,
                       count_width(out), out->meta.p, d_rules);
    SCN_HIP_CHECK(hipGetLastError());
    if (in->nActive > 0) {
      hipLaunchKernelGGL(k_terminal_scatter,
                         dim3(scn_ceil_div(in->nActive, 256)), dim3(256), 0,
                         ctx->stream, vin, in->ekey.p, in->erow.p,
                         count_active(in), out->sampleStart.p, count_width(out),
                         out->meta.p, d_rules);
      SCN_HIP_CHECK(hipGetLastError());
    }
    return SCN_OK;
  }
  const Geom &g = out->geom;
  long long total = (long long)out->nSites * g.width;
  SCN_REQUIRE(capacity >= total, SCN_ERR_CAPACITY,
              "scn_rules_fill: %lld rules, capacity %lld", total,
              (long long)capacity);
  if (total == 0)
    return SCN_OK;
  SCN_REQUIRE(d_rules, SCN_ERR_ARG, "scn_rules_fill: null rules buffer");
  const bool tri = g.mode == MODE_TRI_NOMIN || g.mode == MODE_TRI_MIN;
  const int *inv = tri ? out->invOrd.p : nullptr;
  // the output mask is final (the emit pass has run): its rank prefix rides
  // along as one more workgroup when it is short enough for one
  const bool scan = !out->rankValid && out->nWords + 1 <= SCAN1_MAX_ELEMS;
  const RankScan rs = {out->bits.p, out->prefix.p, scan ? out->nWords + 1 : 0};
  const unsigned extra = scan ? 1 : 0;
  dim3 grid(scn_ceil_div(total, 256) + extra), block(256);
#define SCN_FILL_DIM(KERNEL, ...)                                              \
  switch (g.d) {                                                               \
  case 1:                                                                      \
    if (scan)                                                                  \
      hipLaunchKernelGGL((KERNEL<1, true>), __VA_ARGS__);                      \
    else                                                                       \
      hipLaunchKernelGGL((KERNEL<1, false>), __VA_ARGS__);                     \
    break;                                                                     \
  case 2:                                                                      \
    if (scan)                                                                  \
      hipLaunchKernelGGL((KERNEL<2, true>), __VA_ARGS__);                      \
    else                                                                       \
      hipLaunchKernelGGL((KERNEL<2, false>), __VA_ARGS__);                     \
    break;                                                                     \
  default:                                                                     \
    if (scan)                                                                  \
      hipLaunchKernelGGL((KERNEL<3, true>), __VA_ARGS__);                      \
    else                                                                       \
      hipLaunchKernelGGL((KERNEL<3, false>), __VA_ARGS__);                     \
    break;                                                                     \
  }
  // rule rows a workgroup of the run kernel collects in LDS
  const int rowsPerBlock =
      g.width > 0 && FILL_LDS_INTS / g.width < 256 ? FILL_LDS_INTS / g.width : 256;
  if (!tri && g.size >= 2 && g.mode != MODE_SQ_FMP && rowsPerBlock >= 1) {
    const int pitch = g.width | 1;
    const unsigned magicWidth = (unsigned)((1ull << 32) / (unsigned)g.width + 1);
    const unsigned magicSize = (unsigned)((1ull << 32) / (unsigned)g.size + 1);
    dim3 runs(extra ? (unsigned)scn_ceil_div(out->nSites, rowsPerBlock) + extra
                    : xcd_grid(scn_ceil_div(out->nSites, rowsPerBlock)));
    const size_t stagedBytes = ((size_t)rowsPerBlock * pitch + 4) * sizeof(int);
#define SCN_FILL_RUNS(D, SC)                                                   \
  if (g.size == 2)                                                             \
    hipLaunchKernelGGL((k_rules_fill_runs<D, SC, 2>), runs, block, stagedBytes,\
                       ctx->stream, vin, g, out->siteKey.p, count_sites(out),  \
                       out->meta.p, d_rules, rs, rowsPerBlock, pitch,          \
                       magicWidth, magicSize);                                 \
  else if (g.size == 3)                                                        \
    hipLaunchKernelGGL((k_rules_fill_runs<D, SC, 3>), runs, block, stagedBytes,\
                       ctx->stream, vin, g, out->siteKey.p, count_sites(out),  \
                       out->meta.p, d_rules, rs, rowsPerBlock, pitch,          \
                       magicWidth, magicSize);                                 \
  else                                                                         \
    hipLaunchKernelGGL((k_rules_fill_runs<D, SC, 0>), runs, block, stagedBytes,\
                       ctx->stream, vin, g, out->siteKey.p, count_sites(out),  \
                       out->meta.p, d_rules, rs, rowsPerBlock, pitch,          \
                       magicWidth, magicSize);
    switch (g.d) {
    case 1:
      if (scan) { SCN_FILL_RUNS(1, true) } else { SCN_FILL_RUNS(1, false) }
      break;
    case 2:
      if (scan) { SCN_FILL_RUNS(2, true) } else { SCN_FILL_RUNS(2, false) }
      break;
    default:
      if (scan) { SCN_FILL_RUNS(3, true) } else { SCN_FILL_RUNS(3, false) }
      break;
    }
#undef SCN_FILL_RUNS
  } else {
    SCN_FILL_DIM(k_rules_fill, grid, block, 0, ctx->stream, vin, g,
                 out->siteKey.p, count_sites(out), out->meta.p, inv, d_rules, rs)
  }
#undef SCN_FILL_DIM
  SCN_HIP_CHECK(hipGetLastError());
  if (scan)
    out->rankValid = true;
  return SCN_OK;
}
