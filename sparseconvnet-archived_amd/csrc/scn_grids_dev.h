// Types and device helpers shared by the translation units that build sparse
// grids and rule books (scn_grids.hip: one layer at a time through tables in
// HBM; scn_chain.hip: all layers of a net at once, one workgroup per sample).
#pragma once
#include "scn_common.h"
#include "scn_scan_dev.h"

struct __align__(16) Slot {
  long long key;
  int row;
  int pad;
};
#define SLOT_EMPTY (-1LL)

enum { MODE_SQ_NOMIN = 0, MODE_SQ_MIN, MODE_SQ_VALID, MODE_TRI_NOMIN, MODE_TRI_MIN, MODE_SQ_FMP };
enum { PLAN_NONE = 0, PLAN_REGIONS = 1, PLAN_TERMINAL = 2 };

struct Geom {
  int d;
  int nIn, nOut, size, stride, minActive, mode;
  long long volIn, volOut;
  int width; // rule-row width: size^d or triangleSize(size, d)
  int cube;  // size^d
  unsigned magicStride; // floor(2^32 / stride) + 1 (div_magic)
  // MODE_SQ_FMP: per-sample, per-axis region tables (fractional max-pooling).
  // inputL at ticks[(b d + a) nOut + j], inputR the same at tInR; outputL and
  // outputR at tOutL / tOutR + (b d + a) nIn + i.  Null otherwise.
  const int *ticks;
  long long tInR, tOutL, tOutR;
};
__device__ __forceinline__ int fmp_inputL(const Geom &g, int b, int a, int j) {
  return g.ticks[((long long)b * g.d + a) * g.nOut + j];
}
__device__ __forceinline__ int fmp_inputR(const Geom &g, int b, int a, int j) {
  return g.ticks[g.tInR + ((long long)b * g.d + a) * g.nOut + j];
}

struct GridView {
  Slot *table; // look-ups by coordinate: a hash table, or for small batches
  int *dense;  // the row of every site of the field (valid where the mask is set)
  unsigned shift, mask;
  unsigned long long *bits;
  const unsigned *prefix;
  const int *rankRow; // row of the site at each position of iteration order
  const int *bg;
  long long vol;
  int n, d, batch;
};

// A count the host may not know yet: an upper bound, and where the real value
// is (device memory written by an earlier kernel of the same stream); live ==
// null means the bound is exact.
struct Count {
  long long bound;
  const long long *live;
};
__device__ __forceinline__ long long count_now(const Count &c) {
  if (!c.live)
    return c.bound;
  const long long v = *c.live;
  return v < c.bound ? v : c.bound;
}
// The block a workgroup stands for.  Workgroups are dealt to the 8 XCDs
// round-robin and every XCD has an L2 of its own; the kernels that walk
// entries or rows in key order read, for each, the mask rows and rank rows of
// its neighbourhood, which their neighbours in the walk read too.  So the
// blocks that hold real work (the first nLive) are dealt out in runs of
// XCD_RUN consecutive blocks to one XCD, run after run round the XCDs: the
// neighbours meet in one L2, and what the eight XCDs write at any moment still
// lies close together.  The last, incomplete round of runs and the blocks
// without work keep their own numbers.  A permutation of the grid, which must
// be a multiple of 8 blocks.
#define XCD_RUN 32
__device__ __forceinline__ long long xcd_contiguous_block(long long nLive) {
  const long long b = blockIdx.x;
  const long long whole = nLive / (8 * XCD_RUN) * (8 * XCD_RUN);
  if (b >= whole)
    return b;
  const long long turn = b / 8, xcd = b % 8;
  return ((turn / XCD_RUN) * 8 + xcd) * XCD_RUN + turn % XCD_RUN;
}
// (host side: the grid such kernels are launched with)
static inline unsigned xcd_grid(long long blocks) {
  return (unsigned)((blocks + 7) / 8 * 8);
}
// per-grids device record
enum { META_SITES = 0, META_ACTIVE = 1, META_OVERFLOW = 2, META_WIDTH = 3 };

struct scn_grids {
  int batch = 0, d = 0, n = 0;
  long long vol = 0;
  long long nActive = 0;
  int nSites = 0;
  unsigned log2cap = 0;
  size_t nWords = 0;
  // What is current beside the entry list: the occupancy mask (indexValid;
  // false for grids a chain of recorded plans produced: those hold the entry
  // list, backgroundCol and the counts, and the rest is built from them on
  // demand), its rank prefix (rankValid), the rows by rank (rankRowValid) and
  // the hash table (tableValid).  Rule books are built from mask, prefix and
  // rows by rank; look-ups by coordinate (scn_grids_find, the source of a
  // chain of recorded plans) go through a dense row table when the batch's
  // fields are small enough for one (SCN_DENSE_MAX_SITES, filled as the grids
  // are built) and through a hash table otherwise (filled on demand).
  bool rankValid = false;
  bool rankRowValid = false;
  bool tableValid = false;
  bool indexValid = true;
  bool chained = false; // plan and rules came from a chain of recorded plans
  long long seenSample = 0; // most active sites one sample has had (chained plans)
  // how much of table / bits is known to be empty right now (scn_grids_clear_many)
  size_t cleanSlots = 0, cleanWords = 0;
  // Deferred counts: while pending, nActive / nSites / termS hold upper bounds
  // and the real values are in meta (device) and on their way to the pinned
  // slot; seen* are the largest values this object has ever held, from which
  // the next bounds are derived.
  bool pending = false;
  int pinnedSlot = -1;
  long long seenRows = 0, seenActive = 0, seenWidth = 0;
  DevBuf<long long> meta; // META_* words
  DevBuf<Slot> table;
  DevBuf<int> dense;
  DevBuf<unsigned long long> bits;
  DevBuf<unsigned> prefix;
  DevBuf<int> rankRow;
  DevBuf<long long> ekey;
  DevBuf<int> erow;
  DevBuf<int> bg;
  DevBuf<unsigned> scanTmp;
  // state of the plan that produced this object
  int planKind = PLAN_NONE;
  const scn_grids *planIn = nullptr;
  Geom geom;
  long long termS = 0;
  DevBuf<long long> siteKey; // per output row: sample and coordinates (pack_row_site), or -1 - sample for a background row
  DevBuf<unsigned> cnt, base;
  DevBuf<unsigned long long> ownMask;
  DevBuf<unsigned> rankOf;
  DevBuf<int> bgBefore;
  DevBuf<unsigned> sampleStart;
  DevBuf<int> invOrd;
  DevBuf<int> ticks; // region tables of a fractional max-pooling plan
  // scratch for download
  DevBuf<int> dlSample, dlRow;
  DevBuf<long long> dlKey;
};

// ---------------------------------------------------------------- device

__device__ __forceinline__ unsigned hash_slot(long long p, unsigned shift) {
  return (unsigned)(((unsigned long long)p * 0x9E3779B97F4A7C15ull) >> shift);
}

__device__ __forceinline__ void hash_insert(Slot *t, unsigned shift,
                                            unsigned mask, long long p,
                                            int row) {
  unsigned s = hash_slot(p, shift);
  for (;;) {
    unsigned long long prev =
        atomicCAS((unsigned long long *)&t[s].key,
                  (unsigned long long)SLOT_EMPTY, (unsigned long long)p);
    if (prev == (unsigned long long)SLOT_EMPTY ||
        prev == (unsigned long long)p) {
      t[s].row = row;
      return;
    }
    s = (s + 1) & mask;
  }
}

// sites of a batch (batch * spatialSize^d) up to which look-ups by coordinate
// use a dense row table instead of a hash table
#define SCN_DENSE_MAX_SITES (1ll << 24)

__device__ __forceinline__ int hash_find(const Slot *t, unsigned shift,
                                         unsigned mask, long long p) {
  unsigned s = hash_slot(p, shift);
  for (;;) {
    const int4 v = *reinterpret_cast<const int4 *>(&t[s]); // one 128-bit load
    long long k = ((long long)v.y << 32) | (unsigned)v.x;
    if (k == p)
      return v.z;
    if (k == SLOT_EMPTY)
      return -1;
    s = (s + 1) & mask;
  }
}

// consecutive mask words fetched as one request (global memory takes 16-byte
// loads at any 4-byte boundary)
struct __attribute__((packed, aligned(8))) Words2 {
  unsigned long long a, b;
};
struct __attribute__((packed, aligned(4))) Dwords2 {
  unsigned a, b;
};

// row of the site at packed position p, -1 when it is not active
__device__ __forceinline__ int grid_row(const GridView &g, long long p) {
  if (g.dense)
    return (g.bits[p >> 6] >> (p & 63)) & 1ull ? g.dense[p] : -1;
  return hash_find(g.table, g.shift, g.mask, p);
}

// `len` (1..32) mask bits starting at bit position p
__device__ __forceinline__ unsigned get_bits(const unsigned long long *bits,
                                             long long p, int len) {
  long long w = p >> 6;
  int sh = (int)(p & 63);
  unsigned long long lo = bits[w] >> sh;
  if (sh + len > 64)
    lo |= bits[w + 1] << (64 - sh);
  unsigned m = (len >= 32) ? 0xFFFFFFFFu : ((1u << len) - 1u);
  return (unsigned)lo & m;
}

__device__ __forceinline__ unsigned rank_of(const GridView &g, long long p) {
  const long long w = p >> 6;
  const unsigned long long word = g.bits[w];
  // the set bits below p in its word, counted in 32-bit halves (64-bit shifts
  // by a variable run at a quarter of the rate)
  const unsigned d0 = (unsigned)word, d1 = (unsigned)(word >> 32);
  const unsigned below = (1u << ((unsigned)p & 31u)) - 1u;
  const unsigned n = p & 32 ? (unsigned)__popc(d0) + (unsigned)__popc(d1 & below)
                            : (unsigned)__popc(d0 & below);
  return g.prefix[w] + n;
}

__device__ __forceinline__ int sq_outputL(int size, int stride, int i) {
  int v = (i - size + stride) / stride; // truncation toward zero, as in C
  return v > 0 ? v : 0;
}
__device__ __forceinline__ int sq_outputR(int stride, int nOut, int i) {
  int v = i / stride + 1;
  return v < nOut ? v : nOut;
}

template <int D>
__device__ __forceinline__ void decode_key(long long key, int n, int *c) {
#pragma unroll
  for (int a = D - 1; a >= 0; --a) {
    c[a] = (int)(key % n);
    key /= n;
  }
}
template <int D>
__device__ __forceinline__ long long encode_key(const int *c, int n) {
  long long k = 0;
#pragma unroll
  for (int a = 0; a < D; ++a)
    k = k * n + c[a];
  return k;
}

// Is any site of the window with origin w active at a window offset that
// precedes offset a (row-major)?  The window has ext[axis] sites along each
// axis (all equal for the regular regions).
template <int D>
__device__ __forceinline__ bool any_before(const unsigned long long *bits,
                                           long long sampleBase, int nIn,
                                           const int *ext, const int *w,
                                           const int *a) {
  if (D == 1) {
    return a[0] > 0 && get_bits(bits, sampleBase + w[0], a[0]) != 0;
  } else if (D == 2) {
    for (int q0 = 0; q0 < a[0]; ++q0)
      if (get_bits(bits, sampleBase + (long long)(w[0] + q0) * nIn + w[1], ext[1]))
        return true;
    return a[1] > 0 &&
           get_bits(bits, sampleBase + (long long)(w[0] + a[0]) * nIn + w[1],
                    a[1]) != 0;
  } else {
    for (int q0 = 0; q0 <= a[0]; ++q0) {
      int q1max = (q0 < a[0]) ? ext[1] : a[1];
      for (int q1 = 0; q1 < q1max; ++q1)
        if (get_bits(bits,
                     sampleBase +
                         ((long long)(w[0] + q0) * nIn + (w[1] + q1)) * nIn +
                         w[2],
                     ext[2]))
          return true;
    }
    return a[2] > 0 &&
           get_bits(bits,
                    sampleBase +
                        ((long long)(w[0] + a[0]) * nIn + (w[1] + a[1])) * nIn +
                        w[2],
                    a[2]) != 0;
  }
}

// number of active sites in the window; TRI counts only offsets with
// coordinate sum < size
template <int D, bool TRI>
__device__ __forceinline__ int count_active(const unsigned long long *bits,
                                            long long sampleBase, int nIn,
                                            int size, const int *w) {
  int c = 0;
  if (D == 1) {
    c = __popc(get_bits(bits, sampleBase + w[0], size));
  } else if (D == 2) {
    for (int q0 = 0; q0 < size; ++q0) {
      int len = TRI ? size - q0 : size;
      c += __popc(get_bits(bits, sampleBase + (long long)(w[0] + q0) * nIn + w[1], len));
    }
  } else {
    for (int q0 = 0; q0 < size; ++q0) {
      int q1n = TRI ? size - q0 : size;
      for (int q1 = 0; q1 < q1n; ++q1) {
        int len = TRI ? size - q0 - q1 : size;
        c += __popc(get_bits(
            bits,
            sampleBase + ((long long)(w[0] + q0) * nIn + (w[1] + q1)) * nIn + w[2],
            len));
      }
    }
  }
  return c;
}

// The box [lo, hi) of output sites whose window holds the input site i
// (Regions.cu:13-29), or for valid mode the single site (i0-1, i1-1) when
// 1 <= i <= nOut on each axis (Regions.cu:693-697).  False when empty.
template <int D>
__device__ __forceinline__ bool cand_box(const Geom &g, int b, const int *i,
                                         int *lo, int *hi) {
  if (g.mode == MODE_SQ_FMP) { // tables (Regions.cu:143-150)
#pragma unroll
    for (int a = 0; a < D; ++a) {
      const long long t = ((long long)b * g.d + a) * g.nIn + i[a];
      lo[a] = g.ticks[g.tOutL + t];
      hi[a] = g.ticks[g.tOutR + t];
      if (lo[a] >= hi[a])
        return false;
    }
  } else if (g.mode == MODE_SQ_VALID) {
#pragma unroll
    for (int a = 0; a < D; ++a) {
      if (i[a] < 1 || i[a] > g.nOut)
        return false;
      lo[a] = i[a] - 1;
      hi[a] = i[a];
    }
  } else {
#pragma unroll
    for (int a = 0; a < D; ++a) {
      lo[a] = sq_outputL(g.size, g.stride, i[a]);
      hi[a] = sq_outputR(g.stride, g.nOut, i[a]);
      if (lo[a] >= hi[a])
        return false;
    }
  }
  return true;
}

// Does input site i of sample b own candidate output j?  (the active input
// with the smallest key in j's window owns it; Min modes also need enough
// active inputs; the triangular lattice only has outputs with sum(j) < nOut)
template <int D>
__device__ __forceinline__ bool owns(const GridView &in, const Geom &g, int b,
                                     long long sampleBase, const int *i,
                                     const int *j) {
  if (g.mode == MODE_TRI_NOMIN || g.mode == MODE_TRI_MIN) {
    int sum = 0;
#pragma unroll
    for (int a = 0; a < D; ++a)
      sum += j[a];
    if (sum >= g.nOut) // Regions.cu:874,900
      return false;
  }
  if (g.mode == MODE_SQ_VALID)
    return true;
  int w[D], off[D], ext[D];
  if (g.mode == MODE_SQ_FMP) {
#pragma unroll
    for (int a = 0; a < D; ++a) {
      w[a] = fmp_inputL(g, b, a, j[a]);
      ext[a] = fmp_inputR(g, b, a, j[a]) - w[a];
      off[a] = i[a] - w[a];
    }
  } else {
#pragma unroll
    for (int a = 0; a < D; ++a) {
      w[a] = j[a] * g.stride;
      ext[a] = g.size;
      off[a] = i[a] - w[a];
    }
  }
  if (any_before<D>(in.bits, sampleBase, g.nIn, ext, w, off))
    return false;
  if (g.mode == MODE_SQ_MIN)
    return count_active<D, false>(in.bits, sampleBase, g.nIn, g.size, w) >=
           g.minActive;
  if (g.mode == MODE_TRI_MIN)
    return count_active<D, true>(in.bits, sampleBase, g.nIn, g.size, w) >=
           g.minActive;
  return true;
}

// Visits, in ascending output key, the output sites owned by the input site
// with coordinates i of sample b; f(outKey, c) is called for each, c being the
// position of the site among the candidates of the box.
template <int D, typename F>
__device__ __forceinline__ void for_each_owned(const GridView &in,
                                               const Geom &g, int b,
                                               const int *i, F f) {
  int lo[D], hi[D];
  if (!cand_box<D>(g, b, i, lo, hi))
    return;
  const long long sampleBase = (long long)b * g.volIn;
  int j[D];
#pragma unroll
  for (int a = 0; a < D; ++a)
    j[a] = lo[a];
  for (int c = 0;; ++c) {
    if (owns<D>(in, g, b, sampleBase, i, j))
      f(encode_key<D>(j, g.nOut), c);
    // odometer, last axis fastest
    int a = D - 1;
    for (; a >= 0; --a) {
      if (++j[a] < hi[a])
        break;
      j[a] = lo[a];
    }
    if (a < 0)
      break;
  }
}


// x / d for x d < 2^32, magic = floor(2^32 / d) + 1 (d >= 2)
__device__ __forceinline__ unsigned div_magic(unsigned x, unsigned d, unsigned magic) {
  return d == 1 ? x : __umulhi(x, magic);
}


// `len` (<= 32) mask bits of the row with leading coordinates lead[0 .. D-2],
// columns c0 .. c0 + len - 1; sites outside the field read as inactive.  Both
// words are always fetched (the mask has a spare word), so that a lane's reads
// do not wait for one another.  The field starts at bit `base` of the mask
// (Pos: unsigned for a sample's mask in LDS, long long for a batch's in HBM).
template <int D, typename Pos>
__device__ __forceinline__ unsigned row_bits(const unsigned long long *bits,
                                             Pos base, const int *lead, int c0,
                                             int len, int n) {
  bool inside = true;
  Pos p = 0;
#pragma unroll
  for (int q = 0; q < D - 1; ++q) {
    inside = inside && (unsigned)lead[q] < (unsigned)n;
    p = p * (Pos)n + (Pos)lead[q];
  }
  const int lo = c0 > 0 ? c0 : 0;
  const int hi = c0 + len < n ? c0 + len : n;
  p = p * (Pos)n + (Pos)lo;
  if (!inside || hi <= lo)
    p = 0; // any valid address; the result is masked away
  p += base;
  // the two 32-bit words at the 4-byte boundary below p in one request, and a
  // funnel shift (64-bit shifts by a variable run at a quarter of the rate)
  Dwords2 ww;
  __builtin_memcpy(&ww, reinterpret_cast<const unsigned *>(bits) + (p >> 5), sizeof(ww));
  const unsigned v = __builtin_amdgcn_alignbit(ww.b, ww.a, (unsigned)p & 31u);
  const int m = hi - lo;
  unsigned r = v & (m >= 32 ? 0xFFFFFFFFu : ((1u << (m > 0 ? m : 0)) - 1u));
  r = (!inside || hi <= lo) ? 0u : r;
  return r << (lo - c0 > 0 ? lo - c0 : 0);
}

// `len` (<= 32) mask bits from bit position p on, no questions asked
template <typename Pos>
__device__ __forceinline__ unsigned bits_at(const unsigned long long *bits, Pos p, int len) {
  Dwords2 ww;
  __builtin_memcpy(&ww, reinterpret_cast<const unsigned *>(bits) + (p >> 5), sizeof(ww));
  const unsigned v = __builtin_amdgcn_alignbit(ww.b, ww.a, (unsigned)p & 31u);
  return v & (len >= 32 ? 0xFFFFFFFFu : ((1u << len) - 1u));
}

// Square regions without a minimum (Regions.cu:528-653), window side S: which
// of the outputs whose window holds input site i is first touched by i, i.e.
// has no active site before i in its window (row-major).  All mask reads of a
// site are issued together -- the S rows (2-D) or S (2S - 1) rows (3-D) of its
// neighbourhood -- and every candidate is then decided in registers.  Bit c of
// the result stands for candidate c of the box [lo, hi) in ascending key;
// f(j) is called for the owned ones.
// The same for windows that do not overlap (stride == S, the usual max-pooling
// geometry): the one output whose window holds site i is owned by i when no
// site of that window before i is active.  The window's S^(D-1) rows are
// requested together.
template <int D, int S, typename Pos, typename F>
__device__ __forceinline__ unsigned
owned_disjoint(const unsigned long long *bits, Pos base, const int *i,
               const int *lo, const int *hi, int nIn, unsigned magicStride,
               F f) {
  int j[D], a[D];
  bool ok = true;
#pragma unroll
  for (int q = 0; q < D; ++q) {
    j[q] = (int)div_magic((unsigned)i[q], (unsigned)S, magicStride);
    a[q] = i[q] - j[q] * S;
    ok = ok && j[q] >= lo[q] && j[q] < hi[q];
  }
  unsigned before = 0;
  if (D == 2) {
#pragma unroll
    for (int r = 0; r < S; ++r) {
      const int lead[1] = {j[0] * S + r};
      const unsigned row = row_bits<2>(bits, base, lead, j[1] * S, S, nIn);
      before |= r < a[0] ? row : (r == a[0] ? row & ((1u << a[1]) - 1u) : 0u);
    }
  } else {
#pragma unroll
    for (int pl = 0; pl < S; ++pl)
#pragma unroll
      for (int r = 0; r < S; ++r) {
        const int lead[2] = {j[0] * S + pl, j[1] * S + r};
        const unsigned row = row_bits<3>(bits, base, lead, j[D - 1] * S, S, nIn);
        const bool whole = pl < a[0] || (pl == a[0] && r < a[1]);
        const bool part = pl == a[0] && r == a[1];
        before |= whole ? row : (part ? row & ((1u << a[D - 1]) - 1u) : 0u);
      }
  }
  if (!ok || before != 0)
    return 0u;
  f(j);
  return 1u; // the box has this one candidate
}

template <int D, int S, typename Pos, typename F>
__device__ __forceinline__ unsigned
owned_nomin(const unsigned long long *bits, Pos base, const int *i,
            const int *lo, const int *hi, int nIn, int stride,
            unsigned magicStride, F f) {
  static_assert(D == 2 || D == 3, "two or three dimensions");
  if (stride == S)
    return owned_disjoint<D, S>(bits, base, i, lo, hi, nIn, magicStride, f);
  constexpr int W = 2 * S - 1;
  constexpr unsigned FULL = (1u << S) - 1u;
  unsigned m = 0;
  // a site whose whole neighbourhood lies inside the field (nearly all) needs
  // no clipping: its rows are at fixed distances from the first
  bool interior = i[0] >= S - 1;
#pragma unroll
  for (int a = 1; a < D; ++a)
    interior = interior && i[a] >= S - 1 && i[a] + S - 1 < nIn;
  if (D == 2) {
    unsigned nb[S];
    if (interior) {
      const Pos p0 = base + (Pos)(i[0] - (S - 1)) * (Pos)nIn + (Pos)(i[1] - (S - 1));
#pragma unroll
      for (int r = 0; r < S; ++r)
        nb[r] = bits_at(bits, p0 + (Pos)(r * nIn), W);
    } else {
#pragma unroll
      for (int r = 0; r < S; ++r) {
        const int lead[1] = {i[0] - (S - 1) + r};
        nb[r] = row_bits<2>(bits, base, lead, i[1] - (S - 1), W, nIn);
      }
    }
#pragma unroll
    for (int a0 = 0; a0 < S; ++a0) {
      const int d0 = i[0] - a0;
      const int j0 = (int)div_magic((unsigned)(d0 > 0 ? d0 : 0), (unsigned)stride, magicStride);
      const bool ok0 = d0 >= 0 && j0 * stride == d0 && j0 >= lo[0] && j0 < hi[0];
      unsigned above = 0;
#pragma unroll
      for (int r = S - 1 - a0; r < S - 1; ++r)
        above |= nb[r];
#pragma unroll
      for (int a1 = 0; a1 < S; ++a1) {
        const int d1 = i[1] - a1;
        const int j1 = (int)div_magic((unsigned)(d1 > 0 ? d1 : 0), (unsigned)stride, magicStride);
        const bool ok1 = d1 >= 0 && j1 * stride == d1 && j1 >= lo[1] && j1 < hi[1];
        const unsigned before = (above & (FULL << (S - 1 - a1))) |
                                (nb[S - 1] & (((1u << a1) - 1u) << (S - 1 - a1)));
        if (ok0 && ok1 && before == 0) {
          const int j[2] = {j0, j1};
          m |= 1u << ((j0 - lo[0]) * (hi[1] - lo[1]) + (j1 - lo[1]));
          f(j);
        }
      }
    }
  } else {
    unsigned nb[S][W];
    if (interior) {
      const Pos plane = (Pos)nIn * (Pos)nIn;
      const Pos p0 = base + (Pos)(i[0] - (S - 1)) * plane + (Pos)(i[1] - (S - 1)) * (Pos)nIn +
                     (Pos)(i[2] - (S - 1));
#pragma unroll
      for (int pl = 0; pl < S; ++pl)
#pragma unroll
        for (int r = 0; r < W; ++r)
          nb[pl][r] = bits_at(bits, p0 + (Pos)pl * plane + (Pos)(r * nIn), W);
    } else {
#pragma unroll
      for (int pl = 0; pl < S; ++pl)
#pragma unroll
        for (int r = 0; r < W; ++r) {
          const int lead[2] = {i[0] - (S - 1) + pl, i[1] - (S - 1) + r};
          nb[pl][r] = row_bits<3>(bits, base, lead, i[2] - (S - 1), W, nIn);
        }
    }
#pragma unroll
    for (int a0 = 0; a0 < S; ++a0) {
      const int d0 = i[0] - a0;
      const int j0 = (int)div_magic((unsigned)(d0 > 0 ? d0 : 0), (unsigned)stride, magicStride);
      const bool ok0 = d0 >= 0 && j0 * stride == d0 && j0 >= lo[0] && j0 < hi[0];
#pragma unroll
      for (int a1 = 0; a1 < S; ++a1) {
        const int d1 = i[1] - a1;
        const int j1 = (int)div_magic((unsigned)(d1 > 0 ? d1 : 0), (unsigned)stride, magicStride);
        const bool ok1 = d1 >= 0 && j1 * stride == d1 && j1 >= lo[1] && j1 < hi[1];
        // whole planes before the site's, then whole rows of its plane
        unsigned above = 0;
#pragma unroll
        for (int pl = S - 1 - a0; pl < S - 1; ++pl)
#pragma unroll
          for (int q1 = 0; q1 < S; ++q1)
            above |= nb[pl][S - 1 - a1 + q1];
#pragma unroll
        for (int q1 = 0; q1 < a1; ++q1)
          above |= nb[S - 1][S - 1 - a1 + q1];
#pragma unroll
        for (int a2 = 0; a2 < S; ++a2) {
          const int d2 = i[2] - a2;
          const int j2 = (int)div_magic((unsigned)(d2 > 0 ? d2 : 0), (unsigned)stride, magicStride);
          const bool ok2 = d2 >= 0 && j2 * stride == d2 && j2 >= lo[2] && j2 < hi[2];
          const unsigned before =
              (above & (FULL << (S - 1 - a2))) |
              (nb[S - 1][S - 1] & (((1u << a2) - 1u) << (S - 1 - a2)));
          if (ok0 && ok1 && ok2 && before == 0) {
            const int j[3] = {j0, j1, j2};
            m |= 1u << (((j0 - lo[0]) * (hi[1] - lo[1]) + (j1 - lo[1])) *
                            (hi[2] - lo[2]) +
                        (j2 - lo[2]));
            f(j);
          }
        }
      }
    }
  }
  return m;
}


// What a rule-book plan keeps per output row: sample and coordinates in fixed
// bit fields, so that the lanes that fill the rule rows shift instead of
// dividing.  40 bits of coordinates (40, 20 or 13 an axis), the sample above.
template <int D> struct RowSite {
  static constexpr int AX = D == 1 ? 40 : (D == 2 ? 20 : 13);
};
template <int D>
__device__ __forceinline__ long long pack_row_site(int b, const int *j) {
  unsigned long long v = (unsigned long long)b;
#pragma unroll
  for (int a = 0; a < D; ++a)
    v = (v << RowSite<D>::AX) | (unsigned long long)(unsigned)j[a];
  return (long long)v;
}
template <int D>
__device__ __forceinline__ int unpack_row_site(long long sk, int *j) {
  unsigned long long v = (unsigned long long)sk;
#pragma unroll
  for (int a = D - 1; a >= 0; --a) {
    j[a] = (int)(v & ((1ull << RowSite<D>::AX) - 1ull));
    v >>= RowSite<D>::AX;
  }
  return (int)v;
}

// sample and coordinates of the packed position p = sample * vol + key; the
// key is taken apart in 32-bit arithmetic when the field allows it
template <int D>
__device__ __forceinline__ int split_site(long long p, long long vol, int n,
                                          int *c) {
  // (64-bit division is a long routine: most batches' masks have fewer than 2^32 bits)
  const int b = ((unsigned long long)(p | vol) >> 32) == 0 ? (int)((unsigned)p / (unsigned)vol)
                                                           : (int)(p / vol);
  const long long key = p - (long long)b * vol;
  if (vol < (1ll << 31)) {
    unsigned k = (unsigned)key;
#pragma unroll
    for (int a = D - 1; a >= 0; --a) {
      const unsigned up = k / (unsigned)n;
      c[a] = (int)(k - up * (unsigned)n);
      k = up;
    }
  } else {
    decode_key<D>(key, n, c);
  }
  return b;
}

// ---- host helpers shared by scn_grids.hip and scn_chain.hip
GridView view_of(const scn_grids *g);
long long grow_bound(long long seen, long long slack, long long cap);
void mark_pending(scn_ctx *ctx, scn_grids *g, int slot);
// fills the hash table of grids that do not have it yet (scn_grids.hip)
int scn_grids_ensure_table(scn_ctx *ctx, scn_grids *g);

// Chains of recorded plans (scn_chain.hip).  The record functions set *taken
// when the call joined the chain being recorded; otherwise the caller runs it
// the ordinary way (after scn_chain_flush).
int scn_chain_record_regions(scn_ctx *ctx, scn_grids *in, scn_grids *out,
                             const Geom &g, long long fullSize,
                             long long maxCand, int64_t *nOutSites,
                             bool *taken);
int scn_chain_record_terminal(scn_ctx *ctx, scn_grids *in, scn_grids *out,
                              int64_t *ruleWidth, bool *taken);
int scn_chain_record_fill(scn_ctx *ctx, const scn_grids *in, scn_grids *out,
                          int32_t *d_rules, int64_t capacity, bool *taken);
void scn_chain_settled(scn_ctx *ctx, scn_grids *g, long long sampleMax,
                       bool overflowed);
