// Rule books of a whole net from the output side (square windows without a
// minimum, Regions.cu:528-653), one sample at a time.
//
// gridRules walks the input map in ascending key and creates an output site
// the first time one of its window's inputs is met (Regions.cu:557-576).  So an
// output site exists iff its window holds an active input; it is *owned* by
// the first active input of its window in row-major order; and the outputs get
// their rows in the order (owner's key, output's key).  Everything a layer's
// rule book needs therefore follows from occupancy masks alone:
//
//   pass A  the masks of all layers of the sample: each is its input mask
//           OR-ed over the window and thinned by the stride, up to 64 sites of
//           a row at a time (pyr_dilate_pieces), plus a popcount prefix per
//           word (the rank of a site = its position in iteration order);
//   pass B  per output site, in five sweeps over ALL layers at once (or, for a
//           sample too large for that, over as many consecutive layers as
//           the LDS holds, window after window) with one barrier between
//           them: enumerate the sites by rank; find each
//           site's owner (first set bit of its window) and mark, in the owner's
//           16-bit ownership mask, which of its candidates this is (an LDS
//           atomic OR); prefix sums of the owned counts per layer; a site's row
//           = its owner's base + how many later candidates the owner also owns
//           (a later candidate is an earlier output); and the rule rows, which
//           look the input sites' rows up by rank.
//
// The code below is the per-lane body of every sweep.  It is written against
// plain pointers ("lds" is just memory) so that the same text compiles for the
// device (scn_chain.hip) and for the host, where a harness runs the lanes one
// after the other with the barriers between sweeps (tests/chain_cpu_harness.cpp).
#pragma once
#include <stdint.h>
#include <type_traits>

#if defined(__HIPCC__)
#define PYR_FN __host__ __device__ __forceinline__
#else
#define PYR_FN static inline
#endif

#define PYR_MAX_LEVELS 24  // recorded layers of a chain
#define PYR_HDR_BYTES 5248 // pass B's header and level tables in LDS
#define PYR_CUBE_MAX 16    // ownership masks are 16 bits
#define PYR_ROWS_MAX 65000 // rows of one sample at one layer (16-bit rows)
enum { PYR_REGIONS = 0, PYR_TERMINAL = 1 };

typedef unsigned long long pyr_u64;

// Level 0 is the source grid; level l >= 1 is the output of recorded layer l
// (input: level l - 1).  A terminal layer can only be the last one.
struct PyrLevel {
  int kind;
  int nIn, nOut, size, stride, width; // width = size^d
  int words;   // 64-bit words of this level's mask (two spare words follow)
  int maskOff; // of the mask in a sample's pyramid, in 64-bit words
  unsigned magicN, magicS; // floor(2^32 / nOut) + 1, floor(2^32 / size) + 1
  unsigned seg;    // output sites a piece of the dilation covers (the last piece of a row: what is left)
  long long volOut, fullSize;
  // where the layer's results go
  int *rules;
  long long capacity;
  long long *ekey;
  int *erow;
  int *bg;
  long long *meta;
  long long boundRows, boundActive;
  int slot;
  unsigned segs, magicSegs; // pieces in a row of the output field, floor(2^32 / segs) + 1
};

struct PyrArgs {
  int nLevels; // recorded layers: levels 1 .. nLevels
  int nMasks;  // levels with a mask: 0 .. nMasks - 1 (the terminal layer has none)
  int batch, d;
  const int *dense; // row of every site of the source field, or
  const void *table; // the source's hash table (device builds only)
  unsigned shift, mask;
  const pyr_u64 *bits; // the source batch's occupancy mask
  const int *bg;       // and background rows
  int maskWords;       // 64-bit words of all masks of a sample, spares included
  int pyrStride;       // 64-bit words a sample takes in `pyramid`: masks, then 16-bit prefixes
  pyr_u64 *pyramid;
  int *counts; // [nLevels + 1][batch][2]: sites, has a background row
  unsigned long long *flag;
  unsigned long long ticket;
  long long *scalars;
  const long long *badSites;
  int ldsBytesB; // dynamic LDS pass B is launched with
  PyrLevel lv[PYR_MAX_LEVELS + 1];
};

// ---------------------------------------------------------------- bit helpers
PYR_FN int pyr_popc64(pyr_u64 x) { return __builtin_popcountll(x); }
PYR_FN int pyr_popc32(unsigned x) { return __builtin_popcount(x); }
PYR_FN int pyr_ctz64(pyr_u64 x) { return __builtin_ctzll(x); }
PYR_FN int pyr_ctz32(unsigned x) { return __builtin_ctz(x); }
PYR_FN unsigned pyr_mulhi(unsigned a, unsigned b) {
  return (unsigned)(((pyr_u64)a * (pyr_u64)b) >> 32);
}
// x / d for x d < 2^32, magic = floor(2^32 / d) + 1
PYR_FN unsigned pyr_div(unsigned x, unsigned d, unsigned magic) {
  return d == 1 ? x : pyr_mulhi(x, magic);
}
PYR_FN pyr_u64 pyr_even_bits(pyr_u64 x) {
  x &= 0x5555555555555555ull;
  x = (x | (x >> 1)) & 0x3333333333333333ull;
  x = (x | (x >> 2)) & 0x0F0F0F0F0F0F0F0Full;
  x = (x | (x >> 4)) & 0x00FF00FF00FF00FFull;
  x = (x | (x >> 8)) & 0x0000FFFF0000FFFFull;
  x = (x | (x >> 16)) & 0x00000000FFFFFFFFull;
  return x;
}
// Bits that straddle words are taken out in 32-bit pieces: (hi:lo) >> s for s
// below 32 is one instruction on the device, where a 64-bit shift by a
// variable amount issues at a quarter of the rate of a 32-bit operation.
PYR_FN unsigned pyr_alignbit(unsigned hi, unsigned lo, unsigned s) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_alignbit(hi, lo, s);
#else
  s &= 31u;
  return s ? (lo >> s) | (hi << (32u - s)) : lo;
#endif
}
struct PyrBits128 {
  unsigned w[4];
};
// 128 mask bits from position p on, as four 32-bit words (the mask has two spare words)
PYR_FN PyrBits128 pyr_bits128(const pyr_u64 *bits, unsigned p) {
  unsigned d[5];
  __builtin_memcpy(d, reinterpret_cast<const unsigned *>(bits) + (p >> 5), sizeof(d));
  PyrBits128 r;
  for (int i = 0; i < 4; ++i)
    r.w[i] = pyr_alignbit(d[i + 1], d[i], p & 31u);
  return r;
}
// `len` (<= 16) mask bits from position p on
PYR_FN unsigned pyr_bits(const pyr_u64 *bits, unsigned p, int len) {
  unsigned d[2];
  __builtin_memcpy(d, reinterpret_cast<const unsigned *>(bits) + (p >> 5), sizeof(d));
  return pyr_alignbit(d[1], d[0], p & 31u) & ((1u << len) - 1u);
}
PYR_FN unsigned pyr_rank(const pyr_u64 *bits, const unsigned short *pref, unsigned p) {
  const unsigned w = p >> 6;
  const pyr_u64 word = bits[w];
  const unsigned d0 = (unsigned)word, d1 = (unsigned)(word >> 32);
  const unsigned below = (1u << (p & 31u)) - 1u;
  const int n = p & 32u ? pyr_popc32(d0) + pyr_popc32(d1 & below) : pyr_popc32(d0 & below);
  return pref[w] + (unsigned)n;
}

// Sites travel as packed coordinates: 30 bits in one dimension, 15 bits an axis
// in two, 10 in three.
template <int D> struct PyrPacked {
  static constexpr int BITS = D == 1 ? 30 : (D == 2 ? 15 : 10);
  static constexpr unsigned MASK = (1u << BITS) - 1u;
};
template <int D> PYR_FN unsigned pyr_pack(const int *c) {
  unsigned v = 0;
#if defined(__HIPCC__)
#pragma unroll
#endif
  for (int q = 0; q < D; ++q)
    v |= (unsigned)c[q] << (q * PyrPacked<D>::BITS);
  return v;
}
template <int D> PYR_FN void pyr_unpack(unsigned v, int *c) {
#if defined(__HIPCC__)
#pragma unroll
#endif
  for (int q = 0; q < D; ++q)
    c[q] = (int)((v >> (q * PyrPacked<D>::BITS)) & PyrPacked<D>::MASK);
}
template <int D> PYR_FN unsigned pyr_key(const int *c, int n) {
  unsigned k = 0;
#if defined(__HIPCC__)
#pragma unroll
#endif
  for (int q = 0; q < D; ++q)
    k = k * (unsigned)n + (unsigned)c[q];
  return k;
}

// ------------------------------------------------------------------- pass A
// A layer's output mask from its input mask (one sample), a lane per PIECE: a
// run of up to `seg` neighbouring output sites in one row of the output field.
// The piece ORs the size^(D-1) input rows of its windows (128 bits a request),
// ORs `size` shifts of that, keeps every stride-th bit and ORs the result into
// the one or two words of the output mask it falls in (which start as zero).
// (a piece reads (len - 1) stride + size input bits, at most 128, and gives at
// most 64 bits)
PYR_FN unsigned pyr_seg(int size, int stride) {
  const unsigned most = stride <= 1 ? 64u : (unsigned)((128 - size) / stride + 1);
  return most < 64u ? most : 64u;
}
PYR_FN void pyr_set_pieces(PyrLevel &L) {
  L.seg = pyr_seg(L.size, L.stride);
  L.segs = ((unsigned)L.nOut + L.seg - 1u) / L.seg;
  L.magicSegs = (unsigned)((1ull << 32) / (L.segs > 0 ? L.segs : 1u) + 1ull);
}
#if defined(__HIPCC__) && defined(__HIP_DEVICE_COMPILE__)
#define PYR_ATOMIC_OR64(ptr, v) atomicOr(reinterpret_cast<unsigned long long *>(ptr), (unsigned long long)(v))
#else
#define PYR_ATOMIC_OR64(ptr, v) (*(ptr) |= (v))
#endif
// (SIZE, STRIDE: the layer's, when known at compile time; 0: take the arguments)
template <int D, int SIZE, int STRIDE>
PYR_FN void pyr_dilate_pieces(const pyr_u64 *in, pyr_u64 *out, int nIn, int nOut, int size_, int stride_,
                              unsigned magicN, unsigned seg, unsigned segs, unsigned magicSegs, int t, int T) {
  const int size = SIZE ? SIZE : size_;
  const int stride = STRIDE ? STRIDE : stride_;
  unsigned rows = 1;
  for (int q = 0; q < D - 1; ++q)
    rows *= (unsigned)nOut;
  const unsigned pieces = rows * segs;
  for (unsigned p = (unsigned)t; p < pieces; p += (unsigned)T) {
    const unsigned row = pyr_div(p, segs, magicSegs);
    const unsigned jl = (p - row * segs) * seg; // the piece's first site along the last axis
    unsigned len = (unsigned)nOut - jl;
    len = len < seg ? len : seg;
    // (a piece reads (len - 1) stride + size bits; what lies beyond them in
    // the 128 fetched only reaches result bits from len on, cleared below)
    unsigned x[5] = {0u, 0u, 0u, 0u, 0u};
    auto add = [&](unsigned from) {
      const PyrBits128 v = pyr_bits128(in, from);
      for (int i = 0; i < 4; ++i)
        x[i] |= v.w[i];
    };
    if (D == 1) {
      add(jl * (unsigned)stride);
    } else if (D == 2) {
      for (int q0 = 0; q0 < size; ++q0)
        add((row * (unsigned)stride + (unsigned)q0) * (unsigned)nIn + jl * (unsigned)stride);
    } else {
      const unsigned j0 = pyr_div(row, (unsigned)nOut, magicN), j1 = row - j0 * (unsigned)nOut;
      for (int q0 = 0; q0 < size; ++q0)
        for (int q1 = 0; q1 < size; ++q1)
          add(((j0 * (unsigned)stride + (unsigned)q0) * (unsigned)nIn + (j1 * (unsigned)stride + (unsigned)q1)) *
                  (unsigned)nIn +
              jl * (unsigned)stride);
    }
    // bit t: any of the `size` sites from t on
    unsigned y[4] = {x[0], x[1], x[2], x[3]};
    for (int q = 1; q < size; ++q)
      for (int i = 0; i < 4; ++i)
        y[i] |= pyr_alignbit(x[i + 1], x[i], (unsigned)q); // (sides stay below 32)
    const pyr_u64 ylo = (pyr_u64)y[0] | ((pyr_u64)y[1] << 32), yhi = (pyr_u64)y[2] | ((pyr_u64)y[3] << 32);
    pyr_u64 r;
    if (stride == 1) {
      r = ylo;
    } else if (stride == 2) {
      r = pyr_even_bits(ylo) | (pyr_even_bits(yhi) << 32);
    } else {
      r = 0;
      for (unsigned i = 0; i < len; ++i) {
        const unsigned at = i * (unsigned)stride;
        const pyr_u64 bit = at < 64 ? (ylo >> at) : (yhi >> (at - 64));
        r |= (bit & 1ull) << i;
      }
    }
    if (len < 64)
      r &= (1ull << len) - 1ull;
    if (!r)
      continue;
    const unsigned pos = row * (unsigned)nOut + jl, w = pos >> 6, sh = pos & 63u;
    PYR_ATOMIC_OR64(&out[w], r << sh);
    if (sh && (r >> (64u - sh)))
      PYR_ATOMIC_OR64(&out[w + 1], r >> (64u - sh));
  }
}
// The same with the usual windows (2/1, 3/2, 2/2, 3/1) compiled in
template <int D>
PYR_FN void pyr_sweep_dilate(const pyr_u64 *in, pyr_u64 *out, int nIn, int nOut, int size, int stride,
                             unsigned magicN, unsigned seg, unsigned segs, unsigned magicSegs, int t, int T) {
  if (D >= 2 && size == 2 && stride == 1)
    pyr_dilate_pieces<D, 2, 1>(in, out, nIn, nOut, size, stride, magicN, seg, segs, magicSegs, t, T);
  else if (D >= 2 && size == 3 && stride == 2)
    pyr_dilate_pieces<D, 3, 2>(in, out, nIn, nOut, size, stride, magicN, seg, segs, magicSegs, t, T);
  else if (D >= 2 && size == 2 && stride == 2)
    pyr_dilate_pieces<D, 2, 2>(in, out, nIn, nOut, size, stride, magicN, seg, segs, magicSegs, t, T);
  else if (D >= 2 && size == 3 && stride == 1)
    pyr_dilate_pieces<D, 3, 1>(in, out, nIn, nOut, size, stride, magicN, seg, segs, magicSegs, t, T);
  else
    pyr_dilate_pieces<D, 0, 0>(in, out, nIn, nOut, size, stride, magicN, seg, segs, magicSegs, t, T);
}

// Word w of the source mask of sample b: its slice of the batch's mask
PYR_FN pyr_u64 pyr_source_word(const pyr_u64 *bits, long long vol, int b, unsigned w) {
  const long long left = vol - 64ll * w;
  if (left <= 0)
    return 0ull;
  const long long p = (long long)b * vol + 64ll * w;
  const long long gw = p >> 6;
  const int sh = (int)(p & 63);
  pyr_u64 v = bits[gw] >> sh;
  if (sh)
    v |= bits[gw + 1] << (64 - sh);
  if (left < 64)
    v &= (1ull << left) - 1ull;
  return v;
}

// Pass B takes a sample's layers a WINDOW of levels xa .. xb at a time: level
// xa as input only (its rows known: the source's, or from the window before),
// layers xa + 1 .. xb built.  LDS bytes of a window for a sample with n[x]
// sites at level x: per site key (4), row, ownership mask, base (2 each),
// which candidate of its owner it is (1); the input level's batch-global rows
// (4 more); every array padded to 16 bytes
PYR_FN long long pyr_lds_window(const PyrArgs &a, const int *n, int xa, int xb) {
  long long total = 0;
  for (int x = xa; x <= xb; ++x)
    total += n[x];
  return PYR_HDR_BYTES + 8ll * a.pyrStride + 11ll * total + 4ll * n[xa] + 6 * 16;
}
// The window that starts at level xa: as many layers as fit (at least one,
// when there is one)
PYR_FN int pyr_window_end(const PyrArgs &a, const int *n, int xa) {
  int xb = xa + 1 < a.nMasks ? xa + 1 : xa;
  long long total = n[xa] + (xb > xa ? n[xb] : 0);
  const long long fixed = PYR_HDR_BYTES + 8ll * a.pyrStride + 4ll * n[xa] + 6 * 16;
  while (xb + 1 < a.nMasks && fixed + 11ll * (total + n[xb + 1]) <= a.ldsBytesB) {
    total += n[xb + 1];
    ++xb;
  }
  return xb;
}
// Whether every layer of the sample fits by itself
PYR_FN bool pyr_fits(const PyrArgs &a, const int *n) {
  bool fits = pyr_lds_window(a, n, 0, a.nMasks > 1 ? 1 : 0) <= a.ldsBytesB;
  for (int x = 1; x + 1 < a.nMasks; ++x)
    fits = fits && pyr_lds_window(a, n, x, x + 1) <= a.ldsBytesB;
  return fits;
}

// ------------------------------------------------------------------- pass B
struct PyrHdr {
  int n[PYR_MAX_LEVELS + 1];       // this sample's sites at level x
  int hasBg[PYR_MAX_LEVELS + 1];   // and whether it has a background row there
  int siteOff[PYR_MAX_LEVELS + 2]; // where level x of the current window starts in the per-site arrays
  int itemOff[PYR_MAX_LEVELS + 2]; // output sites of the window's layers before layer l (index l)
  int maxAct[PYR_MAX_LEVELS + 1];  // largest sample of the batch at level x
  long long actBefore[PYR_MAX_LEVELS + 1], bgBefore[PYR_MAX_LEVELS + 1]; // of the samples before this one
  long long actAll[PYR_MAX_LEVELS + 1], bgAll[PYR_MAX_LEVELS + 1];
  int over; // some layer outgrew its bounds, or a sample the LDS
  int total; // sites of this sample over the levels of the current window
};
// What the sweeps need of layer l, once per item: kept in LDS (the kernel
// arguments are far away for a lane that wants the entry of ITS layer), the
// geometry in one 16-byte read, the rest as the sweeps come to it.
struct PyrLv {
  int size, stride, nIn, nOut;
  int width;
  unsigned magicS;
  int inMaskOff, inSiteOff; // mask and sites of the layer's input (level l - 1)
  int siteOff, n;           // sites of the layer's output (level l)
  int bgIn;                 // batch-global row of the input's background row, or -1
  int flags;                // PYR_LV_SOURCE: the input is the window's first level, its rows are in srcRow; PYR_LV_TERMINAL
  long long rowBase;        // batch-global row of this sample's row 0 at level l
  long long actBefore;      // entries of the samples before this one at level l
  long long inRowBase;      // rowBase of the input level (0 for the source)
  long long volOut;
  int *rules;
  long long capacity;
  long long *ekey;
  int *erow;
  long long boundActive;
  int *bg;
};
enum { PYR_LV_SOURCE = 1, PYR_LV_TERMINAL = 2 };
// What the enumeration needs of level x (x < nMasks), in one 16-byte read
struct PyrEn {
  int maskOff, nOut;
  unsigned magicN;
  int siteOff;
};
#define PYR_LV_AT 1536
#define PYR_EN_AT (PYR_LV_AT + (PYR_MAX_LEVELS + 1) * (int)sizeof(PyrLv))
static_assert(sizeof(PyrHdr) <= PYR_LV_AT, "header");
static_assert(PYR_EN_AT + (PYR_MAX_LEVELS + 1) * sizeof(PyrEn) <= PYR_HDR_BYTES, "level tables");
static_assert(sizeof(PyrLv) % 16 == 0, "16-byte reads");

// pass B's view of its LDS
struct PyrLds {
  PyrHdr *h;
  PyrLv *lv;             // [nLevels + 1]
  PyrEn *en;             // [nMasks]
  pyr_u64 *masks;        // a.maskWords words
  unsigned short *pref;  // one per mask word
  unsigned *srcRow;      // [n[xa]] batch-global rows of the sites of the window's first level
  unsigned *key;         // [total] packed coordinates by (level, rank)
  unsigned short *row;   // [total] rows, numbered from 0 within sample and level
  unsigned *own;         // [total] 16-bit ownership masks, two to a word
  unsigned short *base;  // [total] rows owned by the sites before, same level
  unsigned char *kOf;    // [total] which of its owner's candidates a site is (the owner's rank waits in `row`)
};
// (total: sites of the window's levels, nFirst: of its first level.  srcRow
// comes first: the rows a window leaves for the next one are written there
// while the old window's arrays, which all lie behind it, are still read)
PYR_FN PyrLds pyr_lds_view(const PyrArgs &a, unsigned char *lds, int total, int nFirst) {
  PyrLds v;
  v.h = reinterpret_cast<PyrHdr *>(lds);
  v.lv = reinterpret_cast<PyrLv *>(lds + PYR_LV_AT);
  v.en = reinterpret_cast<PyrEn *>(lds + PYR_EN_AT);
  unsigned char *p = lds + PYR_HDR_BYTES;
  v.masks = reinterpret_cast<pyr_u64 *>(p);
  v.pref = reinterpret_cast<unsigned short *>(p + 8ll * a.maskWords);
  p += 8ll * a.pyrStride;
  auto pad = [](long long x) { return (x + 15) / 16 * 16; };
  v.srcRow = reinterpret_cast<unsigned *>(p);
  p += pad(4ll * nFirst);
  v.key = reinterpret_cast<unsigned *>(p);
  p += pad(4ll * total);
  v.row = reinterpret_cast<unsigned short *>(p);
  p += pad(2ll * total);
  v.own = reinterpret_cast<unsigned *>(p);
  p += pad(2ll * total);
  v.base = reinterpret_cast<unsigned short *>(p);
  p += pad(2ll * total);
  v.kOf = p;
  return v;
}

// Entry l of the level table (lane l of the workgroup fills it, once a
// window).  L: layer l's arguments, which the lane has fetched already;
// inMaskOff: level l - 1's; bgSource: the source's background row for this
// sample; xa: the window's first level
PYR_FN void pyr_fill_level(const PyrLevel &L, int inMaskOff, int bgSource, const PyrLds &s, int l, int xa) {
  const PyrHdr *h = s.h;
  PyrLv v;
  v.size = L.size;
  v.stride = L.stride;
  v.nIn = L.nIn;
  v.nOut = L.nOut;
  v.width = L.width;
  v.magicS = L.magicS;
  v.inMaskOff = inMaskOff;
  v.inSiteOff = h->siteOff[l - 1];
  const bool region = L.kind == PYR_REGIONS;
  v.siteOff = region ? h->siteOff[l] : 0;
  v.n = region ? h->n[l] : 0;
  const int x = l - 1;
  v.flags = (x == xa ? PYR_LV_SOURCE : 0) | (region ? 0 : PYR_LV_TERMINAL);
  v.inRowBase = x == 0 ? 0 : h->actBefore[x] + h->bgBefore[x];
  v.bgIn = x == 0 ? bgSource : (h->hasBg[x] ? (int)v.inRowBase + h->n[x] : -1);
  v.rowBase = region ? h->actBefore[l] + h->bgBefore[l] : 0;
  v.actBefore = region ? h->actBefore[l] : 0;
  v.volOut = L.volOut;
  v.rules = L.rules;
  v.capacity = L.capacity;
  v.ekey = L.ekey;
  v.erow = L.erow;
  v.boundActive = L.boundActive;
  v.bg = L.bg;
  s.lv[l] = v;
}

// Where the levels of the window xa .. xb start in the per-site arrays, and
// the window's layers among its items: lane t does entry t (t <= nMasks)
PYR_FN void pyr_fill_offsets(PyrHdr *h, int xa, int xb, int t) {
  if (t < xa || t > xb + 1)
    return;
  int sum = 0;
  for (int x = xa; x < t; ++x)
    sum += h->n[x];
  h->siteOff[t] = sum;
  h->itemOff[t] = t > xa ? sum - h->n[xa] : 0;
  if (t == xb + 1)
    h->total = sum;
}

// Entry x of the enumeration's table (x < nMasks; siteOff: in the current window)
PYR_FN void pyr_fill_en(const PyrLevel &L, unsigned char *lds, int x, int siteOff) {
  PyrEn e;
  e.maskOff = L.maskOff;
  e.nOut = L.nOut;
  e.magicN = L.magicN;
  e.siteOff = siteOff;
  reinterpret_cast<PyrEn *>(lds + PYR_EN_AT)[x] = e;
}

// The layer an item of the flattened sweeps belongs to: a lane's items come in
// ascending order, so it moves a cursor (starts at the window's first layer;
// lb: its last)
PYR_FN int pyr_item_level(const PyrHdr *h, int lb, int it, int l) {
  while (l < lb && it >= h->itemOff[l + 1])
    ++l;
  return l;
}

// Window geometry known at compile time: S sites a side (in one dimension the
// side is taken from the layer instead: one row of up to 16 sites), so that
// the rows of a window live in registers.
template <int D, int S> struct PyrGeo {
  static constexpr int ROWS = D == 1 ? 1 : (D == 2 ? S : S * S);
};
template <int D, typename F> PYR_FN void pyr_by_size(int size, F f) {
  if (D == 1 || size == 1) {
    f(std::integral_constant<int, 1>());
    return;
  }
  switch (size) {
  case 2:
    f(std::integral_constant<int, 2>());
    break;
  case 3:
    f(std::integral_constant<int, 3>());
    break;
  default:
    f(std::integral_constant<int, 4>());
    break;
  }
}

// The window of output site j over the input mask: bit k of the result =
// window offset k (row-major) is active.  rowPos[i] = position of the window's
// i-th row in the input field.
template <int D, int S>
PYR_FN unsigned pyr_window(const pyr_u64 *in, int size, int stride, int nIn, const int *j,
                           unsigned *rowPos) {
  const int side = D == 1 ? size : S; // sites of a window row
  unsigned win = 0;
  if (D == 1) {
    rowPos[0] = (unsigned)(j[0] * stride);
    win = pyr_bits(in, rowPos[0], side);
  } else if (D == 2) {
#if defined(__HIPCC__)
#pragma unroll
#endif
    for (int q0 = 0; q0 < S; ++q0) {
      rowPos[q0] = (unsigned)((j[0] * stride + q0) * nIn + j[D - 1] * stride);
      win |= pyr_bits(in, rowPos[q0], side) << (q0 * S);
    }
  } else {
#if defined(__HIPCC__)
#pragma unroll
#endif
    for (int q0 = 0; q0 < S; ++q0)
#if defined(__HIPCC__)
#pragma unroll
#endif
      for (int q1 = 0; q1 < S; ++q1) {
        const int i = q0 * S + q1;
        rowPos[i] = (unsigned)(((j[0] * stride + q0) * nIn + (j[D > 1 ? 1 : 0] * stride + q1)) * nIn +
                               j[D - 1] * stride);
        win |= pyr_bits(in, rowPos[i], side) << (i * S);
      }
  }
  return win;
}

// Owner of output site r of the layer v: which window offset (k) and which
// input rank
template <int D>
PYR_FN void pyr_owner(const PyrLv &v, const PyrLds &s, int r, int *kStar, unsigned *ownerRank) {
  const pyr_u64 *in = s.masks + v.inMaskOff;
  const unsigned short *pref = s.pref + v.inMaskOff;
  int j[D];
  pyr_unpack<D>(s.key[v.siteOff + r], j);
  const int size = v.size, stride = v.stride, nIn = v.nIn;
  const unsigned magicS = v.magicS;
  pyr_by_size<D>(size, [&](auto sz) {
    constexpr int S = decltype(sz)::value;
    constexpr int ROWS = PyrGeo<D, S>::ROWS;
    unsigned rowPos[ROWS];
    const unsigned win = pyr_window<D, S>(in, size, stride, nIn, j, rowPos);
    const int k = pyr_ctz32(win); // (an output site's window holds an active input)
    const int side = D == 1 ? size : S;
    const int wr = D == 1 ? 0 : (int)pyr_div((unsigned)k, (unsigned)side, magicS);
    unsigned p = rowPos[0];
    // (a select over the rows instead of an indexed read of a register array)
#if defined(__HIPCC__)
#pragma unroll
#endif
    for (int i = 1; i < ROWS; ++i)
      p = i == wr ? rowPos[i] : p;
    p += (unsigned)(k - wr * side);
    *kStar = k;
    *ownerRank = pyr_rank(in, pref, p);
  });
}

#if defined(__HIP_DEVICE_COMPILE__)
#define PYR_ATOMIC_OR(ptr, v) atomicOr((ptr), (v))
#else
#define PYR_ATOMIC_OR(ptr, v) (*(ptr) |= (v))
#endif

// ---- sweep 0: the ownership masks start empty (no barrier is needed between
// this and sweep 1: they touch different arrays)
PYR_FN void pyr_sweep_clear(const PyrLds &s, int t, int T) {
  for (int i = t; i < (s.h->total + 1) / 2; i += T)
    s.own[i] = 0u;
}

// Position of the k-th set bit of v (k < popcount(v)), by halving
PYR_FN unsigned pyr_select64(pyr_u64 v, unsigned k) {
  unsigned part = (unsigned)v, off = 0;
  unsigned c = (unsigned)pyr_popc32(part);
  if (k >= c) {
    k -= c;
    part = (unsigned)(v >> 32);
    off = 32;
  }
  c = (unsigned)pyr_popc32(part & 0xFFFFu);
  if (k >= c) {
    k -= c;
    part >>= 16;
    off += 16;
  }
  c = (unsigned)pyr_popc32(part & 0xFFu);
  if (k >= c) {
    k -= c;
    part >>= 8;
    off += 8;
  }
  c = (unsigned)pyr_popc32(part & 0xFu);
  if (k >= c) {
    k -= c;
    part >>= 4;
    off += 4;
  }
  c = (unsigned)pyr_popc32(part & 3u);
  if (k >= c) {
    k -= c;
    part >>= 2;
    off += 2;
  }
  return off + (k >= (part & 1u) ? 1u : 0u);
}

// ---- sweep 1: the sites of every level by rank, a lane per SITE (a lane per
// mask word leaves most lanes waiting for the one with the fullest word): the
// word that holds rank r is the last one whose prefix is <= r, found by
// bisection; the site is the (r - prefix)-th set bit of it.  A lane's sites
// come in ascending order, so the level is a cursor.  Of the window's first
// level only the source needs its coordinates (to look its rows up).
template <int D>
PYR_FN void pyr_sweep_enumerate(const PyrArgs &a, const PyrLds &s, int xa, int xb, int t, int T) {
  const int total = s.h->total;
  int x = xa;
  for (int i = (xa > 0 ? s.h->n[xa] : 0) + t; i < total; i += T) {
    while (x + 1 <= xb && i >= s.en[x + 1].siteOff)
      ++x;
    const PyrEn e = s.en[x];
    const unsigned r = (unsigned)(i - e.siteOff);
    // (the level's two spare words have the level's count as prefix: > r)
    const int span = (x + 1 < a.nMasks ? s.en[x + 1].maskOff : a.maskWords) - e.maskOff;
    const unsigned short *pref = s.pref + e.maskOff;
    int lo = 0, hi = span;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (pref[mid] <= r)
        lo = mid;
      else
        hi = mid;
    }
    unsigned k = 64u * (unsigned)lo + pyr_select64(s.masks[e.maskOff + lo], r - pref[lo]);
    int c[D];
    for (int q = D - 1; q >= 0; --q) {
      const unsigned up = pyr_div(k, (unsigned)e.nOut, e.magicN);
      c[q] = (int)(k - up * (unsigned)e.nOut);
      k = up;
    }
    s.key[i] = pyr_pack<D>(c);
  }
}

// ---- sweep 2: every output site tells its owner which candidate it is
template <int D>
PYR_FN void pyr_sweep_owners(const PyrLds &s, int la, int lb, int t, int T) {
  const PyrHdr *h = s.h;
  const int items = h->itemOff[lb + 1];
  int l = la;
  for (int it = t; it < items; it += T) {
    l = pyr_item_level(h, lb, it, l);
    const PyrLv &v = s.lv[l];
    int k;
    unsigned rank;
    const int r = it - h->itemOff[l];
    pyr_owner<D>(v, s, r, &k, &rank);
    const unsigned at = (unsigned)v.inSiteOff + rank;
    PYR_ATOMIC_OR(&s.own[at >> 1], 1u << (k + 16 * (int)(at & 1u)));
    // (kept for sweep 4, which then has no window to look at)
    s.row[v.siteOff + r] = (unsigned short)rank;
    s.kOf[v.siteOff + r] = (unsigned char)k;
  }
}

PYR_FN unsigned pyr_own_mask(const PyrLds &s, unsigned at) {
  return (s.own[at >> 1] >> (16 * (at & 1u))) & 0xFFFFu;
}

// ---- sweep 4: rows of the output sites; the layers' entry lists
template <int D>
PYR_FN void pyr_sweep_rows(const PyrLds &s, int la, int lb, int b, int t, int T) {
  const PyrHdr *h = s.h;
  const int items = h->itemOff[lb + 1];
  int l = la;
  for (int it = t; it < items; it += T) {
    l = pyr_item_level(h, lb, it, l);
    const PyrLv &v = s.lv[l];
    const int r = it - h->itemOff[l];
    const int k = s.kOf[v.siteOff + r];
    const unsigned at = (unsigned)v.inSiteOff + s.row[v.siteOff + r];
    // the owner's candidates after this one are the outputs before it
    const unsigned row = s.base[at] + (unsigned)pyr_popc32(pyr_own_mask(s, at) >> (k + 1));
    s.row[v.siteOff + r] = (unsigned short)row;
    int j[D];
    pyr_unpack<D>(s.key[v.siteOff + r], j);
    const long long entry = v.actBefore + row;
    if (entry >= 0 && entry <= v.boundActive) { // (the entry list holds boundActive + 1)
      v.ekey[entry] = (long long)b * v.volOut + pyr_key<D>(j, v.nOut);
      v.erow[entry] = (int)(v.rowBase + row);
    }
  }
}

// batch-global row of the input site with rank `rank` of layer v
PYR_FN int pyr_in_row(const PyrLv &v, const PyrLds &s, unsigned rank) {
  if (v.flags & PYR_LV_SOURCE)
    return (int)s.srcRow[rank];
  return (int)v.inRowBase + (int)s.row[v.inSiteOff + rank];
}
// batch-global row of level x's background row of this sample (-1: none)
PYR_FN int pyr_bg_row(const PyrArgs &a, const PyrLds &s, int x, int b) {
  const PyrHdr *h = s.h;
  if (x == 0)
    return a.bg[b];
  return h->hasBg[x] ? (int)(h->actBefore[x] + h->bgBefore[x]) + h->n[x] : -1;
}

struct alignas(8) PyrInt2 {
  int x, y;
};
struct alignas(16) PyrInt4 {
  int x, y, z, w;
};

// ---- sweep 5: rule rows
template <int D>
PYR_FN void pyr_sweep_rules(const PyrLds &s, int la, int lb, int t, int T) {
  const PyrHdr *h = s.h;
  const int items = h->itemOff[lb + 1];
  int l = la;
  for (int it = t; it < items; it += T) {
    l = pyr_item_level(h, lb, it, l);
    const PyrLv &v = s.lv[l];
    if (!v.rules)
      continue;
    const int r = it - h->itemOff[l];
    const pyr_u64 *in = s.masks + v.inMaskOff;
    const unsigned short *pref = s.pref + v.inMaskOff;
    int j[D];
    pyr_unpack<D>(s.key[v.siteOff + r], j);
    const int bgIn = v.bgIn;
    const long long row = v.rowBase + s.row[v.siteOff + r];
    if (row < 0 || (row + 1) * v.width > v.capacity)
      continue; // (cannot happen while counts and masks agree; never write outside the caller's buffer)
    int *dst = v.rules + row * v.width;
    const int size = v.size, stride = v.stride, nIn = v.nIn;
    pyr_by_size<D>(size, [&](auto sz) {
      constexpr int S = decltype(sz)::value;
      constexpr int ROWS = PyrGeo<D, S>::ROWS;
      unsigned rowPos[ROWS];
      const unsigned win = pyr_window<D, S>(in, size, stride, nIn, j, rowPos);
      const int side = D == 1 ? size : S;
#if defined(__HIPCC__)
#pragma unroll
#endif
      for (int i = 0; i < ROWS; ++i) {
        const unsigned present = (win >> (i * side)) & ((1u << side) - 1u);
        // the active sites of a window row are neighbours in rank
        unsigned rank = present ? pyr_rank(in, pref, rowPos[i]) : 0u;
        if constexpr (D >= 2 && S % 2 == 0) {
          // (a rule row of 4 or 8 or 16 ... entries starts on 16 bytes: two
          // or four entries a store)
          int val[S];
#if defined(__HIPCC__)
#pragma unroll
#endif
          for (int q = 0; q < S; ++q) {
            val[q] = bgIn;
            if ((present >> q) & 1u)
              val[q] = pyr_in_row(v, s, rank++);
          }
          if constexpr (S == 2) {
            PyrInt2 o = {val[0], val[1]};
            *reinterpret_cast<PyrInt2 *>(dst + i * S) = o;
          } else {
            PyrInt4 o = {val[0], val[1], val[2], val[3]};
            *reinterpret_cast<PyrInt4 *>(dst + i * S) = o;
          }
        } else {
          for (int q = 0; q < side; ++q) {
            int val = bgIn;
            if ((present >> q) & 1u)
              val = pyr_in_row(v, s, rank++);
            dst[i * side + q] = val;
          }
        }
      }
    });
  }
}

// ---- the rows of the window's last level, batch-global, where the next
// window (which starts at that level) looks its input's rows up.  The
// destination lies before everything the old window still holds.
PYR_FN void pyr_sweep_carry(const PyrLds &s, unsigned char *lds, const PyrArgs &a, int xb, int t, int T) {
  const PyrHdr *h = s.h;
  const unsigned short *row = s.row + h->siteOff[xb];
  unsigned *dst = reinterpret_cast<unsigned *>(lds + PYR_HDR_BYTES + 8ll * a.pyrStride);
  const long long rowBase = h->actBefore[xb] + h->bgBefore[xb];
  for (int i = t; i < h->n[xb]; i += T)
    dst[i] = (unsigned)(rowBase + row[i]);
}

// ---- the all-background rows, backgroundCol of the window's layers, a
// wavefront per layer; with the last window (xb = nMasks - 1) the terminal
// layer's rules, if the chain ends in one (all lanes)
PYR_FN void pyr_sweep_tail(const PyrArgs &a, const PyrLds &s, int la, int lb, int b, int t, int T) {
  const PyrHdr *h = s.h;
  const int W = T >= 64 ? 64 : T;
  const int lane = t % W, wave = t / W, waves = T / W;
  for (int l = la + wave; l <= lb; l += waves) {
    const PyrLv &v = s.lv[l];
    const int bgOut = pyr_bg_row(a, s, l, b);
    if (h->hasBg[l] && v.rules && bgOut >= 0 &&
        ((long long)bgOut + 1) * v.width <= v.capacity) { // Regions.cu:647-652
      const int bgIn = v.bgIn;
      int *dst = v.rules + (long long)bgOut * v.width;
      for (int q = lane; q < v.width; q += W)
        dst[q] = bgIn;
    }
    if (lane == 0)
      v.bg[b] = bgOut;
  }
  if (lb != a.nMasks - 1 || a.nLevels == lb)
    return;
  const PyrLv &v = s.lv[a.nLevels];
  {
    // terminalGridPoolingRules (TerminalPoolingLayer.cu:8-20): the rows in
    // iteration order, or the background row of a sample without sites;
    // padded with -1 to the batch's largest sample (:90-96)
    const int x = a.nLevels - 1;
    const long long width = h->maxAct[x] > 1 ? h->maxAct[x] : 1;
    if (v.rules && ((long long)b + 1) * width <= v.capacity) {
      const int n = h->n[x];
      int *dst = v.rules + (long long)b * width;
      for (long long i = t; i < width; i += T) {
        int val = -1;
        if (n == 0 && i == 0)
          val = v.bgIn;
        else if (i < n)
          val = pyr_in_row(v, s, (unsigned)i);
        dst[i] = val;
      }
    }
    if (t == 0) { // the output grid: site 0 of sample b is row b
      v.ekey[b] = b;
      v.erow[b] = b;
      v.bg[b] = -1;
    }
  }
}

// What a layer reports: sites, active sites, whether it outgrew its bounds,
// and the terminal width or the largest sample (the header holds the sums)
struct PyrReport {
  long long nSites, nActive, over, extra;
};
PYR_FN PyrReport pyr_report(const PyrArgs &a, const PyrLevel &L, const PyrHdr *h, int l) {
  PyrReport r;
  if (L.kind == PYR_TERMINAL) {
    const long long width = h->maxAct[l - 1] > 1 ? h->maxAct[l - 1] : 1;
    r.nSites = r.nActive = a.batch;
    r.extra = width;
    r.over = width > L.boundRows || (L.rules && width * a.batch > L.capacity);
  } else {
    r.nSites = h->actAll[l] + h->bgAll[l];
    r.nActive = h->actAll[l];
    r.extra = h->maxAct[l];
    r.over = r.nSites > L.boundRows || r.nActive > L.boundActive ||
             (L.rules && r.nSites * L.width > L.capacity);
  }
  return r;
}
