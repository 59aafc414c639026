// Rule books of every layer of a net in two launches (small fields).
//
// BatchProducer::preprocessBatch (BatchProducer.cu:40-87) calls preprocess()
// of every layer back to back, and gridRules runs per sample
// (ConvolutionalLayer.cu:114-118, MaxPoolingLayer.cu:116-118): the samples of
// a batch never meet until their rows are numbered.  scn_grids.hip builds one
// layer at a time over the whole batch through tables in HBM, four launches
// per layer; for a 2-D net that is some fifty dependent launches of a few
// microseconds each.  Here the plan and fill calls of consecutive layers are
// only recorded (scn_ctx_chain_rules) and then run together, in one of two ways.
//
// Chains of square windows without a minimum of active inputs (a terminal
// layer may end them) are built from the output side (second half of this
// file, per-lane bodies in scn_pyr_dev.h):
//
//   k_pyr_masks     one wavefront per sample: the occupancy masks of all
//                   layers, each the dilation of the one before, their rank
//                   prefixes and the sample's site counts;
//   k_pyr_rules     one workgroup per sample: the counts of the samples before
//                   it, then per output site in sweeps over all layers at once
//                   -- sites by rank, owners, rows, entry lists, rule rows --
//                   written at their batch-global places.
//
// Every other chain (a minimum of active inputs, triangular lattices, windows
// of more than 16 sites) goes the older way, from the input side:
//
//   k_chain_sample  one workgroup per sample carries the sample's grid --
//                   occupancy mask, rank prefix, (key, row) by rank -- in LDS
//                   through all recorded layers: owner test and counts, prefix
//                   sum, output sites, rule rows, with rows numbered from zero
//                   within the sample; rule rows and site keys go to a staging
//                   area at sample-local positions;
//   k_chain_place   one workgroup per (sample, layer) adds up the counts of
//                   the samples before it and copies the staged rows to their
//                   batch-global place, adding the row offsets of the sample.
//
// Row numbers are the reference's: first touch while the input map is
// iterated in ascending key (Regions.cu:557-576), background row last
// (:647-652), samples concatenated in batch order.  The grids objects of the
// recorded layers get their entry lists, backgroundCol and counts; their hash
// tables and masks are only built if somebody asks (ensure_index).
#include "scn_grids_dev.h"
#include "scn_pyr_dev.h"
#include <stdlib.h>
#include <string.h>
#include <mutex>

#define CHAIN_MAX_LEVELS 24
#ifndef CHAIN_THREADS
#define CHAIN_THREADS 512
#endif
#define CHAIN_WAVES (CHAIN_THREADS / 64)
#define CHAIN_LDS_MAX (152 * 1024)
// most LDS a workgroup of k_pyr_rules asks for
#define PYR_LDS_MAX CHAIN_LDS_MAX
#define CHAIN_HEADER_BYTES 512
#define CHAIN_MIN_ARENA (16 * 1024)
// bytes of arena per entry of the input grid (key, row, ownership mask, base)
// and of the output grid (key, row)
#define CHAIN_IN_BYTES 16
#define CHAIN_OUT_BYTES 8

enum { CH_REGIONS = 0, CH_TERMINAL = 1 };

struct ChainLevel {
  int kind;
  int mode, nIn, nOut, size, stride, minActive, width, cube;
  int capRows; // rows of one sample the staging area holds
  int slot;    // pinned slot of the deferred counts
  // floor(2^32 / d) + 1 for d = width / size, width and size: x / d without a division
  unsigned magicRuns, magicWidth, magicSize, magicStride;
  long long fullSize; // sites of a full output grid
  // staging, in ints: rule rows of sample b at stRules + b capRows width,
  // site keys at stKeys + b capRows
  long long stRules, stKeys;
  int *rules; // the caller's buffer (null: no rules wanted)
  long long capacity;
  long long *ekey;
  int *erow;
  int *bg;
  long long *meta;
  long long boundRows, boundActive; // terminal: boundRows bounds the width
};

struct ChainArgs {
  int nLevels, batch, d, n0;
  const Slot *table; // the source grids: hash table,
  const int *dense;  // or dense row table
  unsigned shift, mask;
  const unsigned long long *bits;
  const int *bg;
  long long vol0;
  int maskOff[3], prefOff[2], arenaOff, arenaBytes; // LDS layout, bytes
  int maskWords[3]; // capacity of the three mask buffers, 64-bit words
  int *counts; // [nLevels][batch][2]
  unsigned long long *flag;
  unsigned long long ticket;
  int *staging;
  long long *scalars;
  const long long *badSites;
  ChainLevel lv[CHAIN_MAX_LEVELS];
};
static_assert(sizeof(ChainArgs) <= 4096, "kernel arguments");

struct ChainRec {
  scn_grids *in, *out;
  ChainLevel lv;
  Geom geom;
  bool filled;
};
struct ChainState {
  bool on = false;
  bool wide = false; // a sample has outgrown a tight arena: use the largest
  long long nChains = 0, nPlans = 0; // run so far
  std::vector<ChainRec> recs;
  DevBuf<int> staging, counts;
  DevBuf<unsigned long long> flag;
  // chains of square layers without a minimum, built from the output side
  DevBuf<unsigned long long> pyramid;
  bool pyramids = true; // (false: such chains go through k_chain_sample too)
  bool pyrAtMax = false; // the last such chain had all the LDS there is
  int pyrMisses = 0;     // such chains in a row that still outgrew it
  scn_grids *pyrSource = nullptr; // source of the last such chain: its largest sample comes back in h_pinned[13]
  long long nPyramids = 0;
};

// ------------------------------------------------------------------ device

// A barrier that orders LDS traffic only.  __syncthreads() also waits for the
// global stores in flight (the staged rule rows), a microsecond or two each
// time; nothing a workgroup stores to global memory is read back by it.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ unsigned wave_scan_incl(unsigned v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    unsigned up = __shfl_up(v, off, 64);
    if (lane >= off)
      v += up;
  }
  return v;
}

// The same sums through the lanes' cross-lane data path instead of the LDS
// crossbar: shifts within a row of 16 lanes, then the last lane of rows 0 and 2
// into the rows after them, then lane 31 into rows 2 and 3 (a lane that a step
// does not reach adds 0).
__device__ __forceinline__ unsigned wave_scan_incl_dpp(unsigned v) {
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false); // row_shr:1
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false); // row_shr:2
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false); // row_shr:4
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false); // row_shr:8
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false); // row_bcast:15
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false); // row_bcast:31
  return v;
}
__device__ __forceinline__ unsigned wave_last(unsigned v) {
  return (unsigned)__builtin_amdgcn_readlane((int)v, 63);
}

// Exclusive prefix sums over two sequences held in LDS at once, by the whole
// workgroup: putX(i, sum of getX(0..i)); the totals come back to every lane.
// Every lane takes a run of consecutive values.  ws: 2 * CHAIN_WAVES words.
template <typename GetA, typename PutA, typename GetB, typename PutB>
__device__ __forceinline__ void chain_scan2(int nA, GetA getA, PutA putA,
                                            unsigned &totalA, int nB, GetB getB,
                                            PutB putB, unsigned &totalB,
                                            unsigned *ws) {
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int perA = (nA + CHAIN_THREADS - 1) / CHAIN_THREADS;
  const int a0 = t * perA < nA ? t * perA : nA;
  const int a1 = a0 + perA < nA ? a0 + perA : nA;
  const int perB = (nB + CHAIN_THREADS - 1) / CHAIN_THREADS;
  const int b0 = t * perB < nB ? t * perB : nB;
  const int b1 = b0 + perB < nB ? b0 + perB : nB;
  unsigned sA = 0, sB = 0;
  for (int i = a0; i < a1; ++i)
    sA += getA(i);
  for (int i = b0; i < b1; ++i)
    sB += getB(i);
  const unsigned inclA = wave_scan_incl(sA, lane);
  const unsigned inclB = wave_scan_incl(sB, lane);
  if (lane == 63) {
    ws[wave] = inclA;
    ws[CHAIN_WAVES + wave] = inclB;
  }
  lds_barrier();
  unsigned beforeA = 0, beforeB = 0;
  totalA = totalB = 0;
#pragma unroll
  for (int w = 0; w < CHAIN_WAVES; ++w) {
    const unsigned x = ws[w], y = ws[CHAIN_WAVES + w];
    beforeA += w < wave ? x : 0u;
    beforeB += w < wave ? y : 0u;
    totalA += x;
    totalB += y;
  }
  unsigned run = beforeA + inclA - sA;
  for (int i = a0; i < a1; ++i) {
    const unsigned v = getA(i);
    putA(i, run);
    run += v;
  }
  run = beforeB + inclB - sB;
  for (int i = b0; i < b1; ++i) {
    const unsigned v = getB(i);
    putB(i, run);
    run += v;
  }
  lds_barrier();
}

__device__ __forceinline__ unsigned lds_rank(const unsigned long long *bits,
                                             const unsigned short *pref,
                                             unsigned p) {
  const unsigned w = p >> 6, sh = p & 63;
  const unsigned long long below = sh ? (bits[w] & ((1ull << sh) - 1ull)) : 0ull;
  return pref[w] + (unsigned)__popcll(below);
}

// Entries carry their site as packed coordinates, so that no lane divides:
// 30 bits in one dimension, 15 bits an axis in two, 10 in three.
template <int D> struct Packed {
  static constexpr int BITS = D == 1 ? 30 : (D == 2 ? 15 : 10);
  static constexpr unsigned MASK = (1u << BITS) - 1u;
};
template <int D> __device__ __forceinline__ unsigned pack_site(const int *c) {
  unsigned v = 0;
#pragma unroll
  for (int q = 0; q < D; ++q)
    v |= (unsigned)c[q] << (q * Packed<D>::BITS);
  return v;
}
template <int D> __device__ __forceinline__ void unpack_site(unsigned v, int *c) {
#pragma unroll
  for (int q = 0; q < D; ++q)
    c[q] = (int)((v >> (q * Packed<D>::BITS)) & Packed<D>::MASK);
}
template <int D> __device__ __forceinline__ unsigned site_key(const int *c, int n) {
  unsigned k = 0;
#pragma unroll
  for (int q = 0; q < D; ++q)
    k = k * (unsigned)n + (unsigned)c[q];
  return k;
}
// The sample could not be carried (LDS or staging too small): every plan of
// the chain is reported as outgrown, and the caller plans the batch again
// layer by layer.
__device__ __forceinline__ void chain_give_up(const ChainArgs &a) {
  if (threadIdx.x == 0)
    atomicMax(a.flag, a.ticket);
}

template <int D>
__global__ void __launch_bounds__(CHAIN_THREADS) k_chain_sample(ChainArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int b = blockIdx.x, t = threadIdx.x;
  unsigned *ws = reinterpret_cast<unsigned *>(lds); // 2 * CHAIN_WAVES words
  int *invOrd = reinterpret_cast<int *>(lds + 128); // up to 64 offsets
  auto M = [&](int x) {
    return reinterpret_cast<unsigned long long *>(lds + a.maskOff[x]);
  };
  auto P = [&](int x) {
    return reinterpret_cast<unsigned short *>(lds + a.prefOff[x]);
  };
  unsigned *arena = reinterpret_cast<unsigned *>(lds + a.arenaOff);
  const int arenaWords = a.arenaBytes / 4;
  // ---- the source grid of this sample: its slice of the batch's mask
  long long vol = a.vol0;
  int words = (int)((vol + 63) >> 6);
  {
    unsigned long long *bitsA = M(0);
    const long long p0 = (long long)b * vol;
    for (int w = t; w <= words; w += CHAIN_THREADS) {
      unsigned long long v = 0;
      const long long left = vol - 64ll * w;
      if (left > 0) {
        const long long p = p0 + 64ll * w;
        const long long gw = p >> 6;
        const int sh = (int)(p & 63);
        v = a.bits[gw] >> sh;
        if (sh)
          v |= a.bits[gw + 1] << (64 - sh);
        if (left < 64)
          v &= (1ull << left) - 1ull;
      }
      bitsA[w] = v;
    }
    // the masks of the first two output grids start empty
    for (int w = t; w < a.maskWords[1]; w += CHAIN_THREADS)
      M(1)[w] = 0ull;
    for (int w = t; w < a.maskWords[2]; w += CHAIN_THREADS)
      M(2)[w] = 0ull;
  }
  lds_barrier();
  unsigned nA;
  {
    const unsigned long long *bitsA = M(0);
    unsigned short *prefA = P(0);
    unsigned none;
    chain_scan2(
        words, [&](int i) { return (unsigned)__popcll(bitsA[i]); },
        [&](int i, unsigned v) { prefA[i] = (unsigned short)v; }, nA, 0,
        [&](int) { return 0u; }, [&](int, unsigned) {}, none, ws);
  }
  if ((long long)nA * CHAIN_IN_BYTES > a.arenaBytes) {
    chain_give_up(a);
    return;
  }
  // entries by rank at the bottom of the arena: site[nA], row[nA]
  unsigned *keyA = arena, *rowA = arena + nA;
  {
    const unsigned long long *bitsA = M(0);
    const unsigned short *prefA = P(0);
    for (int w = t; w < words; w += CHAIN_THREADS) {
      unsigned long long v = bitsA[w];
      unsigned r = prefA[w];
      while (v) {
        keyA[r++] = 64u * w + (unsigned)(__ffsll((long long)v) - 1);
        v &= v - 1;
      }
    }
    lds_barrier();
    // One lane per entry, eight entries a lane at a time: their first probes
    // of the table are requested together (a probe is a trip to HBM, and at
    // load factor 1/2 three look-ups in four end with the first).
    const long long p0 = (long long)b * vol;
    constexpr int EU = 8;
    if (a.dense) { // the row of every site of the field: one load an entry
      for (unsigned r = t; r < nA; r += CHAIN_THREADS) {
        unsigned kk = keyA[r];
        rowA[r] = (unsigned)a.dense[p0 + kk];
        int c[D];
#pragma unroll
        for (int q = D - 1; q >= 0; --q) {
          const unsigned up = kk / (unsigned)a.n0;
          c[q] = (int)(kk - up * (unsigned)a.n0);
          kk = up;
        }
        keyA[r] = pack_site<D>(c);
      }
    } else
    for (unsigned r0 = t; r0 < nA; r0 += EU * CHAIN_THREADS) {
      unsigned key[EU], slot[EU];
      int4 first[EU];
#pragma unroll
      for (int u = 0; u < EU; ++u) {
        const unsigned r = r0 + u * CHAIN_THREADS;
        key[u] = keyA[r < nA ? r : t];
        slot[u] = hash_slot(p0 + key[u], a.shift);
        first[u] = *reinterpret_cast<const int4 *>(&a.table[slot[u]]);
      }
#pragma unroll
      for (int u = 0; u < EU; ++u) {
        const unsigned r = r0 + u * CHAIN_THREADS;
        if (r >= nA)
          continue;
        const long long p = p0 + key[u];
        long long k = ((long long)first[u].y << 32) | (unsigned)first[u].x;
        int row = first[u].z;
        unsigned sl = slot[u];
        while (k != p && k != SLOT_EMPTY) { // the rest of the probe sequence
          sl = (sl + 1) & a.mask;
          const int4 v = *reinterpret_cast<const int4 *>(&a.table[sl]);
          k = ((long long)v.y << 32) | (unsigned)v.x;
          row = v.z;
        }
        rowA[r] = (unsigned)(k == p ? row : -1);
        unsigned kk = key[u];
        int c[D];
#pragma unroll
        for (int q = D - 1; q >= 0; --q) {
          const unsigned up = kk / (unsigned)a.n0;
          c[q] = (int)(kk - up * (unsigned)a.n0);
          kk = up;
        }
        keyA[r] = pack_site<D>(c);
      }
    }
  }
  int bgA = a.bg[b];
  lds_barrier();

  for (int l = 0; l < a.nLevels; ++l) {
    const ChainLevel &L = a.lv[l];
    const unsigned long long *bitsA = M(l % 3);
    const unsigned short *prefA = P(l & 1);
    int *st = a.staging + L.stRules + (long long)b * L.capRows * L.width;
    if (L.kind == CH_TERMINAL) {
      // terminalGridPoolingRules (TerminalPoolingLayer.cu:8-20): the rows in
      // iteration order, or the background row of a sample without sites
      if (nA == 0) {
        if (t == 0)
          st[0] = bgA;
      } else {
        for (unsigned r = t; r < nA; r += CHAIN_THREADS)
          st[r] = (int)rowA[r];
      }
      if (t == 0) {
        a.counts[((long long)l * a.batch + b) * 2] = (int)nA;
        a.counts[((long long)l * a.batch + b) * 2 + 1] = 0;
      }
      return; // nothing is recorded behind a terminal layer
    }
    if ((long long)nA * CHAIN_IN_BYTES > a.arenaBytes) {
      chain_give_up(a);
      return;
    }
    Geom g;
    g.d = D;
    g.nIn = L.nIn;
    g.nOut = L.nOut;
    g.size = L.size;
    g.stride = L.stride;
    g.minActive = L.minActive;
    g.mode = L.mode;
    g.volIn = vol;
    long long volOut = 1;
#pragma unroll
    for (int q = 0; q < D; ++q)
      volOut *= L.nOut;
    g.volOut = volOut;
    g.width = L.width;
    g.cube = L.cube;
    g.ticks = nullptr;
    g.tInR = g.tOutL = g.tOutR = 0;
    const bool tri = L.mode == MODE_TRI_NOMIN || L.mode == MODE_TRI_MIN;
    unsigned long long *bitsB = M((l + 1) % 3);
    unsigned short *prefB = P((l + 1) & 1);
    const int wordsB = (int)((volOut + 63) >> 6);
    // ownership masks and bases beside the input's entries: above them when
    // those sit at the bottom of the arena (even layers), below them otherwise
    unsigned *maskS, *keyB, *rowB;
    unsigned short *baseS;
    const unsigned halfA = (nA + 1) / 2; // words of nA 16-bit bases
    if (l & 1) {
      maskS = keyA - nA - halfA;
      baseS = reinterpret_cast<unsigned short *>(keyA - halfA);
    } else {
      maskS = rowA + nA;
      baseS = reinterpret_cast<unsigned short *>(maskS + nA);
    }
    GridView vin;
    vin.bits = const_cast<unsigned long long *>(bitsA);

    // -- which candidates each input owns; the output mask
    const bool fast = D >= 2 && L.mode == MODE_SQ_NOMIN && (L.size == 2 || L.size == 3);
    for (unsigned r = t; r < nA; r += CHAIN_THREADS) {
      int i[D], lo[D], hi[D], j[D];
      unpack_site<D>(keyA[r], i);
      unsigned m = 0;
      auto mark = [&](const int *jj) {
        const unsigned ok = site_key<D>(jj, L.nOut);
        atomicOr(&bitsB[ok >> 6], 1ull << (ok & 63));
      };
      if (!cand_box<D>(g, b, i, lo, hi)) {
        m = 0;
      } else if (fast) {
        if constexpr (D >= 2) {
          if (L.size == 2)
            m = owned_nomin<D, 2>(bitsA, 0u, i, lo, hi, L.nIn, L.stride, L.magicStride, mark);
          else
            m = owned_nomin<D, 3>(bitsA, 0u, i, lo, hi, L.nIn, L.stride, L.magicStride, mark);
        }
      } else {
#pragma unroll
        for (int q = 0; q < D; ++q)
          j[q] = lo[q];
        for (int c = 0;; ++c) {
          if (owns<D>(vin, g, b, 0ll, i, j)) {
            m |= 1u << c;
            mark(j);
          }
          int q = D - 1;
          for (; q >= 0; --q) {
            if (++j[q] < hi[q])
              break;
            j[q] = lo[q];
          }
          if (q < 0)
            break;
        }
      }
      maskS[r] = m;
    }
    if (tri && t == 0) { // inverse of RegularTriangularRegions::ord (Regions.cu:810-826)
      int S = 0;
      for (int q = 0; q < L.cube; ++q) {
        int x = q, sum = 0;
        while (x > 0) {
          sum += x % L.size;
          x /= L.size;
        }
        if (sum < L.size)
          invOrd[S++] = q;
      }
    }
    lds_barrier();

    // -- rows of the outputs: prefix sum of the owned counts, and the rank
    //    prefix of the output mask
    unsigned nB, nBits;
    chain_scan2(
        (int)nA, [&](int i) { return (unsigned)__popc(maskS[i]); },
        [&](int i, unsigned v) { baseS[i] = (unsigned short)v; }, nB, wordsB,
        [&](int i) { return (unsigned)__popcll(bitsB[i]); },
        [&](int i, unsigned v) { prefB[i] = (unsigned short)v; }, nBits, ws);
    const int hasBg = (long long)nB < L.fullSize;
    if ((long long)nA * CHAIN_IN_BYTES + (long long)nB * CHAIN_OUT_BYTES >
            a.arenaBytes ||
        (long long)nB + 1 > L.capRows) {
      chain_give_up(a);
      return;
    }
    if (t == 0) {
      a.counts[((long long)l * a.batch + b) * 2] = (int)nB;
      a.counts[((long long)l * a.batch + b) * 2 + 1] = hasBg;
    }
    if (l & 1) {
      keyB = arena;
      rowB = arena + nB;
    } else {
      keyB = arena + arenaWords - 2 * nB;
      rowB = keyB + nB;
    }
    int *stKey = a.staging + L.stKeys + (long long)b * L.capRows;

    // -- the output grid's entries by rank; site keys by row to the staging area
    for (unsigned r = t; r < nA; r += CHAIN_THREADS) {
      unsigned m = maskS[r];
      if (!m)
        continue;
      unsigned row = baseS[r];
      int i[D], lo[D], hi[D], j[D];
      unpack_site<D>(keyA[r], i);
      (void)cand_box<D>(g, b, i, lo, hi);
      while (m) { // ascending candidate = ascending output key
        int rem = __ffs((int)m) - 1;
        m &= m - 1;
#pragma unroll
        for (int q = D - 1; q >= 0; --q) {
          const unsigned ext = (unsigned)(hi[q] - lo[q]);
          const unsigned up = (unsigned)rem / ext;
          j[q] = lo[q] + (int)((unsigned)rem - up * ext);
          rem = (int)up;
        }
        const unsigned ok = site_key<D>(j, L.nOut);
        const unsigned rk = lds_rank(bitsB, prefB, ok);
        keyB[rk] = pack_site<D>(j);
        rowB[rk] = row;
        stKey[row] = (int)ok;
        ++row;
      }
    }
    { // the mask of the grid after the next starts empty (its buffer held
      // the grid before this layer's input, which nothing reads any more)
      unsigned long long *z = M((l + 2) % 3);
      const int nz = l == 0 ? 0 : a.maskWords[(l + 2) % 3];
      for (int w = t; w < nz; w += CHAIN_THREADS)
        z[w] = 0ull;
    }
    lds_barrier();

    // -- rule rows (sample-local row numbers) to the staging area
    if (L.rules) {
      if (!tri && L.size >= 2) {
        // one lane per run of `size` entries along the innermost axis: their
        // input sites are neighbours in the mask and in rank
        const unsigned runsPerRow = (unsigned)(L.width / L.size);
        const unsigned items = nB * runsPerRow;
        for (unsigned it = t; it < items; it += CHAIN_THREADS) {
          const unsigned rk = div_magic(it, runsPerRow, L.magicRuns);
          const int run0 = (int)(it - rk * runsPerRow);
          int j[D], c[D];
          unpack_site<D>(keyB[rk], j);
          c[D - 1] = j[D - 1] * L.stride;
          if (D == 2) {
            c[0] = j[0] * L.stride + run0;
          } else if (D == 3) {
            const int hiRun = (int)div_magic((unsigned)run0, (unsigned)L.size, L.magicSize);
            c[1] = j[1] * L.stride + (run0 - hiRun * L.size);
            c[0] = j[0] * L.stride + hiRun;
          }
          const unsigned p0 = site_key<D>(c, L.nIn);
          const unsigned present = get_bits(bitsA, (long long)p0, L.size);
          const unsigned rank0 = lds_rank(bitsA, prefA, p0);
          int *dst = st + (long long)rowB[rk] * L.width + run0 * L.size;
          for (int q = 0; q < L.size; ++q)
            dst[q] = (present >> q) & 1u
                         ? (int)rowA[rank0 + __popc(present & ((1u << q) - 1u))]
                         : bgA;
        }
      } else {
        const unsigned items = nB * (unsigned)L.width;
        for (unsigned it = t; it < items; it += CHAIN_THREADS) {
          const unsigned rk = div_magic(it, (unsigned)L.width, L.magicWidth);
          const int q = (int)(it - rk * L.width);
          int off = tri ? invOrd[q] : q;
          int j[D], c[D];
          unpack_site<D>(keyB[rk], j);
#pragma unroll
          for (int x = D - 1; x >= 0; --x) {
            const int hiOff = (int)div_magic((unsigned)off, (unsigned)L.size, L.magicSize);
            c[x] = j[x] * L.stride + (off - hiOff * L.size);
            off = hiOff;
          }
          const unsigned p = site_key<D>(c, L.nIn);
          const bool present = (bitsA[p >> 6] >> (p & 63)) & 1ull;
          st[(long long)rowB[rk] * L.width + q] =
              present ? (int)rowA[lds_rank(bitsA, prefA, p)] : bgA;
        }
      }
      if (hasBg) // the all-background row (Regions.cu:647-652)
        for (int q = t; q < L.width; q += CHAIN_THREADS)
          st[(long long)nB * L.width + q] = bgA;
    }
    lds_barrier();
    // the output grid is the next layer's input
    keyA = keyB;
    rowA = rowB;
    nA = nB;
    bgA = hasBg ? (int)nB : -1;
    vol = volOut;
  }
}

// Sums over the samples of a layer's counts: what lies before sample b, the
// totals, and the largest sample; and the first row of sample b in the layer's
// input (the same sums of the layer before).  Every lane adds up its samples,
// the lane sums meet in LDS and are folded in two short steps (a shuffle tree
// over six 64-bit values would cost this short kernel more than its copy).
#define PLACE_THREADS 256
struct PlaceSums {
  long long actBefore, bgBefore, actAll, bgAll, maxAct, inBase;
};
__device__ __forceinline__ PlaceSums place_sums(const int *cnt, const int *cntIn,
                                                int batch, int b,
                                                long long (*part)[PLACE_THREADS],
                                                long long (*fold)[8]) {
  const int t = threadIdx.x;
  long long v[6] = {0, 0, 0, 0, 0, 0};
  for (int s = t; s < batch; s += PLACE_THREADS) {
    const int n = cnt[2 * s], h = cnt[2 * s + 1];
    if (s < b) {
      v[0] += n;
      v[1] += h;
      if (cntIn)
        v[5] += cntIn[2 * s] + cntIn[2 * s + 1];
    }
    v[2] += n;
    v[3] += h;
    v[4] = n > v[4] ? n : v[4];
  }
#pragma unroll
  for (int k = 0; k < 6; ++k)
    part[k][t] = v[k];
  __syncthreads();
  if (t < 48) { // eight lanes a value, 32 lane sums each
    const int k = t >> 3, seg = t & 7;
    long long x = 0;
    for (int i = 0; i < PLACE_THREADS / 8; ++i) {
      const long long y = part[k][seg * (PLACE_THREADS / 8) + i];
      x = k == 4 ? (y > x ? y : x) : x + y;
    }
    fold[k][seg] = x;
  }
  __syncthreads();
  long long r[6];
#pragma unroll
  for (int k = 0; k < 6; ++k) {
    long long x = 0;
#pragma unroll
    for (int seg = 0; seg < 8; ++seg) {
      const long long y = fold[k][seg];
      x = k == 4 ? (y > x ? y : x) : x + y;
    }
    r[k] = x;
  }
  PlaceSums out;
  out.actBefore = r[0];
  out.bgBefore = r[1];
  out.actAll = r[2];
  out.bgAll = r[3];
  out.maxAct = r[4];
  out.inBase = r[5];
  return out;
}

__global__ void __launch_bounds__(PLACE_THREADS) k_chain_place(ChainArgs a) {
  __shared__ long long part[6][PLACE_THREADS];
  __shared__ long long fold[6][8];
  const int b = blockIdx.x, l = blockIdx.y, t = threadIdx.x;
  const ChainLevel &L = a.lv[l];
  const int *cnt = a.counts + (long long)l * a.batch * 2;
  const bool gaveUp = *reinterpret_cast<volatile unsigned long long *>(a.flag) == a.ticket;
  const PlaceSums me = place_sums(cnt, l > 0 ? cnt - (long long)a.batch * 2 : nullptr,
                                  a.batch, b, part, fold);
  const long long inBase = me.inBase; // first row of this sample in the layer's input
  const bool terminal = L.kind == CH_TERMINAL;
  long long nSites, nActive, width;
  bool over = gaveUp;
  if (terminal) {
    width = me.maxAct > 1 ? me.maxAct : 1; // TerminalPoolingLayer.cu:90-96
    nSites = nActive = a.batch;
    over = over || width > L.boundRows ||
           (L.rules && width * a.batch > L.capacity);
  } else {
    width = L.width;
    nSites = me.actAll + me.bgAll;
    nActive = me.actAll;
    over = over || nSites > L.boundRows || nActive > L.boundActive ||
           (L.rules && nSites * width > L.capacity);
  }
  if (b == 0 && t == 0) {
    L.meta[META_SITES] = over ? 0 : nSites;
    L.meta[META_ACTIVE] = over ? 0 : nActive;
    L.meta[META_OVERFLOW] = over;
    L.meta[META_WIDTH] = terminal ? width : 0;
    volatile long long *slot = a.scalars + 16 + 4 * L.slot;
    slot[0] = nSites;
    slot[1] = nActive;
    slot[2] = over;
    slot[3] = terminal ? width : me.maxAct;
    if (l == 0)
      a.scalars[15] = *a.badSites;
  }
  if (over)
    return;
  const int n = cnt[2 * b], hasBg = cnt[2 * b + 1];
  const int *st = a.staging + L.stRules + (long long)b * L.capRows * L.width;
  if (terminal) {
    if (L.rules) {
      const int have = n > 1 ? n : 1;
      int *dst = L.rules + (long long)b * width;
      for (long long i = t; i < width; i += PLACE_THREADS) {
        int v = -1;
        if (i < have) {
          v = st[i];
          v = v < 0 ? v : v + (int)inBase;
        }
        dst[i] = v;
      }
    }
    if (t == 0) { // the output grid: site 0 of sample b is row b
      L.ekey[b] = b;
      L.erow[b] = b;
      L.bg[b] = -1;
    }
    return;
  }
  const long long rowBase = me.actBefore + me.bgBefore;
  if (L.rules) {
    const long long total = (long long)(n + hasBg) * L.width;
    int *dst = L.rules + rowBase * L.width;
    // eight loads in flight per lane (the staged rows were written by the
    // kernel before this one: every load is a trip to the L2 at least)
    constexpr int PU = 8;
    const int total32 = (int)total; // capRows * width fits 31 bits
    int i = t;
    for (; i + (PU - 1) * PLACE_THREADS < total32; i += PU * PLACE_THREADS) {
      int v[PU];
#pragma unroll
      for (int u = 0; u < PU; ++u)
        v[u] = st[i + u * PLACE_THREADS];
#pragma unroll
      for (int u = 0; u < PU; ++u)
        dst[i + u * PLACE_THREADS] = v[u] < 0 ? v[u] : v[u] + (int)inBase;
    }
    for (; i < total32; i += PLACE_THREADS) {
      const int v = st[i];
      dst[i] = v < 0 ? v : v + (int)inBase;
    }
  }
  const int *stKey = a.staging + L.stKeys + (long long)b * L.capRows;
  long long volOut = 1;
  for (int q = 0; q < a.d; ++q)
    volOut *= L.nOut;
  for (int i = t; i < n; i += PLACE_THREADS) {
    L.ekey[me.actBefore + i] = (long long)b * volOut + stKey[i];
    L.erow[me.actBefore + i] = (int)(rowBase + i);
  }
  if (t == 0)
    L.bg[b] = hasBg ? (int)(rowBase + n) : -1;
}

// ------------------------------------------------ chains built from the output side
//
// scn_pyr_dev.h has the per-lane bodies; here are the two kernels around them.
// k_pyr_masks, one workgroup per sample: the occupancy masks of all layers
// (each the dilation of the one before), their rank prefixes and the sample's
// site counts, left in global memory.  k_pyr_rules, one workgroup per sample:
// everything per site, in sweeps over all layers at once -- the sums over the
// samples before (which k_pyr_masks has finished writing), sites by rank,
// owners, rows, entry lists and rule rows at their batch-global places.  Nothing
// is staged and nothing is copied afterwards.
// k_pyr_masks runs ONE wavefront per sample.  With four wavefronts per
// workgroup the kernel was measured to give wrong mask words now and then --
// only while workgroups of other streams' chains shared the compute units, with
// either kind of barrier, its arguments, its input and its own first level
// intact, and never with one chain at a time; the instruction stream shows
// every wait in place.  The cause was not found.  A single wavefront has no
// barrier to pass and gave no wrong word in any run; it costs a 126 x 126 field
// about 2 us and a 47^3 one about 20.
#define PYR_A_THREADS 64
#define PYR_A_BARRIER() lds_barrier()
#define PYR_B_THREADS 1024
static_assert(sizeof(PyrArgs) <= 4096, "kernel arguments");

// A layer's geometry as k_pyr_masks keeps it in LDS: one broadcast read a layer
// instead of trips to the kernel arguments
struct PyrGeoA {
  int nIn, nOut, size, stride;
  int words, offIn, offOut;
  unsigned magicN, seg, segs, magicSegs;
  int pad;
};
static_assert(sizeof(PyrGeoA) == 48, "three 16-byte reads");
#define PYR_A_EXTRA (128 + (PYR_MAX_LEVELS + 1) * (int)sizeof(PyrGeoA)) // counts, geometry: after the pyramid

// Rank prefixes of `words` mask words (the two spare words included) by one
// wavefront; the number of set bits comes back
__device__ __forceinline__ unsigned pyr_prefixes(const pyr_u64 *m, unsigned short *p, int words, int lane) {
  unsigned carry = 0;
  for (int w0 = 0; w0 < words + 2; w0 += 64) {
    const int w = w0 + lane;
    const unsigned pc = w < words ? (unsigned)pyr_popc64(m[w]) : 0u;
    const unsigned incl = wave_scan_incl_dpp(pc);
    if (w < words + 2)
      p[w] = (unsigned short)(carry + incl - pc);
    carry += wave_last(incl);
  }
  return carry;
}

template <int D>
__global__ void __launch_bounds__(PYR_A_THREADS) k_pyr_masks(PyrArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  pyr_u64 *masks = reinterpret_cast<pyr_u64 *>(lds);
  unsigned short *pref = reinterpret_cast<unsigned short *>(lds + 8ll * a.maskWords);
  int *cnt = reinterpret_cast<int *>(lds + 8ll * a.pyrStride);
  PyrGeoA *geo = reinterpret_cast<PyrGeoA *>(lds + 8ll * a.pyrStride + 128);
  const int b = blockIdx.x, t = threadIdx.x;
  static_assert(PYR_A_THREADS == 64, "one wavefront: the levels below pass no barrier");
  if (t >= 1 && t < a.nMasks) {
    const PyrLevel &L = a.lv[t];
    PyrGeoA g;
    g.nIn = L.nIn;
    g.nOut = L.nOut;
    g.size = L.size;
    g.stride = L.stride;
    g.words = L.words;
    g.offIn = a.lv[t - 1].maskOff;
    g.offOut = L.maskOff;
    g.magicN = L.magicN;
    g.seg = L.seg;
    g.segs = L.segs;
    g.magicSegs = L.magicSegs;
    g.pad = 0;
    geo[t] = g;
  }
  { // level 0: the sample's slice of the source mask, four words a lane at a time
    const PyrLevel &L = a.lv[0];
    const int words = L.words;
    const long long vol = L.volOut;
    unsigned carry = 0;
    for (int w0 = 0; w0 < words + 2; w0 += 256) {
      pyr_u64 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int w = w0 + 64 * u + t;
        v[u] = w < words ? pyr_source_word(a.bits, vol, b, (unsigned)w) : 0ull;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int w = w0 + 64 * u + t;
        const unsigned pc = (unsigned)pyr_popc64(v[u]);
        const unsigned incl = wave_scan_incl_dpp(pc);
        if (w < words + 2) {
          masks[w] = v[u];
          pref[w] = (unsigned short)(carry + incl - pc);
        }
        carry += wave_last(incl);
      }
    }
    if (t == 0)
      cnt[0] = (int)carry;
    // the other levels start empty: their pieces are OR-ed in
    for (int w = words + 2 + t; w < a.maskWords; w += PYR_A_THREADS)
      masks[w] = 0ull;
  }
  PYR_A_BARRIER();
  for (int x = 1; x < a.nMasks; ++x) {
    // (wavefront-uniform values, told to the compiler: the loops over a window's
    // rows then branch on scalars)
    PyrGeoA g = geo[x];
    g.nIn = __builtin_amdgcn_readfirstlane(g.nIn);
    g.nOut = __builtin_amdgcn_readfirstlane(g.nOut);
    g.size = __builtin_amdgcn_readfirstlane(g.size);
    g.stride = __builtin_amdgcn_readfirstlane(g.stride);
    g.words = __builtin_amdgcn_readfirstlane(g.words);
    g.offIn = __builtin_amdgcn_readfirstlane(g.offIn);
    g.offOut = __builtin_amdgcn_readfirstlane(g.offOut);
    g.magicN = (unsigned)__builtin_amdgcn_readfirstlane((int)g.magicN);
    g.seg = (unsigned)__builtin_amdgcn_readfirstlane((int)g.seg);
    g.segs = (unsigned)__builtin_amdgcn_readfirstlane((int)g.segs);
    g.magicSegs = (unsigned)__builtin_amdgcn_readfirstlane((int)g.magicSegs);
    pyr_sweep_dilate<D>(masks + g.offIn, masks + g.offOut, g.nIn, g.nOut, g.size, g.stride, g.magicN, g.seg, g.segs,
                        g.magicSegs, t, PYR_A_THREADS);
    PYR_A_BARRIER();
    const unsigned n = pyr_prefixes(masks + g.offOut, pref + g.offOut, g.words, t);
    if (t == 0)
      cnt[x] = (int)n;
    PYR_A_BARRIER();
  }
  {
    uint4 *dst = reinterpret_cast<uint4 *>(a.pyramid + (long long)b * a.pyrStride);
    const uint4 *src = reinterpret_cast<const uint4 *>(lds);
    for (int i = t; i < a.pyrStride / 2; i += PYR_A_THREADS)
      dst[i] = src[i];
  }
  if (t < a.nMasks) {
    int *c = a.counts + ((long long)t * a.batch + b) * 2;
    c[0] = cnt[t];
    c[1] = (long long)cnt[t] < a.lv[t].fullSize;
  }
  if (t == 0) {
    bool fits = pyr_fits(a, cnt);
    for (int x = 0; x < a.nMasks; ++x)
      fits = fits && cnt[x] <= PYR_ROWS_MAX;
    if (!fits)
      atomicMax(a.flag, a.ticket);
  }
}

template <int D>
__global__ void __launch_bounds__(PYR_B_THREADS) k_pyr_rules(PyrArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  PyrHdr *h = reinterpret_cast<PyrHdr *>(lds);
  const int b = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  constexpr int T = PYR_B_THREADS;
  const bool gaveUp = *reinterpret_cast<volatile unsigned long long *>(a.flag) == a.ticket;
  // lane t keeps layer t's arguments from here on: fetched while the masks
  // come in, not when the level table wants them
  PyrLevel mine;
  int inMaskOff = 0;
  const int bgSource = a.bg[b];
  if (t <= a.nLevels) {
    mine = a.lv[t];
    inMaskOff = a.lv[t > 0 ? t - 1 : 0].maskOff;
  }
  if (t == 0)
    h->over = 0;
  { // the sample's masks and prefixes
    const uint4 *src = reinterpret_cast<const uint4 *>(a.pyramid + (long long)b * a.pyrStride);
    uint4 *dst = reinterpret_cast<uint4 *>(lds + PYR_HDR_BYTES);
    for (int i = t; i < a.pyrStride / 2; i += T)
      dst[i] = src[i];
  }
  // sums over the samples, a wavefront per level
  for (int x = wave; x < a.nMasks; x += T / 64) {
    const int *cnt = a.counts + (long long)x * a.batch * 2;
    // (a batch's rows are numbered in 32 bits, so these sums fit)
    unsigned v0 = 0, v1 = 0, v2 = 0, v3 = 0;
    int mx = 0;
    for (int s = lane; s < a.batch; s += 64) {
      const int2 c = reinterpret_cast<const int2 *>(cnt)[s];
      const int n = c.x, hb = c.y;
      if (s < b) {
        v0 += n;
        v1 += hb;
      }
      v2 += n;
      v3 += hb;
      mx = n > mx ? n : mx;
    }
    v0 = wave_last(wave_scan_incl_dpp(v0));
    v1 = wave_last(wave_scan_incl_dpp(v1));
    v2 = wave_last(wave_scan_incl_dpp(v2));
    v3 = wave_last(wave_scan_incl_dpp(v3));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const int o = __shfl_xor(mx, off, 64);
      mx = o > mx ? o : mx;
    }
    if (lane == 0) {
      h->n[x] = cnt[2 * b];
      h->hasBg[x] = cnt[2 * b + 1];
      h->actBefore[x] = v0;
      h->bgBefore[x] = v1;
      h->actAll[x] = v2;
      h->bgAll[x] = v3;
      h->maxAct[x] = mx;
    }
  }
  lds_barrier();
  if (t >= 1 && t <= a.nLevels && pyr_report(a, mine, h, t).over)
    atomicOr(&h->over, 1);
  if (t == 0 && !pyr_fits(a, h->n))
    atomicOr(&h->over, 2);
  lds_barrier();
  const bool over = h->over != 0 || gaveUp;
  if (b == 0 && t >= 1 && t <= a.nLevels) {
    const PyrLevel &L = mine;
    const PyrReport r = pyr_report(a, mine, h, t);
    L.meta[META_SITES] = over ? 0 : r.nSites;
    L.meta[META_ACTIVE] = over ? 0 : r.nActive;
    L.meta[META_OVERFLOW] = over;
    L.meta[META_WIDTH] = L.kind == PYR_TERMINAL ? r.extra : 0;
    volatile long long *slot = a.scalars + 16 + 4 * L.slot;
    slot[0] = r.nSites;
    slot[1] = r.nActive;
    slot[2] = over;
    slot[3] = r.extra;
  }
  if (b == 0 && t == 0) {
    a.scalars[15] = *a.badSites;
    a.scalars[13] = h->maxAct[0];
  }
  if (over)
    return;
  // the layers a window of levels at a time: as many as the LDS holds (all of
  // them, for all but the largest samples)
  for (int xa = 0;;) {
    const int xb = pyr_window_end(a, h->n, xa);
    const int la = xa + 1, lb = xb;
    const bool last = xb == a.nMasks - 1;
    pyr_fill_offsets(h, xa, xb, t);
    lds_barrier();
    if (t < a.nMasks)
      pyr_fill_en(mine, lds, t, h->siteOff[t]);
    const PyrLds s = pyr_lds_view(a, lds, h->total, h->n[xa]);
    if ((t >= la && t <= lb) || (last && t == a.nLevels && t > lb))
      pyr_fill_level(mine, inMaskOff, bgSource, s, t, xa);
    pyr_sweep_clear(s, t, T);
    lds_barrier();
    pyr_sweep_enumerate<D>(a, s, xa, xb, t, T);
    lds_barrier();
    if (xa == 0) { // the batch's rows of the source's sites: their loads go out first
      const PyrLevel &L = a.lv[0];
      const long long p0 = (long long)b * L.volOut;
      const Slot *table = reinterpret_cast<const Slot *>(a.table);
      for (int r = t; r < h->n[0]; r += T) {
        int c[D];
        pyr_unpack<D>(s.key[r], c);
        long long p = p0 + pyr_key<D>(c, L.nOut);
        p = p < (long long)a.batch * L.volOut ? p : 0; // (a mask never has a site beyond the field)
        s.srcRow[r] = (unsigned)(a.dense ? a.dense[p] : hash_find(table, a.shift, a.mask, p));
      }
    }
    pyr_sweep_owners<D>(s, la, lb, t, T);
    lds_barrier();
    // rows owned by the sites before, a wavefront per level
    for (int x = xa + wave; x < xb; x += T / 64) {
      const int n = h->n[x];
      const unsigned off = (unsigned)h->siteOff[x];
      unsigned carry = 0;
      for (int r0 = 0; r0 < n; r0 += 64) {
        const int r = r0 + lane;
        const unsigned v = r < n ? (unsigned)pyr_popc32(pyr_own_mask(s, off + r)) : 0u;
        const unsigned incl = wave_scan_incl_dpp(v);
        if (r < n)
          s.base[off + r] = (unsigned short)(carry + incl - v);
        carry += wave_last(incl);
      }
    }
    lds_barrier();
    pyr_sweep_rows<D>(s, la, lb, b, t, T);
    lds_barrier();
    pyr_sweep_rules<D>(s, la, lb, t, T);
    pyr_sweep_tail(a, s, la, lb, b, t, T);
    if (last)
      break;
    lds_barrier();
    pyr_sweep_carry(s, lds, a, xb, t, T);
    lds_barrier();
    xa = xb;
  }
}

// -------------------------------------------------------------------- host

static ChainState *chain_state(scn_ctx *ctx) {
  if (!ctx->chain) {
    ctx->chain = new ChainState();
    // SCN_CHAIN_PYRAMID=0: a diagnostic switch for A/B runs, every chain through
    // k_chain_sample / k_chain_place (the rule books are the same)
    const char *e = getenv("SCN_CHAIN_PYRAMID");
    if (e && e[0] == '0')
      ctx->chain->pyramids = false;
  }
  return ctx->chain;
}

void scn_chain_release(scn_ctx *ctx) {
  if (!ctx->chain)
    return;
  ctx->chain->staging.release();
  ctx->chain->counts.release();
  ctx->chain->flag.release();
  ctx->chain->pyramid.release();
  delete ctx->chain;
  ctx->chain = nullptr;
}

extern "C" int scn_ctx_chain_rules(scn_ctx *ctx, int on) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_ctx_chain_rules: null context");
  if (!on)
    SCN_TRY(scn_chain_flush(ctx));
  chain_state(ctx)->on = on != 0;
  return SCN_OK;
}

extern "C" int scn_ctx_chain_count(scn_ctx *ctx, int64_t *chains, int64_t *plans) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_ctx_chain_count: null context");
  if (chains)
    *chains = ctx->chain ? ctx->chain->nChains : 0;
  if (plans)
    *plans = ctx->chain ? ctx->chain->nPlans : 0;
  return SCN_OK;
}

// LDS bytes of everything but the arena for a chain over grids of these
// volumes (the source first); fills the layout when `a` is given
static long long chain_fixed_lds(const std::vector<long long> &vols, ChainArgs *a) {
  long long mw[3] = {1, 1, 1}, pw[2] = {1, 1};
  for (size_t k = 0; k < vols.size(); ++k) {
    const long long w = (vols[k] + 63) / 64 + 1;
    mw[k % 3] = w > mw[k % 3] ? w : mw[k % 3];
    pw[k & 1] = w > pw[k & 1] ? w : pw[k & 1];
  }
  long long off = CHAIN_HEADER_BYTES;
  for (int x = 0; x < 3; ++x) {
    if (a) {
      a->maskOff[x] = (int)off;
      a->maskWords[x] = (int)mw[x];
    }
    off += 8 * mw[x];
  }
  for (int x = 0; x < 2; ++x) {
    if (a)
      a->prefOff[x] = (int)off;
    off += (2 * pw[x] + 15) / 16 * 16;
  }
  if (a)
    a->arenaOff = (int)off;
  return off;
}

static std::vector<long long> chain_volumes(const ChainState *cs) {
  std::vector<long long> vols;
  if (cs->recs.empty())
    return vols;
  vols.push_back(cs->recs[0].in->vol);
  for (const ChainRec &r : cs->recs)
    if (r.lv.kind == CH_REGIONS)
      vols.push_back(r.geom.volOut);
  return vols;
}

// Can a plan from `in` into `out` join the chain being recorded?
static bool chain_accepts(scn_ctx *ctx, const scn_grids *in, const scn_grids *out,
                          long long volOut) {
  ChainState *cs = ctx->chain;
  if (!cs || !cs->on || !ctx->deferCounts)
    return false;
  if ((int)ctx->pendingGrids.size() >= SCN_MAX_PENDING ||
      (int)cs->recs.size() >= CHAIN_MAX_LEVELS)
    return false;
  if (in->batch < 1 || in->d < 1 || in->d > 3 || in->vol >= (1ll << 31))
    return false;
  // sites travel as packed coordinates: 30, 15 or 10 bits an axis
  if (in->n >= (in->d == 1 ? (1 << 30) : (in->d == 2 ? (1 << 15) : (1 << 10))))
    return false;
  if (cs->recs.empty()) {
    // the source: grids with a table and a mask, counts known
    if (in->pending || !in->indexValid)
      return false;
  } else {
    const ChainRec &last = cs->recs.back();
    if (last.out != in || last.lv.kind == CH_TERMINAL)
      return false;
  }
  for (const ChainRec &r : cs->recs)
    if (r.out == out || r.in == out)
      return false;
  std::vector<long long> vols = chain_volumes(cs);
  if (vols.empty())
    vols.push_back(in->vol);
  vols.push_back(volOut);
  return chain_fixed_lds(vols, nullptr) + CHAIN_MIN_ARENA <= CHAIN_LDS_MAX;
}

static void chain_mark_output(scn_ctx *ctx, scn_grids *in, scn_grids *out,
                              int n, long long vol, long long boundActive,
                              long long boundRows, int slot) {
  out->batch = in->batch;
  out->d = in->d;
  out->n = n;
  out->vol = vol;
  out->nActive = boundActive;
  out->nSites = (int)boundRows;
  out->rankValid = false;
  out->rankRowValid = false;
  out->tableValid = false;
  out->indexValid = false;
  out->chained = true;
  out->planIn = in;
  mark_pending(ctx, out, slot);
}

int scn_chain_record_regions(scn_ctx *ctx, scn_grids *in, scn_grids *out,
                             const Geom &g, long long fullSize,
                             long long maxCand, int64_t *nOutSites,
                             bool *taken) {
  *taken = false;
  if (g.mode == MODE_SQ_FMP || maxCand > 32 || g.cube > 64 || out->seenRows <= 0 ||
      !chain_accepts(ctx, in, out, g.volOut))
    return SCN_OK;
  ChainState *cs = ctx->chain;
  const long long volOutAll = (long long)in->batch * g.volOut;
  const long long boundActive = grow_bound(out->seenActive, 64, volOutAll);
  const long long boundRows = grow_bound(out->seenRows, 64, boundActive + in->batch);
  if (boundRows >= 2147483647ll)
    return SCN_OK;
  SCN_TRY(out->meta.reserve(8));
  SCN_TRY(out->ekey.reserve((size_t)boundActive + 1));
  SCN_TRY(out->erow.reserve((size_t)boundActive + 1));
  SCN_TRY(out->bg.reserve((size_t)in->batch + 1));
  ChainRec r;
  r.in = in;
  r.out = out;
  r.geom = g;
  r.filled = false;
  ChainLevel &L = r.lv;
  memset(&L, 0, sizeof(L));
  L.kind = CH_REGIONS;
  L.mode = g.mode;
  L.nIn = g.nIn;
  L.nOut = g.nOut;
  L.size = g.size;
  L.stride = g.stride;
  L.minActive = g.minActive;
  L.width = g.width;
  L.cube = g.cube;
  L.fullSize = fullSize;
  L.magicRuns = (unsigned)((1ull << 32) / (unsigned)(g.width / g.size > 0 ? g.width / g.size : 1) + 1);
  L.magicWidth = (unsigned)((1ull << 32) / (unsigned)g.width + 1);
  L.magicSize = (unsigned)((1ull << 32) / (unsigned)g.size + 1);
  L.magicStride = (unsigned)((1ull << 32) / (unsigned)g.stride + 1);
  L.slot = (int)ctx->pendingGrids.size();
  L.ekey = out->ekey.p;
  L.erow = out->erow.p;
  L.bg = out->bg.p;
  L.meta = out->meta.p;
  L.boundRows = boundRows;
  L.boundActive = boundActive;
  cs->recs.push_back(r);
  chain_mark_output(ctx, in, out, g.nOut, g.volOut, boundActive, boundRows, L.slot);
  out->geom = g;
  out->planKind = PLAN_REGIONS;
  *nOutSites = boundRows;
  *taken = true;
  return SCN_OK;
}

int scn_chain_record_terminal(scn_ctx *ctx, scn_grids *in, scn_grids *out,
                              int64_t *ruleWidth, bool *taken) {
  *taken = false;
  if (out->seenWidth <= 0 || !chain_accepts(ctx, in, out, 1))
    return SCN_OK;
  ChainState *cs = ctx->chain;
  const long long boundWidth = grow_bound(out->seenWidth, 8, in->vol);
  SCN_TRY(out->meta.reserve(8));
  SCN_TRY(out->ekey.reserve((size_t)in->batch + 1));
  SCN_TRY(out->erow.reserve((size_t)in->batch + 1));
  SCN_TRY(out->bg.reserve((size_t)in->batch + 1));
  ChainRec r;
  r.in = in;
  r.out = out;
  memset(&r.geom, 0, sizeof(r.geom));
  r.geom.volOut = 1;
  r.filled = false;
  ChainLevel &L = r.lv;
  memset(&L, 0, sizeof(L));
  L.kind = CH_TERMINAL;
  L.nOut = 1;
  L.width = 1;
  L.fullSize = 1;
  L.slot = (int)ctx->pendingGrids.size();
  L.ekey = out->ekey.p;
  L.erow = out->erow.p;
  L.bg = out->bg.p;
  L.meta = out->meta.p;
  L.boundRows = boundWidth;
  L.boundActive = in->batch;
  cs->recs.push_back(r);
  chain_mark_output(ctx, in, out, 1, 1, in->batch, in->batch, L.slot);
  out->termS = boundWidth;
  out->planKind = PLAN_TERMINAL;
  *ruleWidth = boundWidth;
  *taken = true;
  return SCN_OK;
}

int scn_chain_record_fill(scn_ctx *ctx, const scn_grids *in, scn_grids *out,
                          int32_t *d_rules, int64_t capacity, bool *taken) {
  *taken = false;
  ChainState *cs = ctx->chain;
  if (!cs || cs->recs.empty())
    return SCN_OK;
  ChainRec &r = cs->recs.back();
  if (r.out != out || r.in != in || r.filled)
    return SCN_OK;
  const long long total = r.lv.kind == CH_TERMINAL
                              ? (long long)in->batch * out->termS
                              : (long long)out->nSites * r.lv.width;
  SCN_REQUIRE(capacity >= total, SCN_ERR_CAPACITY,
              "scn_rules_fill: %lld rules, capacity %lld", total,
              (long long)capacity);
  SCN_REQUIRE(d_rules || total == 0, SCN_ERR_ARG,
              "scn_rules_fill: null rules buffer");
  r.lv.rules = d_rules;
  r.lv.capacity = capacity;
  r.filled = true;
  *taken = true;
  return SCN_OK;
}

// Chains of square layers without a minimum (and a terminal layer at the end)
// are built from the output side by k_pyr_masks / k_pyr_rules.  *done = false:
// this chain is not of that kind (or its masks do not fit), run it the other way.
static int chain_flush_pyramid(scn_ctx *ctx, ChainState *cs, std::vector<ChainRec> &recs,
                               bool *done) {
  *done = false;
  scn_grids *src = recs[0].in;
  const int d = src->d;
  for (size_t i = 0; i < recs.size(); ++i) {
    const ChainLevel &L = recs[i].lv;
    if (L.kind == CH_TERMINAL) {
      if (i + 1 != recs.size())
        return SCN_OK;
      continue;
    }
    if (L.mode != MODE_SQ_NOMIN || L.cube > PYR_CUBE_MAX || L.size < 1 ||
        (d >= 2 && L.size > 4) || L.stride < 1)
      return SCN_OK;
    if ((uintptr_t)L.rules & 15) // (rule rows are stored two or four entries at a time)
      return SCN_OK;
  }
  if ((int)recs.size() > PYR_MAX_LEVELS)
    return SCN_OK;
  PyrArgs a;
  memset(&a, 0, sizeof(a));
  a.nLevels = (int)recs.size();
  a.batch = src->batch;
  a.d = d;
  auto magic = [](long long x) { return (unsigned)((1ull << 32) / (unsigned long long)(x > 0 ? x : 1) + 1); };
  long long maskWords = 0;
  {
    PyrLevel &L = a.lv[0];
    L.kind = PYR_REGIONS;
    L.nIn = L.nOut = src->n;
    L.size = L.stride = L.width = 1;
    L.volOut = src->vol;
    L.fullSize = src->vol + 1; // (the source's background rows are the caller's)
    L.words = (int)((src->vol + 63) / 64);
    L.maskOff = 0;
    L.magicN = magic(src->n);
    L.magicS = magic(1);
    maskWords = L.words + 2;
  }
  a.nMasks = 1;
  for (int l = 1; l <= a.nLevels; ++l) {
    const ChainRec &r = recs[l - 1];
    PyrLevel &L = a.lv[l];
    L.kind = r.lv.kind == CH_TERMINAL ? PYR_TERMINAL : PYR_REGIONS;
    L.nIn = r.lv.nIn;
    L.nOut = r.lv.nOut;
    L.size = r.lv.size;
    L.stride = r.lv.stride;
    L.width = r.lv.width;
    L.volOut = r.geom.volOut;
    L.fullSize = r.lv.fullSize;
    L.magicN = magic(L.nOut);
    L.magicS = magic(L.size);
    pyr_set_pieces(L);
    L.rules = r.lv.rules;
    L.capacity = r.lv.capacity;
    L.ekey = r.lv.ekey;
    L.erow = r.lv.erow;
    L.bg = r.lv.bg;
    L.meta = r.lv.meta;
    L.boundRows = r.lv.boundRows;
    L.boundActive = r.lv.boundActive;
    L.slot = r.lv.slot;
    if (L.kind == PYR_REGIONS) {
      L.words = (int)((L.volOut + 63) / 64);
      L.maskOff = (int)maskWords;
      maskWords += L.words + 2;
      a.nMasks = l + 1;
    }
  }
  long long pyrStride = maskWords + (maskWords + 3) / 4;
  pyrStride = (pyrStride + 1) / 2 * 2;
  const long long fixedB = PYR_HDR_BYTES + 8 * pyrStride + 6 * 16;
  if (fixedB + CHAIN_MIN_ARENA > PYR_LDS_MAX)
    return SCN_OK;
  a.maskWords = (int)maskWords;
  a.pyrStride = (int)pyrStride;
  // pass B's LDS: from the largest samples seen at every level, or all there is
  long long ldsB = PYR_LDS_MAX;
  {
    bool known = !cs->wide && src->seenSample > 0;
    long long sites = src->seenSample + src->seenSample / 2 + 64;
    long long need = 15 * sites;
    for (int l = 1; l < a.nMasks; ++l) {
      const long long seen = recs[l - 1].out->seenSample;
      known = known && seen > 0;
      need += 11 * (seen + seen / 2 + 64);
    }
    if (known) {
      need += fixedB;
      ldsB = need < ldsB ? need : ldsB;
    }
  }
  ldsB = (ldsB + 15) / 16 * 16;
  a.ldsBytesB = (int)ldsB;
  cs->pyrAtMax = ldsB >= PYR_LDS_MAX;
  *done = true;
  cs->nPyramids += 1;
  SCN_TRY(scn_grids_ensure_table(ctx, src)); // pass B reads the source's rows through it
  a.table = src->table.p;
  a.dense = (long long)src->batch * src->vol <= SCN_DENSE_MAX_SITES ? src->dense.p : nullptr;
  a.shift = 64 - src->log2cap;
  a.mask = (1u << src->log2cap) - 1u;
  a.bits = src->bits.p;
  a.bg = src->bg.p;
  SCN_TRY(cs->pyramid.reserve((size_t)a.batch * (size_t)pyrStride + 2));
  SCN_TRY(cs->counts.reserve((size_t)a.nMasks * a.batch * 2 + 2));
  if (!cs->flag.p) {
    SCN_TRY(cs->flag.reserve(2));
    SCN_TRY(scn_fill32(ctx, cs->flag.p, 0u, 4));
  }
  a.pyramid = cs->pyramid.p;
  a.counts = cs->counts.p;
  a.flag = cs->flag.p;
  a.ticket = (unsigned long long)++ctx->ticket;
  a.scalars = (long long *)ctx->d_pinned;
  a.badSites = (const long long *)(ctx->d_scalars + 15);
  cs->pyrSource = src;
  {
    // (above 64 KB of LDS a kernel has to be told so once)
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
      const void *k[6] = {reinterpret_cast<const void *>(&k_pyr_masks<1>),
                          reinterpret_cast<const void *>(&k_pyr_masks<2>),
                          reinterpret_cast<const void *>(&k_pyr_masks<3>),
                          reinterpret_cast<const void *>(&k_pyr_rules<1>),
                          reinterpret_cast<const void *>(&k_pyr_rules<2>),
                          reinterpret_cast<const void *>(&k_pyr_rules<3>)};
      for (int i = 0; i < 6 && attr == hipSuccess; ++i)
        attr = hipFuncSetAttribute(k[i], hipFuncAttributeMaxDynamicSharedMemorySize,
                                   CHAIN_LDS_MAX);
    });
    SCN_HIP_CHECK(attr);
  }
  const size_t ldsA = (size_t)(8 * pyrStride + PYR_A_EXTRA);
  const dim3 grid((unsigned)a.batch);
  switch (d) {
  case 1:
    hipLaunchKernelGGL(k_pyr_masks<1>, grid, dim3(PYR_A_THREADS), ldsA, ctx->stream, a);
    hipLaunchKernelGGL(k_pyr_rules<1>, grid, dim3(PYR_B_THREADS), (size_t)ldsB, ctx->stream, a);
    break;
  case 2:
    hipLaunchKernelGGL(k_pyr_masks<2>, grid, dim3(PYR_A_THREADS), ldsA, ctx->stream, a);
    hipLaunchKernelGGL(k_pyr_rules<2>, grid, dim3(PYR_B_THREADS), (size_t)ldsB, ctx->stream, a);
    break;
  default:
    hipLaunchKernelGGL(k_pyr_masks<3>, grid, dim3(PYR_A_THREADS), ldsA, ctx->stream, a);
    hipLaunchKernelGGL(k_pyr_rules<3>, grid, dim3(PYR_B_THREADS), (size_t)ldsB, ctx->stream, a);
    break;
  }
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

int scn_chain_flush(scn_ctx *ctx) {
  ChainState *cs = ctx->chain;
  if (!cs || cs->recs.empty())
    return SCN_OK;
  std::vector<ChainRec> recs;
  recs.swap(cs->recs);
  cs->nChains += 1;
  cs->nPlans += (long long)recs.size();
  ProfScope ps(ctx, SCN_K_RULES);
  scn_grids *src = recs[0].in;
  if (cs->pyramids) {
    bool done = false;
    SCN_TRY(chain_flush_pyramid(ctx, cs, recs, &done));
    if (done)
      return SCN_OK;
  }
  SCN_TRY(scn_grids_ensure_table(ctx, src)); // the kernel reads the source's rows through it
  ChainArgs a;
  memset(&a, 0, sizeof(a));
  a.nLevels = (int)recs.size();
  a.batch = src->batch;
  a.d = src->d;
  a.n0 = src->n;
  a.table = src->table.p;
  a.dense = (long long)src->batch * src->vol <= SCN_DENSE_MAX_SITES ? src->dense.p : nullptr;
  a.shift = 64 - src->log2cap;
  a.mask = (1u << src->log2cap) - 1u;
  a.bits = src->bits.p;
  a.bg = src->bg.p;
  a.vol0 = src->vol;
  std::vector<long long> vols;
  vols.push_back(src->vol);
  for (const ChainRec &r : recs)
    if (r.lv.kind == CH_REGIONS)
      vols.push_back(r.geom.volOut);
  const long long fixed = chain_fixed_lds(vols, &a);
  // the arena: sized from the largest sample seen at any layer, or as large
  // as the LDS allows while that is unknown or has proved too tight
  long long arena = CHAIN_LDS_MAX - fixed;
  long long sampleBound = 0;
  bool known = !cs->wide;
  for (const ChainRec &r : recs)
    if (r.lv.kind == CH_REGIONS) {
      known = known && r.out->seenSample > 0;
      sampleBound = r.out->seenSample > sampleBound ? r.out->seenSample : sampleBound;
    }
  if (known) {
    sampleBound += sampleBound / 2 + 64;
    long long want = (CHAIN_IN_BYTES + CHAIN_OUT_BYTES) * sampleBound;
    want = want < CHAIN_MIN_ARENA ? CHAIN_MIN_ARENA : want;
    arena = want < arena ? want : arena;
  }
  arena = arena / 16 * 16;
  a.arenaBytes = (int)arena;
  const long long entriesMax = arena / CHAIN_OUT_BYTES;
  long long stagingInts = 0;
  for (int l = 0; l < a.nLevels; ++l) {
    ChainLevel &L = recs[l].lv;
    long long cap = entriesMax < L.fullSize ? entriesMax : L.fullSize;
    if (L.kind == CH_TERMINAL)
      cap = entriesMax; // rows of the input that one sample may list
    else if (known) {
      const long long tight = 2 * recs[l].out->seenSample + 64;
      cap = tight < cap ? tight : cap;
    }
    L.capRows = (int)cap + 1;
    L.stRules = stagingInts;
    stagingInts += (long long)a.batch * L.capRows * L.width;
    stagingInts = (stagingInts + 3) / 4 * 4;
    L.stKeys = stagingInts;
    stagingInts += (long long)a.batch * L.capRows;
    stagingInts = (stagingInts + 3) / 4 * 4;
    a.lv[l] = L;
  }
  SCN_TRY(cs->staging.reserve((size_t)stagingInts + 4));
  SCN_TRY(cs->counts.reserve((size_t)a.nLevels * a.batch * 2 + 2));
  if (!cs->flag.p) {
    SCN_TRY(cs->flag.reserve(2));
    SCN_TRY(scn_fill32(ctx, cs->flag.p, 0u, 4));
  }
  a.staging = cs->staging.p;
  a.counts = cs->counts.p;
  a.flag = cs->flag.p;
  a.ticket = (unsigned long long)++ctx->ticket;
  a.scalars = (long long *)ctx->d_pinned;
  a.badSites = (const long long *)(ctx->d_scalars + 15);
  const size_t ldsBytes = (size_t)(fixed + arena);
  {
    // (above 64 KB of LDS a kernel has to be told so once)
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
      const void *k[3] = {reinterpret_cast<const void *>(&k_chain_sample<1>),
                          reinterpret_cast<const void *>(&k_chain_sample<2>),
                          reinterpret_cast<const void *>(&k_chain_sample<3>)};
      for (int i = 0; i < 3 && attr == hipSuccess; ++i)
        attr = hipFuncSetAttribute(k[i], hipFuncAttributeMaxDynamicSharedMemorySize,
                                   CHAIN_LDS_MAX);
    });
    SCN_HIP_CHECK(attr);
  }
  const dim3 grid((unsigned)a.batch), block(CHAIN_THREADS);
  switch (a.d) {
  case 1:
    hipLaunchKernelGGL(k_chain_sample<1>, grid, block, ldsBytes, ctx->stream, a);
    break;
  case 2:
    hipLaunchKernelGGL(k_chain_sample<2>, grid, block, ldsBytes, ctx->stream, a);
    break;
  default:
    hipLaunchKernelGGL(k_chain_sample<3>, grid, block, ldsBytes, ctx->stream, a);
    break;
  }
  SCN_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(k_chain_place, dim3((unsigned)a.batch, (unsigned)a.nLevels),
                     dim3(PLACE_THREADS), 0, ctx->stream, a);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// what scn_rules_settle learns about a chained plan from its pinned slot
void scn_chain_settled(scn_ctx *ctx, scn_grids *g, long long sampleMax,
                       bool overflowed) {
  bool pyramid = false; // the first layer of a chain built from the output side
  if (ctx->chain && ctx->chain->pyrSource) {
    // its source's largest sample
    scn_grids *src = ctx->chain->pyrSource;
    const long long m = ctx->h_pinned[13];
    if (!overflowed)
      src->seenSample = m > src->seenSample ? m : src->seenSample;
    ctx->chain->pyrSource = nullptr;
    pyramid = true;
  }
  if (overflowed) {
    if (ctx->chain) {
      // a sample one of whose layers does not fit the LDS with its input may
      // still fit the other construction, which keeps less per site; a context
      // that meets such samples time and again stops trying
      if (pyramid && ctx->chain->wide && ctx->chain->pyrAtMax && ++ctx->chain->pyrMisses >= 3)
        ctx->chain->pyramids = false;
      ctx->chain->wide = true;
    }
    return;
  }
  if (pyramid && ctx->chain)
    ctx->chain->pyrMisses = 0;
  if (g->planKind == PLAN_REGIONS)
    g->seenSample = sampleMax > g->seenSample ? sampleMax : g->seenSample;
}
