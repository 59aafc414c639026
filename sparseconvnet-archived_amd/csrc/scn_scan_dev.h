// Device-side exclusive prefix sum by ONE workgroup of 1024 lanes.  For arrays
// up to 65536 elements this is one launch instead of the three of the tiled
// scan, and launch count is what small batches pay for.
//
// Every lane owns 32 (or 64) consecutive elements and keeps them in registers: all of
// its loads are issued back to back (one memory latency, not one per load),
// the 1024 lane sums are scanned through wavefront shuffles and 17 words of
// LDS, and the prefixes are written from the registers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SCAN1_THREADS 1024
// elements per lane: 32, or 64 for arrays of up to 65536 elements (64 value
// registers per lane, which a 1024-lane workgroup can still afford)
#define SCAN1_SMALL_ELEMS (SCAN1_THREADS * 32)
#define SCAN1_MAX_ELEMS (SCAN1_THREADS * 64)

// Four consecutive elements starting at i (i % 4 == 0); elements at or past n
// read as zero.  The loads are unconditional: a group that starts past the end
// reads group 0 instead, and the group that straddles n reads up to 12 bytes
// (24 for 64-bit words) past it -- inside the same aligned 16 / 32 bytes, so
// which the caller must have allocated (in must be 16-byte aligned).
template <bool POPC>
__device__ __forceinline__ uint4 scan1_load4(const void *in, size_t i, size_t n) {
  const size_t at = i < n ? i : 0;
  uint4 v;
  if (POPC) {
    const ulonglong2 *p =
        reinterpret_cast<const ulonglong2 *>((const unsigned long long *)in + at);
    const ulonglong2 a = p[0], b = p[1];
    v = make_uint4(__popcll(a.x), __popcll(a.y), __popcll(b.x), __popcll(b.y));
  } else {
    v = *reinterpret_cast<const uint4 *>((const uint32_t *)in + at);
  }
  v.x = i < n ? v.x : 0u;
  v.y = i + 1 < n ? v.y : 0u;
  v.z = i + 2 < n ? v.z : 0u;
  v.w = i + 3 < n ? v.w : 0u;
  return v;
}

// out[i] = sum of in[0..i), out[n] = total, n <= 1024 SCAN1_PER_LANE.  Must be
// called by all 1024 lanes of a workgroup; lds needs 17 words; in and out
// 16-byte aligned.  Returns the total to every lane.
template <bool POPC, int SCAN1_PER_LANE>
__device__ __forceinline__ uint32_t block_scan_loop(const void *in,
                                                    uint32_t *out, size_t n,
                                                    uint32_t *lds) {
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  if (n == 0) { // nothing to read (in may be null); uniform, so no barrier is skipped by some
    if (t == 0)
      out[0] = 0;
    return 0;
  }
  const size_t start = (size_t)t * SCAN1_PER_LANE;
  uint4 v[SCAN1_PER_LANE / 4];
#pragma unroll
  for (int j = 0; j < SCAN1_PER_LANE / 4; ++j)
    v[j] = scan1_load4<POPC>(in, start + 4 * j, n);
  uint32_t s = 0;
#pragma unroll
  for (int j = 0; j < SCAN1_PER_LANE / 4; ++j)
    s += v[j].x + v[j].y + v[j].z + v[j].w;
  // inclusive scan of s across the wavefront, then across the 16 wavefronts
  uint32_t incl = s;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    uint32_t up = __shfl_up(incl, off, 64);
    if (lane >= off)
      incl += up;
  }
  if (lane == 63)
    lds[wave] = incl;
  __syncthreads();
  if (wave == 0) {
    uint32_t w = lane < 16 ? lds[lane] : 0u;
    uint32_t wi = w;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      uint32_t up = __shfl_up(wi, off, 64);
      if (lane >= off)
        wi += up;
    }
    if (lane < 16)
      lds[lane] = wi - w; // exclusive offset of each wavefront
    if (lane == 15)
      lds[16] = wi; // grand total
  }
  __syncthreads();
  uint32_t run = lds[wave] + (incl - s);
  const uint32_t total = lds[16];
#pragma unroll
  for (int j = 0; j < SCAN1_PER_LANE / 4; ++j) {
    uint4 o;
    o.x = run;
    o.y = o.x + v[j].x;
    o.z = o.y + v[j].y;
    o.w = o.z + v[j].z;
    run = o.w + v[j].w;
    const size_t i = start + 4 * j;
    if (i + 4 <= n) {
      *reinterpret_cast<uint4 *>(out + i) = o;
    } else if (i < n) {
      out[i] = o.x;
      if (i + 1 < n)
        out[i + 1] = o.y;
      if (i + 2 < n)
        out[i + 2] = o.z;
    }
  }
  if (t == 0)
    out[n] = total;
  __syncthreads();
  return total;
}
