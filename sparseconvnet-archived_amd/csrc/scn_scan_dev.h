// Device-side exclusive prefix sum by ONE workgroup of 256 lanes.  For arrays
// up to SCAN1_MAX_ELEMS elements this is one launch instead of the three of the tiled
// scan, and launch count is what small batches pay for.
//
// The workgroup walks the array in chunks of 8192 elements.  Every lane owns
// 32 consecutive elements of a chunk and keeps them in registers: all of its
// loads are issued back to back (one memory latency, not one per load), the
// next chunk's loads are in flight while this chunk is scanned, the 256 lane
// sums are scanned through wavefront shuffles and a few words of LDS, and the
// prefixes are written from the registers.
//
// 256 lanes, not 1024: a workgroup of sixteen wavefronts needs four free
// slots on every SIMD of one compute unit at the same moment, and while a
// persistent kernel of another stream (the NiN kernels) holds the chip it can
// wait for that until that kernel ends; four wavefronts find room at once.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SCAN1_THREADS 256
#define SCAN1_WAVES (SCAN1_THREADS / 64)
#define SCAN1_PER_LANE 32
#define SCAN1_CHUNK (SCAN1_THREADS * SCAN1_PER_LANE)
#define SCAN1_MAX_ELEMS 65536
#define SCAN1_LDS_WORDS (2 * SCAN1_WAVES)

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

// out[i] = sum of in[0..i), out[n] = total.  Must be called by all 256 lanes of
// a workgroup; lds needs SCAN1_LDS_WORDS words; in and out 16-byte aligned.
// Returns the total to every lane.
template <bool POPC>
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
  constexpr int G = SCAN1_PER_LANE / 4;
  uint4 v[G], nxt[G];
#pragma unroll
  for (int j = 0; j < G; ++j)
    v[j] = scan1_load4<POPC>(in, (size_t)t * SCAN1_PER_LANE + 4 * j, n);
  uint32_t carry = 0;
  int flip = 0;
  for (size_t base = 0; base < n; base += SCAN1_CHUNK) {
    const size_t start = base + (size_t)t * SCAN1_PER_LANE;
    // the next chunk (past the end these read group 0 and count as zero)
#pragma unroll
    for (int j = 0; j < G; ++j)
      nxt[j] = scan1_load4<POPC>(in, start + SCAN1_CHUNK + 4 * j, n);
    uint32_t s = 0;
#pragma unroll
    for (int j = 0; j < G; ++j)
      s += v[j].x + v[j].y + v[j].z + v[j].w;
    // inclusive scan of s across the wavefront, then across the wavefronts
    uint32_t incl = s;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      uint32_t up = __shfl_up(incl, off, 64);
      if (lane >= off)
        incl += up;
    }
    uint32_t *ws = lds + flip * SCAN1_WAVES; // two sets: one barrier per chunk
    if (lane == 63)
      ws[wave] = incl;
    __syncthreads();
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < SCAN1_WAVES; ++w) {
      const uint32_t x = ws[w];
      before += w < wave ? x : 0u;
      total += x;
    }
    uint32_t run = carry + before + (incl - s);
#pragma unroll
    for (int j = 0; j < G; ++j) {
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
    carry += total;
    flip ^= 1;
#pragma unroll
    for (int j = 0; j < G; ++j)
      v[j] = nxt[j];
  }
  if (t == 0)
    out[n] = carry;
  __syncthreads();
  return carry;
}
