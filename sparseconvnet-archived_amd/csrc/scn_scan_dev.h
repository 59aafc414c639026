// Device-side exclusive prefix sum by ONE workgroup of 1024 lanes.  For arrays
// up to about a hundred thousand elements this is one launch instead of the
// three of the tiled scan, and launch count is what small batches pay for.
//
// Every lane owns one contiguous chunk: it sums the chunk (all loads in flight
// at once, no barrier in between), the 1024 chunk sums are scanned through
// wavefront shuffles and 17 words of LDS, and the lane walks its chunk a
// second time (served by the caches) to write the prefixes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SCAN1_THREADS 1024
#define SCAN1_MAX_ELEMS (SCAN1_THREADS * 32) // above this one compute unit's bandwidth loses to the three-launch tiled scan

template <bool POPC>
__device__ __forceinline__ uint32_t scan1_load(const void *in, size_t i) {
  if (POPC)
    return (uint32_t)__popcll(((const unsigned long long *)in)[i]);
  return ((const uint32_t *)in)[i];
}

// four consecutive elements starting at i (i % 4 == 0); elements at or past n
// read as zero
template <bool POPC>
__device__ __forceinline__ uint4 scan1_load4(const void *in, size_t i,
                                             size_t n) {
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (i + 4 <= n) {
    if (POPC) {
      const ulonglong2 *p =
          reinterpret_cast<const ulonglong2 *>((const unsigned long long *)in + i);
      ulonglong2 a = p[0], b = p[1];
      v = make_uint4(__popcll(a.x), __popcll(a.y), __popcll(b.x), __popcll(b.y));
    } else {
      v = *reinterpret_cast<const uint4 *>((const uint32_t *)in + i);
    }
  } else {
    if (i < n)
      v.x = scan1_load<POPC>(in, i);
    if (i + 1 < n)
      v.y = scan1_load<POPC>(in, i + 1);
    if (i + 2 < n)
      v.z = scan1_load<POPC>(in, i + 2);
  }
  return v;
}

// out[i] = sum of in[0..i), out[n] = total.  Must be called by all 1024 lanes
// of a workgroup; lds needs 17 words; in and out 16-byte aligned.  Returns the
// total to every lane.
template <bool POPC>
__device__ __forceinline__ uint32_t block_scan_loop(const void *in,
                                                    uint32_t *out, size_t n,
                                                    uint32_t *lds) {
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  size_t chunk = (n + SCAN1_THREADS - 1) / SCAN1_THREADS;
  chunk = (chunk + 3) & ~(size_t)3;
  const size_t start = (size_t)t * chunk;
  uint32_t s = 0;
  for (size_t k = 0; k < chunk && start + k < n; k += 4) {
    uint4 v = scan1_load4<POPC>(in, start + k, n);
    s += v.x + v.y + v.z + v.w;
  }
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
  for (size_t k = 0; k < chunk && start + k < n; k += 4) {
    uint4 v = scan1_load4<POPC>(in, start + k, n);
    uint4 o;
    o.x = run;
    o.y = o.x + v.x;
    o.z = o.y + v.y;
    o.w = o.z + v.z;
    run = o.w + v.w;
    size_t i = start + k;
    if (i + 4 <= n) {
      *reinterpret_cast<uint4 *>(out + i) = o;
    } else {
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
