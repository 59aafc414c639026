// Exclusive prefix sums over uint32 counts (or popcounts of 64-bit words),
// three-phase: per-tile totals, recursive scan of the totals, per-tile rescan.
#include "scn_common.h"
#include "scn_scan_dev.h"

#define SCAN_THREADS 256
#define SCAN_PER_THREAD 8
#define SCAN_TILE (SCAN_THREADS * SCAN_PER_THREAD)

template <bool POPC>
__device__ __forceinline__ uint32_t scan_load(const void *in, size_t i) {
  if (POPC)
    return (uint32_t)__popcll(((const uint64_t *)in)[i]);
  return ((const uint32_t *)in)[i];
}

// a thread's SCAN_PER_THREAD consecutive values; a tile that lies wholly inside
// the input is read with 16-byte loads
template <bool POPC>
__device__ __forceinline__ void scan_load_tile(const void *in, size_t base, size_t n,
                                               bool whole, uint32_t *v) {
  static_assert(SCAN_PER_THREAD == 8, "eight values a thread");
  if (whole) {
    if (POPC) {
      const ulonglong2 *p = reinterpret_cast<const ulonglong2 *>((const uint64_t *)in + base);
      ulonglong2 w[4];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        w[k] = p[k];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[2 * k] = (uint32_t)__popcll(w[k].x);
        v[2 * k + 1] = (uint32_t)__popcll(w[k].y);
      }
    } else {
      const uint4 *p = reinterpret_cast<const uint4 *>((const uint32_t *)in + base);
      const uint4 a = p[0], b = p[1];
      v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w;
      v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
    }
  } else {
#pragma unroll
    for (int k = 0; k < SCAN_PER_THREAD; ++k)
      v[k] = (base + k < n) ? scan_load<POPC>(in, base + k) : 0u;
  }
}

// exclusive scan of one value per thread across the block; *total = block sum.
// Within a wavefront by lane shuffles, across the four wavefronts through LDS:
// two barriers.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v,
                                                         uint32_t *lds,
                                                         uint32_t *total) {
  static_assert(SCAN_THREADS == 256, "four wavefronts");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t below = __shfl_up(incl, off, 64);
    if (lane >= off)
      incl += below;
  }
  if (lane == 63)
    lds[wave] = incl;
  __syncthreads();
  const uint32_t s0 = lds[0], s1 = lds[1], s2 = lds[2], s3 = lds[3];
  __syncthreads(); // lds may be written again by the caller's next scan
  const uint32_t before = (wave > 0 ? s0 : 0u) + (wave > 1 ? s1 : 0u) + (wave > 2 ? s2 : 0u);
  *total = s0 + s1 + s2 + s3;
  return before + incl - v;
}

// the block's sum in thread 0 (every thread gets it)
__device__ __forceinline__ uint32_t block_sum(uint32_t v, uint32_t *lds) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
    v += __shfl_xor(v, off, 64);
  if (lane == 0)
    lds[wave] = v;
  __syncthreads();
  return lds[0] + lds[1] + lds[2] + lds[3];
}

template <bool POPC>
__global__ void __launch_bounds__(SCAN_THREADS)
    k_scan_reduce(const void *in, size_t n, uint32_t *tileSums) {
  __shared__ uint32_t lds[SCAN_THREADS];
  size_t base = (size_t)blockIdx.x * SCAN_TILE + (size_t)threadIdx.x * SCAN_PER_THREAD;
  const bool whole = ((size_t)blockIdx.x + 1) * SCAN_TILE <= n && ((uintptr_t)in & 15) == 0;
  uint32_t v[SCAN_PER_THREAD];
  scan_load_tile<POPC>(in, base, n, whole, v);
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_PER_THREAD; ++k)
    s += v[k];
  const uint32_t total = block_sum(s, lds);
  if (threadIdx.x == 0)
    tileSums[blockIdx.x] = total;
}

// out[i] = tileOffsets[tile] + exclusive prefix inside the tile; the block that
// owns element n - 1 also writes out[n] = grand total.
template <bool POPC>
__global__ void __launch_bounds__(SCAN_THREADS)
    k_scan_final(const void *in, uint32_t *out, size_t n,
                 const uint32_t *tileOffsets) {
  __shared__ uint32_t lds[SCAN_THREADS];
  size_t base = (size_t)blockIdx.x * SCAN_TILE + (size_t)threadIdx.x * SCAN_PER_THREAD;
  const bool whole = ((size_t)blockIdx.x + 1) * SCAN_TILE <= n && ((uintptr_t)in & 15) == 0 &&
                     ((uintptr_t)out & 15) == 0;
  uint32_t v[SCAN_PER_THREAD];
  scan_load_tile<POPC>(in, base, n, whole, v);
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_PER_THREAD; ++k)
    s += v[k];
  uint32_t total;
  uint32_t excl = block_exclusive_scan(s, lds, &total);
  uint32_t off = tileOffsets ? tileOffsets[blockIdx.x] : 0u;
  uint32_t run = off + excl;
  if (whole) {
    uint32_t r[SCAN_PER_THREAD];
#pragma unroll
    for (int k = 0; k < SCAN_PER_THREAD; ++k) {
      r[k] = run;
      run += v[k];
    }
    uint4 *o = reinterpret_cast<uint4 *>(out + base);
    o[0] = make_uint4(r[0], r[1], r[2], r[3]);
    o[1] = make_uint4(r[4], r[5], r[6], r[7]);
  } else {
#pragma unroll
    for (int k = 0; k < SCAN_PER_THREAD; ++k) {
      if (base + k < n)
        out[base + k] = run;
      run += v[k];
    }
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0)
    out[n] = off + total;
}

template <bool POPC>
__global__ void __launch_bounds__(SCAN1_THREADS)
    k_scan_single(const void *in, uint32_t *out, size_t n) {
  __shared__ uint32_t lds[SCAN1_LDS_WORDS];
  (void)block_scan_loop<POPC>(in, out, n, lds);
}

size_t scn_scan_tmp_elems(size_t n) {
  size_t total = 0;
  while (n > SCAN_TILE) {
    size_t nb = (n + SCAN_TILE - 1) / SCAN_TILE;
    total += 2 * nb + 8; // tile sums + their exclusive scan (nb + 1)
    n = nb;
  }
  return total + 8;
}

template <bool POPC>
static int scan_impl(hipStream_t s, const void *in, uint32_t *out, size_t n,
                     uint32_t *tmp) {
  if (n <= SCAN1_MAX_ELEMS) { // one launch; n == 0 still writes out[0] = 0
    hipLaunchKernelGGL(k_scan_single<POPC>, dim3(1), dim3(SCAN1_THREADS), 0, s,
                       in, out, n);
    SCN_HIP_CHECK(hipGetLastError());
    return SCN_OK;
  }
  size_t nb = (n + SCAN_TILE - 1) / SCAN_TILE;
  if (nb <= 1) {
    hipLaunchKernelGGL(k_scan_final<POPC>, dim3(1), dim3(SCAN_THREADS), 0, s, in,
                       out, n, (const uint32_t *)nullptr);
    SCN_HIP_CHECK(hipGetLastError());
    return SCN_OK;
  }
  uint32_t *sums = tmp;
  uint32_t *offs = tmp + nb + 4;
  hipLaunchKernelGGL(k_scan_reduce<POPC>, dim3((unsigned)nb), dim3(SCAN_THREADS),
                     0, s, in, n, sums);
  SCN_HIP_CHECK(hipGetLastError());
  SCN_TRY(scan_impl<false>(s, sums, offs, nb, tmp + 2 * nb + 8));
  hipLaunchKernelGGL(k_scan_final<POPC>, dim3((unsigned)nb), dim3(SCAN_THREADS),
                     0, s, in, out, n, (const uint32_t *)offs);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

int scn_scan_exclusive_u32(hipStream_t s, const uint32_t *in, uint32_t *out,
                           size_t n, uint32_t *tmp) {
  return scan_impl<false>(s, in, out, n, tmp);
}

int scn_scan_exclusive_popc64(hipStream_t s, const uint64_t *words,
                              uint32_t *out, size_t n, uint32_t *tmp) {
  return scan_impl<true>(s, words, out, n, tmp);
}
