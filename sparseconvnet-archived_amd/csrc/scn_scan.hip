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

// exclusive scan of one value per thread across the block; *total = block sum
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v,
                                                         uint32_t *lds,
                                                         uint32_t *total) {
  const int t = threadIdx.x;
  lds[t] = v;
  __syncthreads();
  for (int off = 1; off < SCAN_THREADS; off <<= 1) {
    uint32_t add = (t >= off) ? lds[t - off] : 0u;
    __syncthreads();
    lds[t] += add;
    __syncthreads();
  }
  uint32_t incl = lds[t];
  *total = lds[SCAN_THREADS - 1];
  __syncthreads();
  return incl - v;
}

template <bool POPC>
__global__ void __launch_bounds__(SCAN_THREADS)
    k_scan_reduce(const void *in, size_t n, uint32_t *tileSums) {
  __shared__ uint32_t lds[SCAN_THREADS];
  size_t base = (size_t)blockIdx.x * SCAN_TILE + (size_t)threadIdx.x * SCAN_PER_THREAD;
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_PER_THREAD; ++k)
    if (base + k < n)
      s += scan_load<POPC>(in, base + k);
  uint32_t total;
  (void)block_exclusive_scan(s, lds, &total);
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
  uint32_t v[SCAN_PER_THREAD];
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_PER_THREAD; ++k) {
    v[k] = (base + k < n) ? scan_load<POPC>(in, base + k) : 0u;
    s += v[k];
  }
  uint32_t total;
  uint32_t excl = block_exclusive_scan(s, lds, &total);
  uint32_t off = tileOffsets ? tileOffsets[blockIdx.x] : 0u;
  uint32_t run = off + excl;
#pragma unroll
  for (int k = 0; k < SCAN_PER_THREAD; ++k) {
    if (base + k < n)
      out[base + k] = run;
    run += v[k];
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
