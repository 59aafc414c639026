// Exclusive prefix sums over uint32 counts (or popcounts of 64-bit words).
// Short arrays: one workgroup (scn_scan_dev.h).  Long ones: one pass with a
// decoupled look-back -- every workgroup takes the next tile, sums it, publishes
// the sum, adds up what the tiles before it have published (walking back until
// it meets one that already knows its whole prefix) and writes its prefixes; the
// input is read once and nothing is launched in between.
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

// A tile's word of state: bits 63..62 say what the low 32 bits are -- nothing
// yet (0), the tile's own sum (1), the sum of everything up to and including
// the tile (2).  One 64-bit word, so flag and value arrive together.
#define LB_SUM (1ull << 62)
#define LB_PREFIX (2ull << 62)

__global__ void k_scan_clear(unsigned long long *state, size_t words) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < words)
    state[i] = 0ull;
}

// state[0 .. nb): the tiles' words; state[nb]: the ticket counter (tiles are
// handed out in the order the workgroups arrive, so a workgroup only ever waits
// for workgroups that are already running).  All zero at launch.
template <bool POPC>
__global__ void __launch_bounds__(SCAN_THREADS)
    k_scan_lookback(const void *in, uint32_t *out, size_t n, unsigned long long *state,
                    unsigned nb) {
  __shared__ uint32_t lds[SCAN_THREADS];
  __shared__ unsigned sTile;
  __shared__ uint32_t sBefore;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0)
    sTile = atomicAdd(reinterpret_cast<unsigned *>(state + nb), 1u);
  __syncthreads();
  const unsigned tile = sTile;
  const size_t base = (size_t)tile * SCAN_TILE + (size_t)threadIdx.x * SCAN_PER_THREAD;
  const bool whole = ((size_t)tile + 1) * SCAN_TILE <= n && ((uintptr_t)in & 15) == 0 &&
                     ((uintptr_t)out & 15) == 0;
  uint32_t v[SCAN_PER_THREAD];
  scan_load_tile<POPC>(in, base, n, whole, v);
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_PER_THREAD; ++k)
    s += v[k];
  uint32_t total;
  const uint32_t excl = block_exclusive_scan(s, lds, &total);
  if (wave == 0) {
    if (lane == 0)
      __hip_atomic_store(&state[tile], (tile == 0 ? LB_PREFIX : LB_SUM) | total, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    uint32_t before = 0;
    if (tile > 0) {
      // lane i looks at tile - 1 - i, then 64 further back, ...; tiles before
      // the first count as knowing their prefix: 0
      long long j = (long long)tile - 1 - lane;
      for (;;) {
        unsigned long long w;
        for (;;) {
          w = j >= 0 ? __hip_atomic_load(&state[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : LB_PREFIX;
          if (!__any((w >> 62) == 0ull))
            break;
          __builtin_amdgcn_s_sleep(1);
        }
        const unsigned long long known = __ballot((w >> 62) >= 2ull);
        const int first = known ? __ffsll((long long)known) - 1 : 64;
        uint32_t c = lane <= first ? (uint32_t)w : 0u;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
          c += __shfl_xor(c, off, 64);
        before += c;
        if (known)
          break;
        j -= 64;
      }
      if (lane == 0)
        __hip_atomic_store(&state[tile], LB_PREFIX | (unsigned long long)(uint32_t)(before + total),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (lane == 0)
      sBefore = before;
  }
  __syncthreads();
  const uint32_t off = sBefore;
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
  if (tile == nb - 1 && threadIdx.x == 0)
    out[n] = off + total;
}

template <bool POPC>
__global__ void __launch_bounds__(SCAN1_THREADS)
    k_scan_single(const void *in, uint32_t *out, size_t n) {
  __shared__ uint32_t lds[SCAN1_LDS_WORDS];
  (void)block_scan_loop<POPC>(in, out, n, lds);
}

size_t scn_scan_tmp_elems(size_t n) {
  const size_t nb = (n + SCAN_TILE - 1) / SCAN_TILE;
  return 2 * (nb + 1) + 8; // a 64-bit word a tile, one for the tickets, room to align them
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
  const size_t nb = (n + SCAN_TILE - 1) / SCAN_TILE;
  SCN_REQUIRE(nb < 0x7FFFFFFFull, SCN_ERR_CAPACITY, "scan: %zu elements", n);
  unsigned long long *state =
      reinterpret_cast<unsigned long long *>(((uintptr_t)tmp + 7) & ~(uintptr_t)7);
  hipLaunchKernelGGL(k_scan_clear, dim3((unsigned)((nb + 1 + 255) / 256)), dim3(256), 0, s,
                     state, nb + 1);
  SCN_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(k_scan_lookback<POPC>, dim3((unsigned)nb), dim3(SCAN_THREADS), 0, s, in,
                     out, n, state, (unsigned)nb);
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
