// Exclusive prefix sums over uint32 counts (or popcounts of 64-bit words).
// Short arrays: one workgroup (scn_scan_dev.h).  Long ones: one pass -- every
// workgroup takes the next tile, sums it, publishes the sum, adds up what all
// the tiles before it have published and writes its prefixes; the input is
// read once and nothing is launched in between.
#include "scn_common.h"
#include "scn_scan_dev.h"

#define SCAN_THREADS 256

// A tile's word of state: bit 62 says that the low 32 bits hold the tile's sum.
// One 64-bit word, so flag and value arrive together.
#define LB_SUM (1ull << 62)

// the block's sum, to every thread (two barriers)
__device__ __forceinline__ uint32_t block_sum(uint32_t v, uint32_t *lds) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
    v += __shfl_xor(v, off, 64);
  if (lane == 0)
    lds[wave] = v;
  __syncthreads();
  const uint32_t s = lds[0] + lds[1] + lds[2] + lds[3];
  __syncthreads();
  return s;
}

__global__ void k_scan_clear(unsigned long long *state, size_t words) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < words)
    state[i] = 0ull;
}

// state[0 .. nb): the tiles' words; state[nb]: the ticket counter (tiles are
// handed out in the order the workgroups arrive, so a workgroup only ever waits
// for workgroups that are already running).  All zero at launch.  A tile is
// 8192 elements, kept in registers between the sum and the prefixes.  A
// workgroup publishes its tile's sum and then adds up the
// sums of ALL tiles before it, 256 of them at a time, a lane waiting for the
// one it reads: no tile waits for another's prefix, so nothing propagates from
// tile to tile, and a scan of a thousand tiles that are all resident at once
// looks back four times.
#define LB_ROWS 8
#define LB_TILE (SCAN_THREADS * 4 * LB_ROWS)

// inclusive sums across the wavefront through the cross-lane data path: shifts
// within a row of 16 lanes, then lane 15 of rows 0 and 2 into the rows after
// them, then lane 31 into rows 2 and 3 (a lane a step does not reach adds 0)
__device__ __forceinline__ uint32_t wave_incl_dpp(uint32_t v) {
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);
  return v;
}

// A wavefront owns 2048 consecutive elements of the tile as LB_ROWS rows of 64
// lanes x 4 elements: every load and every store of a wavefront is one
// contiguous kilobyte (two for 64-bit words).
template <bool POPC>
__global__ void __launch_bounds__(SCAN_THREADS)
    k_scan_lookback(const void *in, uint32_t *out, size_t n, unsigned long long *state,
                    unsigned nb) {
  __shared__ uint32_t lds[SCAN_THREADS];
  __shared__ unsigned sTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0)
    sTile = atomicAdd(reinterpret_cast<unsigned *>(state + nb), 1u);
  __syncthreads();
  const unsigned tile = sTile;
  const size_t start = (size_t)tile * LB_TILE + (size_t)wave * (256 * LB_ROWS) + (size_t)lane * 4;
  uint4 v[LB_ROWS];
#pragma unroll
  for (int k = 0; k < LB_ROWS; ++k)
    v[k] = scan1_load4<POPC>(in, start + 256 * k, n);
  // before[k]: what lies before this lane's four elements of row k within the wavefront's part
  uint32_t before[LB_ROWS];
  uint32_t mineW = 0; // running total of the rows
#pragma unroll
  for (int k = 0; k < LB_ROWS; ++k) {
    const uint32_t s = v[k].x + v[k].y + v[k].z + v[k].w;
    const uint32_t incl = wave_incl_dpp(s);
    before[k] = mineW + incl - s;
    mineW += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
  }
  // across the four wavefronts
  if (lane == 0)
    lds[wave] = mineW;
  __syncthreads();
  const uint32_t w0 = lds[0], w1 = lds[1], w2 = lds[2], w3 = lds[3];
  __syncthreads();
  const uint32_t total = w0 + w1 + w2 + w3;
  const uint32_t waveBefore = (wave > 0 ? w0 : 0u) + (wave > 1 ? w1 : 0u) + (wave > 2 ? w2 : 0u);
  if (threadIdx.x == 0)
    __hip_atomic_store(&state[tile], LB_SUM | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  uint32_t mine = 0;
  for (long long j = threadIdx.x; j < (long long)tile; j += SCAN_THREADS) {
    unsigned long long w;
    for (;;) {
      w = __hip_atomic_load(&state[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (w & LB_SUM)
        break;
      __builtin_amdgcn_s_sleep(1);
    }
    mine += (uint32_t)w;
  }
  const uint32_t off = block_sum(mine, lds);
#pragma unroll
  for (int k = 0; k < LB_ROWS; ++k) {
    uint4 o;
    o.x = off + waveBefore + before[k];
    o.y = o.x + v[k].x;
    o.z = o.y + v[k].y;
    o.w = o.z + v[k].z;
    const size_t i = start + 256 * k;
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
  const size_t nb = (n + LB_TILE - 1) / LB_TILE;
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
  const size_t nb = (n + LB_TILE - 1) / LB_TILE;
  SCN_REQUIRE(nb < 0x7FFFFFFFull, SCN_ERR_CAPACITY, "scan: %zu elements", n);
  SCN_REQUIRE(((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0, SCN_ERR_ARG,
              "scan: buffers must be 16-byte aligned");
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
