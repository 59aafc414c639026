// The backward pass and the weight update behind the C ABI: what the layers'
// backwards() call in the reference, one entry point per free function there.
//   softmax + NLL gradient     SoftmaxClassifier.cu:7-14
//   activation derivatives     SigmoidLayer.cu:23-177, NetworkInNetworkPReLULayer.cu:25-47
//   bias gradient              columnSum, NetworkInNetworkLayer.cu:84-105
//   weight gradient  A^T D     d_rowMajorSGEMM_alphaAtB_betaC, utilities.cu:144-155
//   input gradient   D W^T     d_rowMajorSGEMM_alphaABt_betaC, utilities.cu:157-168
//   weight update              dGradientDescent(KeepPositive), NetworkInNetworkLayer.cu:27-41
//   convolution                dPropBackwardFromMatrixMultiplyOutput, ConvolutionalLayer.cu:42-63
//   max-pooling                dMaxPoolBackProp, MaxPoolingLayer.cu:74-82
//   terminal pooling           dTerminalPoolBackProp, TerminalPoolingLayer.cu:48-62
#include <mutex>
#include "scn_common.h"
#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

typedef float floatx4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- softmax
__global__ void k_softmax_grad(const float *__restrict__ probs,
                               const int *__restrict__ labels,
                               float *__restrict__ delta, long long total,
                               int N) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total)
    return;
  long long k = i / N;
  int c = (int)(i - k * N);
  delta[i] = probs[i] - (c == labels[k] ? 1.f : 0.f);
}

extern "C" int scn_softmax_grad(scn_ctx *ctx, const float *d_probs,
                                const int32_t *d_labels, float *d_delta,
                                int64_t batch, int N) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_softmax_grad: null context");
  SCN_REQUIRE(batch >= 0 && N >= 1, SCN_ERR_ARG,
              "scn_softmax_grad: batch %lld N %d", (long long)batch, N);
  if (batch == 0)
    return SCN_OK;
  SCN_REQUIRE(d_probs && d_labels && d_delta, SCN_ERR_ARG,
              "scn_softmax_grad: null buffer");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  long long total = batch * N;
  hipLaunchKernelGGL(k_softmax_grad, dim3(scn_ceil_div(total, 256)), dim3(256),
                     0, ctx->stream, d_probs, d_labels, d_delta, total, N);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// ------------------------------------------------- activation derivatives
// One pass over the [M x N] gradient: multiplies it in place by the
// derivative of the activation (expressed through the layer's output, as the
// reference does), and leaves the column sums of the result in db (the bias
// gradient) and, for PReLU, the slope gradient in dprelu.  A workgroup covers
// P columns (the power of two that covers min(N, 64)) with 256 / P lanes per
// column, which interleave rows and take four of them per trip so that eight
// loads are in flight per lane.
__device__ __forceinline__ float act_derivative(int act, float b, float d,
                                                float alpha, float &t) {
  switch (act) {
  case SCN_RELU:
    return b > 0 ? d : 0.f;
  case SCN_LEAKYRELU:
  case SCN_VLEAKYRELU:
    return b > 0 ? d : d * alpha;
  case SCN_TANH:
    return d * (1 + b) * (1 - b);
  case SCN_SIGMOID:
    return d * b * (1 - b);
  case SCN_PRELU:
    t += d * (b > 0 ? 0.f : b / alpha);
    return b > 0 ? d : d * alpha;
  default: // SOFTMAX (folded into the classifier's gradient), NOSIGMOID
    return d;
  }
}
__global__ __launch_bounds__(256) void k_act_backward(
    const float *__restrict__ out, float *__restrict__ delta, long long M,
    int N, int act, const float *__restrict__ prelu, float *__restrict__ db,
    float *__restrict__ dprelu, int P) {
  __shared__ float sS[256], sT[256];
  const int tx = threadIdx.x % P, ty = threadIdx.x / P, lanesPerCol = 256 / P;
  const int c = blockIdx.x * P + tx;
  float s = 0.f, t = 0.f;
  if (c < N) {
    const float alpha = act == SCN_PRELU      ? prelu[c]
                        : act == SCN_LEAKYRELU ? 0.01f
                                               : 0.333f;
    const long long step = (long long)lanesPerCol * gridDim.y;
    long long r = (long long)blockIdx.y * lanesPerCol + ty;
    for (; r + 3 * step < M; r += 4 * step) {
      float b[4], d[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        b[u] = out[(r + u * step) * N + c];
        d[u] = delta[(r + u * step) * N + c];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        d[u] = act_derivative(act, b[u], d[u], alpha, t);
        delta[(r + u * step) * N + c] = d[u];
        s += d[u];
      }
    }
    for (; r < M; r += step) {
      const float d = act_derivative(act, out[r * N + c], delta[r * N + c], alpha, t);
      delta[r * N + c] = d;
      s += d;
    }
  }
  sS[threadIdx.x] = s;
  sT[threadIdx.x] = t;
  __syncthreads();
  if (ty == 0 && c < N) {
    s = 0.f, t = 0.f;
    for (int k = 0; k < lanesPerCol; ++k) {
      s += sS[k * P + tx];
      t += sT[k * P + tx];
    }
    unsafeAtomicAdd(db + c, s);
    if (act == SCN_PRELU)
      unsafeAtomicAdd(dprelu + c, t);
  }
}

static int activation_backward(scn_ctx *ctx, const float *d_out,
                               float *d_delta, int64_t M, int N, int act,
                               const float *d_prelu, float *d_db,
                               float *d_dprelu, bool clear) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_activation_backward: null context");
  SCN_REQUIRE(M >= 0 && N >= 1, SCN_ERR_ARG,
              "scn_activation_backward: M %lld N %d", (long long)M, N);
  SCN_REQUIRE(act >= SCN_NOSIGMOID && act <= SCN_SIGMOID, SCN_ERR_ARG,
              "scn_activation_backward: activation %d", act);
  SCN_REQUIRE(d_db, SCN_ERR_ARG, "scn_activation_backward: null d_db");
  SCN_REQUIRE(act != SCN_PRELU || (d_prelu && d_dprelu), SCN_ERR_ARG,
              "scn_activation_backward: PReLU needs slopes and their gradient");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  if (clear) {
    SCN_TRY(scn_fill32(ctx, d_db, 0, (size_t)N));
    if (act == SCN_PRELU)
      SCN_TRY(scn_fill32(ctx, d_dprelu, 0, (size_t)N));
  }
  if (M == 0)
    return SCN_OK;
  SCN_REQUIRE(d_out && d_delta, SCN_ERR_ARG,
              "scn_activation_backward: null buffer");
  int P = 1;
  while (P < N && P < 64)
    P <<= 1;
  const int lanesPerCol = 256 / P;
  int colBlocks = scn_ceil_div(N, P);
  // every workgroup ends with one atomic per column onto the same N
  // addresses, and those serialise (about 25 ns each): few, long-lived
  // workgroups, two per compute unit
  int rowBlocks = scn_ceil_div(M, 8 * lanesPerCol); // at least eight rows per lane
  int cap = (ctx->numCU * 2 + colBlocks - 1) / colBlocks;
  if (rowBlocks > cap)
    rowBlocks = cap;
  if (rowBlocks < 1)
    rowBlocks = 1;
  hipLaunchKernelGGL(k_act_backward, dim3(colBlocks, rowBlocks), dim3(256), 0,
                     ctx->stream, d_out, d_delta, (long long)M, N, act,
                     d_prelu, d_db, d_dprelu, P);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

extern "C" int scn_activation_backward(scn_ctx *ctx, const float *d_out,
                                       float *d_delta, int64_t M, int N,
                                       int act, const float *d_prelu,
                                       float *d_db, float *d_dprelu) {
  return activation_backward(ctx, d_out, d_delta, M, N, act, d_prelu, d_db,
                             d_dprelu, true);
}

extern "C" int scn_activation_backward_acc(scn_ctx *ctx, const float *d_out,
                                           float *d_delta, int64_t M, int N,
                                           int act, const float *d_prelu,
                                           float *d_db, float *d_dprelu) {
  return activation_backward(ctx, d_out, d_delta, M, N, act, d_prelu, d_db,
                             d_dprelu, false);
}

// ------------------------------------------------------- dW = A^T D (MFMA)
// Output tile 64 (rows of dW = columns of A) x 64 (columns of D) per
// workgroup, reduction over a range of the M rows; the row ranges of one tile
// add their partial tiles into dW with float atomics.  A chunk of 32 rows of
// both operands is staged in LDS (row pitch 80 words: the four row groups
// that one v_mfma_f32_16x16x4_f32 operand read touches fall on disjoint
// banks); wavefront w owns columns 16 w .. 16 w + 15 of the tile and all 64 of
// its rows (four accumulator tiles).
#define ATB_ROWS 32
#define ATB_PITCH 80
__global__ __launch_bounds__(256) void k_gemm_atb(
    const float *__restrict__ A, const float *__restrict__ D,
    float *__restrict__ dW, long long M, int K, int N, int nTiles,
    long long rowsPerSplit) {
  __shared__ float sA[ATB_ROWS * ATB_PITCH], sD[ATB_ROWS * ATB_PITCH];
  const int k0 = (blockIdx.x / nTiles) * 64, n0 = (blockIdx.x % nTiles) * 64;
  const long long m0 = (long long)blockIdx.y * rowsPerSplit;
  const long long m1 = m0 + rowsPerSplit < M ? m0 + rowsPerSplit : M;
  const int t = threadIdx.x, col = t & 63, rg = t >> 6;
  const int lane = t & 63, w = t >> 6, c = lane & 15, q = lane >> 4;
  const bool aIn = k0 + col < K, dIn = n0 + col < N;
  floatx4 acc[4];
  for (int i = 0; i < 4; ++i)
    acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the next chunk's loads are in flight under this chunk's MFMAs
  float ra[ATB_ROWS / 4], rd[ATB_ROWS / 4];
  auto fetch = [&](long long m) {
#pragma unroll
    for (int i = 0; i < ATB_ROWS / 4; ++i) {
      const long long row = m + rg + 4 * i;
      const bool live = row < m1;
      ra[i] = live && aIn ? A[row * K + k0 + col] : 0.f;
      rd[i] = live && dIn ? D[row * N + n0 + col] : 0.f;
    }
  };
  fetch(m0);
  for (long long m = m0; m < m1; m += ATB_ROWS) {
#pragma unroll
    for (int i = 0; i < ATB_ROWS / 4; ++i) {
      const int r = rg + 4 * i;
      sA[r * ATB_PITCH + col] = ra[i];
      sD[r * ATB_PITCH + col] = rd[i];
    }
    __syncthreads();
    if (m + ATB_ROWS < m1)
      fetch(m + ATB_ROWS);
#pragma unroll
    for (int s = 0; s < ATB_ROWS / 4; ++s) {
      const float *pa = sA + (4 * s + q) * ATB_PITCH + c;
      const float b = sD[(4 * s + q) * ATB_PITCH + 16 * w + c];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[16 * i], b, acc[i], 0,
                                                      0, 0);
    }
    __syncthreads();
  }
  const int n = n0 + 16 * w + c;
  if (n < N)
    for (int i = 0; i < 4; ++i)
      for (int v = 0; v < 4; ++v) {
        const int k = k0 + 16 * i + 4 * q + v;
        if (k < K)
          unsafeAtomicAdd(dW + (long long)k * N + n, acc[i][v]);
      }
}

// The same product for shapes that fill wider tiles (K and N multiples of 4,
// 16-byte aligned operands).  WK x WN wavefronts per workgroup, 64 x 64 of
// the output each: 16 accumulator tiles per wavefront fed by ONE 128-bit LDS
// read per operand and k-step (lane (c, q) reads columns 4c..4c+3 of row
// 4s + q, so MFMA tile i covers the output rows 4 * (its A-operand index) + i
// and tile j the output columns 4c + j: 0.125 LDS reads per MFMA instead of
// 1.25).  Chunks of 16 rows, double-buffered: the global loads of the next
// chunk are in flight under the MFMAs of this one, one barrier per chunk.
#define ATBW_ROWS 16
template <int WK, int WN>
__global__ __launch_bounds__(64 * WK * WN) void k_gemm_atb_wide(
    const float *__restrict__ A, const float *__restrict__ D,
    float *__restrict__ dW, long long M, int K, int N, int nTiles,
    long long rowsPerSplit) {
  constexpr int TK = 64 * WK, TN = 64 * WN, PA = TK + 16, PD = TN + 16;
  constexpr int NT = 64 * WK * WN;
  constexpr int LA = ATBW_ROWS * TK / 4 / NT; // float4 loads per lane, A
  constexpr int LD = ATBW_ROWS * TN / 4 / NT; // ... and D
  static_assert(LA * NT * 4 == ATBW_ROWS * TK && LD * NT * 4 == ATBW_ROWS * TN &&
                    LD >= 1,
                "chunk loads divide evenly");
  __shared__ __align__(16) float sA[2][ATBW_ROWS * PA];
  __shared__ __align__(16) float sD[2][ATBW_ROWS * PD];
  const int k0 = (blockIdx.x / nTiles) * TK, n0 = (blockIdx.x % nTiles) * TN;
  const long long m0 = (long long)blockIdx.y * rowsPerSplit;
  const long long m1 = m0 + rowsPerSplit < M ? m0 + rowsPerSplit : M;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wk = wave / WN, wn = wave % WN, c = lane & 15, q = lane >> 4;
  floatx4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
  float4 ra[LA], rd[LD];
  auto fetch = [&](long long m) {
#pragma unroll
    for (int u = 0; u < LA; ++u) {
      const int f = t + u * NT, r = f / (TK / 4), col = (f % (TK / 4)) * 4;
      const long long row = m + r;
      ra[u] = row < m1 && k0 + col < K
                  ? *(const float4 *)(A + row * K + k0 + col)
                  : float4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < LD; ++u) {
      const int f = t + u * NT, r = f / (TN / 4), col = (f % (TN / 4)) * 4;
      const long long row = m + r;
      rd[u] = row < m1 && n0 + col < N
                  ? *(const float4 *)(D + row * N + n0 + col)
                  : float4{0.f, 0.f, 0.f, 0.f};
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int u = 0; u < LA; ++u) {
      const int f = t + u * NT, r = f / (TK / 4), col = (f % (TK / 4)) * 4;
      *(float4 *)(&sA[buf][r * PA + col]) = ra[u];
    }
#pragma unroll
    for (int u = 0; u < LD; ++u) {
      const int f = t + u * NT, r = f / (TN / 4), col = (f % (TN / 4)) * 4;
      *(float4 *)(&sD[buf][r * PD + col]) = rd[u];
    }
  };
  fetch(m0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (long long m = m0; m < m1; m += ATBW_ROWS, buf ^= 1) {
    const bool more = m + ATBW_ROWS < m1;
    if (more)
      fetch(m + ATBW_ROWS);
    const float *pa = &sA[buf][q * PA + wk * 64 + 4 * c];
    const float *pd = &sD[buf][q * PD + wn * 64 + 4 * c];
#pragma unroll
    for (int s4 = 0; s4 < ATBW_ROWS / 4; ++s4) {
      const float4 a = *(const float4 *)(pa + 4 * s4 * PA);
      const float4 d = *(const float4 *)(pd + 4 * s4 * PD);
      const float av[4] = {a.x, a.y, a.z, a.w}, dv[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], dv[j],
                                                           acc[i][j], 0, 0, 0);
    }
    if (more)
      stage(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int k = k0 + wk * 64 + 4 * (4 * q + v) + i;
      if (k >= K)
        continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + wn * 64 + 4 * c + j;
        if (n < N)
          unsafeAtomicAdd(dW + (long long)k * N + n, acc[i][j][v]);
      }
    }
}

template <int WK, int WN>
static int launch_atb_wide(scn_ctx *ctx, const float *d_A, const float *d_D,
                           float *d_dW, int64_t M, int K, int N) {
  constexpr int TK = 64 * WK, TN = 64 * WN;
  const int kTiles = scn_ceil_div(K, TK), nTiles = scn_ceil_div(N, TN);
  const long long tiles = (long long)kTiles * nTiles;
  // Row ranges: more of them shorten every workgroup's walk, but each adds
  // one more tile of float atomics onto the same K x N addresses, and those
  // serialise.  Measured on MI355X: a workgroup walks a row in about 60 ns
  // (it waits for memory more than for the matrix cores; four of them share a
  // compute unit), the part retires about 45 contended atomics per ns.  Take
  // the count that minimises the sum.
  const long long maxSplits = (M + 8 * ATBW_ROWS - 1) / (8 * ATBW_ROWS);
  const double flushNs = (double)K * N / (double)tiles / 45.0;
  long long splits = 1;
  double best = 1e300;
  for (long long cand = 1; cand <= maxSplits && cand <= 4096;
       cand += cand < 16 ? 1 : cand / 8) {
    const long long wgs = tiles * cand;
    const long long rounds = (wgs + 4 * ctx->numCU - 1) / (4 * ctx->numCU);
    const double cost = (double)rounds * ((double)M / cand) * 60.0 +
                        (double)wgs * flushNs;
    if (cost < best) {
      best = cost;
      splits = cand;
    }
  }
  long long rowsPerSplit = (M + splits - 1) / splits;
  rowsPerSplit = (rowsPerSplit + ATBW_ROWS - 1) / ATBW_ROWS * ATBW_ROWS;
  splits = (M + rowsPerSplit - 1) / rowsPerSplit;
  hipLaunchKernelGGL((k_gemm_atb_wide<WK, WN>),
                     dim3((unsigned)tiles, (unsigned)splits),
                     dim3(64 * WK * WN), 0, ctx->stream, d_A, d_D, d_dW,
                     (long long)M, K, N, nTiles, rowsPerSplit);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

static int sgemm_AtB(scn_ctx *ctx, const float *d_A, const float *d_D,
                     float *d_dW, int64_t M, int K, int N, bool clear) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_sgemm_AtB: null context");
  SCN_REQUIRE(M >= 0 && K >= 1 && N >= 1, SCN_ERR_ARG,
              "scn_sgemm_AtB: M %lld K %d N %d", (long long)M, K, N);
  SCN_REQUIRE(d_dW, SCN_ERR_ARG, "scn_sgemm_AtB: null d_dW");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  if (clear)
    SCN_TRY(scn_fill32(ctx, d_dW, 0, (size_t)K * N));
  if (M == 0)
    return SCN_OK;
  SCN_REQUIRE(d_A && d_D, SCN_ERR_ARG, "scn_sgemm_AtB: null buffer");
  // The wide tiles pay on long walks over the rows (measured: 200000 x 1728 x
  // 64 and 100000 x 800 x 800 gain 20 %); up to some ten thousand rows, or with
  // an output of a few tiles only, the narrow kernel's many short walks win.
  if (K % 4 == 0 && N % 4 == 0 && N >= 48 && M >= 65536 &&
      ((long long)K * N >= 160 * 1024 || (K >= 1024 && N >= 64)) &&
      ((uintptr_t)d_A & 15) == 0 && ((uintptr_t)d_D & 15) == 0) {
    // 256 x 64 or 128 x 128 tiles: whichever pads the output less
    const long long pad41 = (long long)scn_ceil_div(K, 256) * 256 *
                            scn_ceil_div(N, 64) * 64;
    const long long pad22 = (long long)scn_ceil_div(K, 128) * 128 *
                            scn_ceil_div(N, 128) * 128;
    return pad41 < pad22 ? launch_atb_wide<4, 1>(ctx, d_A, d_D, d_dW, M, K, N)
                         : launch_atb_wide<2, 2>(ctx, d_A, d_D, d_dW, M, K, N);
  }
  const int kTiles = scn_ceil_div(K, 64), nTiles = scn_ceil_div(N, 64);
  const long long tiles = (long long)kTiles * nTiles;
  SCN_REQUIRE(tiles <= 0x7fffffffll, SCN_ERR_CAPACITY,
              "scn_sgemm_AtB: %lld tiles", tiles);
  long long splits = (ctx->numCU * 4 + tiles - 1) / tiles;
  const long long maxSplits = (M + 8 * ATB_ROWS - 1) / (8 * ATB_ROWS);
  if (splits > maxSplits)
    splits = maxSplits;
  if (splits > 65535)
    splits = 65535;
  if (splits < 1)
    splits = 1;
  long long rowsPerSplit = (M + splits - 1) / splits;
  rowsPerSplit = (rowsPerSplit + ATB_ROWS - 1) / ATB_ROWS * ATB_ROWS;
  splits = (M + rowsPerSplit - 1) / rowsPerSplit;
  hipLaunchKernelGGL(k_gemm_atb, dim3((unsigned)tiles, (unsigned)splits),
                     dim3(256), 0, ctx->stream, d_A, d_D, d_dW, (long long)M, K,
                     N, nTiles, rowsPerSplit);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

extern "C" int scn_sgemm_AtB(scn_ctx *ctx, const float *d_A, const float *d_D,
                             float *d_dW, int64_t M, int K, int N) {
  return sgemm_AtB(ctx, d_A, d_D, d_dW, M, K, N, true);
}

// the kernels only ever add to dW, so beta = 1 is the same launch without the
// clearing one before it
extern "C" int scn_sgemm_AtB_acc(scn_ctx *ctx, const float *d_A,
                                 const float *d_D, float *d_dW, int64_t M,
                                 int K, int N) {
  return sgemm_AtB(ctx, d_A, d_D, d_dW, M, K, N, false);
}

// ------------------------------------------------------------ dA = D W^T
// The forward contraction with W transposed: the transposed copy (and the
// zero bias the forward kernels add) live in the caller's workspace.
__global__ void k_transpose(const float *__restrict__ W, float *__restrict__ Wt,
                            int K, int N) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8
  const int k0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
  for (int i = ty; i < 32; i += 8)
    if (k0 + i < K && n0 + tx < N)
      tile[i][tx] = W[(long long)(k0 + i) * N + n0 + tx];
  __syncthreads();
  for (int i = ty; i < 32; i += 8)
    if (n0 + i < N && k0 + tx < K)
      Wt[(long long)(n0 + i) * K + k0 + tx] = tile[tx][i];
}

extern "C" int64_t scn_sgemm_ABt_workspace(int N, int K) {
  return (int64_t)N * K + K;
}

extern "C" int scn_sgemm_ABt(scn_ctx *ctx, const float *d_D, const float *d_W,
                             float *d_dA, int64_t M, int N, int K,
                             float *d_workspace) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_sgemm_ABt: null context");
  SCN_REQUIRE(M >= 0 && K >= 1 && N >= 1, SCN_ERR_ARG,
              "scn_sgemm_ABt: M %lld N %d K %d", (long long)M, N, K);
  if (M == 0)
    return SCN_OK;
  SCN_REQUIRE(d_D && d_W && d_dA && d_workspace, SCN_ERR_ARG,
              "scn_sgemm_ABt: null buffer");
  // the zero bias: the context's own zeros when they are enough of them
  float *Wt = d_workspace, *zeros = d_workspace + (size_t)N * K;
  {
    ProfScope prof(ctx, SCN_K_BACKWARD);
    hipLaunchKernelGGL(k_transpose, dim3(scn_ceil_div(N, 32), scn_ceil_div(K, 32)),
                       dim3(256), 0, ctx->stream, d_W, Wt, K, N);
    SCN_HIP_CHECK(hipGetLastError());
    if (K <= SCN_ZERO_FLOATS)
      zeros = ctx->d_zeros;
    else
      SCN_TRY(scn_fill32(ctx, zeros, 0, (size_t)K));
  }
  return scn_nin_forward(ctx, d_D, Wt, zeros, nullptr, d_dA, M, N, K, 1.0f,
                         SCN_NOSIGMOID, SCN_FP32);
}

// dA = D W^T for callers that may not allocate (code under HIP graph capture,
// serving loops, harnesses that forbid hipMalloc): the transposed weights and
// the zero bias live in a file-scope device array instead of a caller's
// workspace.  Every device the library runs on holds its own copy of the array
// at its own address; host code reaches it only through the pointer that
// hipGetSymbolAddress returned for that device.
#define ABT_STATIC_FLOATS (1 << 20) // 4 MiB per device
static __device__ __align__(256) float scratch[ABT_STATIC_FLOATS];
#define ABT_MAX_DEVICES 64
// per device, set once by scn_ctx_create: the array's address, an event that
// marks the end of the last call that used it, and whose call that was
static float *g_abtScratch[ABT_MAX_DEVICES];
static hipEvent_t g_abtDone[ABT_MAX_DEVICES];
static const scn_ctx *g_abtUser[ABT_MAX_DEVICES];
static std::mutex g_abtMutex;

int scn_abt_static_setup(int device) {
  SCN_REQUIRE(device >= 0 && device < ABT_MAX_DEVICES, SCN_ERR_ARG,
              "device %d: at most %d devices", device, ABT_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_abtMutex); // (contexts are made by several threads)
  if (g_abtScratch[device])
    return SCN_OK;
  float *ptr = nullptr;
  SCN_HIP_CHECK(hipSetDevice(device));
  SCN_HIP_CHECK(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
  SCN_REQUIRE(ptr != nullptr, SCN_ERR_HIP,
              "hipGetSymbolAddress returned no address for the static scratch");
  SCN_HIP_CHECK(hipEventCreateWithFlags(&g_abtDone[device], hipEventDisableTiming));
  g_abtScratch[device] = ptr;
  return SCN_OK;
}

// a context that is destroyed gives the array up
void scn_abt_static_forget(const scn_ctx *ctx) {
  std::lock_guard<std::mutex> lock(g_abtMutex);
  for (int d = 0; d < ABT_MAX_DEVICES; ++d)
    if (g_abtUser[d] == ctx)
      g_abtUser[d] = nullptr;
}

extern "C" int64_t scn_sgemm_ABt_static_limit(void) { return ABT_STATIC_FLOATS; }

extern "C" int scn_sgemm_ABt_static(scn_ctx *ctx, const float *d_D,
                                    const float *d_W, float *d_dA, int64_t M,
                                    int N, int K) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_sgemm_ABt_static: null context");
  SCN_REQUIRE(M >= 0 && K >= 1 && N >= 1, SCN_ERR_ARG,
              "scn_sgemm_ABt_static: M %lld N %d K %d", (long long)M, N, K);
  SCN_REQUIRE(scn_sgemm_ABt_workspace(N, K) <= ABT_STATIC_FLOATS,
              SCN_ERR_CAPACITY,
              "scn_sgemm_ABt_static: N %d x K %d weights need %lld floats of "
              "scratch, the static array holds %d; use scn_sgemm_ABt with a "
              "workspace",
              N, K, (long long)scn_sgemm_ABt_workspace(N, K), ABT_STATIC_FLOATS);
  const int dev = ctx->device;
  float *ptr = dev >= 0 && dev < ABT_MAX_DEVICES ? g_abtScratch[dev] : nullptr;
  SCN_REQUIRE(ptr, SCN_ERR_STATE,
              "scn_sgemm_ABt_static: no scratch address for device %d", dev);
  if (M == 0)
    return SCN_OK;
  // One array a device: calls of one context follow each other on its stream;
  // a call of another context while the last one has not finished is refused.
  // (a stream under capture records and queries nothing: its owner has to
  // keep other users of the array away for as long as the graph may run)
  std::lock_guard<std::mutex> lock(g_abtMutex);
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  SCN_HIP_CHECK(hipStreamIsCapturing(ctx->stream, &capturing));
  if (g_abtUser[dev] && g_abtUser[dev] != ctx) {
    const hipError_t busy = hipEventQuery(g_abtDone[dev]);
    SCN_REQUIRE(busy != hipErrorNotReady, SCN_ERR_STATE,
                "scn_sgemm_ABt_static: the device's static array is still in "
                "use by a call of another context");
    SCN_HIP_CHECK(busy);
  }
  // (the kernels clear and fill what they use of the array: nothing of an
  // earlier call is read)
  SCN_TRY(scn_sgemm_ABt(ctx, d_D, d_W, d_dA, M, N, K, ptr));
  if (capturing == hipStreamCaptureStatusNone) {
    SCN_HIP_CHECK(hipEventRecord(g_abtDone[dev], ctx->stream));
    g_abtUser[dev] = ctx;
  }
  return SCN_OK;
}

// ---------------------------------------------------------- weight update
__global__ void k_nag_update(const float *__restrict__ delta,
                             float *__restrict__ mom, float *__restrict__ wts,
                             long long n, float lr, float mu, int keepPositive) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n)
    return;
  float w = wts[i], m = mom[i];
  const float d = delta[i];
  w -= m * mu;
  m = mu * m - lr * (1 - mu) * d;
  w += m * (1 + mu);
  if (keepPositive)
    w = w > 0.001f ? w : 0.001f;
  wts[i] = w;
  mom[i] = m;
}

extern "C" int scn_nag_update(scn_ctx *ctx, const float *d_delta,
                              float *d_momentum, float *d_weights, int64_t n,
                              float learningRate, float momentum,
                              int keepPositive) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_nag_update: null context");
  SCN_REQUIRE(n >= 0, SCN_ERR_ARG, "scn_nag_update: n %lld", (long long)n);
  if (n == 0)
    return SCN_OK;
  SCN_REQUIRE(d_delta && d_momentum && d_weights, SCN_ERR_ARG,
              "scn_nag_update: null buffer");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  hipLaunchKernelGGL(k_nag_update, dim3(scn_ceil_div(n, 256)), dim3(256), 0,
                     ctx->stream, d_delta, d_momentum, d_weights, (long long)n,
                     learningRate, momentum, keepPositive);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// The momentum step of several tensors (a layer's W, B and PReLU slopes) in
// one launch: a workgroup finds its tensor from the running workgroup counts.
// With `clear` the gradient is left zero, so the next batch's accumulating
// products need no clearing launch.
struct NagList {
  float *delta[SCN_NAG_MAX];
  float *mom[SCN_NAG_MAX];
  float *wts[SCN_NAG_MAX];
  long long n[SCN_NAG_MAX];
  unsigned firstBlock[SCN_NAG_MAX + 1];
  int keepPositive[SCN_NAG_MAX];
  int count;
};

__global__ __launch_bounds__(256) void k_nag_update_many(NagList l, float lr,
                                                         float mu, int clear) {
  int t = 0;
  while (t + 1 < l.count && blockIdx.x >= l.firstBlock[t + 1])
    ++t;
  const long long i =
      (long long)(blockIdx.x - l.firstBlock[t]) * blockDim.x + threadIdx.x;
  if (i >= l.n[t])
    return;
  float w = l.wts[t][i], m = l.mom[t][i];
  const float d = l.delta[t][i];
  w -= m * mu;
  m = mu * m - lr * (1 - mu) * d;
  w += m * (1 + mu);
  if (l.keepPositive[t])
    w = w > 0.001f ? w : 0.001f;
  l.wts[t][i] = w;
  l.mom[t][i] = m;
  if (clear)
    l.delta[t][i] = 0.f;
}

extern "C" int scn_nag_update_many(scn_ctx *ctx, const scn_nag_item *items,
                                   int nItems, float learningRate,
                                   float momentum, int clearGradients) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_nag_update_many: null context");
  SCN_REQUIRE(nItems >= 0 && nItems <= SCN_NAG_MAX && (items || nItems == 0),
              SCN_ERR_ARG, "scn_nag_update_many: %d items (at most %d)",
              nItems, SCN_NAG_MAX);
  NagList l;
  l.count = 0;
  long long blocks = 0;
  for (int k = 0; k < nItems; ++k) {
    const scn_nag_item &it = items[k];
    SCN_REQUIRE(it.n >= 0, SCN_ERR_ARG, "scn_nag_update_many: item %d n %lld",
                k, (long long)it.n);
    if (it.n == 0)
      continue;
    SCN_REQUIRE(it.d_delta && it.d_momentum && it.d_weights, SCN_ERR_ARG,
                "scn_nag_update_many: item %d null buffer", k);
    const int c = l.count++;
    l.delta[c] = it.d_delta;
    l.mom[c] = it.d_momentum;
    l.wts[c] = it.d_weights;
    l.n[c] = it.n;
    l.keepPositive[c] = it.keepPositive;
    l.firstBlock[c] = (unsigned)blocks;
    blocks += scn_ceil_div(it.n, 256);
    SCN_REQUIRE(blocks <= 0x7fffffffll, SCN_ERR_CAPACITY,
                "scn_nag_update_many: %lld workgroups", blocks);
  }
  if (l.count == 0)
    return SCN_OK;
  l.firstBlock[l.count] = (unsigned)blocks;
  ProfScope prof(ctx, SCN_K_BACKWARD);
  hipLaunchKernelGGL(k_nag_update_many, dim3((unsigned)blocks), dim3(256), 0,
                     ctx->stream, l, learningRate, momentum, clearGradients);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// ------------------------------------------------- scatter-add through rules
// A group of P lanes (P = the power of two that covers min(nIn, 64)) walks a
// run of consecutive rule entries; lane j of it owns channel j (+ P, + 2P ..).
// Consecutive entries that name the same input row (a sample's background row
// fills most of a sparse rule book) are summed in a register and reach memory
// as one atomic add.  Runs of 8: measured on the 2-D benchmark net, one atomic
// per entry and runs of 32 both cost 10 % more of a training step.
#define SCATTER_RUN 8
__global__ __launch_bounds__(256) void k_gather_backward(
    float *__restrict__ din, const float *__restrict__ dconv,
    const int *__restrict__ rules, long long count, int nIn, int P) {
  const long long lane = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long group = lane / P;
  const int li = (int)(lane - group * P);
  const long long e0 = group * SCATTER_RUN;
  if (e0 >= count)
    return;
  const long long e1 = e0 + SCATTER_RUN < count ? e0 + SCATTER_RUN : count;
  // the run's rules and values are all requested before the first is used
  int rl[SCATTER_RUN];
#pragma unroll
  for (int u = 0; u < SCATTER_RUN; ++u)
    rl[u] = e0 + u < e1 ? rules[e0 + u] : -1;
  for (int j = li; j < nIn; j += P) {
    float dv[SCATTER_RUN];
#pragma unroll
    for (int u = 0; u < SCATTER_RUN; ++u)
      dv[u] = e0 + u < e1 ? dconv[(e0 + u) * nIn + j] : 0.f;
    int cur = -1;
    float acc = 0.f;
#pragma unroll
    for (int u = 0; u < SCATTER_RUN; ++u) {
      const int r = rl[u];
      if (r < 0)
        continue;
      if (r != cur) {
        if (cur >= 0)
          unsafeAtomicAdd(din + (long long)cur * nIn + j, acc);
        cur = r;
        acc = 0.f;
      }
      acc += dv[u];
    }
    if (cur >= 0)
      unsafeAtomicAdd(din + (long long)cur * nIn + j, acc);
  }
}

static int group_width(int n) {
  int P = 1;
  while (P < n && P < 64)
    P <<= 1;
  return P;
}

extern "C" int scn_gather_rows_backward(scn_ctx *ctx, float *d_din,
                                        const float *d_dconv,
                                        const int32_t *d_rules, int64_t count,
                                        int nIn) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_gather_rows_backward: null context");
  SCN_REQUIRE(count >= 0 && nIn >= 1, SCN_ERR_ARG,
              "scn_gather_rows_backward: count %lld nIn %d", (long long)count,
              nIn);
  if (count == 0)
    return SCN_OK;
  SCN_REQUIRE(d_din && d_dconv && d_rules, SCN_ERR_ARG,
              "scn_gather_rows_backward: null buffer");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  const int P = group_width(nIn);
  const long long groups = (count + SCATTER_RUN - 1) / SCATTER_RUN;
  const long long blocks = (groups * P + 255) / 256;
  SCN_REQUIRE(blocks <= 0x7fffffffll, SCN_ERR_CAPACITY,
              "scn_gather_rows_backward: %lld workgroups", blocks);
  hipLaunchKernelGGL(k_gather_backward, dim3((unsigned)blocks), dim3(256), 0,
                     ctx->stream, d_din, d_dconv, d_rules, (long long)count,
                     nIn, P);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// dMaxPoolBackProp: the same walk over output rows, every lane following the
// choices of its own channel.
__global__ __launch_bounds__(256) void k_maxpool_backward(
    float *__restrict__ din, const float *__restrict__ dout, long long count,
    int C, const int *__restrict__ choice, int P) {
  const long long lane = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long group = lane / P;
  const int li = (int)(lane - group * P);
  const long long r0 = group * SCATTER_RUN;
  if (r0 >= count)
    return;
  const long long r1 = r0 + SCATTER_RUN < count ? r0 + SCATTER_RUN : count;
  for (int j = li; j < C; j += P) {
    int tg[SCATTER_RUN];
    float dv[SCATTER_RUN];
#pragma unroll
    for (int u = 0; u < SCATTER_RUN; ++u) {
      const bool live = r0 + u < r1;
      tg[u] = live ? choice[(r0 + u) * C + j] : -1;
      dv[u] = live ? dout[(r0 + u) * C + j] : 0.f;
    }
    int cur = -1;
    float acc = 0.f;
#pragma unroll
    for (int u = 0; u < SCATTER_RUN; ++u) {
      if (tg[u] < 0)
        continue;
      if (tg[u] != cur) {
        if (cur >= 0)
          unsafeAtomicAdd(din + cur, acc);
        cur = tg[u];
        acc = 0.f;
      }
      acc += dv[u];
    }
    if (cur >= 0)
      unsafeAtomicAdd(din + cur, acc);
  }
}

extern "C" int scn_maxpool_backward(scn_ctx *ctx, float *d_din,
                                    const float *d_dout, int64_t count, int C,
                                    const int32_t *d_choice) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_maxpool_backward: null context");
  SCN_REQUIRE(count >= 0 && C >= 1, SCN_ERR_ARG,
              "scn_maxpool_backward: count %lld C %d", (long long)count, C);
  if (count == 0)
    return SCN_OK;
  SCN_REQUIRE(d_din && d_dout && d_choice, SCN_ERR_ARG,
              "scn_maxpool_backward: null buffer");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  const int P = group_width(C);
  const long long groups = (count + SCATTER_RUN - 1) / SCATTER_RUN;
  const long long blocks = (groups * P + 255) / 256;
  SCN_REQUIRE(blocks <= 0x7fffffffll, SCN_ERR_CAPACITY,
              "scn_maxpool_backward: %lld workgroups", blocks);
  hipLaunchKernelGGL(k_maxpool_backward, dim3((unsigned)blocks), dim3(256), 0,
                     ctx->stream, d_din, d_dout, (long long)count, C, d_choice,
                     P);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// dTerminalPoolBackProp: every row listed for a sample receives (not
// accumulates) the sample's gradient divided by the number of rows listed.
__global__ void k_terminal_backward(float *__restrict__ din,
                                    const float *__restrict__ dout,
                                    const int *__restrict__ rules, int C,
                                    int S) {
  const long long b = blockIdx.x;
  const int *rr = rules + b * S;
  int maxP = 0;
  while (maxP < S && rr[maxP] >= 0)
    ++maxP;
  for (int j = threadIdx.x; j < C; j += blockDim.x) {
    const float t = dout[b * C + j] / (float)maxP;
    for (int p = 0; p < maxP; ++p)
      din[(long long)rr[p] * C + j] = t;
  }
}

extern "C" int scn_terminal_pool_backward(scn_ctx *ctx, float *d_din,
                                          const float *d_dout,
                                          const int32_t *d_rules,
                                          int64_t count, int C, int S) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_terminal_pool_backward: null context");
  SCN_REQUIRE(count >= 0 && C >= 1 && S >= 1, SCN_ERR_ARG,
              "scn_terminal_pool_backward: count %lld C %d S %d",
              (long long)count, C, S);
  if (count == 0)
    return SCN_OK;
  SCN_REQUIRE(count <= 0x7fffffffll, SCN_ERR_CAPACITY,
              "scn_terminal_pool_backward: %lld samples", (long long)count);
  SCN_REQUIRE(d_din && d_dout && d_rules, SCN_ERR_ARG,
              "scn_terminal_pool_backward: null buffer");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  hipLaunchKernelGGL(k_terminal_backward, dim3((unsigned)count),
                     dim3(C >= 256 ? 256 : 64), 0, ctx->stream, d_din, d_dout,
                     d_rules, C, S);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// ------------------------------------------------ dropout during training
// A training batch keeps a random subset of every layer's features
// (featuresPresent); the layer then works on the sub-matrix of its weights
// that joins the kept inputs to the kept outputs.
__global__ void k_shrink_matrix(const float *__restrict__ W,
                                float *__restrict__ w,
                                const int *__restrict__ inPresent,
                                const int *__restrict__ outPresent, int nOut,
                                long long total, int nOutP) {
  long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total)
    return;
  const long long i = idx / nOutP;
  const int j = (int)(idx - i * nOutP);
  const long long row = inPresent ? inPresent[i] : i;
  w[idx] = W[row * nOut + outPresent[j]];
}

extern "C" int scn_shrink_matrix(scn_ctx *ctx, const float *d_W, float *d_w,
                                 const int32_t *d_inPresent,
                                 const int32_t *d_outPresent, int nOut,
                                 int nInPresent, int nOutPresent) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_shrink_matrix: null context");
  SCN_REQUIRE(nOut >= 1 && nInPresent >= 0 && nOutPresent >= 0 &&
                  nOutPresent <= nOut,
              SCN_ERR_ARG, "scn_shrink_matrix: nOut %d present %d x %d", nOut,
              nInPresent, nOutPresent);
  const long long total = (long long)nInPresent * nOutPresent;
  if (total == 0)
    return SCN_OK;
  SCN_REQUIRE(d_W && d_w && d_outPresent, SCN_ERR_ARG,
              "scn_shrink_matrix: null buffer");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  hipLaunchKernelGGL(k_shrink_matrix, dim3(scn_ceil_div(total, 256)), dim3(256),
                     0, ctx->stream, d_W, d_w, d_inPresent, d_outPresent, nOut,
                     total, nOutPresent);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// dGradientDescentShrunkMatrix: the momentum step on the entries of W (and MW)
// that the batch used; delta is the gradient of the shrunk matrix.
__global__ void k_nag_update_shrunk(const float *__restrict__ delta,
                                    float *__restrict__ mom,
                                    float *__restrict__ wts,
                                    const int *__restrict__ inPresent,
                                    const int *__restrict__ outPresent,
                                    int nOut, long long total, int nOutP,
                                    float lr, float mu) {
  long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total)
    return;
  const long long i = idx / nOutP;
  const int j = (int)(idx - i * nOutP);
  const long long row = inPresent ? inPresent[i] : i;
  const long long at = row * nOut + outPresent[j];
  float w = wts[at], m = mom[at];
  const float d = delta[idx];
  w -= m * mu;
  m = mu * m - lr * (1 - mu) * d;
  w += m * (1 + mu);
  wts[at] = w;
  mom[at] = m;
}

extern "C" int scn_nag_update_shrunk(scn_ctx *ctx, const float *d_delta,
                                     float *d_momentum, float *d_weights,
                                     const int32_t *d_inPresent,
                                     const int32_t *d_outPresent, int nOut,
                                     int nInPresent, int nOutPresent,
                                     float learningRate, float momentum) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_nag_update_shrunk: null context");
  SCN_REQUIRE(nOut >= 1 && nInPresent >= 0 && nOutPresent >= 0 &&
                  nOutPresent <= nOut,
              SCN_ERR_ARG, "scn_nag_update_shrunk: nOut %d present %d x %d",
              nOut, nInPresent, nOutPresent);
  const long long total = (long long)nInPresent * nOutPresent;
  if (total == 0)
    return SCN_OK;
  SCN_REQUIRE(d_delta && d_momentum && d_weights && d_outPresent, SCN_ERR_ARG,
              "scn_nag_update_shrunk: null buffer");
  ProfScope prof(ctx, SCN_K_BACKWARD);
  hipLaunchKernelGGL(k_nag_update_shrunk, dim3(scn_ceil_div(total, 256)),
                     dim3(256), 0, ctx->stream, d_delta, d_momentum, d_weights,
                     d_inPresent, d_outPresent, nOut, total, nOutPresent,
                     learningRate, momentum);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// ------------------------------------------------ weight rescaling passes
// What a RESCALEBATCH needs of vectorCUDA<float>: meanAbs() and
// multiplicativeRescale() (vectorCUDA.cu:121-170).
__global__ __launch_bounds__(256) void k_sum_abs(const float *__restrict__ x,
                                                 long long n, double *out) {
  __shared__ double part[4];
  double s = 0;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x)
    s += fabsf(x[i]);
  for (int o = 32; o > 0; o >>= 1)
    s += __shfl_down(s, o, 64);
  if ((threadIdx.x & 63) == 0)
    part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0)
    unsafeAtomicAdd(out, part[0] + part[1] + part[2] + part[3]);
}

extern "C" int scn_sum_abs(scn_ctx *ctx, const float *d_x, int64_t n,
                           double *h_sum) {
  SCN_REQUIRE(ctx && h_sum, SCN_ERR_ARG, "scn_sum_abs: null argument");
  SCN_REQUIRE(n >= 0, SCN_ERR_ARG, "scn_sum_abs: n %lld", (long long)n);
  *h_sum = 0;
  if (n == 0)
    return SCN_OK;
  SCN_REQUIRE(d_x, SCN_ERR_ARG, "scn_sum_abs: null buffer");
  double *acc = (double *)(ctx->d_scalars + 8); // words 8..9: free for this
  SCN_TRY(scn_fill32(ctx, acc, 0u, 2));
  int blocks = scn_ceil_div(n, 256 * 16);
  if (blocks > ctx->numCU * 8)
    blocks = ctx->numCU * 8;
  hipLaunchKernelGGL(k_sum_abs, dim3(blocks), dim3(256), 0, ctx->stream, d_x,
                     (long long)n, acc);
  SCN_HIP_CHECK(hipGetLastError());
  return scn_d2h(ctx, h_sum, acc, sizeof(double));
}

__global__ void k_scale(float *__restrict__ x, long long n, float m) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    x[i] *= m;
}

extern "C" int scn_scale(scn_ctx *ctx, float *d_x, int64_t n,
                         float multiplier) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_scale: null context");
  SCN_REQUIRE(n >= 0, SCN_ERR_ARG, "scn_scale: n %lld", (long long)n);
  if (n == 0)
    return SCN_OK;
  SCN_REQUIRE(d_x, SCN_ERR_ARG, "scn_scale: null buffer");
  hipLaunchKernelGGL(k_scale, dim3(scn_ceil_div(n, 256)), dim3(256), 0,
                     ctx->stream, d_x, (long long)n, multiplier);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}
