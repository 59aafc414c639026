// NetworkInNetwork forward: out = act(p * (A W + B)), bias and activation
// fused into the contraction's epilogue (the reference runs replicateArray,
// cublasSgemm and applySigmoid / PreLU as three passes over the output).
#include "scn_common.h"

int scn_softmax_launch(scn_ctx *ctx, const float *d_in, float *d_out,
                       long long M, int N);

struct Epilogue {
  const float *bias;
  const float *prelu;
  float p;
  float slope;
  int act;
};

__device__ __forceinline__ float apply_act(float acc, int n,
                                           const Epilogue &e) {
  // alpha * (A W) + beta * C with C preset to the bias and alpha = beta = p
  // (NetworkInNetworkLayer.cu:188-194)
  float v = e.p * acc + e.p * e.bias[n];
  switch (e.act) {
  case SCN_RELU:
    return v > 0.f ? v : 0.f;
  case SCN_LEAKYRELU:
  case SCN_VLEAKYRELU:
    return v > 0.f ? v : v * e.slope;
  case SCN_PRELU:
    return v > 0.f ? v : v * e.prelu[n];
  default:
    return v;
  }
}

// ---- generic path: any M, K, N; 64x64 tile, 4x4 per lane, fp32 FMA --------
#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

__global__ void __launch_bounds__(256)
    k_nin_generic(const float *__restrict__ A, const float *__restrict__ W,
                  float *__restrict__ out, long long M, int K, int N,
                  Epilogue ep) {
  __shared__ float sA[GT_BK][GT_BM + 4];
  __shared__ float sW[GT_BK][GT_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const long long m0 = (long long)blockIdx.x * GT_BM;
  const int n0 = blockIdx.y * GT_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += GT_BK) {
    // A tile: 64 rows x 16 k ; 1024 elements, 4 per lane
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      int e = tid + u * 256;
      int r = e >> 4, kk = e & 15;
      long long m = m0 + r;
      int k = k0 + kk;
      sA[kk][r] = (m < M && k < K) ? A[m * K + k] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      int e = tid + u * 256;
      int kk = e >> 6, c = e & 63;
      int k = k0 + kk, n = n0 + c;
      sW[kk][c] = (k < K && n < N) ? W[(long long)k * N + n] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GT_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = sA[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w[j] = sW[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    long long m = m0 + ty * 4 + i;
    if (m >= M)
      continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int n = n0 + tx * 4 + j;
      if (n < N)
        out[m * N + n] = apply_act(acc[i][j], n, ep);
    }
  }
}

// ---- MFMA path: fp32 operands, v_mfma_f32_32x32x2_f32 ----------------------
// Block = 4 wavefronts laid out WM x WN; every wavefront owns a 32 x (32 NT)
// patch of the output as NT accumulator tiles of 32x32 (16 VGPRs per lane
// each).  Operands are staged through LDS in k-slabs of MF_BK, double
// buffered: A transposed to [k][row] (row stride odd, so both the transposing
// stores and the operand reads hit every bank evenly), W as [k][col].  One
// MFMA consumes k = 2: lane l supplies A[row = l % 32][k = l / 32] and
// W[k = l / 32][col = l % 32]; accumulator register v of lane l is
// D[row = 8 (v / 4) + 4 (l / 32) + v % 4][col = l % 32].
#define MF_BK 32
typedef float floatx16 __attribute__((ext_vector_type(16)));

//
// GATHER: A is never materialised.  Row m of A is the receptive field of
// output site m, column q * nIn + c = channel c of input row
// rules[m * fs + q] (what scn_gather_rows would have written); the block's
// rules are staged in LDS once and the A slabs are fetched through them.
#define GF_MAX_FS 27
struct GatherSource {
  const int *rules; // [M x fs]
  int fs;           // rule-row width
  int nIn;          // channels of the gathered matrix, nIn % 4 == 0
};

template <int WM, int WN, int NT, int BK, bool GATHER>
__global__ void __launch_bounds__(256)
    k_nin_mfma(const float *__restrict__ A, const float *__restrict__ W,
               float *__restrict__ out, long long M, int K, int N,
               Epilogue ep, GatherSource gs) {
  constexpr int BM = 32 * WM;
  constexpr int BN = 32 * NT * WN;
  constexpr int BMP = BM + 1;
  constexpr int A_CHUNKS = BM * BK / 4; // float4 chunks per slab
  constexpr int W_CHUNKS = BK * BN / 4;
  constexpr int A_PER = (A_CHUNKS + 255) / 256;
  constexpr int W_PER = (W_CHUNKS + 255) / 256;
  __shared__ float sA[2][BK * BMP];
  __shared__ float sW[2][BK * BN];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // Consecutive workgroup ids go to consecutive XCDs (8, each with its own
  // L2).  The n-blocks that share an A slab are given ids that land on ONE
  // XCD: id = slot * 8 + xcd  ->  tile = xcd * (grid / 8) + slot.
  const int nBlocksN = (N + BN - 1) / BN;
  const long long nTiles = ((M + BM - 1) / BM) * nBlocksN;
  const long long tile =
      (long long)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (tile >= nTiles)
    return; // the grid is rounded up to a multiple of 8
  const long long m0 = (tile / nBlocksN) * BM;
  const int n0 = (int)(tile % nBlocksN) * BN;
  floatx16 acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      acc[j][v] = 0.f;
  __shared__ int sR[GATHER ? BM * GF_MAX_FS : 1];
  if (GATHER) {
    // the rules of rows m0 .. m0 + BM are one contiguous run
    const long long first = m0 * gs.fs;
    const long long limit = M * gs.fs;
    for (int idx = tid; idx < BM * gs.fs; idx += 256)
      sR[idx] = first + idx < limit ? gs.rules[first + idx] : -1;
    __syncthreads();
  }

  float4 ra[A_PER], rw[W_PER];
  auto load_slab = [&](int k0) {
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      int c = tid + u * 256;
      int r = c / (BK / 4), kc = c % (BK / 4);
      long long m = m0 + r;
      int k = k0 + kc * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (c < A_CHUNKS && m < M && k < K) { // K % 4 == 0: a chunk is all in or all out
        if (GATHER) {
          int q = k / gs.nIn;
          int rule = sR[r * gs.fs + q];
          if (rule >= 0)
            v = *reinterpret_cast<const float4 *>(
                A + (long long)rule * gs.nIn + (k - q * gs.nIn));
        } else {
          v = *reinterpret_cast<const float4 *>(A + m * K + k);
        }
      }
      ra[u] = v;
    }
#pragma unroll
    for (int u = 0; u < W_PER; ++u) {
      int c = tid + u * 256;
      int kk = c / (BN / 4), nc = c % (BN / 4);
      int k = k0 + kk, n = n0 + nc * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (c < W_CHUNKS && k < K && n < N) // N % 4 == 0
        v = *reinterpret_cast<const float4 *>(W + (long long)k * N + n);
      rw[u] = v;
    }
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      int c = tid + u * 256;
      if (c < A_CHUNKS) {
        int r = c / (BK / 4), kc = c % (BK / 4);
        float *dst = &sA[buf][(kc * 4) * BMP + r];
        dst[0] = ra[u].x;
        dst[BMP] = ra[u].y;
        dst[2 * BMP] = ra[u].z;
        dst[3 * BMP] = ra[u].w;
      }
    }
#pragma unroll
    for (int u = 0; u < W_PER; ++u) {
      int c = tid + u * 256;
      if (c < W_CHUNKS)
        *reinterpret_cast<float4 *>(&sW[buf][c * 4]) = rw[u];
    }
  };

  const int nSlabs = (K + BK - 1) / BK;
  load_slab(0);
  store_slab(0);
  __syncthreads();
  for (int s = 0; s < nSlabs; ++s) {
    const int buf = s & 1;
    if (s + 1 < nSlabs)
      load_slab((s + 1) * BK); // in flight while this slab is multiplied
    const float *pa = &sA[buf][(lane >> 5) * BMP + wm * 32 + (lane & 31)];
    const float *pw = &sW[buf][(lane >> 5) * BN + wn * 32 * NT + (lane & 31)];
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      float a = pa[kk * BMP];
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        float b = pw[kk * BN + 32 * j];
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[j], 0, 0, 0);
      }
    }
    if (s + 1 < nSlabs)
      store_slab(buf ^ 1);
    __syncthreads();
  }

  const int col = lane & 31;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    int n = n0 + (wn * NT + j) * 32 + col;
    if (n >= N)
      continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      long long m = m0 + wm * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
      if (m < M)
        out[m * N + n] = apply_act(acc[j][v], n, ep);
    }
  }
}

// ---- MFMA path with bf16 operands: v_mfma_f32_32x32x16_bf16 ----------------
// A and W stay fp32 in HBM; they are rounded to bf16 (nearest even) on their
// way into LDS and accumulated in fp32.  One MFMA consumes k = 16: lane l
// supplies eight consecutive k of row / column l % 32 starting at
// k = 8 (l / 32), so both operands sit in LDS with k contiguous:
// sA[row][k], sW[col][k], rows padded to 40 elements (80 bytes) so that the
// 128-bit operand reads spread over all banks.
//
// SPLIT keeps the rounding residue as a second bf16 (x = hi + lo up to 2^-17)
// and issues three MFMAs per tile, hi*hi + hi*lo + lo*hi: fp32-grade results
// at a third of the bf16 rate, still several times the fp32 MFMA rate.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
#define BF_ROW 40

__device__ __forceinline__ unsigned short to_bf16(float f) {
  unsigned u = __float_as_uint(f);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}
__device__ __forceinline__ uint4 pack_bf16x8(const float *v) {
  uint4 r;
  r.x = to_bf16(v[0]) | ((unsigned)to_bf16(v[1]) << 16);
  r.y = to_bf16(v[2]) | ((unsigned)to_bf16(v[3]) << 16);
  r.z = to_bf16(v[4]) | ((unsigned)to_bf16(v[5]) << 16);
  r.w = to_bf16(v[6]) | ((unsigned)to_bf16(v[7]) << 16);
  return r;
}
// v[i] -= float(bf16(v[i])): what the first rounding lost
__device__ __forceinline__ void residue8(float *v) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    v[i] -= __uint_as_float((unsigned)to_bf16(v[i]) << 16);
}

template <int WM, int WN, int NT, bool SPLIT>
__global__ void __launch_bounds__(256)
    k_nin_mfma_bf16(const float *__restrict__ A, const float *__restrict__ W,
                    float *__restrict__ out, long long M, int K, int N,
                    Epilogue ep) {
  constexpr int BM = 32 * WM;
  constexpr int BN = 32 * NT * WN;
  constexpr int A_ITEMS = BM * (MF_BK / 8); // one item = 8 consecutive k of a row
  constexpr int W_ITEMS = BN * (MF_BK / 8); // 8 consecutive k of a column
  constexpr int A_PER = (A_ITEMS + 255) / 256;
  constexpr int W_PER = (W_ITEMS + 255) / 256;
  constexpr int PARTS = SPLIT ? 2 : 1; // hi, lo
  __shared__ __attribute__((aligned(16))) unsigned short sA[2][PARTS][BM * BF_ROW];
  __shared__ __attribute__((aligned(16))) unsigned short sW[2][PARTS][BN * BF_ROW];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int nBlocksN = (N + BN - 1) / BN;
  const long long m0 = (long long)(blockIdx.x / nBlocksN) * BM;
  const int n0 = (int)(blockIdx.x % nBlocksN) * BN;
  floatx16 acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      acc[j][v] = 0.f;

  uint4 ra[A_PER][PARTS], rw[W_PER][PARTS];
  auto load_slab = [&](int k0) {
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      int c = tid + u * 256;
      int r = c / (MF_BK / 8), kc = c % (MF_BK / 8);
      long long m = m0 + r;
      int k = k0 + kc * 8;
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (c < A_ITEMS && m < M) {
        const float *src = A + m * K + k;
        if (k + 8 <= K) {
          float4 x = *reinterpret_cast<const float4 *>(src);
          float4 y = *reinterpret_cast<const float4 *>(src + 4);
          v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
          v[4] = y.x, v[5] = y.y, v[6] = y.z, v[7] = y.w;
        } else if (k < K) { // K % 4 == 0: exactly four left
          float4 x = *reinterpret_cast<const float4 *>(src);
          v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
        }
      }
      ra[u][0] = pack_bf16x8(v);
      if (SPLIT) {
        residue8(v);
        ra[u][PARTS - 1] = pack_bf16x8(v);
      }
    }
#pragma unroll
    for (int u = 0; u < W_PER; ++u) {
      int c = tid + u * 256;
      int kc = c / BN, nn = c % BN; // consecutive lanes: consecutive columns
      int n = n0 + nn, k = k0 + kc * 8;
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (c < W_ITEMS && n < N) {
#pragma unroll
        for (int q = 0; q < 8; ++q)
          if (k + q < K)
            v[q] = W[(long long)(k + q) * N + n];
      }
      rw[u][0] = pack_bf16x8(v);
      if (SPLIT) {
        residue8(v);
        rw[u][PARTS - 1] = pack_bf16x8(v);
      }
    }
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      int c = tid + u * 256;
      if (c < A_ITEMS) {
        int r = c / (MF_BK / 8), kc = c % (MF_BK / 8);
#pragma unroll
        for (int h = 0; h < PARTS; ++h)
          *reinterpret_cast<uint4 *>(&sA[buf][h][r * BF_ROW + kc * 8]) = ra[u][h];
      }
    }
#pragma unroll
    for (int u = 0; u < W_PER; ++u) {
      int c = tid + u * 256;
      if (c < W_ITEMS) {
        int kc = c / BN, nn = c % BN;
#pragma unroll
        for (int h = 0; h < PARTS; ++h)
          *reinterpret_cast<uint4 *>(&sW[buf][h][nn * BF_ROW + kc * 8]) = rw[u][h];
      }
    }
  };

  const int nSlabs = (K + MF_BK - 1) / MF_BK;
  load_slab(0);
  store_slab(0);
  __syncthreads();
  const int offA = (wm * 32 + (lane & 31)) * BF_ROW + 8 * (lane >> 5);
  const int offW = (wn * 32 * NT + (lane & 31)) * BF_ROW + 8 * (lane >> 5);
  for (int s = 0; s < nSlabs; ++s) {
    const int buf = s & 1;
    if (s + 1 < nSlabs)
      load_slab((s + 1) * MF_BK);
#pragma unroll
    for (int kk = 0; kk < MF_BK; kk += 16) {
      bf16x8 a = *reinterpret_cast<const bf16x8 *>(&sA[buf][0][offA + kk]);
      bf16x8 al;
      if (SPLIT)
        al = *reinterpret_cast<const bf16x8 *>(&sA[buf][PARTS - 1][offA + kk]);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const int o = offW + 32 * j * BF_ROW + kk;
        bf16x8 b = *reinterpret_cast<const bf16x8 *>(&sW[buf][0][o]);
        if (SPLIT) {
          bf16x8 bl = *reinterpret_cast<const bf16x8 *>(&sW[buf][PARTS - 1][o]);
          // small terms first
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, b, acc[j], 0, 0, 0);
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bl, acc[j], 0, 0, 0);
        }
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
      }
    }
    if (s + 1 < nSlabs)
      store_slab(buf ^ 1);
    __syncthreads();
  }

  const int col = lane & 31;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    int n = n0 + (wn * NT + j) * 32 + col;
    if (n >= N)
      continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      long long m = m0 + wm * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
      if (m < M)
        out[m * N + n] = apply_act(acc[j][v], n, ep);
    }
  }
}

template <int WM, int WN, int NT>
static void launch_mfma_bf16(scn_ctx *ctx, const float *A, const float *W,
                             float *out, long long M, int K, int N,
                             const Epilogue &ep, bool split) {
  constexpr int BM = 32 * WM, BN = 32 * NT * WN;
  dim3 grid((unsigned)((long long)scn_ceil_div(N, BN) * scn_ceil_div(M, BM)));
  if (split)
    hipLaunchKernelGGL((k_nin_mfma_bf16<WM, WN, NT, true>), grid, dim3(256), 0,
                       ctx->stream, A, W, out, M, K, N, ep);
  else
    hipLaunchKernelGGL((k_nin_mfma_bf16<WM, WN, NT, false>), grid, dim3(256), 0,
                       ctx->stream, A, W, out, M, K, N, ep);
}

template <int WM, int WN, int NT, int BK = MF_BK>
static void launch_mfma(scn_ctx *ctx, const float *A, const float *W,
                        float *out, long long M, int K, int N,
                        const Epilogue &ep, const GatherSource *gs = nullptr) {
  constexpr int BM = 32 * WM, BN = 32 * NT * WN;
  long long tiles = (long long)scn_ceil_div(N, BN) * scn_ceil_div(M, BM);
  dim3 grid((unsigned)((tiles + 7) / 8 * 8));
  if (gs)
    hipLaunchKernelGGL((k_nin_mfma<WM, WN, NT, BK, true>), grid, dim3(256), 0,
                       ctx->stream, A, W, out, M, K, N, ep, *gs);
  else
    hipLaunchKernelGGL((k_nin_mfma<WM, WN, NT, BK, false>), grid, dim3(256), 0,
                       ctx->stream, A, W, out, M, K, N, ep, GatherSource());
}

static int nin_forward(scn_ctx *ctx, const float *d_A, const float *d_W,
                       const float *d_B, const float *d_prelu, float *d_out,
                       int64_t M, int K, int N, float p, int act, int precision,
                       const GatherSource *gs) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_nin_forward: null context");
  SCN_REQUIRE(M >= 0 && K >= 1 && N >= 1, SCN_ERR_ARG,
              "scn_nin_forward: M %lld K %d N %d", (long long)M, K, N);
  SCN_REQUIRE(act == SCN_NOSIGMOID || act == SCN_RELU || act == SCN_VLEAKYRELU ||
                  act == SCN_LEAKYRELU || act == SCN_SOFTMAX || act == SCN_PRELU,
              SCN_ERR_ARG, "scn_nin_forward: activation %d is not supported",
              act);
  SCN_REQUIRE(precision == SCN_FP32 || precision == SCN_BF16 ||
                  precision == SCN_BF16X3,
              SCN_ERR_ARG,
              "scn_nin_forward: precision %d", precision);
  if (M == 0)
    return SCN_OK;
  SCN_REQUIRE(d_A && d_W && d_B && d_out, SCN_ERR_ARG,
              "scn_nin_forward: null buffer");
  SCN_REQUIRE(act != SCN_PRELU || d_prelu, SCN_ERR_ARG,
              "scn_nin_forward: PReLU needs the slope vector");
  Epilogue ep;
  ep.bias = d_B;
  ep.prelu = d_prelu;
  ep.p = p;
  // SigmoidLayer.cu:204-213
  ep.slope = act == SCN_LEAKYRELU ? 0.01f : (act == SCN_VLEAKYRELU ? 0.333f : 0.f);
  ep.act = act;
  ProfScope prof(ctx, gs ? SCN_K_CONV_NIN : SCN_K_NIN);
  const bool vec = K % 4 == 0 && N % 4 == 0 && ((uintptr_t)d_A & 15) == 0 &&
                   ((uintptr_t)d_W & 15) == 0;
  // bf16 operands only where the contraction is big enough to matter; the
  // classifier head and the thin first layers stay fp32
  if (vec && K >= 64 && act != SCN_SOFTMAX && precision != SCN_FP32) {
    const bool split = precision == SCN_BF16X3;
    long long blocksLarge = (long long)scn_ceil_div(M, 128) * scn_ceil_div(N, 64);
    if (N <= 32)
      launch_mfma_bf16<4, 1, 1>(ctx, d_A, d_W, d_out, M, K, N, ep, split);
    else if (blocksLarge >= ctx->numCU)
      launch_mfma_bf16<4, 1, 2>(ctx, d_A, d_W, d_out, M, K, N, ep, split);
    else
      launch_mfma_bf16<1, 4, 1>(ctx, d_A, d_W, d_out, M, K, N, ep, split);
  } else if ((vec && K >= 8) || gs) {
    // Tall tiles (128 rows), 64 columns wide, or 96 where that divides N
    // (measured on 12928 x 1280 x 480: 93 TFLOP/s against 73 with 64-column
    // tiles; wider tiles leave too few workgroups for 256 compute units).
    const int maxCols = N % 96 == 0 ? 96 : 64;
    const int nChunks = (N + maxCols - 1) / maxCols;
    const int nt = ((N + 31) / 32 + nChunks - 1) / nChunks; // 1..6
    long long blocksTall = (long long)scn_ceil_div(M, 128) * nChunks;
    if (blocksTall * 2 < ctx->numCU && N > 32) {
      // too few rows to fill the chip with tall tiles: 32-row tiles
      launch_mfma<1, 4, 1>(ctx, d_A, d_W, d_out, M, K, N, ep, gs);
    } else {
      switch (nt) {
      case 1:
        launch_mfma<4, 1, 1>(ctx, d_A, d_W, d_out, M, K, N, ep, gs);
        break;
      case 2:
        launch_mfma<4, 1, 2>(ctx, d_A, d_W, d_out, M, K, N, ep, gs);
        break;
      default:
        launch_mfma<4, 1, 3>(ctx, d_A, d_W, d_out, M, K, N, ep, gs);
        break;
      }
    }
  } else {
    dim3 grid(scn_ceil_div(M, GT_BM), scn_ceil_div(N, GT_BN));
    hipLaunchKernelGGL(k_nin_generic, grid, dim3(256), 0, ctx->stream, d_A,
                       d_W, d_out, (long long)M, K, N, ep);
  }
  SCN_HIP_CHECK(hipGetLastError());
  if (act == SCN_SOFTMAX)
    SCN_TRY(scn_softmax_launch(ctx, d_out, d_out, (long long)M, N));
  return SCN_OK;
}

extern "C" int scn_nin_forward(scn_ctx *ctx, const float *d_A,
                               const float *d_W, const float *d_B,
                               const float *d_prelu, float *d_out, int64_t M,
                               int K, int N, float p, int act, int precision) {
  return nin_forward(ctx, d_A, d_W, d_B, d_prelu, d_out, M, K, N, p, act,
                     precision, nullptr);
}

extern "C" int scn_conv_nin_supported(int fs, int nIn, int N) {
  return fs >= 1 && fs <= GF_MAX_FS && nIn >= 4 && nIn % 4 == 0 && N % 4 == 0;
}

extern "C" int scn_conv_nin_forward(scn_ctx *ctx, const float *d_in,
                                    const int32_t *d_rules, int fs, int nIn,
                                    const float *d_W, const float *d_B,
                                    const float *d_prelu, float *d_out,
                                    int64_t M, int N, float p, int act) {
  SCN_REQUIRE(scn_conv_nin_supported(fs, nIn, N), SCN_ERR_ARG,
              "scn_conv_nin_forward: fs %d nIn %d N %d is outside the fused "
              "kernel's range (fs <= %d, nIn and N multiples of 4)",
              fs, nIn, N, GF_MAX_FS);
  SCN_REQUIRE(d_rules || M == 0, SCN_ERR_ARG,
              "scn_conv_nin_forward: null rules");
  SCN_REQUIRE(((uintptr_t)d_in & 15) == 0 && ((uintptr_t)d_W & 15) == 0,
              SCN_ERR_ARG, "scn_conv_nin_forward: buffers must be 16-byte aligned");
  GatherSource gs;
  gs.rules = d_rules;
  gs.fs = fs;
  gs.nIn = nIn;
  return nin_forward(ctx, d_in, d_W, d_B, d_prelu, d_out, M, fs * nIn, N, p,
                     act, SCN_FP32, &gs);
}
