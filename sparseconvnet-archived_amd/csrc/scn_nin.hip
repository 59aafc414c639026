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

extern "C" int scn_nin_forward(scn_ctx *ctx, const float *d_A,
                               const float *d_W, const float *d_B,
                               const float *d_prelu, float *d_out, int64_t M,
                               int K, int N, float p, int act, int precision) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_nin_forward: null context");
  SCN_REQUIRE(M >= 0 && K >= 1 && N >= 1, SCN_ERR_ARG,
              "scn_nin_forward: M %lld K %d N %d", (long long)M, K, N);
  SCN_REQUIRE(act == SCN_NOSIGMOID || act == SCN_RELU || act == SCN_VLEAKYRELU ||
                  act == SCN_LEAKYRELU || act == SCN_SOFTMAX || act == SCN_PRELU,
              SCN_ERR_ARG, "scn_nin_forward: activation %d is not supported",
              act);
  SCN_REQUIRE(precision == SCN_FP32 || precision == SCN_BF16, SCN_ERR_ARG,
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
  ProfScope prof(ctx, SCN_K_NIN);
  dim3 grid(scn_ceil_div(M, GT_BM), scn_ceil_div(N, GT_BN));
  hipLaunchKernelGGL(k_nin_generic, grid, dim3(256), 0, ctx->stream, d_A, d_W,
                     d_out, (long long)M, K, N, ep);
  SCN_HIP_CHECK(hipGetLastError());
  if (act == SCN_SOFTMAX)
    SCN_TRY(scn_softmax_launch(ctx, d_out, d_out, (long long)M, N));
  return SCN_OK;
}
