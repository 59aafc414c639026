// Rule-driven feature kernels: gather, max-pool with argmax, terminal
// average, softmax.  All of them move bytes: they are sized and indexed for
// HBM bandwidth (128-bit accesses wherever the channel count allows, rule
// offsets staged in LDS, 64-bit element offsets).
#include "scn_common.h"

#define GATHER_TILE 256 // rules per block iteration
#define GATHER_THREADS 256

// out[c * nIn + j] = in[rules[c] * nIn + j]   (ConvolutionalLayer.cu:12-31)
// The output is one contiguous run per tile, so consecutive lanes write
// consecutive 16-byte chunks; reads are contiguous per rule.  A negative rule
// (the reference reads out of bounds on one) gathers a row of zeros.
template <typename VecT, int VEC>
__global__ void __launch_bounds__(GATHER_THREADS)
    k_gather(const float *__restrict__ in, float *__restrict__ out,
             const int *__restrict__ rules, long long count, int nIn,
             int chunks) {
  __shared__ long long roff[GATHER_TILE];
  const int tid = threadIdx.x;
  const int q0 = tid / chunks, ch0 = tid - q0 * chunks;
  const int dq = GATHER_THREADS / chunks, dch = GATHER_THREADS - dq * chunks;
  for (long long c0 = (long long)blockIdx.x * GATHER_TILE; c0 < count;
       c0 += (long long)gridDim.x * GATHER_TILE) {
    long long left = count - c0;
    const int n = left < GATHER_TILE ? (int)left : GATHER_TILE;
    if (tid < n) {
      int rule = rules[c0 + tid];
      roff[tid] = rule < 0 ? -1 : (long long)rule * nIn;
    }
    __syncthreads();
    const int items = n * chunks;
    VecT *dst = reinterpret_cast<VecT *>(out + c0 * nIn);
    int q = q0, ch = ch0;
    int idx = tid;
    // four independent loads in flight per lane
    for (; idx + 3 * GATHER_THREADS < items; idx += 4 * GATHER_THREADS) {
      VecT v[4];
      int qq = q, cc = ch;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        long long ro = roff[qq];
        v[u] = ro < 0 ? VecT{} : *reinterpret_cast<const VecT *>(in + ro + cc * VEC);
        qq += dq;
        cc += dch;
        if (cc >= chunks) {
          cc -= chunks;
          ++qq;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        dst[idx + u * GATHER_THREADS] = v[u];
      q = qq;
      ch = cc;
    }
    for (; idx < items; idx += GATHER_THREADS) {
      long long ro = roff[q];
      dst[idx] = ro < 0 ? VecT{} : *reinterpret_cast<const VecT *>(in + ro + ch * VEC);
      q += dq;
      ch += dch;
      if (ch >= chunks) {
        ch -= chunks;
        ++q;
      }
    }
    __syncthreads();
  }
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

extern "C" int scn_gather_rows(scn_ctx *ctx, const float *d_in, float *d_out,
                               const int32_t *d_rules, int64_t count,
                               int nIn) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_gather_rows: null context");
  SCN_REQUIRE(count >= 0 && nIn >= 1, SCN_ERR_ARG,
              "scn_gather_rows: count %lld nIn %d", (long long)count, nIn);
  if (count == 0)
    return SCN_OK;
  SCN_REQUIRE(d_in && d_out && d_rules, SCN_ERR_ARG,
              "scn_gather_rows: null buffer");
  ProfScope ps(ctx, SCN_K_GATHER);
  long long tiles = (count + GATHER_TILE - 1) / GATHER_TILE;
  long long maxBlocks = (long long)ctx->numCU * 16;
  int blocks = (int)(tiles < maxBlocks ? tiles : maxBlocks);
  if (nIn % 4 == 0 && aligned16(d_in) && aligned16(d_out)) {
    hipLaunchKernelGGL((k_gather<float4, 4>), dim3(blocks),
                       dim3(GATHER_THREADS), 0, ctx->stream, d_in, d_out,
                       d_rules, (long long)count, nIn, nIn / 4);
  } else {
    hipLaunchKernelGGL((k_gather<float, 1>), dim3(blocks),
                       dim3(GATHER_THREADS), 0, ctx->stream, d_in, d_out,
                       d_rules, (long long)count, nIn, nIn);
  }
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// dMaxPool (MaxPoolingLayer.cu:9-35): strict '<' so the first maximum wins,
// negative rules skipped.  One lane owns VEC channels of one output row.
template <int VEC>
__global__ void __launch_bounds__(256)
    k_maxpool(const float *__restrict__ in, float *__restrict__ out,
              const int *__restrict__ rules, long long nOutSites, int ps,
              int C, int chunks, int *__restrict__ choice,
              const float *__restrict__ spare) {
  long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= nOutSites * chunks)
    return;
  long long r = idx / chunks;
  int c0 = (int)(idx - r * chunks) * VEC;
  const int *rr = rules + r * ps;
  float best[VEC];
  int arg[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    best[k] = 0.f;
    arg[k] = 0;
  }
  bool none = true;
  // Nine candidates at a time: their rules are requested together, then
  // their values (a skipped rule reads the context's spare row -- never `in`,
  // which may have no rows at all -- and is dropped below), so that a window
  // costs two trips to memory rather than two per candidate; they are
  // compared in rule order.
  constexpr int MP = 9;
  for (int p0 = 0; p0 < ps; p0 += MP) {
    int rule[MP];
#pragma unroll
    for (int u = 0; u < MP; ++u)
      rule[u] = rr[p0 + u < ps ? p0 + u : ps - 1];
    float v[MP][VEC];
#pragma unroll
    for (int u = 0; u < MP; ++u) {
      const float *src = rule[u] >= 0 ? in + (long long)rule[u] * C + c0
                                      : spare + (c0 & (SCN_ZERO_FLOATS - VEC));
      if (VEC == 4) {
        float4 t = *reinterpret_cast<const float4 *>(src);
        v[u][0] = t.x;
        v[u][1] = t.y;
        v[u][2] = t.z;
        v[u][3] = t.w;
      } else {
        v[u][0] = src[0];
      }
    }
#pragma unroll
    for (int u = 0; u < MP; ++u) {
      if (p0 + u >= ps || rule[u] < 0)
        continue;
      // 32-bit, as the reference's poolingChoices (the entry points refuse
      // inputs of 2^31 elements and more where they know the input's size)
      const int flat = (int)((unsigned)rule[u] * (unsigned)C + (unsigned)c0);
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        if (none || best[k] < v[u][k]) {
          best[k] = v[u][k];
          arg[k] = flat + k;
        }
      none = false;
    }
  }
  long long o = r * C + c0;
  if (VEC == 4) {
    *reinterpret_cast<float4 *>(out + o) =
        make_float4(best[0], best[1], best[2], best[3]);
    *reinterpret_cast<int4 *>(choice + o) =
        make_int4(arg[0], arg[1], arg[2], arg[3]);
  } else {
    out[o] = best[0];
    choice[o] = arg[0];
  }
}

extern "C" int scn_maxpool(scn_ctx *ctx, const float *d_in, float *d_out,
                           const int32_t *d_rules, int64_t nOutSites, int ps,
                           int C, int32_t *d_choice) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_maxpool: null context");
  SCN_REQUIRE(nOutSites >= 0 && ps >= 1 && C >= 1, SCN_ERR_ARG,
              "scn_maxpool: nOutSites %lld ps %d C %d", (long long)nOutSites,
              ps, C);
  if (nOutSites == 0)
    return SCN_OK;
  // (d_in may be null: an input without rows, every rule negative)
  SCN_REQUIRE(d_out && d_rules && d_choice, SCN_ERR_ARG,
              "scn_maxpool: null buffer");
  ProfScope prof(ctx, SCN_K_MAXPOOL);
  if (C % 4 == 0 && aligned16(d_in) && aligned16(d_out) && aligned16(d_choice)) {
    long long total = nOutSites * (C / 4);
    hipLaunchKernelGGL(k_maxpool<4>, dim3(scn_ceil_div(total, 256)), dim3(256),
                       0, ctx->stream, d_in, d_out, d_rules,
                       (long long)nOutSites, ps, C, C / 4, d_choice,
                       (const float *)ctx->d_zeros);
  } else {
    long long total = nOutSites * C;
    hipLaunchKernelGGL(k_maxpool<1>, dim3(scn_ceil_div(total, 256)), dim3(256),
                       0, ctx->stream, d_in, d_out, d_rules,
                       (long long)nOutSites, ps, C, C, d_choice,
                       (const float *)ctx->d_zeros);
  }
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

extern "C" int scn_maxpool_checked(scn_ctx *ctx, const float *d_in,
                                   int64_t nInRows, float *d_out,
                                   const int32_t *d_rules, int64_t nOutSites,
                                   int ps, int C, int32_t *d_choice) {
  SCN_REQUIRE(nInRows >= 0 && C >= 1, SCN_ERR_ARG,
              "scn_maxpool_checked: nInRows %lld C %d", (long long)nInRows, C);
  SCN_REQUIRE(nInRows * (int64_t)C <= 2147483647ll, SCN_ERR_CAPACITY,
              "scn_maxpool: %lld input rows of %d features are %lld elements; "
              "the 32-bit pooling choices index at most 2^31 - 1",
              (long long)nInRows, C, (long long)(nInRows * (int64_t)C));
  return scn_maxpool(ctx, d_in, d_out, d_rules, nOutSites, ps, C, d_choice);
}

// dTerminalPool (TerminalPoolingLayer.cu:22-34): sequential fp32 sum in rule
// order, then divide by the number of rows summed.
__global__ void k_terminal_pool(const float *__restrict__ in,
                                float *__restrict__ out,
                                const int *__restrict__ rules, long long count,
                                int S, int C, const float *__restrict__ spare) {
  long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count * C)
    return;
  long long b = idx / C;
  int j = (int)(idx - b * C);
  const int *rr = rules + b * S;
  float t = 0.f;
  int p = 0;
  // four rows at a time: their rules requested together, then their values
  // (a rule past the sample's last reads the context's spare row, never `in`,
  // and ends the sum); added in rule order
  bool more = true;
  for (int p0 = 0; p0 < S && more; p0 += 4) {
    int rule[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      rule[u] = p0 + u < S ? rr[p0 + u] : -1;
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      v[u] = rule[u] >= 0 ? in[(long long)rule[u] * C + j] : spare[j & (SCN_ZERO_FLOATS - 1)];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      more = more && rule[u] >= 0;
      if (more) {
        t += v[u];
        ++p;
      }
    }
  }
  out[idx] = t / (float)p;
}

extern "C" int scn_terminal_pool(scn_ctx *ctx, const float *d_in, float *d_out,
                                 const int32_t *d_rules, int64_t count, int S,
                                 int C) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_terminal_pool: null context");
  SCN_REQUIRE(count >= 0 && S >= 1 && C >= 1, SCN_ERR_ARG,
              "scn_terminal_pool: count %lld S %d C %d", (long long)count, S,
              C);
  if (count == 0)
    return SCN_OK;
  // (d_in may be null: an input without rows, every rule negative)
  SCN_REQUIRE(d_out && d_rules, SCN_ERR_ARG,
              "scn_terminal_pool: null buffer");
  ProfScope prof(ctx, SCN_K_TERMINAL);
  hipLaunchKernelGGL(k_terminal_pool, dim3(scn_ceil_div(count * C, 256)),
                     dim3(256), 0, ctx->stream, d_in, d_out, d_rules,
                     (long long)count, S, C, (const float *)ctx->d_zeros);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// dSigmoidSoftmax (SigmoidLayer.cu:160-177): running maximum starts at -10000.
// One wavefront per row; lanes stride over the classes.
__global__ void __launch_bounds__(256)
    k_softmax(const float *in, float *out, long long M, int N) {
  const int lane = threadIdx.x & 63;
  long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= M)
    return;
  const float *a = in + row * N;
  float *b = out + row * N;
  float mx = -10000.0f;
  for (int k = lane; k < N; k += 64)
    mx = fmaxf(mx, a[k]);
  for (int off = 32; off > 0; off >>= 1)
    mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  float acc = 0.f;
  for (int k = lane; k < N; k += 64) {
    float e = expf(a[k] - mx);
    b[k] = e;
    acc += e;
  }
  for (int off = 32; off > 0; off >>= 1)
    acc += __shfl_xor(acc, off, 64);
  for (int k = lane; k < N; k += 64)
    b[k] = b[k] / acc;
}

// dSigmoidTanh / dSigmoidLogistic (SigmoidLayer.cu:43-48, 80-85): in place,
// four elements per lane where the count allows
__global__ void __launch_bounds__(256)
    k_squash(float *x, long long n, int logistic) {
  const long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i + 4 <= n && ((uintptr_t)x & 15) == 0) {
    float4 v = *reinterpret_cast<float4 *>(x + i);
    if (logistic) {
      v.x = 1.0f / (1.0f + expf(-v.x)), v.y = 1.0f / (1.0f + expf(-v.y));
      v.z = 1.0f / (1.0f + expf(-v.z)), v.w = 1.0f / (1.0f + expf(-v.w));
    } else {
      v.x = tanhf(v.x), v.y = tanhf(v.y), v.z = tanhf(v.z), v.w = tanhf(v.w);
    }
    *reinterpret_cast<float4 *>(x + i) = v;
  } else {
    for (long long k = i; k < n && k < i + 4; ++k)
      x[k] = logistic ? 1.0f / (1.0f + expf(-x[k])) : tanhf(x[k]);
  }
}
int scn_squash_launch(scn_ctx *ctx, float *d_x, long long n, int logistic) {
  if (n <= 0)
    return SCN_OK;
  hipLaunchKernelGGL(k_squash, dim3((unsigned)scn_ceil_div(scn_ceil_div(n, 4), 256)),
                     dim3(256), 0, ctx->stream, d_x, n, logistic);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

int scn_softmax_launch(scn_ctx *ctx, const float *d_in, float *d_out,
                       long long M, int N) {
  hipLaunchKernelGGL(k_softmax, dim3(scn_ceil_div(M, 4)), dim3(256), 0,
                     ctx->stream, d_in, d_out, M, N);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

extern "C" int scn_softmax_rows(scn_ctx *ctx, const float *d_in, float *d_out,
                                int64_t M, int N) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_softmax_rows: null context");
  SCN_REQUIRE(M >= 0 && N >= 1, SCN_ERR_ARG, "scn_softmax_rows: M %lld N %d",
              (long long)M, N);
  if (M == 0)
    return SCN_OK;
  SCN_REQUIRE(d_in && d_out, SCN_ERR_ARG, "scn_softmax_rows: null buffer");
  ProfScope prof(ctx, SCN_K_SOFTMAX);
  return scn_softmax_launch(ctx, d_in, d_out, (long long)M, N);
}
