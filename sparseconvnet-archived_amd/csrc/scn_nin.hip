// NetworkInNetwork forward: out = act(p * (A W + B)), bias and activation
// fused into the contraction's epilogue (the reference runs replicateArray,
// cublasSgemm and applySigmoid / PreLU as three passes over the output).
#include "scn_common.h"
#include <mutex>
#include <type_traits>

// Kernel attributes (the dynamic LDS limit) are set per device: fn runs once for
// every device a context of this process lives on, and again if it failed.
struct OncePerDevice {
  std::mutex m;
  unsigned long long done = 0;
  template <class F> int run(int device, F fn) {
    std::lock_guard<std::mutex> lock(m);
    if (device >= 0 && device < 64 && ((done >> device) & 1ull))
      return SCN_OK;
    const int rc = fn();
    if (rc == SCN_OK && device >= 0 && device < 64)
      done |= 1ull << device;
    return rc;
  }
};

int scn_squash_launch(scn_ctx *ctx, float *d_x, long long n, int logistic);
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

// The same, branch-free, for kernels that keep the column's constants in
// registers: every supported activation is v > 0 ? v : v * slope with slope
// 1 (none), 0 (ReLU), a constant (leaky) or PReLU's learnt per-column value.
struct ColEpilogue {
  float pb;    // p * bias[n]
  float p;
  float slope;
};
__device__ __forceinline__ ColEpilogue load_col(const Epilogue &e, int n) {
  ColEpilogue c;
  c.p = e.p;
  c.pb = e.p * e.bias[n];
  c.slope = e.act == SCN_PRELU
                ? e.prelu[n]
                : (e.act == SCN_RELU ? 0.f
                                     : (e.act == SCN_LEAKYRELU || e.act == SCN_VLEAKYRELU ? e.slope : 1.f));
  return c;
}
__device__ __forceinline__ float finish(float acc, const ColEpilogue &c) {
  const float v = c.p * acc + c.pb;
  const float neg = c.slope == 0.f ? 0.f : v * c.slope;
  return v > 0.f ? v : neg;
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

//
// GATHER: A is never materialised.  Row m of A is the receptive field of
// output site m, column q * nIn + c = channel c of input row
// rules[m * fs + q] (what scn_gather_rows would have written); the block's
// rules are staged in LDS once and the A slabs are fetched through them.
#define GF_MAX_FS 27
struct GatherSource {
  const int *rules;   // [M x fs]
  int fs;             // rule-row width
  int nIn;            // channels of the gathered matrix, nIn % 4 == 0
  unsigned magic;     // floor(2^32 / nIn) + 1: k / nIn == mulhi(k, magic) for k nIn < 2^32
  const float *zeros; // at least nIn zeros: the row a negative rule stands for
};
// k / nIn for the kernels that take any number of channels (the factor does
// not fit 32 bits for a single channel)
__device__ __forceinline__ int gather_rule_of(const GatherSource &gs, int k) {
  return gs.nIn == 1 ? k : (int)__umulhi((unsigned)k, gs.magic);
}


// ---- few rows: split-k FMA kernel --------------------------------------------
// The classifier head and the deepest layers of small batches have a few
// hundred rows: tiles would leave most of the chip idle and run a long k-loop
// in a handful of workgroups.  Here a workgroup owns FR_ROWS rows x 64 columns
// and its eight wavefronts split K between them: a lane owns one column, loads
// its share of that column of W with FR_DEPTH loads in flight (W is small
// and served by the caches) and multiplies it with the rows of A staged in LDS
// (gathered through the rules if asked); the eight partial sums meet in LDS.
#define FR_ROWS 8
#define FR_DEPTH 32
#define FR_WAVES 8
#define FR_THREADS (64 * FR_WAVES)
#define FR_MAX_M 512
#define FR_MAX_K 1024
// NB: columns a lane owns (n, n + 64, ...), i.e. a workgroup covers 64 NB
// columns.  SOFTMAX (the classifier: N <= 64 NB, one workgroup per group of
// rows holds whole rows): the soft-max of a row is taken by the wavefront
// that sums it, with the arithmetic of the kernel that does it as a pass of
// its own (running maximum from -10000, lanes striding over the classes).
template <int NB, bool SOFTMAX>
__global__ void __launch_bounds__(FR_THREADS)
    k_nin_fewrows(const float *__restrict__ A, const float *__restrict__ W,
                  float *__restrict__ out, long long M, int K, int N,
                  Epilogue ep, GatherSource gs, bool gather) {
  __shared__ float sA[FR_ROWS * FR_MAX_K];
  __shared__ float part[FR_WAVES][FR_ROWS][64 * NB];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long long m0 = (long long)blockIdx.x * FR_ROWS;
  const int nBase = blockIdx.y * 64 * NB;
  // this wavefront's share of K, and the first batch of its columns of W on
  // its way before the rows of A are staged
  constexpr int DEPTH = FR_DEPTH / NB;
  const int per = (K + FR_WAVES - 1) / FR_WAVES;
  const int k0 = wave * per < K ? wave * per : K, k1 = min(K, k0 + per);
  const float *w[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int n = nBase + 64 * j + lane;
    w[j] = W + (n < N ? n : 0);
  }
  float wv[NB][DEPTH];
#pragma unroll
  for (int i = 0; i < DEPTH; ++i) {
    const int kk = k0 + i < k1 ? k0 + i : (k1 > 0 ? k1 - 1 : 0); // clamped, the product is dropped below
#pragma unroll
    for (int j = 0; j < NB; ++j)
      wv[j][i] = w[j][(long long)kk * N];
  }
  // the rows of A: all FR_ROWS values of a lane's column requested together
  // (through the rules: the rules together, then the values)
  for (int k = tid; k < K; k += FR_THREADS) {
    float v[FR_ROWS];
    if (gather) {
      const int f = gather_rule_of(gs, k);
      int rule[FR_ROWS];
#pragma unroll
      for (int r = 0; r < FR_ROWS; ++r)
        rule[r] = m0 + r < M ? gs.rules[(m0 + r) * gs.fs + f] : -1;
#pragma unroll
      for (int r = 0; r < FR_ROWS; ++r)
        v[r] = rule[r] >= 0 ? A[(long long)rule[r] * gs.nIn + (k - f * gs.nIn)] : 0.f;
    } else {
#pragma unroll
      for (int r = 0; r < FR_ROWS; ++r)
        v[r] = m0 + r < M ? A[(m0 + r) * K + k] : 0.f;
    }
#pragma unroll
    for (int r = 0; r < FR_ROWS; ++r)
      sA[r * K + k] = v[r];
  }
  __syncthreads();
  float acc[NB][FR_ROWS];
#pragma unroll
  for (int j = 0; j < NB; ++j)
#pragma unroll
    for (int r = 0; r < FR_ROWS; ++r)
      acc[j][r] = 0.f;
  for (int k = k0; k < k1; k += DEPTH) {
    if (k > k0) {
#pragma unroll
      for (int i = 0; i < DEPTH; ++i) {
        const int kk = k + i < k1 ? k + i : k1 - 1;
#pragma unroll
        for (int j = 0; j < NB; ++j)
          wv[j][i] = w[j][(long long)kk * N];
      }
    }
#pragma unroll
    for (int i = 0; i < DEPTH; ++i)
      if (k + i < k1) {
#pragma unroll
        for (int r = 0; r < FR_ROWS; ++r) {
          const float a = sA[r * K + k + i];
#pragma unroll
          for (int j = 0; j < NB; ++j)
            acc[j][r] = fmaf(a, wv[j][i], acc[j][r]);
        }
      }
  }
#pragma unroll
  for (int j = 0; j < NB; ++j)
#pragma unroll
    for (int r = 0; r < FR_ROWS; ++r)
      part[wave][r][64 * j + lane] = acc[j][r];
  __syncthreads();
  // the partial sums are always added in wavefront order
  if (!SOFTMAX) {
    for (int x = tid; x < FR_ROWS * 64 * NB; x += FR_THREADS) {
      const int r = x / (64 * NB), c = x - r * (64 * NB);
      const long long m = m0 + r;
      const int nn = nBase + c;
      if (m < M && nn < N) {
        float v = part[0][r][c];
#pragma unroll
        for (int u = 1; u < FR_WAVES; ++u)
          v += part[u][r][c];
        out[m * N + nn] = apply_act(v, nn, ep);
      }
    }
  } else {
    static_assert(FR_WAVES == FR_ROWS, "one wavefront per row");
    const int r = wave;
    const long long m = m0 + r;
    if (m >= M)
      return;
    float z[NB];
    float mx = -10000.0f;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int c = 64 * j + lane;
      float v = part[0][r][c];
#pragma unroll
      for (int u = 1; u < FR_WAVES; ++u)
        v += part[u][r][c];
      z[j] = 0.f;
      if (c < N) {
        z[j] = apply_act(v, c, ep); // bias and scale; the activation itself is the soft-max below
        mx = fmaxf(mx, z[j]);
      }
    }
    for (int off = 32; off > 0; off >>= 1)
      mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < NB; ++j)
      if (64 * j + lane < N) {
        z[j] = expf(z[j] - mx);
        sum += z[j];
      }
    for (int off = 32; off > 0; off >>= 1)
      sum += __shfl_xor(sum, off, 64);
#pragma unroll
    for (int j = 0; j < NB; ++j)
      if (64 * j + lane < N)
        out[m * N + 64 * j + lane] = z[j] / sum;
  }
}

// ---- few input channels: one lane per four outputs ------------------------
// The first NiN layer of a net multiplies a tall matrix by a tiny W (K = 3 fs
// or so): bandwidth only.  W sits in LDS; a lane reads its row of A (16-byte
// loads, shared by the eight lanes of the row through the cache) and writes
// four adjacent outputs.
#define TK_MAX_K 32
__global__ void __launch_bounds__(256)
    k_nin_thin(const float *__restrict__ A, const float *__restrict__ W,
               float *__restrict__ out, long long M, int K, int N, Epilogue ep) {
  __shared__ __attribute__((aligned(16))) float sW[TK_MAX_K * 32];
  const int tid = threadIdx.x;
  const int n0 = blockIdx.y * 32;
  for (int x = tid; x < K * 32; x += 256) {
    const int k = x >> 5, c = x & 31;
    sW[x] = n0 + c < N ? W[(long long)k * N + n0 + c] : 0.f;
  }
  __syncthreads();
  const long long m = (long long)blockIdx.x * 32 + (tid >> 3);
  const int c4 = (tid & 7) * 4;
  if (m >= M)
    return;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  const float4 *arow = reinterpret_cast<const float4 *>(A + m * K);
  for (int k4 = 0; k4 < K / 4; ++k4) { // K % 4 == 0
    const float4 a = arow[k4];
    const float av[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float4 wv = *reinterpret_cast<const float4 *>(&sW[(4 * k4 + i) * 32 + c4]);
      acc.x = fmaf(av[i], wv.x, acc.x);
      acc.y = fmaf(av[i], wv.y, acc.y);
      acc.z = fmaf(av[i], wv.z, acc.z);
      acc.w = fmaf(av[i], wv.w, acc.w);
    }
  }
  const int n = n0 + c4;
  if (n < N) { // N % 4 == 0: the four columns are in or out together
    float4 r;
    r.x = apply_act(acc.x, n, ep);
    r.y = apply_act(acc.y, n + 1, ep);
    r.z = apply_act(acc.z, n + 2, ep);
    r.w = apply_act(acc.w, n + 3, ep);
    *reinterpret_cast<float4 *>(out + m * N + n) = r;
  }
}

// The same with the row of A read through the rules (the receptive field of
// output site m) -- any number of channels, so a convolution over one to three
// input channels, the first layer of most nets, needs no matrix either.  A
// workgroup gathers its rows into LDS once (eight lanes a row, up to four
// values a lane) and walks all of its columns, CT_COLS at most, in blocks of
// 32; the products of an output are those of the plain kernel on the gathered
// matrix, in the same order.
#define CT_COLS 256
#define CT_GROUPS 2 // groups of 32 rows a workgroup takes: all their loads are in flight together
__global__ void __launch_bounds__(256)
    k_conv_thin(const float *__restrict__ A, const float *__restrict__ W,
                float *__restrict__ out, long long M, int K, int N, Epilogue ep,
                GatherSource gs) {
  // LDS: the gathered rows, then this workgroup's columns of W at pitch wp
  extern __shared__ __attribute__((aligned(16))) float ctLds[];
  float *const sA = ctLds;
  float *const sW = ctLds + CT_GROUPS * 32 * TK_MAX_K;
  const int wp = N < CT_COLS ? N : CT_COLS;
  const int tid = threadIdx.x;
  const int n0 = blockIdx.y * CT_COLS;
  const int cols = N - n0 < CT_COLS ? N - n0 : CT_COLS; // a multiple of 4
  const int r = tid >> 3;
  const long long mFirst = (long long)blockIdx.x * (32 * CT_GROUPS) + r;
  int rule[CT_GROUPS][TK_MAX_K / 8];
#pragma unroll
  for (int g = 0; g < CT_GROUPS; ++g)
#pragma unroll
    for (int j = 0; j < TK_MAX_K / 8; ++j) {
      const int k = (tid & 7) + 8 * j;
      const long long m = mFirst + 32 * g;
      rule[g][j] = k < K && m < M ? gs.rules[m * gs.fs + gather_rule_of(gs, k)] : -1;
    }
  for (int k = tid >> 6; k < K; k += 4) // a wavefront a row of W
    for (int c = 4 * (tid & 63); c < cols; c += 256)
      *reinterpret_cast<float4 *>(&sW[k * wp + c]) =
          *reinterpret_cast<const float4 *>(W + (long long)k * N + n0 + c);
#pragma unroll
  for (int g = 0; g < CT_GROUPS; ++g)
#pragma unroll
    for (int j = 0; j < TK_MAX_K / 8; ++j) {
      const int k = (tid & 7) + 8 * j;
      float v = 0.f;
      if (rule[g][j] >= 0)
        v = A[(long long)rule[g][j] * gs.nIn + (k - gather_rule_of(gs, k) * gs.nIn)];
      sA[(32 * g + r) * TK_MAX_K + k] = v;
    }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < CT_GROUPS; ++g) {
    const long long m = mFirst + 32 * g;
    if (m >= M)
      break;
    const float *arow = sA + (32 * g + r) * TK_MAX_K;
    for (int c4 = (tid & 7) * 4; c4 < cols; c4 += 32) {
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int k = 0; k < K; ++k) {
        const float a = arow[k];
        const float4 wv = *reinterpret_cast<const float4 *>(&sW[k * wp + c4]);
        acc.x = fmaf(a, wv.x, acc.x);
        acc.y = fmaf(a, wv.y, acc.y);
        acc.z = fmaf(a, wv.z, acc.z);
        acc.w = fmaf(a, wv.w, acc.w);
      }
      const int n = n0 + c4;
      float4 o;
      o.x = apply_act(acc.x, n, ep);
      o.y = apply_act(acc.y, n + 1, ep);
      o.z = apply_act(acc.z, n + 2, ep);
      o.w = apply_act(acc.w, n + 3, ep);
      *reinterpret_cast<float4 *>(out + m * N + n) = o;
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

  // Slab loads are unconditional: addresses are clamped into the operands and
  // what lies outside is replaced by zero afterwards, so that the loads sit in
  // one basic block with the MFMAs around them and the compiler can count them.
  float4 ra[A_PER], rw[W_PER];
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  auto load_slab = [&](int k0) {
    const float *src[A_PER];
    bool inside[A_PER];
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      int c = tid + u * 256;
      c = c < A_CHUNKS ? c : A_CHUNKS - 1;
      const int r = c / (BK / 4), kc = c % (BK / 4);
      const long long m = m0 + r;
      const int k = k0 + kc * 4;
      const int kIn = k < K ? k : K - 4; // K % 4 == 0: a chunk is all in or all out
      inside[u] = k < K && m < M;
      if (GATHER) {
        const int q = (int)__umulhi((unsigned)kIn, gs.magic); // kIn / nIn
        const int rule = sR[r * gs.fs + q]; // -1 for rows past M
        src[u] = (rule >= 0 ? A + (long long)rule * gs.nIn : gs.zeros) +
                 (kIn - q * gs.nIn);
      } else {
        src[u] = A + (m < M ? m : M - 1) * K + kIn;
      }
    }
#pragma unroll
    for (int u = 0; u < A_PER; ++u)
      ra[u] = *reinterpret_cast<const float4 *>(src[u]);
#pragma unroll
    for (int u = 0; u < W_PER; ++u) {
      int c = tid + u * 256;
      c = c < W_CHUNKS ? c : W_CHUNKS - 1;
      const int kk = c / (BN / 4), nc = c % (BN / 4);
      const int k = k0 + kk, n = n0 + nc * 4;
      const bool in = k < K && n < N; // N % 4 == 0
      rw[u] = *reinterpret_cast<const float4 *>(
          W + (long long)(k < K ? k : K - 1) * N + (n < N ? n : N - 4));
      if (!in)
        rw[u] = zero4;
    }
#pragma unroll
    for (int u = 0; u < A_PER; ++u)
      if (!inside[u])
        ra[u] = zero4;
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

// ---- MFMA shapes used by the W-resident path --------------------------------
//   ROWS 32: v_mfma_f32_32x32x2_f32, lane = (c = l % 32, q = l / 32)
//   ROWS 16: v_mfma_f32_16x16x4_f32, lane = (c = l % 16, q = l / 16)
// Lane (c, q) supplies A[row c][k-slot q] and W[k-slot q][column c]; accumulator
// register v of that lane is D[row 4 q + v][column c] (16 rows) or
// D[row 8 (v / 4) + 4 q + v % 4][column c] (32 rows).
typedef float floatx4 __attribute__((ext_vector_type(4)));
template <int ROWS> struct DirectAcc;
template <> struct DirectAcc<32> {
  typedef floatx16 type;
  static __device__ __forceinline__ type mfma(float a, float b, type c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};
template <> struct DirectAcc<16> {
  typedef floatx4 type;
  static __device__ __forceinline__ type mfma(float a, float b, type c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
};

// ---- W-resident MFMA path ---------------------------------------------------
// For the many layers whose weight slice fits in LDS (K x NW floats, up to
// 160 KB).  A workgroup of eight wavefronts copies its slice of W into LDS once
// and then every wavefront walks its own row panels (ROWS rows x NW columns):
// A goes from global memory straight into the MFMA register layout (a lane
// fetches 16 contiguous bytes of its row, k = KS t + 4 q + i, and MFMA i of
// the step consumes element i, so k-slot q of that MFMA stands for that k in
// both operands), prefetched SA - 1 k-steps ahead and across panel boundaries,
// W is read from LDS one step ahead.  No barrier is executed after the W copy.
// LDS row pitch NW + 4 keeps the two or four k-rows a wavefront reads at once
// in different banks.
//
// Loads and stores retire in issue order through one counter, and the compiler
// derives every wait from what it can prove is in flight.  So (1) every load in
// the pipeline is unconditional (addresses are clamped instead); (2) a panel's
// first k-steps, which run while the previous panel's stores drain, are a code
// copy of their own, entered only from an epilogue, so that their waits count
// those stores instead of waiting for them; (3) the one ragged panel (M not a
// multiple of ROWS), whose stores are predicated, is handled after the loop.
template <int ROWS, int NT, int SA> struct WresPipe {
  typedef typename DirectAcc<ROWS>::type acc_t;
  static constexpr int KQ = 64 / ROWS;
  static constexpr int KS = 4 * KQ;
  static constexpr int VPT = ROWS * ROWS / 64;
  static constexpr int NW = ROWS * NT;
  static constexpr int PITCH = NW + 4;

  float4 a[SA];
  float b[2][4][NT];
  acc_t acc[NT];

  // Lane (c, q) owns columns NT c .. NT c + NT - 1 of the slice: tile j of the
  // MFMA is the columns {NT c + j}.  Its NT operands of a k are then adjacent
  // in LDS (one wide read) and its NT results of a row adjacent in the output
  // (one wide store).  wl points at sW + 4 q PITCH + NT c.
  __device__ __forceinline__ void read_w(const float *wl, int t, int slot) {
    const float *wk = wl + KS * t * PITCH;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float *p = wk + i * PITCH;
      if (NT % 4 == 0) {
#pragma unroll
        for (int j = 0; j < NT; j += 4) {
          const float4 v = *reinterpret_cast<const float4 *>(p + j);
          b[slot][i][j] = v.x, b[slot][i][j + 1] = v.y;
          b[slot][i][j + 2] = v.z, b[slot][i][j + 3] = v.w;
        }
      } else if (NT % 2 == 0) {
#pragma unroll
        for (int j = 0; j < NT; j += 2) {
          const float2 v = *reinterpret_cast<const float2 *>(p + j);
          b[slot][i][j] = v.x, b[slot][i][j + 1] = v.y;
        }
      } else {
#pragma unroll
        for (int j = 0; j < NT; ++j)
          b[slot][i][j] = p[j];
      }
    }
  }
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int v = 0; v < VPT; ++v)
        acc[j][v] = 0.f;
  }
  // SA k-steps starting at t0 (t0 % SA == 0; SA is even, so the W slot parity
  // survives from group to group).  addr(tt) is where this lane's 16 bytes of
  // k-step tt are; it is called with consecutive tt, and tt >= T means step
  // tt - T of the next panel.
  template <class Addr>
  __device__ __forceinline__ void group(int t0, int T, Addr &addr,
                                        const float *wl) {
#pragma unroll
    for (int s = 0; s < SA; ++s) {
      const int t = t0 + s;
      a[(s + SA - 1) % SA] =
          *reinterpret_cast<const float4 *>(addr(t + SA - 1));
      read_w(wl, t + 1 < T ? t + 1 : 0, (s + 1) & 1);
      const float av[4] = {a[s].x, a[s].y, a[s].z, a[s].w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          acc[j] = DirectAcc<ROWS>::mfma(av[i], b[s & 1][i][j], acc[j]);
      spread();
    }
  }
  // The order of a step's instructions.  A wavefront issues in order, so a
  // load or LDS read that has to wait for its unit holds back the MFMAs behind
  // it, and the eight wavefronts of a workgroup, which walk in step, all ask
  // for those units at once.  With the step's prefetches dealt out among its
  // MFMAs, one after every MFMA_PER of them together with a share of the
  // address arithmetic, such a wait passes while the matrix pipe is still busy
  // with the MFMA before it.  The prefetches stay inside the step.
  static constexpr int MFMA_PER = NT >= 3 ? 2 : 1;
  __device__ __forceinline__ void spread() {
#pragma unroll
    for (int i = 0; i < 4 * NT / MFMA_PER; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, MFMA_PER, 0); // MFMA
      __builtin_amdgcn_sched_group_barrier(0x320, 1, 0); // a load, an LDS read or write
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0); // vector arithmetic
      __builtin_amdgcn_sched_group_barrier(0x004, 2, 0); // scalar arithmetic
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // SA k-steps whose W is the slab at wslab (lane-offset as wl is); b[0] holds
  // its first step's W on entry.  stage() puts the next slab into the other
  // buffer, which nobody reads any more since the barrier before this slab:
  // among the MFMAs of the last step but one when the slab is long enough for
  // its loads to have arrived by then, else with the last step's.  Before the
  // last step's MFMAs every wavefront has read all it needs of this slab:
  // sync() is the barrier, and the first W of the next slab (at wnext) is read
  // under those MFMAs.
  template <class Addr, class Stage, class Sync>
  __device__ __forceinline__ void slab(int t0, Addr &addr, const float *wslab,
                                       const float *wnext, Stage &stage,
                                       Sync &sync) {
#pragma unroll
    for (int s = 0; s < SA; ++s) {
      a[(s + SA - 1) % SA] =
          *reinterpret_cast<const float4 *>(addr(t0 + s + SA - 1));
      if (s + 1 < SA)
        read_w(wslab, s + 1, (s + 1) & 1);
      if (s == (SA >= 4 ? SA - 2 : SA - 1))
        stage();
      if (s + 1 == SA) {
        sync();
        read_w(wnext, 0, 0);
      }
      const float av[4] = {a[s].x, a[s].y, a[s].z, a[s].w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          acc[j] = DirectAcc<ROWS>::mfma(av[i], b[s & 1][i][j], acc[j]);
      spread();
    }
  }
  // orow: row 4 q of the panel, column NT c of the slice
  template <bool GUARDED>
  __device__ __forceinline__ void store(float *orow, int N, long long rowsLeft,
                                        int q, const ColEpilogue (&col)[NT]) {
    static_assert(ROWS == 16, "lane-contiguous columns are laid out for 16-row panels");
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
      if (GUARDED && 4 * q + v >= rowsLeft)
        continue;
      float r[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
        r[j] = finish(acc[j][v], col[j]);
      float *o = orow + (long long)v * N;
      if (NT % 4 == 0) {
#pragma unroll
        for (int j = 0; j < NT; j += 4)
          *reinterpret_cast<float4 *>(o + j) =
              make_float4(r[j], r[j + 1], r[j + 2], r[j + 3]);
      } else if (NT % 2 == 0) {
#pragma unroll
        for (int j = 0; j < NT; j += 2)
          *reinterpret_cast<float2 *>(o + j) = make_float2(r[j], r[j + 1]);
      } else {
#pragma unroll
        for (int j = 0; j < NT; ++j)
          o[j] = r[j];
      }
    }
  }
};

// GRU: 0 = A is a plain matrix; else A is gathered through the rules and GRU
// is the number of 64-int loads that cover one panel's rules (16 fs <= 64 GRU)
template <int ROWS, int NT, int SA, int GRU>
__global__ void __launch_bounds__(512)
    k_nin_wres(const float *__restrict__ A, const float *__restrict__ W,
               float *__restrict__ out, long long M, int K, int N, Epilogue ep,
               GatherSource gs, int nSplits) {
  typedef WresPipe<ROWS, NT, SA> Pipe;
  constexpr bool GATHER = GRU > 0;
  constexpr int KS = Pipe::KS, NW = Pipe::NW, PITCH = Pipe::PITCH;
  extern __shared__ __attribute__((aligned(16))) float sW[]; // [K][PITCH]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane % ROWS, q = lane / ROWS;
  const int split = blockIdx.x % nSplits; // workgroups that share rows are neighbours
  const int wg = blockIdx.x / nSplits;
  const int wgs = gridDim.x / nSplits;
  const int n0 = split * NW;
  const long long nFull = M / ROWS;
  const long long nPanels = (M + ROWS - 1) / ROWS;
  const long long stride = (long long)wgs * 8;
  long long panel = (long long)wg * 8 + wave; // a workgroup takes eight neighbouring panels: they gather common rows
  const int T = K / KS;

  // Where lane (c, q) finds k-steps of a panel.  Plain: a row of A.  GATHER:
  // through this wavefront's copy of the panel's rules in LDS, two buffers
  // (this panel, next panel); the rule for the next call is fetched one call
  // ahead so that its LDS latency is off the path.
  int *const sRw = reinterpret_cast<int *>(sW + (size_t)K * PITCH) +
                   wave * (2 * ROWS * gs.fs);
  const int rulesPerPanel = ROWS * gs.fs;
  auto row_of = [&](long long pnl) {
    long long m = pnl * ROWS + c;
    return m < M ? m : M - 1; // rows past the end: read a valid row, store nothing
  };
  struct {
    const float *cur, *nxt; // plain
    long long wrap;
    int bufCur, bufNext, rule, ch; // gather
  } st;
  auto addr = [&](int tt) -> const float * {
    if (!GATHER)
      return st.cur + KS * tt + (tt >= T ? st.wrap : 0ll);
    const float *p =
        (st.rule >= 0 ? A + (long long)st.rule * gs.nIn : gs.zeros) + st.ch;
    const int tn = tt + 1;
    const int kn = KS * (tn >= T ? tn - T : tn) + 4 * q;
    const int fn = (int)__umulhi((unsigned)kn, gs.magic);
    st.ch = kn - fn * gs.nIn;
    st.rule = sRw[(tn >= T ? st.bufNext : st.bufCur) + c * gs.fs + fn];
    return p;
  };
  // GATHER: the rules of panel pnl, 64 consecutive ints per load
  constexpr int RU = GATHER ? GRU : 1;
  int rr[RU];
  auto fetch_rules = [&](long long pnl) {
    if (pnl >= nPanels)
      pnl = nPanels - 1;
    const long long first = pnl * rulesPerPanel, last = M * gs.fs - 1;
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      long long i = first + lane + 64 * u;
      rr[u] = gs.rules[i < last ? i : last];
    }
  };
  auto keep_rules = [&](int buf) {
#pragma unroll
    for (int u = 0; u < RU; ++u)
      if (lane + 64 * u < rulesPerPanel)
        sRw[buf + lane + 64 * u] = rr[u];
  };

  // this workgroup's columns of W go to LDS in batches of U 16-byte loads per lane
  const int perRow = NW / 4;
  const int chunks = K * perRow;
  constexpr int U = 12;
  float4 w[U];
  int dst[U];
  auto w_load = [&](int base) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // past the end: the last chunk again (same value to the same place)
      int x = base + 512 * u;
      x = x < chunks ? x : chunks - 1;
      const int k = x / perRow, nc = x - k * perRow;
      dst[u] = k * PITCH + 4 * nc;
      w[u] = *reinterpret_cast<const float4 *>(W + (long long)k * N + n0 + 4 * nc);
    }
  };
  auto w_store = [&]() {
    // all of the batch's loads are in flight before the first store (left
    // alone the compiler sinks each load to its store and waits one by one)
#define SCN_PIN4(v) "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)
    asm volatile("" : SCN_PIN4(w[0]), SCN_PIN4(w[1]), SCN_PIN4(w[2]),
                      SCN_PIN4(w[3]), SCN_PIN4(w[4]), SCN_PIN4(w[5]));
    asm volatile("" : SCN_PIN4(w[6]), SCN_PIN4(w[7]), SCN_PIN4(w[8]),
                      SCN_PIN4(w[9]), SCN_PIN4(w[10]), SCN_PIN4(w[11]));
#undef SCN_PIN4
#pragma unroll
    for (int u = 0; u < U; ++u)
      *reinterpret_cast<float4 *>(&sW[dst[u]]) = w[u];
  };

  // Prologue.  Order of issue = order of arrival: what is needed first goes
  // first, and the first batch of W travels while the rules are put in place.
  Pipe pipe;
  if (GATHER) {
    st.bufCur = 0;
    st.bufNext = rulesPerPanel;
    fetch_rules(panel);
    w_load(tid);
    keep_rules(0);
    fetch_rules(panel + stride);
    st.ch = 4 * q - (int)__umulhi((unsigned)(4 * q), gs.magic) * gs.nIn;
    st.rule = sRw[c * gs.fs + (int)__umulhi((unsigned)(4 * q), gs.magic)];
    if (panel + stride >= nPanels)
      st.bufNext = 0; // no next panel: the prefetch past the end re-reads this one
  } else {
    st.cur = A + row_of(panel < nPanels ? panel : 0) * K + 4 * q;
  }
  // with T >= SA the first SA - 1 steps are all inside the first panel
  st.wrap = 0;
#pragma unroll
  for (int s = 0; s < SA - 1; ++s)
    pipe.a[s] = *reinterpret_cast<const float4 *>(addr(s));
  if (!GATHER)
    w_load(tid);
  w_store();
  for (int base = tid + 512 * U; base < chunks; base += 512 * U) {
    w_load(base);
    w_store();
  }
  __syncthreads();

  const float *wl = sW + 4 * q * PITCH + NT * c;
  pipe.read_w(wl, 0, 0);
  ColEpilogue col[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
    col[j] = load_col(ep, n0 + NT * c + j);

  // aim: set up the prefetch that runs past this panel's end into the next
  auto aim = [&]() {
    const long long next = panel + stride;
    if (GATHER) {
      // rr holds the next panel's rules (fetched a panel ago): into the
      // buffer the previous panel has finished with; then fetch the ones after
      if (next < nPanels)
        keep_rules(st.bufNext);
      fetch_rules(next + stride);
    } else {
      // past the last panel the prefetch re-reads this panel's first steps
      st.nxt = next < nPanels ? A + row_of(next) * K + 4 * q : st.cur;
      st.wrap = (st.nxt - st.cur) - (long long)KS * T;
    }
    pipe.clear();
  };
  auto advance = [&]() {
    panel += stride;
    if (GATHER) {
      const int b = st.bufCur;
      st.bufCur = st.bufNext;
      st.bufNext = panel + stride < nPanels ? b : st.bufCur;
    } else {
      st.cur = st.nxt;
    }
  };
  float *const obase = out + (long long)(4 * q) * N + n0 + NT * c;

  if (panel < nFull) { // first panel: entered with only loads in flight
    aim();
    for (int t0 = 0; t0 < T; t0 += SA)
      pipe.group(t0, T, addr, wl);
    pipe.template store<false>(obase + panel * ROWS * N, N, ROWS, q, col);
    advance();
    while (panel < nFull) { // entered with the previous panel's stores in flight
      aim();
      pipe.group(0, T, addr, wl);
      for (int t0 = SA; t0 < T; t0 += SA)
        pipe.group(t0, T, addr, wl);
      pipe.template store<false>(obase + panel * ROWS * N, N, ROWS, q, col);
      advance();
    }
  }
  if (panel < nPanels) { // the ragged last panel
    aim();
    for (int t0 = 0; t0 < T; t0 += SA)
      pipe.group(t0, T, addr, wl);
    pipe.template store<true>(obase + panel * ROWS * N, N, M - panel * ROWS, q, col);
  }
}

// T = K / KS must be a multiple of SA (the prefetch ring wraps at panel ends)
#define WRES_LDS_BYTES (160 * 1024)
// LDS the gathering variant adds: 8 wavefronts x 2 buffers x 16 rows x fs rules
#define WRES_RULE_BYTES(fs) (8 * 2 * 16 * (fs) * 4)
template <int NT, int SA>
static int launch_wres(scn_ctx *ctx, const float *A, const float *W, float *out,
                       long long M, int K, int N, const Epilogue &ep,
                       const GatherSource *gs) {
  constexpr int ROWS = 16, NW = ROWS * NT;
  const int nSplits = N / NW;
  const size_t lds = (size_t)K * (NW + 4) * sizeof(float) +
                     (gs ? WRES_RULE_BYTES(gs->fs) : 0);
  long long wgs = scn_ceil_div(scn_ceil_div(M, ROWS), 8);
  // Two workgroups per compute unit where LDS allows, except when that would
  // leave every wavefront a single panel: then one workgroup per compute unit,
  // whose wavefronts fetch their second panel under the first one's MFMAs
  // (measured on 60478 x 128 x 64: 17.8 us against 19.1).
  long long cap = (long long)ctx->numCU * (lds * 2 <= WRES_LDS_BYTES ? 2 : 1);
  if (wgs <= cap && wgs > ctx->numCU)
    cap = ctx->numCU;
  if (wgs > cap)
    wgs = cap;
  static OncePerDevice configured; // one set of attribute calls per instantiation and device
  const int rc = configured.run(ctx->device, [&]() {
    int rc = SCN_OK;
#define SCN_WRES_LDS(G)                                                        \
  if (hipFuncSetAttribute(                                                     \
          reinterpret_cast<const void *>(k_nin_wres<ROWS, NT, SA, G>),         \
          hipFuncAttributeMaxDynamicSharedMemorySize,                          \
          WRES_LDS_BYTES) != hipSuccess)                                       \
    rc = SCN_ERR_HIP;
    SCN_WRES_LDS(0) SCN_WRES_LDS(1) SCN_WRES_LDS(3) SCN_WRES_LDS(7)
#undef SCN_WRES_LDS
    return rc;
  });
  SCN_REQUIRE(rc == SCN_OK, SCN_ERR_HIP, "hipFuncSetAttribute failed");
  const dim3 grid((unsigned)(wgs * nSplits));
#define SCN_WRES_GO(G, src)                                                    \
  hipLaunchKernelGGL((k_nin_wres<ROWS, NT, SA, G>), grid, dim3(512), lds,      \
                     ctx->stream, A, W, out, M, K, N, ep, src, nSplits)
  if (!gs)
    SCN_WRES_GO(0, GatherSource());
  else if (gs->fs <= 4)
    SCN_WRES_GO(1, *gs);
  else if (gs->fs <= 12)
    SCN_WRES_GO(3, *gs);
  else
    SCN_WRES_GO(7, *gs);
#undef SCN_WRES_GO
  return SCN_OK;
}

// Picks the column width of the W slices and launches; false when the shape is
// not one for this path (the tiled kernel takes it then).  The choice depends
// on M, K, N only, so that a fused convolution and the gather + NiN pair it
// replaces run the same arithmetic in the same order.
static bool wres_forward(scn_ctx *ctx, const float *A, const float *W,
                         float *out, long long M, int K, int N,
                         const Epilogue &ep, const GatherSource *gs) {
  if (K % 32 != 0 || N % 16 != 0)
    return false; // 16 k per step, an even number of steps
  const int sa = (K / 16) % 4 == 0 ? 4 : 2;
  const long long panels = scn_ceil_div(M, 16);
  // widest slice that fits LDS (with room for the rules of the widest filter)
  // and still gives every SIMD a wavefront; else the narrowest
  static const int widths[] = {6, 4, 3, 2, 1};
  int nt = 0;
  for (int w : widths) {
    const int nw = 16 * w;
    if (N % nw != 0 ||
        (size_t)K * (nw + 4) * 4 + WRES_RULE_BYTES(GF_MAX_FS) > WRES_LDS_BYTES)
      continue;
    nt = w;
    if (panels * (N / nw) >= 1024)
      break;
  }
  if (nt == 0)
    return false;
  // every slice re-reads A: fine while that stays in the caches
  const int nSplits = N / (16 * nt);
  if (nSplits > 1 && (double)M * K * 4 * nSplits > 64e6)
    return false;
#define SCN_WRES_CASE(T)                                                       \
  case T:                                                                      \
    return (sa == 4 ? launch_wres<T, 4>(ctx, A, W, out, M, K, N, ep, gs)       \
                    : launch_wres<T, 2>(ctx, A, W, out, M, K, N, ep, gs)) ==   \
           SCN_OK;
  switch (nt) {
    SCN_WRES_CASE(1)
    SCN_WRES_CASE(2)
    SCN_WRES_CASE(3)
    SCN_WRES_CASE(4)
    SCN_WRES_CASE(6)
  }
#undef SCN_WRES_CASE
  return false;
}

// ---- W streamed through LDS, A direct to registers ---------------------------
// For contractions whose slice of W does not fit LDS.  The inner loop is the
// W-resident kernel's (A goes from global memory straight into the MFMA
// operand registers, only W is read from LDS), but W passes through two LDS
// buffers in slabs of SA k-steps.  The eight wavefronts of a workgroup take
// eight consecutive 16-row panels and walk k in step, so one slab serves all
// of them: one barrier per slab, none inside it.  Each thread fetches its part
// of the next slab at the start of a slab and puts it into the other buffer
// towards the end; the slab after a panel's last is the next panel's first, so
// the stream never drains.
//
// ONE (gathered A only): the input has a multiple of the slab's k channels, so
// a slab lies within one filter position and its k-steps are consecutive
// pieces of one input row.  The rule look-up and the 64-bit address then cost
// once per slab, not once per step; the steps and their order are the same.
template <int NT, int SA, int GRU, bool ONE>
__global__ void __launch_bounds__(512, NT <= 4 ? 2 : 1)
    k_nin_wstream(const float *__restrict__ A, const float *__restrict__ W,
                  float *__restrict__ out, long long M, int K, int N,
                  Epilogue ep, GatherSource gs, int nSplits) {
  constexpr int ROWS = 16;
  typedef WresPipe<ROWS, NT, SA> Pipe;
  constexpr bool GATHER = GRU > 0;
  static_assert(GATHER || !ONE, "ONE is a way of gathering");
  constexpr int KS = Pipe::KS, NW = Pipe::NW, PITCH = Pipe::PITCH;
  constexpr int SLAB = KS * SA;            // k per slab
  constexpr int SLAB_FLOATS = SLAB * PITCH;
  extern __shared__ __attribute__((aligned(16))) float sW[]; // [2][SLAB][PITCH]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane % ROWS, q = lane / ROWS;
  const long long nPanels = (M + ROWS - 1) / ROWS;
  const long long nGroups = (nPanels + 7) / 8;    // eight panels, one per wavefront
  const long long nFullGroups = (M / ROWS) / 8;   // ... all of them whole
  const int T = K / KS, nSlabs = T / SA;
  // Workgroups are dealt to the 8 XCDs round-robin and every XCD has an L2 of
  // its own.  A long walk over one column slice (many groups per workgroup)
  // is therefore cut into eight contiguous ranges, one per XCD, so that
  // panels which gather the same input rows -- neighbours in the rule book --
  // meet in one L2; otherwise workgroup w takes groups w, w + wgs, ...
  const int wgs = gridDim.x / nSplits;
  const bool ranges = nSplits == 1 && wgs % 8 == 0 && nGroups >= 2ll * wgs;
  const int split = blockIdx.x % nSplits;
  const int xcd = blockIdx.x % 8;
  const long long perXcd = (nGroups + 7) / 8;
  const int pgStep = ranges ? wgs / 8 : wgs;
  const long long pgEnd =
      ranges && (xcd + 1) * perXcd < nGroups ? (xcd + 1) * perXcd : nGroups;
  const int n0 = split * NW;
  long long pg = ranges ? xcd * perXcd + blockIdx.x / 8 : blockIdx.x / nSplits;
  long long panel = pg * 8 + wave; // may lie past the end

  int *const sRw = reinterpret_cast<int *>(sW + 2 * SLAB_FLOATS) +
                   wave * (2 * ROWS * gs.fs);
  const int rulesPerPanel = ROWS * gs.fs;
  auto row_of = [&](long long pnl) {
    long long m = pnl * ROWS + c;
    return m < M ? m : M - 1; // rows past the end: read a valid row, store nothing
  };
  struct {
    const float *cur, *nxt; // plain
    long long wrap;
    int bufCur, bufNext, rule, ch; // gather
  } st;
  // ONE: p walks the slab in hand; the second request of a slab is the first
  // step of the next slab, which starts at pn.  The rule behind pn's successor
  // is read from LDS a slab before it is turned into an address.
  struct {
    const float *p, *pn;
    int ruleNext, chNext, cnt;
  } one;
  // slab G of this panel (G >= nSlabs: slab G - nSlabs of the next panel):
  // the rule it gathers through and its first channel
  auto slab_rule = [&](int G, int &ch) -> int {
    const bool wrap = G >= nSlabs;
    const int k = SLAB * (wrap ? G - nSlabs : G);
    const int f = (int)__umulhi((unsigned)k, gs.magic);
    ch = k - f * gs.nIn;
    return sRw[(wrap ? st.bufNext : st.bufCur) + c * gs.fs + f];
  };
  auto row_ptr = [&](int rule, int ch) -> const float * {
    return (rule >= 0 ? A + (long long)rule * gs.nIn : gs.zeros) + ch + 4 * q;
  };
  // as in the W-resident kernel: tt >= T means step tt - T of the next panel
  auto addr = [&](int tt) -> const float * {
    if (!GATHER)
      return st.cur + KS * tt + (tt >= T ? st.wrap : 0ll);
    if (ONE) {
      if (one.cnt == 1)
        one.p = one.pn;
      ++one.cnt;
      const float *p = one.p;
      one.p += KS;
      return p;
    }
    const float *p =
        (st.rule >= 0 ? A + (long long)st.rule * gs.nIn : gs.zeros) + st.ch;
    const int tn = tt + 1;
    const int kn = KS * (tn >= T ? tn - T : tn) + 4 * q;
    const int fn = (int)__umulhi((unsigned)kn, gs.magic);
    st.ch = kn - fn * gs.nIn;
    st.rule = sRw[(tn >= T ? st.bufNext : st.bufCur) + c * gs.fs + fn];
    return p;
  };
  constexpr int RU = GATHER ? GRU : 1;
  int rr[RU];
  auto fetch_rules = [&](long long pnl) {
    if (pnl >= nPanels)
      pnl = nPanels - 1;
    const long long first = pnl * rulesPerPanel, last = M * gs.fs - 1;
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      long long i = first + lane + 64 * u;
      rr[u] = gs.rules[i < last ? i : last];
    }
  };
  auto keep_rules = [&](int buf) {
#pragma unroll
    for (int u = 0; u < RU; ++u)
      if (lane + 64 * u < rulesPerPanel)
        sRw[buf + lane + 64 * u] = rr[u];
  };

  // a slab of this workgroup's columns of W: WPER 16-byte pieces per thread,
  // the same pieces of every slab
  constexpr int PER_ROW = NW / 4;
  constexpr int CHUNKS = SLAB * PER_ROW;
  constexpr int WPER = (CHUNKS + 511) / 512;
  float4 w[WPER];
  int dst[WPER];
  const float *src[WPER];
#pragma unroll
  for (int u = 0; u < WPER; ++u) {
    // past the end: the last piece again (same value to the same place)
    int x = tid + 512 * u;
    x = x < CHUNKS ? x : CHUNKS - 1;
    const int k = x / PER_ROW, nc = x - k * PER_ROW;
    dst[u] = k * PITCH + 4 * nc;
    src[u] = W + (long long)k * N + n0 + 4 * nc;
  }
  auto w_load = [&](int slab) {
    const long long off = (long long)slab * SLAB * N;
#pragma unroll
    for (int u = 0; u < WPER; ++u)
      w[u] = *reinterpret_cast<const float4 *>(src[u] + off);
  };
  auto w_store = [&](int buf) {
#pragma unroll
    for (int u = 0; u < WPER; ++u) {
      // the loads stay where they were issued, a slab earlier
      asm volatile("" : "+v"(w[u].x), "+v"(w[u].y), "+v"(w[u].z), "+v"(w[u].w));
      *reinterpret_cast<float4 *>(&sW[buf * SLAB_FLOATS + dst[u]]) = w[u];
    }
  };

  Pipe pipe;
  const bool more = pg + pgStep < pgEnd; // uniform over the workgroup
  if (GATHER) {
    st.bufCur = 0;
    st.bufNext = rulesPerPanel;
    fetch_rules(panel);
    w_load(0);
    keep_rules(0);
    fetch_rules(panel + 8ll * pgStep);
    if (!more)
      st.bufNext = 0; // no next panel: the prefetch past the end re-reads this one
    if (ONE) {
      int ch0;
      const int r0 = slab_rule(0, ch0);
      one.p = row_ptr(r0, ch0);
      one.ruleNext = slab_rule(1, one.chNext);
      one.cnt = 2;
    } else {
      st.ch = 4 * q - (int)__umulhi((unsigned)(4 * q), gs.magic) * gs.nIn;
      st.rule = sRw[c * gs.fs + (int)__umulhi((unsigned)(4 * q), gs.magic)];
    }
  } else {
    st.cur = A + row_of(panel) * K + 4 * q;
  }
  st.wrap = 0;
#pragma unroll
  for (int s = 0; s < SA - 1; ++s)
    pipe.a[s] = *reinterpret_cast<const float4 *>(addr(s));
  if (!GATHER)
    w_load(0);
  w_store(0);
  __syncthreads();
  int cur = 0; // the buffer the next slab is read from
  pipe.read_w(sW + 4 * q * PITCH + NT * c, 0, 0);

  const float *const wl = sW + 4 * q * PITCH + NT * c;
  float *const obase = out + (long long)(4 * q) * N + n0 + NT * c;

  auto run_panel = [&](auto guarded) {
    const long long next = panel + 8ll * pgStep;
    const bool hasNext = pg + pgStep < pgEnd;
    if (GATHER) {
      if (hasNext)
        keep_rules(st.bufNext);
      fetch_rules(next + 8ll * pgStep);
    } else {
      st.nxt = hasNext ? A + row_of(next) * K + 4 * q : st.cur;
      st.wrap = (st.nxt - st.cur) - (long long)KS * T;
    }
    pipe.clear();
    for (int g = 0; g < nSlabs; ++g) {
      w_load(g + 1 < nSlabs ? g + 1 : 0);
      if (ONE) {
        one.pn = row_ptr(one.ruleNext, one.chNext);
        one.ruleNext = slab_rule(g + 2, one.chNext);
        one.cnt = 0;
      }
      auto stage = [&]() { w_store(cur ^ 1); };
      auto sync = [&]() { __syncthreads(); };
      pipe.slab(g * SA, addr, wl + cur * SLAB_FLOATS,
                wl + (cur ^ 1) * SLAB_FLOATS, stage, sync);
      cur ^= 1;
    }
    // (the columns' constants are fetched here, once per panel of K / 16
    // steps, rather than held in registers through the loop)
    ColEpilogue col[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j)
      col[j] = load_col(ep, n0 + NT * c + j);
    pipe.template store<decltype(guarded)::value>(obase + panel * ROWS * N, N,
                                                  M - panel * ROWS, q, col);
    pg += pgStep;
    panel = next;
    if (GATHER) {
      const int b = st.bufCur;
      st.bufCur = st.bufNext;
      st.bufNext = pg + pgStep < pgEnd ? b : st.bufCur;
    } else {
      st.cur = st.nxt;
    }
  };
  while (pg < pgEnd && pg < nFullGroups)
    run_panel(std::false_type());
  if (pg < pgEnd) // the last group: a ragged panel, panels past the end
    run_panel(std::true_type());
}

#define WSTREAM_LDS_BYTES(nw, sa) (2 * 16 * (sa) * ((nw) + 4) * 4)
#define WSTREAM_ROUNDS 32
template <int NT, int SA>
static int launch_wstream(scn_ctx *ctx, const float *A, const float *W,
                          float *out, long long M, int K, int N,
                          const Epilogue &ep, const GatherSource *gs) {
  constexpr int NW = 16 * NT;
  const int nSplits = N / NW;
  const size_t lds =
      WSTREAM_LDS_BYTES(NW, SA) + (gs ? WRES_RULE_BYTES(gs->fs) : 0);
  long long wgs = scn_ceil_div(scn_ceil_div(M, 16), 8);
  // Not one workgroup per slot that walks to the end of the matrix, but up to
  // 32 times as many, each with at least three panel groups.  Alone the kernel
  // takes the same time (a workgroup's start is hidden behind its neighbour on
  // the compute unit, the MFMA pipe is the bound); beside other streams it
  // lets their kernels onto the chip whenever a workgroup retires instead of
  // after the last one (a batch of 6.3 M rows: 17.7 -> 16.6 ms in the
  // pipeline, whose producer otherwise waits out every launch).  The price is
  // in the gathered rows: workgroups that come and go drift apart, the panels
  // that share input rows meet less often in L2, and the kernel reads 8 %
  // more from HBM at three groups a workgroup (50 % more at one).  A multiple
  // of 8 workgroups and two groups each keep the kernel's per-XCD ranges.
  const long long slots = (long long)ctx->numCU * (lds * 2 <= WRES_LDS_BYTES ? 2 : 1);
  if (wgs > slots) {
    long long rounds = wgs / (3 * slots);
    if (rounds > WSTREAM_ROUNDS)
      rounds = WSTREAM_ROUNDS;
    wgs = slots * (rounds > 1 ? rounds : 1);
  }
  static OncePerDevice configured; // one set of attribute calls per instantiation and device
  const int rc = configured.run(ctx->device, [&]() {
    int rc = SCN_OK;
#define SCN_WSTREAM_LDS(G, ONE)                                                \
  if (hipFuncSetAttribute(                                                     \
          reinterpret_cast<const void *>(k_nin_wstream<NT, SA, G, ONE>),       \
          hipFuncAttributeMaxDynamicSharedMemorySize,                          \
          WRES_LDS_BYTES) != hipSuccess)                                       \
    rc = SCN_ERR_HIP;
    SCN_WSTREAM_LDS(0, false)
    SCN_WSTREAM_LDS(1, false) SCN_WSTREAM_LDS(3, false) SCN_WSTREAM_LDS(7, false)
    SCN_WSTREAM_LDS(1, true) SCN_WSTREAM_LDS(3, true) SCN_WSTREAM_LDS(7, true)
#undef SCN_WSTREAM_LDS
    return rc;
  });
  SCN_REQUIRE(rc == SCN_OK, SCN_ERR_HIP, "hipFuncSetAttribute failed");
  const dim3 grid((unsigned)(wgs * nSplits));
#define SCN_WSTREAM_GO(G, ONE, src)                                            \
  hipLaunchKernelGGL((k_nin_wstream<NT, SA, G, ONE>), grid, dim3(512), lds,    \
                     ctx->stream, A, W, out, M, K, N, ep, src, nSplits)
#define SCN_WSTREAM_EITHER(G)                                                  \
  do {                                                                         \
    if (one)                                                                   \
      SCN_WSTREAM_GO(G, true, *gs);                                            \
    else                                                                       \
      SCN_WSTREAM_GO(G, false, *gs);                                           \
  } while (0)
  // a slab within one filter position, and at least two slabs to a panel
  const bool one = gs && gs->nIn % (16 * SA) == 0 && K >= 2 * 16 * SA;
  if (!gs)
    SCN_WSTREAM_GO(0, false, GatherSource());
  else if (gs->fs <= 4)
    SCN_WSTREAM_EITHER(1);
  else if (gs->fs <= 12)
    SCN_WSTREAM_EITHER(3);
  else
    SCN_WSTREAM_EITHER(7);
#undef SCN_WSTREAM_EITHER
#undef SCN_WSTREAM_GO
  return SCN_OK;
}

// As wres_forward: the choice depends on M, K, N only.
static bool wstream_forward(scn_ctx *ctx, const float *A, const float *W,
                            float *out, long long M, int K, int N,
                            const Epilogue &ep, const GatherSource *gs) {
  if (K % 32 != 0 || K < 64 || N % 16 != 0 || M < 1024)
    return false;
  const int sa = K % 64 == 0 ? 4 : 2;
  // widest slice that still fills every compute unit; else the narrowest
  static const int widths[] = {6, 4, 3, 2};
  const long long groups = scn_ceil_div(scn_ceil_div(M, 16), 8);
  int nt = 0;
  for (int w : widths) {
    if (N % (16 * w) != 0)
      continue;
    nt = w;
    if (groups * (N / (16 * w)) >= (long long)ctx->numCU * (w <= 4 ? 2 : 1))
      break; // (the widest runs one workgroup per compute unit)
  }
  if (nt == 0)
    return false;
#define SCN_WSTREAM_CASE(T)                                                    \
  case T:                                                                      \
    return (sa == 4 ? launch_wstream<T, 4>(ctx, A, W, out, M, K, N, ep, gs)    \
                    : launch_wstream<T, 2>(ctx, A, W, out, M, K, N, ep, gs)) == \
           SCN_OK;
  switch (nt) {
    SCN_WSTREAM_CASE(2)
    SCN_WSTREAM_CASE(3)
    SCN_WSTREAM_CASE(4)
    SCN_WSTREAM_CASE(6)
  }
#undef SCN_WSTREAM_CASE
  return false;
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

// ---- W streamed through LDS with bf16 operands --------------------------------
// k_nin_wstream with v_mfma_f32_16x16x32_bf16: one MFMA consumes 32 k, lane
// (c, q) supplies the eight consecutive k = 32 t + 8 q .. + 7 of row c (two
// 16-byte loads of fp32 A, rounded to bf16 in registers: v_cvt_pk_bf16_f32,
// nearest even) and of its columns of W.  W is rounded on its way into LDS and
// kept there as [group of 8 k][tile j][lane c][8 bf16] (column NT c + j), so
// the 16 lanes that read a tile's operands read 256 contiguous bytes.  A slab is 64 k = two steps;
// the A prefetch ring holds RD steps and the loop body is unrolled over BL
// steps (a multiple of both), which K / 32 must be a multiple of.  Accumulation
// and epilogue are fp32 as everywhere.  With GATHER the channels of a rule
// must come in multiples of 8.
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) {
  floatx2 f = {a, b};
  bf16x2 h = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(unsigned, h);
}
__device__ __forceinline__ bf16x8 pack_bf16x8(const float4 &x, const float4 &y) {
  uint4 r;
  r.x = pack_bf16x2(x.x, x.y);
  r.y = pack_bf16x2(x.z, x.w);
  r.z = pack_bf16x2(y.x, y.y);
  r.w = pack_bf16x2(y.z, y.w);
  return __builtin_bit_cast(bf16x8, r);
}

// A16: the rows the rules point at are bf16 already (a copy of the fp32 matrix
// rounded once, nearest even, by k_to_bf16): a lane's eight k of a step are one
// 16-byte load instead of two and need no conversion.  The values that reach
// the MFMA are the same, so the results are too, bit for bit.
template <int NT, int RD, int BL, int GRU, bool A16>
__global__ void __launch_bounds__(512, NT <= 4 ? 2 : 1)
    k_nin_wstream_bf16(const float *__restrict__ A, const float *__restrict__ W,
                       float *__restrict__ out, long long M, int K, int N,
                       Epilogue ep, GatherSource gs, int nSplits) {
  static_assert(BL % 2 == 0 && BL % RD == 0, "body = whole slabs and whole turns of the ring");
  constexpr int ROWS = 16, KS = 32, NW = ROWS * NT;
  constexpr bool GATHER = GRU > 0;
  static_assert(GATHER || !A16, "bf16 rows are read through the rules only");
  constexpr int ES = A16 ? 2 : 4; // bytes of an element of A
  constexpr int GROUP_BYTES = NW * 16 + 16;   // one group of 8 k: NW columns x 8 bf16, padded
  constexpr int SLAB_BYTES = 8 * GROUP_BYTES; // 64 k
  extern __shared__ __attribute__((aligned(16))) unsigned char sWb[]; // [2][SLAB_BYTES], then the rules
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane % ROWS, q = lane / ROWS;
  const long long nPanels = (M + ROWS - 1) / ROWS;
  const long long nGroups = (nPanels + 7) / 8;
  const long long nFullGroups = (M / ROWS) / 8;
  const int T = K / KS, nSlabs = T / 2;
  // the walk over the panel groups: as k_nin_wstream
  const int wgs = gridDim.x / nSplits;
  const bool ranges = nSplits == 1 && wgs % 8 == 0 && nGroups >= 2ll * wgs;
  const int split = blockIdx.x % nSplits;
  const int xcd = blockIdx.x % 8;
  const long long perXcd = (nGroups + 7) / 8;
  const int pgStep = ranges ? wgs / 8 : wgs;
  const long long pgEnd =
      ranges && (xcd + 1) * perXcd < nGroups ? (xcd + 1) * perXcd : nGroups;
  const int n0 = split * NW;
  long long pg = ranges ? xcd * perXcd + blockIdx.x / 8 : blockIdx.x / nSplits;
  long long panel = pg * 8 + wave; // may lie past the end

  int *const sRw = reinterpret_cast<int *>(sWb + 2 * SLAB_BYTES) +
                   wave * (2 * ROWS * gs.fs);
  const int rulesPerPanel = ROWS * gs.fs;
  auto row_of = [&](long long pnl) {
    long long m = pnl * ROWS + c;
    return m < M ? m : M - 1;
  };
  struct {
    const float *cur, *nxt;
    long long wrap;
    int bufCur, bufNext, rule, ch;
  } st;
  // where this lane's 8 elements of step tt are; tt >= T: step tt - T of the next panel
  const unsigned char *const Ab = reinterpret_cast<const unsigned char *>(A);
  const unsigned char *const zb = reinterpret_cast<const unsigned char *>(gs.zeros);
  auto addr = [&](int tt) -> const unsigned char * {
    if (!GATHER)
      return reinterpret_cast<const unsigned char *>(st.cur + KS * tt + (tt >= T ? st.wrap : 0ll));
    const unsigned char *p =
        (st.rule >= 0 ? Ab + (long long)st.rule * gs.nIn * ES : zb) + st.ch * ES;
    const int tn = tt + 1;
    const int kn = KS * (tn >= T ? tn - T : tn) + 8 * q;
    const int fn = (int)__umulhi((unsigned)kn, gs.magic);
    st.ch = kn - fn * gs.nIn;
    st.rule = sRw[(tn >= T ? st.bufNext : st.bufCur) + c * gs.fs + fn];
    return p;
  };
  constexpr int RU = GATHER ? GRU : 1;
  int rr[RU];
  auto fetch_rules = [&](long long pnl) {
    if (pnl >= nPanels)
      pnl = nPanels - 1;
    const long long first = pnl * rulesPerPanel, last = M * gs.fs - 1;
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      long long i = first + lane + 64 * u;
      rr[u] = gs.rules[i < last ? i : last];
    }
  };
  auto keep_rules = [&](int buf) {
#pragma unroll
    for (int u = 0; u < RU; ++u)
      if (lane + 64 * u < rulesPerPanel)
        sRw[buf + lane + 64 * u] = rr[u];
  };

  // a slab of this workgroup's columns of W: one item = 8 consecutive k of one
  // column (8 loads, each coalesced across the lanes of a k-row)
  constexpr int ITEMS = 8 * NW;
  constexpr int WPER = (ITEMS + 511) / 512;
  float wv[WPER][8];
  int dst[WPER];
  const float *src[WPER];
#pragma unroll
  for (int u = 0; u < WPER; ++u) {
    int x = tid + 512 * u;
    x = x < ITEMS ? x : ITEMS - 1; // past the end: the last item again (same value, same place)
    const int kg = x / NW, n = x - kg * NW;
    // column n = NT c + j is item j * 16 + c of its group: the 16 lanes that
    // read tile j of a group read 256 contiguous bytes
    dst[u] = kg * GROUP_BYTES + ((n % NT) * 16 + n / NT) * 16;
    src[u] = W + (long long)(8 * kg) * N + n0 + n;
  }
  auto w_load = [&](int slab) {
    const long long off = (long long)slab * 64 * N;
#pragma unroll
    for (int u = 0; u < WPER; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        wv[u][i] = src[u][off + (long long)i * N];
  };
  auto w_store = [&](int buf) {
#pragma unroll
    for (int u = 0; u < WPER; ++u) {
      asm volatile("" : "+v"(wv[u][0]), "+v"(wv[u][1]), "+v"(wv[u][2]), "+v"(wv[u][3]),
                        "+v"(wv[u][4]), "+v"(wv[u][5]), "+v"(wv[u][6]), "+v"(wv[u][7]));
      uint4 r;
      r.x = pack_bf16x2(wv[u][0], wv[u][1]);
      r.y = pack_bf16x2(wv[u][2], wv[u][3]);
      r.z = pack_bf16x2(wv[u][4], wv[u][5]);
      r.w = pack_bf16x2(wv[u][6], wv[u][7]);
      *reinterpret_cast<uint4 *>(sWb + buf * SLAB_BYTES + dst[u]) = r;
    }
  };

  float4 a[RD][A16 ? 1 : 2]; // (A16: eight bf16 in the one register quad)
  bf16x8 b[2][NT];
  floatx4 acc[NT];
  // this lane's W operands of step s (0, 1) of the slab in buffer buf
  const int bLane = q * GROUP_BYTES + c * 16;
  auto read_b = [&](int buf, int s, int slot) {
    const unsigned char *p = sWb + buf * SLAB_BYTES + 4 * s * GROUP_BYTES + bLane;
#pragma unroll
    for (int j = 0; j < NT; ++j)
      b[slot][j] = *reinterpret_cast<const bf16x8 *>(p + 256 * j);
  };
  auto load_a = [&](int slot, int tt) {
    const unsigned char *p = addr(tt);
    a[slot][0] = *reinterpret_cast<const float4 *>(p);
    if (!A16)
      a[slot][1] = *reinterpret_cast<const float4 *>(p + 16);
  };

  const bool more = pg + pgStep < pgEnd;
  if (GATHER) {
    st.bufCur = 0;
    st.bufNext = rulesPerPanel;
    fetch_rules(panel);
    w_load(0);
    keep_rules(0);
    fetch_rules(panel + 8ll * pgStep);
    st.ch = 8 * q - (int)__umulhi((unsigned)(8 * q), gs.magic) * gs.nIn;
    st.rule = sRw[c * gs.fs + (int)__umulhi((unsigned)(8 * q), gs.magic)];
    if (!more)
      st.bufNext = 0;
  } else {
    st.cur = A + row_of(panel) * K + 8 * q;
  }
  st.wrap = 0;
#pragma unroll
  for (int s = 0; s < RD - 1; ++s)
    load_a(s, s);
  if (!GATHER)
    w_load(0);
  w_store(0);
  __syncthreads();
  int cur = 0;
  read_b(0, 0, 0);

  ColEpilogue col[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
    col[j] = load_col(ep, n0 + NT * c + j);
  float *const obase = out + (long long)(4 * q) * N + n0 + NT * c;

  auto run_panel = [&](auto guarded) {
    const long long next = panel + 8ll * pgStep;
    const bool hasNext = pg + pgStep < pgEnd;
    if (GATHER) {
      if (hasNext)
        keep_rules(st.bufNext);
      fetch_rules(next + 8ll * pgStep);
    } else {
      st.nxt = hasNext ? A + row_of(next) * K + 8 * q : st.cur;
      st.wrap = (st.nxt - st.cur) - (long long)KS * T;
    }
#pragma unroll
    for (int j = 0; j < NT; ++j)
      acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int t0 = 0; t0 < T; t0 += BL) {
#pragma unroll
      for (int s = 0; s < BL; ++s) {
        const int t = t0 + s;
        if ((s & 1) == 0) { // first step of a slab: fetch the next slab, read this slab's second step
          const int slabNext = t / 2 + 1;
          w_load(slabNext < nSlabs ? slabNext : 0);
          load_a((s + RD - 1) % RD, t + RD - 1);
          read_b(cur, 1, 1);
        } else { // second step: hand the next slab over, read its first step
          load_a((s + RD - 1) % RD, t + RD - 1);
          w_store(cur ^ 1);
          __syncthreads();
          cur ^= 1;
          read_b(cur, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        const bf16x8 av = A16 ? __builtin_bit_cast(bf16x8, a[s % RD][0])
                              : pack_bf16x8(a[s % RD][0], a[s % RD][A16 ? 0 : 1]);
#pragma unroll
        for (int j = 0; j < NT; ++j)
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, b[s & 1][j], acc[j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // lane (c, q): rows 4 q + v, columns NT c + j
    float *orow = obase + panel * ROWS * N;
    const long long rowsLeft = M - panel * ROWS;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if (decltype(guarded)::value && 4 * q + v >= rowsLeft)
        continue;
      float r[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
        r[j] = finish(acc[j][v], col[j]);
      float *o = orow + (long long)v * N;
      if (NT % 4 == 0) {
#pragma unroll
        for (int j = 0; j < NT; j += 4)
          *reinterpret_cast<float4 *>(o + j) = make_float4(r[j], r[j + 1], r[j + 2], r[j + 3]);
      } else if (NT % 2 == 0) {
#pragma unroll
        for (int j = 0; j < NT; j += 2)
          *reinterpret_cast<float2 *>(o + j) = make_float2(r[j], r[j + 1]);
      } else {
#pragma unroll
        for (int j = 0; j < NT; ++j)
          o[j] = r[j];
      }
    }
    pg += pgStep;
    panel = next;
    if (GATHER) {
      const int bb = st.bufCur;
      st.bufCur = st.bufNext;
      st.bufNext = pg + pgStep < pgEnd ? bb : st.bufCur;
    } else {
      st.cur = st.nxt;
    }
  };
  while (pg < pgEnd && pg < nFullGroups)
    run_panel(std::false_type());
  if (pg < pgEnd)
    run_panel(std::true_type());
}

#define WSTREAM_BF16_LDS_BYTES(nw) (2 * 8 * ((nw) * 16 + 16))
template <int NT, int RD, int BL>
static int launch_wstream_bf16(scn_ctx *ctx, const float *A, const float *W,
                               float *out, long long M, int K, int N,
                               const Epilogue &ep, const GatherSource *gs,
                               bool a16 = false) {
  constexpr int NW = 16 * NT;
  const int nSplits = N / NW;
  const size_t lds =
      WSTREAM_BF16_LDS_BYTES(NW) + (gs ? WRES_RULE_BYTES(gs->fs) : 0);
  long long wgs = scn_ceil_div(scn_ceil_div(M, 16), 8);
  // (one workgroup per slot: this kernel is bound by the rows it gathers, a
  // workgroup's start is not hidden, and more of them cost 9 us each a slot)
  const long long cap = (long long)ctx->numCU * (lds * 2 <= WRES_LDS_BYTES ? 2 : 1);
  if (wgs > cap)
    wgs = cap;
  static OncePerDevice configured; // one set of attribute calls per instantiation and device
  const int rc = configured.run(ctx->device, [&]() {
    int rc = SCN_OK;
#define SCN_WSB_LDS(G, H)                                                      \
  if (hipFuncSetAttribute(                                                     \
          reinterpret_cast<const void *>(k_nin_wstream_bf16<NT, RD, BL, G, H>), \
          hipFuncAttributeMaxDynamicSharedMemorySize,                          \
          WRES_LDS_BYTES) != hipSuccess)                                       \
    rc = SCN_ERR_HIP;
    SCN_WSB_LDS(0, false) SCN_WSB_LDS(1, false) SCN_WSB_LDS(3, false) SCN_WSB_LDS(7, false)
    SCN_WSB_LDS(1, true) SCN_WSB_LDS(3, true) SCN_WSB_LDS(7, true)
#undef SCN_WSB_LDS
    return rc;
  });
  SCN_REQUIRE(rc == SCN_OK, SCN_ERR_HIP, "hipFuncSetAttribute failed");
  const dim3 grid((unsigned)(wgs * nSplits));
#define SCN_WSB_GO(G, H, src)                                                  \
  hipLaunchKernelGGL((k_nin_wstream_bf16<NT, RD, BL, G, H>), grid, dim3(512),  \
                     lds, ctx->stream, A, W, out, M, K, N, ep, src, nSplits)
  if (!gs)
    SCN_WSB_GO(0, false, GatherSource());
  else if (a16 && gs->fs <= 4)
    SCN_WSB_GO(1, true, *gs);
  else if (a16 && gs->fs <= 12)
    SCN_WSB_GO(3, true, *gs);
  else if (a16)
    SCN_WSB_GO(7, true, *gs);
  else if (gs->fs <= 4)
    SCN_WSB_GO(1, false, *gs);
  else if (gs->fs <= 12)
    SCN_WSB_GO(3, false, *gs);
  else
    SCN_WSB_GO(7, false, *gs);
#undef SCN_WSB_GO
  return SCN_OK;
}

// bf16 operands, shapes this kernel takes: K a multiple of 64, N of 32, any
// number of rows (a fused convolution has no other bf16 kernel to fall back
// on, and the short last batch of a dataset has few rows); with a gather,
// channels in multiples of 8.  The choice depends on (K, N) only.
static bool wstream_bf16_shape(long long M, int K, int N) {
  return K % 64 == 0 && N % 32 == 0 && M >= 1;
}
static bool wstream_bf16_forward(scn_ctx *ctx, const float *A, const float *W,
                                 float *out, long long M, int K, int N,
                                 const Epilogue &ep, const GatherSource *gs,
                                 bool a16 = false) {
  if (!wstream_bf16_shape(M, K, N) || (gs && gs->nIn % 8 != 0) || (a16 && !gs))
    return false;
  const int T = K / 32;
  static const int widths[] = {6, 4, 2};
  const long long groups = scn_ceil_div(scn_ceil_div(M, 16), 8);
  int nt = 0;
  for (int w : widths) {
    if (N % (16 * w) != 0)
      continue;
    nt = w;
    if (groups * (N / (16 * w)) >= (long long)ctx->numCU * (w <= 4 ? 2 : 1))
      break;
  }
  if (nt == 0)
    return false;
#define SCN_WSB_CASE(NTV)                                                      \
  case NTV:                                                                    \
    if (T % 4 == 0)                                                            \
      return launch_wstream_bf16<NTV, 4, 4>(ctx, A, W, out, M, K, N, ep, gs, a16) == SCN_OK; \
    if (T % 6 == 0)                                                            \
      return launch_wstream_bf16<NTV, 3, 6>(ctx, A, W, out, M, K, N, ep, gs, a16) == SCN_OK; \
    return launch_wstream_bf16<NTV, 2, 2>(ctx, A, W, out, M, K, N, ep, gs, a16) == SCN_OK;
  switch (nt) {
    SCN_WSB_CASE(2)
    SCN_WSB_CASE(4)
    SCN_WSB_CASE(6)
  }
#undef SCN_WSB_CASE
  return false;
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

// rows16: a bf16 copy of the matrix the rules point into, or null
static int nin_forward(scn_ctx *ctx, const float *d_A, const float *d_W,
                       const float *d_B, const float *d_prelu, float *d_out,
                       int64_t M, int K, int N, float p, int act, int precision,
                       const GatherSource *gs, const void *rows16 = nullptr) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_nin_forward: null context");
  SCN_REQUIRE(M >= 0 && K >= 1 && N >= 1, SCN_ERR_ARG,
              "scn_nin_forward: M %lld K %d N %d", (long long)M, K, N);
  SCN_REQUIRE(act >= SCN_NOSIGMOID && act <= SCN_SIGMOID, SCN_ERR_ARG,
              "scn_nin_forward: activation %d", act);
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
  bool softmaxDone = false;
  const bool vec = K % 4 == 0 && N % 4 == 0 && ((uintptr_t)d_A & 15) == 0 &&
                   ((uintptr_t)d_W & 15) == 0 && ((uintptr_t)d_out & 15) == 0;
  // bf16 operands only where the contraction is big enough to matter; the
  // classifier head and the thin first layers stay fp32
  if (vec && K >= 64 && act != SCN_SOFTMAX && precision == SCN_BF16 && rows16 && gs &&
      ((uintptr_t)rows16 & 15) == 0 &&
      wstream_bf16_forward(ctx, reinterpret_cast<const float *>(rows16), d_W, d_out, M, K, N, ep, gs, true)) {
    // the same kernel reading rows that are bf16 already
  } else if (vec && K >= 64 && act != SCN_SOFTMAX && precision == SCN_BF16 &&
             wstream_bf16_forward(ctx, d_A, d_W, d_out, M, K, N, ep, gs)) {
    // W-streaming kernel with bf16 operands took it
  } else if (vec && K >= 64 && act != SCN_SOFTMAX && precision != SCN_FP32) {
    SCN_REQUIRE(!gs, SCN_ERR_ARG,
                "fused convolution: shape outside the bf16 kernel's range");
    const bool split = precision == SCN_BF16X3;
    long long blocksLarge = (long long)scn_ceil_div(M, 128) * scn_ceil_div(N, 64);
    if (N <= 32)
      launch_mfma_bf16<4, 1, 1>(ctx, d_A, d_W, d_out, M, K, N, ep, split);
    else if (blocksLarge >= ctx->numCU)
      launch_mfma_bf16<4, 1, 2>(ctx, d_A, d_W, d_out, M, K, N, ep, split);
    else
      launch_mfma_bf16<1, 4, 1>(ctx, d_A, d_W, d_out, M, K, N, ep, split);
  } else if (M <= FR_MAX_M && K <= FR_MAX_K && !(vec && K % 32 == 0 && N % 16 == 0)) {
    // (shapes the W-resident kernel takes are faster there)
    GatherSource none = GatherSource();
    if (act == SCN_SOFTMAX && N <= 128) {
      // whole rows in one workgroup: the soft-max rides along
      softmaxDone = true;
      hipLaunchKernelGGL((k_nin_fewrows<2, true>), dim3(scn_ceil_div(M, FR_ROWS), 1),
                         dim3(FR_THREADS), 0, ctx->stream, d_A, d_W, d_out,
                         (long long)M, K, N, ep, gs ? *gs : none, gs != nullptr);
    } else {
      hipLaunchKernelGGL((k_nin_fewrows<1, false>),
                         dim3(scn_ceil_div(M, FR_ROWS), scn_ceil_div(N, 64)),
                         dim3(FR_THREADS), 0, ctx->stream, d_A, d_W, d_out,
                         (long long)M, K, N, ep, gs ? *gs : none, gs != nullptr);
    }
  } else if (vec && gs && gs->nIn % 4 != 0) {
    // channels in other than fours: K <= TK_MAX_K (scn_conv_nin_supported)
    const size_t lds = (size_t)(CT_GROUPS * 32 * TK_MAX_K + K * (N < CT_COLS ? N : CT_COLS)) * sizeof(float);
    hipLaunchKernelGGL(k_conv_thin, dim3(scn_ceil_div(M, 32 * CT_GROUPS), scn_ceil_div(N, CT_COLS)),
                       dim3(256), lds, ctx->stream, d_A, d_W, d_out, (long long)M,
                       K, N, ep, *gs);
  } else if (vec && !gs && K <= TK_MAX_K) {
    hipLaunchKernelGGL(k_nin_thin, dim3(scn_ceil_div(M, 32), scn_ceil_div(N, 32)),
                       dim3(256), 0, ctx->stream, d_A, d_W, d_out, (long long)M,
                       K, N, ep);
  } else if (vec && wres_forward(ctx, d_A, d_W, d_out, M, K, N, ep, gs)) {
    // W-resident kernel took it
  } else if (vec && ctx->wstream &&
             wstream_forward(ctx, d_A, d_W, d_out, M, K, N, ep, gs)) {
    // W-streaming kernel took it
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
  // softmax, tanh and the logistic function are a pass of their own over the
  // layer's output, as in the reference (the kernels above treat them as
  // "no activation")
  if (act == SCN_SOFTMAX && !softmaxDone)
    SCN_TRY(scn_softmax_launch(ctx, d_out, d_out, (long long)M, N));
  if (act == SCN_TANH || act == SCN_SIGMOID)
    SCN_TRY(scn_squash_launch(ctx, d_out, (long long)M * N, act == SCN_SIGMOID));
  return SCN_OK;
}

extern "C" int scn_nin_forward(scn_ctx *ctx, const float *d_A,
                               const float *d_W, const float *d_B,
                               const float *d_prelu, float *d_out, int64_t M,
                               int K, int N, float p, int act, int precision) {
  return nin_forward(ctx, d_A, d_W, d_B, d_prelu, d_out, M, K, N, p, act,
                     precision, nullptr);
}

// few channels (any number of them) times a small window: the thin kernel
static bool conv_thin_shape(int fs, int nIn, int N) {
  return fs >= 1 && fs <= GF_MAX_FS && nIn >= 1 && nIn % 4 != 0 &&
         fs * nIn <= TK_MAX_K && (fs * nIn) % 4 == 0 && N % 4 == 0;
}
extern "C" int scn_conv_nin_supported(int fs, int nIn, int N) {
  return (fs >= 1 && fs <= GF_MAX_FS && nIn >= 4 && nIn % 4 == 0 &&
          nIn <= SCN_ZERO_FLOATS && N % 4 == 0) ||
         conv_thin_shape(fs, nIn, N);
}
extern "C" int scn_conv_nin_supported_p(int fs, int nIn, int N, int precision) {
  if (!scn_conv_nin_supported(fs, nIn, N))
    return 0;
  // (contractions this short stay fp32 in every mode)
  if (precision == SCN_FP32 || conv_thin_shape(fs, nIn, N))
    return 1;
  // bf16 operands: the shapes of the bf16 W-streaming kernel, whatever M
  return precision == SCN_BF16 && nIn % 8 == 0 &&
         wstream_bf16_shape(1 << 20, fs * nIn, N);
}

// d_out16[i] = bf16(d_in[i]), nearest even (v_cvt_pk_bf16_f32), eight a lane
__global__ void __launch_bounds__(256)
    k_to_bf16(const float4 *__restrict__ in, uint4 *__restrict__ out, long long n8) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n8)
    return;
  const float4 x = in[2 * i], y = in[2 * i + 1];
  uint4 r;
  r.x = pack_bf16x2(x.x, x.y);
  r.y = pack_bf16x2(x.z, x.w);
  r.z = pack_bf16x2(y.x, y.y);
  r.w = pack_bf16x2(y.z, y.w);
  out[i] = r;
}

extern "C" int scn_conv_nin_forward_a16(scn_ctx *ctx, const float *d_in, int64_t nInRows,
                                        void *d_in16, const int32_t *d_rules, int fs,
                                        int nIn, const float *d_W, const float *d_B,
                                        const float *d_prelu, float *d_out, int64_t M,
                                        int N, float p, int act) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_conv_nin_forward_a16: null context");
  SCN_REQUIRE(scn_conv_nin_supported_p(fs, nIn, N, SCN_BF16), SCN_ERR_ARG,
              "scn_conv_nin_forward_a16: fs %d nIn %d N %d is outside the bf16 fused kernel's range", fs,
              nIn, N);
  SCN_REQUIRE(nInRows >= 0 && (d_in16 || nInRows == 0), SCN_ERR_ARG,
              "scn_conv_nin_forward_a16: %lld input rows, no room for their bf16 copy", (long long)nInRows);
  SCN_REQUIRE(d_rules || M == 0, SCN_ERR_ARG, "scn_conv_nin_forward_a16: null rules");
  SCN_REQUIRE(((uintptr_t)d_in & 15) == 0 && ((uintptr_t)d_W & 15) == 0 && ((uintptr_t)d_in16 & 15) == 0,
              SCN_ERR_ARG, "scn_conv_nin_forward_a16: buffers must be 16-byte aligned");
  if (M == 0)
    return SCN_OK;
  const bool copy = nIn % 8 == 0 && nInRows > 0 && d_in;
  if (copy) {
    ProfScope prof(ctx, SCN_K_GATHER);
    const long long n8 = (long long)nInRows * nIn / 8;
    hipLaunchKernelGGL(k_to_bf16, dim3(scn_ceil_div(n8, 256)), dim3(256), 0, ctx->stream,
                       reinterpret_cast<const float4 *>(d_in), reinterpret_cast<uint4 *>(d_in16), n8);
    SCN_HIP_CHECK(hipGetLastError());
  }
  GatherSource gs = GatherSource();
  gs.rules = d_rules;
  gs.fs = fs;
  gs.nIn = nIn;
  gs.magic = (unsigned)((1ull << 32) / (unsigned)nIn + 1);
  gs.zeros = ctx->d_zeros;
  return nin_forward(ctx, d_in, d_W, d_B, d_prelu, d_out, M, fs * nIn, N, p, act, SCN_BF16, &gs,
                     copy ? d_in16 : nullptr);
}

extern "C" int scn_conv_nin_forward(scn_ctx *ctx, const float *d_in,
                                    const int32_t *d_rules, int fs, int nIn,
                                    const float *d_W, const float *d_B,
                                    const float *d_prelu, float *d_out,
                                    int64_t M, int N, float p, int act) {
  return scn_conv_nin_forward_p(ctx, d_in, d_rules, fs, nIn, d_W, d_B, d_prelu,
                                d_out, M, N, p, act, SCN_FP32);
}
extern "C" int scn_conv_nin_forward_p(scn_ctx *ctx, const float *d_in,
                                      const int32_t *d_rules, int fs, int nIn,
                                      const float *d_W, const float *d_B,
                                      const float *d_prelu, float *d_out,
                                      int64_t M, int N, float p, int act,
                                      int precision) {
  SCN_REQUIRE(ctx, SCN_ERR_ARG, "scn_conv_nin_forward: null context");
  SCN_REQUIRE(scn_conv_nin_supported_p(fs, nIn, N, precision), SCN_ERR_ARG,
              "scn_conv_nin_forward: fs %d nIn %d N %d precision %d is outside "
              "the fused kernels' range (fs <= %d, nIn and N multiples of 4, or fs nIn <= 32 and a multiple of 4; "
              "bf16: nIn of 8, fs nIn of 64, N of 32)",
              fs, nIn, N, precision, GF_MAX_FS);
  SCN_REQUIRE(d_rules || M == 0, SCN_ERR_ARG,
              "scn_conv_nin_forward: null rules");
  SCN_REQUIRE(((uintptr_t)d_in & 15) == 0 && ((uintptr_t)d_W & 15) == 0,
              SCN_ERR_ARG, "scn_conv_nin_forward: buffers must be 16-byte aligned");
  GatherSource gs;
  gs.rules = d_rules;
  gs.fs = fs;
  gs.nIn = nIn;
  gs.magic = (unsigned)((1ull << 32) / (unsigned)nIn + 1);
  gs.zeros = ctx->d_zeros;
  return nin_forward(ctx, d_in, d_W, d_B, d_prelu, d_out, M, fs * nIn, N, p,
                     act, precision, &gs);
}
