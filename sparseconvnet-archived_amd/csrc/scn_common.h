// Internal declarations shared by the translation units of libscn_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <vector>
#include "scn_hip.h"

void scn_set_error(const char *fmt, ...);

#define SCN_HIP_CHECK(expr)                                                    \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess) {                                                    \
      scn_set_error("%s:%d: %s failed: %s", __FILE__, __LINE__, #expr,         \
                    hipGetErrorString(e_));                                    \
      return SCN_ERR_HIP;                                                      \
    }                                                                          \
  } while (0)

#define SCN_REQUIRE(cond, code, ...)                                           \
  do {                                                                         \
    if (!(cond)) {                                                             \
      scn_set_error(__VA_ARGS__);                                              \
      return (code);                                                           \
    }                                                                          \
  } while (0)

#define SCN_TRY(expr)                                                          \
  do {                                                                         \
    int rc_ = (expr);                                                          \
    if (rc_ != SCN_OK)                                                         \
      return rc_;                                                              \
  } while (0)

struct ProfSpan {
  int family;
  int tag;
  hipEvent_t a, b;
};

#define SCN_ZERO_FLOATS 4096
#define SCN_MAX_PENDING 62 // plans per settle; 16 + 4 * 62 = 264 pinned words
#define SCN_PINNED_WORDS (16 + 4 * SCN_MAX_PENDING)
struct scn_ctx {
  int device;
  hipStream_t stream;
  int numCU;
  // small pinned buffer for counts that must come back to the host
  int64_t *h_pinned; // SCN_PINNED_WORDS int64, host view
  int64_t *d_pinned; // the same memory as the device sees it
  int64_t *d_scalars; // 16 int64
  float *d_zeros;     // SCN_ZERO_FLOATS zeros: the row a negative rule stands for
  long long ticket;   // number of the last count readback (h_pinned[14] echoes it)
  // deferred counts (scn_ctx_defer_counts): plans whose counts are still on
  // their way; slot i of them reports into h_pinned[16 + 4 i ..]
  bool deferCounts;
  bool wstream; // NiN: W-streaming kernel allowed (SCN_NIN_WSTREAM=0 turns it off)
  std::vector<struct scn_grids *> pendingGrids;
  struct ChainState *chain; // recorded rule-book plans (scn_chain.hip)
  // profiling
  bool prof;
  int profTag;
  std::vector<ProfSpan> spans;
  std::vector<hipEvent_t> freeEvents;
  double profMs[SCN_K_COUNT];
  int64_t profCalls[SCN_K_COUNT];
};

// Records a start event on construction and a stop event on destruction when
// profiling is enabled.
struct ProfScope {
  scn_ctx *ctx;
  int idx;
  ProfScope(scn_ctx *ctx, int family);
  ~ProfScope();
};

// grow-only device buffer
template <typename T> struct DevBuf {
  T *p = nullptr;
  size_t cap = 0; // elements
  int reserve(size_t n) {
    if (n <= cap)
      return SCN_OK;
    size_t want = n + n / 4 + 64;
    T *q = nullptr;
    hipError_t e = hipMalloc((void **)&q, want * sizeof(T));
    if (e != hipSuccess) {
      scn_set_error("hipMalloc(%zu bytes) failed: %s", want * sizeof(T),
                    hipGetErrorString(e));
      return SCN_ERR_HIP;
    }
    if (p)
      (void)hipFree(p);
    p = q;
    cap = want;
    return SCN_OK;
  }
  void release() {
    if (p)
      (void)hipFree(p);
    p = nullptr;
    cap = 0;
  }
};

static inline int scn_ceil_div(int64_t a, int64_t b) {
  return (int)((a + b - 1) / b);
}

// address of the static scratch of scn_sgemm_ABt_static on `device` (scn_train.hip)
int scn_abt_static_setup(int device);
void scn_abt_static_forget(const scn_ctx *ctx);

// runs the recorded rule-book plans of the context, if any (scn_chain.hip)
int scn_chain_flush(scn_ctx *ctx);
void scn_chain_release(scn_ctx *ctx);

// exclusive prefix sum of n uint32 values; out has n + 1 elements (out[n] =
// total).  `tmp` must hold scn_scan_tmp_elems(n) uint32.
size_t scn_scan_tmp_elems(size_t n);
int scn_scan_exclusive_u32(hipStream_t s, const uint32_t *in, uint32_t *out,
                           size_t n, uint32_t *tmp);
// same, over popcounts of 64-bit words
int scn_scan_exclusive_popc64(hipStream_t s, const uint64_t *words,
                              uint32_t *out, size_t n, uint32_t *tmp);
