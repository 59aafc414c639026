// Context, error reporting, raw device memory and per-kernel timing.
#include "scn_common.h"
#include <stdlib.h>
#include <stdarg.h>
#include <string.h>

static thread_local char g_err[512] = "";

void scn_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char *scn_last_error(void) { return g_err; }
extern "C" const char *scn_version(void) { return "scn_hip 0.1 (gfx950)"; }

extern "C" int scn_ctx_create(int device, scn_ctx **out) {
  SCN_REQUIRE(out != nullptr, SCN_ERR_ARG, "scn_ctx_create: null out pointer");
  int n = 0;
  SCN_HIP_CHECK(hipGetDeviceCount(&n));
  if (device < 0)
    device = 0;
  SCN_REQUIRE(device < n, SCN_ERR_ARG, "scn_ctx_create: device %d of %d",
              device, n);
  SCN_HIP_CHECK(hipSetDevice(device));
  SCN_TRY(scn_abt_static_setup(device));
  scn_ctx *c = new scn_ctx();
  c->device = device;
  c->prof = false;
  c->profTag = 0;
  c->ticket = 0;
  c->deferCounts = false;
  c->chain = nullptr;
  {
    const char *e = getenv("SCN_NIN_WSTREAM");
    c->wstream = !(e && e[0] == '0');
  }
  memset(c->profMs, 0, sizeof(c->profMs));
  memset(c->profCalls, 0, sizeof(c->profCalls));
  hipDeviceProp_t prop;
  SCN_HIP_CHECK(hipGetDeviceProperties(&prop, device));
  c->numCU = prop.multiProcessorCount;
  // default priority, and BLOCKING (hipStreamCreate, not hipStreamNonBlocking):
  // a copy made with no context goes through the legacy stream and must wait
  // for this one -- scn_h2d / scn_d2h with a null context count on that
  SCN_HIP_CHECK(hipStreamCreate(&c->stream));
  SCN_HIP_CHECK(hipHostMalloc((void **)&c->h_pinned, SCN_PINNED_WORDS * sizeof(int64_t),
                              hipHostMallocMapped));
  memset(c->h_pinned, 0, SCN_PINNED_WORDS * sizeof(int64_t));
  SCN_HIP_CHECK(hipHostGetDevicePointer((void **)&c->d_pinned, c->h_pinned, 0));
  SCN_HIP_CHECK(hipMalloc((void **)&c->d_scalars, 16 * sizeof(int64_t)));
  SCN_HIP_CHECK(hipMemset(c->d_scalars, 0, 16 * sizeof(int64_t)));
  SCN_HIP_CHECK(hipMalloc((void **)&c->d_zeros, SCN_ZERO_FLOATS * sizeof(float)));
  // (on the context's own stream: HIP gives a stream its hardware queue with
  // the first work it gets, which takes about a millisecond -- here rather
  // than in front of the first batch that happens to use the stream)
  SCN_HIP_CHECK(hipMemsetAsync(c->d_zeros, 0, SCN_ZERO_FLOATS * sizeof(float), c->stream));
  SCN_HIP_CHECK(hipStreamSynchronize(c->stream));
  *out = c;
  return SCN_OK;
}

extern "C" int scn_ctx_destroy(scn_ctx *c) {
  if (!c)
    return SCN_OK;
  (void)scn_chain_flush(c);
  (void)hipStreamSynchronize(c->stream);
  scn_abt_static_forget(c);
  scn_chain_release(c);
  for (auto &s : c->spans) {
    (void)hipEventDestroy(s.a);
    (void)hipEventDestroy(s.b);
  }
  for (auto e : c->freeEvents)
    (void)hipEventDestroy(e);
  (void)hipFree(c->d_scalars);
  (void)hipFree(c->d_zeros);
  (void)hipHostFree(c->h_pinned);
  (void)hipStreamDestroy(c->stream);
  delete c;
  return SCN_OK;
}

extern "C" void *scn_ctx_stream(scn_ctx *c) { return (void *)c->stream; }

extern "C" int scn_sync(scn_ctx *c) {
  SCN_HIP_CHECK(hipStreamSynchronize(c->stream));
  return SCN_OK;
}

extern "C" int scn_malloc(scn_ctx *c, size_t bytes, void **d_ptr) {
  SCN_REQUIRE(c && d_ptr, SCN_ERR_ARG, "scn_malloc: null argument");
  *d_ptr = nullptr;
  if (bytes == 0)
    bytes = 16;
  SCN_HIP_CHECK(hipMalloc(d_ptr, bytes));
  return SCN_OK;
}

extern "C" int scn_free(scn_ctx *c, void *d_ptr) {
  (void)c;
  if (d_ptr)
    SCN_HIP_CHECK(hipFree(d_ptr));
  return SCN_OK;
}

extern "C" int scn_h2d(scn_ctx *c, void *d_dst, const void *h_src,
                       size_t bytes) {
  if (bytes == 0)
    return SCN_OK;
  if (!c) { // no stream named: ordered after the work of every stream
    SCN_HIP_CHECK(hipMemcpy(d_dst, h_src, bytes, hipMemcpyHostToDevice));
    return SCN_OK;
  }
  SCN_HIP_CHECK(
      hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, c->stream));
  SCN_HIP_CHECK(hipStreamSynchronize(c->stream));
  return SCN_OK;
}

extern "C" int scn_d2h(scn_ctx *c, void *h_dst, const void *d_src,
                       size_t bytes) {
  if (bytes == 0)
    return SCN_OK;
  if (!c) {
    SCN_HIP_CHECK(hipMemcpy(h_dst, d_src, bytes, hipMemcpyDeviceToHost));
    return SCN_OK;
  }
  SCN_HIP_CHECK(
      hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, c->stream));
  SCN_HIP_CHECK(hipStreamSynchronize(c->stream));
  return SCN_OK;
}

struct scn_event {
  hipEvent_t ev;
};
extern "C" int scn_host_alloc(scn_ctx *c, size_t bytes, void **h_ptr) {
  SCN_REQUIRE(c && h_ptr, SCN_ERR_ARG, "scn_host_alloc: null argument");
  *h_ptr = nullptr;
  if (bytes == 0)
    return SCN_OK;
  SCN_HIP_CHECK(hipSetDevice(c->device));
  SCN_HIP_CHECK(hipHostMalloc(h_ptr, bytes, hipHostMallocDefault));
  return SCN_OK;
}
extern "C" int scn_host_free(scn_ctx *c, void *h_ptr) {
  (void)c;
  if (h_ptr)
    SCN_HIP_CHECK(hipHostFree(h_ptr));
  return SCN_OK;
}
extern "C" int scn_h2d_async(scn_ctx *c, void *d_dst, const void *h_src,
                             size_t bytes) {
  SCN_REQUIRE(c, SCN_ERR_ARG, "scn_h2d_async: null context");
  if (bytes == 0)
    return SCN_OK;
  SCN_REQUIRE(d_dst && h_src, SCN_ERR_ARG, "scn_h2d_async: null buffer");
  SCN_HIP_CHECK(
      hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, c->stream));
  return SCN_OK;
}
extern "C" int scn_d2h_async(scn_ctx *c, void *h_dst, const void *d_src,
                             size_t bytes) {
  SCN_REQUIRE(c, SCN_ERR_ARG, "scn_d2h_async: null context");
  if (bytes == 0)
    return SCN_OK;
  SCN_REQUIRE(h_dst && d_src, SCN_ERR_ARG, "scn_d2h_async: null buffer");
  SCN_HIP_CHECK(
      hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, c->stream));
  return SCN_OK;
}
extern "C" int scn_event_create(scn_ctx *c, scn_event **event) {
  SCN_REQUIRE(c && event, SCN_ERR_ARG, "scn_event_create: null argument");
  SCN_HIP_CHECK(hipSetDevice(c->device));
  scn_event *e = new scn_event;
  hipError_t rc = hipEventCreateWithFlags(&e->ev, hipEventDisableTiming);
  if (rc != hipSuccess) {
    delete e;
    SCN_HIP_CHECK(rc);
  }
  *event = e;
  return SCN_OK;
}
extern "C" int scn_event_destroy(scn_event *event) {
  if (event) {
    (void)hipEventDestroy(event->ev);
    delete event;
  }
  return SCN_OK;
}
extern "C" int scn_event_record(scn_ctx *c, scn_event *event) {
  SCN_REQUIRE(c && event, SCN_ERR_ARG, "scn_event_record: null argument");
  SCN_HIP_CHECK(hipEventRecord(event->ev, c->stream));
  return SCN_OK;
}
extern "C" int scn_event_wait(scn_event *event) {
  SCN_REQUIRE(event, SCN_ERR_ARG, "scn_event_wait: null event");
  SCN_HIP_CHECK(hipEventSynchronize(event->ev));
  return SCN_OK;
}

// A copy made by a kernel: either side may be device memory or pinned host
// memory (which the device reads and writes over the bus).  Queueing it costs
// the host one kernel launch, where an asynchronous memcpy of a few hundred
// kilobytes costs many times that.
__global__ void k_copy(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                       size_t bytes, int vec) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  if (vec) {
    const size_t n16 = bytes / 16;
    const uint4 *s = reinterpret_cast<const uint4 *>(src);
    uint4 *d = reinterpret_cast<uint4 *>(dst);
    for (size_t k = i; k < n16; k += step)
      d[k] = s[k];
    for (size_t k = n16 * 16 + i; k < bytes; k += step)
      dst[k] = src[k];
  } else {
    for (size_t k = i; k < bytes; k += step)
      dst[k] = src[k];
  }
}
extern "C" int scn_copy(scn_ctx *c, void *dst, const void *src, size_t bytes) {
  SCN_REQUIRE(c, SCN_ERR_ARG, "scn_copy: null context");
  if (bytes == 0)
    return SCN_OK;
  SCN_REQUIRE(dst && src, SCN_ERR_ARG, "scn_copy: null buffer");
  const int vec = (((uintptr_t)dst | (uintptr_t)src) & 15) == 0;
  size_t blocks = (bytes / (vec ? 16 : 1) + 255) / 256;
  blocks = blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks);
  hipLaunchKernelGGL(k_copy, dim3((unsigned)blocks), dim3(256), 0, c->stream,
                     (const uint8_t *)src, (uint8_t *)dst, bytes, vec);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

extern "C" int scn_d2d(scn_ctx *c, void *d_dst, const void *d_src,
                       size_t bytes) {
  return scn_copy(c, d_dst, d_src, bytes);
}

__global__ void k_fill32(uint32_t *dst, uint32_t w, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += step)
    dst[i] = w;
}

extern "C" int scn_fill32(scn_ctx *c, void *d_dst, uint32_t word,
                          size_t nWords) {
  if (nWords == 0)
    return SCN_OK;
  int blocks = (int)((nWords + 255) / 256);
  if (blocks > 65536)
    blocks = 65536;
  hipLaunchKernelGGL(k_fill32, dim3(blocks), dim3(256), 0, c->stream,
                     (uint32_t *)d_dst, word, nWords);
  SCN_HIP_CHECK(hipGetLastError());
  return SCN_OK;
}

// ---- profiling ---------------------------------------------------------

static hipEvent_t take_event(scn_ctx *c) {
  if (!c->freeEvents.empty()) {
    hipEvent_t e = c->freeEvents.back();
    c->freeEvents.pop_back();
    return e;
  }
  hipEvent_t e;
  (void)hipEventCreate(&e);
  return e;
}

ProfScope::ProfScope(scn_ctx *c, int family) : ctx(c), idx(-1) {
  if (!c->prof)
    return;
  ProfSpan s;
  s.family = family;
  s.tag = c->profTag;
  s.a = take_event(c);
  s.b = take_event(c);
  (void)hipEventRecord(s.a, c->stream);
  c->spans.push_back(s);
  idx = (int)c->spans.size() - 1;
}

ProfScope::~ProfScope() {
  if (idx >= 0)
    (void)hipEventRecord(ctx->spans[idx].b, ctx->stream);
}

__global__ void k_nothing() {}
extern "C" int scn_prof_probe(scn_ctx *c, int with_kernel) {
  SCN_REQUIRE(c, SCN_ERR_ARG, "scn_prof_probe: null context");
  ProfScope prof(c, SCN_K_PROBE);
  if (with_kernel) {
    hipLaunchKernelGGL(k_nothing, dim3(1), dim3(64), 0, c->stream);
    SCN_HIP_CHECK(hipGetLastError());
  }
  return SCN_OK;
}

static void drain_spans(scn_ctx *c, int capacity = 0, int32_t *family = nullptr,
                        int32_t *tag = nullptr, double *msOut = nullptr,
                        int32_t *n = nullptr) {
  (void)hipStreamSynchronize(c->stream);
  int kept = 0;
  for (auto &s : c->spans) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, s.a, s.b) == hipSuccess) {
      c->profMs[s.family] += ms;
      c->profCalls[s.family] += 1;
      if (kept < capacity) {
        family[kept] = s.family;
        tag[kept] = s.tag;
        msOut[kept] = ms;
        ++kept;
      }
    }
    c->freeEvents.push_back(s.a);
    c->freeEvents.push_back(s.b);
  }
  c->spans.clear();
  if (n)
    *n = kept;
}

extern "C" int scn_prof_tag(scn_ctx *c, int tag) {
  c->profTag = tag;
  return SCN_OK;
}

extern "C" int scn_prof_spans(scn_ctx *c, int capacity, int32_t *family,
                              int32_t *tag, double *ms, int32_t *n) {
  SCN_REQUIRE(capacity >= 0 && n && (capacity == 0 || (family && tag && ms)),
              SCN_ERR_ARG, "scn_prof_spans: null output");
  drain_spans(c, capacity, family, tag, ms, n);
  return SCN_OK;
}

extern "C" int scn_prof_enable(scn_ctx *c, int on) {
  drain_spans(c);
  c->prof = on != 0;
  return SCN_OK;
}

extern "C" int scn_prof_reset(scn_ctx *c) {
  drain_spans(c);
  memset(c->profMs, 0, sizeof(c->profMs));
  memset(c->profCalls, 0, sizeof(c->profCalls));
  return SCN_OK;
}

extern "C" int scn_prof_read(scn_ctx *c, int family, double *ms,
                             int64_t *calls) {
  SCN_REQUIRE(family >= 0 && family < SCN_K_COUNT, SCN_ERR_ARG,
              "scn_prof_read: family %d", family);
  drain_spans(c);
  if (ms)
    *ms = c->profMs[family];
  if (calls)
    *calls = c->profCalls[family];
  return SCN_OK;
}
