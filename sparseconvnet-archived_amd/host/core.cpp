// Plumbing of the host library: enumerations, random numbers, the
// host/device vector, batch containers, pictures and the dataset container.
#include <algorithm>
#include <cassert>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <mutex>
#include "Picture.h"
#include "SpatiallySparseBatch.h"
#include "SpatiallySparseDataset.h"
#include "SpatiallySparseLayer.h"
#include "types.h"
#include "vectorCUDA.h"

const char *batchTypeNames[] = {"TRAINBATCH", "TESTBATCH", "UNLABELEDBATCH",
                                "RESCALEBATCH"};
const char *sigmoidNames[] = {"", "ReLU", "VeryLeakyReLU", "LeakyReLU", "tanh",
                              "Softmax Classification", "PReLU", "Sigmoid"};
__int128_t multiplyAddCount;
static std::mutex g_macMutex;
void addMultiplyAdds(__int128_t n) {
  std::lock_guard<std::mutex> lock(g_macMutex);
  multiplyAddCount += n;
}

// ---- utilities (utilities.cu:5-56,102-103) -----------------------------------
std::vector<int> range(int n) {
  std::vector<int> r(n);
  for (int i = 0; i < n; ++i)
    r[i] = i;
  return r;
}
int ipow(int base, int exp) {
  int r = 1;
  for (; exp; exp >>= 1, base *= base)
    if (exp & 1)
      r *= base;
  return r;
}
int triangleSize(int linearSize, int dimension) {
  int fs = 1;
  for (int i = 1; i <= dimension; ++i)
    fs = fs * (linearSize + dimension - i) / i;
  return fs;
}
int intRoundUp(int a, int d) { return ((a + d - 1) / d) * d; }
int intRound(int a, int d) { return (int)(round(a * 1.0 / d) * d); }

// Top-k indices, best first; on ties the lower index stays ahead.
template <typename t>
std::vector<int> vectorTopIndices(std::vector<t> &test, int k) {
  std::vector<int> indices(k);
  std::vector<t> best(k);
  best[0] = test[0];
  for (int i = 1; i < (int)test.size(); i++) {
    int j = std::min(i, k);
    if (test[i] > best[j - 1]) {
      if (i >= k)
        --j;
      while (j > 0 && test[i] > best[j - 1]) {
        best[j] = best[j - 1];
        indices[j] = indices[j - 1];
        --j;
      }
    }
    if (j < k) {
      best[j] = test[i];
      indices[j] = i;
    }
  }
  return indices;
}
template std::vector<int> vectorTopIndices<float>(std::vector<float> &, int);

// ---- RNG ------------------------------------------------------------------------
static std::mutex seedMutex;
RNG::RNG() {
  std::lock_guard<std::mutex> lock(seedMutex);
  static unsigned bump = 0;
  // SCN_SEED in the environment: generators seeded from that number instead
  // of the clock, in the order they are made (a repeatable run)
  if (const char *fixed = std::getenv("SCN_SEED")) {
    gen.seed((unsigned)std::strtoul(fixed, nullptr, 10) + 7919u * bump++);
    return;
  }
  auto now = std::chrono::high_resolution_clock::now().time_since_epoch();
  gen.seed((unsigned)now.count() + 7919u * bump++);
}
RNG::RNG(unsigned seed) { gen.seed(seed); }
int RNG::randint(int n) {
  return n <= 1 ? 0 : (int)(gen() % (unsigned)n);
}
float RNG::uniform(float a, float b) {
  return a + (b - a) * (float)((gen() >> 8) * (1.0 / 16777216.0));
}
float RNG::normal(float mean, float sd) {
  float u1 = std::max(uniform(), 1e-7f), u2 = uniform();
  return mean + sd * std::sqrt(-2.0f * std::log(u1)) *
                    std::cos(6.28318530718f * u2);
}
int RNG::bernoulli(float p) { return uniform() < p ? 1 : 0; }
std::vector<int> RNG::NchooseM(int n, int m) {
  std::vector<int> ret(m);
  int left = m;
  for (int i = 0; i < n && left > 0; ++i)
    if (randint(n - i) < left) {
      ret[m - left] = i;
      --left;
    }
  return ret;
}

// ---- context --------------------------------------------------------------------
static scn_ctx *g_defaultCtx = nullptr;
static std::vector<scn_ctx *> g_liveCtx; // oldest first
static std::mutex g_ctxMutex;

// Ends the process the way the reference's error paths do (print, exit),
// but without running static destructors: other threads (batch producers)
// may still be inside the library.
void scnExit(int code) {
  std::fflush(nullptr);
  std::_Exit(code);
}
void scnCheck(int rc, const char *file, int line) {
  if (rc == SCN_OK)
    return;
  // the reference prints the CUDA error and exits (utilities.h:36-67)
  std::fprintf(stderr, "%s:%d: libscn_hip error %d: %s\n", file, line, rc,
               scn_last_error());
  scnExit(EXIT_FAILURE);
}
scn_ctx *scnDefaultContext() {
  if (!g_defaultCtx) {
    std::fprintf(stderr, "no SparseConvNet context: construct the net first\n");
    scnExit(EXIT_FAILURE);
  }
  return g_defaultCtx;
}
cudaMemStream::cudaMemStream() : ctx(nullptr) {
  std::lock_guard<std::mutex> lock(g_ctxMutex);
  SCN_CHECKED(scn_ctx_create(-1, &ctx));
  g_liveCtx.push_back(ctx);
  g_defaultCtx = g_liveCtx.front();
}
cudaMemStream::~cudaMemStream() {
  std::lock_guard<std::mutex> lock(g_ctxMutex);
  g_liveCtx.erase(std::find(g_liveCtx.begin(), g_liveCtx.end(), ctx));
  g_defaultCtx = g_liveCtx.empty() ? nullptr : g_liveCtx.front();
  scn_ctx_destroy(ctx);
}
void *cudaMemStream::stream() const { return scn_ctx_stream(ctx); }
void cudaMemStream::synchronize() const { SCN_CHECKED(scn_sync(ctx)); }

// ---- vectorCUDA -----------------------------------------------------------------
template <typename t>
vectorCUDA<t>::vectorCUDA(bool onGPU, size_t dsize)
    : d_vec(nullptr), dsize(0), dAllocated(0), onGPU(onGPU) {
  if (onGPU) {
    if (dsize > 0)
      resize64(dsize);
  } else {
    vec.resize(dsize);
  }
}
template <typename t>
vectorCUDA<t>::vectorCUDA(vectorCUDA &&o)
    : d_vec(o.d_vec), dsize(o.dsize), dAllocated(o.dAllocated),
      vec(std::move(o.vec)), onGPU(o.onGPU) {
  o.d_vec = nullptr;
  o.dsize = 0;
  o.dAllocated = 0;
}
template <typename t> vectorCUDA<t>::~vectorCUDA() {
  if (d_vec)
    scn_free(nullptr, d_vec);
}
// No stream named (vectorCUDA.cu:26-57, blocking cudaMemcpy): a copy with a
// null context waits for the work of every stream of the device first, so the
// data is complete whichever net's stream produced it.
// The flip itself is serialised: the forward lanes' threads share the layers'
// parameters, and two of them may ask for dPtr() of a vector that a host-side
// writer left on the CPU.
static std::mutex g_flipMutex;
template <typename t> void vectorCUDA<t>::copyToCPU() {
  std::lock_guard<std::mutex> lock(g_flipMutex);
  if (!onGPU)
    return;
  toCPU(nullptr);
}
template <typename t> void vectorCUDA<t>::copyToGPU() {
  std::lock_guard<std::mutex> lock(g_flipMutex);
  if (onGPU)
    return;
  toGPU(nullptr);
}
template <typename t> void vectorCUDA<t>::toCPU(scn_ctx *ctx) {
  onGPU = false;
  vec.resize(dsize);
  if (dsize > 0)
    SCN_CHECKED(scn_d2h(ctx, vec.data(), d_vec, sizeof(t) * (size_t)dsize));
}
template <typename t> void vectorCUDA<t>::toGPU(scn_ctx *ctx) {
  onGPU = true;
  dsize = 0;
  resize64(vec.size());
  if (dsize > 0)
    SCN_CHECKED(scn_h2d(ctx, d_vec, vec.data(), sizeof(t) * (size_t)dsize));
  vec.clear();
}
// the copies go on the named stream and return when they are done, as the
// reference's do (vectorCUDA.cu:58-108 synchronise the stream)
template <typename t>
void vectorCUDA<t>::copyToCPUAsync(cudaMemStream &memStream) {
  if (onGPU)
    toCPU(memStream.ctx);
}
template <typename t>
void vectorCUDA<t>::copyToGPUAsync(cudaMemStream &memStream) {
  if (!onGPU)
    toGPU(memStream.ctx);
}
template <typename t> t *&vectorCUDA<t>::dPtr() {
  copyToGPU();
  return d_vec;
}
template <typename t> std::vector<t> &vectorCUDA<t>::hVector() {
  copyToCPU();
  return vec;
}
template <typename t> unsigned int vectorCUDA<t>::size() {
  return (unsigned int)size64();
}
template <typename t> size_t vectorCUDA<t>::size64() {
  return onGPU ? dsize : vec.size();
}
template <typename t> void vectorCUDA<t>::setZero() {
  if (onGPU) {
    static_assert(sizeof(t) == 4, "32-bit elements");
    // no stream named: done before the call returns, whatever stream uses
    // the memory next
    SCN_CHECKED(scn_fill32(scnDefaultContext(), d_vec, 0u, dsize));
    SCN_CHECKED(scn_sync(scnDefaultContext()));
  } else {
    std::fill(vec.begin(), vec.end(), (t)0);
  }
}
template <typename t> void vectorCUDA<t>::setZero(cudaMemStream &memStream) {
  if (onGPU) {
    static_assert(sizeof(t) == 4, "32-bit elements");
    SCN_CHECKED(scn_fill32(memStream.ctx, d_vec, 0u, dsize));
  } else {
    std::fill(vec.begin(), vec.end(), (t)0);
  }
}
template <typename t> void vectorCUDA<t>::setConstant(float a) {
  bool wasOnGPU = onGPU;
  std::vector<t> &h = hVector();
  std::fill(h.begin(), h.end(), (t)a);
  if (wasOnGPU)
    copyToGPU();
}
template <typename t> void vectorCUDA<t>::setUniform(float a, float b) {
  bool wasOnGPU = onGPU;
  std::vector<t> &h = hVector();
  RNG rng;
  for (auto &x : h)
    x = (t)rng.uniform(a, b);
  if (wasOnGPU)
    copyToGPU();
}
// Device storage grows, never shrinks, and growth does not keep the contents
// (every producer rewrites the whole vector after resizing it).
template <typename t> void vectorCUDA<t>::resize(int n) {
  resize64((size_t)(n < 0 ? 0 : n));
}
template <typename t> void vectorCUDA<t>::resize64(size_t n) {
  if (!onGPU) {
    vec.resize(n);
    return;
  }
  if (n > dAllocated) {
    if (d_vec)
      SCN_CHECKED(scn_free(nullptr, d_vec));
    size_t want = n + n / 4;
    void *p = nullptr;
    SCN_CHECKED(scn_malloc(scnDefaultContext(), want * sizeof(t), &p));
    d_vec = (t *)p;
    dAllocated = want;
  }
  dsize = n;
}
template class vectorCUDA<float>;
template class vectorCUDA<int>;

// ---- batch containers -----------------------------------------------------------
SpatiallySparseBatchSubInterface::SpatiallySparseBatchSubInterface() {
  reset();
}
void SpatiallySparseBatchSubInterface::reset() {
  features.resize(0);
  dfeatures.resize(0);
  poolingChoices.resize(0);
}

SpatiallySparseBatchInterface::SpatiallySparseBatchInterface(
    SpatiallySparseBatchSubInterface *s)
    : sub(s), featuresPresent(false, 0), deviceGrids(nullptr),
      ownsDeviceGrids(false), rules(true, 0), deferredGatherFrom(nullptr) {
  reset();
}
SpatiallySparseBatchInterface::SpatiallySparseBatchInterface(
    SpatiallySparseBatchInterface &&o)
    : sub(o.sub), nFeatures(o.nFeatures),
      featuresPresent(std::move(o.featuresPresent)),
      nSpatialSites(o.nSpatialSites), spatialSize(o.spatialSize),
      backpropErrors(o.backpropErrors), grids(std::move(o.grids)),
      deviceGrids(o.deviceGrids), ownsDeviceGrids(o.ownsDeviceGrids),
      rules(std::move(o.rules)), deferredGatherFrom(nullptr) {
  o.deviceGrids = nullptr;
  o.ownsDeviceGrids = false;
}
SpatiallySparseBatchInterface::~SpatiallySparseBatchInterface() {
  if (deviceGrids && ownsDeviceGrids)
    scn_grids_destroy(nullptr, deviceGrids);
}
void SpatiallySparseBatchInterface::reset() {
  featuresPresent.resize(0);
  nSpatialSites = 0;
  grids.resize(0);
  rules.resize(0);
  backpropErrors = false;
  deferredGatherFrom = nullptr;
  // deviceGrids keeps its tables for the next batch
}
// Rebuilds the host SparseGrid view from the tables in HBM.
void SpatiallySparseBatchInterface::downloadGrids(int batchSize) {
  grids.assign(batchSize, SparseGrid());
  if (!deviceGrids)
    return;
  int64_t nActive = 0;
  SCN_CHECKED(scn_grids_info(deviceGrids, nullptr, nullptr, nullptr, &nActive,
                             nullptr));
  std::vector<int32_t> sample(nActive), row(nActive), bg(batchSize);
  std::vector<int64_t> key(nActive);
  SCN_CHECKED(scn_grids_download(scnDefaultContext(), deviceGrids,
                                 sample.data(), key.data(), row.data(),
                                 bg.data()));
  for (int i = 0; i < batchSize; ++i)
    grids[i].backgroundCol = bg[i];
  for (int64_t e = 0; e < nActive; ++e)
    grids[sample[e]].mp[key[e]] = row[e];
}
void SpatiallySparseBatchInterface::summary() {
  std::cout << "nFeatures " << nFeatures << " featuresPresent "
            << featuresPresent.size() << " spatialSize " << spatialSize
            << " nSpatialSites " << nSpatialSites << " features "
            << sub->features.size() << " rules " << rules.size() << std::endl;
}

BatchResultStage::BatchResultStage()
    : pinned(nullptr), capacity(0), arrived(nullptr), pending(false),
      consumed(nullptr), consumedPending(false), enqueued(true) {}
BatchResultStage::~BatchResultStage() {
  if (arrived)
    scn_event_destroy(arrived);
  if (consumed)
    scn_event_destroy(consumed);
  if (pinned)
    scn_host_free(scnDefaultContext(), pinned);
}

PinnedStage::~PinnedStage() {
  if (p)
    scn_host_free(scnDefaultContext(), p);
}
void PinnedStage::reserve(size_t n) {
  if (n <= bytes)
    return;
  if (p)
    SCN_CHECKED(scn_host_free(scnDefaultContext(), p));
  p = nullptr;
  bytes = n + n / 2 + 4096; // (pinning is slow: with room to grow)
  SCN_CHECKED(scn_host_alloc(scnDefaultContext(), bytes, &p));
}

SpatiallySparseBatch::SpatiallySparseBatch(
    SpatiallySparseBatchSubInterface *inputSub)
    : inputSub(inputSub), preprocessStream(nullptr), forwardStream(nullptr),
      labels(false, 0),
      stagingSample(true, 0), stagingKey(true, 0), stagingRow(true, 0),
      stagingBackground(true, 0), hostSites(0), hostFeatureCount(0),
      result(new BatchResultStage()) {
  interfaces.emplace_back(inputSub);
  reset();
}
void SpatiallySparseBatch::reset() {
  batchSize = 0;
  sampleNumbers.resize(0);
  for (auto &i : interfaces)
    i.reset();
  // emptied first, so moving them to the host copies nothing
  interfaces[0].sub->reset();
  interfaces[0].sub->features.copyToCPU();
  labels.resize(0);
  labels.copyToCPU();
  result->labels.clear();
  predictions.resize(0);
  probabilities.resize(0);
  negativeLogLikelihood = 0;
  mistakes = 0;
}

// ---- pictures and datasets ------------------------------------------------------
Picture::Picture(int label) : label(label) {}
Picture::~Picture() {}
std::string Picture::identify() { return std::string(); }

SparsePointsPicture::SparsePointsPicture(int dimension, int latticeSize,
                                         int nFeatures, int label)
    : Picture(label), dimension(dimension), latticeSize(latticeSize),
      nFeatures(nFeatures) {}
std::string SparsePointsPicture::identify() { return "sparse points"; }
void SparsePointsPicture::codifyInputData(SparseGrid &grid,
                                          std::vector<float> &out,
                                          int &nSpatialSites,
                                          int spatialSize) {
  // background row first, like every Picture of the reference
  // (OpenCVPicture.cpp:373-375)
  for (int i = 0; i < nFeatures; ++i)
    out.push_back(0);
  grid.backgroundCol = nSpatialSites++;
  const int shift = (spatialSize - latticeSize) / 2;
  const size_t nSites = coords.size() / dimension;
  grid.mp.reserve(nSites);
  for (size_t s = 0; s < nSites; ++s) {
    int64_t key = 0;
    bool inside = true;
    for (int a = 0; a < dimension; ++a) {
      int c = coords[s * dimension + a] + shift;
      inside = inside && c >= 0 && c < spatialSize;
      key = key * spatialSize + c;
    }
    // the first point of a site makes its row; later ones change nothing
    if (!inside || !grid.mp.insert(std::make_pair(key, nSpatialSites)).second)
      continue;
    nSpatialSites++;
    out.insert(out.end(), features.begin() + s * nFeatures,
               features.begin() + (s + 1) * nFeatures);
  }
}

SpatiallySparseDataset::SpatiallySparseDataset()
    : nFeatures(0), nClasses(0), type(TESTBATCH) {}
void SpatiallySparseDataset::summary() {
  std::cout << "Name:            " << name << std::endl;
  std::cout << "Type:            " << batchTypeNames[type] << std::endl;
  std::cout << "nFeatures:       " << nFeatures << std::endl;
  std::cout << "nPictures:       " << pictures.size() << std::endl;
  std::cout << "nClasses:        " << nClasses << std::endl;
  std::vector<int> count(std::max(nClasses, 1));
  for (auto *p : pictures)
    if (p->label >= 0 && p->label < nClasses)
      count[p->label]++;
  std::cout << "nPictures/class: ";
  for (int c : count)
    std::cout << c << " ";
  std::cout << std::endl;
}
void SpatiallySparseDataset::shuffle() { rng.vectorShuffle(pictures); }
SpatiallySparseDataset SpatiallySparseDataset::extractValidationSet(float p) {
  SpatiallySparseDataset val;
  val.name = name + std::string(" Validation set");
  name = name + std::string(" minus Validation set");
  val.nFeatures = nFeatures;
  val.nClasses = nClasses;
  val.type = TESTBATCH;
  shuffle();
  size_t size = pictures.size();
  while (pictures.size() > size * (1 - p)) {
    val.pictures.push_back(pictures.back());
    pictures.pop_back();
  }
  return val;
}
void SpatiallySparseDataset::subsetOfClasses(std::vector<int> activeClasses) {
  nClasses = (int)activeClasses.size();
  std::vector<Picture *> keep;
  for (auto *p : pictures) {
    auto it = std::find(activeClasses.begin(), activeClasses.end(), p->label);
    if (it != activeClasses.end()) {
      p->label = (int)(it - activeClasses.begin());
      keep.push_back(p);
    } else {
      delete p;
    }
  }
  pictures = keep;
}
SpatiallySparseDataset SpatiallySparseDataset::subset(int n) {
  SpatiallySparseDataset sub(*this);
  sub.shuffle();
  if ((int)sub.pictures.size() > n)
    sub.pictures.resize(n);
  return sub;
}
SpatiallySparseDataset SpatiallySparseDataset::balancedSample(int n) {
  SpatiallySparseDataset bs;
  bs.name = name + std::string(" balanced sample");
  bs.nFeatures = nFeatures;
  bs.nClasses = nClasses;
  bs.type = type;
  auto perm = range((int)pictures.size());
  rng.vectorShuffle(perm);
  std::vector<int> count(std::max(nClasses, 1));
  int classesDone = 0;
  for (size_t i = 0; i < pictures.size() && classesDone < nClasses; i++) {
    int l = pictures[perm[i]]->label;
    if (l >= 0 && l < nClasses && count[l]++ < n) {
      bs.pictures.push_back(pictures[perm[i]]);
      if (count[l] == n)
        classesDone++;
    }
  }
  return bs;
}
void SpatiallySparseDataset::repeatSamples(int reps) {
  size_t s = pictures.size();
  for (int i = 1; i < reps; ++i)
    for (size_t j = 0; j < s; ++j)
      pictures.push_back(pictures[j]);
}
