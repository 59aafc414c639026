// Net runtime, batch production, public facades and canned architectures.
#include <cstring>
#include <algorithm>
#include <atomic>
#include <cassert>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include "BatchProducer.h"
#include "NetworkArchitectures.h"
#include "SparseConvNet.h"
#include "SparseConvNetCUDA.h"

#define FEATURE_QUANTUM 32 // KERNELBLOCKSIZE of the reference (utilities.h:73)

// ================================================================ runtime
SparseConvNetCUDA::SparseConvNetCUDA(int dimension, int nInputFeatures,
                                     int nClasses, int pciBusID, int nTop,
                                     int nBatchProducerThreads)
    : dimension(dimension), nClasses(nClasses), nTop(nTop),
      inputSpatialSize(0), nInputFeatures(nInputFeatures),
      nOutputFeatures(nInputFeatures), deviceID(0),
      nBatchProducerThreads(nBatchProducerThreads), producerStreamsWanted(0) {
  (void)pciBusID; // one GPU per process: the context picks device 0
  assert(nBatchProducerThreads >= 1 &&
         nBatchProducerThreads <= N_MAX_BATCH_PRODUCER_THREADS);
  std::cout << "Sparse CNN - dimension=" << dimension
            << " nInputFeatures=" << nInputFeatures << " nClasses=" << nClasses
            << std::endl;
  // (lane streams first: streams take hardware queues in order of creation,
  // and the forward passes should not share theirs with producer streams)
  nForwardLanes = nBatchProducerThreads >= 4 ? 2 : 1;
  for (int lane = 1; lane < nForwardLanes; ++lane)
    laneStreams.emplace_back(new cudaMemStream());
  batchPool.reserve(nBatchProducerThreads);
  const int nStreams = std::min(nBatchProducerThreads, N_PRODUCER_STREAMS);
  for (int c = 0; c < nStreams; c++) {
    batchMemStreams.emplace_back(new cudaMemStream());
    freeProducerStreams.push_back(batchMemStreams.back().get());
  }
  for (int c = 0; c < nBatchProducerThreads; c++) {
    initialSubInterfaces.push_back(new SpatiallySparseBatchSubInterface());
    batchPool.emplace_back(initialSubInterfaces.back());
    batchPool.back().preprocessStream = batchMemStreams[c % nStreams].get();
  }
}
// (between passes: no producer thread holds a stream)
void SparseConvNetCUDA::setProducerStreams(int n) {
  std::lock_guard<std::mutex> lock(streamPoolMutex);
  producerStreamsWanted = n;
  const int all = (int)batchMemStreams.size();
  const int use = n < 1 || n > all ? all : n;
  freeProducerStreams.clear();
  for (int c = 0; c < use; c++)
    freeProducerStreams.push_back(batchMemStreams[c].get());
}
int SparseConvNetCUDA::producerStreamsInUse() {
  std::lock_guard<std::mutex> lock(streamPoolMutex);
  const int all = (int)batchMemStreams.size();
  return producerStreamsWanted < 1 || producerStreamsWanted > all ? all : producerStreamsWanted;
}
cudaMemStream *SparseConvNetCUDA::acquireProducerStream(int batchNumber) {
  std::unique_lock<std::mutex> lock(streamPoolMutex);
  auto mine = waitingBatches.insert(batchNumber);
  streamPoolChanged.wait(lock, [&] {
    return !freeProducerStreams.empty() && *waitingBatches.begin() == batchNumber;
  });
  waitingBatches.erase(mine);
  cudaMemStream *s = freeProducerStreams.front(); // the longest idle one
  freeProducerStreams.erase(freeProducerStreams.begin());
  if (!freeProducerStreams.empty() && !waitingBatches.empty())
    streamPoolChanged.notify_all(); // the next waiter may go too
  return s;
}
void SparseConvNetCUDA::releaseProducerStream(cudaMemStream *stream) {
  {
    std::lock_guard<std::mutex> lock(streamPoolMutex);
    freeProducerStreams.push_back(stream);
  }
  streamPoolChanged.notify_all();
}
cudaMemStream &SparseConvNetCUDA::laneStream(int lane) {
  return lane == 0 ? memStream : *laneStreams[lane - 1];
}
void SparseConvNetCUDA::synchronizeLanes() {
  memStream.synchronize();
  for (auto &s : laneStreams)
    s->synchronize();
}
void SparseConvNetCUDA::limitBatchProducerThreads(int n) {
  if (n < 1 || n >= nBatchProducerThreads)
    return;
  nBatchProducerThreads = n;
  if (n < 4)
    nForwardLanes = 1;
  while ((int)batchPool.size() > n)
    batchPool.pop_back();
  const int nStreams = std::min(n, N_PRODUCER_STREAMS);
  while ((int)batchMemStreams.size() > nStreams)
    batchMemStreams.pop_back();
  setProducerStreams(producerStreamsWanted);
  for (int c = 0; c < n; c++)
    batchPool[c].preprocessStream = batchMemStreams[c % nStreams].get();
}
SparseConvNetCUDA::~SparseConvNetCUDA() {
  for (auto &s : batchMemStreams)
    s->synchronize();
  synchronizeLanes();
  batchPool.clear();
  for (auto p : layers)
    delete p;
  for (auto p : initialSubInterfaces)
    delete p;
  for (auto p : sharedSubInterfaces)
    delete p;
  for (auto &lane : laneSubInterfaces)
    for (auto p : lane)
      delete p;
}
// SparseConvNetCUDA.cu:50-70
void SparseConvNetCUDA::addLearntLayer(int nFeatures,
                                       ActivationFunction activationFn,
                                       float dropout, float alpha) {
  // every learnt layer but the classifier is rounded to a multiple of 32
  if (activationFn != SOFTMAX)
    nFeatures = std::max(FEATURE_QUANTUM, intRound(nFeatures, FEATURE_QUANTUM));
  if (dropout > 0)
    dropout = 1 - (intRound(nFeatures * (1 - dropout), FEATURE_QUANTUM) + 0.01f) *
                      1.0f / nFeatures;
  if (dropout < 0)
    dropout = 0;
  std::cout << layers.size() << ":";
  if (activationFn == PRELU)
    layers.push_back(new NetworkInNetworkPReLULayer(
        memStream, nOutputFeatures, nFeatures, dropout, alpha));
  else
    layers.push_back(new NetworkInNetworkLayer(memStream, nOutputFeatures,
                                               nFeatures, dropout,
                                               activationFn, alpha));
  nOutputFeatures = nFeatures;
}
void SparseConvNetCUDA::addNetworkInNetworkLayer(
    int nFeatures, ActivationFunction activationFn, float dropout) {
  addLearntLayer(nFeatures, activationFn, dropout, 1.0f);
}
// SparseConvNetCUDA.cu:75-98: filterSize 1 adds no gather layer
void SparseConvNetCUDA::addConvolutionalLayer(int nFeatures, int filterSize,
                                              int filterStride,
                                              ActivationFunction activationFn,
                                              float dropout,
                                              int minActiveInputs,
                                              float poolingToFollow) {
  if (filterSize > 1) {
    std::cout << layers.size() << ":";
    layers.push_back(new ConvolutionalLayer(memStream, filterSize, filterStride,
                                            dimension, nOutputFeatures,
                                            minActiveInputs));
    nOutputFeatures *= ipow(filterSize, dimension);
  }
  addLearntLayer(nFeatures, activationFn, dropout,
                 powf(filterSize * 1.0 / filterStride / poolingToFollow, 2));
}
// addLeNetLayerPOFMP / PDFMP / ROFMP / RDFMP (SparseConvNetCUDA.cu:112-163)
void SparseConvNetCUDA::addLeNetLayerFMP(int kind, int nFeatures,
                                         int filterSize, int filterStride,
                                         int poolSize, float fmpShrink,
                                         ActivationFunction activationFn,
                                         float dropout, int minActiveInputs) {
  addConvolutionalLayer(nFeatures, filterSize, filterStride, activationFn,
                        dropout, minActiveInputs, fmpShrink);
  if (fmpShrink > 1) {
    std::cout << layers.size() << ":";
    layers.push_back(new FractionalMaxPoolingLayer(
        memStream, (FmpKind)kind, poolSize, fmpShrink, dimension));
  }
}
void SparseConvNetCUDA::addLeNetLayerMP(int nFeatures, int filterSize,
                                        int filterStride, int poolSize,
                                        int poolStride,
                                        ActivationFunction activationFn,
                                        float dropout, int minActiveInputs) {
  addConvolutionalLayer(nFeatures, filterSize, filterStride, activationFn,
                        dropout, minActiveInputs, poolSize);
  if (poolSize > 1) {
    std::cout << layers.size() << ":";
    layers.push_back(
        new MaxPoolingLayer(memStream, poolSize, poolStride, dimension));
  }
}
void SparseConvNetCUDA::addTriangularConvolutionalLayer(
    int nFeatures, int filterSize, int filterStride,
    ActivationFunction activationFn, float dropout, int minActiveInputs,
    float poolingToFollow) {
  if (filterSize > 1) {
    std::cout << layers.size() << ":";
    layers.push_back(new ConvolutionalTriangularLayer(
        memStream, filterSize, filterStride, dimension, nOutputFeatures,
        minActiveInputs));
    nOutputFeatures *= triangleSize(filterSize, dimension);
  }
  addLearntLayer(nFeatures, activationFn, dropout,
                 powf(filterSize * 1.0 / filterStride / poolingToFollow, 2));
}
// The reference hands (.., dropout, poolSize, minActiveInputs) to a callee
// whose parameters are (.., dropout, minActiveInputs, poolingToFollow)
// (SparseConvNetCUDA.cu:165-168 against :183-185): through this builder the
// convolution's minActiveInputs is the pool size.  Kept, because nets built
// with the reference behave that way.
void SparseConvNetCUDA::addTriangularLeNetLayerMP(
    int nFeatures, int filterSize, int filterStride, int poolSize,
    int poolStride, ActivationFunction activationFn, float dropout,
    int minActiveInputs) {
  addTriangularConvolutionalLayer(nFeatures, filterSize, filterStride,
                                  activationFn, dropout, poolSize,
                                  minActiveInputs);
  if (poolSize > 1) {
    std::cout << layers.size() << ":";
    layers.push_back(new MaxPoolingTriangularLayer(memStream, poolSize,
                                                   poolStride, dimension));
  }
}
void SparseConvNetCUDA::addTerminalPoolingLayer(int poolSize, int S) {
  std::cout << layers.size() << ":";
  layers.push_back(new TerminalPoolingLayer(memStream, poolSize, S));
}
// SparseConvNetCUDA.cu:198-210: classifier, then the spatial sizes are worked
// out from the top (size 1) down to the input field
void SparseConvNetCUDA::addSoftmaxLayer() {
  addLearntLayer(nClasses, SOFTMAX, 0.0f, 1);
  inputSpatialSize = 1;
  std::cout << "Spatially sparse CNN with layer sizes: " << inputSpatialSize;
  for (int i = (int)layers.size() - 1; i >= 0; i--)
    inputSpatialSize = layers[i]->calculateInputSpatialSize(inputSpatialSize);
  std::cout << std::endl;
  std::cout << "Input-field dimensions = " << inputSpatialSize;
  for (int i = 1; i < dimension; ++i)
    std::cout << "x" << inputSpatialSize;
  std::cout << std::endl;
}
void SparseConvNetCUDA::setFusedConvolutions(bool on) {
  for (size_t i = 0; i + 1 < layers.size(); ++i) {
    int nOut = 0;
    if (auto *n = dynamic_cast<NetworkInNetworkLayer *>(layers[i + 1]))
      nOut = n->nFeaturesOut;
    else if (auto *n = dynamic_cast<NetworkInNetworkPReLULayer *>(layers[i + 1]))
      nOut = n->nFeaturesOut;
    if (auto *c = dynamic_cast<ConvolutionalLayer *>(layers[i]))
      c->deferGather =
          on && nOut > 0 &&
          scn_conv_nin_supported(c->nFeaturesOut / c->nFeaturesIn,
                                 c->nFeaturesIn, nOut);
    if (auto *c = dynamic_cast<ConvolutionalTriangularLayer *>(layers[i]))
      c->deferGather =
          on && nOut > 0 &&
          scn_conv_nin_supported(c->nFeaturesOut / c->nFeaturesIn,
                                 c->nFeaturesIn, nOut);
  }
}
void SparseConvNetCUDA::ensureInterfaces() {
  // one shared sub-interface per depth, one interface per depth and slot
  // (BatchProducer.cu:28-33)
  while (batchPool[0].interfaces.size() <= layers.size()) {
    sharedSubInterfaces.push_back(new SpatiallySparseBatchSubInterface());
    for (auto &slot : batchPool)
      slot.interfaces.emplace_back(sharedSubInterfaces.back());
  }
  // ... and one more set per forward lane beyond the first
  laneSubInterfaces.resize(laneStreams.size());
  for (auto &lane : laneSubInterfaces)
    while (lane.size() < sharedSubInterfaces.size())
      lane.push_back(new SpatiallySparseBatchSubInterface());
}
// every grids object the slot owns, emptied in one launch at the start of a batch
static void clearDeviceGrids(scn_ctx *ctx, SpatiallySparseBatch &b) {
  std::vector<scn_grids *> owned;
  for (auto &iface : b.interfaces)
    if (iface.deviceGrids && iface.ownsDeviceGrids)
      owned.push_back(iface.deviceGrids);
  if (!owned.empty())
    SCN_CHECKED(scn_grids_clear_many(ctx, owned.data(), (int)owned.size()));
}
// Every layer's rule book for the batch in slot b, on ctx's stream.  First with
// deferred counts: no host round trip per layer, sizes are upper bounds until
// one scn_rules_settle at the end, after which the real sizes are put in
// place.  A batch that outgrows the bounds (or the first batch of a slot, which
// has no bounds yet: its plans simply wait) is planned again the exact way.
static void buildRuleBooks(SparseConvNetCUDA &cnn, scn_ctx *ctx,
                           SpatiallySparseBatch &b) {
  auto all = [&]() {
    for (size_t i = 0; i < cnn.layers.size(); i++) {
      scn_prof_tag(ctx, (int)i);
      cnn.layers[i]->preprocess(b, b.interfaces[i], b.interfaces[i + 1]);
    }
  };
  // (plans that continue from one another are recorded and run together)
  SCN_CHECKED(scn_ctx_defer_counts(ctx, 1));
  SCN_CHECKED(scn_ctx_chain_rules(ctx, cnn.chainRuleBooks ? 1 : 0));
  all();
  SCN_CHECKED(scn_ctx_chain_rules(ctx, 0));
  SCN_CHECKED(scn_ctx_defer_counts(ctx, 0));
  const int rc = scn_rules_settle(ctx);
  if (rc == SCN_ERR_CAPACITY) {
    all(); // every plan empties its own output tables again
    return;
  }
  SCN_CHECKED(rc);
  // real sizes: a layer that owns its grids asks them, the others inherit
  for (size_t i = 0; i < cnn.layers.size(); i++) {
    SpatiallySparseBatchInterface &in = b.interfaces[i], &out = b.interfaces[i + 1];
    if (out.ownsDeviceGrids && out.deviceGrids) {
      int32_t nSites = 0;
      int64_t width = 0;
      SCN_CHECKED(scn_grids_info(out.deviceGrids, nullptr, nullptr, nullptr,
                                 nullptr, &nSites));
      SCN_CHECKED(scn_rules_width(out.deviceGrids, &width));
      out.nSpatialSites = nSites;
      out.rules.resize64((size_t)nSites * (size_t)width);
    } else {
      out.nSpatialSites = in.nSpatialSites;
    }
  }
}
// Host-resident input of at least this many bytes is uploaded by the copy
// engine rather than read over the bus by the kernels that use it.
static const size_t kCopyEngineBytes = 4u << 20;
void SparseConvNetCUDA::preprocessResident(int cc, const ResidentBatch &input) {
  SpatiallySparseBatch &b = batchPool[cc];
  scn_ctx *ctx = b.preprocessStream ? b.preprocessStream->ctx : memStream.ctx;
  b.reset();
  b.type = UNLABELEDBATCH;
  b.batchSize = input.batchSize;
  SpatiallySparseBatchInterface &in = b.interfaces[0];
  in.nFeatures = nInputFeatures;
  in.spatialSize = inputSpatialSize;
  in.nSpatialSites = input.nSpatialSites;
  in.featuresPresent.hVector() = range(nInputFeatures);
  if (!in.deviceGrids) {
    SCN_CHECKED(scn_grids_create(ctx, &in.deviceGrids));
    in.ownsDeviceGrids = true;
  }
  scn_prof_tag(ctx, -1);
  clearDeviceGrids(ctx, b);
  const int32_t *d_sample = input.d_sample, *d_row = input.d_row,
                *d_background = input.d_background;
  const int64_t *d_key = input.d_key;
  // input.onHost: the arrays are pinned host memory (the upload of
  // BatchProducer.cu:127-134, on this slot's stream).  A small batch is read
  // over the bus by the grid-building kernel and the copy below themselves,
  // which costs no launch of its own.  A large one goes through the copy
  // engine into this slot's staging first: kernels that wait for the bus
  // would hold the wavefront slots that the other batches' layers need for as
  // long as the transfer takes.
  size_t nElems = (size_t)input.nSpatialSites * nInputFeatures;
  const bool byCopyEngine =
      input.onHost &&
      (size_t)input.nActive * 16 + nElems * sizeof(float) >= kCopyEngineBytes;
  if (byCopyEngine) {
    const size_t n = (size_t)input.nActive;
    b.stagingSample.resize64(n);
    b.stagingKey.resize64(2 * n);
    b.stagingRow.resize64(n);
    SCN_CHECKED(scn_h2d_async(ctx, b.stagingSample.dPtr(), d_sample, n * 4));
    SCN_CHECKED(scn_h2d_async(ctx, b.stagingKey.dPtr(), d_key, n * 8));
    SCN_CHECKED(scn_h2d_async(ctx, b.stagingRow.dPtr(), d_row, n * 4));
    d_sample = b.stagingSample.dPtr();
    d_key = (const int64_t *)b.stagingKey.dPtr();
    d_row = b.stagingRow.dPtr();
  }
  SCN_CHECKED(scn_grids_build(ctx, in.deviceGrids, input.batchSize, dimension,
                              in.spatialSize, d_sample, d_key, d_row,
                              input.nActive, d_background,
                              input.nSpatialSites));
  in.sub->features.copyToGPU();
  in.sub->features.resize64(nElems);
  if (byCopyEngine)
    SCN_CHECKED(scn_h2d_async(ctx, in.sub->features.dPtr(), input.d_features,
                              nElems * sizeof(float)));
  else
    SCN_CHECKED(scn_copy(ctx, in.sub->features.dPtr(), input.d_features,
                         nElems * sizeof(float)));
  buildRuleBooks(*this, ctx, b);
  SCN_CHECKED(scn_sync(ctx));
}
void SparseConvNetCUDA::setPrecision(int precision) {
  for (auto *l : layers) {
    if (auto *n = dynamic_cast<NetworkInNetworkLayer *>(l))
      n->precision = precision;
    if (auto *n = dynamic_cast<NetworkInNetworkPReLULayer *>(l))
      n->precision = precision;
  }
}
// SparseConvNetCUDA.cu:227-271, forward branch
void SparseConvNetCUDA::processBatch(SpatiallySparseBatch &batch,
                                     float learningRate, float momentum,
                                     std::ofstream &f, std::ofstream &g) {
  forwardBatch(batch);
  if (batch.type == TRAINBATCH)
    backwardBatch(batch, learningRate, momentum);
  finishBatch(batch, f, g);
}
// The training half of processBatch (SparseConvNetCUDA.cu:248-252): the
// classifier has left d cost / d soft-max input in the top interface; every
// layer, last to first, hands the gradient down and updates its weights.
void SparseConvNetCUDA::backwardBatch(SpatiallySparseBatch &batch,
                                      float learningRate, float momentum) {
  for (int i = (int)layers.size() - 1; i >= 0; i--) {
    scn_prof_tag(memStream.ctx, i);
    layers[i]->backwards(batch, batch.interfaces[i], batch.interfaces[i + 1],
                         learningRate, momentum);
  }
  // the backward kernels read the slot's rule books and features: the slot
  // stays with the consumer until the stream has passed this point
  BatchResultStage &r = *batch.result;
  if (!r.consumed)
    SCN_CHECKED(scn_event_create(memStream.ctx, &r.consumed));
  SCN_CHECKED(scn_event_record(memStream.ctx, r.consumed));
  r.consumedPending = true;
}
// The two halves of processBatch.  forwardBatch only queues work on the net's
// stream (every layer, then the copy of the probabilities to the host);
// finishBatch waits for that copy and does the host-side statistics.  The
// dataset loops queue batch i + 1 before finishing batch i, so the stream never
// runs dry while the host is busy.
void SparseConvNetCUDA::forwardBatch(SpatiallySparseBatch &batch, int lane) {
  assert(lane >= 0 && lane < nForwardLanes);
  assert(lane == 0 || (batch.type != TRAINBATCH && batch.type != RESCALEBATCH));
  // the lane's stream and feature buffers
  cudaMemStream &ms = laneStream(lane);
  batch.forwardStream = lane == 0 ? nullptr : &ms;
  for (size_t i = 0; i < layers.size(); i++)
    batch.interfaces[i + 1].sub =
        lane == 0 ? sharedSubInterfaces[i] : laneSubInterfaces[lane - 1][i];
  // a RESCALEBATCH rescales every layer's weights right after its forward
  // pass (SparseConvNetCUDA.cu:230-241)
  float scalingUnderneath = 1;
  for (size_t i = 0; i < layers.size(); i++) {
    batch.interfaces[i + 1].sub->reset();
    scn_prof_tag(ms.ctx, (int)i);
    layers[i]->forwards(batch, batch.interfaces[i], batch.interfaces[i + 1]);
    if (batch.type == RESCALEBATCH) {
      std::cout << i << ":"
                << batch.interfaces[i].sub->features.size64() * sizeof(float) /
                       (1 << 20)
                << "MB ";
      layers[i]->scaleWeights(batch.interfaces[i], batch.interfaces[i + 1],
                              scalingUnderneath, i == layers.size() - 1);
    }
  }
  SoftmaxClassifierLaunch(batch.interfaces.back(), batch, ms);
}
void SparseConvNetCUDA::finishBatch(SpatiallySparseBatch &batch,
                                    std::ofstream &f, std::ofstream &g) {
  SoftmaxClassifierCollect(batch.interfaces.back(), batch, nTop);
  if (batch.result->consumedPending) {
    SCN_CHECKED(scn_event_wait(batch.result->consumed));
    batch.result->consumedPending = false;
  }
  if (f.is_open())
    for (auto &p : batch.predictions) {
      for (size_t k = 0; k < p.size(); k++)
        f << (k ? " " : "") << p[k];
      f << std::endl;
    }
  if (g.is_open())
    for (auto &p : batch.probabilities) {
      for (size_t k = 0; k < p.size(); k++)
        g << (k ? " " : "") << p[k];
      g << std::endl;
    }
}
static void printThroughput(long long nanoseconds, size_t nPictures) {
  std::cout << " MegaMultiplyAdds/sample:"
            << roundf(multiplyAddCount / nPictures / 1000000)
            << " time:" << nanoseconds / 1000000000L
            << "s GigaMultiplyAdds/s:" << roundf(multiplyAddCount / nanoseconds)
            << " rate:" << roundf(nPictures * 1000000000.0f / nanoseconds)
            << "/s" << std::endl;
}
ForwardQueue::ForwardQueue(SparseConvNetCUDA &cnn, BatchProducer &bp,
                           bool training)
    : cnn(cnn), count(0) {
  lanes = training ? 1 : cnn.nForwardLanes;
  // a batch stays queued while up to `depth` younger ones are queued behind
  // it; each of them holds a slot, and the producers need one to work in
  depth = std::min(lanes, cnn.nBatchProducerThreads - 1);
  if (depth < lanes)
    lanes = std::max(1, depth);
  bp.keepAlive = depth;
  if (lanes > 1)
    for (int lane = 0; lane < lanes; ++lane) {
      workers.emplace_back(new Worker());
      workers.back()->thread = std::thread(&ForwardQueue::work, this, lane);
    }
}
ForwardQueue::~ForwardQueue() {
  for (auto &w : workers) {
    {
      std::lock_guard<std::mutex> lock(w->m);
      w->stop = true;
    }
    w->cv.notify_all();
    w->thread.join();
  }
}
void ForwardQueue::work(int lane) {
  Worker &w = *workers[lane];
  for (;;) {
    SpatiallySparseBatch *b = nullptr;
    {
      std::unique_lock<std::mutex> lock(w.m);
      w.cv.wait(lock, [&] { return w.stop || !w.todo.empty(); });
      if (w.todo.empty())
        return; // (stop is only set once everything queued has been popped)
      b = w.todo.front();
      w.todo.erase(w.todo.begin());
    }
    cnn.forwardBatch(*b, lane);
    b->result->enqueued.store(true, std::memory_order_release);
  }
}
SpatiallySparseBatch *ForwardQueue::push(SpatiallySparseBatch *b) {
  const int lane = count++ % lanes;
  if (workers.empty()) {
    cnn.forwardBatch(*b, lane);
  } else {
    b->result->enqueued.store(false, std::memory_order_relaxed);
    Worker &w = *workers[lane];
    {
      std::lock_guard<std::mutex> lock(w.m);
      w.todo.push_back(b);
    }
    w.cv.notify_one();
  }
  inFlight.push_back(b);
  if ((int)inFlight.size() > depth)
    return pop();
  return nullptr;
}
SpatiallySparseBatch *ForwardQueue::pop() {
  if (inFlight.empty())
    return nullptr;
  SpatiallySparseBatch *b = inFlight.front();
  inFlight.erase(inFlight.begin());
  // its forward pass may still be on its way into the lane's stream
  while (!b->result->enqueued.load(std::memory_order_acquire))
    std::this_thread::yield();
  return b;
}
// SparseConvNetCUDA.cu:272-326
float SparseConvNetCUDA::processDataset(SpatiallySparseDataset &dataset,
                                        int batchSize, float learningRate,
                                        float momentum) {
  assert(dataset.pictures.size() > 0);
  float errorRate = 0, nll = 0;
  multiplyAddCount = 0;
  auto start = std::chrono::system_clock::now();
  std::ofstream f, g;
  BatchProducer bp(*this, dataset, inputSpatialSize, batchSize);
  if (dataset.type == UNLABELEDBATCH) {
    f.open("unlabelledData.predictions");
    g.open("unlabelledData.probabilities");
  }
  const bool oneLane = dataset.type == TRAINBATCH || dataset.type == RESCALEBATCH;
  ForwardQueue queue(*this, bp, oneLane);
  SpatiallySparseBatch *trainQueued = nullptr; // training batch queued, not yet read
  auto finish = [&](SpatiallySparseBatch *batch) {
    finishBatch(*batch, f, g);
    errorRate += batch->mistakes * 1.0 / dataset.pictures.size();
    nll += batch->negativeLogLikelihood * 1.0 / dataset.pictures.size();
  };
  while (SpatiallySparseBatch *batch = bp.nextBatch()) {
    SpatiallySparseBatch *due = nullptr;
    if (batch->type == TRAINBATCH) {
      forwardBatch(*batch);
      backwardBatch(*batch, learningRate, momentum);
      // (one training batch may stay queued while the next is produced)
      due = trainQueued;
      trainQueued = batch;
      if (!bp.keepAlive) {
        due = batch;
        trainQueued = nullptr;
      }
    } else {
      due = queue.push(batch);
    }
    if (due)
      finish(due);
  }
  if (trainQueued)
    finish(trainQueued);
  while (SpatiallySparseBatch *batch = queue.pop())
    finish(batch);
  auto end = std::chrono::system_clock::now();
  auto diff =
      std::chrono::duration_cast<std::chrono::nanoseconds>(end - start).count();
  if (dataset.type != RESCALEBATCH) { // SparseConvNetCUDA.cu:311
    std::cout << dataset.name;
    if (dataset.type != UNLABELEDBATCH)
      std::cout << " Mistakes:" << 100.0 * errorRate << "% NLL:" << nll;
    printThroughput(diff, dataset.pictures.size());
  }
  return nll;
}
// SparseConvNetCUDA.cu:507-538
void SparseConvNetCUDA::processDatasetDumpTopLevelFeatures(
    SpatiallySparseDataset &dataset, int batchSize, int reps) {
  assert(dataset.pictures.size() > 0);
  assert(dataset.type != TRAINBATCH);
  std::ofstream f((dataset.name + ".features").c_str());
  const size_t n = layers.size();
  for (int rep = 0; rep < reps; rep++) {
    BatchProducer bp(*this, dataset, inputSpatialSize, batchSize);
    while (SpatiallySparseBatch *batch = bp.nextBatch()) {
      for (size_t i = 0; i + 1 < n; i++) {
        batch->interfaces[i + 1].sub->reset();
        layers[i]->forwards(*batch, batch->interfaces[i], batch->interfaces[i + 1]);
      }
      SpatiallySparseBatchInterface &top = batch->interfaces[n - 1];
      assert(top.nFeatures == (int)top.featuresPresent.size());
      assert(!top.deferredGatherFrom); // (a convolution is never the last-but-one layer's output here)
      std::vector<float> &v = top.sub->features.hVector(); // waits for the stream
      std::vector<int> &labels = batch->labels.hVector();
      for (int i = 0; i < batch->batchSize; i++) {
        f << batch->sampleNumbers[i] << " " << labels[i];
        for (int j = 0; j < top.nFeatures; j++)
          f << " " << v[(size_t)i * top.nFeatures + j];
        f << std::endl;
      }
    }
  }
}
// SparseConvNetCUDA.cu:540-566
void SparseConvNetCUDA::calculateInputRegularizingConstants(
    SpatiallySparseDataset dataset) { // a copy of the dataset
  inputNormalizingConstants.resize(0); // no rescaling while measuring
  std::cout << "Using " << std::min(10000, (int)dataset.pictures.size())
            << " out of " << dataset.pictures.size()
            << " training samples to calculate regularizing constants."
            << std::endl;
  if (dataset.pictures.size() > 10000)
    dataset.pictures.resize(10000);
  dataset.type = TESTBATCH; // no dropout, no augmentation
  std::vector<float> c(nInputFeatures, 0);
  {
    BatchProducer bp(*this, dataset, inputSpatialSize, 100);
    while (SpatiallySparseBatch *batch = bp.nextBatch()) {
      std::vector<float> &features = batch->interfaces[0].sub->features.hVector();
      for (size_t i = 0; i < features.size(); ++i)
        c[i % nInputFeatures] =
            std::max(c[i % nInputFeatures], std::fabs(features[i]));
    }
  }
  for (int i = 0; i < nInputFeatures; ++i) {
    inputNormalizingConstants.push_back(c[i] > 0 ? 1.0f / c[i] : 0);
    std::cout << inputNormalizingConstants.back() << " ";
  }
  std::cout << std::endl;
}
// SparseConvNetCUDA.cu:327-405: nReps forward passes, probabilities averaged
void SparseConvNetCUDA::processDatasetRepeatTest(
    SpatiallySparseDataset &dataset, int batchSize, int nReps,
    std::string predictionsFilename, std::string confusionMatrixFilename) {
  assert(dataset.pictures.size() > 0);
  multiplyAddCount = 0;
  auto start = std::chrono::system_clock::now();
  const size_t nPictures = dataset.pictures.size();
  std::vector<std::vector<int>> votes(nPictures,
                                      std::vector<int>(dataset.nClasses));
  std::vector<std::vector<float>> probs(nPictures,
                                        std::vector<float>(dataset.nClasses));
  for (int rep = 1; rep <= nReps; ++rep) {
    {
      BatchProducer bp(*this, dataset, inputSpatialSize, batchSize);
      ForwardQueue queue(*this, bp, false);
      auto finish = [&](SpatiallySparseBatch *batch) {
        std::ofstream f, g;
        finishBatch(*batch, f, g);
        for (int i = 0; i < batch->batchSize; ++i) {
          int ii = batch->sampleNumbers[i];
          votes[ii][batch->predictions[i][0]]++;
          for (int j = 0; j < dataset.nClasses; ++j)
            probs[ii][j] += batch->probabilities[i][j];
        }
      };
      while (SpatiallySparseBatch *batch = bp.nextBatch())
        if (SpatiallySparseBatch *due = queue.push(batch))
          finish(due);
      while (SpatiallySparseBatch *batch = queue.pop())
        finish(batch);
    }
    int errors = (int)nPictures;
    float nll = 0;
    if (dataset.type != UNLABELEDBATCH)
      for (size_t i = 0; i < nPictures; ++i) {
        std::vector<int> predictions = vectorTopIndices(probs[i], nTop);
        for (int j = 0; j < nTop; j++)
          if (predictions[j] == dataset.pictures[i]->label)
            errors--;
        nll -= log(std::max(probs[i][dataset.pictures[i]->label] / rep,
                            (float)1.0e-15));
      }
    if (!predictionsFilename.empty()) {
      std::cout << predictionsFilename << std::endl;
      std::ofstream f(predictionsFilename.c_str());
      if (!dataset.header.empty())
        f << dataset.header << std::endl;
      for (size_t i = 0; i < nPictures; ++i) {
        f << dataset.pictures[i]->identify();
        if (dataset.type != UNLABELEDBATCH)
          f << "," << dataset.pictures[i]->label;
        for (int j = 0; j < dataset.nClasses; ++j)
          f << "," << probs[i][j] / rep;
        f << std::endl;
      }
    }
    if (!confusionMatrixFilename.empty() && dataset.type != UNLABELEDBATCH) {
      std::vector<float> cm((size_t)dataset.nClasses * dataset.nClasses);
      for (size_t i = 0; i < nPictures; ++i)
        for (int j = 0; j < dataset.nClasses; ++j)
          cm[dataset.pictures[i]->label * dataset.nClasses + j] +=
              probs[i][j] / rep;
      std::ofstream f(confusionMatrixFilename.c_str());
      for (int i = 0; i < dataset.nClasses; ++i) {
        for (int j = 0; j < dataset.nClasses; ++j)
          f << cm[i * dataset.nClasses + j] << " ";
        f << std::endl;
      }
    }
    auto end = std::chrono::system_clock::now();
    auto diff = std::chrono::duration_cast<std::chrono::nanoseconds>(end - start)
                    .count();
    std::cout << dataset.name << " rep " << rep << "/" << nReps;
    if (dataset.type != UNLABELEDBATCH)
      std::cout << " Mistakes: " << 100.0 * errors / nPictures << "% NLL "
                << nll / nPictures;
    printThroughput(diff, nPictures);
  }
}
// raw little-endian fp32, no header (SparseConvNetCUDA.cu:406-442)
void SparseConvNetCUDA::loadWeights(std::string baseName, int epoch,
                                    bool momentum, int firstNlayers) {
  std::string filename = baseName + "_epoch-" + std::to_string(epoch) + ".cnn";
  std::ifstream f(filename.c_str(), std::ios::in | std::ios::binary);
  if (!f) {
    std::cout << "Cannot find " << filename << std::endl;
    scnExit(EXIT_FAILURE);
  }
  std::cout << "Loading network parameters from " << filename << std::endl;
  for (int i = 0; i < std::min((int)layers.size(), firstNlayers); i++)
    layers[i]->loadWeightsFromStream(f, momentum);
  if (inputNormalizingConstants.size() > 0)
    f.read((char *)&inputNormalizingConstants[0],
           sizeof(float) * inputNormalizingConstants.size());
}
void SparseConvNetCUDA::saveWeights(std::string baseName, int epoch,
                                    bool momentum) {
  std::string filename = baseName + "_epoch-" + std::to_string(epoch) + ".cnn";
  std::ofstream f(filename.c_str(), std::ios::binary);
  if (!f) {
    std::cout << "Cannot write " << filename << std::endl;
    scnExit(EXIT_FAILURE);
  }
  for (auto *l : layers)
    l->putWeightsToStream(f, momentum);
  if (inputNormalizingConstants.size() > 0)
    f.write((char *)&inputNormalizingConstants[0],
            sizeof(float) * inputNormalizingConstants.size());
}

// ========================================================== batch producer
SpatiallySparseDataset BatchProducer::emptyDataset;

BatchProducer::BatchProducer(SparseConvNetCUDA &cnn,
                             SpatiallySparseDataset &dataset, int spatialSize,
                             int batchSize)
    : cnn(cnn), batchCounter(-1), dataset(dataset), batchSize(batchSize),
      spatialSize(spatialSize), stopping(false) {
  assert(batchSize > 0);
  nBatches = ((int)dataset.pictures.size() + batchSize - 1) / batchSize;
  permutation = range((int)dataset.pictures.size());
  if (dataset.type == TRAINBATCH && cnn.shuffleTrainingData) {
    RNG rng; // BatchProducer.cu:23-26
    rng.vectorShuffle(permutation);
  }
  start();
}
BatchProducer::BatchProducer(SparseConvNetCUDA &cnn,
                             const ResidentBatch &residentBatch, int nBatches)
    : BatchProducer(cnn, std::vector<ResidentBatch>(1, residentBatch), nBatches) {}
BatchProducer::BatchProducer(SparseConvNetCUDA &cnn,
                             const std::vector<ResidentBatch> &residentBatches,
                             int nBatches)
    : cnn(cnn), batchCounter(-1), nBatches(nBatches), dataset(emptyDataset),
      batchSize(residentBatches.at(0).batchSize),
      spatialSize(cnn.inputSpatialSize), residents(residentBatches),
      stopping(false) {
  start();
}
void BatchProducer::start() {
  cnn.ensureInterfaces();
  slotFull.assign(cnn.nBatchProducerThreads, 0);
  for (int c = 0; c < cnn.nBatchProducerThreads; c++)
    cnn.batchPool[c].batchSize = 0;
  for (int nThread = 0; nThread < cnn.nBatchProducerThreads; ++nThread)
    workers.emplace_back(&BatchProducer::batchProducerThread, this, nThread);
}
BatchProducer::~BatchProducer() {
  {
    std::lock_guard<std::mutex> lock(slotMutex);
    stopping = true;
  }
  slotChanged.notify_all();
  for (auto &w : workers)
    if (w.joinable())
      w.join();
}
// CPU half of BatchProducer.cu:40-87: distort, codify, normalise
void BatchProducer::preprocessBatch(int c, int cc, RNG &rng) {
  SpatiallySparseBatch &b = cnn.batchPool[cc];
  b.reset();
  b.type = dataset.type;
  SpatiallySparseBatchInterface &in = b.interfaces[0];
  in.nFeatures = dataset.nFeatures;
  in.spatialSize = spatialSize;
  in.featuresPresent.hVector() = range(dataset.nFeatures);
  const int last = std::min((c + 1) * batchSize, (int)dataset.pictures.size());
  for (int i = c * batchSize; i < last; i++) {
    Picture *pic = dataset.pictures[permutation[i]]->distort(rng, dataset.type);
    b.sampleNumbers.push_back(permutation[i]);
    b.batchSize++;
    in.grids.push_back(SparseGrid());
    b.labels.hVector().push_back(pic->label);
    pic->codifyInputData(in.grids.back(), in.sub->features.hVector(),
                         in.nSpatialSites, in.spatialSize);
    if (pic != dataset.pictures[permutation[i]])
      delete pic;
  }
  assert(in.sub->features.size64() ==
         (size_t)in.nFeatures * (size_t)in.nSpatialSites);
  if (cnn.inputNormalizingConstants.size() > 0) {
    std::vector<float> &features = in.sub->features.hVector();
    for (size_t i = 0; i < features.size(); ++i)
      features[i] *= cnn.inputNormalizingConstants[i % in.nFeatures];
  }
  // The grids as the four arrays scn_grids_build takes, and the features, in
  // the slot's pinned staging: still on the CPU's time, no stream is held yet,
  // and the upload is then five queued copies.
  size_t n = 0;
  for (auto &g : in.grids)
    n += g.mp.size();
  b.hostSample.reserve(n * sizeof(int32_t));
  b.hostKey.reserve(n * sizeof(int64_t));
  b.hostRow.reserve(n * sizeof(int32_t));
  b.hostBackground.reserve((size_t)b.batchSize * sizeof(int32_t));
  int32_t *sample = b.hostSample.as<int32_t>(), *row = b.hostRow.as<int32_t>(),
          *bg = b.hostBackground.as<int32_t>();
  int64_t *key = b.hostKey.as<int64_t>();
  size_t at = 0;
  for (int item = 0; item < b.batchSize; ++item) {
    bg[item] = in.grids[item].backgroundCol;
    for (auto &e : in.grids[item].mp.entries()) {
      sample[at] = item;
      key[at] = e.first;
      row[at] = e.second;
      ++at;
    }
  }
  b.hostSites = n;
  std::vector<float> &features = in.sub->features.hVector();
  b.hostFeatureCount = features.size();
  b.hostFeatures.reserve(features.size() * sizeof(float));
  if (!features.empty())
    std::memcpy(b.hostFeatures.p, features.data(), features.size() * sizeof(float));
  features.clear();
}
// GPU half: the input grids go to HBM, then every layer builds its rule book,
// all on the slot's stream
void BatchProducer::preprocessBatchOnDevice(int cc) {
  SpatiallySparseBatch &b = cnn.batchPool[cc];
  SpatiallySparseBatchInterface &in = b.interfaces[0];
  cudaMemStream &ms = b.preprocessStream ? *b.preprocessStream : cnn.memStream;
  scn_ctx *ctx = ms.ctx;
  // (flattened into pinned memory by preprocessBatch)
  const size_t n = b.hostSites;
  b.stagingSample.resize64(n);
  b.stagingKey.resize64(2 * n);
  b.stagingRow.resize64(n);
  b.stagingBackground.resize64((size_t)b.batchSize);
  SCN_CHECKED(scn_h2d_async(ctx, b.stagingSample.dPtr(), b.hostSample.p, n * 4));
  SCN_CHECKED(scn_h2d_async(ctx, b.stagingKey.dPtr(), b.hostKey.p, n * 8));
  SCN_CHECKED(scn_h2d_async(ctx, b.stagingRow.dPtr(), b.hostRow.p, n * 4));
  SCN_CHECKED(scn_h2d_async(ctx, b.stagingBackground.dPtr(), b.hostBackground.p,
                            (size_t)b.batchSize * 4));
  if (!in.deviceGrids) {
    SCN_CHECKED(scn_grids_create(ctx, &in.deviceGrids));
    in.ownsDeviceGrids = true;
  }
  scn_prof_tag(ctx, -1);
  clearDeviceGrids(ctx, b);
  SCN_CHECKED(scn_grids_build(ctx, in.deviceGrids, b.batchSize, cnn.dimension,
                              in.spatialSize, b.stagingSample.dPtr(),
                              (const int64_t *)b.stagingKey.dPtr(),
                              b.stagingRow.dPtr(), (int64_t)n,
                              b.stagingBackground.dPtr(), in.nSpatialSites));
  in.sub->features.copyToGPU(); // (its host vector is empty: nothing moves)
  in.sub->features.resize64(b.hostFeatureCount);
  SCN_CHECKED(scn_h2d_async(ctx, in.sub->features.dPtr(), b.hostFeatures.p,
                            b.hostFeatureCount * sizeof(float)));
  if (b.type == TRAINBATCH) {
    // the classifier's gradient reads the labels on the device: uploaded here,
    // on this slot's stream, so that the net's stream is never waited for
    b.result->labels = b.labels.hVector();
    b.labels.copyToGPUAsync(ms);
  }
  buildRuleBooks(cnn, ctx, b);
  SCN_CHECKED(scn_sync(ctx));
}
void BatchProducer::batchProducerThread(int nThread) {
  RNG rng;
  for (int c = nThread; c < nBatches; c += cnn.nBatchProducerThreads) {
    {
      std::unique_lock<std::mutex> lock(slotMutex);
      slotChanged.wait(lock, [&] { return stopping || !slotFull[nThread]; });
      if (stopping)
        return;
    }
    {
      std::lock_guard<std::mutex> slot(cnn.batchLock[nThread]);
      const bool resident = !residents.empty();
      if (!resident)
        preprocessBatch(c, nThread, rng); // CPU half
      // GPU half, on a stream borrowed for it
      cudaMemStream *stream = cnn.acquireProducerStream(c);
      cnn.batchPool[nThread].preprocessStream = stream;
      if (resident)
        cnn.preprocessResident(nThread, residents[c % residents.size()]);
      else
        preprocessBatchOnDevice(nThread);
      cnn.releaseProducerStream(stream);
    }
    {
      std::lock_guard<std::mutex> lock(slotMutex);
      slotFull[nThread] = 1;
    }
    slotChanged.notify_all();
  }
}
int BatchProducer::slotsReady() {
  std::lock_guard<std::mutex> lock(slotMutex);
  int n = 0;
  for (char full : slotFull)
    n += full != 0;
  // (slots of batches already handed out stay marked until they are given back)
  const int out = std::min(batchCounter + 1, keepAlive + 1);
  return std::max(0, n - std::max(0, out));
}
SpatiallySparseBatch *BatchProducer::nextBatch() {
  if (batchCounter - keepAlive >= 0) { // hand a finished slot back to its worker
    int cc = (batchCounter - keepAlive) % cnn.nBatchProducerThreads;
    const BatchResultStage &r = *cnn.batchPool[cc].result;
    if (r.pending || r.consumedPending) {
      std::fprintf(stderr, "BatchProducer: slot %d handed back while the net's "
                           "stream may still read it\n", cc);
      scnExit(EXIT_FAILURE);
    }
    cnn.batchPool[cc].batchSize = 0;
    {
      std::lock_guard<std::mutex> lock(slotMutex);
      slotFull[cc] = 0;
    }
    slotChanged.notify_all();
  }
  batchCounter++;
  if (batchCounter >= nBatches) {
    for (auto &w : workers)
      if (w.joinable())
        w.join();
    return NULL;
  }
  int cc = batchCounter % cnn.nBatchProducerThreads;
  {
    std::unique_lock<std::mutex> lock(slotMutex);
    slotChanged.wait(lock, [&] { return slotFull[cc] != 0; });
  }
  return &cnn.batchPool[cc];
}

// ================================================================= facades
SparseConvNet::SparseConvNet(int dimension, int nInputFeatures, int nClasses,
                             int pciBusID, int nTop)
    : cnn(new SparseConvNetCUDA(dimension, nInputFeatures, nClasses, pciBusID,
                                nTop)) {}
SparseConvNet::~SparseConvNet() {}
void SparseConvNet::addLeNetLayerMP(int nFeatures, int filterSize,
                                    int filterStride, int poolSize,
                                    int poolStride,
                                    ActivationFunction activationFn,
                                    float dropout, int minActiveInputs) {
  cnn->addLeNetLayerMP(nFeatures, filterSize, filterStride, poolSize,
                       poolStride, activationFn, dropout, minActiveInputs);
}
void SparseConvNet::addLeNetLayerPOFMP(int nFeatures, int filterSize,
                                       int filterStride, int poolSize,
                                       float fmpShrink,
                                       ActivationFunction activationFn,
                                       float dropout, int minActiveInputs) {
  cnn->addLeNetLayerFMP(FMP_PSEUDORANDOM_OVERLAPPING, nFeatures, filterSize, filterStride, poolSize,
                        fmpShrink, activationFn, dropout, minActiveInputs);
}
void SparseConvNet::addLeNetLayerROFMP(int nFeatures, int filterSize,
                                       int filterStride, int poolSize,
                                       float fmpShrink,
                                       ActivationFunction activationFn,
                                       float dropout, int minActiveInputs) {
  cnn->addLeNetLayerFMP(FMP_RANDOM_OVERLAPPING, nFeatures, filterSize, filterStride, poolSize,
                        fmpShrink, activationFn, dropout, minActiveInputs);
}
void SparseConvNet::addLeNetLayerPDFMP(int nFeatures, int filterSize,
                                       int filterStride, int poolSize,
                                       float fmpShrink,
                                       ActivationFunction activationFn,
                                       float dropout, int minActiveInputs) {
  cnn->addLeNetLayerFMP(FMP_PSEUDORANDOM_NONOVERLAPPING, nFeatures, filterSize, filterStride, poolSize,
                        fmpShrink, activationFn, dropout, minActiveInputs);
}
void SparseConvNet::addLeNetLayerRDFMP(int nFeatures, int filterSize,
                                       int filterStride, int poolSize,
                                       float fmpShrink,
                                       ActivationFunction activationFn,
                                       float dropout, int minActiveInputs) {
  cnn->addLeNetLayerFMP(FMP_RANDOM_NONOVERLAPPING, nFeatures, filterSize, filterStride, poolSize,
                        fmpShrink, activationFn, dropout, minActiveInputs);
}
void SparseConvNet::addTerminalPoolingLayer(int poolSize) {
  cnn->addTerminalPoolingLayer(poolSize, ipow(poolSize, cnn->dimension));
}
void SparseConvNet::addSoftmaxLayer() { cnn->addSoftmaxLayer(); }
float SparseConvNet::processDataset(SpatiallySparseDataset &dataset,
                                    int batchSize, float learningRate,
                                    float momentum) {
  return cnn->processDataset(dataset, batchSize, learningRate, momentum);
}
void SparseConvNet::processDatasetRepeatTest(
    SpatiallySparseDataset &dataset, int batchSize, int nReps,
    std::string predictionsFilename, std::string confusionMatrixFilename) {
  cnn->processDatasetRepeatTest(dataset, batchSize, nReps, predictionsFilename,
                                confusionMatrixFilename);
}
void SparseConvNet::processDatasetDumpTopLevelFeatures(
    SpatiallySparseDataset &dataset, int batchSize, int reps) {
  cnn->processDatasetDumpTopLevelFeatures(dataset, batchSize, reps);
}
void SparseConvNet::calculateInputRegularizingConstants(
    SpatiallySparseDataset dataset) {
  cnn->calculateInputRegularizingConstants(dataset);
}
void SparseConvNet::loadWeights(std::string baseName, int epoch, bool momentum,
                                int firstNlayers) {
  cnn->loadWeights(baseName, epoch, momentum, firstNlayers);
}
void SparseConvNet::saveWeights(std::string baseName, int epoch,
                                bool momentum) {
  cnn->saveWeights(baseName, epoch, momentum);
}

SparseConvTriangLeNet::SparseConvTriangLeNet(int dimension, int nInputFeatures,
                                             int nClasses, int pciBusID,
                                             int nTop)
    : cnn(new SparseConvNetCUDA(dimension, nInputFeatures, nClasses, pciBusID,
                                nTop)) {}
SparseConvTriangLeNet::~SparseConvTriangLeNet() {}
void SparseConvTriangLeNet::addLeNetLayerMP(int nFeatures, int filterSize,
                                            int filterStride, int poolSize,
                                            int poolStride,
                                            ActivationFunction activationFn,
                                            float dropout,
                                            int minActiveInputs) {
  cnn->addTriangularLeNetLayerMP(nFeatures, filterSize, filterStride, poolSize,
                                 poolStride, activationFn, dropout,
                                 minActiveInputs);
}
void SparseConvTriangLeNet::addTerminalPoolingLayer(int poolSize) {
  cnn->addTerminalPoolingLayer(poolSize,
                               triangleSize(poolSize, cnn->dimension));
}
void SparseConvTriangLeNet::addSoftmaxLayer() { cnn->addSoftmaxLayer(); }
float SparseConvTriangLeNet::processDataset(SpatiallySparseDataset &dataset,
                                            int batchSize, float learningRate,
                                            float momentum) {
  return cnn->processDataset(dataset, batchSize, learningRate, momentum);
}
void SparseConvTriangLeNet::processDatasetRepeatTest(
    SpatiallySparseDataset &dataset, int batchSize, int nReps,
    std::string predictionsFilename, std::string confusionMatrixFilename) {
  cnn->processDatasetRepeatTest(dataset, batchSize, nReps, predictionsFilename,
                                confusionMatrixFilename);
}
void SparseConvTriangLeNet::processDatasetDumpTopLevelFeatures(
    SpatiallySparseDataset &dataset, int batchSize, int reps) {
  cnn->processDatasetDumpTopLevelFeatures(dataset, batchSize, reps);
}
void SparseConvTriangLeNet::calculateInputRegularizingConstants(
    SpatiallySparseDataset dataset) {
  cnn->calculateInputRegularizingConstants(dataset);
}
void SparseConvTriangLeNet::loadWeights(std::string baseName, int epoch,
                                        bool momentum, int firstNlayers) {
  cnn->loadWeights(baseName, epoch, momentum, firstNlayers);
}
void SparseConvTriangLeNet::saveWeights(std::string baseName, int epoch,
                                        bool momentum) {
  cnn->saveWeights(baseName, epoch, momentum);
}

// ============================================================ architectures
// NetworkArchitectures.cpp:3-68
DeepCNet::DeepCNet(int dimension, int l, int k, ActivationFunction fn,
                   int nInputFeatures, int nClasses, float p, int cudaDevice,
                   int nTop)
    : SparseConvNet(dimension, nInputFeatures, nClasses, cudaDevice, nTop) {
  for (int i = 0; i <= l; i++)
    addLeNetLayerMP((i + 1) * k, i == 0 ? 3 : 2, 1, i < l ? 3 : 1,
                    i < l ? 2 : 1, fn, p * i * 1.0f / l);
  addSoftmaxLayer();
}
DeepC2::DeepC2(int dimension, int l, int k, ActivationFunction fn,
               int nInputFeatures, int nClasses, float p, int cudaDevice,
               int nTop)
    : SparseConvNet(dimension, nInputFeatures, nClasses, cudaDevice, nTop) {
  for (int i = 0; i <= l; i++)
    addLeNetLayerMP((i + 1) * k, 2, 1, i < l ? 3 : 1, i < l ? 2 : 1, fn,
                    p * i * 1.0f / l);
  addSoftmaxLayer();
}
DeepCNiN::DeepCNiN(int dimension, int l, int k, ActivationFunction fn,
                   int nInputFeatures, int nClasses, float p, int cudaDevice,
                   int nTop)
    : SparseConvNet(dimension, nInputFeatures, nClasses, cudaDevice, nTop) {
  for (int i = 0; i <= l; i++) {
    addLeNetLayerMP((i + 1) * k, 2, 1, i < l ? 3 : 1, i < l ? 2 : 1, fn,
                    p * i * 1.0f / l);
    addLeNetLayerMP((i + 1) * k, 1, 1, 1, 1, fn, p * i * 1.0f / l);
  }
  addSoftmaxLayer();
}
DeepC2C2::DeepC2C2(int dimension, int l, int k, ActivationFunction fn,
                   int nInputFeatures, int nClasses, float p, int cudaDevice,
                   int nTop)
    : SparseConvNet(dimension, nInputFeatures, nClasses, cudaDevice, nTop) {
  for (int i = 0; i < l; i++) {
    addLeNetLayerMP((i + 1) * k, 2, 1, 1, 1, fn, p * i * 1.0f / l);
    addLeNetLayerMP((i + 1) * k, 2, 1, 3, 2, fn, p * i * 1.0f / l);
  }
  addLeNetLayerMP((l + 1) * k, 2, 1, 1, 1, fn, p);
  addLeNetLayerMP((l + 1) * k, 1, 1, 1, 1, fn, p);
  addSoftmaxLayer();
}
DeepC3C3::DeepC3C3(int dimension, int l, int k, ActivationFunction fn,
                   int nInputFeatures, int nClasses, float p, int cudaDevice,
                   int nTop)
    : SparseConvNet(dimension, nInputFeatures, nClasses, cudaDevice, nTop) {
  for (int i = 0; i < l; i++) {
    addLeNetLayerMP((i + 1) * k, 3, 1, 1, 1, fn, p * i * 1.0f / l);
    addLeNetLayerMP((i + 1) * k, 3, 1, 3, 2, fn, p * i * 1.0f / l);
  }
  addLeNetLayerMP((l + 1) * k, 3, 1, 1, 1, fn, p);
  addLeNetLayerMP((l + 1) * k, 1, 1, 1, 1, fn, p);
  addSoftmaxLayer();
}
DeepC3C3Valid::DeepC3C3Valid(int dimension, int l, int k,
                             ActivationFunction fn, int nInputFeatures,
                             int nClasses, float p, int cudaDevice, int nTop)
    : SparseConvNet(dimension, nInputFeatures, nClasses, cudaDevice, nTop) {
  for (int i = 0; i < l; i++) {
    addLeNetLayerMP((i + 1) * k, 3, 1, 1, 1, fn, p * i * 1.0f / l, -1);
    addLeNetLayerMP((i + 1) * k, 3, 1, 3, 2, fn, p * i * 1.0f / l, -1);
  }
  // one ordinary convolution at the end, in case no site survived
  addLeNetLayerMP((l + 1) * k, 3, 1, 1, 1, fn, p, +1);
  addLeNetLayerMP((l + 1) * k, 1, 1, 1, 1, fn, p);
  addSoftmaxLayer();
}

// NetworkArchitectures.cpp:72-122: l levels of C2 + fractional max-pooling,
// then C2 and a 1x1 NiN, dropout rising to p
#define SCN_FMP_ARCHITECTURE(Name, Builder)                                    \
  Name::Name(int dimension, int l, int k, float fmpShrink,                     \
             ActivationFunction fn, int nInputFeatures, int nClasses, float p, \
             int cudaDevice, int nTop)                                         \
      : SparseConvNet(dimension, nInputFeatures, nClasses, cudaDevice, nTop) { \
    for (int i = 0; i < l; i++)                                                \
      Builder(k * (i + 1), 2, 1, 2, fmpShrink, fn, p * i / (l + 1));           \
    addLeNetLayerMP(k * (l + 1), 2, 1, 1, 1, fn, p * l / (l + 1));             \
    addLeNetLayerMP(k * (l + 2), 1, 1, 1, 1, fn, p);                           \
    addSoftmaxLayer();                                                         \
  }
SCN_FMP_ARCHITECTURE(POFMPSparseConvNet, addLeNetLayerPOFMP)
SCN_FMP_ARCHITECTURE(ROFMPSparseConvNet, addLeNetLayerROFMP)
SCN_FMP_ARCHITECTURE(PDFMPSparseConvNet, addLeNetLayerPDFMP)
SCN_FMP_ARCHITECTURE(RDFMPSparseConvNet, addLeNetLayerRDFMP)
#undef SCN_FMP_ARCHITECTURE
