// One batch travelling through the net (SpatiallySparseBatch.h:7-22).
#pragma once
#include <atomic>
#include <memory>
#include <vector>
#include "SpatiallySparseBatchInterface.h"
#include "types.h"
#include "vectorCUDA.h"

// Where a batch's class probabilities land: pinned host memory filled by a
// copy queued behind the batch's forward pass, and the event that says it has
// arrived.  Lets the caller queue the next batch before reading this one.
struct BatchResultStage {
  float *pinned;
  size_t capacity; // floats
  scn_event *arrived;
  bool pending;
  // a training batch: the point of the net's stream behind the backward pass,
  // the last reader of the slot's rule books and features.  The slot goes
  // back to its producer only after this point has been passed.
  scn_event *consumed;
  bool consumedPending;
  // set by the thread that queued the batch's forward pass once all of it is
  // queued (the dataset loops may leave that to a thread per forward lane)
  std::atomic<bool> enqueued;
  // the labels as the statistics need them, on the host, while batch.labels
  // is in device memory for the gradient of a training batch
  std::vector<int> labels;
  BatchResultStage();
  ~BatchResultStage();
  BatchResultStage(const BatchResultStage &) = delete;
  BatchResultStage &operator=(const BatchResultStage &) = delete;
};

// Pinned host memory that only grows: what a batch slot flattens its input
// grids into before it borrows a stream, so that the upload is four queued
// copies and the stream is not held while the CPU walks the grids.
struct PinnedStage {
  void *p;
  size_t bytes;
  PinnedStage() : p(nullptr), bytes(0) {}
  PinnedStage(PinnedStage &&o) : p(o.p), bytes(o.bytes) { o.p = nullptr, o.bytes = 0; }
  PinnedStage(const PinnedStage &) = delete;
  PinnedStage &operator=(const PinnedStage &) = delete;
  ~PinnedStage();
  // at least n bytes (the contents are not kept)
  void reserve(size_t n);
  template <typename T> T *as() { return static_cast<T *>(p); }
};

class SpatiallySparseBatch {
  SpatiallySparseBatchSubInterface *inputSub;

public:
  SpatiallySparseBatch(SpatiallySparseBatchSubInterface *inputSub);
  SpatiallySparseBatch(SpatiallySparseBatch &&) = default;
  // The stream this slot's preprocess() -- grid upload and rule-book kernels
  // -- is issued on (one of the net's batchMemStreams); null: the layer's own.
  cudaMemStream *preprocessStream;
  // The stream this batch's forward pass is issued on when that is not the
  // layers' own (a net with several forward lanes); null: the layers' own.
  cudaMemStream *forwardStream;
  batchType type;
  int batchSize;
  std::vector<int> sampleNumbers;
  std::vector<SpatiallySparseBatchInterface> interfaces;
  vectorCUDA<int> labels;
  std::vector<std::vector<int>> predictions;
  std::vector<std::vector<float>> probabilities;
  float negativeLogLikelihood;
  int mistakes;
  // device staging of the input sites (sample, key as two ints, row,
  // backgroundCol), reused from batch to batch
  vectorCUDA<int> stagingSample, stagingKey, stagingRow, stagingBackground;
  // the same four arrays on the host, pinned, and how many sites they hold
  PinnedStage hostSample, hostKey, hostRow, hostBackground;
  size_t hostSites;
  // ... and the input features, moved there from the interface's host vector
  PinnedStage hostFeatures;
  size_t hostFeatureCount;
  std::unique_ptr<BatchResultStage> result;
  void reset();
};
