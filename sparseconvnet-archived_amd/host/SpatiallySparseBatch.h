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
  std::unique_ptr<BatchResultStage> result;
  void reset();
};
