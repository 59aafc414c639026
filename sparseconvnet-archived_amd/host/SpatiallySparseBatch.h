// One batch travelling through the net (SpatiallySparseBatch.h:7-22).
#pragma once
#include <vector>
#include "SpatiallySparseBatchInterface.h"
#include "types.h"
#include "vectorCUDA.h"

class SpatiallySparseBatch {
  SpatiallySparseBatchSubInterface *inputSub;

public:
  SpatiallySparseBatch(SpatiallySparseBatchSubInterface *inputSub);
  SpatiallySparseBatch(SpatiallySparseBatch &&) = default;
  // The stream this slot's preprocess() -- grid upload and rule-book kernels
  // -- is issued on (one of the net's batchMemStreams); null: the layer's own.
  cudaMemStream *preprocessStream;
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
  void reset();
};
