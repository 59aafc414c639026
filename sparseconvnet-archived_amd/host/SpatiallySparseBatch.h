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
  batchType type;
  int batchSize;
  std::vector<int> sampleNumbers;
  std::vector<SpatiallySparseBatchInterface> interfaces;
  vectorCUDA<int> labels;
  std::vector<std::vector<int>> predictions;
  std::vector<std::vector<float>> probabilities;
  float negativeLogLikelihood;
  int mistakes;
  void reset();
};
