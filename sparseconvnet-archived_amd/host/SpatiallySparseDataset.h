// Dataset container (SpatiallySparseDataset.h:10-29).  The file-format loaders
// of the reference are not part of the forward path.
#pragma once
#include <string>
#include <vector>
#include "Picture.h"
#include "Rng.h"
#include "types.h"

class SpatiallySparseDataset {
  RNG rng;

public:
  std::string name;
  std::string header;
  std::vector<Picture *> pictures;
  int nFeatures;
  int nClasses;
  batchType type;
  SpatiallySparseDataset();
  void summary();
  void shuffle();
  SpatiallySparseDataset extractValidationSet(float p = 0.1);
  void subsetOfClasses(std::vector<int> activeClasses);
  SpatiallySparseDataset subset(int n);
  SpatiallySparseDataset balancedSample(int n);
  void repeatSamples(int reps);
};
