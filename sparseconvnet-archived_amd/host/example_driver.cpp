// A driver written the way the reference's drivers are (one main(), a Picture
// subclass, a canned net, processDataset), against this library's headers.
// It is the source-compatibility check: nothing here names HIP or the C ABI.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include "NetworkArchitectures.h"
#include "SpatiallySparseDataset.h"

// pen-stroke-like sample: a few random walks on a size x size lattice, three
// features per site
class StrokePicture : public Picture {
  std::vector<int> xs, ys;
  std::vector<float> feats;
  int size;

public:
  // shapeSeed fixes where the strokes go, seed the features along them
  StrokePicture(int size, int nSites, unsigned seed, int label,
                unsigned shapeSeed = 0)
      : Picture(label), size(size) {
    RNG rng(shapeSeed ? shapeSeed : seed), featureRng(seed);
    float x = rng.uniform(0.2f * size, 0.8f * size);
    float y = rng.uniform(0.2f * size, 0.8f * size);
    float angle = rng.uniform(0, 6.2831853f);
    for (int i = 0; i < nSites; ++i) {
      if (i % (nSites / 4 + 1) == 0) { // new stroke
        x = rng.uniform(0.2f * size, 0.8f * size);
        y = rng.uniform(0.2f * size, 0.8f * size);
      }
      angle += rng.normal(0, 0.35f);
      x = std::min(std::max(x + std::cos(angle), 0.0f), size - 1.0f);
      y = std::min(std::max(y + std::sin(angle), 0.0f), size - 1.0f);
      xs.push_back((int)std::lround(x));
      ys.push_back((int)std::lround(y));
      for (int c = 0; c < 3; ++c)
        feats.push_back(shapeSeed ? featureRng.uniform(0.5f, 1)
                                  : rng.uniform(-1, 1));
    }
  }
  // the contract of Picture::codifyInputData: background row first, then one
  // row per new site, key = x * spatialSize + y
  void codifyInputData(SparseGrid &grid, std::vector<float> &features,
                       int &nSpatialSites, int spatialSize) {
    for (int c = 0; c < 3; ++c)
      features.push_back(0);
    grid.backgroundCol = nSpatialSites++;
    int shift = (spatialSize - size) / 2;
    for (size_t i = 0; i < xs.size(); ++i) {
      int64_t n = (int64_t)(xs[i] + shift) * spatialSize + (ys[i] + shift);
      if (grid.mp.find(n) == grid.mp.end()) {
        grid.mp[n] = nSpatialSites++;
        for (int c = 0; c < 3; ++c)
          features.push_back(feats[3 * i + c]);
      }
    }
  }
  std::string identify() { return "stroke picture"; }
};

int main(int argc, char **argv) {
  // weights, dropout and the order of the pictures come from generators that
  // the reference seeds from the clock; here from a fixed number, so that the
  // check on the training below means the same in every run
  setenv("SCN_SEED", "20150101", 0);
  int nPictures = argc > 1 ? std::atoi(argv[1]) : 500;
  int batchSize = argc > 2 ? std::atoi(argv[2]) : 100;
  SpatiallySparseDataset testSet;
  testSet.name = "Synthetic strokes (test)";
  testSet.type = TESTBATCH;
  testSet.nFeatures = 3;
  testSet.nClasses = 100;
  for (int i = 0; i < nPictures; ++i)
    testSet.pictures.push_back(new StrokePicture(96, 400, 1000u + i, i % 100));
  testSet.summary();

  DeepC2 cnn(2, 5, 32, VLEAKYRELU, testSet.nFeatures, testSet.nClasses, 0.1f);
  float nll = cnn.processDataset(testSet, batchSize);
  cnn.saveWeights("/tmp/scn_example", 1);
  cnn.loadWeights("/tmp/scn_example", 1);
  float nll2 = cnn.processDataset(testSet, batchSize);
  cnn.processDatasetRepeatTest(testSet, batchSize, 2);
  for (auto *p : testSet.pictures)
    delete p;
  std::remove("/tmp/scn_example_epoch-1.cnn");
  if (!(std::fabs(nll - nll2) <= 1e-6f * std::fabs(nll))) {
    std::cout << "NLL changed across a weight save/load: " << nll << " " << nll2
              << std::endl;
    return 1;
  }
  // Training, the way the reference's drivers loop over epochs: ten classes,
  // each a fixed set of strokes with varying features; a small net with
  // dropout learns to tell them apart.
  SpatiallySparseDataset trainSet;
  trainSet.name = "Synthetic strokes (train)";
  trainSet.type = TRAINBATCH;
  trainSet.nFeatures = 3;
  trainSet.nClasses = 10;
  for (int i = 0; i < 200; ++i)
    trainSet.pictures.push_back(
        new StrokePicture(28, 80, 5000u + i, i % 10, 77u + i % 10));
  SpatiallySparseDataset validationSet = trainSet; // same pictures, test mode
  validationSet.name = "Synthetic strokes (validation)";
  validationSet.type = TESTBATCH;
  DeepC2 small(2, 3, 16, VLEAKYRELU, trainSet.nFeatures, trainSet.nClasses,
               0.2f);
  float before = small.processDataset(validationSet, 100);
  for (int epoch = 1; epoch <= 20; epoch++) {
    std::cout << "epoch: " << epoch << " " << std::flush;
    small.processDataset(trainSet, 100, 0.003 * exp(-0.01 * epoch));
  }
  float after = small.processDataset(validationSet, 100);
  // a net with fractional max-pooling: every pass draws new pooling regions,
  // so two passes over the same pictures give slightly different costs
  POFMPSparseConvNet fmp(2, 5, 8, 1.5f, VLEAKYRELU, trainSet.nFeatures,
                         trainSet.nClasses);
  float fmp1 = fmp.processDataset(validationSet, 100);
  float fmp2 = fmp.processDataset(validationSet, 100);
  for (auto *p : trainSet.pictures)
    delete p;
  if (!(fmp1 > 0 && fmp2 > 0 && fmp1 < 50 && fmp2 < 50)) {
    std::cout << "fractional max-pooling net: NLL " << fmp1 << " " << fmp2
              << std::endl;
    return 1;
  }
  if (!(after < 0.25f * before)) {
    std::cout << "training did not lower the cost: " << before << " -> "
              << after << std::endl;
    return 1;
  }
  std::cout << "example driver ok, NLL " << nll << ", trained " << before
            << " -> " << after << std::endl;
  return 0;
}
