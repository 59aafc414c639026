// The public host API in one header: dataset container, the two net facades
// and the canned architectures.  The headers named after the reference's
// (SparseConvNet.h, NetworkArchitectures.h, SpatiallySparseDataset.h) include
// this file, so driver code written for the reference finds every class where
// it expects it.
#pragma once
#include <fstream>
#include <memory>
#include <string>
#include <vector>
#include "Picture.h"
#include "Rng.h"
#include "types.h"

// ---------------------------------------------------------------- dataset
// Container of Pictures with the fields the batch producer reads
// (reference SpatiallySparseDataset.h:10-29).  The file-format loaders of the
// reference are not part of the forward path.
class SpatiallySparseDataset {
  RNG rng;

public:
  SpatiallySparseDataset();
  std::string name;   // printed by processDataset
  std::string header; // first line of a predictions file
  std::vector<Picture *> pictures;
  int nFeatures; // channels per site
  int nClasses;
  batchType type; // TRAINBATCH, TESTBATCH, UNLABELEDBATCH or RESCALEBATCH

  void summary();
  void shuffle();
  void repeatSamples(int reps);
  void subsetOfClasses(std::vector<int> activeClasses);
  SpatiallySparseDataset subset(int n);
  SpatiallySparseDataset balancedSample(int n);
  SpatiallySparseDataset extractValidationSet(float p = 0.1);
};

// ------------------------------------------------------------------- nets
class SparseConvNetCUDA;

// Builder and processing calls shared by the square-lattice and the
// triangular-lattice facade (reference SparseConvNet.h:25-66 and :75-98):
// same names, argument order and defaults.  The index-learner head is not
// part of this library and is not declared.
#define SCN_FACADE_METHODS                                                     \
  void addLeNetLayerMP(int nFeatures, int filterSize, int filterStride,        \
                       int poolSize, int poolStride,                           \
                       ActivationFunction activationFn = RELU,                 \
                       float dropout = 0.0f, int minActiveInputs = 1);         \
  void addTerminalPoolingLayer(int poolSize);                                  \
  void addSoftmaxLayer();                                                      \
  float processDataset(SpatiallySparseDataset &dataset, int batchSize = 100,   \
                       float learningRate = 0, float momentum = 0.99);         \
  void processDatasetRepeatTest(SpatiallySparseDataset &dataset,               \
                                int batchSize = 100, int nReps = 12,           \
                                std::string predictionsFilename = "",          \
                                std::string confusionMatrixFilename = "");     \
  void processDatasetDumpTopLevelFeatures(SpatiallySparseDataset &dataset,     \
                                          int batchSize, int reps = 1);        \
  void calculateInputRegularizingConstants(SpatiallySparseDataset dataset);    \
  void loadWeights(std::string baseName, int epoch, bool momentum = false,     \
                   int firstNlayers = 1000000);                                \
  void saveWeights(std::string baseName, int epoch, bool momentum = false);

#define SCN_FMP_BUILDER(Name)                                                  \
  void Name(int nFeatures, int filterSize, int filterStride, int poolSize,     \
            float fmpShrink, ActivationFunction activationFn = RELU,           \
            float dropout = 0.0f, int minActiveInputs = 1);
class SparseConvNet {
public:
  std::unique_ptr<SparseConvNetCUDA> cnn; // public in the reference too
  SparseConvNet(int dimension, int nInputFeatures, int nClasses,
                int pciBusID = -1, int nTop = 1);
  ~SparseConvNet();
  SCN_FACADE_METHODS
  // convolution + NiN + fractional max-pooling: pseudorandom / random,
  // overlapping / disjoint regions (SparseConvNet.h:32-47)
  SCN_FMP_BUILDER(addLeNetLayerPOFMP)
  SCN_FMP_BUILDER(addLeNetLayerROFMP)
  SCN_FMP_BUILDER(addLeNetLayerPDFMP)
  SCN_FMP_BUILDER(addLeNetLayerRDFMP)
};
#undef SCN_FMP_BUILDER

class SparseConvTriangLeNet {
  std::unique_ptr<SparseConvNetCUDA> cnn;

public:
  SparseConvTriangLeNet(int dimension, int nInputFeatures, int nClasses,
                        int pciBusID = -1, int nTop = 1);
  ~SparseConvTriangLeNet();
  SCN_FACADE_METHODS
  SparseConvNetCUDA *runtime() { return cnn.get(); }
};

// ---------------------------------------------------------- architectures
// Nets assembled from addLeNetLayerMP (reference NetworkArchitectures.cpp:3-68):
// l + 1 convolutional levels with k * (level + 1) features, dropout rising
// linearly to p, then the softmax classifier.
//   DeepCNet       C3 on the input, then C2; MP3/2 between levels
//   DeepC2         C2 - MP3/2 levels
//   DeepCNiN       DeepC2 with a 1x1 NiN after every convolution
//   DeepC2C2       two C2 per level
//   DeepC3C3       two C3 per level
//   DeepC3C3Valid  the same with 'valid' convolutions (minActiveInputs -1, 2-D)
#define SCN_ARCHITECTURE(Name)                                                 \
  class Name : public SparseConvNet {                                         \
  public:                                                                      \
    Name(int dimension, int l, int k, ActivationFunction fn,                   \
         int nInputFeatures, int nClasses, float p = 0.0f,                     \
         int cudaDevice = -1, int nTop = 1);                                   \
  };
SCN_ARCHITECTURE(DeepCNet)
SCN_ARCHITECTURE(DeepC2)
SCN_ARCHITECTURE(DeepCNiN)
SCN_ARCHITECTURE(DeepC2C2)
SCN_ARCHITECTURE(DeepC3C3)
SCN_ARCHITECTURE(DeepC3C3Valid)
#undef SCN_ARCHITECTURE
// NetworkArchitectures.h:43-69: l levels of C2 followed by fractional
// max-pooling with ratio fmpShrink
#define SCN_FMP_ARCHITECTURE(Name)                                             \
  class Name : public SparseConvNet {                                         \
  public:                                                                      \
    Name(int dimension, int l, int k, float fmpShrink, ActivationFunction fn,  \
         int nInputFeatures, int nClasses, float p = 0.0f,                     \
         int cudaDevice = -1, int nTop = 1);                                   \
  };
SCN_FMP_ARCHITECTURE(POFMPSparseConvNet)
SCN_FMP_ARCHITECTURE(ROFMPSparseConvNet)
SCN_FMP_ARCHITECTURE(PDFMPSparseConvNet)
SCN_FMP_ARCHITECTURE(RDFMPSparseConvNet)
#undef SCN_FMP_ARCHITECTURE
