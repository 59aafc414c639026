// Public API: the reference's SparseConvNet / SparseConvTriangLeNet facades
// (SparseConvNet.h:20-99), same constructors, builders and processing calls.
// Builders for fractional max-pooling and the index-learner head are outside
// the forward path this library covers and are not declared.
#pragma once
#include <fstream>
#include <memory>
#include <string>
#include "SpatiallySparseDataset.h"

class SparseConvNetCUDA;

class SparseConvNet {
public:
  std::unique_ptr<SparseConvNetCUDA> cnn;

  SparseConvNet(int dimension, int nInputFeatures, int nClasses,
                int pciBusID = -1, int nTop = 1);
  ~SparseConvNet();
  void addLeNetLayerMP(int nFeatures, int filterSize, int filterStride,
                       int poolSize, int poolStride,
                       ActivationFunction activationFn = RELU,
                       float dropout = 0.0f, int minActiveInputs = 1);
  void addTerminalPoolingLayer(int poolSize);
  void addSoftmaxLayer();
  float processDataset(SpatiallySparseDataset &dataset, int batchSize = 100,
                       float learningRate = 0, float momentum = 0.99);
  void processDatasetRepeatTest(SpatiallySparseDataset &dataset,
                                int batchSize = 100, int nReps = 12,
                                std::string predictionsFilename = "",
                                std::string confusionMatrixFilename = "");
  void loadWeights(std::string baseName, int epoch, bool momentum = false,
                   int firstNlayers = 1000000);
  void saveWeights(std::string baseName, int epoch, bool momentum = false);
};

class SparseConvTriangLeNet {
private:
  std::unique_ptr<SparseConvNetCUDA> cnn;

public:
  SparseConvTriangLeNet(int dimension, int nInputFeatures, int nClasses,
                        int pciBusID = -1, int nTop = 1);
  ~SparseConvTriangLeNet();
  void addLeNetLayerMP(int nFeatures, int filterSize, int filterStride,
                       int poolSize, int poolStride,
                       ActivationFunction activationFn = RELU,
                       float dropout = 0.0f, int minActiveInputs = 1);
  void addTerminalPoolingLayer(int poolSize);
  void addSoftmaxLayer();
  float processDataset(SpatiallySparseDataset &dataset, int batchSize = 100,
                       float learningRate = 0, float momentum = 0.99);
  void processDatasetRepeatTest(SpatiallySparseDataset &dataset,
                                int batchSize = 100, int nReps = 12,
                                std::string predictionsFilename = "",
                                std::string confusionMatrixFilename = "");
  void loadWeights(std::string baseName, int epoch, bool momentum = false,
                   int firstNlayers = 1000000);
  void saveWeights(std::string baseName, int epoch, bool momentum = false);
  SparseConvNetCUDA *runtime() { return cnn.get(); }
};
