// The layer interface and every layer class.
//
// preprocess() builds the output interface's grids and rule book, forwards()
// runs the feature kernels (SpatiallySparseLayer.h:6-27).  In the reference
// preprocess() is CPU code run by batch-producer threads; here it issues the
// rule-book kernels on the GPU.  backwards() propagates the gradient of the
// cost from the output interface's dfeatures to the input's and, in layers
// with weights, takes one momentum step on the weights the batch used (all of
// them, or with dropout the sub-matrix of the features present); scaleWeights()
// is the per-layer step of a RESCALEBATCH pass.
#pragma once
#include <fstream>
#include <iostream>
#include <mutex>
#include "Rng.h"
#include "SpatiallySparseBatch.h"
#include "SpatiallySparseBatchInterface.h"

class SpatiallySparseLayer {
public:
  cudaMemStream &memStream;
  virtual void preprocess(SpatiallySparseBatch &batch,
                          SpatiallySparseBatchInterface &input,
                          SpatiallySparseBatchInterface &output) = 0;
  virtual void forwards(SpatiallySparseBatch &batch,
                        SpatiallySparseBatchInterface &input,
                        SpatiallySparseBatchInterface &output) = 0;
  virtual void scaleWeights(SpatiallySparseBatchInterface &input,
                            SpatiallySparseBatchInterface &output,
                            float &scalingUnderneath, bool topLayer);
  virtual void backwards(SpatiallySparseBatch &batch,
                         SpatiallySparseBatchInterface &input,
                         SpatiallySparseBatchInterface &output,
                         float learningRate, float momentum);
  SpatiallySparseLayer(cudaMemStream &memStream);
  virtual ~SpatiallySparseLayer();
  virtual void loadWeightsFromStream(std::ifstream &f, bool momentum);
  virtual void putWeightsToStream(std::ofstream &f, bool momentum);
  virtual int calculateInputSpatialSize(int outputSpatialSize) = 0;
};

// ConvolutionalLayer.h:3-33 -- gathers each output site's receptive field
// into one row of the matrix the following NiN layer multiplies.
class ConvolutionalLayer : public SpatiallySparseLayer {
private:
  int fs;

public:
  int inSpatialSize;
  int outSpatialSize;
  int filterSize;
  int filterStride;
  int dimension;
  int nFeaturesIn;
  int nFeaturesOut;
  int minActiveInputs; // 1; > 1; or -1 for 'valid' mode
  // leave the gather to the NiN layer that follows (fused kernel); set by
  // SparseConvNetCUDA::setFusedConvolutions
  bool deferGather;
  ConvolutionalLayer(cudaMemStream &memStream, int filterSize,
                     int filterStride, int dimension, int nFeaturesIn,
                     int minActiveInputs = 1);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};

// ConvolutionalTriangularLayer.h
class ConvolutionalTriangularLayer : public SpatiallySparseLayer {
private:
  int fs;

public:
  int inSpatialSize;
  int outSpatialSize;
  int filterSize;
  int filterStride;
  int dimension;
  int nFeaturesIn;
  int nFeaturesOut;
  int minActiveInputs;
  bool deferGather;
  ConvolutionalTriangularLayer(cudaMemStream &memStream, int filterSize,
                               int filterStride, int dimension,
                               int nFeaturesIn, int minActiveInputs = 1);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};

// NetworkInNetworkLayer.h:5-49 -- W [nFeaturesIn x nFeaturesOut] row-major,
// B [nFeaturesOut]; public so that a harness can set them.
class NetworkInNetworkLayer : public SpatiallySparseLayer {
private:
  RNG rng;
  std::mutex rngMutex; // preprocess() runs on several producer threads
  vectorCUDA<float> dw, db, workspace; // gradients; W transposed for dA
  bool gradsClean = false; // dw and db hold zeros (the momentum step left them so)
  vectorCUDA<float> w, b; // sub-matrix of a training batch with dropout

public:
  vectorCUDA<float> W;
  vectorCUDA<float> MW; // momentum
  vectorCUDA<float> B;
  vectorCUDA<float> MB;
  ActivationFunction fn;
  int nFeaturesIn;
  int nFeaturesOut;
  float dropout;
  int precision; // SCN_FP32 or SCN_BF16 operands for the contraction
  NetworkInNetworkLayer(cudaMemStream &memStream, int nFeaturesIn,
                        int nFeaturesOut, float dropout = 0,
                        ActivationFunction fn = NOSIGMOID, float alpha = 1);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void scaleWeights(SpatiallySparseBatchInterface &input,
                    SpatiallySparseBatchInterface &output,
                    float &scalingUnderneath, bool topLayer);
  void loadWeightsFromStream(std::ifstream &f, bool momentum);
  void putWeightsToStream(std::ofstream &f, bool momentum);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};

// NetworkInNetworkPReLULayer.h
class NetworkInNetworkPReLULayer : public SpatiallySparseLayer {
private:
  RNG rng;
  std::mutex rngMutex;
  vectorCUDA<float> dw, db, dprelu, workspace;
  bool gradsClean = false; // as NetworkInNetworkLayer's
  vectorCUDA<float> w, b;

public:
  vectorCUDA<float> W;
  vectorCUDA<float> MW;
  vectorCUDA<float> B;
  vectorCUDA<float> MB;
  vectorCUDA<float> PReLU; // per-channel slope, initialised to 0.25
  vectorCUDA<float> MPReLU;
  int nFeaturesIn;
  int nFeaturesOut;
  float dropout;
  int precision;
  NetworkInNetworkPReLULayer(cudaMemStream &memStream, int nFeaturesIn,
                             int nFeaturesOut, float dropout = 0,
                             float alpha = 1);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void scaleWeights(SpatiallySparseBatchInterface &input,
                    SpatiallySparseBatchInterface &output,
                    float &scalingUnderneath, bool topLayer);
  void loadWeightsFromStream(std::ifstream &f, bool momentum);
  void putWeightsToStream(std::ofstream &f, bool momentum);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};

// MaxPoolingLayer.h:11-31
class MaxPoolingLayer : public SpatiallySparseLayer {
public:
  int inSpatialSize;
  int outSpatialSize;
  int poolSize;
  int poolStride;
  int dimension;
  int sd;
  MaxPoolingLayer(cudaMemStream &memStream, int poolSize, int poolStride,
                  int dimension);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};

// MaxPoolingTriangularLayer.h
class MaxPoolingTriangularLayer : public SpatiallySparseLayer {
public:
  int inSpatialSize;
  int outSpatialSize;
  int poolSize;
  int poolStride;
  int dimension;
  int S;
  MaxPoolingTriangularLayer(cudaMemStream &memStream, int poolSize,
                            int poolStride, int dimension);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};

// MaxPoolingLayer.h:34-143 -- the four fractional max-pooling layers.  Every
// sample of a batch gets freshly drawn pooling regions along every axis
// (MaxPoolingLayer.cu:181-186); the draw is host work, the rule book is built
// on the GPU from the region tables.
enum FmpKind {
  FMP_PSEUDORANDOM_OVERLAPPING,
  FMP_PSEUDORANDOM_NONOVERLAPPING,
  FMP_RANDOM_OVERLAPPING,
  FMP_RANDOM_NONOVERLAPPING
};
// inputL / inputR of one axis as the reference's tick classes compute them
// (Regions.cu:31-134); stops the program where the reference asserts
void fmpTicks(FmpKind kind, int nIn, int nOut, int poolSize, RNG &rng,
              int *inputL, int *inputR);
class FractionalMaxPoolingLayer : public SpatiallySparseLayer {
  int sd;
  FmpKind kind;
  std::mutex rngMutex; // preprocess() runs on several producer threads

public:
  int inSpatialSize;
  int outSpatialSize;
  float fmpShrink;
  int poolSize;
  int dimension;
  RNG rng;
  FractionalMaxPoolingLayer(cudaMemStream &memStream, FmpKind kind,
                            int poolSize, float fmpShrink, int dimension);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};
#define SCN_FMP_LAYER(Name, Kind)                                              \
  class Name : public FractionalMaxPoolingLayer {                             \
  public:                                                                      \
    Name(cudaMemStream &memStream, int poolSize, float fmpShrink,              \
         int dimension)                                                        \
        : FractionalMaxPoolingLayer(memStream, Kind, poolSize, fmpShrink,      \
                                    dimension) {}                              \
  };
SCN_FMP_LAYER(PseudorandomOverlappingFractionalMaxPoolingLayer,
              FMP_PSEUDORANDOM_OVERLAPPING)
SCN_FMP_LAYER(PseudorandomNonOverlappingFractionalMaxPoolingLayer,
              FMP_PSEUDORANDOM_NONOVERLAPPING)
SCN_FMP_LAYER(RandomOverlappingFractionalMaxPoolingLayer,
              FMP_RANDOM_OVERLAPPING)
SCN_FMP_LAYER(RandomNonOverlappingFractionalMaxPoolingLayer,
              FMP_RANDOM_NONOVERLAPPING)
#undef SCN_FMP_LAYER

// TerminalPoolingLayer.h:5-25 -- averages every active site of a sample.
class TerminalPoolingLayer : public SpatiallySparseLayer {
public:
  int inSpatialSize;  // == poolSize
  int outSpatialSize; // 1
  int poolSize;
  int S; // only printed; the rule width is the batch's largest site count
  TerminalPoolingLayer(cudaMemStream &memStream, int poolSize, int S);
  void preprocess(SpatiallySparseBatch &batch,
                  SpatiallySparseBatchInterface &input,
                  SpatiallySparseBatchInterface &output);
  void forwards(SpatiallySparseBatch &batch,
                SpatiallySparseBatchInterface &input,
                SpatiallySparseBatchInterface &output);
  void backwards(SpatiallySparseBatch &batch,
                 SpatiallySparseBatchInterface &input,
                 SpatiallySparseBatchInterface &output, float learningRate,
                 float momentum);
  int calculateInputSpatialSize(int outputSpatialSize);
};

// SoftmaxClassifier.h:10-12 -- copies the class probabilities to the host,
// takes the top nTop classes per sample, counts mistakes and adds up the
// negative log-likelihood.
void SoftmaxClassifier(SpatiallySparseBatchInterface &input,
                       SpatiallySparseBatch &batch, int nTop,
                       cudaMemStream &memStream);
// its two halves: queue the copy of the probabilities; wait for it and count
void SoftmaxClassifierLaunch(SpatiallySparseBatchInterface &input,
                             SpatiallySparseBatch &batch,
                             cudaMemStream &memStream);
void SoftmaxClassifierCollect(SpatiallySparseBatchInterface &input,
                              SpatiallySparseBatch &batch, int nTop);

// utilities.h
int ipow(int base, int exp);
int triangleSize(int linearSize, int dimension);
int intRound(int a, int d);
int intRoundUp(int a, int d);
std::vector<int> range(int n);
template <typename t>
std::vector<int> vectorTopIndices(std::vector<t> &test, int k);
