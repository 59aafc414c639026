// The net runtime behind the SparseConvNet facade: layer list, layer builders,
// per-batch forward driver, weight files (SparseConvNetCUDA.h:25-114).  The
// class keeps the reference's name; the device code underneath is HIP.
#pragma once
#include <fstream>
#include <iostream>
#include <memory>
#include <condition_variable>
#include <mutex>
#include <set>
#include <string>
#include <vector>
#include "SpatiallySparseBatch.h"
#include "SpatiallySparseDataset.h"
#include "SpatiallySparseLayer.h"

#define N_MAX_BATCH_PRODUCER_THREADS 20
#define N_PRODUCER_STREAMS 5
#define N_HARDWARE_QUEUES 4 // per process (GPU_MAX_HW_QUEUES, HIP's default)

// A batch whose input is already in HBM: active sites (sample, key, row),
// backgroundCol per sample, and the feature matrix [nSpatialSites x
// nInputFeatures]; all device pointers.
struct ResidentBatch {
  int batchSize;
  const int32_t *d_sample;
  const int64_t *d_key;
  const int32_t *d_row;
  const int32_t *d_background;
  int64_t nActive;
  int nSpatialSites;
  const float *d_features;
  // the pointers name pinned host memory instead: every batch uploads them
  bool onHost = false;
};

class SparseConvNetCUDA {
public:
  cudaMemStream memStream; // first member: the context outlives every buffer
  std::vector<SpatiallySparseLayer *> layers;
  std::vector<float> inputNormalizingConstants;
  int dimension;
  int nClasses;
  int nTop;
  int inputSpatialSize;
  int nInputFeatures;
  int nOutputFeatures;
  int deviceID;
  int nBatchProducerThreads;
  // one stream per batch slot: the slot's producer thread issues the grid
  // upload and the rule-book kernels of its batch there, while the forward
  // pass of another batch runs on memStream (the reference declares the same
  // array, SparseConvNetCUDA.h:38, and leaves it unused)
  // The streams the batch slots issue their grid and rule-book kernels on: at
  // most N_PRODUCER_STREAMS (HIP spreads streams over four hardware queues;
  // with more than five producer streams the forward pass's stream has to
  // share its queue).  A producer thread borrows one for the GPU half of batch
  // production (acquireProducerStream: the waiting batch with the lowest
  // number goes first, so the consumer's next batch is never behind a later
  // one); the CPU halves of all threads run side by side.
  std::vector<std::unique_ptr<cudaMemStream>> batchMemStreams;
  // How many of them are in use (all, unless told otherwise).  Kernels of
  // streams that share a hardware queue run one after the other, and HIP has
  // N_HARDWARE_QUEUES of them: with two forward lanes, two producer streams
  // leave every stream a queue of its own, and no rule-book kernel then sits
  // between two kernels of a forward pass.  That is the better choice for a
  // net whose forward pass takes longer than the production of its batches
  // (0.122 against 0.128 ms a batch on a five-level 2-D net); a net that waits
  // for its batches (one layer; a 3-D net, whose rule books are the longer
  // half) wants all of them.
  void setProducerStreams(int n);
  int producerStreamsInUse();
  // Forward lanes.  The kernels of one forward pass follow one another on one
  // stream, and most of them are too short to fill the GPU: with two lanes
  // the dataset loops keep the forward passes of two consecutive test batches
  // in flight, each on a stream and a set of feature buffers of its own (the
  // reference shares one set between all batches because it runs one batch at
  // a time, BatchProducer.cu:28-33).  Lane 0 is memStream and the shared
  // buffers.  Results do not depend on the number of lanes.  Training batches
  // always use lane 0: they update the weights.
  int nForwardLanes;
  std::vector<std::unique_ptr<cudaMemStream>> laneStreams; // lanes 1, 2, ..
  std::vector<std::vector<SpatiallySparseBatchSubInterface *>> laneSubInterfaces;
  cudaMemStream &laneStream(int lane);
  void synchronizeLanes();
  cudaMemStream *acquireProducerStream(int batchNumber);
  void releaseProducerStream(cudaMemStream *stream);
  // fewer producer threads than the net was constructed with
  void limitBatchProducerThreads(int n);

private:
  std::mutex streamPoolMutex;
  std::condition_variable streamPoolChanged;
  std::vector<cudaMemStream *> freeProducerStreams;
  std::multiset<int> waitingBatches;
  int producerStreamsWanted; // 0: all

public:
  std::mutex batchLock[N_MAX_BATCH_PRODUCER_THREADS];
  std::vector<SpatiallySparseBatch> batchPool;
  std::vector<SpatiallySparseBatchSubInterface *> initialSubInterfaces;
  std::vector<SpatiallySparseBatchSubInterface *> sharedSubInterfaces;
  SparseConvNetCUDA(int dimension, int nInputFeatures, int nClasses,
                    int pciBusID = -1, int nTop = 1,
                    int nBatchProducerThreads = 10);
  ~SparseConvNetCUDA();
  void forwardBatch(SpatiallySparseBatch &batch, int lane = 0);
  void backwardBatch(SpatiallySparseBatch &batch, float learningRate,
                     float momentum);
  // training batches are drawn in shuffled order (BatchProducer.cu:23-26);
  // a harness that needs a fixed order turns this off
  bool shuffleTrainingData = true;
  // rule books of consecutive layers are built together, one workgroup per
  // sample, where the library can (scn_ctx_chain_rules); off: layer by layer
  bool chainRuleBooks = true;
  void finishBatch(SpatiallySparseBatch &batch, std::ofstream &f,
                   std::ofstream &g);
  void processBatch(SpatiallySparseBatch &batch, float learningRate,
                    float momentum, std::ofstream &f, std::ofstream &g);
  void addLearntLayer(int nFeatures, ActivationFunction activationFn = RELU,
                      float dropout = 0.0f, float alpha = 1.0f);
  void addNetworkInNetworkLayer(int nFeatures,
                                ActivationFunction activationFn = RELU,
                                float dropout = 0.0f);
  void addConvolutionalLayer(int nFeatures, int filterSize, int filterStride,
                             ActivationFunction activationFn = RELU,
                             float dropout = 0.0f, int minActiveInputs = 1,
                             float poolingToFollow = 1.0f);
  void addLeNetLayerMP(int nFeatures, int filterSize, int filterStride,
                       int poolSize, int poolStride,
                       ActivationFunction activationFn = RELU,
                       float dropout = 0.0f, int minActiveInputs = 1);
  // kind: 0 POFMP, 1 PDFMP, 2 ROFMP, 3 RDFMP (SparseConvNetCUDA.cu:112-163)
  void addLeNetLayerFMP(int kind, int nFeatures, int filterSize,
                        int filterStride, int poolSize, float fmpShrink,
                        ActivationFunction activationFn = RELU,
                        float dropout = 0.0f, int minActiveInputs = 1);
  void addTriangularConvolutionalLayer(int nFeatures, int filterSize,
                                       int filterStride,
                                       ActivationFunction activationFn = RELU,
                                       float dropout = 0.0f,
                                       int minActiveInputs = 1,
                                       float poolingToFollow = 1.0f);
  void addTriangularLeNetLayerMP(int nFeatures, int filterSize,
                                 int filterStride, int poolSize, int poolStride,
                                 ActivationFunction activationFn = RELU,
                                 float dropout = 0.0f, int minActiveInputs = 1);
  void addSoftmaxLayer();
  void addTerminalPoolingLayer(int poolSize, int S);
  float processDataset(SpatiallySparseDataset &dataset, int batchSize = 100,
                       float learningRate = 0, float momentum = 0.99);
  void processDatasetRepeatTest(SpatiallySparseDataset &dataset,
                                int batchSize = 100, int nReps = 12,
                                std::string predictionsFilename = "",
                                std::string confusionMatrixFilename = "");
  // every layer but the last; "<sample> <label> <features...>" per sample into
  // "<dataset.name>.features" (SparseConvNetCUDA.cu:507-538)
  void processDatasetDumpTopLevelFeatures(SpatiallySparseDataset &dataset,
                                          int batchSize, int reps = 1);
  // 1 / max |x| per input feature over (at most 10000 pictures of) the
  // dataset; the producers scale every batch's input by these from then on,
  // and saveWeights / loadWeights carry them (SparseConvNetCUDA.cu:540-566)
  void calculateInputRegularizingConstants(SpatiallySparseDataset dataset);
  void loadWeights(std::string baseName, int epoch, bool momentum,
                   int firstNlayers = 1000000);
  void saveWeights(std::string baseName, int epoch, bool momentum);
  // set the operand precision of every NiN contraction (SCN_FP32 / SCN_BF16)
  void setPrecision(int precision);
  // Fuse every convolutional layer's gather into the NiN layer that follows
  // it (one kernel, the im2col-like matrix is never written).  Same results;
  // the convolution's output interface then holds rules but no features.
  // Off by default, as the reference materialises that matrix.
  void setFusedConvolutions(bool on);
  // grows every slot's interface list to layers.size() + 1
  void ensureInterfaces();
  // Fills slot cc's input interface from a batch that already sits in HBM
  // (see ResidentBatch) and builds every rule book, on the slot's stream.
  void preprocessResident(int cc, const struct ResidentBatch &input);
};
