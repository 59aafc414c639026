// Builds batches for processDataset (BatchProducer.h:8-25).  As in the
// reference, each worker thread owns one batch slot and runs the whole
// preprocessing of its batches: distort + codifyInputData on the CPU, then the
// upload of the input sites and every layer's preprocess() -- here GPU rule-book
// kernels -- on the slot's own stream.  nextBatch() hands finished slots to the
// caller in order, so rule books of the next batches are built while the
// forward pass of the current one runs on the net's stream.
#pragma once
#include <condition_variable>
#include <thread>
#include <vector>
#include "SparseConvNetCUDA.h"
#include "SpatiallySparseBatch.h"
#include "SpatiallySparseDataset.h"

class BatchProducer {
public:
  SparseConvNetCUDA &cnn;
  int batchCounter;
  int nBatches;
  std::vector<std::thread> workers;
  SpatiallySparseDataset &dataset;
  int batchSize;
  int spatialSize;
  std::vector<int> permutation;
  BatchProducer(SparseConvNetCUDA &cnn, SpatiallySparseDataset &dataset,
                int spatialSize, int batchSize);
  // nBatches passes over one batch that is resident in HBM (benchmarking)
  BatchProducer(SparseConvNetCUDA &cnn, const ResidentBatch &resident,
                int nBatches);
  ~BatchProducer();
  // nextBatch() hands the slot of the batch it returned keepAlive + 1 calls
  // ago back to the workers: 0 is the reference's behaviour; 1 lets the caller
  // still read batch i after asking for batch i + 1 (needs >= 2 slots).
  int keepAlive = 0;
  SpatiallySparseBatch *nextBatch();
  void batchProducerThread(int nThread);
  // CPU half: fills slot cc with batch c (codify only)
  void preprocessBatch(int c, int cc, RNG &rng);
  // GPU half: uploads slot cc and builds all rule books
  void preprocessBatchOnDevice(int cc);

private:
  static SpatiallySparseDataset emptyDataset;
  const ResidentBatch *resident;
  ResidentBatch residentCopy;
  void start();
  std::vector<char> slotFull;
  std::condition_variable slotChanged;
  std::mutex slotMutex;
  bool stopping;
};
