// Builds batches for processDataset (BatchProducer.h:8-25).  Worker threads
// run the CPU part (distort + codifyInputData) one batch slot each;
// nextBatch() uploads the slot and issues every layer's preprocess() -- the
// rule-book kernels -- from the calling thread, on the net's stream.
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
  ~BatchProducer();
  SpatiallySparseBatch *nextBatch();
  void batchProducerThread(int nThread);
  // CPU half: fills slot cc with batch c (codify only)
  void preprocessBatch(int c, int cc, RNG &rng);
  // GPU half: uploads slot cc and builds all rule books
  void preprocessBatchOnDevice(int cc);

private:
  std::vector<char> slotFull;
  std::condition_variable slotChanged;
  std::mutex slotMutex;
  bool stopping;
};
