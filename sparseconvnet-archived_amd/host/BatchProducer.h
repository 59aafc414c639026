// Builds batches for processDataset (BatchProducer.h:8-25).  As in the
// reference, each worker thread owns one batch slot and runs the whole
// preprocessing of its batches: distort + codifyInputData on the CPU, then the
// upload of the input sites and every layer's preprocess() -- here GPU rule-book
// kernels -- on the slot's own stream.  nextBatch() hands finished slots to the
// caller in order, so rule books of the next batches are built while the
// forward pass of the current one runs on the net's stream.
#pragma once
#include <mutex>
#include <memory>
#include <condition_variable>
#include <thread>
#include <vector>
#include "SparseConvNetCUDA.h"
#include "SpatiallySparseBatch.h"
#include "SpatiallySparseDataset.h"

class BatchProducer;

// The dataset loops' way through the batches of a BatchProducer: the forward
// pass of a batch is only queued, on the next forward lane in turn, and a batch
// is finished (probabilities read, statistics taken) when as many younger
// ones are queued behind it as the net has lanes -- so the GPU never waits for
// the host between batches.  Training batches run one after the other.
class ForwardQueue {
public:
  ForwardQueue(SparseConvNetCUDA &cnn, BatchProducer &bp, bool training);
  ~ForwardQueue();
  // queues b; returns the batch that has to be finished now, or null
  SpatiallySparseBatch *push(SpatiallySparseBatch *b);
  // the oldest batch still queued, or null when there is none (call until null)
  SpatiallySparseBatch *pop();
  int depth;

private:
  SparseConvNetCUDA &cnn;
  std::vector<SpatiallySparseBatch *> inFlight;
  int lanes, count;
  // With several lanes the kernel launches of a forward pass are made by a
  // thread per lane: queueing a pass costs the host about as long as the GPU
  // needs to run it, and one thread cannot feed two lanes.
  struct Worker {
    std::thread thread;
    std::mutex m;
    std::condition_variable cv;
    std::vector<SpatiallySparseBatch *> todo;
    bool stop = false;
  };
  std::vector<std::unique_ptr<Worker>> workers;
  void work(int lane);
};

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
  // nBatches passes over one batch that is resident in HBM (benchmarking), or
  // over several taken in turn
  BatchProducer(SparseConvNetCUDA &cnn, const ResidentBatch &resident,
                int nBatches);
  BatchProducer(SparseConvNetCUDA &cnn,
                const std::vector<ResidentBatch> &residents, int nBatches);
  ~BatchProducer();
  // nextBatch() hands the slot of the batch it returned keepAlive + 1 calls
  // ago back to the workers: 0 is the reference's behaviour; 1 lets the caller
  // still read batch i after asking for batch i + 1 (needs >= 2 slots).
  int keepAlive = 0;
  SpatiallySparseBatch *nextBatch();
  // slots that hold a finished batch nobody has asked for yet
  int slotsReady();
  void batchProducerThread(int nThread);
  // CPU half: fills slot cc with batch c (codify only)
  void preprocessBatch(int c, int cc, RNG &rng);
  // GPU half: uploads slot cc and builds all rule books
  void preprocessBatchOnDevice(int cc);

private:
  static SpatiallySparseDataset emptyDataset;
  std::vector<ResidentBatch> residents; // empty: batches come from the dataset
  void start();
  std::vector<char> slotFull;
  std::condition_variable slotChanged;
  std::mutex slotMutex;
  bool stopping;
};
