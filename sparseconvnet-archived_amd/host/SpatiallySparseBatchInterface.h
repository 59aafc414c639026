// Data carried between layers (SpatiallySparseBatchInterface.h:8-46).
#pragma once
#include <vector>
#include "SparseGrid.h"
#include "vectorCUDA.h"

// The large vectors of one depth; they stay in HBM and are shared by every
// batch slot (BatchProducer.cu:28-33).
class SpatiallySparseBatchSubInterface {
public:
  vectorCUDA<float> features;
  vectorCUDA<float> dfeatures; // gradient of the cost, training batches only
  vectorCUDA<int> poolingChoices;
  // room for a bf16 copy of `features` (two bytes an element), made by a
  // following fused convolution with bf16 operands whose window is large
  // enough for the rows to be read many times over
  vectorCUDA<float> features16;
  SpatiallySparseBatchSubInterface();
  void reset();
};

class SpatiallySparseBatchInterface {
public:
  SpatiallySparseBatchSubInterface *sub;
  int nFeatures;                   // features per spatial location
  vectorCUDA<int> featuresPresent; // all of them, except under dropout in a training batch
  int nSpatialSites; // active rows of the whole batch, background rows included
  int spatialSize;
  bool backpropErrors;
  // Host view of the sparse grids.  Filled by the Pictures for the input
  // interface; for deeper interfaces the grids are built in HBM
  // (deviceGrids) and this view is only materialised by downloadGrids().
  std::vector<SparseGrid> grids;
  scn_grids *deviceGrids;
  bool ownsDeviceGrids;
  vectorCUDA<int> rules;
  // Output of a fractional max-pooling layer: the regions drawn for this
  // batch, inputL then inputR, each [batchSize][dimension][spatialSize].
  std::vector<int> regionTicks;
  // Set by a convolutional layer that left its gather to the following NiN
  // layer (fused kernel): the interface whose features the rules index.  The
  // feature matrix of THIS interface is then not materialised.
  SpatiallySparseBatchInterface *deferredGatherFrom;
  SpatiallySparseBatchInterface(SpatiallySparseBatchSubInterface *s);
  SpatiallySparseBatchInterface(SpatiallySparseBatchInterface &&o);
  ~SpatiallySparseBatchInterface();
  void downloadGrids(int batchSize);
  void summary();
  void reset();
};
