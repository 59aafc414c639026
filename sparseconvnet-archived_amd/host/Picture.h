// Input samples.  Picture is the reference's abstract input
// (Picture.h:8-17): codifyInputData() appends the sample's feature rows to
// `features`, numbers them from `nSpatialSites`, and records site key -> row
// in `grid` (key = row-major index in the spatialSize^dimension field, first
// axis most significant; OpenCVPicture.cpp:368-402).
#pragma once
#include <string>
#include <vector>
#include "Rng.h"
#include "SparseGrid.h"
#include "types.h"

class Picture {
public:
  virtual void codifyInputData(SparseGrid &grid, std::vector<float> &features,
                               int &nSpatialSites, int spatialSize) = 0;
  virtual Picture *distort(RNG &rng, batchType type) { return this; }
  virtual std::string identify();
  int label; // -1 for unknown
  Picture(int label = -1);
  virtual ~Picture();
};

// A sample given directly as active sites: coordinates in a lattice of side
// `latticeSize`, centred in the net's input field when that is larger (as
// shrec2015.cpp:15,21 renders a 40-wide object into a 126-wide field).
// Emits the background row first, then the sites in the stored order.
class SparsePointsPicture : public Picture {
public:
  int dimension;
  int latticeSize;
  int nFeatures;
  std::vector<int> coords;     // nSites x dimension
  std::vector<float> features; // nSites x nFeatures
  SparsePointsPicture(int dimension, int latticeSize, int nFeatures,
                      int label = -1);
  void codifyInputData(SparseGrid &grid, std::vector<float> &features,
                       int &nSpatialSites, int spatialSize);
  std::string identify();
};
