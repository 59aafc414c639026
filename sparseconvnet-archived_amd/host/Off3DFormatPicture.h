// 3-D surface meshes as input samples: the reference's OffSurfaceModelPicture
// (Off3DFormatPicture.h:7-23), the front-end of its SHREC2015 / ModelNet
// drivers, without Armadillo.  A mesh is read from an OFF file (or given as
// arrays), fitted into a cube of side renderSize, and codified by drawing
// every triangle into the voxel lattice: one input feature, 1 on every voxel
// a triangle touches, rows numbered in the order the voxels are first touched.
#pragma once
#include <string>
#include <vector>
#include "Picture.h"

class OffSurfaceModelPicture : public Picture {
public:
  std::vector<double> points;  // nPoints x 3
  std::vector<int> surfaces;   // nTriangles x 3 (faces are taken as triangles)
  int renderSize;
  bool loaded; // false when the file could not be read as an OFF mesh
  OffSurfaceModelPicture(std::string filename, int renderSize, int label = -1);
  OffSurfaceModelPicture(const double *xyz, int nPoints, const int *triangles,
                         int nTriangles, int renderSize, int label = -1);
  // fit centrally in the cube [-renderSize/2, renderSize/2]^3
  void normalize();
  // points <- points Q, Q the orthogonal factor of a random 3x3 matrix
  void random_rotation(RNG &rng);
  void jiggle(RNG &rng, float alpha);
  void affineTransform(RNG &rng, float alpha);
  void codifyInputData(SparseGrid &grid, std::vector<float> &features,
                       int &nSpatialSites, int spatialSize);
  Picture *distort(RNG &rng, batchType type = TRAINBATCH);
  std::string identify();
};
