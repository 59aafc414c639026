// Input front-ends beyond plain site lists.
#include <algorithm>
#include <cassert>
#include <cmath>
#include <fstream>
#include <sstream>
#include "Off3DFormatPicture.h"

// ---- OffSurfaceModelPicture (Off3DFormatPicture.cpp) ---------------------------
OffSurfaceModelPicture::OffSurfaceModelPicture(std::string filename,
                                               int renderSize, int label)
    : Picture(label), renderSize(renderSize), loaded(false) {
  // Off3DFormatPicture.cpp:53-70: "OFF", then counts, vertices, faces
  std::ifstream file(filename.c_str());
  std::string magic;
  if (!std::getline(file, magic))
    return;
  long nPoints = 0, nFaces = 0, nEdges = 0;
  if (!(file >> nPoints >> nFaces >> nEdges) || nPoints < 0 || nFaces < 0)
    return;
  points.resize((size_t)nPoints * 3);
  for (double &x : points)
    if (!(file >> x))
      return;
  surfaces.resize((size_t)nFaces * 3);
  for (long f = 0; f < nFaces; ++f) {
    int corners = 0;
    if (!(file >> corners >> surfaces[3 * f] >> surfaces[3 * f + 1] >>
          surfaces[3 * f + 2]))
      return;
    for (int k = 0; k < 3; ++k)
      if (surfaces[3 * f + k] < 0 || surfaces[3 * f + k] >= nPoints)
        return;
  }
  loaded = true;
}
OffSurfaceModelPicture::OffSurfaceModelPicture(const double *xyz, int nPoints,
                                               const int *triangles,
                                               int nTriangles, int renderSize,
                                               int label)
    : Picture(label), points(xyz, xyz + (size_t)nPoints * 3),
      surfaces(triangles, triangles + (size_t)nTriangles * 3),
      renderSize(renderSize), loaded(true) {}
std::string OffSurfaceModelPicture::identify() { return "OFF surface model"; }

// Off3DFormatPicture.cpp:73-82
void OffSurfaceModelPicture::normalize() {
  const size_t n = points.size() / 3;
  if (n == 0)
    return;
  double lo[3], hi[3];
  for (int a = 0; a < 3; ++a)
    lo[a] = hi[a] = points[a];
  for (size_t i = 1; i < n; ++i)
    for (int a = 0; a < 3; ++a) {
      lo[a] = std::min(lo[a], points[3 * i + a]);
      hi[a] = std::max(hi[a], points[3 * i + a]);
    }
  // the reference keeps the largest extent in a float
  const float scale =
      (float)std::max(hi[0] - lo[0], std::max(hi[1] - lo[1], hi[2] - lo[2]));
  assert(scale > 0);
  const float factor = renderSize / scale;
  for (size_t i = 0; i < n; ++i)
    for (int a = 0; a < 3; ++a)
      points[3 * i + a] = (points[3 * i + a] - 0.5 * (lo[a] + hi[a])) * factor;
}

// Off3DFormatPicture.cpp:84-92.  The reference takes Q from Armadillo's QR; here
// Q is built from Householder reflections (the textbook factorisation LAPACK
// also uses).  Sign conventions of that third-party routine are not pinned, so
// for one and the same random matrix the two may differ by column signs; any
// such Q is an equally valid draw of the augmentation.
void OffSurfaceModelPicture::random_rotation(RNG &rng) {
  double L[3][3];
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j)
      L[i][j] = rng.uniform();
  double Q[3][3] = {{1, 0, 0}, {0, 1, 0}, {0, 0, 1}};
  for (int k = 0; k < 2; ++k) { // reflect column k below the diagonal to zero
    double norm = 0;
    for (int i = k; i < 3; ++i)
      norm += L[i][k] * L[i][k];
    norm = std::sqrt(norm);
    if (norm == 0)
      continue;
    double v[3] = {0, 0, 0};
    for (int i = k; i < 3; ++i)
      v[i] = L[i][k];
    v[k] += L[k][k] >= 0 ? norm : -norm;
    double vv = 0;
    for (int i = k; i < 3; ++i)
      vv += v[i] * v[i];
    if (vv == 0)
      continue;
    for (int j = 0; j < 3; ++j) { // L <- H L, Q <- Q H with H = I - 2 v v' / v'v
      double dotL = 0, dotQ = 0;
      for (int i = k; i < 3; ++i) {
        dotL += v[i] * L[i][j];
        dotQ += Q[j][i] * v[i];
      }
      for (int i = k; i < 3; ++i) {
        L[i][j] -= 2 * v[i] * dotL / vv;
        Q[j][i] -= 2 * dotQ * v[i] / vv;
      }
    }
  }
  for (size_t i = 0; i < points.size() / 3; ++i) {
    const double x = points[3 * i], y = points[3 * i + 1], z = points[3 * i + 2];
    for (int j = 0; j < 3; ++j)
      points[3 * i + j] = x * Q[0][j] + y * Q[1][j] + z * Q[2][j];
  }
}
// Off3DFormatPicture.cpp:94-97
void OffSurfaceModelPicture::jiggle(RNG &rng, float alpha) {
  for (int a = 0; a < 3; ++a) {
    const double shift = renderSize * rng.uniform(-alpha, alpha);
    for (size_t i = 0; i < points.size() / 3; ++i)
      points[3 * i + a] += shift;
  }
}
// Off3DFormatPicture.cpp:99-105
void OffSurfaceModelPicture::affineTransform(RNG &rng, float alpha) {
  double L[3][3] = {{1, 0, 0}, {0, 1, 0}, {0, 0, 1}};
  for (int i = 0; i < 3; ++i)
    for (int j = 0; j < 3; ++j)
      L[i][j] += rng.uniform(-alpha, alpha);
  for (size_t i = 0; i < points.size() / 3; ++i) {
    const double x = points[3 * i], y = points[3 * i + 1], z = points[3 * i + 2];
    for (int j = 0; j < 3; ++j)
      points[3 * i + j] = x * L[0][j] + y * L[1][j] + z * L[2][j];
  }
}

namespace {
// voxel index along one axis (Off3DFormatPicture.cpp:5-8): the lattice is
// centred on the origin, positions outside are clamped onto its faces
inline int voxelOf(float coord, int side) {
  return std::max(0, std::min(side - 1, (int)(coord + 0.5 * side)));
}
// 0, 1, 2, ... and then `end` itself: the sample positions along a side of
// length `end` (the reference's `x = min(x + 1, end) + (x == end)` stepping)
template <class Visit> inline void unitSteps(float end, Visit visit) {
  for (float x = 0; x <= end;) {
    visit(x);
    if (x == end)
      break;
    x = std::min(x + 1, end);
  }
}
} // namespace

// Off3DFormatPicture.cpp:12-50,107-123.  A triangle {a, a + u, a + v} is
// sampled on a unit-spaced net: rows at unit steps of height above the side u,
// points at unit steps along each row, both closed with the exact end point.
// All of it in single precision and in the reference's order of operations,
// because which voxel a borderline sample falls into depends on the rounding.
void OffSurfaceModelPicture::codifyInputData(SparseGrid &grid,
                                             std::vector<float> &features,
                                             int &nSpatialSites,
                                             int spatialSize) {
  features.push_back(0); // background feature
  grid.backgroundCol = nSpatialSites++;
  const int64_t n = spatialSize;
  for (size_t t = 0; t < surfaces.size() / 3; ++t) {
    const double *A = &points[3 * (size_t)surfaces[3 * t]];
    const double *B = &points[3 * (size_t)surfaces[3 * t + 1]];
    const double *C = &points[3 * (size_t)surfaces[3 * t + 2]];
    const float a[3] = {(float)A[0], (float)A[1], (float)A[2]};
    float u[3] = {(float)(B[0] - A[0]), (float)(B[1] - A[1]), (float)(B[2] - A[2])};
    float v[3] = {(float)(C[0] - A[0]), (float)(C[1] - A[1]), (float)(C[2] - A[2])};
    const float base = powf(u[0] * u[0] + u[1] * u[1] + u[2] * u[2], 0.5);
    for (float &x : u)
      x /= base;
    const float offset = u[0] * v[0] + u[1] * v[1] + u[2] * v[2];
    for (int k = 0; k < 3; ++k)
      v[k] -= offset * u[k];
    const float height = powf(v[0] * v[0] + v[1] * v[1] + v[2] * v[2], 0.5);
    for (float &x : v)
      x /= height;
    // now a + b u + h v, 0 <= h <= height, 0 <= b - offset h / height <= base (1 - h / height)
    unitSteps(height, [&](float h) {
      const float rowLength = base * (1 - h / height);
      unitSteps(rowLength, [&](float b) {
        const float along = b + offset * h / height;
        const float p0 = a[0] + along * u[0] + h * v[0];
        const float p1 = a[1] + along * u[1] + h * v[1];
        const float p2 = a[2] + along * u[2] + h * v[2];
        const int64_t key = (voxelOf(p0, spatialSize) * n + voxelOf(p1, spatialSize)) * n +
                            voxelOf(p2, spatialSize);
        if (grid.mp.find(key) == grid.mp.end()) {
          grid.mp[key] = nSpatialSites++;
          features.push_back(1);
        }
      });
    });
  }
}

// Off3DFormatPicture.cpp:125-134
Picture *OffSurfaceModelPicture::distort(RNG &rng, batchType type) {
  OffSurfaceModelPicture *pic = new OffSurfaceModelPicture(*this);
  pic->random_rotation(rng);
  pic->normalize();
  if (type == TRAINBATCH) {
    pic->affineTransform(rng, 0.2);
    pic->jiggle(rng, 0.2);
  }
  return pic;
}
