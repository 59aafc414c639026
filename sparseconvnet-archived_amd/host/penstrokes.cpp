// OnlineHandwritingPicture: see the header.  Arithmetic follows the reference
// operation by operation (which values are double, which float, where a
// conversion truncates), because cell membership depends on it.
#include "OnlineHandwritingPicture.h"
#include <math.h>
#include <stdlib.h>
#include <algorithm>
#include <fstream>
#include <iterator>
#include <stdexcept>

const int OnlineHandwritingEncodingSize[9] = {1, 8, 4, 3, 6, 14, 32, 1, 1 + 2};

OnlineHandwritingPicture::OnlineHandwritingPicture(int renderSize,
                                                   OnlineHandwritingEncoding enc,
                                                   int label, float penSpeed3d)
    : Picture(label), penSpeed3d(penSpeed3d), offset3d(0),
      renderSize(renderSize), enc(enc) {}

void OnlineHandwritingPicture::addStroke(const double *xy, int nPoints) {
  if (nPoints <= 0)
    return; // (the reference would index an empty matrix)
  ops.emplace_back(xy, xy + 2 * (size_t)nPoints);
}

std::string OnlineHandwritingPicture::identify() {
  return "pen strokes, label " + std::to_string(label);
}

// OnlineHandwritingPicture.cpp:9-25
void OnlineHandwritingPicture::normalize() {
  if (ops.empty())
    return;
  double lo[2] = {HUGE_VAL, HUGE_VAL}, hi[2] = {-HUGE_VAL, -HUGE_VAL};
  for (auto &s : ops)
    for (size_t i = 0; i < s.size(); ++i) {
      lo[i & 1] = std::min(lo[i & 1], s[i]);
      hi[i & 1] = std::max(hi[i & 1], s[i]);
    }
  // float scale = (max - min).max()
  const float scale = (float)std::max(hi[0] - lo[0], hi[1] - lo[1]);
  if (!(scale > 0))
    throw std::runtime_error("OnlineHandwritingPicture::normalize: all points coincide");
  const double mid[2] = {0.5 * (lo[0] + hi[0]), 0.5 * (lo[1] + hi[1])};
  // ops[i] *= renderSize / scale: int / float = float, then double * float
  const float factor = renderSize / scale;
  for (auto &s : ops)
    for (size_t i = 0; i < s.size(); ++i)
      s[i] = (s[i] - mid[i & 1]) * factor;
}

// OnlineHandwritingPicture.cpp:27-53
std::vector<double> constantSpeed(const std::vector<double> &stroke,
                                  float density, int multiplier) {
  const int rows = (int)(stroke.size() / 2);
  std::vector<float> lengths(rows);
  lengths[0] = 0;
  for (int i = 1; i < rows; i++) {
    const double dx = stroke[2 * i] - stroke[2 * i - 2];
    const double dy = stroke[2 * i + 1] - stroke[2 * i - 1];
    lengths[i] = (float)(lengths[i - 1] + pow(pow(dx, 2) + pow(dy, 2), 0.5));
  }
  const float lTotal = lengths[rows - 1];
  int n = (int)(0.5 + lTotal / density);
  n *= multiplier;
  std::vector<double> r(2 * (size_t)(n + 1));
  int j = 0;
  r[0] = stroke[0];
  r[1] = stroke[1];
  for (int i = 1; i <= n; i++) {
    // (j + 1 stays a valid row: rounding could otherwise walk one past the end)
    while (j + 2 < rows && n * lengths[j + 1] < i * lTotal)
      j++;
    const float alpha =
        (lengths[j + 1] - i * lTotal / n) / (lengths[j + 1] - lengths[j]);
    r[2 * i] = stroke[2 * j] * alpha + stroke[2 * j + 2] * (1 - alpha);
    r[2 * i + 1] = stroke[2 * j + 1] * alpha + stroke[2 * j + 3] * (1 - alpha);
  }
  return r;
}

namespace {
// the row of cell n, created (with zero features) when the cell is new
int cell_row(SparseGrid &grid, std::vector<float> &features, int &nSpatialSites,
             int nInputFeatures, int64_t n) {
  auto it = grid.mp.find(n);
  if (it != grid.mp.end())
    return it->second;
  const int row = nSpatialSites++;
  grid.mp[n] = row;
  features.resize((size_t)nInputFeatures * nSpatialSites, 0);
  return row;
}
} // namespace

// OnlineHandwritingPicture.cpp:77-271
void OnlineHandwritingPicture::codifyInputData(SparseGrid &grid,
                                               std::vector<float> &features,
                                               int &nSpatialSites,
                                               int spatialSize) {
  if (enc >= LogSignature1 && enc <= LogSignature4)
    throw std::runtime_error(
        "OnlineHandwritingPicture: the LogSignature encodings need the "
        "reference's log-signature basis tables, which this build does not "
        "carry");
  const int nInputFeatures = OnlineHandwritingEncodingSize[enc];
  grid.backgroundCol = nSpatialSites++; // background feature
  features.resize((size_t)nInputFeatures * nSpatialSites, 0);
  const float piBy4 = (float)(3.1415926536 / 4);
  const bool volume = enc == SpaceTime3d || enc == VectorSpaceTime3d;
  // the last sample of a stroke has no direction of travel
  const bool needsDirection =
      enc == Octogram || enc == UndirectedOctogram || enc == VectorSpaceTime3d;

  std::vector<std::vector<double>> csp;
  int cspLengths = 0;
  for (auto &s : ops) {
    csp.push_back(constantSpeed(s, 0.1f));
    cspLengths += (int)(csp.back().size() / 2);
  }
  int z = 0;
  for (auto &c : csp) {
    const int rows = (int)(c.size() / 2);
    const int last = needsDirection ? rows - 1 : rows;
    for (int j = 0; j < last; ++j) {
      const int a0 = (int)(c[2 * j] + spatialSize / 2.0);
      const int a1 = (int)(c[2 * j + 1] + spatialSize / 2.0);
      int64_t n = (int64_t)a0 * spatialSize + a1;
      bool inside = a0 >= 0 && a1 >= 0 && a0 < spatialSize && a1 < spatialSize;
      if (volume) {
        // int * float + float, int * float, + int: all in float, then truncated
        const int a2 = (int)(renderSize * ((z - cspLengths / 2) * penSpeed3d + offset3d) +
                             spatialSize / 2);
        z++;
        inside = inside && a2 >= 0 && a2 < spatialSize;
        n = n * spatialSize + a2;
      }
      if (!inside)
        continue;
      const int row = cell_row(grid, features, nSpatialSites, nInputFeatures, n);
      float *f = &features[(size_t)nInputFeatures * row];
      if (enc == Simple || enc == SpaceTime3d) {
        ++f[0];
        continue;
      }
      float dx = (float)(c[2 * j + 2] - c[2 * j]);
      float dy = (float)(c[2 * j + 3] - c[2 * j + 1]);
      const float m = powf(dx * dx + dy * dy, 0.5f);
      dx /= m; // (coincident samples: NaN, which passes no test below)
      dy /= m;
      if (enc == VectorSpaceTime3d) {
        f[0]++;
        f[1] += dx;
        f[2] += dy;
      } else if (enc == Octogram) {
        for (int k = 0; k < 8; k++) {
          const float alpha =
              1 - acosf(cosf(k * piBy4) * dx + sinf(k * piBy4) * dy) / piBy4;
          if (alpha > 0)
            f[k] += alpha;
        }
      } else { // UndirectedOctogram
        for (int k = 0; k < 4; k++) {
          const float alpha =
              1 - acosf(fabsf(cosf(k * piBy4) * dx + sinf(k * piBy4) * dy)) / piBy4;
          if (alpha > 0)
            f[k] += alpha;
        }
      }
    }
  }
}

// OnlineHandwritingTriangularPicture.cpp:216-243 (the only definition of
// distort in the reference).  Its `if (r = 2)` assigns: the shear chosen for
// r == 0 or 1 is always overwritten by the rotation, which is kept here.
Picture *OnlineHandwritingPicture::distort(RNG &rng, batchType type) {
  OnlineHandwritingPicture *pic = new OnlineHandwritingPicture(*this);
  if (type == TRAINBATCH) {
    double aff[2][2] = {{1, 0}, {0, 1}};
    aff[0][0] += rng.uniform(-0.3f, 0.3f) / 1; // x stretch
    aff[1][1] += rng.uniform(-0.3f, 0.3f) / 1; // y stretch
    (void)rng.randint(3);
    const float alpha = rng.uniform(-0.3f, 0.3f) / 1;
    const double x[2][2] = {{cos(alpha), -sin(alpha)}, {sin(alpha), cos(alpha)}};
    double m[2][2];
    for (int i = 0; i < 2; ++i)
      for (int j = 0; j < 2; ++j)
        m[i][j] = aff[i][0] * x[0][j] + aff[i][1] * x[1][j];
    double y[2];
    y[0] = renderSize * rng.uniform(-0.1875f, 0.1875f) / 1;
    y[1] = renderSize * rng.uniform(-0.1875f, 0.1875f) / 1;
    for (auto &s : pic->ops)
      for (size_t i = 0; i + 1 < s.size(); i += 2) {
        const double px = s[i], py = s[i + 1];
        s[i] = px * m[0][0] + py * m[1][0] + y[0];
        s[i + 1] = px * m[0][1] + py * m[1][1] + y[1];
      }
    pic->offset3d = rng.uniform(-0.1f, 0.1f);
  }
  return pic;
}

// SpatiallySparseDatasetPenDigits.cpp:15-63
int readPenDigitsFile(std::vector<Picture *> &characters, const char *filename,
                      int renderSize, OnlineHandwritingEncoding enc) {
  std::ifstream f(filename, std::ios::in | std::ios::binary);
  if (!f)
    return -1;
  std::vector<std::string> data;
  std::copy(std::istream_iterator<std::string>(f),
            std::istream_iterator<std::string>(), std::back_inserter(data));
  int pen = 0, added = 0;
  OnlineHandwritingPicture *character =
      new OnlineHandwritingPicture(renderSize, enc, -1);
  std::vector<double> stroke;
  auto finish = [&]() {
    character->normalize();
    characters.push_back(character);
    ++added;
  };
  for (size_t i = 0; i < data.size(); i++) {
    if (data[i] == ".COMMENT") {
      if (character->ops.size() > 0) {
        finish();
        character = new OnlineHandwritingPicture(renderSize, enc, -1);
      }
      if (i + 1 < data.size())
        character->label = atoi(data[i + 1].c_str());
    }
    if (data[i] == ".PEN_UP") {
      pen = 0;
      character->addStroke(stroke.data(), (int)(stroke.size() / 2));
      stroke.clear();
    }
    if (pen == 1 && i + 1 < data.size()) {
      // the file has "x y"; the picture's first coordinate is -(second number)
      const short y = (short)atoi(data[i].c_str());
      i++;
      const short x = (short)-atoi(data[i].c_str());
      stroke.push_back(x);
      stroke.push_back(y);
    }
    if (data[i] == ".PEN_DOWN")
      pen = 1;
  }
  if (character->ops.size() > 0)
    finish();
  else
    delete character;
  return added;
}
