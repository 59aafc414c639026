// OpenCVPicture without OpenCV: see the header.
#include "OpenCVPicture.h"
#include <stdlib.h>
#include <algorithm>
#include <cmath>
#include <fstream>

float OpenCVPicture::scaleUCharColor(float col) { // OpenCVPicture.cpp:4-7
  float div = std::max(255 - backgroundColor, backgroundColor);
  return (col - backgroundColor) / div;
}

OpenCVPicture::OpenCVPicture(int xSize, int ySize, int nInputFeatures,
                             unsigned char backgroundColor, int label)
    : Picture(label), backgroundColor(backgroundColor), trainingJiggle(0) {
  xOffset = -xSize / 2;
  yOffset = -ySize / 2;
  mat.create(xSize, ySize, nInputFeatures);
}

void OpenCVPicture::jiggle(RNG &rng, int offlineJiggle) { // OpenCVPicture.cpp:22-25
  xOffset += rng.randint(offlineJiggle * 2 + 1) - offlineJiggle;
  yOffset += rng.randint(offlineJiggle * 2 + 1) - offlineJiggle;
}

Picture *OpenCVPicture::distort(RNG &rng, batchType type) {
  OpenCVPicture *pic = new OpenCVPicture(*this);
  if (type == TRAINBATCH && trainingJiggle > 0)
    pic->jiggle(rng, trainingJiggle);
  return pic;
}

std::string OpenCVPicture::identify() {
  return "image " + std::to_string(mat.cols) + "x" + std::to_string(mat.rows) +
         ", label " + std::to_string(label);
}

int OpenCVPicture::area() {
  const float *p = reinterpret_cast<const float *>(mat.data);
  const int ch = mat.channels();
  int n = 0;
  for (int k = 0; k < mat.rows * mat.cols; ++k) {
    bool interesting = false;
    for (int i = 0; i < ch; i++)
      if (std::abs(p[k * ch + i] - backgroundColor) > 2)
        interesting = true;
    n += interesting;
  }
  return n;
}

// OpenCVPicture.cpp:368-402
void OpenCVPicture::codifyInputData(SparseGrid &grid,
                                    std::vector<float> &features,
                                    int &nSpatialSites, int spatialSize) {
  const int ch = mat.channels();
  for (int i = 0; i < ch; i++)
    features.push_back(0); // background feature
  grid.backgroundCol = nSpatialSites++;
  // if x0 <= x < x1 and y0 <= y < y1 then pixel (x, y) is in the net's field
  const int x0 = std::max(0, -xOffset - spatialSize / 2);
  const int x1 = std::min(mat.cols, spatialSize - xOffset - spatialSize / 2);
  const int y0 = std::max(0, -yOffset - spatialSize / 2);
  const int y1 = std::min(mat.rows, spatialSize - yOffset - spatialSize / 2);
  const float *matData = reinterpret_cast<const float *>(mat.data);
  for (int x = x0; x < x1; x++) {
    for (int y = y0; y < y1; y++) {
      const int j = x * ch + y * ch * mat.cols;
      bool interestingPixel = false;
      for (int i = 0; i < ch; i++)
        if (std::abs(matData[i + j] - backgroundColor) > 2)
          interestingPixel = true;
      if (interestingPixel) {
        const int n = (x + xOffset + spatialSize / 2) * spatialSize +
                      (y + yOffset + spatialSize / 2);
        grid.mp[n] = nSpatialSites++;
        for (int i = 0; i < ch; i++)
          features.push_back(scaleUCharColor(matData[i + j]));
      }
    }
  }
}

static int bigEndianInt(std::istream &f, bool &ok) {
  unsigned char b[4];
  if (!f.read((char *)b, 4)) {
    ok = false;
    return 0;
  }
  return (b[0] << 24) | (b[1] << 16) | (b[2] << 8) | b[3];
}

int loadMnist(const char *imagesFile, const char *labelsFile,
              std::vector<Picture *> &characters) {
  std::ifstream f(imagesFile, std::ios::in | std::ios::binary);
  std::ifstream g(labelsFile, std::ios::in | std::ios::binary);
  if (!f || !g)
    return -1;
  bool ok = true;
  (void)bigEndianInt(f, ok); // magic
  const int n1 = bigEndianInt(f, ok), n2 = bigEndianInt(f, ok),
            n3 = bigEndianInt(f, ok);
  (void)bigEndianInt(g, ok);
  const int nLabels = bigEndianInt(g, ok);
  if (!ok || n1 < 0 || n2 <= 0 || n3 <= 0 || n2 > 4096 || n3 > 4096 ||
      nLabels < n1)
    return -1;
  std::vector<unsigned char> bitmap((size_t)n2 * n3);
  const size_t first = characters.size();
  for (int i1 = 0; i1 < n1; i1++) {
    char l;
    if (!f.read((char *)bitmap.data(), n2 * n3) || !g.read(&l, 1)) {
      for (size_t k = first; k < characters.size(); ++k)
        delete characters[k];
      characters.resize(first);
      return -1;
    }
    OpenCVPicture *character = new OpenCVPicture(n2, n3, 1, 0, l);
    float *matData = reinterpret_cast<float *>(character->mat.data);
    for (int i = 0; i < n2 * n3; i++)
      matData[i] = bitmap[i];
    characters.push_back(character);
  }
  return n1;
}

// A record is `labelBytes` label bytes, the last of which is the class, then
// the three colour planes: CIFAR-10 has one label byte, CIFAR-100 a coarse
// and a fine one (SpatiallySparseDatasetCIFAR100.cpp:13-15 keeps the fine).
static int read_cifar_file(std::vector<Picture *> &characters,
                           const char *filename, int labelBytes) {
  std::ifstream file(filename, std::ios::in | std::ios::binary);
  if (!file)
    return -1;
  unsigned char labels[2];
  int added = 0;
  while (file.read((char *)labels, labelBytes)) {
    const unsigned char label = labels[labelBytes - 1];
    unsigned char bitmap[3072];
    if (!file.read((char *)bitmap, 3072))
      break; // a truncated record is dropped
    OpenCVPicture *character = new OpenCVPicture(32, 32, 3, 128, label);
    float *matData = reinterpret_cast<float *>(character->mat.data);
    for (int x = 0; x < 32; x++)
      for (int y = 0; y < 32; y++)
        for (int c = 0; c < 3; c++)
          matData[y * 96 + x * 3 + (2 - c)] = bitmap[c * 1024 + y * 32 + x];
    characters.push_back(character);
    ++added;
  }
  return added;
}
int readCIFAR10File(std::vector<Picture *> &characters, const char *filename) {
  return read_cifar_file(characters, filename, 1);
}
int readCIFAR100File(std::vector<Picture *> &characters, const char *filename) {
  return read_cifar_file(characters, filename, 2);
}
