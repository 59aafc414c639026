// Raster images as input samples: the array-backed half of the reference's
// OpenCVPicture (OpenCVPicture.h:9-50) -- the form its MNIST and CIFAR
// readers use -- without OpenCV.  A picture holds float pixels (0..255) in
// `mat`; pixels that differ from the background colour by more than 2 in some
// channel become active sites, with features (colour - background) /
// max(255 - background, background).
//
// Not available: everything the reference delegates to OpenCV (reading image
// files, affine / elastic / colour distortions, blur, noise); those are
// training-time augmentations or decoders.  distort() returns a copy, jiggled
// by `trainingJiggle` pixels for a training batch (mnist.cpp's distortion).
#pragma once
#include <string>
#include <vector>
#include "Picture.h"

// the few members of cv::Mat the reference's readers touch (CV_32FC(n) only)
struct FloatMat {
  int rows = 0, cols = 0;
  unsigned char *data = nullptr; // rows x cols x channels floats
  void create(int rows_, int cols_, int channels_) {
    rows = rows_;
    cols = cols_;
    ch = channels_;
    store.assign((size_t)rows * cols * ch, 0.f);
    data = reinterpret_cast<unsigned char *>(store.data());
  }
  int channels() const { return ch; }
  bool empty() const { return store.empty(); }
  FloatMat() {}
  FloatMat(const FloatMat &o) { *this = o; }
  FloatMat &operator=(const FloatMat &o) {
    rows = o.rows;
    cols = o.cols;
    ch = o.ch;
    store = o.store;
    data = store.empty() ? nullptr : reinterpret_cast<unsigned char *>(store.data());
    return *this;
  }

private:
  int ch = 0;
  std::vector<float> store;
};

class OpenCVPicture : public Picture {
  float scaleUCharColor(float col);

public:
  int xOffset; // shift to the right
  int yOffset; // shift down
  int backgroundColor;
  int trainingJiggle; // distort(): +-pixels for a training batch (0: none)
  FloatMat mat;
  // note the reference's argument order: mat.create(xSize, ySize, ...) makes
  // xSize the number of ROWS (OpenCVPicture.cpp:9-15)
  OpenCVPicture(int xSize, int ySize, int nInputFeatures,
                unsigned char backgroundColor, int label_ = -1);
  Picture *distort(RNG &rng, batchType type = TRAINBATCH);
  void codifyInputData(SparseGrid &grid, std::vector<float> &features,
                       int &nSpatialSites, int spatialSize);
  void jiggle(RNG &rng, int offlineJiggle);
  int area(); // number of non-background pixels
  std::string identify();
};

// MNIST idx files (SpatiallySparseDatasetMnist.cpp:5-60): images appended as
// one-channel pictures with background 0, then their labels.  Return the
// number of pictures appended, -1 when a file cannot be read.
int loadMnist(const char *imagesFile, const char *labelsFile,
              std::vector<Picture *> &characters);
// CIFAR-10 binary batches (SpatiallySparseDatasetCIFAR10.cpp:6-28): 32 x 32
// pictures of 3 channels stored blue, green, red, background 128.
int readCIFAR10File(std::vector<Picture *> &characters, const char *filename);
// CIFAR-100 (SpatiallySparseDatasetCIFAR100.cpp:6-29): a coarse and a fine
// label byte per record, the fine one is the class.
int readCIFAR100File(std::vector<Picture *> &characters, const char *filename);
