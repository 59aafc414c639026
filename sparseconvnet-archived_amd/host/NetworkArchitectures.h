// Canned nets built from addLeNetLayerMP (NetworkArchitectures.h;
// NetworkArchitectures.cpp:3-68).  l+1 conv levels, k*(level+1) features.
#pragma once
#include "SparseConvNet.h"

// C3 first, then C2, MP3/2 between levels
class DeepCNet : public SparseConvNet {
public:
  DeepCNet(int dimension, int l, int k, ActivationFunction fn,
           int nInputFeatures, int nClasses, float p = 0.0f,
           int cudaDevice = -1, int nTop = 1);
};
// C2 - MP3/2 levels
class DeepC2 : public SparseConvNet {
public:
  DeepC2(int dimension, int l, int k, ActivationFunction fn,
         int nInputFeatures, int nClasses, float p = 0.0f, int cudaDevice = -1,
         int nTop = 1);
};
// C2 + 1x1 NiN per level
class DeepCNiN : public SparseConvNet {
public:
  DeepCNiN(int dimension, int l, int k, ActivationFunction fn,
           int nInputFeatures, int nClasses, float p = 0.0f,
           int cudaDevice = -1, int nTop = 1);
};
class DeepC2C2 : public SparseConvNet {
public:
  DeepC2C2(int dimension, int l, int k, ActivationFunction fn,
           int nInputFeatures, int nClasses, float p = 0.0f,
           int cudaDevice = -1, int nTop = 1);
};
class DeepC3C3 : public SparseConvNet {
public:
  DeepC3C3(int dimension, int l, int k, ActivationFunction fn,
           int nInputFeatures, int nClasses, float p = 0.0f,
           int cudaDevice = -1, int nTop = 1);
};
// 'valid' 3x3 convolutions (minActiveInputs = -1), 2-D only
class DeepC3C3Valid : public SparseConvNet {
public:
  DeepC3C3Valid(int dimension, int l, int k, ActivationFunction fn,
                int nInputFeatures, int nClasses, float p = 0.0f,
                int cudaDevice = -1, int nTop = 1);
};
