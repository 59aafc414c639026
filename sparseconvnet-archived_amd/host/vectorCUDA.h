// Host/device vector with the reference's vectorCUDA<T> surface
// (vectorCUDA.h:6-40): the data lives either in a std::vector (onGPU ==
// false) or in HBM (onGPU == true); hVector() and dPtr() migrate it on demand
// and device storage only ever grows (vectorCUDA.cu:171-185).  Device memory
// and copies go through the C ABI of libscn_hip.so.  The type keeps the
// reference's name so that driver code compiles unchanged.
#pragma once
#include <vector>
#include "scn_hip.h"

// The stream object layer constructors take (utilities.h:105-112).  Every
// instance owns one library context, i.e. one HIP stream on the GPU.
class cudaMemStream {
public:
  scn_ctx *ctx;
  cudaMemStream();
  ~cudaMemStream();
  cudaMemStream(const cudaMemStream &) = delete;
  cudaMemStream &operator=(const cudaMemStream &) = delete;
  void *stream() const;
  void synchronize() const;
};

// the context vectorCUDA objects use when no stream is named: the one of the
// oldest live cudaMemStream (the net's own memStream)
scn_ctx *scnDefaultContext();
void scnCheck(int rc, const char *file, int line);
void scnExit(int code); // flush, then leave without static destructors
#define SCN_CHECKED(expr) scnCheck((expr), __FILE__, __LINE__)

template <typename t> class vectorCUDA {
private:
  t *d_vec;
  size_t dsize;       // size while on the GPU
  size_t dAllocated;  // elements allocated on the GPU (>= dsize)
  std::vector<t> vec;
  void toCPU(scn_ctx *ctx);
  void toGPU(scn_ctx *ctx);

public:
  vectorCUDA(bool onGPU = true, size_t dsize = 0);
  ~vectorCUDA();
  vectorCUDA(const vectorCUDA &) = delete;
  vectorCUDA &operator=(const vectorCUDA &) = delete;
  vectorCUDA(vectorCUDA &&o);
  bool onGPU;
  void copyToCPU();
  void copyToGPU();
  void copyToCPUAsync(cudaMemStream &memStream);
  void copyToGPUAsync(cudaMemStream &memStream);
  t *&dPtr();
  std::vector<t> &hVector();
  unsigned int size();
  void setZero();
  void setZero(cudaMemStream &memStream);
  void setConstant(float a = 0);
  void setUniform(float a = 0, float b = 1);
  void resize(int n);
  // 64-bit clean variants: the reference's int sizes overflow on feature
  // matrices beyond 2^31 elements (large 3-D batches)
  void resize64(size_t n);
  size_t size64();
};
