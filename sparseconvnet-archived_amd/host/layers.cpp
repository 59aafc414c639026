// Layer classes.  preprocess() issues the rule-book kernels, forwards() the
// feature kernels, backwards() the gradient kernels and the weight update, all
// through the C ABI of libscn_hip.so on the net's stream.
#include <cassert>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include "SpatiallySparseLayer.h"

static void unsupported(const char *what) {
  std::fprintf(stderr, "%s is not implemented in this library\n", what);
  scnExit(EXIT_FAILURE);
}

SpatiallySparseLayer::SpatiallySparseLayer(cudaMemStream &memStream)
    : memStream(memStream) {}
SpatiallySparseLayer::~SpatiallySparseLayer() {}
void SpatiallySparseLayer::loadWeightsFromStream(std::ifstream &, bool) {}
void SpatiallySparseLayer::putWeightsToStream(std::ofstream &, bool) {}
void SpatiallySparseLayer::scaleWeights(SpatiallySparseBatchInterface &,
                                        SpatiallySparseBatchInterface &,
                                        float &, bool) {}
void SpatiallySparseLayer::backwards(SpatiallySparseBatch &,
                                     SpatiallySparseBatchInterface &,
                                     SpatiallySparseBatchInterface &, float,
                                     float) {}

// preprocess() runs on the batch slot's own stream when it has one, so that
// rule books of several batches are built side by side
static scn_ctx *pre_ctx(SpatiallySparseBatch &batch, cudaMemStream &ms) {
  return batch.preprocessStream ? batch.preprocessStream->ctx : ms.ctx;
}
// forwards() runs on the batch's forward lane when the net has given it one
static cudaMemStream &fwd_stream(SpatiallySparseBatch &batch, cudaMemStream &ms) {
  return batch.forwardStream ? *batch.forwardStream : ms;
}

// the output interface's own grids object, created on first use and kept for
// later batches (its tables only grow)
static scn_grids *own_grids(scn_ctx *ctx,
                            SpatiallySparseBatchInterface &output) {
  if (!output.deviceGrids || !output.ownsDeviceGrids) {
    scn_grids *g = nullptr;
    SCN_CHECKED(scn_grids_create(ctx, &g));
    output.deviceGrids = g;
    output.ownsDeviceGrids = true;
  }
  return output.deviceGrids;
}
// a layer that leaves the grids alone passes its input's object on
// (NetworkInNetworkLayer.cu:152: output.grids = input.grids)
static void share_grids(SpatiallySparseBatchInterface &input,
                        SpatiallySparseBatchInterface &output) {
  if (output.deviceGrids && output.ownsDeviceGrids)
    scn_grids_destroy(scnDefaultContext(), output.deviceGrids);
  output.deviceGrids = input.deviceGrids;
  output.ownsDeviceGrids = false;
}

static void fill_rules(scn_ctx *ctx, SpatiallySparseBatchInterface &input,
                       SpatiallySparseBatchInterface &output, int64_t nRules) {
  output.rules.copyToGPU();
  output.rules.resize64((size_t)nRules);
  SCN_CHECKED(scn_rules_fill(ctx, input.deviceGrids, output.deviceGrids,
                             output.rules.dPtr(), nRules));
}

// materialise the im2col-like matrix of a convolution's output interface
static void gather_now(cudaMemStream &ms, SpatiallySparseBatchInterface &input,
                       SpatiallySparseBatchInterface &output) {
  const size_t nIn = input.featuresPresent.size();
  const size_t width = output.featuresPresent.size(); // fs * nIn
  output.sub->features.resize64((size_t)output.nSpatialSites * width);
  SCN_CHECKED(scn_gather_rows(ms.ctx, input.sub->features.dPtr(),
                              output.sub->features.dPtr(), output.rules.dPtr(),
                              (int64_t)output.nSpatialSites * (width / nIn),
                              (int)nIn));
  output.deferredGatherFrom = nullptr;
}

// ConvolutionalLayer::backwards (ConvolutionalLayer.cu:134-147): scatter-add of
// the gathered matrix's gradient through the rules
static void conv_backwards(SpatiallySparseBatchInterface &input,
                           SpatiallySparseBatchInterface &output,
                           cudaMemStream &ms) {
  if (!input.backpropErrors)
    return;
  const size_t nIn = input.featuresPresent.size();
  const size_t width = output.featuresPresent.size();
  input.sub->dfeatures.resize64((size_t)input.nSpatialSites * nIn);
  input.sub->dfeatures.setZero(ms);
  SCN_CHECKED(scn_gather_rows_backward(
      ms.ctx, input.sub->dfeatures.dPtr(), output.sub->dfeatures.dPtr(),
      output.rules.dPtr(), (int64_t)output.nSpatialSites * (width / nIn),
      (int)nIn));
}

// featuresPresent of a convolution's output: fs copies of the input's list,
// shifted by nf per copy (ConvolutionalLayer.cu:74-80)
static void convolutionFeaturesPresent(std::vector<int> &src,
                                       std::vector<int> &dest, int nf, int nfp,
                                       int nCopies) {
  dest.resize((size_t)nfp * nCopies);
  for (int i = 0; i < nfp * nCopies; ++i)
    dest[i] = src[i % nfp] + nf * (i / nfp);
}

// ---- ConvolutionalLayer (ConvolutionalLayer.cu:82-156) ------------------------
ConvolutionalLayer::ConvolutionalLayer(cudaMemStream &memStream,
                                       int filterSize, int filterStride,
                                       int dimension, int nFeaturesIn,
                                       int minActiveInputs)
    : SpatiallySparseLayer(memStream), inSpatialSize(0), outSpatialSize(0),
      filterSize(filterSize), filterStride(filterStride), dimension(dimension),
      nFeaturesIn(nFeaturesIn), minActiveInputs(minActiveInputs),
      deferGather(false) {
  fs = ipow(filterSize, dimension);
  nFeaturesOut = fs * nFeaturesIn;
  std::cout << "Convolution " << filterSize << "^" << dimension << "x"
            << nFeaturesIn << "->" << nFeaturesOut;
  if (filterStride != 1)
    std::cout << " stride:" << filterStride;
  if (minActiveInputs != 1)
    std::cout << " minActiveInputs:" << minActiveInputs;
  std::cout << std::endl;
}
void ConvolutionalLayer::preprocess(SpatiallySparseBatch &batch,
                                    SpatiallySparseBatchInterface &input,
                                    SpatiallySparseBatchInterface &output) {
  scn_ctx *ctx = pre_ctx(batch, memStream);
  assert(input.nFeatures == nFeaturesIn);
  assert(input.spatialSize >= filterSize);
  assert((input.spatialSize - filterSize) % filterStride == 0);
  output.nFeatures = nFeaturesOut;
  output.spatialSize = (input.spatialSize - filterSize) / filterStride + 1;
  output.backpropErrors = input.backpropErrors;
  int64_t n = 0;
  SCN_CHECKED(scn_rules_square_plan(ctx, input.deviceGrids,
                                    own_grids(ctx, output), inSpatialSize,
                                    outSpatialSize, filterSize, filterStride,
                                    minActiveInputs, &n));
  output.nSpatialSites = (int)n;
  fill_rules(ctx, input, output, n * fs);
  convolutionFeaturesPresent(input.featuresPresent.hVector(),
                             output.featuresPresent.hVector(), input.nFeatures,
                             (int)input.featuresPresent.size(), fs);
}
void ConvolutionalLayer::forwards(SpatiallySparseBatch &batch,
                                  SpatiallySparseBatchInterface &input,
                                  SpatiallySparseBatchInterface &output) {
  // (the backward pass needs the gathered matrix: no deferral while training)
  if (deferGather && batch.type != TRAINBATCH) {
    output.deferredGatherFrom = &input; // the following NiN layer gathers
    return;
  }
  gather_now(fwd_stream(batch, memStream), input, output);
}
void ConvolutionalLayer::backwards(SpatiallySparseBatch &batch,
                                   SpatiallySparseBatchInterface &input,
                                   SpatiallySparseBatchInterface &output,
                                   float learningRate, float momentum) {
  (void)batch, (void)learningRate, (void)momentum;
  conv_backwards(input, output, memStream);
}
int ConvolutionalLayer::calculateInputSpatialSize(int outputSpatialSize) {
  outSpatialSize = outputSpatialSize;
  inSpatialSize = filterSize + (outputSpatialSize - 1) * filterStride;
  std::cout << "-(C" << filterSize;
  if (filterStride != 1)
    std::cout << "/" << filterStride;
  std::cout << ")-" << inSpatialSize;
  return inSpatialSize;
}

// ---- ConvolutionalTriangularLayer (ConvolutionalTriangularLayer.cu) -----------
ConvolutionalTriangularLayer::ConvolutionalTriangularLayer(
    cudaMemStream &memStream, int filterSize, int filterStride, int dimension,
    int nFeaturesIn, int minActiveInputs)
    : SpatiallySparseLayer(memStream), inSpatialSize(0), outSpatialSize(0),
      filterSize(filterSize), filterStride(filterStride), dimension(dimension),
      nFeaturesIn(nFeaturesIn), minActiveInputs(minActiveInputs),
      deferGather(false) {
  fs = triangleSize(filterSize, dimension);
  nFeaturesOut = fs * nFeaturesIn;
  std::cout << dimension
            << "D ConvolutionalTriangularLayer side-length=" << filterSize
            << " " << nFeaturesIn << "x" << fs << "->" << nFeaturesOut;
  if (filterStride > 1)
    std::cout << ", stride " << filterStride;
  std::cout << std::endl;
}
void ConvolutionalTriangularLayer::preprocess(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output) {
  scn_ctx *ctx = pre_ctx(batch, memStream);
  assert(input.nFeatures == nFeaturesIn);
  assert(input.spatialSize >= filterSize);
  assert((input.spatialSize - filterSize) % filterStride == 0);
  output.nFeatures = nFeaturesOut;
  output.spatialSize = (input.spatialSize - filterSize) / filterStride + 1;
  output.backpropErrors = input.backpropErrors;
  int64_t n = 0;
  SCN_CHECKED(scn_rules_triangular_plan(
      ctx, input.deviceGrids, own_grids(ctx, output), inSpatialSize,
      outSpatialSize, filterSize, filterStride, minActiveInputs, &n));
  output.nSpatialSites = (int)n;
  fill_rules(ctx, input, output, n * fs);
  convolutionFeaturesPresent(input.featuresPresent.hVector(),
                             output.featuresPresent.hVector(), input.nFeatures,
                             (int)input.featuresPresent.size(), fs);
}
void ConvolutionalTriangularLayer::forwards(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output) {
  if (deferGather && batch.type != TRAINBATCH) {
    output.deferredGatherFrom = &input; // the following NiN layer gathers
    return;
  }
  gather_now(fwd_stream(batch, memStream), input, output);
}
void ConvolutionalTriangularLayer::backwards(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output, float learningRate, float momentum) {
  (void)batch, (void)learningRate, (void)momentum;
  conv_backwards(input, output, memStream);
}
int ConvolutionalTriangularLayer::calculateInputSpatialSize(
    int outputSpatialSize) {
  outSpatialSize = outputSpatialSize;
  inSpatialSize = filterSize + (outputSpatialSize - 1) * filterStride;
  std::cout << "-(C" << filterSize;
  if (filterStride != 1)
    std::cout << "/" << filterStride;
  std::cout << ")-" << inSpatialSize;
  return inSpatialSize;
}

// ---- NetworkInNetworkLayer (NetworkInNetworkLayer.cu:125-202,290-331) ---------
static void nin_preprocess(int nFeaturesIn, int nFeaturesOut,
                           SpatiallySparseBatch &batch, float dropout,
                           RNG &rng, std::mutex &rngMutex,
                           SpatiallySparseBatchInterface &input,
                           SpatiallySparseBatchInterface &output) {
  assert(input.nFeatures == nFeaturesIn);
  (void)nFeaturesIn;
  output.nFeatures = nFeaturesOut;
  output.spatialSize = input.spatialSize;
  output.nSpatialSites = input.nSpatialSites;
  share_grids(input, output);
  // a training batch keeps a random subset of the output features
  // (NetworkInNetworkLayer.cu:153-154); every other batch keeps them all
  int o = nFeaturesOut * (batch.type == TRAINBATCH ? (1.0f - dropout) : 1.0f);
  if (o == nFeaturesOut) {
    output.featuresPresent.hVector() = range(nFeaturesOut);
  } else {
    std::lock_guard<std::mutex> lock(rngMutex);
    output.featuresPresent.hVector() = rng.NchooseM(nFeaturesOut, o);
  }
  output.backpropErrors = true;
}
// Does this training batch use a sub-matrix of the layer's weights
// (NetworkInNetworkLayer.cu:162-164)?
static bool nin_shrunk(SpatiallySparseBatch &batch, int nFeaturesIn,
                       int nFeaturesOut, SpatiallySparseBatchInterface &input,
                       SpatiallySparseBatchInterface &output) {
  return batch.type == TRAINBATCH &&
         (size_t)nFeaturesIn + nFeaturesOut >
             input.featuresPresent.size() + output.featuresPresent.size();
}
// the training branch of forwards() (NetworkInNetworkLayer.cu:165-184): no
// scaling by the kept fraction, weights and bias of the features present
static void nin_forwards_shrunk(cudaMemStream &ms,
                                SpatiallySparseBatchInterface &input,
                                SpatiallySparseBatchInterface &output,
                                vectorCUDA<float> &W, vectorCUDA<float> &B,
                                vectorCUDA<float> *PReLU, vectorCUDA<float> &w,
                                vectorCUDA<float> &b, int nFeaturesOut,
                                int act, int precision) {
  const int Kp = (int)input.featuresPresent.size();
  const int Np = (int)output.featuresPresent.size();
  w.resize64((size_t)Kp * Np);
  b.resize64((size_t)Np);
  SCN_CHECKED(scn_shrink_matrix(ms.ctx, W.dPtr(), w.dPtr(),
                                input.featuresPresent.dPtr(),
                                output.featuresPresent.dPtr(), nFeaturesOut, Kp,
                                Np));
  // a vector is a matrix of one row
  SCN_CHECKED(scn_shrink_matrix(ms.ctx, B.dPtr(), b.dPtr(), nullptr,
                                output.featuresPresent.dPtr(), nFeaturesOut, 1,
                                Np));
  SCN_CHECKED(scn_nin_forward(ms.ctx, input.sub->features.dPtr(), w.dPtr(),
                              b.dPtr(), PReLU ? PReLU->dPtr() : nullptr,
                              output.sub->features.dPtr(), output.nSpatialSites,
                              Kp, Np, 1.0f, act, precision));
  addMultiplyAdds((__int128_t)output.nSpatialSites * Kp * Np);
}
// When the preceding convolutional layer deferred its gather: run the fused
// kernel (fp32 operands), or gather now if this layer wants bf16 operands.
// Returns false when the input is an ordinary feature matrix.
static bool nin_fused(cudaMemStream &ms, SpatiallySparseBatchInterface &input,
                      SpatiallySparseBatchInterface &output,
                      vectorCUDA<float> &W, vectorCUDA<float> &B,
                      vectorCUDA<float> *prelu, int nFeaturesOut, float p,
                      int act, int precision) {
  SpatiallySparseBatchInterface *src = input.deferredGatherFrom;
  if (!src)
    return false;
  const int nIn = src->nFeatures;
  const int fs = input.nFeatures / nIn;
  if (!scn_conv_nin_supported_p(fs, nIn, nFeaturesOut, precision)) {
    gather_now(ms, *src, input);
    return false;
  }
  // bf16 operands, a window of eight or more sites and a matrix worth the
  // pass: round the input once and let the contraction read the bf16 rows
  // (the same result bit for bit, half the bytes through the caches)
  if (precision == SCN_BF16 && fs >= 8 && nIn % 8 == 0 &&
      (int64_t)output.nSpatialSites * fs >= (int64_t)1 << 20) {
    const size_t elems = (size_t)src->nSpatialSites * nIn;
    src->sub->features16.resize64(elems / 2 + 8);
    SCN_CHECKED(scn_conv_nin_forward_a16(
        ms.ctx, src->sub->features.dPtr(), src->nSpatialSites,
        src->sub->features16.dPtr(), input.rules.dPtr(), fs, nIn, W.dPtr(),
        B.dPtr(), prelu ? prelu->dPtr() : nullptr, output.sub->features.dPtr(),
        output.nSpatialSites, nFeaturesOut, p, act));
    return true;
  }
  SCN_CHECKED(scn_conv_nin_forward_p(
      ms.ctx, src->sub->features.dPtr(), input.rules.dPtr(), fs, nIn, W.dPtr(),
      B.dPtr(), prelu ? prelu->dPtr() : nullptr, output.sub->features.dPtr(),
      output.nSpatialSites, nFeaturesOut, p, act, precision));
  return true;
}

// NetworkInNetwork(PReLU)Layer::backwards
// (NetworkInNetworkLayer.cu:219-289, NetworkInNetworkPReLULayer.cu:190-277):
// activation derivative in place (+ bias and slope gradients), dW = A^T D,
// dA = D W^T with the weights of the forward pass, then the momentum step on
// the slopes, W and B.  Without dropout that step is one launch which also
// leaves the gradients zero (gradsClean), so the next batch's products add to
// them without clearing launches of their own; the reference updates the
// slopes before the products, which nothing after that point reads.
static void nin_backwards(cudaMemStream &ms,
                          SpatiallySparseBatchInterface &input,
                          SpatiallySparseBatchInterface &output, int nFeaturesIn,
                          int nFeaturesOut, vectorCUDA<float> *shrunkW,
                          int act, vectorCUDA<float> &W, vectorCUDA<float> &MW,
                          vectorCUDA<float> &B, vectorCUDA<float> &MB,
                          vectorCUDA<float> *PReLU, vectorCUDA<float> *MPReLU,
                          vectorCUDA<float> &dw, vectorCUDA<float> &db,
                          vectorCUDA<float> *dprelu,
                          vectorCUDA<float> &workspace, bool &gradsClean,
                          float learningRate, float momentum) {
  // with dropout: the features present, and the sub-matrix forwards() left
  // in shrunkW (NetworkInNetworkLayer.cu:235-263)
  const int64_t M = output.nSpatialSites;
  const int K = (int)input.featuresPresent.size();
  const int N = (int)output.featuresPresent.size();
  const bool clean = gradsClean && dw.size64() == (size_t)K * N &&
                     db.size64() == (size_t)N &&
                     (!dprelu || dprelu->size64() == (size_t)N);
  gradsClean = false;
  dw.resize64((size_t)K * N);
  db.resize64((size_t)N);
  if (dprelu)
    dprelu->resize64((size_t)N);
  SCN_CHECKED((clean ? scn_activation_backward_acc : scn_activation_backward)(
      ms.ctx, output.sub->features.dPtr(), output.sub->dfeatures.dPtr(), M, N,
      act, PReLU ? PReLU->dPtr() : nullptr, db.dPtr(),
      dprelu ? dprelu->dPtr() : nullptr));
  SCN_CHECKED((clean ? scn_sgemm_AtB_acc : scn_sgemm_AtB)(
      ms.ctx, input.sub->features.dPtr(), output.sub->dfeatures.dPtr(),
      dw.dPtr(), M, K, N));
  addMultiplyAdds((__int128_t)M * K * N);
  if (input.backpropErrors) {
    input.sub->dfeatures.resize64((size_t)input.nSpatialSites * K);
    workspace.resize64((size_t)scn_sgemm_ABt_workspace(N, K));
    SCN_CHECKED(scn_sgemm_ABt(ms.ctx, output.sub->dfeatures.dPtr(),
                              shrunkW ? shrunkW->dPtr() : W.dPtr(),
                              input.sub->dfeatures.dPtr(), M, N, K,
                              workspace.dPtr()));
    addMultiplyAdds((__int128_t)M * K * N);
  }
  if (shrunkW) {
    if (PReLU)
      SCN_CHECKED(scn_nag_update(ms.ctx, dprelu->dPtr(), MPReLU->dPtr(),
                                 PReLU->dPtr(), N, learningRate, momentum, 1));
    SCN_CHECKED(scn_nag_update_shrunk(
        ms.ctx, dw.dPtr(), MW.dPtr(), W.dPtr(), input.featuresPresent.dPtr(),
        output.featuresPresent.dPtr(), nFeaturesOut, K, N, learningRate,
        momentum));
    SCN_CHECKED(scn_nag_update_shrunk(
        ms.ctx, db.dPtr(), MB.dPtr(), B.dPtr(), nullptr,
        output.featuresPresent.dPtr(), nFeaturesOut, 1, N, learningRate,
        momentum));
  } else {
    scn_nag_item items[3];
    int n = 0;
    if (PReLU)
      items[n++] = {dprelu->dPtr(), MPReLU->dPtr(), PReLU->dPtr(), N, 1};
    items[n++] = {dw.dPtr(), MW.dPtr(), W.dPtr(), (int64_t)K * N, 0};
    items[n++] = {db.dPtr(), MB.dPtr(), B.dPtr(), N, 0};
    SCN_CHECKED(
        scn_nag_update_many(ms.ctx, items, n, learningRate, momentum, 1));
    gradsClean = true;
  }
  (void)nFeaturesIn;
}

static void read_floats(std::ifstream &f, vectorCUDA<float> &v) {
  std::vector<float> &h = v.hVector();
  f.read((char *)h.data(), sizeof(float) * h.size());
  v.copyToGPU();
}
static void write_floats(std::ofstream &f, vectorCUDA<float> &v) {
  std::vector<float> &h = v.hVector();
  f.write((char *)h.data(), sizeof(float) * h.size());
  v.copyToGPU();
}

NetworkInNetworkLayer::NetworkInNetworkLayer(cudaMemStream &memStream,
                                             int nFeaturesIn, int nFeaturesOut,
                                             float dropout,
                                             ActivationFunction fn,
                                             float alpha)
    : SpatiallySparseLayer(memStream),
      W(true, (size_t)nFeaturesIn * nFeaturesOut),
      MW(true, (size_t)nFeaturesIn * nFeaturesOut), B(true, nFeaturesOut),
      MB(true, nFeaturesOut), fn(fn), nFeaturesIn(nFeaturesIn),
      nFeaturesOut(nFeaturesOut), dropout(dropout), precision(SCN_FP32) {
  float scale = std::pow(6.0f / (nFeaturesIn + nFeaturesOut * alpha), 0.5f);
  W.setUniform(-scale, scale);
  MW.setZero();
  B.setZero();
  MB.setZero();
  std::cout << "Learn " << nFeaturesIn << "->" << nFeaturesOut
            << " dropout=" << dropout << " " << sigmoidNames[fn] << std::endl;
}
void NetworkInNetworkLayer::preprocess(SpatiallySparseBatch &batch,
                                       SpatiallySparseBatchInterface &input,
                                       SpatiallySparseBatchInterface &output) {
  nin_preprocess(nFeaturesIn, nFeaturesOut, batch, dropout, rng, rngMutex,
                 input, output);
}
void NetworkInNetworkLayer::forwards(SpatiallySparseBatch &batch,
                                     SpatiallySparseBatchInterface &input,
                                     SpatiallySparseBatchInterface &output) {
  output.sub->features.resize64((size_t)output.nSpatialSites *
                                output.featuresPresent.size());
  if (nin_shrunk(batch, nFeaturesIn, nFeaturesOut, input, output)) {
    nin_forwards_shrunk(memStream, input, output, W, B, nullptr, w, b,
                        nFeaturesOut, (int)fn, precision);
    return;
  }
  // test-time scaling by the kept fraction (NetworkInNetworkLayer.cu:188)
  float p = 1.0f - (batch.type != RESCALEBATCH ? dropout : 0.0f);
  cudaMemStream &ms = fwd_stream(batch, memStream);
  if (!nin_fused(ms, input, output, W, B, nullptr, nFeaturesOut, p,
                 (int)fn, precision))
    SCN_CHECKED(scn_nin_forward(ms.ctx, input.sub->features.dPtr(),
                                W.dPtr(), B.dPtr(), nullptr,
                                output.sub->features.dPtr(),
                                output.nSpatialSites, nFeaturesIn, nFeaturesOut,
                                p, (int)fn, precision));
  addMultiplyAdds((__int128_t)output.nSpatialSites * nFeaturesIn * nFeaturesOut);
}
void NetworkInNetworkLayer::backwards(SpatiallySparseBatch &batch,
                                      SpatiallySparseBatchInterface &input,
                                      SpatiallySparseBatchInterface &output,
                                      float learningRate, float momentum) {
  nin_backwards(memStream, input, output, nFeaturesIn, nFeaturesOut,
                nin_shrunk(batch, nFeaturesIn, nFeaturesOut, input, output)
                    ? &w
                    : nullptr,
                (int)fn, W, MW, B, MB, nullptr, nullptr, dw, db, nullptr,
                workspace, gradsClean, learningRate, momentum);
}
// scaleWeights (NetworkInNetworkLayer.cu:203-218; the PReLU layer's is the
// same, NetworkInNetworkPReLULayer.cu:175-189): bring the mean magnitude of
// the layer's output towards one, undoing what the layer below was scaled by
static void nin_scale_weights(cudaMemStream &ms,
                              SpatiallySparseBatchInterface &output,
                              vectorCUDA<float> &W, vectorCUDA<float> &MW,
                              vectorCUDA<float> &B, vectorCUDA<float> &MB,
                              float &scalingUnderneath, bool topLayer) {
  const size_t n = output.sub->features.size64();
  assert(n > 0 && "call after forwards(...)");
  double total = 0;
  SCN_CHECKED(scn_sum_abs(ms.ctx, output.sub->features.dPtr(), (int64_t)n,
                          &total));
  if (total != total) {
    std::cout << "NaN in vectorCUDA<t>::meanAbs()\n";
    scnExit(1);
  }
  float scale = (float)(total / (double)n);
  std::cout << "featureScale:" << scale << std::endl;
  scale = topLayer ? 1 : powf(scale, -0.1);
  SCN_CHECKED(scn_scale(ms.ctx, W.dPtr(), (int64_t)W.size64(),
                        scale / scalingUnderneath));
  SCN_CHECKED(scn_scale(ms.ctx, B.dPtr(), (int64_t)B.size64(), scale));
  SCN_CHECKED(scn_scale(ms.ctx, MW.dPtr(), (int64_t)MW.size64(),
                        scale / scalingUnderneath));
  SCN_CHECKED(scn_scale(ms.ctx, MB.dPtr(), (int64_t)MB.size64(), scale));
  scalingUnderneath = scale;
}
void NetworkInNetworkLayer::scaleWeights(SpatiallySparseBatchInterface &input,
                                         SpatiallySparseBatchInterface &output,
                                         float &scalingUnderneath,
                                         bool topLayer) {
  (void)input;
  nin_scale_weights(memStream, output, W, MW, B, MB, scalingUnderneath,
                    topLayer);
}
void NetworkInNetworkPReLULayer::scaleWeights(
    SpatiallySparseBatchInterface &input, SpatiallySparseBatchInterface &output,
    float &scalingUnderneath, bool topLayer) {
  (void)input;
  nin_scale_weights(memStream, output, W, MW, B, MB, scalingUnderneath,
                    topLayer);
}
void NetworkInNetworkLayer::loadWeightsFromStream(std::ifstream &f,
                                                  bool momentum) {
  read_floats(f, W);
  read_floats(f, B);
  if (momentum) {
    read_floats(f, MW);
    read_floats(f, MB);
  } else {
    MW.setZero();
    MB.setZero();
  }
}
void NetworkInNetworkLayer::putWeightsToStream(std::ofstream &f,
                                               bool momentum) {
  write_floats(f, W);
  write_floats(f, B);
  if (momentum) {
    write_floats(f, MW);
    write_floats(f, MB);
  }
}
int NetworkInNetworkLayer::calculateInputSpatialSize(int outputSpatialSize) {
  return outputSpatialSize;
}

// ---- NetworkInNetworkPReLULayer (NetworkInNetworkPReLULayer.cu:86-335) --------
NetworkInNetworkPReLULayer::NetworkInNetworkPReLULayer(
    cudaMemStream &memStream, int nFeaturesIn, int nFeaturesOut, float dropout,
    float alpha)
    : SpatiallySparseLayer(memStream),
      W(true, (size_t)nFeaturesIn * nFeaturesOut),
      MW(true, (size_t)nFeaturesIn * nFeaturesOut), B(true, nFeaturesOut),
      MB(true, nFeaturesOut), PReLU(true, nFeaturesOut),
      MPReLU(true, nFeaturesOut), nFeaturesIn(nFeaturesIn),
      nFeaturesOut(nFeaturesOut), dropout(dropout), precision(SCN_FP32) {
  float scale = std::pow(6.0f / (nFeaturesIn + nFeaturesOut * alpha), 0.5f);
  W.setUniform(-scale, scale);
  PReLU.setConstant(0.25f); // NetworkInNetworkPReLULayer.cu:6
  MW.setZero();
  B.setZero();
  MB.setZero();
  MPReLU.setZero();
  std::cout << "Learn " << nFeaturesIn << "->" << nFeaturesOut
            << " dropout=" << dropout << " " << sigmoidNames[PRELU]
            << std::endl;
}
void NetworkInNetworkPReLULayer::preprocess(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output) {
  if (batch.type == TRAINBATCH && dropout > 0)
    // NetworkInNetworkPReLULayer.cu:195: the reference's backward pass then
    // pairs the slopes with the wrong columns and reads past their gradient
    unsupported("training a PReLU layer with dropout of its own");
  nin_preprocess(nFeaturesIn, nFeaturesOut, batch, dropout, rng, rngMutex,
                 input, output);
}
void NetworkInNetworkPReLULayer::forwards(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output) {
  output.sub->features.resize64((size_t)output.nSpatialSites *
                                output.featuresPresent.size());
  if (nin_shrunk(batch, nFeaturesIn, nFeaturesOut, input, output)) {
    nin_forwards_shrunk(memStream, input, output, W, B, &PReLU, w, b,
                        nFeaturesOut, (int)PRELU, precision);
    return;
  }
  float p = 1.0f - (batch.type != RESCALEBATCH ? dropout : 0.0f);
  cudaMemStream &ms = fwd_stream(batch, memStream);
  if (!nin_fused(ms, input, output, W, B, &PReLU, nFeaturesOut, p,
                 (int)PRELU, precision))
    SCN_CHECKED(scn_nin_forward(ms.ctx, input.sub->features.dPtr(),
                                W.dPtr(), B.dPtr(), PReLU.dPtr(),
                                output.sub->features.dPtr(),
                                output.nSpatialSites, nFeaturesIn, nFeaturesOut,
                                p, (int)PRELU, precision));
  addMultiplyAdds((__int128_t)output.nSpatialSites * nFeaturesIn * nFeaturesOut);
}
void NetworkInNetworkPReLULayer::backwards(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output, float learningRate, float momentum) {
  nin_backwards(memStream, input, output, nFeaturesIn, nFeaturesOut,
                nin_shrunk(batch, nFeaturesIn, nFeaturesOut, input, output)
                    ? &w
                    : nullptr,
                (int)PRELU, W, MW, B, MB, &PReLU, &MPReLU, dw, db, &dprelu,
                workspace, gradsClean, learningRate, momentum);
}
void NetworkInNetworkPReLULayer::loadWeightsFromStream(std::ifstream &f,
                                                       bool momentum) {
  read_floats(f, W);
  read_floats(f, B);
  read_floats(f, PReLU);
  if (momentum) {
    read_floats(f, MW);
    read_floats(f, MB);
    read_floats(f, MPReLU);
  } else {
    MW.setZero();
    MB.setZero();
    MPReLU.setZero();
  }
}
void NetworkInNetworkPReLULayer::putWeightsToStream(std::ofstream &f,
                                                    bool momentum) {
  write_floats(f, W);
  write_floats(f, B);
  write_floats(f, PReLU);
  if (momentum) {
    write_floats(f, MW);
    write_floats(f, MB);
    write_floats(f, MPReLU);
  }
}
int NetworkInNetworkPReLULayer::calculateInputSpatialSize(
    int outputSpatialSize) {
  return outputSpatialSize;
}

// ---- MaxPoolingLayer (MaxPoolingLayer.cu:97-155) ------------------------------
MaxPoolingLayer::MaxPoolingLayer(cudaMemStream &memStream, int poolSize,
                                 int poolStride, int dimension)
    : SpatiallySparseLayer(memStream), inSpatialSize(0), outSpatialSize(0),
      poolSize(poolSize), poolStride(poolStride), dimension(dimension) {
  sd = ipow(poolSize, dimension);
  std::cout << "MaxPooling " << poolSize << " " << poolStride << std::endl;
}
void MaxPoolingLayer::preprocess(SpatiallySparseBatch &batch,
                                 SpatiallySparseBatchInterface &input,
                                 SpatiallySparseBatchInterface &output) {
  scn_ctx *ctx = pre_ctx(batch, memStream);
  assert(input.spatialSize == inSpatialSize);
  output.nFeatures = input.nFeatures;
  output.featuresPresent.hVector() = input.featuresPresent.hVector();
  output.spatialSize = outSpatialSize;
  output.backpropErrors = input.backpropErrors;
  int64_t n = 0;
  SCN_CHECKED(scn_rules_square_plan(ctx, input.deviceGrids,
                                    own_grids(ctx, output), inSpatialSize,
                                    outSpatialSize, poolSize, poolStride, 1,
                                    &n));
  output.nSpatialSites = (int)n;
  fill_rules(ctx, input, output, n * sd);
}
static void pool_forwards(cudaMemStream &ms,
                          SpatiallySparseBatchInterface &input,
                          SpatiallySparseBatchInterface &output, int width) {
  const size_t nf = output.featuresPresent.size();
  output.sub->poolingChoices.resize64((size_t)output.nSpatialSites * nf);
  output.sub->features.resize64((size_t)output.nSpatialSites * nf);
  SCN_CHECKED(scn_maxpool_checked(ms.ctx, input.sub->features.dPtr(),
                                  input.nSpatialSites,
                                  output.sub->features.dPtr(),
                                  output.rules.dPtr(), output.nSpatialSites,
                                  width, (int)nf,
                                  output.sub->poolingChoices.dPtr()));
}
// MaxPoolingLayer::backwards (MaxPoolingLayer.cu:134-146)
static void pool_backwards(cudaMemStream &ms,
                           SpatiallySparseBatchInterface &input,
                           SpatiallySparseBatchInterface &output) {
  if (!input.backpropErrors)
    return;
  const size_t nf = output.featuresPresent.size();
  input.sub->dfeatures.resize64((size_t)input.nSpatialSites * nf);
  input.sub->dfeatures.setZero(ms);
  SCN_CHECKED(scn_maxpool_backward(
      ms.ctx, input.sub->dfeatures.dPtr(), output.sub->dfeatures.dPtr(),
      output.nSpatialSites, (int)nf, output.sub->poolingChoices.dPtr()));
}
void MaxPoolingLayer::backwards(SpatiallySparseBatch &batch,
                                SpatiallySparseBatchInterface &input,
                                SpatiallySparseBatchInterface &output,
                                float learningRate, float momentum) {
  (void)batch, (void)learningRate, (void)momentum;
  pool_backwards(memStream, input, output);
}
void MaxPoolingLayer::forwards(SpatiallySparseBatch &batch,
                               SpatiallySparseBatchInterface &input,
                               SpatiallySparseBatchInterface &output) {
  pool_forwards(fwd_stream(batch, memStream), input, output, sd);
}
int MaxPoolingLayer::calculateInputSpatialSize(int outputSpatialSize) {
  outSpatialSize = outputSpatialSize;
  inSpatialSize = poolSize + (outputSpatialSize - 1) * poolStride;
  std::cout << "-(MP" << poolSize;
  if (poolStride != poolSize)
    std::cout << "/" << poolStride;
  std::cout << ")-" << inSpatialSize;
  return inSpatialSize;
}

// ---- MaxPoolingTriangularLayer (MaxPoolingTriangularLayer.cu) -----------------
MaxPoolingTriangularLayer::MaxPoolingTriangularLayer(cudaMemStream &memStream,
                                                     int poolSize,
                                                     int poolStride,
                                                     int dimension)
    : SpatiallySparseLayer(memStream), inSpatialSize(0), outSpatialSize(0),
      poolSize(poolSize), poolStride(poolStride), dimension(dimension) {
  S = triangleSize(poolSize, dimension);
  std::cout << dimension
            << "D MaxPoolingTriangularLayer side-length=" << poolSize
            << " volume=" << S << " stride " << poolStride << std::endl;
}
void MaxPoolingTriangularLayer::preprocess(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output) {
  scn_ctx *ctx = pre_ctx(batch, memStream);
  assert(input.spatialSize == inSpatialSize);
  output.nFeatures = input.nFeatures;
  output.featuresPresent.hVector() = input.featuresPresent.hVector();
  output.spatialSize = outSpatialSize;
  output.backpropErrors = input.backpropErrors;
  int64_t n = 0;
  SCN_CHECKED(scn_rules_triangular_plan(ctx, input.deviceGrids,
                                        own_grids(ctx, output), inSpatialSize,
                                        outSpatialSize, poolSize, poolStride, 1,
                                        &n));
  output.nSpatialSites = (int)n;
  fill_rules(ctx, input, output, n * S);
}
void MaxPoolingTriangularLayer::backwards(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output, float learningRate, float momentum) {
  (void)batch, (void)learningRate, (void)momentum;
  pool_backwards(memStream, input, output);
}
void MaxPoolingTriangularLayer::forwards(SpatiallySparseBatch &batch,
                                         SpatiallySparseBatchInterface &input,
                                         SpatiallySparseBatchInterface &output) {
  pool_forwards(fwd_stream(batch, memStream), input, output, S);
}
int MaxPoolingTriangularLayer::calculateInputSpatialSize(
    int outputSpatialSize) {
  outSpatialSize = outputSpatialSize;
  inSpatialSize = poolSize + (outputSpatialSize - 1) * poolStride;
  std::cout << "-(MP" << poolSize;
  if (poolStride != poolSize)
    std::cout << "/" << poolStride;
  std::cout << ")-" << inSpatialSize;
  return inSpatialSize;
}

// ---- fractional max-pooling (Regions.cu:31-134, MaxPoolingLayer.cu:157-420) ----
static void fmp_stop(const char *what, int nIn, int nOut, int poolSize) {
  std::fprintf(stderr,
               "fractional max-pooling regions: %s (nIn %d, nOut %d, "
               "poolSize %d)\n",
               what, nIn, nOut, poolSize);
  scnExit(EXIT_FAILURE);
}
void fmpTicks(FmpKind kind, int nIn, int nOut, int poolSize, RNG &rng,
              int *inputL, int *inputR) {
  switch (kind) {
  case FMP_PSEUDORANDOM_OVERLAPPING: { // Regions.cu:31-46
    if (nIn < nOut - 1 + poolSize)
      fmp_stop("nIn < nOut - 1 + poolSize", nIn, nOut, poolSize);
    double alpha = (nIn - poolSize) * 1.0 / (nOut - 1);
    double u = rng.uniform(0, 1);
    for (int j = 0; j < nOut; ++j) {
      int i = (int)((j + u) * alpha) - (int)(u * alpha);
      inputL[j] = i;
      inputR[j] = i + poolSize;
    }
    break;
  }
  case FMP_PSEUDORANDOM_NONOVERLAPPING: { // Regions.cu:59-71
    double alpha = nIn * 1.0 / nOut;
    double u = rng.uniform(0, 1);
    if (nIn < nOut - 1 + poolSize || (int)std::ceil(alpha) != poolSize)
      fmp_stop("ceil(nIn / nOut) != poolSize", nIn, nOut, poolSize);
    for (int j = 0; j < nOut; ++j)
      inputL[j] = (int)((j + u) * alpha) - (int)(u * alpha);
    for (int j = 1; j <= nOut; ++j)
      inputR[j - 1] = (int)((j + u) * alpha) - (int)(u * alpha);
    break;
  }
  case FMP_RANDOM_OVERLAPPING: { // Regions.cu:83-98
    if (nIn <= nOut)
      fmp_stop("nIn <= nOut", nIn, nOut, poolSize);
    int alpha = nIn * 1.0 / nOut;
    std::vector<int> inc;
    inc.resize(nOut * (alpha + 1) - nIn, alpha);
    inc.resize(nOut - 1, alpha + 1);
    rng.vectorShuffle(inc);
    inputL[0] = 0;
    inputR[0] = poolSize;
    for (int i = 0; i < nOut - 1; i++) {
      inputL[i + 1] = inputL[i] + inc[i];
      inputR[i + 1] = inputL[i + 1] + poolSize;
    }
    break;
  }
  case FMP_RANDOM_NONOVERLAPPING: { // Regions.cu:109-124
    if (nIn <= nOut)
      fmp_stop("nIn <= nOut", nIn, nOut, poolSize);
    int alpha = nIn * 1.0 / nOut;
    std::vector<int> inc;
    inc.resize(nOut * (alpha + 1) - nIn, alpha);
    inc.resize(nOut, alpha + 1);
    rng.vectorShuffle(inc);
    inputL[0] = 0;
    inputR[0] = inc[0];
    for (int i = 0; i < nOut - 1; i++) {
      inputL[i + 1] = inputL[i] + inc[i];
      inputR[i + 1] = inputR[i] + inc[i + 1];
    }
    break;
  }
  }
  if (inputR[nOut - 1] != nIn) // Regions.cu:47,72,99,125
    fmp_stop("the last region does not end at nIn", nIn, nOut, poolSize);
}
static const char *fmpNames[] = {"Pseudorandom overlapping",
                                 "Pseudorandom non-overlapping",
                                 "Random overlapping",
                                 "Random non-overlapping"};
static const char *fmpTags[] = {"POFMP", "PDFMP", "ROFMP", "RDFMP"};
FractionalMaxPoolingLayer::FractionalMaxPoolingLayer(cudaMemStream &memStream,
                                                     FmpKind kind,
                                                     int poolSize,
                                                     float fmpShrink,
                                                     int dimension)
    : SpatiallySparseLayer(memStream), kind(kind), inSpatialSize(0),
      outSpatialSize(0), fmpShrink(fmpShrink), poolSize(poolSize),
      dimension(dimension) {
  sd = ipow(poolSize, dimension);
  std::cout << fmpNames[kind] << " Fractional Max Pooling " << fmpShrink << " "
            << poolSize << std::endl;
}
void FractionalMaxPoolingLayer::preprocess(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output) {
  scn_ctx *ctx = pre_ctx(batch, memStream);
  assert(input.spatialSize == inSpatialSize);
  output.nFeatures = input.nFeatures;
  output.featuresPresent.hVector() = input.featuresPresent.hVector();
  output.spatialSize = outSpatialSize;
  output.backpropErrors = input.backpropErrors;
  // new regions for every sample, axis 0 first (Regions.cu:126-127)
  const size_t per = (size_t)batch.batchSize * dimension * outSpatialSize;
  std::vector<int> &t = output.regionTicks;
  t.assign(2 * per, 0);
  {
    std::lock_guard<std::mutex> lock(rngMutex);
    for (int item = 0; item < batch.batchSize; item++)
      for (int a = 0; a < dimension; ++a) {
        const size_t o = ((size_t)item * dimension + a) * outSpatialSize;
        fmpTicks(kind, inSpatialSize, outSpatialSize, poolSize, rng, &t[o],
                 &t[per + o]);
      }
  }
  int64_t n = 0;
  SCN_CHECKED(scn_rules_fmp_plan(ctx, input.deviceGrids, own_grids(ctx, output),
                                 inSpatialSize, outSpatialSize, poolSize,
                                 t.data(), t.data() + per, &n));
  output.nSpatialSites = (int)n;
  fill_rules(ctx, input, output, n * sd);
}
void FractionalMaxPoolingLayer::forwards(SpatiallySparseBatch &batch,
                                         SpatiallySparseBatchInterface &input,
                                         SpatiallySparseBatchInterface &output) {
  pool_forwards(fwd_stream(batch, memStream), input, output, sd);
}
void FractionalMaxPoolingLayer::backwards(
    SpatiallySparseBatch &batch, SpatiallySparseBatchInterface &input,
    SpatiallySparseBatchInterface &output, float learningRate, float momentum) {
  (void)batch, (void)learningRate, (void)momentum;
  pool_backwards(memStream, input, output);
}
int FractionalMaxPoolingLayer::calculateInputSpatialSize(
    int outputSpatialSize) {
  outSpatialSize = outputSpatialSize;
  inSpatialSize = outputSpatialSize * fmpShrink + 0.5; // MaxPoolingLayer.cu:213
  if (inSpatialSize == outputSpatialSize)
    inSpatialSize++;
  std::cout << "-(" << fmpTags[kind] << ")-" << inSpatialSize;
  return inSpatialSize;
}

// ---- TerminalPoolingLayer (TerminalPoolingLayer.cu:75-130) --------------------
TerminalPoolingLayer::TerminalPoolingLayer(cudaMemStream &memStream,
                                           int poolSize, int S)
    : SpatiallySparseLayer(memStream), inSpatialSize(poolSize),
      outSpatialSize(1), poolSize(poolSize), S(S) {
  std::cout << "TerminalPooling " << poolSize << " " << S << std::endl;
}
void TerminalPoolingLayer::preprocess(SpatiallySparseBatch &batch,
                                      SpatiallySparseBatchInterface &input,
                                      SpatiallySparseBatchInterface &output) {
  assert(input.spatialSize == inSpatialSize);
  output.nFeatures = input.nFeatures;
  output.featuresPresent.hVector() = input.featuresPresent.hVector();
  output.spatialSize = outSpatialSize;
  output.backpropErrors = input.backpropErrors;
  scn_ctx *ctx = pre_ctx(batch, memStream);
  int64_t width = 0;
  SCN_CHECKED(scn_rules_terminal_plan(ctx, input.deviceGrids,
                                      own_grids(ctx, output), &width));
  output.nSpatialSites = batch.batchSize;
  fill_rules(ctx, input, output, width * batch.batchSize);
}
void TerminalPoolingLayer::forwards(SpatiallySparseBatch &batch,
                                    SpatiallySparseBatchInterface &input,
                                    SpatiallySparseBatchInterface &output) {
  const size_t nf = output.featuresPresent.size();
  output.sub->poolingChoices.resize64((size_t)output.nSpatialSites * nf);
  output.sub->features.resize64((size_t)output.nSpatialSites * nf);
  SCN_CHECKED(scn_terminal_pool(
      fwd_stream(batch, memStream).ctx, input.sub->features.dPtr(),
      output.sub->features.dPtr(),
      output.rules.dPtr(), output.nSpatialSites,
      (int)(output.rules.size64() / batch.batchSize), (int)nf));
}
// TerminalPoolingLayer::backwards (TerminalPoolingLayer.cu:112-125)
void TerminalPoolingLayer::backwards(SpatiallySparseBatch &batch,
                                     SpatiallySparseBatchInterface &input,
                                     SpatiallySparseBatchInterface &output,
                                     float learningRate, float momentum) {
  (void)learningRate, (void)momentum;
  if (!input.backpropErrors)
    return;
  const size_t nf = output.featuresPresent.size();
  input.sub->dfeatures.resize64((size_t)input.nSpatialSites * nf);
  input.sub->dfeatures.setZero(memStream);
  SCN_CHECKED(scn_terminal_pool_backward(
      memStream.ctx, input.sub->dfeatures.dPtr(), output.sub->dfeatures.dPtr(),
      output.rules.dPtr(), output.nSpatialSites, (int)nf,
      (int)(output.rules.size64() / batch.batchSize)));
}
int TerminalPoolingLayer::calculateInputSpatialSize(int outputSpatialSize) {
  assert(outputSpatialSize == 1);
  (void)outputSpatialSize;
  std::cout << "-(TP)-" << inSpatialSize;
  return inSpatialSize;
}

// ---- SoftmaxClassifier (SoftmaxClassifier.cu:16-58) ---------------------------
// In two halves, so that a caller may queue the next batch's forward pass
// between them: the copy of the probabilities to the host is only queued
// (SoftmaxClassifier.cu:24, copyToCPUAsync), the statistics are computed once
// it has arrived (:27 onwards).
void SoftmaxClassifierLaunch(SpatiallySparseBatchInterface &input,
                             SpatiallySparseBatch &batch,
                             cudaMemStream &memStream) {
  assert(batch.batchSize == input.nSpatialSites);
  assert(input.nFeatures == (int)input.featuresPresent.size());
  // (a batch that did not come from a BatchProducer has its labels on the host still)
  if (batch.type != UNLABELEDBATCH &&
      (int)batch.result->labels.size() != batch.batchSize)
    batch.result->labels = batch.labels.hVector();
  if (batch.type == TRAINBATCH) {
    // the backward pass starts here: d cost / d soft-max input
    // (SoftmaxClassifier.cu:22-31)
    input.sub->dfeatures.resize64((size_t)input.nSpatialSites *
                                  input.nFeatures);
    SCN_CHECKED(scn_softmax_grad(memStream.ctx, input.sub->features.dPtr(),
                                 batch.labels.dPtr(),
                                 input.sub->dfeatures.dPtr(), batch.batchSize,
                                 input.nFeatures));
  }
  BatchResultStage &r = *batch.result;
  const size_t n = (size_t)batch.batchSize * input.nFeatures;
  if (n > r.capacity) {
    if (r.pinned)
      SCN_CHECKED(scn_host_free(memStream.ctx, r.pinned));
    r.capacity = n + n / 2;
    SCN_CHECKED(scn_host_alloc(memStream.ctx, r.capacity * sizeof(float),
                               (void **)&r.pinned));
  }
  if (!r.arrived)
    SCN_CHECKED(scn_event_create(memStream.ctx, &r.arrived));
  SCN_CHECKED(scn_d2h_async(memStream.ctx, r.pinned, input.sub->features.dPtr(),
                            n * sizeof(float)));
  SCN_CHECKED(scn_event_record(memStream.ctx, r.arrived));
  r.pending = true;
}
void SoftmaxClassifierCollect(SpatiallySparseBatchInterface &input,
                              SpatiallySparseBatch &batch, int nTop) {
  BatchResultStage &r = *batch.result;
  if (!r.pending)
    return;
  SCN_CHECKED(scn_event_wait(r.arrived));
  r.pending = false;
  const int nClasses = input.nFeatures;
  const float *probs = r.pinned;
  for (int i = 0; i < batch.batchSize; ++i)
    batch.probabilities.push_back(std::vector<float>(
        probs + (size_t)i * nClasses, probs + (size_t)(i + 1) * nClasses));
  for (int i = 0; i < batch.batchSize; i++)
    batch.predictions.push_back(vectorTopIndices(batch.probabilities[i], nTop));
  if (batch.type != UNLABELEDBATCH) {
    const std::vector<int> &labels = r.labels;
    batch.mistakes += batch.batchSize;
    for (int i = 0; i < batch.batchSize; i++) {
      double pr = batch.probabilities[i][labels[i]];
      batch.negativeLogLikelihood -= (float)std::log(std::max(pr, 1.0e-15));
      for (int j = 0; j < nTop; j++)
        if (batch.predictions[i][j] == labels[i])
          batch.mistakes--;
    }
  }
}
void SoftmaxClassifier(SpatiallySparseBatchInterface &input,
                       SpatiallySparseBatch &batch, int nTop,
                       cudaMemStream &memStream) {
  SoftmaxClassifierLaunch(input, batch, memStream);
  SoftmaxClassifierCollect(input, batch, nTop);
}
