// C view of the host classes (see scn_host_c.h).
#include <chrono>
#include "scn_host_c.h"
#include "Off3DFormatPicture.h"
#include "OnlineHandwritingPicture.h"
#include "OpenCVPicture.h"

#include <cstdio>
#include <cstdlib>
#include <memory>
#include "BatchProducer.h"
#include "SparseConvNet.h"
#include "SparseConvNetCUDA.h"

struct scnh_net {
  std::unique_ptr<SparseConvNet> square;
  std::unique_ptr<SparseConvTriangLeNet> triangular;
  SparseConvNetCUDA *cnn = nullptr;
  std::unique_ptr<BatchProducer> producer;
  SpatiallySparseBatch *batch = nullptr;
  bool hasClassifier = false;
  float learningRate = 0, momentum = 0; // of the batches scnh_next_batch runs
  int streamTail = 0;    // batches that follow the timed ones of a stream pass
  int readyAtStart = 0;  // slots that held a finished batch when the clock started
  float *allProbs = nullptr; // where a stream pass leaves every batch's probabilities
  int64_t allProbsCapacity = 0;
};
struct scnh_dataset {
  SpatiallySparseDataset ds;
  ~scnh_dataset() {
    for (auto *p : ds.pictures)
      delete p;
  }
};

extern "C" {

scnh_net *scnh_net_create(int dimension, int nInputFeatures, int nClasses,
                          int nTop, int nBatchProducerThreads,
                          int triangular) {
  scnh_net *n = new scnh_net();
  if (triangular) {
    n->triangular.reset(new SparseConvTriangLeNet(dimension, nInputFeatures,
                                                  nClasses, -1, nTop));
    n->cnn = n->triangular->runtime();
  } else {
    n->square.reset(
        new SparseConvNet(dimension, nInputFeatures, nClasses, -1, nTop));
    n->cnn = n->square->cnn.get();
  }
  // the thread count is fixed at construction in the reference (default 10);
  // a smaller pool is allowed here because every slot owns device tables
  n->cnn->limitBatchProducerThreads(nBatchProducerThreads);
  return n;
}
void scnh_net_destroy(scnh_net *net) {
  if (!net)
    return;
  net->producer.reset();
  delete net;
}
void scnh_add_lenet_layer_mp(scnh_net *net, int nFeatures, int filterSize,
                             int filterStride, int poolSize, int poolStride,
                             int activationFn, float dropout,
                             int minActiveInputs) {
  if (net->triangular)
    net->triangular->addLeNetLayerMP(nFeatures, filterSize, filterStride,
                                     poolSize, poolStride,
                                     (ActivationFunction)activationFn, dropout,
                                     minActiveInputs);
  else
    net->square->addLeNetLayerMP(nFeatures, filterSize, filterStride, poolSize,
                                 poolStride, (ActivationFunction)activationFn,
                                 dropout, minActiveInputs);
}
int scnh_add_lenet_layer_fmp(scnh_net *net, int kind, int nFeatures,
                             int filterSize, int filterStride, int poolSize,
                             float fmpShrink, int activationFn, float dropout,
                             int minActiveInputs) {
  if (!net->square || kind < 0 || kind > 3)
    return -1; // the triangular facade has no such builder
  net->cnn->addLeNetLayerFMP(kind, nFeatures, filterSize, filterStride,
                             poolSize, fmpShrink,
                             (ActivationFunction)activationFn, dropout,
                             minActiveInputs);
  return 0;
}
void scnh_add_terminal_pooling_layer(scnh_net *net, int poolSize) {
  if (net->triangular)
    net->triangular->addTerminalPoolingLayer(poolSize);
  else
    net->square->addTerminalPoolingLayer(poolSize);
}
void scnh_add_softmax_layer(scnh_net *net) {
  if (net->triangular)
    net->triangular->addSoftmaxLayer();
  else
    net->square->addSoftmaxLayer();
  net->hasClassifier = true;
}
int scnh_finish_headless(scnh_net *net, int topSpatialSize) {
  SparseConvNetCUDA *cnn = net->cnn;
  cnn->inputSpatialSize = topSpatialSize;
  std::cout << "Headless stack with layer sizes: " << topSpatialSize;
  for (int i = (int)cnn->layers.size() - 1; i >= 0; i--)
    cnn->inputSpatialSize =
        cnn->layers[i]->calculateInputSpatialSize(cnn->inputSpatialSize);
  std::cout << std::endl;
  return cnn->inputSpatialSize;
}
void scnh_set_fused_convolutions(scnh_net *net, int on) {
  net->cnn->setFusedConvolutions(on != 0);
}
void scnh_set_producer_streams(scnh_net *net, int n) {
  net->cnn->setProducerStreams(n);
}
int scnh_producer_streams_in_use(scnh_net *net) {
  return net->cnn->producerStreamsInUse();
}
void scnh_set_chained_rule_books(scnh_net *net, int on) {
  net->cnn->chainRuleBooks = on != 0;
}
void scnh_set_precision(scnh_net *net, int precision) {
  net->cnn->setPrecision(precision);
}
int scnh_input_spatial_size(scnh_net *net) { return net->cnn->inputSpatialSize; }
int scnh_n_layers(scnh_net *net) { return (int)net->cnn->layers.size(); }
int scnh_layer_info(scnh_net *net, int layer, int *nIn, int *nOut, int *act) {
  SpatiallySparseLayer *l = net->cnn->layers.at(layer);
  int a = -1, i = 0, o = 0, kind = -1;
  if (auto *c = dynamic_cast<ConvolutionalLayer *>(l)) {
    kind = 0, i = c->nFeaturesIn, o = c->nFeaturesOut;
  } else if (auto *c = dynamic_cast<ConvolutionalTriangularLayer *>(l)) {
    kind = 1, i = c->nFeaturesIn, o = c->nFeaturesOut;
  } else if (auto *c = dynamic_cast<NetworkInNetworkLayer *>(l)) {
    kind = 2, i = c->nFeaturesIn, o = c->nFeaturesOut, a = c->fn;
  } else if (auto *c = dynamic_cast<NetworkInNetworkPReLULayer *>(l)) {
    kind = 3, i = c->nFeaturesIn, o = c->nFeaturesOut, a = PRELU;
  } else if (dynamic_cast<MaxPoolingLayer *>(l)) {
    kind = 4;
  } else if (dynamic_cast<MaxPoolingTriangularLayer *>(l)) {
    kind = 5;
  } else if (dynamic_cast<TerminalPoolingLayer *>(l)) {
    kind = 6;
  } else if (dynamic_cast<FractionalMaxPoolingLayer *>(l)) {
    kind = 7;
  }
  if (nIn)
    *nIn = i;
  if (nOut)
    *nOut = o;
  if (act)
    *act = a;
  return kind;
}
static void put(vectorCUDA<float> &v, const float *src) {
  std::vector<float> &h = v.hVector();
  std::copy(src, src + h.size(), h.begin());
  v.copyToGPU();
}
static void get(vectorCUDA<float> &v, float *out) {
  if (!out)
    return;
  SCN_CHECKED(scn_d2h(scnDefaultContext(), out, v.dPtr(),
                      v.size64() * sizeof(float)));
}
int scnh_get_weights(scnh_net *net, int layer, int momentum, float *W,
                     float *B, float *prelu) {
  SpatiallySparseLayer *l = net->cnn->layers.at(layer);
  if (auto *c = dynamic_cast<NetworkInNetworkLayer *>(l)) {
    get(momentum ? c->MW : c->W, W);
    get(momentum ? c->MB : c->B, B);
    return 0;
  }
  if (auto *c = dynamic_cast<NetworkInNetworkPReLULayer *>(l)) {
    get(momentum ? c->MW : c->W, W);
    get(momentum ? c->MB : c->B, B);
    get(momentum ? c->MPReLU : c->PReLU, prelu);
    return 0;
  }
  return -1;
}
int scnh_set_weights(scnh_net *net, int layer, const float *W, const float *B,
                     const float *prelu) {
  SpatiallySparseLayer *l = net->cnn->layers.at(layer);
  if (auto *c = dynamic_cast<NetworkInNetworkLayer *>(l)) {
    put(c->W, W);
    put(c->B, B);
    return 0;
  }
  if (auto *c = dynamic_cast<NetworkInNetworkPReLULayer *>(l)) {
    put(c->W, W);
    put(c->B, B);
    if (prelu)
      put(c->PReLU, prelu);
    return 0;
  }
  return -1;
}
void scnh_save_weights(scnh_net *net, const char *baseName, int epoch, int momentum) {
  net->cnn->saveWeights(baseName, epoch, momentum != 0);
}
void scnh_load_weights(scnh_net *net, const char *baseName, int epoch, int momentum) {
  net->cnn->loadWeights(baseName, epoch, momentum != 0);
}

scnh_dataset *scnh_dataset_create(const char *name, int nFeatures,
                                  int nClasses, int type) {
  scnh_dataset *d = new scnh_dataset();
  d->ds.name = name ? name : "";
  d->ds.nFeatures = nFeatures;
  d->ds.nClasses = nClasses;
  d->ds.type = (batchType)type;
  return d;
}
void scnh_dataset_destroy(scnh_dataset *ds) { delete ds; }
void scnh_dataset_add_points(scnh_dataset *ds, int dimension, int latticeSize,
                             int64_t nSites, const int32_t *coords,
                             const float *features, int label) {
  auto *p = new SparsePointsPicture(dimension, latticeSize, ds->ds.nFeatures,
                                    label);
  p->coords.assign(coords, coords + nSites * dimension);
  p->features.assign(features, features + nSites * ds->ds.nFeatures);
  ds->ds.pictures.push_back(p);
}
int scnh_dataset_add_off_file(scnh_dataset *ds, const char *path, int renderSize,
                              int label) {
  auto *p = new OffSurfaceModelPicture(path, renderSize, label);
  if (!p->loaded) {
    delete p;
    return -1;
  }
  ds->ds.pictures.push_back(p);
  return 0;
}
void scnh_dataset_add_mesh(scnh_dataset *ds, int64_t nPoints,
                           const double *points, int64_t nTriangles,
                           const int32_t *triangles, int renderSize,
                           int label) {
  ds->ds.pictures.push_back(new OffSurfaceModelPicture(
      points, (int)nPoints, triangles, (int)nTriangles, renderSize, label));
}
static bool stroke_encoding_ok(const scnh_dataset *ds, int encoding) {
  const bool known = encoding == Simple || encoding == Octogram ||
                     encoding == UndirectedOctogram || encoding == SpaceTime3d ||
                     encoding == VectorSpaceTime3d;
  return known && ds->ds.nFeatures == OnlineHandwritingEncodingSize[encoding];
}
int scnh_dataset_add_strokes(scnh_dataset *ds, int nStrokes,
                             const int32_t *strokeLengths, const double *xy,
                             int renderSize, int encoding, int label,
                             int normalize) {
  if (!stroke_encoding_ok(ds, encoding))
    return -1;
  auto *p = new OnlineHandwritingPicture(
      renderSize, (OnlineHandwritingEncoding)encoding, label);
  for (int s = 0; s < nStrokes; ++s) {
    p->addStroke(xy, strokeLengths[s]);
    xy += 2 * (size_t)strokeLengths[s];
  }
  if (p->ops.empty()) {
    delete p;
    return -1;
  }
  if (normalize) {
    try {
      p->normalize();
    } catch (const std::exception &) {
      delete p;
      return -1;
    }
  }
  ds->ds.pictures.push_back(p);
  return 0;
}
int64_t scnh_dataset_add_pendigits_file(scnh_dataset *ds, const char *path,
                                        int renderSize, int encoding) {
  if (!stroke_encoding_ok(ds, encoding))
    return -1;
  try {
    return readPenDigitsFile(ds->ds.pictures, path, renderSize,
                             (OnlineHandwritingEncoding)encoding);
  } catch (const std::exception &) {
    return -1;
  }
}
int scnh_dataset_add_image(scnh_dataset *ds, int xSize, int ySize, int channels,
                           const float *pixels, int backgroundColor, int label,
                           int trainingJiggle) {
  if (channels != ds->ds.nFeatures || xSize <= 0 || ySize <= 0 ||
      backgroundColor < 0 || backgroundColor > 255)
    return -1;
  auto *p = new OpenCVPicture(xSize, ySize, channels,
                              (unsigned char)backgroundColor, label);
  p->trainingJiggle = trainingJiggle;
  std::copy(pixels, pixels + (size_t)xSize * ySize * channels,
            reinterpret_cast<float *>(p->mat.data));
  ds->ds.pictures.push_back(p);
  return 0;
}
int64_t scnh_dataset_add_mnist_files(scnh_dataset *ds, const char *imagesPath,
                                     const char *labelsPath) {
  if (ds->ds.nFeatures != 1)
    return -1;
  return loadMnist(imagesPath, labelsPath, ds->ds.pictures);
}
int64_t scnh_dataset_add_cifar10_file(scnh_dataset *ds, const char *path) {
  if (ds->ds.nFeatures != 3)
    return -1;
  return readCIFAR10File(ds->ds.pictures, path);
}
int64_t scnh_dataset_add_cifar100_file(scnh_dataset *ds, const char *path) {
  if (ds->ds.nFeatures != 3)
    return -1;
  return readCIFAR100File(ds->ds.pictures, path);
}
int64_t scnh_constant_speed(const double *xy, int nPoints, float density,
                            int multiplier, double *out, int64_t capacity) {
  if (nPoints <= 0)
    return 0;
  std::vector<double> s(xy, xy + 2 * (size_t)nPoints);
  std::vector<double> r = constantSpeed(s, density, multiplier);
  const int64_t n = (int64_t)(r.size() / 2);
  if (n <= capacity)
    std::copy(r.begin(), r.end(), out);
  return n;
}
int64_t scnh_codify_picture(scnh_dataset *ds, int64_t index, int spatialSize,
                            int64_t seed, int64_t capacity, int64_t *keys,
                            int32_t *rows, int32_t *backgroundRow,
                            float *features) {
  Picture *original = ds->ds.pictures.at((size_t)index);
  Picture *pic = original;
  if (seed >= 0) {
    RNG rng((unsigned)seed);
    pic = original->distort(rng, ds->ds.type);
  }
  SparseGrid grid;
  std::vector<float> f;
  int n = 0;
  pic->codifyInputData(grid, f, n, spatialSize);
  if (pic != original)
    delete pic;
  if (n <= capacity) {
    size_t k = 0;
    for (auto &e : grid.mp.entries()) {
      keys[k] = e.first;
      rows[k++] = e.second;
    }
    *backgroundRow = grid.backgroundCol;
    std::copy(f.begin(), f.end(), features);
  }
  return n;
}
int64_t scnh_dataset_size(scnh_dataset *ds) {
  return (int64_t)ds->ds.pictures.size();
}
int scnh_dataset_label(scnh_dataset *ds, int64_t index) {
  if (index < 0 || index >= (int64_t)ds->ds.pictures.size())
    return -1;
  return ds->ds.pictures[(size_t)index]->label;
}

float scnh_process_dataset(scnh_net *net, scnh_dataset *ds, int batchSize) {
  return net->cnn->processDataset(ds->ds, batchSize);
}
float scnh_process_dataset_train(scnh_net *net, scnh_dataset *ds,
                                 int batchSize, float learningRate,
                                 float momentum) {
  return net->cnn->processDataset(ds->ds, batchSize, learningRate, momentum);
}
void scnh_set_training(scnh_net *net, float learningRate, float momentum,
                       int shuffle) {
  net->learningRate = learningRate;
  net->momentum = momentum;
  net->cnn->shuffleTrainingData = shuffle != 0;
}
void scnh_process_dataset_repeat_test(scnh_net *net, scnh_dataset *ds,
                                      int batchSize, int nReps) {
  net->cnn->processDatasetRepeatTest(ds->ds, batchSize, nReps);
}

void scnh_process_dataset_dump_top_level_features(scnh_net *net,
                                                  scnh_dataset *ds,
                                                  int batchSize, int reps) {
  net->cnn->processDatasetDumpTopLevelFeatures(ds->ds, batchSize, reps);
}
void scnh_calculate_input_regularizing_constants(scnh_net *net,
                                                 scnh_dataset *ds) {
  net->cnn->calculateInputRegularizingConstants(ds->ds);
}
int scnh_input_normalizing_constants(scnh_net *net, float *out, int capacity) {
  const auto &c = net->cnn->inputNormalizingConstants;
  if ((int)c.size() <= capacity)
    std::copy(c.begin(), c.end(), out);
  return (int)c.size();
}

void scnh_begin(scnh_net *net, scnh_dataset *ds, int batchSize) {
  net->batch = nullptr;
  net->producer.reset(new BatchProducer(*net->cnn, ds->ds,
                                        net->cnn->inputSpatialSize, batchSize));
}
static void forward_layers(scnh_net *net, SpatiallySparseBatch &b) {
  SparseConvNetCUDA *cnn = net->cnn;
  if (net->hasClassifier) {
    std::ofstream f, g;
    cnn->processBatch(b, net->learningRate, net->momentum, f, g);
  } else {
    for (size_t i = 0; i < cnn->layers.size(); i++) {
      b.interfaces[i + 1].sub->reset();
      scn_prof_tag(cnn->memStream.ctx, (int)i);
      cnn->layers[i]->forwards(b, b.interfaces[i], b.interfaces[i + 1]);
    }
  }
}
int scnh_next_batch(scnh_net *net) {
  if (!net->producer)
    return 0;
  net->batch = net->producer->nextBatch();
  if (!net->batch) {
    net->producer.reset();
    return 0;
  }
  forward_layers(net, *net->batch);
  net->cnn->memStream.synchronize();
  return 1;
}
void scnh_end(scnh_net *net) {
  net->batch = nullptr;
  net->producer.reset();
}
int scnh_batch_size(scnh_net *net) { return net->batch->batchSize; }
int scnh_batch_mistakes(scnh_net *net) { return net->batch->mistakes; }
float scnh_batch_nll(scnh_net *net) { return net->batch->negativeLogLikelihood; }
void scnh_batch_probabilities(scnh_net *net, float *out) {
  for (auto &p : net->batch->probabilities)
    out = std::copy(p.begin(), p.end(), out);
}
void scnh_batch_predictions(scnh_net *net, int32_t *out) {
  for (auto &p : net->batch->predictions)
    out = std::copy(p.begin(), p.end(), out);
}
void scnh_batch_sample_numbers(scnh_net *net, int32_t *out) {
  std::copy(net->batch->sampleNumbers.begin(), net->batch->sampleNumbers.end(),
            out);
}
void scnh_iface_info(scnh_net *net, int i, int *nFeatures, int *nSpatialSites,
                     int *spatialSize, int64_t *nRules, int64_t *nFeatureElems,
                     int64_t *nChoices, int64_t *nGridEntries) {
  SpatiallySparseBatchInterface &f = net->batch->interfaces.at(i);
  // the width of the feature matrix: all features, or during a training
  // batch with dropout the ones present
  *nFeatures = (int)f.featuresPresent.size();
  *nSpatialSites = f.nSpatialSites;
  *spatialSize = f.spatialSize;
  *nRules = (int64_t)f.rules.size64();
  *nFeatureElems =
      f.deferredGatherFrom
          ? 0
          : (int64_t)f.nSpatialSites * (int64_t)f.featuresPresent.size();
  *nChoices = (int64_t)f.sub->poolingChoices.size64();
  int64_t n = 0;
  if (f.deviceGrids)
    SCN_CHECKED(scn_grids_info(f.deviceGrids, nullptr, nullptr, nullptr, &n,
                               nullptr));
  *nGridEntries = n;
}
void scnh_iface_rules(scnh_net *net, int i, int32_t *out) {
  SpatiallySparseBatchInterface &f = net->batch->interfaces.at(i);
  SCN_CHECKED(scn_d2h(net->cnn->memStream.ctx, out, f.rules.dPtr(),
                      f.rules.size64() * sizeof(int32_t)));
}
void scnh_iface_features(scnh_net *net, int i, float *out) {
  SpatiallySparseBatchInterface &f = net->batch->interfaces.at(i);
  SCN_CHECKED(scn_d2h(net->cnn->memStream.ctx, out, f.sub->features.dPtr(),
                      (size_t)f.nSpatialSites * f.featuresPresent.size() *
                          sizeof(float)));
}
int scnh_iface_features_present(scnh_net *net, int i, int32_t *out) {
  SpatiallySparseBatchInterface &f = net->batch->interfaces.at(i);
  std::vector<int> &v = f.featuresPresent.hVector();
  if (out)
    std::copy(v.begin(), v.end(), out);
  return (int)v.size();
}
void scnh_iface_dfeatures(scnh_net *net, int i, float *out) {
  SpatiallySparseBatchInterface &f = net->batch->interfaces.at(i);
  SCN_CHECKED(scn_d2h(net->cnn->memStream.ctx, out, f.sub->dfeatures.dPtr(),
                      f.sub->dfeatures.size64() * sizeof(float)));
}
int64_t scnh_iface_dfeatures_size(scnh_net *net, int i) {
  return (int64_t)net->batch->interfaces.at(i).sub->dfeatures.size64();
}
int64_t scnh_iface_region_ticks_size(scnh_net *net, int i) {
  return (int64_t)net->batch->interfaces.at(i).regionTicks.size();
}
void scnh_iface_region_ticks(scnh_net *net, int i, int32_t *out) {
  std::vector<int> &t = net->batch->interfaces.at(i).regionTicks;
  std::copy(t.begin(), t.end(), out);
}
void scnh_iface_choices(scnh_net *net, int i, int32_t *out) {
  SpatiallySparseBatchInterface &f = net->batch->interfaces.at(i);
  SCN_CHECKED(scn_d2h(net->cnn->memStream.ctx, out,
                      f.sub->poolingChoices.dPtr(),
                      f.sub->poolingChoices.size64() * sizeof(int32_t)));
}
void scnh_iface_grids(scnh_net *net, int i, int32_t *sample, int64_t *key,
                      int32_t *row, int32_t *background) {
  SpatiallySparseBatchInterface &f = net->batch->interfaces.at(i);
  SCN_CHECKED(scn_grids_download(net->cnn->memStream.ctx, f.deviceGrids,
                                 sample, key, row, background));
}

static ResidentBatch resident_of(int batch, const int32_t *d_sample,
                                 const int64_t *d_key, const int32_t *d_row,
                                 const int32_t *d_background, int64_t nActive,
                                 int nSpatialSites, const float *d_features) {
  ResidentBatch r;
  r.batchSize = batch;
  r.d_sample = d_sample;
  r.d_key = d_key;
  r.d_row = d_row;
  r.d_background = d_background;
  r.nActive = nActive;
  r.nSpatialSites = nSpatialSites;
  r.d_features = d_features;
  r.onHost = false;
  return r;
}

int scnh_forward_resident(scnh_net *net, int batch, const int32_t *d_sample,
                          const int64_t *d_key, const int32_t *d_row,
                          const int32_t *d_background, int64_t nActive,
                          int nSpatialSites, const float *d_features,
                          float *h_probs) {
  SparseConvNetCUDA *cnn = net->cnn;
  cnn->ensureInterfaces();
  // everything on the net's own stream: one batch, start to end
  cudaMemStream *keep = cnn->batchPool[0].preprocessStream;
  cnn->batchPool[0].preprocessStream = nullptr;
  cnn->preprocessResident(0, resident_of(batch, d_sample, d_key, d_row,
                                         d_background, nActive, nSpatialSites,
                                         d_features));
  cnn->batchPool[0].preprocessStream = keep;
  SpatiallySparseBatch &b = cnn->batchPool[0];
  net->batch = &b;
  forward_layers(net, b);
  if (net->hasClassifier && h_probs)
    scnh_batch_probabilities(net, h_probs);
  cnn->memStream.synchronize();
  return b.interfaces.back().nSpatialSites;
}

int scnh_forward_resident_stream(scnh_net *net, int nBatches, int batch,
                                 const int32_t *d_sample, const int64_t *d_key,
                                 const int32_t *d_row,
                                 const int32_t *d_background, int64_t nActive,
                                 int nSpatialSites, const float *d_features,
                                 float *h_probs) {
  double seconds = 0;
  return scnh_forward_stream_timed(net, 0, nBatches, batch, d_sample, d_key,
                                   d_row, d_background, nActive, nSpatialSites,
                                   d_features, 0, h_probs, &seconds);
}

// nWarmup + nTimed batches through one BatchProducer, as one dataset pass runs
// them; *seconds is the wall time of the last nTimed, taken between two points
// at which the net's stream is idle and every earlier batch is finished.  The
// producers are not stopped in between: at the first point they hold the next
// batches ready, as they do in the middle of any pass.
int scnh_forward_stream_timed(scnh_net *net, int nWarmup, int nTimed, int batch,
                              const int32_t *sample, const int64_t *key,
                              const int32_t *row, const int32_t *background,
                              int64_t nActive, int nSpatialSites,
                              const float *features, int inputsOnHost,
                              float *h_probs, double *seconds) {
  const int32_t *samples[1] = {sample};
  const int64_t *keys[1] = {key};
  const int32_t *rows[1] = {row};
  const int32_t *backgrounds[1] = {background};
  const float *feats[1] = {features};
  return scnh_forward_stream_timed_many(net, nWarmup, nTimed, 1, &batch, samples,
                                        keys, rows, backgrounds, &nActive,
                                        &nSpatialSites, feats, inputsOnHost,
                                        h_probs, seconds);
}
int scnh_forward_stream_timed_many(
    scnh_net *net, int nWarmup, int nTimed, int nDistinct, const int *batch,
    const int32_t *const *sample, const int64_t *const *key,
    const int32_t *const *row, const int32_t *const *background,
    const int64_t *nActive, const int *nSpatialSites,
    const float *const *features, int inputsOnHost, float *h_probs,
    double *seconds) {
  SparseConvNetCUDA *cnn = net->cnn;
  std::vector<ResidentBatch> rs;
  for (int i = 0; i < nDistinct; ++i) {
    rs.push_back(resident_of(batch[i], sample[i], key[i], row[i], background[i],
                             nActive[i], nSpatialSites[i], features[i]));
    rs.back().onHost = inputsOnHost != 0;
  }
  // The timed batches sit in the middle of a longer pass: nTail more batches
  // follow them, so that the producers are as busy at the end of the timed
  // window as they are at its start (they hold finished batches ready at both
  // ends; without a tail the window would be served in part by work done before
  // the clock started and never paid back).
  const int nTail = net->streamTail > 0 ? net->streamTail : 0;
  BatchProducer bp(*cnn, rs, nWarmup + nTimed + nTail);
  ForwardQueue queue(*cnn, bp, !net->hasClassifier); // (a headless net: layer by layer on lane 0)
  int done = 0, started = 0;
  float *all = net->allProbs;
  int64_t allLeft = net->allProbsCapacity;
  auto t0 = std::chrono::steady_clock::now();
  bool stopped = false;
  auto finish = [&](SpatiallySparseBatch *b) {
    if (net->hasClassifier) {
      std::ofstream f, g;
      cnn->finishBatch(*b, f, g);
      net->batch = b;
      if (h_probs)
        scnh_batch_probabilities(net, h_probs);
      if (all) { // every batch's probabilities, in batch order, while they fit
        const int64_t n = (int64_t)b->probabilities.size() * cnn->nClasses;
        if (n <= allLeft) {
          scnh_batch_probabilities(net, all);
          all += n;
          allLeft -= n;
        }
      }
    }
    net->batch = b;
    ++done;
    if (done == nWarmup + nTimed && !stopped) { // the last timed batch is on the host
      if (seconds)
        *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      stopped = true;
    }
  };
  SpatiallySparseBatch *headless = nullptr;
  while (SpatiallySparseBatch *b = bp.nextBatch()) {
    if (started == nWarmup) { // every warm-up batch done before the clock starts
      while (SpatiallySparseBatch *q = queue.pop())
        finish(q);
      if (headless)
        finish(headless);
      headless = nullptr;
      cnn->synchronizeLanes();
      net->readyAtStart = bp.slotsReady();
      t0 = std::chrono::steady_clock::now();
    }
    const bool firstOfTail = started == nWarmup + nTimed;
    ++started;
    if (net->hasClassifier) {
      if (SpatiallySparseBatch *due = queue.push(b))
        finish(due);
    } else {
      // (nothing is read back from a headless stack: a batch is finished when
      // the net's stream has run it)
      if (firstOfTail && headless) {
        cnn->synchronizeLanes();
        finish(headless);
        headless = nullptr;
      }
      forward_layers(net, *b);
      if (headless)
        finish(headless);
      headless = b;
      if (!bp.keepAlive) {
        if (done + 1 == nWarmup + nTimed)
          cnn->synchronizeLanes();
        finish(headless);
        headless = nullptr;
      }
    }
  }
  while (SpatiallySparseBatch *q = queue.pop())
    finish(q);
  if (headless) {
    cnn->synchronizeLanes();
    finish(headless);
  }
  cnn->synchronizeLanes();
  // net->batch stays at the last batch finished: its interfaces can be read
  // (scnh_iface_*) until the next pass starts
  return done - nTail;
}
void scnh_set_stream_tail(scnh_net *net, int nTail) { net->streamTail = nTail; }
int scnh_stream_ready_at_start(scnh_net *net) { return net->readyAtStart; }
void scnh_collect_probabilities(scnh_net *net, float *h_all, int64_t capacity) {
  net->allProbs = h_all;
  net->allProbsCapacity = h_all ? capacity : 0;
}
void scnh_chain_counts(scnh_net *net, int64_t *chains, int64_t *plans) {
  SparseConvNetCUDA *cnn = net->cnn;
  int64_t c = 0, p = 0;
  auto add = [&](scn_ctx *ctx) {
    int64_t a = 0, b = 0;
    SCN_CHECKED(scn_ctx_chain_count(ctx, &a, &b));
    c += a;
    p += b;
  };
  add(cnn->memStream.ctx);
  for (auto &s : cnn->batchMemStreams)
    add(s->ctx);
  if (chains)
    *chains = c;
  if (plans)
    *plans = p;
}
void *scnh_context(scnh_net *net) { return net->cnn->memStream.ctx; }
double scnh_take_multiply_add_count(void) {
  double v = (double)multiplyAddCount;
  multiplyAddCount = 0;
  return v;
}

} // extern "C"
