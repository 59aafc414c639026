/* C view of the C++ host classes, for callers that cannot link C++ (the
 * Python test and benchmark harness loads it with ctypes).  Every function
 * forwards to the class method named in its comment. */
#ifndef SCN_HOST_C_H
#define SCN_HOST_C_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct scnh_net scnh_net;
typedef struct scnh_dataset scnh_dataset;

/* SparseConvNet / SparseConvTriangLeNet constructors */
scnh_net *scnh_net_create(int dimension, int nInputFeatures, int nClasses,
                          int nTop, int nBatchProducerThreads, int triangular);
void scnh_net_destroy(scnh_net *net);
/* addLeNetLayerMP of the square or triangular facade */
void scnh_add_lenet_layer_mp(scnh_net *net, int nFeatures, int filterSize,
                             int filterStride, int poolSize, int poolStride,
                             int activationFn, float dropout,
                             int minActiveInputs);
/* addLeNetLayerPOFMP / PDFMP / ROFMP / RDFMP (kind 0..3) of the square
 * facade: convolution, NiN, fractional max-pooling; -1 on a triangular net */
int scnh_add_lenet_layer_fmp(scnh_net *net, int kind, int nFeatures,
                             int filterSize, int filterStride, int poolSize,
                             float fmpShrink, int activationFn, float dropout,
                             int minActiveInputs);
void scnh_add_terminal_pooling_layer(scnh_net *net, int poolSize);
void scnh_add_softmax_layer(scnh_net *net);
/* A stack without a classifier: fixes the spatial sizes from the size of the
 * last layer's output; returns the input field size. */
int scnh_finish_headless(scnh_net *net, int topSpatialSize);
void scnh_set_precision(scnh_net *net, int precision);
/* SparseConvNetCUDA::setFusedConvolutions */
void scnh_set_fused_convolutions(scnh_net *net, int on);
/* how many of the net's producer streams take part in batch production
 * (SparseConvNetCUDA::setProducerStreams; n < 1: all of them), to be called
 * between passes; and how many do */
void scnh_set_producer_streams(scnh_net *net, int n);
int scnh_producer_streams_in_use(scnh_net *net);
/* rule books of consecutive layers built together (default) or layer by layer */
void scnh_set_chained_rule_books(scnh_net *net, int on);
int scnh_input_spatial_size(scnh_net *net);
int scnh_n_layers(scnh_net *net);
/* kind: 0 conv, 1 triangular conv, 2 NiN, 3 NiN PReLU, 4 max-pool,
 * 5 triangular max-pool, 6 terminal pool; NiN layers report nIn/nOut/act */
int scnh_layer_info(scnh_net *net, int layer, int *nIn, int *nOut, int *act);
/* NetworkInNetwork(PReLU)Layer::W, B, PReLU */
int scnh_set_weights(scnh_net *net, int layer, const float *W, const float *B,
                     const float *prelu);
/* the same vectors read back (momentum != 0: MW, MB, MPReLU); a null pointer
 * skips that vector */
int scnh_get_weights(scnh_net *net, int layer, int momentum, float *W,
                     float *B, float *prelu);
/* momentum != 0: the momentum arrays follow each layer's parameters */
void scnh_save_weights(scnh_net *net, const char *baseName, int epoch, int momentum);
void scnh_load_weights(scnh_net *net, const char *baseName, int epoch, int momentum);

scnh_dataset *scnh_dataset_create(const char *name, int nFeatures,
                                  int nClasses, int type);
void scnh_dataset_destroy(scnh_dataset *ds);
/* appends a SparsePointsPicture */
void scnh_dataset_add_points(scnh_dataset *ds, int dimension, int latticeSize,
                             int64_t nSites, const int32_t *coords,
                             const float *features, int label);
int64_t scnh_dataset_size(scnh_dataset *ds);
/* Picture::label of picture `index` (-1 when there is no such picture) */
int scnh_dataset_label(scnh_dataset *ds, int64_t index);
/* OffSurfaceModelPicture (Off3DFormatPicture.h): from an OFF file (returns -1
 * when it cannot be read) or from arrays (points: nPoints x 3 doubles,
 * triangles: nTriangles x 3 vertex indices).  The dataset needs nFeatures 1. */
int scnh_dataset_add_off_file(scnh_dataset *ds, const char *path, int renderSize,
                              int label);
void scnh_dataset_add_mesh(scnh_dataset *ds, int64_t nPoints,
                           const double *points, int64_t nTriangles,
                           const int32_t *triangles, int renderSize, int label);
/* OnlineHandwritingPicture (OnlineHandwritingPicture.h): a character from
 * arrays -- nStrokes strokes, stroke s has strokeLengths[s] points, xy holds
 * all points in order as (x, y) doubles -- optionally normalize()d; or every
 * character of a UCI pen-digits file (readPenDigitsFile,
 * SpatiallySparseDatasetPenDigits.cpp:15-63; returns how many were appended).
 * encoding: 0 Simple, 1 Octogram, 2 UndirectedOctogram, 7 SpaceTime3d,
 * 8 VectorSpaceTime3d; the dataset needs the matching nFeatures (1, 8, 4, 1,
 * 3).  Both return -1 for an encoding that is not available (3..6, the
 * LogSignature ones), a wrong nFeatures, or a file that cannot be opened. */
int scnh_dataset_add_strokes(scnh_dataset *ds, int nStrokes,
                             const int32_t *strokeLengths, const double *xy,
                             int renderSize, int encoding, int label,
                             int normalize);
int64_t scnh_dataset_add_pendigits_file(scnh_dataset *ds, const char *path,
                                        int renderSize, int encoding);
/* OpenCVPicture (OpenCVPicture.h), array-backed: pixels is rows x cols x
 * channels floats in 0..255 with rows = xSize (the reference's constructor
 * passes xSize as the row count); the MNIST idx pair and a CIFAR-10 binary
 * batch through the reference's readers (SpatiallySparseDatasetMnist.cpp,
 * SpatiallySparseDatasetCIFAR10.cpp).  trainingJiggle: what distort() moves a
 * training picture by.  The readers return how many pictures they appended;
 * all return -1 on a channel count that is not the dataset's nFeatures or an
 * unreadable file. */
int scnh_dataset_add_image(scnh_dataset *ds, int xSize, int ySize, int channels,
                           const float *pixels, int backgroundColor, int label,
                           int trainingJiggle);
int64_t scnh_dataset_add_mnist_files(scnh_dataset *ds, const char *imagesPath,
                                     const char *labelsPath);
int64_t scnh_dataset_add_cifar10_file(scnh_dataset *ds, const char *path);
int64_t scnh_dataset_add_cifar100_file(scnh_dataset *ds, const char *path);
/* constantSpeed (OnlineHandwritingPicture.cpp:27-53) of one stroke: returns the
 * number of points and, when that fits capacity, writes them to out. */
int64_t scnh_constant_speed(const double *xy, int nPoints, float density,
                            int multiplier, double *out, int64_t capacity);
/* Picture::distort (when seed >= 0, with RNG(seed) and the dataset's batch
 * type) followed by Picture::codifyInputData into an empty grid, on the CPU.
 * Returns the number of rows (background row included); when that fits
 * `capacity`, writes key / row of every site in insertion order, the
 * background row and the rows x nFeatures feature matrix. */
int64_t scnh_codify_picture(scnh_dataset *ds, int64_t index, int spatialSize,
                            int64_t seed, int64_t capacity, int64_t *keys,
                            int32_t *rows, int32_t *backgroundRow,
                            float *features);

/* SparseConvNet::processDataset / processDatasetRepeatTest */
float scnh_process_dataset(scnh_net *net, scnh_dataset *ds, int batchSize);
/* the same with processDataset's learningRate and momentum: one pass of
 * training when the dataset's type is TRAINBATCH */
float scnh_process_dataset_train(scnh_net *net, scnh_dataset *ds,
                                 int batchSize, float learningRate,
                                 float momentum);
/* learning rate and momentum of the batches that scnh_next_batch processes
 * (used by TRAINBATCH datasets), and whether training batches are drawn in
 * shuffled order (the reference always shuffles, BatchProducer.cu:23-26) */
void scnh_set_training(scnh_net *net, float learningRate, float momentum,
                       int shuffle);
void scnh_process_dataset_repeat_test(scnh_net *net, scnh_dataset *ds,
                                      int batchSize, int nReps);

/* SparseConvNet::processDatasetDumpTopLevelFeatures (writes
 * "<dataset name>.features" in the working directory) and
 * calculateInputRegularizingConstants; the constants (nInputFeatures floats,
 * empty before the call) can be read back. */
void scnh_process_dataset_dump_top_level_features(scnh_net *net,
                                                  scnh_dataset *ds,
                                                  int batchSize, int reps);
void scnh_calculate_input_regularizing_constants(scnh_net *net,
                                                 scnh_dataset *ds);
int scnh_input_normalizing_constants(scnh_net *net, float *out, int capacity);

/* Batch-by-batch processing with the batch left in place for inspection:
 * BatchProducer::nextBatch + SparseConvNetCUDA::processBatch. */
void scnh_begin(scnh_net *net, scnh_dataset *ds, int batchSize);
int scnh_next_batch(scnh_net *net); /* 0 when the dataset is exhausted */
void scnh_end(scnh_net *net);
int scnh_batch_size(scnh_net *net);
int scnh_batch_mistakes(scnh_net *net);
float scnh_batch_nll(scnh_net *net);
void scnh_batch_probabilities(scnh_net *net, float *out);
void scnh_batch_predictions(scnh_net *net, int32_t *out);
void scnh_batch_sample_numbers(scnh_net *net, int32_t *out);
/* interface i (0 = input): sizes, then the vectors themselves */
void scnh_iface_info(scnh_net *net, int i, int *nFeatures, int *nSpatialSites,
                     int *spatialSize, int64_t *nRules, int64_t *nFeatureElems,
                     int64_t *nChoices, int64_t *nGridEntries);
void scnh_iface_rules(scnh_net *net, int i, int32_t *out);
void scnh_iface_features(scnh_net *net, int i, float *out);
/* SpatiallySparseBatchInterface::featuresPresent: which of the interface's
 * nFeatures the columns of its feature matrix are (all of them except in a
 * training batch with dropout).  Returns their number; out may be null. */
int scnh_iface_features_present(scnh_net *net, int i, int32_t *out);
/* gradient of the cost with respect to that feature matrix after a TRAINBATCH
 * (SpatiallySparseBatchSubInterface::dfeatures); size in floats, 0 when the
 * backward pass did not reach the interface */
/* the pooling regions a fractional max-pooling layer drew for the batch:
 * inputL then inputR, each [batchSize][dimension][spatialSize of the
 * interface]; size 0 for the output of any other layer */
int64_t scnh_iface_region_ticks_size(scnh_net *net, int i);
void scnh_iface_region_ticks(scnh_net *net, int i, int32_t *out);
int64_t scnh_iface_dfeatures_size(scnh_net *net, int i);
void scnh_iface_dfeatures(scnh_net *net, int i, float *out);
void scnh_iface_choices(scnh_net *net, int i, int32_t *out);
void scnh_iface_grids(scnh_net *net, int i, int32_t *sample, int64_t *key,
                      int32_t *row, int32_t *background);

/* One forward pass over a batch whose input already sits in HBM: active
 * sites (sample, key, row), backgroundCol per sample and the input feature
 * matrix [nSpatialSites x nInputFeatures], all device pointers.  Builds the
 * grids and every rule book, runs every layer and, when the net ends in the
 * softmax classifier, copies the probabilities [batch x nClasses] to h_probs.
 * Returns the number of rows of the last interface. */
int scnh_forward_resident(scnh_net *net, int batch, const int32_t *d_sample,
                          const int64_t *d_key, const int32_t *d_row,
                          const int32_t *d_background, int64_t nActive,
                          int nSpatialSites, const float *d_features,
                          float *h_probs);
/* nBatches forward passes over the same resident batch, produced the way
 * processDataset produces them: the net's batch-producer threads build grids
 * and rule books on their slots' streams while the calling thread runs the
 * forward pass of the previous batch.  Returns the number of batches done. */
int scnh_forward_resident_stream(scnh_net *net, int nBatches, int batch,
                                 const int32_t *d_sample, const int64_t *d_key,
                                 const int32_t *d_row,
                                 const int32_t *d_background, int64_t nActive,
                                 int nSpatialSites, const float *d_features,
                                 float *h_probs);
/* nWarmup untimed and nTimed timed batches in one pass (the producers keep
 * running across the boundary); inputsOnHost: the five arrays are pinned host
 * memory and every batch uploads them on its producer's stream, otherwise
 * device memory.  *seconds: wall time of the timed batches. */
int scnh_forward_stream_timed(scnh_net *net, int nWarmup, int nTimed, int batch,
                              const int32_t *sample, const int64_t *key,
                              const int32_t *row, const int32_t *background,
                              int64_t nActive, int nSpatialSites,
                              const float *features, int inputsOnHost,
                              float *h_probs, double *seconds);
/* The same over nDistinct different batches taken in turn (batch i of the pass
 * is number i % nDistinct): every argument that describes a batch is an array
 * of nDistinct.  h_probs must hold the largest batch. */
int scnh_forward_stream_timed_many(
    scnh_net *net, int nWarmup, int nTimed, int nDistinct, const int *batch,
    const int32_t *const *sample, const int64_t *const *key,
    const int32_t *const *row, const int32_t *const *background,
    const int64_t *nActive, const int *nSpatialSites,
    const float *const *features, int inputsOnHost, float *h_probs,
    double *seconds);
/* nTail batches follow the timed ones of every later scnh_forward_stream_timed
 * (_many) pass, untimed: the timed window then lies in the middle of a pass,
 * with the producers as busy at its end as at its start (0: none). */
void scnh_set_stream_tail(scnh_net *net, int nTail);
/* how many batch slots held a finished batch when the clock of the last such
 * pass started */
int scnh_stream_ready_at_start(scnh_net *net);
/* Every later such pass also leaves the probabilities of all its batches, in
 * batch order, in h_all (capacity in floats; batches that no longer fit are
 * left out; null: switched off).  After a pass the last batch finished stays
 * readable through scnh_iface_* and scnh_batch_* until the next pass. */
void scnh_collect_probabilities(scnh_net *net, float *h_all, int64_t capacity);
/* recorded-plan runs so far on all streams of the net that build rule books
 * (sums of scn_ctx_chain_count) */
void scnh_chain_counts(scnh_net *net, int64_t *chains, int64_t *plans);
/* the library context of the net (scn_ctx *), for timing and raw buffers */
void *scnh_context(scnh_net *net);
/* multiply-accumulates of the NiN layers since the last call */
double scnh_take_multiply_add_count(void);

#ifdef __cplusplus
}
#endif
#endif
