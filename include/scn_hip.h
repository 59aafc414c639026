/*
 * libscn_hip.so -- C ABI of the MI355X (gfx950) implementation of
 * SparseConvNet's spatially-sparse forward path, and of the backward pass
 * and weight update that follow it in a training batch.
 *
 * The reference has no plugin interface; its seam is the set of free functions
 * that the layer classes' preprocess()/forwards()/backwards() call with raw
 * device pointers and a stream.  Each entry point below names the reference function
 * it stands in for (paths relative to the reference's SparseConvNet/ folder).
 *
 * Conventions
 *   - every function returns SCN_OK or an SCN_ERR_* code; scn_last_error()
 *     gives the message of the calling thread's last failure (the reference
 *     prints and exit(-1)s instead, utilities.h:36-67);
 *   - all device work is issued on the context's single stream
 *     (cudaMemStream, utilities.cu:171-178) and is asynchronous unless the
 *     function has to hand a count back to the host;
 *   - pointers named d_* are device pointers, h_* host pointers;
 *   - feature matrices are row-major fp32 [rows x channels]; rule books are
 *     row-major int32 [output rows x rule width]; rows are batch-global;
 *   - numeric kernels never allocate: every buffer is the caller's
 *     (SpatiallySparseBatchSubInterface, SpatiallySparseBatchInterface.h:8-17).
 *     scn_grids objects own their tables and only ever grow them.
 */
#ifndef SCN_HIP_H
#define SCN_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum {
  SCN_OK = 0,
  SCN_ERR_ARG = 1,      /* bad argument (the reference would assert) */
  SCN_ERR_HIP = 2,      /* a HIP runtime call failed */
  SCN_ERR_CAPACITY = 3, /* a caller buffer or an index range is too small */
  SCN_ERR_STATE = 4     /* call order violated (e.g. fill without plan) */
};

/* ActivationFunction, types.h:11-20 (same numbering) */
enum {
  SCN_NOSIGMOID = 0,
  SCN_RELU = 1,
  SCN_VLEAKYRELU = 2,
  SCN_LEAKYRELU = 3,
  SCN_TANH = 4,
  SCN_SOFTMAX = 5,
  SCN_PRELU = 6,
  SCN_SIGMOID = 7
};

/* Operand precision of the NiN contraction (accumulation is always fp32):
 * fp32 MFMA; bf16 operands; or bf16 hi + lo pairs with three MFMAs per tile,
 * which keeps fp32-grade results at bf16-matrix-core speed. */
enum { SCN_FP32 = 0, SCN_BF16 = 1, SCN_BF16X3 = 2 };

typedef struct scn_ctx scn_ctx;
typedef struct scn_grids scn_grids;

const char *scn_last_error(void);
const char *scn_version(void);

/* ---- context: device, stream, copies --------------------------------- */
/* initializeGPU (utilities.cu:105-130) + cudaMemStream ctor (:171-174).
 * device < 0 selects device 0. */
int scn_ctx_create(int device, scn_ctx **ctx);
int scn_ctx_destroy(scn_ctx *ctx);
/* the hipStream_t all work is issued on */
void *scn_ctx_stream(scn_ctx *ctx);
int scn_sync(scn_ctx *ctx);
/* vectorCUDA<T> device storage (vectorCUDA.cu:26-108): raw allocate / free /
 * blocking copies / fill. */
int scn_malloc(scn_ctx *ctx, size_t bytes, void **d_ptr);
int scn_free(scn_ctx *ctx, void *d_ptr);
/* (a null ctx names no stream: the copy waits for every stream of the device) */
int scn_h2d(scn_ctx *ctx, void *d_dst, const void *h_src, size_t bytes);
int scn_d2h(scn_ctx *ctx, void *h_dst, const void *d_src, size_t bytes);
/* The asynchronous half of the same interface (vectorCUDA<T>::copyToCPUAsync,
 * vectorCUDA.cu:110-127, followed by cudaStreamSynchronize in
 * SoftmaxClassifier.cu:24-27): pinned host memory, a copy that is only queued
 * on the context's stream, and an event to wait for it while later work is
 * already queued behind it. */
typedef struct scn_event scn_event;
int scn_host_alloc(scn_ctx *ctx, size_t bytes, void **h_ptr);
int scn_host_free(scn_ctx *ctx, void *h_ptr);
int scn_d2h_async(scn_ctx *ctx, void *h_pinned_dst, const void *d_src, size_t bytes);
/* the upload of the same interface (vectorCUDA<T>::copyToGPUAsync,
 * vectorCUDA.cu:58-87, as BatchProducer::nextBatch uses it for the input
 * features, BatchProducer.cu:127-134): queued on the context's stream; the
 * source must stay untouched until the stream has passed the copy */
int scn_h2d_async(scn_ctx *ctx, void *d_dst, const void *h_pinned_src, size_t bytes);
int scn_event_create(scn_ctx *ctx, scn_event **event);
int scn_event_destroy(scn_event *event);
/* marks the point the stream has reached */
int scn_event_record(scn_ctx *ctx, scn_event *event);
/* blocks the calling thread until the stream has passed the recorded point */
int scn_event_wait(scn_event *event);
/* device-to-device, asynchronous on the context's stream */
int scn_d2d(scn_ctx *ctx, void *d_dst, const void *d_src, size_t bytes);
/* The same copy made by a kernel, for which either side may also be pinned
 * host memory (scn_host_alloc) that the device reaches over the bus: an
 * upload or download that costs the host one kernel launch. */
int scn_copy(scn_ctx *ctx, void *dst, const void *src, size_t bytes);
int scn_fill32(scn_ctx *ctx, void *d_dst, uint32_t word, size_t nWords);

/* ---- sparse grids ----------------------------------------------------- */
/* A scn_grids holds, for one depth of the net, the SparseGrid of every sample
 * of the batch (SparseGrid.h:26-37, SpatiallySparseBatchInterface.h:36), over
 * packed coordinates sample * spatialSize^dimension + key: an occupancy bit
 * mask with a rank prefix per word, the batch-global rows of the active sites
 * in map iteration order (sample, then ascending key), the entry list, and
 * backgroundCol per sample.  Look-ups by coordinate (scn_grids_find) go
 * through a dense table of rows, filled as the grids are built, for batches
 * of up to 2^24 lattice sites, and otherwise through an open-addressing hash
 * table in HBM from packed coordinate to row that the first look-up fills. */
int scn_grids_create(scn_ctx *ctx, scn_grids **grids);
int scn_grids_destroy(scn_ctx *ctx, scn_grids *grids);
/* Start of a batch (SpatiallySparseBatch::reset, SpatiallySparseBatch.cu:14-27,
 * which empties every interface's grids): empties the masks (and the hash
 * tables that are in use) of all n objects in one launch, so that the build / plan calls of the batch
 * need not do it one by one.  Optional; objects it has not seen are emptied
 * by the call that fills them. */
int scn_grids_clear_many(scn_ctx *ctx, scn_grids **grids, int n);
/* The input-layer grids as Picture::codifyInputData leaves them
 * (Picture.h:10-11; OpenCVPicture.cpp:368-402): n active sites given as
 * (sample, key, row) in any order, key = row-major site index in the
 * spatialSize^dimension field, plus backgroundCol per sample (-1: none) and
 * the interface's nSpatialSites.  Keys must be unique within a sample. */
int scn_grids_build(scn_ctx *ctx, scn_grids *grids, int batch, int dimension,
                    int spatialSize, const int32_t *d_sample,
                    const int64_t *d_key, const int32_t *d_row, int64_t n,
                    const int32_t *d_background, int32_t nSpatialSites);
int scn_grids_info(const scn_grids *grids, int *batch, int *dimension,
                   int *spatialSize, int64_t *nActive, int32_t *nSpatialSites);
/* Every entry in map iteration order (sample, then ascending key), and
 * backgroundCol[batch].  Host arrays of nActive / batch elements. */
int scn_grids_download(scn_ctx *ctx, const scn_grids *grids, int32_t *h_sample,
                       int64_t *h_key, int32_t *h_row, int32_t *h_background);
/* mp.find() for n packed queries (sample, key) -> row or -1; device arrays. */
int scn_grids_find(scn_ctx *ctx, const scn_grids *grids,
                   const int32_t *d_sample, const int64_t *d_key, int64_t n,
                   int32_t *d_row);

/* ---- rule books -------------------------------------------------------- */
/* Rule construction is split in two so that the caller owns the rules buffer
 * (SpatiallySparseBatchInterface::rules): plan() finds the output sites,
 * numbers them in the reference's first-touch order under ascending-key map
 * iteration and builds `out`; fill() writes the rules.
 *
 * gridRules(in, out, RegularSquareRegions(nIn, nOut, dimension, size, stride),
 *           nOutputSpatialSites, rules, true, minActive) for every sample
 * (Regions.h:84-87; Regions.cu:528-653 NoMin, :338-526 Min, :658-780 Valid,
 * dispatcher :782-802), as ConvolutionalLayer::preprocess and
 * MaxPoolingLayer::preprocess call it (ConvolutionalLayer.cu:110-118,
 * MaxPoolingLayer.cu:113-118).  minActive: 1, >1, or -1 (valid, 2-D size 3). */
int scn_rules_square_plan(scn_ctx *ctx, const scn_grids *in, scn_grids *out,
                          int nIn, int nOut, int size, int stride,
                          int minActive, int64_t *nOutputSpatialSites);
/* gridRules(in, out, RegularTriangularRegions(...), n, rules, minActive)
 * (Regions.h:120-127; Regions.cu:834-970 NoMin, :972-1164 Min). */
int scn_rules_triangular_plan(scn_ctx *ctx, const scn_grids *in,
                              scn_grids *out, int nIn, int nOut, int size,
                              int stride, int minActive,
                              int64_t *nOutputSpatialSites);
/* gridRules over FractionalPoolingRegions (Regions.cu:121-156; dispatcher
 * :782-802), the rule books of the four fractional max-pooling layers
 * (MaxPoolingLayer.cu:157-420).  The regions of sample b along axis a are
 * [h_inputL[(b d + a) nOut + j], h_inputR[..]) for output coordinate j: what
 * the reference's tick constructors draw (Regions.cu:31-119), host arrays of
 * batch * dimension * nOut ints each.  Region extents lie in 1..poolSize and
 * both bounds are non-decreasing in j.  Rule rows are poolSize^d wide; offsets
 * beyond a region's extent hold -1 (Regions.cu:177-178), which scn_maxpool
 * skips.  Plan, then scn_rules_fill, as for the regular regions. */
int scn_rules_fmp_plan(scn_ctx *ctx, const scn_grids *in, scn_grids *out,
                       int nIn, int nOut, int poolSize,
                       const int32_t *h_inputL, const int32_t *h_inputR,
                       int64_t *nOutSites);
/* TerminalPoolingLayer::preprocess + terminalGridPoolingRules
 * (TerminalPoolingLayer.cu:8-20,81-97).  *ruleWidth = S. */
int scn_rules_terminal_plan(scn_ctx *ctx, const scn_grids *in, scn_grids *out,
                            int64_t *ruleWidth);
/* Rule width of the plan held by `out` (size^d, triangleSize, or S). */
/* Deferred counts.  BatchProducer::preprocessBatch (BatchProducer.cu:40-87)
 * runs every layer's preprocess() back to back on the CPU; on the GPU every
 * plan call above would wait for its counts, one host round trip per layer.
 * With deferral on, a plan whose `out` object has held a plan before returns
 * at once: *nOutSites (or *ruleWidth) is an UPPER BOUND derived from the
 * largest counts that object has seen, buffers sized by it are large enough,
 * and scn_rules_fill on such a pair is bounded the same way.  scn_rules_settle
 * then waits once for the stream and makes the real counts readable
 * (scn_grids_info, scn_rules_width).  It returns SCN_ERR_CAPACITY when a
 * batch outgrew a bound: nothing out of range was written, and the caller
 * plans the batch again with deferral off (that also raises the bounds). */
int scn_ctx_defer_counts(scn_ctx *ctx, int on);
int scn_rules_settle(scn_ctx *ctx);
/* Recorded plans.  gridRules runs per sample (ConvolutionalLayer.cu:114-118,
 * MaxPoolingLayer.cu:116-118) and the layers' preprocess() calls follow one
 * another without anything else in between (BatchProducer.cu:79-81).  With
 * recording on (and deferred counts on), scn_rules_square_plan,
 * scn_rules_triangular_plan, scn_rules_terminal_plan and scn_rules_fill calls
 * that continue from one another -- each plan's `in` being the `out` of the
 * plan before -- are only noted, provided every `out` has held a plan before
 * and a sample's grids fit the LDS of a compute unit (2-D and small 3-D
 * fields); scn_ctx_chain_rules(ctx, 0), scn_rules_settle or any call that
 * cannot join then runs all of them in two launches, one workgroup carrying
 * one sample through every layer.  Results (rules, counts, grids as seen
 * through scn_grids_download / scn_grids_find) are those of the calls made one
 * by one; a sample too large for the LDS is reported by scn_rules_settle as
 * SCN_ERR_CAPACITY like any outgrown bound. */
int scn_ctx_chain_rules(scn_ctx *ctx, int on);
/* how many chains of recorded plans the context has run, and how many plans
 * they held in all (a plan that could not join is not counted) */
int scn_ctx_chain_count(scn_ctx *ctx, int64_t *chains, int64_t *plans);
int scn_rules_width(const scn_grids *out, int64_t *width);
/* Writes nOutputSpatialSites * width int32 rules; capacity in int32s. */
int scn_rules_fill(scn_ctx *ctx, const scn_grids *in, scn_grids *out,
                   int32_t *d_rules, int64_t capacity);

/* ---- feature kernels --------------------------------------------------- */
/* propForwardToMatrixMultiply (ConvolutionalLayer.h:38-40;
 * ConvolutionalLayer.cu:12-41): out[c*nIn + j] = in[rules[c]*nIn + j],
 * c < count.  A negative rule, which the reference's kernel does not guard
 * (ConvolutionalLayer.cu:20-27), gathers a row of zeros; rule books built by
 * this library never hold one here. */
int scn_gather_rows(scn_ctx *ctx, const float *d_in, float *d_out,
                    const int32_t *d_rules, int64_t count, int nIn);
/* replicateArray + d_rowMajorSGEMM_alphaAB_betaC(alpha = beta = p) +
 * applySigmoid / PreLU, test-time branch (NetworkInNetworkLayer.cu:187-200,
 * NetworkInNetworkPReLULayer.cu:158-169; utilities.cu:135-142;
 * SigmoidLayer.cu:187-222): out[M x N] = act(p * (A[M x K] W[K x N] + B)).
 * d_prelu is the per-channel slope vector for SCN_PRELU, else ignored.
 * SCN_SOFTMAX applies dSigmoidSoftmax (SigmoidLayer.cu:160-177) to the rows. */
int scn_nin_forward(scn_ctx *ctx, const float *d_A, const float *d_W,
                    const float *d_B, const float *d_prelu, float *d_out,
                    int64_t M, int K, int N, float p, int act, int precision);
/* Gather and NiN in one kernel: out[M x N] = act(p * (G W + B)) where row m of
 * G is the receptive field of output site m, G[m][q * nIn + c] =
 * in[rules[m * fs + q] * nIn + c], without ever writing G to memory.  Same
 * result as scn_gather_rows followed by scn_nin_forward (fp32), bit for bit.
 * The reference keeps such a fused layer as disabled code
 * (ReallyConvolutionalLayer.cu:27-60, switched off at SparseConvNetCUDA.cu:81);
 * what it replaces on the live path is ConvolutionalLayer::forwards +
 * NetworkInNetwork(PReLU)Layer::forwards (ConvolutionalLayer.cu:125-133,
 * NetworkInNetworkLayer.cu:187-200).  W is [fs * nIn x N].
 * scn_conv_nin_supported tells whether (fs, nIn, N) is in the kernels' range:
 * windows of up to 27 sites over channels in multiples of 4 with N a multiple
 * of 4, or any number of channels when fs * nIn is at most 32 and a multiple
 * of 4 (the first layer of a net: one to three input channels). */
int scn_conv_nin_supported(int fs, int nIn, int N);
int scn_conv_nin_forward(scn_ctx *ctx, const float *d_in,
                         const int32_t *d_rules, int fs, int nIn,
                         const float *d_W, const float *d_B,
                         const float *d_prelu, float *d_out, int64_t M, int N,
                         float p, int act);
/* The same with the operand precision of scn_nin_forward: SCN_FP32, or SCN_BF16
 * for shapes with nIn a multiple of 8, fs * nIn of 64 and N of 32 (operands
 * rounded to bf16 on their way to the MFMA, fp32 accumulation); bit-identical to
 * scn_gather_rows followed by scn_nin_forward with that precision.  (Contractions
 * of up to 32 stay fp32 in every precision, fused or not.) */
int scn_conv_nin_supported_p(int fs, int nIn, int N, int precision);
int scn_conv_nin_forward_p(scn_ctx *ctx, const float *d_in,
                           const int32_t *d_rules, int fs, int nIn,
                           const float *d_W, const float *d_B,
                           const float *d_prelu, float *d_out, int64_t M, int N,
                           float p, int act, int precision);
/* scn_conv_nin_forward_p with SCN_BF16 for a caller that can spare room for a
 * bf16 copy of the input matrix: the nInRows x nIn values are rounded once
 * (nearest even) into d_in16 (2 bytes each, 16-byte aligned) and the
 * contraction reads its rows from there, half the bytes for a matrix whose
 * rows the rules visit many times over.  The operands that reach the MFMA are
 * the ones scn_conv_nin_forward_p(SCN_BF16) rounds in registers, so the result
 * is the same bit for bit; shapes the bf16 W-streaming kernel does not take
 * run as scn_conv_nin_forward_p(SCN_BF16) does.  Same reference operator
 * (NetworkInNetworkLayer.cu:187-200 after ConvolutionalLayer.cu:125-133). */
int scn_conv_nin_forward_a16(scn_ctx *ctx, const float *d_in, int64_t nInRows,
                             void *d_in16, const int32_t *d_rules, int fs,
                             int nIn, const float *d_W, const float *d_B,
                             const float *d_prelu, float *d_out, int64_t M,
                             int N, float p, int act);
/* maxPool (MaxPoolingLayer.h:6-7; MaxPoolingLayer.cu:9-72): first maximum
 * wins, negative rules skipped, choice = rule * C + channel. */
int scn_maxpool(scn_ctx *ctx, const float *d_in, float *d_out,
                const int32_t *d_rules, int64_t nOutSites, int ps, int C,
                int32_t *d_choice);
/* The same for a caller that knows how many rows d_in has: the choices are
 * 32-bit element indices into d_in, as the reference's poolingChoices are
 * (MaxPoolingLayer.cu:9-35), so an input of more than 2^31 - 1 elements is
 * refused with SCN_ERR_CAPACITY instead of being indexed modulo 2^32. */
int scn_maxpool_checked(scn_ctx *ctx, const float *d_in, int64_t nInRows,
                        float *d_out, const int32_t *d_rules,
                        int64_t nOutSites, int ps, int C, int32_t *d_choice);
/* terminalPool (TerminalPoolingLayer.cu:22-46): mean over the rows listed
 * before the first negative rule, summed in rule order. */
int scn_terminal_pool(scn_ctx *ctx, const float *d_in, float *d_out,
                      const int32_t *d_rules, int64_t count, int S, int C);
/* dSigmoidSoftmax (SigmoidLayer.cu:160-177). */
int scn_softmax_rows(scn_ctx *ctx, const float *d_in, float *d_out, int64_t M,
                     int N);

/* ---- backward pass and weight update (training) -------------------------- */
/* dDerivativeOfCostWRTpreSoftmaxTopLevelWeights (SoftmaxClassifier.cu:7-14):
 * delta[k][i] = probs[k][i] - (i == labels[k]), the gradient of the negative
 * log-likelihood with respect to the soft-max layer's input. */
int scn_softmax_grad(scn_ctx *ctx, const float *d_probs,
                     const int32_t *d_labels, float *d_delta, int64_t batch,
                     int N);
/* What NetworkInNetwork(PReLU)Layer::backwards does to the output gradient
 * before the two matrix products: applySigmoidBackProp in place
 * (NetworkInNetworkLayer.cu:222, SigmoidLayer.cu:23-177 and :224-262; the
 * derivative is written through the layer's output b: ReLU and the leaky
 * forms test b > 0, tanh is (1 + b)(1 - b), the logistic b(1 - b), soft-max
 * and none pass the gradient through) or PReLUBackprop
 * (NetworkInNetworkPReLULayer.cu:25-47: dprelu[c] = sum d * (b > 0 ? 0 :
 * b / alpha_c), then d *= b > 0 ? 1 : alpha_c), and columnSum of the result
 * into the bias gradient (NetworkInNetworkLayer.cu:84-105).  d_db[N] and, for
 * SCN_PRELU, d_dprelu[N] are overwritten. */
int scn_activation_backward(scn_ctx *ctx, const float *d_out, float *d_delta,
                            int64_t M, int N, int act, const float *d_prelu,
                            float *d_db, float *d_dprelu);
/* d_rowMajorSGEMM_alphaAtB_betaC with alpha 1, beta 0 (utilities.cu:144-152;
 * call site NetworkInNetworkLayer.cu:225-228): dW[K x N] = A^T D, A [M x K],
 * D [M x N], all row-major.  fp32 MFMA, fp32 atomics across row ranges. */
int scn_sgemm_AtB(scn_ctx *ctx, const float *d_A, const float *d_D,
                  float *d_dW, int64_t M, int K, int N);
/* d_rowMajorSGEMM_alphaABt_betaC with alpha 1, beta 0 (utilities.cu:153-161;
 * call site NetworkInNetworkLayer.cu:269-272): dA[M x K] = D[M x N] W^T,
 * W [K x N].  d_workspace holds scn_sgemm_ABt_workspace(N, K) floats (the
 * transposed weights, which the forward contraction kernels then stream). */
int64_t scn_sgemm_ABt_workspace(int N, int K);
int scn_sgemm_ABt(scn_ctx *ctx, const float *d_D, const float *d_W,
                  float *d_dA, int64_t M, int N, int K, float *d_workspace);
/* scn_sgemm_ABt for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): no
 * counterpart in the reference.  The transposed weights go to a static device
 * array of scn_sgemm_ABt_static_limit() floats (4 MiB, held by every device
 * the library runs on until the process ends) instead of a workspace; the call
 * allocates and frees nothing.  scn_sgemm_ABt_workspace(N, K) beyond the limit
 * is refused with SCN_ERR_CAPACITY.  All calls on one device share the array:
 * calls that overlap on one device (two contexts, two streams) race. */
int64_t scn_sgemm_ABt_static_limit(void);
int scn_sgemm_ABt_static(scn_ctx *ctx, const float *d_D, const float *d_W,
                         float *d_dA, int64_t M, int N, int K);
/* dGradientDescent / dGradientDescentKeepPositive (NetworkInNetworkLayer.cu:
 * 27-41, NetworkInNetworkPReLULayer.cu:68-83), "NAG light": w -= m mu;
 * m = mu m - lr (1 - mu) d; w += m (1 + mu); keepPositive clamps w at 0.001. */
int scn_nag_update(scn_ctx *ctx, const float *d_delta, float *d_momentum,
                   float *d_weights, int64_t n, float learningRate,
                   float momentum, int keepPositive);
/* The same step on up to SCN_NAG_MAX tensors in one launch (what backwards()
 * applies to W, B and the PReLU slopes one after the other,
 * NetworkInNetworkLayer.cu:274-287, NetworkInNetworkPReLULayer.cu:211-214 and
 * :262-275).  With clearGradients the gradients are left zero, which is what
 * the accumulating products below expect of the next batch. */
#define SCN_NAG_MAX 4
typedef struct scn_nag_item {
  float *d_delta;
  float *d_momentum;
  float *d_weights;
  int64_t n;
  int keepPositive;
} scn_nag_item;
int scn_nag_update_many(scn_ctx *ctx, const scn_nag_item *items, int nItems,
                        float learningRate, float momentum,
                        int clearGradients);
/* scn_activation_backward and scn_sgemm_AtB with beta 1: they add to d_db,
 * d_dprelu and d_dW instead of overwriting them (the reference's products are
 * all beta 0; a caller that keeps its gradient buffers zero between batches,
 * as scn_nag_update_many leaves them, saves the clearing launches). */
int scn_activation_backward_acc(scn_ctx *ctx, const float *d_out,
                                float *d_delta, int64_t M, int N, int act,
                                const float *d_prelu, float *d_db,
                                float *d_dprelu);
int scn_sgemm_AtB_acc(scn_ctx *ctx, const float *d_A, const float *d_D,
                      float *d_dW, int64_t M, int K, int N);
/* Dropout during training.  dShrinkMatrixForDropout / dShrinkVectorForDropout
 * (NetworkInNetworkLayer.cu:7-25): w[i][j] = W[inPresent[i]][outPresent[j]],
 * W with rows of nOut floats; a null d_inPresent keeps the rows (row i of w
 * is row i of W), so a vector is a matrix of one row.  dGradientDescentShrunkMatrix / ...ShrunkVector
 * (NetworkInNetworkLayer.cu:43-82): the momentum step of scn_nag_update on
 * exactly those entries, delta being the gradient of the shrunk matrix. */
int scn_shrink_matrix(scn_ctx *ctx, const float *d_W, float *d_w,
                      const int32_t *d_inPresent, const int32_t *d_outPresent,
                      int nOut, int nInPresent, int nOutPresent);
int scn_nag_update_shrunk(scn_ctx *ctx, const float *d_delta,
                          float *d_momentum, float *d_weights,
                          const int32_t *d_inPresent,
                          const int32_t *d_outPresent, int nOut,
                          int nInPresent, int nOutPresent, float learningRate,
                          float momentum);
/* What a RESCALEBATCH pass (scaleWeights, NetworkInNetworkLayer.cu:203-218)
 * needs of vectorCUDA<float>: meanAbs (vectorCUDA.cu:121-155; here the sum of
 * |x[i]| in double, returned to the host: the call waits for the stream) and
 * multiplicativeRescale (vectorCUDA.cu:156-170). */
int scn_sum_abs(scn_ctx *ctx, const float *d_x, int64_t n, double *h_sum);
int scn_scale(scn_ctx *ctx, float *d_x, int64_t n, float multiplier);
/* propBackwardFromMatrixMultiply (ConvolutionalLayer.cu:42-72):
 * din[rules[c] * nIn + j] += dconv[c * nIn + j], c < count; the caller zeroes
 * din first (ConvolutionalLayer.cu:141).  Negative rules are skipped. */
int scn_gather_rows_backward(scn_ctx *ctx, float *d_din, const float *d_dconv,
                             const int32_t *d_rules, int64_t count, int nIn);
/* maxPoolBackProp (MaxPoolingLayer.cu:74-93): din[choice[i]] += dout[i] over
 * the count x C elements of dout; the caller zeroes din first. */
int scn_maxpool_backward(scn_ctx *ctx, float *d_din, const float *d_dout,
                         int64_t count, int C, const int32_t *d_choice);
/* terminalPoolBackProp (TerminalPoolingLayer.cu:48-73): every row listed for
 * sample b before the first negative rule is assigned dout[b] / (number of
 * rows listed); the caller zeroes din first. */
int scn_terminal_pool_backward(scn_ctx *ctx, float *d_din, const float *d_dout,
                               const int32_t *d_rules, int64_t count, int C,
                               int S);

/* ---- per-kernel timing -------------------------------------------------- */
/* HIP events recorded on the context's stream around every kernel of one
 * family; off by default.  The reference only times whole dataset passes
 * (SparseConvNetCUDA.cu:277-324). */
enum {
  SCN_K_GRID_BUILD = 0,
  SCN_K_RULES = 1,
  SCN_K_GATHER = 2,
  SCN_K_NIN = 3,
  SCN_K_MAXPOOL = 4,
  SCN_K_TERMINAL = 5,
  SCN_K_SOFTMAX = 6,
  SCN_K_CONV_NIN = 7, /* gather fused into the NiN contraction */
  SCN_K_PROBE = 8,    /* scn_prof_probe: what a span costs by itself */
  SCN_K_BACKWARD = 9, /* every kernel of the backward pass and the update */
  SCN_K_COUNT = 10
};
int scn_prof_enable(scn_ctx *ctx, int on);
/* label attached to the spans recorded from now on (e.g. the layer index) */
int scn_prof_tag(scn_ctx *ctx, int tag);
/* synchronises and hands back every span recorded since the last read:
 * family, tag and milliseconds of up to `capacity` spans, *n = their number
 * (spans beyond the capacity are dropped).  Also adds them to the totals. */
int scn_prof_spans(scn_ctx *ctx, int capacity, int32_t *family, int32_t *tag,
                   double *ms, int32_t *n);
int scn_prof_reset(scn_ctx *ctx);
/* Records one span of family SCN_K_PROBE around nothing (with_kernel == 0) or
 * around a kernel of one wavefront that does nothing (with_kernel != 0): the
 * floor under every other span, for callers that want to subtract it. */
int scn_prof_probe(scn_ctx *ctx, int with_kernel);
/* synchronises, then returns accumulated milliseconds and number of calls */
int scn_prof_read(scn_ctx *ctx, int family, double *ms, int64_t *calls);

#ifdef __cplusplus
}
#endif
#endif
