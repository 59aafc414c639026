/*
 * CPU oracle for the spatially-sparse forward path, and for the backward pass
 * and weight update that follow it in a training batch.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the product (the HIP library, the C++ host classes, the Python
 * binding) may include, link or call anything declared here; only tests, the
 * smoke check and the CPU-baseline leg of the benchmark use it as a checker.
 *
 * Every function restates, on the CPU, what the cited reference code computes.
 * Map iteration order is the reference's compile-time option (d), `vectorHash`
 * (SparseGrid.h:15-16,68-77; vectorHash.cpp:40-55): ascending key.
 */
#ifndef SCN_ORACLE_H
#define SCN_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* One SparseGrid per sample of a batch (SparseGrid.h:68-77), dense-vector
 * backed like vectorHash (vectorHash.h:6-19). */
typedef struct orc_grids orc_grids;

orc_grids *orc_grids_create(int batch);
void orc_grids_destroy(orc_grids *g);
int orc_grids_batch(const orc_grids *g);
/* grid.mp[key] = row for n pairs, in the given order; grid.backgroundCol = bg. */
void orc_grids_set(orc_grids *g, int item, int64_t n, const int64_t *keys,
                   const int32_t *rows, int32_t backgroundCol);
int64_t orc_grids_size(const orc_grids *g, int item); /* mp.size() */
int32_t orc_grids_background(const orc_grids *g, int item);
/* entries in iteration (ascending key) order */
void orc_grids_get(const orc_grids *g, int item, int64_t *keys, int32_t *rows);

/* Growable int vector standing in for std::vector<int> rules. */
typedef struct orc_ivec orc_ivec;
orc_ivec *orc_ivec_create(void);
void orc_ivec_destroy(orc_ivec *v);
int64_t orc_ivec_size(const orc_ivec *v);
const int32_t *orc_ivec_data(const orc_ivec *v);

/* Regions.cu:13-29 */
int orc_sq_inputL(int size, int stride, int j);
int orc_sq_inputR(int size, int stride, int j);
int orc_sq_outputL(int size, int stride, int i);
int orc_sq_outputR(int size, int stride, int nOut, int i);
/* utilities.cu:15-32 */
int orc_ipow(int base, int e);
int orc_triangle_size(int linearSize, int dimension);
/* Regions.cu:804-832: fills ord[s^d], returns S */
int orc_tri_ord(int s, int dimension, int32_t *ord);

/* gridRules(..., uniformSizeRegions=true, minActiveInputs) dispatcher,
 * Regions.cu:782-802, applied to every item of the batch in order as
 * ConvolutionalLayer::preprocess / MaxPoolingLayer::preprocess do
 * (ConvolutionalLayer.cu:112-118, MaxPoolingLayer.cu:113-118).
 * minActive == 1  -> gridRulesOverlappingNoMin (Regions.cu:528-653)
 * minActive  > 1  -> gridRulesOverlappingMin   (Regions.cu:338-526)
 * minActive == -1 -> gridRulesValid            (Regions.cu:658-780)
 * Returns nOutputSpatialSites (batch-global), -1 on bad arguments. */
int64_t orc_rules_square(const orc_grids *in, orc_grids *out, int dimension,
                         int nIn, int nOut, int size, int stride,
                         int minActive, orc_ivec *rules);
/* gridRules(RegularTriangularRegions) Regions.cu:1166-1174
 * (NoMin :834-970, Min :972-1164). */
int64_t orc_rules_triangular(const orc_grids *in, orc_grids *out,
                             int dimension, int nIn, int nOut, int size,
                             int stride, int minActive, orc_ivec *rules);
/* TerminalPoolingLayer::preprocess + terminalGridPoolingRules
 * (TerminalPoolingLayer.cu:8-20,81-97).  Returns S (rule-row width). */
int64_t orc_rules_terminal(const orc_grids *in, orc_grids *out,
                           orc_ivec *rules);

/* dPropForwardToMatrixMultiplyInput, ConvolutionalLayer.cu:12-31 */
void orc_gather_rows(const float *in, float *out, const int32_t *rules,
                     int64_t count, int nIn);
/* replicateArray + d_rowMajorSGEMM_alphaAB_betaC(alpha=beta=p) + applySigmoid /
 * PreLU, test-time branch: NetworkInNetworkLayer.cu:187-200,
 * NetworkInNetworkPReLULayer.cu:158-169, SigmoidLayer.cu:6-22,118-135,187-222.
 * act uses the reference's ActivationFunction numbering (types.h:11-20).
 * Accumulates in fp32, k ascending. */
void orc_nin_forward(const float *A, const float *W, const float *B,
                     const float *prelu, float *out, int64_t M, int K, int N,
                     float p, int act);
/* same contraction accumulated in double; rounding reference for tolerances */
void orc_nin_forward_f64(const float *A, const float *W, const float *B,
                         const float *prelu, double *out, int64_t M, int K,
                         int N, float p, int act);
/* dSigmoidSoftmax, SigmoidLayer.cu:160-177 */
void orc_softmax_rows(const float *in, float *out, int64_t M, int N);
/* dMaxPool, MaxPoolingLayer.cu:9-35 */
void orc_maxpool(const float *in, float *out, const int32_t *rules,
                 int64_t nOutSites, int ps, int C, int32_t *choice);
/* dTerminalPool, TerminalPoolingLayer.cu:22-34 */
void orc_terminal_pool(const float *in, float *out, const int32_t *rules,
                       int64_t count, int S, int C);
/* vectorTopIndices, utilities.cu:35-56 */
void orc_top_indices(const float *test, int n, int k, int32_t *indices);
/* SoftmaxClassifier, SoftmaxClassifier.cu:33-54 (labelled, non-training part).
 * Fills predictions[batch*nTop]; returns mistakes; *nll accumulates. */
int orc_softmax_classifier(const float *probs, const int32_t *labels,
                           int batch, int nClasses, int nTop,
                           int32_t *predictions, float *nll);

void orc_set_threads(int n); /* OpenMP threads for the numeric loops */
int orc_get_threads(void);

/* ---- fractional max-pooling regions and their rule books ---- */
int orc_fmp_ticks_po(int nIn, int nOut, int poolSize, double u,
                     int32_t *inputL, int32_t *inputR);
int orc_fmp_ticks_pd(int nIn, int nOut, int poolSize, double u,
                     int32_t *inputL, int32_t *inputR);
int orc_fmp_increments(int nIn, int nOut, int overlapping, int32_t *inc);
int orc_fmp_ticks_ro(int nIn, int nOut, int poolSize, const int32_t *inc,
                     int32_t *inputL, int32_t *inputR);
int orc_fmp_ticks_rd(int nIn, int nOut, const int32_t *inc, int32_t *inputL,
                     int32_t *inputR);
int64_t orc_rules_fmp(const orc_grids *in, orc_grids *out, int dimension,
                      int nIn, int nOut, int poolSize, const int32_t *inputL,
                      const int32_t *inputR, int uniform, orc_ivec *rules);

/* ---- backward pass (training); citations in scn_oracle.c ---- */
void orc_softmax_grad(const float *probs, const int32_t *labels, float *delta,
                      int64_t batch, int N);
void orc_activation_backward(const float *out, float *delta, int64_t M, int N,
                             int act, const float *prelu, float *db,
                             float *dprelu);
void orc_sgemm_AtB(const float *A, const float *D, float *dW, int64_t M, int K,
                   int N);
void orc_sgemm_ABt(const float *D, const float *W, float *dA, int64_t M, int N,
                   int K);
void orc_nag_update(const float *delta, float *mom, float *wts, int64_t n,
                    float learningRate, float momentum, int keepPositive);
void orc_gather_rows_backward(float *din, const float *dconv,
                              const int32_t *rules, int64_t count, int nIn);
void orc_maxpool_backward(float *din, const float *dout, int64_t count, int C,
                          const int32_t *choice);
void orc_terminal_pool_backward(float *din, const float *dout,
                                const int32_t *rules, int64_t count, int C,
                                int S);

#ifdef __cplusplus
}
#endif
#endif
