/*
 * CPU oracle for the spatially-sparse forward path (and the training pass
 * behind it).  TEST INFRASTRUCTURE ONLY:
 * the product never links this file.  See scn_oracle.h for the contract and
 * the reference citations of every entry point.
 *
 * Pins (what each function has been checked against, in tests/):
 *   region arithmetic    brute force  j in [outputL(i),outputR(i)) <=> inputL(j) <= i < inputR(j)
 *   square rules NoMin   reference-executed known-answer vectors (tests/golden/rulebook_kats.json)
 *                        + independent brute-force builder (dilation, sort by (min key, key))
 *   square rules Min     brute-force builder, minActive in {2,3}        [no reference vector]
 *   square rules Valid   brute-force builder                            [no reference vector]
 *   triangular NoMin     reference-executed known-answer vector + brute force
 *   triangular Min       brute-force builder                            [no reference vector]
 *   terminal rules       brute force
 *   fractional regions   tick tables: closed forms at u = 0, partition / coverage invariants, extents in
 *                        {floor, ceil} of the ratio; rule books: brute-force builder over explicit windows
 *   gather / max-pool    brute force on random inputs, tie and negative-rule cases
 *   NiN                  numpy float64 GEMM, W = I, W = 0, single non-zero
 *   softmax / top-k      closed forms
 *   backward pass        gather / max-pool / terminal: adjoint identity <P x, y> = <x, P^T y>;
 *                        soft-max gradient, activation derivatives, dW, dB, dA, dPReLU: central finite
 *                        differences of a float64 numpy loss; weight update: algebraic identities
 *                        (momentum 0 is plain gradient descent; w' = w + m' + mu (m' - m))
 * Parity unpinned (no reference vector can exist in this build): the row order
 * the reference gets from google::dense_hash_map iteration (its default map),
 * cuBLAS sgemm's and the atomics' summation order, and every draw of the
 * reference's clock-seeded RNG (dropout subsets, fractional pooling regions,
 * the order of training batches): those are arguments of the functions here.
 *
 * Dimension 4 is refused: the reference's own d == 4 NoMin loop starts axis 0
 * at outputL(0, i1) (Regions.cu:614) and writes outside its rule row.
 */
#include "scn_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define VH_EMPTY (-99) /* vectorHash.cpp:7 */

static int g_threads = 1;
void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int orc_get_threads(void) { return g_threads; }

/* ---------- vectorHash (vectorHash.cpp) ---------- */
typedef struct {
  int32_t *vec;
  int64_t len; /* vec.size() */
  int64_t cap;
  int64_t count;
  int32_t backgroundCol;
} vgrid;

struct orc_grids {
  int batch;
  vgrid *g;
};

static void vg_resize(vgrid *v, int64_t n) { /* vec.resize(n, -99), grow only */
  if (n <= v->len)
    return;
  if (n > v->cap) {
    int64_t c = v->cap ? v->cap : 16;
    while (c < n)
      c *= 2;
    v->vec = (int32_t *)realloc(v->vec, (size_t)c * sizeof(int32_t));
    v->cap = c;
  }
  for (int64_t i = v->len; i < n; ++i)
    v->vec[i] = VH_EMPTY;
  v->len = n;
}
/* vectorHash::operator[] (vectorHash.cpp:5-11) */
static int32_t *vg_at(vgrid *v, int64_t idx) {
  if (idx >= v->len)
    vg_resize(v, idx + 1);
  if (v->vec[idx] == VH_EMPTY)
    v->count++;
  return &v->vec[idx];
}
/* vectorHash::find (vectorHash.cpp:16-22): NULL stands for end() */
static const int32_t *vg_find(const vgrid *v, int64_t idx) {
  if (idx < 0 || idx >= v->len || v->vec[idx] == VH_EMPTY)
    return NULL;
  return &v->vec[idx];
}
static void vg_clear(vgrid *v) {
  free(v->vec);
  v->vec = NULL;
  v->len = v->cap = v->count = 0;
  v->backgroundCol = -1; /* SparseGrid.h:76 */
}

orc_grids *orc_grids_create(int batch) {
  orc_grids *g = (orc_grids *)calloc(1, sizeof(*g));
  g->batch = batch;
  g->g = (vgrid *)calloc((size_t)(batch > 0 ? batch : 1), sizeof(vgrid));
  for (int i = 0; i < batch; ++i)
    g->g[i].backgroundCol = -1;
  return g;
}
void orc_grids_destroy(orc_grids *g) {
  if (!g)
    return;
  for (int i = 0; i < g->batch; ++i)
    free(g->g[i].vec);
  free(g->g);
  free(g);
}
int orc_grids_batch(const orc_grids *g) { return g->batch; }
void orc_grids_set(orc_grids *g, int item, int64_t n, const int64_t *keys,
                   const int32_t *rows, int32_t backgroundCol) {
  vgrid *v = &g->g[item];
  vg_clear(v);
  v->backgroundCol = backgroundCol;
  for (int64_t i = 0; i < n; ++i)
    *vg_at(v, keys[i]) = rows[i];
}
int64_t orc_grids_size(const orc_grids *g, int item) {
  return g->g[item].count;
}
int32_t orc_grids_background(const orc_grids *g, int item) {
  return g->g[item].backgroundCol;
}
void orc_grids_get(const orc_grids *g, int item, int64_t *keys,
                   int32_t *rows) {
  const vgrid *v = &g->g[item];
  int64_t o = 0;
  for (int64_t k = 0; k < v->len; ++k)
    if (v->vec[k] != VH_EMPTY) {
      keys[o] = k;
      rows[o] = v->vec[k];
      ++o;
    }
}

/* ---------- std::vector<int> ---------- */
struct orc_ivec {
  int32_t *d;
  int64_t n, cap;
};
orc_ivec *orc_ivec_create(void) { return (orc_ivec *)calloc(1, sizeof(orc_ivec)); }
void orc_ivec_destroy(orc_ivec *v) {
  if (v) {
    free(v->d);
    free(v);
  }
}
int64_t orc_ivec_size(const orc_ivec *v) { return v->n; }
const int32_t *orc_ivec_data(const orc_ivec *v) { return v->d; }
static void iv_reserve(orc_ivec *v, int64_t n) {
  if (n > v->cap) {
    int64_t c = v->cap ? v->cap : 64;
    while (c < n)
      c *= 2;
    v->d = (int32_t *)realloc(v->d, (size_t)c * sizeof(int32_t));
    v->cap = c;
  }
}
static void iv_push(orc_ivec *v, int32_t x) {
  iv_reserve(v, v->n + 1);
  v->d[v->n++] = x;
}
/* vector::resize(n, fill) */
static void iv_resize(orc_ivec *v, int64_t n, int32_t fill) {
  if (n > v->n) {
    iv_reserve(v, n);
    for (int64_t i = v->n; i < n; ++i)
      v->d[i] = fill;
  }
  v->n = n;
}

/* ---------- region arithmetic ---------- */
int orc_ipow(int base, int e) { /* utilities.cu:15-25 */
  int r = 1;
  while (e) {
    if (e & 1)
      r *= base;
    e >>= 1;
    base *= base;
  }
  return r;
}
int orc_triangle_size(int linearSize, int dimension) { /* utilities.cu:27-32 */
  int fs = 1;
  for (int i = 1; i <= dimension; ++i)
    fs = fs * (linearSize + dimension - i) / i;
  return fs;
}
int orc_sq_inputL(int size, int stride, int j) {
  (void)size;
  return j * stride;
}
int orc_sq_inputR(int size, int stride, int j) { return j * stride + size; }
int orc_sq_outputL(int size, int stride, int i) {
  int v = (i - size + stride) / stride; /* C division truncates toward zero */
  return v > 0 ? v : 0;
}
int orc_sq_outputR(int size, int stride, int nOut, int i) {
  int v = i / stride + 1;
  return v < nOut ? v : nOut;
}
int orc_tri_ord(int s, int dimension, int32_t *ord) { /* Regions.cu:810-826 */
  int S = 0;
  int n = orc_ipow(s, dimension);
  for (int i = 0; i < n; ++i) {
    int j = i, J = 0;
    while (j > 0) {
      J += j % s;
      j /= s;
    }
    ord[i] = (J < s) ? S++ : -1;
  }
  return S;
}

/* key -> coordinates, axis 0 most significant (Regions.cu:560-561,583-585) */
static void decode(int64_t key, int n, int d, int *c) {
  for (int a = d - 1; a >= 0; --a) {
    c[a] = (int)(key % n);
    key /= n;
  }
}
static int64_t encode(const int *c, int n, int d) {
  int64_t k = 0;
  for (int a = 0; a < d; ++a)
    k = k * n + c[a];
  return k;
}
/* advance an odometer j over the box [lo, hi); axis d-1 fastest */
static int odo_next(int *j, const int *lo, const int *hi, int d) {
  for (int a = d - 1; a >= 0; --a) {
    if (++j[a] < hi[a])
      return 1;
    j[a] = lo[a];
  }
  return 0;
}
static int box_nonempty(const int *lo, const int *hi, int d) {
  for (int a = 0; a < d; ++a)
    if (lo[a] >= hi[a])
      return 0;
  return 1;
}

/* append the all-background row when the output grid is not full
 * (Regions.cu:647-652, 520-526, 774-779, 963-969, 1157-1164) */
static void background_row(const vgrid *in, vgrid *out, int64_t fullSize,
                           int width, int64_t *nSites, orc_ivec *rules) {
  if (out->count < fullSize) {
    for (int i = 0; i < width; ++i)
      iv_push(rules, in->backgroundCol);
    out->backgroundCol = (int32_t)((*nSites)++);
  }
}

/* gridRulesOverlappingNoMin, Regions.cu:528-653 */
static void sq_nomin(const vgrid *in, vgrid *out, int d, int nIn, int nOut,
                     int s, int stride, int64_t *nSites, orc_ivec *rules) {
  int sd = orc_ipow(s, d);
  vg_resize(out, orc_ipow(nOut, d)); /* Regions.cu:535-537 */
  for (int64_t key = 0; key < in->len; ++key) {
    if (in->vec[key] == VH_EMPTY)
      continue;
    int i[4], lo[4], hi[4], j[4];
    decode(key, nIn, d, i);
    for (int a = 0; a < d; ++a) {
      lo[a] = orc_sq_outputL(s, stride, i[a]);
      hi[a] = orc_sq_outputR(s, stride, nOut, i[a]);
      j[a] = lo[a];
    }
    if (!box_nonempty(lo, hi, d))
      continue;
    do {
      int64_t outKey = encode(j, nOut, d);
      int off = 0;
      for (int a = 0; a < d; ++a)
        off = off * s + (i[a] - orc_sq_inputL(s, stride, j[a]));
      const int32_t *f = vg_find(out, outKey);
      if (!f) {
        int32_t *slot = vg_at(out, outKey);
        *slot = (int32_t)((*nSites)++);
        iv_resize(rules, *nSites * sd, in->backgroundCol);
        f = slot;
      }
      rules->d[(int64_t)*f * sd + off] = in->vec[key];
    } while (odo_next(j, lo, hi, d));
  }
  background_row(in, out, orc_ipow(nOut, d), sd, nSites, rules);
}

/* gridRulesOverlappingMin, Regions.cu:338-526 */
static void sq_min(const vgrid *in, vgrid *out, int d, int nIn, int nOut,
                   int s, int stride, int minActive, int64_t *nSites,
                   orc_ivec *rules) {
  int sd = orc_ipow(s, d);
  vg_resize(out, orc_ipow(nOut, d));
  for (int64_t key = 0; key < in->len; ++key) {
    if (in->vec[key] == VH_EMPTY)
      continue;
    int i[4], lo[4], hi[4], j[4];
    decode(key, nIn, d, i);
    for (int a = 0; a < d; ++a) {
      lo[a] = orc_sq_outputL(s, stride, i[a]);
      hi[a] = orc_sq_outputR(s, stride, nOut, i[a]);
      j[a] = lo[a];
    }
    if (!box_nonempty(lo, hi, d))
      continue;
    do {
      int64_t outKey = encode(j, nOut, d);
      if (vg_find(out, outKey))
        continue;
      int active = 0;
      int wlo[4], whi[4], ii[4];
      for (int a = 0; a < d; ++a) {
        wlo[a] = orc_sq_inputL(s, stride, j[a]);
        whi[a] = orc_sq_inputR(s, stride, j[a]);
        ii[a] = wlo[a];
      }
      do {
        const int32_t *f = vg_find(in, encode(ii, nIn, d));
        if (!f)
          iv_push(rules, in->backgroundCol);
        else {
          iv_push(rules, *f);
          active++;
        }
      } while (odo_next(ii, wlo, whi, d));
      if (active >= minActive) {
        *vg_at(out, outKey) = (int32_t)((*nSites)++);
      } else {
        *vg_at(out, outKey) = -2;
        iv_resize(rules, *nSites * sd, 0);
      }
    } while (odo_next(j, lo, hi, d));
  }
  for (int64_t k = 0; k < out->len; ++k) /* Regions.cu:517-519 */
    if (out->vec[k] == -2) {
      out->vec[k] = VH_EMPTY;
      out->count--;
    }
  background_row(in, out, orc_ipow(nOut, d), sd, nSites, rules);
}

/* gridRulesValid, Regions.cu:658-780; only its 2-D case is live code */
static int sq_valid(const vgrid *in, vgrid *out, int d, int nIn, int nOut,
                    int s, int stride, int64_t *nSites, orc_ivec *rules) {
  if (s != 3 || d != 2)
    return -1; /* assert(regions.s == 3); cases 1,3,4 assert(0) */
  int sd = orc_ipow(s, d);
  vg_resize(out, orc_ipow(nOut, d));
  for (int64_t key = 0; key < in->len; ++key) {
    if (in->vec[key] == VH_EMPTY)
      continue;
    int i0 = (int)((key / nIn) % nIn), i1 = (int)(key % nIn);
    if (i0 >= 1 && i1 >= 1 && i0 <= nOut && i1 <= nOut) {
      int j0 = i0 - 1, j1 = i1 - 1;
      int64_t outKey = (int64_t)j0 * nOut + j1;
      *vg_at(out, outKey) = (int32_t)((*nSites)++);
      for (int ii0 = orc_sq_inputL(s, stride, j0);
           ii0 < orc_sq_inputR(s, stride, j0); ++ii0)
        for (int ii1 = orc_sq_inputL(s, stride, j1);
             ii1 < orc_sq_inputR(s, stride, j1); ++ii1) {
          const int32_t *f = vg_find(in, (int64_t)ii0 * nIn + ii1);
          iv_push(rules, f ? *f : in->backgroundCol);
        }
    }
  }
  background_row(in, out, orc_ipow(nOut, d), sd, nSites, rules);
  return 0;
}

static void reset_out(orc_grids *out) {
  for (int i = 0; i < out->batch; ++i)
    vg_clear(&out->g[i]);
}

/* ---------- fractional max-pooling regions (Regions.cu:31-156) ----------
 * The random draw itself (u, or the shuffled increments) is the caller's: the
 * reference takes it from a clock-seeded mt19937. */

/* PseudorandomOverlappingFmpTicks, Regions.cu:31-46 */
int orc_fmp_ticks_po(int nIn, int nOut, int poolSize, double u,
                     int32_t *inputL, int32_t *inputR) {
  if (nIn < nOut - 1 + poolSize || nOut < 2)
    return -1;
  double alpha = (nIn - poolSize) * 1.0 / (nOut - 1);
  for (int j = 0; j < nOut; ++j) {
    int i = (int)((j + u) * alpha) - (int)(u * alpha);
    inputL[j] = i;
    inputR[j] = i + poolSize;
  }
  return inputR[nOut - 1] == nIn ? 0 : -1;
}
/* PseudorandomNonOverlappingFmpTicks, Regions.cu:59-71 */
int orc_fmp_ticks_pd(int nIn, int nOut, int poolSize, double u,
                     int32_t *inputL, int32_t *inputR) {
  double alpha = nIn * 1.0 / nOut;
  if (nIn < nOut - 1 + poolSize || (int)ceil(alpha) != poolSize)
    return -1;
  for (int j = 0; j < nOut; ++j)
    inputL[j] = (int)((j + u) * alpha) - (int)(u * alpha);
  for (int j = 1; j <= nOut; ++j)
    inputR[j - 1] = (int)((j + u) * alpha) - (int)(u * alpha);
  return inputR[nOut - 1] == nIn ? 0 : -1;
}
/* the increments RandomOverlappingFmpTicks / RandomNonOverlappingFmpTicks
 * shuffle (Regions.cu:87-90, 113-116); returns how many there are */
int orc_fmp_increments(int nIn, int nOut, int overlapping, int32_t *inc) {
  int alpha = (int)(nIn * 1.0 / nOut);
  int first = nOut * (alpha + 1) - nIn;
  int total = overlapping ? nOut - 1 : nOut;
  for (int k = 0; k < total; ++k)
    inc[k] = k < first ? alpha : alpha + 1;
  return total;
}
/* RandomOverlappingFmpTicks from shuffled increments, Regions.cu:91-98 */
int orc_fmp_ticks_ro(int nIn, int nOut, int poolSize, const int32_t *inc,
                     int32_t *inputL, int32_t *inputR) {
  if (nIn <= nOut)
    return -1;
  inputL[0] = 0;
  inputR[0] = poolSize;
  for (int i = 0; i < nOut - 1; i++) {
    inputL[i + 1] = inputL[i] + inc[i];
    inputR[i + 1] = inputL[i + 1] + poolSize;
  }
  return inputR[nOut - 1] == nIn ? 0 : -1;
}
/* RandomNonOverlappingFmpTicks from shuffled increments, Regions.cu:117-124 */
int orc_fmp_ticks_rd(int nIn, int nOut, const int32_t *inc, int32_t *inputL,
                     int32_t *inputR) {
  if (nIn <= nOut)
    return -1;
  inputL[0] = 0;
  inputR[0] = inc[0];
  for (int i = 0; i < nOut - 1; i++) {
    inputL[i + 1] = inputL[i] + inc[i];
    inputR[i + 1] = inputR[i] + inc[i + 1];
  }
  return inputR[nOut - 1] == nIn ? 0 : -1;
}

/* gridRulesOverlappingNoMin (uniform regions, Regions.cu:528-653) and
 * gridRulesNonOverlapping (Regions.cu:158-336) over FractionalPoolingRegions:
 * outputL / outputR from the ticks as Regions.cu:49-56.  inL / inR hold the
 * regions of this sample, axis after axis (d * nOut ints each). */
static void fmp_rules(const vgrid *in, vgrid *out, int d, int nIn, int nOut,
                      int s, const int32_t *inL, const int32_t *inR,
                      int uniform, int64_t *nSites, orc_ivec *rules) {
  int sd = orc_ipow(s, d);
  int32_t *outL = (int32_t *)malloc(sizeof(int32_t) * 2 * d * nIn);
  int32_t *outR = outL + (size_t)d * nIn;
  for (int a = 0; a < d; ++a) {
    for (int i = 0; i < nIn; ++i) {
      outL[a * nIn + i] = nOut;
      outR[a * nIn + i] = 0;
    }
    for (int j = 0; j < nOut; ++j)
      for (int i = inL[a * nOut + j]; i < inR[a * nOut + j]; ++i) {
        if (j < outL[a * nIn + i])
          outL[a * nIn + i] = j;
        if (j + 1 > outR[a * nIn + i])
          outR[a * nIn + i] = j + 1;
      }
  }
  vg_resize(out, orc_ipow(nOut, d));
  for (int64_t key = 0; key < in->len; ++key) {
    if (in->vec[key] == VH_EMPTY)
      continue;
    int i[4], lo[4], hi[4], j[4];
    decode(key, nIn, d, i);
    for (int a = 0; a < d; ++a) {
      lo[a] = outL[a * nIn + i[a]];
      hi[a] = outR[a * nIn + i[a]];
      j[a] = lo[a];
    }
    if (!box_nonempty(lo, hi, d))
      continue;
    do {
      int64_t outKey = encode(j, nOut, d);
      int off = 0;
      for (int a = 0; a < d; ++a)
        off = off * s + (i[a] - inL[a * nOut + j[a]]);
      const int32_t *f = vg_find(out, outKey);
      if (!f) {
        int32_t *slot = vg_at(out, outKey);
        *slot = (int32_t)((*nSites)++);
        if (uniform) {
          iv_resize(rules, *nSites * sd, in->backgroundCol);
        } else { /* -1, then the background row inside the region's extent */
          iv_resize(rules, *nSites * sd, -1);
          int ii[4] = {0, 0, 0, 0}, zero[4] = {0, 0, 0, 0}, ext[4];
          for (int a = 0; a < d; ++a)
            ext[a] = inR[a * nOut + j[a]] - inL[a * nOut + j[a]];
          do {
            int k = 0;
            for (int a = 0; a < d; ++a)
              k = k * s + ii[a];
            rules->d[(*nSites - 1) * sd + k] = in->backgroundCol;
          } while (odo_next(ii, zero, ext, d));
        }
        f = slot;
      }
      rules->d[(int64_t)*f * sd + off] = in->vec[key];
    } while (odo_next(j, lo, hi, d));
  }
  free(outL);
  background_row(in, out, orc_ipow(nOut, d), sd, nSites, rules);
}

/* one rule book for the batch; inputL / inputR: batch * dimension * nOut ints
 * (sample-major, then axis), as the layers draw new regions for every sample
 * (MaxPoolingLayer.cu:181-186) */
int64_t orc_rules_fmp(const orc_grids *in, orc_grids *out, int dimension,
                      int nIn, int nOut, int poolSize, const int32_t *inputL,
                      const int32_t *inputR, int uniform, orc_ivec *rules) {
  if (in->batch != out->batch || dimension < 1 || dimension > 3)
    return -1;
  reset_out(out);
  rules->n = 0;
  int64_t nSites = 0;
  for (int item = 0; item < in->batch; ++item) {
    const int32_t *l = inputL + (size_t)item * dimension * nOut;
    const int32_t *r = inputR + (size_t)item * dimension * nOut;
    fmp_rules(&in->g[item], &out->g[item], dimension, nIn, nOut, poolSize, l,
              r, uniform, &nSites, rules);
  }
  return nSites;
}

int64_t orc_rules_square(const orc_grids *in, orc_grids *out, int dimension,
                         int nIn, int nOut, int size, int stride,
                         int minActive, orc_ivec *rules) {
  if (dimension < 1 || dimension > 3 || in->batch != out->batch)
    return -1;
  if (nIn != size + (nOut - 1) * stride) /* Regions.cu:17 */
    return -1;
  if (minActive == 0 || minActive < -1)
    return -1; /* the dispatcher runs no generator for these */
  reset_out(out);
  rules->n = 0;
  int64_t nSites = 0;
  for (int item = 0; item < in->batch; ++item) {
    const vgrid *gi = &in->g[item];
    vgrid *go = &out->g[item];
    if (minActive == -1) {
      if (sq_valid(gi, go, dimension, nIn, nOut, size, stride, &nSites, rules))
        return -1;
    } else if (minActive == 1)
      sq_nomin(gi, go, dimension, nIn, nOut, size, stride, &nSites, rules);
    else
      sq_min(gi, go, dimension, nIn, nOut, size, stride, minActive, &nSites,
             rules);
  }
  return nSites;
}

/* gridRulesNoMin (triangular), Regions.cu:834-970 */
static void tri_nomin(const vgrid *in, vgrid *out, int d, int nIn, int nOut,
                      int s, int stride, const int32_t *ord, int S,
                      int64_t *nSites, orc_ivec *rules) {
  vg_resize(out, orc_triangle_size(nOut, d)); /* Regions.cu:845-847 */
  for (int64_t key = 0; key < in->len; ++key) {
    if (in->vec[key] == VH_EMPTY)
      continue;
    int i[4], lo[4], hi[4], j[4];
    decode(key, nIn, d, i);
    for (int a = 0; a < d; ++a) {
      lo[a] = orc_sq_outputL(s, stride, i[a]); /* same formulas, :828-832 */
      hi[a] = orc_sq_outputR(s, stride, nOut, i[a]);
      j[a] = lo[a];
    }
    if (!box_nonempty(lo, hi, d))
      continue;
    do {
      int sum = 0;
      for (int a = 0; a < d; ++a)
        sum += j[a];
      if (sum >= nOut)
        continue;
      int64_t outKey = encode(j, nOut, d);
      const int32_t *f = vg_find(out, outKey);
      if (!f) {
        int32_t *slot = vg_at(out, outKey);
        *slot = (int32_t)((*nSites)++);
        iv_resize(rules, *nSites * S, in->backgroundCol);
        f = slot;
      }
      int cube = 0;
      for (int a = 0; a < d; ++a)
        cube = cube * s + (i[a] - j[a] * stride);
      int off = ord[cube];
      if (off > -1)
        rules->d[(int64_t)*f * S + off] = in->vec[key];
    } while (odo_next(j, lo, hi, d));
  }
  background_row(in, out, orc_triangle_size(nOut, d), S, nSites, rules);
}

/* enumerate the in-triangle offsets of a window in the order of
 * Regions.cu:1025-1027,1068-1070: ii[a] < s - sum(ii[0..a-1]) */
static int tri_next(int *ii, int s, int d) {
  for (int a = d - 1; a >= 0; --a) {
    int before = 0;
    for (int b = 0; b < a; ++b)
      before += ii[b];
    if (++ii[a] < s - before)
      return 1;
    ii[a] = 0;
  }
  return 0;
}

/* gridRulesMin (triangular), Regions.cu:972-1164 */
static void tri_min(const vgrid *in, vgrid *out, int d, int nIn, int nOut,
                    int s, int stride, int S, int minActive, int64_t *nSites,
                    orc_ivec *rules) {
  vg_resize(out, orc_triangle_size(nOut, d));
  for (int64_t key = 0; key < in->len; ++key) {
    if (in->vec[key] == VH_EMPTY)
      continue;
    int i[4], lo[4], hi[4], j[4];
    decode(key, nIn, d, i);
    for (int a = 0; a < d; ++a) {
      lo[a] = orc_sq_outputL(s, stride, i[a]);
      hi[a] = orc_sq_outputR(s, stride, nOut, i[a]);
      j[a] = lo[a];
    }
    if (!box_nonempty(lo, hi, d))
      continue;
    do {
      int sum = 0;
      for (int a = 0; a < d; ++a)
        sum += j[a];
      if (sum >= nOut)
        continue;
      int64_t outKey = encode(j, nOut, d);
      if (vg_find(out, outKey))
        continue;
      int active = 0;
      int ii[4] = {0, 0, 0, 0}, c[4];
      do {
        for (int a = 0; a < d; ++a)
          c[a] = j[a] * stride + ii[a];
        const int32_t *f = vg_find(in, encode(c, nIn, d));
        if (!f)
          iv_push(rules, in->backgroundCol);
        else {
          iv_push(rules, *f);
          active++;
        }
      } while (tri_next(ii, s, d));
      if (active >= minActive) {
        *vg_at(out, outKey) = (int32_t)((*nSites)++);
      } else {
        *vg_at(out, outKey) = -2;
        iv_resize(rules, *nSites * S, 0);
      }
    } while (odo_next(j, lo, hi, d));
  }
  for (int64_t k = 0; k < out->len; ++k)
    if (out->vec[k] == -2) {
      out->vec[k] = VH_EMPTY;
      out->count--;
    }
  background_row(in, out, orc_triangle_size(nOut, d), S, nSites, rules);
}

int64_t orc_rules_triangular(const orc_grids *in, orc_grids *out,
                             int dimension, int nIn, int nOut, int size,
                             int stride, int minActive, orc_ivec *rules) {
  if (dimension < 1 || dimension > 3 || in->batch != out->batch)
    return -1;
  if (nIn != size + (nOut - 1) * stride) /* Regions.cu:823 */
    return -1;
  int32_t ord[4096];
  if (orc_ipow(size, dimension) > 4096)
    return -1;
  int S = orc_tri_ord(size, dimension, ord);
  reset_out(out);
  rules->n = 0;
  int64_t nSites = 0;
  for (int item = 0; item < in->batch; ++item) {
    if (minActive == 1)
      tri_nomin(&in->g[item], &out->g[item], dimension, nIn, nOut, size,
                stride, ord, S, &nSites, rules);
    else
      tri_min(&in->g[item], &out->g[item], dimension, nIn, nOut, size, stride,
              S, minActive, &nSites, rules);
  }
  return nSites;
}

int64_t orc_rules_terminal(const orc_grids *in, orc_grids *out,
                           orc_ivec *rules) {
  if (in->batch != out->batch)
    return -1;
  reset_out(out);
  rules->n = 0;
  int64_t S = 1; /* TerminalPoolingLayer.cu:90-92 */
  for (int i = 0; i < in->batch; ++i)
    if (in->g[i].count > S)
      S = in->g[i].count;
  int64_t nSites = 0;
  for (int item = 0; item < in->batch; ++item) {
    const vgrid *gi = &in->g[item];
    if (gi->count == 0) {
      iv_push(rules, gi->backgroundCol);
    } else {
      for (int64_t k = 0; k < gi->len; ++k)
        if (gi->vec[k] != VH_EMPTY)
          iv_push(rules, gi->vec[k]);
    }
    *vg_at(&out->g[item], 0) = (int32_t)(nSites++);
    iv_resize(rules, S * nSites, -1);
  }
  return S;
}

/* ---------- numeric layers ---------- */

void orc_gather_rows(const float *in, float *out, const int32_t *rules,
                     int64_t count, int nIn) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t c = 0; c < count; ++c)
    memcpy(out + c * nIn, in + (int64_t)rules[c] * nIn,
           (size_t)nIn * sizeof(float));
}

enum { A_NOSIGMOID, A_RELU, A_VLEAKYRELU, A_LEAKYRELU, A_TANH, A_SOFTMAX,
       A_PRELU, A_SIGMOID }; /* types.h:11-20 */

static float activate(float v, int act, float slope) {
  switch (act) {
  case A_RELU:
    return v > 0 ? v : 0;
  case A_VLEAKYRELU:
  case A_LEAKYRELU:
  case A_PRELU:
    return v > 0 ? v : v * slope;
  case A_TANH: /* SigmoidLayer.cu:80-85 */
    return tanhf(v);
  case A_SIGMOID: /* SigmoidLayer.cu:43-48 */
    return 1.0f / (1.0f + expf(-v));
  default:
    return v;
  }
}
static float act_slope(int act) {
  /* SigmoidLayer.cu:204-213: the literals 0.01 and 0.333 reach a float
   * parameter */
  if (act == A_LEAKYRELU)
    return (float)0.01;
  if (act == A_VLEAKYRELU)
    return (float)0.333;
  return 0.f;
}

void orc_nin_forward(const float *A, const float *W, const float *B,
                     const float *prelu, float *out, int64_t M, int K, int N,
                     float p, int act) {
  float slope0 = act_slope(act);
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float *o = out + m * N;
    for (int n = 0; n < N; ++n)
      o[n] = 0.f;
    const float *a = A + m * K;
    for (int k = 0; k < K; ++k) {
      float av = a[k];
      const float *w = W + (int64_t)k * N;
      for (int n = 0; n < N; ++n)
        o[n] += av * w[n];
    }
    for (int n = 0; n < N; ++n) {
      float v = p * o[n] + p * B[n];
      o[n] = activate(v, act, act == A_PRELU ? prelu[n] : slope0);
    }
  }
  if (act == A_SOFTMAX)
    orc_softmax_rows(out, out, M, N);
}

void orc_nin_forward_f64(const float *A, const float *W, const float *B,
                         const float *prelu, double *out, int64_t M, int K,
                         int N, float p, int act) {
  double slope0 = act_slope(act);
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    double *o = out + m * N;
    for (int n = 0; n < N; ++n)
      o[n] = 0.0;
    for (int k = 0; k < K; ++k) {
      double av = A[m * K + k];
      const float *w = W + (int64_t)k * N;
      for (int n = 0; n < N; ++n)
        o[n] += av * (double)w[n];
    }
    for (int n = 0; n < N; ++n) {
      double v = (double)p * (o[n] + (double)B[n]);
      double sl = act == A_PRELU ? (double)prelu[n] : slope0;
      if (act == A_RELU)
        v = v > 0 ? v : 0;
      else if (act == A_LEAKYRELU || act == A_VLEAKYRELU || act == A_PRELU)
        v = v > 0 ? v : v * sl;
      else if (act == A_TANH)
        v = tanh(v);
      else if (act == A_SIGMOID)
        v = 1.0 / (1.0 + exp(-v));
      o[n] = v;
    }
    if (act == A_SOFTMAX) {
      double mx = -10000.0, acc = 0;
      for (int n = 0; n < N; ++n)
        if (o[n] > mx)
          mx = o[n];
      for (int n = 0; n < N; ++n) {
        o[n] = exp(o[n] - mx);
        acc += o[n];
      }
      for (int n = 0; n < N; ++n)
        o[n] /= acc;
    }
  }
}

void orc_softmax_rows(const float *in, float *out, int64_t M, int N) {
  for (int64_t i = 0; i < M; ++i) {
    float acc = 0.0f;
    float mx = -10000.0f;
    for (int k = 0; k < N; ++k)
      if (in[i * N + k] > mx)
        mx = in[i * N + k];
    for (int k = 0; k < N; ++k) {
      out[i * N + k] = expf(in[i * N + k] - mx);
      acc += out[i * N + k];
    }
    for (int k = 0; k < N; ++k)
      out[i * N + k] /= acc;
  }
}

void orc_maxpool(const float *in, float *out, const int32_t *rules,
                 int64_t nOutSites, int ps, int C, int32_t *choice) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t r = 0; r < nOutSites; ++r) {
    const int32_t *rr = rules + r * ps;
    for (int j = 0; j < C; ++j) {
      int none = 1;
      float t = 0.f;
      int32_t c = 0;
      for (int p = 0; p < ps; ++p) {
        if (rr[p] >= 0) {
          int32_t idx = rr[p] * C + j; /* 32-bit like the reference */
          float s = in[(int64_t)rr[p] * C + j];
          if (none || t < s) {
            none = 0;
            c = idx;
            t = s;
          }
        }
      }
      out[r * C + j] = t;
      choice[r * C + j] = c;
    }
  }
}

void orc_terminal_pool(const float *in, float *out, const int32_t *rules,
                       int64_t count, int S, int C) {
  for (int64_t b = 0; b < count; ++b)
    for (int j = 0; j < C; ++j) {
      float t = 0;
      int p = 0;
      for (; p < S && rules[b * S + p] >= 0; p++)
        t += in[(int64_t)rules[b * S + p] * C + j];
      out[b * C + j] = t / p;
    }
}

void orc_top_indices(const float *test, int n, int k, int32_t *indices) {
  float *q = (float *)calloc((size_t)k, sizeof(float));
  for (int i = 0; i < k; ++i)
    indices[i] = 0;
  q[0] = test[0];
  for (int i = 1; i < n; i++) {
    int j = i < k ? i : k;
    if (test[i] > q[j - 1]) {
      if (i >= k)
        --j;
      for (; j > 0 && test[i] > q[j - 1]; --j) {
        q[j] = q[j - 1];
        indices[j] = indices[j - 1];
      }
    }
    if (j < k) {
      q[j] = test[i];
      indices[j] = i;
    }
  }
  free(q);
}

int orc_softmax_classifier(const float *probs, const int32_t *labels,
                           int batch, int nClasses, int nTop,
                           int32_t *predictions, float *nll) {
  int mistakes = batch;
  for (int i = 0; i < batch; ++i)
    orc_top_indices(probs + (int64_t)i * nClasses, nClasses, nTop,
                    predictions + (int64_t)i * nTop);
  for (int i = 0; i < batch; ++i) {
    double pr = probs[(int64_t)i * nClasses + labels[i]];
    *nll -= (float)log(pr > 1.0e-15 ? pr : 1.0e-15);
    for (int j = 0; j < nTop; ++j)
      if (predictions[(int64_t)i * nTop + j] == labels[i])
        mistakes--;
  }
  return mistakes;
}

/* ---------- backward pass (training) ---------- */

/* dDerivativeOfCostWRTpreSoftmaxTopLevelWeights, SoftmaxClassifier.cu:7-14 */
void orc_softmax_grad(const float *probs, const int32_t *labels, float *delta,
                      int64_t batch, int N) {
  for (int64_t k = 0; k < batch; ++k)
    for (int i = 0; i < N; ++i)
      delta[k * N + i] = probs[k * N + i] - (i == labels[k]);
}

/* applySigmoidBackProp in place as NetworkInNetworkLayer::backwards calls it
 * (NetworkInNetworkLayer.cu:222; kernels SigmoidLayer.cu:23-177), or
 * PReLUBackprop (NetworkInNetworkPReLULayer.cu:25-47), followed by columnSum
 * (NetworkInNetworkLayer.cu:84-105).  The sums are taken in double and
 * rounded once (the reference's atomics fix no order). */
void orc_activation_backward(const float *out, float *delta, int64_t M, int N,
                             int act, const float *prelu, float *db,
                             float *dprelu) {
  double *s = (double *)calloc((size_t)N, sizeof(double));
  double *t = (double *)calloc((size_t)N, sizeof(double));
  for (int64_t r = 0; r < M; ++r)
    for (int c = 0; c < N; ++c) {
      float b = out[r * N + c], d = delta[r * N + c];
      switch (act) {
      case A_RELU:
        d = b > 0 ? d : 0;
        break;
      case A_LEAKYRELU:
        d = b > 0 ? d : d * 0.01f;
        break;
      case A_VLEAKYRELU:
        d = b > 0 ? d : d * 0.333f;
        break;
      case A_TANH:
        d = d * (1 + b) * (1 - b);
        break;
      case A_SIGMOID:
        d = d * b * (1 - b);
        break;
      case A_PRELU:
        t[c] += d * (b > 0 ? 0 : b / prelu[c]);
        d = b > 0 ? d : d * prelu[c];
        break;
      default:
        break;
      }
      delta[r * N + c] = d;
      s[c] += d;
    }
  for (int c = 0; c < N; ++c) {
    db[c] = (float)s[c];
    if (act == A_PRELU)
      dprelu[c] = (float)t[c];
  }
  free(s);
  free(t);
}

/* d_rowMajorSGEMM_alphaAtB_betaC, alpha 1 beta 0 (utilities.cu:144-152):
 * dW[K x N] = A^T D, accumulated in double. */
void orc_sgemm_AtB(const float *A, const float *D, float *dW, int64_t M, int K,
                   int N) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int k = 0; k < K; ++k) {
    double *acc = (double *)calloc((size_t)N, sizeof(double));
    for (int64_t m = 0; m < M; ++m) {
      double a = A[m * K + k];
      const float *d = D + m * N;
      for (int n = 0; n < N; ++n)
        acc[n] += a * (double)d[n];
    }
    for (int n = 0; n < N; ++n)
      dW[(int64_t)k * N + n] = (float)acc[n];
    free(acc);
  }
}

/* d_rowMajorSGEMM_alphaABt_betaC, alpha 1 beta 0 (utilities.cu:153-161):
 * dA[M x K] = D W^T, accumulated in double. */
void orc_sgemm_ABt(const float *D, const float *W, float *dA, int64_t M, int N,
                   int K) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t m = 0; m < M; ++m)
    for (int k = 0; k < K; ++k) {
      double acc = 0;
      for (int n = 0; n < N; ++n)
        acc += (double)D[m * N + n] * (double)W[(int64_t)k * N + n];
      dA[m * K + k] = (float)acc;
    }
}

/* dGradientDescent / dGradientDescentKeepPositive
 * (NetworkInNetworkLayer.cu:27-41, NetworkInNetworkPReLULayer.cu:68-83) */
void orc_nag_update(const float *delta, float *mom, float *wts, int64_t n,
                    float learningRate, float momentum, int keepPositive) {
  for (int64_t j = 0; j < n; ++j) {
    float w = wts[j], m = mom[j], d = delta[j];
    w -= m * momentum;
    m = momentum * m - learningRate * (1 - momentum) * d;
    w += m * (1 + momentum);
    if (keepPositive)
      w = (w > 0.001f) ? w : 0.001f;
    wts[j] = w;
    mom[j] = m;
  }
}

/* dPropBackwardFromMatrixMultiplyOutput (ConvolutionalLayer.cu:42-63); din is
 * zeroed by the caller.  Summed in entry order. */
void orc_gather_rows_backward(float *din, const float *dconv,
                              const int32_t *rules, int64_t count, int nIn) {
  for (int64_t c = 0; c < count; ++c)
    if (rules[c] >= 0)
      for (int j = 0; j < nIn; ++j)
        din[(int64_t)rules[c] * nIn + j] += dconv[c * nIn + j];
}

/* dMaxPoolBackProp (MaxPoolingLayer.cu:74-82) */
void orc_maxpool_backward(float *din, const float *dout, int64_t count, int C,
                          const int32_t *choice) {
  for (int64_t j = 0; j < count * C; ++j)
    din[choice[j]] += dout[j];
}

/* dTerminalPoolBackProp (TerminalPoolingLayer.cu:48-62): assignment, not sum */
void orc_terminal_pool_backward(float *din, const float *dout,
                                const int32_t *rules, int64_t count, int C,
                                int S) {
  for (int64_t b = 0; b < count; ++b) {
    int maxP = 0;
    while (maxP < S && rules[b * S + maxP] >= 0)
      ++maxP;
    for (int j = 0; j < C; ++j) {
      float t = dout[b * C + j] / maxP;
      for (int p = 0; p < maxP; ++p)
        din[(int64_t)rules[b * S + p] * C + j] = t;
    }
  }
}
