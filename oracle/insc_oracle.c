/*
 * CPU oracle for the sparse-convolution inference path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the algorithms of the
 * reference's CPU path so that the HIP library can be checked against them.  Nothing in
 * the shipped library links, loads or calls it; only tests/, the smoke check and the
 * cpu_baseline leg of the benchmark do.
 *
 * Every function names the reference source it follows (paths relative to the reference
 * checkout, sparseconvnet/SCN/...).  Where the reference's CPU and GPU variants disagree
 * the choice is stated at the function.
 *
 * Parity status: the reference ships no tests, fixtures or golden vectors for this path and
 * cannot be built here, so each function below is pinned by tests/test_oracle_*.py against
 * closed forms, brute force and library routines (torch conv3d / conv_transpose3d /
 * batch_norm, numpy unique).  None is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef int32_t Int;

/* Arithmetic type of the feature operators.  The default build (float) is the restatement of
 * the reference's fp32 CPU path.  A second build with -DORC_REAL=double (liborc64.so) runs the
 * same operators, in the same order, in double precision: the yardstick that says how far each
 * fp32 implementation - the reference's order of operations as restated here, and the HIP
 * kernels' - is from the exact result, so that a tolerance can be stated per element. */
#ifndef ORC_REAL
#define ORC_REAL float
#endif
typedef ORC_REAL real;
#define REAL_POW(x, y) (sizeof(real) == sizeof(float) ? (real)powf((float)(x), (float)(y)) : (real)pow((double)(x), (double)(y)))
int orc_real_bytes(void) { return (int)sizeof(real); }

/* ------------------------------------------------------------------------------------
 * Point -> site map.  Stands in for google::dense_hash_map<Point<4>, Int, IntArrayHash>
 * (Metadata/Metadata.h:95-106); the hash is the reference's FNV variant
 * (Metadata/32bits.h:79-88): hash = 16777619; for x in p: hash *= 2166136261; hash ^= x.
 * The point carries (x, y, z, batch); the reference keeps one map per batch sample
 * (Metadata.h:104 SparseGrids), which is the same relation.
 * ------------------------------------------------------------------------------------ */
typedef struct {
  Int *keys; /* [cap][4] */
  Int *vals; /* [cap], -1 = empty */
  int64_t cap, n;
} PMap;

static uint32_t fnv4(const Int *p) {
  uint32_t h = 16777619u;
  for (int i = 0; i < 4; i++) {
    h *= 2166136261u;
    h ^= (uint32_t)p[i];
  }
  return h;
}

static void pmap_init(PMap *m, int64_t expect) {
  int64_t cap = 64;
  while (cap < 2 * expect + 2) cap <<= 1;
  m->cap = cap;
  m->n = 0;
  m->keys = (Int *)malloc(sizeof(Int) * 4 * cap);
  m->vals = (Int *)malloc(sizeof(Int) * cap);
  for (int64_t i = 0; i < cap; i++) m->vals[i] = -1;
}
static void pmap_free(PMap *m) {
  free(m->keys);
  free(m->vals);
}
static Int pmap_find(const PMap *m, const Int *p) {
  int64_t s = fnv4(p) & (m->cap - 1);
  while (m->vals[s] >= 0) {
    const Int *k = m->keys + 4 * s;
    if (k[0] == p[0] && k[1] == p[1] && k[2] == p[2] && k[3] == p[3]) return m->vals[s];
    s = (s + 1) & (m->cap - 1);
  }
  return -1;
}
/* insert if absent with value v; returns the stored value */
static Int pmap_insert(PMap *m, const Int *p, Int v) {
  int64_t s = fnv4(p) & (m->cap - 1);
  while (m->vals[s] >= 0) {
    const Int *k = m->keys + 4 * s;
    if (k[0] == p[0] && k[1] == p[1] && k[2] == p[2] && k[3] == p[3]) return m->vals[s];
    s = (s + 1) & (m->cap - 1);
  }
  memcpy(m->keys + 4 * s, p, sizeof(Int) * 4);
  m->vals[s] = v;
  m->n++;
  return v;
}

/* ------------------------------------------------------------------------------------
 * Input layer rules, modes 1-4 site numbering.
 * Follows Metadata/IOLayersRules.h:62-96 (inputLayerRules): walk the input rows in order;
 * the first row at a location creates site nActive++; every row is appended to its
 * site's list.  Returns the number of sites; site_of_point[p] is the row's site,
 * site_coords[site] = (x,y,z,b) of the site, count[site] = rows at that site.
 * ------------------------------------------------------------------------------------ */
int64_t orc_grid_build(const Int *coords4, int64_t P, Int *site_of_point, Int *site_coords4, Int *count) {
  PMap m;
  pmap_init(&m, P);
  Int n = 0;
  for (int64_t p = 0; p < P; p++) {
    const Int *c = coords4 + 4 * p;
    Int s = pmap_insert(&m, c, n);
    if (s == n) {
      memcpy(site_coords4 + 4 * (int64_t)n, c, sizeof(Int) * 4);
      if (count) count[n] = 0;
      n++;
    }
    site_of_point[p] = s;
    if (count) count[s]++;
  }
  pmap_free(&m);
  return n;
}

/* Query a set of sites: out[q] = site id or -1.  (SparseGrid::mp.find, Metadata.h:95-103;
 * the GPU variant returns 0xFFFFFFFF for a miss, CUDA/CUDPPWrapper.cu:144-160.) */
void orc_grid_query(const Int *site_coords4, int64_t N, const Int *q4, int64_t Q, Int *out) {
  PMap m;
  pmap_init(&m, N);
  for (int64_t i = 0; i < N; i++) pmap_insert(&m, site_coords4 + 4 * i, (Int)i);
  for (int64_t q = 0; q < Q; q++) out[q] = pmap_find(&m, q4 + 4 * q);
  pmap_free(&m);
}

/* ------------------------------------------------------------------------------------
 * Input layer forward, modes 3 (sum) and 4 (mean).
 * Follows CPU/IOLayers.cpp:11-29 (InputLayer_ForwardPass): output zeroed, then for each
 * site, for its rows in input order: out += multiplier * in, multiplier = 1/nActive for
 * mode 4.  Written without the rule table: rows are visited in input order, which gives
 * each site the same order of additions.
 * ------------------------------------------------------------------------------------ */
void orc_input_forward(const real *in, int64_t P, int C, const Int *site_of_point, const Int *count, int64_t N,
                       int average, real *out) {
  memset(out, 0, sizeof(real) * N * C);
  for (int64_t p = 0; p < P; p++) {
    Int s = site_of_point[p];
    real mult = (average && count[s] > 0) ? 1.0f / (real)count[s] : 1.0f;
    for (int c = 0; c < C; c++) out[(int64_t)s * C + c] += mult * in[p * C + c];
  }
}

/* Output layer forward.  Follows CPU/IOLayers.cpp:99-115 (cpu_OutputLayer_updateOutput ->
 * InputLayer_BackwardPass with average=false): every original input row receives its
 * site's feature row, multiplier 1. */
void orc_output_forward(const real *feats, int C, const Int *site_of_point, int64_t P, real *out) {
  for (int64_t p = 0; p < P; p++)
    memcpy(out + p * C, feats + (int64_t)site_of_point[p] * C, sizeof(real) * C);
}

/* ------------------------------------------------------------------------------------
 * Submanifold 3x3x3 rulebook.
 * Follows Metadata/SubmanifoldConvolutionRules.h:114-150 (SubmanifoldConvolution_SgToRules,
 * dilated_rate 1): for every output site and every point of its 3^3 input region, if the
 * point is active emit (input site, output site) into rules[offset].
 * Offset numbering: the reference's GPU builder and upstream SCN enumerate the region
 * x-outermost, z-innermost (CUDA/SubmanifoldRules_cuda.cu:45-77; RectangularRegions.h:78-93),
 * offset = (dx+1)*9 + (dy+1)*3 + (dz+1), input = output + (dx,dy,dz).  INS-Conv's rewritten
 * CPU generator (SubmanifoldConvolutionRules.h:39-52) enumerates z-outermost instead; the
 * two differ by the permutation k <-> (k%3)*9 + ((k/3)%3)*3 + k/9.  zmajor=0 selects the
 * GPU/upstream order (the one the weights of upstream SCN are trained with), zmajor=1 the
 * CPU rewrite's.
 * Output: nbr[o*27+k] = input site or -1; counts[k]; pairs = 27 lists back to back,
 * each (in,out) in ascending out order.  Returns total pairs.
 * ------------------------------------------------------------------------------------ */
int64_t orc_ssc_rules(const Int *site_coords4, int64_t N, int zmajor, Int *nbr, Int *counts, Int *pairs) {
  PMap m;
  pmap_init(&m, N);
  for (int64_t i = 0; i < N; i++) pmap_insert(&m, site_coords4 + 4 * i, (Int)i);
  for (int k = 0; k < 27; k++) counts[k] = 0;
  for (int64_t o = 0; o < N; o++) {
    const Int *c = site_coords4 + 4 * o;
    for (int k = 0; k < 27; k++) {
      int a = k / 9 - 1, b = (k / 3) % 3 - 1, d = k % 3 - 1;
      Int q[4];
      if (zmajor) {
        q[0] = c[0] + d; q[1] = c[1] + b; q[2] = c[2] + a;
      } else {
        q[0] = c[0] + a; q[1] = c[1] + b; q[2] = c[2] + d;
      }
      q[3] = c[3];
      Int i = pmap_find(&m, q);
      nbr[o * 27 + k] = i;
      if (i >= 0) counts[k]++;
    }
  }
  int64_t total = 0;
  if (pairs) {
    int64_t w = 0;
    for (int k = 0; k < 27; k++)
      for (int64_t o = 0; o < N; o++)
        if (nbr[o * 27 + k] >= 0) {
          pairs[2 * w] = nbr[o * 27 + k];
          pairs[2 * w + 1] = (Int)o;
          w++;
        }
    total = w;
  } else {
    for (int k = 0; k < 27; k++) total += counts[k];
  }
  pmap_free(&m);
  return total;
}

/* ------------------------------------------------------------------------------------
 * Size-2 stride-2 convolution rulebook and output grid.
 * Follows Metadata/ConvolutionRules.h:95-118 (Convolution_InputSgToRulesAndOutputSg) with
 * RectangularRegions.h:117-141: for size = stride = 2 the output region of an input point
 * is the single point in/2, created on first use (outputGrid.ctr++), and
 * rulesOffset = inRegion.offset(in) = (x&1)*4 + (y&1)*2 + (z&1)  (last dimension fastest,
 * RectangularRegions.h:52-60; the GPU kernel computes the same number,
 * CUDA/SubmanifoldRules_cuda.cu:760-766).  Input sites are visited in id order.
 * Output: parent[i] = coarse site of fine site i, offset[i] in 0..7, coarse_coords4.
 * Returns the number of coarse sites.
 * ------------------------------------------------------------------------------------ */
int64_t orc_down2_rules(const Int *fine_coords4, int64_t Nf, Int *parent, Int *offset, Int *coarse_coords4) {
  PMap m;
  pmap_init(&m, Nf);
  Int n = 0;
  for (int64_t i = 0; i < Nf; i++) {
    const Int *c = fine_coords4 + 4 * i;
    Int q[4] = {c[0] / 2, c[1] / 2, c[2] / 2, c[3]};
    Int s = pmap_insert(&m, q, n);
    if (s == n) {
      memcpy(coarse_coords4 + 4 * (int64_t)n, q, sizeof(Int) * 4);
      n++;
    }
    parent[i] = s;
    offset[i] = (c[0] - 2 * q[0]) * 4 + (c[1] - 2 * q[1]) * 2 + (c[2] - 2 * q[2]);
  }
  pmap_free(&m);
  return n;
}

/* ------------------------------------------------------------------------------------
 * Rulebook convolution forward (submanifold, strided, and deconvolution).
 * Follows CPU/Convolution.cpp:36-71,115-149 and CPU/Deconvolution.cpp:8-44: output =
 * bias (or zero); for each offset k with nRules>0: input_rows = rule_index_select(in),
 * output_rows = mm(input_rows, W[k]), rule_index_add_(out, output_rows).  The reference
 * parallelises the row loops with OpenMP (Convolution.cpp:15,26), as here.
 * pairs: K lists back to back, list k holds counts[k] pairs (a, b).  swap=0: gather rows
 * a, add into rows b (conv / submanifold); swap=1: gather rows b, add into rows a
 * (deconvolution, Deconvolution.cpp:37-40).  Returns multiply-adds (the "flops" the
 * reference returns).  Within one offset every destination row occurs at most once, so
 * the parallel add is race-free (the reference relies on the same fact).
 * ------------------------------------------------------------------------------------ */
double orc_conv_forward(const real *in, real *out, int64_t n_out, const real *W, const real *bias, const Int *pairs,
                        const Int *counts, int K, int Cin, int Cout, int swap) {
  for (int64_t r = 0; r < n_out; r++)
    for (int c = 0; c < Cout; c++) out[r * Cout + c] = bias ? bias[c] : 0.0f;
  double flops = 0;
  int64_t base = 0;
  for (int k = 0; k < K; k++) {
    int64_t nr = counts[k];
    if (nr) {
      flops += (double)nr * Cin * Cout;
      const Int *r = pairs + 2 * base;
      const real *w = W + (int64_t)k * Cin * Cout;
      real *rows = (real *)malloc(sizeof(real) * nr * Cout);
#pragma omp parallel for schedule(static)
      for (int64_t i = 0; i < nr; i++) {
        const real *x = in + (int64_t)r[2 * i + (swap ? 1 : 0)] * Cin;
        real *y = rows + i * Cout;
        for (int c = 0; c < Cout; c++) y[c] = 0.0f;
        for (int ci = 0; ci < Cin; ci++) {
          real xv = x[ci];
          const real *wr = w + (int64_t)ci * Cout;
          for (int c = 0; c < Cout; c++) y[c] += xv * wr[c];
        }
      }
#pragma omp parallel for schedule(static)
      for (int64_t i = 0; i < nr; i++) {
        real *t = out + (int64_t)r[2 * i + (swap ? 0 : 1)] * Cout;
        const real *s = rows + i * Cout;
        for (int c = 0; c < Cout; c++) t[c] += s[c];
      }
      free(rows);
    }
    base += nr;
  }
  return flops;
}

/* ------------------------------------------------------------------------------------
 * Batch normalisation, inference, with leaky ReLU.
 * Follows CPU/BatchNormalization.cpp:41-61 (train == false branch):
 * invstd = powf(var + eps, -0.5); w = invstd * gamma; b = -mean * w + beta;
 * y = x*w + b; y *= (y > 0) ? 1 : leakiness.
 * ------------------------------------------------------------------------------------ */
void orc_bn_forward(const real *in, real *out, int64_t N, int C, const real *mean, const real *var,
                    const real *gamma, const real *beta, float eps, float leakiness) {
  real *w = (real *)malloc(sizeof(real) * C), *b = (real *)malloc(sizeof(real) * C);
  for (int c = 0; c < C; c++) {
    real invstd = REAL_POW(var[c] + (real)eps, (real)-0.5);
    w[c] = invstd * (gamma ? gamma[c] : 1.0f);
    b[c] = -mean[c] * w[c] + (beta ? beta[c] : 0.0f);
  }
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N; r++)
    for (int c = 0; c < C; c++) {
      real o = in[r * C + c] * w[c] + b[c];
      real s = (o > 0) ? 1.0f : leakiness;
      out[r * C + c] = o * s;
    }
  free(w);
  free(b);
}

/* Network-in-network (1x1 linear).  Follows CPU/NetworkInNetwork.cpp:8-23:
 * out = bias (or zero); out.addmm_(in, W).  Returns multiply-adds. */
double orc_nin_forward(const real *in, real *out, int64_t N, const real *W, const real *bias, int Cin, int Cout) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N; r++) {
    real *y = out + r * Cout;
    for (int c = 0; c < Cout; c++) y[c] = bias ? bias[c] : 0.0f;
    for (int ci = 0; ci < Cin; ci++) {
      real xv = in[r * Cin + ci];
      const real *wr = W + (int64_t)ci * Cout;
      for (int c = 0; c < Cout; c++) y[c] += xv * wr[c];
    }
  }
  return (double)N * Cin * Cout;
}

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
