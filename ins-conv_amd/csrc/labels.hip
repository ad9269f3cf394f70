// Per-voxel label fusion: the step that follows the logits in the reference's online
// segmentation loop.  The reference keeps a CPU hash map voxel -> (label, confidence)
// (Result<dimension>, Metadata/resultHash.h:23-150) or voxel -> running logits (ResultOfWeight,
// resultHash.h:153-218) and walks it point by point on the host; here the map is a hash grid
// (voxel -> row) plus device arrays, and one call handles a frame's points.
//
// Order of application.  The reference applies the rows of a call one after the other
// (its second loop is an OpenMP loop over rows, so rows of ONE voxel in one call race there);
// here the rows of a voxel are applied in ascending row order, which is what its loop does
// when run by one thread.
#include <algorithm>

#include "common.h"
#include "grid.h"

struct insc_labels {
  insc_grid *grid = nullptr;
  int kind = 0;         // 0: (label, confidence) per voxel; 1: running scores per voxel
  int C = 0;            // kind 1: scores per voxel (fixed by the first update)
  float cap_conf = 0;   // kind 0: confidence ceiling
  int64_t cap = 0;      // rows of the arrays below
  int32_t *label = nullptr;  // [cap]
  float *conf = nullptr;     // [cap]
  float *scores = nullptr;   // [cap, C]
  int32_t *head = nullptr;   // [cap] per-voxel list head, -1 when idle
};

namespace insc {

__device__ __forceinline__ void row_max(const float *__restrict__ x, int C, int &arg, float &val) {
  arg = 0;
  val = x[0];
  for (int c = 1; c < C; c++)
    if (x[c] > val) {  // first maximum, as torch.max / torch.argmax
      val = x[c];
      arg = c;
    }
}

__global__ void labels_push_kernel(const int32_t *__restrict__ sop, int64_t P, int32_t *__restrict__ head,
                                   int32_t *__restrict__ next) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int s = sop[p];
  next[p] = (s >= 0) ? atomicExch(&head[s], (int)p) : -1;
}

// MODE 0: Result::set, 1: Result::update, 2: ResultOfWeight::update.  The row left at the head of
// a voxel's list applies the list in ascending row order and empties it.
template <int MODE>
__global__ void labels_apply_kernel(const float *__restrict__ scores_in, int64_t ld, int C,
                                    const int32_t *__restrict__ sop, int64_t P, int32_t *__restrict__ head,
                                    const int32_t *__restrict__ next, const int32_t *__restrict__ d_n,
                                    int32_t *__restrict__ label, float *__restrict__ conf,
                                    float *__restrict__ scores, float cap_conf) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int s = sop[p];
  if (s < 0 || head[s] != (int)p) return;
  bool exists = s < d_n[1];  // the voxel was in the table before this call
  int lab = exists ? label[s] : 0;
  float cf = exists ? conf[s] : 0.0f;
  int done = -1;
  for (;;) {
    int q = 0x7fffffff;
    for (int t = (int)p; t >= 0; t = next[t])
      if (t > done && t < q) q = t;
    if (q == 0x7fffffff) break;
    done = q;
    const float *x = scores_in + (int64_t)q * ld;
    if (MODE == 2) {
      float *dst = scores + (int64_t)s * C;
      for (int c = 0; c < C; c++) dst[c] = exists ? dst[c] * 0.5f + x[c] : x[c];
    } else {
      int val;
      float prob;
      row_max(x, C, val, prob);
      if (MODE == 0) {
        lab = val;
        cf = 0.0f;
      } else if (!exists) {
        lab = val;
        cf = prob;
      } else {
        if (lab == val)
          cf = fminf(cap_conf, cf + prob);
        else
          cf -= prob;
        if (cf < 0.0f) {
          lab = val;
          cf = -cf;
        }
      }
    }
    exists = true;
  }
  if (MODE != 2) {
    label[s] = lab;
    conf[s] = cf;
  }
  head[s] = -1;
}

__global__ void labels_lookup_kernel(const int32_t *__restrict__ site, int64_t Q, int kind, int C,
                                     const int32_t *__restrict__ label, const float *__restrict__ scores,
                                     int32_t *__restrict__ out) {
  int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= Q) return;
  const int s = site[q];
  int v = -1;
  if (s >= 0) {
    if (kind == 0) {
      v = label[s];
    } else {
      float m;
      row_max(scores + (int64_t)s * C, C, v, m);
    }
  }
  out[q] = v;
}

__global__ void labels_export_kernel(const int32_t *__restrict__ coords, const int32_t *__restrict__ d_n,
                                     int64_t n_upper, int kind, int C, const int32_t *__restrict__ label,
                                     const float *__restrict__ conf, const float *__restrict__ scores,
                                     int32_t *__restrict__ out4, float *__restrict__ out_conf) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= min((int64_t)*d_n, n_upper)) return;
  int4 c = reinterpret_cast<const int4 *>(coords)[i];
  if (kind == 0) {
    c.w = label[i];
    if (out_conf) out_conf[i] = conf[i];
  } else {
    float m;
    row_max(scores + i * C, C, c.w, m);
    if (out_conf) out_conf[i] = m;
  }
  reinterpret_cast<int4 *>(out4)[i] = c;
}

__global__ void labels_mark_kernel(const int32_t *__restrict__ site, int64_t M, int32_t *__restrict__ mark) {
  int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= M) return;
  const int s = site[q];
  if (s >= 0) mark[s] = 1;
}

// kept voxel i moves to row excl[i]; rows past the kept ones get a coordinate the insert skips
__global__ void labels_compact_kernel(const int32_t *__restrict__ coords, const int32_t *__restrict__ mark,
                                      const int32_t *__restrict__ excl, const int32_t *__restrict__ total,
                                      int64_t n, int C, const int32_t *__restrict__ label,
                                      const float *__restrict__ conf, const float *__restrict__ scores,
                                      int32_t *__restrict__ coords_out, int32_t *__restrict__ label_out,
                                      float *__restrict__ conf_out, float *__restrict__ scores_out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (i >= *total) reinterpret_cast<int4 *>(coords_out)[i] = make_int4(COORD_SKIP, 0, 0, 0);
  if (!mark[i]) return;
  const int j = excl[i];
  reinterpret_cast<int4 *>(coords_out)[j] = reinterpret_cast<const int4 *>(coords)[i];
  if (label) {
    label_out[j] = label[i];
    conf_out[j] = conf[i];
  }
  if (scores)
    for (int c = 0; c < C; c++) scores_out[(int64_t)j * C + c] = scores[i * C + c];
}

template <typename T>
static int regrow(T **p, size_t old_count, size_t new_count, hipStream_t s) {
  T *q = nullptr;
  INSC_HIP(hipMalloc((void **)&q, sizeof(T) * (new_count ? new_count : 1)));
  if (*p && old_count) INSC_HIP(hipMemcpyAsync(q, *p, sizeof(T) * old_count, hipMemcpyDeviceToDevice, s));
  INSC_HIP(hipStreamSynchronize(s));
  if (*p) INSC_HIP(hipFree(*p));
  *p = q;
  return INSC_OK;
}

static int labels_reserve(insc_labels *l, int64_t need, hipStream_t s) {
  if (need <= l->cap) return INSC_OK;
  const int64_t cap = std::max<int64_t>(std::max<int64_t>(need, l->cap * 2), 1024);
  int rc = insc_grid_reserve(l->grid, cap, (void *)s);
  if (rc) return rc;
  if (l->kind == 0) {
    if ((rc = regrow(&l->label, (size_t)l->cap, (size_t)cap, s))) return rc;
    if ((rc = regrow(&l->conf, (size_t)l->cap, (size_t)cap, s))) return rc;
  } else if (l->C > 0) {
    if ((rc = regrow(&l->scores, (size_t)l->cap * l->C, (size_t)cap * l->C, s))) return rc;
  }
  if ((rc = regrow(&l->head, (size_t)l->cap, (size_t)cap, s))) return rc;
  if ((rc = insc_fill_i32(l->head + l->cap, cap - l->cap, -1, (void *)s))) return rc;
  l->cap = cap;
  return INSC_OK;
}

static int labels_apply(insc_labels *l, int mode, const int32_t *d_coords4, const float *d_scores, int64_t ld,
                        int64_t P, int C, hipStream_t s, const char *who) {
  INSC_REQUIRE(l && P >= 0 && C >= 1 && ld >= C, INSC_ERR_ARG, "%s: bad arguments", who);
  INSC_REQUIRE(P == 0 || (d_coords4 && d_scores), INSC_ERR_ARG, "%s: null pointer", who);
  INSC_REQUIRE((mode == 2) == (l->kind == 1), INSC_ERR_STATE, "%s: wrong kind of label table", who);
  if (P == 0) return INSC_OK;
  int rc;
  if (l->kind == 1) {
    INSC_REQUIRE(l->C == 0 || l->C == C, INSC_ERR_ARG, "%s: %d scores per row, the table holds %d", who, C, l->C);
    if (l->C == 0) {  // first update fixes the width
      l->C = C;
      if ((rc = regrow(&l->scores, 0, (size_t)l->cap * C, s))) return rc;
    }
  }
  // the bound counts every row as a new voxel: refresh it before growing
  if (l->grid->n_upper + P > l->cap) {
    int64_t n = 0;
    if ((rc = insc_grid_size(l->grid, &n, (void *)s))) return rc;
    if ((rc = labels_reserve(l, n + P, s))) return rc;
  }
  void *ws;
  if ((rc = workspace(WS_LABELS, s, sizeof(int32_t) * 2 * (size_t)P + 256, &ws))) return rc;
  int32_t *sop = (int32_t *)ws, *next = sop + P;
  if ((rc = grid_insert_nosync(l->grid, d_coords4, P, sop, s))) return rc;
  const unsigned nb = grid_for(P, 256);
  hipLaunchKernelGGL(labels_push_kernel, dim3(nb), dim3(256), 0, s, sop, P, l->head, next);
  if (mode == 0)
    hipLaunchKernelGGL(labels_apply_kernel<0>, dim3(nb), dim3(256), 0, s, d_scores, ld, C, sop, P, l->head, next,
                       l->grid->d_n, l->label, l->conf, l->scores, l->cap_conf);
  else if (mode == 1)
    hipLaunchKernelGGL(labels_apply_kernel<1>, dim3(nb), dim3(256), 0, s, d_scores, ld, C, sop, P, l->head, next,
                       l->grid->d_n, l->label, l->conf, l->scores, l->cap_conf);
  else
    hipLaunchKernelGGL(labels_apply_kernel<2>, dim3(nb), dim3(256), 0, s, d_scores, ld, C, sop, P, l->head, next,
                       l->grid->d_n, l->label, l->conf, l->scores, l->cap_conf);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_labels_create(int64_t capacity_voxels, int kind, float maximum, insc_labels **out) {
  INSC_REQUIRE(out && (kind == 0 || kind == 1) && capacity_voxels >= 0, INSC_ERR_ARG, "insc_labels_create: bad arguments");
  insc_labels *l = new insc_labels();
  l->kind = kind;
  // the reference stores its `float maximum` argument in an int member (resultHash.h:25,30), so
  // the ceiling it applies is the argument truncated towards zero: 0.7, its default, acts as 0
  l->cap_conf = (float)(int)maximum;
  int rc = insc_grid_create(std::max<int64_t>(capacity_voxels, 1024), &l->grid);
  if (rc) {
    delete l;
    return rc;
  }
  rc = labels_reserve(l, std::max<int64_t>(capacity_voxels, 1024), nullptr);
  if (rc) {
    insc_grid_destroy(l->grid);
    delete l;
    return rc;
  }
  *out = l;
  return INSC_OK;
}

int insc_labels_destroy(insc_labels *l) {
  if (!l) return INSC_OK;
  (void)hipDeviceSynchronize();
  if (l->grid) insc_grid_destroy(l->grid);
  void *ps[] = {l->label, l->conf, l->scores, l->head};
  for (void *p : ps)
    if (p) (void)hipFree(p);
  delete l;
  return INSC_OK;
}

int insc_labels_clear(insc_labels *l, void *stream) {
  INSC_REQUIRE(l, INSC_ERR_ARG, "insc_labels_clear: null table");
  return insc_grid_clear(l->grid, stream);
}

int insc_labels_set(insc_labels *l, const int32_t *d_coords4, const float *d_scores, int64_t ld, int64_t P, int C,
                    void *stream) {
  return labels_apply(l, 0, d_coords4, d_scores, ld, P, C, (hipStream_t)stream, "insc_labels_set");
}

int insc_labels_update(insc_labels *l, const int32_t *d_coords4, const float *d_scores, int64_t ld, int64_t P, int C,
                       void *stream) {
  INSC_REQUIRE(l, INSC_ERR_ARG, "insc_labels_update: null table");
  return labels_apply(l, l->kind == 0 ? 1 : 2, d_coords4, d_scores, ld, P, C, (hipStream_t)stream,
                      "insc_labels_update");
}

int insc_labels_query(insc_labels *l, const int32_t *d_coords4, int64_t Q, int32_t *d_label, void *stream) {
  INSC_REQUIRE(l && Q >= 0 && (Q == 0 || (d_coords4 && d_label)), INSC_ERR_ARG, "insc_labels_query: bad arguments");
  if (Q == 0) return INSC_OK;
  hipStream_t s = (hipStream_t)stream;
  int rc = insc_grid_query(l->grid, d_coords4, Q, d_label, stream);  // sites first, replaced in place
  if (rc) return rc;
  hipLaunchKernelGGL(labels_lookup_kernel, dim3(grid_for(Q, 256)), dim3(256), 0, s, d_label, Q, l->kind, l->C,
                     l->label, l->scores, d_label);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_labels_count(insc_labels *l, int64_t *h_n, void *stream) {
  INSC_REQUIRE(l && h_n, INSC_ERR_ARG, "insc_labels_count: null argument");
  return insc_grid_size(l->grid, h_n, stream);
}

int insc_labels_export(insc_labels *l, int32_t *d_out4, float *d_conf, int64_t rows, void *stream) {
  INSC_REQUIRE(l && rows >= 0 && (rows == 0 || d_out4), INSC_ERR_ARG, "insc_labels_export: bad arguments");
  if (rows == 0) return INSC_OK;
  hipLaunchKernelGGL(labels_export_kernel, dim3(grid_for(rows, 256)), dim3(256), 0, (hipStream_t)stream,
                     insc_grid_coords(l->grid), l->grid->d_n, rows, l->kind, l->C, l->label, l->conf, l->scores, d_out4,
                     d_conf);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_labels_finalize(insc_labels *l, const int32_t *d_keep4, int64_t M, void *stream) {
  INSC_REQUIRE(l && M >= 0 && (M == 0 || d_keep4), INSC_ERR_ARG, "insc_labels_finalize: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  int64_t n = 0;
  int rc = insc_grid_size(l->grid, &n, stream);
  if (rc) return rc;
  if (n == 0) return INSC_OK;
  if (M == 0) return insc_grid_clear(l->grid, stream);
  const int C = l->kind == 1 ? l->C : 0;
  // scratch: site per kept point | mark | exclusive ranks | total | compacted coords, labels, conf, scores
  const size_t ints = (size_t)M + 3 * (size_t)n + 64 + 4 * (size_t)n + (size_t)n;
  void *ws;
  if ((rc = workspace(WS_LABELS, s, sizeof(int32_t) * ints + sizeof(float) * ((size_t)n + (size_t)n * C) + 256, &ws)))
    return rc;
  int32_t *site = (int32_t *)ws, *mark = site + M, *excl = mark + n, *row2 = excl + n, *total = row2 + n,
          *coords2 = total + 64, *label2 = coords2 + 4 * n;
  float *conf2 = (float *)(label2 + n), *scores2 = conf2 + n;
  if ((rc = insc_grid_query(l->grid, d_keep4, M, site, stream))) return rc;
  if ((rc = insc_fill_i32(mark, n, 0, stream))) return rc;
  hipLaunchKernelGGL(labels_mark_kernel, dim3(grid_for(M, 256)), dim3(256), 0, s, site, M, mark);
  INSC_LAUNCH_CHECK();
  if ((rc = scan_exclusive_i32(mark, excl, n, total, s))) return rc;
  hipLaunchKernelGGL(labels_compact_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, insc_grid_coords(l->grid), mark,
                     excl, total, n, C, l->kind == 0 ? l->label : nullptr, l->conf, l->kind == 1 ? l->scores : nullptr,
                     coords2, label2, conf2, scores2);
  INSC_LAUNCH_CHECK();
  // rebuild the grid from the kept voxels, in their old order (so row j is voxel j of the list)
  if ((rc = insc_grid_clear(l->grid, stream))) return rc;
  if ((rc = grid_insert_nosync(l->grid, coords2, n, row2, s))) return rc;
  if (l->kind == 0) {
    INSC_HIP(hipMemcpyAsync(l->label, label2, sizeof(int32_t) * (size_t)n, hipMemcpyDeviceToDevice, s));
    INSC_HIP(hipMemcpyAsync(l->conf, conf2, sizeof(float) * (size_t)n, hipMemcpyDeviceToDevice, s));
  } else if (C > 0) {
    INSC_HIP(hipMemcpyAsync(l->scores, scores2, sizeof(float) * (size_t)n * C, hipMemcpyDeviceToDevice, s));
  }
  int64_t kept = 0;
  return insc_grid_size(l->grid, &kept, stream);  // refreshes the host count (and waits for the copies)
}

}  // extern "C"
