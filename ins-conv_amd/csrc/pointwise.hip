// Row-wise streaming kernels: inference batch norm + leaky ReLU, add, column-slice copy,
// input-layer accumulation / mean, output-layer gather.  All are HBM-bandwidth bound: one
// thread owns a fixed group of four channels and walks rows, so loads and stores are
// 16-byte wide and coalesced along a row.
#include "common.h"
#include "grid.h"

namespace insc {

__device__ __forceinline__ int64_t row_count(const int32_t *d_n_rows, int64_t n_rows) {
  return d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
}

// V = 4: float4 path (C, strides multiples of 4, 16-byte aligned bases); V = 1: scalar path
template <int V>
struct Vec;
template <>
struct Vec<4> {
  typedef float4 T;
  static __device__ __forceinline__ T ld(const float *p) { return *reinterpret_cast<const float4 *>(p); }
  static __device__ __forceinline__ void st(float *p, T v) { *reinterpret_cast<float4 *>(p) = v; }
};
template <>
struct Vec<1> {
  typedef float T;
  static __device__ __forceinline__ T ld(const float *p) { return *p; }
  static __device__ __forceinline__ void st(float *p, T v) { *p = v; }
};

template <int V>
__global__ __launch_bounds__(256) void bn_kernel(const float *__restrict__ in, int64_t ld_in, float *__restrict__ out,
                                                 int64_t ld_out, const float *__restrict__ mean,
                                                 const float *__restrict__ var, const float *__restrict__ gamma,
                                                 const float *__restrict__ beta, float eps, float leak,
                                                 const int32_t *__restrict__ rows,
                                                 const int32_t *__restrict__ d_n_rows, int64_t n_rows, int C,
                                                 const uint8_t *__restrict__ row_mask) {
  const int64_t n = row_count(d_n_rows, n_rows);
  const int groups = C / V;  // channel groups per row
  const int rpb = 256 / groups > 0 ? 256 / groups : 1;
  const int g = threadIdx.x % groups, lr = threadIdx.x / groups;
  if (lr >= rpb || groups > 256) return;
  float w[V], b[V];
#pragma unroll
  for (int i = 0; i < V; i++) {
    bn_coeffs(mean, var, gamma, beta, eps, g * V + i, w[i], b[i]);
  }
  for (int64_t t = (int64_t)blockIdx.x * rpb + lr; t < n; t += (int64_t)gridDim.x * rpb) {
    const int row = rows ? rows[t] : (int)t;
    if (row < 0 || (row_mask && !row_mask[row])) continue;
    typename Vec<V>::T x = Vec<V>::ld(in + (int64_t)row * ld_in + g * V);
    float *xf = reinterpret_cast<float *>(&x);
#pragma unroll
    for (int i = 0; i < V; i++) xf[i] = leaky(fmaf(xf[i], w[i], b[i]), leak);
    Vec<V>::st(out + (int64_t)row * ld_out + g * V, x);
  }
}

// wide rows (more than 256 channel groups): one thread per element, any C
__global__ __launch_bounds__(256) void bn_wide_kernel(const float *__restrict__ in, int64_t ld_in,
                                                      float *__restrict__ out, int64_t ld_out,
                                                      const float *__restrict__ mean, const float *__restrict__ var,
                                                      const float *__restrict__ gamma, const float *__restrict__ beta,
                                                      float eps, float leak, const int32_t *__restrict__ rows,
                                                      const int32_t *__restrict__ d_n_rows, int64_t n_rows, int C,
                                                      const uint8_t *__restrict__ row_mask) {
  const int64_t n = row_count(d_n_rows, n_rows);
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n * C; e += (int64_t)gridDim.x * 256) {
    const int64_t t = e / C;
    const int c = (int)(e - t * C);
    const int row = rows ? rows[t] : (int)t;
    if (row < 0 || (row_mask && !row_mask[row])) continue;
    float wv, bv;
    bn_coeffs(mean, var, gamma, beta, eps, c, wv, bv);
    out[(int64_t)row * ld_out + c] = leaky(fmaf(in[(int64_t)row * ld_in + c], wv, bv), leak);
  }
}

// out = a + b (HAS_B) or out = a, on listed rows
template <int V, bool HAS_B>
__global__ __launch_bounds__(256) void add_kernel(const float *__restrict__ a, int64_t ld_a,
                                                  const float *__restrict__ b, int64_t ld_b, float *__restrict__ out,
                                                  int64_t ld_out, const int32_t *__restrict__ rows,
                                                  const int32_t *__restrict__ d_n_rows, int64_t n_rows, int C,
                                                  const uint8_t *__restrict__ row_mask, BnEpilogue ep) {
  const int64_t n = row_count(d_n_rows, n_rows);
  const int groups = C / V;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n * groups; e += (int64_t)gridDim.x * 256) {
    const int64_t t = e / groups;
    const int g = (int)(e - t * groups);
    const int row = rows ? rows[t] : (int)t;
    if (row < 0 || (row_mask && !row_mask[row])) continue;
    typename Vec<V>::T x = Vec<V>::ld(a + (int64_t)row * ld_a + g * V);
    if (HAS_B) {
      typename Vec<V>::T y = Vec<V>::ld(b + (int64_t)row * ld_b + g * V);
      float *xf = reinterpret_cast<float *>(&x);
      const float *yf = reinterpret_cast<const float *>(&y);
#pragma unroll
      for (int i = 0; i < V; i++) xf[i] += yf[i];
    }
    if (out) Vec<V>::st(out + (int64_t)row * ld_out + g * V, x);
    if (ep.out2) {
      float *xf = reinterpret_cast<float *>(&x);
#pragma unroll
      for (int i = 0; i < V; i++) xf[i] = leaky(fmaf(xf[i], ep.w[g * V + i], ep.b[g * V + i]), ep.leak);
      Vec<V>::st(ep.out2 + (int64_t)row * ep.ld2 + g * V, x);
    }
  }
}

__global__ void bn_scale_shift_kernel(const float *__restrict__ mean, const float *__restrict__ var,
                                      const float *__restrict__ gamma, const float *__restrict__ beta, float eps,
                                      int C, float *__restrict__ w, float *__restrict__ b) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  float wv, bv;
  bn_coeffs(mean, var, gamma, beta, eps, c, wv, bv);
  w[c] = wv;
  b[c] = bv;
}

__global__ __launch_bounds__(256) void gather_rows_kernel(const float *__restrict__ in, int64_t ld_in,
                                                          const int32_t *__restrict__ src, int64_t P, int C,
                                                          float *__restrict__ out) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < P * C; e += (int64_t)gridDim.x * 256) {
    const int64_t p = e / C;
    const int c = (int)(e - p * C);
    const int s = src[p];
    out[e] = (s >= 0) ? in[(int64_t)s * ld_in + c] : 0.0f;
  }
}

// ---- input layer -----------------------------------------------------------------------
// Input layer.  The rows of one site are chained: every row pushes itself on its site's list
// (an atomic exchange on the list head), and the row left at the head owns the site.  The owner
// visits the rows of the list in ascending row order - the order InputLayer_fp_ adds them in
// (CUDA/IOLayers.cu:17-32), so the float sum has the reference's rounding - and the lists are
// short (rows of one voxel in one call).
__global__ void input_push_kernel(const int32_t *__restrict__ sop, int64_t P, int32_t *__restrict__ head,
                                  int32_t *__restrict__ next) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int s = sop[p];
  next[p] = (s >= 0) ? atomicExch(&head[s], (int)p) : -1;
}

// one thread per (row, channel); only the threads of a list's head row work
__global__ __launch_bounds__(256) void input_reduce_kernel(const float *__restrict__ feats, int C,
                                                           const int32_t *__restrict__ sop, int64_t P,
                                                           const int32_t *__restrict__ head,
                                                           const int32_t *__restrict__ next, int mode,
                                                           float *__restrict__ sum, const int32_t *__restrict__ cnt) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < P * C; e += (int64_t)gridDim.x * 256) {
    const int64_t p = e / C;
    const int c = (int)(e - p * C);
    const int s = sop[p];
    if (s < 0 || head[s] != (int)p) continue;
    float acc = sum[(int64_t)s * C + c];
    if (mode == 1 || mode == 2) {  // keep the first / the last row of the site
      int pick = (int)p;
      for (int q = (int)p; q >= 0; q = next[q]) pick = mode == 1 ? min(pick, q) : max(pick, q);
      if (mode == 2 || cnt[s] == 0) acc = feats[(int64_t)pick * C + c];
    } else {
      int done = -1;
      for (;;) {
        int best = 0x7fffffff;
        for (int q = (int)p; q >= 0; q = next[q])
          if (q > done && q < best) best = q;
        if (best == 0x7fffffff) break;
        acc += feats[(int64_t)best * C + c];
        done = best;
      }
    }
    sum[(int64_t)s * C + c] = acc;
  }
}

// counts the rows of every list and empties it
__global__ void input_count_kernel(const int32_t *__restrict__ sop, int64_t P, int32_t *__restrict__ head,
                                   const int32_t *__restrict__ next, int32_t *__restrict__ cnt) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int s = sop[p];
  if (s < 0 || head[s] != (int)p) return;
  int n = 0;
  for (int q = (int)p; q >= 0; q = next[q]) n++;
  cnt[s] += n;
  head[s] = -1;
}

__global__ __launch_bounds__(256) void input_finish_kernel(const float *__restrict__ sum,
                                                           const int32_t *__restrict__ cnt, int mode,
                                                           float *__restrict__ out, int64_t ld_out,
                                                           const int32_t *__restrict__ rows,
                                                           const int32_t *__restrict__ d_n_rows, int64_t n_rows,
                                                           int C, const uint8_t *__restrict__ row_mask) {
  const int64_t n = row_count(d_n_rows, n_rows);
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n * C; e += (int64_t)gridDim.x * 256) {
    const int64_t t = e / C;
    const int c = (int)(e - t * C);
    const int row = rows ? rows[t] : (int)t;
    if (row < 0 || (row_mask && !row_mask[row])) continue;
    float v = sum[(int64_t)row * C + c];
    if (mode == 4) {
      const int k = cnt[row];
      if (k > 1) v = v / (float)k;
    }
    out[(int64_t)row * ld_out + c] = v;
  }
}

// Size-2 stride-2 pooling over the child map: one thread per (coarse site, channel).
//   MODE 0: max over the children, starting from zero (MaxPooling_fp, CUDA/MaxPooling.cu:10-33,
//           on an output that cuda_MaxPooling_updateOutput has zeroed)
//   MODE 1: sum over the children of x/8 in ascending offset order (AveragePooling_fp,
//           CUDA/AveragePooling.cu:10-33 with alpha = 1/filterVolume, one launch per offset)
template <int MODE>
__global__ __launch_bounds__(256) void pool_down2_kernel(const float *__restrict__ in, int64_t ld_in,
                                                         const int32_t *__restrict__ child, int64_t n_coarse, int C,
                                                         float *__restrict__ out, int64_t ld_out) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n_coarse * C; e += (int64_t)gridDim.x * 256) {
    const int64_t row = e / C;
    const int c = (int)(e - row * C);
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const int f = child[row * 8 + k];
      if (f < 0) continue;
      const float x = in[(int64_t)f * ld_in + c];
      if (MODE == 0)
        acc = (acc < x) ? x : acc;
      else
        acc += 0.125f * x;
    }
    out[row * ld_out + c] = acc;
  }
}

// Dense [batch, C, X, Y, Z] copy of a sparse feature matrix (SparseToDense_fp,
// CUDA/SparseToDense.cu:9-30; cell offset as RectangularRegion::offset, last axis fastest).
__global__ __launch_bounds__(256) void sparse_to_dense_kernel(const float *__restrict__ in, int64_t ld_in,
                                                              const int32_t *__restrict__ coords, int64_t n, int C,
                                                              int64_t X, int64_t Y, int64_t Z, int batch,
                                                              float *__restrict__ out) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n * C; e += (int64_t)gridDim.x * 256) {
    const int64_t row = e / C;
    const int c = (int)(e - row * C);
    const int4 p = reinterpret_cast<const int4 *>(coords)[row];
    if (p.x >= X || p.y >= Y || p.z >= Z || p.w >= batch) continue;
    out[(((int64_t)p.w * C + c) * X + p.x) * Y * Z + (int64_t)p.y * Z + p.z] = in[row * ld_in + c];
  }
}

static inline bool vec4_ok(const void *p, int64_t ld) { return ((uintptr_t)p % 16 == 0) && (ld % 4 == 0); }

int launch_bn(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_mean, const float *d_var,
              const float *d_gamma, const float *d_beta, float eps, float leakiness, const int32_t *d_rows,
              const int32_t *d_n_rows, int64_t n_rows, int C, const uint8_t *row_mask, hipStream_t s) {
  if (n_rows == 0) return INSC_OK;
  const bool v4 = C % 4 == 0 && vec4_ok(d_in, ld_in) && vec4_ok(d_out, ld_out);
  const int groups = v4 ? C / 4 : C;
  if (groups <= 256) {
    const int rpb = 256 / groups;
    const unsigned nb = grid_for(n_rows, rpb * 4, 1 << 16);
    if (v4)
      hipLaunchKernelGGL(bn_kernel<4>, dim3(nb), dim3(256), 0, s, d_in, ld_in, d_out, ld_out, d_mean, d_var, d_gamma,
                         d_beta, eps, leakiness, d_rows, d_n_rows, n_rows, C, row_mask);
    else
      hipLaunchKernelGGL(bn_kernel<1>, dim3(nb), dim3(256), 0, s, d_in, ld_in, d_out, ld_out, d_mean, d_var, d_gamma,
                         d_beta, eps, leakiness, d_rows, d_n_rows, n_rows, C, row_mask);
  } else {
    hipLaunchKernelGGL(bn_wide_kernel, dim3(grid_for(n_rows * C, 1024, 1 << 16)), dim3(256), 0, s, d_in, ld_in, d_out,
                       ld_out, d_mean, d_var, d_gamma, d_beta, eps, leakiness, d_rows, d_n_rows, n_rows, C, row_mask);
  }
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int bn_scale_shift(const float *mean, const float *var, const float *gamma, const float *beta, float eps, int C,
                   float *w, float *b, hipStream_t s) {
  hipLaunchKernelGGL(bn_scale_shift_kernel, dim3(grid_for(C, 256)), dim3(256), 0, s, mean, var, gamma, beta, eps, C, w,
                     b);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int launch_add(const float *d_a, int64_t ld_a, const float *d_b, int64_t ld_b, float *d_out, int64_t ld_out,
               const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C, const uint8_t *row_mask,
               hipStream_t s, BnEpilogue ep) {
  if (n_rows == 0) return INSC_OK;
  const bool v4 = C % 4 == 0 && vec4_ok(d_a, ld_a) && (!d_b || vec4_ok(d_b, ld_b)) &&
                  (!d_out || vec4_ok(d_out, ld_out)) && (!ep.out2 || vec4_ok(ep.out2, ep.ld2));
  const unsigned nb = grid_for(n_rows * (v4 ? C / 4 : C), 1024, 1 << 16);
  if (d_b) {
    if (v4)
      hipLaunchKernelGGL((add_kernel<4, true>), dim3(nb), dim3(256), 0, s, d_a, ld_a, d_b, ld_b, d_out, ld_out,
                         d_rows, d_n_rows, n_rows, C, row_mask, ep);
    else
      hipLaunchKernelGGL((add_kernel<1, true>), dim3(nb), dim3(256), 0, s, d_a, ld_a, d_b, ld_b, d_out, ld_out,
                         d_rows, d_n_rows, n_rows, C, row_mask, ep);
  } else {
    if (v4)
      hipLaunchKernelGGL((add_kernel<4, false>), dim3(nb), dim3(256), 0, s, d_a, ld_a, d_b, ld_b, d_out, ld_out,
                         d_rows, d_n_rows, n_rows, C, row_mask, ep);
    else
      hipLaunchKernelGGL((add_kernel<1, false>), dim3(nb), dim3(256), 0, s, d_a, ld_a, d_b, ld_b, d_out, ld_out,
                         d_rows, d_n_rows, n_rows, C, row_mask, ep);
  }
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int launch_input_finish(const float *d_sum, const int32_t *d_cnt, int mode, float *d_out, int64_t ld_out,
                        const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C,
                        const uint8_t *row_mask, hipStream_t s) {
  if (n_rows == 0) return INSC_OK;
  hipLaunchKernelGGL(input_finish_kernel, dim3(grid_for(n_rows * C, 256, 1 << 16)), dim3(256), 0, s, d_sum, d_cnt,
                     mode, d_out, ld_out, d_rows, d_n_rows, n_rows, C, row_mask);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_bn_leaky(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_mean,
                  const float *d_var, const float *d_gamma, const float *d_beta, float eps, float leakiness,
                  const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && C > 0 && ld_in >= C && ld_out >= C, INSC_ERR_ARG, "insc_bn_leaky: bad sizes");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && d_mean && d_var), INSC_ERR_ARG, "insc_bn_leaky: null pointer");
  return launch_bn(d_in, ld_in, d_out, ld_out, d_mean, d_var, d_gamma, d_beta, eps, leakiness, d_rows, d_n_rows,
                   n_rows, C, nullptr, (hipStream_t)stream);
}

int insc_add(const float *d_a, int64_t ld_a, const float *d_b, int64_t ld_b, float *d_out, int64_t ld_out,
             const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && C > 0 && ld_a >= C && ld_b >= C && ld_out >= C, INSC_ERR_ARG, "insc_add: bad sizes");
  INSC_REQUIRE(n_rows == 0 || (d_a && d_b && d_out), INSC_ERR_ARG, "insc_add: null pointer");
  return launch_add(d_a, ld_a, d_b, ld_b, d_out, ld_out, d_rows, d_n_rows, n_rows, C, nullptr, (hipStream_t)stream);
}

int insc_copy_rows(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const int32_t *d_rows,
                   const int32_t *d_n_rows, int64_t n_rows, int C, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && C > 0 && ld_in >= C && ld_out >= C, INSC_ERR_ARG, "insc_copy_rows: bad sizes");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out), INSC_ERR_ARG, "insc_copy_rows: null pointer");
  return launch_add(d_in, ld_in, nullptr, 0, d_out, ld_out, d_rows, d_n_rows, n_rows, C, nullptr,
                    (hipStream_t)stream);
}

int insc_input_accumulate(const float *d_feats, int64_t P, int C, const int32_t *d_site_of_point, int mode,
                          float *d_sum, int32_t *d_cnt, int64_t n_sites_upper, void *stream) {
  INSC_REQUIRE(P >= 0 && C > 0 && mode >= 0 && mode <= 4 && n_sites_upper >= 0, INSC_ERR_ARG,
               "insc_input_accumulate: bad arguments");
  INSC_REQUIRE(P == 0 || (d_feats && d_site_of_point && d_sum && d_cnt), INSC_ERR_ARG,
               "insc_input_accumulate: null pointer");
  if (P == 0) return INSC_OK;
  hipStream_t s = (hipStream_t)stream;
  void *ws;
  int rc = workspace(WS_API, s, sizeof(int32_t) * (size_t)(P + n_sites_upper) + 256, &ws);
  if (rc) return rc;
  int32_t *next = (int32_t *)ws, *head = next + P;
  if (n_sites_upper > 0 && (rc = insc_fill_i32(head, n_sites_upper, -1, stream))) return rc;
  const unsigned nb = grid_for(P, 256);
  hipLaunchKernelGGL(input_push_kernel, dim3(nb), dim3(256), 0, s, d_site_of_point, P, head, next);
  hipLaunchKernelGGL(input_reduce_kernel, dim3(grid_for(P * C, 256, 1 << 16)), dim3(256), 0, s, d_feats, C,
                     d_site_of_point, P, head, next, mode, d_sum, d_cnt);
  hipLaunchKernelGGL(input_count_kernel, dim3(nb), dim3(256), 0, s, d_site_of_point, P, head, next, d_cnt);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_input_finish(const float *d_sum, const int32_t *d_cnt, int mode, float *d_out, int64_t ld_out,
                      const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && C > 0 && ld_out >= C, INSC_ERR_ARG, "insc_input_finish: bad sizes");
  INSC_REQUIRE(n_rows == 0 || (d_sum && d_cnt && d_out), INSC_ERR_ARG, "insc_input_finish: null pointer");
  return launch_input_finish(d_sum, d_cnt, mode, d_out, ld_out, d_rows, d_n_rows, n_rows, C, nullptr,
                             (hipStream_t)stream);
}

int insc_output_gather(const float *d_in, int64_t ld_in, const int32_t *d_site_of_point, int64_t P, int C,
                       float *d_out, void *stream) {
  INSC_REQUIRE(P >= 0 && C > 0 && ld_in >= C, INSC_ERR_ARG, "insc_output_gather: bad sizes");
  INSC_REQUIRE(P == 0 || (d_in && d_site_of_point && d_out), INSC_ERR_ARG, "insc_output_gather: null pointer");
  if (P == 0) return INSC_OK;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(grid_for(P * C, 256, 1 << 16)), dim3(256), 0, (hipStream_t)stream, d_in,
                     ld_in, d_site_of_point, P, C, d_out);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_pool_down2(const float *d_in, int64_t ld_in, const int32_t *d_child, int64_t n_coarse, int C, int mode,
                    float *d_out, int64_t ld_out, void *stream) {
  INSC_REQUIRE(n_coarse >= 0 && C > 0 && ld_in >= C && ld_out >= C && (mode == 0 || mode == 1), INSC_ERR_ARG,
               "insc_pool_down2: bad arguments");
  if (n_coarse == 0) return INSC_OK;
  INSC_REQUIRE(d_in && d_child && d_out, INSC_ERR_ARG, "insc_pool_down2: null pointer");
  const dim3 g(grid_for(n_coarse * C, 256, 1 << 16));
  if (mode == 0)
    hipLaunchKernelGGL(pool_down2_kernel<0>, g, dim3(256), 0, (hipStream_t)stream, d_in, ld_in, d_child, n_coarse, C,
                       d_out, ld_out);
  else
    hipLaunchKernelGGL(pool_down2_kernel<1>, g, dim3(256), 0, (hipStream_t)stream, d_in, ld_in, d_child, n_coarse, C,
                       d_out, ld_out);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_sparse_to_dense(const insc_grid *g, const float *d_in, int64_t ld_in, int64_t n, int C, int64_t X, int64_t Y,
                         int64_t Z, int batch, float *d_out, void *stream) {
  INSC_REQUIRE(g && n >= 0 && n <= g->capacity_sites && C > 0 && ld_in >= C && X > 0 && Y > 0 && Z > 0 && batch > 0,
               INSC_ERR_ARG, "insc_sparse_to_dense: bad arguments");
  INSC_REQUIRE(d_out && (n == 0 || d_in), INSC_ERR_ARG, "insc_sparse_to_dense: null pointer");
  hipStream_t s = (hipStream_t)stream;
  INSC_HIP(hipMemsetAsync(d_out, 0, sizeof(float) * (size_t)batch * C * X * Y * Z, s));
  if (n == 0) return INSC_OK;
  hipLaunchKernelGGL(sparse_to_dense_kernel, dim3(grid_for(n * C, 256, 1 << 16)), dim3(256), 0, s, d_in, ld_in,
                     g->coords, n, C, X, Y, Z, batch, d_out);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // extern "C"
