// Residual frames: the reference's own incremental mode (its Incre_* operators).
//
// A frame's points get a site set of their own (a fresh grid at every scale); the features that
// travel through the network are differences to the state saved by the last full forward for
// sites that existed then, and plain values for sites that did not.  pre_exist[i] is the id the
// frame's site i has in the saved site set of the same scale, or -1.  Every operator here is
// exact for the rows it produces; the mode as a whole is an approximation because a 3^3
// convolution leaves the rows around the frame's sites untouched.
//
// All kernels are streaming (one thread per channel group of a row); the two convolutions are
// the ordinary kernels with the saved features as a second source (a second set of blocks in
// the same launch, or a second pass for the shapes without such a kernel).
#include "common.h"
#include "grid.h"

namespace insc {

// Input layer (InputLayer_inc_fp_, CUDA/IOLayers.cu:81-105): with n rows of this frame and pn
// saved rows at a voxel, m = 1/(n+pn) for the mean (1 otherwise),
//   out = m * sum_new + pre * (pn*m - 1)      for a voxel that existed,    out = m * sum_new  else.
// n and pn are the lengths of the rule rows: 1 for modes 1 and 2, the number of points for 3, 4.
__global__ __launch_bounds__(256) void incre_input_kernel(const float *__restrict__ sum,
                                                          const int32_t *__restrict__ cnt, int mode,
                                                          const int32_t *__restrict__ pre_exist,
                                                          const float *__restrict__ pre_out, int64_t ld_pre,
                                                          const int32_t *__restrict__ pre_cnt,
                                                          float *__restrict__ out, int64_t ld_out, int64_t n, int C) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n * C; e += (int64_t)gridDim.x * 256) {
    const int64_t row = e / C;
    const int c = (int)(e - row * C);
    const int pe = pre_exist[row];
    const int na = mode >= 3 ? cnt[row] : 1;
    const int pn = pe >= 0 ? (mode >= 3 ? pre_cnt[pe] : 1) : 0;
    const float m = (mode == 4 && na > 0) ? 1.0f / (float)(na + pn) : 1.0f;
    float v = m * sum[row * C + c];
    if (pe >= 0) v = v + pre_out[(int64_t)pe * ld_pre + c] * ((float)pn * m - 1.0f);
    out[row * ld_out + c] = v;
  }
}

// Batch norm + leaky ReLU (Incre_BatchNormalization_f_test, CUDA/BatchNormalization.cu:112-150):
//   o = w*x + b;  existing site: leaky(o + w*pre_in) - pre_out;  new site: leaky(o)
__global__ __launch_bounds__(256) void incre_bn_kernel(const float *__restrict__ in, int64_t ld_in,
                                                       float *__restrict__ out, int64_t ld_out,
                                                       const float *__restrict__ mean, const float *__restrict__ var,
                                                       const float *__restrict__ gamma, const float *__restrict__ beta,
                                                       float eps, float leak, const float *__restrict__ wv,
                                                       const float *__restrict__ bv,
                                                       const int32_t *__restrict__ pre_exist,
                                                       const float *__restrict__ pre_in, int64_t ld_pin,
                                                       const float *__restrict__ pre_out, int64_t ld_pout, int64_t n,
                                                       int C) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n * C; e += (int64_t)gridDim.x * 256) {
    const int64_t row = e / C;
    const int c = (int)(e - row * C);
    float w, b;
    if (wv) {  // scale / shift already formed (bn_scale_shift: the same two numbers)
      w = wv[c];
      b = bv[c];
    } else {
      bn_coeffs(mean, var, gamma, beta, eps, c, w, b);
    }
    const float o = fmaf(in[row * ld_in + c], w, b);
    const int pe = pre_exist[row];
    float y;  // (the same operations, one by one, as the fused form in the convolution's epilogue)
    if (pe >= 0)
      y = sub_exact(leaky(fmaf(pre_in[(int64_t)pe * ld_pin + c], w, o), leak), pre_out[(int64_t)pe * ld_pout + c]);
    else
      y = leaky(o, leak);
    out[row * ld_out + c] = y;
  }
}

// Deconvolution: which saved coarse row a fine site also reads (dDeconvolution_incre_KMxKN_forwardA,
// CUDA/Deconvolution.cu:84-150: the saved input joins in when the coarse site existed and the
// fine site did not).
__global__ void incre_parent_kernel(const int32_t *__restrict__ parent, const int32_t *__restrict__ pre_exist_in,
                                    const int32_t *__restrict__ pre_exist_out, int64_t n_fine, int64_t n_coarse,
                                    int32_t *__restrict__ parent2) {
  const int64_t f = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= n_fine) return;
  const int p = parent[f];
  int r = -1;
  if (p >= 0 && p < n_coarse && pre_exist_out[f] < 0) r = pre_exist_in[p];
  parent2[f] = r;
}

// Output layer (InputLayer_inc_bp_, CUDA/IOLayers.cu:122-141): residual + saved value.
__global__ __launch_bounds__(256) void incre_output_kernel(const float *__restrict__ in, int64_t ld_in,
                                                           const float *__restrict__ pre_in, int64_t ld_pre,
                                                           const int32_t *__restrict__ pre_exist,
                                                           const int32_t *__restrict__ sop, int64_t P, int C,
                                                           float *__restrict__ out) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < P * C; e += (int64_t)gridDim.x * 256) {
    const int64_t p = e / C;
    const int c = (int)(e - p * C);
    const int s = sop[p];
    float v = 0.0f;
    if (s >= 0) {
      v = in[(int64_t)s * ld_in + c];
      const int pe = pre_exist[s];
      if (pe >= 0) v += pre_in[(int64_t)pe * ld_pre + c];
    }
    out[e] = v;
  }
}

int launch_incre_bn(const float *in, int64_t ld_in, float *out, int64_t ld_out, const float *mean, const float *var,
                    const float *gamma, const float *beta, float eps, float leak, const float *w, const float *b,
                    const int32_t *pre_exist, const float *pre_in, int64_t ld_pin, const float *pre_out,
                    int64_t ld_pout, int64_t n, int C, hipStream_t s) {
  if (n == 0) return INSC_OK;
  hipLaunchKernelGGL(incre_bn_kernel, dim3(grid_for(n * C, 256, 1 << 16)), dim3(256), 0, s, in, ld_in, out, ld_out,
                     mean, var, gamma, beta, eps, leak, w, b, pre_exist, pre_in, ld_pin, pre_out, ld_pout, n, C);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int incre_conv_ssc(const float *in, int64_t ld_in, const float *pre_in, int64_t ld_pre, int64_t n_pre_rows, float *out,
                   int64_t ld_out, const float *W, const float *Wp, const float *bias, const int32_t *nbr,
                   const int32_t *nbr_pre, int64_t n, int Cin, int Cout, BnEpilogue ep, hipStream_t s) {
  // rules inside the frame's site set, on the residual features (CUDA/Convolution.cpp:264-268,283);
  // new sites also gather the saved features of their neighbours in the saved set (:274,287)
  const float *res = ep.res;
  const int64_t ldr = ep.ldr;
  if (n_pre_rows == 0)
    return launch_conv(in, ld_in, n, out, ld_out, W, Wp, bias, nbr, nullptr, MAP_NBR, 27, nullptr, nullptr, n, Cin, Cout,
                       nullptr, nullptr, s, ep, TilePlan(), 1);
  if (conv_two_sources_ok(MAP_NBR, 27, in, ld_in, pre_in, ld_pre, n_pre_rows, Cin, 1)) {
    // one launch: a second set of blocks per tile walks the saved features
    ep.src2_in = pre_in;
    ep.src2_ld = ld_pre;
    ep.src2_rows = n_pre_rows;
    ep.src2_map = nbr_pre;
    return launch_conv(in, ld_in, n, out, ld_out, W, Wp, bias, nbr, nullptr, MAP_NBR, 27, nullptr, nullptr, n, Cin, Cout,
                       nullptr, nullptr, s, ep, TilePlan(), 1);
  }
  // two passes, the second adding to the first (and the element-wise sum, if any, behind them)
  if (ep.out2 || ep.pre_exist) {
    set_error("incre_conv_ssc: no fused batch norm for a layer that runs in two passes (Cin=%d)", Cin);
    return INSC_ERR_ARG;
  }
  int rc = launch_conv(in, ld_in, n, out, ld_out, W, Wp, bias, nbr, nullptr, MAP_NBR, 27, nullptr, nullptr, n, Cin, Cout,
                       nullptr, nullptr, s, BnEpilogue(), TilePlan(), 1);
  if (rc) return rc;
  BnEpilogue e2;
  e2.res = out;
  e2.ldr = ld_out;
  rc = launch_conv(pre_in, ld_pre, n_pre_rows, out, ld_out, W, Wp, nullptr, nbr_pre, nullptr, MAP_NBR, 27, nullptr,
                   nullptr, n, Cin, Cout, nullptr, nullptr, s, e2, TilePlan(), 1);
  if (rc || !res) return rc;
  return launch_add(out, ld_out, res, ldr, out, ld_out, nullptr, nullptr, n, Cout, nullptr, s);
}

int incre_deconv_down2(const float *in, int64_t ld_in, int64_t n_in_rows, const float *pre_in, int64_t ld_pre,
                       int64_t n_pre_rows, float *out, int64_t ld_out, const float *W, const float *Wp,
                       const float *bias, const int32_t *parent, const int32_t *offset, const int32_t *pre_exist_in,
                       const int32_t *pre_exist_out, int64_t n_rows, int Cin, int Cout, const float *res, int64_t ldr,
                       hipStream_t s, const int32_t *parent2_ready) {
  BnEpilogue ep;
  ep.res = res;
  ep.ldr = ldr;
  if (n_pre_rows == 0)
    return launch_conv(in, ld_in, n_in_rows, out, ld_out, W, Wp, bias, parent, offset, MAP_PARENT, 8, nullptr, nullptr,
                       n_rows, Cin, Cout, nullptr, nullptr, s, ep);
  // the saved coarse row a fine site also reads
  int rc;
  const int32_t *parent2 = parent2_ready;
  if (!parent2) {
    void *ws;
    rc = workspace(WS_INCRE, s, sizeof(int32_t) * (size_t)n_rows, &ws);
    if (rc) return rc;
    hipLaunchKernelGGL(incre_parent_kernel, dim3(grid_for(n_rows, 256)), dim3(256), 0, s, parent, pre_exist_in,
                       pre_exist_out, n_rows, n_in_rows, (int32_t *)ws);
    INSC_LAUNCH_CHECK();
    parent2 = (const int32_t *)ws;
  }
  if (conv_two_sources_ok(MAP_PARENT, 8, in, ld_in, pre_in, ld_pre, n_pre_rows, Cin, 0)) {
    ep.src2_in = pre_in;
    ep.src2_ld = ld_pre;
    ep.src2_rows = n_pre_rows;
    ep.src2_map = parent2;
    return launch_conv(in, ld_in, n_in_rows, out, ld_out, W, Wp, bias, parent, offset, MAP_PARENT, 8, nullptr, nullptr,
                       n_rows, Cin, Cout, nullptr, nullptr, s, ep);
  }
  rc = launch_conv(in, ld_in, n_in_rows, out, ld_out, W, Wp, bias, parent, offset, MAP_PARENT, 8, nullptr, nullptr,
                   n_rows, Cin, Cout, nullptr, nullptr, s);
  if (rc) return rc;
  BnEpilogue e2;
  e2.res = out;
  e2.ldr = ld_out;
  rc = launch_conv(pre_in, ld_pre, n_pre_rows, out, ld_out, W, Wp, nullptr, parent2, offset, MAP_PARENT, 8, nullptr,
                   nullptr, n_rows, Cin, Cout, nullptr, nullptr, s, e2);
  if (rc || !res) return rc;
  return launch_add(out, ld_out, res, ldr, out, ld_out, nullptr, nullptr, n_rows, Cout, nullptr, s);
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_incre_input(const float *d_sum, const int32_t *d_cnt, int mode, const int32_t *d_pre_exist,
                     const float *d_pre_out, int64_t ld_pre, const int32_t *d_pre_cnt, float *d_out, int64_t ld_out,
                     int64_t n, int C, void *stream) {
  INSC_REQUIRE(n >= 0 && C > 0 && mode >= 0 && mode <= 4 && ld_out >= C && ld_pre >= C, INSC_ERR_ARG,
               "insc_incre_input: bad arguments");
  if (n == 0) return INSC_OK;
  INSC_REQUIRE(d_sum && d_cnt && d_pre_exist && d_pre_out && d_pre_cnt && d_out, INSC_ERR_ARG,
               "insc_incre_input: null pointer");
  hipLaunchKernelGGL(incre_input_kernel, dim3(grid_for(n * C, 256, 1 << 16)), dim3(256), 0, (hipStream_t)stream, d_sum,
                     d_cnt, mode, d_pre_exist, d_pre_out, ld_pre, d_pre_cnt, d_out, ld_out, n, C);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_incre_conv_ssc(const float *d_in, int64_t ld_in, const float *d_pre_in, int64_t ld_pre, int64_t n_pre_rows,
                        float *d_out, int64_t ld_out, const float *d_W, const float *d_Wp, const float *d_bias,
                        const int32_t *d_nbr, const int32_t *d_nbr_pre, int64_t n, int Cin, int Cout, void *stream) {
  INSC_REQUIRE(n >= 0 && n_pre_rows >= 0 && Cin > 0 && Cout > 0 && ld_in >= Cin && ld_pre >= Cin && ld_out >= Cout,
               INSC_ERR_ARG, "insc_incre_conv_ssc: bad sizes");
  if (n == 0) return INSC_OK;
  INSC_REQUIRE(d_in && d_out && (d_W || d_Wp) && d_nbr && d_nbr_pre && (d_pre_in || n_pre_rows == 0), INSC_ERR_ARG,
               "insc_incre_conv_ssc: null pointer");
  return incre_conv_ssc(d_in, ld_in, d_pre_in, ld_pre, n_pre_rows, d_out, ld_out, d_W, d_Wp, d_bias, d_nbr, d_nbr_pre, n,
                        Cin, Cout, BnEpilogue(), (hipStream_t)stream);
}

int insc_incre_bn_leaky(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_mean,
                        const float *d_var, const float *d_gamma, const float *d_beta, float eps, float leakiness,
                        const int32_t *d_pre_exist, const float *d_pre_in, int64_t ld_pre_in, const float *d_pre_out,
                        int64_t ld_pre_out, int64_t n, int C, void *stream) {
  INSC_REQUIRE(n >= 0 && C > 0 && ld_in >= C && ld_out >= C && ld_pre_in >= C && ld_pre_out >= C, INSC_ERR_ARG,
               "insc_incre_bn_leaky: bad sizes");
  if (n == 0) return INSC_OK;
  INSC_REQUIRE(d_in && d_out && d_mean && d_var && d_pre_exist && d_pre_in && d_pre_out, INSC_ERR_ARG,
               "insc_incre_bn_leaky: null pointer");
  return launch_incre_bn(d_in, ld_in, d_out, ld_out, d_mean, d_var, d_gamma, d_beta, eps, leakiness, nullptr, nullptr,
                         d_pre_exist, d_pre_in, ld_pre_in, d_pre_out, ld_pre_out, n, C, (hipStream_t)stream);
}

int insc_incre_deconv_down2(const float *d_in, int64_t ld_in, int64_t n_in_rows, const float *d_pre_in, int64_t ld_pre,
                            int64_t n_pre_rows, float *d_out, int64_t ld_out, const float *d_W, const float *d_Wp,
                            const float *d_bias, const int32_t *d_parent, const int32_t *d_offset,
                            const int32_t *d_pre_exist_in, const int32_t *d_pre_exist_out, int64_t n_rows, int Cin,
                            int Cout, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && n_in_rows >= 0 && n_pre_rows >= 0 && Cin > 0 && Cout > 0 && ld_in >= Cin &&
                   ld_pre >= Cin && ld_out >= Cout,
               INSC_ERR_ARG, "insc_incre_deconv_down2: bad sizes");
  if (n_rows == 0) return INSC_OK;
  INSC_REQUIRE(d_in && d_out && (d_W || d_Wp) && d_parent && d_offset && d_pre_exist_in && d_pre_exist_out &&
                   (d_pre_in || n_pre_rows == 0),
               INSC_ERR_ARG, "insc_incre_deconv_down2: null pointer");
  return incre_deconv_down2(d_in, ld_in, n_in_rows, d_pre_in, ld_pre, n_pre_rows, d_out, ld_out, d_W, d_Wp, d_bias,
                            d_parent, d_offset, d_pre_exist_in, d_pre_exist_out, n_rows, Cin, Cout, nullptr, 0,
                            (hipStream_t)stream);
}

int insc_incre_output(const float *d_in, int64_t ld_in, const float *d_pre_in, int64_t ld_pre,
                      const int32_t *d_pre_exist, const int32_t *d_site_of_point, int64_t P, int C, float *d_out,
                      void *stream) {
  INSC_REQUIRE(P >= 0 && C > 0 && ld_in >= C && ld_pre >= C, INSC_ERR_ARG, "insc_incre_output: bad sizes");
  if (P == 0) return INSC_OK;
  INSC_REQUIRE(d_in && d_pre_in && d_pre_exist && d_site_of_point && d_out, INSC_ERR_ARG,
               "insc_incre_output: null pointer");
  hipLaunchKernelGGL(incre_output_kernel, dim3(grid_for(P * C, 256, 1 << 16)), dim3(256), 0, (hipStream_t)stream, d_in,
                     ld_in, d_pre_in, ld_pre, d_pre_exist, d_site_of_point, P, C, d_out);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // extern "C"
