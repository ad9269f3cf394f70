// Output-stationary sparse convolution (submanifold 3^3, strided 2^3, 1x1) and the size-2
// stride-2 deconvolution.
//
// Work unit: a tile of 32 output rows per wavefront.  For each filter offset k the wavefront
// looks up the 32 input rows (neighbour map), skips the offset when none exists, otherwise
// gathers the rows straight from HBM/L2 into registers (two lanes per row, 64 contiguous
// bytes each) and multiplies them with W[k] on the matrix cores (v_mfma_f32_32x32x2_f32,
// fp32 in, fp32 accumulate).  Accumulators stay in registers for all offsets, so every
// output row is written exactly once and no atomics are needed: the result of a row does
// not depend on which other rows share its tile, nor on the launch shape.
#include "common.h"

namespace insc {

typedef float f16v __attribute__((ext_vector_type(16)));

enum { MAP_NBR = 0, MAP_IDENTITY = 1, MAP_PARENT = 2 };

constexpr int CONV_WAVES = 4;
constexpr int TILE_M = 32;
constexpr int MAXK = 27;

// ---------------------------------------------------------------------------------------
// generic kernel: any Cin / Cout, one thread per (row, output channel).  Used for shapes
// the MFMA kernel does not cover (the 3-channel stem).
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void conv_generic_kernel(const float *__restrict__ in, int64_t ld_in,
                                                           float *__restrict__ out, int64_t ld_out,
                                                           const float *__restrict__ W,
                                                           const float *__restrict__ bias,
                                                           const int32_t *__restrict__ map0,
                                                           const int32_t *__restrict__ map1, int mode, int K,
                                                           const int32_t *__restrict__ rows,
                                                           const int32_t *__restrict__ d_n_rows, int64_t n_rows,
                                                           int Cin, int Cout) {
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int cpb = 256 / Cout > 0 ? 256 / Cout : 1;  // rows per block (Cout <= 256)
  const int lr = threadIdx.x / Cout, co = threadIdx.x % Cout;
  if (lr >= cpb) return;
  for (int64_t t = (int64_t)blockIdx.x * cpb + lr; t < n; t += (int64_t)gridDim.x * cpb) {
    const int row = rows ? rows[t] : (int)t;
    if (row < 0) continue;
    float acc = bias ? bias[co] : 0.0f;
    for (int k = 0; k < K; k++) {
      int src;
      if (mode == MAP_NBR)
        src = map0[(int64_t)row * K + k];
      else if (mode == MAP_IDENTITY)
        src = row;
      else
        src = (map1[row] == k) ? map0[row] : -1;
      if (src < 0) continue;
      const float *x = in + (int64_t)src * ld_in;
      const float *w = W + (int64_t)k * Cin * Cout + co;
      for (int ci = 0; ci < Cin; ci++) acc = fmaf(x[ci], w[(int64_t)ci * Cout], acc);
    }
    out[(int64_t)row * ld_out + co] = acc;
  }
}

// ---------------------------------------------------------------------------------------
// MFMA kernel.  Cin % 16 == 0, rows of `in` 16-byte aligned.  Each block column
// (blockIdx.y) covers NB*32 output channels starting at blockIdx.y*NB*32.
// ---------------------------------------------------------------------------------------
template <int NB>
__global__ __launch_bounds__(CONV_WAVES * 64) void conv_mfma_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ W, const float *__restrict__ bias, const int32_t *__restrict__ map0,
    const int32_t *__restrict__ map1, int mode, int K, const int32_t *__restrict__ rows,
    const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout) {
  __shared__ int nbl[CONV_WAVES][TILE_M * MAXK];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int64_t t0 = ((int64_t)blockIdx.x * CONV_WAVES + wave) * TILE_M;
  const int col0 = blockIdx.y * NB * 32;

  int my_row = -1;
  if (t0 + r < n) my_row = rows ? rows[t0 + r] : (int)(t0 + r);

  // stage the tile's slice of the neighbour map in LDS
  int *nl = nbl[wave];
  for (int e = lane; e < TILE_M * K; e += 64) {
    const int rr = e / K, kk = e - rr * K;
    const int rid = __shfl(my_row, rr, 64);
    int v = -1;
    if (rid >= 0) {
      if (mode == MAP_NBR)
        v = map0[(int64_t)rid * K + kk];
      else if (mode == MAP_IDENTITY)
        v = rid;
      else
        v = (map1[rid] == kk) ? map0[rid] : -1;
    }
    nl[e] = v;
  }
  __syncthreads();
  if (t0 >= n) return;  // whole wavefront idle; no barrier follows

  f16v acc[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) {
    const int c = col0 + b * 32 + r;
    const float bv = (bias && c < Cout) ? bias[c] : 0.0f;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[b][v] = bv;
  }

  for (int k = 0; k < K; k++) {
    const int src = nl[r * K + k];
    if (__ballot(src >= 0) == 0ull) continue;
    const float *wk = W + (int64_t)k * Cin * Cout;
    for (int c0 = 0; c0 < Cin; c0 += 32) {
      const int half = (Cin - c0 >= 32) ? 16 : 8;  // Cin % 16 == 0
      float a[16];
      const float4 *xp = reinterpret_cast<const float4 *>(in + (int64_t)(src < 0 ? 0 : src) * ld_in + c0 + h * half);
      if (half == 16) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
          float4 v = (src >= 0) ? xp[q] : make_float4(0.f, 0.f, 0.f, 0.f);
          a[4 * q] = v.x; a[4 * q + 1] = v.y; a[4 * q + 2] = v.z; a[4 * q + 3] = v.w;
        }
        const float *wp = wk + (int64_t)(c0 + h * 16) * Cout + col0 + r;
#pragma unroll
        for (int s = 0; s < 16; s++) {
#pragma unroll
          for (int b = 0; b < NB; b++) {
            const float bv = (col0 + b * 32 + r < Cout) ? wp[(int64_t)s * Cout + b * 32] : 0.0f;
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], bv, acc[b], 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int q = 0; q < 2; q++) {
          float4 v = (src >= 0) ? xp[q] : make_float4(0.f, 0.f, 0.f, 0.f);
          a[4 * q] = v.x; a[4 * q + 1] = v.y; a[4 * q + 2] = v.z; a[4 * q + 3] = v.w;
        }
        const float *wp = wk + (int64_t)(c0 + h * 8) * Cout + col0 + r;
#pragma unroll
        for (int s = 0; s < 8; s++) {
#pragma unroll
          for (int b = 0; b < NB; b++) {
            const float bv = (col0 + b * 32 + r < Cout) ? wp[(int64_t)s * Cout + b * 32] : 0.0f;
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], bv, acc[b], 0, 0, 0);
          }
        }
      }
    }
  }

  // D layout of the 32x32 MFMA: lane holds column (lane & 31), rows 8*(v/4) + 4*(lane>>5) + (v&3)
#pragma unroll
  for (int v = 0; v < 16; v++) {
    const int i = 8 * (v >> 2) + 4 * h + (v & 3);
    const int rid = __shfl(my_row, i, 64);
    if (rid < 0) continue;
    float *op = out + (int64_t)rid * ld_out + col0 + r;
#pragma unroll
    for (int b = 0; b < NB; b++)
      if (col0 + b * 32 + r < Cout) op[b * 32] = acc[b][v];
  }
}

__global__ void count_rules_kernel(const int32_t *__restrict__ map0, int K, const int32_t *__restrict__ rows,
                                   const int32_t *__restrict__ d_n_rows, int64_t n_rows,
                                   unsigned long long *__restrict__ total) {
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int c = 0;
  if (t < n) {
    const int row = rows ? rows[t] : (int)t;
    if (row >= 0)
      for (int k = 0; k < K; k++) c += map0[(int64_t)row * K + k] >= 0 ? 1 : 0;
  }
  for (int d = 32; d > 0; d >>= 1) c += __shfl_down(c, d, 64);
  if ((threadIdx.x & 63) == 0 && c) atomicAdd(total, (unsigned long long)c);
}

static int launch_conv(const float *in, int64_t ld_in, float *out, int64_t ld_out, const float *W, const float *bias,
                       const int32_t *map0, const int32_t *map1, int mode, int K, const int32_t *rows,
                       const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout, hipStream_t s) {
  if (n_rows == 0) return INSC_OK;
  const bool aligned = ((uintptr_t)in % 16 == 0) && (ld_in % 4 == 0);
  if (Cin % 16 == 0 && aligned && K <= MAXK) {
    const int64_t tiles = cdiv(n_rows, TILE_M);
    const unsigned gx = (unsigned)cdiv(tiles, CONV_WAVES);
    const int nb_total = (Cout + 31) / 32;
    int NB = nb_total > 7 ? 4 : nb_total;  // wide outputs: column groups of 4 blocks
    const unsigned gy = (unsigned)cdiv(nb_total, NB);
    dim3 grid(gx, gy), block(CONV_WAVES * 64);
#define INSC_CONV_CASE(NBV)                                                                                     \
  case NBV:                                                                                                     \
    hipLaunchKernelGGL(conv_mfma_kernel<NBV>, grid, block, 0, s, in, ld_in, out, ld_out, W, bias, map0, map1,   \
                       mode, K, rows, d_n_rows, n_rows, Cin, Cout);                                             \
    break;
    switch (NB) {
      INSC_CONV_CASE(1)
      INSC_CONV_CASE(2)
      INSC_CONV_CASE(3)
      INSC_CONV_CASE(4)
      INSC_CONV_CASE(5)
      INSC_CONV_CASE(6)
      INSC_CONV_CASE(7)
    }
#undef INSC_CONV_CASE
  } else {
    if (Cout > 256) {
      set_error("conv: Cout=%d > 256 is not supported for Cin=%d", Cout, Cin);
      return INSC_ERR_ARG;
    }
    const int cpb = 256 / Cout;
    hipLaunchKernelGGL(conv_generic_kernel, dim3(grid_for(n_rows, cpb, 65536)), dim3(256), 0, s, in, ld_in, out,
                       ld_out, W, bias, map0, map1, mode, K, rows, d_n_rows, n_rows, Cin, Cout);
  }
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_conv_nbr(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_W,
                  const float *d_bias, const int32_t *d_nbr, int K, const int32_t *d_rows, const int32_t *d_n_rows,
                  int64_t n_rows, int Cin, int Cout, double *h_muladds, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && Cin > 0 && Cout > 0 && K > 0 && K <= MAXK, INSC_ERR_ARG,
               "insc_conv_nbr: bad sizes (n_rows=%lld Cin=%d Cout=%d K=%d)", (long long)n_rows, Cin, Cout, K);
  INSC_REQUIRE(ld_in >= Cin && ld_out >= Cout, INSC_ERR_ARG, "insc_conv_nbr: row stride smaller than channel count");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && d_W), INSC_ERR_ARG, "insc_conv_nbr: null pointer");
  INSC_REQUIRE(d_nbr || K == 1, INSC_ERR_ARG, "insc_conv_nbr: a null map needs K == 1");
  hipStream_t s = (hipStream_t)stream;
  int rc = launch_conv(d_in, ld_in, d_out, ld_out, d_W, d_bias, d_nbr, nullptr, d_nbr ? MAP_NBR : MAP_IDENTITY, K,
                       d_rows, d_n_rows, n_rows, Cin, Cout, s);
  if (rc) return rc;
  if (h_muladds) {
    unsigned long long h = 0;
    if (n_rows > 0 && d_nbr) {
      void *ws;
      rc = workspace(WS_API, s, 256, &ws);
      if (rc) return rc;
      rc = insc_fill_i32((int32_t *)ws, 2, 0, stream);
      if (rc) return rc;
      hipLaunchKernelGGL(count_rules_kernel, dim3(grid_for(n_rows, 256)), dim3(256), 0, s, d_nbr, K, d_rows, d_n_rows,
                         n_rows, (unsigned long long *)ws);
      INSC_LAUNCH_CHECK();
      INSC_HIP(hipMemcpyAsync(&h, ws, 8, hipMemcpyDeviceToHost, s));
      INSC_HIP(hipStreamSynchronize(s));
    } else if (n_rows > 0) {
      int32_t hn = (int32_t)n_rows;
      if (d_n_rows) {
        INSC_HIP(hipMemcpyAsync(&hn, d_n_rows, 4, hipMemcpyDeviceToHost, s));
        INSC_HIP(hipStreamSynchronize(s));
      }
      h = (unsigned long long)hn;
    }
    *h_muladds = (double)h * Cin * Cout;
  }
  return INSC_OK;
}

int insc_deconv_down2(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_W,
                      const float *d_bias, const int32_t *d_parent, const int32_t *d_offset, const int32_t *d_rows,
                      const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && Cin > 0 && Cout > 0, INSC_ERR_ARG, "insc_deconv_down2: bad sizes");
  INSC_REQUIRE(ld_in >= Cin && ld_out >= Cout, INSC_ERR_ARG, "insc_deconv_down2: row stride too small");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && d_W && d_parent && d_offset), INSC_ERR_ARG,
               "insc_deconv_down2: null pointer");
  return launch_conv(d_in, ld_in, d_out, ld_out, d_W, d_bias, d_parent, d_offset, MAP_PARENT, 8, d_rows, d_n_rows,
                     n_rows, Cin, Cout, (hipStream_t)stream);
}

}  // extern "C"
