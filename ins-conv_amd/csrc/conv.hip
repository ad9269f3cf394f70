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
// Weight packing.  The MFMA kernel wants, for filter offset k, input-channel chunk ch (32
// channels) and output-channel block nb (32 channels), the 16 B-operand values of a lane
// contiguous: lane = h*32 + j holds W[k][ch*32 + h*16 + s][nb*32 + j], s = 0..15.  One
// wavefront then reads its 4 KB operand tile with four 16-byte loads per lane.  Channels
// beyond Cin / Cout are zero.
// ---------------------------------------------------------------------------------------
__host__ __device__ static inline int conv_nch(int Cin) { return (Cin + 31) / 32; }
static inline int conv_nb_per_group(int Cout) {
  const int nbt = (Cout + 31) / 32;
  return nbt > 7 ? 4 : nbt;
}
static inline int conv_nbt_padded(int Cout) {
  const int nbt = (Cout + 31) / 32, nb = conv_nb_per_group(Cout);
  return (int)cdiv(nbt, nb) * nb;
}

__global__ void pack_weights_kernel(const float *__restrict__ W, int K, int Cin, int Cout, int nch, int nbtp,
                                    float *__restrict__ Wp) {
  const int64_t total = (int64_t)K * nch * nbtp * 1024;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int s = (int)(e & 15), lane = (int)((e >> 4) & 63);
    int64_t q = e >> 10;
    const int nb = (int)(q % nbtp);
    q /= nbtp;
    const int ch = (int)(q % nch), k = (int)(q / nch);
    const int cin = ch * 32 + (lane >> 5) * 16 + s, col = nb * 32 + (lane & 31);
    Wp[e] = (cin < Cin && col < Cout) ? W[((int64_t)k * Cin + cin) * Cout + col] : 0.0f;
  }
}

// ---------------------------------------------------------------------------------------
// MFMA kernel.  Cin % 16 == 0, rows of `in` 16-byte aligned, packed weights.
// Software pipeline: while the 16*NB MFMAs of one (offset, channel chunk) run, the gather of
// the next chunk's input rows and the next weight tile are already in flight.
// ---------------------------------------------------------------------------------------
struct Frag {
  float4 q[4];
};

// Lanes whose row has no neighbour at the current offset read this row of zeros instead, so
// the gather needs no branch and no select.
__device__ __attribute__((aligned(64))) float g_zero_row[16];

__device__ __forceinline__ Frag load_frag(const float *p) {
  Frag f;
  const float4 *p4 = reinterpret_cast<const float4 *>(p);
#pragma unroll
  for (int i = 0; i < 4; i++) f.q[i] = p4[i];
  return f;
}
__device__ __forceinline__ float frag_at(const Frag &f, int s) {
  const float4 v = f.q[s >> 2];
  return (s & 3) == 0 ? v.x : (s & 3) == 1 ? v.y : (s & 3) == 2 ? v.z : v.w;
}

template <int NB>
__global__ __launch_bounds__(CONV_WAVES * 64) void conv_mfma_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ Wp, const float *__restrict__ bias, const int32_t *__restrict__ map0,
    const int32_t *__restrict__ map1, int mode, int K, const int32_t *__restrict__ rows,
    const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout, int nbtp) {
  __shared__ int nbl[CONV_WAVES][TILE_M * MAXK];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int64_t t0 = ((int64_t)blockIdx.x * CONV_WAVES + wave) * TILE_M;
  const int cb0 = blockIdx.y * NB;  // first output-channel block of this column group
  const int nch = conv_nch(Cin);

  int my_row = -1;
  if (t0 + r < n) my_row = rows ? rows[t0 + r] : (int)(t0 + r);

  // stage the tile's slice of the neighbour map in LDS and find the offsets it uses
  int *nl = nbl[wave];
  unsigned mymask = 0;
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
    if (v >= 0) mymask |= 1u << kk;
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) mymask |= (unsigned)__shfl_xor((int)mymask, d, 64);
  __syncthreads();
  if (t0 >= n) return;  // whole wavefront idle; no barrier follows
  unsigned rest = (unsigned)__builtin_amdgcn_readfirstlane((int)mymask);

  f16v acc[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) {
    const int c = (cb0 + b) * 32 + r;
    const float bv = (bias && c < Cout) ? bias[c] : 0.0f;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[b][v] = bv;
  }

  if (rest) {
    const int64_t wtile = 1024;  // floats per (k, chunk, block) weight tile
    int k = __builtin_ctz(rest);
    rest &= rest - 1;
    int ch = 0;
    int src = nl[r * K + k];
    // the second half-wave of a 16-channel tail chunk has no input channels
    bool a_on = src >= 0 && (h == 0 || Cin - ch * 32 >= 32);
    Frag a_next = load_frag(a_on ? in + (int64_t)src * ld_in + ch * 32 + h * 16 : g_zero_row);
    Frag b_pref = load_frag(Wp + (((int64_t)k * nch + ch) * nbtp + cb0) * wtile + lane * 16);
    for (;;) {
      const Frag a_cur = a_next;
      bool has_next = true;
      int k2 = k, ch2 = ch + 1, src2 = src;
      if (ch2 == nch) {
        if (rest == 0) {
          has_next = false;
        } else {
          k2 = __builtin_ctz(rest);
          rest &= rest - 1;
          ch2 = 0;
          src2 = nl[r * K + k2];
        }
      }
      if (has_next) {
        a_on = src2 >= 0 && (h == 0 || Cin - ch2 * 32 >= 32);
        a_next = load_frag(a_on ? in + (int64_t)src2 * ld_in + ch2 * 32 + h * 16 : g_zero_row);
      }
#pragma unroll
      for (int b = 0; b < NB; b++) {
        const Frag b_cur = b_pref;
        if (b + 1 < NB)
          b_pref = load_frag(Wp + (((int64_t)k * nch + ch) * nbtp + cb0 + b + 1) * wtile + lane * 16);
        else if (has_next)
          b_pref = load_frag(Wp + (((int64_t)k2 * nch + ch2) * nbtp + cb0) * wtile + lane * 16);
#pragma unroll
        for (int s = 0; s < 16; s++)
          acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(a_cur, s), frag_at(b_cur, s), acc[b], 0, 0, 0);
      }
      if (!has_next) break;
      k = k2;
      ch = ch2;
      src = src2;
    }
  }

  // D layout of the 32x32 MFMA: lane holds column (lane & 31), rows 8*(v/4) + 4*(lane>>5) + (v&3)
#pragma unroll
  for (int v = 0; v < 16; v++) {
    const int i = 8 * (v >> 2) + 4 * h + (v & 3);
    const int rid = __shfl(my_row, i, 64);
    if (rid < 0) continue;
    float *op = out + (int64_t)rid * ld_out + cb0 * 32 + r;
#pragma unroll
    for (int b = 0; b < NB; b++)
      if ((cb0 + b) * 32 + r < Cout) op[b * 32] = acc[b][v];
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

static bool conv_uses_mfma(const float *in, int64_t ld_in, int Cin, int K) {
  return Cin % 16 == 0 && ((uintptr_t)in % 16 == 0) && (ld_in % 4 == 0) && K <= MAXK;
}

static int64_t packed_floats(int K, int Cin, int Cout) {
  return (int64_t)K * conv_nch(Cin) * conv_nbt_padded(Cout) * 1024;
}

static int pack_weights(const float *W, int K, int Cin, int Cout, float *Wp, hipStream_t s) {
  const int64_t total = packed_floats(K, Cin, Cout);
  hipLaunchKernelGGL(pack_weights_kernel, dim3(grid_for(total, 256, 4096)), dim3(256), 0, s, W, K, Cin, Cout,
                     conv_nch(Cin), conv_nbt_padded(Cout), Wp);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

// W: raw [K,Cin,Cout] weights (always needed by the generic kernel); Wp: packed weights or
// null, in which case they are packed into scratch memory first.
static int launch_conv(const float *in, int64_t ld_in, float *out, int64_t ld_out, const float *W, const float *Wp,
                       const float *bias, const int32_t *map0, const int32_t *map1, int mode, int K,
                       const int32_t *rows, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                       hipStream_t s) {
  if (n_rows == 0) return INSC_OK;
  if (conv_uses_mfma(in, ld_in, Cin, K)) {
    if (!Wp) {
      void *ws;
      int rc = workspace(WS_API, s, sizeof(float) * (size_t)packed_floats(K, Cin, Cout), &ws);
      if (rc) return rc;
      rc = pack_weights(W, K, Cin, Cout, (float *)ws, s);
      if (rc) return rc;
      Wp = (const float *)ws;
    }
    const int64_t tiles = cdiv(n_rows, TILE_M);
    const unsigned gx = (unsigned)cdiv(tiles, CONV_WAVES);
    const int NB = conv_nb_per_group(Cout), nbtp = conv_nbt_padded(Cout);
    dim3 grid(gx, (unsigned)(nbtp / NB)), block(CONV_WAVES * 64);
#define INSC_CONV_CASE(NBV)                                                                                      \
  case NBV:                                                                                                      \
    hipLaunchKernelGGL(conv_mfma_kernel<NBV>, grid, block, 0, s, in, ld_in, out, ld_out, Wp, bias, map0, map1,   \
                       mode, K, rows, d_n_rows, n_rows, Cin, Cout, nbtp);                                        \
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
    if (!W) {
      set_error("conv: this shape (Cin=%d) runs on the generic kernel, which needs the unpacked weights", Cin);
      return INSC_ERR_ARG;
    }
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

int64_t insc_conv_packed_floats(int K, int Cin, int Cout) {
  if (K <= 0 || Cin <= 0 || Cout <= 0) return 0;
  return packed_floats(K, Cin, Cout);
}

int insc_conv_pack_weights(const float *d_W, int K, int Cin, int Cout, float *d_Wp, void *stream) {
  INSC_REQUIRE(d_W && d_Wp && K > 0 && K <= MAXK && Cin > 0 && Cout > 0, INSC_ERR_ARG,
               "insc_conv_pack_weights: bad arguments");
  return pack_weights(d_W, K, Cin, Cout, d_Wp, (hipStream_t)stream);
}

int insc_conv_nbr(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_W,
                  const float *d_Wp, const float *d_bias, const int32_t *d_nbr, int K, const int32_t *d_rows,
                  const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout, double *h_muladds, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && Cin > 0 && Cout > 0 && K > 0 && K <= MAXK, INSC_ERR_ARG,
               "insc_conv_nbr: bad sizes (n_rows=%lld Cin=%d Cout=%d K=%d)", (long long)n_rows, Cin, Cout, K);
  INSC_REQUIRE(ld_in >= Cin && ld_out >= Cout, INSC_ERR_ARG, "insc_conv_nbr: row stride smaller than channel count");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && (d_W || d_Wp)), INSC_ERR_ARG, "insc_conv_nbr: null pointer");
  INSC_REQUIRE(d_nbr || K == 1, INSC_ERR_ARG, "insc_conv_nbr: a null map needs K == 1");
  hipStream_t s = (hipStream_t)stream;
  int rc = launch_conv(d_in, ld_in, d_out, ld_out, d_W, d_Wp, d_bias, d_nbr, nullptr,
                       d_nbr ? MAP_NBR : MAP_IDENTITY, K, d_rows, d_n_rows, n_rows, Cin, Cout, s);
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
                      const float *d_Wp, const float *d_bias, const int32_t *d_parent, const int32_t *d_offset,
                      const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                      void *stream) {
  INSC_REQUIRE(n_rows >= 0 && Cin > 0 && Cout > 0, INSC_ERR_ARG, "insc_deconv_down2: bad sizes");
  INSC_REQUIRE(ld_in >= Cin && ld_out >= Cout, INSC_ERR_ARG, "insc_deconv_down2: row stride too small");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && (d_W || d_Wp) && d_parent && d_offset), INSC_ERR_ARG,
               "insc_deconv_down2: null pointer");
  return launch_conv(d_in, ld_in, d_out, ld_out, d_W, d_Wp, d_bias, d_parent, d_offset, MAP_PARENT, 8, d_rows,
                     d_n_rows, n_rows, Cin, Cout, (hipStream_t)stream);
}

}  // extern "C"
