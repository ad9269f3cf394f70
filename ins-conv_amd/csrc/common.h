// Internal helpers shared by the HIP translation units of libinsc.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/insc.h"

namespace insc {

// ---- error reporting -------------------------------------------------------------------
void set_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what, const char *file, int line);

#define INSC_HIP(call)                                                        \
  do {                                                                        \
    hipError_t e__ = (call);                                                  \
    if (e__ != hipSuccess) return insc::hip_fail(e__, #call, __FILE__, __LINE__); \
  } while (0)

#define INSC_REQUIRE(cond, code, ...) \
  do {                                \
    if (!(cond)) {                    \
      insc::set_error(__VA_ARGS__);   \
      return (code);                  \
    }                                 \
  } while (0)

#define INSC_LAUNCH_CHECK() INSC_HIP(hipGetLastError())

// ---- per-stream scratch memory ---------------------------------------------------------
// Temporary device memory for scans, sorts and compactions.  One arena per (device, stream);
// it only ever grows, so steady-state calls allocate nothing.  Work using an arena is
// ordered by its stream.
// Arena 0 belongs to the scan primitive, arena 1 to the sort primitive, arena 2 to the
// API-level function that is running (none of which calls another arena-2 user; the convolution
// launcher packs weights there when the caller brings none), arena 5 to the residual-frame
// operators, which call that launcher, arena 6 to the flag and count words of
// insc_grid_insert_scales (whose helpers use arenas 0-2).
enum { WS_SCAN = 0, WS_SORT = 1, WS_API = 2, WS_CONV = 3, WS_LABELS = 4, WS_INCRE = 5, WS_INSERT = 6 };
int workspace(int which, hipStream_t stream, size_t bytes, void **out);
int device_cus();
// `count` int32 counters per (device, stream), zero at kernel start; users leave them at zero
int zero_counters(hipStream_t stream, size_t count, int32_t **out);

// ---- device primitives (scan_sort.hip) -------------------------------------------------
int sort_pairs_u64_into(uint64_t *keys, int32_t *vals_in, int32_t *vals_out, int64_t n, int key_bits, hipStream_t s);
int scan_exclusive_i32(const int32_t *in, int32_t *out, int64_t n, int32_t *total, hipStream_t s);
// Several sorts of the same key width in shared launches (two per 8-bit pass, whatever the number of
// jobs).  Per job: vals_out receives vals_in in key order and inv_out (nullable) the inverse,
// inv_out[vals_out[i]] = i (the values must then be a permutation of 0..n-1); keys and vals_in are scratch
// afterwards.  1 <= n <= SORT_BATCH_MAX_N per job.
struct SortJob {
  uint64_t *keys;
  int32_t *vals_in, *vals_out, *inv_out;
  int64_t n;
};
constexpr int SORT_BATCH_MAX_JOBS = 8;
constexpr int64_t SORT_BATCH_MAX_N = 262144;
int sort_pairs_u64_into_batch(const SortJob *jobs, int n_jobs, int key_bits, hipStream_t s);
int sort_pairs_u64(uint64_t *keys, int32_t *vals, int64_t n, int key_bits, hipStream_t s);

// ---- feature kernels shared with the network executor (conv.hip, pointwise.hip) ----------
enum { MAP_NBR = 0, MAP_IDENTITY = 1, MAP_PARENT = 2 };
// tile_flags: one byte per 32-row tile of `rows` (matrix-core kernel); row_mask: one byte per
// site (generic kernel and the streaming kernels).  Null = everything.
// Optional fused inference batch norm + leaky ReLU behind a producing kernel:
//   y = fmaf(x, w[c], b[c]); y *= (y > 0 ? 1 : leak)  ->  out2 (row stride ld2), out2 nullable
// w, b are the per-channel scale / shift (bn_scale_shift).  The producer still writes its raw
// result x to its own output unless that pointer is null.
struct BnEpilogue {
  const float *w = nullptr, *b = nullptr;
  float leak = 0.0f;
  float *out2 = nullptr;
  int64_t ld2 = 0;
  // optional residual: x = producer result + res[row][c] before anything is written (the
  // element-wise sum of a residual block, folded into the convolution that ends the block)
  const float *res = nullptr;
  int64_t ldr = 0;
  // optional second batch norm, over another matrix with the producer's rows and columns (the other
  // half of a channel concatenation whose batch norm this producer computes as well):
  //   side_out[row][c] = leaky(side_in[row][c] * side_w[c] + side_b[c]), row stride of side_out = ld2,
  // same leak.  Deconvolutions only (conv_mfma_kernel with the parent map).
  const float *side_in = nullptr;
  int64_t ld_side = 0;
  float *side_out = nullptr;
  const float *side_w = nullptr, *side_b = nullptr;
  // optional second source of a split launch (residual frames: the saved features join the frame's
  // own): a second set of blocks per (tile, output block) gathers from src2_in through src2_map
  // (in the place of map0; a parent map shares map1) with the same weights, and the sums of both
  // sets are added up in block order.  src2_rows: rows of src2_in.
  const float *src2_in = nullptr;
  int64_t src2_ld = 0, src2_rows = 0;
  const int32_t *src2_map = nullptr;
  // optional: the batch norm behind out2 is that of a residual frame (incre_bn_kernel, same
  // arithmetic): for a row whose site existed (pre_exist[row] = its saved row, or -1)
  //   out2 = leaky(w * pre_in[saved row] + (w * x + b)) - pre_out[saved row].
  // Split launches of 3^3 layers with latency != 0 only.
  const int32_t *pre_exist = nullptr;
  const float *pre_in = nullptr, *pre_out = nullptr;
  int64_t ld_pin = 0, ld_pout = 0;
};
// w = gamma / sqrt(var + eps), b = beta - mean * w   (gamma / beta nullable)
int bn_scale_shift(const float *mean, const float *var, const float *gamma, const float *beta, float eps, int C,
                   float *w, float *b, hipStream_t s);

// Tile plan of a 3^3 map for one processing order: map[k * ld + p] = neighbour k of the site at
// position p of the order (-1: none; positions up to the end of the last 32-row tile are
// filled), tmask[t] = offsets some row of tile t has.  Optional: kernels fall back to the
// site-indexed map.
struct TilePlan {
  const int32_t *map = nullptr;
  int64_t ld = 0;
  const uint32_t *tmask = nullptr;
  const int32_t *sched = nullptr;  // [ld / 32] tiles by falling cost, or null
  unsigned cus = 256;              // compute units of the device (launch_conv fills it in)
};
int build_tile_plan(const int32_t *nbr, const int32_t *order, const int32_t *d_n, int64_t n_rows, int64_t ld,
                    int32_t *map, uint32_t *tmask, int32_t *sched, hipStream_t s);
// the same for up to 16 maps in two launches (a map with n_rows == 0 is skipped)
struct TilePlanJob {
  const int32_t *nbr, *order, *d_n;
  int64_t n_rows, ld;
  int32_t *map;
  uint32_t *tmask;
  int32_t *sched;
};
struct TilePlanBatch {
  TilePlanJob job[16];
  int n;
};
// (a job with nbr == null keeps its map and only has its schedule rebuilt)
int build_tile_plans(const TilePlanBatch &b, hipStream_t s);
// the columns of the sites added by the last insert (positions from d_n[1] on), for plans whose
// older part is up to date; a job with map == null is skipped
int tile_plan_append_batch(const TilePlanBatch &b, int64_t n_new_upper, hipStream_t s);

// in_rows: rows of the input matrix (bounds the gather).  out may be null when ep.out2 is set.
// latency != 0 picks the launch shape for small row counts (residual frames).
// expect_rows (0: n_rows): how many rows the launch will probably find in *d_n_rows, when that is
// far below the bound n_rows - it only picks among kernels that give the same bits.
int launch_conv(const float *in, int64_t ld_in, int64_t in_rows, float *out, int64_t ld_out, const float *W,
                const float *Wp, const float *bias, const int32_t *map0, const int32_t *map1, int mode, int K,
                const int32_t *rows, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                const uint8_t *tile_flags, const uint8_t *row_mask, hipStream_t s, BnEpilogue ep = BnEpilogue(),
                TilePlan plan = TilePlan(), int latency = 0, int64_t expect_rows = 0);
// whether launch_conv takes a second source (BnEpilogue::src2_*) for this shape
bool conv_two_sources_ok(int mode, int K, const float *in, int64_t ld_in, const float *in2, int64_t ld_in2,
                         int64_t in2_rows, int Cin, int latency);
int64_t packed_floats(int K, int Cin, int Cout);
int pack_weights(const float *W, int K, int Cin, int Cout, float *Wp, hipStream_t s);
int launch_bn(const float *in, int64_t ld_in, float *out, int64_t ld_out, const float *mean, const float *var,
              const float *gamma, const float *beta, float eps, float leak, const int32_t *rows,
              const int32_t *d_n_rows, int64_t n_rows, int C, const uint8_t *row_mask, hipStream_t s);
// out = a + b (b != null) or out = a
int launch_add(const float *a, int64_t ld_a, const float *b, int64_t ld_b, float *out, int64_t ld_out,
               const int32_t *rows, const int32_t *d_n_rows, int64_t n_rows, int C, const uint8_t *row_mask,
               hipStream_t s, BnEpilogue ep = BnEpilogue());
// batch norm of a residual frame (incre.hip); w, b: precomputed scale / shift or null
int launch_incre_bn(const float *in, int64_t ld_in, float *out, int64_t ld_out, const float *mean, const float *var,
                    const float *gamma, const float *beta, float eps, float leak, const float *w, const float *b,
                    const int32_t *pre_exist, const float *pre_in, int64_t ld_pin, const float *pre_out,
                    int64_t ld_pout, int64_t n, int C, hipStream_t s);
// the two convolutions of a residual frame (incre.hip; insc_incre_conv_ssc / insc_incre_deconv_down2
// with an optional element-wise sum: out = result + res; the 3^3 one also takes the batch norm of
// a residual frame in ep where conv_two_sources_ok says that it runs as one launch)
int incre_conv_ssc(const float *in, int64_t ld_in, const float *pre_in, int64_t ld_pre, int64_t n_pre_rows, float *out,
                   int64_t ld_out, const float *W, const float *Wp, const float *bias, const int32_t *nbr,
                   const int32_t *nbr_pre, int64_t n, int Cin, int Cout, BnEpilogue ep, hipStream_t s);
int incre_deconv_down2(const float *in, int64_t ld_in, int64_t n_in_rows, const float *pre_in, int64_t ld_pre,
                       int64_t n_pre_rows, float *out, int64_t ld_out, const float *W, const float *Wp,
                       const float *bias, const int32_t *parent, const int32_t *offset, const int32_t *pre_exist_in,
                       const int32_t *pre_exist_out, int64_t n_rows, int Cin, int Cout, const float *res, int64_t ldr,
                       hipStream_t s, const int32_t *parent2 = nullptr);  // parent2: incre_parent_kernel's answer, if at hand
int launch_input_finish(const float *sum, const int32_t *cnt, int mode, float *out, int64_t ld_out,
                        const int32_t *rows, const int32_t *d_n_rows, int64_t n_rows, int C,
                        const uint8_t *row_mask, hipStream_t s);

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline unsigned grid_for(int64_t n, int block, int64_t cap = 1 << 20) {
  int64_t g = cdiv(n, block);
  if (g < 1) g = 1;
  if (g > cap) g = cap;
  return (unsigned)g;
}

// ---- device helpers shared by the streaming kernels ------------------------------------
__device__ __forceinline__ float leaky(float o, float leak) { return o * ((o > 0.0f) ? 1.0f : leak); }
// a - b as a subtraction of its own, never contracted with the product that formed a (two code
// sites that must give the same bits use it)
__device__ __forceinline__ float sub_exact(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

// per-channel scale / shift of inference batch norm; every kernel that normalises goes through
// this one function so that fused and unfused paths give the same bits
__device__ __forceinline__ void bn_coeffs(const float *__restrict__ mean, const float *__restrict__ var,
                                          const float *__restrict__ gamma, const float *__restrict__ beta, float eps,
                                          int c, float &w, float &b) {
  const float invstd = 1.0f / sqrtf(var[c] + eps);
  w = invstd * (gamma ? gamma[c] : 1.0f);
  b = fmaf(-mean[c], w, beta ? beta[c] : 0.0f);
}

// ---- key packing ------------------------------------------------------------------------
// 64-bit voxel key: batch:16 | z:16 | y:16 | x:16.  Ascending key order is (batch, z, y, x).
#define INSC_EMPTY_KEY 0xFFFFFFFFFFFFFFFFull

__host__ __device__ static inline bool coord_ok(int x, int y, int z, int b) {
  return ((unsigned)x | (unsigned)y | (unsigned)z) < 65536u && (unsigned)b < 32768u;
}
__host__ __device__ static inline uint64_t pack_key(int x, int y, int z, int b) {
  return ((uint64_t)(unsigned)b << 48) | ((uint64_t)(unsigned)z << 32) | ((uint64_t)(unsigned)y << 16) |
         (uint64_t)(unsigned)x;
}

}  // namespace insc
