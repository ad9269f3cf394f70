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
#include <algorithm>

#include "common.h"

#include <atomic>

namespace insc {

typedef float f16v __attribute__((ext_vector_type(16)));


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
                                                           int Cin, int Cout,
                                                           const uint8_t *__restrict__ row_mask, BnEpilogue ep) {
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int cpb = 256 / Cout > 0 ? 256 / Cout : 1;  // rows per block (Cout <= 256)
  const int lr = threadIdx.x / Cout, co = threadIdx.x % Cout;
  if (lr >= cpb) return;
  for (int64_t t = (int64_t)blockIdx.x * cpb + lr; t < n; t += (int64_t)gridDim.x * cpb) {
    const int row = rows ? rows[t] : (int)t;
    if (row < 0 || (row_mask && !row_mask[row])) continue;
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
    if (ep.res) acc += ep.res[(int64_t)row * ep.ldr + co];
    if (out) out[(int64_t)row * ld_out + co] = acc;
    if (ep.out2) {
      const float y = fmaf(acc, ep.w[co], ep.b[co]);
      ep.out2[(int64_t)row * ep.ld2 + co] = y * ((y > 0.0f) ? 1.0f : ep.leak);
    }
  }
}

// ---------------------------------------------------------------------------------------
// 3^3 layers with 1..4 input channels (the RGB stem of a U-Net): same thread layout - a thread per (row,
// output channel) - and the same order of operations as the generic kernel (so the same bits), but the
// 27 x CIN weights of a thread's output channel stay in registers over all its rows, and the neighbour ids
// and input values of a batch of rows are fetched once per block, one (row, offset) per thread, and read
// back from LDS by the threads of the row (one 16-byte broadcast read per offset): with every thread
// fetching its row's 27 ids and 81 values itself the kernel was bound by the number of load instructions
// (92 us for 150k rows and 32 output channels).
// ---------------------------------------------------------------------------------------
constexpr int STEM_ROWS = 16;  // rows per batch at most (those of 256 / Cout rows that a block handles at a time)
template <int CIN>
__global__ __launch_bounds__(256) void conv_stem_kernel(const float *__restrict__ in, int64_t ld_in,
                                                        float *__restrict__ out, int64_t ld_out,
                                                        const float *__restrict__ W, const float *__restrict__ bias,
                                                        const int32_t *__restrict__ map0,
                                                        const int32_t *__restrict__ rows,
                                                        const int32_t *__restrict__ d_n_rows, int64_t n_rows,
                                                        int Cout, const uint8_t *__restrict__ row_mask,
                                                        BnEpilogue ep) {
  constexpr int K = 27;
  __shared__ float4 xs[2][STEM_ROWS][K];  // input values of (row, offset); two batches in turn
  __shared__ int vs[2][STEM_ROWS][K];     // 1: the row has a neighbour at the offset
  __shared__ int rid[2][STEM_ROWS];       // row of the batch, -1: none
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int cpb = min(256 / Cout, STEM_ROWS);  // rows per batch (Cout <= 256)
  const int lr = threadIdx.x / Cout, co = threadIdx.x % Cout;
  const bool worker = lr < cpb;
  float w[K][CIN];
#pragma unroll
  for (int k = 0; k < K; k++)
#pragma unroll
    for (int ci = 0; ci < CIN; ci++) w[k][ci] = worker ? W[((int64_t)k * CIN + ci) * Cout + co] : 0.0f;
  const float bv = (bias && worker) ? bias[co] : 0.0f;
  const float ew = (ep.out2 && worker) ? ep.w[co] : 0.0f, eb = (ep.out2 && worker) ? ep.b[co] : 0.0f;
  int buf = 0;
  for (int64_t t0 = (int64_t)blockIdx.x * cpb; t0 < n; t0 += (int64_t)gridDim.x * cpb, buf ^= 1) {
    // fetch: one (row, offset) per thread
    for (int e = threadIdx.x; e < cpb * K; e += 256) {
      const int er = e / K, k = e - er * K;
      const int64_t t = t0 + er;
      int row = t < n ? (rows ? rows[t] : (int)t) : -1;
      if (row >= 0 && row_mask && !row_mask[row]) row = -1;
      const int src = row >= 0 ? map0[(int64_t)row * K + k] : -1;
      float x[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (src >= 0) {
        const float *p = in + (int64_t)src * ld_in;
#pragma unroll
        for (int ci = 0; ci < CIN; ci++) x[ci] = p[ci];
      }
      xs[buf][er][k] = make_float4(x[0], x[1], x[2], x[3]);
      vs[buf][er][k] = src >= 0 ? 1 : 0;
      if (k == 0) rid[buf][er] = row;
    }
    __syncthreads();  // (one barrier per batch: the next batch fills the other buffer)
    const int row = worker ? rid[buf][lr] : -1;
    if (row < 0) continue;
    float acc = bv;
#pragma unroll
    for (int k = 0; k < K; k++) {
      const float4 xv = xs[buf][lr][k];
      const float x[4] = {xv.x, xv.y, xv.z, xv.w};
      float a = acc;
#pragma unroll
      for (int ci = 0; ci < CIN; ci++) a = fmaf(x[ci], w[k][ci], a);
      acc = vs[buf][lr][k] ? a : acc;
    }
    if (ep.res) acc += ep.res[(int64_t)row * ep.ldr + co];
    if (out) out[(int64_t)row * ld_out + co] = acc;
    if (ep.out2) {
      const float y = fmaf(acc, ew, eb);
      ep.out2[(int64_t)row * ep.ld2 + co] = y * ((y > 0.0f) ? 1.0f : ep.leak);
    }
  }
}

// ---------------------------------------------------------------------------------------
// Weight packing.  For filter offset k, input-channel chunk ch (32 channels) and
// output-channel block nb (32 channels), lane = h*32 + j of the MFMA kernel needs the 16
// B-operand values W[k][ch*32 + h*16 + s][nb*32 + j], s = 0..15.  The 4 KB tile is stored as
// four 1 KB quarters; quarter q holds, for lane 0..63 in turn, the values s = 4q..4q+3.  One
// 16-byte load per lane then reads a quarter fully coalesced.  Channels beyond Cin / Cout
// are zero.
// ---------------------------------------------------------------------------------------
__host__ __device__ static inline int conv_nch(int Cin) { return (Cin + 31) / 32; }
static inline int conv_nb_per_group(int Cout) {
  const int nbt = (Cout + 31) / 32;
  return nbt > 4 ? 4 : nbt;
}
static inline int conv_nbt_padded(int Cout) {
  const int nbt = (Cout + 31) / 32, nb = conv_nb_per_group(Cout);
  return (int)cdiv(nbt, nb) * nb;
}

__global__ void pack_weights_kernel(const float *__restrict__ W, int K, int Cin, int Cout, int nch, int nbtp,
                                    float *__restrict__ Wp) {
  const int64_t total = (int64_t)K * nch * nbtp * 1024;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int s = (int)(((e >> 8) & 3) * 4 + (e & 3)), lane = (int)((e >> 2) & 63);
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

__device__ __forceinline__ float frag_at(const Frag &f, int s) {
  const float4 v = f.q[s >> 2];
  return (s & 3) == 0 ? v.x : (s & 3) == 1 ? v.y : (s & 3) == 2 ? v.z : v.w;
}

// Gather: every lane reads the 64 bytes of its own input row that the MFMA A operand needs, with
// buffer loads: one 32-bit offset per item, rows without a neighbour get an out-of-range offset
// and the hardware returns zeros, and the weight tile is addressed by a scalar offset - a
// handful of non-MFMA instructions per 16 MFMAs (ordinary VALU work does not overlap with MFMAs
// on this part, so it is paid in matrix-core time).
// Items in flight per wavefront (ring depth): whole-tile wavefronts, and wavefronts that share a
// tile.  (For the latter a ring of four measured 4-10 % slower than one of two at every scale of the
// U-Net: with 91 instead of 140 registers more wavefronts fit a SIMD, and a turn of the unrolled loop
// wastes fewer steps past a wavefront's last item.)
#ifndef INSC_CONV_DEPTH
#define INSC_CONV_DEPTH 2
#endif
#ifndef INSC_CONV_DEPTH_SPLIT
#define INSC_CONV_DEPTH_SPLIT 2
#endif

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// offsets at or beyond this bound make a buffer load return zeros
constexpr uint32_t BUF_OOB = 0xFFFFF000u;  // room for the per-load immediate on top

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
}

// S == 1: every wavefront of the block owns a tile and walks all of its filter offsets.
// S  > 1: the S wavefronts of a block share ONE tile; the (offset, channel chunk) items are dealt
//         out round robin and the partial sums are added in wavefront order at the end.  This is for
//         the coarse scales of a U-Net, where a layer has a handful of tiles but hundreds of
//         channels and a single wavefront would run tens of thousands of dependent MFMAs.  Which
//         terms a wavefront sums depends on k only, so a row's result is a function of S alone
//         (S is a fixed property of the layer shape), never of the tile it happens to sit in.
//         With gridDim.z = G > 1 the deal goes over S * G wavefronts in G blocks (different
//         compute units): a coarse scale has so few tiles that the matrix cores of the few
//         units holding them would bound the layer.
template <int NB, int K, int MODE, int S>
__global__ __launch_bounds__((S == 1 ? CONV_WAVES : S) * 64) void conv_mfma_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ Wp, const float *__restrict__ bias, const int32_t *__restrict__ map0,
    const int32_t *__restrict__ map1, const int32_t *__restrict__ rows,
    const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout, int nbtp,
    const uint8_t *__restrict__ tile_flags, uint32_t in_bytes, uint32_t wp_bytes, BnEpilogue ep,
    float *__restrict__ part, int32_t *__restrict__ pcount, TilePlan plan) {
  static_assert(S == 1 || NB == 1, "split tiles use one output block per wavefront");
  constexpr int WAVES = S == 1 ? CONV_WAVES : S;
  __shared__ int nbl[S == 1 ? WAVES : 1][TILE_M * K];
  __shared__ float red[S > 1 ? S : 1][S > 1 ? 16 * 64 : 1];  // (slot S - 1: only when all wavefronts share the tail)
  __shared__ unsigned wmask[S];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  // (the wavefront's number as a scalar: the item cursor below then runs on the scalar unit)
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  // (with a tile schedule the blocks of a split launch take the tiles by falling cost: blocks go to the
  // compute units round robin, so every unit then holds a mix of expensive and cheap tiles)
  // Which (tile slot, output block, share of the split) this block works on.  Split launches with a
  // tile schedule renumber their blocks: the hardware hands out blocks in the order x, y, z, round robin
  // over the compute units, so block L goes - all blocks being resident at once - to unit L mod CUS.
  // Ranked by cost (tile slot major: the output blocks and shares of a tile cost the same), the first CUS
  // blocks take ranks in order, the next CUS in reverse order and so on in turns, so that the compute unit
  // that drew the most expensive block of one turn gets the cheapest of the next.
  unsigned bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  if (S > 1 && MODE == MAP_NBR && K == 27 && plan.map != nullptr && plan.sched != nullptr) {
    const unsigned CUS = plan.cus;
    const unsigned gyz = gridDim.y * gridDim.z;
    const unsigned total = (unsigned)((n + TILE_M - 1) / TILE_M) * gyz;
    const unsigned L = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    if (L >= total) return;  // (launches are sized by an upper bound of the row count)
    const unsigned rnd = L / CUS, pos = L % CUS, m = min(CUS, total - rnd * CUS);
    const unsigned R = rnd * CUS + ((rnd & 1u) ? m - 1 - pos : pos);
    bx = R / gyz;
    const unsigned rem = R - bx * gyz;
    by = rem / gridDim.z;
    bz = rem - by * gridDim.z;
  }
  const int64_t slot = S == 1 ? (int64_t)bx * WAVES + wave : (int64_t)bx;
  const bool by_cost = MODE == MAP_NBR && K == 27 && plan.map != nullptr && plan.sched != nullptr && slot * TILE_M < n;
  const int64_t t0 = (by_cost ? (int64_t)plan.sched[slot] : slot) * TILE_M;
  const int cb0 = by * NB;  // first output-channel block of this column group
  const int nch = conv_nch(Cin);
  // the items of a tile are dealt to S wavefronts in each of G blocks; gridDim.z = GZ holds G blocks
  // per source (two sources: the blocks from G on gather from the second one, through its own map)
  const int GZ = S == 1 ? 1 : (int)gridDim.z;
  const bool second = S > 1 && ep.src2_in != nullptr && (int)bz >= GZ / 2;
  const int G = (S > 1 && ep.src2_in != nullptr) ? GZ / 2 : GZ, ST = S * G;
  const int ws = wave * G + (S == 1 ? 0 : (int)bz - (second ? G : 0));
  if (second) {
    in = ep.src2_in;
    ld_in = ep.src2_ld;
    in_bytes = (uint32_t)(ep.src2_rows * ep.src2_ld * 4);
    map0 = ep.src2_map;
    bias = nullptr;
  }

  // blocks beyond the row count leave at once (launches are sized by an upper bound of it)
  if ((S == 1 ? (int64_t)bx * WAVES : (int64_t)bx) * TILE_M >= n) return;
  // a tile is skipped when it lies beyond the row count or, with tile flags, is not marked
  const bool live = t0 < n && (!tile_flags || tile_flags[t0 >> 5]);
  int my_row = -1;
  if (live && t0 + r < n) my_row = rows ? rows[t0 + r] : (int)(t0 + r);
  // (residual-frame batch norm in the epilogue: the saved row of this lane's row, asked for here so
  // that the main loop hides the load)
  int my_pe = -1;
  if (S > 1 && ep.pre_exist && my_row >= 0) my_pe = ep.pre_exist[my_row];

  // stage the tile's slice of the neighbour map in LDS and find the offsets it uses; all the
  // loads are issued before the first one is consumed.  With a tile plan (the map transposed into
  // processing order, one 128-byte run per (offset, tile), and the offsets of every tile) the
  // loads are coalesced, need no row id and the LDS copy is offset-major.
  const bool planned = MODE == MAP_NBR && K == 27 && plan.map != nullptr;
  int *nl = nbl[S == 1 ? wave : 0];
  unsigned mymask = 0;
  constexpr int NSTAGE = (TILE_M * K + 64 * S - 1) / (64 * S);
  int staged[NSTAGE];
  if (planned) {
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = (S == 1 ? i : i * S + wave) * 64 + lane;  // e = k * 32 + row
      staged[i] = (live && e < TILE_M * K) ? plan.map[(int64_t)(e >> 5) * plan.ld + t0 + (e & 31)] : -1;
    }
    if (live) mymask = plan.tmask[t0 >> 5];
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = (S == 1 ? i : i * S + wave) * 64 + lane;
      if (e < TILE_M * K) nl[e] = staged[i];
    }
  } else {
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = (S == 1 ? i : i * S + wave) * 64 + lane;
      const int rr = e / K, kk = e - rr * K;
      const int rid = __shfl(my_row, rr & (TILE_M - 1), 64);
      int v = -1;
      if (e < TILE_M * K && rid >= 0) {
        if (MODE == MAP_NBR)
          v = map0[(int64_t)rid * K + kk];
        else if (MODE == MAP_IDENTITY)
          v = rid;
        else
          v = (map1[rid] == kk) ? map0[rid] : -1;
      }
      staged[i] = v;
    }
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = (S == 1 ? i : i * S + wave) * 64 + lane;
      if (e < TILE_M * K) {
        nl[e] = staged[i];
        if (staged[i] >= 0) mymask |= 1u << (e % K);
      }
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) mymask |= (unsigned)__shfl_xor((int)mymask, d, 64);
  }
  if (S > 1 && lane == 0) wmask[wave] = mymask;
  __syncthreads();
  if (!live) return;  // the whole block (S > 1) or wavefront (S == 1) is idle; no barrier follows
  // Split launches: what the tail of this wavefront will read besides the sums - the other operand of a
  // folded element-wise sum, the saved rows of a residual frame's batch norm - is asked for here, for
  // the rows the wavefront finishes, so that the main loop hides these loads.
  constexpr int NVP = S > 1 ? 16 / S : 1;
  float pre_res[NVP], pre_pin[NVP], pre_pout[NVP];
  int pre_pe[NVP];
  if (S > 1) {
    const int c = cb0 * 32 + r;
#pragma unroll
    for (int j = 0; j < NVP; j++) {
      const int v = wave * NVP + j, src_lane = 8 * (v >> 2) + 4 * h + (v & 3);
      const int row = __shfl(my_row, src_lane, 64);
      pre_pe[j] = __shfl(my_pe, src_lane, 64);
      pre_res[j] = (ep.res && row >= 0 && c < Cout) ? ep.res[(int64_t)row * ep.ldr + c] : 0.0f;
      const bool sv = pre_pe[j] >= 0 && c < Cout;
      pre_pin[j] = sv ? ep.pre_in[(int64_t)pre_pe[j] * ep.ld_pin + c] : 0.0f;
      pre_pout[j] = sv ? ep.pre_out[(int64_t)pre_pe[j] * ep.ld_pout + c] : 0.0f;
    }
  }
  // Offsets some row of the tile uses.  With S wavefronts per tile, the (offset k, chunk ch)
  // items are dealt out by (k * nch + ch) % S: wavefront w takes, of offset k, the chunks
  // ch0(k), ch0(k) + S, ... with ch0(k) = (w - k * nch) mod S.  The deal depends on k, ch and
  // the layer shape only, so a row's sum is formed the same way whatever tile it sits in.
  unsigned rest;  // offsets that hold at least one item of this wavefront
  int nitems = 0;
  if (S == 1) {
    rest = (unsigned)__builtin_amdgcn_readfirstlane((int)mymask);
    nitems = __builtin_popcount(rest) * nch;
  } else {
    unsigned act = 0;
#pragma unroll
    for (int w = 0; w < S; w++) act |= wmask[w];
    act = (unsigned)__builtin_amdgcn_readfirstlane((int)act);
    // (lane k looks at offset k: one ballot and a sum over the lanes instead of a scalar loop over the offsets)
    const int c0 = (ws - lane * nch) & (ST - 1);
    const bool has = lane < K && ((act >> (lane & 31)) & 1u) && c0 < nch;
    rest = (unsigned)__ballot(has);
    int cnt = has ? (nch - c0 + ST - 1) >> __builtin_ctz(ST) : 0;
#pragma unroll
    for (int d = 16; d > 0; d >>= 1) cnt += __shfl_xor(cnt, d, 64);
    nitems = __builtin_amdgcn_readfirstlane(cnt);
  }

  f16v acc[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) {
    const int c = (cb0 + b) * 32 + r;
    const float bv = (bias && c < Cout && (S == 1 || ws == 0)) ? bias[c] : 0.0f;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[b][v] = bv;
  }

  // per-channel scale / shift of the fused batch norm for this lane's columns (loaded here so
  // that the latency is hidden behind the main loop)
  float ew[NB], eb[NB], sw[NB], sb[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) {
    const int c = (cb0 + b) * 32 + r;
    const bool on = ep.out2 && c < Cout;
    ew[b] = on ? ep.w[c] : 0.0f;
    eb[b] = on ? ep.b[c] : 0.0f;
    const bool son = MODE == MAP_PARENT && ep.side_in && c < Cout;
    sw[b] = son ? ep.side_w[c] : 0.0f;
    sb[b] = son ? ep.side_b[c] : 0.0f;
  }

  if (rest) {
    // Work items of this tile: (active offset k, 32-channel chunk ch), offsets ascending, chunks
    // inside.  A cursor walks them with scalar selects only (no branches: a branchy iterator
    // splits the loop body into many blocks and the load/MFMA overlap below is lost).  Past the
    // last item it yields k = -1, and loads for such an item are sent out of range: they
    // return zeros and move no data.
    struct Cursor {
      int k, ch;
      unsigned rest;
    };
    auto ch0 = [&](int k) -> int { return S == 1 ? 0 : ((ws - k * nch) & (ST - 1)); };
    auto step = [&](const Cursor &c) -> Cursor {
      const bool wrap = c.ch + ST >= nch;
      const int nk = c.rest ? __builtin_ctz(c.rest) : -1;
      Cursor n;
      n.ch = wrap ? ch0(nk) : c.ch + ST;
      n.k = wrap ? nk : c.k;
      n.rest = wrap ? (c.rest & (c.rest - 1)) : c.rest;
      return n;
    };
    Cursor first;
    first.k = __builtin_ctz(rest);
    first.ch = ch0(first.k);
    first.rest = rest & (rest - 1);

    const __amdgpu_buffer_rsrc_t rin = make_rsrc(in, in_bytes), rw = make_rsrc(Wp, wp_bytes);
    const uint32_t ld4 = (uint32_t)ld_in * 4u, lane16 = (uint32_t)lane * 16u;
    // lane (r, h) reads channels ch*32 + h*16 .. +15 of its own row; the second half-wave of a
    // 16-channel tail chunk has no channels
    auto gather = [&](const Cursor &c) -> Frag {
      const int kk = c.k < 0 ? 0 : c.k;
      const int src = nl[planned ? kk * TILE_M + r : r * K + kk];
      const bool on = c.k >= 0 && src >= 0 && (h == 0 || Cin - c.ch * 32 >= 32);
      const uint32_t voff = on ? (uint32_t)src * ld4 + (uint32_t)(c.ch * 128 + h * 64) : BUF_OOB;
      Frag f;
#pragma unroll
      for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rin, voff + 16u * q, 0);
      return f;
    };
    auto wload = [&](const Cursor &c, int b) -> Frag {
      const int tile = ((c.k < 0 ? 0 : c.k) * nch + c.ch) * nbtp + cb0 + b;
      const uint32_t soff = (uint32_t)__builtin_amdgcn_readfirstlane(tile * 4096);
      const uint32_t voff = c.k >= 0 ? lane16 : BUF_OOB;
      Frag f;
#pragma unroll
      for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rw, voff + 1024u * q, soff);
      return f;
    };

    // Pipeline: while item t runs on the matrix cores, the gathers of items t+1 .. t+D-1 are in
    // flight; so are their weight tiles when a wavefront owns a single output block (otherwise
    // the weight tiles of the (item, block) sequence are fetched one step ahead).  Register
    // slots are compile-time (the body is unrolled over a full turn of the rings) because
    // copying a fragment would wait for the load that fills it.  Every load is issued
    // unconditionally: a load under a branch would force the wait before the MFMAs to drain
    // all outstanding loads.  The sched_barrier / memory-clobber pairs keep the loads above the
    // MFMAs they overlap and their consumers below.
    constexpr int D = (S == 1 || S >= 16) ? INSC_CONV_DEPTH : INSC_CONV_DEPTH_SPLIT;
    constexpr bool WRING = NB == 1;                         // weight tiles ride in the same ring
    constexpr int TURN = (WRING || NB % 2 == 0) ? D : (D % 2 == 0 ? D : 2 * D);
    Frag g[D], bw[WRING ? D : 2];
    Cursor ci = first;  // next item to issue
#pragma unroll
    for (int d = 0; d < D - 1; d++) {
      g[d] = gather(ci);
      if constexpr (WRING) bw[d] = wload(ci, 0);
      ci = step(ci);
    }
    Cursor c0 = first, c1 = step(first);  // item on the matrix cores and its successor
    if constexpr (!WRING) bw[0] = wload(c0, 0);
    // One loop turn = TURN items; the last turn may run past the last item: those steps issue
    // out-of-range loads and skip their MFMAs (a uniform branch around the MFMAs only).
    for (int t0i = 0; t0i < nitems; t0i += TURN) {
#pragma unroll
      for (int u = 0; u < TURN; u++) {
        g[(u + D - 1) % D] = gather(ci);
        if constexpr (WRING) bw[(u + D - 1) % D] = wload(ci, 0);
        ci = step(ci);
        const bool real = t0i + u < nitems;
#pragma unroll
        for (int b = 0; b < NB; b++) {
          const int nn = u * NB + b;
          if constexpr (!WRING) bw[(nn + 1) % 2] = (b + 1 < NB) ? wload(c0, b + 1) : wload(c1, 0);
          asm volatile("" ::: "memory");
          __builtin_amdgcn_sched_barrier(0);
          const Frag &bf = bw[WRING ? u % D : nn % 2];
          if (real) {
#pragma unroll
            for (int s = 0; s < 16; s++)
              acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[u % D], s), frag_at(bf, s), acc[b], 0, 0, 0);
          }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        c0 = c1;
        c1 = step(c1);
      }
    }
  }

  if (S > 1) {
    // Every wavefront leaves its partial sum in LDS; each then adds up - in wavefront order - and
    // finishes 16 / S of the rows of the tile, so that the tail of the block (partial sums through
    // memory, residual loads, two stores per row with a fused batch norm) is shared by all of them.
    // D layout of the 32x32 MFMA: lane holds column (lane & 31), rows 8*(v/4) + 4*(lane>>5) + (v&3).
    constexpr int NV = 16 / (S > 1 ? S : 16);
#pragma unroll
    for (int v = 0; v < 16; v++) red[wave][v * 64 + lane] = acc[0][v];
    __syncthreads();
    float a[NV];
    int rid[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int v = wave * NV + j;
      a[j] = red[0][v * 64 + lane];
#pragma unroll
      for (int w = 1; w < S; w++) a[j] += red[w][v * 64 + lane];
      rid[j] = __shfl(my_row, 8 * (v >> 2) + 4 * h + (v & 3), 64);
    }
    if (GZ > 1) {
      // The blocks of a (tile, output block) leave their sums in memory; of the wavefronts that
      // hold the same rows, the one that arrives last adds the sums in block order (so the result
      // does not depend on the arrival order), writes the rows and puts the arrival counter back to
      // zero.  Nobody waits for anybody.
      // (stores and loads of the sums go past the XCD-local L2 - device-scope atomics - so that no
      // cache write-back or invalidation is needed: a full fence flushes the whole L2 and costs
      // more than the layer)
      // Why the last arrival sees every sum.  (1) The sums are written with agent-scope atomic stores:
      // on this part such a store is not kept in the writer's XCD-local L2 but written through to the
      // level all XCDs share, and it is acknowledged from there.  (2) vmcnt(0) makes the wavefront wait
      // for those acknowledgements before it issues the counter's read-modify-write, which is performed
      // at that same shared level: a wavefront's increment is ordered after its own sums.  (3) The
      // wavefront that reads GZ - 1 back has therefore been preceded by all other increments, hence by
      // all other sums.  (4) Its loads below are issued only after that value has returned (the branch
      // depends on it; wavefronts issue in order) and are agent-scope atomic loads, which do not hit a
      // stale line of the reader's own L2.  The compiler fences pin the program order this relies on
      // (they emit no instructions).  An acquire/release pair at agent scope would say the same in the
      // language's terms but writes back and invalidates the whole L2.
      const int unit = (int)(bx * gridDim.y + by);
      float *mine = part + ((int64_t)unit * GZ + bz) * 1024 + (wave * NV) * 64 + lane;
#pragma unroll
      for (int j = 0; j < NV; j++) __hip_atomic_store(mine + j * 64, a[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the stores have been acknowledged
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
      int old = 0;
      if (lane == 0) old = atomicAdd(pcount + unit * S + wave, 1);
      if (__builtin_amdgcn_readfirstlane(old) != GZ - 1) return;
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
      const float *all = part + (int64_t)unit * GZ * 1024 + (wave * NV) * 64 + lane;
      // (the sums of eight blocks at a time are requested together and added in block order: one trip
      // to memory per eight blocks instead of one per block)
      constexpr int GP = 8;
      for (int g0 = 0; g0 < GZ; g0 += GP) {
        float pv[GP][NV];
#pragma unroll
        for (int gg = 0; gg < GP; gg++) {
          if (g0 + gg < GZ) {
#pragma unroll
            for (int j = 0; j < NV; j++)
              pv[gg][j] = __hip_atomic_load(all + (g0 + gg) * 1024 + j * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
#pragma unroll
        for (int gg = 0; gg < GP; gg++) {
          if (g0 + gg < GZ) {
#pragma unroll
            for (int j = 0; j < NV; j++) a[j] = (g0 + gg == 0) ? pv[0][j] : a[j] + pv[gg][j];
          }
        }
      }
      if (lane == 0) pcount[unit * S + wave] = 0;
    }
    const int c = cb0 * 32 + r;
    if (c >= Cout) return;
    if (ep.res) {
#pragma unroll
      for (int j = 0; j < NV; j++) a[j] += pre_res[j];
    }
    float sv[NV];
    if (MODE == MAP_PARENT && ep.side_in) {
#pragma unroll
      for (int j = 0; j < NV; j++) sv[j] = rid[j] >= 0 ? ep.side_in[(int64_t)rid[j] * ep.ld_side + c] : 0.0f;
      __builtin_amdgcn_sched_barrier(0);  // (all loads above the stores)
    }
    if (MODE == MAP_NBR && K == 27 && ep.pre_exist && ep.out2) {
      // batch norm of a residual frame, with the saved input and output of the rows that existed
#pragma unroll
      for (int j = 0; j < NV; j++) {
        if (rid[j] < 0) continue;
        if (out) out[(int64_t)rid[j] * ld_out + c] = a[j];
        const float o = fmaf(a[j], ew[0], eb[0]);
        const float y =
            pre_pe[j] >= 0 ? sub_exact(leaky(fmaf(pre_pin[j], ew[0], o), ep.leak), pre_pout[j]) : leaky(o, ep.leak);
        ep.out2[(int64_t)rid[j] * ep.ld2 + c] = y;
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < NV; j++) {
      if (rid[j] < 0) continue;
      if (out) out[(int64_t)rid[j] * ld_out + c] = a[j];
      if (ep.out2) {
        const float y = fmaf(a[j], ew[0], eb[0]);  // fused batch norm + leaky ReLU
        ep.out2[(int64_t)rid[j] * ep.ld2 + c] = y * ((y > 0.0f) ? 1.0f : ep.leak);
      }
      if (MODE == MAP_PARENT && ep.side_in) {
        const float y = fmaf(sv[j], sw[0], sb[0]);  // batch norm of the other half of a joined matrix
        ep.side_out[(int64_t)rid[j] * ep.ld2 + c] = y * ((y > 0.0f) ? 1.0f : ep.leak);
      }
    }
    return;
  }

  // D layout of the 32x32 MFMA: lane holds column (lane & 31), rows 8*(v/4) + 4*(lane>>5) + (v&3).
  // All row ids are fetched from their lanes first, then the stores go out back to back.
  int rid[16];
#pragma unroll
  for (int v = 0; v < 16; v++) rid[v] = __shfl(my_row, 8 * (v >> 2) + 4 * h + (v & 3), 64);
  // (the values of the residual input are all fetched before the first store: a store may alias them
  // as far as the compiler knows, and loads issued between the stores would wait one by one)
  if (ep.res) {
    float rv[NB][16];
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const float *rp = ep.res + (int64_t)(rid[v] < 0 ? 0 : rid[v]) * ep.ldr + cb0 * 32 + r;
#pragma unroll
      for (int b = 0; b < NB; b++) rv[b][v] = (rid[v] >= 0 && (cb0 + b) * 32 + r < Cout) ? rp[b * 32] : 0.0f;
    }
#pragma unroll
    for (int v = 0; v < 16; v++) {
#pragma unroll
      for (int b = 0; b < NB; b++) acc[b][v] += rv[b][v];
    }
    __builtin_amdgcn_sched_barrier(0);  // (the sums stay above the stores)
  }
#pragma unroll
  for (int v = 0; v < 16; v++) {
    if (rid[v] < 0) continue;
    if (out) {
      float *op = out + (int64_t)rid[v] * ld_out + cb0 * 32 + r;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if ((cb0 + b) * 32 + r < Cout) op[b * 32] = acc[b][v];
    }
    if (ep.out2) {
      // fused batch norm + leaky ReLU
      float *op2 = ep.out2 + (int64_t)rid[v] * ep.ld2 + cb0 * 32 + r;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if ((cb0 + b) * 32 + r < Cout) {
          const float y = fmaf(acc[b][v], ew[b], eb[b]);
          op2[b * 32] = y * ((y > 0.0f) ? 1.0f : ep.leak);
        }
    }
  }
  if (MODE == MAP_PARENT && ep.side_in) {
    // batch norm of the other half of a joined matrix, same rows and columns
#pragma unroll
    for (int v = 0; v < 16; v++) {
      float x[NB];
#pragma unroll
      for (int b = 0; b < NB; b++)
        x[b] = (rid[v] >= 0 && (cb0 + b) * 32 + r < Cout) ? ep.side_in[(int64_t)rid[v] * ep.ld_side + (cb0 + b) * 32 + r] : 0.0f;
      if (rid[v] < 0) continue;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if ((cb0 + b) * 32 + r < Cout) {
          const float y = fmaf(x[b], sw[b], sb[b]);
          ep.side_out[(int64_t)rid[v] * ep.ld2 + (cb0 + b) * 32 + r] = y * ((y > 0.0f) ? 1.0f : ep.leak);
        }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Narrow 3^3 layers (Cin <= 32, Cout <= 32): the whole packed filter (27 tiles of 4 KB) stays in
// LDS for the life of the block, so the only traffic between L2 and the CU is the gather itself
// - with the weight tiles re-read per item that path carries twice the bytes and bounds the
// kernel.  Blocks are persistent: block b owns every gridDim.x-th tile and its wavefronts draw
// them one by one.
// The sums are formed exactly as in conv_mfma_kernel<1, 27, MAP_NBR, 1> (offsets ascending,
// same MFMA sequence), so both kernels give the same bits.
// ---------------------------------------------------------------------------------------
#ifndef INSC_WL_WAVES
#define INSC_WL_WAVES 12
#endif
constexpr int WL_WAVES = INSC_WL_WAVES;
#ifndef INSC_WL_DEPTH
#define INSC_WL_DEPTH 4
#endif
constexpr int WL_DEPTH = INSC_WL_DEPTH;
constexpr int WL_MIN_TILES = 4096;  // smaller launches go to conv_mfma_kernel (default of the knob below)
constexpr int WL_SCHED = 256;  // a block orders up to this many tiles of its own by cost

__global__ __launch_bounds__(WL_WAVES * 64) void conv_wlds_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ Wp, const float *__restrict__ bias, const int32_t *__restrict__ map0,
    const int32_t *__restrict__ rows, const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout,
    const uint8_t *__restrict__ tile_flags, uint32_t in_bytes, uint32_t map_bytes, BnEpilogue ep, TilePlan plan) {
  constexpr int K = 27;
  constexpr int NSTAGE = (TILE_M * K + 63) / 64;
  __shared__ __attribute__((aligned(16))) float wl[K * 1024];
  __shared__ int nbl[WL_WAVES][TILE_M * K];
  __shared__ int next_turn;
  __shared__ int cost_l[WL_SCHED], sched_l[WL_SCHED];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;

  // the filter: 27 KB-quarters x 4, copied as is (already in per-lane order)
  {
    const float4 *src = reinterpret_cast<const float4 *>(Wp);
    float4 *dst = reinterpret_cast<float4 *>(wl);
    for (int i = threadIdx.x; i < K * 256; i += WL_WAVES * 64) dst[i] = src[i];
  }
  if (threadIdx.x == 0) next_turn = 0;
  const int64_t ntiles = (n + TILE_M - 1) / TILE_M;
  // Blocks are dealt to the eight XCDs round robin (block b runs on XCD b % 8) and every XCD has an
  // L2 of its own: rank the blocks XCD by XCD, so that the tiles an XCD works on at any time are
  // neighbours in the processing order and share gathered rows in its L2.
  const int G8 = gridDim.x >> 3;
  const int brank = (gridDim.x & 7) == 0 ? (int)(blockIdx.x & 7) * G8 + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  // The block of rank q owns the tiles q, q + gridDim.x, ...  With a tile plan it takes them most
  // expensive first (cost = offsets the tile uses; ties in tile order): its wavefronts then finish
  // within a cheap tile of each other instead of an average one.
  const int my_tiles = ntiles > brank ? (int)((ntiles - brank + gridDim.x - 1) / gridDim.x) : 0;
  const bool lpt = plan.map != nullptr && my_tiles > WL_WAVES && my_tiles <= WL_SCHED;
  if (lpt) {
    for (int j = threadIdx.x; j < my_tiles; j += WL_WAVES * 64) {
      const int64_t tt = (int64_t)j * gridDim.x + brank;
      cost_l[j] = (!tile_flags || tile_flags[tt]) ? __builtin_popcount(plan.tmask[tt]) : -1;
    }
  }
  __syncthreads();
  if (lpt) {
    for (int j = threadIdx.x; j < my_tiles; j += WL_WAVES * 64) {
      const int c = cost_l[j];
      int rank = 0;
      for (int i = 0; i < my_tiles; i++) {
        const int ci = cost_l[i];
        rank += (ci > c || (ci == c && i < j)) ? 1 : 0;
      }
      sched_l[rank] = j;
    }
    __syncthreads();
  }

  int *nl = nbl[wave];
  const __amdgpu_buffer_rsrc_t rin = make_rsrc(in, in_bytes), rmap = make_rsrc(map0, map_bytes);
  // the outputs are addressed with 32-bit byte offsets as well; rows that do not exist get an
  // out-of-range offset and the hardware drops the store
  const __amdgpu_buffer_rsrc_t rout = make_rsrc(out, out ? BUF_OOB : 0u), rout2 = make_rsrc(ep.out2, ep.out2 ? BUF_OOB : 0u);
  const uint32_t ld4 = (uint32_t)ld_in * 4u, ldo4 = (uint32_t)ld_out * 4u, ldo24 = (uint32_t)ep.ld2 * 4u;
  const bool half_on = h == 0 || Cin >= 32;  // a 16-channel layer has nothing for the upper half-wave
  const int col = r;
  const float bv = (bias && col < Cout) ? bias[col] : 0.0f;
  const float ew = (ep.out2 && col < Cout) ? ep.w[col] : 0.0f;
  const float eb = (ep.out2 && col < Cout) ? ep.b[col] : 0.0f;

  // The wavefronts of a block draw its tiles from a counter in LDS
  // (tile costs differ by 3x: a fixed deal per wavefront leaves the slowest one far behind).
  // draw(): the next tile of this block that has work, or ntiles.
  // With fewer than three tiles per wavefront the draws ahead of the tile pipeline (up to three tiles
  // in hand per wavefront) would leave late wavefronts with nothing: then the turns are dealt instead,
  // back and forth: wavefront w takes w, 2 WL_WAVES - 1 - w, 2 WL_WAVES + w, ...  (What a block lasts is the
  // matrix core of its busiest SIMD, which three wavefronts share - w, w + 4, w + 8; with the turns going
  // round the same way, w + WL_WAVES next, the SIMD that starts with the three most expensive tiles also
  // gets the first of the second round.)
  const bool dealt = my_tiles < 3 * WL_WAVES;
  int my_turn = wave, my_round = 0;
  auto draw = [&]() -> int64_t {
    for (;;) {
      int turn;
      if (dealt) {
        turn = my_turn;
        my_round++;
        my_turn = my_round * WL_WAVES + ((my_round & 1) ? WL_WAVES - 1 - wave : wave);
      } else {
        int v = 0;
        if (lane == 0) v = atomicAdd(&next_turn, 1);
        turn = __builtin_amdgcn_readfirstlane(v);
      }
      if (turn >= my_tiles) return ntiles;
      const int64_t t = (int64_t)(lpt ? sched_l[turn] : turn) * gridDim.x + brank;
      if (!tile_flags || tile_flags[t]) return t;
    }
  };
  auto load_row = [&](int64_t t) -> int {
    const int64_t p = t * TILE_M + r;
    return (t < ntiles && p < n) ? (rows ? rows[p] : (int)p) : -1;
  };
  // issue the loads of a tile's slice of the neighbour map; bit i of the result: element i of
  // this lane exists (a load sent out of range returns 0, which would pass for a site).  With a
  // tile plan the slice is 27 coalesced runs that need no row id; the LDS copy is offset-major.
  const bool planned = plan.map != nullptr;
  const __amdgpu_buffer_rsrc_t rplan = make_rsrc(plan.map, planned ? (uint32_t)(plan.ld * K * 4) : 0u);
  auto stage_issue = [&](int64_t tt, int my_row, int (&st)[NSTAGE]) -> unsigned {
    unsigned valid = 0;
    if (planned) {
#pragma unroll
      for (int i = 0; i < NSTAGE; i++) {
        const int e = i * 64 + lane;  // e = k * 32 + row
        const bool ok = e < TILE_M * K && tt < ntiles;
        if (ok) valid |= 1u << i;
        const uint32_t voff = ok ? (uint32_t)((e >> 5) * (int)plan.ld + (int)(tt * TILE_M) + (e & 31)) * 4u : BUF_OOB;
        st[i] = __builtin_amdgcn_raw_buffer_load_b32(rplan, (int)voff, 0, 0);
      }
      return valid;
    }
    int srow[NSTAGE];
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) srow[i] = __shfl(my_row, ((i * 64 + lane) / K) & (TILE_M - 1), 64);
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = i * 64 + lane;
      const int kk = e - (e / K) * K;
      const bool ok = e < TILE_M * K && srow[i] >= 0;
      if (ok) valid |= 1u << i;
      st[i] = __builtin_amdgcn_raw_buffer_load_b32(rmap, (int)(ok ? (uint32_t)(srow[i] * K + kk) * 4u : BUF_OOB), 0, 0);
    }
    return valid;
  };

  // Software pipeline over tiles: while tile t is computed, the neighbour-map slice of the next
  // tile and the row ids of the one after it are in flight.
  int64_t t = draw();
  int my_row = load_row(t);
  int st[NSTAGE];
  unsigned valid = stage_issue(t, my_row, st);
  int64_t tn = t < ntiles ? draw() : ntiles;
  int my_row_n = load_row(tn);

  while (t < ntiles) {
    // neighbour-map slice -> LDS (private to the wavefront), and the offsets the tile uses
    unsigned mymask = 0;
    if (planned) {
      mymask = plan.tmask[t];
#pragma unroll
      for (int i = 0; i < NSTAGE; i++) {
        const int e = i * 64 + lane;
        if (e < TILE_M * K) nl[e] = st[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < NSTAGE; i++) {
        const int e = i * 64 + lane;
        if (e < TILE_M * K) {
          const bool have = ((valid >> i) & 1u) && st[i] >= 0;
          nl[e] = have ? st[i] : -1;
          if (have) mymask |= 1u << (e % K);
        }
      }
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) mymask |= (unsigned)__shfl_xor((int)mymask, d, 64);
    }
    unsigned rest = (unsigned)__builtin_amdgcn_readfirstlane((int)mymask);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // next tile's loads
    int stn[NSTAGE];
    const unsigned valid_n = stage_issue(tn, my_row_n, stn);
    const int64_t tnn = tn < ntiles ? draw() : ntiles;
    const int my_row_nn = load_row(tnn);

    f16v acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = bv;

    if (rest) {
      const int nitems = __builtin_popcount(rest);
      // cursor over the active offsets, branch-free; -1 past the end (loads go out of range)
      auto next_k = [&]() -> int {
        const int k = rest ? __builtin_ctz(rest) : -1;
        rest &= rest - 1;
        return k;
      };
      auto gather = [&](int k) -> Frag {
        const int kk = k < 0 ? 0 : k;
        const int src = nl[planned ? kk * TILE_M + r : r * K + kk];
        const bool on = k >= 0 && src >= 0 && half_on;
        const uint32_t voff = on ? (uint32_t)src * ld4 + (uint32_t)(h * 64) : BUF_OOB;
        Frag f;
#pragma unroll
        for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rin, voff + 16u * q, 0);
        return f;
      };
      auto wread = [&](int k) -> Frag {
        const float4 *p = reinterpret_cast<const float4 *>(wl + (k < 0 ? 0 : k) * 1024) + lane;
        Frag f;
#pragma unroll
        for (int q = 0; q < 4; q++) f.q[q] = p[q * 64];
        return f;
      };
      constexpr int D = WL_DEPTH;
      Frag g[D];
      int kq[D];  // offsets of the items in the ring
#pragma unroll
      for (int d = 0; d < D - 1; d++) {
        kq[d] = next_k();
        g[d] = gather(kq[d]);
      }
      // The loads of the item D - 1 ahead and the weight tile of the next item are issued in the
      // shadow of this item's MFMAs (a dependent MFMA issues every 64 cycles; whatever sits between
      // two of them is free), in four slices pinned by scheduling barriers.
      // (one turn of the loop covers both rings: D register slots for the gathered rows, two for the weights)
      constexpr int TURN = D % 2 == 0 ? D : 2 * D;
      Frag bw[2];
      bw[0] = wread(kq[0]);
      for (int i0 = 0; i0 < nitems; i0 += TURN) {
#pragma unroll
        for (int u = 0; u < TURN; u++) {
          const bool real = i0 + u < nitems;
          const Frag &bf = bw[u % 2];
          __builtin_amdgcn_sched_barrier(0);
          if (real) {
#pragma unroll
            for (int s = 0; s < 4; s++)
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[u % D], s), frag_at(bf, s), acc, 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          const int kn = next_k();
          kq[(u + D - 1) % D] = kn;
          const int src = nl[planned ? (kn < 0 ? 0 : kn) * TILE_M + r : r * K + (kn < 0 ? 0 : kn)];
          __builtin_amdgcn_sched_barrier(0);
          if (real) {
#pragma unroll
            for (int s = 4; s < 8; s++)
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[u % D], s), frag_at(bf, s), acc, 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          {
            const bool on = kn >= 0 && src >= 0 && half_on;
            const uint32_t voff = on ? (uint32_t)src * ld4 + (uint32_t)(h * 64) : BUF_OOB;
#pragma unroll
            for (int q = 0; q < 4; q++) g[(u + D - 1) % D].q[q] = buf_load16(rin, voff + 16u * q, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          if (real) {
#pragma unroll
            for (int s = 8; s < 12; s++)
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[u % D], s), frag_at(bf, s), acc, 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          bw[(u + 1) % 2] = wread(kq[(u + 1) % D]);
          __builtin_amdgcn_sched_barrier(0);
          if (real) {
#pragma unroll
            for (int s = 12; s < 16; s++)
              acc = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[u % D], s), frag_at(bf, s), acc, 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }

    // D layout of the 32x32 MFMA: lane holds column (lane & 31), rows 8*(v/4) + 4*(lane>>5) + (v&3)
    int rid[16];
#pragma unroll
    for (int v = 0; v < 16; v++) rid[v] = __shfl(my_row, 8 * (v >> 2) + 4 * h + (v & 3), 64);
    const uint32_t col4 = (uint32_t)col * 4u;
    // (the residual input is fetched before the first store, which may alias it as far as the
    // compiler knows: loads issued between the stores would wait one by one)
    float rv[16];
#pragma unroll
    for (int v = 0; v < 16; v++)
      rv[v] = (ep.res && rid[v] >= 0 && col < Cout) ? ep.res[(int64_t)rid[v] * ep.ldr + col] : 0.0f;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const bool ok = rid[v] >= 0 && col < Cout;
      float av = acc[v];  // (a bit cast applied to the vector element itself reads element 0)
      if (ep.res && ok) av += rv[v];
      if (out)
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(av), rout,
                                              (int)(ok ? __umul24((unsigned)rid[v], ldo4) + col4 : BUF_OOB), 0, 0);
      if (ep.out2) {
        // fused batch norm + leaky ReLU
        const float y = fmaf(av, ew, eb);
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(y * ((y > 0.0f) ? 1.0f : ep.leak)), rout2,
                                              (int)(ok ? __umul24((unsigned)rid[v], ldo24) + col4 : BUF_OOB), 0, 0);
      }
    }
    // the next tile overwrites this wavefront's LDS slice: all lanes must be done reading it
    __builtin_amdgcn_wave_barrier();

    t = tn;
    my_row = my_row_n;
    valid = valid_n;
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) st[i] = stn[i];
    tn = tnn;
    my_row_n = my_row_nn;
  }
}

// ---------------------------------------------------------------------------------------
// Wide 3^3 layers with many tiles: persistent blocks of S wavefronts.  A block works through
// units (tile, output block) of a cost-ordered list (plan.sched: tiles by falling number of active
// offsets); block b takes the units b, 2B-1-b, 2B+b, ... (every other round reversed, so a block
// that starts with an expensive unit continues with a cheap one).  While a unit is computed the
// neighbour-map slice, row ids and tile id of the next ones are in flight, so that no wavefront
// ever waits for a launch, a map or a row id between two units - with one block per unit the
// matrix cores idle through 5-10 us of such latencies per wavefront, and the units a compute unit
// happens to receive differ by 2x in cost.
// The S wavefronts deal the (offset, chunk) items of the unit exactly as conv_mfma_kernel<1, 27,
// MAP_NBR, S> with one block per tile does, and the partial sums are added in the same order: both
// kernels give the same bits.  All wavefronts share the final sum and the stores (8 * 4 / S rows each).
// ---------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(S * 64) __attribute__((amdgpu_waves_per_eu(3, 3))) void conv_pers_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ Wp, const float *__restrict__ bias, const int32_t *__restrict__ rows,
    const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout, int nbt, int nbtp,
    const uint8_t *__restrict__ tile_flags, uint32_t in_bytes, uint32_t wp_bytes, BnEpilogue ep, TilePlan plan) {
  constexpr int K = 27;
  constexpr int NSTAGE = (TILE_M * K + 64 * S - 1) / (64 * S);
  constexpr int VPW = 16 / S;  // accumulator registers (groups of 4 rows x 2 half-waves) a wavefront finishes
  __shared__ int nl[2][TILE_M * K];
  __shared__ float red[2][S][16 * 64];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int64_t ntiles = (n + TILE_M - 1) / TILE_M, units = ntiles * nbt;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int nch = conv_nch(Cin);
  const int64_t B = gridDim.x, b = blockIdx.x;
  const __amdgpu_buffer_rsrc_t rplan = make_rsrc(plan.map, (uint32_t)(plan.ld * K * 4));
  // unit j of this block: b, 2B - 1 - b, 2B + b, ...
  auto unit_at = [&](int64_t j) -> int64_t { return j * B + ((j & 1) ? B - 1 - b : b); };
  // Tile id, tile flag and offset mask of a unit are the same for every lane, but they are fetched
  // with vector loads: scalar loads share their counter with the LDS reads of the item loop, which
  // would then wait for them.
  const __amdgpu_buffer_rsrc_t rsched = make_rsrc(plan.sched, (uint32_t)(ntiles * 4));
  const __amdgpu_buffer_rsrc_t rtmask = make_rsrc(plan.tmask, (uint32_t)(ntiles * 4));
  const __amdgpu_buffer_rsrc_t rflag = make_rsrc(tile_flags, tile_flags ? (uint32_t)ntiles : 0u);
  auto tile_issue = [&](int64_t u) -> int {  // out of range: 0, never used
    return __builtin_amdgcn_raw_buffer_load_b32(rsched, (int)(u < units ? (uint32_t)(u / nbt) * 4u : BUF_OOB), 0, 0);
  };
  auto stage_issue = [&](int tile, int (&st)[NSTAGE]) {
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = (i * S + wave) * 64 + lane;  // e = k * 32 + row
      const bool ok = tile >= 0 && e < TILE_M * K;  // (the value of a load sent out of range is never used)
      const uint32_t voff = ok ? (uint32_t)((e >> 5) * (int)plan.ld + tile * TILE_M + (e & 31)) * 4u : BUF_OOB;
      st[i] = __builtin_amdgcn_raw_buffer_load_b32(rplan, (int)voff, 0, 0);
    }
  };
  auto row_of = [&](int tile) -> int {
    const int64_t p = (int64_t)tile * TILE_M + r;
    return (tile >= 0 && p < n) ? (rows ? rows[p] : (int)p) : -1;
  };
  auto flag_issue = [&](int tile) -> int {
    return (int)__builtin_amdgcn_raw_buffer_load_b8(rflag, (int)(tile >= 0 ? (uint32_t)tile : BUF_OOB), 0, 0);
  };
  auto mask_issue = [&](int tile) -> int {
    return __builtin_amdgcn_raw_buffer_load_b32(rtmask, (int)(tile >= 0 ? (uint32_t)tile * 4u : BUF_OOB), 0, 0);
  };

  const __amdgpu_buffer_rsrc_t rin = make_rsrc(in, in_bytes), rw = make_rsrc(Wp, wp_bytes);
  const uint32_t ld4 = (uint32_t)ld_in * 4u, lane16 = (uint32_t)lane * 16u;
  // outputs and the residual input are addressed with 32-bit byte offsets as well (the host checks
  // the sizes); rows that do not exist get an out-of-range offset and the hardware drops the access
  const __amdgpu_buffer_rsrc_t rout = make_rsrc(out, out ? BUF_OOB : 0u), rout2 = make_rsrc(ep.out2, ep.out2 ? BUF_OOB : 0u);
  const __amdgpu_buffer_rsrc_t rres = make_rsrc(ep.res, ep.res ? BUF_OOB : 0u);
  const __amdgpu_buffer_rsrc_t rbias = make_rsrc(bias, bias ? (uint32_t)Cout * 4u : 0u);
  const __amdgpu_buffer_rsrc_t rew = make_rsrc(ep.w, ep.out2 ? (uint32_t)Cout * 4u : 0u);
  const __amdgpu_buffer_rsrc_t reb = make_rsrc(ep.b, ep.out2 ? (uint32_t)Cout * 4u : 0u);
  const uint32_t ldo4 = (uint32_t)ld_out * 4u, ldo24 = (uint32_t)ep.ld2 * 4u, ldr4 = (uint32_t)ep.ldr * 4u;
  // Offsets of which this wavefront holds at least 1, 2, .. items (it takes, of offset k, the chunks
  // ch0(k), ch0(k) + S, ... with ch0(k) = (wave - k * nch) mod S): the items of a tile with offset
  // mask m are then counted with a few population counts.
  constexpr int MAXQ = 4;  // nch <= MAXQ * S
  unsigned kmask[MAXQ];
#pragma unroll
  for (int q = 0; q < MAXQ; q++) kmask[q] = 0;
  for (int k = 0; k < K; k++) {
    const int c0 = (wave - k * nch) & (S - 1);
    const int cnt = c0 < nch ? (nch - c0 + S - 1) / S : 0;
#pragma unroll
    for (int q = 0; q < MAXQ; q++)
      if (cnt > q) kmask[q] |= 1u << k;
  }
  // bias and the fused batch norm's scale / shift for this lane's column of output block ob (sent
  // out of range, they read as zero)
  auto col_issue = [&](int ob, float &bv, float &ew, float &eb) {
    const uint32_t off = (uint32_t)(ob * 32 + r) * 4u;
    bv = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(rbias, (int)(wave == 0 ? off : BUF_OOB), 0, 0));
    ew = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(rew, (int)off, 0, 0));
    eb = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(reb, (int)off, 0, 0));
  };

  // LDS copies of the map slice and of the partial sums are double buffered (parity par): one
  // barrier per unit publishes the partial sums of this unit and the map slice of the next
  // Pipeline over the units of this block: while unit j is computed, the map slice, row ids, flag
  // and mask of unit j + 1 and the tile id of unit j + 2 are in flight.
  int64_t j = 0, u = unit_at(0);
  int tile_c = u < units ? __builtin_amdgcn_readfirstlane(tile_issue(u)) : -1;
  int tile_n = unit_at(1) < units ? __builtin_amdgcn_readfirstlane(tile_issue(unit_at(1))) : -1;
  int par = 0;
  {
    int st[NSTAGE];
    stage_issue(tile_c, st);
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = (i * S + wave) * 64 + lane;
      if (e < TILE_M * K) nl[0][e] = st[i];
    }
  }
  int my_row = row_of(tile_c);
  bool live = tile_c >= 0 && (!tile_flags || __builtin_amdgcn_readfirstlane(flag_issue(tile_c)) != 0);
  unsigned tmask_c = (unsigned)__builtin_amdgcn_readfirstlane(mask_issue(tile_c));
  float bv, ew, eb;
  col_issue((int)(u % nbt), bv, ew, eb);
  __syncthreads();

  while (u < units) {
    const int ob = (int)(u % nbt);
    const int64_t un = unit_at(j + 1), unn = unit_at(j + 2);
    const int tile_nn_v = tile_issue(unn);
    int stn[NSTAGE];
    stage_issue(tile_n, stn);
    const int my_row_n = row_of(tile_n);
    const int flag_n_v = flag_issue(tile_n);
    const int tmask_n_v = mask_issue(tile_n);
    float bv_n, ew_n, eb_n;
    col_issue((int)(un % nbt), bv_n, ew_n, eb_n);
    const int *nlc = nl[par];
    const int c = ob * 32 + r;
    f16v acc;
    int rid[VPW];
    float rv[VPW];

    if (live) {
      // Items (active offset k, 32-channel chunk ch), dealt by (k * nch + ch) % S: wavefront w takes,
      // of offset k, the chunks ch0(k), ch0(k) + S, ... with ch0(k) = (w - k * nch) mod S.
      const unsigned rest = tmask_c & kmask[0];
      int nitems = 0;
#pragma unroll
      for (int q = 0; q < MAXQ; q++) nitems += __builtin_popcount(tmask_c & kmask[q]);
#pragma unroll
      for (int v = 0; v < 16; v++) acc[v] = bv;

      if (rest) {
        struct Cursor {
          int k, ch;
          unsigned rest;
        };
        auto ch0 = [&](int k) -> int { return (wave - k * nch) & (S - 1); };
        auto step = [&](const Cursor &cu) -> Cursor {
          const bool wrap = cu.ch + S >= nch;
          const int nk = cu.rest ? __builtin_ctz(cu.rest) : -1;
          Cursor nx;
          nx.ch = wrap ? ch0(nk) : cu.ch + S;
          nx.k = wrap ? nk : cu.k;
          nx.rest = wrap ? (cu.rest & (cu.rest - 1)) : cu.rest;
          return nx;
        };
        Cursor first;
        first.k = __builtin_ctz(rest);
        first.ch = ch0(first.k);
        first.rest = rest & (rest - 1);
        auto gather = [&](const Cursor &cu) -> Frag {
          const int kk = cu.k < 0 ? 0 : cu.k;
          const int src = nlc[kk * TILE_M + r];
          const bool on = cu.k >= 0 && src >= 0 && (h == 0 || Cin - cu.ch * 32 >= 32);
          const uint32_t voff = on ? (uint32_t)src * ld4 + (uint32_t)(cu.ch * 128 + h * 64) : BUF_OOB;
          Frag f;
#pragma unroll
          for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rin, voff + 16u * q, 0);
          return f;
        };
        auto wload = [&](const Cursor &cu) -> Frag {
          const int tile = ((cu.k < 0 ? 0 : cu.k) * nch + cu.ch) * nbtp + ob;
          const uint32_t soff = (uint32_t)__builtin_amdgcn_readfirstlane(tile * 4096);
          const uint32_t voff = cu.k >= 0 ? lane16 : BUF_OOB;
          Frag f;
#pragma unroll
          for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rw, voff + 1024u * q, soff);
          return f;
        };
        // the same ring of D items in flight as in conv_mfma_kernel
        constexpr int D = INSC_CONV_DEPTH_SPLIT;
        Frag g[D], bw[D];
        Cursor ci = first;
#pragma unroll
        for (int d = 0; d < D - 1; d++) {
          g[d] = gather(ci);
          bw[d] = wload(ci);
          ci = step(ci);
        }
        for (int t0i = 0; t0i < nitems; t0i += D) {
#pragma unroll
          for (int uu = 0; uu < D; uu++) {
            g[(uu + D - 1) % D] = gather(ci);
            bw[(uu + D - 1) % D] = wload(ci);
            ci = step(ci);
            const bool real = t0i + uu < nitems;
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            if (real) {
#pragma unroll
              for (int s2 = 0; s2 < 16; s2++)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[uu], s2), frag_at(bw[uu], s2), acc, 0, 0, 0);
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }

    }
    // the next unit's slice of the map and its scalars (taken before the loads and stores of this
    // unit's output are issued: a wait for them placed later would wait for those as well)
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const int e = (i * S + wave) * 64 + lane;
      if (e < TILE_M * K) nl[par ^ 1][e] = stn[i];
    }
    const int tile_nn = unn < units ? __builtin_amdgcn_readfirstlane(tile_nn_v) : -1;
    const bool live_n = tile_n >= 0 && (!tile_flags || __builtin_amdgcn_readfirstlane(flag_n_v) != 0);
    const unsigned tmask_n = tile_n >= 0 ? (unsigned)__builtin_amdgcn_readfirstlane(tmask_n_v) : 0u;
    if (live) {
      // partial sums of all wavefronts through LDS
#pragma unroll
      for (int v = 0; v < 16; v++) red[par][wave][v * 64 + lane] = acc[v];
      // rows this wavefront will store, and their residual input (in flight across the barrier)
#pragma unroll
      for (int q = 0; q < VPW; q++) {
        const int v = wave * VPW + q;
        rid[q] = __shfl(my_row, 8 * (v >> 2) + 4 * h + (v & 3), 64);
        if (c >= Cout) rid[q] = -1;
        rv[q] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(
            rres, (int)(rid[q] >= 0 ? __umul24((unsigned)rid[q], ldr4) + (uint32_t)c * 4u : BUF_OOB), 0, 0));
      }
    }
    __syncthreads();
    if (live) {
      // wavefront w adds the partial sums, in wavefront order, for the accumulator registers
      // w * VPW .. and stores those rows
      float a[VPW];
#pragma unroll
      for (int q = 0; q < VPW; q++) {
        const int v = wave * VPW + q;
        a[q] = red[par][0][v * 64 + lane];
#pragma unroll
        for (int w = 1; w < S; w++) a[q] += red[par][w][v * 64 + lane];
        if (ep.res) a[q] += rv[q];
      }
#pragma unroll
      for (int q = 0; q < VPW; q++) {
        const uint32_t c4 = (uint32_t)c * 4u;
        if (out)
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(a[q]), rout,
                                                (int)(rid[q] >= 0 ? __umul24((unsigned)rid[q], ldo4) + c4 : BUF_OOB), 0, 0);
        if (ep.out2) {
          const float y = fmaf(a[q], ew, eb);  // fused batch norm + leaky ReLU
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(y * ((y > 0.0f) ? 1.0f : ep.leak)), rout2,
                                                (int)(rid[q] >= 0 ? __umul24((unsigned)rid[q], ldo24) + c4 : BUF_OOB), 0, 0);
        }
      }
    }
    j++;
    u = un;
    tile_c = tile_n;
    tile_n = tile_nn;
    my_row = my_row_n;
    live = live_n;
    tmask_c = tmask_n;
    bv = bv_n;
    ew = ew_n;
    eb = eb_n;
    par ^= 1;
  }
}

// ---------------------------------------------------------------------------------------
// Wide 3^3 layers with many tiles, second design: the bytes a compute unit pulls through its L1
// bound these layers (8 KB per 16 MFMAs: a gathered chunk and a weight tile), so here the four
// wavefronts of a block work on four consecutive tiles and walk the union of their offsets in
// step: the weight tile of a step goes from L2 into LDS once per block (buffer loads that write
// LDS directly, a quarter per wavefront) and is read from there by all four, and a wavefront
// computes NB output blocks from one gathered chunk.  A wavefront owns its tile: no partial sums
// cross wavefronts.  To give the bits of conv_mfma_kernel<1, 27, MAP_NBR, ST> it keeps that
// kernel's ST partial sums - the items (k, ch) with (k * nch + ch) % ST == p, in ascending order,
// bias in sum 0 - in ST accumulators per output block and adds them in order at the end.
// Blocks are persistent over units (group of four tiles, NB output blocks) taken from the cost-
// ordered group schedule as in conv_pers_kernel.
// The two weight buffers and the two A slots alternate with the parity of the step, and the step
// loop is unrolled by two so that each is a compile-time choice: the compiler then knows that a
// read of one weight buffer cannot touch the load into the other that is still in flight (for a
// single array it would wait for every outstanding load before each LDS read).
// ---------------------------------------------------------------------------------------
#define INSC_LDS_PTR(x) ((__attribute__((address_space(3))) void *)(x))
template <int NB, int ST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NB * ST > 4 ? 2 : 3, NB * ST > 4 ? 2 : 3))) void conv_wshare_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ Wp, const float *__restrict__ bias, const int32_t *__restrict__ rows,
    const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout, int nbt, int nbtp,
    const uint8_t *__restrict__ tile_flags, uint32_t in_bytes, uint32_t wp_bytes, BnEpilogue ep, TilePlan plan) {
  constexpr int K = 27, WV = 4;
  constexpr int NSTAGE = (TILE_M * K + 63) / 64;  // 14 loads of 64 entries; the last one half empty
  __shared__ int nl[WV][NSTAGE * 64];
  __shared__ float4 wl0[NB][256];
  __shared__ float4 wl1[NB][256];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int ntiles = (int)((n + TILE_M - 1) / TILE_M), ngroups = (ntiles + WV - 1) / WV;
  const int nug = (nbt + NB - 1) / NB;  // units per group
  const int64_t units = (int64_t)ngroups * nug;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int nch = conv_nch(Cin);
  const int64_t B = gridDim.x, b = blockIdx.x;
  const __amdgpu_buffer_rsrc_t rplan = make_rsrc(plan.map, (uint32_t)(plan.ld * K * 4));
  const __amdgpu_buffer_rsrc_t rsched = make_rsrc(plan.sched + (plan.ld + 31) / 32, (uint32_t)ngroups * 4u);  // group schedule
  const __amdgpu_buffer_rsrc_t rtmask = make_rsrc(plan.tmask, (uint32_t)ntiles * 4u);
  const __amdgpu_buffer_rsrc_t rflag = make_rsrc(tile_flags, tile_flags ? (uint32_t)ntiles : 0u);
  const __amdgpu_buffer_rsrc_t rin = make_rsrc(in, in_bytes), rw = make_rsrc(Wp, wp_bytes);
  const __amdgpu_buffer_rsrc_t rout = make_rsrc(out, out ? BUF_OOB : 0u), rout2 = make_rsrc(ep.out2, ep.out2 ? BUF_OOB : 0u);
  const __amdgpu_buffer_rsrc_t rres = make_rsrc(ep.res, ep.res ? BUF_OOB : 0u);
  const __amdgpu_buffer_rsrc_t rbias = make_rsrc(bias, bias ? (uint32_t)Cout * 4u : 0u);
  const __amdgpu_buffer_rsrc_t rew = make_rsrc(ep.w, ep.out2 ? (uint32_t)Cout * 4u : 0u);
  const __amdgpu_buffer_rsrc_t reb = make_rsrc(ep.b, ep.out2 ? (uint32_t)Cout * 4u : 0u);
  const uint32_t ld4 = (uint32_t)ld_in * 4u, ldo4 = (uint32_t)ld_out * 4u, ldo24 = (uint32_t)ep.ld2 * 4u,
                 ldr4 = (uint32_t)ep.ldr * 4u;
  int *nlw = nl[wave];

  auto unit_at = [&](int64_t j) -> int64_t { return j * B + ((j & 1) ? B - 1 - b : b); };
  auto group_issue = [&](int64_t u) -> int {
    return __builtin_amdgcn_raw_buffer_load_b32(rsched, (int)(u < units ? (uint32_t)(u / nug) * 4u : BUF_OOB), 0, 0);
  };
  // offset masks of the four tiles of a group (0 for a tile that does not exist or is not flagged):
  // lanes 0..3 fetch one each, every wavefront the same four
  auto masks_issue = [&](int g, int &mv, int &fv) {
    const int t = g * WV + (lane & 3);
    const bool ok = g >= 0 && t < ntiles;
    mv = __builtin_amdgcn_raw_buffer_load_b32(rtmask, (int)(ok ? (uint32_t)t * 4u : BUF_OOB), 0, 0);
    fv = tile_flags ? (int)__builtin_amdgcn_raw_buffer_load_b8(rflag, (int)(ok ? (uint32_t)t : BUF_OOB), 0, 0) : (ok ? 1 : 0);
  };
  // this wavefront's slice of the map, straight into LDS (entry e = k * 32 + row at nlw[e])
  // (load i covers the offsets 2i and 2i + 1: one per half-wave; the lane's part of the address is the
  // same for every i, the rest is a scalar)
  auto stage_issue = [&](int tile) {
    if (tile < 0) return;  // no such tile: its wavefront never reads the slice
    const uint32_t base = (uint32_t)(h * (int)plan.ld + tile * TILE_M + r) * 4u;
    const uint32_t pair = (uint32_t)plan.ld * 8u;
#pragma unroll
    for (int i = 0; i < NSTAGE; i++) {
      const uint32_t voff = (2 * i + 1 < K || h == 0) ? base : BUF_OOB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rplan, INSC_LDS_PTR(nlw + i * 64), 4, (int)voff, (int)(i * pair), 0, 0);
    }
  };
  auto row_of = [&](int tile) -> int {
    const int64_t p = (int64_t)tile * TILE_M + r;
    return (tile >= 0 && p < n) ? (rows ? rows[p] : (int)p) : -1;
  };
  struct Step {
    int k, ch;
    unsigned rest;
  };
  auto step_next = [&](const Step &c) -> Step {  // past the end: k = -1
    Step nx;
    const bool wrap = c.ch + 1 >= nch;
    const int nk = c.rest ? __builtin_ctz(c.rest) : -1;
    nx.ch = wrap ? 0 : c.ch + 1;
    nx.k = wrap ? nk : c.k;
    nx.rest = wrap ? (c.rest & (c.rest - 1)) : c.rest;
    return nx;
  };

  int64_t j = 0, u = unit_at(0);
  int g_c = u < units ? __builtin_amdgcn_readfirstlane(group_issue(u)) : -1;
  int g_n = unit_at(1) < units ? __builtin_amdgcn_readfirstlane(group_issue(unit_at(1))) : -1;
  int mv_c, fv_c;
  masks_issue(g_c, mv_c, fv_c);
  int tile = g_c >= 0 && g_c * WV + wave < ntiles ? g_c * WV + wave : -1;
  stage_issue(tile);
  int my_row = row_of(tile);

  while (u < units) {
    const int ob0 = (int)(u % nug) * NB;
    const int64_t un = unit_at(j + 1), unn = unit_at(j + 2);
    const int g_nn_v = group_issue(unn);
    int mv_n, fv_n;
    masks_issue(g_n, mv_n, fv_n);
    const int tile_n = g_n >= 0 && g_n * WV + wave < ntiles ? g_n * WV + wave : -1;
    const int my_row_n = row_of(tile_n);
    // masks of the group: mine and the union
    unsigned mt[WV];
#pragma unroll
    for (int w = 0; w < WV; w++)
      mt[w] = __builtin_amdgcn_readlane(fv_c, w) ? (unsigned)__builtin_amdgcn_readlane(mv_c, w) : 0u;
    unsigned mine = 0, uni = 0;
#pragma unroll
    for (int w = 0; w < WV; w++) {
      uni |= mt[w];
      if (w == wave) mine = mt[w];
    }
    if (tile < 0) mine = 0;

    if (uni) {
      // bias and the fused batch norm's coefficients of this lane's columns
      float bv[NB], ew[NB], eb[NB];
#pragma unroll
      for (int o = 0; o < NB; o++) {
        const uint32_t off = (uint32_t)((ob0 + o) * 32 + r) * 4u;
        bv[o] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(rbias, (int)off, 0, 0));
        ew[o] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(rew, (int)off, 0, 0));
        eb[o] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(reb, (int)off, 0, 0));
      }
      f16v acc[ST][NB];  // partial sum p holds the items with (k * nch + ch) % ST == p; bias in sum 0
#pragma unroll
      for (int pp = 0; pp < ST; pp++) {
#pragma unroll
        for (int o = 0; o < NB; o++) {
#pragma unroll
          for (int v = 0; v < 16; v++) acc[pp][o][v] = pp == 0 ? bv[o] : 0.0f;
        }
      }
      const int nsteps = __builtin_popcount(uni) * nch;
      // weight tiles of a step -> LDS, a quarter (1 KB) per wavefront and output block
      auto w_issue0 = [&](const Step &c) {
#pragma unroll
        for (int o = 0; o < NB; o++) {
          const uint32_t soff = (uint32_t)(((c.k < 0 ? 0 : c.k) * nch + c.ch) * nbtp + ob0 + o) * 4096u;
          const bool ok = c.k >= 0 && ob0 + o < nbt;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, INSC_LDS_PTR(&wl0[o][wave * 64]), 16,
                                                   (int)(ok ? (uint32_t)(wave * 1024 + lane * 16) : BUF_OOB), (int)soff, 0, 0);
        }
      };
      auto w_issue1 = [&](const Step &c) {
#pragma unroll
        for (int o = 0; o < NB; o++) {
          const uint32_t soff = (uint32_t)(((c.k < 0 ? 0 : c.k) * nch + c.ch) * nbtp + ob0 + o) * 4096u;
          const bool ok = c.k >= 0 && ob0 + o < nbt;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, INSC_LDS_PTR(&wl1[o][wave * 64]), 16,
                                                   (int)(ok ? (uint32_t)(wave * 1024 + lane * 16) : BUF_OOB), (int)soff, 0, 0);
        }
      };
      auto gather = [&](const Step &c) -> Frag {
        const int kk = c.k < 0 ? 0 : c.k;
        const int src = nlw[kk * TILE_M + r];
        const bool on = c.k >= 0 && ((mine >> kk) & 1u) && src >= 0 && (h == 0 || Cin - c.ch * 32 >= 32);
        const uint32_t voff = on ? (uint32_t)src * ld4 + (uint32_t)(c.ch * 128 + h * 64) : BUF_OOB;
        Frag f;
#pragma unroll
        for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rin, voff + 16u * q, 0);
        return f;
      };
      auto compute = [&](const Step &c, const Frag &a, const float4 (*wl)[256]) {
        if (c.k < 0 || !((mine >> c.k) & 1u)) return;  // (the same for every lane of the wavefront)
        const int part = (c.k * nch + c.ch) & (ST - 1);
#pragma unroll
        for (int o = 0; o < NB; o++) {
          if (ob0 + o >= nbt) break;
          Frag bf;
#pragma unroll
          for (int q = 0; q < 4; q++) bf.q[q] = wl[o][q * 64 + lane];
#pragma unroll
          for (int pp = 0; pp < ST; pp++) {
            if (part != pp) continue;  // (one copy of the MFMA block per partial sum: the accumulator is a compile-time choice)
#pragma unroll
            for (int s2 = 0; s2 < 16; s2++)
              acc[pp][o] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(a, s2), frag_at(bf, s2), acc[pp][o], 0, 0, 0);
          }
        }
      };
      Step c0;  // step on the matrix cores
      c0.k = __builtin_ctz(uni);
      c0.ch = 0;
      c0.rest = uni & (uni - 1);
      Step c1 = step_next(c0);
      __builtin_amdgcn_sched_barrier(0);
      w_issue0(c0);
      __builtin_amdgcn_sched_barrier(0);
      Frag a0 = gather(c0), a1;
      __builtin_amdgcn_sched_barrier(0);
      // Before a barrier every wavefront waits until its own quarter of the step's weight tiles has
      // landed in LDS: everything but the four gather loads issued after it (vmcnt(4); the order of
      // the loads is pinned).
      for (int s0 = 0; s0 < nsteps; s0 += 2) {
        // even step: weights in wl0, chunk in a0
        __builtin_amdgcn_s_waitcnt(0x0F74);
        __syncthreads();  // W(s0) is complete for every wavefront, and nobody reads wl1 any more
        __builtin_amdgcn_sched_barrier(0);
        w_issue1(c1);
        __builtin_amdgcn_sched_barrier(0);
        a1 = gather(c1);
        __builtin_amdgcn_sched_barrier(0);
        compute(c0, a0, wl0);
        c0 = step_next(c1);
        // odd step: weights in wl1, chunk in a1
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F74);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        w_issue0(c0);
        __builtin_amdgcn_sched_barrier(0);
        a0 = gather(c0);
        __builtin_amdgcn_sched_barrier(0);
        compute(c1, a1, wl1);
        c1 = step_next(c0);
        __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();  // the weight buffers are free for the next unit

      // this unit's rows; the next unit's map slice goes out first (nobody reads nl any more)
      stage_issue(tile_n);
      int rid[16];
#pragma unroll
      for (int v = 0; v < 16; v++) rid[v] = __shfl(my_row, 8 * (v >> 2) + 4 * h + (v & 3), 64);
      if (mine) {
#pragma unroll
        for (int o = 0; o < NB; o++) {
          const int cc = (ob0 + o) * 32 + r;
          if (ob0 + o >= nbt) break;
          float rv[16];
#pragma unroll
          for (int v = 0; v < 16; v++)
            rv[v] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(
                rres, (int)((rid[v] >= 0 && cc < Cout) ? __umul24((unsigned)rid[v], ldr4) + (uint32_t)cc * 4u : BUF_OOB), 0, 0));
#pragma unroll
          for (int v = 0; v < 16; v++) {
            const bool ok = rid[v] >= 0 && cc < Cout;
            float a = acc[0][o][v];
#pragma unroll
            for (int pp = 1; pp < ST; pp++) a += acc[pp][o][v];
            if (ep.res) a += rv[v];
            if (out)
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(a), rout,
                                                    (int)(ok ? __umul24((unsigned)rid[v], ldo4) + (uint32_t)cc * 4u : BUF_OOB), 0, 0);
            if (ep.out2) {
              const float y = fmaf(a, ew[o], eb[o]);
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(y * ((y > 0.0f) ? 1.0f : ep.leak)), rout2,
                                                    (int)(ok ? __umul24((unsigned)rid[v], ldo24) + (uint32_t)cc * 4u : BUF_OOB), 0, 0);
            }
          }
        }
      }
    } else {
      stage_issue(tile_n);
    }
    j++;
    u = un;
    g_c = g_n;
    g_n = unn < units ? __builtin_amdgcn_readfirstlane(g_nn_v) : -1;
    mv_c = mv_n;
    fv_c = fv_n;
    tile = tile_n;
    my_row = my_row_n;
  }
}

// ---------------------------------------------------------------------------------------
// Wide 3^3 layers of middling size (a few hundred to a few thousand tiles): one wavefront per unit
// (tile, output block), nothing shared between wavefronts - no barrier, no partial sums through LDS,
// no wait for the slowest of four.  To give the bits of conv_mfma_kernel<1, 27, MAP_NBR, ST> the
// wavefront keeps that kernel's ST partial sums - the items (k, ch) with (k * nch + ch) % ST == p, in
// ascending order, bias in sum 0 - in ST accumulators and adds them in order at the end.  Units
// follow the cost-ordered tile schedule, output blocks of a tile side by side on neighbouring SIMDs of
// one compute unit, so they meet the tile's map slice and gathered rows in L1.
// ---------------------------------------------------------------------------------------
// D = items in flight per wavefront (2 with three wavefronts per SIMD; deeper rings at two wavefronts per
// SIMD measured the same, and so did fewer wavefronts that draw their units from a counter: what the
// launch lasts is the SIMD with the largest sum of items, hence the fixed assignment below).
constexpr int OWN_WAVES = 12;  // one block per compute unit, three wavefronts per SIMD
template <int ST, int D>
__global__ __launch_bounds__(OWN_WAVES * 64) __attribute__((amdgpu_waves_per_eu(3, 3))) void conv_own_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ Wp, const float *__restrict__ bias, const int32_t *__restrict__ rows,
    const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout, int nbt, int nbtp,
    const uint8_t *__restrict__ tile_flags, uint32_t in_bytes, uint32_t wp_bytes, BnEpilogue ep, TilePlan plan) {
  constexpr int K = 27;
  constexpr int NSTAGE = (TILE_M * K + 63) / 64;
  __shared__ int nlb[OWN_WAVES][TILE_M * K];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int64_t ntiles = (n + TILE_M - 1) / TILE_M, units = ntiles * nbt;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int nch = conv_nch(Cin);
  int *nl = nlb[wave];
  // (wavefronts are on their own: no workgroup barrier anywhere below)
  // One block per compute unit; wavefront w sits on SIMD w % 4, so bin = (block, w % 4) names a SIMD and
  // turn = w / 4 one of its three wavefronts.  Units come by falling cost: the first turn hands them to the
  // bins in order, every later turn in reverse order, so the SIMDs that drew the expensive units of the
  // first turn get the cheap ones afterwards (largest sum of a SIMD at 39k sites and 64 channels: 72 items against
  // 90 when every SIMD takes three units in a row; 66 is the best any assignment reaches).
  const int64_t nbins = (int64_t)gridDim.x * 4;
  const int64_t bin = (int64_t)blockIdx.x * 4 + (wave & 3);
  for (int64_t rnd = wave >> 2; rnd * nbins < units; rnd += OWN_WAVES / 4) {
  const int64_t u = rnd * nbins + (rnd == 0 ? bin : nbins - 1 - bin);
  if (u >= units) continue;
  const int tile = __builtin_amdgcn_readfirstlane(plan.sched[u / nbt]);
  const int ob = (int)(u % nbt);
  if (tile_flags && !tile_flags[tile]) continue;
  // (the slice of the last unit has been read to the end before this one overwrites it)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  // the tile's slice of the map: 27 coalesced runs of the plan
  int st[NSTAGE];
#pragma unroll
  for (int i = 0; i < NSTAGE; i++) {
    const int e = i * 64 + lane;  // e = k * 32 + row
    st[i] = e < TILE_M * K ? plan.map[(int64_t)(e >> 5) * plan.ld + (int64_t)tile * TILE_M + (e & 31)] : -1;
  }
  const int64_t pr = (int64_t)tile * TILE_M + r;
  const int my_row = pr < n ? (rows ? rows[pr] : (int)pr) : -1;
  const unsigned tmask = (unsigned)__builtin_amdgcn_readfirstlane((int)plan.tmask[tile]);
  const int c = ob * 32 + r;
  const float bv = (bias && c < Cout) ? bias[c] : 0.0f;
  const float ew = (ep.out2 && c < Cout) ? ep.w[c] : 0.0f;
  const float eb = (ep.out2 && c < Cout) ? ep.b[c] : 0.0f;
#pragma unroll
  for (int i = 0; i < NSTAGE; i++) {
    const int e = i * 64 + lane;
    if (e < TILE_M * K) nl[e] = st[i];
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  f16v acc[ST];
#pragma unroll
  for (int pp = 0; pp < ST; pp++) {
#pragma unroll
    for (int v = 0; v < 16; v++) acc[pp][v] = pp == 0 ? bv : 0.0f;
  }
  if (tmask) {
    struct Cursor {
      int k, ch;
      unsigned rest;
    };
    auto step = [&](const Cursor &cu) -> Cursor {  // past the end: k = -1
      const bool wrap = cu.ch + 1 >= nch;
      const int nk = cu.rest ? __builtin_ctz(cu.rest) : -1;
      Cursor nx;
      nx.ch = wrap ? 0 : cu.ch + 1;
      nx.k = wrap ? nk : cu.k;
      nx.rest = wrap ? (cu.rest & (cu.rest - 1)) : cu.rest;
      return nx;
    };
    const __amdgpu_buffer_rsrc_t rin = make_rsrc(in, in_bytes), rw = make_rsrc(Wp, wp_bytes);
    const uint32_t ld4 = (uint32_t)ld_in * 4u, lane16 = (uint32_t)lane * 16u;
    auto gather = [&](const Cursor &cu) -> Frag {
      const int kk = cu.k < 0 ? 0 : cu.k;
      const int src = nl[kk * TILE_M + r];
      const bool on = cu.k >= 0 && src >= 0 && (h == 0 || Cin - cu.ch * 32 >= 32);
      const uint32_t voff = on ? (uint32_t)src * ld4 + (uint32_t)(cu.ch * 128 + h * 64) : BUF_OOB;
      Frag f;
#pragma unroll
      for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rin, voff + 16u * q, 0);
      return f;
    };
    auto wload = [&](const Cursor &cu) -> Frag {
      const int wt = ((cu.k < 0 ? 0 : cu.k) * nch + cu.ch) * nbtp + ob;
      const uint32_t soff = (uint32_t)__builtin_amdgcn_readfirstlane(wt * 4096);
      const uint32_t voff = cu.k >= 0 ? lane16 : BUF_OOB;
      Frag f;
#pragma unroll
      for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rw, voff + 1024u * q, soff);
      return f;
    };
    const int nitems = __builtin_popcount(tmask) * nch;
    Cursor first;
    first.k = __builtin_ctz(tmask);
    first.ch = 0;
    first.rest = tmask & (tmask - 1);
    Frag g[D], bw[D];
    Cursor ci = first, c0 = first;
#pragma unroll
    for (int d = 0; d < D - 1; d++) {
      g[d] = gather(ci);
      bw[d] = wload(ci);
      ci = step(ci);
    }
    for (int t0i = 0; t0i < nitems; t0i += D) {
#pragma unroll
      for (int uu = 0; uu < D; uu++) {
        g[(uu + D - 1) % D] = gather(ci);
        bw[(uu + D - 1) % D] = wload(ci);
        ci = step(ci);
        // which partial sum the item on the matrix cores belongs to (-1 past the last item)
        const int part = t0i + uu < nitems ? ((c0.k * nch + c0.ch) & (ST - 1)) : -1;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pp = 0; pp < ST; pp++) {
          if (part != pp) continue;  // (one copy of the MFMA block per partial sum: the accumulator is a compile-time choice)
#pragma unroll
          for (int s2 = 0; s2 < 16; s2++)
            acc[pp] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[uu], s2), frag_at(bw[uu], s2), acc[pp], 0, 0, 0);
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        c0 = step(c0);
      }
    }
  }
  // rows and epilogue (D layout of the 32x32 MFMA: lane holds column (lane & 31), rows 8*(v/4) + 4*(lane>>5) + (v&3))
  const __amdgpu_buffer_rsrc_t rout = make_rsrc(out, out ? BUF_OOB : 0u), rout2 = make_rsrc(ep.out2, ep.out2 ? BUF_OOB : 0u);
  const __amdgpu_buffer_rsrc_t rres = make_rsrc(ep.res, ep.res ? BUF_OOB : 0u);
  const uint32_t ldo4 = (uint32_t)ld_out * 4u, ldo24 = (uint32_t)ep.ld2 * 4u, ldr4 = (uint32_t)ep.ldr * 4u;
  int rid[16];
#pragma unroll
  for (int v = 0; v < 16; v++) rid[v] = __shfl(my_row, 8 * (v >> 2) + 4 * h + (v & 3), 64);
  float rv[16];
#pragma unroll
  for (int v = 0; v < 16; v++)
    rv[v] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(
        rres, (int)((rid[v] >= 0 && c < Cout) ? __umul24((unsigned)rid[v], ldr4) + (uint32_t)c * 4u : BUF_OOB), 0, 0));
#pragma unroll
  for (int v = 0; v < 16; v++) {
    const bool ok = rid[v] >= 0 && c < Cout;
    float a = acc[0][v];
#pragma unroll
    for (int pp = 1; pp < ST; pp++) a += acc[pp][v];
    if (ep.res) a += rv[v];
    if (out)
      __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(a), rout,
                                            (int)(ok ? __umul24((unsigned)rid[v], ldo4) + (uint32_t)c * 4u : BUF_OOB), 0, 0);
    if (ep.out2) {
      const float y = fmaf(a, ew, eb);  // fused batch norm + leaky ReLU
      __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(y * ((y > 0.0f) ? 1.0f : ep.leak)), rout2,
                                            (int)(ok ? __umul24((unsigned)rid[v], ldo24) + (uint32_t)c * 4u : BUF_OOB), 0, 0);
    }
  }
  }  // units of this wavefront
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

// map[k * ld + p] = nbr[order[p]][k] for p < n, -1 up to the end of the last tile; tmask[t] = OR of
// the offsets the rows of tile t have.  One thread per position; the writes of one offset are
// coalesced across the wavefront.
__device__ __forceinline__ void tile_plan_body(const int32_t *__restrict__ nbr, const int32_t *__restrict__ order,
                                               const int32_t *__restrict__ d_n, int64_t n_rows, int64_t ld,
                                               int32_t *__restrict__ map, uint32_t *__restrict__ tmask) {
  // A block transposes the rows of 256 positions through LDS: the rows are read 27 consecutive words at a
  // time (consecutive threads, consecutive offsets), the plan is written one 1 KB run per offset.  (With a
  // thread per position reading its own row every load instruction touched 64 different lines.)
  __shared__ int site_l[256];
  __shared__ int row_l[256 * 27];  // [position][offset]: stride 27, odd, so the reads below are conflict-free
  const int64_t n = d_n ? min((int64_t)*d_n, n_rows) : n_rows;
  const int64_t padded = (n + TILE_M - 1) / TILE_M * TILE_M;
  const int64_t p0 = (int64_t)blockIdx.x * 256, p = p0 + threadIdx.x;
  if (p0 >= padded) return;  // (the whole block)
  site_l[threadIdx.x] = p < n ? (order ? order[p] : (int)p) : -1;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 27; i++) {
    const int e = i * 256 + threadIdx.x, lp = e / 27, k = e - lp * 27;
    const int site = site_l[lp];
    row_l[e] = site >= 0 ? nbr[(int64_t)site * 27 + k] : -1;
  }
  __syncthreads();
  if (p >= padded) return;  // whole 32-lane groups leave together (padded is a multiple of 32)
  unsigned m = 0;
#pragma unroll
  for (int k = 0; k < 27; k++) {
    const int v = row_l[threadIdx.x * 27 + k];
    map[(int64_t)k * ld + p] = v;
    if (v >= 0) m |= 1u << k;
  }
#pragma unroll
  for (int d = 16; d > 0; d >>= 1) m |= (unsigned)__shfl_xor((int)m, d, 64);
  if ((threadIdx.x & 31) == 0) tmask[p >> 5] = m;
}
__global__ __launch_bounds__(256) void tile_plan_kernel(const int32_t *__restrict__ nbr,
                                                        const int32_t *__restrict__ order,
                                                        const int32_t *__restrict__ d_n, int64_t n_rows, int64_t ld,
                                                        int32_t *__restrict__ map, uint32_t *__restrict__ tmask) {
  tile_plan_body(nbr, order, d_n, n_rows, ld, map, tmask);
}
// the plans of several maps (the scales of a network) in one launch: blockIdx.y picks the map
__global__ __launch_bounds__(256) void tile_plan_batch_kernel(TilePlanBatch b) {
  const TilePlanJob &j = b.job[blockIdx.y];
  if (!j.nbr) return;  // this plan is up to date: only its schedule is wanted
  tile_plan_body(j.nbr, j.order, j.d_n, j.n_rows, j.ld, j.map, j.tmask);
}

// The columns of the sites added by the last insert, appended to a plan that holds the older
// sites already: positions [first, end of the last tile) of every offset row (first = site count
// before the insert; positions follow the processing order, in which new sites come last).  The
// offset masks of the tiles they open have been cleared beforehand; the mask of a tile is the OR
// over its rows.  One thread per (position, offset).
__global__ __launch_bounds__(256) void tile_plan_append_batch_kernel(TilePlanBatch b) {
  const TilePlanJob &j = b.job[blockIdx.y];
  if (!j.map) return;
  const int64_t first = j.d_n[1], n = j.d_n[0];
  // one wavefront per tile, from the tile that holds position `first` on; lane = (row of the tile,
  // parity of the offset)
  const int lane = threadIdx.x & 63, r = lane & 31, h = lane >> 5;
  const int64_t tile = first / TILE_M + (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile * TILE_M >= n) return;
  const int64_t p = tile * TILE_M + r;
  const bool mine = p >= first;  // (older positions of the first tile keep their entries)
  const int site = (mine && p < n) ? (j.order ? j.order[p] : (int)p) : -1;
  unsigned m = 0;
  for (int k = h; k < 28; k += 2) {
    const int v = (site >= 0 && k < 27) ? j.nbr[(int64_t)site * 27 + k] : -1;
    if (mine && k < 27) j.map[(int64_t)k * j.ld + p] = v;
    const unsigned long long bal = __ballot(v >= 0);
    if ((unsigned)bal) m |= 1u << k;
    if ((unsigned)(bal >> 32)) m |= 1u << (k + 1);
  }
  if (lane == 0 && m) atomicOr(&j.tmask[tile], m);
}

int tile_plan_append_batch(const TilePlanBatch &b, int64_t n_new_upper, hipStream_t s) {
  if (b.n <= 0 || n_new_upper <= 0) return INSC_OK;
  // (the new sites touch at most n_new_upper / 32 + 2 tiles; four tiles per block)
  hipLaunchKernelGGL(tile_plan_append_batch_kernel, dim3(grid_for(n_new_upper / TILE_M + 2, 4), (unsigned)b.n), dim3(256),
                     0, s, b);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

// sched = the tiles by falling number of active offsets (a counting sort over the 28 classes by one
// workgroup; the order inside a class is the order of arrival and has no influence on any result).
__device__ __forceinline__ void tile_sched_body(const uint32_t *__restrict__ tmask, const int32_t *__restrict__ d_n,
                                                int64_t n_rows, int32_t *__restrict__ sched,
                                                int32_t *__restrict__ gsched) {
  __shared__ int cnt[28], base[28];
  const int64_t n = d_n ? min((int64_t)*d_n, n_rows) : n_rows;
  const int64_t ntiles = (n + TILE_M - 1) / TILE_M;
  if (threadIdx.x < 28) cnt[threadIdx.x] = 0;
  __syncthreads();
  for (int64_t t = threadIdx.x; t < ntiles; t += 1024) atomicAdd(&cnt[27 - __builtin_popcount(tmask[t] & 0x7FFFFFFu)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int a = 0;
    for (int c = 0; c < 28; c++) {
      base[c] = a;
      a += cnt[c];
      cnt[c] = 0;
    }
  }
  __syncthreads();
  for (int64_t t = threadIdx.x; t < ntiles; t += 1024) {
    const int c = 27 - __builtin_popcount(tmask[t] & 0x7FFFFFFu);
    sched[base[c] + atomicAdd(&cnt[c], 1)] = (int32_t)t;
  }
  // the same for groups of four consecutive tiles, by the offsets any of the four uses; the group
  // schedule follows the tile schedule at gsched
  const int64_t ngroups = (ntiles + 3) / 4;
  auto gmask = [&](int64_t g) -> unsigned {
    unsigned m = 0;
    for (int64_t t = g * 4; t < min(g * 4 + 4, ntiles); t++) m |= tmask[t];
    return m & 0x7FFFFFFu;
  };
  __syncthreads();
  if (threadIdx.x < 28) cnt[threadIdx.x] = 0;
  __syncthreads();
  for (int64_t g = threadIdx.x; g < ngroups; g += 1024) atomicAdd(&cnt[27 - __builtin_popcount(gmask(g))], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int a = 0;
    for (int c = 0; c < 28; c++) {
      base[c] = a;
      a += cnt[c];
      cnt[c] = 0;
    }
  }
  __syncthreads();
  for (int64_t g = threadIdx.x; g < ngroups; g += 1024) {
    const int c = 27 - __builtin_popcount(gmask(g));
    gsched[base[c] + atomicAdd(&cnt[c], 1)] = (int32_t)g;
  }
}
__global__ __launch_bounds__(1024) void tile_sched_kernel(const uint32_t *__restrict__ tmask,
                                                          const int32_t *__restrict__ d_n, int64_t n_rows,
                                                          int32_t *__restrict__ sched, int32_t *__restrict__ gsched) {
  tile_sched_body(tmask, d_n, n_rows, sched, gsched);
}
__global__ __launch_bounds__(1024) void tile_sched_batch_kernel(TilePlanBatch b) {
  const TilePlanJob &j = b.job[blockIdx.x];
  if (j.sched) tile_sched_body(j.tmask, j.d_n, j.n_rows, j.sched, j.sched + (j.ld + 31) / 32);
}

int build_tile_plans(const TilePlanBatch &b, hipStream_t s) {
  int64_t most = 0;
  bool any_sched = false;
  for (int i = 0; i < b.n; i++) {
    if (b.job[i].nbr) most = std::max(most, cdiv(b.job[i].n_rows, TILE_M) * TILE_M);
    any_sched = any_sched || b.job[i].sched;
  }
  if (b.n <= 0) return INSC_OK;
  if (most > 0) hipLaunchKernelGGL(tile_plan_batch_kernel, dim3(grid_for(most, 256), (unsigned)b.n), dim3(256), 0, s, b);
  if (any_sched) hipLaunchKernelGGL(tile_sched_batch_kernel, dim3((unsigned)b.n), dim3(1024), 0, s, b);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int build_tile_plan(const int32_t *nbr, const int32_t *order, const int32_t *d_n, int64_t n_rows, int64_t ld,
                    int32_t *map, uint32_t *tmask, int32_t *sched, hipStream_t s) {
  if (n_rows <= 0) return INSC_OK;
  const int64_t padded = cdiv(n_rows, TILE_M) * TILE_M;
  hipLaunchKernelGGL(tile_plan_kernel, dim3(grid_for(padded, 256)), dim3(256), 0, s, nbr, order, d_n, n_rows, ld, map,
                     tmask);
  if (sched)
    hipLaunchKernelGGL(tile_sched_kernel, dim3(1), dim3(1024), 0, s, tmask, d_n, n_rows, sched, sched + (ld + 31) / 32);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

static bool conv_uses_mfma(const float *in, int64_t ld_in, int Cin, int K) {
  return Cin % 16 == 0 && ((uintptr_t)in % 16 == 0) && (ld_in % 4 == 0) && (K == 27 || K == 8 || K == 1);
}

int64_t packed_floats(int K, int Cin, int Cout) {
  return (int64_t)K * conv_nch(Cin) * conv_nbt_padded(Cout) * 1024;
}

int pack_weights(const float *W, int K, int Cin, int Cout, float *Wp, hipStream_t s) {
  const int64_t total = packed_floats(K, Cin, Cout);
  hipLaunchKernelGGL(pack_weights_kernel, dim3(grid_for(total, 256, 4096)), dim3(256), 0, s, W, K, Cin, Cout,
                     conv_nch(Cin), conv_nbt_padded(Cout), Wp);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

// Launch policy of wide 3^3 layers (64..159 input channels, a tile schedule).  All kernels give the same
// bits; the bounds only move time.
// The persistent kernel is off by default: since the one-block-per-unit kernel keeps two items in flight
// and numbers its blocks for balance across the compute units it is the faster one at every size measured
// (96 -> 96 at 10k sites: 37 us against 43 us; 64 -> 64 at 21k sites: 36 against 46).
static std::atomic<int64_t> g_pers_min_units{INT64_MAX};
// With at least this many (group of four tiles, output block) units: the kernel whose blocks share the
// weight tiles through LDS (faster from about 60k sites at 64 channels).
static std::atomic<int64_t> g_shared_min_units{896};
// Below that, with at least this many (tile, output block) units - half as many again for layers of more
// than 64 input channels, whose units are longer - the kernel that gives every unit a wavefront of its own
// (64 -> 64 at 39k sites = 2452 units: 50 us against 56 us; 2084 units: 48 against 50; 1840: 41 against 44;
// 1716: 41.1 against 41.5; 1472: 41 against 39 - the split kernel's launch is whole rounds of 1024 blocks, four to
// a compute unit, this kernel's is the SIMD with the most units).
static std::atomic<int64_t> g_own_min_units{1750};
// Narrow 3^3 layers (Cin, Cout <= 32) with at least this many 32-row tiles run on the persistent
// kernel that keeps the whole filter in LDS; smaller ones on the one-wavefront-per-tile kernel.
// Same bits either way.
static std::atomic<int64_t> g_wl_min_tiles{WL_MIN_TILES};

// W: raw [K,Cin,Cout] weights (always needed by the generic kernel); Wp: packed weights or
// null, in which case they are packed into scratch memory first.
// Whether one launch can gather from two sources (BnEpilogue::src2_*): the shapes that the split
// kernel serves - 3^3 layers of a residual frame (latency != 0) and stride-2 deconvolutions, from 32
// input channels on.
bool conv_two_sources_ok(int mode, int K, const float *in, int64_t ld_in, const float *in2, int64_t ld_in2,
                         int64_t in2_rows, int Cin, int latency) {
  if (!in2 || Cin < 32 || !conv_uses_mfma(in, ld_in, Cin, K) || !conv_uses_mfma(in2, ld_in2, Cin, K)) return false;
  if (in2_rows < 0 || in2_rows * ld_in2 * 4 >= (int64_t)BUF_OOB) return false;
  return (mode == MAP_NBR && K == 27 && latency) || (mode == MAP_PARENT && K == 8);
}

int launch_conv(const float *in, int64_t ld_in, int64_t in_rows, float *out, int64_t ld_out, const float *W,
                const float *Wp, const float *bias, const int32_t *map0, const int32_t *map1, int mode, int K,
                const int32_t *rows, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                const uint8_t *tile_flags, const uint8_t *row_mask, hipStream_t s, BnEpilogue ep, TilePlan plan,
                int latency, int64_t expect_rows) {
  if (n_rows == 0) return INSC_OK;
  if (ep.side_in && !(mode == MAP_PARENT && K == 8 && conv_uses_mfma(in, ld_in, Cin, K) && ep.side_out && ep.side_w && ep.side_b)) {
    set_error("conv: a second batch norm in the epilogue is for deconvolutions on the matrix-core kernel only");
    return INSC_ERR_ARG;
  }
  if (ep.src2_in && !conv_two_sources_ok(mode, K, in, ld_in, ep.src2_in, ep.src2_ld, ep.src2_rows, Cin, latency)) {
    set_error("conv: no kernel with two sources for this shape (K=%d, map mode %d, Cin=%d)", K, mode, Cin);
    return INSC_ERR_ARG;
  }
  if (ep.src2_in) plan = TilePlan();  // (a plan describes the first source's map only)
  if (ep.pre_exist && !(ep.out2 && ep.pre_in && ep.pre_out && latency && mode == MAP_NBR && K == 27 && Cin >= 32 &&
                        conv_uses_mfma(in, ld_in, Cin, K))) {
    set_error("conv: the batch norm of a residual frame is fused into 3^3 layers on the split kernel only (Cin=%d)", Cin);
    return INSC_ERR_ARG;
  }
  if (expect_rows <= 0 || expect_rows > n_rows) expect_rows = n_rows;
  if (plan.map && (mode != MAP_NBR || K != 27 || plan.ld * 27 * 4 >= (int64_t)BUF_OOB || plan.ld < cdiv(n_rows, TILE_M) * TILE_M))
    plan = TilePlan();  // only the 3^3 map has a plan; an unusable one is ignored
  plan.cus = (unsigned)device_cus();
  if (conv_uses_mfma(in, ld_in, Cin, K)) {
    // the gather addresses rows with 32-bit byte offsets (buffer loads)
    const int64_t in_bytes64 = in_rows * ld_in * 4, wp_bytes64 = packed_floats(K, Cin, Cout) * 4;
    if (in_rows < 0 || in_bytes64 >= (int64_t)BUF_OOB || wp_bytes64 >= (int64_t)BUF_OOB) {
      set_error("conv: input matrix (%lld rows x %lld floats) or weights exceed the 4 GB the kernel addresses",
                (long long)in_rows, (long long)ld_in);
      return INSC_ERR_ARG;
    }
    const uint32_t in_bytes = (uint32_t)in_bytes64, wp_bytes = (uint32_t)wp_bytes64;
    if (!Wp) {
      void *ws;
      int rc = workspace(WS_API, s, sizeof(float) * (size_t)packed_floats(K, Cin, Cout), &ws);
      if (rc) return rc;
      rc = pack_weights(W, K, Cin, Cout, (float *)ws, s);
      if (rc) return rc;
      Wp = (const float *)ws;
    }
    const int64_t tiles = cdiv(n_rows, TILE_M);
    // Rows of the neighbour map and of the outputs: one per listed row, or - with a row list,
    // which only 3^3 layers over one site set use - one per input site.  (The two differ when a
    // layer gathers from another site set than the one it writes.)
    const int64_t out_rows = rows ? in_rows : std::max(in_rows, n_rows);
    const int64_t map_bytes64 = out_rows * 27 * 4;
    // (row ids and row strides go through 24-bit multiplies)
    const bool small_ids = in_rows < (1 << 24) && out_rows < (1 << 24) && ld_out * 4 < (1 << 24) &&
                           ep.ld2 * 4 < (1 << 24) && out_rows * ld_out * 4 < (int64_t)BUF_OOB &&
                           out_rows * ep.ld2 * 4 < (int64_t)BUF_OOB;
    // (below some four thousand tiles the persistent kernel's start-up - every block copies the
    // whole filter into LDS - costs more than it saves: 34 us against 21 us at 32k sites, even at
    // 150k; both kernels give the same bits)
    if (mode == MAP_NBR && K == 27 && Cin <= 32 && Cout <= 32 && map_bytes64 < (int64_t)BUF_OOB && small_ids &&
        cdiv(expect_rows, TILE_M) >= g_wl_min_tiles.load(std::memory_order_relaxed) && !latency) {
      const uint32_t map_bytes = (uint32_t)map_bytes64;
      // persistent blocks, a multiple of the XCD count, at most one per compute unit
      const int64_t want = cdiv(tiles, WL_WAVES);
      const unsigned nblk = (unsigned)std::min<int64_t>(device_cus(), want);
      hipLaunchKernelGGL(conv_wlds_kernel, dim3(nblk), dim3(WL_WAVES * 64), 0, s, in, ld_in, out, ld_out, Wp, bias,
                         map0, rows, d_n_rows, n_rows, Cin, Cout, tile_flags, in_bytes, map_bytes, ep, plan);
      INSC_LAUNCH_CHECK();
      return INSC_OK;
    }
    const int nbt = (Cout + 31) / 32;
    // Launch shape, a function of the layer shape only (so results never depend on the scene):
    //  Cin < 64: each wavefront computes all output blocks of its tile (the gathered rows are
    //    reused across them);
    //  wider layers sit at the coarse scales of a U-Net, which have few tiles: one output block
    //    per wavefront, and for 3^3 / 2^3 maps the items of a tile are dealt to S wavefronts
    //    (four for 3^3) in each of G blocks.
    // latency != 0 (residual frames: a few thousand rows at most, so a launch lasts as long as
    // its most expensive tile): the items of every 3^3 tile are dealt to four wavefronts whatever
    // the width, and to more blocks for the wide layers.  Also a function of the layer shape only.
    const bool lat = latency && mode == MAP_NBR && K == 27 && Cin >= 32;
    const bool two = ep.src2_in != nullptr;  // (checked above: a shape that the split kernel serves)
    const bool split = lat || two || (Cin >= 64 && K > 1 && (mode == MAP_NBR || (mode == MAP_PARENT && Cin >= 96)));
    const int NB0 = split ? 1 : conv_nb_per_group(Cout);
    const int nbtp = conv_nbt_padded(Cout);
    int S = 1;
    if (split) S = K == 27 ? (Cin >= 160 ? 8 : 4) : ((Cin >= 96 || two) ? 4 : 1);  // K == 8: conv and deconv
    const int NB = (S == 1 && Cin >= 96) ? 1 : NB0;
    // (the split across blocks is for scales with few tiles; in a U-Net the width grows with the depth,
    // and a layer that narrows to at most 96 channels sits at a fine scale with many tiles)
    // (eight blocks from 224 -> 192 channels: the two coarsest scales of a seven-scale U-Net, a few tiles,
    // where a wavefront's item loop is most of the launch - 224 -> 224 at 70 sites 15 -> 12 us; at 192 input
    // channels, and for 256 -> 128 and 320 -> 160 with their more numerous tiles, it gains nothing)
    int G = (split && K == 27 && Cout > 96) ? ((Cin >= 224 && Cout >= 192) ? 8 : Cin >= 160 ? 4 : Cin >= 128 ? 2 : 1) : 1;
    if (lat) {
      G = Cin >= 128 ? 4 : Cin >= 64 ? 2 : 1;
      S = 4;
    }
    if (G > 1) S = 4;
    const bool wide_planned = mode == MAP_NBR && K == 27 && S == 4 && G == 1 && !lat && plan.map && plan.sched &&
                              small_ids && ep.ldr * 4 < (1 << 24) && out_rows * ep.ldr * 4 < (int64_t)BUF_OOB;
    // (a layer with one output block has half the weight bytes per gathered row to share: 64 -> 32 at 150k
    // sites takes 95 us there against 88 us with a wavefront per unit, so its bound is twice as high)
    if (wide_planned && cdiv(tiles, 4) * nbt >= g_shared_min_units.load(std::memory_order_relaxed) * (nbt == 1 ? 2 : 1)) {
      // blocks of four tiles that share the weight tiles through LDS
      // with enough units left, two output blocks per gathered chunk (eight accumulators: two
      // wavefronts per SIMD instead of three, but a third fewer bytes per MFMA)
      if (nbt >= 2 && cdiv(tiles, 4) * cdiv(nbt, 2) * 3 >= g_shared_min_units.load(std::memory_order_relaxed) * 2) {
        static int per_cu4 = 0;
        if (!per_cu4) {
          INSC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu4, conv_wshare_kernel<2, 4>, 256, 0));
          if (per_cu4 < 1) per_cu4 = 1;
        }
        const int64_t wunits = cdiv(tiles, 4) * cdiv(nbt, 2);
        const unsigned nblk = (unsigned)std::min<int64_t>((int64_t)device_cus() * per_cu4, wunits);
        hipLaunchKernelGGL((conv_wshare_kernel<2, 4>), dim3(nblk), dim3(256), 0, s, in, ld_in, out, ld_out, Wp, bias, rows,
                           d_n_rows, n_rows, Cin, Cout, nbt, nbtp, tile_flags, in_bytes, wp_bytes, ep, plan);
        INSC_LAUNCH_CHECK();
        return INSC_OK;
      }
      static int per_cu2 = 0;
      if (!per_cu2) {
        INSC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu2, conv_wshare_kernel<1, 4>, 256, 0));
        if (per_cu2 < 1) per_cu2 = 1;
      }
      const int64_t wunits = cdiv(tiles, 4) * nbt;
      const unsigned nblk = (unsigned)std::min<int64_t>((int64_t)device_cus() * per_cu2, wunits);
      hipLaunchKernelGGL((conv_wshare_kernel<1, 4>), dim3(nblk), dim3(256), 0, s, in, ld_in, out, ld_out, Wp, bias, rows,
                         d_n_rows, n_rows, Cin, Cout, nbt, nbtp, tile_flags, in_bytes, wp_bytes, ep, plan);
      INSC_LAUNCH_CHECK();
      return INSC_OK;
    }
    const int64_t own_min = g_own_min_units.load(std::memory_order_relaxed);
    if (wide_planned && tiles * nbt >= (Cin > 64 ? own_min + own_min / 2 : own_min)) {
      // one wavefront per (tile, output block): enough units that every SIMD gets one to three
      hipLaunchKernelGGL((conv_own_kernel<4, 2>), dim3((unsigned)device_cus()), dim3(OWN_WAVES * 64), 0, s, in, ld_in, out,
                         ld_out, Wp, bias, rows, d_n_rows, n_rows, Cin, Cout, nbt, nbtp, tile_flags, in_bytes, wp_bytes, ep,
                         plan);
      INSC_LAUNCH_CHECK();
      return INSC_OK;
    }
    if (wide_planned && tiles * nbt >= g_pers_min_units.load(std::memory_order_relaxed)) {
      // persistent blocks, as many as fit on the device at once
      static int per_cu = 0;
      if (!per_cu) {
        INSC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, conv_pers_kernel<4>, 256, 0));
        if (per_cu < 1) per_cu = 1;
      }
      const unsigned nblk = (unsigned)std::min<int64_t>((int64_t)device_cus() * per_cu, tiles * nbt);
      hipLaunchKernelGGL(conv_pers_kernel<4>, dim3(nblk), dim3(256), 0, s, in, ld_in, out, ld_out, Wp, bias, rows,
                         d_n_rows, n_rows, Cin, Cout, nbt, nbtp, tile_flags, in_bytes, wp_bytes, ep, plan);
      INSC_LAUNCH_CHECK();
      return INSC_OK;
    }
    const unsigned gx = (unsigned)(S == 1 ? cdiv(tiles, CONV_WAVES) : tiles);
    const int GZ = two ? 2 * G : G;  // blocks per (tile, output block): G per source
    dim3 grid(gx, (unsigned)(NB == 1 ? nbt : nbtp / NB), (unsigned)GZ), block((S == 1 ? CONV_WAVES : S) * 64);
    float *part = nullptr;
    int32_t *pcount = nullptr;
    if (GZ > 1) {
      const size_t units = (size_t)gx * grid.y;
      void *ws;
      int rc = workspace(WS_CONV, s, units * GZ * 1024 * sizeof(float), &ws);
      if (rc) return rc;
      part = (float *)ws;
      if ((rc = zero_counters(s, units * (size_t)S, &pcount))) return rc;  // one counter per wavefront of a unit
    }
    bool shape_ok = true;
#define INSC_CONV_LAUNCH(NBV, KV, MV, SV)                                                                       \
  hipLaunchKernelGGL((conv_mfma_kernel<NBV, KV, MV, SV>), grid, block, 0, s, in, ld_in, out, ld_out, Wp, bias,  \
                     map0, map1, rows, d_n_rows, n_rows, Cin, Cout, nbtp, tile_flags, in_bytes, wp_bytes, ep, part,  \
                     pcount, plan)
#define INSC_CONV_CASE(NBV)                                      \
  case NBV:                                                      \
    if (mode == MAP_NBR && K == 27)                              \
      INSC_CONV_LAUNCH(NBV, 27, MAP_NBR, 1);                     \
    else if (mode == MAP_NBR && K == 8)                          \
      INSC_CONV_LAUNCH(NBV, 8, MAP_NBR, 1);                      \
    else if (mode == MAP_PARENT && K == 8)                       \
      INSC_CONV_LAUNCH(NBV, 8, MAP_PARENT, 1);                   \
    else if (mode == MAP_IDENTITY && K == 1)                     \
      INSC_CONV_LAUNCH(NBV, 1, MAP_IDENTITY, 1);                 \
    else                                                         \
      shape_ok = false;                                          \
    break;
    if (S > 1 && mode == MAP_NBR && K == 27) {
      switch (S) {
        case 2: INSC_CONV_LAUNCH(1, 27, MAP_NBR, 2); break;
        case 4: INSC_CONV_LAUNCH(1, 27, MAP_NBR, 4); break;
        case 8: INSC_CONV_LAUNCH(1, 27, MAP_NBR, 8); break;
        default: shape_ok = false;
      }
    } else if (S > 1 && mode == MAP_NBR && K == 8) {
      switch (S) {
        case 4: INSC_CONV_LAUNCH(1, 8, MAP_NBR, 4); break;
        default: shape_ok = false;
      }
    } else if (S == 4 && mode == MAP_PARENT && K == 8) {
      INSC_CONV_LAUNCH(1, 8, MAP_PARENT, 4);
    } else if (S > 1) {
      shape_ok = false;
    } else {
      switch (NB) {
        INSC_CONV_CASE(1)
        INSC_CONV_CASE(2)
        INSC_CONV_CASE(3)
        INSC_CONV_CASE(4)
        default:
          shape_ok = false;
      }
    }
    if (!shape_ok) {
      set_error("conv: no matrix-core kernel for K=%d with map mode %d", K, mode);
      return INSC_ERR_ARG;
    }
#undef INSC_CONV_LAUNCH
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
    if (mode == MAP_NBR && K == 27 && Cin <= 4) {
      // enough blocks to fill the machine, few enough that the weights are fetched rarely
      const dim3 sg(grid_for(n_rows, std::min(cpb, STEM_ROWS), (unsigned)device_cus() * 8));
#define INSC_STEM(CI)                                                                                          \
  hipLaunchKernelGGL(conv_stem_kernel<CI>, sg, dim3(256), 0, s, in, ld_in, out, ld_out, W, bias, map0, rows, \
                     d_n_rows, n_rows, Cout, row_mask, ep)
      if (Cin == 1)
        INSC_STEM(1);
      else if (Cin == 2)
        INSC_STEM(2);
      else if (Cin == 3)
        INSC_STEM(3);
      else
        INSC_STEM(4);
#undef INSC_STEM
      INSC_LAUNCH_CHECK();
      return INSC_OK;
    }
    hipLaunchKernelGGL(conv_generic_kernel, dim3(grid_for(n_rows, cpb, 65536)), dim3(256), 0, s, in, ld_in, out,
                       ld_out, W, bias, map0, map1, mode, K, rows, d_n_rows, n_rows, Cin, Cout, row_mask, ep);
  }
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_conv_set_persistent_min_units(int64_t units) {
  INSC_REQUIRE(units >= 1, INSC_ERR_ARG, "insc_conv_set_persistent_min_units: units must be >= 1");
  g_pers_min_units.store(units, std::memory_order_relaxed);
  return INSC_OK;
}

int insc_conv_set_shared_weights_min_units(int64_t units) {
  INSC_REQUIRE(units >= 1, INSC_ERR_ARG, "insc_conv_set_shared_weights_min_units: units must be >= 1");
  g_shared_min_units.store(units, std::memory_order_relaxed);
  return INSC_OK;
}

int insc_conv_set_wavefront_per_unit_min_units(int64_t units) {
  INSC_REQUIRE(units >= 1, INSC_ERR_ARG, "insc_conv_set_wavefront_per_unit_min_units: units must be >= 1");
  g_own_min_units.store(units, std::memory_order_relaxed);
  return INSC_OK;
}

int insc_conv_set_filter_lds_min_tiles(int64_t tiles) {
  INSC_REQUIRE(tiles >= 1, INSC_ERR_ARG, "insc_conv_set_filter_lds_min_tiles: tiles must be >= 1");
  g_wl_min_tiles.store(tiles, std::memory_order_relaxed);
  return INSC_OK;
}

int64_t insc_conv_packed_floats(int K, int Cin, int Cout) {
  if (K <= 0 || Cin <= 0 || Cout <= 0) return 0;
  return packed_floats(K, Cin, Cout);
}

int insc_conv_pack_weights(const float *d_W, int K, int Cin, int Cout, float *d_Wp, void *stream) {
  INSC_REQUIRE(d_W && d_Wp && K > 0 && K <= MAXK && Cin > 0 && Cout > 0, INSC_ERR_ARG,
               "insc_conv_pack_weights: bad arguments");
  return pack_weights(d_W, K, Cin, Cout, d_Wp, (hipStream_t)stream);
}

int insc_conv_nbr(const float *d_in, int64_t ld_in, int64_t n_in_rows, float *d_out, int64_t ld_out,
                  const float *d_W, const float *d_Wp, const float *d_bias, const int32_t *d_nbr, int K,
                  const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                  double *h_muladds, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && Cin > 0 && Cout > 0 && K > 0 && K <= MAXK, INSC_ERR_ARG,
               "insc_conv_nbr: bad sizes (n_rows=%lld Cin=%d Cout=%d K=%d)", (long long)n_rows, Cin, Cout, K);
  INSC_REQUIRE(ld_in >= Cin && ld_out >= Cout, INSC_ERR_ARG, "insc_conv_nbr: row stride smaller than channel count");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && (d_W || d_Wp)), INSC_ERR_ARG, "insc_conv_nbr: null pointer");
  INSC_REQUIRE(d_nbr || K == 1, INSC_ERR_ARG, "insc_conv_nbr: a null map needs K == 1");
  hipStream_t s = (hipStream_t)stream;
  INSC_REQUIRE(n_in_rows >= 0, INSC_ERR_ARG, "insc_conv_nbr: n_in_rows is negative");
  int rc = launch_conv(d_in, ld_in, n_in_rows, d_out, ld_out, d_W, d_Wp, d_bias, d_nbr, nullptr,
                       d_nbr ? MAP_NBR : MAP_IDENTITY, K, d_rows, d_n_rows, n_rows, Cin, Cout, nullptr, nullptr, s);
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

int insc_plan_build(const int32_t *d_nbr, const int32_t *d_order, const int32_t *d_n_rows, int64_t n_rows,
                    int64_t plan_ld, int32_t *d_plan, uint32_t *d_tmask, int32_t *d_sched, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && plan_ld >= cdiv(n_rows, TILE_M) * TILE_M, INSC_ERR_ARG,
               "insc_plan_build: plan_ld must cover the rows rounded up to a multiple of 32");
  INSC_REQUIRE(n_rows == 0 || (d_nbr && d_plan && d_tmask), INSC_ERR_ARG, "insc_plan_build: null pointer");
  return build_tile_plan(d_nbr, d_order, d_n_rows, n_rows, plan_ld, d_plan, d_tmask, d_sched, (hipStream_t)stream);
}

int insc_conv_ssc_plan(const float *d_in, int64_t ld_in, int64_t n_in_rows, float *d_out, int64_t ld_out,
                       const float *d_W, const float *d_Wp, const float *d_bias, const int32_t *d_nbr,
                       const int32_t *d_plan, int64_t plan_ld, const uint32_t *d_tmask, const int32_t *d_sched,
                       const int32_t *d_order, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                       void *stream) {
  INSC_REQUIRE(n_rows >= 0 && Cin > 0 && Cout > 0 && n_in_rows >= 0, INSC_ERR_ARG, "insc_conv_ssc_plan: bad sizes");
  INSC_REQUIRE(ld_in >= Cin && ld_out >= Cout, INSC_ERR_ARG, "insc_conv_ssc_plan: row stride smaller than channel count");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && (d_W || d_Wp) && d_nbr && d_plan && d_tmask), INSC_ERR_ARG,
               "insc_conv_ssc_plan: null pointer");
  INSC_REQUIRE(plan_ld >= cdiv(n_rows, TILE_M) * TILE_M, INSC_ERR_ARG, "insc_conv_ssc_plan: plan_ld too small");
  TilePlan plan;
  plan.map = d_plan;
  plan.ld = plan_ld;
  plan.tmask = d_tmask;
  plan.sched = d_sched;
  return launch_conv(d_in, ld_in, n_in_rows, d_out, ld_out, d_W, d_Wp, d_bias, d_nbr, nullptr, MAP_NBR, 27, d_order,
                     d_n_rows, n_rows, Cin, Cout, nullptr, nullptr, (hipStream_t)stream, BnEpilogue(), plan);
}

int insc_deconv_down2(const float *d_in, int64_t ld_in, int64_t n_in_rows, float *d_out, int64_t ld_out,
                      const float *d_W, const float *d_Wp, const float *d_bias, const int32_t *d_parent,
                      const int32_t *d_offset, const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows,
                      int Cin, int Cout, void *stream) {
  INSC_REQUIRE(n_rows >= 0 && Cin > 0 && Cout > 0, INSC_ERR_ARG, "insc_deconv_down2: bad sizes");
  INSC_REQUIRE(ld_in >= Cin && ld_out >= Cout, INSC_ERR_ARG, "insc_deconv_down2: row stride too small");
  INSC_REQUIRE(n_rows == 0 || (d_in && d_out && (d_W || d_Wp) && d_parent && d_offset), INSC_ERR_ARG,
               "insc_deconv_down2: null pointer");
  INSC_REQUIRE(n_in_rows >= 0, INSC_ERR_ARG, "insc_deconv_down2: n_in_rows is negative");
  return launch_conv(d_in, ld_in, n_in_rows, d_out, ld_out, d_W, d_Wp, d_bias, d_parent, d_offset, MAP_PARENT, 8, d_rows,
                     d_n_rows, n_rows, Cin, Cout, nullptr, nullptr, (hipStream_t)stream);
}

}  // extern "C"
