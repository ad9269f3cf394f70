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
    if (out) out[(int64_t)row * ld_out + co] = acc;
    if (ep.out2) {
      const float y = fmaf(acc, ep.w[co], ep.b[co]);
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

// Lanes whose row has no neighbour at the current offset read this row of zeros instead, so
// the gather needs no branch and no select.
__device__ __attribute__((aligned(64))) float g_zero_row[16];  // all lanes read the first 16 bytes

__device__ __forceinline__ Frag load_frag(const float *p) {
  Frag f;
  const float4 *p4 = reinterpret_cast<const float4 *>(p);
#pragma unroll
  for (int i = 0; i < 4; i++) f.q[i] = p4[i];
  return f;
}
// weight tile: quarter q of the tile starts at q*256 floats, this lane's values at lane*4
__device__ __forceinline__ Frag load_wfrag(const float *tile, int lane) {
  Frag f;
  const float4 *p4 = reinterpret_cast<const float4 *>(tile) + lane;
#pragma unroll
  for (int i = 0; i < 4; i++) f.q[i] = p4[i * 64];
  return f;
}
__device__ __forceinline__ float frag_at(const Frag &f, int s) {
  const float4 v = f.q[s >> 2];
  return (s & 3) == 0 ? v.x : (s & 3) == 1 ? v.y : (s & 3) == 2 ? v.z : v.w;
}

// LDS row stride of the gather tile in floats: 32 channels + 4 of padding, so that both the
// row-wise 16-byte writes and the column-block reads of the MFMA layout spread over all banks.
constexpr int AT_LD = 36;

// Gather flavour.  DIRECT_GATHER: every lane reads the 64 bytes of its own input row that the
// MFMA A operand needs, with buffer loads: one 32-bit offset per item, rows without a
// neighbour get an out-of-range offset and the hardware returns zeros, and the weight tile is
// addressed by a scalar offset - a handful of non-MFMA instructions per 16 MFMAs (ordinary
// VALU work does not overlap with MFMAs on this part, so it is paid in matrix-core time).
// Otherwise: coalesced 128-byte row segments, transposed through LDS into the A layout
// (fewer cache-line touches per instruction, but ~100 extra instructions per item).
#ifndef INSC_CONV_DIRECT
#define INSC_CONV_DIRECT 1
#endif
constexpr bool DIRECT_GATHER = INSC_CONV_DIRECT != 0;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// offsets at or beyond this bound make a buffer load return zeros
constexpr uint32_t BUF_OOB = 0xFFFFFF00u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
}

// S == 1: every wavefront of the block owns a tile and walks all of its filter offsets.
// S  > 1: the S wavefronts of a block share ONE tile; wavefront w takes the offsets k with
//         k % S == w and the partial sums are added in wavefront order at the end.  This is for
//         the coarse scales of a U-Net, where a layer has a handful of tiles but hundreds of
//         channels and a single wavefront would run tens of thousands of dependent MFMAs.  Which
//         terms a wavefront sums depends on k only, so a row's result is a function of S alone
//         (S is a fixed property of the layer shape), never of the tile it happens to sit in.
template <int NB, int K, int MODE, int S>
__global__ __launch_bounds__((S == 1 ? CONV_WAVES : S) * 64) void conv_mfma_kernel(
    const float *__restrict__ in, int64_t ld_in, float *__restrict__ out, int64_t ld_out,
    const float *__restrict__ Wp, const float *__restrict__ bias, const int32_t *__restrict__ map0,
    const int32_t *__restrict__ map1, const int32_t *__restrict__ rows,
    const int32_t *__restrict__ d_n_rows, int64_t n_rows, int Cin, int Cout, int nbtp,
    const uint8_t *__restrict__ tile_flags, uint32_t in_bytes, uint32_t wp_bytes, BnEpilogue ep) {
  static_assert(S == 1 || NB == 1, "split tiles use one output block per wavefront");
  constexpr int WAVES = S == 1 ? CONV_WAVES : S;
  __shared__ int nbl[S == 1 ? WAVES : 1][TILE_M * K];
  __shared__ __attribute__((aligned(16))) float atile[DIRECT_GATHER ? 1 : WAVES][DIRECT_GATHER ? 4 : TILE_M * AT_LD];
  __shared__ float red[S > 1 ? S - 1 : 1][S > 1 ? 16 * 64 : 1];
  const int64_t n = d_n_rows ? min((int64_t)*d_n_rows, n_rows) : n_rows;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int64_t t0 = (S == 1 ? (int64_t)blockIdx.x * WAVES + wave : (int64_t)blockIdx.x) * TILE_M;
  const int cb0 = blockIdx.y * NB;  // first output-channel block of this column group
  const int nch = conv_nch(Cin);

  // a tile is skipped when it lies beyond the row count or, with tile flags, is not marked
  const bool live = t0 < n && (!tile_flags || tile_flags[t0 >> 5]);
  int my_row = -1;
  if (live && t0 + r < n) my_row = rows ? rows[t0 + r] : (int)(t0 + r);

  // stage the tile's slice of the neighbour map in LDS and find the offsets it uses; all the
  // loads are issued before the first one is consumed
  int *nl = nbl[S == 1 ? wave : 0];
  unsigned mymask = 0;
  constexpr int NSTAGE = (TILE_M * K + 64 * S - 1) / (64 * S);
  int staged[NSTAGE];
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
  if (S == 1) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) mymask |= (unsigned)__shfl_xor((int)mymask, d, 64);
  }
  __syncthreads();
  if (!live) return;  // the whole block (S > 1) or wavefront (S == 1) is idle; no barrier follows
  unsigned rest;
  if (S == 1) {
    rest = (unsigned)__builtin_amdgcn_readfirstlane((int)mymask);
  } else {
    // offsets of this wavefront that some row of the tile uses
    rest = 0;
    for (int k = wave; k < K; k += S)
      if (__ballot(nl[r * K + k] >= 0) != 0ull) rest |= 1u << k;
  }

  f16v acc[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) {
    const int c = (cb0 + b) * 32 + r;
    const float bv = (bias && c < Cout && (S == 1 || wave == 0)) ? bias[c] : 0.0f;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[b][v] = bv;
  }

  if (rest) {
    // Work items of this tile: (active offset k, 32-channel chunk ch), in order.
    struct Item {
      int k, ch;
    };
    // next item, or the same item again with `last` set when there is none
    auto advance = [&](Item it, bool &last) -> Item {
      last = false;
      if (it.ch + 1 < nch) {
        it.ch++;
      } else if (rest) {
        it.k = __builtin_ctz(rest);
        rest &= rest - 1;
        it.ch = 0;
      } else {
        last = true;
      }
      return it;
    };
    Item it0;
    it0.k = __builtin_ctz(rest);
    rest &= rest - 1;
    it0.ch = 0;
    // Pipeline: while item t runs on the matrix cores, the gathers of items t+1 and t+2 and the
    // weight tile(s) of the next item(s) are in flight.  Register slots are compile-time (the
    // loop bodies are unrolled) because copying a fragment would wait for the load that fills
    // it.  Every load is issued unconditionally (past the last item the last item is simply
    // fetched again): a load under a branch would force the wait before the MFMAs to drain all
    // outstanding loads, which serialises the pipeline.  The sched_barrier / memory-clobber
    // pairs keep the loads above the MFMAs they overlap and their consumers below.
    bool last0, last1;
    if constexpr (DIRECT_GATHER) {
      const __amdgpu_buffer_rsrc_t rin = make_rsrc(in, in_bytes), rw = make_rsrc(Wp, wp_bytes);
      const uint32_t ld4 = (uint32_t)ld_in * 4u, lane16 = (uint32_t)lane * 16u;
      // lane (r, h) reads channels ch*32 + h*16 .. +15 of its own row; the second half-wave of
      // a 16-channel tail chunk has no channels
      auto gather = [&](const Item &it) -> Frag {
        const int src = nl[r * K + it.k];
        const bool on = src >= 0 && (h == 0 || Cin - it.ch * 32 >= 32);
        const uint32_t voff = on ? (uint32_t)src * ld4 + (uint32_t)(it.ch * 128 + h * 64) : BUF_OOB;
        Frag f;
#pragma unroll
        for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rin, voff + 16u * q, 0);
        return f;
      };
      auto wload = [&](const Item &it, int b) -> Frag {
        const uint32_t soff = (uint32_t)((((it.k * nch + it.ch) * nbtp) + cb0 + b) * 4096);
        Frag f;
#pragma unroll
        for (int q = 0; q < 4; q++) f.q[q] = buf_load16(rw, lane16 + 1024u * q, soff);
        return f;
      };
      Frag g[3];
      g[0] = gather(it0);
      Item it1 = advance(it0, last0);  // last0: it0 is the final item
      g[1] = gather(it1);
      if constexpr (S == 1) {
        Frag bw[2];
        bw[0] = wload(it0, 0);
        bool done = false;
        while (!done) {
#pragma unroll
          for (int u = 0; u < 6; u++) {
            // item t = g[u%3] (arrived or arriving), t+1 = g[(u+1)%3] in flight, slot (u+2)%3 free
            const Item it2 = advance(it1, last1);
            g[(u + 2) % 3] = gather(it2);
#pragma unroll
            for (int b = 0; b < NB; b++) {
              const int nn = u * NB + b;
              bw[(nn + 1) % 2] = (b + 1 < NB) ? wload(it0, b + 1) : wload(it1, 0);
              asm volatile("" ::: "memory");
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int s = 0; s < 16; s++)
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[u % 3], s), frag_at(bw[nn % 2], s), acc[b],
                                                              0, 0, 0);
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            if (last0) {
              done = true;
              break;
            }
            it0 = it1;
            it1 = it2;
            last0 = last1;
          }
        }
      } else {
        // few wavefronts per SIMD: the weight tiles are fetched two items ahead as well
        Frag bw[3];
        bw[0] = wload(it0, 0);
        bw[1] = wload(it1, 0);
        bool done = false;
        while (!done) {
#pragma unroll
          for (int u = 0; u < 3; u++) {
            const Item it2 = advance(it1, last1);
            g[(u + 2) % 3] = gather(it2);
            bw[(u + 2) % 3] = wload(it2, 0);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 16; s++)
              acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(g[u % 3], s), frag_at(bw[u % 3], s), acc[0], 0,
                                                            0, 0);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            if (last0) {
              done = true;
              break;
            }
            it0 = it1;
            it1 = it2;
            last0 = last1;
          }
        }
      }
    } else {
      const int64_t wtile = 1024;  // floats per (k, chunk, block) weight tile
      // Gather of one item, coalesced: load i (0..3) of lane l reads 16 bytes of input row
      // 8*i + l/8 at channel 4*(l%8), so eight lanes cover one 128-byte row segment and every
      // quad of lanes reads 64 contiguous bytes.  Rows without a neighbour (and the upper half
      // of a 16-channel tail chunk) read a row of zeros.
      const int grow = lane >> 3, gcol = (lane & 7) * 4;
      auto gather = [&](const Item &it) -> Frag {
        Frag f;
        const bool col_ok = it.ch * 32 + gcol < Cin;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int src = nl[(8 * i + grow) * K + it.k];
          const float *p = (src >= 0 && col_ok) ? in + (int64_t)src * ld_in + it.ch * 32 + gcol : g_zero_row;
          f.q[i] = *reinterpret_cast<const float4 *>(p);
        }
        return f;
      };
      // through LDS into the MFMA A layout: lane (r, h) gets channels h*16 .. h*16+15 of row r
      float *at = atile[wave];
      auto transpose = [&](const Frag &gg) -> Frag {
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<float4 *>(at + (8 * i + grow) * AT_LD + gcol) = gg.q[i];
        Frag a;
#pragma unroll
        for (int q = 0; q < 4; q++) a.q[q] = *reinterpret_cast<const float4 *>(at + r * AT_LD + h * 16 + 4 * q);
        return a;
      };
      auto wtile_of = [&](const Item &it, int b) -> const float * {
        return Wp + (((int64_t)it.k * nch + it.ch) * nbtp + cb0 + b) * wtile;
      };
      Frag g[2], bw[2];
      g[0] = gather(it0);
      bw[0] = load_wfrag(wtile_of(it0, 0), lane);
      Item it1 = advance(it0, last0);
      g[1] = gather(it1);
      Frag a = transpose(g[0]);
      bool done = false;
      while (!done) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
          const Item it2 = advance(it1, last1);
          g[u % 2] = gather(it2);
#pragma unroll
          for (int b = 0; b < NB; b++) {
            const int nn = u * NB + b;
            if (b + 1 < NB)
              bw[(nn + 1) % 2] = load_wfrag(wtile_of(it0, b + 1), lane);
            else
              bw[(nn + 1) % 2] = load_wfrag(wtile_of(it1, 0), lane);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 16; s++)
              acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_at(a, s), frag_at(bw[nn % 2], s), acc[b], 0, 0, 0);
          }
          asm volatile("" ::: "memory");
          __builtin_amdgcn_sched_barrier(0);
          if (last0) {
            done = true;
            break;
          }
          a = transpose(g[(u + 1) % 2]);
          it0 = it1;
          it1 = it2;
          last0 = last1;
        }
      }
    }
  }

  if (S > 1) {
    // partial sums of wavefronts 1..S-1 go through LDS and are added in wavefront order
    if (wave > 0) {
#pragma unroll
      for (int v = 0; v < 16; v++) red[wave - 1][v * 64 + lane] = acc[0][v];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < S - 1; w++) {
#pragma unroll
      for (int v = 0; v < 16; v++) acc[0][v] += red[w][v * 64 + lane];
    }
  }

  // fused batch norm + leaky ReLU: per-channel scale / shift of this lane's columns
  float ew[NB], eb[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) {
    const int c = (cb0 + b) * 32 + r;
    ew[b] = (ep.out2 && c < Cout) ? ep.w[c] : 0.0f;
    eb[b] = (ep.out2 && c < Cout) ? ep.b[c] : 0.0f;
  }
  // D layout of the 32x32 MFMA: lane holds column (lane & 31), rows 8*(v/4) + 4*(lane>>5) + (v&3)
#pragma unroll
  for (int v = 0; v < 16; v++) {
    const int i = 8 * (v >> 2) + 4 * h + (v & 3);
    const int rid = __shfl(my_row, i, 64);
    if (rid < 0) continue;
    if (out) {
      float *op = out + (int64_t)rid * ld_out + cb0 * 32 + r;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if ((cb0 + b) * 32 + r < Cout) op[b * 32] = acc[b][v];
    }
    if (ep.out2) {
      float *op2 = ep.out2 + (int64_t)rid * ep.ld2 + cb0 * 32 + r;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if ((cb0 + b) * 32 + r < Cout) {
          const float y = fmaf(acc[b][v], ew[b], eb[b]);
          op2[b * 32] = y * ((y > 0.0f) ? 1.0f : ep.leak);
        }
    }
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

// W: raw [K,Cin,Cout] weights (always needed by the generic kernel); Wp: packed weights or
// null, in which case they are packed into scratch memory first.
int launch_conv(const float *in, int64_t ld_in, int64_t in_rows, float *out, int64_t ld_out, const float *W,
                const float *Wp, const float *bias, const int32_t *map0, const int32_t *map1, int mode, int K,
                const int32_t *rows, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                const uint8_t *tile_flags, const uint8_t *row_mask, hipStream_t s, BnEpilogue ep) {
  if (n_rows == 0) return INSC_OK;
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
    const int nbt = (Cout + 31) / 32;
    // Launch shape, a function of the layer shape only (so results never depend on the scene):
    //  narrow layers (Cin < 96): each wavefront computes all output blocks of its tile (the
    //    gathered rows are reused across them);
    //  wide layers: one output block per wavefront (more wavefronts for the few tiles of a
    //    coarse scale), and for 3^3 / 2^3 maps the offsets of a tile are split over S wavefronts.
    const bool wide = Cin >= 96;
    const int NB = wide ? 1 : conv_nb_per_group(Cout);
    const int nbtp = conv_nbt_padded(Cout);
    int S = 1;
    if (wide && mode == MAP_NBR && K == 27) S = Cin >= 160 ? 8 : 4;
    if (wide && mode == MAP_NBR && K == 8) S = 4;
    const unsigned gx = (unsigned)(S == 1 ? cdiv(tiles, CONV_WAVES) : tiles);
    dim3 grid(gx, (unsigned)(NB == 1 ? nbt : nbtp / NB)), block((S == 1 ? CONV_WAVES : S) * 64);
    bool shape_ok = true;
#define INSC_CONV_LAUNCH(NBV, KV, MV, SV)                                                                       \
  hipLaunchKernelGGL((conv_mfma_kernel<NBV, KV, MV, SV>), grid, block, 0, s, in, ld_in, out, ld_out, Wp, bias,  \
                     map0, map1, rows, d_n_rows, n_rows, Cin, Cout, nbtp, tile_flags, in_bytes, wp_bytes, ep)
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
    if (S == 8) {
      INSC_CONV_LAUNCH(1, 27, MAP_NBR, 8);
    } else if (S == 4 && K == 27) {
      INSC_CONV_LAUNCH(1, 27, MAP_NBR, 4);
    } else if (S == 4) {
      INSC_CONV_LAUNCH(1, 8, MAP_NBR, 4);
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
    hipLaunchKernelGGL(conv_generic_kernel, dim3(grid_for(n_rows, cpb, 65536)), dim3(256), 0, s, in, ld_in, out,
                       ld_out, W, bias, map0, map1, mode, K, rows, d_n_rows, n_rows, Cin, Cout, row_mask, ep);
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
