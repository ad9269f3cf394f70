// Internal view of the hash grid, shared by grid.hip and the network executor.
#pragma once
#include "common.h"

namespace insc {

struct __attribute__((aligned(16))) Slot {
  unsigned long long key;
  int val;
  int pad;
};

constexpr int VAL_UNSET = 0x7FFFFFFF;
constexpr int VAL_PENDING = 0x40000000;  // VAL_PENDING + p : claimed during this insert by row p

}  // namespace insc

struct insc_grid {
  insc::Slot *table = nullptr;
  int64_t n_slots = 0;         // power of two
  int64_t capacity_sites = 0;  // rows of coords
  int32_t *coords = nullptr;   // [capacity_sites, 4]
  int32_t *d_n = nullptr;      // device site counter; d_n[1] = the count before the last insert
  int32_t *d_err = nullptr;    // device flag: bit0 bad coordinate, bit1 table full
  int64_t n_upper = 0;         // host upper bound of the site count
  int64_t n_exact = -1;        // host copy of the count, -1 = stale
  // pinned host words that the last kernel of insc_grid_insert writes: [0] site count, [1] error flags.
  // h_fresh: they describe the grid's current state, once h_stream has been waited for.
  int32_t *h_n = nullptr;
  bool h_fresh = false;
  void *h_stream = nullptr;
  // insert scratch, grown on demand
  int32_t *slot_of_point = nullptr;
  int32_t *flags = nullptr;
  int64_t scratch_rows = 0;
  int32_t *part = nullptr;  // partition counters and offsets of the large insert (PART_INTS words, zero between calls)
  int device = 0;
};

namespace insc {

// Point coordinate that the insert skips silently (site -1, no error): used to pad a fixed-size
// launch whose real length is only known on the device.
constexpr int32_t COORD_SKIP = INT32_MIN;

// Device-side variants used inside a frame: nothing here synchronises with the host.
// All of them act on the sites added by the grid's most recent insert, [*d_n_prev, *d_n).
int grid_insert_nosync(insc_grid *g, const int32_t *d_coords4, int64_t P, int32_t *d_site_of_point, hipStream_t s);
// the neighbour maps of the new sites of several grids (the scales of a network, at most 16) in one
// launch; every grid acts on the sites of its own most recent insert
// plans (nullable; per grid, plan null = none): tile plans to keep up to date with the map - the
// entries of older sites that gain a neighbour are patched and the offset masks of the tiles the new
// sites open are cleared; the new sites' own columns follow with tile_plan_append_batch
struct PlanRef {
  int32_t *plan;
  uint32_t *tmask;
  const int32_t *pos;
  int64_t ld;
};
int ssc3_new_sites_batch(const insc_grid *const *grids, int32_t *const *d_nbr, int n, int64_t n_new_upper,
                         hipStream_t s, const PlanRef *plans = nullptr, bool all_new = false);
// (all_new: the caller knows that grids without older sites - d_n[1] == 0 - are to get whole maps, as in a
// full frame: their rows are set to -1 first and every neighbour pair is looked up once)
// Processing orders of several scales built from scratch in shared launches (insc_order_build +
// insc_order_by_offset + their inverses, scale by scale, take three times as many): order / pos = the
// order of the 3^3 layers and its inverse over sites 0..n-1; with offset != null also bo_order / bo_pos,
// the same sites grouped by their position inside the parent cell.  n <= SORT_BATCH_MAX_N per scale.
struct OrderBuildJob {
  const insc_grid *g;
  const int32_t *nbr, *offset;
  int64_t n;
  int32_t *order, *pos, *bo_order, *bo_pos;
};
int order_build_batch(const OrderBuildJob *jobs, int n_jobs, hipStream_t s);
// Residual frames, all scales in two launches: d_pre_exist[l][i] = the saved site (grid pre[l]) at the
// coordinates of site i of grids[l], or -1; d_nbr_pre[l] = the 27 saved neighbours of the sites that
// have none (insc_grid_query + insc_incre_rulebook_ssc3); d_parent2[l][i], for l + 1 < n, = the saved
// site of the coarse parent (d_parent[l]) of a site that has none.  Sized by n_upper, an upper bound
// of every scale's site count; the counts themselves are read on the device.
int incre_links_batch(const insc_grid *const *grids, const insc_grid *const *pre, const int32_t *const *d_parent,
                      int32_t *const *d_pre_exist, int32_t *const *d_nbr_pre, int32_t *const *d_parent2, int n,
                      int64_t n_upper, hipStream_t s);
// The inserts of a whole frame at all scales at once: the points go into lv[0].grid, the sites that adds
// (halved) into lv[1].grid and so on, with the parent /
// offset / child link of every scale to the next coarser one filled in for the new sites.  Every
// grid then reports the sites of this insert as its newest ([d_n[1], d_n[0])).  d_coords: int32
// [P, cols] (cols 3 or 4).  If any coordinate is out of range nothing is inserted anywhere, *d_bad
// = frame, and every row of d_sop is -1.  h_counts (nullable, host memory the device can write):
// receives per scale the site count and error flags, then at [2 * n_levels] `frame` for a dropped frame else 0.
struct FrameInsertLevel {
  insc_grid *grid;
  int32_t *parent, *offset, *child;
};
int frame_insert_levels(const FrameInsertLevel *lv, int n_levels, const int32_t *d_coords, int cols, int64_t P,
                        int32_t *d_bad, int32_t frame, int32_t *d_sop, int32_t *h_counts, hipStream_t s);
// looks up, for the current device, the address of the scratch array of insc_grid_insert_noalloc
// (called by insc_init; the entry point does it itself on a device that was never initialised)
int grid_noalloc_setup();
// The new sites of several grids appended to their processing orders in ONE launch, sorted among
// themselves by the key of insc_order_build (needs their rows of the neighbour map), and to the orders
// grouped by their position inside the parent cell (d_offset[i] null: the grid has no coarser scale
// above it and only gets the first order)
int order_append_new_sites_both_batch(const insc_grid *const *grids, const int32_t *const *d_nbr,
                                      const int32_t *const *d_offset, int32_t *const *d_order, int32_t *const *d_pos,
                                      int32_t *const *d_bo_order, int32_t *const *d_bo_pos, int n, int64_t n_new_upper,
                                      hipStream_t s, bool all = false);  // all: every site of each grid, from position 0
// insc_grid_clear for several grids in one launch; with grid i the int32 array minus1[i] (n_minus1[i]
// words, nullable) is set to -1, and `zero` (nullable, zero_bytes a multiple of 4) is zeroed
int grid_clear_batch(insc_grid *const *grids, int32_t *const *minus1, const int64_t *n_minus1, int n, void *zero,
                     int64_t zero_bytes, hipStream_t s);
// most sites the two sorted appends put in order (more keep their arrival order)
int64_t order_sorted_max();
// Sort key of a site in the processing orders, from its coordinates and the 27-bit pattern m of the
// neighbours it has (see insc_order_build): batch parity, Morton code of the 64^3 block (4 bits per axis:
// blocks 1024 voxels apart share a group, harmless), pattern.
constexpr int ORDER_KEY_BITS = 40;
__device__ __forceinline__ uint64_t order_spread3(uint64_t v) {  // 4 bits -> every third bit
  v &= 0xf;
  v = (v | (v << 4)) & 0xc3ull;
  v = (v | (v << 2)) & 0x249ull;
  return v;
}
__device__ __forceinline__ uint64_t order_key(int4 c, uint32_t m) {
  const uint64_t mort = order_spread3((uint64_t)(c.x >> 6)) | (order_spread3((uint64_t)(c.y >> 6)) << 1) |
                        (order_spread3((uint64_t)(c.z >> 6)) << 2);
  return ((uint64_t)(c.w & 1) << 39) | (mort << 27) | (uint64_t)m;
}
// device pointer to the site count before the most recent insert
static inline const int32_t *grid_n_prev_ptr(const insc_grid *g) { return g->d_n + 1; }

}  // namespace insc
