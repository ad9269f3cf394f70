// Hash grid: open addressing on 64-bit packed voxel keys, 16-byte slots.
//
// Home slot: the eight voxels (x, y, z0..z0+7) of one z-run share one aligned group of eight
// slots (128 bytes, one L2 line), voxel z at position z&7.  The three z-neighbours of a
// 3x3x3 query therefore read the same line, and the lanes of a wavefront that handle
// consecutive filter offsets probe it together.
//
// Probe order: a key stays inside the aligned run of PART_SLOTS slots that holds its home slot (the whole
// table if it is smaller) - its partition - which lets a large insert build the table partition by
// partition in LDS (part_* kernels below).  From a taken slot it moves on by an odd number of groups (taken
// from hash bits the home slot does not use) and one position inside the group; once it has seen as many
// slots as the partition has groups it walks the partition slot by slot from the home slot, so that every
// slot is reached (never seen in practice: at load <= 0.5 that takes a hundred-odd taken slots in a row).
// Moving on to the neighbouring slot instead - plain linear probing - does badly with these homes: the
// groups of a scene fill up whole, so a key whose home group is shared sits eight or more slots away
// (200 000 voxels of a room in 2^20 slots: 4 % of the keys at 8 or more probes, 1 % at 16 or more, which
// is what nearly every wavefront then waits for; this way 9 % of the keys take a second probe and the
// longest walk is 8).
//
// Numbering: a site's id is its rank among first occurrences in the inserted list, offset by
// the count before the call - deterministic and append-only.
#include <mutex>

#include "common.h"
#include "grid.h"

namespace insc {

__device__ __forceinline__ uint64_t mix64(uint64_t h) {
  h ^= h >> 33;
  h *= 0xff51afd7ed558ccdull;
  h ^= h >> 33;
  h *= 0xc4ceb9fe1a85ec53ull;
  h ^= h >> 33;
  return h;
}

constexpr int PART_SHIFT = 11;
constexpr int64_t PART_SLOTS = 1ll << PART_SHIFT;

struct Walk {
  int64_t part;            // first slot of the key's partition
  int wm;                  // slots of a partition - 1
  int home, loc, step, i;  // slots inside the partition: home, current; groups to move on by; probes so far
};
__device__ __forceinline__ Walk walk_begin(uint64_t key, int64_t mask) {
  // z's low three bits stay out of the hashed part and come back as the position in the group
  const uint64_t zlow = (key >> 32) & 7ull;
  const uint64_t h = mix64(key & ~(7ull << 32));
  const int64_t home = (int64_t)(((h << 3) | zlow) & (uint64_t)mask);
  Walk w;
  w.wm = (int)(mask < PART_SLOTS - 1 ? mask : PART_SLOTS - 1);
  w.part = home & ~(int64_t)w.wm;
  w.home = w.loc = (int)(home & w.wm);
  w.step = (int)(h >> 44) | 1;
  w.i = 0;
  return w;
}
__device__ __forceinline__ int64_t walk_slot(const Walk &w) { return w.part + w.loc; }
// the next slot to look at; false: the whole partition has been seen
__device__ __forceinline__ bool walk_next(Walk &w) {
  const int groups = (w.wm + 1) >> 3;
  w.i++;
  if (w.i < groups) {
    w.loc = ((((w.loc >> 3) + w.step) & (groups - 1)) << 3) | ((w.loc + 1) & 7);
    return true;
  }
  if (w.i > groups + w.wm) return false;
  w.loc = (w.home + (w.i - groups)) & w.wm;
  return true;
}

__device__ __forceinline__ int grid_find(const Slot *__restrict__ table, int64_t mask, uint64_t key) {
  Walk w = walk_begin(key, mask);
  do {
    const int64_t s = walk_slot(w);
    unsigned long long k = table[s].key;
    if (k == key) return table[s].val;
    if (k == INSC_EMPTY_KEY) return -1;
  } while (walk_next(w));
  return -1;
}

__global__ void grid_clear_kernel(Slot *table, int64_t n_slots, int32_t *d_n, int32_t *d_err) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n_slots; i += stride) {
    Slot e;
    e.key = INSC_EMPTY_KEY;
    e.val = VAL_UNSET;
    e.pad = 0;
    table[i] = e;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    d_n[0] = 0;
    d_n[1] = 0;
    *d_err = 0;
  }
}

// ---- numbering the new cells of an insert ----------------------------------------------------
// A site's id is the rank of its first row in the inserted list, so every new cell needs the smallest
// row that falls into it.  Protocol on a slot (key, val, pad), one claim kernel, then whatever ranks:
//   * the row whose compare-and-swap sets the key - the slot's first claimant - leaves row + 1 in
//     `pad` (a plain store: it is read by later kernels only) and is the cell's winner for now;
//   * every other row of the call that finds the key there lowers `val` to VAL_PENDING + row with an
//     atomic minimum (skipped when the value it read is already a smaller row's claim);
//   * afterwards the cell's first row is min(pad - 1, val - VAL_PENDING), which only the rows of the
//     second kind look at: a point list without repeats costs one atomic per new site and no second
//     visit of its slot (one compare-and-swap plus one minimum per point, and a visit of the slot by
//     every row to see who won, measured 55 + 8 us for 220 000 points).
// A slot that holds an id (0 <= val < VAL_PENDING) was numbered by an earlier insert.
// State of a row after the claim kernel, in site_of_point: its own row index (first claimant), ST_DUP
// (other claimant, to be resolved), -2 - id (cell numbered earlier), -1 (skipped / bad / table full).
constexpr int32_t ST_DUP = INT32_MIN + 1;

__global__ void grid_claim_kernel(Slot *table, int64_t mask, const int32_t *__restrict__ coords4, int64_t P,
                                  int32_t *__restrict__ slot_of_point, int32_t *__restrict__ flags,
                                  int32_t *__restrict__ site_of_point, int32_t *d_err) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  int4 c = reinterpret_cast<const int4 *>(coords4)[p];
  int32_t slot = -1, state = -1, flag = 0;
  if (c.x != COORD_SKIP) {
    if (!coord_ok(c.x, c.y, c.z, c.w)) {
      atomicOr(d_err, 1);
    } else {
      const uint64_t key = pack_key(c.x, c.y, c.z, c.w);
      Walk w = walk_begin(key, mask);
      bool full = true;
      do {
        const int64_t s = walk_slot(w);
        const int4 raw = *reinterpret_cast<const int4 *>(&table[s]);  // key (two words), val, pad
        unsigned long long k = ((unsigned long long)(unsigned)raw.y << 32) | (unsigned)raw.x;
        const bool seen = k == key;
        if (seen && raw.z >= 0 && raw.z < VAL_PENDING) {  // numbered by an earlier insert
          slot = (int32_t)s;
          state = -2 - raw.z;
          full = false;
          break;
        }
        bool first = false;
        if (k == INSC_EMPTY_KEY) {
          k = atomicCAS(&table[s].key, INSC_EMPTY_KEY, (unsigned long long)key);
          first = k == INSC_EMPTY_KEY;
        }
        if (first) {
          // (written through, so that later claimants on other XCDs may see it and spare their atomic)
          __hip_atomic_store(&table[s].pad, (int)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          slot = (int32_t)s;
          state = (int32_t)p;
          flag = 1;
          full = false;
          break;
        }
        if (k == key) {
          // no atomic for a row that has seen a smaller row in the slot - as the first claimant (pad) or
          // as a later one (val): it cannot be the cell's first row.  (The values only ever go down during
          // a call, so a stale read errs on the side of one more atomic.)
          const bool beaten = seen && ((raw.w > 0 && raw.w - 1 < (int)p) || (raw.z >= VAL_PENDING && raw.z <= VAL_PENDING + (int)p));
          if (!beaten) atomicMin(&table[s].val, VAL_PENDING + (int)p);
          slot = (int32_t)s;
          state = ST_DUP;
          full = false;
          break;
        }
      } while (walk_next(w));
      if (full) atomicOr(d_err, 2);
    }
  }
  slot_of_point[p] = slot;
  site_of_point[p] = state;
  if (flags) flags[p] = flag;
}

// pass 2 of a large insert, for the rows that found their key claimed by another row of the call: who
// numbers the cell.  If it is this row (the smallest of the later claimants, and smaller than the
// first claimant) it takes the first claimant's place.  Row 0 also saves the site count from before
// the insert beside the scan's total, so that pass 3 can replace the counters while its other threads
// still read it.
__global__ void grid_resolve_kernel(const Slot *__restrict__ table, const int32_t *__restrict__ slot_of_point, int64_t P,
                                    int32_t *__restrict__ flags, int32_t *__restrict__ site_of_point,
                                    const int32_t *__restrict__ d_n, int32_t *__restrict__ n_before) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  if (p == 0) *n_before = d_n[0];
  if (site_of_point[p] != ST_DUP) return;
  const int4 raw = *reinterpret_cast<const int4 *>(&table[slot_of_point[p]]);
  if (raw.z >= 0 && raw.z < VAL_PENDING) {  // (the key was there all along; the row had read a stale empty slot)
    site_of_point[p] = -2 - raw.z;
    return;
  }
  const int first = raw.w - 1, later = raw.z - VAL_PENDING;  // (later: huge when no row lowered the value)
  if (later == (int)p && (int)p < first) {
    flags[p] = 1;
    site_of_point[p] = (int32_t)p;
    flags[first] = 0;
    site_of_point[first] = (int32_t)p;
  } else {
    site_of_point[p] = first < later ? first : later;
  }
}

// pass 3: winners take id = n_before + rank, publish it in the slot and record the coordinates; every
// row learns its site from its winner's rank; row 0 moves the counters on
__global__ void grid_assign_kernel(Slot *table, const int32_t *__restrict__ coords4,
                                   const int32_t *__restrict__ slot_of_point, const int32_t *__restrict__ excl,
                                   int64_t P, int32_t *__restrict__ d_n, const int32_t *__restrict__ total,
                                   int32_t *__restrict__ site_coords, int64_t capacity_sites, int32_t *d_err,
                                   int32_t *__restrict__ site_of_point, int32_t *__restrict__ h_n) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int n_before = total[1];
  if (p == 0) {
    // (more new sites than there is room for: the rows beyond get no site below and raise the flag, but
    // perhaps only after this thread has read it - so it is worked out here as well)
    const bool over = (int64_t)n_before + total[0] > capacity_sites;
    const int n_new = over ? (int)(capacity_sites - n_before) : total[0];
    d_n[1] = n_before;
    d_n[0] = n_before + n_new;
    if (h_n) {  // the host's copy of the count and of the error flags (pinned memory)
      h_n[0] = n_before + n_new;
      h_n[1] = __hip_atomic_load(d_err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) | (over ? 2 : 0);
    }
  }
  int r = site_of_point[p];
  if (r < 0) {
    if (r < -1) site_of_point[p] = -2 - r;
    return;
  }
  int id = n_before + excl[r];
  if (id >= capacity_sites) {
    site_of_point[p] = -1;
    if (r == p) atomicOr(d_err, 2);
    return;
  }
  site_of_point[p] = id;
  if (r == p) {
    table[slot_of_point[p]].val = id;
    reinterpret_cast<int4 *>(site_coords)[id] = reinterpret_cast<const int4 *>(coords4)[p];
  }
}

// Passes 2-3 and the counter update in one workgroup, for inserts of up to FINISH_SMALL_MAX rows
// (an incremental frame): thread t owns a contiguous run of rows, so the ids come out in row
// order exactly as from the scan-based passes.  site_of_point holds the rows' states on entry and
// their sites on exit.
constexpr int FINISH_SMALL_MAX = 16384;
__global__ __launch_bounds__(1024) void grid_finish_small_kernel(Slot *table, const int32_t *__restrict__ coords4,
                                                                 const int32_t *__restrict__ slot_of_point, int P,
                                                                 int32_t *d_n, int32_t *__restrict__ site_coords,
                                                                 int64_t capacity_sites, int32_t *d_err,
                                                                 int32_t *site_of_point, int32_t *__restrict__ h_n) {
  __shared__ int wave_total[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = (P + 1023) / 1024, p0 = tid * per;
  const int n_before = d_n[0];
  // later claimants find out who numbers their cell (grid_resolve_kernel)
  for (int j = 0; j < per; j++) {
    const int p = p0 + j;
    if (p >= P || site_of_point[p] != ST_DUP) continue;
    const int4 raw = *reinterpret_cast<const int4 *>(&table[slot_of_point[p]]);
    if (raw.z >= 0 && raw.z < VAL_PENDING) {
      site_of_point[p] = -2 - raw.z;
      continue;
    }
    const int first = raw.w - 1, later = raw.z - VAL_PENDING;
    if (later == p && p < first) {
      site_of_point[p] = p;
      site_of_point[first] = p;
    } else {
      site_of_point[p] = first < later ? first : later;
    }
  }
  __threadfence_block();
  __syncthreads();
  int st[16];
  unsigned win = 0;
  int cnt = 0;
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int p = p0 + j;
    st[j] = (j < per && p < P) ? site_of_point[p] : -1;
    if (j < per && p < P && st[j] == p) {
      win |= 1u << j;
      cnt++;
    }
  }
  // exclusive scan of cnt over the workgroup
  int incl = cnt;
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_up(incl, d, 64);
    if (lane >= d) incl += v;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  int base = n_before + incl - cnt, total = 0;
  for (int w = 0; w < 16; w++) {
    if (w < wave) base += wave_total[w];
    total += wave_total[w];
  }
#pragma unroll
  for (int j = 0; j < 16; j++) {
    if (!((win >> j) & 1u)) continue;
    const int p = p0 + j, id = base++;
    if (id >= capacity_sites) {
      atomicOr(d_err, 2);
      site_of_point[p] = -1;
      continue;
    }
    table[slot_of_point[p]].val = id;
    reinterpret_cast<int4 *>(site_coords)[id] = reinterpret_cast<const int4 *>(coords4)[p];
    site_of_point[p] = id;
  }
  __threadfence_block();
  __syncthreads();
  // every other row takes its site from the row that numbered its cell
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int p = p0 + j;
    if (j >= per || p >= P || ((win >> j) & 1u)) continue;
    if (st[j] < -1)
      site_of_point[p] = -2 - st[j];
    else if (st[j] >= 0)
      site_of_point[p] = site_of_point[st[j]];
  }
  const bool over = total > capacity_sites - n_before;
  if (over) total = (int)(capacity_sites - n_before);
  if (tid == 0) {
    d_n[1] = n_before;
    d_n[0] = n_before + total;
    if (h_n) {  // the host's copy of the count and of the error flags (pinned memory)
      h_n[0] = n_before + total;
      h_n[1] = __hip_atomic_load(d_err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) | (over ? 2 : 0);
    }
  }
}

// ---- large inserts into an empty grid: the table built partition by partition in LDS ---------
// The claim kernel above sends one atomic per point to a slot somewhere in the table, and the lines of
// the table travel between the L2s of the chip's dies for it.  A large insert into an empty grid sorts
// its rows by home partition first (count, scatter: coalesced passes with LDS histograms) and then one
// workgroup per partition plays the same protocol on its PART_SLOTS slots in LDS: winners (the smallest
// row of every new cell), the prefix sum over the rows' winner flags that ranks them, and one pass that
// stores the numbered slots - the only time the table itself is touched.  Measured on 220 000 points
// into 2^20 slots: 54 MB of memory traffic and 41 us, against 74 MB and 44 us for the claim kernel's way.
// A grid that holds sites takes the claim kernel: its partitions would have to be read from the table
// first (measured with 80 000 rows onto 150 000 sites: 31 against 25 us).
constexpr int PART_MAX = 4096;   // partitions of the largest table that takes this path
constexpr int PART_PAD = 16;     // ints between two partitions' counters (their atomics spread over the L2 channels)
constexpr int PART_ROWS = 2;     // rows per thread of count / scatter
constexpr int PART_INTS = 2 * PART_MAX * PART_PAD + PART_MAX + 64;  // cnt | cursor | base

__device__ __forceinline__ int part_of_row(const int32_t *__restrict__ coords4, int64_t p, int64_t mask, int32_t *d_err,
                                           bool report, uint64_t *key_out = nullptr) {
  const int4 c = reinterpret_cast<const int4 *>(coords4)[p];
  if (c.x == COORD_SKIP) return -1;
  if (!coord_ok(c.x, c.y, c.z, c.w)) {
    if (report) atomicOr(d_err, 1);
    return -1;
  }
  const uint64_t key = pack_key(c.x, c.y, c.z, c.w);
  if (key_out) *key_out = key;
  return (int)(walk_begin(key, mask).part >> PART_SHIFT);
}
__device__ __forceinline__ int4 unpack_key(uint64_t key) {
  return make_int4((int)(key & 0xFFFF), (int)((key >> 16) & 0xFFFF), (int)((key >> 32) & 0xFFFF), (int)(key >> 48));
}

// rows per partition
__global__ __launch_bounds__(1024) void part_count_kernel(const int32_t *__restrict__ coords4, int64_t P, int64_t mask,
                                                          int n_parts, int32_t *cnt, int32_t *d_err) {
  extern __shared__ int32_t hist[];
  const int tid = threadIdx.x;
  for (int i = tid; i < n_parts; i += 1024) hist[i] = 0;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < PART_ROWS; j++) {
    const int64_t p = ((int64_t)blockIdx.x * PART_ROWS + j) * 1024 + tid;
    if (p >= P) break;
    const int q = part_of_row(coords4, p, mask, d_err, true);
    if (q >= 0) atomicAdd(&hist[q], 1);
  }
  __syncthreads();
  for (int i = tid; i < n_parts; i += 1024)
    if (hist[i]) atomicAdd(&cnt[i * PART_PAD], hist[i]);
}

// rows and their keys sorted by partition (any order inside one), so that the kernels that follow read them
// in order instead of gathering coordinates (with all workgroups gathering at once, the slowest took 13 us
// over it); the rows that go nowhere get their answer here.  Every
// workgroup turns the counts into offsets for itself (a prefix sum over at most PART_MAX values; a
// single workgroup doing it for all would have to publish them through a fence that writes the L2 back,
// measured 15 us), the first one stores them for the kernels that follow.
__global__ __launch_bounds__(1024) void part_scatter_kernel(const int32_t *__restrict__ coords4, int64_t P, int64_t mask,
                                                            int n_parts, const int32_t *__restrict__ cnt, int32_t *cursor,
                                                            int32_t *__restrict__ base, int32_t *__restrict__ part_rows,
                                                            uint64_t *__restrict__ part_keys,
                                                            int32_t *__restrict__ site_of_point, int32_t *__restrict__ flags) {
  extern __shared__ int32_t lds[];
  int32_t *hist = lds, *off = lds + n_parts;
  __shared__ int wave_total[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < n_parts; i += 1024) hist[i] = 0;
  // exclusive prefix sum of the counts: thread t takes partitions 4t .. 4t+3
  int v[4], sum = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int i = tid * 4 + j;
    v[j] = i < n_parts ? cnt[i * PART_PAD] : 0;
    sum += v[j];
  }
  int incl = sum;
  for (int d = 1; d < 64; d <<= 1) {
    const int u = __shfl_up(incl, d, 64);
    if (lane >= d) incl += u;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  int run = incl - sum;
  for (int w = 0; w < wave; w++) run += wave_total[w];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int i = tid * 4 + j;
    if (i < n_parts) {
      off[i] = run;
      if (blockIdx.x == 0) base[i] = run;
      run += v[j];
    }
  }
  if (blockIdx.x == 0 && tid == 1023) base[n_parts] = run;  // (the last thread's total: all rows that go somewhere)
  int q[PART_ROWS], r[PART_ROWS];
  uint64_t key[PART_ROWS];
#pragma unroll
  for (int j = 0; j < PART_ROWS; j++) {
    const int64_t p = ((int64_t)blockIdx.x * PART_ROWS + j) * 1024 + tid;
    q[j] = -2;
    if (p >= P) continue;
    q[j] = part_of_row(coords4, p, mask, nullptr, false, &key[j]);
    if (q[j] >= 0) {
      r[j] = atomicAdd(&hist[q[j]], 1);
    } else {
      site_of_point[p] = -1;
      flags[p] = 0;
    }
  }
  __syncthreads();
  for (int i = tid; i < n_parts; i += 1024)
    if (hist[i]) off[i] += atomicAdd(&cursor[i * PART_PAD], hist[i]);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < PART_ROWS; j++) {
    const int64_t p = ((int64_t)blockIdx.x * PART_ROWS + j) * 1024 + tid;
    if (q[j] >= 0) {
      const int at = off[q[j]] + r[j];
      part_rows[at] = (int32_t)p;
      part_keys[at] = key[j];
    }
  }
}

// slot of `key` in the LDS copy of its partition, claiming the first empty slot of its walk; -1: full
__device__ __forceinline__ int part_slot(unsigned long long *keys, unsigned long long key, int64_t mask) {
  Walk w = walk_begin(key, mask);
  do {
    unsigned long long k = keys[w.loc];
    if (k == INSC_EMPTY_KEY) {
      k = atomicCAS(&keys[w.loc], INSC_EMPTY_KEY, key);
      if (k == INSC_EMPTY_KEY) return w.loc;
    }
    if (k == key) return w.loc;
  } while (walk_next(w));
  return -1;
}

// One workgroup per partition plays the insert on the partition's slots in LDS, all empty at the start.
// Per row, in partition order: state = the smallest row of the row's cell (flags 1 for that row itself),
// -1 if the partition is full; where = the cell's slot in the table.  Leaves the partition's counters zero.
constexpr int PART_THREADS = 512;
constexpr int PART_KEEP = 2;  // rows per thread kept in registers between the two passes (more are looked up again)
__global__ __launch_bounds__(PART_THREADS) void part_winners_kernel(
    int64_t mask, const int32_t *__restrict__ base,
    const int32_t *__restrict__ part_rows, const uint64_t *__restrict__ part_keys, const int32_t *__restrict__ d_n,
    int32_t *__restrict__ flags, int32_t *__restrict__ state, int32_t *__restrict__ where, int32_t *cnt, int32_t *cursor,
    int32_t *__restrict__ n_before, int32_t *d_err) {
  __shared__ unsigned long long keys[PART_SLOTS];
  __shared__ int vals[PART_SLOTS];
  const int q = blockIdx.x, tid = threadIdx.x;
  const int W = (int)(mask < PART_SLOTS - 1 ? mask + 1 : PART_SLOTS);
  const int b0 = base[q], b1 = base[q + 1];
  if (tid == 0) {
    if (q == 0) *n_before = d_n[0];
    cnt[q * PART_PAD] = 0;
    cursor[q * PART_PAD] = 0;
  }
  int pr[PART_KEEP], sr[PART_KEEP];
  uint64_t kr[PART_KEEP];
#pragma unroll
  for (int j = 0; j < PART_KEEP; j++) {
    const int i = b0 + j * PART_THREADS + tid;
    pr[j] = i < b1 ? part_rows[i] : -1;
    kr[j] = i < b1 ? part_keys[i] : 0;
  }
  for (int i = tid; i < W; i += PART_THREADS) {
    keys[i] = INSC_EMPTY_KEY;
    vals[i] = VAL_UNSET;
  }
  __syncthreads();
  auto claim = [&](int p, const uint64_t key) -> int {
    const int s = part_slot(keys, key, mask);
    if (s < 0)
      atomicOr(d_err, 2);
    else
      atomicMin(&vals[s], VAL_PENDING + p);
    return s;
  };
  auto answer = [&](int i, int p, int s) {
    const int st = s >= 0 ? vals[s] - VAL_PENDING : -1;
    state[i] = st;
    where[i] = s < 0 ? -1 : (int)((int64_t)q * W + s);
    flags[p] = st == p ? 1 : 0;
  };
#pragma unroll
  for (int j = 0; j < PART_KEEP; j++)
    if (pr[j] >= 0) sr[j] = claim(pr[j], kr[j]);
  for (int i = b0 + PART_KEEP * PART_THREADS + tid; i < b1; i += PART_THREADS) claim(part_rows[i], part_keys[i]);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < PART_KEEP; j++)
    if (pr[j] >= 0) answer(b0 + j * PART_THREADS + tid, pr[j], sr[j]);
  for (int i = b0 + PART_KEEP * PART_THREADS + tid; i < b1; i += PART_THREADS) {
    const uint64_t key = part_keys[i];
    answer(i, part_rows[i], part_slot(keys, key, mask));  // (finds what the first pass left)
  }
}

// numbered: every row takes id = n_before + rank of its cell's winner; the winners store their slots
// (16 bytes each, the only writes to the table) and their coordinates; the first thread moves the
// counters on (as grid_assign_kernel).  One thread per row, in partition order.
__global__ __launch_bounds__(256) void part_assign_kernel(Slot *table, const int32_t *__restrict__ base, int n_parts,
                                                          const int32_t *__restrict__ part_rows,
                                                          const uint64_t *__restrict__ part_keys,
                                                          const int32_t *__restrict__ state,
                                                          const int32_t *__restrict__ where,
                                                          const int32_t *__restrict__ excl, int32_t *__restrict__ d_n,
                                                          const int32_t *__restrict__ total,
                                                          int32_t *__restrict__ site_coords, int64_t capacity_sites,
                                                          int32_t *d_err, int32_t *__restrict__ site_of_point,
                                                          int32_t *__restrict__ h_n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int n_before = total[1];
  if (i == 0) {
    const bool over = (int64_t)n_before + total[0] > capacity_sites;
    const int n_new = over ? (int)(capacity_sites - n_before) : total[0];
    d_n[1] = n_before;
    d_n[0] = n_before + n_new;
    if (h_n) {
      h_n[0] = n_before + n_new;
      h_n[1] = __hip_atomic_load(d_err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) | (over ? 2 : 0);
    }
  }
  if (i >= base[n_parts]) return;
  const int p = part_rows[i], r = state[i];
  if (r < 0) {
    site_of_point[p] = -1;  // (the partition was full)
    return;
  }
  const int id = n_before + excl[r];
  if (id >= capacity_sites) {
    site_of_point[p] = -1;
    if (r == p) atomicOr(d_err, 2);
    return;
  }
  site_of_point[p] = id;
  if (r != p) return;
  const uint64_t key = part_keys[i];
  *reinterpret_cast<int4 *>(&table[where[i]]) = make_int4((int)(uint32_t)key, (int)(uint32_t)(key >> 32), id, 0);
  reinterpret_cast<int4 *>(site_coords)[id] = unpack_key(key);
}

// Point query, one thread per query.  (Eight lanes per query reading a whole group of the table at once paid
// while keys sat up to dozens of slots from home in the same and the following lines; with walks of one
// or two probes, each in a line of its own, there is nothing to share.)
__global__ __launch_bounds__(256) void grid_query_kernel(const Slot *__restrict__ table, int64_t mask,
                                                         const int32_t *__restrict__ coords4, int64_t Q,
                                                         int32_t *__restrict__ out) {
  const int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= Q) return;
  const int4 c = reinterpret_cast<const int4 *>(coords4)[q];
  out[q] = coord_ok(c.x, c.y, c.z, c.w) ? grid_find(table, mask, pack_key(c.x, c.y, c.z, c.w)) : -1;
}

// re-insert site i with value i (used after a resize; keys are unique so no min is needed)
__global__ void grid_rehash_kernel(Slot *table, int64_t mask, const int32_t *__restrict__ site_coords,
                                   const int32_t *__restrict__ d_n, int32_t *d_err) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= *d_n) return;
  int4 c = reinterpret_cast<const int4 *>(site_coords)[i];
  uint64_t key = pack_key(c.x, c.y, c.z, c.w);
  Walk w = walk_begin(key, mask);
  do {
    const int64_t s = walk_slot(w);
    unsigned long long k = atomicCAS(&table[s].key, INSC_EMPTY_KEY, (unsigned long long)key);
    if (k == INSC_EMPTY_KEY) {
      table[s].val = (int)i;
      return;
    }
  } while (walk_next(w));
  atomicOr(d_err, 2);
}

// 27-neighbour map, one thread per (site, offset); see insc_rulebook_ssc3
__global__ void ssc3_nbr_kernel(const Slot *__restrict__ table, int64_t mask, const int32_t *__restrict__ site_coords,
                                int64_t first, int64_t n, int32_t *__restrict__ nbr, int patch_reverse) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * 27) return;
  int64_t o = first + t / 27;
  int k = (int)(t % 27);
  int4 c = reinterpret_cast<const int4 *>(site_coords)[o];
  int x = c.x + k / 9 - 1, y = c.y + (k / 3) % 3 - 1, z = c.z + k % 3 - 1;
  int r = -1;
  if (k == 13)
    r = (int)o;
  else if (coord_ok(x, y, z, c.w))
    r = grid_find(table, mask, pack_key(x, y, z, c.w));
  nbr[o * 27 + k] = r;
  if (patch_reverse && r >= 0 && r < first) nbr[(int64_t)r * 27 + (26 - k)] = (int)o;
}

// The same map when every site of the grid gets its row in this call (n = all sites, rows pre-filled
// with -1): a site being neighbour k of another makes that one neighbour 26 - k of the first, so a
// thread per (site, offset < 13) looks the neighbour up and writes both entries - half the probes.
__device__ __forceinline__ void ssc3_nbr_sym_body(const Slot *__restrict__ table, int64_t mask,
                                                  const int32_t *__restrict__ site_coords, int64_t n,
                                                  int32_t *__restrict__ nbr, int64_t t) {
  if (t >= n * 14) return;
  const int64_t o = t / 14;
  const int k = (int)(t % 14);
  if (k == 13) {
    nbr[o * 27 + 13] = (int)o;
    return;
  }
  const int4 c = reinterpret_cast<const int4 *>(site_coords)[o];
  const int x = c.x + k / 9 - 1, y = c.y + (k / 3) % 3 - 1, z = c.z + k % 3 - 1;
  if (!coord_ok(x, y, z, c.w)) return;
  const int r = grid_find(table, mask, pack_key(x, y, z, c.w));
  if (r < 0 || r >= n) return;
  nbr[o * 27 + k] = r;
  nbr[(int64_t)r * 27 + (26 - k)] = (int)o;
}
__global__ void ssc3_nbr_sym_kernel(const Slot *__restrict__ table, int64_t mask, const int32_t *__restrict__ site_coords,
                                    int64_t n, int32_t *__restrict__ nbr) {
  ssc3_nbr_sym_body(table, mask, site_coords, n, nbr, (int64_t)blockIdx.x * blockDim.x + threadIdx.x);
}

// Neighbours, in another (saved) grid, of the sites that the saved grid does not hold; see
// insc_incre_rulebook_ssc3
__global__ void incre_ssc3_nbr_kernel(const Slot *__restrict__ pre_table, int64_t pre_mask,
                                      const int32_t *__restrict__ site_coords,
                                      const int32_t *__restrict__ pre_exist, int64_t n, int32_t *__restrict__ nbr) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * 27) return;
  int64_t o = t / 27;
  int k = (int)(t % 27);
  int r = -1;
  if (pre_exist[o] < 0 && k != 13) {
    int4 c = reinterpret_cast<const int4 *>(site_coords)[o];
    int x = c.x + k / 9 - 1, y = c.y + (k / 3) % 3 - 1, z = c.z + k % 3 - 1;
    if (coord_ok(x, y, z, c.w)) r = grid_find(pre_table, pre_mask, pack_key(x, y, z, c.w));
  }
  nbr[t] = r;
}

__global__ void down2_coords_kernel(const int32_t *__restrict__ fine_coords, int64_t first, int64_t n,
                                    int32_t *__restrict__ half, int32_t *__restrict__ offset) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  int4 c = reinterpret_cast<const int4 *>(fine_coords)[first + t];
  offset[first + t] = (c.x & 1) * 4 + (c.y & 1) * 2 + (c.z & 1);
  reinterpret_cast<int4 *>(half)[t] = make_int4(c.x >> 1, c.y >> 1, c.z >> 1, c.w);
}

__global__ void down2_child_kernel(const int32_t *__restrict__ parent, const int32_t *__restrict__ offset,
                                   int64_t first, int64_t n, int32_t *__restrict__ child) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  int64_t i = first + t;
  int p = parent[i];
  if (p >= 0) child[(int64_t)p * 8 + offset[i]] = (int)i;
}

// ---- variants over the sites added by the last insert, [d_n[1], d_n[0]) --------------------
// With a tile plan (plan, tmask, pos, ld: the map transposed into processing order, see
// build_tile_plan) the plan is kept up to date as well: the entry of every older site that gains a
// neighbour is patched, and the offset masks of the tiles the new sites will open are cleared (their
// columns follow once the new sites have their positions, tile_plan_append).
__device__ __forceinline__ void ssc3_nbr_new_body(const Slot *__restrict__ table, int64_t mask,
                                                  const int32_t *__restrict__ site_coords,
                                                  const int32_t *__restrict__ d_n, int32_t *__restrict__ nbr,
                                                  int32_t *__restrict__ plan = nullptr,
                                                  uint32_t *__restrict__ tmask = nullptr,
                                                  const int32_t *__restrict__ pos = nullptr, int64_t ld = 0,
                                                  int symmetric = 0) {
  const int64_t first = d_n[1], n = (int64_t)d_n[0] - first;
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (symmetric && first == 0 && !plan) {  // every site is new and the rows hold -1: half the probes
    ssc3_nbr_sym_body(table, mask, site_coords, n, nbr, t);
    return;
  }
  if (plan) {
    const int64_t tile = (first + 31) / 32 + t;
    if (tile < (first + n + 31) / 32) tmask[tile] = 0;
  }
  if (t >= n * 27) return;
  int64_t o = first + t / 27;
  int k = (int)(t % 27);
  int4 c = reinterpret_cast<const int4 *>(site_coords)[o];
  int x = c.x + k / 9 - 1, y = c.y + (k / 3) % 3 - 1, z = c.z + k % 3 - 1;
  int r = -1;
  if (k == 13)
    r = (int)o;
  else if (coord_ok(x, y, z, c.w))
    r = grid_find(table, mask, pack_key(x, y, z, c.w));
  nbr[o * 27 + k] = r;
  if (r >= 0 && r < first) {
    nbr[(int64_t)r * 27 + (26 - k)] = (int)o;
    if (plan) {
      const int pr = pos[r];
      plan[(int64_t)(26 - k) * ld + pr] = (int)o;
      atomicOr(&tmask[pr >> 5], 1u << (26 - k));
    }
  }
}
// for several grids (the scales of a network) in one launch: blockIdx.y picks the grid
struct NewSitesJob {
  const Slot *table;
  int64_t mask;
  const int32_t *coords, *d_n;
  int32_t *nbr;
  int32_t *plan;  // optional tile plan to keep up to date
  uint32_t *tmask;
  const int32_t *pos;
  int64_t ld;
};
struct NewSitesBatch {
  NewSitesJob job[16];
  int symmetric;  // grids whose sites are all new have their rows at -1 (ssc3_nbr_fill_batch_kernel)
};
__global__ void ssc3_nbr_new_batch_kernel(NewSitesBatch b) {
  const NewSitesJob &j = b.job[blockIdx.y];
  ssc3_nbr_new_body(j.table, j.mask, j.coords, j.d_n, j.nbr, j.plan, j.tmask, j.pos, j.ld, b.symmetric);
}
// rows of the grids whose sites are all new set to -1, ahead of the symmetric form of the kernel above
__global__ void ssc3_nbr_fill_batch_kernel(NewSitesBatch b) {
  const NewSitesJob &j = b.job[blockIdx.y];
  if (j.d_n[1] != 0 || j.plan) return;
  const int64_t words = (int64_t)j.d_n[0] * 27, stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += stride) j.nbr[i] = -1;
}

static int grid_alloc_table(insc_grid *g, int64_t capacity_sites) {
  int64_t slots = 1024;
  while (slots < 2 * capacity_sites) slots <<= 1;
  INSC_HIP(hipMalloc((void **)&g->table, sizeof(Slot) * (size_t)slots));
  g->n_slots = slots;
  return INSC_OK;
}

static int grid_sync_errors(insc_grid *g, hipStream_t s, const char *who) {
  int32_t h[2];
  if (g->h_fresh && g->h_stream == (void *)s) {
    // the last insert left both words in pinned host memory: waiting for its stream is all it takes
    // (two small device-to-host copies and their waits cost ~50 us per call, most of a 220 000-point insert)
    INSC_HIP(hipStreamSynchronize(s));
    h[0] = g->h_n[0];
    h[1] = g->h_n[1];
  } else {
    int32_t both[17];  // d_n[0] .. d_err (= d_n + 16) in one copy
    INSC_HIP(hipMemcpyAsync(both, g->d_n, sizeof(both), hipMemcpyDeviceToHost, s));
    INSC_HIP(hipStreamSynchronize(s));
    h[0] = both[0];
    h[1] = both[16];
  }
  g->n_exact = h[0];
  g->n_upper = h[0];
  if (h[1]) {
    // reported once: the rows at fault got site -1, every other row of the call was handled, and
    // the grid stays usable
    INSC_HIP(hipMemsetAsync(g->d_err, 0, sizeof(int32_t), s));
    INSC_HIP(hipStreamSynchronize(s));
    if (g->h_n) g->h_n[1] = 0;
  }
  if (h[1] & 1) {
    set_error("%s: a coordinate is outside 0..65535 (batch 0..32767)", who);
    return INSC_ERR_COORD;
  }
  if (h[1] & 2) {
    set_error("%s: grid capacity %lld exceeded", who, (long long)g->capacity_sites);
    return INSC_ERR_CAPACITY;
  }
  return INSC_OK;
}

static int grid_ensure_scratch(insc_grid *g, int64_t P, hipStream_t s) {
  if (g->scratch_rows < P) {
    INSC_HIP(hipStreamSynchronize(s));
    if (g->slot_of_point) INSC_HIP(hipFree(g->slot_of_point));
    if (g->flags) INSC_HIP(hipFree(g->flags));
    g->slot_of_point = g->flags = nullptr;
    int64_t rows = (P + P / 2 + 1) & ~1ll;
    // (with the large insert's row states, slots and keys: five arrays of `rows` words)
    INSC_HIP(hipMalloc((void **)&g->slot_of_point, sizeof(int32_t) * 5 * (size_t)rows));
    INSC_HIP(hipMalloc((void **)&g->flags, sizeof(int32_t) * (size_t)(rows + 64)));
    g->scratch_rows = rows;
  }
  return INSC_OK;
}

// the insert proper: the caller has made sure that P more sites fit
static int grid_insert_launch(insc_grid *g, const int32_t *d_coords4, int64_t P, int32_t *d_site_of_point,
                              hipStream_t s) {
  int rc = grid_ensure_scratch(g, P, s);
  if (rc) return rc;
  const int64_t mask = g->n_slots - 1;
  const unsigned nb = grid_for(P, 256);
  int32_t *total = g->flags + g->scratch_rows;  // spare int after the flags
  const bool small = P <= FINISH_SMALL_MAX;
  const int64_t n_parts = g->n_slots >> PART_SHIFT;
  if (!small && g->n_upper == 0 && g->part && n_parts >= 1 && n_parts <= PART_MAX) {  // empty: built in LDS
    int32_t *cnt = g->part, *cursor = cnt + PART_MAX * PART_PAD, *base = cursor + PART_MAX * PART_PAD;
    int32_t *part_rows = g->slot_of_point, *state = part_rows + g->scratch_rows, *where = state + g->scratch_rows;
    uint64_t *part_keys = reinterpret_cast<uint64_t *>(where + g->scratch_rows);
    const unsigned blocks = (unsigned)((P + 1024 * PART_ROWS - 1) / (1024 * PART_ROWS));
    const size_t lds = sizeof(int32_t) * (size_t)n_parts;
    hipLaunchKernelGGL(part_count_kernel, dim3(blocks), dim3(1024), lds, s, d_coords4, P, mask, (int)n_parts, cnt, g->d_err);
    hipLaunchKernelGGL(part_scatter_kernel, dim3(blocks), dim3(1024), 2 * lds, s, d_coords4, P, mask, (int)n_parts, cnt,
                       cursor, base, part_rows, part_keys, d_site_of_point, g->flags);
    hipLaunchKernelGGL(part_winners_kernel, dim3((unsigned)n_parts), dim3(PART_THREADS), 0, s, mask, base,
                       part_rows, part_keys, g->d_n, g->flags, state, where, cnt, cursor, total + 1, g->d_err);
    INSC_LAUNCH_CHECK();
    rc = scan_exclusive_i32(g->flags, g->flags, P, total, s);
    if (rc) return rc;
    hipLaunchKernelGGL(part_assign_kernel, dim3(nb), dim3(256), 0, s, g->table, base, (int)n_parts, part_rows, part_keys,
                       state, where, g->flags, g->d_n, total, g->coords, g->capacity_sites, g->d_err, d_site_of_point,
                       g->h_n);
    INSC_LAUNCH_CHECK();
    g->n_upper += P;
    g->n_exact = -1;
    g->h_fresh = g->h_n != nullptr;
    g->h_stream = (void *)s;
    return INSC_OK;
  }
  hipLaunchKernelGGL(grid_claim_kernel, dim3(nb), dim3(256), 0, s, g->table, mask, d_coords4, P, g->slot_of_point,
                     small ? nullptr : g->flags, d_site_of_point, g->d_err);
  if (small) {
    hipLaunchKernelGGL(grid_finish_small_kernel, dim3(1), dim3(1024), 0, s, g->table, d_coords4, g->slot_of_point,
                       (int)P, g->d_n, g->coords, g->capacity_sites, g->d_err, d_site_of_point, g->h_n);
    INSC_LAUNCH_CHECK();
    g->n_upper += P;
    g->n_exact = -1;
    g->h_fresh = g->h_n != nullptr;
    g->h_stream = (void *)s;
    return INSC_OK;
  }
  hipLaunchKernelGGL(grid_resolve_kernel, dim3(nb), dim3(256), 0, s, g->table, g->slot_of_point, P, g->flags,
                     d_site_of_point, g->d_n, total + 1);
  INSC_LAUNCH_CHECK();
  rc = scan_exclusive_i32(g->flags, g->flags, P, total, s);
  if (rc) return rc;
  hipLaunchKernelGGL(grid_assign_kernel, dim3(nb), dim3(256), 0, s, g->table, d_coords4, g->slot_of_point, g->flags,
                     P, g->d_n, total, g->coords, g->capacity_sites, g->d_err, d_site_of_point, g->h_n);
  INSC_LAUNCH_CHECK();
  g->n_upper += P;
  g->n_exact = -1;
  g->h_fresh = g->h_n != nullptr;
  g->h_stream = (void *)s;
  return INSC_OK;
}

int grid_insert_nosync(insc_grid *g, const int32_t *d_coords4, int64_t P, int32_t *d_site_of_point, hipStream_t s) {
  if (P <= 0) return INSC_OK;
  if (g->n_upper + P > g->capacity_sites) {
    set_error("grid_insert_nosync: %lld sites + %lld points exceed capacity %lld", (long long)g->n_upper,
              (long long)P, (long long)g->capacity_sites);
    return INSC_ERR_CAPACITY;
  }
  return grid_insert_launch(g, d_coords4, P, d_site_of_point, s);
}

// The sites of the last insert, appended to a processing order sorted among themselves (one
// workgroup, bitonic sort in LDS): tiles made of sites in arrival order use every filter offset
// and gather from all over the scene, which costs a convolution a quarter of its speed.
// Key = Morton code of the 64^3 block | neighbour pattern (the key of insc_order_build).
// More new sites than SORT_NEW_MAX keep their arrival order (any order gives the same results).
constexpr int SORT_NEW_MAX = 8192;
// LDS of the two appends: the keys of the new sites, their indices in two buffers that a radix pass reads
// and writes in turn, the digit counters of a pass ([digit][wavefront], 17 words per digit so that the
// lanes of a wavefront - same wavefront, different digits - fall into different banks) twice (the other
// set is zeroed for the pass that follows), and a few words for sums across the wavefronts.
// LDS of the two appends: the keys of the new sites in two buffers that a merge round reads and writes in turn
struct OrderLds {
  uint64_t key[2][SORT_NEW_MAX];
};
// Sorted by (key, arrival) - one 64-bit word per site, sort key in the upper 51 bits, index among the new
// sites in the lower 13, so no two words are equal - by one workgroup (all of it on one compute unit: what
// it costs is the number of instructions, ~14 us for 3000 sites): every wavefront sorts runs of 64
// words in registers (a bitonic network over the lanes), then rounds of merges double the runs: a word's
// place in the merged run is its place in its own run plus the number of smaller words in the sibling run,
// found by a binary search of a fixed number of steps, the searches of a thread's words side by side.
// log2(n / 64) rounds with one barrier each.  (A bitonic network over all keys took 78 passes for 4096 of
// them, 40-48 us for the 2-3k new sites of a frame; a radix sort eight bits a pass, 3 us per pass.)
__device__ __forceinline__ void order_append_sorted_body(const int first, const int n,
                                                         const int32_t *__restrict__ coords,
                                                         const int32_t *__restrict__ nbr, int32_t *__restrict__ order,
                                                         int32_t *__restrict__ pos, OrderLds &L) {
  const int tid = threadIdx.x, lane = tid & 63;
  if (n <= 0) return;
  if (n > SORT_NEW_MAX) {
    for (int i = tid; i < n; i += 1024) {
      order[first + i] = first + i;
      if (pos) pos[first + i] = first + i;
    }
    return;
  }
  const int N = (n + 63) & ~63;  // whole runs of 64; the words past n have all key bits set and end up last
  for (int i = tid; i < N; i += 1024) {
    uint64_t k = ~8191ull | (uint64_t)i;
    if (i < n) {
      const int v = first + i;
      const int4 c = reinterpret_cast<const int4 *>(coords)[v];
      uint32_t m = 0;
      for (int j = 0; j < 27; j++) m |= (nbr[(int64_t)v * 27 + j] >= 0 ? 1u : 0u) << j;
      k = (order_key(c, m) << 13) | (uint64_t)i;
    }
    // the run of 64 that this word belongs to is held by one wavefront (i and lane agree mod 64): sorted here
#pragma unroll
    for (int kk = 2; kk <= 64; kk <<= 1) {
#pragma unroll
      for (int j = kk >> 1; j > 0; j >>= 1) {
        const uint64_t y = __shfl_xor(k, j, 64);
        const bool keep_small = ((lane & j) == 0) == ((lane & kk) == 0);
        k = keep_small ? (k < y ? k : y) : (k < y ? y : k);
      }
    }
    L.key[0][i] = k;
  }
  __syncthreads();
  int src = 0;
  for (int len = 64, lg = 6; len < N; len <<= 1, lg++) {
    const uint64_t *a = L.key[src];
    uint64_t *d = L.key[src ^ 1];
    uint64_t w[8];
    int sib[8], sib_n[8], lo[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int p = e * 1024 + tid;
      if (e * 1024 >= N) continue;  // (uniform)
      const int run = p >> lg;
      w[e] = p < N ? a[p] : 0;
      sib[e] = (run ^ 1) << lg;
      sib_n[e] = p < N ? min(max(N - sib[e], 0), len) : 0;
      lo[e] = 0;
    }
    // words of the sibling run that come before w: the smaller ones
    for (int step = len; step >= 1; step >>= 1) {
#pragma unroll
      for (int e = 0; e < 8; e++) {
        if (e * 1024 >= N) continue;
        const int probe = lo[e] + step;
        if (probe <= sib_n[e]) {
          if (a[sib[e] + probe - 1] < w[e]) lo[e] = probe;
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int p = e * 1024 + tid;
      if (e * 1024 >= N || p >= N) continue;
      const int run = p >> lg;
      d[((run >> 1) << (lg + 1)) + (p & (len - 1)) + lo[e]] = w[e];
    }
    __syncthreads();
    src ^= 1;
  }
  for (int i = tid; i < n; i += 1024) {
    const int v = first + (int)(L.key[src][i] & 8191);
    order[first + i] = v;
    if (pos) pos[v] = first + i;
  }
}
// The new sites in the order grouped by the position inside the parent cell (eight groups, each in the
// sequence of the processing order just written): a stable counting sort of that order, which gives
// what sorting by (group, position) gives.  One workgroup of 1024 threads, thread t owns the positions
// 8t .. 8t+7 of the new sites; counts per group travel as eight 16-bit fields in two 64-bit words
// (at most SORT_NEW_MAX = 8192 sites, so no field overflows).
__device__ __forceinline__ void order_append_grouped_body(const int first, const int n,
                                                          const int32_t *__restrict__ offset,
                                                          const int32_t *__restrict__ order,
                                                          int32_t *__restrict__ bo_order, int32_t *__restrict__ bo_pos,
                                                          uint64_t *lds) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (n <= 0) return;
  if (n > SORT_NEW_MAX) {
    for (int i = tid; i < n; i += 1024) {
      bo_order[first + i] = first + i;
      bo_pos[first + i] = first + i;
    }
    return;
  }
  int v[8], o[8];
  uint64_t c0 = 0, c1 = 0;  // groups 0..3 and 4..7
#pragma unroll
  for (int e = 0; e < 8; e++) {
    const int q = tid * 8 + e;
    v[e] = q < n ? order[first + q] : -1;
    o[e] = v[e] >= 0 ? (offset[v[e]] & 7) : 0;
    if (v[e] >= 0) {
      if (o[e] < 4) c0 += 1ull << (16 * o[e]);
      else c1 += 1ull << (16 * (o[e] - 4));
    }
  }
  // inclusive scan over the threads: inside a wavefront, then over the 16 wavefronts through LDS
  uint64_t s0 = c0, s1 = c1;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint64_t a0 = __shfl_up(s0, d, 64), a1 = __shfl_up(s1, d, 64);
    if (lane >= d) {
      s0 += a0;
      s1 += a1;
    }
  }
  if (lane == 63) {
    lds[wave * 2] = s0;
    lds[wave * 2 + 1] = s1;
  }
  __syncthreads();
  uint64_t w0 = 0, w1 = 0, t0 = 0, t1 = 0;  // sums of the wavefronts before this one; of all
  for (int w = 0; w < 16; w++) {
    const uint64_t a0 = lds[w * 2], a1 = lds[w * 2 + 1];
    if (w < wave) {
      w0 += a0;
      w1 += a1;
    }
    t0 += a0;
    t1 += a1;
  }
  const uint64_t e0 = w0 + s0 - c0, e1 = w1 + s1 - c1;  // exclusive: sites of each group before this thread
  int base[8], run[8];
  int acc = 0;
#pragma unroll
  for (int g = 0; g < 8; g++) {
    base[g] = acc;
    acc += (int)(((g < 4 ? t0 : t1) >> (16 * (g & 3))) & 0xFFFF);
    run[g] = (int)(((g < 4 ? e0 : e1) >> (16 * (g & 3))) & 0xFFFF);
  }
#pragma unroll
  for (int e = 0; e < 8; e++) {
    if (v[e] < 0) continue;
    int dest = 0;
#pragma unroll
    for (int g = 0; g < 8; g++) {
      if (o[e] == g) {
        dest = first + base[g] + run[g];
        run[g]++;
      }
    }
    bo_order[dest] = v[e];
    bo_pos[v[e]] = dest;
  }
}

// both orders of a scale by one workgroup: the processing order of the 3^3 layers, then - where the
// scale has a coarser one above it - the order grouped by the position inside the parent cell
struct OrderBothJob {
  const int32_t *d_n, *coords, *nbr, *offset;  // offset null: no second order
  int32_t *order, *pos, *bo_order, *bo_pos;
  int all;  // order every site of the grid, not only those of the last insert
};
struct OrderBothBatch {
  OrderBothJob job[16];
};
__global__ __launch_bounds__(1024) void order_append_both_batch_kernel(OrderBothBatch b) {
  __shared__ OrderLds L;
  const OrderBothJob &j = b.job[blockIdx.x];
  const int first = j.all ? 0 : j.d_n[1], n = j.d_n[0] - first;
  order_append_sorted_body(first, n, j.coords, j.nbr, j.order, j.pos, L);
  if (!j.offset) return;
  __syncthreads();  // the order written above is read below (by other threads than wrote it), and the LDS is reused
  order_append_grouped_body(first, n, j.offset, j.order, j.bo_order, j.bo_pos, L.key[0]);
}

int64_t order_sorted_max() { return SORT_NEW_MAX; }

// Several grids emptied in one launch, and with each (optionally) an int32 array set to -1 - the child
// map that hangs off it - and one more array zeroed (running sums of an input layer).
struct ClearJob {
  Slot *table;
  int64_t n_slots;
  int32_t *d_n, *d_err;
  int32_t *minus1;
  int64_t n_minus1;
};
struct ClearBatch {
  ClearJob job[16];
  uint32_t *zero;  // 4-byte words
  int64_t n_zero;
};
__global__ __launch_bounds__(256) void grid_clear_batch_kernel(ClearBatch b, int n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if ((int)blockIdx.y == n) {
    for (int64_t i = t; i < b.n_zero; i += stride) b.zero[i] = 0u;
    return;
  }
  const ClearJob &j = b.job[blockIdx.y];
  for (int64_t i = t; i < j.n_slots; i += stride) {
    Slot e;
    e.key = INSC_EMPTY_KEY;
    e.val = VAL_UNSET;
    e.pad = 0;
    j.table[i] = e;
  }
  for (int64_t i = t; i < j.n_minus1; i += stride) j.minus1[i] = -1;
  if (t == 0) {
    j.d_n[0] = 0;
    j.d_n[1] = 0;
    *j.d_err = 0;
  }
}

int grid_clear_batch(insc_grid *const *grids, int32_t *const *minus1, const int64_t *n_minus1, int n, void *zero,
                     int64_t zero_bytes, hipStream_t s) {
  if (n <= 0 || n > 16 || (zero_bytes & 3)) {
    set_error("grid_clear_batch: 1..16 grids, a multiple of four bytes to zero");
    return INSC_ERR_ARG;
  }
  ClearBatch b;
  int64_t most = zero_bytes / 4;
  for (int i = 0; i < n; i++) {
    insc_grid *g = grids[i];
    b.job[i] = ClearJob{g->table, g->n_slots, g->d_n, g->d_err, minus1 ? minus1[i] : nullptr,
                        (minus1 && minus1[i]) ? n_minus1[i] : 0};
    most = std::max(most, std::max(g->n_slots, b.job[i].n_minus1));
    g->n_upper = 0;
    g->n_exact = 0;
    g->h_fresh = false;
  }
  b.zero = (uint32_t *)zero;
  b.n_zero = zero ? zero_bytes / 4 : 0;
  hipLaunchKernelGGL(grid_clear_batch_kernel, dim3(grid_for(most, 256, 2048), (unsigned)(n + (b.n_zero ? 1 : 0))), dim3(256),
                     0, s, b, n);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

// ---- the inserts of a whole frame, all scales at once ----------------------------------------
// The reference inserts scale by scale: the sites a frame adds at one scale are halved and inserted
// at the next coarser one, a chain in which every step waits for the ids of the step before.  The
// chain is not needed: a site that is new at scale l has only new sites below it, so the order in
// which that chain numbers the new sites of scale l - first appearance among the new sites of scale
// l - 1 in id order - is the order of the smallest ROW of the frame's point list that falls into
// each new cell.  So every scale takes the frame's points themselves (coordinates >> l) and ranks
// its new cells by their smallest row, all scales at the same time, in three launches for up to
// FINISH_SMALL_MAX points: claim (one thread per row and scale; a row that finds its cell already
// numbered is done - at the coarse scales that is nearly every row), finish (one workgroup per
// scale ranks the winners in row order and hands out the ids), link (parent / offset / child
// between the scales).  A frame is all or nothing: if some coordinate is out of range, finish takes
// the frame's claims out of the tables again (they sit in slots that were empty before, so the
// tables are then exactly what they were) and nothing is numbered.
// Values that other rows of the frame may have changed are read past the L1 (atomic loads): the
// claims are atomics performed in L2.
struct FrameLevelDev {
  Slot *table;
  int64_t mask, capacity;
  int32_t *coords, *d_n, *d_err;
  int32_t *parent, *offset, *child;  // link to the next coarser scale (null at the coarsest)
};
struct FrameInsertArgs {
  FrameLevelDev lv[16];
  int n_levels;
};
__device__ __forceinline__ int table_val(const Slot *table, int64_t s) {
  return __hip_atomic_load(&table[s].val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr uint32_t REC_SITE = 0x80000000u;  // rec = REC_SITE | id: the cell was numbered before this frame
constexpr uint32_t REC_DUP = 0x40000000u;   // rec = REC_DUP | slot: the cell was claimed first by another row of the frame
constexpr uint32_t REC_NONE = 0xFFFFFFFFu;  // no slot: bad coordinate, or the table is full
__device__ __forceinline__ bool rec_is_slot(uint32_t r) { return r != REC_NONE && !(r & REC_SITE); }
__device__ __forceinline__ int64_t rec_slot(uint32_t r) { return (int64_t)(r & ~REC_DUP); }
__device__ __forceinline__ int4 frame_point(const int32_t *__restrict__ coords_in, int cols, int p, int l) {
  const int32_t *c = coords_in + (int64_t)p * cols;
  return make_int4(c[0] >> l, c[1] >> l, c[2] >> l, cols > 3 ? c[3] : 0);
}
// rec[l * P + p]: what row p found at scale l - REC_SITE | id, the slot it claimed first, REC_DUP | the slot
// another row claimed first, or REC_NONE (protocol: see grid_claim_kernel).  With flag / rep (frames
// ranked by a prefix sum) the first claimants also enter themselves as winners there: flag 1, rep -1.
__global__ __launch_bounds__(256) void frame_claim_kernel(FrameInsertArgs a, const int32_t *__restrict__ coords_in,
                                                          int cols, int P, int32_t *__restrict__ bad, int32_t frame,
                                                          uint32_t *__restrict__ rec, int shared_from,
                                                          int32_t *__restrict__ flag, int32_t *__restrict__ rep,
                                                          int p_begin, int p_end) {
  const int l = blockIdx.y;
  const FrameLevelDev &L = a.lv[l];
  const int p = p_begin + blockIdx.x * 256 + threadIdx.x;  // (this launch serves rows p_begin .. p_end - 1)
  if (p >= p_end) return;
  const int64_t idx = (int64_t)l * P + p;
  const int32_t *c0 = coords_in + (int64_t)p * cols;
  if (!coord_ok(c0[0], c0[1], c0[2], cols > 3 ? c0[3] : 0)) {
    if (l == 0) bad[0] = frame;
    rec[idx] = REC_NONE;
    if (flag) {
      flag[idx] = 0;
      rep[idx] = -1;
    }
    return;
  }
  const int4 c = frame_point(coords_in, cols, p, l);
  const uint64_t key = pack_key(c.x, c.y, c.z, c.w);
  auto claim = [&]() -> uint32_t {
    Walk w = walk_begin(key, L.mask);
    do {
      const int64_t s = walk_slot(w);
      const int4 raw = *reinterpret_cast<const int4 *>(&L.table[s]);  // key (two words), val, pad
      unsigned long long k = ((unsigned long long)(unsigned)raw.y << 32) | (unsigned)raw.x;
      if (k == key && raw.z >= 0 && raw.z < VAL_PENDING) return REC_SITE | (uint32_t)raw.z;  // numbered before this frame
      const bool seen = k == key;  // the slot already held this key when it was read
      if (k == INSC_EMPTY_KEY) {
        k = atomicCAS(&L.table[s].key, INSC_EMPTY_KEY, (unsigned long long)key);
        if (k == INSC_EMPTY_KEY) {  // first claimant
          __hip_atomic_store(&L.table[s].pad, p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          return (uint32_t)s;
        }
      }
      if (k == key) {
        // (a smaller row that this row has seen in the slot - first claimant in pad, later one in val -
        // stands: the values only ever go down during a frame, so a stale read errs on the side of one
        // more atomic; a dropped frame takes its pads out again)
        const bool beaten = seen && ((raw.w > 0 && raw.w - 1 < p) || (raw.z >= VAL_PENDING && raw.z <= VAL_PENDING + p));
        if (!beaten) atomicMin(&L.table[s].val, VAL_PENDING + p);
        return REC_DUP | (uint32_t)s;
      }
    } while (walk_next(w));
    return REC_NONE;
  };
  uint32_t r = REC_NONE;
  if (l < shared_from) {
    r = claim();
  } else {
    // Above the input scale the rows of a wavefront often fall into the same cell (at the coarsest scale
    // of a full frame thousands of rows per cell), and atomics on one address are served one at a time.
    // Of the lanes that share a cell only the first - the smallest row, rows ascending with the lanes -
    // sends a claim, and the others take its answer, as later claimants: whoever numbers the cell, it is
    // not one of them.  Finding the first lane of every cell takes 64 broadcasts and no memory access,
    // and the first lanes then claim side by side.
    const int lane = (int)(threadIdx.x & 63);
    const uint32_t klo = (uint32_t)key, khi = (uint32_t)(key >> 32);
    int leader = lane;
    const uint64_t live = __ballot(true);
    for (int i = 0; i < 64; i++) {
      if (!((live >> i) & 1ull)) continue;  // (uniform)
      const uint32_t ilo = (uint32_t)__builtin_amdgcn_readlane((int)klo, i), ihi = (uint32_t)__builtin_amdgcn_readlane((int)khi, i);
      if (i < leader && ilo == klo && ihi == khi) leader = i;
    }
    uint32_t mine = REC_NONE;
    if (lane == leader) mine = claim();
    const uint32_t got = (uint32_t)__shfl((int)mine, leader, 64);
    r = (lane == leader || !rec_is_slot(got)) ? got : (got | REC_DUP);
  }
  if (r == REC_NONE) atomicOr(L.d_err, 2);
  rec[idx] = r;
  if (flag) {
    flag[idx] = (rec_is_slot(r) && !(r & REC_DUP)) ? 1 : 0;
    rep[idx] = -1;
  }
}

// site[l * P + p] = site of row p at scale l (while the kernel runs: the row's state, as site_of_point
// in grid_finish_small_kernel)
__global__ __launch_bounds__(1024) void frame_finish_kernel(FrameInsertArgs a, const int32_t *__restrict__ coords_in,
                                                            int cols, int P, const int32_t *__restrict__ bad,
                                                            int32_t frame, int32_t *__restrict__ sop,
                                                            int32_t *site, const uint32_t *__restrict__ rec,
                                                            int32_t *h_counts) {
  __shared__ int wave_total[16];
  const int l = blockIdx.x;
  const FrameLevelDev &L = a.lv[l];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = (P + 1023) / 1024, p0 = tid * per;
  const int n_before = L.d_n[0];
  site += (int64_t)l * P;
  rec += (int64_t)l * P;
  uint32_t rr[16];
#pragma unroll
  for (int j = 0; j < 16; j++) rr[j] = (j < per && p0 + j < P) ? rec[p0 + j] : REC_NONE;
  if (bad[0] == frame) {
    // the frame is dropped: its claims leave the table, no row gets a site
#pragma unroll
    for (int j = 0; j < 16; j++) {
      if (j >= per || p0 + j >= P) continue;
      if (rec_is_slot(rr[j])) {
        __hip_atomic_store(&L.table[rec_slot(rr[j])].val, VAL_UNSET, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&L.table[rec_slot(rr[j])].pad, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&L.table[rec_slot(rr[j])].key, INSC_EMPTY_KEY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      site[p0 + j] = -1;
      if (l == 0) sop[p0 + j] = -1;
    }
    if (tid == 0) {
      L.d_n[1] = n_before;
      if (h_counts) {
        h_counts[2 * l] = n_before;
        h_counts[2 * l + 1] = 0;
        if (l == 0) h_counts[2 * a.n_levels] = frame;
      }
    }
    return;
  }
  // states: own row (first claimant), ST_DUP, -2 - id (numbered before this frame), -1
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int p = p0 + j;
    if (j >= per || p >= P) continue;
    const uint32_t r = rr[j];
    site[p] = r == REC_NONE ? -1 : (r & REC_SITE) ? -2 - (int)(r & ~REC_SITE) : (r & REC_DUP) ? ST_DUP : p;
  }
  __threadfence_block();
  __syncthreads();
  // later claimants find out who numbers their cell
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int p = p0 + j;
    if (j >= per || p >= P || !rec_is_slot(rr[j]) || !(rr[j] & REC_DUP)) continue;
    const int4 raw = *reinterpret_cast<const int4 *>(&L.table[rec_slot(rr[j])]);
    if (raw.z >= 0 && raw.z < VAL_PENDING) {  // (the key was there all along; the row had read a stale empty slot)
      site[p] = -2 - raw.z;
      continue;
    }
    const int first = raw.w - 1, later = raw.z - VAL_PENDING;
    if (later == p && p < first) {
      site[p] = p;
      site[first] = p;
    } else {
      site[p] = first < later ? first : later;
    }
  }
  __threadfence_block();
  __syncthreads();
  // winners, ranked in row order
  int st[16];
  unsigned win = 0;
  int cnt = 0;
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int p = p0 + j;
    st[j] = (j < per && p < P) ? site[p] : -1;
    if (j < per && p < P && st[j] == p) {
      win |= 1u << j;
      cnt++;
    }
  }
  int incl = cnt;
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_up(incl, d, 64);
    if (lane >= d) incl += v;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  int base = n_before + incl - cnt, total = 0;
  for (int w = 0; w < 16; w++) {
    if (w < wave) base += wave_total[w];
    total += wave_total[w];
  }
  // winners publish their id and record the new site
#pragma unroll
  for (int j = 0; j < 16; j++) {
    if (!((win >> j) & 1u)) continue;
    const int p = p0 + j, id = base++;
    if (id >= L.capacity) {
      atomicOr(L.d_err, 2);
      site[p] = -1;
      if (l == 0) sop[p] = -1;
      continue;
    }
    const int4 c = frame_point(coords_in, cols, p, l);
    L.table[rec_slot(rr[j])].val = id;
    reinterpret_cast<int4 *>(L.coords)[id] = c;
    if (L.offset) L.offset[id] = (c.x & 1) * 4 + (c.y & 1) * 2 + (c.z & 1);
    site[p] = id;
    if (l == 0) sop[p] = id;
  }
  __threadfence_block();
  __syncthreads();
  // every other row takes its site from the row that numbered its cell
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int p = p0 + j;
    if (j >= per || p >= P || ((win >> j) & 1u)) continue;
    const int v = st[j] < -1 ? -2 - st[j] : st[j] >= 0 ? site[st[j]] : -1;
    site[p] = v;
    if (l == 0) sop[p] = v;
  }
  if (total > L.capacity - n_before) total = (int)(L.capacity - n_before);  // (the error flag is up)
  if (tid == 0) {
    L.d_n[1] = n_before;
    L.d_n[0] = n_before + total;
    if (h_counts) {
      h_counts[2 * l] = n_before + total;
      h_counts[2 * l + 1] = __hip_atomic_load(L.d_err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (l == 0) h_counts[2 * a.n_levels] = 0;
    }
  }
}

// the links of the new sites of scale blockIdx.y to the scale above: every row that fell into a new
// cell writes that cell's parent (rows of one cell write the same values)
__global__ void frame_link_kernel(FrameInsertArgs a, int P, const int32_t *__restrict__ site) {
  const int l = blockIdx.y;
  const FrameLevelDev &F = a.lv[l];
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int i = site[(int64_t)l * P + p];
  if (i < F.d_n[1]) return;  // not a site of this frame (or no site at all)
  const int par = site[(int64_t)(l + 1) * P + p];
  F.parent[i] = par;
  if (par >= 0 && F.child) F.child[(int64_t)par * 8 + F.offset[i]] = i;
}

// Frames of more points than one workgroup per scale can rank: the same three steps with the ranking
// done by a prefix sum over all (scale, row) pairs at once - flag (is this row the winner of its
// cell; if not, which row is), scan, assign (a winner publishes its id and the site's coordinates;
// every row works out its site from the prefix sums alone, a loser through its winner's row, so no
// row has to wait for another one's write).
__global__ __launch_bounds__(256) void frame_flag_kernel(FrameInsertArgs a, int P, uint32_t *__restrict__ rec,
                                                         int32_t *__restrict__ flag, int32_t *__restrict__ rep,
                                                         int32_t *__restrict__ n_before) {
  const int l = blockIdx.y;
  const FrameLevelDev &L = a.lv[l];
  const int p = blockIdx.x * 256 + threadIdx.x;
  if (p == 0) {
    n_before[l] = L.d_n[0];
    if (l == 0) flag[(int64_t)a.n_levels * P] = 0;  // (one entry past the end: the scan then leaves the grand total there)
  }
  if (p >= P) return;
  const int64_t lp = (int64_t)l * P, idx = lp + p;
  const uint32_t r = rec[idx];
  // (first claimants entered themselves as winners in the claim kernel; only later claimants look at their slot)
  if (!rec_is_slot(r) || !(r & REC_DUP)) return;
  const int4 raw = *reinterpret_cast<const int4 *>(&L.table[rec_slot(r)]);
  if (raw.z >= 0 && raw.z < VAL_PENDING) {  // (the key was there all along; the row had read a stale empty slot)
    rec[idx] = REC_SITE | (uint32_t)raw.z;
    return;
  }
  const int first = raw.w - 1, later = raw.z - VAL_PENDING;
  if (later == p && p < first) {
    flag[idx] = 1;
    flag[lp + first] = 0;
    rep[lp + first] = p;
  } else {
    rep[idx] = first < later ? first : later;
  }
}

__global__ __launch_bounds__(256) void frame_assign_kernel(FrameInsertArgs a, const int32_t *__restrict__ coords_in,
                                                           int cols, int P, const int32_t *__restrict__ bad,
                                                           int32_t frame, int32_t *__restrict__ sop,
                                                           int32_t *__restrict__ site, const uint32_t *__restrict__ rec,
                                                           const int32_t *__restrict__ excl,
                                                           const int32_t *__restrict__ rep,
                                                           const int32_t *__restrict__ n_before_all, int32_t *h_counts) {
  const int l = blockIdx.y;
  const FrameLevelDev &L = a.lv[l];
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int n_before = n_before_all[l];
  const int64_t lp = (int64_t)l * P;
  const bool dropped = bad[0] == frame;
  if (p == 0) {
    int total = dropped ? 0 : excl[lp + P] - excl[lp];
    // (more new sites than the scale has room for: the rows beyond get no site below; the flag is worked
    // out here as well, since those rows may raise it only after this thread has read it)
    const bool over = total > L.capacity - n_before;
    if (over) {
      total = (int)(L.capacity - n_before);
      atomicOr(L.d_err, 2);
    }
    L.d_n[1] = n_before;
    L.d_n[0] = n_before + total;
    if (h_counts) {
      h_counts[2 * l] = n_before + total;
      h_counts[2 * l + 1] =
          dropped ? 0 : (__hip_atomic_load(L.d_err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) | (over ? 2 : 0));
      if (l == 0) h_counts[2 * a.n_levels] = dropped ? frame : 0;
    }
  }
  if (p >= P) return;
  const uint32_t r = rec[lp + p];
  int st = -1;
  if (dropped) {
    // the frame is dropped: its claims leave the table, no row gets a site
    if (rec_is_slot(r)) {
      __hip_atomic_store(&L.table[rec_slot(r)].val, VAL_UNSET, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&L.table[rec_slot(r)].pad, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&L.table[rec_slot(r)].key, INSC_EMPTY_KEY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else if (r != REC_NONE) {
    if (r & REC_SITE) {
      st = (int)(r & ~REC_SITE);
    } else {
      const int e = excl[lp + p];
      const bool win = excl[lp + p + 1] - e == 1;
      const int wrow = win ? p : rep[lp + p];
      if (wrow >= 0) {
        const int id = n_before + (win ? e : excl[lp + wrow]) - excl[lp];
        if (id < L.capacity) {
          st = id;
          if (win) {
            const int4 c = frame_point(coords_in, cols, p, l);
            L.table[rec_slot(r)].val = id;
            reinterpret_cast<int4 *>(L.coords)[id] = c;
            if (L.offset) L.offset[id] = (c.x & 1) * 4 + (c.y & 1) * 2 + (c.z & 1);
          }
        } else if (win) {
          atomicOr(L.d_err, 2);
        }
      }
    }
  }
  site[lp + p] = st;
  if (l == 0) sop[p] = st;
}

int frame_insert_levels(const FrameInsertLevel *lv, int n_levels, const int32_t *d_coords, int cols, int64_t P,
                        int32_t *d_bad, int32_t frame, int32_t *d_sop, int32_t *h_counts, hipStream_t s) {
  if (P <= 0) return INSC_OK;
  if (n_levels < 1 || n_levels > 16 || P * n_levels >= (1ll << 30)) {
    set_error("frame_insert_levels: %d scales, %lld points (at most 16 scales, 2^30 (scale, point) pairs)", n_levels,
              (long long)P);
    return INSC_ERR_ARG;
  }
  FrameInsertArgs a;
  a.n_levels = n_levels;
  for (int l = 0; l < n_levels; l++) {
    insc_grid *g = lv[l].grid;
    if (g->n_upper + P > g->capacity_sites) {
      set_error("frame_insert_levels: %lld sites + %lld points exceed the capacity %lld of scale %d", (long long)g->n_upper,
                (long long)P, (long long)g->capacity_sites, l);
      return INSC_ERR_CAPACITY;
    }
    if (g->n_slots > (1ll << 30)) {  // (a row's record keeps the slot in 30 bits)
      set_error("frame_insert_levels: the table of scale %d has more than 2^30 slots", l);
      return INSC_ERR_ARG;
    }
    a.lv[l] = FrameLevelDev{g->table, g->n_slots - 1, g->capacity_sites, g->coords, g->d_n, g->d_err,
                            lv[l].parent, lv[l].offset, lv[l].child};
  }
  const bool large = P > FINISH_SMALL_MAX;
  const size_t PL = (size_t)P * n_levels;
  void *ws;
  int rc = workspace(WS_API, s, PL * (large ? 4 : 2) * sizeof(int32_t) + 512, &ws);
  if (rc) return rc;
  int32_t *site = (int32_t *)ws;
  uint32_t *rec = (uint32_t *)(site + PL);
  // (above the input scale the rows of a wavefront that fall into one cell share a claim)
  const int shared_from = 1;
  int32_t *rep = large ? (int32_t *)(rec + PL) : nullptr, *flag = large ? rep + PL : nullptr;
  // The claims are bound by the rate of atomics on scattered addresses (some 6 per nanosecond on this
  // part, whatever their width or scope), and with all rows in flight at once every row of a cell sends
  // one: 7 x 165 000 for a full frame of a 7-scale network, though its coarse scales hold a few thousand
  // cells.  A cell's first row is its smallest, so the first sixteenth of the rows go ahead in a launch
  // of their own: they claim nearly every cell of the coarse scales, and the rows of the second launch,
  // which find a smaller row there, send nothing.  165 000 points at 7 scales: 132 us in one launch,
  // 18 + 64 us in two (a sixty-fourth of the rows first: 13 + 79 us; a quarter: 43 + 49 us).
  const int64_t head = large ? std::max<int64_t>(P / 16, 1024) : P;
  for (int part = 0; part < (head < P ? 2 : 1); part++) {
    const int64_t b = part ? head : 0, e = (part || head >= P) ? P : head;
    hipLaunchKernelGGL(frame_claim_kernel, dim3(grid_for(e - b, 256), (unsigned)n_levels), dim3(256), 0, s, a, d_coords,
                       cols, (int)P, d_bad, frame, rec, shared_from, flag, rep, (int)b, (int)e);
  }
  if (large) {
    int32_t *n_before = flag + PL + 1;
    hipLaunchKernelGGL(frame_flag_kernel, dim3(grid_for(P, 256), (unsigned)n_levels), dim3(256), 0, s, a, (int)P, rec, flag,
                       rep, n_before);
    INSC_LAUNCH_CHECK();
    if ((rc = scan_exclusive_i32(flag, flag, (int64_t)PL + 1, nullptr, s))) return rc;
    hipLaunchKernelGGL(frame_assign_kernel, dim3(grid_for(P, 256), (unsigned)n_levels), dim3(256), 0, s, a, d_coords, cols,
                       (int)P, (const int32_t *)d_bad, frame, d_sop, site, (const uint32_t *)rec, (const int32_t *)flag,
                       (const int32_t *)rep, (const int32_t *)n_before, h_counts);
  } else {
    hipLaunchKernelGGL(frame_finish_kernel, dim3((unsigned)n_levels), dim3(1024), 0, s, a, d_coords, cols, (int)P,
                       (const int32_t *)d_bad, frame, d_sop, site, (const uint32_t *)rec, h_counts);
  }
  if (n_levels > 1)
    hipLaunchKernelGGL(frame_link_kernel, dim3(grid_for(P, 256), (unsigned)(n_levels - 1)), dim3(256), 0, s, a, (int)P,
                       (const int32_t *)site);
  INSC_LAUNCH_CHECK();
  for (int l = 0; l < n_levels; l++) {
    lv[l].grid->n_upper += P;
    lv[l].grid->n_exact = -1;
    lv[l].grid->h_fresh = false;
  }
  return INSC_OK;
}


// ---- insert without allocation -------------------------------------------------------------
// Scratch of insc_grid_insert_noalloc: the slot every row of the call claimed (what the grid's own,
// growable slot_of_point buffer holds for insc_grid_insert).  One copy of the array lives on every
// device the library's code is loaded on, at its own address; the name below is only the host's
// handle for hipGetSymbolAddress and is never passed to a kernel.  Every entry a call reads was
// written by the same call's first kernel, so nothing has to be cleared between calls.
constexpr int NOALLOC_MAX_POINTS = FINISH_SMALL_MAX;
static __device__ __align__(256) int32_t scratch[NOALLOC_MAX_POINTS];
constexpr int MAX_DEVICES = 64;
static int32_t *g_scratch_ptr[MAX_DEVICES] = {nullptr};
static std::mutex g_scratch_mu;

// address of `scratch` on the current device, looked up once per device
static int scratch_on_current_device(int32_t **out) {
  int dev = -1;
  INSC_HIP(hipGetDevice(&dev));
  INSC_REQUIRE(dev >= 0 && dev < MAX_DEVICES, INSC_ERR_STATE, "device %d is beyond the %d this library keeps scratch for",
               dev, MAX_DEVICES);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    int32_t *p = nullptr;
    INSC_HIP(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
    INSC_REQUIRE(p, INSC_ERR_HIP, "hipGetSymbolAddress gave no address for the insert scratch on device %d", dev);
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return INSC_OK;
}

int grid_noalloc_setup() {
  int32_t *p;
  return scratch_on_current_device(&p);
}

int ssc3_new_sites_batch(const insc_grid *const *grids, int32_t *const *d_nbr, int n, int64_t n_new_upper,
                         hipStream_t s, const PlanRef *plans, bool all_new) {
  if (n <= 0 || n_new_upper <= 0) return INSC_OK;
  if (n > 16) {
    set_error("ssc3_new_sites_batch: at most 16 grids");
    return INSC_ERR_ARG;
  }
  NewSitesBatch b;
  for (int i = 0; i < n; i++) {
    b.job[i] = NewSitesJob{grids[i]->table, grids[i]->n_slots - 1, grids[i]->coords, grids[i]->d_n, d_nbr[i], nullptr, nullptr, nullptr, 0};
    if (plans && plans[i].plan) {
      b.job[i].plan = plans[i].plan;
      b.job[i].tmask = plans[i].tmask;
      b.job[i].pos = plans[i].pos;
      b.job[i].ld = plans[i].ld;
    }
  }
  b.symmetric = all_new ? 1 : 0;
  if (all_new)
    hipLaunchKernelGGL(ssc3_nbr_fill_batch_kernel, dim3(grid_for(n_new_upper * 27, 1024, 4096), (unsigned)n), dim3(256), 0,
                       s, b);
  hipLaunchKernelGGL(ssc3_nbr_new_batch_kernel, dim3(grid_for(n_new_upper * 27, 256, 1ll << 30), (unsigned)n), dim3(256),
                     0, s, b);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

// ---- residual frames: the links of a frame's site sets to the saved ones, all scales at once ------
struct IncreLinkJob {
  const Slot *pre_table;
  int64_t pre_mask;
  const int32_t *coords, *d_n, *parent;
  int32_t *pre_exist, *nbr_pre, *parent2;
};
struct IncreLinkBatch {
  IncreLinkJob job[16];
};
// pre_exist (insc_grid_query of the saved grid with the scale's own coordinates) and, for the sites the
// saved grid does not hold, their neighbours there (incre_ssc3_nbr_kernel).  Thread = (site, offset);
// every thread looks its own site up, the one of the centre offset records the answer.
__global__ void incre_links_batch_kernel(IncreLinkBatch b) {
  const IncreLinkJob &j = b.job[blockIdx.y];
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= (int64_t)j.d_n[0] * 27) return;
  const int64_t o = t / 27;
  const int k = (int)(t % 27);
  const int4 c = reinterpret_cast<const int4 *>(j.coords)[o];
  const int pe = grid_find(j.pre_table, j.pre_mask, pack_key(c.x, c.y, c.z, c.w));
  if (k == 13) j.pre_exist[o] = pe;
  int r = -1;
  if (pe < 0 && k != 13) {
    const int x = c.x + k / 9 - 1, y = c.y + (k / 3) % 3 - 1, z = c.z + k % 3 - 1;
    if (coord_ok(x, y, z, c.w)) r = grid_find(j.pre_table, j.pre_mask, pack_key(x, y, z, c.w));
  }
  j.nbr_pre[t] = r;
}
// the saved coarse row that a fine site new to the saved set also reads (incre_parent_kernel); job l
// holds the fine scale's parent map and answer, job l + 1 the coarse scale
__global__ void incre_parents_batch_kernel(IncreLinkBatch b) {
  const IncreLinkJob &f = b.job[blockIdx.y], &cs = b.job[blockIdx.y + 1];
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= f.d_n[0]) return;
  const int p = f.parent[i];
  f.parent2[i] = (p >= 0 && p < cs.d_n[0] && f.pre_exist[i] < 0) ? cs.pre_exist[p] : -1;
}

int incre_links_batch(const insc_grid *const *grids, const insc_grid *const *pre, const int32_t *const *d_parent,
                      int32_t *const *d_pre_exist, int32_t *const *d_nbr_pre, int32_t *const *d_parent2, int n,
                      int64_t n_upper, hipStream_t s) {
  if (n <= 0 || n_upper <= 0) return INSC_OK;
  if (n > 16) {
    set_error("incre_links_batch: at most 16 grids");
    return INSC_ERR_ARG;
  }
  IncreLinkBatch b;
  for (int i = 0; i < n; i++)
    b.job[i] = IncreLinkJob{pre[i]->table, pre[i]->n_slots - 1, grids[i]->coords, grids[i]->d_n,
                            i + 1 < n ? d_parent[i] : nullptr, d_pre_exist[i], d_nbr_pre[i],
                            i + 1 < n ? d_parent2[i] : nullptr};
  hipLaunchKernelGGL(incre_links_batch_kernel, dim3(grid_for(n_upper * 27, 256, 1ll << 30), (unsigned)n), dim3(256), 0,
                     s, b);
  if (n > 1)
    hipLaunchKernelGGL(incre_parents_batch_kernel, dim3(grid_for(n_upper, 256), (unsigned)(n - 1)), dim3(256), 0, s, b);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int order_append_new_sites_both_batch(const insc_grid *const *grids, const int32_t *const *d_nbr,
                                      const int32_t *const *d_offset, int32_t *const *d_order, int32_t *const *d_pos,
                                      int32_t *const *d_bo_order, int32_t *const *d_bo_pos, int n, int64_t n_new_upper,
                                      hipStream_t s, bool all) {
  if (n <= 0 || n_new_upper <= 0) return INSC_OK;
  if (n > 16) {
    set_error("order_append_new_sites_both_batch: at most 16 grids");
    return INSC_ERR_ARG;
  }
  OrderBothBatch b;
  for (int i = 0; i < n; i++)
    b.job[i] = OrderBothJob{grids[i]->d_n, grids[i]->coords, d_nbr[i], d_offset[i], d_order[i], d_pos[i], d_bo_order[i], d_bo_pos[i], all ? 1 : 0};
  hipLaunchKernelGGL(order_append_both_batch_kernel, dim3((unsigned)n), dim3(1024), 0, s, b);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_grid_create(int64_t capacity_sites, insc_grid **out) {
  INSC_REQUIRE(out, INSC_ERR_ARG, "insc_grid_create: out is null");
  INSC_REQUIRE(capacity_sites >= 0 && capacity_sites < (1ll << 30), INSC_ERR_ARG,
               "insc_grid_create: capacity %lld out of range", (long long)capacity_sites);
  if (capacity_sites < 1024) capacity_sites = 1024;
  insc_grid *g = new insc_grid();
  INSC_HIP(hipGetDevice(&g->device));
  g->capacity_sites = capacity_sites;
  int rc = grid_alloc_table(g, capacity_sites);
  if (rc) {
    delete g;
    return rc;
  }
  INSC_HIP(hipMalloc((void **)&g->coords, sizeof(int32_t) * 4 * (size_t)capacity_sites));
  INSC_HIP(hipMalloc((void **)&g->d_n, 256));
  g->d_err = g->d_n + 16;
  INSC_HIP(hipHostMalloc((void **)&g->h_n, 64, hipHostMallocDefault));
  g->h_n[0] = g->h_n[1] = 0;
  INSC_HIP(hipMalloc((void **)&g->part, sizeof(int32_t) * PART_INTS));
  INSC_HIP(hipMemset(g->part, 0, sizeof(int32_t) * PART_INTS));
  *out = g;
  return insc_grid_clear(g, nullptr);
}

int insc_grid_destroy(insc_grid *g) {
  if (!g) return INSC_OK;
  (void)hipDeviceSynchronize();
  if (g->table) (void)hipFree(g->table);
  if (g->coords) (void)hipFree(g->coords);
  if (g->d_n) (void)hipFree(g->d_n);
  if (g->h_n) (void)hipHostFree(g->h_n);
  if (g->slot_of_point) (void)hipFree(g->slot_of_point);
  if (g->flags) (void)hipFree(g->flags);
  if (g->part) (void)hipFree(g->part);
  delete g;
  return INSC_OK;
}

int insc_grid_clear(insc_grid *g, void *stream) {
  INSC_REQUIRE(g, INSC_ERR_ARG, "insc_grid_clear: grid is null");
  hipLaunchKernelGGL(grid_clear_kernel, dim3(grid_for(g->n_slots, 256, 8192)), dim3(256), 0, (hipStream_t)stream,
                     g->table, g->n_slots, g->d_n, g->d_err);
  INSC_LAUNCH_CHECK();
  g->n_upper = 0;
  g->n_exact = 0;
  g->h_fresh = false;
  return INSC_OK;
}

int insc_grid_reserve(insc_grid *g, int64_t capacity_sites, void *stream) {
  INSC_REQUIRE(g, INSC_ERR_ARG, "insc_grid_reserve: grid is null");
  INSC_REQUIRE(capacity_sites < (1ll << 30), INSC_ERR_ARG, "insc_grid_reserve: capacity out of range");
  if (capacity_sites <= g->capacity_sites) return INSC_OK;
  hipStream_t s = (hipStream_t)stream;
  INSC_HIP(hipStreamSynchronize(s));
  g->h_fresh = false;
  int32_t *coords = nullptr;
  INSC_HIP(hipMalloc((void **)&coords, sizeof(int32_t) * 4 * (size_t)capacity_sites));
  INSC_HIP(hipMemcpyAsync(coords, g->coords, sizeof(int32_t) * 4 * (size_t)g->capacity_sites,
                          hipMemcpyDeviceToDevice, s));
  INSC_HIP(hipStreamSynchronize(s));
  INSC_HIP(hipFree(g->coords));
  g->coords = coords;
  g->capacity_sites = capacity_sites;
  if (g->n_slots < 2 * capacity_sites) {
    INSC_HIP(hipFree(g->table));
    g->table = nullptr;
    int rc = grid_alloc_table(g, capacity_sites);
    if (rc) return rc;
    // clear the new table but keep the counter
    int32_t n_keep = 0;
    INSC_HIP(hipMemcpy(&n_keep, g->d_n, sizeof(int32_t), hipMemcpyDeviceToHost));
    hipLaunchKernelGGL(grid_clear_kernel, dim3(grid_for(g->n_slots, 256, 8192)), dim3(256), 0, s, g->table,
                       g->n_slots, g->d_n, g->d_err);
    INSC_HIP(hipMemcpyAsync(g->d_n, &n_keep, sizeof(int32_t), hipMemcpyHostToDevice, s));
    INSC_HIP(hipStreamSynchronize(s));
    if (n_keep > 0) {
      hipLaunchKernelGGL(grid_rehash_kernel, dim3(grid_for(n_keep, 256)), dim3(256), 0, s, g->table,
                         g->n_slots - 1, g->coords, g->d_n, g->d_err);
      INSC_LAUNCH_CHECK();
    }
    return grid_sync_errors(g, s, "insc_grid_reserve");
  }
  return INSC_OK;
}

int insc_grid_insert(insc_grid *g, const int32_t *d_coords4, int64_t P, int32_t *d_site_of_point, int64_t *h_n_sites,
                     void *stream) {
  INSC_REQUIRE(g, INSC_ERR_ARG, "insc_grid_insert: grid is null");
  INSC_REQUIRE(P >= 0 && P < VAL_PENDING - 1, INSC_ERR_ARG, "insc_grid_insert: P=%lld out of range", (long long)P);
  INSC_REQUIRE(P == 0 || (d_coords4 && d_site_of_point), INSC_ERR_ARG, "insc_grid_insert: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (P > 0) {
    if (g->n_upper + P > g->capacity_sites) {
      // the bound may be loose (duplicates): refresh it before growing
      int rc = grid_sync_errors(g, s, "insc_grid_insert");
      if (rc) return rc;
      if (g->n_upper + P > g->capacity_sites) {
        int64_t want = g->capacity_sites * 2;
        if (want < g->n_upper + P) want = g->n_upper + P;
        rc = insc_grid_reserve(g, want, stream);
        if (rc) return rc;
      }
    }
    int rc = grid_insert_launch(g, d_coords4, P, d_site_of_point, s);
    if (rc) return rc;
  }
  if (h_n_sites) {
    int rc = grid_sync_errors(g, s, "insc_grid_insert");
    if (rc) return rc;
    *h_n_sites = g->n_exact;
  }
  return INSC_OK;
}

int insc_grid_insert_noalloc(insc_grid *g, const int32_t *d_coords4, int64_t P, int32_t *d_site_of_point,
                             int64_t *h_n_sites, void *stream) {
  INSC_REQUIRE(g, INSC_ERR_ARG, "insc_grid_insert_noalloc: grid is null");
  INSC_REQUIRE(P >= 0, INSC_ERR_ARG, "insc_grid_insert_noalloc: P=%lld is negative", (long long)P);
  INSC_REQUIRE(P <= NOALLOC_MAX_POINTS, INSC_ERR_CAPACITY,
               "insc_grid_insert_noalloc: %lld points exceed the %d one call takes (split the list, or use "
               "insc_grid_insert, which may allocate)",
               (long long)P, NOALLOC_MAX_POINTS);
  INSC_REQUIRE(P == 0 || (d_coords4 && d_site_of_point), INSC_ERR_ARG, "insc_grid_insert_noalloc: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (P > 0) {
    int dev = -1;
    INSC_HIP(hipGetDevice(&dev));
    INSC_REQUIRE(dev == g->device, INSC_ERR_STATE, "insc_grid_insert_noalloc: the grid lives on device %d, current is %d",
                 g->device, dev);
    int32_t *slot_of_point = nullptr;
    int rc = scratch_on_current_device(&slot_of_point);
    if (rc) return rc;
    // this entry point never grows the grid: the host-side bound (every row a new site) must fit
    INSC_REQUIRE(g->n_upper + P <= g->capacity_sites, INSC_ERR_CAPACITY,
                 "insc_grid_insert_noalloc: up to %lld sites + %lld points may exceed the capacity of %lld; call "
                 "insc_grid_reserve first (or insc_grid_size to tighten the bound after inserts with repeats)",
                 (long long)g->n_upper, (long long)P, (long long)g->capacity_sites);
    hipLaunchKernelGGL(grid_claim_kernel, dim3(grid_for(P, 256)), dim3(256), 0, s, g->table, g->n_slots - 1, d_coords4,
                       P, slot_of_point, (int32_t *)nullptr, d_site_of_point, g->d_err);
    hipLaunchKernelGGL(grid_finish_small_kernel, dim3(1), dim3(1024), 0, s, g->table, d_coords4, slot_of_point, (int)P,
                       g->d_n, g->coords, g->capacity_sites, g->d_err, d_site_of_point, g->h_n);
    INSC_LAUNCH_CHECK();
    g->n_upper += P;
    g->n_exact = -1;
    g->h_fresh = g->h_n != nullptr;
    g->h_stream = (void *)s;
  }
  if (h_n_sites) {
    int rc = grid_sync_errors(g, s, "insc_grid_insert_noalloc");
    if (rc) return rc;
    *h_n_sites = g->n_exact;
  }
  return INSC_OK;
}

int insc_order_append(const insc_grid *g, const int32_t *d_nbr, const int32_t *d_offset, int32_t *d_order, int32_t *d_pos,
                      int32_t *d_bo_order, int32_t *d_bo_pos, int64_t n_new_upper, void *stream) {
  INSC_REQUIRE(g && d_nbr && d_order, INSC_ERR_ARG, "insc_order_append: null argument");
  INSC_REQUIRE(!d_offset || (d_bo_order && d_bo_pos), INSC_ERR_ARG,
               "insc_order_append: with d_offset, d_bo_order and d_bo_pos are needed as well");
  const insc_grid *gs[1] = {g};
  const int32_t *nbr[1] = {d_nbr}, *off[1] = {d_offset};
  int32_t *order[1] = {d_order}, *pos[1] = {d_pos}, *bo[1] = {d_bo_order}, *bop[1] = {d_bo_pos};
  return order_append_new_sites_both_batch(gs, nbr, off, order, pos, bo, bop, 1, n_new_upper, (hipStream_t)stream);
}

int insc_grid_query(const insc_grid *g, const int32_t *d_coords4, int64_t Q, int32_t *d_site, void *stream) {
  INSC_REQUIRE(g, INSC_ERR_ARG, "insc_grid_query: grid is null");
  INSC_REQUIRE(Q >= 0 && (Q == 0 || (d_coords4 && d_site)), INSC_ERR_ARG, "insc_grid_query: bad arguments");
  if (Q == 0) return INSC_OK;
  hipLaunchKernelGGL(grid_query_kernel, dim3(grid_for(Q, 256)), dim3(256), 0, (hipStream_t)stream, g->table,
                     g->n_slots - 1, d_coords4, Q, d_site);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_grid_size(insc_grid *g, int64_t *h_n_sites, void *stream) {
  INSC_REQUIRE(g && h_n_sites, INSC_ERR_ARG, "insc_grid_size: null argument");
  if (g->n_exact < 0) {
    int rc = grid_sync_errors(g, (hipStream_t)stream, "insc_grid_size");
    if (rc) return rc;
  }
  *h_n_sites = g->n_exact;
  return INSC_OK;
}

const int32_t *insc_grid_coords(const insc_grid *g) { return g ? g->coords : nullptr; }
const int32_t *insc_grid_count_ptr(const insc_grid *g) { return g ? g->d_n : nullptr; }
int64_t insc_grid_capacity(const insc_grid *g) { return g ? g->capacity_sites : 0; }

int insc_rulebook_ssc3(const insc_grid *g, int64_t first, int64_t n, int32_t *d_nbr, int patch_reverse,
                       void *stream) {
  INSC_REQUIRE(g, INSC_ERR_ARG, "insc_rulebook_ssc3: grid is null");
  INSC_REQUIRE(first >= 0 && n >= 0 && first + n <= g->capacity_sites, INSC_ERR_ARG,
               "insc_rulebook_ssc3: rows [%lld,%lld) outside capacity %lld", (long long)first,
               (long long)(first + n), (long long)g->capacity_sites);
  INSC_REQUIRE(n == 0 || d_nbr, INSC_ERR_ARG, "insc_rulebook_ssc3: d_nbr is null");
  if (n == 0) return INSC_OK;
  if (first == 0 && n == g->n_exact) {
    // every site of the grid: rows to -1, then half the probes (each found pair fills two entries)
    int rc = insc_fill_i32(d_nbr, n * 27, -1, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(ssc3_nbr_sym_kernel, dim3(grid_for(n * 14, 256, 1ll << 30)), dim3(256), 0, (hipStream_t)stream,
                       g->table, g->n_slots - 1, g->coords, n, d_nbr);
    INSC_LAUNCH_CHECK();
    return INSC_OK;
  }
  hipLaunchKernelGGL(ssc3_nbr_kernel, dim3(grid_for(n * 27, 256, 1ll << 30)), dim3(256), 0, (hipStream_t)stream,
                     g->table, g->n_slots - 1, g->coords, first, n, d_nbr, patch_reverse);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_incre_rulebook_ssc3(const insc_grid *g, const insc_grid *pre, const int32_t *d_pre_exist, int64_t n,
                             int32_t *d_nbr_pre, void *stream) {
  INSC_REQUIRE(g && pre && g != pre, INSC_ERR_ARG, "insc_incre_rulebook_ssc3: needs two different grids");
  INSC_REQUIRE(n >= 0 && n <= g->capacity_sites, INSC_ERR_ARG, "insc_incre_rulebook_ssc3: n outside capacity");
  INSC_REQUIRE(n == 0 || (d_pre_exist && d_nbr_pre), INSC_ERR_ARG, "insc_incre_rulebook_ssc3: null pointer");
  if (n == 0) return INSC_OK;
  hipLaunchKernelGGL(incre_ssc3_nbr_kernel, dim3(grid_for(n * 27, 256, 1ll << 30)), dim3(256), 0, (hipStream_t)stream,
                     pre->table, pre->n_slots - 1, g->coords, d_pre_exist, n, d_nbr_pre);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_rulebook_down2(const insc_grid *fine, insc_grid *coarse, int64_t first, int64_t n, int32_t *d_parent,
                        int32_t *d_offset, int32_t *d_child, int64_t child_rows, void *stream) {
  INSC_REQUIRE(fine && coarse && fine != coarse, INSC_ERR_ARG, "insc_rulebook_down2: bad grids");
  INSC_REQUIRE(first >= 0 && n >= 0 && first + n <= fine->capacity_sites, INSC_ERR_ARG,
               "insc_rulebook_down2: rows outside capacity");
  INSC_REQUIRE(n == 0 || (d_parent && d_offset), INSC_ERR_ARG, "insc_rulebook_down2: null pointer");
  if (n == 0) return INSC_OK;
  hipStream_t s = (hipStream_t)stream;
  void *ws;
  int rc = workspace(WS_API, s, sizeof(int32_t) * 4 * (size_t)n, &ws);
  if (rc) return rc;
  int32_t *half = (int32_t *)ws;
  hipLaunchKernelGGL(down2_coords_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, fine->coords, first, n, half,
                     d_offset);
  INSC_LAUNCH_CHECK();
  rc = insc_grid_insert(coarse, half, n, d_parent + first, nullptr, stream);
  if (rc) return rc;
  if (d_child) {
    INSC_REQUIRE(child_rows >= coarse->capacity_sites, INSC_ERR_CAPACITY,
                 "insc_rulebook_down2: child map has %lld rows, coarse grid capacity is %lld", (long long)child_rows,
                 (long long)coarse->capacity_sites);
    hipLaunchKernelGGL(down2_child_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, d_parent, d_offset, first, n,
                       d_child);
    INSC_LAUNCH_CHECK();
  }
  return INSC_OK;
}

int insc_grid_insert_scales(insc_grid *const *grids, int32_t *const *d_parent, int32_t *const *d_offset,
                            int32_t *const *d_child, int n_scales, const int32_t *d_coords, int coord_cols, int64_t P,
                            int32_t *d_site_of_point, int64_t *h_n_sites, void *stream) {
  INSC_REQUIRE(grids && n_scales >= 1 && n_scales <= 16, INSC_ERR_ARG, "insc_grid_insert_scales: 1..16 scales");
  INSC_REQUIRE(P >= 0 && (coord_cols == 3 || coord_cols == 4), INSC_ERR_ARG, "insc_grid_insert_scales: bad arguments");
  INSC_REQUIRE(P == 0 || (d_coords && d_site_of_point), INSC_ERR_ARG, "insc_grid_insert_scales: null pointer");
  INSC_REQUIRE(n_scales == 1 || (d_parent && d_offset && d_child), INSC_ERR_ARG,
               "insc_grid_insert_scales: the link arrays are missing");
  hipStream_t s = (hipStream_t)stream;
  FrameInsertLevel lv[16];
  for (int l = 0; l < n_scales; l++) {
    INSC_REQUIRE(grids[l], INSC_ERR_ARG, "insc_grid_insert_scales: grid %d is null", l);
    for (int k = 0; k < l; k++) INSC_REQUIRE(grids[k] != grids[l], INSC_ERR_ARG, "insc_grid_insert_scales: grid %d given twice", l);
    const bool link = l + 1 < n_scales;
    INSC_REQUIRE(!link || (d_parent[l] && d_offset[l] && d_child[l]), INSC_ERR_ARG,
                 "insc_grid_insert_scales: link arrays of scale %d are null", l);
    lv[l] = FrameInsertLevel{grids[l], link ? d_parent[l] : nullptr, link ? d_offset[l] : nullptr, link ? d_child[l] : nullptr};
  }
  if (P > 0) {
    // the flag "some coordinate is bad" and the counts the kernels leave: 2 * scales + 2 words
    void *ws;
    int rc = workspace(WS_INSERT, s, 64 * sizeof(int32_t), &ws);
    if (rc) return rc;
    int32_t *d_bad = (int32_t *)ws, *d_counts = d_bad + 1;
    INSC_HIP(hipMemsetAsync(d_bad, 0, sizeof(int32_t), s));
    if ((rc = frame_insert_levels(lv, n_scales, d_coords, coord_cols, P, d_bad, 1, d_site_of_point, d_counts, s))) return rc;
    int32_t dropped = 0;
    INSC_HIP(hipMemcpyAsync(&dropped, d_counts + 2 * n_scales, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    INSC_HIP(hipStreamSynchronize(s));
    // the exact counts, and the capacity flag of every scale (reported once, then cleared)
    int first_err = INSC_OK;
    for (int l = 0; l < n_scales; l++) {
      rc = grid_sync_errors(grids[l], s, "insc_grid_insert_scales");
      if (rc && !first_err) first_err = rc;
    }
    INSC_REQUIRE(dropped != 1, INSC_ERR_COORD,
                 "insc_grid_insert_scales: a coordinate is outside 0..65535 (batch 0..32767); nothing was inserted");
    if (first_err) return first_err;
  }
  if (h_n_sites)
    for (int l = 0; l < n_scales; l++) {
      int64_t n = 0;
      int rc = insc_grid_size(grids[l], &n, stream);
      if (rc) return rc;
      h_n_sites[l] = n;
    }
  return INSC_OK;
}

}  // extern "C"
