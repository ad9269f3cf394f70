// Network executor: runs a whole sparse U-Net style network, full or incremental, from one
// host call.  It owns the per-scale hash grids, rulebooks, cached feature matrices and the
// dirty-set bookkeeping, and enqueues every kernel of a frame back to back on one stream with
// one host round trip per incremental frame (the site counts, read back once the grids are updated).
//
// The reference keeps this state spread over Python module attributes (save_meta,
// save_input_feats, save_output: sparseconvnet/submanifoldConvolution.py:53-54,
// batchNormalization.py:60-61, ioLayers.py:69,106-107) and a Metadata object per frame
// (Metadata/Metadata.h:218-386); here it is one object with an explicit program.
#include <algorithm>
#include <map>
#include <set>
#include <vector>

#include "common.h"
#include "grid.h"

namespace insc {

enum OpKind { OP_SSC, OP_BN, OP_CONV, OP_DECONV, OP_NIN, OP_ADD, OP_COPY, OP_JOIN };
enum DirtyKind { D_INPUT, D_DILATE, D_PARENTS, D_CHILDREN, D_UNION };
// Scales this small are recomputed whole by incremental frames: the input scale up to 128 tiles, the
// coarser ones up to 512.  (Every launch then has all its tiles resident at once - what it lasts is its
// longest block, not the number of blocks - and with the eight 3^3 layers of such a scale and of each
// coarser one a change anywhere reaches nearly every site of it anyway: in the 150k-voxel sweep the sets
// of the 10k-site scale hold 10 405 to 10 414 of its 10 414 sites.  No set is computed for such a scale:
// 1 % of the frame.  The input scale keeps the lower bound: its sets start at the frame's own voxels.)
constexpr int64_t DIRTY_FULL_SITES = 4096;
constexpr int64_t DIRTY_FULL_SITES_COARSE = 16384;
// Scales from this size on may run a layer over a list of dirty rows instead of over flagged tiles.
constexpr int64_t COMPACT_MIN_SITES = 32768;

struct Level {
  insc_grid *grid = nullptr;
  int64_t cap = 0;
  int32_t *nbr = nullptr;       // [cap,27]
  int32_t *order = nullptr;     // [cap] processing order of the 3^3 convolutions
  int32_t *pos = nullptr;       // [cap] inverse of order
  int32_t *plan = nullptr;      // [27,cap] tile plan of the 3^3 map in processing order
  uint32_t *tmask = nullptr;    // [cap/32] offsets used per tile
  int32_t *sched = nullptr;     // [cap/32] tiles by falling number of offsets used
  int32_t *parent = nullptr;    // [cap] site at the next coarser level
  int32_t *offset = nullptr;    // [cap] position inside the parent cell
  int32_t *child = nullptr;     // [cap_coarse,8] (owned by the FINE level's link)
  int64_t child_rows = 0;
  int32_t *bo_order = nullptr;  // [cap] fine sites grouped by offset (deconvolution order)
  int32_t *bo_pos = nullptr;    // [cap]
  int64_t n = 0;                // exact count after the last completed frame
  int64_t n_upper = 0;          // bound valid during the frame being enqueued
  int64_t new_upper = 0;        // bound on sites added in this frame
  bool plan_valid = false;      // the tile plan holds every site of the last completed frame
  int64_t n_sorted = 0;         // sites that the last order built from scratch covers (later ones are appended)
};

struct Buffer {
  int level = 0;
  int ld = 0;
  float *p = nullptr;
  int64_t rows = 0;
};

struct Tensor {
  int level = 0, C = 0, buf = -1, col0 = 0, dirty = -1;
  bool kept = true;  // false: nothing reads it any more (its batch norm moved into its producer)
};

struct Op {
  int kind = 0, in0 = -1, in1 = -1, out = -1;
  const float *W = nullptr, *bias = nullptr, *mean = nullptr, *var = nullptr, *gamma = nullptr, *beta = nullptr;
  float *Wp = nullptr;  // packed weights, owned
  float eps = 0, leak = 0;
  int Cin = 0, Cout = 0;
  // batch norm folded into the kernel that produces its input
  float *bn_w = nullptr, *bn_b = nullptr;  // per-channel scale / shift of an OP_BN, owned
  int fused_add = -1;                      // convolution side: index of the OP_ADD it also computes
  int fused_bn = -1;                       // producer side: index of the OP_BN it also computes
  int fused_join_bn = -1;                  // deconvolution side: OP_BN over a join of its output with another tensor
  int join_other = -1;                     //   ... that other tensor
  bool write_raw = true;                   // producer side: its own output has other readers
  bool fused = false;                      // OP_BN / OP_ADD side: computed by its producer, no kernel of its own
};

struct DirtyNode {
  int kind = 0, level = 0, src0 = -1, src1 = -1;
  bool tiles_by_offset = false;  // tile flags follow the deconvolution order
  uint8_t *mask = nullptr;       // [cap] one byte per site
  uint8_t *tflag = nullptr;      // [cap/32+1] one byte per 32-row tile of the level's order
  uint8_t *tflag_bo = nullptr;   // same for the by-offset order (only if some deconvolution needs it)
  std::set<int> ancestors;
  // A set that stays small against its scale is also kept as a list of its rows (in processing
  // order), so that a layer works on tiles made of dirty rows only instead of on every tile that
  // holds one: depth = 3^3 layers between the frame's points and this set at the input scale (-1:
  // the set does not qualify), crows / ccount = the list and its length (ccount lies in the mask
  // arena and is zero when a frame starts), compact = this frame uses the list.
  int depth = -1;
  int32_t *crows = nullptr;
  int32_t *ccount = nullptr;
  int64_t crows_cap = 0;
  bool compact = false;
  int64_t expect_rows = 0;  // estimate of the set's size in this frame
};

}  // namespace insc

namespace insc {
// Everything a residual frame needs besides the saved state: the frame's own site set (fresh
// grids and maps at every scale), its links to the saved one, and feature matrices sized for
// the frame.  Built anew by every residual frame; nothing in it outlives the frame.
struct ResidualFrame {
  std::vector<Level> levels;            // grid, nbr, parent, offset, child of the frame's sites
  std::vector<int32_t *> pre_exist;     // [cap] id in the saved site set of the scale, or -1
  std::vector<int32_t *> nbr_pre;       // [cap,27] saved neighbours of the sites new to the saved set
  std::vector<int32_t *> parent2;       // [cap] saved row of the coarse parent of such a site (scales with a coarser one)
  std::vector<Buffer> buffers;          // same layout as the program's buffers, rows = sites of the frame
  std::vector<int> ld;                  // row stride of every buffer (0: unused)
  int64_t cap = 0;                      // sites every scale can hold
  float *in_sum = nullptr;
  int32_t *in_cnt = nullptr, *chain_head = nullptr, *chain_next = nullptr, *sop = nullptr;
  std::vector<uint8_t> bn_done;         // per op, this frame: a batch norm that its producer has computed
};
}  // namespace insc

struct insc_net {
  int n_levels = 0, in_channels = 0, mode = 4;
  bool finalized = false, have_state = false;
  bool last_inc = false;  // the last completed frame was an incremental one (its dirty flags are still in place)
  bool keep_raw = false;  // keep the input of every batch norm (residual frames read it)
  int order_refresh_pct = 10;  // an incremental frame re-sorts the orders once this share of a large scale is appended (0: never)
  insc::ResidualFrame rf;
  std::vector<insc::Level> levels;
  std::vector<insc::Buffer> buffers;
  std::vector<insc::Tensor> tensors;
  std::vector<insc::Op> ops;
  std::vector<insc::DirtyNode> dirty;
  std::map<std::vector<int>, int> dirty_index;
  // input layer state
  float *in_sum = nullptr;
  int32_t *in_cnt = nullptr;
  int32_t *chain_head = nullptr;  // [cap0] per-site list head, -1 when idle
  int32_t *chain_next = nullptr;  // [points_cap]
  int32_t *site_of_point = nullptr;  // all points since the last full frame
  int64_t points_cap = 0, n_points = 0, n_points_frame = 0;
  uint8_t *mask_arena = nullptr;
  size_t mask_arena_bytes = 0;
  std::vector<uint8_t> dirty_full;      // per set, last incremental frame: known to hold every row (no mask kept)
  int32_t *h_counts = nullptr;  // pinned: per level count, error flags
  int32_t *d_bad = nullptr;     // number of the last frame that held a coordinate out of range
  int32_t frame_id = 0;         // frames are numbered from 1
  const int32_t *frame_sop = nullptr;  // site of every point of the frame being enqueued
  int64_t frame_P = 0;
  int out_tensor = -1;
  bool profiling = false;
  hipEvent_t ev[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
  bool ev_valid = false;
  hipEvent_t ev_counts = nullptr;  // the frame's inserts are done: the site counts lie in h_counts
};

namespace insc {

// -----------------------------------------------------------------------------------------
// kernels private to the executor
// -----------------------------------------------------------------------------------------
__global__ void invert_perm_kernel(const int32_t *__restrict__ order, int64_t n, int32_t *__restrict__ pos) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) pos[order[t]] = (int)t;
}

// Input layer, step 1: thread p pushes itself on the list of its site.
__global__ void chain_push_kernel(const int32_t *__restrict__ sop, int64_t P, int32_t *__restrict__ head,
                                  int32_t *__restrict__ next) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int s = sop[p];
  next[p] = (s >= 0) ? atomicExch(&head[s], (int)p) : -1;
}

// Input layer, step 2: the row left at the head of a site's list owns the site.  It adds the
// rows of the list to the running sum in ascending row order (the order InputLayer_fp_ visits
// them, CUDA/IOLayers.cu:17-32) and resets the head.  Lists are short (rows of one voxel in one
// frame); each pass picks the smallest row index not yet added.
__global__ void chain_sum_kernel(const float *__restrict__ feats, int C, const int32_t *__restrict__ sop, int64_t P,
                                 int32_t *__restrict__ head, const int32_t *__restrict__ next,
                                 float *__restrict__ sum, int32_t *__restrict__ cnt, uint8_t *__restrict__ mask,
                                 uint8_t *__restrict__ tflag, const int32_t *__restrict__ pos) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int s = sop[p];
  if (s < 0 || head[s] != (int)p) return;
  int done = -1, n = 0;
  for (;;) {
    int best = 0x7fffffff;
    for (int q = (int)p; q >= 0; q = next[q])
      if (q > done && q < best) best = q;
    if (best == 0x7fffffff) break;
    for (int c = 0; c < C; c++) sum[(int64_t)s * C + c] += feats[(int64_t)best * C + c];
    done = best;
    n++;
  }
  cnt[s] += n;
  head[s] = -1;
  if (mask) {
    mask[s] = 1;
    tflag[pos[s] >> 5] = 1;
  }
}

__global__ void dirty_dilate_kernel(const int32_t *__restrict__ nbr, const uint8_t *__restrict__ mask_in,
                                    uint8_t *__restrict__ mask_out, uint8_t *__restrict__ tflag,
                                    const int32_t *__restrict__ pos, uint8_t *__restrict__ tflag_bo,
                                    const int32_t *__restrict__ bo_pos, const int32_t *__restrict__ d_n,
                                    int64_t n_upper) {
  const int64_t n = min((int64_t)*d_n, n_upper);
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * 27) return;
  if (!mask_in[t / 27]) return;
  const int j = nbr[t];
  if (j < 0) return;
  mask_out[j] = 1;
  tflag[pos[j] >> 5] = 1;
  if (tflag_bo) tflag_bo[bo_pos[j] >> 5] = 1;
}

// the same from a list of the source set's rows (a short list beats a pass over every site of the
// scale); entries may repeat, -1 is skipped
__global__ void dirty_dilate_list_kernel(const int32_t *__restrict__ nbr, const int32_t *__restrict__ rows,
                                         const int32_t *__restrict__ d_count, int64_t n_fixed,
                                         uint8_t *__restrict__ mask_out, uint8_t *__restrict__ tflag,
                                         const int32_t *__restrict__ pos, uint8_t *__restrict__ tflag_bo,
                                         const int32_t *__restrict__ bo_pos) {
  const int64_t n = d_count ? (int64_t)*d_count : n_fixed;
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n * 27; t += (int64_t)gridDim.x * blockDim.x) {
    const int r = rows[t / 27];
    if (r < 0) continue;
    const int j = nbr[(int64_t)r * 27 + t % 27];
    if (j < 0) continue;
    mask_out[j] = 1;
    tflag[pos[j] >> 5] = 1;
    if (tflag_bo) tflag_bo[bo_pos[j] >> 5] = 1;
  }
}

__global__ void dirty_parents_kernel(const int32_t *__restrict__ parent, const uint8_t *__restrict__ mask_fine,
                                     uint8_t *__restrict__ mask_out, uint8_t *__restrict__ tflag,
                                     const int32_t *__restrict__ pos, const int32_t *__restrict__ d_n_fine,
                                     int64_t n_upper) {
  const int64_t n = min((int64_t)*d_n_fine, n_upper);
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n || !mask_fine[i]) return;
  const int j = parent[i];
  if (j < 0) return;
  mask_out[j] = 1;
  tflag[pos[j] >> 5] = 1;
}

__global__ void dirty_children_kernel(const int32_t *__restrict__ parent, const uint8_t *__restrict__ mask_coarse,
                                      uint8_t *__restrict__ mask_out, uint8_t *__restrict__ tflag,
                                      const int32_t *__restrict__ pos, uint8_t *__restrict__ tflag_bo,
                                      const int32_t *__restrict__ bo_pos, const int32_t *__restrict__ d_n_fine,
                                      int64_t n_upper) {
  const int64_t n = min((int64_t)*d_n_fine, n_upper);
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int j = parent[i];
  if (j < 0 || !mask_coarse[j]) return;
  mask_out[i] = 1;
  tflag[pos[i] >> 5] = 1;
  if (tflag_bo) tflag_bo[bo_pos[i] >> 5] = 1;
}

__global__ void dirty_union_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                   uint8_t *__restrict__ mask_out, uint8_t *__restrict__ tflag,
                                   const int32_t *__restrict__ pos, uint8_t *__restrict__ tflag_bo,
                                   const int32_t *__restrict__ bo_pos, const int32_t *__restrict__ d_n,
                                   int64_t n_upper) {
  const int64_t n = min((int64_t)*d_n, n_upper);
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n || !(a[i] | b[i])) return;
  mask_out[i] = 1;
  tflag[pos[i] >> 5] = 1;
  if (tflag_bo) tflag_bo[bo_pos[i] >> 5] = 1;
}

// rows = the sites of the processing order whose mask byte is set.  A block compacts a run of
// 1024 positions, keeping their order, and claims room for them with one atomic: the runs come out
// in any order (no result depends on the order of a row list).  *count must be zero beforehand.
__global__ __launch_bounds__(256) void dirty_compact_rows_kernel(const uint8_t *__restrict__ mask,
                                                                 const int32_t *__restrict__ order,
                                                                 const int32_t *__restrict__ d_n, int64_t n_upper,
                                                                 int32_t *__restrict__ rows, int32_t *count) {
  __shared__ int wave_total[4];
  __shared__ int base_s;
  const int64_t n = min((int64_t)*d_n, n_upper);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t p0 = (int64_t)blockIdx.x * 1024 + tid * 4;
  int site[4], cnt = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    site[j] = p0 + j < n ? order[p0 + j] : -1;
    if (site[j] >= 0 && !mask[site[j]]) site[j] = -1;
    cnt += site[j] >= 0 ? 1 : 0;
  }
  int incl = cnt;
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_up(incl, d, 64);
    if (lane >= d) incl += v;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  int before = incl - cnt, total = 0;
  for (int w = 0; w < 4; w++) {
    if (w < wave) before += wave_total[w];
    total += wave_total[w];
  }
  if (tid == 0) base_s = total ? atomicAdd(count, total) : 0;
  __syncthreads();
  int at = base_s + before;
#pragma unroll
  for (int j = 0; j < 4; j++)
    if (site[j] >= 0) rows[at++] = site[j];
}

// dirty rows of one set: one count per block, added up with an atomic per block
__global__ __launch_bounds__(256) void count_mask_kernel(const uint8_t *__restrict__ mask, int64_t n,
                                                         unsigned long long *__restrict__ out) {
  __shared__ int part[256];
  int c = 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) c += mask[i] ? 1 : 0;
  part[threadIdx.x] = c;
  __syncthreads();
  for (int d = 128; d > 0; d >>= 1) {
    if ((int)threadIdx.x < d) part[threadIdx.x] += part[threadIdx.x + d];
    __syncthreads();
  }
  if (threadIdx.x == 0 && part[0]) atomicAdd(out, (unsigned long long)part[0]);
}

__global__ void fill_bytes_kernel(uint4 *p, size_t n16) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n16; i += stride) p[i] = make_uint4(0, 0, 0, 0);
}

__global__ void gather_out_kernel(const float *__restrict__ in, int64_t ld_in, const int32_t *__restrict__ sop,
                                  int64_t P, int C, float *__restrict__ out) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < P * C; e += (int64_t)gridDim.x * 256) {
    const int64_t p = e / C;
    const int c = (int)(e - p * C);
    const int s = sop[p];
    out[e] = (s >= 0) ? in[(int64_t)s * ld_in + c] : 0.0f;
  }
}

// -----------------------------------------------------------------------------------------
// host side
// -----------------------------------------------------------------------------------------
template <typename T>
static int dev_alloc(T **p, size_t count) {
  *p = nullptr;
  if (count == 0) count = 1;
  INSC_HIP(hipMalloc((void **)p, sizeof(T) * count));
  return INSC_OK;
}

template <typename T>
static int dev_grow(T **p, size_t old_count, size_t new_count, hipStream_t s) {
  T *q = nullptr;
  INSC_HIP(hipMalloc((void **)&q, sizeof(T) * (new_count ? new_count : 1)));
  if (*p && old_count) INSC_HIP(hipMemcpyAsync(q, *p, sizeof(T) * old_count, hipMemcpyDeviceToDevice, s));
  INSC_HIP(hipStreamSynchronize(s));
  if (*p) INSC_HIP(hipFree(*p));
  *p = q;
  return INSC_OK;
}

static int fill_i32(int32_t *p, int64_t n, int32_t v, hipStream_t s) { return insc_fill_i32(p, n, v, (void *)s); }

static float *tensor_ptr(insc_net *net, int t) {
  const Tensor &T = net->tensors[t];
  return net->buffers[T.buf].p + T.col0;
}
static int64_t tensor_ld(insc_net *net, int t) { return net->buffers[net->tensors[t].buf].ld; }

static int dirty_node(insc_net *net, int kind, int level, int a, int b) {
  std::vector<int> key = {kind, level, a, b};
  auto it = net->dirty_index.find(key);
  if (it != net->dirty_index.end()) return it->second;
  DirtyNode d;
  d.kind = kind;
  d.level = level;
  d.src0 = a;
  d.src1 = b;
  if (a >= 0) d.ancestors = net->dirty[a].ancestors;
  if (b >= 0) d.ancestors.insert(net->dirty[b].ancestors.begin(), net->dirty[b].ancestors.end());
  const int id = (int)net->dirty.size();
  d.ancestors.insert(id);
  net->dirty.push_back(d);
  net->dirty_index[key] = id;
  return id;
}

// Every propagation rule only grows a set, so a set derived from another contains it and the
// union of the two is the derived one.
static int dirty_union(insc_net *net, int a, int b) {
  if (a == b) return a;
  if (net->dirty[b].ancestors.count(a)) return b;
  if (net->dirty[a].ancestors.count(b)) return a;
  return dirty_node(net, D_UNION, net->dirty[a].level, std::min(a, b), std::max(a, b));
}

// (re)allocate everything that is sized by the capacity of level l
static int level_reserve(insc_net *net, int l, int64_t cap, hipStream_t s) {
  Level &L = net->levels[l];
  if (cap <= L.cap) return INSC_OK;
  cap = std::max<int64_t>(cap, 1024);
  cap = (cap + 31) / 32 * 32;
  int rc;
  if (!L.grid) {
    rc = insc_grid_create(cap, &L.grid);
  } else {
    rc = insc_grid_reserve(L.grid, cap, (void *)s);
  }
  if (rc) return rc;
  const int64_t old = L.cap;
  if ((rc = dev_grow(&L.nbr, (size_t)old * 27, (size_t)cap * 27, s))) return rc;
  if ((rc = dev_grow(&L.order, (size_t)old, (size_t)cap, s))) return rc;
  if ((rc = dev_grow(&L.pos, (size_t)old, (size_t)cap, s))) return rc;
  if ((rc = dev_grow(&L.plan, 0, (size_t)cap * 27, s))) return rc;  // contents dropped: rebuilt by the next frame
  L.plan_valid = false;
  if ((rc = dev_grow(&L.tmask, 0, (size_t)cap / 32 + 1, s))) return rc;
  if ((rc = dev_grow(&L.sched, 0, (size_t)cap / 32 + (size_t)cap / 128 + 3, s))) return rc;  // tiles, then groups of 4
  if (l + 1 < net->n_levels) {
    if ((rc = dev_grow(&L.parent, (size_t)old, (size_t)cap, s))) return rc;
    if ((rc = dev_grow(&L.offset, (size_t)old, (size_t)cap, s))) return rc;
    if ((rc = dev_grow(&L.bo_order, (size_t)old, (size_t)cap, s))) return rc;
    if ((rc = dev_grow(&L.bo_pos, (size_t)old, (size_t)cap, s))) return rc;
  }
  if (l > 0) {  // child map of the link from the finer level has one row per site of this level
    Level &F = net->levels[l - 1];
    if ((rc = dev_grow(&F.child, (size_t)F.child_rows * 8, (size_t)cap * 8, s))) return rc;
    if ((rc = fill_i32(F.child + F.child_rows * 8, (cap - F.child_rows) * 8, -1, s))) return rc;
    F.child_rows = cap;
  }
  if (l == 0) {
    if ((rc = dev_grow(&net->in_sum, (size_t)old * net->in_channels, (size_t)cap * net->in_channels, s))) return rc;
    if ((rc = dev_grow(&net->in_cnt, (size_t)old, (size_t)cap, s))) return rc;
    if ((rc = dev_grow(&net->chain_head, (size_t)old, (size_t)cap, s))) return rc;
    INSC_HIP(hipMemsetAsync(net->in_sum + old * net->in_channels, 0, sizeof(float) * (cap - old) * net->in_channels, s));
    INSC_HIP(hipMemsetAsync(net->in_cnt + old, 0, sizeof(int32_t) * (cap - old), s));
    if ((rc = fill_i32(net->chain_head + old, cap - old, -1, s))) return rc;
  }
  for (Buffer &B : net->buffers)
    if (B.level == l) {
      if ((rc = dev_grow(&B.p, (size_t)B.rows * B.ld, (size_t)cap * B.ld, s))) return rc;
      B.rows = cap;
    }
  L.cap = cap;
  // masks of this level live in the arena: rebuild it
  size_t bytes = 0;
  for (DirtyNode &d : net->dirty) {
    const int64_t c = net->levels[d.level].cap;
    bytes += ((size_t)c + 255) / 256 * 256 * 1 + 3 * (((size_t)c / 32 + 1 + 255) / 256 * 256);
  }
  if (bytes > net->mask_arena_bytes) {
    INSC_HIP(hipStreamSynchronize(s));
    if (net->mask_arena) INSC_HIP(hipFree(net->mask_arena));
    INSC_HIP(hipMalloc((void **)&net->mask_arena, bytes));
    net->mask_arena_bytes = bytes;
  }
  size_t off = 0;
  for (DirtyNode &d : net->dirty) {
    const size_t c = (size_t)net->levels[d.level].cap;
    const size_t mb = (c + 255) / 256 * 256, tb = (c / 32 + 1 + 255) / 256 * 256;
    d.mask = net->mask_arena + off;
    d.tflag = d.mask + mb;
    d.tflag_bo = d.tflag + tb;
    d.ccount = (int32_t *)(d.tflag_bo + tb);
    off += mb + 3 * tb;
    if (d.depth >= 0 && d.crows_cap < (int64_t)c) {
      INSC_HIP(hipStreamSynchronize(s));
      if (d.crows) INSC_HIP(hipFree(d.crows));
      d.crows = nullptr;
      INSC_HIP(hipMalloc((void **)&d.crows, sizeof(int32_t) * c));
      d.crows_cap = (int64_t)c;
    }
  }
  return INSC_OK;
}

static int points_reserve(insc_net *net, int64_t need, hipStream_t s) {
  if (need <= net->points_cap) return INSC_OK;
  const int64_t cap = std::max<int64_t>(need + need / 2, 4096);
  int rc;
  if ((rc = dev_grow(&net->site_of_point, (size_t)net->n_points, (size_t)cap, s))) return rc;
  if ((rc = dev_grow(&net->chain_next, 0, (size_t)cap, s))) return rc;
  net->points_cap = cap;
  return INSC_OK;
}

// the site counts and error flags of all scales, as the insert kernels left them in net->h_counts
static int apply_counts(insc_net *net, const char *who) {
  const int L = net->n_levels;
  for (int l = 0; l < L; l++) {
    Level &Lv = net->levels[l];
    Lv.n = Lv.n_upper = net->h_counts[2 * l];
    Lv.grid->n_exact = Lv.grid->n_upper = Lv.n;
  }
  if (net->h_counts[2 * L] == net->frame_id) {
    // (nothing of the frame was inserted: the state is that of the previous frame)
    set_error("%s: a coordinate is outside 0..65535 (batch 0..32767); the frame was dropped", who);
    return INSC_ERR_COORD;
  }
  for (int l = 0; l < L; l++) {
    const int err = net->h_counts[2 * l + 1];
    if (err & 1) {
      set_error("%s: a coordinate is outside 0..65535 (batch 0..32767)", who);
      return INSC_ERR_COORD;
    }
    if (err & 2) {
      set_error("%s: capacity of scale %d exceeded", who, l);
      return INSC_ERR_CAPACITY;
    }
  }
  return INSC_OK;
}

// ---- one layer ------------------------------------------------------------------------
static int run_op(insc_net *net, const Op &op, bool incremental, hipStream_t s) {
  if (op.fused) return INSC_OK;
  const Tensor &To = net->tensors[op.out];
  const Level &Lo = net->levels[To.level];
  // (a set known to hold every row needs no flags: the layer runs as in a full frame)
  const DirtyNode *d = incremental && !net->dirty_full[(size_t)To.dirty] ? &net->dirty[To.dirty] : nullptr;
  // (the host has had the exact site counts since the structure phase - apply_counts - so the layers take
  // their row count by value: a kernel that starts by loading it from device memory has one more
  // dependent memory round trip ahead of its first useful load)
  const int32_t *d_n = nullptr;
  const int64_t n_up = Lo.n_upper;
  // a convolution that also forms the sum of its residual block writes what the OP_ADD would
  const Op *add = op.fused_add >= 0 ? &net->ops[op.fused_add] : nullptr;
  const Op &tail = add ? *add : op;  // the op whose outputs this kernel writes
  float *out = tail.write_raw ? tensor_ptr(net, tail.out) : nullptr;
  const int64_t ld_out = tensor_ld(net, tail.out);
  BnEpilogue ep;
  if (add) {
    const int other = add->in0 == op.out ? add->in1 : add->in0;
    ep.res = tensor_ptr(net, other);
    ep.ldr = tensor_ld(net, other);
  }
  if (tail.fused_bn >= 0) {
    const Op &bn = net->ops[tail.fused_bn];
    ep.w = bn.bn_w;
    ep.b = bn.bn_b;
    ep.leak = bn.leak;
    ep.out2 = tensor_ptr(net, bn.out);
    ep.ld2 = tensor_ld(net, bn.out);
  }
  if (op.fused_join_bn >= 0) {
    // batch norm of [other | own output]: columns of the normalised matrix by the place each half has
    // in the joined one
    const Op &bn = net->ops[op.fused_join_bn];
    const Tensor &Tj = net->tensors[bn.in0], &Tx = net->tensors[op.out], &Ty = net->tensors[op.join_other];
    const int cx = Tx.col0 - Tj.col0, cy = Ty.col0 - Tj.col0;
    ep.w = bn.bn_w + cx;
    ep.b = bn.bn_b + cx;
    ep.leak = bn.leak;
    ep.out2 = tensor_ptr(net, bn.out) + cx;
    ep.ld2 = tensor_ld(net, bn.out);
    ep.side_in = tensor_ptr(net, op.join_other);
    ep.ld_side = tensor_ld(net, op.join_other);
    ep.side_out = tensor_ptr(net, bn.out) + cy;
    ep.side_w = bn.bn_w + cy;
    ep.side_b = bn.bn_b + cy;
  }
  const float *in0 = tensor_ptr(net, op.in0);
  const int64_t ld0 = tensor_ld(net, op.in0);
  const int64_t rows0 = net->buffers[net->tensors[op.in0].buf].rows;
  switch (op.kind) {
    case OP_SSC: {
      if (d && d->compact)  // tiles made of the set's rows only (no tile plan: its positions are the full order's)
        return launch_conv(in0, ld0, rows0, out, ld_out, op.W, op.Wp, op.bias, Lo.nbr, nullptr, MAP_NBR, 27, d->crows,
                           d->ccount, n_up, op.Cin, op.Cout, nullptr, d->mask, s, ep, TilePlan(), 0, d->expect_rows);
      TilePlan plan;
      plan.map = Lo.plan;
      plan.ld = Lo.cap;
      plan.tmask = Lo.tmask;
      plan.sched = Lo.sched;
      return launch_conv(in0, ld0, rows0, out, ld_out, op.W, op.Wp, op.bias, Lo.nbr, nullptr, MAP_NBR, 27, Lo.order, d_n,
                         n_up, op.Cin, op.Cout, d ? d->tflag : nullptr, d ? d->mask : nullptr, s, ep, plan);
    }
    case OP_NIN:
      return launch_conv(in0, ld0, rows0, out, ld_out, op.W, op.Wp, op.bias, nullptr, nullptr, MAP_IDENTITY, 1, Lo.order,
                         d_n, n_up, op.Cin, op.Cout, d ? d->tflag : nullptr, d ? d->mask : nullptr, s, ep);
    case OP_CONV: {
      const Level &Lf = net->levels[To.level - 1];
      return launch_conv(in0, ld0, rows0, out, ld_out, op.W, op.Wp, op.bias, Lf.child, nullptr, MAP_NBR, 8, Lo.order, d_n,
                         n_up, op.Cin, op.Cout, d ? d->tflag : nullptr, d ? d->mask : nullptr, s, ep);
    }
    case OP_DECONV:
      return launch_conv(in0, ld0, rows0, out, ld_out, op.W, op.Wp, op.bias, Lo.parent, Lo.offset, MAP_PARENT, 8,
                         Lo.bo_order, d_n, n_up, op.Cin, op.Cout, d ? d->tflag_bo : nullptr, d ? d->mask : nullptr,
                         s, ep);
    case OP_BN:
      return launch_bn(in0, ld0, out, ld_out, op.mean, op.var, op.gamma, op.beta, op.eps, op.leak, nullptr, d_n,
                       n_up, op.Cout, d ? d->mask : nullptr, s);
    case OP_ADD:
      return launch_add(in0, ld0, tensor_ptr(net, op.in1), tensor_ld(net, op.in1), out, ld_out, nullptr, d_n, n_up,
                        op.Cout, d ? d->mask : nullptr, s, ep);
    case OP_COPY:
      return launch_add(in0, ld0, nullptr, 0, out, ld_out, nullptr, d_n, n_up, op.Cout, d ? d->mask : nullptr, s);
    case OP_JOIN:
      return INSC_OK;  // the inputs are column slices of the output
  }
  set_error("run_op: unknown op kind %d", op.kind);
  return INSC_ERR_STATE;
}

static int run_dirty_node(insc_net *net, int id, hipStream_t s) {
  DirtyNode &d = net->dirty[id];
  const Level &L = net->levels[d.level];
  uint8_t *tbo = d.tiles_by_offset ? d.tflag_bo : nullptr;
  switch (d.kind) {
    case D_INPUT:
      return INSC_OK;  // marked by the input layer
    case D_DILATE: {
      if (L.n_upper == 0) return INSC_OK;
      const DirtyNode &src = net->dirty[d.src0];
      if (src.kind == D_INPUT && net->frame_sop && net->frame_P * 8 <= L.n_upper) {
        // the source is the frame's own points
        if (net->frame_P == 0) return INSC_OK;
        hipLaunchKernelGGL(dirty_dilate_list_kernel, dim3(grid_for(net->frame_P * 27, 256)), dim3(256), 0, s, L.nbr,
                           net->frame_sop, (const int32_t *)nullptr, net->frame_P, d.mask, d.tflag, L.pos, tbo, L.bo_pos);
        break;
      }
      if (src.compact) {
        hipLaunchKernelGGL(dirty_dilate_list_kernel, dim3(grid_for(src.expect_rows * 27 * 2, 256, 1 << 16)), dim3(256), 0, s,
                           L.nbr, src.crows, src.ccount, 0, d.mask, d.tflag, L.pos, tbo, L.bo_pos);
        break;
      }
      hipLaunchKernelGGL(dirty_dilate_kernel, dim3(grid_for(L.n_upper * 27, 256, 1ll << 30)), dim3(256), 0, s, L.nbr,
                         net->dirty[d.src0].mask, d.mask, d.tflag, L.pos, tbo, L.bo_pos, L.grid->d_n, L.n_upper);
      break;
    }
    case D_PARENTS: {
      const Level &F = net->levels[d.level - 1];
      if (F.n_upper == 0) return INSC_OK;
      hipLaunchKernelGGL(dirty_parents_kernel, dim3(grid_for(F.n_upper, 256)), dim3(256), 0, s, F.parent,
                         net->dirty[d.src0].mask, d.mask, d.tflag, L.pos, F.grid->d_n, F.n_upper);
      break;
    }
    case D_CHILDREN:
      if (L.n_upper == 0) return INSC_OK;
      hipLaunchKernelGGL(dirty_children_kernel, dim3(grid_for(L.n_upper, 256)), dim3(256), 0, s, L.parent,
                         net->dirty[d.src0].mask, d.mask, d.tflag, L.pos, tbo, L.bo_pos, L.grid->d_n, L.n_upper);
      break;
    case D_UNION:
      if (L.n_upper == 0) return INSC_OK;
      hipLaunchKernelGGL(dirty_union_kernel, dim3(grid_for(L.n_upper, 256)), dim3(256), 0, s,
                         net->dirty[d.src0].mask, net->dirty[d.src1].mask, d.mask, d.tflag, L.pos, tbo, L.bo_pos,
                         L.grid->d_n, L.n_upper);
      break;
  }
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}


// What one convolution of the last frame worked on (diagnostics): one wavefront per 32-row tile of the
// layer's processing order (or of its list of dirty rows).  For the tiles the layer computed:
// acc[0] += output rows, acc[1] += rules (existing (row, offset) pairs), acc[2] += 32 x offsets the
// tile uses (the (row, offset) slots the matrix cores are issued work for, empty ones included).
__global__ __launch_bounds__(256) void conv_work_kernel(const int32_t *__restrict__ map0, const int32_t *__restrict__ map1,
                                                        int mode, int K, const int32_t *__restrict__ rows,
                                                        const int32_t *__restrict__ d_n, int64_t n_rows,
                                                        const uint8_t *__restrict__ tile_flags,
                                                        unsigned long long *__restrict__ acc) {
  const int64_t n = d_n ? min((int64_t)*d_n, n_rows) : n_rows;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t * 32 >= n) return;
  if (tile_flags && !tile_flags[t]) return;
  const int64_t p = t * 32 + (lane & 31);
  unsigned bits = 0;
  int rules = 0, valid = 0;
  if (lane < 32 && p < n) {
    const int64_t row = rows ? rows[p] : p;
    valid = 1;
    if (mode == MAP_NBR) {
      for (int k = 0; k < K; k++)
        if (map0[row * K + k] >= 0) {
          bits |= 1u << k;
          rules++;
        }
    } else if (mode == MAP_PARENT) {
      bits = 1u << map1[row];
      rules = 1;
    } else {
      bits = 1u;
      rules = 1;
    }
  }
  for (int o = 32; o >= 1; o >>= 1) {
    bits |= __shfl_xor(bits, o);
    rules += __shfl_xor(rules, o);
    valid += __shfl_xor(valid, o);
  }
  if (lane == 0) {
    atomicAdd(acc + 0, (unsigned long long)valid);
    atomicAdd(acc + 1, (unsigned long long)rules);
    atomicAdd(acc + 2, (unsigned long long)(__popc(bits) * 32));
  }
}

}  // namespace insc

using namespace insc;

extern "C" {

int insc_net_create(int n_levels, int in_channels, int mode, insc_net **out) {
  INSC_REQUIRE(out && n_levels >= 1 && n_levels <= 16 && in_channels >= 1, INSC_ERR_ARG,
               "insc_net_create: bad arguments");
  INSC_REQUIRE(mode == 0 || mode == 3 || mode == 4, INSC_ERR_ARG,
               "insc_net_create: input mode %d (0, 3 and 4 are provided)", mode);
  insc_net *net = new insc_net();
  net->n_levels = n_levels;
  net->in_channels = in_channels;
  net->mode = mode;
  net->levels.resize(n_levels);
  // tensor 0: the input layer's output
  Tensor t;
  t.level = 0;
  t.C = in_channels;
  Buffer b;
  b.level = 0;
  b.ld = in_channels;
  net->buffers.push_back(b);
  t.buf = 0;
  net->tensors.push_back(t);
  INSC_HIP(hipHostMalloc((void **)&net->h_counts, sizeof(int32_t) * 64, hipHostMallocDefault));
  INSC_HIP(hipEventCreateWithFlags(&net->ev_counts, hipEventDisableTiming));
  INSC_HIP(hipMalloc((void **)&net->d_bad, 256));
  INSC_HIP(hipMemset(net->d_bad, 0, 256));
  *out = net;
  return INSC_OK;
}

int insc_net_destroy(insc_net *net) {
  if (!net) return INSC_OK;
  (void)hipDeviceSynchronize();
  for (Level &L : net->levels) {
    if (L.grid) insc_grid_destroy(L.grid);
    void *ps[] = {L.nbr, L.order, L.pos, L.plan, L.tmask, L.sched, L.parent, L.offset, L.child, L.bo_order, L.bo_pos};
    for (void *p : ps)
      if (p) (void)hipFree(p);
  }
  for (Buffer &B : net->buffers)
    if (B.p) (void)hipFree(B.p);
  for (DirtyNode &d : net->dirty)
    if (d.crows) (void)hipFree(d.crows);
  for (Op &op : net->ops) {
    if (op.Wp) (void)hipFree(op.Wp);
    if (op.bn_w) (void)hipFree(op.bn_w);
    if (op.bn_b) (void)hipFree(op.bn_b);
  }
  for (Level &L : net->rf.levels) {
    if (L.grid) insc_grid_destroy(L.grid);
    void *ps[] = {L.nbr, L.parent, L.offset, L.child};
    for (void *p : ps)
      if (p) (void)hipFree(p);
  }
  for (int32_t *p : net->rf.pre_exist)
    if (p) (void)hipFree(p);
  for (int32_t *p : net->rf.nbr_pre)
    if (p) (void)hipFree(p);
  for (int32_t *p : net->rf.parent2)
    if (p) (void)hipFree(p);
  for (Buffer &B : net->rf.buffers)
    if (B.p) (void)hipFree(B.p);
  void *rps[] = {net->rf.in_sum, net->rf.in_cnt, net->rf.chain_head, net->rf.chain_next, net->rf.sop};
  for (void *p : rps)
    if (p) (void)hipFree(p);
  void *ps[] = {net->in_sum, net->in_cnt, net->chain_head, net->chain_next, net->site_of_point, net->mask_arena, net->d_bad};
  for (void *p : ps)
    if (p) (void)hipFree(p);
  if (net->h_counts) (void)hipHostFree(net->h_counts);
  for (hipEvent_t e : net->ev)
    if (e) (void)hipEventDestroy(e);
  if (net->ev_counts) (void)hipEventDestroy(net->ev_counts);
  delete net;
  return INSC_OK;
}

/* New feature matrix with C channels at scale `level`; *out_id receives its id. */
int insc_net_tensor(insc_net *net, int level, int C, int *out_id) {
  INSC_REQUIRE(net && out_id && !net->finalized, INSC_ERR_STATE, "insc_net_tensor: net is null or finalized");
  INSC_REQUIRE(level >= 0 && level < net->n_levels && C >= 1, INSC_ERR_ARG, "insc_net_tensor: bad level/channels");
  Buffer b;
  b.level = level;
  b.ld = C;
  net->buffers.push_back(b);
  Tensor t;
  t.level = level;
  t.C = C;
  t.buf = (int)net->buffers.size() - 1;
  net->tensors.push_back(t);
  *out_id = (int)net->tensors.size() - 1;
  return INSC_OK;
}

/* Channel concatenation without copies: tensor `out` (Ca+Cb channels) is declared first, then
 * a and b are re-homed as column slices of its matrix, so their producers write in place. */
int insc_net_join(insc_net *net, int a, int b, int out) {
  INSC_REQUIRE(net && !net->finalized, INSC_ERR_STATE, "insc_net_join: net is null or finalized");
  const int nt = (int)net->tensors.size();
  INSC_REQUIRE(a > 0 && a < nt && b > 0 && b < nt && out > 0 && out < nt && a != b, INSC_ERR_ARG,
               "insc_net_join: bad tensor ids");
  Tensor &A = net->tensors[a], &B = net->tensors[b], &O = net->tensors[out];
  INSC_REQUIRE(A.level == O.level && B.level == O.level && A.C + B.C == O.C, INSC_ERR_ARG,
               "insc_net_join: shapes do not add up");
  INSC_REQUIRE(net->buffers[A.buf].ld == A.C && net->buffers[B.buf].ld == B.C && A.col0 == 0 && B.col0 == 0,
               INSC_ERR_ARG, "insc_net_join: an input is already part of another join");
  net->buffers[A.buf].ld = 0;  // the stand-alone matrices are no longer needed
  net->buffers[B.buf].ld = 0;
  A.buf = O.buf;
  A.col0 = O.col0;
  B.buf = O.buf;
  B.col0 = O.col0 + A.C;
  // no kernel runs for a join; the entry only carries the dirty-set rule (union of the inputs)
  Op op;
  op.kind = OP_JOIN;
  op.in0 = a;
  op.in1 = b;
  op.out = out;
  net->ops.push_back(op);
  return INSC_OK;
}

static int add_op(insc_net *net, Op op) {
  INSC_REQUIRE(net && !net->finalized, INSC_ERR_STATE, "insc_net_op: net is null or finalized");
  const int nt = (int)net->tensors.size();
  INSC_REQUIRE(op.in0 >= 0 && op.in0 < nt && op.out > 0 && op.out < nt && op.in1 < nt, INSC_ERR_ARG,
               "insc_net_op: bad tensor ids");
  net->ops.push_back(op);
  return INSC_OK;
}

/* kind: 0 submanifold 3^3 (W [27,Cin,Cout]), 2 convolution 2/2 to the next coarser scale
 * (W [8,Cin,Cout]), 3 deconvolution 2/2 to the next finer scale, 4 network-in-network
 * (W [Cin,Cout]).  The weight and bias pointers must stay valid for the life of the net. */
int insc_net_op_conv(insc_net *net, int kind, int in, int out, const float *d_W, const float *d_bias) {
  INSC_REQUIRE(kind == OP_SSC || kind == OP_CONV || kind == OP_DECONV || kind == OP_NIN, INSC_ERR_ARG,
               "insc_net_op_conv: bad kind %d", kind);
  INSC_REQUIRE(net && d_W, INSC_ERR_ARG, "insc_net_op_conv: null argument");
  const int nt = (int)net->tensors.size();
  INSC_REQUIRE(in >= 0 && in < nt && out > 0 && out < nt, INSC_ERR_ARG, "insc_net_op_conv: bad tensor ids");
  const Tensor &Ti = net->tensors[in], &To = net->tensors[out];
  const int dl = kind == OP_CONV ? 1 : kind == OP_DECONV ? -1 : 0;
  INSC_REQUIRE(To.level == Ti.level + dl, INSC_ERR_ARG, "insc_net_op_conv: scales of input and output do not fit");
  Op op;
  op.kind = kind;
  op.in0 = in;
  op.out = out;
  op.W = d_W;
  op.bias = d_bias;
  op.Cin = Ti.C;
  op.Cout = To.C;
  return add_op(net, op);
}

int insc_net_op_bn(insc_net *net, int in, int out, const float *d_mean, const float *d_var, const float *d_gamma,
                   const float *d_beta, float eps, float leakiness) {
  INSC_REQUIRE(net && d_mean && d_var, INSC_ERR_ARG, "insc_net_op_bn: null argument");
  const int nt = (int)net->tensors.size();
  INSC_REQUIRE(in >= 0 && in < nt && out > 0 && out < nt, INSC_ERR_ARG, "insc_net_op_bn: bad tensor ids");
  INSC_REQUIRE(net->tensors[in].C == net->tensors[out].C && net->tensors[in].level == net->tensors[out].level,
               INSC_ERR_ARG, "insc_net_op_bn: shapes differ");
  Op op;
  op.kind = OP_BN;
  op.in0 = in;
  op.out = out;
  op.mean = d_mean;
  op.var = d_var;
  op.gamma = d_gamma;
  op.beta = d_beta;
  op.eps = eps;
  op.leak = leakiness;
  op.Cin = op.Cout = net->tensors[out].C;
  return add_op(net, op);
}

int insc_net_op_add(insc_net *net, int a, int b, int out) {
  INSC_REQUIRE(net, INSC_ERR_ARG, "insc_net_op_add: null argument");
  const int nt = (int)net->tensors.size();
  INSC_REQUIRE(a >= 0 && a < nt && b >= 0 && b < nt && out > 0 && out < nt, INSC_ERR_ARG,
               "insc_net_op_add: bad tensor ids");
  INSC_REQUIRE(net->tensors[a].C == net->tensors[out].C && net->tensors[b].C == net->tensors[out].C &&
                   net->tensors[a].level == net->tensors[out].level &&
                   net->tensors[b].level == net->tensors[out].level,
               INSC_ERR_ARG, "insc_net_op_add: shapes differ");
  Op op;
  op.kind = OP_ADD;
  op.in0 = a;
  op.in1 = b;
  op.out = out;
  op.Cin = op.Cout = net->tensors[out].C;
  return add_op(net, op);
}

/* Freeze the program: derive the dirty-set dataflow, pack the weights, reserve capacity. */
int insc_net_finalize(insc_net *net, int out_tensor, int64_t capacity_sites, void *stream) {
  INSC_REQUIRE(net && !net->finalized, INSC_ERR_STATE, "insc_net_finalize: net is null or already finalized");
  INSC_REQUIRE(out_tensor >= 0 && out_tensor < (int)net->tensors.size() && net->tensors[out_tensor].level == 0,
               INSC_ERR_ARG, "insc_net_finalize: the output tensor must be at the input scale");
  hipStream_t s = (hipStream_t)stream;
  net->out_tensor = out_tensor;
  // a tensor re-homed by a join whose producer is not in the program (the input) needs a copy;
  // this cannot happen for tensor 0 because insc_net_join rejects it.
  net->tensors[0].dirty = dirty_node(net, D_INPUT, 0, -1, -1);
  for (Op &op : net->ops) {
    const Tensor &Ti = net->tensors[op.in0];
    Tensor &To = net->tensors[op.out];
    INSC_REQUIRE(Ti.dirty >= 0, INSC_ERR_STATE, "insc_net_finalize: op reads a tensor that nothing produced");
    switch (op.kind) {
      case OP_SSC:
        To.dirty = dirty_node(net, D_DILATE, To.level, Ti.dirty, -1);
        break;
      case OP_CONV:
        To.dirty = dirty_node(net, D_PARENTS, To.level, Ti.dirty, -1);
        break;
      case OP_DECONV:
        To.dirty = dirty_node(net, D_CHILDREN, To.level, Ti.dirty, -1);
        net->dirty[To.dirty].tiles_by_offset = true;
        break;
      case OP_ADD:
      case OP_JOIN:
        INSC_REQUIRE(net->tensors[op.in1].dirty >= 0, INSC_ERR_STATE,
                     "insc_net_finalize: op reads a tensor that nothing produced");
        To.dirty = dirty_union(net, Ti.dirty, net->tensors[op.in1].dirty);
        break;
      default:
        To.dirty = Ti.dirty;
    }
    if (op.kind == OP_SSC || op.kind == OP_CONV || op.kind == OP_DECONV || op.kind == OP_NIN) {
      const int K = op.kind == OP_SSC ? 27 : op.kind == OP_NIN ? 1 : 8;
      if (op.Cin % 16 == 0) {
        const int64_t nf = packed_floats(K, op.Cin, op.Cout);
        int rc = dev_alloc(&op.Wp, (size_t)nf);
        if (rc) return rc;
        rc = pack_weights(op.W, K, op.Cin, op.Cout, op.Wp, s);
        if (rc) return rc;
      }
    }
  }
  // sets at the input scale that are reached from the frame's points through 3^3 layers only
  for (DirtyNode &d : net->dirty) {
    if (d.kind == D_INPUT)
      d.depth = 0;
    else if (d.kind == D_DILATE && d.level == 0 && d.src0 >= 0 && net->dirty[(size_t)d.src0].depth >= 0)
      d.depth = net->dirty[(size_t)d.src0].depth + 1;
  }
  // Fold each batch norm into the kernel that produces its input (one fewer pass over the rows
  // and one fewer launch); the producer keeps writing its raw result only if something else
  // reads it.  A tensor nothing reads any more loses its matrix.
  {
    const int nt = (int)net->tensors.size();
    std::vector<int> producer(nt, -1), readers(nt, 0);
    for (int i = 0; i < (int)net->ops.size(); i++) {
      const Op &op = net->ops[i];
      if (op.kind != OP_JOIN) producer[op.out] = producer[op.out] == -1 ? i : -2;
      readers[op.in0]++;
      if (op.in1 >= 0) readers[op.in1]++;
    }
    readers[out_tensor]++;
    for (int i = 0; i < (int)net->ops.size(); i++) {
      Op &bn = net->ops[i];
      if (bn.kind != OP_BN) continue;
      int rc;
      if ((rc = dev_alloc(&bn.bn_w, (size_t)bn.Cout))) return rc;
      if ((rc = dev_alloc(&bn.bn_b, (size_t)bn.Cout))) return rc;
      if ((rc = bn_scale_shift(bn.mean, bn.var, bn.gamma, bn.beta, bn.eps, bn.Cout, bn.bn_w, bn.bn_b, s))) return rc;
      if (bn.in0 == bn.out || producer[bn.in0] < 0 || producer[bn.out] != i) continue;
      Op &A = net->ops[producer[bn.in0]];
      const bool can = A.kind == OP_SSC || A.kind == OP_CONV || A.kind == OP_DECONV || A.kind == OP_NIN || A.kind == OP_ADD;
      if (!can || A.fused_bn >= 0 || producer[bn.in0] > i) continue;
      A.fused_bn = i;
      bn.fused = true;
      A.write_raw = readers[bn.in0] > 1 || net->keep_raw;
      if (!A.write_raw) {
        Tensor &T = net->tensors[bn.in0];
        Buffer &B = net->buffers[T.buf];
        if (T.col0 == 0 && B.ld == T.C) B.ld = 0;
        T.kept = false;
      }
    }
    // A batch norm over a channel concatenation [other | deconvolution output] (the decoder of a
    // U-Net): the deconvolution normalises its own columns in its epilogue and, row by row, the other
    // tensor's columns as well - same rows (the sets of rows due must be the same one), same column
    // blocks (equal widths), and the other tensor is complete by then.
    for (int i = 0; i < (int)net->ops.size(); i++) {
      Op &bn = net->ops[i];
      if (bn.kind != OP_BN || bn.fused || bn.in0 == bn.out || producer[bn.out] != i) continue;
      int jn = -1;
      for (int k = 0; k < i; k++)
        if (net->ops[k].kind == OP_JOIN && net->ops[k].out == bn.in0) jn = k;
      if (jn < 0) continue;
      const Op &J = net->ops[jn];
      for (int side = 0; side < 2; side++) {
        const int x = side ? J.in0 : J.in1, y = side ? J.in1 : J.in0;  // x: the deconvolution's output
        const int a = producer[x], py = producer[y];
        if (a < 0 || a > i || py < 0 || py > a) continue;
        Op &A = net->ops[a];
        if (A.kind != OP_DECONV || A.fused_bn >= 0 || A.fused_join_bn >= 0 || A.Cin % 16 != 0) continue;
        const Tensor &Tx = net->tensors[x], &Ty = net->tensors[y];
        if (Tx.C != Ty.C || Tx.C != A.Cout || !Ty.kept) continue;
        if (Tx.dirty != net->tensors[bn.out].dirty) continue;
        A.fused_join_bn = i;
        A.join_other = y;
        bn.fused = true;
        break;
      }
    }
  }
  // Fold the element-wise sum that ends a residual block into the convolution that feeds it
  // (the other operand must exist by then and both must be due on the same rows).
  {
    const int nt = (int)net->tensors.size();
    std::vector<int> producer(nt, -1), readers(nt, 0);
    for (int i = 0; i < (int)net->ops.size(); i++) {
      const Op &op = net->ops[i];
      if (op.kind != OP_JOIN) producer[op.out] = producer[op.out] == -1 ? i : -2;
      readers[op.in0]++;
      if (op.in1 >= 0) readers[op.in1]++;
    }
    readers[out_tensor]++;
    for (int i = 0; i < (int)net->ops.size(); i++) {
      Op &add = net->ops[i];
      if (add.kind != OP_ADD || add.fused || add.in0 == add.in1) continue;
      for (int side = 0; side < 2; side++) {
        const int x = side ? add.in0 : add.in1, other = side ? add.in1 : add.in0;  // prefer in1 (the block body)
        const int a = producer[x];
        if (a < 0 || a > i || readers[x] != 1) continue;
        Op &A = net->ops[a];
        const bool conv = A.kind == OP_SSC || A.kind == OP_CONV || A.kind == OP_DECONV || A.kind == OP_NIN;
        if (!conv || A.fused_bn >= 0 || A.fused_join_bn >= 0 || A.fused_add >= 0) continue;
        if (other != 0 && (producer[other] < 0 || producer[other] > a)) continue;  // not computed yet when A runs
        if (!net->tensors[other].kept) continue;
        if (net->tensors[x].dirty != net->tensors[add.out].dirty) continue;
        if (add.out == x || add.out == other) continue;
        A.fused_add = i;
        add.fused = true;
        Tensor &T = net->tensors[x];
        Buffer &B = net->buffers[T.buf];
        if (T.col0 == 0 && B.ld == T.C) B.ld = 0;
        T.kept = false;
        break;
      }
    }
  }
  net->finalized = true;
  int64_t cap = std::max<int64_t>(capacity_sites, 1024);
  for (int l = 0; l < net->n_levels; l++) {
    int rc = level_reserve(net, l, cap, s);
    if (rc) return rc;
    cap = std::max<int64_t>(cap / 2, 1024);
  }
  INSC_HIP(hipStreamSynchronize(s));
  return INSC_OK;
}

/* Re-pack the weights after the caller changed them in place.  The rows cached by earlier frames were
 * computed with the old parameters, so they are forgotten: the next frame must be a full one (an
 * incremental or residual frame before it fails with INSC_ERR_STATE instead of mixing old and new rows). */
int insc_net_refresh_weights(insc_net *net, void *stream) {
  INSC_REQUIRE(net && net->finalized, INSC_ERR_STATE, "insc_net_refresh_weights: net is not finalized");
  net->have_state = false;
  for (Op &op : net->ops)
    if (op.Wp) {
      const int K = op.kind == OP_SSC ? 27 : op.kind == OP_NIN ? 1 : 8;
      int rc = pack_weights(op.W, K, op.Cin, op.Cout, op.Wp, (hipStream_t)stream);
      if (rc) return rc;
    }
  for (Op &op : net->ops)
    if (op.bn_w) {
      int rc = bn_scale_shift(op.mean, op.var, op.gamma, op.beta, op.eps, op.Cout, op.bn_w, op.bn_b,
                              (hipStream_t)stream);
      if (rc) return rc;
    }
  return INSC_OK;
}

int insc_net_op_count(const insc_net *net) { return net ? (int)net->ops.size() : 0; }

int insc_net_rebind_op(insc_net *net, int op, const float *d_W, const float *d_bias, const float *d_mean,
                       const float *d_var, const float *d_gamma, const float *d_beta) {
  INSC_REQUIRE(net && op >= 0 && op < (int)net->ops.size(), INSC_ERR_ARG, "insc_net_rebind_op: no op %d", op);
  Op &o = net->ops[op];
  net->have_state = false;  // cached rows belong to the old parameters
  if (o.kind == OP_SSC || o.kind == OP_CONV || o.kind == OP_DECONV || o.kind == OP_NIN) {
    INSC_REQUIRE(d_W, INSC_ERR_ARG, "insc_net_rebind_op: op %d is a convolution and needs d_W", op);
    o.W = d_W;
    o.bias = d_bias;
  } else if (o.kind == OP_BN) {
    INSC_REQUIRE(d_mean && d_var, INSC_ERR_ARG, "insc_net_rebind_op: op %d is a batch norm and needs d_mean, d_var", op);
    o.mean = d_mean;
    o.var = d_var;
    o.gamma = d_gamma;
    o.beta = d_beta;
  } else {
    set_error("insc_net_rebind_op: op %d has no parameters", op);
    return INSC_ERR_ARG;
  }
  return INSC_OK;
}

/* One frame.  d_coords: int32 [P, coord_cols] (x,y,z[,batch]); d_feats: float32 [P,in_channels].
 * increment == 0: forget all state and run a full forward over these points.
 * increment != 0: append the points to the scene of the previous frames and recompute only
 *                 the rows they affect; the result equals a full forward over all points.
 * d_out (nullable): one row of the output tensor per point - of this frame's points
 * (out_all == 0, [P,C]) or of every point since the last full frame (out_all != 0).
 * h_n_sites (nullable): receives the number of active sites at the input scale.
 * The call returns once the frame is ENQUEUED on `stream` (it waits only for the site counts of the
 * structure phase).  d_coords, d_feats and d_out are read / written by kernels that may still be
 * running when it returns: they must stay valid, and the inputs unmodified, until the stream has
 * reached the end of the frame (work enqueued on the same stream afterwards is ordered behind it). */
int insc_net_forward(insc_net *net, const int32_t *d_coords, int coord_cols, const float *d_feats, int64_t P,
                     int increment, float *d_out, int out_all, int64_t *h_n_sites, void *stream) {
  INSC_REQUIRE(net && net->finalized, INSC_ERR_STATE, "insc_net_forward: net is not finalized");
  INSC_REQUIRE(P >= 0 && (P == 0 || (d_coords && d_feats)) && (coord_cols == 3 || coord_cols == 4), INSC_ERR_ARG,
               "insc_net_forward: bad arguments");
  INSC_REQUIRE(!increment || net->have_state, INSC_ERR_STATE,
               "insc_net_forward: incremental frame without a full frame before it (none yet, or the weights "
               "were rebound / refreshed since)");
  hipStream_t s = (hipStream_t)stream;
  const int L = net->n_levels;
  const int C0 = net->in_channels;
  int rc;
  const bool inc = increment != 0;
  net->frame_id = net->frame_id == INT32_MAX ? 1 : net->frame_id + 1;
  // Sites that arrive with incremental frames are appended to the processing orders, frame by frame, each
  // batch sorted among itself; tiles made of such batches use more filter offsets and gather from farther
  // apart than tiles of an order sorted as a whole (a sweep that grew a scene from 37k to 150k voxels in 49
  // frames: layers 2.42 ms against 2.11 ms per frame).  Once the appended part of a large scale passes a
  // share of the sorted part, the frame sorts the orders of all scales from scratch, as a full frame does
  // (results do not depend on the order).
  bool refresh = false;
  if (inc && P > 0 && net->order_refresh_pct > 0)
    for (int l = 0; l < L; l++) {
      const Level &Lv = net->levels[l];
      if (Lv.n > order_sorted_max() && (Lv.n - Lv.n_sorted) * 100 > Lv.n_sorted * net->order_refresh_pct) refresh = true;
    }

  if (!inc) {
    // all grids emptied, the child maps back to -1 and the input layer's running sums to zero: one launch
    insc_grid *gs[16];
    int32_t *chi[16];
    int64_t nchi[16];
    for (int l = 0; l < L; l++) {
      Level &Lv = net->levels[l];
      gs[l] = Lv.grid;
      chi[l] = (l + 1 < L && Lv.child_rows) ? Lv.child : nullptr;
      nchi[l] = Lv.child_rows * 8;
      Lv.n = Lv.n_upper = 0;
    }
    if ((rc = grid_clear_batch(gs, chi, nchi, L, net->in_sum, (int64_t)sizeof(float) * net->levels[0].cap * C0, s)))
      return rc;
    INSC_HIP(hipMemsetAsync(net->in_cnt, 0, sizeof(int32_t) * (size_t)net->levels[0].cap, s));
    net->n_points = 0;
    net->have_state = false;
  }
  // capacity: every new point may be a new site at every scale
  for (int l = 0; l < L; l++) {
    Level &Lv = net->levels[l];
    if (Lv.n + P > Lv.cap)
      if ((rc = level_reserve(net, l, std::max(Lv.n + P, Lv.cap + Lv.cap / 2), s))) return rc;
    Lv.new_upper = P;
    Lv.n_upper = Lv.n + P;
  }
  if ((rc = points_reserve(net, net->n_points + P, s))) return rc;

  if (net->profiling) INSC_HIP(hipEventRecord(net->ev[0], s));
  int32_t *sop = net->site_of_point + net->n_points;
  net->frame_sop = sop;
  net->frame_P = P;
  // A frame inserts at all scales at once (three launches up to 16k points, seven beyond), which also
  // leaves the new site counts in host memory; the host picks them up further down, while the GPU is
  // busy with the neighbour maps and orders of the new sites.
  if (P > 0) {
    {
      FrameInsertLevel fl[16];
      for (int l = 0; l < L; l++) {
        Level &Lv = net->levels[l];
        fl[l] = FrameInsertLevel{Lv.grid, Lv.parent, Lv.offset, Lv.child};
      }
      if ((rc = frame_insert_levels(fl, L, d_coords, coord_cols, P, net->d_bad, net->frame_id, sop, net->h_counts, s)))
        return rc;
      INSC_HIP(hipEventRecord(net->ev_counts, s));
    }
  }
  // the dirty masks, tile flags and list counters of the last frame go back to zero (behind the insert:
  // nothing before the input accumulation reads them, and the host gets its site counts that much earlier)
  if (inc && net->mask_arena_bytes) {
    hipLaunchKernelGGL(fill_bytes_kernel, dim3(1024), dim3(256), 0, s, (uint4 *)net->mask_arena,
                       net->mask_arena_bytes / 16);
    INSC_LAUNCH_CHECK();
  }
  if (P > 0) {
    // ---- neighbour maps and processing orders of the new sites, all scales per launch ------
    const insc_grid *grids[16];
    int32_t *nbrs[16], *orders[16], *poss[16], *bo_orders[16], *bo_poss[16];
    const int32_t *cnbrs[16], *offsets[16], *cposs[16];
    for (int l = 0; l < L; l++) {
      Level &Lv = net->levels[l];
      grids[l] = Lv.grid;
      nbrs[l] = Lv.nbr;
      cnbrs[l] = Lv.nbr;
      orders[l] = Lv.order;
      poss[l] = Lv.pos;
      cposs[l] = Lv.pos;
      offsets[l] = Lv.offset;
      bo_orders[l] = Lv.bo_order;
      bo_poss[l] = Lv.bo_pos;
    }
    // (an incremental frame keeps the tile plans of its scales up to date instead of rebuilding them:
    // entries of older sites are patched along with the map, the new sites' columns are appended
    // once they have their positions)
    PlanRef prefs[16];
    TilePlanBatch app;
    app.n = L;
    for (int l = 0; l < L; l++) {
      Level &Lv = net->levels[l];
      const bool keep = inc && !refresh && Lv.plan_valid;
      prefs[l] = keep ? PlanRef{Lv.plan, Lv.tmask, Lv.pos, Lv.cap} : PlanRef{nullptr, nullptr, nullptr, 0};
      app.job[l] = TilePlanJob{Lv.nbr, Lv.order, Lv.grid->d_n, 0, Lv.cap, keep ? Lv.plan : nullptr, Lv.tmask, nullptr};
    }
    if ((rc = ssc3_new_sites_batch(grids, nbrs, L, P, s, prefs, !inc))) return rc;
    if (inc && !refresh) {
      offsets[L - 1] = nullptr;  // the coarsest scale has no order by position inside a parent cell
      if ((rc = order_append_new_sites_both_batch(grids, cnbrs, offsets, orders, poss, bo_orders, bo_poss, L, P, s)))
        return rc;
      if ((rc = tile_plan_append_batch(app, P, s))) return rc;
    }  // (a full frame builds its orders from scratch further down, once the counts are known; so does a
       // frame that refreshes them)
  }
  // ---- input scale: accumulate the points' features per site (an incremental frame marks the tiles of
  // the touched sites, so the sites must have their positions by then) ---------------------------------
  auto accumulate_input = [&]() -> int {
    if (P <= 0) return INSC_OK;
    DirtyNode &din = net->dirty[net->tensors[0].dirty];
    const unsigned nb = grid_for(P, 256);
    hipLaunchKernelGGL(chain_push_kernel, dim3(nb), dim3(256), 0, s, sop, P, net->chain_head, net->chain_next);
    hipLaunchKernelGGL(chain_sum_kernel, dim3(nb), dim3(256), 0, s, d_feats, C0, sop, P, net->chain_head,
                       net->chain_next, net->in_sum, net->in_cnt, inc ? din.mask : nullptr,
                       inc ? din.tflag : nullptr, net->levels[0].pos);
    INSC_LAUNCH_CHECK();
    return INSC_OK;
  };
  if (!refresh && (rc = accumulate_input())) return rc;
  if (!inc || refresh) {
    // A full frame may synchronise: learn the exact counts, then build the processing orders
    // (pattern-sorted for the 3^3 convolutions, offset-grouped for the deconvolutions).
    if (P > 0) {
      INSC_HIP(hipEventSynchronize(net->ev_counts));
      if ((rc = apply_counts(net, "insc_net_forward"))) return rc;
    }
    // With a large scale around, the radix passes that it needs carry the other scales along in the same
    // launches (their duration is the largest scale's); otherwise - or where a scale exceeds what those
    // shared launches take - the small scales are sorted by one workgroup each, all in one launch.
    OrderBuildJob big[16];
    int n_big = 0, n_nonempty = 0;
    bool any_large = false, batch_ok = true;
    for (int l = 0; l < L; l++) {
      const Level &Lv = net->levels[l];
      if (Lv.n == 0) continue;
      n_nonempty++;
      if (Lv.n > order_sorted_max()) any_large = true;
      if (Lv.n > SORT_BATCH_MAX_N) batch_ok = false;
    }
    batch_ok = batch_ok && any_large && n_nonempty <= SORT_BATCH_MAX_JOBS;
    if (!batch_ok) {
      const insc_grid *sg[16];
      const int32_t *snbr[16], *soff[16];
      int32_t *sord[16], *spos[16], *sbo[16], *sbp[16];
      int ns = 0;
      int64_t nmax = 0;
      for (int l = 0; l < L; l++) {
        Level &Lv = net->levels[l];
        if (Lv.n == 0 || Lv.n > order_sorted_max()) continue;
        sg[ns] = Lv.grid;
        snbr[ns] = Lv.nbr;
        soff[ns] = l + 1 < L ? Lv.offset : nullptr;
        sord[ns] = Lv.order;
        spos[ns] = Lv.pos;
        sbo[ns] = Lv.bo_order;
        sbp[ns] = Lv.bo_pos;
        nmax = std::max(nmax, Lv.n);
        ns++;
      }
      if (ns > 0 && (rc = order_append_new_sites_both_batch(sg, snbr, soff, sord, spos, sbo, sbp, ns, nmax, s, true)))
        return rc;
    } else {
      for (int l = 0; l < L; l++) {
        Level &Lv = net->levels[l];
        if (Lv.n == 0) continue;
        big[n_big++] = OrderBuildJob{Lv.grid, Lv.nbr, l + 1 < L ? Lv.offset : nullptr, Lv.n, Lv.order, Lv.pos, Lv.bo_order, Lv.bo_pos};
      }
      if ((rc = order_build_batch(big, n_big, s))) return rc;
    }
    for (int l = 0; l < L && !batch_ok; l++) {
      Level &Lv = net->levels[l];
      if (Lv.n == 0 || Lv.n <= order_sorted_max()) continue;
      if ((rc = insc_order_build(Lv.grid, Lv.nbr, 0, Lv.n, Lv.order, stream))) return rc;
      hipLaunchKernelGGL(invert_perm_kernel, dim3(grid_for(Lv.n, 256)), dim3(256), 0, s, Lv.order, Lv.n, Lv.pos);
      if (l + 1 < L) {
        if ((rc = insc_order_by_offset(Lv.order, Lv.offset, Lv.n, Lv.bo_order, stream))) return rc;
        hipLaunchKernelGGL(invert_perm_kernel, dim3(grid_for(Lv.n, 256)), dim3(256), 0, s, Lv.bo_order, Lv.n,
                           Lv.bo_pos);
      }
      INSC_LAUNCH_CHECK();
    }
    for (int l = 0; l < L; l++) {
      net->levels[l].n_sorted = net->levels[l].n;
      if (refresh) net->levels[l].plan_valid = false;  // rebuilt below for the new order
    }
    if (refresh && (rc = accumulate_input())) return rc;
  } else {
    // An incremental frame learns the exact counts here as well: one short host round trip
    // (tens of microseconds) buys launches sized to the real number of tiles.  With the bound
    // "every new point is a new site at every scale" a coarse scale of 70 sites would be
    // launched for thousands, and idle blocks cost more than the convolution itself.
    if (P > 0) {
      INSC_HIP(hipEventSynchronize(net->ev_counts));
      if ((rc = apply_counts(net, "insc_net_forward"))) return rc;
    }
  }

  // tile plans of the 3^3 maps, shared by all the layers of a scale
  {
    TilePlanBatch batch;
    batch.n = 0;
    for (int l = 0; l < L; l++) {
      Level &Lv = net->levels[l];
      if (Lv.n <= 0) continue;
      // (a plan kept up to date by this incremental frame only needs its tile schedule redone)
      const bool keep = inc && Lv.plan_valid;
      batch.job[batch.n++] = TilePlanJob{keep ? nullptr : Lv.nbr, Lv.order, Lv.grid->d_n, Lv.n, Lv.cap, Lv.plan, Lv.tmask, Lv.sched};
      Lv.plan_valid = true;
    }
    if ((rc = build_tile_plans(batch, s))) return rc;
  }

  // ---- input layer output ------------------------------------------------------------------
  {
    Level &L0 = net->levels[0];
    const DirtyNode &din = net->dirty[net->tensors[0].dirty];
    if ((rc = launch_input_finish(net->in_sum, net->in_cnt, net->mode, tensor_ptr(net, 0), tensor_ld(net, 0), nullptr,
                                  L0.grid->d_n, L0.n_upper, C0, inc ? din.mask : nullptr, s)))
      return rc;
  }
  // ---- dirty sets, then the layers ---------------------------------------------------------
  if (net->profiling) INSC_HIP(hipEventRecord(net->ev[1], s));
  if (inc) {
    // A scale of at most DIRTY_FULL_SITES (_COARSE above the input scale) sites is recomputed whole: every set of it and of the
    // coarser scales is "all rows" (recomputing a clean row reproduces its bits).  Being all rows
    // is inherited along the program - the children of all coarse sites are all fine sites, a
    // union with everything is everything, ... - so the decoder's sets at the finer scales are
    // known to be full as well.  Such sets cost no launch and keep no mask.
    int l_full = L;
    for (int l = L - 1; l >= 0 && net->levels[l].n <= (l == 0 ? DIRTY_FULL_SITES : DIRTY_FULL_SITES_COARSE); l--) l_full = l;
    net->dirty_full.assign(net->dirty.size(), 0);
    for (size_t i = 0; i < net->dirty.size(); i++) {  // (a set's sources come before it)
      const DirtyNode &dn = net->dirty[i];
      bool full = dn.level >= l_full;
      if (dn.src0 >= 0 && net->dirty_full[(size_t)dn.src0]) full = true;
      if (dn.src1 >= 0 && net->dirty_full[(size_t)dn.src1]) full = true;
      net->dirty_full[i] = full ? 1 : 0;
    }
    // A set is also listed row by row when it is expected to stay well below its scale: from the
    // sweeps measured, d 3^3 layers turn P touched voxels into about P * (6 d - 2) dirty rows.
    // Either way every dirty row is recomputed and no other row is written: same results.
    for (int i = 0; i < (int)net->dirty.size(); i++) {
      DirtyNode &dn = net->dirty[(size_t)i];
      const Level &Lv = net->levels[dn.level];
      dn.expect_rows = P * (6 * dn.depth - 2);
      dn.compact = !net->dirty_full[(size_t)i] && dn.depth >= 1 && dn.crows && Lv.n_upper >= COMPACT_MIN_SITES &&
                   dn.expect_rows * 2 <= Lv.n_upper;
      if (net->dirty_full[(size_t)i]) continue;
      if ((rc = run_dirty_node(net, i, s))) return rc;
      if (dn.compact) {
        hipLaunchKernelGGL(dirty_compact_rows_kernel, dim3(grid_for(Lv.n_upper, 1024)), dim3(256), 0, s, dn.mask, Lv.order,
                           Lv.grid->d_n, Lv.n_upper, dn.crows, dn.ccount);
        INSC_LAUNCH_CHECK();
      }
    }
  }
  if (net->profiling) INSC_HIP(hipEventRecord(net->ev[2], s));
  for (const Op &op : net->ops)
    if ((rc = run_op(net, op, inc, s))) return rc;
  if (net->profiling) INSC_HIP(hipEventRecord(net->ev[3], s));

  // ---- output layer ------------------------------------------------------------------------
  const int64_t n_out_pts = out_all ? net->n_points + P : P;
  if (d_out && n_out_pts > 0) {
    const Tensor &To = net->tensors[net->out_tensor];
    hipLaunchKernelGGL(gather_out_kernel, dim3(grid_for(n_out_pts * To.C, 256, 1 << 16)), dim3(256), 0, s,
                       tensor_ptr(net, net->out_tensor), tensor_ld(net, net->out_tensor),
                       out_all ? net->site_of_point : sop, n_out_pts, To.C, d_out);
    INSC_LAUNCH_CHECK();
  }
  net->n_points += P;
  net->have_state = true;
  net->last_inc = inc;
  if (net->profiling) INSC_HIP(hipEventRecord(net->ev[4], s));
  // (no wait here: the host has had the site counts since the structure phase, the output rows are ready in
  // stream order, and what the caller enqueues next - a classifier on d_out - follows without a gap)
  net->ev_valid = net->profiling;
  if (h_n_sites) *h_n_sites = net->levels[0].n;
  return INSC_OK;
}

int insc_net_set_order_refresh(insc_net *net, int percent) {
  INSC_REQUIRE(net && percent >= 0, INSC_ERR_ARG, "insc_net_set_order_refresh: net is null or percent < 0");
  net->order_refresh_pct = percent;
  return INSC_OK;
}

/* Ask for residual frames (insc_net_forward_residual) before insc_net_finalize: the input of
 * every batch norm is then kept although its producer computes the batch norm itself. */
int insc_net_enable_residual(insc_net *net) {
  INSC_REQUIRE(net && !net->finalized, INSC_ERR_STATE, "insc_net_enable_residual: net is null or already finalized");
  net->keep_raw = true;
  return INSC_OK;
}

}  // extern "C"

namespace insc {

static void free_dev(void *p) {
  if (p) (void)hipFree(p);
}

// (re)allocate the frame's structures for `cap` sites per scale; nothing is preserved
static int rframe_reserve(insc_net *net, int64_t need, hipStream_t s) {
  ResidualFrame &R = net->rf;
  const int L = net->n_levels;
  if (R.levels.empty()) {
    R.levels.resize(L);
    R.pre_exist.assign(L, nullptr);
    R.nbr_pre.assign(L, nullptr);
    R.parent2.assign(L, nullptr);
    R.buffers.resize(net->buffers.size());
    R.ld.assign(net->buffers.size(), 0);
    for (size_t b = 0; b < net->buffers.size(); b++) R.buffers[b].level = net->buffers[b].level;
    // the program's buffers may have lost matrices nothing reads in a fused frame; here every
    // tensor is written, so strides come from the tensors: widest column range per buffer
    for (const Tensor &T : net->tensors) R.ld[T.buf] = std::max(R.ld[T.buf], T.col0 + T.C);
    for (size_t b = 0; b < net->buffers.size(); b++) R.buffers[b].ld = R.ld[b];
  }
  if (need <= R.cap) return INSC_OK;
  INSC_HIP(hipStreamSynchronize(s));
  const int64_t cap = (std::max<int64_t>(need + need / 2, 4096) + 31) / 32 * 32;
  int rc;
  for (int l = 0; l < L; l++) {
    Level &Lv = R.levels[l];
    if (Lv.grid) insc_grid_destroy(Lv.grid);
    Lv.grid = nullptr;
    if ((rc = insc_grid_create(cap, &Lv.grid))) return rc;
    free_dev(Lv.nbr);
    free_dev(Lv.parent);
    free_dev(Lv.offset);
    free_dev(Lv.child);
    free_dev(R.pre_exist[l]);
    free_dev(R.nbr_pre[l]);
    free_dev(R.parent2[l]);
    R.parent2[l] = nullptr;
    Lv.parent = Lv.offset = Lv.child = nullptr;
    if ((rc = dev_alloc(&Lv.nbr, (size_t)cap * 27))) return rc;
    if ((rc = dev_alloc(&R.pre_exist[l], (size_t)cap))) return rc;
    if ((rc = dev_alloc(&R.nbr_pre[l], (size_t)cap * 27))) return rc;
    if (l + 1 < L) {
      if ((rc = dev_alloc(&Lv.parent, (size_t)cap))) return rc;
      if ((rc = dev_alloc(&Lv.offset, (size_t)cap))) return rc;
      if ((rc = dev_alloc(&Lv.child, (size_t)cap * 8))) return rc;
      if ((rc = dev_alloc(&R.parent2[l], (size_t)cap))) return rc;
      Lv.child_rows = cap;
    }
    Lv.cap = cap;
  }
  free_dev(R.in_sum);
  free_dev(R.in_cnt);
  free_dev(R.chain_head);
  free_dev(R.chain_next);
  free_dev(R.sop);
  if ((rc = dev_alloc(&R.in_sum, (size_t)cap * net->in_channels))) return rc;
  if ((rc = dev_alloc(&R.in_cnt, (size_t)cap))) return rc;
  if ((rc = dev_alloc(&R.chain_head, (size_t)cap))) return rc;
  if ((rc = dev_alloc(&R.chain_next, (size_t)cap))) return rc;
  if ((rc = dev_alloc(&R.sop, (size_t)cap))) return rc;
  if ((rc = fill_i32(R.chain_head, cap, -1, s))) return rc;  // the accumulation leaves it at -1
  R.cap = cap;
  return INSC_OK;
}

static int rframe_buffers(insc_net *net, hipStream_t s) {
  ResidualFrame &R = net->rf;
  for (size_t b = 0; b < R.buffers.size(); b++) {
    Buffer &B = R.buffers[b];
    const int64_t n = R.levels[B.level].n;
    if (B.ld == 0 || n <= B.rows) continue;
    INSC_HIP(hipStreamSynchronize(s));
    free_dev(B.p);
    B.p = nullptr;
    const int64_t rows = std::max<int64_t>(n + n / 2, 256);
    int rc = dev_alloc(&B.p, (size_t)rows * B.ld);
    if (rc) return rc;
    B.rows = rows;
  }
  return INSC_OK;
}

static float *rtensor_ptr(insc_net *net, int t) {
  const Tensor &T = net->tensors[t];
  return net->rf.buffers[T.buf].p + T.col0;
}
static int64_t rtensor_ld(insc_net *net, int t) { return net->rf.buffers[net->tensors[t].buf].ld; }

// one layer of a residual frame, on all rows of the frame: every op runs on its own, except that the
// element-wise sum of a residual block is formed by the convolution before it
static int run_op_residual(insc_net *net, int index, hipStream_t s) {
  ResidualFrame &R = net->rf;
  const Op &op = net->ops[(size_t)index];
  if (op.kind == OP_BN && R.bn_done[(size_t)index]) return INSC_OK;
  const Tensor &To = net->tensors[op.out];
  const Level &Lo = R.levels[To.level];
  const int64_t n = Lo.n;
  if (n == 0 || op.kind == OP_JOIN) return INSC_OK;
  if (op.kind == OP_ADD && op.fused) return INSC_OK;  // formed by the convolution that feeds it
  const float *in0 = rtensor_ptr(net, op.in0);
  const int64_t ld0 = rtensor_ld(net, op.in0);
  // a convolution that also forms the sum of its residual block writes what the OP_ADD would
  const Op *add = op.fused_add >= 0 ? &net->ops[op.fused_add] : nullptr;
  float *out = rtensor_ptr(net, add ? add->out : op.out);
  const int64_t ld_out = rtensor_ld(net, add ? add->out : op.out);
  BnEpilogue ep;
  if (add) {
    const int other = add->in0 == op.out ? add->in1 : add->in0;
    ep.res = rtensor_ptr(net, other);
    ep.ldr = rtensor_ld(net, other);
  }
  const int li = net->tensors[op.in0].level;
  const int64_t n_in = R.levels[li].n;
  // the saved input of the layer and the saved site count of its scale
  const float *pre0 = net->tensors[op.in0].kept ? tensor_ptr(net, op.in0) : nullptr;
  const int64_t ldp0 = net->tensors[op.in0].kept ? tensor_ld(net, op.in0) : 0;
  const int64_t n_pre_in = net->levels[li].n;
  switch (op.kind) {
    case OP_SSC:
      INSC_REQUIRE(pre0, INSC_ERR_STATE, "residual frame: the input of a convolution was not kept");
      {
        // the batch norm that reads the result (the layer's own or, with the sum folded in, the sum's) rides
        // in the epilogue when the layer runs as one launch
        const Op &tail = add ? *add : op;
        const Op *bn = tail.fused_bn >= 0 ? &net->ops[(size_t)tail.fused_bn] : nullptr;
        if (bn && bn->bn_w && n_pre_in > 0 && net->tensors[bn->in0].kept && net->tensors[bn->out].kept &&
            conv_two_sources_ok(MAP_NBR, 27, in0, ld0, pre0, ldp0, n_pre_in, op.Cin, 1)) {
          ep.w = bn->bn_w;
          ep.b = bn->bn_b;
          ep.leak = bn->leak;
          ep.out2 = rtensor_ptr(net, bn->out);
          ep.ld2 = rtensor_ld(net, bn->out);
          ep.pre_exist = R.pre_exist[To.level];
          ep.pre_in = tensor_ptr(net, bn->in0);
          ep.ld_pin = tensor_ld(net, bn->in0);
          ep.pre_out = tensor_ptr(net, bn->out);
          ep.ld_pout = tensor_ld(net, bn->out);
          R.bn_done[(size_t)tail.fused_bn] = 1;
        }
      }
      return incre_conv_ssc(in0, ld0, pre0, ldp0, n_pre_in, out, ld_out, op.W, op.Wp, op.bias, Lo.nbr,
                            R.nbr_pre[To.level], n, op.Cin, op.Cout, ep, s);
    case OP_NIN:
      return launch_conv(in0, ld0, n_in, out, ld_out, op.W, op.Wp, op.bias, nullptr, nullptr, MAP_IDENTITY, 1, nullptr,
                         nullptr, n, op.Cin, op.Cout, nullptr, nullptr, s, ep);
    case OP_CONV:
      return launch_conv(in0, ld0, n_in, out, ld_out, op.W, op.Wp, op.bias, R.levels[li].child, nullptr, MAP_NBR, 8,
                         nullptr, nullptr, n, op.Cin, op.Cout, nullptr, nullptr, s, ep);
    case OP_DECONV:
      INSC_REQUIRE(pre0, INSC_ERR_STATE, "residual frame: the input of a deconvolution was not kept");
      return incre_deconv_down2(in0, ld0, n_in, pre0, ldp0, n_pre_in, out, ld_out, op.W, op.Wp, op.bias, Lo.parent,
                                Lo.offset, R.pre_exist[li], R.pre_exist[To.level], n, op.Cin, op.Cout, ep.res, ep.ldr, s,
                                R.parent2[To.level]);
    case OP_BN:
      INSC_REQUIRE(pre0 && net->tensors[op.out].kept, INSC_ERR_STATE,
                   "residual frame: the input of a batch norm was not kept (insc_net_enable_residual before finalize)");
      return launch_incre_bn(in0, ld0, out, ld_out, op.mean, op.var, op.gamma, op.beta, op.eps, op.leak, op.bn_w,
                             op.bn_b, R.pre_exist[To.level], pre0, ldp0, tensor_ptr(net, op.out),
                             tensor_ld(net, op.out), n, op.Cout, s);
    case OP_ADD:
      return launch_add(in0, ld0, rtensor_ptr(net, op.in1), rtensor_ld(net, op.in1), out, ld_out, nullptr, nullptr, n,
                        op.Cout, nullptr, s);
    case OP_COPY:
      return launch_add(in0, ld0, nullptr, 0, out, ld_out, nullptr, nullptr, n, op.Cout, nullptr, s);
  }
  set_error("run_op_residual: unknown op kind %d", op.kind);
  return INSC_ERR_STATE;
}

}  // namespace insc

extern "C" {

/* One residual frame, the reference's own incremental mode (Incre_* operators; the module
 * tree's increment="residual"): the frame's points form a site set of their own, features are
 * differences to the state saved by the last full / exact incremental frame, and that state
 * is left as it is.  d_out: [P, C] rows of the output tensor, saved value + residual, one per
 * point of the frame.  h_n_sites (nullable): sites of the frame at the input scale.
 * Needs insc_net_enable_residual before insc_net_finalize.  The call returns once the frame's
 * site counts are known; the layers may still be running on the stream. */
int insc_net_forward_residual(insc_net *net, const int32_t *d_coords, int coord_cols, const float *d_feats, int64_t P,
                              float *d_out, int64_t *h_n_sites, void *stream) {
  INSC_REQUIRE(net && net->finalized, INSC_ERR_STATE, "insc_net_forward_residual: net is not finalized");
  INSC_REQUIRE(net->keep_raw, INSC_ERR_STATE,
               "insc_net_forward_residual: call insc_net_enable_residual before insc_net_finalize");
  INSC_REQUIRE(net->have_state, INSC_ERR_STATE, "insc_net_forward_residual: residual frame before any full frame");
  INSC_REQUIRE(P >= 0 && (P == 0 || (d_coords && d_feats)) && (coord_cols == 3 || coord_cols == 4), INSC_ERR_ARG,
               "insc_net_forward_residual: bad arguments");
  if (h_n_sites) *h_n_sites = 0;
  if (P == 0) return INSC_OK;
  hipStream_t s = (hipStream_t)stream;
  const int L = net->n_levels;
  const int C0 = net->in_channels;
  ResidualFrame &R = net->rf;
  int rc;
  if ((rc = rframe_reserve(net, P, s))) return rc;

  // ---- the frame's own site set --------------------------------------------------------------
  {
    insc_grid *gs[16];
    int32_t *chi[16];
    int64_t nchi[16];
    for (int l = 0; l < L; l++) {
      gs[l] = R.levels[l].grid;
      chi[l] = l + 1 < L ? R.levels[l].child : nullptr;
      nchi[l] = P * 8;  // a scale has at most P sites
    }
    if ((rc = grid_clear_batch(gs, chi, nchi, L, R.in_sum, (int64_t)sizeof(float) * P * C0, s))) return rc;
  }
  INSC_HIP(hipMemsetAsync(R.in_cnt, 0, sizeof(int32_t) * (size_t)P, s));
  const unsigned nb = grid_for(P, 256);
  // the inserts of all scales at once, as in an exact frame; the counts arrive in host memory
  net->frame_id = net->frame_id == INT32_MAX ? 1 : net->frame_id + 1;
  {
    FrameInsertLevel fl[16];
    for (int l = 0; l < L; l++) {
      Level &Lv = R.levels[l];
      Lv.grid->n_upper = 0;
      fl[l] = FrameInsertLevel{Lv.grid, Lv.parent, Lv.offset, Lv.child};
    }
    if ((rc = frame_insert_levels(fl, L, d_coords, coord_cols, P, net->d_bad, net->frame_id, R.sop, net->h_counts, s)))
      return rc;
    INSC_HIP(hipEventRecord(net->ev_counts, s));
  }
  hipLaunchKernelGGL(chain_push_kernel, dim3(nb), dim3(256), 0, s, R.sop, P, R.chain_head, R.chain_next);
  hipLaunchKernelGGL(chain_sum_kernel, dim3(nb), dim3(256), 0, s, d_feats, C0, R.sop, P, R.chain_head, R.chain_next,
                     R.in_sum, R.in_cnt, (uint8_t *)nullptr, (uint8_t *)nullptr, (const int32_t *)nullptr);
  INSC_LAUNCH_CHECK();
  {
    // the neighbour maps of all scales in one launch
    const insc_grid *grids[16];
    int32_t *nbrs[16];
    for (int l = 0; l < L; l++) {
      grids[l] = R.levels[l].grid;
      nbrs[l] = R.levels[l].nbr;
    }
    if ((rc = ssc3_new_sites_batch(grids, nbrs, L, P, s))) return rc;
    // the links to the saved site set, all scales at once
    const insc_grid *pre[16];
    const int32_t *par[16];
    for (int l = 0; l < L; l++) {
      pre[l] = net->levels[l].grid;
      par[l] = R.levels[l].parent;
    }
    if ((rc = incre_links_batch(grids, pre, par, R.pre_exist.data(), R.nbr_pre.data(), R.parent2.data(), L, P, s)))
      return rc;
  }
  // the exact site counts size every later launch (one short wait, as in an exact frame)
  INSC_HIP(hipEventSynchronize(net->ev_counts));
  INSC_REQUIRE(net->h_counts[2 * L] != net->frame_id, INSC_ERR_COORD,
               "insc_net_forward_residual: a coordinate is outside 0..65535 (batch 0..32767)");
  for (int l = 0; l < L; l++) {
    Level &Lv = R.levels[l];
    Lv.n = Lv.n_upper = net->h_counts[2 * l];
    Lv.grid->n_exact = Lv.grid->n_upper = Lv.n;
    const int err = net->h_counts[2 * l + 1];
    INSC_REQUIRE(!(err & 1), INSC_ERR_COORD,
                 "insc_net_forward_residual: a coordinate is outside 0..65535 (batch 0..32767)");
    INSC_REQUIRE(!(err & 2), INSC_ERR_CAPACITY, "insc_net_forward_residual: capacity of scale %d exceeded", l);
  }
  if ((rc = rframe_buffers(net, s))) return rc;
  // ---- input layer, layers, output layer -----------------------------------------------------------
  const int64_t n0 = R.levels[0].n;
  if (net->mode == 0) {
    if ((rc = launch_input_finish(R.in_sum, R.in_cnt, 0, rtensor_ptr(net, 0), rtensor_ld(net, 0), nullptr, nullptr, n0,
                                  C0, nullptr, s)))
      return rc;
  } else if ((rc = insc_incre_input(R.in_sum, R.in_cnt, net->mode, R.pre_exist[0], tensor_ptr(net, 0),
                                    tensor_ld(net, 0), net->in_cnt, rtensor_ptr(net, 0), rtensor_ld(net, 0), n0, C0,
                                    stream))) {
    return rc;
  }
  R.bn_done.assign(net->ops.size(), 0);
  for (int i = 0; i < (int)net->ops.size(); i++)
    if ((rc = run_op_residual(net, i, s))) return rc;
  if (d_out) {
    const Tensor &To = net->tensors[net->out_tensor];
    if ((rc = insc_incre_output(rtensor_ptr(net, net->out_tensor), rtensor_ld(net, net->out_tensor),
                                tensor_ptr(net, net->out_tensor), tensor_ld(net, net->out_tensor), R.pre_exist[0],
                                R.sop, P, To.C, d_out, stream)))
      return rc;
  }
  if (h_n_sites) *h_n_sites = n0;
  return INSC_OK;
}

/* Inspection: device pointer, row stride and row count of a tensor (valid until the next
 * frame that grows the scene past the reserved capacity). */
int insc_net_tensor_view(insc_net *net, int tensor, float **d_ptr, int64_t *ld, int64_t *rows, int *channels) {
  INSC_REQUIRE(net && net->finalized && tensor >= 0 && tensor < (int)net->tensors.size(), INSC_ERR_ARG,
               "insc_net_tensor_view: bad arguments");
  INSC_REQUIRE(net->tensors[tensor].kept, INSC_ERR_STATE,
               "insc_net_tensor_view: tensor %d is not kept (its only reader, a batch norm, is computed by its producer)",
               tensor);
  if (d_ptr) *d_ptr = tensor_ptr(net, tensor);
  if (ld) *ld = tensor_ld(net, tensor);
  if (rows) *rows = net->levels[net->tensors[tensor].level].n;
  if (channels) *channels = net->tensors[tensor].C;
  return INSC_OK;
}

int insc_net_profile(insc_net *net, int enable, float *h_ms4) {
  INSC_REQUIRE(net, INSC_ERR_ARG, "insc_net_profile: null net");
  if (h_ms4) {
    INSC_REQUIRE(net->ev_valid, INSC_ERR_STATE, "insc_net_profile: no frame has been timed yet");
    INSC_HIP(hipEventSynchronize(net->ev[4]));
    for (int i = 0; i < 4; i++) INSC_HIP(hipEventElapsedTime(h_ms4 + i, net->ev[i], net->ev[i + 1]));
  }
  if (enable && !net->ev[0])
    for (int i = 0; i < 5; i++) INSC_HIP(hipEventCreate(&net->ev[i]));
  net->profiling = enable != 0;
  if (!enable) net->ev_valid = false;
  return INSC_OK;
}

/* The dirty sets of the last exact incremental frame: for set i (program order; i < *h_n_sets
 * <= max_sets) h_level[i] = its scale, h_kind[i] = how it is derived (0 input, 1 dilated by a 3^3
 * layer, 2 parents, 3 children, 4 union) and h_rows[i] = its number of rows.  Synchronises. */
int insc_net_dirty_counts(insc_net *net, int max_sets, int *h_n_sets, int *h_level, int *h_kind, int64_t *h_rows,
                          void *stream) {
  INSC_REQUIRE(net && net->finalized && h_n_sets && h_level && h_kind && h_rows && max_sets >= 0, INSC_ERR_ARG,
               "insc_net_dirty_counts: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  const int ns = std::min<int>(max_sets, (int)net->dirty.size());
  *h_n_sets = ns;
  if (ns == 0) return INSC_OK;
  void *ws;
  int rc = workspace(WS_API, s, sizeof(unsigned long long) * (size_t)ns, &ws);
  if (rc) return rc;
  unsigned long long *d = (unsigned long long *)ws;
  INSC_HIP(hipMemsetAsync(d, 0, sizeof(unsigned long long) * (size_t)ns, s));
  for (int i = 0; i < ns; i++) {
    const DirtyNode &dn = net->dirty[i];
    const int64_t n = net->levels[dn.level].n;
    h_level[i] = dn.level;
    h_kind[i] = dn.kind;
    if (i < (int)net->dirty_full.size() && net->dirty_full[(size_t)i]) continue;  // every row: filled in below
    if (n > 0 && dn.mask) {
      hipLaunchKernelGGL(count_mask_kernel, dim3(grid_for(n, 256, 1024)), dim3(256), 0, s, dn.mask, n, d + i);
      INSC_LAUNCH_CHECK();
    }
  }
  std::vector<unsigned long long> h((size_t)ns);
  INSC_HIP(hipMemcpyAsync(h.data(), d, sizeof(unsigned long long) * (size_t)ns, hipMemcpyDeviceToHost, s));
  INSC_HIP(hipStreamSynchronize(s));
  for (int i = 0; i < ns; i++)
    h_rows[i] = (i < (int)net->dirty_full.size() && net->dirty_full[(size_t)i]) ? net->levels[net->dirty[i].level].n
                                                                                : (int64_t)h[(size_t)i];
  return INSC_OK;
}

/* What every convolution of the last completed frame (insc_net_forward) worked on - diagnostics for
 * the benchmark's flop accounting.  For convolution i in program order (i < *h_n_ops <= max_ops):
 * h_kind[i] (0 3^3 submanifold, 2 strided, 3 transposed, 4 1x1), h_level[i] = scale of its output,
 * h_cin / h_cout, and over the tiles it computed in that frame (all of them after a full frame, the
 * flagged ones or the listed rows after an incremental one) h_rows[i] = output rows, h_rules[i] =
 * rules, h_slots[i] = 32 x (offsets used per tile): useful multiply-adds = rules x Cin x Cout, the
 * matrix cores are issued slots x Cin x Cout (Cin rounded up to 32).  Synchronises. */
int insc_net_frame_work(insc_net *net, int max_ops, int *h_n_ops, int *h_kind, int *h_level, int *h_cin, int *h_cout,
                        int64_t *h_rows, int64_t *h_rules, int64_t *h_slots, void *stream) {
  INSC_REQUIRE(net && net->finalized && h_n_ops && h_kind && h_level && h_cin && h_cout && h_rows && h_rules && h_slots &&
                   max_ops >= 0, INSC_ERR_ARG, "insc_net_frame_work: bad arguments");
  INSC_REQUIRE(net->have_state, INSC_ERR_STATE, "insc_net_frame_work: no frame has run");
  hipStream_t s = (hipStream_t)stream;
  std::vector<const Op *> convs;
  for (const Op &op : net->ops)
    if (!op.fused && (op.kind == OP_SSC || op.kind == OP_CONV || op.kind == OP_DECONV || op.kind == OP_NIN))
      convs.push_back(&op);
  const int nc = std::min<int>(max_ops, (int)convs.size());
  *h_n_ops = nc;
  if (nc == 0) return INSC_OK;
  void *ws;
  int rc = workspace(WS_API, s, sizeof(unsigned long long) * 3 * (size_t)nc, &ws);
  if (rc) return rc;
  unsigned long long *acc = (unsigned long long *)ws;
  INSC_HIP(hipMemsetAsync(acc, 0, sizeof(unsigned long long) * 3 * (size_t)nc, s));
  for (int i = 0; i < nc; i++) {
    const Op &op = *convs[(size_t)i];
    const Tensor &To = net->tensors[op.out];
    const Level &Lo = net->levels[To.level];
    const DirtyNode *d = net->last_inc && !net->dirty_full[(size_t)To.dirty] ? &net->dirty[To.dirty] : nullptr;
    h_kind[i] = op.kind;
    h_level[i] = To.level;
    h_cin[i] = op.Cin;
    h_cout[i] = op.Cout;
    if (Lo.n <= 0) continue;
    const int32_t *map0 = nullptr, *map1 = nullptr, *rows = Lo.order, *d_n = Lo.grid->d_n;
    const uint8_t *flags = d ? d->tflag : nullptr;
    int mode = MAP_NBR, K = 27;
    int64_t n = Lo.n;
    if (op.kind == OP_SSC) {
      map0 = Lo.nbr;
      if (d && d->compact) {
        rows = d->crows;
        d_n = d->ccount;
        flags = nullptr;
      }
    } else if (op.kind == OP_NIN) {
      mode = MAP_IDENTITY;
      K = 1;
    } else if (op.kind == OP_CONV) {
      map0 = net->levels[To.level - 1].child;
      K = 8;
    } else {
      map0 = Lo.parent;
      map1 = Lo.offset;
      mode = MAP_PARENT;
      K = 8;
      rows = Lo.bo_order;
      flags = d ? d->tflag_bo : nullptr;
    }
    hipLaunchKernelGGL(conv_work_kernel, dim3(grid_for(cdiv(n, 32), 4)), dim3(256), 0, s, map0, map1, mode, K, rows, d_n, n,
                       flags, acc + 3 * i);
    INSC_LAUNCH_CHECK();
  }
  std::vector<unsigned long long> h(3 * (size_t)nc);
  INSC_HIP(hipMemcpyAsync(h.data(), acc, sizeof(unsigned long long) * h.size(), hipMemcpyDeviceToHost, s));
  INSC_HIP(hipStreamSynchronize(s));
  for (int i = 0; i < nc; i++) {
    h_rows[i] = (int64_t)h[3 * (size_t)i];
    h_rules[i] = (int64_t)h[3 * (size_t)i + 1];
    h_slots[i] = (int64_t)h[3 * (size_t)i + 2];
  }
  return INSC_OK;
}

int insc_net_counts(insc_net *net, int64_t *h_sites_per_level, int64_t *h_points) {
  INSC_REQUIRE(net && net->finalized, INSC_ERR_ARG, "insc_net_counts: bad arguments");
  if (h_sites_per_level)
    for (int l = 0; l < net->n_levels; l++) h_sites_per_level[l] = net->levels[l].n;
  if (h_points) *h_points = net->n_points;
  return INSC_OK;
}

}  // extern "C"
