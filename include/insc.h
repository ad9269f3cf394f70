/*
 * insc.h - C ABI of the MI355X (gfx950) sparse-convolution inference library.
 *
 * This is the drop-in boundary for the reference's native extension `sparseconvnet.SCN`
 * (reference: sparseconvnet/SCN/pybind.cpp:153-258, sparseconvnet/SCN/sparseconvnet.h).
 * The reference passes at::Tensor objects; here every argument is a plain pointer or size.
 * Unless a parameter name starts with h_ it is a DEVICE pointer valid on the device bound
 * with insc_init.  Every function returns 0 on success or a negative INSC_ERR_* code and
 * never aborts the process (the reference calls assert/abort/exit on failure,
 * CUDA/CUDPPWrapper.hpp:17-27); insc_last_error() gives the message of the calling thread's
 * last failure.  `stream` is a hipStream_t passed as void* (NULL = the default stream);
 * work is enqueued asynchronously on it and functions that hand a value back to the host
 * (h_ arguments) synchronise that stream first.
 *
 * Feature matrices are row-major float32 with an explicit row stride `ld` (in floats), so
 * a layer can read or write a column slice of a wider matrix (channel concatenation without
 * a copy).  Site ids are int32; -1 means "no site".  Coordinates are int32 quadruples
 * (x, y, z, batch) with 0 <= x,y,z <= 65535 and 0 <= batch <= 32767.
 *
 * Row subsets: the feature functions take `rows` (int32 list of output rows to compute, or
 * NULL for rows 0..n_rows-1), `d_n_rows` (device int32 holding the list length, or NULL to
 * use n_rows) and `n_rows` (the length, or an upper bound on *d_n_rows used to size the
 * launch).  Rows not listed are left untouched: this is what the incremental path uses to
 * recompute only dirty rows.
 */
#ifndef INSC_H
#define INSC_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define INSC_OK 0
#define INSC_ERR_ARG -1      /* bad argument (null pointer, negative size, unsupported shape) */
#define INSC_ERR_HIP -2      /* a HIP runtime call failed; message holds hipGetErrorString */
#define INSC_ERR_CAPACITY -3 /* a fixed-capacity structure would overflow */
#define INSC_ERR_STATE -4    /* call order violated (e.g. library not initialised) */
#define INSC_ERR_COORD -5    /* a coordinate is outside the representable range */

typedef struct insc_grid insc_grid;

/* Binds the library to a HIP device (hipSetDevice) and checks that it is a gfx950 part.
 * No counterpart in the reference, which uses whatever device torch selected. */
int insc_init(int device);
const char *insc_last_error(void);
const char *insc_version(void);

/* ---------------------------------------------------------------------------------------
 * Hash grid: the set of active sites of one spatial scale.  Replaces the reference's
 * Multival_Point_Hashtable<3> over the CUDPP cuckoo hash (CUDA/CUDPPWrapper.hpp:736-1010)
 * and GPU_SparseGrid (Metadata/Metadata.h:114-122).  Open addressing on 64-bit packed keys.
 * Sites are numbered by first appearance in the inserted coordinate list (the numbering of
 * the reference's CPU path, Metadata/IOLayersRules.h:69-79) and numbering is append-only:
 * a later insert never renumbers existing sites.
 * ------------------------------------------------------------------------------------- */
int insc_grid_create(int64_t capacity_sites, insc_grid **out);
int insc_grid_destroy(insc_grid *g);
/* Forget all sites, keep the allocation (reference: Metadata<D>::clear, Metadata.cpp:68-75). */
int insc_grid_clear(insc_grid *g, void *stream);
/* Grow so that capacity_sites fit; rehashes the existing sites, ids unchanged. */
int insc_grid_reserve(insc_grid *g, int64_t capacity_sites, void *stream);
/* Insert P coordinates (duplicates allowed).  d_site_of_point[p] receives the site of row p.
 * h_n_sites (nullable, host) receives the site count after the insert (synchronises).
 * A coordinate outside the representable range gets site -1 and the next synchronising call on
 * the grid returns INSC_ERR_COORD once; every other row of the call is inserted and the grid stays
 * usable.
 * Replaces HashInputPointClouds + InsertAndCompactPointCloud (CUDPPWrapper.hpp:668-686,
 * 766-796; kernels CUDPPWrapper.cu:72-100,212-231). */
int insc_grid_insert(insc_grid *g, const int32_t *d_coords4, int64_t P, int32_t *d_site_of_point, int64_t *h_n_sites,
                     void *stream);
/* The points of a frame inserted at ALL scales of a network at once: grids[0] takes the points
 * (d_coords: int32 [P, coord_cols], coord_cols 3 or 4), grids[l] the cells coordinate >> l, and for
 * every scale l < n_scales - 1 the link to the next coarser one is filled in for the sites this call
 * adds: d_parent[l][i] = coarse site, d_offset[l][i] = (x&1)*4 + (y&1)*2 + (z&1), d_child[l][parent*8 +
 * offset] = i (rows of new coarse sites must have been filled with -1 by the caller).  Same grids, ids
 * and links as insc_grid_insert on grids[0] followed by insc_rulebook_down2 scale by scale - the
 * reference's order of construction (Metadata.cpp inputLayer, then getRuleBook / ConvolutionRules.h:
 * 344-380 per scale) - in 3 to 7 kernel launches for any number of scales: a site that is new at scale l
 * has only new sites below it, so the ids that chain hands out follow the smallest row of the point
 * list that falls into each new cell, which every scale can work out from the points themselves.
 * d_site_of_point: [P] site at grids[0].  h_n_sites (nullable): [n_scales] site counts after the call.
 * Differences to the chain: a frame is all or nothing (one bad coordinate: INSC_ERR_COORD and nothing
 * is inserted anywhere), and no grid grows (every grid must have room for P more sites:
 * INSC_ERR_CAPACITY otherwise; insc_grid_reserve beforehand).  The call synchronises the stream. */
int insc_grid_insert_scales(insc_grid *const *grids, int32_t *const *d_parent, int32_t *const *d_offset,
                            int32_t *const *d_child, int n_scales, const int32_t *d_coords, int coord_cols, int64_t P,
                            int32_t *d_site_of_point, int64_t *h_n_sites, void *stream);
/* insc_grid_insert for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it).  No counterpart in the reference.  Same result
 * as insc_grid_insert, with two limits: at most 16384 points per call (INSC_ERR_CAPACITY beyond),
 * and the grid is never grown - the host-side bound "sites so far + P" must fit the capacity
 * (INSC_ERR_CAPACITY otherwise; reserve beforehand).  It calls no hipMalloc / hipFree: the per-row
 * scratch is a 64 KB array in the library's device image, one per GPU, shared by all calls on that
 * GPU - calls that overlap on one GPU (different streams or threads) race; calls on one stream do
 * not.  Nothing in the scratch has to survive or be cleared between calls.  With h_n_sites == NULL
 * the call only enqueues two kernels; with it, it copies the count back and synchronises. */
int insc_grid_insert_noalloc(insc_grid *g, const int32_t *d_coords4, int64_t P, int32_t *d_site_of_point,
                             int64_t *h_n_sites, void *stream);
/* d_site[q] = site id of coordinate q, or -1.  Replaces Multival retrieve +
 * _dMultivalHashGetValue (CUDPPWrapper.cu:144-160), whose miss value is 0xFFFFFFFF. */
int insc_grid_query(const insc_grid *g, const int32_t *d_coords4, int64_t Q, int32_t *d_site, void *stream);
/* Site count (synchronises `stream` if an insert is still in flight). */
int insc_grid_size(insc_grid *g, int64_t *h_n_sites, void *stream);
/* Device pointer to the [capacity,4] coordinate table; rows 0..n-1 are valid
 * (reference: getAllPoints, read by Metadata<D>::getSpatialLocations, Metadata.cpp:793-821). */
const int32_t *insc_grid_coords(const insc_grid *g);
/* Device pointer to the int32 site counter. */
const int32_t *insc_grid_count_ptr(const insc_grid *g);
int64_t insc_grid_capacity(const insc_grid *g);

/* ---------------------------------------------------------------------------------------
 * Rulebooks.
 * ------------------------------------------------------------------------------------- */
/* Submanifold 3x3x3 neighbour map for sites [first, first+n): d_nbr[o*27+k] = id of the
 * site at coordinate(o) + (dx,dy,dz), k = (dx+1)*9 + (dy+1)*3 + (dz+1), or -1.  With
 * patch_reverse != 0 it also writes d_nbr[j*27 + 26-k] = o for every neighbour j found, which
 * brings the rows of older sites up to date after an append.  Replaces
 * SubmanifoldBuildObject (CUDA/SubmanifoldRules_cuda.cpp:38-228; kernels
 * SubmanifoldRules_cuda.cu:45-77,91-114) - same relation and offset numbering, kept as a
 * dense map instead of 27 compacted lists. */
int insc_rulebook_ssc3(const insc_grid *g, int64_t first, int64_t n, int32_t *d_nbr, int patch_reverse, void *stream);
/* The reference's list form of the same rulebook (RuleBook = 27 lists of (in,out) pairs,
 * Metadata/Metadata.h:86): d_counts[k] pairs for offset k, lists back to back in d_pairs,
 * each in ascending `out` order.  h_total (nullable) receives the pair count. */
int insc_rulebook_pairs(const int32_t *d_nbr, int64_t N, int K, int32_t *d_counts, int32_t *d_pairs,
                        int64_t pairs_capacity, int64_t *h_total, void *stream);
/* Size-2 stride-2 rulebook for fine sites [first, first+n): inserts coordinate>>1 into the
 * coarse grid, d_parent[i] = coarse site, d_offset[i] = (x&1)*4 + (y&1)*2 + (z&1), and if
 * d_child != NULL, d_child[parent*8 + offset] = i (rows of new coarse sites must have been
 * filled with -1 by the caller; child_rows = rows allocated for d_child, which must cover the
 * coarse grid's capacity).  Replaces
 * Convolution_InputSgToRulesAndOutputSg_FastDownSampleMode (Metadata/ConvolutionRules.h:344-380,
 * kernel SubmanifoldRules_cuda.cu:744-780). */
int insc_rulebook_down2(const insc_grid *fine, insc_grid *coarse, int64_t first, int64_t n, int32_t *d_parent,
                        int32_t *d_offset, int32_t *d_child, int64_t child_rows, void *stream);
/* A processing order for the sites first..first+n-1, written to d_order[first..first+n): a
 * permutation of those ids that puts sites of one 64^3 block with the same neighbour pattern
 * next to each other, so that row tiles of the convolution kernel skip whole filter offsets.
 * Results of the convolution do not depend on it.  No counterpart in the reference (its chunk
 * builder, SubmanifoldRules_cuda.cpp:572-1112, serves the same purpose for its
 * shared-memory kernel). */
int insc_order_build(const insc_grid *g, const int32_t *d_nbr, int64_t first, int64_t n, int32_t *d_order,
                     void *stream);

/* d_out = the sites of d_order[0..n) (or 0..n-1 if d_order is NULL) regrouped by their
 * offset inside the parent cell (d_offset[site], 0..7), keeping the given order within a
 * group.  A row tile of the deconvolution then uses a single weight slice.  No counterpart in
 * the reference (its rulebook is already split by offset, Metadata/Metadata.h:86). */
int insc_order_by_offset(const int32_t *d_order, const int32_t *d_offset, int64_t n, int32_t *d_out, void *stream);

/* Both orders and their inverses for n_scales (1..8) scales at once, the radix passes of all scales
 * in the same launches: for scale i over its sites 0..n[i]-1 (1 <= n[i] <= 262144),
 *   d_order[i]   = what insc_order_build(grids[i], d_nbr[i], 0, n[i]) gives,  d_pos[i][d_order[i][t]] = t,
 * and, where d_offset[i] is not NULL,
 *   d_bo_order[i] = what insc_order_by_offset(d_order[i], d_offset[i], n[i]) gives, d_bo_pos[i] its inverse.
 * Same results as the two calls scale by scale (both are stable sorts of the same keys), in about a
 * third of the launches.  No counterpart in the reference. */
int insc_order_build_scales(const insc_grid *const *grids, const int32_t *const *d_nbr, const int32_t *const *d_offset,
                            const int64_t *n, int n_scales, int32_t *const *d_order, int32_t *const *d_pos,
                            int32_t *const *d_bo_order, int32_t *const *d_bo_pos, void *stream);

/* The sites added by the grid's most recent insert - [count before it, count) - appended to the grid's
 * processing order in ONE launch (one workgroup, a radix sort in shared memory): d_order[first..count) =
 * those sites sorted among themselves by the key of insc_order_build (what that call gives for the same
 * range), equal keys in id order;
 * d_pos (nullable) the inverse over the same range.  With d_offset (position inside the parent cell,
 * from insc_rulebook_down2) also d_bo_order / d_bo_pos: the same sites grouped by that position, each
 * group in the sequence of d_order.  d_nbr: the grid's 27-neighbour map, up to date for the new sites.
 * More than 8192 new sites keep their id order (every order gives the same results; insc_order_build
 * sorts any number).  n_new_upper: a host-side upper bound of the number of new sites (0: nothing to
 * do); the counts themselves are read on the device.  No counterpart in the reference. */
int insc_order_append(const insc_grid *g, const int32_t *d_nbr, const int32_t *d_offset, int32_t *d_order,
                      int32_t *d_pos, int32_t *d_bo_order, int32_t *d_bo_pos, int64_t n_new_upper, void *stream);

/* ---------------------------------------------------------------------------------------
 * Feature kernels.
 * ------------------------------------------------------------------------------------- */
/* Output-stationary sparse convolution over a neighbour map:
 *   out[o,:] = bias + sum_k  in[nbr[o*K+k], :] . W[k]      (terms with nbr = -1 skipped)
 * K = 27 with an insc_rulebook_ssc3 map is SubmanifoldConvolution_updateOutput
 * (CUDA/Convolution.cpp:152-218); K = 8 with a child map is Convolution_updateOutput for
 * size 2 / stride 2 (CUDA/Convolution.cpp:52-81); K = 1 with d_nbr = NULL (identity map) is
 * NetworkInNetwork_updateOutput (CUDA/NetworkInNetwork.cpp:9-25).  d_W is [K,Cin,Cout]; d_Wp
 * (nullable) is the same weights packed by insc_conv_pack_weights - give it to skip the
 * per-call packing (then d_W may be NULL when Cin is a multiple of 16).
 * n_in_rows = rows of d_in (the gather is bounds-checked against it; n_in_rows*ld_in*4 must stay
 * below 4 GB).  h_muladds (nullable) receives the multiply-add count the reference returns
 * (synchronises). */
int insc_conv_nbr(const float *d_in, int64_t ld_in, int64_t n_in_rows, float *d_out, int64_t ld_out,
                  const float *d_W, const float *d_Wp, const float *d_bias, const int32_t *d_nbr, int K,
                  const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                  double *h_muladds, void *stream);
/* Weights in the operand layout of the matrix-core kernel (no counterpart in the reference,
 * whose kernels stage W[k] through shared memory per launch, CUDA/Convolution.cu:81-223).
 * insc_conv_packed_floats gives the size of d_Wp in floats. */
int64_t insc_conv_packed_floats(int K, int Cin, int Cout);
int insc_conv_pack_weights(const float *d_W, int K, int Cin, int Cout, float *d_Wp, void *stream);
/* Tile plan of a 3^3 neighbour map for one processing order (no counterpart in the reference;
 * its chunk rulebook, SubmanifoldRules_cuda.cpp:572-1112, plays this role for its kernel):
 * d_plan[k*plan_ld + p] = d_nbr[d_order[p]*27 + k] for p < n_rows and -1 up to the next multiple of
 * 32; d_tmask[t] = bit k set if some row of tile t (positions 32t..32t+31) has neighbour k.
 * d_sched (nullable) = the tiles by falling number of neighbours in use (plan_ld/32 entries), then
 * the groups of four consecutive tiles by falling number of neighbours any of the four uses: the
 * orders in which the persistent kernels of wide layers take them.
 * plan_ld >= n_rows rounded up to a multiple of 32; d_plan holds 27*plan_ld int32, d_tmask
 * plan_ld/32 entries, d_sched plan_ld/32 + plan_ld/128 + 1.  d_order NULL = identity.  Rebuild after the map or the order changed. */
int insc_plan_build(const int32_t *d_nbr, const int32_t *d_order, const int32_t *d_n_rows, int64_t n_rows,
                    int64_t plan_ld, int32_t *d_plan, uint32_t *d_tmask, int32_t *d_sched, void *stream);
/* insc_conv_nbr for K = 27 over the rows d_order[0..n_rows) with their tile plan: same result
 * (bit for bit), without the per-launch staging of the site-indexed map.  d_sched may be NULL. */
int insc_conv_ssc_plan(const float *d_in, int64_t ld_in, int64_t n_in_rows, float *d_out, int64_t ld_out,
                       const float *d_W, const float *d_Wp, const float *d_bias, const int32_t *d_nbr,
                       const int32_t *d_plan, int64_t plan_ld, const uint32_t *d_tmask, const int32_t *d_sched,
                       const int32_t *d_order, const int32_t *d_n_rows, int64_t n_rows, int Cin, int Cout,
                       void *stream);
/* Launch policy of a 3^3 layer of 64..159 input channels with a tile schedule: by default one block per
 * (tile, 32-column output block) pair; persistent blocks once it has at least `units` pairs (off by
 * default: the one-block-per-pair kernel measures faster at every size); with at least `units` (four
 * consecutive tiles, output block) pairs (default 896) the kernel whose blocks share the weight tiles
 * through LDS.  Same bits in all cases: tuning and test knobs with no counterpart in the reference. */
int insc_conv_set_persistent_min_units(int64_t units);
int insc_conv_set_shared_weights_min_units(int64_t units);
/* ... and between the two, from `units` (tile, output block) pairs up (default 2400; half as many again
 * for more than 64 input channels), on the kernel that gives every pair a wavefront of its own.  Same
 * bits again. */
int insc_conv_set_wavefront_per_unit_min_units(int64_t units);
/* A 3^3 layer with at most 32 input and 32 output channels runs, from `tiles` 32-row tiles up
 * (default 4096, i.e. 131k sites), on persistent blocks that keep the whole filter in LDS; below,
 * one wavefront per tile.  Same bits in both cases: a tuning and test knob like the two above. */
int insc_conv_set_filter_lds_min_tiles(int64_t tiles);
/* Size-2 stride-2 deconvolution: out[i,:] = bias + in[parent[i],:] . W[offset[i]]
 * (Deconvolution_updateOutput, CUDA/Deconvolution.cpp:28-58: the convolution's rules with
 * the roles of input and output swapped). */
int insc_deconv_down2(const float *d_in, int64_t ld_in, int64_t n_in_rows, float *d_out, int64_t ld_out,
                      const float *d_W, const float *d_Wp, const float *d_bias, const int32_t *d_parent,
                      const int32_t *d_offset, const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows,
                      int Cin, int Cout, void *stream);
/* Inference batch norm + leaky ReLU: y = x*w + b, y *= (y>0 ? 1 : leakiness),
 * w = gamma*(var+eps)^-1/2, b = beta - mean*w; gamma/beta nullable
 * (BatchNormalization_updateOutput with train=false, CUDA/BatchNormalization.cpp:39-61,
 * kernel BatchNormalization.cu:78-107). */
int insc_bn_leaky(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_mean,
                  const float *d_var, const float *d_gamma, const float *d_beta, float eps, float leakiness,
                  const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C, void *stream);
/* out = a + b on the listed rows (AddTable, sparseconvnet/tables.py:28-40). */
int insc_add(const float *d_a, int64_t ld_a, const float *d_b, int64_t ld_b, float *d_out, int64_t ld_out,
             const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C, void *stream);
/* out[r, :] = in[r, :] on the listed rows (column-slice copy used for JoinTable,
 * sparseconvnet/tables.py:13-25). */
int insc_copy_rows(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const int32_t *d_rows,
                   const int32_t *d_n_rows, int64_t n_rows, int C, void *stream);

/* Input layer accumulation: adds the P feature rows to the per-site running sums
 * d_sum[site,:] (float32 [*,C]) and counts d_cnt[site], rows of one site in ascending row
 * order (the order InputLayer_fp_ visits them, CUDA/IOLayers.cu:17-32).  The caller zeroes
 * the rows of d_sum / d_cnt that belong to sites it has not accumulated into before.
 * mode 1 keeps the first row of a site, mode 2 the last (CPU rule builder,
 * Metadata/IOLayersRules.h:104-115), modes 0/3/4 sum. */
int insc_input_accumulate(const float *d_feats, int64_t P, int C, const int32_t *d_site_of_point, int mode,
                          float *d_sum, int32_t *d_cnt, int64_t n_sites_upper, void *stream);
/* out[s,:] = sum[s,:] / cnt[s] (mode 4) or sum[s,:] (other modes) on the listed rows. */
int insc_input_finish(const float *d_sum, const int32_t *d_cnt, int mode, float *d_out, int64_t ld_out,
                      const int32_t *d_rows, const int32_t *d_n_rows, int64_t n_rows, int C, void *stream);
/* Output layer: out[p,:] = in[site_of_point[p],:] (OutputLayer_updateOutput,
 * CUDA/IOLayers.cpp:123-145: InputLayer_bp_ with multiplier 1). */
int insc_output_gather(const float *d_in, int64_t ld_in, const int32_t *d_site_of_point, int64_t P, int C,
                       float *d_out, void *stream);
/* Size-2 stride-2 pooling to the next coarser scale over the child map of insc_rulebook_down2:
 * mode 0 = MaxPooling_updateOutput (CUDA/MaxPooling.cpp:18-36; the output starts at zero, so the
 * result is max(0, max over the children)), mode 1 = AveragePooling_updateOutput
 * (CUDA/AveragePooling.cpp:19-39: sum over the children divided by the filter volume 8).  The
 * reference's nFeaturesToDrop is a pointer offset on d_in.  UnPooling_updateOutput
 * (CUDA/UnPooling.cpp:17-37), out_fine[i] = in_coarse[parent[i]], is insc_output_gather with the
 * parent map in place of site_of_point. */
int insc_pool_down2(const float *d_in, int64_t ld_in, const int32_t *d_child, int64_t n_coarse, int C, int mode,
                    float *d_out, int64_t ld_out, void *stream);
/* Dense [batch, C, X, Y, Z] float32 copy (zero where no site is active) of the feature matrix of
 * the grid's first n sites (SparseToDense_updateOutput, CUDA/SparseToDense.cpp:16-41; cell offset
 * as RectangularRegion::offset, Metadata/RectangularRegions.h:52-60).  Sites outside the box or
 * the batch range are skipped. */
int insc_sparse_to_dense(const insc_grid *g, const float *d_in, int64_t ld_in, int64_t n, int C, int64_t X, int64_t Y,
                         int64_t Z, int batch, float *d_out, void *stream);

/* ---------------------------------------------------------------------------------------
 * Dirty-site propagation for the incremental forward.  Masks are uint8 per site.
 * The reference's incremental path does not dilate (CUDA/Convolution.cpp:221-303 computes
 * residuals only at the increment's own sites); these functions implement the exact rule:
 * a row must be recomputed iff any input it reads changed.
 * ------------------------------------------------------------------------------------- */
int insc_fill_u8(uint8_t *d_p, int64_t n, int value, void *stream);
int insc_fill_i32(int32_t *d_p, int64_t n, int32_t value, void *stream);
/* mask[site_of_point[p]] = 1 */
int insc_dirty_mark(const int32_t *d_site_of_point, int64_t P, uint8_t *d_mask, void *stream);
/* mask_out[j] = 1 for every j = nbr[i*27+k] >= 0 with mask_in[i] != 0 (includes i itself). */
int insc_dirty_dilate3(const int32_t *d_nbr, const uint8_t *d_mask_in, uint8_t *d_mask_out, const int32_t *d_n,
                       int64_t n_upper, void *stream);
/* mask_coarse[parent[i]] = 1 for dirty fine i. */
int insc_dirty_parents(const int32_t *d_parent, const uint8_t *d_mask_fine, uint8_t *d_mask_coarse,
                       const int32_t *d_n_fine, int64_t n_upper, void *stream);
/* mask_fine[i] |= mask_coarse[parent[i]]. */
int insc_dirty_children(const int32_t *d_parent, const uint8_t *d_mask_coarse, uint8_t *d_mask_fine,
                        const int32_t *d_n_fine, int64_t n_upper, void *stream);
/* mask_out = mask_a | mask_b */
int insc_dirty_or(const uint8_t *d_a, const uint8_t *d_b, uint8_t *d_out, const int32_t *d_n, int64_t n_upper,
                  void *stream);
/* d_rows = the sites s (taken in the sequence d_order[0..n) if given, else 0..n) with
 * mask[s] != 0; *d_count = how many.  h_count nullable (synchronises). */
int insc_dirty_compact(const uint8_t *d_mask, const int32_t *d_order, const int32_t *d_n, int64_t n_upper,
                       int32_t *d_rows, int32_t *d_count, int64_t *h_count, void *stream);

/* ---------------------------------------------------------------------------------------
 * Network executor: a whole network (input layer, 3^3 submanifold convolutions, 2/2
 * convolutions and deconvolutions, batch norm + ReLU, 1x1 layers, add, channel join, output
 * layer) run from one host call, full or incremental.  It plays the part of the reference's
 * Python module graph plus its per-module saved state (sparseconvnet/sequential.py:20-25,
 * submanifoldConvolution.py:53-54, batchNormalization.py:60-61, ioLayers.py:69,106-107):
 * a full frame corresponds to Model(x, increment=False), an incremental frame to
 * Model(x, increment=True) (demo.py:26-38), except that the incremental result equals a full
 * forward over all points seen so far.
 *
 * Scales are numbered 0 (input resolution) upward, one per 2/2 convolution.  Tensor 0 is the
 * input layer's output; weight, bias and batch-norm pointers are device pointers that must
 * outlive the net.
 * ------------------------------------------------------------------------------------- */
typedef struct insc_net insc_net;
int insc_net_create(int n_levels, int in_channels, int input_mode, insc_net **out);
int insc_net_destroy(insc_net *net);
/* New feature matrix with `channels` columns at scale `level`. */
int insc_net_tensor(insc_net *net, int level, int channels, int *out_id);
/* Declare tensor `out` as the channel concatenation [a | b] (JoinTable): a and b become
 * column slices of out's matrix, so their producers write in place and nothing is copied. */
int insc_net_join(insc_net *net, int a, int b, int out);
/* kind 0: submanifold 3^3, W [27,Cin,Cout]; 2: convolution 2/2 to the next coarser scale,
 * W [8,Cin,Cout]; 3: deconvolution 2/2 to the next finer scale; 4: 1x1, W [Cin,Cout]. */
int insc_net_op_conv(insc_net *net, int kind, int in, int out, const float *d_W, const float *d_bias);
int insc_net_op_bn(insc_net *net, int in, int out, const float *d_mean, const float *d_var, const float *d_gamma,
                   const float *d_beta, float eps, float leakiness);
int insc_net_op_add(insc_net *net, int a, int b, int out);
/* Freeze the program; out_tensor feeds the output layer; capacity_sites is reserved at scale 0
 * (half of it at each coarser scale; everything grows on demand). */
int insc_net_finalize(insc_net *net, int out_tensor, int64_t capacity_sites, void *stream);
/* Before insc_net_finalize: also keep the input of every batch norm, which residual frames
 * (insc_net_forward_residual) read and which the fused layers would otherwise not store. */
int insc_net_enable_residual(insc_net *net);
/* Incremental frames append their new sites to the processing orders of the scales (the order in
 * which a scale's rows are cut into 32-row tiles), each frame's batch sorted among itself.  Once the
 * appended part of a scale of more than 8192 sites exceeds `percent` % of the part that was sorted
 * as a whole, the next incremental frame sorts the orders of all scales from scratch, as a full
 * frame does (0.1-0.2 ms once, for layers that then run some 10 % faster).  Results do not
 * depend on the order.  Default 10; 0: never.  No counterpart in the reference, which rebuilds
 * its rulebooks on every call. */
int insc_net_set_order_refresh(insc_net *net, int percent);
/* Re-pack the weights after the caller changed them in place.  The rows cached by earlier frames
 * were computed with the old parameters and are forgotten: the next frame must be a full one
 * (an incremental or residual frame before it returns INSC_ERR_STATE). */
int insc_net_refresh_weights(insc_net *net, void *stream);
/* Ops added so far (joins included); the op added last has index insc_net_op_count() - 1. */
int insc_net_op_count(const insc_net *net);
/* Point op `op` at parameters that moved (e.g. the caller's framework re-allocated them when a
 * checkpoint was restored): d_W / d_bias for a convolution op, d_mean / d_var / d_gamma / d_beta for
 * a batch norm; same shapes as when the op was added.  Follow with insc_net_refresh_weights.
 * Like that call it forgets the cached state of earlier frames.  No counterpart in the reference, whose modules pass their tensors on every call. */
int insc_net_rebind_op(insc_net *net, int op, const float *d_W, const float *d_bias, const float *d_mean,
                       const float *d_var, const float *d_gamma, const float *d_beta);
/* One frame: d_coords int32 [P,coord_cols] (x,y,z[,batch]), d_feats float32 [P,in_channels].
 * increment == 0 forgets all state and runs a full forward; increment != 0 appends the points
 * and recomputes only the rows they affect.  d_out (nullable) receives one row of the output
 * tensor per point of this frame (out_all == 0) or per point since the last full frame.
 * Returns once the frame is enqueued on `stream` (the host has waited for the site counts of the
 * frame's insert by then, nothing else); d_out and the state are ready in stream order, and
 * d_coords, d_feats and d_out must stay valid - the two inputs unmodified - until the stream has
 * reached the end of the frame (kernels that read them may still be running when the call
 * returns; work enqueued on the same stream afterwards is ordered behind them).
 * A frame is all or nothing: if any of its coordinates is outside the representable range the call returns INSC_ERR_COORD and the state is that of the
 * previous frame (after a full frame that failed: no state; the next frame must be a full one). */
int insc_net_forward(insc_net *net, const int32_t *d_coords, int coord_cols, const float *d_feats, int64_t P,
                     int increment, float *d_out, int out_all, int64_t *h_n_sites, void *stream);
/* The dirty sets of the last exact incremental frame (diagnostics; no counterpart in the
 * reference, whose incremental frames do not propagate): for set i in program order,
 * h_level[i] = its scale, h_kind[i] = 0 input, 1 dilated by a 3^3 layer, 2 parents, 3 children,
 * 4 union, h_rows[i] = its number of rows.  *h_n_sets <= max_sets sets are reported.  Synchronises. */
int insc_net_dirty_counts(insc_net *net, int max_sets, int *h_n_sets, int *h_level, int *h_kind, int64_t *h_rows,
                          void *stream);
/* One residual frame: the reference's own incremental forward (demo.py:26-38 with
 * increment=True; Incre_* operators, pybind.cpp:218-258) as one call.  The frame's points form a
 * site set of their own, features are differences to the state saved by the last
 * insc_net_forward, and that state is not modified.  d_out (nullable): [P,C], saved value +
 * residual for every point of the frame (cuda_Incre_OutputLayer_updateOutput,
 * CUDA/IOLayers.cpp:339-368).  h_n_sites (nullable): sites of the frame at the input scale.
 * Returns once the frame's site counts are known; the layers may still be running on the stream. */
int insc_net_forward_residual(insc_net *net, const int32_t *d_coords, int coord_cols, const float *d_feats, int64_t P,
                              float *d_out, int64_t *h_n_sites, void *stream);
/* What every convolution of the last completed frame worked on (diagnostics for flop accounting; the
 * reference's operators return their multiply-add count instead, e.g. CUDA/Convolution.cpp:152-218).
 * For convolution i in program order (i < *h_n_ops <= max_ops): h_kind[i] (0 3^3 submanifold,
 * 2 strided, 3 transposed, 4 1x1), h_level[i] = scale of its output, h_cin[i], h_cout[i], and over
 * the 32-row tiles it computed in that frame h_rows[i] = output rows, h_rules[i] = rules,
 * h_slots[i] = 32 x offsets used per tile.  Useful multiply-adds = rules x Cin x Cout; the matrix
 * cores are issued slots x Cin x Cout.  Synchronises. */
int insc_net_frame_work(insc_net *net, int max_ops, int *h_n_ops, int *h_kind, int *h_level, int *h_cin, int *h_cout,
                        int64_t *h_rows, int64_t *h_rules, int64_t *h_slots, void *stream);
int insc_net_tensor_view(insc_net *net, int tensor, float **d_ptr, int64_t *ld, int64_t *rows, int *channels);
int insc_net_counts(insc_net *net, int64_t *h_sites_per_level, int64_t *h_points);
/* Phase timing (the reference brackets the same phases with easy_profiler blocks,
 * Metadata/Metadata.cpp:442-509, CUDA/Convolution.cpp:152-218).  enable != 0: every frame
 * records four stream events; h_ms4 then receives the GPU time in ms of the last frame's phases:
 * [0] grids, rulebooks and input accumulation, [1] dirty-set propagation, [2] the layers,
 * [3] output gather and count read-back. */
int insc_net_profile(insc_net *net, int enable, float *h_ms4);

/* ---------------------------------------------------------------------------------------
 * Per-voxel label fusion over frames (Result<3> and ResultOfWeight, Metadata/resultHash.h:23-218;
 * bound as SCN.Result_3 / SCN.ResultOfWeight, pybind.cpp:36-45,275-282).  The reference keeps a
 * CPU hash map and handles points one by one; here the map is a hash grid plus device arrays.
 * kind 0: (label, confidence) per voxel; kind 1: running scores per voxel (new = 0.5*old + row).
 * Rows of one voxel inside a call are applied in ascending row order.
 * `maximum` is truncated towards zero, as the reference does by storing it in an int member
 * (resultHash.h:25,30): its default 0.7 acts as a ceiling of 0.
 * ------------------------------------------------------------------------------------- */
typedef struct insc_labels insc_labels;
int insc_labels_create(int64_t capacity_voxels, int kind, float maximum, insc_labels **out);
int insc_labels_destroy(insc_labels *l);
int insc_labels_clear(insc_labels *l, void *stream);
/* Result::set (resultHash.h:36-47): label = argmax of the row, confidence 0; the last row of a voxel wins. */
int insc_labels_set(insc_labels *l, const int32_t *d_coords4, const float *d_scores, int64_t ld, int64_t P, int C,
                    void *stream);
/* Result::update (resultHash.h:49-101) for kind 0: a new voxel takes (argmax, max); a known one
 * gains the row's maximum if the label agrees (up to the ceiling), loses it otherwise, and flips
 * to the row's label when the confidence falls below zero.  ResultOfWeight::update
 * (resultHash.h:158-170) for kind 1. */
int insc_labels_update(insc_labels *l, const int32_t *d_coords4, const float *d_scores, int64_t ld, int64_t P, int C,
                       void *stream);
/* multiQuery (resultHash.h:110-118,179-187): label per coordinate, -1 for an unknown voxel. */
int insc_labels_query(insc_labels *l, const int32_t *d_coords4, int64_t Q, int32_t *d_label, void *stream);
int insc_labels_count(insc_labels *l, int64_t *h_n, void *stream);
/* get_all_points_labels (resultHash.h:120-132,189-201): rows (x, y, z, label) of the first `rows`
 * voxels; d_conf (nullable) receives the confidence (kind 0) or the best score (kind 1). */
int insc_labels_export(insc_labels *l, int32_t *d_out4, float *d_conf, int64_t rows, void *stream);
/* finalize (resultHash.h:134-145,203-214): forget every voxel that is not in the list. */
int insc_labels_finalize(insc_labels *l, const int32_t *d_keep4, int64_t M, void *stream);

/* ---------------------------------------------------------------------------------------
 * Residual frames: the reference's own incremental operators (Incre_*, pybind.cpp:218-258).
 * The frame's points form a site set of their own (fresh grids g at every scale); `pre` names
 * the grids and feature matrices saved by the last full forward.  d_pre_exist[i] = id of the
 * frame's site i in the saved grid of the same scale or -1 (getPreExistMaps,
 * Metadata/Metadata.cpp:609-626) - obtain it with insc_grid_query(pre, insc_grid_coords(g), n, ..).
 * Features of sites that existed are differences to the saved state, features of new sites are
 * plain values.  Nothing here changes the saved state.
 * ------------------------------------------------------------------------------------- */
/* d_nbr_pre[i*27+k] = id, in the saved grid, of the neighbour k of the frame's site i if that
 * site is new (d_pre_exist[i] < 0), -1 otherwise; the centre offset is always -1.  The rules of
 * IncreSubmanifoldBuildObject (CUDA/SubmanifoldRules_cuda.cpp:233-472, kernel
 * SubmanifoldRules_cuda.cu:132-156) as a dense map. */
int insc_incre_rulebook_ssc3(const insc_grid *g, const insc_grid *pre, const int32_t *d_pre_exist, int64_t n,
                             int32_t *d_nbr_pre, void *stream);
/* Input layer of a residual frame (cuda_Incre_InputLayer_updateOutput, CUDA/IOLayers.cpp:290-337;
 * kernel IOLayers.cu:81-105).  d_sum / d_cnt: this frame's per-site sums and counts
 * (insc_input_accumulate on the fresh grid); d_pre_out / d_pre_cnt: the saved input-layer output
 * and point counts.  With na, pn the rule lengths (point counts for modes 3 and 4, 1 for modes 1
 * and 2) and m = 1/(na+pn) in mode 4, 1 otherwise:
 *   out = m*sum + pre_out*(pn*m - 1) for a voxel that existed, out = m*sum for a new one. */
int insc_incre_input(const float *d_sum, const int32_t *d_cnt, int mode, const int32_t *d_pre_exist,
                     const float *d_pre_out, int64_t ld_pre, const int32_t *d_pre_cnt, float *d_out, int64_t ld_out,
                     int64_t n, int C, void *stream);
/* 3^3 submanifold convolution of a residual frame (cuda_Incre_SubmanifoldConvolution_updateOutput,
 * CUDA/Convolution.cpp:221-303):
 *   out[i] = bias + sum_k in[nbr[i,k]].W[k] + sum_k pre_in[nbr_pre[i,k]].W[k]
 * d_nbr is the frame's own map (insc_rulebook_ssc3 on g), d_nbr_pre the map of
 * insc_incre_rulebook_ssc3; d_in has n rows, d_pre_in n_pre_rows. */
int insc_incre_conv_ssc(const float *d_in, int64_t ld_in, const float *d_pre_in, int64_t ld_pre, int64_t n_pre_rows,
                        float *d_out, int64_t ld_out, const float *d_W, const float *d_Wp, const float *d_bias,
                        const int32_t *d_nbr, const int32_t *d_nbr_pre, int64_t n, int Cin, int Cout, void *stream);
/* Batch norm + leaky ReLU of a residual frame (cuda_Incre_BatchNormalization_updateOutput,
 * CUDA/BatchNormalization.cpp:63-91; kernel BatchNormalization.cu:112-150): with o = w*x + b,
 *   out = leaky(o + w*pre_in[pe]) - pre_out[pe] for a site that existed, leaky(o) for a new one. */
int insc_incre_bn_leaky(const float *d_in, int64_t ld_in, float *d_out, int64_t ld_out, const float *d_mean,
                        const float *d_var, const float *d_gamma, const float *d_beta, float eps, float leakiness,
                        const int32_t *d_pre_exist, const float *d_pre_in, int64_t ld_pre_in, const float *d_pre_out,
                        int64_t ld_pre_out, int64_t n, int C, void *stream);
/* Size-2 stride-2 deconvolution of a residual frame (cuda_Incre_Deconvolution_updateOutput,
 * CUDA/Deconvolution.cpp:61-96; kernel Deconvolution.cu:84-150):
 *   out[f] = bias + (in[c] + pre_in[pre_exist_in[c]] * [c existed and f is new]) . W[offset[f]],
 * c = parent[f].  (The size-2 stride-2 convolution of a residual frame is insc_conv_nbr on the
 * frame's own child map, Incre_Convolution_updateOutput, CUDA/Convolution.cpp:83-113.) */
int insc_incre_deconv_down2(const float *d_in, int64_t ld_in, int64_t n_in_rows, const float *d_pre_in, int64_t ld_pre,
                            int64_t n_pre_rows, float *d_out, int64_t ld_out, const float *d_W, const float *d_Wp,
                            const float *d_bias, const int32_t *d_parent, const int32_t *d_offset,
                            const int32_t *d_pre_exist_in, const int32_t *d_pre_exist_out, int64_t n_rows, int Cin,
                            int Cout, void *stream);
/* Output layer of a residual frame (cuda_Incre_OutputLayer_updateOutput, CUDA/IOLayers.cpp:339-368;
 * kernel IOLayers.cu:122-141): out[p] = in[s] + pre_in[pre_exist[s]] (second term for sites that
 * existed), s = site_of_point[p]. */
int insc_incre_output(const float *d_in, int64_t ld_in, const float *d_pre_in, int64_t ld_pre,
                      const int32_t *d_pre_exist, const int32_t *d_site_of_point, int64_t P, int C, float *d_out,
                      void *stream);

/* ---------------------------------------------------------------------------------------
 * Device utilities exported for tests and callers.
 * ------------------------------------------------------------------------------------- */
/* Exclusive prefix sum of n int32 values; d_total (nullable) receives the sum. */
int insc_scan_exclusive_i32(const int32_t *d_in, int32_t *d_out, int64_t n, int32_t *d_total, void *stream);
/* Stable ascending sort of n (key,value) pairs on the low key_bits bits of the 64-bit keys.
 * Keys and values are sorted in place (d_keys / d_vals hold the result). */
int insc_sort_pairs_u64(uint64_t *d_keys, int32_t *d_vals, int64_t n, int key_bits, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* INSC_H */
