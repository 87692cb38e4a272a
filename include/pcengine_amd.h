/* pcengine_amd — C ABI of the MI355X (gfx950) sparse-convolution hot path.
 *
 * Plain pointers and sizes only; every pointer named "device" is HIP device memory owned by the
 * caller.  The library allocates no device memory and launches all work on the stream it is given.
 * Functions return PCE_OK (0) or an error code; the text of the last error on the calling thread is
 * returned by pce_last_error().
 *
 * State the library keeps between calls: (1) per device, a ring of eight pinned host blocks (32 KB
 * each, allocated on the first pce_kmap_build / pce_kmap_build_batch on that device, never freed)
 * from which the descriptors of a batched map build are copied to the device, guarded by one mutex,
 * so calls from several host threads are safe; (2) a static device array of 32 MiB per GPU the library
 * runs on, the accumulator of pce_conv_fwd_fod_static, with its device address looked up once per device
 * (pce_conv_fod_static_init, or the first call); calls of that entry point that overlap on one GPU race;
 * (3) the number of compute units of each device, asked once; (4) the thread-local text of
 * pce_last_error().  Nothing else: no caches, no tables, no switches.  (The stage mask a benchmark uses to
 * time one kernel of a dataflow alone exists only in the separately built measurement library, see
 * pcengine_amd_measure.h; that library carries a static array of its own.)
 *
 * Versioning: pce_version() returns PCE_ABI_VERSION of the header the library was built from.  The structs
 * below (pce_epilogue_t, pce_kmap_problem_t, pce_pyr_*_t) have no size field: a caller compiles against the
 * header of the library it loads, zero-initialises every struct with the sizeof of that header, and refuses to
 * run when pce_version() differs from its PCE_ABI_VERSION.  Version 200 against 100: pce_epilogue_t grew
 * ld_in / ld_out, pce_kmap_problem_t grew n_batch / flags / order and its status became int32[8], the row
 * order grew records, pce_conv_fwd_oso and pce_row_order take three counts, pce_select_dataflow takes mid and
 * transposed, pce_set_stage_mask left this library; pce_pyramid_*, pce_outcoords_chain_planned,
 * pce_conv_oso_takes and pce_conv_fod_static_init are new.
 *
 * These entry points are what the reference's five pybind functions
 * (backend/pybind_cuda.cpp:8-14) decompose into:
 *
 *   mapping_d2_cuda  = HashMapD2  (backend/hash.h:37-58,  backend/hash.cu:258-435)
 *       -> pce_outcoords_build/_emit (strided only) + pce_kmap_build
 *   mapping_d1_cuda  = HashMapD1  (backend/hash.h:11-34,  backend/hash.cu:20-255)
 *       -> the same, with the CSR outputs of pce_kmap_build requested
 *   conv_fwd_d2_cuda = ConvolutionForwardD2 (backend/spconv.h:28-40, backend/spconv.cu:224-398)
 *       -> pce_conv_fwd_fod
 *   conv_fwd_d1_cuda = ConvolutionForwardD1 (backend/spconv.h:11-25, backend/spconv.cu:24-222)
 *       -> pce_conv_fwd_gms
 *   conv_bwd_d1_cuda = ConvolutionBackwardD1 (backend/spconv.h:43-58, backend/spconv.cu:400-629)
 *       -> pce_conv_wgrad (kernel gradient) + pce_conv_fwd_fod over the swapped map with the
 *          per-offset transposed kernel (feature gradient)
 */
#ifndef PCENGINE_AMD_H
#define PCENGINE_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *pce_stream_t; /* hipStream_t */

enum {
  PCE_OK = 0,
  PCE_EINVAL = 1,     /* bad argument (shape mismatch, null pointer, unsupported size) */
  PCE_ECAPACITY = 2,  /* a documented capacity limit would be exceeded */
  PCE_EHIP = 3,       /* a HIP runtime call or kernel launch failed */
  PCE_EWORKSPACE = 4, /* workspace too small */
  PCE_ECOORD = 5      /* a coordinate is outside the representable range */
};

enum { PCE_F16 = 0, PCE_F32 = 1, PCE_F64 = 2 /* points of pce_voxelize only */ };

/* dataflows of the forward convolution */
enum {
  PCE_DATAFLOW_FOD = 0, /* fetch-on-demand fused gather-matmul-scatter (reference "D2") */
  PCE_DATAFLOW_GMS = 1, /* gather - grouped GEMM - scatter over a staging buffer (reference "D1") */
  PCE_DATAFLOW_OS = 2,  /* output-stationary fetch-on-demand: no atomics, no staging buffer */
  PCE_DATAFLOW_FDS = 3, /* fetch-on-demand with deferred scatter: pair tiles write partial rows to a
                           staging buffer, the centre GEMM's epilogue sums them per output row */
  PCE_DATAFLOW_OSO = 4  /* output-stationary over rows ordered by their neighbour pattern (pce_row_order):
                           fp16 layers up to 64 channels and of 64 / 96 -> 65..128 and 128 -> 65..96 channels, submanifold
                           or strided; fp32 submanifold layers up to 32 channels; one launch, no partial rows */
};

#define PCE_QUANTUM 128        /* rows per tile of the pair list; qkpos granularity (backend/hash.cu:203-205) */
#define PCE_CSR_CODE 1186111   /* CSR entry code = kp * PCE_CSR_CODE + rank (backend/hash.cuh:7-9) */
#define PCE_COORD_BOUND 3259   /* spatial coordinates of a strided conv's output must be < this (backend/hash.cuh:503) */
#define PCE_COORD_LIMIT 32000  /* |coordinate| limit of the packed 64-bit hash key */

/* Geometry of one convolution; what the reference passes as four packed codes plus bounds
 * (backend/hash.cu:57-76, script/spconv.py:354-367). */
typedef struct pce_geom {
  int32_t ks[3];      /* kernel size */
  int32_t stride[3];  /* layer stride */
  int32_t pad[3];     /* padding */
  int32_t cmin[3];    /* lower bound of output coordinates */
  int32_t cmax[3];    /* upper bound of output coordinates, already reduced for strided layers */
  int32_t subm;       /* 1: submanifold (out coords = in coords, centre offset handled densely) */
} pce_geom_t;

#define PCE_ABI_VERSION 200
int pce_version(void);
const char *pce_last_error(void);

/* ---- coordinate hash table: open addressing on the packed (b,x,y,z) 64-bit key ------------- */

/* Slot count for n keys: 2 * 2^ceil(log2 n), the reference's load factor (backend/hash.cu:46). */
int64_t pce_hash_slots(int64_t n);
/* Bytes of a table with that many slots (16 bytes per slot: key + row). */
int64_t pce_hash_table_bytes(int64_t n);
/* Insert rows 0..n-1 of coords[n,4] (replaces insertHash + insertVal, backend/hash.cuh:55-91).
 * status (device int32[2]) receives [0] = 1 if a coordinate was out of range,
 * [1] = 1 if probing exhausted the table; the caller zeroes it first. */
int pce_hash_build(void *table_dev, int64_t slots, const int32_t *coords_dev, int64_t n,
                   int32_t *status_dev, pce_stream_t stream);
/* rows_dev[q] = row of qcoords[q] in the table, or -1 (probe loop of backend/hash.cuh:154-161). */
int pce_hash_query(const void *table_dev, int64_t slots, const int32_t *qcoords_dev, int64_t nq,
                   int32_t *rows_dev, pce_stream_t stream);

/* ---- output coordinates of a strided convolution -------------------------------------------- *
 * Replaces coordsDownsampleExpand + remove + sort + unique + coordsGenerator
 * (backend/hash.cuh:535-641, backend/hash.cu:141-173).  Always the generic rule; the reference's
 * stride==kernel shortcut is not reproduced because it disagrees with its own query kernels.
 *
 * n_batch is the batch count the reference carries as spTensor.batchsize and hands to its mapping
 * call (script/spconv.py:363).  With n_batch > 0 and a modest output bounding box (geometry cmin /
 * cmax) the candidates are marked in an occupancy bitmap in (b,x,y,z) order and a popcount scan
 * de-duplicates, sorts and counts them at once; a batch index >= n_batch is then PCE_EINVAL.
 * With n_batch <= 0, or a box too large or too empty for a bitmap, candidates go through a hash
 * table and a radix sort of their codes instead.  Both give the same coordinates.  The three calls
 * of one build take the same (n_in, g, n_batch). */
int64_t pce_outcoords_workspace_bytes(int64_t n_in, const pce_geom_t *g, int32_t n_batch);
/* Builds the sorted unique output set inside the workspace and returns its size in
 * *n_out_host.  Synchronises the stream once (the count has to reach the host). */
int pce_outcoords_build(const int32_t *in_coords_dev, int64_t n_in, const pce_geom_t *g, int32_t n_batch,
                        void *ws_dev, int64_t ws_bytes, int64_t *n_out_host, pce_stream_t stream);
/* Decodes it into out_coords_dev[n_out,4] (same workspace, untouched since _build). */
int pce_outcoords_emit(const void *ws_dev, int64_t n_in, const pce_geom_t *g, int32_t n_batch, int64_t n_out,
                       int32_t *out_coords_dev, pce_stream_t stream);

/* The output coordinates of several strided layers in a row -- the levels of a network, each reading the
 * coordinates the one before it wrote -- with ONE wait of the host instead of one per level: the count of a level
 * stays on the device for the next and the launches are sized for its bound (the reference builds level by level,
 * script/spconv.py:363 once per strided layer).  Every level has to qualify for the occupancy bitmap
 * (n_batch > 0, modest boxes).
 *   pce_outcoords_chain_plan: PCE_OK and, per level, the workspace bytes and the capacity (rows) its output
 *       buffer needs; PCE_CHAIN_NOT_APPLICABLE when some level does not qualify (build level by level then).
 *   pce_outcoords_chain: builds all levels; out_coords_dev[l] receives n_out_host[l] rows of (b,x,y,z), identical
 *       to what pce_outcoords_build/_emit give level by level.  Synchronises the stream once. */
#define PCE_MAX_CHAIN 8
#define PCE_CHAIN_NOT_APPLICABLE 100
int pce_outcoords_chain_plan(int64_t n_in, int32_t levels, const pce_geom_t *geoms, int32_t n_batch,
                             int64_t *ws_bytes, int64_t *capacity);
int pce_outcoords_chain(const int32_t *in_coords_dev, int64_t n_in, int32_t levels, const pce_geom_t *geoms,
                        int32_t n_batch, void *const *ws_dev, const int64_t *ws_bytes, int32_t *const *out_coords_dev,
                        int64_t *n_out_host, pce_stream_t stream);
/* The same through workspaces laid out for n_plan >= n_in rows (pce_outcoords_chain_plan(n_plan, ...)): whether a level
 * takes the bitmap depends on the row count, and a plan kept for several clouds must not change its mind. */
int pce_outcoords_chain_planned(const int32_t *in_coords_dev, int64_t n_in, int64_t n_plan, int32_t levels,
                                const pce_geom_t *geoms, int32_t n_batch, void *const *ws_dev, const int64_t *ws_bytes,
                                int32_t *const *out_coords_dev, int64_t *n_out_host, pce_stream_t stream);

/* ---- voxelisation ----------------------------------------------------------------------------- *
 * Replaces sparse_quantize + ravel_hash (script/utils.py:18-55), which the reference runs in NumPy
 * on the host: voxel = floor(point / voxel_size) in double precision; the unique voxels in
 * ascending (x,y,z) order (the order of the ravelled code); for every voxel the first point that
 * falls into it (numpy.unique return_index); for every point its voxel (return_inverse).
 * points_dev[n_points,3] are PCE_F32 or PCE_F64.  pce_voxelize synchronises the stream twice
 * (coordinate bounds, then the voxel count) and returns the count and the bounds of the integer
 * coordinates on the host; pce_voxelize_emit (same workspace, untouched since; the bounds handed
 * back) writes coords_out[n_voxels,4] = (batch_index, x, y, z), index_out[n_voxels] and
 * inverse_out[n_points]; any of the three may be NULL.  Negative coordinates are kept, as in the
 * reference (the kernel-map entry points need them shifted to >= 0 by the caller,
 * check_fwd.py:51). */
int64_t pce_voxelize_workspace_bytes(int64_t n_points);
int pce_voxelize(const void *points_dev, int32_t dtype, int64_t n_points, const double *voxel_size3_host,
                 void *ws_dev, int64_t ws_bytes, int64_t *n_voxels_host, int32_t *coords_min3_host,
                 int32_t *coords_max3_host, pce_stream_t stream);
int pce_voxelize_emit(const void *ws_dev, int64_t n_points, int64_t n_voxels,
                      const int32_t *coords_min3_host, const int32_t *coords_max3_host,
                      int32_t batch_index, int32_t *coords_out_dev, int32_t *index_out_dev,
                      int32_t *inverse_out_dev, pce_stream_t stream);

/* ---- kernel map ------------------------------------------------------------------------------ *
 * Replaces the four _queryhash_* kernels, exclusive_scan_for_kernel_quantified, mapping_counter and
 * the thrust remove/scan calls (backend/hash.cuh:97-497, backend/hash.cu:180-243) and the
 * nonzero-compaction done in Python (script/spconv.py:370-372).
 *
 * Outputs (device, caller-allocated; nothing needs pre-initialising):
 *   imap, omap   int32[kv*n_in] capacity; the first M = kpos[kv] entries are the (input row,
 *                output row) pairs ordered by (offset, input row)
 *   knnz[kv], kpos[kv+1], qkpos[kv+1]
 *   optional (pass NULL to skip), all four or none:
 *     icsr[n_in+1], icode[kv*n_in cap], ocsr[n_out+1], ocode[kv*n_in cap]: CSR-coded map,
 *     entry = kp*PCE_CSR_CODE + rank, ascending kp inside a row, rank = position inside the offset
 *   optional, with the CSR outputs: islot, oslot int32[kv*n_in cap]: for pair p, the position of
 *     its entry in icode / ocode (the inverse permutation of the CSR orders)
 *   optional nbr_out int32[kv*n_out]: output-major table nbr[kp*n_out + o] = input row or -1
 *     (centre offset of a submanifold layer = the row itself)
 *   optional nbr_in int32[kv*n_in]: input-major table nbr[kp*n_in + i] = output row or -1, the
 *     layout of the reference's dense fetch-on-demand map (backend/hash.cuh:331,417); it is the
 *     output-major table of the transposed layer
 *   status int32[4]: [0] coordinate out of range, [1] table exhausted, [2] an offset holds
 *     >= PCE_CSR_CODE pairs (CSR code would overflow), [3] the column grid of pce_kmap_build_batch
 *     could not be used (see there).  Caller zeroes it; read it after a sync. */
int64_t pce_kmap_workspace_bytes(int64_t n_in, int64_t n_out, int32_t kv, int32_t want_csr);
int pce_kmap_build(const int32_t *in_coords_dev, int64_t n_in, const int32_t *out_coords_dev,
                   int64_t n_out, const pce_geom_t *g, void *ws_dev, int64_t ws_bytes,
                   int32_t *imap_dev, int32_t *omap_dev, int32_t *knnz_dev, int32_t *kpos_dev,
                   int32_t *qkpos_dev, int32_t *icsr_dev, int32_t *icode_dev, int32_t *ocsr_dev,
                   int32_t *ocode_dev, int32_t *islot_dev, int32_t *oslot_dev, int32_t *nbr_out_dev,
                   int32_t *nbr_in_dev, int32_t *status_dev, pce_stream_t stream);

/* The maps of several layers in one call (a network needs one per distinct layer geometry of a
 * point cloud: script/spconv.py:330-372 runs once per such layer).  Every stage of the build is
 * one launch shared by all problems of the batch, so a batch costs the launches of one build.
 * Each problem carries the arguments of pce_kmap_build with the same meaning and its own
 * workspace; the problems must not share outputs or workspaces, and the output coordinates of
 * every problem must be complete before the call.  At most PCE_KMAP_MAX_BATCH problems.
 * The call queues one small host-to-device copy (the descriptors of the batch, from pinned memory
 * the library keeps) ahead of its kernels and does not wait for the stream. */
#define PCE_KMAP_MAX_BATCH 16
typedef struct pce_kmap_problem {
  const int32_t *in_coords;
  int64_t n_in;
  const int32_t *out_coords;
  int64_t n_out;
  pce_geom_t geom;
  void *ws;
  int64_t ws_bytes;
  int32_t *imap, *omap, *knnz, *kpos, *qkpos; /* imap / omap may be NULL with PCE_KMAP_TABLE_ONLY over the column grid */
  int32_t *icsr, *icode, *ocsr, *ocode; /* all four or none */
  int32_t *islot, *oslot;               /* optional, with the CSR outputs */
  int32_t *nbr_out, *nbr_in;            /* optional */
  int32_t *status;                      /* int32[8] per problem, zeroed by the caller: [0] coordinate out of range, [1] hash
                                           table exhausted, [2] CSR code overflow, [3] column grid not applicable (see
                                           below), [4] n_heavy of `order`, [5] 1 = no pair lists were written,
                                           [6] n_nonzero and [7] n_single of `order` */
  int32_t n_batch;                      /* batch count (spTensor.batchsize), 0 = unknown: see the column grid below */
  int32_t flags;                        /* PCE_KMAP_* */
  int32_t *order;                       /* optional, needs nbr_out and kv <= 31: the row order of pce_row_order
                                           (pce_row_order_elems(n_out) ints, 16-byte aligned), built with the map at the
                                           cost of three launches per batch; status[4] receives its n_heavy */
} pce_kmap_problem_t;
int pce_kmap_build_batch(const pce_kmap_problem_t *problems_host, int32_t n_problems, pce_stream_t stream);

/* The column grid.  The reference looks neighbours up in a hash table whatever the input
 * (backend/hash.cuh:55-168).  When a problem states its batch count (n_batch > 0), the (b,x,y) box that its
 * geometry bounds (cmin / cmax of the output coordinates) is modest -- at most 2^26 columns and at most
 * 32 n_out + 65536 -- and its workspace has the size pce_kmap_workspace_bytes_grid returns, the build indexes
 * the output coordinates by column instead: one cell per (b,x,y) with the first row of the column and the row
 * behind its last, the rows of a column searched in z.  That needs the output coordinates strictly ascending in
 * (b,x,y,z) order -- what pce_outcoords_emit, pce_voxelize_emit and the reference's sparse_quantize produce --
 * inside the box and with b < n_batch; a build that finds otherwise sets status[3] and leaves its outputs
 * undefined: the caller runs it again with PCE_KMAP_NO_GRID.  Same maps, bit for bit, either way. */
#define PCE_KMAP_NO_GRID 1
/* The caller reads the neighbour table (nbr_out), the row order and the counts (knnz, kpos, qkpos) only -- what the
 * output-stationary dataflows read -- and waives the pair lists: a 3x3x3 submanifold problem over the column grid
 * without CSR outputs and without nbr_in then skips them (status[5] = 1: imap / omap are not written) and is four
 * launches shorter; any other problem ignores the flag.  The reference always compacts its dense map into pair
 * lists (script/spconv.py:370-372). */
#define PCE_KMAP_TABLE_ONLY 2
int64_t pce_kmap_workspace_bytes_grid(int64_t n_in, int64_t n_out, const pce_geom_t *g, int32_t n_batch,
                                      int32_t want_csr);

/* ---- the maps of a whole network in one allocation and two calls ------------------------------- *
 * The reference builds a network's maps layer by layer as its forward pass meets them, each with its own
 * allocations (script/spconv.py:331-437; scratch sizing script/sptensor.py:63-78).  pce_pyramid_plan lays the
 * output coordinates of the strided levels (the chain of pce_outcoords_chain: kernel = stride, no padding, batch
 * count stated) and every requested map out in ONE allocation from upper bounds: level 0 holds at most n_cap rows,
 * level l + 1 at most what pce_outcoords_chain_plan reports for it.  A request names the levels its map reads and
 * writes (equal for a submanifold map; level_out = level_in + 1 for the map of a strided level, whose geometry
 * repeats strided[level_in]) and what it wants beside pair lists, output-major table and row order.  The plan is
 * plain data the caller keeps; arena_bytes is the size of the device allocation it needs (256-byte aligned).
 * pce_pyramid_build then builds everything for one cloud of at most n_cap rows into that allocation -- the chained
 * coordinates, one wait for their counts, all maps in the launches of one batched build, one wait for their counts
 * -- and fills level_n and, per map, n_in / n_out / n_pairs / qsum and the host copy `meta` = knnz[kv] | kpos[kv+1] |
 * qkpos[kv+1] | status[8]; the arrays of map i start at arena + map[i].off[...] (-1: not requested), the
 * coordinates of level l >= 1 at arena + off_coords[l].  PCE_CHAIN_NOT_APPLICABLE (plan) and PCE_PYR_UNSORTED (build:
 * a map found rows unsorted or outside the stated box) tell the caller to build that cloud level by level. */
#define PCE_PYR_MAX_LEVELS 8
#define PCE_PYR_MAX_MAPS 16
#define PCE_PYR_UNSORTED 101
enum { PCE_PYR_IMAP = 0, PCE_PYR_OMAP, PCE_PYR_NBR_OUT, PCE_PYR_NBR_IN, PCE_PYR_ORDER, PCE_PYR_ICSR, PCE_PYR_OCSR, PCE_PYR_ICODE,
       PCE_PYR_OCODE, PCE_PYR_ISLOT, PCE_PYR_OSLOT, PCE_PYR_META, PCE_PYR_WS, PCE_PYR_ARRAYS };
typedef struct pce_pyr_request {
  int32_t level_in, level_out;
  pce_geom_t geom;
  int32_t want_csr, want_nbr_in, table_only, pad;
} pce_pyr_request_t;
typedef struct pce_pyr_map {
  int64_t off[PCE_PYR_ARRAYS];
  int64_t cap_in, cap_out, ws_bytes;
  int64_t n_in, n_out, n_pairs, qsum;   /* filled by pce_pyramid_build */
  int32_t meta[3 * 31 + 2 + 8];
  int32_t kv;
} pce_pyr_map_t;
typedef struct pce_pyr_plan {
  int32_t n_levels, n_maps, n_batch, pad;
  pce_geom_t strided[PCE_PYR_MAX_LEVELS];
  int64_t level_cap[PCE_PYR_MAX_LEVELS + 1], level_n[PCE_PYR_MAX_LEVELS + 1];
  int64_t off_coords[PCE_PYR_MAX_LEVELS + 1], off_chain_ws[PCE_PYR_MAX_LEVELS], chain_ws_bytes[PCE_PYR_MAX_LEVELS];
  int64_t off_meta, meta_bytes, arena_bytes;
  pce_pyr_request_t req[PCE_PYR_MAX_MAPS];
  pce_pyr_map_t map[PCE_PYR_MAX_MAPS];
} pce_pyr_plan_t;
int64_t pce_pyramid_plan_sizeof(void);   /* sizeof(pce_pyr_plan_t) as this library was compiled: a binding checks its own */
int pce_pyramid_plan(int64_t n_cap, int32_t n_levels, const pce_geom_t *strided, int32_t n_batch,
                     const pce_pyr_request_t *requests, int32_t n_requests, pce_pyr_plan_t *plan_out);
int pce_pyramid_build(pce_pyr_plan_t *plan, const int32_t *in_coords_dev, int64_t n_in, void *arena_dev, int64_t arena_bytes,
                      pce_stream_t stream);

/* ---- forward convolution --------------------------------------------------------------------- *
 * Common arguments: in_feats[n_in,c_in], weight[kv,c_in,c_out], out_feats[n_out,c_out], all of
 * `dtype` (PCE_F16: fp16 storage, fp32 accumulate; PCE_F32), row-major, device.
 * mid >= 0 selects the submanifold centre offset handled as a dense GEMM over identical rows
 * (requires n_in == n_out); mid < 0 for strided / transposed layers.
 * For a transposed layer pass the map with the roles swapped (imap<->omap, icsr<->ocsr), as the
 * reference front end does (script/spconv.py:142-151, 236-244). */

/* Fused epilogue of a forward layer: out = act(conv + bias + residual).  bias[c_out] and
 * residual[n_out,c_out] have the layer's dtype and live on the device; either may be NULL.
 * residual must not alias out_feats.  Every forward entry point takes `const pce_epilogue_t *`,
 * NULL for the plain convolution.  The output-stationary, deferred-scatter and dense entry points
 * apply it in the kernel that stores the output rows; fetch-on-demand and gather-GEMM-scatter run
 * one extra in-place pass over the output.  It replaces the separate bias add, activation and
 * residual add of the reference front end (script/spconv.py:453-454, script/activation.py:6-15,
 * script/sptensor.py:80-91); a BatchNorm in inference mode folds into weight and bias beforehand
 * (script/batchnorm.py:7-10). */
enum { PCE_ACT_NONE = 0, PCE_ACT_RELU = 1, PCE_ACT_LEAKY_RELU = 2 };
typedef struct pce_epilogue {
  const void *bias;
  const void *residual;
  int32_t act;         /* PCE_ACT_* */
  float slope;         /* negative slope of PCE_ACT_LEAKY_RELU */
  /* Row strides, in elements, of in_feats and out_feats when they are column slices of wider row-major
   * matrices; 0 = dense (c_in / c_out).  With them the two producers of a skip connection -- the transposed
   * layer and the encoder layer whose output is kept -- write their halves of the concatenated matrix in place
   * and the layers that read one half gather from it, so the concatenation (script/utils.py:152-164) costs no
   * pass over the data.  Multiples of 8 elements, at least the channel count; taken by pce_conv_fwd_fds and
   * pce_conv_fwd_os (any dtype) and pce_conv_fwd_oso, PCE_EINVAL elsewhere.  residual, bias and the partial-row buffer stay dense. */
  int64_t ld_in;
  int64_t ld_out;
} pce_epilogue_t;

/* fp16 weights can be handed over a second time in the order the kernels stage them into LDS
 * (pce_pack_weights, once per weight tensor); every forward entry point takes that copy as
 * `weight_packed`, or NULL to stage from the row-major tensor.  fp32 has no packed form. */
int64_t pce_packed_weight_bytes(int32_t dtype, int32_t kv, int32_t c_in, int32_t c_out);
int pce_pack_weights(const void *weight, int32_t dtype, int32_t kv, int32_t c_in, int32_t c_out,
                     void *packed_dev, pce_stream_t stream);

/* Fetch-on-demand: pairs (imap, omap, kpos, qkpos) and qsum = qkpos[kv] on the host.
 * fp16 needs an fp32 accumulation scratch of pce_conv_fod_workspace_bytes(); fp32 needs none. */
int64_t pce_conv_fod_workspace_bytes(int64_t n_out, int32_t c_out, int32_t dtype);
int pce_conv_fwd_fod(const void *in_feats, const void *weight, const void *weight_packed,
                     void *out_feats, int32_t dtype,
                     int64_t n_in, int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv,
                     int32_t mid, const int32_t *imap_dev, const int32_t *omap_dev,
                     const int32_t *kpos_dev, const int32_t *qkpos_dev, int64_t qsum,
                     void *ws_dev, int64_t ws_bytes, const pce_epilogue_t *epilogue, pce_stream_t stream);

/* pce_conv_fwd_fod without the workspace argument, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid it).  It has no counterpart in the
 * reference.  The fp32 accumulator of the fp16 dataflow lives in a static device array inside the library,
 * pce_conv_fod_static_capacity_bytes() = 32 MiB per GPU the library runs on, held until the process ends;
 * a layer whose accumulator (n_out * c_out * 4 bytes) is larger returns PCE_ECAPACITY.  PCE_F32 needs no
 * accumulator and has no size limit.  The call allocates nothing (no hipMalloc / hipFree, no allocating
 * library routine) and clears nothing with hipMemsetAsync: the centre GEMM, or a fill kernel when the layer
 * has no centre offset, overwrites the accumulator rows before they are added to.  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (different streams or host threads) race and
 * must be serialised by the caller.  Same results as pce_conv_fwd_fod up to the order of its fp32 atomic
 * additions.
 * The device address of the array is looked up once per device, with hipGetSymbolAddress under a mutex, on
 * the first call on that device: a caller that captures calls into a HIP graph runs
 * pce_conv_fod_static_init() on the device beforehand, outside the capture (it does that look-up and nothing
 * else; an uncaptured first call of pce_conv_fwd_fod_static serves as well). */
int64_t pce_conv_fod_static_capacity_bytes(void);
int pce_conv_fod_static_init(void);
int pce_conv_fwd_fod_static(const void *in_feats, const void *weight, const void *weight_packed,
                            void *out_feats, int32_t dtype,
                            int64_t n_in, int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv,
                            int32_t mid, const int32_t *imap_dev, const int32_t *omap_dev,
                            const int32_t *kpos_dev, const int32_t *qkpos_dev, int64_t qsum,
                            const pce_epilogue_t *epilogue, pce_stream_t stream);

/* Gather - GEMM - scatter: CSR-coded map; `buffer` holds qsum*(c_in+c_out) elements of dtype
 * (first qsum*c_in gathered inputs, then the GEMM outputs; backend/spconv.cu:121). */
int pce_conv_fwd_gms(const void *in_feats, const void *weight, const void *weight_packed,
                     void *out_feats, int32_t dtype,
                     int64_t n_in, int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv,
                     int32_t mid, const int32_t *icsr_dev, const int32_t *icode_dev,
                     const int32_t *ocsr_dev, const int32_t *ocode_dev, const int32_t *kpos_dev,
                     const int32_t *qkpos_dev, int64_t qsum, void *buffer_dev,
                     int64_t buffer_elems, const pce_epilogue_t *epilogue, pce_stream_t stream);

/* Fetch-on-demand with deferred scatter.  Gather side: the pair list (imap, kpos, qkpos).  Scatter
 * side: oslot[p] = position of pair p among the entries of its output row in CSR order, and the
 * row pointers ocsr.  Pair tiles store their partial row at buffer[oslot[p]]; the epilogue of the
 * centre GEMM (or a row-sum kernel when there is no centre offset) adds rows
 * buffer[ocsr[o] .. ocsr[o+1]) in fp32 and stores output row o once.  `buffer` holds
 * n_pairs*c_out elements of dtype.  kpos_host / qkpos_host are optional host copies of kpos / qkpos
 * (kv+1 entries): with them the kernels take the offsets from their arguments.
 * omap_dev (optional, may be NULL) is the output row of every pair.  With it, and 16-byte aligned
 * rows of at most 64 channels, a submanifold layer runs as two launches: pair tiles and centre
 * GEMM together (neither reads what the other writes), then one pass over the pairs that adds
 * each output row's partial rows to the centre term already stored there.  Rows with partial
 * rows are then rounded to dtype twice (centre term, final sum).
 * buffer_dev may be NULL when the layer has no centre offset (mid < 0), omap_dev is given and
 * n_pairs == n_out: the caller then states that every output row has exactly one pair (a transposed
 * layer whose kernel size equals its stride: every fine voxel has one parent), and each pair's product
 * is stored straight to its output row with the epilogue, without partial rows or a second pass.
 * route_dev (optional, may be NULL; the array filled by pce_pair_route) routes the pairs of a layer
 * without centre offset: a pair that is the only one of its output row stores the finished row with
 * the epilogue, the others store partial rows, and the row sum visits only the rows whose pair count is
 * not one (a strided layer whose kernel equals its stride on a surface-like cloud has one pair for
 * nearly every row).  Used for fp16 layers with c_in >= 64 a multiple of 32 and c_out >= 96 when the
 * host copies of kpos / qkpos are given; ignored otherwise.  Without an epilogue the output equals that
 * of the unrouted call bit for bit; with one, a single-pair row is rounded to dtype once instead of twice.
 * The array must have been built from this call's omap_dev / oslot_dev / ocsr_dev with the same n_pairs and
 * n_out (its entries are row indices the kernels store to, trusted like the map arrays themselves).
 * No counterpart in the reference: it is ConvolutionForwardD2 with the atomic scatter-add replaced
 * by the output-stationary sum of ConvolutionForwardD1 (backend/spconv.cu:149-161), fused with
 * the centre GEMM. */
int pce_conv_fwd_fds(const void *in_feats, const void *weight, const void *weight_packed,
                     void *out_feats, int32_t dtype, int64_t n_in, int64_t n_out, int32_t c_in,
                     int32_t c_out, int32_t kv, int32_t mid, const int32_t *imap_dev,
                     const int32_t *omap_dev, const int32_t *oslot_dev, const int32_t *kpos_dev,
                     const int32_t *qkpos_dev,
                     const int32_t *kpos_host, const int32_t *qkpos_host, const int32_t *ocsr_dev,
                     const int32_t *route_dev, int64_t n_pairs, int64_t qsum, void *buffer_dev,
                     int64_t buffer_elems, const pce_epilogue_t *epilogue, pce_stream_t stream);

/* Routing array of a layer without centre offset for pce_conv_fwd_fds, int32 on the device:
 *   route[0]              number of output rows whose pair count is not one (route[1..3] are zero)
 *   route[4 .. 4+M)       destination of pair p: omap[p] when p is the only pair of its output row (ocsr
 *                         tells), else n_out + oslot[p]
 *   route[4+M .. 4+M+n_out)  the rows whose pair count is not one, route[0] of them, in no particular order
 * pce_pair_route_elems gives the length (4 + n_pairs + n_out); n_out + n_pairs must stay below 2^31.
 * Two launches on `stream`, no read-back.  No counterpart in the reference, whose fetch-on-demand
 * kernels add every pair's product atomically (backend/spconv.cuh:1567-1730). */
int64_t pce_pair_route_elems(int64_t n_pairs, int64_t n_out);
int pce_pair_route(const int32_t *omap_dev, const int32_t *oslot_dev, const int32_t *ocsr_dev,
                   int64_t n_pairs, int64_t n_out, int32_t *route_dev, int64_t route_elems,
                   pce_stream_t stream);

/* Output-stationary: nbr[kv*n_out] from pce_kmap_build (for a transposed layer, a table built
 * with the roles swapped).  One kernel, one store per output row.  No counterpart in the
 * reference: it is the same fetch-on-demand computation with the scatter-add replaced by
 * register accumulation. */
int pce_conv_fwd_os(const void *in_feats, const void *weight, const void *weight_packed,
                    void *out_feats, int32_t dtype,
                    int64_t n_in, int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv,
                    const int32_t *nbr_dev, const pce_epilogue_t *epilogue, pce_stream_t stream);

/* Output-stationary over ordered rows, for narrow layers on clouds where most voxels have few
 * neighbours (surfaces: 0.2 pairs per voxel on a 64 x 2048 LiDAR scan at 0.1 m).
 *
 * pce_row_order derives from the output-major neighbour table, once per map, the order in which the rows are
 * visited -- rows without neighbours first, in their own order, then the rows with one neighbour sorted by its
 * offset, the rows with two sorted by (lowest, second-lowest) offset, the rows with three or more likewise -- and
 * what the kernels read of every row:
 *   order_dev = perm[n_rows] | mask[n_rows] | 8192 ints of scratch
 *             | rec[n_rows]  (16 bytes each, at the positions of rows with a neighbour: {row, mask, neighbour at
 *                             the lowest offset of the mask, neighbour at the second-lowest or -1})
 *             | srec[n_rows / 8 + 32]  (128 bytes each, for the i-th row with two neighbours or more: {row, mask,
 *                             neighbour at offset 0 ... 29, -1 where there is none}; written only where those
 *                             rows are at most n_rows / 8 + 32)
 * pce_row_order_elems(n_rows) ints in all, 16-byte aligned; kv <= 31; four launches and one wait for counts_host[0]
 * = n_heavy, the number of rows with three neighbours or more, counts_host[1] = n_nonzero, the number with any
 * neighbour, and counts_host[2] = n_single, the number with exactly one.  The positions of rows with equal keys
 * depend on the run, the results of the layer do not.  pce_kmap_build_batch builds the same with the map (status
 * words 4, 6, 7).
 *
 * pce_conv_fwd_oso runs the layer as one launch over that order and takes the three counts as
 * order_counts_host: THE COUNTS THAT CAME WITH THIS ORDER (the kernels find a row's records by them; counts of
 * another order make them read rows that do not exist), or -1 for n_nonzero and n_single when they are not known.
 * A wavefront takes 32 rows of the order, multiplies their centre rows, gathers for each offset any of them has
 * the neighbours of the rows that have it, and stores each finished row once (epilogue fused); chunks of rows with
 * two neighbours or more (three or more when only n_heavy is stated) go to a workgroup whose four wavefronts share
 * the offsets.  With all counts stated, a centre offset (mid >= 0), PCE_F16 with 48-64 input channels, at most half
 * the rows with a neighbour, at most an eighth with two or more, and few enough rows that all workgroups are
 * resident at once, the launch has three kinds of workgroup instead: the bulk of the rows streamed in storage
 * order, 64 per wavefront, stored where their mask is empty; rows with one neighbour by their 16-byte records; rows
 * with two or more by their 128-byte records, 32 to a workgroup whose wavefronts split the input channels.
 *
 * Layers taken (pce_conv_oso_takes): PCE_F16 with packed weights, c_in a multiple of 16 and c_out of 8: both at most
 * 64; or c_in 64..128 with c_out 65..128 and (c_in / 16) * ceil(c_out / 32) <= 24 (these stream an offset's
 * weights from the packed copy K step by K step); PCE_F32: c_in and c_out multiples of 8 and at most 32
 * (weight_packed is not read) and mid >= 0; PCE_EINVAL otherwise.  In PCE_F16 a layer without a centre offset
 * (mid = -1: a strided layer, n_in != n_out, nbr_dev = its output-major table [kv][n_out], order from pce_row_order
 * with mid = -1) runs the same way from zero sums: every output row of a 2x2x2 stride-2 layer has one to eight pairs,
 * the order groups the rows by where they have them.  Takes the row strides of pce_epilogue_t.  No counterpart in
 * the reference: it computes what the fetch-on-demand kernels compute (backend/spconv.cuh:1567-1730) with the
 * scatter-add replaced by register accumulation, as pce_conv_fwd_os. */
int64_t pce_row_order_elems(int64_t n_rows);
int pce_row_order(const int32_t *nbr_dev, int32_t kv, int64_t n_rows, int32_t mid, int32_t *order_dev,
                  int64_t order_elems, int64_t *counts_host /* [3] */, pce_stream_t stream);
int pce_conv_fwd_oso(const void *in_feats, const void *weight, const void *weight_packed,
                     void *out_feats, int32_t dtype,
                     int64_t n_in, int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid,
                     const int32_t *nbr_dev, const int32_t *order_dev, const int64_t *order_counts_host /* [3] */,
                     const pce_epilogue_t *epilogue, pce_stream_t stream);

/* ---- batch normalisation over the rows of a feature matrix ------------------------------------- *
 * The reference normalises the features of a sparse tensor with torch.nn.BatchNorm1d
 * (script/batchnorm.py:7-10).  Its forward and backward passes are two column reductions and two
 * per-column affine maps over feats[n,c] (dtype PCE_F16 or PCE_F32, row-major, device); the c-element
 * arithmetic between them (mean, variance, running statistics, coefficients) is the caller's.
 *   pce_col_sums:   out[j] = sum_r a[r][j],  out[c+j] = sum_r a[r][j] * b[r][j]   (b NULL: b = a)
 *                   fp64 results, same bits every run; ws holds pce_col_sums_workspace_bytes(n, c)
 *                   forward statistics: (x, NULL); backward: (dy, x)
 *   pce_col_affine: y[r][j] = act(x[r][j]*kx[j] + d[r][j]*kd[j] + k0[j])   (d, kd NULL: no second term)
 *                   forward: kx = w*rstd, k0 = b - mean*kx; backward dx: x := dy, d := x,
 *                   kx = w*rstd, kd = -w*rstd^2*S/n, k0 = -w*rstd*sum(dy)/n + w*rstd^2*mean*S/n,
 *                   S = sum(dy * xhat).  y may alias x or d. */
int64_t pce_col_sums_workspace_bytes(int64_t n, int32_t c);
int pce_col_sums(const void *a_dev, const void *b_dev, int32_t dtype, int64_t n, int32_t c, void *ws_dev,
                 int64_t ws_bytes, double *out_dev /* [2c] */, pce_stream_t stream);
int pce_col_affine(const void *x_dev, const void *d_dev, void *y_dev, int32_t dtype, int64_t n, int32_t c,
                   const float *kx_dev, const float *kd_dev, const float *k0_dev, int32_t act, float slope,
                   pce_stream_t stream);
/* The whole pass in one call (three launches: partial sums, one wavefront per channel for the statistics
 * and coefficients, the affine map).  weight, bias (fp32 [c], NULL: 1 and 0), running_mean / running_var
 * (fp32 [c]; updated in place with `momentum` and the unbiased variance when use_batch_stats and
 * momentum >= 0; read when !use_batch_stats) follow torch.nn.BatchNorm1d.  save_mean / save_rstd (fp32 [c])
 * receive what pce_bn_backward needs.  grad_weight / grad_bias (fp32 [c]) may be NULL.  ws: device,
 * pce_bn_workspace_bytes(n, c).  y may alias x; dx may alias dy.
 * The block that follows the norm in the reference's networks -- the residual sum of spTensor.__add__
 * (script/sptensor.py:80-91) and the ReLU / LeakyReLU of script/activation.py:6-15 -- can ride on the same
 * passes: forward y = act(bn(x) + residual) (residual_dev [n,c] of the same dtype, or NULL); backward takes
 * dy with respect to y together with y itself (y_act_dev) and the activation, multiplies dy by the
 * activation's derivative (y > 0 ? 1 : 0 or slope) while it reads it, and returns the gradient with respect
 * to x; the gradient with respect to the residual is that masked dy, which the caller forms itself when it
 * needs it (then it passes the masked dy and PCE_ACT_NONE).  LeakyReLU needs slope > 0. */
int64_t pce_bn_workspace_bytes(int64_t n, int32_t c);
int pce_bn_forward(const void *x_dev, const void *residual_dev, void *y_dev, int32_t dtype, int64_t n, int32_t c,
                   const float *weight_dev, const float *bias_dev, float *running_mean_dev, float *running_var_dev,
                   int32_t use_batch_stats, float momentum, float eps, float *save_mean_dev,
                   float *save_rstd_dev, void *ws_dev, int64_t ws_bytes, int32_t act, float slope,
                   pce_stream_t stream);
int pce_bn_backward(const void *x_dev, const void *dy_dev, const void *y_act_dev, int32_t act, float slope,
                    void *dx_dev, int32_t dtype, int64_t n, int32_t c, const float *weight_dev,
                    const float *save_mean_dev, const float *save_rstd_dev, int32_t use_batch_stats,
                    float *grad_weight_dev, float *grad_bias_dev, void *ws_dev, int64_t ws_bytes,
                    pce_stream_t stream);

/* out[n, c_a + c_b] = (a[n, c_a], b[n, c_b]): the skip concatenation of the reference's `cat`
 * (script/utils.py:152-164) for two tensors on the same rows.  Rows must be whole 16-byte vectors
 * (c_a, c_b multiples of 8 for PCE_F16, 4 for PCE_F32) and the pointers 16-byte aligned (PCE_EINVAL
 * otherwise: the caller concatenates some other way); at most 256 vectors per output row. */
int pce_concat_cols(const void *a_dev, int32_t c_a, const void *b_dev, int32_t c_b, void *out_dev, int32_t dtype,
                    int64_t n, pce_stream_t stream);

/* out[n,c_out] = in[n,c_in] * weight[c_in,c_out]: the 1x1 stride-1 shortcut of the front end
 * (script/spconv.py:297-304), on the same MFMA tile kernel. */
int pce_conv_fwd_dense(const void *in_feats, const void *weight, const void *weight_packed,
                       void *out_feats, int32_t dtype,
                       int64_t n, int32_t c_in, int32_t c_out, const pce_epilogue_t *epilogue,
                       pce_stream_t stream);

/* ---- backward ------------------------------------------------------------------------------- *
 * Replaces ConvolutionBackwardD1 (backend/spconv.h:43-58, backend/spconv.cu:400-629).
 * The gradient with respect to the features is a forward call: pass grad_out as in_feats, the
 * kernel with every offset transposed ([kv, c_out, c_in]) as weight and the map with the roles
 * swapped; any forward entry point and dataflow serves.  The gradient with respect to the kernel is
 * pce_conv_wgrad: grad_w[kp] = sum over the pairs of offset kp of in_feats[imap[p]]^T (x)
 * grad_out[omap[p]], plus in_feats^T * grad_out for the centre offset when mid >= 0.  grad_w is
 * fp32 [kv, c_in, c_out] whatever `dtype` the features have; the call zeroes it first.  Pair lists
 * as for pce_conv_fwd_fod (swap imap / omap for a transposed layer; n_in rows of in_feats, n_out
 * rows of grad_out).  Products are accumulated in fp32 on the matrix cores (fp16 tensors on the fp16
 * MFMA, fp32 tensors on the fp32 MFMA) and runs of pair tiles are combined with fp32 atomic adds, so
 * the last bits of grad_w depend on the order in which workgroups finish (1e-7 relative from run
 * to run); a 1x1 layer is the call with kv = 1, mid = 0, qsum = 0 and no pair lists. */
int pce_conv_wgrad(const void *in_feats, const void *grad_out, int32_t dtype, int64_t n_in,
                   int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid,
                   const int32_t *imap_dev, const int32_t *omap_dev, const int32_t *kpos_dev,
                   const int32_t *qkpos_dev, int64_t qsum, float *grad_w_f32_dev, pce_stream_t stream);

/* Per-layer dataflow choice from map density (pairs per output row), channel widths and the layer's kind:
 * `mid` as in the forward entry points (the centre offset of a submanifold layer, -1 otherwise), `transposed`
 * 1 for a transposed layer (n_in / n_out are then the rows read and written by that layer, i.e. the map's
 * swapped).  Returns a PCE_DATAFLOW_* code whose entry point takes the layer: PCE_DATAFLOW_OSO only where
 * pce_conv_oso_takes() is 1 and the layer is not transposed.  (Replaces the reference's fixed choice per layer
 * class, PCEngine/script/spconv.py:94-124: D1 or D2 by the tag the model file sets.) */
int pce_select_dataflow(int64_t n_in, int64_t n_out, int64_t n_pairs, int32_t c_in, int32_t c_out,
                        int32_t kv, int32_t mid, int32_t transposed, int32_t dtype);

/* 1 when pce_conv_fwd_oso takes a layer of this dtype, these widths, kernel volume and centre offset (it checks
 * alignment and the packed weights besides), else 0. */
int pce_conv_oso_takes(int32_t dtype, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid);

#ifdef __cplusplus
}
#endif
#endif /* PCENGINE_AMD_H */
