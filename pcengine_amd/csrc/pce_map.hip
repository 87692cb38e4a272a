// Coordinate hash table, output-coordinate generation and kernel-map construction for gfx950.
//
// All kernels are integer / byte work bound by HBM and L2 traffic: one lane per voxel row, row
// indices contiguous across a wavefront so that every table of the form t[kp * n + row] is read and
// written with full 256-byte wave transactions; per-offset ranks come from wave ballots, so the
// (offset, input row) order of the pair list is fixed by construction and needs no atomics.
#include <stdarg.h>
#include <string.h>

#include <mutex>

#include "pce_common.h"

// ------------------------------------------------------------------------------------------------
// host-side error text
// ------------------------------------------------------------------------------------------------
static thread_local char g_err[512] = "";

void pce_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char *pce_last_error(void) { return g_err; }
extern "C" int pce_version(void) { return PCE_ABI_VERSION; }

// ------------------------------------------------------------------------------------------------
// small device helpers
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned long long lanemask_lt() {
  unsigned lane = __lane_id();
  return lane == 0 ? 0ull : (~0ull >> (64 - lane));
}

__global__ void fill_u32_kernel(unsigned *p, long long n, unsigned v) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  long long step = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = v;
}

static int fill_u32(void *p, int64_t n_words, unsigned v, hipStream_t s) {
  if (n_words <= 0) return PCE_OK;
  int64_t blocks = pce_div_up(n_words, 256 * 8);
  if (blocks > 65535 * 16) blocks = 65535 * 16;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (unsigned *)p,
                     (long long)n_words, v);
  PCE_LAUNCH_CHECK("fill_u32");
  return PCE_OK;
}

// ------------------------------------------------------------------------------------------------
// hash table
// ------------------------------------------------------------------------------------------------
// Insert key -> row.  Equal keys keep the smallest row, so the table content does not depend on
// the order in which lanes arrive.  The probe loop is bounded by the slot count.
__device__ __forceinline__ bool table_insert(pce_slot_t *table, unsigned long long slots,
                                             unsigned long long key, unsigned row, bool *was_new) {
  unsigned long long s = pce_home_slot(key, slots);
  for (unsigned long long it = 0; it < slots; ++it) {
    unsigned long long prev = atomicCAS(&table[s].key, PCE_EMPTY_KEY, key);
    if (prev == PCE_EMPTY_KEY || prev == key) {
      atomicMin(&table[s].row, row);
      if (was_new) *was_new = (prev == PCE_EMPTY_KEY);
      return true;
    }
    s = (s + 1) & (slots - 1);
  }
  return false;
}

__device__ __forceinline__ int table_find(const pce_slot_t *__restrict__ table,
                                          unsigned long long slots, unsigned long long key) {
  unsigned long long s = pce_home_slot(key, slots);
  for (unsigned long long it = 0; it < slots; ++it) {
    // one 16-byte load returns key and row together
    const uint4 e = *reinterpret_cast<const uint4 *>(&table[s]);
    unsigned long long k = ((unsigned long long)e.y << 32) | e.x;
    if (k == key) return (int)e.z;
    if (k == PCE_EMPTY_KEY) return -1;
    s = (s + 1) & (slots - 1);
  }
  return -1;
}

__global__ void __launch_bounds__(256) hash_insert_kernel(pce_slot_t *table, unsigned long long slots,
                                                          const int4 *__restrict__ coords,
                                                          long long n, int *status) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int4 c = coords[i];
  if (!pce_coord_ok(c.x, c.y, c.z, c.w)) {
    status[0] = 1;
    return;
  }
  if (!table_insert(table, slots, pce_pack_key(c.x, c.y, c.z, c.w), (unsigned)i, nullptr)) status[1] = 1;
}

__global__ void __launch_bounds__(256) hash_query_kernel(const pce_slot_t *__restrict__ table,
                                                         unsigned long long slots,
                                                         const int4 *__restrict__ q, long long nq,
                                                         int *__restrict__ rows) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nq) return;
  int4 c = q[i];
  rows[i] = pce_coord_ok(c.x, c.y, c.z, c.w) ? table_find(table, slots, pce_pack_key(c.x, c.y, c.z, c.w)) : -1;
}

extern "C" int64_t pce_hash_slots(int64_t n) {
  int64_t p = 1;
  while (p < n) p <<= 1;
  int64_t s = 2 * p;
  return s < 8 ? 8 : s;
}

extern "C" int64_t pce_hash_table_bytes(int64_t n) { return pce_hash_slots(n) * (int64_t)sizeof(pce_slot_t); }

static int table_clear(void *table, int64_t slots, hipStream_t s) {
  return fill_u32(table, slots * 4, 0xFFFFFFFFu, s);
}

extern "C" int pce_hash_build(void *table, int64_t slots, const int32_t *coords, int64_t n,
                              int32_t *status, pce_stream_t stream) {
  hipStream_t s = (hipStream_t)stream;
  if (!table || !status || (n > 0 && !coords)) PCE_FAIL(PCE_EINVAL, "pce_hash_build: null pointer");
  if (slots < 8 || (slots & (slots - 1)) || slots < 2 * n)
    PCE_FAIL(PCE_EINVAL, "pce_hash_build: slots=%lld must be a power of two >= 2*n", (long long)slots);
  if (n >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "pce_hash_build: n=%lld exceeds int32 rows", (long long)n);
  int rc = table_clear(table, slots, s);
  if (rc) return rc;
  if (n == 0) return PCE_OK;
  hipLaunchKernelGGL(hash_insert_kernel, dim3((unsigned)pce_div_up(n, 256)), dim3(256), 0, s,
                     (pce_slot_t *)table, (unsigned long long)slots, (const int4 *)coords, (long long)n, status);
  PCE_LAUNCH_CHECK("hash_insert");
  return PCE_OK;
}

extern "C" int pce_hash_query(const void *table, int64_t slots, const int32_t *q, int64_t nq,
                              int32_t *rows, pce_stream_t stream) {
  if (!table || (nq > 0 && (!q || !rows))) PCE_FAIL(PCE_EINVAL, "pce_hash_query: null pointer");
  if (slots < 8 || (slots & (slots - 1))) PCE_FAIL(PCE_EINVAL, "pce_hash_query: slots must be a power of two");
  if (nq == 0) return PCE_OK;
  hipLaunchKernelGGL(hash_query_kernel, dim3((unsigned)pce_div_up(nq, 256)), dim3(256), 0, (hipStream_t)stream,
                     (const pce_slot_t *)table, (unsigned long long)slots, (const int4 *)q, (long long)nq, rows);
  PCE_LAUNCH_CHECK("hash_query");
  return PCE_OK;
}

// ------------------------------------------------------------------------------------------------
// exclusive scan of int32 in place (three launches, any length)
// ------------------------------------------------------------------------------------------------
#define SCAN_ITEMS 8
#define SCAN_TILE (256 * SCAN_ITEMS)

__device__ __forceinline__ int wave_inclusive_scan(int v) {
#pragma unroll
  for (int d = 1; d < PCE_WAVE; d <<= 1) {
    int t = __shfl_up(v, d, PCE_WAVE);
    if ((int)__lane_id() >= d) v += t;
  }
  return v;
}

// exclusive prefix of v over the 256 threads of the block; *total = block sum
__device__ __forceinline__ int block_exclusive_scan(int v, int *total) {
  __shared__ int wsum[4];
  int inc = wave_inclusive_scan(v);
  int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 63) wsum[wave] = inc;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += wsum[w];
  *total = wsum[0] + wsum[1] + wsum[2] + wsum[3];
  __syncthreads();
  return base + inc - v;
}

// Two launches for up to two arrays at once: (1) every block scans its SCAN_TILE items in place
// (exclusive) and records its total; (2) every block adds the totals of the blocks before it in
// the same array.  Blocks [0, nbA) belong to array A, the rest to array B.
struct ScanPair {
  int *a;
  long long na;
  int *b;
  long long nb;
  int blocks_a;
  const unsigned *popc_a;  // when set, the input of array A is popcount(popc_a[i]) instead of a[i]
};

__device__ __forceinline__ void scan_pick(const ScanPair &p, int *&data, long long &n, int &blk) {
  if ((int)blockIdx.x < p.blocks_a) {
    data = p.a;
    n = p.na;
    blk = blockIdx.x;
  } else {
    data = p.b;
    n = p.nb;
    blk = blockIdx.x - p.blocks_a;
  }
}

__global__ void __launch_bounds__(256) scan_local_kernel(ScanPair p, int *__restrict__ sums) {
  int *data;
  long long n;
  int blk;
  scan_pick(p, data, n, blk);
  long long base = (long long)blk * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
  int v[SCAN_ITEMS];
  int acc = 0;
  const bool popc = p.popc_a && (int)blockIdx.x < p.blocks_a;
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j) {
    v[j] = 0;
    if (base + j < n) v[j] = popc ? __popc(p.popc_a[base + j]) : data[base + j];
    acc += v[j];
  }
  int total;
  int run = block_exclusive_scan(acc, &total);
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j) {
    if (base + j < n) data[base + j] = run;
    run += v[j];
  }
  if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

__global__ void __launch_bounds__(256) scan_add_kernel(ScanPair p, const int *__restrict__ sums) {
  int *data;
  long long n;
  int blk;
  scan_pick(p, data, n, blk);
  if (blk == 0) return;
  int first = (int)blockIdx.x - blk;  // first block of this array
  int acc = 0;
  for (int j = threadIdx.x; j < blk; j += 256) acc += sums[first + j];
  int total;
  block_exclusive_scan(acc, &total);
  long long base = (long long)blk * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j)
    if (base + j < n) data[base + j] += total;
}

static int64_t scan_tmp_ints(int64_t n) { return pce_div_up(n, SCAN_TILE) + 1; }

// exclusive scans of a[0..na) and b[0..nb) in place (b may be null); tmp holds one int per block
static int scan_exclusive2(int *a, int64_t na, int *b, int64_t nb, int *tmp, hipStream_t s,
                           const unsigned *popc_a = nullptr) {
  ScanPair p;
  p.popc_a = popc_a;
  p.a = a;
  p.na = na;
  p.b = b;
  p.nb = b ? nb : 0;
  p.blocks_a = (int)pce_div_up(na, SCAN_TILE);
  int blocks = p.blocks_a + (int)pce_div_up(p.nb, SCAN_TILE);
  if (blocks <= 0) return PCE_OK;
  hipLaunchKernelGGL(scan_local_kernel, dim3(blocks), dim3(256), 0, s, p, tmp);
  PCE_LAUNCH_CHECK("scan_local");
  if (p.blocks_a > 1 || blocks - p.blocks_a > 1) {
    hipLaunchKernelGGL(scan_add_kernel, dim3(blocks), dim3(256), 0, s, p, (const int *)tmp);
    PCE_LAUNCH_CHECK("scan_add");
  }
  return PCE_OK;
}

static int scan_exclusive(int *data, int64_t n, int *tmp, hipStream_t s) {
  return scan_exclusive2(data, n, nullptr, 0, tmp, s);
}

// ------------------------------------------------------------------------------------------------
// geometry
// ------------------------------------------------------------------------------------------------
struct GeomDev {
  int ks[3], stride[3], pad[3], cmin[3], cmax[3];
  int bump[3];  // +1 on odd kernel sizes > 1 for strided layers (backend/hash.cuh:235-237)
  int half[3];  // (ks-1)/2
  int subm, kv, mid;
  int sym;  // submanifold layer whose kernel sizes are all odd: pair (i,o,kp) <=> pair (o,i,kv-1-kp)
};

static int make_geom(const pce_geom_t *g, GeomDev *d) {
  if (!g) PCE_FAIL(PCE_EINVAL, "geometry is null");
  int64_t kv = 1;
  for (int a = 0; a < 3; ++a) {
    if (g->ks[a] < 1 || g->stride[a] < 1 || g->pad[a] < 0)
      PCE_FAIL(PCE_EINVAL, "geometry: kernel size and stride must be >= 1, padding >= 0");
    d->ks[a] = g->ks[a];
    d->stride[a] = g->stride[a];
    d->pad[a] = g->pad[a];
    d->cmin[a] = g->cmin[a];
    d->cmax[a] = g->cmax[a];
    d->half[a] = (g->ks[a] - 1) / 2;
    d->bump[a] = (!g->subm && g->ks[a] % 2 == 1 && g->ks[a] > 1) ? 1 : 0;
    kv *= g->ks[a];
  }
  if (kv > 1024) PCE_FAIL(PCE_ECAPACITY, "kernel volume %lld exceeds 1024", (long long)kv);
  d->subm = g->subm ? 1 : 0;
  d->sym = (g->subm && g->ks[0] % 2 == 1 && g->ks[1] % 2 == 1 && g->ks[2] % 2 == 1) ? 1 : 0;
  d->kv = (int)kv;
  d->mid = d->half[0] * g->ks[1] * g->ks[2] + d->half[1] * g->ks[2] + d->half[2];
  if (g->subm && (g->stride[0] != 1 || g->stride[1] != 1 || g->stride[2] != 1))
    PCE_FAIL(PCE_EINVAL, "a submanifold layer has stride 1");
  return PCE_OK;
}

// offset index (ix,iy,iz) -> d(kp), advanced incrementally by the callers
struct OffsetIter {
  int ix, iy, iz;
  __device__ __forceinline__ void init() { ix = iy = iz = 0; }
  __device__ __forceinline__ void next(const GeomDev &g) {
    if (++iz == g.ks[2]) {
      iz = 0;
      if (++iy == g.ks[1]) {
        iy = 0;
        ++ix;
      }
    }
  }
  __device__ __forceinline__ int dx(const GeomDev &g) const { return ix - g.half[0] + g.bump[0]; }
  __device__ __forceinline__ int dy(const GeomDev &g) const { return iy - g.half[1] + g.bump[1]; }
  __device__ __forceinline__ int dz(const GeomDev &g) const { return iz - g.half[2] + g.bump[2]; }
};

// Output coordinate reached from input coordinate c through offset d on one axis of a strided
// layer: (c - d + pad) / stride when it divides and lies in [cmin, cmax]  (backend/hash.cuh:596-605).
__device__ __forceinline__ bool strided_axis(int c, int d, int pad, int stride, int lo, int hi, int *o) {
  int cand = c - d + pad;
  int q = cand / stride;
  *o = q;
  return (cand % stride == 0) && q >= lo && q <= hi;
}

// ------------------------------------------------------------------------------------------------
// output coordinates of a strided layer
// ------------------------------------------------------------------------------------------------
// Two ways to the sorted unique output coordinates.  When the caller bounds the batch count and the
// output bounding box is small enough, every candidate sets one bit of an occupancy bitmap laid
// out in (b,x,y,z) order: a popcount scan then yields count, order and de-duplication at once.
// Otherwise candidates are de-duplicated through a hash table and their codes radix-sorted.
struct BitGrid {
  int lo[3], ext[3];
  int n_batch;
};

struct OutCoordLayout {
  int bitmap;          // 1: occupancy bitmap, 0: hash table + radix sort
  BitGrid grid;
  int64_t words;       // 32-bit words of the bitmap (one spare word of zeros at the end)
  int64_t off_bits, off_cnt;
  int64_t upper;       // bound on the number of candidates that survive
  int64_t slots;       // de-duplication table
  int64_t off_table, off_codes_a, off_codes_b, off_hist, off_scan, off_counters, total;
  int64_t sort_blocks;
};

#define SORT_KEYS_PER_BLOCK 1024  // one wavefront per block, 16 rounds of 64 keys
#define BITMAP_MAX_BITS (1ll << 28)

static void outcoord_layout(int64_t n_in, const GeomDev &g, int n_batch, OutCoordLayout *L) {
  int64_t per = 1;
  for (int a = 0; a < 3; ++a) per *= pce_div_up(g.ks[a], g.stride[a]);
  L->upper = n_in * per;
  if (L->upper < 1) L->upper = 1;
  L->bitmap = 0;
  L->words = 0;
  if (n_batch > 0) {
    int64_t bits = n_batch;
    bool ok = true;
    for (int a = 0; a < 3; ++a) {
      int lo = g.cmin[a] > 0 ? g.cmin[a] : 0;
      int hi = g.cmax[a] < PCE_COORD_BOUND - 1 ? g.cmax[a] : PCE_COORD_BOUND - 1;
      L->grid.lo[a] = lo;
      L->grid.ext[a] = hi - lo + 1;
      if (hi < lo) ok = false;
      else bits *= (hi - lo + 1);   // <= 32768 * 3259^3 < 2^63
    }
    L->grid.n_batch = n_batch;
    int64_t words = pce_div_up(bits, 32) + 1;
    int64_t dense_enough = 32 * L->upper > (1ll << 16) ? 32 * L->upper : (1ll << 16);
    if (ok && bits <= BITMAP_MAX_BITS && words <= dense_enough) {
      L->bitmap = 1;
      L->words = words;
    }
  }
  if (L->bitmap) {
    int64_t o = 0;
    L->off_bits = o;
    o += pce_align_up(L->words * 4, 256);
    L->off_counters = o;  // directly behind the bitmap: one fill clears both
    o += 256;
    L->off_cnt = o;
    o += pce_align_up(L->words * 4, 256);
    L->off_scan = o;
    o += pce_align_up(scan_tmp_ints(L->words) * 4, 256);
    L->total = o;
    return;
  }
  L->slots = pce_hash_slots(L->upper);
  L->sort_blocks = pce_div_up(L->upper, SORT_KEYS_PER_BLOCK);
  int64_t o = 0;
  L->off_table = o;
  o += pce_align_up(L->slots * 16, 256);
  L->off_codes_a = o;
  o += pce_align_up(L->upper * 8, 256);
  L->off_codes_b = o;
  o += pce_align_up(L->upper * 8, 256);
  L->off_hist = o;
  o += pce_align_up((256 * L->sort_blocks + 1) * 4, 256);
  L->off_scan = o;
  o += pce_align_up(scan_tmp_ints(256 * L->sort_blocks + 1) * 4, 256);
  L->off_counters = o;
  o += 256;
  L->total = o;
}

// status[0]: coordinate out of range, status[2]: batch index >= the caller's batch count
// n_dev (optional): the number of input rows, on the device -- the count a previous level of a chained build left;
// n_in is then the bound the grid was sized for.
__global__ void __launch_bounds__(256) outcoord_mark_kernel(const int4 *__restrict__ coords, long long n_in, GeomDev g,
                                                            BitGrid grid, unsigned *__restrict__ bits, int *status,
                                                            const int *__restrict__ n_dev) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (n_dev) n_in = *n_dev;
  if (i >= n_in) return;
  int4 c = coords[i];
  if (!pce_coord_ok(c.x, c.y, c.z, c.w)) {
    status[0] = 1;
    return;
  }
  if (c.x >= grid.n_batch) {
    status[2] = 1;
    return;
  }
  OffsetIter it;
  it.init();
  for (int kp = 0; kp < g.kv; ++kp, it.next(g)) {
    int ox, oy, oz;
    bool ok = strided_axis(c.y, it.dx(g), g.pad[0], g.stride[0], g.cmin[0], g.cmax[0], &ox);
    ok &= strided_axis(c.z, it.dy(g), g.pad[1], g.stride[1], g.cmin[1], g.cmax[1], &oy);
    ok &= strided_axis(c.w, it.dz(g), g.pad[2], g.stride[2], g.cmin[2], g.cmax[2], &oz);
    if (!ok) continue;
    if (ox < 0 || oy < 0 || oz < 0 || ox >= PCE_COORD_BOUND || oy >= PCE_COORD_BOUND || oz >= PCE_COORD_BOUND) {
      status[0] = 1;
      continue;
    }
    long long bit = (((long long)c.x * grid.ext[0] + (ox - grid.lo[0])) * grid.ext[1] + (oy - grid.lo[1])) * grid.ext[2] +
                    (oz - grid.lo[2]);
    atomicOr(&bits[bit >> 5], 1u << (bit & 31));
  }
}

// cnt[w] = number of set bits before word w (exclusive scan of the popcounts)
__global__ void __launch_bounds__(256) outcoord_expand_kernel(const unsigned *__restrict__ bits, const int *__restrict__ cnt,
                                                              long long words, BitGrid grid, int4 *__restrict__ out) {
  long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (w >= words) return;
  unsigned m = bits[w];
  if (!m) return;
  int o = cnt[w];
  while (m) {
    int b = __ffs((int)m) - 1;
    m &= m - 1;
    long long idx = w * 32 + b;
    int4 c;
    c.w = (int)(idx % grid.ext[2]) + grid.lo[2];
    idx /= grid.ext[2];
    c.z = (int)(idx % grid.ext[1]) + grid.lo[1];
    idx /= grid.ext[1];
    c.y = (int)(idx % grid.ext[0]) + grid.lo[0];
    c.x = (int)(idx / grid.ext[0]);
    out[o++] = c;
  }
}

// counters[0] = number of unique candidates, counters[1] = largest code
__global__ void __launch_bounds__(256) outcoord_candidates_kernel(const int4 *__restrict__ coords, long long n_in,
                                                                  GeomDev g, pce_slot_t *table,
                                                                  unsigned long long slots,
                                                                  unsigned long long *__restrict__ codes,
                                                                  unsigned long long *counters, int *status) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  bool live = i < n_in;
  int4 c = live ? coords[i] : make_int4(0, 0, 0, 0);
  if (live && !pce_coord_ok(c.x, c.y, c.z, c.w)) {
    status[0] = 1;
    live = false;
  }
  OffsetIter it;
  it.init();
  unsigned long long my_max = 0;
  for (int kp = 0; kp < g.kv; ++kp, it.next(g)) {
    bool fresh = false;
    unsigned long long code = 0;
    if (live) {
      int ox, oy, oz;
      bool ok = strided_axis(c.y, it.dx(g), g.pad[0], g.stride[0], g.cmin[0], g.cmax[0], &ox);
      ok &= strided_axis(c.z, it.dy(g), g.pad[1], g.stride[1], g.cmin[1], g.cmax[1], &oy);
      ok &= strided_axis(c.w, it.dz(g), g.pad[2], g.stride[2], g.cmin[2], g.cmax[2], &oz);
      if (ok) {
        if (ox < 0 || oy < 0 || oz < 0 || ox >= PCE_COORD_BOUND || oy >= PCE_COORD_BOUND || oz >= PCE_COORD_BOUND) {
          status[0] = 1;
        } else {
          if (!table_insert(table, slots, pce_pack_key(c.x, ox, oy, oz), 0u, &fresh)) status[1] = 1;
          // base-3259 code whose ascending order is (b,x,y,z) order (backend/hash.cuh:607-608)
          code = (((unsigned long long)c.x * PCE_COORD_BOUND + ox) * PCE_COORD_BOUND + oy) * PCE_COORD_BOUND + oz;
        }
      }
    }
    unsigned long long bal = __ballot(fresh);
    if (bal) {
      unsigned long long base = 0;
      int leader = __ffsll((long long)bal) - 1;
      if ((int)__lane_id() == leader) base = atomicAdd(&counters[0], (unsigned long long)__popcll(bal));
      base = __shfl(base, leader, PCE_WAVE);
      if (fresh) {
        codes[base + __popcll(bal & lanemask_lt())] = code;
        my_max = code > my_max ? code : my_max;
      }
    }
  }
  // wave max, one atomic per wave
  for (int d = 32; d >= 1; d >>= 1) {
    unsigned long long o = __shfl_xor(my_max, d, PCE_WAVE);
    my_max = o > my_max ? o : my_max;
  }
  if (__lane_id() == 0 && my_max) atomicMax(&counters[1], my_max);
}

// --- stable LSD radix sort on 64-bit codes, 8 bits per pass, one wavefront per block -------------
__global__ void __launch_bounds__(64) sort_hist_kernel(const unsigned long long *__restrict__ keys, long long n,
                                                       int shift, int *__restrict__ hist, int nblocks) {
  __shared__ int bins[256];
  for (int j = threadIdx.x; j < 256; j += 64) bins[j] = 0;
  __syncthreads();
  long long base = (long long)blockIdx.x * SORT_KEYS_PER_BLOCK;
  for (int r = 0; r < SORT_KEYS_PER_BLOCK / 64; ++r) {
    long long i = base + r * 64 + threadIdx.x;
    if (i < n) atomicAdd(&bins[(keys[i] >> shift) & 255], 1);
  }
  __syncthreads();
  for (int j = threadIdx.x; j < 256; j += 64) hist[(long long)j * nblocks + blockIdx.x] = bins[j];
}

__global__ void __launch_bounds__(64) sort_scatter_kernel(const unsigned long long *__restrict__ src,
                                                          unsigned long long *__restrict__ dst, long long n,
                                                          int shift, const int *__restrict__ offs, int nblocks) {
  __shared__ int run[256];  // keys of each digit already placed by this block
  for (int j = threadIdx.x; j < 256; j += 64) run[j] = 0;
  __syncthreads();
  long long base = (long long)blockIdx.x * SORT_KEYS_PER_BLOCK;
  for (int r = 0; r < SORT_KEYS_PER_BLOCK / 64; ++r) {
    long long i = base + r * 64 + threadIdx.x;
    bool live = i < n;
    unsigned long long key = live ? src[i] : 0;
    int d = (int)((key >> shift) & 255);
    // lanes holding the same digit
    unsigned long long peers = __ballot(live);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      unsigned long long bal = __ballot((d >> b) & 1);
      peers &= ((d >> b) & 1) ? bal : ~bal;
    }
    int before = 0, old = 0;
    if (live) {
      before = __popcll(peers & lanemask_lt());
      int leader = __ffsll((long long)peers) - 1;
      if (before == 0) {
        old = run[d];
        run[d] = old + __popcll(peers);
      }
      old = __shfl(old, leader, PCE_WAVE);
      dst[(long long)offs[(long long)d * nblocks + blockIdx.x] + old + before] = key;
    }
    __syncthreads();
  }
}

// ascending sort of n 64-bit keys whose values need `bits` bits; the result is in *sorted (a or b)
static int radix_sort_u64(unsigned long long *a, unsigned long long *b, int64_t n, int bits, int *hist, int *scan_tmp,
                          hipStream_t s, unsigned long long **sorted) {
  int passes = (bits + 7) / 8;
  if (passes < 1) passes = 1;
  int nblocks = (int)pce_div_up(n, SORT_KEYS_PER_BLOCK);
  unsigned long long *src = a, *dst = b;
  int rc;
  for (int p = 0; p < passes; ++p) {
    hipLaunchKernelGGL(sort_hist_kernel, dim3(nblocks), dim3(64), 0, s, (const unsigned long long *)src, (long long)n,
                       8 * p, hist, nblocks);
    PCE_LAUNCH_CHECK("sort_hist");
    if ((rc = scan_exclusive(hist, 256ll * nblocks, scan_tmp, s))) return rc;
    hipLaunchKernelGGL(sort_scatter_kernel, dim3(nblocks), dim3(64), 0, s, (const unsigned long long *)src, dst,
                       (long long)n, 8 * p, (const int *)hist, nblocks);
    PCE_LAUNCH_CHECK("sort_scatter");
    unsigned long long *t = src;
    src = dst;
    dst = t;
  }
  *sorted = src;
  return PCE_OK;
}

__global__ void decode_codes_kernel(const unsigned long long *__restrict__ codes, long long n, int4 *__restrict__ out) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  unsigned long long c = codes[i];
  int4 o;
  o.w = (int)(c % PCE_COORD_BOUND);
  c /= PCE_COORD_BOUND;
  o.z = (int)(c % PCE_COORD_BOUND);
  c /= PCE_COORD_BOUND;
  o.y = (int)(c % PCE_COORD_BOUND);
  c /= PCE_COORD_BOUND;
  o.x = (int)c;
  out[i] = o;
}

extern "C" int64_t pce_outcoords_workspace_bytes(int64_t n_in, const pce_geom_t *g, int32_t n_batch) {
  GeomDev gd;
  if (make_geom(g, &gd)) return -1;
  OutCoordLayout L;
  outcoord_layout(n_in, gd, n_batch, &L);
  return L.total;
}

extern "C" int pce_outcoords_build(const int32_t *in_coords, int64_t n_in, const pce_geom_t *g, int32_t n_batch, void *ws,
                                   int64_t ws_bytes, int64_t *n_out_host, pce_stream_t stream) {
  hipStream_t s = (hipStream_t)stream;
  GeomDev gd;
  int rc = make_geom(g, &gd);
  if (rc) return rc;
  if (!in_coords || !ws || !n_out_host) PCE_FAIL(PCE_EINVAL, "pce_outcoords_build: null pointer");
  if (n_in <= 0 || n_in >= (1ll << 31)) PCE_FAIL(PCE_EINVAL, "pce_outcoords_build: n_in=%lld", (long long)n_in);
  OutCoordLayout L;
  outcoord_layout(n_in, gd, n_batch, &L);
  if (ws_bytes < L.total) PCE_FAIL(PCE_EWORKSPACE, "pce_outcoords_build: workspace %lld < %lld", (long long)ws_bytes, (long long)L.total);
  if (L.upper >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "pce_outcoords_build: candidate bound %lld exceeds int32", (long long)L.upper);
  char *w = (char *)ws;
  if (L.bitmap) {
    unsigned *bits = (unsigned *)(w + L.off_bits);
    int *cnt = (int *)(w + L.off_cnt);
    int *status = (int *)(w + L.off_counters);
    if ((rc = fill_u32(bits, (L.off_counters + 256 - L.off_bits) / 4, 0u, s))) return rc;
    hipLaunchKernelGGL(outcoord_mark_kernel, dim3((unsigned)pce_div_up(n_in, 256)), dim3(256), 0, s,
                       (const int4 *)in_coords, (long long)n_in, gd, L.grid, bits, status, (const int *)nullptr);
    PCE_LAUNCH_CHECK("outcoord_mark");
    // the spare last word is zero, so after the scan cnt[words-1] is the number of set bits
    if ((rc = scan_exclusive2(cnt, L.words, nullptr, 0, (int *)(w + L.off_scan), s, bits))) return rc;
    int host[4];
    PCE_HIP(hipMemcpyAsync(&host[0], cnt + (L.words - 1), sizeof(int), hipMemcpyDeviceToHost, s));
    PCE_HIP(hipMemcpyAsync(&host[1], status, 3 * sizeof(int), hipMemcpyDeviceToHost, s));
    PCE_HIP(hipStreamSynchronize(s));
    if (host[1]) PCE_FAIL(PCE_ECOORD, "pce_outcoords_build: coordinate outside [0,%d) or batch index out of range", PCE_COORD_BOUND);
    if (host[3]) PCE_FAIL(PCE_EINVAL, "pce_outcoords_build: a batch index is >= n_batch=%d", (int)n_batch);
    *n_out_host = host[0];
    return PCE_OK;
  }
  pce_slot_t *table = (pce_slot_t *)(w + L.off_table);
  unsigned long long *ca = (unsigned long long *)(w + L.off_codes_a);
  unsigned long long *cb = (unsigned long long *)(w + L.off_codes_b);
  int *hist = (int *)(w + L.off_hist);
  int *scan_tmp = (int *)(w + L.off_scan);
  unsigned long long *counters = (unsigned long long *)(w + L.off_counters);
  if ((rc = table_clear(table, L.slots, s))) return rc;
  if ((rc = fill_u32(counters, 64, 0u, s))) return rc;  // counters[0..1] and status at counters[4..]
  int *status = (int *)(counters + 4);
  hipLaunchKernelGGL(outcoord_candidates_kernel, dim3((unsigned)pce_div_up(n_in, 256)), dim3(256), 0, s,
                     (const int4 *)in_coords, (long long)n_in, gd, table, (unsigned long long)L.slots, ca, counters, status);
  PCE_LAUNCH_CHECK("outcoord_candidates");
  unsigned long long host[6];
  PCE_HIP(hipMemcpyAsync(host, counters, sizeof(host), hipMemcpyDeviceToHost, s));
  PCE_HIP(hipStreamSynchronize(s));
  int hstatus[2];
  memcpy(hstatus, &host[4], sizeof(hstatus));
  if (hstatus[0]) PCE_FAIL(PCE_ECOORD, "pce_outcoords_build: coordinate outside [0,%d) or batch index out of range", PCE_COORD_BOUND);
  if (hstatus[1]) PCE_FAIL(PCE_ECAPACITY, "pce_outcoords_build: de-duplication table exhausted");
  int64_t n = (int64_t)host[0];
  *n_out_host = n;
  if (n == 0) return PCE_OK;
  int bits = 0;
  while (bits < 64 && (host[1] >> bits)) ++bits;
  unsigned long long *src = nullptr;
  if ((rc = radix_sort_u64(ca, cb, n, bits, hist, scan_tmp, s, &src))) return rc;
  if (src != ca) PCE_HIP(hipMemcpyAsync(ca, src, (size_t)n * 8, hipMemcpyDeviceToDevice, s));
  return PCE_OK;
}

extern "C" int pce_outcoords_emit(const void *ws, int64_t n_in, const pce_geom_t *g, int32_t n_batch, int64_t n_out,
                                  int32_t *out_coords, pce_stream_t stream) {
  GeomDev gd;
  int rc = make_geom(g, &gd);
  if (rc) return rc;
  if (!ws || (n_out > 0 && !out_coords)) PCE_FAIL(PCE_EINVAL, "pce_outcoords_emit: null pointer");
  OutCoordLayout L;
  outcoord_layout(n_in, gd, n_batch, &L);
  if (n_out < 0 || n_out > L.upper) PCE_FAIL(PCE_EINVAL, "pce_outcoords_emit: n_out=%lld out of range", (long long)n_out);
  if (n_out == 0) return PCE_OK;
  if (L.bitmap) {
    const char *w = (const char *)ws;
    hipLaunchKernelGGL(outcoord_expand_kernel, dim3((unsigned)pce_div_up(L.words, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const unsigned *)(w + L.off_bits), (const int *)(w + L.off_cnt), (long long)L.words, L.grid,
                       (int4 *)out_coords);
    PCE_LAUNCH_CHECK("outcoord_expand");
    return PCE_OK;
  }
  const unsigned long long *ca = (const unsigned long long *)((const char *)ws + L.off_codes_a);
  hipLaunchKernelGGL(decode_codes_kernel, dim3((unsigned)pce_div_up(n_out, 256)), dim3(256), 0, (hipStream_t)stream, ca,
                     (long long)n_out, (int4 *)out_coords);
  PCE_LAUNCH_CHECK("decode_codes");
  return PCE_OK;
}

// ---- all levels of a chain at once -------------------------------------------------------------------------------
// When every layer of the chain has kernel = stride and no padding (the down-sampling layers of a U-Net), the voxel
// a point falls into at level l is its coordinate divided l times, whatever the other points do: one kernel pushes
// every first-level point through all levels and marks a bit per level, and the scans and the decoding of all
// levels share their launches -- five launches for the chain instead of five per level.
struct ChainLevel {
  unsigned *bits;
  int *cnt, *sums, *status;
  int4 *out;
  long long words, fill_ints;
  int fill_blk0, scan_blk0, word_blk0;   // first block of this level in the fill / scan / decode grids
  BitGrid grid;
  int stride[3], lo[3], hi[3];
};
struct ChainDev {
  int levels;
  int *summary;                           // [levels][4]: count, status[0..2]
  ChainLevel lv[PCE_MAX_CHAIN];
};
#define CHAIN_FILL_INTS 2048              // per block

__device__ __forceinline__ int chain_level_of(const ChainDev &d, int blk, int which) {
  int l = 0;
  for (int i = 1; i < d.levels; ++i) {
    int b0 = which == 0 ? d.lv[i].fill_blk0 : (which == 1 ? d.lv[i].scan_blk0 : d.lv[i].word_blk0);
    if (blk >= b0) l = i;
  }
  return l;
}

__global__ void __launch_bounds__(256) chain_fill_kernel(ChainDev d) {
  const int l = chain_level_of(d, blockIdx.x, 0);
  const ChainLevel &v = d.lv[l];
  long long base = (long long)(blockIdx.x - v.fill_blk0) * CHAIN_FILL_INTS;
  for (int j = threadIdx.x; j < CHAIN_FILL_INTS; j += 256)
    if (base + j < v.fill_ints) v.bits[base + j] = 0u;
}

__global__ void __launch_bounds__(256) chain_mark_kernel(const int4 *__restrict__ coords, long long n_in, ChainDev d) {
  // no lane leaves early: the lanes of a wavefront combine their bits below
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  bool live = i < n_in;
  int4 c = live ? coords[i] : make_int4(0, 0, 0, 0);
  if (live && !pce_coord_ok(c.x, c.y, c.z, c.w)) {
    d.lv[0].status[0] = 1;
    live = false;
  }
  if (live && c.x >= d.lv[0].grid.n_batch) {
    d.lv[0].status[2] = 1;
    live = false;
  }
  const int lane = threadIdx.x & 63;
  int p[3] = {c.y, c.z, c.w};
  for (int l = 0; l < d.levels; ++l) {
    const ChainLevel &v = d.lv[l];
    bool ok = true, bad = false;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      int q = p[a] / v.stride[a];           // kernel = stride, no padding: the one offset that divides ...
      if (p[a] % v.stride[a] < 0) --q;      // ... which is the floor, for a negative coordinate too
      p[a] = q;
      ok &= q >= v.lo[a] && q <= v.hi[a];
      bad |= q < 0 || q >= PCE_COORD_BOUND;
    }
    if (!ok) live = false;                  // clipped here: absent from every deeper level too
    if (live && bad) {                      // inside the stated bounds but outside what a strided layer can address
      d.lv[0].status[0] = 1;
      live = false;
    }
    const long long bit = !live ? 0ll
                                : (((long long)c.x * v.grid.ext[0] + (p[0] - v.grid.lo[0])) * v.grid.ext[1] + (p[1] - v.grid.lo[1])) *
                                          v.grid.ext[2] + (p[2] - v.grid.lo[2]);
    const long long word = bit >> 5;
    const unsigned m = 1u << (bit & 31);
    bool pending = live;
    if (l > 0) {
      // Below the first level many lanes of a wavefront (consecutive points of a sorted cloud) fall into one word:
      // the lanes of up to four words combine their bits and one lane issues the atomic; what is left goes alone.
      unsigned long long todo = __ballot(pending);
      for (int it = 0; it < 4 && todo; ++it) {
        const int leader = __ffsll((long long)todo) - 1;
        const long long lw = ((long long)__shfl((int)(word >> 32), leader, PCE_WAVE) << 32) |
                             (unsigned)__shfl((int)(word & 0xFFFFFFFFll), leader, PCE_WAVE);
        const bool same = pending && word == lw;
        unsigned mm = same ? m : 0u;
#pragma unroll
        for (int dd = 1; dd < PCE_WAVE; dd <<= 1) mm |= (unsigned)__shfl_xor((int)mm, dd, PCE_WAVE);
        if (lane == leader) atomicOr(&v.bits[lw], mm);
        if (same) pending = false;
        todo &= ~__ballot(same);
      }
    }
    if (pending) atomicOr(&v.bits[word], m);
  }
}

__global__ void __launch_bounds__(256) chain_scan_local_kernel(ChainDev d) {
  const int l = chain_level_of(d, blockIdx.x, 1);
  const ChainLevel &v = d.lv[l];
  const int blk = blockIdx.x - v.scan_blk0;
  long long base = (long long)blk * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
  int x[SCAN_ITEMS];
  int acc = 0;
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j) {
    x[j] = base + j < v.words ? __popc(v.bits[base + j]) : 0;
    acc += x[j];
  }
  int total;
  int run = block_exclusive_scan(acc, &total);
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j) {
    if (base + j < v.words) v.cnt[base + j] = run;
    run += x[j];
  }
  if (threadIdx.x == 0) v.sums[blk] = total;
}

__global__ void __launch_bounds__(256) chain_scan_add_kernel(ChainDev d) {
  const int l = chain_level_of(d, blockIdx.x, 1);
  const ChainLevel &v = d.lv[l];
  const int blk = blockIdx.x - v.scan_blk0;
  if (blk == 0) return;
  int acc = 0;
  for (int j = threadIdx.x; j < blk; j += 256) acc += v.sums[j];
  int total;
  block_exclusive_scan(acc, &total);
  long long base = (long long)blk * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j)
    if (base + j < v.words) v.cnt[base + j] += total;
}

__global__ void __launch_bounds__(256) chain_expand_kernel(ChainDev d) {
  const int l = chain_level_of(d, blockIdx.x, 2);
  const ChainLevel &v = d.lv[l];
  long long w = (long long)(blockIdx.x - v.word_blk0) * 256 + threadIdx.x;
  if (w >= v.words) return;
  if (w == v.words - 1) {                   // the spare last word is zero: its prefix is the level's count
    int *sm = d.summary + 4 * l;
    sm[0] = v.cnt[w];
    sm[1] = d.lv[0].status[0];
    sm[2] = d.lv[0].status[1];
    sm[3] = d.lv[0].status[2];
  }
  unsigned m = v.bits[w];
  if (!m) return;
  int o = v.cnt[w];
  while (m) {
    int b = __ffs((int)m) - 1;
    m &= m - 1;
    long long idx = w * 32 + b;
    int4 c;
    c.w = (int)(idx % v.grid.ext[2]) + v.grid.lo[2];
    idx /= v.grid.ext[2];
    c.z = (int)(idx % v.grid.ext[1]) + v.grid.lo[1];
    idx /= v.grid.ext[1];
    c.y = (int)(idx % v.grid.ext[0]) + v.grid.lo[0];
    c.x = (int)(idx / v.grid.ext[0]);
    v.out[o++] = c;
  }
}

// ---- the output coordinates of several strided layers in a row, one wait of the host ---------------------------
// Level l reads the coordinates level l-1 wrote; their number stays on the device (the last word of the scanned
// popcounts) and the launches are sized for its bound, so nothing has to reach the host between the levels.
static int chain_plan(int64_t n_in, int levels, const pce_geom_t *geoms, int32_t n_batch, GeomDev *gd, OutCoordLayout *L,
                      int64_t *bound_in) {
  if (levels < 1 || levels > PCE_MAX_CHAIN || !geoms) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: levels=%d (1..%d)", levels, PCE_MAX_CHAIN);
  if (n_in <= 0 || n_in >= (1ll << 31)) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: n_in=%lld", (long long)n_in);
  int64_t bound = n_in;
  for (int l = 0; l < levels; ++l) {
    int rc = make_geom(&geoms[l], &gd[l]);
    if (rc) return rc;
    bound_in[l] = bound;
    outcoord_layout(bound, gd[l], n_batch, &L[l]);
    if (!L[l].bitmap) return -1;   // not an error: the caller builds level by level
    int64_t cells = (int64_t)L[l].grid.n_batch * L[l].grid.ext[0] * L[l].grid.ext[1] * L[l].grid.ext[2];
    bound = L[l].upper < cells ? L[l].upper : cells;
    if (bound >= (1ll << 31)) return -1;
  }
  return PCE_OK;
}

extern "C" int pce_outcoords_chain_plan(int64_t n_in, int32_t levels, const pce_geom_t *geoms, int32_t n_batch,
                                        int64_t *ws_bytes, int64_t *capacity) {
  GeomDev gd[PCE_MAX_CHAIN];
  OutCoordLayout L[PCE_MAX_CHAIN];
  int64_t bound_in[PCE_MAX_CHAIN];
  if (!ws_bytes || !capacity) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain_plan: null pointer");
  int rc = chain_plan(n_in, levels, geoms, n_batch, gd, L, bound_in);
  if (rc < 0) return PCE_CHAIN_NOT_APPLICABLE;
  if (rc) return rc;
  for (int l = 0; l < levels; ++l) {
    ws_bytes[l] = L[l].total;
    int64_t cells = (int64_t)L[l].grid.n_batch * L[l].grid.ext[0] * L[l].grid.ext[1] * L[l].grid.ext[2];
    capacity[l] = L[l].upper < cells ? L[l].upper : cells;
  }
  return PCE_OK;
}

extern "C" int pce_outcoords_chain(const int32_t *in_coords, int64_t n_in, int32_t levels, const pce_geom_t *geoms,
                                   int32_t n_batch, void *const *ws, const int64_t *ws_bytes, int32_t *const *out_coords,
                                   int64_t *n_out_host, pce_stream_t stream) {
  return pce_outcoords_chain_planned(in_coords, n_in, n_in, levels, geoms, n_batch, ws, ws_bytes, out_coords, n_out_host, stream);
}

// n_plan: the row count the workspaces were laid out for (pce_outcoords_chain_plan); a smaller cloud runs through
// the same layout (whether a level takes the bitmap depends on the row count: a plan must not change its mind)
extern "C" int pce_outcoords_chain_planned(const int32_t *in_coords, int64_t n_in, int64_t n_plan, int32_t levels,
                                           const pce_geom_t *geoms, int32_t n_batch, void *const *ws, const int64_t *ws_bytes,
                                           int32_t *const *out_coords, int64_t *n_out_host, pce_stream_t stream) {
  hipStream_t s = (hipStream_t)stream;
  GeomDev gd[PCE_MAX_CHAIN];
  OutCoordLayout L[PCE_MAX_CHAIN];
  int64_t bound_in[PCE_MAX_CHAIN];
  if (!in_coords || !ws || !ws_bytes || !out_coords || !n_out_host) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: null pointer");
  if (n_in <= 0 || n_in > n_plan) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: %lld rows, planned for %lld", (long long)n_in, (long long)n_plan);
  int rc = chain_plan(n_plan, levels, geoms, n_batch, gd, L, bound_in);
  if (rc < 0) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: a level does not take the occupancy bitmap (ask pce_outcoords_chain_plan first)");
  if (rc) return rc;
  int host[PCE_MAX_CHAIN][4];
  const int4 *src = (const int4 *)in_coords;
  const int *n_dev = nullptr;
  bool all_at_once = levels >= 2;
  for (int l = 0; l < levels; ++l) {
    if (!ws[l] || !out_coords[l]) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: null pointer at level %d", l);
    if (ws_bytes[l] < L[l].total) PCE_FAIL(PCE_EWORKSPACE, "pce_outcoords_chain: workspace %lld < %lld at level %d", (long long)ws_bytes[l], (long long)L[l].total, l);
    for (int a = 0; a < 3; ++a) all_at_once &= gd[l].ks[a] == gd[l].stride[a] && gd[l].pad[a] == 0;
  }
  if (all_at_once) {
    ChainDev d;
    d.levels = levels;
    int fill_blk = 0, scan_blk = 0, word_blk = 0;
    for (int l = 0; l < levels; ++l) {
      char *w = (char *)ws[l];
      ChainLevel &v = d.lv[l];
      v.bits = (unsigned *)(w + L[l].off_bits);
      v.cnt = (int *)(w + L[l].off_cnt);
      v.sums = (int *)(w + L[l].off_scan);
      v.status = (int *)(w + L[l].off_counters);
      v.out = (int4 *)out_coords[l];
      v.words = L[l].words;
      v.fill_ints = (L[l].off_counters + 256 - L[l].off_bits) / 4;   // the bitmap and the counters behind it
      v.fill_blk0 = fill_blk;
      v.scan_blk0 = scan_blk;
      v.word_blk0 = word_blk;
      fill_blk += (int)pce_div_up(v.fill_ints, CHAIN_FILL_INTS);
      scan_blk += (int)pce_div_up(v.words, SCAN_TILE);
      word_blk += (int)pce_div_up(v.words, 256);
      v.grid = L[l].grid;
      for (int a = 0; a < 3; ++a) {
        v.stride[a] = gd[l].stride[a];
        v.lo[a] = gd[l].cmin[a];
        v.hi[a] = gd[l].cmax[a];
      }
    }
    d.summary = d.lv[0].status + 16;          // inside the 256 bytes of counters behind the first level's bitmap
    hipLaunchKernelGGL(chain_fill_kernel, dim3((unsigned)fill_blk), dim3(256), 0, s, d);
    PCE_LAUNCH_CHECK("chain_fill");
    hipLaunchKernelGGL(chain_mark_kernel, dim3((unsigned)pce_div_up(n_in, 256)), dim3(256), 0, s, (const int4 *)in_coords,
                       (long long)n_in, d);
    PCE_LAUNCH_CHECK("chain_mark");
    hipLaunchKernelGGL(chain_scan_local_kernel, dim3((unsigned)scan_blk), dim3(256), 0, s, d);
    PCE_LAUNCH_CHECK("chain_scan_local");
    hipLaunchKernelGGL(chain_scan_add_kernel, dim3((unsigned)scan_blk), dim3(256), 0, s, d);
    PCE_LAUNCH_CHECK("chain_scan_add");
    hipLaunchKernelGGL(chain_expand_kernel, dim3((unsigned)word_blk), dim3(256), 0, s, d);
    PCE_LAUNCH_CHECK("chain_expand");
    PCE_HIP(hipMemcpyAsync(&host[0][0], d.summary, (size_t)levels * 4 * sizeof(int), hipMemcpyDeviceToHost, s));
    PCE_HIP(hipStreamSynchronize(s));
    for (int l = 0; l < levels; ++l) {
      if (host[l][1]) PCE_FAIL(PCE_ECOORD, "pce_outcoords_chain: coordinate outside [0,%d) or batch index out of range", PCE_COORD_BOUND);
      if (host[l][3]) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: a batch index is >= n_batch=%d", (int)n_batch);
      n_out_host[l] = host[l][0];
    }
    return PCE_OK;
  }
  for (int l = 0; l < levels; ++l) {
    char *w = (char *)ws[l];
    unsigned *bits = (unsigned *)(w + L[l].off_bits);
    int *cnt = (int *)(w + L[l].off_cnt);
    int *status = (int *)(w + L[l].off_counters);
    if ((rc = fill_u32(bits, (L[l].off_counters + 256 - L[l].off_bits) / 4, 0u, s))) return rc;
    const long long rows_l = l == 0 ? (long long)n_in : (long long)bound_in[l];   // (level 0: the cloud itself, not its plan)
    hipLaunchKernelGGL(outcoord_mark_kernel, dim3((unsigned)pce_div_up(rows_l, 256)), dim3(256), 0, s, src, rows_l, gd[l], L[l].grid,
                       bits, status, n_dev);
    PCE_LAUNCH_CHECK("outcoord_mark");
    if ((rc = scan_exclusive2(cnt, L[l].words, nullptr, 0, (int *)(w + L[l].off_scan), s, bits))) return rc;
    hipLaunchKernelGGL(outcoord_expand_kernel, dim3((unsigned)pce_div_up(L[l].words, 256)), dim3(256), 0, s,
                       (const unsigned *)bits, (const int *)cnt, (long long)L[l].words, L[l].grid, (int4 *)out_coords[l]);
    PCE_LAUNCH_CHECK("outcoord_expand");
    PCE_HIP(hipMemcpyAsync(&host[l][0], cnt + (L[l].words - 1), sizeof(int), hipMemcpyDeviceToHost, s));
    PCE_HIP(hipMemcpyAsync(&host[l][1], status, 3 * sizeof(int), hipMemcpyDeviceToHost, s));
    src = (const int4 *)out_coords[l];
    n_dev = cnt + (L[l].words - 1);
  }
  PCE_HIP(hipStreamSynchronize(s));
  for (int l = 0; l < levels; ++l) {
    if (host[l][1]) PCE_FAIL(PCE_ECOORD, "pce_outcoords_chain: coordinate outside [0,%d) or batch index out of range (level %d)", PCE_COORD_BOUND, l);
    if (host[l][3]) PCE_FAIL(PCE_EINVAL, "pce_outcoords_chain: a batch index is >= n_batch=%d", (int)n_batch);
    n_out_host[l] = host[l][0];
  }
  return PCE_OK;
}

// ------------------------------------------------------------------------------------------------
// voxelisation: floor(point / voxel), one representative per voxel, lexicographic (x,y,z) order
// ------------------------------------------------------------------------------------------------
// Follows sparse_quantize (script/utils.py:33-55): the unique voxels come out in ascending order of
// the ravelled code ((x-min_x)*E_y + (y-min_y))*E_z + (z-min_z) (ravel_hash, script/utils.py:18-30),
// index[v] is the first point (smallest point index) that falls into voxel v and inverse[p] the
// voxel of point p (numpy.unique's return_index / return_inverse).
//
// Sort key = code << idx_bits | point index, so that equal codes are ordered by point index.
#define VOX_LIMIT (1 << 30)

struct VoxLayout {
  int64_t off_q, off_keys_a, off_keys_b, off_hist, off_scan, off_flags, off_counters, total;
};

static void vox_layout(int64_t n, VoxLayout *L) {
  int64_t nblocks = pce_div_up(n, SORT_KEYS_PER_BLOCK);
  int64_t o = 0;
  L->off_q = o;
  o += pce_align_up(n * 16, 256);
  L->off_keys_a = o;
  o += pce_align_up(n * 8, 256);
  L->off_keys_b = o;
  o += pce_align_up(n * 8, 256);
  L->off_hist = o;
  o += pce_align_up((256 * nblocks + 1) * 4, 256);
  L->off_scan = o;
  int64_t scan_n = 256 * nblocks + 1 > n + 1 ? 256 * nblocks + 1 : n + 1;
  o += pce_align_up(scan_tmp_ints(scan_n) * 4, 256);
  L->off_flags = o;
  o += pce_align_up((n + 1) * 4, 256);
  L->off_counters = o;  // int[16]: min xyz, max xyz, status
  o += 256;
  L->total = o;
}

// counters: [0..2] min, [3..5] max, [6] a point is not finite or its voxel index exceeds +-2^30
template <typename F>
__global__ void __launch_bounds__(256) vox_quantize_kernel(const F *__restrict__ pts, long long n, double vx, double vy,
                                                           double vz, int4 *__restrict__ q, int *counters) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  int lo[3] = {VOX_LIMIT, VOX_LIMIT, VOX_LIMIT}, hi[3] = {-VOX_LIMIT, -VOX_LIMIT, -VOX_LIMIT};
  if (i < n) {
    double c[3] = {floor((double)pts[3 * i] / vx), floor((double)pts[3 * i + 1] / vy), floor((double)pts[3 * i + 2] / vz)};
    bool ok = true;
#pragma unroll
    for (int a = 0; a < 3; ++a) ok &= (c[a] > -(double)VOX_LIMIT) && (c[a] < (double)VOX_LIMIT);  // false for NaN
    if (!ok) {
      counters[6] = 1;
      c[0] = c[1] = c[2] = 0.0;
    }
    q[i] = make_int4((int)c[0], (int)c[1], (int)c[2], 0);
#pragma unroll
    for (int a = 0; a < 3; ++a) lo[a] = hi[a] = (int)c[a];
  }
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    for (int d = 32; d >= 1; d >>= 1) {
      int l = __shfl_xor(lo[a], d, PCE_WAVE), h = __shfl_xor(hi[a], d, PCE_WAVE);
      lo[a] = l < lo[a] ? l : lo[a];
      hi[a] = h > hi[a] ? h : hi[a];
    }
    if (__lane_id() == 0 && lo[a] <= hi[a]) {
      atomicMin(&counters[a], lo[a]);
      atomicMax(&counters[3 + a], hi[a]);
    }
  }
}

struct VoxGrid {
  int lo[3];
  long long ey, ez;  // extents of y and z
  int idx_bits;
};

__global__ void __launch_bounds__(256) vox_keys_kernel(const int4 *__restrict__ q, long long n, VoxGrid g,
                                                       unsigned long long *__restrict__ keys) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int4 c = q[i];
  unsigned long long code = ((unsigned long long)(c.x - g.lo[0]) * g.ey + (c.y - g.lo[1])) * g.ez + (c.z - g.lo[2]);
  keys[i] = (code << g.idx_bits) | (unsigned long long)i;
}

// flags[i] = 1 where sorted position i starts a new voxel; flags[n] = 0 (takes the total after the scan)
__global__ void __launch_bounds__(256) vox_flag_kernel(const unsigned long long *__restrict__ keys, long long n,
                                                       int idx_bits, int *__restrict__ flags) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i > n) return;
  int f = 0;
  if (i < n) f = (i == 0) || ((keys[i] >> idx_bits) != (keys[i - 1] >> idx_bits));
  flags[i] = f;
}

// ex = exclusive scan of the flags: sorted position i belongs to voxel ex[i+1]-1 and opens it iff ex[i+1] != ex[i]
__global__ void __launch_bounds__(256) vox_emit_kernel(const unsigned long long *__restrict__ keys, long long n,
                                                       const int *__restrict__ ex, VoxGrid g, int batch,
                                                       int4 *__restrict__ coords, int *__restrict__ index,
                                                       int *__restrict__ inverse) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  unsigned long long key = keys[i];
  int v = ex[i + 1] - 1;
  int idx = (int)(key & ((1ull << g.idx_bits) - 1));
  if (inverse) inverse[idx] = v;
  if (ex[i + 1] != ex[i]) {
    unsigned long long code = key >> g.idx_bits;
    int z = (int)(code % (unsigned long long)g.ez);
    code /= (unsigned long long)g.ez;
    int y = (int)(code % (unsigned long long)g.ey);
    int x = (int)(code / (unsigned long long)g.ey);
    if (coords) coords[v] = make_int4(batch, x + g.lo[0], y + g.lo[1], z + g.lo[2]);
    if (index) index[v] = idx;
  }
}

extern "C" int64_t pce_voxelize_workspace_bytes(int64_t n_points) {
  if (n_points <= 0) return -1;
  VoxLayout L;
  vox_layout(n_points, &L);
  return L.total;
}

extern "C" int pce_voxelize(const void *points, int32_t dtype, int64_t n_points, const double *voxel_size, void *ws,
                            int64_t ws_bytes, int64_t *n_voxels_host, int32_t *coords_min_host, int32_t *coords_max_host,
                            pce_stream_t stream) {
  hipStream_t s = (hipStream_t)stream;
  if (!points || !voxel_size || !ws || !n_voxels_host || !coords_min_host || !coords_max_host) PCE_FAIL(PCE_EINVAL, "pce_voxelize: null pointer");
  if (dtype != PCE_F32 && dtype != PCE_F64) PCE_FAIL(PCE_EINVAL, "pce_voxelize: points must be PCE_F32 or PCE_F64");
  if (n_points <= 0 || n_points >= (1ll << 29)) PCE_FAIL(PCE_EINVAL, "pce_voxelize: n_points=%lld outside (0, 2^29)", (long long)n_points);
  for (int a = 0; a < 3; ++a)
    if (!(voxel_size[a] > 0.0)) PCE_FAIL(PCE_EINVAL, "pce_voxelize: voxel sizes must be positive");
  VoxLayout L;
  vox_layout(n_points, &L);
  if (ws_bytes < L.total) PCE_FAIL(PCE_EWORKSPACE, "pce_voxelize: workspace %lld < %lld", (long long)ws_bytes, (long long)L.total);
  char *w = (char *)ws;
  int4 *q = (int4 *)(w + L.off_q);
  unsigned long long *ka = (unsigned long long *)(w + L.off_keys_a), *kb = (unsigned long long *)(w + L.off_keys_b);
  int *counters = (int *)(w + L.off_counters);
  int *flags = (int *)(w + L.off_flags);
  int rc;
  int init[16] = {VOX_LIMIT, VOX_LIMIT, VOX_LIMIT, -VOX_LIMIT, -VOX_LIMIT, -VOX_LIMIT, 0};
  PCE_HIP(hipMemcpyAsync(counters, init, sizeof(init), hipMemcpyHostToDevice, s));
  unsigned blocks = (unsigned)pce_div_up(n_points, 256);
  if (dtype == PCE_F32)
    hipLaunchKernelGGL(vox_quantize_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float *)points,
                       (long long)n_points, voxel_size[0], voxel_size[1], voxel_size[2], q, counters);
  else
    hipLaunchKernelGGL(vox_quantize_kernel<double>, dim3(blocks), dim3(256), 0, s, (const double *)points,
                       (long long)n_points, voxel_size[0], voxel_size[1], voxel_size[2], q, counters);
  PCE_LAUNCH_CHECK("vox_quantize");
  int host[8];
  PCE_HIP(hipMemcpyAsync(host, counters, sizeof(host), hipMemcpyDeviceToHost, s));
  PCE_HIP(hipStreamSynchronize(s));
  if (host[6]) PCE_FAIL(PCE_ECOORD, "pce_voxelize: a point is not finite or its voxel index exceeds +-2^30");
  VoxGrid g;
  int idx_bits = 1;
  while ((1ll << idx_bits) < n_points) ++idx_bits;
  g.idx_bits = idx_bits;
  long long ext[3];
  for (int a = 0; a < 3; ++a) {
    g.lo[a] = host[a];
    ext[a] = (long long)host[3 + a] - host[a] + 1;
    coords_min_host[a] = host[a];
    coords_max_host[a] = host[3 + a];
  }
  g.ey = ext[1];
  g.ez = ext[2];
  // ext <= 2^31 each: the product is formed in floating point first to stay clear of overflow
  double cells = (double)ext[0] * (double)ext[1] * (double)ext[2];
  int code_bits = 1;
  while (code_bits < 64 && cells > (double)(1ull << code_bits)) ++code_bits;
  if (code_bits + idx_bits > 64)
    PCE_FAIL(PCE_ECAPACITY, "pce_voxelize: %lld x %lld x %lld cells with %lld points do not fit a 64-bit sort key",
             ext[0], ext[1], ext[2], (long long)n_points);
  hipLaunchKernelGGL(vox_keys_kernel, dim3(blocks), dim3(256), 0, s, (const int4 *)q, (long long)n_points, g, ka);
  PCE_LAUNCH_CHECK("vox_keys");
  unsigned long long *sorted = nullptr;
  if ((rc = radix_sort_u64(ka, kb, n_points, code_bits + idx_bits, (int *)(w + L.off_hist), (int *)(w + L.off_scan), s,
                           &sorted)))
    return rc;
  hipLaunchKernelGGL(vox_flag_kernel, dim3((unsigned)pce_div_up(n_points + 1, 256)), dim3(256), 0, s,
                     (const unsigned long long *)sorted, (long long)n_points, idx_bits, flags);
  PCE_LAUNCH_CHECK("vox_flag");
  if ((rc = scan_exclusive(flags, n_points + 1, (int *)(w + L.off_scan), s))) return rc;
  if (sorted != ka) PCE_HIP(hipMemcpyAsync(ka, sorted, (size_t)n_points * 8, hipMemcpyDeviceToDevice, s));
  int total = 0;
  PCE_HIP(hipMemcpyAsync(&total, flags + n_points, sizeof(int), hipMemcpyDeviceToHost, s));
  PCE_HIP(hipStreamSynchronize(s));
  *n_voxels_host = total;
  return PCE_OK;
}

extern "C" int pce_voxelize_emit(const void *ws, int64_t n_points, int64_t n_voxels, const int32_t *coords_min_host,
                                 const int32_t *coords_max_host, int32_t batch_index,
                                 int32_t *coords_out, int32_t *index_out, int32_t *inverse_out, pce_stream_t stream) {
  if (!ws || !coords_min_host || !coords_max_host) PCE_FAIL(PCE_EINVAL, "pce_voxelize_emit: null pointer");
  if (n_points <= 0 || n_points >= (1ll << 29) || n_voxels <= 0 || n_voxels > n_points)
    PCE_FAIL(PCE_EINVAL, "pce_voxelize_emit: n_points=%lld n_voxels=%lld", (long long)n_points, (long long)n_voxels);
  VoxLayout L;
  vox_layout(n_points, &L);
  VoxGrid g;
  g.idx_bits = 1;
  while ((1ll << g.idx_bits) < n_points) ++g.idx_bits;
  for (int a = 0; a < 3; ++a) g.lo[a] = coords_min_host[a];
  g.ey = (long long)coords_max_host[1] - coords_min_host[1] + 1;
  g.ez = (long long)coords_max_host[2] - coords_min_host[2] + 1;
  const char *w = (const char *)ws;
  const unsigned long long *sorted = (const unsigned long long *)(w + L.off_keys_a);
  hipLaunchKernelGGL(vox_emit_kernel, dim3((unsigned)pce_div_up(n_points, 256)), dim3(256), 0, (hipStream_t)stream, sorted,
                     (long long)n_points, (const int *)(w + L.off_flags), g, (int)batch_index, (int4 *)coords_out, index_out,
                     inverse_out);
  PCE_LAUNCH_CHECK("vox_emit");
  return PCE_OK;
}

// ------------------------------------------------------------------------------------------------
// kernel map
// ------------------------------------------------------------------------------------------------
// One build call serves a batch of layers: every stage is ONE launch whose workgroups are dealt to the
// problems of the batch (a build is ~12 small kernels, most of them at the few-microsecond floor of a
// launch; a network needs nine maps per point cloud).  The problem descriptors, the work lists of the
// stages and the lists of arrays to fill and to scan travel to the device in one copy.
#define PCE_MAX_BATCH PCE_KMAP_MAX_BATCH
#define KMAP_DESC_BYTES 32768  // descriptor area at the end of every kernel-map workspace

struct KmapLayout {
  int64_t slots, nseg, scan_len;
  int64_t off_table, off_dense, off_seg, off_scan, off_orank, off_irank, off_desc, total;
};

// Column grid: the lookup structure of a build whose table coordinates (the output coordinates) are sorted by
// (b,x,y,z) and lie in a modest (b,x,y) box.  One cell per column (b,x,y) holds the first row of the column and
// the row behind its last; the z of every row sits in a compact array beside it.  Sorted rows make columns
// contiguous, so building it is one pass without atomics, and a lookup is one 8-byte cell read plus a short
// search in z; neighbouring input rows read neighbouring cells, which a hash scatters over the whole table.
struct GridBox {
  int lo[2], ext[2];   // x and y
  int n_batch;
  long long cells;
};
#define GRID_MAX_CELLS (1ll << 26)

static bool grid_box(const GeomDev &g, int n_batch, int64_t n_out, GridBox *b) {
  if (n_batch <= 0) return false;
  long long cells = n_batch;
  for (int a = 0; a < 2; ++a) {
    if (g.cmax[a] < g.cmin[a]) return false;
    b->lo[a] = g.cmin[a];
    b->ext[a] = g.cmax[a] - g.cmin[a] + 1;
    cells *= b->ext[a];
    if (cells > GRID_MAX_CELLS) return false;
  }
  b->n_batch = n_batch;
  b->cells = cells;
  // clearing and reading the grid must stay cheap next to the rows themselves
  return cells <= 32 * n_out + 65536;
}

static int64_t grid_bytes(const GridBox &b, int64_t n_out) { return pce_align_up(b.cells * 8, 256) + pce_align_up(n_out * 4, 256); }

// table_bytes: what the lookup structure of this build needs (hash table, or the larger of it and the column grid)
static void kmap_layout(int64_t n_in, int64_t n_out, int kv, int want_csr, int sym, int64_t table_bytes, KmapLayout *L) {
  L->slots = pce_hash_slots(n_out);
  L->nseg = pce_div_up(n_in, PCE_WAVE);
  L->scan_len = (int64_t)kv * L->nseg + 1;
  int64_t o = 0;
  L->off_table = o;
  o += pce_align_up(table_bytes > L->slots * 16 ? table_bytes : L->slots * 16, 256);
  L->off_dense = o;
  o += pce_align_up((int64_t)kv * n_in * 4, 256);
  L->off_seg = o;
  o += pce_align_up(L->scan_len * 4, 256);
  L->off_scan = o;
  o += pce_align_up((scan_tmp_ints(L->scan_len) + scan_tmp_ints(n_in + 1) + scan_tmp_ints(n_out + 1)) * 4, 256);
  L->off_orank = o;
  if (want_csr && !sym) o += pce_align_up((int64_t)kv * n_out * 4, 256);
  L->off_irank = o;
  if (want_csr) o += pce_align_up((int64_t)kv * n_in * 4, 256);
  L->off_desc = o;
  o += KMAP_DESC_BYTES;
  L->total = o;
}

#define PCE_GLOBAL __attribute__((address_space(1)))
typedef int pce_v2i __attribute__((ext_vector_type(2)));
typedef int pce_v4i __attribute__((ext_vector_type(4)));

// device-side view of one problem of the batch
struct ProbDev {
  const int4 *in_coords, *out_coords;
  long long n_in, n_out, nseg;
  GeomDev g;
  pce_slot_t *table;
  unsigned long long slots;
  int *dense, *irank, *orank, *seg;
  int *imap, *omap, *knnz, *kpos, *qkpos, *icsr, *icode, *ocsr, *ocode, *islot, *oslot, *nbr_out, *status;
  int *order;        // row order of the ordered output-stationary dataflow, or null
  int want_csr;
  int fused;         // the probe wrote the output-major table (nbr_out), masks and counts itself: no probe table
  int lazy;          // no pair lists: counts per offset only (knnz by atomics, kpos / qkpos from them)
  int use_grid;      // column grid instead of the hash table
  int2 *grid;        // [cells] = {first row of the column, row behind its last}, -1 for an empty column
  int *zcol;         // z of every table row
  GridBox box;
};

// a contiguous range of workgroups of one launch: workgroups [blk0, next job's blk0) work on `prob`
struct Job {
  unsigned blk0;
  int prob;
  int kind;
  int pad;
};
enum { JOB_CSR_SUBM = 0, JOB_CSR_IN = 1, JOB_CSR_COUNT_OUT = 2, JOB_CSR_OUT = 3, JOB_ORDER_SCATTER = 4 };

struct FillRegion {
  unsigned *p;
  long long n_words;
  unsigned blk0;
  unsigned zero;   // fill with zeros instead of the launch's value
};

struct ScanArr {
  int *data;
  long long n;
  int *sums;  // one int per tile of this array
  unsigned blk0;
  unsigned pad;
};

struct JobList {
  const Job *jobs;
  int n;
};

__device__ __forceinline__ const Job &find_job(const JobList &l, unsigned b) {
  int j = 0;
  while (j + 1 < l.n && b >= l.jobs[j + 1].blk0) ++j;
  return l.jobs[j];
}

#define FILL_WORDS_PER_BLOCK (256 * 8)
__global__ void __launch_bounds__(256) multi_fill_kernel(const FillRegion *__restrict__ regs, int n_regs, unsigned value) {
  int r = 0;
  while (r + 1 < n_regs && blockIdx.x >= regs[r + 1].blk0) ++r;
  const FillRegion reg = regs[r];
  long long base = (long long)(blockIdx.x - reg.blk0) * FILL_WORDS_PER_BLOCK;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    long long i = base + k * 256 + threadIdx.x;
    if (i < reg.n_words) reg.p[i] = reg.zero ? 0u : value;
  }
}

__global__ void __launch_bounds__(256) batch_insert_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  long long i = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  if (i >= q.n_out) return;
  int4 c = q.out_coords[i];
  if (!pce_coord_ok(c.x, c.y, c.z, c.w)) {
    q.status[0] = 1;
    return;
  }
  if (!table_insert(q.table, q.slots, pce_pack_key(c.x, c.y, c.z, c.w), (unsigned)i, nullptr)) q.status[1] = 1;
}

// Probe batches: the first-probe loads of PROBE_BATCH offsets are issued together, then resolved;
// only a probe that lands on another key continues along the chain.  (One dependent probe loop per
// offset kept a lane waiting on 26 load latencies in a row.)
#define PROBE_BATCH 7

// One lane per input row.  For every offset kp the lane asks which output row the input reaches:
//   submanifold: out = in - d(kp)          (pair (i,o,kp) <=> coords[i] == coords[o] + d(kp))
//   strided:     out = (in - d(kp) + pad) / stride when it divides
// dense[kp*n_in + i] = output row or -1.
// A submanifold map with odd kernel sizes is symmetric: pair (i,o,kp) <=> pair (o,i,kv-1-kp), because
// d(kv-1-kp) == -d(kp).  Only the offsets below the centre are probed; a hit also writes the mirrored
// entry dense[(kv-1-kp)*n + o] = i.  The rows of dense from the centre upwards are pre-filled with -1.
// With an even kernel size on some axis the offsets are not mirror images of each other (2x2x2: d in
// {0,1}^3, backend/hash.cuh:147-149): every offset but the centre is probed, as the reference does.
__global__ void __launch_bounds__(256) kmap_query_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  const GeomDev &g = q.g;
  const long long n_in = q.n_in;
  const pce_slot_t *__restrict__ table = q.table;
  const unsigned long long slots = q.slots;
  int *__restrict__ dense = q.dense;
  long long i = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  bool live = i < n_in;
  int4 c = live ? q.in_coords[i] : make_int4(0, 0, 0, 0);
  if (live && !pce_coord_ok(c.x, c.y, c.z, c.w)) {
    q.status[0] = 1;
    live = false;
  }
  const int kend = g.sym ? g.mid : g.kv;
  OffsetIter it;
  it.init();
  for (int kp0 = 0; kp0 < kend; kp0 += PROBE_BATCH) {
    unsigned long long key[PROBE_BATCH], slot[PROBE_BATCH];
    uint4 e[PROBE_BATCH];
    bool ok[PROBE_BATCH];
#pragma unroll
    for (int j = 0; j < PROBE_BATCH; ++j) {
      ok[j] = live && kp0 + j < kend && !(g.subm && kp0 + j == g.mid);   // the centre offset is never probed
      int ox = 0, oy = 0, oz = 0;
      if (ok[j]) {
        if (g.subm) {
          ox = c.y - it.dx(g);
          oy = c.z - it.dy(g);
          oz = c.w - it.dz(g);
        } else {
          bool v = strided_axis(c.y, it.dx(g), g.pad[0], g.stride[0], g.cmin[0], g.cmax[0], &ox);
          v &= strided_axis(c.z, it.dy(g), g.pad[1], g.stride[1], g.cmin[1], g.cmax[1], &oy);
          v &= strided_axis(c.w, it.dz(g), g.pad[2], g.stride[2], g.cmin[2], g.cmax[2], &oz);
          ok[j] = v;
        }
      }
      key[j] = pce_pack_key(c.x, ox, oy, oz);
      slot[j] = pce_home_slot(key[j], slots);
      e[j] = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0u);
      if (ok[j]) e[j] = *reinterpret_cast<const uint4 *>(&table[slot[j]]);
      if (kp0 + j < kend) it.next(g);
    }
#pragma unroll
    for (int j = 0; j < PROBE_BATCH; ++j) {
      int kp = kp0 + j;
      if (kp >= kend) break;
      int res = -1;
      if (ok[j]) {
        unsigned long long k = ((unsigned long long)e[j].y << 32) | e[j].x;
        if (k == key[j]) {
          res = (int)e[j].z;
        } else if (k != PCE_EMPTY_KEY) {
          unsigned long long sl = (slot[j] + 1) & (slots - 1);
          for (unsigned long long t = 1; t < slots; ++t) {
            const uint4 f = *reinterpret_cast<const uint4 *>(&table[sl]);
            unsigned long long k2 = ((unsigned long long)f.y << 32) | f.x;
            if (k2 == key[j]) {
              res = (int)f.z;
              break;
            }
            if (k2 == PCE_EMPTY_KEY) break;
            sl = (sl + 1) & (slots - 1);
          }
        }
      }
      if (i < n_in) {
        dense[(long long)kp * n_in + i] = res;
        if (g.sym && res >= 0) dense[(long long)(g.kv - 1 - kp) * n_in + res] = (int)i;
      }
    }
  }
}

// ---- column grid -------------------------------------------------------------------------------------
__device__ __forceinline__ long long grid_cell(const GridBox &b, int bi, int x, int y) {
  const int gx = x - b.lo[0], gy = y - b.lo[1];
  if (bi < 0 || bi >= b.n_batch || gx < 0 || gx >= b.ext[0] || gy < 0 || gy >= b.ext[1]) return -1;
  return ((long long)bi * b.ext[0] + gx) * b.ext[1] + gy;
}

// One lane per table row.  Checks that the rows ascend strictly in (b,x,y,z) and lie in the box (status[3]
// otherwise: the caller rebuilds this map through the hash table), writes z to the compact array, and the
// first / last row of every column writes the column's cell.
__global__ void __launch_bounds__(256) grid_build_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  const long long n = q.n_out;
  long long j = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  if (j >= n) return;
  const int4 c = q.out_coords[j];
  if (!pce_coord_ok(c.x, c.y, c.z, c.w)) {
    q.status[0] = 1;
    return;
  }
  const long long cell = grid_cell(q.box, c.x, c.y, c.z);
  if (cell < 0) {
    q.status[3] = 1;
    return;
  }
  q.zcol[j] = c.w;
  const unsigned long long key = pce_pack_key(c.x, c.y, c.z, c.w);
  bool first = j == 0, last = j == n - 1;
  if (j > 0) {
    const int4 p = q.out_coords[j - 1];
    if (pce_pack_key(p.x, p.y, p.z, p.w) >= key) q.status[3] = 1;   // not sorted, or a duplicate row
    first = p.x != c.x || p.y != c.y || p.z != c.z;
  }
  if (j < n - 1) {
    const int4 nx = q.out_coords[j + 1];
    last = nx.x != c.x || nx.y != c.y || nx.z != c.z;
  }
  if (first) q.grid[cell].x = (int)j;
  if (last) q.grid[cell].y = (int)j + 1;
}

// row of the column [s, e) whose z equals tz, or -1; rows of a column ascend in z
__device__ __forceinline__ int grid_search(const int *__restrict__ zcol, int s, int e, int tz) {
  while (e - s > 4) {
    const int m = (s + e) >> 1;
    if (zcol[m] <= tz)
      s = m;
    else
      e = m;
  }
  for (int j = s; j < e; ++j)
    if (zcol[j] == tz) return j;
  return -1;
}

// The probe of kmap_query_kernel over the column grid: one lane per input row; the offsets are walked column by
// column (ix, iy), GRID_BATCH columns at a time: their cells are read together, then the first four z of every
// column (most columns of a surface-like cloud are that short), then the offsets of the column are resolved.
// SUBM3: the 3x3x3 submanifold layer with everything known at compile time (5 columns, 13 offsets, no divisions);
// otherwise the geometry is read from the problem.
#define GRID_BATCH 5
template <bool SUBM3>
__global__ void __launch_bounds__(256) grid_query_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  const GeomDev &g = q.g;
  const long long n_in = q.n_in;
  const int2 *__restrict__ grid = q.grid;
  const int *__restrict__ zcol = q.zcol;
  int *__restrict__ dense = q.dense;
  long long i = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  bool live = i < n_in;
  int4 c = live ? q.in_coords[i] : make_int4(0, 0, 0, 0);
  if (live && !pce_coord_ok(c.x, c.y, c.z, c.w)) {
    q.status[0] = 1;
    live = false;
  }
  const bool subm = SUBM3 ? true : g.subm != 0;
  const bool sym = SUBM3 ? true : g.sym != 0;
  const int kv = SUBM3 ? 27 : g.kv, mid = SUBM3 ? 13 : g.mid;
  const int kend = sym ? mid : kv;                            // offsets [0, kend) are looked up
  const int ksy = SUBM3 ? 3 : g.ks[1], ksz = SUBM3 ? 3 : g.ks[2];
  const int ncol = SUBM3 ? 5 : (kend + ksz - 1) / ksz;        // columns (ix, iy) that hold one of them
  const int hx = SUBM3 ? 1 : g.half[0] - g.bump[0], hy = SUBM3 ? 1 : g.half[1] - g.bump[1], hz = SUBM3 ? 1 : g.half[2] - g.bump[2];
  for (int col0 = 0; col0 < ncol; col0 += GRID_BATCH) {
    int2 se[GRID_BATCH];
    int zz[GRID_BATCH][4];
    long long cellj[GRID_BATCH];
#pragma unroll
    for (int j = 0; j < GRID_BATCH; ++j) {
      const int col = col0 + j;
      se[j] = make_int2(-1, -1);
      cellj[j] = -1;
      if (live && col < ncol) {
        const int ix = col / ksy, iy = col - ix * ksy;
        const int dx = ix - hx, dy = iy - hy;
        int tx, ty;
        bool ok = true;
        if (subm) {
          tx = c.y - dx;
          ty = c.z - dy;
        } else {
          ok = strided_axis(c.y, dx, g.pad[0], g.stride[0], g.cmin[0], g.cmax[0], &tx);
          ok &= strided_axis(c.z, dy, g.pad[1], g.stride[1], g.cmin[1], g.cmax[1], &ty);
        }
        cellj[j] = ok ? grid_cell(q.box, c.x, tx, ty) : -1;
      }
    }
    // every load goes out from a valid address and is masked afterwards: loads under a lane condition are compiled
    // to branches with a wait each, one trip to memory after the other
#pragma unroll
    for (int j = 0; j < GRID_BATCH; ++j) {
      const int2 v = grid[cellj[j] >= 0 ? cellj[j] : 0];
      if (cellj[j] >= 0) se[j] = v;
    }
#pragma unroll
    for (int j = 0; j < GRID_BATCH; ++j)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int r = se[j].x + t;
        const bool in = se[j].x >= 0 && r < se[j].y;
        const int z = zcol[in ? r : 0];
        zz[j][t] = in ? z : (int)0x80000000;
      }
#pragma unroll
    for (int j = 0; j < GRID_BATCH; ++j) {
      const int col = col0 + j;
      if (col >= ncol) break;
#pragma unroll
      for (int iz = 0; iz < (SUBM3 ? 3 : 1024); ++iz) {
        if (!SUBM3 && iz >= ksz) break;
        const int kp = col * ksz + iz;
        if (kp >= kend) break;
        int res = -1;
        if (live && se[j].x >= 0 && !(subm && kp == mid)) {
          const int dz = iz - hz;
          int tz;
          bool ok = true;
          if (subm)
            tz = c.w - dz;
          else
            ok = strided_axis(c.w, dz, g.pad[2], g.stride[2], g.cmin[2], g.cmax[2], &tz);
          if (ok) {
            if (se[j].y - se[j].x <= 4) {
#pragma unroll
              for (int t = 0; t < 4; ++t)
                if (zz[j][t] == tz) res = se[j].x + t;     // padding entries hold INT_MIN, which no valid z equals
            } else {
              res = grid_search(zcol, se[j].x, se[j].y, tz);
            }
          }
        }
        if (i < n_in) {
          dense[(long long)kp * n_in + i] = res;
          if (sym && res >= 0) dense[(long long)(kv - 1 - kp) * n_in + res] = (int)i;
        }
      }
    }
  }
}

// ---- row order of the ordered output-stationary dataflow -----------------------------------------------------
// Output rows of a map in an order that puts equal neighbour patterns side by side: rows without neighbours
// first (block by block, each block's rows in their own order), then the rows with one or two neighbours sorted
// by the (lowest, second-lowest) offset they have one at, then the rows with ORDER_HEAVY_POPC or more, sorted
// likewise.  A counting sort: masks and a histogram of the keys, one block that turns the histogram into
// bases, a scatter pass with one cursor per key.  The kernels exist twice: over the job lists of a batched map
// build, and with plain arguments for an order requested on its own (pce_row_order).
__device__ __forceinline__ int order_key(unsigned m) {   // m != 0
  const int first = __ffs((int)m) - 1;
  const unsigned rest = m & (m - 1u);
  // rows with a single neighbour come first, by its offset (keys 0 .. 31); then the rows with two, by (lowest,
  // second-lowest) offset (keys 32 .. 1023: first <= 29 whatever the kernel volume up to 31); then, from key 1024,
  // the rows with ORDER_HEAVY_POPC or more, likewise
  if (!rest) return first;
  const int second = __ffs((int)rest) - 1;
  return (__popc(m) >= ORDER_HEAVY_POPC ? 1024 : 0) + 32 + first * 32 + second;
}

// mask[row] = offsets (other than the centre) at which the row has a neighbour; hist[key] += the block's count.
// The keys of a block of 256 rows are counted in LDS first: on a dense cloud nearly every row has a key and a few
// keys hold most rows, and one global atomic per row on those few addresses costs milliseconds.
__device__ __forceinline__ void order_mask_block(const int *__restrict__ nbr, int kv, long long n_rows, int mid,
                                                 int *__restrict__ order, unsigned blk) {
  __shared__ int cnt[ORDER_KEYS];
  for (int i = threadIdx.x; i < ORDER_KEYS; i += 256) cnt[i] = 0;
  __syncthreads();
  const long long row = (long long)blk * 256 + threadIdx.x;
  if (row < n_rows) {
    unsigned m = 0;
    for (int k = 0; k < kv; ++k)
      if (k != mid && nbr[(long long)k * n_rows + row] >= 0) m |= 1u << k;
    order[n_rows + row] = (int)m;
    if (m) atomicAdd(&cnt[order_key(m)], 1);   // rows without neighbours are placed by the scatter pass
  }
  __syncthreads();
  int *hist = order + 2 * n_rows + ORDER_HIST;
  for (int i = threadIdx.x; i < ORDER_KEYS; i += 256)
    if (cnt[i]) atomicAdd(&hist[i], cnt[i]);
}

// base[key] = first position of the key's rows behind the rows without neighbours (one block of 1024); the counts
__device__ __forceinline__ void order_scan_block(int *tail, int *n_heavy_out) {
  __shared__ int part[1024];
  const int *hist = tail + ORDER_HIST;
  int *base = tail + ORDER_BASE;
  constexpr int per = ORDER_KEYS / 1024;
  int sum = 0;
#pragma unroll
  for (int j = 0; j < per; ++j) sum += hist[threadIdx.x * per + j];
  part[threadIdx.x] = sum;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    int v = (int)threadIdx.x >= d ? part[threadIdx.x - d] : 0;
    __syncthreads();
    part[threadIdx.x] += v;
    __syncthreads();
  }
  if (threadIdx.x == 1023) {
    tail[ORDER_N_NONZERO] = part[1023];
    tail[ORDER_N_HEAVY] = part[1023] - part[511];      // keys 1024 .. 2047 belong to threads 512 .. 1023
    tail[ORDER_N_SINGLE] = part[32 / per - 1];          // keys 0 .. 31: rows with exactly one neighbour
    if (n_heavy_out) {   // status words 4, 6 and 7 of a batched build
      n_heavy_out[0] = part[1023] - part[511];
      n_heavy_out[2] = part[1023];
      n_heavy_out[3] = part[32 / per - 1];
    }
  }
  int run = part[threadIdx.x] - sum;
#pragma unroll
  for (int j = 0; j < per; ++j) {
    base[threadIdx.x * per + j] = run;
    run += hist[threadIdx.x * per + j];
  }
}

// perm: the rows of one block of 256 (block `blk` of the map), placed as described above.  A block takes one range
// per key it holds (one global atomic per key and block); its rows of a key keep the ranks LDS atomics gave them.
// `nbr` is the output-major neighbour table, or (mirror >= 0) the probe table of a symmetric map, whose row
// mirror - k is the output-major row k: the table the same launch may still be writing is never read.
__device__ __forceinline__ void order_scatter_block(long long n_rows, int *__restrict__ order, unsigned blk,
                                                    const int *__restrict__ nbr, int mirror) {
  __shared__ int cnt[ORDER_KEYS], gbase[ORDER_KEYS];
  __shared__ int wcount[4], wbase;
  int *perm = order, *tail = order + 2 * n_rows;
  for (int i = threadIdx.x; i < ORDER_KEYS; i += 256) cnt[i] = 0;
  const long long n_plain = n_rows - tail[ORDER_N_NONZERO];
  long long row = (long long)blk * 256 + threadIdx.x;
  const bool live = row < n_rows;
  const unsigned m = live ? (unsigned)order[n_rows + row] : 1u;
  const bool plain = live && m == 0;
  const unsigned long long b = __ballot(plain);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) wcount[wave] = __popcll(b);
  __syncthreads();
  if (threadIdx.x == 0) wbase = atomicAdd(&tail[ORDER_PLAIN_CURSOR], wcount[0] + wcount[1] + wcount[2] + wcount[3]);
  const int key = (live && !plain) ? order_key(m) : -1;
  int rank = 0;
  if (key >= 0) rank = atomicAdd(&cnt[key], 1);
  __syncthreads();
  for (int i = threadIdx.x; i < ORDER_KEYS; i += 256)
    if (cnt[i]) gbase[i] = tail[ORDER_BASE + i] + atomicAdd(&tail[ORDER_CURSOR + i], cnt[i]);
  __syncthreads();
  if (plain) {
    int before = __popcll(b & ((1ull << lane) - 1ull));
    for (int w2 = 0; w2 < wave; ++w2) before += wcount[w2];
    perm[wbase + before] = (int)row;
  } else if (key >= 0) {
    const long long p = n_plain + gbase[key] + rank;
    perm[p] = (int)row;
    // the record of the row: what a wavefront of the ordered dataflow reads of it in one load
    const int k1 = __ffs((int)m) - 1;
    const unsigned rest = m & (m - 1u);
    const int k2 = rest ? __ffs((int)rest) - 1 : -1;
    int4 r;
    r.x = (int)row;
    r.y = (int)m;
    r.z = nbr[(long long)(mirror >= 0 ? mirror - k1 : k1) * n_rows + row];
    r.w = k2 >= 0 ? nbr[(long long)(mirror >= 0 ? mirror - k2 : k2) * n_rows + row] : -1;
    reinterpret_cast<int4 *>(order + PCE_ORDER_REC_OFFSET(n_rows))[p] = r;
    // rows with two neighbours or more: the 128-byte record with the neighbour at every offset
    const long long n_single = tail[ORDER_N_SINGLE];
    const long long si = (long long)gbase[key] + rank - n_single;
    if (key >= 32 && (long long)tail[ORDER_N_NONZERO] - n_single <= PCE_ORDER_SREC_ROWS(n_rows)) {
      int v[32];
      v[0] = (int)row;
      v[1] = (int)m;
#pragma unroll
      for (int k = 0; k < PCE_ORDER_SREC_KV; ++k) {   // (loads from an address valid for every k, selected afterwards)
        const bool has = (m >> k) & 1u;
        const int x = nbr[(long long)(has ? (mirror >= 0 ? mirror - k : k) : 0) * n_rows + row];
        v[2 + k] = has ? x : -1;
      }
      pce_v4i *dst = reinterpret_cast<pce_v4i *>(order + PCE_ORDER_SREC_OFFSET(n_rows) + si * 32);
#pragma unroll
      for (int q = 0; q < 8; ++q) dst[q] = pce_v4i{v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
    }
  }
}

// The 3x3x3 submanifold map over the column grid in one pass, output-major: lane o looks up all 26 neighbours of
// its own row (nine cells; a probe of half the offsets with mirrored writes, as above, leaves a row's results
// scattered over the lanes of other rows) and so holds everything about the row at once -- it writes the
// output-major table nbr_out[k][o] = row at coords[o] + d(k) (coalesced, the centre row the identity), the row's
// offset mask and the key histogram of the row order, and what the pair lists need: by the symmetry of such a map
// row o is the INPUT of a pair at offset k exactly when it has a neighbour at 26 - k, so the wave ballots are the
// (offset, 64-row segment) counts of the pair lists and the popcount of the mask is the row's CSR length.  No
// probe table, no counting pass, no -1 prefill.  lazy: no pair lists are wanted; the counts per offset go to knnz
// through one atomic per offset and workgroup.
// (Written without branches around loads: every load goes out from a valid address and is masked afterwards, the
// nine cells together, then the first four z of the nine columns together; pointers read from the problem
// descriptor are cast to the global address space, or the loads are compiled as flat ones.)
__global__ void __launch_bounds__(256) grid_query_full3_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  const long long n = q.n_in, nseg = q.nseg;
  const PCE_GLOBAL pce_v2i *grid = (const PCE_GLOBAL pce_v2i *)q.grid;
  const PCE_GLOBAL int *zcol = (const PCE_GLOBAL int *)q.zcol;
  PCE_GLOBAL int *nbr = (PCE_GLOBAL int *)q.nbr_out;
  const bool order = q.order != nullptr, lazy = q.lazy != 0, want_csr = q.want_csr != 0;      // the same for the whole workgroup
  const GridBox box = q.box;
  const long long i = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  const long long seg = i >> 6;
  const int lane = __lane_id();
  bool live = i < n;
  const pce_v4i cv = ((const PCE_GLOBAL pce_v4i *)q.in_coords)[live ? i : 0];
  const int4 c = make_int4(cv.x, cv.y, cv.z, cv.w);
  if (live && !pce_coord_ok(c.x, c.y, c.z, c.w)) {
    q.status[0] = 1;
    live = false;
  }
  __shared__ int keycnt[ORDER_KEYS];
  __shared__ int offcnt[32];
  if (order)
    for (int t = threadIdx.x; t < ORDER_KEYS; t += 256) keycnt[t] = 0;
  if (threadIdx.x < 32) offcnt[threadIdx.x] = 0;
  __syncthreads();
  int2 se[9];
#pragma unroll
  for (int col = 0; col < 9; ++col) {
    const int ix = col / 3, iy = col - ix * 3;
    // (no early-out as in grid_cell: a branch per column put a wait behind every one of the nine loads)
    const int gx = c.y + ix - 1 - box.lo[0], gy = c.z + iy - 1 - box.lo[1];
    const bool in = live & ((unsigned)c.x < (unsigned)box.n_batch) & ((unsigned)gx < (unsigned)box.ext[0]) &
                    ((unsigned)gy < (unsigned)box.ext[1]);
    const long long cell = ((long long)c.x * box.ext[0] + gx) * box.ext[1] + gy;
    const pce_v2i v = grid[in ? cell : 0];
    se[col].x = in ? v.x : -1;
    se[col].y = in ? v.y : -1;
  }
  int zz[9][4], lb[9];
  bool tall = false;
#pragma unroll
  for (int col = 0; col < 9; ++col) {
    lb[col] = se[col].x;
    tall |= se[col].x >= 0 && se[col].y - se[col].x > 4;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int r = se[col].x + t;
      const bool in = se[col].x >= 0 && r < se[col].y;
      const int z = zcol[in ? r : 0];
      zz[col][t] = in ? z : (int)0x80000000;
    }
  }
  if (__any(tall)) {
    // a column of more than four rows (a wall, a pole): one search for the first row at or above z - 1; the three
    // rows from there are the only candidates for z - 1, z and z + 1 (the rows of a column ascend strictly in z)
#pragma unroll
    for (int col = 0; col < 9; ++col) {
      if (se[col].x >= 0 && se[col].y - se[col].x > 4) {
        int lo = se[col].x, hi = se[col].y;          // first row of [lo, hi) whose z >= c.w - 1, or hi
        while (lo < hi) {
          const int md = (lo + hi) >> 1;
          if (zcol[md] < c.w - 1)
            lo = md + 1;
          else
            hi = md;
        }
        lb[col] = lo;
#pragma unroll
        for (int t = 0; t < 3; ++t) zz[col][t] = lo + t < se[col].y ? zcol[lo + t] : (int)0x80000000;
        zz[col][3] = (int)0x80000000;
      }
    }
  }
  // the 27 results of the row; their ballots are the pair lists' (offset, segment) counts, mirrored
  int res[27];
  unsigned m = 0;
  int mine = 0;       // lane l < 27 ends up with the wavefront's count for offset l
#pragma unroll
  for (int kp = 0; kp < 27; ++kp) {
    const int col = kp / 3, iz = kp - col * 3;
    int r = -1;
    if (kp == 13) {
      r = live ? (int)i : -1;
    } else {
      const int tz = c.w + iz - 1;
#pragma unroll
      for (int t = 0; t < 4; ++t) r = (zz[col][t] == tz) ? lb[col] + t : r;   // padding entries hold INT_MIN, which no valid z equals
      r = (live && se[col].x >= 0) ? r : -1;
    }
    res[kp] = r;
    const bool hit = r >= 0 && kp != 13;
    m |= hit ? 1u << kp : 0u;
    const int cnt = __popcll(__ballot(hit));
    mine = lane == kp ? cnt : mine;
  }
  if (live) {
#pragma unroll
    for (int kp = 0; kp < 27; ++kp) nbr[(long long)kp * n + i] = res[kp];
  }
  // row o is the input of a pair at offset k exactly when it has a neighbour at 26 - k
  if (lane < 27) {
    if (lazy) {
      if (mine) atomicAdd(&offcnt[26 - lane], mine);
    } else if (seg < nseg) {
      q.seg[(long long)(26 - lane) * nseg + seg] = mine;
    }
  }
  if (!lazy) {
    if (want_csr && i <= n) q.icsr[i] = live ? __popc(m) : 0;   // icsr[n] = 0 receives the total after the scan
    if (i == 0) q.seg[27 * nseg] = 0;
  }
  if (order && live) {
    q.order[n + i] = (int)m;
    if (m) atomicAdd(&keycnt[order_key(m)], 1);   // rows without neighbours are placed by the scatter pass
  }
  __syncthreads();
  if (order) {
    int *hist = q.order + 2 * n + ORDER_HIST;
    for (int t = threadIdx.x; t < ORDER_KEYS; t += 256)
      if (keycnt[t]) atomicAdd(&hist[t], keycnt[t]);
  }
  if (lazy && threadIdx.x < 27 && offcnt[threadIdx.x]) atomicAdd(&q.knnz[threadIdx.x], offcnt[threadIdx.x]);
}

// The per-row loops over the offsets below load ROW_BATCH table entries before using any of them.
#define ROW_BATCH 9

// One pass over the probe results: hits per (offset, 64-row segment) from wave ballots, and hits per
// row (the row lengths of the CSR view, mapping_counter of backend/hash.cuh:422-437).
__global__ void __launch_bounds__(256) kmap_count_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  const long long n_in = q.n_in, nseg = q.nseg;
  const int kv = q.g.kv;
  const int *__restrict__ dense = q.dense;
  int *__restrict__ segcnt = q.seg;
  int *__restrict__ rowcnt = q.want_csr ? q.icsr : nullptr;
  long long i = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  long long seg = i >> 6;
  bool live = i < n_in;
  // A symmetric map's output-major table is its probe table mirrored (nbr_out[kp] = dense[kv-1-kp]), so the offset
  // masks and the key histogram of its row order come out of this pass (order_mask_block does the same from nbr_out).
  const bool masks = q.order && q.g.sym;      // the same for the whole workgroup
  __shared__ int keycnt[ORDER_KEYS];
  if (masks) {
    for (int t = threadIdx.x; t < ORDER_KEYS; t += 256) keycnt[t] = 0;
    __syncthreads();
  }
  unsigned m = 0;
  int c = 0;
  for (int kp0 = 0; kp0 < kv; kp0 += ROW_BATCH) {
    int v[ROW_BATCH];
#pragma unroll
    for (int j = 0; j < ROW_BATCH; ++j) v[j] = (live && kp0 + j < kv) ? dense[(long long)(kp0 + j) * n_in + i] : -1;
#pragma unroll
    for (int j = 0; j < ROW_BATCH; ++j) {
      if (kp0 + j >= kv) break;
      bool hit = v[j] >= 0;
      c += hit;
      if (masks && hit && kp0 + j != q.g.mid) m |= 1u << (kv - 1 - (kp0 + j));
      unsigned long long bal = __ballot(hit);
      if (__lane_id() == 0 && seg < nseg) segcnt[(long long)(kp0 + j) * nseg + seg] = __popcll(bal);
    }
  }
  if (rowcnt && i <= n_in) rowcnt[i] = live ? c : 0;  // rowcnt[n_in] = 0 receives the total after the scan
  if (i == 0) segcnt[(long long)kv * nseg] = 0;
  if (masks) {
    if (live) {
      q.order[n_in + i] = (int)m;
      if (m) atomicAdd(&keycnt[order_key(m)], 1);
    }
    __syncthreads();
    int *hist = q.order + 2 * n_in + ORDER_HIST;
    for (int t = threadIdx.x; t < ORDER_KEYS; t += 256)
      if (keycnt[t]) atomicAdd(&hist[t], keycnt[t]);
  }
}

// Exclusive scans of several arrays in two launches: every workgroup scans its SCAN_TILE items in place
// and records its total; then every workgroup adds the totals of the workgroups before it in its array.
__global__ void __launch_bounds__(256) multi_scan_local_kernel(const ScanArr *__restrict__ arrs, int n_arrs) {
  int a = 0;
  while (a + 1 < n_arrs && blockIdx.x >= arrs[a + 1].blk0) ++a;
  const ScanArr arr = arrs[a];
  const int blk = blockIdx.x - arr.blk0;
  long long base = (long long)blk * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
  int v[SCAN_ITEMS];
  int acc = 0;
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j) {
    v[j] = base + j < arr.n ? arr.data[base + j] : 0;
    acc += v[j];
  }
  int total;
  int run = block_exclusive_scan(acc, &total);
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j) {
    if (base + j < arr.n) arr.data[base + j] = run;
    run += v[j];
  }
  if (threadIdx.x == 0) arr.sums[blk] = total;
}

__global__ void __launch_bounds__(256) multi_scan_add_kernel(const ScanArr *__restrict__ arrs, int n_arrs) {
  int a = 0;
  while (a + 1 < n_arrs && blockIdx.x >= arrs[a + 1].blk0) ++a;
  const ScanArr arr = arrs[a];
  const int blk = blockIdx.x - arr.blk0;
  if (blk == 0) return;
  int acc = 0;
  for (int j = threadIdx.x; j < blk; j += 256) acc += arr.sums[j];
  int total;
  block_exclusive_scan(acc, &total);
  long long base = (long long)blk * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
#pragma unroll
  for (int j = 0; j < SCAN_ITEMS; ++j)
    if (base + j < arr.n) arr.data[base + j] += total;
}

// kpos[kp] = first pair of offset kp; then the scan of counts rounded up to the tile height
// (backend/hash.cuh:478-497).  One workgroup per problem.
// Workgroups [n_probs, 2 n_probs): the bases of the row order's counting sort for the maps whose key histogram the
// counting pass has filled (symmetric maps).
__global__ void __launch_bounds__(1024) kmap_offsets_kernel(const ProbDev *__restrict__ P, int n_probs) {
  if ((int)blockIdx.x >= n_probs) {
    const ProbDev &o = P[blockIdx.x - n_probs];
    if (o.order && o.g.sym) order_scan_block(o.order + 2 * o.n_out, o.status + 4);   // the same for the whole workgroup
    return;
  }
  const ProbDev &q = P[blockIdx.x];
  const int *__restrict__ segoff = q.seg;
  const long long nseg = q.nseg;
  const int kv = q.g.kv;
  if (q.lazy) {   // the counts per offset are complete (the probe added them up): their two scans
    if (threadIdx.x == 0) {
      int a = 0, qq = 0;
      q.kpos[0] = 0;
      q.qkpos[0] = 0;
      for (int kp = 0; kp < kv; ++kp) {
        const int c = q.knnz[kp];
        a += c;
        qq += (c + PCE_QUANTUM - 1) / PCE_QUANTUM * PCE_QUANTUM;
        q.kpos[kp + 1] = a;
        q.qkpos[kp + 1] = qq;
      }
      q.status[5] = 1;   // this map holds no pair lists
    }
    return;
  }
  for (int kp = threadIdx.x; kp <= kv; kp += blockDim.x) {
    int a = segoff[(long long)kp * nseg];
    q.kpos[kp] = a;
    if (kp < kv) q.knnz[kp] = segoff[(long long)(kp + 1) * nseg] - a;
  }
  if (threadIdx.x == 0) {
    int qq = 0;
    q.qkpos[0] = 0;
    for (int kp = 0; kp < kv; ++kp) {
      int c = segoff[(long long)(kp + 1) * nseg] - segoff[(long long)kp * nseg];
      qq += (c + PCE_QUANTUM - 1) / PCE_QUANTUM * PCE_QUANTUM;
      q.qkpos[kp + 1] = qq;
    }
  }
}

// segoff = exclusive scan of segcnt in (kp, segment) order = position of the segment's first pair.
// Emits the pair lists in (offset, input row) order from ballot ranks, the rank of every pair inside
// its offset (irank, and orank scattered by output row for strided layers), and the output-major
// neighbour table: scattered for strided layers, read off the mirrored row for submanifold ones.
__global__ void __launch_bounds__(256) kmap_fill_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  if (job.kind == JOB_ORDER_SCATTER) {   // the row order of a symmetric map: masks and bases are complete by now
    // (a symmetric map: the fill jobs of this launch may be writing nbr_out, so the probe table is read, mirrored,
    // unless the probe wrote the output-major table itself)
    if (q.fused)
      order_scatter_block(q.n_out, q.order, blockIdx.x - job.blk0, q.nbr_out, -1);
    else
      order_scatter_block(q.n_out, q.order, blockIdx.x - job.blk0, q.dense, q.g.kv - 1);
    return;
  }
  const long long n_in = q.n_in, n_out = q.n_out, nseg = q.nseg;
  const int kv = q.g.kv, subm = q.g.subm, sym = q.g.sym, mid = q.g.mid, fused = q.fused;
  // (pointers read from the descriptor are cast to the global address space, or the loads are compiled as flat
  // ones; every load of a batch goes out from a valid address and is masked afterwards, or each is compiled to a
  // branch with a wait behind it)
  const PCE_GLOBAL int *table = (const PCE_GLOBAL int *)(fused ? q.nbr_out : q.dense);
  const PCE_GLOBAL int *segoff = (const PCE_GLOBAL int *)q.seg;
  int *__restrict__ imap = q.imap;
  int *__restrict__ omap = q.omap;
  int *__restrict__ irank = q.irank;
  int *__restrict__ orank = q.orank;
  int *__restrict__ nbr_out = q.nbr_out;
  long long i = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  long long seg = i >> 6;
  bool live = i < n_in;
  const bool mirror = !fused && nbr_out && sym;
  for (int kp0 = 0; kp0 < kv; kp0 += ROW_BATCH) {
    int vv[ROW_BATCH], mm[ROW_BATCH], base[ROW_BATCH], first[ROW_BATCH];
#pragma unroll
    for (int j = 0; j < ROW_BATCH; ++j) {
      const int kp = kp0 + j;
      const bool in = kp < kv;
      // (fused: the probe wrote the output-major table, whose row kv-1-kp is the probe table's row kp)
      const bool want_v = live && in && !(fused && kp == mid);
      const int v = table[want_v ? (long long)(fused ? kv - 1 - kp : kp) * n_in + i : 0];
      vv[j] = want_v ? v : -1;
      const bool want_m = mirror && live && in && kp != mid;
      const int mv = mirror ? table[want_m ? (long long)(kv - 1 - kp) * n_in + i : 0] : -1;
      mm[j] = want_m ? mv : -1;
      const bool want_b = in && seg < nseg;
      const int b = segoff[want_b ? (long long)kp * nseg + seg : 0];
      base[j] = want_b ? b : 0;
      const int f = segoff[in ? (long long)kp * nseg : 0];
      first[j] = in ? f : 0;
    }
#pragma unroll
    for (int j = 0; j < ROW_BATCH; ++j) {
      int kp = kp0 + j;
      if (kp >= kv) break;
      int v = vv[j];
      unsigned long long bal = __ballot(v >= 0);
      int rank = -1;
      if (v >= 0) {
        int p = base[j] + __popcll(bal & lanemask_lt());
        imap[p] = (int)i;
        omap[p] = v;
        if (nbr_out && !sym) nbr_out[(long long)kp * n_out + v] = (int)i;   // (a fused map is symmetric)
        rank = p - first[j];
        if (irank && rank >= PCE_CSR_CODE) q.status[2] = 1;
        if (orank) orank[(long long)kp * n_out + v] = rank;
      }
      if (irank && live) irank[(long long)kp * n_in + i] = rank;
      if (nbr_out && sym && !fused && live)  // nbr_out[kp][o] = input of the pair whose output is o = mirrored probe result
        nbr_out[(long long)kp * n_out + i] = kp == mid ? (int)i : mm[j];
      if (nbr_out && subm && !sym && live && kp == mid) nbr_out[(long long)kp * n_out + i] = (int)i;
    }
  }
}

// CSR-coded views.  Entries of every row in ascending offset order, code = kp * PCE_CSR_CODE + rank, plus,
// for every pair (offset kp, rank rk), the slot of its entry: slot_of_pair[kpos[kp] + rk] = position.
// Jobs of one launch (the kind is uniform over a workgroup):
//   JOB_CSR_SUBM      symmetric submanifold map (odd kernel sizes), both views in one pass: the input-side entry of row r at offset kp
//                     is the pair (r, dense[kp][r], kp); the output-side entry is the pair
//                     (dense[kv-1-kp][r], r, kp), whose rank is read from the rank table at its input row.
//                     Both views have the same row pointers.
//   JOB_CSR_IN / JOB_CSR_OUT   one view of a strided map from its rank table (irank / orank)
//   JOB_CSR_COUNT_OUT          entries per output row of a strided map (mapping_counter,
//                              backend/hash.cuh:422-437), scanned before JOB_CSR_OUT runs
__device__ __forceinline__ void csr_fill_rows(const int *__restrict__ rank, long long n, int kv, const int *__restrict__ csr,
                                              int *__restrict__ code, const int *__restrict__ kpos,
                                              int *__restrict__ slot_of_pair, long long r) {
  if (r >= n) return;
  int pos = csr[r];
  for (int kp = 0; kp < kv; ++kp) {
    int rk = rank[(long long)kp * n + r];
    if (rk >= 0) {
      code[pos] = kp * PCE_CSR_CODE + rk;
      if (slot_of_pair) slot_of_pair[kpos[kp] + rk] = pos;
      ++pos;
    }
  }
}

__global__ void __launch_bounds__(256) csr_stage_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  const int kv = q.g.kv;
  long long r = (long long)(blockIdx.x - job.blk0) * blockDim.x + threadIdx.x;
  if (job.kind == JOB_CSR_IN) {
    csr_fill_rows(q.irank, q.n_in, kv, q.icsr, q.icode, q.kpos, q.islot, r);
    return;
  }
  if (job.kind == JOB_CSR_OUT) {
    csr_fill_rows(q.orank, q.n_out, kv, q.ocsr, q.ocode, q.kpos, q.oslot, r);
    return;
  }
  if (job.kind == JOB_CSR_COUNT_OUT) {
    const long long n = q.n_out;
    if (r > n) return;
    int c = 0;
    if (r < n)
      for (int kp = 0; kp < kv; ++kp) c += q.orank[(long long)kp * n + r] >= 0;
    q.ocsr[r] = c;  // ocsr[n] = 0 receives the total after the scan
    return;
  }
  // JOB_CSR_SUBM
  const long long n = q.n_in;
  const int fused = q.fused, mid = q.g.mid;
  // (global address space and unconditional loads from valid addresses, as in kmap_fill_kernel)
  const PCE_GLOBAL int *table = (const PCE_GLOBAL int *)(fused ? q.nbr_out : q.dense);
  const PCE_GLOBAL int *irank = (const PCE_GLOBAL int *)q.irank;
  const PCE_GLOBAL int *csr = (const PCE_GLOBAL int *)q.icsr;
  const PCE_GLOBAL int *kpos = (const PCE_GLOBAL int *)q.kpos;
  int *__restrict__ icode = q.icode;
  int *__restrict__ ocode = q.ocode;
  int *__restrict__ islot = q.islot;
  int *__restrict__ oslot = q.oslot;
  if (r > n) return;
  if (r == n) {
    q.ocsr[n] = csr[n];
    return;
  }
  int pi = csr[r], po = pi;
  q.ocsr[r] = pi;
  for (int kp0 = 0; kp0 < kv; kp0 += ROW_BATCH) {
    int rk[ROW_BATCH], src[ROW_BATCH], rk2[ROW_BATCH], kb[ROW_BATCH];
#pragma unroll
    for (int j = 0; j < ROW_BATCH; ++j) {
      const int kp = kp0 + j;
      const bool in = kp < kv;
      const int a = irank[in ? (long long)kp * n + r : 0];
      rk[j] = in ? a : -1;
      // the input of the pair whose output is r at offset kp: the output-major table's entry (fused; its centre
      // row holds the identity and is no pair), else the probe table's mirrored entry
      const bool want = in && !(fused && kp == mid);
      const int b = table[want ? (long long)(fused ? kp : kv - 1 - kp) * n + r : 0];
      src[j] = want ? b : -1;
      const int c = kpos[in ? kp : 0];
      kb[j] = in ? c : 0;
    }
#pragma unroll
    for (int j = 0; j < ROW_BATCH; ++j) {
      const int a = irank[src[j] >= 0 ? (long long)(kp0 + j < kv ? kp0 + j : 0) * n + src[j] : 0];
      rk2[j] = src[j] >= 0 ? a : -1;
    }
#pragma unroll
    for (int j = 0; j < ROW_BATCH; ++j) {
      int kp = kp0 + j;
      if (rk[j] >= 0) {
        icode[pi] = kp * PCE_CSR_CODE + rk[j];
        if (islot) islot[kb[j] + rk[j]] = pi;
        ++pi;
      }
      if (src[j] >= 0) {
        ocode[po] = kp * PCE_CSR_CODE + rk2[j];
        if (oslot) oslot[kb[j] + rk2[j]] = po;
        ++po;
      }
    }
  }
}

extern "C" int64_t pce_kmap_workspace_bytes(int64_t n_in, int64_t n_out, int32_t kv, int32_t want_csr) {
  KmapLayout L;
  kmap_layout(n_in, n_out, kv, want_csr, 0, 0, &L);  // the strided layout is the larger one
  return L.total;
}

extern "C" int64_t pce_kmap_workspace_bytes_grid(int64_t n_in, int64_t n_out, const pce_geom_t *g, int32_t n_batch,
                                                 int32_t want_csr) {
  GeomDev d;
  if (make_geom(g, &d) != PCE_OK || n_in <= 0 || n_out <= 0) return -1;
  GridBox box;
  const int64_t table = grid_box(d, n_batch, n_out, &box) ? grid_bytes(box, n_out) : 0;
  KmapLayout L;
  kmap_layout(n_in, n_out, d.kv, want_csr, 0, table, &L);
  return L.total;
}

// stages of a batched build, each one launch with its own job list
__global__ void order_clear_kernel(int *tail) {
  for (int i = threadIdx.x; i < PCE_ORDER_TAIL; i += blockDim.x) tail[i] = 0;
}
__global__ void __launch_bounds__(256) order_mask_kernel(const int *__restrict__ nbr, int kv, long long n_rows, int mid,
                                                         int *__restrict__ order) {
  order_mask_block(nbr, kv, n_rows, mid, order, blockIdx.x);
}
__global__ void __launch_bounds__(1024) order_scan_kernel(int *tail) { order_scan_block(tail, nullptr); }
__global__ void __launch_bounds__(256) order_scatter_kernel(long long n_rows, int *__restrict__ order,
                                                            const int *__restrict__ nbr) {
  order_scatter_block(n_rows, order, blockIdx.x, nbr, -1);
}

// the same over the problems of a batched build; status[4] of a problem receives its number of heavy rows
__global__ void __launch_bounds__(256) order_mask_batch_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  order_mask_block(q.nbr_out, q.g.kv, q.n_out, q.g.subm ? q.g.mid : -1, q.order, blockIdx.x - job.blk0);
}
__global__ void __launch_bounds__(1024) order_scan_batch_kernel(const ProbDev *__restrict__ P) {
  const ProbDev &q = P[blockIdx.x];
  if (!q.order || q.g.sym) return;   // a symmetric map's histogram was scanned with the pair offsets
  order_scan_block(q.order + 2 * q.n_out, q.status + 4);
}
__global__ void __launch_bounds__(256) order_scatter_batch_kernel(const ProbDev *__restrict__ P, JobList jl) {
  const Job &job = find_job(jl, blockIdx.x);
  const ProbDev &q = P[job.prob];
  order_scatter_block(q.n_out, q.order, blockIdx.x - job.blk0, q.nbr_out, -1);
}

extern "C" int64_t pce_row_order_elems(int64_t n_rows) { return n_rows < 0 ? 0 : PCE_ORDER_ELEMS(n_rows); }

extern "C" int pce_row_order(const int32_t *nbr, int32_t kv, int64_t n_rows, int32_t mid, int32_t *order, int64_t order_elems,
                             int64_t *counts_host, pce_stream_t stream) {
  if (!nbr || !order || !counts_host) PCE_FAIL(PCE_EINVAL, "pce_row_order: null pointer");
  if (kv < 1 || kv > ORDER_MAX_KV - 1) PCE_FAIL(PCE_EINVAL, "pce_row_order: kernel volume %d outside [1, %d]", (int)kv, ORDER_MAX_KV - 1);
  if (n_rows <= 0 || n_rows >= (1ll << 30)) PCE_FAIL(PCE_EINVAL, "pce_row_order: n_rows=%lld", (long long)n_rows);
  if (mid >= kv) PCE_FAIL(PCE_EINVAL, "pce_row_order: centre offset %d outside the kernel volume %d", (int)mid, (int)kv);
  if ((uintptr_t)order & 15) PCE_FAIL(PCE_EINVAL, "pce_row_order: the order array must be 16-byte aligned");
  if (order_elems < pce_row_order_elems(n_rows))
    PCE_FAIL(PCE_EWORKSPACE, "pce_row_order: order holds %lld elements, needs %lld", (long long)order_elems, (long long)pce_row_order_elems(n_rows));
  hipStream_t s = (hipStream_t)stream;
  int *tail = order + 2 * n_rows;
  const unsigned blocks = (unsigned)pce_div_up(n_rows, 256);
  hipLaunchKernelGGL(order_clear_kernel, dim3(1), dim3(1024), 0, s, tail);
  PCE_LAUNCH_CHECK("order_clear");
  hipLaunchKernelGGL(order_mask_kernel, dim3(blocks), dim3(256), 0, s, nbr, (int)kv, (long long)n_rows, (int)mid, order);
  PCE_LAUNCH_CHECK("order_mask");
  hipLaunchKernelGGL(order_scan_kernel, dim3(1), dim3(1024), 0, s, tail);
  PCE_LAUNCH_CHECK("order_scan");
  hipLaunchKernelGGL(order_scatter_kernel, dim3(blocks), dim3(256), 0, s, (long long)n_rows, order, (const int *)nbr);
  PCE_LAUNCH_CHECK("order_scatter");
  static_assert(ORDER_N_HEAVY == ORDER_N_NONZERO + 1 && ORDER_N_NONZERO == ORDER_N_SINGLE + 1, "the counts are read back in one copy");
  int counts[3] = {0, 0, 0};
  PCE_HIP(hipMemcpyAsync(counts, tail + ORDER_N_SINGLE, 3 * sizeof(int), hipMemcpyDeviceToHost, s));
  PCE_HIP(hipStreamSynchronize(s));
  counts_host[0] = counts[2];   // rows with three neighbours or more
  counts_host[1] = counts[1];   // rows with any neighbour
  counts_host[2] = counts[0];   // rows with exactly one
  return PCE_OK;
}

enum { ST_INSERT = 0, ST_QUERY, ST_COUNT, ST_FILL, ST_CSR_A, ST_CSR_B, ST_GRID_BUILD, ST_GRID_QUERY, ST_GRID_QUERY3, ST_GRID_FULL3,
       ST_ORDER_MASK, ST_ORDER_SCATTER, ST_COUNT_ };

// host-side image of everything the kernels of one batch read
struct BatchImage {
  ProbDev prob[PCE_MAX_BATCH];
  Job jobs[ST_COUNT_][2 * PCE_MAX_BATCH];      // per stage
  int n_jobs[ST_COUNT_];
  FillRegion fills[5 * PCE_MAX_BATCH];
  ScanArr scans[2][2 * PCE_MAX_BATCH];  // first scan (segments, input rows), second scan (output rows)
};

// The descriptor block travels from pinned host memory, so the copy is queued like a kernel and the
// host does not wait for earlier work on the stream.  A small ring of pinned blocks per device; a
// block is reused once the copy that read it has completed.
#define DESC_RING 8
#define DESC_MAX_DEVICES 16
struct DescRing {
  BatchImage *host[DESC_RING];
  hipEvent_t done[DESC_RING];
  int next;
  bool ready;
};
static DescRing g_desc_ring[DESC_MAX_DEVICES];
static std::mutex g_desc_mutex;

static int desc_upload(const BatchImage &img, void *dst, hipStream_t s) {
  int dev = 0;
  PCE_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= DESC_MAX_DEVICES) PCE_FAIL(PCE_ECAPACITY, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_desc_mutex);
  DescRing &r = g_desc_ring[dev];
  if (!r.ready) {
    for (int k = 0; k < DESC_RING; ++k) {
      PCE_HIP(hipHostMalloc((void **)&r.host[k], sizeof(BatchImage), hipHostMallocDefault));
      PCE_HIP(hipEventCreateWithFlags(&r.done[k], hipEventDisableTiming));
    }
    r.next = 0;
    r.ready = true;
  }
  const int k = r.next;
  r.next = (k + 1) % DESC_RING;
  PCE_HIP(hipEventSynchronize(r.done[k]));  // returns at once for an event never recorded
  memcpy(r.host[k], &img, sizeof(BatchImage));
  PCE_HIP(hipMemcpyAsync(dst, r.host[k], sizeof(BatchImage), hipMemcpyHostToDevice, s));
  PCE_HIP(hipEventRecord(r.done[k], s));
  return PCE_OK;
}

extern "C" int pce_kmap_build_batch(const pce_kmap_problem_t *probs, int32_t n_probs, pce_stream_t stream) {
  hipStream_t s = (hipStream_t)stream;
  if (!probs || n_probs < 1 || n_probs > PCE_MAX_BATCH)
    PCE_FAIL(PCE_EINVAL, "pce_kmap_build_batch: 1..%d problems per call", PCE_MAX_BATCH);
  static_assert(sizeof(BatchImage) <= KMAP_DESC_BYTES, "descriptor area too small");
  BatchImage img;
  memset(&img, 0, sizeof(img));
  unsigned blk[ST_COUNT_] = {};
  unsigned fill_blk = 0, scan_blk[2] = {0, 0};
  int n_fill = 0, n_scan[2] = {0, 0};
  auto add_job = [&](int stage, int prob, int kind, long long items) {
    Job &j = img.jobs[stage][img.n_jobs[stage]++];
    j.blk0 = blk[stage];
    j.prob = prob;
    j.kind = kind;
    blk[stage] += (unsigned)pce_div_up(items, 256);
  };
  auto add_fill = [&](void *p, long long words, unsigned zero = 0) {
    if (words <= 0) return;
    FillRegion &f = img.fills[n_fill++];
    f.p = (unsigned *)p;
    f.n_words = words;
    f.zero = zero;
    f.blk0 = fill_blk;
    fill_blk += (unsigned)pce_div_up(words, FILL_WORDS_PER_BLOCK);
  };
  auto add_scan = [&](int which, int *data, long long n, int *sums) {
    ScanArr &a = img.scans[which][n_scan[which]++];
    a.data = data;
    a.n = n;
    a.sums = sums;
    a.blk0 = scan_blk[which];
    scan_blk[which] += (unsigned)pce_div_up(n, SCAN_TILE);
  };
  long long total_blocks = 0;
  for (int p = 0; p < n_probs; ++p) {
    const pce_kmap_problem_t &u = probs[p];
    ProbDev &q = img.prob[p];
    int rc = make_geom(&u.geom, &q.g);
    if (rc) return rc;
    if (!u.in_coords || !u.out_coords || !u.ws || !u.knnz || !u.kpos || !u.qkpos || !u.status)
      PCE_FAIL(PCE_EINVAL, "pce_kmap_build: null pointer");
    int ncsr = (u.icsr != nullptr) + (u.icode != nullptr) + (u.ocsr != nullptr) + (u.ocode != nullptr);
    if (ncsr != 0 && ncsr != 4) PCE_FAIL(PCE_EINVAL, "pce_kmap_build: pass all four CSR outputs or none");
    const int want_csr = ncsr == 4;
    if (!want_csr && (u.islot || u.oslot)) PCE_FAIL(PCE_EINVAL, "pce_kmap_build: slot outputs need the CSR outputs");
    const int64_t n_in = u.n_in, n_out = u.n_out;
    if (n_in <= 0 || n_out <= 0) PCE_FAIL(PCE_EINVAL, "pce_kmap_build: empty tensor (n_in=%lld, n_out=%lld)", (long long)n_in, (long long)n_out);
    if (q.g.subm && n_in != n_out) PCE_FAIL(PCE_EINVAL, "pce_kmap_build: submanifold layer needs n_in == n_out");
    if ((int64_t)q.g.kv * n_in >= (1ll << 31) || (int64_t)q.g.kv * n_out >= (1ll << 31))
      PCE_FAIL(PCE_ECAPACITY, "pce_kmap_build: kv*n exceeds int32 pair indexing");
    // The column grid serves when the caller bounds the batch indices, the (b,x,y) box of the table coordinates
    // is modest and the workspace was sized for it (pce_kmap_workspace_bytes_grid); else the hash table.
    KmapLayout L;
    GridBox box;
    int use_grid = 0;
    if (!(u.flags & PCE_KMAP_NO_GRID) && grid_box(q.g, u.n_batch, n_out, &box)) {
      kmap_layout(n_in, n_out, q.g.kv, want_csr, q.g.sym, grid_bytes(box, n_out), &L);
      use_grid = u.ws_bytes >= L.total;
    }
    if (!use_grid) kmap_layout(n_in, n_out, q.g.kv, want_csr, q.g.sym, 0, &L);
    if (u.ws_bytes < L.total) PCE_FAIL(PCE_EWORKSPACE, "pce_kmap_build: workspace %lld < %lld", (long long)u.ws_bytes, (long long)L.total);
    // the 3x3x3 submanifold map over the column grid is probed output-major in one pass (grid_query_full3_kernel)
    // when the output-major table is wanted and the probe table is not; without pair lists if the caller waives them
    const bool subm3 = q.g.sym && q.g.ks[0] == 3 && q.g.ks[1] == 3 && q.g.ks[2] == 3;
    const int fused = use_grid && subm3 && u.nbr_out && !u.nbr_in;
    const int lazy = fused && (u.flags & PCE_KMAP_TABLE_ONLY) && !want_csr;
    if (!lazy && (!u.imap || !u.omap))
      PCE_FAIL(PCE_EINVAL, "pce_kmap_build: null pair lists (only a map built with PCE_KMAP_TABLE_ONLY over the column grid goes without)");
    char *w = (char *)u.ws;
    q.in_coords = (const int4 *)u.in_coords;
    q.out_coords = (const int4 *)u.out_coords;
    q.n_in = n_in;
    q.n_out = n_out;
    q.nseg = L.nseg;
    q.table = (pce_slot_t *)(w + L.off_table);
    q.slots = (unsigned long long)L.slots;
    q.dense = u.nbr_in ? u.nbr_in : (int *)(w + L.off_dense);  // the input-major table is the probe result itself
    q.irank = want_csr ? (int *)(w + L.off_irank) : nullptr;
    q.orank = (want_csr && !q.g.sym) ? (int *)(w + L.off_orank) : nullptr;
    q.seg = (int *)(w + L.off_seg);
    q.imap = u.imap;
    q.omap = u.omap;
    q.knnz = u.knnz;
    q.kpos = u.kpos;
    q.qkpos = u.qkpos;
    q.icsr = u.icsr;
    q.icode = u.icode;
    q.ocsr = u.ocsr;
    q.ocode = u.ocode;
    q.islot = u.islot;
    q.oslot = u.oslot;
    q.nbr_out = u.nbr_out;
    q.status = u.status;
    q.order = nullptr;
    if (u.order) {
      // the row order of the ordered output-stationary dataflow, derived from the output-major table once it is filled
      if (!u.nbr_out) PCE_FAIL(PCE_EINVAL, "pce_kmap_build: the row order needs the output-major neighbour table (nbr_out)");
      if (q.g.kv > ORDER_MAX_KV - 1) PCE_FAIL(PCE_EINVAL, "pce_kmap_build: the row order takes kernel volumes up to %d", ORDER_MAX_KV - 1);
      if (n_out >= (1ll << 30)) PCE_FAIL(PCE_ECAPACITY, "pce_kmap_build: too many rows for a row order");
      q.order = u.order;
      add_fill(u.order + 2 * n_out, PCE_ORDER_TAIL, 1);
      if (!q.g.sym) {   // a symmetric map's order rides on the counting, offset and fill launches (see there)
        add_job(ST_ORDER_MASK, p, 0, n_out);
        add_job(ST_ORDER_SCATTER, p, 0, n_out);
      }
    }
    q.want_csr = want_csr;
    q.fused = fused;
    q.lazy = lazy;
    q.use_grid = use_grid;
    if (use_grid) {
      q.box = box;
      q.grid = (int2 *)(w + L.off_table);
      q.zcol = (int *)(w + L.off_table + pce_align_up(box.cells * 8, 256));
    }
    // 1. lookup structure over the output coordinates (for a submanifold layer these are the input coordinates)
    if (use_grid)
      add_fill(q.grid, box.cells * 2);
    else
      add_fill(q.table, L.slots * 4);
    if (fused) {
      if (lazy) add_fill(q.knnz, q.g.kv, 1);   // the probe adds the counts per offset up with atomics
    } else if (q.g.sym) {
      // rows of the probe table that the mirrored writes only touch on a hit (and the centre row)
      add_fill(q.dense + (int64_t)q.g.mid * n_in, (int64_t)(q.g.kv - q.g.mid) * n_in);
    } else {
      if (q.nbr_out) add_fill(q.nbr_out, (int64_t)q.g.kv * n_out);
      if (q.orank) add_fill(q.orank, (int64_t)q.g.kv * n_out);
    }
    add_job(use_grid ? ST_GRID_BUILD : ST_INSERT, p, 0, n_out);
    // 2. probe, count per (offset, segment) and per row; 3. their scans; 4. pair lists
    if (fused) {
      add_job(ST_GRID_FULL3, p, 0, n_in + 1);
    } else {
      add_job(use_grid ? (subm3 ? ST_GRID_QUERY3 : ST_GRID_QUERY) : ST_QUERY, p, 0, n_in);
      add_job(ST_COUNT, p, 0, n_in + 1);
    }
    int *scan_tmp = (int *)(w + L.off_scan);
    if (!lazy) {
      add_scan(0, q.seg, L.scan_len, scan_tmp);
      if (want_csr) add_scan(0, q.icsr, n_in + 1, scan_tmp + scan_tmp_ints(L.scan_len));
      add_job(ST_FILL, p, 0, n_in);
    }
    if (q.order && q.g.sym) add_job(ST_FILL, p, JOB_ORDER_SCATTER, n_out);
    // 5. CSR-coded views
    if (want_csr && q.g.sym) {
      add_job(ST_CSR_A, p, JOB_CSR_SUBM, n_in + 1);
    } else if (want_csr) {
      add_job(ST_CSR_A, p, JOB_CSR_IN, n_in);
      add_job(ST_CSR_A, p, JOB_CSR_COUNT_OUT, n_out + 1);
      add_scan(1, q.ocsr, n_out + 1, scan_tmp + scan_tmp_ints(L.scan_len) + scan_tmp_ints(n_in + 1));
      add_job(ST_CSR_B, p, JOB_CSR_OUT, n_out);
    }
    total_blocks += pce_div_up(n_in + 1, 256) + pce_div_up(n_out + 1, 256) +
                    pce_div_up(use_grid ? box.cells * 2 : L.slots * 4, FILL_WORDS_PER_BLOCK) +
                    3 * pce_div_up((int64_t)q.g.kv * (n_in > n_out ? n_in : n_out), FILL_WORDS_PER_BLOCK);
  }
  if (total_blocks >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "pce_kmap_build_batch: the batch exceeds the grid limit");
  // one copy carries the descriptors; they live in the first problem's workspace
  KmapLayout L0;
  kmap_layout(probs[0].n_in, probs[0].n_out, img.prob[0].g.kv, img.prob[0].want_csr, img.prob[0].g.sym,
              img.prob[0].use_grid ? grid_bytes(img.prob[0].box, probs[0].n_out) : 0, &L0);
  char *desc = (char *)probs[0].ws + L0.off_desc;
  if (int rc = desc_upload(img, desc, s)) return rc;
  const BatchImage *D = (const BatchImage *)desc;
  const ProbDev *P = D->prob;
  auto jl = [&](int stage) {
    JobList l;
    l.jobs = D->jobs[stage];
    l.n = img.n_jobs[stage];
    return l;
  };
  hipLaunchKernelGGL(multi_fill_kernel, dim3(fill_blk), dim3(256), 0, s, (const FillRegion *)D->fills, n_fill, 0xFFFFFFFFu);
  PCE_LAUNCH_CHECK("multi_fill");
  if (blk[ST_INSERT]) {
    hipLaunchKernelGGL(batch_insert_kernel, dim3(blk[ST_INSERT]), dim3(256), 0, s, P, jl(ST_INSERT));
    PCE_LAUNCH_CHECK("hash_insert");
  }
  if (blk[ST_GRID_BUILD]) {
    hipLaunchKernelGGL(grid_build_kernel, dim3(blk[ST_GRID_BUILD]), dim3(256), 0, s, P, jl(ST_GRID_BUILD));
    PCE_LAUNCH_CHECK("grid_build");
  }
  if (blk[ST_QUERY]) {
    hipLaunchKernelGGL(kmap_query_kernel, dim3(blk[ST_QUERY]), dim3(256), 0, s, P, jl(ST_QUERY));
    PCE_LAUNCH_CHECK("kmap_query");
  }
  if (blk[ST_GRID_QUERY]) {
    hipLaunchKernelGGL(grid_query_kernel<false>, dim3(blk[ST_GRID_QUERY]), dim3(256), 0, s, P, jl(ST_GRID_QUERY));
    PCE_LAUNCH_CHECK("grid_query");
  }
  if (blk[ST_GRID_QUERY3]) {
    hipLaunchKernelGGL(grid_query_kernel<true>, dim3(blk[ST_GRID_QUERY3]), dim3(256), 0, s, P, jl(ST_GRID_QUERY3));
    PCE_LAUNCH_CHECK("grid_query3");
  }
  if (blk[ST_GRID_FULL3]) {
    hipLaunchKernelGGL(grid_query_full3_kernel, dim3(blk[ST_GRID_FULL3]), dim3(256), 0, s, P, jl(ST_GRID_FULL3));
    PCE_LAUNCH_CHECK("grid_query_full3");
  }
  if (blk[ST_COUNT]) {
    hipLaunchKernelGGL(kmap_count_kernel, dim3(blk[ST_COUNT]), dim3(256), 0, s, P, jl(ST_COUNT));
    PCE_LAUNCH_CHECK("kmap_count");
  }
  if (scan_blk[0]) {
    hipLaunchKernelGGL(multi_scan_local_kernel, dim3(scan_blk[0]), dim3(256), 0, s, (const ScanArr *)D->scans[0], n_scan[0]);
    PCE_LAUNCH_CHECK("scan_local");
    hipLaunchKernelGGL(multi_scan_add_kernel, dim3(scan_blk[0]), dim3(256), 0, s, (const ScanArr *)D->scans[0], n_scan[0]);
    PCE_LAUNCH_CHECK("scan_add");
  }
  hipLaunchKernelGGL(kmap_offsets_kernel, dim3(2 * n_probs), dim3(1024), 0, s, P, (int)n_probs);
  PCE_LAUNCH_CHECK("kmap_offsets");
  if (blk[ST_FILL]) {
    hipLaunchKernelGGL(kmap_fill_kernel, dim3(blk[ST_FILL]), dim3(256), 0, s, P, jl(ST_FILL));
    PCE_LAUNCH_CHECK("kmap_fill");
  }
  if (blk[ST_CSR_A]) {
    hipLaunchKernelGGL(csr_stage_kernel, dim3(blk[ST_CSR_A]), dim3(256), 0, s, P, jl(ST_CSR_A));
    PCE_LAUNCH_CHECK("csr_stage_a");
  }
  if (blk[ST_CSR_B]) {
    hipLaunchKernelGGL(multi_scan_local_kernel, dim3(scan_blk[1]), dim3(256), 0, s, (const ScanArr *)D->scans[1], n_scan[1]);
    PCE_LAUNCH_CHECK("scan_local");
    hipLaunchKernelGGL(multi_scan_add_kernel, dim3(scan_blk[1]), dim3(256), 0, s, (const ScanArr *)D->scans[1], n_scan[1]);
    PCE_LAUNCH_CHECK("scan_add");
    hipLaunchKernelGGL(csr_stage_kernel, dim3(blk[ST_CSR_B]), dim3(256), 0, s, P, jl(ST_CSR_B));
    PCE_LAUNCH_CHECK("csr_stage_b");
  }
  if (blk[ST_ORDER_MASK]) {
    hipLaunchKernelGGL(order_mask_batch_kernel, dim3(blk[ST_ORDER_MASK]), dim3(256), 0, s, P, jl(ST_ORDER_MASK));
    PCE_LAUNCH_CHECK("order_mask");
    hipLaunchKernelGGL(order_scan_batch_kernel, dim3(n_probs), dim3(1024), 0, s, P);
    PCE_LAUNCH_CHECK("order_scan");
    hipLaunchKernelGGL(order_scatter_batch_kernel, dim3(blk[ST_ORDER_SCATTER]), dim3(256), 0, s, P, jl(ST_ORDER_SCATTER));
    PCE_LAUNCH_CHECK("order_scatter");
  }
  return PCE_OK;
}

extern "C" int pce_kmap_build(const int32_t *in_coords, int64_t n_in, const int32_t *out_coords, int64_t n_out,
                              const pce_geom_t *g, void *ws, int64_t ws_bytes, int32_t *imap, int32_t *omap,
                              int32_t *knnz, int32_t *kpos, int32_t *qkpos, int32_t *icsr, int32_t *icode,
                              int32_t *ocsr, int32_t *ocode, int32_t *islot, int32_t *oslot, int32_t *nbr_out,
                              int32_t *nbr_in, int32_t *status, pce_stream_t stream) {
  if (!g) PCE_FAIL(PCE_EINVAL, "geometry is null");
  pce_kmap_problem_t u;
  u.in_coords = in_coords;
  u.n_in = n_in;
  u.out_coords = out_coords;
  u.n_out = n_out;
  u.geom = *g;
  u.ws = ws;
  u.ws_bytes = ws_bytes;
  u.imap = imap;
  u.omap = omap;
  u.knnz = knnz;
  u.kpos = kpos;
  u.qkpos = qkpos;
  u.icsr = icsr;
  u.icode = icode;
  u.ocsr = ocsr;
  u.ocode = ocode;
  u.islot = islot;
  u.oslot = oslot;
  u.nbr_out = nbr_out;
  u.nbr_in = nbr_in;
  u.status = status;
  u.n_batch = 0;   // no batch bound in this signature: the hash table
  u.flags = 0;
  u.order = nullptr;
  return pce_kmap_build_batch(&u, 1, stream);
}
