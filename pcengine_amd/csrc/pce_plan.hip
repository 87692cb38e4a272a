// pcengine_amd -- the planner of a network's kernel maps (map reuse and workspace planner).
//
// A network asks for a pyramid of maps per point cloud: the output coordinates of its strided levels, a map per
// strided level and a submanifold map per level.  The reference builds them layer by layer as the forward pass
// meets them, each with its own allocations (script/spconv.py:331-437, script/sptensor.py:63-78).  Here one host
// call lays all of them out in ONE allocation from upper bounds (pce_pyramid_plan: a level holds at most as many
// rows as the bitmap of its coordinates has cells and as the level above has rows), and one call builds them
// (pce_pyramid_build: the chained output coordinates, then every map in the launches of one batched build), with
// nothing but a few microseconds of host arithmetic between the two waits for counts.
#include <string.h>

#include "pce_common.h"

static const int META_STATUS = 8;

static int64_t meta_ints(int kv) { return 3 * (int64_t)kv + 2 + META_STATUS; }

extern "C" int64_t pce_pyramid_plan_sizeof(void) { return (int64_t)sizeof(pce_pyr_plan_t); }

extern "C" int pce_pyramid_plan(int64_t n_cap, int32_t n_levels, const pce_geom_t *strided, int32_t n_batch,
                                const pce_pyr_request_t *requests, int32_t n_requests, pce_pyr_plan_t *plan) {
  if (!plan || !requests || (n_levels > 0 && !strided)) PCE_FAIL(PCE_EINVAL, "pce_pyramid_plan: null pointer");
  if (n_cap <= 0 || n_levels < 0 || n_levels > PCE_PYR_MAX_LEVELS || n_requests < 1 || n_requests > PCE_PYR_MAX_MAPS || n_batch <= 0)
    PCE_FAIL(PCE_EINVAL, "pce_pyramid_plan: %lld rows, %d levels (at most %d), %d maps (1..%d), %d batches", (long long)n_cap,
             (int)n_levels, PCE_PYR_MAX_LEVELS, (int)n_requests, PCE_PYR_MAX_MAPS, (int)n_batch);
  memset(plan, 0, sizeof(*plan));
  plan->n_levels = n_levels;
  plan->n_maps = n_requests;
  plan->n_batch = n_batch;
  plan->level_cap[0] = n_cap;
  int64_t off = 0;
  auto take = [&](int64_t bytes) {
    const int64_t at = off;
    off += pce_align_up(bytes > 0 ? bytes : 1, 256);
    return at;
  };
  if (n_levels > 0) {
    int64_t ws[PCE_PYR_MAX_LEVELS], cap[PCE_PYR_MAX_LEVELS];
    const int rc = pce_outcoords_chain_plan(n_cap, n_levels, strided, n_batch, ws, cap);
    if (rc) return rc;   // PCE_CHAIN_NOT_APPLICABLE: the caller builds level by level
    for (int l = 0; l < n_levels; ++l) {
      plan->strided[l] = strided[l];
      plan->chain_ws_bytes[l] = ws[l];
      plan->off_chain_ws[l] = take(ws[l]);
      plan->level_cap[l + 1] = cap[l];
      plan->off_coords[l + 1] = take(16 * cap[l]);
    }
  }
  // the counts and status words of all maps sit together: one copy reads them back
  plan->off_meta = off;
  for (int i = 0; i < n_requests; ++i) {
    const pce_pyr_request_t &r = requests[i];
    if (r.level_in < 0 || r.level_in > n_levels || r.level_out < r.level_in || r.level_out > n_levels ||
        (r.geom.subm != 0) != (r.level_in == r.level_out))
      PCE_FAIL(PCE_EINVAL, "pce_pyramid_plan: map %d reads level %d and writes level %d", i, (int)r.level_in, (int)r.level_out);
    const int64_t kv = (int64_t)r.geom.ks[0] * r.geom.ks[1] * r.geom.ks[2];
    if (kv < 1 || kv > 31) PCE_FAIL(PCE_EINVAL, "pce_pyramid_plan: map %d has kernel volume %lld (1..31)", i, (long long)kv);
    plan->req[i] = r;
    plan->map[i].kv = (int32_t)kv;
    plan->map[i].off[PCE_PYR_META] = off;
    off += meta_ints((int)kv) * 4;
  }
  plan->meta_bytes = off - plan->off_meta;
  off = pce_align_up(off, 256);
  for (int i = 0; i < n_requests; ++i) {
    const pce_pyr_request_t &r = requests[i];
    pce_pyr_map_t &m = plan->map[i];
    const int64_t kv = m.kv, ci = plan->level_cap[r.level_in], co = plan->level_cap[r.level_out];
    m.cap_in = ci;
    m.cap_out = co;
    for (int a = 0; a < PCE_PYR_ARRAYS; ++a)
      if (a != PCE_PYR_META) m.off[a] = -1;
    const int64_t ws = pce_kmap_workspace_bytes_grid(ci, co, &r.geom, n_batch, r.want_csr);
    if (ws < 0) PCE_FAIL(PCE_EINVAL, "pce_pyramid_plan: map %d has no valid geometry", i);
    m.ws_bytes = ws;
    m.off[PCE_PYR_WS] = take(ws);
    m.off[PCE_PYR_IMAP] = take(4 * kv * ci);
    m.off[PCE_PYR_OMAP] = take(4 * kv * ci);
    m.off[PCE_PYR_NBR_OUT] = take(4 * kv * co);
    if (r.want_nbr_in) m.off[PCE_PYR_NBR_IN] = take(4 * kv * ci);
    // the row order comes with every submanifold map and every strided map of at most 8 offsets
    if (r.geom.subm || kv <= 8) m.off[PCE_PYR_ORDER] = take(4 * pce_row_order_elems(co));
    if (r.want_csr) {
      m.off[PCE_PYR_ICSR] = take(4 * (ci + 1));
      m.off[PCE_PYR_OCSR] = take(4 * (co + 1));
      m.off[PCE_PYR_ICODE] = take(4 * kv * ci);
      m.off[PCE_PYR_OCODE] = take(4 * kv * ci);
      m.off[PCE_PYR_ISLOT] = take(4 * kv * ci);
      m.off[PCE_PYR_OSLOT] = take(4 * kv * ci);
    }
  }
  plan->arena_bytes = off;
  return PCE_OK;
}

extern "C" int pce_pyramid_build(pce_pyr_plan_t *plan, const int32_t *in_coords, int64_t n_in, void *arena, int64_t arena_bytes,
                                 pce_stream_t stream) {
  if (!plan || !in_coords || !arena) PCE_FAIL(PCE_EINVAL, "pce_pyramid_build: null pointer");
  if (n_in <= 0 || n_in > plan->level_cap[0])
    PCE_FAIL(PCE_ECAPACITY, "pce_pyramid_build: %lld rows, the plan holds %lld", (long long)n_in, (long long)plan->level_cap[0]);
  if (arena_bytes < plan->arena_bytes || ((uintptr_t)arena & 255))
    PCE_FAIL(PCE_EWORKSPACE, "pce_pyramid_build: the arena holds %lld bytes, the plan needs %lld (256-byte aligned)",
             (long long)arena_bytes, (long long)plan->arena_bytes);
  hipStream_t s = (hipStream_t)stream;
  char *base = (char *)arena;
  const int32_t *coords[PCE_PYR_MAX_LEVELS + 1];
  coords[0] = in_coords;
  plan->level_n[0] = n_in;
  if (plan->n_levels > 0) {
    void *ws[PCE_PYR_MAX_LEVELS];
    int32_t *outs[PCE_PYR_MAX_LEVELS];
    int64_t n_out[PCE_PYR_MAX_LEVELS];
    for (int l = 0; l < plan->n_levels; ++l) {
      ws[l] = base + plan->off_chain_ws[l];
      outs[l] = (int32_t *)(base + plan->off_coords[l + 1]);
      coords[l + 1] = outs[l];
    }
    // (the chain's own plan was made for the capacity: a smaller cloud fits its workspaces and buffers)
    const int rc = pce_outcoords_chain_planned(in_coords, n_in, plan->level_cap[0], plan->n_levels, plan->strided, plan->n_batch, ws,
                                               plan->chain_ws_bytes, outs, n_out, stream);
    if (rc) return rc;
    for (int l = 0; l < plan->n_levels; ++l) {
      if (n_out[l] > plan->level_cap[l + 1])
        PCE_FAIL(PCE_ECAPACITY, "pce_pyramid_build: level %d holds %lld rows, planned for %lld", l + 1, (long long)n_out[l], (long long)plan->level_cap[l + 1]);
      plan->level_n[l + 1] = n_out[l];
    }
  }
  PCE_HIP(hipMemsetAsync(base + plan->off_meta, 0, (size_t)plan->meta_bytes, s));
  pce_kmap_problem_t probs[PCE_PYR_MAX_MAPS];
  memset(probs, 0, sizeof(probs));
  for (int i = 0; i < plan->n_maps; ++i) {
    const pce_pyr_request_t &r = plan->req[i];
    pce_pyr_map_t &m = plan->map[i];
    pce_kmap_problem_t &u = probs[i];
    m.n_in = plan->level_n[r.level_in];
    m.n_out = plan->level_n[r.level_out];
    if (m.n_in <= 0 || m.n_out <= 0) PCE_FAIL(PCE_EINVAL, "pce_pyramid_build: level without rows");
    auto at = [&](int a) { return m.off[a] < 0 ? nullptr : (int32_t *)(base + m.off[a]); };
    u.in_coords = coords[r.level_in];
    u.n_in = m.n_in;
    u.out_coords = coords[r.level_out];
    u.n_out = m.n_out;
    u.geom = r.geom;
    u.ws = base + m.off[PCE_PYR_WS];
    u.ws_bytes = m.ws_bytes;
    u.imap = at(PCE_PYR_IMAP);
    u.omap = at(PCE_PYR_OMAP);
    int32_t *meta = at(PCE_PYR_META);
    u.knnz = meta;
    u.kpos = meta + m.kv;
    u.qkpos = meta + 2 * m.kv + 1;
    u.status = meta + 3 * m.kv + 2;
    u.icsr = at(PCE_PYR_ICSR);
    u.icode = at(PCE_PYR_ICODE);
    u.ocsr = at(PCE_PYR_OCSR);
    u.ocode = at(PCE_PYR_OCODE);
    u.islot = at(PCE_PYR_ISLOT);
    u.oslot = at(PCE_PYR_OSLOT);
    u.nbr_out = at(PCE_PYR_NBR_OUT);
    u.nbr_in = at(PCE_PYR_NBR_IN);
    u.order = at(PCE_PYR_ORDER);
    u.n_batch = plan->n_batch;
    u.flags = r.table_only ? PCE_KMAP_TABLE_ONLY : 0;
  }
  const int rc = pce_kmap_build_batch(probs, plan->n_maps, stream);
  if (rc) return rc;
  int32_t host[PCE_PYR_MAX_MAPS * (3 * 31 + 2 + META_STATUS)];
  PCE_HIP(hipMemcpyAsync(host, base + plan->off_meta, (size_t)plan->meta_bytes, hipMemcpyDeviceToHost, s));
  PCE_HIP(hipStreamSynchronize(s));
  int fallback = 0;
  for (int i = 0; i < plan->n_maps; ++i) {
    pce_pyr_map_t &m = plan->map[i];
    const int32_t *h = host + (m.off[PCE_PYR_META] - plan->off_meta) / 4;
    memcpy(m.meta, h, (size_t)meta_ints(m.kv) * 4);
    const int32_t *st = h + 3 * m.kv + 2;
    if (st[0]) PCE_FAIL(PCE_ECOORD, "pce_pyramid_build: a coordinate of map %d is outside the supported range", i);
    if (st[1]) PCE_FAIL(PCE_ECAPACITY, "pce_pyramid_build: hash table of map %d exhausted", i);
    if (st[2]) PCE_FAIL(PCE_ECAPACITY, "pce_pyramid_build: an offset of map %d holds too many pairs for the CSR code", i);
    if (st[3]) fallback = 1;   // unsorted rows or rows outside the stated box: the caller builds this cloud map by map
    m.n_pairs = h[2 * m.kv];
    m.qsum = h[3 * m.kv + 1];
  }
  return fallback ? PCE_PYR_UNSORTED : PCE_OK;
}
