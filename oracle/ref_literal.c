/* Sequential, literal restatement of the reference's map-building kernels.
 * TEST INFRASTRUCTURE ONLY: loaded by tests/ (ctypes) to cross-check oracle/oracle.py.
 *
 * Each function follows one reference kernel, executed by a single host thread in
 * ascending thread-id order:
 *   lit_coord_hash         backend/hash.cuh:11-15
 *   lit_table_size         backend/hash.cu:46
 *   lit_insert_hash        backend/hash.cuh:55-75   (atomicExch eviction chain, step 97)
 *   lit_insert_val         backend/hash.cuh:77-91
 *   lit_query              backend/hash.cuh:154-161 (equality on the 64-bit linear hash value)
 *   lit_out_coords         backend/hash.cuh:535-610 + backend/hash.cu:141-173
 *                          (expand, remove(-1), sort, unique, decode)
 *   lit_map_d2             backend/hash.cuh:265-419 + backend/hash.cuh:478-497
 *   lit_map_d1             backend/hash.cuh:97-260, 422-437 + backend/hash.cu:210-243
 *
 * Where the reference lets atomic timing decide (the rank of a pair inside its offset,
 * backend/hash.cuh:163,255) the rank is the position in (offset, input row) order, i.e. the
 * order the reference's own dense fetch-on-demand map yields after compaction
 * (script/spconv.py:370-372).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BOUND 3259LL
#define CSR_CODE 1186111

uint64_t lit_coord_hash(int b, int x, int y, int z) {
  return ((uint64_t)b * 23783141ULL + (uint64_t)x * 73856093ULL + (uint64_t)y * 19349669ULL +
          (uint64_t)z * 83492791ULL + 1ULL);
}

int lit_table_size(int n) { return (int)(2 * pow(2, ceil(log2((double)n)))); }

void lit_insert_hash(int nnz, int size, const int *coord, int *idx) {
  for (int id = 0; id < nnz; id++) {
    uint64_t v = lit_coord_hash(coord[4 * id], coord[4 * id + 1], coord[4 * id + 2], coord[4 * id + 3]);
    uint64_t t = v % (uint64_t)size;
    int old = idx[t];
    idx[t] = id;
    while (old > -1) {
      t = (t + 97) % (uint64_t)size;
      int o2 = idx[t];
      idx[t] = old;
      old = o2;
    }
  }
}

void lit_insert_val(int nnz, int size, const int *coord, const int *idx, uint64_t *val) {
  for (int id = 0; id < size; id++) {
    int in = idx[id];
    if (in < nnz && in > -1)
      val[id] = lit_coord_hash(coord[4 * in], coord[4 * in + 1], coord[4 * in + 2], coord[4 * in + 3]);
  }
}

int lit_query(int size, const uint64_t *val, const int *idx, int b, int x, int y, int z) {
  uint64_t tv = lit_coord_hash(b, x, y, z);
  uint64_t t = tv % (uint64_t)size;
  while (val[t] != tv && idx[t] > -1) t = (t + 97) % (uint64_t)size;
  return idx[t];
}

static int cmp_i64(const void *a, const void *b) {
  int64_t x = *(const int64_t *)a, y = *(const int64_t *)b;
  return (x > y) - (x < y);
}

static void offset_of(int kp, const int *ks, int strided, int *d) {
  d[0] = kp / (ks[2] * ks[1]) - (ks[0] - 1) / 2;
  d[1] = (kp / ks[2]) % ks[1] - (ks[1] - 1) / 2;
  d[2] = kp % ks[2] - (ks[2] - 1) / 2;
  if (strided)
    for (int a = 0; a < 3; a++) d[a] += (ks[a] % 2 == 0 || ks[a] == 1) ? 0 : 1;
}

/* returns n_out; out_coords must hold n_in*kv rows */
int lit_out_coords(int n_in, const int *coords, const int *ks, const int *stride, const int *pad,
                   const int *cmin, const int *cmax, int *out_coords) {
  int kv = ks[0] * ks[1] * ks[2];
  int64_t *codes = (int64_t *)malloc(sizeof(int64_t) * (size_t)n_in * kv);
  size_t nvalid = 0;
  for (int i = 0; i < n_in; i++) {
    for (int kp = 0; kp < kv; kp++) {
      int d[3], div[3], ok = 1;
      offset_of(kp, ks, 1, d);
      for (int a = 0; a < 3; a++) {
        int cand = coords[4 * i + 1 + a] - d[a] + pad[a];
        div[a] = cand / stride[a];
        if (div[a] < cmin[a] || div[a] > cmax[a] || cand % stride[a] != 0) ok = 0;
      }
      if (!ok) continue;
      codes[nvalid++] = (((int64_t)coords[4 * i] * BOUND + div[0]) * BOUND + div[1]) * BOUND + div[2];
    }
  }
  qsort(codes, nvalid, sizeof(int64_t), cmp_i64);
  int n_out = 0;
  for (size_t j = 0; j < nvalid; j++) {
    if (j && codes[j] == codes[j - 1]) continue;
    int64_t c = codes[j];
    out_coords[4 * n_out + 3] = (int)(c % BOUND); c /= BOUND;
    out_coords[4 * n_out + 2] = (int)(c % BOUND); c /= BOUND;
    out_coords[4 * n_out + 1] = (int)(c % BOUND); c /= BOUND;
    out_coords[4 * n_out] = (int)c;
    n_out++;
  }
  free(codes);
  return n_out;
}

static void scan_quantified(int kv, const int *knnz, int q, int *kpos, int *qkpos) {
  for (int id = 1; id <= kv; id++) {
    int acc = 0, qacc = 0;
    for (int i = 0; i < id; i++) {
      acc += knnz[i];
      qacc += (knnz[i] + q - 1) / q * q;
    }
    kpos[id] = acc;
    qkpos[id] = qacc;
  }
}

/* dense_map: kv*n_in ints, caller pre-fills with -1; knnz kv zeros; kpos,qkpos kv+1 zeros */
void lit_map_d2(int n_in, const int *in_coords, int n_out, const int *out_coords, const int *ks,
                const int *stride, const int *pad, int subm, int *dense_map, int *knnz, int *kpos,
                int *qkpos) {
  int kv = ks[0] * ks[1] * ks[2];
  int size = lit_table_size(n_in);
  int *idx = (int *)malloc(sizeof(int) * size);
  uint64_t *val = (uint64_t *)calloc(size, sizeof(uint64_t));
  for (int i = 0; i < size; i++) idx[i] = -1;
  lit_insert_hash(n_in, size, in_coords, idx);
  lit_insert_val(n_in, size, in_coords, idx, val);
  int mid = (ks[0] - 1) / 2 * ks[1] * ks[2] + (ks[1] - 1) / 2 * ks[2] + (ks[2] - 1) / 2;
  for (int o = 0; o < n_out; o++) {
    int b = out_coords[4 * o];
    int base[3];
    for (int a = 0; a < 3; a++)
      base[a] = subm ? out_coords[4 * o + 1 + a] : out_coords[4 * o + 1 + a] * stride[a] - pad[a];
    for (int kp = 0; kp < kv; kp++) {
      if (subm && kp == mid) continue;
      int d[3];
      offset_of(kp, ks, !subm, d);
      int in = lit_query(size, val, idx, b, base[0] + d[0], base[1] + d[1], base[2] + d[2]);
      if (in < 0 || in >= n_in) continue;
      knnz[kp]++;
      dense_map[(size_t)kp * n_in + in] = o;
    }
  }
  scan_quantified(kv, knnz, 128, kpos, qkpos);
  free(idx);
  free(val);
}

/* From the dense map: coded imap (n_in*kv, compacted in place to M entries), omap likewise,
 * icsr (n_in+1), ocsr (n_out+1).  imap/omap pre-filled with -1 by the caller. */
void lit_map_d1(int n_in, int n_out, int kv, const int *dense_map, int *imap, int *omap, int *icsr,
                int *ocsr) {
  for (int kp = 0; kp < kv; kp++) {
    int rank = 0;
    for (int i = 0; i < n_in; i++) {
      int o = dense_map[(size_t)kp * n_in + i];
      if (o < 0) continue;
      int code = kp * CSR_CODE + rank++;
      imap[(size_t)i * kv + kp] = code;
      omap[(size_t)o * kv + kp] = code;
    }
  }
  for (int pass = 0; pass < 2; pass++) {
    int n = pass ? n_out : n_in;
    int *map = pass ? omap : imap;
    int *csr = pass ? ocsr : icsr;
    size_t w = 0;
    int acc = 0;
    for (int r = 0; r < n; r++) {
      csr[r] = acc;
      for (int k = 0; k < kv; k++) {
        int c = map[(size_t)r * kv + k];
        if (c >= 0) { map[w++] = c; acc++; }
      }
    }
    csr[n] = acc;
  }
}
