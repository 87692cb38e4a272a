// Internal helpers shared by the HIP translation units of libpcengine_amd.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "pcengine_amd.h"

#define PCE_WAVE 64

// Host-side error text of the calling thread.
void pce_set_error(const char *fmt, ...);

#define PCE_FAIL(code, ...)      \
  do {                           \
    pce_set_error(__VA_ARGS__);  \
    return (code);               \
  } while (0)

#define PCE_HIP(expr)                                                                  \
  do {                                                                                 \
    hipError_t e_ = (expr);                                                            \
    if (e_ != hipSuccess) PCE_FAIL(PCE_EHIP, "%s: %s", #expr, hipGetErrorString(e_));  \
  } while (0)

#define PCE_LAUNCH_CHECK(name)                                                              \
  do {                                                                                      \
    hipError_t e_ = hipGetLastError();                                                      \
    if (e_ != hipSuccess) PCE_FAIL(PCE_EHIP, "launch %s: %s", name, hipGetErrorString(e_)); \
  } while (0)

static inline int64_t pce_align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }
static inline int64_t pce_div_up(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------------------------------------
// Packed coordinate key and slot function.
//
// key = b:16 | x+32768:16 | y+32768:16 | z+32768:16.  All-ones is the empty marker, so b < 32768.
// Four keys that differ only in the two low z bits share a 64-byte bucket (4 slots of 16 bytes):
// the +-1 z neighbours of a 3x3x3 stencil start probing in the same cache line.
// ---------------------------------------------------------------------------------------------
struct __attribute__((aligned(16))) pce_slot_t {
  unsigned long long key;
  unsigned int row;
  unsigned int pad;
};

#define PCE_EMPTY_KEY 0xFFFFFFFFFFFFFFFFull

__host__ __device__ static inline bool pce_coord_ok(int b, int x, int y, int z) {
  return b >= 0 && b < 32768 && x > -PCE_COORD_LIMIT && x < PCE_COORD_LIMIT && y > -PCE_COORD_LIMIT &&
         y < PCE_COORD_LIMIT && z > -PCE_COORD_LIMIT && z < PCE_COORD_LIMIT;
}

__host__ __device__ static inline unsigned long long pce_pack_key(int b, int x, int y, int z) {
  return ((unsigned long long)(unsigned)(b & 0xFFFF) << 48) |
         ((unsigned long long)(unsigned)((x + 32768) & 0xFFFF) << 32) |
         ((unsigned long long)(unsigned)((y + 32768) & 0xFFFF) << 16) |
         (unsigned long long)(unsigned)((z + 32768) & 0xFFFF);
}

__host__ __device__ static inline unsigned long long pce_mix64(unsigned long long h) {
  h ^= h >> 33;
  h *= 0xff51afd7ed558ccdull;
  h ^= h >> 33;
  h *= 0xc4ceb9fe1a85ec53ull;
  h ^= h >> 33;
  return h;
}

// slots is a power of two >= 4.
__host__ __device__ static inline unsigned long long pce_home_slot(unsigned long long key,
                                                                   unsigned long long slots) {
  unsigned long long bucket = pce_mix64(key >> 2) & ((slots >> 2) - 1);
  return (bucket << 2) | (key & 3ull);
}

// ---------------------------------------------------------------------------------------------
// Row order of the ordered output-stationary dataflow (pce_row_order, pce_conv_fwd_oso):
// order = perm[n_rows] | mask[n_rows] | tail[PCE_ORDER_TAIL] | rec[n_rows] (int4, 16-byte aligned) | srec[PCE_ORDER_SREC_ROWS][32].
// The tail holds the histogram, the cursors and the bases of the counting sort over ORDER_KEYS keys -- the offset of
// the rows with one neighbour, then (lowest, second-lowest) offset of the rows with two, then of the rows with more
// -- and the counts.  rec[p], for the positions p of rows that have a neighbour, repeats what a wavefront needs of the
// row at perm[p] in one 16-byte load: {row, mask, neighbour at the lowest offset of the mask, neighbour at the
// second-lowest or -1}.  srec[i], for the i-th row with two neighbours or more in the order (position n_plain +
// n_single + i), holds {row, mask, neighbour at offset 0, 1, ... 29 (-1 where the mask has no bit)}; it is written
// only where those rows number at most PCE_ORDER_SREC_ROWS (an eighth of the rows: the clouds the kernel that
// reads it is meant for).
// ---------------------------------------------------------------------------------------------
#define PCE_ORDER_TAIL 8192
#define PCE_ORDER_REC_OFFSET(n_rows) ((2 * (long long)(n_rows) + PCE_ORDER_TAIL + 3) & ~3ll)
#define PCE_ORDER_SREC_OFFSET(n_rows) (PCE_ORDER_REC_OFFSET(n_rows) + 4 * (long long)(n_rows))
#define PCE_ORDER_SREC_ROWS(n_rows) ((long long)(n_rows) / 8 + 32)
#define PCE_ORDER_SREC_KV 30
#define PCE_ORDER_ELEMS(n_rows) (PCE_ORDER_SREC_OFFSET(n_rows) + 32 * PCE_ORDER_SREC_ROWS(n_rows))
#define ORDER_MAX_KV 32
#define ORDER_KEYS 2048
#define ORDER_HIST 0
#define ORDER_CURSOR 2048
#define ORDER_BASE 4096
#define ORDER_N_SINGLE 8187   // rows with exactly one neighbour
#define ORDER_N_NONZERO 8188  // rows with any neighbour
#define ORDER_N_HEAVY 8189    // rows with ORDER_HEAVY_POPC neighbours or more
#define ORDER_PLAIN_CURSOR 8191
#define ORDER_HEAVY_POPC 3

