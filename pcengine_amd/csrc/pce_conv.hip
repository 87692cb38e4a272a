// Forward sparse convolution on gfx950: one MFMA tile kernel serving the fetch-on-demand,
// grouped-GEMM, dense-centre and output-stationary modes, plus the streaming gather / scatter /
// convert kernels of the gather-GEMM-scatter dataflow.
//
// Tile: 128 rows (4 wavefronts x 32 rows) x NT output channels, K staged through LDS in chunks.
// fp16: v_mfma_f32_32x32x16_f16, fp32 accumulate.  fp32: v_mfma_f32_32x32x2_f32.
// The A operand (feature rows) goes global -> registers with 16-byte loads, one row per lane; only
// the per-offset weight tile passes through LDS, laid out so that a lane's B fragment is one
// conflict-free 16-byte read.
#include <mutex>

#include "pce_common.h"

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T, int N>
struct VecOfC;
template <>
struct VecOfC<half_t, 8> { typedef half8 type; };
template <>
struct VecOfC<float, 4> { typedef f32x4 type; };
template <>
struct VecOfC<half_t, 4> { typedef _Float16 type __attribute__((ext_vector_type(4))); };

// plain store, or one with the non-temporal hint (see store_rows_via_lds) when the host asked for it
template <typename V>
__device__ __forceinline__ void store_maybe_stream(V *p, const V &v, bool stream) {
  if (stream)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

enum {
  MODE_FOD = 0,      // A row = imap[pair], out row = omap[pair]
  MODE_BUF = 1,      // A row = out row = quantised pair row (staging buffer)
  MODE_DENSE = 2,    // A row = out row = tile row, one fixed weight
  MODE_OS = 3,       // out row = tile row, A row = nbr[kp][row], loop over all offsets
  MODE_FOD_BUF = 4   // A row = imap[pair], out row = oslot[pair] (partial-row buffer in output-CSR order)
};
enum {
  EPI_ATOMIC_F32 = 0,  // fp32 atomic add, one column per lane
  EPI_ROWS = 1,        // store T, 16 bytes per lane along the row
  EPI_ROWS_F32 = 2,    // store fp32 (accumulator of the atomic dataflow), 16 bytes per lane
  EPI_ROWS_CSR = 3     // EPI_ROWS plus the sum of partial rows buf[ocsr[row] .. ocsr[row+1])
};

#define PCE_ROUTE_HEAD 4  // ints in front of the pair destinations of a routing array (pce_pair_route)
#define MAX_KV_ARGS 32  // kpos / qkpos travel in the kernel arguments up to this kernel volume

struct TileArgs {
  const void *A;
  const void *W;
  const void *Wp;  // fp16 weights in LDS-image order, or null
  void *out;
  const int *imap;
  const int *omap;
  const int *kpos;
  const int *qkpos;
  const int *nbr;
  const int *ocsr;
  const int *oslot;
  const void *buf;
  long long n_rows;  // MODE_DENSE / MODE_OS: rows of the output
  long long items;   // (tile, column slab) work items of the launch
  int slabs;         // column slabs per tile
  int kv, c_in, c_out;
  int lda, ldo;      // elements between consecutive rows of A and of `out` (rows of buf, res and out_alt are dense)
  int w_fixed;
  int mode, epi;
  int a_vec, w_vec, o_vec, b_vec;  // 16-byte accesses allowed on A rows / W rows / out rows / buf rows
  int k8_total, n_pad;             // packed weight extents
  int host_pos;                    // kpos_h / qkpos_h are valid
  const void *bias;                // fused epilogue of the launch that stores output rows: out = act(acc + bias + res)
  const void *res;
  int act;
  float slope;
  int act_alone_only;               // apply the activation only to rows without partial rows (ocsr tells)
  int stream;                       // output rows leave with the non-temporal hint (set_out)
  void *out_alt;                    // routed pair tiles: destination d < n_split is row d of `out` (a finished output
  int n_split;                      // row, takes the epilogue), d >= n_split is row d - n_split of `out_alt`
  int kpos_h[MAX_KV_ARGS + 1];
  int qkpos_h[MAX_KV_ARGS + 1];
};

template <typename T>
struct Cfg;
template <>
struct Cfg<half_t> {
  static constexpr int KC = 64;  // K chunk held in LDS
};
template <>
struct Cfg<float> {
  static constexpr int KC = 32;
};

// ---- packed fp16 weights -----------------------------------------------------------------------
// P[kp][k/8][n][k%8], n padded to a multiple of 32, k to a multiple of 8, zero filled: the 8
// consecutive k of one column are 16 contiguous bytes, which is what one lane feeds to the MFMA
// as its B fragment, and a (k-chunk, column-slab) tile is copied to LDS with 16-byte accesses.
__global__ void __launch_bounds__(256) pack_weights_kernel(const half_t *__restrict__ W, half_t *__restrict__ P, int kv,
                                                           int c_in, int c_out, int k8_total, int n_pad) {
  long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  long long total = (long long)kv * k8_total * n_pad;
  if (e >= total) return;
  int n = (int)(e % n_pad);
  int k8 = (int)((e / n_pad) % k8_total);
  int kp = (int)(e / ((long long)n_pad * k8_total));
  half8 v;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    int k = k8 * 8 + j;
    v[j] = (n < c_out && k < c_in) ? W[((long long)kp * c_in + k) * c_out + n] : (half_t)0;
  }
  *reinterpret_cast<half8 *>(&P[e * 8]) = v;
}

// XCD-aware work mapping.  Workgroups are dealt to the 8 XCDs round-robin in launch order and each
// XCD has its own L2.  Neighbouring tiles read overlapping feature rows, so every XCD gets one
// contiguous range of the (tile, column slab) items instead of every eighth one.  The launch is one-
// dimensional with ceil8(items) workgroups; returns false for the padding workgroups.
#define PCE_XCDS 8
__device__ __forceinline__ bool xcd_item(long long items, int slabs, bool remap, long long *tile, int *slab) {
  long long lid = blockIdx.x;
  long long per = (items + PCE_XCDS - 1) / PCE_XCDS;
  long long item = remap ? (lid % PCE_XCDS) * per + lid / PCE_XCDS : lid;
  if ((remap && lid / PCE_XCDS >= per) || item >= items) return false;
  *tile = item / slabs;
  *slab = (int)(item % slabs);
  return true;
}

// Workgroup barrier that orders LDS accesses only.  __syncthreads() also waits for every outstanding
// global load; here loads for later use (feature rows, partial rows) stay in flight across the
// barrier and are waited for where their registers are first read.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- weight chunk: global -> registers -> LDS --------------------------------------------------
// The global loads are issued together with the feature-row loads, before the first barrier of a
// chunk, so that both latencies overlap; the registers are written to LDS after that barrier.
// fp16 LDS layout: Wl[k/8][n][k%8];  fp32 LDS layout: Wl[k][n].
template <typename T, int NT>
struct WRegs;
template <int NT>
struct WRegs<half_t, NT> {
  static constexpr int N = (Cfg<half_t>::KC / 8) * NT / 256;
  half8 v[N];
};
template <int NT>
struct WRegs<float, NT> {
  static constexpr int N = Cfg<float>::KC * NT / 4 / 256;
  f32x4 v[N];
};

template <int NT, bool FAST>
__device__ __forceinline__ void load_weights(WRegs<half_t, NT> &r, const half_t *__restrict__ Wk,
                                             const half_t *__restrict__ Pk, int k0, int n0, const TileArgs &a) {
#pragma unroll
  for (int i = 0; i < WRegs<half_t, NT>::N; ++i) {
    int e = threadIdx.x + i * 256;
    int n = e % NT, k8 = e / NT;
    int gn = n0 + n, gk = k0 + k8 * 8;
    half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (FAST || Pk) {
      if (gk / 8 < a.k8_total && gn < a.n_pad) v = *reinterpret_cast<const half8 *>(&Pk[((long long)(gk / 8) * a.n_pad + gn) * 8]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (gn < a.c_out && gk + j < a.c_in) v[j] = Wk[(long long)(gk + j) * a.c_out + gn];
    }
    r.v[i] = v;
  }
}

template <int NT>
__device__ __forceinline__ void store_weights(half_t *Wl, const WRegs<half_t, NT> &r) {
#pragma unroll
  for (int i = 0; i < WRegs<half_t, NT>::N; ++i) {
    int e = threadIdx.x + i * 256;
    int n = e % NT, k8 = e / NT;
    *reinterpret_cast<half8 *>(&Wl[(k8 * NT + n) * 8]) = r.v[i];
  }
}

template <int NT, bool FAST>
__device__ __forceinline__ void load_weights(WRegs<float, NT> &r, const float *__restrict__ Wk, const float * /*Pk*/,
                                             int k0, int n0, const TileArgs &a) {
#pragma unroll
  for (int i = 0; i < WRegs<float, NT>::N; ++i) {
    int e = threadIdx.x + i * 256;
    int n = (e % (NT / 4)) * 4, k = e / (NT / 4);
    int gn = n0 + n, gk = k0 + k;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (gk < a.c_in) {
      if (FAST) {
        if (gn < a.c_out) v = *reinterpret_cast<const f32x4 *>(&Wk[(long long)gk * a.c_out + gn]);
      } else if (a.w_vec && gn + 4 <= a.c_out) {
        v = *reinterpret_cast<const f32x4 *>(&Wk[(long long)gk * a.c_out + gn]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (gn + j < a.c_out) v[j] = Wk[(long long)gk * a.c_out + gn + j];
      }
    }
    r.v[i] = v;
  }
}

template <int NT>
__device__ __forceinline__ void store_weights(float *Wl, const WRegs<float, NT> &r) {
#pragma unroll
  for (int i = 0; i < WRegs<float, NT>::N; ++i) {
    int e = threadIdx.x + i * 256;
    int n = (e % (NT / 4)) * 4, k = e / (NT / 4);
    *reinterpret_cast<f32x4 *>(&Wl[k * NT + n]) = r.v[i];
  }
}

// ---- feature rows of one K chunk: global -> registers in MFMA operand order -------------------
template <typename T>
struct AFrag;
template <>
struct AFrag<half_t> {
  half8 v[Cfg<half_t>::KC / 16];
};
template <>
struct AFrag<float> {
  f32x4 v[Cfg<float>::KC / 8];
};

template <bool FAST>
__device__ __forceinline__ void load_rows(AFrag<half_t> &f, const half_t *__restrict__ A, int arow, int k0, int klen,
                                          int c_in, int lda, int a_vec, int g) {
#pragma unroll
  for (int s = 0; s < Cfg<half_t>::KC / 16; ++s) {
    int k = k0 + s * 16 + g * 8;
    half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (arow >= 0 && s * 16 < klen) {
      const half_t *p = A + (long long)arow * lda + k;
      if (FAST) {
        if (k < c_in) v = *reinterpret_cast<const half8 *>(p);
      } else if (a_vec && k + 8 <= c_in) {
        v = *reinterpret_cast<const half8 *>(p);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (k + j < c_in) v[j] = p[j];
      }
    }
    f.v[s] = v;
  }
}

template <bool FAST>
__device__ __forceinline__ void load_rows(AFrag<float> &f, const float *__restrict__ A, int arow, int k0, int klen,
                                          int c_in, int lda, int a_vec, int g) {
#pragma unroll
  for (int s = 0; s < Cfg<float>::KC / 8; ++s) {
    int k = k0 + s * 8 + g * 4;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (arow >= 0 && s * 8 < klen) {
      const float *p = A + (long long)arow * lda + k;
      if (FAST) {
        if (k < c_in) v = *reinterpret_cast<const f32x4 *>(p);
      } else if (a_vec && k + 4 <= c_in) {
        v = *reinterpret_cast<const f32x4 *>(p);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (k + j < c_in) v[j] = p[j];
      }
    }
    f.v[s] = v;
  }
}

// ---- one K chunk of MFMA work for a wavefront ---------------------------------------------------
// ROWMAJOR = false: D[row][col], lane (l32, g) holds column l32 of rows 8*(j/4) + 4*g + j%4 (one
//   column per lane: what the atomic epilogue wants).
// ROWMAJOR = true: the operands are exchanged, D'[col][row]: lane (l32, g) holds, for ITS OWN row
//   l32, columns 8*(j/4) + 4*g + j%4 of every 32-column block (what the row epilogue wants).
template <int NB, bool ROWMAJOR>
__device__ __forceinline__ void mma_chunk(f32x16 (&acc)[NB], const half_t *Wl, const AFrag<half_t> &f, int klen,
                                          int l32, int g) {
  constexpr int NT = NB * 32;
#pragma unroll
  for (int s = 0; s < Cfg<half_t>::KC / 16; ++s) {
    if (s * 16 < klen) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        half8 b = *reinterpret_cast<const half8 *>(&Wl[((s * 2 + g) * NT + nb * 32 + l32) * 8]);
        if (ROWMAJOR)
          acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, f.v[s], acc[nb], 0, 0, 0);
        else
          acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.v[s], b, acc[nb], 0, 0, 0);
      }
    }
  }
}

template <int NB, bool ROWMAJOR>
__device__ __forceinline__ void mma_chunk(f32x16 (&acc)[NB], const float *Wl, const AFrag<float> &f, int klen,
                                          int l32, int g) {
  constexpr int NT = NB * 32;
#pragma unroll
  for (int s = 0; s < Cfg<float>::KC / 8; ++s) {
    if (s * 8 < klen) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // this MFMA contracts k = s*8 + e (lanes 0-31) and k = s*8 + 4 + e (lanes 32-63)
        int kk = s * 8 + g * 4 + e;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          float b = Wl[kk * NT + nb * 32 + l32];
          if (ROWMAJOR)
            acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(b, f.v[s][e], acc[nb], 0, 0, 0);
          else
            acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.v[s][e], b, acc[nb], 0, 0, 0);
        }
      }
    }
  }
}

// ---- epilogues ---------------------------------------------------------------------------------
template <int NB>
__device__ __forceinline__ void epilogue_atomic(const f32x16 (&acc)[NB], int orow, const TileArgs &a, int n0, int l32,
                                                int g) {
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    int r = 8 * (j >> 2) + 4 * g + (j & 3);
    int dst = __shfl(orow, r, PCE_WAVE);
    if (dst < 0) continue;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      int col = n0 + nb * 32 + l32;
      if (col < a.c_out) unsafeAtomicAdd((float *)a.out + (long long)dst * a.c_out + col, acc[nb][j]);
    }
  }
}

// Row epilogue, first step: the two lanes of a row (g = 0, 1) exchange 4-column pieces so that each
// ends with 8 consecutive columns per 16-column group: lane g owns columns 16*h + 8*g + 0..7,
// h = 0, 1, of every 32-column block.
template <int NB>
__device__ __forceinline__ void gather_row_pieces(const f32x16 (&acc)[NB], float (&V)[NB][2][8], int g) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int qa = 2 * h, qb = 2 * h + 1;  // lane g=0 keeps piece qa, lane g=1 keeps piece qb
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (NB > 2) {
          // wide tiles: a shuffle and two selects (the swap below costs the kernels that hold 64 accumulators per lane
          // a tenth of a network forward)
          float lo = acc[nb][4 * qa + i], hi = acc[nb][4 * qb + i];
          float recv = __shfl_xor(g == 0 ? hi : lo, 32, PCE_WAVE);
          V[nb][h][i] = g == 0 ? lo : recv;
          V[nb][h][4 + i] = g == 0 ? recv : hi;
        } else {
          // one instruction swaps the upper half of `lo` with the lower half of `hi`: lanes 0-31 then hold (own lo,
          // partner's lo), lanes 32-63 (partner's hi, own hi)
          auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[nb][4 * qa + i]), __float_as_uint(acc[nb][4 * qb + i]), false, false);
          V[nb][h][i] = __uint_as_float(r[0]);
          V[nb][h][4 + i] = __uint_as_float(r[1]);
        }
      }
    }
  }
}

// Per-wavefront LDS region, in 16-byte pieces: big enough for 16 fp32 rows or 32 fp16 rows of the
// output tile with 8 elements of padding per row.  It first stages partial rows, then the finished
// rows on their way to memory.
template <int NB>
struct WaveLds {
  static constexpr int NT = NB * 32;
  static constexpr int PIECES = 4 * (NT + 8);
};

// Partial rows of a tile's 128 output rows are one contiguous range [tb, te) of the buffer.  The
// workgroup copies it through LDS CH rows at a time with coalesced 16-byte loads (PARTIAL_LOADS per
// thread, all in flight together; the first round is requested at kernel start), and every lane
// adds the rows [e0, e1) of its own output row.  Sharing the rounds among the four wavefronts keeps
// a tile inside a dense cluster from serialising many small rounds in one wavefront.
#define PARTIAL_LOADS 4  // 16-byte pieces per thread and round

template <typename T, int NB>
struct Partials {
  static constexpr int NT = NB * 32;
  static constexpr int CPL = 16 / sizeof(T);  // elements per 16-byte piece
  static constexpr int PPR = NT / CPL;        // pieces per partial row (of this column slab)
  static constexpr int LOADS = PARTIAL_LOADS;
  static constexpr int CAP = LOADS * 256 < 4 * WaveLds<NB>::PIECES ? LOADS * 256 : 4 * WaveLds<NB>::PIECES;
  static constexpr int CH = CAP / PPR;        // partial rows per round
  typedef typename VecOfC<T, CPL>::type PV;
};

template <typename T, int NB, typename PV>
__device__ __forceinline__ void load_partial_chunk(PV (&r)[PARTIAL_LOADS], int cb, int te, const TileArgs &a, int n0) {
  typedef Partials<T, NB> P;
  const T *buf = (const T *)a.buf;
#pragma unroll
  for (int i = 0; i < P::LOADS; ++i) {
    int pc = threadIdx.x + 256 * i;
    int ent = pc / P::PPR, piece = pc - ent * P::PPR;
    int e = cb + ent;
    int col = n0 + piece * P::CPL;
    PV v;
#pragma unroll
    for (int j = 0; j < P::CPL; ++j) v[j] = (T)0;
    if (ent < P::CH && e < te && col < a.c_out) v = *reinterpret_cast<const PV *>(buf + (long long)e * a.c_out + col);
    r[i] = v;
  }
}

template <typename T, int NB, typename PV>
__device__ __forceinline__ void add_partials(float (&V)[NB][2][8], PV *Pl, PV (&first)[PARTIAL_LOADS], int e0, int e1,
                                             int tb, int te, const TileArgs &a, int n0, int g) {
  typedef Partials<T, NB> P;
  for (int cb = tb; cb < te; cb += P::CH) {  // tb, te are uniform over the workgroup
    if (cb > tb) load_partial_chunk<T, NB, PV>(first, cb, te, a, n0);
#pragma unroll
    for (int i = 0; i < P::LOADS; ++i)
      if (threadIdx.x + 256 * i < P::CH * P::PPR) Pl[threadIdx.x + 256 * i] = first[i];
    lds_barrier();
    int lo = e0 > cb ? e0 : cb, hi = e1 < cb + P::CH ? e1 : cb + P::CH;
    for (int e = lo; e < hi; ++e) {
      const PV *rowp = Pl + (e - cb) * P::PPR;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          if (sizeof(T) == 2) {
            PV x = rowp[nb * 4 + 2 * h + g];
#pragma unroll
            for (int j = 0; j < 8; ++j) V[nb][h][j] += (float)x[j % P::CPL];
          } else {
            PV x0 = rowp[nb * 8 + 4 * h + 2 * g], x1 = rowp[nb * 8 + 4 * h + 2 * g + 1];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              V[nb][h][j] += (float)x0[j];
              V[nb][h][4 + j] += (float)x1[j];
            }
          }
        }
      }
    }
    lds_barrier();  // the region is rewritten by the next round or by the store phase
  }
}

// element-wise partial-row sum for rows that are not 16-byte multiples
template <typename T, int NB>
__device__ __forceinline__ void add_partials_slow(float (&V)[NB][2][8], int e0, int e1, const TileArgs &a, int n0,
                                                  int g) {
  const T *buf = (const T *)a.buf;
  for (int e = e0; e < e1; ++e) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          int col = n0 + nb * 32 + 16 * h + 8 * g + j;
          if (col < a.c_out) V[nb][h][j] += (float)buf[(long long)e * a.c_out + col];
        }
  }
}

// ---- fused epilogue: out = act(acc + bias + residual) -------------------------------------------
// Written without branches: with `act` a kernel argument the compiler turned the three-way form into scalar
// compares, jumps and a reload of the slope around every element of an unrolled epilogue.  The two
// coefficients depend on `act` alone and are hoisted out of the loops.
struct ActK {
  float mul;      // what a non-positive value is multiplied by ...
  unsigned keep;  // ... and whether the product survives
};
// `on` may differ from lane to lane (rows that get their activation in a later pass): it goes into the
// coefficients, not into a test around every element
__device__ __forceinline__ ActK act_coeffs(int act, float slope, bool on) {
  ActK k;
  k.mul = (on && act == PCE_ACT_LEAKY_RELU) ? slope : 1.f;
  k.keep = (on && act == PCE_ACT_RELU) ? 0u : ~0u;
  return k;
}
__device__ __forceinline__ float act_apply(float v, const ActK &k) {
  const float t = __uint_as_float(__float_as_uint(v * k.mul) & k.keep);
  return v > 0.f ? v : t;  // no activation: t == v
}
__device__ __forceinline__ float act_apply(float v, int act, float slope) { return act_apply(v, act_coeffs(act, slope, true)); }
// derivative of the activation where its output is `out` (ReLU and LeakyReLU with a positive slope keep the sign)
__device__ __forceinline__ float act_slope_at(float out, int act, float slope) {
  const float neg = act == PCE_ACT_RELU ? 0.f : (act == PCE_ACT_LEAKY_RELU ? slope : 1.f);
  return out > 0.f ? 1.f : neg;
}

// eight consecutive elements of a row of T as floats; VEC: the address is 16-byte aligned
template <typename T, bool VEC>
__device__ __forceinline__ void add8(float (&v)[8], const T *p, int valid) {
  if (VEC) {
    if (sizeof(T) == 2) {
      half8 x = *reinterpret_cast<const half8 *>(p);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] += (float)x[j];
    } else {
      f32x4 x0 = *reinterpret_cast<const f32x4 *>(p), x1 = *reinterpret_cast<const f32x4 *>(p + 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] += (float)x0[j];
        v[4 + j] += (float)x1[j];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < valid) v[j] += (float)p[j];
  }
}

// one 16-byte-aligned piece of eight elements of T, loaded whole (two 16-byte loads for fp32)
template <typename T>
struct Piece8;
template <>
struct Piece8<half_t> {
  half8 x;
  __device__ __forceinline__ void load(const half_t *p) { x = *reinterpret_cast<const half8 *>(p); }
  __device__ __forceinline__ float at(int j) const { return (float)x[j]; }
};
template <>
struct Piece8<float> {
  f32x4 x0, x1;
  __device__ __forceinline__ void load(const float *p) {
    x0 = *reinterpret_cast<const f32x4 *>(p);
    x1 = *reinterpret_cast<const f32x4 *>(p + 4);
  }
  __device__ __forceinline__ float at(int j) const { return j < 4 ? x0[j] : x1[j - 4]; }
};

// on the row pieces of the tile epilogue (lane g of row `orow` owns columns n0 + 32*nb + 16*h + 8*g + 0..7).
// VEC: every piece is 16-byte aligned and lies wholly inside or outside the row.  The pieces of the bias, then
// those of the residual row, are requested together from addresses that are valid for every lane (a lane
// without a row or column reads the base and drops the value), so that a lane waits once per operand: loads
// guarded piece by piece were issued and waited for one after the other, sixteen round trips at the end of
// every workgroup of a 128-column tile.
// Used where the register budget is fixed by the launch bounds anyway (the pipelined kernel: 128 registers, four
// workgroups per CU); in the tile kernel and the barrier-free kernel the addresses and pieces in flight cost a
// resident wavefront (output-stationary tile kernel at 128 columns: 97 -> 145 us), so those keep the guarded form.
// NBB: column blocks whose pieces are in flight together (8 registers per block for fp16 rows, 16 for fp32).
template <typename T, int NB, bool VEC, int NBB>
__device__ __forceinline__ void epilogue_row_pieces_batched(float (&V)[NB][2][8], const TileArgs &a, int orow, int n0, int g,
                                                            bool with_act) {
  const T *bias = (const T *)a.bias;
  const T *res = (const T *)a.res;
  if (VEC) {
#pragma unroll
    for (int op = 0; op < 2; ++op) {
      const T *base = op == 0 ? bias : res;
      if (!base) continue;
      const long long row_off = op == 0 ? 0ll : (long long)(orow >= 0 ? orow : 0) * a.c_out;
#pragma unroll
      for (int nb0 = 0; nb0 < NB; nb0 += NBB) {
        Piece8<T> x[NBB][2];
#pragma unroll
        for (int nb = 0; nb < NBB; ++nb)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            int c0 = n0 + (nb0 + nb) * 32 + 16 * h + 8 * g;
            bool ok = nb0 + nb < NB && orow >= 0 && c0 < a.c_out;
            x[nb][h].load(ok ? base + row_off + c0 : base);
          }
#pragma unroll
        for (int nb = 0; nb < NBB; ++nb)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            if (nb0 + nb >= NB) continue;
            int c0 = n0 + (nb0 + nb) * 32 + 16 * h + 8 * g;
            bool ok = orow >= 0 && c0 < a.c_out;
#pragma unroll
            for (int j = 0; j < 8; ++j) V[nb0 + nb][h][j] += ok ? x[nb][h].at(j) : 0.f;
          }
      }
    }
  } else {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        int c0 = n0 + nb * 32 + 16 * h + 8 * g;
        int valid = a.c_out - c0;
        if (valid > 0 && orow >= 0) {
          if (bias) add8<T, false>(V[nb][h], bias + c0, valid);
          if (res) add8<T, false>(V[nb][h], res + (long long)orow * a.c_out + c0, valid);
        }
      }
  }
  const ActK k = act_coeffs(a.act, a.slope, with_act);
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 8; ++j) V[nb][h][j] = act_apply(V[nb][h][j], k);
}

// the same with every piece guarded and added as it arrives: fewest registers
template <typename T, int NB, bool VEC>
__device__ __forceinline__ void epilogue_row_pieces(float (&V)[NB][2][8], const TileArgs &a, int orow, int n0, int g,
                                                    bool with_act) {
  const T *bias = (const T *)a.bias;
  const T *res = (const T *)a.res;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int c0 = n0 + nb * 32 + 16 * h + 8 * g;
      int valid = a.c_out - c0;
      if (valid > 0 && orow >= 0) {
        if (bias) add8<T, VEC>(V[nb][h], bias + c0, valid);
        if (res) add8<T, VEC>(V[nb][h], res + (long long)orow * a.c_out + c0, valid);
      }
      if (with_act) {
#pragma unroll
        for (int j = 0; j < 8; ++j) V[nb][h][j] = act_apply(V[nb][h][j], a.act, a.slope);
      }
    }
}

// element-wise stores straight from the row pieces (rows that are not 16-byte multiples)
template <typename TO, int NB>
__device__ __forceinline__ void store_row_pieces_slow(const float (&V)[NB][2][8], TO *out, int orow, const TileArgs &a,
                                                      int n0, int g) {
  if (orow < 0) return;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        int col = n0 + nb * 32 + 16 * h + 8 * g + j;
        if (col < a.c_out) out[(long long)orow * a.ldo + col] = (TO)V[nb][h][j];
      }
}

// Finished rows -> memory through the wavefront's LDS region: the lane that owns (row, 8 columns)
// writes its pieces; then 16 bytes per lane are read back along the rows, so that NT*sizeof(TO)/16
// consecutive lanes store one full row segment (whole 128-byte lines at 64 fp16 channels).
// a.stream: the stores carry the non-temporal hint.  Rows kept as ordinary dirty lines are written back in one
// burst when the kernel ends (2.3 of 9.3 us on the 150 k-voxel layer); streamed out they leave while the kernel
// runs, but the next layer then finds none of them in the L2 of its XCD.  The host decides per launch (set_out).
template <typename TO, int NB, int ROWS = (sizeof(TO) == 2 ? 32 : 16), bool SPLIT = false>
__device__ __forceinline__ void store_rows_via_lds(const float (&V)[NB][2][8], void *region, TO *out, int orow,
                                                   const TileArgs &a, int n0, int lane, int l32, int g, bool stream,
                                                   int ld_out = -1) {   // row stride of `out` where it is not a.ldo
  constexpr int NT = NB * 32;
  constexpr int EPP = 16 / sizeof(TO);              // elements per piece
  constexpr int LDP = (NT + 8) / EPP;               // row stride in pieces; ROWS rows per pass
  constexpr int PPR = NT / EPP;                     // pieces per row
  constexpr int ITS = ROWS * PPR / 64;
  typedef typename VecOfC<TO, EPP>::type OV;
  OV *R = (OV *)region;
#pragma unroll
  for (int pass = 0; pass < 32 / ROWS; ++pass) {
    if ((l32 / ROWS) == pass) {
      int lr = l32 % ROWS;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          int c0 = nb * 32 + 16 * h + 8 * g;  // first of this lane's 8 columns
          if (sizeof(TO) == 2) {
            OV y;
#pragma unroll
            for (int j = 0; j < 8; ++j) y[j % EPP] = (TO)V[nb][h][j];
            R[lr * LDP + c0 / EPP] = y;
          } else {
            OV y0, y1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              y0[j] = (TO)V[nb][h][j];
              y1[j] = (TO)V[nb][h][4 + j];
            }
            R[lr * LDP + c0 / EPP] = y0;
            R[lr * LDP + c0 / EPP + 1] = y1;
          }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
      int idx = it * 64 + lane;
      int lr = idx / PPR, ch = idx - lr * PPR;
      int dst = __shfl(orow, pass * ROWS + lr, PCE_WAVE);
      int col = n0 + ch * EPP;
      OV y = R[lr * LDP + ch];
      TO *base = out;
      int ld = ld_out >= 0 ? ld_out : a.ldo;
      if (SPLIT && dst >= a.n_split) {
        base = (TO *)a.out_alt;
        dst -= a.n_split;
        ld = a.c_out;
      }
      if (dst >= 0 && col < a.c_out) {
        OV *dp = reinterpret_cast<OV *>(base + (long long)dst * ld + col);
        if (stream)
          __builtin_nontemporal_store(y, dp);
        else
          *dp = y;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

// FAST: every row (features, weights or packed weights, output, partial buffer) is a multiple of
// 16 bytes and 16-byte aligned, fp16 weights are packed: no element-wise access path is compiled.
// TMODE / TEPI >= 0 fix the mode and the epilogue at compile time (the hot combinations); -1 reads
// them from the arguments.
template <typename T, int NB, bool FAST, int TMODE, int TEPI>
__global__ void __launch_bounds__(256, ((TMODE >= 0 && sizeof(T) == 2 && NB <= 2) ? 5 : 1)) tile_gemm_kernel(TileArgs a) {
  const int mode = TMODE >= 0 ? TMODE : a.mode;
  const int epi = TEPI >= 0 ? TEPI : a.epi;
  constexpr int NT = NB * 32;
  constexpr int KC = Cfg<T>::KC;
  typedef Partials<T, NB> P;
  __shared__ __attribute__((aligned(16))) T Wl[KC * NT];
  __shared__ __attribute__((aligned(16))) typename P::PV Pl[4][WaveLds<NB>::PIECES];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  long long tile;
  int slab;
  // only the output-stationary mode re-reads rows across tiles; streaming modes keep launch order
  if (!xcd_item(a.items, a.slabs, mode == MODE_OS, &tile, &slab)) return;
  const int n0 = slab * NT;
  const T *A = (const T *)a.A;
  const T *W = (const T *)a.W;
  const T *Wp = (const T *)a.Wp;

  int arow = -1, orow = -1;
  int w_begin, w_end;
  long long row = tile * 128 + wave * 32 + l32;
  if (mode == MODE_DENSE || mode == MODE_OS) {
    bool ok = row < a.n_rows;
    orow = ok ? (int)row : -1;
    arow = (mode == MODE_DENSE) ? orow : -1;
    w_begin = (mode == MODE_DENSE) ? a.w_fixed : 0;
    w_end = (mode == MODE_DENSE) ? a.w_fixed + 1 : a.kv;
  } else {
    // indicator: which offset owns this tile = number of segment ends at or before its first row
    long long q0 = tile * 128;
    int widx = 0;
    long long p;
    bool ok;
    if (a.host_pos) {
      for (int i = 0; i < a.kv; ++i) widx += ((long long)a.qkpos_h[i + 1] <= q0) ? 1 : 0;
      if (widx >= a.kv) return;
      p = q0 - a.qkpos_h[widx] + a.kpos_h[widx] + wave * 32 + l32;
      ok = p < (long long)a.kpos_h[widx + 1];
    } else {
      int cnt = 0;
      for (int base = 0; base < a.kv; base += 64) {
        int i = base + lane;
        bool pr = (i < a.kv) && ((long long)a.qkpos[i + 1] <= q0);
        cnt += __popcll(__ballot(pr));
      }
      widx = __builtin_amdgcn_readfirstlane(cnt);
      if (widx >= a.kv) return;
      p = q0 - a.qkpos[widx] + a.kpos[widx] + wave * 32 + l32;
      ok = p < (long long)a.kpos[widx + 1];
    }
    if (ok) {
      arow = (mode == MODE_BUF) ? (int)row : a.imap[p];
      orow = (mode == MODE_FOD) ? a.omap[p] : (mode == MODE_FOD_BUF ? a.oslot[p] : (int)row);
    }
    w_begin = widx;
    w_end = widx + 1;
  }
  // MODE_DENSE and the pair modes use one offset: issue its first chunk of loads now, ahead of the
  // partial-row metadata, so that nothing delays them
  const int klen0 = a.c_in < KC ? a.c_in : KC;
  WRegs<T, NT> wr;
  AFrag<T> af;
  if (mode != MODE_OS) {
    load_weights<NT, FAST>(wr, W + (long long)w_begin * a.c_in * a.c_out,
                           Wp ? Wp + (long long)w_begin * a.k8_total * a.n_pad * 8 : nullptr, 0, n0, a);
    load_rows<FAST>(af, A, arow, 0, klen0, a.c_in, a.lda, a.a_vec, g);
  }
  // Partial rows: the tile's contiguous range [tb, te) comes from two scalar loads (uniform index),
  // so the first round of partial rows is requested together with the feature rows; the per-lane
  // bounds [e0, e1) of the lane's own row are only needed in the epilogue.
  int e0 = 0, e1 = 0, tb = 0, te = 0;
  typename P::PV first[P::LOADS];
  const bool csr_fast = (epi == EPI_ROWS_CSR) && (FAST || a.b_vec);
  if (epi == EPI_ROWS_CSR) {
    long long r0 = tile * 128;
    if (r0 < a.n_rows) {
      long long r1 = r0 + 128 < a.n_rows ? r0 + 128 : a.n_rows;
      tb = a.ocsr[r0];
      te = a.ocsr[r1];
    }
    if (csr_fast) load_partial_chunk<T, NB, typename P::PV>(first, tb, te, a, n0);
    if (orow >= 0) {
      e0 = a.ocsr[orow];
      e1 = a.ocsr[orow + 1];
    }
  }

  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;

  const bool rowmajor = epi != EPI_ATOMIC_F32;
  bool lds_used = false;
  for (int w = w_begin; w < w_end; ++w) {
    if (mode == MODE_OS) {
      arow = orow >= 0 ? a.nbr[(long long)w * a.n_rows + orow] : -1;
      if (!__syncthreads_or(arow >= 0)) continue;
    }
    const bool wave_has = __ballot(arow >= 0) != 0ull;
    const T *Wk = W + (long long)w * a.c_in * a.c_out;
    const T *Pk = Wp ? Wp + (long long)w * a.k8_total * a.n_pad * 8 : nullptr;
    for (int k0 = 0; k0 < a.c_in; k0 += KC) {
      int klen = a.c_in - k0 < KC ? a.c_in - k0 : KC;
      if (mode == MODE_OS || k0 > 0) {
        load_weights<NT, FAST>(wr, Wk, Pk, k0, n0, a);
        load_rows<FAST>(af, A, arow, k0, klen, a.c_in, a.lda, a.a_vec, g);
      }
      if (lds_used) lds_barrier();  // the previous chunk's LDS reads are complete
      store_weights<NT>(Wl, wr);
      lds_barrier();
      lds_used = true;
      if (wave_has) {
        if (rowmajor)
          mma_chunk<NB, true>(acc, Wl, af, klen, l32, g);
        else
          mma_chunk<NB, false>(acc, Wl, af, klen, l32, g);
      }
    }
  }

  if (!rowmajor) {
    epilogue_atomic<NB>(acc, orow, a, n0, l32, g);
    return;
  }
  float V[NB][2][8];
  gather_row_pieces<NB>(acc, V, g);
  if (epi == EPI_ROWS_CSR) {
    if (csr_fast)
      add_partials<T, NB, typename P::PV>(V, &Pl[0][0], first, e0, e1, tb, te, a, n0, g);
    else
      add_partials_slow<T, NB>(V, e0, e1, a, n0, g);
  }
  const bool f32out = (epi == EPI_ROWS_F32) || sizeof(T) == 4;
  if (a.bias || a.res || a.act) {  // set only on launches that store finished output rows
    bool with_act = a.act != PCE_ACT_NONE;
    // rows that receive partial rows in a later pass get their activation there
    if (with_act && a.act_alone_only) with_act = orow >= 0 && a.ocsr[orow] == a.ocsr[orow + 1];
    if (FAST)
      epilogue_row_pieces<T, NB, true>(V, a, orow, n0, g, with_act);
    else
      epilogue_row_pieces<T, NB, false>(V, a, orow, n0, g, with_act);
  }
  if (FAST || a.o_vec) {
    if (f32out)
      store_rows_via_lds<float, NB>(V, Pl[wave], (float *)a.out, orow, a, n0, lane, l32, g, a.stream);
    else
      store_rows_via_lds<half_t, NB>(V, Pl[wave], (half_t *)a.out, orow, a, n0, lane, l32, g, a.stream);
  } else {
    if (f32out)
      store_row_pieces_slow<float, NB>(V, (float *)a.out, orow, a, n0, g);
    else
      store_row_pieces_slow<half_t, NB>(V, (half_t *)a.out, orow, a, n0, g);
  }
}

// ---- wavefront-independent form of the pair tiles and of the centre GEMM -------------------------
// For fp16 rows of at most 64 channels a layer is bound by memory, and a workgroup that stages its
// weight tile through LDS behind a barrier makes all resident workgroups read, compute and write in
// step.  Here every wavefront owns 32 rows (pairs or output rows) and takes its weight fragments
// straight from the packed copy (8 KB per offset: it stays in cache), so there is no workgroup
// barrier and wavefronts drift apart.  Chunks [0, pair.items) are pair chunks, the rest rows of the
// centre GEMM.
//
// The 32 rows of a chunk reach LDS with global -> LDS copies in line order (eight lanes per 128-byte row, so
// a load instruction touches 8 whole lines; the MFMA fragment order, one lane per row, touches 32 lines per
// instruction with 32 bytes of each and was 1.3 us slower on the 150 k-voxel layer), and the fragments are
// read from there.  Which 16-byte piece of its row a lane fetches is XORed with the row index, so that the
// fragment reads of 8 consecutive rows fall into different banks.  The region then stages the finished rows
// on their way out (full lines, streaming stores).
template <int PPR>
__device__ __forceinline__ int row_swizzle(int row) {
  return (PPR >= 8 && PPR % 8 == 0) ? (row & 7) : ((PPR == 4 || (PPR > 8 && PPR % 4 == 0)) ? (row & 3) : (PPR == 2 ? (row & 1) : 0));
}

template <int NB, int KS>
__global__ void __launch_bounds__(256, 4) wave_gemm_kernel(TileArgs pair, TileArgs centre) {
  constexpr int PPR = KS * 2;   // 16-byte pieces per input row
  constexpr int NI = KS;        // global -> LDS instructions per chunk: 32 rows x PPR pieces / 64 lanes
  // a wavefront's region holds its 32 input rows first, then its finished rows on their way out
  constexpr int REGION = WaveLds<NB>::PIECES > 32 * PPR ? WaveLds<NB>::PIECES : 32 * PPR;
  __shared__ __attribute__((aligned(16))) half8 Pl[4][REGION];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const long long chunk = (long long)blockIdx.x * 4 + wave;   // 32 rows (pairs or output rows) per wavefront
  const bool is_pair = chunk < pair.items;
  if (!is_pair && chunk - pair.items >= centre.items) return;
  // features, weights and shapes are those of `pair` for both kinds of chunk; only the destination
  // differs (selecting a whole argument block at run time would copy it to private memory)
  const TileArgs &a = pair;
  const half_t *A = (const half_t *)a.A;
  int orow = -1, widx;
  long long src[NI];   // the row whose piece this lane fetches in instruction `it` (a valid row stands in for a missing one)
  if (is_pair) {
    const long long q0 = chunk * 32;
    widx = 0;
    for (int i = 0; i < pair.kv; ++i) widx += ((long long)pair.qkpos_h[i + 1] <= q0) ? 1 : 0;
    if (widx >= pair.kv) return;
    const long long p0 = q0 - pair.qkpos_h[widx] + pair.kpos_h[widx], pend = pair.kpos_h[widx + 1];
    if (p0 + l32 < pend) orow = pair.oslot[p0 + l32];
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int r = (it * 64 + lane) / PPR;
      src[it] = p0 + r < pend ? (long long)pair.imap[p0 + r] : 0ll;
    }
  } else {
    widx = centre.w_fixed;
    const long long row0 = (chunk - pair.items) * 32;
    orow = row0 + l32 < centre.n_rows ? (int)(row0 + l32) : -1;
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int r = (it * 64 + lane) / PPR;
      src[it] = row0 + r < centre.n_rows ? row0 + r : centre.n_rows - 1;
    }
  }
#pragma unroll
  for (int it = 0; it < NI; ++it) {
    const int e = it * 64 + lane, r = e / PPR, sl = e % PPR;
    const half_t *gp = A + src[it] * a.lda + ((sl ^ row_swizzle<PPR>(r)) * 8);
    // LDS destination: wave-uniform base, the hardware adds lane * 16 bytes
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                     (__attribute__((address_space(3))) void *)&Pl[wave][it * 64], 16, 0, 0);
  }
  const half_t *Wk = (const half_t *)a.Wp + (long long)widx * a.k8_total * a.n_pad * 8;
  half8 wf[KS][NB];
#pragma unroll
  for (int s = 0; s < KS; ++s)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      wf[s][nb] = *reinterpret_cast<const half8 *>(Wk + ((long long)(2 * s + g) * a.n_pad + nb * 32 + l32) * 8);
  // the global -> LDS copies have landed once nothing is outstanding; the fragment reads stay behind this statement
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;
  // a missing row (a padding pair of the offset's last chunk, a row past the end of the tensor) multiplies
  // whatever stands in for it: its products stay in its own lane and are never stored
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const half8 af = Pl[wave][l32 * PPR + ((2 * s + g) ^ row_swizzle<PPR>(l32))];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[s][nb], af, acc[nb], 0, 0, 0);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();   // every lane has read its fragments: the region becomes the output staging area
  float V[NB][2][8];
  gather_row_pieces<NB>(acc, V, g);
  if (!is_pair && (centre.bias || centre.res || centre.act)) {
    // rows that receive partial rows later get their activation from the pass that adds them
    const bool alone = orow >= 0 && centre.ocsr[orow] == centre.ocsr[orow + 1];
    epilogue_row_pieces<half_t, NB, true>(V, centre, orow, 0, g, false);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) V[nb][h][j] = alone ? act_apply(V[nb][h][j], centre.act, centre.slope) : V[nb][h][j];
  }
  half_t *out = (half_t *)(is_pair ? pair.out : centre.out);
  store_rows_via_lds<half_t, NB>(V, Pl[wave], out, orow, a, 0, lane, l32, g, is_pair ? pair.stream : centre.stream,
                                 is_pair ? pair.ldo : centre.ldo);
}

// pair chunks and centre rows of one layer in one launch (either part may be empty): 32 rows per wavefront, the
// caller sizes pair.items / centre.items for that
static int launch_wave_gemm(const TileArgs &pair, const TileArgs &centre, hipStream_t s) {
  long long chunks = pair.items + centre.items;
  if (chunks <= 0) return PCE_OK;
  if (chunks / 4 >= (1ll << 31) - 8) PCE_FAIL(PCE_ECAPACITY, "chunk count %lld exceeds the grid limit", chunks);
  unsigned grid = (unsigned)pce_div_up(chunks, 4);
  int nb = (pair.c_out + 31) / 32, ks = pair.c_in / 16;  // both blocks come from base_args of one layer
#define PCE_WAVE_CASE(NB_, KS_)                                                                              \
  if (nb == NB_ && ks == KS_) {                                                                              \
    hipLaunchKernelGGL((wave_gemm_kernel<NB_, KS_>), dim3(grid), dim3(256), 0, s, pair, centre);             \
    PCE_LAUNCH_CHECK("wave_gemm");                                                                           \
    return PCE_OK;                                                                                           \
  }
  PCE_WAVE_CASE(1, 1) PCE_WAVE_CASE(1, 2) PCE_WAVE_CASE(1, 3) PCE_WAVE_CASE(1, 4)
  PCE_WAVE_CASE(2, 1) PCE_WAVE_CASE(2, 2) PCE_WAVE_CASE(2, 3) PCE_WAVE_CASE(2, 4)
#undef PCE_WAVE_CASE
  PCE_FAIL(PCE_EINVAL, "wave_gemm: unsupported shape c_in=%d c_out=%d", pair.c_in, pair.c_out);
}

// shapes the wavefront-independent kernel takes: fp16, packed weights, 16-byte rows everywhere
static bool wave_gemm_ok(const TileArgs &a, int elem_size) {
  return elem_size == 2 && a.Wp && a.a_vec && a.o_vec && a.c_in % 16 == 0 && a.c_in <= 64 && a.c_out <= 64;
}

// Stage selection exists in the measurement build only (libpcengine_amd_measure.so, compiled with
// -DPCE_MEASURE): there a benchmark can run one kernel of a dataflow alone or pick a kernel family.  The
// product library compiles every test below to `true` and keeps no such state.
#ifdef PCE_MEASURE
static unsigned g_stage_mask = 0xFFFFFFFFu;
static inline bool stage_on(int bit) { return (g_stage_mask >> bit) & 1u; }
#else
static constexpr bool stage_on(int) { return true; }
#endif

// Output rows leave with the non-temporal hint when the tensor they belong to is larger than PCE_STREAM_MIN_BYTES:
// a tensor that size is written back from the L2s in one burst at the end of the kernel anyway, and streaming it
// out while the kernel runs hides that (150 k rows x 64 channels, 19 MB: 9.3 -> 7.0 us); a smaller one is better
// left in the L2 of the XCD that wrote it, where the next layer's tiles of the same rows find it.
#define PCE_STREAM_MIN_BYTES (16ll << 20)
static int stream_policy(long long bytes) {
  return stage_on(10) && (!stage_on(11) || bytes >= PCE_STREAM_MIN_BYTES);
}


// ---- pipelined tile GEMM for wide fp16 layers ---------------------------------------------------
// The single-offset modes (pair tiles, centre / dense GEMM) at wide channels: 128 rows x 128 columns
// per workgroup, 32 rows per wavefront.  K advances in chunks of 32; the chunk's weight tile (8 KB) is
// copied global -> LDS without passing through registers, two chunks ahead, into a ring of three
// stages; the feature fragments of the next chunk are requested before the MFMAs of the current one.
// One workgroup barrier per chunk.  (An output-stationary variant of this kernel, with 256-row tiles
// as well, was measured and lost to the single-stage tile kernel except where tile counts happened to
// fill the machine better; it is not kept.)
#define PIPE_KC 32
#define PIPE_ST 3
#define PIPE_NB 4

// The feature fragments of the pipelined kernel are requested by loads the compiler does not track:
// it would otherwise wait for every outstanding load (the ones just issued included) before the first
// use of a fragment inside the loop.  The waits are written by hand instead (pipe_wait_barrier).
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x4 load16_untracked(const void *p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}

// Every wavefront of the pipelined kernels issues, per K chunk, exactly PIPE_CHUNK_VMEM vector-memory
// operations: PIPE_ROW_LOADS untracked 16-byte loads of its own rows' fragments (pipe_load_rows) and
// PIPE_W_LOADS global -> LDS copies of its share of the weight chunk (pipe_issue_weights), both issued
// unconditionally.  Vector-memory operations complete in issue order, so "at most c * PIPE_CHUNK_VMEM
// outstanding" means "everything but the youngest c chunks has landed": the hand-written wait immediates
// are derived from these constants and nothing else.  A wavefront that issued fewer operations for some
// chunk would pass the wait early and read fragment registers before their loads have written them (an
// ablation build that dropped the weight copies did exactly that and took a memory fault).
constexpr int PIPE_ROW_LOADS = PIPE_KC / 16;   // one 16-byte load per lane covers k = 16 s2 + 8 g .. + 7 of the lane's row
constexpr int PIPE_W_LOADS = 2;                // 64 fragments of 16 bytes per instruction and wavefront
constexpr int PIPE_CHUNK_VMEM = PIPE_ROW_LOADS + PIPE_W_LOADS;
static_assert(PIPE_ROW_LOADS == 2, "pipe_wait_copy moves exactly two landed fragments");
static_assert(4 * PIPE_W_LOADS * 64 == (PIPE_KC / 8) * 128, "the copies of four wavefronts cover one 32 x 128 weight chunk exactly");
static_assert(2 * 2 * PIPE_CHUNK_VMEM <= 63, "vmcnt is a 6-bit counter");

// Waits until at most CNT vector-memory operations are outstanding, joins the workgroup barrier and only then
// reads the two fragments: the copies are made inside the same statement, after the wait, so that no read
// of a fragment register can be scheduled before its load has landed.
template <int CNT>
__device__ __forceinline__ void pipe_wait_copy(const u32x4 &f0, const u32x4 &f1, u32x4 &o0, u32x4 &o1) {
  static_assert(CNT % PIPE_CHUNK_VMEM == 0, "waits are counted in whole chunks");
  asm volatile("s_waitcnt vmcnt(%16)\n\ts_barrier\n\t"
               "v_mov_b32 %0, %8\n\tv_mov_b32 %1, %9\n\tv_mov_b32 %2, %10\n\tv_mov_b32 %3, %11\n\t"
               "v_mov_b32 %4, %12\n\tv_mov_b32 %5, %13\n\tv_mov_b32 %6, %14\n\tv_mov_b32 %7, %15"
               : "=&v"(o0.x), "=&v"(o0.y), "=&v"(o0.z), "=&v"(o0.w), "=&v"(o1.x), "=&v"(o1.y), "=&v"(o1.z), "=&v"(o1.w)
               : "v"(f0.x), "v"(f0.y), "v"(f0.z), "v"(f0.w), "v"(f1.x), "v"(f1.y), "v"(f1.z), "v"(f1.w), "n"(CNT)
               : "memory");
}
// `chunks_in_flight`: how many of the youngest chunks' operations may still be outstanding (0, 1 or 2)
__device__ __forceinline__ void pipe_wait_barrier(int chunks_in_flight, const u32x4 &f0, const u32x4 &f1, u32x4 &o0,
                                                  u32x4 &o1) {
  if (chunks_in_flight >= 2)
    pipe_wait_copy<2 * PIPE_CHUNK_VMEM>(f0, f1, o0, o1);
  else if (chunks_in_flight == 1)
    pipe_wait_copy<PIPE_CHUNK_VMEM>(f0, f1, o0, o1);
  else
    pipe_wait_copy<0>(f0, f1, o0, o1);
}
// two more fragments that the same wait has covered: volatile statements keep their order, so these copies
// stay behind the wait of the pipe_wait_barrier in front of them
__device__ __forceinline__ void pipe_copy_landed(const u32x4 &f0, const u32x4 &f1, u32x4 &o0, u32x4 &o1) {
  asm volatile("v_mov_b32 %0, %8\n\tv_mov_b32 %1, %9\n\tv_mov_b32 %2, %10\n\tv_mov_b32 %3, %11\n\t"
               "v_mov_b32 %4, %12\n\tv_mov_b32 %5, %13\n\tv_mov_b32 %6, %14\n\tv_mov_b32 %7, %15"
               : "=&v"(o0.x), "=&v"(o0.y), "=&v"(o0.z), "=&v"(o0.w), "=&v"(o1.x), "=&v"(o1.y), "=&v"(o1.z), "=&v"(o1.w)
               : "v"(f0.x), "v"(f0.y), "v"(f0.z), "v"(f0.w), "v"(f1.x), "v"(f1.y), "v"(f1.z), "v"(f1.w)
               : "memory");
}

// this wavefront's quarter of the weight chunk (k0 .. k0+31, columns n0 .. n0+127) -> LDS stage
__device__ __forceinline__ void pipe_issue_weights(const half_t *Wk, int k0, int n0, int n_pad, half8 *stage, int wave,
                                                   int lane) {
  // stage layout [k8 = 0..3][n = 0..127] of 16-byte fragments; one instruction moves 64 of them
#pragma unroll
  for (int i = 0; i < PIPE_W_LOADS; ++i) {
    int part = wave * PIPE_W_LOADS + i;          // 0..7: k8 = part / 2, column half = part % 2
    int k8 = part >> 1, nh = part & 1;
    int n = n0 + nh * 64 + lane;
    n = n < n_pad ? n : n_pad - 1;    // columns past the padded width are never stored: any valid address will do
    const half_t *src = Wk + ((long long)(k0 / 8 + k8) * n_pad + n) * 8;
    half8 *dst = stage + k8 * 128 + nh * 64;  // wave-uniform; the hardware adds lane * 16 bytes
    // issued by every wavefront in every round: pipe_wait_barrier counts on it
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                     (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
  }
}

// always issued (row 0 stands in for a missing row; the caller zeroes it when the fragment is taken into
// use): the wait before the barrier counts the loads of a round
__device__ __forceinline__ void pipe_load_rows(u32x4 (&raw)[PIPE_ROW_LOADS], const half_t *A, int arow, int lda, int k0, int g) {
  int r = arow >= 0 ? arow : 0;
#pragma unroll
  for (int s2 = 0; s2 < PIPE_ROW_LOADS; ++s2) raw[s2] = load16_untracked(A + (long long)r * lda + k0 + s2 * 16 + g * 8);
}

// PMODE = MODE_DENSE or MODE_FOD_BUF: every tile is of that kind and `c` is not read.  PMODE = PIPE_BOTH:
// the pair tiles of `a` come first, then the centre tiles of `c` (same features, weights and widths; its
// own output, epilogue and row count) -- the centre GEMM of a deferred-scatter layer is too small to fill
// the machine by itself and neither kind of tile reads what the other writes.
#define PIPE_BOTH 100
template <int PMODE>
__global__ void __launch_bounds__(256, 4) pipe_gemm_kernel(TileArgs a, TileArgs c) {
  constexpr int NB = PIPE_NB, NT = 128, KC = PIPE_KC;
  constexpr int STAGE = (KC / 8) * NT;                       // fragments per stage
  constexpr int RING = PIPE_ST * STAGE;
  constexpr int EPI = 4 * WaveLds<NB>::PIECES;               // epilogue staging reuses the ring
  __shared__ __attribute__((aligned(16))) half8 lds[RING > EPI ? RING : EPI];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  // contiguous item ranges per XCD: the column slabs of a tile, and the tiles of one offset, share an L2
  long long tile;
  int slab;
  if (!xcd_item(PMODE == PIPE_BOTH ? a.items + c.items : a.items, a.slabs, true, &tile, &slab)) return;
  const int n0 = slab * NT;
  const half_t *A = (const half_t *)a.A;
  const int kch = a.c_in / KC;
  // the argument block is never selected as a whole at run time (that would copy it to private memory)
  const long long pair_tiles = PMODE == PIPE_BOTH ? a.items / a.slabs : 0;
  const bool dense = PMODE == MODE_DENSE || (PMODE == PIPE_BOTH && tile >= pair_tiles);
  const long long n_rows = PMODE == PIPE_BOTH ? c.n_rows : a.n_rows;
  const int w_fixed = PMODE == PIPE_BOTH ? c.w_fixed : a.w_fixed;

  int orow = -1, arow = -1, widx;
  if (dense) {
    long long row = (tile - pair_tiles) * 128 + wave * 32 + l32;
    orow = arow = row < n_rows ? (int)row : -1;
    widx = w_fixed;
  } else {  // pair tile: one 128-pair quantum of one offset
    long long q0 = tile * 128;
    widx = 0;
    for (int i = 0; i < a.kv; ++i) widx += ((long long)a.qkpos_h[i + 1] <= q0) ? 1 : 0;
    if (widx >= a.kv) return;
    long long p = q0 - a.qkpos_h[widx] + a.kpos_h[widx] + wave * 32 + l32;
    if (p < (long long)a.kpos_h[widx + 1]) {
      orow = a.oslot[p];
      arow = a.imap[p];
    }
  }
  const half_t *Wk = (const half_t *)a.Wp + (long long)widx * a.k8_total * a.n_pad * 8;

  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;

  // prologue: weight chunks 0 and 1, feature chunks 0 and 1 (issue order: W0, A0, W1, A1)
  u32x4 raw[2][PIPE_ROW_LOADS];
  pipe_issue_weights(Wk, 0, n0, a.n_pad, lds, wave, lane);
  pipe_load_rows(raw[0], A, arow, a.lda, 0, g);
  if (kch > 1) {
    pipe_issue_weights(Wk, KC, n0, a.n_pad, lds + STAGE, wave, lane);
    pipe_load_rows(raw[1], A, arow, a.lda, KC, g);
  }
  const bool wave_has = __ballot(arow >= 0) != 0ull;
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  int st = 0, st2 = 2 % PIPE_ST;
  // One round: the features of chunk t were requested two rounds ago, its weights too.  Everything
  // issued before the weights of chunk t has landed once at most the loads of the previous round (the
  // features of chunk t+1, the weights of chunk t+1) are still in flight.
#define PCE_PIPE_ROUND(T_, SLOT_)                                                                          \
  {                                                                                                        \
    const int t = (T_);                                                                                    \
    u32x4 landed[2];                                                                                       \
    /* only the operations of chunk t+1 (issued one round ago) may still be outstanding */                  \
    pipe_wait_barrier(t + 1 < kch ? 1 : 0, raw[SLOT_][0], raw[SLOT_][1], landed[0], landed[1]);             \
    half8 af[2];                                                                                           \
    _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2)                                                       \
        af[s2] = arow >= 0 ? __builtin_bit_cast(half8, landed[s2]) : zero;                                 \
    /* features of chunk t+2 first, so that the weight loads below are the youngest in flight */           \
    if (t + 2 < kch) {                                                                                     \
      pipe_load_rows(raw[SLOT_], A, arow, a.lda, (t + 2) * KC, g);                                        \
      /* weight chunk t+2 -> the stage that chunk t-1 has just released */                                 \
      pipe_issue_weights(Wk, (t + 2) * KC, n0, a.n_pad, lds + st2 * STAGE, wave, lane);                    \
      st2 = st2 + 1 == PIPE_ST ? 0 : st2 + 1;                                                              \
    }                                                                                                      \
    if (wave_has) {                                                                                        \
      const half8 *stp = lds + st * STAGE;                                                                 \
      _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) _Pragma("unroll") for (int nb = 0; nb < NB; ++nb) { \
        half8 b = stp[(2 * s2 + g) * NT + nb * 32 + l32];                                                  \
        acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, af[s2], acc[nb], 0, 0, 0);                     \
      }                                                                                                    \
    }                                                                                                      \
    st = st + 1 == PIPE_ST ? 0 : st + 1;                                                                   \
  }
  for (int t0 = 0; t0 < kch; t0 += 2) {
    PCE_PIPE_ROUND(t0, 0)
    if (t0 + 1 < kch) PCE_PIPE_ROUND(t0 + 1, 1)
  }
#undef PCE_PIPE_ROUND
  __syncthreads();  // the ring becomes the epilogue staging area
  float V[NB][2][8];
  gather_row_pieces<NB>(acc, V, g);
  if (PMODE == PIPE_BOTH) {
    if (dense && (c.bias || c.res || c.act)) {
      bool with_act = c.act != PCE_ACT_NONE;
      if (with_act && c.act_alone_only) with_act = orow >= 0 && c.ocsr[orow] == c.ocsr[orow + 1];
      epilogue_row_pieces_batched<half_t, NB, true, NB>(V, c, orow, n0, g, with_act);
    }
  } else if (a.bias || a.res || a.act) {
    bool with_act = a.act != PCE_ACT_NONE;
    if (with_act && a.act_alone_only) with_act = orow >= 0 && a.ocsr[orow] == a.ocsr[orow + 1];
    int erow = orow;
    if (PMODE == MODE_FOD_BUF && a.out_alt && orow >= a.n_split) {  // a partial row: its epilogue comes with the row sum
      erow = -1;
      with_act = false;
    }
    epilogue_row_pieces_batched<half_t, NB, true, NB>(V, a, erow, n0, g, with_act);
  }
  half_t *out = (half_t *)((PMODE == PIPE_BOTH && dense) ? c.out : a.out);
  if (PMODE == MODE_FOD_BUF && a.out_alt)
    store_rows_via_lds<half_t, NB, 32, true>(V, lds + wave * WaveLds<NB>::PIECES, out, orow, a, n0, lane, l32, g, a.stream);
  else
    store_rows_via_lds<half_t, NB>(V, lds + wave * WaveLds<NB>::PIECES, out, orow, a, n0, lane, l32, g,
                                   (PMODE == PIPE_BOTH && dense) ? c.stream : a.stream,
                                   (PMODE == PIPE_BOTH && dense) ? c.ldo : a.ldo);
}

// The eight weight fragments of a step are requested before its first MFMA, and every MFMA waits only for
// its own fragment (LDS reads return in order).  Left to the compiler the reads are issued two at a time,
// each pair in front of the MFMAs that use it, which leaves the LDS latency exposed four times per step
// when few wavefronts share a SIMD.
__device__ __forceinline__ void step_mfma(f32x16 (&acc)[4], const half8 (&af)[2], const half8 *frag0) {
  unsigned addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)frag0;
  u32x4 b0, b1, b2, b3, b4, b5, b6, b7;
  asm volatile(
      "ds_read_b128 %0, %14\n\t"
      "ds_read_b128 %1, %14 offset:512\n\t"
      "ds_read_b128 %2, %14 offset:1024\n\t"
      "ds_read_b128 %3, %14 offset:1536\n\t"
      "ds_read_b128 %4, %14 offset:4096\n\t"
      "ds_read_b128 %5, %14 offset:4608\n\t"
      "ds_read_b128 %6, %14 offset:5120\n\t"
      "ds_read_b128 %7, %14 offset:5632\n\t"
      "s_waitcnt lgkmcnt(7)\n\tv_mfma_f32_32x32x16_f16 %8, %0, %12, %8\n\t"
      "s_waitcnt lgkmcnt(6)\n\tv_mfma_f32_32x32x16_f16 %9, %1, %12, %9\n\t"
      "s_waitcnt lgkmcnt(5)\n\tv_mfma_f32_32x32x16_f16 %10, %2, %12, %10\n\t"
      "s_waitcnt lgkmcnt(4)\n\tv_mfma_f32_32x32x16_f16 %11, %3, %12, %11\n\t"
      "s_waitcnt lgkmcnt(3)\n\tv_mfma_f32_32x32x16_f16 %8, %4, %13, %8\n\t"
      "s_waitcnt lgkmcnt(2)\n\tv_mfma_f32_32x32x16_f16 %9, %5, %13, %9\n\t"
      "s_waitcnt lgkmcnt(1)\n\tv_mfma_f32_32x32x16_f16 %10, %6, %13, %10\n\t"
      "s_waitcnt lgkmcnt(0)\n\tv_mfma_f32_32x32x16_f16 %11, %7, %13, %11"
      : "=&v"(b0), "=&v"(b1), "=&v"(b2), "=&v"(b3), "=&v"(b4), "=&v"(b5), "=&v"(b6), "=&v"(b7), "+v"(acc[0]),
        "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])
      : "v"(af[0]), "v"(af[1]), "v"(addr)
      : "memory");
}

// ---- pipelined output-stationary kernel for wide fp16 layers ----------------------------------------
// The single-stage tile kernel requests the weight chunk and the gathered rows of a (offset, K chunk) step
// right before it needs them; a layer of a few hundred tiles is one round of workgroups with nothing
// else resident to hide that latency (1.6 us per step against 0.2 us of MFMA work on 26 k rows x 256
// channels).  Here the steps of a tile -- its populated offsets times the K chunks -- form one sequence
// that runs through the ring of pipe_gemm_kernel: weights global -> LDS and feature fragments by
// untracked loads, both two steps ahead, one barrier per step.  The neighbour rows of all offsets are
// read once into LDS; an offset none of the tile's rows has a neighbour at is left out of the sequence,
// and a wavefront skips the MFMAs of an offset none of its own 32 rows has.
// SUB K chunks share a step (one wait, one barrier, 8 SUB MFMAs per wavefront): with one or two workgroups
// per CU the barrier, the wait and the LDS latency in front of a step's first MFMA cost more than its
// MFMAs, so input widths that are multiples of 64 take two chunks per step.
#define OSP_MAX_KV 32
template <int SUB>
__global__ void __launch_bounds__(256, SUB == 1 ? 3 : 2) os_pipe_kernel(TileArgs a) {
  constexpr int NB = PIPE_NB, NT = 128, KC = PIPE_KC;
  constexpr int STAGE = (KC / 8) * NT;          // fragments of one chunk
  constexpr int RSTAGE = SUB * STAGE;           // fragments of one ring stage
  constexpr int RING = PIPE_ST * RSTAGE;
  constexpr int EPI = 4 * WaveLds<NB>::PIECES;
  __shared__ __attribute__((aligned(16))) half8 lds[RING > EPI ? RING : EPI];
  __shared__ int nbrs[OSP_MAX_KV][128];
  __shared__ unsigned wave_masks[4];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  long long tile;
  int slab;
  if (!xcd_item(a.items, a.slabs, true, &tile, &slab)) return;
  const int n0 = slab * NT;
  const half_t *A = (const half_t *)a.A;
  const int kch = a.c_in / (KC * SUB);   // steps per offset
  const long long row = tile * 128 + wave * 32 + l32;
  const int orow = row < a.n_rows ? (int)row : -1;

  // neighbour rows of every offset -> LDS; offsets this wavefront / this tile has any neighbour at
  unsigned wmask = 0;
  for (int kp = 0; kp < a.kv; ++kp) {
    int nb_row = orow >= 0 ? a.nbr[(long long)kp * a.n_rows + orow] : -1;
    if (g == 0) nbrs[kp][wave * 32 + l32] = nb_row;
    if (__ballot(nb_row >= 0) != 0ull) wmask |= 1u << kp;
  }
  if (lane == 0) wave_masks[wave] = wmask;
  __syncthreads();
  const unsigned active = wave_masks[0] | wave_masks[1] | wave_masks[2] | wave_masks[3];
  const int rounds = __popc(active) * kch;

  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;

  // issue cursor (two steps ahead of the consume cursor): offset, chunk, LDS stage
  int ikp = active ? __ffs(active) - 1 : -1, it = 0, ist = 0;
  int ckp = ikp, ct = 0, cst = 0;
  u32x4 raw[2][SUB][PIPE_ROW_LOADS];
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  int carow[2] = {-1, -1};   // the row whose fragments sit in raw[slot]
#define OSP_ISSUE(SLOT_)                                                                                     \
  {                                                                                                          \
    const half_t *Wk = (const half_t *)a.Wp + (long long)ikp * a.k8_total * a.n_pad * 8;                     \
    const int arow_i = nbrs[ikp][wave * 32 + l32];                                                           \
    carow[SLOT_] = arow_i;                                                                                   \
    _Pragma("unroll") for (int sub = 0; sub < SUB; ++sub) {                                                  \
      pipe_load_rows(raw[SLOT_][sub], A, arow_i, a.lda, (it * SUB + sub) * KC, g);                          \
      pipe_issue_weights(Wk, (it * SUB + sub) * KC, n0, a.n_pad, lds + ist * RSTAGE + sub * STAGE, wave, lane); \
    }                                                                                                        \
    ist = ist + 1 == PIPE_ST ? 0 : ist + 1;                                                                  \
    if (++it == kch) {                                                                                       \
      it = 0;                                                                                                \
      unsigned rest = ikp >= 31 ? 0u : (active & ~((2u << ikp) - 1u));                                       \
      ikp = rest ? __ffs(rest) - 1 : -1;                                                                     \
    }                                                                                                        \
  }
  // issue order per step: feature fragments, then weights; the prologue issues steps 0 and 1
  if (rounds > 0) OSP_ISSUE(0)
  if (rounds > 1) OSP_ISSUE(1)
#define OSP_ROUND(R_, SLOT_)                                                                                 \
  {                                                                                                          \
    const int r = (R_);                                                                                      \
    u32x4 landed[SUB][2];                                                                                    \
    /* everything older than the SUB chunks of step r+1 (issued one step ago) has landed */                 \
    pipe_wait_barrier(r + 1 < rounds ? SUB : 0, raw[SLOT_][0][0], raw[SLOT_][0][1], landed[0][0], landed[0][1]); \
    if (SUB == 2) pipe_copy_landed(raw[SLOT_][SUB - 1][0], raw[SLOT_][SUB - 1][1], landed[SUB - 1][0], landed[SUB - 1][1]); \
    half8 af[SUB][2];                                                                                        \
    const int arow_c = carow[SLOT_];                                                                         \
    _Pragma("unroll") for (int sub = 0; sub < SUB; ++sub) _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2)   \
        af[sub][s2] = arow_c >= 0 ? __builtin_bit_cast(half8, landed[sub][s2]) : zero;                       \
    if (r + 2 < rounds) OSP_ISSUE(SLOT_)                                                                     \
    if ((wmask >> ckp) & 1u) {                                                                               \
      _Pragma("unroll") for (int sub = 0; sub < SUB; ++sub)                                                  \
          step_mfma(acc, af[sub], lds + cst * RSTAGE + sub * STAGE + g * NT + l32);                          \
    }                                                                                                        \
    cst = cst + 1 == PIPE_ST ? 0 : cst + 1;                                                                  \
    if (++ct == kch) {                                                                                       \
      ct = 0;                                                                                                \
      unsigned rest = ckp >= 31 ? 0u : (active & ~((2u << ckp) - 1u));                                       \
      ckp = rest ? __ffs(rest) - 1 : 0;                                                                      \
    }                                                                                                        \
  }
  for (int r0 = 0; r0 < rounds; r0 += 2) {
    OSP_ROUND(r0, 0)
    if (r0 + 1 < rounds) OSP_ROUND(r0 + 1, 1)
  }
#undef OSP_ROUND
#undef OSP_ISSUE
  __syncthreads();  // the ring becomes the epilogue staging area
  float V[NB][2][8];
  gather_row_pieces<NB>(acc, V, g);
  if (a.bias || a.res || a.act) epilogue_row_pieces_batched<half_t, NB, true, NB>(V, a, orow, n0, g, a.act != PCE_ACT_NONE);
  store_rows_via_lds<half_t, NB>(V, lds + wave * WaveLds<NB>::PIECES, (half_t *)a.out, orow, a, n0, lane, l32, g, a.stream);
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// shapes the pipelined kernel takes
static bool pipe_gemm_ok(const TileArgs &a, int elem_size) {
  return elem_size == 2 && a.Wp && a.a_vec && a.o_vec && a.c_in % PIPE_KC == 0 && a.c_in >= 64 && a.c_out >= 96 &&
         aligned16(a.bias) && aligned16(a.res) && a.epi == EPI_ROWS &&
         (a.mode == MODE_DENSE || (a.mode == MODE_FOD_BUF && a.host_pos));
}

static int launch_pipe_gemm(TileArgs a, long long tiles, hipStream_t s) {
  a.slabs = (a.c_out + 127) / 128;
  a.items = tiles * a.slabs;
  if (a.items >= (1ll << 31) - 8) PCE_FAIL(PCE_ECAPACITY, "tile count %lld exceeds the grid limit", tiles);
  const unsigned grid = (unsigned)(pce_div_up(a.items, PCE_XCDS) * PCE_XCDS);
  if (a.mode == MODE_DENSE)
    hipLaunchKernelGGL((pipe_gemm_kernel<MODE_DENSE>), dim3(grid), dim3(256), 0, s, a, a);
  else
    hipLaunchKernelGGL((pipe_gemm_kernel<MODE_FOD_BUF>), dim3(grid), dim3(256), 0, s, a, a);
  PCE_LAUNCH_CHECK("pipe_gemm");
  return PCE_OK;
}

// pair tiles (a: MODE_FOD_BUF) and centre tiles (c: MODE_DENSE) of one layer in one launch
static int launch_pipe_both(TileArgs a, long long pair_tiles, TileArgs c, long long centre_tiles, hipStream_t s) {
  a.slabs = c.slabs = (a.c_out + 127) / 128;
  a.items = pair_tiles * a.slabs;
  c.items = centre_tiles * c.slabs;
  const long long items = a.items + c.items;
  if (items <= 0) return PCE_OK;
  if (items >= (1ll << 31) - 8) PCE_FAIL(PCE_ECAPACITY, "tile count %lld exceeds the grid limit", items);
  const unsigned grid = (unsigned)(pce_div_up(items, PCE_XCDS) * PCE_XCDS);
  hipLaunchKernelGGL((pipe_gemm_kernel<PIPE_BOTH>), dim3(grid), dim3(256), 0, s, a, c);
  PCE_LAUNCH_CHECK("pipe_gemm");
  return PCE_OK;
}

// shapes the pipelined output-stationary kernel takes
static bool os_pipe_ok(const TileArgs &a, int elem_size) {
  return elem_size == 2 && a.mode == MODE_OS && a.epi == EPI_ROWS && a.Wp && a.a_vec && a.o_vec && a.c_in % PIPE_KC == 0 &&
         a.c_in >= 64 && a.c_out >= 96 && a.kv <= OSP_MAX_KV && aligned16(a.bias) && aligned16(a.res);
}

static int launch_os_pipe(TileArgs a, long long tiles, hipStream_t s) {
  a.slabs = (a.c_out + 127) / 128;
  a.items = tiles * a.slabs;
  if (a.items >= (1ll << 31) - 8) PCE_FAIL(PCE_ECAPACITY, "tile count %lld exceeds the grid limit", tiles);
  const unsigned grid = (unsigned)(pce_div_up(a.items, PCE_XCDS) * PCE_XCDS);
  if (a.c_in % (2 * PIPE_KC) == 0)
    hipLaunchKernelGGL(os_pipe_kernel<2>, dim3(grid), dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL(os_pipe_kernel<1>, dim3(grid), dim3(256), 0, s, a);
  PCE_LAUNCH_CHECK("os_pipe");
  return PCE_OK;
}

static unsigned xcd_grid(TileArgs *a, long long tiles, int slabs) {
  a->slabs = slabs;
  a->items = tiles * slabs;
  return (unsigned)(pce_div_up(a->items, PCE_XCDS) * PCE_XCDS);
}

template <typename T, bool FAST, int TMODE, int TEPI>
static void launch_tile_nb(TileArgs a, long long tiles, hipStream_t s) {
  int nb = (a.c_out + 31) / 32;
  if (nb >= 4) {
    unsigned grid = xcd_grid(&a, tiles, (a.c_out + 127) / 128);
    hipLaunchKernelGGL((tile_gemm_kernel<T, 4, FAST, TMODE, TEPI>), dim3(grid), dim3(256), 0, s, a);
  } else if (nb == 3) {
    unsigned grid = xcd_grid(&a, tiles, 1);
    hipLaunchKernelGGL((tile_gemm_kernel<T, 3, FAST, TMODE, TEPI>), dim3(grid), dim3(256), 0, s, a);
  } else if (nb == 2) {
    unsigned grid = xcd_grid(&a, tiles, 1);
    hipLaunchKernelGGL((tile_gemm_kernel<T, 2, FAST, TMODE, TEPI>), dim3(grid), dim3(256), 0, s, a);
  } else {
    unsigned grid = xcd_grid(&a, tiles, 1);
    hipLaunchKernelGGL((tile_gemm_kernel<T, 1, FAST, TMODE, TEPI>), dim3(grid), dim3(256), 0, s, a);
  }
}

template <typename T>
static int launch_tile(const TileArgs &a, long long tiles, hipStream_t s) {
  if (tiles <= 0) return PCE_OK;
  if (tiles * ((a.c_out + 127) / 128) >= (1ll << 31) - 8) PCE_FAIL(PCE_ECAPACITY, "tile count %lld exceeds the grid limit", tiles);
  // plain GEMMs of 96 columns and at most 128 input channels stay with the tile kernel below: 12.1 vs 13.8 us on
  // 100 k rows (128 -> 96), 75 vs 80 and 87 vs 94 us on 950 k rows (96 -> 96, 128 -> 96); from 128 columns the pipelined
  // kernel leads
  const bool small_dense = a.mode == MODE_DENSE && a.epi == EPI_ROWS && a.n_pad <= 96 && a.c_in <= 128;
  if (stage_on(5) && pipe_gemm_ok(a, sizeof(T)) && !small_dense)
    return launch_pipe_gemm(a, tiles, s);
  // measured: 154 instead of 177 us and 88 instead of 96 us on 406 (tile, slab) items (26 k rows, 256 output
  // channels), 66 instead of 62 us and 113 instead of 111 us on 515 (66 k rows, 128 output channels)
  if (stage_on(9) && os_pipe_ok(a, sizeof(T)) && tiles * ((a.c_out + 127) / 128) <= 448) return launch_os_pipe(a, tiles, s);
  bool fast = a.a_vec && a.o_vec && (sizeof(T) == 2 ? a.Wp != nullptr : a.w_vec != 0) &&
              (a.epi != EPI_ROWS_CSR || a.b_vec) && aligned16(a.bias) && aligned16(a.res);
  if (!fast)
    launch_tile_nb<T, false, -1, -1>(a, tiles, s);
  else if (a.mode == MODE_DENSE && a.epi == EPI_ROWS_CSR)
    launch_tile_nb<T, true, MODE_DENSE, EPI_ROWS_CSR>(a, tiles, s);
  else if (a.mode == MODE_DENSE && a.epi == EPI_ROWS)
    launch_tile_nb<T, true, MODE_DENSE, EPI_ROWS>(a, tiles, s);
  else if (a.mode == MODE_FOD_BUF && a.epi == EPI_ROWS)
    launch_tile_nb<T, true, MODE_FOD_BUF, EPI_ROWS>(a, tiles, s);
  else if (a.mode == MODE_OS && a.epi == EPI_ROWS)
    launch_tile_nb<T, true, MODE_OS, EPI_ROWS>(a, tiles, s);
  else if (a.mode == MODE_FOD && a.epi == EPI_ATOMIC_F32)
    launch_tile_nb<T, true, MODE_FOD, EPI_ATOMIC_F32>(a, tiles, s);
  else if (a.mode == MODE_BUF && a.epi == EPI_ROWS)
    launch_tile_nb<T, true, MODE_BUF, EPI_ROWS>(a, tiles, s);
  else if (a.mode == MODE_DENSE && a.epi == EPI_ROWS_F32)
    launch_tile_nb<T, true, MODE_DENSE, EPI_ROWS_F32>(a, tiles, s);
  else
    launch_tile_nb<T, true, -1, -1>(a, tiles, s);
  PCE_LAUNCH_CHECK("tile_gemm");
  return PCE_OK;
}

// ---- streaming kernels of the gather-GEMM-scatter dataflow -------------------------------------
// V = 16-byte vector when rows are 16-byte multiples and aligned, else one element.
// G lanes cooperate on one row; a row's vector v is handled by lane v mod G.
template <typename V>
__global__ void __launch_bounds__(256) gather_rows_kernel(const V *__restrict__ in, long long n_in, int row_vecs, int G,
                                                          const int *__restrict__ icsr, const int *__restrict__ icode,
                                                          const int *__restrict__ qkpos, V *__restrict__ buf) {
  int rows_per_block = 256 / G;
  long long row = (long long)blockIdx.x * rows_per_block + threadIdx.x / G;
  int sub = threadIdx.x % G;
  if (row >= n_in) return;
  int e0 = icsr[row], e1 = icsr[row + 1];
  if (e0 == e1) return;
  for (int v = sub; v < row_vecs; v += G) {
    V x = in[row * row_vecs + v];
    for (int e = e0; e < e1; ++e) {
      int code = icode[e];
      long long q = (long long)qkpos[code / PCE_CSR_CODE] + code % PCE_CSR_CODE;
      buf[q * row_vecs + v] = x;
    }
  }
}

template <typename T, int VEC>
struct VecOf;
template <>
struct VecOf<half_t, 8> { typedef half8 type; };
template <>
struct VecOf<float, 4> { typedef f32x4 type; };
template <>
struct VecOf<half_t, 1> { typedef half_t type; };
template <>
struct VecOf<float, 1> { typedef float type; };

template <typename T, int VEC>
__global__ void __launch_bounds__(256) scatter_rows_kernel(const T *__restrict__ buf, long long n_out, int c_out, int G,
                                                           const int *__restrict__ ocsr, const int *__restrict__ ocode,
                                                           const int *__restrict__ qkpos, T *__restrict__ out,
                                                           int add_existing, const T *__restrict__ bias,
                                                           const T *__restrict__ res, int act, float slope) {
  typedef typename VecOf<T, VEC>::type V;
  int rows_per_block = 256 / G;
  long long row = (long long)blockIdx.x * rows_per_block + threadIdx.x / G;
  int sub = threadIdx.x % G;
  if (row >= n_out) return;
  int e0 = ocsr[row], e1 = ocsr[row + 1];
  // a row without staging rows keeps its centre term as it is, unless an epilogue has to touch it
  if (add_existing && e0 == e1 && !bias && !res && act == PCE_ACT_NONE) return;
  int row_vecs = c_out / VEC;
  for (int v = sub; v < row_vecs; v += G) {
    float acc[VEC];
    if (add_existing) {
      V x = *reinterpret_cast<const V *>(&out[row * c_out + (long long)v * VEC]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = (float)(reinterpret_cast<const T *>(&x)[j]);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
    }
    for (int e = e0; e < e1; ++e) {
      int code = ocode[e];
      long long q = (long long)qkpos[code / PCE_CSR_CODE] + code % PCE_CSR_CODE;
      V x = *reinterpret_cast<const V *>(&buf[q * c_out + (long long)v * VEC]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&x)[j]);
    }
    V y;
    if (bias) {
      V b = *reinterpret_cast<const V *>(&bias[(long long)v * VEC]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&b)[j]);
    }
    if (res) {
      V r = *reinterpret_cast<const V *>(&res[row * c_out + (long long)v * VEC]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&r)[j]);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) reinterpret_cast<T *>(&y)[j] = (T)act_apply(acc[j], act, slope);
    *reinterpret_cast<V *>(&out[row * c_out + (long long)v * VEC]) = y;
  }
}

// out[row] = sum of the contiguous partial rows buf[csr[row] .. csr[row+1]), fp32 accumulate.  With `rows` the
// kernel visits rows[0 .. *count) instead of every row (count read on the device, the grid is sized by the host
// for the list's capacity and strides over it).
template <typename T, int VEC>
__global__ void __launch_bounds__(256) rowsum_kernel(const T *__restrict__ buf, long long n_out, int c_out, int G,
                                                     const int *__restrict__ csr, T *__restrict__ out,
                                                     const T *__restrict__ bias, const T *__restrict__ res, int act,
                                                     float slope, const int *__restrict__ rows,
                                                     const int *__restrict__ count, int stream, int ldo) {
  typedef typename VecOf<T, VEC>::type V;
  int rows_per_block = 256 / G;
  int sub = threadIdx.x % G;
  const long long n_items = rows ? (long long)*count : n_out;
  for (long long item = (long long)blockIdx.x * rows_per_block + threadIdx.x / G; item < n_items;
       item += (long long)gridDim.x * rows_per_block) {
    long long row = rows ? (long long)rows[item] : item;
    int e0 = csr[row], e1 = csr[row + 1];
    int row_vecs = c_out / VEC;
    for (int v = sub; v < row_vecs; v += G) {
      float acc[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
      const T *bp = buf + (long long)v * VEC;
      int e = e0;
      for (; e + 4 <= e1; e += 4) {  // four partial rows in flight
        V x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const V *>(bp + (long long)(e + u) * c_out);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&x[u])[j]);
      }
      for (; e < e1; ++e) {
        V x = *reinterpret_cast<const V *>(bp + (long long)e * c_out);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&x)[j]);
      }
      V y;
      if (bias) {
        V b = *reinterpret_cast<const V *>(&bias[(long long)v * VEC]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&b)[j]);
      }
      if (res) {
        V r = *reinterpret_cast<const V *>(&res[row * c_out + (long long)v * VEC]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&r)[j]);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) reinterpret_cast<T *>(&y)[j] = (T)act_apply(acc[j], act, slope);
      store_maybe_stream(reinterpret_cast<V *>(&out[row * ldo + (long long)v * VEC]), y, stream != 0);
    }
  }
}

// in-place epilogue for the dataflows whose last kernel cannot take it: out = act(out + bias + res)
template <typename T, int VEC>
__global__ void __launch_bounds__(256) epilogue_rows_kernel(T *__restrict__ out, long long n_out, int c_out,
                                                            const T *__restrict__ bias, const T *__restrict__ res,
                                                            int act, float slope) {
  typedef typename VecOf<T, VEC>::type V;
  int row_vecs = c_out / VEC;
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_out * row_vecs) return;
  long long row = i / row_vecs;
  int v = (int)(i - row * row_vecs);
  V x = *reinterpret_cast<const V *>(&out[row * c_out + (long long)v * VEC]);
  float acc[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) acc[j] = (float)(reinterpret_cast<const T *>(&x)[j]);
  if (bias) {
    V b = *reinterpret_cast<const V *>(&bias[(long long)v * VEC]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&b)[j]);
  }
  if (res) {
    V r = *reinterpret_cast<const V *>(&res[row * c_out + (long long)v * VEC]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&r)[j]);
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) reinterpret_cast<T *>(&x)[j] = (T)act_apply(acc[j], act, slope);
  *reinterpret_cast<V *>(&out[row * c_out + (long long)v * VEC]) = x;
}

// out[o] = act(out[o] + sum of the partial rows of o) for the rows that have any.  BY_ROW = false: one
// group of G lanes per pair, and the pair whose partial row is the first of its output row does the
// whole row (few pairs per row: most rows are never visited).  BY_ROW = true: one group per output row
// (more pairs than rows).  Partial rows are requested four at a time.
template <typename T, int VEC, bool BY_ROW>
__global__ void __launch_bounds__(256) rowsum_pairs_kernel(const T *__restrict__ buf, long long n_items, int c_out, int G,
                                                           const int *__restrict__ omap, const int *__restrict__ oslot,
                                                           const int *__restrict__ csr, T *__restrict__ out, int act,
                                                           float slope, int stream, int ldo) {
  typedef typename VecOf<T, VEC>::type V;
  long long item = (long long)blockIdx.x * (256 / G) + threadIdx.x / G;
  int sub = threadIdx.x % G;
  if (item >= n_items) return;
  int row, e0, e1;
  if (BY_ROW) {
    row = (int)item;
    e0 = csr[row];
    e1 = csr[row + 1];
    if (e0 >= e1) return;
  } else {
    row = omap[item];
    e0 = csr[row];
    if (oslot[item] != e0) return;
    e1 = csr[row + 1];
  }
  int row_vecs = c_out / VEC;
  for (int v = sub; v < row_vecs; v += G) {
    const T *bp = buf + (long long)v * VEC;
    V x = *reinterpret_cast<const V *>(&out[(long long)row * ldo + (long long)v * VEC]);
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = (float)(reinterpret_cast<const T *>(&x)[j]);
    int e = e0;
    for (; e + 4 <= e1; e += 4) {
      V y[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) y[u] = *reinterpret_cast<const V *>(bp + (long long)(e + u) * c_out);
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&y[u])[j]);
    }
    for (; e < e1; ++e) {
      V y = *reinterpret_cast<const V *>(bp + (long long)e * c_out);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += (float)(reinterpret_cast<const T *>(&y)[j]);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) reinterpret_cast<T *>(&x)[j] = (T)act_apply(acc[j], act, slope);
    store_maybe_stream(reinterpret_cast<V *>(&out[(long long)row * ldo + (long long)v * VEC]), x, stream != 0);
  }
}

// picks the vector width and the iteration space of the row sum
template <typename T>
static int launch_rowsum_pairs(const T *buffer, T *out, int64_t n_out, int64_t n_pairs, int c_out, const int *omap,
                               const int *oslot, const int *ocsr, int act, float slope, hipStream_t s, int ldo = 0) {
  if (ldo <= 0) ldo = c_out;
  if (n_pairs <= 0) return PCE_OK;
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  const bool vec = (c_out % VEC == 0) && (((uintptr_t)out | (uintptr_t)buffer) & 15) == 0;
  int G = 1;
  while (G < (vec ? c_out / VEC : c_out)) G <<= 1;
  if (G > 64) G = 64;
  const bool by_row = n_pairs > n_out;
  const long long items = by_row ? n_out : n_pairs;
  dim3 grid((unsigned)pce_div_up(items, 256 / G)), block(256);
#define PCE_ROWSUM(V_, B_)                                                                                        \
  hipLaunchKernelGGL((rowsum_pairs_kernel<T, V_, B_>), grid, block, 0, s, buffer, items, c_out, G, omap, oslot, ocsr, out, \
                     act, slope, stream_policy((long long)n_out * c_out * (long long)sizeof(T)), ldo)
  if (vec && by_row)
    PCE_ROWSUM(VEC, true);
  else if (vec)
    PCE_ROWSUM(VEC, false);
  else if (by_row)
    PCE_ROWSUM(1, true);
  else
    PCE_ROWSUM(1, false);
#undef PCE_ROWSUM
  PCE_LAUNCH_CHECK("rowsum_pairs");
  return PCE_OK;
}


__global__ void __launch_bounds__(256) convert_f32_f16_kernel(const float *__restrict__ in, half_t *__restrict__ out,
                                                              long long n) {
  long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i + 8 <= n) {
    f32x4 a = *reinterpret_cast<const f32x4 *>(in + i);
    f32x4 b = *reinterpret_cast<const f32x4 *>(in + i + 4);
    half8 h;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      h[j] = (half_t)a[j];
      h[4 + j] = (half_t)b[j];
    }
    *reinterpret_cast<half8 *>(out + i) = h;
  } else {
    for (; i < n; ++i) out[i] = (half_t)in[i];
  }
}

__global__ void zero_f32_kernel(float *p, long long n) {
  long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i + 4 <= n) {
    f32x4 z = {0.f, 0.f, 0.f, 0.f};
    *reinterpret_cast<f32x4 *>(p + i) = z;
  } else {
    for (; i < n; ++i) p[i] = 0.f;
  }
}

#ifdef PCE_MEASURE
extern "C" void pce_set_stage_mask(uint32_t mask) { g_stage_mask = mask; }
#endif

static int pow2_at_least(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}


static int check_common(const char *fn, const void *in, const void *w, const void *out, int dtype, int64_t n_in,
                        int64_t n_out, int c_in, int c_out, int kv, int mid) {
  if (!in || !w || !out) PCE_FAIL(PCE_EINVAL, "%s: null feature / weight pointer", fn);
  if (dtype != PCE_F16 && dtype != PCE_F32) PCE_FAIL(PCE_EINVAL, "%s: dtype must be PCE_F16 or PCE_F32", fn);
  if (n_in <= 0 || n_out <= 0 || c_in <= 0 || c_out <= 0 || kv <= 0)
    PCE_FAIL(PCE_EINVAL, "%s: sizes must be positive (n_in=%lld n_out=%lld c_in=%d c_out=%d kv=%d)", fn, (long long)n_in, (long long)n_out, c_in, c_out, kv);
  if (n_in >= (1ll << 31) || n_out >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "%s: row count exceeds int32", fn);
  if (mid >= kv) PCE_FAIL(PCE_EINVAL, "%s: mid=%d >= kv=%d", fn, mid, kv);
  if (mid >= 0 && n_in != n_out) PCE_FAIL(PCE_EINVAL, "%s: a centre offset needs n_in == n_out", fn);
  return PCE_OK;
}

static int check_qsum(const char *fn, int64_t qsum) {
  if (qsum < 0 || qsum % PCE_QUANTUM) PCE_FAIL(PCE_EINVAL, "%s: qsum=%lld is not a multiple of %d", fn, (long long)qsum, PCE_QUANTUM);
  if (qsum >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "%s: staging rows exceed int32", fn);
  return PCE_OK;
}

// features / weights / packed weights / sizes common to every launch of one layer
template <typename T>
static TileArgs base_args(const void *in, const void *w, const void *wp, int kv, int c_in, int c_out, int lda = 0) {
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  TileArgs a = {};
  a.A = in;
  a.W = w;
  a.Wp = sizeof(T) == 2 ? wp : nullptr;
  a.kv = kv;
  a.c_in = c_in;
  a.c_out = c_out;
  a.lda = lda > 0 ? lda : c_in;
  a.ldo = c_out;
  a.k8_total = (c_in + 7) / 8;
  a.n_pad = (c_out + 31) / 32 * 32;
  a.a_vec = (c_in % VEC == 0) && aligned16(in);
  a.w_vec = (c_out % VEC == 0) && aligned16(w);
  return a;
}

// `rows` = rows of the tensor `out` points to (0: not known, no streaming)
template <typename T>
static void set_out(TileArgs *a, void *out, bool f32out, long long rows = 0, int ldo = 0) {
  // a lane of the row epilogue owns 8 consecutive columns, whatever the element type
  a->out = out;
  a->ldo = ldo > 0 ? ldo : a->c_out;
  a->o_vec = (a->c_out % 8 == 0) && aligned16(out);
  a->stream = rows > 0 ? stream_policy(rows * a->c_out * (f32out ? 4 : (long long)sizeof(T))) : 0;
}

static void set_host_pos(TileArgs *a, const int32_t *kpos_host, const int32_t *qkpos_host) {
  a->host_pos = 0;
  if (kpos_host && qkpos_host && a->kv <= MAX_KV_ARGS) {
    a->host_pos = 1;
    for (int i = 0; i <= a->kv; ++i) {
      a->kpos_h[i] = kpos_host[i];
      a->qkpos_h[i] = qkpos_host[i];
    }
  }
}

struct Epi {
  const void *bias, *res;
  int act;
  float slope;
  int lda, ldo;   // row strides of the input and output matrices in elements, 0 = dense
  bool any() const { return bias || res || act != PCE_ACT_NONE; }
};

static int read_epilogue(const char *fn, const pce_epilogue_t *e, const void *out, Epi *o, int c_in = 0, int c_out = 0) {
  o->bias = o->res = nullptr;
  o->act = PCE_ACT_NONE;
  o->slope = 0.f;
  o->lda = o->ldo = 0;
  if (!e) return PCE_OK;
  // row strides: only the entry points that pass their channel counts take them
  if ((e->ld_in != 0 && e->ld_in != c_in) || (e->ld_out != 0 && e->ld_out != c_out)) {
    if (c_in <= 0) PCE_FAIL(PCE_EINVAL, "%s: this entry point takes dense feature matrices only (ld_in=%lld, ld_out=%lld)", fn, (long long)e->ld_in, (long long)e->ld_out);
    if ((e->ld_in != 0 && (e->ld_in < c_in || e->ld_in % 8)) || (e->ld_out != 0 && (e->ld_out < c_out || e->ld_out % 8)) ||
        e->ld_in >= (1ll << 31) || e->ld_out >= (1ll << 31))
      PCE_FAIL(PCE_EINVAL, "%s: row strides (ld_in=%lld, ld_out=%lld) must be multiples of 8 elements, at least the channel counts (%d, %d)", fn, (long long)e->ld_in, (long long)e->ld_out, c_in, c_out);
    o->lda = (int)e->ld_in;
    o->ldo = (int)e->ld_out;
  }
  if (e->act != PCE_ACT_NONE && e->act != PCE_ACT_RELU && e->act != PCE_ACT_LEAKY_RELU)
    PCE_FAIL(PCE_EINVAL, "%s: unknown activation %d", fn, (int)e->act);
  if (e->residual && e->residual == out) PCE_FAIL(PCE_EINVAL, "%s: the residual must not alias the output", fn);
  o->bias = e->bias;
  o->res = e->residual;
  o->act = e->act;
  o->slope = e->slope;
  return PCE_OK;
}

static void set_epi(TileArgs *a, const Epi &e) {
  a->bias = e.bias;
  a->res = e.res;
  a->act = e.act;
  a->slope = e.slope;
}

static bool epi_aligned(const Epi &e) { return aligned16(e.bias) && aligned16(e.res); }

// one in-place pass: out = act(out + bias + res)
template <typename T>
static int launch_epilogue_pass(T *out, int64_t n_out, int c_out, const Epi &e, hipStream_t s) {
  if (!e.any()) return PCE_OK;
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  if (c_out % VEC == 0 && aligned16(out) && epi_aligned(e)) {
    long long total = (long long)n_out * (c_out / VEC);
    hipLaunchKernelGGL((epilogue_rows_kernel<T, VEC>), dim3((unsigned)pce_div_up(total, 256)), dim3(256), 0, s, out,
                       (long long)n_out, c_out, (const T *)e.bias, (const T *)e.res, e.act, e.slope);
  } else {
    long long total = (long long)n_out * c_out;
    hipLaunchKernelGGL((epilogue_rows_kernel<T, 1>), dim3((unsigned)pce_div_up(total, 256)), dim3(256), 0, s, out,
                       (long long)n_out, c_out, (const T *)e.bias, (const T *)e.res, e.act, e.slope);
  }
  PCE_LAUNCH_CHECK("epilogue_rows");
  return PCE_OK;
}

extern "C" int64_t pce_packed_weight_bytes(int32_t dtype, int32_t kv, int32_t c_in, int32_t c_out) {
  if (dtype != PCE_F16) return 0;
  return (int64_t)kv * ((c_in + 7) / 8) * ((c_out + 31) / 32 * 32) * 16;
}

extern "C" int pce_pack_weights(const void *w, int32_t dtype, int32_t kv, int32_t c_in, int32_t c_out, void *packed,
                                pce_stream_t stream) {
  if (dtype != PCE_F16) return PCE_OK;  // fp32 weights are used as they are
  if (!w || !packed) PCE_FAIL(PCE_EINVAL, "pce_pack_weights: null pointer");
  if (kv <= 0 || c_in <= 0 || c_out <= 0) PCE_FAIL(PCE_EINVAL, "pce_pack_weights: sizes must be positive");
  if (!aligned16(packed)) PCE_FAIL(PCE_EINVAL, "pce_pack_weights: destination must be 16-byte aligned");
  int k8 = (c_in + 7) / 8, n_pad = (c_out + 31) / 32 * 32;
  long long total = (long long)kv * k8 * n_pad;
  hipLaunchKernelGGL(pack_weights_kernel, dim3((unsigned)pce_div_up(total, 256)), dim3(256), 0, (hipStream_t)stream,
                     (const half_t *)w, (half_t *)packed, kv, c_in, c_out, k8, n_pad);
  PCE_LAUNCH_CHECK("pack_weights");
  return PCE_OK;
}

extern "C" int64_t pce_conv_fod_workspace_bytes(int64_t n_out, int32_t c_out, int32_t dtype) {
  return dtype == PCE_F16 ? pce_align_up(n_out * (int64_t)c_out * 4, 256) : 0;
}

template <typename T>
static int fod_impl(const void *in, const void *w, const void *wp, void *out, int64_t n_out, int c_in, int c_out, int kv,
                    int mid, const int *imap, const int *omap, const int *kpos, const int *qkpos, int64_t qsum,
                    float *acc, const Epi &e, hipStream_t s) {
  TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out);
  set_out<T>(&a, acc, true, n_out);
  int rc;
  long long total = (long long)n_out * c_out;
  if (!stage_on(0)) {
  } else if (mid >= 0) {
    // centre offset: dense GEMM over identical rows, initialises the accumulator (beta = 0)
    a.mode = MODE_DENSE;
    a.epi = EPI_ROWS_F32;
    a.w_fixed = mid;
    a.n_rows = n_out;
    if ((rc = launch_tile<T>(a, pce_div_up(n_out, 128), s))) return rc;
  } else {
    hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)pce_div_up(total, 1024)), dim3(256), 0, s, acc, total);
    PCE_LAUNCH_CHECK("zero_f32");
  }
  a.mode = MODE_FOD;
  a.epi = EPI_ATOMIC_F32;
  a.imap = imap;
  a.omap = omap;
  a.kpos = kpos;
  a.qkpos = qkpos;
  if (stage_on(1) && (rc = launch_tile<T>(a, qsum / PCE_QUANTUM, s))) return rc;
  if (sizeof(T) == 2 && stage_on(2)) {
    hipLaunchKernelGGL(convert_f32_f16_kernel, dim3((unsigned)pce_div_up(total, 2048)), dim3(256), 0, s,
                       (const float *)acc, (half_t *)out, total);
    PCE_LAUNCH_CHECK("convert_f32_f16");
  }
  if (!stage_on(2)) return PCE_OK;
  return launch_epilogue_pass<T>((T *)out, n_out, c_out, e, s);
}

extern "C" int pce_conv_fwd_fod(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid, const int32_t *imap,
                                const int32_t *omap, const int32_t *kpos, const int32_t *qkpos, int64_t qsum, void *ws,
                                int64_t ws_bytes, const pce_epilogue_t *epilogue, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_fod", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_fwd_fod", qsum))) return rc;
  Epi e;
  if ((rc = read_epilogue("pce_conv_fwd_fod", epilogue, out, &e))) return rc;
  if (qsum > 0 && (!imap || !omap || !kpos || !qkpos)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod: null map pointer");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16) {
    int64_t need = pce_conv_fod_workspace_bytes(n_out, c_out, dtype);
    if (!ws || ws_bytes < need) PCE_FAIL(PCE_EWORKSPACE, "pce_conv_fwd_fod: fp16 needs an fp32 accumulator of %lld bytes", (long long)need);
    if (!aligned16(ws) || !aligned16(out)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod: workspace and output must be 16-byte aligned");
    return fod_impl<half_t>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, qsum, (float *)ws, e, s);
  }
  if (!aligned16(out)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod: output must be 16-byte aligned");
  return fod_impl<float>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, qsum, (float *)out, e, s);
}

// ---- fetch-on-demand without a workspace argument ---------------------------------------------------
// For callers that cannot allocate device memory (code under HIP graph capture, serving loops, harnesses
// that forbid it): the fp32 accumulator of the fp16 dataflow lives in a file-scope device array.  Every GPU
// the library runs on holds its own copy of the array, at its own address, until the process ends; the
// address is looked up once per device and that pointer -- never the array's name, which in host code is
// only a stand-in for the symbol -- is what the kernels receive.
#define PCE_STATIC_SCRATCH_BYTES (32ll << 20)
#define PCE_STATIC_MAX_DEVICES 16
static __device__ __align__(256) unsigned char scratch[PCE_STATIC_SCRATCH_BYTES];
static void *g_scratch_ptr[PCE_STATIC_MAX_DEVICES];
static std::mutex g_scratch_mutex;

// device address of this device's copy of `scratch` (looked up by pce_conv_fod_static_init, or on the first call on the device)
static int static_scratch(void **ptr) {
  int dev = 0;
  PCE_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= PCE_STATIC_MAX_DEVICES) PCE_FAIL(PCE_ECAPACITY, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    PCE_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) PCE_FAIL(PCE_EHIP, "hipGetSymbolAddress returned a null address for the static scratch array");
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return PCE_OK;
}

extern "C" int64_t pce_conv_fod_static_capacity_bytes(void) { return PCE_STATIC_SCRATCH_BYTES; }

extern "C" int pce_conv_fod_static_init(void) {
  void *p = nullptr;
  return static_scratch(&p);
}

extern "C" int pce_conv_fwd_fod_static(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                       int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid,
                                       const int32_t *imap, const int32_t *omap, const int32_t *kpos, const int32_t *qkpos,
                                       int64_t qsum, const pce_epilogue_t *epilogue, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_fod_static", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_fwd_fod_static", qsum))) return rc;
  Epi e;
  if ((rc = read_epilogue("pce_conv_fwd_fod_static", epilogue, out, &e))) return rc;
  if (qsum > 0 && (!imap || !omap || !kpos || !qkpos)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod_static: null map pointer");
  if (!aligned16(out)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod_static: output must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F32)  // fp32 accumulates in the output itself: no scratch at all
    return fod_impl<float>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, qsum, (float *)out, e, s);
  const int64_t need = pce_conv_fod_workspace_bytes(n_out, c_out, dtype);
  if (need > PCE_STATIC_SCRATCH_BYTES)
    PCE_FAIL(PCE_ECAPACITY, "pce_conv_fwd_fod_static: the fp32 accumulator of %lld rows x %d channels needs %lld bytes, the static "
             "scratch array holds %lld (use pce_conv_fwd_fod with a workspace)", (long long)n_out, (int)c_out, (long long)need,
             (long long)PCE_STATIC_SCRATCH_BYTES);
  void *acc = nullptr;
  if ((rc = static_scratch(&acc))) return rc;
  // the centre GEMM (or the zero fill of a layer without centre offset) overwrites every accumulator row this
  // call uses before the pair tiles add to it: nothing of an earlier call's contents is read
  return fod_impl<half_t>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, qsum, (float *)acc, e, s);
}

template <typename T>
static int launch_scatter(const T *buf_out, T *out, int64_t n_out, int c_out, const int *ocsr, const int *ocode,
                          const int *qkpos, int add_existing, const Epi &e, hipStream_t s) {
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  bool vec_out = (c_out % VEC == 0) && aligned16(out) && aligned16(buf_out) && epi_aligned(e);
  if (vec_out) {
    int G = pow2_at_least(c_out / VEC);
    if (G > 64) G = 64;
    hipLaunchKernelGGL((scatter_rows_kernel<T, VEC>), dim3((unsigned)pce_div_up(n_out, 256 / G)), dim3(256), 0, s,
                       buf_out, (long long)n_out, c_out, G, ocsr, ocode, qkpos, out, add_existing, (const T *)e.bias,
                       (const T *)e.res, e.act, e.slope);
  } else {
    int G = pow2_at_least(c_out);
    if (G > 64) G = 64;
    hipLaunchKernelGGL((scatter_rows_kernel<T, 1>), dim3((unsigned)pce_div_up(n_out, 256 / G)), dim3(256), 0, s,
                       buf_out, (long long)n_out, c_out, G, ocsr, ocode, qkpos, out, add_existing, (const T *)e.bias,
                       (const T *)e.res, e.act, e.slope);
  }
  PCE_LAUNCH_CHECK("scatter_rows");
  return PCE_OK;
}

template <typename T>
static int gms_impl(const void *in, const void *w, const void *wp, void *out, int64_t n_in, int64_t n_out, int c_in,
                    int c_out, int kv, int mid, const int *icsr, const int *icode, const int *ocsr, const int *ocode,
                    const int *kpos, const int *qkpos, int64_t qsum, T *buffer, const Epi &e, hipStream_t s) {
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  T *buf_in = buffer;
  T *buf_out = buffer + qsum * c_in;  // backend/spconv.cu:121
  int rc;
  if (qsum > 0 && stage_on(3)) {
    // gather: every input row to the staging rows of its pairs
    bool vec_in = (c_in % VEC == 0) && aligned16(in) && aligned16(buf_in);
    if (vec_in) {
      int row_vecs = c_in / VEC;
      int G = pow2_at_least(row_vecs);
      if (G > 64) G = 64;
      typedef typename VecOf<T, VEC>::type V;
      hipLaunchKernelGGL((gather_rows_kernel<V>), dim3((unsigned)pce_div_up(n_in, 256 / G)), dim3(256), 0, s,
                         (const V *)in, (long long)n_in, row_vecs, G, icsr, icode, qkpos, (V *)buf_in);
    } else {
      int G = pow2_at_least(c_in);
      if (G > 64) G = 64;
      hipLaunchKernelGGL((gather_rows_kernel<T>), dim3((unsigned)pce_div_up(n_in, 256 / G)), dim3(256), 0, s,
                         (const T *)in, (long long)n_in, c_in, G, icsr, icode, qkpos, buf_in);
    }
    PCE_LAUNCH_CHECK("gather_rows");
  }
  if (qsum > 0 && stage_on(1)) {
    // grouped GEMM: every 128-row tile of the staging buffer belongs to one offset
    TileArgs a = base_args<T>(buf_in, w, wp, kv, c_in, c_out);
    set_out<T>(&a, buf_out, false, qsum);
    a.kpos = kpos;
    a.qkpos = qkpos;
    a.mode = MODE_BUF;
    a.epi = EPI_ROWS;
    if ((rc = launch_tile<T>(a, qsum / PCE_QUANTUM, s))) return rc;
  }
  if (mid >= 0 && stage_on(0)) {
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out);
    set_out<T>(&a, out, false, n_out);
    a.mode = MODE_DENSE;
    a.epi = EPI_ROWS;
    a.w_fixed = mid;
    a.n_rows = n_out;
    if ((rc = launch_tile<T>(a, pce_div_up(n_out, 128), s))) return rc;
  }
  if (!stage_on(2)) return PCE_OK;
  // scatter: output-stationary sum over each row's staging rows, fp32 accumulate
  return launch_scatter<T>(buf_out, (T *)out, n_out, c_out, ocsr, ocode, qkpos, mid >= 0 ? 1 : 0, e, s);
}

extern "C" int pce_conv_fwd_gms(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid,
                                const int32_t *icsr, const int32_t *icode, const int32_t *ocsr, const int32_t *ocode,
                                const int32_t *kpos, const int32_t *qkpos, int64_t qsum, void *buffer,
                                int64_t buffer_elems, const pce_epilogue_t *epilogue, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_gms", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_fwd_gms", qsum))) return rc;
  Epi e;
  if ((rc = read_epilogue("pce_conv_fwd_gms", epilogue, out, &e))) return rc;
  if (!icsr || !ocsr || !kpos || !qkpos || (qsum > 0 && (!icode || !ocode))) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_gms: null map pointer");
  if (qsum > 0 && (!buffer || buffer_elems < qsum * ((int64_t)c_in + c_out)))
    PCE_FAIL(PCE_EWORKSPACE, "pce_conv_fwd_gms: buffer holds %lld elements, needs %lld", (long long)buffer_elems, (long long)(qsum * ((int64_t)c_in + c_out)));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16)
    return gms_impl<half_t>(in, w, wp, out, n_in, n_out, c_in, c_out, kv, mid, icsr, icode, ocsr, ocode, kpos, qkpos, qsum, (half_t *)buffer, e, s);
  return gms_impl<float>(in, w, wp, out, n_in, n_out, c_in, c_out, kv, mid, icsr, icode, ocsr, ocode, kpos, qkpos, qsum, (float *)buffer, e, s);
}

// Fetch-on-demand with deferred scatter: pair tiles gather their input rows, multiply and store the
// partial row at its slot in output-CSR order (no atomics); the scatter is the epilogue of the
// centre GEMM, which adds each output row's contiguous partial rows in fp32 and stores the row once.
template <typename T>
static int fds_impl(const void *in, const void *w, const void *wp, void *out, int64_t n_out, int c_in, int c_out, int kv,
                    int mid, const int *imap, const int *omap, const int *oslot, const int *kpos, const int *qkpos,
                    const int32_t *kpos_host, const int32_t *qkpos_host, const int *ocsr, const int *route, int64_t n_pairs,
                    int64_t qsum, T *buffer, const Epi &e, hipStream_t s) {
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  int rc;
  const int *multi_rows = nullptr, *multi_count = nullptr;  // set by the routed pair tiles
  if (!buffer && qsum > 0) {
    // Every output row has exactly one pair (a transposed layer whose kernel equals its stride: each fine
    // voxel has one parent): a pair's product is its output row, stored once with the epilogue, no partial rows.
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
    set_out<T>(&a, out, false, n_out, e.ldo);
    set_host_pos(&a, kpos_host, qkpos_host);
    a.imap = imap;
    a.oslot = omap;
    a.kpos = kpos;
    a.qkpos = qkpos;
    a.mode = MODE_FOD_BUF;
    a.epi = EPI_ROWS;
    set_epi(&a, e);
    return launch_tile<T>(a, qsum / PCE_QUANTUM, s);
  }
  if (mid >= 0 && qsum > 0 && omap && stage_on(4)) {
    // Pair chunks and centre GEMM share one launch (neither reads what the other writes); a pass
    // over the pairs then adds every output row's partial rows to the centre term stored there.
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
    set_out<T>(&a, buffer, false, n_pairs);
    set_host_pos(&a, kpos_host, qkpos_host);
    a.imap = imap;
    a.oslot = oslot;
    a.items = qsum / 32;
    TileArgs c = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
    set_out<T>(&c, out, false, n_out, e.ldo);
    c.w_fixed = mid;
    c.n_rows = n_out;
    c.items = pce_div_up(n_out, 32);
    c.ocsr = ocsr;
    a.stream = c.stream;   // the partial rows of a layer leave the way its output rows do
    set_epi(&c, e);
    if (a.host_pos && wave_gemm_ok(a, sizeof(T)) && wave_gemm_ok(c, sizeof(T)) && aligned16(buffer) && epi_aligned(e)) {
      if (stage_on(1) && (rc = launch_wave_gemm(a, c, s))) return rc;
      if (stage_on(2) && (rc = launch_rowsum_pairs<T>((const T *)buffer, (T *)out, n_out, n_pairs, c_out, omap, oslot, ocsr,
                                                      e.act, e.slope, s, e.ldo)))
        return rc;
      return PCE_OK;
    }
  }
  if (mid < 0 && route && buffer && qsum > 0 && stage_on(1) && stage_on(2) && stage_on(5) && n_out + n_pairs < (1ll << 31)) {
    // Routed pair tiles (a layer without centre offset): the only pair of an output row stores the finished row
    // with the epilogue, the pairs of the other rows store partial rows; the row sum then visits only rows with
    // two pairs or more.  Taken by the pipelined kernel's shapes; the others ignore the routing.
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
    set_out<T>(&a, out, false, n_out, e.ldo);
    set_host_pos(&a, kpos_host, qkpos_host);
    a.imap = imap;
    a.oslot = route + PCE_ROUTE_HEAD;
    a.kpos = kpos;
    a.qkpos = qkpos;
    a.mode = MODE_FOD_BUF;
    a.epi = EPI_ROWS;
    a.out_alt = buffer;
    a.n_split = (int)n_out;
    set_epi(&a, e);
    if (pipe_gemm_ok(a, sizeof(T)) && aligned16(buffer)) {
      if ((rc = launch_pipe_gemm(a, qsum / PCE_QUANTUM, s))) return rc;
      multi_count = route;
      multi_rows = route + PCE_ROUTE_HEAD + n_pairs;
    }
  }
  if (qsum > 0 && stage_on(1) && !multi_rows) {
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
    set_out<T>(&a, buffer, false, n_pairs);
    set_host_pos(&a, kpos_host, qkpos_host);
    a.imap = imap;
    a.oslot = oslot;
    a.kpos = kpos;
    a.qkpos = qkpos;
    a.mode = MODE_FOD_BUF;
    a.epi = EPI_ROWS;
    if (mid >= 0 && omap && stage_on(2) && stage_on(4) && stage_on(5) && stage_on(6) && qsum <= 4 * n_out &&
        pce_div_up(n_out, 128) * ((c_out + 127) / 128) < 2048 && pipe_gemm_ok(a, sizeof(T))) {
      // wide fp16 layer with few pairs per row: pair tiles and the plain centre GEMM (bias and residual fused,
      // activation on rows without partial rows) share one launch, then the pass that adds each row's partial
      // rows.  Measured: 24 instead of 31 us at 0.3 pairs per row (C 96), 55 instead of 61 at 2.4 (C 128), equal
      // at 9 (C 128), 4-6 % slower at 9-13 pairs per row with 256 channels, where the launches stay separate;
      // so do those of a centre GEMM that fills the machine twice over by itself (nothing to gain, and a
      // network on 954 k voxels ran 3 % slower with them combined).
      TileArgs c = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
      set_out<T>(&c, out, false, n_out, e.ldo);
      c.mode = MODE_DENSE;
      c.epi = EPI_ROWS;
      c.w_fixed = mid;
      c.n_rows = n_out;
      c.ocsr = ocsr;
      c.act_alone_only = 1;
      set_epi(&c, e);
      if (pipe_gemm_ok(c, sizeof(T))) {
        if ((rc = launch_pipe_both(a, qsum / PCE_QUANTUM, c, pce_div_up(n_out, 128), s))) return rc;
        return launch_rowsum_pairs<T>((const T *)buffer, (T *)out, n_out, n_pairs, c_out, omap, oslot, ocsr, e.act, e.slope, s, e.ldo);
      }
    }
    if (a.host_pos && wave_gemm_ok(a, sizeof(T)) && stage_on(4)) {
      TileArgs none = a;
      none.items = 0;
      a.items = qsum / 32;
      if ((rc = launch_wave_gemm(a, none, s))) return rc;
    } else if ((rc = launch_tile<T>(a, qsum / PCE_QUANTUM, s))) {
      return rc;
    }
  }
  if (!stage_on(2)) return PCE_OK;
  if (mid >= 0 && omap && stage_on(4)) {
    // plain centre GEMM (bias and residual fused, activation on rows without partial rows), then the
    // pass over the pairs that adds each row's partial rows: no partial-row staging in the GEMM epilogue
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
    set_out<T>(&a, out, false, n_out, e.ldo);
    a.mode = MODE_DENSE;
    a.epi = EPI_ROWS;
    a.w_fixed = mid;
    a.n_rows = n_out;
    a.ocsr = ocsr;
    a.act_alone_only = 1;
    set_epi(&a, e);
    if ((rc = launch_tile<T>(a, pce_div_up(n_out, 128), s))) return rc;
    return launch_rowsum_pairs<T>((const T *)buffer, (T *)out, n_out, n_pairs, c_out, omap, oslot, ocsr, e.act, e.slope, s, e.ldo);
  }
  if (mid >= 0) {
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
    set_out<T>(&a, out, false, n_out, e.ldo);
    a.mode = MODE_DENSE;
    a.epi = EPI_ROWS_CSR;
    a.w_fixed = mid;
    a.n_rows = n_out;
    a.ocsr = ocsr;
    a.buf = buffer;
    a.b_vec = (c_out % 8 == 0) && aligned16(buffer);
    set_epi(&a, e);
    return launch_tile<T>(a, pce_div_up(n_out, 128), s);
  }
  bool vec = (c_out % VEC == 0) && aligned16(out) && aligned16(buffer) && epi_aligned(e);
  if (vec) {
    int G = pow2_at_least(c_out / VEC);
    if (G > 64) G = 64;
    // routed layer: the list holds at most n_out rows; a bounded grid strides over what it holds
    long long blocks = pce_div_up(n_out, 256 / G);
    if (multi_rows && blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL((rowsum_kernel<T, VEC>), dim3((unsigned)blocks), dim3(256), 0, s,
                       (const T *)buffer, (long long)n_out, c_out, G, ocsr, (T *)out, (const T *)e.bias, (const T *)e.res,
                       e.act, e.slope, multi_rows, multi_count, stream_policy((long long)n_out * c_out * (long long)sizeof(T)),
                       e.ldo > 0 ? e.ldo : c_out);
  } else {
    int G = pow2_at_least(c_out);
    if (G > 64) G = 64;
    long long blocks = pce_div_up(n_out, 256 / G);
    if (multi_rows && blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL((rowsum_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, s,
                       (const T *)buffer, (long long)n_out, c_out, G, ocsr, (T *)out, (const T *)e.bias, (const T *)e.res,
                       e.act, e.slope, multi_rows, multi_count, stream_policy((long long)n_out * c_out * (long long)sizeof(T)),
                       e.ldo > 0 ? e.ldo : c_out);
  }
  PCE_LAUNCH_CHECK("rowsum");
  return PCE_OK;
}

// Routing of the pairs of a layer without centre offset.  route[0] = number of output rows whose pair count is
// not one, route[4 .. 4+M) = destination of every pair (the output row itself where the pair is the row's only
// one, else n_out + the pair's partial-row slot), route[4+M .. 4+M+n_out) = the rows whose pair count is not
// one, in the order in which they were counted (any order serves the row sum, which visits exactly these).
__global__ void route_clear_kernel(int *route) {
  if (threadIdx.x < PCE_ROUTE_HEAD) route[threadIdx.x] = 0;
}
__global__ void __launch_bounds__(256) pair_route_kernel(const int *__restrict__ omap, const int *__restrict__ oslot,
                                                         const int *__restrict__ ocsr, long long n_pairs, int n_out,
                                                         int *__restrict__ route) {
  long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n_pairs) {
    int o = omap[t];
    route[PCE_ROUTE_HEAD + t] = (ocsr[o + 1] - ocsr[o] == 1) ? o : n_out + oslot[t];
  }
  if (t < n_out && ocsr[t + 1] - ocsr[t] != 1) route[PCE_ROUTE_HEAD + n_pairs + atomicAdd(&route[0], 1)] = (int)t;
}

extern "C" int64_t pce_pair_route_elems(int64_t n_pairs, int64_t n_out) {
  return (n_pairs < 0 || n_out < 0) ? 0 : PCE_ROUTE_HEAD + n_pairs + n_out;
}

extern "C" int pce_pair_route(const int32_t *omap, const int32_t *oslot, const int32_t *ocsr, int64_t n_pairs, int64_t n_out,
                              int32_t *route, int64_t route_elems, pce_stream_t stream) {
  if (n_pairs < 0 || n_out < 0) PCE_FAIL(PCE_EINVAL, "pce_pair_route: negative count");
  if (!route || !ocsr || (n_pairs > 0 && (!omap || !oslot))) PCE_FAIL(PCE_EINVAL, "pce_pair_route: null pointer");
  if (n_out + n_pairs >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "pce_pair_route: n_out + n_pairs = %lld exceeds int32", (long long)(n_out + n_pairs));
  if (route_elems < pce_pair_route_elems(n_pairs, n_out))
    PCE_FAIL(PCE_EWORKSPACE, "pce_pair_route: route holds %lld elements, needs %lld", (long long)route_elems, (long long)pce_pair_route_elems(n_pairs, n_out));
  hipLaunchKernelGGL(route_clear_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, route);
  PCE_LAUNCH_CHECK("route_clear");
  long long threads = n_pairs > n_out ? n_pairs : n_out;
  if (threads == 0) return PCE_OK;
  hipLaunchKernelGGL(pair_route_kernel, dim3((unsigned)pce_div_up(threads, 256)), dim3(256), 0, (hipStream_t)stream, omap, oslot,
                     ocsr, (long long)n_pairs, (int)n_out, route);
  PCE_LAUNCH_CHECK("pair_route");
  return PCE_OK;
}

extern "C" int pce_conv_fwd_fds(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid, const int32_t *imap,
                                const int32_t *omap, const int32_t *oslot, const int32_t *kpos, const int32_t *qkpos,
                                const int32_t *kpos_host, const int32_t *qkpos_host, const int32_t *ocsr,
                                const int32_t *route, int64_t n_pairs, int64_t qsum, void *buffer, int64_t buffer_elems,
                                const pce_epilogue_t *epilogue, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_fds", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_fwd_fds", qsum))) return rc;
  Epi e;
  if ((rc = read_epilogue("pce_conv_fwd_fds", epilogue, out, &e, c_in, c_out))) return rc;
  if (!ocsr || !kpos || !qkpos || (qsum > 0 && (!imap || !oslot))) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fds: null map pointer");
  if (n_pairs < 0 || n_pairs > qsum) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fds: n_pairs=%lld outside [0, qsum]", (long long)n_pairs);
  if (!buffer && n_pairs > 0) {
    // no partial-row buffer: the caller states that every output row has exactly one pair
    if (mid >= 0 || !omap || n_pairs != n_out)
      PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fds: without a buffer the layer must have no centre offset, omap and n_pairs == n_out");
  } else if (n_pairs > 0 && buffer_elems < n_pairs * (int64_t)c_out) {
    PCE_FAIL(PCE_EWORKSPACE, "pce_conv_fwd_fds: buffer holds %lld elements, needs %lld", (long long)buffer_elems, (long long)(n_pairs * (int64_t)c_out));
  }
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16)
    return fds_impl<half_t>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, oslot, kpos, qkpos, kpos_host, qkpos_host, ocsr, route, n_pairs, qsum, (half_t *)buffer, e, s);
  return fds_impl<float>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, oslot, kpos, qkpos, kpos_host, qkpos_host, ocsr, route, n_pairs, qsum, (float *)buffer, e, s);
}

template <typename T>
static int os_impl(const void *in, const void *w, const void *wp, void *out, int64_t n_out, int c_in, int c_out, int kv,
                   const int *nbr, const Epi &e, hipStream_t s) {
  TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out, e.lda);
  set_out<T>(&a, out, false, n_out, e.ldo);
  set_epi(&a, e);
  a.nbr = nbr;
  a.n_rows = n_out;
  a.mode = MODE_OS;
  a.epi = EPI_ROWS;
  return launch_tile<T>(a, pce_div_up(n_out, 128), s);
}

extern "C" int pce_conv_fwd_os(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                               int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, const int32_t *nbr,
                               const pce_epilogue_t *epilogue, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_os", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, -1);
  if (rc) return rc;
  if (!nbr) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_os: null neighbour table");
  Epi e;
  if ((rc = read_epilogue("pce_conv_fwd_os", epilogue, out, &e, c_in, c_out))) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16) return os_impl<half_t>(in, w, wp, out, n_out, c_in, c_out, kv, nbr, e, s);
  return os_impl<float>(in, w, wp, out, n_out, c_in, c_out, kv, nbr, e, s);
}

// ---- output-stationary over rows ordered by their neighbour pattern --------------------------------------------
// On a surface-like cloud most voxels of a submanifold layer have no neighbour at most offsets (64 x 2048 LiDAR rays at
// 0.1 m: 0.2 pairs per voxel, 87 % of the voxels none at all).  A wavefront that owns 32 consecutive rows still meets
// the union of their patterns -- 3.9 offsets on that cloud -- and the dataflows above avoid that by treating pairs
// apart from the centre term, at the price of partial rows and a second launch.  Here the rows are visited in an order
// that puts equal patterns side by side: sorted by (lowest, second-lowest) offset present, rows without neighbours
// first and in their own order.  The union over 32 such rows is 0.6 offsets on the same cloud, so one wavefront
// does the centre product of its rows from LDS (line-ordered global -> LDS copies, as wave_gemm_kernel), then for
// each offset of the union gathers the rows that have it with lane-masked loads, accumulates in the same registers
// and stores every finished row once: no partial rows, no atomics, one launch.
// Workgroups [0, heavy_wgs) take the rows with three neighbours or more, 32 rows per WORKGROUP: a wavefront spends one
// trip to memory per offset, one after the other, and a dense cluster has rows with twenty offsets, so the four
// wavefronts share the offsets of the chunk's union among them (wavefront 0 also does the centre product) and add
// their accumulators through LDS at the end.  The other workgroups take four chunks of the remaining rows, one per
// wavefront, last chunks first (the rows with one or two neighbours are the last of that part).
// A strided layer (mid < 0) has no centre term: every output row has one to kv pairs, the same order groups the rows
// by the offsets of their pairs, and the kernel starts from zero sums.
template <int NB, int KS>
__global__ void __launch_bounds__(256, 4) wave_os_kernel(TileArgs a, const int *__restrict__ perm,
                                                         const unsigned *__restrict__ rmask, int mid, long long n_main,
                                                         int heavy_wgs) {
  constexpr int PPR = KS * 2;   // 16-byte pieces per input row
  constexpr int NI = KS;        // global -> LDS instructions for the 32 centre rows
  constexpr int REGION0 = WaveLds<NB>::PIECES > 32 * PPR ? WaveLds<NB>::PIECES : 32 * PPR;
  constexpr int REGION = REGION0 > 256 ? REGION0 : 256;   // also one accumulator block of 64 lanes (see below)
  static_assert(REGION * 16 >= 64 * 64, "a wavefront's region holds one accumulator block of all its lanes");
  __shared__ __attribute__((aligned(16))) half8 Pl[4][REGION];
  __shared__ __attribute__((aligned(16))) half8 Wc[KS * 2 * NB * 32];   // the centre offset's weights, shared by the workgroup
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const half_t *Wp = (const half_t *)a.Wp;
  const long long wstep = (long long)a.k8_total * a.n_pad * 8;
  // every wavefront copies its share of the centre weights (one copy of them per workgroup instead of one per wavefront);
  // a layer without a centre offset (mid < 0: strided) has no such term and starts from zero sums
  if (mid >= 0) {
    constexpr int FR = KS * 2 * NB * 32;   // fragments: [k8][column]
#pragma unroll
    for (int i = 0; i < (FR + 255) / 256; ++i) {
      const int f = i * 256 + wave * 64 + lane;
      const half_t *gp = Wp + mid * wstep + (long long)(f < FR ? f : FR - 1) * 8;
      if (i * 256 + wave * 64 < FR)   // wavefront-uniform
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                         (__attribute__((address_space(3))) void *)&Wc[i * 256 + wave * 64], 16, 0, 0);
    }
  }
  const bool heavy = (int)blockIdx.x < heavy_wgs;   // the same for the whole workgroup
  long long j0, j_end;
  bool idle = false;
  if (heavy) {
    j0 = n_main + (long long)blockIdx.x * 32;
    j_end = a.n_rows;
  } else {
    const long long chunks = (n_main + 31) / 32;
    const long long chunk = chunks - 1 - (((long long)blockIdx.x - heavy_wgs) * 4 + wave);
    idle = chunk < 0;
    j0 = idle ? 0 : chunk * 32;
    j_end = n_main;
  }
  if (idle) {   // still joins the barrier behind the weight copies
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    return;
  }
  const half_t *A = (const half_t *)a.A;
  const int orow = j0 + l32 < j_end ? perm[j0 + l32] : -1;
  const unsigned m = orow >= 0 ? rmask[orow] : 0u;
  unsigned u = m;
#pragma unroll
  for (int d = 1; d < 32; d <<= 1) u |= (unsigned)__shfl_xor((int)u, d, PCE_WAVE);
  unsigned todo = __builtin_amdgcn_readfirstlane(u);   // offsets any of the 32 rows has: the same in every lane
  // this wavefront's share of them: the offsets whose number is its own modulo four.  (A split that depends on the
  // offset alone: the sums of a row are then grouped the same way whichever rows share its chunk, and the result
  // of a layer does not depend on where the counting sort happened to put a row among those of its key.)
  if (heavy) todo &= 0x11111111u << wave;
  const bool centre = mid >= 0 && (!heavy || wave == 0);
  half8 wf[KS][NB];
  if (centre) {
    // centre rows -> LDS, in line order (a valid row stands in for one past the end)
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int e = it * 64 + lane, r = e / PPR, sl = e % PPR;
      const long long j = j0 + r < j_end ? j0 + r : j_end - 1;
      const half_t *gp = A + (long long)perm[j] * a.lda + ((sl ^ row_swizzle<PPR>(r)) * 8);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                       (__attribute__((address_space(3))) void *)&Pl[wave][it * 64], 16, 0, 0);
    }
  }
  // the neighbour of this lane's row at the first offset of the union, requested while the centre rows travel
  int k_next = todo ? __ffs((int)todo) - 1 : -1;
  int nb_next = (k_next >= 0 && ((m >> k_next) & 1u)) ? a.nbr[(long long)k_next * a.n_rows + orow] : -1;
  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();   // the centre weights of all four wavefronts' copies (and this wavefront's rows) are in LDS
  if (centre) {
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) wf[s][nb] = Wc[(2 * s + g) * (NB * 32) + nb * 32 + l32];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const half8 af = Pl[wave][l32 * PPR + ((2 * s + g) ^ row_swizzle<PPR>(l32))];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[s][nb], af, acc[nb], 0, 0, 0);
    }
  }
  // the offsets, one after the other: rows that have the offset fetch their neighbour's fragments themselves
  // (a lane per row and K step; lanes of rows without it stay idle and multiply zeros)
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  while (k_next >= 0) {
    const int k = k_next, nrow = nb_next;
    todo &= todo - 1u;
    half8 af[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s)
      af[s] = nrow >= 0 ? *reinterpret_cast<const half8 *>(A + (long long)nrow * a.lda + s * 16 + g * 8) : zero;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        wf[s][nb] = *reinterpret_cast<const half8 *>(Wp + k * wstep + ((long long)(2 * s + g) * a.n_pad + nb * 32 + l32) * 8);
    k_next = todo ? __ffs((int)todo) - 1 : -1;
    nb_next = (k_next >= 0 && ((m >> k_next) & 1u)) ? a.nbr[(long long)k_next * a.n_rows + orow] : -1;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[s][nb], af[s], acc[nb], 0, 0, 0);
  }
  if (heavy) {
    // wavefronts 1..3 hand their accumulators to wavefront 0, one 32-column block at a time through their own regions
    f32x16 *mine = reinterpret_cast<f32x16 *>(&Pl[wave][0]);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      __syncthreads();                       // the regions are free (centre fragments read, the previous block added)
      if (wave > 0) mine[lane] = acc[nb];
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int w2 = 1; w2 < 4; ++w2) {
          const f32x16 other = reinterpret_cast<const f32x16 *>(&Pl[w2][0])[lane];
#pragma unroll
          for (int j = 0; j < 16; ++j) acc[nb][j] += other[j];
        }
      }
    }
    if (wave > 0) return;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();   // every lane has read its centre fragments: the region becomes the output staging area
  float V[NB][2][8];
  gather_row_pieces<NB>(acc, V, g);
  if (a.bias || a.res || a.act) epilogue_row_pieces<half_t, NB, true>(V, a, orow, 0, g, a.act != PCE_ACT_NONE);
  store_rows_via_lds<half_t, NB>(V, Pl[wave], (half_t *)a.out, orow, a, 0, lane, l32, g, a.stream);
}

// A chunk of 32 rows with two neighbours or more, NBW column blocks of it from column n0 on, by one workgroup.
// The four wavefronts split the INPUT CHANNELS, 16 each (one K step of the MFMA), and all walk the offsets of the
// chunk's union: a step then holds 16 bytes of a neighbour row and 16 bytes of weights per column block in a lane
// -- 12 registers at 64 columns, 8 at 32 -- so six or ten offsets are in flight per wavefront, where a wavefront that
// owns whole offsets (wave_os_kernel: k mod 4) has registers for one and spends one trip to memory per offset, seven
// in a row on a dense cluster.  The four partial sums of a row meet through LDS in wavefront 0, which stores the row.
// The rows of the chunk come as 128-byte records {row, mask, neighbour at offset 0, 1, ...} (the row order writes
// them for the rows with two neighbours or more): thread t fetches 16 bytes of the record of row t / 8 and files
// them by [slot][row] in LDS (33 words per slot: the eight threads of a row hit eight banks).  One trip to memory
// stands between the start of the workgroup and its first row gather; the centre product is one more offset of
// the walk (its neighbour is the row itself), so the workgroup copies neither centre rows nor centre weights.
// sb, s_end: the chunk's first record and the end of its section of the records.
template <int NBW, int KS, int REGION>
__device__ __forceinline__ void os2_shared_chunk(const TileArgs &a, const int *__restrict__ order, int mid, long long sb,
                                                 long long s_end, int n0, half8 (&Pl)[4][REGION]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const half_t *Wp = (const half_t *)a.Wp;
  const half_t *A = (const half_t *)a.A;
  const long long wstep = (long long)a.k8_total * a.n_pad * 8;
  const long long n = a.n_rows;
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int IDX_LD = 33;
  int *idxL = reinterpret_cast<int *>(&Pl[0][0]);
  static_assert(32 * IDX_LD * 4 <= 2 * REGION * 16, "the index table fits two regions");
  {
    const int r = threadIdx.x >> 3, q = threadIdx.x & 7;
    const bool have = sb + r < s_end;
    typedef int v4i_t __attribute__((ext_vector_type(4)));
    const v4i_t v = *reinterpret_cast<const __attribute__((address_space(1))) v4i_t *>(
        (const __attribute__((address_space(1))) int *)(order + PCE_ORDER_SREC_OFFSET(n)) + ((have ? sb + r : sb) * 32 + q * 4));
#pragma unroll
    for (int j = 0; j < 4; ++j) idxL[(4 * q + j) * IDX_LD + r] = have ? v[j] : (4 * q + j == 1 ? 0 : -1);
  }
  __syncthreads();
  const int orow = idxL[l32];
  const unsigned m = (unsigned)idxL[IDX_LD + l32];
  unsigned uu = m;
#pragma unroll
  for (int d = 1; d < 32; d <<= 1) uu |= (unsigned)__shfl_xor((int)uu, d, PCE_WAVE);
  const unsigned u = (unsigned)__builtin_amdgcn_readfirstlane((int)uu) | (1u << mid);   // the chunk's offsets and the centre
  f32x16 acc[NBW];
#pragma unroll
  for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;
  if (wave < KS) {
    const int s = wave;   // this wavefront's K step: input channels [16 s, 16 s + 16)
    // slot j holds the row fragment, the row's index and the weight fragments of one offset
    constexpr int SLOTS = NBW == 2 ? 6 : 10;
    half8 rf[SLOTS], wf[SLOTS][NBW];
    int ri[SLOTS];
    unsigned rem_issue = u;
    const half_t *Ab = A + s * 16 + g * 8;
    const half_t *Wb = Wp + ((long long)(2 * s + g) * a.n_pad + n0 + l32) * 8;
    // (every step issues its loads and its MFMAs unconditionally -- a slot beyond the last offset loads from a
    // valid address and multiplies zeros -- so that the waits in front of the MFMAs are counted exactly and leave the
    // loads of the other slots in flight; with the loads under a condition every wait became a full one)
#define PCE_OS2_ISSUE(J_)                                                                                          \
  {                                                                                                                \
    const int k_ = rem_issue ? __ffs((int)rem_issue) - 1 : 0;                                                      \
    const int v_ = idxL[(2 + k_) * IDX_LD + l32];                                                                  \
    ri[J_] = rem_issue ? (k_ == mid ? orow : v_) : -1;                                                             \
    rem_issue &= rem_issue - 1u;                                                                                   \
    rf[J_] = *reinterpret_cast<const half8 *>(Ab + (long long)(ri[J_] >= 0 ? ri[J_] : 0) * a.lda);                 \
    _Pragma("unroll") for (int nb = 0; nb < NBW; ++nb)                                                             \
      wf[J_][nb] = *reinterpret_cast<const half8 *>(Wb + k_ * wstep + nb * 32 * 8);                                \
  }
#define PCE_OS2_USE(J_)                                                                                            \
  {                                                                                                                \
    const half8 f_ = ri[J_] >= 0 ? rf[J_] : zero;                                                                  \
    _Pragma("unroll") for (int nb = 0; nb < NBW; ++nb)                                                             \
      acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[J_][nb], f_, acc[nb], 0, 0, 0);                          \
  }
#pragma unroll
    for (int j = 0; j < SLOTS; ++j) PCE_OS2_ISSUE(j)
    for (int round = (__popc(u) + SLOTS - 1) / SLOTS; round > 0; --round) {   // wavefront-uniform
#pragma unroll
      for (int j = 0; j < SLOTS; ++j) {
        __builtin_amdgcn_sched_barrier(0);
        PCE_OS2_USE(j)
        PCE_OS2_ISSUE(j)
      }
    }
#undef PCE_OS2_ISSUE
#undef PCE_OS2_USE
  }
  // wavefronts 1..3 hand their accumulators to wavefront 0, one 32-column block at a time through their own regions
  // (wavefront 1's region holds the end of the index table: the first barrier below stands behind its last reader);
  // a lane's 16 values go as four 16-byte pieces, piece j of all lanes side by side: no bank conflicts
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  f32x4_t *mine = reinterpret_cast<f32x4_t *>(&Pl[wave][0]);
#pragma unroll
  for (int nb = 0; nb < NBW; ++nb) {
    __syncthreads();
    if (wave > 0 && wave < KS) {
#pragma unroll
      for (int j = 0; j < 4; ++j) mine[j * 64 + lane] = f32x4_t{acc[nb][4 * j], acc[nb][4 * j + 1], acc[nb][4 * j + 2], acc[nb][4 * j + 3]};
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int w2 = 1; w2 < 4; ++w2) {
        if (w2 < KS) {
          const f32x4_t *theirs = reinterpret_cast<const f32x4_t *>(&Pl[w2][0]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const f32x4_t o = theirs[j * 64 + lane];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[nb][4 * j + i] += o[i];
          }
        }
      }
    }
  }
  if (wave > 0) return;
  float V[NBW][2][8];
  gather_row_pieces<NBW>(acc, V, g);
  if (a.bias || a.res || a.act) epilogue_row_pieces<half_t, NBW, true>(V, a, orow, n0, g, a.act != PCE_ACT_NONE);
  store_rows_via_lds<half_t, NBW>(V, Pl[0], (half_t *)a.out, orow, a, n0, lane, l32, g, a.stream);
}

// The same layer for clouds where most rows have no neighbour at all (at least half of them), in three kinds of
// workgroup, so that every wavefront of the launch is resident from the start and none waits for more trips to
// memory than its rows need (per-wavefront timestamps of wave_os_kernel on the 150 k-voxel scan: two rounds of
// wavefronts of 7 us each, of which 3 us go to the two dependent loads in front of the rows; beside them chains of
// one trip per offset, up to twelve in a row, in the chunks whose rows have two neighbours or more):
//   stream  (the bulk): a wavefront takes 64 consecutive rows in STORAGE order -- no row index to fetch first: the
//           rows travel to LDS with the first instructions of the wavefront, their offset masks beside them --
//           multiplies them by the centre weights and stores those whose mask is empty; rows with neighbours are
//           left to the two other kinds (their centre product is computed twice: a seventh of the rows on a LiDAR scan);
//   single  32 rows with exactly one neighbour, from the row order's records {row, mask, neighbour, -}: one trip for
//           the records, one for the centre rows, the neighbour's fragments and the weights of the chunk's first
//           offset (the order sorts these rows by their offset: a chunk has one offset, two at a boundary);
//   shared  32 rows with two neighbours or more per workgroup, from the row order's 128-byte records {row, mask,
//           neighbour at every offset}: one trip for the records, then the four wavefronts, which split the input
//           channels, walk the offsets of the chunk (the centre among them) with six in flight each.
// A row's sum is formed per wavefront over its offsets in ascending order, then wavefront 0 adds the others' in
// turn: the same for every run and every position of the row in the order, but not the order of additions of
// wave_os_kernel, so rows with two neighbours or more may differ from that kernel's in their last bits.
template <int NB, int KS>
__global__ void __launch_bounds__(256, 4) wave_os2_kernel(TileArgs a, const int *__restrict__ order, int mid, long long n_plain,
                                                          long long n_single, long long n_two, int heavy_wgs,
                                                          int shared_wgs, int single_wgs) {
  constexpr int PPR = KS * 2;   // 16-byte pieces per input row
  constexpr int REGION0 = WaveLds<NB>::PIECES > 64 * PPR ? WaveLds<NB>::PIECES : 64 * PPR;
  constexpr int REGION = REGION0 > 256 ? REGION0 : 256;   // also one accumulator block of 64 lanes
  static_assert(REGION * 16 >= 64 * 64, "a wavefront's region holds one accumulator block of all its lanes");
  __shared__ __attribute__((aligned(16))) half8 Pl[4][REGION];
  __shared__ __attribute__((aligned(16))) half8 Wc[KS * 2 * NB * 32];   // the centre offset's weights, shared by the workgroup
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const half_t *Wp = (const half_t *)a.Wp;
  const half_t *A = (const half_t *)a.A;
  const long long wstep = (long long)a.k8_total * a.n_pad * 8;
  const long long n = a.n_rows;
  // ---- shared: 32 rows with two neighbours or more per workgroup ------------------------------------------------
  // first the chunks of rows with three neighbours or more, the longest walks of the launch: at 33-64 output
  // channels two workgroups each, one per block of 32 columns (ten offsets in flight instead of six); then the
  // chunks of rows with two
  // (first in the code as well: these workgroups have the longest way to go, and what a wavefront runs before its
  // first load it fetches from a cold instruction cache)
  const long long n_shared = n - n_plain - n_single;
  if ((int)blockIdx.x < heavy_wgs) {
    if (NB == 2)
      os2_shared_chunk<1, KS, REGION>(a, order, mid, n_two + (long long)(blockIdx.x >> 1) * 32, n_shared, (blockIdx.x & 1) * 32, Pl);
    else
      os2_shared_chunk<NB, KS, REGION>(a, order, mid, n_two + (long long)blockIdx.x * 32, n_shared, 0, Pl);
    return;
  }
  if ((int)blockIdx.x < shared_wgs) {
    os2_shared_chunk<NB, KS, REGION>(a, order, mid, ((long long)blockIdx.x - heavy_wgs) * 32, n_two, 0, Pl);
    return;
  }
  {   // (the shared workgroups read the centre weights as they read the others')
    constexpr int FR = KS * 2 * NB * 32;   // fragments: [k8][column]
#pragma unroll
    for (int i = 0; i < (FR + 255) / 256; ++i) {
      const int f = i * 256 + wave * 64 + lane;
      const half_t *gp = Wp + mid * wstep + (long long)(f < FR ? f : FR - 1) * 8;
      if (i * 256 + wave * 64 < FR)   // wavefront-uniform
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                         (__attribute__((address_space(3))) void *)&Wc[i * 256 + wave * 64], 16, 0, 0);
    }
  }
  const int first_stream = shared_wgs + single_wgs;
  if ((int)blockIdx.x >= first_stream) {
    // ---- stream: 64 consecutive rows --------------------------------------------------------------------------
    const long long r0 = (((long long)blockIdx.x - first_stream) * 4 + wave) * 64;
    if (r0 >= n) {   // still joins the barrier behind the weight copies
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      return;
    }
#pragma unroll
    for (int it = 0; it < PPR; ++it) {
      const int e = it * 64 + lane, r = e / PPR, sl = e % PPR;
      const long long row = r0 + r < n ? r0 + r : n - 1;
      const half_t *gp = A + row * a.lda + ((sl ^ row_swizzle<PPR>(r)) * 8);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                       (__attribute__((address_space(3))) void *)&Pl[wave][it * 64], 16, 0, 0);
    }
    // the mask of row r0 + lane (no order: a plain GEMM, every row is stored)
    const unsigned mrow = order ? ((const unsigned *)(order + n))[r0 + lane < n ? r0 + lane : n - 1] : 0u;
    f32x16 acc[2][NB];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[h][nb][j] = 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // the centre weights of all four wavefronts' copies (and this wavefront's rows) are in LDS
    // (K step by K step: the weight fragments of one step serve both halves of the rows; holding those of all steps
    // beside 64 accumulator registers spilled)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      half8 wf[NB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) wf[nb] = Wc[(2 * s + g) * (NB * 32) + nb * 32 + l32];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int r = h * 32 + l32;
        const half8 af = Pl[wave][r * PPR + ((2 * s + g) ^ row_swizzle<PPR>(r))];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[h][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[nb], af, acc[h][nb], 0, 0, 0);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();   // every lane has read its fragments: the region becomes the output staging area
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const long long row = r0 + h * 32 + l32;
      const unsigned mh = (unsigned)__shfl((int)mrow, h * 32 + l32, PCE_WAVE);
      const int orow = (row < n && mh == 0u) ? (int)row : -1;   // rows with neighbours belong to the other workgroups
      float V[NB][2][8];
      gather_row_pieces<NB>(acc[h], V, g);
      if (a.bias || a.res || a.act) epilogue_row_pieces<half_t, NB, true>(V, a, orow, 0, g, a.act != PCE_ACT_NONE);
      store_rows_via_lds<half_t, NB>(V, Pl[wave], (half_t *)a.out, orow, a, 0, lane, l32, g, a.stream);
    }
    return;
  }
  const int4 *rec = reinterpret_cast<const int4 *>(order + PCE_ORDER_REC_OFFSET(n));
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // a lane's K half of a row, from an address that is valid for every lane; zeroed where there is no row
#define PCE_OS2_FRAGS(F_, NROW_)                                                                                   \
  {                                                                                                                \
    const int nr_ = (NROW_);                                                                                       \
    const half_t *rp_ = A + (long long)(nr_ >= 0 ? nr_ : 0) * a.lda + g * 8;                                       \
    _Pragma("unroll") for (int s = 0; s < KS; ++s) F_[s] = *reinterpret_cast<const half8 *>(rp_ + s * 16);         \
    _Pragma("unroll") for (int s = 0; s < KS; ++s) F_[s] = nr_ >= 0 ? F_[s] : zero;                                \
  }
  if ((int)blockIdx.x >= shared_wgs) {
    // ---- single: 32 rows with one neighbour each ---------------------------------------------------------------
    const long long p0 = n_plain + (((long long)blockIdx.x - shared_wgs) * 4 + wave) * 32, p_end = n_plain + n_single;
    if (p0 >= p_end) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      return;
    }
    const bool valid = p0 + l32 < p_end;
    const int4 rc = rec[valid ? p0 + l32 : p0];   // {row, mask (one bit), neighbour, -1}
    const int orow = valid ? rc.x : -1;
    const unsigned m = valid ? (unsigned)rc.y : 0u;
    unsigned u = m;
#pragma unroll
    for (int d = 1; d < 32; d <<= 1) u |= (unsigned)__shfl_xor((int)u, d, PCE_WAVE);
    unsigned todo = __builtin_amdgcn_readfirstlane(u);   // offsets any of the 32 rows has: the same in every lane
#pragma unroll
    for (int it = 0; it < KS; ++it) {   // centre rows -> LDS, in line order (the row of a lane past the end is the chunk's first)
      const int e = it * 64 + lane, r = e / PPR, sl = e % PPR;
      const int row = __shfl(rc.x, r, PCE_WAVE);
      const half_t *gp = A + (long long)row * a.lda + ((sl ^ row_swizzle<PPR>(r)) * 8);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                       (__attribute__((address_space(3))) void *)&Pl[wave][it * 64], 16, 0, 0);
    }
    half8 fa[KS], wk[KS][NB];
    PCE_OS2_FRAGS(fa, valid ? rc.z : -1)
    int k = __ffs((int)todo) - 1;   // a valid chunk has a row, the row an offset
    todo &= todo - 1u;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        wk[s][nb] = *reinterpret_cast<const half8 *>(Wp + k * wstep + ((long long)(2 * s + g) * a.n_pad + nb * 32 + l32) * 8);
    f32x16 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const half8 af = Pl[wave][l32 * PPR + ((2 * s + g) ^ row_swizzle<PPR>(l32))];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Wc[(2 * s + g) * (NB * 32) + nb * 32 + l32], af, acc[nb], 0, 0, 0);
    }
    while (true) {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const half8 fs = ((m >> k) & 1u) ? fa[s] : zero;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wk[s][nb], fs, acc[nb], 0, 0, 0);
      }
      if (!todo) break;
      k = __ffs((int)todo) - 1;
      todo &= todo - 1u;
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          wk[s][nb] = *reinterpret_cast<const half8 *>(Wp + k * wstep + ((long long)(2 * s + g) * a.n_pad + nb * 32 + l32) * 8);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();   // every lane has read its centre fragments: the region becomes the output staging area
    float V[NB][2][8];
    gather_row_pieces<NB>(acc, V, g);
    if (a.bias || a.res || a.act) epilogue_row_pieces<half_t, NB, true>(V, a, orow, 0, g, a.act != PCE_ACT_NONE);
    store_rows_via_lds<half_t, NB>(V, Pl[wave], (half_t *)a.out, orow, a, 0, lane, l32, g, a.stream);
    return;
  }
#undef PCE_OS2_FRAGS
}

// compute units of the current device (asked once per device)
static int cu_count() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (!cached[dev]) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached[dev] = v;
  }
  return cached[dev];
}

// workgroups of the three-kind kernel over a row order
static long long os2_workgroups(long long n_out, long long n_nonzero, long long n_single, long long n_heavy, int nb) {
  return pce_div_up(n_heavy, 32) * (nb == 2 ? 2 : 1) + pce_div_up(n_nonzero - n_single - n_heavy, 32) +
         pce_div_up(pce_div_up(n_single, 32), 4) + pce_div_up(pce_div_up(n_out, 64), 4);
}

// the three-kind kernel over a row order, or (order == nullptr) its stream workgroups alone: a plain GEMM
static int launch_wave_os2(const TileArgs &a, const int *order, int mid, long long n_out, long long n_nonzero, long long n_single,
                           long long n_heavy, int nb, int ks, hipStream_t s) {
  const long long n_plain = n_out - n_nonzero, n_two = n_nonzero - n_single - n_heavy;
  const long long heavy_wgs = pce_div_up(n_heavy, 32) * (nb == 2 ? 2 : 1), shared_wgs = heavy_wgs + pce_div_up(n_two, 32),
                  single_wgs = pce_div_up(pce_div_up(n_single, 32), 4), stream_wgs = pce_div_up(pce_div_up(n_out, 64), 4);
  if (shared_wgs + single_wgs + stream_wgs >= (1ll << 31) - 8) PCE_FAIL(PCE_ECAPACITY, "%lld rows exceed the grid limit", (long long)n_out);
  const unsigned grid2 = (unsigned)(shared_wgs + single_wgs + stream_wgs);
#define PCE_WOS2_CASE(NB_, KS_)                                                                                    \
  if (nb == NB_ && ks == KS_) {                                                                                    \
    hipLaunchKernelGGL((wave_os2_kernel<NB_, KS_>), dim3(grid2), dim3(256), 0, s, a, order, mid, n_plain, n_single, \
                       n_two, (int)heavy_wgs, (int)shared_wgs, (int)single_wgs);                                   \
    PCE_LAUNCH_CHECK("wave_os2");                                                                                  \
    return PCE_OK;                                                                                                 \
  }
  PCE_WOS2_CASE(1, 1) PCE_WOS2_CASE(1, 2) PCE_WOS2_CASE(1, 3) PCE_WOS2_CASE(1, 4)
  PCE_WOS2_CASE(2, 1) PCE_WOS2_CASE(2, 2) PCE_WOS2_CASE(2, 3) PCE_WOS2_CASE(2, 4)
#undef PCE_WOS2_CASE
  PCE_FAIL(PCE_EINVAL, "wave_os2: unsupported shape c_in=%d c_out=%d", a.c_in, a.c_out);
}

// The same dataflow for layers of 64 to 128 input and 65 to 128 output channels (fp16).  The weights of an offset
// (12 to 24 KB) come straight from the packed copy in L2, all KS x NB fragments of the offset requested before the
// first MFMA waits for one (in two batches where they would not leave three wavefronts per SIMD their registers);
// no workgroup copy of the centre weights, no barrier.  A bare loop lets the scheduler pair every fragment's load
// with its MFMA, two loads in flight: the layer took 39 us instead of 24, hence the scheduling barriers below.
template <int NB, int KS>
__global__ void __launch_bounds__(256, 2) wave_osw_kernel(TileArgs a, const int *__restrict__ perm,
                                                          const unsigned *__restrict__ rmask, int mid, long long n_main,
                                                          int heavy_wgs) {
  constexpr int PPR = KS * 2;   // 16-byte pieces per input row
  constexpr int NI = KS;        // global -> LDS instructions for the 32 centre rows
  constexpr int REGION0 = WaveLds<NB>::PIECES > 32 * PPR ? WaveLds<NB>::PIECES : 32 * PPR;
  constexpr int REGION = REGION0 > 256 ? REGION0 : 256;
  __shared__ __attribute__((aligned(16))) half8 Pl[4][REGION];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const half_t *Wp = (const half_t *)a.Wp;
  const long long wstep = (long long)a.k8_total * a.n_pad * 8;
  const bool heavy = (int)blockIdx.x < heavy_wgs;   // the same for the whole workgroup
  long long j0, j_end;
  if (heavy) {
    j0 = n_main + (long long)blockIdx.x * 32;
    j_end = a.n_rows;
  } else {
    const long long chunks = (n_main + 31) / 32;
    const long long chunk = chunks - 1 - (((long long)blockIdx.x - heavy_wgs) * 4 + wave);
    if (chunk < 0) return;
    j0 = chunk * 32;
    j_end = n_main;
  }
  const half_t *A = (const half_t *)a.A;
  const int orow = j0 + l32 < j_end ? perm[j0 + l32] : -1;
  const unsigned m = orow >= 0 ? rmask[orow] : 0u;
  unsigned u = m;
#pragma unroll
  for (int d = 1; d < 32; d <<= 1) u |= (unsigned)__shfl_xor((int)u, d, PCE_WAVE);
  unsigned todo = __builtin_amdgcn_readfirstlane(u);
  if (heavy) todo &= 0x11111111u << wave;   // see wave_os_kernel: a split that depends on the offset alone
  const bool centre = mid >= 0 && (!heavy || wave == 0);
  if (centre) {
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int e = it * 64 + lane, r = e / PPR, sl = e % PPR;
      const long long j = j0 + r < j_end ? j0 + r : j_end - 1;
      const half_t *gp = A + (long long)perm[j] * a.lda + ((sl ^ row_swizzle<PPR>(r)) * 8);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                       (__attribute__((address_space(3))) void *)&Pl[wave][it * 64], 16, 0, 0);
    }
  }
  int k_next = todo ? __ffs((int)todo) - 1 : -1;
  int nb_next = (k_next >= 0 && ((m >> k_next) & 1u)) ? a.nbr[(long long)k_next * a.n_rows + orow] : -1;
  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;
  // the weight fragments of an offset, GB K steps at a time: all of them up to 18 (72 registers), else two batches
  constexpr int GB = KS * NB <= 18 ? KS : (KS + 1) / 2;   // (the second batch of an odd KS is one step shorter)
  if (centre) {
    const half_t *Wk = Wp + mid * wstep + ((long long)g * a.n_pad + l32) * 8;
#pragma unroll
    for (int b0 = 0; b0 < KS; b0 += GB) {
      half8 wf[GB][NB];
#pragma unroll
      for (int s = 0; s < GB; ++s)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          if (b0 + s < KS) wf[s][nb] = *reinterpret_cast<const half8 *>(Wk + ((long long)(2 * (b0 + s)) * a.n_pad + nb * 32) * 8);
      // the global -> LDS copies have landed once nothing is outstanding; the fragment reads stay behind this statement
      // (the first batch of weights travels with the rows)
      if (b0 == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int s = 0; s < GB; ++s) {
        if (b0 + s < KS) {
          const half8 af = Pl[wave][l32 * PPR + ((2 * (b0 + s) + g) ^ row_swizzle<PPR>(l32))];
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[s][nb], af, acc[nb], 0, 0, 0);
        }
      }
    }
  }
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  while (k_next >= 0) {
    const int k = k_next, nrow = nb_next;
    todo &= todo - 1u;
    // every load of the offset goes out before anything waits for one (the scheduler, left alone, pairs each weight
    // fragment's load with its MFMA and keeps two in flight): the row fragments from a valid address, zeroed afterwards
    // where the row has no neighbour here, the first batch of weight fragments, the next offset's neighbour index
    half8 af[KS];
    const half_t *rp = A + (long long)(nrow >= 0 ? nrow : 0) * a.lda + g * 8;
#pragma unroll
    for (int s = 0; s < KS; ++s) af[s] = *reinterpret_cast<const half8 *>(rp + s * 16);
    const half_t *Wk = Wp + k * wstep + ((long long)g * a.n_pad + l32) * 8;
    k_next = todo ? __ffs((int)todo) - 1 : -1;
    const long long nidx = (k_next >= 0 && ((m >> k_next) & 1u)) ? (long long)k_next * a.n_rows + orow : 0;
#pragma unroll
    for (int b0 = 0; b0 < KS; b0 += GB) {
      half8 wf[GB][NB];
#pragma unroll
      for (int s = 0; s < GB; ++s)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          if (b0 + s < KS) wf[s][nb] = *reinterpret_cast<const half8 *>(Wk + ((long long)(2 * (b0 + s)) * a.n_pad + nb * 32) * 8);
      if (b0 == 0) {
        nb_next = a.nbr[nidx];
        __builtin_amdgcn_sched_barrier(0);
        if (!(k_next >= 0 && ((m >> k_next) & 1u))) nb_next = -1;
#pragma unroll
        for (int s = 0; s < KS; ++s) af[s] = nrow >= 0 ? af[s] : zero;
      } else {
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int s = 0; s < GB; ++s)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          if (b0 + s < KS) acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[s][nb], af[b0 + s], acc[nb], 0, 0, 0);
    }
  }
  if (heavy) {
    f32x16 *mine = reinterpret_cast<f32x16 *>(&Pl[wave][0]);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      __syncthreads();
      if (wave > 0) mine[lane] = acc[nb];
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int w2 = 1; w2 < 4; ++w2) {
          const f32x16 other = reinterpret_cast<const f32x16 *>(&Pl[w2][0])[lane];
#pragma unroll
          for (int j = 0; j < 16; ++j) acc[nb][j] += other[j];
        }
      }
    }
    if (wave > 0) return;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();   // every lane has read its centre fragments: the region becomes the output staging area
  float V[NB][2][8];
  gather_row_pieces<NB>(acc, V, g);
  if (a.bias || a.res || a.act) epilogue_row_pieces<half_t, NB, true>(V, a, orow, 0, g, a.act != PCE_ACT_NONE);
  store_rows_via_lds<half_t, NB>(V, Pl[wave], (half_t *)a.out, orow, a, 0, lane, l32, g, a.stream);
}

// shapes the K-stepped form takes: fp16, 64 or 96 channels in and 65 to 128 out, or 128 in and 65 to 96 out (the shapes
// it was measured to lead on; 128 -> 128 and 192 -> 128 ran 3 to 30 % behind deferred scatter)
// widths the K-stepped kernel is built for: 4 to 8 K steps of 16 input channels, 3 or 4 blocks of 32 output columns,
// at most 24 weight fragments per offset and lane (what leaves a wavefront its accumulators beside them)
static bool osw_widths(int c_in, int c_out) {
  const int ks = c_in / 16, nb = (c_out + 31) / 32;
  return c_in % 16 == 0 && c_out % 8 == 0 && ks >= 4 && ks <= 8 && nb >= 3 && nb <= 4 && ks * nb <= 24;
}
// widths of the ordered-row kernel proper (fp16) and of its fp32 form
static bool os_widths(int c_in, int c_out) { return c_in % 16 == 0 && c_in <= 64 && c_out % 8 == 0 && c_out <= 64; }
static bool os_f32_widths(int c_in, int c_out) { return c_in % 8 == 0 && c_in <= 32 && c_out % 8 == 0 && c_out <= 32; }
// layers pce_conv_fwd_oso takes, by dtype, widths, kernel volume and centre offset alone (it checks alignment and
// the packed weights besides): what the selector may answer PCE_DATAFLOW_OSO for
static bool oso_layer(int dtype, int c_in, int c_out, int kv, int mid) {
  if (kv < 1 || kv >= ORDER_MAX_KV || mid >= kv || c_in <= 0 || c_out <= 0) return false;
  if (dtype == PCE_F32) return mid >= 0 && os_f32_widths(c_in, c_out);
  return dtype == PCE_F16 && (os_widths(c_in, c_out) || osw_widths(c_in, c_out));
}

static bool wave_osw_ok(const TileArgs &a, int kv, int mid) {
  return a.Wp && a.a_vec && a.o_vec && osw_widths(a.c_in, a.c_out) && kv < ORDER_MAX_KV && mid < kv &&
         aligned16(a.bias) && aligned16(a.res);
}

// The same dataflow for very narrow fp32 layers (c_in = 8 KQ up to 32, c_out up to 32: the 16-channel fp32 layer
// of the reference's own test case).  Rows are 32 to 128 bytes, so nothing is staged on the way in: of a row's c_in
// values the lane with g = 0 holds the first half, the lane with g = 1 the second (KQ 16-byte loads each), and MFMA
// step (q, e) of v_mfma_f32_32x32x2_f32 contracts k = 4 q + e (lanes 0-31) with k = c_in / 2 + 4 q + e (lanes 32-63);
// the weights of an offset are read in that order, one value per lane and step, 128 contiguous bytes per half.
// (A form on v_mfma_f32_16x16x4_f32 -- half the MFMA time at 16 output columns -- with the offsets in a three-stage
// software pipeline measured 10.5 us where this kernel takes 9.8 on a 21 k-voxel surface cloud at 16 -> 16 channels,
// and 23.3 against 17.1 at 32 -> 32: the layer is bound by its gathers, not by the MFMA chain, and that form issues
// more of them per offset.)
template <int KQ>
__global__ void __launch_bounds__(256, 4) wave_os_f32_kernel(TileArgs a, const int *__restrict__ perm,
                                                             const unsigned *__restrict__ rmask, int mid, long long n_main,
                                                             int heavy_wgs) {
  constexpr int KH = 4 * KQ;   // values of a row per lane
  constexpr int REGION = WaveLds<1>::PIECES > 256 ? WaveLds<1>::PIECES : 256;   // output staging; one accumulator block of 64 lanes
  __shared__ __attribute__((aligned(16))) f32x4 Pl[4][REGION];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const bool heavy = (int)blockIdx.x < heavy_wgs;   // the same for the whole workgroup
  long long j0, j_end;
  if (heavy) {
    j0 = n_main + (long long)blockIdx.x * 32;
    j_end = a.n_rows;
  } else {
    const long long chunks = (n_main + 31) / 32;
    const long long chunk = chunks - 1 - (((long long)blockIdx.x - heavy_wgs) * 4 + wave);
    if (chunk < 0) return;
    j0 = chunk * 32;
    j_end = n_main;
  }
  const float *A = (const float *)a.A;
  const float *W = (const float *)a.W;
  const int orow = j0 + l32 < j_end ? perm[j0 + l32] : -1;
  const unsigned m = orow >= 0 ? rmask[orow] : 0u;
  unsigned u = m;
#pragma unroll
  for (int d = 1; d < 32; d <<= 1) u |= (unsigned)__shfl_xor((int)u, d, PCE_WAVE);
  unsigned todo = __builtin_amdgcn_readfirstlane(u);   // offsets any of the 32 rows has: the same in every lane
  if (heavy) todo &= 0x11111111u << wave;               // see wave_os_kernel: a split that depends on the offset alone
  const bool centre = !heavy || wave == 0;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  // this lane's half of a row; the weights of offset k in the order the MFMA steps contract them
  // (every load is issued by every lane, from a valid address, and zeroed afterwards where it does not count: a load
  // under a lane condition becomes a branch with its own wait, and the loads of an offset would go out in pairs)
  auto load_row = [&](int row, f32x4 (&af)[KQ]) {
    const float *p = A + (long long)(row >= 0 ? row : 0) * a.lda + g * KH;
#pragma unroll
    for (int q = 0; q < KQ; ++q) af[q] = *reinterpret_cast<const f32x4 *>(p + 4 * q);
    if (row < 0) {
#pragma unroll
      for (int q = 0; q < KQ; ++q) af[q] = zero4;
    }
  };
  auto load_weights = [&](int k, float (&wf)[KH]) {
    const float *Wk = W + ((long long)k * a.c_in + g * KH) * a.c_out + (l32 < a.c_out ? l32 : 0);
#pragma unroll
    for (int s = 0; s < KH; ++s) wf[s] = Wk[(long long)s * a.c_out];
    if (l32 >= a.c_out) {
#pragma unroll
      for (int s = 0; s < KH; ++s) wf[s] = 0.f;
    }
  };
  f32x16 acc[1];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[0][j] = 0.f;
  int k_next = todo ? __ffs((int)todo) - 1 : -1;
  int nb_next = (k_next >= 0 && ((m >> k_next) & 1u)) ? a.nbr[(long long)k_next * a.n_rows + orow] : -1;
  if (centre) {
    f32x4 af[KQ];
    float wf[KH];
    load_row(orow, af);
    load_weights(mid, wf);
#pragma unroll
    for (int s = 0; s < KH; ++s) acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[s], af[s / 4][s % 4], acc[0], 0, 0, 0);
  }
  while (k_next >= 0) {
    const int k = k_next, nrow = nb_next;
    todo &= todo - 1u;
    f32x4 af[KQ];
    float wf[KH];
    load_row(nrow, af);
    load_weights(k, wf);
    k_next = todo ? __ffs((int)todo) - 1 : -1;
    nb_next = (k_next >= 0 && ((m >> k_next) & 1u)) ? a.nbr[(long long)k_next * a.n_rows + orow] : -1;
#pragma unroll
    for (int s = 0; s < KH; ++s) acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[s], af[s / 4][s % 4], acc[0], 0, 0, 0);
  }
  if (heavy) {
    // wavefronts 1..3 hand their accumulators to wavefront 0 through their own regions
    f32x16 *mine = reinterpret_cast<f32x16 *>(&Pl[wave][0]);
    if (wave > 0) mine[lane] = acc[0];
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w2 = 1; w2 < 4; ++w2) {
      const f32x16 other = reinterpret_cast<const f32x16 *>(&Pl[w2][0])[lane];
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[0][j] += other[j];
    }
  }
  float V[1][2][8];
  gather_row_pieces<1>(acc, V, g);
  if (a.bias || a.res || a.act) epilogue_row_pieces<float, 1, true>(V, a, orow, 0, g, a.act != PCE_ACT_NONE);
  store_rows_via_lds<float, 1>(V, Pl[wave], (float *)a.out, orow, a, 0, lane, l32, g, a.stream);
}

// shapes the fp32 form takes
static bool wave_os_f32_ok(const TileArgs &a, int kv, int mid) {
  return a.a_vec && a.o_vec && a.c_in % 8 == 0 && a.c_in <= 32 && a.c_out % 8 == 0 && a.c_out <= 32 && kv < ORDER_MAX_KV &&
         mid >= 0 && mid < kv && aligned16(a.bias) && aligned16(a.res);
}

// shapes the ordered-row kernel takes: fp16, at most 64 channels either side, a centre offset
static bool wave_os_ok(const TileArgs &a, int kv, int mid) {
  return wave_gemm_ok(a, 2) && kv < ORDER_MAX_KV && mid < kv && aligned16(a.bias) && aligned16(a.res);
}

extern "C" int pce_conv_fwd_oso(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid, const int32_t *nbr,
                                const int32_t *order, const int64_t *order_counts, const pce_epilogue_t *epilogue,
                                pce_stream_t stream) {
  if (!order_counts) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: null order counts");
  const int64_t n_heavy = order_counts[0], n_nonzero = order_counts[1], n_single = order_counts[2];
  int rc = check_common("pce_conv_fwd_oso", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc) return rc;
  if (!nbr || !order) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: null neighbour table or row order");
  Epi e;
  if ((rc = read_epilogue("pce_conv_fwd_oso", epilogue, out, &e, c_in, c_out))) return rc;
  const bool f32 = dtype == PCE_F32;
  TileArgs a = f32 ? base_args<float>(in, w, wp, kv, c_in, c_out, e.lda) : base_args<half_t>(in, w, wp, kv, c_in, c_out, e.lda);
  if (f32)
    set_out<float>(&a, out, false, n_out, e.ldo);
  else
    set_out<half_t>(&a, out, false, n_out, e.ldo);
  set_epi(&a, e);
  const bool wide = !f32 && wave_osw_ok(a, kv, mid);
  if (!wide && (f32 ? !wave_os_f32_ok(a, kv, mid) : !wave_os_ok(a, kv, mid)))
    PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: takes layers in fp16 of at most 64 channels (multiples of 16 in, 8 out, packed "
                         "weights), of 64..128 -> 65..128 channels with c_in / 16 * ceil(c_out / 32) <= 24, or submanifold layers in fp32 "
                         "of at most 32 (multiples of 8), 16-byte aligned rows, kernel volumes up to 31; got dtype %d, %d -> %d channels, "
                         "kv %d, mid %d", (int)dtype, (int)c_in, (int)c_out, (int)kv, (int)mid);
  if (n_heavy < 0 || n_heavy > n_out) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: n_heavy=%lld outside [0, n_out]", (long long)n_heavy);
  if (n_nonzero >= 0 && (n_nonzero < n_heavy || n_nonzero > n_out))
    PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: n_nonzero=%lld outside [n_heavy, n_out]", (long long)n_nonzero);
  if (n_nonzero >= 0 && n_single >= 0 && n_single > n_nonzero - n_heavy)
    PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: n_single=%lld exceeds the %lld rows with one or two neighbours", (long long)n_single, (long long)(n_nonzero - n_heavy));
  if ((uintptr_t)order & 15) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: the order array must be 16-byte aligned");
  a.nbr = nbr;
  a.n_rows = n_out;
  // Chunks of rows with two neighbours or more (the end of the order: rows with two, then rows with three or more)
  // take a workgroup each, its four wavefronts splitting the offsets; the chunks before them a wavefront each.  A
  // caller that states only the count of rows with three or more gets those split.  (Splitting the rows with two as
  // well: 15.1 -> 10.4 us on a 21 k-voxel surface cloud in fp32 16 -> 16, 14.3 -> 11.9 in fp16 64 -> 64, where the
  // few chunks of such rows, each with a union of eight offsets or more walked by one wavefront, ended last; 0-8 %
  // on the levels of a LiDAR pyramid.)
  const long long n_split = (n_nonzero >= 0 && n_single >= 0) ? n_nonzero - n_single : n_heavy;
  const long long n_main = n_out - n_split;
  const long long heavy_wgs = pce_div_up(n_split, 32), main_wgs = pce_div_up(pce_div_up(n_main, 32), 4);
  if (heavy_wgs + main_wgs >= (1ll << 31) - 8) PCE_FAIL(PCE_ECAPACITY, "pce_conv_fwd_oso: %lld rows exceed the grid limit", (long long)n_out);
  const unsigned grid = (unsigned)(heavy_wgs + main_wgs);
  const int *perm = order;
  const unsigned *rmask = (const unsigned *)(order + n_out);
  if (f32) {
    hipStream_t s32 = (hipStream_t)stream;
#define PCE_WOS32_CASE(KQ_)                                                                                       \
  if (c_in == 8 * KQ_) {                                                                                           \
    hipLaunchKernelGGL((wave_os_f32_kernel<KQ_>), dim3(grid), dim3(256), 0, s32, a, perm, rmask, (int)mid, n_main,  \
                       (int)heavy_wgs);                                                                            \
    PCE_LAUNCH_CHECK("wave_os_f32");                                                                               \
    return PCE_OK;                                                                                                 \
  }
    PCE_WOS32_CASE(1) PCE_WOS32_CASE(2) PCE_WOS32_CASE(3) PCE_WOS32_CASE(4)
#undef PCE_WOS32_CASE
    PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: unsupported fp32 width c_in=%d", (int)c_in);
  }
  const int nb = (c_out + 31) / 32, ks = c_in / 16;
  if (a.n_pad != nb * 32 || a.k8_total != 2 * ks)
    PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: packed weights are %d x %d fragments per offset, expected %d x %d", a.k8_total, a.n_pad, 2 * ks, nb * 32);
  hipStream_t s = (hipStream_t)stream;
  if (wide) {
#define PCE_WOSW_CASE(NB_, KS_)                                                                              \
  if (nb == NB_ && ks == KS_) {                                                                              \
    hipLaunchKernelGGL((wave_osw_kernel<NB_, KS_>), dim3(grid), dim3(256), 0, s, a, perm, rmask, (int)mid, n_main,  \
                       (int)heavy_wgs);                                                                      \
    PCE_LAUNCH_CHECK("wave_osw");                                                                            \
    return PCE_OK;                                                                                           \
  }
    PCE_WOSW_CASE(3, 4) PCE_WOSW_CASE(3, 5) PCE_WOSW_CASE(3, 6) PCE_WOSW_CASE(3, 7) PCE_WOSW_CASE(3, 8)
    PCE_WOSW_CASE(4, 4) PCE_WOSW_CASE(4, 5) PCE_WOSW_CASE(4, 6)
#undef PCE_WOSW_CASE
    PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: unsupported shape c_in=%d c_out=%d", (int)c_in, (int)c_out);
  }
  // Clouds whose rows mostly have no neighbour, few of them two or more, and small enough that every workgroup of the
  // three-kind kernel is resident at once (four per CU): that kernel, the bulk streamed in storage order.  It shortens
  // the chains of dependent trips to memory that set the duration of a launch of one round of wavefronts; it
  // multiplies the rows with neighbours twice, which costs more than that saves once the rows come in several rounds.
  // Needs the counts of rows with any neighbour and with exactly one; a caller that does not state them (-1), a
  // layer without a centre offset, fewer than 48 input channels (its shared rows are walked by one wavefront per
  // 16 input channels) and other clouds take the kernel that visits every row through the order.  This kernel /
  // that one, 64 -> 64 channels: 11.2 / 11.8 us on a 150 k-voxel LiDAR scan (4 % of the rows with two neighbours or
  // more), 8.5 / 10.0 on a 100 k scan; 32.4 / 32.4 on four scans in a batch (that kernel either way); 32 -> 32: 7.6 /
  // 7.8 on the 150 k scan, 6.6 / 5.7 on the 100 k scan, 5.9 / 4.7 on half of it; 16 -> 32: 7.0 / 6.7.
  if (mid >= 0 && kv <= PCE_ORDER_SREC_KV && ks >= 3 && n_nonzero >= 0 && n_single >= 0 && 2 * n_nonzero <= n_out &&
      n_nonzero - n_single <= PCE_ORDER_SREC_ROWS(n_out) && 8 * (n_nonzero - n_single) <= n_out &&
      os2_workgroups(n_out, n_nonzero, n_single, n_heavy, nb) <= 4ll * cu_count() && stage_on(12))
    return launch_wave_os2(a, order, (int)mid, n_out, n_nonzero, n_single, n_heavy, nb, ks, s);
#define PCE_WOS_CASE(NB_, KS_)                                                                              \
  if (nb == NB_ && ks == KS_) {                                                                              \
    hipLaunchKernelGGL((wave_os_kernel<NB_, KS_>), dim3(grid), dim3(256), 0, s, a, perm, rmask, (int)mid, n_main,   \
                       (int)heavy_wgs);                                                                      \
    PCE_LAUNCH_CHECK("wave_os");                                                                             \
    return PCE_OK;                                                                                           \
  }
  PCE_WOS_CASE(1, 1) PCE_WOS_CASE(1, 2) PCE_WOS_CASE(1, 3) PCE_WOS_CASE(1, 4)
  PCE_WOS_CASE(2, 1) PCE_WOS_CASE(2, 2) PCE_WOS_CASE(2, 3) PCE_WOS_CASE(2, 4)
#undef PCE_WOS_CASE
  PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_oso: unsupported shape c_in=%d c_out=%d", (int)c_in, (int)c_out);
}

template <typename T>
static int dense_impl(const void *in, const void *w, const void *wp, void *out, int64_t n, int c_in, int c_out,
                      const Epi &e, hipStream_t s) {
  TileArgs a = base_args<T>(in, w, wp, 1, c_in, c_out);
  set_out<T>(&a, out, false, n);
  set_epi(&a, e);
  a.n_rows = n;
  a.mode = MODE_DENSE;
  a.epi = EPI_ROWS;
  // narrow fp16 layers: the stream workgroups of the three-kind ordered kernel alone (64 consecutive rows per
  // wavefront, weights once per workgroup through LDS): 7.1 us on 150 k rows of 64 -> 64 channels, the tile kernel 8.3
  if (sizeof(T) == 2 && wave_os_ok(a, 1, 0) && stage_on(12))
    return launch_wave_os2(a, nullptr, 0, n, 0, 0, 0, (c_out + 31) / 32, c_in / 16, s);
  return launch_tile<T>(a, pce_div_up(n, 128), s);
}

extern "C" int pce_conv_fwd_dense(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n,
                                  int32_t c_in, int32_t c_out, const pce_epilogue_t *epilogue, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_dense", in, w, out, dtype, n, n, c_in, c_out, 1, -1);
  if (rc) return rc;
  Epi e;
  if ((rc = read_epilogue("pce_conv_fwd_dense", epilogue, out, &e))) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16) return dense_impl<half_t>(in, w, wp, out, n, c_in, c_out, e, s);
  return dense_impl<float>(in, w, wp, out, n, c_in, c_out, e, s);
}

// Kernel gradient: gw[kp][ci][co] = sum over the pairs p of offset kp of in[imap[p]][ci] * gout[omap[p]][co]
// (ConvolutionBackwardD1's per-offset GEMM, backend/spconv.cu:400-629): per offset a GEMM whose reduction
// runs over the pairs.  A workgroup owns a BLK x BLK block of (ci, co) and a run of consecutive 128-pair
// quanta (then 128-row tiles of the centre offset); its four wavefronts hold (BLK/2) x (BLK/2) each in
// fp32 MFMA accumulators (v_mfma_f32_32x32x2_f32, also for fp16 tensors: they are widened when staged, and
// with the pair index as the reduction index the fp16 MFMA would need its operands transposed).  Rows
// are staged in LDS 32 pairs at a time.  The accumulators are added to the fp32 result with atomics only
// when the offset changes or the run ends: one atomic per element per run instead of one per quantum (the
// order of the additions, and so the last bits, still vary from run to run).
#define WGRAD_KP 32   // pairs per LDS stage

// PER consecutive channels of one row as fp32 (zeros for a missing row or past the last channel); the vector
// form needs a channel count that is a multiple of the 16-byte vector, so a vector lies inside the row or past it
template <typename T, int PER>
__device__ __forceinline__ void wgrad_fetch(float (&v)[PER], const T *__restrict__ base, int row, int c_total, int c0,
                                            bool vec) {
  constexpr int EPV = 16 / (int)sizeof(T);
  typedef typename VecOfC<T, EPV>::type V;
  if (vec) {
#pragma unroll
    for (int q = 0; q < PER / EPV; ++q) {
      V x;
#pragma unroll
      for (int j = 0; j < EPV; ++j) x[j] = (T)0;
      if (row >= 0 && c0 + q * EPV < c_total) x = *reinterpret_cast<const V *>(base + (long long)row * c_total + c0 + q * EPV);
#pragma unroll
      for (int j = 0; j < EPV; ++j) v[q * EPV + j] = (float)x[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < PER; ++j) v[j] = (row >= 0 && c0 + j < c_total) ? (float)base[(long long)row * c_total + c0 + j] : 0.f;
  }
}
// fp16 tensors: the same block / run structure on the fp16 MFMA (32x32x16: 8 consecutive pairs per lane
// and operand).  Its operands are [channel][pair], the transpose of how rows lie in memory.  A thread
// fetches the same 8 channels of 4 consecutive pairs (four 16-byte loads), regroups them in registers into
// 8 channel rows of 4 pairs and writes each as one 8-byte LDS store; the MFMA fragments are then 16
// contiguous bytes.  A stage holds KP pairs (64 for 128-wide blocks, the whole tile for 64-wide ones) and
// channel rows lie KP + 8 halfs apart, which keeps both the 8-byte stores of a half wavefront and the
// 16-byte fragment reads of 16 consecutive channels in distinct banks.
template <int BLK>
__global__ void __launch_bounds__(BLK == 256 ? 512 : 256, BLK == 256 ? 1 : 2) wgrad_f16_kernel(const half_t *__restrict__ in, const half_t *__restrict__ gout,
                                                        long long n_rows, int c_in, int c_out, int kv, int mid,
                                                        const int *__restrict__ imap, const int *__restrict__ omap,
                                                        const int *__restrict__ kpos, const int *__restrict__ qkpos,
                                                        long long pair_tiles, long long tiles, int run, int ci_blocks,
                                                        int co_blocks, float *__restrict__ gw) {
  constexpr int NT = BLK == 256 ? 512 : 256;  // threads: 4 x 2 wavefronts on a 256-wide block, else 2 x 2
  constexpr int WR = NT / 128;                // wavefronts along ci (two along co)
  constexpr int RI = BLK / (32 * WR), RJ = BLK / 64;  // 32 x 32 MFMA tiles per wavefront along ci, co
  constexpr int KP = BLK == 64 ? 128 : 64;    // pairs per stage
  constexpr int PG = KP / 4;                  // groups of 4 pairs; PG * (BLK / 8) == NT threads
  constexpr int LD = KP + 8;                  // halfs per channel row
  static_assert(PG * (BLK / 8) == NT, "one thread per (4 pairs, 8 channels) cell of a stage");
  __shared__ __attribute__((aligned(16))) half_t At[BLK][LD];
  __shared__ __attribute__((aligned(16))) half_t Gt[BLK][LD];
  __shared__ int rows_in[4][128], rows_out[4][128];  // row indices of a tile, a ring of four tiles
  __shared__ int tile_w[4];                          // and its offset (-1: none)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int wr = wave >> 1, wc = wave & 1;
  // workgroups are dealt to the 8 XCDs in turn: all (ci, co) blocks of one run of tiles go to the same XCD,
  // whose L2 then serves the rows they gather in common; groups past the last run find no tile
  const long long slot = blockIdx.x >> 3;
  const int rest = (int)(slot % (ci_blocks * co_blocks));
  const long long grp = (slot / (ci_blocks * co_blocks)) * 8 + (blockIdx.x & 7);
  const int ci0 = (rest / co_blocks) * BLK, co0 = (rest % co_blocks) * BLK;

  f32x16 acc[RI][RJ];
#pragma unroll
  for (int i = 0; i < RI; ++i)
#pragma unroll
    for (int j = 0; j < RJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  int cur = -1;
  auto flush = [&](int widx) {
    float *dst = gw + (long long)widx * c_in * c_out;
#pragma unroll
    for (int i = 0; i < RI; ++i)
#pragma unroll
      for (int j = 0; j < RJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          int ci = ci0 + wr * (BLK / WR) + i * 32 + (e / 4) * 8 + g * 4 + (e % 4);
          int co = co0 + wc * (BLK / 2) + j * 32 + l32;
          float v = acc[i][j][e];
          if (ci < c_in && co < c_out && v != 0.f) unsafeAtomicAdd(dst + (long long)ci * c_out + co, v);
          acc[i][j][e] = 0.f;
        }
  };
  const bool vec_in = (c_in % 8 == 0) && (((uintptr_t)in) & 15) == 0;
  const bool vec_out = (c_out % 8 == 0) && (((uintptr_t)gout) & 15) == 0;
  const int pg = threadIdx.x % PG, cg = threadIdx.x / PG;  // the thread's cell: pairs 4 pg .. +3, channels 8 cg .. +7
  // one operand's 8 channels of one pair as 4 dwords (channels 2d, 2d + 1 in dword d)
  auto fetch_row = [&](const half_t *base, int row, int c, int c0, bool vec) -> u32x4 {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < 0 || c0 + cg * 8 >= c) return v;
    const half_t *src = base + (long long)row * c + c0 + cg * 8;
    if (vec) return *reinterpret_cast<const u32x4 *>(src);  // c is a multiple of 8: the 8 channels lie inside the row
    half8 h = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (c0 + cg * 8 + j < c) h[j] = src[j];
    return *reinterpret_cast<u32x4 *>(&h);
  };
  // [4 pairs][8 channels] in registers -> 8 channel rows of 4 pairs in LDS
  auto put = [&](half_t (*dst)[LD], const u32x4 (&v)[4]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      u32x2 even, odd;
      even[0] = __builtin_amdgcn_perm(v[1][d], v[0][d], 0x05040100u);
      even[1] = __builtin_amdgcn_perm(v[3][d], v[2][d], 0x05040100u);
      odd[0] = __builtin_amdgcn_perm(v[1][d], v[0][d], 0x07060302u);
      odd[1] = __builtin_amdgcn_perm(v[3][d], v[2][d], 0x07060302u);
      *reinterpret_cast<u32x2 *>(&dst[cg * 8 + 2 * d][pg * 4]) = even;
      *reinterpret_cast<u32x2 *>(&dst[cg * 8 + 2 * d + 1][pg * 4]) = odd;
    }
  };
  const long long t_begin = grp * run;
  const long long t_end = (grp + 1) * run < tiles ? (grp + 1) * run : tiles;
  if (t_begin >= t_end) return;  // uniform
  constexpr int SPT = 128 / KP;  // stages per tile
  const int n_stage = (int)(t_end - t_begin) * SPT;

  // The loop runs over the stages of all tiles of the run as one sequence.  What stage s multiplies was
  // gathered during stages s - 2 and s - 1 (two register sets alternate) from row indices published in LDS at
  // the top of stage s - 2 and loaded from the map during stage s - 3, so neither the map read nor the gather
  // is waited for at a tile boundary, and two stages of rows are in flight while one is multiplied.
  int lw = 0;  // offset of the tile whose rows are loaded next (tiles of a run come in offset order)
  if (t_begin < pair_tiles)
    for (int i = 0; i < kv; ++i) lw += ((long long)qkpos[i + 1] <= t_begin * 128) ? 1 : 0;
  int nri = -1, nro = -1, nw = -1;
  auto load_rows = [&](long long tile) {  // map entries of a tile into registers
    nri = nro = nw = -1;
    if (tile >= t_end) return;
    if (tile < pair_tiles) {
      const long long q0 = tile * 128;
      while (lw < kv && (long long)qkpos[lw + 1] <= q0) ++lw;
      if (lw >= kv) return;
      nw = lw;
      const long long p = q0 - qkpos[lw] + kpos[lw] + threadIdx.x;
      if (threadIdx.x < 128 && p < (long long)kpos[lw + 1]) {
        nri = imap[p];
        nro = omap[p];
      }
    } else {
      nw = mid;
      const long long row = (tile - pair_tiles) * 128 + threadIdx.x;
      if (threadIdx.x < 128 && row < n_rows) nri = nro = (int)row;
    }
  };
  auto store_rows = [&](int buf) {
    if (threadIdx.x < 128) {
      rows_in[buf][threadIdx.x] = nri;
      rows_out[buf][threadIdx.x] = nro;
    }
    if (threadIdx.x == 0) tile_w[buf] = nw;
  };
  u32x4 va0[4], vg0[4], va1[4], vg1[4];
  auto fetch = [&](u32x4 (&va)[4], u32x4 (&vg)[4], int stage) {
    const int buf = (stage / SPT) & 3, p0 = (stage % SPT) * KP;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      va[q] = fetch_row(in, rows_in[buf][p0 + pg * 4 + q], c_in, ci0, vec_in);
      vg[q] = fetch_row(gout, rows_out[buf][p0 + pg * 4 + q], c_out, co0, vec_out);
    }
  };
  auto body = [&](int v, u32x4 (&va)[4], u32x4 (&vg)[4]) {
    if ((v + 2) % SPT == 0) store_rows(((v + 2) / SPT) & 3);  // rows of the tile of stage v + 2, loaded a stage ago
    __syncthreads();  // the MFMAs of the previous stage have read their operands
    put(At, va);
    put(Gt, vg);
    __syncthreads();
    if (v % SPT == 0) {  // first stage of a tile: do its sums go to another offset's block than the last tile's?
      const int w = __builtin_amdgcn_readfirstlane(tile_w[(v / SPT) & 3]);
      if (w >= 0 && w != cur) {
        if (cur >= 0) flush(cur);
        cur = w;
      }
    }
    if ((v + 3) % SPT == 0) load_rows(t_begin + (v + 3) / SPT);
    if (v + 2 < n_stage) fetch(va, vg, v + 2);
#pragma unroll
    for (int k0 = 0; k0 < KP; k0 += 16) {
      half8 av[RI], bv[RJ];
#pragma unroll
      for (int i = 0; i < RI; ++i) av[i] = *reinterpret_cast<const half8 *>(&At[wr * (BLK / WR) + i * 32 + l32][k0 + 8 * g]);
#pragma unroll
      for (int j = 0; j < RJ; ++j) bv[j] = *reinterpret_cast<const half8 *>(&Gt[wc * (BLK / 2) + j * 32 + l32][k0 + 8 * g]);
#pragma unroll
      for (int i = 0; i < RI; ++i)
#pragma unroll
        for (int j = 0; j < RJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
  };
  // what stages -3, -2 and -1 would have done for stages 0 and 1
  load_rows(t_begin);
  store_rows(0);
  __syncthreads();
  if (SPT == 1) load_rows(t_begin + 1);
  fetch(va0, vg0, 0);
  if (SPT == 1) store_rows(1);
  __syncthreads();
  load_rows(t_begin + 2 / SPT);
  if (1 < n_stage) fetch(va1, vg1, 1);
  for (int v = 0; v < n_stage; v += 2) {
    body(v, va0, vg0);
    if (v + 1 < n_stage) body(v + 1, va1, vg1);
  }
  if (cur >= 0) flush(cur);
}

template <typename T, int BLK>
__global__ void __launch_bounds__(256) wgrad_kernel(const T *__restrict__ in, const T *__restrict__ gout, long long n_rows,
                                                    int c_in, int c_out, int kv, int mid, const int *__restrict__ imap,
                                                    const int *__restrict__ omap, const int *__restrict__ kpos,
                                                    const int *__restrict__ qkpos, long long pair_tiles, long long tiles,
                                                    int run, int ci_blocks, int co_blocks, float *__restrict__ gw) {
  constexpr int R = BLK / 64;              // 32x32 MFMA tiles per wavefront and dimension
  constexpr int LD = BLK + 32;             // row stride in floats: the two k rows an MFMA reads fall into different banks
  constexpr int PER = BLK / 8;             // channels a thread stages per row
  __shared__ float As[WGRAD_KP][LD];
  __shared__ float Gs[WGRAD_KP][LD];
  __shared__ int rows_in[128], rows_out[128];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int wr = wave >> 1, wc = wave & 1;
  // workgroups are dealt to the 8 XCDs in turn: all (ci, co) blocks of one run of tiles go to the same XCD,
  // whose L2 then serves the rows they gather in common; groups past the last run find no tile
  const long long slot = blockIdx.x >> 3;
  const int rest = (int)(slot % (ci_blocks * co_blocks));
  const long long grp = (slot / (ci_blocks * co_blocks)) * 8 + (blockIdx.x & 7);
  const int ci0 = (rest / co_blocks) * BLK, co0 = (rest % co_blocks) * BLK;

  f32x16 acc[R][R];
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  int cur = -1;  // offset the accumulators belong to

  auto flush = [&](int widx) {
    float *dst = gw + (long long)widx * c_in * c_out;
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
      for (int j = 0; j < R; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          int ci = ci0 + wr * (BLK / 2) + i * 32 + (e / 4) * 8 + g * 4 + (e % 4);
          int co = co0 + wc * (BLK / 2) + j * 32 + l32;
          float v = acc[i][j][e];
          if (ci < c_in && co < c_out && v != 0.f) unsafeAtomicAdd(dst + (long long)ci * c_out + co, v);
          acc[i][j][e] = 0.f;
        }
  };

  // 16-byte loads when a thread's channels lie inside the tensor and its rows are 16-byte multiples
  constexpr int EPV = 16 / (int)sizeof(T);
  const bool vec_in = (c_in % EPV == 0) && (((uintptr_t)in) & 15) == 0;
  const bool vec_out = (c_out % EPV == 0) && (((uintptr_t)gout) & 15) == 0;
  const long long t_end = (grp + 1) * run < tiles ? (grp + 1) * run : tiles;
  for (long long tile = grp * run; tile < t_end; ++tile) {
    int widx;
    __syncthreads();  // rows_in / rows_out of the previous tile are no longer read
    if (tile < pair_tiles) {
      long long q0 = tile * 128;
      widx = 0;
      for (int i = 0; i < kv; ++i) widx += ((long long)qkpos[i + 1] <= q0) ? 1 : 0;
      if (widx >= kv) break;  // uniform
      if (threadIdx.x < 128) {
        long long p = q0 - qkpos[widx] + kpos[widx] + threadIdx.x;
        bool ok = p < (long long)kpos[widx + 1];
        rows_in[threadIdx.x] = ok ? imap[p] : -1;
        rows_out[threadIdx.x] = ok ? omap[p] : -1;
      }
    } else {  // centre offset of a submanifold layer: every row pairs with itself
      widx = mid;
      if (threadIdx.x < 128) {
        long long row = (tile - pair_tiles) * 128 + threadIdx.x;
        rows_in[threadIdx.x] = rows_out[threadIdx.x] = row < n_rows ? (int)row : -1;
      }
    }
    if (cur >= 0 && widx != cur) flush(cur);
    cur = widx;
    __syncthreads();
    // stage 32 rows x BLK channels of both operands as fp32: PER consecutive channels per thread and matrix.
    // The rows of stage s+1 are requested before the MFMAs of stage s.
    const int r = threadIdx.x / 8, c = (threadIdx.x % 8) * PER;
    float va[PER], vg[PER];
    auto fetch = [&](int p0) {
      const int ri = rows_in[p0 + r], ro = rows_out[p0 + r];
      wgrad_fetch<T, PER>(va, in, ri, c_in, ci0 + c, vec_in);
      wgrad_fetch<T, PER>(vg, gout, ro, c_out, co0 + c, vec_out);
    };
    fetch(0);
    for (int p0 = 0; p0 < 128; p0 += WGRAD_KP) {
      __syncthreads();  // the MFMAs of the previous stage have read their operands
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        As[r][c + j] = va[j];
        Gs[r][c + j] = vg[j];
      }
      __syncthreads();
      if (p0 + WGRAD_KP < 128) fetch(p0 + WGRAD_KP);
#pragma unroll 4
      for (int k = 0; k < WGRAD_KP; k += 2) {
        float av[R], bv[R];
#pragma unroll
        for (int i = 0; i < R; ++i) av[i] = As[k + g][wr * (BLK / 2) + i * 32 + l32];
#pragma unroll
        for (int j = 0; j < R; ++j) bv[j] = Gs[k + g][wc * (BLK / 2) + j * 32 + l32];
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
          for (int j = 0; j < R; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
      }
    }
  }
  if (cur >= 0) flush(cur);
}

extern "C" int pce_conv_wgrad(const void *in, const void *gout, int32_t dtype, int64_t n_in, int64_t n_out, int32_t c_in,
                              int32_t c_out, int32_t kv, int32_t mid, const int32_t *imap, const int32_t *omap,
                              const int32_t *kpos, const int32_t *qkpos, int64_t qsum, float *gw, pce_stream_t stream) {
  int rc = check_common("pce_conv_wgrad", in, gout, gw, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_wgrad", qsum))) return rc;
  if (!kpos || !qkpos || (qsum > 0 && (!imap || !omap))) PCE_FAIL(PCE_EINVAL, "pce_conv_wgrad: null map pointer");
  hipStream_t s = (hipStream_t)stream;
  long long total = (long long)kv * c_in * c_out;
  hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)pce_div_up(total, 1024)), dim3(256), 0, s, gw, total);
  PCE_LAUNCH_CHECK("zero_f32");
  long long pair_tiles = qsum / PCE_QUANTUM;
  long long tiles = pair_tiles + (mid >= 0 ? pce_div_up(n_out, 128) : 0);
  if (tiles <= 0) return PCE_OK;
  // 128 x 128 blocks of (ci, co) for wide layers, 64 x 64 otherwise.  Every run of tiles ends with one atomic
  // per element of its block, and on layers of 10^5 rows those atomics cost as much as the tiles: runs are
  // made long enough to leave one workgroup per CU, more only where the tiles are many (measured on the
  // layers of a 100k-voxel U-Net: 128 -> 128, 5111 tiles: 135 / 87 / 98 / 113 / 168 us at 128 / 256 / 512 /
  // 1024 / 2048 workgroups; 256 -> 256, four blocks, 5111 tiles: 498 / 279 / 268 / 246 / 247 us)
  const int blk = (c_in > 64 || c_out > 64) ? 128 : 64;
  const int ci_blocks = (c_in + blk - 1) / blk, co_blocks = (c_out + blk - 1) / blk;
  const long long tile_blocks = tiles * ci_blocks * co_blocks;
  long long target_wgs = 256;
  if (blk == 128 && ci_blocks * co_blocks >= 4) target_wgs = 1024;
  if (blk == 64 && tile_blocks >= 2048) target_wgs = 512;
  long long run = tile_blocks / target_wgs;
  run = run < 1 ? 1 : (run > 256 ? 256 : run);
  long long blocks = pce_div_up(pce_div_up(tiles, run), 8) * 8 * ci_blocks * co_blocks;
  if (blocks >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "pce_conv_wgrad: %lld workgroups exceed the grid limit", blocks);
#define PCE_WGRAD(T_, BLK_)                                                                                              \
  hipLaunchKernelGGL((wgrad_kernel<T_, BLK_>), dim3((unsigned)blocks), dim3(256), 0, s, (const T_ *)in, (const T_ *)gout, \
                     (long long)n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, pair_tiles, tiles, (int)run,       \
                     ci_blocks, co_blocks, gw)
#define PCE_WGRAD16(BLK_)                                                                                            \
  hipLaunchKernelGGL((wgrad_f16_kernel<BLK_>), dim3((unsigned)blocks), dim3(256), 0, s, (const half_t *)in,            \
                     (const half_t *)gout, (long long)n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, pair_tiles, \
                     tiles, (int)run, ci_blocks, co_blocks, gw)
  if (dtype == PCE_F16 && blk == 128)
    PCE_WGRAD16(128);
  else if (dtype == PCE_F16)
    PCE_WGRAD16(64);
  else if (blk == 128)
    PCE_WGRAD(float, 128);
  else
    PCE_WGRAD(float, 64);
#undef PCE_WGRAD
#undef PCE_WGRAD16
  PCE_LAUNCH_CHECK("wgrad");
  return PCE_OK;
}

// ---- batch normalisation over the rows of a feature matrix (script/batchnorm.py:7-10) -----------------
// Two kernels carry the forward and the backward pass of nn.BatchNorm1d on [n, c]:
//   column sums:   out[j] = sum_r a[r][j],  out[c + j] = sum_r a[r][j] * b[r][j]   (b = a when b is null)
//     forward statistics from (x, x): sum and sum of squares; backward from (dy, x): sum dy, sum dy*x
//   column affine: y[r][j] = act(x[r][j] * kx[j] + d[r][j] * kd[j] + k0[j])         (d may be null)
//     forward: y = x * (w*rstd) + (b - mean*w*rstd); backward: dx = dy*k1 + x*k2 + k3
// The per-channel coefficients between them are c-element vector arithmetic left to the caller.
// A thread owns VEC adjacent columns (one 16-byte vector when the layout allows) and walks down the rows in
// steps of the grid, 8 rows requested at a time; sums are accumulated in fp32 over those 8 rows, then in fp64:
// per workgroup through LDS, across workgroups by a second kernel over the per-workgroup partial sums (no
// atomics: same bits every run).  At most BN_MAX_ROW_BLOCKS workgroups share the rows: three per CU, what the
// vector forms keep resident, so that no second, partial round of workgroups follows the first.
#define BN_ROWS_IN_FLIGHT 8
#define BN_MAX_ROW_BLOCKS 768
template <typename T, int VEC>
__device__ __forceinline__ float vec_get(const typename VecOf<T, VEC>::type &v, int j) {
  if constexpr (VEC == 1)
    return (float)v;
  else
    return (float)v[j];
}
template <typename T, int VEC>
__device__ __forceinline__ typename VecOf<T, VEC>::type vec_zero() {
  typename VecOf<T, VEC>::type v;
  if constexpr (VEC == 1) {
    v = (T)0;
  } else {
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] = (T)0;
  }
  return v;
}
// GATED: a third operand (the gate) is read, and half as many rows are requested per step
template <typename T, int VEC, bool GATED>
__global__ void __launch_bounds__(256) col_sums_partial_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                               const T *__restrict__ gate, int gate_act, float gate_slope,
                                                               long long n, int c, int cols_per_block,
                                                               double *__restrict__ partial) {
  typedef typename VecOf<T, VEC>::type V;
  constexpr int ROWS = GATED ? BN_ROWS_IN_FLIGHT / 2 : BN_ROWS_IN_FLIGHT;
  // thread -> (vector column, row lane): a workgroup covers cols_per_block vector columns (a power of two up to
  // 256) with 256 / cols_per_block row lanes; blockIdx.y walks over the column blocks
  const int tc = threadIdx.x % cols_per_block;
  const int col0 = (blockIdx.y * cols_per_block + tc) * VEC;
  const int lanes = 256 / cols_per_block, rl = threadIdx.x / cols_per_block;
  double s1[VEC], s2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) s1[j] = s2[j] = 0.0;
  if (col0 < c) {
    const long long stride = (long long)gridDim.x * lanes;
    for (long long r0 = (long long)blockIdx.x * lanes + rl; r0 < n; r0 += stride * ROWS) {
      // all loads of a step are requested before the first is used
      V xs[ROWS], ys[ROWS], gs[GATED ? ROWS : 1];
      const V zero = vec_zero<T, VEC>();
#pragma unroll
      for (int k = 0; k < ROWS; ++k) {
        const long long r = r0 + k * stride;
        xs[k] = r < n ? *reinterpret_cast<const V *>(a + r * c + col0) : zero;
        ys[k] = b ? (r < n ? *reinterpret_cast<const V *>(b + r * c + col0) : zero) : xs[k];
        if (GATED) gs[k] = r < n ? *reinterpret_cast<const V *>(gate + r * c + col0) : zero;
      }
      float f1[VEC], f2[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) f1[j] = f2[j] = 0.f;
#pragma unroll
      for (int k = 0; k < ROWS; ++k)
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          float x = vec_get<T, VEC>(xs[k], j);
          const float y = vec_get<T, VEC>(ys[k], j);
          if (GATED) x *= act_slope_at(vec_get<T, VEC>(gs[k], j), gate_act, gate_slope);
          f1[j] += x;
          f2[j] += x * y;
        }
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        s1[j] += (double)f1[j];
        s2[j] += (double)f2[j];
      }
    }
  }
  // the row lanes of a column are cols_per_block threads apart: halving tree over them, both sums at once
  __shared__ double red[2 * VEC * 256];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    red[j * 256 + threadIdx.x] = s1[j];
    red[(VEC + j) * 256 + threadIdx.x] = s2[j];
  }
  __syncthreads();
  // a thread keeps its own sums in registers and publishes them only while a later step still reads them
  for (int off = lanes >> 1; off >= 1; off >>= 1) {
    if (rl < off) {
      double other[2 * VEC];
#pragma unroll
      for (int q = 0; q < 2 * VEC; ++q) other[q] = red[q * 256 + threadIdx.x + off * cols_per_block];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        s1[j] += other[j];
        s2[j] += other[VEC + j];
      }
      if (rl >= (off >> 1) && off > 1) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          red[j * 256 + threadIdx.x] = s1[j];
          red[(VEC + j) * 256 + threadIdx.x] = s2[j];
        }
      }
    }
    __syncthreads();
  }
  if (rl == 0 && col0 < c) {
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      if (col0 + j < c) {
        partial[((long long)blockIdx.x * 2 + 0) * c + col0 + j] = s1[j];
        partial[((long long)blockIdx.x * 2 + 1) * c + col0 + j] = s2[j];
      }
  }
}

// both partial sums of channel j over all workgroups, by one wavefront; the result is valid in lane 0
__device__ __forceinline__ void wave_sum_partials(const double *__restrict__ partial, long long blocks, int c, int j,
                                                  double *s1, double *s2) {
  double a = 0.0, b = 0.0;
  // four blocks per lane and step, all eight loads requested before the first is added
  for (long long i0 = threadIdx.x; i0 < blocks; i0 += 256) {
    double x[4], y[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const long long i = i0 + 64 * k;
      x[k] = i < blocks ? partial[(i * 2 + 0) * c + j] : 0.0;
      y[k] = i < blocks ? partial[(i * 2 + 1) * c + j] : 0.0;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      a += x[k];
      b += y[k];
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    a += __shfl_down(a, off, 64);
    b += __shfl_down(b, off, 64);
  }
  *s1 = a;
  *s2 = b;
}

__global__ void __launch_bounds__(64) col_sums_final_kernel(const double *__restrict__ partial, long long blocks, int c,
                                                             double *__restrict__ out) {
  const int col = blockIdx.x;   // one wavefront per column
  double s1 = 0.0, s2 = 0.0;
  wave_sum_partials(partial, blocks, c, col, &s1, &s2);
  if (threadIdx.x == 0) {
    out[col] = s1;
    out[c + col] = s2;
  }
}

// upper bound of the row blocks of any layout of n rows (the workspace is sized for it)
static int64_t bn_max_row_blocks(int64_t n) {
  const int64_t by_rows = pce_div_up(n, BN_ROWS_IN_FLIGHT);
  return by_rows < BN_MAX_ROW_BLOCKS ? by_rows : BN_MAX_ROW_BLOCKS;
}

extern "C" int64_t pce_col_sums_workspace_bytes(int64_t n, int32_t c) {
  if (n <= 0 || c <= 0) return 0;
  return bn_max_row_blocks(n) * 2 * c * (int64_t)sizeof(double);
}

// launches the partial-sum kernel; *blocks_out = row blocks written (partial[block][2][c])
static int bn_partial(const void *a, const void *b, const void *gate, int gate_act, float gate_slope, int32_t dtype, int64_t n,
                      int32_t c, double *partial, int64_t *blocks_out, hipStream_t s) {
  const int full = dtype == PCE_F16 ? 8 : 4;
  const int vec = (c % full == 0 && aligned16(a) && aligned16(b) && aligned16(gate)) ? full : 1;
  const int vcols = c / vec;
  int cpb = 1;   // vector columns per workgroup: the power of two >= vcols, at most 256
  while (cpb < vcols && cpb < 256) cpb <<= 1;
  const int lanes = 256 / cpb;
  int64_t blocks = pce_div_up(n, (int64_t)lanes * BN_ROWS_IN_FLIGHT);
  if (blocks > BN_MAX_ROW_BLOCKS) blocks = BN_MAX_ROW_BLOCKS;
  dim3 grid((unsigned)blocks, (unsigned)pce_div_up(vcols, cpb));
#define PCE_COLSUMS(T_, V_)                                                                                                   \
  if (gate)                                                                                                                  \
    hipLaunchKernelGGL((col_sums_partial_kernel<T_, V_, true>), grid, dim3(256), 0, s, (const T_ *)a,       \
                       (const T_ *)b, (const T_ *)gate, gate_act, gate_slope, (long long)n, c, cpb, partial);                \
  else                                                                                                                       \
    hipLaunchKernelGGL((col_sums_partial_kernel<T_, V_, false>), grid, dim3(256), 0, s, (const T_ *)a,                       \
                       (const T_ *)b, (const T_ *)gate, gate_act, gate_slope, (long long)n, c, cpb, partial)
  if (dtype == PCE_F16 && vec == 8)
    PCE_COLSUMS(half_t, 8);
  else if (dtype == PCE_F16)
    PCE_COLSUMS(half_t, 1);
  else if (vec == 4)
    PCE_COLSUMS(float, 4);
  else
    PCE_COLSUMS(float, 1);
#undef PCE_COLSUMS
  PCE_LAUNCH_CHECK("col_sums_partial");
  *blocks_out = blocks;
  return PCE_OK;
}

extern "C" int pce_col_sums(const void *a, const void *b, int32_t dtype, int64_t n, int32_t c, void *ws, int64_t ws_bytes,
                            double *out, pce_stream_t stream) {
  if (!a || !out) PCE_FAIL(PCE_EINVAL, "pce_col_sums: null pointer");
  if (dtype != PCE_F16 && dtype != PCE_F32) PCE_FAIL(PCE_EINVAL, "pce_col_sums: dtype %d", (int)dtype);
  if (n <= 0 || c <= 0) PCE_FAIL(PCE_EINVAL, "pce_col_sums: n=%lld c=%d", (long long)n, (int)c);
  const int64_t need = pce_col_sums_workspace_bytes(n, c);
  if (!ws || ws_bytes < need) PCE_FAIL(PCE_EWORKSPACE, "pce_col_sums: workspace %lld < %lld", (long long)ws_bytes, (long long)need);
  hipStream_t s = (hipStream_t)stream;
  int64_t blocks = 0;
  int rc = bn_partial(a, b, nullptr, PCE_ACT_NONE, 0.f, dtype, n, c, (double *)ws, &blocks, s);
  if (rc) return rc;
  hipLaunchKernelGGL(col_sums_final_kernel, dim3((unsigned)c), dim3(64), 0, s, (const double *)ws,
                     (long long)blocks, c, out);
  PCE_LAUNCH_CHECK("col_sums_final");
  return PCE_OK;
}

// One wavefront per channel: adds up the per-workgroup partial sums and turns them into what the affine pass
// needs.  Forward (sums of x and x*x): mean, biased variance, rstd; coefficients kx = w*rstd,
// k0 = b - mean*kx; running statistics updated with the unbiased variance (torch.nn.BatchNorm1d).
__global__ void __launch_bounds__(64) bn_finish_forward_kernel(const double *__restrict__ partial, long long blocks,
                                                                long long n, int c, const float *__restrict__ weight,
                                                                const float *__restrict__ bias, float *running_mean,
                                                                float *running_var, int use_batch_stats, float momentum,
                                                                float eps, float *__restrict__ save_mean,
                                                                float *__restrict__ save_rstd, float *__restrict__ kx,
                                                                float *__restrict__ k0, float *__restrict__ ones) {
  const int j = blockIdx.x;   // one wavefront per channel
  double mean, var;
  if (use_batch_stats) {
    double s1 = 0.0, s2 = 0.0;
    wave_sum_partials(partial, blocks, c, j, &s1, &s2);
    if (threadIdx.x != 0) return;
    mean = s1 / (double)n;
    var = s2 / (double)n - mean * mean;
    if (var < 0.0) var = 0.0;
    if (momentum >= 0.f && running_mean && running_var) {
      double unbiased = n > 1 ? var * ((double)n / (double)(n - 1)) : var;
      running_mean[j] = (float)((1.0 - momentum) * running_mean[j] + momentum * mean);
      running_var[j] = (float)((1.0 - momentum) * running_var[j] + momentum * unbiased);
    }
  } else {
    if (threadIdx.x != 0) return;
    mean = running_mean[j];
    var = running_var[j];
  }
  double rstd = 1.0 / sqrt(var + (double)eps);
  double w = weight ? (double)weight[j] : 1.0, b = bias ? (double)bias[j] : 0.0;
  save_mean[j] = (float)mean;
  save_rstd[j] = (float)rstd;
  kx[j] = (float)(w * rstd);
  k0[j] = (float)(b - mean * w * rstd);
  if (ones) ones[j] = 1.f;   // coefficient of the residual term of the affine map
}

// Backward (sums of dy and dy*x): grad_bias = sum dy, grad_weight = S = sum dy*xhat,
// dx = dy*k1 + x*kd + k0 with k1 = w*rstd, kd = -k1*rstd*S/n, k0 = -k1*sum(dy)/n - kd*mean
// (statistics of the batch), or dx = dy*k1 (fixed statistics).
__global__ void __launch_bounds__(64) bn_finish_backward_kernel(const double *__restrict__ partial, long long blocks,
                                                                 long long n, int c, const float *__restrict__ weight,
                                                                 const float *__restrict__ save_mean,
                                                                 const float *__restrict__ save_rstd, int use_batch_stats,
                                                                 float *__restrict__ grad_weight, float *__restrict__ grad_bias,
                                                                 float *__restrict__ k1, float *__restrict__ kd,
                                                                 float *__restrict__ k0) {
  const int j = blockIdx.x;   // one wavefront per channel
  double s1 = 0.0, s2 = 0.0;
  wave_sum_partials(partial, blocks, c, j, &s1, &s2);
  if (threadIdx.x != 0) return;
  const double mean = save_mean[j], rstd = save_rstd[j], w = weight ? (double)weight[j] : 1.0;
  const double S = rstd * (s2 - mean * s1);
  if (grad_weight) grad_weight[j] = (float)S;
  if (grad_bias) grad_bias[j] = (float)s1;
  const double a = w * rstd;
  k1[j] = (float)a;
  if (use_batch_stats) {
    const double d = -a * rstd * S / (double)n;
    kd[j] = (float)d;
    k0[j] = (float)(-a * s1 / (double)n - d * mean);
  } else {
    kd[j] = 0.f;
    k0[j] = 0.f;
  }
}

template <typename T, int VEC>
__global__ void __launch_bounds__(256) col_affine_kernel(const T *__restrict__ x, const T *__restrict__ d, T *__restrict__ y,
                                                         long long n, int c, const float *__restrict__ kx,
                                                         const float *__restrict__ kd, const float *__restrict__ k0, int act,
                                                         float slope, const T *__restrict__ gate, int gate_act,
                                                         float gate_slope) {
  typedef typename VecOf<T, VEC>::type V;
  const int row_vecs = c / VEC;
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * row_vecs) return;
  const int v = (int)(i - (i / row_vecs) * row_vecs);
  V xv = *reinterpret_cast<const V *>(x + i * VEC);
  V dv = xv, gv = xv;
  if (d) dv = *reinterpret_cast<const V *>(d + i * VEC);
  if (gate) gv = *reinterpret_cast<const V *>(gate + i * VEC);
  V out;
  // the thread's VEC coefficients are contiguous: 16-byte loads when VEC is a multiple of four
  float cx[VEC], c0[VEC], cd[VEC];
  if (VEC % 4 == 0) {
#pragma unroll
    for (int q = 0; q < VEC / 4; ++q) {
      f32x4 a = *reinterpret_cast<const f32x4 *>(kx + v * VEC + q * 4);
      f32x4 b = *reinterpret_cast<const f32x4 *>(k0 + v * VEC + q * 4);
      f32x4 e = a;
      if (d) e = *reinterpret_cast<const f32x4 *>(kd + v * VEC + q * 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        cx[q * 4 + j] = a[j];
        c0[q * 4 + j] = b[j];
        cd[q * 4 + j] = e[j];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      cx[j] = kx[v * VEC + j];
      c0[j] = k0[v * VEC + j];
      cd[j] = d ? kd[v * VEC + j] : 0.f;
    }
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    float xj = (float)(reinterpret_cast<const T *>(&xv)[j]);
    if (gate) xj *= act_slope_at((float)(reinterpret_cast<const T *>(&gv)[j]), gate_act, gate_slope);
    float r = xj * cx[j] + c0[j];
    if (d) r += (float)(reinterpret_cast<const T *>(&dv)[j]) * cd[j];
    reinterpret_cast<T *>(&out)[j] = (T)act_apply(r, act, slope);
  }
  *reinterpret_cast<V *>(y + i * VEC) = out;
}

// y = act(x' * kx + d * kd + k0), x' = x times the derivative of another activation where its output was `gate`
static int col_affine_launch(const char *who, const void *x, const void *d, const void *gate, void *y, int32_t dtype, int64_t n,
                             int32_t c, const float *kx, const float *kd, const float *k0, int32_t act, float slope,
                             int32_t gate_act, float gate_slope, hipStream_t s) {
  const int vec = dtype == PCE_F16 ? 8 : 4;
  const bool aligned = aligned16(x) && aligned16(y) && aligned16(d) && aligned16(gate) && c % vec == 0;
  const long long items = aligned ? n * (c / vec) : n * c;
  if (pce_div_up(items, 256) >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "%s: tensor too large for one launch", who);
  dim3 grid((unsigned)pce_div_up(items, 256));
#define PCE_AFFINE(T_, V_)                                                                                               \
  hipLaunchKernelGGL((col_affine_kernel<T_, V_>), grid, dim3(256), 0, s, (const T_ *)x, (const T_ *)d, (T_ *)y, (long long)n, c, \
                     kx, kd, k0, act, slope, (const T_ *)gate, gate_act, gate_slope)
  if (dtype == PCE_F16 && aligned)
    PCE_AFFINE(half_t, 8);
  else if (dtype == PCE_F16)
    PCE_AFFINE(half_t, 1);
  else if (aligned)
    PCE_AFFINE(float, 4);
  else
    PCE_AFFINE(float, 1);
#undef PCE_AFFINE
  PCE_LAUNCH_CHECK("col_affine");
  return PCE_OK;
}

static bool act_known(int32_t act) { return act == PCE_ACT_NONE || act == PCE_ACT_RELU || act == PCE_ACT_LEAKY_RELU; }

extern "C" int pce_col_affine(const void *x, const void *d, void *y, int32_t dtype, int64_t n, int32_t c, const float *kx,
                              const float *kd, const float *k0, int32_t act, float slope, pce_stream_t stream) {
  if (!x || !y || !kx || !k0 || (d && !kd)) PCE_FAIL(PCE_EINVAL, "pce_col_affine: null pointer");
  if (dtype != PCE_F16 && dtype != PCE_F32) PCE_FAIL(PCE_EINVAL, "pce_col_affine: dtype %d", (int)dtype);
  if (n <= 0 || c <= 0) PCE_FAIL(PCE_EINVAL, "pce_col_affine: n=%lld c=%d", (long long)n, (int)c);
  if (!act_known(act)) PCE_FAIL(PCE_EINVAL, "pce_col_affine: activation %d", (int)act);
  return col_affine_launch("pce_col_affine", x, d, nullptr, y, dtype, n, c, kx, kd, k0, act, slope, PCE_ACT_NONE, 0.f,
                           (hipStream_t)stream);
}

// workspace of the fused entry points: the partial sums, then 3*c floats of coefficients
extern "C" int64_t pce_bn_workspace_bytes(int64_t n, int32_t c) {
  if (n <= 0 || c <= 0) return 0;
  return pce_align_up(pce_col_sums_workspace_bytes(n, c), 256) + 3 * (int64_t)c * (int64_t)sizeof(float);
}

extern "C" int pce_bn_forward(const void *x, const void *residual, void *y, int32_t dtype, int64_t n, int32_t c, const float *weight,
                              const float *bias, float *running_mean, float *running_var, int32_t use_batch_stats,
                              float momentum, float eps, float *save_mean, float *save_rstd, void *ws, int64_t ws_bytes,
                              int32_t act, float slope, pce_stream_t stream) {
  if (!x || !y || !save_mean || !save_rstd) PCE_FAIL(PCE_EINVAL, "pce_bn_forward: null pointer");
  if (dtype != PCE_F16 && dtype != PCE_F32) PCE_FAIL(PCE_EINVAL, "pce_bn_forward: dtype %d", (int)dtype);
  if (n <= 0 || c <= 0) PCE_FAIL(PCE_EINVAL, "pce_bn_forward: n=%lld c=%d", (long long)n, (int)c);
  if (!use_batch_stats && (!running_mean || !running_var)) PCE_FAIL(PCE_EINVAL, "pce_bn_forward: fixed statistics need running_mean and running_var");
  if (!act_known(act)) PCE_FAIL(PCE_EINVAL, "pce_bn_forward: activation %d", (int)act);
  if (!ws || ws_bytes < pce_bn_workspace_bytes(n, c)) PCE_FAIL(PCE_EWORKSPACE, "pce_bn_forward: workspace %lld < %lld", (long long)ws_bytes, (long long)pce_bn_workspace_bytes(n, c));
  hipStream_t s = (hipStream_t)stream;
  double *partial = (double *)ws;
  float *coef = (float *)((char *)ws + pce_align_up(pce_col_sums_workspace_bytes(n, c), 256));
  int64_t blocks = 0;
  int rc;
  if (use_batch_stats && (rc = bn_partial(x, nullptr, nullptr, PCE_ACT_NONE, 0.f, dtype, n, c, partial, &blocks, s))) return rc;
  hipLaunchKernelGGL(bn_finish_forward_kernel, dim3((unsigned)c), dim3(64), 0, s, (const double *)partial,
                     (long long)blocks, (long long)n, c, weight, bias, running_mean, running_var, use_batch_stats, momentum, eps,
                     save_mean, save_rstd, coef, coef + c, residual ? coef + 2 * c : nullptr);
  PCE_LAUNCH_CHECK("bn_finish_forward");
  return col_affine_launch("pce_bn_forward", x, residual, nullptr, y, dtype, n, c, coef, residual ? coef + 2 * c : nullptr, coef + c,
                           act, slope, PCE_ACT_NONE, 0.f, s);
}

extern "C" int pce_bn_backward(const void *x, const void *dy, const void *y_act, int32_t act, float slope, void *dx,
                               int32_t dtype, int64_t n, int32_t c, const float *weight, const float *save_mean,
                               const float *save_rstd, int32_t use_batch_stats, float *grad_weight, float *grad_bias, void *ws,
                               int64_t ws_bytes, pce_stream_t stream) {
  if (!x || !dy || !dx || !save_mean || !save_rstd) PCE_FAIL(PCE_EINVAL, "pce_bn_backward: null pointer");
  if (!act_known(act)) PCE_FAIL(PCE_EINVAL, "pce_bn_backward: activation %d", (int)act);
  if (act != PCE_ACT_NONE && !y_act) PCE_FAIL(PCE_EINVAL, "pce_bn_backward: the gradient of an activation needs its output");
  if (act == PCE_ACT_NONE) y_act = nullptr;
  if (dtype != PCE_F16 && dtype != PCE_F32) PCE_FAIL(PCE_EINVAL, "pce_bn_backward: dtype %d", (int)dtype);
  if (n <= 0 || c <= 0) PCE_FAIL(PCE_EINVAL, "pce_bn_backward: n=%lld c=%d", (long long)n, (int)c);
  if (!ws || ws_bytes < pce_bn_workspace_bytes(n, c)) PCE_FAIL(PCE_EWORKSPACE, "pce_bn_backward: workspace %lld < %lld", (long long)ws_bytes, (long long)pce_bn_workspace_bytes(n, c));
  hipStream_t s = (hipStream_t)stream;
  double *partial = (double *)ws;
  float *coef = (float *)((char *)ws + pce_align_up(pce_col_sums_workspace_bytes(n, c), 256));
  int64_t blocks = 0;
  int rc = bn_partial(dy, x, y_act, act, slope, dtype, n, c, partial, &blocks, s);
  if (rc) return rc;
  hipLaunchKernelGGL(bn_finish_backward_kernel, dim3((unsigned)c), dim3(64), 0, s, (const double *)partial,
                     (long long)blocks, (long long)n, c, weight, save_mean, save_rstd, use_batch_stats, grad_weight, grad_bias, coef,
                     coef + c, coef + 2 * c);
  PCE_LAUNCH_CHECK("bn_finish_backward");
  return col_affine_launch("pce_bn_backward", dy, x, y_act, dx, dtype, n, c, coef, coef + c, coef + 2 * c, PCE_ACT_NONE, 0.f, act,
                           slope, s);
}

// ---- channel concatenation of two feature matrices on the same rows (script/utils.py:152-164) ---------
// out[r] = (a[r], b[r]).  One 16-byte vector per thread; threadIdx.x walks along the output row, so a
// wavefront reads and writes whole rows.  va / vb = vectors per row of a / b.
__global__ void __launch_bounds__(256) concat_cols_kernel(const u32x4 *__restrict__ a, const u32x4 *__restrict__ b,
                                                          u32x4 *__restrict__ out, long long n, int va, int vb, int stream) {
  const long long r = (long long)blockIdx.x * blockDim.y + threadIdx.y;
  const int v = threadIdx.x;
  if (r >= n || v >= va + vb) return;
  store_maybe_stream(&out[r * (va + vb) + v], v < va ? a[r * va + v] : b[r * vb + (v - va)], stream != 0);
}

extern "C" int pce_concat_cols(const void *a, int32_t c_a, const void *b, int32_t c_b, void *out, int32_t dtype, int64_t n,
                               pce_stream_t stream) {
  if (!a || !b || !out) PCE_FAIL(PCE_EINVAL, "pce_concat_cols: null pointer");
  if (dtype != PCE_F16 && dtype != PCE_F32) PCE_FAIL(PCE_EINVAL, "pce_concat_cols: dtype %d", (int)dtype);
  if (n <= 0 || c_a <= 0 || c_b <= 0) PCE_FAIL(PCE_EINVAL, "pce_concat_cols: n=%lld c_a=%d c_b=%d", (long long)n, (int)c_a, (int)c_b);
  const int per = dtype == PCE_F16 ? 8 : 4;   // elements per 16-byte vector
  if (c_a % per || c_b % per || !aligned16(a) || !aligned16(b) || !aligned16(out))
    PCE_FAIL(PCE_EINVAL, "pce_concat_cols: rows of %d and %d elements are not whole 16-byte vectors, or a pointer is unaligned", (int)c_a, (int)c_b);
  const int va = c_a / per, vb = c_b / per;
  if (va + vb > 256) PCE_FAIL(PCE_ECAPACITY, "pce_concat_cols: %d channels exceed one workgroup per row", (int)(c_a + c_b));
  int tx = 1;
  while (tx < va + vb) tx <<= 1;
  const int ty = 256 / tx;
  const long long blocks = pce_div_up(n, ty);
  if (blocks >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "pce_concat_cols: %lld workgroups exceed the grid limit", blocks);
  hipLaunchKernelGGL(concat_cols_kernel, dim3((unsigned)blocks), dim3(tx, ty), 0, (hipStream_t)stream, (const u32x4 *)a,
                     (const u32x4 *)b, (u32x4 *)out, (long long)n, va, vb, stream_policy((long long)n * (va + vb) * 16));
  PCE_LAUNCH_CHECK("concat_cols");
  return PCE_OK;
}

extern "C" int pce_conv_oso_takes(int32_t dtype, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid) {
  return oso_layer(dtype, c_in, c_out, kv, mid) ? 1 : 0;
}

// Map density rho = pairs per output row.  The deferred-scatter dataflow does only the useful
// multiplications and pays M*(c_in + 2*c_out) elements of gather / partial-row traffic for them; the
// output-stationary kernel touches no intermediate memory but multiplies every offset of every
// 128-row tile, populated or not.  So the density at which output-stationary takes over rises with the
// channel product: the wider the layer, the dearer its wasted multiplications and the cheaper, per
// flop, the partial-row traffic.  Thresholds from two MinkUNet-style networks measured layer by layer
// with every dataflow (100 k LiDAR voxels, channels 32..256; 954 k indoor voxels in 8 scenes, channels
// 64..512): up to 64x64 channels output-stationary leads from rho = 4 (2x at rho = 5), up to 128x128
// from rho = 5..6, up to 256x256 the two are within 10 % between rho = 9 and 13 and output-stationary
// leads by 1.35x at rho = 20; at 512 channels deferred scatter leads at every density seen.  A
// 2x2x2 stride-2 layer covers every input exactly once and favours output-stationary up to 64x64; up to
// 128x128 it does from two pairs per row (128 -> 128 at rho = 4.0: 31 vs 46 us, at rho = 2.5: 22 vs 25 us),
// while on surface-like clouds (rho near 1) deferred scatter stores nearly every row straight from its only
// pair and leads (64 -> 128 at rho = 1.03: 23 vs 43 us).  Products up to 128x256 sit between the 128x128 and
// 256x256 classes: output-stationary leads at rho = 10.3 (155 vs 178 us) and 19.5 (85 vs 154 us).
// The atomic fetch-on-demand and the staged gather-GEMM-scatter dataflows of the reference were never
// the fastest (gather-GEMM-scatter comes first only on a 4-channel input layer, by 10 %).
extern "C" int pce_select_dataflow(int64_t n_in, int64_t n_out, int64_t n_pairs, int32_t c_in, int32_t c_out, int32_t kv,
                                   int32_t mid, int32_t transposed, int32_t dtype) {
  if (n_out <= 0) return PCE_DATAFLOW_FDS;
  if (kv == 1) return PCE_DATAFLOW_OS;
  const double rho = (double)n_pairs / (double)n_out;
  const int64_t prod = (int64_t)c_in * c_out;
  // The ordered dataflow, where pce_conv_fwd_oso takes the layer (never a transposed one: its rows are the inputs').
  const bool oso = !transposed && oso_layer(dtype, c_in, c_out, kv, mid);
  const bool subm = mid >= 0, down = mid < 0 && kv <= 8 && n_out < n_in;
  // narrow fp16 submanifold layers: one launch over rows ordered by neighbour pattern.  Measured against deferred
  // scatter with bias, residual and ReLU fused: 0.78-0.93 of its time at 0.1-0.2 pairs per row (100-150 k voxels,
  // 16-64 channels), 0.62-0.83 at 0.8, 0.64-0.83 at 3, 0.60-0.62 at 5.3 (541 k voxels, where it equals plain
  // output-stationary); beyond that the dense output-stationary tiles below take over.
  // the fp32 form is bound by its MFMAs (c_in / 4 of them per offset and 16 rows): measured against deferred scatter
  // at 4.7 pairs per row 0.76 (8 channels), 0.87 (16), 1.15 (32); at 0.2 pairs per row 0.49, 0.62, 0.82
  if (oso && subm && dtype == PCE_F32 && rho <= (c_in <= 16 ? 6.0 : 2.0)) return PCE_DATAFLOW_OSO;
  // (a cloud of fewer than two 128-row tiles per compute unit -- 256 of them -- leaves the dense tiles' launch short
  // of workgroups: 24 k rows at 9.2 pairs per row, 48 -> 48 channels: ordered rows 17 us, deferred scatter 21, tiles 28)
  if (oso && subm && dtype == PCE_F16 && os_widths(c_in, c_out) && rho <= (n_out < 2 * 256 * 128 ? 12.0 : 6.0)) return PCE_DATAFLOW_OSO;
  // the K-stepped form of the same kernel (wave_osw_kernel): a wavefront walks c_in / 16 K steps per offset of its
  // rows' union, so the density up to which it leads falls with the input width.  Measured on the levels of a
  // 100 k-voxel LiDAR pyramid against the faster of deferred scatter and the dense tiles: 64 -> 96, 96 -> 96, 64 -> 128
  // (4 to 6 K steps) at 0.13 / 0.8 / 3.0 / 8.9 pairs per row 0.89-0.93 / 0.77-0.85 / 0.71-0.79 / 0.81-0.91 of its time
  // (equal at 19.5; 80 -> 80 at 0.06 on 50 k rows: 0.66); 128 -> 96 (8 K steps) 0.97 at 0.13, 0.81 at 0.8, 0.91 at 3.0,
  // 1.03-1.12 beyond
  if (oso && subm && dtype == PCE_F16 && osw_widths(c_in, c_out) && rho <= (c_in <= 96 ? 12.0 : 4.0))
    return PCE_DATAFLOW_OSO;
  // narrow fp16 stride-2 layers (every input row in exactly one pair, 1-8 per output row), through the same ordered
  // rows without a centre term: 0.58-0.66 of the output-stationary tiles' time at 1.0-1.4 pairs per row (66-146 k
  // output rows, 32 and 64 channels; 680 k rows: 0.71), 0.57 at 2.4 on 27 k rows and 1.05 at 2.5 on 276 k rows of
  // indoor scenes, where half the rows have three pairs or more
  if (oso && down && dtype == PCE_F16 && os_widths(c_in, c_out) && rho <= 2.0) return PCE_DATAFLOW_OSO;
  // ... and of the K-stepped kernel's shapes: 64 -> 128, 64 / 96 -> 96, 96 -> 128, 128 -> 96 at 1.0-2.5 pairs per row on
  // five levels of LiDAR and indoor pyramids (26 k to 541 k output rows) 0.64-0.94 of the faster of deferred scatter
  // and the dense tiles (64 -> 128 on the 146 k-row level of the headline cloud: 21.3 vs 24.5 us); 128 -> 128 (32
  // weight fragments per offset: beyond what the kernel is built for) ran from 0.72 to 1.06 of it with nothing in
  // (rows, density) to tell the cases apart
  if (oso && down && dtype == PCE_F16 && osw_widths(c_in, c_out) && rho <= 2.6) return PCE_DATAFLOW_OSO;
  if (kv <= 8 && n_out <= n_in && rho >= 1.0 && prod <= 64 * 64 && dtype == PCE_F16) return PCE_DATAFLOW_OS;
  if (kv <= 8 && n_out <= n_in && rho >= 2.0 && prod <= 128 * 128 && dtype == PCE_F16) return PCE_DATAFLOW_OS;
  double takeover;
  if (prod <= 64 * 64)
    takeover = 4.0;
  else if (prod <= 128 * 128)
    takeover = 5.0;
  else if (prod <= 128 * 256)
    takeover = 10.0;
  else if (prod <= 256 * 256)
    takeover = 12.0;
  else
    return PCE_DATAFLOW_FDS;
  // fp32 multiplies at a fraction of the fp16 MFMA rate: wasted multiplications cost more (configuration 1,
  // fp32 16x16 channels at rho = 4.7, is 1.35x faster with deferred scatter)
  if (dtype == PCE_F32) takeover *= 2.0;
  return rho >= takeover ? PCE_DATAFLOW_OS : PCE_DATAFLOW_FDS;
}
