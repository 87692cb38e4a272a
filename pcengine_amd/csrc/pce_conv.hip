// Forward sparse convolution on gfx950: one MFMA tile kernel serving the fetch-on-demand,
// grouped-GEMM, dense-centre and output-stationary modes, plus the streaming gather / scatter /
// convert kernels of the gather-GEMM-scatter dataflow.
//
// Tile: 128 rows (4 wavefronts x 32 rows) x NT output channels, K staged through LDS in chunks.
// fp16: v_mfma_f32_32x32x16_f16, fp32 accumulate.  fp32: v_mfma_f32_32x32x2_f32.
// The A operand (feature rows) goes global -> registers with 16-byte loads, one row per lane; only
// the per-offset weight tile passes through LDS, laid out so that a lane's B fragment is one
// conflict-free 16-byte read.
#include "pce_common.h"

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

enum {
  MODE_FOD = 0,      // A row = imap[pair], out row = omap[pair]
  MODE_BUF = 1,      // A row = out row = quantised pair row (staging buffer)
  MODE_DENSE = 2,    // A row = out row = tile row, one fixed weight
  MODE_OS = 3,       // out row = tile row, A row = nbr[kp][row], loop over all offsets
  MODE_FOD_BUF = 4   // A row = imap[pair], out row = quantised pair row (staging buffer)
};
enum {
  EPI_ATOMIC_F32 = 0,  // fp32 atomic add, one column per lane
  EPI_ROWS = 1,        // store T, 16 bytes per lane along the row
  EPI_ROWS_F32 = 2,    // store fp32 (accumulator of the atomic dataflow), 16 bytes per lane
  EPI_ROWS_CSR = 3     // EPI_ROWS plus the sum of the row's staging-buffer rows (CSR-coded list)
};

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
  const int *ocode;
  const void *buf;
  long long n_rows;  // MODE_DENSE / MODE_OS: rows of the output
  int kv, c_in, c_out;
  int w_fixed;
  int mode, epi;
  int a_vec, w_vec, o_vec, b_vec;  // 16-byte accesses allowed on A rows / W rows / out rows / buf rows
  int k8_total, n_pad;             // packed weight extents
  int host_pos;                    // kpos_h / qkpos_h are valid
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

// ---- weight chunk -> LDS -----------------------------------------------------------------------
// fp16 LDS layout: Wl[k/8][n][k%8]
template <int NT>
__device__ __forceinline__ void stage_weights(half_t *Wl, const half_t *__restrict__ Wk, const half_t *__restrict__ Pk,
                                              int k0, int n0, const TileArgs &a) {
  constexpr int KC = Cfg<half_t>::KC;
  for (int e = threadIdx.x; e < (KC / 8) * NT; e += 256) {
    int n = e % NT, k8 = e / NT;
    int gn = n0 + n, gk = k0 + k8 * 8;
    half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (Pk) {
      if (gk / 8 < a.k8_total && gn < a.n_pad) v = *reinterpret_cast<const half8 *>(&Pk[((long long)(gk / 8) * a.n_pad + gn) * 8]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (gn < a.c_out && gk + j < a.c_in) v[j] = Wk[(long long)(gk + j) * a.c_out + gn];
    }
    *reinterpret_cast<half8 *>(&Wl[(k8 * NT + n) * 8]) = v;
  }
}

// fp32 LDS layout: Wl[k][n]
template <int NT>
__device__ __forceinline__ void stage_weights(float *Wl, const float *__restrict__ Wk, const float * /*Pk*/, int k0,
                                              int n0, const TileArgs &a) {
  constexpr int KC = Cfg<float>::KC;
  for (int e = threadIdx.x; e < KC * NT / 4; e += 256) {
    int n = (e % (NT / 4)) * 4, k = e / (NT / 4);
    int gn = n0 + n, gk = k0 + k;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (gk < a.c_in) {
      if (a.w_vec && gn + 4 <= a.c_out) {
        v = *reinterpret_cast<const f32x4 *>(&Wk[(long long)gk * a.c_out + gn]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (gn + j < a.c_out) v[j] = Wk[(long long)gk * a.c_out + gn + j];
      }
    }
    *reinterpret_cast<f32x4 *>(&Wl[k * NT + n]) = v;
  }
}

// ---- one K chunk of MFMA work for a wavefront ---------------------------------------------------
template <int NB>
__device__ __forceinline__ void mma_chunk(f32x16 (&acc)[NB], const half_t *Wl, const half_t *__restrict__ A,
                                          int arow, int k0, int klen, int c_in, int a_vec, int l32, int g) {
  constexpr int NT = NB * 32;
  constexpr int KC = Cfg<half_t>::KC;
  half8 a[KC / 16];
  // issue every row load of the chunk before the first MFMA
#pragma unroll
  for (int s = 0; s < KC / 16; ++s) {
    int k = k0 + s * 16 + g * 8;
    half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (arow >= 0 && s * 16 < klen) {
      const half_t *p = A + (long long)arow * c_in + k;
      if (a_vec && k + 8 <= c_in) {
        v = *reinterpret_cast<const half8 *>(p);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (k + j < c_in) v[j] = p[j];
      }
    }
    a[s] = v;
  }
#pragma unroll
  for (int s = 0; s < KC / 16; ++s) {
    if (s * 16 < klen) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        half8 b = *reinterpret_cast<const half8 *>(&Wl[((s * 2 + g) * NT + nb * 32 + l32) * 8]);
        acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s], b, acc[nb], 0, 0, 0);
      }
    }
  }
}

template <int NB>
__device__ __forceinline__ void mma_chunk(f32x16 (&acc)[NB], const float *Wl, const float *__restrict__ A, int arow,
                                          int k0, int klen, int c_in, int a_vec, int l32, int g) {
  constexpr int NT = NB * 32;
  constexpr int KC = Cfg<float>::KC;
  f32x4 a[KC / 8];
#pragma unroll
  for (int s = 0; s < KC / 8; ++s) {
    int k = k0 + s * 8 + g * 4;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (arow >= 0 && s * 8 < klen) {
      const float *p = A + (long long)arow * c_in + k;
      if (a_vec && k + 4 <= c_in) {
        v = *reinterpret_cast<const f32x4 *>(p);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (k + j < c_in) v[j] = p[j];
      }
    }
    a[s] = v;
  }
#pragma unroll
  for (int s = 0; s < KC / 8; ++s) {
    if (s * 8 < klen) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // this MFMA contracts k = s*8 + e (lanes 0-31) and k = s*8 + 4 + e (lanes 32-63)
        int kk = s * 8 + g * 4 + e;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          float b = Wl[kk * NT + nb * 32 + l32];
          acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s][e], b, acc[nb], 0, 0, 0);
        }
      }
    }
  }
}

// ---- epilogues ---------------------------------------------------------------------------------
// MFMA layout: lane (l32, g) holds column l32 of rows 8*(j/4) + 4*g + j%4, j = 0..15.
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

template <typename TB, int CPL>
__device__ __forceinline__ void add_buf_row(float (&v)[CPL], const TB *__restrict__ p, int ncol, int vec_ok);

template <>
__device__ __forceinline__ void add_buf_row<half_t, 8>(float (&v)[8], const half_t *__restrict__ p, int ncol, int vec_ok) {
  if (vec_ok && ncol >= 8) {
    half8 b = *reinterpret_cast<const half8 *>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] += (float)b[j];
  } else {
    for (int j = 0; j < 8 && j < ncol; ++j) v[j] += (float)p[j];
  }
}
template <>
__device__ __forceinline__ void add_buf_row<float, 4>(float (&v)[4], const float *__restrict__ p, int ncol, int vec_ok) {
  if (vec_ok && ncol >= 4) {
    f32x4 b = *reinterpret_cast<const f32x4 *>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] += b[j];
  } else {
    for (int j = 0; j < 4 && j < ncol; ++j) v[j] += p[j];
  }
}
template <>
__device__ __forceinline__ void add_buf_row<half_t, 4>(float (&)[4], const half_t *__restrict__, int, int) {}

// Row-wise epilogue.  The wavefront transposes its 32 x NT accumulator through LDS, 16 rows at a
// time, so that a lane owns CPL consecutive columns of one row: stores (and the staging-buffer
// rows added in EPI_ROWS_CSR) are 16-byte accesses along the row.
template <typename T, int NB, bool F32OUT>
__device__ __forceinline__ void epilogue_rows(const f32x16 (&acc)[NB], float *El, int orow, int e0, int e1,
                                              const TileArgs &a, int n0, int lane, int l32, int g) {
  constexpr int NT = NB * 32, LD = NT + 8;
  constexpr int CPL = (F32OUT || sizeof(T) == 4) ? 4 : 8;
  constexpr int LPR = NT / CPL;
  const bool csr = a.epi == EPI_ROWS_CSR;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      int lr = 8 * (jj >> 2) + 4 * g + (jj & 3);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) El[lr * LD + nb * 32 + l32] = acc[nb][8 * half + jj];
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int idx = lane; idx < 16 * LPR; idx += 64) {  // 16 * LPR is a multiple of 64
      int lr = idx / LPR, ch = idx - lr * LPR;
      int r = 16 * half + lr;
      int dst = __shfl(orow, r, PCE_WAVE);
      int s0 = __shfl(e0, r, PCE_WAVE), s1 = __shfl(e1, r, PCE_WAVE);
      int col = n0 + ch * CPL;
      int ncol = a.c_out - col;
      if (dst < 0 || ncol <= 0) continue;
      float v[CPL];
#pragma unroll
      for (int q4 = 0; q4 < CPL / 4; ++q4) {
        f32x4 x = *reinterpret_cast<const f32x4 *>(&El[lr * LD + ch * CPL + q4 * 4]);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[q4 * 4 + j] = x[j];
      }
      if (csr) {
        const T *buf = (const T *)a.buf;
        for (int e = s0; e < s1; ++e) {
          int code = a.ocode[e];
          int kq = code / PCE_CSR_CODE;
          long long q = (long long)(a.host_pos ? a.qkpos_h[kq] : a.qkpos[kq]) + (code - kq * PCE_CSR_CODE);
          add_buf_row<T, CPL>(v, buf + q * a.c_out + col, ncol, a.b_vec);
        }
      }
      long long off = (long long)dst * a.c_out + col;
      if (F32OUT || sizeof(T) == 4) {
        float *o = (float *)a.out + off;
        if (a.o_vec && ncol >= 4) {
          f32x4 y = {v[0], v[1], v[2], v[3]};
          *reinterpret_cast<f32x4 *>(o) = y;
        } else {
          for (int j = 0; j < 4 && j < ncol; ++j) o[j] = v[j];
        }
      } else {
        half_t *o = (half_t *)a.out + off;
        if (a.o_vec && ncol >= 8) {
          half8 y;
#pragma unroll
          for (int j = 0; j < CPL; ++j) y[j] = (half_t)v[j];
          *reinterpret_cast<half8 *>(o) = y;
        } else {
          for (int j = 0; j < CPL && j < ncol; ++j) o[j] = (half_t)v[j];
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

template <typename T, int NB>
__global__ void __launch_bounds__(256) tile_gemm_kernel(TileArgs a) {
  constexpr int NT = NB * 32;
  constexpr int KC = Cfg<T>::KC;
  __shared__ __attribute__((aligned(16))) T Wl[KC * NT];
  __shared__ __attribute__((aligned(16))) float El[4][16 * (NT + 8)];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int n0 = blockIdx.y * NT;
  const long long tile = blockIdx.x;
  const T *A = (const T *)a.A;
  const T *W = (const T *)a.W;
  const T *Wp = (const T *)a.Wp;

  int arow = -1, orow = -1;
  int w_begin, w_end;
  long long row = tile * 128 + wave * 32 + l32;
  if (a.mode == MODE_DENSE || a.mode == MODE_OS) {
    bool ok = row < a.n_rows;
    orow = ok ? (int)row : -1;
    arow = (a.mode == MODE_DENSE) ? orow : -1;
    w_begin = (a.mode == MODE_DENSE) ? a.w_fixed : 0;
    w_end = (a.mode == MODE_DENSE) ? a.w_fixed + 1 : a.kv;
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
      arow = (a.mode == MODE_BUF) ? (int)row : a.imap[p];
      orow = (a.mode == MODE_FOD) ? a.omap[p] : (int)row;
    }
    w_begin = widx;
    w_end = widx + 1;
  }
  // CSR range of this lane's row, fetched early: the epilogue needs it last
  int e0 = 0, e1 = 0;
  if (a.epi == EPI_ROWS_CSR && orow >= 0) {
    e0 = a.ocsr[orow];
    e1 = a.ocsr[orow + 1];
  }

  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[nb][j] = 0.f;

  for (int w = w_begin; w < w_end; ++w) {
    if (a.mode == MODE_OS) {
      arow = orow >= 0 ? a.nbr[(long long)w * a.n_rows + orow] : -1;
      if (!__syncthreads_or(arow >= 0)) continue;
    }
    const bool wave_has = __ballot(arow >= 0) != 0ull;
    const T *Wk = W + (long long)w * a.c_in * a.c_out;
    const T *Pk = Wp ? Wp + (long long)w * a.k8_total * a.n_pad * 8 : nullptr;
    for (int k0 = 0; k0 < a.c_in; k0 += KC) {
      __syncthreads();
      stage_weights<NT>(Wl, Wk, Pk, k0, n0, a);
      __syncthreads();
      int klen = a.c_in - k0 < KC ? a.c_in - k0 : KC;
      if (wave_has) mma_chunk<NB>(acc, Wl, A, arow, k0, klen, a.c_in, a.a_vec, l32, g);
    }
  }

  if (a.epi == EPI_ATOMIC_F32) {
    epilogue_atomic<NB>(acc, orow, a, n0, l32, g);
  } else if (a.epi == EPI_ROWS_F32) {
    epilogue_rows<T, NB, true>(acc, El[wave], orow, e0, e1, a, n0, lane, l32, g);
  } else {
    epilogue_rows<T, NB, false>(acc, El[wave], orow, e0, e1, a, n0, lane, l32, g);
  }
}

template <typename T>
static int launch_tile(const TileArgs &a, long long tiles, hipStream_t s) {
  if (tiles <= 0) return PCE_OK;
  if (tiles >= (1ll << 31)) PCE_FAIL(PCE_ECAPACITY, "tile count %lld exceeds the grid limit", tiles);
  int nb = (a.c_out + 31) / 32;
  if (nb >= 4) {
    dim3 grid((unsigned)tiles, (unsigned)((a.c_out + 127) / 128));
    hipLaunchKernelGGL((tile_gemm_kernel<T, 4>), grid, dim3(256), 0, s, a);
  } else if (nb == 3) {
    hipLaunchKernelGGL((tile_gemm_kernel<T, 3>), dim3((unsigned)tiles, 1), dim3(256), 0, s, a);
  } else if (nb == 2) {
    hipLaunchKernelGGL((tile_gemm_kernel<T, 2>), dim3((unsigned)tiles, 1), dim3(256), 0, s, a);
  } else {
    hipLaunchKernelGGL((tile_gemm_kernel<T, 1>), dim3((unsigned)tiles, 1), dim3(256), 0, s, a);
  }
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
                                                           int add_existing) {
  typedef typename VecOf<T, VEC>::type V;
  int rows_per_block = 256 / G;
  long long row = (long long)blockIdx.x * rows_per_block + threadIdx.x / G;
  int sub = threadIdx.x % G;
  if (row >= n_out) return;
  int e0 = ocsr[row], e1 = ocsr[row + 1];
  if (add_existing && e0 == e1) return;
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
#pragma unroll
    for (int j = 0; j < VEC; ++j) reinterpret_cast<T *>(&y)[j] = (T)acc[j];
    *reinterpret_cast<V *>(&out[row * c_out + (long long)v * VEC]) = y;
  }
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

static unsigned g_stage_mask = 0xFFFFFFFFu;
extern "C" void pce_set_stage_mask(uint32_t mask) { g_stage_mask = mask; }
static inline bool stage_on(int bit) { return (g_stage_mask >> bit) & 1u; }

static int pow2_at_least(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

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
static TileArgs base_args(const void *in, const void *w, const void *wp, int kv, int c_in, int c_out) {
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  TileArgs a = {};
  a.A = in;
  a.W = w;
  a.Wp = sizeof(T) == 2 ? wp : nullptr;
  a.kv = kv;
  a.c_in = c_in;
  a.c_out = c_out;
  a.k8_total = (c_in + 7) / 8;
  a.n_pad = (c_out + 31) / 32 * 32;
  a.a_vec = (c_in % VEC == 0) && aligned16(in);
  a.w_vec = (c_out % VEC == 0) && aligned16(w);
  return a;
}

template <typename T>
static void set_out(TileArgs *a, void *out, bool f32out) {
  int vec = (f32out || sizeof(T) == 4) ? 4 : 8;
  a->out = out;
  a->o_vec = (a->c_out % vec == 0) && aligned16(out);
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
                    float *acc, hipStream_t s) {
  TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out);
  set_out<T>(&a, acc, true);
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
  return PCE_OK;
}

extern "C" int pce_conv_fwd_fod(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid, const int32_t *imap,
                                const int32_t *omap, const int32_t *kpos, const int32_t *qkpos, int64_t qsum, void *ws,
                                int64_t ws_bytes, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_fod", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_fwd_fod", qsum))) return rc;
  if (qsum > 0 && (!imap || !omap || !kpos || !qkpos)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod: null map pointer");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16) {
    int64_t need = pce_conv_fod_workspace_bytes(n_out, c_out, dtype);
    if (!ws || ws_bytes < need) PCE_FAIL(PCE_EWORKSPACE, "pce_conv_fwd_fod: fp16 needs an fp32 accumulator of %lld bytes", (long long)need);
    if (!aligned16(ws) || !aligned16(out)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod: workspace and output must be 16-byte aligned");
    return fod_impl<half_t>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, qsum, (float *)ws, s);
  }
  if (!aligned16(out)) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fod: output must be 16-byte aligned");
  return fod_impl<float>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, omap, kpos, qkpos, qsum, (float *)out, s);
}

template <typename T>
static int launch_scatter(const T *buf_out, T *out, int64_t n_out, int c_out, const int *ocsr, const int *ocode,
                          const int *qkpos, int add_existing, hipStream_t s) {
  constexpr int VEC = sizeof(T) == 2 ? 8 : 4;
  bool vec_out = (c_out % VEC == 0) && aligned16(out) && aligned16(buf_out);
  if (vec_out) {
    int G = pow2_at_least(c_out / VEC);
    if (G > 64) G = 64;
    hipLaunchKernelGGL((scatter_rows_kernel<T, VEC>), dim3((unsigned)pce_div_up(n_out, 256 / G)), dim3(256), 0, s,
                       buf_out, (long long)n_out, c_out, G, ocsr, ocode, qkpos, out, add_existing);
  } else {
    int G = pow2_at_least(c_out);
    if (G > 64) G = 64;
    hipLaunchKernelGGL((scatter_rows_kernel<T, 1>), dim3((unsigned)pce_div_up(n_out, 256 / G)), dim3(256), 0, s,
                       buf_out, (long long)n_out, c_out, G, ocsr, ocode, qkpos, out, add_existing);
  }
  PCE_LAUNCH_CHECK("scatter_rows");
  return PCE_OK;
}

template <typename T>
static int gms_impl(const void *in, const void *w, const void *wp, void *out, int64_t n_in, int64_t n_out, int c_in,
                    int c_out, int kv, int mid, const int *icsr, const int *icode, const int *ocsr, const int *ocode,
                    const int *kpos, const int *qkpos, int64_t qsum, T *buffer, hipStream_t s) {
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
    set_out<T>(&a, buf_out, false);
    a.kpos = kpos;
    a.qkpos = qkpos;
    a.mode = MODE_BUF;
    a.epi = EPI_ROWS;
    if ((rc = launch_tile<T>(a, qsum / PCE_QUANTUM, s))) return rc;
  }
  if (mid >= 0 && stage_on(0)) {
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out);
    set_out<T>(&a, out, false);
    a.mode = MODE_DENSE;
    a.epi = EPI_ROWS;
    a.w_fixed = mid;
    a.n_rows = n_out;
    if ((rc = launch_tile<T>(a, pce_div_up(n_out, 128), s))) return rc;
  }
  if (!stage_on(2)) return PCE_OK;
  // scatter: output-stationary sum over each row's staging rows, fp32 accumulate
  return launch_scatter<T>(buf_out, (T *)out, n_out, c_out, ocsr, ocode, qkpos, mid >= 0 ? 1 : 0, s);
}

extern "C" int pce_conv_fwd_gms(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid,
                                const int32_t *icsr, const int32_t *icode, const int32_t *ocsr, const int32_t *ocode,
                                const int32_t *kpos, const int32_t *qkpos, int64_t qsum, void *buffer,
                                int64_t buffer_elems, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_gms", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_fwd_gms", qsum))) return rc;
  if (!icsr || !ocsr || !kpos || !qkpos || (qsum > 0 && (!icode || !ocode))) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_gms: null map pointer");
  if (qsum > 0 && (!buffer || buffer_elems < qsum * ((int64_t)c_in + c_out)))
    PCE_FAIL(PCE_EWORKSPACE, "pce_conv_fwd_gms: buffer holds %lld elements, needs %lld", (long long)buffer_elems, (long long)(qsum * ((int64_t)c_in + c_out)));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16)
    return gms_impl<half_t>(in, w, wp, out, n_in, n_out, c_in, c_out, kv, mid, icsr, icode, ocsr, ocode, kpos, qkpos, qsum, (half_t *)buffer, s);
  return gms_impl<float>(in, w, wp, out, n_in, n_out, c_in, c_out, kv, mid, icsr, icode, ocsr, ocode, kpos, qkpos, qsum, (float *)buffer, s);
}

// Fetch-on-demand with deferred scatter: pair tiles gather their input rows, multiply and store
// the partial rows to the staging buffer (no atomics); the scatter is the epilogue of the centre
// GEMM, which adds each output row's staging rows in fp32 and stores the row once.
template <typename T>
static int fds_impl(const void *in, const void *w, const void *wp, void *out, int64_t n_out, int c_in, int c_out, int kv,
                    int mid, const int *imap, const int *kpos, const int *qkpos, const int32_t *kpos_host,
                    const int32_t *qkpos_host, const int *ocsr, const int *ocode, int64_t qsum, T *buffer,
                    hipStream_t s) {
  int rc;
  if (qsum > 0 && stage_on(1)) {
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out);
    set_out<T>(&a, buffer, false);
    set_host_pos(&a, kpos_host, qkpos_host);
    a.imap = imap;
    a.kpos = kpos;
    a.qkpos = qkpos;
    a.mode = MODE_FOD_BUF;
    a.epi = EPI_ROWS;
    if ((rc = launch_tile<T>(a, qsum / PCE_QUANTUM, s))) return rc;
  }
  if (!stage_on(2)) return PCE_OK;
  if (mid >= 0) {
    TileArgs a = base_args<T>(in, w, wp, kv, c_in, c_out);
    set_out<T>(&a, out, false);
    set_host_pos(&a, kpos_host, qkpos_host);
    a.qkpos = qkpos;
    a.mode = MODE_DENSE;
    a.epi = EPI_ROWS_CSR;
    a.w_fixed = mid;
    a.n_rows = n_out;
    a.ocsr = ocsr;
    a.ocode = ocode;
    a.buf = buffer;
    a.b_vec = a.o_vec && aligned16(buffer);
    return launch_tile<T>(a, pce_div_up(n_out, 128), s);
  }
  return launch_scatter<T>(buffer, (T *)out, n_out, c_out, ocsr, ocode, qkpos, 0, s);
}

extern "C" int pce_conv_fwd_fds(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                                int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, int32_t mid, const int32_t *imap,
                                const int32_t *kpos, const int32_t *qkpos, const int32_t *kpos_host,
                                const int32_t *qkpos_host, const int32_t *ocsr, const int32_t *ocode, int64_t qsum,
                                void *buffer, int64_t buffer_elems, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_fds", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, mid);
  if (rc || (rc = check_qsum("pce_conv_fwd_fds", qsum))) return rc;
  if (!ocsr || !kpos || !qkpos || (qsum > 0 && (!imap || !ocode))) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_fds: null map pointer");
  if (qsum > 0 && (!buffer || buffer_elems < qsum * (int64_t)c_out))
    PCE_FAIL(PCE_EWORKSPACE, "pce_conv_fwd_fds: buffer holds %lld elements, needs %lld", (long long)buffer_elems, (long long)(qsum * (int64_t)c_out));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16)
    return fds_impl<half_t>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, kpos, qkpos, kpos_host, qkpos_host, ocsr, ocode, qsum, (half_t *)buffer, s);
  return fds_impl<float>(in, w, wp, out, n_out, c_in, c_out, kv, mid, imap, kpos, qkpos, kpos_host, qkpos_host, ocsr, ocode, qsum, (float *)buffer, s);
}

extern "C" int pce_conv_fwd_os(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n_in,
                               int64_t n_out, int32_t c_in, int32_t c_out, int32_t kv, const int32_t *nbr,
                               pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_os", in, w, out, dtype, n_in, n_out, c_in, c_out, kv, -1);
  if (rc) return rc;
  if (!nbr) PCE_FAIL(PCE_EINVAL, "pce_conv_fwd_os: null neighbour table");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16) {
    TileArgs a = base_args<half_t>(in, w, wp, kv, c_in, c_out);
    set_out<half_t>(&a, out, false);
    a.nbr = nbr;
    a.n_rows = n_out;
    a.mode = MODE_OS;
    a.epi = EPI_ROWS;
    return launch_tile<half_t>(a, pce_div_up(n_out, 128), s);
  }
  TileArgs a = base_args<float>(in, w, wp, kv, c_in, c_out);
  set_out<float>(&a, out, false);
  a.nbr = nbr;
  a.n_rows = n_out;
  a.mode = MODE_OS;
  a.epi = EPI_ROWS;
  return launch_tile<float>(a, pce_div_up(n_out, 128), s);
}

extern "C" int pce_conv_fwd_dense(const void *in, const void *w, const void *wp, void *out, int32_t dtype, int64_t n,
                                  int32_t c_in, int32_t c_out, pce_stream_t stream) {
  int rc = check_common("pce_conv_fwd_dense", in, w, out, dtype, n, n, c_in, c_out, 1, -1);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PCE_F16) {
    TileArgs a = base_args<half_t>(in, w, wp, 1, c_in, c_out);
    set_out<half_t>(&a, out, false);
    a.n_rows = n;
    a.mode = MODE_DENSE;
    a.epi = EPI_ROWS;
    return launch_tile<half_t>(a, pce_div_up(n, 128), s);
  }
  TileArgs a = base_args<float>(in, w, wp, 1, c_in, c_out);
  set_out<float>(&a, out, false);
  a.n_rows = n;
  a.mode = MODE_DENSE;
  a.epi = EPI_ROWS;
  return launch_tile<float>(a, pce_div_up(n, 128), s);
}

// Map density rho = pairs per output row.  With few pairs per row the fetch-on-demand family wins:
// it moves each pair's rows once and stages one weight tile per 128 pairs; the deferred-scatter
// form replaces the atomics and the fp32 accumulator of the plain form by a small staging buffer.
// The output-stationary kernel re-stages a weight tile per (row tile, offset) but never touches an
// accumulator in memory, so it wins once most offsets of a 128-row tile are populated.  The staged
// gather-GEMM-scatter dataflow pays 2*M*(c_in+c_out) of buffer traffic and is chosen only where
// its plain streaming GEMM dominates (wide channels on a moderately dense map).
extern "C" int pce_select_dataflow(int64_t n_in, int64_t n_out, int64_t n_pairs, int32_t c_in, int32_t c_out, int32_t kv,
                                   int32_t dtype) {
  (void)n_in;
  (void)dtype;
  (void)c_in;
  (void)c_out;
  if (n_out <= 0) return PCE_DATAFLOW_FDS;
  double rho = (double)n_pairs / (double)n_out;
  if (kv == 1) return PCE_DATAFLOW_OS;
  if (rho >= 2.0) return PCE_DATAFLOW_OS;
  return PCE_DATAFLOW_FDS;
}
