// conv_nd forward / data-gradient / filter-gradient as implicit GEMMs on the
// gfx950 matrix cores (v_mfma_f32_16x16x4_f32, v_mfma_f64_16x16x4_f64).
//
// No im2col matrix is ever written to HBM.  A block gathers its operand tiles
// straight from the NCHW tensors into LDS -- zero padding is a predicate on the
// gathered coordinate -- and the 64-wide wavefronts feed the MFMA units from
// LDS.  Three GEMM views (the closed-form sums are in the header):
//
//   forward   M = F, K = (c, tap),        N = (n, g)     gathers x
//   dgrad     M = C, K = (f, tap),        N = (n, i)     gathers grad; a stride
//             > 1 splits the input pixels i into prod(stride) phases, each a
//             dense smaller convolution with its own slice of the (f, tap) table
//   wgrad     M = F, N = (c, tap),        K = (n, g)     gathers grad and x; the
//             long K is split over blocks, partial sums are added in a fixed
//             order by a second kernel (no atomics, run-to-run identical)
#include "conv_kernels.h"
#include "internal.h"

#include <algorithm>
#include <array>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace mg {

// Tables that every lane of a wavefront reads at the same index are addressed
// through the constant address space, which lets the compiler fetch them with
// scalar loads (one request per wavefront, no vector-memory wait) instead of 64
// identical vector loads.
#define MG_CONSTANT __attribute__((address_space(4)))
typedef int int4v __attribute__((ext_vector_type(4)));
static_assert(sizeof(TabEntry) == sizeof(int4v), "a table row is read as one 16-byte vector");
__device__ __forceinline__ const int4v MG_CONSTANT *as_constant(const TabEntry *p) {
  return (const int4v MG_CONSTANT *)(p);
}
__device__ __forceinline__ const int MG_CONSTANT *as_constant(const int *p) { return (const int MG_CONSTANT *)(p); }
__device__ __forceinline__ TabEntry table_row(const int4v MG_CONSTANT *tab, int i) {
  const int4v v = tab[i];
  return TabEntry{v.x, v.y, v.z, v.w};
}
// The wavefront-uniform value of x as a scalar register.
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

// D(16x16) += A(16x4) * B(4x16) on one wavefront.  Lane l supplies A[l%16][l/16]
// and B[l/16][l%16].  Lane l receives four elements of column l%16 of D; their
// rows are row_of(l, r), r = 0..3, which differs between the two instructions.
template <typename T>
struct Mma;

template <>
struct Mma<float> {
  using Acc = f32x4;
  static __device__ __forceinline__ Acc run(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row_of(int lane, int r) { return 4 * (lane >> 4) + r; }
};

template <>
struct Mma<double> {
  using Acc = f64x4;
  static __device__ __forceinline__ Acc run(double a, double b, Acc c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row_of(int lane, int r) { return 4 * r + (lane >> 4); }
};

// ------------------------------------------------------------------------------------------
// filter packing: the tap-major GEMMs want the filter operand with M contiguous
//   mode 2 (forward) : Ap[(t*C + c)][f] = w[f][c][t]
//   mode 3 (dgrad)   : Ap[(t*F + f)][c] = w[f][c][t]
//   mode 6 (forward, K tiles of table rows) : Ap[(c*taps + t)][f] = w[f][c][t]
//   modes 4 / 5 (dgrad / forward with the three taps t2 of the last axis folded into the rows;
//           u is the tap of the other axes):
//           Ap[(u*F + f)][3*c + t2] = w[f][c][u][t2]      Ap[(u*C + c)][3*f + 2 - t2] = w[f][c][u][t2]
//           (the row of a tap is added to dst one position to the right of the row after it:
//           the forward pass reads x to the right of a later tap, the gradient to the left)
// Every row is padded with zeros to a multiple of four values (`ld` values per row), so
// that the kernels can read a row sixteen bytes at a time whatever M is.  (The
// table-driven kernel reads the filter bank in place.)
// ------------------------------------------------------------------------------------------
// One tap, forward, tap-major (mode 2 with wvol == 1 and ld == F): Ap[c][f] = w[f][c], a plain
// transposition of an F x C matrix -- what a matrix product's left operand needs.  32 x 32
// tiles through LDS: read along c, written along f, both coalesced.
template <typename T>
__global__ void __launch_bounds__(256) pack_transpose_kernel(const T *__restrict__ w, T *__restrict__ ap, int F, int C) {
  __shared__ T tile[32][33];
  const int c0 = blockIdx.x * 32, f0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int f = f0 + ty + 8 * j, c = c0 + tx;
    if (f < F && c < C) tile[ty + 8 * j][tx] = w[(long long)f * C + c];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = c0 + ty + 8 * j, f = f0 + tx;
    if (f < F && c < C) ap[(long long)c * F + f] = tile[tx][ty + 8 * j];
  }
}

// Stride phases as rows (see GemmParams::phase_count): Ap[(e * F + f)][c * phases + phase] = w[f][c][tap of offset e in
// that phase], zero where the phase has no tap at that offset; taps[e * phases + phase] names the tap (-1: none).
template <typename T>
__global__ void __launch_bounds__(256) pack_phase_rows_kernel(const T *__restrict__ w, T *__restrict__ ap, const int *__restrict__ taps,
                                                              int entries, int phases, int F, int C, int wvol, int ld) {
  const long long total = (long long)entries * F * ld;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
    const int m = (int)(idx % ld);
    const long long row = idx / ld;
    const int f = (int)(row % F), e = (int)(row / F);
    T v = T(0);
    if (m < phases * C) {
      const int tap = taps[e * phases + m % phases];
      if (tap >= 0) v = w[((long long)f * C + m / phases) * wvol + tap];
    }
    ap[idx] = v;
  }
}

template <typename T>
__global__ void __launch_bounds__(256) pack_filters_kernel(const T *__restrict__ w, T *__restrict__ ap, int F, int C,
                                                           int wvol, int mode, int ld) {
  const int M = (mode == 2 || mode == 6) ? F : mode == 3 ? C : mode == 4 ? 3 * C : 3 * F;
  const int total = (F * C * wvol / M) * ld;
  for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
    // idx enumerates the packed layout so that stores are coalesced
    const int m = idx % ld;
    const int row = idx / ld;
    if (sizeof(T) == 8 && mode >= 4 && mode <= 5) {
      // double precision orders the folded rows (block of 16, tap, one of the 16): the wave tile of
      // its MFMA holds a lane's two rows of each tap 16 rows apart
      const int n = mode == 4 ? C : F;
      const int one = (m / 48) * 16 + m % 16, tap = (m % 48) / 16;
      T v = T(0);
      if (one < n) {
        const int f = mode == 4 ? row % F : one, c = mode == 4 ? one : row % C;
        const int t = (row / (mode == 4 ? F : C)) * 3 + (mode == 4 ? tap : 2 - tap);
        v = w[((long long)f * C + c) * wvol + t];
      }
      ap[idx] = v;
      continue;
    }
    if (m >= M) {
      ap[idx] = T(0);
      continue;
    }
    int f, c, t;
    if (mode == 2) {
      f = m;
      c = row % C;
      t = row / C;
    } else if (mode == 6) {
      f = m;
      t = row % wvol;
      c = row / wvol;
    } else if (mode == 3) {
      c = m;
      f = row % F;
      t = row / F;
    } else if (mode == 4) {
      c = m / 3;
      f = row % F;
      t = (row / F) * 3 + m % 3;
    } else {
      f = m / 3;
      c = row % C;
      t = (row / C) * 3 + 2 - m % 3;
    }
    ap[idx] = w[((long long)f * C + c) * wvol + t];
  }
}

// Packed filters of a data gradient on table rows: Ap[k][c] = w[arow[k] + c * taps], where arow[k]
// is the offset of row k's (filter, tap) for channel 0, or negative for a padding row (zeros).
template <typename T>
__global__ void __launch_bounds__(256) pack_rows_kernel(const T *__restrict__ w, T *__restrict__ ap, const int *__restrict__ arow,
                                                        int rows, int C, int wvol, int ld) {
  const int total = rows * ld;
  for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
    const int c = idx % ld, k = idx / ld;
    const int at = arow[k];
    ap[idx] = (c < C && at >= 0) ? w[(long long)at + (long long)c * wvol] : T(0);
  }
}

// ------------------------------------------------------------------------------------------
// gather-GEMM (forward and data gradient)
// ------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int BK, int WM, int WN>
__global__ void __launch_bounds__(256) gather_gemm_kernel(const GemmParams p) {
  static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per block");
  static_assert(BK % 4 == 0 && WM % 16 == 0 && WN % 16 == 0, "MFMA 16x16x4 tiling");
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int WAVES_N = BN / WN;
  constexpr int AROWS = 256 / BM;  // table rows covered by one pass of the block over the A tile
  constexpr int ALOADS = (BK + AROWS - 1) / AROWS;
  constexpr int BROWS = 256 / BN;
  constexpr int BLOADS = (BK + BROWS - 1) / BROWS;
  constexpr int LDA = BM + 4, LDB = BN + 4;

  __shared__ T As[2][BK][LDA];
  __shared__ T Bs[2][BK][LDB];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WM;
  const int wn0 = (wave % WAVES_N) * WN;

  // which phase does this block belong to
  int pi = 0;
  while (pi + 1 < p.nphases && (int)blockIdx.x >= p.phases[pi + 1].blk_begin) ++pi;
  const Phase ph = p.phases[pi];
  const int pos0 = ((int)blockIdx.x - ph.blk_begin) * BN;
  const int m0 = blockIdx.y * BM;
  const int j12 = ph.J[1] * ph.J[2];
  const int jvol = ph.J[0] * j12;

  const T *__restrict__ A = static_cast<const T *>(p.A);
  const int4v MG_CONSTANT *tab = as_constant(p.tab + ph.k_begin);
  const int MG_CONSTANT *arow = as_constant(p.arow + ph.k_begin);

  // ---- loader state: this thread's position in the B tile
  static_assert(BN % 64 == 0, "a wavefront loads one table row of the B tile at a time");
  const int bcol = tid % BN;
  const int brow0 = uniform(tid / BN);
  int qb0 = 0, qb1 = 0, qb2 = 0, lin = 0;
  const bool pos_ok = pos0 + bcol < ph.npos;
  const T *__restrict__ srcn = static_cast<const T *>(p.src);
  {
    const unsigned pos = pos_ok ? (unsigned)(pos0 + bcol) : 0u;
    const unsigned n = ph.by_jvol.div(pos);
    unsigned r = pos - n * (unsigned)jvol;
    const unsigned j0 = ph.by_j12.div(r);
    r -= j0 * (unsigned)j12;
    const unsigned j1 = ph.by_j2.div(r);
    const unsigned j2 = r - j1 * (unsigned)ph.J[2];
    qb0 = (int)j0 * p.sj[0];
    qb1 = (int)j1 * p.sj[1];
    qb2 = (int)j2 * p.sj[2];
    lin = qb0 * p.qs[0] + qb1 * p.qs[1] + qb2 * p.qs[2];
    srcn += (long long)n * p.src_nstride;
  }
  const int acol = tid % BM;
  const int arow0 = BM % 64 == 0 ? uniform(tid / BM) : tid / BM;
  const bool m_ok = (m0 + acol) < p.M;
  const int acol_safe = m_ok ? m0 + acol : 0;
  const int klast = ph.k_count - 1;

  T ra[ALOADS], rb[BLOADS];
  bool oka[ALOADS], okb[BLOADS];

  // Every load is issued unconditionally from a clamped (always valid) address and
  // the padding zeros are selected afterwards, so that the loads of a tile go out
  // back to back instead of sitting behind one branch each.
  auto fetch = [&](int kt) {
    const int kbase = kt * BK;
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) {
      const int kk = arow0 + r * AROWS;
      const int kidx = kbase + kk;
      oka[r] = (kk < BK) & (kidx <= klast) & m_ok;
      const int row = arow[min(kidx, klast)];
      ra[r] = A[(long long)row + (long long)acol_safe * p.a_mstride];
    }
#pragma unroll
    for (int r = 0; r < BLOADS; ++r) {
      const int kk = brow0 + r * BROWS;
      const int kidx = kbase + kk;
      const TabEntry e = table_row(tab, min(kidx, klast));
      const bool ok = (kk < BK) & (kidx <= klast) & pos_ok & ((unsigned)(qb0 + e.d0) < (unsigned)p.Q[0]) &
                      ((unsigned)(qb1 + e.d1) < (unsigned)p.Q[1]) & ((unsigned)(qb2 + e.d2) < (unsigned)p.Q[2]);
      okb[r] = ok;
      rb[r] = srcn[ok ? lin + e.off : 0];
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) {
      const int kk = arow0 + r * AROWS;
      if (kk < BK) As[buf][kk][acol] = oka[r] ? ra[r] : T(0);
    }
#pragma unroll
    for (int r = 0; r < BLOADS; ++r) {
      const int kk = brow0 + r * BROWS;
      if (kk < BK) Bs[buf][kk][bcol] = okb[r] ? rb[r] : T(0);
    }
  };

  typename Mma<T>::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = typename Mma<T>::Acc{0, 0, 0, 0};

  const int ktiles = (ph.k_count + BK - 1) / BK;
  int buf = 0;
  if (ktiles > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();
  for (int kt = 0; kt < ktiles; ++kt) {
    const bool more = kt + 1 < ktiles;
    if (more) fetch(kt + 1);
    const int l16 = lane & 15, lk = lane >> 4;
#pragma unroll
    for (int k4 = 0; k4 < BK / 4; ++k4) {
      T a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[buf][k4 * 4 + lk][wm0 + i * 16 + l16];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Bs[buf][k4 * 4 + lk][wn0 + j * 16 + l16];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mma<T>::run(a[i], b[j], acc[i][j]);
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  // ---- epilogue: lane owns column (lane % 16) of every 16x16 tile
  T *__restrict__ dst = static_cast<T *>(p.dst);
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int ipos = pos0 + wn0 + j * 16 + (lane & 15);
    if (ipos >= ph.npos) continue;
    const unsigned pos = (unsigned)ipos;
    const unsigned n = ph.by_jvol.div(pos);
    unsigned r = pos - n * (unsigned)jvol;
    const int j0 = (int)ph.by_j12.div(r);
    r -= (unsigned)j0 * (unsigned)j12;
    const int j1 = (int)ph.by_j2.div(r);
    const int j2 = (int)r - j1 * ph.J[2];
    T *out = dst + (long long)n * p.dst_nstride + (long long)(ph.o0[0] + j0 * p.oj[0]) * p.os[0] +
             (long long)(ph.o0[1] + j1 * p.oj[1]) * p.os[1] + (long long)(ph.o0[2] + j2 * p.oj[2]) * p.os[2];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m0 + wm0 + i * 16 + Mma<T>::row_of(lane, q);
        if (m < p.M) out[(long long)m * p.dst_mstride] = acc[i][j][q];
      }
  }
}

// ------------------------------------------------------------------------------------------
// filter gradient: split-K GEMM over positions, then a fixed-order reduction
// ------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int BK, int WM, int WN>
__global__ void __launch_bounds__(256) wgrad_kernel(const WgradParams p) {
  static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per block");
  static_assert(256 % BK == 0 && BK % 4 == 0, "K tile");
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int WAVES_N = BN / WN;
  constexpr int ROWS = 256 / BK;  // tile rows covered by one pass of the block
  constexpr int ALOADS = (BM + ROWS - 1) / ROWS;
  constexpr int BLOADS = (BN + ROWS - 1) / ROWS;
  constexpr int LDK = BK + 2;

  __shared__ T As[2][BM][LDK];  // grad tile   [f][position]
  __shared__ T Bs[2][BN][LDK];  // window tile [column][position]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WM;
  const int wn0 = (wave % WAVES_N) * WN;
  const int n0 = blockIdx.x * BN;  // first column (c, tap)
  const int m0 = blockIdx.y * BM;  // first filter
  const int kbeg = (int)blockIdx.z * p.kchunk;
  const int kend = min(kbeg + p.kchunk, p.kpos);

  const T *__restrict__ grad = static_cast<const T *>(p.grad);
  const T *__restrict__ x = static_cast<const T *>(p.x);
  const int kcol = tid % BK;  // this thread's position inside the K tile
  const int row0 = BK % 64 == 0 ? uniform(tid / BK) : tid / BK;
  const int g12 = p.G[1] * p.G[2];
  const int4v MG_CONSTANT *tab = as_constant(p.tab);

  T ra[ALOADS], rb[BLOADS];
  bool oka[ALOADS], okb[BLOADS];

  // Unconditional loads from clamped addresses, zeros selected afterwards (see the
  // gather-GEMM above).  A thread keeps one position of the K tile and walks the
  // tile's rows, so the position is decoded once per tile.
  auto fetch = [&](int kt) {
    const int ipos = kbeg + kt * BK + kcol;
    const bool pos_ok = ipos < kend;
    const unsigned pos = pos_ok ? (unsigned)ipos : (unsigned)kbeg;
    const unsigned n = p.by_gvol.div(pos);
    const unsigned gflat = pos - n * (unsigned)p.gvol;
    const unsigned g0 = p.by_g12.div(gflat);
    const unsigned r12 = gflat - g0 * (unsigned)g12;
    const unsigned g1 = p.by_g2.div(r12);
    const unsigned g2 = r12 - g1 * (unsigned)p.G[2];
    const int qb0 = (int)g0 * p.sj[0];
    const int qb1 = (int)g1 * p.sj[1];
    const int qb2 = (int)g2 * p.sj[2];
    const int lin = qb0 * p.qs[0] + qb1 * p.qs[1] + qb2 * p.qs[2];
    const T *gn = grad + (long long)n * p.g_nstride + gflat;
    const T *xn = x + (long long)n * p.x_nstride;
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) {
      const int row = row0 + r * ROWS;
      const int f = m0 + row;
      oka[r] = (row < BM) & pos_ok & (f < p.F);
      ra[r] = gn[(long long)min(f, p.F - 1) * p.gvol];
    }
#pragma unroll
    for (int r = 0; r < BLOADS; ++r) {
      const int row = row0 + r * ROWS;
      const int col = n0 + row;
      const TabEntry e = table_row(tab, min(col, p.CT - 1));
      const bool ok = (row < BN) & pos_ok & (col < p.CT) & ((unsigned)(qb0 + e.d0) < (unsigned)p.Q[0]) &
                      ((unsigned)(qb1 + e.d1) < (unsigned)p.Q[1]) & ((unsigned)(qb2 + e.d2) < (unsigned)p.Q[2]);
      okb[r] = ok;
      rb[r] = xn[ok ? lin + e.off : 0];
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) {
      const int row = row0 + r * ROWS;
      if (row < BM) As[buf][row][kcol] = oka[r] ? ra[r] : T(0);
    }
#pragma unroll
    for (int r = 0; r < BLOADS; ++r) {
      const int row = row0 + r * ROWS;
      if (row < BN) Bs[buf][row][kcol] = okb[r] ? rb[r] : T(0);
    }
  };

  typename Mma<T>::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = typename Mma<T>::Acc{0, 0, 0, 0};

  const int ktiles = kend > kbeg ? (kend - kbeg + BK - 1) / BK : 0;
  int buf = 0;
  if (ktiles > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();
  for (int kt = 0; kt < ktiles; ++kt) {
    const bool more = kt + 1 < ktiles;
    if (more) fetch(kt + 1);
    const int l16 = lane & 15, lk = lane >> 4;
#pragma unroll
    for (int k4 = 0; k4 < BK / 4; ++k4) {
      T a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[buf][wm0 + i * 16 + l16][k4 * 4 + lk];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Bs[buf][wn0 + j * 16 + l16][k4 * 4 + lk];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mma<T>::run(a[i], b[j], acc[i][j]);
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  T *__restrict__ out = static_cast<T *>(p.out) + (long long)blockIdx.z * p.F * p.CT;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn0 + j * 16 + (lane & 15);
    if (col >= p.CT) continue;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int f = m0 + wm0 + i * 16 + Mma<T>::row_of(lane, q);
        if (f < p.F) out[(long long)f * p.CT + col] = acc[i][j][q];
      }
  }
}

// ((p[0] + p[stride]) + p[2*stride]) + ... over `terms` terms: always this order, so
// the result does not change from run to run; sixteen loads are in flight at a time
// (the partial sums were written by other XCDs a moment ago: every load is a trip
// past this XCD's L2).
template <typename T>
__device__ __forceinline__ T sum_in_order(const T *__restrict__ p, long long stride, int terms) {
  constexpr int BATCH = 16;
  T s = p[0];
  int k = 1;
  for (; k + BATCH <= terms; k += BATCH) {
    T v[BATCH];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) v[u] = p[(long long)(k + u) * stride];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) s += v[u];
  }
  if (k < terms) {
    // the rest in one more batch: loads past the end repeat the last term and are not added
    T v[BATCH];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) v[u] = p[(long long)min(k + u, terms - 1) * stride];
#pragma unroll
    for (int u = 0; u < BATCH; ++u)
      if (k + u < terms) s += v[u];
  }
  return s;
}

// dw[i] = ((part[0][i] + part[1][i]) + part[2][i]) + ...   (fixed order)
// RUNS > 1: the splits are cut into RUNS consecutive runs, each summed in order by its own
// thread, and the runs' totals are added in order (for a small dw, where one thread per
// element would leave most of the device idle behind a long chain of dependent loads).
template <typename T, int RUNS>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const T *__restrict__ part, T *__restrict__ dw, int count,
                                                            int splits) {
  constexpr int WIDTH = 256 / RUNS;
  const int q = threadIdx.x / WIDTH, lane = threadIdx.x % WIDTH;
  const int i = blockIdx.x * WIDTH + lane;
  if constexpr (RUNS == 1) {
    if (i < count) dw[i] = sum_in_order(part + i, count, splits);
    return;
  }
  __shared__ T runs[RUNS][WIDTH];
  const int per = (splits + RUNS - 1) / RUNS;
  const int first = min(q * per, splits), last = min(first + per, splits);
  // an empty run holds +0.0, which changes no total (a total of -0.0 cannot come out of
  // accumulators that start from +0.0)
  runs[q][lane] = (i < count && first < last) ? sum_in_order(part + (long long)first * count + i, count, last - first) : T(0);
  __syncthreads();
  if (q == 0 && i < count) {
    T sum = runs[0][lane];
#pragma unroll
    for (int r = 1; r < RUNS; ++r) sum += runs[r][lane];
    dw[i] = sum;
  }
}

}  // namespace mg

#include "conv_tap_kernels.h"

namespace mg {

// ------------------------------------------------------------------------------------------
// host side: descriptor checks, cached plans (tables live in device memory), launches
// ------------------------------------------------------------------------------------------
namespace {

enum ConvOp { OP_FWD = 0, OP_DGRAD = 1, OP_WGRAD = 2 };

struct Geometry {
  int nd, dtype;
  int N, C, F;
  int X[3], W[3], G[3], S[3], P[3], D[3];
  long long xvol, wvol, gvol;
};

// The tap-major kernels address their operands with 32-bit byte offsets and mark
// padding with an offset of 2 GiB, so every tensor they read must be smaller.
bool fits_buffer_loads(const Geometry &g) {
  const long long elem = g.dtype == MG_F64 ? 8 : 4;
  const long long limit = 1ll << 31;
  return (long long)g.N * g.C * g.xvol * elem < limit && (long long)g.N * g.F * g.gvol * elem < limit &&
         (long long)(g.F + 3) * (g.C + 3) * g.wvol * elem < limit;  // packed filter rows are padded to 4 values
}

// K tile of the gather-GEMMs (positions x filters-or-channels x BK).
int gemm_bk(int dtype) { return dtype == MG_F64 ? 8 : 16; }
// K tile of a tap-major plan that contracts `channels` channels per tap.  Double precision: 16
// where the channels allow it -- a K tile of 8 is 64 MFMAs per wave between two barriers, and
// the barriers then cost a tenth of the time (config 4: forward 122 -> 115 us, dx 130 -> 119 us).
int tap_bk(int dtype, int channels) { return dtype == MG_F64 && channels % 16 != 0 ? 8 : 16; }

struct Plan {
  void *blob = nullptr;  // one device allocation holding every table below
  TabEntry *tab = nullptr;
  int *arow = nullptr;
  Phase *phases = nullptr;
  KTile *ktiles = nullptr;
  WGroup *groups = nullptr;
  void *zeros = nullptr;
  int nphases = 0;
  int pos_blocks = 0;  // position blocks of the gather-GEMM (all phases)
  int bm = 0, bn = 0;
  int bk = 0;           // depth of a K tile of the kernel chosen for this plan
  void *pos_tab = nullptr;  // filter gradient: one row per position (WgradParams::pos_tab), its own allocation
  int m_tiles = 1;     // row tiles per position block
  int full_tiles = 0;  // tiles computed whole by one block (tap-major kernel)
  int tail_split = 1;  // blocks sharing each of the remaining tiles
  int blocks_per_cu = 1;  // persistent blocks per compute unit (streaming gather-GEMM)
  // even shares of the last round (GemmParams::share_first): set by upload_plan when tail_split == 0
  int *share_first = nullptr;
  ShareSlice *share_slices = nullptr;
  ShareFix *share_fix = nullptr;
  int share_grid = 0, share_slots = 0, share_fixes = 0;
  bool tap_major = false;  // which kernel family the tables are for
  bool single_dense_phase = false;  // positions enumerate the destination tensor in order
  bool table_rows = false;          // tap-major kernel whose K tiles are rows of the gather table (channel count no multiple of the K tile)
  int table_count = 0;              // data gradient on table rows: rows of the (padded) table = rows of the packed filters
  int fold_row = 0;                 // data gradient with the last axis' three taps folded into the rows: length of a row of positions
  int phase_rows = 0;               // data gradient with the stride phases as rows of the GEMM (GemmParams::phase_count): the channel count
  int phase_count = 0;              // ... and the number of phases; table_count is then the number of distinct gathered offsets
  bool deep_k = false;              // table-driven, a few microseconds of work: 16 x 64 tiles with a K tile four times as deep
  // fused stride phases of the data gradient (see GemmParams::nph)
  int nph = 1;
  int kcut[4] = {0, 0, 0, 0};
  int po0[4][3] = {};
  int pJ[4][3] = {};
  // few rows, single precision: one position per lane on the 4x4x1 MFMA (see ThinParams)
  bool thin = false;
  int thin_rg = 1;  // groups of four rows
  int thin_chunks = 0, thin_kgroups = 0;
  long long thin_src_group = 0, thin_w_group = 0;  // elements of src / of the filter bank between consecutive groups
  int thin_w_mstride = 0;
  Phase thin_grid{};  // J, npos and divisors of the positions (host copy)
  // wgrad
  int splits = 1;
  int kchunk = 0;
  char note[200] = "";  // what mg_last_plan() reports after a call that ran this plan
};

std::map<std::string, Plan> &plans() {
  static std::map<std::string, Plan> m;
  return m;
}

int check_desc(const mg_conv_desc *d, Geometry *g) {
  if (!d) return fail(MG_ERR_BAD_ARG, "conv descriptor is null");
  if (d->dtype != MG_F32 && d->dtype != MG_F64)
    return fail(MG_ERR_UNSUPPORTED, "conv dtype %d (only float32=0 / float64=1)", d->dtype);
  if (d->nd < 1 || d->nd > MG_MAX_ND) return fail(MG_ERR_UNSUPPORTED, "spatial rank %d (1..%d)", d->nd, MG_MAX_ND);
  if (d->N < 1 || d->C < 1 || d->F < 1)
    return fail(MG_ERR_BAD_ARG, "N=%lld C=%lld F=%lld must be positive", (long long)d->N, (long long)d->C,
                (long long)d->F);
  const long long lim = (1ll << 31) - 4096;
  long long xvol = 1, wvol = 1, gvol = 1;
  for (int k = 0; k < 3; ++k) {
    if (d->X[k] < 1 || d->W[k] < 1 || d->G[k] < 1 || d->stride[k] < 1 || d->dil[k] < 1 || d->pad[k] < 0)
      return fail(MG_ERR_BAD_ARG, "axis %d: X=%lld W=%lld G=%lld stride=%lld dil=%lld pad=%lld", k, (long long)d->X[k],
                  (long long)d->W[k], (long long)d->G[k], (long long)d->stride[k], (long long)d->dil[k],
                  (long long)d->pad[k]);
    if (k < 3 - d->nd &&
        (d->X[k] != 1 || d->W[k] != 1 || d->G[k] != 1 || d->stride[k] != 1 || d->dil[k] != 1 || d->pad[k] != 0))
      return fail(MG_ERR_BAD_ARG, "axis %d lies outside rank %d and must be trivial", k, d->nd);
    if (d->X[k] > lim || d->W[k] > lim || d->stride[k] > lim || d->dil[k] > lim || d->pad[k] > lim)
      return fail(MG_ERR_UNSUPPORTED, "axis %d: extent beyond 2^31", k);
    const long long span = (d->W[k] - 1) * d->dil[k] + 1;
    const long long room = d->X[k] + 2 * d->pad[k] - span;
    if (room < 0 || d->G[k] > room / d->stride[k] + 1)
      return fail(MG_ERR_BAD_ARG, "axis %d: G=%lld exceeds (X+2*pad-span)/stride+1", k, (long long)d->G[k]);
    xvol *= d->X[k];
    wvol *= d->W[k];
    gvol *= d->G[k];
    if (xvol > lim || wvol > lim || gvol > lim) return fail(MG_ERR_UNSUPPORTED, "per-sample volume beyond 2^31");
    g->X[k] = (int)d->X[k];
    g->W[k] = (int)d->W[k];
    g->G[k] = (int)d->G[k];
    g->S[k] = (int)d->stride[k];
    g->P[k] = (int)d->pad[k];
    g->D[k] = (int)d->dil[k];
  }
  // Offsets inside one batch item and position counts are 32-bit in the kernels.
  if (d->N > lim || d->C > lim || d->F > lim || d->C * xvol > lim || d->F * gvol > lim || d->N * gvol > lim ||
      d->N * xvol > lim || d->F * d->C * wvol > lim)
    return fail(MG_ERR_UNSUPPORTED, "tensor too large for 32-bit in-sample offsets");
  g->nd = d->nd;
  g->dtype = d->dtype;
  g->N = (int)d->N;
  g->C = (int)d->C;
  g->F = (int)d->F;
  g->xvol = xvol;
  g->wvol = wvol;
  g->gvol = gvol;
  return MG_OK;
}

// Largest row tile whose round-up waste stays small.
int pick_bm(int M) {
  const int cands[4] = {128, 64, 32, 16};
  for (int c : cands) {
    const int padded = (int)ceil_div(M, c) * c;
    if (padded - M <= M / 8) return c;
  }
  return 16;
}

template <typename K>
int resident_blocks(K kernel, int threads) {
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, threads, 0) != hipSuccess || n < 1) {
    (void)hipGetLastError();
    n = 1;
  }
  return n;
}

// Tile shapes of the gather-GEMM kernels: rows x positions, and the wave tile.
#define MG_GEMM_SHAPES(T, X) \
  X(T, 128, 128, 64, 64)     \
  X(T, 128, 64, 64, 32)      \
  X(T, 64, 256, 64, 64)      \
  X(T, 64, 128, 32, 64)      \
  X(T, 32, 256, 32, 64)      \
  X(T, 32, 128, 16, 64)      \
  X(T, 16, 256, 16, 64)

// Tile shapes of the data gradient with 2 / 4 fused stride phases (float only): a wave keeps one
// set of accumulators per phase, so these are the shapes with at most 32 / 16 accumulator
// registers per set, which leaves room for two blocks on a compute unit.
#define MG_FUSED2_SHAPES(T, X) \
  X(T, 128, 64, 64, 32)        \
  X(T, 64, 128, 32, 64)        \
  X(T, 32, 256, 32, 64)        \
  X(T, 16, 256, 16, 64)
#define MG_FUSED4_SHAPES(T, X) \
  X(T, 64, 64, 32, 32)         \
  X(T, 32, 128, 16, 64)        \
  X(T, 16, 256, 16, 64)

// Blocks of the persistent tap-major gather-GEMM that a compute unit holds at once.
template <typename T>
int gemm_blocks_per_cu(int bm, int bn, int nph = 1, int bk = 0) {
  constexpr int BK = sizeof(T) == 8 ? 8 : 16;
#define MG_OCC(TT, BM, BN, WM, WN)                                                                                       \
  if (bm == BM && bn == BN)                                                                                              \
    return bk == 2 * BK ? resident_blocks(tap_gemm_kernel<TT, BM, BN, (sizeof(TT) == 8 ? 2 * BK : BK), WM, WN>, 512)     \
                        : resident_blocks(tap_gemm_kernel<TT, BM, BN, BK, WM, WN>, 512);
#define MG_OCC2(TT, BM, BN, WM, WN) \
  if (bm == BM && bn == BN) return resident_blocks(tap_gemm_kernel<TT, BM, BN, BK, WM, WN, 2>, 512);
#define MG_OCC4(TT, BM, BN, WM, WN)                                                                                       \
  if (bm == BM && bn == BN)                                                                                                \
    return bk == 2 * BK ? resident_blocks(tap_gemm_kernel<TT, BM, BN, (sizeof(TT) == 4 ? 2 * BK : BK), WM, WN, 4>, 512)     \
                        : resident_blocks(tap_gemm_kernel<TT, BM, BN, BK, WM, WN, 4>, 512);
  if constexpr (sizeof(T) == 4) {
    if (nph == 2) {
      MG_FUSED2_SHAPES(T, MG_OCC2)
      return 1;
    }
    if (nph == 4) {
      MG_FUSED4_SHAPES(T, MG_OCC4)
      return 1;
    }
  }
  MG_GEMM_SHAPES(T, MG_OCC)
#undef MG_OCC
#undef MG_OCC2
#undef MG_OCC4
  return 1;
}

// Picks the tile of the gather-GEMM, how many persistent blocks run per compute unit
// and how the last, partial round of tiles is shared out.  With r blocks per unit the
// grid has r x CUs blocks; block b takes tiles b, b + grid, ...  A unit's MFMA pipes are
// shared by its blocks, so one round of the grid costs r tile times.  After
// floor(T / grid) whole rounds, T % grid tiles are left that would keep only some
// units busy; each of those is cut into `split` K slices so that every unit gets
// about the same share of them (the busiest gets ceil(rem x split / CUs) slices).
// Smaller tiles give more tiles (finer balance, less padding) at some cost in operand
// reuse.  Kernels that do not stream run one block per tile (r = 1 in this arithmetic:
// the hardware refills a unit as soon as a block leaves).
// Fewest K tiles in a block's share of the leftover tiles (see build_shares).
constexpr long long kMinRun = 8;

struct TileChoice {
  int bm, bn, m_tiles, full_tiles, tail_split;
  int blocks_per_cu;  // persistent blocks per compute unit (streaming kernels)
  long long tiles;
};

TileChoice choose_tile(int M, const std::vector<long long> &phase_npos, int min_ktiles, bool tap_major, size_t elem, int nph = 1, int bk = 0,
                       int avg_ktiles = -1) {
  if (avg_ktiles < 0) avg_ktiles = min_ktiles;  // K tiles of an average tile (phases of a data gradient differ)
  struct Cfg {
    int bm, bn;
    double penalty;  // relative cost of a flop in this tile shape
    bool tap_only;
  };
  static const Cfg plain[] = {{128, 128, 1.00, false}, {128, 64, 1.05, true}, {64, 256, 1.00, false}, {64, 128, 1.08, true},
                              {32, 256, 1.00, false},  {32, 128, 1.10, true}, {16, 256, 1.00, false}};
  static const Cfg fused2[] = {{128, 64, 1.05, true}, {64, 128, 1.08, true}, {32, 256, 1.00, true}, {16, 256, 1.00, true}};
  static const Cfg fused4[] = {{64, 64, 1.10, true}, {32, 128, 1.10, true}, {16, 256, 1.00, true}};
  const Cfg *cfgs = nph == 4 ? fused4 : nph == 2 ? fused2 : plain;
  const int ncfgs = nph == 4 ? 3 : nph == 2 ? 4 : 7;
  // MYGRAD_HIP_TILE="rows,positions[,blocks per unit]" (diagnostics and the tests of every tile shape;
  // read whenever a plan is built, and part of the plan's key): only that tile shape, where it exists
  struct Forced {
    int bm = 0, bn = 0, r = 0;
  };
  const Forced forced = [] {
    Forced f;
    if (const char *v = getenv("MYGRAD_HIP_TILE")) sscanf(v, "%d,%d,%d", &f.bm, &f.bn, &f.r);
    return f;
  }();
  // MYGRAD_HIP_SHARES=0: the last round's tiles are cut into equal K slices instead (the older scheme)
  static const bool shares_on = [] {
    const char *flag = getenv("MYGRAD_HIP_SHARES");
    return !(flag && flag[0] == '0');
  }();
  bool forced_fits = false;
  for (int ci = 0; ci < ncfgs; ++ci)
    forced_fits |= cfgs[ci].bm == forced.bm && cfgs[ci].bn == forced.bn && (!cfgs[ci].tap_only || tap_major) &&
                   !(tap_major && elem == 8 && cfgs[ci].bn * cfgs[ci].bm >= 128 * 128);  // (no such double-precision tile)
  const int bm = forced_fits ? forced.bm : nph == 4 ? std::min(pick_bm(M), 64) : pick_bm(M);
  const int cus = runtime().props.multiProcessorCount;
  TileChoice best{};
  double best_cost = 0;
  for (int ci = 0; ci < ncfgs; ++ci) {
    const Cfg &c = cfgs[ci];
    if (c.bm != bm || (c.tap_only && !tap_major) || (forced_fits && c.bn != forced.bn)) continue;
    // 64x64 fp64 wave tiles hold 128 accumulator registers: only one 8-wave block
    // fits on a compute unit, so the tap-major kernels use the half-size shapes
    if (tap_major && elem == 8 && c.bn * c.bm >= 128 * 128) continue;
    const bool stream = tap_major && tap_gemm_streams(c.bm, (int)elem);
    const int per_cu = !stream ? 1 : elem == 8 ? gemm_blocks_per_cu<double>(c.bm, c.bn, 1, bk) : gemm_blocks_per_cu<float>(c.bm, c.bn, nph, bk);
    long long pos_blocks = 0;
    for (long long n : phase_npos) pos_blocks += ceil_div(n, c.bn);
    // (most blocks first: where the rounds come out the same, more resident blocks cover more of one
    // another's waits -- 128 x 64 tiles, C = F = 128 at 28 x 28: 244 us with two per unit, 236 us with three)
    for (int r = per_cu; r >= 1; --r) {
      if (forced_fits && forced.r > 0 && r != std::min(forced.r, per_cu)) continue;
      TileChoice t{};
      t.bm = c.bm;
      t.bn = c.bn;
      t.blocks_per_cu = r;
      t.m_tiles = (int)ceil_div(M, c.bm);
      t.tiles = pos_blocks * t.m_tiles;
      t.full_tiles = (int)t.tiles;
      t.tail_split = 1;
      const long long grid = (long long)r * cus;
      const long long rem = t.tiles % grid;
      // a streaming block alone on its unit leaves the MFMA pipes idle while it waits
      // at its barriers; two or more cover for one another
      const double alone = stream && r == 1 ? 1.4 : 1.0;
      if (stream && shares_on && t.tiles < 2 * (long long)cus) {
        // Fewer than two tiles per unit (few positions under many channels: the late stages of a
        // network).  Equal K slices of the leftover tiles then leave a large part of the device idle
        // in the last round however they are cut (196 tiles of 288 K tiles on 256 units: 0.85 tile
        // times at best where 0.77 are due, and measured 1.0), and with more tiles per unit the
        // slices below lose 1 - 3 % less to their partial sums than the shares do.
        // Persistent blocks take even shares of what the whole tiles leave over (build_shares).
        // Blocks b, b + CUs, ... share a unit, so a unit gets the tiles t = b (mod CUs): q = T / CUs
        // whole tiles, worked off by its r blocks, and the T mod CUs tiles beyond that are shared
        // out as K tiles: every unit gets (T mod CUs) / CUs tile times of them, whatever the
        // remainder.  What it costs is the partial sums of the tiles that are cut: about one slice
        // per run and one more per tile that is cut, written and read once (priced in tile times:
        // a tile's flops at three quarters of the unit's peak against its bytes at 4 TB/s for the
        // whole device, plus the fix-up launch).
        const long long q = t.tiles / cus, left = t.tiles % cus;
        // (within a unit the r blocks take q / r whole tiles each; if r does not divide q the last
        // q mod r tiles run with fewer blocks than r, a single one without cover for its barriers)
        const int over = (int)(q % r);
        double units = (double)(q / r) * r + (over == 1 && r > 1 ? 1.4 : (double)over) + (double)left / cus;
        if (left > 0) {
          t.full_tiles = (int)(q * cus);
          t.tail_split = 0;  // marks the plan for build_shares
          const double depth = (double)std::max(avg_ktiles, 1) * (bk > 0 ? bk : (elem == 8 ? 8 : 16));
          const double tile_seconds = 2.0 * c.bm * c.bn * depth / (0.75 * (elem == 8 ? 78.6e12 : 157.3e12) / cus);
          const long long runs = std::max<long long>(1, std::min<long long>(grid, left * (long long)std::max(avg_ktiles, 1) / kMinRun));
          const double slices = (double)(runs - 1) + (double)std::min<long long>(left, runs - 1);
          const double fix_seconds = slices * c.bm * c.bn * (double)elem * nph * 2.0 / 4.0e12 + 4e-6;
          units += fix_seconds / tile_seconds;
        }
        const double cost = units * alone * c.bm * c.bn * c.penalty;
        if (best.bm == 0 || cost < best_cost) {
          best = t;
          best_cost = cost;
        }
        continue;
      }
      double tail = 0;  // tile times the busiest unit spends on the remaining tiles
      if (rem > 0) {
        tail = (double)ceil_div(rem, cus);
        if (tap_major) {
          // slices of at least two K tiles, at most 32 MB of partial sums
          const long long tile_bytes = (long long)c.bm * c.bn * (long long)elem * nph;
          const int smax = (int)std::max<long long>(1, std::min<long long>({(long long)min_ktiles / 2, 32ll, (32ll << 20) / (rem * tile_bytes)}));
          for (int sp = 2; sp <= smax; ++sp) {
            const double share = (double)ceil_div(rem * sp, cus) / sp + 0.01 * sp;  // + a little for the fix-up pass
            if (share < tail - 1e-9) {
              tail = share;
              t.tail_split = sp;
            }
          }
          if (t.tail_split > 1) t.full_tiles = (int)(t.tiles - rem);
        }
      }
      const double cost = ((double)(t.tiles / grid) * r + tail) * alone * c.bm * c.bn * c.penalty;
      if (best.bm == 0 || cost < best_cost) {
        best = t;
        best_cost = cost;
      }
      // The same grid with the tail counted per unit instead of per round of the grid: blocks
      // b, b + CUs, ... share a unit, so a unit gets the tiles t = b (mod CUs): q = T / CUs whole
      // tiles each, and only the T mod CUs tiles beyond that are cut into slices (at most one
      // slice per unit: little partial-sum traffic).  Within a unit the r blocks take q / r tiles
      // each; if r does not divide q the last q mod r tiles run with fewer blocks than r.
      if (stream && r > 1 && rem > 0) {
        TileChoice u = t;
        const long long q = u.tiles / cus, left = u.tiles % cus;
        const int over = (int)(q % r);
        double time = (double)(q / r) * r + (over == 1 ? 1.4 : (double)over);
        u.full_tiles = (int)u.tiles;
        u.tail_split = 1;
        if (left > 0) {
          double share = 1.0;
          const long long tile_bytes = (long long)c.bm * c.bn * (long long)elem * nph;
          const int smax = (int)std::max<long long>(1, std::min<long long>({(long long)min_ktiles / 2, 32ll, (32ll << 20) / (left * tile_bytes)}));
          for (int sp = 2; sp <= smax; ++sp) {
            const double sh = (double)ceil_div(left * sp, cus) / sp + 0.01 * sp;
            if (sh < share - 1e-9) share = sh, u.tail_split = sp;
          }
          if (u.tail_split > 1) u.full_tiles = (int)(q * cus);
          time += share;
        }
        const double ucost = time * c.bm * c.bn * c.penalty;
        if (q > 0 && ucost < best_cost) {
          best = u;
          best_cost = ucost;
        }
      }
    }
  }
  return best;
}

void set_divisors(Phase &ph) {
  ph.by_jvol = make_fastdiv((unsigned)(ph.J[0] * ph.J[1] * ph.J[2]));
  ph.by_j12 = make_fastdiv((unsigned)(ph.J[1] * ph.J[2]));
  ph.by_j2 = make_fastdiv((unsigned)ph.J[2]);
}

struct Tables {
  std::vector<TabEntry> tab;
  std::vector<int> arow;
  std::vector<Phase> phases;
  std::vector<KTile> ktiles;
  std::vector<WGroup> groups;
  std::vector<int> share_first;
  std::vector<ShareSlice> share_slices;
  std::vector<ShareFix> share_fix;
};

// Even shares of what the whole tiles leave over: the K tiles of the tiles from pl.full_tiles on,
// laid end to end, are cut into runs of equal length (to within one K tile; at least kMinRun K
// tiles each, so at most one run per block), one run per block from the last block down (with
// full_tiles no multiple of the grid those have one whole tile fewer); a run is cut where it
// crosses from one tile into the next.  A tile that lies in one run is computed whole and stored
// directly; the slices of any other leave partial sums in consecutive slots, in K order, which
// the fix-up pass adds in that order.  Tiles without K tiles (a stride phase that no tap reaches)
// are all zeros: dealt out one by one, stored directly.
void build_shares(Plan &pl, Tables &t, int grid) {
  const long long tiles = (long long)pl.pos_blocks * pl.m_tiles;
  std::vector<int> kcount;  // K tiles of each tail tile
  long long total = 0;
  size_t pi = 0;
  for (long long tile = pl.full_tiles; tile < tiles; ++tile) {
    const int pblk = (int)(tile / pl.m_tiles);
    while (pi + 1 < t.phases.size() && pblk >= t.phases[pi + 1].blk_begin) ++pi;
    kcount.push_back(t.phases[pi].k_count);
    total += t.phases[pi].k_count;
  }
  const long long runs = std::max<long long>(1, std::min<long long>(grid, total / kMinRun));
  std::vector<std::vector<ShareSlice>> mine((size_t)grid);
  std::vector<int> slices_of(kcount.size(), 0);
  size_t cur = 0;      // tail tile the next run starts in
  long long done = 0;  // K tiles of that tile that earlier runs took
  for (long long j = 0; j < runs; ++j) {
    std::vector<ShareSlice> &list = mine[(size_t)(grid - 1 - j)];
    long long want = total * (j + 1) / runs - total * j / runs;
    while (want > 0 && cur < kcount.size()) {
      if (kcount[cur] == 0) {
        ++cur;
        continue;
      }
      const long long take = std::min<long long>(want, kcount[cur] - done);
      list.push_back(ShareSlice{(int)(pl.full_tiles + cur), (int)done, (int)(done + take), 0});
      ++slices_of[cur];
      done += take;
      want -= take;
      if (done == kcount[cur]) ++cur, done = 0;
    }
  }
  int dealt = 0;
  for (size_t i = 0; i < kcount.size(); ++i)
    if (kcount[i] == 0) {
      mine[(size_t)(grid - 1 - dealt % grid)].push_back(ShareSlice{(int)(pl.full_tiles + i), 0, 0, 0});
      slices_of[i] = 1;
      ++dealt;
    }
  // slots: a tile's slices lie in consecutive runs, i.e. in descending blocks; numbered in K order
  std::vector<int> first_slot(kcount.size(), -1);
  int slots = 0;
  for (size_t i = 0; i < kcount.size(); ++i)
    if (slices_of[i] > 1) {
      first_slot[i] = slots;
      t.share_fix.push_back(ShareFix{(int)(pl.full_tiles + i), slots, slices_of[i], 0});
      slots += slices_of[i];
    }
  std::vector<int> used(kcount.size(), 0);
  for (long long b = grid - 1; b >= 0; --b)
    for (ShareSlice &sl : mine[(size_t)b]) {
      const size_t i = (size_t)(sl.tile - pl.full_tiles);
      sl.slot = first_slot[i] < 0 ? -1 : first_slot[i] + used[i]++;
    }
  t.share_first.assign(grid + 1, 0);
  for (int b = 0; b < grid; ++b) {
    t.share_first[b] = (int)t.share_slices.size();
    // a block's cursor over the phase table only moves forward: its tiles in ascending order
    std::stable_sort(mine[(size_t)b].begin(), mine[(size_t)b].end(), [](const ShareSlice &x, const ShareSlice &y) { return x.tile < y.tile; });
    for (const ShareSlice &sl : mine[(size_t)b]) t.share_slices.push_back(sl);
  }
  t.share_first[grid] = (int)t.share_slices.size();
  pl.share_grid = grid;
  pl.share_slots = slots;
  pl.share_fixes = (int)t.share_fix.size();
}

template <typename V>
size_t padded_bytes(const V &v) {
  return (v.size() * sizeof(typename V::value_type) + 255) & ~size_t(255);
}

int upload_plan(Plan &pl, Tables &t) {
  if (pl.tap_major && pl.tail_split == 0) {
    const long long tiles = (long long)pl.pos_blocks * pl.m_tiles;
    if (tiles > pl.full_tiles) build_shares(pl, t, pl.blocks_per_cu * runtime().props.multiProcessorCount);
  }
  if (pl.tail_split == 0 && pl.share_grid == 0) pl.tail_split = 1;
  const size_t zero_b = 256;
  const size_t off_tab = zero_b;
  const size_t off_arow = off_tab + padded_bytes(t.tab);
  const size_t off_ph = off_arow + padded_bytes(t.arow);
  const size_t off_kt = off_ph + padded_bytes(t.phases);
  const size_t off_gr = off_kt + padded_bytes(t.ktiles);
  const size_t off_sf = off_gr + padded_bytes(t.groups);
  const size_t off_ss = off_sf + padded_bytes(t.share_first);
  const size_t off_sx = off_ss + padded_bytes(t.share_slices);
  const size_t total = off_sx + padded_bytes(t.share_fix) + 256;
  std::vector<char> host(total, 0);
  auto put = [&](size_t off, const void *src, size_t n) {
    if (n) memcpy(host.data() + off, src, n);
  };
  put(off_tab, t.tab.data(), t.tab.size() * sizeof(TabEntry));
  put(off_arow, t.arow.data(), t.arow.size() * sizeof(int));
  put(off_ph, t.phases.data(), t.phases.size() * sizeof(Phase));
  put(off_kt, t.ktiles.data(), t.ktiles.size() * sizeof(KTile));
  put(off_gr, t.groups.data(), t.groups.size() * sizeof(WGroup));
  put(off_sf, t.share_first.data(), t.share_first.size() * sizeof(int));
  put(off_ss, t.share_slices.data(), t.share_slices.size() * sizeof(ShareSlice));
  put(off_sx, t.share_fix.data(), t.share_fix.size() * sizeof(ShareFix));
  MG_HIP(hipMalloc(&pl.blob, host.size()));
  hipError_t err = hipMemcpy(pl.blob, host.data(), host.size(), hipMemcpyHostToDevice);
  if (err != hipSuccess) {
    (void)hipFree(pl.blob);
    pl.blob = nullptr;
    return hip_fail(err, "hipMemcpy(plan tables)", __FILE__, __LINE__);
  }
  char *base = static_cast<char *>(pl.blob);
  pl.zeros = base;  // the first 256 bytes stay zero: target of padding loads
  pl.tab = reinterpret_cast<TabEntry *>(base + off_tab);
  pl.arow = reinterpret_cast<int *>(base + off_arow);
  pl.phases = reinterpret_cast<Phase *>(base + off_ph);
  pl.ktiles = reinterpret_cast<KTile *>(base + off_kt);
  pl.groups = reinterpret_cast<WGroup *>(base + off_gr);
  if (pl.share_grid > 0) {
    pl.share_first = reinterpret_cast<int *>(base + off_sf);
    pl.share_slices = reinterpret_cast<ShareSlice *>(base + off_ss);
    pl.share_fix = reinterpret_cast<ShareFix *>(base + off_sx);
  }
  pl.nphases = (int)t.phases.size();
  return MG_OK;
}

// rows (c, t0, t1, t2) in the filter's own row-major order
void fwd_table(const Geometry &g, std::vector<TabEntry> &tab) {
  const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
  tab.clear();
  tab.reserve((size_t)g.C * g.wvol);
  for (int c = 0; c < g.C; ++c)
    for (int t0 = 0; t0 < g.W[0]; ++t0)
      for (int t1 = 0; t1 < g.W[1]; ++t1)
        for (int t2 = 0; t2 < g.W[2]; ++t2) {
          TabEntry e;
          e.d0 = t0 * g.D[0] - g.P[0];
          e.d1 = t1 * g.D[1] - g.P[1];
          e.d2 = t2 * g.D[2] - g.P[2];
          e.off = (int)(c * g.xvol) + e.d0 * qs[0] + e.d1 * qs[1] + e.d2 * qs[2];
          tab.push_back(e);
        }
}

// Whether the three taps of the last axis can be rows of the GEMM (see GemmParams::fold_row)
// for a problem with `rows` rows (filters in the forward pass, channels in the data gradient):
// float, few rows (with 16 or 32 the plain tiles are bound by the gather, not by the matrix
// pipes: a gathered element feeds three times the MFMAs this way), a 3-tap "same" last axis
// with unit stride and dilation, and rows of positions that a wave's 64 positions hold whole
// (up to 64 long, padded to a power of two).  MYGRAD_HIP_FOLD=0 switches it off.
// `depth`: the channels contracted per tap (channels in the forward pass, filters in the data
// gradient).  With 17 to 32 rows the plain 32-row tiles are less starved, and measured against
// them the 96-row folded tile wins with 16 and 32 channels per tap (3 - 8 %) and loses with 256
// (10 %): taken up to 64.
int fold_padded_row(int row) {
  int padded = 4;
  while (padded < row) padded *= 2;
  return padded;
}

bool fold_applies(const Geometry &g, int rows, int depth) {
  static const bool fold_on = [] {
    const char *flag = getenv("MYGRAD_HIP_FOLD");
    return !(flag && flag[0] == '0');
  }();
  // a row of positions is padded to a power of two (a wave's 64 positions are whole padded rows);
  // the padding positions cost MFMA time and store nothing: at most an eighth of a row
  const int padded = fold_padded_row(g.X[2]);
  const bool row_fits = g.X[2] >= 4 && g.X[2] <= 64 && (padded - g.X[2]) * 8 <= padded &&
                        (long long)g.N * g.X[0] * g.X[1] * padded < (1ll << 31);
  return fold_on && (rows <= 16 || (rows <= 32 && depth <= 64)) && g.W[2] == 3 && g.P[2] == 1 &&
         g.D[2] == 1 && g.S[2] == 1 && g.G[2] == g.X[2] && row_fits;
}

// The positions of a folded plan: rows of the last axis padded to `fold_row` positions each.
void pad_fold_rows(const Geometry &g, Plan &pl, Phase &ph) {
  pl.fold_row = fold_padded_row(g.X[2]);
  ph.J[2] = pl.fold_row;
  ph.npos = (int)((long long)g.N * ph.J[0] * ph.J[1] * ph.J[2]);
  set_divisors(ph);
}

// Tile of a plan with folded taps: 48 rows x 256 positions for up to 16 channels (one block per
// tile), 96 x 128 for up to 32 (persistent blocks, as many as fit on the device, every tile whole).
void set_fold_tile(const Geometry &g, Plan &pl, int rows, int bk) {
  pl.m_tiles = 1, pl.tail_split = 1, pl.blocks_per_cu = 1;
  if (rows <= 16) {
    pl.bm = 48, pl.bn = 256;
  } else {
    pl.bm = 96, pl.bn = 128;
  }
  // persistent blocks (all double-precision tiles, and float tiles of 64 rows or more): as many
  // as the device holds
  if (g.dtype == MG_F64) {
    if (rows <= 16)
      pl.blocks_per_cu = bk == 16 ? resident_blocks(tap_gemm_kernel<double, 48, 256, 16, 48, 64, 1, true>, 512)
                                  : resident_blocks(tap_gemm_kernel<double, 48, 256, 8, 48, 64, 1, true>, 512);
    else
      pl.blocks_per_cu = bk == 16 ? resident_blocks(tap_gemm_kernel<double, 96, 128, 16, 48, 64, 1, true>, 512)
                                  : resident_blocks(tap_gemm_kernel<double, 96, 128, 8, 48, 64, 1, true>, 512);
  } else if (rows > 16) {
    pl.blocks_per_cu = resident_blocks(tap_gemm_kernel<float, 96, 128, 16, 48, 64, 1, true>, 512);
  }
}

// A problem of a few microseconds is bound by its launches and by the chain of K tiles a
// block runs through, each a round trip to memory, not by the matrix pipes.
// MYGRAD_HIP_TINY=0 plans such a problem like a large one (read whenever a plan is built, and
// part of the plan's key: the parity tests run their small cases both ways).
// MYGRAD_HIP_PHASE_ROWS=0 plans the data gradient of a few channels under a stride phase by phase
// (read whenever a plan is built, and part of the plan's key: the parity tests run both ways).
bool phase_rows_enabled() {
  const char *flag = getenv("MYGRAD_HIP_PHASE_ROWS");
  return !(flag && flag[0] == '0');
}

bool tiny_plans_enabled() {
  const char *flag = getenv("MYGRAD_HIP_TINY");
  return !(flag && flag[0] == '0');
}

bool is_tiny(const Geometry &g) {
  return tiny_plans_enabled() &&
         2.0 * (double)g.N * (double)g.gvol * (double)g.F * (double)g.C * (double)g.wvol < 1e8;
}

// Whether a tiny problem with `rows` rows and a contraction of `depth` (channels x taps, or
// filters x taps) is better off on the table-driven kernel -- one launch, no packing: when a
// block's chain of K tiles there is at most five long (its K tile is 64 / 32 deep for up to 16
// rows, 16 / 8 beyond; float / double).  Measured on MNIST-sized layers: a contraction of 25 or
// 144 is faster there, one of 250 or 500 is 1.3 - 2.4 x slower than the tap-major kernel on
// table rows.
bool tiny_table(const Geometry &g, int rows, long long depth) {
  const int k_tile = (rows <= 16 ? 4 : 1) * gemm_bk(g.dtype);
  return is_tiny(g) && depth <= 5 * k_tile;
}

// The table-driven kernel for such a problem: more, smaller tiles and a quarter of the K steps.
void deepen_if_tiny(const Geometry &g, Plan &pl) {
  if (pl.tap_major || !is_tiny(g) || pl.bm != 16) return;
  pl.bn = 64;
  pl.deep_k = true;
}

bool table_rows_on() {
  static const bool on = [] {
    const char *flag = getenv("MYGRAD_HIP_TABLE_ROWS");
    return !(flag && flag[0] == '0');
  }();
  return on;
}


// ---- few rows (channels of a data gradient, filters of a forward pass), single precision,
// enough positions to fill the device: the 4x4x1 MFMA kernel, one position per lane.
// MYGRAD_HIP_THIN=0 switches it off (read whenever a plan is built, and part of the plan's key).
bool thin_on() {
  const char *flag = getenv("MYGRAD_HIP_THIN");
  return !(flag && flag[0] == '0');
}

// Groups of four rows the kernel would run `rows` as (a power of two; more than 64 rows without
// stride phases: sixteen per pass), 0 if it has no such shape.
int thin_row_groups(int rows, int nph) {
  int rg = 1;
  while (rg * 4 < rows && rg < 16) rg *= 2;
  if (rg * 4 < rows && nph != 1) return 0;
  return (nph == 1 || nph == 2 || nph == 4) && thin_gemm_has(nph, rg) ? rg : 0;
}

// Positions: one wave per SIMD (65536) where a gathered element feeds several MFMAs (stride
// phases, row groups) -- the 16-row tiles take two to three times as long there; four waves per
// SIMD where it feeds a single one and the kernel is bound by its loads (at one wave per SIMD
// it loses a quarter, at sixteen it is ahead by one).
bool thin_applies(const Geometry &g, int rows, long long positions, long long depth, long long nph) {
  const int rg = thin_row_groups(rows, (int)nph);
  // (the packed filters take up to 128 bytes per element of the contraction and are addressed
  // with 32-bit offsets like everything else)
  return thin_on() && g.dtype == MG_F32 && rg != 0 && fits_buffer_loads(g) && positions >= (nph * rg == 1 ? 4 : 1) * 65536 &&
         depth < (1 << 23) && !tiny_table(g, rows, depth);
}

// One gathered element of a thin plan: its coordinate offsets and, per phase, the filter tap it
// meets there (-1: none).
struct ThinUse {
  int d[3];
  int tap[4];
};

// Lays the entries out in chunks of 16 / nph.  `groups` consecutive source channels may be taken
// together (their count must divide the channel count) so that fewer slots of a register of
// packed filters stay empty.  The kernel's time goes with its loads (one per entry and step,
// plus the register of filters), and a chunk's set-up before its loop over the channel groups
// costs about two thirds of a load per entry (measured: 25 taps, 32 filters take the same time
// as 25 chunks x 2 steps and as 2 padded chunks x 32 steps); the cheapest grouping is taken.
void thin_tables(Plan &pl, Tables &t, const std::vector<ThinUse> &uses, int nph, int rows, int channels, long long src_cstride,
                 const int qs[3], long long w_kstride, long long w_mstride) {
  const int rg = thin_row_groups(rows, nph);
  const int epv = 16 / (nph * rg);
  const int ne = (int)uses.size();
  int groups = 1;
  long long best = -1;
  for (int cand : {1, 2, 4, 8, 16}) {
    if (channels % cand != 0) continue;
    const long long chunks = ceil_div((long long)cand * ne, epv);
    const long long cost = chunks * (13 * epv + 20ll * (channels / cand) * (epv + 1));
    if (best < 0 || cost < best) best = cost, groups = cand;
  }
  // a slot of the packed filters is (entry within its chunk, phase, row group): the offset of the
  // group's first row in the filter bank, -1 where the phase has no tap for the entry or the group
  // lies beyond the rows
  auto push_slots = [&](const ThinUse *u, int ksub) {
    for (int f = 0; f < nph; ++f)
      for (int r = 0; r < rg; ++r)
        t.arow.push_back(u == nullptr || u->tap[f] < 0 || 4 * r >= rows ? -1 : (int)(ksub * w_kstride + u->tap[f] + 4 * r * w_mstride));
  };
  for (int ksub = 0; ksub < groups; ++ksub)
    for (const ThinUse &u : uses) {
      TabEntry e;
      e.d0 = u.d[0], e.d1 = u.d[1], e.d2 = u.d[2];
      e.off = (int)(ksub * src_cstride) + u.d[0] * qs[0] + u.d[1] * qs[1] + u.d[2] * qs[2];
      t.tab.push_back(e);
      push_slots(&u, ksub);
    }
  TabEntry outside{};
  outside.d0 = outside.d1 = outside.d2 = 1 << 29;
  while (t.tab.size() % epv != 0) {
    t.tab.push_back(outside);
    push_slots(nullptr, 0);
  }
  pl.thin = true;
  pl.nph = nph;
  pl.thin_rg = rg;
  pl.thin_chunks = (int)t.tab.size() / epv;
  pl.thin_kgroups = channels / groups;
  pl.thin_src_group = groups * src_cstride;
  pl.thin_w_group = groups * w_kstride;
  pl.thin_w_mstride = (int)w_mstride;
}

int build_fwd_plan(const Geometry &g, Plan &pl) {
  Tables t;
  if ((g.F <= 4 || (g.F <= 1024 && g.C % gemm_bk(g.dtype) != 0)) && thin_applies(g, g.F, (long long)g.N * g.gvol, (long long)g.C * g.wvol, 1)) {
    // up to four filters, or a first layer (channels that fill no K tile; passes of 64 filters), in
    // single precision: one output position per lane
    const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
    std::vector<ThinUse> uses;
    for (int t0 = 0; t0 < g.W[0]; ++t0)
      for (int t1 = 0; t1 < g.W[1]; ++t1)
        for (int t2 = 0; t2 < g.W[2]; ++t2)
          uses.push_back(ThinUse{{t0 * g.D[0] - g.P[0], t1 * g.D[1] - g.P[1], t2 * g.D[2] - g.P[2]}, {(t0 * g.W[1] + t1) * g.W[2] + t2, -1, -1, -1}});
    thin_tables(pl, t, uses, 1, g.F, g.C, g.xvol, qs, g.wvol, (long long)g.C * g.wvol);
    Phase grid{};
    for (int k = 0; k < 3; ++k) {
      grid.J[k] = g.G[k];
      pl.po0[0][k] = 0;
      pl.pJ[0][k] = g.G[k];
    }
    grid.npos = (int)((long long)g.N * g.gvol);
    set_divisors(grid);
    pl.thin_grid = grid;
    pl.pos_blocks = (int)ceil_div(grid.npos, 256);
    pl.bm = 4, pl.bn = 256;
    return upload_plan(pl, t);
  }
  pl.tap_major = g.C % gemm_bk(g.dtype) == 0 && fits_buffer_loads(g);
  // Channels that do not fill K tiles (a first layer's one or three): the same kernel, its K
  // tiles 16 rows of the gather table each -- unless the problem is tiny (few launches matter
  // more) or MYGRAD_HIP_TABLE_ROWS=0 asks for the plain table-driven kernel.
  static const bool rows_on = [] {
    const char *flag = getenv("MYGRAD_HIP_TABLE_ROWS");
    return !(flag && flag[0] == '0');
  }();
  pl.table_rows = rows_on && !pl.tap_major && fits_buffer_loads(g) && !tiny_table(g, g.F, (long long)g.C * g.wvol);
  if (pl.table_rows) pl.tap_major = true;
  const int bk = pl.table_rows ? 16 : pl.tap_major ? tap_bk(g.dtype, g.C) : gemm_bk(g.dtype);
  pl.bk = bk;
  pl.single_dense_phase = true;
  {
    const long long ktiles = pl.table_rows ? ceil_div((long long)g.C * g.wvol, bk)
                             : pl.tap_major ? g.wvol * (g.C / bk) : ceil_div((long long)g.C * g.wvol, bk);
    const TileChoice tc = choose_tile(g.F, {(long long)g.N * g.gvol}, (int)ktiles, pl.tap_major, g.dtype == MG_F64 ? 8 : 4, 1, bk);
    pl.bm = tc.bm, pl.bn = tc.bn, pl.m_tiles = tc.m_tiles, pl.full_tiles = tc.full_tiles, pl.tail_split = tc.tail_split, pl.blocks_per_cu = tc.blocks_per_cu;
    deepen_if_tiny(g, pl);
  }
  Phase ph{};
  for (int k = 0; k < 3; ++k) {
    ph.J[k] = g.G[k];
    ph.o0[k] = 0;
  }
  ph.k_begin = 0;
  ph.blk_begin = 0;
  ph.npos = (int)((long long)g.N * g.gvol);
  set_divisors(ph);
  if (pl.table_rows) {
    // the table in the filter's own row order (c, taps), padded to whole K tiles with rows that
    // lie outside every input (and meet rows of A beyond its end: zeros)
    fwd_table(g, t.tab);
    const int rows = (int)t.tab.size();
    for (int k0 = 0; k0 < rows; k0 += bk) {
      KTile e{};
      e.a_row0 = k0;
      e.coff = k0;  // first table row of the tile
      t.ktiles.push_back(e);
    }
    TabEntry outside{};
    outside.d0 = outside.d1 = outside.d2 = 1 << 29;
    while (t.tab.size() % bk != 0) t.tab.push_back(outside);
    ph.k_count = (int)t.ktiles.size();
    t.phases.push_back(ph);
    pl.pos_blocks = (int)ceil_div(ph.npos, pl.bn);
    return upload_plan(pl, t);
  }
  if (pl.tap_major && fold_applies(g, g.F, g.C)) {
    // rows (filter, tap of the last axis); K tiles over the taps of the other axes
    const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
    for (int c0 = 0; c0 < g.C; c0 += bk)
      for (int t0 = 0; t0 < g.W[0]; ++t0)
        for (int t1 = 0; t1 < g.W[1]; ++t1) {
          KTile e{};
          e.d0 = t0 * g.D[0] - g.P[0];
          e.d1 = t1 * g.D[1] - g.P[1];
          e.d2 = 0;
          e.a_row0 = (t0 * g.W[1] + t1) * g.C + c0;
          e.coff = (int)(c0 * g.xvol) + e.d0 * qs[0] + e.d1 * qs[1];
          t.ktiles.push_back(e);
        }
    ph.k_count = (int)t.ktiles.size();
    pad_fold_rows(g, pl, ph);
    set_fold_tile(g, pl, g.F, bk);
    pl.pos_blocks = (int)ceil_div(ph.npos, pl.bn);
    pl.full_tiles = pl.pos_blocks;
    t.phases.push_back(ph);
    return upload_plan(pl, t);
  }
  if (pl.tap_major) {
    // K tiles run channel block by channel block, all taps of a block back to back:
    // the taps of one channel block re-read the same few rows of x, which then come
    // from L1/L2 instead of crossing HBM once per tap.
    const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
    for (int c0 = 0; c0 < g.C; c0 += bk)
      for (int t0 = 0; t0 < g.W[0]; ++t0)
        for (int t1 = 0; t1 < g.W[1]; ++t1)
          for (int t2 = 0; t2 < g.W[2]; ++t2) {
            const int tflat = (t0 * g.W[1] + t1) * g.W[2] + t2;
            KTile e{};
            e.d0 = t0 * g.D[0] - g.P[0];
            e.d1 = t1 * g.D[1] - g.P[1];
            e.d2 = t2 * g.D[2] - g.P[2];
            e.a_row0 = tflat * g.C + c0;
            e.coff = (int)(c0 * g.xvol) + e.d0 * qs[0] + e.d1 * qs[1] + e.d2 * qs[2];
            t.ktiles.push_back(e);
          }
    ph.k_count = (int)t.ktiles.size();
  } else {
    fwd_table(g, t.tab);
    t.arow.resize(t.tab.size());
    for (size_t i = 0; i < t.arow.size(); ++i) t.arow[i] = (int)i;
    ph.k_count = (int)t.tab.size();
  }
  t.phases.push_back(ph);
  pl.pos_blocks = (int)ceil_div(ph.npos, pl.bn);
  return upload_plan(pl, t);
}

bool deep_fused_on() {
  static const bool on = [] {
    const char *flag = getenv("MYGRAD_HIP_FUSE_BK32");
    return !(flag && flag[0] == '0');
  }();
  return on;
}

int build_dgrad_plan(const Geometry &g, Plan &pl) {
  Tables t;
  // a tiny problem with a handful of channels is bound by its launches: the table-driven kernel
  // with its deep K tiles needs neither packed filters nor a pass over partial sums.  (Measured,
  // whole steps: 3 channels 38.5 -> 28 us; with 16 channels the tap-major kernels are 4 us
  // ahead, and with 32 or 64 the table-driven kernel's few, long-running blocks cost 2 - 5 x.)
  pl.tap_major = g.F % gemm_bk(g.dtype) == 0 && fits_buffer_loads(g) && !(tiny_table(g, g.C, (long long)g.F * g.wvol) && g.C <= 8);
  // filter counts that fill no K tile (10, 20, ...): the tap-major kernel on rows of the gather
  // table, as in the forward pass (MYGRAD_HIP_TABLE_ROWS=0: the plain table-driven kernel)
  pl.table_rows = table_rows_on() && g.F % gemm_bk(g.dtype) != 0 && fits_buffer_loads(g) && !tiny_table(g, g.C, (long long)g.F * g.wvol);
  if (pl.table_rows) pl.tap_major = true;
  const int bk = pl.table_rows ? 16 : pl.tap_major ? tap_bk(g.dtype, g.F) : gemm_bk(g.dtype);
  pl.bk = bk;
  pl.single_dense_phase = g.S[0] == 1 && g.S[1] == 1 && g.S[2] == 1;
  const int gs[3] = {g.G[1] * g.G[2], g.G[2], 1};
  long long nphase = (long long)g.S[0] * g.S[1] * g.S[2];
  if (nphase > 4096) return fail(MG_ERR_UNSUPPORTED, "prod(stride) = %lld phases (limit 4096)", nphase);

  // ---- the stride phases: which input pixels, which taps reach them
  struct PhaseTaps {
    Phase ph;
    std::vector<int> taps[3], offs[3];
  };
  std::vector<PhaseTaps> found;
  for (int r0 = 0; r0 < g.S[0]; ++r0)
    for (int r1 = 0; r1 < g.S[1]; ++r1)
      for (int r2 = 0; r2 < g.S[2]; ++r2) {
        const int rho[3] = {r0, r1, r2};
        PhaseTaps pt{};
        bool empty = false;
        for (int k = 0; k < 3; ++k) {
          // input pixels i with (i + pad) % stride == rho
          const int i0 = ((rho[k] - g.P[k]) % g.S[k] + g.S[k]) % g.S[k];
          pt.ph.o0[k] = i0;
          pt.ph.J[k] = i0 < g.X[k] ? (g.X[k] - i0 + g.S[k] - 1) / g.S[k] : 0;
          if (pt.ph.J[k] == 0) empty = true;
          // taps that can reach them: t*dil % stride == rho; the window index is then
          // g = j + (i0 + pad - t*dil) / stride  (exact division)
          for (int tt = 0; tt < g.W[k]; ++tt)
            if ((tt * g.D[k]) % g.S[k] == rho[k]) {
              pt.taps[k].push_back(tt);
              pt.offs[k].push_back((i0 + g.P[k] - tt * g.D[k]) / g.S[k]);
            }
        }
        if (empty) continue;
        pt.ph.npos = (int)((long long)g.N * pt.ph.J[0] * pt.ph.J[1] * pt.ph.J[2]);
        set_divisors(pt.ph);
        found.push_back(pt);
      }

  // ---- up to four channels (single precision): one position of the coarse grid ceil(X / stride)
  // per lane, all of its stride phases at once
  {
    long long coarse_pos = g.N;
    for (int k = 0; k < 3; ++k) coarse_pos *= (g.X[k] + g.S[k] - 1) / g.S[k];
    if (g.C <= 4 && thin_applies(g, g.C, coarse_pos, (long long)g.F * g.wvol, nphase) && (long long)found.size() == nphase) {
      std::stable_sort(found.begin(), found.end(), [](const PhaseTaps &a, const PhaseTaps &b) {
        if (a.ph.o0[0] != b.ph.o0[0]) return a.ph.o0[0] < b.ph.o0[0];
        if (a.ph.o0[1] != b.ph.o0[1]) return a.ph.o0[1] < b.ph.o0[1];
        return a.ph.o0[2] < b.ph.o0[2];
      });
      std::map<std::array<int, 3>, ThinUse> seen;  // ordered by offset: neighbours along the last axis share a chunk
      for (int f = 0; f < (int)nphase; ++f) {
        const PhaseTaps &pt = found[f];
        for (int k = 0; k < 3; ++k) {
          pl.po0[f][k] = pt.ph.o0[k];
          pl.pJ[f][k] = pt.ph.J[k];
        }
        for (size_t a = 0; a < pt.taps[0].size(); ++a)
          for (size_t b = 0; b < pt.taps[1].size(); ++b)
            for (size_t c = 0; c < pt.taps[2].size(); ++c) {
              const std::array<int, 3> d{pt.offs[0][a], pt.offs[1][b], pt.offs[2][c]};
              auto it = seen.find(d);
              if (it == seen.end()) it = seen.emplace(d, ThinUse{{d[0], d[1], d[2]}, {-1, -1, -1, -1}}).first;
              it->second.tap[f] = (pt.taps[0][a] * g.W[1] + pt.taps[1][b]) * g.W[2] + pt.taps[2][c];
            }
      }
      std::vector<ThinUse> uses;
      for (const auto &kv : seen) uses.push_back(kv.second);
      thin_tables(pl, t, uses, (int)nphase, g.C, g.F, g.gvol, gs, (long long)g.C * g.wvol, g.wvol);
      Phase coarse{};
      for (int k = 0; k < 3; ++k) coarse.J[k] = (g.X[k] + g.S[k] - 1) / g.S[k];
      coarse.npos = (int)coarse_pos;
      set_divisors(coarse);
      pl.thin_grid = coarse;
      pl.pos_blocks = (int)ceil_div(coarse.npos, 256);
      pl.bm = 4, pl.bn = 256;
      return upload_plan(pl, t);
    }
  }

  // ---- few channels, unit strides, a 3-tap "same" last axis (float): the rows of the GEMM are
  // (channel, tap of the last axis), three times as many as there are channels, and the K tiles
  // run over the taps of the other axes only.  A gathered element of grad then feeds three
  // times the MFMAs -- with 16 channels the plain tiles are bound by the gather, not by the
  // matrix pipes -- and the epilogue adds the three rows of a channel, shifted along the last
  // axis, into dx.  A wave's 64 positions must be whole rows: rows of up to 64 positions, padded
  // to a power of two.
  if (fold_applies(g, g.C, g.F) && pl.tap_major && !pl.table_rows && nphase == 1 && found.size() == 1) {
    const PhaseTaps &pt = found[0];
    Phase ph = pt.ph;
    for (int f0 = 0; f0 < g.F; f0 += bk)
      for (size_t a = 0; a < pt.taps[0].size(); ++a)
        for (size_t b = 0; b < pt.taps[1].size(); ++b) {
          KTile e{};
          e.d0 = pt.offs[0][a];
          e.d1 = pt.offs[1][b];
          e.d2 = 0;
          e.a_row0 = (pt.taps[0][a] * g.W[1] + pt.taps[1][b]) * g.F + f0;
          e.coff = (int)(f0 * g.gvol) + e.d0 * gs[0] + e.d1 * gs[1];
          t.ktiles.push_back(e);
        }
    ph.k_begin = 0;
    ph.k_count = (int)t.ktiles.size();
    ph.blk_begin = 0;
    pad_fold_rows(g, pl, ph);
    set_fold_tile(g, pl, g.C, bk);
    pl.pos_blocks = (int)ceil_div(ph.npos, pl.bn);
    pl.full_tiles = pl.pos_blocks;
    t.phases.push_back(ph);
    return upload_plan(pl, t);
  }

  // ---- a few channels under a stride, not taken by the kernel above (double precision, or too few
  // positions for it): the stride phases become rows of the GEMM.  With three channels a 16-row tile
  // has three live rows per phase; with the rows (phase, channel) over the coarse grid ceil(X / stride)
  // it has phases x channels of them, and every gathered element of grad serves all phases of its
  // coarse position (a zero in the packed filters where a phase has no tap for it).
  const bool phase_rows_on = phase_rows_enabled();
  if (phase_rows_on && pl.tap_major && !pl.table_rows && nphase >= 2 && nphase <= 4 && (long long)found.size() == nphase &&
      nphase * g.C <= 16 && g.C <= 8 && 2.0 * g.N * g.F * g.gvol * g.C * g.wvol >= 2e8) {
    std::stable_sort(found.begin(), found.end(), [](const PhaseTaps &a, const PhaseTaps &b) {
      if (a.ph.o0[0] != b.ph.o0[0]) return a.ph.o0[0] < b.ph.o0[0];
      if (a.ph.o0[1] != b.ph.o0[1]) return a.ph.o0[1] < b.ph.o0[1];
      return a.ph.o0[2] < b.ph.o0[2];
    });
    std::map<std::array<int, 3>, std::array<int, 4>> seen;  // gathered offset -> the tap it meets in each phase (-1: none)
    for (int f = 0; f < (int)nphase; ++f) {
      const PhaseTaps &pt = found[f];
      for (int k = 0; k < 3; ++k) {
        pl.po0[f][k] = pt.ph.o0[k];
        pl.pJ[f][k] = pt.ph.J[k];
      }
      for (size_t a = 0; a < pt.taps[0].size(); ++a)
        for (size_t b = 0; b < pt.taps[1].size(); ++b)
          for (size_t c = 0; c < pt.taps[2].size(); ++c) {
            const std::array<int, 3> d{pt.offs[0][a], pt.offs[1][b], pt.offs[2][c]};
            auto it = seen.find(d);
            if (it == seen.end()) it = seen.emplace(d, std::array<int, 4>{-1, -1, -1, -1}).first;
            it->second[f] = (pt.taps[0][a] * g.W[1] + pt.taps[1][b]) * g.W[2] + pt.taps[2][c];
          }
    }
    std::vector<std::array<int, 3>> offsets;
    for (const auto &kv : seen) {
      offsets.push_back(kv.first);
      for (int f = 0; f < (int)nphase; ++f) t.arow.push_back(kv.second[f]);
    }
    const int entries = (int)offsets.size();
    for (int f0 = 0; f0 < g.F; f0 += bk)  // filter block outermost: its offsets share a neighbourhood of grad
      for (int e = 0; e < entries; ++e) {
        KTile kt{};
        kt.d0 = offsets[e][0], kt.d1 = offsets[e][1], kt.d2 = offsets[e][2];
        kt.a_row0 = e * g.F + f0;
        kt.coff = (int)(f0 * g.gvol) + kt.d0 * gs[0] + kt.d1 * gs[1] + kt.d2 * gs[2];
        t.ktiles.push_back(kt);
      }
    Phase coarse{};
    for (int k = 0; k < 3; ++k) coarse.J[k] = (g.X[k] + g.S[k] - 1) / g.S[k];
    coarse.k_begin = 0;
    coarse.k_count = (int)t.ktiles.size();
    coarse.blk_begin = 0;
    coarse.npos = (int)((long long)g.N * coarse.J[0] * coarse.J[1] * coarse.J[2]);
    set_divisors(coarse);
    const TileChoice tc = choose_tile((int)nphase * g.C, {(long long)coarse.npos}, coarse.k_count, true, g.dtype == MG_F64 ? 8 : 4, 1, bk);
    if (tc.bm != 0 && coarse.k_count > 0) {
      pl.bm = tc.bm, pl.bn = tc.bn, pl.m_tiles = tc.m_tiles, pl.full_tiles = tc.full_tiles, pl.tail_split = tc.tail_split, pl.blocks_per_cu = tc.blocks_per_cu;
      pl.phase_rows = g.C;
      pl.phase_count = (int)nphase;
      pl.table_count = entries;
      t.phases.push_back(coarse);
      pl.pos_blocks = (int)ceil_div(coarse.npos, pl.bn);
      return upload_plan(pl, t);
    }
    t.arow.clear();
    t.ktiles.clear();
  }

  // ---- stride 2 along the last axis: the phases' elements alternate in dx, and phases that
  // write them at different times make every line of dx cross HBM several times, partly
  // filled.  With 2 or 4 phases in all, every tile computes all of them for its patch of the
  // coarse grid J = ceil(X / stride) and writes them together (float only: one set of
  // accumulators per phase has to fit next to the other registers).
  static const bool fuse_on = [] {
    const char *flag = getenv("MYGRAD_HIP_FUSE");
    return !(flag && flag[0] == '0');
  }();
  // Four phases of short rows are left apart: what the fusion buys is whole lines of dx, and a row of
  // 13 elements is no whole line either way, while the fused tiles (64 x 64, four sets of
  // accumulators) are the slower ones.  Measured on twelve 3x3 stride-2 layers, fused against
  // apart: rows of 55 elements 0.67, of 27 elements 0.74 - 1.02 (0.83 on configuration 3b), of 13
  // elements 1.00 - 1.16, of 7 elements 1.19.
  // (MYGRAD_HIP_FUSE_MIN_ROW sets the shortest row that is still fused; read whenever a plan is
  // built and part of the plan's key, for the tests of the fused kernels on small problems)
  const int fuse_min_row = [] {
    const char *v = getenv("MYGRAD_HIP_FUSE_MIN_ROW");
    return v ? atoi(v) : 20;
  }();
  const bool fused = fuse_on && pl.tap_major && !pl.table_rows && g.dtype == MG_F32 && g.S[2] == 2 && g.S[0] <= 2 && g.S[1] <= 2 &&
                     (nphase == 2 || nphase == 4) && (long long)found.size() == nphase && (nphase == 2 || g.X[2] >= fuse_min_row);
  if (fused) {
    std::stable_sort(found.begin(), found.end(), [](const PhaseTaps &a, const PhaseTaps &b) {
      if (a.ph.o0[0] != b.ph.o0[0]) return a.ph.o0[0] < b.ph.o0[0];
      if (a.ph.o0[1] != b.ph.o0[1]) return a.ph.o0[1] < b.ph.o0[1];
      return a.ph.o0[2] < b.ph.o0[2];
    });
    pl.nph = (int)nphase;
    // Four phases share a tile's time: a K tile of 16 would be 16 MFMAs per wave between two
    // barriers.  With 32 filters per K tile the barriers cost half as much.
    const int fbk = nphase == 4 && g.F % 32 == 0 && deep_fused_on() ? 32 : bk;
    pl.bk = fbk;
    Phase coarse{};
    long long total_ktiles = 0;
    for (int k = 0; k < 3; ++k) coarse.J[k] = (g.X[k] + g.S[k] - 1) / g.S[k];
    int taps_so_far = 0;
    for (int f = 0; f < pl.nph; ++f) {
      const PhaseTaps &pt = found[f];
      for (int k = 0; k < 3; ++k) {
        pl.po0[f][k] = pt.ph.o0[k];
        pl.pJ[f][k] = pt.ph.J[k];
      }
      taps_so_far += (int)(pt.taps[0].size() * pt.taps[1].size() * pt.taps[2].size());
      pl.kcut[f] = taps_so_far;  // every filter tap belongs to exactly one phase: W taps in all
    }
    // filter block outermost, then the phases, then a phase's taps: all taps of one filter block
    // read the same neighbourhood of grad, whichever phase they belong to
    for (int f0 = 0; f0 < g.F; f0 += fbk)
      for (int f = 0; f < pl.nph; ++f) {
        const PhaseTaps &pt = found[f];
        for (size_t a = 0; a < pt.taps[0].size(); ++a)
          for (size_t b = 0; b < pt.taps[1].size(); ++b)
            for (size_t c = 0; c < pt.taps[2].size(); ++c) {
              const int tflat = (pt.taps[0][a] * g.W[1] + pt.taps[1][b]) * g.W[2] + pt.taps[2][c];
              KTile e{};
              e.d0 = pt.offs[0][a];
              e.d1 = pt.offs[1][b];
              e.d2 = pt.offs[2][c];
              e.a_row0 = tflat * g.F + f0;
              e.coff = (int)(f0 * g.gvol) + e.d0 * gs[0] + e.d1 * gs[1] + e.d2 * gs[2];
              t.ktiles.push_back(e);
            }
      }
    total_ktiles = (long long)t.ktiles.size();
    coarse.k_begin = 0;
    coarse.k_count = (int)total_ktiles;
    coarse.blk_begin = 0;
    coarse.npos = (int)((long long)g.N * coarse.J[0] * coarse.J[1] * coarse.J[2]);
    set_divisors(coarse);
    const TileChoice tc = choose_tile(g.C, {(long long)coarse.npos}, (int)total_ktiles, true, 4, pl.nph, fbk);
    if (tc.bm != 0 && total_ktiles > 0) {
      pl.bm = tc.bm, pl.bn = tc.bn, pl.m_tiles = tc.m_tiles, pl.full_tiles = tc.full_tiles, pl.tail_split = tc.tail_split, pl.blocks_per_cu = tc.blocks_per_cu;
      t.phases.push_back(coarse);
      pl.pos_blocks = (int)ceil_div(coarse.npos, pl.bn);
      return upload_plan(pl, t);
    }
    // no tile shape for this row count: the phases run one after the other
    pl.nph = 1;
    pl.bk = bk;
    t.ktiles.clear();
  }

  // Phases with more taps have longer K loops; their blocks go first so that the
  // short ones fill in at the end (blocks are dispatched in index order).
  std::stable_sort(found.begin(), found.end(), [](const PhaseTaps &a, const PhaseTaps &b) {
    return a.taps[0].size() * a.taps[1].size() * a.taps[2].size() > b.taps[0].size() * b.taps[1].size() * b.taps[2].size();
  });

  // ---- tile shape and tail sharing
  {
    std::vector<long long> npos;
    long long min_ktiles = 1 << 30;
    for (const PhaseTaps &pt : found) {
      npos.push_back(pt.ph.npos);
      const long long ntaps = (long long)pt.taps[0].size() * pt.taps[1].size() * pt.taps[2].size();
      min_ktiles = std::min(min_ktiles, pl.tap_major && !pl.table_rows ? ntaps * (g.F / bk) : ceil_div(ntaps * g.F, bk));
    }
    long long all_ktiles = 0, all_pos = 0;
    for (const PhaseTaps &pt : found) {
      const long long ntaps = (long long)pt.taps[0].size() * pt.taps[1].size() * pt.taps[2].size();
      all_ktiles += ceil_div(ntaps * g.F, bk) * pt.ph.npos;
      all_pos += pt.ph.npos;
    }
    const TileChoice tc = choose_tile(g.C, npos, (int)std::max<long long>(min_ktiles, 0), pl.tap_major, g.dtype == MG_F64 ? 8 : 4, 1, bk,
                                      (int)(all_ktiles / std::max<long long>(all_pos, 1)));
    pl.bm = tc.bm, pl.bn = tc.bn, pl.m_tiles = tc.m_tiles, pl.full_tiles = tc.full_tiles, pl.tail_split = tc.tail_split, pl.blocks_per_cu = tc.blocks_per_cu;
    deepen_if_tiny(g, pl);
  }

  // ---- tables
  int blk = 0;
  for (PhaseTaps &pt : found) {
    Phase &ph = pt.ph;
    ph.k_begin = pl.tap_major ? (int)t.ktiles.size() : (int)t.tab.size();
    if (pl.table_rows) {
      // the phase's rows (filter, tap), padded to whole K tiles with rows that lie outside every
      // input and name no element of the filter bank (a zero row of the packed filters)
      const int first_row = (int)t.tab.size();
      for (int f = 0; f < g.F; ++f)
        for (size_t a = 0; a < pt.taps[0].size(); ++a)
          for (size_t b = 0; b < pt.taps[1].size(); ++b)
            for (size_t c = 0; c < pt.taps[2].size(); ++c) {
              TabEntry e;
              e.d0 = pt.offs[0][a];
              e.d1 = pt.offs[1][b];
              e.d2 = pt.offs[2][c];
              e.off = (int)(f * g.gvol) + e.d0 * gs[0] + e.d1 * gs[1] + e.d2 * gs[2];
              t.tab.push_back(e);
              t.arow.push_back((int)(f * g.C * g.wvol) + (pt.taps[0][a] * g.W[1] + pt.taps[1][b]) * g.W[2] + pt.taps[2][c]);
            }
      TabEntry outside{};
      outside.d0 = outside.d1 = outside.d2 = 1 << 29;
      while ((t.tab.size() - first_row) % bk != 0) {
        t.tab.push_back(outside);
        t.arow.push_back(-1);
      }
      for (int k0 = first_row; k0 < (int)t.tab.size(); k0 += bk) {
        KTile e{};
        e.a_row0 = k0;
        e.coff = k0;  // first table row of the tile
        t.ktiles.push_back(e);
      }
      ph.k_count = (int)t.ktiles.size() - ph.k_begin;
    } else if (pl.tap_major) {
      for (int f0 = 0; f0 < g.F; f0 += bk)  // filter block outermost: its taps share rows of grad
        for (size_t a = 0; a < pt.taps[0].size(); ++a)
          for (size_t b = 0; b < pt.taps[1].size(); ++b)
            for (size_t c = 0; c < pt.taps[2].size(); ++c) {
              const int tflat = (pt.taps[0][a] * g.W[1] + pt.taps[1][b]) * g.W[2] + pt.taps[2][c];
              KTile e{};
              e.d0 = pt.offs[0][a];
              e.d1 = pt.offs[1][b];
              e.d2 = pt.offs[2][c];
              e.a_row0 = tflat * g.F + f0;
              e.coff = (int)(f0 * g.gvol) + e.d0 * gs[0] + e.d1 * gs[1] + e.d2 * gs[2];
              t.ktiles.push_back(e);
            }
      ph.k_count = (int)t.ktiles.size() - ph.k_begin;
    } else {
      for (int f = 0; f < g.F; ++f)
        for (size_t a = 0; a < pt.taps[0].size(); ++a)
          for (size_t b = 0; b < pt.taps[1].size(); ++b)
            for (size_t c = 0; c < pt.taps[2].size(); ++c) {
              TabEntry e;
              e.d0 = pt.offs[0][a];
              e.d1 = pt.offs[1][b];
              e.d2 = pt.offs[2][c];
              e.off = (int)(f * g.gvol) + e.d0 * gs[0] + e.d1 * gs[1] + e.d2 * gs[2];
              t.tab.push_back(e);
              t.arow.push_back((int)(f * g.C * g.wvol) + (pt.taps[0][a] * g.W[1] + pt.taps[1][b]) * g.W[2] + pt.taps[2][c]);
            }
      ph.k_count = (int)t.tab.size() - ph.k_begin;
    }
    ph.blk_begin = blk;
    blk += (int)ceil_div(ph.npos, pl.bn);
    t.phases.push_back(ph);
  }
  pl.pos_blocks = blk;
  pl.table_count = (int)t.tab.size();
  return upload_plan(pl, t);
}

// Tile shapes of the filter-gradient kernels: rows (filters) x columns x K tile, and the
// wave tile.  The table-driven kernel has the 64-column shapes only.
#define MG_WGRAD_SHAPES(T, X)                                                          \
  X(T, 128, 128, (sizeof(T) == 8 ? 16 : 32), 64, 64)                                   \
  X(T, 64, 64, (sizeof(T) == 8 ? 32 : 64), 32, 32)                                     \
  X(T, 32, 128, (sizeof(T) == 8 ? 16 : 32), 32, 32)                                    \
  X(T, 32, 64, (sizeof(T) == 8 ? 32 : 64), 32, 16)                                     \
  X(T, 16, 64, (sizeof(T) == 8 ? 32 : 64), 16, 16)

// Blocks of the filter-gradient kernel that fit on one compute unit at a time.
// Tile shapes that only the table-row mode of the tap-major filter-gradient kernel has.
#define MG_WGRAD_TABLE_SHAPES(T, X)                \
  X(T, 64, 80, (sizeof(T) == 8 ? 32 : 64), 16, 80) \
  X(T, 64, 32, (sizeof(T) == 8 ? 32 : 64), 32, 16)

template <typename T>
int wgrad_blocks_per_cu(int bm, int bn, bool tap_major) {
#define MG_OCC_TABLE(TT, BM, BN, BK, WM, WN) \
  if (bm == BM && bn == BN && tap_major) return resident_blocks(tap_wgrad_kernel<TT, BM, BN, BK, WM, WN, true, true>, 512);
  MG_WGRAD_TABLE_SHAPES(T, MG_OCC_TABLE)
#undef MG_OCC_TABLE
#define MG_OCC(TT, BM, BN, BK, WM, WN)                                                     \
  if (bm == BM && bn == BN) {                                                              \
    if (tap_major) return resident_blocks(tap_wgrad_kernel<TT, BM, BN, BK, WM, WN, true>, 512);  \
    if constexpr (BN == 64) return resident_blocks(wgrad_kernel<TT, BM, BN, BK, WM, WN>, 256); \
  }
  MG_WGRAD_SHAPES(T, MG_OCC)
#undef MG_OCC
  return 1;
}

// The position table of the tap-major filter-gradient kernel: row idx describes position
// (n, g0, g1, g2) = idx in row-major order (see WgradParams::pos_tab).  The coordinate offsets
// (d0, d1, d2) of tap t lie at taps[t * tap_ints ...]: in the column groups of the first channel
// block, one per tap, or in the first channel's rows of the gather table.
__global__ void __launch_bounds__(256) wgrad_pos_table_kernel(unsigned *__restrict__ tab, const int *__restrict__ taps, int tap_ints, int wvol, int kpos,
                                                              int gvol, int g12, int g2n, int sj0, int sj1, int sj2, int qs0, int qs1, int qs2,
                                                              int q0, int q1, int q2, long long x_nstride, long long grad_extra,
                                                              int elem) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= kpos) return;
  const int n = idx / gvol;
  const int gflat = idx - n * gvol;
  const int g0 = gflat / g12;
  const int r = gflat - g0 * g12;
  const int g1 = r / g2n;
  const int g2 = r - g1 * g2n;
  const int qb0 = g0 * sj0, qb1 = g1 * sj1, qb2 = g2 * sj2;
  unsigned lo = 0, hi = 0;
  for (int t = 0; t < wvol; ++t) {
    const int *d = taps + (long long)t * tap_ints;
    const bool ok = ((unsigned)(qb0 + d[0]) < (unsigned)q0) & ((unsigned)(qb1 + d[1]) < (unsigned)q1) & ((unsigned)(qb2 + d[2]) < (unsigned)q2);
    if (ok) (t < 32 ? lo : hi) |= 1u << (t & 31);
  }
  uint4 row;
  row.x = (unsigned)((n * x_nstride + (long long)qb0 * qs0 + (long long)qb1 * qs1 + (long long)qb2 * qs2) * elem);
  row.y = lo;
  row.z = hi;
  row.w = (unsigned)(n * grad_extra * elem);
  reinterpret_cast<uint4 *>(tab)[idx] = row;
}

// MYGRAD_HIP_POS_TABLE=0 keeps the filter-gradient kernel on its in-kernel position arithmetic.
// Single precision only: measured with the table, config 5 271 -> 263 us, config 3b 129.5 -> 123.6 us,
// a 4096^3 product's da 1015 -> 973 us, config 3a unchanged, a 7x7 stride-2 first layer on table rows
// 372 -> 344 us; double precision 1 % (config 4) to 7 % (the same first layer) slower.
inline bool pos_table_enabled() {
  const char *flag = getenv("MYGRAD_HIP_POS_TABLE");
  return !(flag && flag[0] == '0');
}

int build_pos_table(const Geometry &g, Plan &pl) {
  const long long kpos = (long long)g.N * g.gvol;
  if (!pl.tap_major || g.dtype != MG_F32 || g.wvol > 64 || kpos * 16 > (32ll << 20) || !pos_table_enabled()) return MG_OK;
  if (hipMalloc(&pl.pos_tab, (size_t)kpos * 16) != hipSuccess) {
    // no room for the table: the kernels do the arithmetic themselves
    (void)hipGetLastError();
    pl.pos_tab = nullptr;
    return MG_OK;
  }
  // both kinds of row start with an element offset, followed by the three coordinate offsets
  const int *taps = pl.table_rows ? reinterpret_cast<const int *>(pl.tab) + 1 : reinterpret_cast<const int *>(pl.groups) + 1;
  const int tap_ints = (int)((pl.table_rows ? sizeof(TabEntry) : sizeof(WGroup)) / sizeof(int));
  hipLaunchKernelGGL(wgrad_pos_table_kernel, dim3((unsigned)ceil_div(kpos, 256)), dim3(256), 0, runtime().stream,
                     static_cast<unsigned *>(pl.pos_tab), taps, tap_ints, (int)g.wvol, (int)kpos, (int)g.gvol, g.G[1] * g.G[2], g.G[2], g.S[0], g.S[1],
                     g.S[2], g.X[1] * g.X[2], g.X[2], 1, g.X[0], g.X[1], g.X[2], (long long)g.C * g.xvol, (long long)(g.F - 1) * g.gvol,
                     g.dtype == MG_F64 ? 8 : 4);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int build_wgrad_plan(const Geometry &g, Plan &pl) {
  Tables t;
  const bool f64 = g.dtype == MG_F64;
  const long long ct = (long long)g.C * g.wvol;
  const long long kpos = (long long)g.N * g.gvol;
  const int cus = runtime().props.multiProcessorCount;
  // Split K so that all blocks are resident at once (one round: no half-empty second
  // round), with at least 4 K tiles per block.
  auto splits_for = [&](int bm, int bn, int bk, bool tap) {
    const long long tiles = ceil_div(ct, bn) * ceil_div(g.F, bm);
    const long long ktiles = ceil_div(kpos, bk);
    const int per_cu = f64 ? wgrad_blocks_per_cu<double>(bm, bn, tap) : wgrad_blocks_per_cu<float>(bm, bn, tap);
    const long long slots = (long long)per_cu * cus;
    const long long max_splits = std::max<long long>(1, std::min<long long>(ktiles / 4, 1024));
    if (tiles > slots) {
      // More tiles than block slots (a large dw, as in a matrix product): the blocks run in
      // rounds and the last round may be nearly empty.  Splitting K evens the rounds out at
      // the price of one more copy of dw written and read back per split: take the split
      // that minimises  (time of the rounds) + (time of that traffic).
      const double work = 2.0 * (double)g.F * (double)ct * (double)kpos / (0.7 * (f64 ? 78.6e12 : 157.3e12));
      const double copy = 2.0 * (double)g.F * (double)ct * (f64 ? 8.0 : 4.0) / 4.0e12;
      long long best = 1;
      double best_time = 0;
      for (long long sp = 1; sp <= std::min<long long>(max_splits, 16); ++sp) {
        const long long blocks = tiles * sp;
        const double rounds = (double)ceil_div(blocks, slots) * (double)slots / (double)blocks;
        const double time = work * rounds + copy * (double)sp;
        if (sp == 1 || time < best_time) best = sp, best_time = time;
      }
      return best;
    }
    return std::max<long long>(1, std::min(slots / tiles, max_splits));
  };
  // Tap-major candidates in the order of preference: the first shape wins that divides F, wastes
  // little on padding the columns to whole tiles and still fills most block slots of the device
  // with tiles x K splits.  128 x 128 re-reads grad and x least.  With 64 filters the tile is square
  // with the K tile 64 deep (half the barriers, one column group per gathering thread): tiles of
  // 64 x 192 and 64 x 128 with K tiles of 32, forced in turn on four layers with 64 filters, were
  // 3 - 13 % slower (3x3 at 56x56: 240 / 250 / 294 us; 5x5 dilated: 173 / 192 / 197 us) and are
  // no longer built.
  struct Cand {
    int bm, bn, bk;
  };
  const Cand cands[] = {{128, 128, f64 ? 16 : 32}, {64, 64, f64 ? 32 : 64}, {32, 128, f64 ? 16 : 32},
                        {32, 64, f64 ? 32 : 64},   {16, 64, f64 ? 32 : 64}};
  long long best_splits = 1;
  pl.bm = 0;
  // MYGRAD_HIP_WGRAD_TILE="rows,columns" (diagnostics and the tests of every tile shape; part of the
  // plan's key): that candidate or, where it does not apply, the usual choice
  int forced_bm = 0, forced_bn = 0;
  if (const char *v = getenv("MYGRAD_HIP_WGRAD_TILE")) sscanf(v, "%d,%d", &forced_bm, &forced_bn);
  bool forced = false;
  for (const Cand &c : cands)
    forced |= c.bm == forced_bm && c.bn == forced_bn && g.F % c.bm == 0 && !(c.bm == 32 && c.bn == 128 && !f64);
  if (g.C % 16 == 0 && fits_buffer_loads(g)) {
    for (const Cand &c : cands) {
      if (forced && (c.bm != forced_bm || c.bn != forced_bn)) continue;
      if (g.F % c.bm != 0) continue;
      // 32x64 double-precision tiles are bound by LDS reads (the 4x4x4 MFMA takes an operand
      // per 512 flops); the wider tile halves them per flop and is worth more padding.
      // In single precision 32x128 measured slower than 32x64.
      if (c.bm == 32 && c.bn == 128 && !f64) continue;
      const long long col_tiles = ceil_div(ct, c.bn), row_tiles = g.F / c.bm;
      const long long splits = splits_for(c.bm, c.bn, c.bk, true);
      if (c.bn > 64 && !forced) {
        const int per_cu = f64 ? wgrad_blocks_per_cu<double>(c.bm, c.bn, true) : wgrad_blocks_per_cu<float>(c.bm, c.bn, true);
        const double waste = (double)(col_tiles * c.bn - ct) / (double)ct;
        const double filled = (double)(col_tiles * row_tiles * splits) / ((double)per_cu * cus);
        if (waste > (c.bm == 32 ? 0.15 : 0.12) || filled < 0.75) continue;
      }
      best_splits = splits;
      pl.bm = c.bm, pl.bn = c.bn, pl.bk = c.bk;
      break;
    }
  }
  pl.tap_major = pl.bm != 0;
  if (!pl.tap_major) {
    // Channels that fill no group of 16 columns: the tap-major kernel with one table row per
    // column (64-column tiles, filters in whole row tiles), unless the problem is tiny or
    // MYGRAD_HIP_TABLE_ROWS=0 asks for the plain table-driven kernel.
    static const bool rows_on = [] {
      const char *flag = getenv("MYGRAD_HIP_TABLE_ROWS");
      return !(flag && flag[0] == '0');
    }();
    // filters in row tiles of 16, 32 or 64, the last one possibly short: its rows beyond F read
    // whatever follows in grad (or zeros past its end) and are not stored
    const int row_tile = g.F <= 16 ? 16 : g.F <= 32 ? 32 : g.F <= 48 ? 16 : 64;
    if (rows_on && fits_buffer_loads(g)) {
      pl.tap_major = pl.table_rows = true;
      pl.bm = row_tile;
      pl.bn = 64;
      pl.bk = f64 ? 32 : 64;
      if (row_tile == 64) {
        // 64-row tiles also come 32 and 80 columns wide: the width that pads the columns least
        // (a 7x7 filter on three channels: 147 columns are 160 in tiles of 80, 192 in tiles of 64)
        for (int bn : {80, 32})
          if (ceil_div(ct, bn) * bn < ceil_div(ct, pl.bn) * pl.bn) pl.bn = bn;
      }
      best_splits = splits_for(pl.bm, pl.bn, pl.bk, true);
    } else {
      pl.bm = g.F <= 16 ? 16 : (g.F <= 32 ? 32 : 64);
      pl.bn = 64;
      pl.bk = f64 ? 32 : 64;
      best_splits = splits_for(pl.bm, pl.bn, pl.bk, false);
    }
  }
  const long long col_tiles = ceil_div(ct, pl.bn);
  const long long ktiles = ceil_div(kpos, pl.bk);
  const long long tiles_per_split = ceil_div(ktiles, best_splits);
  pl.kchunk = (int)(tiles_per_split * pl.bk);
  pl.splits = (int)ceil_div(kpos, pl.kchunk);
  if (pl.table_rows) {
    fwd_table(g, t.tab);
    TabEntry outside{};
    outside.d0 = outside.d1 = outside.d2 = 1 << 29;
    while ((long long)t.tab.size() < col_tiles * pl.bn) t.tab.push_back(outside);
  } else if (pl.tap_major) {
    const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
    const long long ngroups = col_tiles * (pl.bn / 16);
    for (long long gi = 0; gi < ngroups; ++gi) {
      WGroup e{};
      const long long col = gi * 16;  // group gi = (channel block, tap), taps innermost
      if (col < ct) {
        const int tflat = (int)(gi % g.wvol), c0 = (int)(gi / g.wvol) * 16;
        const int t2 = tflat % g.W[2], t1 = (tflat / g.W[2]) % g.W[1], t0 = tflat / (g.W[2] * g.W[1]);
        e.d0 = t0 * g.D[0] - g.P[0];
        e.d1 = t1 * g.D[1] - g.P[1];
        e.d2 = t2 * g.D[2] - g.P[2];
        e.coff = (int)(c0 * g.xvol) + e.d0 * qs[0] + e.d1 * qs[1] + e.d2 * qs[2];
        e.valid = 1;
      }
      t.groups.push_back(e);
    }
  } else {
    fwd_table(g, t.tab);
  }
  if (int rc = upload_plan(pl, t)) return rc;
  return build_pos_table(g, pl);
}

int get_plan(ConvOp op, const mg_conv_desc *d, const Geometry &g, Plan **out) {
  std::string key(reinterpret_cast<const char *>(d), sizeof *d);
  key.push_back((char)op);
  key.push_back(tiny_plans_enabled() ? 't' : 'T');
  key.push_back(thin_on() ? 'n' : 'N');
  key.push_back(phase_rows_enabled() ? 'p' : 'P');
  key.push_back(pos_table_enabled() ? 'q' : 'Q');
  if (const char *tile = getenv("MYGRAD_HIP_TILE")) key.append(tile);
  if (const char *tile = getenv("MYGRAD_HIP_WGRAD_TILE")) key.append("w").append(tile);
  if (const char *row = getenv("MYGRAD_HIP_FUSE_MIN_ROW")) key.append("r").append(row);
  auto it = plans().find(key);
  if (it == plans().end()) {
    if (plans().size() >= 256) {
      // crude bound on cached tables; kernels in flight may still read the old ones
      MG_HIP(hipStreamSynchronize(runtime().stream));
      release_conv_plans();
    }
    Plan pl;
    int rc = op == OP_FWD ? build_fwd_plan(g, pl) : op == OP_DGRAD ? build_dgrad_plan(g, pl) : build_wgrad_plan(g, pl);
    if (rc) return rc;
    char tail[64];
    if (pl.share_grid > 0)
      snprintf(tail, sizeof tail, "even shares of the rest (%d partial slices)", pl.share_slots);
    else
      snprintf(tail, sizeof tail, "tail split %d", pl.tail_split);
    snprintf(pl.note, sizeof pl.note,
             "%s: %s%s%s tile %dx%dx%d, %d phase(s) (%d fused per tile), %d position blocks x %d row tiles, %d whole tiles + %s, "
             "%d block(s) per unit, K splits %d",
             op == OP_FWD ? "fwd" : op == OP_DGRAD ? "dgrad" : "wgrad",
             pl.thin ? "one position per lane" : pl.tap_major ? "tap-major" : "table-driven", pl.table_rows ? ", table rows" : pl.phase_rows ? ", stride phases as rows" : "",
             pl.fold_row ? ", folded taps" : "", pl.bm, pl.bn, pl.bk, pl.nphases, pl.nph, pl.pos_blocks, pl.m_tiles, pl.full_tiles, tail,
             pl.blocks_per_cu, pl.splits);
    // MYGRAD_HIP_TRACE=1 reports, once per new descriptor, what was planned
    static const bool trace = getenv("MYGRAD_HIP_TRACE") != nullptr;
    if (trace) fprintf(stderr, "[mygrad_hip] plan %s (K chunk %d)\n", pl.note, pl.kchunk);
    it = plans().emplace(key, pl).first;
  }
  *out = &it->second;
  note_plan(it->second.note);
  return MG_OK;
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int NPH = 1, bool FOLD = false, bool ROWS = false>
void launch_gemm(GemmParams &gp, const Plan &pl, hipStream_t s) {
  if (pl.tap_major) {
    const long long tiles = (long long)pl.pos_blocks * pl.m_tiles;
    const long long tail_tiles = tiles - pl.full_tiles;
    const long long slots = tap_gemm_streams(BM, (int)sizeof(T)) ? (long long)pl.blocks_per_cu * runtime().props.multiProcessorCount : (1ll << 40);
    gp.share_first = pl.share_first, gp.share_slices = pl.share_slices, gp.share_fix = pl.share_fix;
    if (pl.share_grid > 0) {
      // whole tiles b, b + grid, ... and then one even share of the remaining tiles' K tiles per block
      gp.items = pl.full_tiles;
      hipLaunchKernelGGL((tap_gemm_kernel<T, BM, BN, BK, WM, WN, NPH, FOLD, ROWS>), dim3((unsigned)pl.share_grid), dim3(512), 0, s, gp);
      if (pl.share_fixes > 0)
        hipLaunchKernelGGL((tail_fixup_kernel<T, BM, BN, NPH>), dim3((unsigned)ceil_div(BM * BN, 256), (unsigned)pl.share_fixes),
                           dim3(256), 0, s, gp);
      return;
    }
    gp.items = (int)(pl.full_tiles + tail_tiles * pl.tail_split);
    const long long grid = std::min<long long>(gp.items, slots);
    // MYGRAD_HIP_XCD_CHUNK=0 (read at every launch): every block starts on the tile of its own number
    const bool chunks_on = [] {
      const char *flag = getenv("MYGRAD_HIP_XCD_CHUNK");
      return !(flag && flag[0] == '0');
    }();
    const int c = pl.m_tiles;
    gp.xcd_chunk = chunks_on && tap_gemm_streams(BM, (int)sizeof(T)) && grid == slots && (c == 2 || c == 4 || c == 8) && grid % (8 * c) == 0 ? c : 1;
    hipLaunchKernelGGL((tap_gemm_kernel<T, BM, BN, BK, WM, WN, NPH, FOLD, ROWS>), dim3((unsigned)grid), dim3(512), 0, s, gp);
    if (tail_tiles > 0)
      hipLaunchKernelGGL((tail_fixup_kernel<T, BM, BN, NPH>), dim3((unsigned)ceil_div(BM * BN, 256), (unsigned)tail_tiles),
                         dim3(256), 0, s, gp);
  } else if constexpr (NPH == 1 && !FOLD && !ROWS) {
    const dim3 grid((unsigned)pl.pos_blocks, (unsigned)pl.m_tiles);
    hipLaunchKernelGGL((gather_gemm_kernel<T, BM, BN, BK, WM, WN>), grid, dim3(256), 0, s, gp);
  }
}

// Bytes of partial sums the shared tail tiles of this plan need.
size_t tail_bytes(const Plan &pl, size_t elem) {
  const long long tail_tiles = (long long)pl.pos_blocks * pl.m_tiles - pl.full_tiles;
  if (pl.share_grid > 0) return (size_t)pl.share_slots * pl.nph * pl.bm * pl.bn * elem;
  return pl.tap_major ? (size_t)tail_tiles * pl.tail_split * pl.nph * pl.bm * pl.bn * elem : 0;
}

template <typename T>
int run_gemm(GemmParams &gp, const Plan &pl, int tag, hipStream_t s) {
  constexpr int BK = sizeof(T) == 8 ? 8 : 16;
  if (pl.pos_blocks <= 0) return MG_OK;
  gp.tab = pl.tab;
  gp.arow = pl.arow;
  gp.phases = pl.phases;
  gp.nphases = pl.nphases;
  gp.ktiles = pl.ktiles;
  gp.zeros = pl.zeros;
  gp.m_tiles = pl.m_tiles;
  gp.full_tiles = pl.tap_major ? pl.full_tiles : pl.pos_blocks * pl.m_tiles;
  gp.tail_split = pl.tail_split;
  // a lane may store its 4 positions as one vector when they are adjacent in dst
  // (positions run through dst in order, the per-sample volume is a multiple of 4,
  // and every row starts 16-byte aligned)
  gp.vec_store = pl.single_dense_phase && gp.dst_mstride % 4 == 0 && gp.dst_nstride % 4 == 0 &&
                 reinterpret_cast<uintptr_t>(gp.dst) % 16 == 0;
  gp.run_store = pl.single_dense_phase && !gp.vec_store;
  gp.nph = pl.nph;
  gp.phase_count = pl.phase_rows ? pl.phase_count : 0;
  // (the phases are sorted by their offsets, the last axis innermost: with a stride of two there, phases 2q and
  // 2q + 1 differ by one element along it)
  gp.phase_pairs = pl.phase_rows && gp.oj[2] == 2 && gp.os[2] == 1;
  if (pl.phase_rows)
    for (int f = 0; f < 4; ++f)
      for (int k = 0; k < 3; ++k) gp.po0[f][k] = pl.po0[f][k], gp.pJ[f][k] = pl.pJ[f][k];
  if (pl.nph > 1) {
    for (int f = 0; f < 4; ++f) {
      gp.kcut[f] = pl.kcut[f];
      for (int k = 0; k < 3; ++k) gp.po0[f][k] = pl.po0[f][k], gp.pJ[f][k] = pl.pJ[f][k];
    }
    // the two phases of a pair have the same positions (an even extent along the last axis),
    // and 2 * TN adjacent elements of a row of dst start 16-byte aligned
    gp.vec_store = pl.pJ[0][2] == pl.pJ[1][2] && gp.os[1] % 4 == 0 && gp.os[0] % 4 == 0 && gp.dst_mstride % 4 == 0 &&
                   gp.dst_nstride % 4 == 0 && reinterpret_cast<uintptr_t>(gp.dst) % 16 == 0;
  }
  ScopedTiming timed(tag);
  bool launched = false;
  if (pl.deep_k) {
    launch_gemm<T, 16, 64, 4 * BK, 16, 16>(gp, pl, s);
    launched = true;
  }
  if constexpr (sizeof(T) == 8) {
    if (pl.tap_major && pl.bk == 2 * BK && !pl.table_rows && !pl.fold_row) {
#define MG_LAUNCH_DEEP(TT, BM, BN, WM, WN)                \
  if (!launched && pl.bm == BM && pl.bn == BN) {          \
    launch_gemm<TT, BM, BN, 2 * BK, WM, WN>(gp, pl, s);   \
    launched = true;                                      \
  }
      MG_GEMM_SHAPES(T, MG_LAUNCH_DEEP)
#undef MG_LAUNCH_DEEP
    }
  }
  if (pl.table_rows) {
#define MG_LAUNCH_ROWS(TT, BM, BN, WM, WN)                              \
  if (!launched && pl.bm == BM && pl.bn == BN) {                        \
    launch_gemm<TT, BM, BN, 16, WM, WN, 1, false, true>(gp, pl, s);     \
    launched = true;                                                    \
  }
    MG_GEMM_SHAPES(T, MG_LAUNCH_ROWS)
#undef MG_LAUNCH_ROWS
  }
  gp.fold_row = pl.fold_row;
  if (pl.fold_row) {
    // a lane's four positions are adjacent in dst and all exist or all do not when the rows are
    // whole 16-byte pieces (positions do not run through dst in order: rows are padded)
    const int piece = (int)(16 / sizeof(T));
    gp.vec_store = gp.Q[2] % piece == 0 && gp.dst_mstride % piece == 0 && gp.dst_nstride % piece == 0 &&
                   gp.os[0] % piece == 0 && gp.os[1] % piece == 0 && reinterpret_cast<uintptr_t>(gp.dst) % 16 == 0;
  }
  if (pl.fold_row && !launched) {
    if (pl.bk == 2 * BK && sizeof(T) == 8) {
      if (pl.bm == 48)
        launch_gemm<T, 48, 256, (sizeof(T) == 8 ? 2 * BK : BK), 48, 64, 1, true>(gp, pl, s);
      else
        launch_gemm<T, 96, 128, (sizeof(T) == 8 ? 2 * BK : BK), 48, 64, 1, true>(gp, pl, s);
    } else if (pl.bm == 48) {
      launch_gemm<T, 48, 256, BK, 48, 64, 1, true>(gp, pl, s);
    } else {
      launch_gemm<T, 96, 128, BK, 48, 64, 1, true>(gp, pl, s);
    }
    launched = true;
  }
#define MG_LAUNCH(TT, BM, BN, WM, WN)                     \
  if (!launched && pl.bm == BM && pl.bn == BN) {          \
    launch_gemm<TT, BM, BN, BK, WM, WN>(gp, pl, s);       \
    launched = true;                                      \
  }
#define MG_LAUNCH2(TT, BM, BN, WM, WN)                    \
  if (!launched && pl.bm == BM && pl.bn == BN) {          \
    launch_gemm<TT, BM, BN, BK, WM, WN, 2>(gp, pl, s);    \
    launched = true;                                      \
  }
#define MG_LAUNCH4(TT, BM, BN, WM, WN)                    \
  if (!launched && pl.bm == BM && pl.bn == BN) {          \
    launch_gemm<TT, BM, BN, BK, WM, WN, 4>(gp, pl, s);    \
    launched = true;                                      \
  }
  if constexpr (sizeof(T) == 4) {
    if (pl.nph == 2) {
      MG_FUSED2_SHAPES(T, MG_LAUNCH2)
    } else if (pl.nph == 4 && pl.bk == 2 * BK) {
#define MG_LAUNCH4_DEEP(TT, BM, BN, WM, WN)                      \
  if (!launched && pl.bm == BM && pl.bn == BN) {                 \
    launch_gemm<TT, BM, BN, 2 * BK, WM, WN, 4>(gp, pl, s);       \
    launched = true;                                             \
  }
      MG_FUSED4_SHAPES(T, MG_LAUNCH4_DEEP)
#undef MG_LAUNCH4_DEEP
    } else if (pl.nph == 4) {
      MG_FUSED4_SHAPES(T, MG_LAUNCH4)
    }
  }
  if (pl.nph == 1) {
    MG_GEMM_SHAPES(T, MG_LAUNCH)
  }
#undef MG_LAUNCH
#undef MG_LAUNCH2
#undef MG_LAUNCH4
  if (!launched) return fail(MG_ERR_UNSUPPORTED, "no kernel for tile %d x %d", pl.bm, pl.bn);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// Packs the filters into the front of the library workspace; `extra` more bytes
// behind them (256-byte aligned) are reserved for the caller and returned in *behind.
// Values per row of the packed filters: M rounded up to a multiple of four.
inline int packed_ld(int M, bool tap_major) { return tap_major ? (M + 3) / 4 * 4 : M; }

// Values per packed row when the three taps of the last axis are rows (n channels or filters):
// 3n rounded up to four in single precision, whole 48-row wave tiles in double.
template <typename T>
int folded_ld(int n) {
  return sizeof(T) == 8 ? 48 * (int)ceil_div(n, 16) : (3 * n + 3) / 4 * 4;
}

template <typename T>
int pack_filters(const Geometry &g, const void *w, int mode, void **packed, size_t extra = 0, void **behind = nullptr) {
  const int M = (mode == 2 || mode == 6) ? g.F : mode == 3 ? g.C : mode == 4 ? 3 * g.C : 3 * g.F;
  const int ld = mode == 4 || mode == 5 ? folded_ld<T>(M / 3) : packed_ld(M, true);
  const size_t count = (size_t)g.F * g.C * g.wvol / M * ld;
  const size_t packed_bytes = (count * sizeof(T) + 255) & ~size_t(255);
  if (mode == 3 && g.wvol == 1 && ld == g.C && reinterpret_cast<uintptr_t>(w) % 16 == 0) {
    // one tap, input gradient: the packed layout [f][c] is w's own, nothing to do
    void *scratch = nullptr;
    if (int rc = workspace(extra, &scratch)) return rc;
    *packed = const_cast<void *>(w);
    if (behind) *behind = scratch;
    return MG_OK;
  }
  if (int rc = workspace(packed_bytes + extra, packed)) return rc;
  if (behind) *behind = static_cast<char *>(*packed) + packed_bytes;
  if (mode == 2 && g.wvol == 1 && ld == g.F) {
    // one tap, forward: a transposition of the F x C matrix
    ScopedTiming timed(TAG_PACK_FILTERS);
    hipLaunchKernelGGL(pack_transpose_kernel<T>, dim3((unsigned)ceil_div(g.C, 32), (unsigned)ceil_div(g.F, 32)), dim3(256), 0,
                       runtime().stream, static_cast<const T *>(w), static_cast<T *>(*packed), (int)g.F, (int)g.C);
    MG_HIP(hipGetLastError());
    return MG_OK;
  }
  const unsigned blocks = (unsigned)std::min<long long>(ceil_div((long long)count, 256), 4096);
  ScopedTiming timed(TAG_PACK_FILTERS);
  hipLaunchKernelGGL(pack_filters_kernel<T>, dim3(blocks), dim3(256), 0, runtime().stream, static_cast<const T *>(w),
                     static_cast<T *>(*packed), g.F, g.C, (int)g.wvol, mode, ld);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// The 4x4x1 MFMA kernel for a plan with few rows: packs the filters into its
// register-sized groups, then one position per lane.
int run_thin(const Plan &pl, ThinParams &tp, const void *w, int tag) {
  void *packed = nullptr;
  const size_t a_bytes = (size_t)pl.thin_chunks * pl.thin_kgroups * 256;  // per pass
  const int passes = (int)ceil_div(tp.M, 4 * pl.thin_rg);
  if (int rc = workspace(a_bytes * passes, &packed)) return rc;
  {
    ScopedTiming timed(TAG_PACK_FILTERS);
    if (int rc = launch_thin_pack(static_cast<const float *>(w), static_cast<float *>(packed), pl.arow, pl.thin_chunks, pl.thin_kgroups,
                                  pl.thin_w_group, pl.thin_w_mstride, tp.M, pl.thin_rg, passes, runtime().stream))
      return rc;
  }
  tp.A = static_cast<const float *>(packed);
  tp.a_bytes = (unsigned)a_bytes;
  tp.tab = pl.tab;
  tp.chunks = pl.thin_chunks;
  tp.kgroups = pl.thin_kgroups;
  // channel groups per block (measured on the stem's dx: 16 or 8 the same time, 4 slower by 4 %, 2 by 20 %)
  tp.kblock = std::min(8, pl.thin_kgroups);
  tp.group_bytes = (unsigned)(pl.thin_src_group * 4);
  tp.npos = pl.thin_grid.npos;
  tp.by_jvol = pl.thin_grid.by_jvol, tp.by_j12 = pl.thin_grid.by_j12, tp.by_j2 = pl.thin_grid.by_j2;
  tp.nph = pl.nph;
  tp.rg = pl.thin_rg;
  tp.passes = passes;
  tp.pass_floats = (long long)(a_bytes / 4);
  for (int k = 0; k < 3; ++k) tp.J[k] = pl.thin_grid.J[k];
  for (int f = 0; f < pl.nph; ++f)
    for (int k = 0; k < 3; ++k) {
      tp.po0[f][k] = pl.po0[f][k];
      tp.pJ[f][k] = pl.pJ[f][k];
    }
  // phases 2q and 2q + 1 side by side along the last axis, every pair 8-byte aligned in dst
  bool pairs = pl.nph > 1 && tp.oj[2] == 2 && tp.os[2] == 1 && tp.os[1] % 2 == 0 && tp.os[0] % 2 == 0 && tp.dst_mstride % 2 == 0 &&
               tp.dst_nstride % 2 == 0 && reinterpret_cast<uintptr_t>(tp.dst) % 8 == 0;
  for (int f = 0; pairs && f + 1 < pl.nph; f += 2)
    pairs = pl.po0[f][2] == 0 && pl.po0[f + 1][2] == 1 && pl.po0[f][0] == pl.po0[f + 1][0] && pl.po0[f][1] == pl.po0[f + 1][1] &&
            pl.pJ[f][0] == pl.pJ[f + 1][0] && pl.pJ[f][1] == pl.pJ[f + 1][1] && pl.pJ[f][2] == pl.pJ[f + 1][2];
  tp.pair_store = pairs ? 1 : 0;
  ScopedTiming timed(tag);
  return launch_thin_gemm(tp, runtime().stream);
}

template <typename T>
int conv_fwd_impl(const Geometry &g, const Plan &pl, const void *x, const void *w, void *out) {
  if (pl.thin) {
    ThinParams tp{};
    tp.src = static_cast<const float *>(x);
    tp.dst = static_cast<float *>(out);
    tp.M = g.F;
    const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
    const int os[3] = {g.G[1] * g.G[2], g.G[2], 1};
    for (int k = 0; k < 3; ++k) {
      tp.Q[k] = g.X[k];
      tp.sj[k] = g.S[k];
      tp.qs[k] = qs[k];
      tp.oj[k] = 1;
      tp.os[k] = os[k];
    }
    tp.dst_mstride = (int)g.gvol;
    tp.src_nstride = (long long)g.C * g.xvol;
    tp.dst_nstride = (long long)g.F * g.gvol;
    tp.src_bytes = (unsigned)((size_t)g.N * g.C * g.xvol * 4);
    return run_thin(pl, tp, w, TAG_CONV_FWD);
  }
  void *packed = nullptr;
  void *partial = nullptr;
  if (!pl.tap_major) {
    packed = const_cast<void *>(w);  // read in place: row k = (c, taps) of filter m lies at w[m * C*taps + k]
  } else if (int rc = pack_filters<T>(g, w, pl.table_rows ? 6 : pl.fold_row ? 5 : 2, &packed, tail_bytes(pl, sizeof(T)), &partial)) {
    return rc;
  }
  GemmParams gp{};
  gp.partial = partial;
  gp.A = packed;
  gp.a_mstride = (int)(g.C * g.wvol);
  gp.src = x;
  gp.dst = out;
  gp.M = g.F;
  const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
  const int os[3] = {g.G[1] * g.G[2], g.G[2], 1};
  for (int k = 0; k < 3; ++k) {
    gp.Q[k] = g.X[k];
    gp.sj[k] = g.S[k];
    gp.qs[k] = qs[k];
    gp.oj[k] = 1;
    gp.os[k] = os[k];
  }
  gp.dst_mstride = (int)g.gvol;
  gp.src_cstride = (int)g.xvol;
  gp.src_nstride = (long long)g.C * g.xvol;
  gp.dst_nstride = (long long)g.F * g.gvol;
  gp.a_ld = pl.fold_row ? folded_ld<T>(g.F) : packed_ld(g.F, pl.tap_major);
  gp.a_bytes = (unsigned)((size_t)g.C * (pl.fold_row ? g.wvol / 3 : g.wvol) * gp.a_ld * sizeof(T));
  gp.src_bytes = pl.tap_major ? (unsigned)((size_t)g.N * g.C * g.xvol * sizeof(T)) : 0;
  return run_gemm<T>(gp, pl, TAG_CONV_FWD, runtime().stream);
}

template <typename T>
int conv_dgrad_impl(const Geometry &g, const Plan &pl, const void *grad, const void *w, void *dx) {
  if (pl.thin) {
    ThinParams tp{};
    tp.src = static_cast<const float *>(grad);
    tp.dst = static_cast<float *>(dx);
    tp.M = g.C;
    const int qs[3] = {g.G[1] * g.G[2], g.G[2], 1};
    const int os[3] = {g.X[1] * g.X[2], g.X[2], 1};
    for (int k = 0; k < 3; ++k) {
      tp.Q[k] = g.G[k];
      tp.sj[k] = 1;
      tp.qs[k] = qs[k];
      tp.oj[k] = g.S[k];
      tp.os[k] = os[k];
    }
    tp.dst_mstride = (int)g.xvol;
    tp.src_nstride = (long long)g.F * g.gvol;
    tp.dst_nstride = (long long)g.C * g.xvol;
    tp.src_bytes = (unsigned)((size_t)g.N * g.F * g.gvol * 4);
    return run_thin(pl, tp, w, TAG_CONV_DGRAD);
  }
  void *packed = nullptr;
  void *partial = nullptr;
  if (!pl.tap_major) {
    packed = const_cast<void *>(w);  // read in place: row k = (f, tap) of channel m lies at w[(f * C + m) * taps + tap]
  } else if (pl.table_rows) {
    const int ld = packed_ld(g.C, true);
    const size_t packed_bytes = ((size_t)pl.table_count * ld * sizeof(T) + 255) & ~size_t(255);
    if (int rc = workspace(packed_bytes + tail_bytes(pl, sizeof(T)), &packed)) return rc;
    partial = static_cast<char *>(packed) + packed_bytes;
    if (pl.table_count > 0) {  // no phase may have a tap at all (an axis of one element that every window steps over): dx is zero
      ScopedTiming timed(TAG_PACK_FILTERS);
      const unsigned blocks = (unsigned)std::min<long long>(ceil_div((long long)pl.table_count * ld, 256), 4096);
      hipLaunchKernelGGL(pack_rows_kernel<T>, dim3(blocks), dim3(256), 0, runtime().stream, static_cast<const T *>(w),
                         static_cast<T *>(packed), pl.arow, pl.table_count, (int)g.C, (int)g.wvol, ld);
      MG_HIP(hipGetLastError());
    }
  } else if (pl.phase_rows) {
    const int ld = packed_ld(pl.phase_count * g.C, true);
    const size_t packed_bytes = ((size_t)pl.table_count * g.F * ld * sizeof(T) + 255) & ~size_t(255);
    if (int rc = workspace(packed_bytes + tail_bytes(pl, sizeof(T)), &packed)) return rc;
    partial = static_cast<char *>(packed) + packed_bytes;
    ScopedTiming timed(TAG_PACK_FILTERS);
    const unsigned blocks = (unsigned)std::min<long long>(ceil_div((long long)pl.table_count * g.F * ld, 256), 4096);
    hipLaunchKernelGGL(pack_phase_rows_kernel<T>, dim3(blocks), dim3(256), 0, runtime().stream, static_cast<const T *>(w),
                       static_cast<T *>(packed), pl.arow, pl.table_count, pl.phase_count, (int)g.F, (int)g.C, (int)g.wvol, ld);
    MG_HIP(hipGetLastError());
  } else if (int rc = pack_filters<T>(g, w, pl.fold_row ? 4 : 3, &packed, tail_bytes(pl, sizeof(T)), &partial)) {
    return rc;
  }
  GemmParams gp{};
  gp.partial = partial;
  gp.A = packed;
  gp.a_mstride = (int)g.wvol;
  gp.src = grad;
  gp.dst = dx;
  gp.M = pl.phase_rows ? pl.phase_count * g.C : g.C;
  const int qs[3] = {g.G[1] * g.G[2], g.G[2], 1};
  const int os[3] = {g.X[1] * g.X[2], g.X[2], 1};
  for (int k = 0; k < 3; ++k) {
    gp.Q[k] = g.G[k];
    gp.sj[k] = 1;
    gp.qs[k] = qs[k];
    gp.oj[k] = g.S[k];
    gp.os[k] = os[k];
  }
  gp.dst_mstride = (int)g.xvol;
  gp.src_cstride = (int)g.gvol;
  gp.src_nstride = (long long)g.F * g.gvol;
  gp.dst_nstride = (long long)g.C * g.xvol;
  gp.a_ld = pl.fold_row ? folded_ld<T>(g.C) : packed_ld(g.C, pl.tap_major);
  gp.a_bytes = pl.table_rows ? (unsigned)((size_t)pl.table_count * gp.a_ld * sizeof(T))
                             : (unsigned)((size_t)g.F * (pl.fold_row ? g.wvol / 3 : g.wvol) * gp.a_ld * sizeof(T));
  if (pl.phase_rows) {
    gp.a_ld = packed_ld(pl.phase_count * g.C, true);
    gp.a_bytes = (unsigned)((size_t)pl.table_count * g.F * gp.a_ld * sizeof(T));
  }
  gp.src_bytes = pl.tap_major ? (unsigned)((size_t)g.N * g.F * g.gvol * sizeof(T)) : 0;
  return run_gemm<T>(gp, pl, TAG_CONV_DGRAD, runtime().stream);
}

template <typename T, int BM, int BN, int BK, int WM, int WN>
void launch_table_wgrad(WgradParams &wp, hipStream_t s) {
  wp.col_tiles = (int)ceil_div(wp.CT, BN);
  wp.row_tiles = (int)ceil_div(wp.F, BM);
  const long long blocks = (long long)wp.splits * wp.col_tiles * wp.row_tiles;
  const bool wide = wp.gvol % (int)(16 / sizeof(T)) == 0;
  if (wp.pos_tab != nullptr) {
    if (wide)
      hipLaunchKernelGGL((tap_wgrad_kernel<T, BM, BN, BK, WM, WN, true, true, true>), dim3((unsigned)blocks), dim3(512), 0, s, wp);
    else
      hipLaunchKernelGGL((tap_wgrad_kernel<T, BM, BN, BK, WM, WN, false, true, true>), dim3((unsigned)blocks), dim3(512), 0, s, wp);
  } else if (wide) {
    hipLaunchKernelGGL((tap_wgrad_kernel<T, BM, BN, BK, WM, WN, true, true>), dim3((unsigned)blocks), dim3(512), 0, s, wp);
  } else {
    hipLaunchKernelGGL((tap_wgrad_kernel<T, BM, BN, BK, WM, WN, false, true>), dim3((unsigned)blocks), dim3(512), 0, s, wp);
  }
}

template <typename T, int BM, int BN, int BK, int WM, int WN>
void launch_wgrad(WgradParams &wp, bool tap_major, bool table_rows, hipStream_t s) {
  wp.col_tiles = (int)ceil_div(wp.CT, BN);
  wp.row_tiles = (int)ceil_div(wp.F, BM);
  if (table_rows) {
    if constexpr (BN == 64) launch_table_wgrad<T, BM, BN, BK, WM, WN>(wp, s);
  } else if (tap_major) {
    // one-dimensional grid, runs of (split, tile) pairs per XCD (see the kernel)
    const long long blocks = (long long)wp.splits * wp.col_tiles * wp.row_tiles;
    if (wp.gvol % (int)(16 / sizeof(T)) == 0)
      hipLaunchKernelGGL((tap_wgrad_kernel<T, BM, BN, BK, WM, WN, true>), dim3((unsigned)blocks), dim3(512), 0, s, wp);
    else
      hipLaunchKernelGGL((tap_wgrad_kernel<T, BM, BN, BK, WM, WN, false>), dim3((unsigned)blocks), dim3(512), 0, s, wp);
  } else if constexpr (BN == 64) {
    const dim3 grid((unsigned)wp.col_tiles, (unsigned)wp.row_tiles, (unsigned)wp.splits);
    hipLaunchKernelGGL((wgrad_kernel<T, BM, BN, BK, WM, WN>), grid, dim3(256), 0, s, wp);
  }
}

template <typename T>
int conv_wgrad_impl(const Geometry &g, const Plan &pl, const void *grad, const void *x, void *dw) {
  hipStream_t s = runtime().stream;
  const int ct = (int)(g.C * g.wvol);
  // The tap-major kernel writes its columns in (tap, channel) order, so its result goes
  // through the reduction kernel, which also restores (channel, tap) -- unless there is a
  // single tap (a matrix product), where the two orders are the same, and a single split.
  const bool staged = pl.splits > 1 || (pl.tap_major && !pl.table_rows && g.wvol > 1);
  void *target = dw;
  if (staged)
    if (int rc = workspace((size_t)pl.splits * g.F * ct * sizeof(T), &target)) return rc;
  WgradParams wp{};
  wp.grad = grad;
  wp.x = x;
  wp.out = target;
  wp.tab = pl.tab;
  wp.groups = pl.groups;
  wp.zeros = pl.zeros;
  wp.F = g.F;
  wp.CT = ct;
  const int qs[3] = {g.X[1] * g.X[2], g.X[2], 1};
  for (int k = 0; k < 3; ++k) {
    wp.G[k] = g.G[k];
    wp.Q[k] = g.X[k];
    wp.sj[k] = g.S[k];
    wp.qs[k] = qs[k];
  }
  wp.gvol = (int)g.gvol;
  wp.x_cstride = (int)g.xvol;
  wp.grad_bytes = pl.tap_major ? (unsigned)((size_t)g.N * g.F * g.gvol * sizeof(T)) : 0;
  wp.x_bytes = pl.tap_major ? (unsigned)((size_t)g.N * g.C * g.xvol * sizeof(T)) : 0;
  wp.x_nstride = (long long)g.C * g.xvol;
  wp.g_nstride = (long long)g.F * g.gvol;
  wp.kpos = (int)((long long)g.N * g.gvol);
  wp.kchunk = pl.kchunk;
  wp.splits = pl.splits;
  wp.by_gvol = make_fastdiv((unsigned)g.gvol);
  wp.by_g12 = make_fastdiv((unsigned)(g.G[1] * g.G[2]));
  wp.by_g2 = make_fastdiv((unsigned)g.G[2]);
  wp.pos_tab = pl.pos_tab;
  wp.wvol = (int)g.wvol;
  {
    ScopedTiming timed(TAG_CONV_WGRAD);
    bool launched = false;
    if (pl.table_rows) {
#define MG_LAUNCH_TABLE(TT, BM, BN, BK, WM, WN)             \
  if (!launched && pl.bm == BM && pl.bn == BN) {            \
    launch_table_wgrad<TT, BM, BN, BK, WM, WN>(wp, s);      \
    launched = true;                                        \
  }
      MG_WGRAD_TABLE_SHAPES(T, MG_LAUNCH_TABLE)
#undef MG_LAUNCH_TABLE
    }
#define MG_LAUNCH(TT, BM, BN, BK, WM, WN)                               \
  if (!launched && pl.bm == BM && pl.bn == BN) {                        \
    launch_wgrad<TT, BM, BN, BK, WM, WN>(wp, pl.tap_major, pl.table_rows, s);        \
    launched = true;                                                    \
  }
    MG_WGRAD_SHAPES(T, MG_LAUNCH)
#undef MG_LAUNCH
    if (!launched) return fail(MG_ERR_UNSUPPORTED, "no filter-gradient kernel for tile %d x %d", pl.bm, pl.bn);
  }
  MG_HIP(hipGetLastError());
  if (staged) {
    const int count = g.F * ct;
    ScopedTiming timed(TAG_WGRAD_REDUCE);
    if (pl.tap_major && !pl.table_rows) {
      // four runs of splits per element when one thread per element would leave units idle
      if (ceil_div(count, 256) < runtime().props.multiProcessorCount && pl.splits >= 16)
        hipLaunchKernelGGL((tap_reduce_kernel<T, 4>), dim3((unsigned)ceil_div(count, 64)), dim3(256), 0, s,
                           static_cast<const T *>(target), static_cast<T *>(dw), g.F, g.C, (int)g.wvol, pl.splits);
      else
        hipLaunchKernelGGL((tap_reduce_kernel<T, 1>), dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, s,
                           static_cast<const T *>(target), static_cast<T *>(dw), g.F, g.C, (int)g.wvol, pl.splits);
    } else {
      if (ceil_div(count, 256) < runtime().props.multiProcessorCount / 8 && pl.splits >= 64)
        hipLaunchKernelGGL((splitk_reduce_kernel<T, 16>), dim3((unsigned)ceil_div(count, 16)), dim3(256), 0, s,
                           static_cast<const T *>(target), static_cast<T *>(dw), count, pl.splits);
      else
        hipLaunchKernelGGL((splitk_reduce_kernel<T, 1>), dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, s,
                           static_cast<const T *>(target), static_cast<T *>(dw), count, pl.splits);
    }
    MG_HIP(hipGetLastError());
  }
  return MG_OK;
}

}  // namespace

void release_conv_plans() {
  note_plan("");  // it may point into a plan
  for (auto &kv : plans()) {
    if (kv.second.blob) (void)hipFree(kv.second.blob);
    if (kv.second.pos_tab) (void)hipFree(kv.second.pos_tab);
  }
  plans().clear();
}

}  // namespace mg

using namespace mg;

// The fast (tap-major) kernels need the reduction -- K for the product and for da, M for dx --
// and da's row count M to be multiples of 16.  A large product whose extents are not is run on
// zero-padded copies of its operands (two bandwidth-bound passes over the operands against a
// matrix product that runs more than twice as fast); small ones take the table-driven kernels.
namespace {
constexpr int64_t kMatmulUnit = 16;
inline int64_t padded(int64_t n) { return (n + kMatmulUnit - 1) / kMatmulUnit * kMatmulUnit; }
// MYGRAD_HIP_PAD=0 leaves every operand as it is (the table-driven kernels then take the
// awkward extents): for comparisons
inline bool padding_allowed() {
  static const bool on = [] {
    const char *flag = getenv("MYGRAD_HIP_PAD");
    return !(flag && flag[0] == '0');
  }();
  return on;
}
inline bool worth_padding(int64_t batch, int64_t M, int64_t K, int64_t N) {
  return padding_allowed() && 2.0 * (double)batch * (double)M * (double)K * (double)N >= 2.0e8;
}

// dst:(batch, drows, dcols) takes src:(batch, srows, scols) where both have an element, zero elsewhere
template <typename T>
__global__ void __launch_bounds__(256) pad2d_kernel(const T *__restrict__ src, T *__restrict__ dst, long long total, int srows,
                                                    int scols, int drows, int dcols) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const long long plane = (long long)drows * dcols;
  const long long b = idx / plane;
  const int rem = (int)(idx - b * plane);
  const int r = rem / dcols, c = rem - r * dcols;
  dst[idx] = (r < srows && c < scols) ? src[(b * srows + r) * scols + c] : T(0);
}

// src:(batch, srows, scols) re-laid as (batch, drows, dcols) into dst
int relay_into(int dtype, const void *src, int64_t batch, int64_t srows, int64_t scols, int64_t drows, int64_t dcols, void *dst) {
  void *where = dst;
  void **block = &where;
  const long long total = batch * drows * dcols;
  if (srows >= (1ll << 31) || scols >= (1ll << 31) || drows * dcols >= (1ll << 31) || ceil_div(total, 256) >= (1ll << 31))
    return fail(MG_ERR_UNSUPPORTED, "matrix product: an extent of 2^31 or more");
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  const dim3 grid((unsigned)ceil_div(total, 256)), blk(256);
  ScopedTiming timed(TAG_COPY);
  if (dtype == MG_F32)
    hipLaunchKernelGGL(pad2d_kernel<float>, grid, blk, 0, runtime().stream, (const float *)src, (float *)*block, total, (int)srows,
                       (int)scols, (int)drows, (int)dcols);
  else
    hipLaunchKernelGGL(pad2d_kernel<double>, grid, blk, 0, runtime().stream, (const double *)src, (double *)*block, total, (int)srows,
                       (int)scols, (int)drows, (int)dcols);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// a pooled block holding src:(batch, srows, scols) re-laid as (batch, drows, dcols)
int relaid(int dtype, const void *src, int64_t batch, int64_t srows, int64_t scols, int64_t drows, int64_t dcols, void **block) {
  if (int rc = mg_malloc(block, (size_t)(batch * drows * dcols) * (dtype == MG_F32 ? 4 : 8))) return rc;
  return relay_into(dtype, src, batch, srows, scols, drows, dcols, *block);
}

// Channel (or filter) count to zero-pad `channels` to so that the tap-major kernels apply, or 0
// to leave it: already a multiple of 16, too small a problem to repay two extra passes over
// the operands, or more than a third of padding.
inline double conv_flops(const Geometry &g) {
  return 2.0 * (double)g.N * (double)g.F * (double)g.gvol * (double)g.C * (double)g.wvol;
}
inline int64_t channels_to_pad_to(int64_t channels, double flops) {
  if (channels % kMatmulUnit == 0 || flops < 2.0e8 || !padding_allowed()) return 0;
  const int64_t up = padded(channels);
  return 3 * up <= 4 * channels ? up : 0;
}

// frees pooled blocks when the call that used them returns (the pool keeps them in stream order)
struct Blocks {
  void *held[4] = {nullptr, nullptr, nullptr, nullptr};
  ~Blocks() {
    for (void *p : held)
      if (p) (void)mg_free(p);
  }
};
}  // namespace


extern "C" {

int mg_conv_fwd(const mg_conv_desc *desc, const void *x, const void *w, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  Geometry g;
  if (int rc = check_desc(desc, &g)) return rc;
  if (!x || !w || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_conv_fwd");
  if (const int64_t Cp = channels_to_pad_to(g.C, conv_flops(g))) {
    // zero channels added to x and to the filters: the same sums, on the tap-major kernels
    Blocks tmp;
    if (int rc = relaid(g.dtype, x, g.N, g.C, g.xvol, Cp, g.xvol, &tmp.held[0])) return rc;
    if (int rc = relaid(g.dtype, w, g.F, g.C, g.wvol, Cp, g.wvol, &tmp.held[1])) return rc;
    mg_conv_desc wider = *desc;
    wider.C = Cp;
    return mg_conv_fwd(&wider, tmp.held[0], tmp.held[1], out);
  }
  Plan *pl = nullptr;
  if (int rc = get_plan(OP_FWD, desc, g, &pl)) return rc;
  return g.dtype == MG_F32 ? conv_fwd_impl<float>(g, *pl, x, w, out) : conv_fwd_impl<double>(g, *pl, x, w, out);
}

int mg_conv_dgrad(const mg_conv_desc *desc, const void *grad, const void *w, void *dx) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  Geometry g;
  if (int rc = check_desc(desc, &g)) return rc;
  if (!grad || !w || !dx) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_conv_dgrad");
  if (const int64_t Fp = channels_to_pad_to(g.F, conv_flops(g))) {
    // zero filters added to grad and to the filter bank
    Blocks tmp;
    if (int rc = relaid(g.dtype, grad, g.N, g.F, g.gvol, Fp, g.gvol, &tmp.held[0])) return rc;
    if (int rc = relaid(g.dtype, w, 1, g.F, (int64_t)g.C * g.wvol, Fp, (int64_t)g.C * g.wvol, &tmp.held[1])) return rc;
    mg_conv_desc wider = *desc;
    wider.F = Fp;
    return mg_conv_dgrad(&wider, tmp.held[0], tmp.held[1], dx);
  }
  Plan *pl = nullptr;
  if (int rc = get_plan(OP_DGRAD, desc, g, &pl)) return rc;
  return g.dtype == MG_F32 ? conv_dgrad_impl<float>(g, *pl, grad, w, dx)
                           : conv_dgrad_impl<double>(g, *pl, grad, w, dx);
}

int mg_conv_wgrad(const mg_conv_desc *desc, const void *grad, const void *x, void *dw) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  Geometry g;
  if (int rc = check_desc(desc, &g)) return rc;
  if (!grad || !x || !dw) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_conv_wgrad");
  {
    const int64_t Cp = channels_to_pad_to(g.C, conv_flops(g)), Fp = channels_to_pad_to(g.F, conv_flops(g));
    if (Cp || Fp) {
      // zero channels / filters added to x / grad; the rows and columns of dw that exist are kept
      const int64_t C2 = Cp ? Cp : g.C, F2 = Fp ? Fp : g.F;
      Blocks tmp;
      const void *x2 = x, *g2 = grad;
      if (Cp) {
        if (int rc = relaid(g.dtype, x, g.N, g.C, g.xvol, Cp, g.xvol, &tmp.held[0])) return rc;
        x2 = tmp.held[0];
      }
      if (Fp) {
        if (int rc = relaid(g.dtype, grad, g.N, g.F, g.gvol, Fp, g.gvol, &tmp.held[1])) return rc;
        g2 = tmp.held[1];
      }
      if (int rc = mg_malloc(&tmp.held[2], (size_t)(F2 * C2 * g.wvol) * (g.dtype == MG_F32 ? 4 : 8))) return rc;
      mg_conv_desc wider = *desc;
      wider.C = C2;
      wider.F = F2;
      if (int rc = mg_conv_wgrad(&wider, g2, x2, tmp.held[2])) return rc;
      return relay_into(g.dtype, tmp.held[2], g.F, C2, g.wvol, g.C, g.wvol, dw);
    }
  }
  Plan *pl = nullptr;
  if (int rc = get_plan(OP_WGRAD, desc, g, &pl)) return rc;
  return g.dtype == MG_F32 ? conv_wgrad_impl<float>(g, *pl, grad, x, dw)
                           : conv_wgrad_impl<double>(g, *pl, grad, x, dw);
}

// ---- matrix product: a convolution with a window of one element -------------------------
//
// out[b] = a @ x[b] with a:(M, K) shared by the batch and x:(batch, K, N) is the convolution of
// x (batch entries, K channels, N positions) with M filters of one tap: the same implicit-GEMM
// kernels with a reduction of length K.  Its two gradients are the convolution's.
namespace {
int matmul_desc(const char *who, int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, mg_conv_desc *d) {
  if (batch < 1 || M < 1 || K < 1 || N < 1)
    return fail(MG_ERR_BAD_ARG, "%s: batch=%lld M=%lld K=%lld N=%lld must be positive", who, (long long)batch, (long long)M,
                (long long)K, (long long)N);
  *d = mg_conv_desc{};
  d->dtype = dtype;
  d->nd = 1;
  d->N = batch;
  d->C = K;
  d->F = M;
  for (int k = 0; k < MG_MAX_ND; ++k) d->X[k] = d->W[k] = d->G[k] = d->stride[k] = d->dil[k] = 1;
  d->X[MG_MAX_ND - 1] = d->G[MG_MAX_ND - 1] = N;
  return MG_OK;
}
}  // namespace

int mg_matmul(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, const void *a, const void *x, void *out) {
  mg_conv_desc d;
  if (int rc = matmul_desc("mg_matmul", dtype, batch, M, K, N, &d)) return rc;
  if (K % kMatmulUnit != 0 && (dtype == MG_F32 || dtype == MG_F64) && a && x && out && worth_padding(batch, M, K, N)) {
    const int64_t Kp = padded(K);
    Blocks tmp;
    if (int rc = relaid(dtype, a, 1, M, K, M, Kp, &tmp.held[0])) return rc;          // zero columns
    if (int rc = relaid(dtype, x, batch, K, N, Kp, N, &tmp.held[1])) return rc;      // zero rows
    if (int rc = matmul_desc("mg_matmul", dtype, batch, M, Kp, N, &d)) return rc;
    return mg_conv_fwd(&d, tmp.held[1], tmp.held[0], out);
  }
  return mg_conv_fwd(&d, x, a, out);
}

int mg_matmul_da(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, const void *grad, const void *x, void *da) {
  mg_conv_desc d;
  if (int rc = matmul_desc("mg_matmul_da", dtype, batch, M, K, N, &d)) return rc;
  // da's rows are the filter-gradient kernel's tile rows, which must divide M: a large M is padded
  // to whole 128-row (64-row) tiles rather than left to the 16- or 32-row ones
  const int64_t row_unit = M >= 1024 ? 128 : (M >= 256 ? 64 : kMatmulUnit);
  const int64_t Mp = (M + row_unit - 1) / row_unit * row_unit;
  if ((K % kMatmulUnit != 0 || Mp != M) && (dtype == MG_F32 || dtype == MG_F64) && grad && x && da &&
      worth_padding(batch, M, K, N)) {
    const int64_t Kp = padded(K);
    Blocks tmp;
    const void *g2 = grad, *x2 = x;
    if (Mp != M) {
      if (int rc = relaid(dtype, grad, batch, M, N, Mp, N, &tmp.held[0])) return rc;
      g2 = tmp.held[0];
    }
    if (Kp != K) {
      if (int rc = relaid(dtype, x, batch, K, N, Kp, N, &tmp.held[1])) return rc;
      x2 = tmp.held[1];
    }
    if (int rc = mg_malloc(&tmp.held[2], (size_t)Mp * Kp * (dtype == MG_F32 ? 4 : 8))) return rc;
    if (int rc = matmul_desc("mg_matmul_da", dtype, batch, Mp, Kp, N, &d)) return rc;
    if (int rc = mg_conv_wgrad(&d, g2, x2, tmp.held[2])) return rc;
    // the rows and columns that belong to da
    return relay_into(dtype, tmp.held[2], 1, Mp, Kp, M, K, da);
  }
  return mg_conv_wgrad(&d, grad, x, da);
}

int mg_matmul_dx(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, const void *grad, const void *a, void *dx) {
  mg_conv_desc d;
  if (int rc = matmul_desc("mg_matmul_dx", dtype, batch, M, K, N, &d)) return rc;
  if (M % kMatmulUnit != 0 && (dtype == MG_F32 || dtype == MG_F64) && grad && a && dx && worth_padding(batch, M, K, N)) {
    const int64_t Mp = padded(M);
    Blocks tmp;
    if (int rc = relaid(dtype, a, 1, M, K, Mp, K, &tmp.held[0])) return rc;          // zero rows
    if (int rc = relaid(dtype, grad, batch, M, N, Mp, N, &tmp.held[1])) return rc;   // zero rows
    if (int rc = matmul_desc("mg_matmul_dx", dtype, batch, Mp, K, N, &d)) return rc;
    return mg_conv_dgrad(&d, tmp.held[1], tmp.held[0], dx);
  }
  return mg_conv_dgrad(&d, grad, a, dx);
}

}  // extern "C"
