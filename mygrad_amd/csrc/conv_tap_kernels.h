// Tap-major implicit-GEMM kernels: the fast path of conv.hip.
//
// The contraction index of the forward / data-gradient GEMM is ordered
// (tap, channel) with the channel innermost, and a K tile is BK consecutive
// channels under ONE tap.  For a fixed output position all BK gathered elements
// of a tile then share the tap's padding test and differ by a constant address
// step (the channel stride), so a thread spends one validity test and one
// pointer select per tile and one add per load, instead of a table row, three
// compares and two selects per element.  Padding loads are pointed at a block
// of zeros in device memory, so no select follows the load either.  The filter
// gradient orders its columns by channel block of 16, then tap, then channel.
//
// Needs the channel count (filter count for dgrad) to be a multiple of BK; other
// shapes take the table-driven kernels.
#pragma once

namespace mg {

typedef int int8v __attribute__((ext_vector_type(8)));
static_assert(sizeof(KTile) == sizeof(int8v) && sizeof(WGroup) == sizeof(int8v), "32-byte table rows");

template <typename T, int N>
struct VecOf {
  typedef T type __attribute__((ext_vector_type(N)));
};

// N consecutive elements from LDS / to global memory as one vector access
// (the address must be aligned to N * sizeof(T), at most 16 bytes at a time).
template <typename T, int N>
__device__ __forceinline__ void load_vec(const T *src, T (&dst)[N]) {
  if constexpr (N == 1) {
    dst[0] = src[0];
  } else {
    const typename VecOf<T, N>::type v = *reinterpret_cast<const typename VecOf<T, N>::type *>(src);
#pragma unroll
    for (int i = 0; i < N; ++i) dst[i] = v[i];
  }
}

template <typename T, int N>
__device__ __forceinline__ void store_vec(T *dst, const T (&src)[N]) {
  if constexpr (N == 1) {
    dst[0] = src[0];
  } else {
    typename VecOf<T, N>::type v;
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = src[i];
    *reinterpret_cast<typename VecOf<T, N>::type *>(dst) = v;
  }
}

// ------------------------------------------------------------------------------------------
// forward and data gradient
// ------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int BK, int WM, int WN>
__global__ void __launch_bounds__(512) tap_gemm_kernel(const GemmParams p) {
  static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per block");
  static_assert(BK % 4 == 0 && WM % 16 == 0 && WN % 16 == 0 && BN % 64 == 0, "MFMA 16x16x4 tiling");
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int WAVES_N = BN / WN;
  constexpr int AROWS = 256 / BM;
  constexpr int ALOADS = (BK + AROWS - 1) / AROWS;
  constexpr int BROWS = 256 / BN;
  constexpr int BLOADS = BK / BROWS;
  constexpr int PAD = 16 / sizeof(T);  // rows stay 16-byte aligned for the vector reads
  constexpr int LDA = BM + PAD, LDB = BN + PAD;

  __shared__ __attribute__((aligned(16))) T As[2][BK][LDA];
  __shared__ __attribute__((aligned(16))) T Bs[2][BK][LDB];

  // Eight wavefronts with two roles.  Waves 0-3 only read LDS and issue MFMAs; waves
  // 4-7 only gather: global loads -> registers -> LDS, one tile ahead.  One of each
  // sits on every SIMD, so the gather's address arithmetic, memory instructions and
  // LDS stores are issued in the shadow of the other wave's MFMAs instead of taking
  // turns with them in one instruction stream.
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const bool loader = wave >= 4;
  const int tid = threadIdx.x & 255;  // index inside the role
  const int wm0 = ((wave & 3) / WAVES_N) * WM;
  const int wn0 = ((wave & 3) % WAVES_N) * WN;
  const int l16 = lane & 15, lk = lane >> 4;

  // Tiles are numbered with the row tile (m) innermost, so that the row tiles of one
  // position block, which gather the same elements, run next to each other.  The
  // first p.full_tiles blocks compute one whole tile each.  The tiles that remain
  // would fill only part of the device in a last round, so each of them is shared
  // by p.tail_split blocks, each taking a slice of the K loop and leaving its partial
  // sums in a workspace for tail_fixup_kernel.
  const int bid = blockIdx.x;
  int tile = bid, piece = 0;
  const bool partial = bid >= p.full_tiles;
  if (partial) {
    const int j = bid - p.full_tiles;
    tile = p.full_tiles + j / p.tail_split;
    piece = j % p.tail_split;
  }
  const int pblk = tile / p.m_tiles;
  int pi = 0;
  while (pi + 1 < p.nphases && pblk >= p.phases[pi + 1].blk_begin) ++pi;
  const Phase ph = p.phases[pi];
  const int pos0 = (pblk - ph.blk_begin) * BN;
  const int m0 = (tile % p.m_tiles) * BM;
  const int j12 = ph.J[1] * ph.J[2];
  const int jvol = ph.J[0] * j12;

  const T *__restrict__ A = static_cast<const T *>(p.A);
  const T *__restrict__ zeros = static_cast<const T *>(p.zeros);
  const int8v MG_CONSTANT *ktab = (const int8v MG_CONSTANT *)(p.ktiles + ph.k_begin);

  // ---- this thread's column of the B tile: one output position
  const int bcol = tid % BN;
  const int brow0 = uniform(tid / BN);
  int qb0, qb1, qb2;
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
    srcn += (long long)n * p.src_nstride + (qb0 * p.qs[0] + qb1 * p.qs[1] + qb2 * p.qs[2]) + brow0 * p.src_cstride;
  }
  // ---- this thread's column of the A tile: one row m of the packed filters
  const int acol = tid % BM;
  const int arow0 = BM % 64 == 0 ? uniform(tid / BM) : tid / BM;
  const bool a_ok = (m0 + acol < p.M) & (arow0 < BK);
  const T *__restrict__ an = A + ((long long)arow0 * p.M + m0 + acol);
  const long long astep = a_ok ? (long long)AROWS * p.M : 0;

  // two register sets: a tile is requested two iterations before it is parked in LDS
  T ra0[ALOADS], rb0[BLOADS], ra1[ALOADS], rb1[BLOADS];

  auto fetch = [&](T(&ra)[ALOADS], T(&rb)[BLOADS], int kt) {
    const int8v e = ktab[kt];  // a_row0, coff, d0, d1, d2
    const T *ap = a_ok ? an + (long long)e[0] * p.M : zeros;
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) ra[r] = ap[r * astep];
    const bool ok = pos_ok & ((unsigned)(qb0 + e[2]) < (unsigned)p.Q[0]) & ((unsigned)(qb1 + e[3]) < (unsigned)p.Q[1]) &
                    ((unsigned)(qb2 + e[4]) < (unsigned)p.Q[2]);
    const T *bp = ok ? srcn + e[1] : zeros;
    const long long bstep = ok ? (long long)(BROWS * p.src_cstride) : 0;
#pragma unroll
    for (int r = 0; r < BLOADS; ++r) rb[r] = bp[r * bstep];
  };
  auto stash = [&](const T(&ra)[ALOADS], const T(&rb)[BLOADS], int buf) {
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) {
      const int kk = arow0 + r * AROWS;
      if (kk < BK) As[buf][kk][acol] = ra[r];
    }
#pragma unroll
    for (int r = 0; r < BLOADS; ++r) Bs[buf][brow0 + r * BROWS][bcol] = rb[r];
  };

  // Lane (l16, lk) feeds row/column l16 of every 16x16 tile.  Tile i of the wave
  // takes the rows m = wm0 + l16*TM + i (and tile j the positions wn0 + l16*TN + j),
  // so the TM (TN) operands of a lane are adjacent in LDS and come in one read.
  int kt_begin = 0, kt_end = ph.k_count;
  if (partial) {
    const int per = (ph.k_count + p.tail_split - 1) / p.tail_split;
    kt_begin = min(piece * per, ph.k_count);
    kt_end = min(kt_begin + per, ph.k_count);
  }
  // The two roles run separate loops (their registers never coexist) that meet at
  // the same barriers: one after the first tile is in LDS, one per K tile.
  if (loader) {
    // tile kt_begin + i travels in register set i % 2
    if (kt_begin < kt_end) {
      fetch(ra0, rb0, kt_begin);
      stash(ra0, rb0, 0);
      if (kt_begin + 1 < kt_end) fetch(ra1, rb1, kt_begin + 1);
      if (kt_begin + 2 < kt_end) fetch(ra0, rb0, kt_begin + 2);
    }
    __syncthreads();
    // each half of the loop body parks tile kt+1 (requested two iterations ago) in
    // the idle buffer and requests tile kt+3 into the registers that just emptied
    for (int kt = kt_begin; kt < kt_end; kt += 2) {
      if (kt + 1 < kt_end) {
        stash(ra1, rb1, 1);
        if (kt + 3 < kt_end) fetch(ra1, rb1, kt + 3);
      }
      __syncthreads();
      if (kt + 1 < kt_end) {
        if (kt + 2 < kt_end) {
          stash(ra0, rb0, 0);
          if (kt + 4 < kt_end) fetch(ra0, rb0, kt + 4);
        }
        __syncthreads();
      }
    }
    return;
  }

  typename Mma<T>::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = typename Mma<T>::Acc{0, 0, 0, 0};
  __syncthreads();
  {
    int buf = 0;
    for (int kt = kt_begin; kt < kt_end; ++kt) {
#pragma unroll
      for (int k4 = 0; k4 < BK / 4; ++k4) {
        T a[TM], b[TN];
        load_vec<T, TM>(&As[buf][k4 * 4 + lk][wm0 + l16 * TM], a);
        load_vec<T, TN>(&Bs[buf][k4 * 4 + lk][wn0 + l16 * TN], b);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = Mma<T>::run(a[i], b[j], acc[i][j]);
      }
      __syncthreads();
      buf ^= 1;
    }
  }

  // ---- epilogue
  if (partial) {
    // raw tile [BM][BN] of this slice, lane's TN positions stored as one vector
    T *slot = static_cast<T *>(p.partial) +
              ((long long)(tile - p.full_tiles) * p.tail_split + piece) * (BM * BN) + (wn0 + l16 * TN);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int ml = wm0 + Mma<T>::row_of(lane, q) * TM + i;
        T v[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) v[j] = acc[i][j][q];
        if constexpr (sizeof(T) * TN <= 16) {
          store_vec<T, TN>(slot + ml * BN, v);
        } else {
          T lo[TN / 2], hi[TN / 2];
#pragma unroll
          for (int j = 0; j < TN / 2; ++j) {
            lo[j] = v[j];
            hi[j] = v[TN / 2 + j];
          }
          store_vec<T, TN / 2>(slot + ml * BN, lo);
          store_vec<T, TN / 2>(slot + ml * BN + TN / 2, hi);
        }
      }
    return;
  }
  T *__restrict__ dst = static_cast<T *>(p.dst);
  auto dst_of = [&](int ipos) -> T * {
    const unsigned pos = (unsigned)ipos;
    const unsigned n = ph.by_jvol.div(pos);
    unsigned r = pos - n * (unsigned)jvol;
    const int j0 = (int)ph.by_j12.div(r);
    r -= (unsigned)j0 * (unsigned)j12;
    const int j1 = (int)ph.by_j2.div(r);
    const int j2 = (int)r - j1 * ph.J[2];
    return dst + (long long)n * p.dst_nstride + (long long)(ph.o0[0] + j0 * p.oj[0]) * p.os[0] +
           (long long)(ph.o0[1] + j1 * p.oj[1]) * p.os[1] + (long long)(ph.o0[2] + j2 * p.oj[2]) * p.os[2];
  };
  const int first = pos0 + wn0 + l16 * TN;
  if (p.vec_store) {
    // the TN positions of this lane are adjacent in dst and all exist (npos % TN == 0)
    if (first < ph.npos) {
      T *out = dst_of(first);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = m0 + wm0 + Mma<T>::row_of(lane, q) * TM + i;
          if (m < p.M) {
            T v[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] = acc[i][j][q];
            if constexpr (sizeof(T) * TN <= 16) {
              store_vec<T, TN>(out + (long long)m * p.dst_mstride, v);
            } else {
              T lo[TN / 2], hi[TN / 2];
#pragma unroll
              for (int j = 0; j < TN / 2; ++j) {
                lo[j] = v[j];
                hi[j] = v[TN / 2 + j];
              }
              store_vec<T, TN / 2>(out + (long long)m * p.dst_mstride, lo);
              store_vec<T, TN / 2>(out + (long long)m * p.dst_mstride + TN / 2, hi);
            }
          }
        }
    }
  } else {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if (first + j >= ph.npos) continue;
      T *out = dst_of(first + j);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = m0 + wm0 + Mma<T>::row_of(lane, q) * TM + i;
          if (m < p.M) out[(long long)m * p.dst_mstride] = acc[i][j][q];
        }
    }
  }
}

// Adds the K slices of the shared tail tiles in slice order (always the same order,
// so results repeat exactly) and stores them where the tile's epilogue would have.
// One thread per tile element; blockIdx.y is the tail tile.
template <typename T, int BM, int BN>
__global__ void __launch_bounds__(256) tail_fixup_kernel(const GemmParams p) {
  const int e = blockIdx.x * 256 + threadIdx.x;  // element of the [BM][BN] tile
  if (e >= BM * BN) return;
  const int tile = p.full_tiles + blockIdx.y;
  const int pblk = tile / p.m_tiles;
  int pi = 0;
  while (pi + 1 < p.nphases && pblk >= p.phases[pi + 1].blk_begin) ++pi;
  const Phase ph = p.phases[pi];
  const int ipos = (pblk - ph.blk_begin) * BN + e % BN;
  const int m = (tile % p.m_tiles) * BM + e / BN;
  if (ipos >= ph.npos || m >= p.M) return;
  const T *slot = static_cast<const T *>(p.partial) + (long long)blockIdx.y * p.tail_split * (BM * BN) + e;
  const T sum = sum_in_order(slot, (long long)BM * BN, p.tail_split);
  const int j12 = ph.J[1] * ph.J[2];
  const unsigned pos = (unsigned)ipos;
  const unsigned n = ph.by_jvol.div(pos);
  unsigned r = pos - n * (unsigned)(ph.J[0] * j12);
  const int j0 = (int)ph.by_j12.div(r);
  r -= (unsigned)j0 * (unsigned)j12;
  const int j1 = (int)ph.by_j2.div(r);
  const int j2 = (int)r - j1 * ph.J[2];
  T *out = static_cast<T *>(p.dst) + (long long)n * p.dst_nstride + (long long)(ph.o0[0] + j0 * p.oj[0]) * p.os[0] +
           (long long)(ph.o0[1] + j1 * p.oj[1]) * p.os[1] + (long long)(ph.o0[2] + j2 * p.oj[2]) * p.os[2];
  out[(long long)m * p.dst_mstride] = sum;
}

// ------------------------------------------------------------------------------------------
// filter gradient
// ------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int BK, int WM, int WN>
__global__ void __launch_bounds__(512) tap_wgrad_kernel(const WgradParams p) {
  static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per block");
  static_assert(256 % BK == 0 && BK % 16 == 0 && BN % 16 == 0, "K tile");
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int WAVES_N = BN / WN;
  constexpr int ROWS = 256 / BK;  // tile rows covered by one pass of the block
  static_assert(16 % ROWS == 0 && BM % ROWS == 0, "row passes must not straddle a column group");
  constexpr int ALOADS = BM / ROWS;
  constexpr int NGROUPS = BN / 16;
  constexpr int GLOADS = 16 / ROWS;  // loads per thread per column group
  constexpr int LDK = BK + 16 / sizeof(T);
  constexpr int KQ = BK / 4;  // K indices owned by one quarter-wave

  __shared__ __attribute__((aligned(16))) T As[2][BM][LDK];  // grad tile   [f][position]
  __shared__ __attribute__((aligned(16))) T Bs[2][BN][LDK];  // window tile [column][position]

  // eight wavefronts, two roles, as in tap_gemm_kernel: waves 0-3 issue the MFMAs,
  // waves 4-7 gather grad and x two K tiles ahead
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const bool loader = wave >= 4;
  const int tid = threadIdx.x & 255;  // index inside the role
  const int wm0 = ((wave & 3) / WAVES_N) * WM;
  const int wn0 = ((wave & 3) % WAVES_N) * WN;
  const int l16 = lane & 15, lk = lane >> 4;
  // Blocks are handed to the 8 XCDs round-robin, and each XCD has its own L2.  All
  // tiles of one K split read the same positions of grad and x, so they are given to
  // one XCD, next to each other in its dispatch order: block b is the (b/8)-th block
  // of XCD b%8, and an XCD takes whole splits.
  // (Only when the number of splits is a multiple of 8; otherwise plain order.)
  const int tiles_per_split = p.col_tiles * p.row_tiles;
  int split, tile;
  if (p.splits % 8 == 0) {
    const int xcd = blockIdx.x % 8, nth = blockIdx.x / 8;
    split = (nth / tiles_per_split) * 8 + xcd;
    tile = nth % tiles_per_split;
  } else {
    split = blockIdx.x / tiles_per_split;
    tile = blockIdx.x % tiles_per_split;
  }
  const int n0 = (tile % p.col_tiles) * BN;  // first column
  const int m0 = (tile / p.col_tiles) * BM;  // first filter (F % BM == 0)
  const int kbeg = split * p.kchunk;
  const int kend = min(kbeg + p.kchunk, p.kpos);

  const T *__restrict__ grad = static_cast<const T *>(p.grad);
  const T *__restrict__ x = static_cast<const T *>(p.x);
  const T *__restrict__ zeros = static_cast<const T *>(p.zeros);
  const int kcol = tid % BK;
  const int row0 = BK % 64 == 0 ? uniform(tid / BK) : tid / BK;
  const int g12 = p.G[1] * p.G[2];

  // the block's column groups never change: keep their table rows in registers
  const int8v MG_CONSTANT *gtab = (const int8v MG_CONSTANT *)(p.groups) + n0 / 16;
  int8v grp[NGROUPS];
#pragma unroll
  for (int j = 0; j < NGROUPS; ++j) grp[j] = gtab[j];

  constexpr int NB = NGROUPS * GLOADS;
  T ra0[ALOADS], rb0[NB], ra1[ALOADS], rb1[NB];

  auto fetch = [&](T(&ra)[ALOADS], T(&rb)[NB], int kt) {
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
    const T *ap = pos_ok ? grad + ((long long)n * p.g_nstride + gflat + (long long)(m0 + row0) * p.gvol) : zeros;
    const long long astep = pos_ok ? (long long)ROWS * p.gvol : 0;
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) ra[r] = ap[r * astep];
    const T *xn = x + ((long long)n * p.x_nstride + (qb0 * p.qs[0] + qb1 * p.qs[1] + qb2 * p.qs[2]) +
                       (long long)row0 * p.x_cstride);
#pragma unroll
    for (int j = 0; j < NGROUPS; ++j) {
      const int8v e = grp[j];  // coff, d0, d1, d2, valid
      const bool ok = pos_ok & (e[4] != 0) & ((unsigned)(qb0 + e[1]) < (unsigned)p.Q[0]) &
                      ((unsigned)(qb1 + e[2]) < (unsigned)p.Q[1]) & ((unsigned)(qb2 + e[3]) < (unsigned)p.Q[2]);
      const T *bp = ok ? xn + e[0] : zeros;
      const long long bstep = ok ? (long long)ROWS * p.x_cstride : 0;
#pragma unroll
      for (int r = 0; r < GLOADS; ++r) rb[j * GLOADS + r] = bp[r * bstep];
    }
  };
  auto stash = [&](const T(&ra)[ALOADS], const T(&rb)[NB], int buf) {
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) As[buf][row0 + r * ROWS][kcol] = ra[r];
#pragma unroll
    for (int j = 0; j < NGROUPS; ++j)
#pragma unroll
      for (int r = 0; r < GLOADS; ++r) Bs[buf][j * 16 + row0 + r * ROWS][kcol] = rb[j * GLOADS + r];
  };

  const int ktiles = kend > kbeg ? (kend - kbeg + BK - 1) / BK : 0;
  if (loader) {
    // tile i travels in register set i % 2 and lands in LDS buffer i % 2
    if (ktiles > 0) {
      fetch(ra0, rb0, 0);
      stash(ra0, rb0, 0);
      if (1 < ktiles) fetch(ra1, rb1, 1);
      if (2 < ktiles) fetch(ra0, rb0, 2);
    }
    __syncthreads();
    for (int kt = 0; kt < ktiles; kt += 2) {
      if (kt + 1 < ktiles) {
        stash(ra1, rb1, 1);
        if (kt + 3 < ktiles) fetch(ra1, rb1, kt + 3);
      }
      __syncthreads();
      if (kt + 1 < ktiles) {
        if (kt + 2 < ktiles) {
          stash(ra0, rb0, 0);
          if (kt + 4 < ktiles) fetch(ra0, rb0, kt + 4);
        }
        __syncthreads();
      }
    }
    return;
  }

  typename Mma<T>::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = typename Mma<T>::Acc{0, 0, 0, 0};

  // The order in which the K tile is contracted is free: quarter-wave lk takes the
  // K indices lk*KQ .. lk*KQ+KQ-1, one per MFMA step, so that four steps' operands
  // of a lane are adjacent in LDS and come in one read.
  __syncthreads();
  int buf = 0;
  for (int kt = 0; kt < ktiles; ++kt) {
#pragma unroll
    for (int s4 = 0; s4 < KQ / 4; ++s4) {
      T a[TM][4], b[TN][4];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const T *src = &As[buf][wm0 + i * 16 + l16][lk * KQ + s4 * 4];
        if constexpr (sizeof(T) == 4) {
          load_vec<T, 4>(src, a[i]);
        } else {
          T lo[2], hi[2];
          load_vec<T, 2>(src, lo);
          load_vec<T, 2>(src + 2, hi);
          a[i][0] = lo[0], a[i][1] = lo[1], a[i][2] = hi[0], a[i][3] = hi[1];
        }
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const T *src = &Bs[buf][wn0 + j * 16 + l16][lk * KQ + s4 * 4];
        if constexpr (sizeof(T) == 4) {
          load_vec<T, 4>(src, b[j]);
        } else {
          T lo[2], hi[2];
          load_vec<T, 2>(src, lo);
          load_vec<T, 2>(src + 2, hi);
          b[j][0] = lo[0], b[j][1] = lo[1], b[j][2] = hi[0], b[j][3] = hi[1];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = Mma<T>::run(a[i][u], b[j][u], acc[i][j]);
    }
    __syncthreads();
    buf ^= 1;
  }

  // partial sums [split][f][column]
  T *__restrict__ out = static_cast<T *>(p.out) + (long long)split * p.F * p.CT;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn0 + j * 16 + l16;
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

// dw[f][c][t] = ((part[0] + part[1]) + part[2]) + ...  of  part[s][f][col], where the
// columns run over channel blocks of 16, then taps, then the channel inside the block:
// col = ((c/16) * wvol + t) * 16 + c%16
template <typename T>
__global__ void __launch_bounds__(256) tap_reduce_kernel(const T *__restrict__ part, T *__restrict__ dw, int F, int C,
                                                         int wvol, int splits) {
  const int count = F * C * wvol;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;  // index into dw
  if (i >= count) return;
  const int ct = C * wvol;
  const int f = i / ct;
  const int r = i - f * ct;
  const int c = r / wvol;
  const int t = r - c * wvol;
  const int src = f * ct + ((c / 16) * wvol + t) * 16 + c % 16;
  dw[i] = sum_in_order(part + src, count, splits);
}

}  // namespace mg
