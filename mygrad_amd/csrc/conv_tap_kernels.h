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

#include <type_traits>

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

// A row of the phase table through the scalar data path (the index is wave-uniform).
__device__ __forceinline__ Phase load_phase(const Phase *phases, int i) {
  const int8v MG_CONSTANT *q = (const int8v MG_CONSTANT *)(phases + uniform(i));
  const int8v a = q[0], b = q[1], c = q[2];
  Phase ph;
  ph.J[0] = a[0], ph.J[1] = a[1], ph.J[2] = a[2];
  ph.o0[0] = a[3], ph.o0[1] = a[4], ph.o0[2] = a[5];
  ph.k_begin = a[6], ph.k_count = a[7];
  ph.blk_begin = b[0], ph.npos = b[1];
  ph.by_jvol = FastDiv{(unsigned)b[2], (unsigned)b[3], (unsigned)b[4], 0u};
  ph.by_j12 = FastDiv{(unsigned)b[6], (unsigned)b[7], (unsigned)c[0], 0u};
  ph.by_j2 = FastDiv{(unsigned)c[2], (unsigned)c[3], (unsigned)c[4], 0u};
  return ph;
}
__device__ __forceinline__ int phase_first_block(const Phase *phases, int i) {
  return ((const int MG_CONSTANT *)(phases + uniform(i)))[8];
}

// Gathers go through buffer loads: address = base + per-lane byte offset (VGPR) +
// wave-uniform byte offset (SGPR).  The channel step of a K tile's rows is uniform,
// so it rides in the SGPR and costs no vector instruction per load, and a lane
// whose tap falls in the padding gets a byte offset past the end of the buffer,
// for which the hardware returns zero without touching memory.  Vector ALU
// instructions of the loader waves are what the MFMA waves on the same SIMD wait
// for, so the loaders issue as few of them as possible.
// Tensors must be smaller than 2 GiB (kOutside must lie past the end).
constexpr unsigned kOutside = 0x80000000u;

// Sixteen bytes (VEC = 16 / sizeof(T) consecutive elements) per lane.
template <typename T>
__device__ __forceinline__ typename VecOf<T, 16 / sizeof(T)>::type buffer_load16(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_bytes,
                                                                               unsigned uniform_bytes) {
  typedef unsigned u4 __attribute__((ext_vector_type(4)));
  const u4 raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_bytes, (int)uniform_bytes, 0);
  return __builtin_bit_cast(typename VecOf<T, 16 / sizeof(T)>::type, raw);
}

constexpr int gcd_of(int a, int b) { return b == 0 ? a : gcd_of(b, a % b); }

// Whether tap_gemm_kernel with BM rows per tile runs persistent blocks that stream
// through several work items (else: one block per item).
constexpr bool tap_gemm_streams(int bm, int elem) { return bm >= 64 || elem == 8; }

template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const void *base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

template <typename T>
__device__ __forceinline__ T buffer_load(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_bytes, unsigned uniform_bytes) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_bytes, (int)uniform_bytes, 0));
  } else {
    return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)lane_bytes, (int)uniform_bytes, 0));
  }
}

// Double precision runs on v_mfma_f64_4x4x4_4b_f64: four independent 4x4x4 products
// ("blocks") per instruction, 16 cycles each, which reaches the device's fp64 matrix
// peak; v_mfma_f64_16x16x4_f64 measured 105 cycles on gfx950, 61 % of that peak.
// Lane l = 16*k + 4*b + r holds A[b][r][k], B[b][k][r] and (with k read as the row)
// D[b][k][r].  The four blocks are laid out 2x2 over an 8x8 patch of the output:
// block b covers rows 4*(b/2).. and columns 4*(b%2)..  With l16 = l % 16, lk = l / 16:
//   lane feeds row  quad_row(l16) = 4*(l16/8) + l16%4  of the patch (two lanes share each),
//        feeds column             l16 % 8              of the patch,
//        holds D at row 4*(l16/8) + lk, column l16 % 8.
struct Quad {
  static __device__ __forceinline__ int feed_row(int l16) { return ((l16 >> 3) << 2) | (l16 & 3); }
  static __device__ __forceinline__ int feed_col(int l16) { return l16 & 7; }
  static __device__ __forceinline__ int held_row(int l16, int lk) { return ((l16 >> 3) << 2) | lk; }
  static __device__ __forceinline__ double run(double a, double b, double c) {
    return __builtin_amdgcn_mfma_f64_4x4x4f64(a, b, c, 0, 0, 0);
  }
};

// ------------------------------------------------------------------------------------------
// forward and data gradient
// ------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int BK, int WM, int WN, int NPH = 1, bool FOLD = false, bool ROWS = false>
__global__ void __launch_bounds__(512) tap_gemm_kernel(const GemmParams p) {
  // ROWS: the BK rows of a K tile are any rows of the gather table (GemmParams::tab: element
  // offset and coordinate offsets of one (channel, tap) each), not BK channels under one tap;
  // KTile::coff is then the index of the tile's first table row.  For channel counts that are
  // no multiple of the K tile (a first layer's three): every row costs the gathering waves its
  // own bounds test, but the structure of the kernel -- and its MFMA waves -- stay the same.
  static_assert(!ROWS || (NPH == 1 && !FOLD), "table rows: plain tiles only");
  // FOLD: the three taps of the last axis are rows of the tile (see GemmParams::fold_row): three
  // times the rows per gathered element, a third of the K tiles.  A wave makes 48 rows (16
  // channels x 3 taps) x 64 positions, which are whole rows of the last axis.
  static_assert(!FOLD || (NPH == 1 && WM == 48 && WN == 64), "folded taps: 48 x 64 wave tiles");
  // NPH > 1: every tile computes NPH stride phases of the data gradient (see GemmParams::nph):
  // the K tiles of the phases follow each other in the tile's stream, each phase has its own
  // accumulators, and the epilogue writes the phases together.
  static_assert(NPH == 1 || NPH == 2 || NPH == 4, "1, 2 or 4 fused stride phases");
  // Tiles of 64 rows and more, and all double-precision tiles, run as persistent
  // blocks (see below).  The short float tiles of thin filter banks get one block per
  // item instead: moving the gather on to the next item from inside the K loop keeps
  // that code's inputs in scalar registers, which costs those shapes a resident block
  // per compute unit and more than the streaming gains them.
  constexpr bool STREAM = tap_gemm_streams(BM, (int)sizeof(T));
  static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per block");
  static_assert(BK % 4 == 0 && WM % 16 == 0 && WN % 16 == 0 && BN % 64 == 0, "MFMA 16x16x4 tiling");
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int WAVES_N = BN / WN;
  // the A tile (BK rows of BM packed filter values) is loaded and parked 16 bytes at a time
  constexpr int VEC = 16 / sizeof(T);
  constexpr int ALANES = BM / VEC;      // lanes that cover one row
  constexpr int AROWS = 256 / ALANES;   // rows covered by one pass of the loader waves
  constexpr int ALOADS = (BK + AROWS - 1) / AROWS;
  typedef typename VecOf<T, VEC>::type AVec;
  constexpr int BROWS = 256 / BN;
  constexpr int BLOADS = BK / BROWS;
  constexpr int PAD = 16 / sizeof(T);  // rows stay 16-byte aligned for the vector reads
  constexpr int LDA = BM + PAD, LDB = BN + PAD;

  __shared__ __attribute__((aligned(16))) T As[2][BK][LDA];
  __shared__ __attribute__((aligned(16))) T Bs[2][BK][LDB];

  // Eight wavefronts with two roles.  Waves 0-3 only read LDS and issue MFMAs; waves
  // 4-7 only gather: global loads -> registers -> LDS, ahead of the MFMA waves.  One of
  // each sits on every SIMD, so the gather's memory instructions and LDS stores are
  // issued in the shadow of the other wave's MFMAs.
  //
  // Blocks are persistent: block b works through the items b, b + gridDim.x, ...  An
  // item is a whole tile or, for the tiles of the last partial round, one K slice of a
  // tile (its partial sums go to a workspace for tail_fixup_kernel).  The K tiles of a
  // block's items form one stream: stream element s lives in LDS buffer s % 2, and the
  // loader waves run ahead of the MFMA waves across item boundaries, so the first
  // operands of the next tile are already on their way while this tile is finished
  // and stored.  One barrier at the start, then one per stream element.
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const bool loader = wave >= 4;
  const int tid = threadIdx.x & 255;  // index inside the role
  const int wm0 = ((wave & 3) / WAVES_N) * WM;
  const int wn0 = ((wave & 3) % WAVES_N) * WN;
  const int l16 = lane & 15, lk = lane >> 4;

  // ---- one work item (all wave-uniform).  Tiles are numbered with the row tile (m)
  // innermost, so that the row tiles of one position block, which gather the same
  // elements, run next to each other; items >= p.full_tiles are K slices.
  struct Item {
    int tile, piece, pos0, m0, kt_begin, kt_end, slot;
    bool partial;
    Phase ph;
  };
  // Even shares of the last round (see GemmParams::share_first): the block's own run of slices
  const bool shares = p.share_first != nullptr;
  const int share_begin = shares ? ((const int MG_CONSTANT *)p.share_first)[uniform((int)blockIdx.x)] : 0;
  const int share_end = shares ? ((const int MG_CONSTANT *)p.share_first)[uniform((int)blockIdx.x) + 1] : 0;
  const int item_end = shares ? p.full_tiles + share_end : p.items;
  // the block's place in the order of the tiles (see GemmParams::xcd_chunk)
  const int chunk = p.xcd_chunk;
  const int place = chunk > 1 ? (((int)blockIdx.x >> 3) / chunk * 8 + ((int)blockIdx.x & 7)) * chunk + ((int)blockIdx.x >> 3) % chunk
                              : (int)blockIdx.x;
  const int item_first = (!shares || place < p.full_tiles) ? place : p.full_tiles + share_begin;
  auto next_item = [&](int item) -> int {
    if (!shares) return item + (int)gridDim.x;
    if (item >= p.full_tiles) return item + 1;
    return item + (int)gridDim.x < p.full_tiles ? item + (int)gridDim.x : p.full_tiles + share_begin;
  };
  auto locate = [&](int item, int &pi, Item &it) {  // pi: phase of the previous item of this cursor (tiles ascend)
    it.tile = item;
    it.piece = 0;
    it.slot = 0;
    it.partial = item >= p.full_tiles;
    int4v row = {0, 0, 0, 0};
    if (it.partial) {
      if (shares) {
        row = ((const int4v MG_CONSTANT *)p.share_slices)[uniform(item - p.full_tiles)];
        it.tile = row[0];
        it.slot = row[3];
        it.partial = row[3] >= 0;
      } else {
        const int j = item - p.full_tiles;
        it.tile = p.full_tiles + j / p.tail_split;
        it.piece = j % p.tail_split;
        it.slot = j;
      }
    }
    const int pblk = it.tile / p.m_tiles;
    while (pi + 1 < p.nphases && pblk >= phase_first_block(p.phases, pi + 1)) ++pi;
    it.ph = load_phase(p.phases, pi);
    it.pos0 = (pblk - it.ph.blk_begin) * BN;
    it.m0 = (it.tile % p.m_tiles) * BM;
    it.kt_begin = 0;
    it.kt_end = it.ph.k_count;
    if (shares && item >= p.full_tiles) {
      it.kt_begin = row[1];
      it.kt_end = row[2];
    } else if (it.partial) {
      const int per = (it.ph.k_count + p.tail_split - 1) / p.tail_split;
      it.kt_begin = min(it.piece * per, it.ph.k_count);
      it.kt_end = min(it.kt_begin + per, it.ph.k_count);
    }
  };

  if (loader) {
    const __amdgpu_buffer_rsrc_t a_buf = buffer_of<T>(p.A, p.a_bytes);
    const __amdgpu_buffer_rsrc_t src_buf = buffer_of<T>(p.src, p.src_bytes);
    const int bcol = tid % BN;
    const int brow0 = uniform(tid / BN);
    const int acol = (tid % ALANES) * VEC;
    const int arow0 = tid / ALANES;
    const unsigned a_row_bytes = (unsigned)p.a_ld * (unsigned)sizeof(T);
    const unsigned b_step = (unsigned)(BROWS * p.src_cstride) * (unsigned)sizeof(T);

    // ---- fetch cursor: the item being gathered and this thread's place in it
    Item it;
    int pi = 0, item = -1, kt = 0;
    const int8v MG_CONSTANT *ktab = nullptr;
    int qb0 = 0, qb1 = 0, qb2 = 0;
    bool pos_ok = false;
    unsigned src_at = 0;  // byte offset of the position's tap (0,0,0), channel brow0
    unsigned a_at = kOutside;
    // moves the cursor to the first item at or after `from` that has K tiles; false if none
    auto enter = [&](int from) -> bool {
      for (int i = from; i < item_end; i = next_item(i)) {
        locate(i, pi, it);
        if (it.kt_begin >= it.kt_end) continue;
        item = i;
        kt = it.kt_begin;
        ktab = (const int8v MG_CONSTANT *)(p.ktiles + it.ph.k_begin);
        const int j12 = it.ph.J[1] * it.ph.J[2];
        pos_ok = it.pos0 + bcol < it.ph.npos;
        const unsigned pos = pos_ok ? (unsigned)(it.pos0 + bcol) : 0u;
        const unsigned n = it.ph.by_jvol.div(pos);
        unsigned r = pos - n * (unsigned)(it.ph.J[0] * j12);
        const unsigned j0 = it.ph.by_j12.div(r);
        r -= j0 * (unsigned)j12;
        const unsigned j1 = it.ph.by_j2.div(r);
        const unsigned j2 = r - j1 * (unsigned)it.ph.J[2];
        qb0 = (int)j0 * p.sj[0];
        qb1 = (int)j1 * p.sj[1];
        qb2 = (int)j2 * p.sj[2];
        src_at = (unsigned)((long long)n * p.src_nstride + (qb0 * p.qs[0] + qb1 * p.qs[1] + qb2 * p.qs[2]) +
                            (ROWS ? 0 : brow0 * p.src_cstride)) * (unsigned)sizeof(T);
        const bool a_ok = (it.m0 + acol < p.a_ld) & (arow0 < BK);  // rows are padded to whole 16-byte pieces
        a_at = a_ok ? (unsigned)(arow0 * p.a_ld + it.m0 + acol) * (unsigned)sizeof(T) : kOutside;
        return true;
      }
      return false;
    };
    // K tile under the cursor -> registers; then the cursor moves on.  Past the end of
    // the stream it stays on the last K tile (the data is never used): every call
    // issues the same loads, so the compiler can count them exactly.
    bool live = false;  // the cursor is on a K tile that has not been requested yet
    int requested = 0;  // stream elements requested so far
    auto fetch = [&](AVec(&ra)[ALOADS], T(&rb)[BLOADS]) {
      const int8v e = ktab[kt];  // a_row0, coff, d0, d1, d2
      const unsigned a_tile = (unsigned)e[0] * a_row_bytes;
#pragma unroll
      for (int r = 0; r < ALOADS; ++r) ra[r] = buffer_load16<T>(a_buf, a_at, a_tile + (unsigned)(r * AROWS) * a_row_bytes);
      if constexpr (ROWS) {
        const int4v MG_CONSTANT *rows = (const int4v MG_CONSTANT *)(p.tab) + e[1];
#pragma unroll
        for (int r = 0; r < BLOADS; ++r) {
          const int4v t = rows[brow0 + r * BROWS];  // off, d0, d1, d2 (the row is the same for the whole wave)
          const bool ok = pos_ok & ((unsigned)(qb0 + t[1]) < (unsigned)p.Q[0]) & ((unsigned)(qb1 + t[2]) < (unsigned)p.Q[1]) &
                          ((unsigned)(qb2 + t[3]) < (unsigned)p.Q[2]);
          rb[r] = buffer_load<T>(src_buf, ok ? src_at + (unsigned)(t[0] * (int)sizeof(T)) : kOutside, 0u);
        }
      } else {
        const bool ok = pos_ok & ((unsigned)(qb0 + e[2]) < (unsigned)p.Q[0]) & ((unsigned)(qb1 + e[3]) < (unsigned)p.Q[1]) &
                        ((unsigned)(qb2 + e[4]) < (unsigned)p.Q[2]);
        const unsigned at = ok ? src_at + (unsigned)(e[1] * (int)sizeof(T)) : kOutside;
#pragma unroll
        for (int r = 0; r < BLOADS; ++r) rb[r] = buffer_load<T>(src_buf, at, (unsigned)r * b_step);
      }
      if (live) {
        ++requested;
        if (kt + 1 < it.kt_end)
          ++kt;
        else if constexpr (STREAM)
          live = enter(next_item(item));  // no further item: the cursor stays where it is
        else
          live = false;
      }
    };
    auto stash = [&](const AVec(&ra)[ALOADS], const T(&rb)[BLOADS], int buf) {
#pragma unroll
      for (int r = 0; r < ALOADS; ++r) {
        const int kk = arow0 + r * AROWS;
        if (kk < BK) *reinterpret_cast<AVec *>(&As[buf][kk][acol]) = ra[r];
      }
#pragma unroll
      for (int r = 0; r < BLOADS; ++r) Bs[buf][brow0 + r * BROWS][bcol] = rb[r];
    };

    // two register sets: stream element s travels in set s % 2 and is requested two
    // elements before it is parked in LDS
    AVec ra0[ALOADS], ra1[ALOADS];
    T rb0[BLOADS], rb1[BLOADS];
    live = enter(item_first);
    if (live) {
      fetch(ra0, rb0);
      stash(ra0, rb0, 0);
      fetch(ra1, rb1);
      fetch(ra0, rb0);
    }
    __syncthreads();
    // While the MFMA waves work on element s, element s+1 (requested two steps ago) is
    // parked in the idle buffer and element s+3 requested into the registers it left.
    // Requests run three elements ahead, so `requested` is final before s reaches it.
    for (int s = 0; s < requested;) {
      stash(ra1, rb1, 1);
      fetch(ra1, rb1);
      __syncthreads();
      if (++s >= requested) break;
      stash(ra0, rb0, 0);
      fetch(ra0, rb0);
      __syncthreads();
      ++s;
    }
    return;
  }

  // ---- MFMA waves
  Item it;
  int pi = 0;
  int buf = 0;
  T *__restrict__ dst = static_cast<T *>(p.dst);
  if (item_first < item_end) locate(item_first, pi, it);  // (with even shares a block may have nothing to do)
  __syncthreads();
  // AHEAD: operands of one K step (k4: which four rows of the K tile in `buf`), see `step` below
  constexpr bool AHEAD = sizeof(T) == 4 && BM == 64 && BN == 256 && NPH == 1 && !FOLD;
  constexpr int OPA = AHEAD ? TM : 1, OPB = AHEAD ? TN : 1;
  T cur_a[OPA], cur_b[OPB];
  auto read_step = [&](int k4, T(&a)[OPA], T(&b)[OPB]) {
    if constexpr (AHEAD) {
      load_vec<T, TM>(&As[buf][k4 * 4 + lk][wm0 + l16 * TM], a);
      load_vec<T, TN>(&Bs[buf][k4 * 4 + lk][wn0 + l16 * TN], b);
    }
  };
  read_step(0, cur_a, cur_b);
  for (int item = item_first; item < item_end; item = next_item(item)) {
    if (item != item_first) locate(item, pi, it);
    const Phase &ph = it.ph;
    const int pos0 = it.pos0, m0 = it.m0;
    const int j12 = ph.J[1] * ph.J[2];
    const int jvol = ph.J[0] * j12;
    // position -> sample and grid coordinates of its phase (the coarse grid when phases are fused)
    auto split_pos = [&](int ipos, int &n, int &j0, int &j1, int &j2) {
      const unsigned pos = (unsigned)ipos;
      const unsigned nn = ph.by_jvol.div(pos);
      unsigned r = pos - nn * (unsigned)jvol;
      j0 = (int)ph.by_j12.div(r);
      r -= (unsigned)j0 * (unsigned)j12;
      j1 = (int)ph.by_j2.div(r);
      j2 = (int)r - j1 * ph.J[2];
      n = (int)nn;
    };
    auto dst_of = [&](int ipos) -> T * {
      int n, j0, j1, j2;
      split_pos(ipos, n, j0, j1, j2);
      return dst + (long long)n * p.dst_nstride + (long long)(ph.o0[0] + j0 * p.oj[0]) * p.os[0] +
             (long long)(ph.o0[1] + j1 * p.oj[1]) * p.os[1] + (long long)(ph.o0[2] + j2 * p.oj[2]) * p.os[2];
    };
    // fused phases: where coarse position (n, j) of phase f lies in dst, and whether it exists
    auto fused_dst = [&](int f, int n, int j0, int j1, int j2) -> T * {
      return dst + (long long)n * p.dst_nstride + (long long)(p.po0[f][0] + j0 * p.oj[0]) * p.os[0] +
             (long long)(p.po0[f][1] + j1 * p.oj[1]) * p.os[1] + (long long)(p.po0[f][2] + j2 * p.oj[2]) * p.os[2];
    };
    auto fused_ok = [&](int f, int j0, int j1, int j2) -> bool {
      return (j0 < p.pJ[f][0]) & (j1 < p.pJ[f][1]) & (j2 < p.pJ[f][2]);
    };
    T *slot = static_cast<T *>(p.partial) + (long long)it.slot * (NPH * BM * BN);

    if constexpr (sizeof(T) == 8) {
      // The wave tile is cut into 8-row and 8-column groups; group pairs are interleaved
      // (row = pair*16 + 2*patch_row + half) so that a lane's two operands of a pair are
      // adjacent in LDS and the 8 distinct lanes of a read cover 128 contiguous bytes.
      constexpr int GM = WM / 8, GN = WN / 8;
      const int arow = wm0 + Quad::feed_row(l16) * 2;
      const int bcol8 = wn0 + Quad::feed_col(l16) * 2;
      const int drow = wm0 + Quad::held_row(l16, lk) * 2;
      double acc[NPH][GM][GN];
#pragma unroll
      for (int f = 0; f < NPH; ++f)
#pragma unroll
        for (int i = 0; i < GM; ++i)
#pragma unroll
          for (int j = 0; j < GN; ++j) acc[f][i][j] = 0.0;
      auto step = [&](auto fc) {  // one K tile into accumulator set f
        constexpr int f = decltype(fc)::value;
#pragma unroll
        for (int k4 = 0; k4 < BK / 4; ++k4) {
          T a[GM], b[GN];
#pragma unroll
          for (int g = 0; g < GM / 2; ++g) {
            T two[2];
            load_vec<T, 2>(&As[buf][k4 * 4 + lk][arow + g * 16], two);
            a[2 * g] = two[0], a[2 * g + 1] = two[1];
          }
#pragma unroll
          for (int g = 0; g < GN / 2; ++g) {
            T two[2];
            load_vec<T, 2>(&Bs[buf][k4 * 4 + lk][bcol8 + g * 16], two);
            b[2 * g] = two[0], b[2 * g + 1] = two[1];
          }
#pragma unroll
          for (int i = 0; i < GM; ++i)
#pragma unroll
            for (int j = 0; j < GN; ++j) acc[f][i][j] = Quad::run(a[i], b[j], acc[f][i][j]);
        }
        __syncthreads();
        buf ^= 1;
      };
      if constexpr (NPH == 1) {
        for (int kt = it.kt_begin; kt < it.kt_end; ++kt) step(std::integral_constant<int, 0>{});
      } else {
        // K tiles of a fused tile run filter block by filter block; inside a block the taps
        // of phase 0 come first, then those of phase 1, ...: tile `off` of a block belongs to
        // the phase f with kcut[f - 1] <= off < kcut[f].
        int kt = it.kt_begin;
        int off = kt % p.kcut[NPH - 1];
        while (kt < it.kt_end) {
          for (; off < p.kcut[0] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 0>{});
          for (; off < p.kcut[1] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 1>{});
          if constexpr (NPH == 4) {
            for (; off < p.kcut[2] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 2>{});
            for (; off < p.kcut[3] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 3>{});
          }
          off = 0;
        }
      }
      // ---- epilogue: acc[.][i][j] is row drow + (i/2)*16 + i%2, column bcol8 + (j/2)*16 + j%2
      if (it.partial) {
#pragma unroll
        for (int f = 0; f < NPH; ++f)
#pragma unroll
          for (int i = 0; i < GM; ++i) {
            const int ml = drow + (i / 2) * 16 + i % 2;
#pragma unroll
            for (int g = 0; g < GN / 2; ++g) {
              const T two[2] = {acc[f][i][2 * g], acc[f][i][2 * g + 1]};
              store_vec<T, 2>(slot + f * (BM * BN) + ml * BN + bcol8 + g * 16, two);
            }
          }
        continue;
      }
      if constexpr (FOLD) {
        // Double precision with folded taps.  Rows are ordered (tap of the last axis, channel), so
        // that the lane's row pairs i = 0,1 / 2,3 / 4,5 are taps 0 / 1 / 2 of its two channels
        // drow, drow + 1.  A lane holds the position pairs first, first + 1 (first = 2q + 16g, q its
        // place among the eight lanes that share its rows):
        //   dst[pos] = tap1[pos] + tap0[pos + 1] + tap2[pos - 1]
        // pos + 1 of an odd position and pos - 1 of an even one are with the lane next door (the
        // first pair of q = 0 and the last of q = 7: with the lane at the other end, one pair over),
        // and beyond the ends of a (padded) row there is nothing to add.
        static_assert(GM == 6 && GN == 8, "three taps x two channels, four position pairs per lane");
        const int q8 = l16 & 7;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const int m = (m0 + wm0) / 3 + (drow - wm0) + r;  // channel
          T out_e[GN / 2], out_o[GN / 2];
#pragma unroll
          for (int g = 0; g < GN / 2; ++g) {
            const T t0e = acc[0][r][2 * g], t0o = acc[0][r][2 * g + 1];
            const T t1e = acc[0][2 + r][2 * g], t1o = acc[0][2 + r][2 * g + 1];
            const T t2e = acc[0][4 + r][2 * g], t2o = acc[0][4 + r][2 * g + 1];
            // the odd position to the left of this pair, the even one to its right
            const T left_near = __shfl_up(t2o, 1, 8);
            const T left_far = __shfl(g > 0 ? acc[0][4 + r][2 * g - 1] : T(0), 7, 8);
            const T right_near = __shfl_down(t0e, 1, 8);
            const T right_far = __shfl(g + 1 < GN / 2 ? acc[0][r][2 * g + 2] : T(0), 0, 8);
            const int first = pos0 + bcol8 + g * 16;
            const unsigned in_row = (unsigned)first & (unsigned)(p.fold_row - 1);
            const T left = in_row == 0 ? T(0) : (q8 > 0 ? left_near : left_far);
            const T right = in_row + 2 == (unsigned)p.fold_row ? T(0) : (q8 < 7 ? right_near : right_far);
            out_e[g] = (t1e + t0o) + left;
            out_o[g] = (t1o + right) + t2e;
          }
#pragma unroll
          for (int g = 0; g < GN / 2; ++g) {
            const int first = pos0 + bcol8 + g * 16;
            const int real = p.Q[2] - (int)((unsigned)first & (unsigned)(p.fold_row - 1));
            if (first >= ph.npos || real <= 0 || m >= p.M) continue;
            T *out = dst_of(first) + (long long)m * p.dst_mstride;
            if (p.vec_store) {
              const T two[2] = {out_e[g], out_o[g]};
              store_vec<T, 2>(out, two);
            } else {
              out[0] = out_e[g];
              if (real > 1) out[1] = out_o[g];
            }
          }
        }
        continue;
      }
#pragma unroll
      for (int g = 0; g < GN / 2; ++g) {
        const int first = pos0 + bcol8 + g * 16;
        if constexpr (NPH > 1) {
          if (p.vec_store && ph.J[2] % 2 == 0) {
            // both coarse positions exist, lie in one row, and their phases are adjacent in dst
            if (first >= ph.npos) continue;
            int n, j0, j1, j2;
            split_pos(first, n, j0, j1, j2);
            // phases f and f+1 alternate along the last axis: four adjacent elements of dst
#pragma unroll
            for (int f = 0; f < NPH; f += 2) {
              if (!fused_ok(f, j0, j1, j2)) continue;
              T *out = fused_dst(f, n, j0, j1, j2);
#pragma unroll
              for (int i = 0; i < GM; ++i) {
                const int m = m0 + drow + (i / 2) * 16 + i % 2;
                const T lo[2] = {acc[f][i][2 * g], acc[f + 1][i][2 * g]};
                const T hi[2] = {acc[f][i][2 * g + 1], acc[f + 1][i][2 * g + 1]};
                if (m < p.M) {
                  store_vec<T, 2>(out + (long long)m * p.dst_mstride, lo);
                  store_vec<T, 2>(out + (long long)m * p.dst_mstride + 2, hi);
                }
              }
            }
          } else {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              if (first + h >= ph.npos) continue;
              int n, j0, j1, j2;
              split_pos(first + h, n, j0, j1, j2);
#pragma unroll
              for (int f = 0; f < NPH; ++f) {
                if (!fused_ok(f, j0, j1, j2)) continue;
                T *out = fused_dst(f, n, j0, j1, j2);
#pragma unroll
                for (int i = 0; i < GM; ++i) {
                  const int m = m0 + drow + (i / 2) * 16 + i % 2;
                  if (m < p.M) out[(long long)m * p.dst_mstride] = acc[f][i][2 * g + h];
                }
              }
            }
          }
        } else if (p.vec_store) {
          // both positions exist (npos % 4 == 0) and are adjacent in dst
          if (first >= ph.npos) continue;
          T *out = dst_of(first);
#pragma unroll
          for (int i = 0; i < GM; ++i) {
            const int m = m0 + drow + (i / 2) * 16 + i % 2;
            const T two[2] = {acc[0][i][2 * g], acc[0][i][2 * g + 1]};
            if (m < p.M) store_vec<T, 2>(out + (long long)m * p.dst_mstride, two);
          }
        } else if (p.phase_count != 0) {
          // rows are (channel, stride phase): each goes to its phase's element of the coarse position.
          // The lane's rows 2r, 2r + 1 are phases 2q, 2q + 1 of one channel: neighbours along the
          // last axis when that is where the stride is, stored together.
          typedef T OutPair __attribute__((ext_vector_type(2), aligned(sizeof(T))));
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            if (first + h >= ph.npos) continue;
            int n, j0, j1, j2;
            split_pos(first + h, n, j0, j1, j2);
#pragma unroll
            for (int i = 0; i < GM; i += 2) {
              const int m = m0 + drow + (i / 2) * 16;  // even: phase f even
              if (m >= p.M) continue;
              const int c = m / p.phase_count, f = m - c * p.phase_count;
              const bool even = fused_ok(f, j0, j1, j2), odd = fused_ok(f + 1, j0, j1, j2);
              T *out = fused_dst(f, n, j0, j1, j2) + (long long)c * p.dst_mstride;
              if (p.phase_pairs && even && odd) {
                OutPair v;
                v[0] = acc[0][i][2 * g + h], v[1] = acc[0][i + 1][2 * g + h];
                *reinterpret_cast<OutPair *>(out) = v;
              } else {
                if (even) out[0] = acc[0][i][2 * g + h];
                if (odd) fused_dst(f + 1, n, j0, j1, j2)[(long long)c * p.dst_mstride] = acc[0][i + 1][2 * g + h];
              }
            }
          }
        } else {
          // positions adjacent in dst but not 16-byte aligned: the pair as one vector of element
          // alignment when both lie in one sample
          bool together = false;
          if (p.run_store && first + 2 <= ph.npos) {
            const unsigned nn = ph.by_jvol.div((unsigned)first);
            together = (unsigned)first - nn * (unsigned)jvol + 2u <= (unsigned)jvol;
          }
          if (together) {
            typedef T OutPair __attribute__((ext_vector_type(2), aligned(sizeof(T))));
            T *out = dst_of(first);
#pragma unroll
            for (int i = 0; i < GM; ++i) {
              const int m = m0 + drow + (i / 2) * 16 + i % 2;
              if (m < p.M) {
                OutPair v;
                v[0] = acc[0][i][2 * g], v[1] = acc[0][i][2 * g + 1];
                *reinterpret_cast<OutPair *>(out + (long long)m * p.dst_mstride) = v;
              }
            }
          } else {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              if (first + h >= ph.npos) continue;
              T *out = dst_of(first + h);
#pragma unroll
              for (int i = 0; i < GM; ++i) {
                const int m = m0 + drow + (i / 2) * 16 + i % 2;
                if (m < p.M) out[(long long)m * p.dst_mstride] = acc[0][i][2 * g + h];
              }
            }
          }
        }
      }
    } else {
      // Lane (l16, lk) feeds row/column l16 of every 16x16 tile.  Tile i of the wave
      // takes the rows m = wm0 + l16*TM + i (and tile j the positions wn0 + l16*TN + j),
      // so the TM (TN) operands of a lane are adjacent in LDS and come in one read.
      typename Mma<T>::Acc acc[NPH][TM][TN];
#pragma unroll
      for (int f = 0; f < NPH; ++f)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[f][i][j] = typename Mma<T>::Acc{0, 0, 0, 0};
      // AHEAD (64 x 256 float tiles): the operands of a K step are read from LDS one step ahead
      // of the MFMAs that use them, and the barrier that ends a K tile stands before the tile's
      // last step: by then the wave has read all of the tile (the last step's operands are in
      // registers), so the gathering waves may refill its buffer, and the first operands of the
      // next tile are on their way from LDS while the last MFMAs of this one run.  (cur_a /
      // cur_b: the operands of the next step to run, carried from tile to tile and item to item.)
      // Measured: config 3a forward 247 -> 232 us; the other tile shapes lose 1 - 5 % with it.
      auto step = [&](auto fc) {  // one K tile into accumulator set f
        constexpr int f = decltype(fc)::value;
        if constexpr (AHEAD) {
#pragma unroll
          for (int k4 = 0; k4 < BK / 4; ++k4) {
            T na[TM], nb[TN];
            if (k4 + 1 < BK / 4) {
              read_step(k4 + 1, na, nb);
            } else {
              __syncthreads();
              buf ^= 1;
              read_step(0, na, nb);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j) acc[f][i][j] = Mma<T>::run(cur_a[i], cur_b[j], acc[f][i][j]);
#pragma unroll
            for (int i = 0; i < TM; ++i) cur_a[i] = na[i];
#pragma unroll
            for (int j = 0; j < TN; ++j) cur_b[j] = nb[j];
          }
        } else {
#pragma unroll
          for (int k4 = 0; k4 < BK / 4; ++k4) {
            T a[TM], b[TN];
            if constexpr (TM == 3) {
#pragma unroll
              for (int i = 0; i < TM; ++i) a[i] = As[buf][k4 * 4 + lk][wm0 + l16 * TM + i];
            } else {
              load_vec<T, TM>(&As[buf][k4 * 4 + lk][wm0 + l16 * TM], a);
            }
            load_vec<T, TN>(&Bs[buf][k4 * 4 + lk][wn0 + l16 * TN], b);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j) acc[f][i][j] = Mma<T>::run(a[i], b[j], acc[f][i][j]);
          }
          __syncthreads();
          buf ^= 1;
        }
      };
      if constexpr (NPH == 1) {
        for (int kt = it.kt_begin; kt < it.kt_end; ++kt) step(std::integral_constant<int, 0>{});
      } else {
        // K tiles of a fused tile run filter block by filter block; inside a block the taps
        // of phase 0 come first, then those of phase 1, ...: tile `off` of a block belongs to
        // the phase f with kcut[f - 1] <= off < kcut[f].
        int kt = it.kt_begin;
        int off = kt % p.kcut[NPH - 1];
        while (kt < it.kt_end) {
          for (; off < p.kcut[0] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 0>{});
          for (; off < p.kcut[1] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 1>{});
          if constexpr (NPH == 4) {
            for (; off < p.kcut[2] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 2>{});
            for (; off < p.kcut[3] && kt < it.kt_end; ++off, ++kt) step(std::integral_constant<int, 3>{});
          }
          off = 0;
        }
      }

      // ---- epilogue
      if (it.partial) {
        // raw tile [BM][BN] of this slice (one per phase), lane's TN positions stored as one vector
        T *mine = slot + (wn0 + l16 * TN);
#pragma unroll
        for (int f = 0; f < NPH; ++f)
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int ml = wm0 + Mma<T>::row_of(lane, q) * TM + i;
              T v[TN];
#pragma unroll
              for (int j = 0; j < TN; ++j) v[j] = acc[f][i][j][q];
              store_vec<T, TN>(mine + f * (BM * BN) + ml * BN, v);
            }
        continue;
      }
      const int first = pos0 + wn0 + l16 * TN;
      if constexpr (NPH > 1) {
        // Phases f and f + 1 alternate along the last axis of dst (coarse position j2 of phase f is
        // element 2 * j2 of the row, of phase f + 1 element 2 * j2 + 1), so what a lane holds for
        // PER coarse positions of one row are 2 * PER adjacent elements.  Rows of dst need not
        // start on 16-byte boundaries (an exact window grid under stride 2 has an odd extent):
        // the stores only assume the alignment of an element.  The phase with the odd elements is
        // one position shorter when the extent is odd: the pair that reaches beyond a row's end is
        // stored element by element.
        constexpr int PER = TN < 2 ? TN : 2;  // coarse positions per (up to) 16-byte store
        typedef T OutVec __attribute__((ext_vector_type(2 * PER), aligned(sizeof(T))));
        if (ph.J[2] % PER == 0) {
          // the PER coarse positions of a store lie in one row of the coarse grid
#pragma unroll
          for (int h = 0; h < TN / PER; ++h) {
            if (first + h * PER >= ph.npos) continue;
            int n, j0, j1, j2;
            split_pos(first + h * PER, n, j0, j1, j2);
#pragma unroll
            for (int f = 0; f < NPH; f += 2) {
              if (!((j0 < p.pJ[f][0]) & (j1 < p.pJ[f][1]))) continue;
              T *out = fused_dst(f, n, j0, j1, j2);
              const bool whole = (j2 + PER <= p.pJ[f][2]) & (j2 + PER <= p.pJ[f + 1][2]);
#pragma unroll
              for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  const int m = m0 + wm0 + Mma<T>::row_of(lane, q) * TM + i;
                  if (m >= p.M) continue;
                  T *row = out + (long long)m * p.dst_mstride;
                  if (whole) {
                    OutVec v;
#pragma unroll
                    for (int t = 0; t < PER; ++t) {
                      v[2 * t] = acc[f][i][h * PER + t][q];
                      v[2 * t + 1] = acc[f + 1][i][h * PER + t][q];
                    }
                    *reinterpret_cast<OutVec *>(row) = v;
                  } else {
#pragma unroll
                    for (int t = 0; t < PER; ++t) {
                      if (j2 + t < p.pJ[f][2]) row[2 * t] = acc[f][i][h * PER + t][q];
                      if (j2 + t < p.pJ[f + 1][2]) row[2 * t + 1] = acc[f + 1][i][h * PER + t][q];
                    }
                  }
                }
            }
          }
        } else {
          // an odd number of coarse positions per row: one position, two adjacent elements, at a time
          typedef T Pair __attribute__((ext_vector_type(2), aligned(sizeof(T))));
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            if (first + j >= ph.npos) continue;
            int n, j0, j1, j2;
            split_pos(first + j, n, j0, j1, j2);
#pragma unroll
            for (int f = 0; f < NPH; f += 2) {
              if (!((j0 < p.pJ[f][0]) & (j1 < p.pJ[f][1]))) continue;
              T *out = fused_dst(f, n, j0, j1, j2);
              const bool even = j2 < p.pJ[f][2], odd = j2 < p.pJ[f + 1][2];
#pragma unroll
              for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  const int m = m0 + wm0 + Mma<T>::row_of(lane, q) * TM + i;
                  if (m >= p.M) continue;
                  T *row = out + (long long)m * p.dst_mstride;
                  if (even & odd) {
                    Pair v;
                    v[0] = acc[f][i][j][q], v[1] = acc[f + 1][i][j][q];
                    *reinterpret_cast<Pair *>(row) = v;
                  } else {
                    if (even) row[0] = acc[f][i][j][q];
                    if (odd) row[1] = acc[f + 1][i][j][q];
                  }
                }
            }
          }
        }
      } else if constexpr (FOLD) {
        // Tile i of the wave holds tap i of the last axis for the lane's channels 4*lk + q and its
        // TN = 4 adjacent positions first .. first + 3 of one row:
        //   dst[pos] = tap1[pos] + tap0[pos + 1] + tap2[pos - 1]
        // with zeros beyond the ends of the row.  pos + 1 and pos - 1 are in the lane itself or
        // in its neighbours of the same quarter-wave (a wave's positions are whole rows, so the
        // first and last lane of a quarter never need a neighbour).
        static_assert(TM == 3 && TN == 4, "three taps, four positions per lane");
        // (A row of positions is padded to fold_row, a power of two; the padding positions
        // gather nothing, so their sums are zero -- which is what the last real position of a
        // row must see to its right -- and they are not stored.)
        const unsigned in_row = (unsigned)first & (unsigned)(p.fold_row - 1);
        const bool has_prev = in_row != 0, has_next = in_row + TN != (unsigned)p.fold_row;
        const int real = p.Q[2] - (int)in_row;  // positions of this lane that exist: min(real, TN), none if <= 0
        const bool exists = first < ph.npos && real > 0;
        T *out = dst_of(exists ? first : 0);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const T from_prev = __shfl_up(acc[0][2][TN - 1][q], 1, 16);
          const T from_next = __shfl_down(acc[0][0][0][q], 1, 16);
          T v[TN];
          v[0] = (acc[0][1][0][q] + acc[0][0][1][q]) + (has_prev ? from_prev : T(0));
          v[1] = (acc[0][1][1][q] + acc[0][0][2][q]) + acc[0][2][0][q];
          v[2] = (acc[0][1][2][q] + acc[0][0][3][q]) + acc[0][2][1][q];
          v[3] = (acc[0][1][3][q] + (has_next ? from_next : T(0))) + acc[0][2][2][q];
          const int m = (m0 + wm0) / 3 + Mma<T>::row_of(lane, q);
          if (exists && m < p.M) {
            if (p.vec_store) {
              store_vec<T, TN>(out + (long long)m * p.dst_mstride, v);
            } else {
#pragma unroll
              for (int j = 0; j < TN; ++j)
                if (j < real) out[(long long)m * p.dst_mstride + j] = v[j];
            }
          }
        }
      } else if (p.vec_store) {
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
                for (int j = 0; j < TN; ++j) v[j] = acc[0][i][j][q];
                store_vec<T, TN>(out + (long long)m * p.dst_mstride, v);
              }
            }
        }
      } else if (p.phase_count != 0) {
        // rows are (channel, stride phase): each goes to its phase's element of the coarse position
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if (first + j >= ph.npos) continue;
          int n, j0, j1, j2;
          split_pos(first + j, n, j0, j1, j2);
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int m = m0 + wm0 + Mma<T>::row_of(lane, q) * TM + i;
              if (m >= p.M) continue;
              const int c = m / p.phase_count, f = m - c * p.phase_count;
              if (fused_ok(f, j0, j1, j2)) fused_dst(f, n, j0, j1, j2)[(long long)c * p.dst_mstride] = acc[0][i][j][q];
            }
        }
      } else {
        // a sample's positions are adjacent in dst but no whole 16-byte pieces (49, 729, ... of them):
        // the lanes whose TN positions lie in one sample still store them as one vector
        bool together = false;
        if (p.run_store && TN > 1 && first + TN <= ph.npos) {
          const unsigned nn = ph.by_jvol.div((unsigned)first);
          together = (unsigned)first - nn * (unsigned)jvol + (unsigned)TN <= (unsigned)jvol;
        }
        if (together) {
          typedef T OutVec __attribute__((ext_vector_type(TN), aligned(sizeof(T))));
          T *out = dst_of(first);
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int m = m0 + wm0 + Mma<T>::row_of(lane, q) * TM + i;
              if (m < p.M) {
                OutVec v;
#pragma unroll
                for (int j = 0; j < TN; ++j) v[j] = acc[0][i][j][q];
                *reinterpret_cast<OutVec *>(out + (long long)m * p.dst_mstride) = v;
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
                if (m < p.M) out[(long long)m * p.dst_mstride] = acc[0][i][j][q];
              }
          }
        }
      }
    }
  }
}

// Adds the K slices of the shared tail tiles in slice order (always the same order,
// so results repeat exactly) and stores them where the tile's epilogue would have.
// One thread per tile element; blockIdx.y is the tail tile.
template <typename T, int BM, int BN, int NPH = 1>
__global__ void __launch_bounds__(256) tail_fixup_kernel(const GemmParams p) {
  const int e = blockIdx.x * 256 + threadIdx.x;  // element of the [BM][BN] tile
  if (e >= BM * BN) return;
  // the tile, where its slices' partial sums start and how many there are
  int tile = p.full_tiles + blockIdx.y, first_slot = (int)blockIdx.y * p.tail_split, slots = p.tail_split;
  if (p.share_fix != nullptr) {
    const ShareFix fx = p.share_fix[blockIdx.y];
    tile = fx.tile, first_slot = fx.first_slot, slots = fx.slots;
  }
  const int pblk = tile / p.m_tiles;
  int pi = 0;
  while (pi + 1 < p.nphases && pblk >= p.phases[pi + 1].blk_begin) ++pi;
  const Phase ph = p.phases[pi];
  const int ipos = (pblk - ph.blk_begin) * BN + e % BN;
  const int m = (tile % p.m_tiles) * BM + e / BN;
  if (ipos >= ph.npos || m >= p.M) return;
  const int j12 = ph.J[1] * ph.J[2];
  const unsigned pos = (unsigned)ipos;
  const unsigned n = ph.by_jvol.div(pos);
  unsigned r = pos - n * (unsigned)(ph.J[0] * j12);
  const int j0 = (int)ph.by_j12.div(r);
  r -= (unsigned)j0 * (unsigned)j12;
  const int j1 = (int)ph.by_j2.div(r);
  const int j2 = (int)r - j1 * ph.J[2];
  const long long slice = (long long)NPH * BM * BN;  // elements of one K slice of a tile: one [BM][BN] per phase
  const T *slot = static_cast<const T *>(p.partial) + (long long)first_slot * slice + e;
  if (NPH == 1 && p.phase_count != 0) {
    // row m is stride phase m % phase_count of channel m / phase_count
    const int c = m / p.phase_count, f = m - c * p.phase_count;
    if (!((j0 < p.pJ[f][0]) & (j1 < p.pJ[f][1]) & (j2 < p.pJ[f][2]))) return;
    const T sum = sum_in_order(slot, slice, slots);
    T *out = static_cast<T *>(p.dst) + (long long)n * p.dst_nstride + (long long)(p.po0[f][0] + j0 * p.oj[0]) * p.os[0] +
             (long long)(p.po0[f][1] + j1 * p.oj[1]) * p.os[1] + (long long)(p.po0[f][2] + j2 * p.oj[2]) * p.os[2];
    out[(long long)c * p.dst_mstride] = sum;
    return;
  }
#pragma unroll
  for (int f = 0; f < NPH; ++f) {
    const int o0 = NPH == 1 ? ph.o0[0] : p.po0[f][0], o1 = NPH == 1 ? ph.o0[1] : p.po0[f][1], o2 = NPH == 1 ? ph.o0[2] : p.po0[f][2];
    if (NPH > 1 && !((j0 < p.pJ[f][0]) & (j1 < p.pJ[f][1]) & (j2 < p.pJ[f][2]))) continue;
    const T sum = sum_in_order(slot + (long long)f * (BM * BN), slice, slots);
    T *out = static_cast<T *>(p.dst) + (long long)n * p.dst_nstride + (long long)(o0 + j0 * p.oj[0]) * p.os[0] +
             (long long)(o1 + j1 * p.oj[1]) * p.os[1] + (long long)(o2 + j2 * p.oj[2]) * p.os[2];
    out[(long long)m * p.dst_mstride] = sum;
  }
}

// ------------------------------------------------------------------------------------------
// filter gradient
// ------------------------------------------------------------------------------------------
// WIDE: the positions of one sample are a multiple of 16 bytes, so 16 bytes of grad (4 or
// 2 consecutive positions of one filter) never straddle two samples and the grad tile
// is loaded and parked 16 bytes per lane; otherwise element by element.
// TABLE: the columns are any rows of the gather table (WgradParams::tab, one (channel, tap) each,
// in dw's own order, padded to whole tiles with rows that lie outside every input), not groups
// of 16 channels under one tap -- for channel counts that fill no group.  Every column then
// costs the gathering waves its own bounds test.
// POS (TABLE only): the columns' bounds tests come from the position table (WgradParams::pos_tab,
// which must be there) instead of the gather table's coordinate offsets; the other kernels take
// the position table whenever the plan has one.
template <typename T, int BM, int BN, int BK, int WM, int WN, bool WIDE, bool TABLE = false, bool POS = false>
__global__ void __launch_bounds__(512) tap_wgrad_kernel(const WgradParams p) {
  static_assert(TABLE || !POS, "POS selects between the two forms of the TABLE kernel");
  static_assert((BM / WM) * (BN / WN) == 4, "four wavefronts per block");
  static_assert(256 % BK == 0 && BK % 16 == 0 && BN % 16 == 0, "K tile");
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int WAVES_N = BN / WN;
  constexpr int ROWS = 256 / BK;  // tile rows covered by one pass of the block
  static_assert(16 % ROWS == 0 && BM % ROWS == 0, "row passes must not straddle a column group");
  constexpr int VEC = 16 / sizeof(T);
  constexpr int APIECES = BK / VEC;      // 16-byte pieces per row of the grad tile
  constexpr int APASS = 256 / APIECES;   // rows covered by one pass when loading pieces
  static_assert(!WIDE || BM % APASS == 0, "grad tile passes");
  constexpr int ALOADS = WIDE ? BM / APASS : BM / ROWS;
  typedef typename VecOf<T, VEC>::type AVec;
  typedef typename std::conditional<WIDE, AVec, T>::type AReg;
  constexpr int NGROUPS = BN / 16;
  // A loader thread owns one position of the K tile and one of ROWS row slots.  The
  // padding test is per (position, column group), so the slots share out the groups
  // first (GSPLIT ways) and only then the 16 channels of a group (CSPLIT ways): a
  // thread tests MYGROUPS groups per K tile and loads CLOADS channels of each.
  constexpr int GSPLIT = gcd_of(ROWS, NGROUPS);
  constexpr int MYGROUPS = NGROUPS / GSPLIT;
  constexpr int CSPLIT = ROWS / GSPLIT;
  constexpr int CLOADS = 16 / CSPLIT;
  static_assert(NGROUPS % GSPLIT == 0 && ROWS % GSPLIT == 0 && 16 % CSPLIT == 0, "loader slots");
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
  // tiles of one K split read the same positions of grad and x, so they should meet in
  // one L2.  The (split, tile) pairs, splits outermost, are cut into 8 runs of equal
  // length (to within one), one per XCD: block b is the (b/8)-th block of XCD b%8 and
  // takes the (b/8)-th pair of that XCD's run.  An XCD then works on whole splits, one
  // after the other, and shares at most the split at either end of its run with a
  // neighbour; any number of splits can be used.
  // (A single split -- a matrix product's many tiles -- keeps the plain order: neighbouring
  // tiles on neighbouring XCDs re-read less of the operands than eight long runs do.)
  const int tiles_per_split = p.col_tiles * p.row_tiles;
  const int xcd = blockIdx.x % 8, nth = blockIdx.x / 8;
  const int per_xcd = gridDim.x / 8, extra = gridDim.x % 8;
  const int pair = p.splits == 1 ? (int)blockIdx.x : xcd * per_xcd + min(xcd, extra) + nth;
  const int split = pair / tiles_per_split;
  const int tile = pair % tiles_per_split;
  const int n0 = (tile % p.col_tiles) * BN;  // first column
  const int m0 = (tile / p.col_tiles) * BM;  // first filter (F % BM == 0)
  const int kbeg = split * p.kchunk;
  const int kend = min(kbeg + p.kchunk, p.kpos);

  const __amdgpu_buffer_rsrc_t grad_buf = buffer_of<T>(p.grad, p.grad_bytes);
  const __amdgpu_buffer_rsrc_t x_buf = buffer_of<T>(p.x, p.x_bytes);
  const int kcol = tid % BK;
  const int row0 = BK % 64 == 0 ? uniform(tid / BK) : tid / BK;
  const int g12 = p.G[1] * p.G[2];

  const int gsel = row0 % GSPLIT, csel = row0 / GSPLIT;

  // the thread's column groups never change: keep their table rows in registers
  const int8v MG_CONSTANT *gtab = (const int8v MG_CONSTANT *)(p.groups) + n0 / 16;
  int8v grp[MYGROUPS];
  if constexpr (!TABLE) {
#pragma unroll
    for (int i = 0; i < MYGROUPS; ++i) grp[i] = gtab[gsel + i * GSPLIT];
  }
  // TABLE: this thread's columns (gsel + j*GSPLIT)*16 + csel + r*CSPLIT of the tile, one table row each
  constexpr int NB = MYGROUPS * CLOADS;
  int4v ent[TABLE && !POS ? NB : 1];
  // POS: a column is its element offset into x and its tap (a column past the last one: an offset
  // outside x)
  unsigned col_off[TABLE && POS ? NB : 1], col_tap[TABLE && POS ? NB : 1];
  if constexpr (TABLE) {
    const int4v MG_CONSTANT *rows = (const int4v MG_CONSTANT *)(p.tab) + n0;
#pragma unroll
    for (int j = 0; j < MYGROUPS; ++j)
#pragma unroll
      for (int r = 0; r < CLOADS; ++r) {
        const int col = (gsel + j * GSPLIT) * 16 + csel + r * CSPLIT;
        if constexpr (POS) {
          col_off[j * CLOADS + r] = n0 + col < p.CT ? (unsigned)(rows[col][0] * (int)sizeof(T)) : kOutside;
          col_tap[j * CLOADS + r] = (unsigned)((n0 + col) % p.wvol);
        } else {
          ent[j * CLOADS + r] = rows[col];
        }
      }
  }

  AReg ra0[ALOADS], ra1[ALOADS];
  T rb0[NB], rb1[NB];
  // Position table (WgradParams::pos_tab): what a position contributes to the addresses and which
  // taps it has, so that a K tile costs a table row instead of three divisions, the products with
  // the strides and a bounds test per axis.  A row is asked for one round of its register set
  // ahead and rides along in pe0 / pe1 (and, for the grad tile's own positions, pa0 / pa1).
  const bool tabled = TABLE ? POS : p.pos_tab != nullptr;
  typedef unsigned u4 __attribute__((ext_vector_type(4)));
  const __amdgpu_buffer_rsrc_t pos_buf = buffer_of<T>(p.pos_tab, tabled ? (unsigned)p.kpos * 16u : 0u);
  unsigned tap_bit[MYGROUPS], col_bytes[MYGROUPS];
  bool tap_high[MYGROUPS];
  if constexpr (!TABLE) {
#pragma unroll
    for (int i = 0; i < MYGROUPS; ++i) {
      const int tap = (n0 / 16 + gsel + i * GSPLIT) % p.wvol;
      tap_bit[i] = grp[i][4] != 0 ? 1u << (tap & 31) : 0u;
      tap_high[i] = tap >= 32;
      col_bytes[i] = (unsigned)((grp[i][0] + csel * p.x_cstride) * (int)sizeof(T));
    }
  }
  u4 pe0 = {0, 0, 0, 0}, pe1 = {0, 0, 0, 0};
  unsigned pa0 = 0, pa1 = 0;
  const unsigned a_step = (unsigned)((WIDE ? APASS : ROWS) * p.gvol) * (unsigned)sizeof(T);
  const int apiece = tid % APIECES, arow = tid / APIECES;  // WIDE: this thread's piece of the grad tile
  const unsigned b_step = (unsigned)(CSPLIT * p.x_cstride) * (unsigned)sizeof(T);

  // the table rows of K tile kt for this thread: of its own position, and (WIDE) of its grad piece
  auto ask = [&](u4 &pe, unsigned &pa, int kt) {
    const int ipos = kbeg + kt * BK + kcol;
    pe = __builtin_amdgcn_raw_buffer_load_b128(pos_buf, (ipos < kend ? ipos : kbeg) * 16, 0, 0);
    if constexpr (WIDE) {
      const int apos = kbeg + kt * BK + apiece * VEC;
      pa = __builtin_amdgcn_raw_buffer_load_b32(pos_buf, (apos < kend ? apos : kbeg) * 16 + 12, 0, 0);
    }
  };
  auto fetch_tabled = [&](AReg(&ra)[ALOADS], T(&rb)[NB], u4 &pe, unsigned &pa, int kt, int kt_next) {
    // the rows of the set's next tile first: whoever waits for them leaves this tile's loads in flight
    u4 pe_next;
    unsigned pa_next;
    ask(pe_next, pa_next, kt_next);
    const int ipos = kbeg + kt * BK + kcol;
    const bool pos_ok = ipos < kend;
    if constexpr (WIDE) {
      const int apos = kbeg + kt * BK + apiece * VEC;
      const unsigned g_at = apos < kend ? (unsigned)(apos + (m0 + arow) * p.gvol) * (unsigned)sizeof(T) + pa : kOutside;
#pragma unroll
      for (int r = 0; r < ALOADS; ++r) ra[r] = buffer_load16<T>(grad_buf, g_at, (unsigned)r * a_step);
    } else {
      const unsigned g_at = pos_ok ? (unsigned)(ipos + (m0 + row0) * p.gvol) * (unsigned)sizeof(T) + pe[3] : kOutside;
#pragma unroll
      for (int r = 0; r < ALOADS; ++r) ra[r] = buffer_load<T>(grad_buf, g_at, (unsigned)r * a_step);
    }
    if constexpr (TABLE && POS) {
      const unsigned long long taps = ((unsigned long long)pe[2] << 32) | pe[1];
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const bool ok = pos_ok & (((taps >> col_tap[i]) & 1ull) != 0ull);
        rb[i] = buffer_load<T>(x_buf, ok ? pe[0] + col_off[i] : kOutside, 0u);
      }
    } else if constexpr (!TABLE) {
#pragma unroll
      for (int j = 0; j < MYGROUPS; ++j) {
        const unsigned word = tap_high[j] ? pe[2] : pe[1];
        const bool ok = pos_ok & ((word & tap_bit[j]) != 0u);
        const unsigned at = ok ? pe[0] + col_bytes[j] : kOutside;
#pragma unroll
        for (int r = 0; r < CLOADS; ++r) rb[j * CLOADS + r] = buffer_load<T>(x_buf, at, (unsigned)r * b_step);
      }
    }
    pe = pe_next, pa = pa_next;
  };
  auto fetch = [&](AReg(&ra)[ALOADS], T(&rb)[NB], int kt) {
    if constexpr (WIDE) {
      const int apos = kbeg + kt * BK + apiece * VEC;  // the piece lies inside one sample and inside the split or not at all
      const unsigned an = p.by_gvol.div((unsigned)apos);
      const unsigned aflat = (unsigned)apos - an * (unsigned)p.gvol;
      const unsigned g_at = apos < kend ? (unsigned)((long long)an * p.g_nstride + aflat + (long long)(m0 + arow) * p.gvol) * (unsigned)sizeof(T)
                                        : kOutside;
#pragma unroll
      for (int r = 0; r < ALOADS; ++r) ra[r] = buffer_load16<T>(grad_buf, g_at, (unsigned)r * a_step);
    }
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
    if constexpr (!WIDE) {
      const unsigned g_at =
          pos_ok ? (unsigned)((long long)n * p.g_nstride + gflat + (long long)(m0 + row0) * p.gvol) * (unsigned)sizeof(T) : kOutside;
#pragma unroll
      for (int r = 0; r < ALOADS; ++r) ra[r] = buffer_load<T>(grad_buf, g_at, (unsigned)r * a_step);
    }
    const unsigned x_at = (unsigned)((long long)n * p.x_nstride + (qb0 * p.qs[0] + qb1 * p.qs[1] + qb2 * p.qs[2]) +
                                     (TABLE ? 0ll : (long long)csel * p.x_cstride)) * (unsigned)sizeof(T);
    if constexpr (TABLE && !POS) {
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const int4v e = ent[i];  // off, d0, d1, d2
        const bool ok = pos_ok & ((unsigned)(qb0 + e[1]) < (unsigned)p.Q[0]) & ((unsigned)(qb1 + e[2]) < (unsigned)p.Q[1]) &
                        ((unsigned)(qb2 + e[3]) < (unsigned)p.Q[2]);
        rb[i] = buffer_load<T>(x_buf, ok ? x_at + (unsigned)(e[0] * (int)sizeof(T)) : kOutside, 0u);
      }
    } else if constexpr (!TABLE) {
#pragma unroll
      for (int j = 0; j < MYGROUPS; ++j) {
        const int8v e = grp[j];  // coff, d0, d1, d2, valid
        const bool ok = pos_ok & (e[4] != 0) & ((unsigned)(qb0 + e[1]) < (unsigned)p.Q[0]) &
                        ((unsigned)(qb1 + e[2]) < (unsigned)p.Q[1]) & ((unsigned)(qb2 + e[3]) < (unsigned)p.Q[2]);
        const unsigned at = ok ? x_at + (unsigned)(e[0] * (int)sizeof(T)) : kOutside;
#pragma unroll
        for (int r = 0; r < CLOADS; ++r) rb[j * CLOADS + r] = buffer_load<T>(x_buf, at, (unsigned)r * b_step);
      }
    }
  };
  auto stash = [&](const AReg(&ra)[ALOADS], const T(&rb)[NB], int buf) {
#pragma unroll
    for (int r = 0; r < ALOADS; ++r) {
      if constexpr (WIDE)
        *reinterpret_cast<AVec *>(&As[buf][arow + r * APASS][apiece * VEC]) = ra[r];
      else
        As[buf][row0 + r * ROWS][kcol] = ra[r];
    }
#pragma unroll
    for (int j = 0; j < MYGROUPS; ++j)
#pragma unroll
      for (int r = 0; r < CLOADS; ++r) Bs[buf][(gsel + j * GSPLIT) * 16 + csel + r * CSPLIT][kcol] = rb[j * CLOADS + r];
  };

  const int ktiles = kend > kbeg ? (kend - kbeg + BK - 1) / BK : 0;
  if (loader) {
    // tile i travels in register set i % 2 and lands in LDS buffer i % 2; the loads
    // of every path are the same (see tap_gemm_kernel), tiles past the end are clamped
    const int last = ktiles - 1;
    if (tabled) {
      // the same schedule with the table rows one round ahead: set 0 takes tiles 0, 2, 4, ...,
      // set 1 tiles 1, 3, 5, ... (each clamped to the last)
      if (ktiles > 0) {
        ask(pe0, pa0, 0);
        ask(pe1, pa1, min(1, last));
        fetch_tabled(ra0, rb0, pe0, pa0, 0, min(2, last));
        stash(ra0, rb0, 0);
        fetch_tabled(ra1, rb1, pe1, pa1, min(1, last), min(3, last));
        fetch_tabled(ra0, rb0, pe0, pa0, min(2, last), min(4, last));
      }
      __syncthreads();
      int kt = 0;
      for (; kt + 1 < ktiles; kt += 2) {
        stash(ra1, rb1, 1);
        fetch_tabled(ra1, rb1, pe1, pa1, min(kt + 3, last), min(kt + 5, last));
        __syncthreads();
        stash(ra0, rb0, 0);
        fetch_tabled(ra0, rb0, pe0, pa0, min(kt + 4, last), min(kt + 6, last));
        __syncthreads();
      }
      if (kt < ktiles) __syncthreads();
      return;
    }
    if (ktiles > 0) {
      fetch(ra0, rb0, 0);
      stash(ra0, rb0, 0);
      fetch(ra1, rb1, min(1, last));
      fetch(ra0, rb0, min(2, last));
    }
    __syncthreads();
    int kt = 0;
    for (; kt + 1 < ktiles; kt += 2) {
      stash(ra1, rb1, 1);
      fetch(ra1, rb1, min(kt + 3, last));
      __syncthreads();
      stash(ra0, rb0, 0);
      fetch(ra0, rb0, min(kt + 4, last));
      __syncthreads();
    }
    if (kt < ktiles) __syncthreads();
    return;
  }
  // The MFMA waves go ahead of the gathering waves on their SIMD whenever both have an
  // instruction ready (measured: the double-precision filter gradient 163 -> 156 us, float
  // 158 -> 154 us; the same setting in tap_gemm_kernel changed nothing for the convolutions
  // and cost a 4096^3 matrix product 4 %, so it is not set there).
  __builtin_amdgcn_s_setprio(3);

  if constexpr (sizeof(T) == 8) {
    // 4x4x4 four-block MFMAs on 8-row x 8-column patches (see Quad); quarter-wave lk
    // contracts the K indices lk*KQ .. lk*KQ+KQ-1, four adjacent ones per LDS read
    constexpr int GM = WM / 8, GN = WN / 8;
    const int arow = wm0 + Quad::feed_row(l16);
    const int bcol8 = wn0 + Quad::feed_col(l16);
    const int drow = wm0 + Quad::held_row(l16, lk);
    double acc[GM][GN];
#pragma unroll
    for (int i = 0; i < GM; ++i)
#pragma unroll
      for (int j = 0; j < GN; ++j) acc[i][j] = 0.0;
    __syncthreads();
    int buf = 0;
    for (int kt = 0; kt < ktiles; ++kt) {
#pragma unroll
      for (int s4 = 0; s4 < KQ / 4; ++s4) {
        T a[GM][4], b[GN][4];
#pragma unroll
        for (int i = 0; i < GM; ++i) {
          const T *src = &As[buf][arow + i * 8][lk * KQ + s4 * 4];
          T lo[2], hi[2];
          load_vec<T, 2>(src, lo);
          load_vec<T, 2>(src + 2, hi);
          a[i][0] = lo[0], a[i][1] = lo[1], a[i][2] = hi[0], a[i][3] = hi[1];
        }
#pragma unroll
        for (int j = 0; j < GN; ++j) {
          const T *src = &Bs[buf][bcol8 + j * 8][lk * KQ + s4 * 4];
          T lo[2], hi[2];
          load_vec<T, 2>(src, lo);
          load_vec<T, 2>(src + 2, hi);
          b[j][0] = lo[0], b[j][1] = lo[1], b[j][2] = hi[0], b[j][3] = hi[1];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int i = 0; i < GM; ++i)
#pragma unroll
            for (int j = 0; j < GN; ++j) acc[i][j] = Quad::run(a[i][u], b[j][u], acc[i][j]);
      }
      __syncthreads();
      buf ^= 1;
    }
    T *__restrict__ out = static_cast<T *>(p.out) + (long long)split * p.F * p.CT;
#pragma unroll
    for (int j = 0; j < GN; ++j) {
      const int col = n0 + bcol8 + j * 8;
      if (col >= p.CT) continue;
#pragma unroll
      for (int i = 0; i < GM; ++i) {
        const int f = m0 + drow + i * 8;
        if (f < p.F) out[(long long)f * p.CT + col] = acc[i][j];
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

// dw[f][c][t] = the sum over K splits of part[s][f][col], where the columns run over
// channel blocks of 16, then taps, then the channel inside the block:
// col = ((c/16) * wvol + t) * 16 + c%16.
// The splits are cut into RUNS runs (1 or 4); wave q of the block adds run q in split
// order for 256 / RUNS consecutive elements, and the run sums are added in run order:
// always the same association for a given plan, so the result repeats exactly.  Four
// runs put four times the loads in flight, which pays when dw is too small to fill
// the device with one thread per element.
template <typename T, int RUNS>
__global__ void __launch_bounds__(256) tap_reduce_kernel(const T *__restrict__ part, T *__restrict__ dw, int F, int C,
                                                         int wvol, int splits) {
  constexpr int WIDTH = 256 / RUNS;
  __shared__ T runs[4][64];
  const int count = F * C * wvol;
  const int q = threadIdx.x / WIDTH, lane = threadIdx.x % WIDTH;
  // Threads run through the partial sums' own layout, so a wave reads consecutive
  // addresses of every split (the few stores to dw are the scattered side).
  const int src = blockIdx.x * WIDTH + lane;  // index into one split: f * C*wvol + column
  const int per = (splits + RUNS - 1) / RUNS;
  const int first = min(q * per, splits), last = min(first + per, splits);
  T sum = T(0);
  int i = count;  // index into dw
  if (src < count) {
    const int ct = C * wvol;
    const int f = src / ct;
    const int col = src - f * ct;
    const int group = col / 16;  // (channel block, tap)
    const int cb = group / wvol, t = group - cb * wvol;
    i = f * ct + (cb * 16 + col % 16) * wvol + t;
    if (first < last) sum = sum_in_order(part + (long long)first * count + src, count, last - first);
  }
  if constexpr (RUNS == 1) {
    if (i < count) dw[i] = sum;
    return;
  }
  runs[q][lane] = sum;
  __syncthreads();
  if (q == 0 && i < count) {
    // runs past the last split are empty and hold +0.0; adding them changes nothing
    // except that a total of -0.0 would read +0.0, which a sum of products starting
    // from +0.0 accumulators cannot be
    dw[i] = ((runs[0][lane] + runs[1][lane]) + runs[2][lane]) + runs[3][lane];
  }
}

}  // namespace mg
