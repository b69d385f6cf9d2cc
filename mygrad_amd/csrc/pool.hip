// Max-pool forward and backward (gather form) for gfx950.
//
// Index algebra (rank padded to 3, row-major):
//   out[l, g]  = max_a x[l, g*S + a]                      a in prod [0, P_k)
//   dx[l, i]  += grad[l, g]  for every window g whose first-occurrence argmax
//                (row-major inside the window; the first NaN if any) is i,
//                windows taken in ascending row-major order, sum started at
//                +0.0 and carried in double.
#include "internal.h"

#include <cstdlib>

#include <algorithm>
#include <optional>

namespace mg {

struct PoolParams {
  int X[3], P[3], S[3], G[3];
  long long lead, xvol, gvol;
};

// `cand` replaces `best` when it is the first NaN, or strictly greater than a
// non-NaN best: ties keep the earlier element, a NaN once met is never replaced.
template <typename T>
__device__ __forceinline__ bool takes_over(T cand, T best) {
  return (best == best) && !(cand <= best);  // "not <=" is true for cand > best and for a NaN cand
}

// MARK (here and below): also record, one byte per window, where its maximum sits:
// the row-major offset (a0 * P1 + a1) * P2 + a2 of the first-occurrence argmax inside
// the window.  The backward pass can then route gradients without reading x again.
template <typename T, bool MARK>
__global__ void __launch_bounds__(256) maxpool_fwd_kernel(PoolParams p, const T *__restrict__ x,
                                                          T *__restrict__ out, unsigned char *__restrict__ mark) {
  const long long total = p.lead * p.gvol;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const long long l = idx / p.gvol;
    int r = (int)(idx - l * p.gvol);
    const int g2 = r % p.G[2];
    r /= p.G[2];
    const int g1 = r % p.G[1];
    const int g0 = r / p.G[1];
    const T *w = x + l * p.xvol + ((long long)(g0 * p.S[0]) * p.X[1] + g1 * p.S[1]) * p.X[2] + g2 * p.S[2];
    T best = w[0];
    int code = 0;
    for (int a0 = 0; a0 < p.P[0]; ++a0)
      for (int a1 = 0; a1 < p.P[1]; ++a1) {
        const T *row = w + ((long long)a0 * p.X[1] + a1) * p.X[2];
        for (int a2 = 0; a2 < p.P[2]; ++a2) {
          const T v = row[a2];
          if (takes_over(v, best)) {
            best = v;
            code = (a0 * p.P[1] + a1) * p.P[2] + a2;
          }
        }
      }
    if (out) out[idx] = best;  // null: only the argmax offsets are wanted
    if constexpr (MARK) mark[idx] = (unsigned char)code;
  }
}

template <typename T, typename TD>
__global__ void __launch_bounds__(256) maxpool_bwd_kernel(PoolParams p, const T *__restrict__ x,
                                                          const T *__restrict__ grad, TD *__restrict__ dx) {
  const long long total = p.lead * p.xvol;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const long long l = idx / p.xvol;
    const int me = (int)(idx - l * p.xvol);
    int r = me;
    const int i2 = r % p.X[2];
    r /= p.X[2];
    const int i1 = r % p.X[1];
    const int i0 = r / p.X[1];
    const int i[3] = {i0, i1, i2};
    int lo[3], hi[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const int first = i[k] - p.P[k] + 1;  // smallest window origin/S that still covers i
      lo[k] = first > 0 ? (first + p.S[k] - 1) / p.S[k] : 0;
      hi[k] = min(p.G[k] - 1, i[k] / p.S[k]);
    }
    const T *xp = x + l * p.xvol;
    const T *gp = grad + l * p.gvol;
    double acc = 0.0;
    for (int g0 = lo[0]; g0 <= hi[0]; ++g0)
      for (int g1 = lo[1]; g1 <= hi[1]; ++g1)
        for (int g2 = lo[2]; g2 <= hi[2]; ++g2) {
          const int origin = ((g0 * p.S[0]) * p.X[1] + g1 * p.S[1]) * p.X[2] + g2 * p.S[2];
          T best = xp[origin];
          int where = origin;
          for (int a0 = 0; a0 < p.P[0]; ++a0)
            for (int a1 = 0; a1 < p.P[1]; ++a1) {
              const int rowoff = origin + (a0 * p.X[1] + a1) * p.X[2];
              for (int a2 = 0; a2 < p.P[2]; ++a2) {
                const T v = xp[rowoff + a2];
                if (takes_over(v, best)) {
                  best = v;
                  where = rowoff + a2;
                }
              }
            }
          if (where == me) acc += (double)gp[(g0 * p.G[1] + g1) * p.G[2] + g2];
        }
    dx[idx] = (TD)acc;
  }
}

// ------------------------------------------------------------------------------------------
// LDS-tiled kernels
//
// A block stages one contiguous chunk of x in LDS with wide coalesced loads --
// either a band of rows of one pooled volume plus the halo its windows need, or
// several whole small volumes -- so that every element of x crosses HBM once.
// Forward: each thread then reduces windows out of LDS.  Backward: the block first
// records every window's first-occurrence argmax (as an LDS index), then each
// thread owns input elements and walks the few windows that cover them in
// ascending row-major order, adding grad where the window's argmax is the
// element itself: a gather, so no atomics, and the sum order of np.add.at.
// ------------------------------------------------------------------------------------------
struct FastDivP {
  unsigned mul, shr, d, pad_;
  __device__ __forceinline__ unsigned div(unsigned n) const { return d == 1u ? n : __umulhi(n, mul) >> shr; }
};

static FastDivP make_fastdiv_p(unsigned d) {
  FastDivP f{0u, 0u, d, 0u};
  if (d > 1u) {
    unsigned lg = 0;
    while ((1ull << lg) < d) ++lg;
    const unsigned p = 31u + lg;
    f.mul = (unsigned)(((1ull << p) + d - 1ull) / d);
    f.shr = p - 32u;
  }
  return f;
}

struct PoolTileParams {
  int X[3], P[3], S[3], G[3];
  int axis;     // first pooled axis with extent > 1: the one that is cut into bands
  int inner_x;  // elements of x per unit of that axis
  int inner_g;  // windows per unit of that axis
  int band;     // forward: windows per band; backward: input rows owned per band
  int bands;    // bands per volume (1 when a block takes whole volumes)
  int volumes;  // whole volumes per block (1 when a volume is cut into bands)
  int xvol, gvol;
  long long lead;
  FastDivP by_x12, by_x2, by_g12, by_g2, by_xvol, by_gvol;
  FastDivP by_s[3];
  FastDivP by_p12, by_p2;  // a recorded argmax offset back to (a0, a1, a2)
  int cand[3];  // windows that can cover one element, per axis: ceil(P/S)
  int nranks;   // their product
};

// What one block-iteration works on: a contiguous chunk of x and the windows in it.
struct TileGeom {
  long long l0;           // first leading index
  long long chunk_start;  // element offset of the chunk in x
  long long gstart;       // element offset of the windows' run in grad / out
  int nvol;               // whole volumes in the chunk (1 when a volume is cut into bands)
  int own_lo, own_hi;     // rows of the band axis this tile writes (backward)
  int first_flat;         // flat index inside a volume of chunk element 0
  int chunk_len;          // elements of x staged
  int pad;                // chunk_start % VEC: shift that aligns LDS and global together
  int nwin, win_base;     // windows evaluated; flat window index of the first
  int gpad;               // gstart % VEC
};

template <typename T, bool BWD>
__device__ __forceinline__ TileGeom tile_geom(const PoolTileParams &p, long long blk) {
  constexpr int VEC = 16 / sizeof(T);
  TileGeom t;
  t.l0 = (blk / p.bands) * p.volumes;
  const int band = (int)(blk % p.bands);
  t.nvol = (int)min((long long)p.volumes, p.lead - t.l0);
  const int a = p.axis;
  const int XA = p.X[a], GA = p.G[a], PA = p.P[a], SA = p.S[a];
  // rows [own_lo, own_hi) are written (backward); windows [g_lo, g_hi] along the band
  // axis are evaluated; rows [row_lo, row_hi) are what those windows and rows read
  int own_lo = 0, own_hi = XA, g_lo = 0, g_hi = GA - 1;
  if (p.bands > 1) {
    if (BWD) {
      own_lo = band * p.band;
      own_hi = min(own_lo + p.band, XA);
      const int first = own_lo - PA + 1;
      g_lo = first > 0 ? (first + SA - 1) / SA : 0;
      g_hi = min(GA - 1, (own_hi - 1) / SA);
    } else {
      g_lo = band * p.band;
      g_hi = min(g_lo + p.band, GA) - 1;
    }
  }
  const bool any_window = g_lo <= g_hi;
  int row_lo, row_hi;
  if (BWD) {
    row_lo = any_window ? min(own_lo, g_lo * SA) : own_lo;
    row_hi = any_window ? max(own_hi, g_hi * SA + PA) : own_hi;
  } else {
    row_lo = g_lo * SA;
    row_hi = g_hi * SA + PA;
  }
  t.own_lo = own_lo;
  t.own_hi = own_hi;
  t.first_flat = row_lo * p.inner_x;
  t.chunk_len = p.bands > 1 ? (row_hi - row_lo) * p.inner_x : t.nvol * p.xvol;
  t.chunk_start = t.l0 * p.xvol + t.first_flat;
  t.pad = (int)(t.chunk_start % VEC);
  t.nwin = any_window ? (p.bands > 1 ? (g_hi - g_lo + 1) * p.inner_g : t.nvol * p.gvol) : 0;
  t.win_base = p.bands > 1 ? g_lo * p.inner_g : 0;
  t.gstart = t.l0 * p.gvol + t.win_base;
  t.gpad = (int)(t.gstart % VEC);
  return t;
}

// A chunk on its way from global memory to LDS.  issue() sends DEPTH 16-byte loads per
// thread and returns at once; commit() stores what came back, and moves whatever the
// registers did not cover (the unaligned head and tail, anything beyond DEPTH) directly.
// tile[pad + e] = src[start + e], with pad = start % VEC so both sides align together.
template <typename T, int DEPTH>
struct ChunkInFlight {
  static constexpr int VEC = 16 / sizeof(T);
  typedef T Vec __attribute__((ext_vector_type(VEC)));
  Vec held[DEPTH];
  T edge;  // threads 0 .. VEC-2: one element of the unaligned head; the next VEC-1 threads: one of the tail

  __device__ __forceinline__ static int head_of(int len, int pad) { return min(len, (VEC - pad) % VEC); }

  __device__ __forceinline__ void issue(const T *__restrict__ src, long long start, int len, int pad) {
    const int head = head_of(len, pad);
    const int body = (len - head) / VEC;
    const Vec *vsrc = reinterpret_cast<const Vec *>(src + start + head);
    // clamped, never predicated: a load behind a branch would wait for the one before it
    const int last = max(body - 1, 0);
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) held[u] = vsrc[min(u * 256 + (int)threadIdx.x, last)];
    // the elements before the first and after the last whole vector travel with them,
    // one per thread, instead of being fetched when the chunk is parked
    const int t = (int)threadIdx.x;
    const int e = t < VEC - 1 ? t : head + body * VEC + (t - (VEC - 1));
    edge = src[start + min(e, max(len - 1, 0))];
  }

  __device__ __forceinline__ void commit(T *tile, const T *__restrict__ src, long long start, int len, int pad) {
    const int head = head_of(len, pad);
    const int body = (len - head) / VEC;
    Vec *vdst = reinterpret_cast<Vec *>(tile + pad + head);
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const int v = u * 256 + (int)threadIdx.x;
      if (v < body) vdst[v] = held[u];
    }
    const Vec *vsrc = reinterpret_cast<const Vec *>(src + start + head);
    for (int v = DEPTH * 256 + (int)threadIdx.x; v < body; v += 256) vdst[v] = vsrc[v];
    const int t = (int)threadIdx.x;
    if (t < VEC - 1) {
      if (t < head) tile[pad + t] = edge;
    } else if (t < 2 * (VEC - 1)) {
      const int e = head + body * VEC + (t - (VEC - 1));
      if (e < len) tile[pad + e] = edge;
    }
  }
};

// Persistent blocks: each walks tiles blk, blk + gridDim.x, ...  While a tile is being
// processed out of LDS, the next tile's x (and grad) are already on their way into
// registers, so the memory system always has this block's next 16-48 KB in flight.
// PSIG names a pool extent known at compile time, P0*100 + P1*10 + P2 (each 1..3), whose
// window scan is fully unrolled: all its LDS reads are issued before the first compare
// instead of one read-compare round trip per element; 0 = any extent, looped.
// FROM_MARK (backward only): x is neither loaded nor scanned; each window's argmax comes from
// the byte a MARK forward pass recorded, staged through LDS at mark_offset like the gradients.
template <typename T, typename TD, typename ACC, bool BWD, int DEPTH, int PSIG, bool MARK = false,
          bool FROM_MARK = false>
__global__ void __launch_bounds__(256) maxpool_tile_kernel(PoolTileParams p, const T *__restrict__ x,
                                                           const T *__restrict__ grad, void *__restrict__ result,
                                                           long long ntiles, int tile_elems, int win_slots,
                                                           int acc_offset, unsigned char *__restrict__ mark = nullptr,
                                                           int mark_offset = 0) {
  static_assert(!FROM_MARK || BWD, "only the backward pass reads recorded positions");
  // LDS: [x tile | one packed int per window | grad of those windows | accumulators];
  // win_slots is a multiple of 4.  The accumulators alias the x tile (acc_offset == 0)
  // when they are no wider than T: x is dead once every window knows its argmax.
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T *tile = reinterpret_cast<T *>(smem);
  int *winner = reinterpret_cast<int *>(smem + (size_t)tile_elems * sizeof(T));
  T *gtile = reinterpret_cast<T *>(smem + (size_t)tile_elems * sizeof(T) + (size_t)win_slots * sizeof(int));
  ACC *acc = reinterpret_cast<ACC *>(smem + acc_offset);
  unsigned char *mtile = smem + mark_offset;
  constexpr int GDEPTH = 2;
  const int x12 = p.X[1] * p.X[2], g12 = p.G[1] * p.G[2];

  ChunkInFlight<T, DEPTH> xin;
  ChunkInFlight<T, GDEPTH> gin;
  ChunkInFlight<unsigned char, 1> marks_in;
  long long blk = blockIdx.x;
  if (blk >= ntiles) return;
  TileGeom t = tile_geom<T, BWD>(p, blk);
  if constexpr (FROM_MARK)
    marks_in.issue(mark, t.gstart, t.nwin, (int)(t.gstart % 16));
  else
    xin.issue(x, t.chunk_start, t.chunk_len, t.pad);
  if (BWD) gin.issue(grad, t.gstart, t.nwin, t.gpad);

  for (; blk < ntiles; blk += gridDim.x) {
    const int mpad = (int)(t.gstart % 16);
    if constexpr (FROM_MARK)
      marks_in.commit(mtile, mark, t.gstart, t.nwin, mpad);
    else
      xin.commit(tile, x, t.chunk_start, t.chunk_len, t.pad);
    if (BWD) gin.commit(gtile, grad, t.gstart, t.nwin, t.gpad);
    __syncthreads();

    // next tile: loads go out now and land while this tile is processed
    const long long nblk = blk + gridDim.x;
    TileGeom tn = t;
    if (nblk < ntiles) {
      tn = tile_geom<T, BWD>(p, nblk);
      if constexpr (FROM_MARK)
        marks_in.issue(mark, tn.gstart, tn.nwin, (int)(tn.gstart % 16));
      else
        xin.issue(x, tn.chunk_start, tn.chunk_len, tn.pad);
      if (BWD) gin.issue(grad, tn.gstart, tn.nwin, tn.gpad);
    }

    // ---- one thread per window: the maximum (forward) or where it is (backward)
    for (int w = threadIdx.x; w < t.nwin; w += 256) {
      const unsigned vol = p.by_gvol.div((unsigned)w);  // 0 when a volume is cut into bands
      const unsigned wf = (unsigned)w - vol * (unsigned)p.gvol + (unsigned)t.win_base;
      const unsigned g0 = p.by_g12.div(wf);
      const unsigned r = wf - g0 * (unsigned)g12;
      const unsigned g1 = p.by_g2.div(r);
      const unsigned g2 = r - g1 * (unsigned)p.G[2];
      const int origin = (int)((g0 * p.S[0] * p.X[1] + g1 * p.S[1]) * p.X[2] + g2 * p.S[2]) - t.first_flat +
                         (int)vol * p.xvol + t.pad;
      T best = FROM_MARK ? T(0) : tile[origin];
      int where = origin;
      int code = 0;  // the argmax as an offset inside the window (what MARK records)
      if constexpr (FROM_MARK) {
        const unsigned recorded = mtile[mpad + w];
        unsigned a0, a1, a2;
        if constexpr (PSIG != 0) {
          constexpr unsigned Q1 = (PSIG / 10) % 10, Q2 = PSIG % 10;
          a0 = recorded / (Q1 * Q2);
          a1 = (recorded - a0 * Q1 * Q2) / Q2;
          a2 = recorded - (a0 * Q1 + a1) * Q2;
        } else {
          a0 = p.by_p12.div(recorded);
          const unsigned r12 = recorded - a0 * (unsigned)(p.P[1] * p.P[2]);
          a1 = p.by_p2.div(r12);
          a2 = r12 - a1 * (unsigned)p.P[2];
        }
        where = origin + (int)((a0 * p.X[1] + a1) * p.X[2] + a2);
      } else if constexpr (PSIG != 0) {
        constexpr int Q0 = PSIG / 100, Q1 = (PSIG / 10) % 10, Q2 = PSIG % 10;
        T v[Q0 * Q1 * Q2];
#pragma unroll
        for (int a0 = 0; a0 < Q0; ++a0)
#pragma unroll
          for (int a1 = 0; a1 < Q1; ++a1)
#pragma unroll
            for (int a2 = 0; a2 < Q2; ++a2) v[(a0 * Q1 + a1) * Q2 + a2] = tile[origin + (a0 * p.X[1] + a1) * p.X[2] + a2];
#pragma unroll
        for (int a0 = 0; a0 < Q0; ++a0)
#pragma unroll
          for (int a1 = 0; a1 < Q1; ++a1)
#pragma unroll
            for (int a2 = 0; a2 < Q2; ++a2) {
              const T c = v[(a0 * Q1 + a1) * Q2 + a2];
              if (takes_over(c, best)) {
                best = c;
                where = origin + (a0 * p.X[1] + a1) * p.X[2] + a2;
                code = (a0 * Q1 + a1) * Q2 + a2;
              }
            }
      } else {
        for (int a0 = 0; a0 < p.P[0]; ++a0)
          for (int a1 = 0; a1 < p.P[1]; ++a1) {
            const int rowoff = origin + (a0 * p.X[1] + a1) * p.X[2];
            for (int a2 = 0; a2 < p.P[2]; ++a2) {
              const T v = tile[rowoff + a2];
              if (takes_over(v, best)) {
                best = v;
                where = rowoff + a2;
                code = (a0 * p.P[1] + a1) * p.P[2] + a2;
              }
            }
          }
      }
      if (BWD) {
        // Rank of this window among the windows that cover its argmax element, in
        // ascending row-major window order: per axis min(g, (P-1-a)/S) with a the
        // argmax's offset inside the window.  Two windows with the same argmax
        // element never share a rank, and adding ranks 0, 1, 2, ... in turn is the
        // order np.add.at visits them in.
        const unsigned off = (unsigned)(where - origin);
        const unsigned a0 = p.by_x12.div(off);
        const unsigned r12 = off - a0 * (unsigned)x12;
        const unsigned a1 = p.by_x2.div(r12);
        const unsigned a2 = r12 - a1 * (unsigned)p.X[2];
        const unsigned k0 = min(g0, p.by_s[0].div((unsigned)p.P[0] - 1u - a0));
        const unsigned k1 = min(g1, p.by_s[1].div((unsigned)p.P[1] - 1u - a1));
        const unsigned k2 = min(g2, p.by_s[2].div((unsigned)p.P[2] - 1u - a2));
        const unsigned rank = (k0 * (unsigned)p.cand[1] + k1) * (unsigned)p.cand[2] + k2;
        winner[w] = where | (int)(rank << 20);
      } else {
        static_cast<T *>(result)[t.gstart + w] = best;
        if constexpr (MARK) mark[t.gstart + w] = (unsigned char)code;
      }
    }

    if (BWD) {
      __syncthreads();
      // ---- accumulators start at +0.0 (they may sit where the x tile was)
      // in 16-byte stores; the round-up stays inside the tile's own LDS region
      const int used = t.chunk_len + t.pad;
      {
        constexpr int VA = 16 / sizeof(ACC);
        typedef ACC AVec __attribute__((ext_vector_type(VA), aligned(16)));
        AVec zero;
#pragma unroll
        for (int i = 0; i < VA; ++i) zero[i] = ACC(0);
        AVec *vacc = reinterpret_cast<AVec *>(acc);
        const int nvec = (used + VA - 1) / VA;
        for (int v = threadIdx.x; v < nvec; v += 256) vacc[v] = zero;
      }
      __syncthreads();

      // ---- one pass per rank: every window of that rank adds its gradient to its
      // argmax element.  Within a pass no two windows touch the same element, so plain
      // LDS read-modify-writes are race-free; across passes the barrier orders them.
      for (int rank = 0; rank < p.nranks; ++rank) {
        for (int w = threadIdx.x; w < t.nwin; w += 256) {
          const int packed = winner[w];
          if ((packed >> 20) == rank) {
            const int e = packed & 0xFFFFF;
            acc[e] = acc[e] + (ACC)gtile[t.gpad + w];
          }
        }
        __syncthreads();
      }

      // ---- write the rows this tile owns
      const int own_first = p.bands > 1 ? t.own_lo * p.inner_x : 0;
      const int own_len = p.bands > 1 ? (t.own_hi - t.own_lo) * p.inner_x : t.nvol * p.xvol;
      const int shift = own_first - t.first_flat + t.pad;
      // in 16-byte stores: dx index and LDS index are congruent modulo a 16-byte load
      // of x (that is what pad is for), hence also modulo a 16-byte store of dx
      constexpr int VD = 16 / sizeof(TD);
      typedef TD DVec __attribute__((ext_vector_type(VD)));
      constexpr int AALIGN = VD * sizeof(ACC) < 16 ? VD * sizeof(ACC) : 16;
      typedef ACC SVec __attribute__((ext_vector_type(VD), aligned(AALIGN)));
      const long long d0 = t.l0 * p.xvol + own_first;
      TD *dx = static_cast<TD *>(result) + d0;
      const int head = min(own_len, (VD - (int)(d0 % VD)) % VD);
      const int body = (own_len - head) / VD;
      DVec *vdx = reinterpret_cast<DVec *>(dx + head);
      const SVec *from = reinterpret_cast<const SVec *>(acc + shift + head);
      for (int v = threadIdx.x; v < body; v += 256) {
        const SVec a = from[v];
        DVec d;
#pragma unroll
        for (int i = 0; i < VD; ++i) d[i] = (TD)a[i];
        vdx[v] = d;
      }
      for (int e = threadIdx.x; e < head; e += 256) dx[e] = (TD)acc[e + shift];
      for (int e = head + body * VD + (int)threadIdx.x; e < own_len; e += 256) dx[e] = (TD)acc[e + shift];
    }
    __syncthreads();  // LDS is about to be overwritten by the next tile
    t = tn;
  }
}

// ------------------------------------------------------------------------------------------
// Windows that tile the input exactly (stride == pool extent, X == G * P on every axis):
// every element belongs to exactly one window, so nothing is staged or accumulated.  A
// thread takes one 16-byte piece of a row for each of the P0 x P1 rows of a window
// slab -- 16 / (P2 * sizeof(T)) whole windows -- straight from global memory, reduces
// them in registers and stores 16-byte pieces of dx (or its share of out).  Consecutive
// lanes take consecutive pieces: every access of a wave is one contiguous run.
// float32 rows that are whole 8-byte but not whole 16-byte pieces (14, 30, ... columns under
// two-column windows) take pieces of 8 bytes, one window wide (VEC = 2).
// ------------------------------------------------------------------------------------------
struct PoolExactParams {
  int X1, X2;            // extents of the two inner pooled axes
  int G0, G1;            // windows along the two outer pooled axes
  int vec;               // elements per piece: 16 bytes, or 8 bytes for float32 rows of 4k + 2 columns
  int pieces;            // pieces per row of x
  long long xvol, gvol;  // elements of x / windows per leading index
  long long total;       // work items: lead * G0 * G1 * pieces
  FastDivP by_pieces, by_g1, by_g0;
};

template <typename T, typename TD, int P0, int P1, int P2, bool BWD, bool MARK = false, int VEC = 16 / sizeof(T)>
__global__ void __launch_bounds__(256) maxpool_exact_kernel(PoolExactParams p, const T *__restrict__ x,
                                                            const T *__restrict__ grad, void *__restrict__ result,
                                                            unsigned char *__restrict__ mark = nullptr) {
  constexpr int WPT = VEC / P2;  // windows per thread
  static_assert(VEC % P2 == 0 && WPT >= 1, "a piece holds whole windows");
  typedef T Vec __attribute__((ext_vector_type(VEC)));
  typedef T WVec __attribute__((ext_vector_type(WPT)));
  const long long item = (long long)blockIdx.x * 256 + threadIdx.x;
  // with MARK every thread stays for the block-wide store of the recorded bytes: a thread
  // past the end works on the last item again and stores nothing
  const bool live = item < p.total;
  if (!MARK && !live) return;
  // item -> (leading index, g0, g1, piece); total < 2^32 is checked by the host
  const unsigned u = (unsigned)(live ? item : p.total - 1);
  const unsigned q1 = p.by_pieces.div(u), piece = u - q1 * (unsigned)p.pieces;
  const unsigned q2 = p.by_g1.div(q1), g1 = q1 - q2 * (unsigned)p.G1;
  const unsigned lead = p.by_g0.div(q2), g0 = q2 - lead * (unsigned)p.G0;
  const long long xrow0 = (long long)lead * p.xvol + ((long long)(g0 * P0) * p.X1 + g1 * P1) * p.X2 + piece * VEC;
  Vec v[P0][P1];
#pragma unroll
  for (int a0 = 0; a0 < P0; ++a0)
#pragma unroll
    for (int a1 = 0; a1 < P1; ++a1) v[a0][a1] = *reinterpret_cast<const Vec *>(x + xrow0 + ((long long)a0 * p.X1 + a1) * p.X2);
  const long long w0 = (long long)lead * p.gvol + ((long long)g0 * p.G1 + g1) * (p.pieces * WPT) + piece * WPT;
  // first-occurrence maximum (the first NaN if any) of each window, row-major inside it
  T best[WPT];
  int where[WPT];
#pragma unroll
  for (int j = 0; j < WPT; ++j) {
    best[j] = v[0][0][j * P2];
    where[j] = 0;
#pragma unroll
    for (int a0 = 0; a0 < P0; ++a0)
#pragma unroll
      for (int a1 = 0; a1 < P1; ++a1)
#pragma unroll
        for (int a2 = 0; a2 < P2; ++a2) {
          const T c = v[a0][a1][j * P2 + a2];
          if (takes_over(c, best[j])) {
            best[j] = c;
            where[j] = (a0 * P1 + a1) * P2 + a2;
          }
        }
  }
  if constexpr (!BWD) {
    WVec o;
#pragma unroll
    for (int j = 0; j < WPT; ++j) o[j] = best[j];
    if (live) *reinterpret_cast<WVec *>(static_cast<T *>(result) + w0) = o;
    if constexpr (MARK) {
      // The windows of item i are windows i * WPT ... of the whole tensor, so a block's
      // bytes are one contiguous run: gathered in LDS and stored 16 at a time.
      __shared__ __attribute__((aligned(16))) unsigned char stage[256 * WPT];
#pragma unroll
      for (int j = 0; j < WPT; ++j) stage[threadIdx.x * WPT + j] = (unsigned char)where[j];
      __syncthreads();
      const long long run0 = (long long)blockIdx.x * 256 * WPT, run_end = p.total * WPT;
      const int at = (int)threadIdx.x * 16;
      if (at < 256 * WPT) {
        if (run0 + at + 16 <= run_end) {
          *reinterpret_cast<uint4 *>(mark + run0 + at) = *reinterpret_cast<const uint4 *>(stage + at);
        } else {
          for (int b = 0; b < 16 && run0 + at + b < run_end; ++b) mark[run0 + at + b] = stage[at + b];
        }
      }
    }
  } else {
    const WVec g = *reinterpret_cast<const WVec *>(grad + w0);
    typedef TD DVec __attribute__((ext_vector_type(VEC)));
    TD *dx = static_cast<TD *>(result);
#pragma unroll
    for (int a0 = 0; a0 < P0; ++a0)
#pragma unroll
      for (int a1 = 0; a1 < P1; ++a1) {
        DVec d;
#pragma unroll
        for (int j = 0; j < WPT; ++j)
#pragma unroll
          for (int a2 = 0; a2 < P2; ++a2) {
            // the one window's gradient added to +0.0 (so -0.0 becomes +0.0), or +0.0
            const TD term = (TD)(T(0) + g[j]);
            d[j * P2 + a2] = where[j] == (a0 * P1 + a1) * P2 + a2 ? term : TD(0);
          }
        *reinterpret_cast<DVec *>(dx + xrow0 + ((long long)a0 * p.X1 + a1) * p.X2) = d;
      }
  }
}

// ------------------------------------------------------------------------------------------
// Backward from the argmax positions a MARK forward pass recorded: x is not read again.
// A thread owns VD consecutive elements of dx (one 16-byte store).  Each element walks the
// windows that cover it in ascending row-major order and adds grad where the window's
// recorded offset is the element's own offset inside that window: the order and the
// +0.0 start of np.add.at, carried in double and rounded once.
// ------------------------------------------------------------------------------------------
struct PoolMarkParams {
  int X[3], P[3], S[3], G[3];
  int xvol, gvol, x12;
  int leads;        // leading indices per blockIdx.y: leads * xvol < 2^31
  long long lead;   // leading indices in all
  FastDivP by_xvol, by_x12, by_x2, by_s[3];
};

template <typename T, typename TD, int VD>
__global__ void __launch_bounds__(256) maxpool_from_mark_kernel(PoolMarkParams p, const unsigned char *__restrict__ mark,
                                                                const T *__restrict__ grad, TD *__restrict__ dx) {
  const long long lead0 = (long long)blockIdx.y * p.leads;
  const unsigned here = (unsigned)min((long long)p.leads, p.lead - lead0) * (unsigned)p.xvol;  // elements in this slice
  const unsigned first = (blockIdx.x * 256u + threadIdx.x) * (unsigned)VD;
  if (first >= here) return;
  const unsigned l = p.by_xvol.div(first);
  unsigned r = first - l * (unsigned)p.xvol;
  int i0 = (int)p.by_x12.div(r);
  r -= (unsigned)i0 * (unsigned)p.x12;
  int i1 = (int)p.by_x2.div(r);
  int i2 = (int)r - i1 * p.X[2];
  const unsigned char *m = mark + (lead0 + l) * p.gvol;
  const T *g = grad + (lead0 + l) * p.gvol;

  // windows g_k in [lo, hi] cover coordinate i along axis k
  auto lo_of = [&](int k, int i) { return i >= p.P[k] ? (int)p.by_s[k].div((unsigned)(i - p.P[k] + p.S[k])) : 0; };
  auto hi_of = [&](int k, int i) { return min(p.G[k] - 1, (int)p.by_s[k].div((unsigned)i)); };
  int lo0 = lo_of(0, i0), hi0 = hi_of(0, i0), lo1 = lo_of(1, i1), hi1 = hi_of(1, i1);

  TD vals[VD];
#pragma unroll
  for (int v = 0; v < VD; ++v) {
    double acc = 0.0;
    if (first + v < here) {
      const int lo2 = lo_of(2, i2), hi2 = hi_of(2, i2);
      for (int g0 = lo0; g0 <= hi0; ++g0)
        for (int g1 = lo1; g1 <= hi1; ++g1) {
          const int row = (g0 * p.G[1] + g1) * p.G[2];
          const int mine01 = ((i0 - g0 * p.S[0]) * p.P[1] + (i1 - g1 * p.S[1])) * p.P[2];
          for (int g2 = lo2; g2 <= hi2; ++g2)
            if ((int)m[row + g2] == mine01 + (i2 - g2 * p.S[2])) acc += (double)g[row + g2];
        }
      // the next element: along the row, wrapping into the next row / plane / leading index
      if (++i2 == p.X[2]) {
        i2 = 0;
        if (++i1 == p.X[1]) {
          i1 = 0;
          if (++i0 == p.X[0]) {
            i0 = 0;
            m += p.gvol;
            g += p.gvol;
          }
          lo0 = lo_of(0, i0);
          hi0 = hi_of(0, i0);
        }
        lo1 = lo_of(1, i1);
        hi1 = hi_of(1, i1);
      }
    }
    vals[v] = (TD)acc;
  }
  TD *to = dx + lead0 * p.xvol + first;
  if (VD > 1 && first + VD <= here) {
    typedef TD DVec __attribute__((ext_vector_type(VD)));
    DVec d;
#pragma unroll
    for (int v = 0; v < VD; ++v) d[v] = vals[v];
    *reinterpret_cast<DVec *>(to) = d;
  } else {
#pragma unroll
    for (int v = 0; v < VD; ++v)
      if (first + v < here) to[v] = vals[v];
  }
}

// Forward pass for windows whose extent and step are known at compile time (P0 x P1 x P2 placed
// every S0, S1, S2; P0 = S0 = 1 for windows over the last two axes), straight from global memory.
// Lane l of a wavefront takes the l-th 16-byte piece of a window row's P1 rows of x -- consecutive
// lanes, consecutive pieces: every load of the wavefront is one contiguous run -- in each of the
// window's P0 planes, one after the other, and reduces the VEC / S2 windows that start inside its
// piece.  The P2 - S2 columns those reach beyond the piece come from the next lane by a
// cross-lane move, not from memory; the last lane of a wavefront only supplies them (the next
// wavefront starts on its piece again).  A window that would need columns of the next row does
// not exist.  Rows and planes that two windows share are loaded by both (the second time out of
// L1 / L2: the items that share them run next to each other); nothing is staged.
// Pieces are counted in columns, not in addresses: a row need not start on a 16-byte boundary
// (the loads only assume the alignment of an element), and a row that is no whole number of
// pieces ends in a short one of `tail` columns.  The lane of a short piece loads the last VEC
// columns of the row instead and moves its own to the front, so no load leaves the row; what is
// then behind them belongs to no window.  An exact window grid over 3 x 3 windows placed every
// other column always has an odd last extent, i.e. such rows.
// Needs VEC % S2 == 0, P2 - S2 <= VEC and X2 >= VEC.
#define POOL_ROWS_PER_THREAD 3
struct PoolRowsParams {
  int X0, X1, X2, G0, G1, G2;
  int pieces;        // 16-byte pieces per row of x, the short one included
  int tail;          // columns of the short piece (X2 % VEC); 0: none
  int groups;        // groups of POOL_ROWS_PER_THREAD window rows per window plane
  long long planes;  // lead * G0: window planes
  long long items;   // planes * groups * pieces: one per (group of window rows, piece)
  FastDivP by_pieces, by_groups, by_g0;
};

template <typename T>
__device__ __forceinline__ T from_next_lane(T value) {
  return __shfl_down(value, 1, 64);
}

// Blocks are handed to the 8 XCDs round-robin, and each XCD has its own L2.  Neighbouring work
// items share rows and planes of x (windows overlap) and entries of the record, so the blocks
// b, b + 8, ... of one XCD take consecutive runs of items: block b is the (b / 8)-th block of XCD
// b % 8 and takes the (b / 8)-th run of that XCD's eighth of the work.
__device__ __forceinline__ unsigned xcd_run(unsigned block, unsigned blocks) {
  const unsigned xcd = block % 8u, nth = block / 8u;
  const unsigned per = blocks / 8u, extra = blocks % 8u;
  return xcd * per + min(xcd, extra) + nth;
}

template <typename T, int P0, int P1, int P2, int S0, int S1, int S2, bool MARK, bool STORE_OUT = true>
__global__ void __launch_bounds__(256) maxpool_rows_fwd_kernel(PoolRowsParams p, const T *__restrict__ x, T *__restrict__ out,
                                                              unsigned char *__restrict__ mark) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int WO = VEC / S2;   // windows that start inside a piece
  constexpr int HALO = P2 - S2;  // columns the last of them reaches into the next piece
  constexpr int RW = POOL_ROWS_PER_THREAD;   // window rows per thread: the rows two of them share are loaded once
  constexpr int NR = (RW - 1) * S1 + P1;     // rows of x under them
  static_assert(VEC % S2 == 0 && HALO >= 0 && HALO <= VEC, "piece / window geometry");
  typedef T Vec __attribute__((ext_vector_type(VEC), aligned(sizeof(T))));
  const int lane = threadIdx.x & 63;
  const long long wave = (long long)xcd_run(blockIdx.x, gridDim.x) * 4 + (threadIdx.x >> 6);
  const long long item = wave * 63 + lane;  // wavefronts overlap by one lane
  const unsigned u = (unsigned)(item < p.items ? item : p.items - 1);  // clamped: every lane loads, some do not store
  const unsigned q = p.by_pieces.div(u), piece = u - q * (unsigned)p.pieces;
  const unsigned plane = p.by_groups.div(q);  // window plane: (leading index, g0)
  const int g1_first = (int)(q - plane * (unsigned)p.groups) * RW;
  const unsigned lead = p.by_g0.div(plane);
  const long long xplane = (long long)lead * p.X0 + (long long)(plane - lead * (unsigned)p.G0) * S0;  // the first plane of x under the window plane
  const bool short_piece = p.tail != 0 && (int)piece == p.pieces - 1;
  const T *rows = x + xplane * p.X1 * p.X2 + (short_piece ? p.X2 - VEC : (int)piece * VEC);
  const int row_first = g1_first * S1;
  const bool idle = lane == 63 || item >= p.items;  // supplies its neighbour's columns only

  T best[RW][WO];
  int code[RW][WO];
#pragma unroll
  for (int a0 = 0; a0 < P0; ++a0) {
    T v[NR][VEC + HALO];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      // rows beyond the last one belong to window rows that do not exist: read the last row instead
      const Vec mine = *reinterpret_cast<const Vec *>(rows + ((long long)a0 * p.X1 + min(row_first + r, p.X1 - 1)) * p.X2);
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[r][i] = mine[i];
    }
    if (p.tail != 0) {
      // a short piece's own columns are the last `tail` of what it loaded
#pragma unroll
      for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int i = 0; i < VEC - 1; ++i) {
          T moved = v[r][i];
#pragma unroll
          for (int k = i + 1; k < VEC; ++k)
            if (p.tail == k) moved = v[r][i + VEC - k];
          v[r][i] = short_piece ? moved : v[r][i];
        }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
      for (int i = 0; i < HALO; ++i) v[r][VEC + i] = from_next_lane(v[r][i]);
#pragma unroll
    for (int w = 0; w < RW; ++w)
#pragma unroll
      for (int t = 0; t < WO; ++t) {
        if (a0 == 0) {
          best[w][t] = v[w * S1][t * S2];
          code[w][t] = 0;
        }
#pragma unroll
        for (int a1 = 0; a1 < P1; ++a1)
#pragma unroll
          for (int a2 = 0; a2 < P2; ++a2) {
            const T c = v[w * S1 + a1][t * S2 + a2];
            if (takes_over(c, best[w][t])) {
              best[w][t] = c;
              code[w][t] = (a0 * P1 + a1) * P2 + a2;
            }
          }
      }
  }
  if (idle) return;
#pragma unroll
  for (int w = 0; w < RW; ++w) {
    const int g1 = g1_first + w;
    if (g1 >= p.G1) break;
    const long long w0 = ((long long)plane * p.G1 + g1) * p.G2 + (long long)piece * WO;
    // the piece's windows are neighbours in out and in the record: one store each when all exist
    if (WO > 1 && (int)piece * WO + WO <= p.G2) {
      if constexpr (STORE_OUT) {
        typedef T OVec __attribute__((ext_vector_type(WO), aligned(sizeof(T))));
        OVec o;
#pragma unroll
        for (int t = 0; t < WO; ++t) o[t] = best[w][t];
        *reinterpret_cast<OVec *>(out + w0) = o;
      }
      if constexpr (MARK) {
        typedef unsigned char CVec __attribute__((ext_vector_type(WO), aligned(1)));
        CVec c;
#pragma unroll
        for (int t = 0; t < WO; ++t) c[t] = (unsigned char)code[w][t];
        *reinterpret_cast<CVec *>(mark + w0) = c;
      }
    } else {
#pragma unroll
      for (int t = 0; t < WO; ++t)
        if ((int)piece * WO + t < p.G2) {
          if constexpr (STORE_OUT) out[w0 + t] = best[w][t];
          if constexpr (MARK) mark[w0 + t] = (unsigned char)code[w][t];
        }
    }
  }
}

// The same gather for windows whose extent and step are known at compile time (P0 x P1 x P2
// placed every S0, S1, S2; P0 = S0 = 1 for windows over the last two axes).  A thread owns a
// 16-byte piece of S1 consecutive rows in S0 consecutive planes of dx: the rows k1*S1 ..
// k1*S1 + S1 - 1 are covered by the same ceil(P1/S1) window rows (the planes by the same
// ceil(P0/S0) window planes), and the piece's columns by the same ceil(P2/S2) - 1 + VD/S2 windows
// along the row, whichever thread -- so their recorded offsets and gradients are loaded up front
// (never predicated: a window that does not exist is loaded from a neighbour's place and
// masked), and every element adds, in ascending window order, the gradient of the windows whose
// recorded offset names it: no loop bounds to compute, no divisions by runtime values, no LDS.
// Needs VD % S2 == 0 (a piece starts on a window boundary) and at least pool_gather_run() windows
// per row.
// Pieces are counted in columns: rows of dx need not start on 16-byte boundaries (the stores only
// assume the alignment of an element), and the short piece at the end of a row that is no whole
// number of pieces is stored element by element.
struct PoolGatherParams {
  int X0, X1, X2, G0, G1, G2;
  int pieces;        // 16-byte pieces per row of dx, the short one included
  int tail;          // columns of the short piece (X2 % VD); 0: none
  int groups;        // groups of S1 rows per plane: ceil(X1 / S1)
  int groups0;       // groups of S0 planes per leading index: ceil(X0 / S0)
  long long planes;  // lead * groups0
  int leads;         // leading positions: each has G0 * G1 * G2 windows
  FastDivP by_pieces, by_groups, by_groups0;
};

// acc += term on the lanes where code == wanted; the others keep acc (adding +0.0 to a sum that
// started at +0.0 would leave it as it is, too).  The comparison narrows the execution mask for the
// one addition, which takes half the vector instructions of two selects and an addition; the mask
// is put back before the statement ends.
__device__ __forceinline__ void add_where_equal(double &acc, double term, int code, int wanted) {
  unsigned long long all;
  asm("s_mov_b64 %1, exec\n\tv_cmpx_eq_u32_e32 vcc, %4, %3\n\tv_add_f64 %0, %0, %2\n\ts_mov_b64 exec, %1"
      : "+v"(acc), "=&s"(all)
      : "v"(term), "v"(code), "s"(wanted)
      : "vcc");
}

template <typename T, typename TD, int P0, int P1, int P2, int S0, int S1, int S2>
__global__ void __launch_bounds__(256) maxpool_mark_gather_kernel(PoolGatherParams p, const unsigned char *__restrict__ mark,
                                                                 const T *__restrict__ grad, TD *__restrict__ dx) {
  constexpr int VD = 16 / sizeof(TD);
  constexpr int C0 = (P0 + S0 - 1) / S0, C1 = (P1 + S1 - 1) / S1, C2 = (P2 + S2 - 1) / S2;
  constexpr int NW2 = (VD - 1) / S2 + C2;  // windows along the row that can reach the piece
  constexpr int LW = NW2 <= 2 ? 2 : NW2 <= 4 ? 4 : 8;  // windows loaded per window row
  static_assert(VD % S2 == 0 && NW2 <= 8, "a piece starts on a window boundary");
  typedef TD DVec __attribute__((ext_vector_type(VD), aligned(sizeof(TD))));
  typedef unsigned char CVec __attribute__((ext_vector_type(LW), aligned(1)));
  typedef T GVec __attribute__((ext_vector_type(LW), aligned(sizeof(T))));
  struct Where {  // an item: the piece `piece` of the rows k1 * S1 ... in the planes k0 * S0 ... of leading position `lead`
    unsigned lead;
    int k0, k1, piece;
  };
  struct Asked {  // the windows that can reach it, as loaded
    CVec lc[C0][C1];
    GVec lg[C0][C1];
  };
  const long long total = p.planes * p.groups * p.pieces;
  const int gvol = p.G0 * p.G1 * p.G2;
  const auto where_of = [&](long long item) {
    const unsigned u = (unsigned)item;
    const unsigned q = p.by_pieces.div(u);
    const unsigned plane = p.by_groups.div(q);  // (leading index, group of S0 planes)
    Where w;
    w.piece = (int)(u - q * (unsigned)p.pieces);
    w.k1 = (int)(q - plane * (unsigned)p.groups);
    w.lead = p.by_groups0.div(plane);
    w.k0 = (int)(plane - w.lead * (unsigned)p.groups0);
    return w;
  };
  // The NW2 windows of a window row are neighbours in the record and in grad: LW of them (a power
  // of two that holds NW2) come as one load each, starting at the first window wanted.  That one
  // may lie before the row and the last ones beyond it: what is loaded there belongs to
  // neighbouring rows and is masked (such windows do not exist), and only at the two ends of the
  // whole record does the run have to move inside -- by `shift`, and the window wanted at place e
  // is then the loaded one at place e + shift.  Returns where the run starts in the leading
  // position's part of the record.
  const auto run_start = [&](const Where &w, int d0, int d, int &shift, bool &exists) {
    const int g0 = w.k0 - (C0 - 1) + d0, g1 = w.k1 - (C1 - 1) + d, g2_first = w.piece * VD / S2 - (C2 - 1);
    exists = (g0 >= 0) & (g0 < p.G0) & (g1 >= 0) & (g1 < p.G1);
    const int wanted = (min(max(g0, 0), p.G0 - 1) * p.G1 + min(max(g1, 0), p.G1 - 1)) * p.G2 + g2_first;
    const int lowest = w.lead == 0 ? 0 : -LW, highest = (int)w.lead == p.leads - 1 ? gvol - LW : gvol;
    const int r = min(max(wanted, lowest), highest);
    shift = wanted - r;
    return r;
  };
  const auto ask = [&](const Where &w, Asked &a) {
    const unsigned char *m = mark + (long long)w.lead * gvol;
    const T *g = grad + (long long)w.lead * gvol;
#pragma unroll
    for (int d0 = 0; d0 < C0; ++d0)
#pragma unroll
      for (int d = 0; d < C1; ++d) {
        int shift;
        bool exists;
        const int r = run_start(w, d0, d, shift, exists);
        a.lc[d0][d] = *reinterpret_cast<const CVec *>(m + r);
        a.lg[d0][d] = *reinterpret_cast<const GVec *>(g + r);
      }
  };
  const auto finish = [&](const Where &w, const Asked &a) {
    const int i2 = w.piece * VD, g2_first = i2 / S2 - (C2 - 1);
    const int live = (p.tail != 0 && w.piece == p.pieces - 1) ? p.tail : VD;  // columns of this piece
    int code[C0][C1][NW2];
    double term[C0][C1][NW2];
    int shift[C0][C1];
    bool exists[C0][C1];
    int moved = 0;
#pragma unroll
    for (int d0 = 0; d0 < C0; ++d0)
#pragma unroll
      for (int d = 0; d < C1; ++d) {
        run_start(w, d0, d, shift[d0][d], exists[d0][d]);
        moved |= shift[d0][d];
#pragma unroll
        for (int e = 0; e < NW2; ++e) {
          const int g2 = g2_first + e;
          const bool ok = exists[d0][d] & (g2 >= 0) & (g2 < p.G2);
          code[d0][d][e] = ok ? (int)a.lc[d0][d][e] : -1;  // a window that does not exist names no element
          term[d0][d][e] = (double)a.lg[d0][d][e];
        }
      }
    if (moved != 0) {  // some of the first and the last threads of the grid only
#pragma unroll
      for (int d0 = 0; d0 < C0; ++d0)
#pragma unroll
        for (int d = 0; d < C1; ++d)
#pragma unroll
          for (int e = 0; e < NW2; ++e) {
            const int g2 = g2_first + e;
            const bool ok = exists[d0][d] & (g2 >= 0) & (g2 < p.G2);
            int c = -1;
            T t = T(0);
#pragma unroll
            for (int k = 0; k < LW; ++k) {
              const bool here = e + shift[d0][d] == k;
              c = here ? (int)a.lc[d0][d][k] : c;
              t = here ? a.lg[d0][d][k] : t;
            }
            code[d0][d][e] = ok ? c : -1;
            term[d0][d][e] = (double)t;
          }
    }
    TD *to = dx + (((long long)w.lead * p.X0 + (long long)w.k0 * S0) * p.X1 + (long long)w.k1 * S1) * p.X2 + i2;
#pragma unroll
    for (int pp = 0; pp < S0; ++pp) {
      if (w.k0 * S0 + pp >= p.X0) break;
#pragma unroll
      for (int rr = 0; rr < S1; ++rr) {
        if (w.k1 * S1 + rr >= p.X1) break;
        DVec out;
#pragma unroll
        for (int v = 0; v < VD; ++v) {
          double acc = 0.0;
#pragma unroll
          for (int d0 = 0; d0 < C0; ++d0) {
            const int a0 = pp + (C0 - 1 - d0) * S0;  // the plane's offset inside window plane d0: known at compile time
            if (a0 >= P0) continue;
#pragma unroll
            for (int d = 0; d < C1; ++d) {
              const int a1 = rr + (C1 - 1 - d) * S1;  // the row's offset inside window row d
              if (a1 >= P1) continue;                 // that window row does not reach this row
#pragma unroll
              for (int e = 0; e < C2; ++e) {
                const int wd = v / S2 + e;                    // which of the loaded windows
                const int a2 = (v % S2) + (C2 - 1 - e) * S2;  // the element's offset inside it
                if (a2 >= P2) continue;
                add_where_equal(acc, term[d0][d][wd], code[d0][d][wd], (a0 * P1 + a1) * P2 + a2);
              }
            }
          }
          out[v] = (TD)acc;
        }
        TD *row = to + ((long long)pp * p.X1 + rr) * p.X2;
        if (live == VD) {
          *reinterpret_cast<DVec *>(row) = out;
        } else {
#pragma unroll
          for (int v = 0; v < VD - 1; ++v)
            if (v < live) row[v] = out[v];
        }
      }
    }
  };

  const long long item = (long long)xcd_run(blockIdx.x, gridDim.x) * 256 + threadIdx.x;
  if (item >= total) return;
  const Where w = where_of(item);
  Asked a;
  ask(w, a);
  finish(w, a);
}

// The same for windows that tile the input exactly: an element belongs to one window, so a
// thread reads the recorded offsets and gradients of its 16 / (P2 * sizeof(T)) windows and
// writes their P0 x P1 rows of dx.
template <typename T, typename TD, int P0, int P1, int P2, int VEC = 16 / sizeof(T)>
__global__ void __launch_bounds__(256) maxpool_exact_from_mark_kernel(PoolExactParams p,
                                                                      const unsigned char *__restrict__ mark,
                                                                      const T *__restrict__ grad, TD *__restrict__ dx) {
  constexpr int WPT = VEC / P2;
  static_assert(VEC % P2 == 0 && WPT >= 1, "a piece holds whole windows");
  typedef T WVec __attribute__((ext_vector_type(WPT)));
  typedef TD DVec __attribute__((ext_vector_type(VEC)));
  const long long item = (long long)blockIdx.x * 256 + threadIdx.x;
  if (item >= p.total) return;
  const unsigned u = (unsigned)item;
  const unsigned q1 = p.by_pieces.div(u), piece = u - q1 * (unsigned)p.pieces;
  const unsigned q2 = p.by_g1.div(q1), g1 = q1 - q2 * (unsigned)p.G1;
  const unsigned lead = p.by_g0.div(q2), g0 = q2 - lead * (unsigned)p.G0;
  const long long xrow0 = (long long)lead * p.xvol + ((long long)(g0 * P0) * p.X1 + g1 * P1) * p.X2 + piece * VEC;
  const long long w0 = (long long)lead * p.gvol + ((long long)g0 * p.G1 + g1) * (p.pieces * WPT) + piece * WPT;
  const WVec g = *reinterpret_cast<const WVec *>(grad + w0);
  int where[WPT];
#pragma unroll
  for (int j = 0; j < WPT; ++j) where[j] = (int)mark[w0 + j];
#pragma unroll
  for (int a0 = 0; a0 < P0; ++a0)
#pragma unroll
    for (int a1 = 0; a1 < P1; ++a1) {
      DVec d;
#pragma unroll
      for (int j = 0; j < WPT; ++j)
#pragma unroll
        for (int a2 = 0; a2 < P2; ++a2) {
          const TD term = (TD)(T(0) + g[j]);  // added to +0.0, so -0.0 becomes +0.0
          d[j * P2 + a2] = where[j] == (a0 * P1 + a1) * P2 + a2 ? term : TD(0);
        }
      *reinterpret_cast<DVec *>(dx + xrow0 + ((long long)a0 * p.X1 + a1) * p.X2) = d;
    }
}

// ------------------------------------------------------------------------------------------
// Pooling over four or five axes runs as two stages: the last three axes first (`inner`: every
// leading position pooled on its own), then the leading pooled axes over the merged grid of the
// first stage (`outer`: windows of one element along that merged axis).  Both stages record where
// each of their windows found its maximum, and together the two records name the element of x a
// whole window routes its gradient to: the first stage's byte inside the leading position that
// the second stage's byte picks.  A thread owns one element of dx and walks the whole windows
// that cover it in ascending row-major order -- windows along the leading axes outermost, as
// np.add.at visits them (pooling.py:147-148) -- adding grad where both records name the
// element: one sequential sum from +0.0, carried in double, the reference's order bit for bit.
// (Routing stage by stage adds a leading position's windows first and the positions afterwards:
// the same terms, another association.)
// ------------------------------------------------------------------------------------------
struct PoolStagedParams {
  int X[3], P[3], S[3], G[3];      // inner stage: the last three pooled axes
  int OX[2], OP[2], OS[2], OG[2];  // second stage: the two pooled axes in front of them (extent 1 where there is none)
  int RX[2], RP[2], RS[2], RG[2];  // third stage: the two in front of those (all ones without a third stage)
  int xvol, gvol;                  // elements of x / windows per leading position of the inner stage
  long long total;                 // elements of dx
  FastDivP by_xvol, by_x12, by_x2, by_ox1, by_ox01, by_rx1, by_rx01, by_s[3], by_os[2], by_rs[2];
};

// With six or seven pooled axes there is a third stage over the merged grid of the first two
// (`third_mark`, else null): three records name the element, and its windows along the two
// foremost axes are the outermost loops.
template <typename T, typename TD>
__global__ void __launch_bounds__(256) maxpool_staged_gather_kernel(PoolStagedParams p, const unsigned char *__restrict__ inner_mark,
                                                                   const unsigned char *__restrict__ outer_mark,
                                                                   const unsigned char *__restrict__ third_mark,
                                                                   const T *__restrict__ grad, TD *__restrict__ dx) {
  for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < p.total; idx += (long long)gridDim.x * 256) {
    // element -> (leading index, q0, q1 | i0, i1, i2); leading positions fit 32 bits (checked by the host)
    const unsigned pos = (unsigned)(idx / p.xvol);  // (leading index, q0, q1)
    unsigned r = (unsigned)(idx - (long long)pos * p.xvol);
    const int i0 = (int)p.by_x12.div(r);
    r -= (unsigned)i0 * (unsigned)(p.X[1] * p.X[2]);
    const int i1 = (int)p.by_x2.div(r);
    const int i2 = (int)r - i1 * p.X[2];
    const unsigned lead = p.by_ox01.div(pos);  // (leading index, r0, r1): the second stage's leading position
    const unsigned q01 = pos - lead * (unsigned)(p.OX[0] * p.OX[1]);
    const int q0 = (int)p.by_ox1.div(q01), q1 = (int)q01 - q0 * p.OX[1];
    const unsigned lead3 = p.by_rx01.div(lead);  // the third stage's leading position
    const unsigned r01 = lead - lead3 * (unsigned)(p.RX[0] * p.RX[1]);
    const int r0 = (int)p.by_rx1.div(r01), r1 = (int)r01 - r0 * p.RX[1];
    const int i[3] = {i0, i1, i2}, q[2] = {q0, q1}, rr[2] = {r0, r1};
    int lo[3], hi[3], olo[2], ohi[2], rlo[2], rhi[2];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      lo[k] = i[k] >= p.P[k] ? (int)p.by_s[k].div((unsigned)(i[k] - p.P[k] + p.S[k])) : 0;
      hi[k] = min(p.G[k] - 1, (int)p.by_s[k].div((unsigned)i[k]));
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      olo[k] = q[k] >= p.OP[k] ? (int)p.by_os[k].div((unsigned)(q[k] - p.OP[k] + p.OS[k])) : 0;
      ohi[k] = min(p.OG[k] - 1, (int)p.by_os[k].div((unsigned)q[k]));
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      rlo[k] = rr[k] >= p.RP[k] ? (int)p.by_rs[k].div((unsigned)(rr[k] - p.RP[k] + p.RS[k])) : 0;
      rhi[k] = min(p.RG[k] - 1, (int)p.by_rs[k].div((unsigned)rr[k]));
    }
    const unsigned char *m1 = inner_mark + (long long)pos * p.gvol;
    const long long ovol = (long long)p.OG[0] * p.OG[1] * p.gvol;  // windows of the first two stages per leading position of the third
    double acc = 0.0;
    for (int k0 = rlo[0]; k0 <= rhi[0]; ++k0)
      for (int k1 = rlo[1]; k1 <= rhi[1]; ++k1) {
        const int mine_third = (r0 - k0 * p.RS[0]) * p.RP[1] + (r1 - k1 * p.RS[1]);
        const long long trow = (((long long)lead3 * p.RG[0] + k0) * p.RG[1] + k1) * ovol;  // into the third record and grad
        for (int h0 = olo[0]; h0 <= ohi[0]; ++h0)
          for (int h1 = olo[1]; h1 <= ohi[1]; ++h1) {
            const int mine_outer = (q0 - h0 * p.OS[0]) * p.OP[1] + (q1 - h1 * p.OS[1]);
            const long long orow = (((long long)lead * p.OG[0] + h0) * p.OG[1] + h1) * p.gvol;  // into the second record
            const long long grow = trow + ((long long)h0 * p.OG[1] + h1) * p.gvol;            // (= orow without a third stage)
            for (int g0 = lo[0]; g0 <= hi[0]; ++g0)
              for (int g1 = lo[1]; g1 <= hi[1]; ++g1) {
                const int row = (g0 * p.G[1] + g1) * p.G[2];
                const int mine01 = ((i0 - g0 * p.S[0]) * p.P[1] + (i1 - g1 * p.S[1])) * p.P[2];
                for (int g2 = lo[2]; g2 <= hi[2]; ++g2) {
                  const bool here = (int)m1[row + g2] == mine01 + (i2 - g2 * p.S[2]) && (int)outer_mark[orow + row + g2] == mine_outer &&
                                    (third_mark == nullptr || (int)third_mark[grow + row + g2] == mine_third);
                  if (here) acc += (double)grad[grow + row + g2];
                }
              }
          }
      }
    dx[idx] = (TD)acc;
  }
}

static int check_pool_desc(const mg_pool_desc *d, PoolParams *p) {
  if (!d) return fail(MG_ERR_BAD_ARG, "pool descriptor is null");
  if (d->dtype != MG_F32 && d->dtype != MG_F64)
    return fail(MG_ERR_UNSUPPORTED, "pool dtype %d (only float32=0 / float64=1)", d->dtype);
  if (d->dx_dtype != d->dtype && d->dx_dtype != MG_F64)
    return fail(MG_ERR_UNSUPPORTED, "pool dx_dtype %d with dtype %d", d->dx_dtype, d->dtype);
  if (d->nd < 1 || d->nd > MG_MAX_ND) return fail(MG_ERR_UNSUPPORTED, "pooled rank %d (1..%d)", d->nd, MG_MAX_ND);
  if (d->lead < 1) return fail(MG_ERR_BAD_ARG, "lead = %lld", (long long)d->lead);
  long long xvol = 1, gvol = 1;
  for (int k = 0; k < 3; ++k) {
    if (d->X[k] < 1 || d->P[k] < 1 || d->S[k] < 1 || d->G[k] < 1)
      return fail(MG_ERR_BAD_ARG, "axis %d: X=%lld P=%lld S=%lld G=%lld must all be positive", k,
                  (long long)d->X[k], (long long)d->P[k], (long long)d->S[k], (long long)d->G[k]);
    if (k < 3 - d->nd && (d->X[k] != 1 || d->P[k] != 1 || d->S[k] != 1 || d->G[k] != 1))
      return fail(MG_ERR_BAD_ARG, "axis %d lies outside rank %d and must be all ones", k, d->nd);
    if (d->P[k] > d->X[k] || d->G[k] > (d->X[k] - d->P[k]) / d->S[k] + 1)
      return fail(MG_ERR_BAD_ARG, "axis %d: G=%lld exceeds (X-P)/S+1 = %lld", k, (long long)d->G[k],
                  (long long)((d->X[k] - d->P[k]) / d->S[k] + 1));
    xvol *= d->X[k];
    gvol *= d->G[k];
    if (xvol >= (1ll << 31)) return fail(MG_ERR_UNSUPPORTED, "pooled volume of one leading index exceeds 2^31");
    p->X[k] = (int)d->X[k];
    p->P[k] = (int)d->P[k];
    p->S[k] = (int)d->S[k];
    p->G[k] = (int)d->G[k];
  }
  p->lead = d->lead;
  p->xvol = xvol;
  p->gvol = gvol;
  return MG_OK;
}

// LDS the tiled kernels may use per block: small enough for several blocks per
// compute unit (160 KB each), large enough for whole 2-D planes of common sizes.
static const int kTileBudgetBytes = 48 * 1024;

// Chooses bands / volumes per block; returns false when not even one row of the
// band axis plus its halo fits (the thread-per-element kernels handle that).
static bool plan_tiles(const PoolParams &pp, size_t elem, size_t acc_elem, bool bwd, PoolTileParams *t,
                       int *tile_elems, int *win_slots, int *acc_offset, size_t *lds_bytes, long long *blocks) {
  // accumulators wider than an element of x cannot reuse the x tile
  const size_t acc_extra = (bwd && acc_elem > elem) ? acc_elem : 0;
  PoolTileParams q{};
  int a = 0;
  while (a < 2 && pp.X[a] == 1) ++a;
  for (int k = 0; k < 3; ++k) {
    q.X[k] = pp.X[k];
    q.P[k] = pp.P[k];
    q.S[k] = pp.S[k];
    q.G[k] = pp.G[k];
  }
  q.axis = a;
  q.inner_x = 1;
  q.inner_g = 1;
  for (int k = a + 1; k < 3; ++k) {
    q.inner_x *= pp.X[k];
    q.inner_g *= pp.G[k];
  }
  q.xvol = (int)pp.xvol;
  q.gvol = (int)pp.gvol;
  q.lead = pp.lead;
  const int vec = (int)(16 / elem);
  // backward keeps, per window, an argmax slot (int) and its gradient (one element)
  const long long per_win = bwd ? 4 + (long long)elem : 0;
  const long long per_x = (long long)(elem + acc_extra);
  const long long per_vol = (long long)pp.xvol * per_x + pp.gvol * per_win;
  long long tile = 0, nwin = 0;
  if (per_vol + 64 <= kTileBudgetBytes) {
    // whole volumes: as many as fit, but keep enough blocks to fill the device
    long long fit = (kTileBudgetBytes - 64) / per_vol;
    const long long want_blocks = 8ll * runtime().props.multiProcessorCount;
    const long long spread = std::max<long long>(1, pp.lead / want_blocks);
    q.volumes = (int)std::max<long long>(1, std::min<long long>(std::min(fit, spread), 64));
    q.bands = 1;
    q.band = bwd ? pp.X[a] : pp.G[a];
    tile = (long long)q.volumes * pp.xvol;
    nwin = (long long)q.volumes * pp.gvol;
    *blocks = ceil_div(pp.lead, q.volumes);
  } else {
    q.volumes = 1;
    const int P = pp.P[a], S = pp.S[a], XA = pp.X[a], GA = pp.G[a];
    // rows of x and windows a band needs, exactly as the kernel derives them
    auto need = [&](int band, long long *rows, long long *wins) {
      *rows = 0;
      *wins = 0;
      const int count = (int)ceil_div(bwd ? XA : GA, band);
      for (int b = 0; b < count; ++b) {
        int g_lo, g_hi, row_lo, row_hi;
        if (bwd) {
          const int own_lo = b * band, own_hi = std::min(own_lo + band, XA);
          const int first = own_lo - P + 1;
          g_lo = first > 0 ? (first + S - 1) / S : 0;
          g_hi = std::min(GA - 1, (own_hi - 1) / S);
          const bool any = g_lo <= g_hi;
          row_lo = any ? std::min(own_lo, g_lo * S) : own_lo;
          row_hi = any ? std::max(own_hi, g_hi * S + P) : own_hi;
          if (any) *wins = std::max<long long>(*wins, (long long)(g_hi - g_lo + 1) * q.inner_g);
        } else {
          g_lo = b * band;
          g_hi = std::min(g_lo + band, GA) - 1;
          row_lo = g_lo * S;
          row_hi = g_hi * S + P;
        }
        *rows = std::max<long long>(*rows, row_hi - row_lo);
      }
    };
    // largest band that fits; backward bands are whole multiples of the stride
    // when possible so that neighbouring bands share as few windows as possible
    const int limit = bwd ? XA : GA;
    int best = 0;
    long long best_rows = 0, best_wins = 0;
    for (int band = limit; band >= 1; --band) {
      if (bwd && band > S && band % S != 0) continue;
      long long rows, wins;
      need(band, &rows, &wins);
      if (rows * q.inner_x * per_x + wins * per_win + 64 <= kTileBudgetBytes) {
        best = band;
        best_rows = rows;
        best_wins = wins;
        break;
      }
      if (limit > 4096 && band > 64) band = std::max(64, band / 2) + 1;  // keep the search short
    }
    if (best == 0) return false;
    q.band = best;
    q.bands = (int)ceil_div(limit, best);
    tile = best_rows * q.inner_x;
    nwin = best_wins;
    *blocks = pp.lead * q.bands;
  }
  if (*blocks >= (1ll << 31)) return false;
  q.by_x12 = make_fastdiv_p((unsigned)(pp.X[1] * pp.X[2]));
  q.by_x2 = make_fastdiv_p((unsigned)pp.X[2]);
  q.by_g12 = make_fastdiv_p((unsigned)(pp.G[1] * pp.G[2]));
  q.by_g2 = make_fastdiv_p((unsigned)pp.G[2]);
  q.by_xvol = make_fastdiv_p((unsigned)pp.xvol);
  q.by_gvol = make_fastdiv_p((unsigned)pp.gvol);
  for (int k = 0; k < 3; ++k) q.by_s[k] = make_fastdiv_p((unsigned)pp.S[k]);
  q.by_p12 = make_fastdiv_p((unsigned)(pp.P[1] * pp.P[2]));
  q.by_p2 = make_fastdiv_p((unsigned)pp.P[2]);
  q.nranks = 1;
  for (int k = 0; k < 3; ++k) {
    q.cand[k] = (pp.P[k] - 1) / pp.S[k] + 1;
    q.nranks *= q.cand[k];
  }
  if (q.nranks > 2047) return false;  // the rank shares a packed int with the argmax index
  *tile_elems = (int)(tile + vec);  // room for the alignment shift
  *tile_elems = (*tile_elems + 3) & ~3;
  *win_slots = bwd ? (int)((nwin + 3) & ~3ll) : 0;
  size_t bytes = (size_t)*tile_elems * elem + (bwd ? (size_t)*win_slots * 4 + ((size_t)nwin + vec) * elem : 0);
  bytes = (bytes + 15) & ~size_t(15);
  *acc_offset = 0;
  if (acc_extra) {
    *acc_offset = (int)bytes;
    bytes += (size_t)*tile_elems * acc_elem;
  }
  if (*tile_elems >= (1 << 20) || bytes > 64 * 1024) return false;
  *lds_bytes = bytes;
  *t = q;
  return true;
}

// Blocks of the persistent tile kernels: as many as fit on the device at once
// (LDS-limited, at most 8 per compute unit), never more than there are tiles.
static unsigned persistent_grid(long long tiles, size_t lds_bytes) {
  const hipDeviceProp_t &pr = runtime().props;
  const size_t lds_per_cu = 160 * 1024;
  long long per_cu = (long long)(lds_per_cu / std::max<size_t>(lds_bytes, 1));
  per_cu = std::max<long long>(1, std::min<long long>(per_cu, 8));
  return (unsigned)std::min<long long>(tiles, per_cu * pr.multiProcessorCount);
}

// Pool extents with an unrolled kernel instance (see PSIG); 0 selects the looped one.
static int pool_signature(const PoolParams &p) {
  const int sig = p.P[0] * 100 + p.P[1] * 10 + p.P[2];
  return (p.P[0] <= 3 && p.P[1] <= 3 && p.P[2] <= 3 && (sig == 133 || sig == 122 || sig == 222)) ? sig : 0;
}

static unsigned grid_for(long long total) {
  long long blocks = ceil_div(total, 256);
  const long long cap = (long long)runtime().props.multiProcessorCount * 32;
  return (unsigned)(blocks < cap ? blocks : cap);
}

// The exact-tiling kernels apply when stride == pool extent and X == G * P on every axis,
// the pool extent is one of the instantiated ones, rows are whole 16-byte pieces and the
// tensors are 16-byte aligned.  Returns 0 if not applicable, else P0*100 + P1*10 + P2.
static int exact_signature(const PoolParams &p, size_t elem, const void *a, const void *b, const void *c, size_t c_elem,
                           PoolExactParams *e) {
  for (int k = 0; k < 3; ++k)
    if (p.S[k] != p.P[k] || p.X[k] != p.G[k] * p.P[k]) return 0;
  const int sig = p.P[0] * 100 + p.P[1] * 10 + p.P[2];
  if (sig != 122 && sig != 222) return 0;
  int vec = (int)(16 / elem);
  if (p.X[2] % vec != 0) {
    if (elem != 4 || p.X[2] % 2 != 0) return 0;
    vec = 2;
  }
  const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c);
  if (bits % 16 != 0) return 0;
  (void)c_elem;
  e->vec = vec;
  e->X1 = p.X[1];
  e->X2 = p.X[2];
  e->G0 = p.G[0];
  e->G1 = p.G[1];
  e->pieces = p.X[2] / vec;
  e->xvol = p.xvol;
  e->gvol = p.gvol;
  e->total = p.lead * p.G[0] * p.G[1] * e->pieces;
  if (e->total >= (1ll << 32)) return 0;
  e->by_pieces = make_fastdiv_p((unsigned)e->pieces);
  e->by_g1 = make_fastdiv_p((unsigned)p.G[1]);
  e->by_g0 = make_fastdiv_p((unsigned)p.G[0]);
  return sig;
}

// ---- the kernels for windows known at compile time: when they apply, and their launches
// P0 P1 P2 S0 S1 S2 as one number; the instances: 3x3 every other position, 3x3 and 2x2 at every
// position (windows over the last two axes), 3x3x3 every other position.
static int window_signature6(const PoolParams &p) {
  int sig = 0;
  for (int k = 0; k < 3; ++k) sig = sig * 10 + (p.P[k] < 10 ? p.P[k] : 0);
  for (int k = 0; k < 3; ++k) sig = sig * 10 + (p.S[k] < 10 ? p.S[k] : 0);
  return sig;
}
#define MG_POOL_WINDOW_INSTANCES(X) X(1, 3, 3, 1, 2, 2) X(1, 3, 3, 1, 1, 1) X(1, 2, 2, 1, 1, 1) X(3, 3, 3, 2, 2, 2)
static bool has_rows_instance(const PoolParams &p) {
  const int sig6 = window_signature6(p);
#define MG_POOL_HAS(A, B, C, D, E, F) \
  if (sig6 == ((((A * 10 + B) * 10 + C) * 10 + D) * 10 + E) * 10 + F) return true;
  MG_POOL_WINDOW_INSTANCES(MG_POOL_HAS)
#undef MG_POOL_HAS
  return false;
}

static bool rows_forward_applies(const PoolParams &p, bool f32, const void *x) {
  static const bool on = [] {
    const char *flag = getenv("MYGRAD_HIP_POOL_ROWS");
    return !(flag && flag[0] == '0');
  }();
  const int vec = f32 ? 4 : 2;
  const long long items = p.lead * p.G[0] * ceil_div(p.G[1], POOL_ROWS_PER_THREAD) * ceil_div(p.X[2], vec);
  return on && has_rows_instance(p) && p.X[2] >= vec && vec % p.S[2] == 0 &&
         reinterpret_cast<uintptr_t>(x) % (f32 ? 4 : 8) == 0 && items < (1ll << 31);
}

// out may be null (with mark set): only the argmax offsets are wanted
static int launch_rows_forward(const PoolParams &p, bool f32, const void *x, void *out, unsigned char *mark, hipStream_t s) {
  const int vec = f32 ? 4 : 2;
  const int sig6 = window_signature6(p);
  PoolRowsParams q{};
  q.X0 = p.X[0], q.X1 = p.X[1], q.X2 = p.X[2], q.G0 = p.G[0], q.G1 = p.G[1], q.G2 = p.G[2];
  q.pieces = (int)ceil_div(p.X[2], vec);
  q.tail = p.X[2] % vec;
  q.groups = (int)ceil_div(p.G[1], POOL_ROWS_PER_THREAD);
  q.planes = p.lead * p.G[0];
  q.items = q.planes * q.groups * q.pieces;
  q.by_pieces = make_fastdiv_p((unsigned)q.pieces);
  q.by_groups = make_fastdiv_p((unsigned)q.groups);
  q.by_g0 = make_fastdiv_p((unsigned)p.G[0]);
  // a wavefront covers 63 items (its last lane only supplies its neighbour), a block 4 wavefronts
  const dim3 grid((unsigned)ceil_div(ceil_div(q.items, 63), 4)), block(256);
  bool launched = false;
#define MG_POOL_ROWS_SIG(T, MK, OUT, A, B, C, D, E, F)                                                              \
  if (!launched && sig6 == ((((A * 10 + B) * 10 + C) * 10 + D) * 10 + E) * 10 + F) {                                \
    hipLaunchKernelGGL((maxpool_rows_fwd_kernel<T, A, B, C, D, E, F, MK, OUT>), grid, block, 0, s, q, (const T *)x, \
                       (T *)out, mark);                                                                             \
    launched = true;                                                                                                \
  }
#define MG_POOL_ROWS_MK(T, MK, OUT)                                                             \
  do {                                                                                          \
    MG_POOL_ROWS_SIG(T, MK, OUT, 1, 3, 3, 1, 2, 2)                                              \
    MG_POOL_ROWS_SIG(T, MK, OUT, 1, 3, 3, 1, 1, 1)                                              \
    MG_POOL_ROWS_SIG(T, MK, OUT, 1, 2, 2, 1, 1, 1)                                              \
    MG_POOL_ROWS_SIG(T, MK, OUT, 3, 3, 3, 2, 2, 2)                                              \
  } while (0)
#define MG_POOL_ROWS(T)                                 \
  do {                                                  \
    if (!out) MG_POOL_ROWS_MK(T, true, false);          \
    else if (mark) MG_POOL_ROWS_MK(T, true, true);      \
    else MG_POOL_ROWS_MK(T, false, true);               \
  } while (0)
  if (f32) MG_POOL_ROWS(float); else MG_POOL_ROWS(double);
#undef MG_POOL_ROWS
#undef MG_POOL_ROWS_MK
#undef MG_POOL_ROWS_SIG
  if (!launched) return fail(MG_ERR_UNSUPPORTED, "no compile-time instance for pooling window signature %d", sig6);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// Windows the gather kernel loads per window row (its LW): needs that many in a row.
static int pool_gather_run(const PoolParams &p, int vd) {
  const int nw2 = (vd - 1) / p.S[2] + (p.P[2] + p.S[2] - 1) / p.S[2];
  return nw2 <= 2 ? 2 : nw2 <= 4 ? 4 : 8;
}

static bool mark_gather_applies(const PoolParams &p, bool f32, bool wide, const void *dx) {
  static const bool on = [] {
    const char *flag = getenv("MYGRAD_HIP_POOL_GATHER");
    return !(flag && flag[0] == '0');
  }();
  const int vd = (f32 && !wide) ? 4 : 2;
  const long long items = p.lead * ceil_div(p.X[0], p.S[0]) * ceil_div(p.X[1], p.S[1]) * ceil_div(p.X[2], vd);
  return on && has_rows_instance(p) && vd % p.S[2] == 0 && reinterpret_cast<uintptr_t>(dx) % (16 / vd) == 0 &&
         p.G[2] >= pool_gather_run(p, vd) && items < (1ll << 31) && p.gvol < (1ll << 30);
}

static int launch_mark_gather(const PoolParams &p, bool f32, bool wide, const unsigned char *mark, const void *grad, void *dx,
                              hipStream_t s) {
  const int vd = (f32 && !wide) ? 4 : 2;
  const int sig6 = window_signature6(p);
  PoolGatherParams q{};
  q.X0 = p.X[0], q.X1 = p.X[1], q.X2 = p.X[2], q.G0 = p.G[0], q.G1 = p.G[1], q.G2 = p.G[2];
  q.pieces = (int)ceil_div(p.X[2], vd);
  q.tail = p.X[2] % vd;
  q.groups = (int)ceil_div(p.X[1], p.S[1]);
  q.groups0 = (int)ceil_div(p.X[0], p.S[0]);
  q.planes = p.lead * q.groups0;
  q.leads = (int)p.lead;
  q.by_pieces = make_fastdiv_p((unsigned)q.pieces);
  q.by_groups = make_fastdiv_p((unsigned)q.groups);
  q.by_groups0 = make_fastdiv_p((unsigned)q.groups0);
  const dim3 grid((unsigned)ceil_div(q.planes * q.groups * q.pieces, 256)), block(256);
  bool launched = false;
#define MG_POOL_GATHER_SIG(T, TD, A, B, C, D, E, F)                                                                  \
  if (!launched && sig6 == ((((A * 10 + B) * 10 + C) * 10 + D) * 10 + E) * 10 + F) {                                 \
    hipLaunchKernelGGL((maxpool_mark_gather_kernel<T, TD, A, B, C, D, E, F>), grid, block, 0, s, q, mark,            \
                       (const T *)grad, (TD *)dx);                                                                   \
    launched = true;                                                                                                 \
  }
#define MG_POOL_GATHER(T, TD)                               \
  do {                                                      \
    MG_POOL_GATHER_SIG(T, TD, 1, 3, 3, 1, 2, 2)             \
    MG_POOL_GATHER_SIG(T, TD, 1, 3, 3, 1, 1, 1)             \
    MG_POOL_GATHER_SIG(T, TD, 1, 2, 2, 1, 1, 1)             \
    MG_POOL_GATHER_SIG(T, TD, 3, 3, 3, 2, 2, 2)             \
  } while (0)
  if (!f32)
    MG_POOL_GATHER(double, double);
  else if (wide)
    MG_POOL_GATHER(float, double);
  else
    MG_POOL_GATHER(float, float);
#undef MG_POOL_GATHER
#undef MG_POOL_GATHER_SIG
  if (!launched) return fail(MG_ERR_UNSUPPORTED, "no compile-time instance for pooling window signature %d", sig6);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// Forward pass; `mark`, when not null, receives one byte per window (see MARK).
static int maxpool_fwd_impl(const mg_pool_desc *desc, const void *x, void *out, unsigned char *mark) {
  PoolParams p;
  if (int rc = check_pool_desc(desc, &p)) return rc;
  if (!x || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in the max-pool forward pass");
  if (mark && (long long)p.P[0] * p.P[1] * p.P[2] > 256)
    return fail(MG_ERR_UNSUPPORTED, "a window of %lld elements does not fit the one-byte argmax record (at most 256)",
                (long long)p.P[0] * p.P[1] * p.P[2]);
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_POOL_FWD);
  PoolExactParams ep;
  if (const int sig = exact_signature(p, desc->dtype == MG_F32 ? 4 : 8, x, out, mark ? (const void *)mark : out, 0, &ep)) {
    note_plan(ep.vec * (desc->dtype == MG_F32 ? 4 : 8) == 16 ? "pool fwd: exact tiling, registers, 16-byte pieces"
                                                            : "pool fwd: exact tiling, registers, 8-byte pieces");
    const dim3 grid((unsigned)ceil_div(ep.total, 256)), block(256);
#define MG_POOL_EXACT_FWD_V(T, MK, V)                                                                            \
  do {                                                                                                          \
    if (sig == 122)                                                                                             \
      hipLaunchKernelGGL((maxpool_exact_kernel<T, T, 1, 2, 2, false, MK, V>), grid, block, 0, s, ep, (const T *)x, \
                         (const T *)nullptr, out, mark);                                                        \
    else                                                                                                        \
      hipLaunchKernelGGL((maxpool_exact_kernel<T, T, 2, 2, 2, false, MK, V>), grid, block, 0, s, ep, (const T *)x, \
                         (const T *)nullptr, out, mark);                                                        \
  } while (0)
#define MG_POOL_EXACT_FWD(T, MK)                                           \
  do {                                                                     \
    if (ep.vec == (int)(16 / sizeof(T))) MG_POOL_EXACT_FWD_V(T, MK, 16 / sizeof(T)); \
    else MG_POOL_EXACT_FWD_V(T, MK, 2);                                    \
  } while (0)
    if (desc->dtype == MG_F32) {
      if (mark) MG_POOL_EXACT_FWD(float, true); else MG_POOL_EXACT_FWD(float, false);
    } else {
      if (mark) MG_POOL_EXACT_FWD(double, true); else MG_POOL_EXACT_FWD(double, false);
    }
#undef MG_POOL_EXACT_FWD_V
#undef MG_POOL_EXACT_FWD
    MG_HIP(hipGetLastError());
    return MG_OK;
  }
  if (rows_forward_applies(p, desc->dtype == MG_F32, x)) {
    note_plan(p.X[2] % (desc->dtype == MG_F32 ? 4 : 2) ? "pool fwd: compile-time window, registers, rows with a short piece"
                                                       : "pool fwd: compile-time window, registers, whole pieces");
    return launch_rows_forward(p, desc->dtype == MG_F32, x, out, mark, s);
  }
  PoolTileParams tp;
  int tile_elems = 0, win_slots = 0, acc_offset = 0;
  size_t lds = 0;
  long long blocks = 0;
  const size_t elem = desc->dtype == MG_F32 ? 4 : 8;
  if (plan_tiles(p, elem, elem, false, &tp, &tile_elems, &win_slots, &acc_offset, &lds, &blocks)) {
    // one tile per block measured faster than persistent blocks for the forward pass:
    // its stores trail the next tile's loads in the same in-order memory counter
    note_plan(tp.bands > 1 ? "pool fwd: LDS tiles, bands of rows" : "pool fwd: LDS tiles, whole volumes");
    const dim3 grid((unsigned)blocks), block(256);
    const bool deep = (size_t)tile_elems * elem > 8 * 4096;  // 16-byte loads per thread to cover the tile
    const int sig = pool_signature(p);
#define MG_POOL_FWD_SIG(T, DEPTH, SIG, MK)                                                                         \
  hipLaunchKernelGGL((maxpool_tile_kernel<T, T, T, false, DEPTH, SIG, MK>), grid, block, lds, s, tp, (const T *)x, \
                     (const T *)nullptr, out, blocks, tile_elems, win_slots, acc_offset, mark)
#define MG_POOL_FWD_MK(T, DEPTH, MK)                       \
  do {                                                     \
    switch (sig) {                                         \
      case 133: MG_POOL_FWD_SIG(T, DEPTH, 133, MK); break; \
      case 122: MG_POOL_FWD_SIG(T, DEPTH, 122, MK); break; \
      case 222: MG_POOL_FWD_SIG(T, DEPTH, 222, MK); break; \
      default: MG_POOL_FWD_SIG(T, DEPTH, 0, MK); break;    \
    }                                                      \
  } while (0)
#define MG_POOL_FWD(T, DEPTH)                                                         \
  do {                                                                                \
    if (mark) MG_POOL_FWD_MK(T, DEPTH, true); else MG_POOL_FWD_MK(T, DEPTH, false);   \
  } while (0)
    if (desc->dtype == MG_F32) {
      if (deep) MG_POOL_FWD(float, 12); else MG_POOL_FWD(float, 8);
    } else {
      if (deep) MG_POOL_FWD(double, 12); else MG_POOL_FWD(double, 8);
    }
#undef MG_POOL_FWD
#undef MG_POOL_FWD_MK
#undef MG_POOL_FWD_SIG
    MG_HIP(hipGetLastError());
    return MG_OK;
  }
  note_plan("pool fwd: thread per window, no staging");
  const unsigned grid = grid_for(p.lead * p.gvol);
#define MG_POOL_FWD_PLAIN(T, MK) \
  hipLaunchKernelGGL((maxpool_fwd_kernel<T, MK>), dim3(grid), dim3(256), 0, s, p, (const T *)x, (T *)out, mark)
  if (desc->dtype == MG_F32) {
    if (mark) MG_POOL_FWD_PLAIN(float, true); else MG_POOL_FWD_PLAIN(float, false);
  } else {
    if (mark) MG_POOL_FWD_PLAIN(double, true); else MG_POOL_FWD_PLAIN(double, false);
  }
#undef MG_POOL_FWD_PLAIN
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// Backward pass from recorded argmax offsets.
static int maxpool_bwd_from_mark(const mg_pool_desc *desc, const unsigned char *mark, const void *grad, void *dx,
                                 bool own_timing = true) {
  PoolParams p;
  if (int rc = check_pool_desc(desc, &p)) return rc;
  if (!mark || !grad || !dx) return fail(MG_ERR_BAD_ARG, "null tensor pointer in the max-pool backward pass");
  if ((long long)p.P[0] * p.P[1] * p.P[2] > 256)
    return fail(MG_ERR_UNSUPPORTED, "a window of %lld elements does not fit the one-byte argmax record (at most 256)",
                (long long)p.P[0] * p.P[1] * p.P[2]);
  hipStream_t s = runtime().stream;
  std::optional<ScopedTiming> timed;
  if (own_timing) timed.emplace(TAG_POOL_BWD);  // else: a part of the caller's pass
  const bool f32 = desc->dtype == MG_F32, wide = desc->dx_dtype == MG_F64;
  PoolExactParams ep;
  // the exact-tiling test looks at the alignment of x; grad stands in for it here
  if (const int sig = exact_signature(p, f32 ? 4 : 8, grad, grad, dx, 0, &ep)) {
    note_plan(ep.vec * (f32 ? 4 : 8) == 16 ? "pool bwd from argmax: exact tiling, registers, 16-byte pieces"
                                          : "pool bwd from argmax: exact tiling, registers, 8-byte pieces");
    const dim3 grid((unsigned)ceil_div(ep.total, 256)), block(256);
#define MG_POOL_EXACT_MARK_V(T, TD, V)                                                                                \
  do {                                                                                                               \
    if (sig == 122)                                                                                                  \
      hipLaunchKernelGGL((maxpool_exact_from_mark_kernel<T, TD, 1, 2, 2, V>), grid, block, 0, s, ep, mark, (const T *)grad, \
                         (TD *)dx);                                                                                  \
    else                                                                                                             \
      hipLaunchKernelGGL((maxpool_exact_from_mark_kernel<T, TD, 2, 2, 2, V>), grid, block, 0, s, ep, mark, (const T *)grad, \
                         (TD *)dx);                                                                                  \
  } while (0)
#define MG_POOL_EXACT_MARK(T, TD)                                              \
  do {                                                                         \
    if (ep.vec == (int)(16 / sizeof(T))) MG_POOL_EXACT_MARK_V(T, TD, 16 / sizeof(T)); \
    else MG_POOL_EXACT_MARK_V(T, TD, 2);                                       \
  } while (0)
    if (!f32)
      MG_POOL_EXACT_MARK(double, double);
    else if (wide)
      MG_POOL_EXACT_MARK(float, double);
    else
      MG_POOL_EXACT_MARK(float, float);
#undef MG_POOL_EXACT_MARK_V
#undef MG_POOL_EXACT_MARK
    MG_HIP(hipGetLastError());
    return MG_OK;
  }
  if (mark_gather_applies(p, f32, wide, dx)) {
    note_plan(p.X[2] % ((f32 && !wide) ? 4 : 2) ? "pool bwd from argmax: compile-time window, register gather, rows with a short piece"
                                                : "pool bwd from argmax: compile-time window, register gather, whole pieces");
    return launch_mark_gather(p, f32, wide, mark, grad, dx, s);
  }
  {
    PoolTileParams tp;
    int tile_elems = 0, win_slots = 0, acc_offset = 0;
    size_t lds = 0;
    long long blocks = 0;
    bool overlap = false;
    for (int k = 0; k < 3; ++k) overlap |= p.P[k] > p.S[k];
    const size_t elem = f32 ? 4 : 8, acc_elem = (f32 && !overlap) ? 4 : 8;
    if (plan_tiles(p, elem, acc_elem, true, &tp, &tile_elems, &win_slots, &acc_offset, &lds, &blocks) &&
        lds + (size_t)win_slots + 32 <= 64 * 1024) {
      // the staged bytes go behind everything else; 16 spare bytes for the alignment shift
      note_plan(tp.bands > 1 ? "pool bwd from argmax: LDS tiles, bands of rows" : "pool bwd from argmax: LDS tiles, whole volumes");
      const int mark_offset = (int)lds;
      lds += ((size_t)win_slots + 16 + 15) & ~size_t(15);
      const dim3 grid(persistent_grid(blocks, lds)), block(256);
      const int sig = pool_signature(p);
      unsigned char *marks = const_cast<unsigned char *>(mark);  // only read in this mode
#define MG_POOL_MARK_SIG(T, TD, ACC, SIG)                                                                          \
  hipLaunchKernelGGL((maxpool_tile_kernel<T, TD, ACC, true, 1, SIG, false, true>), grid, block, lds, s, tp,         \
                     (const T *)nullptr, (const T *)grad, dx, blocks, tile_elems, win_slots, acc_offset, marks,     \
                     mark_offset)
#define MG_POOL_MARK_TILED(T, TD, ACC)                      \
  do {                                                      \
    switch (sig) {                                          \
      case 133: MG_POOL_MARK_SIG(T, TD, ACC, 133); break;   \
      case 122: MG_POOL_MARK_SIG(T, TD, ACC, 122); break;   \
      case 222: MG_POOL_MARK_SIG(T, TD, ACC, 222); break;   \
      default: MG_POOL_MARK_SIG(T, TD, ACC, 0); break;      \
    }                                                       \
  } while (0)
      if (!f32)
        MG_POOL_MARK_TILED(double, double, double);
      else if (overlap && wide)
        MG_POOL_MARK_TILED(float, double, double);
      else if (overlap)
        MG_POOL_MARK_TILED(float, float, double);
      else if (wide)
        MG_POOL_MARK_TILED(float, double, float);
      else
        MG_POOL_MARK_TILED(float, float, float);
#undef MG_POOL_MARK_TILED
#undef MG_POOL_MARK_SIG
      MG_HIP(hipGetLastError());
      return MG_OK;
    }
  }
  note_plan("pool bwd from argmax: thread per 16 bytes of dx, no staging");
  PoolMarkParams q{};
  for (int k = 0; k < 3; ++k) {
    q.X[k] = p.X[k];
    q.P[k] = p.P[k];
    q.S[k] = p.S[k];
    q.G[k] = p.G[k];
    q.by_s[k] = make_fastdiv_p((unsigned)p.S[k]);
  }
  q.xvol = (int)p.xvol;
  q.gvol = (int)p.gvol;
  q.x12 = p.X[1] * p.X[2];
  q.lead = p.lead;
  q.by_xvol = make_fastdiv_p((unsigned)p.xvol);
  q.by_x12 = make_fastdiv_p((unsigned)q.x12);
  q.by_x2 = make_fastdiv_p((unsigned)p.X[2]);
  // slices of whole leading indices whose element count stays below 2^31 (32-bit index
  // arithmetic inside a slice); a multiple of 4 of them so every slice starts 16-byte aligned
  const long long cap = ((1ll << 31) - 1024) / p.xvol;
  long long leads = std::min<long long>(p.lead, cap);
  if (leads < p.lead) leads -= leads % 4;
  const size_t dx_elem = (f32 && !wide) ? 4 : 8;
  const bool vector_ok = leads >= 1 && reinterpret_cast<uintptr_t>(dx) % 16 == 0;
  if (leads < 1) leads = 1;
  q.leads = (int)leads;
  const int vd = vector_ok ? (int)(16 / dx_elem) : 1;
  const long long slice = leads * p.xvol;
  const dim3 grid((unsigned)ceil_div(ceil_div(slice, vd), 256), (unsigned)ceil_div(p.lead, leads)), block(256);
#define MG_POOL_MARK(T, TD)                                                                                        \
  do {                                                                                                             \
    if (vd > 1)                                                                                                    \
      hipLaunchKernelGGL((maxpool_from_mark_kernel<T, TD, 16 / sizeof(TD)>), grid, block, 0, s, q, mark,           \
                         (const T *)grad, (TD *)dx);                                                               \
    else                                                                                                           \
      hipLaunchKernelGGL((maxpool_from_mark_kernel<T, TD, 1>), grid, block, 0, s, q, mark, (const T *)grad, (TD *)dx); \
  } while (0)
  if (!f32)
    MG_POOL_MARK(double, double);
  else if (wide)
    MG_POOL_MARK(float, double);
  else
    MG_POOL_MARK(float, float);
#undef MG_POOL_MARK
  MG_HIP(hipGetLastError());
  return MG_OK;
}

}  // namespace mg

using namespace mg;

extern "C" {

int mg_maxpool_fwd(const mg_pool_desc *desc, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  return maxpool_fwd_impl(desc, x, out, nullptr);
}

int mg_maxpool_fwd_argmax(const mg_pool_desc *desc, const void *x, void *out, void *argmax) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (!argmax) return fail(MG_ERR_BAD_ARG, "null argmax pointer in mg_maxpool_fwd_argmax");
  return maxpool_fwd_impl(desc, x, out, static_cast<unsigned char *>(argmax));
}

int mg_maxpool_bwd_argmax(const mg_pool_desc *desc, const void *argmax, const void *grad, void *dx) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  return maxpool_bwd_from_mark(desc, static_cast<const unsigned char *>(argmax), grad, dx);
}

static int staged_gather(const mg_pool_desc *inner, const mg_pool_desc *outer, const mg_pool_desc *third, const void *inner_argmax,
                         const void *outer_argmax, const void *third_argmax, const void *grad, void *dx) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  PoolParams pi, po, pt;
  if (int rc = check_pool_desc(inner, &pi)) return rc;
  if (int rc = check_pool_desc(outer, &po)) return rc;
  if (third)
    if (int rc = check_pool_desc(third, &pt)) return rc;
  if (!inner_argmax || !outer_argmax || (third && !third_argmax) || !grad || !dx)
    return fail(MG_ERR_BAD_ARG, "null pointer in mg_maxpool_bwd_argmax_staged");
  if (inner->dtype != outer->dtype || inner->dx_dtype != outer->dx_dtype || (third && (third->dtype != inner->dtype || third->dx_dtype != inner->dx_dtype)))
    return fail(MG_ERR_BAD_ARG, "the stages disagree on the types");
  // the outer stage pools the leading axes over the inner stage's windows: its last axis is their
  // merged grid with a window of one element, and its positions are the inner stage's leading indices
  if (po.X[2] != pi.gvol || po.P[2] != 1 || po.S[2] != 1 || po.G[2] != pi.gvol || po.lead * po.X[0] * po.X[1] != pi.lead)
    return fail(MG_ERR_BAD_ARG, "the outer stage (lead %lld, extents %d x %d x %d) does not pool the inner stage's %lld positions of %lld windows",
                po.lead, po.X[0], po.X[1], po.X[2], pi.lead, pi.gvol);
  if ((long long)pi.P[0] * pi.P[1] * pi.P[2] > 256 || (long long)po.P[0] * po.P[1] > 256)
    return fail(MG_ERR_UNSUPPORTED, "a window of more than 256 elements does not fit the one-byte argmax record");
  if (pi.lead >= (1ll << 31) || po.lead * po.G[0] * po.G[1] * pi.gvol >= (1ll << 40))
    return fail(MG_ERR_UNSUPPORTED, "too many leading positions for the staged gather");
  // a third stage pools two more axes over the merged grid of the first two, in the same way
  if (third && (pt.X[2] != po.gvol || pt.P[2] != 1 || pt.S[2] != 1 || pt.G[2] != po.gvol || pt.lead * pt.X[0] * pt.X[1] != po.lead))
    return fail(MG_ERR_BAD_ARG, "the third stage (lead %lld, extents %d x %d x %d) does not pool the second stage's %lld positions of %lld windows",
                pt.lead, pt.X[0], pt.X[1], pt.X[2], po.lead, po.gvol);
  if (third && (long long)pt.P[0] * pt.P[1] > 256)
    return fail(MG_ERR_UNSUPPORTED, "a window of more than 256 elements does not fit the one-byte argmax record");
  PoolStagedParams q{};
  for (int k = 0; k < 2; ++k) {
    q.RX[k] = third ? pt.X[k] : 1, q.RP[k] = third ? pt.P[k] : 1, q.RS[k] = third ? pt.S[k] : 1, q.RG[k] = third ? pt.G[k] : 1;
    q.by_rs[k] = make_fastdiv_p((unsigned)q.RS[k]);
  }
  q.by_rx1 = make_fastdiv_p((unsigned)q.RX[1]);
  q.by_rx01 = make_fastdiv_p((unsigned)(q.RX[0] * q.RX[1]));
  for (int k = 0; k < 3; ++k) {
    q.X[k] = pi.X[k], q.P[k] = pi.P[k], q.S[k] = pi.S[k], q.G[k] = pi.G[k];
    q.by_s[k] = make_fastdiv_p((unsigned)pi.S[k]);
  }
  for (int k = 0; k < 2; ++k) {
    q.OX[k] = po.X[k], q.OP[k] = po.P[k], q.OS[k] = po.S[k], q.OG[k] = po.G[k];
    q.by_os[k] = make_fastdiv_p((unsigned)po.S[k]);
  }
  q.xvol = (int)pi.xvol;
  q.gvol = (int)pi.gvol;
  q.total = pi.lead * pi.xvol;
  q.by_xvol = make_fastdiv_p((unsigned)pi.xvol);
  q.by_x12 = make_fastdiv_p((unsigned)(pi.X[1] * pi.X[2]));
  q.by_x2 = make_fastdiv_p((unsigned)pi.X[2]);
  q.by_ox1 = make_fastdiv_p((unsigned)po.X[1]);
  q.by_ox01 = make_fastdiv_p((unsigned)(po.X[0] * po.X[1]));
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_POOL_BWD);
  note_plan(third ? "pool bwd from three stages' argmax: thread per element of dx, whole windows in row-major order"
                  : "pool bwd from two stages' argmax: thread per element of dx, whole windows in row-major order");
  const unsigned grid = grid_for(q.total);
  const unsigned char *m1 = static_cast<const unsigned char *>(inner_argmax), *m2 = static_cast<const unsigned char *>(outer_argmax),
                      *m3 = static_cast<const unsigned char *>(third_argmax);
  if (inner->dtype == MG_F64)
    hipLaunchKernelGGL((maxpool_staged_gather_kernel<double, double>), dim3(grid), dim3(256), 0, s, q, m1, m2, m3, (const double *)grad, (double *)dx);
  else if (inner->dx_dtype == MG_F64)
    hipLaunchKernelGGL((maxpool_staged_gather_kernel<float, double>), dim3(grid), dim3(256), 0, s, q, m1, m2, m3, (const float *)grad, (double *)dx);
  else
    hipLaunchKernelGGL((maxpool_staged_gather_kernel<float, float>), dim3(grid), dim3(256), 0, s, q, m1, m2, m3, (const float *)grad, (float *)dx);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_maxpool_bwd_argmax_staged(const mg_pool_desc *inner, const mg_pool_desc *outer, const void *inner_argmax,
                                 const void *outer_argmax, const void *grad, void *dx) {
  return staged_gather(inner, outer, nullptr, inner_argmax, outer_argmax, nullptr, grad, dx);
}

int mg_maxpool_bwd_argmax_staged3(const mg_pool_desc *inner, const mg_pool_desc *outer, const mg_pool_desc *third,
                                  const void *inner_argmax, const void *outer_argmax, const void *third_argmax, const void *grad,
                                  void *dx) {
  if (!third) return fail(MG_ERR_BAD_ARG, "null descriptor of the third stage");
  return staged_gather(inner, outer, third, inner_argmax, outer_argmax, third_argmax, grad, dx);
}

int mg_maxpool_bwd(const mg_pool_desc *desc, const void *x, const void *grad, void *dx) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  PoolParams p;
  if (int rc = check_pool_desc(desc, &p)) return rc;
  if (!x || !grad || !dx) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_maxpool_bwd");
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_POOL_BWD);
  PoolExactParams ep;
  if (const int sig = exact_signature(p, desc->dtype == MG_F32 ? 4 : 8, x, grad, dx, 0, &ep)) {
    note_plan(ep.vec * (desc->dtype == MG_F32 ? 4 : 8) == 16 ? "pool bwd: exact tiling, registers, 16-byte pieces"
                                                            : "pool bwd: exact tiling, registers, 8-byte pieces");
    const dim3 grid((unsigned)ceil_div(ep.total, 256)), block(256);
#define MG_POOL_EXACT_BWD_V(T, TD, V)                                                                                      \
  do {                                                                                                                    \
    if (sig == 122)                                                                                                       \
      hipLaunchKernelGGL((maxpool_exact_kernel<T, TD, 1, 2, 2, true, false, V>), grid, block, 0, s, ep, (const T *)x, (const T *)grad, dx); \
    else                                                                                                                  \
      hipLaunchKernelGGL((maxpool_exact_kernel<T, TD, 2, 2, 2, true, false, V>), grid, block, 0, s, ep, (const T *)x, (const T *)grad, dx); \
  } while (0)
#define MG_POOL_EXACT_BWD(T, TD)                                              \
  do {                                                                        \
    if (ep.vec == (int)(16 / sizeof(T))) MG_POOL_EXACT_BWD_V(T, TD, 16 / sizeof(T)); \
    else MG_POOL_EXACT_BWD_V(T, TD, 2);                                       \
  } while (0)
    if (desc->dtype == MG_F64)
      MG_POOL_EXACT_BWD(double, double);
    else if (desc->dx_dtype == MG_F64)
      MG_POOL_EXACT_BWD(float, double);
    else
      MG_POOL_EXACT_BWD(float, float);
#undef MG_POOL_EXACT_BWD_V
#undef MG_POOL_EXACT_BWD
    MG_HIP(hipGetLastError());
    return MG_OK;
  }
  if (rows_forward_applies(p, desc->dtype == MG_F32, x) &&
      mark_gather_applies(p, desc->dtype == MG_F32, desc->dx_dtype == MG_F64, dx)) {
    // two passes straight from global memory: every window's first-occurrence argmax as one
    // byte in the library workspace (x is read, nothing else is written), then the gather
    // from those bytes -- less traffic through LDS than finding and routing in one kernel
    note_plan("pool bwd: compile-time window, argmax pass + register gather");
    void *marks = nullptr;
    if (int rc = workspace((size_t)(p.lead * p.gvol), &marks)) return rc;
    if (int rc = launch_rows_forward(p, desc->dtype == MG_F32, x, nullptr, (unsigned char *)marks, s)) return rc;
    return launch_mark_gather(p, desc->dtype == MG_F32, desc->dx_dtype == MG_F64, (const unsigned char *)marks, grad, dx, s);
  }
  PoolTileParams tp;
  int tile_elems = 0, win_slots = 0, acc_offset = 0;
  size_t lds = 0;
  long long blocks = 0;
  // float32 input whose windows overlap sums several float32 terms per element: that
  // sum is carried in double (the reference's dx is float64) and rounded once.  When
  // no two windows overlap an element gets at most one term and float32 is exact.
  bool overlap = false;
  for (int k = 0; k < 3; ++k) overlap |= p.P[k] > p.S[k];
  const bool f32 = desc->dtype == MG_F32;
  const size_t elem = f32 ? 4 : 8, acc_elem = (f32 && !overlap) ? 4 : 8;
  if (plan_tiles(p, elem, acc_elem, true, &tp, &tile_elems, &win_slots, &acc_offset, &lds, &blocks)) {
    note_plan(tp.bands > 1 ? "pool bwd: LDS tiles, bands of rows" : "pool bwd: LDS tiles, whole volumes");
    const dim3 grid(persistent_grid(blocks, lds)), block(256);
    const bool wide = desc->dx_dtype == MG_F64;
    const bool deep = (size_t)tile_elems * elem > 8 * 4096;
    const int sig = pool_signature(p);
#define MG_POOL_BWD_SIG(T, TD, ACC, DEPTH, SIG)                                                                   \
  hipLaunchKernelGGL((maxpool_tile_kernel<T, TD, ACC, true, DEPTH, SIG>), grid, block, lds, s, tp, (const T *)x,  \
                     (const T *)grad, dx, blocks, tile_elems, win_slots, acc_offset)
#define MG_POOL_BWD_D(T, TD, ACC, DEPTH)                          \
  do {                                                            \
    switch (sig) {                                                \
      case 133: MG_POOL_BWD_SIG(T, TD, ACC, DEPTH, 133); break;   \
      case 122: MG_POOL_BWD_SIG(T, TD, ACC, DEPTH, 122); break;   \
      case 222: MG_POOL_BWD_SIG(T, TD, ACC, DEPTH, 222); break;   \
      default: MG_POOL_BWD_SIG(T, TD, ACC, DEPTH, 0); break;      \
    }                                                             \
  } while (0)
#define MG_POOL_BWD(T, TD, ACC)                   \
  do {                                            \
    if (deep)                                     \
      MG_POOL_BWD_D(T, TD, ACC, 12);              \
    else                                          \
      MG_POOL_BWD_D(T, TD, ACC, 8);               \
  } while (0)
    if (!f32)
      MG_POOL_BWD(double, double, double);
    else if (overlap && wide)
      MG_POOL_BWD(float, double, double);
    else if (overlap)
      MG_POOL_BWD(float, float, double);
    else if (wide)
      MG_POOL_BWD(float, double, float);
    else
      MG_POOL_BWD(float, float, float);
#undef MG_POOL_BWD
#undef MG_POOL_BWD_D
#undef MG_POOL_BWD_SIG
    MG_HIP(hipGetLastError());
    return MG_OK;
  }
  if ((long long)p.P[0] * p.P[1] * p.P[2] <= 256) {
    // No room in LDS for a band of this shape: one pass that records every window's argmax in the
    // library workspace (a thread per window), then the routing from those bytes (a thread per 16
    // bytes of dx walks the few windows that cover it).  The kernel below, a thread per element
    // that scans every covering window itself, reads x prod(P) / prod(S) times over.
    void *marks = nullptr;
    if (int rc = workspace((size_t)(p.lead * p.gvol), &marks)) return rc;
    const unsigned mgrid = grid_for(p.lead * p.gvol);
    if (desc->dtype == MG_F32)
      hipLaunchKernelGGL((maxpool_fwd_kernel<float, true>), dim3(mgrid), dim3(256), 0, s, p, (const float *)x, (float *)nullptr,
                         (unsigned char *)marks);
    else
      hipLaunchKernelGGL((maxpool_fwd_kernel<double, true>), dim3(mgrid), dim3(256), 0, s, p, (const double *)x, (double *)nullptr,
                         (unsigned char *)marks);
    MG_HIP(hipGetLastError());
    const int rc = maxpool_bwd_from_mark(desc, (const unsigned char *)marks, grad, dx, false);
    note_plan("pool bwd: argmax pass (thread per window) + routing from the record, no staging");
    return rc;
  }
  note_plan("pool bwd: thread per element, no staging");
  const unsigned grid = grid_for(p.lead * p.xvol);
  if (desc->dtype == MG_F64)
    hipLaunchKernelGGL((maxpool_bwd_kernel<double, double>), dim3(grid), dim3(256), 0, s, p, (const double *)x,
                       (const double *)grad, (double *)dx);
  else if (desc->dx_dtype == MG_F64)
    hipLaunchKernelGGL((maxpool_bwd_kernel<float, double>), dim3(grid), dim3(256), 0, s, p, (const float *)x,
                       (const float *)grad, (double *)dx);
  else
    hipLaunchKernelGGL((maxpool_bwd_kernel<float, float>), dim3(grid), dim3(256), 0, s, p, (const float *)x,
                       (const float *)grad, (float *)dx);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

}  // extern "C"
