// The other consumers of the window index map, for gfx950: `repeat` (forward, and its gradient,
// which the reference forms as a sum over a windowed view of the incoming gradient) and a
// contiguous copy of a sliding-window view.  All three move bytes: bandwidth-bound, one
// element or one 16-byte piece per lane, coalesced on the side that is written (forward,
// window copy) or on the rows of `inner` elements (gradient).
//
//   repeat      out[o, j, i] = a[o, src(j), i]        a:(outer, n, inner), out:(outer, total, inner)
//   gradient    da[o, s, i]  = sum_{j: src(j) = s} grad[o, j, i], ascending j, from +0.0
//   window copy out[g, l, w] = x[l, g*S + w*D]        out:(G..., lead, W...) contiguous
#include "internal.h"

#include <algorithm>

namespace mg {

namespace {

struct FastDivT {
  unsigned mul, shr, d, pad_;
  __device__ __forceinline__ unsigned div(unsigned n) const { return d == 1u ? n : __umulhi(n, mul) >> shr; }
};

FastDivT make_fastdiv_t(unsigned d) {
  FastDivT f{0u, 0u, d, 0u};
  if (d > 1u) {
    unsigned lg = 0;
    while ((1ull << lg) < d) ++lg;
    const unsigned p = 31u + lg;
    f.mul = (unsigned)(((1ull << p) + d - 1ull) / d);
    f.shr = p - 32u;
  }
  return f;
}

struct RepeatParams {
  unsigned rows_out;  // outer * total
  unsigned rows_in;   // outer * n
  unsigned pieces;    // pieces per row: inner / (elements per piece)
  unsigned n, total, repeats;
  FastDivT by_pieces, by_total, by_n, by_repeats;
  long long inner;
};

template <int BYTES>
struct Word;
template <>
struct Word<1> { typedef unsigned char type; };
template <>
struct Word<2> { typedef unsigned short type; };
template <>
struct Word<4> { typedef unsigned type; };
template <>
struct Word<8> { typedef unsigned long long type; };
struct alignas(16) Word16 { unsigned v[4]; };
template <>
struct Word<16> { typedef Word16 type; };

// One thread per piece of `out` (PIECE bytes: one element, or 16 bytes of a row).
template <int PIECE>
__global__ void __launch_bounds__(256) repeat_fwd_kernel(RepeatParams p, const int *__restrict__ src_of,
                                                         const typename Word<PIECE>::type *__restrict__ a,
                                                         typename Word<PIECE>::type *__restrict__ out, unsigned count) {
  const unsigned t = blockIdx.x * 256u + threadIdx.x;
  if (t >= count) return;
  const unsigned row = p.by_pieces.div(t), ip = t - row * p.pieces;
  const unsigned o = p.by_total.div(row), j = row - o * p.total;
  const unsigned src = src_of ? (unsigned)src_of[j] : p.by_repeats.div(j);
  out[t] = a[((size_t)o * p.n + src) * p.pieces + ip];
}

// One thread per piece of `da`: adds its run of rows of grad in ascending order from +0.0,
// each addition rounded in T (np.add.at's order and arithmetic for unequal repeats).
template <typename T, int VEC>
__global__ void __launch_bounds__(256) repeat_bwd_kernel(RepeatParams p, const long long *__restrict__ offsets,
                                                         const T *__restrict__ grad, T *__restrict__ da, unsigned count) {
  typedef T V __attribute__((ext_vector_type(VEC)));
  const unsigned t = blockIdx.x * 256u + threadIdx.x;
  if (t >= count) return;
  const unsigned row = p.by_pieces.div(t), ip = t - row * p.pieces;
  const unsigned o = p.by_n.div(row), s = row - o * p.n;
  const unsigned first = offsets ? (unsigned)offsets[s] : s * p.repeats;
  const unsigned last = offsets ? (unsigned)offsets[s + 1] : first + p.repeats;
  const V *g = reinterpret_cast<const V *>(grad) + ((size_t)o * p.total + first) * p.pieces + ip;
  V acc;
#pragma unroll
  for (int k = 0; k < VEC; ++k) acc[k] = T(0);
#pragma unroll 4
  for (unsigned j = first; j < last; ++j, g += p.pieces) {
    const V v = *g;
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] += v[k];
  }
  reinterpret_cast<V *>(da)[t] = acc;
}

// Equal repeats along the last axis (or of the flattened array): out[f] = a[f / repeats] over
// the flat index.  One thread per 16-byte piece of `out`: it divides once and walks on.
template <int BYTES>
__global__ void __launch_bounds__(256) repeat_last_fwd_kernel(FastDivT by_repeats, unsigned repeats,
                                                              const typename Word<BYTES>::type *__restrict__ a,
                                                              typename Word<BYTES>::type *__restrict__ out, unsigned pieces) {
  typedef typename Word<BYTES>::type W;
  constexpr int VEC = 16 / BYTES;
  typedef W V __attribute__((ext_vector_type(VEC)));
  const unsigned t = blockIdx.x * 256u + threadIdx.x;
  if (t >= pieces) return;
  unsigned src = by_repeats.div(t * VEC), used = t * VEC - src * repeats;
  V v;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    v[k] = a[src];
    if (++used == repeats) {
      used = 0;
      ++src;
    }
  }
  reinterpret_cast<V *>(out)[t] = v;
}

// Its gradient: da[s] = grad[s*repeats] + ... + grad[s*repeats + repeats - 1], added in that
// order from +0.0.  One thread per 16-byte piece of `da`: the VEC * repeats gradient elements
// it needs are contiguous and start on a 16-byte boundary, so it reads them as `repeats`
// 16-byte pieces and deals each element to the sum it belongs to.
template <typename T>
__global__ void __launch_bounds__(256) repeat_last_bwd_kernel(unsigned repeats, const T *__restrict__ grad, T *__restrict__ da,
                                                              unsigned pieces) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T V __attribute__((ext_vector_type(VEC)));
  const unsigned t = blockIdx.x * 256u + threadIdx.x;
  if (t >= pieces) return;
  const V *g = reinterpret_cast<const V *>(grad) + (size_t)t * repeats;
  V acc;
#pragma unroll
  for (int m = 0; m < VEC; ++m) acc[m] = T(0);
  unsigned target = 0, used = 0;
#pragma unroll 2
  for (unsigned q = 0; q < repeats; ++q) {
    const V v = g[q];
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
#pragma unroll
      for (int m = 0; m < VEC; ++m) acc[m] = target == (unsigned)m ? acc[m] + v[k] : acc[m];
      if (++used == repeats) {
        used = 0;
        ++target;
      }
    }
  }
  reinterpret_cast<V *>(da)[t] = acc;
}

struct WindowParams {
  int nd;
  unsigned lead, wvol, xvol, gvol;
  unsigned W[MG_MAX_ND], G[MG_MAX_ND];
  unsigned step[MG_MAX_ND], dil[MG_MAX_ND];    // in elements of x along each axis
  unsigned xstride[MG_MAX_ND];                 // elements between neighbours along each axis
  FastDivT by_wvol, by_w[MG_MAX_ND], by_g[MG_MAX_ND];
};

// Block (x = placement g, y = slice of the (lead, window) pairs): the placement's offset in x is
// the same for the whole block and is worked out on the scalar unit; a thread divides only by
// the window's volume and extents.  Writes are contiguous per placement: out[g] is one run of
// lead * wvol elements.
template <int BYTES>
__global__ void __launch_bounds__(256) window_gather_kernel(WindowParams p, const typename Word<BYTES>::type *__restrict__ x,
                                                            typename Word<BYTES>::type *__restrict__ out) {
  // blocks are dealt to the eight XCDs in turn: give each XCD a contiguous range of
  // placements, whose windows overlap in x, so that its L2 serves the overlap
  // (the grid's x extent is 8 * ceil(gvol / 8))
  const unsigned placement = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (placement >= p.gvol) return;
  unsigned g = placement;
  size_t base = 0;
#pragma unroll
  for (int k = MG_MAX_ND - 1; k >= 0; --k) {
    const unsigned gq = p.by_g[k].div(g);
    base += (size_t)((g - gq * p.G[k]) * p.step[k]) * p.xstride[k];
    g = gq;
  }
  const unsigned per_g = p.lead * p.wvol;
  typename Word<BYTES>::type *dst = out + (size_t)placement * per_g;
  for (unsigned t = blockIdx.y * 256u + threadIdx.x; t < per_g; t += gridDim.y * 256u) {
    const unsigned l = p.by_wvol.div(t);
    unsigned w = t - l * p.wvol;
    size_t at = base + (size_t)l * p.xvol;
#pragma unroll
    for (int k = MG_MAX_ND - 1; k >= 0; --k) {
      const unsigned wq = p.by_w[k].div(w);
      at += (size_t)((w - wq * p.W[k]) * p.dil[k]) * p.xstride[k];
      w = wq;
    }
    dst[t] = x[at];
  }
}

// The staged variant.  A block takes `tg` consecutive placements along the last windowed axis
// (all other placement indices fixed) and `planes` of the leading entries.  It first brings the
// part of x those windows cover into LDS: per plane, one run of `span` contiguous elements for
// every row of the window (a row = one setting of the window's indices but the last), read
// coalesced and once.  Then it writes, for each of its placements, the run of planes * wvol
// output elements from LDS.  Without the staging every 64-byte line of x is fetched again for
// each placement that touches it, and the L2-to-L1 traffic, not HBM, sets the pace.
constexpr int kMaxWindowRows = 64;
constexpr int kMaxWindowVolume = 1024;

struct WindowTile {
  unsigned tg, planes, rows, span_max, tiles_last, chunks;
  unsigned hop_l, hop_w;                 // 256 = hop_l * wvol + hop_w: one round of the block through (plane, w)
  unsigned row_offset[kMaxWindowRows];   // offset in x of each row of the window
  FastDivT by_tiles_last, by_chunks, by_rows, by_span[2], by_wlast;  // by_span: [0] a full tile, [1] the last, shorter one
};

template <int BYTES>
__global__ void __launch_bounds__(256) window_tile_kernel(WindowParams p, WindowTile q, const typename Word<BYTES>::type *__restrict__ x,
                                                          typename Word<BYTES>::type *__restrict__ out) {
  typedef typename Word<BYTES>::type W;
  extern __shared__ __align__(16) unsigned char staged_raw[];
  __shared__ unsigned within_plane[kMaxWindowVolume];  // window position w -> offset in a staged plane (placement 0)
  W *staged = reinterpret_cast<W *>(staged_raw);
  constexpr int LAST = MG_MAX_ND - 1;
  // blocks that run together write neighbouring runs: the slice of planes varies fastest
  const unsigned group = q.by_chunks.div(blockIdx.x), chunk = blockIdx.x - group * q.chunks;
  unsigned g = q.by_tiles_last.div(group);             // flat index of the other placement axes
  const unsigned gl0 = (group - g * q.tiles_last) * q.tg;
  const unsigned ng = min(q.tg, p.G[LAST] - gl0);
  const size_t out_row0 = (size_t)g * p.G[LAST] + gl0;  // flat placement index of the block's first
  size_t base = (size_t)gl0 * p.step[LAST];
#pragma unroll
  for (int k = LAST - 1; k >= 0; --k) {
    const unsigned gq = p.by_g[k].div(g);
    base += (size_t)((g - gq * p.G[k]) * p.step[k]) * p.xstride[k];
    g = gq;
  }
  const unsigned l0 = chunk * q.planes;
  const unsigned nl = min(q.planes, p.lead - l0);
  const unsigned span = (ng - 1) * p.step[LAST] + (p.W[LAST] - 1) * p.dil[LAST] + 1;
  const FastDivT by_span = q.by_span[ng == q.tg ? 0 : 1];

  for (unsigned w = threadIdx.x; w < p.wvol; w += 256u) {
    const unsigned r = q.by_wlast.div(w);
    within_plane[w] = r * q.span_max + (w - r * p.W[LAST]) * p.dil[LAST];
  }
  const W *src = x + (size_t)l0 * p.xvol + base;
  const unsigned loads = nl * q.rows * span;
  // eight loads in flight per thread before the first is stored to LDS
  for (unsigned t0 = threadIdx.x; t0 < loads; t0 += 256u * 8u) {
    W value[8];
    unsigned where[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const unsigned t = t0 + u * 256u;
      if (t < loads) {
        const unsigned lr = by_span.div(t), c = t - lr * span;  // lr = l * rows + r
        const unsigned l = q.by_rows.div(lr), r = lr - l * q.rows;
        where[u] = lr * q.span_max + c;
        value[u] = src[l * p.xvol + q.row_offset[r] + c];
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (t0 + u * 256u < loads) staged[where[u]] = value[u];
  }
  __syncthreads();
  // per placement one contiguous run of nl * wvol elements; a thread steps through (plane, w)
  // by additions: each round of the block advances it by 256 = hop_l * wvol + hop_w
  const unsigned items = nl * p.wvol;
  const unsigned plane_size = q.rows * q.span_max;
  const unsigned start_l = p.by_wvol.div(threadIdx.x), start_w = threadIdx.x - start_l * p.wvol;
  for (unsigned gi = 0; gi < ng; ++gi) {
    W *dst = out + ((out_row0 + gi) * p.lead + l0) * p.wvol;
    const W *from = staged + gi * p.step[LAST];
    unsigned l = start_l, w = start_w;
#pragma unroll 2
    for (unsigned rest = threadIdx.x; rest < items; rest += 256u) {
      dst[rest] = from[l * plane_size + within_plane[w]];
      l += q.hop_l;
      w += q.hop_w;
      if (w >= p.wvol) {
        w -= p.wvol;
        ++l;
      }
    }
  }
}

constexpr long long kMaxCount = (1ll << 31) - 1;  // threads of one launch, and the 32-bit index arithmetic

int repeat_params(const char *who, int64_t outer, int64_t n, int64_t inner, int64_t repeats, int64_t total, bool uniform,
                  int64_t per_piece, RepeatParams *p) {
  if (outer < 1 || n < 1 || inner < 1 || total < 0 || repeats < 0)
    return fail(MG_ERR_BAD_ARG, "%s: outer=%lld n=%lld inner=%lld must be positive, total=%lld repeats=%lld non-negative", who,
                (long long)outer, (long long)n, (long long)inner, (long long)total, (long long)repeats);
  if (uniform && total != n * repeats)
    return fail(MG_ERR_BAD_ARG, "%s: total=%lld is not n*repeats=%lld", who, (long long)total, (long long)(n * repeats));
  const int64_t pieces = inner / per_piece;
  if (outer * std::max(total, n) * pieces > kMaxCount || outer * std::max(total, n) > kMaxCount)
    return fail(MG_ERR_UNSUPPORTED, "%s: more than 2^31 - 1 pieces", who);
  p->rows_out = (unsigned)(outer * total);
  p->rows_in = (unsigned)(outer * n);
  p->pieces = (unsigned)pieces;
  p->n = (unsigned)n;
  p->total = (unsigned)total;
  p->repeats = (unsigned)repeats;
  p->by_pieces = make_fastdiv_t((unsigned)pieces);
  p->by_total = make_fastdiv_t((unsigned)std::max<int64_t>(total, 1));
  p->by_n = make_fastdiv_t((unsigned)n);
  p->by_repeats = make_fastdiv_t((unsigned)std::max<int64_t>(repeats, 1));
  p->inner = inner;
  return MG_OK;
}

bool aligned16(std::initializer_list<const void *> ptrs) {
  for (const void *q : ptrs)
    if (reinterpret_cast<uintptr_t>(q) % 16 != 0) return false;
  return true;
}

template <int PIECE>
void launch_repeat_fwd(const RepeatParams &p, const int *src_of, const void *a, void *out) {
  typedef typename Word<PIECE>::type W;
  const unsigned count = p.rows_out * p.pieces;
  hipLaunchKernelGGL(repeat_fwd_kernel<PIECE>, dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, runtime().stream, p, src_of,
                     (const W *)a, (W *)out, count);
}

template <typename T>
void launch_repeat_bwd(const RepeatParams &p, bool wide, const long long *offsets, const void *grad, void *da) {
  constexpr int VEC = 16 / sizeof(T);
  const unsigned count = p.rows_in * p.pieces;
  const dim3 grid((unsigned)ceil_div(count, 256)), block(256);
  if (wide)
    hipLaunchKernelGGL((repeat_bwd_kernel<T, VEC>), grid, block, 0, runtime().stream, p, offsets, (const T *)grad, (T *)da, count);
  else
    hipLaunchKernelGGL((repeat_bwd_kernel<T, 1>), grid, block, 0, runtime().stream, p, offsets, (const T *)grad, (T *)da, count);
}

// ------------------------------------------------------------------------------------------
// Transposition: out = x.transpose(perm), C-contiguous.  The host drops axes of length one
// and merges output axes that are neighbours in the input as well; what is left has at most
// kMaxPermuteAxes axes, described per OUTPUT axis by its extent and its stride in the input.
//   rows  the last output axis is also the input's fastest one: whole runs are copied, 16
//         bytes per lane where the runs allow it;
//   tile  otherwise some other output axis p is the input's fastest one: 32 x 32 tiles over
//         (axis p, last axis) go through LDS, read along p and written along the last axis,
//         so that both sides are coalesced.
// ------------------------------------------------------------------------------------------
constexpr int kMaxPermuteAxes = 6;

struct PermuteParams {
  int nd;
  unsigned size[kMaxPermuteAxes];
  long long in_stride[kMaxPermuteAxes];  // rows: in pieces; tile: in elements
  FastDivT by_size[kMaxPermuteAxes];
  unsigned pieces;  // rows: pieces per run
  FastDivT by_pieces;
  unsigned count;   // rows: pieces in all
  int p_axis;       // tile: the output axis that is the input's fastest
  long long p_out_stride;
  unsigned tiles_c, tiles_r, nrest;
  FastDivT by_tiles_c;
};

template <int PIECE>
__global__ void __launch_bounds__(256) permute_rows_kernel(PermuteParams p, const typename Word<PIECE>::type *__restrict__ x,
                                                           typename Word<PIECE>::type *__restrict__ out) {
  const unsigned t = blockIdx.x * 256u + threadIdx.x;
  if (t >= p.count) return;
  unsigned row = p.by_pieces.div(t);
  long long at = t - row * p.pieces;
  for (int k = p.nd - 2; k >= 0; --k) {
    const unsigned q = p.by_size[k].div(row);
    at += (long long)(row - q * p.size[k]) * p.in_stride[k];
    row = q;
  }
  out[t] = x[at];
}

// VEC elements (16 bytes, or one element when the extents or the pointers do not allow it) per
// lane on both sides: along axis p when reading, along the last axis when writing.
template <int BYTES, int VEC>
__global__ void __launch_bounds__(256) permute_tile_kernel(PermuteParams p, const typename Word<BYTES>::type *__restrict__ x,
                                                           typename Word<BYTES>::type *__restrict__ out) {
  typedef typename Word<BYTES>::type W;
  typedef W WV __attribute__((ext_vector_type(VEC)));
  constexpr int LX = 32 / VEC, LY = 256 / LX, ITERS = 32 / LY;
  __shared__ W tile[32][33];
  const int last = p.nd - 1;
  const unsigned tr = p.by_tiles_c.div(blockIdx.x), tc = blockIdx.x - tr * p.tiles_c;
  const unsigned r0 = tr * 32u, c0 = tc * 32u;
  const unsigned tx = threadIdx.x % LX, ty = threadIdx.x / LX;
  const unsigned rn = p.size[p.p_axis], cn = p.size[last];
  const long long sc = p.in_stride[last];
  for (unsigned rest = blockIdx.y; rest < p.nrest; rest += gridDim.y) {
    // the other axes: offsets of this tile's plane in the input and in the output
    long long in0 = 0, out0 = 0, out_stride = cn;
    unsigned rem = rest;
    for (int k = last - 1; k >= 0; --k) {
      if (k == p.p_axis) {
        out_stride *= p.size[k];
        continue;
      }
      const unsigned q = p.by_size[k].div(rem);
      const unsigned i = rem - q * p.size[k];
      rem = q;
      in0 += (long long)i * p.in_stride[k];
      out0 += (long long)i * out_stride;
      out_stride *= p.size[k];
    }
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const unsigned r = r0 + tx * VEC, row = ty + LY * j, c = c0 + row;
      if (r < rn && c < cn) {  // VEC > 1: rn is a multiple of VEC, so the whole piece is inside
        const W *src = x + in0 + r + (long long)c * sc;
        if constexpr (VEC == 1) {
          tile[row][tx] = *src;
        } else {
          const WV v = *reinterpret_cast<const WV *>(src);
#pragma unroll
          for (int k = 0; k < VEC; ++k) tile[row][tx * VEC + k] = v[k];
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      const unsigned c = c0 + tx * VEC, row = ty + LY * j, r = r0 + row;
      if (r < rn && c < cn) {
        W *dst = out + out0 + (long long)r * p.p_out_stride + c;
        if constexpr (VEC == 1) {
          *dst = tile[tx][row];
        } else {
          WV v;
#pragma unroll
          for (int k = 0; k < VEC; ++k) v[k] = tile[tx * VEC + k][row];
          *reinterpret_cast<WV *>(dst) = v;
        }
      }
    }
    __syncthreads();
  }
}

// ------------------------------------------------------------------------------------------
// Copy between a dense array and an array addressed through arbitrary strides: element
// (i_0, ..., i_{nd-1}) of the dense side pairs with offset sum_k i_k * stride_k of the other.
// With a stride that is the sum of two of a tensor's strides this walks a diagonal:
// gather takes it out (dense[t] = strided[off]), scatter writes it back (strided[off] =
// dense[t]; the offsets of distinct elements must differ).
// ------------------------------------------------------------------------------------------
struct StridedParams {
  int nd;
  unsigned size[kMaxPermuteAxes];
  long long stride[kMaxPermuteAxes];
  FastDivT by_size[kMaxPermuteAxes];
  unsigned total;
};

template <int BYTES, bool SCATTER>
__global__ void __launch_bounds__(256) strided_copy_kernel(StridedParams p, const typename Word<BYTES>::type *__restrict__ src,
                                                           typename Word<BYTES>::type *__restrict__ dst) {
  const unsigned t = blockIdx.x * 256u + threadIdx.x;
  if (t >= p.total) return;
  unsigned rem = t;
  long long off = 0;
  for (int k = p.nd - 1; k >= 0; --k) {
    const unsigned q = p.by_size[k].div(rem);
    off += (long long)(rem - q * p.size[k]) * p.stride[k];
    rem = q;
  }
  if (SCATTER)
    dst[off] = src[t];
  else
    dst[t] = src[off];
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_repeat_fwd(int elem_bytes, int64_t outer, int64_t n, int64_t inner, int64_t repeats, int64_t total, const int32_t *src_of,
                  const void *a, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return fail(MG_ERR_UNSUPPORTED, "mg_repeat_fwd: elements of %d bytes (1, 2, 4 or 8)", elem_bytes);
  const bool wide = inner > 0 && (inner * elem_bytes) % 16 == 0 && aligned16({a, out});
  RepeatParams p;
  if (int rc = repeat_params("mg_repeat_fwd", outer, n, inner, repeats, total, src_of == nullptr, wide ? 16 / elem_bytes : 1, &p))
    return rc;
  if (total == 0) return MG_OK;
  if (!a || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_repeat_fwd");
  ScopedTiming timed(TAG_REPEAT_FWD);
  const int64_t flat = outer * total;
  if (!src_of && inner == 1 && elem_bytes >= 4 && (flat * elem_bytes) % 16 == 0 && aligned16({out})) {
    const unsigned pieces = (unsigned)(flat * elem_bytes / 16);
    const dim3 grid((unsigned)ceil_div(pieces, 256)), block(256);
    if (elem_bytes == 4)
      hipLaunchKernelGGL(repeat_last_fwd_kernel<4>, grid, block, 0, runtime().stream, p.by_repeats, p.repeats, (const unsigned *)a,
                         (unsigned *)out, pieces);
    else
      hipLaunchKernelGGL(repeat_last_fwd_kernel<8>, grid, block, 0, runtime().stream, p.by_repeats, p.repeats,
                         (const unsigned long long *)a, (unsigned long long *)out, pieces);
  } else if (wide)
    launch_repeat_fwd<16>(p, src_of, a, out);
  else if (elem_bytes == 8)
    launch_repeat_fwd<8>(p, src_of, a, out);
  else if (elem_bytes == 4)
    launch_repeat_fwd<4>(p, src_of, a, out);
  else if (elem_bytes == 2)
    launch_repeat_fwd<2>(p, src_of, a, out);
  else
    launch_repeat_fwd<1>(p, src_of, a, out);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_repeat_bwd(int dtype, int64_t outer, int64_t n, int64_t inner, int64_t repeats, int64_t total, const int64_t *offsets,
                  const void *grad, void *da) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (dtype != MG_F32 && dtype != MG_F64) return fail(MG_ERR_UNSUPPORTED, "mg_repeat_bwd: dtype %d (only float32=0 / float64=1)", dtype);
  const int elem = dtype == MG_F32 ? 4 : 8;
  const bool wide = inner > 0 && (inner * elem) % 16 == 0 && aligned16({grad, da});
  RepeatParams p;
  if (int rc = repeat_params("mg_repeat_bwd", outer, n, inner, repeats, total, offsets == nullptr, wide ? 16 / elem : 1, &p)) return rc;
  if (!da || (total > 0 && !grad)) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_repeat_bwd");
  ScopedTiming timed(TAG_REPEAT_BWD);
  const int64_t flat = outer * n;
  if (!offsets && inner == 1 && repeats > 0 && (flat * elem) % 16 == 0 && aligned16({grad, da})) {
    const unsigned pieces = (unsigned)(flat * elem / 16);
    const dim3 grid((unsigned)ceil_div(pieces, 256)), block(256);
    if (dtype == MG_F32)
      hipLaunchKernelGGL(repeat_last_bwd_kernel<float>, grid, block, 0, runtime().stream, p.repeats, (const float *)grad, (float *)da, pieces);
    else
      hipLaunchKernelGGL(repeat_last_bwd_kernel<double>, grid, block, 0, runtime().stream, p.repeats, (const double *)grad, (double *)da,
                         pieces);
  } else if (dtype == MG_F32)
    launch_repeat_bwd<float>(p, wide, (const long long *)offsets, grad, da);
  else
    launch_repeat_bwd<double>(p, wide, (const long long *)offsets, grad, da);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_window_gather(const mg_window_desc *d, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (!d) return fail(MG_ERR_BAD_ARG, "mg_window_gather: descriptor is null");
  if (d->elem_bytes != 1 && d->elem_bytes != 2 && d->elem_bytes != 4 && d->elem_bytes != 8)
    return fail(MG_ERR_UNSUPPORTED, "mg_window_gather: elements of %d bytes (1, 2, 4 or 8)", d->elem_bytes);
  if (d->nd < 1 || d->nd > MG_MAX_ND) return fail(MG_ERR_UNSUPPORTED, "mg_window_gather: %d windowed axes (1..%d)", d->nd, MG_MAX_ND);
  if (d->lead < 1) return fail(MG_ERR_BAD_ARG, "mg_window_gather: lead=%lld must be positive", (long long)d->lead);
  WindowParams p{};
  p.nd = d->nd;
  int64_t xvol = 1, wvol = 1, gvol = 1;
  for (int k = MG_MAX_ND - 1; k >= 0; --k) {
    const int64_t X = d->X[k], W = d->W[k], S = d->S[k], D = d->D[k], G = d->G[k];
    if (X < 1 || W < 1 || S < 1 || D < 1 || G < 0)
      return fail(MG_ERR_BAD_ARG, "mg_window_gather: axis %d: X=%lld W=%lld step=%lld dilation=%lld G=%lld", k, (long long)X,
                  (long long)W, (long long)S, (long long)D, (long long)G);
    if (G > 0 && (G - 1) * S + (W - 1) * D + 1 > X)
      return fail(MG_ERR_BAD_ARG, "mg_window_gather: axis %d: %lld placements of a window spanning %lld at step %lld leave x (%lld)", k,
                  (long long)G, (long long)((W - 1) * D + 1), (long long)S, (long long)X);
    p.W[k] = (unsigned)W;
    p.G[k] = (unsigned)std::max<int64_t>(G, 1);
    p.step[k] = (unsigned)S;
    p.dil[k] = (unsigned)D;
    p.xstride[k] = (unsigned)xvol;
    p.by_w[k] = make_fastdiv_t((unsigned)W);
    p.by_g[k] = make_fastdiv_t(p.G[k]);
    xvol *= X;
    wvol *= W;
    gvol *= G;
    if (xvol > kMaxCount || wvol > kMaxCount || gvol > kMaxCount) return fail(MG_ERR_UNSUPPORTED, "mg_window_gather: more than 2^31 - 1 elements");
  }
  const int64_t count = gvol * d->lead * wvol;
  if (count > kMaxCount || d->lead * xvol > kMaxCount) return fail(MG_ERR_UNSUPPORTED, "mg_window_gather: more than 2^31 - 1 elements");
  if (count == 0) return MG_OK;
  if (!x || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_window_gather");
  p.lead = (unsigned)d->lead;
  p.wvol = (unsigned)wvol;
  p.xvol = (unsigned)xvol;
  p.by_wvol = make_fastdiv_t((unsigned)wvol);
  p.gvol = (unsigned)gvol;
  hipStream_t s = runtime().stream;
  const dim3 block(256);
  ScopedTiming timed(TAG_WINDOW_GATHER);

  // staged variant: 16 placements along the last axis per block, as many planes as 16 KiB of LDS
  // hold (eight blocks per compute unit; larger stages measured slower)
  constexpr int LAST = MG_MAX_ND - 1;
  WindowTile q{};
  q.tg = (unsigned)std::min<int64_t>(d->G[LAST], 16);
  q.rows = (unsigned)(wvol / d->W[LAST]);
  q.span_max = (unsigned)((q.tg - 1) * d->S[LAST] + (d->W[LAST] - 1) * d->D[LAST] + 1);
  const int64_t per_plane = (int64_t)q.rows * q.span_max * d->elem_bytes;
  const int64_t fit = (16 << 10) / std::max<int64_t>(per_plane, 1);
  q.tiles_last = (unsigned)ceil_div(d->G[LAST], q.tg);
  const int64_t groups = gvol / d->G[LAST] * q.tiles_last;
  if (q.rows <= kMaxWindowRows && wvol <= kMaxWindowVolume && fit >= 1 && groups <= kMaxCount) {
    q.planes = (unsigned)std::min<int64_t>({fit, d->lead, 256});
  }
  if (q.planes >= 1 && groups * ceil_div(d->lead, q.planes) <= kMaxCount) {
    for (unsigned r = 0; r < q.rows; ++r) {
      unsigned rest = r, offset = 0;
      for (int k = LAST - 1; k >= 0; --k) {
        offset += (rest % p.W[k]) * p.dil[k] * p.xstride[k];
        rest /= p.W[k];
      }
      q.row_offset[r] = offset;
    }
    const unsigned tail_g = (unsigned)(d->G[LAST] - (int64_t)(q.tiles_last - 1) * q.tg);
    q.by_tiles_last = make_fastdiv_t(q.tiles_last);
    q.by_rows = make_fastdiv_t(q.rows);
    q.by_span[0] = make_fastdiv_t(q.span_max);
    q.by_span[1] = make_fastdiv_t((unsigned)((tail_g - 1) * d->S[LAST] + (d->W[LAST] - 1) * d->D[LAST] + 1));
    q.hop_l = 256u / p.wvol;
    q.hop_w = 256u % p.wvol;
    q.by_wlast = make_fastdiv_t(p.W[LAST]);
    q.chunks = (unsigned)ceil_div(d->lead, q.planes);
    q.by_chunks = make_fastdiv_t(q.chunks);
    const dim3 tiles((unsigned)(groups * q.chunks));
    const size_t lds = (size_t)q.planes * per_plane;
    switch (d->elem_bytes) {
      case 8: hipLaunchKernelGGL(window_tile_kernel<8>, tiles, block, lds, s, p, q, (const unsigned long long *)x, (unsigned long long *)out); break;
      case 4: hipLaunchKernelGGL(window_tile_kernel<4>, tiles, block, lds, s, p, q, (const unsigned *)x, (unsigned *)out); break;
      case 2: hipLaunchKernelGGL(window_tile_kernel<2>, tiles, block, lds, s, p, q, (const unsigned short *)x, (unsigned short *)out); break;
      default: hipLaunchKernelGGL(window_tile_kernel<1>, tiles, block, lds, s, p, q, (const unsigned char *)x, (unsigned char *)out); break;
    }
    MG_HIP(hipGetLastError());
    return MG_OK;
  }

  // windows too large to stage: one placement per block, straight from x
  const dim3 grid((unsigned)(8 * ceil_div(gvol, 8)), (unsigned)std::min<int64_t>(ceil_div(d->lead * wvol, 256), 65535));
  switch (d->elem_bytes) {
    case 8: hipLaunchKernelGGL(window_gather_kernel<8>, grid, block, 0, s, p, (const unsigned long long *)x, (unsigned long long *)out); break;
    case 4: hipLaunchKernelGGL(window_gather_kernel<4>, grid, block, 0, s, p, (const unsigned *)x, (unsigned *)out); break;
    case 2: hipLaunchKernelGGL(window_gather_kernel<2>, grid, block, 0, s, p, (const unsigned short *)x, (unsigned short *)out); break;
    default: hipLaunchKernelGGL(window_gather_kernel<1>, grid, block, 0, s, p, (const unsigned char *)x, (unsigned char *)out); break;
  }
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_permute(int elem_bytes, int nd, const int64_t *shape, const int32_t *perm, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (elem_bytes != 4 && elem_bytes != 8) return fail(MG_ERR_UNSUPPORTED, "mg_permute: element size %d (4 or 8 bytes)", elem_bytes);
  if (nd < 0 || nd > 16 || (nd > 0 && (!shape || !perm))) return fail(MG_ERR_BAD_ARG, "mg_permute: nd = %d or null shape / perm", nd);
  long long total = 1;
  long long stride[16];
  bool seen[16] = {false};
  for (int k = nd - 1; k >= 0; --k) {
    if (shape[k] < 0) return fail(MG_ERR_BAD_ARG, "mg_permute: negative extent");
    if (perm[k] < 0 || perm[k] >= nd || seen[perm[k]]) return fail(MG_ERR_BAD_ARG, "mg_permute: perm is not a permutation of 0..%d", nd - 1);
    seen[perm[k]] = true;
    stride[k] = total;
    total *= shape[k];
    if (total >= (1ll << 31)) return fail(MG_ERR_UNSUPPORTED, "mg_permute: 2^31 or more elements");
  }
  if (total == 0) return MG_OK;
  if (!x || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_permute");
  // output axes as (extent, stride in the input); length-one axes dropped, neighbours that are
  // neighbours in the input too merged
  long long size[16], from[16];
  int m = 0;
  for (int i = 0; i < nd; ++i) {
    const long long n = shape[perm[i]], st = stride[perm[i]];
    if (n == 1) continue;
    if (m > 0 && from[m - 1] == st * n) {
      size[m - 1] *= n;
      from[m - 1] = st;
    } else {
      size[m] = n;
      from[m] = st;
      ++m;
    }
  }
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_PERMUTE);
  if (m <= 1) {  // the same order in memory
    MG_HIP(hipMemcpyAsync(out, x, (size_t)total * elem_bytes, hipMemcpyDeviceToDevice, s));
    return MG_OK;
  }
  if (m > kMaxPermuteAxes) return fail(MG_ERR_UNSUPPORTED, "mg_permute: %d axes left after merging (at most %d)", m, kMaxPermuteAxes);
  PermuteParams p{};
  p.nd = m;
  for (int k = 0; k < m; ++k) {
    p.size[k] = (unsigned)size[k];
    p.in_stride[k] = from[k];
    p.by_size[k] = make_fastdiv_t((unsigned)size[k]);
  }
  const dim3 block(256);
  if (from[m - 1] == 1) {
    // runs of size[m-1] elements; every other stride is a multiple of that run
    const long long run_bytes = size[m - 1] * elem_bytes;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out);
    const int piece = (run_bytes % 16 == 0 && bits % 16 == 0) ? 16 : elem_bytes;
    const long long epp = piece / elem_bytes;
    p.pieces = (unsigned)(run_bytes / piece);
    p.by_pieces = make_fastdiv_t(p.pieces);
    p.count = (unsigned)(total / epp);
    for (int k = 0; k < m - 1; ++k) p.in_stride[k] = from[k] / epp;
    const dim3 grid((unsigned)ceil_div((long long)p.count, 256));
    switch (piece) {
      case 16: hipLaunchKernelGGL(permute_rows_kernel<16>, grid, block, 0, s, p, (const Word16 *)x, (Word16 *)out); break;
      case 8: hipLaunchKernelGGL(permute_rows_kernel<8>, grid, block, 0, s, p, (const unsigned long long *)x, (unsigned long long *)out); break;
      default: hipLaunchKernelGGL(permute_rows_kernel<4>, grid, block, 0, s, p, (const unsigned *)x, (unsigned *)out); break;
    }
  } else {
    p.p_axis = -1;
    long long out_stride = 1, rest = 1;
    for (int k = m - 1; k >= 0; --k) {
      if (from[k] == 1) {
        p.p_axis = k;
        p.p_out_stride = out_stride;
      } else if (k != m - 1) {
        rest *= size[k];
      }
      out_stride *= size[k];
    }
    if (p.p_axis < 0) return fail(MG_ERR_HIP, "mg_permute: no output axis is the input's fastest one");
    p.tiles_c = (unsigned)ceil_div(size[m - 1], 32);
    p.tiles_r = (unsigned)ceil_div(size[p.p_axis], 32);
    p.by_tiles_c = make_fastdiv_t(p.tiles_c);
    p.nrest = (unsigned)rest;
    const dim3 grid(p.tiles_c * p.tiles_r, (unsigned)std::min<long long>(rest, 65535));
    // 16 bytes per lane when both tiled extents are whole pieces (every other stride on either
    // side is a multiple of one of them) and the tensors are aligned
    const long long per16 = 16 / elem_bytes;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out);
    const bool wide = size[p.p_axis] % per16 == 0 && size[m - 1] % per16 == 0 && bits % 16 == 0;
    if (elem_bytes == 8) {
      if (wide)
        hipLaunchKernelGGL((permute_tile_kernel<8, 2>), grid, block, 0, s, p, (const unsigned long long *)x, (unsigned long long *)out);
      else
        hipLaunchKernelGGL((permute_tile_kernel<8, 1>), grid, block, 0, s, p, (const unsigned long long *)x, (unsigned long long *)out);
    } else {
      if (wide)
        hipLaunchKernelGGL((permute_tile_kernel<4, 4>), grid, block, 0, s, p, (const unsigned *)x, (unsigned *)out);
      else
        hipLaunchKernelGGL((permute_tile_kernel<4, 1>), grid, block, 0, s, p, (const unsigned *)x, (unsigned *)out);
    }
  }
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_strided_copy(int elem_bytes, int nd, const int64_t *shape, const int64_t *strides, int64_t extent, int scatter, const void *x,
                    void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (elem_bytes != 4 && elem_bytes != 8) return fail(MG_ERR_UNSUPPORTED, "mg_strided_copy: element size %d (4 or 8 bytes)", elem_bytes);
  if (nd < 1 || nd > kMaxPermuteAxes || !shape || !strides)
    return fail(MG_ERR_BAD_ARG, "mg_strided_copy: nd = %d (1..%d) or null shape / strides", nd, kMaxPermuteAxes);
  StridedParams p{};
  p.nd = nd;
  long long total = 1, reach = 0;
  for (int k = 0; k < nd; ++k) {
    if (shape[k] < 0 || strides[k] < 0) return fail(MG_ERR_BAD_ARG, "mg_strided_copy: negative extent or stride");
    total *= shape[k];
    if (total >= (1ll << 31)) return fail(MG_ERR_UNSUPPORTED, "mg_strided_copy: 2^31 or more elements");
    if (shape[k] > 0) reach += (shape[k] - 1) * strides[k];
    p.size[k] = (unsigned)shape[k];
    p.stride[k] = strides[k];
    p.by_size[k] = make_fastdiv_t((unsigned)std::max<int64_t>(shape[k], 1));
  }
  if (total == 0) return MG_OK;
  if (reach >= extent) return fail(MG_ERR_BAD_ARG, "mg_strided_copy: the strides reach element %lld of %lld", reach, (long long)extent);
  if (!x || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_strided_copy");
  p.total = (unsigned)total;
  hipStream_t s = runtime().stream;
  const dim3 grid((unsigned)ceil_div(total, 256)), block(256);
  ScopedTiming timed(TAG_PERMUTE);
#define MG_STRIDED(BYTES, W)                                                                                        \
  do {                                                                                                              \
    if (scatter)                                                                                                    \
      hipLaunchKernelGGL((strided_copy_kernel<BYTES, true>), grid, block, 0, s, p, (const W *)x, (W *)out);         \
    else                                                                                                            \
      hipLaunchKernelGGL((strided_copy_kernel<BYTES, false>), grid, block, 0, s, p, (const W *)x, (W *)out);        \
  } while (0)
  if (elem_bytes == 8)
    MG_STRIDED(8, unsigned long long);
  else
    MG_STRIDED(4, unsigned);
#undef MG_STRIDED
  MG_HIP(hipGetLastError());
  return MG_OK;
}

}  // extern "C"
