// Batch normalisation over every axis but axis 1 of x:(N, C, S...) for gfx950.
//
//   mean_c = E[x_c], var_c = E[(x_c - mean_c)^2]          (over the N * S elements of channel c)
//   y      = (x - mean_c) / sqrt(var_c + eps) [* gamma_c] [+ beta_c]
//   dx     = ((g - E[g_c]) - xn * sum_c(g * xn) / (N*S)) / sqrt(var_c + eps) [* gamma_c]
//   dgamma = sum_c(g * xn),  dbeta = sum_c(g)              with xn = (x - mean_c) / std_c
//
// Bandwidth-bound: one reduction pass and one element-wise pass in each direction.  The
// reductions run over a fixed partition of each channel (the same blocks, the same tree,
// every run), carried in double; the element-wise arithmetic is done in the tensor's own
// precision in the order the reference applies its NumPy operations.
#include "internal.h"

#include <algorithm>

namespace mg {

namespace {

struct FastDivB {
  unsigned mul, shr, d, pad_;
  __device__ __forceinline__ unsigned div(unsigned n) const { return d == 1u ? n : __umulhi(n, mul) >> shr; }
};

FastDivB make_fastdiv_b(unsigned d) {
  FastDivB f{0u, 0u, d, 0u};
  if (d > 1u) {
    unsigned lg = 0;
    while ((1ull << lg) < d) ++lg;
    const unsigned p = 31u + lg;
    f.mul = (unsigned)(((1ull << p) + d - 1ull) / d);
    f.shr = p - 32u;
  }
  return f;
}

// How the threads of a launch walk a channel.
//   ROWS / ROWS_WIDE  block (chunk j, channel c) takes elements [j*chunk, (j+1)*chunk) of the
//                     channel's N*S elements, one (ROWS) or 16 bytes (ROWS_WIDE: S is a
//                     multiple of the vector width, so a piece never leaves its row of S) per
//                     lane: coalesced when S is long.
//   COLS              x seen as an (N, C*S) matrix: thread j takes column j = c*S + s, block
//                     row `blockIdx.y` takes `chunk` of the N rows: coalesced across channels
//                     when S is short (down to S = 1, the (N, C) batch of a dense layer).
enum Walk { ROWS = 0, ROWS_WIDE = 1, COLS = 2 };

struct BnParams {
  int N, C, S;
  int M;          // N * S, elements per channel (< 2^31)
  int J;          // C * S, columns of the (N, C*S) view
  int walk;       // Walk the host chose (ROWS stands for both row walks)
  int chunks;     // pieces a channel (ROWS*) or the batch axis (COLS) is cut into
  int chunk;      // ROWS*: elements of a channel per block; COLS: rows per block
  int terms;      // partial sums per channel: chunks (ROWS*) or chunks * S (COLS)
  FastDivB by_s;  // division by S
  int c0;         // row walks: channel of blockIdx.y == 0 (launches of at most 65535 channels each)
  double eps;
  int has_gamma, has_beta;
};

template <typename T>
struct Wide {
  static constexpr int N = 16 / sizeof(T);
  typedef T type __attribute__((ext_vector_type(N)));
};

// Sum over the 64 lanes of a wavefront by exchanges at distance 32, 16, ... 1: both partners
// of an exchange add the same two numbers, so every lane ends with the same bits.
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int distance = 32; distance > 0; distance >>= 1) v += __shfl_xor(v, distance, 64);
  return v;
}

// Two sums over the 256 threads of a block: wavefront sums, then the four of them in order.
// `slots` holds 8 doubles; one barrier.
__device__ __forceinline__ void block_sum2(double &a, double &b, double *slots) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    slots[wave] = a;
    slots[4 + wave] = b;
  }
  __syncthreads();
  a = ((slots[0] + slots[1]) + slots[2]) + slots[3];
  b = ((slots[4] + slots[5]) + slots[6]) + slots[7];
}

// The channel this thread works on, and whether it has work at all (COLS: columns past the
// last one idle).
template <int WALK>
__device__ __forceinline__ int my_channel(const BnParams &p, bool *active) {
  if constexpr (WALK == COLS) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    *active = j < p.J;
    return (int)p.by_s.div((unsigned)min(j, p.J - 1));
  } else {
    *active = true;
    return p.c0 + blockIdx.y;
  }
}

// Hands `f` the offset in x of every element (ROWS, COLS) or 16-byte piece (ROWS_WIDE) of this
// thread's share.
template <typename T, int WALK, typename F>
__device__ __forceinline__ void visit(const BnParams &p, F f) {
  if constexpr (WALK == COLS) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    const int first = blockIdx.y * p.chunk, last = min(first + p.chunk, p.N);
#pragma unroll 4
    for (int n = first; n < last; ++n) f((long long)n * p.J + j);
  } else {
    constexpr int VEC = WALK == ROWS_WIDE ? Wide<T>::N : 1;
    const int c = p.c0 + blockIdx.y;
    const int begin = blockIdx.x * p.chunk, end = min(begin + p.chunk, p.M);
#pragma unroll 4
    for (int e = begin + (int)threadIdx.x * VEC; e < end; e += 256 * VEC) {
      const unsigned n = p.by_s.div((unsigned)e);
      const unsigned s = (unsigned)e - n * (unsigned)p.S;
      f(((long long)n * p.C + c) * p.S + s);
    }
  }
}

// Index (in pairs of doubles) of partial sum `t` of channel `c`, t in [0, terms).
__device__ __forceinline__ long long term_index(const BnParams &p, int c, int t) {
  if (p.walk != COLS) return (long long)c * p.chunks + t;
  const int piece = (int)p.by_s.div((unsigned)t);
  return (long long)piece * p.J + (long long)c * p.S + (t - piece * p.S);
}

// Leaves this thread's (COLS) or this block's (ROWS*) pair of sums where term_index finds it.
template <int WALK>
__device__ __forceinline__ void put_partial(const BnParams &p, int c, bool active, double a, double b, double *partial,
                                            double *slots) {
  if constexpr (WALK == COLS) {
    if (!active) return;
    double *out = partial + ((long long)blockIdx.y * p.J + blockIdx.x * 256 + threadIdx.x) * 2;
    out[0] = a;
    out[1] = b;
  } else {
    block_sum2(a, b, slots);
    if (threadIdx.x == 0) {
      double *out = partial + ((long long)c * p.chunks + blockIdx.x) * 2;
      out[0] = a;
      out[1] = b;
    }
  }
}

// One wavefront per channel adds the channel's partial sums: lane l takes terms l, l + 64, ...
// in order, then the lanes are summed.
__device__ __forceinline__ void channel_totals(const BnParams &p, int c, const double *__restrict__ partial, double *a, double *b) {
  const int lane = threadIdx.x & 63;
  double sa = 0.0, sb = 0.0;
  for (int t = lane; t < p.terms; t += 64) {
    const long long at = term_index(p, c, t) * 2;
    sa += partial[at];
    sb += partial[at + 1];
  }
  *a = wave_sum(sa);
  *b = wave_sum(sb);
}

// The pilot value of channel c: the mean of a few samples spread evenly over the channel (64
// per wavefront for the row walks, 8 per thread for the column walk).  Every thread of a
// launch that works on channel c forms it from the same samples in the same order, so all of
// them subtract the same number.  It only has to be near the mean: sums of (x - pilot) and
// (x - pilot)^2 then lose nothing to cancellation, where sums of x and x^2 would.
template <typename T, int WALK>
__device__ __forceinline__ double pilot_of(const BnParams &p, const T *__restrict__ x, int c) {
  if constexpr (WALK == COLS) {
    const int count = min(p.N, 8);
    double sum = 0.0;
    for (int i = 0; i < count; ++i) sum += (double)x[(((long long)i * p.N) >> 3) * p.J + (long long)c * p.S];
    const double pilot = sum / count;
    return isfinite(pilot) ? pilot : 0.0;
  } else {
    const int lane = threadIdx.x & 63;
    double sample = 0.0;
    if (lane < p.M) {
      const unsigned e = p.M >= 64 ? (unsigned)(((long long)lane * p.M) >> 6) : (unsigned)lane;
      const unsigned n = p.by_s.div(e);
      sample = (double)x[((long long)n * p.C + c) * p.S + (e - n * (unsigned)p.S)];
    }
    const double pilot = wave_sum(sample) / (double)min(p.M, 64);
    return isfinite(pilot) ? pilot : 0.0;  // an infinite sample must still give an infinite mean, not inf - inf
  }
}

// mean and variance of a channel from the totals of (x - pilot) and (x - pilot)^2, rounded once
template <typename T>
__device__ __forceinline__ void write_stats(const BnParams &p, int c, double sd, double sdd, double pilot, T *mean, T *var) {
  const double m = sd / p.M;
  mean[c] = (T)(pilot + m);
  const double v = sdd / p.M - m * m;
  var[c] = (T)(v < 0.0 ? 0.0 : v);  // rounding may leave a tiny negative value; a NaN stays a NaN
}

// sums[c] = (sum g, sum g * xn) in double from the totals of g and g * (x - mean); dbeta and
// dgamma are the same rounded to T
template <typename T>
__device__ __forceinline__ void write_bwd_sums(const BnParams &p, int c, double sg, double sgx, const T *var, double *sums, T *dgamma,
                                               T *dbeta) {
  sgx /= (double)(T)sqrt(var[c] + (T)p.eps);
  sums[2 * c] = sg;
  sums[2 * c + 1] = sgx;
  if (dbeta) dbeta[c] = (T)sg;
  if (dgamma) dgamma[c] = (T)sgx;
}

// Partial sums of (x - pilot_c) and (x - pilot_c)^2; the pilots go behind the partial sums.
template <typename T, int WALK>
__global__ void __launch_bounds__(256) bn_stats_kernel(BnParams p, const T *__restrict__ x, double *__restrict__ partial) {
  typedef typename Wide<T>::type V;
  __shared__ double slots[8];
  bool active;
  const int c = my_channel<WALK>(p, &active);
  const double pilot = pilot_of<T, WALK>(p, x, c);
  double sd = 0.0, sdd = 0.0;
  if (active)
    visit<T, WALK>(p, [&](long long at) {
      if constexpr (WALK == ROWS_WIDE) {
        const V v = *reinterpret_cast<const V *>(x + at);
#pragma unroll
        for (int k = 0; k < Wide<T>::N; ++k) {
          const double d = (double)v[k] - pilot;
          sd += d;
          sdd += d * d;
        }
      } else {
        const double d = (double)x[at] - pilot;
        sd += d;
        sdd += d * d;
      }
    });
  put_partial<WALK>(p, c, active, sd, sdd, partial, slots);
  double *pilots = partial + (long long)p.C * p.terms * 2;
  if constexpr (WALK == COLS) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (active && blockIdx.y == 0 && j == c * p.S) pilots[c] = pilot;
  } else {
    if (blockIdx.x == 0 && threadIdx.x == 0) pilots[c] = pilot;
  }
}

// mean and variance of each channel
template <typename T>
__global__ void __launch_bounds__(256) bn_finish_stats_kernel(BnParams p, const double *__restrict__ partial, T *__restrict__ mean,
                                                              T *__restrict__ var) {
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= p.C) return;
  double sd, sdd;
  channel_totals(p, c, partial, &sd, &sdd);
  if ((threadIdx.x & 63) != 0) return;
  write_stats(p, c, sd, sdd, partial[(long long)p.C * p.terms * 2 + c], mean, var);
}

// y = (x - mean) / std [* gamma] [+ beta], each step rounded in T like the reference's
// sequence of array operations; std = sqrt(var + eps) in T.
template <typename T, int WALK>
__global__ void __launch_bounds__(256) bn_apply_kernel(BnParams p, const T *__restrict__ x, const T *__restrict__ mean,
                                                       const T *__restrict__ var, const T *__restrict__ gamma,
                                                       const T *__restrict__ beta, T *__restrict__ y) {
  typedef typename Wide<T>::type V;
  bool active;
  const int c = my_channel<WALK>(p, &active);
  if (!active) return;
  const T m = mean[c];
  const T sd = (T)sqrt(var[c] + (T)p.eps);
  const T ga = p.has_gamma ? gamma[c] : T(1);
  const T be = p.has_beta ? beta[c] : T(0);
  auto one = [&](T v) -> T {
    T r = (v - m) / sd;
    if (p.has_gamma) r = r * ga;
    if (p.has_beta) r = r + be;
    return r;
  };
  visit<T, WALK>(p, [&](long long at) {
    if constexpr (WALK == ROWS_WIDE) {
      const V v = *reinterpret_cast<const V *>(x + at);
      V r;
#pragma unroll
      for (int k = 0; k < Wide<T>::N; ++k) r[k] = one(v[k]);
      *reinterpret_cast<V *>(y + at) = r;
    } else {
      y[at] = one(x[at]);
    }
  });
}

// Partial sums of g and of g * (x - mean), in double; the division by std that turns the
// second into sum(g * xn) is done once per channel afterwards.
template <typename T, int WALK>
__global__ void __launch_bounds__(256) bn_bwd_sums_kernel(BnParams p, const T *__restrict__ x, const T *__restrict__ g,
                                                          const T *__restrict__ mean, double *__restrict__ partial) {
  typedef typename Wide<T>::type V;
  __shared__ double slots[8];
  bool active;
  const int c = my_channel<WALK>(p, &active);
  const double m = (double)mean[c];
  double sg = 0.0, sgx = 0.0;
  if (active)
    visit<T, WALK>(p, [&](long long at) {
      if constexpr (WALK == ROWS_WIDE) {
        const V xv = *reinterpret_cast<const V *>(x + at);
        const V gv = *reinterpret_cast<const V *>(g + at);
#pragma unroll
        for (int k = 0; k < Wide<T>::N; ++k) {
          sg += (double)gv[k];
          sgx += (double)gv[k] * ((double)xv[k] - m);
        }
      } else {
        sg += (double)g[at];
        sgx += (double)g[at] * ((double)x[at] - m);
      }
    });
  put_partial<WALK>(p, c, active, sg, sgx, partial, slots);
}

// the channel sums of the backward pass
template <typename T>
__global__ void __launch_bounds__(256) bn_finish_bwd_kernel(BnParams p, const double *__restrict__ partial, const T *__restrict__ var,
                                                            double *__restrict__ sums, T *__restrict__ dgamma, T *__restrict__ dbeta) {
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= p.C) return;
  double sg, sgx;
  channel_totals(p, c, partial, &sg, &sgx);
  if ((threadIdx.x & 63) == 0) write_bwd_sums(p, c, sg, sgx, var, sums, dgamma, dbeta);
}

// dx = (((g - mean_g) - xn * (dot / M)) / std) [* gamma], each step rounded in T, in the
// reference's order (batchnorm.py:86-100) but for dot / M, which is formed once per channel
template <typename T, int WALK>
__global__ void __launch_bounds__(256) bn_bwd_apply_kernel(BnParams p, const T *__restrict__ x, const T *__restrict__ g,
                                                           const T *__restrict__ mean, const T *__restrict__ var,
                                                           const T *__restrict__ gamma, const double *__restrict__ sums,
                                                           T *__restrict__ dx) {
  typedef typename Wide<T>::type V;
  bool active;
  const int c = my_channel<WALK>(p, &active);
  if (!active) return;
  const T m = mean[c];
  const T sd = (T)sqrt(var[c] + (T)p.eps);
  const T mean_g = (T)(sums[2 * c] / p.M);
  const T share = (T)sums[2 * c + 1] / (T)p.M;  // sum_c(g * xn) / count, once per channel
  const T ga = p.has_gamma ? gamma[c] : T(1);
  auto one = [&](T xv, T gv) -> T {
    const T xn = (xv - m) / sd;
    T r = gv - mean_g;
    r = r - xn * share;
    r = r / sd;
    if (p.has_gamma) r = r * ga;
    return r;
  };
  visit<T, WALK>(p, [&](long long at) {
    if constexpr (WALK == ROWS_WIDE) {
      const V xv = *reinterpret_cast<const V *>(x + at);
      const V gv = *reinterpret_cast<const V *>(g + at);
      V r;
#pragma unroll
      for (int k = 0; k < Wide<T>::N; ++k) r[k] = one(xv[k], gv[k]);
      *reinterpret_cast<V *>(dx + at) = r;
    } else {
      dx[at] = one(x[at], g[at]);
    }
  });
}

// ------------------------------------------------------------------------------------------
// Plain sums over the same walks: out[c] = sum over n and s of x[n, c, s], carried in double
// over the same fixed partition and trees as the statistics above.
// ------------------------------------------------------------------------------------------
template <typename T, int WALK, bool PRODUCT>
__device__ __forceinline__ void axis_sum_body(const BnParams &p, const T *__restrict__ x, const T *__restrict__ y, double *__restrict__ partial) {
  typedef typename Wide<T>::type V;
  __shared__ double slots[8];
  bool active;
  const int c = my_channel<WALK>(p, &active);
  double even = 0.0, odd = 0.0;  // two running sums, added at the end
  if (active)
    visit<T, WALK>(p, [&](long long at) {
#pragma clang fp contract(off)  // the product is rounded to T, like a product formed first: no fused multiply-add
      if constexpr (WALK == ROWS_WIDE) {
        V v = *reinterpret_cast<const V *>(x + at);
        if constexpr (PRODUCT) v = v * *reinterpret_cast<const V *>(y + at);
#pragma unroll
        for (int k = 0; k < Wide<T>::N; k += 2) {
          even += (double)v[k];
          odd += (double)v[k + 1];
        }
      } else {
        T v = x[at];
        if constexpr (PRODUCT) v = v * y[at];
        even += (double)v;
      }
    });
  put_partial<WALK>(p, c, active, even, odd, partial, slots);
}

template <typename T, int WALK>
__global__ void __launch_bounds__(256) axis_sum_kernel(BnParams p, const T *__restrict__ x, double *__restrict__ partial) {
  axis_sum_body<T, WALK, false>(p, x, nullptr, partial);
}

// The same sum of x * y: the product is rounded to T before it is added, so the result is
// that of multiplying first and summing afterwards, in one pass over both operands.
template <typename T, int WALK>
__global__ void __launch_bounds__(256) axis_sum_product_kernel(BnParams p, const T *__restrict__ x, const T *__restrict__ y,
                                                               double *__restrict__ partial) {
  axis_sum_body<T, WALK, true>(p, x, y, partial);
}

template <typename T>
__global__ void __launch_bounds__(256) axis_sum_finish_kernel(BnParams p, const double *__restrict__ partial, T *__restrict__ out) {
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= p.C) return;
  double even, odd;
  channel_totals(p, c, partial, &even, &odd);
  if ((threadIdx.x & 63) == 0) out[c] = (T)(even + odd);
}

// out[o, i] = sum over m of x[o, m, i] for x:(outer, n, inner).  A thread owns VEC consecutive
// i of one o and walks `chunk` of the n entries of the middle axis, inner elements apart;
// lanes are consecutive in i, so each step of the walk is one coalesced access.  With more
// than one chunk the sums go to `partial` as doubles and a second kernel adds them in order.
struct MiddleParams {
  long long outer, outs;  // outs = outer * inner, results
  int n, inner;
  int chunk, chunks;
};

template <typename T, int VEC, bool PRODUCT>
__global__ void __launch_bounds__(256) sum_middle_kernel(MiddleParams p, const T *__restrict__ x, const T *__restrict__ y,
                                                         T *__restrict__ out, double *__restrict__ partial) {
  typedef T V __attribute__((ext_vector_type(VEC)));
  const long long piece = (long long)blockIdx.x * 256 + threadIdx.x;
  const int per_row = p.inner / VEC;
  if (piece >= p.outer * per_row) return;
  const long long o = piece / per_row;
  const int i = (int)(piece - o * per_row) * VEC;
  const int first = blockIdx.y * p.chunk, last = min(first + p.chunk, p.n);
  const long long start = (o * p.n + first) * p.inner + i;
  const T *src = x + start;
  const T *other = PRODUCT ? y + start : nullptr;  // x * y is rounded to T before it is added
  double acc[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) acc[k] = 0.0;
#pragma unroll 4
  for (int m = first; m < last; ++m) {
#pragma clang fp contract(off)  // no fused multiply-add: the product is rounded first
    if constexpr (VEC == 1) {
      T v = *src;
      if constexpr (PRODUCT) v = v * *other;
      acc[0] += (double)v;
    } else {
      V v = *reinterpret_cast<const V *>(src);
      if constexpr (PRODUCT) v = v * *reinterpret_cast<const V *>(other);
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[k] += (double)v[k];
    }
    src += p.inner;
    if constexpr (PRODUCT) other += p.inner;
  }
  const long long at = o * p.inner + i;
  if (p.chunks == 1) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) out[at + k] = (T)acc[k];
  } else {
#pragma unroll
    for (int k = 0; k < VEC; ++k) partial[(long long)blockIdx.y * p.outs + at + k] = acc[k];
  }
}

template <typename T>
__global__ void __launch_bounds__(256) sum_middle_finish_kernel(MiddleParams p, const double *__restrict__ partial, T *__restrict__ out) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e >= p.outs) return;
  double total = 0.0;
  for (int c = 0; c < p.chunks; ++c) total += partial[(long long)c * p.outs + e];
  out[e] = (T)total;
}

// many_channels: the caller cuts its launches to the grid's y extent of 65535 itself
int make_params(const mg_bn_desc *d, BnParams *p, const char *who, bool many_channels = false) {
  if (!d) return fail(MG_ERR_BAD_ARG, "%s: descriptor is null", who);
  if (d->dtype != MG_F32 && d->dtype != MG_F64) return fail(MG_ERR_UNSUPPORTED, "%s: dtype %d (only float32=0 / float64=1)", who, d->dtype);
  if (d->N < 1 || d->C < 1 || d->S < 1) return fail(MG_ERR_BAD_ARG, "%s: N=%lld C=%lld S=%lld must be positive", who, (long long)d->N, (long long)d->C, (long long)d->S);
  if (d->N * d->S >= (1ll << 31) || d->C * d->S >= (1ll << 31) || (d->C > 65535 && !many_channels))
    return fail(MG_ERR_UNSUPPORTED, "%s: 2^31 or more elements per channel or per batch entry, or more than 65535 channels", who);
  if (!(d->eps >= 0.0)) return fail(MG_ERR_BAD_ARG, "%s: eps = %g must be non-negative", who, d->eps);
  p->N = (int)d->N;
  p->C = (int)d->C;
  p->S = (int)d->S;
  p->M = (int)(d->N * d->S);
  p->J = (int)(d->C * d->S);
  p->eps = d->eps;
  p->has_gamma = d->has_gamma != 0;
  p->has_beta = d->has_beta != 0;
  p->by_s = make_fastdiv_b((unsigned)d->S);
  p->c0 = 0;
  const long long slots = 16ll * runtime().props.multiProcessorCount;  // blocks wanted: 16 per compute unit
  if (d->S < 64) {
    // short rows: walk columns.  32 to 256 rows per block: enough blocks to fill the device
    // (four per compute unit when the batch allows) while the partial sums stay a small
    // fraction of x; no more than 65535 pieces (the grid's y extent)
    p->walk = COLS;
    const long long across = ceil_div((long long)p->J, 256);
    const long long balanced = std::min<long long>(256, std::max<long long>(32, (long long)p->N * across / (4ll * runtime().props.multiProcessorCount)));
    p->chunk = (int)std::max<long long>(balanced, ceil_div((long long)p->N, 65535));
    p->chunks = (int)ceil_div((long long)p->N, p->chunk);
    p->terms = p->chunks * p->S;
  } else {
    p->walk = ROWS;
    const long long want = std::max<long long>(1, slots / d->C);
    const long long unit = 1024;  // elements; a multiple of every vector width
    p->chunk = (int)std::max<long long>(unit, ceil_div(ceil_div((long long)p->M, want), unit) * unit);
    p->chunks = (int)ceil_div((long long)p->M, p->chunk);
    p->terms = p->chunks;
  }
  return MG_OK;
}

// ROWS_WIDE when every row of S is a whole number of aligned 16-byte pieces
int walk_for(const BnParams &p, size_t elem, std::initializer_list<const void *> ptrs) {
  if (p.walk == COLS) return COLS;
  if (p.S % (int)(16 / elem) != 0) return ROWS;
  for (const void *q : ptrs)
    if (q && reinterpret_cast<uintptr_t>(q) % 16 != 0) return ROWS;
  return ROWS_WIDE;
}

dim3 grid_for(const BnParams &p) {
  return p.walk == COLS ? dim3((unsigned)ceil_div(p.J, 256), (unsigned)p.chunks) : dim3((unsigned)p.chunks, (unsigned)p.C);
}

// launches KERNEL<T, walk> for the walk chosen at run time
#define MG_BN_LAUNCH(KERNEL, walk, ...)                                                                  \
  do {                                                                                                   \
    if ((walk) == COLS)                                                                                  \
      hipLaunchKernelGGL((KERNEL<T, COLS>), grid, block, 0, s, __VA_ARGS__);                             \
    else if ((walk) == ROWS_WIDE)                                                                        \
      hipLaunchKernelGGL((KERNEL<T, ROWS_WIDE>), grid, block, 0, s, __VA_ARGS__);                        \
    else                                                                                                 \
      hipLaunchKernelGGL((KERNEL<T, ROWS>), grid, block, 0, s, __VA_ARGS__);                             \
  } while (0)

template <typename T>
int fwd_impl(const BnParams &p, const void *x, const void *gamma, const void *beta, void *y, void *mean, void *var) {
  hipStream_t s = runtime().stream;
  void *partial = nullptr;
  if (int rc = workspace(((size_t)p.C * p.terms * 2 + p.C) * sizeof(double), &partial)) return rc;
  const dim3 grid = grid_for(p), block(256);
  const int walk = walk_for(p, sizeof(T), {x, y});
  {
    ScopedTiming timed(TAG_BN_STATS);
    MG_BN_LAUNCH(bn_stats_kernel, walk, p, (const T *)x, (double *)partial);
    hipLaunchKernelGGL(bn_finish_stats_kernel<T>, dim3((unsigned)ceil_div(p.C, 4)), block, 0, s, p, (const double *)partial,
                       (T *)mean, (T *)var);
  }
  {
    ScopedTiming timed(TAG_BN_APPLY);
    MG_BN_LAUNCH(bn_apply_kernel, walk, p, (const T *)x, (const T *)mean, (const T *)var, (const T *)gamma, (const T *)beta, (T *)y);
  }
  MG_HIP(hipGetLastError());
  return MG_OK;
}

template <typename T>
int bwd_impl(const BnParams &p, const void *x, const void *grad, const void *gamma, const void *mean, const void *var, void *dx,
             void *dgamma, void *dbeta) {
  hipStream_t s = runtime().stream;
  void *scratch = nullptr;
  const size_t partial_doubles = (size_t)p.C * p.terms * 2;
  if (int rc = workspace((partial_doubles + (size_t)p.C * 2) * sizeof(double), &scratch)) return rc;
  double *partial = static_cast<double *>(scratch);
  double *sums = partial + partial_doubles;
  const dim3 grid = grid_for(p), block(256);
  const int walk = walk_for(p, sizeof(T), {x, grad, dx});
  {
    ScopedTiming timed(TAG_BN_BWD_SUMS);
    MG_BN_LAUNCH(bn_bwd_sums_kernel, walk, p, (const T *)x, (const T *)grad, (const T *)mean, partial);
    hipLaunchKernelGGL(bn_finish_bwd_kernel<T>, dim3((unsigned)ceil_div(p.C, 4)), block, 0, s, p, (const double *)partial,
                       (const T *)var, sums, (T *)dgamma, (T *)dbeta);
  }
  if (dx) {
    ScopedTiming timed(TAG_BN_BWD_APPLY);
    MG_BN_LAUNCH(bn_bwd_apply_kernel, walk, p, (const T *)x, (const T *)grad, (const T *)mean, (const T *)var, (const T *)gamma,
                 (const double *)sums, (T *)dx);
  }
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// out[c] = sum over n, s of x[n, c, s] (times y[n, c, s] if y is given)
template <typename T>
int axis_sum_impl(BnParams p, const void *x, const void *y, void *out) {
  hipStream_t s = runtime().stream;
  void *partial = nullptr;
  if (int rc = workspace((size_t)p.C * p.terms * 2 * sizeof(double), &partial)) return rc;
  const dim3 block(256);
  const int walk = y ? walk_for(p, sizeof(T), {x, y}) : walk_for(p, sizeof(T), {x});
  ScopedTiming timed(TAG_SUM_OVER);
  auto launch = [&](const dim3 grid) {
    if (y)
      MG_BN_LAUNCH(axis_sum_product_kernel, walk, p, (const T *)x, (const T *)y, (double *)partial);
    else
      MG_BN_LAUNCH(axis_sum_kernel, walk, p, (const T *)x, (double *)partial);
  };
  if (p.walk == COLS) {
    launch(grid_for(p));
  } else {
    const int channels = p.C;
    for (int c0 = 0; c0 < channels; c0 += 65535) {  // the grid's y extent
      p.c0 = c0;
      launch(dim3((unsigned)p.chunks, (unsigned)std::min(65535, channels - c0)));
    }
    p.c0 = 0;
  }
  hipLaunchKernelGGL(axis_sum_finish_kernel<T>, dim3((unsigned)ceil_div(p.C, 4)), block, 0, s, p, (const double *)partial, (T *)out);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// out[o, i] = sum over m of x[o, m, i] (times y[o, m, i] if y is given)
template <typename T>
int middle_sum_impl(long long outer, long long n, long long inner, const void *x, const void *y, void *out) {
  hipStream_t s = runtime().stream;
  constexpr int WIDE = 16 / sizeof(T);
  const bool wide = inner % WIDE == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int vec = wide ? WIDE : 1;
  MiddleParams p;
  p.outer = outer;
  p.outs = outer * inner;
  p.n = (int)n;
  p.inner = (int)inner;
  const long long blocks = ceil_div(outer * (inner / vec), 256);
  // few results and a long middle axis: cut the axis so that about four blocks per compute
  // unit are in flight, no piece shorter than 16 entries
  const long long want = 4ll * runtime().props.multiProcessorCount;
  long long chunks = std::max<long long>(1, std::min<long long>(ceil_div(want, blocks), n / 16));
  chunks = std::min<long long>(chunks, 65535);
  p.chunk = (int)ceil_div(n, chunks);
  p.chunks = (int)ceil_div(n, p.chunk);
  void *partial = nullptr;
  if (p.chunks > 1)
    if (int rc = workspace((size_t)p.chunks * p.outs * sizeof(double), &partial)) return rc;
  const dim3 grid((unsigned)blocks, (unsigned)p.chunks), block(256);
  ScopedTiming timed(TAG_SUM_OVER);
#define MG_MIDDLE(VEC, PRODUCT) \
  hipLaunchKernelGGL((sum_middle_kernel<T, VEC, PRODUCT>), grid, block, 0, s, p, (const T *)x, (const T *)y, (T *)out, (double *)partial)
  if (wide) {
    if (y) MG_MIDDLE(WIDE, true); else MG_MIDDLE(WIDE, false);
  } else {
    if (y) MG_MIDDLE(1, true); else MG_MIDDLE(1, false);
  }
#undef MG_MIDDLE
  if (p.chunks > 1)
    hipLaunchKernelGGL(sum_middle_finish_kernel<T>, dim3((unsigned)ceil_div(p.outs, 256)), block, 0, s, p, (const double *)partial, (T *)out);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

#undef MG_BN_LAUNCH

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_batchnorm_fwd(const mg_bn_desc *desc, const void *x, const void *gamma, const void *beta, void *y, void *mean, void *var) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  BnParams p;
  if (int rc = make_params(desc, &p, "mg_batchnorm_fwd")) return rc;
  if (!x || !y || !mean || !var) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_batchnorm_fwd");
  if ((p.has_gamma && !gamma) || (p.has_beta && !beta)) return fail(MG_ERR_BAD_ARG, "mg_batchnorm_fwd: gamma / beta announced but null");
  return desc->dtype == MG_F32 ? fwd_impl<float>(p, x, gamma, beta, y, mean, var) : fwd_impl<double>(p, x, gamma, beta, y, mean, var);
}

int mg_batchnorm_bwd(const mg_bn_desc *desc, const void *x, const void *grad, const void *gamma, const void *mean, const void *var,
                     void *dx, void *dgamma, void *dbeta) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  BnParams p;
  if (int rc = make_params(desc, &p, "mg_batchnorm_bwd")) return rc;
  if (!x || !grad || !mean || !var) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_batchnorm_bwd");
  if (p.has_gamma && !gamma) return fail(MG_ERR_BAD_ARG, "mg_batchnorm_bwd: gamma announced but null");
  if (!dx && !dgamma && !dbeta) return fail(MG_ERR_BAD_ARG, "mg_batchnorm_bwd: nothing to compute (dx, dgamma and dbeta are all null)");
  return desc->dtype == MG_F32 ? bwd_impl<float>(p, x, grad, gamma, mean, var, dx, dgamma, dbeta)
                               : bwd_impl<double>(p, x, grad, gamma, mean, var, dx, dgamma, dbeta);
}

namespace {
int sum_over(const char *who, int dtype, int64_t outer, int64_t n, int64_t inner, int over_middle, const void *x, const void *y, void *out);
}

int mg_sum_over(int dtype, int64_t outer, int64_t n, int64_t inner, int over_middle, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  return sum_over("mg_sum_over", dtype, outer, n, inner, over_middle, x, nullptr, out);
}

int mg_sum_product_over(int dtype, int64_t outer, int64_t n, int64_t inner, int over_middle, const void *x, const void *y, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (!y) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_sum_product_over");
  return sum_over("mg_sum_product_over", dtype, outer, n, inner, over_middle, x, y, out);
}

}  // extern "C"

namespace {

int sum_over(const char *who, int dtype, int64_t outer, int64_t n, int64_t inner, int over_middle, const void *x, const void *y, void *out) {
  if (dtype != MG_F32 && dtype != MG_F64) return fail(MG_ERR_UNSUPPORTED, "%s: dtype %d (only float32=0 / float64=1)", who, dtype);
  if (outer < 1 || n < 1 || inner < 1)
    return fail(MG_ERR_BAD_ARG, "%s: outer=%lld n=%lld inner=%lld must be positive", who, (long long)outer, (long long)n, (long long)inner);
  if (!x || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in %s", who);
  if (over_middle) {
    if (n >= (1ll << 31) || inner >= (1ll << 31) || ceil_div(outer * inner, 256) >= (1ll << 31))
      return fail(MG_ERR_UNSUPPORTED, "%s: an axis of 2^31 or more entries, or 2^39 or more results", who);
    return dtype == MG_F32 ? middle_sum_impl<float>(outer, n, inner, x, y, out) : middle_sum_impl<double>(outer, n, inner, x, y, out);
  }
  mg_bn_desc desc{};
  desc.dtype = dtype;
  desc.N = outer;
  desc.C = n;
  desc.S = inner;
  desc.eps = 0.0;
  BnParams p;
  if (int rc = make_params(&desc, &p, who, true)) return rc;
  return dtype == MG_F32 ? axis_sum_impl<float>(p, x, y, out) : axis_sum_impl<double>(p, x, y, out);
}

}  // namespace
