// Element-wise and whole-array kernels either side of conv_nd / max_pool in a chain
// such as conv -> relu -> pool -> (. * g) -> sum: bandwidth-bound, 16 bytes per lane.
//
//   multiply   out[i] = a[i] * b[i]            (one IEEE multiply: bit-exact with NumPy)
//              also with operands that are broadcast along some of the axes
//   relu       out[i] = x[i] * (x[i] > 0)      (so negative inputs give -0.0, NaN stays NaN)
//   relu bwd   dx[i]  = grad[i] * (x[i] > 0)
//   sum        *out   = sum_i x[i]             (fixed summation tree, carried in double)
//   fill       out[i] = *value
#include "internal.h"

#include <algorithm>
#include <type_traits>

namespace mg {

namespace {

template <typename T>
struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  typedef T type __attribute__((ext_vector_type(N)));
};

enum ElementwiseOp { EW_MUL = 0, EW_RELU = 1, EW_RELU_BWD = 2 };

template <typename T, int OP>
__device__ __forceinline__ T apply(T a, T b) {
  if constexpr (OP == EW_MUL) return a * b;
  if constexpr (OP == EW_RELU) return a * (a > T(0) ? T(1) : T(0));
  return b * (a > T(0) ? T(1) : T(0));  // a = x, b = grad
}

// out = op(a, b) over n elements; `a`, `b` and `out` are 16-byte aligned (device
// allocations are), the last n % VEC elements are handled one by one.
template <typename T, int OP>
__global__ void __launch_bounds__(256) elementwise_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                          T *__restrict__ out, long long n) {
  typedef typename Vec16<T>::type V;
  constexpr int VEC = Vec16<T>::N;
  const long long nvec = n / VEC;
  const long long stride = (long long)gridDim.x * 256;
  const V *va = reinterpret_cast<const V *>(a);
  const V *vb = reinterpret_cast<const V *>(b);
  V *vo = reinterpret_cast<V *>(out);
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  for (; i < nvec; i += stride) {
    const V x = va[i];
    V y = x;
    if constexpr (OP != EW_RELU) y = vb[i];
    V r;
#pragma unroll
    for (int k = 0; k < VEC; ++k) r[k] = apply<T, OP>(x[k], y[k]);
    vo[i] = r;
  }
  if (blockIdx.x == 0) {
    const long long i = nvec * VEC + threadIdx.x;
    if (i < n) out[i] = apply<T, OP>(a[i], OP != EW_RELU ? b[i] : a[i]);
  }
}

// out = a * b where each operand lacks some of the axes of `out` (NumPy's broadcasting).  The
// host merges neighbouring axes that both operands treat alike, so `out` is (d[0], ..., d[nd-1])
// with the last axis `inner` long; an operand's stride along an axis is 0 where it is
// broadcast, and along the last axis 1 or 0.  A thread makes VEC consecutive results of one
// row: an operand present along the last axis is read 16 bytes at a time, a broadcast one once.
struct BroadcastParams {
  int outer_dims;         // axes before the last one (at most 5)
  unsigned extent[5];     // their lengths, first axis first
  unsigned a_step[5], b_step[5];  // element strides of a and b along them
  unsigned a_inner, b_inner;      // 1 or 0: strides along the last axis
  unsigned inner, pieces;         // length of the last axis, ceil(inner / VEC)
  unsigned threads;               // rows x pieces
};

template <typename T, bool ALIGNED>
__global__ void __launch_bounds__(256) multiply_broadcast_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ out,
                                                                 BroadcastParams p) {
  typedef typename Vec16<T>::type V;
  constexpr int VEC = Vec16<T>::N;
  for (unsigned t = blockIdx.x * 256u + threadIdx.x; t < p.threads; t += gridDim.x * 256u) {
    const unsigned piece = t % p.pieces;
    unsigned row = t / p.pieces;
    const size_t at = (size_t)row * p.inner + (size_t)piece * VEC;  // in `out`
    unsigned ia = 0, ib = 0;
    for (int d = p.outer_dims - 1; d >= 0; --d) {
      const unsigned c = row % p.extent[d];
      row /= p.extent[d];
      ia += c * p.a_step[d];
      ib += c * p.b_step[d];
    }
    if constexpr (ALIGNED) {  // inner is a multiple of VEC: every piece is whole and 16-byte aligned in all three
      V x, y, r;
      if (p.a_inner) {
        x = *reinterpret_cast<const V *>(a + ia + piece * VEC);
      } else {
        const T v = a[ia];
#pragma unroll
        for (int k = 0; k < VEC; ++k) x[k] = v;
      }
      if (p.b_inner) {
        y = *reinterpret_cast<const V *>(b + ib + piece * VEC);
      } else {
        const T v = b[ib];
#pragma unroll
        for (int k = 0; k < VEC; ++k) y[k] = v;
      }
#pragma unroll
      for (int k = 0; k < VEC; ++k) r[k] = x[k] * y[k];
      *reinterpret_cast<V *>(out + at) = r;
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const unsigned col = piece * VEC + k;
        if (col < p.inner) out[at + k] = a[ia + col * p.a_inner] * b[ib + col * p.b_inner];
      }
    }
  }
}

// Block b adds the elements of chunk b: thread t takes the 16-byte pieces t, t + 256,
// ... of the chunk in that order (in double), then the 256 thread sums are added in a
// fixed binary tree.  The chunking depends only on n, so the result repeats exactly.
template <typename T>
__global__ void __launch_bounds__(256) sum_chunks_kernel(const T *__restrict__ x, long long n, long long chunk,
                                                         double *__restrict__ partial) {
  typedef typename Vec16<T>::type V;
  constexpr int VEC = Vec16<T>::N;
  __shared__ double tree[256];
  const long long begin = (long long)blockIdx.x * chunk;  // chunk is a multiple of VEC
  const long long end = min(begin + chunk, n);
  const long long nvec = (end - begin) / VEC;
  const V *vx = reinterpret_cast<const V *>(x + begin);
  // four running sums per thread (pieces t, t + 256, t + 512, t + 768 of each round of
  // 1024), added as (s0 + s1) + (s2 + s3): four loads in flight, still one fixed order
  double s4[4] = {0.0, 0.0, 0.0, 0.0};
  long long i = threadIdx.x;
  for (; i + 768 < nvec; i += 1024) {
    V v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = vx[i + u * 256];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int k = 0; k < VEC; ++k) s4[u] += (double)v[u][k];
  }
  for (int u = 0; i < nvec; i += 256, ++u) {
    const V v = vx[i];
#pragma unroll
    for (int k = 0; k < VEC; ++k) s4[u] += (double)v[k];
  }
  double s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
  {
    const long long i = begin + nvec * VEC + threadIdx.x;  // the array's last n % VEC elements
    if (i < end) s += (double)x[i];
  }
  tree[threadIdx.x] = s;
  __syncthreads();
  for (int half = 128; half > 0; half >>= 1) {
    if ((int)threadIdx.x < half) tree[threadIdx.x] += tree[threadIdx.x + half];
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = tree[0];
}

// One block adds the chunk sums (thread t takes t, t + 256, ... in order, then the same
// tree) and rounds once to T.
template <typename T>
__global__ void __launch_bounds__(256) sum_final_kernel(const double *__restrict__ partial, int count, T *__restrict__ out) {
  __shared__ double tree[256];
  double s = 0.0;
  for (int i = threadIdx.x; i < count; i += 256) s += partial[i];
  tree[threadIdx.x] = s;
  __syncthreads();
  for (int half = 128; half > 0; half >>= 1) {
    if ((int)threadIdx.x < half) tree[threadIdx.x] += tree[threadIdx.x + half];
    __syncthreads();
  }
  if (threadIdx.x == 0) *out = (T)tree[0];
}

template <typename T>
__global__ void __launch_bounds__(256) fill_from_kernel(const T *__restrict__ value, T *__restrict__ out, long long n) {
  typedef typename Vec16<T>::type V;
  constexpr int VEC = Vec16<T>::N;
  const T v = *value;
  V vv;
#pragma unroll
  for (int k = 0; k < VEC; ++k) vv[k] = v;
  const long long nvec = n / VEC;
  V *vo = reinterpret_cast<V *>(out);
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (long long)gridDim.x * 256) vo[i] = vv;
  if (blockIdx.x == 0) {
    const long long i = nvec * VEC + threadIdx.x;
    if (i < n) out[i] = v;
  }
}

unsigned streaming_grid(long long n, size_t elem) {
  const long long pieces = std::max<long long>(1, n / (long long)(16 / elem));
  const long long cap = (long long)runtime().props.multiProcessorCount * 16;  // 16 blocks of 256 threads per unit
  return (unsigned)std::min<long long>(ceil_div(pieces, 256), cap);
}

int check_elementwise(int dtype, int64_t n, const char *who) {
  if (dtype != MG_F32 && dtype != MG_F64) return fail(MG_ERR_UNSUPPORTED, "%s: dtype %d (only float32=0 / float64=1)", who, dtype);
  if (n < 0) return fail(MG_ERR_BAD_ARG, "%s: n = %lld", who, (long long)n);
  return MG_OK;
}

template <int OP>
int launch_elementwise(int dtype, int64_t n, const void *a, const void *b, void *out, int tag) {
  if (n == 0) return MG_OK;
  hipStream_t s = runtime().stream;
  ScopedTiming timed(tag);
  if (dtype == MG_F32)
    hipLaunchKernelGGL((elementwise_kernel<float, OP>), dim3(streaming_grid(n, 4)), dim3(256), 0, s, (const float *)a,
                       (const float *)b, (float *)out, (long long)n);
  else
    hipLaunchKernelGGL((elementwise_kernel<double, OP>), dim3(streaming_grid(n, 8)), dim3(256), 0, s, (const double *)a,
                       (const double *)b, (double *)out, (long long)n);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

bool misaligned(const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 != 0; }

// relu with its mask kept as one bit per element: bit i % 8 of mask[i / 8] is x[i] > 0.  A
// thread takes eight consecutive elements (two or four 16-byte pieces) and one byte of the mask.
//   forward:  out[i] = x[i] * (x[i] > 0), and the mask
//   backward: dx[i]  = grad[i] * (bit i)          -- x is not read
template <typename T, bool BACKWARD>
__global__ void __launch_bounds__(256) relu_mask_kernel(const T *__restrict__ in, T *__restrict__ out, unsigned char *__restrict__ mask,
                                                        long long n) {
  typedef typename Vec16<T>::type V;
  constexpr int VEC = Vec16<T>::N, PIECES = 8 / VEC;
  const long long groups = (n + 7) / 8;
  for (long long grp = (long long)blockIdx.x * 256 + threadIdx.x; grp < groups; grp += (long long)gridDim.x * 256) {
    const long long first = grp * 8;
    unsigned bits = BACKWARD ? (unsigned)mask[grp] : 0u;
    if (first + 8 <= n) {
      const V *vi = reinterpret_cast<const V *>(in + first);
      V *vo = reinterpret_cast<V *>(out + first);
      V v[PIECES];
#pragma unroll
      for (int q = 0; q < PIECES; ++q) v[q] = vi[q];
#pragma unroll
      for (int q = 0; q < PIECES; ++q) {
        V r;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          const int bit = q * VEC + k;
          if constexpr (BACKWARD) {
            r[k] = v[q][k] * (((bits >> bit) & 1u) ? T(1) : T(0));
          } else {
            const bool positive = v[q][k] > T(0);
            bits |= (positive ? 1u : 0u) << bit;
            r[k] = v[q][k] * (positive ? T(1) : T(0));
          }
        }
        vo[q] = r;
      }
    } else {  // the array's last, partial group
      for (int bit = 0; first + bit < n; ++bit) {
        const T value = in[first + bit];
        if constexpr (BACKWARD) {
          out[first + bit] = value * (((bits >> bit) & 1u) ? T(1) : T(0));
        } else {
          const bool positive = value > T(0);
          bits |= (positive ? 1u : 0u) << bit;
          out[first + bit] = value * (positive ? T(1) : T(0));
        }
      }
    }
    if constexpr (!BACKWARD) mask[grp] = (unsigned char)bits;
  }
}

template <bool BACKWARD>
int launch_relu_mask(int dtype, int64_t n, const void *in, void *out, void *mask) {
  if (n == 0) return MG_OK;
  hipStream_t s = runtime().stream;
  const long long groups = ((long long)n + 7) / 8;
  const unsigned grid = (unsigned)std::min<long long>(ceil_div(groups, 256), (long long)runtime().props.multiProcessorCount * 16);
  ScopedTiming timed(TAG_ELEMENTWISE);
  if (dtype == MG_F32)
    hipLaunchKernelGGL((relu_mask_kernel<float, BACKWARD>), dim3(grid), dim3(256), 0, s, (const float *)in, (float *)out,
                       (unsigned char *)mask, (long long)n);
  else
    hipLaunchKernelGGL((relu_mask_kernel<double, BACKWARD>), dim3(grid), dim3(256), 0, s, (const double *)in, (double *)out,
                       (unsigned char *)mask, (long long)n);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// Kernels of the gradient bookkeeping between operations: out = (B) x, acc = (A)(acc + inc)
// in the wider of the two types (what NumPy's `acc += inc` computes), out = value.  A thread
// takes four consecutive elements of each array (16 or 32 bytes).
template <typename A, typename B, bool ADD>
__global__ void __launch_bounds__(256) convert_kernel(A *__restrict__ acc, const B *__restrict__ inc, long long n) {
  typedef A VA __attribute__((ext_vector_type(4)));
  typedef B VB __attribute__((ext_vector_type(4)));
  typedef typename std::conditional<(sizeof(A) > sizeof(B)), A, B>::type P;
  const long long nvec = n / 4;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (long long)gridDim.x * 256) {
    const VB b = reinterpret_cast<const VB *>(inc)[i];
    VA r;
    if constexpr (ADD) {
      const VA a = reinterpret_cast<const VA *>(acc)[i];
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = (A)((P)a[k] + (P)b[k]);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = (A)b[k];
    }
    reinterpret_cast<VA *>(acc)[i] = r;
  }
  if (blockIdx.x == 0) {
    const long long i = nvec * 4 + threadIdx.x;
    if (i < n) acc[i] = ADD ? (A)((P)acc[i] + (P)inc[i]) : (A)inc[i];
  }
}

template <typename T>
__global__ void __launch_bounds__(256) fill_value_kernel(T *__restrict__ out, T value, long long n) {
  typedef typename Vec16<T>::type V;
  constexpr int VEC = Vec16<T>::N;
  V vv;
#pragma unroll
  for (int k = 0; k < VEC; ++k) vv[k] = value;
  const long long nvec = n / VEC;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (long long)gridDim.x * 256) reinterpret_cast<V *>(out)[i] = vv;
  if (blockIdx.x == 0) {
    const long long i = nvec * VEC + threadIdx.x;
    if (i < n) out[i] = value;
  }
}

template <bool ADD>
int launch_convert(int a_dtype, int b_dtype, int64_t n, void *acc, const void *inc) {
  if (n == 0) return MG_OK;
  hipStream_t s = runtime().stream;
  const unsigned grid = (unsigned)std::min<long long>(ceil_div(ceil_div(n, 4), 256), (long long)runtime().props.multiProcessorCount * 16);
  ScopedTiming timed(TAG_ELEMENTWISE);
#define MG_CONVERT(A, B) hipLaunchKernelGGL((convert_kernel<A, B, ADD>), dim3(grid), dim3(256), 0, s, (A *)acc, (const B *)inc, (long long)n)
#define MG_CONVERT_FROM(A)                               \
  do {                                                   \
    if (b_dtype == MG_F32) MG_CONVERT(A, float);         \
    else if (b_dtype == MG_F64) MG_CONVERT(A, double);   \
    else MG_CONVERT(A, _Float16);                        \
  } while (0)
  if (a_dtype == MG_F32) MG_CONVERT_FROM(float);
  else if (a_dtype == MG_F64) MG_CONVERT_FROM(double);
  else MG_CONVERT_FROM(_Float16);
#undef MG_CONVERT_FROM
#undef MG_CONVERT
  MG_HIP(hipGetLastError());
  return MG_OK;
}

// How mg_sum_all cuts x: chunks of 128 KiB, at most 4096 of them (then the chunks grow); a
// function of n and the element size only, so that the order of the additions is too.
struct SumChunking {
  long long chunk, chunks;
};
SumChunking sum_chunking(int dtype, int64_t n) {
  const long long elem = dtype == MG_F32 ? 4 : 8;
  const long long vec = 16 / elem;
  long long chunk = (128 * 1024) / elem;
  long long chunks = std::max<long long>(1, ceil_div(n, chunk));
  if (chunks > 4096) {
    chunk = ceil_div(ceil_div(n, 4096), vec) * vec;
    chunks = ceil_div(n, chunk);
  }
  return {chunk, chunks};
}

int check_sum_all(int dtype, int64_t n, const void *x, const void *out, const char *who) {
  if (int rc = check_elementwise(dtype, n, who)) return rc;
  if (!out || (n > 0 && !x)) return fail(MG_ERR_BAD_ARG, "null pointer in %s", who);
  if (misaligned(x)) return fail(MG_ERR_BAD_ARG, "%s: x must be 16-byte aligned", who);
  return MG_OK;
}

// The two kernels of the whole-array sum; `partial` holds one double per chunk.
int launch_sum_all(int dtype, int64_t n, const void *x, void *out, double *partial) {
  hipStream_t s = runtime().stream;
  const SumChunking c = sum_chunking(dtype, n);
  if (dtype == MG_F32) {
    hipLaunchKernelGGL(sum_chunks_kernel<float>, dim3((unsigned)c.chunks), dim3(256), 0, s, (const float *)x, (long long)n, c.chunk,
                       partial);
    hipLaunchKernelGGL(sum_final_kernel<float>, dim3(1), dim3(256), 0, s, (const double *)partial, (int)c.chunks, (float *)out);
  } else {
    hipLaunchKernelGGL(sum_chunks_kernel<double>, dim3((unsigned)c.chunks), dim3(256), 0, s, (const double *)x, (long long)n, c.chunk,
                       partial);
    hipLaunchKernelGGL(sum_final_kernel<double>, dim3(1), dim3(256), 0, s, (const double *)partial, (int)c.chunks, (double *)out);
  }
  MG_HIP(hipGetLastError());
  return MG_OK;
}

}  // namespace

// Chunk sums of mg_sum_all_static: device memory that belongs to the code object, so that entry
// point needs no allocation.  Every device the library runs on holds its own copy at its own
// address; the array's name is only a host-side handle for hipGetSymbolAddress, the kernels get
// the resolved pointer.  Every chunk sum a call reads is written by that call first, so nothing
// has to be cleared between calls; two calls that overlap on one device would race on it.
constexpr int kStaticChunks = 4096;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) double scratch[kStaticChunks];
static double *scratch_ptr[kMaxDevices];

// Called by mg_init with `device` current: looks up where this device keeps `scratch`.
int resolve_static_scratch(int device) {
  if (device < 0 || device >= kMaxDevices) return fail(MG_ERR_UNSUPPORTED, "device index %d beyond the %d this library keeps scratch pointers for", device, kMaxDevices);
  if (scratch_ptr[device]) return MG_OK;
  double *ptr = nullptr;
  MG_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) return fail(MG_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch array");
  scratch_ptr[device] = ptr;
  return MG_OK;
}

}  // namespace mg

using namespace mg;

extern "C" {

int mg_multiply(int dtype, int64_t n, const void *a, const void *b, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_elementwise(dtype, n, "mg_multiply")) return rc;
  if (n > 0 && (!a || !b || !out)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_multiply");
  if (misaligned(a) || misaligned(b) || misaligned(out)) return fail(MG_ERR_BAD_ARG, "mg_multiply: pointers must be 16-byte aligned");
  return launch_elementwise<EW_MUL>(dtype, n, a, b, out, TAG_ELEMENTWISE);
}

int mg_relu_fwd(int dtype, int64_t n, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_elementwise(dtype, n, "mg_relu_fwd")) return rc;
  if (n > 0 && (!x || !out)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_relu_fwd");
  if (misaligned(x) || misaligned(out)) return fail(MG_ERR_BAD_ARG, "mg_relu_fwd: pointers must be 16-byte aligned");
  return launch_elementwise<EW_RELU>(dtype, n, x, x, out, TAG_ELEMENTWISE);
}

int mg_relu_bwd(int dtype, int64_t n, const void *x, const void *grad, void *dx) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_elementwise(dtype, n, "mg_relu_bwd")) return rc;
  if (n > 0 && (!x || !grad || !dx)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_relu_bwd");
  if (misaligned(x) || misaligned(grad) || misaligned(dx)) return fail(MG_ERR_BAD_ARG, "mg_relu_bwd: pointers must be 16-byte aligned");
  return launch_elementwise<EW_RELU_BWD>(dtype, n, x, grad, dx, TAG_ELEMENTWISE);
}

int mg_relu_fwd_mask(int dtype, int64_t n, const void *x, void *out, void *mask) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_elementwise(dtype, n, "mg_relu_fwd_mask")) return rc;
  if (n > 0 && (!x || !out || !mask)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_relu_fwd_mask");
  if (misaligned(x) || misaligned(out)) return fail(MG_ERR_BAD_ARG, "mg_relu_fwd_mask: x and out must be 16-byte aligned");
  return launch_relu_mask<false>(dtype, n, x, out, mask);
}

int mg_relu_bwd_mask(int dtype, int64_t n, const void *mask, const void *grad, void *dx) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_elementwise(dtype, n, "mg_relu_bwd_mask")) return rc;
  if (n > 0 && (!mask || !grad || !dx)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_relu_bwd_mask");
  if (misaligned(grad) || misaligned(dx)) return fail(MG_ERR_BAD_ARG, "mg_relu_bwd_mask: grad and dx must be 16-byte aligned");
  return launch_relu_mask<true>(dtype, n, grad, dx, const_cast<void *>(mask));
}

int mg_multiply_broadcast(int dtype, int nd, const int64_t *shape, const int64_t *a_strides, const int64_t *b_strides, const void *a,
                          const void *b, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (dtype != MG_F32 && dtype != MG_F64) return fail(MG_ERR_UNSUPPORTED, "mg_multiply_broadcast: dtype %d (only float32=0 / float64=1)", dtype);
  if (nd < 1 || nd > 6) return fail(MG_ERR_UNSUPPORTED, "mg_multiply_broadcast: %d axes (1 to 6 after merging)", nd);
  if (!shape || !a_strides || !b_strides) return fail(MG_ERR_BAD_ARG, "null pointer in mg_multiply_broadcast");
  const int vec = dtype == MG_F32 ? 4 : 2;  // elements in 16 bytes
  long long n = 1, a_span = 1, b_span = 1;  // elements of out; one past the farthest element read of a and b
  for (int d = 0; d < nd; ++d) {
    if (shape[d] < 0 || a_strides[d] < 0 || b_strides[d] < 0) return fail(MG_ERR_BAD_ARG, "mg_multiply_broadcast: negative extent or stride");
    if (shape[d] == 0) return MG_OK;
    n *= shape[d];
    if (n >= (1ll << 31)) return fail(MG_ERR_UNSUPPORTED, "mg_multiply_broadcast: 2^31 elements or more");
    a_span += (shape[d] - 1) * a_strides[d];
    b_span += (shape[d] - 1) * b_strides[d];
  }
  if (a_span > n || b_span > n) return fail(MG_ERR_BAD_ARG, "mg_multiply_broadcast: an operand reaches beyond the extent of the result");
  if (a_strides[nd - 1] > 1 || b_strides[nd - 1] > 1)
    return fail(MG_ERR_BAD_ARG, "mg_multiply_broadcast: the stride along the last axis must be 1 or 0");
  if (!a || !b || !out) return fail(MG_ERR_BAD_ARG, "null pointer in mg_multiply_broadcast");
  if (misaligned(a) || misaligned(b) || misaligned(out)) return fail(MG_ERR_BAD_ARG, "mg_multiply_broadcast: buffers must be 16-byte aligned");
  BroadcastParams p{};
  p.outer_dims = nd - 1;
  bool aligned = shape[nd - 1] % vec == 0;
  for (int d = 0; d < nd - 1; ++d) {
    p.extent[d] = (unsigned)shape[d];
    p.a_step[d] = (unsigned)a_strides[d];
    p.b_step[d] = (unsigned)b_strides[d];
    // 16-byte pieces of an operand must start on 16 bytes: every stride a multiple of the piece
    aligned = aligned && (a_strides[nd - 1] == 0 || a_strides[d] % vec == 0) && (b_strides[nd - 1] == 0 || b_strides[d] % vec == 0);
  }
  p.a_inner = (unsigned)a_strides[nd - 1];
  p.b_inner = (unsigned)b_strides[nd - 1];
  p.inner = (unsigned)shape[nd - 1];
  p.pieces = (unsigned)ceil_div(shape[nd - 1], (long long)vec);
  const long long threads = (n / shape[nd - 1]) * p.pieces;
  if (threads >= (1ll << 32) - 256 * 4096) return fail(MG_ERR_UNSUPPORTED, "mg_multiply_broadcast: too many rows of a short last axis");
  p.threads = (unsigned)threads;
  const unsigned grid = (unsigned)std::min<long long>(ceil_div(threads, 256), (long long)runtime().props.multiProcessorCount * 16);
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_ELEMENTWISE);
#define MG_LAUNCH(T, ALIGNED) \
  hipLaunchKernelGGL((multiply_broadcast_kernel<T, ALIGNED>), dim3(grid), dim3(256), 0, s, (const T *)a, (const T *)b, (T *)out, p)
  if (dtype == MG_F32) {
    if (aligned) MG_LAUNCH(float, true); else MG_LAUNCH(float, false);
  } else {
    if (aligned) MG_LAUNCH(double, true); else MG_LAUNCH(double, false);
  }
#undef MG_LAUNCH
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_sum_all(int dtype, int64_t n, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_sum_all(dtype, n, x, out, "mg_sum_all")) return rc;
  void *partial = nullptr;
  if (int rc = workspace((size_t)sum_chunking(dtype, n).chunks * sizeof(double), &partial)) return rc;
  ScopedTiming timed(TAG_REDUCE_ALL);
  return launch_sum_all(dtype, n, x, out, (double *)partial);
}

int mg_sum_all_static(int dtype, int64_t n, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_sum_all(dtype, n, x, out, "mg_sum_all_static")) return rc;
  if (n > MG_SUM_STATIC_MAX_N)
    return fail(MG_ERR_UNSUPPORTED, "mg_sum_all_static: n = %lld exceeds the %lld elements its fixed scratch array is sized for",
                (long long)n, (long long)MG_SUM_STATIC_MAX_N);
  const int device = runtime().device;
  double *partial = device >= 0 && device < kMaxDevices ? scratch_ptr[device] : nullptr;
  if (!partial) return fail(MG_ERR_NOT_INIT, "mg_sum_all_static: the scratch array was not resolved on device %d", device);
  if (sum_chunking(dtype, n).chunks > kStaticChunks) return fail(MG_ERR_UNSUPPORTED, "mg_sum_all_static: more chunks than the scratch array holds");
  // no timing events here: creating them allocates
  return launch_sum_all(dtype, n, x, out, partial);
}

// float16 is a storage type: the two conversions take it, nothing else does
static int check_storage(int dtype, int64_t n, const char *who) {
  if (dtype != MG_F32 && dtype != MG_F64 && dtype != MG_F16)
    return fail(MG_ERR_UNSUPPORTED, "%s: dtype %d (float32=0 / float64=1 / float16=2)", who, dtype);
  if (n < 0) return fail(MG_ERR_BAD_ARG, "%s: n = %lld", who, (long long)n);
  return MG_OK;
}

int mg_cast(int from_dtype, int to_dtype, int64_t n, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_storage(from_dtype, n, "mg_cast")) return rc;
  if (int rc = check_storage(to_dtype, n, "mg_cast")) return rc;
  if (n > 0 && (!x || !out)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_cast");
  if (reinterpret_cast<uintptr_t>(x) % 32 != 0 || reinterpret_cast<uintptr_t>(out) % 32 != 0)
    return fail(MG_ERR_BAD_ARG, "mg_cast: buffers must be 32-byte aligned");
  return launch_convert<false>(to_dtype, from_dtype, n, out, x);
}

int mg_accumulate(int acc_dtype, int inc_dtype, int64_t n, void *acc, const void *inc) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_storage(acc_dtype, n, "mg_accumulate")) return rc;
  if (int rc = check_storage(inc_dtype, n, "mg_accumulate")) return rc;
  if (n > 0 && (!acc || !inc)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_accumulate");
  if (reinterpret_cast<uintptr_t>(acc) % 32 != 0 || reinterpret_cast<uintptr_t>(inc) % 32 != 0)
    return fail(MG_ERR_BAD_ARG, "mg_accumulate: buffers must be 32-byte aligned");
  return launch_convert<true>(acc_dtype, inc_dtype, n, acc, inc);
}

int mg_fill_value(int dtype, int64_t n, double value, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_elementwise(dtype, n, "mg_fill_value")) return rc;
  if (n > 0 && !out) return fail(MG_ERR_BAD_ARG, "null pointer in mg_fill_value");
  if (misaligned(out)) return fail(MG_ERR_BAD_ARG, "mg_fill_value: out must be 16-byte aligned");
  if (n == 0) return MG_OK;
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_ELEMENTWISE);
  if (dtype == MG_F32)
    hipLaunchKernelGGL(fill_value_kernel<float>, dim3(streaming_grid(n, 4)), dim3(256), 0, s, (float *)out, (float)value, (long long)n);
  else
    hipLaunchKernelGGL(fill_value_kernel<double>, dim3(streaming_grid(n, 8)), dim3(256), 0, s, (double *)out, value, (long long)n);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_fill_from(int dtype, int64_t n, const void *value, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (int rc = check_elementwise(dtype, n, "mg_fill_from")) return rc;
  if (!value || (n > 0 && !out)) return fail(MG_ERR_BAD_ARG, "null pointer in mg_fill_from");
  if (misaligned(out)) return fail(MG_ERR_BAD_ARG, "mg_fill_from: out must be 16-byte aligned");
  if (n == 0) return MG_OK;
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_ELEMENTWISE);
  if (dtype == MG_F32)
    hipLaunchKernelGGL(fill_from_kernel<float>, dim3(streaming_grid(n, 4)), dim3(256), 0, s, (const float *)value, (float *)out,
                       (long long)n);
  else
    hipLaunchKernelGGL(fill_from_kernel<double>, dim3(streaming_grid(n, 8)), dim3(256), 0, s, (const double *)value, (double *)out,
                       (long long)n);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

}  // extern "C"
