// Products of many small matrix pairs in one launch: out[p] = op(a[p]) @ op(b[p]), p < batch,
// where op transposes or not.  A pair of stacks whose matrices are too small to fill the device
// one pair at a time (np.matmul on two stacks, an einsum with a label that both operands and
// the result carry) is bound by launches, not arithmetic, when each pair gets a launch of the
// convolution kernels; here a wavefront makes one 16x16 tile of one product on the matrix cores,
// reading its operands where they lie (a transposed operand is a pair of swapped strides), so the
// whole stack is one grid.  Pairs of 32 x 32 results or more go through a second kernel, where a
// block of four wavefronts makes a 64 x 64 tile of one product from operands it has copied to
// LDS once (16 bytes per lane, coalesced) instead of every wavefront fetching its own rows and
// columns through L1.  Large pairs stay with the tiled convolution kernels.
#include "internal.h"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace mg {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

// D(16x16) += A(16x4) * B(4x16) on one wavefront: lane l supplies A[l%16][l/16] and
// B[l/16][l%16] and receives four elements of column l%16 of D, in rows row_of(l, r).
template <typename T>
struct Tile;

template <>
struct Tile<float> {
  using Acc = f32x4;
  static __device__ __forceinline__ Acc run(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row_of(int lane, int r) { return 4 * (lane >> 4) + r; }
};

template <>
struct Tile<double> {
  using Acc = f64x4;
  static __device__ __forceinline__ Acc run(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row_of(int lane, int r) { return 4 * r + (lane >> 4); }
};

struct BatchedParams {
  int M, K, N;
  int row_tiles, col_tiles;
  long long tiles;                   // batch * row_tiles * col_tiles
  long long a_pair, a_row, a_col;    // element strides of op(a): between pairs, along M, along K
  long long b_pair, b_row, b_col;    // of op(b): between pairs, along K, along N
};

// AV / BV: op(a) / op(b) is contiguous along K and K is a multiple of the 16-byte piece, so a
// lane reads a piece of VEC consecutive k at once.  The sum over k may run in any order as long
// as both operands use the same one: in a block of 4 * VEC values of k, the four lane groups
// (lane / 16 = q) take k = k0 + VEC * q + s at step s, which makes a lane's VEC steps one piece.
template <typename T, bool AV, bool BV>
__global__ void __launch_bounds__(256) batched_product_kernel(BatchedParams p, const T *__restrict__ a, const T *__restrict__ b,
                                                              T *__restrict__ out) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T V __attribute__((ext_vector_type(VEC)));
  const int lane = threadIdx.x & 63;
  const long long tile = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);  // the same for a whole wavefront
  if (tile >= p.tiles) return;
  const int per_pair = p.row_tiles * p.col_tiles;
  const long long pair = tile / per_pair;
  const int within = (int)(tile - pair * per_pair);
  const int row0 = (within / p.col_tiles) * 16, col0 = (within % p.col_tiles) * 16;
  const int i = row0 + (lane & 15), j = col0 + (lane & 15), kk = lane >> 4;
  // rows and columns beyond the matrix supply zeros and are not stored
  const bool row_in = i < p.M, col_in = j < p.N;
  const T *pa = a + pair * p.a_pair + (row_in ? (long long)i * p.a_row : 0);
  const T *pb = b + pair * p.b_pair + (col_in ? (long long)j * p.b_col : 0);
  typename Tile<T>::Acc acc = {0, 0, 0, 0};
  const int whole = p.K & ~3;
  int done = 0;
  if constexpr (AV || BV) {
    const int blocked = p.K - p.K % (4 * VEC);
    for (; done < blocked; done += 4 * VEC) {
      const int k = done + VEC * kk;
      T av[VEC], bv[VEC];
      if constexpr (AV) {
        V v = {};
        if (row_in) v = *reinterpret_cast<const V *>(pa + k);
#pragma unroll
        for (int s = 0; s < VEC; ++s) av[s] = v[s];
      } else {
#pragma unroll
        for (int s = 0; s < VEC; ++s) av[s] = row_in ? pa[(long long)(k + s) * p.a_col] : T(0);
      }
      if constexpr (BV) {
        V v = {};
        if (col_in) v = *reinterpret_cast<const V *>(pb + k);
#pragma unroll
        for (int s = 0; s < VEC; ++s) bv[s] = v[s];
      } else {
#pragma unroll
        for (int s = 0; s < VEC; ++s) bv[s] = col_in ? pb[(long long)(k + s) * p.b_row] : T(0);
      }
#pragma unroll
      for (int s = 0; s < VEC; ++s) acc = Tile<T>::run(av[s], bv[s], acc);
    }
  }
  auto step = [&](int k0) {
    const int k = k0 + kk;
    const T av = row_in ? pa[(long long)k * p.a_col] : T(0);
    const T bv = col_in ? pb[(long long)k * p.b_row] : T(0);
    acc = Tile<T>::run(av, bv, acc);
  };
  if constexpr (AV || BV) {
    for (int k0 = done; k0 < whole; k0 += 4) step(k0);  // at most 4 * VEC - 1 values of k are left
  } else {
#pragma unroll 4
    for (int k0 = 0; k0 < whole; k0 += 4) step(k0);
  }
  if (whole < p.K) {  // the last one to three columns of op(a) / rows of op(b)
    const int k = whole + kk;
    const bool k_in = k < p.K;
    const T av = row_in && k_in ? pa[(long long)k * p.a_col] : T(0);
    const T bv = col_in && k_in ? pb[(long long)k * p.b_row] : T(0);
    acc = Tile<T>::run(av, bv, acc);
  }
  if (!col_in) return;
  T *po = out + pair * ((long long)p.M * p.N) + j;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = row0 + Tile<T>::row_of(lane, r);
    if (row < p.M) po[(long long)row * p.N] = acc[r];
  }
}


// ---- 64 x 64 tiles of one product per block, operands staged in LDS ---------------------------
// A block copies the 64 x 64 pieces of op(a) and op(b) that its tile needs, K chunk by K chunk,
// into LDS in the orientation they have in memory (a transposed operand is read differently, not
// stored differently), zeros beyond the matrices' edges.  Wavefront w makes the 32 x 32 quarter
// (w / 2, w % 2) of the tile: per step of four k, two fragments of each operand and four MFMAs.
// Row lengths in LDS: an operand whose MFMA lanes (lane % 16) run down its memory rows gets
// 64 + 4 floats per row (sixteen rows start in sixteen different groups of four banks), one
// whose lanes run along a row gets 64 + 16 (the four k of a step start sixteen banks apart).
template <typename T, bool ROWS_ARE_LANES>
struct StagedLd {
  static constexpr int value = sizeof(T) == 4 ? (ROWS_ARE_LANES ? 68 : 80) : (ROWS_ARE_LANES ? 66 : 72);
};

template <typename T, bool TA, bool TB, bool VA, bool VB>
__global__ void __launch_bounds__(256) batched_staged_kernel(BatchedParams p, const T *__restrict__ a, const T *__restrict__ b,
                                                             T *__restrict__ out) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T V __attribute__((ext_vector_type(VEC)));
  constexpr int LDA = StagedLd<T, !TA>::value;  // not transposed: memory rows are m, the lanes' index
  constexpr int LDB = StagedLd<T, TB>::value;   // transposed: memory rows are n, the lanes' index
  __shared__ __attribute__((aligned(16))) T As[64 * LDA];
  __shared__ __attribute__((aligned(16))) T Bs[64 * LDB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lk = lane >> 4;
  const int per_pair = p.row_tiles * p.col_tiles;
  const long long pair = (long long)blockIdx.x / per_pair;
  const int within = (int)((long long)blockIdx.x - pair * per_pair);
  const int row0 = (within / p.col_tiles) * 64, col0 = (within % p.col_tiles) * 64;
  const T *pa = a + pair * p.a_pair;
  const T *pb = b + pair * p.b_pair;

  // The 64 x 64 piece of a stored matrix (`rows` x `cols`, row-major) that starts at (r0, c0)
  // travels through registers (`fetch`, zeros outside the matrix) into LDS (`park`, row length
  // `ld`); the loads of both operands are issued before either is parked, so that a chunk
  // costs one trip to memory, not two.
  constexpr int PIECES = 64 / VEC, PASS = 256 / PIECES, NV = 64 / PASS;
  struct Regs {
    V v[NV];   // 16-byte pieces: rows tid / PIECES + i * PASS, piece tid % PIECES
    T e[16];   // single elements: rows tid / 64 + 4 * i, column tid % 64
  };
  auto fetch = [&](const T *src, int rows, int cols, int r0, int c0, Regs &reg, auto vec) {
    if constexpr (decltype(vec)::value) {
      const int piece = tid % PIECES, r = tid / PIECES;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int rr = r0 + r + i * PASS, cc = c0 + piece * VEC;
        reg.v[i] = V{};
        if (rr < rows && cc < cols) reg.v[i] = *reinterpret_cast<const V *>(src + (long long)rr * cols + cc);  // cols % VEC == 0
      }
    } else {
      const int c = tid % 64, r = tid / 64;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int rr = r0 + r + i * 4, cc = c0 + c;
        reg.e[i] = (rr < rows && cc < cols) ? src[(long long)rr * cols + cc] : T(0);
      }
    }
  };
  auto park = [&](const Regs &reg, T *dst, int ld, auto vec) {
    if constexpr (decltype(vec)::value) {
      const int piece = tid % PIECES, r = tid / PIECES;
#pragma unroll
      for (int i = 0; i < NV; ++i) *reinterpret_cast<V *>(dst + (r + i * PASS) * ld + piece * VEC) = reg.v[i];
    } else {
      const int c = tid % 64, r = tid / 64;
#pragma unroll
      for (int i = 0; i < 16; ++i) dst[(r + i * 4) * ld + c] = reg.e[i];
    }
  };
  const std::integral_constant<bool, VA> vec_a{};
  const std::integral_constant<bool, VB> vec_b{};
  auto fetch_chunk = [&](int k0, Regs &ra, Regs &rb) {
    if constexpr (TA)
      fetch(pa, p.K, p.M, k0, row0, ra, vec_a);  // stored (K, M)
    else
      fetch(pa, p.M, p.K, row0, k0, ra, vec_a);  // stored (M, K)
    if constexpr (TB)
      fetch(pb, p.N, p.K, col0, k0, rb, vec_b);  // stored (N, K)
    else
      fetch(pb, p.K, p.N, k0, col0, rb, vec_b);  // stored (K, N)
  };

  const int wr = (wave >> 1) * 32, wc = (wave & 1) * 32;
  typename Tile<T>::Acc acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = typename Tile<T>::Acc{0, 0, 0, 0};

  Regs ra, rb;
  fetch_chunk(0, ra, rb);
  for (int k0 = 0; k0 < p.K; k0 += 64) {
    if (k0 > 0) __syncthreads();  // everyone has finished with the previous chunk
    park(ra, As, LDA, vec_a);
    park(rb, Bs, LDB, vec_b);
    __syncthreads();
    if (k0 + 64 < p.K) fetch_chunk(k0 + 64, ra, rb);  // on its way while this chunk is multiplied
    const int steps = (min(64, p.K - k0) + 3) / 4;
    for (int ks = 0; ks < steps; ++ks) {
      const int k = ks * 4 + lk;
      T av[2], bv[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int m = wr + i * 16 + l16;
        av[i] = TA ? As[k * LDA + m] : As[m * LDA + k];
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = wc + j * 16 + l16;
        bv[j] = TB ? Bs[n * LDB + k] : Bs[k * LDB + n];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Tile<T>::run(av[i], bv[j], acc[i][j]);
    }
  }

  T *po = out + pair * ((long long)p.M * p.N);
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = col0 + wc + j * 16 + l16;
    if (col >= p.N) continue;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = row0 + wr + i * 16 + Tile<T>::row_of(lane, r);
        if (row < p.M) po[(long long)row * p.N + col] = acc[i][j][r];
      }
  }
}

template <typename T>
void launch_staged(const BatchedParams &p, long long batch, bool ta, bool tb, bool va, bool vb, const void *a, const void *b,
                   void *out, hipStream_t s) {
  const dim3 grid((unsigned)(batch * p.row_tiles * p.col_tiles)), block(256);
#define MG_STAGED(TA, TB, VA, VB)                                                                                      \
  if (ta == TA && tb == TB && va == VA && vb == VB)                                                                    \
    hipLaunchKernelGGL((batched_staged_kernel<T, TA, TB, VA, VB>), grid, block, 0, s, p, (const T *)a, (const T *)b, (T *)out);
#define MG_STAGED_V(TA, TB) MG_STAGED(TA, TB, false, false) MG_STAGED(TA, TB, false, true) MG_STAGED(TA, TB, true, false) MG_STAGED(TA, TB, true, true)
  MG_STAGED_V(false, false)
  MG_STAGED_V(false, true)
  MG_STAGED_V(true, false)
  MG_STAGED_V(true, true)
#undef MG_STAGED_V
#undef MG_STAGED
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_matmul_batched(int dtype, int64_t batch, int64_t M, int64_t K, int64_t N, int trans_a, int trans_b, const void *a, const void *b,
                      void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  if (dtype != MG_F32 && dtype != MG_F64) return fail(MG_ERR_UNSUPPORTED, "mg_matmul_batched: dtype %d (only float32=0 / float64=1)", dtype);
  if (batch < 0 || M < 0 || K < 0 || N < 0)
    return fail(MG_ERR_BAD_ARG, "mg_matmul_batched: batch=%lld M=%lld K=%lld N=%lld", (long long)batch, (long long)M, (long long)K, (long long)N);
  if (batch == 0 || M == 0 || N == 0) return MG_OK;
  if (M >= (1 << 24) || K >= (1 << 24) || N >= (1 << 24) || batch >= (1ll << 31))
    return fail(MG_ERR_UNSUPPORTED, "mg_matmul_batched: an extent of 2^24 or more, or 2^31 pairs or more");
  if (!out || (K > 0 && (!a || !b))) return fail(MG_ERR_BAD_ARG, "null pointer in mg_matmul_batched");
  BatchedParams p{};
  p.M = (int)M, p.K = (int)K, p.N = (int)N;
  p.row_tiles = (int)ceil_div(M, 16);
  p.col_tiles = (int)ceil_div(N, 16);
  p.tiles = batch * p.row_tiles * p.col_tiles;
  if (ceil_div(p.tiles, 4) >= (1ll << 31)) return fail(MG_ERR_UNSUPPORTED, "mg_matmul_batched: 2^33 tiles of 16 x 16 results or more");
  p.a_pair = M * K, p.b_pair = K * N;
  p.a_row = trans_a ? 1 : K, p.a_col = trans_a ? M : 1;  // a[p] is stored (K, M) when transposed
  p.b_row = trans_b ? 1 : N, p.b_col = trans_b ? K : 1;  // b[p] is stored (N, K) when transposed
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_BATCHED_PRODUCT);
  // Pairs of 32 x 32 results or more whose 64 x 64 tiles are at least half full: staged in LDS.
  // MYGRAD_HIP_BMM_STAGED=0 keeps every pair on the kernel that reads its operands in place.
  static const bool staged_on = [] {
    const char *flag = getenv("MYGRAD_HIP_BMM_STAGED");
    return !(flag && flag[0] == '0');
  }();
  const long long t64 = ceil_div(M, 64) * ceil_div(N, 64);
  if (staged_on && K > 0 && M >= 32 && N >= 32 && 2 * M * N >= t64 * 64 * 64 && batch * t64 < (1ll << 31)) {
    const int vec = dtype == MG_F32 ? 4 : 2;
    // 16-byte pieces along a stored matrix's rows: the row length is a whole number of pieces
    // (so is the distance between pairs, then) and the stack itself is aligned
    const bool va = (trans_a ? M : K) % vec == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0;
    const bool vb = (trans_b ? K : N) % vec == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0;
    p.row_tiles = (int)ceil_div(M, 64);
    p.col_tiles = (int)ceil_div(N, 64);
    if (dtype == MG_F32)
      launch_staged<float>(p, batch, trans_a != 0, trans_b != 0, va, vb, a, b, out, s);
    else
      launch_staged<double>(p, batch, trans_a != 0, trans_b != 0, va, vb, a, b, out, s);
    MG_HIP(hipGetLastError());
    return MG_OK;
  }
  const dim3 grid((unsigned)ceil_div(p.tiles, 4)), block(256);
  // 16-byte pieces along K: the operand is contiguous there, K is a whole number of pieces (so
  // every row starts on one) and the stack itself is aligned
  const int vec = dtype == MG_F32 ? 4 : 2;
  const bool av = p.a_col == 1 && K % vec == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0;
  const bool bv = p.b_row == 1 && K % vec == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0;
#define MG_BATCHED(T, AV, BV) \
  hipLaunchKernelGGL((batched_product_kernel<T, AV, BV>), grid, block, 0, s, p, (const T *)a, (const T *)b, (T *)out)
#define MG_BATCHED_T(T)                 \
  do {                                  \
    if (av && bv) MG_BATCHED(T, true, true);        \
    else if (av) MG_BATCHED(T, true, false);        \
    else if (bv) MG_BATCHED(T, false, true);        \
    else MG_BATCHED(T, false, false);               \
  } while (0)
  if (dtype == MG_F32) MG_BATCHED_T(float); else MG_BATCHED_T(double);
#undef MG_BATCHED_T
#undef MG_BATCHED
  MG_HIP(hipGetLastError());
  return MG_OK;
}

}  // extern "C"
