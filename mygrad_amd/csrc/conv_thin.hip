// Gather-GEMM with one position per lane, for convolutions whose rows come in few groups of
// four: the data gradient of a layer with a handful of channels (the first layer of an image
// network), the forward pass of a layer with a handful of filters, and the forward pass of a
// first layer itself (one or three channels; more than 64 filters in passes of 64).  Single
// precision.
//
// A 16-row MFMA tile would carry 3 or 4 live rows of such a data gradient, and K tiles of 16
// suit 3 channels badly.  v_mfma_f32_4x4x1_16b_f32 multiplies
// sixteen independent 4x1 by 1x4 blocks: lane l supplies B[l] and receives D[i][l], i = 0..3,
// in its four accumulator registers; with the A operand broadcast from one block (cbsz = 4,
// abid = the block), D[i][l] += A[4 * abid + i] * B[l].  So a lane IS a position: it gathers its
// own elements of src straight from memory (consecutive lanes, consecutive addresses), no LDS
// and no barrier, and one register of packed filters -- sixteen blocks of four rows -- feeds
// sixteen MFMAs.  With a stride, a lane owns one position of the coarse grid ceil(X / stride)
// and all of its stride phases, one accumulator each: the phases read the same neighbourhood
// of grad, so each gathered element feeds up to nph MFMAs (with weights that are zero where
// the phase has no tap for it).  More than four rows are RG groups of four, one accumulator
// each as well: the sixteen blocks of a register of filters are (entry, phase, row group), and a
// gathered element feeds NPH * RG MFMAs.  With 64 filters a register holds one (channel, tap)
// of all of them, and the forward pass of a first layer does sixteen MFMAs per two loads.
#include "conv_kernels.h"
#include "internal.h"

namespace mg {

namespace {

#define MG_CONSTANT __attribute__((address_space(4)))
typedef int int4v __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr unsigned kOutside = 0x80000000u;  // a byte offset past the end of any tensor (each below 2 GiB): reads as zero

__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const void *base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buffer_load(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_bytes, unsigned uniform_bytes) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_bytes, (int)uniform_bytes, 0));
}

// acc[j] += A[block I * NACC + j] * v for every accumulator; the block index is an immediate of the instruction
template <int NACC, int I, int J = 0>
__device__ __forceinline__ void feed(f32x4 (&acc)[NACC], float a, float v) {
  if constexpr (J < NACC) {
    if constexpr (NACC >= 8) {
      // Many accumulators: written as the instruction itself, accumulating in place.  (Through the
      // builtin the compiler gives the unrolled steps' results new registers and moves all of
      // them back at the end of every round of the loop, 128 moves for 16 MFMAs.)  An accumulator
      // is used again eight or more MFMAs later, long after its result has been written.
      asm volatile("v_mfma_f32_4x4x1_16b_f32 %0, %1, %2, %0 cbsz:4 abid:%3" : "+a"(acc[J]) : "v"(a), "v"(v), "n"(I * NACC + J));
    } else {
      acc[J] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, v, acc[J], 4, I * NACC + J, 0);
    }
    feed<NACC, I, J + 1>(acc, a, v);
  }
}

template <int NACC, int EPV, int I = 0>
__device__ __forceinline__ void feed_all(f32x4 (&acc)[NACC], float a, const float (&v)[EPV]) {
  if constexpr (I < EPV) {
    feed<NACC, I>(acc, a, v[I]);
    feed_all<NACC, EPV, I + 1>(acc, a, v);
  }
}

template <int NPH, int RG>
__global__ void __launch_bounds__(256) thin_gemm_kernel(ThinParams p) {
  constexpr int NACC = NPH * RG;   // accumulators: (stride phase, group of four rows)
  constexpr int EPV = 16 / NACC;   // entries per register of packed filters
  // feed() writes the MFMA as the instruction itself from 8 accumulators on, where the compiler
  // inserts no wait states: the code relies on an accumulator being written again only NACC
  // MFMAs after its last write (feed_all runs through all NACC for every entry) and on the two
  // s_nop 7 before the epilogue.  Fewer than 8 accumulators go through the builtin, which the
  // compiler schedules itself; any other count must revisit both.
  static_assert(NACC == 1 || NACC == 2 || NACC == 4 || NACC == 8 || NACC == 16, "accumulator counts the hazard analysis covers");
  static_assert(NACC * EPV == 16, "a register of packed filters feeds sixteen MFMAs");
  const int lane = threadIdx.x & 63;
  const int pos = blockIdx.x * 256 + threadIdx.x;
  const bool active = pos < p.npos;
  const unsigned upos = active ? (unsigned)pos : 0u;
  const unsigned n = p.by_jvol.div(upos);
  unsigned rest = upos - n * (unsigned)(p.J[0] * p.J[1] * p.J[2]);
  const unsigned j0 = p.by_j12.div(rest);
  rest -= j0 * (unsigned)(p.J[1] * p.J[2]);
  const unsigned j1 = p.by_j2.div(rest);
  const unsigned j2 = rest - j1 * (unsigned)p.J[2];
  const int c0 = (int)j0 * p.sj[0], c1 = (int)j1 * p.sj[1], c2 = (int)j2 * p.sj[2];
  const unsigned src_at =
      (unsigned)(((long long)n * p.src_nstride + (long long)c0 * p.qs[0] + (long long)c1 * p.qs[1] + (long long)c2 * p.qs[2]) * 4);

  // a pass is a block of 4 * RG rows: its own packed filters, its own rows of dst
  const int pass = blockIdx.y;
  const int rows_left = p.M - pass * 4 * RG;
  const __amdgpu_buffer_rsrc_t a_buf = buffer_of(p.A + (long long)pass * p.pass_floats, p.a_bytes);
  const __amdgpu_buffer_rsrc_t src_buf = buffer_of(p.src, p.src_bytes);
  const int4v MG_CONSTANT *tab = (const int4v MG_CONSTANT *)p.tab;

  f32x4 acc[NACC];
#pragma unroll
  for (int j = 0; j < NACC; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // One step = one chunk of entries under one group of channels: a register of filters, EPV
  // gathered elements, 16 MFMAs.  The steps of all chunks form one pipeline: two sets of
  // registers take turns, the loads of one step are in flight while the other feeds the MFMAs,
  // also across the change from one chunk to the next (where the entries' offsets are renewed).
  unsigned a_lane = (unsigned)lane * 4u;  // past the last step: kOutside (the range check is on the per-lane offset)
  unsigned at[EPV];
  // The rows of the table come through the scalar data path; with few entries per chunk the
  // chunks change often, and the rows of the next chunk are asked for a chunk ahead so that
  // nobody waits for them.
  constexpr bool AHEAD = EPV <= 4;
  int4v rows[EPV];
  auto ask_rows = [&](int q) {
#pragma unroll
    for (int i = 0; i < EPV; ++i) rows[i] = tab[q * EPV + i];  // off, d0, d1, d2: the same for every lane
  };
  auto enter_chunk = [&](int q) {
    if constexpr (!AHEAD) ask_rows(q);
#pragma unroll
    for (int i = 0; i < EPV; ++i) {
      const int4v e = rows[i];
      const bool ok = active & ((unsigned)(c0 + e.y) < (unsigned)p.Q[0]) & ((unsigned)(c1 + e.z) < (unsigned)p.Q[1]) &
                      ((unsigned)(c2 + e.w) < (unsigned)p.Q[2]);  // no branches: the rows are the same for every lane
      at[i] = ok ? src_at + (unsigned)(e.x * 4) : kOutside;
    }
    if constexpr (AHEAD) ask_rows(q + 1 < p.chunks ? q + 1 : 0);
  };
  if constexpr (AHEAD) ask_rows(0);
  // The channel groups are taken in blocks of p.kblock: all chunks under one block, then the
  // next block.  The chunks read overlapping neighbourhoods of the same channels (the taps of a
  // window; the rows of grad the stride phases share), and with every channel between two
  // chunks the second one found nothing of the first in the caches: the stem's data gradient
  // read grad 4.7 times from HBM.
  int q = 0, kg = 0, kbegin = 0, kend = min(p.kblock, p.kgroups);
  unsigned a_uni = 0u, s_uni = 0u;
  auto fetch = [&](float &a, float (&v)[EPV]) {
    a = buffer_load(a_buf, a_lane, a_uni);
#pragma unroll
    for (int i = 0; i < EPV; ++i) v[i] = buffer_load(src_buf, at[i], s_uni);
    __builtin_amdgcn_sched_barrier(0);  // all of a step's loads are issued before the MFMAs that follow in the source
  };
  // moves on to the next step; past the last one every load lies outside its buffer and reads as
  // zero: the per-lane offsets of the filters and of the entries are set outside (the hardware
  // checks the per-lane offset against the buffer's size, not the scalar one added to it)
  auto advance = [&]() {
    a_uni += 256u;
    s_uni += p.group_bytes;
    if (++kg == kend) {
      if (++q == p.chunks) {
        q = 0;
        kbegin = kend;
        kend = min(kbegin + p.kblock, p.kgroups);
      }
      kg = kbegin;
      if (kbegin < p.kgroups) {
        a_uni = (unsigned)(q * p.kgroups + kg) * 256u;
        s_uni = (unsigned)kg * p.group_bytes;
        enter_chunk(q);
      } else {
#pragma unroll
        for (int i = 0; i < EPV; ++i) at[i] = kOutside;
        a_lane = kOutside;
        a_uni = 0u;
        s_uni = 0u;
      }
    }
  };
  // DEPTH sets of registers take turns; the loads of DEPTH - 1 steps are in flight while one step
  // feeds the MFMAs.  A step with few entries is short (16 MFMAs whatever their number), and its
  // loads would not be back in time with one step of lead.
  constexpr int DEPTH = EPV <= 2 ? 4 : 2;
  float a[DEPTH], v[DEPTH][EPV];
  enter_chunk(0);
  fetch(a[0], v[0]);
#pragma unroll
  for (int d = 1; d < DEPTH - 1; ++d) {
    advance();
    fetch(a[d], v[d]);
  }
  const int steps = p.chunks * p.kgroups;
  for (int step = 0; step < steps; step += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      advance();
      fetch(a[(d + DEPTH - 1) % DEPTH], v[(d + DEPTH - 1) % DEPTH]);
      feed_all<NACC, EPV>(acc, a[d], v[d]);
    }
  }

  // The compiler does not know that the statements above are MFMAs, whose results may be read
  // only a few cycles after issue: sixteen idle cycles before the epilogue (whose reads of the
  // accumulators lie behind the branches on `active` and on the phase's extent).
  if constexpr (NACC >= 8) asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
  if (!active) return;
  float *const dst_n = p.dst + (long long)n * p.dst_nstride + (long long)pass * 4 * RG * p.dst_mstride;
#pragma unroll
  for (int ph = 0; ph < NPH; ++ph) {
    const bool here = (int)j0 < p.pJ[ph][0] && (int)j1 < p.pJ[ph][1] && (int)j2 < p.pJ[ph][2];
    const long long o = (long long)((int)j0 * p.oj[0] + p.po0[ph][0]) * p.os[0] + (long long)((int)j1 * p.oj[1] + p.po0[ph][1]) * p.os[1] +
                        (long long)((int)j2 * p.oj[2] + p.po0[ph][2]) * p.os[2];
    if (NPH > 1 && p.pair_store) {
      // phases 2q and 2q + 1 lie side by side in dst: one 8-byte store for both
      if ((ph & 1) == 0 && here) {
#pragma unroll
        for (int r = 0; r < RG; ++r)
#pragma unroll
          for (int m = 0; m < 4; ++m)
            if (r * 4 + m < rows_left)
              *reinterpret_cast<f32x2 *>(dst_n + (long long)(r * 4 + m) * p.dst_mstride + o) = f32x2{acc[ph * RG + r][m], acc[(ph | 1) * RG + r][m]};
      }
    } else if (here) {
#pragma unroll
      for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int m = 0; m < 4; ++m)
          if (r * 4 + m < rows_left) dst_n[(long long)(r * 4 + m) * p.dst_mstride + o] = acc[ph * RG + r][m];
    }
  }
}

// packed[((pass * chunks + q) * kgroups + kg) * 64 + slot * 4 + m] =
//     w[arow[q * 16 + slot] + kg * group_stride + (pass * 4 * rg + m) * m_stride]
// (zero where arow is negative or the slot's row group, slot % rg, ends before that row)
__global__ void __launch_bounds__(256) thin_pack_kernel(const float *__restrict__ w, float *__restrict__ packed, const int *__restrict__ arow,
                                                        int chunks, int kgroups, long long group_stride, int m_stride, int M, int rg,
                                                        int passes) {
  const long long per_pass = (long long)chunks * kgroups * 64;
  const long long total = per_pass * passes;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
    const int pass = (int)(i / per_pass);
    const long long j = i - (long long)pass * per_pass;
    const int m = (int)(j & 3), slot = (int)((j >> 2) & 15);
    const long long qk = j >> 6;
    const int q = (int)(qk / kgroups), kg = (int)(qk - (long long)q * kgroups);
    const int row = arow[q * 16 + slot];
    const int first = pass * 4 * rg;  // first row of the pass; the slot's group starts (slot % rg) * 4 rows further on
    packed[i] = (row >= 0 && first + (slot % rg) * 4 + m < M) ? w[row + kg * group_stride + (long long)(first + m) * m_stride] : 0.f;
  }
}

}  // namespace

int launch_thin_pack(const float *w, float *packed, const int *arow, int chunks, int kgroups, long long group_stride, int m_stride, int M,
                     int rg, int passes, hipStream_t s) {
  const long long total = (long long)chunks * kgroups * 64 * passes;
  const unsigned blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  hipLaunchKernelGGL(thin_pack_kernel, dim3(blocks ? blocks : 1), dim3(256), 0, s, w, packed, arow, chunks, kgroups, group_stride, m_stride, M,
                     rg, passes);
  hipError_t err = hipGetLastError();
  return err == hipSuccess ? MG_OK : hip_fail(err, "thin_pack_kernel", __FILE__, __LINE__);
}

// (stride phases, row groups) the kernel is built for: their product is at most 16.  The callers
// use stride phases for the data gradient of up to four channels (one row group) and row groups
// for the forward pass (one phase); each pair listed here has an exact-integer test.
#define MG_THIN_SHAPES(X) X(1, 1) X(1, 2) X(1, 4) X(1, 8) X(1, 16) X(2, 1) X(4, 1)

bool thin_gemm_has(int nph, int rg) {
#define MG_THIN_HAS(NPH, RG) \
  if (nph == NPH && rg == RG) return true;
  MG_THIN_SHAPES(MG_THIN_HAS)
#undef MG_THIN_HAS
  return false;
}

int launch_thin_gemm(const ThinParams &p, hipStream_t s) {
  const unsigned blocks = (unsigned)((p.npos + 255) / 256);
  bool launched = false;
#define MG_THIN_LAUNCH(NPH, RG)                                                               \
  if (p.nph == NPH && p.rg == RG) {                                                            \
    hipLaunchKernelGGL((thin_gemm_kernel<NPH, RG>), dim3(blocks, (unsigned)p.passes), dim3(256), 0, s, p); \
    launched = true;                                                                           \
  }
  MG_THIN_SHAPES(MG_THIN_LAUNCH)
#undef MG_THIN_LAUNCH
  if (!launched) return fail(MG_ERR_UNSUPPORTED, "one-position-per-lane gather-GEMM with %d phases x %d row groups", p.nph, p.rg);
  hipError_t err = hipGetLastError();
  return err == hipSuccess ? MG_OK : hip_fail(err, "thin_gemm_kernel", __FILE__, __LINE__);
}

}  // namespace mg
