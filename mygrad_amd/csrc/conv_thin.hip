// Gather-GEMM for convolutions with at most four rows: the data gradient of a layer with up
// to four channels (the first layer of an image network), the forward pass of a layer with
// up to four filters.  Single precision.
//
// A 16-row MFMA tile would carry 3 or 4 live rows.  v_mfma_f32_4x4x1_16b_f32 multiplies
// sixteen independent 4x1 by 1x4 blocks: lane l supplies B[l] and receives D[i][l], i = 0..3,
// in its four accumulator registers; with the A operand broadcast from one block (cbsz = 4,
// abid = the block), D[i][l] += A[4 * abid + i] * B[l].  So a lane IS a position: it gathers its
// own elements of src straight from memory (consecutive lanes, consecutive addresses), no LDS
// and no barrier, and one register of packed filters -- sixteen blocks of four rows -- feeds
// sixteen MFMAs.  With a stride, a lane owns one position of the coarse grid ceil(X / stride)
// and all of its stride phases, one accumulator each: the phases read the same neighbourhood
// of grad, so each gathered element feeds up to nph MFMAs (with weights that are zero where
// the phase has no tap for it).
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

// acc[ph] += A[block I * NPH + ph] * v for every phase; the block index is an immediate of the instruction
template <int NPH, int I>
__device__ __forceinline__ void feed(f32x4 (&acc)[NPH], float a, float v) {
  acc[0] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, v, acc[0], 4, I * NPH, 0);
  if constexpr (NPH >= 2) acc[1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, v, acc[1], 4, I * NPH + 1, 0);
  if constexpr (NPH >= 4) {
    acc[2] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, v, acc[2], 4, I * NPH + 2, 0);
    acc[3] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, v, acc[3], 4, I * NPH + 3, 0);
  }
}

template <int NPH, int EPV, int I = 0>
__device__ __forceinline__ void feed_all(f32x4 (&acc)[NPH], float a, const float (&v)[EPV]) {
  if constexpr (I < EPV) {
    feed<NPH, I>(acc, a, v[I]);
    feed_all<NPH, EPV, I + 1>(acc, a, v);
  }
}

template <int NPH>
__global__ void __launch_bounds__(256) thin_gemm_kernel(ThinParams p) {
  constexpr int EPV = 16 / NPH;  // entries per register of packed filters
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

  const __amdgpu_buffer_rsrc_t a_buf = buffer_of(p.A, p.a_bytes);
  const __amdgpu_buffer_rsrc_t src_buf = buffer_of(p.src, p.src_bytes);
  const int4v MG_CONSTANT *tab = (const int4v MG_CONSTANT *)p.tab;

  f32x4 acc[NPH];
#pragma unroll
  for (int ph = 0; ph < NPH; ++ph) acc[ph] = f32x4{0.f, 0.f, 0.f, 0.f};

  const unsigned a_lane = (unsigned)lane * 4u;
  for (int q = 0; q < p.chunks; ++q) {
    unsigned at[EPV];
#pragma unroll
    for (int i = 0; i < EPV; ++i) {
      const int4v e = tab[q * EPV + i];  // off, d0, d1, d2: the same for every lane
      const bool ok = active && (unsigned)(c0 + e.y) < (unsigned)p.Q[0] && (unsigned)(c1 + e.z) < (unsigned)p.Q[1] &&
                      (unsigned)(c2 + e.w) < (unsigned)p.Q[2];
      at[i] = ok ? src_at + (unsigned)(e.x * 4) : kOutside;
    }
    // two sets of registers take turns: the loads of one group are in flight while the other feeds the MFMAs
    const unsigned a_base = (unsigned)q * (unsigned)p.kgroups * 256u;
    float a0, a1, v0[EPV], v1[EPV];
    auto fetch = [&](int kg, float &a, float (&v)[EPV]) {
      a = buffer_load(a_buf, a_lane, a_base + (unsigned)kg * 256u);
      const unsigned s_uni = (unsigned)kg * p.group_bytes;
#pragma unroll
      for (int i = 0; i < EPV; ++i) v[i] = buffer_load(src_buf, at[i], s_uni);
      __builtin_amdgcn_sched_barrier(0);  // all of a group's loads are issued before the MFMAs that follow in the source
    };
    fetch(0, a0, v0);
    const int last = p.kgroups - 1;
    for (int kg = 0; kg < last; kg += 2) {
      fetch(kg + 1, a1, v1);
      feed_all<NPH, EPV>(acc, a0, v0);
      fetch(min(kg + 2, last), a0, v0);  // past the end: the last group once more, not fed
      feed_all<NPH, EPV>(acc, a1, v1);
    }
    if (p.kgroups & 1) feed_all<NPH, EPV>(acc, a0, v0);
  }

  if (!active) return;
  float *const dst_n = p.dst + (long long)n * p.dst_nstride;
#pragma unroll
  for (int ph = 0; ph < NPH; ++ph) {
    const bool here = (int)j0 < p.pJ[ph][0] && (int)j1 < p.pJ[ph][1] && (int)j2 < p.pJ[ph][2];
    const long long o = (long long)((int)j0 * p.oj[0] + p.po0[ph][0]) * p.os[0] + (long long)((int)j1 * p.oj[1] + p.po0[ph][1]) * p.os[1] +
                        (long long)((int)j2 * p.oj[2] + p.po0[ph][2]) * p.os[2];
    if (NPH > 1 && p.pair_store) {
      // phases 2q and 2q + 1 lie side by side in dst: one 8-byte store for both
      if ((ph & 1) == 0 && here) {
#pragma unroll
        for (int m = 0; m < 4; ++m)
          if (m < p.M) *reinterpret_cast<f32x2 *>(dst_n + (long long)m * p.dst_mstride + o) = f32x2{acc[ph][m], acc[ph | 1][m]};
      }
    } else if (here) {
#pragma unroll
      for (int m = 0; m < 4; ++m)
        if (m < p.M) dst_n[(long long)m * p.dst_mstride + o] = acc[ph][m];
    }
  }
}

// packed[(q * kgroups + kg) * 64 + slot * 4 + m] = w[arow[q * 16 + slot] + kg * group_stride + m * m_stride]
// (zero where arow is negative or m >= M)
__global__ void __launch_bounds__(256) thin_pack_kernel(const float *__restrict__ w, float *__restrict__ packed, const int *__restrict__ arow,
                                                        int chunks, int kgroups, long long group_stride, int m_stride, int M) {
  const long long total = (long long)chunks * kgroups * 64;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
    const int m = (int)(i & 3), slot = (int)((i >> 2) & 15);
    const long long qk = i >> 6;
    const int q = (int)(qk / kgroups), kg = (int)(qk - (long long)q * kgroups);
    const int row = arow[q * 16 + slot];
    packed[i] = (row >= 0 && m < M) ? w[row + kg * group_stride + (long long)m * m_stride] : 0.f;
  }
}

}  // namespace

int launch_thin_pack(const float *w, float *packed, const int *arow, int chunks, int kgroups, long long group_stride, int m_stride, int M,
                     hipStream_t s) {
  const long long total = (long long)chunks * kgroups * 64;
  const unsigned blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  hipLaunchKernelGGL(thin_pack_kernel, dim3(blocks ? blocks : 1), dim3(256), 0, s, w, packed, arow, chunks, kgroups, group_stride, m_stride, M);
  hipError_t err = hipGetLastError();
  return err == hipSuccess ? MG_OK : hip_fail(err, "thin_pack_kernel", __FILE__, __LINE__);
}

int launch_thin_gemm(const ThinParams &p, hipStream_t s) {
  const unsigned blocks = (unsigned)((p.npos + 255) / 256);
  if (p.nph == 1)
    hipLaunchKernelGGL(thin_gemm_kernel<1>, dim3(blocks), dim3(256), 0, s, p);
  else if (p.nph == 2)
    hipLaunchKernelGGL(thin_gemm_kernel<2>, dim3(blocks), dim3(256), 0, s, p);
  else if (p.nph == 4)
    hipLaunchKernelGGL(thin_gemm_kernel<4>, dim3(blocks), dim3(256), 0, s, p);
  else
    return fail(MG_ERR_UNSUPPORTED, "thin gather-GEMM with %d phases", p.nph);
  hipError_t err = hipGetLastError();
  return err == hipSuccess ? MG_OK : hip_fail(err, "thin_gemm_kernel", __FILE__, __LINE__);
}

}  // namespace mg
