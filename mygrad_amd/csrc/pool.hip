// Max-pool forward and backward (gather form) for gfx950.
//
// Index algebra (rank padded to 3, row-major):
//   out[l, g]  = max_a x[l, g*S + a]                      a in prod [0, P_k)
//   dx[l, i]  += grad[l, g]  for every window g whose first-occurrence argmax
//                (row-major inside the window; the first NaN if any) is i,
//                windows taken in ascending row-major order, sum started at
//                +0.0 and carried in double.
#include "internal.h"

namespace mg {

struct PoolParams {
  int X[3], P[3], S[3], G[3];
  long long lead, xvol, gvol;
};

// `cand` replaces `best` when it is the first NaN, or strictly greater than a
// non-NaN best: ties keep the earlier element, a NaN once met is never replaced.
template <typename T>
__device__ __forceinline__ bool takes_over(T cand, T best) {
  return (best == best) && (cand > best || cand != cand);
}

template <typename T>
__global__ void __launch_bounds__(256) maxpool_fwd_kernel(PoolParams p, const T *__restrict__ x,
                                                          T *__restrict__ out) {
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
    for (int a0 = 0; a0 < p.P[0]; ++a0)
      for (int a1 = 0; a1 < p.P[1]; ++a1) {
        const T *row = w + ((long long)a0 * p.X[1] + a1) * p.X[2];
        for (int a2 = 0; a2 < p.P[2]; ++a2) {
          const T v = row[a2];
          if (takes_over(v, best)) best = v;
        }
      }
    out[idx] = best;
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

static unsigned grid_for(long long total) {
  long long blocks = ceil_div(total, 256);
  const long long cap = (long long)runtime().props.multiProcessorCount * 32;
  return (unsigned)(blocks < cap ? blocks : cap);
}

}  // namespace mg

using namespace mg;

extern "C" {

int mg_maxpool_fwd(const mg_pool_desc *desc, const void *x, void *out) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  PoolParams p;
  if (int rc = check_pool_desc(desc, &p)) return rc;
  if (!x || !out) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_maxpool_fwd");
  const unsigned grid = grid_for(p.lead * p.gvol);
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_POOL_FWD);
  if (desc->dtype == MG_F32)
    hipLaunchKernelGGL(maxpool_fwd_kernel<float>, dim3(grid), dim3(256), 0, s, p, (const float *)x, (float *)out);
  else
    hipLaunchKernelGGL(maxpool_fwd_kernel<double>, dim3(grid), dim3(256), 0, s, p, (const double *)x, (double *)out);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_maxpool_bwd(const mg_pool_desc *desc, const void *x, const void *grad, void *dx) {
  std::lock_guard<std::recursive_mutex> guard(api_mutex());
  MG_REQUIRE_INIT();
  PoolParams p;
  if (int rc = check_pool_desc(desc, &p)) return rc;
  if (!x || !grad || !dx) return fail(MG_ERR_BAD_ARG, "null tensor pointer in mg_maxpool_bwd");
  const unsigned grid = grid_for(p.lead * p.xvol);
  hipStream_t s = runtime().stream;
  ScopedTiming timed(TAG_POOL_BWD);
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
