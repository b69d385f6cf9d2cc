/* Definition-level CPU reference for conv_nd / max_pool.  TEST INFRASTRUCTURE.
 *
 * Written from the closed-form definitions the reference implements
 *   conv fwd  src/mygrad/nnet/layers/conv.py:86-103
 *   conv dx   src/mygrad/nnet/layers/conv.py:115-138
 *   conv dw   src/mygrad/nnet/layers/conv.py:143-155
 *   pool      src/mygrad/nnet/layers/pooling.py:93, :109-149
 * as plain loops (no im2col, no BLAS), accumulating in double whatever the input
 * type, so it is independent of the NumPy restatement and usable at the full
 * benchmark sizes.  Spatial rank is always 3 here: callers pad missing leading
 * axes with extent 1 (stride 1, padding 0, dilation 1).
 *
 * Only tests, the smoke check and the benchmark's checker may load this.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

typedef struct {
  int64_t N, C, F;
  int64_t X[3], W[3], G[3], S[3], P[3], D[3];
} conv_shape;

#define XVOL(s) ((s)->X[0] * (s)->X[1] * (s)->X[2])
#define WVOL(s) ((s)->W[0] * (s)->W[1] * (s)->W[2])
#define GVOL(s) ((s)->G[0] * (s)->G[1] * (s)->G[2])

#define DEFINE_CONV(T, SUF)                                                                  \
  /* out[n,f,g] = sum_{c,t} w[f,c,t] * x[n,c,g*s+t*d-p]  (zero outside x) */                 \
  void direct_conv_fwd_##SUF(const conv_shape *s, const T *x, const T *w, double *out) {     \
    const int64_t xv = XVOL(s), wv = WVOL(s), gv = GVOL(s);                                  \
    _Pragma("omp parallel for collapse(2) schedule(dynamic)")                                \
    for (int64_t n = 0; n < s->N; ++n)                                                       \
      for (int64_t f = 0; f < s->F; ++f) {                                                   \
        double *o = out + (n * s->F + f) * gv;                                               \
        memset(o, 0, sizeof(double) * (size_t)gv);                                           \
        for (int64_t c = 0; c < s->C; ++c) {                                                 \
          const T *xp = x + (n * s->C + c) * xv;                                             \
          const T *wp = w + (f * s->C + c) * wv;                                             \
          for (int64_t t0 = 0; t0 < s->W[0]; ++t0)                                           \
            for (int64_t t1 = 0; t1 < s->W[1]; ++t1)                                         \
              for (int64_t t2 = 0; t2 < s->W[2]; ++t2) {                                     \
                const double wt = (double)wp[(t0 * s->W[1] + t1) * s->W[2] + t2];            \
                for (int64_t g0 = 0; g0 < s->G[0]; ++g0) {                                   \
                  const int64_t q0 = g0 * s->S[0] + t0 * s->D[0] - s->P[0];                  \
                  if (q0 < 0 || q0 >= s->X[0]) continue;                                     \
                  for (int64_t g1 = 0; g1 < s->G[1]; ++g1) {                                 \
                    const int64_t q1 = g1 * s->S[1] + t1 * s->D[1] - s->P[1];                \
                    if (q1 < 0 || q1 >= s->X[1]) continue;                                   \
                    const T *xr = xp + (q0 * s->X[1] + q1) * s->X[2];                        \
                    double *orow = o + (g0 * s->G[1] + g1) * s->G[2];                        \
                    const int64_t off = t2 * s->D[2] - s->P[2], st = s->S[2];                \
                    for (int64_t g2 = 0; g2 < s->G[2]; ++g2) {                               \
                      const int64_t q2 = g2 * st + off;                                      \
                      if (q2 >= 0 && q2 < s->X[2]) orow[g2] += wt * (double)xr[q2];          \
                    }                                                                        \
                  }                                                                          \
                }                                                                            \
              }                                                                              \
        }                                                                                    \
      }                                                                                      \
  }                                                                                          \
  /* dx[n,c,q] = sum over (f,t,g) with g*s+t*d-p == q of grad[n,f,g]*w[f,c,t] */             \
  void direct_conv_dx_##SUF(const conv_shape *s, const T *grad, const T *w, double *dx) {    \
    const int64_t xv = XVOL(s), wv = WVOL(s), gv = GVOL(s);                                  \
    _Pragma("omp parallel for collapse(2) schedule(dynamic)")                                \
    for (int64_t n = 0; n < s->N; ++n)                                                       \
      for (int64_t c = 0; c < s->C; ++c) {                                                   \
        double *o = dx + (n * s->C + c) * xv;                                                \
        memset(o, 0, sizeof(double) * (size_t)xv);                                           \
        for (int64_t f = 0; f < s->F; ++f) {                                                 \
          const T *gp = grad + (n * s->F + f) * gv;                                          \
          const T *wp = w + (f * s->C + c) * wv;                                             \
          for (int64_t t0 = 0; t0 < s->W[0]; ++t0)                                           \
            for (int64_t t1 = 0; t1 < s->W[1]; ++t1)                                         \
              for (int64_t t2 = 0; t2 < s->W[2]; ++t2) {                                     \
                const double wt = (double)wp[(t0 * s->W[1] + t1) * s->W[2] + t2];            \
                for (int64_t g0 = 0; g0 < s->G[0]; ++g0) {                                   \
                  const int64_t q0 = g0 * s->S[0] + t0 * s->D[0] - s->P[0];                  \
                  if (q0 < 0 || q0 >= s->X[0]) continue;                                     \
                  for (int64_t g1 = 0; g1 < s->G[1]; ++g1) {                                 \
                    const int64_t q1 = g1 * s->S[1] + t1 * s->D[1] - s->P[1];                \
                    if (q1 < 0 || q1 >= s->X[1]) continue;                                   \
                    double *orow = o + (q0 * s->X[1] + q1) * s->X[2];                        \
                    const T *grow = gp + (g0 * s->G[1] + g1) * s->G[2];                      \
                    const int64_t off = t2 * s->D[2] - s->P[2], st = s->S[2];                \
                    for (int64_t g2 = 0; g2 < s->G[2]; ++g2) {                               \
                      const int64_t q2 = g2 * st + off;                                      \
                      if (q2 >= 0 && q2 < s->X[2]) orow[q2] += wt * (double)grow[g2];        \
                    }                                                                        \
                  }                                                                          \
                }                                                                            \
              }                                                                              \
        }                                                                                    \
      }                                                                                      \
  }                                                                                          \
  /* dw[f,c,t] = sum_{n,g} grad[n,f,g] * x[n,c,g*s+t*d-p] */                                 \
  void direct_conv_dw_##SUF(const conv_shape *s, const T *grad, const T *x, double *dw) {    \
    const int64_t xv = XVOL(s), wv = WVOL(s), gv = GVOL(s);                                  \
    _Pragma("omp parallel for collapse(2) schedule(dynamic)")                                \
    for (int64_t f = 0; f < s->F; ++f)                                                       \
      for (int64_t c = 0; c < s->C; ++c) {                                                   \
        double *o = dw + (f * s->C + c) * wv;                                                \
        for (int64_t t0 = 0; t0 < s->W[0]; ++t0)                                             \
          for (int64_t t1 = 0; t1 < s->W[1]; ++t1)                                           \
            for (int64_t t2 = 0; t2 < s->W[2]; ++t2) {                                       \
              double acc = 0.0;                                                              \
              for (int64_t n = 0; n < s->N; ++n) {                                           \
                const T *gp = grad + (n * s->F + f) * gv;                                    \
                const T *xp = x + (n * s->C + c) * xv;                                       \
                for (int64_t g0 = 0; g0 < s->G[0]; ++g0) {                                   \
                  const int64_t q0 = g0 * s->S[0] + t0 * s->D[0] - s->P[0];                  \
                  if (q0 < 0 || q0 >= s->X[0]) continue;                                     \
                  for (int64_t g1 = 0; g1 < s->G[1]; ++g1) {                                 \
                    const int64_t q1 = g1 * s->S[1] + t1 * s->D[1] - s->P[1];                \
                    if (q1 < 0 || q1 >= s->X[1]) continue;                                   \
                    const T *xr = xp + (q0 * s->X[1] + q1) * s->X[2];                        \
                    const T *grow = gp + (g0 * s->G[1] + g1) * s->G[2];                      \
                    const int64_t off = t2 * s->D[2] - s->P[2], st = s->S[2];                \
                    double row = 0.0;                                                        \
                    for (int64_t g2 = 0; g2 < s->G[2]; ++g2) {                               \
                      const int64_t q2 = g2 * st + off;                                      \
                      if (q2 >= 0 && q2 < s->X[2]) row += (double)grow[g2] * (double)xr[q2]; \
                    }                                                                        \
                    acc += row;                                                              \
                  }                                                                          \
                }                                                                            \
              }                                                                              \
              o[(t0 * s->W[1] + t1) * s->W[2] + t2] = acc;                                   \
            }                                                                                \
      }                                                                                      \
  }

DEFINE_CONV(float, f32)
DEFINE_CONV(double, f64)

typedef struct {
  int64_t lead;
  int64_t X[3], P[3], S[3], G[3];
} pool_shape;

/* Per leading index, windows in ascending row-major grid order; the window's
 * gradient goes to the first element (row-major inside the window) that
 * attains the maximum, or to the first NaN; dx accumulates in double from +0.0.
 * `grad` and `dx` may be NULL to run the forward only. */
#define DEFINE_POOL(T, SUF)                                                                  \
  void direct_pool_##SUF(const pool_shape *s, const T *x, const T *grad, T *out, double *dx) { \
    const int64_t xv = s->X[0] * s->X[1] * s->X[2], gv = s->G[0] * s->G[1] * s->G[2];        \
    _Pragma("omp parallel for schedule(static)")                                             \
    for (int64_t l = 0; l < s->lead; ++l) {                                                  \
      const T *xp = x + l * xv;                                                              \
      if (dx) memset(dx + l * xv, 0, sizeof(double) * (size_t)xv);                           \
      for (int64_t g0 = 0; g0 < s->G[0]; ++g0)                                               \
        for (int64_t g1 = 0; g1 < s->G[1]; ++g1)                                             \
          for (int64_t g2 = 0; g2 < s->G[2]; ++g2) {                                         \
            int64_t best = -1;                                                               \
            T bv = 0;                                                                        \
            int done = 0;                                                                    \
            for (int64_t a0 = 0; a0 < s->P[0] && !done; ++a0)                                \
              for (int64_t a1 = 0; a1 < s->P[1] && !done; ++a1)                              \
                for (int64_t a2 = 0; a2 < s->P[2]; ++a2) {                                   \
                  const int64_t q = ((g0 * s->S[0] + a0) * s->X[1] + g1 * s->S[1] + a1) *    \
                                        s->X[2] + g2 * s->S[2] + a2;                         \
                  const T v = xp[q];                                                         \
                  if (v != v) { best = q; bv = v; done = 1; break; }                         \
                  if (best < 0 || v > bv) { best = q; bv = v; }                              \
                }                                                                            \
            const int64_t go = (g0 * s->G[1] + g1) * s->G[2] + g2;                           \
            if (out) out[l * gv + go] = bv;                                                  \
            if (dx) dx[l * xv + best] += (double)grad[l * gv + go];                          \
          }                                                                                  \
    }                                                                                        \
  }

DEFINE_POOL(float, f32)
DEFINE_POOL(double, f64)
