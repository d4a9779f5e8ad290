/*
 * mellin_oracle.c -- CPU restatement of the reference's Mellin / linear
 * convolution arithmetic.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP kernels are compared against; it is
 * also timed as the host-CPU baseline.  Nothing in the shipped package may
 * import, link or call it: only tests/, the smoke check and the benchmark's
 * cpu_baseline leg do.
 *
 * Every routine restates an algorithm of the reference (paths relative to the
 * reference checkout):
 *   size functions        c/cpu/include/cdrobert/mellin/mconv.h:452-672
 *                         (Python twins mconv.py:73-118)
 *   tap index relations   mconv.h:24-25 (mconv), :65 (mcorr), :105-107
 *                         (mconv x lconv), :168-171 (mcorr x lcorr)
 *   tap range derivation  mconv.h:679-747
 *   MCorr1D               mconv.h:988-1021   (v1 loop nest: fx -> ci)
 *   MConv1D               mconv.h:827-862
 *   MCorrLCorr            mconv.h:1196-1242  (loop nest fx -> fy -> ci, then h[i] += acc)
 *   MConvLConv            mconv.h:1143-1190
 *   Snd2Col / Col2Snd     mconv.h:1247-1304
 *   Spec2Col / Col2Spec   mconv.h:1309-1380
 *   accumulator type      mconv.h:749-753 (float data -> float accumulator,
 *                         double -> double)
 *
 * How the restatement is organised.  The four reference kernels differ only
 * in how an output index and a filter index select a signal index along each
 * axis, so one loop nest is written once and parameterised by an "axis kind":
 *
 *   AX_MCORR  g = (h + s)(f + d)/(p + 1) - u      kept iff the division is exact
 *   AX_MCONV  g = (p + 1)(h + s)/(f + d) - u      kept iff the division is exact
 *   AX_LCORR  g = (s h + d f - p)/u               kept iff the division is exact
 *   AX_LCONV  g = (s h - d f + p)/u               kept iff the division is exact
 *
 * and in every case the tap is kept only when 0 <= g < ng.  The reference
 * reaches the same set of taps by first narrowing the filter range with
 * ceiling divisions (mconv.h:1220-1224, :1168-1172) and then testing the
 * remainder; outputs at or beyond min(support size, allocated size) are
 * skipped outright, as the reference's `if (hx >= Nhx) continue` does
 * (mconv.h:1204-1206, :1215).  A pure linear 2-D correlation
 * ("lconv2d"), which the reference delegates to torch.nn.Conv2d
 * (models.py:334-336), is the same loop nest with AX_LCORR on both axes.
 *
 * Parity pins (see tests/test_oracle_*.py): every known-answer table of
 * c/tests/test_*_buffers.h (float64, 1e-10), the compiled reference header
 * (oracle/_ref) on random and asymmetric cases, brute force from the index
 * relations above, torch.nn.functional.conv1d/conv2d for the linear axis, and
 * adjointness for the gradient identities.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

typedef int64_t i64;

enum { AX_MCORR = 0, AX_MCONV = 1, AX_LCORR = 2, AX_LCONV = 3 };

/* ---- integer helpers (floor division: mconv.h:774-778) ------------------ */
static i64 floordiv(i64 a, i64 b) {
  i64 q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
  return q;
}
static i64 imax0(i64 a) { return a > 0 ? a : 0; }

/* ---- the eight size functions (mconv.h:452-672, mconv.py:73-118) -------- */
i64 oracle_mconv_valid_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  (void)nf;
  return imax0(floordiv(d * (ng + u - 1), p + 1) - s + 1);
}
i64 oracle_mconv_support_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return imax0(floordiv((nf + d - 1) * (ng + u - 1), p + 1) - s + 1);
}
i64 oracle_lconv_valid_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  (void)nf; (void)d;
  return imax0(floordiv(u * (ng - 1) - p, s) + 1);
}
i64 oracle_lconv_support_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return imax0(floordiv(u * (ng - 1) + d * (nf - 1) - p, s) + 1);
}
i64 oracle_mcorr_valid_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return imax0(floordiv((ng + u - 1) * (p + 1), nf + d - 1) - s + 1);
}
i64 oracle_mcorr_support_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  (void)nf;
  return imax0(floordiv((ng + u - 1) * (p + 1), d) - s + 1);
}
i64 oracle_lcorr_valid_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return imax0(floordiv(u * (ng - 1) - d * (nf - 1) + p, s) + 1);
}
i64 oracle_lcorr_support_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  (void)nf; (void)d;
  return imax0(floordiv(u * (ng - 1) + p, s) + 1);
}

/* ---- tap relation -------------------------------------------------------
 * Returns the signal index selected by output index h and filter index f, or
 * -1 when the tap does not exist (inexact division or outside [0, ng)).
 * This is also the reference's explicit valid-index mask
 * (idx_map, mconv.h:1107-1113). */
i64 oracle_tap(int kind, i64 h, i64 f, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  i64 num, den, g;
  switch (kind) {
    case AX_MCORR: num = (h + s) * (f + d); den = p + 1; break;
    case AX_MCONV: num = (p + 1) * (h + s); den = f + d; break;
    case AX_LCORR: num = s * h + d * f - p; den = u; break;
    default:       num = s * h - d * f + p; den = u; break;
  }
  if (den == 0 || num % den != 0) return -1;
  g = num / den;
  if (kind == AX_MCORR || kind == AX_MCONV) g -= u;
  return (g >= 0 && g < ng) ? g : -1;
}

/* Fill map[h * nf + f] with oracle_tap(...) for h < nh, f < nf. */
void oracle_tap_map(int kind, i64 nf, i64 ng, i64 nh, i64 s, i64 d, i64 p, i64 u,
                    i64 *map) {
  for (i64 h = 0; h < nh; ++h)
    for (i64 f = 0; f < nf; ++f)
      map[h * nf + f] = oracle_tap(kind, h, f, ng, s, d, p, u);
}

/* min(support size, allocated size): outputs at or past it are skipped
 * (mconv.h:835, :995, :1151-1153, :1204-1206). */
static i64 support_clip(int kind, i64 nf, i64 ng, i64 nh, i64 s, i64 d, i64 p,
                        i64 u) {
  i64 sup;
  switch (kind) {
    case AX_MCORR: sup = oracle_mcorr_support_size(nf, ng, s, d, p, u); break;
    case AX_MCONV: sup = oracle_mconv_support_size(nf, ng, s, d, p, u); break;
    case AX_LCORR: sup = oracle_lcorr_support_size(nf, ng, s, d, p, u); break;
    default:       sup = oracle_lconv_support_size(nf, ng, s, d, p, u); break;
  }
  return sup < nh ? sup : nh;
}

/* ---- the shared loop nest ------------------------------------------------
 * h[n, co, hx, hy] += sum over fx, fy, ci of
 *     f[co, ci, fx, fy] * g[n, ci, tap_x(hx, fx), tap_y(hy, fy)]
 * with one work item per output element and the accumulation order
 * fx -> fy -> ci of mconv.h:1226-1240.  Layout flags follow mconv.h:29-50:
 * f is (c_out, c_in, ...) or (c_in, c_out, ...) when transposed_f, and
 * likewise g (batch, c_in) and h (batch, c_out). */
#define DEFINE_SEPCONV(NAME, T, ACC)                                           \
  void NAME(int kind_x, int kind_y, const T *f, const T *g, i64 c_out,         \
            i64 c_in, i64 batch, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx,  \
            i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux,   \
            i64 uy, int transposed_f, int transposed_g, int transposed_h,      \
            T *h) {                                                            \
    const i64 nf = nfx * nfy, ng = ngx * ngy;                                  \
    const i64 f_ci_stride = transposed_f ? c_out * nf : nf;                    \
    const i64 g_ci_stride = transposed_g ? batch * ng : ng;                    \
    const i64 total = batch * c_out * nhx * nhy;                               \
    const i64 Nhx = support_clip(kind_x, nfx, ngx, nhx, sx, dx, px, ux);       \
    const i64 Nhy = support_clip(kind_y, nfy, ngy, nhy, sy, dy, py, uy);       \
    if (total <= 0 || Nhx <= 0 || Nhy <= 0) return;                            \
    /* index maps first, as MCorr1D v3 does (mconv.h:1100-1113) */             \
    i64 *xmap = (i64 *)malloc(sizeof(i64) * (size_t)(Nhx * nfx + 1));          \
    i64 *ymap = (i64 *)malloc(sizeof(i64) * (size_t)(Nhy * nfy + 1));          \
    oracle_tap_map(kind_x, nfx, ngx, Nhx, sx, dx, px, ux, xmap);               \
    oracle_tap_map(kind_y, nfy, ngy, Nhy, sy, dy, py, uy, ymap);               \
    _Pragma("omp parallel for schedule(static)")                               \
    for (i64 i = 0; i < total; ++i) {                                          \
      const i64 hy = i % nhy, hx = (i / nhy) % nhx, ip = i / (nhy * nhx);      \
      if (hx >= Nhx || hy >= Nhy) continue;                                    \
      const i64 co = transposed_h ? ip / batch : ip % c_out;                   \
      const i64 bt = transposed_h ? ip % batch : ip / c_out;                   \
      const T *f_co = f + (transposed_f ? co : co * c_in) * nf;                \
      const T *g_bt = g + (transposed_g ? bt : bt * c_in) * ng;                \
      const i64 *xm = xmap + hx * nfx, *ym = ymap + hy * nfy;                  \
      ACC acc = 0;                                                             \
      for (i64 fx = 0; fx < nfx; ++fx) {                                       \
        const i64 gx = xm[fx];                                                 \
        if (gx < 0) continue;                                                  \
        for (i64 fy = 0; fy < nfy; ++fy) {                                     \
          const i64 gy = ym[fy];                                               \
          if (gy < 0) continue;                                                \
          const T *fp = f_co + fx * nfy + fy, *gp = g_bt + gx * ngy + gy;      \
          for (i64 ci = 0; ci < c_in; ++ci)                                    \
            acc += fp[ci * f_ci_stride] * gp[ci * g_ci_stride];                \
        }                                                                      \
      }                                                                        \
      h[i] += acc;                                                             \
    }                                                                          \
    free(xmap);                                                                \
    free(ymap);                                                                \
  }

DEFINE_SEPCONV(oracle_sepconv_f32, float, float)
DEFINE_SEPCONV(oracle_sepconv_f64, double, double)

/* ---- the reference's four kernels as instances of the loop nest --------- */
#define DEFINE_OPS(SUF, T)                                                     \
  void oracle_mcorrlcorr_##SUF(const T *f, const T *g, i64 c_out, i64 c_in,    \
      i64 batch, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy, i64 sx, \
      i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, int tf, int tg,  \
      int th, T *h) {                                                          \
    oracle_sepconv_##SUF(AX_MCORR, AX_LCORR, f, g, c_out, c_in, batch, nfx,    \
        nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux, uy, tf, tg, th,   \
        h);                                                                    \
  }                                                                            \
  void oracle_mconvlconv_##SUF(const T *f, const T *g, i64 c_out, i64 c_in,    \
      i64 batch, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy, i64 sx, \
      i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, int tf, int tg,  \
      int th, T *h) {                                                          \
    oracle_sepconv_##SUF(AX_MCONV, AX_LCONV, f, g, c_out, c_in, batch, nfx,    \
        nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux, uy, tf, tg, th,   \
        h);                                                                    \
  }                                                                            \
  /* linear on both axes: the "lconv2d" of the non-Mellin model */             \
  void oracle_lcorrlcorr_##SUF(const T *f, const T *g, i64 c_out, i64 c_in,    \
      i64 batch, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy, i64 sx, \
      i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, int tf, int tg,  \
      int th, T *h) {                                                          \
    oracle_sepconv_##SUF(AX_LCORR, AX_LCORR, f, g, c_out, c_in, batch, nfx,    \
        nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux, uy, tf, tg, th,   \
        h);                                                                    \
  }                                                                            \
  void oracle_lconvlconv_##SUF(const T *f, const T *g, i64 c_out, i64 c_in,    \
      i64 batch, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy, i64 sx, \
      i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, int tf, int tg,  \
      int th, T *h) {                                                          \
    oracle_sepconv_##SUF(AX_LCONV, AX_LCONV, f, g, c_out, c_in, batch, nfx,    \
        nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux, uy, tf, tg, th,   \
        h);                                                                    \
  }                                                                            \
  /* 1-D Mellin ops are the 2-D ops with a unit linear axis, the way           \
     c/tests/test_mcorrlcorr.cc:36-46 runs the 1-D tables through 2-D */       \
  void oracle_mcorr1d_##SUF(const T *f, const T *g, i64 c_out, i64 c_in,       \
      i64 batch, i64 nf, i64 ng, i64 nh, i64 s, i64 d, i64 p, i64 u, int tf,   \
      int tg, int th, T *h) {                                                  \
    oracle_sepconv_##SUF(AX_MCORR, AX_LCORR, f, g, c_out, c_in, batch, nf, 1,  \
        ng, 1, nh, 1, s, 1, d, 1, p, 0, u, 1, tf, tg, th, h);                  \
  }                                                                            \
  void oracle_mconv1d_##SUF(const T *f, const T *g, i64 c_out, i64 c_in,       \
      i64 batch, i64 nf, i64 ng, i64 nh, i64 s, i64 d, i64 p, i64 u, int tf,   \
      int tg, int th, T *h) {                                                  \
    oracle_sepconv_##SUF(AX_MCONV, AX_LCONV, f, g, c_out, c_in, batch, nf, 1,  \
        ng, 1, nh, 1, s, 1, d, 1, p, 0, u, 1, tf, tg, th, h);                  \
  }

DEFINE_OPS(f32, float)
DEFINE_OPS(f64, double)

/* ---- column ops (mconv.h:1247-1380) --------------------------------------
 * spec2col gathers gg[n, ci, fx, fy, x, y] = g[n, ci, tap_x(x, fx), tap_y(y, fy)]
 * (zero where the tap does not exist); col2spec is its adjoint written in
 * gather form: g[n, ci, gx, gy] = sum over fx, fy of gg[n, ci, fx, fy, x, y]
 * with x, y the outputs whose taps land on (gx, gy).  The 1-D ops are the
 * nfy = ngy = nggy = 1 instances.  The inverse tap of AX_MCORR is AX_MCONV
 * with (s, u) exchanged, and of AX_LCORR is AX_LCONV with (s, u) exchanged
 * (mconv.h:1294-1298, :1362-1372). */
#define DEFINE_COL(SUF, T, ACC)                                                \
  void oracle_spec2col_##SUF(const T *g, i64 c_in, i64 batch, i64 nfx,         \
      i64 nfy, i64 ngx, i64 ngy, i64 nggx, i64 nggy, i64 sx, i64 sy, i64 dx,   \
      i64 dy, i64 px, i64 py, i64 ux, i64 uy, int transposed_g,                \
      int transposed_gg, T *gg) {                                              \
    const i64 total = batch * c_in * nfx * nfy * nggx * nggy;                  \
    _Pragma("omp parallel for schedule(static)")                               \
    for (i64 i = 0; i < total; ++i) {                                          \
      i64 r = i;                                                               \
      const i64 y = r % nggy; r /= nggy;                                       \
      const i64 x = r % nggx; r /= nggx;                                       \
      const i64 fy = r % nfy; r /= nfy;                                        \
      const i64 fx = r % nfx; r /= nfx;                                        \
      const i64 ci = transposed_gg ? r / batch : r % c_in;                     \
      const i64 bt = transposed_gg ? r % batch : r / c_in;                     \
      const i64 gx = oracle_tap(AX_MCORR, x, fx, ngx, sx, dx, px, ux);         \
      const i64 gy = oracle_tap(AX_LCORR, y, fy, ngy, sy, dy, py, uy);         \
      T v = 0;                                                                 \
      if (gx >= 0 && gy >= 0)                                                  \
        v = g[((transposed_g ? ci * batch + bt : bt * c_in + ci) * ngx + gx)   \
              * ngy + gy];                                                     \
      gg[i] = v;                                                               \
    }                                                                          \
  }                                                                            \
  void oracle_col2spec_##SUF(const T *gg, i64 c_in, i64 batch, i64 nfx,        \
      i64 nfy, i64 ngx, i64 ngy, i64 nggx, i64 nggy, i64 sx, i64 sy, i64 dx,   \
      i64 dy, i64 px, i64 py, i64 ux, i64 uy, int transposed_g,                \
      int transposed_gg, T *g) {                                               \
    const i64 total = batch * c_in * ngx * ngy;                                \
    _Pragma("omp parallel for schedule(static)")                               \
    for (i64 i = 0; i < total; ++i) {                                          \
      i64 r = i;                                                               \
      const i64 gy = r % ngy; r /= ngy;                                        \
      const i64 gx = r % ngx; r /= ngx;                                        \
      const i64 ci = transposed_g ? r / batch : r % c_in;                      \
      const i64 bt = transposed_g ? r % batch : r / c_in;                      \
      const T *src = gg + (transposed_gg ? ci * batch + bt : bt * c_in + ci)   \
                          * nfx * nfy * nggx * nggy;                           \
      ACC acc = 0;                                                             \
      for (i64 fx = 0; fx < nfx; ++fx) {                                       \
        const i64 x = oracle_tap(AX_MCONV, gx, fx, nggx, ux, dx, px, sx);      \
        if (x < 0) continue;                                                   \
        for (i64 fy = 0; fy < nfy; ++fy) {                                     \
          const i64 y = oracle_tap(AX_LCONV, gy, fy, nggy, uy, dy, py, sy);    \
          if (y < 0) continue;                                                 \
          acc += src[((fx * nfy + fy) * nggx + x) * nggy + y];                 \
        }                                                                      \
      }                                                                        \
      g[i] = (T)acc;                                                           \
    }                                                                          \
  }                                                                            \
  void oracle_snd2col_##SUF(const T *g, i64 c_in, i64 batch, i64 nf, i64 ng,   \
      i64 ngg, i64 s, i64 d, i64 p, i64 u, int transposed_g,                   \
      int transposed_gg, T *gg) {                                              \
    oracle_spec2col_##SUF(g, c_in, batch, nf, 1, ng, 1, ngg, 1, s, 1, d, 1, p, \
        0, u, 1, transposed_g, transposed_gg, gg);                             \
  }                                                                            \
  void oracle_col2snd_##SUF(const T *gg, i64 c_in, i64 batch, i64 nf, i64 ng,  \
      i64 ngg, i64 s, i64 d, i64 p, i64 u, int transposed_g,                   \
      int transposed_gg, T *g) {                                               \
    oracle_col2spec_##SUF(gg, c_in, batch, nf, 1, ng, 1, ngg, 1, s, 1, d, 1,   \
        p, 0, u, 1, transposed_g, transposed_gg, g);                           \
  }

DEFINE_COL(f32, float, float)
DEFINE_COL(f64, double, double)
