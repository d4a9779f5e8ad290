// ref_shim.cpp -- C entry points onto the UNMODIFIED reference header.
// TEST INFRASTRUCTURE ONLY; built by oracle/Makefile into oracle/_ref/ when a
// reference checkout is present, never committed, never used by the product.
//
// The reference's CPU kernels are header-only templates
// (c/cpu/include/cdrobert/mellin/mconv.h, installed copy under ext/include
// together with the shipped config_cpu.h that selects the algorithm versions:
// MConv1D v2, MCorr1D v3, 2-D and column ops v1).  This translation unit only
// includes that header from where it lies and instantiates it for float and
// double behind extern "C" names so that Python (ctypes) can call the real
// thing: to validate the restatement in mellin_oracle.c and, optionally, to
// time the reference itself on the host cores.
#include <cstdint>
#include "cdrobert/mellin/mconv.h"

namespace cm = cdrobert::mellin;
typedef int64_t i64;

#define CONV2D(NAME, FUNC, T)                                                  \
  extern "C" void NAME(const T *f, const T *g, i64 c_out, i64 c_in, i64 batch, \
      i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy,    \
      i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, int tf, int tg, int th,  \
      T *h) {                                                                  \
    cm::FUNC<T>(f, g, c_out, c_in, batch, nfx, nfy, ngx, ngy, nhx, nhy, sx,    \
                sy, dx, dy, px, py, ux, uy, tf, tg, th, h);                    \
  }
#define CONV1D(NAME, FUNC, T)                                                  \
  extern "C" void NAME(const T *f, const T *g, i64 c_out, i64 c_in, i64 batch, \
      i64 nf, i64 ng, i64 nh, i64 s, i64 d, i64 p, i64 u, int tf, int tg,      \
      int th, T *h) {                                                          \
    cm::FUNC<T>(f, g, c_out, c_in, batch, nf, ng, nh, s, d, p, u, tf, tg, th,  \
                h);                                                            \
  }
#define COL2D(NAME, FUNC, T)                                                   \
  extern "C" void NAME(const T *in, i64 c_in, i64 batch, i64 nfx, i64 nfy,     \
      i64 ngx, i64 ngy, i64 nggx, i64 nggy, i64 sx, i64 sy, i64 dx, i64 dy,    \
      i64 px, i64 py, i64 ux, i64 uy, int tg, int tgg, T *out) {               \
    cm::FUNC<T>(in, c_in, batch, nfx, nfy, ngx, ngy, nggx, nggy, sx, sy, dx,   \
                dy, px, py, ux, uy, tg, tgg, out);                             \
  }
#define COL1D(NAME, FUNC, T)                                                   \
  extern "C" void NAME(const T *in, i64 c_in, i64 batch, i64 nf, i64 ng,       \
      i64 ngg, i64 s, i64 d, i64 p, i64 u, int tg, int tgg, T *out) {          \
    cm::FUNC<T>(in, c_in, batch, nf, ng, ngg, s, d, p, u, tg, tgg, out);       \
  }

CONV2D(ref_mcorrlcorr_f32, MCorrLCorr, float)
CONV2D(ref_mcorrlcorr_f64, MCorrLCorr, double)
CONV2D(ref_mconvlconv_f32, MConvLConv, float)
CONV2D(ref_mconvlconv_f64, MConvLConv, double)
CONV1D(ref_mcorr1d_f32, MCorr1D, float)
CONV1D(ref_mcorr1d_f64, MCorr1D, double)
CONV1D(ref_mconv1d_f32, MConv1D, float)
CONV1D(ref_mconv1d_f64, MConv1D, double)
COL2D(ref_spec2col_f32, Spec2Col, float)
COL2D(ref_spec2col_f64, Spec2Col, double)
COL2D(ref_col2spec_f32, Col2Spec, float)
COL2D(ref_col2spec_f64, Col2Spec, double)
COL1D(ref_snd2col_f32, Snd2Col, float)
COL1D(ref_snd2col_f64, Snd2Col, double)
COL1D(ref_col2snd_f32, Col2Snd, float)
COL1D(ref_col2snd_f64, Col2Snd, double)

// size functions keep the reference's own (shorter) argument lists
extern "C" i64 ref_mconv_valid_size(i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return cm::MConvValidSize(ng, s, d, p, u);
}
extern "C" i64 ref_mconv_support_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return cm::MConvSupportSize(nf, ng, s, d, p, u);
}
extern "C" i64 ref_lconv_valid_size(i64 ng, i64 s, i64 p, i64 u) {
  return cm::LConvValidSize(ng, s, p, u);
}
extern "C" i64 ref_lconv_support_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return cm::LConvSupportSize(nf, ng, s, d, p, u);
}
extern "C" i64 ref_mcorr_valid_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return cm::MCorrValidSize(nf, ng, s, d, p, u);
}
extern "C" i64 ref_mcorr_support_size(i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return cm::MCorrSupportSize(ng, s, d, p, u);
}
extern "C" i64 ref_lcorr_valid_size(i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  return cm::LCorrValidSize(nf, ng, s, d, p, u);
}
extern "C" i64 ref_lcorr_support_size(i64 ng, i64 s, i64 p, i64 u) {
  return cm::LCorrSupportSize(ng, s, p, u);
}
