// Shared declarations of libmellin_hip: problem descriptors, the per-axis tap
// relation, and the launchers each translation unit exports to the C API.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace mellin {

typedef int64_t i64;

enum AxisKind : int { AX_MCORR = 0, AX_MCONV = 1, AX_LCORR = 2, AX_LCONV = 3 };

// One axis of a separable tap structure: output index h and filter index f
// select signal index g, or nothing.
struct Axis {
  int kind;
  i64 nf, ng, nh;    // filter, signal, allocated output lengths
  i64 s, d, p, u;
  i64 nh_eff;        // min(nh, support size): outputs at or past it have no tap
};

// h[n, m, hx, hy] (+)= sum_{c, fx, fy} f[m, c, fx, fy] * g[n, c, tap_x(hx, fx), tap_y(hy, fy)]
// with every tensor addressed through explicit element strides so that the
// transposed layouts of the reference contract and the role swaps of the
// backward passes need no copies.
struct SepConv {
  Axis x, y;
  i64 batch, c_out, c_in;        // c_out: output channels (m), c_in: contracted channels (c)
  i64 f_m, f_c;                  // filter strides; spatial part is dense (nfx, nfy)
  i64 g_n, g_c;                  // signal strides; spatial part is dense (ngx, ngy)
  i64 h_n, h_m;                  // output strides; spatial part is dense (nhx, nhy)
  int accumulate;                // 1: h += result (h pre-initialised); 0: h = bias + result
  int relu = 0;                  // with accumulate == 0: h = max(0, bias + result)
  int out_half = 0;              // with accumulate == 0: h is half-precision storage (matrix-core kernel only)
  int in_half = 0;               // f, g and bias are half-precision storage (matrix-core kernel only; accumulate == 0)
  // One residue class of a Mellin x axis (matrix-core kernel, bf16 / f16 forms only): the
  // launch covers the output rows cls_first, cls_first + cls_stride, ... and the cls_nfx
  // filter rows listed in cls_fx (four bits each, lowest first) -- the rows and filter rows
  // among which every pair has its tap (tile_gemm.hpp: mellin_classes).  cls_nfx == 0: all.
  int cls_stride = 1, cls_first = 0, cls_nfx = 0;
  unsigned long long cls_fx = 0;
  int math = 0;                  // MATH_FP32: fp32 matrix instructions; MATH_BF16X3: bf16 ones on three-part operands
};

enum MathMode : int { MATH_FP32 = 0, MATH_BF16X3 = 1, MATH_BF16X3_ALWAYS = 2 };   // ALWAYS: no size heuristics

// Reduction form used by the weight gradient:
// w[m, c, fx, fy] = sum_{n, hx, hy} a[n, m, hx, hy] * g[n, c, tap_x(hx, fx), tap_y(hy, fy)]
struct SepReduce {
  Axis x, y;                     // nf = filter size (output of the reduction), nh = size of `a`
  i64 batch, c_out, c_in;
};

__host__ __device__ inline i64 floor_div(i64 a, i64 b) {
  i64 q = a / b;
  return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q;
}

// Signal index chosen by (h, f) on one axis, or -1.  p1 = p + 1.
__host__ __device__ inline i64 tap_index(int kind, i64 h, i64 f, i64 ng, i64 s,
                                         i64 d, i64 p, i64 u) {
  i64 num, den, off = 0;
  switch (kind) {
    case AX_MCORR: num = (h + s) * (f + d); den = p + 1; off = u; break;
    case AX_MCONV: num = (p + 1) * (h + s); den = f + d; off = u; break;
    case AX_LCORR: num = s * h + d * f - p; den = u; break;
    default:       num = s * h - d * f + p; den = u; break;
  }
  if (num % den != 0) return -1;
  const i64 g = num / den - off;
  return (g >= 0 && g < ng) ? g : -1;
}

// Signal index chosen by (h, f) on one axis, or -1, in 32-bit arithmetic with a
// float-reciprocal division.  Exact while numerators stay below 2^22 (launchers check
// axis_fits_tap32); p1 = p + 1.
__device__ __forceinline__ int tap32(int kind, int h, int f, int ng, int s, int d, int p, int u) {
  int num, den, off = 0;
  switch (kind) {
    case AX_MCORR: num = (h + s) * (f + d); den = p + 1; off = u; break;
    case AX_MCONV: num = (p + 1) * (h + s); den = f + d; off = u; break;
    case AX_LCORR: num = s * h + d * f - p; den = u; break;
    default:       num = s * h - d * f + p; den = u; break;
  }
  if (num < 0) return -1;                               // linear kinds only; a negative index is no tap
  int q = (int)((float)num * (1.0f / (float)den));
  int r = num - q * den;
  if (r < 0) { --q; r += den; }
  else if (r >= den) { ++q; r -= den; }
  if (r != 0) return -1;
  const int g = q - off;
  return (g >= 0 && g < ng) ? g : -1;
}

// Every numerator of the tap relations of `a` stays below 2^22 (what tap32 needs).
inline bool axis_fits_tap32(const Axis &a) {
  const i64 lim = (i64)1 << 22;
  return (a.nh + a.s) * (a.nf + a.d) < lim && (a.p + 1) * (a.nh + a.s) < lim &&
         a.s * a.nh + a.d * a.nf + (a.p < 0 ? -a.p : a.p) < lim && a.u < lim && a.p + 1 < lim && a.nf + a.d < lim;
}

inline i64 support_size(int kind, i64 nf, i64 ng, i64 s, i64 d, i64 p, i64 u) {
  i64 v;
  switch (kind) {
    case AX_MCORR: v = floor_div((ng + u - 1) * (p + 1), d) - s + 1; break;
    case AX_MCONV: v = floor_div((nf + d - 1) * (ng + u - 1), p + 1) - s + 1; break;
    case AX_LCORR: v = floor_div(u * (ng - 1) + p, s) + 1; break;
    default:       v = floor_div(u * (ng - 1) + d * (nf - 1) - p, s) + 1; break;
  }
  return v > 0 ? v : 0;
}

inline Axis make_axis(int kind, i64 nf, i64 ng, i64 nh, i64 s, i64 d, i64 p, i64 u) {
  Axis a;
  a.kind = kind; a.nf = nf; a.ng = ng; a.nh = nh; a.s = s; a.d = d; a.p = p; a.u = u;
  const i64 sup = support_size(kind, nf, ng, s, d, p, u);
  a.nh_eff = sup < nh ? sup : nh;
  return a;
}

// Opt a kernel in to more dynamic LDS than a launch gets by default (asked for from 48 KB on).  The attribute belongs to the
// function, for the whole process, while launches come from any thread (PyTorch runs backward
// passes on a thread of its own): it is set once per kernel instance, to all a CU has (160 KB on
// gfx950), so that no later launch with another size on another thread can find it too small.
// `done`: one flag per kernel instance.
inline hipError_t allow_large_lds(const void *kernel, size_t lds_bytes, std::atomic<int> &done) {
  if (lds_bytes <= 48 * 1024 || done.load(std::memory_order_acquire)) return hipSuccess;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (e == hipSuccess) done.store(1, std::memory_order_release);
  return e;
}

// ---- launchers (each returns the hipError_t of the launch) ----------------
template <typename T>
hipError_t launch_sepconv_generic(const SepConv &pr, const T *f, const T *g,
                                  const T *bias, T *h, hipStream_t stream);
template <typename T>
hipError_t launch_sepreduce_generic(const SepReduce &pr, const T *a, const T *g,
                                    T *w, hipStream_t stream);

// (half_out: grad_input is half-precision storage, each fp32 sum rounded once)
hipError_t launch_fold_x(const Axis &x, i64 batch_cin, i64 ngx, i64 ngy, const float *Y,
                         void *grad_input, hipStream_t stream, bool half_out = false);

template <typename T>
hipError_t launch_spec2col(const Axis &x, const Axis &y, i64 c_in, i64 batch, int transposed_g,
                           int transposed_gg, const T *g, T *gg, hipStream_t stream);
// (O: the type g is stored in; sums are formed in T)
template <typename T, typename O = T>
hipError_t launch_col2spec(const Axis &x, const Axis &y, i64 c_in, i64 batch, int transposed_g,
                           int transposed_gg, const T *gg, O *g, hipStream_t stream);

bool launch_col2spec_padded(const Axis &x, const Axis &y, i64 pairs, i64 taps_padded, const float *gg,
                            float *g, hipStream_t stream, hipError_t *err);

hipError_t launch_fold_xy(const Axis &x, const Axis &y, i64 batch_cin, int nf_pad, const float *Z,
                          float *grad_input, hipStream_t stream);

// pointwise.hip: log compression and dilation lift over x viewed as (outer, t, inner).
// params (device memory, or null): {eps, tau} read by the kernels instead of the arguments
size_t log_lift_workspace_bytes(i64 outer, i64 t, i64 inner, size_t elem);
template <typename T>
hipError_t launch_log_lift_forward(const T *x, T eps, T tau, bool with_log, bool with_lift, i64 outer, i64 t,
                                   i64 inner, T *y, hipStream_t stream, const T *params = nullptr);
template <typename T>
hipError_t launch_log_lift_backward(const T *x, const T *gy, T eps, T tau, bool with_log, bool with_lift,
                                    i64 outer, i64 t, i64 inner, T *gx, T *grad_params, T *workspace,
                                    hipStream_t stream, const T *params = nullptr);

// pointwise.hip: per-channel sums of grad_out (N, C, plane), optionally masked by out > 0 (the masked
// gradient is then written to grad_masked); workspace of bias_grad_workspace_bytes()
size_t bias_grad_workspace_bytes(i64 batch, i64 channels, i64 plane);
// (T: float or _Float16; the sums are fp32 either way)
template <typename T>
hipError_t launch_bias_grad(const T *grad_out, const T *out, i64 batch, i64 channels, i64 plane,
                            T *grad_masked, T *grad_bias, float *workspace, hipStream_t stream);

// pointwise.hip: max over pairs of neighbours along the last axis of x (rows, f), and its backward
template <typename T>
hipError_t launch_pool_pairs_forward(const T *x, i64 rows, i64 f, T *y, unsigned char *which,
                                     hipStream_t stream);
template <typename T>
hipError_t launch_pool_pairs_backward(const T *gy, const unsigned char *which, i64 rows, i64 f, T *gx,
                                      hipStream_t stream);

// half <-> float copies of n elements (16 bytes at a time when both buffers are 16-byte aligned)
hipError_t launch_half_to_float(const void *src, float *dst, i64 n, hipStream_t stream);
hipError_t launch_float_to_half(const float *src, void *dst, i64 n, hipStream_t stream);

}  // namespace mellin
