// Column ops: the gather that unfolds a signal into one column per (filter
// tap, output position) pair, and its adjoint.
//
//   spec2col  gg[n, c, fx, fy, x, y] = g[n, c, tap_x(x, fx), tap_y(y, fy)]  (0 if no tap)
//   col2spec  g[n, c, gx, gy] = sum over the (fx, x), (fy, y) whose tap is (gx, gy) of gg[...]
//
// with a Mellin (or linear) correlation relation on x and a linear correlation
// relation on y; snd2col / col2snd are the nfy = ngy = nggy = 1 instances.
// col2spec is written as a gather over the inverse relation (the convolution
// kind with s and u exchanged), so each output sums its taps in ascending
// (fx, fy): a fixed order, no atomics.  One thread per output element,
// coalesced along y; both are pure data movement (HBM bound).
#include "mellin_common.hpp"

namespace mellin {

namespace {

template <typename T>
__global__ __launch_bounds__(256) void spec2col_kernel(const T *__restrict__ g, T *__restrict__ gg,
                                                       Axis x, Axis y, i64 c_in, i64 batch,
                                                       int transposed_g, int transposed_gg) {
  // x, y: correlation-kind axes with nf = taps, ng = signal extent, nh = column extent
  const i64 total = batch * c_in * x.nf * y.nf * x.nh * y.nh;
  const i64 step = (i64)gridDim.x * blockDim.x;
  for (i64 i = (i64)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
    i64 r = i;
    const i64 oy = r % y.nh; r /= y.nh;
    const i64 ox = r % x.nh; r /= x.nh;
    const i64 fy = r % y.nf; r /= y.nf;
    const i64 fx = r % x.nf; r /= x.nf;
    const i64 ci = transposed_gg ? r / batch : r % c_in;
    const i64 bt = transposed_gg ? r % batch : r / c_in;
    const i64 gx = tap_index(x.kind, ox, fx, x.ng, x.s, x.d, x.p, x.u);
    const i64 gy = tap_index(y.kind, oy, fy, y.ng, y.s, y.d, y.p, y.u);
    T v = 0;
    if (gx >= 0 && gy >= 0)
      v = g[((transposed_g ? ci * batch + bt : bt * c_in + ci) * x.ng + gx) * y.ng + gy];
    gg[i] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void col2spec_kernel(const T *__restrict__ gg, T *__restrict__ g,
                                                       Axis x, Axis y, i64 c_in, i64 batch,
                                                       int transposed_g, int transposed_gg) {
  // x, y: convolution-kind axes with nf = taps, ng = column extent, nh = signal extent
  const i64 total = batch * c_in * x.nh * y.nh;
  const i64 step = (i64)gridDim.x * blockDim.x;
  for (i64 i = (i64)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
    i64 r = i;
    const i64 gy = r % y.nh; r /= y.nh;
    const i64 gx = r % x.nh; r /= x.nh;
    const i64 ci = transposed_g ? r / batch : r % c_in;
    const i64 bt = transposed_g ? r % batch : r / c_in;
    const T *src = gg + (transposed_gg ? ci * batch + bt : bt * c_in + ci) * x.nf * y.nf * x.ng * y.ng;
    T acc = 0;
    for (i64 fx = 0; fx < x.nf; ++fx) {
      const i64 ox = tap_index(x.kind, gx, fx, x.ng, x.s, x.d, x.p, x.u);
      if (ox < 0) continue;
      for (i64 fy = 0; fy < y.nf; ++fy) {
        const i64 oy = tap_index(y.kind, gy, fy, y.ng, y.s, y.d, y.p, y.u);
        if (oy >= 0) acc += src[((fx * y.nf + fy) * x.ng + ox) * y.ng + oy];
      }
    }
    g[i] = acc;
  }
}

unsigned blocks_for(i64 total) {
  i64 b = (total + 255) / 256;
  if (b > (1 << 20)) b = 1 << 20;
  return (unsigned)b;
}

}  // namespace

template <typename T>
hipError_t launch_spec2col(const Axis &x, const Axis &y, i64 c_in, i64 batch, int transposed_g,
                           int transposed_gg, const T *g, T *gg, hipStream_t stream) {
  const i64 total = batch * c_in * x.nf * y.nf * x.nh * y.nh;
  if (total == 0) return hipSuccess;
  hipLaunchKernelGGL(spec2col_kernel<T>, dim3(blocks_for(total)), dim3(256), 0, stream, g, gg, x, y, c_in,
                     batch, transposed_g, transposed_gg);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_col2spec(const Axis &x, const Axis &y, i64 c_in, i64 batch, int transposed_g,
                           int transposed_gg, const T *gg, T *g, hipStream_t stream) {
  const i64 total = batch * c_in * x.nh * y.nh;
  if (total == 0) return hipSuccess;
  hipLaunchKernelGGL(col2spec_kernel<T>, dim3(blocks_for(total)), dim3(256), 0, stream, gg, g, x, y, c_in,
                     batch, transposed_g, transposed_gg);
  return hipGetLastError();
}

template hipError_t launch_spec2col<float>(const Axis &, const Axis &, i64, i64, int, int, const float *,
                                           float *, hipStream_t);
template hipError_t launch_spec2col<double>(const Axis &, const Axis &, i64, i64, int, int, const double *,
                                            double *, hipStream_t);
template hipError_t launch_col2spec<float>(const Axis &, const Axis &, i64, i64, int, int, const float *,
                                           float *, hipStream_t);
template hipError_t launch_col2spec<double>(const Axis &, const Axis &, i64, i64, int, int, const double *,
                                            double *, hipStream_t);

}  // namespace mellin
