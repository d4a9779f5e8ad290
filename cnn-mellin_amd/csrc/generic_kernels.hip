// Always-correct kernels: one thread per output element (gather form) and one
// workgroup per weight element (reduction form).  They take every parameter
// combination the index relations allow, any layout expressible by strides,
// and float or double data.  The tiled kernels are used instead wherever
// their preconditions hold; these remain the fallback and the in-library
// cross-check.
#include "mellin_common.hpp"

namespace mellin {

namespace {

constexpr int kThreads = 256;

template <typename T>
__global__ __launch_bounds__(kThreads) void sepconv_generic_kernel(
    SepConv pr, const T *__restrict__ f, const T *__restrict__ g,
    const T *__restrict__ bias, T *__restrict__ h) {
  const i64 nhx = pr.x.nh, nhy = pr.y.nh;
  const i64 nfx = pr.x.nf, nfy = pr.y.nf, ngy = pr.y.ng;
  const i64 total = pr.batch * pr.c_out * nhx * nhy;
  const i64 step = (i64)gridDim.x * blockDim.x;
  for (i64 i = (i64)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
    const i64 hy = i % nhy;
    i64 r = i / nhy;
    const i64 hx = r % nhx;
    r /= nhx;
    const i64 m = r % pr.c_out, n = r / pr.c_out;
    T *out = h + n * pr.h_n + m * pr.h_m + hx * nhy + hy;
    const bool live = hx < pr.x.nh_eff && hy < pr.y.nh_eff;
    T acc = 0;
    if (live) {
      const T *fm = f + m * pr.f_m;
      const T *gn = g + n * pr.g_n;
      for (i64 fx = 0; fx < nfx; ++fx) {
        const i64 gx = tap_index(pr.x.kind, hx, fx, pr.x.ng, pr.x.s, pr.x.d, pr.x.p, pr.x.u);
        if (gx < 0) continue;
        for (i64 fy = 0; fy < nfy; ++fy) {
          const i64 gy = tap_index(pr.y.kind, hy, fy, ngy, pr.y.s, pr.y.d, pr.y.p, pr.y.u);
          if (gy < 0) continue;
          const T *fp = fm + fx * nfy + fy;
          const T *gp = gn + gx * ngy + gy;
          for (i64 c = 0; c < pr.c_in; ++c) acc += fp[c * pr.f_c] * gp[c * pr.g_c];
        }
      }
    }
    if (pr.accumulate) {
      if (live) *out += acc;
    } else {
      const T v = (bias ? bias[m] : T(0)) + acc;
      *out = (pr.relu && v < T(0)) ? T(0) : v;
    }
  }
}

// w[m, c, fx, fy] = sum over (n, hx, hy) in a fixed order: each thread sums a
// strided subsequence, then a binary tree in LDS combines the 256 partials.
template <typename T>
__global__ __launch_bounds__(kThreads) void sepreduce_generic_kernel(
    SepReduce pr, const T *__restrict__ a, const T *__restrict__ g, T *__restrict__ w) {
  __shared__ T part[kThreads];
  const i64 nfx = pr.x.nf, nfy = pr.y.nf;
  const i64 nhx = pr.x.nh, nhy = pr.y.nh, ngx = pr.x.ng, ngy = pr.y.ng;
  const i64 ex = pr.x.nh_eff, ey = pr.y.nh_eff;
  const i64 nout = pr.c_out * pr.c_in * nfx * nfy;
  for (i64 o = blockIdx.x; o < nout; o += gridDim.x) {
    const i64 fy = o % nfy;
    i64 r = o / nfy;
    const i64 fx = r % nfx;
    r /= nfx;
    const i64 c = r % pr.c_in, m = r / pr.c_in;
    T acc = 0;
    const i64 terms = pr.batch * ex * ey;
    for (i64 j = threadIdx.x; j < terms; j += kThreads) {
      const i64 hy = j % ey;
      i64 q = j / ey;
      const i64 hx = q % ex, n = q / ex;
      const i64 gx = tap_index(pr.x.kind, hx, fx, ngx, pr.x.s, pr.x.d, pr.x.p, pr.x.u);
      const i64 gy = tap_index(pr.y.kind, hy, fy, ngy, pr.y.s, pr.y.d, pr.y.p, pr.y.u);
      if (gx < 0 || gy < 0) continue;
      acc += a[((n * pr.c_out + m) * nhx + hx) * nhy + hy] *
             g[((n * pr.c_in + c) * ngx + gx) * ngy + gy];
    }
    part[threadIdx.x] = acc;
    __syncthreads();
    for (int width = kThreads / 2; width > 0; width >>= 1) {
      if ((int)threadIdx.x < width) part[threadIdx.x] += part[threadIdx.x + width];
      __syncthreads();
    }
    if (threadIdx.x == 0) w[o] = part[0];
    __syncthreads();
  }
}

inline unsigned grid_for(i64 items, i64 per_block) {
  i64 blocks = (items + per_block - 1) / per_block;
  const i64 cap = 1 << 20;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

}  // namespace

template <typename T>
hipError_t launch_sepconv_generic(const SepConv &pr, const T *f, const T *g,
                                  const T *bias, T *h, hipStream_t stream) {
  const i64 total = pr.batch * pr.c_out * pr.x.nh * pr.y.nh;
  if (total == 0) return hipSuccess;
  hipLaunchKernelGGL(sepconv_generic_kernel<T>, dim3(grid_for(total, kThreads)),
                     dim3(kThreads), 0, stream, pr, f, g, bias, h);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_sepreduce_generic(const SepReduce &pr, const T *a, const T *g,
                                    T *w, hipStream_t stream) {
  const i64 nout = pr.c_out * pr.c_in * pr.x.nf * pr.y.nf;
  if (nout == 0) return hipSuccess;
  hipLaunchKernelGGL(sepreduce_generic_kernel<T>, dim3(grid_for(nout, 1)),
                     dim3(kThreads), 0, stream, pr, a, g, w);
  return hipGetLastError();
}

template hipError_t launch_sepconv_generic<float>(const SepConv &, const float *,
    const float *, const float *, float *, hipStream_t);
template hipError_t launch_sepconv_generic<double>(const SepConv &, const double *,
    const double *, const double *, double *, hipStream_t);
template hipError_t launch_sepreduce_generic<float>(const SepReduce &, const float *,
    const float *, float *, hipStream_t);
template hipError_t launch_sepreduce_generic<double>(const SepReduce &, const double *,
    const double *, double *, hipStream_t);

}  // namespace mellin
