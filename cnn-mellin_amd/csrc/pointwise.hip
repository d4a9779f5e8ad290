// The two pointwise layers that sit in front of the first convolution of the
// reference's acoustic model (models.py:414-417), fused into one pass each way:
//
//   log compression   y = log(eps + |x|)                 (layers.py:79-101)
//   dilation lift     y[.., t, ..] = (t + 1)^tau * x     (layers.py:8-21)
//   both              y = (t + 1)^tau * log(eps + |x|)
//
// x is dense, viewed as (outer, T, inner) with the lifted axis in the middle.
// PyTorch runs the pair as six elementwise launches forward (abs, add, log,
// arange/pow, mul, reshape copy) and more backward; here the forward reads x and
// writes y once, and the backward reads x and grad_y once, writes grad_x once and
// leaves the two parameter gradients as per-block partial sums that a second
// small kernel adds up in index order (bit-reproducible, no float atomics).
//
// A thread owns one (t, inner) column of the (T, inner) plane and walks down the
// outer axis: the power (t + 1)^tau, the only expensive function, is evaluated
// once per thread, and consecutive threads touch consecutive words.
#include "mellin_common.hpp"

namespace mellin {

namespace {

constexpr int kPwThreads = 256;

template <typename T> __device__ __forceinline__ T sign_of(T v) { return v > T(0) ? T(1) : (v < T(0) ? T(-1) : T(0)); }

template <typename T, bool LOG, bool LIFT>
__global__ __launch_bounds__(kPwThreads) void log_lift_forward_kernel(
    const T *__restrict__ x, T eps, T tau, const T *__restrict__ params, i64 outer, i64 plane, i64 inner,
    i64 rows_per_block, T *__restrict__ y) {
  const i64 col = (i64)blockIdx.x * kPwThreads + threadIdx.x;      // t * inner + i
  if (col >= plane) return;
  if (params) { eps = params[0]; tau = params[1]; }               // the values live on the device
  T p = T(1);
  if (LIFT) p = pow((T)(col / inner + 1), tau);
  const i64 n0 = (i64)blockIdx.y * rows_per_block, n1 = min(outer, n0 + rows_per_block);
  for (i64 n = n0; n < n1; ++n) {
    const T v = x[n * plane + col];
    const T l = LOG ? log(eps + fabs(v)) : v;
    y[n * plane + col] = LIFT ? p * l : l;
  }
}

// grad_x, and partial sums of d/d eps and d/d tau per block (two values per block)
template <typename T, bool LOG, bool LIFT>
__global__ __launch_bounds__(kPwThreads) void log_lift_backward_kernel(
    const T *__restrict__ x, const T *__restrict__ gy, T eps, T tau, const T *__restrict__ params, i64 outer,
    i64 plane, i64 inner, i64 rows_per_block, T *__restrict__ gx, T *__restrict__ partial) {
  __shared__ T red[2][kPwThreads / 64];
  if (params) { eps = params[0]; tau = params[1]; }
  const i64 col = (i64)blockIdx.x * kPwThreads + threadIdx.x;
  T s_eps = T(0), s_tau = T(0);
  if (col < plane) {
    T p = T(1), lnt = T(0);
    if (LIFT) {
      const T t1 = (T)(col / inner + 1);
      p = pow(t1, tau);
      lnt = log(t1);
    }
    const i64 n0 = (i64)blockIdx.y * rows_per_block, n1 = min(outer, n0 + rows_per_block);
    for (i64 n = n0; n < n1; ++n) {
      const T v = x[n * plane + col], g = gy[n * plane + col];
      const T gp = g * p;                                  // gradient reaching the logarithm
      if (LOG) {
        const T a = eps + fabs(v);
        const T inv = gp / a;
        gx[n * plane + col] = inv * sign_of(v);
        s_eps += inv;
        if (LIFT) s_tau += gp * lnt * log(a);
      } else {
        gx[n * plane + col] = gp;
        s_tau += gp * lnt * v;
      }
    }
  }
  // wave sums by shuffles (fixed tree), then the block's wavefronts in order
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    s_eps += __shfl_down(s_eps, o);
    s_tau += __shfl_down(s_tau, o);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { red[0][wave] = s_eps; red[1][wave] = s_tau; }
  __syncthreads();
  if (threadIdx.x == 0) {
    T a = T(0), b = T(0);
    for (int w = 0; w < kPwThreads / 64; ++w) { a += red[0][w]; b += red[1][w]; }
    const i64 blk = (i64)blockIdx.y * gridDim.x + blockIdx.x;
    partial[2 * blk] = a;
    partial[2 * blk + 1] = b;
  }
}

// grad_params[0 .. 1] = sums of the partials, in index order (one wavefront:
// lane l adds partials l, l + 64, ..., then a fixed shuffle tree)
template <typename T>
__global__ __launch_bounds__(64) void log_lift_reduce_kernel(const T *__restrict__ partial, i64 blocks,
                                                             T *__restrict__ grad_params) {
  T a = T(0), b = T(0);
  for (i64 i = threadIdx.x; i < blocks; i += 64) { a += partial[2 * i]; b += partial[2 * i + 1]; }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    a += __shfl_down(a, o);
    b += __shfl_down(b, o);
  }
  if (threadIdx.x == 0) { grad_params[0] = a; grad_params[1] = b; }
}

// Blocks along the outer axis: enough workgroups to fill the chip several times
// over, but rows_per_block >= 4 so that the power is amortised.
void shape_grid(i64 outer, i64 plane, dim3 &grid, i64 &rows_per_block) {
  const i64 gx = (plane + kPwThreads - 1) / kPwThreads;
  i64 gy = std::max<i64>(1, std::min<i64>((4096 + gx - 1) / gx, (outer + 3) / 4));
  gy = std::min<i64>(gy, 65535);
  rows_per_block = (outer + gy - 1) / gy;
  gy = (outer + rows_per_block - 1) / rows_per_block;
  grid = dim3((unsigned)gx, (unsigned)gy);
}

}  // namespace

size_t log_lift_workspace_bytes(i64 outer, i64 t, i64 inner, size_t elem) {
  if (outer <= 0 || t <= 0 || inner <= 0) return 0;
  dim3 grid;
  i64 rpb;
  shape_grid(outer, t * inner, grid, rpb);
  return (size_t)grid.x * grid.y * 2 * elem;
}

template <typename T>
hipError_t launch_log_lift_forward(const T *x, T eps, T tau, bool with_log, bool with_lift, i64 outer, i64 t,
                                   i64 inner, T *y, hipStream_t stream, const T *params) {
  if (outer <= 0 || t <= 0 || inner <= 0) return hipSuccess;
  dim3 grid;
  i64 rpb;
  shape_grid(outer, t * inner, grid, rpb);
#define MELLIN_PW_FWD(L_, F_)                                                                    \
  hipLaunchKernelGGL((log_lift_forward_kernel<T, L_, F_>), grid, dim3(kPwThreads), 0, stream, x, \
                     eps, tau, params, outer, t * inner, inner, rpb, y)
  if (with_log && with_lift) MELLIN_PW_FWD(true, true);
  else if (with_log) MELLIN_PW_FWD(true, false);
  else MELLIN_PW_FWD(false, true);
#undef MELLIN_PW_FWD
  return hipGetLastError();
}

template <typename T>
hipError_t launch_log_lift_backward(const T *x, const T *gy, T eps, T tau, bool with_log, bool with_lift,
                                    i64 outer, i64 t, i64 inner, T *gx, T *grad_params, T *workspace,
                                    hipStream_t stream, const T *params) {
  if (outer <= 0 || t <= 0 || inner <= 0) {
    hipLaunchKernelGGL((log_lift_reduce_kernel<T>), dim3(1), dim3(64), 0, stream, workspace, (i64)0, grad_params);
    return hipGetLastError();
  }
  dim3 grid;
  i64 rpb;
  shape_grid(outer, t * inner, grid, rpb);
#define MELLIN_PW_BWD(L_, F_)                                                                     \
  hipLaunchKernelGGL((log_lift_backward_kernel<T, L_, F_>), grid, dim3(kPwThreads), 0, stream, x, \
                     gy, eps, tau, params, outer, t * inner, inner, rpb, gx, workspace)
  if (with_log && with_lift) MELLIN_PW_BWD(true, true);
  else if (with_log) MELLIN_PW_BWD(true, false);
  else MELLIN_PW_BWD(false, true);
#undef MELLIN_PW_BWD
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((log_lift_reduce_kernel<T>), dim3(1), dim3(64), 0, stream, workspace,
                     (i64)grid.x * grid.y, grad_params);
  return hipGetLastError();
}

// ---- bias gradient, with the backward of a fused ReLU ---------------------------------
// grad_bias[c] = sum over images and positions of g[n, c, :], where g = grad_out or, when
// the layer's ReLU was applied by the forward kernel, grad_out where out > 0 and zero
// elsewhere (g is then also written: it is what the gradient kernels take).  One pass over
// the operands; sums in a fixed order: a block adds up 4096 consecutive elements of one
// (image, channel) plane (lanes strided, a shuffle tree per wavefront, the wavefronts in
// order), a second kernel adds a channel's blocks in index order.
namespace {

constexpr int kBiasChunk = 4096;

// T: float, or _Float16 (sums in fp32 either way)
template <bool MASK, typename T>
__global__ __launch_bounds__(kPwThreads) void bias_grad_kernel(const T *__restrict__ go,
                                                               const T *__restrict__ out,
                                                               T *__restrict__ gm, float *__restrict__ partial,
                                                               i64 plane, int chunks) {
  __shared__ float red[kPwThreads / 64];
  const int chunk = blockIdx.x, c = blockIdx.y, n = blockIdx.z, C = gridDim.y, N = gridDim.z;
  const i64 base = ((i64)n * C + c) * plane + (i64)chunk * kBiasChunk;
  const int len = (int)min((i64)kBiasChunk, plane - (i64)chunk * kBiasChunk);
  float s = 0.f;
#pragma unroll 4
  for (int i = threadIdx.x; i < len; i += kPwThreads) {
    T v = go[base + i];
    if (MASK) {
      v = out[base + i] > (T)0 ? v : (T)0;
      gm[base + i] = v;
    }
    s += (float)v;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_down(s, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float a = 0.f;
    for (int w = 0; w < kPwThreads / 64; ++w) a += red[w];
    partial[((i64)c * N + n) * chunks + chunk] = a;
  }
}

template <typename T>                                  // T: type of the result (rounded once)
__global__ __launch_bounds__(64) void bias_reduce_kernel(const float *__restrict__ partial, i64 per_channel,
                                                         T *__restrict__ grad_bias) {
  const float *p = partial + (i64)blockIdx.x * per_channel;
  float a = 0.f;
  for (i64 i = threadIdx.x; i < per_channel; i += 64) a += p[i];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) a += __shfl_down(a, o);
  if (threadIdx.x == 0) grad_bias[blockIdx.x] = (T)a;
}

}  // namespace

size_t bias_grad_workspace_bytes(i64 batch, i64 channels, i64 plane) {
  if (batch <= 0 || channels <= 0 || plane <= 0) return 0;
  const i64 chunks = (plane + kBiasChunk - 1) / kBiasChunk;
  return (size_t)(batch * channels * chunks) * sizeof(float);
}

template <typename T>
hipError_t launch_bias_grad(const T *grad_out, const T *out, i64 batch, i64 channels, i64 plane,
                            T *grad_masked, T *grad_bias, float *workspace, hipStream_t stream) {
  if (channels <= 0) return hipSuccess;
  if (batch <= 0 || plane <= 0) {                       // empty sums
    hipLaunchKernelGGL(bias_reduce_kernel<T>, dim3((unsigned)channels), dim3(64), 0, stream, workspace, (i64)0,
                       grad_bias);
    return hipGetLastError();
  }
  const i64 chunks = (plane + kBiasChunk - 1) / kBiasChunk;
  const dim3 grid((unsigned)chunks, (unsigned)channels, (unsigned)batch);
  if (out)
    hipLaunchKernelGGL((bias_grad_kernel<true, T>), grid, dim3(kPwThreads), 0, stream, grad_out, out, grad_masked,
                       workspace, plane, (int)chunks);
  else
    hipLaunchKernelGGL((bias_grad_kernel<false, T>), grid, dim3(kPwThreads), 0, stream, grad_out, out, grad_masked,
                       workspace, plane, (int)chunks);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(bias_reduce_kernel<T>, dim3((unsigned)channels), dim3(64), 0, stream, workspace, batch * chunks,
                     grad_bias);
  return hipGetLastError();
}
template hipError_t launch_bias_grad<float>(const float *, const float *, i64, i64, i64, float *, float *, float *,
                                            hipStream_t);
template hipError_t launch_bias_grad<_Float16>(const _Float16 *, const _Float16 *, i64, i64, i64, _Float16 *,
                                               _Float16 *, float *, hipStream_t);

// ---- max over pairs of neighbours along the last axis (frequency pooling, window 2) -----
// y[r, j] = max(x[r, 2 j], x[r, 2 j + 1]) for x (rows, f), j < f / 2 (an odd last column is
// dropped), as max_pool2d(x, (1, 2)) does; `which` keeps one byte per output: 1 when the
// second of the pair was taken (strictly greater, or NaN), so that the backward pass
// needs neither x nor 8-byte indices.
namespace {

// I: index type (unsigned 32-bit when rows * f fits: a 64-bit division per element costs more
// than the memory traffic)
template <typename I, typename T>
__global__ __launch_bounds__(kPwThreads) void pool_pairs_forward_kernel(const T *__restrict__ x, I rows, I f,
                                                                        I fo, T *__restrict__ y,
                                                                        unsigned char *__restrict__ which) {
  const I total = rows * fo;
  for (I i = (I)blockIdx.x * kPwThreads + threadIdx.x; i < total; i += (I)gridDim.x * kPwThreads) {
    const I r = i / fo, j = i - r * fo;
    const T a = x[r * f + 2 * j], b = x[r * f + 2 * j + 1];
    const bool second = b > a || b != b;
    y[i] = second ? b : a;
    which[i] = second ? 1 : 0;
  }
}

template <typename T>
__global__ __launch_bounds__(kPwThreads) void zero_words_kernel(T *__restrict__ p, i64 n) {
  for (i64 i = (i64)blockIdx.x * kPwThreads + threadIdx.x; i < n; i += (i64)gridDim.x * kPwThreads) p[i] = (T)0;
}

// one thread per pair: both words of the pair, and the odd last column with the row's last pair
template <typename I, typename T>
__global__ __launch_bounds__(kPwThreads) void pool_pairs_backward_kernel(const T *__restrict__ gy,
                                                                         const unsigned char *__restrict__ which,
                                                                         I rows, I f, I fo,
                                                                         T *__restrict__ gx) {
  const I total = rows * fo;
  for (I i = (I)blockIdx.x * kPwThreads + threadIdx.x; i < total; i += (I)gridDim.x * kPwThreads) {
    const I r = i / fo, j = i - r * fo;
    const T g = gy[i];
    const bool second = which[i] != 0;
    T *o = gx + r * f + 2 * j;
    o[0] = second ? (T)0 : g;
    o[1] = second ? g : (T)0;
    if (j == fo - 1 && (f & 1)) o[2] = (T)0;
  }
}

}  // namespace

template <typename T>
hipError_t launch_pool_pairs_forward(const T *x, i64 rows, i64 f, T *y, unsigned char *which,
                                     hipStream_t stream) {
  const i64 fo = f / 2;
  if (rows <= 0 || fo <= 0) return hipSuccess;
  const i64 blocks = std::min<i64>((rows * fo + kPwThreads - 1) / kPwThreads, 1 << 20);
  if (rows * f < ((i64)1 << 31))
    hipLaunchKernelGGL((pool_pairs_forward_kernel<unsigned, T>), dim3((unsigned)blocks), dim3(kPwThreads), 0, stream, x,
                       (unsigned)rows, (unsigned)f, (unsigned)fo, y, which);
  else
    hipLaunchKernelGGL((pool_pairs_forward_kernel<i64, T>), dim3((unsigned)blocks), dim3(kPwThreads), 0, stream, x, rows,
                       f, fo, y, which);
  return hipGetLastError();
}

template hipError_t launch_pool_pairs_forward<float>(const float *, i64, i64, float *, unsigned char *, hipStream_t);
template hipError_t launch_pool_pairs_forward<_Float16>(const _Float16 *, i64, i64, _Float16 *, unsigned char *,
                                                        hipStream_t);

template <typename T>
hipError_t launch_pool_pairs_backward(const T *gy, const unsigned char *which, i64 rows, i64 f, T *gx,
                                      hipStream_t stream) {
  if (rows <= 0 || f <= 0) return hipSuccess;
  const i64 fo = f / 2;
  if (fo == 0) {                                        // one column: nothing was pooled (a kernel, not a memset
    // node: the call may be recorded into a graph)
    hipLaunchKernelGGL(zero_words_kernel<T>, dim3((unsigned)std::min<i64>((rows + kPwThreads - 1) / kPwThreads, 4096)),
                       dim3(kPwThreads), 0, stream, gx, rows);
    return hipGetLastError();
  }
  const i64 blocks = std::min<i64>((rows * fo + kPwThreads - 1) / kPwThreads, 1 << 20);
  if (rows * f < ((i64)1 << 31))
    hipLaunchKernelGGL((pool_pairs_backward_kernel<unsigned, T>), dim3((unsigned)blocks), dim3(kPwThreads), 0, stream, gy,
                       which, (unsigned)rows, (unsigned)f, (unsigned)fo, gx);
  else
    hipLaunchKernelGGL((pool_pairs_backward_kernel<i64, T>), dim3((unsigned)blocks), dim3(kPwThreads), 0, stream, gy,
                       which, rows, f, fo, gx);
  return hipGetLastError();
}
template hipError_t launch_pool_pairs_backward<float>(const float *, const unsigned char *, i64, i64, float *,
                                                      hipStream_t);
template hipError_t launch_pool_pairs_backward<_Float16>(const _Float16 *, const unsigned char *, i64, i64,
                                                         _Float16 *, hipStream_t);

// ---- half <-> float copies (the half-precision entry points compute in fp32) ------
namespace {

// eight elements per thread where the run and the pointers (vec) allow 16-byte accesses,
// singly otherwise
__global__ __launch_bounds__(kPwThreads) void half_to_float_kernel(const _Float16 *__restrict__ src,
                                                                   float *__restrict__ dst, i64 n, bool vec) {
  const i64 i0 = ((i64)blockIdx.x * kPwThreads + threadIdx.x) * 8;
  if (vec && i0 + 8 <= n) {
    typedef _Float16 half8 __attribute__((ext_vector_type(8)));
    const half8 v = *(const half8 *)(src + i0);
    float4 a = make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
    float4 b = make_float4((float)v[4], (float)v[5], (float)v[6], (float)v[7]);
    *(float4 *)(dst + i0) = a;
    *(float4 *)(dst + i0 + 4) = b;
  } else {
    for (i64 i = i0; i < min(i0 + 8, n); ++i) dst[i] = (float)src[i];
  }
}

__global__ __launch_bounds__(kPwThreads) void float_to_half_kernel(const float *__restrict__ src,
                                                                   _Float16 *__restrict__ dst, i64 n, bool vec) {
  const i64 i0 = ((i64)blockIdx.x * kPwThreads + threadIdx.x) * 8;
  if (vec && i0 + 8 <= n) {
    typedef _Float16 half8 __attribute__((ext_vector_type(8)));
    const float4 a = *(const float4 *)(src + i0), b = *(const float4 *)(src + i0 + 4);
    half8 v;
    v[0] = (_Float16)a.x; v[1] = (_Float16)a.y; v[2] = (_Float16)a.z; v[3] = (_Float16)a.w;
    v[4] = (_Float16)b.x; v[5] = (_Float16)b.y; v[6] = (_Float16)b.z; v[7] = (_Float16)b.w;
    *(half8 *)(dst + i0) = v;
  } else {
    for (i64 i = i0; i < min(i0 + 8, n); ++i) dst[i] = (_Float16)src[i];
  }
}

}  // namespace

// 16-byte accesses when both pointers are 16-byte aligned (torch allocations and the
// workspace regions are; a view into a half tensor may start at any even address)
hipError_t launch_half_to_float(const void *src, float *dst, i64 n, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  const i64 blocks = (n + 8 * kPwThreads - 1) / (8 * kPwThreads);
  const bool vec = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
  hipLaunchKernelGGL(half_to_float_kernel, dim3((unsigned)blocks), dim3(kPwThreads), 0, stream,
                     (const _Float16 *)src, dst, n, vec);
  return hipGetLastError();
}

hipError_t launch_float_to_half(const float *src, void *dst, i64 n, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  const i64 blocks = (n + 8 * kPwThreads - 1) / (8 * kPwThreads);
  const bool vec = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
  hipLaunchKernelGGL(float_to_half_kernel, dim3((unsigned)blocks), dim3(kPwThreads), 0, stream, src,
                     (_Float16 *)dst, n, vec);
  return hipGetLastError();
}

template hipError_t launch_log_lift_forward<float>(const float *, float, float, bool, bool, i64, i64, i64,
                                                   float *, hipStream_t, const float *);
template hipError_t launch_log_lift_forward<double>(const double *, double, double, bool, bool, i64, i64, i64,
                                                    double *, hipStream_t, const double *);
template hipError_t launch_log_lift_backward<float>(const float *, const float *, float, float, bool, bool, i64,
                                                    i64, i64, float *, float *, float *, hipStream_t, const float *);
template hipError_t launch_log_lift_backward<double>(const double *, const double *, double, double, bool, bool,
                                                     i64, i64, i64, double *, double *, double *, hipStream_t,
                                                     const double *);

}  // namespace mellin
