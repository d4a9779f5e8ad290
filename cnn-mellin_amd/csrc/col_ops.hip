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
// (fx, fy): a fixed order, no atomics.  Both are pure data movement (HBM bound).
//
// The *_plane kernels are the ones that run unless an extent is out of their
// 32-bit range: a thread owns one position of the (x, y) plane, works out its taps
// once (float-reciprocal index splits, no integer division) and then walks over
// the (image, channel) pairs, so the index arithmetic is amortised and consecutive
// threads touch consecutive words.  The generic kernels (one thread per element,
// 64-bit arithmetic throughout) remain for everything else.
#include <algorithm>

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

// O: the type g is stored in (sums are formed in T)
template <typename T, typename O = T>
__global__ __launch_bounds__(256) void col2spec_kernel(const T *__restrict__ gg, O *__restrict__ g,
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
    g[i] = (O)acc;
  }
}

// gg[nc, tap, q] = g[nc', tap source of q] for q in the (x.nh, y.nh) plane
template <typename T>
__global__ __launch_bounds__(256) void spec2col_plane_kernel(const T *__restrict__ g, T *__restrict__ gg,
                                                             Axis x, Axis y, int c_in, int batch,
                                                             int transposed_g, int transposed_gg) {
  const int plane = (int)(x.nh * y.nh), ng = (int)(x.ng * y.ng), nfy = (int)y.nf;
  // Workgroups are dealt to the eight dies in turn, each with an L2 of its own: renumber them so
  // that a die writes one contiguous run of gg, and the cache lines that neighbouring blocks
  // each write a part of are completed in one L2.
  const unsigned per_z = gridDim.x * gridDim.y, total = per_z * gridDim.z;
  const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const unsigned die = lin & 7u, mine = die * (total >> 3) + min(die, total & 7u) + (lin >> 3);
  const unsigned block_z = mine / per_z, in_z = mine - block_z * per_z;
  const unsigned block_y = in_z / gridDim.x, block_x = in_z - block_y * gridDim.x;
  const int q = (int)block_x * 256 + threadIdx.x;
  if (q >= plane) return;
  const int tap = (int)block_y, fx = tap / nfy, fy = tap - fx * nfy;
  int ox = (int)((float)q * (1.0f / (float)y.nh));
  int oy = q - ox * (int)y.nh;
  if (oy < 0) { --ox; oy += (int)y.nh; } else if (oy >= (int)y.nh) { ++ox; oy -= (int)y.nh; }
  const int gx = tap32(x.kind, ox, fx, (int)x.ng, (int)x.s, (int)x.d, (int)x.p, (int)x.u);
  const int gy = tap32(y.kind, oy, fy, (int)y.ng, (int)y.s, (int)y.d, (int)y.p, (int)y.u);
  const int src = (gx >= 0 && gy >= 0) ? gx * (int)y.ng + gy : -1;
  const int taps = (int)(x.nf * y.nf), pairs = batch * c_in;
#pragma unroll 4
  for (int nc = (int)block_z; nc < pairs; nc += gridDim.z) {     // nc: (image, channel) in gg's own order
    int nc_g = nc;
    if (transposed_g != transposed_gg) {
      const int a = transposed_gg ? nc / batch : nc / c_in;       // ci : bt
      const int b = transposed_gg ? nc - a * batch : nc - a * c_in;
      nc_g = transposed_gg ? b * c_in + a : b * batch + a;
    }
    const T v = src >= 0 ? g[(i64)nc_g * ng + src] : T(0);
    gg[((i64)nc * taps + tap) * plane + q] = v;
  }
}

// g[nc', q] = sum over taps of gg[nc, tap, source of q] for q in the (x.nh, y.nh) signal plane;
// eight (image, channel) pairs per thread share the tap arithmetic.  The y taps are worked out
// once per thread; for a filter row with a tap, the loads of four filter columns of all eight
// pairs are requested before the first is summed (positions without a tap read a word that is
// there and add zero), so a thread waits for memory once per filter row, not once per tap.
template <typename T, typename O = T>
__global__ __launch_bounds__(256) void col2spec_plane_kernel(const T *__restrict__ gg, O *__restrict__ g,
                                                             Axis x, Axis y, int c_in, int batch,
                                                             int transposed_g, int transposed_gg,
                                                             i64 per_pair) {   // words from one pair's columns to the next
  constexpr int NB = 8, FY = 4;
  const int plane = (int)(x.nh * y.nh), nfx = (int)x.nf, nfy = (int)y.nf;
  // Workgroups are dealt to the eight dies in turn, each with an L2 of its own: renumber them so
  // that a die takes one contiguous run of (pair group, 256-position block), whose neighbouring
  // rows of gg share cache lines.
  const unsigned total = gridDim.x * gridDim.z, lin = blockIdx.x + gridDim.x * blockIdx.z;
  const unsigned die = lin & 7u, slot = lin >> 3;
  const unsigned mine = die * (total >> 3) + min(die, total & 7u) + slot;
  const unsigned block_z = mine / gridDim.x, block_x = mine - block_z * gridDim.x;
  const int q = (int)block_x * 256 + threadIdx.x;
  if (q >= plane) return;
  int gx = (int)((float)q * (1.0f / (float)y.nh));
  int gy = q - gx * (int)y.nh;
  if (gy < 0) { --gx; gy += (int)y.nh; } else if (gy >= (int)y.nh) { ++gx; gy -= (int)y.nh; }
  auto y_taps = [&](int fy0, int (&oy)[FY]) {
#pragma unroll
    for (int j = 0; j < FY; ++j)
      oy[j] = fy0 + j < nfy ? tap32(y.kind, gy, fy0 + j, (int)y.ng, (int)y.s, (int)y.d, (int)y.p, (int)y.u) : -1;
  };
  int oy_first[FY];
  y_taps(0, oy_first);
  const int pairs = batch * c_in;
  for (int nc0 = (int)block_z * NB; nc0 < pairs; nc0 += gridDim.z * NB) {   // nc: pairs in g's own order
    const T *src[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      int nc = min(nc0 + b, pairs - 1), nc_gg = nc;
      if (transposed_g != transposed_gg) {
        const int a = transposed_g ? nc / batch : nc / c_in;
        const int r = transposed_g ? nc - a * batch : nc - a * c_in;
        nc_gg = transposed_g ? r * c_in + a : r * batch + a;
      }
      src[b] = gg + (i64)nc_gg * per_pair;
    }
    T acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b] = T(0);
    if (nfy == 1 && nfx <= 8) {
      // one column per filter row (the fold over x alone): the taps of all filter rows are
      // worked out first, then every load is requested (a row without a tap re-reads the
      // pair's first word and adds a zero), then the sums are formed in filter-row order --
      // one wait for memory instead of one per filter row
      int off[8];
#pragma unroll
      for (int fx = 0; fx < 8; ++fx) {
        const int ox = fx < nfx ? tap32(x.kind, gx, fx, (int)x.ng, (int)x.s, (int)x.d, (int)x.p, (int)x.u) : -1;
        off[fx] = (ox >= 0 && oy_first[0] >= 0) ? (fx * (int)x.ng + ox) * (int)y.ng + oy_first[0] : -1;
      }
      T v[8][NB];
#pragma unroll
      for (int fx = 0; fx < 8; ++fx)
#pragma unroll
        for (int b = 0; b < NB; ++b) v[fx][b] = src[b][max(off[fx], 0)];
#pragma unroll
      for (int fx = 0; fx < 8; ++fx)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b] += off[fx] >= 0 ? v[fx][b] : T(0);
    } else
    for (int fx = 0; fx < nfx; ++fx) {
      const int ox = tap32(x.kind, gx, fx, (int)x.ng, (int)x.s, (int)x.d, (int)x.p, (int)x.u);
      if (ox < 0) continue;
      for (int fy0 = 0; fy0 < nfy; fy0 += FY) {
        int oy[FY];
        if (fy0 == 0) {
#pragma unroll
          for (int j = 0; j < FY; ++j) oy[j] = oy_first[j];
        } else {
          y_taps(fy0, oy);
        }
        T v[FY][NB];
#pragma unroll
        for (int j = 0; j < FY; ++j) {
          const int fy = min(fy0 + j, nfy - 1);
          const int off = ((fx * nfy + fy) * (int)x.ng + ox) * (int)y.ng + max(oy[j], 0);
#pragma unroll
          for (int b = 0; b < NB; ++b) v[j][b] = src[b][off];
        }
#pragma unroll
        for (int j = 0; j < FY; ++j)
#pragma unroll
          for (int b = 0; b < NB; ++b) acc[b] += oy[j] >= 0 ? v[j][b] : T(0);
      }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
      if (nc0 + b < pairs) g[(i64)(nc0 + b) * plane + q] = (O)acc[b];
  }
}

// the plane kernels' range: tap numerators and plane sizes within the float-reciprocal
// splits, per-pair extents within 32 bits
bool fits_plane_kernels(const Axis &x, const Axis &y, i64 c_in, i64 batch, i64 plane, i64 per_pair) {
  return axis_fits_tap32(x) && axis_fits_tap32(y) && plane < ((i64)1 << 22) && per_pair < ((i64)1 << 31) &&
         batch * c_in < ((i64)1 << 30) && x.nf * y.nf <= 65535 && x.ng * y.ng < ((i64)1 << 31);
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
  const i64 plane = x.nh * y.nh;
  if (fits_plane_kernels(x, y, c_in, batch, plane, x.nf * y.nf * plane)) {
    // enough workgroups to fill the chip, few enough that a thread's tap arithmetic is reused
    const i64 gx = (plane + 255) / 256, gy = x.nf * y.nf;
    const i64 gz = std::max<i64>(1, std::min<i64>(batch * c_in, std::min<i64>(65535, (8192 + gx * gy - 1) / (gx * gy))));
    hipLaunchKernelGGL(spec2col_plane_kernel<T>, dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), dim3(256), 0,
                       stream, g, gg, x, y, (int)c_in, (int)batch, transposed_g, transposed_gg);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(spec2col_kernel<T>, dim3(blocks_for(total)), dim3(256), 0, stream, g, gg, x, y, c_in,
                     batch, transposed_g, transposed_gg);
  return hipGetLastError();
}

template <typename T, typename O>
hipError_t launch_col2spec(const Axis &x, const Axis &y, i64 c_in, i64 batch, int transposed_g,
                           int transposed_gg, const T *gg, O *g, hipStream_t stream) {
  const i64 total = batch * c_in * x.nh * y.nh;
  if (total == 0) return hipSuccess;
  const i64 plane = x.nh * y.nh;
  if (fits_plane_kernels(x, y, c_in, batch, plane, x.nf * y.nf * x.ng * y.ng)) {
    const i64 gx = (plane + 255) / 256, groups = (batch * c_in + 7) / 8;
    const i64 gz = std::max<i64>(1, std::min<i64>(groups, std::min<i64>(65535, (8192 + gx - 1) / gx)));
    hipLaunchKernelGGL((col2spec_plane_kernel<T, O>), dim3((unsigned)gx, 1, (unsigned)gz), dim3(256), 0, stream, gg,
                       g, x, y, (int)c_in, (int)batch, transposed_g, transposed_gg, x.nf * y.nf * x.ng * y.ng);
    return hipGetLastError();
  }
  hipLaunchKernelGGL((col2spec_kernel<T, O>), dim3(blocks_for(total)), dim3(256), 0, stream, gg, g, x, y, c_in,
                     batch, transposed_g, transposed_gg);
  return hipGetLastError();
}

// The same adjoint over columns whose tap planes are padded to `taps_padded` per pair
// (the tap products of the input gradient); false if the plane kernel's range is exceeded.
bool launch_col2spec_padded(const Axis &x, const Axis &y, i64 pairs, i64 taps_padded, const float *gg,
                            float *g, hipStream_t stream, hipError_t *err) {
  const i64 plane = x.nh * y.nh, per_pair = taps_padded * x.ng * y.ng;
  if (!fits_plane_kernels(x, y, pairs, 1, plane, per_pair)) return false;
  const i64 gx = (plane + 255) / 256, groups = (pairs + 7) / 8;
  const i64 gz = std::max<i64>(1, std::min<i64>(groups, std::min<i64>(65535, (8192 + gx - 1) / gx)));
  hipLaunchKernelGGL(col2spec_plane_kernel<float>, dim3((unsigned)gx, 1, (unsigned)gz), dim3(256), 0, stream, gg,
                     g, x, y, (int)pairs, 1, 0, 0, per_pair);
  *err = hipGetLastError();
  return true;
}

template hipError_t launch_spec2col<float>(const Axis &, const Axis &, i64, i64, int, int, const float *,
                                           float *, hipStream_t);
template hipError_t launch_spec2col<double>(const Axis &, const Axis &, i64, i64, int, int, const double *,
                                            double *, hipStream_t);
template hipError_t launch_col2spec<float, float>(const Axis &, const Axis &, i64, i64, int, int, const float *,
                                                  float *, hipStream_t);
template hipError_t launch_col2spec<float, _Float16>(const Axis &, const Axis &, i64, i64, int, int, const float *,
                                                     _Float16 *, hipStream_t);
template hipError_t launch_col2spec<double, double>(const Axis &, const Axis &, i64, i64, int, int, const double *,
                                                    double *, hipStream_t);

}  // namespace mellin
