// Gathers that finish the input gradient of layers with few input channels.
//
// fold_x: second half of the two-pass input gradient.  The first pass (the matrix-core gather-GEMM, run with one output
// channel per (input channel, filter row) pair) leaves
//
//   Y[n, ci * nfx + fx, hx, gy] = sum_{co, fy} weight[co, ci, fx, fy] *
//                                 grad_out[n, co, hx, tap_y^-1(gy, fy)]
//
// i.e. everything but the sum over the filter's x taps.  This kernel finishes:
//
//   grad_input[n, ci, gx, gy] = sum_{fx} Y[n, ci * nfx + fx, hx(gx, fx), gy]
//
// over the fx whose tap exists, in ascending fx (a fixed order: no atomics).  That
// is the column-to-signal adjoint with a trivial y axis, so the column-op kernel
// does it (col_ops.hip).
#include "mellin_common.hpp"

namespace mellin {

namespace {

// Gather that finishes the tap-product input gradient:
//
//   grad_input[n, ci, gx, gy] = sum_{fx, fy} Z[n, ci, fx * nfy + fy, hx(gx, fx), hy(gy, fy)]
//
// over the taps that exist, in ascending (fx, fy): a fixed order, no atomics.
// Z has nf_pad tap rows per (n, ci).  One thread per output, coalesced along gy.
// SMALL: every index product fits the 32-bit path above.
template <bool SMALL>
__global__ __launch_bounds__(256) void fold_xy_kernel(Axis x, Axis y, i64 batch_cin, int nf_pad,
                                                      const float *__restrict__ Z,
                                                      float *__restrict__ gi) {
  // x, y: convolution-kind axes with nf = filter extent, ng = grad_out extent, nh = grad_input extent
  const i64 ngx = x.nh, ngy = y.nh, nhx = x.ng, nhy = y.ng;
  const i64 total = batch_cin * ngx * ngy;
  const i64 nh = nhx * nhy;
  const i64 step = (i64)gridDim.x * blockDim.x;
  for (i64 i = (i64)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
    i64 gy, gx, nc;                                     // nc = n * c_in + ci
    if (SMALL) {
      const unsigned ui = (unsigned)i, r = ui / (unsigned)ngy;
      gy = ui - r * (unsigned)ngy;
      nc = r / (unsigned)ngx;
      gx = r - (unsigned)nc * (unsigned)ngx;
    } else {
      gy = i % ngy;
      const i64 r = i / ngy;
      gx = r % ngx;
      nc = r / ngx;
    }
    const float *Znc = Z + nc * nf_pad * nh;
    float acc = 0.f;
    if (gx < x.nh_eff && gy < y.nh_eff) {
      // the column's y taps are the same for every filter row: work them out once
      // (as offsets into a tap row of Z, -1 = no tap) when the filter is narrow enough
      constexpr int kHoist = 8;
      int yoff[kHoist];
      const int nfy = (int)y.nf;
      const bool hoisted = nfy <= kHoist;
      if (hoisted) {
#pragma unroll
        for (int fy = 0; fy < kHoist; ++fy) {
          i64 hy = -1;
          if (fy < nfy)
            hy = SMALL ? (i64)tap32(y.kind, (int)gy, fy, (int)nhy, (int)y.s, (int)y.d, (int)y.p, (int)y.u)
                       : tap_index(y.kind, gy, fy, nhy, y.s, y.d, y.p, y.u);
          yoff[fy] = hy < 0 ? -1 : (int)hy;
        }
      }
      for (int fx = 0; fx < (int)x.nf; ++fx) {
        const i64 hx = SMALL ? (i64)tap32(x.kind, (int)gx, fx, (int)nhx, (int)x.s, (int)x.d, (int)x.p, (int)x.u)
                             : tap_index(x.kind, gx, fx, nhx, x.s, x.d, x.p, x.u);
        if (hx < 0) continue;
        const float *Zf = Znc + (i64)fx * y.nf * nh + hx * nhy;
        if (hoisted) {
#pragma unroll
          for (int fy = 0; fy < kHoist; ++fy)
            if (fy < nfy && yoff[fy] >= 0) acc += Zf[(i64)fy * nh + yoff[fy]];
        } else {
          for (int fy = 0; fy < nfy; ++fy) {
            const i64 hy = SMALL ? (i64)tap32(y.kind, (int)gy, fy, (int)nhy, (int)y.s, (int)y.d, (int)y.p, (int)y.u)
                                 : tap_index(y.kind, gy, fy, nhy, y.s, y.d, y.p, y.u);
            if (hy >= 0) acc += Zf[(i64)fy * nh + hy];
          }
        }
      }
    }
    gi[i] = acc;
  }
}

}  // namespace

hipError_t launch_fold_xy(const Axis &x, const Axis &y, i64 batch_cin, int nf_pad, const float *Z,
                          float *grad_input, hipStream_t stream) {
  const i64 total = batch_cin * x.nh * y.nh;
  if (total == 0) return hipSuccess;
  {
    // the column-to-signal adjoint over padded tap planes: a thread works out a
    // position's taps once for eight (image, channel) pairs
    hipError_t e = hipSuccess;
    if (launch_col2spec_padded(x, y, batch_cin, nf_pad, Z, grad_input, stream, &e)) return e;
  }
  i64 blocks = (total + 255) / 256;
  if (blocks > (1 << 20)) blocks = 1 << 20;
  // the 32-bit path: every numerator of the tap relations and the flat index below 2^22 / 2^32
  const bool small = axis_fits_tap32(x) && axis_fits_tap32(y) && total < ((i64)1 << 32);
  if (small)
    hipLaunchKernelGGL(fold_xy_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, x, y, batch_cin,
                       nf_pad, Z, grad_input);
  else
    hipLaunchKernelGGL(fold_xy_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, x, y, batch_cin,
                       nf_pad, Z, grad_input);
  return hipGetLastError();
}

hipError_t launch_fold_x(const Axis &x, i64 batch_cin, i64 ngx, i64 ngy, const float *Y,
                         void *grad_input, hipStream_t stream, bool half_out) {
  // x: convolution-kind axis with nf = nfx, ng = nhx (rows of Y), nh = ngx (rows of grad_input);
  // Y is (batch_cin, nfx, 1, nhx, ngy): columns with an identity y axis
  (void)ngx;
  const Axis y = make_axis(AX_LCONV, 1, ngy, ngy, 1, 1, 0, 1);
  if (half_out) return launch_col2spec<float, _Float16>(x, y, batch_cin, 1, 0, 0, Y, (_Float16 *)grad_input, stream);
  return launch_col2spec<float, float>(x, y, batch_cin, 1, 0, 0, Y, (float *)grad_input, stream);
}

}  // namespace mellin
