// Second half of the two-pass input gradient used when the layer has few input
// channels.  The first pass (the matrix-core gather-GEMM, run with one output
// channel per (input channel, filter row) pair) leaves
//
//   Y[n, ci * nfx + fx, hx, gy] = sum_{co, fy} weight[co, ci, fx, fy] *
//                                 grad_out[n, co, hx, tap_y^-1(gy, fy)]
//
// i.e. everything but the sum over the filter's x taps.  This kernel finishes:
//
//   grad_input[n, ci, gx, gy] = sum_{fx} Y[n, ci * nfx + fx, hx(gx, fx), gy]
//
// over the fx whose tap exists, in ascending fx (a fixed order: no atomics).
// One thread per output element, coalesced along gy.
#include "mellin_common.hpp"

namespace mellin {

namespace {

__global__ __launch_bounds__(256) void fold_x_kernel(Axis x, i64 batch_cin, i64 ngx, i64 ngy,
                                                     const float *__restrict__ Y,
                                                     float *__restrict__ gi) {
  // x: convolution-kind axis with nf = nfx, ng = nhx (rows of Y), nh = ngx (rows of grad_input)
  const i64 total = batch_cin * ngx * ngy;
  const i64 nhx = x.ng, nfx = x.nf;
  const i64 step = (i64)gridDim.x * blockDim.x;
  for (i64 i = (i64)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
    const i64 gy = i % ngy;
    const i64 r = i / ngy;
    const i64 gx = r % ngx, nc = r / ngx;              // nc = n * c_in + ci
    const float *Ync = Y + nc * nfx * nhx * ngy + gy;
    float acc = 0.f;
    if (gx < x.nh_eff) {
      for (i64 fx = 0; fx < nfx; ++fx) {
        const i64 hx = tap_index(x.kind, gx, fx, nhx, x.s, x.d, x.p, x.u);
        if (hx >= 0) acc += Ync[(fx * nhx + hx) * ngy];
      }
    }
    gi[i] = acc;
  }
}

}  // namespace

hipError_t launch_fold_x(const Axis &x, i64 batch_cin, i64 ngx, i64 ngy, const float *Y,
                         float *grad_input, hipStream_t stream) {
  const i64 total = batch_cin * ngx * ngy;
  if (total == 0) return hipSuccess;
  i64 blocks = (total + 255) / 256;
  if (blocks > (1 << 20)) blocks = 1 << 20;
  hipLaunchKernelGGL(fold_x_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, batch_cin, ngx,
                     ngy, Y, grad_input);
  return hipGetLastError();
}

}  // namespace mellin
