// Descriptor of the fused input-gradient kernel for layers with few input
// channels and a linear x axis (igrad_gemm.hip).
#pragma once

#include "mellin_common.hpp"

namespace mellin {

struct IgradPlan {
  // problem: forward layer out[n, co, hx, hy] = sum w[co, ci, fx, fy] *
  // in[n, ci, sx hx + dx fx - px, sy hy + dy fy - py]   (ux = uy = 1)
  int batch, c_in, c_out;
  int nfx, nfy, nf;
  int nhx, nhy, nh;                // grad_out extent and nhx * nhy
  int ngx, ngy;                    // grad_input extent
  int sx, dx, px, sy, dy, py;
  // blocking
  int mtn;                         // 32-tap tiles per input channel
  int units;                       // c_in * mtn: wavefronts per job
  int jobs;                        // (image, strip) jobs that share a workgroup
  int ksteps;                      // (c_out rounded up) / 2: template instance
  int nt;                          // 32-position tiles per chunk: template instance
  int H;                           // grad_out rows that have a tap inside grad_input
  int Th, strips;                  // grad_out rows per workgroup; workgroups per image
  int nshared;                     // grad_input rows fed by both strips at a boundary
  int Rp, Wp;                      // accumulator plane: rows and row length (words)
  int pipe;                        // streaming variant (fold overlapped with the multiplies)
  int batched_fold;                // taps with congruent matrix rows never share a word: fold them in batches
  int stream;                      // the bf16 form: four wavefronts per strip, grad_out through registers
  int rw;                          // stream: grad_out rows per wavefront (Th = 4 * rw)
  size_t lds_bytes, ws_bytes;      // ws: partial rows at the strip boundaries
};

// force_nt / force_Th (0 = automatic) pin the chunk width and the strip height;
// force_pipe = 0 rules the streaming variant out.
// False when the layer does not suit the kernel (Mellin x axis, ux or uy != 1,
// too many channels, planes that do not fit in LDS, sizes beyond 32-bit indexing).
bool make_igrad_plan(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx,
                     i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py,
                     i64 ux, i64 uy, IgradPlan &pl, int force_nt = 0, int force_Th = 0, int force_pipe = -1,
                     int math = MATH_FP32);

hipError_t launch_igrad(const IgradPlan &pl, const float *weight, const float *grad_out,
                        float *grad_input, float *workspace, hipStream_t stream);

// The `stream` form of a plan on half-precision tensors (f16 matrix cores; the workspace
// keeps fp32 partial rows): weight, grad_out and grad_input are half-precision storage.
hipError_t launch_igrad_half(const IgradPlan &pl, const void *weight, const void *grad_out,
                             void *grad_input, float *workspace, hipStream_t stream);

// Tap products of the input gradient for layers with few input channels, any x
// axis kind: Z[n, ci, m, hx, hy] = sum_co w[co, ci, m] * grad_out[n, co, hx, hy]
// for every tap m = fx * nfy + fy (rows padded to a multiple of 32 per input
// channel; padded rows are not written).  A gather (fold_x.hip) finishes.
struct TapProductPlan {
  int batch, c_in, c_out, nf, nh;
  int mtn, units, jobs, ksteps;
  int chunks_per_image, cpw;         // 64-position chunks; chunks per workgroup
  int nf_pad;                        // mtn * 32
  size_t lds_bytes, ws_bytes;        // ws: Z
  // yfold: the kernel sums the four filter columns of a filter row itself and stores
  //   Y[n, ci, fx, hx, gy] = sum_fy Z[n, ci, fx * 4 + fy, hx, gy + py - fy]
  // (a quarter of Z; ws then holds Y, (batch, c_in, nfx, nhx, ngy)); a fold over x finishes.
  // A workgroup then takes rows_wg whole rows of grad_out.
  int yfold, nfx, nhx, nhy, ngy, py, rows_wg;
};

// Switches the plan to the y-folding form where it applies: four filter columns, unit
// stride, dilation and up-sampling along y, left padding only, grad_out rows of three
// positions or more, and a grad_input row that the taps of a grad_out row cover
// (ngy <= nhy + 3 - py).
void enable_tap_yfold(TapProductPlan &pl, i64 nfx, i64 nfy, i64 nhx, i64 nhy, i64 ngy, i64 sy, i64 dy, i64 py,
                      i64 uy);

bool make_tap_product_plan(i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 nhx, i64 nhy,
                           TapProductPlan &pl);

hipError_t launch_tap_product(const TapProductPlan &pl, const float *weight, const float *grad_out,
                              float *z, hipStream_t stream);

}  // namespace mellin
