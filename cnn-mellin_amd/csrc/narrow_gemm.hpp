// Descriptor of one launch of the few-channel linear x linear forward kernel (narrow_gemm.hip).
#pragma once

#include "mellin_common.hpp"

namespace mellin {

struct NarrowPlan {
  int batch, M, C;                 // images, output channels, input channels
  int nfx, nfy, nf, K;             // filter extent, nfx * nfy, C * nf
  int ngy, noy, Q;                 // signal columns, output columns, output positions per image
  int sx, dx, span;                // x stride and dilation; dx * (nfx - 1)
  i64 f_m, g_n, g_c, h_n, h_m;
  int relu;
  int mt, steps;                   // 32-channel tiles per workgroup; matrix steps of 16 taps of the instance that runs
  int tiles_per_image, total_tiles;
  unsigned mg_tpi, mg_noy;         // floor(2^32 / d) for tiles_per_image and noy (see udiv)
  unsigned mg_noy_v;               // floor(2^32 / noy) + 1: floor(q * m / 2^32) == q / noy for every q < Q (checked by the plan)
  unsigned mg_cw;                  // floor(2^32 / (R * ngy)) + 1: exact quotients below 2048 (checked by the plan)
  int R;                           // signal rows a tile can need per channel
  int n_elem, plane_bytes, sig_bytes;   // C * R * ngy; bytes of one part plane of a tile's pair words (rounded up to 16), of the three
  int g_bytes;                     // bytes from an image's first word to the end of its last channel
  size_t lds_bytes;
};

// false: the form does not apply.  It takes fp32 layers in the bf16x3 math mode whose axes are
// both correlations without padding, up-sampling or extra output rows, with unit stride and
// dilation along y and an even number of filter columns, c_in * nfx * nfy <= 128, dense filter
// layout, and (unless any_size) at least 1024 tiles of 256 positions x 64 channels.
bool make_narrow_plan(const SepConv &pr, NarrowPlan &np, bool any_size = false);

hipError_t launch_narrow_forward(const NarrowPlan &np, const float *f, const float *g, const float *bias, float *h,
                                 hipStream_t stream);

}  // namespace mellin
