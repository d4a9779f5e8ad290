// Descriptors of the LDS-gather kernels (gather_kernels.hip): few input channels, vector ALUs.
#pragma once

#include "mellin_common.hpp"

namespace mellin {

constexpr int kGatherTile = 20;                    // output positions per tile (and accumulators per lane)

struct GatherPlan {
  int batch, M, C, nfx, nfy;
  int ngx, ngy, nox, noy;
  i64 f_m, f_c, g_n, g_c, h_n, h_m;
  int kind_x, sx, dx, px, ux;      // x axis: any tap relation, resolved per (output row, filter row)
  int py;                          // y axis: a correlation with unit stride and dilation, no up-sampling
  int relu;
  int rows, rmax;                  // C * nfx: signal rows an output row reads; rounded up to a multiple of 8
  int pt, tiles, items;            // positions per tile; tiles per output row; batch * nox * tiles
  int m_blocks;                    // blocks of 64 output channels
  int waves;                       // wavefronts per workgroup
  size_t lds_bytes;
};

// false: the form does not apply (accumulate-into-h, half precision, residue classes, a y axis
// with a stride, a dilation or up-sampling, more than 8 filter columns or more than 32
// (input channel, filter row) pairs)
bool make_gather_forward_plan(const SepConv &pr, GatherPlan &gp);

hipError_t launch_gather_forward(const GatherPlan &gp, const float *f, const float *g, const float *bias, float *h,
                                 hipStream_t stream);

}  // namespace mellin
