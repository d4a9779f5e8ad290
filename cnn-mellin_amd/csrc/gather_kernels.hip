// The LDS-gather kernels: layers with few input channels on the vector ALUs, no matrix
// instructions.
//
// A wavefront owns one tile of PT consecutive output positions of one output row (n, ox) and
// 64 output channels, ONE CHANNEL PER LANE.  The signal rows the output row reads -- for every
// (input channel, filter row) pair the row tap_x(ox, fx), i.e. the multiplicative gather of a
// Mellin axis resolved per row -- are staged in the wavefront's own piece of LDS (the window of
// PT + nfy - 1 columns the tile reads, zero where a tap or a column does not exist); the filter
// block lies in LDS channel-fastest, so that a lane fetches the nfy weights of its channel for a
// staged row with one 16-byte read that no other lane's read collides with.  In the inner loop a
// signal value is the same for all 64 lanes (an LDS broadcast read of four values at a time)
// and a weight is private to its lane: every vector instruction is 64 useful multiply-adds,
// with one LDS read per 10 to 16 of them and nothing to reduce across lanes.  Wavefronts share
// nothing but the filter block and never wait for each other (no barrier after the first), so
// the 16 wavefronts of a workgroup drift apart and one's loads and stores run behind the
// others' arithmetic.
//
// This is the non-matrix form the matrix-core kernels are measured against.  Its floor is the
// fp32 rate of the vector ALUs (one multiply-add per lane and cycle; packed fp32 instructions
// are not used), 78.6 TFLOP/s on the chip, against 2.5 PFLOP/s of bf16 matrix instructions at
// six per product -- but it has no fragments to build, no tile geometry and no phases that a
// whole workgroup walks through in step, which is what the matrix kernels spend their time on
// when a layer is as small as the benchmark's Mellin layer (0.48 GMAC).
#include <algorithm>
#include <atomic>

#include "gather_kernels.hpp"
#include "mellin_common.hpp"

namespace mellin {

namespace {

constexpr int kMaxRows = 32;                       // (input channel, filter row) pairs a tile stages

typedef const __attribute__((address_space(4))) GatherPlan ConstGather;

// NFY: filter columns (1 .. 8); PT: output positions per tile; RMAX: staged rows the instance
// holds (a multiple of 8 at or above the layer's c_in * nfx)
template <int NFY, int PT, int RMAX>
__global__ __launch_bounds__(1024, 1) void gather_forward_kernel(
    GatherPlan plan_arg, const float *__restrict__ F, const float *__restrict__ G,
    const float *__restrict__ bias, float *__restrict__ H) {
  ConstGather *const pl = (ConstGather *)__builtin_amdgcn_kernarg_segment_ptr();
  extern __shared__ __align__(16) float lds[];
  constexpr int NFYP = NFY <= 4 ? 4 : 8;                 // weights per (row, lane) slot
  constexpr int RWS = (PT + NFY - 1 + 3) & ~3;           // staged words per row (the window, padded to 16 bytes)
  static_assert(RWS <= 64, "a lane stages one word of a row");
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = nthreads >> 6;
  const int rows = pl->rows, nfx = pl->nfx;
  float *const Wl = lds;                                  // [rows][64][NFYP]
  float *const Xw = lds + rows * 64 * NFYP + wave * (RMAX * RWS);   // this wavefront's [RMAX][RWS]
  const int m0 = blockIdx.y * 64, m = m0 + lane;

  // ---- the filter block of these 64 channels, once per workgroup -----------------------------
  {
    const int K = rows * NFY;
    for (int idx = tid; idx < 64 * K; idx += nthreads) {
      const int co = idx / K, k = idx - co * K;
      const int r = k / NFY, fy = k - r * NFY;
      const int c = r / nfx, fx = r - c * nfx;
      Wl[(r * 64 + co) * NFYP + fy] =
          m0 + co < pl->M ? F[(i64)(m0 + co) * pl->f_m + (i64)c * pl->f_c + fx * NFY + fy] : 0.f;
    }
    if (NFYP > NFY)
      for (int idx = tid; idx < rows * 64; idx += nthreads)
#pragma unroll
        for (int fy = NFY; fy < NFYP; ++fy) Wl[idx * NFYP + fy] = 0.f;
  }
  __syncthreads();
  const float b = (bias && m < pl->M) ? bias[m] : 0.f;

  // what the item loop needs of the plan, read once
  const int tiles = pl->tiles, nox = pl->nox, noy = pl->noy, ngy = pl->ngy, ngx = pl->ngx, py = pl->py;
  const int kind_x = pl->kind_x, sx = pl->sx, dx = pl->dx, px = pl->px, ux = pl->ux, items = pl->items;
  const bool relu = pl->relu;
  const i64 g_n = pl->g_n, h_n = pl->h_n, h_m = pl->h_m;
  const int g_c = (int)pl->g_c;
  const unsigned image_bytes = (unsigned)pl->C * (unsigned)g_c * 4u;
  // staged row `lane` = (input channel, filter row), fixed for the launch
  const int my_c = min(lane, rows - 1) / nfx, my_fx = min(lane, rows - 1) - my_c * nfx;
  constexpr unsigned kDead = 0x40000000u;                 // a byte offset past any image: the load returns zero

  // ---- items: (image, output row, tile), dealt to the wavefronts of the launch in turn -------
  const int total_waves = gridDim.x * waves;
  for (int item = blockIdx.x * waves + wave; item < items; item += total_waves) {
    const int t = item % tiles, row_id = item / tiles;
    const int ox = row_id % nox, n = row_id / nox;
    const int start = min(t * PT, max(noy - PT, 0));       // (the last tile ends with the row)
    // stage: staged row r = (c, fx) holds columns start - py .. of signal row tap_x(ox, fx).
    // Lane r works out where row r starts in the image (one tap per lane, all rows at once);
    // the loads then take a row's start as their scalar offset and the lane's column as the
    // vector offset of a buffer load, which returns zero for what lies outside the image.
    {
      const int gx = tap32(kind_x, ox, my_fx, ngx, sx, dx, px, ux);
      const unsigned row_off = (gx >= 0 && lane < rows) ? (unsigned)(my_c * g_c + gx * ngy) * 4u : kDead;
      const int col = start - py + lane;
      const unsigned voff = (lane < RWS && col >= 0 && col < ngy) ? (unsigned)col * 4u : kDead;
      const __amdgpu_buffer_rsrc_t rsrc =
          __builtin_amdgcn_make_buffer_rsrc((void *)(G + (i64)n * g_n), 0, (int)image_bytes, 0x00020000);
      float v[RMAX];
#pragma unroll
      for (int r = 0; r < RMAX; ++r) {
        const unsigned so = __builtin_amdgcn_readlane(row_off, r);
        // (a row without a source: its offset alone is past the image, whatever the column)
        v[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(so == kDead ? kDead : voff),
                                                                              (int)(so == kDead ? 0u : so), 0));
      }
      if (lane < RWS) {
#pragma unroll
        for (int r = 0; r < RMAX; ++r) Xw[r * RWS + lane] = v[r];
      }
    }
    float acc[PT];
#pragma unroll
    for (int j = 0; j < PT; ++j) acc[j] = b;
    for (int r = 0; r < rows; ++r) {
      float w[NFYP], xw[RWS];
      {
        const float4 *wp = (const float4 *)(Wl + (r * 64 + lane) * NFYP);
#pragma unroll
        for (int i = 0; i < NFYP / 4; ++i) {
          const float4 q = wp[i];
          w[4 * i] = q.x; w[4 * i + 1] = q.y; w[4 * i + 2] = q.z; w[4 * i + 3] = q.w;
        }
        const float4 *xp = (const float4 *)(Xw + r * RWS);       // the same address in every lane: a broadcast
#pragma unroll
        for (int i = 0; i < RWS / 4; ++i) {
          const float4 q = xp[i];
          xw[4 * i] = q.x; xw[4 * i + 1] = q.y; xw[4 * i + 2] = q.z; xw[4 * i + 3] = q.w;
        }
      }
#pragma unroll
      for (int fy = 0; fy < NFY; ++fy)
#pragma unroll
        for (int j = 0; j < PT; ++j) acc[j] = fmaf(xw[j + fy], w[fy], acc[j]);
    }
    if (m < pl->M) {
      float *o = H + (i64)n * h_n + (i64)m * h_m + (i64)ox * noy + start;
      if (relu) {
#pragma unroll
        for (int j = 0; j < PT; ++j) acc[j] = fmaxf(acc[j], 0.f);
      }
      if (start + PT <= noy) {
#pragma unroll
        for (int j = 0; j < PT; ++j) o[j] = acc[j];
      } else {
#pragma unroll
        for (int j = 0; j < PT; ++j)
          if (start + j < noy) o[j] = acc[j];
      }
    }
  }
}

template <int NFY, int PT, int RMAX>
hipError_t launch_gather_forward_instance(const GatherPlan &gp, dim3 grid, const float *f, const float *g,
                                          const float *bias, float *h, hipStream_t stream) {
  auto kern = gather_forward_kernel<NFY, PT, RMAX>;
  static std::atomic<int> lds_allowed{0};                  // (one per kernel instance)
  hipError_t e = allow_large_lds((const void *)kern, gp.lds_bytes, lds_allowed);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, grid, dim3(64 * gp.waves), gp.lds_bytes, stream, gp, f, g, bias, h);
  return hipGetLastError();
}

}  // namespace

bool make_gather_forward_plan(const SepConv &pr, GatherPlan &gp) {
  if (pr.accumulate || pr.in_half || pr.out_half || pr.cls_nfx) return false;
  const Axis &X = pr.x, &Y = pr.y;
  if (Y.kind != AX_LCORR || Y.s != 1 || Y.d != 1 || Y.u != 1 || Y.nf < 1 || Y.nf > 8) return false;
  if (pr.c_in < 1 || X.nf < 1 || pr.c_in * X.nf > kMaxRows) return false;
  if (!axis_fits_tap32(X)) return false;
  const i64 lim = (i64)1 << 30;
  if (pr.batch < 1 || pr.c_out < 1 || X.nh < 1 || Y.nh < 1 || X.ng < 1 || Y.ng < 1) return false;
  if (pr.batch * X.nh >= lim || pr.c_out >= lim || Y.nh >= (1 << 20) || Y.ng >= (1 << 20) || X.ng >= lim) return false;
  if (Y.p > (1 << 20) || Y.p < -(1 << 20)) return false;
  if (pr.g_c < 0 || pr.c_in * pr.g_c >= ((i64)1 << 28)) return false;      // byte offsets inside an image stay below 2^30
  if (pr.f_c != X.nf * Y.nf && pr.c_in > 1) {}            // (any filter strides: the staging goes through f_m and f_c)
  gp.batch = (int)pr.batch; gp.M = (int)pr.c_out; gp.C = (int)pr.c_in;
  gp.nfx = (int)X.nf; gp.nfy = (int)Y.nf;
  gp.ngx = (int)X.ng; gp.ngy = (int)Y.ng; gp.nox = (int)X.nh; gp.noy = (int)Y.nh;
  gp.f_m = pr.f_m; gp.f_c = pr.f_c; gp.g_n = pr.g_n; gp.g_c = pr.g_c; gp.h_n = pr.h_n; gp.h_m = pr.h_m;
  gp.kind_x = X.kind; gp.sx = (int)X.s; gp.dx = (int)X.d; gp.px = (int)X.p; gp.ux = (int)X.u;
  gp.py = (int)Y.p;
  gp.relu = pr.relu;
  gp.rows = (int)(pr.c_in * X.nf);
  gp.pt = kGatherTile;
  gp.tiles = (int)((Y.nh + gp.pt - 1) / gp.pt);
  const i64 items = pr.batch * X.nh * gp.tiles;
  if (items >= lim) return false;
  gp.items = (int)items;
  gp.m_blocks = (int)((pr.c_out + 63) / 64);
  gp.rmax = (gp.rows + 7) & ~7;
  const int nfyp = gp.nfy <= 4 ? 4 : 8, rws = (gp.pt + gp.nfy - 1 + 3) & ~3;
  // wavefronts per workgroup: 16 when the launch has the items for them, and the LDS
  const size_t w_bytes = 4 * (size_t)gp.rows * 64 * nfyp, per_wave = 4 * (size_t)gp.rmax * rws;
  int waves = 16;
  while (waves > 4 && (items * gp.m_blocks < (i64)256 * waves || w_bytes + waves * per_wave > 150 * 1024)) waves >>= 1;
  if (w_bytes + waves * per_wave > 150 * 1024) return false;
  gp.waves = waves;
  gp.lds_bytes = w_bytes + waves * per_wave;
  return true;
}

hipError_t launch_gather_forward(const GatherPlan &gp, const float *f, const float *g, const float *bias, float *h,
                                 hipStream_t stream) {
  const i64 wgs = std::min<i64>(((i64)gp.items + gp.waves - 1) / gp.waves, std::max(1, 256 / gp.m_blocks));
  dim3 grid((unsigned)wgs, (unsigned)gp.m_blocks);
#define MELLIN_GATHER_CASE(NFY_)                                                                       \
  if (gp.nfy == NFY_) {                                                                                \
    if (gp.rmax == 8) return launch_gather_forward_instance<NFY_, kGatherTile, 8>(gp, grid, f, g, bias, h, stream);   \
    if (gp.rmax == 16) return launch_gather_forward_instance<NFY_, kGatherTile, 16>(gp, grid, f, g, bias, h, stream); \
    if (gp.rmax == 24) return launch_gather_forward_instance<NFY_, kGatherTile, 24>(gp, grid, f, g, bias, h, stream); \
    return launch_gather_forward_instance<NFY_, kGatherTile, 32>(gp, grid, f, g, bias, h, stream);     \
  }
  MELLIN_GATHER_CASE(1) MELLIN_GATHER_CASE(2) MELLIN_GATHER_CASE(3) MELLIN_GATHER_CASE(4)
  MELLIN_GATHER_CASE(5) MELLIN_GATHER_CASE(6) MELLIN_GATHER_CASE(7) MELLIN_GATHER_CASE(8)
#undef MELLIN_GATHER_CASE
  return hipErrorInvalidValue;
}

}  // namespace mellin
