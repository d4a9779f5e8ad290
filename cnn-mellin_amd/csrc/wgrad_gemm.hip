// Weight gradient on the fp32 matrix cores.
//
//   W[m, (c, fx, fy)] = sum_{n, ox, oy} A[n, m, ox, oy] *
//                       G[n, c, tap_x(ox, fx), tap_y(oy, fy)]
//
// (A = grad_out, G = layer input) is a (M x positions) * (positions x J)
// product, J = c_in * nfx * nfy, whose long dimension is the reduction.  The
// reduction is split over S persistent workgroups in a FIXED way: the position
// tiles of the forward kernel's tiling are numbered with the image running
// fastest and workgroup s takes the s-th contiguous range of them (the same
// positions of successive images come one after the other, so what the staging
// works out for one serves the next), each wavefront a quarter of every tile;
// a workgroup keeps its MT x JT accumulator tiles in registers for its whole life.  At the end the
// four wavefronts are summed through LDS in wave order, the workgroup writes
// one partial block to the workspace, and a second kernel adds the S partials
// in index order.  No floating-point atomics: the result is bit-reproducible.
//
// Operands are staged exactly as in the forward kernel (direct global->LDS
// loads, two buffers): the input as affine "virtual rows", so that the B
// operand of lane (column j) at position q is the LDS word
// col_offset[j] + pos_offset[q], and grad_out as one dense row of P positions
// per output channel (the A operand).
#include <algorithm>

#include "mellin_common.hpp"
#include "tile_gemm.hpp"
#include "tile_stage.hpp"

namespace mellin {

namespace {

constexpr int kGemmMemo = 8;                       // 64-word blocks per wave whose staging sources are kept
template <int MT, int JT, int NT>
__global__ __launch_bounds__(kThreads, 2) void wgrad_gemm_kernel(
    WgradPlan wp, const float *__restrict__ A, const float *__restrict__ G,
    float *__restrict__ ws) {
  extern __shared__ float lds[];
  const TilePlan &pl = wp.t;
  constexpr int M_T = MT * 32, J_T = JT * 32;
  constexpr int PW = NT * 32;                        // positions per wavefront and tile
  constexpr int P = kWaves * PW;
  constexpr int GS = 4;                              // position pairs per operand group
  const int x_words = wp.CCj * pl.R * pl.RS;
  const int a_words = M_T * wp.GSS;
  float *Xs0 = lds;                                  // [2][CCj][R][RS]
  float *As0 = Xs0 + 2 * x_words;                    // [2][M_T][GSS]
  int *posoff0 = (int *)(As0 + 2 * a_words);         // [2][P]
  const unsigned lds_base = lds_address(lds);

  const int tid = threadIdx.x;
  // the wave index is wave-uniform: say so, and everything derived from it (row
  // loops, base addresses) is computed on the scalar unit
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;

  // block of the output this workgroup owns
  const int mg = blockIdx.y / wp.j_groups, jg = blockIdx.y - mg * wp.j_groups;
  const int m0 = mg * M_T, j0 = jg * J_T;
  const int c_lo = j0 / pl.nf;
  const int j_last = min(wp.J, j0 + J_T) - 1;
  const int ccj = j_last / pl.nf - c_lo + 1;

  // LDS word of column j's tap relative to a position's base (constant per lane)
  int col_off[JT];
  {
    const FastDiv by_nf(pl.nf), by_nfy(pl.nfy);
#pragma unroll
    for (int t = 0; t < JT; ++t) {
      const int j = min(j0 + t * 32 + l32, wp.J - 1);   // columns past J are computed but never stored
      int c, tt, fx, fy;
      by_nf.divmod(j, c, tt);
      by_nfy.divmod(tt, fx, fy);
      col_off[t] = (c - c_lo) * pl.R * pl.RS + pl.Bx * fx * pl.RS + pl.by * fy;
    }
  }

  const FastDiv by_noy(pl.noy);
  // Tiles are numbered with the image running fastest and a workgroup takes a
  // contiguous range of them: consecutive tiles are then the same positions of
  // successive images, and where a staged word comes from, which words are zeros and
  // the positions' tap offsets stay what they were for the tile before.
  const int share = pl.total_tiles / (int)gridDim.x, extra = pl.total_tiles - share * (int)gridDim.x;
  const int my_tiles = share + ((int)blockIdx.x < extra ? 1 : 0);
  const int first_tile = (int)blockIdx.x * share + min((int)blockIdx.x, extra);
  auto tile_of = [&](int ti, int &n) {                    // the tile's number in the (image, tile) order
    const int i = first_tile + ti, t = i / pl.batch;
    n = i - t * pl.batch;
    return n * pl.tiles_per_image + t;
  };

  StageMemo<kGemmMemo> memo = {};
  auto issue_stage = [&](int ti) {
    int n_img;
    const TileGeom tg = tile_geometry<P>(pl, tile_of(ti, n_img), mellin_x);
    const int b = ti & 1;
    // tiles since the positions last changed (or since this workgroup started): the
    // memo is renewed at 0, and each of the two buffers gets its zeros and tap
    // offsets the first time it holds these positions
    const int run = min(n_img, ti);
    const bool fresh = run < 2;
    // (a zero the compiler cannot see through, added to the wave index: the staging
    // addresses are then worked out here and not once for the whole kernel, where
    // they would sit in registers across the matrix loops)
    unsigned zero;
    asm volatile("s_mov_b32 %0, 0" : "=s"(zero));
    const int wv = wave + (int)zero;
    issue_signal<kWaves, kGemmMemo>(pl, tg, G, c_lo, ccj, Xs0 + b * x_words, lds_base + 4u * (unsigned)(b * x_words),
                                    mellin_x, lane, wv, &memo, run == 0, fresh);
    // grad_out rows: P consecutive positions per output channel, zeros past the tile
    float *As = As0 + b * a_words;
    const int m_live = max(0, min(M_T, pl.M - m0));
    const i64 row_step = (i64)kWaves * wp.a_m;
    const unsigned dst_step = 4u * (unsigned)(kWaves * wp.GSS);
    for (int pb = 0; pb < P; pb += 64) {
      const int p = pb + lane;
      if (p < tg.count) {
        const float *row = A + (i64)tg.n * wp.a_n + tg.q0 + (i64)(m0 + wv) * wp.a_m;
        unsigned dst = lds_base + 4u * (unsigned)(2 * x_words + b * a_words + wv * wp.GSS + pb);
        for (int m = wv; m < m_live; m += kWaves) {
          load_to_lds_at(row, (unsigned)p * 4u, dst);
          row += row_step;
          dst += dst_step;
        }
        if (fresh)
          for (int m = m_live + wv; m < M_T; m += kWaves) As[m * wp.GSS + p] = 0.f;
      } else if (fresh) {
        for (int m = wv; m < M_T; m += kWaves) As[m * wp.GSS + p] = 0.f;
      }
    }
    // LDS word of every position's (fx = 0, fy = 0) tap
    if (fresh) {
      int *posoff = posoff0 + b * P;
      for (int p = tid; p < P; p += kThreads) {
        const int q = tg.q0 + (p < tg.count ? p : 0);       // past the tile: any valid position
        int ox, oy;
        by_noy.divmod(q, ox, oy);
        posoff[p] = (pl.Ax * (ox - tg.ox_lo) + pl.Cx0) * pl.RS + pl.ay * (oy - tg.oy_lo) - pl.by_min;
      }
    }
  };

  floatx16 acc[MT][JT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < JT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  if (my_tiles > 0) issue_stage(0);

  for (int ti = 0; ti < my_tiles; ++ti) {
    wait_all_memory();
    __syncthreads();
    if (ti + 1 < my_tiles) {
      __builtin_amdgcn_s_setprio(3);                     // staging ahead of the other wavefronts' multiplies
      issue_stage(ti + 1);
      __builtin_amdgcn_s_setprio(0);
    }

    const int tile = (first_tile + ti) / pl.batch;
    int count;
    if (pl.segment) count = min(P, pl.noy - (tile % pl.chunks_per_row) * P);
    else count = min(P, pl.Q - tile * P);
    const int cnt_w = max(0, min(PW, count - wave * PW));  // this wavefront's live positions
    const int steps = (cnt_w + 1) >> 1;
    const int full = cnt_w >> 1;                           // pairs with both positions live

    const float *Xs = Xs0 + (ti & 1) * x_words;
    const float *ap = As0 + (ti & 1) * a_words + l32 * wp.GSS + wave * PW + half;
    const int *pp = posoff0 + (ti & 1) * P + wave * PW + half;
    const int arow = 32 * wp.GSS;
    const int groups = full / GS;
    float a0[GS][MT], b0[GS][JT], a1[GS][MT], b1[GS][JT];
    auto fetch = [&](int g, float (&a)[GS][MT], float (&b)[GS][JT]) {
      int po[GS];
#pragma unroll
      for (int k = 0; k < GS; ++k) po[k] = pp[2 * (g * GS + k)];
#pragma unroll
      for (int k = 0; k < GS; ++k) {
#pragma unroll
        for (int i = 0; i < MT; ++i) a[k][i] = ap[2 * (g * GS + k) + i * arow];
#pragma unroll
        for (int t = 0; t < JT; ++t) b[k][t] = Xs[col_off[t] + po[k]];
      }
    };
    auto multiply = [&](float (&a)[GS][MT], float (&b)[GS][JT]) {
#pragma unroll
      for (int k = 0; k < GS; ++k)
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int t = 0; t < JT; ++t)
            acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[k][i], b[k][t], acc[i][t], 0, 0, 0);
    };
    int g = 0;
    if (groups > 0) fetch(0, a0, b0);
    for (; g + 1 < groups; g += 2) {
      fetch(g + 1, a1, b1);
      multiply(a0, b0);
      if (g + 2 < groups) fetch(g + 2, a0, b0);
      multiply(a1, b1);
    }
    if (g < groups) multiply(a0, b0);
    for (int s = groups * GS; s < steps; ++s) {
      const int po = pp[2 * s];
      float a[MT], b[JT];
#pragma unroll
      for (int i = 0; i < MT; ++i) a[i] = ap[2 * s + i * arow];
      // the odd last position of a tile multiplies a zero of grad_out; force the
      // other operand to zero as well so that a non-finite input cannot leak in
#pragma unroll
      for (int t = 0; t < JT; ++t) b[t] = (s >= full && half) ? 0.f : Xs[col_off[t] + po];
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < JT; ++t)
          acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[t], acc[i][t], 0, 0, 0);
    }
  }

  // ---- sum the four wavefronts in wave order, then write the partial block ------
  __syncthreads();
  float *red = lds;                                   // [M_T][J_T]
  for (int w = 0; w < kWaves; ++w) {
    if (wave == w) {
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < JT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = i * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            float *dst = red + m * J_T + t * 32 + l32;
            if (w == 0) *dst = acc[i][t][r];
            else *dst += acc[i][t][r];
          }
    }
    __syncthreads();
  }
  float *out = ws + (i64)blockIdx.x * wp.M_pad * wp.J_pad + (i64)m0 * wp.J_pad + j0;
  for (int e = tid; e < M_T * J_T; e += kThreads) {
    const int m = e / J_T, jj = e - m * J_T;
    out[(i64)m * wp.J_pad + jj] = red[e];
  }
}

// Row-wise variant for layers whose outputs are walked a whole row at a time
// (unit y stride, rows of at least four outputs that fit one tile).  A unit of work
// is 4 * rpw consecutive output rows of one image, rpw rows per wavefront.  Within
// a row every operand address is affine in the column: position oy of output
// row ox reads grad_out word  row_base + oy  and, for column j = (c, fx, fy),
// input word  col_offset[j] + virtual_row(ox) * RS + oy - by_min,  so the loop
// over the row needs no index arithmetic at all: LDS reads with immediate
// offsets and matrix instructions only.  (On this chip the fp32 matrix
// instructions run on the same ALUs as ordinary vector instructions: every
// vector instruction saved in the loop is matrix throughput gained.)
// grad_out rows arrive by 16-byte direct loads (the four rows of a unit are
// contiguous per channel); the input rows are staged as in the forward kernel.
constexpr int kRowsMemo = 8;                       // 64-word blocks per wave whose staging sources are kept
template <int MT, int JT>
__global__ __launch_bounds__(kThreads) void wgrad_rows_kernel(
    WgradPlan wp, const float *__restrict__ A, const float *__restrict__ G,
    float *__restrict__ ws) {
  extern __shared__ __align__(16) float lds[];
  const TilePlan &pl = wp.t;
  constexpr int M_T = MT * 32, J_T = JT * 32;
  const int RB = kWaves * wp.rpw;                    // output rows per unit
  const int x_words = (wp.CCj * pl.R * pl.RS + 3) & ~3;
  const int a_words = M_T * wp.GSS;
  float *Xs0 = lds;                                  // [nbuf][CCj][R][RS]
  float *As0 = Xs0 + wp.nbuf * x_words;              // [nbuf][M_T][GSS]

  const int tid = threadIdx.x;
  // the wave index is wave-uniform: say so, and everything derived from it (row
  // loops, base addresses) is computed on the scalar unit
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;

  const int mg = blockIdx.y / wp.j_groups, jg = blockIdx.y - mg * wp.j_groups;
  const int m0 = mg * M_T, j0 = jg * J_T;
  const int c_lo = j0 / pl.nf;
  const int j_last = min(wp.J, j0 + J_T) - 1;
  const int ccj = j_last / pl.nf - c_lo + 1;
  const int m_live = max(0, min(M_T, pl.M - m0));

  int col_off[JT];
  {
    const FastDiv by_nf(pl.nf), by_nfy(pl.nfy);
#pragma unroll
    for (int t = 0; t < JT; ++t) {
      const int j = min(j0 + t * 32 + l32, wp.J - 1);   // columns past J are computed but never stored
      int c, tt, fx, fy;
      by_nf.divmod(j, c, tt);
      by_nfy.divmod(tt, fx, fy);
      col_off[t] = (c - c_lo) * pl.R * pl.RS + pl.Bx * fx * pl.RS + pl.by * fy;
    }
  }
  // grad_out rows of channels past M are never loaded: zeros, once
  if (m_live < M_T) {
    const int dead = (M_T - m_live) * wp.GSS;
    for (int i = tid; i < dead; i += kThreads) {
      As0[m_live * wp.GSS + i] = 0.f;
      if (wp.nbuf == 2) As0[a_words + m_live * wp.GSS + i] = 0.f;
    }
  }

  // Units are numbered with the image running fastest and a workgroup takes a
  // contiguous range of them: consecutive units are then the same rows of successive
  // images, and where a staged word comes from (and which words are zeros) stays what
  // it was for the unit before.
  const int units_per_image = (pl.nox_eff + RB - 1) / RB;
  const int total_units = pl.batch * units_per_image;
  const int share = total_units / (int)gridDim.x, extra = total_units - share * (int)gridDim.x;
  const int my_units = share + ((int)blockIdx.x < extra ? 1 : 0);
  const int first_unit = (int)blockIdx.x * share + min((int)blockIdx.x, extra);
  const unsigned lds_base = lds_address(lds);
  const unsigned as_addr = lds_base + 4u * (unsigned)(wp.nbuf * x_words);

  auto unit_geometry = [&](int unit) {
    TileGeom g;
    const int u = unit / pl.batch;
    g.n = unit - u * pl.batch;
    g.ox_lo = u * RB;
    const int rows = min(RB, pl.nox_eff - g.ox_lo);
    g.oy_lo = 0;
    g.q0 = g.ox_lo * pl.noy;
    g.count = rows * pl.noy;
    g.R_tile = mellin_x ? rows * pl.nfx : pl.ax * (rows - 1) + pl.bx_span + 1;
    g.vx_min = pl.ax * g.ox_lo + pl.cx + pl.bx_min;
    g.vy_min = pl.cy + pl.by_min;
    g.RSL = pl.ay * (pl.noy - 1) + pl.by_span + 1;
    return g;
  };
  StageMemo<kRowsMemo> memo = {};
  auto issue_stage = [&](int ui) {
    const TileGeom tg = unit_geometry(first_unit + ui);
    const int b = wp.nbuf == 2 ? (ui & 1) : 0;
    // units since the rows last changed (or since this workgroup started): the memo is
    // renewed at 0, and a buffer's zeros are written the first time it holds these rows
    const int run = min(tg.n, ui);
    // (a zero the compiler cannot see through, added to the wave index: the staging
    // addresses are then worked out here and not once for the whole kernel, where
    // they would sit in registers across the matrix loops)
    unsigned zero;
    asm volatile("s_mov_b32 %0, 0" : "=s"(zero));
    issue_signal<kWaves, kRowsMemo>(pl, tg, G, c_lo, ccj, Xs0 + b * x_words, lds_base + 4u * (unsigned)(b * x_words),
                                    mellin_x, lane, wave + (int)zero, &memo, run == 0, run < wp.nbuf);
    // grad_out: the unit's rows are one run of `count` words per channel
    const float *An = A + (i64)tg.n * wp.a_n;
    const int count4 = tg.count & ~3;
    for (int m = wave; m < m_live; m += kWaves) {
      const float *src = An + (i64)(m0 + m) * wp.a_m;
      const unsigned dst = as_addr + 4u * (unsigned)(b * a_words + m * wp.GSS);
      for (int w0 = 0; w0 < count4; w0 += 256) {
        const int idx = w0 + 4 * lane;
        if (idx < count4) load16_to_lds_at(src, (unsigned)(tg.q0 + idx) * 4u, dst + 4u * (unsigned)w0);
      }
      if (lane < tg.count - count4)
        load_to_lds_at(src, (unsigned)(tg.q0 + count4 + lane) * 4u, dst + 4u * (unsigned)count4);
    }
  };

  floatx16 acc[MT][JT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < JT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  const int pairs = pl.noy >> 1;
  auto multiply_unit = [&](int ui) {
    const int ox_lo = ((first_unit + ui) / pl.batch) * RB;
    for (int row = wave; row < RB && ox_lo + row < pl.nox_eff; row += kWaves) {   // this wavefront's rows
      const int b = wp.nbuf == 2 ? (ui & 1) : 0;
      const float *Xs = Xs0 + b * x_words;
      const float *As = As0 + b * a_words;
      int ao = l32 * wp.GSS + row * pl.noy + half;
      int bo[JT];
#pragma unroll
      for (int t = 0; t < JT; ++t)
        bo[t] = col_off[t] + (pl.Ax * row + pl.Cx0) * pl.RS - pl.by_min + half;
      int s = 0;
      for (; s + 8 <= pairs; s += 8) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          float a[MT], b[JT];
#pragma unroll
          for (int i = 0; i < MT; ++i) a[i] = As[ao + i * 32 * wp.GSS + 2 * k];
#pragma unroll
          for (int t = 0; t < JT; ++t) b[t] = Xs[bo[t] + 2 * k];
#pragma unroll
          for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int t = 0; t < JT; ++t)
              acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[t], acc[i][t], 0, 0, 0);
        }
        ao += 16;
#pragma unroll
        for (int t = 0; t < JT; ++t) bo[t] += 16;
      }
      // the row's last up-to-seven pairs and, if the row is odd, its last position alone:
      // every step sits at a fixed distance from where the groups of eight stopped, so
      // the reads take immediate offsets and the steps cost no vector arithmetic
      const int left = pairs - s + (pl.noy & 1);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (k < left) {
          float a[MT], b[JT];
#pragma unroll
          for (int i = 0; i < MT; ++i) a[i] = As[ao + i * 32 * wp.GSS + 2 * k];
#pragma unroll
          for (int t = 0; t < JT; ++t) b[t] = Xs[bo[t] + 2 * k];
          if (s + k == pairs) {                           // a position alone: the other half-wave multiplies zeros
#pragma unroll
            for (int i = 0; i < MT; ++i) a[i] = half ? 0.f : a[i];
#pragma unroll
            for (int t = 0; t < JT; ++t) b[t] = half ? 0.f : b[t];
          }
#pragma unroll
          for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int t = 0; t < JT; ++t)
              acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[t], acc[i][t], 0, 0, 0);
        }
      }
    }
  };
  __syncthreads();
  if (wp.nbuf == 2) {
    // two buffers: the loads of the next unit fly during the multiplies of this one
    if (my_units > 0) issue_stage(0);
    for (int ui = 0; ui < my_units; ++ui) {
      wait_all_memory();
      __syncthreads();
      if (ui + 1 < my_units) {
        __builtin_amdgcn_s_setprio(3);
        issue_stage(ui + 1);
        __builtin_amdgcn_s_setprio(0);
      }
      multiply_unit(ui);
    }
  } else {
    // one buffer and more workgroups per CU: they cover each other's loads
    for (int ui = 0; ui < my_units; ++ui) {
      __builtin_amdgcn_s_setprio(3);                   // staging ahead of the other workgroups' multiplies
      issue_stage(ui);
      __builtin_amdgcn_s_setprio(0);
      wait_all_memory();
      __syncthreads();
      multiply_unit(ui);
      __syncthreads();
    }
  }

  // ---- sum the four wavefronts, then write the partial block -------------------------------
  // Every workgroup of the one-round grid gets here at the same moment, so this is on the launch's
  // critical path.  Two slabs: wavefronts 0 and 2 store their sums, 1 and 3 add theirs on top, and
  // the block is slab 0 + slab 1, i.e. (w0 + w1) + (w2 + w3) whatever the timing; the write-out
  // has several words in flight per thread.
  __syncthreads();
  float *red = lds;                                   // [2][M_T][J_T]
  for (int phase = 0; phase < 2; ++phase) {
    if ((wave & 1) == phase) {
      float *slab = red + (wave >> 1) * (M_T * J_T);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < JT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = i * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            float *dst = slab + m * J_T + t * 32 + l32;
            if (phase == 0) *dst = acc[i][t][r];
            else *dst += acc[i][t][r];
          }
    }
    __syncthreads();
  }
  float *out = ws + (i64)blockIdx.x * wp.M_pad * wp.J_pad + (i64)m0 * wp.J_pad + j0;
  constexpr int kTrip = 4;                             // words a thread has in flight (M_T * J_T is a multiple of 1024)
  for (int e0 = tid; e0 < M_T * J_T; e0 += kTrip * kThreads) {
    float v[kTrip];
#pragma unroll
    for (int u = 0; u < kTrip; ++u) v[u] = red[e0 + u * kThreads] + red[M_T * J_T + e0 + u * kThreads];
#pragma unroll
    for (int u = 0; u < kTrip; ++u) {
      const int e = e0 + u * kThreads, m = e / J_T, jj = e - m * J_T;
      out[(i64)m * wp.J_pad + jj] = v[u];
    }
  }
}

// The row-wise weight gradient on the bf16 matrix cores (tile_stage.hpp: every fp32 operand
// as the exact sum of three bf16 parts, six products each).  Same units and partial-sum
// scheme as above; what differs is how the operands reach the matrix instructions.
//
//   * A step covers 16 positions, two groups of eight consecutive outputs of one row (one
//     per half-wave); a row of noy outputs is NG = ceil(noy / 8) groups, the last one moved
//     back to start at noy - 8 so that it is eight whole positions too (the ones it shares
//     with the group before it meet zeros in the other operand).  The groups of a unit are
//     numbered row by row and paired into steps regardless of rows; wavefront w takes steps
//     w, w + 4, ...
//   * grad_out (95 % of the bytes) never touches LDS: the eight positions of a lane's
//     channel are 32 consecutive bytes of global memory, loaded straight into registers
//     two steps ahead and split there.  Every grad_out value is loaded and split once.
//   * the input words a unit needs are loaded into registers while the unit before it
//     multiplies, then split once, by all threads, into 16-byte fragments
//     Bf[part][channel][virtual row][group][fy]: the eight input words that the group's
//     positions read through filter column fy (zeros for padding and for rows without a
//     tap).  One thread makes all nfy fragments of a (channel, row, group): it splits the
//     8 + nfy - 1 words once and assembles the shifted copies from the packed halves.  A
//     lane (column j = (c, fx, fy)) fetches its operand of a step with three aligned
//     16-byte LDS reads.
// Nothing here uses the direct global->LDS loads, so the compiler counts every load in
// flight and a wait for one never drags in the younger ones.  Needs unit y stride, no y
// up-sampling and unit y dilation (consecutive filter columns read consecutive words).
constexpr int kStreamTasks = 2;                    // (channel, row, group) tasks a thread can hold in registers
template <int MT, int JT>
__global__ __launch_bounds__(kThreads, (MT == 1 ? 3 : 2)) void wgrad_stream_kernel(
    WgradPlan wp, const float *__restrict__ A, const float *__restrict__ G,
    float *__restrict__ ws) {
  extern __shared__ __align__(16) float lds[];
  const TilePlan &pl = wp.t;
  constexpr int M_T = MT * 32, J_T = JT * 32;
  const int RB = kWaves * wp.rpw;                    // output rows per unit
  const int NG = (pl.noy + 7) >> 3;                  // groups per row
  const int tail0 = pl.noy - 8;                      // first position of a row's last group
  const int tasks_max = wp.CCj * pl.R * NG;          // (channel, virtual row, group) triples
  const int bf_part = tasks_max * pl.nfy + 1;        // fragments per part; the last word of a part is zeros
  uintx4 *Bf = (uintx4 *)lds;                        // [3][CCj][R][NG][nfy] (+ the zero word)
  int2 *step_tab = (int2 *)(Bf + 3 * bf_part);       // [groups of a full unit]: grad_out offset, fragment offset

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;

  const int mg = blockIdx.y / wp.j_groups, jg = blockIdx.y - mg * wp.j_groups;
  const int m0 = mg * M_T, j0 = jg * J_T;
  const int c_lo = j0 / pl.nf;
  const int j_last = min(wp.J, j0 + J_T) - 1;
  const int ccj = j_last / pl.nf - c_lo + 1;

  // fragment word of column j's tap for (unit row 0, group 0)
  int col_word[JT];
  {
    const FastDiv by_nf(pl.nf), by_nfy(pl.nfy);
#pragma unroll
    for (int t = 0; t < JT; ++t) {
      const int j = min(j0 + t * 32 + l32, wp.J - 1);   // columns past J are computed but never stored
      int c, tt, fx, fy;
      by_nf.divmod(j, c, tt);
      by_nfy.divmod(tt, fx, fy);
      col_word[t] = ((c - c_lo) * pl.R + pl.Bx * fx + pl.Cx0) * NG * pl.nfy + fy;
    }
  }
  // this lane's grad_out channel per tile, as a word offset within an image (channels past M
  // read the last one; their rows of the result are never used)
  int a_off[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) a_off[i] = min(m0 + i * 32 + l32, pl.M - 1) * (int)wp.a_m;

  const int units_per_image = (pl.nox_eff + RB - 1) / RB;
  const int total_units = pl.batch * units_per_image;
  const int share = total_units / (int)gridDim.x, extra = total_units - share * (int)gridDim.x;
  const int my_units = share + ((int)blockIdx.x < extra ? 1 : 0);
  const int first_unit = (int)blockIdx.x * share + min((int)blockIdx.x, extra);

  const FastDiv by_ng(NG), by_r(pl.R), by_nfx(pl.nfx);
  for (int i = tid; i < RB * NG + 1; i += kThreads) {
    int r, g;
    by_ng.divmod(i, r, g);                              // group i of the unit: row r, group g of the row
    step_tab[i] = make_int2(r * pl.noy + (g == NG - 1 ? tail0 : 8 * g), (pl.Ax * r * NG + g) * pl.nfy);
  }
  if (tid < 3) Bf[tid * bf_part + bf_part - 1] = uintx4{0u, 0u, 0u, 0u};

  // ---- the input words of a unit, in registers --------------------------------------
  // task tk = (cl * R + vrow) * NG + g; a thread takes tasks tid, tid + 256, ...  A task loads
  // the E = 8 + nfy - 1 words its nfy fragments share (up to 16).  What does not change
  // from unit to unit is worked out once: the task's virtual row (-1: no such task), the
  // offset of its first word within an image apart from the row, which of its words lie
  // inside the image, and how many leading positions the group before already covers.
  const int E = 8 + pl.nfy - 1, n4 = (E + 3) >> 2;
  struct XRegs { float v[kStreamTasks][16]; };
  int t_row[kStreamTasks], t_off[kStreamTasks], t_mask[kStreamTasks], t_dead[kStreamTasks];
#pragma unroll
  for (int k = 0; k < kStreamTasks; ++k) {
    const int tk = tid + k * kThreads;
    int rest, g, cl, vrow;
    by_ng.divmod(tk, rest, g);
    by_r.divmod(rest, cl, vrow);
    const bool tail = g == NG - 1;
    const int c0 = (tail ? tail0 : 8 * g) + pl.cy;         // signal column of the group's first position, fy = 0
    int mask = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) mask |= (e < E && c0 + e >= 0 && c0 + e < pl.ngy) ? 1 << e : 0;
    // the whole run of 4 * n4 words lies inside the row: it can be loaded 16 bytes at a time
    if (c0 >= 0 && c0 + 4 * n4 <= pl.ngy) mask |= 1 << 16;
    t_row[k] = (tk < tasks_max && cl < ccj) ? vrow : -1;
    t_off[k] = cl * (int)pl.g_c + c0;                      // fits: c_in * ngx * ngy < 2^31
    t_mask[k] = mask;
    t_dead[k] = tail ? 8 * g - tail0 : 0;
  }
  auto load_x = [&](int ui, XRegs &xr) {
    const int unit = first_unit + ui;
    const int u = unit / pl.batch, n = unit - u * pl.batch;
    const int ox_lo = u * RB, rows = min(RB, pl.nox_eff - ox_lo);
    const int R_tile = mellin_x ? rows * pl.nfx : pl.ax * (rows - 1) + pl.bx_span + 1;
    const int vx_min = pl.ax * ox_lo + pl.cx + pl.bx_min;
    const float *Gn = G + (i64)n * pl.g_n + (i64)c_lo * pl.g_c;
#pragma unroll
    for (int k = 0; k < kStreamTasks; ++k) {
      const int vrow = t_row[k];
      int gx = -1;
      if (vrow >= 0 && vrow < R_tile) {
        if (mellin_x) {
          int oxl, fx;
          by_nfx.divmod(vrow, oxl, fx);
          gx = mellin_tap32(pl.kind_x, ox_lo + oxl, fx, pl.ngx, pl.sx, pl.dx, pl.px + 1, pl.ux, pl.mg_p1);
        } else {
          const int vx = vx_min + vrow;
          if (vx >= 0) {
            if (pl.ux == 1) { if (vx < pl.ngx) gx = vx; }
            else { const int qx = vx / pl.ux; if (qx * pl.ux == vx && qx < pl.ngx) gx = qx; }
          }
        }
      }
      const float *src = Gn + (t_off[k] + max(gx, 0) * pl.ngy);
      const int mask = gx >= 0 ? t_mask[k] : 0;
      if (mask >> 16) {
        typedef float4 __attribute__((aligned(4))) float4u;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float4 w = make_float4(0.f, 0.f, 0.f, 0.f);
          if (q < n4) w = *(const float4u *)(src + 4 * q);
          xr.v[k][4 * q] = w.x; xr.v[k][4 * q + 1] = w.y; xr.v[k][4 * q + 2] = w.z; xr.v[k][4 * q + 3] = w.w;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) xr.v[k][e] = (mask >> e & 1) ? src[e] : 0.f;
      }
    }
  };
  auto store_x = [&](const XRegs &xr) {
#pragma unroll
    for (int k = 0; k < kStreamTasks; ++k) {
      const int tk = tid + k * kThreads;
      if (tk >= tasks_max) continue;
      // the three parts of every word, packed in pairs: P[part][q] = words 2 q, 2 q + 1
      unsigned P[3][8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        split_pair(xr.v[k][2 * q], xr.v[k][2 * q + 1], P[0][q], P[1][q], P[2][q]);
      }
      // positions the group before already covers become zeros (pairs 2 i, 2 i + 1 of the fragment)
      const int dead = t_dead[k];
      unsigned keep[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) keep[i] = 2 * i + 1 < dead ? 0u : (2 * i < dead ? 0xFFFF0000u : 0xFFFFFFFFu);
#pragma unroll
      for (int fy = 0; fy < 8; ++fy) {
        if (fy < pl.nfy) {
#pragma unroll
          for (int part = 0; part < 3; ++part) {
            uintx4 w;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              // words fy + 2 i, fy + 2 i + 1
              const unsigned v = (fy & 1) ? __builtin_amdgcn_alignbit(P[part][(fy + 1) / 2 + i < 8 ? (fy + 1) / 2 + i : 7],
                                                                       P[part][(fy - 1) / 2 + i], 16)
                                          : P[part][fy / 2 + i];
              w[i] = v & keep[i];
            }
            Bf[part * bf_part + tk * pl.nfy + fy] = w;
          }
        }
      }
    }
  };

  floatx16 acc[MT][JT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < JT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  // ---- steps ----------------------------------------------------------------------------
  // Operands of step s of the current unit for this lane: the grad_out words come from
  // global memory (requested two steps ahead), the fragments from LDS.
  struct AOp { float4 lo[MT], hi[MT]; int bword; };
  const float *abase = A;                               // grad_out of the unit's image and first row (wave-uniform)
  int live_groups = 0;                                  // groups of the current unit
  auto load_a = [&](int s, AOp &o) {
    int gi = 2 * s + half;
    const bool live = gi < live_groups;
    if (!live) gi = 0;                                  // past the last group: any valid words, and zeros on the other side
    const int2 e = step_tab[gi];
    o.bword = live ? e.y : -1;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      typedef float4 __attribute__((aligned(4))) float4u;   // a row starts wherever the rows before it end
      const float *p = abase + (a_off[i] + e.x);
      o.lo[i] = *(const float4u *)p;
      o.hi[i] = *(const float4u *)(p + 4);
    }
  };
  auto multiply_step = [&](const AOp &o) {
    uintx4 bh[JT], bm[JT], bl[JT];
#pragma unroll
    for (int t = 0; t < JT; ++t) {
      const uintx4 *b = Bf + (o.bword >= 0 ? col_word[t] + o.bword : bf_part - 1);
      bh[t] = b[0]; bm[t] = b[bf_part]; bl[t] = b[2 * bf_part];
    }
    uintx4 ah[MT], am[MT], al[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const float x[8] = {o.lo[i].x, o.lo[i].y, o.lo[i].z, o.lo[i].w, o.hi[i].x, o.hi[i].y, o.hi[i].z, o.hi[i].w};
      split8(x, ah[i], am[i], al[i]);
    }
#pragma unroll
    for (int t = 0; t < JT; ++t)
#pragma unroll
      for (int i = 0; i < MT; ++i) mfma_split6(acc[i][t], ah[i], am[i], al[i], bh[t], bm[t], bl[t]);
  };

  XRegs xr;
  if (my_units > 0) load_x(0, xr);
  for (int ui = 0; ui < my_units; ++ui) {
    const int unit = first_unit + ui;
    const int u = unit / pl.batch, n = unit - u * pl.batch;
    const int ox_lo = u * RB, rows = min(RB, pl.nox_eff - ox_lo);
    live_groups = rows * NG;
    const int steps = (live_groups + 1) >> 1;
    abase = A + (i64)n * wp.a_n + (i64)ox_lo * pl.noy;
    __syncthreads();                                     // every wavefront is done with the fragments of the unit before
    // this wavefront's first two steps: their grad_out words travel while the input is split
    AOp b0, b1, b2;
    load_a(min(wave, steps - 1), b0);
    load_a(min(wave + kWaves, steps - 1), b1);
    b2 = b1;
    store_x(xr);
    __syncthreads();                                     // fragments complete
    if (ui + 1 < my_units) load_x(ui + 1, xr);           // consumed at the top of the next unit
    // three operand buffers in rotation, two steps in flight; no copies, so no wait for a
    // younger load sneaks in
    for (int s = wave; s < steps; s += 3 * kWaves) {
      if (s + 2 * kWaves < steps) load_a(s + 2 * kWaves, b2);
      multiply_step(b0);
      if (s + kWaves >= steps) break;
      if (s + 3 * kWaves < steps) load_a(s + 3 * kWaves, b0);
      multiply_step(b1);
      if (s + 2 * kWaves >= steps) break;
      if (s + 4 * kWaves < steps) load_a(s + 4 * kWaves, b1);
      multiply_step(b2);
    }
  }

  // ---- sum the four wavefronts in wave order, then write the partial block ------
  __syncthreads();
  float *red = lds;                                   // [M_T][J_T]
  for (int w = 0; w < kWaves; ++w) {
    if (wave == w) {
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < JT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = i * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            float *dst = red + m * J_T + t * 32 + l32;
            if (w == 0) *dst = acc[i][t][r];
            else *dst += acc[i][t][r];
          }
    }
    __syncthreads();
  }
  float *out = ws + (i64)blockIdx.x * wp.M_pad * wp.J_pad + (i64)m0 * wp.J_pad + j0;
  for (int e = tid; e < M_T * J_T; e += kThreads) {
    const int m = e / J_T, jj = e - m * J_T;
    out[(i64)m * wp.J_pad + jj] = red[e];
  }
}

// W[m, j] = sum over the S partial blocks, in index order.  A block of 256
// threads handles 16 outputs: 16 threads per output add every 16th partial,
// then thread 0 of each output adds the 16 sums in order.
template <typename O>                                  // O: float, or _Float16 (rounded once)
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float *__restrict__ ws,
                                                           O *__restrict__ W, int S, int M,
                                                           int J, int M_pad, int J_pad) {
  __shared__ float part[16][17];
  const int el = threadIdx.x & 15, ph = threadIdx.x >> 4;
  const int e = blockIdx.x * 16 + el;
  float sum = 0.f;
  if (e < M * J) {
    const int m = e / J, j = e - m * J;
    const float *src = ws + (i64)m * J_pad + j;
    const i64 stride = (i64)M_pad * J_pad;
    int s = ph;
    for (; s + 48 < S; s += 64) {
      const float v0 = src[(i64)s * stride], v1 = src[(i64)(s + 16) * stride];
      const float v2 = src[(i64)(s + 32) * stride], v3 = src[(i64)(s + 48) * stride];
      sum += v0; sum += v1; sum += v2; sum += v3;
    }
    for (; s < S; s += 16) sum += src[(i64)s * stride];
  }
  part[ph][el] = sum;
  __syncthreads();
  if (ph == 0 && e < M * J) {
    float tot = part[0][el];
#pragma unroll
    for (int k = 1; k < 16; ++k) tot += part[k][el];
    W[e] = (O)tot;
  }
}

template <int MT, int JT, int NT>
hipError_t launch_variant(const WgradPlan &wp, size_t lds_bytes, dim3 grid, const float *a,
                          const float *g, float *ws, hipStream_t stream) {
  auto kern = wgrad_gemm_kernel<MT, JT, NT>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, stream, wp, a, g, ws);
  return hipGetLastError();
}

template <int MT, int JT>
hipError_t launch_rows(const WgradPlan &wp, dim3 grid, const float *a, const float *g, float *ws,
                       hipStream_t stream) {
  auto kern = wgrad_rows_kernel<MT, JT>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, wp.lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), wp.lds_bytes, stream, wp, a, g, ws);
  return hipGetLastError();
}

template <int MT, int JT>
hipError_t launch_stream(const WgradPlan &wp, dim3 grid, const float *a, const float *g, float *ws,
                         hipStream_t stream) {
  auto kern = wgrad_stream_kernel<MT, JT>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, wp.lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), wp.lds_bytes, stream, wp, a, g, ws);
  return hipGetLastError();
}

}  // namespace

// Plan the weight gradient of the layer whose FORWARD problem is `fwd`
// (filter = weight, signal = input, output = grad_out, write mode).
static bool make_wgrad_plan_jt(const SepConv &fwd, WgradPlan &wp, bool g_allow_rows, int rows_opt_mt,
                               int rows_opt_nbuf, int rows_opt_rpw, int jt_max);

bool make_wgrad_plan(const SepConv &fwd_in, WgradPlan &wp, bool g_allow_rows, int rows_opt_mt, int rows_opt_nbuf,
                     int rows_opt_rpw) {
  // (the forward tiling is only borrowed for its staging geometry: plan it for the fp32 kernel)
  SepConv fwd = fwd_in;
  fwd.math = MATH_FP32;
  wp.split = fwd_in.math != MATH_FP32;
  // narrower column blocks touch fewer input channels and so need less LDS
  for (int jt_max = 3; jt_max >= 1; --jt_max)
    if (make_wgrad_plan_jt(fwd, wp, g_allow_rows, rows_opt_mt, rows_opt_nbuf, rows_opt_rpw, jt_max)) return true;
  return false;
}

static bool make_wgrad_plan_jt(const SepConv &fwd, WgradPlan &wp, bool g_allow_rows, int rows_opt_mt,
                               int rows_opt_nbuf, int rows_opt_rpw, int jt_max) {
  size_t lds_fwd;
  int mt, nt;
  // 128 positions per tile: the staged grad_out tile (channels x positions, two
  // buffers) is what fills LDS here
  if (!make_tile_plan(fwd, wp.t, &lds_fwd, &mt, &nt, 1)) return false;
  TilePlan &pl = wp.t;
  wp.J = pl.C * pl.nf;
  wp.mt = 1;
  wp.jt = std::min(jt_max, wp.J > 64 ? 3 : (wp.J > 32 ? 2 : 1));
  const int M_T = wp.mt * 32, J_T = wp.jt * 32;
  wp.m_groups = (pl.M + M_T - 1) / M_T;
  wp.j_groups = (wp.J + J_T - 1) / J_T;
  wp.M_pad = wp.m_groups * M_T;
  wp.J_pad = wp.j_groups * J_T;
  wp.a_n = (i64)pl.M * pl.Q;
  wp.a_m = pl.Q;
  // the forward plan fixed the position tiling (nt) and the row geometry
  wp.nt = nt;
  wp.rows_mode = 0;
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;
  // Rows of under eight outputs are three or four matrix steps long: on a linear x axis
  // the position-tile kernel, which does not care where rows end, is then the faster one
  // (rows of 5 and 7: 12 % and 25 %).  On a Mellin axis its tiles stage a virtual row per
  // (row, filter row) pair for only 128 positions and the row-wise kernel stays ahead.
  const int min_row = mellin_x ? 4 : 8;
  // (Linear x axis only: on a Mellin axis a unit's fragments cover a virtual row per (row,
  // filter row) pair, most of them without a tap, and the fp32 row-wise kernel measured
  // 10-65 % faster on the 64..256-channel layers of the 10-layer stack.)
  if (wp.split && !mellin_x && !pl.segment && pl.ay == 1 && pl.uy == 1 && pl.by == 1 && pl.nfy <= 8 && pl.noy >= 8 &&
      pl.nox_eff >= 1 && g_allow_rows && (i64)pl.M * pl.Q < ((i64)1 << 30)) {
    // The bf16 form (wgrad_stream_kernel): grad_out goes through registers, LDS holds the
    // fragments of the input rows a unit needs.  The largest unit whose fragment tasks a
    // workgroup's threads can hold (two each) and that still lets three workgroups share a
    // CU, else two.  All 64 channels in one workgroup where there are that many: the input
    // fragments are then made once for twice the products.
    const int NG = (pl.noy + 7) / 8;
    const int mt_s = (pl.M > 32 && rows_opt_mt != 1) ? 2 : 1;
    const int m_groups = (pl.M + mt_s * 32 - 1) / (mt_s * 32);
    const int ccj = std::min(pl.C, (J_T - 1 + pl.nf - 1) / pl.nf + 1);
    const int blocks_y = m_groups * wp.j_groups;
    for (int pass = 0; pass < 2 && !wp.rows_mode; ++pass)
      for (int rpw = rows_opt_rpw > 0 ? rows_opt_rpw : 4; rpw >= 1; --rpw) {
        const int rb = kWaves * rpw;
        const i64 Rr = mellin_x ? (i64)rb * pl.nfx : (i64)pl.ax * (rb - 1) + pl.bx_span + 1;
        const i64 tasks = (i64)ccj * Rr * NG;
        const size_t bytes = std::max((size_t)48 * (tasks * pl.nfy + 1) + 8 * (size_t)(rb * NG + 2),
                                      4 * (size_t)mt_s * 32 * J_T);
        if (Rr > 8192 || tasks > 2 * kThreads) continue;
        const int cap = mt_s == 2 ? 2 : 3;                 // registers
        if (bytes > (size_t)(pass == 0 && cap == 3 ? 52 : 78) * 1024) { if (rows_opt_rpw > 0) break; continue; }
        const int per_cu = std::max(1, std::min((int)((160 * 1024) / (bytes + 512)), cap));
        const i64 units = (i64)pl.batch * ((pl.nox_eff + rb - 1) / rb);
        const i64 S = std::min<i64>(std::max<i64>(1, (256 * per_cu) / blocks_y), units);
        wp.rows_mode = 2;
        pl.R = (int)Rr;
        wp.CCj = ccj;
        wp.lds_bytes = bytes;
        wp.nbuf = 1;
        wp.rpw = rpw;
        wp.mt = mt_s;
        wp.m_groups = m_groups;
        wp.M_pad = m_groups * mt_s * 32;
        wp.S = (int)S;
        wp.ws_bytes = (size_t)wp.S * wp.M_pad * wp.J_pad * sizeof(float);
        break;
      }
    if (wp.rows_mode) return true;
  }
  if (!pl.segment && pl.ay == 1 && pl.noy >= min_row && pl.nox_eff >= 1 && g_allow_rows) {
    // Row-wise variant: units of kWaves * rpw output rows, about 300 positions per
    // unit (two rows of 38 per wavefront, sixteen rows of 5).
    const int ccj = std::min(pl.C, (J_T - 1 + pl.nf - 1) / pl.nf + 1);
    const int rpw_auto = std::max(2, std::min(16, (76 + pl.noy - 1) / pl.noy));
    // Candidate shapes {rows per wavefront, buffers}: the largest unit with a single
    // buffer first (several workgroups per CU cover each other's loads), then smaller
    // units, which need less LDS.  Every workgroup lives for the whole launch, so what counts
    // is how evenly S * blocks fill the chip: the CU that gets the most workgroups sets
    // the time, and a CU runs k workgroups at eff[k] of its full rate.
    int shapes[32][2], n_shapes = 0;
    for (int r = rpw_auto; r >= 1; --r) {
      shapes[n_shapes][0] = r; shapes[n_shapes++][1] = 1;
      shapes[n_shapes][0] = r; shapes[n_shapes++][1] = 2;
    }
    static const double eff[7] = {0, 0.45, 0.79, 1.0, 1.0, 1.0, 1.0};   // fitted to measured layers
    const int vgpr_cap = wp.jt == 3 ? 3 : (wp.jt == 2 ? 4 : 5);   // wavefronts per SIMD the registers allow
    double best = 0;
    for (int si = 0; si < n_shapes; ++si) {
      const int *shape = shapes[si];
      const int rpw = rows_opt_rpw > 0 ? rows_opt_rpw : shape[0];
      const int nbuf = rows_opt_nbuf > 0 ? rows_opt_nbuf : shape[1];
      const int rb = kWaves * rpw;
      const i64 Rr = mellin_x ? (i64)rb * pl.nfx : (i64)pl.ax * (rb - 1) + pl.bx_span + 1;
      int pitch = (rb * pl.noy + 3) & ~3;
      if (((pitch >> 2) & 1) == 0) pitch += 4;            // 4 x odd: channels spread over the banks
      const size_t xw = ((size_t)ccj * Rr * pl.RS + 3) & ~(size_t)3;
      // all channels in one workgroup (two 32-row tiles) only on request: fewer, fatter
      // workgroups have measured slower
      int mt_rows = (pl.M > 32 && rows_opt_mt == 2) ? 2 : 1;
      // (the second term: two slabs of sums at the end)
      size_t bytes = 4 * std::max(nbuf * (xw + (size_t)mt_rows * 32 * pitch), 2 * (size_t)mt_rows * 32 * J_T);
      if (mt_rows == 2 && bytes > 150 * 1024) {
        mt_rows = 1;
        bytes = 4 * std::max(nbuf * (xw + (size_t)32 * pitch), 2 * (size_t)32 * J_T);
      }
      if (Rr > 8192 || pitch * 32 * 4 >= 65536 || bytes > (mt_rows == 2 ? 150 : 78) * 1024) continue;
      const int m_groups = (pl.M + mt_rows * 32 - 1) / (mt_rows * 32);
      const int blocks_y_rows = m_groups * wp.j_groups;
      const i64 units = (i64)pl.batch * ((pl.nox_eff + rb - 1) / rb);
      const int per_cu = std::max(1, std::min((int)((160 * 1024) / (bytes + 512)), mt_rows == 2 ? 2 : vgpr_cap));
      // S for every number k of workgroups per CU that fits; rate = work done per unit time
      for (int k = per_cu; k >= 1; --k) {
        i64 S = std::min<i64>(std::max<i64>(1, (256 * k) / blocks_y_rows), units);
        const i64 total = S * blocks_y_rows;
        const i64 rounds = (total + 256 * per_cu - 1) / (256 * per_cu);      // > 1 only when S == 1 cannot fit at once
        const int kmax = (int)std::min<i64>(per_cu, (total + 255) / 256);
        // small units pay their set-up more often; a second buffer hides the loads
        const double unit = 1.0 + 40.0 / (rpw * pl.noy) + (nbuf == 2 ? -0.07 : 0.0);
        const double rate = (double)total / rounds * eff[kmax] / kmax / unit;
        if (rate <= best * 1.01) continue;                // earlier candidates win ties
        best = rate;
        wp.rows_mode = 1;
        pl.R = (int)Rr;
        wp.GSS = pitch;
        wp.CCj = ccj;
        wp.lds_bytes = bytes;
        wp.nbuf = nbuf;
        wp.rpw = rpw;
        wp.mt = mt_rows;
        wp.m_groups = m_groups;
        wp.M_pad = wp.m_groups * mt_rows * 32;
        wp.S = (int)S;
        wp.ws_bytes = (size_t)wp.S * wp.M_pad * wp.J_pad * sizeof(float);
      }
      if (rows_opt_rpw > 0 && rows_opt_nbuf > 0) break;   // a forced shape: nothing else to try
    }
    if (wp.rows_mode) return true;
  }
  const int P = kWaves * nt * 32;
  wp.GSS = P + 1;
  wp.CCj = std::min(pl.C, (J_T - 1 + pl.nf - 1) / pl.nf + 1);
  const size_t words = 2 * (size_t)wp.CCj * pl.R * pl.RS + 2 * (size_t)M_T * wp.GSS + 2 * (size_t)P;
  const size_t red_words = (size_t)M_T * J_T;
  wp.lds_bytes = 4 * std::max(words, red_words);
  if (wp.lds_bytes > 96 * 1024) return false;
  // position shares: persistent workgroups, at most three per CU (registers) over all output blocks
  const int blocks_y = wp.m_groups * wp.j_groups;
  int per_cu = (int)((160 * 1024) / (wp.lds_bytes + 512));
  per_cu = std::max(1, std::min(per_cu, 3));
  int S = std::max(1, (256 * per_cu) / blocks_y);
  S = std::min(S, pl.total_tiles);
  wp.S = S;
  wp.ws_bytes = (size_t)S * wp.M_pad * wp.J_pad * sizeof(float);
  return true;
}

hipError_t launch_wgrad(const WgradPlan &wp, const float *grad_out, const float *input,
                        float *grad_weight, float *workspace, hipStream_t stream) {
  dim3 grid((unsigned)wp.S, (unsigned)(wp.m_groups * wp.j_groups));
  hipError_t e = hipErrorInvalidValue;
  if (wp.rows_mode == 2) {
#define MELLIN_STREAM_CASE(MT_, JT_)                                                       \
  if (wp.mt == MT_ && wp.jt == JT_) e = launch_stream<MT_, JT_>(wp, grid, grad_out, input, workspace, stream);
    MELLIN_STREAM_CASE(1, 1) MELLIN_STREAM_CASE(1, 2) MELLIN_STREAM_CASE(1, 3)
    MELLIN_STREAM_CASE(2, 1) MELLIN_STREAM_CASE(2, 2) MELLIN_STREAM_CASE(2, 3)
#undef MELLIN_STREAM_CASE
  } else if (wp.rows_mode) {
#define MELLIN_ROWS_CASE(MT_, JT_)                                                         \
  if (wp.mt == MT_ && wp.jt == JT_) e = launch_rows<MT_, JT_>(wp, grid, grad_out, input, workspace, stream);
    MELLIN_ROWS_CASE(1, 1) MELLIN_ROWS_CASE(1, 2) MELLIN_ROWS_CASE(1, 3)
    MELLIN_ROWS_CASE(2, 1) MELLIN_ROWS_CASE(2, 2) MELLIN_ROWS_CASE(2, 3)
#undef MELLIN_ROWS_CASE
  } else {
#define MELLIN_WGRAD_CASE(MT_, JT_, NT_)                                                   \
  if (wp.mt == MT_ && wp.jt == JT_ && wp.nt == NT_)                                          \
    e = launch_variant<MT_, JT_, NT_>(wp, wp.lds_bytes, grid, grad_out, input, workspace, stream);
  MELLIN_WGRAD_CASE(1, 3, 1)
  MELLIN_WGRAD_CASE(1, 2, 1)
  MELLIN_WGRAD_CASE(1, 1, 1)
#undef MELLIN_WGRAD_CASE
  }
  if (e != hipSuccess) return e;
  const int outputs = wp.t.M * wp.J;
  hipLaunchKernelGGL(wgrad_reduce_kernel<float>, dim3((unsigned)((outputs + 15) / 16)), dim3(256), 0, stream,
                     (const float *)workspace, grad_weight, wp.S, wp.t.M, wp.J, wp.M_pad, wp.J_pad);
  return hipGetLastError();
}

hipError_t launch_wgrad_reduce(const float *partials_ws, void *W, bool half_out, int partials, int M, int J,
                               int M_pad, int J_pad, hipStream_t stream) {
  const dim3 grid((unsigned)((M * J + 15) / 16));
  if (half_out)
    hipLaunchKernelGGL(wgrad_reduce_kernel<_Float16>, grid, dim3(256), 0, stream, partials_ws, (_Float16 *)W,
                       partials, M, J, M_pad, J_pad);
  else
    hipLaunchKernelGGL(wgrad_reduce_kernel<float>, grid, dim3(256), 0, stream, partials_ws, (float *)W, partials,
                       M, J, M_pad, J_pad);
  return hipGetLastError();
}

}  // namespace mellin
