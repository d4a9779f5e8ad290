// Gather-GEMM on the fp32 matrix cores (v_mfma_f32_32x32x2_f32).
//
//   H[n, m, ox, oy] = bias[m] + sum_{c, fx, fy} F[m, c, fx, fy] *
//                     G[n, c, tap_x(ox, fx), tap_y(oy, fy)]
//
// is computed per workgroup as a (M_T x K) * (K x P) product, K = (c, fx, fy),
// over P consecutive output positions of one image.  All the irregular work
// happens while the operands are staged in LDS:
//
//   * the signal rows a tile needs are copied into "virtual rows" whose
//     position is an AFFINE function of (output row, filter row):
//       Mellin axis  row = (ox - ox_lo) * nfx + fx, holding signal row
//                    tap_x(ox, fx) or zeros if that tap does not exist;
//       linear axis  row = ax * ox + bx * fx + cx - min, holding the signal row
//                    at that (zero-stuffed, zero-padded) coordinate;
//     columns are laid out the same way along y, so zero padding, stride,
//     dilation, up-sampling and the divisibility rule never reach the inner
//     loop: there the B operand of lane (position j) for tap k is one LDS
//     word at  lane_base[j] + tap_offset[k];
//   * the filter block is stored channel-major with an odd row stride so that
//     the A operand of lane (channel i) is one LDS word and the 32 channels of
//     a half-wave fall in 32 different banks.
//
// Staging uses the direct global->LDS loads of gfx950 (no VGPR round trip):
// a wavefront issues one load per virtual row, 64 columns wide, and writes
// zeros for the columns or rows that have no source.  The loads of stage i+1
// are issued before the matrix-core loop of stage i (two LDS buffers), so a
// persistent workgroup needs one barrier per stage and global latency hides
// behind the multiplies.  A stage is one (tile, channel chunk) pair.
//
// One wavefront owns all M_T output channels of NT * 32 positions and keeps
// MT * NT accumulator tiles (16 registers each).  Stores write 128-byte runs
// of one output row.
#include <algorithm>

#include "mellin_common.hpp"
#include "tile_gemm.hpp"
#include "tile_stage.hpp"

namespace mellin {

namespace {

#ifndef MELLIN_STAMP
#define MELLIN_STAMP(i)
#define MELLIN_PROBE_DECL
#endif

template <int MT, int NT, bool ACC>
__global__ __launch_bounds__(kThreads, 2) void tile_gemm_kernel(
    TilePlan pl, const float *__restrict__ F, const float *__restrict__ G,
    const float *__restrict__ bias, float *__restrict__ H) {
  extern __shared__ float lds[];
  constexpr int M_T = MT * 32;
  constexpr int P = kWaves * NT * 32;
  constexpr int GS = 4;                              // tap pairs per operand group
  const int g_words = pl.CC * pl.R * pl.RS;          // one signal buffer
  const int w_words = M_T * pl.WSS;                  // one filter buffer
  float *Gs0 = lds;                                  // [2][CC][R][RS]
  float *Ws0 = Gs0 + 2 * g_words;                    // [1 or 2][M_T][WSS]
  const bool single_chunk = pl.CC >= pl.C;
  int *tapoff = (int *)(Ws0 + (single_chunk ? 1 : 2) * w_words);   // [KCp]
  float *Bs = (float *)(tapoff + pl.KCp);            // [M_T] bias (zeros when accumulating)

  MELLIN_PROBE_DECL
  const int tid = threadIdx.x;
  // the wave index is wave-uniform: say so, and everything derived from it (row
  // loops, base addresses) is computed on the scalar unit
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const int m0 = blockIdx.y * M_T;
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;
  const int chunks = (pl.C + pl.CC - 1) / pl.CC;

  // ---- filter block: Ws[m][k], k = cl * nf + t, row stride WSS (odd) --------------
  // one direct load per (m, 64 taps): lane k fetches F[m0 + m, c0 + cl, t], coalesced
  // along the taps; taps past the chunk and channels past M are zero
  const unsigned lds_base = lds_address(lds);
  auto issue_filter = [&](int c0, int cc, int ws_word) {        // ws_word: where the block starts in lds[]
    const int KC = cc * pl.nf;
    const FastDiv by_nf(pl.nf);
    const int m_live = max(0, min(M_T, pl.M - m0));       // channels of this block that exist
    for (int kb = 0; kb < pl.KCp; kb += 64) {
      const int k = kb + lane;
      int cl, t;
      by_nf.divmod(k, cl, t);
      const unsigned voff = (unsigned)(((i64)(c0 + cl) * pl.f_c + t) * 4);   // < 4 GB: checked by the plan
      if (k < KC) {
        for (int m = wave; m < m_live; m += kWaves)
          load_to_lds_at(F + (i64)(m0 + m) * pl.f_m, voff, lds_base + 4u * (unsigned)(ws_word + m * pl.WSS + kb));
        for (int m = m_live + wave; m < M_T; m += kWaves) lds[ws_word + m * pl.WSS + k] = 0.f;
      } else if (k < pl.KCp) {
        for (int m = wave; m < M_T; m += kWaves) lds[ws_word + m * pl.WSS + k] = 0.f;
      }
    }
  };

  // ---- stages owned by this workgroup ------------------------------------------
  // tiles blockIdx.x, blockIdx.x + gridDim.x, ...; each tile has `chunks` stages
  const int my_tiles = (int)blockIdx.x < pl.total_tiles
                           ? (pl.total_tiles - 1 - (int)blockIdx.x) / (int)gridDim.x + 1 : 0;
  const int my_stages = my_tiles * chunks;
  auto issue_stage = [&](int st) {
    const int ti = st / chunks, ch = st - ti * chunks;
    const TileGeom tg = tile_geometry<P>(pl, blockIdx.x + ti * gridDim.x, mellin_x);
    const int c0 = ch * pl.CC, cc = min(pl.CC, pl.C - c0);
    issue_signal(pl, tg, G, c0, cc, Gs0 + (st & 1) * g_words, lds_base + 4u * (unsigned)((st & 1) * g_words),
                 mellin_x, lane, wave);
    if (!single_chunk) issue_filter(c0, cc, 2 * g_words + (st & 1) * w_words);
  };

  {
    const FastDiv by_nf(pl.nf), by_nfy(pl.nfy);
    for (int k = tid; k < pl.KCp; k += kThreads) {
      int cl, t, fx, fy;
      by_nf.divmod(k, cl, t);
      by_nfy.divmod(t, fx, fy);
      tapoff[k] = cl * pl.R * pl.RS + pl.Bx * fx * pl.RS + pl.by * fy;
    }
    for (int m = tid; m < M_T; m += kThreads)
      Bs[m] = (!ACC && bias && m0 + m < pl.M) ? bias[m0 + m] : 0.f;
  }
  MELLIN_STAMP(0);
  if (my_stages > 0) {
    if (single_chunk) issue_filter(0, pl.C, 2 * g_words);
    issue_stage(0);
  }
  MELLIN_STAMP(1);

  const FastDiv by_noy(pl.noy);
  floatx16 acc[MT][NT];
  int lane_base[NT], lane_q[NT];
  TileGeom tg;

  // ---- epilogue: 32 consecutive lanes write 32 consecutive positions of one
  // channel.  It runs one stage late (after the next stage's loads are issued,
  // before its multiplies) so that the stores drain behind the next matrix
  // loop instead of holding up the wait for those loads.
  auto epilogue = [&]() {
    float *Hq = H + (i64)tg.n * pl.h_n + (i64)(m0 + half * 4) * pl.h_m;
    const int m_left = pl.M - m0 - half * 4;              // channels from this lane's first row on
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int local = (wave * NT + t) * 32 + l32;
      bool live = local < tg.count;
      if (ACC) {
        int ox, oy;
        by_noy.divmod(lane_q[t], ox, oy);
        live = live && ox < pl.nox_eff && oy < pl.noy_eff;
      }
      if (!live) continue;
      float *Ht = Hq + lane_q[t];
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int mo = i * 32 + (r >> 2) * 8 + (r & 3);
          if (mo < m_left) {
            float *dst = Ht + (i64)mo * pl.h_m;
            if (ACC) *dst += acc[i][t][r];
            else *dst = acc[i][t][r];
          }
        }
    }
  };

  for (int st = 0; st < my_stages; ++st) {
    const int ti = st / chunks, ch = st - ti * chunks;
    // every wave's loads for this stage have landed, and every wave is done
    // reading the buffer the next stage will fill
    wait_all_memory();
    MELLIN_STAMP(2);
    __syncthreads();
    MELLIN_STAMP(3);
    if (st + 1 < my_stages) { MELLIN_STAMP(7); issue_stage(st + 1); MELLIN_STAMP(8); }
    MELLIN_STAMP(4);

    if (ch == 0) {
      if (st > 0) epilogue();                             // the tile finished one stage ago
      MELLIN_STAMP(5);
      tg = tile_geometry<P>(pl, blockIdx.x + ti * gridDim.x, mellin_x);
      // position -> LDS word of its (fx = 0, fy = 0) tap
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        int local = (wave * NT + t) * 32 + l32;
        if (local >= tg.count) local = 0;                 // masked lane: any valid position
        const int q = tg.q0 + local;
        int ox, oy;
        by_noy.divmod(q, ox, oy);
        lane_q[t] = q;
        lane_base[t] = (pl.Ax * (ox - tg.ox_lo) + pl.Cx0) * pl.RS + pl.ay * (oy - tg.oy_lo) - pl.by_min;
      }
      // accumulators start from the bias of the channel each register holds
#pragma unroll
      for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const float4 bv = *(const float4 *)(Bs + a * 32 + g4 * 8 + half * 4);
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            acc[a][t][4 * g4 + 0] = bv.x; acc[a][t][4 * g4 + 1] = bv.y;
            acc[a][t][4 * g4 + 2] = bv.z; acc[a][t][4 * g4 + 3] = bv.w;
          }
        }
    }

    // ---- matrix-core loop over tap pairs: operands of the next group of GS
    // pairs are fetched from LDS while the current group multiplies
    {
      const int cc = min(pl.CC, pl.C - ch * pl.CC);
      const int KC = cc * pl.nf;
      const int steps = (KC + 1) >> 1;
      const float *Gs = Gs0 + (st & 1) * g_words;
      const float *wa = Ws0 + (single_chunk ? 0 : (st & 1) * w_words) + l32 * pl.WSS + half;
      const int *tp = tapoff + half;
      const int wrow = 32 * pl.WSS;                        // next 32 channels
      const int full = (KC & 1) ? steps - 1 : steps;       // steps whose two taps both exist
      const int groups = full / GS;
      float a0[GS][MT], b0[GS][NT], a1[GS][MT], b1[GS][NT];
      auto fetch = [&](int g, float (&a)[GS][MT], float (&b)[GS][NT]) {
        int off[GS];
#pragma unroll
        for (int j = 0; j < GS; ++j) off[j] = tp[2 * (g * GS + j)];
#pragma unroll
        for (int j = 0; j < GS; ++j) {
#pragma unroll
          for (int i = 0; i < MT; ++i) a[j][i] = wa[2 * (g * GS + j) + i * wrow];
#pragma unroll
          for (int t = 0; t < NT; ++t) b[j][t] = Gs[lane_base[t] + off[j]];
        }
      };
      auto multiply = [&](float (&a)[GS][MT], float (&b)[GS][NT]) {
#pragma unroll
        for (int j = 0; j < GS; ++j)
#pragma unroll
          for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int t = 0; t < NT; ++t)
              acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j][i], b[j][t], acc[i][t], 0, 0, 0);
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
        const int off = tp[2 * s];
        float a[MT], b[NT];
#pragma unroll
        for (int i = 0; i < MT; ++i) a[i] = wa[2 * s + i * wrow];
#pragma unroll
        for (int t = 0; t < NT; ++t) b[t] = (s >= full && half) ? 0.f : Gs[lane_base[t] + off];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[t], acc[i][t], 0, 0, 0);
      }
    }
    MELLIN_STAMP(6);
  }
  if (my_stages > 0) epilogue();
  MELLIN_STAMP(9);
}

template <int MT, int NT, bool ACC>
hipError_t launch_variant(const TilePlan &pl, size_t lds_bytes, dim3 grid, const float *f,
                          const float *g, const float *bias, float *h, hipStream_t stream) {
  auto kern = tile_gemm_kernel<MT, NT, ACC>;
  if (lds_bytes > 64 * 1024) {
    // opt in to more than the default 64 KB of dynamic LDS (gfx950 has 160 KB per CU)
    static thread_local size_t granted = 0;
    if (granted < lds_bytes) {
      hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds_bytes);
      if (e != hipSuccess) return e;
      granted = lds_bytes;
    }
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, stream, pl, f, g, bias, h);
  return hipGetLastError();
}

}  // namespace

// Fill `pl` for the problem `pr`; returns false when the tiled kernel does not
// apply (sizes beyond 32-bit indexing or a single channel not fitting in LDS).
bool make_tile_plan(const SepConv &pr, TilePlan &pl, size_t *lds_bytes, int *mt, int *nt, int force_nt) {
  const i64 lim = (i64)1 << 30;
  const i64 nf = pr.x.nf * pr.y.nf, ng = pr.x.ng * pr.y.ng, Q = pr.x.nh * pr.y.nh;
  if (nf <= 0 || ng <= 0 || Q <= 0 || pr.c_in <= 0 || pr.c_out <= 0 || pr.batch <= 0) return false;
  if (nf > 4096 || ng >= lim || Q >= lim || pr.c_in >= lim || pr.c_out >= lim || pr.batch >= lim) return false;
  if (pr.c_in * ng >= lim * 2 || pr.batch * (Q / 64 + 1) >= lim) return false;
  const Axis &X = pr.x, &Y = pr.y;
  if (Y.kind != AX_LCORR && Y.kind != AX_LCONV) return false;
  if (X.s > 4096 || X.d > 4096 || X.u > 4096 || X.p > 4096 || Y.s > 64 || Y.d > 4096 || Y.u > 64) return false;
  if (Y.p > lim || Y.p < -lim || X.p < -lim) return false;

  pl.batch = (int)pr.batch; pl.M = (int)pr.c_out; pl.C = (int)pr.c_in;
  pl.nfx = (int)X.nf; pl.nfy = (int)Y.nf; pl.nf = (int)nf;
  pl.ngx = (int)X.ng; pl.ngy = (int)Y.ng; pl.nox = (int)X.nh; pl.noy = (int)Y.nh; pl.Q = (int)Q;
  pl.nox_eff = (int)X.nh_eff; pl.noy_eff = (int)Y.nh_eff;
  pl.f_m = pr.f_m; pl.f_c = pr.f_c; pl.g_n = pr.g_n; pl.g_c = pr.g_c; pl.h_n = pr.h_n; pl.h_m = pr.h_m;
  pl.accumulate = pr.accumulate;
  pl.kind_x = X.kind; pl.sx = (int)X.s; pl.dx = (int)X.d; pl.px = (int)X.p; pl.ux = (int)X.u;
  pl.uy = (int)Y.u;

  *mt = pr.c_out > 32 ? 2 : 1;
  const int M_T = *mt * 32;
  const i64 m_tiles = (pr.c_out + M_T - 1) / M_T;
  // two N tiles per wavefront once that still leaves every CU several tiles
  *nt = (pr.batch * ((Q + 255) / 256) * m_tiles >= 4 * 256) ? 2 : 1;
  if (force_nt) *nt = force_nt;
  const int P = kWaves * (*nt) * 32;

  // y axis: column = ay * oy + by * fy + cy - min
  pl.ay = (int)Y.s;
  pl.by = Y.kind == AX_LCORR ? (int)Y.d : -(int)Y.d;
  pl.cy = Y.kind == AX_LCORR ? -(int)Y.p : (int)Y.p;
  const i64 by_ext = (i64)pl.by * (pl.nfy - 1);
  pl.by_min = (int)(by_ext < 0 ? by_ext : 0);
  pl.by_span = (int)(by_ext < 0 ? -by_ext : by_ext);

  // tiling of the flattened (ox, oy) positions
  pl.segment = pl.noy > P;
  pl.chunks_per_row = (pl.noy + P - 1) / P;
  pl.tiles_per_image = pl.segment ? pl.nox * pl.chunks_per_row : (pl.Q + P - 1) / P;
  pl.total_tiles = pl.batch * pl.tiles_per_image;
  const int RT = pl.segment ? 1 : std::min(pl.nox, (P - 1 + pl.noy - 1) / pl.noy + 1);
  const int oy_span = pl.segment ? P : pl.noy;
  const i64 RSL = (i64)pl.ay * (oy_span - 1) + pl.by_span + 1;

  // x axis
  const bool mellin_x = X.kind == AX_MCORR || X.kind == AX_MCONV;
  i64 R;
  if (mellin_x) {
    pl.ax = 0; pl.bx = 0; pl.cx = 0; pl.bx_min = 0; pl.bx_span = 0;
    pl.Ax = pl.nfx; pl.Bx = 1; pl.Cx0 = 0;
    R = (i64)RT * pl.nfx;
  } else {
    pl.ax = (int)X.s;
    pl.bx = X.kind == AX_LCORR ? (int)X.d : -(int)X.d;
    pl.cx = X.kind == AX_LCORR ? -(int)X.p : (int)X.p;
    const i64 bx_ext = (i64)pl.bx * (pl.nfx - 1);
    pl.bx_min = (int)(bx_ext < 0 ? bx_ext : 0);
    pl.bx_span = (int)(bx_ext < 0 ? -bx_ext : bx_ext);
    pl.Ax = pl.ax; pl.Bx = pl.bx; pl.Cx0 = -pl.bx_min;
    R = (i64)pl.ax * (RT - 1) + pl.bx_span + 1;
  }
  if (RSL > 8192 || R > 8192) return false;
  if (mellin_x) {
    // 32-bit tap arithmetic: (h + s)(f + d) and (p + 1)(h + s) must fit
    const i64 hmax = X.nh + X.s, fmax = X.nf + X.d;
    if (hmax * fmax >= lim || (X.p + 1) * hmax >= lim) return false;
  }
  if (Q >= ((i64)1 << 22) || pr.c_in * ng >= lim) return false;   // float-reciprocal index splits
  if (pr.c_in * pr.f_c + nf >= lim || pr.f_c < 0 || pr.f_m < 0) return false;   // 32-bit byte offsets into the filter
  pl.R = (int)R;
  pl.RS = (int)RSL | 1;                                            // odd stride spreads LDS banks
  // Linear axes without up-sampling or left padding, tiles spanning whole rows
  // that use every signal column: a virtual row is a signal row.  Give it the
  // signal's pitch, and a tile's rows are one contiguous run per channel.
  pl.contig = !mellin_x && !pl.segment && pl.ux == 1 && pl.uy == 1 && pl.cy + pl.by_min == 0 &&
              RSL <= pl.ngy && pl.ngy <= RSL + 8;
  if (pl.contig) pl.RS = pl.ngy;


  // channels per chunk from the LDS budget: two signal buffers, and two
  // filter buffers unless every channel fits in one chunk
  const i64 budget_words = (72 * 1024) / 4;
  const i64 fixed = M_T + 16;
  const i64 g_per_c = (i64)pl.R * pl.RS, w_per_c = (i64)pl.nf * M_T, t_per_c = pl.nf;
  i64 cc;
  if (2 * g_per_c * pl.C + w_per_c * pl.C + 3 * M_T + t_per_c * pl.C + 2 + fixed <= budget_words) {
    cc = pl.C;
  } else {
    cc = (budget_words - fixed - 6 * M_T - 2) / (2 * g_per_c + 2 * w_per_c + t_per_c);
    if (cc < 1) return false;
    if (cc > pl.C) cc = pl.C;
    if (cc > 64) cc = 64;
  }
  if (cc * pl.R >= ((i64)1 << 22)) return false;
  pl.CC = (int)cc;
  pl.KCp = ((pl.CC * pl.nf + 1) / 2) * 2;
  pl.WSS = pl.KCp + 1;                                             // odd: 32 channels -> 32 banks
  const bool single = pl.CC >= pl.C;
  *lds_bytes = 4 * (2 * (size_t)pl.CC * pl.R * pl.RS + (single ? 1 : 2) * (size_t)M_T * pl.WSS +
                    pl.KCp + M_T);
  return *lds_bytes <= 76 * 1024;
}

hipError_t launch_tile_gemm(const TilePlan &pl, size_t lds_bytes, int mt, int nt,
                            const float *f, const float *g, const float *bias,
                            float *h, hipStream_t stream) {
  const int M_T = mt * 32;
  // persistent workgroups: as many as fit at once (by LDS, two per CU at most) on the 256 CUs
  const int m_tiles = (pl.M + M_T - 1) / M_T;
  int per_cu = (int)((160 * 1024) / (lds_bytes + 512));
  per_cu = std::max(1, std::min(per_cu, nt == 2 ? 3 : 4));
  int gx = std::max(1, (256 * per_cu) / m_tiles);
  gx = std::min(gx, pl.total_tiles);
  dim3 grid((unsigned)gx, (unsigned)m_tiles);
#define MELLIN_TILE_CASE(MT_, NT_)                                                           \
  if (mt == MT_ && nt == NT_)                                                                \
    return pl.accumulate ? launch_variant<MT_, NT_, true>(pl, lds_bytes, grid, f, g, bias, h, stream) \
                         : launch_variant<MT_, NT_, false>(pl, lds_bytes, grid, f, g, bias, h, stream);
  MELLIN_TILE_CASE(2, 2)
  MELLIN_TILE_CASE(2, 1)
  MELLIN_TILE_CASE(1, 2)
  MELLIN_TILE_CASE(1, 1)
#undef MELLIN_TILE_CASE
  return hipErrorInvalidValue;
}

}  // namespace mellin
