// Forward pass of a linear x linear layer with few input channels on the bf16 matrix cores:
// the benchmark's "lconv2d" shape class, with everything per tile that is not a matrix
// instruction or a store cut to what this class needs.
//
//   H[n, m, ox, oy] = bias[m] + sum_{c, fx, fy} F[m, c, fx, fy] * G[n, c, sx ox + dx fx, oy + fy]
//
// (both axes correlations without padding or up-sampling, unit stride and dilation along y,
// an even number of filter columns, c_in * nfx * nfy <= 128: one chunk of taps).  The product
// is the tiled kernel's: a workgroup of four wavefronts owns 256 consecutive flattened output
// positions of one image and 64 output channels, a wavefront 64 positions of all of them
// (2 x 2 tiles of 32 x 32, 64 accumulator registers).  What differs:
//
//   * the rows a tile reads are ONE contiguous run per input channel (R signal rows as they
//     lie).  Every thread loads eight of these words and their right-hand neighbours into
//     registers one tile ahead, and turns them into "pair words": element e -> three 32-bit
//     words (hi, mid, lo), word `part` holding the bf16 part of x[e] in its low half and of
//     x[e + 1] in its high half.  The eight taps a lane feeds to one matrix instruction are
//     four pairs of neighbouring columns, so the multiply loop reads its operands ready-made
//     (the LDS words of a pair through one address) and spends no vector instructions on
//     them, where the tiled kernel cuts every operand in the loop (44 vector instructions
//     per 16 taps and position tile);
//   * the pair words of two tiles are resident, so one barrier per tile is enough, and no
//     wave ever waits for its stores: a tile's order is  barrier | multiply | cut the next
//     tile's words | a quarter of the stores | request the words of the tile after the next |
//     the other stores.  The request lies behind a quarter of the stores so that the wait
//     for it (vmcnt counts loads and stores in order, 63 at most) leaves the later 48 stores
//     in flight: they drain under the next tile's matrix instructions;
//   * every size the loop needs is a kernel argument held in scalar registers, and the
//     position arithmetic uses multiply-high by precomputed reciprocals;
//   * a channel's two 32-position pieces go out back to back (see tile_gemm.hip).
#include <algorithm>
#include <atomic>
#include <type_traits>

#include "mellin_common.hpp"
#include "narrow_gemm.hpp"
#include "tile_stage.hpp"

namespace mellin {

namespace {

constexpr int kConvert = 8;                        // words a thread cuts per tile (at most 256 * 8 staged elements)
constexpr int kDeadOffset = 0x7FFFFFF0;            // past every buffer range: loads give 0, stores are dropped
constexpr int kRaw = 0x00020000;                   // buffer descriptor word 3: raw 32-bit accesses

// STEPS: matrix steps of 16 taps (K16 / 16); MT: 32-channel tiles per workgroup (1 or 2)
template <int MT, int STEPS>
__global__ __launch_bounds__(kThreads, 2) void narrow_forward_kernel(
    const NarrowPlan np, const float *__restrict__ F, const float *__restrict__ G,
    const float *__restrict__ bias, float *__restrict__ H) {
  extern __shared__ __align__(16) float lds[];
  constexpr int NT = 2, M_T = MT * 32, P = kWaves * NT * 32;
  constexpr int K16 = STEPS * 16, groups = K16 >> 3;
  // LDS: fragments [3][groups][M_T] x 16 B | bias [M_T] | pair offsets [K16 / 2] | pair words of two tiles, [part][element]
  uintx4 *const frag = (uintx4 *)lds;
  float *const bias_s = lds + 12 * groups * M_T;
  int *const pairoff = (int *)(bias_s + M_T);
  char *const sig0 = (char *)(pairoff + (K16 >> 1));
  const int sig_bytes = np.sig_bytes, plane = np.plane_bytes;
  const int n_elem = np.n_elem;                          // C * R * ngy

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const int m0 = blockIdx.y * M_T;
  const int bx = blockIdx.x, gx = gridDim.x;
  const int my_tiles = bx < np.total_tiles ? (np.total_tiles - 1 - bx) / gx + 1 : 0;
  if (my_tiles == 0) return;
  const int K = np.K, ngy = np.ngy, noy = np.noy, chan_words = np.R * ngy;
  const int m_live = min(M_T, np.M - m0);

  struct Tile { int n, q0, count, ox_lo; };
  auto tile_of = [&](int tile_id) {
    Tile t;
    t.n = udiv(tile_id, np.tiles_per_image, np.mg_tpi);
    t.q0 = (tile_id - t.n * np.tiles_per_image) * P;
    t.count = min(P, np.Q - t.q0);
    t.ox_lo = udiv(t.q0, noy, np.mg_noy);
    return t;
  };
  // Element e = tid + 256 i of a tile's window is word (e mod chan_words) of channel e / chan_words, counted
  // from the tile's first row: the same byte offset for every tile.  Words past the image read as 0 (the
  // descriptor's range); words of rows the tile does not use are read and never looked at.
  int voff[kConvert];
#pragma unroll
  for (int i = 0; i < kConvert; ++i) {
    const int e = tid + i * kThreads, cl = (int)__umulhi((unsigned)e, np.mg_cw);   // exact below 2048 (the plan checks)
    voff[i] = e < n_elem ? (cl * (int)np.g_c + (e - cl * chan_words)) * 4 : kDeadOffset;
  }
  auto load_rows = [&](const Tile &t, float (&ra)[kConvert], float (&rb)[kConvert]) {
    const int first = np.sx * t.ox_lo * ngy * 4;
    const __amdgpu_buffer_rsrc_t g_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((char *)G + (i64)t.n * np.g_n * 4 + first), 0, np.g_bytes - first, kRaw);
#pragma unroll
    for (int i = 0; i < kConvert; ++i) {
      ra[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(g_rsrc, voff[i], 0, 0));
      rb[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(g_rsrc, voff[i] + 4, 0, 0));
    }
  };
  auto cut_rows = [&](int which, const float (&ra)[kConvert], const float (&rb)[kConvert]) {
    char *const dst = sig0 + which * sig_bytes + 4 * tid;
#pragma unroll
    for (int i = 0; i < kConvert; ++i) {
      unsigned h, m, l;
      split_pair(ra[i], rb[i], h, m, l);
      if (tid + i * kThreads < n_elem) {
        *(unsigned *)(dst + 4 * kThreads * i) = h;
        *(unsigned *)(dst + plane + 4 * kThreads * i) = m;
        *(unsigned *)(dst + 2 * plane + 4 * kThreads * i) = l;
      }
    }
  };

  // ---- once per workgroup ---------------------------------------------------------------------
  Tile t_cur = tile_of(bx);
  float ra[kConvert], rb[kConvert];                      // a tile's words and their right-hand neighbours
  {
    // One trip to memory: the first tile's words, the second's, the filter block, the bias.
    float ra0[kConvert], rb0[kConvert];
    load_rows(t_cur, ra0, rb0);
    if (my_tiles > 1) load_rows(tile_of(bx + gx), ra, rb);
    constexpr int ITER = (groups * M_T + kThreads - 1) / kThreads;
    const __amdgpu_buffer_rsrc_t f_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((char *)F + (i64)m0 * np.f_m * 4), 0, m_live * (int)np.f_m * 4, kRaw);
    // thread -> (group of 8 taps, channel), channels fastest: the fragment writes below are then conflict-free;
    // the loads are 32 bytes per lane, 16 at a time where the quads of taps are whole (K a multiple of 4)
    float x[ITER][8];
    const bool quads = (K & 3) == 0;
#pragma unroll
    for (int j = 0; j < ITER; ++j) {
      const int idx = tid + j * kThreads, g = idx / M_T, m = idx - g * M_T;
      // (the taps of a channel are K consecutive words: f_c == nfx * nfy is a condition of the plan;
      //  channels past M lie past the descriptor's range)
      const int at = (m * (int)np.f_m + 8 * g) * 4;
      if (quads) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(f_rsrc, 8 * g + 4 * h < K ? at + 16 * h : kDeadOffset, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; ++i) x[j][4 * h + i] = __uint_as_float(v[i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          x[j][i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(f_rsrc, 8 * g + i < K ? at + 4 * i : kDeadOffset, 0, 0));
      }
    }
    float bv = 0.f;
    if (bias && tid < m_live) bv = bias[m0 + tid];
    for (int p = tid; p < (K16 >> 1); p += kThreads) {
      const int k = 2 * p, cl = k / np.nf, t = k - cl * np.nf, fx = t / np.nfy, fy = t - fx * np.nfy;
      // (taps past K meet zero weights: they read the lane's own first word)
      pairoff[p] = k < K ? 4 * (cl * chan_words + np.dx * fx * ngy + fy) : 0;
    }
    cut_rows(0, ra0, rb0);
    if (tid < M_T) bias_s[tid] = bv;
#pragma unroll
    for (int j = 0; j < ITER; ++j) {
      const int idx = tid + j * kThreads, g = idx / M_T, m = idx - g * M_T;
      if (idx < groups * M_T) store_frag(frag, groups, M_T, g, m, x[j]);
    }
  }
  // The loop's own waits count the stores that follow a request; nothing of the prologue may be in
  // flight when it starts, or the first tile's words would be taken for landed too early.
  __builtin_amdgcn_s_waitcnt(0x0F70);                     // vmcnt(0)

  // the pair offsets of this lane's half, every step's: the loop has no address that waits for an LDS read
  __syncthreads();
  int poff[STEPS][4];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int4 po = *(const int4 *)(pairoff + 4 * (2 * s + half));
    poff[s][0] = po.x; poff[s][1] = po.y; poff[s][2] = po.z; poff[s][3] = po.w;
  }

  auto lds_bytes_at = [&](int byte) { return (const char *)lds + byte; };
  floatx16 acc[MT][NT];
  int lane_base[NT][3];                                   // byte address of the lane's position in the three part planes
  struct Ops { uintx4 ah[MT], am[MT], al[MT], bh[NT], bm[NT], bl[NT]; };
  // (every register of an operand is the target of one LDS read: nothing to move afterwards)
  auto fetch_ops = [&](int s, Ops &o) {
    const int g = 2 * s + half;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o.bh[t][i] = *(const unsigned *)(lds_bytes_at(lane_base[t][0] + poff[s][i]));
        o.bm[t][i] = *(const unsigned *)(lds_bytes_at(lane_base[t][1] + poff[s][i]));
        o.bl[t][i] = *(const unsigned *)(lds_bytes_at(lane_base[t][2] + poff[s][i]));
      }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      o.ah[i] = frag[(0 * groups + g) * M_T + i * 32 + l32];
      o.am[i] = frag[(1 * groups + g) * M_T + i * 32 + l32];
      o.al[i] = frag[(2 * groups + g) * M_T + i * 32 + l32];
    }
  };
  auto multiply = [&](const Ops &o) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int t = 0; t < NT; ++t) mfma_split6(acc[i][t], o.ah[i], o.am[i], o.al[i], o.bh[t], o.bm[t], o.bl[t]);
  };

  const int hm1 = (int)np.h_m * 4;
  const bool relu = np.relu;
  constexpr int kFirstStores = 8;                         // accumulator registers stored before the next request

  for (int it = 0; it < my_tiles; ++it) {
    __syncthreads();    // this tile's pair words (first time: the tables too) are in place; every wave is done with the other tile's
    const int sig_at = (int)(sig0 - (char *)lds) + (it & 1) * sig_bytes;
    int q[NT];
    bool live[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      int local = (wave * NT + t) * 32 + l32;
      live[t] = local < t_cur.count;
      if (!live[t]) local = 0;                            // masked lane: any valid position
      q[t] = t_cur.q0 + local;
      const int ox = (int)__umulhi((unsigned)q[t], np.mg_noy_v), oy = q[t] - ox * noy;   // exact: q < 2^22 (the plan checks the reciprocal)
      lane_base[t][0] = sig_at + 4 * (np.sx * (ox - t_cur.ox_lo) * ngy + oy);
      lane_base[t][1] = lane_base[t][0] + plane;
      lane_base[t][2] = lane_base[t][1] + plane;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const float4 bq = *(const float4 *)(bias_s + i * 32 + g4 * 8 + half * 4);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][t][g4 * 4 + r] = (&bq.x)[r];
      }
    {
      // The operands of a step are requested while the step before it multiplies: two LDS reads after
      // each matrix instruction, pinned, or the scheduler moves every read next to its first use.
      auto interleave = [] {
#pragma unroll
        for (int k = 0; k < MT * NT * 6; ++k) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     // one matrix instruction
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);     // two LDS reads
        }
      };
      Ops a, b;
      fetch_ops(0, a);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < STEPS; s += 2) {
        if (s + 1 < STEPS) fetch_ops(s + 1, b);
        multiply(a);
        interleave();
        __builtin_amdgcn_sched_barrier(0);
        if (s + 1 < STEPS) {
          if (s + 2 < STEPS) fetch_ops(s + 2, a);
          multiply(b);
          interleave();
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (relu) {
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][t][r] = fmaxf(acc[i][t][r], 0.f);
    }
    if (it + 1 < my_tiles) cut_rows((it + 1) & 1, ra, rb);        // (that buffer's readers passed this iteration's barrier)
    // One descriptor over the block's channels that exist: stores to channels past M, and those of
    // lanes past the tile's last position (an offset past the descriptor), are dropped by the range check.
    const __amdgpu_buffer_rsrc_t h_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((char *)H + ((i64)t_cur.n * np.h_n + (i64)m0 * np.h_m) * 4), 0, m_live * hm1, kRaw);
    int hoff[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) hoff[t] = live[t] ? (half * 4) * hm1 + q[t] * 4 : kDeadOffset;
    auto store_regs = [&](int i, int r_lo, int r_hi) {
#pragma unroll
      for (int r = r_lo; r < r_hi; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[i][t][r]), h_rsrc, hoff[t],
                                                (i * 32 + (r >> 2) * 8 + (r & 3)) * hm1, 0);
    };
    store_regs(0, 0, kFirstStores);
    if (it + 1 < my_tiles) {
      t_cur = tile_of(bx + (it + 1) * gx);
      if (it + 2 < my_tiles) load_rows(tile_of(bx + (it + 2) * gx), ra, rb);
    }
    store_regs(0, kFirstStores, 16);
#pragma unroll
    for (int i = 1; i < MT; ++i) store_regs(i, 0, 16);
  }
}

template <int MT, int STEPS>
hipError_t launch_narrow_variant(const NarrowPlan &np, dim3 grid, const float *f, const float *g, const float *bias,
                                 float *h, hipStream_t stream) {
  auto kern = narrow_forward_kernel<MT, STEPS>;
  static std::atomic<int> lds_allowed{0};                  // (one per kernel instance)
  hipError_t e = allow_large_lds((const void *)kern, np.lds_bytes, lds_allowed);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), np.lds_bytes, stream, np, f, g, bias, h);
  return hipGetLastError();
}

}  // namespace

bool make_narrow_plan(const SepConv &pr, NarrowPlan &np, bool any_size) {
  if (pr.accumulate || pr.in_half || pr.out_half || pr.cls_nfx || pr.math == MATH_FP32) return false;
  const Axis &X = pr.x, &Y = pr.y;
  if (X.kind != AX_LCORR || Y.kind != AX_LCORR) return false;
  if (X.u != 1 || X.p != 0 || X.s < 1 || X.d < 1 || Y.u != 1 || Y.p != 0 || Y.s != 1 || Y.d != 1 || (Y.nf & 1)) return false;
  const i64 K = pr.c_in * X.nf * Y.nf, Q = X.nh * Y.nh;
  if (K < 1 || K > 128 || pr.c_in > 16 || Q < 1 || Q >= ((i64)1 << 22) || pr.batch < 1 || pr.c_out < 1) return false;
  // every output reads inside the signal, and the layout is the dense one
  if (X.s * (X.nh - 1) + X.d * (X.nf - 1) >= X.ng || (Y.nh - 1) + (Y.nf - 1) >= Y.ng) return false;
  if (pr.f_c != X.nf * Y.nf || pr.f_m != pr.c_in * pr.f_c) return false;
  const i64 lim = (i64)1 << 30;
  if (pr.batch >= lim || pr.c_out >= lim || pr.c_in * pr.g_c >= lim || X.s > 64 || X.d > 64 || Y.ng > 4096) return false;
  np.batch = (int)pr.batch; np.M = (int)pr.c_out; np.C = (int)pr.c_in;
  np.nfx = (int)X.nf; np.nfy = (int)Y.nf; np.nf = np.nfx * np.nfy; np.K = (int)K;
  np.ngy = (int)Y.ng; np.noy = (int)Y.nh; np.Q = (int)Q;
  np.sx = (int)X.s; np.dx = (int)X.d; np.span = (int)(X.d * (X.nf - 1));
  np.f_m = pr.f_m; np.g_n = pr.g_n; np.g_c = pr.g_c; np.h_n = pr.h_n; np.h_m = pr.h_m;
  np.relu = pr.relu;
  np.mt = pr.c_out > 32 ? 2 : 1;
  const int want = (int)((K + 15) / 16);
  np.steps = want <= 4 ? want : (want <= 6 ? 6 : 8);
  const int M_T = np.mt * 32, P = kWaves * 2 * 32;
  if ((i64)(M_T + 8) * pr.h_m * 4 >= ((i64)1 << 31)) return false;
  auto magic = [](int d) { return d <= 1 ? 0xFFFFFFFFu : (unsigned)(0x100000000ull / (unsigned)d); };
  np.tiles_per_image = (int)((Q + P - 1) / P);
  if ((i64)np.batch * np.tiles_per_image >= lim) return false;
  np.total_tiles = np.batch * np.tiles_per_image;
  np.mg_tpi = magic(np.tiles_per_image);
  np.mg_noy = magic(np.noy);
  // a reciprocal that is exact for every position index (floor(q * m / 2^32) == q / noy for q < Q)
  np.mg_noy_v = (unsigned)(((unsigned long long)1 << 32) / (unsigned)np.noy + 1);
  if (np.noy == 1) return false;
  for (i64 k = 1; k <= X.nh; ++k)                                  // (checked where the quotient steps: the ends of every row)
    for (i64 e = k * np.noy - 1; e <= k * np.noy && e < Q; ++e)
      if ((i64)(((unsigned long long)e * np.mg_noy_v) >> 32) != e / np.noy) return false;
  const i64 RT = std::min<i64>(X.nh, (P - 1 + Y.nh - 1) / Y.nh + 1);
  np.R = (int)(X.s * (RT - 1) + np.span + 1);
  const i64 n_elem = (i64)np.C * np.R * np.ngy;
  if (n_elem > kThreads * kConvert) return false;
  np.n_elem = (int)n_elem;
  {
    const unsigned cw = (unsigned)(np.R * np.ngy);
    np.mg_cw = (unsigned)(((unsigned long long)1 << 32) / cw + 1);
    for (unsigned e = 0; e < (unsigned)(kThreads * kConvert); ++e)
      if ((unsigned)(((unsigned long long)e * np.mg_cw) >> 32) != e / cw) return false;
  }
  np.plane_bytes = (int)((4 * n_elem + 15) & ~(i64)15);
  np.sig_bytes = 3 * np.plane_bytes;
  // the window of an image's last tile may reach past the signal: the descriptor ends with the last channel's last row
  const i64 g_bytes = ((pr.c_in - 1) * pr.g_c + X.ng * Y.ng) * 4;
  if (g_bytes >= ((i64)1 << 31) || pr.g_c < X.ng * Y.ng) return false;
  np.g_bytes = (int)g_bytes;
  const int K16 = np.steps * 16;
  np.lds_bytes = 48 * (size_t)(K16 >> 3) * M_T + 4 * (size_t)M_T + 4 * (size_t)(K16 >> 1) + 2 * (size_t)np.sig_bytes;
  if (np.lds_bytes > 80 * 1024) return false;             // two workgroups to a CU
  // (two workgroups to a CU: worth it only when the launch has tiles for them)
  if (!any_size && (i64)np.total_tiles * ((np.M + M_T - 1) / M_T) < 1024) return false;
  return true;
}

hipError_t launch_narrow_forward(const NarrowPlan &np, const float *f, const float *g, const float *bias, float *h,
                                 hipStream_t stream) {
  const int M_T = np.mt * 32;
  const int m_tiles = (np.M + M_T - 1) / M_T;
  int gx = std::max(1, (256 * 2) / m_tiles);
  gx = std::min(gx, np.total_tiles);
  dim3 grid((unsigned)gx, (unsigned)m_tiles);
#define MELLIN_NARROW_CASE(MT_, STEPS_) \
  if (np.mt == MT_ && np.steps == STEPS_) return launch_narrow_variant<MT_, STEPS_>(np, grid, f, g, bias, h, stream);
  MELLIN_NARROW_CASE(2, 1) MELLIN_NARROW_CASE(2, 2) MELLIN_NARROW_CASE(2, 3) MELLIN_NARROW_CASE(2, 4)
  MELLIN_NARROW_CASE(2, 6) MELLIN_NARROW_CASE(2, 8)
  MELLIN_NARROW_CASE(1, 1) MELLIN_NARROW_CASE(1, 2) MELLIN_NARROW_CASE(1, 3) MELLIN_NARROW_CASE(1, 4)
  MELLIN_NARROW_CASE(1, 6) MELLIN_NARROW_CASE(1, 8)
#undef MELLIN_NARROW_CASE
  return hipErrorInvalidValue;
}

}  // namespace mellin
