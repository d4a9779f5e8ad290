// Weight gradient with the matrix instructions running along the output positions: for
// half-precision layers on the f16 matrix cores, for fp32 layers on the bf16 ones.
//
//   W[m, (c, fx, fy)] = sum_{n, ox, oy} A[n, m, ox, oy] *
//                       G[n, c, tap_x(ox, fx), tap_y(oy, fy)]
//
// A = grad_out and G = the layer's input are read as they lie.  Half precision: products of
// half values are exact in fp32 and v_mfma_f32_32x32x16_f16 sums them in fp32, so the
// arithmetic is that of the fp32 kernels on the widened operands, in another order.  fp32:
// both operands are split into three bf16 parts in registers and a product is six bf16
// matrix instructions (tile_stage.hpp).
//
// The product is (M x positions) * (positions x J), J = c_in * nfx * nfy, and the k index of
// a matrix instruction runs over sixteen CONSECUTIVE output positions of one image (rows
// flattened), eight per half-wave:
//   * grad_out: the eight positions of a lane's channel are consecutive in global memory
//     (any element alignment): one or two 16-byte loads per lane straight into registers, a
//     few steps ahead, no LDS -- for half precision the instruction's operand as it is;
//   * input: the rows a unit of work touches are staged as in the forward kernel (direct
//     global->LDS loads into affine virtual rows, one value per LDS word), and the operand
//     of lane (column j) for position q is the word at col_offset[j] + pos_offset[q];
//     pos_offset is a table in LDS, the same for every unit.
// A unit is RB output rows of one image.  A workgroup owns 64 * mbw output channels and
// JT * 32 columns for its whole life and walks a contiguous range of units (image running
// fastest, so that consecutive units stage the same rows of successive images); its four
// wavefronts are mbw side by side along the channels times 4 / mbw shares of a unit's
// steps.  Every wavefront writes its accumulators as one partial block; wgrad_reduce adds
// the partial blocks in index order (no floating-point atomics: bit-reproducible).
#include <algorithm>
#include <type_traits>

#include "mellin_common.hpp"
#include "tile_gemm.hpp"
#include "tile_stage.hpp"

namespace mellin {

namespace {

constexpr int kF16Memo = 8;                        // 64-word blocks per wave whose staging sources are kept

struct __attribute__((packed, aligned(2))) Bytes16At2 { uintx4 v; };
struct __attribute__((packed, aligned(4))) Bytes16At4 { uintx4 v; };

// F16: A and G are half-precision storage (else float)
template <int JT, bool F16>
__global__ __launch_bounds__(kThreads, 2) void wgrad_pos_kernel(
    WgradPosPlan wp, const void *__restrict__ Av, const void *__restrict__ G,
    float *__restrict__ ws) {
  typedef typename std::conditional<F16, _Float16, float>::type T;
  constexpr int EB = sizeof(T);
  // (deeper rings and requests batched four steps at a time measured 3-8 % slower)
  constexpr int kBatch = 1;                          // steps whose grad_out is requested together
  constexpr int kAhead = 2 * kBatch;                 // steps whose grad_out operands are held
  constexpr int kRaw = F16 ? 1 : 2;                  // 16-byte words of eight values
  const T *A = (const T *)Av;
  extern __shared__ __align__(16) float lds[];
  const TilePlan &pl = wp.t;
  constexpr int MT = 2;
  const int x_words = (wp.CCj * pl.R * pl.RS + 3) & ~3;
  float *Xs0 = lds;                                  // [2][CCj][R][RS], one half value per word
  int *pos_off = (int *)(Xs0 + 2 * x_words);         // [UP] byte offset of a position's (fx, fy) = (0, 0) word

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;
  const int mb = wave % wp.mbw, ps = wave / wp.mbw, PS = kWaves / wp.mbw;

  const int mg = blockIdx.y / wp.j_groups, jg = blockIdx.y - mg * wp.j_groups;
  const int M_T = 64 * wp.mbw, J_T = JT * 32;
  const int m0 = mg * M_T + mb * 64, j0 = jg * J_T;
  const int c_lo = j0 / pl.nf;
  const int j_last = min(wp.J, j0 + J_T) - 1;
  const int ccj = j_last / pl.nf - c_lo + 1;

  int col_off[JT];                                   // bytes
  {
    const FastDiv by_nf(pl.nf), by_nfy(pl.nfy);
#pragma unroll
    for (int t = 0; t < JT; ++t) {
      const int j = min(j0 + t * 32 + l32, wp.J - 1);   // columns past J are computed but never read back
      int c, tt, fx, fy;
      by_nf.divmod(j, c, tt);
      by_nfy.divmod(tt, fx, fy);
      col_off[t] = ((c - c_lo) * pl.R * pl.RS + pl.Bx * fx * pl.RS + pl.by * fy) * 4;
    }
  }
  {
    const FastDiv by_noy(pl.noy);
    for (int p = tid; p < wp.UP; p += kThreads) {
      int oxl, oy;
      by_noy.divmod(p, oxl, oy);
      pos_off[p] = oxl < wp.RB ? ((pl.Ax * oxl + pl.Cx0) * pl.RS + pl.ay * oy - pl.by_min) * 4 : 0;
    }
  }

  // units: image fastest; this workgroup's contiguous range
  const int units_per_image = (pl.nox_eff + wp.RB - 1) / wp.RB;
  const int total_units = pl.batch * units_per_image;
  const int share = total_units / (int)gridDim.x, extra = total_units - share * (int)gridDim.x;
  const int my_units = share + ((int)blockIdx.x < extra ? 1 : 0);
  const int first_unit = (int)blockIdx.x * share + min((int)blockIdx.x, extra);
  const unsigned lds_base = lds_address(lds);

  auto unit_geometry = [&](int unit) {
    TileGeom g;
    const int u = unit / pl.batch;
    g.n = unit - u * pl.batch;
    g.ox_lo = u * wp.RB;
    const int rows = min(wp.RB, pl.nox_eff - g.ox_lo);
    g.oy_lo = 0;
    g.q0 = g.ox_lo * pl.noy;
    g.count = rows * pl.noy;
    g.R_tile = mellin_x ? rows * pl.nfx : pl.ax * (rows - 1) + pl.bx_span + 1;
    g.vx_min = pl.ax * g.ox_lo + pl.cx + pl.bx_min;
    g.vy_min = pl.cy + pl.by_min;
    g.RSL = pl.ay * (pl.noy - 1) + pl.by_span + 1;
    return g;
  };
  StageMemo<kF16Memo> memo = {};
  auto issue_stage = [&](int ui) {
    const TileGeom tg = unit_geometry(first_unit + ui);
    const int b = ui & 1;
    // units since the rows last changed (or since this workgroup started): the memo is
    // renewed at 0, and a buffer's zeros are written the first two times it holds these rows
    const int run = min(tg.n, ui);
    unsigned zero;                                     // a zero the compiler cannot see through (see tile_gemm.hip)
    asm volatile("s_mov_b32 %0, 0" : "=s"(zero));
    issue_signal<kWaves, kF16Memo, EB>(pl, tg, G, c_lo, ccj, Xs0 + b * x_words, lds_base + 4u * (unsigned)(b * x_words),
                                      mellin_x, lane, wave + (int)zero, &memo, run == 0, run < 2);
  };

  floatx16 acc[MT][JT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < JT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  // this lane's two channels (one past M reads the last channel's values instead: its rows
  // of the partial block are never read back)
  int m_off[MT];                                       // elements: M * Q < 2^30
#pragma unroll
  for (int i = 0; i < MT; ++i) m_off[i] = min(m0 + i * 32 + l32, pl.M - 1) * (int)wp.a_m + 8 * half;

  // grad_out of one step as loaded: the lane's eight values per channel tile
  struct RawA { uintx4 v[MT][kRaw]; };
  auto load_a = [&](const T *An, int s, RawA &a) {           // whole steps only
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const T *p = An + m_off[i] + 16 * s;
      if constexpr (F16) {
        a.v[i][0] = ((const Bytes16At2 *)p)->v;
      } else {
        a.v[i][0] = ((const Bytes16At4 *)p)->v;
        a.v[i][1] = ((const Bytes16At4 *)(p + 4))->v;
      }
    }
  };
  // one step: the input words of the lane's columns at the step's sixteen positions times
  // grad_out; `left` < 8: only that many of this half-wave's positions exist (both operands
  // are cleared past them)
  auto multiply_step = [&](const float *Xs, int s, const RawA &a, int left) {
    const int4 o0 = *(const int4 *)(pos_off + 16 * s + 8 * half), o1 = *(const int4 *)(pos_off + 16 * s + 8 * half + 4);
    const int off[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
    if constexpr (F16) {
      unsigned keep[4];
#pragma unroll
      for (int w = 0; w < 4; ++w) keep[w] = (2 * w < left ? 0xFFFFu : 0u) | (2 * w + 1 < left ? 0xFFFF0000u : 0u);
#pragma unroll
      for (int t = 0; t < JT; ++t) {
        uintx4 b;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          ushortx2 pair;
          pair.x = *(const unsigned short *)((const char *)Xs + (col_off[t] + off[2 * i]));
          pair.y = *(const unsigned short *)((const char *)Xs + (col_off[t] + off[2 * i + 1]));
          b[i] = __builtin_bit_cast(unsigned, pair);
          if (left < 8) b[i] &= keep[i];
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
          acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a.v[i][0]),
                                                             __builtin_bit_cast(halfx8, b), acc[i][t], 0, 0, 0);
      }
    } else {
      uintx4 ah[MT], am[MT], al[MT];
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        float x[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) x[k] = __uint_as_float(a.v[i][k >> 2][k & 3]);
        split8(x, ah[i], am[i], al[i]);
      }
#pragma unroll
      for (int t = 0; t < JT; ++t) {
        float x[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          x[k] = *(const float *)((const char *)Xs + (col_off[t] + off[k]));
          if (left < 8 && k >= left) x[k] = 0.f;
        }
        uintx4 bh, bm, bl;
        split8(x, bh, bm, bl);
#pragma unroll
        for (int i = 0; i < MT; ++i) mfma_split6(acc[i][t], ah[i], am[i], al[i], bh, bm, bl);
      }
    }
  };

  __syncthreads();                                     // pos_off
  if (my_units > 0) issue_stage(0);
  for (int ui = 0; ui < my_units; ++ui) {
    const TileGeom tg = unit_geometry(first_unit + ui);
    const T *An = A + (i64)tg.n * wp.a_n + tg.q0;
    const int whole = tg.count >> 4;                   // steps of sixteen positions that exist
    // this wavefront's steps ps, ps + PS, ...: the first few operands are requested before
    // the wait for the staged rows
    RawA ring[kAhead];
#pragma unroll
    for (int d = 0; d < kAhead; ++d)
      if (ps + d * PS < whole) load_a(An, ps + d * PS, ring[d]);
    wait_all_memory();
    __syncthreads();
    if (ui + 1 < my_units) {
      __builtin_amdgcn_s_setprio(3);
      issue_stage(ui + 1);
      __builtin_amdgcn_s_setprio(0);
    }
    const float *Xs = Xs0 + (ui & 1) * x_words;
    for (int s0 = ps; s0 < whole; s0 += kAhead * PS) {
#pragma unroll
      for (int g = 0; g < 2; ++g) {
#pragma unroll
        for (int d = g * kBatch; d < (g + 1) * kBatch; ++d) {
          const int s = s0 + d * PS;
          if (s < whole) multiply_step(Xs, s, ring[d], 8);
        }
        // the group's slots are free: their next occupants are requested together (with one
        // share of steps per unit they are neighbours in memory, and a line fetched for the
        // first is still in the cache for the others)
#pragma unroll
        for (int d = g * kBatch; d < (g + 1) * kBatch; ++d) {
          const int s = s0 + d * PS;
          if (s + kAhead * PS < whole) load_a(An, s + kAhead * PS, ring[d]);
        }
      }
    }
    // the last, partial step (by the wavefront whose turn it is): positions past the unit's
    // end belong to the next unit or to nothing, so both operands are cleared there
    if ((tg.count & 15) && whole % PS == ps) {
      const int left = min(8, max(0, tg.count - 16 * whole - 8 * half));     // of this half-wave's eight positions
      RawA a;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const T *src = An + m_off[i] + 16 * whole;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          if constexpr (F16) {
            const unsigned v = k < left ? (unsigned)((const unsigned short *)src)[k] : 0u;
            if (k & 1) a.v[i][0][k >> 1] |= v << 16;
            else a.v[i][0][k >> 1] = v;
          } else {
            a.v[i][k >> 2][k & 3] = k < left ? __float_as_uint(src[k]) : 0u;
          }
        }
      }
      multiply_step(Xs, whole, a, left);
    }
  }

  // ---- every wavefront writes its partial block ------------------------------------
  float *out = ws + ((i64)((int)blockIdx.x * PS + ps) * wp.M_pad + m0) * wp.J_pad + j0;
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < JT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = i * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
        out[(i64)m * wp.J_pad + t * 32 + l32] = acc[i][t][r];
      }
}

template <int JT, bool F16>
hipError_t launch_pos(const WgradPosPlan &wp, dim3 grid, const void *a, const void *g, float *ws,
                      hipStream_t stream) {
  auto kern = wgrad_pos_kernel<JT, F16>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, wp.lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), wp.lds_bytes, stream, wp, a, g, ws);
  return hipGetLastError();
}

}  // namespace

bool make_wgrad_pos_plan(const SepConv &fwd_in, WgradPosPlan &wp, bool half) {
  wp.half = half;
  // (the forward tiling is only borrowed for its staging geometry: plan it for the fp32 kernel)
  SepConv fwd = fwd_in;
  fwd.math = MATH_FP32;
  fwd.in_half = 0;
  fwd.out_half = 0;
  fwd.accumulate = 0;
  size_t lds_fwd;
  int mt, nt;
  if (!make_tile_plan(fwd, wp.t, &lds_fwd, &mt, &nt, 1)) return false;
  TilePlan &pl = wp.t;
  if (pl.segment || pl.nox_eff < 1 || pl.noy_eff < 1) return false;
  if ((i64)pl.M * pl.Q >= ((i64)1 << 30)) return false;          // 32-bit element offsets inside an image
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;
  // whole output rows are staged, element by element
  pl.contig = 0;
  pl.RS = (pl.ay * (pl.noy - 1) + pl.by_span + 1) | 1;
  wp.J = pl.C * pl.nf;
  // (four column tiles in both precisions; the fp32 instance then holds 244 registers, without spills:
  //  grad_out is re-read once per block of 128 columns instead of 96)
  wp.jt = std::min(4, (wp.J + 31) / 32);
  wp.mbw = pl.M > 128 ? 4 : (pl.M > 64 ? 2 : 1);
  const int M_T = 64 * wp.mbw, J_T = wp.jt * 32;
  wp.m_groups = (pl.M + M_T - 1) / M_T;
  wp.j_groups = (wp.J + J_T - 1) / J_T;
  wp.M_pad = wp.m_groups * M_T;
  wp.J_pad = wp.j_groups * J_T;
  wp.a_n = (i64)pl.M * pl.Q;
  wp.a_m = pl.Q;
  wp.CCj = std::min(pl.C, (J_T - 1 + pl.nf - 1) / pl.nf + 1);
  if ((i64)wp.CCj * pl.ngx * pl.ngy >= ((i64)1 << 30)) return false;
  // the largest unit whose rows fit twice in the LDS of a workgroup (two to a CU)
  wp.RB = 0;
  for (int rb = std::min(pl.nox_eff, 64); rb >= 1; --rb) {
    const i64 Rr = mellin_x ? (i64)rb * pl.nfx : (i64)pl.ax * (rb - 1) + pl.bx_span + 1;
    const i64 up = (((i64)rb * pl.noy + 15) / 16) * 16;
    const i64 xw = ((i64)wp.CCj * Rr * pl.RS + 3) & ~(i64)3;
    const i64 bytes = 4 * (2 * xw + up);
    if (Rr > 8192 || up > 4096 || bytes > 76 * 1024) continue;
    wp.RB = rb;
    wp.UP = (int)up;
    pl.R = (int)Rr;
    wp.lds_bytes = (size_t)bytes;
    break;
  }
  if (!wp.RB) return false;
  const i64 units = (i64)pl.batch * ((pl.nox_eff + wp.RB - 1) / wp.RB);
  const int blocks_y = wp.m_groups * wp.j_groups;
  wp.S = (int)std::min<i64>(std::max<i64>(1, (256 * 2) / blocks_y), units);
  wp.ws_bytes = (size_t)wp.S * (kWaves / wp.mbw) * wp.M_pad * wp.J_pad * sizeof(float);
  return true;
}

hipError_t launch_wgrad_pos(const WgradPosPlan &wp, const void *grad_out, const void *input,
                            void *grad_weight, float *workspace, hipStream_t stream) {
  dim3 grid((unsigned)wp.S, (unsigned)(wp.m_groups * wp.j_groups));
  hipError_t e = hipErrorInvalidValue;
  if (wp.half) {
    if (wp.jt == 1) e = launch_pos<1, true>(wp, grid, grad_out, input, workspace, stream);
    if (wp.jt == 2) e = launch_pos<2, true>(wp, grid, grad_out, input, workspace, stream);
    if (wp.jt == 3) e = launch_pos<3, true>(wp, grid, grad_out, input, workspace, stream);
    if (wp.jt == 4) e = launch_pos<4, true>(wp, grid, grad_out, input, workspace, stream);
  } else {
    if (wp.jt == 1) e = launch_pos<1, false>(wp, grid, grad_out, input, workspace, stream);
    if (wp.jt == 2) e = launch_pos<2, false>(wp, grid, grad_out, input, workspace, stream);
    if (wp.jt == 3) e = launch_pos<3, false>(wp, grid, grad_out, input, workspace, stream);
    if (wp.jt == 4) e = launch_pos<4, false>(wp, grid, grad_out, input, workspace, stream);
  }
  if (e != hipSuccess) return e;
  return launch_wgrad_reduce(workspace, grad_weight, wp.half, wp.S * (kWaves / wp.mbw), wp.t.M, wp.J,
                             wp.M_pad, wp.J_pad, stream);
}

}  // namespace mellin
