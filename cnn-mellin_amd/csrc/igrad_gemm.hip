// Input gradient of a correlation layer with few input channels and a linear
// x axis, in one kernel on the fp32 matrix cores.
//
//   grad_input[n, ci, gx, gy] = sum_{co, fx, fy} w[co, ci, fx, fy] *
//                               grad_out[n, co, hx, hy]
//   over the (hx, fx), (hy, fy) with  gx = sx hx + dx fx - px,  gy = sy hy + dy fy - py.
//
// With only a few input channels the gather form (one matrix row per input
// channel) leaves the 32-row matrix tiles almost empty.  Here the matrix rows
// are the FILTER TAPS instead: for one input channel ci
//
//   Z[(fx, fy), (hx, hy)] = sum_co w[co, ci, fx, fy] * grad_out[n, co, hx, hy]
//
// is a dense (taps x c_out) * (c_out x positions) product whose B operand is
// grad_out as it lies in memory (no gather, no padding), and every element of
// Z belongs to exactly one grad_input element, at (sx hx + dx fx - px,
// sy hy + dy fy - py).  Z never leaves the chip: each wavefront adds its
// accumulator tile straight into an LDS image of the grad_input rows its
// workgroup owns.
//
// Work split: one workgroup per (image, strip of T grad_input rows).  It walks
// the grad_out rows that have a tap in the strip, 32 * NT positions at a time
// (two LDS buffers filled by direct global->LDS loads, the next chunk in flight
// while this one multiplies).  One wavefront per (input channel, 32-tap tile):
// its filter operand stays in registers for the whole kernel, and it alone
// adds into its own LDS plane, in program order, so the result does not depend
// on scheduling (no two wavefronts ever add to the same word; lanes of one
// instruction that share a word are ordered by the hardware).  Rows of the
// plane above and below the strip catch the taps that fall outside it: the
// neighbouring strips recompute those.  At the end the planes of one input
// channel are summed in tile order and written out, coalesced along gy.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "igrad_gemm.hpp"
#include "tile_stage.hpp"

namespace mellin {

namespace {

template <int KSTEPS, int NT>
__global__ __launch_bounds__(512) void igrad_kernel(const IgradPlan pl, const float *__restrict__ W,
                                                    const float *__restrict__ GO,
                                                    float *__restrict__ GI) {
  extern __shared__ __align__(16) float lds[];
  constexpr int K = 2 * KSTEPS, P = NT * 32;
  float *Bs0 = lds;                                    // [2][K][P] grad_out chunk, channel-major
  float *planes = lds + 2 * K * P;                     // [units][Rp][Wp]

  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  const int n = blockIdx.x / pl.strips, strip = blockIdx.x - n * pl.strips;
  const int a = strip * pl.T, b = min(a + pl.T, pl.ngx);      // grad_input rows [a, b)

  // grad_out rows hx with sx hx + dx fx - px inside [a, b) for some fx
  const int reach = pl.dx * (pl.nfx - 1);
  int hx_lo = a + pl.px - reach;
  hx_lo = hx_lo > 0 ? (hx_lo + pl.sx - 1) / pl.sx : 0;
  int hx_hi = b - 1 + pl.px;
  hx_hi = hx_hi >= 0 ? min(pl.nhx - 1, hx_hi / pl.sx) : -1;
  const int q_lo = hx_lo * pl.nhy, q_end = (hx_hi + 1) * pl.nhy;
  const int nchunks = hx_hi >= hx_lo ? (q_end - q_lo + P - 1) / P : 0;
  const int plane_words = pl.Rp * pl.Wp;

  for (int i = tid; i < pl.units * plane_words; i += nthreads) planes[i] = 0.f;
  // rows past c_out and lanes past the image are never loaded: keep them finite
  for (int i = tid; i < 2 * K * P; i += nthreads) Bs0[i] = 0.f;

  // filter operand of this wavefront: A[tap m = l32][k = 2 s + half] = w[k, ci, m]
  const int ci = wave / pl.mtn, mt = wave - ci * pl.mtn;
  float areg[KSTEPS];
  {
    const int m = mt * 32 + l32;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = 2 * s + half;
      areg[s] = (k < pl.c_out && m < pl.nf) ? W[((i64)k * pl.c_in + ci) * pl.nf + m] : 0.f;
    }
  }
  // accumulator register r of this lane holds tap m(r); its offset in the plane
  int off[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = mt * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
    const int fx = m / pl.nfy, fy = m - fx * pl.nfy;
    off[r] = m < pl.nf ? pl.dx * fx * pl.Wp + pl.dy * fy : -1;
  }
  float *plane = planes + wave * plane_words;
  const float *GOn = GO + (i64)n * pl.c_out * pl.nh;
  const FastDiv by_nhy(pl.nhy);

  // Chunk c: channel k's P positions go to words [k * P, (k + 1) * P) of a buffer.
  // Odd channels are stored with every pair of 32-position halves exchanged, so
  // the two half-waves of the multiply loop (channels 2 s and 2 s + 1) read
  // disjoint banks.  Away from the end of the image one instruction moves
  // 16 bytes per lane: 1024 / (4 P) whole channels.
  constexpr int LPR = P / 4;                           // lanes per channel row
  constexpr int RPI = 64 / LPR;                        // channel rows per instruction
  const int row_in = lane / LPR, seg = lane - row_in * LPR;
  auto issue = [&](int c) {
    float *Bs = Bs0 + (c & 1) * K * P;
    const int q0 = q_lo + c * P;
    if (q0 + P <= pl.nh) {
      for (int k0 = wave * RPI; k0 < pl.c_out; k0 += pl.units * RPI) {
        const int k = k0 + row_in;
        const unsigned voff = (unsigned)(row_in * pl.nh + q0 + 4 * (seg ^ ((k & 1) << 3))) * 4u;
        if (k < pl.c_out) load16_to_lds(GOn + (i64)k0 * pl.nh, voff, Bs + k0 * P);
      }
    } else {
      for (int k = wave; k < pl.c_out; k += pl.units)
#pragma unroll
        for (int t2 = 0; t2 < P; t2 += 64) {
          const int q = q0 + t2 + (lane ^ ((k & 1) << 5));
          if (q < pl.nh) load_to_lds(GOn + (i64)k * pl.nh, (unsigned)q * 4u, Bs + k * P + t2);
        }
    }
  };

  __syncthreads();
  if (nchunks > 0) issue(0);
  for (int c = 0; c < nchunks; ++c) {
    // chunk c has landed for every wavefront, and nobody still reads the other buffer
    wait_all_memory();
    __syncthreads();
    if (c + 1 < nchunks) issue(c + 1);

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
    // this lane's channel of step s is 2 s + half; odd channels hold 32-position
    // tile t where tile t ^ 1 would be
    const float *Bs[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) Bs[t] = Bs0 + (c & 1) * K * P + half * P + ((t ^ half) << 5) + l32;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], Bs[t][2 * s * P], acc[t], 0, 0, 0);

    // fold: Z[m, position] joins grad_input word base(position) + off(m), by plain
    // read-add-write (this wavefront owns the plane).  The 32 lanes of a half-wave
    // hold one tap at 32 different positions: never the same word.  Registers r
    // with the same r % 4 (and the two half-waves) hold different taps; when the
    // plan has shown that those cannot meet either, they go as one batch.
    // Matrix rows past the last tap (off < 0) hold zeros and must not touch the plane.
    auto fold = [&](auto padded_rows) {
      constexpr bool kPadded = decltype(padded_rows)::value;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int rel = c * P + t * 32 + l32;              // position counted from q_lo
        int hxr, hy;
        by_nhy.divmod(rel, hxr, hy);
        float *dst = plane + pl.sx * hxr * pl.Wp + pl.sy * hy;
        if (q_lo + rel < q_end) {
          if (pl.batched_fold) {
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
              float v[4];
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (!kPadded || off[4 * j + c4] >= 0) v[j] = dst[off[4 * j + c4]];
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (!kPadded || off[4 * j + c4] >= 0) dst[off[4 * j + c4]] = v[j] + acc[t][4 * j + c4];
            }
          } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              // one half-wave at a time; the wave barriers keep the two phases apart
              if (half == 0 && (!kPadded || off[r] >= 0)) dst[off[r]] += acc[t][r];
              __builtin_amdgcn_wave_barrier();
              if (half == 1 && (!kPadded || off[r] >= 0)) dst[off[r]] += acc[t][r];
              __builtin_amdgcn_wave_barrier();
            }
          }
        }
      }
    };
    if ((pl.nf & 31) == 0) fold(std::false_type());
    else fold(std::true_type());
  }
  __syncthreads();

  // write the strip: plane row i is grad_input row g_lo + i, plane column j is gy = j - py
  const int rows = b - a;
  const int g_lo = pl.sx * hx_lo - pl.px;
  const int total = pl.c_in * rows * pl.ngy;
  const FastDiv by_ngy(pl.ngy), by_rows(rows);
  for (int i = tid; i < total; i += nthreads) {
    int r2, gy, cc, gxr;
    by_ngy.divmod(i, r2, gy);
    by_rows.divmod(r2, cc, gxr);
    const int pi = a + gxr - g_lo, pj = gy + pl.py;
    float v = 0.f;
    if (nchunks > 0 && pi >= 0 && pi < pl.Rp && pj >= 0 && pj < pl.Wp) {
      const float *src = planes + cc * pl.mtn * plane_words + pi * pl.Wp + pj;
      for (int m2 = 0; m2 < pl.mtn; ++m2) v += src[m2 * plane_words];
    }
    GI[((i64)(n * pl.c_in + cc) * pl.ngx + a + gxr) * pl.ngy + gy] = v;
  }
}

template <int KSTEPS, int NT>
hipError_t launch_instance(const IgradPlan &pl, const float *w, const float *go, float *gi,
                           hipStream_t stream) {
  auto kern = igrad_kernel<KSTEPS, NT>;
  if (pl.lds_bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)pl.lds_bytes);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(pl.batch * pl.strips)), dim3(64 * pl.units),
                     pl.lds_bytes, stream, pl, w, go, gi);
  return hipGetLastError();
}

}  // namespace

bool make_igrad_plan(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx,
                     i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py,
                     i64 ux, i64 uy, IgradPlan &pl, int force_nt, int force_T) {
  if (kind_x != AX_LCORR || ux != 1 || uy != 1) return false;
  if (px < 0 || py < 0) return false;
  const i64 nf = nfx * nfy, nh = nhx * nhy, ng = ngx * ngy;
  if (batch < 1 || c_in < 1 || c_out < 1 || nf < 1 || nh < 1 || ng < 1) return false;
  const i64 lim = (i64)1 << 28;
  if (batch * c_out * nh / nh != batch * c_out || nh >= lim || ng >= lim || c_out * c_in * nf >= lim)
    return false;
  if (sx >= 4096 || sy >= 4096 || dx >= 4096 || dy >= 4096 || px >= lim || py >= lim) return false;
  // few input channels, and taps that fill their 32-row tiles reasonably
  const i64 mtn = (nf + 31) / 32;
  const i64 units = c_in * mtn;
  if (c_in >= 16 || units > 8 || mtn * 32 * 2 > nf * 3) return false;
  if (c_out > 128) return false;
  pl.batch = (int)batch; pl.c_in = (int)c_in; pl.c_out = (int)c_out;
  pl.nfx = (int)nfx; pl.nfy = (int)nfy; pl.nf = (int)nf;
  pl.nhx = (int)nhx; pl.nhy = (int)nhy; pl.nh = (int)nh;
  pl.ngx = (int)ngx; pl.ngy = (int)ngy;
  pl.sx = (int)sx; pl.dx = (int)dx; pl.px = (int)px;
  pl.sy = (int)sy; pl.dy = (int)dy; pl.py = (int)py;
  pl.mtn = (int)mtn; pl.units = (int)units;
  // Taps whose matrix rows are congruent mod 4 are folded in one batch.  That is
  // safe when no two of them can send two of 32 consecutive positions to the
  // same grad_input word: positions (hx, hy), (hx', hy') and taps (fx, fy),
  // (fx', fy') meet iff sx (hx - hx') = dx (fx' - fx) and sy (hy - hy') = dy (fy' - fy).
  pl.batched_fold = 1;
  for (i64 m = 0; m < nf && pl.batched_fold; ++m)
    for (i64 m2 = m + 4; m2 < nf && m2 / 32 == m / 32; m2 += 4) {
      const i64 ax = dx * (m2 / nfy - m / nfy), ay = dy * (m2 % nfy - m % nfy);
      if (ax % sx != 0 || ay % sy != 0) continue;
      const i64 ex = ax / sx, ey = ay / sy;              // position difference that would meet
      const i64 span = ex * nhy + ey;
      if (std::abs(ey) < nhy && std::abs(span) >= 1 && std::abs(span) <= 31) { pl.batched_fold = 0; break; }
    }
  pl.ksteps = c_out <= 32 ? 16 : c_out <= 64 ? 32 : 64;
  const i64 K = 2 * pl.ksteps;
  const i64 Wp = sy * (nhy - 1) + dy * (nfy - 1) + 1;
  const i64 reach = dx * (nfx - 1);
  if (Wp >= 4096) return false;
  // strip height: enough workgroups to fill the chip about three times over, but
  // strips at least twice as tall as the rows recomputed at their borders
  const i64 want_strips = std::max<i64>(1, (768 + batch - 1) / batch);
  i64 T = std::max<i64>((ngx + want_strips - 1) / want_strips, std::max<i64>(2 * reach / sx, 4));
  if (force_T > 0) T = force_T;
  T = std::min(T, ngx);
  // LDS tiers: three, two, one workgroup per CU; within a tier the wider chunk
  const size_t tiers[3] = {53 * 1024, 80 * 1024, 160 * 1024 - 512};
  for (i64 t = T; t >= 1; t = (t > 8 ? t * 3 / 4 : t - 1)) {
    const i64 Rp = sx * ((t - 1 + reach) / sx) + reach + 1;
    if ((t + reach + 2) * std::max(nhy, Wp) >= ((i64)1 << 22)) continue;   // float-reciprocal index splits
    if (c_in * t * ngy >= ((i64)1 << 22)) continue;
    for (int tier = 0; tier < 3; ++tier)
      for (int nt = 4; nt >= 2; nt -= 2) {
        if (force_nt > 0 && nt != force_nt) continue;
        const size_t lds = 4 * (size_t)(2 * K * nt * 32 + units * Rp * Wp);
        if (lds > tiers[tier]) continue;
        pl.nt = nt; pl.T = (int)t; pl.strips = (int)((ngx + t - 1) / t);
        pl.Rp = (int)Rp; pl.Wp = (int)Wp; pl.lds_bytes = lds;
        return (i64)pl.batch * pl.strips < ((i64)1 << 31);
      }
  }
  return false;
}

hipError_t launch_igrad(const IgradPlan &pl, const float *weight, const float *grad_out,
                        float *grad_input, hipStream_t stream) {
#define MELLIN_IGRAD_CASE(KS, NT_)                                                       \
  if (pl.ksteps == KS && pl.nt == NT_)                                                   \
    return launch_instance<KS, NT_>(pl, weight, grad_out, grad_input, stream);
  MELLIN_IGRAD_CASE(16, 2) MELLIN_IGRAD_CASE(16, 4)
  MELLIN_IGRAD_CASE(32, 2) MELLIN_IGRAD_CASE(32, 4)
  MELLIN_IGRAD_CASE(64, 2) MELLIN_IGRAD_CASE(64, 4)
#undef MELLIN_IGRAD_CASE
  return hipErrorInvalidValue;
}

}  // namespace mellin
