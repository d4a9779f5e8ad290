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
// accumulator tile straight into an LDS image ("plane") of the grad_input rows
// its workgroup can reach.
//
// Work split: one workgroup per (image, strip of Th grad_out rows), so every
// grad_out element is read and multiplied once.  The strip is walked 32 * NT
// positions at a time: all channels of the chunk are copied to LDS by direct
// global->LDS loads (16 bytes per lane), then multiplied.  The buffer is single:
// several small workgroups share a CU and cover each other's load latency.
// One wavefront per (input channel, 32-tap tile): its filter operand stays in
// registers for the whole kernel, and it alone adds into its own plane, in
// program order, so the result does not depend on scheduling.
//
// A grad_input row whose taps all come from one strip is written by that
// strip's workgroup.  The few rows fed by two neighbouring strips (dx (nfx - 1)
// - sx + 1 rows per boundary) are written as two partial rows into a small
// workspace and summed, upper strip first, by a second kernel.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "igrad_gemm.hpp"
#include "tile_stage.hpp"

namespace mellin {

namespace {

// Strips [lo, hi] that feed grad_input row gx: the strips of the first and last
// grad_out rows hx with sx hx + dx fx - px = gx for some fx in [0, nfx), clamped
// to the rows that exist.  lo == hi for most rows; hi == lo + 1 next to a
// strip boundary (the plan keeps strips taller than a filter's reach).  A row
// that nothing feeds belongs to the strip of the last grad_out row before it.
struct StripMap {
  FastDiv by_sx, by_th;
  int px, reach, sx, H;
  __device__ explicit StripMap(const IgradPlan &pl)
      : by_sx(pl.sx), by_th(pl.Th), px(pl.px), reach(pl.dx * (pl.nfx - 1)), sx(pl.sx), H(pl.H) {}
  __device__ __forceinline__ void feeding(int gx, int &lo, int &hi) const {
    int q, r;
    const int a0 = gx + px - reach;                    // ceil(a0 / sx), clamped below at 0
    int h0 = 0;
    if (a0 > 0) { by_sx.divmod(a0 + sx - 1, q, r); h0 = q; }
    by_sx.divmod(gx + px, q, r);                       // gx + px >= 0
    int h1 = q;
    h0 = min(h0, H - 1);
    h1 = min(h1, H - 1);
    if (h0 > h1) h0 = h1;                              // no row feeds gx (stride wider than the reach)
    by_th.divmod(h0, lo, r);
    by_th.divmod(h1, hi, r);
  }
};

// Up to twelve wavefronts per workgroup (168 registers each) wherever the instance can live with that.
template <int KSTEPS, int NT, bool PIPE>
__global__ __launch_bounds__((KSTEPS * NT <= 128 ? 768 : 512)) void igrad_kernel(const IgradPlan pl, const float *__restrict__ W,
                                                    const float *__restrict__ GO,
                                                    float *__restrict__ GI, float *__restrict__ WS) {
  extern __shared__ __align__(16) float lds[];
  constexpr int K = 2 * KSTEPS, P = NT * 32;
  constexpr int BW = PIPE ? K * 96 : K * P;            // words of the chunk buffer

  // A workgroup runs pl.jobs independent (image, strip) jobs side by side, one
  // group of pl.units wavefronts each with its own slice of LDS: same strip,
  // consecutive images, hence the same trip counts and barriers.  That makes the
  // wavefront count a multiple of four (all four SIMDs of a CU equally loaded).
  // (wave-uniform quantities are marked as such: what derives from them is then
  // computed on the scalar unit)
  const int wave_in_group = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int job = wave_in_group / pl.units;
  const int wave = wave_in_group - job * pl.units;
  const int lane = threadIdx.x & 63;
  const int tid = wave * 64 + lane, nthreads = pl.units * 64;
  const int half = lane >> 5, l32 = lane & 31;
  const int image_group = blockIdx.x / pl.strips, strip = blockIdx.x - image_group * pl.strips;
  const int n_want = image_group * pl.jobs + job;
  const bool active = n_want < pl.batch;               // a job past the last image only keeps the barriers
  const int n = active ? n_want : pl.batch - 1;
  const int ha = strip * pl.Th, hb = min(ha + pl.Th, pl.H);    // grad_out rows [ha, hb)
  const int q_lo = ha * pl.nhy, q_end = hb * pl.nhy;
  const int nchunks = (q_end - q_lo + P - 1) / P;
  const int plane_words = pl.Rp * pl.Wp;
  float *job_lds = lds + job * (((BW + pl.units * plane_words) + 3) & ~3);
  float *Bs = job_lds;                                 // grad_out chunk buffer, channel-major
  float *planes = job_lds + BW;                        // [units][Rp][Wp]

  for (int i = tid; i < pl.units * plane_words; i += nthreads) planes[i] = 0.f;
  // channels past c_out are never loaded, nor are positions past the end of the
  // image: keep what the multiply loop reads there finite
  if (PIPE || q_lo + nchunks * P > pl.nh) {
    for (int i = tid; i < BW; i += nthreads) Bs[i] = 0.f;
  } else {
    for (int i = pl.c_out * P + tid; i < BW; i += nthreads) Bs[i] = 0.f;
  }

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
  // (-1: a matrix row past the last tap)
  int off[16];
  {
    const FastDiv by_nfy(pl.nfy);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = mt * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
      int fx, fy;
      by_nfy.divmod(m, fx, fy);
      off[r] = m < pl.nf ? pl.dx * fx * pl.Wp + pl.dy * fy : -1;
    }
  }
  float *plane = planes + wave * plane_words;
  const float *GOn = GO + (i64)n * pl.c_out * pl.nh;
  const FastDiv by_nhy(pl.nhy);

  // Chunk c: channel k's P positions go to words [k * P, (k + 1) * P) of the buffer.
  // Odd channels are stored with every pair of 32-position halves exchanged, so
  // the two half-waves of the multiply loop (channels 2 s and 2 s + 1) read
  // disjoint banks.  Away from the end of the image one instruction moves
  // 16 bytes per lane: 1024 / (4 P) whole channels.
  constexpr int LPR = P / 4;                           // lanes per channel row
  constexpr int RPI = 64 / LPR;                        // channel rows per instruction
  constexpr int KH = K / 2;                            // channels per half of the buffer
  const int row_in = lane / LPR, seg = lane - row_in * LPR;
  const unsigned bs_addr = lds_address(Bs);
  auto issue = [&](int c, int k_lo) {                  // channels [k_lo, k_lo + KH) of chunk c
    const int q0 = q_lo + c * P;
    const int k_hi = min(k_lo + KH, pl.c_out);
    if (q0 + P <= pl.nh) {
      for (int k0 = k_lo + wave * RPI; k0 < k_hi; k0 += pl.units * RPI) {
        const int k = k0 + row_in;
        const unsigned voff = (unsigned)(row_in * pl.nh + q0 + 4 * (seg ^ ((k & 1) << 3))) * 4u;
        if (k < k_hi) load16_to_lds_at(GOn + (i64)k0 * pl.nh, voff, bs_addr + 4u * (unsigned)(k0 * P));
      }
    } else {
      for (int k = k_lo + wave; k < k_hi; k += pl.units)
#pragma unroll
        for (int t2 = 0; t2 < P; t2 += 64) {
          const int q = q0 + t2 + (lane ^ ((k & 1) << 5));
          if (q < pl.nh) load_to_lds_at(GOn + (i64)k * pl.nh, (unsigned)q * 4u, bs_addr + 4u * (unsigned)(k * P + t2));
        }
    }
  };

  // The buffer is single, but its two channel halves are refilled separately:
  // as soon as every wavefront has multiplied a half, the same half of the next
  // chunk is requested, so the loads fly during the other half's multiplies
  // and the fold.
  // this lane's channel of step s is 2 s + half; odd channels hold 32-position
  // tile t where tile t ^ 1 would be
  int bo[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) bo[t] = half * P + ((t ^ half) << 5) + l32;
  // fold: Z[m, position] joins grad_input word base(position) + off(m), by plain
  // read-add-write (this wavefront owns the plane).  The 32 lanes of a half-wave
  // hold one tap at 32 different positions: never the same word.  Registers r
  // with the same r % 4 (and the two half-waves) hold different taps; when the
  // plan has shown that those cannot meet either, they go as one batch.
  auto fold = [&](auto padded_rows, int c, const floatx16 (&acc)[NT]) {
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

  if constexpr (PIPE) {
    // Batched fold and every matrix row a tap: positions stream through in tiles
    // of 32.  Tile p lives in block p % 3 of the buffer ([3][K][32] words); the
    // block of tile p - 1 is refilled with tile p + 2 as soon as every wavefront
    // has multiplied it, two tile phases before it is needed.  The fold of tile
    // p - 1 is cut into its four batches and spread between the multiplies of
    // tile p, so its LDS round trips hide behind the matrix pipe.
    constexpr int NBUF = 3, SPB = KSTEPS / 4;            // multiply steps per fold batch
    const int ntiles = (q_end - q_lo + 31) / 32;
    const int row8 = lane >> 3, seg8 = lane & 7;         // 8 lanes x 16 bytes per channel row
    auto issue_tile = [&](int p) {
      const int q0 = q_lo + p * 32;
      const unsigned blk = bs_addr + 4u * (unsigned)((p % NBUF) * K * 32);
      if (q0 + 32 <= pl.nh) {
        for (int k0 = wave * 8; k0 < pl.c_out; k0 += pl.units * 8) {
          const unsigned voff = (unsigned)(row8 * pl.nh + q0 + 4 * seg8) * 4u;
          if (k0 + row8 < pl.c_out) load16_to_lds_at(GOn + (i64)k0 * pl.nh, voff, blk + 4u * (unsigned)(k0 * 32));
        }
      } else {
        for (int k = wave; k < pl.c_out; k += pl.units)
          if (lane < 32 && q0 + lane < pl.nh)
            load_to_lds_at(GOn + (i64)k * pl.nh, (unsigned)(q0 + lane) * 4u, blk + 4u * (unsigned)(k * 32));
      }
    };
    floatx16 acc0, acc1;
    const int bsrc = half * 32 + l32;                    // this lane's word of channel pair s: + 64 s
    auto tile = [&](auto has_prev, int p, floatx16 &cur, const floatx16 &prev) {
      constexpr bool kPrev = decltype(has_prev)::value;
      int dprev = 0;                                     // plane word of tile p - 1's position
      if (kPrev) {
        int hxr, hy;
        by_nhy.divmod((p - 1) * 32 + l32, hxr, hy);
        dprev = pl.sx * hxr * pl.Wp + pl.sy * hy;
      }
      wait_all_memory();
      __syncthreads();               // tile p has landed for every wavefront; the block of tile p - 1 is free
      const float *blk = Bs + (p % NBUF) * K * 32 + bsrc;
#pragma unroll
      for (int r = 0; r < 16; ++r) cur[r] = 0.f;
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        float v[4];
        if (kPrev) {
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = plane[dprev + off[4 * j + c4]];
        }
#pragma unroll
        for (int s = c4 * SPB; s < (c4 + 1) * SPB; ++s)
          cur = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], blk[64 * s], cur, 0, 0, 0);
        // the refill of tile p - 1's block is requested here, behind the first batch of
        // multiplies: its address arithmetic then runs while the matrix pipe is busy
        // instead of right after the barrier, when every wavefront of the CU would do it
        // at once with the pipe idle
        if (c4 == 0 && p >= 1 && p + 2 < ntiles) issue_tile(p + 2);
        if (kPrev) {
#pragma unroll
          for (int j = 0; j < 4; ++j) plane[dprev + off[4 * j + c4]] = v[j] + prev[4 * j + c4];
        }
      }
    };
    __syncthreads();                                     // zeroes are in place
    issue_tile(0);
    if (ntiles > 1) issue_tile(1);
    if (ntiles > 2) issue_tile(2);
    tile(std::false_type(), 0, acc0, acc1);
    int p = 1;
    for (; p + 1 < ntiles; p += 2) {
      tile(std::true_type(), p, acc1, acc0);
      tile(std::true_type(), p + 1, acc0, acc1);
    }
    if (p < ntiles) {
      tile(std::true_type(), p, acc1, acc0);
      acc0 = acc1;
      ++p;
    }
    // the last tile: not every position need exist
    {
      const int rel = (p - 1) * 32 + l32;
      int hxr, hy;
      by_nhy.divmod(rel, hxr, hy);
      const int d = pl.sx * hxr * pl.Wp + pl.sy * hy;
      if (q_lo + rel < q_end) {
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = plane[d + off[4 * j + c4]];
#pragma unroll
          for (int j = 0; j < 4; ++j) plane[d + off[4 * j + c4]] = v[j] + acc0[4 * j + c4];
        }
      }
    }
  } else {
  __syncthreads();                                     // zeroes are in place
  issue(0, 0);
  issue(0, KH);
  for (int c = 0; c < nchunks; ++c) {
    wait_all_memory();
    __syncthreads();                                   // chunk c has landed for every wavefront

    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
#pragma unroll
    for (int s = 0; s < KSTEPS / 2; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], Bs[bo[t] + 2 * s * P], acc[t], 0, 0, 0);
    __syncthreads();                                   // the first half is free
    if (c + 1 < nchunks) issue(c + 1, 0);
#pragma unroll
    for (int s = KSTEPS / 2; s < KSTEPS; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], Bs[bo[t] + 2 * s * P], acc[t], 0, 0, 0);
    __syncthreads();                                   // the second half is free
    if (c + 1 < nchunks) issue(c + 1, KH);
    if ((pl.nf & 31) == 0) fold(std::false_type(), c, acc);
    else fold(std::true_type(), c, acc);
  }
  }
  __syncthreads();

  // Write the rows this strip feeds: plane row i is grad_input row g0 + i, plane
  // column j is gy = j - py.  First, one thread per plane row works out where the
  // row goes: -1 nowhere (another strip owns it, or it lies outside grad_input),
  // 2 gx straight to grad_input, or 2 (slot index) + 1 a partial row in the workspace.
  // Rows between the reach of this strip and the first row of the next one (a
  // stride wider than the filter) are nobody's: they get zeros from here too.
  const int g0 = pl.sx * ha - pl.px;
  const int rp_t = max(pl.Rp, pl.sx * pl.Th);
  int *row_dst = (int *)Bs;                            // the chunk buffer is free now
  const StripMap map(pl);
  for (int pi = tid; pi < rp_t; pi += nthreads) {
    const int gx = g0 + pi;
    int code = -1;
    if (gx >= 0 && gx < pl.ngx) {
      int s_lo, s_hi;
      map.feeding(gx, s_lo, s_hi);
      if (s_lo == s_hi) {
        if (s_lo == strip) code = 2 * gx;
      } else if (strip == s_lo || strip == s_hi) {
        // boundary s_hi, row number within the boundary's shared rows, upper or lower strip
        const int r = gx - (pl.sx * s_hi * pl.Th - pl.px);
        code = 2 * (((s_hi - 1) * pl.nshared + r) * 2 + (strip - s_lo)) + 1;
      }
    }
    row_dst[pi] = code;
  }
  __syncthreads();
  {
    const int row_words = rp_t * pl.ngy;
    const FastDiv by_ngy(pl.ngy), by_rp(rp_t);
    const i64 nc0 = (i64)n * pl.c_in;
    for (int i = tid; i < pl.c_in * row_words; i += nthreads) {
      int r2, gy, cc, pi;
      by_ngy.divmod(i, r2, gy);
      by_rp.divmod(r2, cc, pi);
      const int code = row_dst[pi];
      if (code < 0 || !active) continue;
      float v = 0.f;
      if (pi < pl.Rp && gy + pl.py < pl.Wp) {
        const float *src = planes + cc * pl.mtn * plane_words + pi * pl.Wp + pl.py + gy;
        for (int m2 = 0; m2 < pl.mtn; ++m2) v += src[m2 * plane_words];
      }
      if (code & 1)
        WS[((nc0 + cc) * (pl.strips - 1) * pl.nshared * 2 + (code >> 1)) * pl.ngy + gy] = v;
      else
        GI[((nc0 + cc) * pl.ngx + (code >> 1)) * pl.ngy + gy] = v;
    }
  }
  // grad_input rows past the reach of the last grad_out row belong to the last strip: zeros
  if (strip == pl.strips - 1 && active) {
    const int z0 = max(0, g0 + rp_t);
    const int zrows = pl.ngx - z0;
    if (zrows > 0) {
      const i64 per_c = (i64)zrows * pl.ngy;
      for (i64 i = tid; i < pl.c_in * per_c; i += nthreads) {
        const i64 cc = i / per_c, w = i - cc * per_c;
        GI[(((i64)n * pl.c_in + cc) * pl.ngx + z0) * pl.ngy + w] = 0.f;
      }
    }
  }
}

// grad_input rows next to a strip boundary: upper strip's partial + lower strip's.
// One workgroup per (boundary, image * c_in + channel) sums that boundary's rows.
template <typename O>                                  // O: float, or _Float16 (the sum rounded once)
__global__ __launch_bounds__(256) void igrad_combine_kernel(const IgradPlan pl,
                                                            const float *__restrict__ WS,
                                                            O *__restrict__ GI) {
  const int b = blockIdx.x + 1;                        // boundary between strips b - 1 and b
  const i64 nc = blockIdx.y;
  const int g_b = pl.sx * b * pl.Th - pl.px;           // first row the boundary can share
  const float *src = WS + ((nc * (pl.strips - 1) + (b - 1)) * pl.nshared * 2) * pl.ngy;
  O *out = GI + nc * pl.ngx * pl.ngy;
  const StripMap map(pl);
  const FastDiv by_ngy(pl.ngy);
  for (int i = threadIdx.x; i < pl.nshared * pl.ngy; i += blockDim.x) {
    int r, gy;
    by_ngy.divmod(i, r, gy);
    const int gx = g_b + r;
    if (gx < 0 || gx >= pl.ngx) continue;
    int s_lo, s_hi;
    map.feeding(gx, s_lo, s_hi);
    if (s_lo == s_hi) continue;                        // not shared after clamping: written directly
    const float *p = src + (i64)r * 2 * pl.ngy + gy;
    out[(i64)gx * pl.ngy + gy] = (O)(p[0] + p[pl.ngy]);
  }
}

template <int KSTEPS, int NT, bool PIPE>
hipError_t launch_instance(const IgradPlan &pl, const float *w, const float *go, float *gi,
                           float *ws, hipStream_t stream) {
  auto kern = igrad_kernel<KSTEPS, NT, PIPE>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, pl.lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  const int groups = (pl.batch + pl.jobs - 1) / pl.jobs;
  hipLaunchKernelGGL(kern, dim3((unsigned)(groups * pl.strips)), dim3(64 * pl.units * pl.jobs),
                     pl.lds_bytes, stream, pl, w, go, gi, ws);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || pl.ws_bytes == 0) return e;
  hipLaunchKernelGGL(igrad_combine_kernel<float>,
                     dim3((unsigned)(pl.strips - 1), (unsigned)(pl.batch * pl.c_in)), dim3(256), 0,
                     stream, pl, ws, gi);
  return hipGetLastError();
}

// The same input gradient on the bf16 matrix cores (tile_stage.hpp: every fp32 operand as
// the exact sum of three bf16 parts, six products each), for layers whose taps fit one
// 32-row tile per input channel (nf <= 32, at most three input channels).
//
// One workgroup of four wavefronts per (image, strip); a wavefront takes a quarter of the
// strip's rows, 32 * NT positions at a time, and ALL input channels' taps of them:
//   * grad_out never touches LDS.  For tap products the reduction runs over the output
//     channels, so a lane's eight values of a step are eight channels of ONE position:
//     eight loads whose 32 lanes read 128 consecutive bytes.  They are requested one step
//     ahead and split in registers (every grad_out value is loaded and split once).
//   * the filter lives in LDS as fragments, built once per workgroup.
//   * a wavefront folds its products into a private LDS image of the grad_input rows its
//     positions reach (no other wavefront touches it); at the end the four images are added
//     up in wave order into the strip's image, which is written out exactly as above.
// F16: weight, grad_out and grad_input are half-precision storage and the products run on
// the f16 matrix cores (exact products, fp32 sums: one instruction where the bf16 form
// needs six, nothing to split); the images, and the partial rows in the workspace, stay
// fp32, and a result is rounded to half once.
template <int MTT, int NT, bool F16 = false>
__global__ __launch_bounds__(256, 2) void igrad_stream_kernel(const IgradPlan pl, const void *__restrict__ Wv,
                                                              const void *__restrict__ GOv,
                                                              void *__restrict__ GIv, float *__restrict__ WS) {
  typedef typename std::conditional<F16, _Float16, float>::type T;
  const T *W = (const T *)Wv, *GO = (const T *)GOv;
  T *GI = (T *)GIv;
  extern __shared__ __align__(16) float lds[];
  constexpr int P = NT * 32, ROWS = MTT * 32;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const int n = blockIdx.x / pl.strips, strip = blockIdx.x - n * pl.strips;
  const int ha = strip * pl.Th, hb = min(ha + pl.Th, pl.H);    // grad_out rows [ha, hb)
  // steps of 16 output channels, an even number of them (the two operand buffers alternate;
  // a step past c_out reads zeros on both sides)
  const int ksteps = ((pl.c_out + 31) >> 5) * 2, kgroups = 2 * ksteps;
  const int plane_words = pl.Rp * pl.Wp;                       // the strip's image, one input channel
  // (a wavefront's image has rows for all 32 matrix rows of a tile, also those past the last
  // tap: their products are exact zeros and are folded like the others, which keeps the
  // fold free of conditions)
  const int Rw = pl.sx * (pl.rw - 1) + pl.dx * (pl.nfx - 1) + 1;
  const int Rw_alloc = pl.sx * (pl.rw - 1) + pl.dx * (31 / pl.nfy) + 1;
  const int wplane_words = Rw_alloc * pl.Wp;                   // a wavefront's image, one input channel
  // LDS: filter fragments [3][kgroups][ROWS] (later the strip's image [c_in][Rp][Wp] and the
  // row table), then the wavefronts' images [4][c_in][Rw][Wp]
  uintx4 *Af = (uintx4 *)lds;
  const int af_part = kgroups * ROWS;
  const int head_words = max(12 * af_part, max(pl.Rp, pl.sx * pl.Th));
  float *wplanes = lds + ((head_words + 3) & ~3);
  float *myplane = wplanes + wave * pl.c_in * wplane_words;

  for (int i = tid; i < kWaves * pl.c_in * wplane_words; i += 256) wplanes[i] = 0.f;
  {
    // a thread splits the eight output channels k = 8 g .. 8 g + 7 of matrix row `row`
    // (tap m = row % 32 of input channel row / 32)
    const FastDiv by_rows(ROWS);
    for (int idx0 = tid; idx0 < kgroups * ROWS; idx0 += 4 * 256) {
      // four tasks at a time: all their loads are requested before the first is split
      T x[4][8];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = idx0 + u * 256;
        int g, row;
        by_rows.divmod(idx, g, row);
        const int ci = row >> 5, m = row & 31;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int k = 8 * g + i;
          x[u][i] = (idx < kgroups * ROWS && k < pl.c_out && ci < pl.c_in && m < pl.nf)
                        ? W[((i64)k * pl.c_in + ci) * pl.nf + m] : (T)0;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = idx0 + u * 256;
        int g, row;
        by_rows.divmod(idx, g, row);
        if (idx < kgroups * ROWS) {
          if constexpr (F16) {
            uintx4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i)
              v[i] = (unsigned)__builtin_bit_cast(unsigned short, x[u][2 * i]) |
                     ((unsigned)__builtin_bit_cast(unsigned short, x[u][2 * i + 1]) << 16);
            Af[g * ROWS + row] = v;                        // one part: the eight values themselves
          } else {
            store_frag(Af, kgroups, ROWS, g, row, x[u]);
          }
        }
      }
    }
  }
  // accumulator register r of this lane holds tap m(r); its offset in an image (-1: no such tap)
  int off[16];
  {
    const FastDiv by_nfy(pl.nfy);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = (r >> 2) * 8 + half * 4 + (r & 3);
      int fx, fy;
      by_nfy.divmod(m, fx, fy);
      off[r] = pl.dx * fx * pl.Wp + pl.dy * fy;             // (also for rows past the last tap: see Rw_alloc)
    }
  }
  // this wavefront's positions [q0, q1) of the image
  const int r0 = min(ha + wave * pl.rw, hb), r1 = min(r0 + pl.rw, hb);
  const int q0 = r0 * pl.nhy, q1 = r1 * pl.nhy;
  const int n_it = (q1 - q0 + P - 1) / P;
  const int total = n_it * ksteps;
  const T *GOn = GO + (i64)n * pl.c_out * pl.nh;
  const FastDiv by_nhy(pl.nhy);

  // step st = (iteration, 16 output channels): this lane's eight channels of NT positions.
  // Addresses are 32-bit byte offsets from the image's grad_out (the plan keeps c_out * nh
  // * 4 below 2^31): one add per load, no 64-bit arithmetic in the loop.
  typedef typename std::conditional<F16, unsigned short, float>::type BWord;
  struct BOp { BWord v[NT][8]; };
  // Buffer loads: a lane's byte offset within the image's grad_out is fixed for a tile
  // (position, and which eight of a step's channels), the channel's offset is wave-uniform
  // and travels in a scalar register, so a load costs no vector arithmetic; offsets past
  // the image's c_out * nh words (a last step reaching past c_out) read zeros.
  const __amdgpu_buffer_rsrc_t go_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)GOn, 0, pl.c_out * pl.nh * (int)sizeof(T), 0x00020000);
  const int nh4 = pl.nh * (int)sizeof(T);                  // bytes from a channel to the next
  auto load_b = [&](int it, int ks, BOp &o) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int q = min(q0 + it * P + t * 32 + l32, q1 - 1);   // past the range: any valid position, never folded
      const int voff = q * (int)sizeof(T) + 8 * half * nh4;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if constexpr (F16)
          o.v[t][i] = (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(go_rsrc, voff, (16 * ks + i) * nh4, 0);
        else
          o.v[t][i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(go_rsrc, voff, (16 * ks + i) * nh4, 0));
      }
    }
  };
  floatx16 acc[MTT][NT];
  // taps 4 j .. 4 j + 3 of a lane (registers r = 4 j + c) are filter columns fy0 + c of one filter
  // row when nfy is a multiple of 4; with dy = 1 they are four consecutive words of the image,
  // reached with immediate offsets from the first
  const bool quad = (pl.nfy & 3) == 0 && pl.dy == 1;
  // A step's operands as the matrix instructions take them: the filter's fragments of the step's
  // 16 channels and the cut grad_out values (F16: one part each, the values themselves).
  constexpr int kParts = F16 ? 1 : 3;
  struct AOp { uintx4 p[kParts][MTT]; };
  struct SOp { uintx4 p[kParts][NT]; };
  auto stage = [&](int ks, const BOp &o, AOp &a, SOp &s) {
    const uintx4 *af = Af + (2 * ks + half) * ROWS + l32;
#pragma unroll
    for (int part = 0; part < kParts; ++part)
#pragma unroll
      for (int m = 0; m < MTT; ++m) a.p[part][m] = af[part * af_part + m * 32];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if constexpr (F16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) s.p[0][t][i] = (unsigned)o.v[t][2 * i] | ((unsigned)o.v[t][2 * i + 1] << 16);
      } else {
        split8(o.v[t], s.p[0][t], s.p[1][t], s.p[2][t]);
      }
    }
  };
  auto multiply = [&](const AOp &a, const SOp &s) {
#pragma unroll
    for (int m = 0; m < MTT; ++m)
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if constexpr (F16)
          acc[m][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a.p[0][m]),
                                                             __builtin_bit_cast(halfx8, s.p[0][t]), acc[m][t], 0, 0, 0);
        else
          mfma_split6(acc[m][t], a.p[0][m], a.p[kParts > 1 ? 1 : 0][m], a.p[kParts > 1 ? 2 : 0][m],
                      s.p[0][t], s.p[kParts > 1 ? 1 : 0][t], s.p[kParts > 1 ? 2 : 0][t]);
      }
  };
  auto clear_sums = [&] {
#pragma unroll
    for (int m = 0; m < MTT; ++m)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[m][t][r] = 0.f;
  };
  auto fold_tiles = [&](int it) {
    {
      // fold: Z[tap, position] joins word base(position) + off(tap) of the input channel's image
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int rel = it * P + t * 32 + l32;              // position counted from q0
        if (q0 + rel < q1) {
          int hxr, hy;
          by_nhy.divmod(rel, hxr, hy);
          float *dst = myplane + pl.sx * hxr * pl.Wp + pl.sy * hy;
          // One filter column at a time (neighbouring positions share words across columns; the
          // four columns of a filter row sit at fixed distances from the first).  The images of
          // the input channels are different memory: their words of a column are read together,
          // added and written together, so that a tile's fold waits for LDS once per filter
          // column and not once per column and channel.
          if (quad) {
            float *pj[MTT][4];
#pragma unroll
            for (int a = 0; a < MTT; ++a)
#pragma unroll
              for (int j = 0; j < 4; ++j) pj[a][j] = dst + a * wplane_words + off[4 * j];
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
              float v[MTT][4];
#pragma unroll
              for (int a = 0; a < MTT; ++a)
#pragma unroll
                for (int j = 0; j < 4; ++j) v[a][j] = pj[a][j][c4];
#pragma unroll
              for (int a = 0; a < MTT; ++a)
#pragma unroll
                for (int j = 0; j < 4; ++j) pj[a][j][c4] = v[a][j] + acc[a][t][4 * j + c4];
            }
            continue;
          }
#pragma unroll
          for (int a = 0; a < MTT; ++a) {
            float *pa = dst + a * wplane_words;
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
              float v[4];
#pragma unroll
              for (int j = 0; j < 4; ++j) v[j] = pa[off[4 * j + c4]];
#pragma unroll
              for (int j = 0; j < 4; ++j) pa[off[4 * j + c4]] = v[j] + acc[a][t][4 * j + c4];
            }
          }
        }
      }
    }
  };
  __syncthreads();                                       // fragments and zeros are in place
  if (n_it > 0) {
    // Steps (tile, 16 output channels) in one sequence.  A step's grad_out values are requested
    // three steps ahead into a ring of four register sets, cut (and its fragments read from LDS)
    // while the step before it multiplies, and every part of that is pinned in place: left to
    // itself the scheduler moves each load next to its first use, and a step then waits for the
    // whole trip to memory.
    constexpr int D = 4;
    BOp ring[D];
    AOp A[2];
    SOp S[2];
    int it_req = 0, ks_req = 0, ks_stage = 0;
    auto request = [&](BOp &o) {
      load_b(min(it_req, n_it - 1), ks_req, o);          // (past the last step: a valid address, never used)
      if (++ks_req == ksteps) { ks_req = 0; ++it_req; }
    };
    auto stage_next = [&](const BOp &o, AOp &a, SOp &sv) {
      stage(ks_stage, o, a, sv);
      if (++ks_stage == ksteps) ks_stage = 0;
    };
    request(ring[0]);
    request(ring[1]);
    request(ring[2]);
    stage_next(ring[0], A[0], S[0]);
    clear_sums();
    int it = 0, ks = 0;
    for (int st = 0; st < total; st += D) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        if (st + u < total) {
          __builtin_amdgcn_sched_barrier(0);
          request(ring[(u + 3) & 3]);
          stage_next(ring[(u + 1) & 3], A[(u + 1) & 1], S[(u + 1) & 1]);   // (after the last step: cut and never used)
          multiply(A[u & 1], S[u & 1]);
          // the requests first, then after every matrix instruction a few of the next step's cuts and one fragment read
          __builtin_amdgcn_sched_group_barrier(0x020, 8 * NT, 0);
#pragma unroll
          for (int k = 0; k < MTT * NT * (F16 ? 1 : 6); ++k) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, F16 ? 8 : 4, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          if (++ks == ksteps) {
            fold_tiles(it);
            clear_sums();
            ks = 0;
            ++it;
          }
        }
      }
    }
  }
  __syncthreads();                                       // every wavefront's image is complete; the fragments are free

  // Write-out.  Row i of the strip's image is grad_input row g0 + i: the sum, in wave order,
  // of the rows of the wavefronts' images that reach it (wavefront w's image starts at row
  // sx * w * rw).  One thread per row first works out everything about the row: where it
  // goes (-1 nowhere: another strip owns it, or it lies outside grad_input; 0 straight to
  // grad_input; 1 a partial row in the workspace, upper strip's share first) at which word
  // of the image's grad_input or workspace slice, which wavefronts' images reach it and
  // where their rows lie.  Then every thread takes words of the strip's image, reading its
  // row's entry from the table.
  const int g0 = pl.sx * ha - pl.px;
  const int rp_t = max(pl.Rp, pl.sx * pl.Th);
  int4 *row_tab = (int4 *)lds;                           // kind, destination word, first image word, images
  const int wave_words = pl.c_in * wplane_words;         // from one wavefront's images to the next one's
  const int wave_step = wave_words - pl.sx * pl.rw * pl.Wp;   // ... to the same image row there
  {
    const StripMap map(pl);
    for (int pi = tid; pi < rp_t; pi += 256) {
      const int gx = g0 + pi;
      int kind = -1, dst = 0;
      if (gx >= 0 && gx < pl.ngx) {
        int s_lo, s_hi;
        map.feeding(gx, s_lo, s_hi);
        if (s_lo == s_hi) {
          if (s_lo == strip) { kind = 0; dst = gx * pl.ngy; }
        } else if (strip == s_lo || strip == s_hi) {
          // boundary s_hi, row number within the boundary's shared rows, upper or lower strip
          const int r = gx - (pl.sx * s_hi * pl.Th - pl.px);
          kind = 1;
          dst = (((s_hi - 1) * pl.nshared + r) * 2 + (strip - s_lo)) * pl.ngy;
        }
      }
      // wavefronts w0 .. w0 + nw - 1 have row pi in their images (none: a row past the reach of
      // the strip's last grad_out row, zeros)
      int w0 = 0, nw = 0;
      for (int w = 0; w < kWaves; ++w) {
        const int wr = pi - pl.sx * w * pl.rw;
        if (pi < pl.Rp && wr >= 0 && wr < Rw) { if (nw == 0) w0 = w; ++nw; }
      }
      row_tab[pi] = make_int4(kind, dst, w0 * wave_words + (pi - pl.sx * w0 * pl.rw) * pl.Wp, nw);
    }
  }
  __syncthreads();
  {
    const int gi_c = pl.ngx * pl.ngy, ws_c = (pl.strips - 1) * pl.nshared * 2 * pl.ngy;   // words per input channel
    T *GIn = GI + (i64)n * pl.c_in * gi_c;
    float *WSn = WS + (i64)n * pl.c_in * ws_c;
    // One word of the strip's image per thread and trip, (row, input channel, column) flattened with
    // the column fastest, four words in flight per thread: everything is per-lane vector code (the
    // row's table entry comes through an LDS read like the data), so nothing waits on a scalar.  A
    // word is the sum of at most reach_w wavefronts' images; words of wavefronts that do not hold
    // the row are read from the first one's and dropped.
    const int cols = pl.c_in * pl.ngy, words = rp_t * cols;
    const int reach_w = min(kWaves, (Rw + pl.sx * pl.rw - 1) / (pl.sx * pl.rw));   // images a row can lie in
    const float inv_cols = 1.0f / (float)cols, inv_ngy = 1.0f / (float)pl.ngy;
    // x / d without a branch (x below 2^22: the float quotient is off by one at most)
    auto quotient = [](int x, int d, float inv) {
      const int q = (int)((float)x * inv), r = x - q * d;
      return q + (r >= d ? 1 : 0) - (r < 0 ? 1 : 0);
    };
    constexpr int kFlight = 4;
    auto write_out = [&](auto reach_tag) {
      constexpr int kReach = decltype(reach_tag)::value;
      for (int e0 = tid; e0 < words; e0 += kFlight * 256) {
        int4 row[kFlight];
        int cc[kFlight], gy[kFlight];
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
          const int e = min(e0 + u * 256, words - 1);
          const int pi = quotient(e, cols, inv_cols), idx = e - pi * cols;
          cc[u] = quotient(idx, pl.ngy, inv_ngy);
          gy[u] = idx - cc[u] * pl.ngy;
          row[u] = row_tab[pi];
        }
        float x[kFlight][kReach];
        bool inside[kFlight];
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
          inside[u] = gy[u] + pl.py < pl.Wp;
          const float *in = wplanes + row[u].z + cc[u] * wplane_words + pl.py + (inside[u] ? gy[u] : 0);
#pragma unroll
          for (int k = 0; k < kReach; ++k) x[u][k] = in[k < row[u].w ? k * wave_step : 0];
        }
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
          float sum = 0.f;
#pragma unroll
          for (int k = 0; k < kReach; ++k) sum += (inside[u] && k < row[u].w) ? x[u][k] : 0.f;
          const int kind = e0 + u * 256 < words ? row[u].x : -1;
          const int dst = cc[u] * (kind > 0 ? ws_c : gi_c) + row[u].y + gy[u];
          if (kind > 0) WSn[dst] = sum;
          else if (kind == 0) GIn[dst] = (T)sum;
        }
      }
    };
    if (reach_w <= 2) write_out(std::integral_constant<int, 2>());
    else write_out(std::integral_constant<int, kWaves>());
  }
  // grad_input rows past the reach of the last grad_out row belong to the last strip: zeros
  if (strip == pl.strips - 1) {
    const int z0 = max(0, g0 + rp_t);
    const int zrows = pl.ngx - z0;
    if (zrows > 0) {
      const i64 per_c = (i64)zrows * pl.ngy;
      for (i64 i = tid; i < pl.c_in * per_c; i += 256) {
        const i64 cc = i / per_c, w = i - cc * per_c;
        GI[(((i64)n * pl.c_in + cc) * pl.ngx + z0) * pl.ngy + w] = (T)0;
      }
    }
  }
}

template <int MTT, int NT, bool F16 = false>
hipError_t launch_stream_instance(const IgradPlan &pl, const void *w, const void *go, void *gi,
                                  float *ws, hipStream_t stream) {
  auto kern = igrad_stream_kernel<MTT, NT, F16>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, pl.lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(pl.batch * pl.strips)), dim3(256), pl.lds_bytes, stream, pl, w, go, gi,
                     ws);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || pl.ws_bytes == 0) return e;
  const dim3 cgrid((unsigned)(pl.strips - 1), (unsigned)(pl.batch * pl.c_in));
  if (F16)
    hipLaunchKernelGGL(igrad_combine_kernel<_Float16>, cgrid, dim3(256), 0, stream, pl, (const float *)ws,
                       (_Float16 *)gi);
  else
    hipLaunchKernelGGL(igrad_combine_kernel<float>, cgrid, dim3(256), 0, stream, pl, (const float *)ws, (float *)gi);
  return hipGetLastError();
}

// Tap products for the gather-fold input gradient (any x axis kind):
//   Z[n, ci, m, q] = sum_co w[co, ci, m] * grad_out[n, co, q]
// Same operands, staging and work split over wavefronts as above; the
// accumulators are stored instead of folded.  A workgroup takes pl.cpw chunks
// of 64 positions of pl.jobs consecutive images.
//
// YF (plan.yfold): a lane's registers 4 g .. 4 g + 3 are the four filter columns fy of filter
// row fx = 2 g + (lane / 32) at the lane's position, and column fy of position q belongs to
// grad_input column hy(q) + fy - py: the sum over fy of a grad_input column takes the value of
// fy = k from the lane k positions back.  Positions are the flattened (hx, hy), so for the first
// three positions of a row "k positions back" reaches into the row before: those terms are
// that row's last three columns (nhy .. nhy + 2), and the lane stores them there.  A workgroup
// takes whole rows and three more positions, which produce the last row's tail; the values of
// the tile before (the three lanes a tile's first lanes reach back to) stay in registers.
template <int KSTEPS, bool YF>
__global__ __launch_bounds__(768) void tap_product_kernel(const TapProductPlan pl,
                                                          const float *__restrict__ W,
                                                          const float *__restrict__ GO,
                                                          float *__restrict__ Z) {
  extern __shared__ __align__(16) float lds[];
  constexpr int K = 2 * KSTEPS, P = 64, NT = 2, KH = K / 2;
  const int wave_in_group = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int job = wave_in_group / pl.units;
  const int wave = wave_in_group - job * pl.units;
  const int lane = threadIdx.x & 63;
  const int tid = wave * 64 + lane, nthreads = pl.units * 64;
  const int half = lane >> 5, l32 = lane & 31;
  const int groups_x = YF ? (pl.nhx + pl.rows_wg - 1) / pl.rows_wg : (pl.chunks_per_image + pl.cpw - 1) / pl.cpw;
  const int image_group = blockIdx.x / groups_x, chunk_group = blockIdx.x - image_group * groups_x;
  const int n_want = image_group * pl.jobs + job;
  const bool active = n_want < pl.batch;
  const int n = active ? n_want : pl.batch - 1;
  // positions [q_lo, q_hi) in chunks of 64 from q_lo (YF: whole rows, and three positions more)
  const int row_a = chunk_group * pl.rows_wg;
  const int q_lo = YF ? row_a * pl.nhy : chunk_group * pl.cpw * P;
  const int q_hi = YF ? min(pl.nhx, row_a + pl.rows_wg) * pl.nhy : pl.nh;
  const int nchunks = YF ? (q_hi - q_lo + 3 + P - 1) / P : min(pl.cpw, pl.chunks_per_image - chunk_group * pl.cpw);
  float *Bs = lds + job * K * P;
  const unsigned bs_addr = lds_address(lds) + 4u * (unsigned)(job * K * P);

  // channels past c_out and positions past the image are never loaded: keep them finite
  if (q_lo + nchunks * P > pl.nh) {
    for (int i = tid; i < K * P; i += nthreads) Bs[i] = 0.f;
  } else {
    for (int i = pl.c_out * P + tid; i < K * P; i += nthreads) Bs[i] = 0.f;
  }
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
  const float *GOn = GO + (i64)n * pl.c_out * pl.nh;
  const int row_in = lane >> 4, seg = lane & 15;          // 16 lanes x 16 bytes per channel row
  auto issue = [&](int c, int k_lo) {                     // channels [k_lo, k_lo + KH) of chunk c
    const int q0 = q_lo + c * P;
    const int k_hi = min(k_lo + KH, pl.c_out);
    if (q0 + P <= pl.nh && (q0 & 3) == 0) {                // (16-byte pieces)
      for (int k0 = k_lo + wave * 4; k0 < k_hi; k0 += pl.units * 4) {
        const int k = k0 + row_in;
        const unsigned voff = (unsigned)(row_in * pl.nh + q0 + 4 * (seg ^ ((k & 1) << 3))) * 4u;
        if (k < k_hi) load16_to_lds_at(GOn + (i64)k0 * pl.nh, voff, bs_addr + 4u * (unsigned)(k0 * P));
      }
    } else {
      for (int k = k_lo + wave; k < k_hi; k += pl.units) {
        const int q = q0 + (lane ^ ((k & 1) << 5));
        if (q < pl.nh) load_to_lds_at(GOn + (i64)k * pl.nh, (unsigned)q * 4u, bs_addr + 4u * (unsigned)(k * P));
      }
    }
  };
  int bo[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) bo[t] = half * P + ((t ^ half) << 5) + l32;
  // rows of Z this lane stores: tap m(r) of input channel ci
  float *Zrow = Z + ((i64)(n * pl.c_in + ci) * pl.nf_pad + mt * 32 + half * 4) * pl.nh;
  const int m_base = mt * 32 + half * 4;

  // YF: columns fy = 1, 2, 3 of the tile before (zeros at the start of the rows)
  float prev[4][3];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int k = 0; k < 3; ++k) prev[g][k] = 0.f;
  const FastDiv by_nhy(YF ? pl.nhy : 1);

  __syncthreads();
  issue(0, 0);
  issue(0, KH);
  for (int c = 0; c < nchunks; ++c) {
    wait_all_memory();
    __syncthreads();
    floatx16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
#pragma unroll
    for (int s = 0; s < KSTEPS / 2; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], Bs[bo[t] + 2 * s * P], acc[t], 0, 0, 0);
    __syncthreads();                                   // the first half is free
    if (c + 1 < nchunks) issue(c + 1, 0);
#pragma unroll
    for (int s = KSTEPS / 2; s < KSTEPS; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], Bs[bo[t] + 2 * s * P], acc[t], 0, 0, 0);
    __syncthreads();                                   // the second half is free
    if (c + 1 < nchunks) issue(c + 1, KH);
    if constexpr (YF) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int q = q_lo + c * P + t * 32 + l32;
        const bool real = q < q_hi;
        int hx, hy;
        by_nhy.divmod(q, hx, hy);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float z[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) z[j] = real ? acc[t][4 * g + j] : 0.f;
          float same = z[0], tail = 0.f;
#pragma unroll
          for (int k = 1; k < 4; ++k) {
            const int from = ((half << 5) | ((l32 - k) & 31)) << 2;       // the lane k positions back, in this tile or the one before
            const float cur = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(z[k])));
            const float old = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(prev[g][k - 1])));
            const float v = l32 >= k ? cur : old;
            if (hy >= k) same += v;
            else tail += v;
          }
#pragma unroll
          for (int k = 1; k < 4; ++k) prev[g][k - 1] = z[k];
          const int fx = mt * 8 + 2 * g + half;
          if (active && fx < pl.nfx) {
            float *Yc = Z + ((i64)(n * pl.c_in + ci) * pl.nfx + fx) * pl.nhx * pl.ngy;
            const int gy = hy - pl.py;
            if (real && gy >= 0 && gy < pl.ngy) Yc[(i64)hx * pl.ngy + gy] = same;
            const int gt = pl.nhy + hy - pl.py;                            // the row before: its columns past nhy - 1
            if (hy < 3 && hx > row_a && q < q_hi + 3 && gt >= 0 && gt < pl.ngy) Yc[(i64)(hx - 1) * pl.ngy + gt] = tail;
          }
        }
      }
    } else if (active) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int q = q_lo + c * P + t * 32 + l32;
        if (q < pl.nh) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int dm = (r >> 2) * 8 + (r & 3);
            if (m_base + dm < pl.nf) Zrow[(i64)dm * pl.nh + q] = acc[t][r];
          }
        }
      }
    }
  }
}

template <int KSTEPS>
hipError_t launch_tap_product_instance(const TapProductPlan &pl, const float *w, const float *go,
                                       float *z, hipStream_t stream) {
  auto kern = pl.yfold ? tap_product_kernel<KSTEPS, true> : tap_product_kernel<KSTEPS, false>;
  {
    static std::atomic<int> lds_allowed[2] = {{0}, {0}};   // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, pl.lds_bytes, lds_allowed[pl.yfold ? 1 : 0]);
    if (e != hipSuccess) return e;
  }
  const int groups_x = pl.yfold ? (pl.nhx + pl.rows_wg - 1) / pl.rows_wg : (pl.chunks_per_image + pl.cpw - 1) / pl.cpw;
  const int image_groups = (pl.batch + pl.jobs - 1) / pl.jobs;
  hipLaunchKernelGGL(kern, dim3((unsigned)(image_groups * groups_x)), dim3(64 * pl.units * pl.jobs),
                     pl.lds_bytes, stream, pl, w, go, z);
  return hipGetLastError();
}

}  // namespace

bool make_tap_product_plan(i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 nhx, i64 nhy,
                           TapProductPlan &pl) {
  const i64 nf = nfx * nfy, nh = nhx * nhy;
  if (batch < 1 || c_in < 1 || c_out < 1 || nf < 1 || nh < 1) return false;
  const i64 lim = (i64)1 << 28;
  if (nh >= lim || c_out * c_in * nf >= lim || batch * c_in >= lim) return false;
  const i64 mtn = (nf + 31) / 32, units = c_in * mtn;
  // few input channels, and taps that fill at least a quarter of their 32-row tiles
  // (even a half-empty tile beats the gather form, whose tiles hold c_in rows)
  if (c_in >= 16 || units > 8 || mtn * 32 > nf * 4 || c_out > 128) return false;
  pl.batch = (int)batch; pl.c_in = (int)c_in; pl.c_out = (int)c_out;
  pl.nf = (int)nf; pl.nh = (int)nh;
  pl.mtn = (int)mtn; pl.units = (int)units; pl.nf_pad = (int)mtn * 32;
  pl.ksteps = c_out <= 32 ? 16 : c_out <= 64 ? 32 : 64;
  const int max_waves = pl.ksteps == 64 ? 8 : 12;
  if (units > max_waves) return false;
  // One image per workgroup: workgroups of a few wavefronts, several to a CU, spread over the
  // chip more evenly than one large workgroup per CU and do not all wait for memory at once.
  pl.jobs = 1;
  pl.chunks_per_image = (int)((nh + 63) / 64);
  // chunks per workgroup: one, unless that makes more workgroups than the chip holds at once
  const i64 image_groups = batch;
  i64 cpw = (image_groups * pl.chunks_per_image + 2047) / 2048;
  pl.cpw = (int)std::max<i64>(1, std::min<i64>(cpw, pl.chunks_per_image));
  pl.lds_bytes = 4 * (size_t)(2 * pl.ksteps * 64) * pl.jobs;
  pl.ws_bytes = 4 * (size_t)batch * c_in * pl.nf_pad * nh;
  if (image_groups * ((pl.chunks_per_image + pl.cpw - 1) / pl.cpw) >= ((i64)1 << 31)) return false;
  pl.yfold = 0;
  pl.nfx = (int)nfx; pl.nhx = (int)nhx; pl.nhy = (int)nhy; pl.ngy = 0; pl.py = 0; pl.rows_wg = 1;
  return true;
}

void enable_tap_yfold(TapProductPlan &pl, i64 nfx, i64 nfy, i64 nhx, i64 nhy, i64 ngy, i64 sy, i64 dy, i64 py,
                      i64 uy) {
  // (rows of at least three positions: "k positions back" then reaches the row before at most)
  if (nfy != 4 || sy != 1 || dy != 1 || uy != 1 || py < 0 || ngy > nhy + 3 - py || ngy < 1 || nhy < 3) return;
  if (nhx * nhy + 64 >= ((i64)1 << 22) || pl.jobs != 1) return;          // (float-reciprocal index split)
  // rows per workgroup: a multiple of what keeps a workgroup's first position a multiple of
  // four (16-byte loads); among those that leave the chip two workgroups per CU, the one
  // whose rows (and three positions more) fill their 64-position chunks best
  const i64 step = nhy % 4 == 0 ? 1 : (nhy % 2 == 0 ? 2 : 4);
  i64 best = step;
  double best_fill = 0;
  for (i64 r = step; r <= 16 * step && r <= std::max<i64>(nhx, step); r += step) {
    const i64 wgs = pl.batch * ((nhx + r - 1) / r);
    const double fill = (double)(r * nhy) / (double)(64 * ((r * nhy + 3 + 63) / 64));
    if (r > step && wgs < 512) break;
    if (fill > best_fill + 1e-9) { best = r; best_fill = fill; }
  }
  if ((double)pl.batch * ((nhx + best - 1) / best) >= (double)((i64)1 << 31)) return;
  pl.yfold = 1;
  pl.ngy = (int)ngy; pl.py = (int)py; pl.rows_wg = (int)best;
  pl.ws_bytes = 4 * (size_t)pl.batch * pl.c_in * nfx * nhx * ngy;
}

hipError_t launch_tap_product(const TapProductPlan &pl, const float *weight, const float *grad_out,
                              float *z, hipStream_t stream) {
  if (pl.ksteps == 16) return launch_tap_product_instance<16>(pl, weight, grad_out, z, stream);
  if (pl.ksteps == 32) return launch_tap_product_instance<32>(pl, weight, grad_out, z, stream);
  if (pl.ksteps == 64) return launch_tap_product_instance<64>(pl, weight, grad_out, z, stream);
  return hipErrorInvalidValue;
}

bool make_igrad_plan(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx,
                     i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py,
                     i64 ux, i64 uy, IgradPlan &pl, int force_nt, int force_Th, int force_pipe, int math) {
  if (kind_x != AX_LCORR || ux != 1 || uy != 1) return false;
  if (px < 0 || py < 0) return false;
  const i64 nf = nfx * nfy, nh = nhx * nhy, ng = ngx * ngy;
  if (batch < 1 || c_in < 1 || c_out < 1 || nf < 1 || nh < 1 || ng < 1) return false;
  const i64 lim = (i64)1 << 28;
  if (nh >= lim || ng >= lim || c_out * c_in * nf >= lim) return false;
  if (sx >= 4096 || sy >= 4096 || dx >= 4096 || dy >= 4096 || px >= lim || py >= lim) return false;
  // few input channels, and taps that fill at least a quarter of their 32-row tiles
  // (even a half-empty tile beats the gather form, whose tiles hold c_in rows)
  const i64 mtn = (nf + 31) / 32;
  const i64 units = c_in * mtn;
  if (c_in >= 16 || units > 8 || mtn * 32 > nf * 4) return false;
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
  // streaming variant: needs batches that cannot collide and no padded matrix rows
  pl.pipe = pl.batched_fold && (nf & 31) == 0 && force_pipe != 0;
  const i64 K = 2 * pl.ksteps;
  const i64 Wp = sy * (nhy - 1) + dy * (nfy - 1) + 1;
  const i64 reach = dx * (nfx - 1);
  if (Wp >= 4096) return false;
  // grad_out rows with a tap inside grad_input
  const i64 H = std::min(nhx, (ngx - 1 + px) / sx + 1);
  if (H < 1) return false;
  // Strip height: about four workgroups per CU (1024 in all), and taller than a
  // filter's reach so that a grad_input row is fed by at most two strips.
  const i64 min_th = reach / sx + 1;
  const i64 want_strips = std::max<i64>(1, (1024 + batch - 1) / batch);
  i64 Th = std::max<i64>((H + want_strips - 1) / want_strips, std::max<i64>(min_th, 2));
  if (force_Th > 0) Th = std::max<i64>(force_Th, min_th);
  Th = std::min(Th, std::max(H, min_th));
  pl.stream = 0;
  pl.rw = 0;
  if (math != MATH_FP32 && mtn == 1 && c_in <= 3 && (nf & 7) == 0 && c_out * nh < ((i64)1 << 29) &&
      pl.batched_fold && force_nt == 0 && force_Th == 0 &&
      force_pipe != 0 && ngx + px + reach + sx < ((i64)1 << 22) && batch * c_in <= 65535 &&
      (reach - sx + 1) * ngy < ((i64)1 << 22)) {
    // The bf16 form (igrad_stream_kernel): four wavefronts per (image, strip), rw rows each.
    // Pick rw for the fewest rounds of workgroups times 64-position passes per wavefront.
    const i64 kgroups = 4 * ((c_out + 31) / 32), rows = c_in * 32;
    double best = 0;
    for (i64 rw = 1; rw <= 32; ++rw) {
      const i64 Th_s = 4 * rw;
      if (Th_s < std::max<i64>(min_th, 2)) continue;
      const i64 Rw = sx * (rw - 1) + reach + 1, Rp = sx * (Th_s - 1) + reach + 1;
      if ((Th_s + 2) * nhy >= ((i64)1 << 22) || c_in * std::max(Rp, sx * Th_s) * ngy >= ((i64)1 << 22)) break;
      const i64 head = std::max<i64>(12 * kgroups * rows, std::max(Rp, sx * Th_s));
      const i64 Rw_alloc = sx * (rw - 1) + dx * (31 / nfy) + 1;     // rows for all 32 matrix rows of a tile
      const size_t lds = 4 * (size_t)(((head + 3) & ~(i64)3) + 4 * c_in * Rw_alloc * Wp);
      if (lds > 150 * 1024) break;
      const i64 per_cu = lds + 512 <= 80 * 1024 ? 2 : 1;
      const i64 strips = (H + Th_s - 1) / Th_s, wgs = batch * strips;
      const i64 tile = c_in == 1 ? 64 : 32;                       // positions per pass (registers)
      const i64 rounds = (wgs + 256 * per_cu - 1) / (256 * per_cu), passes = (rw * nhy + tile - 1) / tile * tile / 32;
      // (a workgroup alone on its CU runs at about 0.6 of the rate of two)
      // (setting up and writing out cost a workgroup about as much as two passes)
      const double rate = (double)(batch * H * nhy) / ((double)rounds * (passes + 2) * (per_cu == 2 ? 1.0 : 1.2));
      if (rate > best * 1.02) {
        best = rate;
        pl.stream = 1; pl.rw = (int)rw; pl.nt = c_in == 1 ? 2 : 1; pl.jobs = 1;
        pl.Th = (int)Th_s; pl.H = (int)H; pl.strips = (int)strips;
        pl.Rp = (int)Rp; pl.Wp = (int)Wp; pl.lds_bytes = lds;
        pl.nshared = (int)std::max<i64>(0, reach - sx + 1);
        pl.ws_bytes = pl.strips > 1 && pl.nshared > 0
                          ? 4 * (size_t)batch * c_in * (pl.strips - 1) * pl.nshared * 2 * ngy : 0;
      }
    }
    if (pl.stream && (i64)pl.batch * pl.strips < ((i64)1 << 31)) return true;
    pl.stream = 0;
  }
  // jobs per workgroup: make the wavefront count a multiple of four when that fits
  const int max_waves = pl.ksteps == 64 ? 8 : 12;      // registers: see the launch bounds
  pl.jobs = 1;
  for (int j = 1; j <= 4; ++j)
    if ((j * units) % 4 == 0 && j * units <= max_waves && j <= batch) { pl.jobs = j; break; }
  if (units > max_waves) return false;
  for (; Th >= min_th; Th = (Th > 8 ? Th * 3 / 4 : Th - 1)) {
    const i64 Rp = sx * (Th - 1) + reach + 1;
    if ((Th + 2) * nhy >= ((i64)1 << 22)) continue;              // float-reciprocal index splits
    if (ngx + px + reach + sx >= ((i64)1 << 22) || batch * c_in > 65535) return false;
    if ((reach - sx + 1) * ngy >= ((i64)1 << 22)) return false;
    if (c_in * std::max(Rp, sx * Th) * ngy >= ((i64)1 << 22) || std::max(Rp, sx * Th) > K * 64) continue;
    // chunk buffer: three 32-position blocks when streaming, else one chunk of 64 or
    // (when the planes are small) 128 positions
    int nt = 2;
    if (!pl.pipe && (force_nt == 4 || (force_nt == 0 && 4 * (K * 128 + units * Rp * Wp) * pl.jobs <= 40 * 1024)))
      nt = 4;
    const i64 job_words = ((K * (pl.pipe ? 96 : nt * 32) + units * Rp * Wp) + 3) & ~(i64)3;
    const size_t lds = 4 * (size_t)job_words * pl.jobs;
    if (lds > 160 * 1024 - 512) continue;
    pl.nt = nt; pl.Th = (int)Th; pl.H = (int)H; pl.strips = (int)((H + Th - 1) / Th);
    pl.Rp = (int)Rp; pl.Wp = (int)Wp; pl.lds_bytes = lds;
    pl.nshared = (int)std::max<i64>(0, reach - sx + 1);
    pl.ws_bytes = pl.strips > 1 && pl.nshared > 0
                      ? 4 * (size_t)batch * c_in * (pl.strips - 1) * pl.nshared * 2 * ngy : 0;
    if ((i64)pl.batch * pl.strips >= ((i64)1 << 31)) return false;
    if ((i64)batch * c_in * pl.strips * pl.nshared * 2 * ngy >= ((i64)1 << 40)) return false;
    return true;
  }
  return false;
}

hipError_t launch_igrad_half(const IgradPlan &pl, const void *weight, const void *grad_out,
                             void *grad_input, float *workspace, hipStream_t stream) {
  if (!pl.stream) return hipErrorInvalidValue;
  if (pl.c_in == 1) return launch_stream_instance<1, 2, true>(pl, weight, grad_out, grad_input, workspace, stream);
  if (pl.c_in == 2) return launch_stream_instance<2, 1, true>(pl, weight, grad_out, grad_input, workspace, stream);
  return launch_stream_instance<3, 1, true>(pl, weight, grad_out, grad_input, workspace, stream);
}

hipError_t launch_igrad(const IgradPlan &pl, const float *weight, const float *grad_out,
                        float *grad_input, float *workspace, hipStream_t stream) {
  if (pl.stream) {
    if (pl.c_in == 1) return launch_stream_instance<1, 2>(pl, weight, grad_out, grad_input, workspace, stream);
    if (pl.c_in == 2) return launch_stream_instance<2, 1>(pl, weight, grad_out, grad_input, workspace, stream);
    return launch_stream_instance<3, 1>(pl, weight, grad_out, grad_input, workspace, stream);
  }
  // the pipelined fold needs batches that cannot collide and no padded matrix rows
  const bool pipe = pl.pipe && pl.nt == 2;
#define MELLIN_IGRAD_CASE(KS, NT_)                                                       \
  if (pl.ksteps == KS && pl.nt == NT_)                                                   \
    return pipe ? launch_instance<KS, NT_, (NT_ == 2)>(pl, weight, grad_out, grad_input, workspace, stream) \
                : launch_instance<KS, NT_, false>(pl, weight, grad_out, grad_input, workspace, stream);
  MELLIN_IGRAD_CASE(16, 2) MELLIN_IGRAD_CASE(16, 4)
  MELLIN_IGRAD_CASE(32, 2) MELLIN_IGRAD_CASE(32, 4)
  MELLIN_IGRAD_CASE(64, 2) MELLIN_IGRAD_CASE(64, 4)
#undef MELLIN_IGRAD_CASE
  return hipErrorInvalidValue;
}

}  // namespace mellin
