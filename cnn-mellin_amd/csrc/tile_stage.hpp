// Device-side pieces shared by the matrix-core kernels: direct global->LDS
// loads, division-free index splitting, position-tile geometry, and the staging
// of signal rows into affine "virtual rows" (see tile_gemm.hip).
#pragma once

#include "mellin_common.hpp"
#include "tile_gemm.hpp"

namespace mellin {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kNarrowRow = 17;                     // staged rows this short are loaded 64 words at a time

typedef __attribute__((address_space(3))) float *lds_float_ptr;

// LDS byte address of a pointer into shared memory (what m0 must hold).
__device__ __forceinline__ unsigned lds_address(const float *p) {
  return (unsigned)(size_t)(lds_float_ptr)p;
}

// Sixteen bytes per active lane: lane l reads the four dwords at `base` +
// `byte_offset` (any 4-byte alignment) and they land at LDS byte address
// `lds_addr` + 16 * l (`lds_addr` wave-uniform; 4-byte alignment is enough).
__device__ __forceinline__ void load16_to_lds_at(const float *base, unsigned byte_offset, unsigned lds_addr) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  const unsigned long long b = (unsigned long long)base;
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  const unsigned long long sbase = ((unsigned long long)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(m0v), "v"(byte_offset), "s"(sbase) : "memory");
}

// One dword per active lane straight from global memory to LDS: lane l reads
// the dword at `base` + `byte_offset` (base wave-uniform, offset per lane) and
// it lands at LDS byte address `lds_addr` + 4 * l (`lds_addr` wave-uniform).
// Completion is counted by vmcnt.  Written as inline assembly on purpose: the
// compiler then does not order later LDS reads after these loads, which is
// what lets the loads of the next stage stay in flight during the matrix
// loop; every consumer waits explicitly (wait_all_memory + barrier).  m0
// carries the LDS base.  Destinations are passed as addresses, not pointers.
// EB = 2: the element in memory is 16 bits wide (any 2-byte alignment) and arrives
// zero-extended, still one element per LDS word.
template <int EB = 4>
__device__ __forceinline__ void load_to_lds_at(const void *base, unsigned byte_offset, unsigned lds_addr) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  const unsigned long long b = (unsigned long long)base;
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  const unsigned long long sbase = ((unsigned long long)hi << 32) | lo;
  if (EB == 2)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2"
                 :: "s"(m0v), "v"(byte_offset), "s"(sbase) : "memory");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(m0v), "v"(byte_offset), "s"(sbase) : "memory");
}

__device__ __forceinline__ void wait_all_memory() {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
}

// x / d for 0 <= x < 2^31 and d >= 1 with m = floor(2^32 / d) (0xFFFFFFFF for d = 1):
// the product's high word is the quotient or one less.  On wave-uniform values this
// is a handful of scalar instructions; a plain integer division goes through the
// vector unit's reciprocal, and vector instructions queue behind the matrix ones.
__device__ __forceinline__ int udiv(int x, int d, unsigned m) {
  unsigned q = __umulhi((unsigned)x, m);
  if ((unsigned)x - q * (unsigned)d >= (unsigned)d) ++q;
  return (int)q;
}

// Signal row chosen by (output row, filter row) on a Mellin axis, in 32-bit
// arithmetic (the plan guarantees that the products fit).  p1 = p + 1.
// mg_p1 = floor(2^32 / p1) (0xFFFFFFFF for p1 = 1).
__device__ __forceinline__ int mellin_tap32(int kind, int h, int f, int ng, int s, int d, int p1, int u,
                                            unsigned mg_p1) {
  int num, den;
  int q;
  if (kind == AX_MCORR) {
    // the divisor is the same for every tap: multiply-high by its reciprocal
    num = (h + s) * (f + d); den = p1;
    q = udiv(num, p1, mg_p1);
  } else {
    num = p1 * (h + s); den = f + d;
    q = num / den;
  }
  if (q * den != num) return -1;
  const int g = q - u;
  return (g >= 0 && g < ng) ? g : -1;
}

// n / d and n % d for 0 <= n < 2^22, d >= 1, without an integer divide.
struct FastDiv {
  int d;
  float inv;
  __device__ explicit FastDiv(int d_) : d(d_), inv(1.0f / (float)d_) {}
  __device__ __forceinline__ void divmod(int n, int &q, int &r) const {
    q = (int)((float)n * inv);
    r = n - q * d;
    if (r < 0) { --q; r += d; }
    else if (r >= d) { ++q; r -= d; }
  }
};

// Uniform description of one position tile.
struct TileGeom {
  int n, q0, count, ox_lo, oy_lo, R_tile, RSL, vx_min, vy_min;
};

// (PL: TilePlan in whatever address space the caller holds it)
template <int P, class PL>
__device__ __forceinline__ TileGeom tile_geometry(const PL &pl, int tile_id, bool mellin_x) {
  TileGeom g;
  g.n = udiv(tile_id, pl.tiles_per_image, pl.mg_tpi);
  const int tile = tile_id - g.n * pl.tiles_per_image;
  int ox_hi, oy_hi;
  if (pl.segment) {
    g.ox_lo = ox_hi = udiv(tile, pl.chunks_per_row, pl.mg_cpr);
    g.oy_lo = (tile - g.ox_lo * pl.chunks_per_row) * P;
    g.count = min(P, pl.noy - g.oy_lo);
    oy_hi = g.oy_lo + g.count - 1;
    g.q0 = g.ox_lo * pl.noy + g.oy_lo;
  } else {
    g.q0 = tile * P;
    g.count = min(P, pl.Q - g.q0);
    g.ox_lo = udiv(g.q0, pl.noy, pl.mg_noy);
    ox_hi = udiv(g.q0 + g.count - 1, pl.noy, pl.mg_noy);
    g.oy_lo = 0;
    oy_hi = pl.noy - 1;
  }
  const int rows = ox_hi - g.ox_lo + 1;
  g.R_tile = mellin_x ? rows * pl.nfx : pl.ax * (rows - 1) + pl.bx_span + 1;
  g.vx_min = pl.ax * g.ox_lo + pl.cx + pl.bx_min;         // linear x only
  g.vy_min = pl.ay * g.oy_lo + pl.cy + pl.by_min;
  g.RSL = pl.ay * (oy_hi - g.oy_lo) + pl.by_span + 1;     // staged columns
  return g;
}


// ---- signal rows of one (tile, channel range) --------------------------------
// Where a staged word comes from depends on the tile, not on the channel, and a
// layer with many channels stages the same tile once per chunk of channels: a
// wave can keep what it worked out for the tile's first chunk (a few registers
// per lane) and spend the later chunks on load instructions only.
template <int MB>                                  // MB: 64-word blocks per wave whose sources are kept
struct StageMemo {
  int row_src, row_dst;                            // row-wise staging: lane j <-> the wave's j-th row
  int word_src[MB > 0 ? MB : 1];                   // word-wise staging: lane's word of the wave's b-th block
};

// The same LDS target in every channel of a chunk: channel cl reads cl * g_c elements
// (of EB bytes) further on and lands cl planes further on.
#define MELLIN_CHANNEL_LOADS(INSTR)                                                                         \
  for (; cl + 4 <= cc; cl += 4) {                    /* four channels per block of straight-line code */   \
    asm volatile("s_mov_b32 m0, %1\n\tv_add_u32 %0, %0, %2\n\t" INSTR " %0, %3\n\t"                       \
                 "s_add_u32 m0, m0, %4\n\tv_add_u32 %0, %0, %2\n\t" INSTR " %0, %3\n\t"                   \
                 "s_add_u32 m0, m0, %4\n\tv_add_u32 %0, %0, %2\n\t" INSTR " %0, %3\n\t"                   \
                 "s_add_u32 m0, m0, %4\n\tv_add_u32 %0, %0, %2\n\t" INSTR " %0, %3"                        \
                 : "+v"(v) : "s"(m0v), "s"(step), "s"(sbase), "s"(pb) : "memory", "scc");                  \
    m0v = __builtin_amdgcn_readfirstlane(m0v + 4u * pb);                                                   \
  }                                                                                                         \
  for (; cl < cc; ++cl) {                                                                                   \
    asm volatile("s_mov_b32 m0, %1\n\tv_add_u32 %0, %0, %2\n\t" INSTR " %0, %3"                            \
                 : "+v"(v) : "s"(m0v), "s"(step), "s"(sbase) : "memory");                                   \
    m0v = __builtin_amdgcn_readfirstlane(m0v + pb);                                                        \
  }
template <int EB = 4>
__device__ __forceinline__ void load_channels(const void *base, int g_c, unsigned voff, unsigned lds_addr,
                                              unsigned plane_bytes, int cc) {
  // One instruction slot is all a staging wavefront gets between the matrix instructions of
  // its SIMD's other wavefront, so the loop is cut to what it needs: the LDS target goes to
  // M0, the lane's byte offset moves on by a channel (which also fills the wait state that
  // M0 wants before the load), the load.  (Offsets stay below 2^32: callers check
  // cc * g_c < 2^30.)
  const unsigned long long b = (unsigned long long)base;
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  const unsigned long long sbase = ((unsigned long long)hi << 32) | lo;
  const unsigned step = __builtin_amdgcn_readfirstlane((unsigned)EB * (unsigned)g_c);
  const unsigned pb = __builtin_amdgcn_readfirstlane(plane_bytes);
  unsigned v = voff - step;
  unsigned m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  cc = __builtin_amdgcn_readfirstlane(cc);           // wave-uniform: say so, or the loop's scalars end up in vector registers
  int cl = 0;
  if (EB == 2) { MELLIN_CHANNEL_LOADS("global_load_lds_ushort") }
  else { MELLIN_CHANNEL_LOADS("global_load_lds_dword") }
}
#undef MELLIN_CHANNEL_LOADS
__device__ __forceinline__ void zero_channels(float *at, int plane, int cc) {
  for (int cl = 0; cl < cc; ++cl) { *at = 0.f; at += plane; }
}

// wave w of the NW that stage together owns virtual rows w, w + NW, ...; 64 lanes
// first work out the source of 64 such rows, then direct loads are issued per row
// with the lanes on columns; columns or rows without a source are written as zeros.
// Words without a source are written only when `fresh` (the buffer last held
// another tile: within a tile the same words are zeros in every chunk).  MB > 0:
// `memo` carries the tile's sources from the call with new_tile set to the calls
// for the tile's other chunks.  MB < 0: no memo, and everything is written on
// every call.
// EB: bytes per element of G (4: float; 2: half precision, staged zero-extended, one
// element per LDS word like the floats)
template <int NW = kWaves, int MB = -1, int EB = 4, class PL>
__device__ __forceinline__ void issue_signal(const PL &pl, const TileGeom &tg,
                                             const void *__restrict__ G, int c0, int cc,
                                             float *Gs, unsigned gs_addr, bool mellin_x, int lane,
                                             int wave, StageMemo<MB> *memo = nullptr, bool new_tile = true,
                                             bool fresh = true) {
  const char *Gimg = (const char *)G + ((i64)tg.n * pl.g_n + (i64)c0 * pl.g_c) * EB;
  const int g_c = (int)pl.g_c;                         // fits: c_in * ngx * ngy < 2^31
  constexpr bool MEMO = MB > 0;
  if (MB < 0) fresh = true;
  if (!MEMO) new_tile = true;
  if (EB == 4 && pl.contig && tg.vx_min >= 0 && tg.vx_min + tg.R_tile <= pl.ngx) {
    // the virtual rows ARE the signal rows vx_min ... of each channel, with the
    // signal's own row pitch: one run of R_tile * ngy words per channel, moved
    // 16 bytes per lane (1 KB per instruction), the pieces dealt out to the waves
    const int count = tg.R_tile * pl.ngy, count4 = count & ~3;
    const int pieces = (count4 + 255) >> 8;
    const float *src0 = (const float *)Gimg + tg.vx_min * pl.ngy;
    for (int cl = 0, pc = wave; pieces > 0; pc += NW) {    // piece pc of channel cl; pieces go round the waves
      while (pc >= pieces) { pc -= pieces; ++cl; }         // (no pieces at all: a run of under four words)
      if (cl >= cc) break;
      const int w0 = pc << 8, idx = w0 + 4 * lane;
      if (idx < count4)
        load16_to_lds_at(src0 + (i64)cl * g_c, (unsigned)idx * 4u, gs_addr + 4u * (unsigned)(cl * pl.R * pl.RS + w0));
    }
    if (count4 < count)
      for (int cl = wave; cl < cc; cl += NW)
        if (lane < count - count4)
          load_to_lds_at(src0 + (i64)cl * g_c, (unsigned)(count4 + lane) * 4u,
                         gs_addr + 4u * (unsigned)(cl * pl.R * pl.RS + count4));
    return;
  }
  const int plane = pl.R * pl.RS;                              // words per channel
  const unsigned plane_bytes = 4u * (unsigned)plane;
  if (pl.RS <= kNarrowRow && (i64)cc * g_c < ((i64)1 << 30)) {
    // Narrow rows (1-D layers, the last layers of a stack whose frequency axis has shrunk
    // to a few bins): a load per row would move a handful of words, so a load moves 64
    // consecutive LDS words of one channel's block instead, lane j fetching the source
    // element of word w0 + j (rows and columns without a source become zeros).  Where a
    // word comes from does not depend on the channel, so a lane works it out once per
    // block of 64 words and the loads of all the chunk's channels reuse it.
    const FastDiv by_RS(pl.RS), by_nfx1(pl.nfx);
    // source element of word w0 + lane: >= 0 its index in the channel plane, -1 none
    // (a zero), -2 past the end of the block
    auto source_of = [&](int w0) -> int {
      const int wd = w0 + lane;
      if (wd >= plane) return -2;
      int r = wd, col = 0;
      if (pl.RS > 1) by_RS.divmod(wd, r, col);
      int gy = -1;
      const int vy = tg.vy_min + col;
      if (col < tg.RSL && vy >= 0) {
        if (pl.uy == 1) gy = vy;
        else { const int qy = vy / pl.uy; if (qy * pl.uy == vy) gy = qy; }
        if (gy >= pl.ngy) gy = -1;
      }
      if (r >= tg.R_tile || gy < 0) return -1;
      int gx = -1;
      if (mellin_x) {
        int oxl, fx;
        by_nfx1.divmod(r, oxl, fx);
        gx = mellin_tap32(pl.kind_x, pl.cls_first + pl.cls_stride * (tg.ox_lo + oxl), class_filter_row(pl.cls_fx, fx), pl.ngx, pl.sx, pl.dx,
                          pl.px + 1, pl.ux, pl.mg_p1);
      } else {
        const int vx = tg.vx_min + r;
        if (vx >= 0) {
          if (pl.ux == 1) { if (vx < pl.ngx) gx = vx; }
          else { const int qx = vx / pl.ux; if (qx * pl.ux == vx && qx < pl.ngx) gx = qx; }
        }
      }
      return gx >= 0 ? gx * pl.ngy + gy : -1;
    };
    auto move = [&](int w0, int src) {
      if (src >= 0) load_channels<EB>(Gimg, g_c, (unsigned)src * EB, gs_addr + 4u * (unsigned)w0, plane_bytes, cc);
      else if (fresh && src == -1) zero_channels(Gs + w0 + lane, plane, cc);
    };
    if (MEMO) {
      // the wave's first MB blocks from the memo, any further ones worked out each time
      if (new_tile) {
        int blk = 0;
        for (int w0 = wave * 64; w0 < plane && blk < MB; w0 += 64 * NW, ++blk) {
          const int src = source_of(w0);
#pragma unroll
          for (int b = 0; b < MB; ++b) memo->word_src[b] = b == blk ? src : memo->word_src[b];
        }
      }
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const int w0 = (wave + NW * b) * 64;
        if (w0 < plane) move(w0, memo->word_src[b]);
      }
      for (int w0 = (wave + NW * MB) * 64; w0 < plane; w0 += 64 * NW) move(w0, source_of(w0));
      return;
    }
    for (int w0 = wave * 64; w0 < plane; w0 += 64 * NW) move(w0, source_of(w0));
    return;
  }
  // Which signal row a virtual row holds does not depend on the channel: the lanes work
  // it out for 64 rows of a channel's block at a time, and the loads of every channel of
  // the chunk reuse it.
  const FastDiv by_nfx(pl.nfx);
  for (int base = 0; base < tg.R_tile; base += 64 * NW) {
    // per-lane: row base + NW * lane + wave of the channel's block
    int src_off, dst_off;
    if (MEMO && base == 0 && !new_tile) {
      src_off = memo->row_src;
      dst_off = memo->row_dst;
    } else {
      const int r = base + NW * lane + wave;
      src_off = -1;
      if (r < tg.R_tile) {
        int gx = -1;
        if (mellin_x) {
          int oxl, fx;
          by_nfx.divmod(r, oxl, fx);
          gx = mellin_tap32(pl.kind_x, pl.cls_first + pl.cls_stride * (tg.ox_lo + oxl), class_filter_row(pl.cls_fx, fx), pl.ngx, pl.sx, pl.dx,
                          pl.px + 1, pl.ux, pl.mg_p1);
        } else {
          const int vx = tg.vx_min + r;
          if (vx >= 0) {
            if (pl.ux == 1) { if (vx < pl.ngx) gx = vx; }
            else { const int qx = vx / pl.ux; if (qx * pl.ux == vx && qx < pl.ngx) gx = qx; }
          }
        }
        if (gx >= 0) src_off = gx * pl.ngy;
      }
      dst_off = r * pl.RS;
      if (MEMO && base == 0) { memo->row_src = src_off; memo->row_dst = dst_off; }
    }
    const int mine = min(64, (tg.R_tile - base - wave + NW - 1) / NW);
    for (int cb = 0; cb < tg.RSL; cb += 64) {
      const int col = cb + lane;
      const int vy = tg.vy_min + col;
      const bool in_row = col < tg.RSL;
      int gy = -1;
      if (in_row && vy >= 0) {
        if (pl.uy == 1) gy = vy;
        else { const int qy = vy / pl.uy; if (qy * pl.uy == vy) gy = qy; }
        if (gy >= pl.ngy) gy = -1;
      }
      const unsigned voff = (unsigned)max(gy, 0) * EB;
      const bool pad_col = gy < 0;
      for (int j = 0; j < mine; ++j) {
        const int s_src = __builtin_amdgcn_readlane(src_off, j);
        const int s_dst = __builtin_amdgcn_readlane(dst_off, j) + cb;
        if (s_src >= 0) {
          // lanes whose column has a source load it; padding columns become zeros
          if (!pad_col) load_channels<EB>(Gimg + (i64)s_src * EB, g_c, voff, gs_addr + 4u * (unsigned)s_dst, plane_bytes, cc);
          if (fresh && pad_col && in_row) zero_channels(Gs + s_dst + lane, plane, cc);
        } else if (fresh && in_row) {
          zero_channels(Gs + s_dst + lane, plane, cc);         // a row without a source
        }
      }
    }
  }
}

// ---- matrix-core loop over the tap pairs of one staged chunk ---------------------
// acc[i][t] += sum_k A[i * 32 + row][k] * B[k][t * 32 + col] on v_mfma_f32_32x32x2_f32:
// lane (l32, half) supplies A[l32][2 s + half] = wa[2 s + i * wrow] and
// B[2 s + half][l32] = Gs[lane_base[t] + tp[2 s]] for tap pair s.  Operands of the
// next group of GS pairs are fetched from LDS while the current group multiplies.
// KC taps (a last odd tap is paired with a zero).
template <int MT, int NT>
__device__ __forceinline__ void multiply_taps(floatx16 (&acc)[MT][NT], const float *wa, int wrow,
                                              const int *tp, const float *Gs, const int (&lane_base)[NT],
                                              int KC, int half) {
  constexpr int GS = 4;                              // tap pairs per operand group
  const int steps = (KC + 1) >> 1;
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

// ---- fp32 products on the bf16 matrix cores ------------------------------------------
// An fp32 value is the exact sum of three bf16 values (8 + 8 + 8 significant bits):
// hi = x rounded to the nearest bf16, mid = (x - hi) rounded likewise, lo = x - hi - mid
// (exact: what is left has at most 8 significant bits).  Both subtractions are exact in fp32.
// With rounding to nearest |mid| <= 2^-8 |x| and |lo| <= 2^-16 |x| (up to a factor 1 + 2^-8).
// A product x * y is then the sum of nine bf16 products, each exact in fp32; the six
// largest (hi hi, hi mid, mid hi, hi lo, lo hi, mid mid) are issued, and the three dropped
// ones (mid lo, lo mid, lo lo) are together below 1.01 * 2^-23 |x y|: two roundings of an
// fp32 product.  v_mfma_f32_32x32x16_bf16 accumulates in fp32 and runs at sixteen times the
// rate of v_mfma_f32_32x32x2_f32 per product, so six of them cost three eighths of the fp32
// instruction's time.
// Values that round to an infinite bf16 (infinities, and finite values above 3.3895e38)
// give NaN parts (inf - inf) and hence NaN results; NaN stays NaN.
__device__ __forceinline__ bf16x8 as_bf16x8(uintx4 v) { return __builtin_bit_cast(bf16x8, v); }

// Two values -> their parts, x0's in the low half and x1's in the high half of each word.
// v_cvt_pk_bf16_f32 rounds both to nearest even and packs them; a part back as fp32 is the
// half moved to the top of a word.
__device__ __forceinline__ void split_pair(float x0, float x1, unsigned &hi, unsigned &mid, unsigned &lo) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef float floatx2 __attribute__((ext_vector_type(2)));
  const floatx2 v = {x0, x1};
  hi = __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
  const floatx2 r1 = {x0 - __uint_as_float(hi << 16), x1 - __uint_as_float(hi & 0xFFFF0000u)};
  mid = __builtin_bit_cast(unsigned, __builtin_convertvector(r1, bf16x2));
  const floatx2 r2 = {r1.x - __uint_as_float(mid << 16), r1.y - __uint_as_float(mid & 0xFFFF0000u)};
  lo = __builtin_bit_cast(unsigned, __builtin_convertvector(r2, bf16x2));
}

// x[0..8) -> packed hi / mid / lo parts (element i in half i & 1 of word i >> 1)
__device__ __forceinline__ void split8(const float (&x)[8], uintx4 &hi, uintx4 &mid, uintx4 &lo) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    unsigned h, m, l;
    split_pair(x[2 * i], x[2 * i + 1], h, m, l);
    hi[i] = h; mid[i] = m; lo[i] = l;
  }
}

// acc += A * B over 16 values of k, both operands as hi / mid / lo parts; small terms first
__device__ __forceinline__ void mfma_split6(floatx16 &acc, const uintx4 &ah, const uintx4 &am, const uintx4 &al,
                                            const uintx4 &bh, const uintx4 &bm, const uintx4 &bl) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(al), as_bf16x8(bh), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(ah), as_bf16x8(bl), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(am), as_bf16x8(bm), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(am), as_bf16x8(bh), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(ah), as_bf16x8(bm), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(ah), as_bf16x8(bh), acc, 0, 0, 0);
}

// Fragment store of a (rows x K) fp32 operand, K a multiple of 16: the parts of the eight
// values k = 8 g .. 8 g + 7 of row r are one 16-byte word at
//   frag[(part * groups + g) * rows + r],   groups = K / 8,
// so the 32 lanes of a half-wave (rows r .. r + 31, one group) read 512 consecutive bytes.
__device__ __forceinline__ void store_frag(uintx4 *frag, int groups, int rows, int g, int r, const float (&x)[8]) {
  uintx4 hi, mid, lo;
  split8(x, hi, mid, lo);
  frag[(0 * groups + g) * rows + r] = hi;
  frag[(1 * groups + g) * rows + r] = mid;
  frag[(2 * groups + g) * rows + r] = lo;
}

// The matrix-core loop of multiply_taps on the bf16 cores: the filter block comes as
// fragments (store_frag: rows = M_T channels, K = KC16 taps, zero past the last tap),
// the signal words are read as in multiply_taps, eight taps per lane and step (lane half
// h takes taps 16 s + 8 h ..), and split in registers.  tp[k] is valid for k < KC16;
// `steps` steps of 16 taps are multiplied (KC16 / 16, or fewer for a shorter chunk).
template <int MT, int NT>
__device__ __forceinline__ void multiply_taps_split(floatx16 (&acc)[MT][NT], const uintx4 *frag, int m_rows,
                                                    const int *tp, const float *Gs, const int (&lane_base)[NT],
                                                    int KC16, int steps, int l32, int half) {
  const int groups = KC16 >> 3;
  struct Ops { uintx4 ah[MT], am[MT], al[MT], bh[NT], bm[NT], bl[NT]; };
  auto fetch = [&](int s, Ops &o) {
    const int g = 2 * s + half;
    const int4 o0 = *(const int4 *)(tp + 8 * g), o1 = *(const int4 *)(tp + 8 * g + 4);
    const int off[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float x[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = Gs[lane_base[t] + off[i]];
      split8(x, o.bh[t], o.bm[t], o.bl[t]);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      o.ah[i] = frag[(0 * groups + g) * m_rows + i * 32 + l32];
      o.am[i] = frag[(1 * groups + g) * m_rows + i * 32 + l32];
      o.al[i] = frag[(2 * groups + g) * m_rows + i * 32 + l32];
    }
  };
  auto multiply = [&](const Ops &o) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int t = 0; t < NT; ++t) mfma_split6(acc[i][t], o.ah[i], o.am[i], o.al[i], o.bh[t], o.bm[t], o.bl[t]);
  };
  // A step's operands are fetched and cut while the step before it multiplies: after every matrix
  // instruction one LDS read and a few of the vector instructions of the cut, pinned (left to
  // itself the scheduler moves every read next to its first use and the step waits for LDS).  The
  // loop body has no exit between a fetch and its use: the fetch past the last step reads the
  // last step's operands again.
  auto interleave = [] {
#pragma unroll
    for (int k = 0; k < MT * NT * 6; ++k) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       // one matrix instruction
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);       // two LDS reads
      __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);       // six vector instructions
    }
  };
  Ops a, b;
  int s = 0;
  if (steps > 0) fetch(0, a);
  for (; s + 1 < steps; s += 2) {
    fetch(s + 1, b);
    multiply(a);
    interleave();
    fetch(min(s + 2, steps - 1), a);
    multiply(b);
    interleave();
  }
  if (s < steps) multiply(a);
}

// ---- half-precision operands on the f16 matrix cores ----------------------------------
// The product of two half-precision values is exact in fp32, so v_mfma_f32_32x32x16_f16
// (fp32 accumulation, subnormal operands kept) needs no splitting: one instruction per
// sixteen taps.  The staged signal holds one half-precision value per LDS word, in the
// word's low half, at the same word offsets as the fp32 kernels' (lane_base and tp are
// BYTE offsets here); the filter block comes as fragments, the eight values
// k = 8 g .. 8 g + 7 of row r as one 16-byte word at frag[g * rows + r].
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef unsigned short ushortx2 __attribute__((ext_vector_type(2)));

template <int MT, int NT>
__device__ __forceinline__ void multiply_taps_f16(floatx16 (&acc)[MT][NT], const uintx4 *frag, int m_rows,
                                                  const int *tp, const float *Gs, const int (&lane_base)[NT],
                                                  int steps, int l32, int half) {
  struct Ops { uintx4 a[MT], b[NT]; };
  auto fetch = [&](int s, Ops &o) {
    const int g = 2 * s + half;
    const int4 o0 = *(const int4 *)(tp + 8 * g), o1 = *(const int4 *)(tp + 8 * g + 4);
    const int off[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ushortx2 pair;
        pair.x = *(const unsigned short *)((const char *)Gs + (lane_base[t] + off[2 * i]));
        pair.y = *(const unsigned short *)((const char *)Gs + (lane_base[t] + off[2 * i + 1]));
        o.b[t][i] = __builtin_bit_cast(unsigned, pair);
      }
#pragma unroll
    for (int i = 0; i < MT; ++i) o.a[i] = frag[g * m_rows + i * 32 + l32];
  };
  auto multiply = [&](const Ops &o) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, o.a[i]),
                                                           __builtin_bit_cast(halfx8, o.b[t]), acc[i][t], 0, 0, 0);
  };
  Ops a, b;
  int s = 0;
  if (steps > 0) fetch(0, a);
  for (; s + 1 < steps; s += 2) {
    fetch(s + 1, b);
    multiply(a);
    if (s + 2 < steps) fetch(s + 2, a);
    multiply(b);
  }
  if (s < steps) multiply(a);
}

}  // namespace mellin
