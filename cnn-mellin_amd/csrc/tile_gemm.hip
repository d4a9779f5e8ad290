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
// a wavefront issues one load per virtual row, 64 columns wide (64 consecutive
// LDS words of any rows when rows are a few words long; 16 bytes per lane when
// the virtual rows are the signal's own), and writes zeros for the columns or
// rows that have no source.  The loads of stage i+1 are issued before the
// matrix-core loop of stage i (two LDS buffers), so a persistent workgroup
// needs one barrier per stage and global latency hides behind the multiplies.
// A stage is one (tile, channel chunk) pair; where a tile's words come from and
// which are zeros is worked out for its first chunk and kept for the others.
//
// One wavefront owns all M_T output channels of NT * 32 positions and keeps
// MT * NT accumulator tiles (16 registers each).  Stores write 128-byte runs
// of one output row.
#include <algorithm>
#include <vector>
#include <type_traits>

#include "mellin_common.hpp"
#include "tile_gemm.hpp"
#include "tile_stage.hpp"

namespace mellin {

namespace {

// MB: 64-word blocks per wave whose staging sources are kept from a tile's first
// chunk for its other chunks (0: nothing kept; the instance for layers whose
// channels fit in one or two chunks).
// HOUT: H is half-precision storage (not with ACC): the fp32 results are rounded to
// nearest even as they are stored.
// SPLIT (1: the channels are one chunk, 2: several): the products run on the bf16 matrix
// cores, every fp32 operand as the exact sum of
// three bf16 parts (tile_stage.hpp).  The filter block then lives in LDS as fragments:
// built once per workgroup when the channels are one chunk, otherwise per stage (the next
// chunk's filter words are requested into registers before a stage's multiplies and split
// into the other fragment buffer after them), or, when AF holds the whole filter as
// fragments already (filter_fragments_kernel), copied from there by direct loads.
// SPLIT 3 (one chunk) and 4 (several; AF required): F, G and bias are half-precision
// storage and the products run on the f16 matrix cores (tile_stage.hpp); the signal is
// staged one value per LDS word like the floats, the filter fragments have one part.
// H is half-precision (HOUT) or fp32 storage.
// bx of gx: this workgroup among those that share the plan at plan_base (the whole launch,
// or one residue class's share of it).
typedef const __attribute__((address_space(4))) TilePlan ConstPlan;
template <int MT, int NT, bool ACC, int MB, bool HOUT, int SPLIT>
__device__ __forceinline__ void tile_gemm_body(
    ConstPlan *const plan_base, const int bx, const int gx, const float *__restrict__ F, const float *__restrict__ G,
    const float *__restrict__ bias, float *__restrict__ H, const float *__restrict__ AF) {
  // The plan is read where it lies, in the kernel-argument segment, through a pointer the
  // compiler must treat as new in every
  // iteration of the stage loop: fields are then re-read by scalar loads where
  // they are used instead of all being held in scalar registers for the whole
  // kernel, which had the register allocator spill hundreds of them to vector
  // lanes around the stores and the staging code.
  constexpr int kMemo = MB;
  ConstPlan *plp = plan_base;
#define pl (*plp)
  extern __shared__ __align__(16) float lds[];
  constexpr int M_T = MT * 32;
  constexpr int P = kWaves * NT * 32;
  constexpr bool F16 = SPLIT >= 3;
  constexpr int EB = F16 ? 2 : 4;                    // bytes per element of F, G and bias
  constexpr int PARTS = F16 ? 1 : 3;
  static_assert(!F16 || !ACC, "half-precision operands: results are written, not added");
  const int g_words = pl.CC * pl.R * pl.RS;          // one signal buffer
  const int w_words = SPLIT ? 4 * PARTS * (pl.KC16 >> 3) * M_T : M_T * pl.WSS;   // one filter buffer (SPLIT: parts x 16-byte fragments)
  float *Gs0 = lds;                                  // [sbuf][CC][R][RS]
  const int ws_word0 = SPLIT ? (pl.sbuf * g_words + 3) & ~3 : pl.sbuf * g_words;
  float *Ws0 = Gs0 + ws_word0;                       // [1 or 2][M_T][WSS], or the fragments
  // (a constant for the bf16 instances: the code that builds fragments per stage costs the
  // one-chunk kernel 24 registers and 6 % of its time when it is merely compiled in)
  const bool single_chunk = SPLIT ? (SPLIT & 1) : pl.CC >= pl.C;
  // SPLIT keeps four tables of KC16 words: signal offset of tap k of a whole chunk and of
  // the last (shorter) chunk, and the same two for the filter word's byte offset
  const int n_tapoff = SPLIT ? 4 * pl.KC16 : pl.KCp;
  int *tapoff = (int *)(Ws0 + (single_chunk ? 1 : 2) * w_words);   // [KCp]
  float *Bs = (float *)(tapoff + n_tapoff);          // [M_T] bias (zeros when accumulating)

  const int tid = threadIdx.x;
  // the wave index is wave-uniform: say so, and everything derived from it (row
  // loops, base addresses) is computed on the scalar unit
  const int lane = tid & 63, wave_id = __builtin_amdgcn_readfirstlane(tid >> 6), wave = wave_id;
  const int half = lane >> 5, l32 = lane & 31;
  const int m0 = blockIdx.y * M_T;
  const bool mellin_x = pl.kind_x == AX_MCORR || pl.kind_x == AX_MCONV;
  const int chunks = (pl.C + pl.CC - 1) / pl.CC;

  // ---- filter block: Ws[m][k], k = cl * nf + t, row stride WSS (odd) --------------
  // direct loads, coalesced along the taps; taps past the chunk and channels past M
  // are zero
  const unsigned lds_base = lds_address(lds);
  // (cl * f_c + t) * 4 of tap k = lane of a chunk: the same in every stage
  unsigned w_voff0;
  {
    const FastDiv by_nf(pl.nf);
    int cl, t;
    by_nf.divmod(lane, cl, t);
    w_voff0 = (unsigned)(((i64)cl * pl.f_c + t) * 4);              // < 4 GB: checked by the plan
  }
  // first: the buffer has not been filled by this workgroup before.  Rows of channels
  // that do not exist and the odd tap's partner are zeros that no load overwrites, so
  // they are written on the first fill only (and again by a last, shorter chunk).
  auto issue_filter = [&](int c0, int cc, int ws_word, bool first) {   // ws_word: where the block starts in lds[]
    const int KC = cc * pl.nf;
    const int m_live = max(0, min(M_T, pl.M - m0));       // channels of this block that exist
    const int KC4 = KC & ~3;
    const bool zero_cols = first || cc < pl.CC;
    const float *row = F + (i64)(m0 + wave) * pl.f_m + (i64)c0 * pl.f_c;   // this wave's first channel
    const i64 row_step = (i64)kWaves * pl.f_m;
    unsigned dst = lds_base + 4u * (unsigned)(ws_word + wave * pl.WSS);
    const unsigned dst_step = 4u * (unsigned)(kWaves * pl.WSS);
    if (pl.f_c == pl.nf && ((KC4 + 255) >> 8) + (KC4 < KC) < ((pl.KCp + 63) >> 6)) {
      // the taps of consecutive channels are one run of KC words per output channel:
      // 16 bytes per lane, then the last KC % 4 words singly (taken when that is
      // fewer instructions than 64 single words at a time)
      for (int m = wave; m < m_live; m += kWaves) {
        for (int kb = 0; kb < KC4; kb += 256)
          if (kb + 4 * lane < KC4) load16_to_lds_at(row, (unsigned)(kb + 4 * lane) * 4u, dst + 4u * (unsigned)kb);
        if (lane < KC - KC4) load_to_lds_at(row, (unsigned)(KC4 + lane) * 4u, dst + 4u * (unsigned)KC4);
        if (zero_cols && lane < pl.KCp - KC) lds[ws_word + m * pl.WSS + KC + lane] = 0.f;
        row += row_step;
        dst += dst_step;
      }
      if (first)
        for (int m = m_live + wave; m < M_T; m += kWaves)
          for (int k = lane; k < pl.KCp; k += 64) lds[ws_word + m * pl.WSS + k] = 0.f;
      return;
    }
    const FastDiv by_nf(pl.nf);
    for (int kb = 0; kb < pl.KCp; kb += 64) {
      const int k = kb + lane;
      unsigned voff = w_voff0;
      if (kb > 0) {
        int cl, t;
        by_nf.divmod(k, cl, t);
        voff = (unsigned)(((i64)cl * pl.f_c + t) * 4);
      }
      if (k < KC) {
        const float *r = row;
        unsigned d = dst + 4u * (unsigned)kb;
        for (int m = wave; m < m_live; m += kWaves) {
          load_to_lds_at(r, voff, d);
          r += row_step;
          d += dst_step;
        }
        if (first)
          for (int m = m_live + wave; m < M_T; m += kWaves) lds[ws_word + m * pl.WSS + k] = 0.f;
      } else if (zero_cols && k < pl.KCp && (first || k == KC)) {
        for (int m = wave; m < M_T; m += kWaves) lds[ws_word + m * pl.WSS + k] = 0.f;
      }
    }
  };

  // (SPLIT) the fragments of chunk ch of this block's channels, ready-made in AF
  auto copy_fragments = [&](int ch, int ws_word) {
    const float *src = AF + ((i64)blockIdx.y * chunks + ch) * w_words;
    const int bytes = 4 * w_words;                       // a multiple of 16
    for (int at = wave_id * 1024; at < bytes; at += kWaves * 1024)
      if (at + 16 * lane < bytes)
        load16_to_lds_at(src, (unsigned)(at + 16 * lane), lds_base + 4u * (unsigned)ws_word + (unsigned)at);
  };

  // ---- stages owned by this workgroup ------------------------------------------
  // tiles bx, bx + gx, ...; each tile has `chunks` stages
  const int my_tiles = bx < pl.total_tiles ? (pl.total_tiles - 1 - bx) / gx + 1 : 0;
  const int my_stages = my_tiles * chunks;
  StageMemo<kMemo> memo = {};
  // (stage_zero: a zero renewed every stage that the compiler cannot see through; adding
  // it to the wave index keeps the staging addresses from being worked out once for the
  // whole kernel and then held in registers across the matrix loops)
  unsigned stage_zero = 0;
  auto issue_stage = [&](int st, int ti, int ch) {           // st = ti * chunks + ch
    const int wave = wave_id + (int)stage_zero;
    const TileGeom tg = tile_geometry<P>(pl, bx + ti * gx, mellin_x);
    const int c0 = ch * pl.CC, cc = min(pl.CC, pl.C - c0);
    const int sb = (st & 1) * (pl.sbuf - 1) * g_words;    // sbuf == 1: a workgroup has one stage only
    // the sources worked out for a tile's first chunk serve its other chunks; a buffer's
    // zeros (padding, rows without a tap) survive from the tile's chunk two stages back
    issue_signal<kWaves, kMemo, EB>(pl, tg, G, c0, cc, Gs0 + sb, lds_base + 4u * (unsigned)sb, mellin_x, lane, wave,
                               &memo, ch == 0, ch < 2);
    if (!SPLIT && !single_chunk) issue_filter(c0, cc, ws_word0 + (st & 1) * w_words, st < 2);
    if (SPLIT && !single_chunk && (AF || SPLIT == 4)) copy_fragments(ch, ws_word0 + (st & 1) * w_words);
  };

  // ---- SPLIT: the filter block as fragments ----------------------------------------
  // Item idx = m * groups + g is the eight taps k = 8 g .. 8 g + 7 of output channel m;
  // a thread takes items first + tid and first + tid + 256.  Words come through buffer loads whose
  // offset is (channel's row) + (table entry of the tap): taps past the chunk and
  // channels past M carry an offset beyond the filter and read as zeros.
  constexpr int kFilterItems = 2;
  constexpr unsigned kDeadOffset = 0x40000000u;
  typedef typename std::conditional<F16, unsigned short, float>::type FilterWord;
  struct FilterWords { FilterWord x[kFilterItems][8]; };
  const int f_groups = SPLIT ? pl.KC16 >> 3 : 1;
  const int cc_last = pl.C - (chunks - 1) * pl.CC;
  __amdgpu_buffer_rsrc_t f_rsrc;
  if (SPLIT) f_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)F, 0, (int)pl.f_bytes, 0x00020000);
  const bool dense = SPLIT == 1 && pl.f_dense;          // (one chunk, the filter's own tap order)
  const int K_dense = pl.C * pl.nf;
  auto load_filter = [&](int ch, int first, FilterWords &fw) {
    const int *ko = tapoff + (ch + 1 == chunks ? 3 : 2) * pl.KC16;
    const int soff = (int)((unsigned)(ch * pl.CC) * (unsigned)pl.f_c * (unsigned)EB);
    const FastDiv by_groups(f_groups);
#pragma unroll
    for (int j = 0; j < kFilterItems; ++j) {
      const int idx = first + tid + j * kThreads;
      if (idx < f_groups * M_T) {
        int m, g;
        if (dense) { g = idx / M_T; m = idx - g * M_T; }   // channels fastest: the fragment writes are conflict-free
        else by_groups.divmod(idx, m, g);
        const unsigned row = m0 + m < pl.M ? (unsigned)(m0 + m) * (unsigned)pl.f_m * (unsigned)EB : kDeadOffset;
        if constexpr (!F16) {
          if (dense) {
            // the eight taps are 32 consecutive bytes of the channel's row (any 4-byte alignment)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              const int k = 8 * g + 4 * h;
              const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(f_rsrc, k < K_dense ? (int)(row + 4u * (unsigned)k) : (int)kDeadOffset, 0, 0);
#pragma unroll
              for (int i = 0; i < 4; ++i) fw.x[j][4 * h + i] = __uint_as_float(v[i]);
            }
            continue;
          }
        }
        const int4 k0 = *(const int4 *)(ko + 8 * g), k1 = *(const int4 *)(ko + 8 * g + 4);
        const int off[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if constexpr (F16)
            fw.x[j][i] = (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(f_rsrc, (int)(row + (unsigned)off[i]), soff, 0);
          else
            fw.x[j][i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(f_rsrc, (int)(row + (unsigned)off[i]), soff, 0));
        }
      }
    }
  };
  auto store_filter = [&](const FilterWords &fw, int first, float *buffer) {
    const FastDiv by_groups(f_groups);
#pragma unroll
    for (int j = 0; j < kFilterItems; ++j) {
      const int idx = first + tid + j * kThreads;
      if (idx < f_groups * M_T) {
        int m, g;
        if (dense) { g = idx / M_T; m = idx - g * M_T; }
        else by_groups.divmod(idx, m, g);
        if constexpr (F16) {
          uintx4 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = (unsigned)fw.x[j][2 * i] | ((unsigned)fw.x[j][2 * i + 1] << 16);
          ((uintx4 *)buffer)[g * M_T + m] = v;
        } else {
          store_frag((uintx4 *)buffer, f_groups, M_T, g, m, fw.x[j]);
        }
      }
    }
  };

  // (dense: the first round of the filter's words is requested before the tables are made; it needs none of them)
  FilterWords fw_first;
  if (dense && my_stages > 0) load_filter(0, 0, fw_first);
  {
    const FastDiv by_nf(pl.nf), by_nfy(pl.nfy);
    for (int k = tid; k < (SPLIT ? pl.KC16 : pl.KCp); k += kThreads) {
      int cl, t, fx, fy;
      by_nf.divmod(k, cl, t);
      by_nfy.divmod(t, fx, fy);
      // (the f16 loop adds byte offsets to byte addresses: one vector instruction per word less)
      const int off = (cl * pl.R * pl.RS + pl.Bx * fx * pl.RS + pl.by * fy) * (F16 ? 4 : 1);
      if (SPLIT) {
        // (the taps are padded to a multiple of 16, and the last chunk may have fewer
        // channels: such a tap reads the lane's first word, always a staged one, and
        // meets a zero weight)
        const bool whole = k < pl.CC * pl.nf, last = k < cc_last * pl.nf;
        const int fo = (cl * pl.f_c + class_filter_row(pl.cls_fx, fx) * pl.f_pitch + pl.f_off + fy) * EB;   // (the layer's filter row and column)
        tapoff[k] = whole ? off : 0;
        tapoff[pl.KC16 + k] = last ? off : 0;
        tapoff[2 * pl.KC16 + k] = whole ? fo : (int)kDeadOffset;
        tapoff[3 * pl.KC16 + k] = last ? fo : (int)kDeadOffset;
      } else {
        tapoff[k] = off;
      }
    }
    for (int m = tid; m < M_T; m += kThreads)
      Bs[m] = (!ACC && bias && m0 + m < pl.M) ? (F16 ? (float)((const _Float16 *)bias)[m0 + m] : bias[m0 + m]) : 0.f;
  }
  if (my_stages > 0) {
    if (SPLIT) {
      __syncthreads();                                    // the offset tables
      // (a filter that is one chunk may have more items than one round of the threads)
      if (!single_chunk && (AF || SPLIT == 4)) copy_fragments(0, ws_word0);
      else for (int first = 0; first < f_groups * M_T; first += kFilterItems * kThreads) {
        if (dense && first == 0) { store_filter(fw_first, 0, Ws0); continue; }
        FilterWords fw;
        load_filter(0, first, fw);
        store_filter(fw, first, Ws0);
      }
    } else if (single_chunk) {
      issue_filter(0, pl.C, ws_word0, true);
    }
    issue_stage(0, 0, 0);
  }

  const FastDiv by_noy(pl.noy);
  floatx16 acc[MT][NT];
  int lane_base[NT], lane_q[NT];
  TileGeom tg;

  // ---- stores: 32 consecutive lanes write 32 consecutive positions of one
  // channel; each lane walks one pointer down the channels in steps of whole
  // channel strides, so the only scalars the stores need are four byte strides.
  constexpr int ES = HOUT ? 2 : 4;                      // bytes per stored element
  const i64 hm1 = pl.h_m * ES, hm2 = 2 * hm1, hm3 = 3 * hm1, hm8 = 8 * hm1;
  const bool full_m = m0 + M_T <= pl.M;
  const bool buffer_stores = (i64)(M_T + 8) * hm1 < ((i64)1 << 31);    // 32-bit offsets inside a block's channels
  const int m_left = pl.M - m0 - half * 4;              // channels from this lane's first row on
  // They run one stage late, after the next stage's loads are issued and before
  // its multiplies, so that they drain behind the next matrix loop.
  auto write_tile = [&](auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    char *Himg = (char *)H + ((i64)tg.n * pl.h_n + (i64)m0 * pl.h_m) * ES;
    bool live[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int local = (wave * NT + t) * 32 + l32;
      live[t] = local < tg.count;
      if (ACC) {
        int ox, oy;
        by_noy.divmod(lane_q[t], ox, oy);
        live[t] = live[t] && ox < pl.nox_eff && oy < pl.noy_eff;
      }
    }
    if (FULL && !ACC && buffer_stores) {
      // One descriptor for the block's channels of this image; a lane's offset is its
      // position plus whole groups of eight channels, the four channels inside a group
      // are scalar offsets: a store and a quarter of a 32-bit add per word, against a
      // store and a 64-bit add with pointers.
      // A channel's 32-position pieces of this wavefront's position tiles go out back to
      // back (tile innermost): the pieces are neighbours in memory and none starts on a
      // 128-byte line, so the line two of them share is completed while the first write to
      // it is still on its way through the CU's write path.  With the channels innermost
      // (each tile's 64 stores, then the next tile's) the shared lines were written twice,
      // in two parts: a store-only launch of this pattern took 36 us for the benchmark's
      // 157 MB against 28.6 us in this order.
      const __amdgpu_buffer_rsrc_t h_rsrc =
          __builtin_amdgcn_make_buffer_rsrc((void *)Himg, 0, (int)(M_T * hm1), 0x00020000);
      int voff[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) voff[t] = live[t] ? (half * 4) * (int)hm1 + lane_q[t] * ES : (int)0x7FFFFFF0;   // (past the descriptor: dropped)
      auto put = [&](float v, int vo, int soff) {
        if constexpr (HOUT)
          __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, (_Float16)v), h_rsrc, vo, soff, 0);
        else
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), h_rsrc, vo, soff, 0);
      };
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int t = 0; t < NT; ++t)
              put(acc[i][t][4 * g4 + r], voff[t], r == 0 ? 0 : (r == 1 ? (int)hm1 : (r == 2 ? (int)hm2 : (int)hm3)));
#pragma unroll
          for (int t = 0; t < NT; ++t) voff[t] += (int)hm8;
        }
      return;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (!live[t]) continue;
      char *o = Himg + (half * 4) * hm1 + (i64)lane_q[t] * ES;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        float old[16];
        if (ACC) {
          // the 16 old values of this channel tile are fetched in one batch: one round
          // trip to memory per 16 stores instead of one per store
          char *q = o;
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            const int mo = i * 32 + g4 * 8;
            old[4 * g4 + 0] = (FULL || mo < m_left) ? *(const float *)q : 0.f;
            old[4 * g4 + 1] = (FULL || mo + 1 < m_left) ? *(const float *)(q + hm1) : 0.f;
            old[4 * g4 + 2] = (FULL || mo + 2 < m_left) ? *(const float *)(q + hm2) : 0.f;
            old[4 * g4 + 3] = (FULL || mo + 3 < m_left) ? *(const float *)(q + hm3) : 0.f;
            q += hm8;
          }
        }
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int mo = i * 32 + g4 * 8;
          auto put = [&](char *at, int row, int r) {
            if (FULL || row < m_left) {
              if (HOUT) *(_Float16 *)at = (_Float16)acc[i][t][r];
              else *(float *)at = ACC ? old[r] + acc[i][t][r] : acc[i][t][r];
            }
          };
          put(o, mo, 4 * g4);
          put(o + hm1, mo + 1, 4 * g4 + 1);
          put(o + hm2, mo + 2, 4 * g4 + 2);
          put(o + hm3, mo + 3, 4 * g4 + 3);
          o += hm8;                                        // next group of four channels: 8 further on
        }
      }
    }
  };
  const bool relu = !ACC && pl.relu;
  auto epilogue = [&]() {
    if (relu) {                                           // the layer's non-linearity, on the way out
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][t][r] = fmaxf(acc[i][t][r], 0.f);
    }
    if (full_m) write_tile(std::true_type());
    else write_tile(std::false_type());
  };
  FilterWords next_filter;
  for (int st = 0, ti = 0, ch = 0; st < my_stages; ++st, ti += (ch + 1 == chunks), ch = (ch + 1 == chunks) ? 0 : ch + 1) {
    {
      unsigned zero;                                      // a zero the compiler cannot see through
      asm volatile("s_mov_b32 %0, 0" : "=s"(zero));
      plp = (ConstPlan *)((const __attribute__((address_space(4))) char *)plan_base + zero);
      stage_zero = zero;
    }
    // every wave's loads for this stage have landed, and every wave is done
    // reading the buffer the next stage will fill
    wait_all_memory();
    __syncthreads();
    if (st + 1 < my_stages) {
      // (at raised priority: a staging wavefront otherwise gets an issue slot only now and
      // then between the matrix instructions of its SIMD's other wavefronts)
      __builtin_amdgcn_s_setprio(3);
      issue_stage(st + 1, ch + 1 == chunks ? ti + 1 : ti, ch + 1 == chunks ? 0 : ch + 1);
      if (SPLIT == 2 && !AF) load_filter(ch + 1 == chunks ? 0 : ch + 1, 0, next_filter);
      __builtin_amdgcn_s_setprio(0);
    }
    if (ch == 0) {
      if (st > 0) epilogue();                             // the tile finished one stage ago
      tg = tile_geometry<P>(pl, bx + ti * gx, mellin_x);
      // position -> LDS word of its (fx = 0, fy = 0) tap
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        int local = (wave * NT + t) * 32 + l32;
        if (local >= tg.count) local = 0;                 // masked lane: any valid position
        const int q = tg.q0 + local;
        int ox, oy;
        by_noy.divmod(q, ox, oy);
        lane_q[t] = (pl.cls_first + pl.cls_stride * ox) * pl.noy + oy;     // (== q unless the launch is a residue class)
        lane_base[t] = ((pl.Ax * (ox - tg.ox_lo) + pl.Cx0) * pl.RS + pl.ay * (oy - tg.oy_lo) - pl.by_min) * (F16 ? 4 : 1);
      }
    }
    if (ch == 0) {
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
    // ---- matrix-core loop over the tap pairs of this chunk
    {
      const int cc = min(pl.CC, pl.C - ch * pl.CC);
      if (F16)
        multiply_taps_f16<MT, NT>(acc, (const uintx4 *)(Ws0 + (single_chunk ? 0 : (st & 1) * w_words)), M_T,
                                  tapoff + (ch + 1 == chunks ? pl.KC16 : 0),
                                  Gs0 + (st & 1) * (pl.sbuf - 1) * g_words, lane_base,
                                  (cc * pl.nf + 15) >> 4, l32, half);
      else if (SPLIT)
        multiply_taps_split<MT, NT>(acc, (const uintx4 *)(Ws0 + (single_chunk ? 0 : (st & 1) * w_words)), M_T,
                                    tapoff + (ch + 1 == chunks ? pl.KC16 : 0),
                                    Gs0 + (st & 1) * (pl.sbuf - 1) * g_words, lane_base, pl.KC16,
                                    (cc * pl.nf + 15) >> 4, l32, half);
      else
      multiply_taps<MT, NT>(acc, Ws0 + (single_chunk ? 0 : (st & 1) * w_words) + l32 * pl.WSS + half, 32 * pl.WSS,
                            tapoff + half, Gs0 + (st & 1) * (pl.sbuf - 1) * g_words, lane_base, cc * pl.nf, half);
    }
    // the next stage's fragments: its buffer was last read two stages ago
    if (SPLIT == 2 && !AF && st + 1 < my_stages) store_filter(next_filter, 0, Ws0 + ((st + 1) & 1) * w_words);
  }
  if (my_stages > 0) epilogue();
#undef pl
}

template <int MT, int NT, bool ACC, int MB, bool HOUT, int SPLIT>
__global__ __launch_bounds__(kThreads, (NT == 1 ? (SPLIT ? 3 : 4) : 2)) void tile_gemm_kernel(
    TilePlan plan_arg, const float *__restrict__ F, const float *__restrict__ G,
    const float *__restrict__ bias, float *__restrict__ H, const float *__restrict__ AF) {
  // (the plan is the first argument: the kernel-argument segment starts with it)
  tile_gemm_body<MT, NT, ACC, MB, HOUT, SPLIT>((ConstPlan *)__builtin_amdgcn_kernarg_segment_ptr(), (int)blockIdx.x,
                                              (int)gridDim.x, F, G, bias, H, AF);
}

// The residue classes of a Mellin layer in one launch: workgroups wg_end[c - 1] .. wg_end[c] - 1
// of grid.x are class c's for their whole life, with that class's plan and fragments.
struct ClassLaunch {
  TilePlan pl[kMaxTileClasses];
  int n, wg_end[kMaxTileClasses];
  long long af_words[kMaxTileClasses];               // where the class's fragments start in AF (floats)
  long long f_bytes[kMaxTileClasses], h_bytes[kMaxTileClasses];   // the class's filter and output: bytes past F and H
};

static_assert(sizeof(ClassLaunch) + 5 * sizeof(void *) <= 4096, "kernel arguments are limited to 4 KB");

template <int MT, int NT, bool HOUT, int SPLIT>
__global__ __launch_bounds__(kThreads, (NT == 1 ? 3 : 2)) void tile_gemm_classes_kernel(
    ClassLaunch args, const float *__restrict__ F, const float *__restrict__ G,
    const float *__restrict__ bias, float *__restrict__ H, const float *__restrict__ AF) {
  typedef const __attribute__((address_space(4))) ClassLaunch ConstArgs;
  ConstArgs *const a = (ConstArgs *)__builtin_amdgcn_kernarg_segment_ptr();
  int c = 0, first = 0;
  for (; c + 1 < a->n && (int)blockIdx.x >= a->wg_end[c]; ++c) first = a->wg_end[c];
  tile_gemm_body<MT, NT, false, 0, HOUT, SPLIT>((ConstPlan *)&a->pl[c], (int)blockIdx.x - first, a->wg_end[c] - first,
                                               (const float *)((const char *)F + a->f_bytes[c]), G, bias,
                                               (float *)((char *)H + a->h_bytes[c]), AF ? AF + a->af_words[c] : AF);
}

// The whole filter as fragments, once per launch, in the order the stages of the SPLIT
// kernel copy them: AF[m_tile][chunk][part][group][row] (16-byte words).  One thread per
// (m_tile, chunk, group, row): eight taps of one output channel, split, three stores.
// F16: F is half-precision storage and a fragment is the eight values themselves (one part).
template <bool F16, class PL>
__device__ __forceinline__ void filter_fragments_body(const PL &pl, int M_T, int chunks, const void *__restrict__ Fv,
                                                      uintx4 *__restrict__ AF) {
  const int groups = pl.KC16 >> 3;
  const int per_block = groups * M_T;
  const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;
  const i64 blocks = (i64)((pl.M + M_T - 1) / M_T) * chunks;
  if (idx >= blocks * per_block) return;
  const int blk = (int)(idx / per_block), within = (int)(idx - (i64)blk * per_block);
  const int m_tile = blk / chunks, ch = blk - m_tile * chunks;
  const int m = within / groups, g = within - m * groups;
  const int cc = min(pl.CC, pl.C - ch * pl.CC), row = m_tile * M_T + m;
  typedef typename std::conditional<F16, unsigned short, float>::type Word;
  const Word *F = (const Word *)Fv;
  Word x[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int k = 8 * g + i, cl = k / pl.nf, t = k - cl * pl.nf;
    const int fx = t / pl.nfy, ta = class_filter_row(pl.cls_fx, fx) * pl.f_pitch + pl.f_off + (t - fx * pl.nfy);   // the layer's tap
    x[i] = (row < pl.M && k < cc * pl.nf) ? F[(i64)row * pl.f_m + (i64)(ch * pl.CC + cl) * pl.f_c + ta] : (Word)0;
  }
  if constexpr (F16) {
    uintx4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (unsigned)x[2 * i] | ((unsigned)x[2 * i + 1] << 16);
    AF[(i64)blk * per_block + g * M_T + m] = v;
  } else {
    store_frag(AF + (i64)blk * 3 * per_block, groups, M_T, g, m, x);
  }
}

template <bool F16>
__global__ __launch_bounds__(256) void filter_fragments_kernel(TilePlan pl, int M_T, int chunks,
                                                               const void *__restrict__ Fv,
                                                               uintx4 *__restrict__ AF) {
  filter_fragments_body<F16>(pl, M_T, chunks, Fv, AF);
}

// The same for every class of a launch at once: blockIdx.y is the class.
template <bool F16>
__global__ __launch_bounds__(256) void filter_fragments_classes_kernel(ClassLaunch args, int M_T,
                                                                       const void *__restrict__ Fv,
                                                                       float *__restrict__ AF) {
  typedef const __attribute__((address_space(4))) ClassLaunch ConstArgs;
  ConstArgs *const a = (ConstArgs *)__builtin_amdgcn_kernarg_segment_ptr();
  const int c = (int)blockIdx.y;
  const auto &pl = a->pl[c];
  filter_fragments_body<F16>(pl, M_T, (pl.C + pl.CC - 1) / pl.CC, (const char *)Fv + a->f_bytes[c],
                             (uintx4 *)(AF + a->af_words[c]));
}

template <int MT, int NT, bool ACC, int MB, bool HOUT = false, int SPLIT = 0>
hipError_t launch_variant(const TilePlan &pl, size_t lds_bytes, dim3 grid, const float *f,
                          const float *g, const float *bias, float *h, hipStream_t stream,
                          const float *af = nullptr) {
  auto kern = tile_gemm_kernel<MT, NT, ACC, MB, HOUT, SPLIT>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, stream, pl, f, g, bias, h, af);
  return hipGetLastError();
}

template <int MT, int NT, bool HOUT, int SPLIT>
hipError_t launch_classes_variant(const ClassLaunch &args, size_t lds_bytes, dim3 grid, const float *f, const float *g,
                                  const float *bias, float *h, hipStream_t stream, const float *af) {
  auto kern = tile_gemm_classes_kernel<MT, NT, HOUT, SPLIT>;
  {
    static std::atomic<int> lds_allowed{0};                // (one per kernel instance)
    hipError_t e = allow_large_lds((const void *)kern, lds_bytes, lds_allowed);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds_bytes, stream, args, f, g, bias, h, af);
  return hipGetLastError();
}

}  // namespace

// Workgroups of the forward kernel that a CU holds at once: bounded by LDS and
// by the registers of the instance (NT == 2 needs more than 128).
static int workgroups_per_cu(size_t lds_bytes, int mt, int nt, bool split) {
  const int by_lds = (int)((160 * 1024) / (lds_bytes + 512));
  (void)mt;
  const int by_regs = split ? (nt == 2 ? 2 : 3) : (nt == 2 ? 3 : 4);
  return std::max(1, std::min(by_lds, by_regs));
}

// Fill `pl` for the problem `pr`; returns false when the tiled kernel does not
// apply (sizes beyond 32-bit indexing or a single channel not fitting in LDS).
bool make_tile_plan(const SepConv &pr, TilePlan &pl, size_t *lds_bytes, int *mt, int *nt, int force_nt,
                    bool trim_columns, int force_mt) {
  const i64 lim = (i64)1 << 30;
  // (a residue class of a Mellin axis: the rows and filter rows of the class)
  const bool cls = pr.cls_nfx > 0;
  if (cls && (pr.accumulate || (pr.x.kind != AX_MCORR && pr.x.kind != AX_MCONV) || pr.cls_nfx > 16 || pr.cls_stride < 1 ||
              pr.cls_first < 0 || pr.x.nf > 16))
    return false;
  const i64 nfx_k = cls ? pr.cls_nfx : pr.x.nf;
  const i64 nox_k = cls ? std::max<i64>(0, (pr.x.nh - pr.cls_first + pr.cls_stride - 1) / pr.cls_stride) : pr.x.nh;
  const i64 nox_eff_k = cls ? std::max<i64>(0, (pr.x.nh_eff - pr.cls_first + pr.cls_stride - 1) / pr.cls_stride) : pr.x.nh_eff;
  // Filter columns with a tap inside the signal for some output column (layers on one or two
  // frequency bins with a padded 4-wide filter: half the columns have none, and a plan that
  // keeps them stages zeros for them and multiplies them).  Only the two ends are cut:
  //   correlation  gy = s oy + d fy - p,   convolution  gy = s oy - d fy + p,   0 <= gy < ng
  // over oy in [0, nh_eff); the kernel then sees columns fy_lo .. fy_hi as a filter of its own
  // with p - d fy_lo for p.
  i64 fy_lo = 0, fy_hi = pr.y.nf - 1;
  if (trim_columns && pr.y.u == 1 && pr.y.nh_eff >= 1 && pr.y.d >= 1 && pr.y.nf >= 1 &&
      (pr.y.kind == AX_LCORR || pr.y.kind == AX_LCONV)) {
    const i64 span = pr.y.s * (pr.y.nh_eff - 1);           // s oy runs over [0, span]
    i64 lo, hi;
    if (pr.y.kind == AX_LCORR) {
      lo = -floor_div(-(pr.y.p - span), pr.y.d);           // d fy - p + span >= 0
      hi = floor_div(pr.y.ng - 1 + pr.y.p, pr.y.d);        // d fy - p <= ng - 1
    } else {
      lo = -floor_div(-(pr.y.p - (pr.y.ng - 1)), pr.y.d);  // -d fy + p <= ng - 1
      hi = floor_div(pr.y.p + span, pr.y.d);               // -d fy + p + span >= 0
    }
    lo = std::max<i64>(lo, 0);
    hi = std::min<i64>(hi, pr.y.nf - 1);
    if (lo <= hi) { fy_lo = lo; fy_hi = hi; }
  }
  const bool trimmed = fy_lo > 0 || fy_hi < pr.y.nf - 1;
  const i64 nfy_k = fy_hi - fy_lo + 1, py_k = pr.y.p - pr.y.d * fy_lo;
  const i64 nf = nfx_k * nfy_k, ng = pr.x.ng * pr.y.ng, Q = nox_k * pr.y.nh;
  if (nf <= 0 || ng <= 0 || Q <= 0 || pr.c_in <= 0 || pr.c_out <= 0 || pr.batch <= 0) return false;
  if (nf > 4096 || ng >= lim || Q >= lim || pr.c_in >= lim || pr.c_out >= lim || pr.batch >= lim) return false;
  if (pr.c_in * ng >= lim * 2 || pr.batch * (Q / 64 + 1) >= lim) return false;
  const Axis &X = pr.x, &Y = pr.y;
  if (Y.kind != AX_LCORR && Y.kind != AX_LCONV) return false;
  if (X.s > 4096 || X.d > 4096 || X.u > 4096 || X.p > 4096 || Y.s > 64 || Y.d > 4096 || Y.u > 64) return false;
  if (Y.p > lim || Y.p < -lim || X.p < -lim) return false;

  pl.batch = (int)pr.batch; pl.M = (int)pr.c_out; pl.C = (int)pr.c_in;
  pl.nfx = (int)nfx_k; pl.nfy = (int)nfy_k; pl.nf = (int)nf;
  pl.f_pitch = (int)Y.nf; pl.f_off = (int)fy_lo;
  pl.ngx = (int)X.ng; pl.ngy = (int)Y.ng; pl.nox = (int)nox_k; pl.noy = (int)Y.nh; pl.Q = (int)Q;
  pl.nox_eff = (int)nox_eff_k; pl.noy_eff = (int)Y.nh_eff;
  pl.cls_stride = cls ? pr.cls_stride : 1;
  pl.cls_first = cls ? pr.cls_first : 0;
  pl.cls_fx = cls ? pr.cls_fx : 0xFEDCBA9876543210ull;
  pl.f_m = pr.f_m; pl.f_c = pr.f_c; pl.g_n = pr.g_n; pl.g_c = pr.g_c; pl.h_n = pr.h_n; pl.h_m = pr.h_m;
  pl.accumulate = pr.accumulate;
  pl.relu = pr.relu && !pr.accumulate;
  pl.out_half = pr.out_half && !pr.accumulate;
  if (pr.in_half && pr.accumulate) return false;         // half-precision operands: results are written, not added
  pl.kind_x = X.kind; pl.sx = (int)X.s; pl.dx = (int)X.d; pl.px = (int)X.p; pl.ux = (int)X.u;
  pl.uy = (int)Y.u;

  // 64 output channels per workgroup, unless the launch would then have fewer than two
  // workgroups per CU: 32 channels double the workgroups of a small problem (1-D layers
  // of 780 frames: input gradient 75 -> 61 us, forward up to 25 % faster)
  *mt = (pr.c_out > 32 && pr.batch * ((Q + 127) / 128) * ((pr.c_out + 63) / 64) >= 512) ? 2 : 1;
  // half-precision operands: 128 channels where the layer has them (the f16 instructions are
  // through with a staged chunk six times sooner, so what a chunk's staging costs is spread
  // over twice the products; the accumulators fit because nothing is split in registers)
  if (pr.in_half && pr.c_out > 64 && pr.batch * ((Q + 255) / 256) * ((pr.c_out + 127) / 128) >= 256) *mt = 4;
  if (force_mt) {
    if ((force_mt != 1 && force_mt != 2 && force_mt != 4) || (force_mt == 4 && !pr.in_half)) return false;
    *mt = force_mt;
  }
  const int M_T = *mt * 32;
  const i64 m_tiles = (pr.c_out + M_T - 1) / M_T;
  // two N tiles per wavefront once that still leaves every CU several tiles (not when
  // accumulating into the output: with the old values to fetch as well, that instance
  // runs out of registers and measured 2-3 times slower than one tile per wavefront)
  *nt = (!pr.accumulate && pr.batch * ((Q + 255) / 256) * m_tiles >= 4 * 256) ? 2 : 1;
  if (*nt == 2) {
    // Workgroups are persistent and take whole tiles: the launch lasts as long as the
    // workgroup with the most tiles.  2400 tiles on 768 resident workgroups are four
    // rounds for 3.1 rounds of work; the same layer cut into 4800 half-size tiles on
    // 1024 workgroups is five rounds for 4.7.  A half-size tile runs at about 0.9 of the
    // full one's rate (measured), so the smaller tile wins when it fills its last round
    // that much better.
    const i64 big = pr.batch * ((Q + 255) / 256) * m_tiles, small = pr.batch * ((Q + 127) / 128) * m_tiles;
    const bool want_split = pr.math != MATH_FP32;
    const i64 slots_big = 256 * (want_split ? 2 : 3), slots_small = 256 * (want_split ? 3 : 4);
    const double fill_big = (double)big / (double)(((big + slots_big - 1) / slots_big) * slots_big);
    const double fill_small = (double)small / (double)(((small + slots_small - 1) / slots_small) * slots_small);
    if (0.9 * fill_small > 1.05 * fill_big) *nt = 1;       // only on a clear margin: layers staged in chunks lose more
  }
  if (force_nt) *nt = force_nt;
  const int P = kWaves * (*nt) * 32;

  // y axis: column = ay * oy + by * fy + cy - min
  pl.ay = (int)Y.s;
  pl.by = Y.kind == AX_LCORR ? (int)Y.d : -(int)Y.d;
  pl.cy = Y.kind == AX_LCORR ? -(int)py_k : (int)py_k;
  const i64 by_ext = (i64)pl.by * (pl.nfy - 1);
  pl.by_min = (int)(by_ext < 0 ? by_ext : 0);
  pl.by_span = (int)(by_ext < 0 ? -by_ext : by_ext);

  // tiling of the flattened (ox, oy) positions
  pl.segment = pl.noy > P;
  pl.chunks_per_row = (pl.noy + P - 1) / P;
  pl.tiles_per_image = pl.segment ? pl.nox * pl.chunks_per_row : (pl.Q + P - 1) / P;
  pl.total_tiles = pl.batch * pl.tiles_per_image;
  auto magic = [](int d) { return d <= 1 ? 0xFFFFFFFFu : (unsigned)(0x100000000ull / (unsigned)d); };
  pl.mg_tpi = magic(pl.tiles_per_image); pl.mg_cpr = magic(pl.chunks_per_row); pl.mg_noy = magic(pl.noy);
  pl.mg_p1 = magic((int)X.p + 1);
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
  if (pr.in_half) pl.contig = 0;                          // (16-byte pieces need 4-byte elements)
  if (pl.contig) pl.RS = pl.ngy;


  // channels per chunk from the LDS budget (a third of a CU's LDS, so that three
  // workgroups stay resident: measured 5-15 % faster on the multi-chunk layers than
  // two workgroups with larger chunks): two signal buffers, and two filter buffers
  // unless every channel fits in one chunk
  // (only when the launch has the workgroups to put three on a CU; a layer that fits
  // whole, or a small launch, takes up to 72 KB)
  const i64 whole_words = (72 * 1024) / 4;
  const i64 budget_words = (i64)pl.total_tiles * m_tiles > 2 * 256 ? (52 * 1024) / 4 : whole_words;
  const i64 fixed = M_T + 16;
  const i64 g_per_c = (i64)pl.R * pl.RS, w_per_c = (i64)pl.nf * M_T, t_per_c = pl.nf;
  i64 cc;
  if (2 * g_per_c * pl.C + w_per_c * pl.C + 3 * M_T + t_per_c * pl.C + 2 + fixed <= whole_words) {
    cc = pl.C;
  } else {
    cc = (budget_words - fixed - 6 * M_T - 2) / (2 * g_per_c + 2 * w_per_c + t_per_c);
    // chunks of under four channels leave a stage too short for what it costs to set up:
    // with several output-channel tiles per position tile, two workgroups per CU with
    // longer stages have measured 7-10 % faster than three with shorter ones
    if (cc < 4 && m_tiles >= 2) cc = (whole_words - fixed - 6 * M_T - 2) / (2 * g_per_c + 2 * w_per_c + t_per_c);
    if (cc < 1) return false;
    if (cc > pl.C) cc = pl.C;
    if (cc > 64) cc = 64;
  }
  if (cc * pl.R >= ((i64)1 << 22)) return false;
  if (cc * ng >= lim) return false;                               // 32-bit byte offsets across a chunk's channels
  pl.CC = (int)cc;
  pl.KCp = ((pl.CC * pl.nf + 1) / 2) * 2;
  pl.WSS = pl.KCp + 1;                                             // odd: 32 channels -> 32 banks
  bool single = pl.CC >= pl.C;
  *lds_bytes = 4 * (2 * (size_t)pl.CC * pl.R * pl.RS + (single ? 1 : 2) * (size_t)M_T * pl.WSS +
                    pl.KCp + M_T);
  if (*lds_bytes > 76 * 1024 && !pr.in_half) return false;
  // the bf16 matrix cores: the filter block as fragments (6 bytes per word, taps padded to
  // a multiple of 16), built by 256 threads of two 8-tap items each
  pl.split = 0;
  pl.f_dense = 0;
  pl.f16 = 0;
  pl.KC16 = 0;
  pl.f_bytes = 0;
  const i64 f_extent = (pr.in_half ? 2 : 4) * ((pr.c_out - 1) * pr.f_m + (pr.c_in - 1) * pr.f_c + pr.x.nf * pr.y.nf);
  const size_t frag_word = pr.in_half ? 2 : 6;              // fragment bytes per filter word
  auto split_lds = [&](int sbuf, i64 ccs, bool one_chunk) {
    const size_t kc16 = (size_t)((ccs * pl.nf + 15) / 16) * 16;
    return 4 * ((((size_t)sbuf * ccs * pl.R * pl.RS) + 3) & ~(size_t)3) + (one_chunk ? 1 : 2) * frag_word * kc16 * M_T +
           4 * (4 * kc16 + M_T);
  };
  if (pr.in_half) {
    // the f16 matrix cores: fragments of one part; a filter of several chunks is always
    // read from ready-made fragments in scratch memory (tile_fragment_bytes)
    if (f_extent > ((i64)1 << 30)) return false;
    i64 best = 0;
    if (split_lds(2, pl.C, true) <= 79 * 1024) {
      best = pl.C;
    } else {
      const size_t budget = *nt == 2 ? 79 * 1024 : 52 * 1024;
      double best_fill = 0;
      for (i64 c = std::min<i64>(pl.C, 64); c >= 1; --c) {
        const i64 kc16 = ((c * pl.nf + 15) / 16) * 16;
        if (split_lds(2, c, false) > budget) continue;
        if (best && c < best - 3) break;
        const i64 n_chunks = (pl.C + c - 1) / c;
        const i64 last = pl.C - (n_chunks - 1) * c;
        const double fill = (double)(pl.C * pl.nf) /
                            (double)((n_chunks - 1) * kc16 + ((last * pl.nf + 15) / 16) * 16);
        if (!best || fill > best_fill + 1e-9) { best = c; best_fill = fill; }
      }
    }
    if (best < 1 || best * pl.R >= ((i64)1 << 22) || best * ng >= lim) return false;
    pl.split = 1;
    pl.f16 = 1;
    pl.CC = (int)best;
    single = pl.CC >= pl.C;
    pl.KC16 = (int)(((best * pl.nf + 15) / 16) * 16);
    pl.KCp = ((pl.CC * pl.nf + 1) / 2) * 2;
    pl.WSS = pl.KCp + 1;
    *lds_bytes = split_lds(2, best, single);
    pl.f_bytes = (unsigned)f_extent;
  } else if (pr.math != MATH_FP32 && f_extent <= ((i64)1 << 30)) {
    const i64 item_cap = (2 * kThreads * 8) / M_T;         // taps per chunk the two items per thread cover
    // (a layer that fits whole as fp32 words but not with its fragments: in chunks when the
    // bf16 form is asked for by name, else it stays on the fp32 instructions)
    const bool whole_split = single && split_lds(2, pl.C, true) <= 79 * 1024;
    if (whole_split) {
      pl.split = 1;
      pl.KC16 = (int)(((pl.C * pl.nf + 15) / 16) * 16);
      // (the kernel's taps are the filter's own, in its own order: fragments can be cut from 16-byte loads)
      pl.f_dense = !cls && pl.f_off == 0 && pl.f_pitch == pl.nfy && pr.f_c == pl.nf && ((pl.C * pl.nf) & 3) == 0;
      *lds_bytes = split_lds(2, pl.C, true);
    } else if (pr.math == MATH_BF16X3_ALWAYS ||
               (!single && (double)pr.batch * (double)Q * (double)pr.c_out * (double)pr.c_in * (double)nf >= 8e8)) {
      // (layers under 0.8 GMAC (virtual rows counted) stay on the fp32 instructions: config 2's 1-D Mellin layers,
      // 0.12-0.52 GMAC, measured 25-60 % slower with fragments staged per chunk)
      // chunks: the largest that fits the LDS of a workgroup (two to a CU with two position
      // tiles per wavefront, else three), preferring among the top few the one whose taps
      // fill their multiple of 16 best
      const size_t budget = *nt == 2 ? 79 * 1024 : 52 * 1024;
      i64 best = 0;
      double best_fill = 0;
      for (i64 c = std::min<i64>(pl.C, 64); c >= 1; --c) {
        const i64 kc16 = ((c * pl.nf + 15) / 16) * 16;
        if (kc16 > item_cap || split_lds(2, c, false) > budget) continue;
        if (best && c < best - 3) break;
        const i64 n_chunks = (pl.C + c - 1) / c;
        const i64 last = pl.C - (n_chunks - 1) * c;
        // matrix steps executed per channel against 1/16 per tap
        const double fill = (double)(pl.C * pl.nf) /
                            (double)((n_chunks - 1) * kc16 + ((last * pl.nf + 15) / 16) * 16);
        if (!best || fill > best_fill + 1e-9) { best = c; best_fill = fill; }
      }
      if (best >= 2 && best * pl.R < ((i64)1 << 22) && best * ng < lim) {
        pl.split = 1;
        pl.CC = (int)best;
        pl.KC16 = (int)(((best * pl.nf + 15) / 16) * 16);
        pl.KCp = ((pl.CC * pl.nf + 1) / 2) * 2;
        pl.WSS = pl.KCp + 1;
        single = pl.CC >= pl.C;
        *lds_bytes = split_lds(2, best, single);
      }
    }
    if (pl.split) pl.f_bytes = (unsigned)f_extent;
  }
  // A launch small enough that every tile gets a workgroup of its own once the
  // second signal buffer is dropped (more workgroups fit per CU) runs as one
  // wave of single-stage workgroups: nothing to prefetch, and no second round
  // in which most of the chip idles.
  pl.sbuf = 2;
  if (single) {
    const size_t one = pl.split ? split_lds(1, pl.C, true) : *lds_bytes - 4 * (size_t)pl.CC * pl.R * pl.RS;
    const i64 slots2 = 256 * (i64)workgroups_per_cu(*lds_bytes, *mt, *nt, pl.split);
    const i64 slots1 = 256 * (i64)workgroups_per_cu(one, *mt, *nt, pl.split);
    const i64 wgs = (i64)pl.total_tiles * m_tiles;
    if (wgs > slots2 && wgs <= slots1) { pl.sbuf = 1; *lds_bytes = one; }
  }
  // (columns, like the filter rows of a class, are picked through the fragment tables)
  if (trimmed && !pl.split) return make_tile_plan(pr, pl, lds_bytes, mt, nt, force_nt, false, force_mt);
  if (cls && !pl.split) return false;
  return true;
}

// Residue classes of a Mellin x axis.  On a correlation axis the tap of (row h, filter row f)
// exists iff (h + s)(f + d) is a multiple of p + 1: rows with the same (h + s) mod (p + 1)
// have taps for the same filter rows.  On a convolution axis it exists iff (p + 1)(h + s) is a
// multiple of f + d, i.e. iff h + s is a multiple of m_f = (f + d) / gcd(f + d, p + 1): rows
// with the same (h + s) mod lcm(m_f) do.  A launch over one class meets no pair without a
// tap (other than taps outside the signal), so nothing is staged or multiplied for them.
int mellin_classes(const Axis &x, MellinClass *out, int max_classes) {
  auto gcd = [](i64 a, i64 b) { while (b) { const i64 t = a % b; a = b; b = t; } return a; };
  if ((x.kind != AX_MCORR && x.kind != AX_MCONV) || x.nf < 1 || x.nf > 16) return 0;
  i64 L = 1;
  if (x.kind == AX_MCORR) {
    L = x.p + 1;
  } else {
    for (i64 f = 0; f < x.nf; ++f) {
      const i64 m = (f + x.d) / gcd(f + x.d, x.p + 1);
      L = L / gcd(L, m) * m;
      if (L > max_classes) return 0;
    }
  }
  if (L < 2 || L > max_classes) return 0;
  const i64 shift = x.s;
  for (i64 r = 0; r < L; ++r) {
    MellinClass &c = out[r];
    c.stride = (int)L;
    c.first = (int)(((r - shift) % L + L) % L);
    c.nfx = 0;
    c.fx = 0;
    for (i64 f = 0; f < x.nf; ++f) {
      const bool has = x.kind == AX_MCORR ? (r * (f + x.d)) % (x.p + 1) == 0
                                          : r % ((f + x.d) / gcd(f + x.d, x.p + 1)) == 0;
      if (has) c.fx |= (unsigned long long)f << (4 * c.nfx++);
    }
  }
  return (int)L;
}

size_t tile_fragment_bytes(const TilePlan &pl, int mt) {
  const int chunks = (pl.C + pl.CC - 1) / pl.CC;
  if (!pl.split || chunks < 2) return 0;
  const size_t m_tiles = (size_t)((pl.M + mt * 32 - 1) / (mt * 32));
  return m_tiles * chunks * (pl.f16 ? 1 : 3) * (size_t)(pl.KC16 >> 3) * (mt * 32) * 16;
}

hipError_t launch_tile_gemm(const TilePlan &pl, size_t lds_bytes, int mt, int nt,
                            const float *f, const float *g, const float *bias,
                            float *h, hipStream_t stream, float *frag_ws) {
  const int M_T = mt * 32;
  const float *af = nullptr;
  if (pl.f16 && pl.accumulate) return hipErrorInvalidValue;
  if (pl.f16 && tile_fragment_bytes(pl, mt) && !frag_ws) return hipErrorInvalidValue;   // no per-stage build in that kernel
  if (frag_ws && tile_fragment_bytes(pl, mt)) {
    const int chunks = (pl.C + pl.CC - 1) / pl.CC;
    const i64 items = (i64)tile_fragment_bytes(pl, mt) / (pl.f16 ? 16 : 48);
    hipLaunchKernelGGL((pl.f16 ? filter_fragments_kernel<true> : filter_fragments_kernel<false>),
                       dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, pl, M_T,
                       chunks, (const void *)f, (uintx4 *)frag_ws);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    af = frag_ws;
  }
  // persistent workgroups: as many as fit at once on the 256 CUs
  const int m_tiles = (pl.M + M_T - 1) / M_T;
  const int per_cu = workgroups_per_cu(lds_bytes, mt, nt, pl.split);
  int gx = std::max(1, (256 * per_cu) / m_tiles);
  gx = std::min(gx, pl.total_tiles);
  if (pl.sbuf == 1 && gx < pl.total_tiles) return hipErrorInvalidValue;   // one buffer: one stage per workgroup
  dim3 grid((unsigned)gx, (unsigned)m_tiles);
  // layers staged in three or more chunks of channels keep a tile's staging sources
  const bool memo = (pl.C + pl.CC - 1) / pl.CC > 2;
#define MELLIN_TILE_CASE(MT_, NT_)                                                           \
  if (mt == MT_ && nt == NT_) {                                                              \
    if (pl.f16) return hipErrorInvalidValue;                                                 \
    if (pl.split && pl.CC >= pl.C) {                                                         \
      if (pl.accumulate) return launch_variant<MT_, NT_, true, 0, false, 1>(pl, lds_bytes, grid, f, g, bias, h, stream, af); \
      if (pl.out_half) return launch_variant<MT_, NT_, false, 0, true, 1>(pl, lds_bytes, grid, f, g, bias, h, stream, af);   \
      return launch_variant<MT_, NT_, false, 0, false, 1>(pl, lds_bytes, grid, f, g, bias, h, stream, af);                   \
    }                                                                                        \
    if (pl.split) {                                                                          \
      if (pl.accumulate) return launch_variant<MT_, NT_, true, 0, false, 2>(pl, lds_bytes, grid, f, g, bias, h, stream, af); \
      if (pl.out_half) return launch_variant<MT_, NT_, false, 0, true, 2>(pl, lds_bytes, grid, f, g, bias, h, stream, af);   \
      return launch_variant<MT_, NT_, false, 0, false, 2>(pl, lds_bytes, grid, f, g, bias, h, stream, af);                   \
    }                                                                                        \
    if (pl.accumulate)                                                                       \
      return memo ? launch_variant<MT_, NT_, true, 8>(pl, lds_bytes, grid, f, g, bias, h, stream)  \
                  : launch_variant<MT_, NT_, true, 0>(pl, lds_bytes, grid, f, g, bias, h, stream); \
    if (pl.out_half)                                                                         \
      return memo ? launch_variant<MT_, NT_, false, 8, true>(pl, lds_bytes, grid, f, g, bias, h, stream)  \
                  : launch_variant<MT_, NT_, false, 0, true>(pl, lds_bytes, grid, f, g, bias, h, stream); \
    return memo ? launch_variant<MT_, NT_, false, 8>(pl, lds_bytes, grid, f, g, bias, h, stream)   \
                : launch_variant<MT_, NT_, false, 0>(pl, lds_bytes, grid, f, g, bias, h, stream);  \
  }
#define MELLIN_F16_CASE(MT_, NT_)                                                            \
  if (pl.f16 && mt == MT_ && nt == NT_) {                                                    \
    if (pl.out_half) {                                                                       \
      if (pl.CC >= pl.C) return launch_variant<MT_, NT_, false, 0, true, 3>(pl, lds_bytes, grid, f, g, bias, h, stream, af); \
      return launch_variant<MT_, NT_, false, 0, true, 4>(pl, lds_bytes, grid, f, g, bias, h, stream, af);                   \
    }                                                                                        \
    if (pl.CC >= pl.C) return launch_variant<MT_, NT_, false, 0, false, 3>(pl, lds_bytes, grid, f, g, bias, h, stream, af); \
    return launch_variant<MT_, NT_, false, 0, false, 4>(pl, lds_bytes, grid, f, g, bias, h, stream, af);                   \
  }
  MELLIN_F16_CASE(4, 2)
  MELLIN_F16_CASE(4, 1)
  MELLIN_F16_CASE(2, 2)
  MELLIN_F16_CASE(2, 1)
  MELLIN_F16_CASE(1, 2)
  MELLIN_F16_CASE(1, 1)
#undef MELLIN_F16_CASE
  MELLIN_TILE_CASE(2, 2)
  MELLIN_TILE_CASE(2, 1)
  MELLIN_TILE_CASE(1, 2)
  MELLIN_TILE_CASE(1, 1)
#undef MELLIN_TILE_CASE
  return hipErrorInvalidValue;
}

bool tile_classes_fit_one_launch(const TilePlan *pls, const int *mts, const int *nts, int n) {
  if (n < 2 || n > kMaxTileClasses) return false;
  for (int i = 0; i < n; ++i) {
    const TilePlan &p = pls[i];
    if (!p.split || p.accumulate || p.sbuf != 2 || p.CC >= p.C) return false;    // bf16 / f16 forms staged in chunks
    if (mts[i] != mts[0] || nts[i] != nts[0] || p.M != pls[0].M || p.f16 != pls[0].f16 || p.out_half != pls[0].out_half)
      return false;
    if (!p.f16 && mts[i] != 2) return false;                                       // (the instances built below)
  }
  return true;
}

hipError_t launch_tile_gemm_classes(const TilePlan *pls, const size_t *lds_bytes, int n, int mt, int nt, const float *f,
                                    const float *g, const float *bias, float *h, hipStream_t stream, float *frag_ws,
                                    const size_t *frag_off, const long long *f_bytes, const long long *h_bytes) {
  if (!tile_classes_fit_one_launch(pls, std::vector<int>(n, mt).data(), std::vector<int>(n, nt).data(), n))
    return hipErrorInvalidValue;
  const int M_T = mt * 32;
  const bool f16 = pls[0].f16;
  if (f16 && !frag_ws) return hipErrorInvalidValue;          // no per-stage build in that kernel
  ClassLaunch args;
  args.n = n;
  size_t lds = 0;
  double work[kMaxTileClasses];                              // per tile
  i64 max_items = 0;                                         // fragment items (eight taps of a channel) of the largest class
  for (int i = 0; i < n; ++i) {
    args.pl[i] = pls[i];
    lds = std::max(lds, lds_bytes[i]);
    const int chunks = (pls[i].C + pls[i].CC - 1) / pls[i].CC;
    work[i] = (double)chunks * pls[i].KC16;
    args.af_words[i] = 0;
    args.f_bytes[i] = f_bytes ? f_bytes[i] : 0;
    args.h_bytes[i] = h_bytes ? h_bytes[i] : 0;
    if (frag_ws) {
      max_items = std::max(max_items, (i64)tile_fragment_bytes(pls[i], mt) / (f16 ? 16 : 48));
      args.af_words[i] = (long long)(frag_off[i] / 4);
    }
  }
  if (frag_ws && max_items > 0) {
    // (wg_end is not read by this kernel)
    for (int i = 0; i < kMaxTileClasses; ++i) args.wg_end[i] = 0;
    hipLaunchKernelGGL((f16 ? filter_fragments_classes_kernel<true> : filter_fragments_classes_kernel<false>),
                       dim3((unsigned)((max_items + 255) / 256), (unsigned)n), dim3(256), 0, stream, args, M_T,
                       (const void *)f, frag_ws);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  // persistent workgroups: as many as fit at once, dealt to the classes by their work
  const int m_tiles = (pls[0].M + M_T - 1) / M_T;
  const int per_cu = workgroups_per_cu(lds, mt, nt, true);
  const int slots = std::max(n, (256 * per_cu) / m_tiles);
  // A class's workgroups take whole tiles in rounds, and the launch lasts as long as the
  // class that finishes last: one workgroup each, then every further one to the class whose
  // rounds times work per tile is largest.
  int gxs[kMaxTileClasses];
  for (int i = 0; i < n; ++i) gxs[i] = 1;
  for (int left = slots - n; left > 0; --left) {
    int worst = -1;
    double worst_cost = 0;
    for (int i = 0; i < n; ++i) {
      if (gxs[i] >= pls[i].total_tiles) continue;
      const double cost = (double)((pls[i].total_tiles + gxs[i] - 1) / gxs[i]) * work[i];
      if (worst < 0 || cost > worst_cost) { worst = i; worst_cost = cost; }
    }
    if (worst < 0) break;
    ++gxs[worst];
  }
  int end = 0;
  for (int i = 0; i < n; ++i) {
    end += gxs[i];
    args.wg_end[i] = end;
  }
  for (int i = n; i < kMaxTileClasses; ++i) args.wg_end[i] = end;
  dim3 grid((unsigned)end, (unsigned)m_tiles);
#define MELLIN_CLASSES_CASE(MT_, NT_, SPLIT_)                                                                  \
  if (mt == MT_ && nt == NT_ && (f16 ? 4 : 2) == SPLIT_) {                                                     \
    if (pls[0].out_half) return launch_classes_variant<MT_, NT_, true, SPLIT_>(args, lds, grid, f, g, bias, h, stream, frag_ws); \
    return launch_classes_variant<MT_, NT_, false, SPLIT_>(args, lds, grid, f, g, bias, h, stream, frag_ws);   \
  }
  MELLIN_CLASSES_CASE(2, 2, 2)
  MELLIN_CLASSES_CASE(2, 1, 2)
  MELLIN_CLASSES_CASE(4, 2, 4)
  MELLIN_CLASSES_CASE(4, 1, 4)
  MELLIN_CLASSES_CASE(2, 2, 4)
  MELLIN_CLASSES_CASE(2, 1, 4)
  MELLIN_CLASSES_CASE(1, 2, 4)
  MELLIN_CLASSES_CASE(1, 1, 4)
#undef MELLIN_CLASSES_CASE
  return hipErrorInvalidValue;
}

}  // namespace mellin
