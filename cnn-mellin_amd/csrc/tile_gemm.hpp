// Descriptor of one launch of the matrix-core gather-GEMM (tile_gemm.hip).
#pragma once

#include "mellin_common.hpp"

namespace mellin {

struct TilePlan {
  // problem (all fit 32 bits; checked by make_tile_plan)
  int batch, M, C;                 // images, output channels, contracted channels
  int nfx, nfy, nf;                // filter extent and nfx * nfy
  // The kernel's filter columns are columns f_off .. f_off + nfy - 1 of a filter whose rows
  // are f_pitch words apart: columns none of whose taps lies inside the signal for any output
  // column are left out of the plan (bf16 / f16 plans only; else f_off = 0, f_pitch = nfy).
  int f_pitch, f_off;
  int ngx, ngy;                    // signal extent
  int nox, noy, Q;                 // allocated output extent and nox * noy
  int nox_eff, noy_eff;            // outputs at or past these have no tap
  i64 f_m, f_c, g_n, g_c, h_n, h_m;
  int accumulate;
  int relu;                        // clamp the result at zero before it is stored (accumulate == 0)
  int out_half;                    // results are rounded to half precision as they are stored (accumulate == 0)
  // x axis: Mellin kinds evaluate taps per (row, filter row); linear kinds use
  // the coordinate ax * ox + bx * fx + cx (divided by ux)
  int kind_x, sx, dx, px, ux;
  int ax, bx, cx, bx_min, bx_span;
  int Ax, Bx, Cx0;                 // LDS row = Ax * (ox - ox_lo) + Bx * fx + Cx0
  // y axis: coordinate ay * oy + by * fy + cy (divided by uy)
  int ay, by, cy, uy, by_min, by_span;
  // tiling
  int segment, chunks_per_row, tiles_per_image, total_tiles;
  unsigned mg_tpi, mg_cpr, mg_noy;  // floor(2^32 / d) for tiles_per_image, chunks_per_row, noy (see udiv)
  unsigned mg_p1;                   // the same for px + 1 (Mellin correlation taps)
  int R, RS;                       // virtual rows per channel and their stride (words)
  int sbuf;                        // signal buffers in LDS: 2, or 1 when no workgroup has a second stage
  int contig;                      // virtual rows coincide with the signal's rows (same pitch): block copies
  int CP, CP_log2;                 // staged columns rounded up to a power of two
  int CC;                          // channels staged per chunk
  int KCp;                         // CC * nf rounded up to even
  int WSS;                         // stride of the K-major filter block (words)
  int split;                       // products on the bf16 matrix cores, operands as three bf16 parts each
  int f_dense;                     // split, one chunk, fp32: a channel's taps are K consecutive words in the kernel's order, K a multiple of 4
  int f16;                         // (with split) half-precision operands on the f16 matrix cores instead: one part
  int KC16;                        // split: CC * nf rounded up to a multiple of 16
  unsigned f_bytes;                // split: bytes from the filter's first word to its last one's end
  // a residue class of a Mellin x axis (SepConv::cls_*): kernel row i is output row
  // cls_first + cls_stride * i, kernel filter row j is the layer's filter row (cls_fx >> 4 j) & 15;
  // nfx / nf / nox / Q above then count the class's rows.  1, 0 and the identity otherwise.
  int cls_stride, cls_first;
  unsigned long long cls_fx;
};

// the layer's filter row behind kernel filter row j
__host__ __device__ inline int class_filter_row(unsigned long long cls_fx, int j) { return (int)((cls_fx >> (4 * j)) & 15); }

constexpr int kMaxTileClasses = 8;                  // residue classes one launch can hold

// One residue class of a Mellin axis: output rows first, first + stride, ...; nfx filter rows, listed in fx
struct MellinClass {
  int stride, first, nfx;
  unsigned long long fx;
};
// The classes of axis x into out[0 .. n); 0: the axis has one class only, more than
// max_classes, or is not a Mellin axis (nothing to gain, or too many launches).
int mellin_classes(const Axis &x, MellinClass *out, int max_classes);

// force_nt: 0 lets the plan pick the number of 32-position tiles per wavefront
// force_mt: likewise for the 32-channel tiles per workgroup (launches that share a kernel instance)
bool make_tile_plan(const SepConv &pr, TilePlan &pl, size_t *lds_bytes, int *mt, int *nt,
                    int force_nt = 0, bool trim_columns = true, int force_mt = 0);

// Bytes of scratch memory in which a launch keeps the filter as bf16 fragments, block by
// block as the stages read them (0: the layer does not run on the bf16 matrix cores, or
// its filter is one block, which every workgroup builds for itself).  Without that
// scratch every workgroup splits each block again in every tile.
size_t tile_fragment_bytes(const TilePlan &pl, int mt);

// frag_ws: tile_fragment_bytes() of device memory, 16-byte aligned, or null (required by
// a half-precision plan whose tile_fragment_bytes() is not zero).  For a plan made from a
// problem with in_half, f, g and bias point to half-precision storage; h is half-precision
// storage when the plan has out_half, else float.
hipError_t launch_tile_gemm(const TilePlan &pl, size_t lds_bytes, int mt, int nt,
                            const float *f, const float *g, const float *bias,
                            float *h, hipStream_t stream, float *frag_ws = nullptr);

// The plans of a Mellin layer's residue classes in ONE launch: every workgroup belongs to one
// class for its whole life, the classes share the chip in proportion to their work.
// tile_classes_fit_one_launch: the plans allow it (same tile shape, all staged in chunks on
// the bf16 / f16 matrix cores).  frag_ws + frag_off[i]: class i's fragments (required for
// half precision), or frag_ws null.  f_bytes[i] / h_bytes[i]: class i's filter and output
// start that many bytes past f and h (null: all at f and h).
bool tile_classes_fit_one_launch(const TilePlan *pls, const int *mts, const int *nts, int n);
hipError_t launch_tile_gemm_classes(const TilePlan *pls, const size_t *lds_bytes, int n, int mt, int nt, const float *f,
                                    const float *g, const float *bias, float *h, hipStream_t stream, float *frag_ws,
                                    const size_t *frag_off,
                                    const long long *f_bytes = nullptr, const long long *h_bytes = nullptr);

// Weight gradient (wgrad_gemm.hip): position tiling and signal staging of the
// forward problem in `t`, plus the blocking of the (c_out) x (c_in * taps) output.
struct WgradPlan {
  TilePlan t;
  i64 a_n, a_m;                    // grad_out strides: image, channel (positions are dense)
  int J;                           // c_in * nfx * nfy
  int mt, jt, nt;                  // 32-wide tiles per workgroup: channels, columns, positions per wave
  int m_groups, j_groups, M_pad, J_pad;
  int CCj;                         // input channels a column block can touch
  int GSS;                         // row stride of the staged grad_out tile (words)
  int S;                           // position shares = persistent workgroups per output block
  int rows_mode;                   // 1: the row-wise kernel (one output row per wavefront); 2: its bf16 form
  int nbuf;                        // row-wise kernel: LDS buffers per operand (1 or 2)
  int rpw;                         // row-wise kernel: output rows per wavefront and unit
  int split;                       // the caller allows the bf16 matrix cores (three-part operands)
  size_t lds_bytes, ws_bytes;
};

// allow_rows = false rules the row-wise kernel out (for comparisons)
// rows_mt / rows_nbuf / rows_rpw pin the row-wise kernel's channel tiles per
// workgroup, buffers, and output rows per wavefront and unit (0 = automatic)
bool make_wgrad_plan(const SepConv &fwd, WgradPlan &wp, bool allow_rows = true, int rows_mt = 0,
                     int rows_nbuf = 0, int rows_rpw = 0);

hipError_t launch_wgrad(const WgradPlan &wp, const float *grad_out, const float *input,
                        float *grad_weight, float *workspace, hipStream_t stream);

// wgrad_gemm.hip: W[m, j] = the sum of `partials` blocks of (M_pad x J_pad) floats, in index order;
// W is float storage, or half-precision storage (rounded once) when half_out
hipError_t launch_wgrad_reduce(const float *partials_ws, void *W, bool half_out, int partials, int M, int J,
                               int M_pad, int J_pad, hipStream_t stream);

// Weight gradient with the matrix instructions along the output positions (wgrad_pos.hip):
// half-precision layers on the f16 matrix cores, fp32 layers on the bf16 ones (three-part operands).
struct WgradPosPlan {
  int half;                        // grad_out, input and grad_weight are half-precision storage (else float)
  TilePlan t;                      // staging geometry of the forward problem
  i64 a_n, a_m;                    // grad_out strides: image, channel (positions are dense)
  int J, jt;                       // c_in * nfx * nfy; 32-column tiles per wavefront
  int mbw;                         // wavefronts side by side along the channels (64 each); the rest share a unit's steps
  int m_groups, j_groups, M_pad, J_pad;
  int CCj;                         // input channels a column block can touch
  int RB, UP;                      // output rows per unit; their positions rounded up to 16
  int S;                           // persistent workgroups per output block
  size_t lds_bytes, ws_bytes;
};

// false: the kernel does not apply (outputs wider than 128 columns, sizes beyond its limits)
bool make_wgrad_pos_plan(const SepConv &fwd, WgradPosPlan &wp, bool half);

// workspace: wp.ws_bytes
hipError_t launch_wgrad_pos(const WgradPosPlan &wp, const void *grad_out, const void *input,
                            void *grad_weight, float *workspace, hipStream_t stream);

}  // namespace mellin
