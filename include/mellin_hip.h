/*
 * mellin_hip.h -- C ABI of libmellin_hip.so: Mellin / linear convolution
 * kernels for AMD MI355X (gfx950), hand-written in HIP.
 *
 * The library replaces the device half of the reference's PyTorch extension:
 * the CUDA adapters of ext/torch_cuda.cu:45-303 and the kernels of
 * c/cuda/include/cdrobert/mellin/mconv_cuda.cuh that those adapters launch.
 * All pointers are DEVICE pointers owned by the caller; the library keeps no
 * reference to them after a call returns.  Every call is asynchronous on the
 * HIP stream passed as `stream` (NULL = the default stream), performs no
 * synchronisation, and allocates no memory.  Every function returns MELLIN_OK
 * or an error code; mellin_last_error() gives the message of the calling
 * thread's most recent failure.
 *
 * Index relations (h = output index, f = filter index, g = signal index; a tap
 * exists only if the division is exact and 0 <= g < ng):
 *
 *   Mellin correlation  g = (h + s)(f + d)/(p + 1) - u     (mconv.h:65)
 *   Mellin convolution  g = (p + 1)(h + s)/(f + d) - u     (mconv.h:24-25)
 *   linear correlation  g = (s h + d f - p)/u              (mconv.h:168-171)
 *   linear convolution  g = (s h - d f + p)/u              (mconv.h:105-107)
 *
 * with s, d, u >= 1 and p >= 0 on a Mellin axis.  "x" is the first spatial
 * axis (time), "y" the second (frequency).
 */
#ifndef MELLIN_HIP_H_
#define MELLIN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MELLIN_OK 0
#define MELLIN_ERR_ARGUMENT 1    /* inconsistent sizes / parameters / null pointer */
#define MELLIN_ERR_RUNTIME 2     /* the HIP runtime reported an error */
#define MELLIN_ERR_WORKSPACE 3   /* workspace missing or too small */

/* Axis kinds for the functions that take one. */
#define MELLIN_AXIS_MCORR 0
#define MELLIN_AXIS_MCONV 1
#define MELLIN_AXIS_LCORR 2
#define MELLIN_AXIS_LCONV 3

/* Library version (major * 10000 + minor * 100 + patch). */
int mellin_version(void);

/* Message for the calling thread's most recent non-OK return ("" if none). */
const char *mellin_last_error(void);

/* ------------------------------------------------------------------------
 * 1. Accumulating kernels: the reference's kernel-level contract.
 *
 * Same argument meaning and order as the reference's host launchers
 *   MCorr1D     mconv.h:92-100   / mconv_cuda.cuh MCorr1DCuda
 *   MConv1D     mconv.h:52-60    / MConv1DCuda
 *   MCorrLCorr  mconv.h:218-227  / MCorrLCorrCuda
 *   MConvLConv  mconv.h:154-163  / MConvLConvCuda
 * which ext/torch_cuda.cu:45-177 binds, plus the trailing stream:
 *   f   filter, (c_out, c_in, nfx[, nfy]) or (c_in, c_out, ...) if transposed_f
 *   g   signal, (batch, c_in, ngx[, ngy]) or (c_in, batch, ...) if transposed_g
 *   h   output, (batch, c_out, nhx[, nhy]) or (c_out, batch, ...) if transposed_h;
 *       caller-allocated and initialised (bias or zeros); results are ADDED
 *       to it.  nh may be smaller or larger than the support size; outputs
 *       at or beyond the support size are left untouched.
 * All three buffers are dense (C-contiguous) in the stated layout.
 * The *_lcorrlcorr / *_lconvlconv variants use the linear relations on both
 * axes; the reference has no such kernel (its non-Mellin model calls
 * torch.nn.Conv2d, models.py:334-336).
 * ------------------------------------------------------------------------ */
#define MELLIN_DECL_1D(NAME, T)                                                \
  int NAME(const T *f, const T *g, int64_t c_out, int64_t c_in, int64_t batch, \
           int64_t nf, int64_t ng, int64_t nh, int64_t s, int64_t d,           \
           int64_t p, int64_t u, int transposed_f, int transposed_g,           \
           int transposed_h, T *h, void *stream)
#define MELLIN_DECL_2D(NAME, T)                                                \
  int NAME(const T *f, const T *g, int64_t c_out, int64_t c_in, int64_t batch, \
           int64_t nfx, int64_t nfy, int64_t ngx, int64_t ngy, int64_t nhx,    \
           int64_t nhy, int64_t sx, int64_t sy, int64_t dx, int64_t dy,        \
           int64_t px, int64_t py, int64_t ux, int64_t uy, int transposed_f,   \
           int transposed_g, int transposed_h, T *h, void *stream)

MELLIN_DECL_1D(mellin_mcorr1d_f32, float);
MELLIN_DECL_1D(mellin_mcorr1d_f64, double);
MELLIN_DECL_1D(mellin_mconv1d_f32, float);
MELLIN_DECL_1D(mellin_mconv1d_f64, double);
MELLIN_DECL_2D(mellin_mcorrlcorr_f32, float);
MELLIN_DECL_2D(mellin_mcorrlcorr_f64, double);
MELLIN_DECL_2D(mellin_mconvlconv_f32, float);
MELLIN_DECL_2D(mellin_mconvlconv_f64, double);
MELLIN_DECL_2D(mellin_lcorrlcorr_f32, float);
MELLIN_DECL_2D(mellin_lcorrlcorr_f64, double);
MELLIN_DECL_2D(mellin_lconvlconv_f32, float);
MELLIN_DECL_2D(mellin_lconvlconv_f64, double);

/* ------------------------------------------------------------------------
 * 2. Operator-level entry points: one launch per pass of a correlation layer.
 *
 * These replace the adapter + autograd glue of the reference for the two
 * layer types (x axis Mellin or linear correlation, y axis always linear
 * correlation):
 *   forward          mcorrlcorr_cuda, ext/torch_cuda.cu:144-177, with
 *                    BuildOutput (ext/torch.cpp:88-101) folded in: `out` is
 *                    WRITTEN, out = bias + correlation (bias may be NULL);
 *   backward_input   the mconvlconv(weight^T, grad_out, u, s, p, d) call of
 *                    MCorrLCorrOp::backward, ext/torch.cpp:284-290;
 *                    `grad_input` is written;
 *   backward_weight  the mcorrlcorr(input^T, grad_out^T, d, s, p, u) call,
 *                    ext/torch.cpp:292-298; `grad_weight` is written.  The
 *                    reduction over batch and output positions runs in a
 *                    fixed order (no floating-point atomics), so results are
 *                    bit-reproducible from run to run.
 * Layouts are the natural dense ones:
 *   input (batch, c_in, ngx, ngy)    weight (c_out, c_in, nfx, nfy)
 *   out / grad_out (batch, c_out, nhx, nhy)      bias (c_out)
 * kind_x is MELLIN_AXIS_MCORR or MELLIN_AXIS_LCORR.  1-D layers pass a unit
 * y axis (nfy = ngy = nhy = 1, sy = dy = uy = 1, py = 0).
 *
 * The backward passes may need scratch memory (partial sums of the weight
 * gradient; for layers with few input channels the partial rows, the tap
 * products or the first-pass result of the input gradient): ask
 * mellin_corr2d_backward_*_workspace() for the byte count (0 = none) and pass
 * a device buffer of at least that size (256-byte aligned); its contents on
 * entry do not matter and are garbage on exit.  The count depends on the
 * variant in force (mellin_set_variant): query and call under the same
 * setting.
 * ------------------------------------------------------------------------ */
#define MELLIN_CORR2D_DIMS                                                     \
  int64_t batch, int64_t c_in, int64_t c_out, int64_t nfx, int64_t nfy,        \
  int64_t ngx, int64_t ngy, int64_t nhx, int64_t nhy, int64_t sx, int64_t sy,  \
  int64_t dx, int64_t dy, int64_t px, int64_t py, int64_t ux, int64_t uy

int mellin_corr2d_forward_f32(int kind_x, const float *input,
                              const float *weight, const float *bias,
                              MELLIN_CORR2D_DIMS, float *out, void *stream);
int mellin_corr2d_forward_f64(int kind_x, const double *input,
                              const double *weight, const double *bias,
                              MELLIN_CORR2D_DIMS, double *out, void *stream);

size_t mellin_corr2d_backward_input_workspace(int kind_x, int elem_bytes,
                                              MELLIN_CORR2D_DIMS);
int mellin_corr2d_backward_input_f32(int kind_x, const float *weight,
                                     const float *grad_out, MELLIN_CORR2D_DIMS,
                                     float *grad_input, void *workspace,
                                     size_t workspace_bytes, void *stream);
int mellin_corr2d_backward_input_f64(int kind_x, const double *weight,
                                     const double *grad_out, MELLIN_CORR2D_DIMS,
                                     double *grad_input, void *workspace,
                                     size_t workspace_bytes, void *stream);

size_t mellin_corr2d_backward_weight_workspace(int kind_x, int elem_bytes,
                                               MELLIN_CORR2D_DIMS);
int mellin_corr2d_backward_weight_f32(int kind_x, const float *input,
                                      const float *grad_out, MELLIN_CORR2D_DIMS,
                                      float *grad_weight, void *workspace,
                                      size_t workspace_bytes, void *stream);
int mellin_corr2d_backward_weight_f64(int kind_x, const double *input,
                                      const double *grad_out, MELLIN_CORR2D_DIMS,
                                      double *grad_weight, void *workspace,
                                      size_t workspace_bytes, void *stream);

/* The weight gradient for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  Same result, bit for bit, as
 * mellin_corr2d_backward_weight_f32, but the partial sums live in a static
 * device array of mellin_static_scratch_bytes() = 16 MiB inside the library
 * (one copy per GPU the library runs on, held until the process ends) instead
 * of a caller's workspace: the call allocates and frees nothing.  Layers whose
 * partial sums need more (mellin_corr2d_backward_weight_workspace() tells) are
 * rejected with MELLIN_ERR_WORKSPACE.  The array's address is looked up on the
 * first call made with a device current (not an allocation, but it loads the
 * code object, which a graph capture does not allow):
 * mellin_static_scratch_prepare() does only that lookup for the current device,
 * for callers to run once before they capture; a first call on a stream that is
 * already capturing is refused with MELLIN_ERR_RUNTIME and a message that says
 * so.  All calls on one GPU share the array: its
 * contents never need clearing (every word read was written by the same
 * call), but two calls that overlap in time on one GPU (different streams or
 * threads) race and give wrong results; serialise them. */
size_t mellin_static_scratch_bytes(void);
int mellin_static_scratch_prepare(void);
int mellin_corr2d_backward_weight_static_f32(int kind_x, const float *input,
                                             const float *grad_out,
                                             MELLIN_CORR2D_DIMS,
                                             float *grad_weight, void *stream);

/* forward with the layer's non-linearity applied on the way out: the acoustic
 * model runs every convolution as nonlinearity(conv(x)) (models.py:423-425), and
 * with ReLU, its default, that is out = max(0, bias + correlation) in the same
 * pass instead of a second read and write of the output.  activation:
 * MELLIN_ACT_NONE (same as mellin_corr2d_forward_*) or MELLIN_ACT_RELU. */
#define MELLIN_ACT_NONE 0
#define MELLIN_ACT_RELU 1
int mellin_corr2d_forward_act_f32(int kind_x, int activation, const float *input,
                                  const float *weight, const float *bias,
                                  MELLIN_CORR2D_DIMS, float *out, void *stream);
int mellin_corr2d_forward_act_f64(int kind_x, int activation, const double *input,
                                  const double *weight, const double *bias,
                                  MELLIN_CORR2D_DIMS, double *out, void *stream);

/* The same forward pass with scratch memory.  Layers whose input channels are staged
 * in several chunks multiply on the bf16 matrix cores from a copy of the filter cut
 * into bf16 parts (MELLIN_MATH_BF16X3); with `workspace` that copy is made once per
 * call, without it every workgroup makes its own for every tile (same result bit for
 * bit, up to 20 % slower on wide layers).  mellin_corr2d_forward_workspace() gives the
 * bytes (0 for layers that need none; the buffer 16-byte aligned); the entry points
 * without a workspace argument stay valid.  Replaces, like them, the adapter call
 * ext/torch_cuda.cu:144-177. */
size_t mellin_corr2d_forward_workspace(int kind_x, int elem_bytes, MELLIN_CORR2D_DIMS);
int mellin_corr2d_forward_ws_f32(int kind_x, int activation, const float *input,
                                 const float *weight, const float *bias,
                                 MELLIN_CORR2D_DIMS, float *out, void *workspace,
                                 size_t workspace_bytes, void *stream);

/* Half precision (the data type the reference's Autocast registration casts to,
 * ext/torch.cpp:407-430, before it calls the CUDA kernels instantiated for
 * c10::Half, ext/torch_cuda.cu:45-177): tensors hold IEEE binary16 values in
 * the layouts above.  Products of half values are exact in fp32 and are summed in
 * fp32; the result is rounded to half once (subnormal operands are not flushed).
 *
 * The kernels read the half tensors as they lie and multiply on the f16 matrix
 * cores (v_mfma_f32_32x32x16_f16), one sixth of the matrix work of the fp32 path
 * on half the bytes: the forward pass and the input gradient through the tiled
 * kernel (variant "mfma-f16"; the input gradient of layers with at most three
 * input channels and a linear x axis through the one-kernel form,
 * "mfma-f16-fused"; with few input channels otherwise, or on a Mellin axis that
 * keeps fewer rows than it is given, as two passes, "mfma-f16+fold" or
 * "mfma-f16-filter-rows+fold", whose intermediate rows are fp32 and whose fold
 * rounds each fp32 sum to half once),
 * the weight gradient through a kernel of its own whose matrix instructions run
 * along the output positions ("mfma-f16"; partial sums in fp32, added in a fixed
 * order).  Scratch memory then holds what those kernels need (the filter cut into
 * matrix fragments for layers staged in chunks of channels, first-pass rows,
 * partial sums) -- often nothing for the forward pass.  Where no such kernel
 * applies (outputs wider than 128 columns in the weight gradient, sizes beyond
 * the kernels' 32-bit limits, the "generic" and "widen" variants) the operands are
 * copied to fp32 in the scratch memory, the fp32 kernels run there and the result
 * is rounded to half: the same arithmetic in another order of summation, so the
 * two routes agree to the last half bit except where an fp32 sum lies within
 * its own rounding error of a boundary between two half values.
 * The byte count of the scratch memory comes from the matching *_workspace() call
 * (256-byte aligned buffer; query and call under the same variant); too little is
 * MELLIN_ERR_WORKSPACE. */
size_t mellin_corr2d_forward_f16_workspace(int kind_x, MELLIN_CORR2D_DIMS);
int mellin_corr2d_forward_f16(int kind_x, const void *input, const void *weight,
                              const void *bias, MELLIN_CORR2D_DIMS, void *out,
                              void *workspace, size_t workspace_bytes,
                              void *stream);
/* The same with the fused activation of mellin_corr2d_forward_act_f32 (applied to the
 * fp32 result, before the rounding); same workspace. */
int mellin_corr2d_forward_act_f16(int kind_x, int activation, const void *input,
                                  const void *weight, const void *bias,
                                  MELLIN_CORR2D_DIMS, void *out, void *workspace,
                                  size_t workspace_bytes, void *stream);
size_t mellin_corr2d_backward_input_f16_workspace(int kind_x, MELLIN_CORR2D_DIMS);
int mellin_corr2d_backward_input_f16(int kind_x, const void *weight,
                                     const void *grad_out, MELLIN_CORR2D_DIMS,
                                     void *grad_input, void *workspace,
                                     size_t workspace_bytes, void *stream);
size_t mellin_corr2d_backward_weight_f16_workspace(int kind_x, MELLIN_CORR2D_DIMS);
int mellin_corr2d_backward_weight_f16(int kind_x, const void *input,
                                      const void *grad_out, MELLIN_CORR2D_DIMS,
                                      void *grad_weight, void *workspace,
                                      size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * 3. Column ops: the gather behind the reference's matrix-multiply path and
 *    its adjoint.
 *
 * Same argument meaning and order as the reference's host launchers
 *   Snd2Col   mconv.h:262-269   / Snd2ColCuda     Col2Snd   mconv.h:301-308   / Col2SndCuda
 *   Spec2Col  mconv.h:360-368   / Spec2ColCuda    Col2Spec  mconv.h:417-425   / Col2SpecCuda
 * which ext/torch_cuda.cu:179-291 binds, plus the trailing stream:
 *   g    signal, (batch, c_in, ngx[, ngy]) or (c_in, batch, ...) if transposed_g
 *   gg   columns, (batch, c_in, nfx[, nfy], nggx[, nggy]) or (c_in, batch, ...)
 *        if transposed_gg
 * x2col WRITES every element of gg:
 *   gg[n, c, fx, fy, x, y] = g[n, c, (x + sx)(fx + dx)/(px + 1) - ux, (sy y + dy fy - py)/uy]
 * or 0 where that tap does not exist (Mellin relation on x, linear on y).
 * col2x WRITES every element of g with the sum of the gg elements whose tap it
 * is (the adjoint; the gradient of x2col), in a fixed order.
 * ------------------------------------------------------------------------ */
#define MELLIN_DECL_SND(NAME, T, SRC, DST)                                      \
  int NAME(const T *SRC, int64_t c_in, int64_t batch, int64_t nf, int64_t ng,  \
           int64_t ngg, int64_t s, int64_t d, int64_t p, int64_t u,            \
           int transposed_g, int transposed_gg, T *DST, void *stream)
#define MELLIN_DECL_SPEC(NAME, T, SRC, DST)                                     \
  int NAME(const T *SRC, int64_t c_in, int64_t batch, int64_t nfx, int64_t nfy, \
           int64_t ngx, int64_t ngy, int64_t nggx, int64_t nggy, int64_t sx,   \
           int64_t sy, int64_t dx, int64_t dy, int64_t px, int64_t py,         \
           int64_t ux, int64_t uy, int transposed_g, int transposed_gg,        \
           T *DST, void *stream)

MELLIN_DECL_SND(mellin_snd2col_f32, float, g, gg);
MELLIN_DECL_SND(mellin_snd2col_f64, double, g, gg);
MELLIN_DECL_SND(mellin_col2snd_f32, float, gg, g);
MELLIN_DECL_SND(mellin_col2snd_f64, double, gg, g);
MELLIN_DECL_SPEC(mellin_spec2col_f32, float, g, gg);
MELLIN_DECL_SPEC(mellin_spec2col_f64, double, g, gg);
MELLIN_DECL_SPEC(mellin_col2spec_f32, float, gg, g);
MELLIN_DECL_SPEC(mellin_col2spec_f64, double, gg, g);

/* ------------------------------------------------------------------------
 * 4. The pointwise layers in front of the first convolution
 *    (models.py:414-417): LogCompression.forward, layers.py:100-101, and
 *    dilation_lift, layers.py:8-21, one pass each way.
 *
 * x, y, grad_y, grad_x are dense and viewed as (outer, t, inner), the lifted
 * axis in the middle (outer = product of the sizes before it, inner = of those
 * after it).  flags selects the function:
 *   MELLIN_PW_LOG                    y = log(eps + |x|)
 *   MELLIN_PW_LIFT                   y[o, k, i] = (k + 1)^tau * x[o, k, i]
 *   MELLIN_PW_LOG | MELLIN_PW_LIFT   y[o, k, i] = (k + 1)^tau * log(eps + |x[o, k, i]|)
 * eps (> 0 with MELLIN_PW_LOG) and tau are the VALUES, not the reference
 * modules' log_eps / log_tau parameters.  backward WRITES grad_x and
 * grad_params[0] = sum grad_y * dy/d eps, grad_params[1] = sum grad_y * dy/d tau
 * (0 for a function that is not selected; |x| has derivative 0 at 0, as in
 * PyTorch); the sums run in a fixed order.  It needs
 * mellin_log_lift_backward_workspace() bytes of scratch (256-byte aligned).
 * ------------------------------------------------------------------------ */
#define MELLIN_PW_LOG 1
#define MELLIN_PW_LIFT 2

int mellin_log_lift_forward_f32(const float *x, double eps, double tau, int flags,
                                int64_t outer, int64_t t, int64_t inner,
                                float *y, void *stream);
int mellin_log_lift_forward_f64(const double *x, double eps, double tau, int flags,
                                int64_t outer, int64_t t, int64_t inner,
                                double *y, void *stream);
size_t mellin_log_lift_backward_workspace(int elem_bytes, int64_t outer,
                                          int64_t t, int64_t inner);
int mellin_log_lift_backward_f32(const float *x, const float *grad_y, double eps,
                                 double tau, int flags, int64_t outer, int64_t t,
                                 int64_t inner, float *grad_x, float *grad_params,
                                 void *workspace, size_t workspace_bytes,
                                 void *stream);
int mellin_log_lift_backward_f64(const double *x, const double *grad_y, double eps,
                                 double tau, int flags, int64_t outer, int64_t t,
                                 int64_t inner, double *grad_x, double *grad_params,
                                 void *workspace, size_t workspace_bytes,
                                 void *stream);

/* The same with eps and tau in DEVICE memory, params = {eps, tau} in the tensors' type
 * (an unused one is ignored): for values that are themselves results of device work --
 * the reference modules' exp(log_eps), exp(log_tau) -- so that a call needs no copy to
 * the host and can be captured in a graph.  eps > 0 is not checked then. */
int mellin_log_lift_forward_dev_f32(const float *x, const float *params, int flags,
                                    int64_t outer, int64_t t, int64_t inner,
                                    float *y, void *stream);
int mellin_log_lift_forward_dev_f64(const double *x, const double *params, int flags,
                                    int64_t outer, int64_t t, int64_t inner,
                                    double *y, void *stream);
int mellin_log_lift_backward_dev_f32(const float *x, const float *grad_y,
                                     const float *params, int flags, int64_t outer,
                                     int64_t t, int64_t inner, float *grad_x,
                                     float *grad_params, void *workspace,
                                     size_t workspace_bytes, void *stream);
int mellin_log_lift_backward_dev_f64(const double *x, const double *grad_y,
                                     const double *params, int flags, int64_t outer,
                                     int64_t t, int64_t inner, double *grad_x,
                                     double *grad_params, void *workspace,
                                     size_t workspace_bytes, void *stream);

/* Bias gradient of a layer, grad_bias[c] = sum over images and positions of
 * g[n, c, :] for grad_out (batch, channels, plane) -- the reference leaves this to
 * grad_out.sum(...) (ext/torch.cpp:231,300) -- in one pass together with the backward of
 * a ReLU that the forward kernel applied (MELLIN_ACT_RELU): with `out` (the layer's
 * output) given, g = grad_out where out > 0 and 0 elsewhere, and g is written to
 * grad_masked, the gradient that the backward_input / backward_weight calls then take;
 * with out == NULL, g = grad_out and grad_masked is not touched.  Sums run in a fixed
 * order.  At most 65535 images and channels.  Scratch: mellin_bias_grad_workspace(). */
size_t mellin_bias_grad_workspace(int64_t batch, int64_t channels, int64_t plane);
int mellin_bias_grad_f32(const float *grad_out, const float *out, int64_t batch,
                         int64_t channels, int64_t plane, float *grad_masked,
                         float *grad_bias, void *workspace, size_t workspace_bytes,
                         void *stream);
/* The same on half-precision tensors (grad_out, out, grad_masked, grad_bias): sums in fp32,
 * grad_bias rounded to half once; same scratch. */
int mellin_bias_grad_f16(const void *grad_out, const void *out, int64_t batch,
                         int64_t channels, int64_t plane, void *grad_masked,
                         void *grad_bias, void *workspace, size_t workspace_bytes,
                         void *stream);

/* Frequency pooling of the convolution stack (BASELINE config 5): the maximum over pairs of
 * neighbours along the last axis, y[r, j] = max(x[r, 2 j], x[r, 2 j + 1]) for x (rows, f) and
 * j < f / 2 -- what max_pool2d(x, (1, 2)) computes (the first of two equal values wins, NaN
 * propagates) -- with one byte per output in `which` (1: the second of the pair was taken)
 * instead of 8-byte indices; backward writes grad_x (rows, f) from grad_y (rows, f / 2). */
int mellin_pool_pairs_forward_f32(const float *x, int64_t rows, int64_t f, float *y,
                                  unsigned char *which, void *stream);
int mellin_pool_pairs_backward_f32(const float *grad_y, const unsigned char *which,
                                   int64_t rows, int64_t f, float *grad_x, void *stream);
/* The same on half-precision tensors. */
int mellin_pool_pairs_forward_f16(const void *x, int64_t rows, int64_t f, void *y,
                                  unsigned char *which, void *stream);
int mellin_pool_pairs_backward_f16(const void *grad_y, const unsigned char *which,
                                   int64_t rows, int64_t f, void *grad_x, void *stream);

/* Name of the kernel variant the most recent operator-level call of the
 * process (on any thread: PyTorch runs backward passes on a thread of its own)
 * dispatched to (for tests and profiling): "generic", "mfma" (tiled
 * matrix-core kernels), "mfma-rows" (row-wise weight gradient), "mfma-positions"
 * (weight gradient of layers with many channels: matrix instructions along the
 * output positions, bf16 matrix cores), "mfma-fused"
 * (one-kernel input gradient, linear x axis, few input channels),
 * "mfma-taps+fold" (tap products + gather, few input channels), "mfma+fold"
 * (two-pass input gradient), "mfma-filter-rows+fold" (the same on a Mellin axis
 * with p > 0, the first pass as a launch per filter row over the rows of
 * grad_out that have a tap of that filter row), "mfma-classes" (a layer on a Mellin axis as one
 * launch of the tiled kernel per residue class of the axis: rows with the same
 * (h + s) mod (p + 1) have taps for the same filter rows, so no launch meets a
 * (row, filter row) pair without a tap), "mfma-f16", "mfma-f16-classes" (the
 * classes of a half-precision layer sharing one launch) and
 * "mfma-f16-class-launches" (a launch each),
 * "mfma-f16-fused", "mfma-f16+fold" and "mfma-f16-filter-rows+fold"
 * (half-precision tensors on the f16 matrix cores), "mfma-narrow" (forward pass
 * of a linear x linear layer with few input channels, bf16 matrix cores) and
 * "lds-gather" (vector-ALU forward kernel, only under mellin_set_variant). */
const char *mellin_last_variant(void);

/* How the matrix-core kernels form their fp32 products (process-wide).
 *   MELLIN_MATH_BF16X3 (default)  every fp32 operand is taken as the exact sum of three
 *     bf16 values (hi = the operand rounded to the nearest bf16, mid = the remainder rounded
 *     likewise, lo = what is left, exactly) and a product as the sum of the six largest of the
 *     nine bf16 cross products, which the bf16 matrix instructions form exactly and accumulate
 *     in fp32.  The three dropped products (mid lo, lo mid, lo lo) are together at most
 *     1.01 * 2^-23 of the product in the worst case: two roundings of an fp32 multiply.
 *     Storage, accumulation and results are fp32.
 *   MELLIN_MATH_FP32  the fp32 matrix instructions (v_mfma_f32_32x32x2_f32), one sixth of
 *     the multiply rate.
 *   MELLIN_MATH_BF16X3_ALWAYS  as MELLIN_MATH_BF16X3, also for layers so small that the
 *     default leaves them on the fp32 instructions because those are faster there (layers
 *     staged in chunks of channels under 0.8 GMAC): for tests and comparisons.
 * Kernels that have no bf16 form yet run in fp32 under any setting.
 * Where the two modes differ on non-finite operands: an operand that rounds to an infinite
 * bf16 (+-infinity, and finite values above 3.3895e38 in magnitude) gives NaN results under
 * the bf16 modes (inf - inf while the operand is cut into parts), where fp32 multiply-add and
 * the reference give +-infinity (or NaN only when infinities of both signs, or infinity and
 * zero, meet).  NaN operands give NaN under every mode. */
#define MELLIN_MATH_FP32 0
#define MELLIN_MATH_BF16X3 1
#define MELLIN_MATH_BF16X3_ALWAYS 2
#define MELLIN_MATH_F16 3            /* reported by mellin_last_math only: half-precision operands on the f16 matrix cores */
int mellin_set_math(int mode);
int mellin_get_math(void);
/* The mode the matrix kernels of the most recent operator-level call actually ran in
 * (MELLIN_MATH_FP32 also for the kernels that use no matrix instructions). */
int mellin_last_math(void);

/* Force a variant for subsequent operator-level calls of the process (all threads):
 * NULL, "" or "auto" = automatic choice; "generic" = the one-thread-per-output
 * kernels; "two-pass" = automatic choice without the specialised gradient
 * kernels ("mfma-fused", "mfma-taps+fold", "mfma-rows", "mfma-positions"), i.e. the
 * tiled ones;
 * "widen" = automatic choice, but the half-precision entry points always go
 * through fp32 copies of their operands (for comparisons); "one-launch" /
 * "classes" = automatic choice, but layers on a Mellin axis never / whatever
 * their size run per residue class ("one-launch" also keeps the first pass of a
 * two-pass input gradient in one launch, and input gradients that would take two
 * passes only for the launches per filter row in the gather form; for comparisons
 * and tests; "tap-columns": automatic choice, but the tap-product input gradient
 * keeps one product per filter column in its workspace instead of summing the four
 * columns of a filter row in the kernel; "whole-classes": automatic choice, but a class's rows are never cut
 * into ranges by where the filter rows' taps leave the signal; "class-launches":
 * like "classes", with a launch per class also where one launch would hold them);
 * "lds-gather": automatic choice, but fp32 forward passes with at most eight input
 * channels and unit stride and dilation along y take the vector-ALU kernel that gathers
 * its taps from LDS (reported as "lds-gather", MELLIN_MATH_FP32: the non-matrix form the
 * matrix kernels are measured against), "no-gather": never; "no-narrow": automatic choice,
 * but linear x linear forward passes with few input channels go through the tiled kernel
 * instead of their own ("mfma-narrow": both axes correlations without padding or
 * up-sampling, unit stride and dilation along y, an even number of filter columns,
 * c_in * nfx * nfy <= 128, at least 1024 tiles of 256 positions x 64 channels), "narrow":
 * that kernel for layers of its class however small (for tests).
 * Unknown names are rejected with MELLIN_ERR_ARGUMENT and change nothing.  The setting (like
 * mellin_set_math's) is several process-wide words: change it while no operator-level call
 * of the process is running, or a call may see part of the old and part of the new one (a
 * workspace query and the call that follows it can then disagree: MELLIN_ERR_WORKSPACE). */
int mellin_set_variant(const char *name);

#ifdef __cplusplus
}
#endif
#endif /* MELLIN_HIP_H_ */
