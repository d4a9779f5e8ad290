// extern "C" surface of libmellin_hip (declared in include/mellin_hip.h):
// argument validation, descriptor construction and kernel-variant dispatch.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <numeric>

#include "../../include/mellin_hip.h"
#include "mellin_common.hpp"
#include "igrad_gemm.hpp"
#include "tile_gemm.hpp"
#include "gather_kernels.hpp"
#include "narrow_gemm.hpp"

using namespace mellin;

// Scratch memory of mellin_corr2d_backward_weight_static_f32: one copy per GPU that runs
// code of this library, held until the process ends.  The name is a host-side handle, not
// a device address: host code only ever uses the per-device address that
// static_scratch() obtains from hipGetSymbolAddress.
#define MELLIN_STATIC_SCRATCH_BYTES (16u << 20)
static __device__ __align__(256) unsigned char scratch[MELLIN_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_error[512] = "";
// Process-wide, not per thread: PyTorch runs the backward pass of device tensors on its
// autograd thread, and a variant forced from the user's thread must hold there too.
std::atomic<const char *> g_variant{""};
std::atomic<int> g_no_classes{0};       // Mellin layers as one launch, not one per residue class (mellin_set_variant "one-launch")
std::atomic<int> g_split_classes{0};    // ... every class a launch of its own ("class-launches": for comparisons)
std::atomic<int> g_all_classes{0};      // ... one per class whatever the layer's size ("classes": for tests)
std::atomic<int> g_no_yfold{0};         // tap products stored per filter column, not summed over them ("tap-columns": for comparisons)
std::atomic<int> g_whole_classes{0};    // ... a class's rows never cut into ranges ("whole-classes": for comparisons)
std::atomic<int> g_gather{0};          // 1: the LDS-gather kernels (vector ALUs) wherever they apply ("lds-gather"); -1: never ("no-gather")
std::atomic<int> g_no_narrow{0};       // 1: few-channel linear forward passes through the tiled kernel ("no-narrow": for comparisons); -1: their own kernel whatever the size ("narrow": for tests)
std::atomic<int> g_widen{0};            // half-precision entry points: always through fp32 copies (mellin_set_variant "widen")
std::atomic<int> g_math{MATH_BF16X3};   // how fp32 products are formed on the matrix cores (mellin_set_math)
std::atomic<int> g_last_math{MATH_FP32};   // what the kernels of the most recent operator-level call multiplied with
std::atomic<int> g_forced{0};    // 0 automatic, 1 generic, 2 automatic without the newer specialised kernels
                                 // and without the row-wise weight gradient

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_hip(hipError_t e, const char *what) {
  if (e == hipSuccess) return MELLIN_OK;
  return fail(MELLIN_ERR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
}

// No form of the input gradient may ask for more scratch memory than this; a layer whose
// specialised forms would need more runs in the gather form, which needs none.
const size_t kMaxWorkspaceBytes = (size_t)1 << 30;

bool mellin_kind(int k) { return k == AX_MCORR || k == AX_MCONV; }

// Parameter domain of one axis.  s, d, u divide or scale indices and must be
// positive; on a Mellin axis p + 1 is a divisor so p >= 0.
int check_axis(const char *fn, const char *ax, int kind, i64 nf, i64 ng, i64 nh,
               i64 s, i64 d, i64 p, i64 u) {
  if (nf < 0 || ng < 0 || nh < 0)
    return fail(MELLIN_ERR_ARGUMENT, "%s: negative size on the %s axis (nf=%lld ng=%lld nh=%lld)",
                fn, ax, (long long)nf, (long long)ng, (long long)nh);
  if (s < 1 || d < 1 || u < 1)
    return fail(MELLIN_ERR_ARGUMENT, "%s: s, d and u must be >= 1 on the %s axis (s=%lld d=%lld u=%lld)",
                fn, ax, (long long)s, (long long)d, (long long)u);
  if (mellin_kind(kind) && p < 0)
    return fail(MELLIN_ERR_ARGUMENT, "%s: p must be >= 0 on the Mellin axis (p=%lld)", fn, (long long)p);
  // keep index products inside 62 bits
  const i64 lim = (i64)1 << 30;
  if (nf > lim || ng > lim || nh > lim || s > lim || d > lim || u > lim || p > lim || p < -lim)
    return fail(MELLIN_ERR_ARGUMENT, "%s: size or parameter too large on the %s axis", fn, ax);
  return MELLIN_OK;
}

int check_channels(const char *fn, i64 c_out, i64 c_in, i64 batch) {
  if (c_out < 0 || c_in < 0 || batch < 0)
    return fail(MELLIN_ERR_ARGUMENT, "%s: negative channel or batch count (c_out=%lld c_in=%lld batch=%lld)",
                fn, (long long)c_out, (long long)c_in, (long long)batch);
  // with the per-axis limit of 2^30, counts up to 2^20 keep every product of sizes the
  // entry points form (a tensor's element count, a fan-in) inside 63 bits
  const i64 lim = (i64)1 << 20;
  if (c_out > lim || c_in > lim || batch > lim)
    return fail(MELLIN_ERR_ARGUMENT, "%s: channel or batch count beyond 2^20 (c_out=%lld c_in=%lld batch=%lld)",
                fn, (long long)c_out, (long long)c_in, (long long)batch);
  return MELLIN_OK;
}

// Element counts of the tensors of a call must stay below 2^60 (no such tensor can exist;
// the test keeps every later product of sizes free of signed overflow).
int check_counts(const char *fn, double a, double b, double c) {
  const double lim = 1152921504606846976.0;   // 2^60
  if (a >= lim || b >= lim || c >= lim)
    return fail(MELLIN_ERR_ARGUMENT, "%s: a tensor of this call would have 2^60 elements or more", fn);
  return MELLIN_OK;
}

// Gather-form dispatch: the matrix-core tile kernel when it applies (fp32,
// sizes within its plan limits), otherwise one thread per output.
template <typename T>
hipError_t run_sepconv(const SepConv &pr, const T *f, const T *g, const T *bias,
                       T *h, hipStream_t stream, void *frag_ws = nullptr, size_t frag_bytes = 0) {
  (void)frag_ws; (void)frag_bytes;
  g_variant = "generic";
  g_last_math = MATH_FP32;
  return launch_sepconv_generic<T>(pr, f, g, bias, h, stream);
}

// A layer on a Mellin x axis as one launch of the tiled kernel per residue class of the axis
// (tile_gemm.hip: mellin_classes): no launch meets a (row, filter row) pair without a tap, so
// none stages or multiplies the zeros that stand for such pairs in the single launch.
constexpr int kMaxClasses = 8;
struct ClassPlans {
  int n = 0;
  TilePlan pl[kMaxClasses];
  size_t lds[kMaxClasses], frag_off[kMaxClasses];
  int mt[kMaxClasses], nt[kMaxClasses];
  size_t frag_bytes = 0;           // all classes' filter fragments, each region 256-byte aligned
  bool cut = false;                // classes cut into ranges of rows (plan_mellin_classes)
};

// False: the layer stays with the single launch (one class only or too many, a class with no
// filter row or no plan on the bf16 / f16 matrix cores, a layer too small to pay for the launches).
bool plan_mellin_classes(const SepConv &pr, ClassPlans &cp, bool allow_cut = true) {
  if (g_forced != 0 || g_no_classes || pr.accumulate || pr.cls_nfx || (!pr.in_half && pr.math == MATH_FP32)) return false;
  const double work = (double)pr.batch * pr.x.nh * pr.y.nh * pr.c_out * pr.c_in * pr.x.nf * pr.y.nf;
  // (correlation axes only, i.e. forward passes: the classes of a convolution axis, six for a
  // four-row filter with p = 1, are launches too small to win -- measured 10-30 % slower on
  // most layers of the 10-layer stack, in half precision on all of them)
  if ((work < 4e9 || pr.x.kind != AX_MCORR) && !g_all_classes) return false;
  MellinClass mc[kMaxClasses];
  const int n = mellin_classes(pr.x, mc, kMaxClasses);
  if (n < 2) return false;
  // the launches: a class, or a range of a class's rows (rows first, first + stride, ... < end)
  struct Item { int stride, first, end, nfx; unsigned long long fx; };
  Item items[kMaxClasses];
  int n_items = 0;
  for (int r = 0; r < n; ++r) {
    if (mc[r].first >= pr.x.nh) continue;                   // no output row in this class
    if (mc[r].nfx == 0) return false;                       // rows that are bias alone: the single launch writes them
    items[n_items++] = Item{mc[r].stride, mc[r].first, (int)pr.x.nh, mc[r].nfx, mc[r].fx};
  }
  cp.cut = false;
  if (pr.x.kind == AX_MCORR && allow_cut && !pr.in_half && !g_whole_classes && !g_split_classes) {
    // On a correlation axis the tap of filter row f is inside the signal for the rows up to
    // h_f = floor((ng - 1 + u)(p + 1) / (f + d)) - s only: a layer whose output reaches past
    // the support of its later filter rows (a stack that keeps its number of rows) stages
    // and multiplies rows of zeros for those pairs.  A class's rows are cut at the h_f of its
    // filter rows, each range a unit of work with the filter rows that still have taps
    // there, when that leaves out a tenth of the (row, filter row) pairs or more and the
    // units stay within the limit; ranges of under sixteen rows join the range before them.
    // The units share one kernel instance and one launch (launch_mellin_classes).  fp32
    // layers only: over the forward passes of the 10-layer stack 8.35 -> 7.44 ms (eight
    // layers 12-21 % faster, the two 128 -> 128 layers on 10 bins 8 % slower); in half
    // precision, where the classes share a launch already, 3.10 -> 3.06 ms with layers
    // moving either way by up to 20 %, so half-precision classes stay whole.
    Item cut[kMaxClasses];
    int n_cut = 0;
    double pairs_whole = 0, pairs_cut = 0;
    bool ok = true;
    for (int i = 0; i < n_items && ok; ++i) {
      const Item &it = items[i];
      i64 end_f[16], ends[16];
      int n_ends = 0;
      for (int j = 0; j < it.nfx; ++j) {
        const i64 f = class_filter_row(it.fx, j);
        const i64 h_f = (pr.x.ng - 1 + pr.x.u) * (pr.x.p + 1) / (f + pr.x.d) - pr.x.s;
        end_f[j] = std::max<i64>(0, std::min<i64>(it.end, h_f + 1));
        bool seen = false;
        for (int e = 0; e < n_ends; ++e) seen = seen || ends[e] == end_f[j];
        if (!seen) ends[n_ends++] = end_f[j];
      }
      std::sort(ends, ends + n_ends);
      if (ends[n_ends - 1] < it.end) { ok = false; break; }           // rows past every tap: bias alone
      pairs_whole += (double)((it.end - it.first + it.stride - 1) / it.stride) * it.nfx;
      i64 lo = 0;
      const int first_of_class = n_cut;
      for (int e = 0; e < n_ends; ++e) {
        const i64 hi = ends[e];
        // the class's first row at or after lo
        const i64 first = lo <= it.first ? it.first : it.first + (lo - it.first + it.stride - 1) / it.stride * it.stride;
        const i64 rows = first < hi ? (hi - first + it.stride - 1) / it.stride : 0;
        if (rows == 0) continue;
        if (rows < 16 && n_cut > first_of_class) {                    // joins the range before it (a superset of its filter rows)
          pairs_cut += (double)rows * cut[n_cut - 1].nfx;
          cut[n_cut - 1].end = (int)hi;
          lo = hi;
          continue;
        }
        if (n_cut == kMaxClasses) { ok = false; break; }
        Item c{it.stride, (int)first, (int)hi, 0, 0};
        for (int j = 0; j < it.nfx; ++j)
          if (end_f[j] >= hi) c.fx |= (unsigned long long)class_filter_row(it.fx, j) << (4 * c.nfx++);
        pairs_cut += (double)rows * c.nfx;
        cut[n_cut++] = c;
        lo = hi;
      }
    }
    if (ok && n_cut > n_items && pairs_cut <= 0.9 * pairs_whole) {
      n_items = n_cut;
      for (int i = 0; i < n_cut; ++i) items[i] = cut[i];
      cp.cut = true;
    }
  }
  cp.n = 0;
  cp.frag_bytes = 0;
  for (int r = 0; r < n_items; ++r) {
    SepConv c = pr;
    c.cls_stride = items[r].stride; c.cls_first = items[r].first; c.cls_nfx = items[r].nfx; c.cls_fx = items[r].fx;
    c.x.nh = items[r].end;
    c.x.nh_eff = std::min<i64>(pr.x.nh_eff, items[r].end);
    if (!c.in_half) c.math = MATH_BF16X3_ALWAYS;
    const int i = cp.n;
    // (ranges of one layer share the tile shape of the first: one kernel instance for all)
    if (!make_tile_plan(c, cp.pl[i], &cp.lds[i], &cp.mt[i], &cp.nt[i], cp.cut && i > 0 ? cp.nt[0] : 0, true,
                        cp.cut && i > 0 ? cp.mt[0] : 0))
      return cp.cut ? plan_mellin_classes(pr, cp, false) : false;
    cp.frag_off[i] = cp.frag_bytes;
    cp.frag_bytes += (tile_fragment_bytes(cp.pl[i], cp.mt[i]) + 255) & ~(size_t)255;
    ++cp.n;
  }
  // (ranges are worth their number only as one launch)
  if (cp.cut && !tile_classes_fit_one_launch(cp.pl, cp.mt, cp.nt, cp.n)) return plan_mellin_classes(pr, cp, false);
  return cp.n >= 2;
}

// frag_ws: cp.frag_bytes of scratch memory, or null / too little (fp32 layers then build the
// fragments per stage; half-precision layers need it when cp.frag_bytes is not zero)
hipError_t launch_mellin_classes(const ClassPlans &cp, const void *f, const void *g, const void *bias, void *h,
                                 hipStream_t stream, void *frag_ws, size_t frag_bytes, bool *one_launch = nullptr) {
  if (one_launch) *one_launch = false;
  const bool use_ws = frag_ws && ((uintptr_t)frag_ws & 15) == 0 && frag_bytes >= cp.frag_bytes;
  // One launch for all classes in half precision (measured 7 % faster over the forward passes
  // of the 10-layer stack than a launch per class: no gaps, the chip shared by the work of the
  // classes); in fp32, where a class's launch is long enough to fill the chip by itself, a
  // launch per class was the faster by 5 %.
  if (!g_split_classes && (cp.pl[0].f16 || cp.cut) && use_ws && tile_classes_fit_one_launch(cp.pl, cp.mt, cp.nt, cp.n)) {
    if (one_launch) *one_launch = true;
    return launch_tile_gemm_classes(cp.pl, cp.lds, cp.n, cp.mt[0], cp.nt[0], (const float *)f, (const float *)g,
                                    (const float *)bias, (float *)h, stream, use_ws ? (float *)frag_ws : nullptr,
                                    cp.frag_off);
  }
  for (int i = 0; i < cp.n; ++i) {
    float *ws = use_ws && tile_fragment_bytes(cp.pl[i], cp.mt[i]) ? (float *)((char *)frag_ws + cp.frag_off[i]) : nullptr;
    hipError_t e = launch_tile_gemm(cp.pl[i], cp.lds[i], cp.mt[i], cp.nt[i], (const float *)f, (const float *)g,
                                    (const float *)bias, (float *)h, stream, ws);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// Where the gather kernel is the faster forward pass (measured on the benchmark's layers): TBD
bool gather_forward_wins(const SepConv &pr) {
  (void)pr;
  return false;
}

template <>
hipError_t run_sepconv<float>(const SepConv &pr, const float *f, const float *g,
                              const float *bias, float *h, hipStream_t stream, void *frag_ws,
                              size_t frag_bytes) {
  {
    ClassPlans cp;
    bool classes = plan_mellin_classes(pr, cp);
    // (ranges need the scratch memory for their fragments: without it, whole classes)
    if (classes && cp.cut && !(frag_ws && ((uintptr_t)frag_ws & 15) == 0 && frag_bytes >= cp.frag_bytes))
      classes = plan_mellin_classes(pr, cp, false);
    if (classes) {
      g_variant = "mfma-classes";
      g_last_math = MATH_BF16X3;
      return launch_mellin_classes(cp, f, g, bias, h, stream, frag_ws, frag_bytes);
    }
  }
  if (g_forced == 0 && g_gather >= 0) {
    // few input channels and a small layer: the vector-ALU gather kernel (gather_kernels.hip)
    GatherPlan gp;
    if ((g_gather > 0 || gather_forward_wins(pr)) && make_gather_forward_plan(pr, gp)) {
      g_variant = "lds-gather";
      g_last_math = MATH_FP32;
      return launch_gather_forward(gp, f, g, bias, h, stream);
    }
  }
  if (g_forced == 0 && g_no_narrow <= 0) {
    // few input channels, linear axes without padding: the signal cut into bf16 parts once per
    // staged element (narrow_gemm.hip)
    NarrowPlan np;
    if (make_narrow_plan(pr, np, g_no_narrow < 0)) {
      g_variant = "mfma-narrow";
      g_last_math = MATH_BF16X3;
      return launch_narrow_forward(np, f, g, bias, h, stream);
    }
  }
  if (g_forced != 1) {
    TilePlan pl;
    size_t lds = 0;
    int mt = 0, nt = 0;
    if (make_tile_plan(pr, pl, &lds, &mt, &nt)) {
      g_variant = "mfma";
      g_last_math = pl.split ? MATH_BF16X3 : MATH_FP32;
      // scratch memory for the filter's bf16 fragments, when the caller brought enough
      const bool use_ws = frag_ws && ((uintptr_t)frag_ws & 15) == 0 && frag_bytes >= tile_fragment_bytes(pl, mt);
      return launch_tile_gemm(pl, lds, mt, nt, f, g, bias, h, stream, use_ws ? (float *)frag_ws : nullptr);
    }
  }
  g_variant = "generic";
  g_last_math = MATH_FP32;
  return launch_sepconv_generic<float>(pr, f, g, bias, h, stream);
}

// ---- section 1: accumulate-into-h kernels ---------------------------------
template <typename T>
int accumulate_2d(const char *fn, int kind_x, int kind_y, const T *f, const T *g,
                  i64 c_out, i64 c_in, i64 batch, i64 nfx, i64 nfy, i64 ngx,
                  i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy,
                  i64 px, i64 py, i64 ux, i64 uy, int tf, int tg, int th, T *h,
                  void *stream) {
  int rc;
  if ((rc = check_channels(fn, c_out, c_in, batch))) return rc;
  if ((rc = check_axis(fn, "x", kind_x, nfx, ngx, nhx, sx, dx, px, ux))) return rc;
  if ((rc = check_axis(fn, "y", kind_y, nfy, ngy, nhy, sy, dy, py, uy))) return rc;
  if ((rc = check_counts(fn, (double)c_out * c_in * nfx * nfy, (double)batch * c_in * ngx * ngy,
                         (double)batch * c_out * nhx * nhy))) return rc;
  const i64 nf = nfx * nfy, ng = ngx * ngy, nh = nhx * nhy;
  if (batch * c_out * nh == 0) return MELLIN_OK;               // nothing to write
  if (c_in * nf * ng == 0) return MELLIN_OK;                   // empty sum: h unchanged
  if (!f || !g || !h) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  SepConv pr;
  pr.x = make_axis(kind_x, nfx, ngx, nhx, sx, dx, px, ux);
  pr.y = make_axis(kind_y, nfy, ngy, nhy, sy, dy, py, uy);
  pr.batch = batch; pr.c_out = c_out; pr.c_in = c_in;
  pr.f_m = tf ? nf : c_in * nf;   pr.f_c = tf ? c_out * nf : nf;
  pr.g_n = tg ? ng : c_in * ng;   pr.g_c = tg ? batch * ng : ng;
  pr.h_n = th ? nh : c_out * nh;  pr.h_m = th ? batch * nh : nh;
  pr.accumulate = 1;
  pr.math = g_math;
  return check_hip(run_sepconv<T>(pr, f, g, (const T *)nullptr, h, (hipStream_t)stream), fn);
}

// ---- section 2: operator-level entry points -------------------------------
int check_corr2d(const char *fn, int kind_x, i64 batch, i64 c_in, i64 c_out,
                 i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy, i64 sx,
                 i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy) {
  int rc;
  if (kind_x != AX_MCORR && kind_x != AX_LCORR)
    return fail(MELLIN_ERR_ARGUMENT, "%s: kind_x must be MELLIN_AXIS_MCORR or MELLIN_AXIS_LCORR", fn);
  if ((rc = check_channels(fn, c_out, c_in, batch))) return rc;
  if ((rc = check_axis(fn, "x", kind_x, nfx, ngx, nhx, sx, dx, px, ux))) return rc;
  if ((rc = check_axis(fn, "y", AX_LCORR, nfy, ngy, nhy, sy, dy, py, uy))) return rc;
  if ((rc = check_counts(fn, (double)c_out * c_in * nfx * nfy, (double)batch * c_in * ngx * ngy,
                         (double)batch * c_out * nhx * nhy))) return rc;
  return MELLIN_OK;
}

SepConv forward_problem(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx,
                        i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px,
                        i64 py, i64 ux, i64 uy) {
  const i64 nf = nfx * nfy, ng = ngx * ngy, nh = nhx * nhy;
  SepConv pr;
  pr.x = make_axis(kind_x, nfx, ngx, nhx, sx, dx, px, ux);
  pr.y = make_axis(AX_LCORR, nfy, ngy, nhy, sy, dy, py, uy);
  pr.batch = batch; pr.c_out = c_out; pr.c_in = c_in;
  pr.f_m = c_in * nf; pr.f_c = nf;
  pr.g_n = c_in * ng; pr.g_c = ng;
  pr.h_n = c_out * nh; pr.h_m = nh;
  pr.accumulate = 0;
  pr.math = g_math;
  return pr;
}

// Scratch bytes with which the tiled kernel keeps the filter of problem `pr` as bf16
// fragments (0: it would not use any).
size_t fragment_bytes(const SepConv &pr) {
  if (g_forced == 1) return 0;
  {
    ClassPlans cp;
    if (plan_mellin_classes(pr, cp)) return cp.frag_bytes;
  }
  TilePlan pl;
  size_t lds = 0;
  int mt = 0, nt = 0;
  if (!make_tile_plan(pr, pl, &lds, &mt, &nt)) return 0;
  return tile_fragment_bytes(pl, mt);
}

template <typename T>
int corr2d_forward(const char *fn, int kind_x, const T *input, const T *weight,
                   const T *bias, i64 batch, i64 c_in, i64 c_out, i64 nfx,
                   i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy,
                   i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, T *out,
                   void *stream, int activation = MELLIN_ACT_NONE, void *half_out = nullptr,
                   bool *wrote_half = nullptr, void *workspace = nullptr, size_t workspace_bytes = 0) {
  int rc = check_corr2d(fn, kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx,
                        nhy, sx, sy, dx, dy, px, py, ux, uy);
  if (rc) return rc;
  if (activation != MELLIN_ACT_NONE && activation != MELLIN_ACT_RELU)
    return fail(MELLIN_ERR_ARGUMENT, "%s: activation must be MELLIN_ACT_NONE or MELLIN_ACT_RELU (got %d)", fn,
                activation);
  const i64 nf = nfx * nfy, ng = ngx * ngy, nh = nhx * nhy;
  if (batch * c_out * nh == 0) return MELLIN_OK;
  if (!out || (c_in * nf * ng != 0 && (!input || !weight)))
    return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  SepConv pr;
  pr.x = make_axis(kind_x, nfx, ngx, nhx, sx, dx, px, ux);
  pr.y = make_axis(AX_LCORR, nfy, ngy, nhy, sy, dy, py, uy);
  if (c_in * nf * ng == 0) pr.x.nh_eff = 0;                   // empty sum: out = bias
  pr.batch = batch; pr.c_out = c_out; pr.c_in = c_in;
  pr.f_m = c_in * nf; pr.f_c = nf;
  pr.g_n = c_in * ng; pr.g_c = ng;
  pr.h_n = c_out * nh; pr.h_m = nh;
  pr.accumulate = 0;
  pr.math = g_math;
  pr.relu = activation == MELLIN_ACT_RELU;
  if (wrote_half) *wrote_half = false;
  if (half_out && sizeof(T) == 4 && g_forced != 1) {
    // the matrix-core kernel can round its fp32 results to half precision as it stores
    // them: no fp32 copy of the output, no second pass over it
    TilePlan pl;
    size_t lds = 0;
    int mt = 0, nt = 0;
    // (not where the fp32 entry point would take the few-channel kernel, which has no half-precision
    // store: the caller rounds that kernel's fp32 result instead, so that both give the same bits)
    NarrowPlan narrow;
    const bool few_channels = g_forced == 0 && g_no_narrow <= 0 && g_gather <= 0 && make_narrow_plan(pr, narrow, g_no_narrow < 0);
    pr.out_half = 1;
    if (!few_channels && make_tile_plan(pr, pl, &lds, &mt, &nt)) {
      g_variant = "mfma";
      g_last_math = pl.split ? MATH_BF16X3 : MATH_FP32;
      if (wrote_half) *wrote_half = true;
      return check_hip(launch_tile_gemm(pl, lds, mt, nt, (const float *)weight, (const float *)input,
                                        (const float *)bias, (float *)half_out, (hipStream_t)stream), fn);
    }
    pr.out_half = 0;
  }
  return check_hip(run_sepconv<T>(pr, weight, input, bias, out, (hipStream_t)stream, workspace, workspace_bytes), fn);
}

// grad_input[n, ci, gx, gy] = sum_{co, fx, fy} weight[co, ci, fx, fy] *
//   grad_out[n, co, hx, hy] over the (hx, hy) whose forward taps land on
// (gx, gy).  Solving the forward relations for the output index gives the
// convolution relations with s and u exchanged:
//   x (Mellin): hx = (p + 1)(gx + u)/(fx + d) - s
//   x (linear): hx = (u gx - d fx + p)/s
//   y (linear): hy = (u gy - d fy + p)/s
// Two-pass input gradient for layers with few input channels.  With c_in output
// channels the matrix-core tile would be mostly padding, so the first pass runs
// the gather-GEMM over the y axis only, with one output channel per
// (input channel, filter row) pair, into a workspace
//   Y[n, ci * nfx + fx, hx, gy] = sum_{co, fy} weight[co, ci, fx, fy] * grad_out[n, co, hx, .]
// and the second pass (fold_x.hip) adds the filter rows whose x tap exists.
struct TwoPassInput {
  TilePlan plan;
  size_t lds, ws_bytes;
  size_t frag_off, frag_bytes;     // the first pass's filter fragments, behind Y in the workspace
  int mt, nt;
  Axis fold;
  // The first pass as a launch per filter row (rows > 0; plan_first_pass_rows): launch i works
  // out the c_in output channels of filter row fx[i], on the rows of grad_out that have a tap
  // of that filter row and on no others.
  int rows = 0;
  bool rows_one_launch = false;    // the launches planned with one tile shape: they share a launch
  TilePlan row_plan[kMaxClasses];
  size_t row_lds[kMaxClasses], row_frag_off[kMaxClasses];    // (fragment regions: offsets from frag_off)
  int row_mt[kMaxClasses], row_nt[kMaxClasses], row_fx[kMaxClasses];
};

// On a Mellin x axis with p > 0 the fold reads Y[., ci * nfx + fx, hx, .] only where
// (hx + s)(fx + d) is a multiple of p + 1 and the tap (hx + s)(fx + d)/(p + 1) - u is a row
// of grad_input: for filter row fx, the rows hx = first, first + q, ... with
// q = (p + 1) / gcd(fx + d, p + 1), up to the last one whose tap is inside.  A launch per
// filter row over exactly those rows (a residue class of an identity axis, c_in output
// channels, the filter and Y addressed with the filter row's offsets and the strides of the
// (input channel, filter row) layout) multiplies nothing the fold does not read; the single
// launch works out every (row, filter row) pair.  Taken when that saves a fifth of the
// 32-channel row blocks or more and the layer is large enough to pay for the launches.
// `first` is the single launch's problem.
bool plan_first_pass_rows(const SepConv &first, i64 c_in, i64 nfx, i64 nfy, i64 nhx, i64 ngx, i64 ngy, i64 sx, i64 dx,
                          i64 px, i64 ux, TwoPassInput &tp) {
  tp.rows = 0;
  if (g_forced != 0 || g_no_classes || px < 1 || nfx < 2 || nfx > kMaxClasses) return false;
  if (!first.in_half && first.math == MATH_FP32) return false;         // (classes run on the bf16 / f16 matrix cores)
  // (a launch and a fragment launch per filter row: layers whose whole first pass is 16 GMAC
  // or more, unless the form is asked for by name -- a 1-D layer of 0.5 GMAC with eight filter
  // rows measured 56 -> 159 us)
  const double work = (double)first.batch * (double)(c_in * nfx) * (double)(nhx * ngy) * (double)first.c_in * (double)nfy;
  if (work < 1.6e10 && !g_all_classes) return false;
  i64 lo[kMaxClasses], hi[kMaxClasses], q[kMaxClasses];
  i64 blocks = 0;
  int n = 0;
  for (i64 fx = 0; fx < nfx; ++fx) {
    const i64 k = fx + dx, g = std::gcd(k, px + 1);
    const i64 step = (px + 1) / g;
    // t = hx + s: a multiple of step with u (p + 1) <= t k <= (ngx - 1 + u)(p + 1), hx in [0, nhx)
    const i64 t_lo = std::max<i64>(sx, (ux * (px + 1) + k - 1) / k);
    const i64 t_hi = std::min<i64>(nhx - 1 + sx, (ngx - 1 + ux) * (px + 1) / k);
    const i64 t_first = (t_lo + step - 1) / step * step, t_last = t_hi / step * step;
    if (t_first > t_last) continue;                                    // no tap of this filter row at all
    lo[n] = t_first - sx; hi[n] = t_last - sx; q[n] = step;
    tp.row_fx[n] = (int)fx;
    blocks += ((c_in + 31) / 32) * ((hi[n] - lo[n]) / step + 1);
    ++n;
  }
  if (n == 0 || blocks * 5 > ((c_in * nfx + 31) / 32) * nhx * 4) return false;
  // every launch with the tile shape it would pick by itself (force_mt = 0), or all with one
  auto plan_all = [&](int force_mt, int force_nt, size_t &frag) {
    frag = 0;
    for (int i = 0; i < n; ++i) {
      SepConv c = first;
      c.x = make_axis(AX_MCORR, 1, nhx, hi[i] + 1, 1, 1, 0, 1);        // tap (h + 1)(0 + 1)/1 - 1 = h: rows pass through
      c.c_out = c_in;
      c.f_m = nfx * nfy;
      c.h_m = nfx * nhx * ngy;
      c.cls_stride = (int)q[i]; c.cls_first = (int)lo[i]; c.cls_nfx = 1; c.cls_fx = 0;
      if (!c.in_half) c.math = MATH_BF16X3_ALWAYS;
      if (!make_tile_plan(c, tp.row_plan[i], &tp.row_lds[i], &tp.row_mt[i], &tp.row_nt[i], force_nt, true, force_mt))
        return false;
      tp.row_frag_off[i] = frag;
      frag += (tile_fragment_bytes(tp.row_plan[i], tp.row_mt[i]) + 255) & ~(size_t)255;
    }
    return true;
  };
  size_t frag = 0;
  if (!plan_all(0, 0, frag)) return false;
  // One launch for all filter rows (tile_gemm_classes_kernel, the workgroups dealt to the
  // filter rows by their work) where the plans allow it with the tile shape of the filter
  // row that has the most rows: the launches of the filter rows with few rows are too
  // short to fill the chip by themselves.
  tp.rows_one_launch = false;
  if (n >= 2 && !g_split_classes) {
    int big = 0;
    for (int i = 1; i < n; ++i)
      if (tp.row_plan[i].Q > tp.row_plan[big].Q) big = i;
    const int mt = tp.row_mt[big], nt = tp.row_nt[big];
    size_t frag_one = 0;
    if (plan_all(mt, nt, frag_one) && tile_classes_fit_one_launch(tp.row_plan, tp.row_mt, tp.row_nt, n)) {
      tp.rows_one_launch = true;
      frag = frag_one;
    } else if (!plan_all(0, 0, frag)) {
      return false;
    }
  }
  tp.rows = n;
  tp.frag_bytes = frag;
  return true;
}

// The first pass of a two-pass plan: Y (fp32) from the weight and grad_out (elem_bytes each).
hipError_t launch_first_pass(const TwoPassInput &tp, const void *weight, const void *grad_out, void *ws,
                             int elem_bytes, hipStream_t stream) {
  float *frag = tp.frag_bytes ? (float *)((char *)ws + tp.frag_off) : nullptr;
  if (tp.rows == 0)
    return launch_tile_gemm(tp.plan, tp.lds, tp.mt, tp.nt, (const float *)weight, (const float *)grad_out, nullptr,
                            (float *)ws, stream, frag);
  if (tp.rows_one_launch && frag && ((uintptr_t)frag & 15) == 0) {
    long long f_bytes[kMaxClasses], h_bytes[kMaxClasses];
    for (int i = 0; i < tp.rows; ++i) {
      const TilePlan &pl = tp.row_plan[i];
      f_bytes[i] = (long long)tp.row_fx[i] * pl.f_pitch * elem_bytes;
      h_bytes[i] = (long long)tp.row_fx[i] * pl.ngx * pl.noy * 4;
    }
    return launch_tile_gemm_classes(tp.row_plan, tp.row_lds, tp.rows, tp.row_mt[0], tp.row_nt[0], (const float *)weight,
                                    (const float *)grad_out, nullptr, (float *)ws, stream, frag, tp.row_frag_off, f_bytes,
                                    h_bytes);
  }
  for (int i = 0; i < tp.rows; ++i) {
    const TilePlan &pl = tp.row_plan[i];
    const i64 fx = tp.row_fx[i];
    float *af = tile_fragment_bytes(pl, tp.row_mt[i]) ? (float *)((char *)frag + tp.row_frag_off[i]) : nullptr;
    hipError_t e = launch_tile_gemm(pl, tp.row_lds[i], tp.row_mt[i], tp.row_nt[i],
                                    (const float *)((const char *)weight + fx * pl.f_pitch * elem_bytes),
                                    (const float *)grad_out, nullptr, (float *)ws + fx * pl.ngx * pl.noy, stream, af);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

bool plan_two_pass_input(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx,
                         i64 ngy, i64 nhx, i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px,
                         i64 py, i64 ux, i64 uy, TwoPassInput &tp, bool half = false) {
  const i64 m2 = c_in * nfx;
  // worth it when c_in alone would leave most of a 32-row tile empty and the
  // (c_in, filter row) pairs fill tiles reasonably
  // ... or when the x axis is Mellin and the layer keeps fewer rows than it is given
  // (nhx well below ngx, as whenever r does not stretch the output): the first pass here
  // works on the nhx rows of grad_out, the gather form on the ngx rows of grad_input,
  // most of whose (position, filter row) pairs have no tap at all
  const bool mellin_wide = kind_x == AX_MCORR && c_in >= 16 && 8 * nhx <= 7 * ngx;
  // ... or when p > 0 and the first pass can run as a launch per filter row
  // (plan_first_pass_rows: no product without a tap, where the gather form multiplies a
  // virtual row of zeros for each), given enough products per word of Y to pay for writing
  // and reading it: c_out * nfy from 256 on (measured on the 10-layer stack: 644 -> 594 us at
  // 256, 1157 -> 795 at 512, 3479 -> 1442 at 1024; 370 -> 451 at 128), in half precision,
  // where the gather form is three times faster and Y is still fp32, from 512 on
  // (with all filter rows in one launch: 453 -> 373 us at 512, 900 -> 549 at 1024;
  // 291 -> 347 at 256)
  const bool mellin_rows = kind_x == AX_MCORR && c_in >= 16 && px >= 1 && c_out * nfy >= (half ? 512 : 256);
  if ((c_in >= 16 && !mellin_wide && !mellin_rows) || nfx < 2) return false;
  if ((double)batch * m2 * nhx * ngy * 4.0 > (double)kMaxWorkspaceBytes) return false;
  const i64 pad = ((m2 + 31) / 32) * 32;
  if (pad * 2 > m2 * 3) return false;
  const i64 nf = nfx * nfy, nh = nhx * nhy;
  SepConv pr;
  pr.x = make_axis(AX_LCORR, 1, nhx, nhx, 1, 1, 0, 1);                 // rows pass through
  pr.y = make_axis(AX_LCONV, nfy, nhy, ngy, uy, dy, py, sy);
  pr.batch = batch; pr.c_out = m2; pr.c_in = c_out;
  pr.f_m = nfy; pr.f_c = c_in * nf;
  pr.g_n = c_out * nh; pr.g_c = nh;
  pr.h_n = m2 * nhx * ngy; pr.h_m = nhx * ngy;
  pr.accumulate = 0;
  pr.math = g_math;
  pr.in_half = half;                                   // weight and grad_out as half-precision tensors, Y in fp32
  if (!make_tile_plan(pr, tp.plan, &tp.lds, &tp.mt, &tp.nt)) return false;
  const int conv_x = kind_x == AX_MCORR ? AX_MCONV : AX_LCONV;
  tp.fold = make_axis(conv_x, nfx, nhx, ngx, ux, dx, px, sx);
  tp.ws_bytes = (size_t)(batch * m2 * nhx * ngy) * sizeof(float);
  tp.frag_bytes = tile_fragment_bytes(tp.plan, tp.mt);
  tp.frag_off = (tp.ws_bytes + 255) & ~(size_t)255;
  if (kind_x == AX_MCORR) plan_first_pass_rows(pr, c_in, nfx, nfy, nhx, ngx, ngy, sx, dx, px, ux, tp);
  if (c_in >= 16 && !mellin_wide && tp.rows == 0) return false;
  if (tp.frag_bytes) tp.ws_bytes = tp.frag_off + tp.frag_bytes;
  return true;
}

// Which form the fp32 input gradient takes, for the query and the call alike.  The three
// specialised forms keep intermediate values in a workspace whose size grows with the
// layer (partial rows, tap products, first-pass rows); a form whose workspace would pass
// kMaxWorkspaceBytes is not taken, and the gather form (tiled or one thread per output),
// which needs none, is the last resort.
enum InputForm { IN_GATHER = 0, IN_FUSED, IN_TAPS, IN_TWO_PASS };

// The gather form: the convolution with the roles of signal and output exchanged,
// "signal" = grad_out (length nh), "output" = grad_input (length ng), weight read transposed.
SepConv input_gather_problem(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx, i64 ngy,
                             i64 nhx, i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy) {
  const i64 nf = nfx * nfy, ng = ngx * ngy, nh = nhx * nhy;
  const int conv_x = kind_x == AX_MCORR ? AX_MCONV : AX_LCONV;
  SepConv pr;
  pr.x = make_axis(conv_x, nfx, nhx, ngx, ux, dx, px, sx);
  pr.y = make_axis(AX_LCONV, nfy, nhy, ngy, uy, dy, py, sy);
  if (c_out * nf * nh == 0) pr.x.nh_eff = 0;
  pr.batch = batch; pr.c_out = c_in; pr.c_in = c_out;
  pr.f_m = nf; pr.f_c = c_in * nf;
  pr.g_n = c_out * nh; pr.g_c = nh;
  pr.h_n = c_in * ng; pr.h_m = ng;
  pr.accumulate = 0;
  pr.math = g_math;
  return pr;
}
struct InputPlans {
  IgradPlan fused;
  TapProductPlan taps;
  TwoPassInput two;
  size_t ws_bytes = 0;
};

int choose_input_plan(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx,
                      i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, InputPlans &ips) {
  const int forced = g_forced;
  ips.ws_bytes = 0;
  if (forced == 1) return IN_GATHER;
  if (forced == 0 && make_igrad_plan(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy,
                                     px, py, ux, uy, ips.fused, 0, 0, -1, g_math) &&
      ips.fused.ws_bytes <= kMaxWorkspaceBytes) {
    ips.ws_bytes = ips.fused.ws_bytes;
    return IN_FUSED;
  }
  if (forced == 0 && make_tap_product_plan(batch, c_in, c_out, nfx, nfy, nhx, nhy, ips.taps) &&
      ips.taps.ws_bytes <= kMaxWorkspaceBytes) {
    if (!g_no_yfold) enable_tap_yfold(ips.taps, nfx, nfy, nhx, nhy, ngy, sy, dy, py, uy);
    ips.ws_bytes = ips.taps.ws_bytes;
    return IN_TAPS;
  }
  if (plan_two_pass_input(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux, uy,
                          ips.two) && ips.two.ws_bytes <= kMaxWorkspaceBytes) {
    ips.ws_bytes = ips.two.ws_bytes;
    return IN_TWO_PASS;
  }
  // (optional for the gather form: without it the kernel splits the filter itself)
  ips.ws_bytes = fragment_bytes(input_gather_problem(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy,
                                                     sx, sy, dx, dy, px, py, ux, uy));
  return IN_GATHER;
}

template <typename T>
int corr2d_backward_input(const char *fn, int kind_x, const T *weight,
                          const T *grad_out, i64 batch, i64 c_in, i64 c_out,
                          i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy,
                          i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux,
                          i64 uy, T *grad_input, void *workspace, size_t workspace_bytes,
                          void *stream, void *half_out = nullptr, bool *wrote_half = nullptr) {
  if (wrote_half) *wrote_half = false;
  int rc = check_corr2d(fn, kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx,
                        nhy, sx, sy, dx, dy, px, py, ux, uy);
  if (rc) return rc;
  const i64 nf = nfx * nfy, ng = ngx * ngy, nh = nhx * nhy;
  if (batch * c_in * ng == 0) return MELLIN_OK;
  if (!grad_input || (c_out * nf * nh != 0 && (!weight || !grad_out)))
    return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  const int conv_x = kind_x == AX_MCORR ? AX_MCONV : AX_LCONV;
  if (sizeof(T) == 4 && c_out * nf * nh != 0) {
    InputPlans ips;
    const int which = choose_input_plan(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy,
                                        px, py, ux, uy, ips);
    if (which != IN_GATHER && ips.ws_bytes && (!workspace || workspace_bytes < ips.ws_bytes))
      return fail(MELLIN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn, ips.ws_bytes,
                  workspace_bytes);
    if (which == IN_FUSED) {
      g_variant = "mfma-fused";
      g_last_math = ips.fused.stream ? MATH_BF16X3 : MATH_FP32;
      return check_hip(launch_igrad(ips.fused, (const float *)weight, (const float *)grad_out,
                                    (float *)grad_input, (float *)workspace, (hipStream_t)stream), fn);
    }
    if (which == IN_TAPS) {
      // tap products through the workspace, then a gather (any x axis kind)
      g_variant = "mfma-taps+fold";
      g_last_math = MATH_FP32;
      hipError_t e = launch_tap_product(ips.taps, (const float *)weight, (const float *)grad_out,
                                        (float *)workspace, (hipStream_t)stream);
      if (e == hipSuccess) {
        const Axis fx = make_axis(conv_x, nfx, nhx, ngx, ux, dx, px, sx);
        const Axis fy = make_axis(AX_LCONV, nfy, nhy, ngy, uy, dy, py, sy);
        if (ips.taps.yfold)                                  // (the kernel has summed the filter columns)
          e = launch_fold_x(fx, batch * c_in, ngx, ngy, (const float *)workspace, grad_input, (hipStream_t)stream);
        else
          e = launch_fold_xy(fx, fy, batch * c_in, ips.taps.nf_pad, (const float *)workspace,
                             (float *)grad_input, (hipStream_t)stream);
      }
      return check_hip(e, fn);
    }
    if (which == IN_TWO_PASS) {
      const TwoPassInput &tp = ips.two;
      g_variant = tp.rows ? "mfma-filter-rows+fold" : "mfma+fold";
      g_last_math = tp.rows || tp.plan.split ? MATH_BF16X3 : MATH_FP32;
      hipError_t e = launch_first_pass(tp, weight, grad_out, workspace, 4, (hipStream_t)stream);
      if (e == hipSuccess)
        e = launch_fold_x(tp.fold, batch * c_in, ngx, ngy, (const float *)workspace,
                          (float *)grad_input, (hipStream_t)stream);
      return check_hip(e, fn);
    }
  }
  SepConv pr = input_gather_problem(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy,
                                    px, py, ux, uy);
  if (half_out && sizeof(T) == 4 && g_forced != 1) {
    // as in the forward pass: the matrix-core kernel stores half precision itself
    TilePlan pl;
    size_t lds = 0;
    int mt = 0, nt = 0;
    pr.out_half = 1;
    if (make_tile_plan(pr, pl, &lds, &mt, &nt)) {
      g_variant = "mfma";
      g_last_math = pl.split ? MATH_BF16X3 : MATH_FP32;
      if (wrote_half) *wrote_half = true;
      return check_hip(launch_tile_gemm(pl, lds, mt, nt, (const float *)weight, (const float *)grad_out, nullptr,
                                        (float *)half_out, (hipStream_t)stream), fn);
    }
    pr.out_half = 0;
  }
  return check_hip(run_sepconv<T>(pr, weight, grad_out, (const T *)nullptr, grad_input,
                                  (hipStream_t)stream, workspace, workspace_bytes), fn);
}

// The fp32 weight gradient through the kernel whose matrix instructions run along the
// output positions (bf16 matrix cores), where the variant and math mode in force allow it
// and it is the faster one: layers with at least 16 input channels and more than 32 output
// channels (its workgroups own 64 channels or more; measured 1.2-2.8 times faster there
// than the row-wise and tiled fp32 kernels, slower on narrower layers).
bool plan_weight_positions(const SepConv &fwd, WgradPosPlan &pp) {
  if (g_forced != 0 || g_math == MATH_FP32 || fwd.c_in < 16 || fwd.c_out <= 32) return false;
  return make_wgrad_pos_plan(fwd, pp, false) && pp.ws_bytes <= kMaxWorkspaceBytes;
}

template <typename T>
int corr2d_backward_weight(const char *fn, int kind_x, const T *input,
                           const T *grad_out, i64 batch, i64 c_in, i64 c_out,
                           i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx, i64 nhy,
                           i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux,
                           i64 uy, T *grad_weight, void *workspace,
                           size_t workspace_bytes, void *stream) {
  int rc = check_corr2d(fn, kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx,
                        nhy, sx, sy, dx, dy, px, py, ux, uy);
  if (rc) return rc;
  const i64 nf = nfx * nfy, ng = ngx * ngy, nh = nhx * nhy;
  if (c_out * c_in * nf == 0) return MELLIN_OK;
  if (!grad_weight || (batch * ng * nh != 0 && (!input || !grad_out)))
    return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  if (sizeof(T) == 4 && batch * ng * nh != 0) {
    WgradPosPlan pp;
    if (plan_weight_positions(forward_problem(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy,
                                              sx, sy, dx, dy, px, py, ux, uy), pp)) {
      if (!workspace || workspace_bytes < pp.ws_bytes)
        return fail(MELLIN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn,
                    pp.ws_bytes, workspace_bytes);
      g_variant = "mfma-positions";
      g_last_math = MATH_BF16X3;
      return check_hip(launch_wgrad_pos(pp, grad_out, input, grad_weight, (float *)workspace, (hipStream_t)stream), fn);
    }
  }
  if (sizeof(T) == 4 && g_forced != 1 && batch * ng * nh != 0) {
    WgradPlan wp;
    if (make_wgrad_plan(forward_problem(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy,
                                        sx, sy, dx, dy, px, py, ux, uy), wp, g_forced != 2)) {
      if (!workspace || workspace_bytes < wp.ws_bytes)
        return fail(MELLIN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn,
                    wp.ws_bytes, workspace_bytes);
      g_variant = wp.rows_mode ? "mfma-rows" : "mfma";
      g_last_math = wp.rows_mode == 2 ? MATH_BF16X3 : MATH_FP32;
      return check_hip(launch_wgrad(wp, (const float *)grad_out, (const float *)input,
                                    (float *)grad_weight, (float *)workspace,
                                    (hipStream_t)stream), fn);
    }
  }
  SepReduce pr;
  pr.x = make_axis(kind_x, nfx, ngx, nhx, sx, dx, px, ux);
  pr.y = make_axis(AX_LCORR, nfy, ngy, nhy, sy, dy, py, uy);
  if (batch * ng * nh == 0) pr.x.nh_eff = 0;
  pr.batch = batch; pr.c_out = c_out; pr.c_in = c_in;
  g_variant = "generic";
  g_last_math = MATH_FP32;
  return check_hip(launch_sepreduce_generic<T>(pr, grad_out, input, grad_weight,
                                               (hipStream_t)stream), fn);
}

// Address of the static scratch array on the current device (nullptr after fail()).  The
// lookup runs once per device, on the first call made with that device current; it
// allocates nothing (the array is part of the loaded code object).
const int kMaxDevices = 64;
void *g_scratch_addr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// stream: the stream the caller is about to launch on, or null when only the lookup is asked
// for; a lookup that has not been made yet is refused while that stream is capturing a graph
// (it loads the code object, which a capture does not allow)
void *static_scratch(const char *fn, hipStream_t stream = nullptr, bool check_capture = false) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { fail(MELLIN_ERR_RUNTIME, "%s: hipGetDevice: %s", fn, hipGetErrorString(e)); return nullptr; }
  if (dev < 0 || dev >= kMaxDevices) { fail(MELLIN_ERR_RUNTIME, "%s: device index %d out of range", fn, dev); return nullptr; }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_addr[dev]) {
    if (check_capture) {
      hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
      if (hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone) {
        fail(MELLIN_ERR_RUNTIME, "%s: the static scratch array of this device has not been looked up yet and the "
             "stream is capturing a graph; call mellin_static_scratch_prepare() before the capture begins", fn);
        return nullptr;
      }
      (void)hipGetLastError();
    }
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      fail(MELLIN_ERR_RUNTIME, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_addr[dev] = ptr;
  }
  return g_scratch_addr[dev];
}

// Column ops (mconv.h:1247-1380): x Mellin correlation, y linear correlation.
template <typename T>
int col_op(const char *fn, bool to_col, const T *src, i64 c_in, i64 batch, i64 nfx, i64 nfy,
           i64 ngx, i64 ngy, i64 nggx, i64 nggy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py,
           i64 ux, i64 uy, int transposed_g, int transposed_gg, T *dst, void *stream) {
  int rc = check_channels(fn, 0, c_in, batch);
  if (!rc) rc = check_axis(fn, "x", AX_MCORR, nfx, ngx, nggx, sx, dx, px, ux);
  if (!rc) rc = check_axis(fn, "y", AX_LCORR, nfy, ngy, nggy, sy, dy, py, uy);
  if (!rc) rc = check_counts(fn, (double)batch * c_in * ngx * ngy,
                             (double)batch * c_in * nfx * nfy * nggx * nggy, 0.0);
  if (rc) return rc;
  const i64 n_g = batch * c_in * ngx * ngy, n_gg = batch * c_in * nfx * nfy * nggx * nggy;
  if ((to_col ? n_gg : n_g) == 0) return MELLIN_OK;
  if (!dst || ((to_col ? n_g : n_gg) != 0 && !src))
    return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  hipError_t e;
  if (to_col) {
    const Axis x = make_axis(AX_MCORR, nfx, ngx, nggx, sx, dx, px, ux);
    const Axis y = make_axis(AX_LCORR, nfy, ngy, nggy, sy, dy, py, uy);
    e = launch_spec2col<T>(x, y, c_in, batch, transposed_g, transposed_gg, src, dst, (hipStream_t)stream);
  } else {
    // inverse relations: the convolution kinds with s and u exchanged (mconv.h:1294-1298, :1362-1372)
    const Axis x = make_axis(AX_MCONV, nfx, nggx, ngx, ux, dx, px, sx);
    const Axis y = make_axis(AX_LCONV, nfy, nggy, ngy, uy, dy, py, sy);
    e = launch_col2spec<T>(x, y, c_in, batch, transposed_g, transposed_gg, src, dst, (hipStream_t)stream);
  }
  return check_hip(e, fn);
}

}  // namespace

#define DEFINE_SND(NAME, T, SRC, DST, TO_COL)                                   \
  MELLIN_DECL_SND(NAME, T, SRC, DST) {                                          \
    return col_op<T>(#NAME, TO_COL, SRC, c_in, batch, nf, 1, ng, 1, ngg, 1, s,  \
                     1, d, 1, p, 0, u, 1, transposed_g, transposed_gg, DST,    \
                     stream);                                                  \
  }
#define DEFINE_SPEC(NAME, T, SRC, DST, TO_COL)                                  \
  MELLIN_DECL_SPEC(NAME, T, SRC, DST) {                                         \
    return col_op<T>(#NAME, TO_COL, SRC, c_in, batch, nfx, nfy, ngx, ngy, nggx, \
                     nggy, sx, sy, dx, dy, px, py, ux, uy, transposed_g,       \
                     transposed_gg, DST, stream);                              \
  }
DEFINE_SND(mellin_snd2col_f32, float, g, gg, true)
DEFINE_SND(mellin_snd2col_f64, double, g, gg, true)
DEFINE_SND(mellin_col2snd_f32, float, gg, g, false)
DEFINE_SND(mellin_col2snd_f64, double, gg, g, false)
DEFINE_SPEC(mellin_spec2col_f32, float, g, gg, true)
DEFINE_SPEC(mellin_spec2col_f64, double, g, gg, true)
DEFINE_SPEC(mellin_col2spec_f32, float, gg, g, false)
DEFINE_SPEC(mellin_col2spec_f64, double, gg, g, false)

// ---- section 4: pointwise layers ----------------------------------------------
int check_log_lift(const char *fn, double eps, int flags, i64 outer, i64 t, i64 inner) {
  if (!(flags & (MELLIN_PW_LOG | MELLIN_PW_LIFT)) || (flags & ~(MELLIN_PW_LOG | MELLIN_PW_LIFT)))
    return fail(MELLIN_ERR_ARGUMENT, "%s: flags must be MELLIN_PW_LOG, MELLIN_PW_LIFT or both (got %d)", fn, flags);
  if (outer < 0 || t < 0 || inner < 0)
    return fail(MELLIN_ERR_ARGUMENT, "%s: negative size (outer=%lld t=%lld inner=%lld)", fn, (long long)outer,
                (long long)t, (long long)inner);
  if ((flags & MELLIN_PW_LOG) && !(eps > 0))
    return fail(MELLIN_ERR_ARGUMENT, "%s: eps must be positive (got %g)", fn, eps);
  if (t * inner >= ((i64)1 << 40) || outer >= ((i64)1 << 40))
    return fail(MELLIN_ERR_ARGUMENT, "%s: sizes beyond the supported range", fn);
  return MELLIN_OK;
}

template <typename T>
int log_lift_forward(const char *fn, const T *x, double eps, double tau, int flags, i64 outer, i64 t, i64 inner,
                     T *y, void *stream, const T *params = nullptr) {
  int rc;
  if ((rc = check_log_lift(fn, eps, flags, outer, t, inner))) return rc;
  if (outer * t * inner == 0) return MELLIN_OK;
  if (!x || !y) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  hipError_t e = launch_log_lift_forward<T>(x, (T)eps, (T)tau, flags & MELLIN_PW_LOG, flags & MELLIN_PW_LIFT,
                                            outer, t, inner, y, (hipStream_t)stream, params);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", fn, hipGetErrorString(e));
  return MELLIN_OK;
}

template <typename T>
int log_lift_backward(const char *fn, const T *x, const T *gy, double eps, double tau, int flags, i64 outer,
                      i64 t, i64 inner, T *gx, T *grad_params, void *workspace, size_t workspace_bytes,
                      void *stream, const T *params = nullptr) {
  int rc;
  if ((rc = check_log_lift(fn, eps, flags, outer, t, inner))) return rc;
  if (!grad_params) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  const size_t need = log_lift_workspace_bytes(outer, t, inner, sizeof(T));
  if (need && (!x || !gy || !gx)) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  if (need && (!workspace || workspace_bytes < need))
    return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", fn, need, workspace_bytes);
  hipError_t e = launch_log_lift_backward<T>(x, gy, (T)eps, (T)tau, flags & MELLIN_PW_LOG, flags & MELLIN_PW_LIFT,
                                             outer, t, inner, gx, grad_params, (T *)workspace,
                                             (hipStream_t)stream, params);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", fn, hipGetErrorString(e));
  return MELLIN_OK;
}

#define CORR2D_ARGS                                                            \
  batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py,    \
  ux, uy

// ---- half-precision entry points: half tensors, fp32 accumulation -----------------
// Where the tiled matrix-core kernel applies (the forward pass; the input gradient of
// layers with many input channels) it reads the half-precision tensors as they lie,
// multiplies on the f16 matrix cores (products of half-precision values are exact in
// fp32, sums are kept in fp32) and stores half precision: no copies, and the workspace
// holds at most the filter's fragments.
// Otherwise each operand is copied to fp32 in the workspace and the fp32 kernels run
// there; they write fp32 into the workspace and the result is copied back to half.
// Regions are 256-byte aligned.
size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

struct HalfNative {
  TilePlan pl;
  size_t lds, frag_bytes;
  int mt, nt;
  bool classes;                    // one launch per residue class of a Mellin axis instead (cls)
  ClassPlans cls;
};

// The tiled kernel's plan for `pr` with half-precision operands and results, if it has one
// and the variant in force allows it.
bool plan_half_native(SepConv pr, HalfNative &hn) {
  if (g_forced == 1 || g_widen) return false;
  pr.in_half = 1;
  pr.out_half = 1;
  hn.classes = plan_mellin_classes(pr, hn.cls);
  if (hn.classes) {
    hn.frag_bytes = hn.cls.frag_bytes;
    return true;
  }
  if (!make_tile_plan(pr, hn.pl, &hn.lds, &hn.mt, &hn.nt)) return false;
  hn.frag_bytes = tile_fragment_bytes(hn.pl, hn.mt);
  return true;
}

int run_half_native(const char *fn, const HalfNative &hn, const void *f, const void *g, const void *bias, void *h,
                    void *workspace, size_t workspace_bytes, void *stream) {
  if (hn.frag_bytes && (!workspace || workspace_bytes < hn.frag_bytes))
    return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", fn, hn.frag_bytes, workspace_bytes);
  if (hn.frag_bytes && ((uintptr_t)workspace & 15))
    return fail(MELLIN_ERR_ARGUMENT, "%s: the workspace must be 16-byte aligned", fn);
  if (!f || !g || !h) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  g_last_math = MELLIN_MATH_F16;
  if (hn.classes) {
    bool one_launch = false;
    const hipError_t e = launch_mellin_classes(hn.cls, f, g, bias, h, (hipStream_t)stream, workspace, workspace_bytes,
                                               &one_launch);
    g_variant = one_launch ? "mfma-f16-classes" : "mfma-f16-class-launches";
    return check_hip(e, fn);
  }
  g_variant = "mfma-f16";
  return check_hip(launch_tile_gemm(hn.pl, hn.lds, hn.mt, hn.nt, (const float *)f, (const float *)g,
                                    (const float *)bias, (float *)h, (hipStream_t)stream,
                                    hn.frag_bytes ? (float *)workspace : nullptr), fn);
}

// The weight gradient on the f16 matrix cores, if the variant in force allows it and the
// kernel applies (n_in, n_out: elements of input and grad_out; nothing to sum: no).
bool plan_half_weight(const SepConv &fwd, i64 n_in, i64 n_out, WgradPosPlan &hp) {
  if (g_forced == 1 || g_widen || n_in == 0 || n_out == 0) return false;
  return make_wgrad_pos_plan(fwd, hp, true) && hp.ws_bytes <= kMaxWorkspaceBytes;
}

// The two-pass input gradient (layers with few input channels) on half-precision tensors,
// if the variant in force allows it and the form applies.
bool plan_half_two_pass(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx,
                        i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, TwoPassInput &tp) {
  if (g_forced == 1 || g_widen || c_out * nfx * nfy * nhx * nhy == 0) return false;
  return plan_two_pass_input(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux, uy,
                             tp, true) &&
         tp.ws_bytes + (size_t)(batch * c_in * ngx * ngy) * 4 <= kMaxWorkspaceBytes;
}

// The one-kernel input gradient of layers with at most three input channels and a linear x
// axis on half-precision tensors, if the variant in force allows it and the form applies.
bool plan_half_fused(int kind_x, i64 batch, i64 c_in, i64 c_out, i64 nfx, i64 nfy, i64 ngx, i64 ngy, i64 nhx,
                     i64 nhy, i64 sx, i64 sy, i64 dx, i64 dy, i64 px, i64 py, i64 ux, i64 uy, IgradPlan &ip) {
  if (g_forced != 0 || g_widen || c_out * nfx * nfy * nhx * nhy == 0) return false;
  return make_igrad_plan(kind_x, batch, c_in, c_out, nfx, nfy, ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux, uy,
                         ip, 0, 0, -1, MATH_BF16X3) &&
         ip.stream && ip.ws_bytes <= kMaxWorkspaceBytes;
}

// Input gradients of layers with fewer input channels than this leave most of a 32-row
// matrix tile empty in the gather form: they keep the fp32 kernels made for them.
constexpr i64 kHalfGatherMinChannels = 16;

struct HalfLayout {
  size_t in_off, w_off, b_off, out_off, inner_off, total;   // byte offsets of the fp32 copies
};

// a, b: element counts of the two operands; bias: of the bias (forward only); r: of the result
HalfLayout half_layout(i64 a, i64 b, i64 bias, i64 r, size_t inner) {
  HalfLayout l;
  l.in_off = 0;
  l.w_off = l.in_off + align256((size_t)a * 4);
  l.b_off = l.w_off + align256((size_t)b * 4);
  l.out_off = l.b_off + align256((size_t)bias * 4);
  l.inner_off = l.out_off + align256((size_t)r * 4);
  l.total = l.inner_off + align256(inner);
  return l;
}

#define CORR2D_COUNTS                                                              \
  const i64 n_in = batch * c_in * ngx * ngy, n_w = c_out * c_in * nfx * nfy,      \
            n_out = batch * c_out * nhx * nhy

template <typename T>
int bias_grad_entry(const char *fn, const T *grad_out, const T *out, int64_t batch, int64_t channels, int64_t plane,
                    T *grad_masked, T *grad_bias, void *workspace, size_t workspace_bytes, void *stream) {
  if (batch < 0 || channels < 0 || plane < 0)
    return fail(MELLIN_ERR_ARGUMENT, "%s: negative extent", fn);
  if (batch > 65535 || channels > 65535 || plane > ((int64_t)1 << 40))
    return fail(MELLIN_ERR_ARGUMENT, "%s: at most 65535 images and channels (got %lld, %lld)", fn, (long long)batch,
                (long long)channels);
  if (channels == 0) return MELLIN_OK;
  if (!grad_bias) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  const size_t need = bias_grad_workspace_bytes(batch, channels, plane);
  if (need && (!grad_out || (out && !grad_masked))) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  if (need && (!workspace || workspace_bytes < need))
    return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", fn, need, workspace_bytes);
  hipError_t e = launch_bias_grad(grad_out, out, batch, channels, plane, grad_masked, grad_bias, (float *)workspace,
                                  (hipStream_t)stream);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", fn, hipGetErrorString(e));
  return MELLIN_OK;
}

template <typename T>
int pool_pairs_forward_entry(const char *fn, const T *x, int64_t rows, int64_t f, T *y, unsigned char *which,
                             void *stream) {
  if (rows < 0 || f < 0 || rows > ((int64_t)1 << 40) || f > ((int64_t)1 << 30) || rows * f > ((int64_t)1 << 44))
    return fail(MELLIN_ERR_ARGUMENT, "%s: extents out of range (%lld rows of %lld)", fn, (long long)rows, (long long)f);
  if (rows * (f / 2) == 0) return MELLIN_OK;
  if (!x || !y || !which) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  hipError_t e = launch_pool_pairs_forward(x, rows, f, y, which, (hipStream_t)stream);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", fn, hipGetErrorString(e));
  return MELLIN_OK;
}
template <typename T>
int pool_pairs_backward_entry(const char *fn, const T *grad_y, const unsigned char *which, int64_t rows, int64_t f,
                              T *grad_x, void *stream) {
  if (rows < 0 || f < 0 || rows > ((int64_t)1 << 40) || f > ((int64_t)1 << 30) || rows * f > ((int64_t)1 << 44))
    return fail(MELLIN_ERR_ARGUMENT, "%s: extents out of range (%lld rows of %lld)", fn, (long long)rows, (long long)f);
  if (rows * f == 0) return MELLIN_OK;
  if (!grad_x || (f / 2 && (!grad_y || !which))) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", fn);
  hipError_t e = launch_pool_pairs_backward(grad_y, which, rows, f, grad_x, (hipStream_t)stream);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", fn, hipGetErrorString(e));
  return MELLIN_OK;
}

extern "C" {

int mellin_version(void) { return 100; }

const char *mellin_last_error(void) { return g_error; }

const char *mellin_last_variant(void) { return g_variant; }

int mellin_corr2d_forward_act_f32(int kind_x, int activation, const float *input, const float *weight,
                                  const float *bias, MELLIN_CORR2D_DIMS, float *out, void *stream) {
  return corr2d_forward<float>(__func__, kind_x, input, weight, bias, CORR2D_ARGS, out, stream, activation);
}
int mellin_corr2d_forward_act_f64(int kind_x, int activation, const double *input, const double *weight,
                                  const double *bias, MELLIN_CORR2D_DIMS, double *out, void *stream) {
  return corr2d_forward<double>(__func__, kind_x, input, weight, bias, CORR2D_ARGS, out, stream, activation);
}
size_t mellin_corr2d_forward_f16_workspace(int kind_x, MELLIN_CORR2D_DIMS) {
  if (check_corr2d(__func__, kind_x, CORR2D_ARGS)) return 0;
  CORR2D_COUNTS;
  HalfNative hn;
  if (plan_half_native(forward_problem(kind_x, CORR2D_ARGS), hn)) return hn.frag_bytes;
  return half_layout(n_in, n_w, c_out, n_out, 0).total;
}
int mellin_corr2d_forward_f16(int kind_x, const void *input, const void *weight, const void *bias,
                              MELLIN_CORR2D_DIMS, void *out, void *workspace, size_t workspace_bytes,
                              void *stream) {
  return mellin_corr2d_forward_act_f16(kind_x, MELLIN_ACT_NONE, input, weight, bias, CORR2D_ARGS, out, workspace,
                                       workspace_bytes, stream);
}
int mellin_corr2d_forward_act_f16(int kind_x, int activation, const void *input, const void *weight,
                                  const void *bias, MELLIN_CORR2D_DIMS, void *out, void *workspace,
                                  size_t workspace_bytes, void *stream) {
  int rc;
  if ((rc = check_corr2d(__func__, kind_x, CORR2D_ARGS))) return rc;
  if (activation != MELLIN_ACT_NONE && activation != MELLIN_ACT_RELU)
    return fail(MELLIN_ERR_ARGUMENT, "%s: activation must be MELLIN_ACT_NONE or MELLIN_ACT_RELU (got %d)", __func__,
                activation);
  CORR2D_COUNTS;
  if (n_out == 0) return MELLIN_OK;
  {
    SepConv pr = forward_problem(kind_x, CORR2D_ARGS);
    pr.relu = activation == MELLIN_ACT_RELU;
    HalfNative hn;
    if (plan_half_native(pr, hn))
      return run_half_native(__func__, hn, weight, input, bias, out, workspace, workspace_bytes, stream);
  }
  const HalfLayout l = half_layout(n_in, n_w, c_out, n_out, 0);
  if (!workspace || workspace_bytes < l.total)
    return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", __func__, l.total, workspace_bytes);
  if (!out || (n_in && !input) || (n_w && !weight)) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
  char *ws = (char *)workspace;
  hipStream_t st = (hipStream_t)stream;
  hipError_t e = launch_half_to_float(input, (float *)(ws + l.in_off), n_in, st);
  if (e == hipSuccess) e = launch_half_to_float(weight, (float *)(ws + l.w_off), n_w, st);
  if (e == hipSuccess && bias) e = launch_half_to_float(bias, (float *)(ws + l.b_off), c_out, st);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", __func__, hipGetErrorString(e));
  bool wrote_half = false;
  rc = corr2d_forward<float>(__func__, kind_x, (const float *)(ws + l.in_off), (const float *)(ws + l.w_off),
                             bias ? (const float *)(ws + l.b_off) : nullptr, CORR2D_ARGS,
                             (float *)(ws + l.out_off), stream, activation, out, &wrote_half);
  if (rc) return rc;
  if (wrote_half) return MELLIN_OK;
  e = launch_float_to_half((const float *)(ws + l.out_off), out, n_out, st);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", __func__, hipGetErrorString(e));
  return MELLIN_OK;
}
size_t mellin_corr2d_backward_input_f16_workspace(int kind_x, MELLIN_CORR2D_DIMS) {
  if (check_corr2d(__func__, kind_x, CORR2D_ARGS)) return 0;
  CORR2D_COUNTS;
  HalfNative hn;
  IgradPlan ip;
  if (plan_half_fused(kind_x, CORR2D_ARGS, ip)) return ip.ws_bytes;
  // (the two-pass form where the fp32 path would take it: few input channels, or a Mellin
  // axis that keeps fewer rows than it is given)
  TwoPassInput tp;
  if (plan_half_two_pass(kind_x, CORR2D_ARGS, tp)) return tp.ws_bytes;
  if (c_in >= kHalfGatherMinChannels && plan_half_native(input_gather_problem(kind_x, CORR2D_ARGS), hn))
    return hn.frag_bytes;
  return half_layout(n_w, n_out, 0, n_in, mellin_corr2d_backward_input_workspace(kind_x, 4, CORR2D_ARGS)).total;
}
int mellin_corr2d_backward_input_f16(int kind_x, const void *weight, const void *grad_out, MELLIN_CORR2D_DIMS,
                                     void *grad_input, void *workspace, size_t workspace_bytes, void *stream) {
  int rc;
  if ((rc = check_corr2d(__func__, kind_x, CORR2D_ARGS))) return rc;
  CORR2D_COUNTS;
  if (n_in == 0) return MELLIN_OK;
  {
    IgradPlan ip;
    if (plan_half_fused(kind_x, CORR2D_ARGS, ip)) {
      if (ip.ws_bytes && (!workspace || workspace_bytes < ip.ws_bytes))
        return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", __func__, ip.ws_bytes,
                    workspace_bytes);
      if (!grad_input || !weight || !grad_out) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
      g_variant = "mfma-f16-fused";
      g_last_math = MELLIN_MATH_F16;
      return check_hip(launch_igrad_half(ip, weight, grad_out, grad_input, (float *)workspace, (hipStream_t)stream),
                       __func__);
    }
    HalfNative hn;
    TwoPassInput tp;
    const bool two_pass = plan_half_two_pass(kind_x, CORR2D_ARGS, tp);
    if (!two_pass && c_in >= kHalfGatherMinChannels && plan_half_native(input_gather_problem(kind_x, CORR2D_ARGS), hn))
      return run_half_native(__func__, hn, weight, grad_out, nullptr, grad_input, workspace, workspace_bytes, stream);
    if (two_pass) {
      // the two-pass form on the half-precision tensors: first-pass rows in fp32 in the
      // workspace, the fold sums them in fp32 and rounds once on the way out
      const size_t need = tp.ws_bytes;
      if (!workspace || workspace_bytes < need)
        return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", __func__, need, workspace_bytes);
      if (!grad_input || !weight || !grad_out) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
      char *ws = (char *)workspace;
      hipStream_t st = (hipStream_t)stream;
      g_variant = tp.rows ? "mfma-f16-filter-rows+fold" : "mfma-f16+fold";
      g_last_math = MELLIN_MATH_F16;
      hipError_t e = launch_first_pass(tp, weight, grad_out, ws, 2, st);
      if (e == hipSuccess) e = launch_fold_x(tp.fold, batch * c_in, ngx, ngy, (const float *)ws, grad_input, st, true);
      return check_hip(e, __func__);
    }
  }
  const size_t inner = mellin_corr2d_backward_input_workspace(kind_x, 4, CORR2D_ARGS);
  const HalfLayout l = half_layout(n_w, n_out, 0, n_in, inner);
  if (!workspace || workspace_bytes < l.total)
    return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", __func__, l.total, workspace_bytes);
  if (!grad_input || (n_w && !weight) || (n_out && !grad_out)) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
  char *ws = (char *)workspace;
  hipStream_t st = (hipStream_t)stream;
  hipError_t e = launch_half_to_float(weight, (float *)(ws + l.in_off), n_w, st);
  if (e == hipSuccess) e = launch_half_to_float(grad_out, (float *)(ws + l.w_off), n_out, st);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", __func__, hipGetErrorString(e));
  bool wrote_half = false;
  rc = corr2d_backward_input<float>(__func__, kind_x, (const float *)(ws + l.in_off), (const float *)(ws + l.w_off),
                                    CORR2D_ARGS, (float *)(ws + l.out_off), ws + l.inner_off, inner, stream,
                                    grad_input, &wrote_half);
  if (rc) return rc;
  if (wrote_half) return MELLIN_OK;
  e = launch_float_to_half((const float *)(ws + l.out_off), grad_input, n_in, st);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", __func__, hipGetErrorString(e));
  return MELLIN_OK;
}
size_t mellin_corr2d_backward_weight_f16_workspace(int kind_x, MELLIN_CORR2D_DIMS) {
  if (check_corr2d(__func__, kind_x, CORR2D_ARGS)) return 0;
  CORR2D_COUNTS;
  WgradPosPlan hp;
  if (plan_half_weight(forward_problem(kind_x, CORR2D_ARGS), n_in, n_out, hp)) return hp.ws_bytes;
  return half_layout(n_in, n_out, 0, n_w, mellin_corr2d_backward_weight_workspace(kind_x, 4, CORR2D_ARGS)).total;
}
int mellin_corr2d_backward_weight_f16(int kind_x, const void *input, const void *grad_out, MELLIN_CORR2D_DIMS,
                                      void *grad_weight, void *workspace, size_t workspace_bytes, void *stream) {
  int rc;
  if ((rc = check_corr2d(__func__, kind_x, CORR2D_ARGS))) return rc;
  CORR2D_COUNTS;
  if (n_w == 0) return MELLIN_OK;
  {
    WgradPosPlan hp;
    if (plan_half_weight(forward_problem(kind_x, CORR2D_ARGS), n_in, n_out, hp)) {
      if (!workspace || workspace_bytes < hp.ws_bytes)
        return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", __func__, hp.ws_bytes,
                    workspace_bytes);
      if (!grad_weight || !input || !grad_out) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
      g_variant = "mfma-f16";
      g_last_math = MELLIN_MATH_F16;
      return check_hip(launch_wgrad_pos(hp, grad_out, input, grad_weight, (float *)workspace, (hipStream_t)stream),
                       __func__);
    }
  }
  const size_t inner = mellin_corr2d_backward_weight_workspace(kind_x, 4, CORR2D_ARGS);
  const HalfLayout l = half_layout(n_in, n_out, 0, n_w, inner);
  if (!workspace || workspace_bytes < l.total)
    return fail(MELLIN_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", __func__, l.total, workspace_bytes);
  if (!grad_weight || (n_in && !input) || (n_out && !grad_out)) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
  char *ws = (char *)workspace;
  hipStream_t st = (hipStream_t)stream;
  hipError_t e = launch_half_to_float(input, (float *)(ws + l.in_off), n_in, st);
  if (e == hipSuccess) e = launch_half_to_float(grad_out, (float *)(ws + l.w_off), n_out, st);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", __func__, hipGetErrorString(e));
  rc = corr2d_backward_weight<float>(__func__, kind_x, (const float *)(ws + l.in_off), (const float *)(ws + l.w_off),
                                     CORR2D_ARGS, (float *)(ws + l.out_off), ws + l.inner_off, inner, stream);
  if (rc) return rc;
  e = launch_float_to_half((const float *)(ws + l.out_off), grad_weight, n_w, st);
  if (e != hipSuccess) return fail(MELLIN_ERR_RUNTIME, "%s: %s", __func__, hipGetErrorString(e));
  return MELLIN_OK;
}

int mellin_log_lift_forward_f32(const float *x, double eps, double tau, int flags, int64_t outer, int64_t t,
                                int64_t inner, float *y, void *stream) {
  return log_lift_forward<float>("mellin_log_lift_forward_f32", x, eps, tau, flags, outer, t, inner, y, stream);
}
int mellin_log_lift_forward_f64(const double *x, double eps, double tau, int flags, int64_t outer, int64_t t,
                                int64_t inner, double *y, void *stream) {
  return log_lift_forward<double>("mellin_log_lift_forward_f64", x, eps, tau, flags, outer, t, inner, y, stream);
}
// eps and tau on the device: params = {eps, tau}
int mellin_log_lift_forward_dev_f32(const float *x, const float *params, int flags, int64_t outer, int64_t t,
                                    int64_t inner, float *y, void *stream) {
  if (!params) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
  return log_lift_forward<float>(__func__, x, 1.0, 0.0, flags, outer, t, inner, y, stream, params);
}
int mellin_log_lift_forward_dev_f64(const double *x, const double *params, int flags, int64_t outer, int64_t t,
                                    int64_t inner, double *y, void *stream) {
  if (!params) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
  return log_lift_forward<double>(__func__, x, 1.0, 0.0, flags, outer, t, inner, y, stream, params);
}
int mellin_log_lift_backward_dev_f32(const float *x, const float *grad_y, const float *params, int flags,
                                     int64_t outer, int64_t t, int64_t inner, float *grad_x, float *grad_params,
                                     void *workspace, size_t workspace_bytes, void *stream) {
  if (!params) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
  return log_lift_backward<float>(__func__, x, grad_y, 1.0, 0.0, flags, outer, t, inner, grad_x, grad_params,
                                  workspace, workspace_bytes, stream, params);
}
int mellin_log_lift_backward_dev_f64(const double *x, const double *grad_y, const double *params, int flags,
                                     int64_t outer, int64_t t, int64_t inner, double *grad_x, double *grad_params,
                                     void *workspace, size_t workspace_bytes, void *stream) {
  if (!params) return fail(MELLIN_ERR_ARGUMENT, "%s: null pointer", __func__);
  return log_lift_backward<double>(__func__, x, grad_y, 1.0, 0.0, flags, outer, t, inner, grad_x, grad_params,
                                   workspace, workspace_bytes, stream, params);
}
size_t mellin_log_lift_backward_workspace(int elem_bytes, int64_t outer, int64_t t, int64_t inner) {
  return log_lift_workspace_bytes(outer, t, inner, (size_t)elem_bytes);
}
int mellin_log_lift_backward_f32(const float *x, const float *grad_y, double eps, double tau, int flags,
                                 int64_t outer, int64_t t, int64_t inner, float *grad_x, float *grad_params,
                                 void *workspace, size_t workspace_bytes, void *stream) {
  return log_lift_backward<float>("mellin_log_lift_backward_f32", x, grad_y, eps, tau, flags, outer, t, inner,
                                  grad_x, grad_params, workspace, workspace_bytes, stream);
}
int mellin_log_lift_backward_f64(const double *x, const double *grad_y, double eps, double tau, int flags,
                                 int64_t outer, int64_t t, int64_t inner, double *grad_x, double *grad_params,
                                 void *workspace, size_t workspace_bytes, void *stream) {
  return log_lift_backward<double>("mellin_log_lift_backward_f64", x, grad_y, eps, tau, flags, outer, t, inner,
                                   grad_x, grad_params, workspace, workspace_bytes, stream);
}

size_t mellin_bias_grad_workspace(int64_t batch, int64_t channels, int64_t plane) {
  if (batch < 0 || channels < 0 || plane < 0 || batch > 65535 || channels > 65535 || plane > ((int64_t)1 << 40)) return 0;
  return bias_grad_workspace_bytes(batch, channels, plane);
}
int mellin_bias_grad_f32(const float *grad_out, const float *out, int64_t batch, int64_t channels, int64_t plane,
                         float *grad_masked, float *grad_bias, void *workspace, size_t workspace_bytes,
                         void *stream) {
  return bias_grad_entry<float>(__func__, grad_out, out, batch, channels, plane, grad_masked, grad_bias, workspace,
                                workspace_bytes, stream);
}
int mellin_bias_grad_f16(const void *grad_out, const void *out, int64_t batch, int64_t channels, int64_t plane,
                         void *grad_masked, void *grad_bias, void *workspace, size_t workspace_bytes,
                         void *stream) {
  return bias_grad_entry<_Float16>(__func__, (const _Float16 *)grad_out, (const _Float16 *)out, batch, channels, plane,
                                   (_Float16 *)grad_masked, (_Float16 *)grad_bias, workspace, workspace_bytes, stream);
}
int mellin_pool_pairs_forward_f32(const float *x, int64_t rows, int64_t f, float *y, unsigned char *which,
                                  void *stream) {
  return pool_pairs_forward_entry<float>(__func__, x, rows, f, y, which, stream);
}
int mellin_pool_pairs_forward_f16(const void *x, int64_t rows, int64_t f, void *y, unsigned char *which,
                                  void *stream) {
  return pool_pairs_forward_entry<_Float16>(__func__, (const _Float16 *)x, rows, f, (_Float16 *)y, which, stream);
}
int mellin_pool_pairs_backward_f32(const float *grad_y, const unsigned char *which, int64_t rows, int64_t f,
                                   float *grad_x, void *stream) {
  return pool_pairs_backward_entry<float>(__func__, grad_y, which, rows, f, grad_x, stream);
}
int mellin_pool_pairs_backward_f16(const void *grad_y, const unsigned char *which, int64_t rows, int64_t f,
                                   void *grad_x, void *stream) {
  return pool_pairs_backward_entry<_Float16>(__func__, (const _Float16 *)grad_y, which, rows, f, (_Float16 *)grad_x,
                                             stream);
}

int mellin_set_math(int mode) {
  if (mode != MELLIN_MATH_FP32 && mode != MELLIN_MATH_BF16X3 && mode != MELLIN_MATH_BF16X3_ALWAYS)
    return fail(MELLIN_ERR_ARGUMENT, "mellin_set_math: unknown mode %d", mode);
  g_math = mode;
  return MELLIN_OK;
}
int mellin_get_math(void) { return g_math; }
int mellin_last_math(void) { return g_last_math; }

int mellin_set_variant(const char *name) {
  // the name is parsed first: an unknown one changes nothing
  struct Setting { int forced, widen, no_classes, all_classes, split_classes, whole_classes, no_yfold, gather, no_narrow; };
  Setting v = {0, 0, 0, 0, 0, 0, 0, 0, 0};
  if (!name || !*name || !strcmp(name, "auto")) {}
  else if (!strcmp(name, "generic")) v.forced = 1;
  else if (!strcmp(name, "two-pass")) v.forced = 2;
  else if (!strcmp(name, "widen")) v.widen = 1;
  else if (!strcmp(name, "one-launch")) v.no_classes = 1;
  else if (!strcmp(name, "classes")) v.all_classes = 1;
  else if (!strcmp(name, "class-launches")) { v.all_classes = 1; v.split_classes = 1; }
  else if (!strcmp(name, "whole-classes")) v.whole_classes = 1;
  else if (!strcmp(name, "tap-columns")) v.no_yfold = 1;
  else if (!strcmp(name, "lds-gather")) v.gather = 1;
  else if (!strcmp(name, "no-gather")) v.gather = -1;
  else if (!strcmp(name, "no-narrow")) v.no_narrow = 1;
  else if (!strcmp(name, "narrow")) v.no_narrow = -1;
  else return fail(MELLIN_ERR_ARGUMENT, "mellin_set_variant: unknown variant '%s'", name);
  g_widen = v.widen;
  g_no_classes = v.no_classes;
  g_all_classes = v.all_classes;
  g_split_classes = v.split_classes;
  g_whole_classes = v.whole_classes;
  g_no_yfold = v.no_yfold;
  g_gather = v.gather;
  g_no_narrow = v.no_narrow;
  g_forced = v.forced;
  return MELLIN_OK;
}

#define DEFINE_1D(NAME, T, KX, KY)                                             \
  MELLIN_DECL_1D(NAME, T) {                                                    \
    return accumulate_2d<T>(#NAME, KX, KY, f, g, c_out, c_in, batch, nf, 1,    \
                            ng, 1, nh, 1, s, 1, d, 1, p, 0, u, 1,              \
                            transposed_f, transposed_g, transposed_h, h,       \
                            stream);                                           \
  }
#define DEFINE_2D(NAME, T, KX, KY)                                             \
  MELLIN_DECL_2D(NAME, T) {                                                    \
    return accumulate_2d<T>(#NAME, KX, KY, f, g, c_out, c_in, batch, nfx, nfy, \
                            ngx, ngy, nhx, nhy, sx, sy, dx, dy, px, py, ux,    \
                            uy, transposed_f, transposed_g, transposed_h, h,   \
                            stream);                                           \
  }

DEFINE_1D(mellin_mcorr1d_f32, float, AX_MCORR, AX_LCORR)
DEFINE_1D(mellin_mcorr1d_f64, double, AX_MCORR, AX_LCORR)
DEFINE_1D(mellin_mconv1d_f32, float, AX_MCONV, AX_LCONV)
DEFINE_1D(mellin_mconv1d_f64, double, AX_MCONV, AX_LCONV)
DEFINE_2D(mellin_mcorrlcorr_f32, float, AX_MCORR, AX_LCORR)
DEFINE_2D(mellin_mcorrlcorr_f64, double, AX_MCORR, AX_LCORR)
DEFINE_2D(mellin_mconvlconv_f32, float, AX_MCONV, AX_LCONV)
DEFINE_2D(mellin_mconvlconv_f64, double, AX_MCONV, AX_LCONV)
DEFINE_2D(mellin_lcorrlcorr_f32, float, AX_LCORR, AX_LCORR)
DEFINE_2D(mellin_lcorrlcorr_f64, double, AX_LCORR, AX_LCORR)
DEFINE_2D(mellin_lconvlconv_f32, float, AX_LCONV, AX_LCONV)
DEFINE_2D(mellin_lconvlconv_f64, double, AX_LCONV, AX_LCONV)

int mellin_corr2d_forward_f32(int kind_x, const float *input, const float *weight,
                              const float *bias, MELLIN_CORR2D_DIMS, float *out,
                              void *stream) {
  return corr2d_forward<float>(__func__, kind_x, input, weight, bias, CORR2D_ARGS, out, stream);
}
int mellin_corr2d_forward_f64(int kind_x, const double *input, const double *weight,
                              const double *bias, MELLIN_CORR2D_DIMS, double *out,
                              void *stream) {
  return corr2d_forward<double>(__func__, kind_x, input, weight, bias, CORR2D_ARGS, out, stream);
}
size_t mellin_corr2d_forward_workspace(int kind_x, int elem_bytes, MELLIN_CORR2D_DIMS) {
  if (elem_bytes != 4) return 0;
  if (check_corr2d(__func__, kind_x, CORR2D_ARGS)) return 0;
  if (!batch || !c_in || !c_out || !nfx || !nfy || !ngx || !ngy || !nhx || !nhy) return 0;
  return fragment_bytes(forward_problem(kind_x, CORR2D_ARGS));
}
int mellin_corr2d_forward_ws_f32(int kind_x, int activation, const float *input, const float *weight,
                                 const float *bias, MELLIN_CORR2D_DIMS, float *out, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  const size_t need = mellin_corr2d_forward_workspace(kind_x, 4, CORR2D_ARGS);
  if (need && (!workspace || workspace_bytes < need))
    return fail(MELLIN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", __func__, need,
                workspace_bytes);
  if (need && ((uintptr_t)workspace & 15))
    return fail(MELLIN_ERR_ARGUMENT, "%s: the workspace must be 16-byte aligned", __func__);
  return corr2d_forward<float>(__func__, kind_x, input, weight, bias, CORR2D_ARGS, out, stream, activation, nullptr,
                               nullptr, workspace, workspace_bytes);
}
size_t mellin_corr2d_backward_input_workspace(int kind_x, int elem_bytes,
                                              MELLIN_CORR2D_DIMS) {
  if (elem_bytes != 4 || g_forced == 1) return 0;
  if (check_corr2d(__func__, kind_x, CORR2D_ARGS)) return 0;
  if (!batch || !c_in || !c_out || !nfx || !nfy || !ngx || !ngy || !nhx || !nhy) return 0;
  InputPlans ips;
  choose_input_plan(kind_x, CORR2D_ARGS, ips);
  return ips.ws_bytes;
}
int mellin_corr2d_backward_input_f32(int kind_x, const float *weight,
                                     const float *grad_out, MELLIN_CORR2D_DIMS,
                                     float *grad_input, void *workspace,
                                     size_t workspace_bytes, void *stream) {
  return corr2d_backward_input<float>(__func__, kind_x, weight, grad_out, CORR2D_ARGS, grad_input,
                                      workspace, workspace_bytes, stream);
}
int mellin_corr2d_backward_input_f64(int kind_x, const double *weight,
                                     const double *grad_out, MELLIN_CORR2D_DIMS,
                                     double *grad_input, void *workspace,
                                     size_t workspace_bytes, void *stream) {
  return corr2d_backward_input<double>(__func__, kind_x, weight, grad_out, CORR2D_ARGS, grad_input,
                                       workspace, workspace_bytes, stream);
}
size_t mellin_corr2d_backward_weight_workspace(int kind_x, int elem_bytes,
                                               MELLIN_CORR2D_DIMS) {
  if (elem_bytes != 4 || g_forced == 1) return 0;
  if (check_corr2d(__func__, kind_x, CORR2D_ARGS)) return 0;
  if (!batch || !c_in || !c_out || !nfx || !nfy || !ngx || !ngy || !nhx || !nhy) return 0;
  WgradPosPlan pp;
  if (plan_weight_positions(forward_problem(kind_x, CORR2D_ARGS), pp)) return pp.ws_bytes;
  WgradPlan wp;
  if (!make_wgrad_plan(forward_problem(kind_x, CORR2D_ARGS), wp, g_forced != 2)) return 0;
  return wp.ws_bytes;
}
int mellin_corr2d_backward_weight_f32(int kind_x, const float *input,
                                      const float *grad_out, MELLIN_CORR2D_DIMS,
                                      float *grad_weight, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  return corr2d_backward_weight<float>(__func__, kind_x, input, grad_out, CORR2D_ARGS,
                                       grad_weight, workspace, workspace_bytes, stream);
}
size_t mellin_static_scratch_bytes(void) { return MELLIN_STATIC_SCRATCH_BYTES; }
int mellin_static_scratch_prepare(void) { return static_scratch(__func__) ? MELLIN_OK : MELLIN_ERR_RUNTIME; }
int mellin_corr2d_backward_weight_static_f32(int kind_x, const float *input, const float *grad_out,
                                             MELLIN_CORR2D_DIMS, float *grad_weight, void *stream) {
  const size_t need = mellin_corr2d_backward_weight_workspace(kind_x, 4, CORR2D_ARGS);
  if (need > MELLIN_STATIC_SCRATCH_BYTES)
    return fail(MELLIN_ERR_WORKSPACE,
                "%s: this layer needs %zu bytes of scratch memory, the static array holds %zu; use "
                "mellin_corr2d_backward_weight_f32 with a workspace", __func__, need,
                (size_t)MELLIN_STATIC_SCRATCH_BYTES);
  void *ws = static_scratch(__func__, (hipStream_t)stream, true);
  if (!ws) return MELLIN_ERR_RUNTIME;
  return corr2d_backward_weight<float>(__func__, kind_x, input, grad_out, CORR2D_ARGS, grad_weight, ws,
                                       MELLIN_STATIC_SCRATCH_BYTES, stream);
}
int mellin_corr2d_backward_weight_f64(int kind_x, const double *input,
                                      const double *grad_out, MELLIN_CORR2D_DIMS,
                                      double *grad_weight, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  return corr2d_backward_weight<double>(__func__, kind_x, input, grad_out, CORR2D_ARGS,
                                        grad_weight, workspace, workspace_bytes, stream);
}

}  // extern "C"
