"""ctypes binding of libmellin_hip.so (the C ABI declared in include/mellin_hip.h).

The library is the only compute back end of this package: if it has not been
built, importing this module raises, and nothing falls back to PyTorch or CPU
code.  Build it with ``python cnn-mellin_amd/build.py`` (hipcc, gfx950).
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmellin_hip.so")

AX_MCORR, AX_MCONV, AX_LCORR, AX_LCONV = 0, 1, 2, 3

_i64 = ctypes.c_int64
_int = ctypes.c_int
_ptr = ctypes.c_void_p
_size_t = ctypes.c_size_t

if not os.path.isfile(LIB_PATH):
    raise ImportError(
        "%s is missing: build the HIP library first (python %s)"
        % (LIB_PATH, os.path.join(_HERE, "build.py"))
    )

lib = ctypes.CDLL(LIB_PATH)

_SUFFIX = {torch.float32: "f32", torch.float64: "f64", torch.float16: "f16"}

# name -> (restype, argtypes); every symbol include/mellin_hip.h declares
_ACC1D = [_ptr, _ptr] + [_i64] * 10 + [_int] * 3 + [_ptr, _ptr]
_ACC2D = [_ptr, _ptr] + [_i64] * 17 + [_int] * 3 + [_ptr, _ptr]
_DIMS = [_i64] * 17
_SND = [_ptr] + [_i64] * 9 + [_int] * 2 + [_ptr, _ptr]
_SPEC = [_ptr] + [_i64] * 16 + [_int] * 2 + [_ptr, _ptr]
SYMBOLS = {
    "mellin_version": (_int, []),
    "mellin_last_error": (ctypes.c_char_p, []),
    "mellin_last_variant": (ctypes.c_char_p, []),
    "mellin_set_variant": (_int, [ctypes.c_char_p]),
    "mellin_set_math": (_int, [_int]),
    "mellin_get_math": (_int, []),
    "mellin_last_math": (_int, []),
    "mellin_corr2d_backward_weight_workspace": (_size_t, [_int, _int] + _DIMS),
    "mellin_corr2d_backward_input_workspace": (_size_t, [_int, _int] + _DIMS),
    "mellin_log_lift_backward_workspace": (_size_t, [_int, _i64, _i64, _i64]),
}
SYMBOLS["mellin_corr2d_forward_workspace"] = (_size_t, [_int, _int] + _DIMS)
SYMBOLS["mellin_corr2d_forward_ws_f32"] = (_int, [_int, _int, _ptr, _ptr, _ptr] + _DIMS + [_ptr, _ptr, _size_t, _ptr])
SYMBOLS["mellin_bias_grad_workspace"] = (_size_t, [_i64, _i64, _i64])
for _t in ("f32", "f16"):
    SYMBOLS["mellin_bias_grad_" + _t] = (_int, [_ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr, _ptr, _size_t, _ptr])
    SYMBOLS["mellin_pool_pairs_forward_" + _t] = (_int, [_ptr, _i64, _i64, _ptr, _ptr, _ptr])
    SYMBOLS["mellin_pool_pairs_backward_" + _t] = (_int, [_ptr, _ptr, _i64, _i64, _ptr, _ptr])
SYMBOLS["mellin_static_scratch_bytes"] = (_size_t, [])
SYMBOLS["mellin_static_scratch_prepare"] = (_int, [])
SYMBOLS["mellin_corr2d_backward_weight_static_f32"] = (_int, [_int, _ptr, _ptr] + _DIMS + [_ptr, _ptr])
for _n in ("forward", "backward_input", "backward_weight"):
    SYMBOLS["mellin_corr2d_%s_f16_workspace" % _n] = (_size_t, [_int] + _DIMS)
SYMBOLS["mellin_corr2d_forward_f16"] = (_int, [_int, _ptr, _ptr, _ptr] + _DIMS + [_ptr, _ptr, _size_t, _ptr])
SYMBOLS["mellin_corr2d_forward_act_f16"] = (_int, [_int, _int, _ptr, _ptr, _ptr] + _DIMS + [_ptr, _ptr, _size_t, _ptr])
SYMBOLS["mellin_corr2d_backward_input_f16"] = (_int, [_int, _ptr, _ptr] + _DIMS + [_ptr, _ptr, _size_t, _ptr])
SYMBOLS["mellin_corr2d_backward_weight_f16"] = (_int, [_int, _ptr, _ptr] + _DIMS + [_ptr, _ptr, _size_t, _ptr])
_dbl = ctypes.c_double
PW_LOG, PW_LIFT = 1, 2
for _t in ("f32", "f64"):
    for _n in ("mcorr1d", "mconv1d"):
        SYMBOLS["mellin_%s_%s" % (_n, _t)] = (_int, _ACC1D)
    for _n in ("mcorrlcorr", "mconvlconv", "lcorrlcorr", "lconvlconv"):
        SYMBOLS["mellin_%s_%s" % (_n, _t)] = (_int, _ACC2D)
    for _n in ("snd2col", "col2snd"):
        SYMBOLS["mellin_%s_%s" % (_n, _t)] = (_int, _SND)
    for _n in ("spec2col", "col2spec"):
        SYMBOLS["mellin_%s_%s" % (_n, _t)] = (_int, _SPEC)
    SYMBOLS["mellin_log_lift_forward_" + _t] = (_int, [_ptr, _dbl, _dbl, _int, _i64, _i64, _i64, _ptr, _ptr])
    SYMBOLS["mellin_log_lift_backward_" + _t] = (
        _int, [_ptr, _ptr, _dbl, _dbl, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _size_t, _ptr])
    SYMBOLS["mellin_log_lift_forward_dev_" + _t] = (_int, [_ptr, _ptr, _int, _i64, _i64, _i64, _ptr, _ptr])
    SYMBOLS["mellin_log_lift_backward_dev_" + _t] = (
        _int, [_ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _size_t, _ptr])
    SYMBOLS["mellin_corr2d_forward_act_" + _t] = (_int, [_int, _int, _ptr, _ptr, _ptr] + _DIMS + [_ptr, _ptr])
    SYMBOLS["mellin_corr2d_forward_" + _t] = (_int, [_int, _ptr, _ptr, _ptr] + _DIMS + [_ptr, _ptr])
    SYMBOLS["mellin_corr2d_backward_input_" + _t] = (
        _int, [_int, _ptr, _ptr] + _DIMS + [_ptr, _ptr, _size_t, _ptr])
    SYMBOLS["mellin_corr2d_backward_weight_" + _t] = (
        _int, [_int, _ptr, _ptr] + _DIMS + [_ptr, _ptr, _size_t, _ptr])

for _name, (_res, _args) in SYMBOLS.items():
    _fn = getattr(lib, _name)          # AttributeError if the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args


def last_error():
    return lib.mellin_last_error().decode()


def last_variant():
    return lib.mellin_last_variant().decode()


def set_variant(name=None):
    _check(lib.mellin_set_variant((name or "").encode()))


MATH_FP32, MATH_BF16X3, MATH_BF16X3_ALWAYS = 0, 1, 2
MATH_F16 = 3          # reported by last_math() only: half-precision operands on the f16 matrix cores


def set_math(mode):
    """MATH_BF16X3 (default): fp32 products as six bf16 products of three-part operands, fp32
    accumulate; MATH_FP32: the fp32 matrix instructions; MATH_BF16X3_ALWAYS: the bf16 form also
    for layers so small that the default leaves them on the fp32 instructions."""
    _check(lib.mellin_set_math(int(mode)))


def get_math():
    return lib.mellin_get_math()


def last_math():
    """The mode the most recent operator-level call's kernels multiplied in."""
    return lib.mellin_last_math()


def _check(code):
    if code != 0:
        raise RuntimeError("libmellin_hip: %s (code %d)" % (last_error(), code))


def suffix(dtype, half_ok=True):
    if dtype == torch.float16 and not half_ok:
        raise RuntimeError("this entry point takes float32 or float64 tensors, got %s" % dtype)
    try:
        return _SUFFIX[dtype]
    except KeyError:
        raise RuntimeError(
            "libmellin_hip takes float16, float32 or float64 tensors, got %s" % dtype) from None


def require_device(*tensors):
    """All tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise RuntimeError(
                "this build runs on AMD GPUs only: expected a HIP ('cuda') tensor, got a "
                "tensor on %s (there is no CPU path)" % t.device)
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("tensors are on different devices: %s and %s" % (dev, t.device))
    return dev


def _stream(dev):
    return _ptr(torch.cuda.current_stream(dev).cuda_stream)


def _dp(t):
    return _ptr(t.data_ptr()) if t is not None and t.numel() else _ptr(0)


def accumulate(name, f, g, h, c_out, c_in, batch, nf, ng, nh, s, d, p, u, tf, tg, th):
    """Call one of the accumulate-into-h kernels; sizes/params are ints (1-D) or pairs (2-D)."""
    dev = require_device(f, g, h)
    fn = getattr(lib, "mellin_%s_%s" % (name, suffix(h.dtype, half_ok=False)))
    with torch.cuda.device(dev):
        if isinstance(nf, int):
            code = fn(_dp(f), _dp(g), c_out, c_in, batch, nf, ng, nh, s, d, p, u,
                      int(tf), int(tg), int(th), _dp(h), _stream(dev))
        else:
            code = fn(_dp(f), _dp(g), c_out, c_in, batch, nf[0], nf[1], ng[0], ng[1],
                      nh[0], nh[1], s[0], s[1], d[0], d[1], p[0], p[1], u[0], u[1],
                      int(tf), int(tg), int(th), _dp(h), _stream(dev))
    _check(code)
    return h


def col_op(name, src, dst, c_in, batch, nf, ng, ngg, s, d, p, u, tg, tgg):
    """snd2col / col2snd (ints) or spec2col / col2spec (pairs): `src` -> `dst`, both dense."""
    dev = require_device(src, dst)
    fn = getattr(lib, "mellin_%s_%s" % (name, suffix(dst.dtype, half_ok=False)))
    with torch.cuda.device(dev):
        if isinstance(nf, int):
            code = fn(_dp(src), c_in, batch, nf, ng, ngg, s, d, p, u, int(tg), int(tgg), _dp(dst),
                      _stream(dev))
        else:
            code = fn(_dp(src), c_in, batch, nf[0], nf[1], ng[0], ng[1], ngg[0], ngg[1], s[0], s[1],
                      d[0], d[1], p[0], p[1], u[0], u[1], int(tg), int(tgg), _dp(dst), _stream(dev))
    _check(code)
    return dst


def log_lift_forward(x, eps, tau, flags, outer, t, inner, y):
    """y = the selected pointwise function of x, both dense and viewed as (outer, t, inner)."""
    dev = require_device(x, y)
    fn = getattr(lib, "mellin_log_lift_forward_" + suffix(y.dtype, half_ok=False))
    with torch.cuda.device(dev):
        _check(fn(_dp(x), float(eps), float(tau), flags, outer, t, inner, _dp(y), _stream(dev)))
    return y


def log_lift_forward_dev(x, params, flags, outer, t, inner, y):
    """As log_lift_forward with params = (eps, tau) in a device tensor of x's type: no copy to the host."""
    dev = require_device(x, params, y)
    _same_dtype(x, params, y)
    fn = getattr(lib, "mellin_log_lift_forward_dev_" + suffix(y.dtype, half_ok=False))
    with torch.cuda.device(dev):
        _check(fn(_dp(x), _dp(params), flags, outer, t, inner, _dp(y), _stream(dev)))
    return y


def log_lift_backward_dev(x, grad_y, params, flags, outer, t, inner, grad_x, grad_params):
    dev = require_device(x, grad_y, params, grad_x, grad_params)
    _same_dtype(x, grad_y, params, grad_x, grad_params)
    fn = getattr(lib, "mellin_log_lift_backward_dev_" + suffix(grad_x.dtype, half_ok=False))
    need = lib.mellin_log_lift_backward_workspace(grad_x.element_size(), outer, t, inner)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _check(fn(_dp(x), _dp(grad_y), _dp(params), flags, outer, t, inner, _dp(grad_x),
                  _ptr(grad_params.data_ptr()), _ptr(ws.data_ptr()), need, _stream(dev)))
    return grad_x, grad_params


def log_lift_backward(x, grad_y, eps, tau, flags, outer, t, inner, grad_x, grad_params):
    """grad_x and grad_params = (d/d eps, d/d tau); allocates the scratch the library asks for."""
    dev = require_device(x, grad_y, grad_x, grad_params)
    fn = getattr(lib, "mellin_log_lift_backward_" + suffix(grad_x.dtype, half_ok=False))
    need = lib.mellin_log_lift_backward_workspace(grad_x.element_size(), outer, t, inner)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _check(fn(_dp(x), _dp(grad_y), float(eps), float(tau), flags, outer, t, inner, _dp(grad_x),
                  _ptr(grad_params.data_ptr()), _ptr(ws.data_ptr()), need, _stream(dev)))
    return grad_x, grad_params


def bias_grad(grad_out, out=None):
    """(g, grad_bias) for a dense float32 or float16 grad_out (N, C, ...): grad_bias = per-channel sums of g, with
    g = grad_out, or grad_out where `out` > 0 (the backward of a ReLU fused into the forward pass)."""
    dev = require_device(grad_out, out)
    _same_dtype(grad_out, out)
    n, c = grad_out.shape[0], grad_out.shape[1]
    plane = grad_out[0, 0].numel() if n and c else 0
    g = torch.empty_like(grad_out) if out is not None else grad_out
    grad_bias = torch.empty(c, dtype=grad_out.dtype, device=dev)
    need = lib.mellin_bias_grad_workspace(n, c, plane)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        fn = getattr(lib, "mellin_bias_grad_" + _pointwise_suffix(grad_out))
        _check(fn(_dp(grad_out), _dp(out), n, c, plane, _dp(g) if out is not None else None,
                  _dp(grad_bias), _ptr(ws.data_ptr()), need, _stream(dev)))
    return g, grad_bias


def _pointwise_suffix(t):
    if t.dtype not in (torch.float32, torch.float16):
        raise RuntimeError("float32 or float16 tensors only, got %s" % t.dtype)
    return _SUFFIX[t.dtype]


def pool_pairs_forward(x):
    """(y, which) for a dense float32 or float16 x (..., f): maxima over pairs of neighbours along the last axis."""
    dev = require_device(x)
    f = x.shape[-1]
    rows = x.numel() // f if f else 0
    y = torch.empty(x.shape[:-1] + (f // 2,), dtype=x.dtype, device=dev)
    which = torch.empty(y.shape, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        fn = getattr(lib, "mellin_pool_pairs_forward_" + _pointwise_suffix(x))
        _check(fn(_dp(x), rows, f, _dp(y), _dp(which), _stream(dev)))
    return y, which


def pool_pairs_backward(grad_y, which, f):
    dev = require_device(grad_y, which)
    grad_x = torch.empty(grad_y.shape[:-1] + (f,), dtype=grad_y.dtype, device=dev)
    rows = grad_x.numel() // f if f else 0
    with torch.cuda.device(dev):
        fn = getattr(lib, "mellin_pool_pairs_backward_" + _pointwise_suffix(grad_y))
        _check(fn(_dp(grad_y), _dp(which), rows, f, _dp(grad_x), _stream(dev)))
    return grad_x


def _dims(batch, c_in, c_out, nf, ng, nh, s, d, p, u):
    return (batch, c_in, c_out, nf[0], nf[1], ng[0], ng[1], nh[0], nh[1],
            s[0], s[1], d[0], d[1], p[0], p[1], u[0], u[1])


def _same_dtype(*tensors):
    dts = {t.dtype for t in tensors if t is not None}
    if len(dts) > 1:
        raise RuntimeError("operands must share one dtype, got %s" % sorted(str(d) for d in dts))


ACT_NONE, ACT_RELU = 0, 1


def corr2d_forward(kind_x, input, weight, bias, out, dims, activation=ACT_NONE, workspace=None,
                   workspace_bytes=None):
    """Forward pass; float32 scratch memory (the filter's bf16 fragments of wide layers) comes
    from `workspace` or, if None, from torch's caching allocator on the launch stream."""
    dev = require_device(input, weight, bias, out)
    _same_dtype(input, weight, bias, out)
    with torch.cuda.device(dev):
        if out.dtype == torch.float16:
            need = lib.mellin_corr2d_forward_f16_workspace(kind_x, *dims)
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
            _check(lib.mellin_corr2d_forward_act_f16(kind_x, activation, _dp(input), _dp(weight), _dp(bias), *dims,
                                                     _dp(out), _ptr(ws.data_ptr()), need, _stream(dev)))
        elif out.dtype == torch.float32:
            if workspace is None:
                workspace_bytes = lib.mellin_corr2d_forward_workspace(kind_x, 4, *dims)
                workspace = (torch.empty(workspace_bytes, dtype=torch.uint8, device=dev)
                             if workspace_bytes else None)
            _check(lib.mellin_corr2d_forward_ws_f32(kind_x, activation, _dp(input), _dp(weight), _dp(bias), *dims,
                                                    _dp(out), _dp(workspace), workspace_bytes or 0, _stream(dev)))
        else:
            fn = getattr(lib, "mellin_corr2d_forward_act_" + suffix(out.dtype))
            _check(fn(kind_x, activation, _dp(input), _dp(weight), _dp(bias), *dims, _dp(out), _stream(dev)))
    return out


def _workspace(kind_x, which, out, dims, workspace, workspace_bytes):
    if workspace is None:
        if out.dtype == torch.float16:
            workspace_bytes = getattr(lib, "mellin_corr2d_backward_%s_f16_workspace" % which)(kind_x, *dims)
        else:
            query = getattr(lib, "mellin_corr2d_backward_%s_workspace" % which)
            workspace_bytes = query(kind_x, out.element_size(), *dims)
        workspace = (torch.empty(workspace_bytes, dtype=torch.uint8, device=out.device)
                     if workspace_bytes else None)
    return workspace, workspace_bytes


def corr2d_backward_input(kind_x, weight, grad_out, grad_input, dims, workspace=None,
                          workspace_bytes=None):
    """Input gradient; scratch memory comes from `workspace` or, if None, from torch's
    caching allocator on the launch stream."""
    dev = require_device(weight, grad_out, grad_input)
    workspace, workspace_bytes = _workspace(kind_x, "input", grad_input, dims, workspace,
                                            workspace_bytes)
    _same_dtype(weight, grad_out, grad_input)
    fn = getattr(lib, "mellin_corr2d_backward_input_" + suffix(grad_input.dtype))
    with torch.cuda.device(dev):
        _check(fn(kind_x, _dp(weight), _dp(grad_out), *dims, _dp(grad_input),
                  _dp(workspace), workspace_bytes, _stream(dev)))
    return grad_input


def corr2d_backward_weight(kind_x, input, grad_out, grad_weight, dims, workspace=None,
                           workspace_bytes=None):
    """Weight gradient; scratch memory comes from `workspace` or, if None, from torch's
    caching allocator on the launch stream."""
    dev = require_device(input, grad_out, grad_weight)
    workspace, workspace_bytes = _workspace(kind_x, "weight", grad_weight, dims, workspace,
                                            workspace_bytes)
    _same_dtype(input, grad_out, grad_weight)
    fn = getattr(lib, "mellin_corr2d_backward_weight_" + suffix(grad_weight.dtype))
    with torch.cuda.device(dev):
        _check(fn(kind_x, _dp(input), _dp(grad_out), *dims, _dp(grad_weight),
                  _dp(workspace), workspace_bytes, _stream(dev)))
    return grad_weight


def corr2d_backward_weight_static(kind_x, input, grad_out, grad_weight, dims):
    """Weight gradient (fp32) with the partial sums in the library's static device array:
    no allocation anywhere on the way.  Layers needing more than
    mellin_static_scratch_bytes() raise; overlapping calls on one GPU race."""
    dev = require_device(input, grad_out, grad_weight)
    _same_dtype(input, grad_out, grad_weight)
    if grad_weight.dtype != torch.float32:
        raise RuntimeError("the allocation-free weight gradient takes float32 tensors, got %s" % grad_weight.dtype)
    with torch.cuda.device(dev):
        _check(lib.mellin_corr2d_backward_weight_static_f32(kind_x, _dp(input), _dp(grad_out), *dims,
                                                            _dp(grad_weight), _stream(dev)))
    return grad_weight
