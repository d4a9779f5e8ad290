"""ctypes front end of the CPU checker.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package never does.

Two back ends share one calling convention:

* ``impl="port"``  -> ``oracle/_build/libmellin_oracle.so``: this repository's
  restatement (``mellin_oracle.c``) of the reference kernels.
* ``impl="ref"``   -> ``oracle/_ref/libmellin_ref.so``: the unmodified reference
  header compiled behind C names (``ref_shim.cpp``); present only where a
  reference checkout was available at build time.

On top of the raw kernels this module restates the reference's host adapters
with numpy arrays so that tests can compare whole operators:

* op level (output size = valid size + r, bias broadcast into the output, then
  the accumulate-into-``h`` kernel): ``ext/torch_cpu.cpp:29-145`` and
  ``ext/torch.cpp:88-101``;
* the backward identities of the autograd functions (role-swapped calls with
  ``transposed_f`` / ``transposed_g`` flags instead of materialised transposes):
  ``ext/torch.cpp:193-239`` (1-D) and ``ext/torch.cpp:261-308`` (2-D).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PORT = os.path.join(_HERE, "_build", "libmellin_oracle.so")
_REF = os.path.join(_HERE, "_ref", "libmellin_ref.so")

AX_MCORR, AX_MCONV, AX_LCORR, AX_LCONV = 0, 1, 2, 3

_i64 = ctypes.c_int64
_int = ctypes.c_int
_ptr = ctypes.c_void_p
_libs = {}


def build(ref=None):
    """Compile the checker (and the reference shim when a checkout exists)."""
    subprocess.check_call(["make", "-C", _HERE, "-s", "all"])
    if ref is None:
        ref = os.path.isdir("/root/reference/ext/include")
    if ref:
        subprocess.check_call(["make", "-C", _HERE, "-s", "ref"])


def have_ref():
    return os.path.isfile(_REF)


def _lib(impl):
    if impl not in _libs:
        path = {"port": _PORT, "ref": _REF}[impl]
        if not os.path.isfile(path):
            if impl == "port":
                build(ref=False)
            else:
                raise FileNotFoundError(path)
        _libs[impl] = ctypes.CDLL(path)
    return _libs[impl]


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError("checker handles float32/float64, got %s" % dtype)


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


# --------------------------------------------------------------------------
# sizes (mconv.py:73-118 argument order: kernel_size, input_size, s, d, p, u)
# --------------------------------------------------------------------------
def _size(name):
    def fn(kernel_size, input_size, s=1, d=1, p=0, u=1, impl="port"):
        if impl == "ref":
            # the reference's C++ functions drop the arguments they do not use
            args = {
                "mconv_valid": (input_size, s, d, p, u),
                "mconv_support": (kernel_size, input_size, s, d, p, u),
                "lconv_valid": (input_size, s, p, u),
                "lconv_support": (kernel_size, input_size, s, d, p, u),
                "mcorr_valid": (kernel_size, input_size, s, d, p, u),
                "mcorr_support": (input_size, s, d, p, u),
                "lcorr_valid": (kernel_size, input_size, s, d, p, u),
                "lcorr_support": (input_size, s, p, u),
            }[name]
            f = getattr(_lib("ref"), "ref_%s_size" % name)
        else:
            args = (kernel_size, input_size, s, d, p, u)
            f = getattr(_lib("port"), "oracle_%s_size" % name)
        f.restype = _i64
        f.argtypes = [_i64] * len(args)
        return int(f(*args))

    fn.__name__ = name + "_size"
    return fn


mconv_valid_size = _size("mconv_valid")
mconv_support_size = _size("mconv_support")
lconv_valid_size = _size("lconv_valid")
lconv_support_size = _size("lconv_support")
mcorr_valid_size = _size("mcorr_valid")
mcorr_support_size = _size("mcorr_support")
lcorr_valid_size = _size("lcorr_valid")
lcorr_support_size = _size("lcorr_support")

_VALID = {
    AX_MCORR: mcorr_valid_size, AX_MCONV: mconv_valid_size,
    AX_LCORR: lcorr_valid_size, AX_LCONV: lconv_valid_size,
}
_SUPPORT = {
    AX_MCORR: mcorr_support_size, AX_MCONV: mconv_support_size,
    AX_LCORR: lcorr_support_size, AX_LCONV: lconv_support_size,
}


def tap(kind, h, f, ng, s=1, d=1, p=0, u=1):
    fn = _lib("port").oracle_tap
    fn.restype = _i64
    fn.argtypes = [_int] + [_i64] * 7
    return int(fn(kind, h, f, ng, s, d, p, u))


def tap_map(kind, nf, ng, nh, s=1, d=1, p=0, u=1):
    """(nh, nf) int64 array: signal index per (output, filter) index or -1."""
    out = np.empty((nh, nf), dtype=np.int64)
    fn = _lib("port").oracle_tap_map
    fn.restype = None
    fn.argtypes = [_int] + [_i64] * 7 + [_ptr]
    fn(kind, nf, ng, nh, s, d, p, u, _p(out))
    return out


# --------------------------------------------------------------------------
# raw kernels (accumulate into a caller-initialised h; mconv.h:46-50)
# --------------------------------------------------------------------------
_OPS2D = {
    (AX_MCORR, AX_LCORR): "mcorrlcorr",
    (AX_MCONV, AX_LCONV): "mconvlconv",
    (AX_LCORR, AX_LCORR): "lcorrlcorr",
    (AX_LCONV, AX_LCONV): "lconvlconv",
}


def kernel2d(kinds, f, g, h, c_out, c_in, batch, nf, ng, nh, s, d, p, u,
             transposed_f=False, transposed_g=False, transposed_h=False, impl="port"):
    """Run one accumulate-into-h kernel on flat C-contiguous buffers.

    ``f``/``g``/``h`` hold the layouts selected by the ``transposed_*`` flags
    (mconv.h:29-50); ``nf``, ``ng``, ``nh``, ``s``, ``d``, ``p``, ``u`` are pairs.
    """
    name = _OPS2D[tuple(kinds)]
    suf = _suffix(f.dtype)
    assert g.dtype == f.dtype and h.dtype == f.dtype
    assert f.flags.c_contiguous and g.flags.c_contiguous and h.flags.c_contiguous
    assert f.size == c_out * c_in * nf[0] * nf[1]
    assert g.size == batch * c_in * ng[0] * ng[1]
    assert h.size == batch * c_out * nh[0] * nh[1]
    if impl == "ref":
        if name not in ("mcorrlcorr", "mconvlconv"):
            raise NotImplementedError("the reference has no %s kernel" % name)
        fn = getattr(_lib("ref"), "ref_%s_%s" % (name, suf))
    else:
        fn = getattr(_lib("port"), "oracle_%s_%s" % (name, suf))
    fn.restype = None
    fn.argtypes = [_ptr, _ptr] + [_i64] * 17 + [_int] * 3 + [_ptr]
    fn(_p(f), _p(g), c_out, c_in, batch, nf[0], nf[1], ng[0], ng[1], nh[0], nh[1],
       s[0], s[1], d[0], d[1], p[0], p[1], u[0], u[1],
       int(transposed_f), int(transposed_g), int(transposed_h), _p(h))
    return h


def kernel1d(kind, f, g, h, c_out, c_in, batch, nf, ng, nh, s, d, p, u,
             transposed_f=False, transposed_g=False, transposed_h=False, impl="port"):
    name = {AX_MCORR: "mcorr1d", AX_MCONV: "mconv1d"}[kind]
    suf = _suffix(f.dtype)
    assert f.flags.c_contiguous and g.flags.c_contiguous and h.flags.c_contiguous
    prefix, lib = ("ref_", _lib("ref")) if impl == "ref" else ("oracle_", _lib("port"))
    fn = getattr(lib, "%s%s_%s" % (prefix, name, suf))
    fn.restype = None
    fn.argtypes = [_ptr, _ptr] + [_i64] * 10 + [_int] * 3 + [_ptr]
    fn(_p(f), _p(g), c_out, c_in, batch, nf, ng, nh, s, d, p, u,
       int(transposed_f), int(transposed_g), int(transposed_h), _p(h))
    return h


def _pair(x):
    return (x, x) if isinstance(x, int) else tuple(int(v) for v in x)


def _layout(x):
    """CheckAndInferArgumentsConv's contiguity rule (ext/torch.cpp:40-52).

    Returns (flat C-contiguous buffer, transposed flag) for a (A, B, ...) array:
    if the array with its first two axes swapped is C-contiguous that memory is
    used as is and the flag is set, otherwise a contiguous copy is made.
    """
    if x.ndim >= 2 and np.swapaxes(x, 0, 1).flags.c_contiguous and not x.flags.c_contiguous:
        return np.swapaxes(x, 0, 1), True
    return np.ascontiguousarray(x), False


def _build_output(dtype, bias, size):
    """BuildOutput (ext/torch.cpp:88-101): bias broadcast over channels, or zeros."""
    out = np.zeros(size, dtype=dtype)
    if bias is not None:
        out += np.asarray(bias, dtype=dtype).reshape((1, size[1]) + (1,) * (len(size) - 2))
    return out


def _op2d(kinds, input, weight, bias, s, d, p, u, r, impl):
    s, d, p, u, r = map(_pair, (s, d, p, u, r))
    fbuf, tf = _layout(weight)
    gbuf, tg = _layout(input)
    c_out, c_in, nfx, nfy = weight.shape
    batch, c_in_g, ngx, ngy = input.shape
    if c_in_g != c_in:
        raise RuntimeError("channel mismatch %d vs %d" % (c_in_g, c_in))
    nhx = _VALID[kinds[0]](nfx, ngx, s[0], d[0], p[0], u[0]) + r[0]
    nhy = _VALID[kinds[1]](nfy, ngy, s[1], d[1], p[1], u[1]) + r[1]
    h = _build_output(weight.dtype, bias, (batch, c_out, nhx, nhy))
    if h.size:
        kernel2d(kinds, fbuf, gbuf, h, c_out, c_in, batch, (nfx, nfy), (ngx, ngy),
                 (nhx, nhy), s, d, p, u, tf, tg, False, impl)
    return h


def mcorrlcorr(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, impl="port"):
    """mcorrlcorr_cpu, ext/torch_cpu.cpp:116-145."""
    return _op2d((AX_MCORR, AX_LCORR), input, weight, bias, s, d, p, u, r, impl)


def mconvlconv(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, impl="port"):
    """mconvlconv_cpu, ext/torch_cpu.cpp:85-114."""
    return _op2d((AX_MCONV, AX_LCONV), input, weight, bias, s, d, p, u, r, impl)


def lcorrlcorr(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, impl="port"):
    """Linear correlation on both axes (what models.py:334-336 gets from Conv2d)."""
    return _op2d((AX_LCORR, AX_LCORR), input, weight, bias, s, d, p, u, r, impl)


def lconvlconv(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, impl="port"):
    return _op2d((AX_LCONV, AX_LCONV), input, weight, bias, s, d, p, u, r, impl)


def _op1d(kind, input, weight, bias, s, d, p, u, r, impl):
    fbuf, tf = _layout(weight)
    gbuf, tg = _layout(input)
    c_out, c_in, nf = weight.shape
    batch, c_in_g, ng = input.shape
    if c_in_g != c_in:
        raise RuntimeError("channel mismatch %d vs %d" % (c_in_g, c_in))
    nh = _VALID[kind](nf, ng, s, d, p, u) + r
    h = _build_output(weight.dtype, bias, (batch, c_out, nh))
    if h.size:
        kernel1d(kind, fbuf, gbuf, h, c_out, c_in, batch, nf, ng, nh, s, d, p, u,
                 tf, tg, False, impl)
    return h


def mcorr1d(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, impl="port"):
    """mcorr1d_cpu, ext/torch_cpu.cpp:57-83."""
    return _op1d(AX_MCORR, input, weight, bias, s, d, p, u, r, impl)


def mconv1d(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, impl="port"):
    """mconv1d_cpu, ext/torch_cpu.cpp:29-55."""
    return _op1d(AX_MCONV, input, weight, bias, s, d, p, u, r, impl)


# --------------------------------------------------------------------------
# backward identities
# --------------------------------------------------------------------------
def mcorr1d_backward(input, weight, grad_out, s=1, d=1, p=0, u=1, impl="port"):
    """MCorr1DOp::backward, ext/torch.cpp:193-239 -> (grad_input, grad_weight, grad_bias)."""
    nf, ng, nh = weight.shape[2], input.shape[2], grad_out.shape[2]
    r = ng - mconv_valid_size(0, nf, u, s, p, d)
    gi = mconv1d(np.swapaxes(weight, 0, 1), grad_out, None, u, s, p, d, r, impl)
    r = nf - mcorr_valid_size(nh, ng, d, s, p, u)
    gw = mcorr1d(np.swapaxes(input, 0, 1), np.swapaxes(grad_out, 0, 1), None,
                 d, s, p, u, r, impl)
    return np.swapaxes(gi, 0, 1), np.swapaxes(gw, 0, 1), grad_out.sum(0).sum(1)


def _backward2d(kinds_fwd, kinds_conv, input, weight, grad_out, s, d, p, u, impl):
    s, d, p, u = map(_pair, (s, d, p, u))
    nfx, nfy = weight.shape[2:]
    ngx, ngy = input.shape[2:]
    nhx, nhy = grad_out.shape[2:]
    rx = ngx - _VALID[kinds_conv[0]](0, nfx, u[0], s[0], p[0], d[0])
    ry = ngy - _VALID[kinds_conv[1]](0, nfy, u[1], s[1], p[1], d[1])
    gi = _op2d(kinds_conv, np.swapaxes(weight, 0, 1), grad_out, None,
               u, s, p, d, (rx, ry), impl)
    rx = nfx - _VALID[kinds_fwd[0]](nhx, ngx, d[0], s[0], p[0], u[0])
    ry = nfy - _VALID[kinds_fwd[1]](nhy, ngy, d[1], s[1], p[1], u[1])
    gw = _op2d(kinds_fwd, np.swapaxes(input, 0, 1), np.swapaxes(grad_out, 0, 1), None,
               d, s, p, u, (rx, ry), impl)
    gb = grad_out.sum(0).reshape(grad_out.shape[1], -1).sum(1)
    return np.swapaxes(gi, 0, 1), np.swapaxes(gw, 0, 1), gb


def mcorrlcorr_backward(input, weight, grad_out, s=1, d=1, p=0, u=1, impl="port"):
    """MCorrLCorrOp::backward, ext/torch.cpp:261-308."""
    return _backward2d((AX_MCORR, AX_LCORR), (AX_MCONV, AX_LCONV),
                       input, weight, grad_out, s, d, p, u, impl)


def lcorrlcorr_backward(input, weight, grad_out, s=1, d=1, p=0, u=1, impl="port"):
    """The same role-swap identities with the linear relation on both axes."""
    return _backward2d((AX_LCORR, AX_LCORR), (AX_LCONV, AX_LCONV),
                       input, weight, grad_out, s, d, p, u, impl)


# --------------------------------------------------------------------------
# column ops (snd2col_cpu ... col2spec_cpu, ext/torch_cpu.cpp:147-245)
# --------------------------------------------------------------------------
def _col_call(name, src, dst, c_in, batch, nf, ng, ngg, s, d, p, u, tg, tgg, impl):
    suf = _suffix(src.dtype)
    prefix, lib = ("ref_", _lib("ref")) if impl == "ref" else ("oracle_", _lib("port"))
    fn = getattr(lib, "%s%s_%s" % (prefix, name, suf))
    fn.restype = None
    if name in ("spec2col", "col2spec"):
        fn.argtypes = [_ptr] + [_i64] * 16 + [_int] * 2 + [_ptr]
        fn(_p(src), c_in, batch, nf[0], nf[1], ng[0], ng[1], ngg[0], ngg[1],
           s[0], s[1], d[0], d[1], p[0], p[1], u[0], u[1], int(tg), int(tgg), _p(dst))
    else:
        fn.argtypes = [_ptr] + [_i64] * 9 + [_int] * 2 + [_ptr]
        fn(_p(src), c_in, batch, nf, ng, ngg, s, d, p, u, int(tg), int(tgg), _p(dst))
    return dst


def snd2col(input, kernel_width, s=1, d=1, p=0, u=1, r=0, impl="port"):
    g, tg = _layout(input)
    batch, c_in, ng = input.shape
    ngg = mcorr_valid_size(kernel_width, ng, s, d, p, u) + r
    gg = np.empty((batch, c_in, kernel_width, ngg), dtype=input.dtype)
    if gg.size:
        _col_call("snd2col", g, gg, c_in, batch, kernel_width, ng, ngg, s, d, p, u,
                  tg, False, impl)
    return gg


def col2snd(input, snd_width, s=1, d=1, p=0, u=1, impl="port"):
    gg, tgg = _layout(input)
    batch, c_in, nf, ngg = input.shape
    g = np.empty((batch, c_in, snd_width), dtype=input.dtype)
    if g.size:
        _col_call("col2snd", gg, g, c_in, batch, nf, snd_width, ngg, s, d, p, u,
                  False, tgg, impl)
    return g


def spec2col(input, kernel_size, s=1, d=1, p=0, u=1, r=0, impl="port"):
    nf, s, d, p, u, r = map(_pair, (kernel_size, s, d, p, u, r))
    g, tg = _layout(input)
    batch, c_in, ngx, ngy = input.shape
    nggx = mcorr_valid_size(nf[0], ngx, s[0], d[0], p[0], u[0]) + r[0]
    nggy = lcorr_valid_size(nf[1], ngy, s[1], d[1], p[1], u[1]) + r[1]
    gg = np.empty((batch, c_in, nf[0], nf[1], nggx, nggy), dtype=input.dtype)
    if gg.size:
        _col_call("spec2col", g, gg, c_in, batch, nf, (ngx, ngy), (nggx, nggy),
                  s, d, p, u, tg, False, impl)
    return gg


def col2spec(input, spec_size, s=1, d=1, p=0, u=1, impl="port"):
    ng, s, d, p, u = map(_pair, (spec_size, s, d, p, u))
    gg, tgg = _layout(input)
    batch, c_in, nfx, nfy, nggx, nggy = input.shape
    g = np.empty((batch, c_in, ng[0], ng[1]), dtype=input.dtype)
    if g.size:
        _col_call("col2spec", gg, g, c_in, batch, (nfx, nfy), ng, (nggx, nggy),
                  s, d, p, u, False, tgg, impl)
    return g


# ---- the pointwise layers in front of the convolutions (numpy, float64) ----------
def log_lift(x, eps=None, tau=None, dim=2):
    """``[t ** tau *] [log(eps + |x|)]`` with ``t = 1 .. T`` along `dim`.

    Follows the reference's ``LogCompression.forward`` (layers.py:100-101:
    ``(input.abs() + eps).log()``) and ``dilation_lift`` (layers.py:8-21: the input
    times ``arange(1, T + 1) ** tau`` broadcast along `dim`); a function that is
    not selected (``eps`` or ``tau`` None) is skipped."""
    y = np.asarray(x, dtype=np.float64)
    if eps is not None:
        y = np.log(np.abs(y) + float(eps))
    if tau is not None:
        shape = [1] * y.ndim
        shape[dim] = y.shape[dim]
        y = y * (np.arange(1, y.shape[dim] + 1, dtype=np.float64) ** float(tau)).reshape(shape)
    return y


def log_lift_backward(x, grad_y, eps=None, tau=None, dim=2):
    """(grad_x, d/d eps, d/d tau) of `log_lift` by the chain rule; |x| has
    derivative 0 at 0, as in PyTorch's ``abs``."""
    x = np.asarray(x, dtype=np.float64)
    g = np.asarray(grad_y, dtype=np.float64)
    p = np.ones_like(x)
    lnt = np.zeros_like(x)
    if tau is not None:
        shape = [1] * x.ndim
        shape[dim] = x.shape[dim]
        t = np.arange(1, x.shape[dim] + 1, dtype=np.float64).reshape(shape)
        p = p * t ** float(tau)
        lnt = lnt + np.log(t)
    gp = g * p
    if eps is not None:
        a = np.abs(x) + float(eps)
        return gp / a * np.sign(x), float((gp / a).sum()), float((gp * lnt * np.log(a)).sum())
    return gp, 0.0, float((gp * lnt * x).sum())
