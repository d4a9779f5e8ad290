"""Mellin / linear correlation layers on AMD MI355X.

Drop-in for the reference's ``mconv`` module (``mconv.py`` at the root of
sdrobert/cnn-mellin): the same public names, argument order and meaning of
``s``, ``d``, ``p``, ``r`` (and of the hidden ``u``), the same output-size
rules and the same error behaviour, but every tensor operation runs in
hand-written HIP kernels (``libmellin_hip.so``, bound in ``_mellin_hip.py``).  There
is no CPU or pure-PyTorch path: tensors must live on a HIP device and the
library must be built, otherwise the calls raise.

Reference counterparts
    size functions          mconv.py:73-118
    argument checks         mconv.py:126-231, ext/torch.cpp:10-54
    mcorr1d / mcorrlcorr    mconv.py:887-990, ops of ext/torch.cpp:467-476
    autograd                ext/torch.cpp:176-309 (MCorr1DOp, MCorrLCorrOp)
    modules                 mconv.py:1020-1288 (_CorrNd, MCorr1d, MCorrLCorr)

Additions (the reference obtains them from ``torch.nn.Conv1d/Conv2d``,
models.py:329-338): ``lcorr1d`` / ``lcorrlcorr`` and the modules ``LCorr1d`` /
``LCorrLCorr`` apply the linear relation on every axis with the same asymmetric
``p`` / ``r`` padding convention as the linear axis of ``mcorrlcorr``.
"""
from typing import Any, Optional, Tuple, Union

import torch

import _mellin_hip as _hip
from _mellin_hip import AX_LCORR, AX_MCORR

__all__ = [
    "lconv_support_size",
    "lconv_valid_size",
    "lcorr_support_size",
    "lcorr_valid_size",
    "mconv_support_size",
    "mconv_valid_size",
    "mcorr_support_size",
    "mcorr_valid_size",
    "mcorr1d",
    "MCorr1d",
    "mcorrlcorr",
    "MCorrLCorr",
    "snd2col",
    "spec2col",
    "lcorr1d",
    "LCorr1d",
    "lcorrlcorr",
    "LCorrLCorr",
]


# ---------------------------------------------------------------------------
# output-length rules: floor division, clamped at zero (mconv.py:73-118)
# ---------------------------------------------------------------------------
def _clamp(v: int) -> int:
    return v if v > 0 else 0


def lconv_support_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                       p: int = 0, u: int = 1) -> int:
    return _clamp((u * (input_size - 1) + d * (kernel_size - 1) - p) // s + 1)


def lconv_valid_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                     p: int = 0, u: int = 1) -> int:
    return _clamp((u * (input_size - 1) - p) // s + 1)


def lcorr_support_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                       p: int = 0, u: int = 1) -> int:
    return _clamp((u * (input_size - 1) + p) // s + 1)


def lcorr_valid_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                     p: int = 0, u: int = 1) -> int:
    return _clamp((u * (input_size - 1) - d * (kernel_size - 1) + p) // s + 1)


def mconv_support_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                       p: int = 0, u: int = 1) -> int:
    return _clamp(((kernel_size + d - 1) * (input_size + u - 1)) // (p + 1) - s + 1)


def mconv_valid_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                     p: int = 0, u: int = 1) -> int:
    return _clamp((d * (input_size + u - 1)) // (p + 1) - s + 1)


def mcorr_support_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                       p: int = 0, u: int = 1) -> int:
    return _clamp(((input_size + u - 1) * (p + 1)) // d - s + 1)


def mcorr_valid_size(kernel_size: int, input_size: int, s: int = 1, d: int = 1,
                     p: int = 0, u: int = 1) -> int:
    return _clamp(((input_size + u - 1) * (p + 1)) // (kernel_size + d - 1) - s + 1)


_VALID_SIZE = {
    _hip.AX_MCORR: mcorr_valid_size, _hip.AX_MCONV: mconv_valid_size,
    _hip.AX_LCORR: lcorr_valid_size, _hip.AX_LCONV: lconv_valid_size,
}


# ---------------------------------------------------------------------------
# argument checks, with the reference's wording (mconv.py:121-150,164-180)
# ---------------------------------------------------------------------------
def _arg_name(name: str, pos: int) -> str:
    return "argument #%d '%s'" % (pos, name) if pos else "'%s'" % name


def _check_dim(c: str, t: torch.Tensor, name: str, pos: int, dim: int) -> None:
    if t.dim() != dim:
        raise RuntimeError(
            "Expected %d-dimensional arg[0], but got %d-dimensional tensor for %s "
            "(while checking arguments for %s)" % (dim, t.dim(), _arg_name(name, pos), c))


def _check_size(c: str, t: torch.Tensor, name: str, pos: int, dim: int, size: int) -> None:
    if t.size(dim) != size:
        raise RuntimeError(
            "Expected tensor to have size %d at dimension %d, but got size %d for %s "
            "(while checking arguments for %s)" % (size, dim, t.size(dim), _arg_name(name, pos), c))


def _check_same_device(c: str, named) -> None:
    first = None
    for t, name, pos in named:
        if t is None:
            continue
        if first is None:
            first = (t, name, pos)
        elif str(first[0].device) != str(t.device):
            raise RuntimeError(
                "Expected tensor for %s to have the same device as tensor for %s, but device "
                "%s does not equal %s (while checking arguments for %s)"
                % (_arg_name(first[1], first[2]), _arg_name(name, pos),
                   first[0].device, t.device, c))


def _ntuple(c: str, name: str, n: int, x: Any) -> Tuple[int, ...]:
    if isinstance(x, int) and not isinstance(x, bool):
        return (x,) * n
    try:
        t = tuple(x)
        if len(t) == n and all(isinstance(v, int) for v in t):
            return t
    except TypeError:
        pass
    raise RuntimeError(
        "Expected '%s' to be either an integer or a tuple of %d integers, got %s "
        "(while checking argumengs for %s)" % (name, n, x, c))


def _single(c: str, name: str, x: Any) -> Tuple[int]:
    return _ntuple(c, name, 1, x)


def _pair(c: str, name: str, x: Any) -> Tuple[int, int]:
    return _ntuple(c, name, 2, x)


def _check_conv_args(c: str, dim: int, weight: torch.Tensor, input: torch.Tensor,
                     bias: Optional[torch.Tensor]):
    """CheckAndInferArgumentsConv (ext/torch.cpp:10-54): returns (c_out, c_in, batch)."""
    _check_dim(c, weight, "weight", 2, dim)
    _check_dim(c, input, "input", 1, dim)
    c_out, c_in, batch = weight.size(0), weight.size(1), input.size(0)
    _check_size(c, input, "input", 1, 1, c_in)
    if bias is not None:
        _check_dim(c, bias, "bias", 3, 1)
        _check_size(c, bias, "bias", 3, 0, c_out)
    _check_same_device(c, [(weight, "weight", 2), (input, "input", 1), (bias, "bias", 3)])
    if weight.dtype != input.dtype or (bias is not None and bias.dtype != input.dtype):
        raise RuntimeError(
            "expected input, weight and bias to share one dtype (while checking arguments for %s)" % c)
    return c_out, c_in, batch


def _dense_or_transposed(t: torch.Tensor):
    """The layout rule of ext/torch.cpp:40-52.

    A tensor whose first two axes are swapped in memory (as the backward
    passes produce with ``.transpose(0, 1)``) is used where it lies and flagged
    as transposed; anything else is made contiguous.
    """
    if t.is_contiguous():
        return t, False
    tt = t.transpose(0, 1)
    if tt.is_contiguous():
        return tt, True
    return t.contiguous(), False


# ---------------------------------------------------------------------------
# differentiable correlation (MCorr1DOp / MCorrLCorrOp, ext/torch.cpp:176-309)
# ---------------------------------------------------------------------------
class _Corr2dFunction(torch.autograd.Function):
    """out = bias + correlation(input, weight); x axis Mellin or linear, y axis linear."""

    # Under torch.autocast the floating-point arguments are cast to half and the op runs
    # with autocast off, as the reference's Autocast registration does
    # (ext/torch.cpp:405-430); the library then computes in fp32 and rounds once.
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(ctx, input, weight, bias, kind_x, s, d, p, u, r, name, activation=None):
        c_out, c_in, batch = _check_conv_args(name, 4, weight, input, bias)
        if activation not in (None, "relu"):
            raise RuntimeError('activation must be None or "relu", got %r (while checking arguments for %s)'
                               % (activation, name))
        fused = activation == "relu"
        nf, ng = tuple(weight.shape[2:]), tuple(input.shape[2:])
        nh = (_VALID_SIZE[kind_x](nf[0], ng[0], s[0], d[0], p[0], u[0]) + r[0],
              lcorr_valid_size(nf[1], ng[1], s[1], d[1], p[1], u[1]) + r[1])
        out = input.new_empty((batch, c_out) + nh)     # a negative size raises here, as in the reference
        input_c, weight_c = input.contiguous(), weight.contiguous()
        bias_c = None if bias is None else bias.contiguous()
        dims = _hip._dims(batch, c_in, c_out, nf, ng, nh, s, d, p, u)
        _hip.corr2d_forward(kind_x, input_c, weight_c, bias_c, out, dims,
                            _hip.ACT_RELU if fused else _hip.ACT_NONE)
        ctx.save_for_backward(input_c, weight_c, *([out] if activation == "relu" else []))
        ctx.has_bias = bias is not None
        ctx.kind_x, ctx.dims = kind_x, dims
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_out):
        input, weight = ctx.saved_tensors[:2]
        out = ctx.saved_tensors[2] if len(ctx.saved_tensors) == 3 else None
        grad_out = grad_out.contiguous()
        grad_bias = None
        want_bias = ctx.has_bias and ctx.needs_input_grad[2]
        if grad_out.dtype in (torch.float32, torch.float16) and grad_out.shape[0] <= 65535 and grad_out.shape[1] <= 65535 and \
                (out is not None or want_bias):
            # one pass: the backward of the fused ReLU (pass where out > 0) and the bias gradient
            grad_out, grad_bias = _hip.bias_grad(grad_out, out)
            if not want_bias:
                grad_bias = None
        else:
            if out is not None:                             # through the fused ReLU: pass where out > 0
                grad_out = grad_out * (out > 0)
            if want_bias:
                grad_bias = grad_out.sum((0, 2, 3))
        grad_input = grad_weight = None
        if ctx.needs_input_grad[0]:
            grad_input = _hip.corr2d_backward_input(
                ctx.kind_x, weight, grad_out, torch.empty_like(input), ctx.dims)
        if ctx.needs_input_grad[1]:
            grad_weight = _hip.corr2d_backward_weight(
                ctx.kind_x, input, grad_out, torch.empty_like(weight), ctx.dims)
        return grad_input, grad_weight, grad_bias, None, None, None, None, None, None, None, None


def _corr2d(kind_x, name, input, weight, bias, s, d, p, u, r, activation=None):
    return _Corr2dFunction.apply(input, weight, bias, kind_x, s, d, p, u, r, name, activation)


def _corr1d(kind, name, input, weight, bias, s, d, p, u, r, activation=None):
    # a 1-D layer is the 2-D layer with a unit second axis
    _check_dim(name, weight, "weight", 2, 3)
    _check_dim(name, input, "input", 1, 3)
    out = _Corr2dFunction.apply(
        input.unsqueeze(-1), weight.unsqueeze(-1), bias, kind,
        (s, 1), (d, 1), (p, 0), (u, 1), (r, 0), name, activation)
    return out.squeeze(-1)


def _ext_mcorr1d(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, activation=None):
    """``torch.ops.mellin.mcorr1d`` (ext/torch.cpp:469): Mellin correlation, differentiable."""
    return _corr1d(AX_MCORR, "mcorr1d", input, weight, bias, s, d, p, u, r, activation)


def _ext_mcorrlcorr(input, weight, bias=None, s=(1, 1), d=(1, 1), p=(0, 0), u=(1, 1), r=(0, 0),
                    activation=None):
    """``torch.ops.mellin.mcorrlcorr`` (ext/torch.cpp:470)."""
    s, d, p, u, r = (_pair("mcorrlcorr", k, v) for k, v in zip("sdpur", (s, d, p, u, r)))
    return _corr2d(AX_MCORR, "mcorrlcorr", input, weight, bias, s, d, p, u, r, activation)


def _ext_lcorr1d(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0, activation=None):
    return _corr1d(AX_LCORR, "lcorr1d", input, weight, bias, s, d, p, u, r, activation)


def _ext_lcorrlcorr(input, weight, bias=None, s=(1, 1), d=(1, 1), p=(0, 0), u=(1, 1), r=(0, 0),
                    activation=None):
    s, d, p, u, r = (_pair("lcorrlcorr", k, v) for k, v in zip("sdpur", (s, d, p, u, r)))
    return _corr2d(AX_LCORR, "lcorrlcorr", input, weight, bias, s, d, p, u, r, activation)


# ---------------------------------------------------------------------------
# the accumulate-into-output kernels as plain ops (no autograd), with the
# reference adapters' layout handling (ext/torch_cuda.cu:45-177)
# ---------------------------------------------------------------------------
def _raw_op(name, kinds, input, weight, bias, s, d, p, u, r):
    dim = 3 if len(kinds) == 1 else 4
    c_out, c_in, batch = _check_conv_args(name, dim, weight, input, bias)
    f, tf = _dense_or_transposed(weight)
    g, tg = _dense_or_transposed(input)
    nf, ng = tuple(weight.shape[2:]), tuple(input.shape[2:])
    nh = tuple(_VALID_SIZE[k](nf[i], ng[i], s[i], d[i], p[i], u[i]) + r[i]
               for i, k in enumerate(kinds))
    h = weight.new_empty((batch, c_out) + nh)
    if bias is None:
        h.zero_()
    else:
        h.copy_(bias.view((1, c_out) + (1,) * len(nh)).expand_as(h))
    if dim == 3:
        _hip.accumulate(name, f, g, h, c_out, c_in, batch, nf[0], ng[0], nh[0],
                        s[0], d[0], p[0], u[0], tf, tg, False)
    else:
        _hip.accumulate(name, f, g, h, c_out, c_in, batch, nf, ng, nh, s, d, p, u, tf, tg, False)
    return h


def _ext_mconv1d(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0):
    """``torch.ops.mellin.mconv1d`` (ext/torch.cpp:468): Mellin convolution, no autograd."""
    return _raw_op("mconv1d", (_hip.AX_MCONV,), input, weight, bias, (s,), (d,), (p,), (u,), (r,))


def _ext_mconvlconv(input, weight, bias=None, s=(1, 1), d=(1, 1), p=(0, 0), u=(1, 1), r=(0, 0)):
    """``torch.ops.mellin.mconvlconv`` (ext/torch.cpp:471)."""
    s, d, p, u, r = (_pair("mconvlconv", k, v) for k, v in zip("sdpur", (s, d, p, u, r)))
    return _raw_op("mconvlconv", (_hip.AX_MCONV, _hip.AX_LCONV), input, weight, bias, s, d, p, u, r)


def _raw_mcorr1d(input, weight, bias=None, s=1, d=1, p=0, u=1, r=0):
    """The accumulate kernel behind mcorr1d, honouring transposed views (no autograd)."""
    return _raw_op("mcorr1d", (AX_MCORR,), input, weight, bias, (s,), (d,), (p,), (u,), (r,))


def _raw_mcorrlcorr(input, weight, bias=None, s=(1, 1), d=(1, 1), p=(0, 0), u=(1, 1), r=(0, 0)):
    s, d, p, u, r = (_pair("mcorrlcorr", k, v) for k, v in zip("sdpur", (s, d, p, u, r)))
    return _raw_op("mcorrlcorr", (AX_MCORR, AX_LCORR), input, weight, bias, s, d, p, u, r)


# ---------------------------------------------------------------------------
# column ops (Snd2ColOp / Spec2ColOp, ext/torch.cpp:310-389; adapters
# ext/torch_cuda.cu:179-291): the gather behind the reference's "mm" path
# ---------------------------------------------------------------------------
def _check_col_args(c: str, dim: int, input: torch.Tensor):
    """CheckAndInferArgumentsCol (ext/torch.cpp:57-85): returns (batch, c_in)."""
    _check_dim(c, input, "input", 1, dim)
    return input.size(0), input.size(1)


class _ToColFunction(torch.autograd.Function):
    """gg = x2col(input); backward is col2x (the adjoint gather)."""

    # autocast: cast to half as the reference does (ext/torch.cpp:433-447).  Half tensors
    # are widened for the library call: the gather moves values unchanged, and the
    # adjoint's sums are then taken in fp32 and rounded once.
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(ctx, input, nf, s, d, p, u, r, name):
        dim = len(nf)
        batch, c_in = _check_col_args(name, dim + 2, input)
        narrow = input.dtype == torch.float16
        if narrow:
            input = input.float()
        ng = tuple(input.shape[2:])
        kinds = (_hip.AX_MCORR, _hip.AX_LCORR)[:dim]
        ngg = tuple(_VALID_SIZE[k](nf[i], ng[i], s[i], d[i], p[i], u[i]) + r[i]
                    for i, k in enumerate(kinds))
        g, tg = _dense_or_transposed(input)
        gg = input.new_empty((batch, c_in) + tuple(nf) + ngg)
        ctx.args = (nf, ng, ngg, s, d, p, u, dim)
        if gg.numel():
            if dim == 1:
                _hip.col_op("snd2col", g, gg, c_in, batch, nf[0], ng[0], ngg[0], s[0], d[0], p[0], u[0],
                            tg, False)
            else:
                _hip.col_op("spec2col", g, gg, c_in, batch, nf, ng, ngg, s, d, p, u, tg, False)
        return gg.half() if narrow else gg

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_out):
        nf, ng, ngg, s, d, p, u, dim = ctx.args
        grad_input = _from_col(grad_out, ng, s, d, p, u, dim)
        return (grad_input,) + (None,) * 7


def _from_col(cols, ng, s, d, p, u, dim):
    """col2snd / col2spec (ext/torch_cuda.cu:208-235, :267-291)."""
    name = "col2snd" if dim == 1 else "col2spec"
    batch, c_in = _check_col_args(name, 2 + 2 * dim, cols)
    if cols.dtype == torch.float16:
        return _from_col(cols.float(), ng, s, d, p, u, dim).half()
    nf = tuple(cols.shape[2:2 + dim])
    ngg = tuple(cols.shape[2 + dim:])
    gg, tgg = _dense_or_transposed(cols)
    g = cols.new_empty((batch, c_in) + tuple(ng))
    if g.numel():
        if dim == 1:
            _hip.col_op(name, gg, g, c_in, batch, nf[0], ng[0], ngg[0], s[0], d[0], p[0], u[0], False, tgg)
        else:
            _hip.col_op(name, gg, g, c_in, batch, nf, tuple(ng), ngg, s, d, p, u, False, tgg)
    return g


def _ext_snd2col(input, kernel_width, s=1, d=1, p=0, u=1, r=0):
    """``torch.ops.mellin.snd2col`` (ext/torch.cpp:473): (N, C, T) -> (N, C, K, T_out)."""
    return _ToColFunction.apply(input, (kernel_width,), (s,), (d,), (p,), (u,), (r,), "snd2col")


def _ext_col2snd(input, snd_width, s=1, d=1, p=0, u=1):
    """``torch.ops.mellin.col2snd`` (ext/torch.cpp:474): the adjoint of snd2col, no autograd."""
    return _from_col(input, (snd_width,), (s,), (d,), (p,), (u,), 1)


def _ext_spec2col(input, kernel_size, s=(1, 1), d=(1, 1), p=(0, 0), u=(1, 1), r=(0, 0)):
    """``torch.ops.mellin.spec2col`` (ext/torch.cpp:475): (N, C, T, F) -> (N, C, Kx, Ky, T_out, F_out)."""
    return _ToColFunction.apply(input, tuple(kernel_size), tuple(s), tuple(d), tuple(p), tuple(u),
                                tuple(r), "spec2col")


def _ext_col2spec(input, spec_size, s=(1, 1), d=(1, 1), p=(0, 0), u=(1, 1)):
    """``torch.ops.mellin.col2spec`` (ext/torch.cpp:476): the adjoint of spec2col, no autograd."""
    return _from_col(input, tuple(spec_size), tuple(s), tuple(d), tuple(p), tuple(u), 2)


# ---------------------------------------------------------------------------
# public functional API (mconv.py:887-1017); ``u`` stays hidden
# ---------------------------------------------------------------------------
def _pick_impl(c: str, _impl):
    # The reference switches to a gather + matmul formulation ("mm") for
    # kernels with fewer than ten taps and asserts that it equals the direct
    # one (tests/test_mconv.py:632-660).  Here one direct kernel family serves
    # every size, so both names select it.
    if _impl in (None, "direct", "mm"):
        return "direct"
    raise NotImplementedError(
        '_impl "%s" not supported (while checking arguments for %s)' % (_impl, c))


def mcorr1d(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
            s: int = 1, d: int = 1, p: int = 0, r: int = 0, _impl=None,
            activation: Optional[str] = None) -> torch.Tensor:
    """1-D Mellin correlation of ``(batch, in_channels, T_in)`` input with
    ``(out_channels, in_channels, T_kern)`` weight; see :class:`MCorr1d`.

    ``activation="relu"`` (not in the reference) returns ``relu(result)`` from the same kernel."""
    _pick_impl("mcorr1d", _impl)
    return _ext_mcorr1d(input, weight, bias, s, d, p, 1, r, activation)


def mcorrlcorr(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               s: Any = 1, d: Any = 1, p: Any = 0, r: Any = 0, _impl=None,
               activation: Optional[str] = None) -> torch.Tensor:
    """2-D correlation, Mellin along axis 2 and linear along axis 3; see :class:`MCorrLCorr`.

    ``activation="relu"`` (not in the reference) returns ``relu(result)`` from the same kernel."""
    s_, d_, p_, r_ = (_pair("mcorrlcorr", k, v) for k, v in zip("sdpr", (s, d, p, r)))
    _pick_impl("mcorrlcorr", _impl)
    return _ext_mcorrlcorr(input, weight, bias, s_, d_, p_, (1, 1), r_, activation)


def lcorr1d(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
            s: int = 1, d: int = 1, p: int = 0, r: int = 0,
            activation: Optional[str] = None) -> torch.Tensor:
    """1-D linear correlation with left padding ``p`` and right padding ``r``."""
    return _ext_lcorr1d(input, weight, bias, s, d, p, 1, r, activation)


def lcorrlcorr(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               s: Any = 1, d: Any = 1, p: Any = 0, r: Any = 0,
               activation: Optional[str] = None) -> torch.Tensor:
    """2-D linear correlation ("lconv2d") with asymmetric padding ``p`` (left) / ``r`` (right)."""
    s_, d_, p_, r_ = (_pair("lcorrlcorr", k, v) for k, v in zip("sdpr", (s, d, p, r)))
    return _ext_lcorrlcorr(input, weight, bias, s_, d_, p_, (1, 1), r_, activation)


def snd2col(input: torch.Tensor, kernel_width: int, s: int = 1, d: int = 1, p: int = 0,
            r: int = 0) -> torch.Tensor:
    return _ext_snd2col(input, kernel_width, s, d, p, 1, r)


def spec2col(input: torch.Tensor, kernel_size: Any, s: Any = 1, d: Any = 1, p: Any = 0,
             r: Any = 0) -> torch.Tensor:
    kernel_size_ = _pair("spec2col", "kernel_size", kernel_size)
    s_, d_, p_, r_ = (_pair("spec2col", k, v) for k, v in zip("sdpr", (s, d, p, r)))
    return _ext_spec2col(input, kernel_size_, s_, d_, p_, (1, 1), r_)


# ---------------------------------------------------------------------------
# modules (mconv.py:1020-1288): same parameter names and shapes, so state
# dicts are interchangeable with the reference's layers
# ---------------------------------------------------------------------------
class _CorrNd(torch.nn.Module):

    __constants__ = ["s", "d", "p", "r"]

    def __init__(self, in_channels: int, out_channels: int, kernel_size: Tuple[int, ...],
                 s: Tuple[int, ...], d: Tuple[int, ...], p: Tuple[int, ...],
                 r: Tuple[int, ...], bias: bool = True):
        super().__init__()
        self.s, self.d, self.p, self.r = s, d, p, r
        self.weight = torch.nn.Parameter(torch.empty(out_channels, in_channels, *kernel_size))
        if bias:
            self.bias = torch.nn.Parameter(torch.empty(out_channels))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def extra_repr(self) -> str:
        return "%d, %d, kernel_size=%s, s=%s, d=%s, p=%s, r=%s" % (
            self.weight.size(1), self.weight.size(0), self.weight.shape[1:],
            self.s, self.d, self.p, self.r)

    def reset_parameters(self) -> None:
        # U(-1/sqrt(fan_in), +1/sqrt(fan_in)) for weight and bias (mconv.py:1062-1067)
        fan_in = 1
        for n in self.weight.shape[1:]:
            fan_in *= int(n)
        bound = fan_in ** -0.5 if fan_in > 0 else 0.0
        torch.nn.init.uniform_(self.weight, -bound, bound)
        if self.bias is not None:
            torch.nn.init.uniform_(self.bias, -bound, bound)


class MCorr1d(_CorrNd):
    r"""1-D Mellin correlation layer.

    For input ``(N, in_channels, T_in)``

        out[n, co, t] = bias[co] + sum_{ci, tau} weight[co, ci, tau] *
                        input[n, ci, (t + s)(tau + d)/(p + 1) - 1]

    where a term exists only if the division is exact and the index lies in
    ``[0, T_in)``.  ``T_out = floor(T_in (p + 1)/(T_kern + d - 1)) - s + 1 + r``;
    ``r = 0`` gives the valid length and ``r`` extends it towards (or past) the
    support length, positions past the support holding only the bias.
    """

    def __init__(self, in_channels: int, out_channels: int, kernel_size: int, s: int = 1,
                 d: int = 1, p: int = 0, r: int = 0, bias: bool = True):
        kernel_size = _single("MCorr1d", "kernel_size", kernel_size)
        s, d = _single("MCorr1d", "s", s), _single("MCorr1d", "d", d)
        p, r = _single("MCorr1d", "p", p), _single("MCorr1d", "r", r)
        super().__init__(in_channels, out_channels, kernel_size, s, d, p, r, bias)

    def forward(self, input: torch.Tensor, activation: Optional[str] = None) -> torch.Tensor:
        return mcorr1d(input, self.weight, self.bias, self.s[0], self.d[0], self.p[0], self.r[0],
                       activation=activation)


class MCorrLCorr(_CorrNd):
    r"""2-D layer: Mellin correlation along axis 2 (time), linear along axis 3 (frequency).

        out[n, co, t, f] = bias[co] + sum_{ci, tau, w} weight[co, ci, tau, w] *
            input[n, ci, (t + s[0])(tau + d[0])/(p[0] + 1) - 1, s[1] f + d[1] w - p[1]]

    ``p[1]`` pads the frequency axis on the left and ``r[1]`` on the right
    (``p[1] = r[1] = padding`` reproduces symmetric padding); ``r[0]`` extends
    the time axis past its valid length.
    """

    def __init__(self, in_channels: int, out_channels: int,
                 kernel_size: Union[int, Tuple[int, int]], s: Union[int, Tuple[int, int]] = 1,
                 d: Union[int, Tuple[int, int]] = 1, p: Union[int, Tuple[int, int]] = 0,
                 r: Union[int, Tuple[int, int]] = 0, bias: bool = True):
        kernel_size = _pair("MCorrLCorr", "kernel_size", kernel_size)
        s, d = _pair("MCorrLCorr", "s", s), _pair("MCorrLCorr", "d", d)
        p, r = _pair("MCorrLCorr", "p", p), _pair("MCorrLCorr", "r", r)
        super().__init__(in_channels, out_channels, kernel_size, s, d, p, r, bias)

    def forward(self, input: torch.Tensor, activation: Optional[str] = None) -> torch.Tensor:
        return mcorrlcorr(input, self.weight, self.bias, self.s, self.d, self.p, self.r, activation=activation)


class LCorr1d(_CorrNd):
    """1-D linear correlation layer with the ``s, d, p, r`` convention of the linear axis."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size: int, s: int = 1,
                 d: int = 1, p: int = 0, r: int = 0, bias: bool = True):
        kernel_size = _single("LCorr1d", "kernel_size", kernel_size)
        s, d = _single("LCorr1d", "s", s), _single("LCorr1d", "d", d)
        p, r = _single("LCorr1d", "p", p), _single("LCorr1d", "r", r)
        super().__init__(in_channels, out_channels, kernel_size, s, d, p, r, bias)

    def forward(self, input: torch.Tensor, activation: Optional[str] = None) -> torch.Tensor:
        return lcorr1d(input, self.weight, self.bias, self.s[0], self.d[0], self.p[0], self.r[0],
                       activation=activation)


class LCorrLCorr(_CorrNd):
    """2-D linear correlation layer ("lconv2d"): the linear relation on both axes."""

    def __init__(self, in_channels: int, out_channels: int,
                 kernel_size: Union[int, Tuple[int, int]], s: Union[int, Tuple[int, int]] = 1,
                 d: Union[int, Tuple[int, int]] = 1, p: Union[int, Tuple[int, int]] = 0,
                 r: Union[int, Tuple[int, int]] = 0, bias: bool = True):
        kernel_size = _pair("LCorrLCorr", "kernel_size", kernel_size)
        s, d = _pair("LCorrLCorr", "s", s), _pair("LCorrLCorr", "d", d)
        p, r = _pair("LCorrLCorr", "p", p), _pair("LCorrLCorr", "r", r)
        super().__init__(in_channels, out_channels, kernel_size, s, d, p, r, bias)

    def forward(self, input: torch.Tensor, activation: Optional[str] = None) -> torch.Tensor:
        return lcorrlcorr(input, self.weight, self.bias, self.s, self.d, self.p, self.r, activation=activation)
