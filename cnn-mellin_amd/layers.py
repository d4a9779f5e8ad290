"""The pointwise layers in front of the convolutions (reference layers.py), on the HIP library.

Same names, arguments, parameters and initialisation as the reference:

* ``dilation_lift(input, tau, dim)`` / ``DilationLift(dim=2)`` (layers.py:8-21, 40-77):
  ``out[..., t - 1, ...] = t ** tau * input[..., t - 1, ...]`` along ``dim``, the module's
  learnable parameter being ``log_tau`` (``tau = exp(log_tau)``), drawn from N(0, 1);
* ``LogCompression()`` (layers.py:79-101): ``log(eps + |input|)`` with learnable ``log_eps``;
* ``ScaledGaussianNoise(dim=1, eps=1e-3)`` (layers.py:24-37, 104-145): noise with a standard
  deviation of ``eps`` times the largest magnitude along ``dim``, in training only (random
  numbers come from PyTorch's generator, so this one stays a composition of PyTorch ops).

``LogCompressionLift(dim=2)`` is the pair the acoustic model applies back to back
(models.py:414-417) as ONE pass over the data each way: the reference runs it as half a
dozen elementwise launches.  Every function here needs the HIP library and GPU tensors;
there is no CPU path.
"""
from typing import Optional

import torch

import _mellin_hip as _hip

__all__ = ["dilation_lift", "log_compression", "log_compression_lift", "DilationLift", "LogCompression",
           "LogCompressionLift", "ScaledGaussianNoise"]


def _check_dim(input: torch.Tensor, dim: int) -> int:
    dim_ = dim + input.dim() if dim < 0 else dim
    if dim_ >= input.dim() or dim_ < 0:
        # the reference's wording (layers.py:11-14)
        raise RuntimeError(f"{dim} not a valid dimension for a tensor if dimension {input.dim()}")
    return dim_


class _LogLiftFunction(torch.autograd.Function):
    """y = [t ** tau *] [log(eps + |x|)] through mellin_log_lift_{forward,backward}."""

    @staticmethod
    def forward(ctx, input, eps, tau, flags, dim):
        _hip.require_device(input)
        x = input.contiguous()
        shape = x.shape
        outer = 1
        for v in shape[:dim]:
            outer *= v
        inner = 1
        for v in shape[dim + 1:]:
            inner *= v
        t = shape[dim] if x.dim() else 1
        # eps and tau are device values (exp of the modules' parameters): they go to the
        # kernels as a two-element device tensor, not through float(), which would wait
        # for the device and cannot be captured in a graph
        one, zero = x.new_ones(()), x.new_zeros(())
        params = torch.stack([eps.detach().to(device=x.device, dtype=x.dtype).reshape(()) if eps is not None else one,
                              tau.detach().to(device=x.device, dtype=x.dtype).reshape(()) if tau is not None else zero])
        y = torch.empty_like(x)
        _hip.log_lift_forward_dev(x, params, flags, outer, t, inner, y)
        ctx.save_for_backward(x, params, eps if isinstance(eps, torch.Tensor) else None,
                              tau if isinstance(tau, torch.Tensor) else None)
        ctx.geometry = (flags, outer, t, inner)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, params, eps, tau = ctx.saved_tensors
        flags, outer, t, inner = ctx.geometry
        grad_x = torch.empty_like(x)
        grad_params = torch.empty(2, dtype=x.dtype, device=x.device)
        _hip.log_lift_backward_dev(x, grad_y.contiguous(), params, flags, outer, t, inner, grad_x, grad_params)
        g_eps = grad_params[0].to(eps.dtype).reshape(eps.shape) if eps is not None and ctx.needs_input_grad[1] else None
        g_tau = grad_params[1].to(tau.dtype).reshape(tau.shape) if tau is not None and ctx.needs_input_grad[2] else None
        return grad_x, g_eps, g_tau, None, None


def _floating(input: torch.Tensor) -> None:
    if input.dtype not in (torch.float32, torch.float64):
        raise RuntimeError("expected a float32 or float64 tensor, got %s" % input.dtype)


def dilation_lift(input: torch.Tensor, tau: torch.Tensor, dim: int) -> torch.Tensor:
    """``out[t - 1] = t ** tau * input[t - 1]`` along `dim` (reference layers.py:8-21)."""
    dim_ = _check_dim(input, dim)
    _floating(input)
    return _LogLiftFunction.apply(input, None, tau, _hip.PW_LIFT, dim_)


def log_compression(input: torch.Tensor, eps: torch.Tensor) -> torch.Tensor:
    """``log(eps + |input|)`` (reference layers.py:100-101, with ``eps = exp(log_eps)``)."""
    _floating(input)
    return _LogLiftFunction.apply(input, eps, None, _hip.PW_LOG, max(input.dim() - 1, 0))


def log_compression_lift(input: torch.Tensor, eps: torch.Tensor, tau: torch.Tensor, dim: int) -> torch.Tensor:
    """``t ** tau * log(eps + |input|)``: `log_compression` then `dilation_lift`, in one pass."""
    dim_ = _check_dim(input, dim)
    _floating(input)
    return _LogLiftFunction.apply(input, eps, tau, _hip.PW_LOG | _hip.PW_LIFT, dim_)


class DilationLift(torch.nn.Module):
    """Reference layers.py:40-77: learnable ``log_tau``, ``forward(x) = dilation_lift(x, exp(log_tau), dim)``."""

    __constants__ = ["dim"]

    def __init__(self, dim: int = 2):
        super().__init__()
        self.log_tau = torch.nn.Parameter(torch.tensor(0.0))
        self.dim = dim
        self.reset_parameters()

    def extra_repr(self) -> str:
        return f"dim={self.dim}"

    def reset_parameters(self) -> None:
        torch.nn.init.normal_(self.log_tau)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return dilation_lift(input, self.log_tau.exp(), self.dim)


class LogCompression(torch.nn.Module):
    """Reference layers.py:79-101: learnable ``log_eps``, ``forward(x) = log(exp(log_eps) + |x|)``."""

    def __init__(self):
        super().__init__()
        self.log_eps = torch.nn.Parameter(torch.tensor(0.0))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        torch.nn.init.normal_(self.log_eps)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return log_compression(input, self.log_eps.exp())


class LogCompressionLift(torch.nn.Module):
    """`LogCompression` followed by `DilationLift(dim)`, as the acoustic model applies them
    (models.py:414-417), with both parameters, in one pass over the data."""

    __constants__ = ["dim"]

    def __init__(self, dim: int = 2):
        super().__init__()
        self.log_eps = torch.nn.Parameter(torch.tensor(0.0))
        self.log_tau = torch.nn.Parameter(torch.tensor(0.0))
        self.dim = dim
        self.reset_parameters()

    def extra_repr(self) -> str:
        return f"dim={self.dim}"

    def reset_parameters(self) -> None:
        torch.nn.init.normal_(self.log_eps)
        torch.nn.init.normal_(self.log_tau)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return log_compression_lift(input, self.log_eps.exp(), self.log_tau.exp(), self.dim)


def scaled_gaussian_noise(x: torch.Tensor, eps: float, dim: int, training: bool = True,
                          generator: Optional[torch.Generator] = None) -> torch.Tensor:
    """Reference layers.py:24-37."""
    _check_dim(x, dim)
    if training is False:
        return x
    mu, _ = x.abs().max(dim, keepdim=True)
    noise = torch.randn(x.shape, dtype=x.dtype, device=x.device, generator=generator)
    return x + (mu * eps) * noise


class ScaledGaussianNoise(torch.nn.Module):
    """Reference layers.py:104-145: ``x + eps * max_t |x| * N(0, 1)`` in training, ``x`` otherwise."""

    __constants__ = ["dim", "eps"]

    def __init__(self, dim: int = 1, eps: float = 1e-3):
        super().__init__()
        self.dim = dim
        self.eps = eps

    def extra_repr(self) -> str:
        return f"dim={self.dim}, eps={self.eps}"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return scaled_gaussian_noise(x, self.eps, self.dim, self.training)
