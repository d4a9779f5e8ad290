"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

RTOL = 1e-5          # north-star tolerance: rtol 1e-5, atol 1e-5 * sqrt(fan_in)


def atol(fan_in):
    return 1e-5 * float(fan_in) ** 0.5


def dev():
    return torch.device("cuda:0")


def to_gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev())


def to_np(t):
    return t.detach().cpu().numpy()


def f64(*arrays):
    """Upcast inputs for a float64 run of the checker.

    Long reductions (weight and bias gradients sum tens of thousands of fp32
    products) are compared against the checker evaluated in float64 on the
    same fp32 inputs: an fp32 sequential sum of n terms carries a rounding
    error of order 6e-8 * |partial sum| * sqrt(n) of its own, which at
    n ~ 1e5 exceeds the stated tolerance, so the fp32 checker cannot anchor
    those comparisons; the exact sum can.
    """
    out = tuple(None if a is None else np.asarray(a, dtype=np.float64) for a in arrays)
    return out if len(out) > 1 else out[0]


def assert_close(got, exp, fan_in, what="", dtype=np.float32):
    got = to_np(got) if isinstance(got, torch.Tensor) else got
    assert got.shape == exp.shape, (what, got.shape, exp.shape)
    if got.dtype == np.float32 and exp.dtype == np.float64:
        exp = exp.astype(np.float32)
    if dtype == np.float64:
        np.testing.assert_allclose(got, exp, rtol=1e-10, atol=1e-10 * float(fan_in) ** 0.5, err_msg=what)
    else:
        np.testing.assert_allclose(got, exp, rtol=RTOL, atol=atol(fan_in), err_msg=what)
