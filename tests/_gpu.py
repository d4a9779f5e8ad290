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


def assert_close(got, exp, fan_in, what="", dtype=np.float32):
    got = to_np(got) if isinstance(got, torch.Tensor) else got
    assert got.shape == exp.shape, (what, got.shape, exp.shape)
    if dtype == np.float64:
        np.testing.assert_allclose(got, exp, rtol=1e-10, atol=1e-10 * float(fan_in) ** 0.5, err_msg=what)
    else:
        np.testing.assert_allclose(got, exp, rtol=RTOL, atol=atol(fan_in), err_msg=what)
