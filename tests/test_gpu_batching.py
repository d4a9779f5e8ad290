"""Batching invariance on the GPU: the result for a batch of N copies of one signal is the
batch-1 result N times.

Mirror of the reference's c/tests/test_batching_cuda.cc over the grid of c/tests/CMakeLists.txt:35-49
(c_in in {1, 128}, c_out in {1, 256}, nf in {3, 10}, ng in {10, 300}, nh in {10, 40}, s in {1, 2},
d in {1, 3}, p in {0, 5}, u in {1, 7}, batch in {2, 10}, the transposed layouts), through the
accumulate-into-h entry points of section 1 of the C ABI (the kernel-level contract those tests
drive: `h` starts as zeros).  The reference gives both axes of its 2-D cases the same sizes; here
the y axis of a 2-D case takes nf = 3, ng = 10 or 41 and nh = 10 with the same s, d, p, u, which
keeps the largest signal at 63 MB instead of 4.6 GB.  Of the sixteen (s, d, p, u) combinations four
are run per case, drawn with a fixed seed, and the transposed flags are drawn per case.

The reference compares with an absolute 1e-8, i.e. bit for bit: its kernels add an output's
products in one fixed order whatever the batch.  The one-thread-per-output kernels here do the
same and are held to that ("generic").  The automatic choice is held to the operator tolerance
(rtol 1e-5, atol 1e-5 * sqrt(fan_in)) instead: which matrix kernel a layer takes, how many
channels it stages per chunk and whether its products run on the fp32 or the bf16 matrix
instructions depend on the size of the whole launch, the batch included, and two such forms
group an output's products differently inside the matrix instructions.  (For a fixed shape every
form is bit-reproducible from run to run; tests/test_gpu_parity.py checks that.)  The share of
cases that come out bit-identical all the same is printed.
"""
import itertools

import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import to_gpu, to_np

pytestmark = pytest.mark.gpu

GRID = list(itertools.product((1, 128), (1, 256), (3, 10), (10, 300), (10, 40)))   # c_in, c_out, nf, ng, nh
PARAMS = list(itertools.product((1, 2), (1, 3), (0, 5), (1, 7)))                  # s, d, p, u


@pytest.fixture(params=["generic", "auto"])
def variant(request):
    hip.set_variant(request.param)
    yield request.param
    hip.set_variant(None)


@pytest.mark.parametrize("op", ["mcorr1d", "mconv1d", "mcorrlcorr", "mconvlconv"])
def test_batch_n_is_batch_1_tiled(op, variant):
    rng = np.random.default_rng({"mcorr1d": 1, "mconv1d": 2, "mcorrlcorr": 3, "mconvlconv": 4}[op])
    two_d = op in ("mcorrlcorr", "mconvlconv")
    cases = nonzero = identical = 0
    for c_in, c_out, nfx, ngx, nhx in GRID:
        for s, d, p, u in [PARAMS[i] for i in rng.choice(len(PARAMS), 4, replace=False)]:
            for batch in (2, 10):
                tf, tg, th = (bool(v) for v in rng.integers(0, 2, 3))
                if two_d:
                    nf, ng, nh = (nfx, 3), (ngx, 10 if ngx == 10 else 41), (nhx, 10)
                    sz = lambda t: t[0] * t[1]
                    pr = ((s, s), (d, d), (p, p), (u, u))
                else:
                    nf, ng, nh = nfx, ngx, nhx
                    sz = lambda t: t
                    pr = (s, d, p, u)
                w = rng.uniform(-1, 1, c_out * c_in * sz(nf)).astype(np.float32)
                g1 = rng.uniform(-1, 1, (c_in, sz(ng))).astype(np.float32)
                # batch 1 (the transposed layouts of one image coincide with the dense ones)
                h1 = torch.zeros(c_out * sz(nh), device="cuda")
                hip.accumulate(op, to_gpu(w), to_gpu(g1.ravel()), h1, c_out, c_in, 1, nf, ng, nh, *pr, tf, tg, th)
                # batch N: g as (batch, c_in, .) or, transposed, (c_in, batch, .)
                gn = np.broadcast_to(g1[:, None, :] if tg else g1[None, :, :],
                                     (c_in, batch, sz(ng)) if tg else (batch, c_in, sz(ng)))
                hn = torch.zeros(batch * c_out * sz(nh), device="cuda")
                hip.accumulate(op, to_gpu(w), to_gpu(np.ascontiguousarray(gn).ravel()), hn, c_out, c_in, batch,
                               nf, ng, nh, *pr, tf, tg, th)
                one = to_np(h1).reshape(c_out, sz(nh))
                many = to_np(hn).reshape((c_out, batch, sz(nh)) if th else (batch, c_out, sz(nh)))
                exp = np.broadcast_to(one[:, None, :] if th else one[None, :, :], many.shape)
                case = (op, c_out, c_in, batch, nf, ng, nh, pr, tf, tg, th)
                same = np.array_equal(many, exp)
                if variant == "generic":
                    assert same, (case, float(np.abs(many - exp).max()))
                else:
                    np.testing.assert_allclose(many, exp, rtol=1e-5, atol=1e-5 * (c_in * sz(nf)) ** 0.5, err_msg=str(case))
                identical += same
                cases += 1
                nonzero += bool(np.any(one != 0))
    print("%s [%s]: %d of %d cases bit-identical" % (op, variant, identical, cases))
    assert cases == len(GRID) * 8 and nonzero > cases // 2
