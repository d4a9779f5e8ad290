"""Host-side behaviour of the drop-in module that needs no GPU: output-length
rules, argument checks and their messages, layer construction, and the
C-ABI's own argument validation (which returns before any kernel launch)."""
import ctypes
import os
import re

import pytest
import torch

import mconv
import _mellin_hip as hip
from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SIZE_FUNCS = ["lconv_support", "lconv_valid", "lcorr_support", "lcorr_valid",
              "mconv_support", "mconv_valid", "mcorr_support", "mcorr_valid"]


def test_public_names_match_reference():
    # mconv.py:22-37 of the reference
    ref_all = ["lconv_support_size", "lconv_valid_size", "lcorr_support_size", "lcorr_valid_size",
               "mconv_support_size", "mconv_valid_size", "mcorr_support_size", "mcorr_valid_size",
               "mcorr1d", "MCorr1d", "mcorrlcorr", "MCorrLCorr", "snd2col", "spec2col"]
    for name in ref_all:
        assert name in mconv.__all__ and hasattr(mconv, name)


@pytest.mark.parametrize("name", SIZE_FUNCS)
def test_size_functions_equal_checker(name):
    g = torch.Generator().manual_seed(3)
    fn, ofn = getattr(mconv, name + "_size"), getattr(oracle, name + "_size")
    for _ in range(2000):
        nf, ng = int(torch.randint(1, 20, (1,), generator=g)), int(torch.randint(1, 900, (1,), generator=g))
        s, d, u = (int(v) for v in torch.randint(1, 6, (3,), generator=g))
        p = int(torch.randint(0, 6, (1,), generator=g))
        assert fn(nf, ng, s, d, p, u) == ofn(nf, ng, s, d, p, u), (name, nf, ng, s, d, p, u)


def test_size_values_of_benchmark_configs():
    # output lengths of the reference's benchmark configurations, worked out by hand from mconv.py:73-118
    assert mconv.mcorr_valid_size(16, 256) == 16 and mconv.mconv_valid_size(16, 256) == 256
    grid = [(s, d, p) for s in (1, 2) for d in (1, 2) for p in (0, 3)]
    assert [mconv.mcorr_valid_size(8, 780, s, d, p) for s, d, p in grid] == [97, 390, 86, 346, 96, 389, 85, 345]
    assert [mconv.lcorr_valid_size(8, 780, s, d, p) for s, d, p in grid] == [773, 776, 766, 769, 387, 388, 383, 385]
    assert (mconv.mcorr_valid_size(8, 512), mconv.lcorr_valid_size(4, 41)) == (64, 38)
    assert (mconv.lcorr_valid_size(3, 256, 1, 2, 2), mconv.lcorr_valid_size(3, 41, 1, 1, 1)) == (254, 40)


def test_timing_tool_counts_the_taps_that_exist():
    """time_layers.py prices a pass by (output position, filter tap) pairs inside the input:
    cfg3 has 512 such pairs on the Mellin axis and 152 on the linear one (64 x 8 and 38 x 4:
    every tap of a valid-size output exists), config 2 the multiply counts of its (s, d, p) grid."""
    import time_layers
    assert time_layers.tap_pairs(hip.AX_MCORR, 8, 512, 64, 1, 1, 0) == 512
    assert time_layers.tap_pairs(hip.AX_LCORR, 4, 41, 38, 1, 1, 0) == 152
    grid = [(s, d, p) for s in (1, 2) for d in (1, 2) for p in (0, 3)]
    gmac = [32 * 128 * 41 * time_layers.tap_pairs(hip.AX_MCORR, 8, 780, mconv.mcorr_valid_size(8, 780, s, d, p), s, d, p) / 1e9
            for s, d, p in grid]
    assert [round(v, 3) for v in gmac] == [0.130, 0.262, 0.116, 0.232, 0.129, 0.261, 0.114, 0.232]
    brute = sum(1 for h in range(20) for f in range(5) if (3 * h + 2 * f - 4) >= 0 and (3 * h + 2 * f - 4) < 30)
    assert time_layers.tap_pairs(hip.AX_LCORR, 5, 30, 20, 3, 2, 4) == brute


def test_argument_errors_have_reference_wording():
    w = torch.zeros(4, 3, 5)
    with pytest.raises(RuntimeError, match=r"Expected 3-dimensional arg\[0\], but got 4-dimensional tensor "
                                           r"for argument #1 'input' \(while checking arguments for mcorr1d\)"):
        mconv.mcorr1d(torch.zeros(2, 3, 9, 1), w)
    with pytest.raises(RuntimeError, match=r"Expected tensor to have size 3 at dimension 1, but got size 2 "
                                           r"for argument #1 'input'"):
        mconv.mcorr1d(torch.zeros(2, 2, 9), w)
    with pytest.raises(RuntimeError, match=r"Expected tensor to have size 4 at dimension 0, but got size 5 "
                                           r"for argument #3 'bias'"):
        mconv.mcorr1d(torch.zeros(2, 3, 9), w, torch.zeros(5))
    with pytest.raises(RuntimeError, match="either an integer or a tuple of 2 integers"):
        mconv.mcorrlcorr(torch.zeros(1, 3, 9, 9), torch.zeros(4, 3, 2, 2), None, s=(1, 2, 3))
    with pytest.raises(NotImplementedError, match='_impl "fft" not supported'):
        mconv.mcorr1d(torch.zeros(2, 3, 9), w, _impl="fft")


def test_cpu_tensors_are_refused_loudly():
    with pytest.raises(RuntimeError, match="no CPU path"):
        mconv.mcorr1d(torch.zeros(2, 3, 9), torch.zeros(4, 3, 5))
    with pytest.raises(RuntimeError, match="no CPU path"):
        mconv.MCorrLCorr(3, 4, (2, 2))(torch.zeros(1, 3, 9, 9))


def test_layers_keep_reference_parameter_layout():
    torch.manual_seed(0)
    m = mconv.MCorrLCorr(3, 64, (8, 4), p=(3, 1), r=(0, 2), bias=True)
    assert list(m.state_dict()) == ["weight", "bias"]
    assert m.weight.shape == (64, 3, 8, 4) and m.bias.shape == (64,)
    bound = (3 * 8 * 4) ** -0.5          # U(+-1/sqrt(fan_in)), mconv.py:1062-1067
    assert float(m.weight.abs().max()) <= bound and float(m.bias.abs().max()) <= bound
    assert float(m.weight.abs().max()) > 0.9 * bound
    assert (m.s, m.d, m.p, m.r) == ((1, 1), (1, 1), (3, 1), (0, 2))
    m1 = mconv.MCorr1d(5, 7, 3, bias=False)
    assert m1.bias is None and m1.weight.shape == (7, 5, 3) and m1.s == (1,)
    assert "kernel_size=" in repr(m)


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mellin_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    names = set(re.findall(r"\b(mellin_[a-z0-9_]+)\s*\(", text))
    names |= set(re.findall(r"MELLIN_DECL_(?:1D|2D|SND|SPEC)\((mellin_[a-z0-9_]+)\s*,", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 23, names
    lib = ctypes.CDLL(hip.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), "libmellin_hip.so lacks %s" % n
    assert set(hip.SYMBOLS) == set(names)
    assert lib.mellin_version() >= 100


def test_cabi_rejects_bad_arguments_before_launch():
    lib = hip.lib
    dims_ok = [1, 1, 1, 2, 2, 4, 4, 2, 3] + [1, 1, 1, 1, 0, 0, 1, 1]
    null = ctypes.c_void_p(0)
    # kind_x must be a correlation kind
    assert lib.mellin_corr2d_forward_f32(hip.AX_MCONV, null, null, null, *dims_ok, null, null) == 1
    assert "kind_x" in hip.last_error()
    bad = list(dims_ok)
    bad[9] = 0                                          # sx = 0
    assert lib.mellin_corr2d_forward_f32(hip.AX_MCORR, null, null, null, *bad, null, null) == 1
    assert "s, d and u must be >= 1" in hip.last_error()
    bad = list(dims_ok)
    bad[13] = -1                                        # px = -1 on the Mellin axis
    assert lib.mellin_corr2d_forward_f32(hip.AX_MCORR, null, null, null, *bad, null, null) == 1
    assert "p must be >= 0" in hip.last_error()
    # null pointers with non-empty sizes
    assert lib.mellin_corr2d_forward_f32(hip.AX_MCORR, null, null, null, *dims_ok, null, null) == 1
    assert "null pointer" in hip.last_error()
    # empty problems are fine and launch nothing
    empty = list(dims_ok)
    empty[0] = 0
    assert lib.mellin_corr2d_forward_f32(hip.AX_MCORR, null, null, null, *empty, null, null) == 0
    assert lib.mellin_set_variant(b"no-such-variant") == 1
    assert lib.mellin_set_variant(b"") == 0


def test_workspace_queries_are_bounded_and_overflow_safe():
    """No form of the input gradient asks for more than 1 GiB of scratch memory (layers that
    would run in the workspace-free gather form), the weight gradient's partial sums stay
    small, and sizes whose product wraps to zero in 64 bits are not mistaken for empty."""
    import random
    cap = 1 << 30
    # the layers that once asked for 773 GB and 5 GB
    big = [(hip.AX_LCORR, 100, 15, 64, (33, 3), (780, 5000), (748, 4998)),
           (hip.AX_MCORR, 100, 15, 64, (33, 3), (780, 5000), (23, 4998)),
           (hip.AX_LCORR, 64, 8, 64, (16, 3), (2000, 80), (1985, 78))]
    rnd = random.Random(5)
    for _ in range(300):
        nf = (rnd.randint(1, 40), rnd.randint(1, 8))
        ng = (rnd.randint(nf[0], 4000), rnd.randint(nf[1], 600))
        big.append((rnd.choice([hip.AX_LCORR, hip.AX_MCORR]), rnd.randint(1, 256), rnd.randint(1, 40),
                    rnd.randint(1, 300), nf, ng, (rnd.randint(1, ng[0]), rnd.randint(1, ng[1]))))
    for kind, n, c_in, c_out, nf, ng, nh in big:
        dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
        assert hip.lib.mellin_corr2d_backward_input_workspace(kind, 4, *dims) <= cap, (kind, dims)
        assert hip.lib.mellin_corr2d_backward_weight_workspace(kind, 4, *dims) <= cap, (kind, dims)
    # extents whose nine-fold product wraps to zero in 64 bits: not an empty layer (an empty
    # layer returns MELLIN_OK without looking at the pointers)
    dims = hip._dims(1 << 16, 1 << 16, 1 << 16, (1, 1), (1 << 16, 1), (1 << 16, 1), (1, 1), (1, 1), (0, 0), (1, 1))
    code = hip.lib.mellin_corr2d_backward_weight_f32(hip.AX_LCORR, None, None, *dims, None, None, 0, None)
    assert code == 1 and "null pointer" in hip.last_error()
    # tensors of 2^60 elements or more are refused outright
    dims = hip._dims(1 << 20, 1 << 20, 1, (1, 1), (1 << 30, 1), (1 << 30, 1), (1, 1), (1, 1), (0, 0), (1, 1))
    code = hip.lib.mellin_corr2d_backward_weight_f32(hip.AX_LCORR, None, None, *dims, None, None, 0, None)
    assert code == 1 and "2^60" in hip.last_error()
    dims = hip._dims(1 << 21, 1, 1, (1, 1), (4, 4), (4, 4), (1, 1), (1, 1), (0, 0), (1, 1))
    code = hip.lib.mellin_corr2d_forward_f32(hip.AX_LCORR, None, None, None, *dims, None, None)
    assert code == 1 and "2^20" in hip.last_error()


def test_traffic_data_file_agrees_with_the_profile_summary():
    """bench.py's roofline.traffic comes from profiles/bench_cfg3_hbm_bytes.json; every total in it is
    a row of the committed profiler summary it names, to the summary's 0.1 MB, with the same kernel
    variant and math mode."""
    import json
    import bench
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(bench.TRAFFIC_FILE) as f:
        data = json.load(f)
    rows = {}
    with open(os.path.join(root, data["source"])) as f:
        for line in f:
            cells = [c.strip() for c in line.split("|")]
            if len(cells) > 8 and cells[1] in data["passes"] and cells[4].count("kernel"):
                rows[cells[1]] = cells
    assert set(rows) == set(data["passes"]) and len(rows) == 6
    for name, e in data["passes"].items():
        cells = rows[name]
        assert (cells[2], cells[3]) == (e["variant"], e["math"])
        assert abs(float(cells[5]) - e["read_bytes"] / 1e6) <= 0.11
        assert abs(float(cells[6]) - e["written_bytes"] / 1e6) <= 0.11
        assert abs(float(cells[7]) - e["bytes"] / 1e6) <= 0.21
        assert bench.measured_traffic(name, e["variant"], e["math"]) == e["bytes"]
        assert bench.measured_traffic(name, "generic", e["math"]) is None
