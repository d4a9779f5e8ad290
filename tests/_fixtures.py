"""Access to the reference's known-answer tables (tests/golden/reference_fixtures.json).

The tables were read from the reference's c/tests/test_*_buffers.h by
tests/golden/make_fixtures.py.  The helpers here lay the operands out the way
the reference's test mains do (c/tests/test_utils_cpu.h:10-94): the filter is
stored (c_out, c_in, n) or (c_in, c_out, n); signal and expected output are
tiled across the batch, optionally stored channel-major, and the expected
output is cut or zero-extended by ``extra`` elements per output axis.
"""
import json
import os

import numpy as np

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                     "reference_fixtures.json")
with open(_PATH) as _fp:
    TABLES = json.load(_fp)


def num_cases(name):
    return TABLES[name]["num_tests"]


def case(name, idx):
    """Parameters of one table row as a dict with 2-D style keys.

    1-D Mellin tables map onto the x axis, 1-D linear tables onto the y axis,
    the other axis being the unit axis (n=1, s=d=u=1, p=0), which is how
    c/tests/test_mcorrlcorr.cc:33-57 feeds them to the 2-D kernels.
    """
    t = TABLES[name]
    out = {"name": name, "idx": idx}
    if "kNFX" in t:
        for k2, k in (("nfx", "kNFX"), ("nfy", "kNFY"), ("ngx", "kNGX"), ("ngy", "kNGY"),
                      ("sx", "kSX"), ("sy", "kSY"), ("dx", "kDX"), ("dy", "kDY"),
                      ("px", "kPX"), ("py", "kPY"), ("ux", "kUX"), ("uy", "kUY")):
            out[k2] = t[k][idx]
    else:
        linear = name in ("lconv1d", "lcorr1d", "lin2col", "col2lin")
        a, b = ("y", "x") if linear else ("x", "y")
        out.update({"nf" + a: t["kNF"][idx], "ng" + a: t["kNG"][idx],
                    "s" + a: t["kS"][idx], "d" + a: t["kD"][idx],
                    "p" + a: t["kP"][idx], "u" + a: t["kU"][idx],
                    "nf" + b: 1, "ng" + b: 1, "s" + b: 1, "d" + b: 1, "p" + b: 0, "u" + b: 1})
    out["c_in"] = t["kCIn"][idx]
    out["c_out"] = t["kCOut"][idx] if "kCOut" in t else None
    out["F"] = np.asarray(t["kF"][idx], dtype=np.float64) if "kF" in t else None
    out["G"] = np.asarray(t["kG"][idx], dtype=np.float64)
    out["H"] = np.asarray(t["kH"][idx], dtype=np.float64)
    return out


def _padded(vals, n):
    """C array initialisers list only the leading values; the rest are zero."""
    out = np.zeros(n, dtype=np.float64)
    k = min(n, len(vals))
    out[:k] = vals[:k]
    return out


def filter_array(c, transposed=False):
    f = _padded(c["F"], c["c_out"] * c["c_in"] * c["nfx"] * c["nfy"])
    f = f.reshape(c["c_out"], c["c_in"], c["nfx"], c["nfy"])
    return np.ascontiguousarray(np.swapaxes(f, 0, 1)) if transposed else f


def tiled(vals, batch, chans, nx, ny, extra_x=0, extra_y=0, transposed=False):
    """(batch, chans, nx+extra_x, ny+extra_y) [or (chans, batch, ...)] from one (chans, nx, ny) table."""
    one = _padded(vals, chans * nx * ny).reshape(chans, nx, ny)
    ox, oy = nx + extra_x, ny + extra_y
    out = np.zeros((chans, ox, oy), dtype=np.float64)
    out[:, :min(nx, ox), :min(ny, oy)] = one[:, :min(nx, ox), :min(ny, oy)]
    out = np.broadcast_to(out, (batch,) + out.shape)
    return np.ascontiguousarray(np.swapaxes(out, 0, 1) if transposed else out)
