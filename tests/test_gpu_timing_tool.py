"""The layer-timing tool runs every pass through the C ABI on the matrix-core kernels and
prints one JSON record per layer (the 1-D grid of config 2: sixteen layers, a second or so)."""
import json

import pytest
import torch

import time_layers

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["float32", "half"])
def test_config2_grid_runs_on_the_matrix_core_kernels(capsys, dtype):
    time_layers.run_cfg2(reps=1, dtype=dtype)
    records = [json.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert len(records) == 16
    t_out = {(r["layer"].split()[1], r["layer"].split(" ", 2)[2]): r["out"][1] for r in records}
    assert t_out[("mcorr1d", "s=1 d=1 p=0")] == 97 and t_out[("lcorr1d", "s=2 d=2 p=3")] == 385
    for r in records:
        assert r["in"] == [41, 780, 1] and r["out"][0] == 128
        for name in ("forward", "grad_input", "grad_weight"):
            assert r[name]["variant"].startswith("mfma"), r
            assert (r[name]["math"] == "f16") == (dtype == torch.float16), r
            assert r[name]["us"] > 0 and r[name]["tflops"] > 0
