"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must keep reproducing them, and the HIP path must match them."""
import glob
import os

import numpy as np
import pytest

import lowbit_oracle as orc

FILES = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "lowbit_*.npz")))


def test_five_fixtures_present():
    assert len(FILES) == 5


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_oracle_reproduces_fixture(path):
    f = np.load(path)
    qtype = int(f["qtype"])
    blob = orc.quantize(f["w"], qtype)
    assert np.array_equal(blob, f["blob"])
    assert np.array_equal(orc.dequantize(blob, qtype, f["w"].shape), f["dequant"])
    assert np.array_equal(orc.mul_mat_exact(blob, f["x"], f["w"].shape, qtype), f["y_exact"])
    assert np.array_equal(orc.mul_mat_q(blob, f["x"], f["w"].shape, qtype), f["y_ggml"])


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_hip_matches_fixture(path):
    import torch
    from gpu_util import dev_dequantize, dev_matmul, dev_quantize, dev_relayout
    f = np.load(path)
    qtype = int(f["qtype"])
    n, k = f["w"].shape
    g = dev_quantize(f["w"], qtype, 0)
    assert np.array_equal(g.cpu().numpy(), f["blob"])
    t = dev_quantize(f["w"], qtype, 1)
    assert np.array_equal(dev_relayout(t, qtype, n, k, 1).cpu().numpy(), f["blob"])
    assert np.array_equal(dev_dequantize(t, qtype, n, k, 1, torch.float32).cpu().numpy(), f["dequant"])
    x = torch.from_numpy(f["x"]).half()
    for fn in ("gemv", "gemm"):
        y = dev_matmul(x, t, qtype, 1, n, fn=fn)
        assert np.abs(y - f["y_exact"]).max() <= 2e-3 * np.abs(f["y_exact"]).max()
        assert np.abs(y - f["y_ggml"]).max() <= 1e-2 * np.abs(f["y_ggml"]).max()
