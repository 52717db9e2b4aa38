"""The MFMA-rate probe behind `bench.py --mfma-probe` runs and reports plausible rates."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_mfma_probe_reports_rates(dev):
    import bench

    out = bench.mfma_probe(torch.float16, torch.device(dev), iters=2000)
    rates = out["tflops"]
    assert set(rates) == {"all ones", "uniform in [-1, 1]", "normal, std 0.02 (weights)", "normal, std 1"}
    # between a tenth of and the full published dense fp16 peak; constant operands are never slower than random ones
    assert all(250.0 < r < 2600.0 for r in rates.values())
    assert rates["all ones"] >= 0.95 * rates["normal, std 1"]
