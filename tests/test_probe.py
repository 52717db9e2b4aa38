"""The MFMA-rate probe behind `bench.py --mfma-probe` runs and reports a rate per kind of operand data
(a diagnostic: nothing is asserted about the rates themselves, which depend on the box)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_mfma_probe_reports_rates(dev):
    import bench

    out = bench.mfma_probe(torch.float16, torch.device(dev), iters=2000)
    rates = out["tflops"]
    assert set(rates) == {"all ones", "uniform in [-1, 1]", "normal, std 0.02 (weights)", "normal, std 1"}
    assert all(r > 0.0 for r in rates.values())
