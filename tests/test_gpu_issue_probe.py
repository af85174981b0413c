"""The calibration probe bench.py prices the decoder's instruction count with: it must run, end,
and report figures in the range this GPU family can produce (a wave64 instruction takes a SIMD
between 2 and 4 cycles; the engine clock lies between 0.5 and 3 GHz)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_issue_rate_classes_and_clock():
    from cachegen_amd import issue_probe
    torch.zeros(1, device="cuda:0")
    cal = issue_probe.calibrate(iters=256)
    for name in ("cheap", "full", "decoder_symbol"):
        assert 500.0 < cal[name]["clock_mhz"] < 3000.0, cal
        assert 1.5 < cal[name]["cycles_per_instruction"] < 5.0, cal
    assert cal["cheap"]["cycles_per_instruction"] < cal["full"]["cycles_per_instruction"]


def test_clock_window_ends_and_reports():
    from cachegen_amd import issue_probe
    side = torch.cuda.Stream()
    issue_probe.clock_window_start(2000, side.cuda_stream)
    x = torch.randn(2048, 2048, device="cuda:0")
    for _ in range(10):
        x = (x @ x).clamp(-1, 1)
    torch.cuda.synchronize()
    mhz, us = issue_probe.clock_window_result()
    assert 1900.0 <= us < 200000.0 and 500.0 < mhz < 3000.0
