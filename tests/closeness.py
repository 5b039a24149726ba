"""Closeness bars shared by the GPU parity tests.

A bar scaled by the largest element of the expected tensor says nothing about what an ordinary element may
be off by, so every bar here is scaled by the root mean square of the expected tensor and comes with a bound
on the mean error.
"""

import torch


def _f64(t):
    return t.detach().float().cpu().double() if t.dtype != torch.float64 else t.detach().cpu()


def half_close(got, want, what="", atol_rms=4e-2, mean_rms=3e-3, rtol=2e-2):
    """16-bit operands against a float64 (or float32) result: every element within ``rtol`` of itself or
    ``atol_rms`` of the result's root mean square, and the mean error an order of magnitude below that."""
    got, want = _f64(got), _f64(want)
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} against {tuple(want.shape)}"
    rms = float(want.pow(2).mean().sqrt()) + 1e-30
    err = (got - want).abs()
    torch.testing.assert_close(got, want, rtol=rtol, atol=atol_rms * rms,
                               msg=lambda m: f"{what}: {m} (max err / rms {float(err.max()) / rms:.3e}, "
                                             f"mean err / rms {float(err.mean()) / rms:.3e})")
    assert float(err.mean()) <= mean_rms * rms, f"{what}: mean err / rms {float(err.mean()) / rms:.3e}"


def fp32_close(got, want64, oracle32=None, what="", rtol=1e-5, atol_rms=1e-5, arbitration=4.0):
    """A float32 result against the float64 value of the same formula: every element within ``rtol`` of
    itself or ``atol_rms`` of the result's root mean square.  An element outside that bar still passes when
    a float32 evaluation on the CPU (``oracle32``) is off the float64 value by a comparable amount there:
    the error of ``got`` may be at most ``arbitration`` times the largest error of ``oracle32`` (both are
    float32 sums of the same terms in different orders, and neither is the truth)."""
    got, want = _f64(got), _f64(want64)
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} against {tuple(want.shape)}"
    rms = float(want.pow(2).mean().sqrt()) + 1e-30
    err = (got - want).abs()
    bar = atol_rms * rms + rtol * want.abs()
    if oracle32 is not None:
        ref_err = (_f64(oracle32) - want).abs()
        bar = torch.maximum(bar, torch.full_like(bar, arbitration * float(ref_err.max())))
    bad = err > bar
    assert not bool(bad.any()), (f"{what}: {int(bad.sum())} of {bad.numel()} elements outside the bar; "
                                 f"max err / rms {float(err.max()) / rms:.3e}, "
                                 f"mean err / rms {float(err.mean()) / rms:.3e}")
