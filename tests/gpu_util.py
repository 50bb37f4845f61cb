"""Helpers for the GPU parity tests: a session Context and tolerance checks.

Tolerances (stated once, used by every GPU test), e = oracle value, a = GPU value:
  f32 kernels   : |a - e| <= 1e-4 * |e| + 1e-4 * rms(e) for every element
                  ("rtol 1e-4"; an element near zero is measured against the tensor's RMS
                  instead of its own magnitude)
  bf16 kernels  : |a - e| <= 2e-2 * |e| + 2e-2 * rms(e)   ("rtol 2e-2 on gradients")
                  for all but at most 1e-4 of the elements, never more than twice that bound,
                  and a relative L2 error ||a - e|| / ||e|| <= 1e-2.  The L2 bound is the
                  sharp one: it is what a systematic error (a dropped term, a wrong scale)
                  breaks; the per-element bound with a 1e-4 outlier allowance is what
                  independent bf16 roundings of 1e5-element tensors can actually meet.
  bf16 training step (many kernels composed; every stored activation adds a bf16 rounding, so the
                  error of a gradient grows with depth like independent roundings do):
                  relative L2 error of every gradient tensor <= 2e-2 and, per element,
                  |a - e| <= 2e-2 * |e| + 2e-2 * max|e|   (assert_close(..., step=True))
  integer/index : bit-exact
A test that widens one of these bounds passes the widened figure to assert_close (outliers, worst_cap, row_scale,
row_floor, step_outliers) and says why at the call; what every comparison of a run observed is printed at its end.
"""
import numpy as np
import pytest

RTOL_F32 = 1e-4
RTOL_BF16 = 2e-2


@pytest.fixture(scope="session")
def ctx():
    from eisen_amd import hip
    c = hip.Context(0)
    yield c
    c.close()


# Every assert_close call leaves its observed figures here; tests/conftest.py prints the worst per tolerance class at the
# end of the run, so the head-room (or lack of it) under the bounds above is visible in the test log.
OBSERVED = []


def _record(name, kind, rtol, a_size, rel_l2, frac_outside, worst_ratio):
    OBSERVED.append(dict(name=name, kind=kind, rtol=rtol, n=int(a_size), rel_l2=float(rel_l2), frac_outside=float(frac_outside),
                         worst_ratio=float(worst_ratio)))


def assert_close(actual, expected, rtol, name="", row_scale=False, l2=None, step=False, step_outliers=0.0, row_floor=0.0, outliers=1e-4, worst_cap=2.0):
    """step: the composed-step criterion above (scale = max|e| instead of rms(e), no outlier allowance,
    relative L2 <= rtol).  step_outliers: fraction of the elements that may exceed the step bound, by at most 4x -- only
    for comparisons of two bf16 results with each other (both sides carry rounding noise), never against the oracle.
    row_scale: take rms(e) per last-dim row instead of over the whole tensor -- for tensors whose
    rows differ by orders of magnitude (an embedding gradient: untouched rows are exactly zero, hot
    rows are large), where one global RMS is not the scale of any element; row_floor: with row_scale, a row's
    scale is never taken below this fraction of the tensor's RMS (for rows whose exact value is zero but whose
    computed value is a rounding residue).  outliers / worst_cap: the bf16-kernel allowance (fraction of the elements
    that may pass the per-element bound, and by how much at most); a test that widens them says why.  l2: bound on the
    relative L2 error for the bf16 check (default 1e-2).
    Every failure message carries the observed relative L2 error, the fraction of elements outside the
    per-element bound and the worst error as a multiple of that bound."""
    a = np.asarray(actual, np.float64)
    e = np.asarray(expected, np.float64)
    assert a.shape == e.shape, f"{name}: shape {a.shape} vs {e.shape}"
    assert np.isfinite(a).all(), f"{name}: non-finite values in the result"
    err = np.abs(a - e)
    den = float(np.sum(e * e))
    rel_l2 = float(np.sqrt(np.sum(err * err) / den)) if den > 0 else 0.0
    if step:
        scale_el = np.abs(e).max(axis=-1, keepdims=True) if (row_scale and e.ndim >= 2) else np.abs(e).max()
        tol = rtol * np.abs(e) + rtol * scale_el + 1e-30
        ratio = err / tol
        frac = float((ratio > 1).mean()) if a.size else 0.0
        worst = float(ratio.max()) if a.size else 0.0
        _record(name, "bf16 step", rtol, a.size, rel_l2, frac, worst)
        seen = f"observed: relative L2 {rel_l2:.3g}, {frac:.3g} of the elements outside the bound, worst error {worst:.3g} x bound"
        if (ratio > 1).sum() > int(step_outliers * a.size) or worst > 4:
            i = int(np.argmax(ratio.reshape(-1)))
            raise AssertionError(f"{name}: {int((ratio > 1).sum())}/{a.size} elements outside the step bound; worst at {i}: "
                                 f"got {a.reshape(-1)[i]:.8g}, expected {e.reshape(-1)[i]:.8g}; {seen}")
        bound = rtol if l2 is None else l2
        assert rel_l2 <= bound, f"{name}: relative L2 error {rel_l2:.3g} > {bound:g}; {seen}"
        return
    if row_scale and e.ndim >= 2:
        rms_el = np.sqrt(np.mean(e * e, axis=-1, keepdims=True))
        if row_floor > 0.0:
            rms_el = np.maximum(rms_el, row_floor * np.sqrt(np.mean(e * e)))
        rms_el = np.broadcast_to(rms_el, e.shape).reshape(-1)
    else:
        rms_el = None
    a, e, err = a.reshape(-1), e.reshape(-1), err.reshape(-1)
    rms = float(np.sqrt(np.mean(e * e))) if e.size else 0.0
    tol = rtol * np.abs(e) + rtol * (rms_el if rms_el is not None else rms) + 1e-30
    ratio = err / tol
    bad = ratio > 1
    frac = float(bad.mean()) if a.size else 0.0
    worst = float(ratio.max()) if a.size else 0.0
    loose = rtol >= RTOL_BF16          # bf16: allow 1e-4 of the elements up to 2x the bound
    _record(name, "bf16 kernel" if loose else "f32 kernel", rtol, a.size, rel_l2, frac, worst)
    seen = f"observed: relative L2 {rel_l2:.3g}, {frac:.3g} of the elements outside the bound, worst error {worst:.3g} x bound"
    allowed = int(outliers * a.size) + 1 if loose else 0
    if bad.sum() > allowed or (loose and worst > worst_cap):
        i = int(np.argmax(ratio))
        raise AssertionError(f"{name}: {int(bad.sum())}/{a.size} elements outside rtol {rtol:g}; worst at {i}: "
                             f"got {a[i]:.8g}, expected {e[i]:.8g}, rms {rms:.4g}; {seen}")
    if loose and rms > 0:
        bound = 1e-2 if l2 is None else l2
        assert rel_l2 <= bound, f"{name}: relative L2 error {rel_l2:.3g} > {bound:g}; {seen}"


def tol_for(dtype):
    from eisen_amd import hip
    return RTOL_BF16 if dtype == hip.BF16 else RTOL_F32


def prep(x, dtype):
    """Input as the device will see it: bf16 inputs are rounded first so oracle and GPU start equal."""
    from eisen_amd import hip
    x = np.ascontiguousarray(x, dtype=np.float32)
    return hip.round_bf16(x) if dtype == hip.BF16 else x
