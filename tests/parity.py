"""The error bounds the GPU parity tests hold the linear operator to, by how the kernel that ran
treats the weights (sbvr.hip.last_rounding()).  yd0: the oracle's unrounded double sums with the
coefficients applied to plane sums (no per-weight rounding, mode 0); yd1: the same sums over
weights rounded to fp16 once, as the reference's decode() rounds them (mode 1).

  exact weights (decode kernels)   against yd0: 1e-2 relative with a floor of 1 % of the RMS
                                   output, and at most 2 fp16 ulps of max(|ref|, RMS);
  weights as decode() rounds them  the same two bounds against yd1 (what is left is the order of
  (table look-up kernels)          the fp32 additions and the one rounding of the output), and the
                                   bound of the line below against yd0;
  weights summed plane by plane    against yd0 and yd1: at most 3e-3 of the RMS output, 1e-2
  (arithmetic decode)              relative for outputs above 0.3 RMS.
"""
import numpy as np

ROUNDING_EXACT, ROUNDING_DECODE, ROUNDING_PLANEWISE = 1, 2, 3


def tight(got, yd, what, rms=None):
    got = np.asarray(got, dtype=np.float64)
    rms = (float(np.sqrt(np.mean(yd ** 2))) if rms is None else float(rms)) + 1e-30
    err = np.abs(got - yd)
    rel = (err / np.maximum(np.abs(yd), 1e-2 * rms)).max()
    assert rel <= 1e-2, f"{what}: relative error {rel:.3e} > 1e-2"
    ulp = (err / (np.maximum(np.abs(yd), rms) * 2.0 ** -10)).max()
    assert ulp <= 2.0, f"{what}: {ulp:.2f} fp16 ulps off"
    return ulp


def loose(got, yd, what, rms=None):
    got = np.asarray(got, dtype=np.float64)
    rms = (float(np.sqrt(np.mean(yd ** 2))) if rms is None else float(rms)) + 1e-30
    err = np.abs(got - yd)
    assert err.max() <= 3e-3 * rms + 2.0 ** -11 * np.abs(yd).max(), f"{what}: {err.max() / rms:.3e} of the RMS output"
    assert (err / np.maximum(np.abs(yd), 0.3 * rms)).max() <= 1e-2, what


def judge(got, yd0, yd1, rounding, what, rms=None):
    """rounding: sbvr.hip.last_rounding() of the call that produced `got`; yd1 may be None for exact weights."""
    if rounding == ROUNDING_EXACT:
        return tight(got, yd0, what, rms)
    assert yd1 is not None, "the oracle's decode()-rounded sums are needed for this kernel"
    loose(got, yd0, what + " (against unrounded weights)", rms)
    if rounding == ROUNDING_DECODE:
        return tight(got, yd1, what + " (against decode()-rounded weights)", rms)
    assert rounding == ROUNDING_PLANEWISE, f"unknown rounding {rounding}"
    return loose(got, yd1, what + " (against decode()-rounded weights)", rms)
