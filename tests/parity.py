"""Parity measures shared by the GPU tests, smoke() and bench.py.

Contract (floating-point outputs of the fast kernels against the lane-order f32 reference):
  * relative L2 error  ||y - y_ref|| / ||y_ref||  <= 1e-3
  * max |y - y_ref| <= 4 f16 ulp of the output's magnitude.
    Near-zero outputs: an output that is small only because thousands of O(rms) terms cancelled carries the f32
    rounding noise of the *reference's own* summation (about 1e-6..1e-5 absolute at these shapes), so no kernel
    with a different summation order can match it to 4 ulp of its tiny magnitude.  The magnitude used for the ulp
    is therefore clamped from below at rms(y_ref)/128; the report also gives the unclamped ("strict") pass fraction
    and the number of outputs that needed the clamp.  The reference's own gate uses an absolute 1e-5 for its
    non-bit-exact kernel (crates/server/src/probes/w4a16/gates.rs:134-138).
"""
import numpy as np

REL_L2_TOL = 1e-3
ULP_TOL = 4.0
CLAMP_DIV = 128.0


def f16_ulp(mag):
    """Spacing of binary16 at magnitude `mag` (2^-24 in the subnormal range)."""
    mag = np.abs(np.asarray(mag, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(mag, 2.0 ** -14)))
    return np.ldexp(1.0, (e - 10).astype(np.int64))


def compare(y, y_ref):
    """Returns a dict of error measures; y and y_ref are float arrays of the same shape."""
    y = np.asarray(y, dtype=np.float64).ravel()
    r = np.asarray(y_ref, dtype=np.float64).ravel()
    d = np.abs(y - r)
    rms = float(np.sqrt(np.mean(r * r))) if r.size else 0.0
    rel_l2 = float(np.sqrt(np.sum(d * d)) / max(np.sqrt(np.sum(r * r)), 1e-300))
    strict = d / f16_ulp(r)
    clamped_mag = np.maximum(np.abs(r), rms / CLAMP_DIV)
    ulps = d / f16_ulp(clamped_mag)
    return {
        "rel_l2": rel_l2,
        "max_abs": float(d.max()) if d.size else 0.0,
        "max_ulp": float(ulps.max()) if d.size else 0.0,
        "max_ulp_strict": float(strict.max()) if d.size else 0.0,
        "strict_pass_frac": float(np.mean(strict <= ULP_TOL)) if d.size else 1.0,
        "clamped": int(np.sum(np.abs(r) < rms / CLAMP_DIV)),
        "count": int(d.size),
        "rms_ref": rms,
        "ulp_hist": np.histogram(ulps, bins=[0, 0.25, 0.5, 1, 2, 4, np.inf])[0].tolist(),
    }


def ok(m):
    return np.isfinite(m["rel_l2"]) and m["rel_l2"] <= REL_L2_TOL and m["max_ulp"] <= ULP_TOL


def assert_close(y, y_ref, what=""):
    m = compare(y, y_ref)
    assert ok(m), "%s parity: %r" % (what, m)
    return m
