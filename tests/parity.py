"""Comparison helpers shared by the parity tests."""
import numpy as np

# Tolerances of the parity contract:
#   bit-exact ............ index / permute / concat / comparison outputs, integer-valued programs
#   ELW_RTOL ............. element-wise chains (relative; at least |ref|_max * ELW_RTOL absolute, because a
#                          fused chain that ends in a subtraction cannot be relatively exact near zero)
#   RED_RTOL * sqrt(N) ... anything that went through a reduction or a matmul over N terms
ELW_RTOL = 1e-6
RED_RTOL = 1e-5


def assert_exact(got, ref, what=""):
    got = np.asarray(got, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    same = (got == ref) | (np.isnan(got) & np.isnan(ref))
    assert same.all(), f"{what}: {np.count_nonzero(~same)} of {got.size} elements differ, first at {np.argwhere(~same)[0]}"


def assert_close(got, ref, rtol, what="", scale=None):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    if got.size == 0:
        return
    finite = np.isfinite(ref)
    assert (np.isfinite(got) == finite).all(), f"{what}: non-finite pattern differs"
    if not finite.any():
        return
    s = float(np.max(np.abs(ref[finite]))) if scale is None else float(scale)
    tol = rtol * np.maximum(np.abs(ref), s if s > 0 else 1.0)
    err = np.abs(got - ref)
    bad = finite & (err > tol)
    assert not bad.any(), (f"{what}: {np.count_nonzero(bad)} of {got.size} elements beyond tolerance {rtol:g}; "
                           f"worst |err|={err[finite].max():.3e} at ref={ref.flat[np.argmax(np.where(finite, err, 0))]:.6e}")


def compare_outputs(got: dict, ref: dict, rules: dict, default):
    """rules: name -> ("exact",) | ("close", rtol); default likewise."""
    for k, rv in ref.items():
        gv = got[k]
        assert not gv.is_none, f"{k}: device returned none"
        assert gv.dim == rv.dim, f"{k}: dim {gv.dim} vs {rv.dim}"
        rule = rules.get(k, default)
        if rule[0] == "exact":
            assert_exact(gv.data, rv.data, k)
        else:
            assert_close(gv.data, rv.data, rule[1], k)
