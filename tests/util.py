"""Shared helpers for the parity tests."""
import numpy as np

# north-star tolerance: max relative error 1e-2 (fp16 out, fp32 accumulate); the denominator is
# floored at 1e-2 * rms(ref) because outputs are sums of signed terms and cross zero.
REL_TOL = 1e-2
# the reference's own acceptance test: no element may differ by more than 0.5
# (spmm_benchmark.cpp:213, sddmm_benchmark.cpp:288)
REF_ABS_TOL = 0.5


def max_rel_err(got, ref):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    if ref.size == 0:
        return 0.0
    floor = REL_TOL * float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    denom = np.maximum(np.abs(ref), max(floor, 1e-30))
    return float(np.max(np.abs(got - ref) / denom))


def assert_parity(got, ref, what=""):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, "%s: shape %s vs %s" % (what, got.shape, ref.shape)
    assert np.all(np.isfinite(got)), "%s: non-finite output" % what
    errors = int(np.sum(np.abs(got - ref) > REF_ABS_TOL))
    assert errors == 0, "%s: %d elements differ by more than %.1f" % (what, errors, REF_ABS_TOL)
    err = max_rel_err(got, ref)
    assert err <= REL_TOL, "%s: max relative error %.3e > %.0e" % (what, err, REL_TOL)
    return err


def retired_variants_built():
    """True when the library was built with VS_RETIRED_VARIANTS=1 (the LDS-DMA gather and four steps in flight of the
    MFMA SpMM, which the default build leaves out): the option values that select them are then accepted."""
    from vectorsparse_amd import _lib
    L = _lib.lib()
    ok = L.vs_set_option(b"spmm_steps", 4) == 0
    L.vs_set_option(b"spmm_steps", 0)
    return ok
