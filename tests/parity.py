"""The floating-point parity bar of the distance and fused paths, in one place.

Contract: the k-th-neighbour distance within 1e-5 relative of the reference arithmetic's (the CPU
oracle: sequential fused multiply-adds, reference include/bits/distance/abstract_gemm.cuh:139-169)
and recall@k >= 0.999.  The kernels report the partial distance v = ||p||^2 - 2 q.p; the distance
itself is v + ||q||^2.  Three measures of the k-th neighbour's error, strictest first:

  completed   |v_gpu - v_ref| / (v_ref + ||q||^2)   relative to the distance itself.  Asserted for
              dim >= 16.  Below that fp32 cannot meet it whatever the order of the operations: the
              distance of a near neighbour among many points is far smaller than ||p||^2, whose
              last bit alone exceeds 1e-5 of it (dim = 8, 2^20 points: distance ~ 0.05, ||p||^2 ~
              2.7), and the oracle's own fp32 result is that far from the exact value.
  of_value    |v_gpu - v_ref| / |v_ref|             relative to the reported value.  Asserted for
              dim < 16, except where the reported value is itself the small difference of its two
              terms (||p||^2 close to 2 q.p): there the bound is 2^-20 of the scale below, 16 units
              in the last place of the terms, which is what fp32 can resolve.
  of_scale    |v_gpu - v_ref| / (|v_ref| + ||q||^2) relative to the terms that cancel.  Always
              asserted.
"""
import numpy as np

REL = 1e-5
MIN_RECALL = 0.999
STRICT_FROM_DIM = 16

# the largest errors seen by assert_kth_distance per (dim class), for the record (pytest -s prints
# them at the end of the session)
margins = {}


RESOLUTION = 2.0 ** -20  # of the scale of the cancelling terms: 16 units in the last place


def kth_errors(queries, exp_kth, got_kth):
    """Largest error of each kind over the queries; of_value skips the queries whose error is
    within RESOLUTION of the scale (the value is a small difference of its terms there)."""
    qn = (queries.astype(np.float64) ** 2).sum(1)
    e = exp_kth.astype(np.float64)
    g = got_kth.astype(np.float64)
    finite = np.isfinite(e) & np.isfinite(g)
    if not finite.any():
        return 0.0, 0.0, 0.0
    e, g, qn = e[finite], g[finite], qn[finite]
    scale = np.abs(e) + qn
    diff = np.abs(g - e)
    with np.errstate(divide="ignore", invalid="ignore"):
        completed = np.where(e + qn > 0, diff / (e + qn), 0.0)
        of_scale = np.where(scale > 0, diff / scale, 0.0)
        of_value = np.where((of_scale <= RESOLUTION) | (diff == 0), 0.0, diff / np.abs(e))
        of_value = np.maximum(of_value, np.where(np.abs(e) > 0, np.minimum(diff / np.abs(e), REL), 0.0))
    return float(completed.max()), float(of_value.max()), float(of_scale.max())


def assert_kth_distance(queries, exp_kth, got_kth, dim, what=""):
    """The k-th neighbour distances `got_kth` (partial distances, one per query) against the
    oracle's `exp_kth`, to the bar described in the module docstring."""
    completed, of_value, of_scale = kth_errors(queries, exp_kth, got_kth)
    key = "dim>=16" if dim >= STRICT_FROM_DIM else "dim<16"
    seen = margins.setdefault(key, {"completed": 0.0, "of_value": 0.0, "of_scale": 0.0})
    seen["completed"] = max(seen["completed"], completed)
    seen["of_value"] = max(seen["of_value"], of_value)
    seen["of_scale"] = max(seen["of_scale"], of_scale)
    assert of_scale <= REL, (what, "of_scale", of_scale)
    if dim >= STRICT_FROM_DIM:
        assert completed <= REL, (what, "completed distance", completed)
    else:
        assert of_value <= REL, (what, "of_value", of_value)
    return completed, of_value, of_scale
