"""Shared helpers for the parity tests."""
import numpy as np

# Required tolerance: max relative error <= 1e-3 against the f32-accumulated reference, in the
# reference's own form max|delta| / max|y_ref| (forward/metal_qwen35.rs:23615-23623).
REL_TOL = 1e-3


def rel_err(got, ref) -> float:
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(got - ref)
    if not np.all(np.isfinite(d)):  # NaN-honest, as max_abs_diff in metal_qwen35.rs:22904-22916
        return float("inf")
    denom = np.max(np.abs(ref))
    return float(np.max(d) / denom) if denom > 0 else float(np.max(d))
