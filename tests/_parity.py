"""Shared helpers for the GPU parity tests."""
import numpy as np

from oracle import binding as orc

REL_TOL = 1e-4          # the path's stated fp32 bound (accumulation order only)
CANCEL_FLOOR = 1 / 64   # outputs smaller than this fraction of their summed term magnitudes are
                        # judged against that fraction instead (cancellation makes |ref| arbitrarily small)


def assert_fp32_parity(got: np.ndarray, ref: np.ndarray, mag: np.ndarray, what: str = "") -> float:
    """|got - ref| <= 1e-4 * max(|ref|, mag/64) element-wise; returns the largest plain relative
    error over the well-conditioned outputs (|ref| >= mag/64) for reporting."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    mag = np.asarray(mag, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    err = np.abs(got - ref)
    scale = np.maximum(np.abs(ref), mag * CANCEL_FLOOR)
    worst = np.max(err / np.maximum(scale, 1e-300))
    assert worst <= REL_TOL, f"{what}: max relative error {worst:.3e} > {REL_TOL}"
    ok = np.abs(ref) >= mag * CANCEL_FLOOR
    ok &= ref != 0          # ref == mag == 0 (an all-zero row): nothing to divide by
    return float(np.max(err[ok] / np.abs(ref[ok]))) if ok.any() else 0.0


def oracle_all_orders(w: np.ndarray, cols: int, q8: np.ndarray):
    return {name: orc.mul_mat_q4k_q8k(w, cols, q8, order) for name, order in orc.ORDERS.items()}
