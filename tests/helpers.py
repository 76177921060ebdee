"""Shared helpers of the parity tests: product object -> oracle spec, tolerance check."""
import numpy as np
import torch

from oracle import tensor_product as otp

ATOL, RTOL = 1e-4, 1e-5  # fp32 contraction / spherical-harmonics tolerance of the benchmark definition


def oracle_spec(tp, user_path_weights=None, **norm_kw):
    """Oracle spec rebuilt from the *raw* constructor arguments of a product TensorProduct.

    Path weights are recomputed by the oracle, so a normalisation bug in the product
    shows up as a mismatch rather than being copied over."""
    upw = user_path_weights or [1.0] * len(tp.instructions)
    ins = [(t.i_in1, t.i_in2, t.i_out, t.connection_mode, t.has_weight, pw) for t, pw in zip(tp.instructions, upw)]
    return otp.make_spec(str(tp.irreps_in1), str(tp.irreps_in2), str(tp.irreps_out), ins, shared_weights=tp.shared_weights, **norm_kw)


ERROR_LOG = []  # one row per comparison against the oracle: printed and written out when the session ends


def record_errors(what, got, ref, atol, rtol):
    """Raw error figures of one comparison: max abs error, max error relative to the largest reference magnitude,
    max element-wise relative error over the entries with |ref| >= 1e-3 max|ref|, and the worst ratio of the error
    to the tolerance (<= 1 passes)."""
    err = np.abs(got - ref)
    scale = float(np.abs(ref).max())
    big = np.abs(ref) >= 1e-3 * scale if scale > 0 else np.zeros(ref.shape, bool)
    row = {
        "what": what, "n": int(ref.size), "max_abs_err": float(err.max()), "max_abs_ref": scale,
        "max_err_over_max_ref": float(err.max() / scale) if scale > 0 else 0.0,
        "max_rel_err": float((err[big] / np.abs(ref[big])).max()) if big.any() else 0.0,
        "worst_err_over_tol": float((err / (atol + rtol * np.abs(ref))).max()), "atol": atol, "rtol": rtol,
    }  # fmt: skip
    ERROR_LOG.append(row)
    return row


def assert_close(got, ref, atol=ATOL, rtol=RTOL, what=""):
    got = got.detach().float().cpu().numpy().astype(np.float64) if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    if got.size == 0:
        return
    err = np.abs(got - ref)
    record_errors(what, got, ref, atol, rtol)
    bad = err > atol + rtol * np.abs(ref)
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} entries off, max abs err {err.max():.3e} (atol {atol}, rtol {rtol})"


def seeded(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale
