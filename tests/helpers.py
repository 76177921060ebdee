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


def assert_close(got, ref, atol=ATOL, rtol=RTOL, what=""):
    got = got.detach().float().cpu().numpy().astype(np.float64) if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    if got.size == 0:
        return
    err = np.abs(got - ref)
    bad = err > atol + rtol * np.abs(ref)
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} entries off, max abs err {err.max():.3e} (atol {atol}, rtol {rtol})"


def seeded(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale
