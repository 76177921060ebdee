"""GPU parity: o3.spherical_harmonics (HIP, through the C ABI) against the CPU oracle and the golden values."""
import math

import numpy as np
import pytest
import torch

from e3nn_amd import o3
from oracle.spherical_harmonics import spherical_harmonics as osh
from tests.helpers import assert_close, seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("normalize", [True, False])
@pytest.mark.parametrize("normalization", ["integral", "component", "norm"])
def test_golden_points(golden_sh, normalize, normalization):
    pts = torch.from_numpy(golden_sh["points"]).float().to(DEV)
    ref = golden_sh[f"lmax8_{int(normalize)}_{normalization}"]
    # closed-form kernel, l <= 3
    got = o3.spherical_harmonics([0, 1, 2, 3], pts, normalize, normalization)
    pts64 = golden_sh["points"].astype(np.float32).astype(np.float64)
    ref32 = osh(list(range(9)), pts64, normalize, normalization)  # oracle on the fp32-rounded inputs
    assert_close(got, ref32[:, :16], what="l<=3")
    # recurrence kernel, l <= 8; un-normalised inputs grow like |x|^l, so the tolerance is relative there
    got = o3.spherical_harmonics(list(range(9)), pts, normalize, normalization)
    assert_close(got, ref32, atol=1e-4, rtol=1e-5 if normalize else 2e-5, what="l<=8")
    if normalize:
        assert_close(got, ref, atol=2e-4, rtol=1e-4, what="l<=8 vs reference golden")


@pytest.mark.parametrize("lmax", [0, 1, 2, 3])
@pytest.mark.parametrize("n", [1, 63, 64, 100_037])
def test_random_vectors_all_tile_shapes(lmax, n):
    x = seeded(n, 3, seed=lmax * 7 + 1)
    got = o3.spherical_harmonics(list(range(lmax + 1)), x.to(DEV), True, "component")
    assert_close(got, osh(list(range(lmax + 1)), x.numpy(), True, "component"), what=f"lmax {lmax} n {n}")
    got = o3.spherical_harmonics(list(range(lmax + 1)), x.to(DEV), False, "integral")
    assert_close(got, osh(list(range(lmax + 1)), x.numpy(), False, "integral"), rtol=2e-5, what=f"raw lmax {lmax} n {n}")


def test_selected_l_lists_and_batch_dims(golden_sh):
    x = seeded(5, 7, 3, seed=3)
    got = o3.spherical_harmonics([2, 0, 3], x.to(DEV), True, "component")
    assert got.shape == (5, 7, 13)
    assert_close(got, osh([2, 0, 3], x.numpy(), True, "component"))
    got = o3.spherical_harmonics(2, x.to(DEV), True, "norm")
    assert_close(got, osh(2, x.numpy(), True, "norm"))
    got = o3.spherical_harmonics("1x1o+1x3o", x.to(DEV), False, "integral")
    assert_close(got, osh([1, 3], x.numpy(), False, "integral"), rtol=2e-5)
    got = o3.spherical_harmonics([12], x.to(DEV), True, "component")
    assert_close(got, osh([12], x.numpy(), True, "component"), atol=5e-4)
    # strided input
    xs = seeded(40, 6, seed=4).to(DEV)[:, ::2]
    assert_close(o3.spherical_harmonics([0, 1, 2], xs, True, "component"), osh([0, 1, 2], xs.cpu().numpy(), True, "component"))


def test_zero_vector_and_empty_input():
    z = o3.spherical_harmonics([0, 1], torch.zeros(1, 3, device=DEV), False, normalization="norm")
    assert torch.equal(z.cpu(), torch.tensor([[1.0, 0, 0, 0]]))  # reference test: value at zero
    z = o3.spherical_harmonics([0, 1, 2, 3], torch.zeros(3, 3, device=DEV), True, "component")
    assert torch.equal(z[:, 0].cpu(), torch.ones(3)) and not z[:, 1:].any()
    e = o3.spherical_harmonics([0, 1, 2], torch.zeros(0, 3, device=DEV), True, "component")
    assert e.shape == (0, 9)
    # ... and its backward and second backward pass: empty gradients of the right shapes
    x0 = torch.zeros(0, 3, device=DEV, requires_grad=True)
    y0 = o3.spherical_harmonics([0, 1, 2], x0, True, "component")
    (g0,) = torch.autograd.grad(y0.sum(), x0, create_graph=True)
    assert g0.shape == (0, 3)
    (h0,) = torch.autograd.grad(g0.sum(), x0)
    assert h0.shape == (0, 3)
    one = o3.spherical_harmonics(0, torch.randn(2, 3, device=DEV), False, normalization="component")
    assert torch.equal(one.cpu(), torch.ones(2, 1))  # reference docstring example


def test_errors():
    with pytest.raises(NotImplementedError):
        o3.SphericalHarmonics([13], True)
    with pytest.raises(ValueError):
        o3.SphericalHarmonics("1x0e+4x1e+3x2e", True, irreps_in="1e+3o")
    with pytest.raises(ValueError):
        o3.SphericalHarmonics("1e", True, irreps_in="1o")
    with pytest.raises(RuntimeError):
        o3.spherical_harmonics(1, torch.randn(4, 3), True)  # CPU tensor: no silent fallback


def test_full_size_benchmark_shape_properties_and_parity():
    # 4 000 000 vectors, direction uniform on S2, norm log-normal(0, 0.5); lmax 3, component
    g = torch.Generator().manual_seed(0)
    d = torch.randn(4_000_000, 3, generator=g)
    d = d / d.norm(dim=1, keepdim=True)
    x = d * torch.exp(0.5 * torch.randn(4_000_000, 1, generator=g))
    xd = x.to(DEV)
    y = o3.spherical_harmonics([0, 1, 2, 3], xd, True, "component")
    assert y.shape == (4_000_000, 16)
    # size-independent properties: |Y^l|^2 = 2l+1, parity, scale invariance under normalize=True
    for l in range(4):
        n2 = y[:, l * l : (l + 1) * (l + 1)].double().pow(2).sum(1)
        assert (n2 - (2 * l + 1)).abs().max().item() < 1e-4 * (2 * l + 1)
    ym = o3.spherical_harmonics([0, 1, 2, 3], -xd, True, "component")
    sign = torch.cat([torch.full((2 * l + 1,), (-1.0) ** l) for l in range(4)]).to(DEV)
    assert torch.equal(ym, y * sign)
    y2 = o3.spherical_harmonics([0, 1, 2, 3], 2.0 * xd, True, "component")
    assert (y2 - y).abs().max().item() < 1e-5
    # parity with the oracle on every vector
    ref = osh([0, 1, 2, 3], x.numpy(), True, "component")
    assert_close(y, ref, what="4M vectors")
    assert abs(y.double().pow(2).mean().item() - 1.0) < 1e-5 * math.sqrt(16)
