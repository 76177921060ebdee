"""GPU property tests mirroring the reference's assert_equivariant (e3nn/util/test.py:158-205):
f(D_in x) == D_out f(x) for a random rotation, with and without inversion."""
import numpy as np
import pytest
import torch

from e3nn_amd import o3
from oracle.rotation import irreps_D, random_rotation
from tests import kernel_sets as ks
from tests.helpers import seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _D(irreps, R, improper):
    return torch.from_numpy(irreps_D(str(irreps), R, improper)).float().to(DEV)


@pytest.mark.parametrize("improper", [False, True])
@pytest.mark.parametrize("maker,Z", [(lambda: ks.cfg3(True), 64), (lambda: ks.cfg4("A"), 16), (ks.cfg1, 64), (ks.mfma_small, 70)])
def test_tensor_product_equivariance(maker, Z, improper):
    tp = maker().to(DEV)
    R = random_rotation(np.random.default_rng(3))
    D1, D2, Do = (_D(i, R, improper) for i in (tp.irreps_in1, tp.irreps_in2, tp.irreps_out))
    x1 = seeded(Z, tp.irreps_in1.dim, seed=1).to(DEV)
    x2 = seeded(Z, tp.irreps_in2.dim, seed=2).to(DEV)
    args = ()
    if tp.weight_numel and not tp.internal_weights:
        args = (seeded(Z, tp.weight_numel, seed=3).to(DEV),)
    a = tp(x1 @ D1.T, x2 @ D2.T, *args)
    b = tp(x1, x2, *args) @ Do.T
    scale = max(1.0, b.abs().max().item())
    assert (a - b).abs().max().item() < 2e-5 * scale


@pytest.mark.parametrize("improper", [False, True])
def test_message_passing_equivariance(improper):
    tp = ks.cfg3(False)
    N, E = 200, 5000
    g = torch.Generator().manual_seed(0)
    src, dst = torch.randint(0, N, (E,), generator=g).to(DEV), torch.randint(0, N, (E,), generator=g).to(DEV)
    R = random_rotation(np.random.default_rng(5))
    Rt = torch.from_numpy(R if not improper else -R).float().to(DEV)
    D1, Do = _D(tp.irreps_in1, R, improper), _D(tp.irreps_out, R, improper)
    node_x, vec, w = seeded(N, 288, seed=1).to(DEV), seeded(E, 3, seed=2).to(DEV), seeded(E, 352, seed=3).to(DEV)

    def model(x, v):
        attr = o3.spherical_harmonics([0, 1, 2], v, True, "component")
        return tp.forward_gather_scatter(x, attr, w, src, dst, N)

    a = model(node_x @ D1.T, vec @ Rt.T)
    b = model(node_x, vec) @ Do.T
    assert (a - b).abs().max().item() < 1e-4 * max(1.0, b.abs().max().item())


@pytest.mark.parametrize("lmax", [3, 6])
def test_spherical_harmonics_equivariance(lmax):
    irreps = o3.Irreps.spherical_harmonics(lmax)
    R = random_rotation(np.random.default_rng(9))
    x = seeded(50, 3, seed=4).to(DEV)
    Rt = torch.from_numpy(R).float().to(DEV)
    y0 = o3.spherical_harmonics(irreps, x, True, "component")
    y1 = o3.spherical_harmonics(irreps, x @ Rt.T, True, "component")
    assert (y1 - y0 @ _D(irreps, R, False).T).abs().max().item() < 2e-5 * (2 * lmax + 1)
    # inversion: Y^l(-x) = (-1)^l Y^l(x)
    y3 = o3.spherical_harmonics(irreps, -x, True, "component")
    assert (y3 - y0 @ _D(irreps, np.eye(3), True).T).abs().max().item() < 1e-5 * (2 * lmax + 1)
