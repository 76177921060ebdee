"""GPU parity at the benchmark's full sizes: the fused message kernel on the whole graphs of the NequIP-style and the
MACE-scale configurations, checked on sampled destination rows against the CPU oracle run on just their in-edges,
and against the unfused path (plain tensor product on gathered rows + index_add_) on the whole output."""
import numpy as np
import pytest
import torch

from e3nn_amd import o3
from e3nn_amd.nn import DstSortedEdges
from oracle import tensor_product as otp
from oracle.spherical_harmonics import spherical_harmonics as osh
from tests import kernel_sets as ks
from tests.helpers import assert_close, oracle_spec

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def radius_graph(n, side, cutoff, seed=0):
    from scipy.spatial import cKDTree

    rng = np.random.default_rng(seed)
    pos = rng.uniform(0.0, side, size=(n, 3))
    pairs = cKDTree(pos).query_pairs(cutoff, output_type="ndarray")
    src = np.concatenate([pairs[:, 0], pairs[:, 1]]).astype(np.int64)
    dst = np.concatenate([pairs[:, 1], pairs[:, 0]]).astype(np.int64)
    return pos, src, dst


def sampled_rows(dst, N, n_random=24, seed=1):
    """first, last, highest in-degree, lowest in-degree (an empty row when there is one), and random rows"""
    deg = torch.bincount(dst.long(), minlength=N)
    rows = {0, N - 1, int(deg.argmax()), int(deg.argmin())}
    g = torch.Generator().manual_seed(seed)
    rows.update(torch.randint(0, N, (n_random,), generator=g).tolist())
    return sorted(rows), deg


def oracle_rows(tp, rows, node_x, attr, w, src, dst, dtype=torch.float32):
    """The oracle's scatter(tp(x[src], attr, w), dst) restricted to the destination rows `rows` (fp64, from the
    device tensors' values): only the in-edges of those rows are evaluated."""
    spec = oracle_spec(tp)
    dst_l = dst.long()
    ref = np.zeros((len(rows), tp.irreps_out.dim))
    n_edges = 0
    for r, row in enumerate(rows):
        e = torch.nonzero(dst_l == row).flatten()
        if e.numel() == 0:
            continue
        s = src[e].long()
        s = torch.where(s < 0, s + node_x.shape[0], s)
        msg = otp.tp_forward(spec, node_x[s].float().cpu().numpy(), attr[e].float().cpu().numpy(), w[e].float().cpu().numpy())
        ref[r] = msg.sum(axis=0)
        n_edges += e.numel()
    return ref, n_edges


def oracle_rows_fp64_attr(tp, rows, node_x, attr64, w, src, dst):
    """As oracle_rows, with the edge attributes given in float64 on the CPU (the oracle's own harmonics)."""
    spec = oracle_spec(tp)
    dst_l = dst.long()
    ref = np.zeros((len(rows), tp.irreps_out.dim))
    n_edges = 0
    for r, row in enumerate(rows):
        e = torch.nonzero(dst_l == row).flatten()
        if e.numel() == 0:
            continue
        s = src[e].long()
        s = torch.where(s < 0, s + node_x.shape[0], s)
        msg = otp.tp_forward(spec, node_x[s].float().cpu().numpy(), attr64[e.cpu()].numpy(), w[e].float().cpu().numpy())
        ref[r] = msg.sum(axis=0)
        n_edges += e.numel()
    return ref, n_edges


def unfused(tp, node_x, attr, w, src, dst, N, chunk=250_000):
    """plain tensor product on gathered rows, then index_add_ (fp32 atomics: the summation order differs)"""
    out = torch.zeros(N, tp.irreps_out.dim, device=DEV, dtype=torch.float32)
    for b in range(0, src.numel(), chunk):
        sl = slice(b, min(b + chunk, src.numel()))
        msg = tp(node_x[src[sl].long()], attr[sl], w[sl])
        out.index_add_(0, dst[sl].long(), msg.float())
    return out


def check_sum_tolerance(fused, other, what, rel):
    # two different summation orders of the same fp32 terms: error relative to the magnitude of the sums
    scale = other.abs().max().item()
    err = (fused.float() - other).abs().max().item()
    assert err <= rel * scale, f"{what}: fused vs unfused max abs diff {err:.3e} at output scale {scale:.3e}"


@pytest.mark.parametrize("side,label", [(86.8, "degree 37"), (40.0, "literal 40 A cube, degree 354")])
def test_nequip_configuration_at_full_size(side, label):
    # N = 50 000 nodes uniform in a cube, 5 A cutoff, int64 indices, 32x0e+32x1o+32x2e x SH(lmax 2), 11 uvu paths,
    # per-edge weights; the 40 A cube has 17.7 M edges and 6.2e9 weight elements (offsets beyond 2^32)
    N = 50_000
    pos, src, dst = radius_graph(N, side, 5.0)
    E = src.shape[0]
    assert (1_800_000 < E < 1_950_000) if side > 80 else (17_000_000 < E < 18_500_000)
    tp = ks.cfg3(merged=True)
    gen = torch.Generator(device=DEV).manual_seed(0)
    node_x = torch.randn(N, 288, device=DEV, generator=gen)
    src_t, dst_t = torch.from_numpy(src).to(DEV), torch.from_numpy(dst).to(DEV)
    pos_t = torch.from_numpy(pos).float().to(DEV)
    vec = pos_t[src_t] - pos_t[dst_t]
    attr = o3.spherical_harmonics([0, 1, 2], vec, True, "component")
    w = torch.randn(E, tp.weight_numel, device=DEV, generator=gen)
    assert w.numel() > 2**32 or side > 80
    edges = DstSortedEdges(src_t, dst_t, N, locality_order=True)
    assert edges.row_order is not None
    out = tp.forward_gather_scatter(node_x, attr, w, edges=edges)
    torch.cuda.synchronize()

    rows, deg = sampled_rows(dst_t, N)
    # edge attributes of the sampled rows from the oracle's own harmonics (fp64 of the fp32 edge vectors)
    for row in rows[:4]:
        e = torch.nonzero(dst_t == row).flatten()
        if e.numel():
            assert_close(attr[e], osh([0, 1, 2], vec[e].cpu().numpy().astype(np.float64), True, "component"), what=f"SH rows of node {row}")
    ref, n_edges = oracle_rows(tp, rows, node_x, attr, w, src_t, dst_t)
    assert n_edges > 20 * len(rows) / 2
    # sums of ~37 (354) messages of magnitude up to ~30: fp32 summation-order tolerance on top of the contraction's
    assert_close(out[rows], ref, atol=1e-4 * max(1.0, (deg.float().mean().item() / 37) ** 0.5), rtol=1e-5, what=f"NequIP uvu full size ({label}), {len(rows)} rows / {n_edges} edges")
    # plain row order gives the same bits
    plain = tp.forward_gather_scatter(node_x, attr, w, edges=DstSortedEdges(src_t, dst_t, N, locality_order=False))
    assert torch.equal(plain, out)
    del plain
    if side > 80:
        check_sum_tolerance(out, unfused(tp, node_x, attr, w, src_t, dst_t, N), "NequIP", 2e-6)
    assert torch.isfinite(out).all()
    # the harmonics formed inside the kernel from the 12-byte edge vectors: against the oracle on the oracle's own
    # harmonics of the sampled rows (fp64 of the fp32 vectors), and against the stored-attribute kernel on every row
    del out
    out_sh = tp.forward_gather_scatter_sh(node_x, vec, w, edges, True, "component")
    attr64 = torch.zeros(E, 9, dtype=torch.float64)
    for row in rows:
        e = torch.nonzero(dst_t == row).flatten().cpu()
        if e.numel():
            attr64[e] = torch.from_numpy(osh([0, 1, 2], vec[e.to(DEV)].cpu().numpy().astype(np.float64), True, "component"))
    ref_sh, _ = oracle_rows_fp64_attr(tp, rows, node_x, attr64, w, src_t, dst_t)
    assert_close(out_sh[rows], ref_sh, atol=1e-4 * max(1.0, (deg.float().mean().item() / 37) ** 0.5), rtol=1e-5, what=f"NequIP uvu, harmonics in the kernel ({label})")
    check_sum_tolerance(out_sh, tp.forward_gather_scatter(node_x, attr, w, edges=edges), "harmonics in the kernel vs stored", 2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mace_configuration_at_full_size(dtype):
    # N = 20 000, E = 500 000 uniformly random int32 edges, 128x0e+128x1o+128x2e+128x3o x SH(lmax 3), 23 uvu paths,
    # per-edge weights N(0,1): w is 5.9 GB, the output 1.0 GB in fp32
    N, E = 20_000, 500_000
    tp = ks.cfg4("A")
    gen = torch.Generator(device=DEV).manual_seed(0)
    node_x = torch.randn(N, 2048, device=DEV, generator=gen).to(dtype)
    unit = torch.nn.functional.normalize(torch.randn(E, 3, device=DEV, generator=gen), dim=1)
    attr = o3.spherical_harmonics([0, 1, 2, 3], unit, True, "component").to(dtype)
    w = torch.randn(E, tp.weight_numel, device=DEV, generator=gen).to(dtype)
    cpu = torch.Generator().manual_seed(1)
    src = torch.randint(0, N, (E,), generator=cpu).to(torch.int32).to(DEV)
    dst = torch.randint(0, N - 1, (E,), generator=cpu).to(torch.int32).to(DEV)  # node N-1 receives nothing
    out = tp.forward_gather_scatter(node_x, attr, w, src, dst, N)
    assert out.dtype == dtype and out.shape == (N, 12672)
    torch.cuda.synchronize()
    rows, deg = sampled_rows(dst, N, n_random=12)
    assert N - 1 in rows and deg[N - 1] == 0 and not out[N - 1].any()
    ref, n_edges = oracle_rows(tp, rows, node_x, attr, w, src, dst)
    if dtype == torch.float32:
        assert_close(out[rows], ref, atol=1e-4, rtol=1e-5, what=f"MACE uvu fp32 full size, {len(rows)} rows / {n_edges} edges")
        check_sum_tolerance(out, unfused(tp, node_x, attr, w, src, dst, N, chunk=100_000), "MACE fp32", 2e-6)
    else:
        # bf16 storage, fp32 accumulation: the output is rounded to bf16 once (2^-9 relative)
        scale = float(np.abs(ref).max())
        assert_close(out[rows], ref, atol=1e-2 * scale / 4, rtol=1e-2, what=f"MACE uvu bf16 storage full size, {len(rows)} rows / {n_edges} edges")
        # int64 indices: same bits
        assert torch.equal(tp.forward_gather_scatter(node_x, attr, w, src.long(), dst.long(), N), out)
    assert torch.isfinite(out.float()).all()
