"""GPU parity: fused gather -> uvu tensor product -> scatter-sum against the CPU oracle."""
import numpy as np
import pytest
import torch

from e3nn_amd import o3
from e3nn_amd.nn import DstSortedEdges
from oracle import tensor_product as otp
from oracle.message_passing import tp_gather_scatter
from tests import kernel_sets as ks
from tests.helpers import assert_close, oracle_spec, seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def random_graph(N, E, seed=0, dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, N, (E,), generator=g).to(dtype), torch.randint(0, N, (E,), generator=g).to(dtype)


def test_conv_matches_reference_golden(golden_tp):
    meta, arr = golden_tp
    tp = ks.golden_tp("conv_small", meta)
    g = {k.split("/")[1]: torch.from_numpy(v) for k, v in arr.items() if k.startswith("conv_small/")}
    attr = o3.spherical_harmonics([0, 1, 2], g["vec"].float().to(DEV), True, "component")
    assert_close(attr, g["attr"].numpy(), what="edge attrs")
    out = tp.forward_gather_scatter(
        g["node_x"].float().to(DEV), attr, g["w"].float().to(DEV), g["src"].to(DEV), g["dst"].to(DEV), g["node_x"].shape[0]
    )
    assert_close(out, g["out"].numpy(), what="conv_small")
    assert not out[-1].any()  # the last node receives no edge: exact zeros


def test_index_handling_is_bit_exact():
    # 1x1 Clebsch-Gordan and path weight 1: with small-integer payloads every product and every
    # partial sum is an exact fp32 integer, so the result is independent of summation order
    tp = ks.scalar_exact()
    assert abs(tp.instructions[0].path_weight - 1.0) < 1e-15
    N, E = 301, 20_000
    g = torch.Generator().manual_seed(5)
    node_x = torch.randint(-8, 9, (N, 32), generator=g).float()
    attr = torch.randint(-4, 5, (E, 1), generator=g).float()
    w = torch.randint(-4, 5, (E, 32), generator=g).float()
    src, dst = random_graph(N, E, seed=6)
    dst = torch.where(dst >= N - 3, dst - 3, dst)  # nodes N-3.. receive nothing
    ref = np.zeros((N, 32), dtype=np.float64)
    np.add.at(ref, dst.numpy(), (w * node_x[src] * attr).double().numpy())
    outs = []
    for dt in (torch.int64, torch.int32):
        out = tp.forward_gather_scatter(node_x.to(DEV), attr.to(DEV), w.to(DEV), src.to(dt).to(DEV), dst.to(dt).to(DEV), N)
        assert np.array_equal(out.cpu().numpy().astype(np.float64), ref)
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    assert not outs[0][N - 3 :].any()
    # negative source indices wrap like torch advanced indexing
    out = tp.forward_gather_scatter(node_x.to(DEV), attr.to(DEV), w.to(DEV), (src - N).to(DEV), dst.to(DEV), N)
    assert torch.equal(out, outs[0])
    # already grouped by destination, and the reverse order: same exact sums
    order = torch.argsort(dst, stable=True)
    for o in (order, order.flip(0)):
        out = tp.forward_gather_scatter(node_x.to(DEV), attr[o].to(DEV), w[o].to(DEV), src[o].to(DEV), dst[o].to(DEV), N)
        assert torch.equal(out, outs[0])


def test_out_of_range_indices_raise_and_empty_graph():
    tp = ks.scalar_exact()
    N, E = 10, 50
    src, dst = random_graph(N, E, seed=1)
    node_x, attr, w = seeded(N, 32).to(DEV), seeded(E, 1).to(DEV), seeded(E, 32).to(DEV)
    bad = dst.clone()
    bad[7] = N
    with pytest.raises(IndexError):
        tp.forward_gather_scatter(node_x, attr, w, src.to(DEV), bad.to(DEV), N)
    bad = dst.clone()
    bad[7] = -1  # scatter_add_ does not wrap
    with pytest.raises(IndexError):
        tp.forward_gather_scatter(node_x, attr, w, src.to(DEV), bad.to(DEV), N)
    bad = src.clone()
    bad[3] = N
    with pytest.raises(IndexError):
        tp.forward_gather_scatter(node_x, attr, w, bad.to(DEV), dst.to(DEV), N)
    bad[3] = -N - 1
    with pytest.raises(IndexError):
        tp.forward_gather_scatter(node_x, attr, w, bad.to(DEV), dst.to(DEV), N)
    e = torch.zeros(0, dtype=torch.int64, device=DEV)
    out = tp.forward_gather_scatter(node_x, attr[:0], w[:0], e, e, N)
    assert out.shape == (N, 32) and not out.any()
    # ... and its backward pass: zero gradients of the right shapes
    a, b, c = node_x.clone().requires_grad_(True), attr[:0].clone().requires_grad_(True), w[:0].clone().requires_grad_(True)
    tp.forward_gather_scatter(a, b, c, e, e, N).backward(torch.ones(N, 32, device=DEV))
    assert a.grad.shape == (N, 32) and not a.grad.any()
    assert b.grad is None or b.grad.shape == (0, 1)
    assert c.grad is None or c.grad.shape == (0, 32)
    # the same through the harmonics of (no) edge vectors, stored and formed in the kernel
    tp2 = ks.cfg3(merged=True)
    nx = seeded(N, tp2.irreps_in1.dim).to(DEV).requires_grad_(True)
    vec = torch.zeros(0, 3, device=DEV, requires_grad=True)
    w2 = torch.zeros(0, tp2.weight_numel, device=DEV, requires_grad=True)
    edges = DstSortedEdges(e, e, N)
    for out in (tp2.forward_gather_scatter(nx, o3.spherical_harmonics([0, 1, 2], vec, True, "component"), w2, edges=edges),
                tp2.forward_gather_scatter_sh(nx, vec, w2, edges, True, "component")):
        assert out.shape == (N, tp2.irreps_out.dim) and not out.any()
        gn, gv, gw = torch.autograd.grad(out.sum(), (nx, vec, w2), allow_unused=True)
        assert gn.shape == nx.shape and not gn.any()
        assert gv is None or gv.shape == (0, 3)
        assert gw is None or gw.shape == (0, tp2.weight_numel)
    # source nodes without edges get a zero gradient row, the others what autograd of the dense form gives
    src2 = torch.where(src < 3, src + 3, src)  # nodes 0, 1, 2 send nothing
    a, c = node_x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    tp.forward_gather_scatter(a, attr, c, src2.to(DEV), dst.to(DEV), N).backward(torch.ones(N, 32, device=DEV))
    assert not a.grad[:3].any() and a.grad[3:].any()
    ref_x = node_x.clone().requires_grad_(True)
    ref_w = w.clone().requires_grad_(True)
    # scalar_exact: 32x0e x 1x0e -> 32x0e, uvu with per-edge weights: message[e, u] = pw * w[e, u] * x[src[e], u] * attr[e, 0]
    pw = float(tp.instructions[0].path_weight) if hasattr(tp.instructions[0], "path_weight") else 1.0
    msg = pw * ref_w * ref_x[src2.to(DEV)] * attr
    torch.zeros(N, 32, device=DEV).index_add(0, dst.to(DEV), msg).sum().backward()
    assert torch.allclose(a.grad, ref_x.grad, atol=1e-5, rtol=1e-5)
    assert torch.allclose(c.grad, ref_w.grad, atol=1e-5, rtol=1e-5)


def test_run_to_run_bit_reproducible_and_prebuilt_edges():
    tp = ks.cfg3(True)
    N, E = 500, 20_000
    src, dst = random_graph(N, E, seed=2)
    node_x, attr, w = seeded(N, 288, seed=1).to(DEV), seeded(E, 9, seed=2).to(DEV), seeded(E, 352, seed=3).to(DEV)
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    assert edges.rowptr[-1].item() == E and edges.rowptr[0].item() == 0
    # stable sort: perm lists the edges of each destination in their original order
    perm = edges.perm.cpu().long()
    assert torch.equal(perm, torch.argsort(dst, stable=True))
    a = tp.forward_gather_scatter(node_x, attr, w, edges=edges)
    b = tp.forward_gather_scatter(node_x, attr, w, src.to(DEV), dst.to(DEV), N)
    assert torch.equal(a, b)
    assert torch.equal(a, tp.forward_gather_scatter(node_x, attr, w, edges=edges))


@pytest.mark.parametrize("idx", [torch.int32, torch.int64])
def test_row_processing_order(idx):
    """The rows are walked in the order of their smallest source row (and, on one node set, of that node's own key, twice
    over; stable), rows without edges last; the order changes which row a wavefront takes, not what it computes: outputs
    are bit-identical with and without it."""
    tp = ks.cfg3(True)
    N, E = 900, 15_000
    src, dst = random_graph(N, E, seed=5, dtype=idx)
    dst = torch.where(dst % 7 == 3, (dst + 1) % N, dst)  # some rows keep no in-edge
    src[::11] -= N  # negative gather indices wrap
    node_x, attr, w = seeded(N, 288, seed=1).to(DEV), seeded(E, 9, seed=2).to(DEV), seeded(E, 352, seed=3).to(DEV)
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N, locality_order=True)
    order = edges.row_order.cpu().long().numpy()
    assert sorted(order.tolist()) == list(range(N))
    key = np.full(N, 2**32 - 1, dtype=np.int64)
    np.minimum.at(key, dst.long().numpy(), (src.long().numpy() % N))
    # sources and destinations are one node set here: rows are grouped by (k3, k2, k1) with k1 the smallest source of the
    # row, k2 = k1 of node k1, k3 = k1 of node k2 -- three stable sorts, the most significant key last
    big = 2**32 - 1
    k2 = np.where(key < N, key[np.minimum(key, N - 1)], big)
    k3 = np.where(k2 < N, key[np.minimum(k2, N - 1)], big)
    want = np.argsort(key, kind="stable")
    want = want[np.argsort(k2[want], kind="stable")]
    want = want[np.argsort(k3[want], kind="stable")]
    assert np.array_equal(order, want)
    assert (key[order[-5:]] == big).all()  # the test graph has more than five empty rows
    plain = DstSortedEdges(src.to(DEV), dst.to(DEV), N, locality_order=False)
    assert plain.row_order is None
    a = tp.forward_gather_scatter(node_x, attr, w, edges=edges)
    b = tp.forward_gather_scatter(node_x, attr, w, edges=plain)
    assert torch.equal(a, b)
    assert not a[torch.from_numpy(key == 2**32 - 1).to(DEV)].any()
    # the transposed edge list (for the gradient with respect to the node features) inherits the choice
    src0 = src % N
    assert DstSortedEdges(src0.to(DEV), dst.to(DEV), N, locality_order=True).transposed().row_order is not None
    assert DstSortedEdges(src0.to(DEV), dst.to(DEV), N, locality_order=False).transposed().row_order is None
    # default ("auto"): uniformly random edges have no neighbourhoods to exploit and keep the plain row order ...
    auto = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    assert auto.row_order is None and auto.locality_score < 0.02
    # ... a radius graph (random node numbering) has them
    g = torch.Generator().manual_seed(1)
    pos = torch.rand(1500, 3, generator=g) * 10.0
    near = (torch.cdist(pos, pos) < 1.6) & ~torch.eye(1500, dtype=torch.bool)
    rs, rd = near.nonzero(as_tuple=True)
    geo = DstSortedEdges(rs.to(idx).to(DEV), rd.to(idx).to(DEV), 1500)
    assert geo.row_order is not None and geo.locality_score > 0.1, geo.locality_score


@pytest.mark.parametrize("maker,N,E,idx", [
    (lambda: ks.cfg3(True), 700, 26_000, torch.int64),
    (lambda: ks.cfg3(False), 300, 9_000, torch.int64),
    (lambda: ks.cfg4("A"), 60, 1_500, torch.int32),
    (lambda: ks.cfg4("B"), 40, 700, torch.int32),
    (ks.odd_mul, 90, 2_000, torch.int32),
    (ks.narrow_message, 150, 4_000, torch.int64),  # 16 channels: two multiplicity indices per lane
])  # fmt: skip
def test_fused_matches_oracle(maker, N, E, idx):
    tp = maker()
    src, dst = random_graph(N, E, seed=3, dtype=idx)
    node_x = seeded(N, tp.irreps_in1.dim, seed=1)
    vec = seeded(E, 3, seed=2)
    lmax = tp.irreps_in2.lmax
    attr = o3.spherical_harmonics(list(range(lmax + 1)), vec.to(DEV), True, "component")
    w = seeded(E, tp.weight_numel, seed=4)
    out = tp.forward_gather_scatter(node_x.to(DEV), attr, w.to(DEV), src.to(DEV), dst.to(DEV), N)
    ref = tp_gather_scatter(oracle_spec(tp), node_x.numpy(), attr.cpu().numpy(), w.numpy(), src.numpy(), dst.numpy(), N)
    # sums of ~E/N messages of magnitude up to ~50: tolerance scales with the accumulated magnitude
    scale = max(1.0, float(np.abs(ref).max()))
    assert_close(out, ref, atol=1e-4 * scale ** 0.5, rtol=1e-5, what=str(tp))
    # same thing as the unfused product path
    msg = tp(node_x.to(DEV)[src.long().to(DEV)], attr, w.to(DEV))
    unfused = torch.zeros_like(out).index_add_(0, dst.long().to(DEV), msg)
    assert (out - unfused).abs().max().item() < 1e-4 * scale


# graph shapes a neighbour list can take: no edges, one edge, one node, every edge onto one row (several passes of 64
# edges over the same accumulators), rows that alternate between empty and full, a heavy-tailed degree distribution, more
# source nodes than rows, a list that is already sorted
@pytest.mark.parametrize("shape,N,Ns,E", [
    ("uniform", 1, 1, 1), ("uniform", 1, 6, 200), ("one_row", 7, 7, 3000), ("half_empty", 60, 60, 2000), ("power", 300, 305, 3000),
    ("sorted", 60, 65, 5), ("uniform", 300, 300, 0), ("power", 2, 2, 5000),
])  # fmt: skip
def test_graph_shapes_through_both_message_entry_points(shape, N, Ns, E):
    tp = ks.cfg3(True)
    g = torch.Generator().manual_seed(N * 7919 + E)
    if shape == "one_row":
        dst = torch.full((E,), 3, dtype=torch.int64)
    elif shape == "half_empty":
        dst = torch.randint(0, N // 2, (E,), generator=g) * 2
    elif shape == "power":
        dst = (torch.rand(E, generator=g) ** 4 * N).long().clamp_(0, N - 1)
    else:
        dst = torch.randint(0, N, (E,), generator=g)
    if shape == "sorted":
        dst = torch.sort(dst).values
    src = torch.randint(0, Ns, (E,), generator=g)
    if E > 2:
        src[1] -= Ns  # a negative source index wraps, as torch indexing does
    node_x, vec, w = seeded(Ns, tp.irreps_in1.dim, seed=1), seeded(E, 3, seed=2), seeded(E, tp.weight_numel, seed=4)
    if E > 3:
        vec[0] = 0  # the zero vector: harmonics (1, 0, ..., 0)
    idx = torch.int32 if E % 2 else torch.int64
    edges = DstSortedEdges(src.to(idx).to(DEV), dst.to(idx).to(DEV), N, num_src_nodes=Ns)
    attr = o3.spherical_harmonics([0, 1, 2], vec.to(DEV), True, "component")
    ref = tp_gather_scatter(oracle_spec(tp), node_x.numpy(), attr.cpu().numpy(), w.numpy(), (src % Ns).numpy(), dst.numpy(), N) if E else np.zeros((N, tp.irreps_out.dim))
    scale = max(1.0, float(np.abs(ref).max()))
    for what, out in (("stored attributes", tp.forward_gather_scatter(node_x.to(DEV), attr, w.to(DEV), edges=edges)),
                      ("harmonics in the kernel", tp.forward_gather_scatter_sh(node_x.to(DEV), vec.to(DEV), w.to(DEV), edges, True, "component"))):
        assert_close(out, ref, atol=1e-4 * scale ** 0.5, rtol=1e-5, what=f"{shape} N={N} E={E}, {what}")
        # rows without edges are exactly zero
        empty = np.setdiff1d(np.arange(N), dst.numpy())
        assert not out[torch.from_numpy(empty).to(DEV)].any()


@pytest.mark.parametrize("idx", [torch.int32, torch.int64])
def test_edge_list_held_in_destination_order(idx):
    # per-edge tensors rewritten once in the order the kernels walk the edges, and an edge list the caller already holds
    # grouped by destination (no permutation handed to the kernels): the same bits as the caller's order in the forward
    # pass and in the per-edge gradients; the gradient of the node features sums the edges leaving a node in the
    # order of the list it is given, so there the two agree to rounding
    tp = ks.cfg3(True)
    N, E = 300, 9_000
    src, dst = random_graph(N, E, seed=11, dtype=idx)
    src[3] = -2
    node_x, attr, w = seeded(N, tp.irreps_in1.dim, seed=1).to(DEV), seeded(E, 9, seed=2).to(DEV), seeded(E, tp.weight_numel, seed=3).to(DEV)
    cot = seeded(N, tp.irreps_out.dim, seed=4).to(DEV)
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    assert edges.walk_perm is not None

    def run(e, a, ww):
        x, a, ww = (t.clone().requires_grad_() for t in (node_x, a, ww))
        out = tp.forward_gather_scatter(x, a, ww, edges=e)
        return (out,) + torch.autograd.grad(out, (x, a, ww), cot)

    ref = run(edges, attr, w)
    se = edges.sorted()
    assert se.walk_perm is None and se.sorted() is se and torch.equal(se.rowptr, edges.rowptr)
    attr_s, w_s = edges.in_sorted_order(attr, w)
    got = run(se, attr_s, w_s)
    perm = edges.perm.long()
    assert torch.equal(got[0], ref[0])
    assert (got[1] - ref[1]).abs().max().item() <= 1e-5 * ref[1].abs().max().item()
    assert torch.equal(got[2], ref[2][perm]) and torch.equal(got[3], ref[3][perm])
    # the caller's own list already grouped by destination: detected, walked by position
    order = torch.argsort(dst.long(), stable=True)
    pre = DstSortedEdges(src[order].to(DEV), dst[order].to(DEV), N)
    assert pre.walk_perm is None and pre.sorted() is pre
    assert pre.in_sorted_order(attr_s) is attr_s
    again = run(pre, attr_s, w_s)
    for a, b in zip(again, got):
        assert torch.equal(a, b)
    # the kernel with the radial network inside and the one that forms the harmonics itself walk such a list by position too
    _, tp_r, net = ks.radial_message_cases()[0]
    net = net.to(DEV)
    scal, vec = seeded(E, net.hs[0], seed=5).to(DEV), seeded(E, 3, seed=6).to(DEV)
    with torch.no_grad():
        ref_r = tp_r.forward_gather_scatter_radial(node_x, attr, scal, net, edges)
        got_r = tp_r.forward_gather_scatter_radial(node_x, attr_s, edges.in_sorted_order(scal), net, se)
        assert ref_r is not None and got_r is not None
        assert (ref_r - got_r).abs().max().item() <= 1e-5 * ref_r.abs().max().item()  # (edge ranges of the workers move with the order)
        assert torch.equal(tp.forward_gather_scatter_sh(node_x, vec, w, edges), tp.forward_gather_scatter_sh(node_x, edges.in_sorted_order(vec), w_s, se))


@pytest.mark.parametrize("maker,N,E,idx,normalize,normalization", [
    (lambda: ks.cfg3(True), 700, 26_000, torch.int64, True, "component"),
    (lambda: ks.cfg3(True), 90, 2_000, torch.int32, False, "integral"),
    (lambda: ks.cfg3(False), 300, 9_000, torch.int64, True, "norm"),
    (lambda: ks.cfg4("A"), 60, 1_500, torch.int32, True, "component"),
    (ks.odd_mul, 90, 2_000, torch.int32, True, "integral"),
    (ks.narrow_message, 70, 1_800, torch.int64, True, "component"),
])  # fmt: skip
def test_fused_with_the_harmonics_formed_in_the_kernel(maker, N, E, idx, normalize, normalization):
    # edge_attr = spherical_harmonics(0 .. lmax, edge_vec) evaluated inside the message kernel from the 12-byte vectors:
    # against the oracle on the oracle's own harmonics (float64), a zero vector and negative source indices included
    from oracle.spherical_harmonics import spherical_harmonics as osh

    tp = maker()
    src, dst = random_graph(N, E, seed=3, dtype=idx)
    src[5] = -1  # wraps to the last node, as torch indexing does
    node_x = seeded(N, tp.irreps_in1.dim, seed=1)
    vec = seeded(E, 3, seed=2) * (1.0 if normalize else 0.7)
    vec[7] = 0.0  # normalize: the l = 0 constant and zeros elsewhere, not NaN
    ls = list(range(tp.irreps_in2.lmax + 1))
    w = seeded(E, tp.weight_numel, seed=4)
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    out = tp.forward_gather_scatter_sh(node_x.to(DEV), vec.to(DEV), w.to(DEV), edges, normalize, normalization)
    attr64 = osh(ls, vec.numpy().astype(np.float64), normalize, normalization)
    ref = tp_gather_scatter(oracle_spec(tp), node_x.numpy(), attr64, w.numpy(), src.numpy(), dst.numpy(), N)
    scale = max(1.0, float(np.abs(ref).max()))
    assert torch.isfinite(out).all()
    assert_close(out, ref, atol=1e-4 * scale ** 0.5, rtol=1e-5, what=f"harmonics in the kernel, {normalization}: {tp}")
    # the two-kernel path (harmonics stored, then the message kernel): same sums up to the harmonics' own rounding
    attr = o3.spherical_harmonics(ls, vec.to(DEV), normalize, normalization)
    two = tp.forward_gather_scatter(node_x.to(DEV), attr, w.to(DEV), edges=edges)
    assert (out - two).abs().max().item() <= 2e-6 * scale


def test_fused_with_the_harmonics_formed_in_the_kernel_gradients_and_refusals():
    from oracle.torch_cpu import spherical_harmonics_torch, tp_gather_scatter_torch

    tp = ks.cfg3(True)
    spec = oracle_spec(tp)
    N, E = 120, 3000
    src, dst = random_graph(N, E, seed=5)
    node_x, vec, w = seeded(N, tp.irreps_in1.dim, seed=1), seeded(E, 3, seed=2), seeded(E, tp.weight_numel, seed=3)
    cot = seeded(N, tp.irreps_out.dim, seed=4)
    a, b, c = (t.double().requires_grad_() for t in (node_x, vec, w))
    ref = tp_gather_scatter_torch(spec, a, spherical_harmonics_torch(2, b, True), c, src, dst, N)
    r1, r2, rw = torch.autograd.grad(ref, (a, b, c), cot.double())
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    x, v, ww = (t.to(DEV).requires_grad_() for t in (node_x, vec, w))
    out = tp.forward_gather_scatter_sh(x, v, ww, edges, True, "component")
    g1, g2, gw = torch.autograd.grad(out, (x, v, ww), cot.to(DEV))
    scale = lambda r: max(1.0, float(r.abs().max()))  # noqa: E731
    assert_close(out, ref.detach().numpy(), atol=1e-4 * scale(ref.detach()) ** 0.5)
    assert_close(g1, r1.numpy(), atol=1e-4 * scale(r1), what="d/dnode_x (harmonics in the kernel)")
    assert_close(g2, r2.numpy(), atol=1e-4 * scale(r2), what="d/dedge_vec (harmonics in the kernel)")
    assert_close(gw, rw.numpy(), what="d/dweight (harmonics in the kernel)")
    # plans whose second input is something else are refused
    other = ks.scalar_exact()
    e2 = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    with pytest.raises(NotImplementedError):
        other.forward_gather_scatter_sh(seeded(N, 32).to(DEV), vec.to(DEV), seeded(E, other.weight_numel).to(DEV), e2)
    with pytest.raises(TypeError):
        tp.forward_gather_scatter_sh(node_x.to(DEV), vec.double().to(DEV), w.to(DEV), edges)


@pytest.mark.parametrize("variant,N,E,idx", [("A", 50, 1000, torch.int32), ("A", 7, 900, torch.int64), ("B", 40, 700, torch.int32),
                                              ("A", 300, 5, torch.int64)])  # fmt: skip
def test_fused_bf16_storage(variant, N, E, idx):
    # bf16 storage of the 128-channel l <= 3 sets runs the message kernel with the contraction on the matrix cores
    # (one workgroup per row, 4 or 6 wavefronts): rows longer than a block of 64 edges (E / N > 64), rows without
    # edges, the per-edge matrices rounded to bf16 once more than in the other kernels
    tp = ks.cfg4(variant)
    assert "uvu_mfma" in tp._plan(torch.bfloat16).key
    src, dst = random_graph(N, E, seed=9, dtype=idx)
    dst = torch.where(dst == 2, dst + 1, dst)  # node 2 receives nothing
    node_x, attr, w = seeded(N, 2048, seed=1), seeded(E, 16, seed=2), seeded(E, tp.weight_numel, seed=3)
    nb, ab, wb = (t.to(DEV).to(torch.bfloat16) for t in (node_x, attr, w))
    out = tp.forward_gather_scatter(nb, ab, wb, src.to(DEV), dst.to(DEV), N)
    assert out.dtype == torch.bfloat16 and not out[2].any()
    ref = tp_gather_scatter(
        oracle_spec(tp), nb.float().cpu().numpy(), ab.float().cpu().numpy(), wb.float().cpu().numpy(), src.numpy(), dst.numpy(), N
    )
    scale = float(np.abs(ref).max())
    assert_close(out, ref, atol=1e-2 * scale / 4, rtol=1e-2, what=f"bf16 fused {variant} N={N} E={E}")
    # bit-reproducible, and the same bits for an edge list already grouped by destination
    assert torch.equal(tp.forward_gather_scatter(nb, ab, wb, src.to(DEV), dst.to(DEV), N), out)
    order = torch.argsort(dst, stable=True)
    od = order.to(DEV)
    assert torch.equal(tp.forward_gather_scatter(nb, ab[od], wb[od], src[order].to(DEV), dst[order].to(DEV), N), out)
    # without the workspace the C entry point runs the vector-ALU kernels: same result up to the rounding of the matrices
    from e3nn_amd import _lib

    plan = tp._plan(torch.bfloat16)
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    plain = torch.empty_like(out)
    s_d = src.to(DEV)
    with torch.cuda.device(DEV):
        _lib.check(_lib.lib().e3x_tp_gather_scatter_ordered(
            plan.handle, _lib.ptr(nb), _lib.ptr(ab), _lib.ptr(wb), _lib.ptr(s_d), s_d.element_size() * 8, _lib.ptr(edges.rowptr),
            _lib.ptr(edges.perm), None, _lib.ptr(plain), E, N, N, _lib.stream_ptr(torch.device(DEV))))  # fmt: skip
    assert_close(plain, ref, atol=1e-2 * scale / 8, rtol=1e-2, what=f"bf16 fused {variant} without workspace")
    assert (plain.float() - out.float()).abs().max().item() <= 1e-2 * scale / 2


@pytest.mark.parametrize("idx", [torch.int32, torch.int64])
def test_source_rows_in_sorted_order(idx):
    # e3x_src_rows_build: the gather indices laid out in the order of the destination-sorted list, negative values
    # wrapped; the message kernels (vector-ALU fp32, matrix-core bf16) give the same bits with and without the list
    from e3nn_amd import _lib

    N, E = 90, 4000
    src, dst = random_graph(N, E, seed=21, dtype=idx)
    src = torch.where(src % 3 == 0, src - N, src)  # a third of the sources as negative indices
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    rows = edges.src_rows
    assert rows.dtype == torch.int32 and rows.shape == (E,)
    assert torch.equal(rows.cpu().long(), (src.long() % N)[edges.perm.cpu().long()])
    L, st = _lib.lib(), _lib.stream_ptr(torch.device(DEV))
    for tp, dtype, width in ((ks.cfg3(), torch.float32, 288), (ks.cfg4("A"), torch.bfloat16, 2048)):
        plan = tp._plan(dtype)
        node_x, attr, w = (seeded(n, d, seed=i).to(DEV).to(dtype) for i, (n, d) in
                           enumerate(((N, width), (E, tp.irreps_in2.dim), (E, tp.weight_numel))))
        outs = []
        with torch.cuda.device(DEV):
            ws_bytes = L.e3x_tp_gather_scatter_workspace_bytes(plan.handle, N)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=DEV)
            s_d = edges.edge_src
            for src_rows in (None, rows):
                out = torch.empty(N, tp.irreps_out.dim, dtype=dtype, device=DEV)
                _lib.check(L.e3x_tp_gather_scatter_ws(
                    plan.handle, _lib.ptr(node_x), _lib.ptr(attr), _lib.ptr(w), _lib.ptr(s_d), s_d.element_size() * 8,
                    _lib.ptr(edges.rowptr), _lib.ptr(edges.perm), None, _lib.ptr(src_rows), _lib.ptr(out), E, N, N,
                    _lib.ptr(ws) if ws_bytes else None, ws_bytes, st))  # fmt: skip
                outs.append(out)
        assert torch.equal(outs[0], outs[1])
        assert torch.equal(tp.forward_gather_scatter(node_x, attr, w, edges=edges), outs[0])


@pytest.mark.parametrize("case,N,E,idx", [
    ("nequip_silu", 400, 9_000, torch.int64), ("nequip_silu", 30, 3, torch.int32), ("nequip_silu", 5, 4_000, torch.int64),
    ("small_tanh", 200, 5_001, torch.int32), ("small_linear", 64, 777, torch.int64),
])  # fmt: skip
def test_message_with_the_radial_network_inside(case, N, E, idx):
    """weight = fc(edge_scalars); scatter(tp(x[src], attr, weight), dst) as ONE kernel, against the float64 oracle of
    the network followed by the oracle of the message step, and against the two separate kernels.  Graphs with
    more workers than groups of four edges, with rows longer than a worker's range, and with rows without edges."""
    from oracle import nn as onn

    name, tp, net = next(c for c in ks.radial_message_cases() if c[0] == case)
    net = net.to(DEV)
    src, dst = random_graph(N, E, seed=11, dtype=idx)
    dst[dst == 2] = 3  # node 2 receives nothing
    node_x = seeded(N, tp.irreps_in1.dim, seed=12)
    lmax = tp.irreps_in2.lmax
    attr = o3.spherical_harmonics(list(range(lmax + 1)), seeded(E, 3, seed=13).to(DEV), True, "component")
    scalars = seeded(E, net.hs[0], seed=14)
    edges = DstSortedEdges(src.to(DEV), dst.to(DEV), N)
    out = tp.forward_gather_scatter_radial(node_x.to(DEV), attr, scalars.to(DEV), net, edges)
    assert out is not None, "the instruction set and the network are inside the kernel's limits"
    ws = [net.layer0.weight.detach().cpu().numpy(), net.layer1.weight.detach().cpu().numpy()]
    act = net.layer0._act_name
    w = onn.fc_forward(ws, scalars.numpy(), act, variance_in=net.layer0.var_in, variance_out=net.layer1.var_out)
    ref = tp_gather_scatter(oracle_spec(tp), node_x.numpy(), attr.cpu().numpy(), w, src.numpy(), dst.numpy(), N)
    scale = max(1.0, float(np.abs(ref).max()))
    assert_close(out, ref, atol=1e-4 * scale, rtol=1e-5, what=f"{case} against the oracle")
    assert not out[2].any()  # exact zeros where no edge arrives
    with torch.no_grad():
        two = tp.forward_gather_scatter(node_x.to(DEV), attr, net(scalars.to(DEV)), edges=edges)
    assert (out - two).abs().max().item() < 1e-4 * scale
    # every row is summed by one worker of the kernel in the order of the sorted edge list: reruns give the same bits
    for _ in range(3):
        assert torch.equal(tp.forward_gather_scatter_radial(node_x.to(DEV), attr, scalars.to(DEV), net, edges), out)


def test_message_with_the_radial_network_declines_what_it_does_not_take():
    from e3nn_amd import nn

    tp = ks.cfg3(merged=True)
    edges = DstSortedEdges(torch.zeros(4, dtype=torch.int64, device=DEV), torch.zeros(4, dtype=torch.int64, device=DEV), 3)
    x, attr = torch.zeros(3, tp.irreps_in1.dim, device=DEV), torch.zeros(4, tp.irreps_in2.dim, device=DEV)
    three_layers = nn.FullyConnectedNet([8, 16, 16, tp.weight_numel], torch.tanh).to(DEV)
    assert tp.forward_gather_scatter_radial(x, attr, torch.zeros(4, 8, device=DEV), three_layers, edges) is None
    odd_hidden = nn.FullyConnectedNet([8, 24, tp.weight_numel], torch.tanh).to(DEV)  # hidden width not a multiple of 16
    assert tp.forward_gather_scatter_radial(x, attr, torch.zeros(4, 8, device=DEV), odd_hidden, edges) is None
    other_mul = ks.cfg4("A")  # multiplicities other than 32
    net = nn.FullyConnectedNet([8, 16, other_mul.weight_numel], torch.tanh).to(DEV)
    assert not other_mul.prepare_gather_scatter_radial(net)


def test_calibration_kernels_move_the_bytes_they_claim():
    # e3x_copy_bytes and e3x_stream_rows are what the profiler counters and the bandwidth figures are scaled by:
    # the copy is exact, the row streamer writes the XOR of the 16-byte pieces of a row, lane by lane
    from e3nn_amd import _lib

    L, st = _lib.lib(), _lib.stream_ptr(torch.device(DEV))
    g = torch.Generator().manual_seed(3)
    a = torch.randint(0, 2**31 - 1, (4096 + 5 * 4,), generator=g, dtype=torch.int32).to(DEV)
    b = torch.zeros_like(a)
    with torch.cuda.device(DEV):
        _lib.check(L.e3x_copy_bytes(_lib.ptr(a), _lib.ptr(b), a.numel() * 4, st))
    assert torch.equal(a, b)
    rows, pieces_in, pieces_out = 7, 150, 70  # ragged against the 64 lanes and the 8 loads in flight
    x = torch.randint(0, 2**31 - 1, (rows, pieces_in, 4), generator=g, dtype=torch.int32).to(DEV)
    out = torch.zeros(rows, pieces_out, 4, dtype=torch.int32, device=DEV)
    with torch.cuda.device(DEV):
        _lib.check(L.e3x_stream_rows(_lib.ptr(x), pieces_in * 16, rows, _lib.ptr(out), pieces_out * 16, st))
    fold = torch.zeros(rows, 64, 4, dtype=torch.int32)
    xc = x.cpu()
    for i in range(pieces_in):
        fold[:, i % 64] ^= xc[:, i]
    assert torch.equal(out.cpu(), fold[:, torch.arange(pieces_out) % 64])
    with pytest.raises(RuntimeError):
        with torch.cuda.device(DEV):
            _lib.check(L.e3x_stream_rows(_lib.ptr(x), 24, rows, _lib.ptr(out), 16, st))
