"""Benchmark of the equivariant message-passing hot path on one MI355X.

Headline workload (the benchmark's third configuration, "NequIP-style interaction"): N = 50 000 nodes uniform in a
cube, radius graph with a 5 A cutoff (cube side 86.8 A -> ~1.87 M directed edges, degree ~37; the edge list grouped by
destination, as a neighbour search emits it), node features 32x0e+32x1o+32x2e fp32, edge attributes = SH(lmax 2) of
the edge vectors, uvu tensor product (11 paths) with per-edge weights from a 2-layer radial MLP, scatter-summed onto
the destination nodes.  One step = one launch of the fused gather -> spherical harmonics -> tensor product -> scatter
kernel over the whole graph, all inputs resident in HBM.  The other configurations are reported in "other".

Prints ONE JSON line.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# L2-miss traffic of one e3x_uvu_sh_fused launch on the headline workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# scaled by the 1 GiB copy kernel (profiles/uvu_sh_fused_nequip.txt), keyed by the code object the counters were read
# on: a kernel that has changed since reports no traffic instead of a stale figure.
NEQUIP_TRAFFIC_BYTES = {
    "uvu_3da245a80ccf1772fda9e383+sh": (2 * 1523940 + 56250) * 1024,  # FETCH_SIZE 1523940 x 2 KiB + WRITE_SIZE 56250 KiB
}
FP32_MFMA_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2500.0


def event_time_ms(fn, steps, warmup):
    """Average duration of fn() over `steps` launches, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    beg.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return beg.elapsed_time(end) / steps


def event_times_ms(fn, steps, warmup):
    """(mean, median, min) duration of fn() over `steps` launches: one HIP event between consecutive launches on the
    current stream, the mean taken from the first to the last event (exactly `steps` launches)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    each = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    return ev[0].elapsed_time(ev[steps]) / steps, each[len(each) // 2], each[0]


def bench_copy(args, dev):
    """Plain 16-byte-per-lane copy of 1 GiB: the measured streaming ceiling and the calibration
    kernel for the FETCH_SIZE / WRITE_SIZE counters (known traffic: 1 GiB read + 1 GiB written)."""
    from e3nn_amd import _lib

    n = 1 << 30
    a = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 255)
    b = torch.empty_like(a)
    L = _lib.lib()

    def step():
        _lib.check(L.e3x_copy_bytes(_lib.ptr(a), _lib.ptr(b), n, _lib.stream_ptr(dev)))

    ms = event_time_ms(step, max(3, args.steps // 5), 2)
    assert torch.equal(a[:4096], b[:4096])
    return {"bytes_read": n, "bytes_written": n, "ms": ms, "gbs": 2 * n / (ms * 1e-3) / 1e9}


def bench_stream_rows(args, dev, n_rows, bytes_total, out_row_bytes):
    """What this chip sustains on the memory traffic of the headline kernel alone: one wavefront per destination row
    streams the row's share of the per-edge bytes (no gather, no arithmetic) and, in the second run, writes an
    output row of the same size as the kernel's.  `bytes_total` is the headline's algorithmic byte count."""
    from e3nn_amd import _lib

    in_row = (bytes_total - n_rows * out_row_bytes) // n_rows // 16 * 16
    a = torch.empty(n_rows * in_row, dtype=torch.uint8, device=dev).random_(0, 255)
    b = torch.empty(n_rows * out_row_bytes, dtype=torch.uint8, device=dev)
    L = _lib.lib()
    res = {"rows": n_rows, "bytes_read_per_row": in_row, "bytes_written_per_row": out_row_bytes}
    for name, out_bytes in (("read_only", 0), ("read_and_row_stores", out_row_bytes)):
        def step():
            _lib.check(L.e3x_stream_rows(_lib.ptr(a), in_row, n_rows, _lib.ptr(b), out_bytes, _lib.stream_ptr(dev)))

        ms = event_time_ms(step, max(3, args.steps // 5), 2)
        moved = n_rows * (in_row + out_bytes)
        res[name] = {"ms": ms, "gbs": moved / (ms * 1e-3) / 1e9}
    return res


def radius_graph(n, side, cutoff, seed=0):
    from scipy.spatial import cKDTree

    rng = np.random.default_rng(seed)
    pos = rng.uniform(0.0, side, size=(n, 3))
    pairs = cKDTree(pos).query_pairs(cutoff, output_type="ndarray")
    src = np.concatenate([pairs[:, 0], pairs[:, 1]])
    dst = np.concatenate([pairs[:, 1], pairs[:, 0]])
    return pos, src.astype(np.int64), dst.astype(np.int64)


def radial_weights(r, cutoff, weight_numel, gen, dev):
    """8 Bessel functions -> 64 -> weight_numel, SiLU, N(0,1) weights, scaled as the reference's
    FullyConnectedNet (e3nn/nn/_fc.py:38-48; basis e3nn/math/_bessel.py:30-37).  Untimed input generation."""
    n = torch.arange(1, 9, dtype=torch.float32, device=dev)
    x = r[:, None]
    basis = math.sqrt(2.0 / cutoff) * torch.sin(n * math.pi / cutoff * x) / x
    w1 = torch.randn(8, 64, generator=gen).to(dev)
    w2 = torch.randn(64, weight_numel, generator=gen).to(dev)
    h = torch.nn.functional.silu(basis @ (w1 / math.sqrt(8))) * 1.679177  # second-moment normalisation of SiLU
    return (h @ (w2 / math.sqrt(64))).contiguous()


def bench_nequip(args, dev):
    from e3nn_amd import o3
    from e3nn_amd.nn import DstSortedEdges
    from e3nn_amd import kernel_sets as ks

    N, side, cutoff = 50_000, 86.8, 5.0
    pos, src_pairs, dst_pairs = radius_graph(N, side, cutoff)
    # The edge list as a neighbour search per node emits it: grouped by the node that asks for its neighbours, the
    # destination.  The reference's models build their graph with torch_cluster's radius_graph and take edge_index[1]
    # as edge_dst (e3nn/nn/models/gate_points_2101.py:322-324, v2106/gate_points_networks.py:69-71), which is that
    # order.  The order of the k-d tree's pair list (every pair once, then every pair reversed) is timed beside it
    # ("pair_order").
    order = np.argsort(dst_pairs, kind="stable")
    src, dst = src_pairs[order], dst_pairs[order]
    E = src.shape[0]
    gen = torch.Generator().manual_seed(0)
    tp = ks.cfg3(merged=True)
    node_x = torch.randn(N, tp.irreps_in1.dim, generator=gen).to(dev)
    pos_t = torch.from_numpy(pos).float().to(dev)
    src_t, dst_t = torch.from_numpy(src).to(dev), torch.from_numpy(dst).to(dev)
    vec = pos_t[src_t] - pos_t[dst_t]
    attr = o3.spherical_harmonics([0, 1, 2], vec, True, "component")
    w = radial_weights(vec.norm(dim=1), cutoff, tp.weight_numel, gen, dev)
    edges = DstSortedEdges(src_t, dst_t, N)  # first call: includes one-off lazy initialisation
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        edges = DstSortedEdges(src_t, dst_t, N)
    torch.cuda.synchronize()
    prep_ms = (time.perf_counter() - t0) * 1e3 / 5  # wall clock incl. allocation and the range-check read-backs
    assert edges.walk_perm is None  # grouped by destination already: the kernels walk the list by position

    out = [None]

    def step():
        # edge attributes = SH(lmax 2) of the edge vectors, formed inside the kernel from the 12-byte vectors
        out[0] = tp.forward_gather_scatter_sh(node_x, vec, w, edges, True, "component")

    ms, ms_median, ms_min = event_times_ms(step, args.steps, args.warmup)
    # algorithmic bytes: per edge weights + SH + two int64 indices, node table read once, output written once
    bytes_algo = E * (4 * tp.weight_numel + 4 * 9 + 2 * 8) + N * 4 * (tp.irreps_in1.dim + tp.irreps_out.dim)
    gbs = bytes_algo / (ms * 1e-3) / 1e9
    frac = lambda t: bytes_algo / (t * 1e-3) / 1e9 / HBM_PEAK_GBS  # noqa: E731
    res = {
        "edges": E, "nodes": N, "ms": ms, "ms_median": ms_median, "ms_min": ms_min, "edges_per_s": E / (ms * 1e-3),
        "bytes_per_launch": bytes_algo, "achieved_gbs": gbs, "edge_preprocessing_ms_per_graph": prep_ms,
        "kernel_key": tp._plan(torch.float32).key + "+sh",
        "edges_per_s_incl_preprocessing": E / ((ms + prep_ms) * 1e-3),
        # the kernel reads the 12-byte vectors where the algorithmic count has the 36-byte attribute rows
        "bytes_read_less_than_counted": E * 4 * (9 - 3),
    }  # fmt: skip
    ctx = dict(tp=tp, node_x=node_x, attr=attr, w=w, src=src_t, dst=dst_t, N=N, out=out[0], vec=vec)
    # the same call on stored edge attributes ([E, 9] read from memory)
    t = event_time_ms(lambda: tp.forward_gather_scatter(node_x, attr, w, edges=edges), args.steps, args.warmup)
    res["stored_edge_attr"] = {"ms": t, "edges_per_s": E / (t * 1e-3), "roofline_frac": frac(t)}
    # part of the default run; skipped when --only selects sections
    if getattr(args, "locality_variants", False) or getattr(args, "only", None) == "":
        # same graph: (a) the edge list in the k-d tree's pair order (the kernels then reach the per-edge tensors
        # through the permutation of the destination sort, built once per graph); (b) nodes renumbered along a Morton
        # curve of their positions (a spatially sorted system), edge list grouped by destination
        def timed(s_np, d_np, nx, a2, w2, v2):
            e2 = DstSortedEdges(torch.from_numpy(s_np).to(dev), torch.from_numpy(d_np).to(dev), N)
            return e2, {
                "harmonics_in_kernel": event_time_ms(lambda: tp.forward_gather_scatter_sh(nx, v2, w2, e2, True, "component"), args.steps, args.warmup),
                "stored_edge_attr": event_time_ms(lambda: tp.forward_gather_scatter(nx, a2, w2, edges=e2), args.steps, args.warmup),
            }  # fmt: skip

        inv = torch.from_numpy(np.argsort(order)).to(dev)  # position of pair-list edge e in the grouped list
        e_pairs, t_pairs = timed(src_pairs, dst_pairs, node_x, attr[inv].contiguous(), w[inv].contiguous(), vec[inv].contiguous())
        assert e_pairs.walk_perm is not None
        c = np.floor(pos / 2.5).astype(np.uint64)

        def spread(v):
            v = v & np.uint64(0x3FF)
            for sh, m in ((16, 0x30000FF), (8, 0x300F00F), (4, 0x30C30C3), (2, 0x9249249)):
                v = (v | (v << np.uint64(sh))) & np.uint64(m)
            return v

        key = spread(c[:, 0]) | (spread(c[:, 1]) << np.uint64(1)) | (spread(c[:, 2]) << np.uint64(2))
        rank = np.empty(N, np.int64)
        rank[np.argsort(key, kind="stable")] = np.arange(N)
        s2, d2 = rank[src], rank[dst]
        nx = torch.empty_like(node_x)
        nx[torch.from_numpy(rank).to(dev)] = node_x
        o = np.argsort(d2, kind="stable")
        ot = torch.from_numpy(o).to(dev)
        _, t_morton = timed(s2[o], d2[o], nx, attr[ot].contiguous(), w[ot].contiguous(), vec[ot].contiguous())
        for name, times in (("pair_order", t_pairs), ("morton_nodes", t_morton)):
            res[name] = {k: {"ms": t, "edges_per_s": E / (t * 1e-3), "roofline_frac": frac(t)} for k, t in times.items()}
    return res, ctx


def cpu_baseline_nequip(ctx, n_edges=200_000, reps=3):
    """The reference's CPU path (torch einsum graph + index + scatter_add_) on a slice of the same workload."""
    from oracle import tensor_product as otp
    from oracle.torch_cpu import tp_gather_scatter_torch

    torch.set_num_threads(os.cpu_count())
    tp = ctx["tp"]
    ins = [(t.i_in1, t.i_in2, t.i_out, t.connection_mode, t.has_weight) for t in tp.instructions]
    spec = otp.make_spec(str(tp.irreps_in1), str(tp.irreps_in2), str(tp.irreps_out), ins, shared_weights=tp.shared_weights)
    E = min(n_edges, ctx["src"].shape[0])
    node_x = ctx["node_x"].cpu()
    attr, w = ctx["attr"][:E].cpu(), ctx["w"][:E].cpu()
    src, dst = ctx["src"][:E].cpu(), ctx["dst"][:E].cpu()
    tp_gather_scatter_torch(spec, node_x, attr, w, src, dst, ctx["N"])
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        tp_gather_scatter_torch(spec, node_x, attr, w, src, dst, ctx["N"])
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    return {
        "value": E / t, "unit": "edges/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"first {E} edges of the same graph, fp32, median of {reps}, torch {torch.__version__} CPU einsum "
                  f"restatement of the reference graph ({os.cpu_count()} host cpus)",
    }  # fmt: skip


def bench_sh(args, dev):
    from e3nn_amd import o3

    n = 4_000_000
    gen = torch.Generator().manual_seed(0)
    d = torch.randn(n, 3, generator=gen)
    d = d / d.norm(dim=1, keepdim=True)
    x = (d * torch.exp(0.5 * torch.randn(n, 1, generator=gen))).to(dev)
    sh = o3.SphericalHarmonics([0, 1, 2, 3], True, "component")
    ms = event_time_ms(lambda: sh(x), args.steps, args.warmup)
    b = n * 76
    return {"vectors": n, "ms": ms, "mvec_per_s": n / (ms * 1e-3) / 1e6, "achieved_gbs": b / (ms * 1e-3) / 1e9,
            "roofline_frac": b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "bytes_per_launch": b}  # fmt: skip


def bench_mace(args, dev, dtype=torch.float32, variant="A"):
    """MACE-style uvu (L=3): variant A keeps 0e,1o,2e,3o outputs (23 paths), B every l <= 3 of either parity (34)."""
    from e3nn_amd.nn import DstSortedEdges
    from e3nn_amd import kernel_sets as ks

    N, E = 20_000, 500_000
    gen = torch.Generator().manual_seed(0)
    tp = ks.cfg4(variant)
    src = torch.randint(0, N, (E,), generator=gen, dtype=torch.int32).to(dev)
    dst = torch.randint(0, N, (E,), generator=gen, dtype=torch.int32).to(dev)
    node_x = torch.randn(N, tp.irreps_in1.dim, generator=gen).to(dev).to(dtype)
    from e3nn_amd import o3

    v = torch.randn(E, 3, generator=gen).to(dev)
    attr = o3.spherical_harmonics([0, 1, 2, 3], v, True, "component").to(dtype)
    w = torch.randn(E, tp.weight_numel, generator=gen).to(dev).to(dtype)
    edges = DstSortedEdges(src, dst, N)
    ms = event_time_ms(lambda: tp.forward_gather_scatter(node_x, attr, w, edges=edges), max(3, args.steps // 4), 2)
    fb = 2 if dtype == torch.bfloat16 else 4
    b = E * (fb * tp.weight_numel + fb * 16 + 2 * 4) + N * fb * (tp.irreps_in1.dim + tp.irreps_out.dim)
    out = {"edges": E, "nodes": N, "ms": ms, "edges_per_s": E / (ms * 1e-3), "achieved_gbs": b / (ms * 1e-3) / 1e9,
           "roofline_frac": b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "bytes_per_launch": b}  # fmt: skip
    if dtype == torch.float32 and variant == "A":
        # forward + backward with respect to node features, edge attributes and weights, from a fixed cotangent
        a, bb, c = (t.clone().requires_grad_(True) for t in (node_x, attr, w))
        cot = torch.randn(N, tp.irreps_out.dim, generator=gen).to(dev)

        def step():
            a.grad = bb.grad = c.grad = None
            tp.forward_gather_scatter(a, bb, c, edges=edges).backward(cot)

        out["ms_forward_backward"] = event_time_ms(step, max(3, args.steps // 10), 1)
    return out


def bench_uvw(args, dev, dtype=torch.float32):
    """Dense uvw: FCTP(128x0e+128x1o+128x2e x same -> same), 65536 rows, shared weights N(0, 1/fan_in)."""
    from e3nn_amd import kernel_sets as ks

    tp = ks.cfg5().to(dev)
    Z = 65536
    gen = torch.Generator().manual_seed(0)
    with torch.no_grad():
        tp.weight.copy_(torch.randn(tp.weight_numel, generator=gen) / 128.0)
    tp = tp.to(dtype)
    x1 = torch.randn(Z, 1152, generator=gen).to(dev).to(dtype)
    x2 = torch.randn(Z, 1152, generator=gen).to(dev).to(dtype)
    ms = event_time_ms(lambda: tp(x1, x2), 3, 1)
    f_min = 2 * Z * 128**3 * 21  # cheapest contraction order per path: sum of min(2l1+1, 2l2+1, 2l3+1) = 21
    f_gemm = 2 * Z * 128**3 * 35  # outer-product order: sum of (2l3+1) = 35
    peak = BF16_MFMA_PEAK_TFLOPS if dtype == torch.bfloat16 else FP32_MFMA_PEAK_TFLOPS
    arithmetic = tp._plan(dtype).arithmetic
    out = {"rows": Z, "ms": ms, "tflops_fmin": f_min / (ms * 1e-3) / 1e12, "tflops_fgemm_equiv": f_gemm / (ms * 1e-3) / 1e12,
           "roofline": {"bound": "mfma", "instruction": arithmetic, "achieved": f_min / (ms * 1e-3) / 1e12, "peak": peak,
                        "unit": "TFLOP/s", "frac": f_min / (ms * 1e-3) / 1e12 / peak}, "flops_per_launch": f_min}  # fmt: skip
    if dtype == torch.float32:
        out["roofline"].update(split_operand_fractions(arithmetic, f_min, ms))
        if "split" in arithmetic and not args.no_instruction_variants:  # the same product on the fp32 matrix instruction, as a plan of its own
            out["ms_fp32_instruction"] = with_env("E3X_UVW_SPLIT", "0", lambda: time_fresh_plan(ks.cfg5, tp.weight, x1, x2))
            out["roofline"]["frac_on_fp32_instruction"] = f_min / (out["ms_fp32_instruction"] * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS
    return out


def split_operand_fractions(arithmetic, flops, ms):
    """Both readings of an fp32 product that runs as six bf16 matrix products of three-way split operands:
    ``frac`` prices the 2mnk flops of the fp32 product against the fp32 matrix peak (what the caller gets);
    ``frac_of_bf16_peak_executed`` prices the six products the matrix cores execute against the peak of the instruction
    they execute.  On the fp32 instruction the two coincide and only ``frac`` is reported."""
    if "split" not in arithmetic:
        return {}
    return {"frac_fp32_equivalent": flops / (ms * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS,
            "frac_of_bf16_peak_executed": 6 * flops / (ms * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS}  # fmt: skip


def with_env(name, value, fn):
    """Runs ``fn`` with one environment variable set (the kernel generator reads its switches at plan creation)."""
    old = os.environ.get(name)
    os.environ[name] = value
    try:
        return fn()
    finally:
        if old is None:
            del os.environ[name]
        else:
            os.environ[name] = old


def time_fresh_plan(maker, weight, x1, x2):
    tp = maker().to(x1.device)
    with torch.no_grad():
        tp.weight.copy_(weight)
    assert "split" not in tp._plan(torch.float32).arithmetic
    return event_time_ms(lambda: tp(x1, x2), 3, 1)


def bench_nequip_cube40(args, dev):
    """The headline configuration as literally stated: 50 000 nodes in a 40 A cube, 5 A cutoff (degree ~354)."""
    from e3nn_amd import o3
    from e3nn_amd.nn import DstSortedEdges
    from e3nn_amd import kernel_sets as ks

    N, side, cutoff = 50_000, 40.0, 5.0
    pos, src, dst = radius_graph(N, side, cutoff)
    E = src.shape[0]
    gen = torch.Generator().manual_seed(0)
    tp = ks.cfg3(merged=True)
    node_x = torch.randn(N, tp.irreps_in1.dim, generator=gen).to(dev)
    pos_t = torch.from_numpy(pos).float().to(dev)
    src_t, dst_t = torch.from_numpy(src).to(dev), torch.from_numpy(dst).to(dev)
    vec = pos_t[src_t] - pos_t[dst_t]
    attr = o3.spherical_harmonics([0, 1, 2], vec, True, "component")
    r = vec.norm(dim=1)
    del pos_t
    w = torch.empty(E, tp.weight_numel, device=dev)
    step = 2_000_000  # radial MLP in slices: its hidden activations are not kept
    for a in range(0, E, step):
        w[a : a + step] = radial_weights(r[a : a + step], cutoff, tp.weight_numel, torch.Generator().manual_seed(0), dev)
    edges = DstSortedEdges(src_t, dst_t, N)
    ms = event_time_ms(lambda: tp.forward_gather_scatter(node_x, attr, w, edges=edges), max(5, args.steps // 5), 2)
    b = E * (4 * tp.weight_numel + 4 * 9 + 2 * 8) + N * 4 * (tp.irreps_in1.dim + tp.irreps_out.dim)
    out = {"edges": E, "nodes": N, "ms": ms, "edges_per_s": E / (ms * 1e-3), "achieved_gbs": b / (ms * 1e-3) / 1e9,
           "roofline_frac": b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "bytes_per_launch": b}  # fmt: skip
    # as the headline is run: the list grouped by destination, the harmonics formed in the kernel (same algorithmic bytes)
    del attr, edges
    order = torch.sort(dst_t, stable=True).indices
    src_g, dst_g, vec_g = src_t[order], dst_t[order], vec[order].contiguous()
    w_g = torch.empty_like(w)
    for a in range(0, E, step):  # in slices: the permuted copy is 25 GB
        w_g[a : a + step] = w[order[a : a + step]]
    del w, vec, order
    edges_g = DstSortedEdges(src_g, dst_g, N)
    ms_g = event_time_ms(lambda: tp.forward_gather_scatter_sh(node_x, vec_g, w_g, edges_g, True, "component"), max(5, args.steps // 5), 2)
    out["grouped_by_destination_harmonics_in_kernel"] = {"ms": ms_g, "edges_per_s": E / (ms_g * 1e-3), "roofline_frac": b / (ms_g * 1e-3) / 1e9 / HBM_PEAK_GBS}
    return out


def bench_convolution(args, dev, ctx):
    """One whole interaction block (reference e3nn/nn/models/v2106/points_convolution.py:99-113) on the headline
    graph: radial network 8 -> 64 -> 352, self-connection, lin1, fused message, lin2, alpha; 4 species."""
    from e3nn_amd.nn import DstSortedEdges
    from e3nn_amd import kernel_sets as ks

    conv = ks.conv_wide().to(dev)
    N, E = ctx["N"], ctx["src"].shape[0]
    gen = torch.Generator().manual_seed(0)
    node_attr = torch.nn.functional.one_hot(torch.randint(0, 4, (N,), generator=gen), 4).float().to(dev)
    edge_scalars = torch.randn(E, 8, generator=gen).to(dev)
    edges = DstSortedEdges(ctx["src"], ctx["dst"], N)
    x = ctx["node_x"].clone().requires_grad_(True)

    def fwd():
        with torch.no_grad():
            return conv(x, node_attr, ctx["src"], ctx["dst"], ctx["attr"], edge_scalars, edges=edges)

    cot = torch.randn(N, conv.irreps_node_output.dim, generator=gen).to(dev)

    def fwd_bwd():  # from a fixed cotangent: no loss function in the timed region
        x.grad = None
        conv.zero_grad(set_to_none=True)
        conv(x, node_attr, ctx["src"], ctx["dst"], ctx["attr"], edge_scalars, edges=edges).backward(cot)

    ms_f = event_time_ms(fwd, max(5, args.steps // 5), 2)
    ms_fb = event_time_ms(fwd_bwd, max(3, args.steps // 10), 1)
    return {"edges": E, "nodes": N, "ms_forward": ms_f, "ms_forward_backward": ms_fb, "edges_per_s_forward": E / (ms_f * 1e-3)}


def bench_radial_network(args, dev, ctx):
    """The radial network of the block above, 8 -> 64 -> 352 with SiLU (reference e3nn/nn/_fc.py:38-48,70-88), on all
    edges of the headline graph: as ONE kernel (no gradient wanted) and layer by layer (the path that has a backward)."""
    from e3nn_amd.nn import FullyConnectedNet

    E = ctx["src"].shape[0]
    net = FullyConnectedNet([8, 64, 352], torch.nn.functional.silu).to(dev)
    x = torch.randn(E, 8, generator=torch.Generator().manual_seed(0)).to(dev)

    def one_kernel():
        with torch.no_grad():
            return net(x)

    def layered():
        return net(x)  # parameters require a gradient: tensor-product and gate kernels, one pair per layer

    assert net.fused_plan().handle is not None
    ms1 = event_time_ms(one_kernel, max(5, args.steps // 2), 3)
    msl = event_time_ms(layered, max(5, args.steps // 5), 2)
    # the backward kernels of the 64 -> 352 layer alone, back to back on random data: weight gradient (SiLU applied to
    # the saved pre-activations as they are loaded) and input gradient (SiLU derivative in the epilogue)
    fwd, bwd = net.layer1.act_dense_plans(net.layer0)
    z = torch.randn(E, 64, generator=torch.Generator().manual_seed(1)).to(dev)
    g = torch.randn(E, 352, generator=torch.Generator().manual_seed(2)).to(dev)
    wt = net.layer1.weight.detach().t().contiguous()
    ms_dw = event_time_ms(lambda: fwd.backward_w(z, g), max(5, args.steps // 5), 2)
    ms_dx = event_time_ms(lambda: bwd.forward(g, [wt], z), max(5, args.steps // 5), 2)
    flop = 2.0 * E * (8 * 64 + 64 * 352)
    out_bytes = E * (8 + 352) * 4
    return {"edges": E, "ms_one_kernel": ms1, "ms_layer_by_layer": msl, "ms_weight_gradient_64x352": ms_dw,
            "ms_input_gradient_352_to_64": ms_dx, "tflops_one_kernel": flop / (ms1 * 1e-3) / 1e12,
            "frac_fp32_mfma_peak": flop / (ms1 * 1e-3) / 1e12 / 157.3, "hbm_gbs_one_kernel": out_bytes / (ms1 * 1e-3) / 1e9,
            "frac_hbm_peak": out_bytes / (ms1 * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "arithmetic": "layer 64->352: six bf16 MFMA products of three-way split operands, fp32 accumulation (fp32-accurate); "
                          "tflops / frac_fp32_mfma_peak count the 2*m*n*k flops of the fp32 product"}  # fmt: skip


def bench_radial_message(args, dev, ctx):
    """weight = fc(edge_scalars); scatter(tp(x[src], attr, weight), dst) on the headline graph and instruction set
    (reference e3nn/nn/models/v2106/points_convolution.py:99-106): the radial network 8 -> 64 -> 352 inside the message
    kernel, against the two kernels run one after the other."""
    from e3nn_amd.nn import DstSortedEdges, FullyConnectedNet

    tp, E = ctx["tp"], ctx["src"].shape[0]
    torch.manual_seed(0)
    net = FullyConnectedNet([8, 64, tp.weight_numel], torch.nn.functional.silu).to(dev)
    s = torch.randn(E, 8, generator=torch.Generator().manual_seed(1)).to(dev)
    edges = DstSortedEdges(ctx["src"], ctx["dst"], ctx["N"])
    with torch.no_grad():
        fused = tp.forward_gather_scatter_radial(ctx["node_x"], ctx["attr"], s, net, edges)
        assert fused is not None
        ref = tp.forward_gather_scatter(ctx["node_x"], ctx["attr"], net(s), edges=edges)
        err = float((fused - ref).abs().max()) / max(1.0, float(ref.abs().max()))
        assert err < 1e-4, err
        ms_f = event_time_ms(lambda: tp.forward_gather_scatter_radial(ctx["node_x"], ctx["attr"], s, net, edges), max(5, args.steps // 2), 3)
        ms_s = event_time_ms(lambda: tp.forward_gather_scatter(ctx["node_x"], ctx["attr"], net(s), edges=edges), max(5, args.steps // 2), 3)
    flop = 2.0 * E * (8 * 64 + 64 * tp.weight_numel)
    return {"edges": E, "ms_one_kernel": ms_f, "ms_network_then_message": ms_s, "edges_per_s_one_kernel": E / (ms_f * 1e-3),
            "network_tflops_one_kernel": flop / (ms_f * 1e-3) / 1e12, "max_rel_difference": err}  # fmt: skip


def bench_library_gemm(args, dev):
    """Context for the matrix-core rooflines: what the vendor GEMM (torch.matmul -> rocBLAS / hipBLASLt) reaches
    on this GPU with N(0,1) data, 8192^3."""
    out = {}
    n = 8192
    for name, dt in (("bf16", torch.bfloat16), ("f32", torch.float32)):
        a = torch.randn(n, n, device=dev).to(dt)
        b = torch.randn(n, n, device=dev).to(dt)
        ms = event_time_ms(lambda: a @ b, 5, 2)
        out[name + "_tflops"] = 2 * n**3 / (ms * 1e-3) / 1e12
    return out


def bench_nequip_backward(args, dev, ctx):
    """Forward + backward of the headline convolution: gradients with respect to node features, edge
    attributes and per-edge weights, from a fixed cotangent."""
    from e3nn_amd.nn import DstSortedEdges

    tp = ctx["tp"]
    edges = DstSortedEdges(ctx["src"], ctx["dst"], ctx["N"])
    a, b, c = (ctx[k].clone().requires_grad_(True) for k in ("node_x", "attr", "w"))
    cot = torch.randn(ctx["N"], tp.irreps_out.dim, device=dev)

    def step():
        a.grad = b.grad = c.grad = None
        tp.forward_gather_scatter(a, b, c, edges=edges).backward(cot)

    ms = event_time_ms(step, max(5, args.steps // 5), 2)
    # node features and weights only (an energy-only training step)
    a2, c2 = (ctx[k].clone().requires_grad_(True) for k in ("node_x", "w"))

    def step_xw():
        a2.grad = c2.grad = None
        tp.forward_gather_scatter(a2, ctx["attr"], c2, edges=edges).backward(cot)

    ms_xw = event_time_ms(step_xw, max(5, args.steps // 5), 2)
    E = ctx["src"].shape[0]
    return {"edges": E, "ms_forward_backward": ms, "ms_forward_backward_node_features_and_weights": ms_xw,
            "edges_per_s": E / (ms * 1e-3)}


def bench_uvw_backward(args, dev):
    """Dense uvw (fp32), forward + backward with respect to both inputs and the shared weights, and the
    weight-gradient kernel alone against the matrix-core peak."""
    from e3nn_amd import kernel_sets as ks

    tp = ks.cfg5().to(dev)
    Z = 65536
    gen = torch.Generator().manual_seed(0)
    with torch.no_grad():
        tp.weight.copy_(torch.randn(tp.weight_numel, generator=gen) / 128.0)
    x1 = torch.randn(Z, 1152, generator=gen).to(dev).requires_grad_(True)
    x2 = torch.randn(Z, 1152, generator=gen).to(dev).requires_grad_(True)
    cot = torch.randn(Z, 1152, generator=gen).to(dev)

    def step():
        x1.grad = x2.grad = tp.weight.grad = None
        tp(x1, x2).backward(cot)

    ms = event_time_ms(step, 2, 1)
    plan = tp._plan(torch.float32)
    a, b = x1.detach(), x2.detach()
    ms_dw = event_time_ms(lambda: plan.backward_w_uvw(a, b, cot, True), 3, 1)
    f_min = 2 * Z * 128**3 * 21
    arithmetic = plan.arithmetic_weight_gradient
    roof = {"bound": "mfma", "instruction": arithmetic, "achieved": f_min / (ms_dw * 1e-3) / 1e12, "peak": FP32_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": f_min / (ms_dw * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS}  # fmt: skip
    roof.update(split_operand_fractions(arithmetic, f_min, ms_dw))
    out = {"rows": Z, "ms_forward_backward": ms, "ms_weight_gradient": ms_dw, "roofline_weight_gradient": roof}
    if "split" in arithmetic and not args.no_instruction_variants:

        def fp32_instruction():
            tp2 = ks.cfg5().to(dev)
            plan2 = tp2._plan(torch.float32)
            ms2 = event_time_ms(lambda: plan2.backward_w_uvw(a, b, cot, True), 3, 1)
            assert "split" not in plan2.arithmetic_weight_gradient
            return ms2

        out["ms_weight_gradient_fp32_instruction"] = with_env("E3X_DW_SPLIT", "0", fp32_instruction)
        roof["frac_on_fp32_instruction"] = f_min / (out["ms_weight_gradient_fp32_instruction"] * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--locality-variants", action="store_true", help="time the headline graph with sorted edges / Morton node ids also when --only is given")
    ap.add_argument("--no-headline", action="store_true", help="profiling aid: run only the sections of --only (those that do not build on the headline graph) and print their results, so that a profile holds the launches of one configuration only")
    ap.add_argument("--no-instruction-variants", action="store_true", help="profiling aid: do not time config 5 on the fp32 matrix instruction beside the default kernels, so that a profile holds one code object per kernel name")
    ap.add_argument("--only", default="", help="comma list of extra sections to run: copy,sh,mace,mace_b,mace_bf16,nequip40,uvw,uvw_bf16,conv,radial,nequip_bwd,uvw_bwd (default: all)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported (no collectives, no sharding)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    from e3nn_amd.csrc.build import ensure_built

    ensure_built()  # a tree that was never built: compile the library (kernels are specialised on first use)

    if args.no_headline:
        sections = {"copy": lambda: bench_copy(args, dev), "sh": lambda: bench_sh(args, dev), "mace": lambda: bench_mace(args, dev),
                    "mace_b": lambda: bench_mace(args, dev, variant="B"), "mace_bf16": lambda: bench_mace(args, dev, torch.bfloat16),
                    "nequip40": lambda: bench_nequip_cube40(args, dev), "uvw": lambda: bench_uvw(args, dev),
                    "uvw_bf16": lambda: bench_uvw(args, dev, torch.bfloat16), "uvw_bwd": lambda: bench_uvw_backward(args, dev)}  # fmt: skip
        names = [n for n in args.only.split(",") if n]
        if not names or any(n not in sections for n in names):
            sys.exit("bench.py --no-headline needs --only with sections out of: " + ",".join(sections))
        print(json.dumps({"sections_only": {n: sections[n]() for n in names}}))
        return

    neq, ctx = bench_nequip(args, dev)
    other = {"nequip_uvu": neq}
    want = set(args.only.split(",")) if args.only else {"copy", "sh", "mace", "mace_b", "mace_bf16", "nequip40", "uvw", "uvw_bf16", "conv", "radial", "nequip_bwd", "uvw_bwd"}
    if "copy" in want:
        other["copy_1GiB"] = bench_copy(args, dev)
        other["stream_rows_headline_bytes"] = bench_stream_rows(args, dev, neq["nodes"], neq["bytes_per_launch"], 4 * ctx["tp"].irreps_out.dim)
    if "sh" in want:
        other["sh_lmax3_4M"] = bench_sh(args, dev)
    if "mace" in want:
        other["mace_uvu_fp32"] = bench_mace(args, dev)
    if "mace_b" in want:
        other["mace_uvu_fp32_variant_b"] = bench_mace(args, dev, variant="B")
    if "nequip40" in want:
        other["nequip_uvu_cube40"] = bench_nequip_cube40(args, dev)
    if "mace_bf16" in want:
        other["mace_uvu_bf16_storage"] = bench_mace(args, dev, torch.bfloat16)
    if "uvw" in want:
        other["uvw_dense_fp32"] = bench_uvw(args, dev)
    if "uvw_bf16" in want:
        other["uvw_dense_bf16"] = bench_uvw(args, dev, torch.bfloat16)
    if "uvw" in want or "uvw_bf16" in want:
        other["library_gemm_8192_randn"] = bench_library_gemm(args, dev)
    if "conv" in want:
        other["convolution_block"] = bench_convolution(args, dev, ctx)
    if "radial" in want:
        other["radial_network_8_64_352"] = bench_radial_network(args, dev, ctx)
    if "radial" in want:
        other["nequip_message_with_radial_network"] = bench_radial_message(args, dev, ctx)
    if "nequip_bwd" in want:
        other["nequip_uvu_forward_backward"] = bench_nequip_backward(args, dev, ctx)
    if "uvw_bwd" in want:
        other["uvw_dense_fp32_forward_backward"] = bench_uvw_backward(args, dev)
    line = {
        "metric": "per-edge uvu TP edges/sec (L=2, fused gather + tensor product + scatter)",
        "value": neq["edges_per_s"],
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": neq["ms"],
        "ms_per_step_median": neq["ms_median"],
        "ms_per_step_min": neq["ms_min"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "NequIP-style uvu interaction: N=50000 nodes, cube side 86.8 A, 5 A cutoff radius graph "
                        f"(E={neq['edges']}, edge list grouped by destination as a neighbour search emits it), 32x0e+32x1o+32x2e x SH(lmax 2) "
                        "of the edge vectors (formed in the kernel), 11 paths, 352 weights/edge from a radial MLP (an input), int64 indices, "
                        "fused scatter-sum; row pointers built once per graph, outside the timed region (edge_preprocessing_ms_per_graph)",
        },
        "roofline": {
            "bound": "hbm", "achieved": neq["achieved_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": neq["achieved_gbs"] / HBM_PEAK_GBS, "traffic": NEQUIP_TRAFFIC_BYTES.get(neq["kernel_key"]), "kernel": "e3x_uvu_sh_fused",
            "algorithmic_bytes": neq["bytes_per_launch"],
            # the same bytes streamed by a kernel that does nothing else (e3x_stream_rows), measured in this run
            "stream_same_bytes_gbs": other.get("stream_rows_headline_bytes", {}).get("read_and_row_stores", {}).get("gbs"),
        },
        "other": other,
    }  # fmt: skip
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_nequip(ctx)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
