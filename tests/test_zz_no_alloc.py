"""e3x_csr_build_static (sort buffers in a static device array, no allocation) against e3x_csr_build.

Integer work: the row pointers and the permutation must be bit-identical.  Two calls in a row share the static
buffers, the second on a smaller edge list, so stale contents of the first call must not leak into it.
"""
import numpy as np
import pytest
import torch

from e3nn_amd import _lib

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _build(dst, N, static):
    L = _lib.lib()
    E = dst.numel()
    rowptr = torch.full((N + 1,), -7, dtype=torch.int32, device=DEV)
    perm = torch.full((max(E, 1),), -7, dtype=torch.int32, device=DEV)
    st = _lib.stream_ptr(DEV)
    bits = dst.element_size() * 8
    if static:
        rc = L.e3x_csr_build_static(_lib.ptr(dst), bits, E, N, _lib.ptr(rowptr), _lib.ptr(perm), st)
    else:
        nbytes = L.e3x_csr_workspace_bytes(E, N)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=DEV)
        rc = L.e3x_csr_build(_lib.ptr(dst), bits, E, N, _lib.ptr(rowptr), _lib.ptr(perm), _lib.ptr(ws), nbytes, st)
    _lib.check(rc)
    torch.cuda.synchronize()
    return rowptr.cpu().numpy(), perm[:E].cpu().numpy()


def _reference(dst, N):
    d = dst.cpu().numpy().astype(np.int64)
    perm = np.argsort(d, kind="stable").astype(np.int32)
    rowptr = np.searchsorted(d[perm], np.arange(N + 1), side="left").astype(np.int32)
    return rowptr, perm


def test_static_scratch_matches_workspace_entry_point_twice_in_a_row():
    g = torch.Generator().manual_seed(5)
    cases = [(200_000, 30_000, torch.int64), (4_321, 97, torch.int32), (0, 11, torch.int64)]
    with torch.cuda.device(DEV):
        for E, N, dt in cases:  # big, then smaller, then empty: all on the same static buffers
            dst = torch.randint(0, N, (E,), generator=g).to(dt).to(DEV)
            rp_s, pm_s = _build(dst, N, static=True)
            rp_w, pm_w = _build(dst, N, static=False)
            rp_r, pm_r = _reference(dst, N)
            assert np.array_equal(rp_s, rp_w) and np.array_equal(pm_s, pm_w), (E, N)
            assert np.array_equal(rp_s, rp_r) and np.array_equal(pm_s, pm_r), (E, N)


def test_static_scratch_reports_bad_indices_and_clears_the_flag():
    with torch.cuda.device(DEV):
        bad = torch.tensor([0, 3, 9, 1], dtype=torch.int64, device=DEV)
        with pytest.raises(IndexError):
            _build(bad, 5, static=True)
        good = torch.tensor([0, 3, 4, 1], dtype=torch.int64, device=DEV)  # the flag of the failed call is gone
        rp, pm = _build(good, 5, static=True)
        assert rp.tolist() == [0, 1, 2, 2, 3, 4] and pm.tolist() == [0, 3, 1, 2]


def test_static_scratch_rejects_edge_lists_beyond_its_buffers():
    L = _lib.lib()
    cap = L.e3x_csr_static_scratch_bytes()
    E = 1 << 21
    assert L.e3x_csr_workspace_bytes(E, 1 << 20) <= cap  # the documented size always fits
    too_many = cap // 4  # three 4-byte arrays per edge alone exceed the buffer
    one = torch.zeros(1, dtype=torch.int32, device=DEV)
    rc = L.e3x_csr_build_static(_lib.ptr(one), 32, too_many, 8, _lib.ptr(one), _lib.ptr(one), _lib.stream_ptr(DEV))
    assert rc == _lib.ERR_INVALID
    assert b"static buffer" in L.e3x_last_error()


def test_static_scratch_host_threads_take_turns():
    # two host threads on streams of their own share the device's one array; the library serialises them (a per-device
    # lock from the first launch to the final synchronisation), so both get the right answer
    import threading

    g = torch.Generator().manual_seed(9)
    jobs = [(150_000, 20_000), (90_000, 7_000)]
    dsts = [torch.randint(0, N, (E,), generator=g).to(DEV) for E, N in jobs]
    results = [None, None]

    def work(i):
        L = _lib.lib()
        E, N = jobs[i]
        with torch.cuda.device(DEV):
            stream = torch.cuda.Stream(device=DEV)
            rowptr = torch.empty(N + 1, dtype=torch.int32, device=DEV)
            perm = torch.empty(E, dtype=torch.int32, device=DEV)
            torch.cuda.synchronize()
            for _ in range(5):
                rc = L.e3x_csr_build_static(_lib.ptr(dsts[i]), 64, E, N, _lib.ptr(rowptr), _lib.ptr(perm), _lib.c_void_p(stream.cuda_stream))
                if rc != 0:
                    results[i] = rc
                    return
            stream.synchronize()
            results[i] = (rowptr.cpu().numpy(), perm.cpu().numpy())

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for i, (E, N) in enumerate(jobs):
        assert isinstance(results[i], tuple), results[i]
        rp, pm = _reference(dsts[i], N)
        assert np.array_equal(results[i][0], rp) and np.array_equal(results[i][1], pm)
