"""The dispatch entry point that allocates nothing (`moe_histogram_scan_static`): called through
the C ABI with caller-owned inputs and outputs, its results must equal, bit for bit, those of
the entry point that takes a workspace, on two calls in a row (the second with a smaller input,
so that the scratch array still holds the first call's histograms), and sizes beyond the fixed
scratch must be refused."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _outputs(R, E):
    i32 = lambda n: torch.full((n,), -7, dtype=torch.int32, device="cuda")
    return i32(E), i32(E + 1), i32(R), i32(R), i32(1)


def _call_static(L, ids, E):
    R = ids.numel()
    counts, offs, p2r, r2p, bad = _outputs(R, E)
    stream = torch.cuda.current_stream().cuda_stream
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    L.call("moe_histogram_scan_static", ids.data_ptr(), R, E, counts.data_ptr(), offs.data_ptr(),
           p2r.data_ptr(), r2p.data_ptr(), bad.data_ptr(), stream)
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # nothing came from torch's allocator
    return counts, offs, p2r, r2p, bad


def _call_workspace(L, ids, E):
    R = ids.numel()
    counts, offs, p2r, r2p, bad = _outputs(R, E)
    nbytes = L.cdll.moe_dispatch_workspace_bytes(R, E)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    L.call("moe_histogram_scan_checked", ids.data_ptr(), R, E, counts.data_ptr(), offs.data_ptr(),
           p2r.data_ptr(), r2p.data_ptr(), bad.data_ptr(), ws.data_ptr(), ws.numel(),
           torch.cuda.current_stream().cuda_stream)
    return counts, offs, p2r, r2p, bad


def test_static_scratch_dispatch_equals_the_workspace_entry(pkg, lib):
    assert torch.cuda.is_available()
    L = lib
    assert L.cdll.moe_static_scratch_bytes() == 4 << 20
    rng = np.random.default_rng(5)
    # two calls in a row on the same stream; the second is smaller and has fewer experts, so
    # its histograms overlay a part of what the first left in the scratch array
    cases = [(131072, 64), (5000, 16), (70000, 512), (300, 9), (0, 4), (1, 1)]
    for R, E in cases:
        print("static dispatch R", R, "E", E, flush=True)
        ids_np = rng.integers(0, E, size=R)
        if R >= 300:
            ids_np[rng.choice(R, size=3, replace=False)] = E + 5   # invalid ids are counted the same way
        ids = torch.from_numpy(ids_np.astype(np.int32)).cuda()
        got = _call_static(L, ids, E)
        want = _call_workspace(L, ids, E)
        torch.cuda.synchronize()
        for a, b, name in zip(got, want, ("counts", "offs", "pos_to_row", "row_to_pos", "bad_ids")):
            assert torch.equal(a, b), (R, E, name)
        assert got[4].item() == (3 if R >= 300 else 0)
        assert got[1][-1].item() == R
        # and against numpy, not only against the library's other entry: counts, offsets, the
        # stable sort by expert and its inverse (ids outside [0, E) go with the nearest expert)
        clipped = np.clip(ids_np, 0, E - 1)
        np_counts = np.bincount(clipped, minlength=E)
        np_p2r = np.argsort(clipped, kind="stable")
        assert np.array_equal(got[0].cpu().numpy(), np_counts), (R, E)
        assert np.array_equal(got[1].cpu().numpy(), np.concatenate([[0], np.cumsum(np_counts)])), (R, E)
        assert np.array_equal(got[2].cpu().numpy(), np_p2r), (R, E)
        inv = np.empty(R, dtype=np.int64)
        inv[np_p2r] = np.arange(R)
        assert np.array_equal(got[3].cpu().numpy(), inv), (R, E)
    # the documented limit, from both sides: the largest size that fits is accepted (and right),
    # one row more is refused with nothing enqueued
    E = 512
    R_max = L.cdll.moe_static_scratch_max_rows(E)
    assert R_max == (4 << 20) // (4 * (E + 1)) * 256 == 523264
    assert L.cdll.moe_static_scratch_max_rows(64) == 4129536
    assert L.cdll.moe_dispatch_workspace_bytes(R_max, E) <= L.cdll.moe_static_scratch_bytes()
    assert L.cdll.moe_dispatch_workspace_bytes(R_max + 1, E) > L.cdll.moe_static_scratch_bytes()
    ids_np = rng.integers(0, E, size=R_max)
    ids = torch.from_numpy(ids_np.astype(np.int32)).cuda()
    got = _call_static(L, ids, E)
    torch.cuda.synchronize()
    assert np.array_equal(got[0].cpu().numpy(), np.bincount(ids_np, minlength=E))
    assert np.array_equal(got[2].cpu().numpy(), np.argsort(ids_np, kind="stable"))
    R = R_max + 1
    ids = torch.zeros(R, dtype=torch.int32, device="cuda")
    counts, offs, p2r, r2p, bad = _outputs(R, E)
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_WORKSPACE"):
        L.call("moe_histogram_scan_static", ids.data_ptr(), R, E, counts.data_ptr(), offs.data_ptr(),
               p2r.data_ptr(), r2p.data_ptr(), bad.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert (counts == -7).all()


def test_static_scratch_dispatch_inside_a_captured_graph(pkg, lib):
    """What the entry point is for: recorded into a HIP graph (where nothing may allocate) and
    replayed on new contents of the same buffers, with eager work and synchronisations between
    the replays; every replay against the workspace entry run eagerly on the same ids."""
    L = lib
    R, E = 40000, 64
    rng = np.random.default_rng(8)
    ids = torch.zeros(R, dtype=torch.int32, device="cuda")
    outs = _outputs(R, E)

    def record():
        L.call("moe_histogram_scan_static", ids.data_ptr(), R, E, outs[0].data_ptr(), outs[1].data_ptr(),
               outs[2].data_ptr(), outs[3].data_ptr(), outs[4].data_ptr(),
               torch.cuda.current_stream().cuda_stream)

    # the set-up call (it looks the scratch array's address up on this device), so that the first
    # call of the entry point may be the captured one
    assert L.cdll.moe_static_scratch_bytes() == 4 << 20
    _call_workspace(L, ids, E)   # (the kernels' code is loaded by an eager launch, not under capture)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        record()
    for rep in range(4):
        new = rng.integers(0, E, size=R).astype(np.int32)
        new[rng.choice(R, size=rep, replace=False)] = -1 - rep   # rep invalid ids
        ids.copy_(torch.from_numpy(new))
        for o in outs:
            o.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        want = _call_workspace(L, ids, E)
        torch.cuda.synchronize()
        for a, b, name in zip(outs, want, ("counts", "offs", "pos_to_row", "row_to_pos", "bad_ids")):
            assert torch.equal(a, b), (rep, name)
        assert outs[4].item() == rep
        # unrelated eager work on the same device between replays
        _ = (torch.randn(1 << 20, device="cuda") * 2).sum().item()
