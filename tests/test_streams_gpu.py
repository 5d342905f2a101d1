"""Concurrent GEMMs on different streams, and the bookkeeping of the per-workspace scratch regions.

The reference allows one `mul` at a time per workspace (fp6_marlin_cuda.cpp:62-63; the locks live there,
fp6_marlin_cuda_kernel.cu:79-98), so calls on different streams with different workspaces may overlap.  Here the
fp32 partial tiles of split column tiles live in a region the library keeps per workspace address: the same calls
must give the serial results bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def operands(m, k, n, qc, gs, seed):
    g = torch.Generator().manual_seed(seed)
    n4 = n - qc
    B = torch.randint(-2 ** 31, 2 ** 31 - 1, (k * n4 // 8 + k * qc * 3 // 16,), generator=g, dtype=torch.int64).to(torch.int32)
    s = (torch.rand((k // gs) * n4 + qc, generator=g) * 0.01 + 0.001).half()
    A = torch.randn((m, k), generator=g).half()
    return A.cuda(), B.cuda(), s.cuda()


def test_two_streams_two_workspaces_match_serial_results():
    import fp6_marlin
    qc, gs = 256, 128
    # both problems split k across workgroups (partial tiles through the scratch): few column tiles, long k
    probs = [(1, 4096, 4096), (16, 11008, 4096), (64, 8192, 2048), (4, 8192, 8192)]
    ops = [operands(m, k, n, qc, gs, 100 + i) for i, (m, k, n) in enumerate(probs)]
    ws = [torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda") for (_, _, n) in probs]
    serial = []
    for (m, k, n), (A, B, s), w in zip(probs, ops, ws):
        C = torch.full((m, n), float("nan"), dtype=torch.half, device="cuda")
        fp6_marlin.mul(A, B, C, s, w, qc, -1, -1, -1, 16, gs)
        torch.cuda.synchronize()
        serial.append(C)
    streams = [torch.cuda.Stream() for _ in probs]
    rounds = 40
    outs = [[torch.full_like(serial[i], float("nan")) for _ in range(rounds)] for i in range(len(probs))]
    torch.cuda.synchronize()
    for r in range(rounds):                                              # no synchronisation between the launches
        for i, ((m, k, n), (A, B, s)) in enumerate(zip(probs, ops)):
            with torch.cuda.stream(streams[i]):
                fp6_marlin.mul(A, B, outs[i][r], s, ws[i], qc, -1, -1, -1, 16, gs)
    torch.cuda.synchronize()
    for i in range(len(probs)):
        for r in range(rounds):
            assert torch.equal(outs[i][r], serial[i]), (probs[i], r)
        assert int(ws[i].abs().sum()) == 0
    for w in ws:
        fp6_marlin.release_workspace(w)


def test_more_workspaces_than_the_region_table_holds():
    """The library keeps 16 regions per device (four built in, the others allocated once and kept).  A workspace it has
    not seen takes a free region, else the one that has gone unused longest, after waiting for the device -- so a
    caller that makes a new workspace per call, like the reference's harness, never runs out.  Results stay right
    throughout, released regions are taken again, and a call under capture that would have to wait is refused."""
    import fp6_marlin
    qc, gs = 256, 128
    m, k, n = 4, 2048, 512                                               # few column tiles, long k: k is split
    A, B, s = operands(m, k, n, qc, gs, 7)
    first = torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda")
    want = torch.full((m, n), float("nan"), dtype=torch.half, device="cuda")
    fp6_marlin.mul(A, B, want, s, first, qc, -1, -1, -1, 16, gs)
    torch.cuda.synchronize()
    keep = [torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda") for _ in range(40)]   # 40 distinct addresses
    assert len({w.data_ptr() for w in keep}) == 40
    for i, w in enumerate(keep):
        C = torch.full((m, n), float("nan"), dtype=torch.half, device="cuda")
        fp6_marlin.mul(A, B, C, s, w, qc, -1, -1, -1, 16, gs)
        assert torch.equal(C, want), i
        fp6_marlin.mul(A, B, C, s, first, qc, -1, -1, -1, 16, gs)       # (keeps `first` recently used: it stays)
        assert torch.equal(C, want), i
    # every region is taken now: a capture with yet another workspace cannot wait for the device and is refused ...
    fresh = torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda")
    C = torch.full((m, n), float("nan"), dtype=torch.half, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="scratch"):
        with torch.cuda.graph(graph):
            fp6_marlin.mul(A, B, C, s, fresh, qc, -1, -1, -1, 16, gs)
    # ... unless a region is free, or the workspace got one ahead of the capture
    fp6_marlin.release_workspace(keep[-1])
    fp6_marlin.release_workspace(keep[-1])                               # a second time: nothing to do
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fp6_marlin.mul(A, B, C, s, fresh, qc, -1, -1, -1, 16, gs)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(C, want)
    fp6_marlin.release_workspace(device=0)                               # all of them
    C = torch.full((m, n), float("nan"), dtype=torch.half, device="cuda")
    fp6_marlin.mul(A, B, C, s, first, qc, -1, -1, -1, 16, gs)
    torch.cuda.synchronize()
    assert torch.equal(C, want)


def test_first_calls_allocate_nothing_and_can_be_captured():
    """An ordinary `mul` with a workspace the library has never seen takes one of its four built-in scratch slots:
    no device memory is allocated, nothing waits for the device, and the call can be captured into a HIP graph
    without fp6m_init_workspace.  Several shapes (every kernel family with a k split), replayed three times with eager
    work in between, each replay bit-identical to the eager result."""
    import fp6_marlin
    fp6_marlin.init(0)
    fp6_marlin.release_workspace(device=0)
    qc, gs = 256, 128
    probs = [(1, 4096, 4096), (16, 8192, 2048), (4, 4096, 1024), (128, 8192, 2048), (40, 2048, 1024)]
    ops = [operands(m, k, n, qc, gs, 300 + i) for i, (m, k, n) in enumerate(probs)]
    outs = [torch.full((m, n), float("nan"), dtype=torch.half, device="cuda") for (m, k, n) in probs]
    old_ws = torch.zeros(4096, dtype=torch.int32, device="cuda")
    want = []
    for (m, k, n), (A, B, s), C in zip(probs, ops, outs):
        fp6_marlin.mul(A, B, C, s, old_ws, qc, -1, -1, -1, 16, gs)
        torch.cuda.synchronize()
        want.append(C.clone())
    ws_eager = torch.zeros(4096, dtype=torch.int32, device="cuda")       # never seen by the library
    ws = torch.zeros(4096, dtype=torch.int32, device="cuda")             # nor this one
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for (m, k, n), (A, B, s), C in zip(probs, ops, outs):
        fp6_marlin.mul(A, B, C, s, ws_eager, qc, -1, -1, -1, 16, gs)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the calls allocated device memory"
    for C, w in zip(outs, want):
        assert torch.equal(C, w)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for (m, k, n), (A, B, s), C in zip(probs, ops, outs):
            fp6_marlin.mul(A, B, C, s, ws, qc, -1, -1, -1, 16, gs)
    for rep in range(3):
        for C in outs:
            C.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for C, w in zip(outs, want):
            assert torch.equal(C, w), rep
        (outs[0] * 2).sum().item()                                       # eager work between the replays
    assert int(ws.abs().sum()) == 0 and int(ws_eager.abs().sum()) == 0
    fp6_marlin.release_workspace(ws)
    fp6_marlin.release_workspace(ws_eager)
    fp6_marlin.release_workspace(old_ws)
