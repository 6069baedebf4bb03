"""pbg_row_adagrad_sparse_static (the entry point that allocates nothing: its
sort scratch is a device array built into the library) against
pbg_row_adagrad_sparse on the same inputs, bit for bit, on two calls in a row,
the second with a smaller input; sizes beyond the built-in scratch are refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run(lib, entry, table, sums, idx, grad, lr, workspace=None):
    stream = torch.cuda.current_stream().cuda_stream
    args = [table.data_ptr(), sums.data_ptr(), table.shape[0], table.shape[1], idx.data_ptr(), grad.data_ptr(),
            idx.shape[0], lr]
    if workspace is not None:
        args += [workspace.data_ptr(), workspace.numel()]
    return getattr(lib, entry)(*args, stream)


def test_static_scratch_entry_point_matches_the_workspace_one(pbg):
    lib = pbg._lib.lib()
    print("no-alloc entry point", flush=True)
    gen = torch.Generator(device=DEV).manual_seed(11)
    rows, dim = 50_000, 100
    limit = lib.pbg_row_adagrad_sparse_static_max_indices()
    assert limit == 1 << 20
    # power-law duplicates on the first call (one row named by a third of the indices), uniform on the second
    for n, hot in ((300_000, True), (4_321, False)):
        print("  call with", n, "indices", flush=True)
        table = torch.randn(rows, dim, generator=gen, device=DEV)
        sums = torch.rand(rows, generator=gen, device=DEV)
        idx = torch.randint(0, rows, (n,), generator=gen, device=DEV)
        if hot:
            idx[torch.rand(n, generator=gen, device=DEV) < 0.33] = 777
        grad = torch.randn(n, dim, generator=gen, device=DEV)
        t_a, s_a, g_a = table.clone(), sums.clone(), grad.clone()
        t_b, s_b, g_b = table.clone(), sums.clone(), grad.clone()
        ws = torch.empty(lib.pbg_row_adagrad_sparse_workspace_bytes(n), dtype=torch.uint8, device=DEV)
        assert _run(lib, "pbg_row_adagrad_sparse", t_a, s_a, idx, g_a, 0.1, ws) == 0
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        free_before, _ = torch.cuda.mem_get_info()  # the driver's view: a hipMalloc inside the library would show here
        assert _run(lib, "pbg_row_adagrad_sparse_static", t_b, s_b, idx, g_b, 0.1) == 0
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(t_a, t_b) and torch.equal(s_a, s_b)
        assert not torch.equal(t_a, table)  # the step did something
    # beyond the built-in scratch: a clear error, nothing launched
    n = limit + 1
    idx = torch.zeros(n, dtype=torch.int64, device=DEV)
    grad = torch.zeros(n, 4, device=DEV)
    table = torch.ones(8, 4, device=DEV)
    sums = torch.zeros(8, device=DEV)
    assert _run(lib, "pbg_row_adagrad_sparse_static", table, sums, idx, grad, 0.1) == pbg._lib.PBG_ERR_WORKSPACE
    assert b"exceeds the built-in scratch" in lib.pbg_last_error()
    torch.cuda.synchronize()
    assert torch.equal(table, torch.ones(8, 4, device=DEV))
    # the largest accepted size runs
    n = limit
    idx = torch.randint(0, 8, (n,), generator=gen, device=DEV)
    grad = torch.full((n, 4), 1e-3, device=DEV)
    want_t, want_s, want_g = table.clone(), sums.clone(), grad.clone()
    ws = torch.empty(lib.pbg_row_adagrad_sparse_workspace_bytes(n), dtype=torch.uint8, device=DEV)
    assert _run(lib, "pbg_row_adagrad_sparse", want_t, want_s, idx, want_g, 0.1, ws) == 0
    assert _run(lib, "pbg_row_adagrad_sparse_static", table, sums, idx, grad, 0.1) == 0
    torch.cuda.synchronize()
    assert torch.equal(table, want_t) and torch.equal(sums, want_s)


def test_static_scratch_entry_point_under_graph_capture(pbg):
    """What the entry point is for: a caller that cannot allocate because it is
    capturing a HIP graph.  One eager call first (the library's per-device set-up
    is not capturable), then the call is captured and replayed three times on
    inputs written into the captured tensors, with eager work and synchronisations
    in between; every replay equals the workspace entry point bit for bit."""
    lib = pbg._lib.lib()
    print("no-alloc entry point under capture", flush=True)
    gen = torch.Generator(device=DEV).manual_seed(12)
    rows, dim, n = 20_000, 100, 30_000
    table = torch.empty(rows, dim, device=DEV)
    sums = torch.empty(rows, device=DEV)
    idx = torch.empty(n, dtype=torch.int64, device=DEV)
    grad = torch.empty(n, dim, device=DEV)

    def fill(hot):
        table.copy_(torch.randn(rows, dim, generator=gen, device=DEV))
        sums.copy_(torch.rand(rows, generator=gen, device=DEV))
        idx.copy_(torch.randint(0, rows, (n,), generator=gen, device=DEV))
        if hot:
            idx[torch.rand(n, generator=gen, device=DEV) < 0.4] = 123
        grad.copy_(torch.randn(n, dim, generator=gen, device=DEV))

    fill(False)
    assert _run(lib, "pbg_row_adagrad_sparse_static", table, sums, idx, grad, 0.1) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert _run(lib, "pbg_row_adagrad_sparse_static", table, sums, idx, grad, 0.1) == 0
    ws = torch.empty(lib.pbg_row_adagrad_sparse_workspace_bytes(n), dtype=torch.uint8, device=DEV)
    for replay, hot in enumerate((False, True, False)):
        fill(hot)
        want_t, want_s, want_g = table.clone(), sums.clone(), grad.clone()
        assert _run(lib, "pbg_row_adagrad_sparse", want_t, want_s, idx, want_g, 0.1, ws) == 0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(table, want_t) and torch.equal(sums, want_s), replay
