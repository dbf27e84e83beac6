"""The allocation-free form of the factored statistics pass against the form that takes a
workspace: same row/column statistics and mean, bit for bit, on two calls in a row (the second
on a smaller input, so it meets whatever the first left in the library's static array)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

BETA2 = 0.999


def _run(lib, g, row0, col0, static):
    rows, cols = g.shape
    row, col = row0.clone(), col0.clone()
    mean = torch.zeros(1, dtype=torch.float32, device=g.device)
    stream = torch.cuda.current_stream().cuda_stream
    if static:
        st = lib.lpmm_factored_stats_static(g.data_ptr(), rows, cols, row.data_ptr(), col.data_ptr(),
                                            mean.data_ptr(), BETA2, stream)
    else:
        work = torch.empty((lib.lpmm_factored_workspace_bytes(rows, cols),), dtype=torch.uint8, device=g.device)
        st = lib.lpmm_factored_stats(g.data_ptr(), rows, cols, row.data_ptr(), col.data_ptr(), mean.data_ptr(),
                                     BETA2, work.data_ptr(), stream)
    assert st == 0
    torch.cuda.synchronize()
    return row.cpu().numpy(), col.cpu().numpy(), mean.cpu().numpy()


def test_static_scratch_stats_equal_workspace_stats():
    from lpmm import _native

    lib = _native.lib()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(11)
    for shape in ((1031, 2752), (130, 517)):  # ragged tiles in both directions; the second call is smaller
        g = torch.randn(shape, device=dev, generator=gen) * 1e-3
        row0 = torch.rand(shape[0], device=dev, generator=gen) * 1e-6
        col0 = torch.rand(shape[1], device=dev, generator=gen) * 1e-6
        want = _run(lib, g, row0, col0, static=False)
        got = _run(lib, g, row0, col0, static=True)
        for a, b, what in zip(got, want, ("row", "col", "mean(row)")):
            np.testing.assert_array_equal(a, b, err_msg=f"{what} {shape}")
        assert np.all(want[0] > 0) and want[2][0] > 0


def test_static_scratch_rejects_what_does_not_fit():
    from lpmm import _native

    lib = _native.lib()
    rows, cols = 1 << 16, 1 << 13  # 1024 row tiles x 8192 columns of doubles: 64 MiB of partials
    assert lib.lpmm_factored_workspace_bytes(rows, cols) > (32 << 20)
    x = torch.zeros(16, device="cuda:0")
    st = lib.lpmm_factored_stats_static(x.data_ptr(), rows, cols, x.data_ptr(), x.data_ptr(), x.data_ptr(), BETA2, None)
    assert st == 3  # LPMM_ERR_SIZE, before anything touches the GPU


def test_static_scratch_call_replayed_from_a_graph():
    """After a warm-up call on the GPU (the first call looks up the array's address and must stay outside
    capture), the allocation-free call records into a HIP graph.  Three replays on changing gradients, with
    eager work and synchronisations in between, each against the workspace form issued eagerly."""
    from lpmm import _native

    lib = _native.lib()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(12)
    warm = torch.randn((64, 128), device=dev, generator=gen)
    _run(lib, warm, torch.zeros(64, device=dev), torch.zeros(128, device=dev), static=True)

    rows, cols = 515, 1400
    g = torch.randn((rows, cols), device=dev, generator=gen) * 1e-3
    row, col = torch.zeros(rows, device=dev), torch.zeros(cols, device=dev)
    mean = torch.zeros(1, device=dev)
    side = torch.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            st = lib.lpmm_factored_stats_static(g.data_ptr(), rows, cols, row.data_ptr(), col.data_ptr(),
                                                mean.data_ptr(), BETA2, torch.cuda.current_stream().cuda_stream)
            assert st == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert float(row.abs().sum()) == 0.0  # capture records, it does not run
    for replay in range(3):
        g.copy_(torch.randn((rows, cols), device=dev, generator=gen) * (1e-3 * (replay + 1)))
        row0, col0 = row.clone(), col.clone()
        want = _run(lib, g, row0, col0, static=False)
        graph.replay()
        torch.cuda.synchronize()
        # eager work between the replays, some of it through the same array
        _run(lib, warm, torch.zeros(64, device=dev), torch.zeros(128, device=dev), static=True)
        for a, b, what in zip((row.cpu().numpy(), col.cpu().numpy(), mean.cpu().numpy()), want, ("row", "col", "mean(row)")):
            np.testing.assert_array_equal(a, b, err_msg=f"{what}, replay {replay}")
