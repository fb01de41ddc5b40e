"""spmm_csr_f32_static, the entry point that allocates nothing: the schedule spmm_csr_f32 runs with a caller-owned
workspace, with the partial rows in the library's own static device array instead. Checked through the C ABI against
that existing entry point, bit for bit, on two calls in a row (the second on a smaller matrix, so that whatever the
first call left in the shared array must not matter), and against the CPU oracle within the 1e-4 bar."""
import numpy as np
import pytest


def _problem(dl, seed, M, K, N, mean_row, sigma):
    ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, seed, M, K, mean_row, sigma)
    va = dl.fill("normal", seed + 1, (ci.size,), 0.0, 1.0)
    B = dl.fill("uniform", seed + 2, (K, N), -1.0, 1.0)
    return ro, ci, va, B


@pytest.mark.gpu
def test_static_entry_point_equals_the_workspace_call_twice_in_a_row(dl, oracle):
    import torch

    d = lambda a: torch.from_numpy(a).cuda()
    limit = dl.static_scratch_bytes()
    assert limit == 8 << 20
    # first a matrix of 0.8 M nonzeros in very uneven rows, then a smaller one (0.55 M) with another width: both take
    # the flat schedule (partial rows of split rows in the scratch array) and fit the array
    for seed, M, K, N, mean_row, sigma in ((21, 4096, 4096, 128, 200.0, 1.5), (31, 3072, 2048, 96, 180.0, 1.0)):
        ro, ci, va, B = _problem(dl, seed, M, K, N, mean_row, sigma)
        nnz = ci.size
        need = dl.workspace_bytes(dl.OP_SPMM, M, K, N, nnz)
        shape = dl.describe_launch(dl.OP_SPMM, M, K, N, nnz, with_workspace=True)
        print(f"static spmm: M={M} K={K} N={N} nnz={nnz} workspace {need} bytes, flat chunk {shape['flat_chunk']}", flush=True)
        assert 0 < need <= limit and shape["flat_chunk"] > 0  # the case is about the scratch buffer: it must be in use
        ro_d, ci_d, va_d, B_d = d(ro), d(ci), d(va), d(B)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        want = dl.spmm(ro_d, ci_d, va_d, B_d, K=K, workspace=ws)
        out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        got = dl.spmm_static(ro_d, ci_d, va_d, B_d, K=K, out=out)
        torch.cuda.synchronize()
        assert torch.equal(got, want), "spmm_csr_f32_static differs from spmm_csr_f32 with a workspace"
        assert oracle.rel_frobenius(got.cpu().numpy(), oracle.spmm(ro, ci, va, B, omp=True)) <= 1e-4
        assert np.array_equal(ro_d.cpu().numpy(), ro) and np.array_equal(ci_d.cpu().numpy(), ci)


@pytest.mark.gpu
def test_static_entry_point_small_sizes_and_limit(dl, oracle):
    import torch

    d = lambda a: torch.from_numpy(a).cuda()
    # a size whose schedule needs no scratch at all: the same result as the plain call
    ro, ci, va, B = _problem(dl, 41, 300, 200, 50, 20.0, 0.8)
    assert dl.workspace_bytes(dl.OP_SPMM, 300, 200, 50, ci.size) == 0
    got = dl.spmm_static(d(ro), d(ci), d(va), d(B))
    assert torch.equal(got, dl.spmm(d(ro), d(ci), d(va), d(B)))
    assert oracle.rel_frobenius(got.cpu().numpy(), oracle.spmm(ro, ci, va, B)) <= 1e-4
    # sizes beyond the array are refused before anything is launched (no device memory is touched: null pointers do)
    M, K, N, nnz = 65536, 8192, 512, 1 << 26
    assert dl.workspace_bytes(dl.OP_SPMM, M, K, N, nnz) > dl.static_scratch_bytes()
    st = dl.lib().spmm_csr_f32_static(M, K, N, nnz, None, None, None, None, None, None)
    assert st == dl.E_STATIC_LIMIT and "spmm_csr_f32_static" in dl.status_string(st)
    assert dl.lib().spmm_csr_f32_static(-1, 1, 1, 0, None, None, None, None, None, None) == dl.E_INVALID_ARG


@pytest.mark.gpu
def test_static_entry_point_allocates_nothing_and_can_be_captured(dl, oracle):
    """What the entry point is for: device memory is the same before and after the call (the driver's free memory and
    PyTorch's own books), the call can be recorded in a HIP graph and replayed on changed inputs with the bits of the eager
    call, and the column-sliced layout of the scratch array (slice boundaries, then partial rows) works like the flat one."""
    import torch

    d = lambda a: torch.from_numpy(a).cuda()
    M, K, N = 3072, 2048, 96
    ro, ci, va, B = _problem(dl, 31, M, K, N, 180.0, 1.0)
    assert 0 < dl.workspace_bytes(dl.OP_SPMM, M, K, N, ci.size) <= dl.static_scratch_bytes()
    ro_d, ci_d, va_d, B_d = d(ro), d(ci), d(va), d(B)
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    dl.spmm_static(ro_d, ci_d, va_d, B_d, K=K, out=out)   # the first call on the device looks the array's address up
    torch.cuda.synchronize()
    free0, allocated0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        dl.spmm_static(ro_d, ci_d, va_d, B_d, K=K, out=out)
    torch.cuda.synchronize()
    assert (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (free0, allocated0, reserved0)
    eager = out.clone()
    # under capture, replayed twice on changed values
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            dl.spmm_static(ro_d, ci_d, va_d, B_d, K=K, out=out)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, eager)
    for rep in range(2):
        va_d.mul_(-0.5)
        B_d.add_(0.25)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = dl.spmm_static(ro_d, ci_d, va_d, B_d, K=K)
        assert torch.equal(out, want), f"replay {rep}"
        assert oracle.rel_frobenius(out.cpu().numpy(), oracle.spmm(ro, ci, va_d.cpu().numpy(), B_d.cpu().numpy(), omp=True)) <= 1e-4
    # the column-sliced layout in the same array: two slices forced on a small matrix
    M, K, N = 1024, 1024, 128
    ro, ci, va, B = _problem(dl, 51, M, K, N, 60.0, 0.8)
    dl.set_tuning(slices=2)
    need = dl.workspace_bytes(dl.OP_SPMM, M, K, N, ci.size)
    assert 0 < need <= dl.static_scratch_bytes() and dl.describe_slices(dl.OP_SPMM, M, K, N, ci.size)[0] == 2
    ro_d, ci_d, va_d, B_d = d(ro), d(ci), d(va), d(B)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = dl.spmm(ro_d, ci_d, va_d, B_d, K=K, workspace=ws)
    got = dl.spmm_static(ro_d, ci_d, va_d, B_d, K=K)
    dl.set_tuning()
    assert torch.equal(got, want)
    assert oracle.rel_frobenius(got.cpu().numpy(), oracle.spmm(ro, ci, va, B, omp=True)) <= 1e-4
