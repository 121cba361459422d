"""s2cnn_so3_analysis_static: the analysis with the library's own scratch buffer instead of a workspace argument (for callers
that cannot allocate).  Called through the raw C ABI and compared bit for bit with s2cnn_so3_analysis, twice in a row, the
second time with a smaller input (the buffer keeps the first call's contents)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _nspec(b):
    return b * (4 * b * b - 1) // 3


def _both(lib, x, table, packed, b_in, b_out):
    """(out of s2cnn_so3_analysis, out of s2cnn_so3_analysis_static) for the real signal x [n, 2b, 2b, 2b]."""
    n = x.size(0)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    nbytes = lib.s2cnn_so3_analysis_workspace(b_in, b_out, n, 0)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    ref = torch.full((_nspec(b_out), n, 2), float("nan"), device=x.device)
    out = torch.full((_nspec(b_out), n, 2), float("nan"), device=x.device)
    assert lib.s2cnn_so3_analysis(p(x), p(table), p(packed), p(ref), p(ws), nbytes, b_in, b_out, n, 0, st) == 0
    assert lib.s2cnn_so3_analysis_static(p(x), p(table), p(packed), p(out), b_in, b_out, n, 0, st) == 0
    torch.cuda.synchronize()
    return ref, out


@pytest.mark.parametrize("b_in,b_out,n_first,n_second", [(32, 32, 9, 4),      # per-volume kernels: scratch = one record per volume
                                                         (32, 22, 5, 2),      # truncated spectrum
                                                         (32, 32, 128, 100),  # the largest scratch of few volumes: two records per volume
                                                         (16, 16, 21, 6),     # the per-volume kernels of the 32^3 grid
                                                         (16, 10, 9, 3),
                                                         (22, 22, 7, 3),      # ... and of the 44^3 grid
                                                         (10, 10, 50, 3),     # ... and of the 20^3 grid
                                                         (12, 8, 40, 7),      # two-stage path: scratch = transformed planes
                                                         (6, 6, 33, 1)])
def test_static_scratch_analysis_equals_workspace_analysis(hip, b_in, b_out, n_first, n_second):
    from s2cnn_amd.soft import so3_fft as PSO3
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(100 * b_in + b_out)
    table = PSO3._setup_wigner(b_in, b_out, True, dev)
    packed = PSO3._setup_packed_wigner(b_in, b_out, True, False, dev)
    for use_packed in (True, False):          # False: the table is repacked into the scratch on every call
        for n in (n_first, n_second):
            x = torch.randn(n, 2 * b_in, 2 * b_in, 2 * b_in, generator=g).to(dev)
            ref, out = _both(hip, x, table, packed if use_packed else None, b_in, b_out)
            assert torch.isfinite(ref).all()
            assert torch.equal(ref, out), (b_in, b_out, n, use_packed)


def test_static_scratch_analysis_allocates_nothing(hip):
    """The defining property: after a first call on the device (which resolves the address of the library's buffer), a
    call leaves the free device memory as it found it, and it can be recorded into a HIP graph (a hipMalloc during a
    capture fails) whose replays give the eager result."""
    from s2cnn_amd.soft import so3_fft as PSO3
    dev = torch.device("cuda:0")
    b = 32
    table = PSO3._setup_wigner(b, b, True, dev)
    packed = PSO3._setup_packed_wigner(b, b, True, False, dev)
    x = torch.randn(6, 2 * b, 2 * b, 2 * b, generator=torch.Generator().manual_seed(7)).to(dev)
    out = torch.empty(_nspec(b), 6, 2, device=dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def run(stream):
        return hip.s2cnn_so3_analysis_static(p(x), p(table), p(packed), p(out), b, b, 6, 0, ctypes.c_void_p(stream.cuda_stream))

    assert run(torch.cuda.current_stream()) == 0
    torch.cuda.synchronize()
    want = out.clone()
    free_before = torch.cuda.mem_get_info(dev)[0]
    for _ in range(3):
        assert run(torch.cuda.current_stream()) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before            # hipMemGetInfo: no device memory was taken
    assert torch.equal(out, want)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        assert run(torch.cuda.current_stream()) == 0                 # the capture stream
    for _ in range(2):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_static_scratch_rejects_what_does_not_fit(hip):
    dev = torch.device("cuda:0")
    fake = ctypes.c_void_p(torch.empty(64, device=dev).data_ptr())
    limit = 64 << 20
    assert hip.s2cnn_so3_analysis_workspace(32, 32, 277, 0) > limit
    assert hip.s2cnn_so3_analysis_static(fake, fake, fake, fake, 32, 32, 277, 0, None) == -4     # S2CNN_ETOOBIG, before any launch
    assert b"static" in hip.s2cnn_strerror(-4)
    assert hip.s2cnn_so3_analysis_static(None, fake, fake, fake, 32, 32, 1, 0, None) == -1
