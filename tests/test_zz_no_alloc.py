"""GPU test of proteus_we_bwd_static, the entry point that allocates nothing: called through the C ABI and
compared with proteus_we_bwd (caller-provided workspace) on the same inputs.  Both run the same kernels in the
same order, so the bar is bit equality.  Two calls in a row share the library's static partial-sum array, the
second with a smaller input, so stale partial sums of the first would show."""
import ctypes

import pytest
import torch

from proteusai_amd import _lib

pytestmark = pytest.mark.gpu


def _inputs(gpu, Z, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    dO = torch.randn(Z, N, 2 * K, generator=g).to(gpu)
    c = (torch.randn(Z, N, K, generator=g) * 3).to(gpu)
    s = (torch.randn(Z, N, K, generator=g) * 3).to(gpu)
    return dO, c, s


def _with_workspace(lib, dO, c, s, Z, N, K, stream):
    nbytes = lib.proteus_we_bwd_workspace_bytes(Z, N, K)
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=dO.device)
    out = torch.full((K,), float("nan"), dtype=torch.float32, device=dO.device)
    rc = lib.proteus_we_bwd(dO.data_ptr(), c.data_ptr(), s.data_ptr(), out.data_ptr(), ws.data_ptr(), nbytes, Z, N, K, stream)
    assert rc == 0, lib.proteus_strerror(rc)
    return out


def _static(lib, dO, c, s, Z, N, K, stream):
    out = torch.full((K,), float("nan"), dtype=torch.float32, device=dO.device)
    rc = lib.proteus_we_bwd_static(dO.data_ptr(), c.data_ptr(), s.data_ptr(), out.data_ptr(), Z, N, K, stream)
    assert rc == 0, lib.proteus_strerror(rc)
    return out


def test_static_scratch_entry_point_matches_the_workspace_one(gpu):
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # a large call first (1024 slabs x 512 wavenumbers: the whole array), then smaller ones that reuse its front
    for Z, N, K, seed in [(2, 6000, 512, 1), (1, 300, 77, 2), (3, 40, 512, 3), (1, 1, 1, 4), (1, 9000, 256, 5)]:
        print(f"proteus_we_bwd_static Z={Z} N={N} K={K}", flush=True)
        dO, c, s = _inputs(gpu, Z, N, K, seed)
        want = _with_workspace(lib, dO, c, s, Z, N, K, stream)
        got = _static(lib, dO, c, s, Z, N, K, stream)
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), (Z, N, K)
        # and against the tensor expression it replaces (isotropic/cuda/wf_embedding.py:75-81), in float64
        ref = ((dO.double()[:, :, 1::2] * c.double()) - (dO.double()[:, :, 0::2] * s.double())).sum(dim=(0, 1))
        err = (got.double() - ref).norm() / ref.norm().clamp_min(1e-300)
        assert err <= 1e-5, (Z, N, K, float(err))


def test_static_scratch_entry_point_rejects_what_does_not_fit(gpu):
    lib = _lib.load()
    p = 0x1000
    assert lib.proteus_we_bwd_static(p, p, p, p, 1, 8, 513, None) == -8
    assert lib.proteus_we_bwd_static(None, p, p, p, 1, 8, 4, None) == -1
    assert lib.proteus_we_bwd_static(p, p, p, p, 0, 8, 4, None) == -2
    assert lib.proteus_we_bwd_static(p + 4, p, p, p, 1, 8, 4, None) == -5
    assert b"capacity" in lib.proteus_strerror(-8)


def test_static_scratch_entry_point_replays_from_a_captured_graph(gpu):
    """The use the entry point exists for.  The first call per GPU resolves the scratch array's address and is made
    eagerly (the tests above did, and so does the warm-up here); after that a call only launches its two kernels and
    can be captured.  Replays, with eager calls on other inputs between them, reproduce the eager result to the bit."""
    lib = _lib.load()
    Z, N, K = 2, 3000, 256
    dO, c, s = _inputs(gpu, Z, N, K, 11)
    other = _inputs(gpu, 1, 500, 512, 12)
    out = torch.full((K,), float("nan"), dtype=torch.float32, device=gpu)
    eager = _static(lib, dO, c, s, Z, N, K, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _static(lib, dO, c, s, Z, N, K, ctypes.c_void_p(side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.proteus_we_bwd_static(dO.data_ptr(), c.data_ptr(), s.data_ptr(), out.data_ptr(), Z, N, K,
                                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.proteus_strerror(rc)
    torch.cuda.synchronize()
    for _ in range(3):
        out.fill_(float("nan"))
        _static(lib, *other, 1, 500, 512, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))   # dirties the shared array
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
