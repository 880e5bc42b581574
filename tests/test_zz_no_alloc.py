"""The LayerNorm backward entry point that allocates nothing (its partial rows live in a device
array inside the library) against the entry point that takes the caller's workspace: the same
kernels in the same order, so the results must be bit-identical.  Two calls in a row, the second on
a smaller input, then a third at the size that needs the whole built-in array."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(runtime, M, N, seed):
    g = torch.Generator().manual_seed(seed)
    x = (2.0 * torch.randn(M, N, generator=g)).half().cuda()
    w = (1 + 0.1 * torch.randn(N, generator=g)).half().cuda()
    b = (0.1 * torch.randn(N, generator=g)).half().cuda()
    dy = (0.1 * torch.randn(M, N, generator=g)).half().cuda()
    y = torch.empty_like(x)
    mean = torch.empty(M, device="cuda")
    rstd = torch.empty(M, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    runtime.call("lego_hip_layernorm_fwd_f16", _ptr(x), _ptr(y), _ptr(w), _ptr(b), _ptr(mean), _ptr(rstd), M, N,
                 ctypes.c_float(1e-5), stream)
    need = ctypes.c_ulonglong(0)
    runtime.call("lego_hip_layernorm_bwd_workspace_bytes", M, N, ctypes.byref(need))
    ws = torch.full((need.value // 4,), float("nan"), device="cuda")
    want = [torch.empty_like(x), torch.empty_like(w), torch.empty_like(b)]
    got = [torch.full_like(x, float("nan")), torch.full_like(w, float("nan")), torch.full_like(b, float("nan"))]
    runtime.call("lego_hip_layernorm_bwd_f16", _ptr(dy), _ptr(x), _ptr(w), _ptr(mean), _ptr(rstd), *map(_ptr, want),
                 _ptr(ws), need, M, N, stream)
    torch.cuda.synchronize()
    # What the device itself reports as free (hipMemGetInfo): a hipMalloc or hipFree inside the library would move
    # it, which torch's own counter, fed by torch's allocator only, cannot see.  The first call on a device looks up
    # the scratch array's address, which may load the array's module: the check is on the calls after it.
    if _both.warmed:
        before = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated())
    runtime.call("lego_hip_layernorm_bwd_f16_noalloc", _ptr(dy), _ptr(x), _ptr(w), _ptr(mean), _ptr(rstd),
                 *map(_ptr, got), M, N, stream)
    torch.cuda.synchronize()
    if _both.warmed:
        assert (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()) == before
    _both.warmed = True
    for name, a, e in zip(("dx", "dw", "db"), got, want):
        assert not torch.isnan(a.float()).any(), name
        assert torch.equal(a, e), f"{name} differs at {M}x{N}"


_both.warmed = False


def test_no_alloc_layernorm_backward_twice_then_full_scratch():
    from lego_amd import runtime
    runtime.load_library()
    assert torch.cuda.is_available()
    # every path of the fp16 backward: registers (N % 8 == 0), ragged rows, rows above 16384 elements
    for M, N, seed in ((1151, 8192, 1), (300, 1024, 2), (129, 781, 3), (70, 32768, 4), (33, 20001, 5), (3, 8, 6)):
        print(f"no-alloc layernorm backward {M}x{N}", flush=True)
        _both(runtime, M, N, seed)
    # 512 partial rows of 8192 floats, twice: exactly the 32 MiB of the built-in array
    print("no-alloc layernorm backward 8192x8192", flush=True)
    _both(runtime, 8192, 8192, 7)
    _both(runtime, 64, 256, 8)


def test_no_alloc_rejects_what_the_workspace_entry_rejects():
    from lego_amd import runtime
    lib = runtime.load_library()
    p = ctypes.c_void_p(4096)
    assert lib.lego_hip_layernorm_bwd_f16_noalloc(p, p, p, p, p, p, p, p, 4, 32776, None) == 1     # row too long
    assert lib.lego_hip_layernorm_bwd_f16_noalloc(p, p, p, p, p, p, p, p, 0, 64, None) == 1
    assert lib.lego_hip_layernorm_bwd_f16_noalloc(None, p, p, p, p, p, p, p, 4, 64, None) == 1
    assert lib.lego_hip_layernorm_bwd_f16_noalloc(ctypes.c_void_p(4101), p, p, p, p, p, p, p, 4, 64, None) == 1


def test_no_alloc_entry_point_replays_from_a_hip_graph():
    """What the entry point is for: a caller under graph capture.  One eager call first (the first call on a
    device looks up the scratch array's address and must happen outside a capture), then the call is captured and
    replayed three times on new data, with eager work between the replays, against the workspace entry point."""
    from lego_amd import runtime
    runtime.load_library()
    M, N = 300, 2048
    g = torch.Generator().manual_seed(11)
    w = (1 + 0.1 * torch.randn(N, generator=g)).half().cuda()
    b = (0.1 * torch.randn(N, generator=g)).half().cuda()
    x = torch.zeros(M, N, dtype=torch.half, device="cuda")
    dy = torch.zeros(M, N, dtype=torch.half, device="cuda")
    y = torch.empty_like(x)
    mean, rstd = torch.empty(M, device="cuda"), torch.empty(M, device="cuda")
    got = [torch.empty_like(x), torch.empty_like(w), torch.empty_like(b)]
    need = ctypes.c_ulonglong(0)
    runtime.call("lego_hip_layernorm_bwd_workspace_bytes", M, N, ctypes.byref(need))
    ws = torch.empty(need.value // 4, device="cuda")

    def forward_and_noalloc():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        runtime.call("lego_hip_layernorm_fwd_f16", _ptr(x), _ptr(y), _ptr(w), _ptr(b), _ptr(mean), _ptr(rstd), M, N,
                     ctypes.c_float(1e-5), stream)
        runtime.call("lego_hip_layernorm_bwd_f16_noalloc", _ptr(dy), _ptr(x), _ptr(w), _ptr(mean), _ptr(rstd),
                     *map(_ptr, got), M, N, stream)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        forward_and_noalloc()                  # eager, outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        forward_and_noalloc()
    for trial in range(3):
        x.copy_((2.0 * torch.randn(M, N, generator=g)).half())
        dy.copy_((0.1 * torch.randn(M, N, generator=g)).half())
        graph.replay()
        torch.cuda.synchronize()
        replayed = [t.clone() for t in got]
        want = [torch.empty_like(x), torch.empty_like(w), torch.empty_like(b)]
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        runtime.call("lego_hip_layernorm_bwd_f16", _ptr(dy), _ptr(x), _ptr(w), _ptr(mean), _ptr(rstd), *map(_ptr, want),
                     _ptr(ws), need, M, N, stream)      # eager work between the replays
        torch.cuda.synchronize()
        for name, a, e in zip(("dx", "dw", "db"), replayed, want):
            assert torch.equal(a, e), f"{name} differs on replay {trial}"
