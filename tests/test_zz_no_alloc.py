"""The allocation-free variant of the reference operator mm8_one (wrapper.cpp:52-79): same kernels as rwkv_mm8_one,
partial sums in the library's built-in device array instead of a caller workspace.  Called through the C ABI on
two shapes in a row, the second smaller, and compared bit for bit with rwkv_mm8_one on the same inputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(n_in, n_out, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n_in, generator=g, dtype=torch.float32).cuda()
    w = torch.randint(0, 256, (n_in, n_out), generator=g, dtype=torch.uint8).cuda()
    r = (torch.rand(n_in, generator=g, dtype=torch.float32) * 9e-4 + 1e-4).cuda()
    y0 = torch.randn(n_out, generator=g, dtype=torch.float32).cuda()      # the operator accumulates into y
    return x, w, r, y0


def test_mm8_one_static_equals_mm8_one_on_two_calls_in_a_row():
    from rwkvstic_amd import _native as N
    L = N.lib()
    st = torch.cuda.current_stream().cuda_stream
    assert L.rwkv_mm8_one_static_max_bytes() == 12 << 20
    for n_in, n_out, seed in ((2560, 10240, 1), (130, 77, 2)):            # the second call is the smaller one
        print(f"mm8_one_static [{n_in} x {n_out}]", flush=True)
        x, w, r, y0 = _case(n_in, n_out, seed)
        y_ws, y_st = y0.clone(), y0.clone()
        ws = torch.empty(L.rwkv_mm8_workspace_bytes(n_in, n_out, 1), dtype=torch.uint8, device="cuda")
        N.check(L.rwkv_mm8_one(st, n_in, n_out, x.data_ptr(), w.data_ptr(), w.stride(0), y_ws.data_ptr(), r.data_ptr(),
                               ws.data_ptr(), ws.numel()))
        N.check(L.rwkv_mm8_one_static(st, n_in, n_out, x.data_ptr(), w.data_ptr(), w.stride(0), y_st.data_ptr(),
                                      r.data_ptr()))
        torch.cuda.synchronize()
        assert torch.equal(y_ws, y_st)                                    # same kernels, same order of additions
        ref = y0.double().cpu() + (x.double().cpu() * r.double().cpu()) @ w.double().cpu()
        assert (y_st.double().cpu() - ref).abs().max() < 2e-4 * max(1.0, float(ref.abs().max()))
    # a shape beyond the built-in array is refused with a clear error, before anything is launched
    big_in, big_out = 1 << 16, 1 << 16
    assert L.rwkv_mm8_workspace_bytes(big_in, big_out, 1) > L.rwkv_mm8_one_static_max_bytes()
    assert L.rwkv_mm8_one_static(st, big_in, big_out, x.data_ptr(), w.data_ptr(), big_out, y_st.data_ptr(), r.data_ptr()) == -3
    assert b"built-in" in L.rwkv_last_error()


def test_mm8_one_static_under_graph_capture_replays_bit_for_bit():
    """The use the entry point exists for: captured into a HIP graph (after the warm-up call that resolves the
    array's address on this device) and replayed several times, with eager work and synchronisations between the
    replays; every replay must equal the eager result bit for bit.  The operator accumulates into y, so y is
    restored by a copy kernel inside the graph (no memset node)."""
    from rwkvstic_amd import _native as N
    L = N.lib()
    assert L.rwkv_mm8_one_static_max_bytes() == 12 << 20                 # also the warm-up on this device
    n_in, n_out = 1024, 4096
    x, w, r, y0 = _case(n_in, n_out, 3)
    eager = y0.clone()
    N.check(L.rwkv_mm8_one_static(torch.cuda.current_stream().cuda_stream, n_in, n_out, x.data_ptr(), w.data_ptr(),
                                  w.stride(0), eager.data_ptr(), r.data_ptr()))
    torch.cuda.synchronize()
    y = torch.empty_like(y0)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        y.copy_(y0)
        N.check(L.rwkv_mm8_one_static(torch.cuda.current_stream().cuda_stream, n_in, n_out, x.data_ptr(), w.data_ptr(),
                                      w.stride(0), y.data_ptr(), r.data_ptr()))
    for i in range(4):
        y.fill_(float("nan"))
        # other users of the array between replays: an eager call on a different shape
        x2, w2, r2, y2 = _case(300 + i, 500, 10 + i)
        N.check(L.rwkv_mm8_one_static(torch.cuda.current_stream().cuda_stream, 300 + i, 500, x2.data_ptr(), w2.data_ptr(),
                                      w2.stride(0), y2.data_ptr(), r2.data_ptr()))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {i}"
