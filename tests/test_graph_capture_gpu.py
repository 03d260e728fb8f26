"""The C-ABI entry points enqueue kernels only (no allocation, no synchronisation, no memset), so a
caller can record them into a HIP graph.  The graph is replayed several times with new input
contents and eager work in between; every replay must equal the eager result bit for bit."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt,tdtype,h", [(0, torch.bfloat16, 256),   # 16-bit MFMA kernels
                                         (2, torch.float32, 250)])   # fp32 matrix-core kernels, odd H
def test_forward_backward_replay_in_a_hip_graph(dt, tdtype, h):
    from rl_kernel_amd import _native

    lib = _native.load()
    dev = torch.device("cuda:0")
    n, v = 700, 3000  # ragged token and vocab tails
    g = torch.Generator(device=dev).manual_seed(5)
    hidden = torch.randn(n, h, device=dev, generator=g).to(tdtype)
    weight = (torch.randn(v, h, device=dev, generator=g) * 0.06).to(tdtype)
    targets = torch.randint(0, v, (n,), device=dev, generator=g)
    targets[::13] = -100
    grad = torch.randn(n, device=dev, generator=g)
    logp = torch.empty(n, device=dev)
    lse = torch.empty(n, device=dev)
    err = torch.zeros(1, device=dev, dtype=torch.int32)
    dh = torch.empty_like(hidden)
    dw = torch.empty(v, h, device=dev)
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_fwd_workspace_bytes(n, h, v, dt, ctypes.byref(need)) == 0
    ws_f = torch.empty(max(need.value, 16), device=dev, dtype=torch.uint8)
    assert lib.rlk_linear_logp_bwd_workspace_bytes(n, h, v, dt, 0, ctypes.byref(need)) == 0
    ws_b = torch.empty(need.value, device=dev, dtype=torch.uint8)

    def enqueue(stream):
        rc = lib.rlk_linear_logp_fwd(hidden.data_ptr(), weight.data_ptr(), None, targets.data_ptr(),
                                     logp.data_ptr(), lse.data_ptr(), ws_f.data_ptr(), ws_f.numel(),
                                     n, h, v, 0, dt, 0.9, -100, 1, 1, err.data_ptr(), stream)
        assert rc == 0, lib.rlk_last_error()
        rc = lib.rlk_linear_logp_bwd(grad.data_ptr(), hidden.data_ptr(), weight.data_ptr(), None,
                                     targets.data_ptr(), lse.data_ptr(), dh.data_ptr(), dw.data_ptr(),
                                     None, ws_b.data_ptr(), ws_b.numel(), 0, n, h, v, 0, dt, 0.9,
                                     -100, 1, stream)
        assert rc == 0, lib.rlk_last_error()

    side = torch.cuda.Stream()           # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue(side.cuda_stream)        # warm-up outside the capture (sets kernel attributes)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        enqueue(side.cuda_stream)

    for it in range(3):
        hidden.copy_(torch.randn(n, h, device=dev, generator=g).to(tdtype))
        grad.copy_(torch.randn(n, device=dev, generator=g))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (logp, lse, dh, dw)]
        scratch = torch.randn(1 << 20, device=dev).sum().item()  # unrelated eager work + sync
        assert scratch == scratch
        enqueue(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for a, b in zip(got, (logp, lse, dh, dw)):
            assert torch.equal(a, b), f"replay {it} differs from the eager result"
        assert int(err.item()) == 0


def test_static_scratch_forward_replays_in_a_hip_graph():
    """rlk_linear_logp_fwd_static is meant for callers under graph capture: after one call outside
    the capture (per-device set-up), it is recorded and replayed with new inputs; every replay
    must carry the bits of the workspace forward on the same inputs."""
    from rl_kernel_amd import _native

    lib = _native.load()
    dev = torch.device("cuda:0")
    n, h, v, dt = 900, 256, 5000, 0
    g = torch.Generator(device=dev).manual_seed(9)
    hidden = torch.randn(n, h, device=dev, generator=g).to(torch.bfloat16)
    weight = (torch.randn(v, h, device=dev, generator=g) * 0.06).to(torch.bfloat16)
    targets = torch.randint(0, v, (n,), device=dev, generator=g)
    logp, lse = torch.empty(n, device=dev), torch.empty(n, device=dev)
    logp_w, lse_w = torch.empty(n, device=dev), torch.empty(n, device=dev)
    err = torch.zeros(1, device=dev, dtype=torch.int32)
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_fwd_workspace_bytes(n, h, v, dt, ctypes.byref(need)) == 0
    ws = torch.empty(max(need.value, 16), device=dev, dtype=torch.uint8)

    def enqueue_static(stream):
        rc = lib.rlk_linear_logp_fwd_static(hidden.data_ptr(), weight.data_ptr(), None, targets.data_ptr(),
                                            logp.data_ptr(), lse.data_ptr(), n, h, v, 0, dt, 1.0, 0, 0, 1,
                                            err.data_ptr(), stream)
        assert rc == 0, lib.rlk_last_error()

    side = torch.cuda.Stream()           # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue_static(side.cuda_stream)  # set-up happens here, outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        enqueue_static(side.cuda_stream)
    for it in range(3):
        hidden.copy_(torch.randn(n, h, device=dev, generator=g).to(torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        _ = torch.randn(1 << 18, device=dev).sum().item()  # unrelated eager work + sync
        rc = lib.rlk_linear_logp_fwd(hidden.data_ptr(), weight.data_ptr(), None, targets.data_ptr(),
                                     logp_w.data_ptr(), lse_w.data_ptr(), ws.data_ptr(), ws.numel(),
                                     n, h, v, 0, dt, 1.0, 0, 0, 1, err.data_ptr(),
                                     torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.rlk_last_error()
        torch.cuda.synchronize()
        assert torch.equal(logp, logp_w) and torch.equal(lse, lse_w), f"replay {it} differs"
        assert int(err.item()) == 0
