"""Weight / bias gradients of the fused head added into caller-owned fp32 buffers
(`rlk_linear_logp_bwd_accum`, op keywords `weight_grad_out` / `bias_grad_out` / `accumulate`).

The reference's backward keeps one fp32 grad_w over all its token chunks and casts at the end
(rl_engine/kernels/ops/pytorch/loss/linear_logp.py:404,423-437); here that buffer is the caller's,
and micro-batches run into it one after another.  Bars: two micro-batches accumulated in place
equal one double batch to fp32 summation order (relative norm <= 1e-5) and the oracle to the
gradient gate of the path (2e-2 relative norm); accumulate=0 is bit-equal to rlk_linear_logp_bwd.
"""
import ctypes

import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

GRAD_REL = 2e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def op():
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp

    return RocmFusedLinearLogpOp()


def rel(a, b):
    return ((a.float().cpu() - b.float().cpu()).norm() / b.float().cpu().norm().clamp_min(1e-30)).item()


def make(seed, n, h, v, dtype, bias):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g).to(dtype)
    weight = (torch.randn(v, h, generator=g) / h ** 0.5).to(dtype)
    b = (torch.randn(v, generator=g) * 0.5).to(dtype) if bias else None
    tgt = torch.randint(0, v, (n,), generator=g)
    tgt[torch.rand(n, generator=g) < 0.05] = -100
    grad = torch.randn(n, generator=g)
    return hidden, weight, b, tgt, grad


@pytest.mark.parametrize("n,h,v,dtype,bias", [
    (600, 128, 2304, torch.bfloat16, False),
    (514, 136, 1500, torch.float16, True),      # ragged everything, bias
    (2048, 256, 9000, torch.bfloat16, True),
    (300, 96, 700, torch.float32, True),        # fp32 matrix-core kernels
])
def test_two_micro_batches_accumulate_to_the_double_batch(dev, op, n, h, v, dtype, bias):
    print(f"case n={n} H={h} V={v} {dtype} bias={bias}", flush=True)
    hidden, weight, b, tgt, grad = make(11, n, h, v, dtype, bias)
    r_dh, r_dw, r_db = O.linear_logp_backward(grad, hidden, weight, tgt, b, temperature=0.7, ignore_index=-100)
    hd, wd = hidden.to(dev), weight.to(dev).requires_grad_(True)
    bd = b.to(dev).requires_grad_(True) if bias else None
    td, gd = tgt.to(dev), grad.to(dev)
    main_w = torch.zeros(v, h, device=dev, dtype=torch.float32)
    main_b = torch.zeros(v, device=dev, dtype=torch.float32) if bias else None
    half = n // 2 + 3  # uneven micro-batches
    dhs = []
    for lo, hi in ((0, half), (half, n)):
        x = hd[lo:hi].clone().requires_grad_(True)
        out = op(x, wd, td[lo:hi], bd, temperature=0.7, ignore_index=-100, weight_grad_out=main_w,
                 bias_grad_out=main_b)
        out.backward(gd[lo:hi])
        dhs.append(x.grad)
    # autograd saw no weight / bias gradient: it went to the buffers
    assert wd.grad is None and (bd is None or bd.grad is None)
    # the same tokens as one batch, overwrite mode, into fresh buffers
    one_w = torch.full((v, h), 7.0, device=dev, dtype=torch.float32)
    one_b = torch.full((v,), 7.0, device=dev, dtype=torch.float32) if bias else None
    x = hd.clone().requires_grad_(True)
    op(x, wd, td, bd, temperature=0.7, ignore_index=-100, weight_grad_out=one_w, bias_grad_out=one_b,
       accumulate=False).backward(gd)
    assert rel(main_w, one_w) <= 1e-5
    assert torch.equal(torch.cat(dhs), x.grad)  # dH rows do not depend on the batch split
    tol = 1e-4 if dtype == torch.float32 else GRAD_REL
    assert rel(main_w, r_dw) <= tol and rel(torch.cat(dhs), r_dh) <= tol
    if bias:
        assert rel(main_b, one_b) <= 1e-5 and rel(main_b, r_db) <= tol
    # a third call keeps adding: the buffer now holds twice the double-batch gradient
    x = hd.clone().requires_grad_(True)
    op(x, wd, td, bd, temperature=0.7, ignore_index=-100, weight_grad_out=main_w, bias_grad_out=main_b).backward(gd)
    assert rel(main_w, 2.0 * one_w) <= 1e-5


def test_frozen_weight_still_fills_the_buffer_and_default_mode_is_unchanged(dev, op):
    hidden, weight, b, tgt, grad = make(5, 300, 64, 1000, torch.bfloat16, False)
    hd, wd, td, gd = hidden.to(dev), weight.to(dev), tgt.to(dev), grad.to(dev)
    buf = torch.zeros(1000, 64, device=dev, dtype=torch.float32)
    x = hd.clone().requires_grad_(True)
    op(x, wd, td, ignore_index=-100, weight_grad_out=buf).backward(gd)  # weight does not require grad
    w2 = wd.clone().requires_grad_(True)
    x2 = hd.clone().requires_grad_(True)
    op(x2, w2, td, ignore_index=-100).backward(gd)
    assert w2.grad.dtype == torch.bfloat16
    assert torch.equal(buf.to(torch.bfloat16), w2.grad) and torch.equal(x.grad, x2.grad)


def test_raw_entry_point_overwrite_equals_plain_backward_and_add_adds(dev):
    from rl_kernel_amd import _native
    from rl_kernel_amd.ops import linear_logp as LL

    lib = _native.load()
    n, h, v = 700, 128, 2304
    hidden, weight, _, tgt, grad = make(9, n, h, v, torch.bfloat16, False)
    hd, wd, td, gd = hidden.to(dev), weight.to(dev), tgt.to(dev), grad.to(dev)
    _, lse, _ = LL.fused_linear_logp_forward(hd, wd, td, ignore_index=-100)
    d_h0, d_w0, _ = LL.fused_linear_logp_backward(gd, hd, wd, td, lse, ignore_index=-100)
    need = ctypes.c_size_t(0)
    _native.check(lib.rlk_linear_logp_bwd_workspace_bytes(n, h, v, 0, 0, ctypes.byref(need)), "ws")
    ws = torch.empty(need.value, device=dev, dtype=torch.uint8)
    dh = torch.empty_like(hd)
    dw = torch.full((v, h), 3.0, device=dev, dtype=torch.float32)
    st = torch.cuda.current_stream().cuda_stream

    def call(acc):
        rc = lib.rlk_linear_logp_bwd_accum(gd.data_ptr(), hd.data_ptr(), wd.data_ptr(), None, td.data_ptr(),
                                           lse.data_ptr(), dh.data_ptr(), dw.data_ptr(), None, ws.data_ptr(),
                                           ws.numel(), 0, n, h, v, 0, 0, 1.0, -100, 1, acc, st)
        _native.check(rc, "rlk_linear_logp_bwd_accum")

    call(0)
    assert torch.equal(dw, d_w0) and torch.equal(dh, d_h0)
    call(1)
    assert rel(dw, 2.0 * d_w0) <= 1e-6 and torch.equal(dh, d_h0)


def test_buffer_argument_errors(dev, op):
    hidden, weight, b, tgt, _ = make(2, 64, 64, 512, torch.bfloat16, True)
    hd, wd, bd, td = hidden.to(dev), weight.to(dev), b.to(dev), tgt.to(dev)
    with pytest.raises(ValueError, match="weight_grad_out"):
        op(hd, wd, td, weight_grad_out=torch.zeros(512, 64, device=dev, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="weight_grad_out"):
        op(hd, wd, td, weight_grad_out=torch.zeros(64, 512, device=dev))
    with pytest.raises(ValueError, match="bias_grad_out given without a bias"):
        op(hd, wd, td, bias_grad_out=torch.zeros(512, device=dev))
    with pytest.raises(ValueError, match="bias_grad_out"):
        op(hd, wd, td, bd, bias_grad_out=torch.zeros(511, device=dev))


def test_backward_holds_nothing_beyond_outputs_and_workspace(dev, op):
    """Extra device memory while the op's backward runs in main-gradient mode = the library's
    workspace (rlk_linear_logp_bwd_workspace_bytes), the fp32 copy of the upstream gradient and
    allocator rounding: no second hidden-sized or weight-sized block."""
    from rl_kernel_amd import _native

    n, h, v = 8192, 1024, 16384
    g = torch.Generator().manual_seed(3)
    hidden = torch.randn(n, h, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
    weight = (0.05 * torch.randn(v, h, generator=g)).to(torch.bfloat16).to(dev).requires_grad_(True)
    ids = torch.randint(0, v, (n,), generator=g).to(dev)
    up = torch.randn(n, generator=g).to(dev)
    main = torch.zeros(v, h, device=dev)
    need = ctypes.c_size_t(0)
    assert _native.load().rlk_linear_logp_bwd_workspace_bytes(n, h, v, 0, 0, ctypes.byref(need)) == 0
    for _ in range(2):  # the second pass measures: every lazy one-time allocation is behind it
        hidden.grad = None
        logp = op(hidden, weight, ids, weight_grad_out=main, check_targets=False)
        loss = (logp * up).sum()
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        loss.backward()
        torch.cuda.synchronize()
        extra = torch.cuda.max_memory_allocated() - base
    d_hidden_bytes = n * h * 2
    assert extra <= need.value + d_hidden_bytes + (4 << 20), (extra, need.value)
