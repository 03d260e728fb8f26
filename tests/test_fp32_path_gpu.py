"""GPU parity of the fp32 matrix-core path (fp32 tensors, 16-bit tensors whose hidden size is not a
multiple of 8 or whose storage is not 16-byte aligned, mixed dtypes) against the CPU oracle; fp32
tolerance 1e-5 on logp (BASELINE config 1 is one of the cases)."""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def op():
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp

    return RocmFusedLinearLogpOp()


@pytest.mark.parametrize("lead,h,v,dtype,bias,temp,ign,atol", [
    ((2, 64), 256, 4096, torch.float32, False, 1.0, False, 1e-5),   # BASELINE config 1
    ((6,), 7, 19, torch.float32, True, 1.0, True, 1e-5),            # shapes of the reference tests
    ((2, 3), 5, 17, torch.float32, True, 0.7, True, 1e-5),
    ((50,), 100, 300, torch.float32, False, 1.3, False, 1e-5),
    ((9,), 7, 19, torch.bfloat16, True, 1.0, False, 1e-3),          # 16-bit but H % 8 != 0
    ((33,), 30, 70, torch.float16, False, 0.7, True, 1e-3),
    ((5,), 3000, 40, torch.float32, False, 1.0, False, 2e-5),       # long contraction, one tile
    ((3, 200), 130, 1000, torch.float32, True, 0.7, True, 1e-5),    # 3 token blocks x 4 vocab tiles, ragged
    ((700,), 515, 777, torch.float32, False, 1.0, False, 2e-5),     # odd H: element-wise loads, 3 H tiles
    ((300,), 260, 520, torch.bfloat16, True, 1.0, True, 1e-3),      # 16-bit, H % 8 != 0, several tiles
    ((2048,), 512, 8192, torch.float32, True, 0.9, True, 2e-5),     # 8 x 32 x 2 tiles, dH in 8 vocab parts
])
def test_forward_backward_match_oracle(dev, op, lead, h, v, dtype, bias, temp, ign, atol):
    g = torch.Generator().manual_seed(h + v)
    hidden = torch.randn(*lead, h, generator=g).to(dtype)
    weight = (torch.randn(v, h, generator=g) * (0.02 if h == 256 else h ** -0.5)).to(dtype)
    b = torch.randn(v, generator=g).to(dtype) if bias else None
    tgt = torch.randint(0, v, lead, generator=g)
    if ign:
        tgt.reshape(-1)[::3] = -100
    grad = torch.randn(*lead, generator=g)
    ii = -100 if ign else None
    ref = O.linear_logp(hidden, weight, tgt, b, temperature=temp, ignore_index=ii)
    r_dh, r_dw, r_db = O.linear_logp_backward(grad, hidden, weight, tgt, b, temperature=temp,
                                              ignore_index=ii)
    hd = hidden.to(dev).requires_grad_(True)
    wd = weight.to(dev).requires_grad_(True)
    bd = b.to(dev).requires_grad_(True) if bias else None
    out = op(hd, wd, tgt.to(dev), bd, temperature=temp, ignore_index=ii)
    out.backward(grad.to(dev))
    assert out.dtype == torch.float32 and out.shape == tuple(lead)
    assert (out.detach().cpu() - ref).abs().max().item() < atol
    if ign:
        assert torch.all(out.detach().cpu()[tgt == -100] == 0.0)
    gtol = 1e-4 if dtype == torch.float32 else 2e-2
    rel = lambda a, r: ((a.float().cpu() - r).norm() / r.norm().clamp_min(1e-30)).item()
    assert rel(hd.grad, r_dh) < gtol and rel(wd.grad, r_dw) < gtol
    if bias:
        assert rel(bd.grad, r_db) < gtol


def test_fp32_errors_and_repeatability(dev, op):
    g = torch.Generator().manual_seed(1)
    hidden, weight = torch.randn(10, 12, generator=g), torch.randn(20, 12, generator=g)
    tgt = torch.randint(0, 20, (10,), generator=g)
    a = op(hidden.to(dev), weight.to(dev), tgt.to(dev))
    assert torch.equal(a, op(hidden.to(dev), weight.to(dev), tgt.to(dev)))
    bad = tgt.clone()
    bad[0] = 20
    with pytest.raises(ValueError, match="out of range"):
        op(hidden.to(dev), weight.to(dev), bad.to(dev))


def test_mixed_dtypes_are_widened_to_fp32(dev, op):
    """An fp32 head over bf16 activations (and the other way round): both operands are widened,
    which is exact, so the result is the oracle's on the widened values; gradients come back in
    each tensor's own dtype."""
    g = torch.Generator().manual_seed(2)
    hidden = torch.randn(40, 48, generator=g).to(torch.bfloat16)
    weight = torch.randn(90, 48, generator=g) * 48 ** -0.5
    tgt = torch.randint(0, 90, (40,), generator=g)
    grad = torch.randn(40, generator=g)
    for h_cpu, w_cpu in ((hidden, weight), (hidden.float(), weight.to(torch.float16))):
        ref = O.linear_logp(h_cpu.float(), w_cpu.float(), tgt)
        r_dh, r_dw, _ = O.linear_logp_backward(grad, h_cpu.float(), w_cpu.float(), tgt)
        hd = h_cpu.to(dev).requires_grad_(True)
        wd = w_cpu.to(dev).requires_grad_(True)
        out = op(hd, wd, tgt.to(dev))
        out.backward(grad.to(dev))
        assert (out.detach().cpu() - ref).abs().max().item() < 1e-5
        assert hd.grad.dtype == h_cpu.dtype and wd.grad.dtype == w_cpu.dtype
        rel = lambda a, r: ((a.float().cpu() - r).norm() / r.norm()).item()
        assert rel(hd.grad, r_dh) < 1e-2 and rel(wd.grad, r_dw) < 1e-2


def test_misaligned_16_bit_storage_takes_the_fp32_kernels(dev, op):
    """Views that start 2 bytes into their storage cannot use 16-byte loads; the result must still
    be the aligned call's up to the fp32 kernels' rounding (products are exact either way)."""
    g = torch.Generator().manual_seed(3)
    n, h, v = 70, 64, 300
    hidden = torch.randn(n, h, generator=g).to(torch.bfloat16)
    weight = (torch.randn(v, h, generator=g) * h ** -0.5).to(torch.bfloat16)
    tgt = torch.randint(0, v, (n,), generator=g)
    ref = O.linear_logp(hidden, weight, tgt)
    hbuf = torch.empty(n * h + 1, dtype=torch.bfloat16, device=dev)
    wbuf = torch.empty(v * h + 1, dtype=torch.bfloat16, device=dev)
    hd = hbuf[1:].view(n, h).copy_(hidden)
    wd = wbuf[1:].view(v, h).copy_(weight)
    assert hd.data_ptr() % 16 != 0 and wd.data_ptr() % 16 != 0
    from rl_kernel_amd.ops.linear_logp import fused_linear_logp_forward, fused_linear_logp_backward

    logp, lse, _ = fused_linear_logp_forward(hd, wd, tgt.to(dev))
    assert (logp.cpu() - ref).abs().max().item() < 1e-3
    grad = torch.randn(n, generator=g)
    r_dh, r_dw, _ = O.linear_logp_backward(grad, hidden, weight, tgt)
    d_h, d_w, _ = fused_linear_logp_backward(grad.to(dev), hd, wd, tgt.to(dev), lse)
    rel = lambda a, r: ((a.float().cpu() - r).norm() / r.norm()).item()
    assert rel(d_h, r_dh) < 2e-2 and rel(d_w, r_dw) < 2e-2


def test_fp32_backward_in_several_token_chunks_and_vocab_parts(dev):
    """A small dZ budget forces several token chunks (dW accumulated across them) and the dH launch
    into several vocab parts; both must reproduce the one-chunk result up to fp32 summation order
    and the oracle."""
    from rl_kernel_amd.ops.linear_logp import fused_linear_logp_forward, fused_linear_logp_backward

    g = torch.Generator().manual_seed(4)
    n, h, v = 1100, 96, 2600
    hidden = torch.randn(n, h, generator=g)
    weight = torch.randn(v, h, generator=g) * h ** -0.5
    bias = torch.randn(v, generator=g) * 0.1
    tgt = torch.randint(0, v, (n,), generator=g)
    tgt[::7] = -100
    grad = torch.randn(n, generator=g)
    r_dh, r_dw, r_db = O.linear_logp_backward(grad, hidden, weight, tgt, bias, temperature=0.8,
                                              ignore_index=-100)
    hd, wd, bd, td, gd = (t.to(dev) for t in (hidden, weight, bias, tgt, grad))
    _, lse, _ = fused_linear_logp_forward(hd, wd, td, bd, temperature=0.8, ignore_index=-100)
    rel = lambda a, r: ((a.float().cpu() - r).norm() / r.norm()).item()
    outs = []
    for budget in (0, 1 << 20):   # default: one chunk; 1 MiB: 256-token chunks
        d_h, d_w, d_b = fused_linear_logp_backward(gd, hd, wd, td, lse, bd, temperature=0.8,
                                                   ignore_index=-100, dz_budget_bytes=budget)
        assert rel(d_h, r_dh) < 1e-4 and rel(d_w, r_dw) < 1e-4 and rel(d_b, r_db) < 1e-4
        assert torch.all(d_h.cpu()[tgt == -100] == 0.0)
        outs.append((d_h, d_w, d_b))
    assert torch.equal(outs[0][0], outs[1][0])          # dH rows do not depend on the chunking
    assert rel(outs[1][1], outs[0][1].cpu()) < 1e-5


def test_registry_dispatches_to_hip_backends(dev):
    from rl_kernel_amd.registry import kernel_registry

    names = {t: type(kernel_registry.get_op(t)).__name__ for t in
             ("linear_logp", "logp", "logp_indexed", "logp_online", "logp_online_indexed",
              "ratio_kl", "grpo_loss", "grpo_loss_from_logp")}
    assert names["linear_logp"] == "RocmFusedLinearLogpOp"
    assert {names[t] for t in ("logp", "logp_indexed", "logp_online", "logp_online_indexed")} == \
        {"RocmFusedLogpOp"}
    assert names["ratio_kl"] == "RocmRatioKLOp" and names["grpo_loss"] == "RocmGRPOLossOp"
    assert kernel_registry.get_op("logp") is kernel_registry.get_op("logp_online")
    with pytest.raises(RuntimeError, match="No functional backend"):
        kernel_registry.get_op("attn")


def test_device_info_reports_what_the_runtime_knows(dev):
    import ctypes

    from rl_kernel_amd import _native

    cu, khz = ctypes.c_int32(0), ctypes.c_int32(0)
    assert _native.load().rlk_device_info(dev.index or 0, ctypes.byref(cu), ctypes.byref(khz)) == 0
    assert cu.value == torch.cuda.get_device_properties(dev).multi_processor_count
    assert 500_000 < khz.value < 5_000_000  # kHz
