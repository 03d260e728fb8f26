"""GPU parity of the scalar-FMA path (fp32 tensors, hidden sizes that are not a multiple of 8)
against the CPU oracle; fp32 tolerance 1e-5 on logp (BASELINE config 1 is one of the cases)."""
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
    ((5,), 3000, 40, torch.float32, False, 1.0, False, 2e-5),       # hidden block spans LDS limits
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
    with pytest.raises(NotImplementedError):
        op(hidden.to(dev), weight.to(dev).half(), tgt.to(dev))


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
