"""GPU parity of the RMSNorm kernels and of the norm + linear log-prob entry points against the CPU
oracle (oracle.rms_norm restates rl_engine/kernels/ops/pytorch/norm/rms_norm.py:54-70).

Tolerances: the norm itself within 1 unit in the last place of the output dtype of the oracle (the
row sum is added in another order; 2e-6 relative in fp32); logp 1e-3 abs for 16-bit inputs and 1e-5
for fp32; gradients 2e-2 relative norm.  The fused entry points must equal the unfused sequence of
this library's own kernels bit for bit."""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def rel(a, b):
    return ((a.float().cpu() - b.float().cpu()).norm() / b.float().norm().clamp_min(1e-30)).item()


@pytest.mark.parametrize("lead,h,dtype", [((2, 16), 4096, torch.float32), ((2, 16), 128, torch.float32),
                                          ((3, 50), 4096, torch.bfloat16), ((70,), 2048, torch.float16),
                                          ((5,), 36, torch.bfloat16), ((9,), 7, torch.float32)])
def test_rmsnorm_forward_matches_oracle(dev, lead, h, dtype):
    from rl_kernel_amd.ops.rms_norm import RocmRMSNormOp

    op = RocmRMSNormOp()
    g = torch.Generator().manual_seed(h)
    x = (torch.randn(*lead, h, generator=g) * 2.0).to(dtype)
    w = (1.0 + 0.3 * torch.randn(h, generator=g)).to(dtype)
    got = op(x.to(dev), w.to(dev))
    want = O.rms_norm(x, w)
    assert got.dtype == dtype and got.shape == x.shape
    if dtype == torch.float32:
        torch.testing.assert_close(got.cpu(), want, rtol=2e-6, atol=2e-6)
    else:   # one rounding step of the 16-bit output at most
        ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        assert ((got.cpu().float() - want.float()).abs() <= ulp * want.float().abs() + 1e-6).all()
        assert (got.cpu() != want).float().mean().item() < 0.01
    fp32 = op.forward_fp32(x.to(dev), w.to(dev))
    assert fp32.dtype == torch.float32
    torch.testing.assert_close(fp32.cpu(), O.rms_norm(x, w, output_dtype=torch.float32), rtol=2e-6, atol=2e-6)
    # a row's output does not depend on how many rows share the batch
    x2 = x.reshape(-1, h).to(dev)
    assert torch.equal(op(x2[:1], w.to(dev)), op(x2, w.to(dev))[:1])
    with pytest.raises(ValueError, match="weight must be 1-D"):
        op(x.to(dev), w[:-1].to(dev))


@pytest.mark.parametrize("n,h,dtype", [(130, 4096, torch.bfloat16), (200, 136, torch.float16),
                                       (65, 50, torch.float32)])
def test_rmsnorm_backward_matches_oracle(dev, n, h, dtype):
    from rl_kernel_amd.ops.rms_norm import RocmRMSNormOp

    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, h, generator=g).to(dtype)
    w = (1.0 + 0.3 * torch.randn(h, generator=g)).to(dtype)
    go = torch.randn(n, h, generator=g).to(dtype)
    xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    RocmRMSNormOp()(xd, wd).backward(go.to(dev))
    d_x, d_w = O.rms_norm_backward(go, x, w)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert rel(xd.grad, d_x) < tol and rel(wd.grad, d_w) < tol
    assert xd.grad.dtype == dtype and wd.grad.dtype == dtype


@pytest.mark.parametrize("lead,h,v,dtype,bias,temp", [
    ((4, 175), 256, 1000, torch.bfloat16, False, 0.7),
    ((300,), 136, 1500, torch.float16, True, 1.0),
    ((1000,), 128, 2304, torch.bfloat16, False, 1.0),
    ((64,), 20, 300, torch.float32, True, 1.3),
])
def test_norm_fused_linear_logp_matches_oracle_and_the_unfused_kernels(dev, lead, h, v, dtype, bias, temp):
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp
    from rl_kernel_amd.ops.rms_norm import RocmRMSNormOp

    g = torch.Generator().manual_seed(h + v)
    x = (torch.randn(*lead, h, generator=g) * 3.0).to(dtype)
    gain = (1.0 + 0.2 * torch.randn(h, generator=g)).to(dtype)
    w = (torch.randn(v, h, generator=g) * 0.1).to(dtype)
    b = (torch.randn(v, generator=g) * 0.3).to(dtype) if bias else None
    tgt = torch.randint(0, v, lead, generator=g)
    tgt.view(-1)[::9] = -100
    up = torch.randn(*lead, generator=g)
    op, norm = RocmFusedLinearLogpOp(), RocmRMSNormOp()

    # oracle composition in fp32: the normalised rows rounded to the input dtype as the reference's
    # norm returns them, then the head
    xo = x.clone().float().requires_grad_(True)
    go_ = gain.clone().float().requires_grad_(True)
    wo = w.clone().float().requires_grad_(True)
    bo = None if b is None else b.clone().float().requires_grad_(True)
    hn = xo * torch.rsqrt(xo.pow(2).mean(dim=-1, keepdim=True) + 1e-6) * go_
    hn_r = hn + (hn.detach().to(dtype).float() - hn.detach())      # straight-through rounding
    want = O.linear_logp(hn_r, wo, tgt, bo, temperature=temp, ignore_index=-100)
    (want * up).sum().backward()

    dev_t = lambda t: None if t is None else t.detach().to(dev)
    x1, g1, w1 = dev_t(x).requires_grad_(True), dev_t(gain).requires_grad_(True), dev_t(w).requires_grad_(True)
    b1 = None if b is None else dev_t(b).requires_grad_(True)
    fused = op(x1, w1, dev_t(tgt), b1, temperature=temp, ignore_index=-100, norm_weight=g1, norm_eps=1e-6)
    (fused * dev_t(up)).sum().backward()
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    assert (fused.detach().cpu() - want.detach()).abs().max().item() < tol
    assert torch.equal(fused.detach().cpu().view(-1)[::9], torch.zeros_like(fused.detach().cpu().view(-1)[::9]))
    gtol = 1e-4 if dtype == torch.float32 else 2e-2
    assert rel(x1.grad, xo.grad) < gtol and rel(g1.grad, go_.grad) < gtol and rel(w1.grad, wo.grad) < gtol
    if b is not None:
        assert rel(b1.grad, bo.grad) < gtol

    # unfused: this library's norm op, then its linear_logp op -- same bits forward and backward
    x2, g2, w2 = dev_t(x).requires_grad_(True), dev_t(gain).requires_grad_(True), dev_t(w).requires_grad_(True)
    b2 = None if b is None else dev_t(b).requires_grad_(True)
    unfused = op(norm(x2, g2), w2, dev_t(tgt), b2, temperature=temp, ignore_index=-100)
    (unfused * dev_t(up)).sum().backward()
    assert torch.equal(fused, unfused)
    assert torch.equal(x1.grad, x2.grad) and torch.equal(g1.grad, g2.grad) and torch.equal(w1.grad, w2.grad)


def test_norm_fused_path_walks_several_token_blocks(dev):
    """More than 8192 tokens: the normalised rows exist one block at a time, dW and d_gain are added
    up across the blocks; checked against the unfused kernels (bitwise forward, gradients within the
    rounding of another summation order) and, on sampled rows, against the oracle."""
    from rl_kernel_amd import _native
    from rl_kernel_amd.ops import linear_logp as LL
    from rl_kernel_amd.ops.rms_norm import rmsnorm_backward, rmsnorm_forward
    import ctypes

    n, h, v, blk = 20000, 512, 4096, 8192
    g = torch.Generator(device=dev).manual_seed(8)
    x = (torch.randn(n, h, device=dev, generator=g) * 2).to(torch.bfloat16)
    gain = (1.0 + 0.2 * torch.randn(h, device=dev, generator=g)).to(torch.bfloat16)
    w = (torch.randn(v, h, device=dev, generator=g) * 0.05).to(torch.bfloat16)
    tgt = torch.randint(0, v, (n,), device=dev, generator=g)
    up = torch.randn(n, device=dev, generator=g)
    logp, lse, err = LL.fused_norm_linear_logp_forward(x, gain, w, tgt, eps=1e-5, temperature=0.9)
    assert int(err.item()) == 0
    d_x, d_g, d_w, _ = LL.fused_norm_linear_logp_backward(up, x, gain, w, tgt, lse, eps=1e-5,
                                                          temperature=0.9)
    # the unfused kernels on the same blocks of 8192 tokens (the launch plan, hence the summation
    # order inside a row, is a function of the token count of a call)
    hn = rmsnorm_forward(x, gain, 1e-5)
    dw_u = torch.zeros_like(d_w)
    dg_u = torch.zeros_like(d_g)
    for t0 in range(0, n, blk):
        sl = slice(t0, min(n, t0 + blk))
        logp_u, lse_u, _ = LL.fused_linear_logp_forward(hn[sl], w, tgt[sl], temperature=0.9)
        assert torch.equal(logp[sl], logp_u) and torch.equal(lse[sl], lse_u)
        dh_b, dw_b, _ = LL.fused_linear_logp_backward(up[sl], hn[sl], w, tgt[sl], lse[sl], temperature=0.9)
        dx_b, dg_b = rmsnorm_backward(x[sl], gain, 1e-5, dh_b)
        assert torch.equal(d_x[sl], dx_b)
        dw_u += dw_b
        dg_u += dg_b
    assert rel(d_w, dw_u) < 1e-5 and rel(d_g, dg_u) < 1e-5
    rows = torch.tensor([0, blk - 1, blk, 2 * blk - 1, 2 * blk, n - 1])
    want = O.linear_logp(O.rms_norm(x[rows].cpu(), gain.cpu(), eps=1e-5), w.cpu(), tgt[rows].cpu(),
                         temperature=0.9)
    assert (logp[rows].cpu() - want).abs().max().item() < 1e-3
    # the workspace does not grow with the token count beyond one block
    lib = _native.load()
    sizes = []
    for tokens in (32768, 65536, 1 << 20):
        need = ctypes.c_size_t(0)
        assert lib.rlk_linear_logp_rmsnorm_bwd_workspace_bytes(tokens, 4096, 128256, 0, 0,
                                                               ctypes.byref(need)) == 0
        sizes.append(need.value)
    assert sizes[0] == sizes[1] == sizes[2] and sizes[0] <= (1 << 29)   # at most 0.5 GiB at the Llama head
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_rmsnorm_fwd_workspace_bytes(32768, 4096, 128256, 0, ctypes.byref(need)) == 0
    assert need.value <= (1 << 27)
    # only d_gain wanted: no d_x buffer to run the norm backward in, the blocks are halved instead
    _, d_g2, _, _ = LL.fused_norm_linear_logp_backward(up, x, gain, w, tgt, lse, eps=1e-5, temperature=0.9,
                                                      need_x=False, need_weight=False)
    assert rel(d_g2, dg_u) < 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp32_gain_over_16_bit_activations_is_not_rounded(dev, dtype):
    """The reference multiplies by weight.float() (rl_engine/kernels/ops/pytorch/norm/rms_norm.py:66-70):
    an fp32 gain over 16-bit activations must enter the product unrounded.  The gain here is chosen
    so that rounding it to the activation dtype first would move many outputs by one unit in the
    last place: the result must equal the oracle's (fp32 gain) wherever the two differ."""
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp
    from rl_kernel_amd.ops.rms_norm import RocmRMSNormOp

    g = torch.Generator().manual_seed(77)
    n, h, v = 192, 256, 700
    x = (torch.randn(n, h, generator=g) * 2.0).to(dtype)
    gain = 1.0 + 0.37 * torch.rand(h, generator=g) + 1.0 / 1024.0 / 3.0   # fp32, off the 16-bit grids
    assert not torch.equal(gain.to(dtype).float(), gain)
    want = O.rms_norm(x, gain)
    rounded_first = O.rms_norm(x, gain.to(dtype))
    assert (want != rounded_first).float().mean().item() > 0.02      # the case does discriminate
    got = RocmRMSNormOp()(x.to(dev), gain.to(dev)).cpu()
    # same fp32 expression as the oracle: at most one unit in the last place apart, and strictly
    # closer to the unrounded-gain result than to the rounded-gain one
    assert torch.allclose(got.float(), want.float(), rtol=2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10,
                          atol=1e-6)
    assert (got != want).float().mean().item() < 0.25 * (rounded_first != want).float().mean().item() + 1e-3

    go = torch.randn(n, h, generator=g).to(dtype)
    xd, gd = x.to(dev).requires_grad_(True), gain.to(dev).requires_grad_(True)
    RocmRMSNormOp()(xd, gd).backward(go.to(dev))
    d_x, d_w = O.rms_norm_backward(go, x, gain)
    assert gd.grad.dtype == torch.float32
    assert rel(xd.grad, d_x) < 1e-2 and rel(gd.grad, d_w) < 1e-4

    # the norm inside the head takes the fp32 gain too: same bits as norm op -> head op
    w = (torch.randn(v, h, generator=g) * 0.1).to(dtype)
    tgt = torch.randint(0, v, (n,), generator=g)
    op = RocmFusedLinearLogpOp()
    fused = op(x.to(dev), w.to(dev), tgt.to(dev), norm_weight=gain.to(dev))
    unfused = op(RocmRMSNormOp()(x.to(dev), gain.to(dev)), w.to(dev), tgt.to(dev))
    assert torch.equal(fused, unfused)
    ref = O.linear_logp(O.rms_norm(x, gain), w, tgt)
    assert (fused.cpu() - ref).abs().max().item() < 1e-3
