"""``compact_ignored`` / ``skip_masked``: the op runs its kernels on the rows whose target is not the
ignore index and puts the results back.  Rows do not interact, so the values must be those of the
uncompacted op up to the grouping of fp32 sums (split / chunk counts follow the row count):
log-probs to a few 1e-6, gradients to one rounding of their output type.  The oracle is the
reference's masked convention (rl_engine/testing/reference_ops.py:15-47 and
rl_engine/executors/deepspeed_trainer.py:618-641 of the reference: masked positions give exactly 0
and receive no gradient)."""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

IGN = -100


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


def _case(n, h, v, dtype, share, seed, bias):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g).to(dtype)
    weight = (0.05 * torch.randn(v, h, generator=g)).to(dtype)
    b = (0.1 * torch.randn(v, generator=g)).to(dtype) if bias else None
    ids = torch.randint(0, v, (n,), generator=g)
    ids[torch.rand(n, generator=g) < share] = IGN
    up = torch.randn(n, generator=g)
    return hidden, weight, b, ids, up


def _run(op, dev, hidden, weight, bias, ids, up, **kw):
    hd = hidden.to(dev).requires_grad_(True)
    wd = weight.to(dev).requires_grad_(True)
    bd = None if bias is None else bias.to(dev).requires_grad_(True)
    logp = op(hd, wd, ids.to(dev), bd, ignore_index=IGN, **kw)
    (logp * up.to(dev)).sum().backward()
    return logp.detach(), hd.grad, wd.grad, None if bd is None else bd.grad


@pytest.mark.parametrize("dtype,n,h,v,share,bias", [
    (torch.bfloat16, 700, 256, 1030, 0.4, False),
    (torch.bfloat16, 1500, 320, 2051, 0.9, True),
    (torch.float16, 513, 128, 777, 0.05, True),
    (torch.float32, 300, 72, 515, 0.5, True),
])
def test_compacted_equals_uncompacted_and_oracle(dev, dtype, n, h, v, share, bias):
    from rl_kernel_amd.registry import kernel_registry

    op = kernel_registry.get_op("linear_logp")
    hidden, weight, b, ids, up = _case(n, h, v, dtype, share, 11 + n, bias)
    full = _run(op, dev, hidden, weight, b, ids, up, temperature=0.8)
    comp = _run(op, dev, hidden, weight, b, ids, up, temperature=0.8, compact_ignored=True)
    assert torch.allclose(comp[0], full[0], rtol=0, atol=2e-6 if dtype == torch.float32 else 4e-6)
    ignored = (ids == IGN).to(dev)
    assert torch.equal(comp[0][ignored], torch.zeros(int(ignored.sum()), device=dev))
    assert not comp[1][ignored].any()
    rel = lambda a, r: ((a.float().cpu() - r.float().cpu()).norm() / r.float().cpu().norm()).item()
    tol_same = 1e-5 if dtype == torch.float32 else 4e-3  # one rounding to 16 bits apart at most
    assert rel(comp[1], full[1]) < tol_same and rel(comp[2], full[2]) < tol_same
    if bias:
        assert rel(comp[3], full[3]) < tol_same
    ref = O.linear_logp(hidden, weight, ids, b, temperature=0.8, ignore_index=IGN)
    dh_ref, dw_ref, db_ref = O.linear_logp_backward(up, hidden, weight, ids, b, temperature=0.8,
                                                    ignore_index=IGN)
    assert torch.allclose(comp[0].cpu(), ref, atol=1e-5 if dtype == torch.float32 else 2e-3)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert rel(comp[1], dh_ref) < tol and rel(comp[2], dw_ref) < tol
    if bias:
        assert rel(comp[3], db_ref) < tol


def test_nothing_or_everything_ignored_takes_the_plain_route(dev):
    from rl_kernel_amd.registry import kernel_registry

    op = kernel_registry.get_op("linear_logp")
    hidden, weight, _, ids, up = _case(260, 128, 600, torch.bfloat16, 0.0, 5, False)
    a = _run(op, dev, hidden, weight, None, ids, up)
    b = _run(op, dev, hidden, weight, None, ids, up, compact_ignored=True)
    assert all(torch.equal(x, y) for x, y in zip(a[:3], b[:3]))
    none = torch.full_like(ids, IGN)
    c = _run(op, dev, hidden, weight, None, none, up, compact_ignored=True)
    assert not c[0].any() and not c[1].any() and not c[2].any()
    # without an ignore index the option has nothing to act on
    d = op(hidden.to(dev), weight.to(dev), ids.to(dev), compact_ignored=True)
    assert torch.equal(d, a[0])


def test_compaction_with_norm_and_main_grad_buffer(dev):
    from rl_kernel_amd.registry import kernel_registry

    op = kernel_registry.get_op("linear_logp")
    hidden, weight, _, ids, up = _case(900, 256, 1300, torch.bfloat16, 0.6, 21, False)
    # fp32 main-gradient buffer: two micro-batches accumulate, compacted or not
    bufs = []
    for compact in (False, True):
        main = torch.zeros(1300, 256, device=dev)
        for _ in range(2):
            hd = hidden.to(dev).requires_grad_(True)
            wd = weight.to(dev).requires_grad_(True)
            logp = op(hd, wd, ids.to(dev), ignore_index=IGN, weight_grad_out=main,
                      compact_ignored=compact)
            (logp * up.to(dev)).sum().backward()
            assert wd.grad is None
        bufs.append(main)
    assert ((bufs[0] - bufs[1]).norm() / bufs[0].norm()).item() < 1e-5
    # final RMSNorm inside the op: the norm is row-wise, so compaction commutes with it
    gain = (1.0 + 0.1 * torch.randn(256)).to(dev)
    outs = []
    for compact in (False, True):
        x = hidden.to(dev).requires_grad_(True)
        gn = gain.clone().requires_grad_(True)
        logp = op(x, weight.to(dev), ids.to(dev), ignore_index=IGN, norm_weight=gn,
                  compact_ignored=compact)
        (logp * up.to(dev)).sum().backward()
        outs.append((logp.detach(), x.grad, gn.grad))
    assert torch.allclose(outs[0][0], outs[1][0], rtol=0, atol=4e-6)
    assert ((outs[0][1].float() - outs[1][1].float()).norm() / outs[0][1].float().norm()).item() < 4e-3
    assert ((outs[0][2] - outs[1][2]).norm() / outs[0][2].norm()).item() < 1e-3


def test_grpo_loss_step_skip_masked_matches_fused_step(dev):
    from rl_kernel_amd.training import grpo_loss_step

    g = torch.Generator().manual_seed(9)
    b, t, h, v = 8, 40, 128, 1031
    head = torch.nn.Linear(h, v, bias=False).to(torch.bfloat16).to(dev)
    hidden = torch.randn(b, t, h, generator=g).to(torch.bfloat16)
    ids = torch.randint(0, v, (b, t), generator=g)
    lens = torch.randint(5, t + 1, (b,), generator=g)
    mask = torch.arange(t)[None, :] < lens[:, None]
    rewards = torch.randn(b, generator=g)
    old = -3.0 + 0.1 * torch.randn(b, t, generator=g)
    ref = -3.0 + 0.1 * torch.randn(b, t, generator=g)
    res = []
    for skip in (False, True):
        head.weight.grad = None
        hd = hidden.to(dev).requires_grad_(True)
        r = grpo_loss_step(hd, head, ids.to(dev), mask.to(dev), old.to(dev), ref.to(dev),
                           rewards.to(dev), samples_per_prompt=4, beta=0.04, skip_masked=skip)
        r.loss.backward()
        res.append((r, hd.grad.clone(), head.weight.grad.clone()))
    (a, dha, dwa), (c, dhc, dwc) = res
    assert torch.allclose(a.current_logps, c.current_logps, rtol=0, atol=4e-6)
    for x, y in ((a.loss, c.loss), (a.kl, c.kl), (a.policy_loss, c.policy_loss)):
        assert abs(x.item() - y.item()) < 1e-6
    assert ((dha.float() - dhc.float()).norm() / dha.float().norm()).item() < 4e-3
    assert ((dwa.float() - dwc.float()).norm() / dwa.float().norm()).item() < 4e-3
