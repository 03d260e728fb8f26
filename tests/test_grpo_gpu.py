"""GPU parity of the log-prob-fed GRPO epilogue, group advantages and the logits-fed ratio/KL and
GRPO-loss op classes against the CPU oracle.  fp32 tolerances: 1e-5 on losses and per-token
terms, 1e-6 on advantages (tests/test_grpo_loss.py:59-153 of the reference uses the same)."""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def ops():
    from rl_kernel_amd.ops import grpo

    return grpo


def _batch(seed, b, t, spread=0.3):
    g = torch.Generator().manual_seed(seed)
    cur = -torch.rand(b, t, generator=g) * 3
    old = cur + spread * torch.randn(b, t, generator=g)
    ref = cur + 0.1 * torch.randn(b, t, generator=g)
    adv = torch.randn(b, generator=g)
    lens = torch.randint(max(1, t // 4), t + 1, (b,), generator=g)
    mask = torch.arange(t)[None, :] < lens[:, None]
    return cur, old, ref, adv, mask


@pytest.mark.parametrize("b,t,beta", [(4, 9, 0.0), (8, 64, 0.04), (64, 512, 0.04), (3, 1, 0.1)])
def test_loss_terms_and_gradient_match_oracle(dev, ops, b, t, beta):
    cur, old, ref, adv, mask = _batch(b * 7 + t, b, t)
    loss, pol, kl, grad = O.grpo_loss_from_logp(cur, old, ref, adv, mask, clip_eps=0.2, beta=beta)
    op = ops.RocmGRPOFromLogpOp()
    c = cur.to(dev).requires_grad_(True)
    got = op(c, old.to(dev), ref.to(dev), adv.to(dev), mask.to(dev), clip_eps=0.2, beta=beta)
    got[0].backward()
    assert got[0].item() == pytest.approx(loss.item(), abs=1e-5)
    assert got[1].item() == pytest.approx(pol.item(), abs=1e-5)
    assert got[2].item() == pytest.approx(kl.item(), abs=1e-5)
    assert torch.allclose(c.grad.cpu(), grad, atol=1e-6, rtol=1e-4)
    assert torch.equal(c.grad.cpu()[~mask], torch.zeros(int((~mask).sum())))
    # per-token advantages give the same result as per-sequence ones
    a_tok = adv[:, None].expand(b, t).contiguous()
    again = op(cur.to(dev), old.to(dev), ref.to(dev), a_tok.to(dev), mask.to(dev), clip_eps=0.2,
               beta=beta)
    assert torch.equal(again[0], got[0].detach())
    # ratio / kl per token, masked -> 0
    ratio, klt = op.ratio_and_kl(cur.to(dev), old.to(dev), ref.to(dev), mask.to(dev))
    assert torch.allclose(ratio.cpu(), O.policy_ratio(cur, old, mask), atol=1e-5, rtol=1e-5)
    assert torch.allclose(klt.cpu(), O.reference_kl(cur, ref, mask), atol=1e-6, rtol=1e-4)


def test_each_output_is_differentiable(dev, ops):
    cur, old, ref, adv, mask = _batch(5, 6, 20)
    op = ops.RocmGRPOFromLogpOp()
    _, _, _, g_tot = O.grpo_loss_from_logp(cur, old, ref, adv, mask, beta=0.5)
    _, _, _, g_pol = O.grpo_loss_from_logp(cur, old, ref, adv, mask, beta=0.0)
    c = cur.to(dev).requires_grad_(True)
    out = op(c, old.to(dev), ref.to(dev), adv.to(dev), mask.to(dev), beta=0.5)
    (gp,) = torch.autograd.grad(out[1], c, retain_graph=True)
    (gk,) = torch.autograd.grad(out[2], c, retain_graph=True)
    assert torch.allclose(gp.cpu(), g_pol, atol=1e-6, rtol=1e-4)
    assert torch.allclose(gk.cpu(), (g_tot - g_pol) / 0.5, atol=1e-6, rtol=1e-3)


def test_invariants(dev, ops):
    op = ops.RocmGRPOFromLogpOp()
    cur, old, ref, adv, mask = _batch(11, 5, 12, spread=0.05)
    args = (old.to(dev), ref.to(dev), adv.to(dev), mask.to(dev))
    base = op(cur.to(dev), *args, beta=0.04)
    junk = torch.where(mask, cur, torch.full_like(cur, 55.0))       # garbage under the mask
    assert torch.equal(op(junk.to(dev), *args, beta=0.04)[0], base[0])
    assert torch.equal(op(cur.to(dev), *args, beta=0.04)[0], base[0])  # bitwise repeatable
    same = op(cur.to(dev), cur.to(dev), cur.to(dev), adv.to(dev), mask.to(dev), beta=1.0)
    a_mean = (adv[:, None] * mask).sum() / mask.sum()
    assert same[2].item() == 0.0 and same[1].item() == pytest.approx(-a_mean.item(), abs=1e-6)
    empty = op(cur.to(dev), old.to(dev), ref.to(dev), adv.to(dev), torch.zeros_like(mask).to(dev))
    assert empty[0].item() == 0.0
    nomask = op(cur.to(dev), old.to(dev), None, adv.to(dev), None)
    ref_l = O.grpo_loss_from_logp(cur, old, cur, adv, torch.ones_like(mask))
    assert nomask[0].item() == pytest.approx(ref_l[0].item(), abs=1e-5) and nomask[2].item() == 0.0
    # gradient scales linearly with the upstream factor (tests/test_ratio_kl.py:163-176, reference)
    c1 = cur.to(dev).requires_grad_(True)
    c2 = cur.to(dev).requires_grad_(True)
    op(c1, *args, beta=0.04)[0].backward()
    (4.0 * op(c2, *args, beta=0.04)[0]).backward()
    assert torch.equal(c2.grad, 4.0 * c1.grad)
    with pytest.raises(ValueError):
        op(cur.to(dev), old.to(dev), ref.to(dev), adv[:3].to(dev), mask.to(dev))


def test_group_advantages(dev, ops):
    rewards = torch.tensor([1.0, 3.0, 10.0, 20.0, 30.0])
    got = ops.group_advantages(rewards.to(dev), group_boundaries=[0, 2, 5]).cpu()
    exp = torch.cat([torch.tensor([-1.0, 1.0]),
                     (torch.tensor([10.0, 20.0, 30.0]) - 20.0) / (200.0 / 3.0) ** 0.5])
    assert torch.allclose(got, exp, atol=1e-5)
    x = torch.randn(64 * 16, generator=torch.Generator().manual_seed(1))
    a = ops.group_advantages(x.to(dev), samples_per_prompt=64).cpu()
    assert torch.allclose(a, O.group_advantages(x, samples_per_prompt=64), atol=1e-5)
    b = ops.group_advantages(x.to(dev), group_boundaries=list(range(0, 1025, 64))).cpu()
    assert torch.equal(a, b)
    big = torch.randn(3000, generator=torch.Generator().manual_seed(2))   # groups beyond one wave
    bounds = [0, 1, 1500, 3000]
    assert torch.allclose(ops.group_advantages(big.to(dev), group_boundaries=bounds).cpu(),
                          O.group_advantages(big, group_boundaries=bounds), atol=1e-4)
    assert torch.equal(ops.group_advantages(torch.ones(4, device=dev), samples_per_prompt=2).cpu(),
                       torch.zeros(4))
    for bad in (dict(), dict(samples_per_prompt=64, group_boundaries=[0, 1024]),
                dict(samples_per_prompt=1), dict(samples_per_prompt=7),
                dict(group_boundaries=[0, 5]), dict(group_boundaries=[0, 0, 1024])):
        with pytest.raises(ValueError):
            ops.group_advantages(x.to(dev), **bad)


def _logits_case(seed, b, t, v, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    pol = torch.randn(b, t, v, generator=g).to(dtype)
    ref = torch.randn(b, t, v, generator=g).to(dtype)
    ids = torch.randint(0, v, (b, t), generator=g)
    old = -torch.rand(b, t, generator=g) * 4
    rewards = torch.randn(b, generator=g)
    mask = torch.rand(b, t, generator=g) > 0.25
    return pol, ref, ids, old, rewards, mask


def test_ratio_kl_op_matches_composition_and_backward(dev, ops):
    pol, ref, ids, old, _, mask = _logits_case(3, 4, 6, 37)
    ids_bad = ids.masked_fill(~mask, -100)          # masked positions may hold junk ids
    p = pol.clone().requires_grad_(True)
    lp = O.logp_from_logits(p, ids) if False else torch.log_softmax(p, -1).gather(-1, ids[..., None]).squeeze(-1)
    lr = torch.log_softmax(ref, -1).gather(-1, ids[..., None]).squeeze(-1)
    ratio_ref = torch.exp((lp - old).masked_fill(~mask, 0.0))
    d = (lr - lp).masked_fill(~mask, 0.0)
    kl_ref = torch.exp(d) - d - 1.0
    w = torch.randn(4, 6, generator=torch.Generator().manual_seed(9))
    ((ratio_ref + 2 * kl_ref) * w).sum().backward()

    op = ops.RocmRatioKLOp()
    pd = pol.to(dev).requires_grad_(True)
    rd = ref.to(dev).requires_grad_(True)
    ratio, kl = op(pd, rd, ids_bad.to(dev), mask.to(dev), old.to(dev))
    ((ratio + 2 * kl) * w.to(dev)).sum().backward()
    assert torch.allclose(ratio.detach().cpu(), ratio_ref.detach(), atol=1e-5, rtol=1e-5)
    assert torch.allclose(kl.detach().cpu(), kl_ref.detach(), atol=1e-5, rtol=1e-4)
    assert torch.all(ratio.detach().cpu()[~mask] == 1.0) and torch.all(kl.detach().cpu()[~mask] == 0.0)
    assert torch.allclose(pd.grad.cpu(), p.grad, atol=1e-5, rtol=1e-4)
    assert rd.grad is None
    assert torch.all(pd.grad.cpu()[~mask] == 0.0)
    with pytest.raises(ValueError, match="out-of-range"):
        op(pd, rd, ids.masked_fill(mask, 37).to(dev), mask.to(dev), old.to(dev))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grpo_loss_op_matches_logp_fed_reference(dev, ops, dtype):
    b, t, v = 8, 10, 53
    pol, ref, ids, old, rewards, mask = _logits_case(4, b, t, v, dtype)
    cur_ref = O.logp_from_logits(pol, ids)
    ref_lp = O.logp_from_logits(ref, ids)
    adv = O.group_advantages(rewards, samples_per_prompt=4)
    loss, pl, kl, _ = O.grpo_loss_from_logp(cur_ref, old, ref_lp, adv, mask, clip_eps=0.2, beta=0.01)
    op = ops.RocmGRPOLossOp()
    pd = pol.to(dev).requires_grad_(True)
    got = op(pd, ref.to(dev), ids.to(dev), old.to(dev), rewards.to(dev), mask.to(dev),
             clip_eps=0.2, beta=0.01, samples_per_prompt=4)
    got[0].backward()
    assert got[0].item() == pytest.approx(loss.item(), abs=1e-5)
    assert got[1].item() == pytest.approx(pl.item(), abs=1e-5)
    assert got[2].item() == pytest.approx(kl.item(), abs=1e-5)
    assert pd.grad is not None and torch.isfinite(pd.grad).all()
    assert torch.all(pd.grad[~mask.to(dev)] == 0.0)
    by_bounds = op(pol.to(dev), ref.to(dev), ids.to(dev), old.to(dev), rewards.to(dev), mask.to(dev),
                   clip_eps=0.2, beta=0.01, group_boundaries=[0, 4, 8])
    assert by_bounds[0].item() == pytest.approx(got[0].item(), abs=1e-6)
    if dtype == torch.float32:      # SGD step lowers the loss (tests/test_grpo_loss.py:315-343)
        stepped = (pd - 0.5 * pd.grad).detach()
        after = op(stepped, ref.to(dev), ids.to(dev), old.to(dev), rewards.to(dev), mask.to(dev),
                   clip_eps=0.2, beta=0.01, samples_per_prompt=4)
        assert after[0].item() < got[0].item()
        # autograd of the same composition on the CPU gives the same logits gradient
        pc = pol.clone().requires_grad_(True)
        cur_c = torch.log_softmax(pc, -1).gather(-1, ids[..., None]).squeeze(-1)
        r = torch.exp(cur_c - old).masked_fill(~mask, 0.0)
        a_tok = adv[:, None].expand(b, t).masked_fill(~mask, 0.0)
        pol_t = -torch.minimum(r * a_tok, r.clamp(0.8, 1.2) * a_tok)
        dd = ref_lp - cur_c
        kl_t = (torch.exp(dd) - dd - 1).masked_fill(~mask, 0.0)
        ((pol_t.sum() + 0.01 * kl_t.sum()) / mask.sum()).backward()
        assert torch.allclose(pd.grad.cpu(), pc.grad, atol=1e-6, rtol=1e-3)


def test_fused_step_linear_logp_into_grpo_epilogue(dev, ops):
    """Config-5 pipeline at a small shape: hidden -> fused logp -> fused epilogue -> dH, dW."""
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp

    g = torch.Generator().manual_seed(21)
    b, t, h, v = 8, 40, 64, 777
    hidden = torch.randn(b, t, h, generator=g).to(torch.bfloat16)
    weight = (torch.randn(v, h, generator=g) * 0.1).to(torch.bfloat16)
    ids = torch.randint(0, v, (b, t), generator=g)
    lens = torch.randint(10, t + 1, (b,), generator=g)
    mask = torch.arange(t)[None, :] < lens[:, None]
    rewards = torch.randn(b, generator=g)
    cur_ref = O.linear_logp(hidden, weight, ids)
    old = cur_ref + 0.05 * torch.randn(b, t, generator=g)
    ref = cur_ref + 0.05 * torch.randn(b, t, generator=g)
    adv = O.group_advantages(rewards, samples_per_prompt=8)
    loss_ref, _, _, dcur = O.grpo_loss_from_logp(cur_ref, old, ref, adv, mask, beta=0.04)
    dh_ref, dw_ref, _ = O.linear_logp_backward(dcur, hidden, weight, ids)

    hd = hidden.to(dev).requires_grad_(True)
    wd = weight.to(dev).requires_grad_(True)
    cur = RocmFusedLinearLogpOp()(hd, wd, ids.masked_fill(~mask, -100).to(dev), ignore_index=-100)
    adv_gpu = ops.group_advantages(rewards.to(dev), samples_per_prompt=8)
    loss = ops.RocmGRPOFromLogpOp()(cur, old.to(dev), ref.to(dev), adv_gpu, mask.to(dev), beta=0.04)[0]
    loss.backward()
    rel = lambda a, r: ((a.float().cpu() - r).norm() / r.norm()).item()
    assert loss.item() == pytest.approx(loss_ref.item(), abs=1e-4)
    assert rel(hd.grad, dh_ref) < 2e-2 and rel(wd.grad, dw_ref) < 2e-2


@pytest.mark.parametrize("b,t,h,v,dtype,per_token_adv,with_ref", [
    (8, 40, 64, 777, torch.bfloat16, False, True),        # ragged vocab tile, per-sequence advantages
    (4, 300, 128, 2304, torch.float16, True, True),       # several loss blocks' worth of threads
    (3, 50, 64, 1000, torch.bfloat16, False, False),      # no reference model: KL term off
    (64, 512, 256, 4096, torch.bfloat16, False, True),    # 32768 tokens: 8 loss blocks, vocab splits
    (5, 60, 50, 600, torch.float32, True, True),          # fp32 inputs: behind the fp32 matrix-core kernels
    (6, 33, 36, 300, torch.bfloat16, False, True),        # 16-bit with H % 8 != 0: same
])
def test_epilogue_folded_into_the_forward_equals_the_two_step_route(dev, ops, b, t, h, v, dtype,
                                                                    per_token_adv, with_ref):
    """rlk_linear_logp_fwd_grpo = rlk_linear_logp_fwd + rlk_grpo_loss_from_logp, bit for bit:
    logp, lse, the three scalars, the per-token terms and d loss / d logp; and the op built on it
    gives the gradients of the two-op composition."""
    from rl_kernel_amd.ops import linear_logp as LL
    from rl_kernel_amd.ops.grpo import grpo_from_logp_raw
    from rl_kernel_amd.ops.grpo_step import RocmFusedGRPOStepOp, fused_linear_logp_grpo_forward

    g = torch.Generator().manual_seed(b * 1000 + t)
    hidden = torch.randn(b, t, h, generator=g).to(dtype).to(dev)
    weight = (torch.randn(v, h, generator=g) * 0.1).to(dtype).to(dev)
    ids = torch.randint(0, v, (b, t), generator=g).to(dev)
    lens = torch.randint(t // 4, t + 1, (b,), generator=g)
    mask = (torch.arange(t)[None, :] < lens[:, None]).to(dev)
    marked = ids.masked_fill(~mask, -100)
    adv = (torch.randn(b, t, generator=g) if per_token_adv else torch.randn(b, generator=g)).to(dev)

    logp, lse, _ = LL.fused_linear_logp_forward(hidden.view(-1, h), weight, marked.view(-1),
                                                temperature=0.9, ignore_index=-100)
    old = (logp + 0.05 * torch.randn(b * t, generator=g).to(dev)).view(b, t)
    ref = (logp + 0.05 * torch.randn(b * t, generator=g).to(dev)).view(b, t) if with_ref else None
    out3, ratio, klt, dcur, dkl = grpo_from_logp_raw(logp.view(b, t), old, ref, adv, mask,
                                                     clip_eps=0.2, beta=0.04, want_grad=True,
                                                     want_terms=True)
    f = fused_linear_logp_grpo_forward(hidden.view(-1, h), weight, marked.view(-1), None, old, ref,
                                       adv, mask, seq_len=t, clip_eps=0.2, beta=0.04,
                                       temperature=0.9, ignore_index=-100, want_grad=True,
                                       want_terms=True)
    f_logp, f_lse, f_err, f_out3, f_ratio, f_klt, f_dcur, f_dkl = f
    assert int(f_err.item()) == 0
    assert torch.equal(f_logp, logp) and torch.equal(f_lse, lse)
    assert torch.equal(f_out3, out3)
    assert torch.equal(f_ratio, ratio.view(-1)) and torch.equal(f_klt, klt.view(-1))
    assert torch.equal(f_dcur, dcur.view(-1)) and torch.equal(f_dkl, dkl.view(-1))
    # against the oracle on the kernel's own log-probs
    # (without a reference model the KL term is off: the oracle gets ref = cur, whose k3 term is 0)
    o_loss, o_pol, o_kl, o_dcur = O.grpo_loss_from_logp(
        logp.view(b, t).cpu(), old.cpu(), (logp.view(b, t) if ref is None else ref).cpu(), adv.cpu(),
        mask.cpu(), clip_eps=0.2, beta=0.04)
    assert f_out3[0].item() == pytest.approx(o_loss.item(), abs=2e-5)
    assert torch.allclose(f_dcur.view(b, t).cpu(), o_dcur, atol=1e-7, rtol=1e-4)

    # the op: same gradients as linear_logp op -> GRPO-from-logp op
    hd = hidden.clone().requires_grad_(True)
    wd = weight.clone().requires_grad_(True)
    loss, pol, kl, cur = RocmFusedGRPOStepOp()(hd, wd, ids, mask, old, ref, adv, clip_eps=0.2,
                                               beta=0.04, temperature=0.9)
    assert torch.equal(cur.view(-1), logp) and not cur.requires_grad
    (loss + 0.5 * kl).backward()
    hd2 = hidden.clone().requires_grad_(True)
    wd2 = weight.clone().requires_grad_(True)
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp

    cur2 = RocmFusedLinearLogpOp()(hd2, wd2, marked, temperature=0.9, ignore_index=-100)
    loss2, pol2, kl2 = ops.RocmGRPOFromLogpOp()(cur2, old, ref, adv, mask, clip_eps=0.2, beta=0.04)
    (loss2 + 0.5 * kl2).backward()
    assert torch.equal(loss, loss2) and torch.equal(pol, pol2) and torch.equal(kl, kl2)
    assert torch.equal(hd.grad, hd2.grad) and torch.equal(wd.grad, wd2.grad)


def test_ratio_kl_entry_points_match_the_closed_forms(dev):
    """rlk_ratio_kl_from_logp / _bwd through the C ABI: values and the coefficient of the logits
    gradient against the formulas of the reference's kernels (ratio = exp(cur - old),
    kl = exp(d) - d - 1 with d = ref - cur, d/dcur = g_r * ratio + g_k * (1 - exp(d))), with and
    without a mask and with either upstream gradient absent."""
    from rl_kernel_amd import _native

    lib = _native.load()
    g = torch.Generator().manual_seed(21)
    n = 1000
    cur = torch.randn(n, generator=g) * 0.3 - 4.0
    ref = cur + torch.randn(n, generator=g) * 0.2
    old = cur + torch.randn(n, generator=g) * 0.2
    mask = torch.rand(n, generator=g) > 0.3
    gr, gk = torch.randn(n, generator=g), torch.randn(n, generator=g)
    st = torch.cuda.current_stream().cuda_stream
    cd, rd, od, md, grd, gkd = (t.to(dev) for t in (cur, ref, old, mask.view(torch.uint8), gr, gk))
    ratio = torch.empty(n, device=dev)
    kl = torch.empty(n, device=dev)
    dcur = torch.empty(n, device=dev)
    for m_cpu, m_dev in ((mask, md), (torch.ones(n, dtype=torch.bool), None)):
        mp = None if m_dev is None else m_dev.data_ptr()
        assert lib.rlk_ratio_kl_from_logp(cd.data_ptr(), rd.data_ptr(), od.data_ptr(), mp, n,
                                          ratio.data_ptr(), kl.data_ptr(), st) == 0
        delta = (cur - old).masked_fill(~m_cpu, 0.0)
        d = (ref - cur).masked_fill(~m_cpu, 0.0)
        assert torch.allclose(ratio.cpu(), torch.exp(delta), rtol=1e-6, atol=1e-7)
        # exp(d) - d - 1 cancels near d = 0: the error is a few ulps of 1.0, not of the result
        assert torch.allclose(kl.cpu(), torch.exp(d) - d - 1.0, rtol=1e-5, atol=5e-7)
        assert torch.all(ratio.cpu()[~m_cpu] == 1.0) and torch.all(kl.cpu()[~m_cpu] == 0.0)
        for use_r, use_k in ((True, True), (True, False), (False, True)):
            assert lib.rlk_ratio_kl_from_logp_bwd(
                cd.data_ptr(), rd.data_ptr(), od.data_ptr(), mp, grd.data_ptr() if use_r else None,
                gkd.data_ptr() if use_k else None, n, dcur.data_ptr(), st) == 0
            want = torch.zeros(n)
            if use_r:
                want = want + gr * torch.exp(cur - old)
            if use_k:
                want = want + gk * (1.0 - torch.exp(ref - cur))
            want = want.masked_fill(~m_cpu, 0.0)
            assert torch.allclose(dcur.cpu(), want, rtol=1e-5, atol=1e-6)
    assert lib.rlk_ratio_kl_from_logp(None, rd.data_ptr(), od.data_ptr(), None, n, ratio.data_ptr(),
                                      kl.data_ptr(), st) < 0
