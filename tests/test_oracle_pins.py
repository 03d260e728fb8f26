"""Pins the CPU oracle (torch restatement + C restatement) before anything trusts it.

Every expected value here is either a known answer held by the reference's own
tests (cited), a closed form, or the agreement of two independent
implementations (torch fp32 library routines vs naive double-precision C loops).
"""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O

# tests/test_reference_ops.py:18-28 (reference tree): log_softmax known answers
KA_LOGITS = [[1.0, 2.0, 3.0], [0.5, -0.5, 1.5]]
KA_IDS = [2, 0]
KA_LOGP = [3.0 - math.log(math.e + math.e**2 + math.e**3),
           0.5 - math.log(math.e**0.5 + math.e**-0.5 + math.e**1.5)]


def test_known_answer_closed_form_values():
    assert KA_LOGP[0] == pytest.approx(-0.40760596, abs=1e-7)
    assert KA_LOGP[1] == pytest.approx(-1.40760596, abs=1e-7)


def test_logp_from_logits_known_answers(c_oracle):
    got = O.logp_from_logits(torch.tensor(KA_LOGITS), torch.tensor(KA_IDS))
    assert got.dtype == torch.float32
    assert torch.allclose(got, torch.tensor(KA_LOGP), atol=1e-6)
    got_c = c_oracle.logp_from_logits(np.array(KA_LOGITS), KA_IDS)
    assert np.allclose(got_c, KA_LOGP, atol=1e-12)


def test_linear_logp_known_answers_via_identity_head(c_oracle):
    # W = I makes logits == hidden, so the logits-level known answers pin the linear form too.
    hidden = torch.tensor(KA_LOGITS)
    got = O.linear_logp(hidden, torch.eye(3), torch.tensor(KA_IDS))
    assert torch.allclose(got, torch.tensor(KA_LOGP), atol=1e-6)
    got_c, lse_c = c_oracle.linear_logp(hidden.numpy(), np.eye(3), KA_IDS)
    assert np.allclose(got_c, KA_LOGP, atol=1e-12)
    assert np.allclose(lse_c, [math.log(math.e + math.e**2 + math.e**3),
                               math.log(math.e**0.5 + math.e**-0.5 + math.e**1.5)], atol=1e-12)


def test_temperature_known_answer(c_oracle):
    # tests/test_reference_ops.py:60-71: logits [1,3,-1], id 1, T=0.5
    expected = 6.0 - math.log(math.e**2 + math.e**6 + math.e**-2)
    assert expected == pytest.approx(-0.0184793, abs=1e-6)
    h = torch.tensor([[1.0, 3.0, -1.0]])
    got = O.linear_logp(h, torch.eye(3), torch.tensor([1]), temperature=0.5)
    assert got.item() == pytest.approx(expected, abs=1e-6)
    got_c, _ = c_oracle.linear_logp(h.numpy(), np.eye(3), [1], temperature=0.5)
    assert got_c[0] == pytest.approx(expected, abs=1e-12)
    with pytest.raises(ValueError, match="temperature"):
        O.linear_logp(h, torch.eye(3), torch.tensor([1]), temperature=0.0)


def test_ignore_index_rows_are_exactly_zero(c_oracle):
    # tests/test_reference_ops.py:42-57 and tests/test_deepspeed_training_worker.py:268-294
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(2, 3, 7, generator=g)
    weight = torch.randn(13, 7, generator=g)
    bias = torch.randn(13, generator=g)
    ids = torch.tensor([[6, -100, 2], [-100, 1, 4]])
    got = O.linear_logp(hidden, weight, ids, bias, ignore_index=-100)
    mask = ids != -100
    assert torch.equal(got[~mask], torch.zeros(2))
    safe = ids.masked_fill(~mask, 0)
    ref = torch.log_softmax(torch.nn.functional.linear(hidden, weight, bias), -1) \
        .gather(-1, safe.unsqueeze(-1)).squeeze(-1).masked_fill(~mask, 0.0)
    assert torch.allclose(got, ref, atol=1e-6)
    got_c, _ = c_oracle.linear_logp(hidden.reshape(-1, 7).numpy(), weight.numpy(),
                                    ids.reshape(-1).numpy(), bias.numpy(), ignore_index=-100)
    assert np.allclose(got_c, got.reshape(-1).numpy(), atol=1e-5)
    with pytest.raises(ValueError):
        O.linear_logp(hidden, weight, ids, bias)  # -100 without ignore_index is out of range


@pytest.mark.parametrize("seed,n,h,v,temp,use_bias", [
    (0, 6, 7, 19, 1.0, True), (1, 9, 5, 16, 0.7, False), (2, 17, 32, 300, 1.3, True)])
def test_torch_and_c_forward_agree(c_oracle, seed, n, h, v, temp, use_bias):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g)
    weight = torch.randn(v, h, generator=g)
    bias = torch.randn(v, generator=g) if use_bias else None
    ids = torch.randint(0, v, (n,), generator=g)
    lp, lse = O.linear_logp(hidden, weight, ids, bias, temperature=temp, return_lse=True)
    lp_c, lse_c = c_oracle.linear_logp(hidden.numpy(), weight.numpy(), ids.numpy(),
                                       None if bias is None else bias.numpy(), temperature=temp)
    assert np.allclose(lp.numpy(), lp_c, atol=2e-5)
    assert np.allclose(lse.numpy(), lse_c, atol=2e-5)


@pytest.mark.parametrize("chunk", [1, 3, 5, 16, 64])
def test_online_stats_are_chunking_invariant(chunk):
    g = torch.Generator().manual_seed(11)
    hidden = torch.randn(8, 5, generator=g)
    weight = torch.randn(16, 5, generator=g)
    bias = torch.randn(16, generator=g)
    ids = torch.tensor([0, 2, 3, 6, 7, 11, 12, 15])
    m, s, zt, owner = O.linear_logp_online_stats(hidden, weight, ids, bias, vocab_chunk=chunk)
    lp, lse = O.linear_logp(hidden, weight, ids, bias, return_lse=True)
    assert torch.all(owner == 1)
    assert torch.allclose(m + torch.log(s), lse, atol=1e-5)
    assert torch.allclose(zt - (m + torch.log(s)), lp, atol=1e-5)


def test_four_shard_partition_matches_unsharded():
    # tests/test_linear_logp.py:64-127: n=8, d=5, V=16, shards [0,3,7,12,16], seed 2026, tol 1e-5
    torch.manual_seed(2026)
    hidden, weight, bias = torch.randn(8, 5), torch.randn(16, 5), torch.randn(16)
    ids = torch.tensor([0, 2, 3, 6, 7, 11, 12, 15])
    bounds = [0, 3, 7, 12, 16]
    parts, owners = [], torch.zeros(8, dtype=torch.int32)
    for a, b in zip(bounds[:-1], bounds[1:]):
        m, s, zt, own = O.linear_logp_online_stats(hidden, weight[a:b], ids, bias[a:b],
                                                   vocab_start=a, vocab_chunk=2)
        parts.append((m, s, zt))
        owners += own
    lp, lse = O.combine_online_stats(parts)
    ref, ref_lse = O.linear_logp(hidden, weight, ids, bias, return_lse=True)
    assert torch.all(owners == 1)
    assert torch.allclose(lp, ref, atol=1e-5)
    assert torch.allclose(lse, ref_lse, atol=1e-5)


@pytest.mark.parametrize("use_bias", [True, False])
@pytest.mark.parametrize("temp", [1.0, 0.7])
def test_backward_matches_autograd_and_c(c_oracle, use_bias, temp):
    # shapes of tests/test_linear_logp.py:255-312: V=19, H=7, N=6, ignored rows carry zero grad
    torch.manual_seed(2027)
    weight = torch.randn(19, 7)
    bias = torch.randn(19) if use_bias else None
    hidden = torch.randn(2, 3, 7)
    ids = torch.tensor([[1, -100, 3], [5, -100, 9]])
    grad = torch.tensor([[0.5, 0.3, -1.25], [0.75, -0.2, 1.5]])
    h = hidden.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    b = bias.clone().requires_grad_(True) if use_bias else None
    safe = ids.masked_fill(ids == -100, 0)
    z = torch.nn.functional.linear(h, w, b) / temp
    lp = torch.log_softmax(z, -1).gather(-1, safe.unsqueeze(-1)).squeeze(-1)
    lp = lp.masked_fill(ids == -100, 0.0)
    (lp * grad).sum().backward()
    for chunk in (1, 2, 4, 64):
        dh, dw, db = O.linear_logp_backward(grad, hidden, weight, ids, bias, temperature=temp,
                                            ignore_index=-100, token_chunk=chunk)
        assert torch.allclose(dh, h.grad, atol=1e-5)
        assert torch.allclose(dw, w.grad, atol=1e-5)
        if use_bias:
            assert torch.allclose(db, b.grad, atol=1e-5)
        else:
            assert db is None
    dh_c, dw_c, db_c = c_oracle.linear_logp_backward(
        grad.reshape(-1).numpy(), hidden.reshape(-1, 7).numpy(), weight.numpy(),
        ids.reshape(-1).numpy(), None if bias is None else bias.numpy(), temperature=temp,
        ignore_index=-100)
    assert np.allclose(dh_c.reshape(2, 3, 7), h.grad.numpy(), atol=1e-5)
    assert np.allclose(dw_c, w.grad.numpy(), atol=1e-5)
    if use_bias:
        assert np.allclose(db_c, b.grad.numpy(), atol=1e-5)
    # ignored rows: exactly zero gradient
    assert torch.equal(dh[ids == -100], torch.zeros(2, 7))


def test_backward_is_layout_permutation_invariant():
    torch.manual_seed(3)
    hidden, weight = torch.randn(6, 7), torch.randn(19, 7)
    ids = torch.tensor([1, 7, 3, 5, 0, 9])
    grad = torch.randn(6)
    dh, dw, _ = O.linear_logp_backward(grad, hidden, weight, ids)
    perm = torch.tensor([5, 2, 1, 0, 4, 3])
    dh2, dw2, _ = O.linear_logp_backward(grad[perm].reshape(3, 2), hidden[perm].reshape(3, 2, 7),
                                         weight, ids[perm].reshape(3, 2))
    assert torch.allclose(dh2.reshape(6, 7), dh[perm], atol=1e-6)
    assert torch.allclose(dw2, dw, atol=1e-5)


def test_out_of_range_logits_target_is_zero():
    logits = torch.randn(4, 9)
    ids = torch.tensor([0, -100, 9, 8])
    got = O.logp_from_logits(logits, ids)
    assert got[1] == 0.0 and got[2] == 0.0
    assert got[0] != 0.0 and got[3] != 0.0
    with pytest.raises(ValueError):
        O.logp_from_logits(logits, ids, out_of_range_is_zero=False)


def test_indexed_rows_only():
    logits = torch.randn(2, 3, 9)
    ids = torch.randint(0, 9, (2, 3))
    out = torch.full((2, 3), 123.0)
    O.logp_from_logits_indexed(logits, ids, torch.tensor([0, 4, 99, -1]), out)
    full = O.logp_from_logits(logits, ids)
    assert out.reshape(-1)[0] == full.reshape(-1)[0] and out.reshape(-1)[4] == full.reshape(-1)[4]
    assert torch.all(out.reshape(-1)[[1, 2, 3, 5]] == 123.0)


def test_masked_reductions_known_answers():
    # tests/test_reference_ops.py:79-85
    values = torch.tensor([[1.0, 100.0], [3.0, 4.0]])
    mask = torch.tensor([[True, False], [True, True]])
    assert O.masked_mean(values, mask).item() == pytest.approx(8.0 / 3.0)
    assert O.masked_mean(values, torch.zeros(2, 2, dtype=torch.bool)).item() == 0.0


def test_ratio_and_kl_known_answers():
    # tests/test_reference_ops.py:88-100: cur-old = 0.5, ref-cur = -0.25 everywhere
    cur = torch.tensor([[0.0, -1.0], [-2.0, -3.0]])
    old = cur - 0.5
    ref = cur - 0.25
    mask = torch.tensor([[True, False], [True, True]])
    r = O.policy_ratio(cur, old, mask)
    k = O.reference_kl(cur, ref, mask)
    assert torch.equal(r[~mask], torch.zeros(1)) and torch.equal(k[~mask], torch.zeros(1))
    assert torch.allclose(r[mask], torch.full((3,), math.exp(0.5)))
    assert torch.allclose(k[mask], torch.full((3,), math.exp(-0.25) + 0.25 - 1.0), atol=1e-7)
    assert torch.allclose(O.policy_ratio(cur, cur), torch.ones(2, 2))  # tests/test_ratio_kl.py:92-97


def test_group_advantages_known_answers(c_oracle):
    # tests/test_grpo_loss.py:110-117
    rewards = torch.tensor([1.0, 3.0, 10.0, 20.0, 30.0])
    expected = torch.cat([torch.tensor([-1.0, 1.0]),
                          (torch.tensor([10.0, 20.0, 30.0]) - 20.0) / (200.0 / 3.0) ** 0.5])
    got = O.group_advantages(rewards, group_boundaries=[0, 2, 5])
    assert torch.allclose(got, expected, atol=1e-5)
    assert np.allclose(c_oracle.group_advantages(rewards.numpy(), [0, 2, 5]), expected.numpy(),
                       atol=1e-9)
    # uniform == boundaries (tests/test_grpo_loss.py:101-107); == (x-mean)/std(unbiased=False)
    x = torch.randn(12, generator=torch.Generator().manual_seed(2))
    a = O.group_advantages(x, samples_per_prompt=4)
    b = O.group_advantages(x, group_boundaries=[0, 4, 8, 12])
    xg = x.view(3, 4)
    c = ((xg - xg.mean(1, keepdim=True)) / xg.std(1, keepdim=True, unbiased=False).clamp_min(1e-6))
    assert torch.allclose(a, b, atol=1e-6) and torch.allclose(a, c.reshape(-1), atol=1e-5)
    # constant group: variance floor eps**2 -> zeros, not NaN
    z = O.group_advantages(torch.ones(4), samples_per_prompt=2)
    assert torch.equal(z, torch.zeros(4))
    with pytest.raises(ValueError):
        O.group_advantages(x)
    with pytest.raises(ValueError):
        O.group_advantages(x, samples_per_prompt=4, group_boundaries=[0, 4, 8, 12])
    with pytest.raises(ValueError):
        O.group_advantages(x, samples_per_prompt=5)


@pytest.mark.parametrize("beta", [0.0, 0.04])
def test_grpo_from_logp_matches_autograd_of_composition_and_c(c_oracle, beta):
    g = torch.Generator().manual_seed(7)
    b, t = 4, 9
    cur = (-torch.rand(b, t, generator=g) * 3).requires_grad_(True)
    old = cur.detach() + 0.3 * torch.randn(b, t, generator=g)   # wide enough to hit both clip sides
    ref = cur.detach() + 0.1 * torch.randn(b, t, generator=g)
    adv = torch.randn(b, generator=g)
    mask = torch.rand(b, t, generator=g) > 0.3
    # composition exactly as the logp-fed callers write it (torch ops only)
    ratio = torch.exp(cur - old).masked_fill(~mask, 0.0)
    a_tok = adv[:, None].expand(b, t).masked_fill(~mask, 0.0)
    pol = -torch.minimum(ratio * a_tok, ratio.clamp(0.8, 1.2) * a_tok)
    d = ref - cur
    kl = (torch.exp(d) - d - 1.0).masked_fill(~mask, 0.0)
    denom = mask.sum().float().clamp_min(1e-8)
    loss_ref = pol.sum() / denom + beta * kl.sum() / denom
    loss_ref.backward()
    loss, pl, k, grad = O.grpo_loss_from_logp(cur.detach(), old, ref, adv, mask,
                                              clip_eps=0.2, beta=beta)
    assert loss.item() == pytest.approx(loss_ref.item(), abs=1e-6)
    assert torch.allclose(grad, cur.grad, atol=1e-6)
    assert torch.equal(grad[~mask], torch.zeros(int((~mask).sum())))
    out3, dcur = c_oracle.grpo_from_logp(cur.detach().numpy(), old.numpy(), ref.numpy(),
                                         a_tok.numpy(), mask.numpy(), 0.2, beta)
    assert out3[0] == pytest.approx(loss_ref.item(), abs=1e-6)
    assert out3[1] == pytest.approx(pl.item(), abs=1e-6)
    assert out3[2] == pytest.approx(k.item(), abs=1e-6)
    assert np.allclose(dcur.reshape(b, t), cur.grad.numpy(), atol=1e-6)


def test_grpo_masked_garbage_invariance_and_gradient_linearity():
    # tests/test_grpo_loss.py:290-299 and tests/test_ratio_kl.py:163-176
    g = torch.Generator().manual_seed(9)
    cur = -torch.rand(3, 5, generator=g)
    old = cur + 0.05 * torch.randn(3, 5, generator=g)
    ref = cur + 0.05 * torch.randn(3, 5, generator=g)
    adv = torch.randn(3, generator=g)
    mask = torch.tensor([[1, 1, 0, 0, 0], [1, 1, 1, 1, 0], [1, 0, 0, 0, 0]], dtype=torch.bool)
    base = O.grpo_loss_from_logp(cur, old, ref, adv, mask, beta=0.04)
    junk = torch.where(mask, cur, torch.full_like(cur, 55.0))
    other = O.grpo_loss_from_logp(junk, old, ref, adv, mask, beta=0.04)
    assert base[0].item() == pytest.approx(other[0].item(), abs=1e-7)
    assert torch.allclose(base[3], other[3])
    empty = O.grpo_loss_from_logp(cur, old, ref, adv, torch.zeros_like(mask), beta=0.04)
    assert empty[0].item() == 0.0 and torch.equal(empty[3], torch.zeros_like(cur))


# --------------------------------------------------------------------------- #
# RMSNorm (the step in front of the head)
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("n", [4096, 128])
def test_rms_norm_matches_torch_rms_norm_and_the_manual_formula(n):
    """tests/test_rms_norm.py:22-49 of the reference: torch's own F.rms_norm is an independent
    implementation (tolerance, the reduction order may differ); the hand-written fp32 formula in
    the same float order must agree bit for bit."""
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 16, n, generator=g)
    w = torch.randn(n, generator=torch.Generator().manual_seed(1))
    got = O.rms_norm(x, w, output_dtype=torch.float32)
    torch.testing.assert_close(got, F.rms_norm(x, (n,), weight=w, eps=1e-6), rtol=1e-6, atol=1e-6)
    x_f = x.float()
    manual = x_f * torch.rsqrt(x_f.pow(2).mean(dim=-1, keepdim=True) + 1e-6) * w.float()
    assert torch.equal(got, manual)
    # a row's output does not depend on how many rows share the batch (same file :55-64)
    assert torch.equal(O.rms_norm(x[:1], w, output_dtype=torch.float32), got[:1])
    assert torch.equal(O.rms_norm(x[1:, 3:5], w, output_dtype=torch.float32), got[1:, 3:5])


def test_rms_norm_closed_form_properties_and_dtype_policy():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 64, generator=g) * 3.0
    ones = torch.ones(64)
    out = O.rms_norm(x, ones, eps=0.0)
    assert torch.allclose(out.pow(2).mean(dim=-1), torch.ones(5), atol=1e-5)      # unit mean square
    assert torch.allclose(O.rms_norm(4.0 * x, ones, eps=0.0), out, atol=1e-6)    # scale invariance
    # known answer: x = [3, 4] -> mean square 12.5 -> [3, 4] / sqrt(12.5) times the gain
    ka = O.rms_norm(torch.tensor([[3.0, 4.0]]), torch.tensor([2.0, 0.5]), eps=0.0)
    assert torch.allclose(ka, torch.tensor([[6.0, 2.0]]) / 12.5 ** 0.5, atol=1e-6)
    # the result is computed in fp32 and cast once to the input dtype
    xb = x.to(torch.bfloat16)
    wb = torch.randn(64, generator=g).to(torch.bfloat16)
    assert O.rms_norm(xb, wb).dtype == torch.bfloat16
    assert torch.equal(O.rms_norm(xb, wb), O.rms_norm(xb, wb, output_dtype=torch.float32).to(torch.bfloat16))
    with pytest.raises(ValueError, match="weight must be 1-D"):
        O.rms_norm(x, torch.ones(63))


def test_rms_norm_backward_matches_autograd():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(7, 48, generator=g, dtype=torch.float64).requires_grad_(True)
    w = torch.randn(48, generator=g, dtype=torch.float64).requires_grad_(True)
    go = torch.randn(7, 48, generator=g, dtype=torch.float64)
    y = x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + 1e-6) * w     # float64 autograd
    (y * go).sum().backward()
    d_x, d_w = O.rms_norm_backward(go.float(), x.detach().float(), w.detach().float())
    assert torch.allclose(d_x.double(), x.grad, atol=1e-5)
    assert torch.allclose(d_w.double(), w.grad, atol=1e-5)
    # scale invariance of the norm: with unit gain and eps = 0 the gradient is orthogonal to x
    d_x0, _ = O.rms_norm_backward(go.float(), x.detach().float(), torch.ones(48), eps=0.0)
    assert (d_x0 * x.detach().float()).sum(dim=-1).abs().max().item() < 1e-4
