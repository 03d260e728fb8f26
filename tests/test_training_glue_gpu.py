"""GPU test of the caller-side glue (extract_logps / grpo_loss_step) against the CPU oracle, with
the fixture of tests/test_deepspeed_training_worker.py:268-294 of the reference (ids
[[6,-100,2],[-100,1,4]], V=13, H=7 -> padded to H=8 for the 16-bit path and H=7 in fp32)."""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


@pytest.mark.parametrize("dtype,h", [(torch.float32, 7), (torch.bfloat16, 8)])
def test_extract_logps_handles_ignore_index_fixture(dev, dtype, h):
    from rl_kernel_amd.registry import kernel_registry
    from rl_kernel_amd.training import extract_logps, safe_token_ids

    torch.manual_seed(3)
    head = torch.nn.Linear(h, 13, bias=True).to(dtype)
    hidden = torch.randn(2, 3, h).to(dtype)
    ids = torch.tensor([[6, -100, 2], [-100, 1, 4]])
    mask = ids != -100
    ref = O.linear_logp(hidden, head.weight.detach(), ids, head.bias.detach(), ignore_index=-100)
    head_d = head.to(dev)
    got = extract_logps(hidden.to(dev), head_d, ids.to(dev), mask.to(dev),
                        kernel_registry.get_op("linear_logp"))
    assert got.dtype == torch.float32
    assert torch.equal(got.cpu()[~mask], torch.zeros(2))
    assert torch.allclose(got.detach().cpu(), ref, atol=1e-5 if dtype == torch.float32 else 1e-3)
    assert torch.equal(safe_token_ids(ids, mask), torch.tensor([[6, 0, 2], [0, 1, 4]]))
    with pytest.raises(ValueError):
        safe_token_ids(ids, mask[:1])


def test_grpo_loss_step_matches_oracle_and_trains(dev):
    from rl_kernel_amd.training import grpo_loss_step

    g = torch.Generator().manual_seed(5)
    b, t, h, v = 8, 24, 64, 515
    head = torch.nn.Linear(h, v, bias=False).to(torch.bfloat16)
    with torch.no_grad():
        head.weight.mul_(0.5)
    hidden = torch.randn(b, t, h, generator=g).to(torch.bfloat16)
    ids = torch.randint(0, v, (b, t), generator=g)
    lens = torch.randint(6, t + 1, (b,), generator=g)
    mask = torch.arange(t)[None, :] < lens[:, None]
    rewards = torch.randn(b, generator=g)
    w = head.weight.detach()
    cur_ref = O.linear_logp(hidden, w, ids.masked_fill(~mask, -100), temperature=0.9,
                            ignore_index=-100)
    old = cur_ref + 0.05 * torch.randn(b, t, generator=g)
    ref = cur_ref + 0.05 * torch.randn(b, t, generator=g)
    adv = O.group_advantages(rewards, samples_per_prompt=4)
    loss_ref, pol_ref, kl_ref, dcur = O.grpo_loss_from_logp(cur_ref, old, ref, adv, mask, beta=0.04)
    dh_ref, dw_ref, _ = O.linear_logp_backward(dcur, hidden, w, ids.masked_fill(~mask, -100),
                                               temperature=0.9, ignore_index=-100)
    head_d = head.to(dev)
    hd = hidden.to(dev).requires_grad_(True)
    res = grpo_loss_step(hd, head_d, ids.to(dev), mask.to(dev), old.to(dev), ref.to(dev),
                         rewards.to(dev), samples_per_prompt=4, beta=0.04, temperature=0.9)
    res.loss.backward()
    assert res.loss.item() == pytest.approx(loss_ref.item(), abs=1e-4)
    assert res.kl.item() == pytest.approx(kl_ref.item(), abs=1e-4)
    assert torch.allclose(res.advantages.cpu(), adv, atol=1e-5)
    rel = lambda a, r: ((a.float().cpu() - r).norm() / r.norm()).item()
    assert rel(hd.grad, dh_ref) < 2e-2 and rel(head_d.weight.grad, dw_ref) < 2e-2
    # one SGD step on the head lowers the loss (tests/test_grpo_loss.py:315-343 of the reference)
    with torch.no_grad():
        head_d.weight -= 2.0 * head_d.weight.grad
    after = grpo_loss_step(hidden.to(dev), head_d, ids.to(dev), mask.to(dev), old.to(dev),
                           ref.to(dev), rewards.to(dev), samples_per_prompt=4, beta=0.04,
                           temperature=0.9)
    assert after.loss.item() < res.loss.item()


@pytest.mark.parametrize("dtype,tol", [("bf16", 1e-3), ("f32", 1e-5)])
def test_single_gpu_grpo_example_trains(dev, dtype, tol):
    """Counterpart of the reference's tests/test_grpo_single_gpu_example.py: the example runs, stays finite,
    agrees with a plain PyTorch recomputation each step and lowers the loss."""
    from rl_kernel_amd.examples.grpo_single_gpu import parse_args, run_training

    metrics = run_training(parse_args(["--steps", "5", "--dtype", dtype, "--seed", "7"]))
    assert len(metrics) == 5
    assert all(m.max_abs_drift < tol for m in metrics)
    assert metrics[0].kl == pytest.approx(0.0, abs=1e-6)        # ref == old == current at step 0
    assert metrics[-1].loss < metrics[0].loss
