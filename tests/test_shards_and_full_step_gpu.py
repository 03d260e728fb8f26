"""GPU parity of three caller-level compositions of the fused linear-logprob kernels:

* the vocab-shard building block at a real shard shape (Llama-3 head cut into 8 shards of 16032
  rows), forward merged on the host the way the reference merges across ranks
  (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:257-266) and backward per shard from the
  merged global lse (same file :285-335);
* the whole GRPO step of BASELINE config 5 at full size (forward -> group advantages -> loss
  epilogue -> backward);
* the tied embedding / lm_head shared gradient (tests/test_linear_logp.py:315-361 of the
  reference).

Tolerances: logp 1e-3 abs (bf16 inputs, fp32 accumulate), gradients 2e-2 relative norm, masked
rows exactly zero.
"""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

LOGP_ATOL = 1e-3
GRAD_REL = 2e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def rel(a, b):
    return ((a.float().cpu() - b.float().cpu()).norm() / b.float().norm().clamp_min(1e-30)).item()


def _randn_rows(rows, cols, dev, gen, dtype, scale=1.0, step=16384):
    out = torch.empty(rows, cols, device=dev, dtype=dtype)
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        out[r0:r1] = (torch.randn(r1 - r0, cols, device=dev, generator=gen) * scale).to(dtype)
    return out


def _dw_rows_from_definition(hidden, weight_rows, vrows, targets, lse, grad, temperature,
                             ignore_index):
    """dW[v] = sum_n g_n / T (1[t_n = v] - exp(z_nv - lse_n)) H[n], fp32 on the host."""
    h = hidden.cpu().float()
    z = h @ weight_rows.cpu().float().t() / temperature
    t = targets.cpu()
    dz = -(z - lse.cpu()[:, None]).exp()
    dz += (t[:, None] == vrows[None, :]).float()
    dz *= (grad.cpu().float() / temperature)[:, None]
    if ignore_index is not None:
        dz[t == ignore_index] = 0.0
    return dz.t() @ h


def test_vocab_shards_at_the_llama_head_forward_and_backward(dev):
    from rl_kernel_amd.ops import linear_logp as LL

    n, h, v, shards = 8192, 4096, 128256, 8
    v_local = v // shards                                  # 16032: not a multiple of the 256-row tile
    assert v_local * shards == v and v_local % 256 != 0
    temp = 0.7
    g = torch.Generator(device=dev).manual_seed(1105)
    hd = _randn_rows(n, h, dev, g, torch.bfloat16)
    wd = _randn_rows(v, h, dev, g, torch.bfloat16, scale=0.02)
    td = torch.randint(0, v, (n,), device=dev, generator=g)
    td[::89] = -100
    # every shard boundary owns at least one target on each side
    for s in range(1, shards):
        td[2 * s] = s * v_local - 1
        td[2 * s + 1] = s * v_local
    gd = torch.randn(n, device=dev, generator=g)
    ignored = td == -100

    # forward: local statistics of every shard, merged on the host
    zt = torch.zeros(n, device=dev)
    lses = []
    for s in range(shards):
        a = s * v_local
        logp_l, lse_l, err = LL.fused_linear_logp_forward(
            hd, wd[a:a + v_local], td, temperature=temp, ignore_index=-100, vocab_start=a,
            strict_targets=False)
        assert int(err.item()) == 0
        owns = (td >= a) & (td < a + v_local)
        zt += torch.where(owns, logp_l + lse_l, torch.zeros_like(logp_l))   # z_t of the owner shard
        lses.append(lse_l)
        # a row whose target lives elsewhere reports logp_local = -lse_local (z_t = 0), bit for bit
        other = ~owns & ~ignored
        assert torch.equal(logp_l[other], -lse_l[other])
        assert torch.equal(logp_l[ignored], torch.zeros_like(logp_l[ignored]))
    lse_g = torch.logsumexp(torch.stack(lses), dim=0)
    logp = torch.where(ignored, torch.zeros_like(zt), zt - lse_g)

    full_logp, full_lse, _ = LL.fused_linear_logp_forward(hd, wd, td, temperature=temp,
                                                          ignore_index=-100)
    assert (logp - full_logp).abs().max().item() < 2e-5       # merged shards == unsharded kernel
    assert (lse_g - full_lse).abs().max().item() < 2e-5
    rows = torch.cat([torch.arange(0, 2 * shards), torch.arange(7, n, n // 16)[:16]])
    ref, ref_lse = O.linear_logp(hd[rows].cpu(), wd.cpu(), td[rows].cpu(), temperature=temp,
                                 ignore_index=-100, return_lse=True)
    assert (logp[rows].cpu() - ref).abs().max().item() < LOGP_ATOL
    assert (lse_g[rows].cpu() - ref_lse).abs().max().item() < LOGP_ATOL

    # backward: every shard from the merged global lse; dH summed over shards, dW concatenated
    dh_sum = torch.zeros(n, h, device=dev)
    dw = torch.empty(v, h, device=dev)
    for s in range(shards):
        a = s * v_local
        d_h, d_w, _ = LL.fused_linear_logp_backward(
            gd, hd, wd[a:a + v_local], td, lse_g, temperature=temp, ignore_index=-100,
            vocab_start=a)
        dh_sum += d_h.float()
        dw[a:a + v_local] = d_w
        del d_h, d_w
    assert torch.equal(dh_sum[ignored], torch.zeros_like(dh_sum[ignored]))
    r_dh, _, _ = O.linear_logp_backward(gd[rows].cpu(), hd[rows].cpu(), wd.cpu(), td[rows].cpu(),
                                        temperature=temp, ignore_index=-100)
    assert rel(dh_sum[rows], r_dh) < GRAD_REL
    full_dh, full_dw, _ = LL.fused_linear_logp_backward(gd, hd, wd, td, full_lse, temperature=temp,
                                                        ignore_index=-100)
    assert rel(dh_sum, full_dh) < GRAD_REL
    assert rel(dw, full_dw) < 2e-3                           # same kernels, other piece boundaries
    del full_dh, full_dw
    # sampled vocab rows on both sides of shard boundaries, and targets of the sampled tokens
    vrows = torch.tensor([0, v_local - 1, v_local, 3 * v_local - 1, 3 * v_local, 5 * v_local + 255,
                          5 * v_local + 256, v - v_local, v - 1])
    ref_dw = _dw_rows_from_definition(hd, wd[vrows], vrows, td, lse_g, gd, temp, -100)
    assert rel(dw[vrows], ref_dw) < GRAD_REL
    col_sum = dw.sum(dim=0)            # every row of dZ sums to zero over the full vocabulary
    assert (col_sum.abs() / dw.abs().sum(dim=0).clamp_min(1e-20)).max().item() < 5e-3


def test_grpo_step_at_the_config_5_shape(dev):
    """BASELINE config 5 at full size: 64 responses x 512 positions (lengths U{128..512}) on the
    Llama-3 head, PPO clip 0.2, k3 KL with beta 0.04, token-mean loss; forward, group advantages,
    loss epilogue and backward chained through the registry ops."""
    from rl_kernel_amd.ops import linear_logp as LL
    from rl_kernel_amd.registry import kernel_registry
    from rl_kernel_amd.training import grpo_loss_step

    b, t, h, v = 64, 512, 4096, 128256
    n = b * t
    g = torch.Generator(device=dev).manual_seed(1005)
    hidden = _randn_rows(n, h, dev, g, torch.bfloat16).view(b, t, h).requires_grad_(True)
    lm_head = torch.nn.Linear(h, v, bias=False, device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        lm_head.weight.copy_(_randn_rows(v, h, dev, g, torch.bfloat16, scale=0.02))
    ids = torch.randint(0, v, (b, t), device=dev, generator=g)
    lens = torch.randint(128, t + 1, (b,), device=dev, generator=g)
    mask = torch.arange(t, device=dev)[None, :] < lens[:, None]
    rewards = torch.randn(b, device=dev, generator=g)

    op = kernel_registry.get_op("linear_logp")
    with torch.no_grad():
        cur0 = op(hidden, lm_head.weight, ids.masked_fill(~mask, -100), ignore_index=-100)
    old = cur0 + 0.05 * torch.randn(b, t, device=dev, generator=g)
    ref = cur0 + 0.05 * torch.randn(b, t, device=dev, generator=g)

    res = grpo_loss_step(hidden, lm_head, ids, mask, old, ref, rewards, samples_per_prompt=b,
                         clip_eps=0.2, beta=0.04)
    res.loss.backward()
    torch.cuda.synchronize()

    cur = res.current_logps.detach()
    assert torch.equal(cur, cur0)                                    # same kernels, same bits
    assert torch.equal(cur[~mask], torch.zeros_like(cur[~mask]))    # masked positions exactly 0
    # forward on sampled rows (first and last position of some responses, a few in between)
    flat_mask = mask.reshape(-1).cpu()
    rows = torch.cat([torch.arange(0, n, t)[:8], torch.arange(300, n, n // 12)[:12]])
    rows = rows[flat_mask[rows]]
    w_cpu = lm_head.weight.detach().cpu()
    h_flat = hidden.detach().reshape(n, h)
    ref_logp = O.linear_logp(h_flat[rows].cpu(), w_cpu, ids.reshape(-1)[rows].cpu())
    assert (cur.reshape(-1)[rows].cpu() - ref_logp).abs().max().item() < LOGP_ATOL

    # the loss terms and d loss / d logp from the oracle on the kernel's own log-probs
    adv_ref = O.group_advantages(rewards.cpu(), samples_per_prompt=b)
    assert torch.allclose(res.advantages.cpu(), adv_ref, atol=1e-5)
    loss_ref, pol_ref, kl_ref, dcur = O.grpo_loss_from_logp(cur.cpu(), old.cpu(), ref.cpu(), adv_ref,
                                                            mask.cpu(), clip_eps=0.2, beta=0.04)
    assert res.loss.item() == pytest.approx(loss_ref.item(), abs=2e-5)
    assert res.policy_loss.item() == pytest.approx(pol_ref.item(), abs=2e-5)
    assert res.kl.item() == pytest.approx(kl_ref.item(), abs=2e-6)

    # backward: masked rows carry no gradient at all; sampled token rows of dH and sampled vocab
    # rows of dW against the definition with the oracle's d loss / d logp as upstream
    d_h = hidden.grad.reshape(n, h)
    assert torch.equal(d_h[~mask.reshape(-1)], torch.zeros_like(d_h[~mask.reshape(-1)]))
    up = dcur.reshape(-1)
    r_dh, _, _ = O.linear_logp_backward(up[rows], h_flat[rows].cpu(), w_cpu,
                                        ids.reshape(-1)[rows].cpu())
    assert rel(d_h[rows], r_dh) < GRAD_REL
    marked = ids.masked_fill(~mask, -100).reshape(-1)
    with torch.no_grad():
        _, lse, _ = LL.fused_linear_logp_forward(h_flat, lm_head.weight.detach(), marked,
                                                 ignore_index=-100)
    hot = ids.reshape(-1)[rows[:3]].cpu()                            # rows that own sampled targets
    vrows = torch.cat([torch.tensor([0, 255, 256, v // 2 + 5, v - 1]), hot])
    ref_dw = _dw_rows_from_definition(h_flat, w_cpu[vrows], vrows, marked, lse, up, 1.0, -100)
    assert rel(lm_head.weight.grad[vrows], ref_dw) < GRAD_REL
    assert torch.isfinite(lm_head.weight.grad).all() and torch.isfinite(d_h).all()


class _EmbeddingLMHead(torch.nn.Module):
    def __init__(self, vocab, hidden_dim):
        super().__init__()
        self.embedding = torch.nn.Embedding(vocab, hidden_dim)
        self.lm_head = torch.nn.Linear(hidden_dim, vocab, bias=False)
        self.lm_head.weight = self.embedding.weight                  # tied

    def forward(self, input_ids):
        return torch.tanh(self.embedding(input_ids))


@pytest.mark.parametrize("dtype,atol_logp,tol_grad", [(torch.float32, 1e-5, 1e-4),
                                                      (torch.bfloat16, 1e-3, 2e-2)])
def test_tied_embedding_shared_gradient_is_layout_invariant(dev, dtype, atol_logp, tol_grad):
    """The lm_head weight is also the embedding table: its gradient is the sum of the head's dW and
    the embedding's scatter of dH, and neither may depend on how the tokens are laid out.  Base
    vectors of the reference's test (tests/test_linear_logp.py:315-361); hidden size 8 instead of
    6 so that the 16-bit run takes the MFMA path."""
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp

    torch.manual_seed(2028)
    model = _EmbeddingLMHead(13, 8).to(dev).to(dtype)
    op = RocmFusedLinearLogpOp()
    base_input_ids = torch.tensor([2, 5, 1, 5, 2, 3])
    base_target = torch.tensor([4, 1, 0, 2, 6, 3])
    base_mask = torch.tensor([True, False, True, True, False, True])
    base_upstream = torch.tensor([0.75, 0.0, -1.25, 0.5, 0.0, 1.0])
    layouts = [((2, 3), [0, 1, 2, 3, 4, 5]), ((3, 2), [5, 2, 1, 0, 4, 3])]

    # oracle: closed-form gradients of the head plus the embedding scatter, in fp32 on the host
    w = model.embedding.weight.detach().cpu().float()
    emb = torch.tanh(w[base_input_ids])                               # [6, 8] hidden states
    emb_r = emb.to(dtype).float()                                     # as the head sees them
    tgt_marked = base_target.masked_fill(~base_mask, -100)
    want_logp = O.linear_logp(emb_r, w, tgt_marked, ignore_index=-100)
    o_dh, o_dw, _ = O.linear_logp_backward(base_upstream, emb_r, w, tgt_marked, ignore_index=-100)
    want_grad = o_dw.clone()
    want_grad.index_add_(0, base_input_ids, o_dh * (1.0 - emb * emb))  # through tanh into the table

    canonical = None
    for lead, order in layouts:
        order_t = torch.tensor(order)
        input_ids = base_input_ids[order_t].reshape(lead).to(dev)
        target = base_target[order_t].reshape(lead)
        mask = base_mask[order_t].reshape(lead)
        upstream = base_upstream[order_t].reshape(lead).masked_fill(~mask, 0.0).to(dev)
        model.zero_grad(set_to_none=True)
        hidden = model(input_ids)
        logps = op(hidden, model.lm_head.weight, target.masked_fill(~mask, -100).to(dev),
                   ignore_index=-100)
        (logps * upstream).sum().backward()
        shared = model.embedding.weight.grad.detach().float().cpu()
        inv = torch.empty(6, dtype=torch.long)
        inv[order_t] = torch.arange(6)
        recovered = logps.detach().reshape(-1).cpu()[inv]
        assert (recovered - want_logp).abs().max().item() < atol_logp
        assert torch.equal(recovered[~base_mask], torch.zeros(2))
        assert rel(shared, want_grad) < tol_grad
        if canonical is None:
            canonical = (recovered, shared)
        else:
            assert torch.allclose(recovered, canonical[0], atol=1e-6)
            assert torch.allclose(shared, canonical[1], atol=1e-6 if dtype == torch.float32 else 2e-2)
