"""Policy head + frozen reference head in one launch (rlk_linear_logp_fwd_pair) and its logits-fed
counterpart (rlk_logp_from_logits_pair): every output must equal the single-head call bit for bit,
and match the CPU oracle within the usual tolerances (logp 1e-3 abs for 16-bit inputs, 1e-5 for
fp32)."""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


@pytest.mark.parametrize("n,h,v,dtype,bias,temp", [
    (300, 64, 1000, torch.bfloat16, False, 1.0),       # ragged token block and vocab tile
    (1500, 256, 9000, torch.bfloat16, False, 0.7),     # several vocab splits + a general tail tile
    (700, 128, 2304, torch.float16, False, 1.0),       # full tiles only: both heads in one pipeline
    (257, 64, 513, torch.float16, True, 1.3),          # biased heads, ragged tiles
    (600, 128, 2304, torch.bfloat16, True, 0.7),       # biased heads on full tiles: each head adds its own bias
    (64, 20, 300, torch.float32, True, 1.0),           # fp32 matrix-core kernels
    (4096, 1024, 40960, torch.bfloat16, False, 1.0),   # many tiles per workgroup and head
])
def test_pair_forward_equals_two_single_forwards(dev, n, h, v, dtype, bias, temp):
    from rl_kernel_amd.ops import linear_logp as LL

    g = torch.Generator().manual_seed(n + v)
    hidden = torch.randn(n, h, generator=g).to(dtype).to(dev)
    w_pol = (torch.randn(v, h, generator=g) * 0.1).to(dtype).to(dev)
    w_ref = (w_pol.float() + 0.02 * torch.randn(v, h, generator=g).to(dev)).to(dtype)
    b_pol = (torch.randn(v, generator=g) * 0.3).to(dev) if bias else None
    b_ref = (torch.randn(v, generator=g) * 0.3).to(dev) if bias else None
    tgt = torch.randint(0, v, (n,), generator=g)
    tgt[::13] = -100
    tgt = tgt.to(dev)

    logp, lse, ref_logp, ref_lse, err = LL.fused_linear_logp_forward_pair(
        hidden, w_pol, w_ref, tgt, b_pol, b_ref, temperature=temp, ignore_index=-100)
    a_logp, a_lse, _ = LL.fused_linear_logp_forward(hidden, w_pol, tgt, b_pol, temperature=temp,
                                                    ignore_index=-100)
    b_logp, b_lse, _ = LL.fused_linear_logp_forward(hidden, w_ref, tgt, b_ref, temperature=temp,
                                                    ignore_index=-100)
    assert int(err.item()) == 0
    assert torch.equal(logp, a_logp) and torch.equal(lse, a_lse)
    assert torch.equal(ref_logp, b_logp) and torch.equal(ref_lse, b_lse)
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    rows = torch.arange(0, n, max(1, n // 64))
    for got, w, b in ((logp, w_pol, b_pol), (ref_logp, w_ref, b_ref)):
        want = O.linear_logp(hidden[rows].cpu(), w.cpu(), tgt[rows].cpu(),
                             None if b is None else b.cpu(), temperature=temp, ignore_index=-100)
        assert (got[rows].cpu() - want).abs().max().item() < tol
    assert torch.equal(ref_logp[::13], torch.zeros_like(ref_logp[::13]))


def test_pair_forward_at_the_llama_head(dev):
    from rl_kernel_amd.ops import linear_logp as LL

    n, h, v = 8192, 4096, 128256
    g = torch.Generator(device=dev).manual_seed(31)
    hidden = torch.randn(n, h, device=dev, generator=g).to(torch.bfloat16)
    w_pol = torch.empty(v, h, device=dev, dtype=torch.bfloat16)
    w_ref = torch.empty(v, h, device=dev, dtype=torch.bfloat16)
    for v0 in range(0, v, 16384):
        v1 = min(v, v0 + 16384)
        base = torch.randn(v1 - v0, h, device=dev, generator=g) * 0.02
        w_pol[v0:v1] = base.to(torch.bfloat16)
        w_ref[v0:v1] = (base + 0.002 * torch.randn(v1 - v0, h, device=dev, generator=g)).to(torch.bfloat16)
    tgt = torch.randint(0, v, (n,), device=dev, generator=g)
    out = LL.fused_linear_logp_forward_pair(hidden, w_pol, w_ref, tgt)
    a = LL.fused_linear_logp_forward(hidden, w_pol, tgt)
    b = LL.fused_linear_logp_forward(hidden, w_ref, tgt)
    assert torch.equal(out[0], a[0]) and torch.equal(out[1], a[1])
    assert torch.equal(out[2], b[0]) and torch.equal(out[3], b[1])
    rows = torch.arange(3, n, n // 12)[:12]
    want = O.linear_logp(hidden[rows].cpu(), w_ref.cpu(), tgt[rows].cpu())
    assert (out[2][rows].cpu() - want).abs().max().item() < 1e-3
    # the k3 KL of the two heads is small and non-negative
    d = out[2] - out[0]
    kl = (d.exp() - d - 1.0)
    assert (kl >= -1e-6).all() and kl.mean().item() < 0.1


def test_op_with_reference_gradients_and_argument_errors(dev):
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp

    op = RocmFusedLinearLogpOp()
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(3, 90, 128, generator=g).to(torch.bfloat16).to(dev)
    w_pol = (torch.randn(1111, 128, generator=g) * 0.1).to(torch.bfloat16).to(dev)
    w_ref = (torch.randn(1111, 128, generator=g) * 0.1).to(torch.bfloat16).to(dev)
    tgt = torch.randint(0, 1111, (3, 90), generator=g).to(dev)
    up = torch.randn(3, 90, generator=g).to(dev)

    h1, w1 = hidden.clone().requires_grad_(True), w_pol.clone().requires_grad_(True)
    w_ref_p = w_ref.clone().requires_grad_(True)
    logp, ref_logp = op.with_reference(h1, w1, w_ref_p, tgt, temperature=0.8)
    assert logp.requires_grad and not ref_logp.requires_grad
    (logp * up).sum().backward()
    assert w_ref_p.grad is None                                   # frozen head
    h2, w2 = hidden.clone().requires_grad_(True), w_pol.clone().requires_grad_(True)
    single = op(h2, w2, tgt, temperature=0.8)
    (single * up).sum().backward()
    assert torch.equal(logp, single)
    assert torch.equal(h1.grad, h2.grad) and torch.equal(w1.grad, w2.grad)
    with torch.no_grad():
        assert torch.equal(ref_logp, op(hidden, w_ref, tgt, temperature=0.8))

    with pytest.raises(ValueError, match="reference weight shape"):
        op.with_reference(hidden, w_pol, w_ref[:-1], tgt)
    with pytest.raises(ValueError, match="bias or neither"):
        op.with_reference(hidden, w_pol, w_ref, tgt, torch.zeros(1111, device=dev))
    with pytest.raises(ValueError, match="target_ids out of range"):
        op.with_reference(hidden, w_pol, w_ref, tgt + 2000)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_logits_pair_scan_equals_two_scans(dev, dtype):
    from rl_kernel_amd import _native
    from rl_kernel_amd.ops.logp import logp_from_logits

    lib = _native.load()
    g = torch.Generator().manual_seed(9)
    n, v = 77, 5003
    a = (torch.randn(n, v, generator=g) * 2).to(dtype).to(dev)
    b = (torch.randn(n, v, generator=g) * 2).to(dtype).to(dev)
    ids = torch.randint(0, v, (n,), generator=g)
    ids[3] = -5                                                   # out-of-range id -> 0
    ids = ids.to(dev)
    rows = torch.tensor([0, 5, 76, 200, -1, 40], device=dev)     # bad rows are skipped
    dt = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}[dtype]
    for row_idx in (None, rows):
        outs = [torch.full((n,), 123.0, device=dev) for _ in range(4)]
        lses = [torch.full((n,), -77.0, device=dev) for _ in range(4)]
        n_launch = n if row_idx is None else row_idx.numel()
        rc = lib.rlk_logp_from_logits_pair(a.data_ptr(), b.data_ptr(), dt, ids.data_ptr(),
                                           outs[0].data_ptr(), outs[1].data_ptr(), 2,
                                           lses[0].data_ptr(), lses[1].data_ptr(),
                                           None if row_idx is None else row_idx.data_ptr(), n_launch,
                                           n, v, torch.cuda.current_stream(dev).cuda_stream)
        assert rc == 0, lib.rlk_last_error()
        logp_from_logits(a, ids, outs[2], row_idx, lses[2])
        logp_from_logits(b, ids, outs[3], row_idx, lses[3])
        assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[3])
        assert torch.equal(lses[0], lses[2]) and torch.equal(lses[1], lses[3])
    want = O.logp_from_logits(b.cpu(), ids.cpu())
    assert (outs[1][torch.tensor([0, 5, 76, 40])].cpu() - want[torch.tensor([0, 5, 76, 40])]).abs().max() < 2e-3


def test_pair_with_heads_of_different_alignment_is_refused_not_rerouted(dev):
    """Raw C ABI: a 16-byte aligned policy head with a misaligned reference head would put both on
    the fp32 matrix-core kernels and change the policy head's bits; the call is answered with
    RLK_ERR_UNSUPPORTED and enqueues nothing.  (The Python op re-aligns its inputs.)"""
    import ctypes

    from rl_kernel_amd import _native

    lib = _native.load()
    n, h, v = 64, 64, 512
    hidden = torch.randn(n, h, device=dev).to(torch.bfloat16)
    w = (torch.randn(v, h, device=dev) * 0.1).to(torch.bfloat16)
    store = torch.empty(v * h + 8, device=dev, dtype=torch.bfloat16)
    w_ref = store[1:1 + v * h].view(v, h)            # starts 2 bytes past a 16-byte boundary
    w_ref.copy_(w)
    assert w.data_ptr() % 16 == 0 and w_ref.data_ptr() % 16 != 0
    tgt = torch.randint(0, v, (n,), device=dev)
    outs = [torch.full((n,), 5.0, device=dev) for _ in range(4)]
    err = torch.zeros(1, device=dev, dtype=torch.int32)
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_fwd_pair_workspace_bytes(n, h, v, 0, ctypes.byref(need)) == 0
    ws = torch.empty(max(need.value, 16), device=dev, dtype=torch.uint8)
    rc = lib.rlk_linear_logp_fwd_pair(hidden.data_ptr(), w.data_ptr(), w_ref.data_ptr(), None, None,
                                      tgt.data_ptr(), *[o.data_ptr() for o in outs], ws.data_ptr(), ws.numel(),
                                      n, h, v, 0, 0, 1.0, 0, 0, 1, err.data_ptr(),
                                      torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == -2 and b"16-byte" in lib.rlk_last_error()
    assert all(torch.equal(o, torch.full((n,), 5.0, device=dev)) for o in outs)   # nothing was written
    # the op re-aligns what it is given: same call through Python works and matches the single heads
    from rl_kernel_amd.ops import linear_logp as LL

    a = LL.fused_linear_logp_forward_pair(hidden, w, LL._aligned_contiguous(w_ref), tgt)
    b = LL.fused_linear_logp_forward(hidden, w, tgt)
    assert torch.equal(a[0], b[0]) and torch.equal(a[2], b[0])
