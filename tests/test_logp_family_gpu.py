"""GPU parity of the logits-fed selected-log-prob family (nine methods) against the CPU oracle.

Checks follow tests/test_op_accuracy.py:43-141 of the reference: values, storage identity of the
`out` variants, untouched rows outside `row_indices`, zero-filled `*_fp32` indexed variants, the
native out-of-range-id rule (0, no error)."""
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def op():
    from rl_kernel_amd.ops.logp import RocmFusedLogpOp

    return RocmFusedLogpOp()


def _data(seed, shape, v, dtype):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(*shape, v, generator=g) * 3).to(dtype)
    ids = torch.randint(0, v, shape, generator=g)
    return logits, ids


@pytest.mark.parametrize("shape,v,dtype,atol", [
    ((7,), 19, torch.float32, 1e-5),
    ((2, 5), 1000, torch.float32, 1e-5),
    ((3, 4), 50257, torch.float32, 2e-5),       # odd vocab: unaligned rows (head/tail scalar path)
    ((33,), 4099, torch.bfloat16, 1e-5),
    ((33,), 4096, torch.float16, 1e-5),
    ((16,), 128256, torch.bfloat16, 2e-5),
])
def test_apply_fp32_matches_oracle(dev, op, shape, v, dtype, atol):
    logits, ids = _data(0, shape, v, dtype)
    ref = O.logp_from_logits(logits, ids)
    got = op.apply_fp32(logits.to(dev), ids.to(dev))
    assert got.dtype == torch.float32 and got.shape == tuple(shape)
    assert (got.cpu() - ref).abs().max().item() < atol
    assert (op.online_fp32(logits.to(dev), ids.to(dev)).cpu() - ref).abs().max().item() < atol


def test_apply_keeps_logits_dtype_and_call_alias(dev, op):
    logits, ids = _data(1, (4, 6), 300, torch.bfloat16)
    ref = O.logp_from_logits(logits, ids)
    got = op(logits.to(dev), ids.to(dev))
    assert got.dtype == torch.bfloat16 and got.shape == (4, 6)
    assert torch.allclose(got.float().cpu(), ref, atol=5e-2)
    assert torch.equal(got, op.apply(logits.to(dev), ids.to(dev)))


@pytest.mark.parametrize("out_dtype", [torch.float64, torch.float32, torch.float16, torch.bfloat16])
def test_out_variants_write_into_the_callers_tensor(dev, op, out_dtype):
    logits, ids = _data(2, (3, 5), 77, torch.float32)
    ref = O.logp_from_logits(logits, ids)
    for method in (op.out, op.online_out):
        output = torch.full((3, 5), 9.0, device=dev, dtype=out_dtype)
        ptr = output.data_ptr()
        ret = method(logits.to(dev), ids.to(dev), output)
        assert ret is output and ret.data_ptr() == ptr
        tol = 1e-5 if out_dtype in (torch.float32, torch.float64) else 5e-2
        assert torch.allclose(output.double().cpu(), ref.double(), atol=tol)
    with pytest.raises(ValueError):
        op.out(logits.to(dev), ids.to(dev), torch.empty(5, 3, device=dev))


def test_indexed_variants_touch_only_listed_rows(dev, op):
    logits, ids = _data(3, (4, 5), 64, torch.float32)
    ref = O.logp_from_logits(logits, ids).reshape(-1)
    rows = torch.tensor([0, 3, 7, 19, 500, -2])          # the last two are outside the tensor
    for method in (op.indexed_out, op.online_indexed_out):
        output = torch.full((4, 5), 123.0, device=dev)
        ret = method(logits.to(dev), ids.to(dev), rows.to(dev), output)
        assert ret is output
        flat = output.cpu().reshape(-1)
        keep = torch.ones(20, dtype=torch.bool)
        keep[[0, 3, 7, 19]] = False
        assert torch.all(flat[keep] == 123.0)
        assert torch.allclose(flat[~keep], ref[~keep], atol=1e-5)
    for method in (op.indexed_fp32, op.online_indexed_fp32):
        got = method(logits.to(dev), ids.to(dev), rows.to(dev)).cpu().reshape(-1)
        keep = torch.ones(20, dtype=torch.bool)
        keep[[0, 3, 7, 19]] = False
        assert torch.all(got[keep] == 0.0) and torch.allclose(got[~keep], ref[~keep], atol=1e-5)
    empty = op.indexed_fp32(logits.to(dev), ids.to(dev), torch.empty(0, dtype=torch.long, device=dev))
    assert torch.all(empty == 0.0)


def test_out_of_range_ids_give_zero_and_masked_logits_are_ignored(dev, op):
    logits, ids = _data(4, (6,), 40, torch.float32)
    ids[1], ids[4] = -100, 40
    logits[2, 5:9] = float("-inf")
    ref = O.logp_from_logits(logits, ids)
    got = op.apply_fp32(logits.to(dev), ids.to(dev)).cpu()
    assert got[1] == 0.0 and got[4] == 0.0
    assert torch.allclose(got, ref, atol=1e-5)


def test_native_symbol_table(dev):
    from rl_kernel_amd import _C

    for name in ("fused_logp", "fused_logp_forward_out", "fused_logp_forward_fp32",
                 "fused_logp_forward_indexed_out", "fused_logp_forward_indexed_fp32",
                 "fused_logp_forward_online_out", "fused_logp_forward_online_fp32",
                 "fused_logp_forward_online_indexed_out", "fused_logp_forward_online_indexed_fp32",
                 "fused_linear_logp", "fused_linear_logp_sm90"):
        assert hasattr(_C, name)
    logits, ids = _data(5, (9,), 31, torch.float16)
    assert _C.fused_logp(logits.to(dev), ids.to(dev)).dtype == torch.float16
    with pytest.raises(RuntimeError):
        _C.fused_logp(logits.to(dev)[0], ids.to(dev))
    with pytest.raises(RuntimeError):
        _C.fused_logp_forward_out(logits.to(dev), ids.to(dev).int(), torch.empty(9, device=dev))
    g = torch.Generator().manual_seed(6)
    hidden = torch.randn(20, 32, generator=g).to(torch.bfloat16)
    weight = torch.randn(50, 32, generator=g).to(torch.bfloat16)
    tgt = torch.randint(0, 50, (20,), generator=g)
    logp, lse = _C.fused_linear_logp(hidden.to(dev), weight.to(dev), tgt.to(dev).int())
    ref, ref_lse = O.linear_logp(hidden, weight, tgt, return_lse=True)
    assert torch.allclose(logp.cpu(), ref, atol=1e-3) and torch.allclose(lse.cpu(), ref_lse, atol=1e-3)


def test_full_vocab_rows_property(dev, op):
    """At the Llama head width the row sum of exp(logp over all ids) must be 1."""
    v = 128256
    g = torch.Generator(device=dev).manual_seed(3)
    logits = (torch.randn(4, v, device=dev, generator=g) * 2).to(torch.bfloat16)
    ids = torch.arange(v, device=dev)
    total = torch.zeros(4, device=dev, dtype=torch.float64)
    for v0 in range(0, v, 4096):
        chunk = ids[v0:v0 + 4096]
        rep = logits[:, None, :].expand(4, chunk.numel(), v).reshape(-1, v)
        lp = op.apply_fp32(rep, chunk.repeat(4))
        total += lp.double().exp().view(4, -1).sum(1)
    assert torch.allclose(total, torch.ones(4, device=dev, dtype=torch.float64), atol=1e-4)


def test_compiled_binding_calls_reach_the_kernels(dev):
    """`fused_linear_logp_sm90` and the `fused_logp_forward_*` family through the compiled PyTorch
    extension (the names of csrc/ops.cpp:75-99 of the reference): values against the oracle,
    storage identity of the `*_out` forms, RuntimeError for malformed arguments."""
    from rl_kernel_amd import _C

    assert _C.COMPILED
    mod = _C.compiled_module
    g = torch.Generator().manual_seed(17)
    hidden = torch.randn(300, 128, generator=g).to(torch.bfloat16)
    weight = (torch.randn(1000, 128, generator=g) * 0.1).to(torch.bfloat16)
    bias = torch.randn(1000, generator=g) * 0.2
    target = torch.randint(0, 1000, (300,), generator=g)
    logp, lse = mod.fused_linear_logp_sm90(hidden.to(dev), weight.to(dev), target.to(dev).int(),
                                           bias.to(dev))
    want, want_lse = O.linear_logp(hidden, weight, target, bias, return_lse=True)
    assert logp.dtype == torch.float32 and (logp.cpu() - want).abs().max().item() < 1e-3
    assert (lse.cpu() - want_lse).abs().max().item() < 1e-3
    no_bias = mod.fused_linear_logp_sm90(hidden.to(dev), weight.to(dev), target.to(dev))
    assert (no_bias[0].cpu() - O.linear_logp(hidden, weight, target)).abs().max().item() < 1e-3
    # a vocab shard: targets outside it report logp = -lse
    shard = mod.fused_linear_logp(hidden.to(dev), weight[:500].contiguous().to(dev), target.to(dev), None)
    outside = (target >= 500).to(dev)
    assert torch.equal(shard[0][outside], -shard[1][outside])
    with pytest.raises(RuntimeError, match="hidden-dim mismatch"):
        mod.fused_linear_logp_sm90(hidden.to(dev), weight[:, :64].contiguous().to(dev), target.to(dev))

    logits = (torch.randn(50, 777, generator=g) * 2).to(torch.float16).to(dev)
    ids = torch.randint(0, 777, (50,), generator=g).to(dev)
    out = torch.full((50,), 123.0, device=dev)
    ret = mod.fused_logp_forward_out(logits, ids, out)
    assert ret.data_ptr() == out.data_ptr()
    ref = O.logp_from_logits(logits.cpu(), ids.cpu())
    assert (out.cpu() - ref).abs().max().item() < 2e-3
    rows = torch.tensor([3, 7, 49], device=dev)
    part = mod.fused_logp_forward_online_indexed_fp32(logits, ids, rows)
    assert torch.equal(part[rows], out[rows]) and part.sum().item() == out[rows].sum().item()
    assert mod.fused_logp(logits, ids).dtype == torch.float16
    with pytest.raises(RuntimeError, match="token_ids must be int64"):
        mod.fused_logp_forward_fp32(logits, ids.int())
