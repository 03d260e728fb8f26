"""Host logic of the registry and op constructors, exercised without a GPU: constructor failure
and import failure fall through to the next backend, failed backends are remembered, instances
are cached (tests/test_kernel_registry.py:10-84 of the reference tests the same contract)."""
import sys
import types

import pytest
import torch


def _fresh_registry():
    from rl_kernel_amd import registry

    return registry, registry.KernelRegistry()


def test_backend_enum_lookup_error_lists_supported_names():
    registry, _ = _fresh_registry()
    assert registry.OpBackend["ROCM_FUSED_LINEAR_LOGP"].value.endswith("RocmFusedLinearLogpOp")
    with pytest.raises(ValueError, match="Supported backends"):
        registry.OpBackend["NOPE"]


@pytest.mark.skipif(torch.cuda.is_available(), reason="CPU-only behaviour")
def test_without_gpu_ops_refuse_to_construct_and_nothing_falls_back_to_cpu():
    from rl_kernel_amd.ops.grpo import RocmGRPOFromLogpOp
    from rl_kernel_amd.ops.linear_logp import RocmFusedLinearLogpOp
    from rl_kernel_amd.ops.logp import RocmFusedLogpOp

    for cls in (RocmFusedLinearLogpOp, RocmFusedLogpOp, RocmGRPOFromLogpOp):
        with pytest.raises(RuntimeError, match="ROCm GPU"):
            cls()
    _, reg = _fresh_registry()
    assert reg.platform() == "cpu"
    with pytest.raises(RuntimeError, match="No functional backend found for linear_logp on cpu"):
        reg.get_op("linear_logp")
    with pytest.raises(RuntimeError, match="No functional backend"):
        reg.get_op("grpo_loss_from_logp")


def test_fallthrough_cache_and_failed_set(monkeypatch):
    registry, reg = _fresh_registry()
    calls = {"bad": 0, "good": 0}

    class Bad:
        def __init__(self):
            calls["bad"] += 1
            raise RuntimeError("native symbol missing")

    class Good:
        def __init__(self):
            calls["good"] += 1

    mod = types.ModuleType("fake_backends")
    mod.Bad, mod.Good = Bad, Good
    monkeypatch.setitem(sys.modules, "fake_backends", mod)

    class FakeBackend:
        def __init__(self, name, value):
            self.name, self.value = name, value

    reg._priority_map["cpu"]["linear_logp"] = [
        FakeBackend("MISSING", "no_such_module_xyz.Op"),
        FakeBackend("BAD", "fake_backends.Bad"),
        FakeBackend("GOOD", "fake_backends.Good"),
    ]
    monkeypatch.setattr(reg, "platform", lambda: "cpu")
    first = reg.get_op("linear_logp")
    assert isinstance(first, Good)
    assert reg._failed_backends == {"MISSING", "BAD"}
    assert reg.get_op("linear_logp") is first           # cached instance, constructors not re-run
    assert calls == {"bad": 1, "good": 1}
    reg._priority_map["cpu"]["only_bad"] = [FakeBackend("BAD", "fake_backends.Bad")]
    with pytest.raises(RuntimeError, match="No functional backend found for only_bad"):
        reg.get_op("only_bad")
    assert calls["bad"] == 1                             # remembered as failed, not retried


def test_argument_validation_needs_no_kernel(monkeypatch):
    """Shape / metadata errors are raised by the Python layer before any launch."""
    from rl_kernel_amd.ops import linear_logp as LL

    op = object.__new__(LL.RocmFusedLinearLogpOp)        # skip the GPU check of the constructor
    h, w, t = torch.randn(4, 8), torch.randn(10, 8), torch.zeros(4, dtype=torch.long)
    with pytest.raises(ValueError, match="must match target_ids shape"):
        op.apply(h, w, torch.zeros(5, dtype=torch.long))
    with pytest.raises(ValueError, match="must match lm_head_weight dim"):
        op.apply(h, torch.randn(10, 7), t)
    with pytest.raises(ValueError, match="vocab_start_index requires"):
        op.apply(h, w, t, vocab_start_index=2)
    with pytest.raises(ValueError, match="global_vocab_size differs"):
        op.apply(h, w, t, global_vocab_size=11)
    with pytest.raises(ValueError, match="temperature"):
        op.apply(h, w, t, temperature=-1.0)
    with pytest.raises(ValueError, match="bias must be 1-D"):
        op.apply(h, w, t, torch.randn(9))
    with pytest.raises(NotImplementedError):
        op.apply(h, w, t)                                # CPU tensors: no HIP path, no fallback
