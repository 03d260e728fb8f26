"""Kernel registry: string-keyed dispatch from a logical op to the best available backend.

Same contract as the reference's ``kernel_registry`` (rl_engine/kernels/registry.py:68-253):
``get_op(op_type)`` walks an ordered list of backends named by dotted class path, imports lazily,
instantiates with no arguments, caches the instance by backend name, remembers failed backends,
and raises ``RuntimeError`` when none works.  On ROCm the gfx950 HIP backends come first; the
reference maintainer's equivalent change is one enum entry per op at the head of
``_priority_map["rocm"]``.  This mirror registers only the gfx950 HIP backends of the fused
linear-logprob path: a HIP backend that fails to load or construct is an error here, never a
silent switch to a portable implementation, and the CPU platform has no backend at all.
"""

from __future__ import annotations

import importlib
from enum import Enum, EnumMeta
from typing import Any, Dict, Optional, Set, Type

from .platform import device_ctx, logger


class _KernelEnumMeta(EnumMeta):
    def __getitem__(cls, name: str):
        try:
            return super().__getitem__(name)
        except KeyError as e:
            valid = ", ".join(cls.__members__.keys())
            raise ValueError(f"Operator '{name}' not found. Supported backends: {valid}") from e


class OpBackend(Enum, metaclass=_KernelEnumMeta):
    # gfx950 HIP backends of this package
    ROCM_FUSED_LINEAR_LOGP = "rl_kernel_amd.ops.linear_logp.RocmFusedLinearLogpOp"
    ROCM_FUSED_LOGP = "rl_kernel_amd.ops.logp.RocmFusedLogpOp"
    ROCM_RATIO_KL = "rl_kernel_amd.ops.grpo.RocmRatioKLOp"
    ROCM_GRPO_LOSS = "rl_kernel_amd.ops.grpo.RocmGRPOLossOp"
    ROCM_GRPO_FROM_LOGP = "rl_kernel_amd.ops.grpo.RocmGRPOFromLogpOp"
    ROCM_GRPO_STEP = "rl_kernel_amd.ops.grpo_step.RocmFusedGRPOStepOp"
    ROCM_RMS_NORM = "rl_kernel_amd.ops.rms_norm.RocmRMSNormOp"


_LOGP_TYPES = ("logp", "logp_indexed", "logp_online", "logp_online_indexed")


class KernelRegistry:
    def __init__(self) -> None:
        self._instance_cache: Dict[str, Any] = {}
        self._failed_backends: Set[str] = set()
        rocm = {
            "linear_logp": [OpBackend.ROCM_FUSED_LINEAR_LOGP],
            "ratio_kl": [OpBackend.ROCM_RATIO_KL],
            "grpo_loss": [OpBackend.ROCM_GRPO_LOSS],
            "grpo_loss_from_logp": [OpBackend.ROCM_GRPO_FROM_LOGP],
            "grpo_step_from_hidden": [OpBackend.ROCM_GRPO_STEP],
            "rms_norm": [OpBackend.ROCM_RMS_NORM],
        }
        for name in _LOGP_TYPES:
            rocm[name] = [OpBackend.ROCM_FUSED_LOGP]
        # no CPU backends: every op type is known on the CPU platform and answers with the
        # "No functional backend" error
        self._priority_map = {"rocm": rocm, "cpu": {name: [] for name in rocm}}
        logger.info("KernelRegistry initialized for %s", device_ctx.device_type)

    def platform(self) -> str:
        return "rocm" if device_ctx.is_rocm else "cpu"

    def get_op(self, op_type: str) -> Any:
        platform = self.platform()
        candidates = self._priority_map.get(platform, {}).get(op_type)
        if candidates is None:
            raise RuntimeError(f"No functional backend found for {op_type} on {platform}")
        for backend in candidates:
            if backend.name in self._instance_cache:
                return self._instance_cache[backend.name]
            if backend.name in self._failed_backends:
                continue
            op_class = self._load_backend(backend)
            if op_class is None:
                self._failed_backends.add(backend.name)
                continue
            try:
                instance = op_class()
            except Exception as e:  # constructor failure => next candidate
                logger.error("Failed to instantiate %s: %s", backend.name, e)
                self._failed_backends.add(backend.name)
                continue
            self._instance_cache[backend.name] = instance
            return instance
        raise RuntimeError(f"No functional backend found for {op_type} on {platform}")

    def _load_backend(self, backend: OpBackend) -> Optional[Type]:
        module_path, class_name = backend.value.rsplit(".", 1)
        try:
            module = importlib.import_module(module_path)
            return getattr(module, class_name)
        except (ImportError, AttributeError) as e:
            missing = str(getattr(e, "name", "") or "")
            own_bug = missing.startswith("rl_kernel_amd") and not (
                missing == module_path or module_path.startswith(missing))
            if own_bug:
                logger.critical("Internal wrapper implementation bug in '%s': %s", module_path, e)
                raise
            logger.warning("Backend %s unavailable: %s. Falling back...", backend.name, e)
            return None


kernel_registry = KernelRegistry()
