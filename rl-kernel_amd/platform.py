"""Device context: which platform the registry should dispatch for.

Mirrors ``DeviceContext`` (rl_engine/platforms/device.py:10-55 of the reference): ROCm is
recognised through ``torch.version.hip``; the preferred dtype on ROCm is bfloat16.
"""

from __future__ import annotations

import logging

import torch

logger = logging.getLogger("rl_kernel_amd")


class DeviceContext:
    def __init__(self) -> None:
        self.device = torch.device("cuda" if torch.cuda.is_available() else "cpu")
        self.is_rocm = False
        self.backend_version = "N/A"
        self.device_type = "cpu"
        if self.device.type == "cuda":
            if getattr(torch.version, "hip", None) is not None:
                self.is_rocm = True
                self.device_type = "rocm"
                self.backend_version = torch.version.hip
            else:
                self.device_type = "cuda"
                self.backend_version = torch.version.cuda

    def get_preferred_dtype(self) -> torch.dtype:
        return torch.bfloat16 if self.is_rocm else torch.float16


device_ctx = DeviceContext()
