"""Kernel-backend selector kept for signature compatibility with the reference.

The reference chooses between a pure-JAX path and a Pallas kernel through
``select_kernel_backend`` and the ``LINEARNEXUS_KERNEL_BACKEND`` environment variable
(linearnexus/kernels/backend.py:13-60).  Here there is exactly one implementation -- the HIP
kernels -- so every request resolves to :attr:`KernelBackend.HIP`; the ``backend=`` keyword of
the ops is accepted and ignored, as the reference's ``delta_rule_chunkwise`` already does
(delta_net.py:224).
"""
from __future__ import annotations

from enum import Enum
from typing import Optional


class KernelBackend(str, Enum):
    HIP = "hip"


def select_kernel_backend(preferred: Optional[str] = None) -> KernelBackend:
    return KernelBackend.HIP
