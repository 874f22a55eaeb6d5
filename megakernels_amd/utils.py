"""Small host helpers (reference ``megakernels/utils.py:12-14,107-109``)."""

from __future__ import annotations

import os

import torch

# Number of workers (compute units) to schedule for when no GPU is visible or
# when a test wants to build a schedule for another machine's worker count.
_WORKER_COUNT_OVERRIDE: int | None = None

# MI355X exposes 256 compute units; used only when nothing else can be probed.
DEFAULT_CU_COUNT = 256


def assert_div(a: int, b: int) -> int:
    """Exact integer division; raises when ``b`` does not divide ``a``
    (reference ``utils.py:12-14``)."""
    if a % b != 0:
        raise AssertionError(f"{a} is not divisible by {b}")
    return a // b


def set_sm_count_override(count: int | None) -> None:
    """Force :func:`get_sm_count` to return ``count`` (``None`` removes the
    override).  Lets schedules be built on a host without a GPU and lets tests
    build the schedules the reference would build for 132 / 148 workers."""
    global _WORKER_COUNT_OVERRIDE
    if count is not None and count <= 0:
        raise ValueError("worker count must be positive")
    _WORKER_COUNT_OVERRIDE = count


def get_sm_count(device) -> int:
    """Number of persistent workers the schedule is built for.

    The reference returns the CUDA multiprocessor count
    (``utils.py:107-109``); on ROCm the same torch property is the compute-unit
    count (256 on MI355X), and one workgroup of the megakernel lives on each.
    Order of precedence: explicit override, ``MK_SM_COUNT`` environment
    variable, the device's CU count, and finally the MI355X default when the
    device is not a GPU.
    """
    if _WORKER_COUNT_OVERRIDE is not None:
        return _WORKER_COUNT_OVERRIDE
    env = os.environ.get("MK_SM_COUNT")
    if env:
        return int(env)
    dev = torch.device(device) if not isinstance(device, torch.device) else device
    if dev.type == "cuda" and torch.cuda.is_available():
        return torch.cuda.get_device_properties(dev).multi_processor_count
    return DEFAULT_CU_COUNT


def trepr(t: torch.Tensor) -> str:
    return f"shape={tuple(t.shape)}, sum={t.sum()}, vals={t}"
