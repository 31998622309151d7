"""Small helpers shared by the host-side operators."""
from __future__ import annotations

import torch

from . import _lib

_checked_devices = set()


def stream_ptr(device: torch.device) -> int:
    """Raw handle of the current HIP stream of ``device`` (what the C ABI launches on)."""
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be on a GPU device (got {t.device}); this library has no CPU path")
    idx = t.device.index if t.device.index is not None else torch.cuda.current_device()
    if idx not in _checked_devices:
        _lib.call("infllmv2_check_device", idx)
        _checked_devices.add(idx)


def ptr(t):
    return 0 if t is None else t.data_ptr()


def flat_rows(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n
