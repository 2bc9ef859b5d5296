"""Copies between host and device, counted.

Every copy that the engine, the sampler, the replay tool and the command line make goes through one of these
functions, so that a report can say how many calls and bytes a workload moved each way, and a test can hold a
step to its budget: one copy to the device (the step's packed metadata), none back. The reference counts the
same six numbers in its runtime (include/microllm/runtime/runtime.h:24-31) and checks that a forward makes no
copy to the host (tests/inference/hip_shape_matrix_test.cpp:101-136).
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Union

import numpy as np
import torch


@dataclass
class TransferStats:
    host_to_device_calls: int = 0
    device_to_host_calls: int = 0
    device_to_device_calls: int = 0
    host_to_device_bytes: int = 0
    device_to_host_bytes: int = 0
    device_to_device_bytes: int = 0


_stats = TransferStats()


def transfer_stats() -> TransferStats:
    return dataclasses.replace(_stats)


def reset_transfer_stats() -> None:
    global _stats
    _stats = TransferStats()


def _bytes(tensor: torch.Tensor) -> int:
    return tensor.numel() * tensor.element_size()


def copy_to_device(destination: torch.Tensor, source: torch.Tensor, non_blocking: bool = False) -> None:
    """``destination`` (device) takes ``source`` (host, pinned if the copy is to overlap)."""
    destination.copy_(source, non_blocking=non_blocking)
    _stats.host_to_device_calls += 1
    _stats.host_to_device_bytes += _bytes(source)


def on_device(values: Union[np.ndarray, torch.Tensor, list], device: torch.device, dtype=None) -> torch.Tensor:
    """A new device tensor holding ``values`` from the host."""
    host = values if isinstance(values, torch.Tensor) else torch.as_tensor(values, dtype=dtype)
    _stats.host_to_device_calls += 1
    _stats.host_to_device_bytes += _bytes(host)
    return host.to(device)


def on_host(tensor: torch.Tensor) -> torch.Tensor:
    """A host copy of a device tensor (waits for the work that makes it)."""
    if tensor.is_cuda:
        _stats.device_to_host_calls += 1
        _stats.device_to_host_bytes += _bytes(tensor)
    return tensor.detach().to("cpu")


def count_copy_to_host(tensor: torch.Tensor) -> None:
    """A copy to the host that the caller makes itself (into pinned memory, without waiting) still counts."""
    _stats.device_to_host_calls += 1
    _stats.device_to_host_bytes += _bytes(tensor)


def device_copy(tensor: torch.Tensor) -> torch.Tensor:
    """A copy on the same device."""
    _stats.device_to_device_calls += 1
    _stats.device_to_device_bytes += _bytes(tensor)
    return tensor.clone()
