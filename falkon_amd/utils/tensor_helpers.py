"""Stride tests and order-preserving allocation.

Same contracts as falkon/utils/tensor_helpers.py:76-213: a tensor is usable when
some stride equals one, outputs are created in the memory order of a model tensor.
"""
from typing import Tuple, Union

import torch

__all__ = ("is_contig", "is_f_contig", "create_C", "create_fortran", "create_same_stride")


def is_contig(tensor: torch.Tensor) -> bool:
    """True when some stride is 1 (falkon/utils/tensor_helpers.py:210-213)."""
    return any(s == 1 for s in tensor.stride())


def is_f_contig(tensor: torch.Tensor, strict: bool = False) -> bool:
    """Column-major test (falkon/utils/tensor_helpers.py:149-198).

    ``strict`` decides how 2-D tensors with a singleton dimension are treated:
    non-strict accepts either unit stride, strict demands the column-major one.
    """
    strides, sizes = tensor.stride(), tensor.shape
    if len(sizes) == 0:
        return True
    if len(sizes) == 1:
        return strides[0] == 1
    if sizes[-2] == 1:
        return strides[-2] == 1 if strict else (strides[-1] == 1 or strides[-2] == 1)
    if sizes[-1] == 1:
        return (strides[-2] == 1 and strides[-1] >= sizes[-2]) if strict else strides[-2] == 1
    return strides[-2] == 1 and strides[-1] >= strides[-2]


def _empty_strided(size, stride, dtype, device, pin_memory) -> torch.Tensor:
    dev = torch.device(device)
    pin = bool(pin_memory) and dev.type == "cpu" and torch.cuda.is_available()
    return torch.empty_strided(tuple(size), tuple(stride), dtype=dtype, device=dev, pin_memory=pin)


def create_C(size: Tuple[int, ...], dtype, device: Union[str, torch.device], pin_memory: bool = False) -> torch.Tensor:
    stride, acc = [], 1
    for s in reversed(size):
        stride.append(acc)
        acc *= max(int(s), 1)
    return _empty_strided(size, stride[::-1], dtype, device, pin_memory)


def create_fortran(size: Tuple[int, ...], dtype, device: Union[str, torch.device], pin_memory: bool = False) -> torch.Tensor:
    stride, acc = [], 1
    for s in size:
        stride.append(acc)
        acc *= max(int(s), 1)
    return _empty_strided(size, stride, dtype, device, pin_memory)


def create_same_stride(size, other: torch.Tensor, dtype, device, pin_memory: bool = False) -> torch.Tensor:
    """Allocate in ``other``'s order: F if it is strictly column-major, else C
    (falkon/utils/tensor_helpers.py:128-140)."""
    if is_f_contig(other, strict=True):
        return create_fortran(size, dtype, device, pin_memory)
    if is_contig(other):
        return create_C(size, dtype, device, pin_memory)
    raise ValueError("Desired stride is not contiguous, cannot create.")
