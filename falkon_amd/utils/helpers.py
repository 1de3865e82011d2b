"""Small dtype / device predicates (falkon/utils/helpers.py:225-269)."""
from typing import Optional

import numpy as np
import torch

__all__ = ("sizeof_dtype", "check_same_dtype", "check_same_device")


def sizeof_dtype(dtype) -> int:
    if isinstance(dtype, torch.dtype):
        if dtype == torch.float64:
            return 8
        if dtype == torch.float32:
            return 4
    elif dtype == np.float64:
        return 8
    elif dtype == np.float32:
        return 4
    raise TypeError(f"Dtype {dtype} not valid")


def check_same_dtype(*args: Optional[torch.Tensor]) -> bool:
    dts = {a.dtype for a in args if a is not None}
    return len(dts) <= 1


def check_same_device(*args: Optional[torch.Tensor]) -> bool:
    devs = {a.device for a in args if a is not None}
    return len(devs) <= 1
