"""What the kernels' choosers need to know about the GPU, read once from its properties.

The rules that pick shapes, splits and shares estimate the time of the fullest compute unit, so they
need the number of units.  It is asked from the device the first time it is needed and kept; nothing
else in the package writes that number down.
"""
from __future__ import annotations

from typing import Optional

MI355X_COMPUTE_UNITS = 256   # what the rules assume where no GPU is visible (their tests run without one)

_units: Optional[int] = None


def compute_units() -> int:
    """Compute units of the current GPU."""
    global _units
    if _units is None:
        import torch

        if torch.cuda.is_available():
            _units = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
        else:
            return MI355X_COMPUTE_UNITS
    return _units
