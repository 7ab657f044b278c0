"""Output conversion of the layer wrappers (reference: python/turbo_transformers/layers/return_type.py:27-45)."""
import enum
from typing import Optional

import torch.utils.dlpack as dlpack

from .. import cxx

__all__ = ['ReturnType', 'convert_returns_as_type']


class ReturnType(enum.Enum):
    turbo_transformers = 0
    TORCH = 1
    NUMPY = 2


def convert_returns_as_type(tensor, rtype: Optional[ReturnType]):
    """cxx.Tensor -> cxx.Tensor | torch.Tensor | numpy.  TORCH hands the buffer over through
    DLPack without a copy: the cxx.Tensor is empty afterwards and torch owns the memory; nothing waits for the
    device, so an error a kernel reported (an embedding id out of range, whose row is NaN in the result) is raised
    by the next `cxx.synchronize()`.  NUMPY copies to the host, which waits for the device anyway, and raises
    such an error itself."""
    if rtype is None:
        rtype = ReturnType.TORCH
    if rtype == ReturnType.turbo_transformers:
        return tensor
    if rtype == ReturnType.TORCH:
        return dlpack.from_dlpack(tensor.to_dlpack())
    if rtype == ReturnType.NUMPY:
        t = dlpack.from_dlpack(tensor.to_dlpack())
        host = t.float().cpu().numpy()
        cxx.synchronize()
        return host
    raise NotImplementedError()
