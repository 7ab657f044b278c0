"""Tensor plumbing shared by the layer wrappers (reference: python/turbo_transformers/layers/utils.py:34-62)."""
from typing import Optional, Union

import numpy as np
import torch
import torch.utils.dlpack as dlpack

from .. import cxx

__all__ = ['try_convert', 'convert2tt_tensor', 'to_param_dict_convert_tt', 'to_param_dict', 'create_empty_if_none',
           'AnyTensor', 'use_current_stream']

AnyTensor = Union[cxx.Tensor, torch.Tensor]


def convert2tt_tensor(t: torch.Tensor):
    """Zero-copy alias of a torch tensor; the cxx.Tensor keeps the torch storage alive."""
    if not t.is_contiguous():
        t = t.contiguous()
    return cxx.Tensor.from_dlpack(dlpack.to_dlpack(t.detach()))


def try_convert(t, device: Optional[torch.device] = None):
    if isinstance(t, torch.Tensor):
        return convert2tt_tensor(t)
    if isinstance(t, np.ndarray):
        dev_name = "GPU" if device is not None and "cuda" in device.type else "CPU"
        return cxx.nparray2tensor(t, dev_name)
    return t


def to_param_dict_convert_tt(torch_module: torch.nn.Module):
    return {k: convert2tt_tensor(v) for k, v in torch_module.named_parameters()}


def to_param_dict(torch_module: torch.nn.Module):
    return {k: v for k, v in torch_module.named_parameters()}


def create_empty_if_none(output):
    return output if output is not None else cxx.Tensor.create_empty()


def use_current_stream():
    """Enqueue the kernels of the following calls on torch's current stream, so they are ordered
    after whatever torch has queued on the inputs."""
    cxx.set_stream(torch.cuda.current_stream().cuda_stream)


def weight_in_out(linear_weight: torch.Tensor) -> torch.Tensor:
    """nn.Linear keeps [out, in]; the layer classes take [in, out] (y = x W)."""
    return torch.clone(torch.t(linear_weight.detach()).contiguous())
