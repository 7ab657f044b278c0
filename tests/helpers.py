"""Shared plumbing of the GPU parity tests: numpy <-> device buffers and tolerances.

torch is used for device memory only; every kernel under test is reached through the
C ABI (ctypes), never through a torch op.
"""
import ctypes

import numpy as np
import torch

from turbotransformers_amd import capi

TORCH_DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
TTMI_DTYPES = {"f32": capi.F32, "f16": capi.F16, "bf16": capi.BF16}
# max-abs tolerance for O(1)-sized outputs: fp32 within 1e-3 of the reference (kernel tests
# use a tighter bound), fp16/bf16 within 2e-2.
TOL = {"f32": 2e-5, "f16": 4e-3, "bf16": 2e-2}
ALL_DTYPES = ["f32", "f16", "bf16"]


def dev(a, dt="f32"):
    """numpy array -> contiguous cuda tensor of storage type dt (floats) or same int type."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.is_floating_point():
        t = t.to(TORCH_DTYPES[dt])
    return t.cuda().contiguous()


def rounded(a, dt):
    """What the device sees: a rounded to dt, back as float32 numpy (the oracle's input)."""
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(TORCH_DTYPES[dt]).float().numpy()


def host(t):
    torch.cuda.synchronize()
    return t.float().cpu().numpy() if t.is_floating_point() else t.cpu().numpy()


_KEEP = []  # tensors whose address was taken; cleared after each test (conftest)


def ptr(t):
    """Device address of t.  The tensor is kept alive until the test ends, so that
    `ptr(dev(x))` written inline cannot hand the kernel memory that torch's caching
    allocator has already given to the next temporary."""
    if t is None:
        return None
    _KEEP.append(t)
    return ctypes.c_void_p(t.data_ptr())


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ok(rc):
    capi.check(rc)


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)))) if np.size(a) else 0.0


def oracle_layer_weights(w, prefix=""):
    """HuggingFace parameter dict (numpy, names as in BertModel.named_parameters) -> the oracle's
    per-layer weights, packed the way BertAttention.from_torch packs them: dense weights
    transposed to [in, out], q/k/v concatenated along the output axis."""
    g = lambda n: np.asarray(w[prefix + n], np.float32)
    return {
        "qkv_w": np.ascontiguousarray(np.concatenate([g("attention.self.query.weight"), g("attention.self.key.weight"),
                                                      g("attention.self.value.weight")], 0).T),
        "qkv_b": np.concatenate([g("attention.self.query.bias"), g("attention.self.key.bias"),
                                 g("attention.self.value.bias")]),
        "attn_out_w": np.ascontiguousarray(g("attention.output.dense.weight").T),
        "attn_out_b": g("attention.output.dense.bias"),
        "attn_ln_g": g("attention.output.LayerNorm.weight"),
        "attn_ln_b": g("attention.output.LayerNorm.bias"),
        "inter_w": np.ascontiguousarray(g("intermediate.dense.weight").T),
        "inter_b": g("intermediate.dense.bias"),
        "out_w": np.ascontiguousarray(g("output.dense.weight").T),
        "out_b": g("output.dense.bias"),
        "out_ln_g": g("output.LayerNorm.weight"),
        "out_ln_b": g("output.LayerNorm.bias"),
    }
