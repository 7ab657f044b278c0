"""The entry point that allocates nothing: ttmi_gemm_bias_layer_norm_static against ttmi_gemm_bias_layer_norm.

Both run the same kernels; the static form keeps the fp32 partial tiles of a product cut along K in a buffer
that is part of the library's device image.  Results must be bit-identical, also when a smaller problem follows a
larger one in the same buffer.
"""
import numpy as np
import pytest
import torch

from turbotransformers_amd import capi
from helpers import TTMI_DTYPES, dev, ok, ptr, stream

pytestmark = pytest.mark.gpu


def _both(ttmi, dt, M, N, K, seed, fp32_residual=False):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    bias, gamma, beta = (dev(rng.standard_normal(N).astype(np.float32), dt) for _ in range(3))
    dA, dW = dev(A, dt), dev(W, dt)
    outs = []
    for fn in (ttmi.ttmi_gemm_bias_layer_norm, ttmi.ttmi_gemm_bias_layer_norm_static):
        out = torch.full((M, N), float("nan"), dtype=dA.dtype, device="cuda")
        if fp32_residual:
            dres, out32 = dev(res), torch.full((M, N), float("nan"), device="cuda")
            ok(fn(ptr(dA), ptr(dW), ptr(out), None, ptr(dres), ptr(bias), ptr(gamma), ptr(beta), ptr(out32), M, N, K, 1e-12,
                  TTMI_DTYPES[dt], stream()))
            outs.append((out, out32))
        else:
            dres = dev(res, dt)
            ok(fn(ptr(dA), ptr(dW), ptr(out), ptr(dres), None, ptr(bias), ptr(gamma), ptr(beta), None, M, N, K, 1e-12,
                  TTMI_DTYPES[dt], stream()))
            outs.append((out,))
    torch.cuda.synchronize()
    for got, want in zip(outs[1], outs[0]):
        assert not torch.isnan(want).any()
        assert torch.equal(got, want)


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_static_scratch_matches_allocating_entry_point_twice_in_a_row(ttmi, dt):
    """Two calls in a row on the same scratch, the second smaller: a split-K shape on the DMA tiles
    (M = 2560: four slices, 31.5 MB of partial tiles), then one short sequence (M = 128, sixteen slices)."""
    _both(ttmi, dt, 2560, 768, 3072, seed=1)
    _both(ttmi, dt, 128, 768, 3072, seed=2)
    _both(ttmi, dt, 100, 768, 768, seed=3)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_static_scratch_fp32_residual_stream(ttmi, dt):
    _both(ttmi, dt, 640, 1024, 4096, seed=4, fp32_residual=True)
    _both(ttmi, dt, 128, 1024, 4096, seed=5, fp32_residual=True)


def test_static_scratch_unsplit_problems_need_no_scratch(ttmi):
    """A problem large enough to run unsplit uses no partial tiles and is accepted at any size."""
    _both(ttmi, "f16", 8192, 768, 768, seed=6)
