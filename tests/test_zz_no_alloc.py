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
    (M = 2560: three slices, 23.6 MB of partial tiles), then one short sequence (M = 128, a few slices of the
    one-wavefront-per-tile kernel)."""
    _both(ttmi, dt, 2560, 768, 3072, seed=1)
    _both(ttmi, dt, 128, 768, 3072, seed=2)
    _both(ttmi, dt, 100, 768, 768, seed=3)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_static_scratch_fp32_residual_stream(ttmi, dt):
    _both(ttmi, dt, 640, 1024, 4096, seed=4, fp32_residual=True)
    _both(ttmi, dt, 128, 1024, 4096, seed=5, fp32_residual=True)


def test_static_scratch_unsplit_problems_need_no_scratch(ttmi):
    """A problem large enough to run unsplit uses no partial tiles and is accepted at any size (with an fp32
    residual stream its fp32 product lives in the caller's own fp32 output buffer)."""
    _both(ttmi, "f16", 8192, 768, 768, seed=6)
    _both(ttmi, "bf16", 8192, 1024, 1024, seed=10, fp32_residual=True)


def test_static_scratch_and_the_two_slices_of_the_large_tile_kernel(ttmi):
    """A product of a few thousand rows that the allocating entry point cuts in two on its large-tile kernel: where the
    two fp32 partial products fit the static buffer (5000 x 768: 30.7 MB) both entry points run the same kernels and
    agree bit for bit; where they do not (6275 x 768: 38.6 MB) the static form is not refused but runs the product
    whole, so the two differ by the rounding of the 16-bit product in front of the LayerNorm and no more."""
    ok(ttmi.ttmi_set_kernel_switch(b"TTMI_W4_SPLITK", 2))  # by itself the library takes two slices from about 5700 rows on
    try:
        _both(ttmi, "f16", 5000, 768, 3072, seed=11)
    finally:
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_W4_SPLITK", -1))
    M, N, K = 6275, 768, 3072
    rng = np.random.default_rng(12)
    dA = dev(rng.standard_normal((M, K)).astype(np.float32), "f16")
    dW = dev((rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32), "f16")
    dres = dev(rng.standard_normal((M, N)).astype(np.float32), "f16")
    bias, gamma, beta = (dev(rng.standard_normal(N).astype(np.float32), "f16") for _ in range(3))
    outs = []
    for fn in (ttmi.ttmi_gemm_bias_layer_norm, ttmi.ttmi_gemm_bias_layer_norm_static):
        out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        ok(fn(ptr(dA), ptr(dW), ptr(out), ptr(dres), None, ptr(bias), ptr(gamma), ptr(beta), None, M, N, K, 1e-12,
              TTMI_DTYPES["f16"], stream()))
        outs.append(out)
    torch.cuda.synchronize()
    assert not torch.isnan(outs[1]).any()
    assert float((outs[0].float() - outs[1].float()).abs().max()) < 2e-2


def test_static_scratch_refuses_what_does_not_fit(ttmi):
    """With the admitted size lowered to 1 MiB the K slices of 2560 x 768 x 3072 (23.6 MB of partial tiles) no longer
    fit: the call is refused with TTMI_EINVAL and a message that names both sizes, nothing is launched and `out`
    keeps its contents; the allocating entry point and a later call with the limit lifted are unaffected."""
    M, N, K = 2560, 768, 3072
    rng = np.random.default_rng(7)
    dA, dW = dev(rng.standard_normal((M, K)).astype(np.float32), "f16"), dev((rng.standard_normal((N, K)) / 55).astype(np.float32), "f16")
    dres = dev(rng.standard_normal((M, N)).astype(np.float32), "f16")
    vec = dev(np.ones(N, np.float32), "f16")
    out = torch.full((M, N), -7.0, dtype=torch.float16, device="cuda")
    ok(ttmi.ttmi_set_kernel_switch(b"TTMI_STATIC_SCRATCH_LIMIT", 1 << 20))
    try:
        rc = ttmi.ttmi_gemm_bias_layer_norm_static(ptr(dA), ptr(dW), ptr(out), ptr(dres), None, ptr(vec), ptr(vec), ptr(vec), None,
                                                   M, N, K, 1e-12, TTMI_DTYPES["f16"], stream())
        assert rc == -1  # TTMI_EINVAL
        msg = ttmi.ttmi_last_error().decode()
        assert "static scratch buffer" in msg and str(1 << 20) in msg
        torch.cuda.synchronize()
        assert torch.all(out == -7.0)
    finally:
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_STATIC_SCRATCH_LIMIT", -1))
    _both(ttmi, "f16", M, N, K, seed=8)


def test_static_scratch_call_under_graph_capture(ttmi):
    """What the entry point is for: a call recorded into a HIP graph (after one eager call, which resolves the
    buffer's address and sets the kernel attributes).  The graph is replayed three times with eager work and
    synchronisations in between and with fresh operands each time; every replay must reproduce the eager result
    of the allocating entry point bit for bit."""
    M, N, K = 128, 768, 3072
    rng = np.random.default_rng(9)
    new = lambda *shape: dev(rng.standard_normal(shape).astype(np.float32), "f16")
    dA, dW, dres = new(M, K), dev((rng.standard_normal((N, K)) / 55).astype(np.float32), "f16"), new(M, N)
    bias, gamma, beta = new(N), new(N), new(N)
    out, want = (torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2))

    def call(fn, dst, s):
        ok(fn(ptr(dA), ptr(dW), ptr(dst), ptr(dres), None, ptr(bias), ptr(gamma), ptr(beta), None, M, N, K, 1e-12,
              TTMI_DTYPES["f16"], s))

    call(ttmi.ttmi_gemm_bias_layer_norm_static, out, stream())  # eager first call
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(ttmi.ttmi_gemm_bias_layer_norm_static, out, stream())  # torch's capture stream is current here
    for turn in range(3):
        dA.copy_(new(M, K))
        dres.copy_(new(M, N))
        out.fill_(float("nan"))
        call(ttmi.ttmi_gemm_bias_layer_norm, want, stream())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert not torch.isnan(want).any()
        assert torch.equal(out, want), "replay %d" % turn
