"""GPU parity of the MFMA GEMM family (MatMul, BatchMatMul, fused epilogues, int8) against the
CPU oracle, through the C ABI.

Inputs are scaled so outputs are O(1); fp32 must agree to 1e-4 (accumulation order only),
fp16 to 4e-3 and bf16 to 3e-2 max-abs (one storage rounding of an O(1..4) value); int8
accumulators are compared bit-exactly against an integer brute force.
"""
import numpy as np
import pytest
import torch

from helpers import ALL_DTYPES, TORCH_DTYPES, TTMI_DTYPES, dev, host, max_abs, ok, ptr, rounded, stream
from turbotransformers_amd import capi

pytestmark = pytest.mark.gpu

GEMM_TOL = {"f32": 1e-4, "f16": 4e-3, "bf16": 3e-2}


def _ab(rng, M, N, K, b_trans):
    A = rng.standard_normal((M, K), np.float32)
    B = (rng.standard_normal((N, K) if b_trans else (K, N), np.float32) / np.sqrt(K)).astype(np.float32)
    return A, B


def test_matmul_known_answer(ttmi):
    # layers/kernels/mat_mul_test.cpp:29-40: [1,2;3,4] x [2,3;4,5] = [10,13;22,29]
    A, B = np.array([[1, 2], [3, 4]], np.float32), np.array([[2, 3], [4, 5]], np.float32)
    for dt in ALL_DTYPES:
        C = torch.zeros((2, 2), dtype=dev(A, dt).dtype, device="cuda")
        ok(ttmi.ttmi_gemm(ptr(dev(A, dt)), ptr(dev(B, dt)), ptr(C), 2, 2, 2, 2, 2, 2, 0, 1.0, 0.0, TTMI_DTYPES[dt], stream()))
        assert np.array_equal(host(C), np.array([[10, 13], [22, 29]], np.float32))
        ok(ttmi.ttmi_gemm(ptr(dev(A, dt)), ptr(dev(np.ascontiguousarray(B.T), dt)), ptr(C), 2, 2, 2, 2, 2, 2, 1, 1.0, 0.0,
                          TTMI_DTYPES[dt], stream()))
        assert np.array_equal(host(C), np.array([[10, 13], [22, 29]], np.float32))


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("b_trans", [0, 1])
@pytest.mark.parametrize("M,N,K", [
    (5, 768, 768), (20, 3072, 768), (20, 768, 3072), (128, 2304, 768), (300, 256, 64), (257, 129, 72),
    (33, 65, 50), (1, 8, 8), (2048, 2304, 768), (8192, 2304, 768), (4100, 1024, 1024), (500, 500, 500)])
def test_matmul(ttmi, oracle, dt, b_trans, M, N, K):
    rng = np.random.default_rng(M + N + K + b_trans)
    A, B = _ab(rng, M, N, K, b_trans)
    dA, dB = dev(A, dt), dev(B, dt)
    C = torch.full((M, N), 3.0, dtype=dA.dtype, device="cuda")
    ok(ttmi.ttmi_gemm(ptr(dA), ptr(dB), ptr(C), M, N, K, K, K if b_trans else N, N, b_trans, 1.0, 0.0,
                      TTMI_DTYPES[dt], stream()))
    want = oracle.matmul(rounded(A, dt), rounded(B, dt), bool(b_trans))
    assert max_abs(host(C), want) <= GEMM_TOL[dt]


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("M,N,K", [(128, 768, 3072), (128, 768, 768), (1, 768, 3072), (100, 2304, 768), (200, 3072, 1024),
                                   (64, 520, 4096), (2560, 768, 3072), (2048, 768, 3072), (1000, 1024, 4096)])
def test_matmul_small_m_long_k(ttmi, oracle, dt, M, N, K):
    """Few output tiles, long K: the split-K path (K slices summed in a fixed order by a second kernel).
    Same bound as any other MatMul, and two runs give the same bits."""
    rng = np.random.default_rng(M + N + K)
    A, B = _ab(rng, M, N, K, 1)
    dA, dB = dev(A, dt), dev(B, dt)
    C1 = torch.empty((M, N), dtype=dA.dtype, device="cuda")
    C2 = torch.empty_like(C1)
    for C in (C1, C2):
        ok(ttmi.ttmi_gemm(ptr(dA), ptr(dB), ptr(C), M, N, K, K, K, N, 1, 1.0, 0.0, TTMI_DTYPES[dt], stream()))
    want = oracle.matmul(rounded(A, dt), rounded(B, dt), True)
    assert max_abs(host(C1), want) <= GEMM_TOL[dt] * max(1.0, float(np.abs(want).max()))
    assert torch.equal(C1, C2)


@pytest.mark.parametrize("dt", ALL_DTYPES)
def test_fused_epilogues_small_m_long_k(ttmi, oracle, dt):
    """bias + GELU and bias + residual through the split-K reduction kernel."""
    import ctypes
    rng = np.random.default_rng(5)
    M, N, K = 96, 768, 3072
    A, W = _ab(rng, M, N, K, 1)
    bias, res = rng.standard_normal(N).astype(np.float32), rng.standard_normal((M, N)).astype(np.float32)
    dA, dW, db, dres = dev(A, dt), dev(W, dt), dev(bias, dt), dev(res, dt)
    base = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    C = torch.empty((M, N), dtype=dA.dtype, device="cuda")
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_BIAS_ACT,
                            ctypes.byref(_epi(bias=db, act=capi.ACT_GELU)), TTMI_DTYPES[dt], stream()))
    assert max_abs(host(C), oracle.add_bias_act(base, rounded(bias, dt), 0)) <= GEMM_TOL[dt] * 3
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_BIAS_RESIDUAL,
                            ctypes.byref(_epi(bias=db, residual=dres)), TTMI_DTYPES[dt], stream()))
    assert max_abs(host(C), base + rounded(bias, dt) + rounded(res, dt)) <= GEMM_TOL[dt] * 3


@pytest.fixture(params=["3 A stages", "2 A stages"])
def large_tile_forced(request, ttmi):
    """Switch TTMI_LARGE_TILE = 1 sends every eligible problem to the one-wavefront-per-SIMD kernel whatever its
    size (set through the C ABI: the library reads its environment variables only once).  Both forms of its K loop:
    three LDS stages for the A operand where they fit (192-wide tiles, row-major outputs), and two everywhere."""
    ok(ttmi.ttmi_set_kernel_switch(b"TTMI_LARGE_TILE", 1))
    if request.param == "2 A stages":
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_W4_A_STAGES", 2))
    yield
    ok(ttmi.ttmi_set_kernel_switch(b"TTMI_LARGE_TILE", -1))
    ok(ttmi.ttmi_set_kernel_switch(b"TTMI_W4_A_STAGES", -1))


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K", [(256, 192, 128), (1, 8, 128), (300, 200, 256), (777, 776, 384), (2560, 768, 768),
                                   (515, 3072, 256), (4100, 1000, 128), (64, 2304, 768)])
def test_large_tile_kernel_against_oracle_and_small_tiles(ttmi, oracle, large_tile_forced, dt, M, N, K):
    """The 256 x 192 tile kernel (four wavefronts, accumulators in AGPRs) on whole, ragged and tiny problems: plain
    product, bias, bias + GELU.  Bound as for any MatMul against the oracle; against the 8-wavefront kernels the
    plain and the bias form may differ by the last bit of the output type and no more (the 16x16x32 matrix instruction
    sums the 32 products of a step in another order than the 32x32x16 one: fp32 rounding of the accumulator)."""
    import ctypes
    rng = np.random.default_rng(M + N + K)
    A, W = _ab(rng, M, N, K, 1)
    bias = rng.standard_normal(N).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    base = oracle.matmul(rounded(A, dt), rounded(W, dt), True)

    def run(epilogue):
        C = torch.full((M, N), float("nan"), dtype=dA.dtype, device="cuda")
        if epilogue is None:
            ok(ttmi.ttmi_gemm(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, 1, 1.0, 0.0, TTMI_DTYPES[dt], stream()))
        elif epilogue == "bias":
            ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_BIAS, ctypes.byref(_epi(bias=db)),
                                    TTMI_DTYPES[dt], stream()))
        else:
            ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_BIAS_ACT,
                                    ctypes.byref(_epi(bias=db, act=capi.ACT_GELU)), TTMI_DTYPES[dt], stream()))
        torch.cuda.synchronize()
        return C

    got = {e: run(e) for e in (None, "bias", "gelu")}
    assert max_abs(host(got[None]), base) <= GEMM_TOL[dt]
    assert max_abs(host(got["bias"]), base + rounded(bias, dt)) <= GEMM_TOL[dt] * 3
    assert max_abs(host(got["gelu"]), oracle.add_bias_act(base, rounded(bias, dt), 0)) <= GEMM_TOL[dt] * 3
    if (M, N, K) != (64, 2304, 768):  # that one is cut along K by the other path: another summation order
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_LARGE_TILE", 0))
        ulp = 2.0 ** -10 if dt == "f16" else 2.0 ** -7  # one step of the output type, relative to the larger neighbour
        for form in (None, "bias"):
            a, b = host(run(form)), host(got[form])
            assert np.all(np.abs(a - b) <= ulp * np.maximum(np.abs(a), np.abs(b)) + 1e-6)
            assert np.mean(a != b) < 0.05  # and the two mostly agree exactly


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("M", [1, 300, 777, 4100])
def test_large_tile_kernel_leaves_rows_past_m_alone(ttmi, oracle, large_tile_forced, dt, M):
    """The last tile row of the 256-row tiles is ragged for every one of these M.  C lives inside a larger tensor
    with 256 sentinel rows behind row M (and 8 in front of row 0): the kernel's row-major stores, plain, bias and
    bias + GELU, must leave every sentinel as it was, and rows 0..M-1 must still be the product."""
    import ctypes
    N, K, GUARD = 776, 256, 256
    rng = np.random.default_rng(M)
    A, W = _ab(rng, M, N, K, 1)
    bias = rng.standard_normal(N).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    base = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = {"plain": base, "bias": base + rounded(bias, dt), "gelu": oracle.add_bias_act(base, rounded(bias, dt), 0)}
    SENTINEL = -7.0
    for form in ("plain", "bias", "gelu"):
        whole = torch.full((8 + M + GUARD, N), SENTINEL, dtype=dA.dtype, device="cuda")
        C = whole[8:8 + M]
        if form == "plain":
            ok(ttmi.ttmi_gemm(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, 1, 1.0, 0.0, TTMI_DTYPES[dt], stream()))
        else:
            epi = _epi(bias=db) if form == "bias" else _epi(bias=db, act=capi.ACT_GELU)
            ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N,
                                    capi.EPI_BIAS if form == "bias" else capi.EPI_BIAS_ACT, ctypes.byref(epi),
                                    TTMI_DTYPES[dt], stream()))
        torch.cuda.synchronize()
        assert torch.all(whole[:8] == SENTINEL), form
        assert torch.all(whole[8 + M:] == SENTINEL), "%s: rows past M were written" % form
        assert max_abs(host(C), want[form]) <= GEMM_TOL[dt] * 3


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("v_transposed", [False, True])
@pytest.mark.parametrize("B,S,h,d", [(2, 40, 12, 64), (16, 128, 12, 64), (3, 100, 6, 64), (2, 300, 16, 64), (64, 32, 12, 64),
                                     (20, 512, 16, 64), (7, 75, 12, 64), (6, 100, 12, 64)])
def test_large_tile_kernel_qkv_split(ttmi, oracle, large_tile_forced, dt, B, S, h, d, v_transposed):
    """The same kernel behind the QKV projection: bias + head split, V row-major or transposed (those tiles run with
    the matrix operands unswapped and leave through the strip column-wise).  Sequence lengths that are and are not
    multiples of 8 and of 32 (eight rows of one V^T store, the 32 rows of a staged group, may straddle two sequences;
    a group of eight positions inside a sequence of a length off the 8-grid is one element-aligned 16-byte store),
    hidden sizes whose V third does and does not start on a multiple of the tile width (then the tile in front of it
    is cut short and a new run of tiles starts there)."""
    import ctypes
    rng = np.random.default_rng(S + h)
    H = h * d
    A, W = _ab(rng, B * S, 3 * H, H, 1)
    bias = rng.standard_normal(3 * H).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    q, k, v = (torch.full((B, h, S, d), float("nan"), dtype=dA.dtype, device="cuda") for _ in range(3))
    pitch = (S + 7) // 8 * 8 + 8 if v_transposed else 0
    if v_transposed:
        v = torch.full((B, h, d, pitch), 7.0, dtype=dA.dtype, device="cuda")
    args = _epi(bias=db, q=q, k=k, v=v, seq=S, heads=h, head_dim=d, v_seq_pitch=pitch)
    name = ctypes.create_string_buffer(64)
    ok(ttmi.ttmi_gemm_describe(B * S, 3 * H, H, capi.EPI_QKV_SPLIT, ctypes.byref(args), TTMI_DTYPES[dt], name, 64))
    assert name.value.decode().startswith("dma_agpr4w")
    if (B, S, h) == (20, 512, 16):  # 40 x 12 tiles of 256 x 256 beat 40 x 17 of 256 x 192: the widest tile's head split
        assert name.value.decode() == "dma_agpr4w_256x256"
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), None, B * S, 3 * H, H, H, H, 3 * H, capi.EPI_QKV_SPLIT,
                            ctypes.byref(args), TTMI_DTYPES[dt], stream()))
    qkv = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = oracle.split_add_bias_transpose(qkv, rounded(bias, dt), B, S, h, d)
    got_v = host(v)
    if v_transposed:
        assert np.all(got_v[..., S:] == 7.0)
        got_v = got_v[..., :S].transpose(0, 1, 3, 2)
    for got, w in zip((host(q), host(k), got_v), want):
        assert max_abs(got, w) <= GEMM_TOL[dt] * 2


LN_TOL = {"f32": 1e-4, "f16": 4e-3, "bf16": 3e-2}  # relative to 1 + |expected|; large shapes round the product to 16 bits first


def _ln_close(got, want, dt):
    return bool(np.all(np.abs(got - want) <= LN_TOL[dt] * (1.0 + np.abs(want))))


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("M,N,K", [(128, 768, 768), (128, 768, 3072), (1, 768, 3072), (2560, 768, 3072), (300, 1024, 4096),
                                   (40, 2052, 1024), (64, 4096, 1024), (64, 520, 256), (4096, 768, 768), (50, 770, 768)])
def test_gemm_bias_layer_norm(ttmi, oracle, dt, M, N, K):
    """Dense projection + AddBiasLayerNorm as one call: shapes that take the split-K kernels (normalised by
    the kernel that sums the slices), and shapes that run the two kernels one after the other."""
    rng = np.random.default_rng(M + N + K)
    A, W = _ab(rng, M, N, K, 1)
    res = rng.standard_normal((M, N)).astype(np.float32)
    bias, gamma, beta = (rng.standard_normal(N).astype(np.float32) for _ in range(3))
    dA, dW, dres = dev(A, dt), dev(W, dt), dev(res, dt)
    out = torch.empty((M, N), dtype=dA.dtype, device="cuda")
    out2 = torch.empty_like(out)
    for o in (out, out2):
        ok(ttmi.ttmi_gemm_bias_layer_norm(ptr(dA), ptr(dW), ptr(o), ptr(dres), None, ptr(dev(bias, dt)), ptr(dev(gamma, dt)),
                                          ptr(dev(beta, dt)), None, M, N, K, 1e-12, TTMI_DTYPES[dt], stream()))
    base = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = oracle.add_bias_layer_norm(base, rounded(res, dt), rounded(bias, dt), rounded(gamma, dt), rounded(beta, dt))
    assert _ln_close(host(out), want, dt)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K", [(128, 768, 3072), (2560, 1024, 4096), (4096, 768, 768)])
def test_gemm_bias_layer_norm_fp32_residual(ttmi, oracle, dt, M, N, K):
    """The same with the residual stream in fp32: the 16-bit output is the rounding of the fp32 one, and
    writing the fp32 result over the residual buffer is allowed."""
    rng = np.random.default_rng(M + N + K + 1)
    A, W = _ab(rng, M, N, K, 1)
    res = rng.standard_normal((M, N)).astype(np.float32)
    bias, gamma, beta = (rng.standard_normal(N).astype(np.float32) for _ in range(3))
    dA, dW, dres = dev(A, dt), dev(W, dt), dev(res)
    out = torch.empty((M, N), dtype=dA.dtype, device="cuda")
    out32 = torch.empty((M, N), device="cuda")
    args = (ptr(dev(bias, dt)), ptr(dev(gamma, dt)), ptr(dev(beta, dt)))
    ok(ttmi.ttmi_gemm_bias_layer_norm(ptr(dA), ptr(dW), ptr(out), None, ptr(dres), *args, ptr(out32), M, N, K, 1e-12,
                                      TTMI_DTYPES[dt], stream()))
    base = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = oracle.add_bias_layer_norm(base, res, rounded(bias, dt), rounded(gamma, dt), rounded(beta, dt))
    assert _ln_close(host(out32), want, dt)
    assert np.array_equal(host(out), rounded(host(out32), dt))
    # with its own fp32 output buffer nothing is rounded between the accumulators and the normalisation, on the
    # K-sliced path and on the large-problem path alike: the fp32 result is as close to the oracle as an fp32 run
    assert _ln_close(host(out32), want, "f32")
    first = out32.clone()
    ok(ttmi.ttmi_gemm_bias_layer_norm(ptr(dA), ptr(dW), ptr(out), None, ptr(dres), *args, ptr(dres), M, N, K, 1e-12,
                                      TTMI_DTYPES[dt], stream()))
    if M <= 128:
        assert torch.equal(dres, first)  # K-sliced: the same kernels either way
    else:
        # a large problem writing over its residual has nowhere to keep an fp32 product: it passes through `out`
        # in the 16-bit type, one more rounding
        assert _ln_close(host(dres), want, dt)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,slices,fp32_residual", [(6275, 768, 3072, -1, False), (6275, 768, 3072, -1, True),
                                                        (700, 384, 768, 3, False), (1, 8, 512, 2, False),
                                                        (1300, 1000, 1024, 4, True), (520, 200, 256, 2, False)])
def test_gemm_bias_layer_norm_k_slices_on_the_large_tile_kernel(ttmi, oracle, dt, M, N, K, slices, fp32_residual):
    """The projection in front of a LayerNorm cut along K on the one-wavefront-per-SIMD kernel: (slice, tile) work
    items, fp32 partial products, summed and normalised by the reduction kernel.  Once where the library chooses that
    path by itself (the second FFN product of a 6275-token batch: 100 tiles for 256 CUs), and forced onto small and
    ragged shapes with 2, 3 and 4 slices (switch TTMI_W4_SPLITK).  Against the oracle, and against the same call with
    the path switched off: both sum fp32 partial sums of the same products, in another order."""
    rng = np.random.default_rng(M + N + K)
    A, W = _ab(rng, M, N, K, 1)
    res = rng.standard_normal((M, N)).astype(np.float32)
    bias, gamma, beta = (rng.standard_normal(N).astype(np.float32) for _ in range(3))
    dA, dW = dev(A, dt), dev(W, dt)
    dres = dev(res) if fp32_residual else dev(res, dt)
    args = (ptr(dev(bias, dt)), ptr(dev(gamma, dt)), ptr(dev(beta, dt)))
    outs = {}
    try:
        for name, value in (("sliced", slices), ("unsliced", 0)):
            ok(ttmi.ttmi_set_kernel_switch(b"TTMI_W4_SPLITK", value))
            out = torch.full((M + 8, N), -7.0, dtype=dA.dtype, device="cuda")
            out32 = torch.full((M + 8, N), -7.0, device="cuda") if fp32_residual else None
            ok(ttmi.ttmi_gemm_bias_layer_norm(ptr(dA), ptr(dW), ptr(out), None if fp32_residual else ptr(dres),
                                              ptr(dres) if fp32_residual else None, *args,
                                              ptr(out32) if fp32_residual else None, M, N, K, 1e-12, TTMI_DTYPES[dt], stream()))
            torch.cuda.synchronize()
            assert torch.all(out[M:] == -7.0), "rows past M were written"
            outs[name] = (out[:M], out32[:M] if fp32_residual else None)
    finally:
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_W4_SPLITK", -1))
    base = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = oracle.add_bias_layer_norm(base, res if fp32_residual else rounded(res, dt), rounded(bias, dt), rounded(gamma, dt),
                                      rounded(beta, dt))
    got, got32 = outs["sliced"]
    assert _ln_close(host(got), want, dt)
    if fp32_residual:
        assert _ln_close(host(got32), want, "f32")  # nothing rounded between the accumulators and the normalisation
        assert np.array_equal(host(got), rounded(host(got32), dt))
        assert max_abs(host(got32), host(outs["unsliced"][1])) < 1e-3
    else:
        assert _ln_close(host(got), host(outs["unsliced"][0]).astype(np.float32), dt)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("forced", [False, True])
@pytest.mark.parametrize("M,N,K,with_bias", [(300, 200, 256, True), (4100, 1024, 1024, False), (2560, 768, 3072, True),
                                             (8192, 768, 768, True), (777, 776, 384, False), (128, 768, 3072, True)])
def test_gemm_with_fp32_output(ttmi, oracle, dt, forced, M, N, K, with_bias):
    """TTMI_EPI_F32_OUT: 16-bit operands, the accumulators (plus an optional bias) stored as fp32.  Tile kernels of
    every family (small tiles, K slices, the 8-wavefront DMA tiles, the one-wavefront-per-SIMD kernel with whole and
    ragged tiles, also forced onto small shapes): the result is the fp32 product of the rounded operands, to fp32
    accumulation error, and rows past M stay untouched."""
    import ctypes
    rng = np.random.default_rng(M + N + K)
    A, W = _ab(rng, M, N, K, 1)
    bias = rng.standard_normal(N).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    whole = torch.full((M + 64, N), -7.0, device="cuda")
    C = whole[:M]
    if forced:
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_LARGE_TILE", 1))
    try:
        ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_F32_OUT,
                                ctypes.byref(_epi(bias=db) if with_bias else _epi()), TTMI_DTYPES[dt], stream()))
    finally:
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_LARGE_TILE", -1))
    want = oracle.matmul(rounded(A, dt), rounded(W, dt), True) + (rounded(bias, dt) if with_bias else 0.0)
    assert max_abs(host(C), want) <= GEMM_TOL["f32"] * max(1.0, float(np.abs(want).max()))
    assert torch.all(whole[M:] == -7.0)


def test_gemm_bias_layer_norm_rejects_bad_arguments(ttmi):
    x = torch.zeros((8, 8), device="cuda")
    v = torch.zeros(8, device="cuda")
    # no residual at all; fp32 residual without its output
    assert ttmi.ttmi_gemm_bias_layer_norm(ptr(x), ptr(x), ptr(x), None, None, ptr(v), ptr(v), ptr(v), None, 8, 8, 8, 1e-12,
                                          TTMI_DTYPES["f32"], stream()) != 0
    assert ttmi.ttmi_gemm_bias_layer_norm(ptr(x), ptr(x), ptr(x), None, ptr(x), ptr(v), ptr(v), ptr(v), None, 8, 8, 8, 1e-12,
                                          TTMI_DTYPES["f32"], stream()) != 0


@pytest.mark.parametrize("dt", ALL_DTYPES)
def test_matmul_alpha_beta_and_ld(ttmi, oracle, dt):
    rng = np.random.default_rng(5)
    M, N, K, lda, ldb, ldc = 70, 90, 64, 80, 72, 96
    A = rng.standard_normal((M, lda), np.float32)
    B = (rng.standard_normal((N, ldb), np.float32) / 8).astype(np.float32)
    C0 = rng.standard_normal((M, ldc), np.float32)
    dC = dev(C0, dt)
    ok(ttmi.ttmi_gemm(ptr(dev(A, dt)), ptr(dev(B, dt)), ptr(dC), M, N, K, lda, ldb, ldc, 1, 0.5, 2.0, TTMI_DTYPES[dt],
                      stream()))
    want = rounded(C0, dt).copy()
    want[:, :N] = 0.5 * (rounded(A, dt)[:, :K].astype(np.float64) @ rounded(B, dt)[:, :K].T.astype(np.float64)) + 2.0 * want[:, :N]
    got = host(dC)
    assert max_abs(got[:, :N], want[:, :N]) <= GEMM_TOL[dt] * 3
    assert np.array_equal(got[:, N:], rounded(C0, dt)[:, N:])  # columns beyond N untouched


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("batch,S,d", [(24, 100, 64), (6, 500, 64), (4, 128, 64), (3, 37, 20)])
def test_batch_matmul_attention_shapes(ttmi, oracle, dt, batch, S, d):
    """batch_gemm3 (Q K^T, alpha = 1/sqrt(d)) and batch_gemm4 (P V) of
    layers/multi_headed_attention.cpp:328-346."""
    rng = np.random.default_rng(S)
    Q, Kt, V = (rng.standard_normal((batch, S, d), np.float32) for _ in range(3))
    alpha = 1.0 / np.sqrt(d)
    dQ, dK, dV = dev(Q, dt), dev(Kt, dt), dev(V, dt)
    score = torch.empty((batch, S, S), dtype=dQ.dtype, device="cuda")
    ok(ttmi.ttmi_gemm_strided_batched(ptr(dQ), ptr(dK), ptr(score), S, S, d, d, d, S, S * d, S * d, S * S, batch, 1,
                                      alpha, 0.0, TTMI_DTYPES[dt], stream()))
    want = oracle.batch_matmul(rounded(Q, dt), rounded(Kt, dt), True, alpha)
    assert max_abs(host(score), want) <= GEMM_TOL[dt] * 4
    P = (rng.random((batch, S, S), np.float32) / S * 2).astype(np.float32)
    dP = dev(P, dt)
    ctx = torch.empty((batch, S, d), dtype=dQ.dtype, device="cuda")
    ok(ttmi.ttmi_gemm_strided_batched(ptr(dP), ptr(dV), ptr(ctx), S, d, S, S, d, d, S * S, S * d, S * d, batch, 0, 1.0,
                                      0.0, TTMI_DTYPES[dt], stream()))
    want = oracle.batch_matmul(rounded(P, dt), rounded(V, dt), False)
    assert max_abs(host(ctx), want) <= GEMM_TOL[dt]


@pytest.mark.parametrize("dt", ALL_DTYPES)
def test_batched_heads_writes_merged_layout(ttmi, oracle, dt):
    """P V with the [B,h,S,d] -> [B,S,h,d] transpose folded into the store."""
    rng = np.random.default_rng(9)
    B, h, S, d = 2, 3, 50, 64
    P = (rng.random((B, h, S, S), np.float32) / S * 2).astype(np.float32)
    V = rng.standard_normal((B, h, S, d), np.float32)
    dP, dV = dev(P, dt), dev(V, dt)
    out = torch.empty((B, S, h, d), dtype=dP.dtype, device="cuda")
    ok(ttmi.ttmi_gemm_batched_heads(ptr(dP), ptr(dV), ptr(out), S, d, S, S, d, h * d, h, h * S * S, S * S, h * S * d,
                                    S * d, S * h * d, d, B, 0, 1.0, 0.0, TTMI_DTYPES[dt], stream()))
    want = oracle.transpose_for_score(oracle.batch_matmul(rounded(P, dt), rounded(V, dt), False))
    assert max_abs(host(out), want) <= GEMM_TOL[dt]


def _epi(**kw):
    a = capi.EpilogueArgs()
    for k, v in kw.items():
        setattr(a, k, v.data_ptr() if isinstance(v, torch.Tensor) else v)
    return a


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("M,N,K", [(100, 3072, 768), (4096, 3072, 768), (77, 768, 3072)])
def test_fused_bias_gelu(ttmi, oracle, dt, M, N, K):
    import ctypes
    rng = np.random.default_rng(M)
    A, W = _ab(rng, M, N, K, 1)
    bias = rng.standard_normal(N).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    C = torch.empty((M, N), dtype=dA.dtype, device="cuda")
    args = _epi(bias=db, act=capi.ACT_GELU)
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_BIAS_ACT, ctypes.byref(args),
                            TTMI_DTYPES[dt], stream()))
    want = oracle.add_bias_act(oracle.matmul(rounded(A, dt), rounded(W, dt), True), rounded(bias, dt), 0)
    assert max_abs(host(C), want) <= GEMM_TOL[dt] * 2


@pytest.mark.parametrize("dt", ALL_DTYPES)
def test_fused_bias_and_bias_residual(ttmi, oracle, dt):
    import ctypes
    rng = np.random.default_rng(11)
    M, N, K = 300, 768, 768
    A, W = _ab(rng, M, N, K, 1)
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N), np.float32)
    dA, dW, db, dres = dev(A, dt), dev(W, dt), dev(bias, dt), dev(res, dt)
    C = torch.empty((M, N), dtype=dA.dtype, device="cuda")
    base = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    args = _epi(bias=db)
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_BIAS, ctypes.byref(args),
                            TTMI_DTYPES[dt], stream()))
    assert max_abs(host(C), base + rounded(bias, dt)) <= GEMM_TOL[dt] * 2
    args = _epi(bias=db, residual=dres)
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), ptr(C), M, N, K, K, K, N, capi.EPI_BIAS_RESIDUAL, ctypes.byref(args),
                            TTMI_DTYPES[dt], stream()))
    assert max_abs(host(C), base + rounded(bias, dt) + rounded(res, dt)) <= GEMM_TOL[dt] * 3


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("v_transposed", [False, True])
@pytest.mark.parametrize("B,S,h,d", [(2, 40, 12, 64), (16, 128, 12, 64), (3, 7, 2, 32), (2, 300, 16, 64), (5, 13, 3, 64),
                                     (20, 100, 12, 64), (6, 60, 12, 64), (4, 27, 2, 64), (300, 5, 12, 64)])  # the last four: lengths off the 8-grid
def test_fused_qkv_split(ttmi, oracle, dt, B, S, h, d, v_transposed):
    """QKV GEMM + SplitAddBiasTransposeForScore; with v_seq_pitch the V third lands transposed,
    [B,h,d,pitch] (pad columns untouched), everything else as before."""
    import ctypes
    rng = np.random.default_rng(S)
    H = h * d
    A, W = _ab(rng, B * S, 3 * H, H, 1)
    bias = rng.standard_normal(3 * H).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    q, k, v = (torch.empty((B, h, S, d), dtype=dA.dtype, device="cuda") for _ in range(3))
    pitch = (S + 7) // 8 * 8 + 8 if v_transposed else 0
    if v_transposed:
        v = torch.full((B, h, d, pitch), 7.0, dtype=dA.dtype, device="cuda")
    args = _epi(bias=db, q=q, k=k, v=v, seq=S, heads=h, head_dim=d, v_seq_pitch=pitch)
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), None, B * S, 3 * H, H, H, H, 3 * H, capi.EPI_QKV_SPLIT,
                            ctypes.byref(args), TTMI_DTYPES[dt], stream()))
    qkv = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = oracle.split_add_bias_transpose(qkv, rounded(bias, dt), B, S, h, d)
    got_v = host(v)
    if v_transposed:
        assert np.all(got_v[..., S:] == 7.0)
        got_v = got_v[..., :S].transpose(0, 1, 3, 2)
    for got, w in zip((host(q), host(k), got_v), want):
        assert max_abs(got, w) <= GEMM_TOL[dt] * 2


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("B,S,h,d", [(2, 11, 4, 64), (3, 128, 12, 64), (2, 5, 3, 20)])
def test_fused_single_projection_to_heads(ttmi, oracle, dt, B, S, h, d):
    """MatMul + AddBiasTransposeForScore of one projection (context attention, multi_headed_attention.cpp:73-88)
    as the one-output case of the QKV epilogue: N = h*d, only q is written."""
    import ctypes
    rng = np.random.default_rng(S * 7)
    H = h * d
    A, W = _ab(rng, B * S, H, H, 1)
    bias = rng.standard_normal(H).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    q = torch.empty((B, h, S, d), dtype=dA.dtype, device="cuda")
    args = _epi(bias=db, q=q, seq=S, heads=h, head_dim=d)
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), None, B * S, H, H, H, H, H, capi.EPI_QKV_SPLIT, ctypes.byref(args),
                            TTMI_DTYPES[dt], stream()))
    proj = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = oracle.add_bias_transpose_for_score(proj, rounded(bias, dt), B, S, h, d)
    assert max_abs(host(q), want) <= GEMM_TOL[dt] * 2


@pytest.mark.parametrize("dt", ALL_DTYPES)
@pytest.mark.parametrize("v_transposed", [False, True])
@pytest.mark.parametrize("lens", [[9, 30, 1, 17], [64, 8, 200, 16, 33]])
def test_fused_qkv_split_pad(ttmi, oracle, dt, lens, v_transposed):
    import ctypes
    rng = np.random.default_rng(21)
    lens = np.array(lens, np.int64)
    h, d = 4, 64
    H, B, maxS, total = h * d, len(lens), int(lens.max()), int(lens.sum())
    A, W = _ab(rng, total, 3 * H, H, 1)
    bias = rng.standard_normal(3 * H).astype(np.float32)
    dA, dW, db = dev(A, dt), dev(W, dt), dev(bias, dt)
    cu = np.zeros(B + 1, np.int32)
    cu[1:] = np.cumsum(lens)
    rows = torch.empty(total, dtype=torch.int32, device="cuda")
    ok(ttmi.ttmi_build_token_rows(ptr(dev(cu)), B, maxS, total, ptr(rows), stream()))
    q, k, v = (torch.zeros((B, h, maxS, d), dtype=dA.dtype, device="cuda") for _ in range(3))
    pitch = (maxS + 7) // 8 * 8 if v_transposed else 0
    if v_transposed:
        v = torch.zeros((B, h, d, pitch), dtype=dA.dtype, device="cuda")
    args = _epi(bias=db, q=q, k=k, v=v, seq=maxS, heads=h, head_dim=d, token_rows=rows, batch=B, v_seq_pitch=pitch)
    ok(ttmi.ttmi_gemm_fused(ptr(dA), ptr(dW), None, total, 3 * H, H, H, H, 3 * H, capi.EPI_QKV_SPLIT_PAD,
                            ctypes.byref(args), TTMI_DTYPES[dt], stream()))
    qkv = oracle.matmul(rounded(A, dt), rounded(W, dt), True)
    want = oracle.split_add_bias_transpose_pad(qkv, rounded(bias, dt), lens, h, d)
    got_v = host(v)
    if v_transposed:
        got_v = got_v[..., :maxS].transpose(0, 1, 3, 2)
    for got, w in zip((host(q), host(k), got_v), want):
        assert max_abs(got, w) <= GEMM_TOL[dt] * 2


@pytest.mark.parametrize("M,N,K", [(20, 768, 768), (2560, 3072, 768), (2560, 768, 3072), (33, 48, 80), (300, 1000, 130)])
def test_gemm_i8_accumulators_bit_exact(ttmi, oracle, M, N, K):
    rng = np.random.default_rng(K)
    A = rng.integers(-127, 128, (M, K)).astype(np.int8)
    B = rng.integers(-127, 128, (N, K)).astype(np.int8)
    C = torch.empty((M, N), dtype=torch.int32, device="cuda")
    ok(ttmi.ttmi_gemm_i8(ptr(dev(A)), ptr(dev(B)), ptr(C), M, N, K, K, K, N, stream()))
    want = A.astype(np.int32) @ B.astype(np.int32).T  # exact integer arithmetic
    assert np.array_equal(host(C), want)
    if M * N * K < 5e7:
        assert np.array_equal(want, oracle.gemm_i8(A, B))


@pytest.mark.parametrize("M,N,K,with_bias", [(2560, 768, 768, False), (2560, 3072, 768, True), (37, 100, 48, True), (300, 1000, 130, False)])
def test_gemm_i8_dequant_equals_unfused(ttmi, oracle, M, N, K, with_bias):
    """The dequantisation folded into the int8 GEMM gives the bits of gemm_i8 + dequant_bias, and those
    are the oracle's scheme: float(acc) * s_x * s_w[n] (+ b[n])."""
    rng = np.random.default_rng(M + N)
    a = rng.integers(-127, 128, (M, K), dtype=np.int8)
    b = rng.integers(-127, 128, (N, K), dtype=np.int8)
    sx = np.array([0.0123, 0.0], np.float32)
    sw = (rng.random(N, np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(N).astype(np.float32) if with_bias else None
    dA, dB, dsx, dsw = dev(a), dev(b), dev(sx), dev(sw)
    dbias = dev(bias) if with_bias else None
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
    two_step, fused = torch.empty((M, N), device="cuda"), torch.empty((M, N), device="cuda")
    ok(ttmi.ttmi_gemm_i8(ptr(dA), ptr(dB), ptr(acc), M, N, K, K, K, N, stream()))
    ok(ttmi.ttmi_dequant_bias(ptr(acc), ptr(dsx), ptr(dsw), ptr(dbias) if with_bias else None, ptr(two_step), M, N, stream()))
    ok(ttmi.ttmi_gemm_i8_dequant(ptr(dA), ptr(dB), ptr(fused), ptr(dsx), ptr(dsw), ptr(dbias) if with_bias else None, -1, M, N,
                                 K, K, K, N, stream()))
    assert np.array_equal(host(fused), host(two_step))
    want = oracle.dequant_bias(oracle.gemm_i8(a, b), sx[0], sw, bias if with_bias else np.zeros(N, np.float32))
    assert max_abs(host(fused), want) <= 1e-5 * max(1.0, float(np.abs(want).max()))
    # with the activation folded in as well: the bits of the stand-alone bias + GELU kernel on the unbiased product
    if with_bias:
        ok(ttmi.ttmi_dequant_bias(ptr(acc), ptr(dsx), ptr(dsw), None, ptr(two_step), M, N, stream()))
        ok(ttmi.ttmi_add_bias_act(ptr(two_step), ptr(dbias), M, N, capi.ACT_GELU, TTMI_DTYPES["f32"], stream()))
        ok(ttmi.ttmi_gemm_i8_dequant(ptr(dA), ptr(dB), ptr(fused), ptr(dsx), ptr(dsw), ptr(dbias), capi.ACT_GELU, M, N, K, K, K,
                                     N, stream()))
        assert max_abs(host(fused), host(two_step)) <= 1e-6 * max(1.0, float(np.abs(want).max()))
        assert max_abs(host(fused), oracle.add_bias_act(want, np.zeros(N, np.float32), 0)) <= 2e-5 * max(1.0, float(np.abs(want).max()))


@pytest.mark.parametrize("B,S,h,d", [(20, 128, 12, 64), (3, 17, 2, 8), (2, 9, 3, 20)])
def test_gemm_i8_dequant_qkv_split_equals_the_two_kernels(ttmi, oracle, B, S, h, d):
    """int8 QKV projection with dequantisation, bias and head split in its store: the bits of
    ttmi_gemm_i8_dequant (no bias) followed by ttmi_split_add_bias_transpose_for_score, and the oracle's values."""
    rng = np.random.default_rng(B + S)
    H = h * d
    M, N, K = B * S, 3 * H, H if H % 16 == 0 else 48
    a = rng.integers(-127, 128, (M, K), dtype=np.int8)
    b = rng.integers(-127, 128, (N, K), dtype=np.int8)
    sx = np.array([0.0123, 0.0], np.float32)
    sw = (rng.random(N, np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(N).astype(np.float32)
    dA, dB, dsx, dsw, dbias = dev(a), dev(b), dev(sx), dev(sw), dev(bias)
    flat = torch.empty((M, N), device="cuda")
    ok(ttmi.ttmi_gemm_i8_dequant(ptr(dA), ptr(dB), ptr(flat), ptr(dsx), ptr(dsw), None, -1, M, N, K, K, K, N, stream()))
    two = [torch.empty((B, h, S, d), device="cuda") for _ in range(3)]
    ok(ttmi.ttmi_split_add_bias_transpose_for_score(ptr(flat), ptr(dbias), ptr(two[0]), ptr(two[1]), ptr(two[2]), B, S, h, d,
                                                    TTMI_DTYPES["f32"], stream()))
    one = [torch.full((B, h, S, d), 7.0, device="cuda") for _ in range(3)]
    ok(ttmi.ttmi_gemm_i8_dequant_qkv_split(ptr(dA), ptr(dB), ptr(dsx), ptr(dsw), ptr(dbias), ptr(one[0]), ptr(one[1]), ptr(one[2]),
                                           M, N, K, K, K, S, h, d, stream()))
    for x, y in zip(one, two):
        assert torch.equal(x, y)
    want = oracle.split_add_bias_transpose(oracle.dequant_bias(oracle.gemm_i8(a, b), sx[0], sw, np.zeros(N, np.float32)), bias,
                                           B, S, h, d)
    for x, y in zip(one, want):
        assert max_abs(host(x), y) <= 1e-5 * max(1.0, float(np.abs(y).max()))


@pytest.mark.parametrize("M,N,K,act", [(2560, 3072, 768, capi.ACT_GELU), (2560, 768, 3072, -1), (200, 384, 256, capi.ACT_GELU),
                                       (777, 100, 64, -1), (40000, 64, 64, -1)])
def test_gemm_i8_dequant_leaves_the_maxima_for_the_next_quantisation(ttmi, M, N, K, act):
    """ttmi_gemm_i8_dequant_absmax: the bits of ttmi_gemm_i8_dequant in c, and, when the launch filled the slots, every
    slot written (they start as NaN here: nothing needs clearing), their maximum exactly max|c|; quantising c from the
    slots gives the bits and the scale of the two-launch quantisation.  A launch with more workgroups than slots
    says so and leaves the slots alone (see the LayerNorm form of this test for a case that does)."""
    import ctypes
    rng = np.random.default_rng(M + N)
    a = rng.integers(-127, 128, (M, K), dtype=np.int8)
    b = rng.integers(-127, 128, (N, K), dtype=np.int8)
    sx, sw = np.array([0.0123, 0.0], np.float32), (rng.random(N, np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(N).astype(np.float32)
    dA, dB, dsx, dsw, dbias = dev(a), dev(b), dev(sx), dev(sw), dev(bias)
    plain, fused = torch.empty((M, N), device="cuda"), torch.empty((M, N), device="cuda")
    slots = torch.full((capi.ABSMAX_SLOTS, ), float("nan"), device="cuda")
    written = ctypes.c_int(-1)
    ok(ttmi.ttmi_gemm_i8_dequant(ptr(dA), ptr(dB), ptr(plain), ptr(dsx), ptr(dsw), ptr(dbias), act, M, N, K, K, K, N, stream()))
    ok(ttmi.ttmi_gemm_i8_dequant_absmax(ptr(dA), ptr(dB), ptr(fused), ptr(dsx), ptr(dsw), ptr(dbias), act, M, N, K, K, K, N,
                                        ptr(slots), ctypes.byref(written), stream()))
    assert torch.equal(fused, plain)
    if written.value == 0:  # (whether a shape's launch fits the slots is the tile picker's business)
        assert torch.isnan(slots).all()
        return
    assert written.value == capi.ABSMAX_SLOTS
    assert not torch.isnan(slots).any() and float(slots.min()) >= 0.0
    assert float(slots.max()) == float(plain.abs().max())
    q1, q2 = (torch.empty((M, N), dtype=torch.int8, device="cuda") for _ in range(2))
    s1, s2 = (torch.full((capi.QUANT_SCALE_FLOATS, ), float("nan"), device="cuda") for _ in range(2))
    ok(ttmi.ttmi_quantize_rows_i8(ptr(plain), ptr(q1), ptr(s1), M, N, stream()))
    ok(ttmi.ttmi_quantize_rows_i8_from_absmax(ptr(plain), ptr(q2), ptr(s2), ptr(slots), M, N, stream()))
    assert torch.equal(q1, q2) and torch.equal(s1[:2], s2[:2])


def test_int8_linear_pipeline(ttmi, oracle):
    """quantize -> int8 GEMM -> dequant+bias, against the oracle's statement of the same scheme."""
    rng = np.random.default_rng(3)
    M, N, K = 200, 384, 256
    x = rng.standard_normal((M, K), np.float32)
    w = (rng.standard_normal((N, K), np.float32) * 0.02).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    qw, sw = oracle.quantize_weight_i8(w)
    qx_want, sx_want = oracle.quantize_tensor_i8(x)
    dq = torch.empty((M, K), dtype=torch.int8, device="cuda")
    scale = torch.full((capi.QUANT_SCALE_FLOATS, ), float("nan"), device="cuda")  # scratch needs no clearing
    ok(ttmi.ttmi_quantize_rows_i8(ptr(dev(x)), ptr(dq), ptr(scale), M, K, stream()))
    assert np.array_equal(host(dq), qx_want)
    assert host(scale)[0] == np.float32(sx_want)
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
    ok(ttmi.ttmi_gemm_i8(ptr(dq), ptr(dev(qw)), ptr(acc), M, N, K, K, K, N, stream()))
    acc_want = oracle.gemm_i8(qx_want, qw)
    assert np.array_equal(host(acc), acc_want)
    out = torch.empty((M, N), device="cuda")
    ok(ttmi.ttmi_dequant_bias(ptr(acc), ptr(scale), ptr(dev(sw)), ptr(dev(bias)), ptr(out), M, N, stream()))
    want = oracle.dequant_bias(acc_want, sx_want, sw, bias)
    assert max_abs(host(out), want) <= 1e-5
    assert max_abs(want, x @ w.T + bias) < 0.05  # and the scheme itself approximates the fp32 Linear


def _v_operand(V, dt, v_transposed, poison=True):
    """-> (device tensor, v_seq_pitch).  The transposed form is [B,h,d,pitch]; its pad columns hold
    NaN so that a kernel that lets them reach the output fails the comparison."""
    if not v_transposed:
        return dev(V, dt), 0
    B, h, S, d = V.shape
    pitch = (S + 7) // 8 * 8
    vt = np.full((B, h, d, pitch), np.nan if poison else 0.0, np.float32)
    vt[..., :S] = V.transpose(0, 1, 3, 2)
    return dev(vt, dt), pitch


@pytest.fixture(params=["auto", "8"])
def attention_waves(request, ttmi):
    """Wavefronts per workgroup of the fused attention kernel: its own choice (eight only for long sequences with a workgroup
    per compute unit, which none of these small shapes has), and eight forced through the switch TTMI_ATTENTION_WAVES."""
    if request.param != "auto":
        ok(ttmi.ttmi_set_kernel_switch(b"TTMI_ATTENTION_WAVES", int(request.param)))
    yield request.param
    ok(ttmi.ttmi_set_kernel_switch(b"TTMI_ATTENTION_WAVES", -1))


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("v_transposed", [False, True])
@pytest.mark.parametrize("B,h,S,masked", [(2, 3, 128, True), (1, 2, 512, False), (3, 2, 100, True), (2, 1, 37, True),
                                         (1, 1, 500, True), (2, 12, 64, False), (1, 2, 1, False), (1, 1, 700, True)])
def test_fused_attention_vs_unfused_oracle(ttmi, oracle, attention_waves, dt, B, h, S, masked, v_transposed):
    """One-kernel softmax(scale QK^T + mask) V against the oracle's four-step chain
    (BatchMatMul, ApplyMaskAndSoftmax, BatchMatMul, TransposeForScore)."""
    rng = np.random.default_rng(S + B)
    d = 64
    Q, K, V = (rng.standard_normal((B, h, S, d), np.float32) for _ in range(3))
    mask = None
    if masked:
        mask = np.zeros((B, 1, 1, S), np.float32)
        mask[0, ..., S // 2 + 1:] = -10000.0
        mask[-1, ..., :S // 3] = -10000.0
    dQ, dK = dev(Q, dt), dev(K, dt)
    dV, pitch = _v_operand(V, dt, v_transposed)
    out = torch.full((B, S, h * d), 9.0, dtype=dQ.dtype, device="cuda")
    ok(ttmi.ttmi_fused_attention(ptr(dQ), ptr(dK), ptr(dV), ptr(dev(mask)) if masked else None, ptr(out), None, B, h, S, d,
                                 pitch, 0.125, TTMI_DTYPES[dt], stream()))
    score = oracle.batch_matmul(rounded(Q, dt), rounded(K, dt), True, 0.125)
    prob = oracle.apply_mask_and_softmax(score, mask, 1.0, True)
    want = oracle.transpose_for_score(oracle.batch_matmul(prob, rounded(V, dt), False)).reshape(B, S, h * d)
    # P is rounded to 16 bits before the second MFMA, as the unfused path stores it
    assert max_abs(host(out), want) <= GEMM_TOL[dt] * 2


@pytest.mark.parametrize("B,h,S,masked", [(2, 3, 128, True), (1, 2, 512, False), (3, 2, 100, True), (2, 1, 37, True),
                                         (1, 1, 500, True), (2, 12, 64, False), (1, 2, 1, False), (1, 1, 700, True),
                                         (3, 2, 260, True), (2, 2, 63, False)])
@pytest.mark.parametrize("v_transposed", [False, True])
def test_fused_attention_fp32_vs_unfused_oracle(ttmi, oracle, attention_waves, B, h, S, masked, v_transposed):
    """The fp32 form of the one-kernel attention (32x32x2 fp32 matrix instructions; V row-major, or transposed with NaN
    in its pad columns) against the oracle's four-step chain, to fp32 accuracy: nothing is rounded to 16 bits on the way."""
    rng = np.random.default_rng(S + 3 * B)
    d = 64
    Q, K, V = (rng.standard_normal((B, h, S, d), np.float32) for _ in range(3))
    mask = None
    if masked:
        mask = np.zeros((B, 1, 1, S), np.float32)
        mask[0, ..., S // 2 + 1:] = -10000.0
        mask[-1, ..., :S // 3] = -10000.0
    dQ, dK = dev(Q, "f32"), dev(K, "f32")
    dV, pitch = _v_operand(V, "f32", v_transposed)
    out = torch.full((B, S, h * d), 9.0, dtype=torch.float32, device="cuda")
    ok(ttmi.ttmi_fused_attention(ptr(dQ), ptr(dK), ptr(dV), ptr(dev(mask)) if masked else None, ptr(out), None, B, h, S, d,
                                 pitch, 0.125, TTMI_DTYPES["f32"], stream()))
    score = oracle.batch_matmul(Q, K, True, 0.125)
    prob = oracle.apply_mask_and_softmax(score, mask, 1.0, True)
    want = oracle.transpose_for_score(oracle.batch_matmul(prob, V, False)).reshape(B, S, h * d)
    assert max_abs(host(out), want) <= 5e-5
    # the form that also leaves the per-workgroup maxima of its output (for the int8 Linear that quantises it next):
    # the same bits, every slot written, their maximum is max|out|
    import ctypes
    out2 = torch.full((B, S, h * d), 9.0, dtype=torch.float32, device="cuda")
    slots = torch.full((capi.ABSMAX_SLOTS, ), float("nan"), device="cuda")
    written = ctypes.c_int(-1)
    ok(ttmi.ttmi_fused_attention_absmax(ptr(dQ), ptr(dK), ptr(dV), ptr(dev(mask)) if masked else None, ptr(out2), None, B, h, S,
                                        d, pitch, 0.125, TTMI_DTYPES["f32"], ptr(slots), ctypes.byref(written), stream()))
    assert torch.equal(out, out2)
    assert written.value == capi.ABSMAX_SLOTS and not torch.isnan(slots).any()
    assert float(slots.max()) == float(out.abs().max())


def test_fused_attention_absmax_reports_no_slots_where_it_leaves_none(ttmi):
    """16-bit types, packed batches and launches with more workgroups than slots: the output as always, 0 slots
    reported, the slots untouched."""
    import ctypes
    d = 64
    for dt, B, h, S, packed in (("f16", 2, 2, 64, False), ("f32", 2, 2, 64, True), ("f32", 90, 12, 32, False)):
        g = torch.Generator(device="cuda").manual_seed(S + B)
        q, k, v = (torch.randn((B, h, S, d), device="cuda", generator=g).to(TORCH_DTYPES[dt]) for _ in range(3))
        cu = torch.arange(0, (B + 1) * S, S, dtype=torch.int32, device="cuda") if packed else None
        outs = []
        for with_slots in (False, True):
            out = torch.zeros((B, S, h * d), dtype=q.dtype, device="cuda")
            slots = torch.full((capi.ABSMAX_SLOTS, ), float("nan"), device="cuda")
            written = ctypes.c_int(-1)
            args = (ptr(q), ptr(k), ptr(v), None, ptr(out), ptr(cu) if packed else None, B, h, S, d, 0, 0.125, TTMI_DTYPES[dt])
            if with_slots:
                ok(ttmi.ttmi_fused_attention_absmax(*args, ptr(slots), ctypes.byref(written), stream()))
                assert written.value == 0 and torch.isnan(slots).all()
            else:
                ok(ttmi.ttmi_fused_attention(*args, stream()))
            outs.append(out)
        assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("v_transposed", [False, True])
@pytest.mark.parametrize("lens", [[70, 5, 129, 33], [300, 5, 257, 256]])
def test_fused_attention_packed_batch(ttmi, oracle, attention_waves, dt, v_transposed, lens):
    """Packed batch: pad rows of q,k,v hold NaN on the device -- the kernel must never let a row
    past a sequence's length reach the output -- and zeros in the oracle's padded chain."""
    rng = np.random.default_rng(17)
    h, d = 2, 64
    B, maxS, total = len(lens), max(lens), sum(lens)
    Q, K, V = (rng.standard_normal((B, h, maxS, d), np.float32) for _ in range(3))
    Qp, Kp, Vp = Q.copy(), K.copy(), V.copy()
    for b, L in enumerate(lens):
        Q[b, :, L:], K[b, :, L:], V[b, :, L:] = 0, 0, 0
        Qp[b, :, L:], Kp[b, :, L:], Vp[b, :, L:] = np.nan, np.nan, np.nan
    cu = np.zeros(B + 1, np.int32)
    cu[1:] = np.cumsum(lens)
    mask = np.where(np.arange(maxS)[None, :] < np.array(lens)[:, None], 0.0, -1e9).astype(np.float32)
    out = torch.full((total, h * d), 9.0, dtype=dev(Q, dt).dtype, device="cuda")
    dV, pitch = _v_operand(Vp, dt, v_transposed)
    ok(ttmi.ttmi_fused_attention(ptr(dev(Qp, dt)), ptr(dev(Kp, dt)), ptr(dV), ptr(dev(mask)), ptr(out), ptr(dev(cu)), B, h,
                                 maxS, d, pitch, 0.125, TTMI_DTYPES[dt], stream()))
    score = oracle.batch_matmul(rounded(Q, dt), rounded(K, dt), True, 0.125)
    prob = oracle.apply_mask_and_softmax(score, mask.reshape(B, 1, 1, maxS), 1.0, True)
    ctx = oracle.batch_matmul(prob, rounded(V, dt), False)
    want = oracle.transpose_for_score_pad(ctx, lens).reshape(total, h * d)
    assert max_abs(host(out), want) <= GEMM_TOL[dt] * 2
