"""Pins every kernel of the CPU oracle against something independent of it: library routines
(torch / numpy in float64), the reference tests' literal known answers, closed-form special
cases and invariants.  A dropped term, wrong sign, wrong index or transposed operand in the
oracle fails at least one of these.  Runs on CPU.
"""
import numpy as np
import pytest
import torch


def _rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------------------- MatMul -----
def test_matmul_known_answers(oracle):
    # layers/kernels/mat_mul_test.cpp:29-40
    A, B = np.array([[1, 2], [3, 4]], np.float32), np.array([[2, 3], [4, 5]], np.float32)
    assert np.array_equal(oracle.matmul(A, B), [[10, 13], [22, 29]])
    assert np.array_equal(oracle.matmul(A, np.ascontiguousarray(B.T), b_trans=True), [[10, 13], [22, 29]])
    # non-square, so a transposed operand or swapped M/N cannot pass
    A = np.arange(6, dtype=np.float32).reshape(2, 3)
    B = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert np.array_equal(oracle.matmul(A, B), A @ B)


@pytest.mark.parametrize("blas", ["vendor", "builtin"])
@pytest.mark.parametrize("M,N,K,bt", [(5, 7, 3, 0), (5, 7, 3, 1), (64, 300, 129, 0), (33, 65, 300, 1), (128, 768, 768, 0)])
def test_matmul_vs_float64(oracle, blas, M, N, K, bt):
    if blas == "builtin":
        oracle.use_builtin_blas()
    try:
        r = _rng(M + N)
        A = r.standard_normal((M, K), np.float32)
        B = r.standard_normal((N, K) if bt else (K, N), np.float32)
        C0 = r.standard_normal((M, N), np.float32)
        want = 0.5 * (A.astype(np.float64) @ (B.T if bt else B).astype(np.float64)) + 2.0 * C0
        got = oracle.matmul(A, B, bool(bt), alpha=0.5, beta=2.0, C=C0.copy())
        assert np.abs(got - want).max() < 1e-4 * np.sqrt(K)
    finally:
        oracle.load_best_blas()


def test_batch_matmul_vs_einsum(oracle):
    r = _rng(1)
    Q, K = r.standard_normal((2, 3, 11, 8), np.float32), r.standard_normal((2, 3, 11, 8), np.float32)
    want = np.einsum("bhsd,bhtd->bhst", Q.astype(np.float64), K.astype(np.float64)) * 0.25
    assert np.abs(oracle.batch_matmul(Q, K, True, 0.25) - want).max() < 1e-5
    P, V = r.random((2, 3, 11, 11), np.float32), r.standard_normal((2, 3, 11, 8), np.float32)
    want = np.einsum("bhst,bhtd->bhsd", P.astype(np.float64), V.astype(np.float64))
    assert np.abs(oracle.batch_matmul(P, V, False) - want).max() < 1e-5


# ------------------------------------------------------------------------ transposes -----
def test_split_add_bias_transpose_is_numpy_permutation(oracle):
    r = _rng(2)
    B, S, h, d = 2, 5, 3, 4
    x = r.standard_normal((B, S, 3, h, d), np.float32)
    bias = r.standard_normal((3, h, d), np.float32)
    q, k, v = oracle.split_add_bias_transpose(x, bias, B, S, h, d)
    want = (x + bias).transpose(2, 0, 3, 1, 4)  # [3,B,h,S,d]
    assert np.array_equal(q, want[0]) and np.array_equal(k, want[1]) and np.array_equal(v, want[2])


def test_transpose_for_score_is_numpy_permutation(oracle):
    x = _rng(3).standard_normal((2, 3, 5, 4), np.float32)
    assert np.array_equal(oracle.transpose_for_score(x), x.transpose(0, 2, 1, 3))


def test_pad_variants_match_unpadded_on_valid_rows(oracle):
    # layers/kernels/transpose_test.cpp:242-377: pad form == dense form on valid rows, pad rows == 0,
    # and TransposeForScorePad undoes the padding exactly.
    r = _rng(4)
    lens, h, d = [3, 1, 5], 2, 4
    total, maxS = sum(lens), max(lens)
    x = r.standard_normal((total, 3, h, d), np.float32)
    bias = r.standard_normal((3, h, d), np.float32)
    q, k, v = oracle.split_add_bias_transpose_pad(x, bias, lens, h, d)
    off = 0
    for b, L in enumerate(lens):
        dq, dk, dv = oracle.split_add_bias_transpose(np.ascontiguousarray(x[off:off + L]), bias, 1, L, h, d)
        for padded, dense in ((q, dq), (k, dk), (v, dv)):
            assert np.array_equal(padded[b, :, :L], dense[0])
            assert not padded[b, :, L:].any()
        off += L
    packed = oracle.transpose_for_score_pad(q, lens)
    assert packed.shape == (total, h, d)
    assert np.array_equal(packed, (x[:, 0] + bias[0]))


# --------------------------------------------------------------------------- softmax -----
@pytest.mark.parametrize("is_2d", [True, False])
def test_softmax_vs_torch(oracle, is_2d):
    r = _rng(5)
    B, h, F, T = 2, 3, 7, 13
    qk = r.standard_normal((B, h, F, T), np.float32) * 4
    mask = np.where(r.random((B, 1, 1 if is_2d else F, T)) < 0.3, -10000.0, 0.0).astype(np.float32)
    mask[..., 0] = 0
    want = torch.softmax(torch.from_numpy(qk).double() * 0.7 + torch.from_numpy(mask).double(), -1).numpy()
    got = oracle.apply_mask_and_softmax(qk, mask, 0.7, is_2d)
    assert np.abs(got - want).max() < 1e-6
    assert np.allclose(got.sum(-1), 1, atol=1e-6)


def test_softmax_special_cases(oracle):
    # constant row -> 1/N; no mask; a -10000 column -> exactly 0 in fp32 (gap > 104)
    const = np.full((1, 1, 2, 8), 3.25, np.float32)
    assert np.allclose(oracle.apply_mask_and_softmax(const, None), 1 / 8, atol=1e-7)
    mask = np.zeros((1, 1, 1, 8), np.float32)
    mask[..., 5] = -10000
    p = oracle.apply_mask_and_softmax(const, mask)
    assert (p[..., 5] == 0).all() and np.allclose(p[..., :5], 1 / 7, atol=1e-7)
    # 3-D mask is indexed by the query row: mask row f only affects output row f
    m3 = np.zeros((1, 1, 2, 8), np.float32)
    m3[0, 0, 1, 0] = -10000
    p = oracle.apply_mask_and_softmax(const, m3, is_2d=False)
    assert np.allclose(p[0, 0, 0], 1 / 8, atol=1e-7) and p[0, 0, 1, 0] == 0


# ------------------------------------------------------------------------- LayerNorm -----
def test_layer_norm_vs_torch(oracle):
    r = _rng(6)
    x = r.standard_normal((9, 768), np.float32) * 2 + 0.5
    g, b = r.standard_normal(768).astype(np.float32), r.standard_normal(768).astype(np.float32)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (768, ), torch.from_numpy(g).double(),
                                          torch.from_numpy(b).double(), eps=1e-12).numpy()
    assert np.abs(oracle.layer_norm(x, g, b) - want).max() < 2e-5


def test_add_bias_layer_norm_vs_torch_and_invariants(oracle):
    r = _rng(7)
    out, inp = r.standard_normal((5, 100), np.float32), r.standard_normal((5, 100), np.float32)
    bias, g, b = (r.standard_normal(100).astype(np.float32) for _ in range(3))
    t = torch.from_numpy(out).double() + torch.from_numpy(inp).double() + torch.from_numpy(bias).double()
    want = torch.nn.functional.layer_norm(t, (100, ), torch.from_numpy(g).double(), torch.from_numpy(b).double(), 1e-12)
    assert np.abs(oracle.add_bias_layer_norm(out, inp, bias, g, b) - want.numpy()).max() < 2e-5
    # gamma=1, beta=0 -> zero mean, unit variance
    y = oracle.add_bias_layer_norm(out, inp, bias, np.ones(100, np.float32), np.zeros(100, np.float32))
    assert np.abs(y.mean(-1)).max() < 1e-5 and np.abs(y.var(-1) - 1).max() < 1e-4


# ------------------------------------------------------------------------ activation -----
def test_add_bias_gelu_vs_torch_tanh_gelu(oracle):
    r = _rng(8)
    x, bias = r.standard_normal((6, 500), np.float32) * 3, r.standard_normal(500).astype(np.float32)
    want = torch.nn.functional.gelu(torch.from_numpy(x).double() + torch.from_numpy(bias).double(), approximate="tanh")
    assert np.abs(oracle.add_bias_act(x, bias, 0) - want.numpy()).max() < 2e-6
    z = np.zeros(4, np.float32)
    special = oracle.add_bias_act(np.array([[0.0, 30.0, -30.0, 1.0]], np.float32), z, 0)[0]
    assert special[0] == 0 and special[1] == 30 and special[2] == 0 and abs(special[3] - 0.841192) < 1e-5
    assert np.allclose(oracle.add_bias_act(x, bias, 1), np.tanh(x.astype(np.float64) + bias), atol=1e-6)
    assert np.array_equal(oracle.add_bias_act(x, bias, 2), np.maximum(x + bias, 0))


# ------------------------------------------------------------------------- embedding -----
def test_lookup_embedding(oracle):
    r = _rng(9)
    table = r.standard_normal((50, 12), np.float32)
    ids = r.integers(0, 50, (3, 4))
    got = oracle.lookup_embedding(table, ids)
    assert np.array_equal(got, table[ids])                       # gather: bit-exact
    got2 = oracle.lookup_embedding(table, ids, out=got.copy(), add=True)
    assert np.array_equal(got2, table[ids] + table[ids])
    with pytest.raises(IndexError):                               # embedding.cpp:59
        oracle.lookup_embedding(table, np.array([0, 50]))


def test_bert_embedding_vs_torch(oracle):
    r = _rng(10)
    H = 32
    word, pos, typ = r.standard_normal((40, H), np.float32), r.standard_normal((16, H), np.float32), r.standard_normal((2, H), np.float32)
    g, b = r.standard_normal(H).astype(np.float32), r.standard_normal(H).astype(np.float32)
    ids, tt = r.integers(0, 40, (2, 9)), r.integers(0, 2, (2, 9))
    pid = np.tile(np.arange(9), (2, 1))
    e = torch.from_numpy(word[ids] + typ[tt] + pos[pid]).double()
    want = torch.nn.functional.layer_norm(e, (H, ), torch.from_numpy(g).double(), torch.from_numpy(b).double(), 1e-12)
    assert np.abs(oracle.bert_embedding(ids, pid, tt, word, pos, typ, g, b) - want.numpy()).max() < 2e-5


def test_prepare_bert_masks(oracle):
    mask = np.array([[1, 1, 0], [1, 0, 0]], np.int64)
    m, t, p, ext = oracle.prepare_bert_masks(2, 3, att_mask=mask)
    assert np.array_equal(p, [[0, 1, 2], [0, 1, 2]]) and not t.any()
    assert np.array_equal(ext.reshape(2, 3), [[0, 0, -10000], [0, -10000, -10000]])
    m, _, _, ext = oracle.prepare_bert_masks(2, 3)
    assert m.all() and not ext.any()


# ------------------------------------------------------------------------------ int8 -----
def test_int8_scheme(oracle):
    r = _rng(11)
    x = r.standard_normal((7, 40), np.float32)
    q, s = oracle.quantize_tensor_i8(x)
    assert s == np.float32(np.abs(x).max() / np.float32(127)) and np.abs(q).max() == 127
    assert np.array_equal(q, np.clip(np.rint(x / np.float32(s)), -127, 127).astype(np.int8))
    w = r.standard_normal((5, 40), np.float32)
    qw, sw = oracle.quantize_weight_i8(w)
    assert np.allclose(sw, np.abs(w).max(1) / 127)
    acc = oracle.gemm_i8(q, qw)
    assert np.array_equal(acc, q.astype(np.int64) @ qw.astype(np.int64).T)
    y = oracle.dequant_bias(acc, s, sw, np.ones(5, np.float32))
    ref = x @ w.T + 1
    assert np.abs(y - ref).max() < 0.03 * np.abs(ref).max()  # 8-bit rounding of both operands
    zq, zs = oracle.quantize_tensor_i8(np.zeros(4, np.float32))
    assert zs == 1.0 and not zq.any()
