"""Pins the oracle's general MultiHeadedAttention composition (oracle/loader.py, after
layers/multi_headed_attention.cpp:35-380) without a GPU: against torch.nn.MultiheadAttention (an
independent implementation of the same mathematics), against torch LayerNorm for the pre/post forms,
and through the invariant that stepwise decoding with a key/value cache equals causal attention."""
import numpy as np
import pytest
import torch


def _weights(mha, ln=None):
    H = mha.embed_dim
    wq, wk, wv = (w.detach().numpy().T.copy() for w in mha.in_proj_weight.split(H))
    bq, bk, bv = (b.detach().numpy().copy() for b in mha.in_proj_bias.split(H))
    w = {"q_w": wq, "k_w": wk, "v_w": wv, "q_b": bq, "k_b": bk, "v_b": bv,
         "qkv_w": np.concatenate([wq, wk, wv], 1), "qkv_b": np.concatenate([bq, bk, bv]),
         "dense_w": mha.out_proj.weight.detach().numpy().T.copy(), "dense_b": mha.out_proj.bias.detach().numpy().copy()}
    if ln is not None:
        w["ln_g"], w["ln_b"] = ln.weight.detach().numpy().copy(), ln.bias.detach().numpy().copy()
    return w


def _modules(H=64, heads=4, seed=0):
    torch.manual_seed(seed)
    mha = torch.nn.MultiheadAttention(H, heads, batch_first=True).eval()
    with torch.no_grad():
        mha.in_proj_bias.normal_(0, 0.1)
        mha.out_proj.bias.normal_(0, 0.1)
    ln = torch.nn.LayerNorm(H, eps=1e-6)
    with torch.no_grad():
        ln.weight.normal_(1, 0.1)
        ln.bias.normal_(0, 0.1)
    return mha, ln


@pytest.mark.parametrize("attn_type", ["self", "context"])
def test_plain_attention_vs_torch_multihead_attention(oracle, attn_type):
    B, F, T, H, heads = 3, 5, (5 if attn_type == "self" else 9), 64, 4
    mha, ln = _modules(H, heads)
    g = torch.Generator().manual_seed(1)
    q = torch.randn(B, F, H, generator=g)
    mem = q if attn_type == "self" else torch.randn(B, T, H, generator=g)
    pad = torch.zeros(B, T, dtype=torch.bool)
    pad[0, T - 2:] = True
    pad[2, :1] = True
    with torch.no_grad():
        want, want_attn = mha(q, mem, mem, key_padding_mask=pad, need_weights=True, average_attn_weights=False)
    mask = np.where(pad.numpy(), -1e9, 0.0).astype(np.float32).reshape(B, 1, T)
    out, attn = oracle.multi_headed_attention(mem.numpy(), mem.numpy(), q.numpy(), mask, _weights(mha), heads, attn_type)
    assert np.abs(out - want.numpy()).max() < 2e-5
    assert np.abs(attn - want_attn.numpy()).max() < 2e-6


def test_per_query_mask_and_output_forms(oracle):
    B, S, H, heads = 2, 6, 64, 4
    mha, ln = _modules(H, heads, seed=2)
    x = torch.randn(B, S, H, generator=torch.Generator().manual_seed(3))
    causal = torch.triu(torch.full((S, S), float("-inf")), diagonal=1)
    with torch.no_grad():
        core = mha(x, x, x, attn_mask=causal, need_weights=False)[0]                 # includes the output bias
        pre = mha(ln(x), ln(x), ln(x), attn_mask=causal, need_weights=False)[0] + x  # pre-LN + residual
        post = torch.nn.functional.layer_norm(core + x, (H,), ln.weight, ln.bias, 1e-12)
    m = np.broadcast_to(np.triu(np.full((S, S), -1e9, np.float32), 1), (B, S, S)).copy()
    w = _weights(mha, ln)
    xs = x.numpy()
    out = oracle.multi_headed_attention(xs, xs, xs, m, w, heads, "self")[0]
    assert np.abs(out - core.numpy()).max() < 2e-5
    out = oracle.multi_headed_attention(xs, xs, xs, m, w, heads, "self", pre_layernorm=True, post_add_input=True)[0]
    assert np.abs(out - pre.numpy()).max() < 5e-5
    out = oracle.multi_headed_attention(xs, xs, xs, m, w, heads, "self", post_layernorm=True)[0]
    assert np.abs(out - post.numpy()).max() < 5e-5


def test_stepwise_self_cache_equals_causal_attention(oracle):
    B, S, H, heads = 2, 7, 64, 4
    mha, ln = _modules(H, heads, seed=4)
    x = torch.randn(B, S, H, generator=torch.Generator().manual_seed(5)).numpy()
    w = _weights(mha)
    m = np.broadcast_to(np.triu(np.full((S, S), -1e9, np.float32), 1), (B, S, S)).copy()
    full = oracle.multi_headed_attention(x, x, x, m, w, heads, "self")[0]
    cache = {"self_keys": None, "self_values": None}
    for t in range(S):
        step = np.ascontiguousarray(x[:, t:t + 1])
        out, attn = oracle.multi_headed_attention(step, step, step, None, w, heads, "self", cache)
        assert attn.shape == (B, heads, 1, t + 1) and cache["self_keys"].shape == (B, heads, t + 1, H // heads)
        assert np.abs(out - full[:, t:t + 1]).max() < 2e-5


def test_context_memory_cache_is_filled_once_and_reused(oracle):
    B, F, T, H, heads = 2, 3, 8, 64, 4
    mha, ln = _modules(H, heads, seed=6)
    g = torch.Generator().manual_seed(7)
    mem, q1, q2 = (torch.randn(B, n, H, generator=g).numpy() for n in (T, F, F))
    w = _weights(mha)
    cache = {"memory_keys": None, "memory_values": None}
    first = oracle.multi_headed_attention(mem, mem, q1, None, w, heads, "context", cache)[0]
    assert cache["memory_keys"].shape == (B, heads, T, H // heads)
    assert np.array_equal(first, oracle.multi_headed_attention(mem, mem, q1, None, w, heads, "context")[0])
    junk = np.full_like(mem, 3.0)
    second = oracle.multi_headed_attention(junk, junk, q2, None, w, heads, "context", cache)[0]
    assert np.array_equal(second, oracle.multi_headed_attention(mem, mem, q2, None, w, heads, "context")[0])


def test_concat_and_single_projection_split(oracle):
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((2, 3, 4, 5), np.float32), rng.standard_normal((2, 3, 2, 5), np.float32)
    c = oracle.concat(a, b, 2)
    assert c.shape == (2, 3, 6, 5) and np.array_equal(c[:, :, :4], a) and np.array_equal(c[:, :, 4:], b)
    x, bias = rng.standard_normal((2, 7, 3, 4), np.float32), rng.standard_normal(12).astype(np.float32)
    got = oracle.add_bias_transpose_for_score(x, bias, 2, 7, 3, 4)
    assert np.array_equal(got, (x + bias.reshape(3, 4)).transpose(0, 2, 1, 3))


def test_feed_forward_blocks_vs_torch(oracle):
    """PositionwiseFeedForward / DistrillFFN compositions against the same mathematics in torch."""
    torch.manual_seed(9)
    H, F = 48, 160
    lin1, lin2, ln = torch.nn.Linear(H, F), torch.nn.Linear(F, H), torch.nn.LayerNorm(H, eps=1e-12)
    with torch.no_grad():
        ln.weight.normal_(1, 0.1)
        ln.bias.normal_(0, 0.1)
    x = torch.randn(2, 5, H)
    n = lambda t: t.detach().numpy().copy()
    args = (n(x), n(lin1.weight).T.copy(), n(lin1.bias), n(lin2.weight).T.copy(), n(lin2.bias), n(ln.weight), n(ln.bias))
    with torch.no_grad():
        want_pw = x + lin2(torch.relu(lin1(ln(x))))
        want_df = ln(x + lin2(torch.nn.functional.gelu(lin1(x), approximate="tanh")))
    assert np.abs(oracle.positionwise_ffn(*args) - want_pw.numpy()).max() < 2e-5
    assert np.abs(oracle.distill_ffn(*args) - want_df.numpy()).max() < 2e-5
