"""The oracle's layer and encoder composition against the committed HuggingFace fixture
(tests/golden/bert_tiny_golden.npz, made by tests/golden/make_bert_golden.py in float64):
weight packing, head split, additive mask, softmax, residual+LayerNorm order, tanh GELU.
Runs on CPU.
"""
import os

import numpy as np
import pytest

from helpers import oracle_layer_weights

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "bert_tiny_golden.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLDEN)


def _ext_mask(gold):
    return (-10000.0 * (1 - gold["attention_mask"])).astype(np.float32).reshape(gold["attention_mask"].shape[0], 1, 1, -1)


def test_embedding_matches_huggingface(oracle, gold):
    B, S = gold["input_ids"].shape
    pos = np.tile(np.arange(S), (B, 1))
    got = oracle.bert_embedding(gold["input_ids"], pos, gold["token_type_ids"], gold["w.embeddings.word_embeddings.weight"],
                                gold["w.embeddings.position_embeddings.weight"],
                                gold["w.embeddings.token_type_embeddings.weight"], gold["w.embeddings.LayerNorm.weight"],
                                gold["w.embeddings.LayerNorm.bias"])
    assert np.abs(got - gold["hidden.0"]).max() < 1e-5


def test_attention_probabilities_and_layers_match_huggingface(oracle, gold):
    heads = int(gold["num_heads"])
    x = gold["hidden.0"]
    for i in range(int(gold["num_layers"])):
        out, attn = oracle.bert_layer(x, _ext_mask(gold), oracle_layer_weights(gold, f"w.encoder.layer.{i}."), heads)
        # HF masks with finfo.min instead of -10000; both give exactly 0 on masked keys of valid rows
        assert np.abs(attn - gold[f"attn.{i}"]).max() < 1e-5
        assert np.abs(out - gold[f"hidden.{i + 1}"]).max() < 2e-5
        x = gold[f"hidden.{i + 1}"]


def test_encoder_matches_huggingface(oracle, gold):
    heads, L = int(gold["num_heads"]), int(gold["num_layers"])
    layers = [oracle_layer_weights(gold, f"w.encoder.layer.{i}.") for i in range(L)]
    got = oracle.bert_encoder(gold["hidden.0"], _ext_mask(gold), layers, heads)
    assert np.abs(got - gold["last_hidden_state"]).max() < 3e-5


def test_smart_batch_equals_dense_per_request(oracle, gold):
    """Packed variable-length attention == dense attention run on each request alone."""
    heads = int(gold["num_heads"])
    w = oracle_layer_weights(gold, "w.encoder.layer.0.")
    lens = [16, 11, 5]
    x = gold["hidden.0"]
    packed = np.ascontiguousarray(np.concatenate([x[b, :L] for b, L in enumerate(lens)])[None])
    mask = np.where(np.arange(16)[None, :] < np.array(lens)[:, None], 0.0, -1e9).astype(np.float32).reshape(3, 1, 16)
    out, attn = oracle.smart_layer(packed, mask, w, lens, heads)
    off = 0
    for b, L in enumerate(lens):
        dense, dattn = oracle.bert_layer(np.ascontiguousarray(x[b:b + 1, :L]), None, w, heads)
        assert np.abs(out[0, off:off + L] - dense[0]).max() < 1e-5
        assert np.abs(attn[b, :, :L, :L] - dattn[0]).max() < 1e-6
        assert not attn[b, :, :L, L:].any()  # -1e9 on pad keys -> exactly zero probability
        off += L
