"""Writes tests/golden/bert_tiny_golden.npz: a small random-init HuggingFace BERT (the
third-party `transformers` package, not the reference) evaluated in float64 on seeded inputs.

The reference's own tests use exactly this comparator -- a random-init HuggingFace module
built from a config, converted with from_torch, compared by max-abs
(python/tests/bert_layer_test.py:65-86, bert_model_test.py:58-85) -- but unseeded and with
erf-GELU, which leaves a ~1e-2 gap to the tanh-GELU kernels.  Here hidden_act is
"gelu_pytorch_tanh", dropout is 0 and the run is float64, so the fixture pins the oracle's
composition (weight packing, head split, mask, softmax, residual + LayerNorm order) to ~1e-6.

Run from the repository root:  python tests/golden/make_bert_golden.py
"""
import os

import numpy as np
import torch
from transformers import BertConfig, BertModel

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bert_tiny_golden.npz")


def main():
    torch.manual_seed(20201125)
    cfg = BertConfig(vocab_size=97, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, intermediate_size=256,
                     max_position_embeddings=40, type_vocab_size=2, hidden_act="gelu_pytorch_tanh",
                     hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, layer_norm_eps=1e-12,
                     attn_implementation="eager")
    model = BertModel(cfg).double().eval()
    with torch.no_grad():  # make biases / LayerNorm parameters non-trivial so a dropped term shows
        for name, p in model.named_parameters():
            if name.endswith("bias") or "LayerNorm.weight" in name:
                p.add_(0.1 * torch.randn_like(p))
    B, S = 3, 16
    g = torch.Generator().manual_seed(7)
    ids = torch.randint(0, cfg.vocab_size, (B, S), generator=g)
    types = torch.randint(0, 2, (B, S), generator=g)
    mask = torch.ones(B, S, dtype=torch.int64)
    mask[1, 11:] = 0
    mask[2, 5:] = 0
    with torch.no_grad():
        out = model(input_ids=ids, attention_mask=mask, token_type_ids=types, output_hidden_states=True,
                    output_attentions=True)
    data = {"input_ids": ids.numpy(), "token_type_ids": types.numpy(), "attention_mask": mask.numpy(),
            "num_heads": np.array(cfg.num_attention_heads), "num_layers": np.array(cfg.num_hidden_layers)}
    for name, p in model.named_parameters():
        data["w." + name] = p.detach().numpy().astype(np.float32)
    for i, h in enumerate(out.hidden_states):  # [0] = embedding output, [i] = output of layer i
        data[f"hidden.{i}"] = h.numpy().astype(np.float32)
    for i, a in enumerate(out.attentions):
        data[f"attn.{i}"] = a.numpy().astype(np.float32)
    data["last_hidden_state"] = out.last_hidden_state.numpy().astype(np.float32)
    data["pooler_output"] = out.pooler_output.numpy().astype(np.float32)
    np.savez(OUT, **data)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
