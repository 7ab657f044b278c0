"""DistilBERT on the BERT encoder path.

A DistilBERT block is a BERT layer under other parameter names (q_lin / k_lin / v_lin / out_lin +
sa_layer_norm, ffn.lin1 / lin2 + output_layer_norm) and its embeddings have no token types, so the model
maps onto BertAttention + BertIntermediate + BertOutput and the embedding kernel with an all-zero
token-type table.  The reference assembles the same model from MultiHeadedAttention and DistrillFFN
(python/turbo_transformers/layers/modeling_distillbert.py:36-314); `DistrillFFN` itself is in `modules.py`.
GELU is the tanh form of the BERT path (HuggingFace DistilBERT uses erf: up to ~1e-2 apart, the
reference's own tolerance).
"""
from typing import Optional

import torch

from .modeling_bert import BertAttention, BertEmbeddings, BertEncoder, BertIntermediate, BertLayer, BertOutput, _require_gpu
from .return_type import ReturnType, convert_returns_as_type
from .utils import AnyTensor, convert2tt_tensor, to_param_dict, try_convert, use_current_stream, weight_in_out, cxx

__all__ = ['DistilBertModel']


def _block_to_bert_layer(block, n_heads: int) -> BertLayer:
    p = to_param_dict(block)
    with torch.no_grad():
        qkv_w = weight_in_out(torch.cat((p['attention.q_lin.weight'], p['attention.k_lin.weight'], p['attention.v_lin.weight']), 0))
        qkv_b = torch.cat((p['attention.q_lin.bias'], p['attention.k_lin.bias'], p['attention.v_lin.bias']), 0).contiguous()
    t = convert2tt_tensor
    attention = BertAttention(t(qkv_w), t(qkv_b), t(weight_in_out(p['attention.out_lin.weight'])), t(p['attention.out_lin.bias']),
                              t(p['sa_layer_norm.weight']), t(p['sa_layer_norm.bias']), n_heads)
    intermediate = BertIntermediate(t(weight_in_out(p['ffn.lin1.weight'])), t(p['ffn.lin1.bias']))
    output = BertOutput(t(weight_in_out(p['ffn.lin2.weight'])), t(p['ffn.lin2.bias']), t(p['output_layer_norm.weight']),
                        t(p['output_layer_norm.bias']))
    return BertLayer(attention, intermediate, output)


class DistilBertModel:
    """`DistilBertModel.from_torch(hf_distilbert_model, device)`; call with (input_ids, attention_mask) ->
    (last_hidden_state,)."""

    def __init__(self, embeddings: BertEmbeddings, encoder: BertEncoder, config):
        self.embeddings = embeddings
        self.encoder = encoder
        self.config = config
        self.prepare = cxx.PrepareBertMasks()

    def __call__(self, input_ids: AnyTensor, attention_masks: Optional[AnyTensor] = None,
                 return_type: Optional[ReturnType] = None):
        use_current_stream()
        inputs = try_convert(input_ids)
        masks = try_convert(attention_masks) if attention_masks is not None else cxx.Tensor.create_empty()
        token_types, positions, ext = cxx.Tensor.create_empty(), cxx.Tensor.create_empty(), cxx.Tensor.create_empty()
        self.prepare(inputs, masks, token_types, positions, ext)  # zeros, 0..S-1, -10000 * (1 - mask)
        hidden = self.embeddings(inputs, position_ids=positions, token_type_ids=token_types,
                                 return_type=ReturnType.turbo_transformers)
        out = self.encoder(hidden_states=hidden, attention_mask=ext, return_type=ReturnType.turbo_transformers)
        return (convert_returns_as_type(out[0], return_type), )

    @staticmethod
    def from_torch(model, device: Optional[torch.device] = None, backend: Optional[str] = None):
        if backend not in (None, "turbo"):
            raise NotImplementedError("only backend='turbo' exists in this build (no onnxruntime path)")
        device = device if device is not None else model.device
        _require_gpu(device)
        model.to(device)
        e = to_param_dict(model.embeddings)
        word = e['word_embeddings.weight']
        no_types = torch.zeros((1, word.shape[1]), dtype=word.dtype, device=word.device)
        t = convert2tt_tensor
        embeddings = BertEmbeddings(t(word), t(e['position_embeddings.weight']), t(no_types), t(e['LayerNorm.weight']),
                                    t(e['LayerNorm.bias']))
        encoder = BertEncoder([_block_to_bert_layer(b, model.config.n_heads) for b in model.transformer.layer])
        return DistilBertModel(embeddings, encoder, model.config)
