"""Quantized BERT (reference: python/turbo_transformers/layers/qmodeling_bert.py).

In the reference, QBertIntermediate / QBertOutput wrap `torch.quantization.quantize_dynamic`
Linear modules (bias removed) and follow them with the turbo fused epilogues
(FusedAddBiasGELU / FusedAddBiasLayerNorm); attention stays fp32.  Here the Linear itself is the
int8 MFMA GEMM of this build (`cxx.QuantizedLinear`: per-output-channel int8 weights, one dynamic
activation scale per call, int32 accumulation, fp32 dequant), the same fused epilogues follow, and
`QBertLayer(..., quantize_attention=True)` (the default) also runs the QKV and output projections in
int8, so that every nn.Linear of the layer is quantized.  Models must be fp32.
"""
from typing import Optional

import torch

from .. import cxx
from .modeling_bert import BertAttention, BertEmbeddings, BertPooler, PoolingMap, PoolingType, SequencePool, _require_gpu
from .return_type import ReturnType, convert_returns_as_type
from .utils import convert2tt_tensor, create_empty_if_none, to_param_dict, try_convert, use_current_stream, weight_in_out

__all__ = ['QBertIntermediate', 'QBertOutput', 'QBertAttention', 'QBertLayer', 'QBertEncoder', 'QBertModel']


class QBertIntermediate:
    def __init__(self, intermediate):
        p = to_param_dict(intermediate)
        # Linear and the reference's FusedAddBiasGELU step (qmodeling_bert.py:17-28) in one kernel
        self.linear = cxx.QuantizedLinear(convert2tt_tensor(weight_in_out(p['dense.weight'])),
                                          convert2tt_tensor(p['dense.bias']), "gelu")

    def __call__(self, input_tensor, return_type: Optional[ReturnType] = None):
        use_current_stream()
        out = cxx.Tensor.create_empty()
        self.linear(try_convert(input_tensor), out)
        return convert_returns_as_type(out, return_type)

    @staticmethod
    def from_torch(intermediate):
        return QBertIntermediate(intermediate)


class QBertOutput:
    def __init__(self, bert_output):
        p = to_param_dict(bert_output)
        self.linear = cxx.QuantizedLinear(convert2tt_tensor(weight_in_out(p['dense.weight'])))
        self.turbo_bias_layernorm = cxx.FusedAddBiasLayerNorm(convert2tt_tensor(p['dense.bias']),
                                                              convert2tt_tensor(p['LayerNorm.weight']),
                                                              convert2tt_tensor(p['LayerNorm.bias']))

    def __call__(self, intermediate_output, attention_output, return_type: Optional[ReturnType] = None):
        use_current_stream()
        out = cxx.Tensor.create_empty()
        self.linear(try_convert(intermediate_output), out)
        self.turbo_bias_layernorm(try_convert(attention_output), out)
        return convert_returns_as_type(out, return_type)

    @staticmethod
    def from_torch(bert_output):
        return QBertOutput(bert_output)


class QBertAttention(cxx.QuantizedBertAttention):
    def __call__(self, input_tensor, attention_mask=None, output_attentions=False,
                 return_type: Optional[ReturnType] = None):
        use_current_stream()
        context_layer = cxx.Tensor.create_empty()
        attn_probs = cxx.Tensor.create_empty() if output_attentions else None
        super().__call__(try_convert(input_tensor), try_convert(create_empty_if_none(attention_mask)), context_layer,
                         attn_probs)
        out = (convert_returns_as_type(context_layer, return_type), )
        if output_attentions:
            out = out + (convert_returns_as_type(attn_probs, ReturnType.turbo_transformers), )
        return out

    @staticmethod
    def from_torch(attention):
        p = to_param_dict(attention)
        qkv_weight, qkv_bias, output_weight = BertAttention.pack_qkv(attention)
        return QBertAttention(convert2tt_tensor(qkv_weight), convert2tt_tensor(qkv_bias), convert2tt_tensor(output_weight),
                              convert2tt_tensor(p['output.dense.bias']), convert2tt_tensor(p['output.LayerNorm.weight']),
                              convert2tt_tensor(p['output.LayerNorm.bias']), attention.self.num_attention_heads)


class QBertLayer:
    def __init__(self, bert_layer, quantize_attention: bool = True):
        self.attention = (QBertAttention if quantize_attention else BertAttention).from_torch(bert_layer.attention)
        self.intermediate = QBertIntermediate.from_torch(bert_layer.intermediate)
        self.output = QBertOutput.from_torch(bert_layer.output)

    def __call__(self, hidden_states, attention_mask=None, head_mask=None, output_attentions=False,
                 return_type: Optional[ReturnType] = None):
        attn_out = self.attention(hidden_states, attention_mask, output_attentions=output_attentions,
                                  return_type=ReturnType.turbo_transformers)
        attention_output = attn_out[0]
        intermediate_output = self.intermediate(attention_output, return_type=ReturnType.turbo_transformers)
        layer_output = self.output(intermediate_output, attention_output, return_type=return_type)
        return (layer_output, ) + attn_out[1:]

    @staticmethod
    def from_torch(bert_layer, quantize_attention: bool = True):
        return QBertLayer(bert_layer, quantize_attention)


class QBertEncoder:
    def __init__(self, layers):
        self.layer = layers

    def __call__(self, hidden_states, attention_mask=None, head_mask=None, output_attentions=False,
                 output_hidden_states=False, return_type: Optional[ReturnType] = None):
        all_hidden_states, all_attentions = (), ()
        hidden_states = try_convert(hidden_states)
        attention_mask = try_convert(attention_mask)
        for layer in self.layer:
            if output_hidden_states:
                all_hidden_states = all_hidden_states + (hidden_states, )
            layer_outputs = layer(hidden_states, attention_mask, output_attentions=output_attentions,
                                  return_type=ReturnType.turbo_transformers)
            hidden_states = layer_outputs[0]
            if output_attentions:
                all_attentions = all_attentions + (layer_outputs[1], )
        outputs = (convert_returns_as_type(hidden_states, return_type), )
        if output_hidden_states:
            outputs = outputs + (all_hidden_states, )
        if output_attentions:
            outputs = outputs + (all_attentions, )
        return outputs

    @staticmethod
    def from_torch(encoder, quantize_attention: bool = True):
        return QBertEncoder([QBertLayer.from_torch(l, quantize_attention) for l in encoder.layer])


class QBertModel:
    def __init__(self, model, backend='turbo', quantize_attention: bool = True):
        if backend != 'turbo':
            raise NotImplementedError("only backend='turbo' exists in this build (no onnxruntime path)")
        _require_gpu(model.device)
        if next(model.parameters()).dtype != torch.float32:
            raise ValueError("QBertModel quantizes an fp32 model")
        self.backend = 'turbo'
        self.config = model.config
        self.embeddings = BertEmbeddings.from_torch(model.embeddings)
        self.encoder = QBertEncoder.from_torch(model.encoder, quantize_attention)
        self.pooler = BertPooler.from_torch(model.pooler)
        self.prepare = cxx.PrepareBertMasks()

    def __call__(self, inputs, attention_masks=None, token_type_ids=None, position_ids=None, head_mask=None,
                 inputs_embeds=None, output_attentions=None, output_hidden_states=None,
                 pooling_type: PoolingType = PoolingType.FIRST, return_type: Optional[ReturnType] = None):
        use_current_stream()
        attention_masks = try_convert(create_empty_if_none(attention_masks))
        token_type_ids = try_convert(create_empty_if_none(token_type_ids))
        position_ids = try_convert(create_empty_if_none(position_ids))
        inputs = try_convert(inputs)
        ext = cxx.Tensor.create_empty()
        self.prepare(inputs, attention_masks, token_type_ids, position_ids, ext)
        hidden = self.embeddings(inputs, position_ids=position_ids, token_type_ids=token_type_ids,
                                 return_type=ReturnType.turbo_transformers)
        enc = self.encoder(hidden, ext, output_attentions=output_attentions, output_hidden_states=output_hidden_states,
                           return_type=ReturnType.turbo_transformers)
        sequence_output = enc[0]
        pooled = SequencePool(PoolingMap[pooling_type])(input_tensor=sequence_output,
                                                        return_type=ReturnType.turbo_transformers)
        pooler_output = self.pooler(pooled, return_type)
        return (convert_returns_as_type(sequence_output, return_type), pooler_output) + enc[1:]

    @staticmethod
    def from_torch(model, backend='turbo', quantize_attention: bool = True):
        return QBertModel(model, backend, quantize_attention)
