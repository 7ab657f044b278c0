"""ALBERT on the same kernels: factorised embeddings (dim E) projected to the hidden size by one
GEMM, then ONE shared layer applied num_hidden_layers times (reference:
python/turbo_transformers/layers/modeling_albert.py).  The projection
`embedding_hidden_mapping_in` runs on the MFMA GEMM with a bias epilogue instead of a torch
Linear, so the whole forward stays on the work stream.
"""
from typing import Optional, Sequence

import torch

from .. import cxx
from .modeling_bert import BertPooler, _require_gpu
from .return_type import ReturnType, convert_returns_as_type
from .utils import (AnyTensor, convert2tt_tensor, create_empty_if_none, to_param_dict, try_convert, use_current_stream,
                    weight_in_out)

__all__ = ['AlbertEmbeddings', 'AlbertAttention', 'AlbertLayer', 'AlbertLayerGroup', 'AlbertTransformer', 'AlbertModel']


class AlbertEmbeddings(cxx.BERTEmbedding):
    def __call__(self, input_ids: AnyTensor, position_ids: AnyTensor, token_type_ids: AnyTensor,
                 return_type: Optional[ReturnType] = None, output: Optional[cxx.Tensor] = None):
        use_current_stream()
        output = create_empty_if_none(output)
        super().__call__(try_convert(input_ids), try_convert(position_ids), try_convert(token_type_ids), output)
        return convert_returns_as_type(output, return_type)

    @staticmethod
    def from_torch(albert_embedding):
        p = {k: convert2tt_tensor(v) for k, v in albert_embedding.named_parameters()}
        return AlbertEmbeddings(p['word_embeddings.weight'], p['position_embeddings.weight'],
                                p['token_type_embeddings.weight'], p['LayerNorm.weight'], p['LayerNorm.bias'])


class AlbertAttention(cxx.BertAttention):
    def __call__(self, input_tensor: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions: Optional[bool] = False,
                 return_type: Optional[ReturnType] = None):
        assert head_mask is None
        use_current_stream()
        context_layer = cxx.Tensor.create_empty()
        attn_probs = cxx.Tensor.create_empty() if output_attentions else None
        super().__call__(try_convert(input_tensor), try_convert(create_empty_if_none(attention_mask)), context_layer,
                         attn_probs, False)
        out = (convert_returns_as_type(context_layer, return_type), )
        if output_attentions:
            out = out + (convert_returns_as_type(attn_probs, ReturnType.turbo_transformers), )
        return out

    @staticmethod
    def from_torch(attention):
        p = to_param_dict(attention)
        with torch.no_grad():
            qkv_weight = weight_in_out(torch.cat((p['query.weight'], p['key.weight'], p['value.weight']), 0))
            qkv_bias = torch.cat((p['query.bias'], p['key.bias'], p['value.bias']), 0).contiguous()
            output_weight = weight_in_out(p['dense.weight'])
        return AlbertAttention(convert2tt_tensor(qkv_weight), convert2tt_tensor(qkv_bias),
                               convert2tt_tensor(output_weight), convert2tt_tensor(p['dense.bias']),
                               convert2tt_tensor(p['LayerNorm.weight']), convert2tt_tensor(p['LayerNorm.bias']),
                               attention.num_attention_heads)


class AlbertLayer(cxx.AlbertLayer):
    def __init__(self, attention: AlbertAttention, ffn, ffn_bias, ffn_output, ffn_output_bias, ln_weight, ln_bias):
        self.attention = attention
        super().__init__(ffn, ffn_bias, ffn_output, ffn_output_bias, ln_weight, ln_bias)

    def __call__(self, hidden_states: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions: Optional[bool] = False,
                 return_type: Optional[ReturnType] = None):
        attention_output = self.attention(hidden_states, attention_mask, output_attentions=output_attentions,
                                          return_type=ReturnType.turbo_transformers)
        use_current_stream()
        hidden_output, output = cxx.Tensor.create_empty(), cxx.Tensor.create_empty()
        super().__call__(attention_output[0], hidden_output, output)
        return (convert_returns_as_type(output, return_type), ) + attention_output[1:]

    @staticmethod
    def from_torch(torch_albert_layer):
        p = to_param_dict(torch_albert_layer)
        return AlbertLayer(AlbertAttention.from_torch(torch_albert_layer.attention),
                           convert2tt_tensor(weight_in_out(p['ffn.weight'])), convert2tt_tensor(p['ffn.bias']),
                           convert2tt_tensor(weight_in_out(p['ffn_output.weight'])),
                           convert2tt_tensor(p['ffn_output.bias']),
                           convert2tt_tensor(p['full_layer_layer_norm.weight']),
                           convert2tt_tensor(p['full_layer_layer_norm.bias']))


class AlbertLayerGroup:
    def __init__(self, layers: Sequence[AlbertLayer]):
        self.albert_layers = layers

    def __call__(self, hidden_states: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions: Optional[bool] = False,
                 output_hidden_states: Optional[bool] = False, return_type: Optional[ReturnType] = None):
        layer_hidden_states, layer_attentions = (), ()
        for layer in self.albert_layers:
            layer_output = layer(hidden_states, attention_mask, output_attentions=output_attentions,
                                 return_type=ReturnType.turbo_transformers)
            hidden_states = layer_output[0]
            if output_attentions:
                layer_attentions = layer_attentions + (layer_output[1], )
            if output_hidden_states:
                layer_hidden_states = layer_hidden_states + (hidden_states, )
        outputs = (convert_returns_as_type(hidden_states, return_type), )
        if output_hidden_states:
            outputs = outputs + (layer_hidden_states, )
        if output_attentions:
            outputs = outputs + (layer_attentions, )
        return outputs

    @staticmethod
    def from_torch(torch_layer_group):
        return AlbertLayerGroup([AlbertLayer.from_torch(l) for l in torch_layer_group.albert_layers])


class AlbertTransformer:
    def __init__(self, mapping_weight, mapping_bias, groups: Sequence[AlbertLayerGroup], config):
        self.mapping = cxx.LinearBias(mapping_weight, mapping_bias)
        self.albert_layer_groups = groups
        self.config = config

    def __call__(self, hidden_states: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions: Optional[bool] = False,
                 output_hidden_states: Optional[bool] = False, return_type: Optional[ReturnType] = None):
        use_current_stream()
        projected = cxx.Tensor.create_empty()
        self.mapping(try_convert(hidden_states), projected)
        hidden_states = projected
        attention_mask = try_convert(attention_mask)
        all_attentions = ()
        all_hidden_states = (hidden_states, ) if output_hidden_states else ()
        n_layers, n_groups = self.config.num_hidden_layers, self.config.num_hidden_groups
        for i in range(n_layers):
            group = self.albert_layer_groups[int(i / (n_layers / n_groups))]
            out = group(hidden_states, attention_mask, output_attentions=output_attentions,
                        output_hidden_states=output_hidden_states, return_type=ReturnType.turbo_transformers)
            hidden_states = out[0]
            if output_attentions:
                all_attentions = all_attentions + out[-1]
            if output_hidden_states:
                all_hidden_states = all_hidden_states + (hidden_states, )
        outputs = (convert_returns_as_type(hidden_states, return_type), )
        if output_hidden_states:
            outputs = outputs + (all_hidden_states, )
        if output_attentions:
            outputs = outputs + (all_attentions, )
        return outputs

    @staticmethod
    def from_torch(torch_transformer, config):
        p = to_param_dict(torch_transformer.embedding_hidden_mapping_in)
        groups = [AlbertLayerGroup.from_torch(g) for g in torch_transformer.albert_layer_groups]
        return AlbertTransformer(convert2tt_tensor(weight_in_out(p['weight'])), convert2tt_tensor(p['bias']), groups,
                                 config)


class AlbertModel:
    def __init__(self, embeddings: AlbertEmbeddings, encoder: AlbertTransformer, pooler: BertPooler, config):
        self.embeddings = embeddings
        self.encoder = encoder
        self.pooler = pooler
        self.config = config
        self.prepare = cxx.PrepareBertMasks()

    def __call__(self, input_ids: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 token_type_ids: Optional[AnyTensor] = None, position_ids: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions: Optional[bool] = False,
                 output_hidden_states: Optional[bool] = False, return_type: Optional[ReturnType] = None):
        use_current_stream()
        attention_mask = try_convert(create_empty_if_none(attention_mask))
        token_type_ids = try_convert(create_empty_if_none(token_type_ids))
        position_ids = try_convert(create_empty_if_none(position_ids))
        input_ids = try_convert(input_ids)
        ext_mask = cxx.Tensor.create_empty()
        self.prepare(input_ids, attention_mask, token_type_ids, position_ids, ext_mask)
        emb = self.embeddings(input_ids, position_ids=position_ids, token_type_ids=token_type_ids,
                              return_type=ReturnType.turbo_transformers)
        encoder_outputs = self.encoder(emb, ext_mask, output_attentions=output_attentions,
                                       output_hidden_states=output_hidden_states,
                                       return_type=ReturnType.turbo_transformers)
        sequence_output = encoder_outputs[0]
        first = cxx.Tensor.create_empty()
        cxx.SequencePool("First")(sequence_output, first)
        pooled = self.pooler(first, return_type)
        return (convert_returns_as_type(sequence_output, return_type), pooled) + encoder_outputs[1:]

    @staticmethod
    def from_torch(torch_model, device: Optional[torch.device] = None):
        device = device if device is not None else torch_model.device
        _require_gpu(device)
        torch_model.to(device)
        p = to_param_dict(torch_model.pooler)
        pooler = BertPooler(convert2tt_tensor(weight_in_out(p['weight'])), convert2tt_tensor(p['bias']))
        return AlbertModel(AlbertEmbeddings.from_torch(torch_model.embeddings),
                           AlbertTransformer.from_torch(torch_model.encoder, torch_model.config), pooler,
                           torch_model.config)
