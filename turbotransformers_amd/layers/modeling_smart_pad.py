"""Variable-length ("smart batch") BERT: requests of different lengths are packed into one
[1, sum(len), H] activation with no padding; only the two batched attention GEMMs and the
softmax run on a zero-padded [B, h, max_len, *] view (reference:
python/turbo_transformers/layers/modeling_smart_pad.py).

Differences from the reference, both on purpose: the embeddings run through the fused
lookup kernel on the packed ids instead of one torch call per request, and the key-padding
mask (-1e9 on columns >= len[b], shape [B,1,max_len]) is filled by a device kernel rather
than a Python double loop.
"""
from typing import Optional, Sequence

import torch

from .. import cxx
from .modeling_bert import (BertEmbeddings, BertIntermediate, BertOutput, BertPooler, PoolingMap, PoolingType,
                            SequencePool, _require_gpu)
from .return_type import ReturnType, convert_returns_as_type
from .utils import (AnyTensor, convert2tt_tensor, create_empty_if_none, to_param_dict, try_convert, use_current_stream,
                    weight_in_out)

__all__ = ['MultiHeadedAttentionSmartBatch', 'BertLayerSmartBatch', 'BertEncoderSmartBatch',
           'BertModelNoPoolerSmartBatch', 'BertModelSmartBatch']


def smart_pad_mask(seq_len_list: Sequence[int]):
    mask = cxx.Tensor.create_empty()
    cxx.build_smart_pad_mask([int(x) for x in seq_len_list], mask)
    return mask


_POSITION_IDS_CACHE = {}


def _packed_position_ids(lens, device):
    """[1, sum(lens)] int64: 0..len-1 per request.  Built on the host in one piece and cached on the
    list of lengths (one upload instead of one arange kernel per request)."""
    key = (lens, str(device))
    hit = _POSITION_IDS_CACHE.get(key)
    if hit is None:
        import numpy as np
        if len(_POSITION_IDS_CACHE) >= 64:
            _POSITION_IDS_CACHE.clear()
        host = np.concatenate([np.arange(n, dtype=np.int64) for n in lens]).reshape(1, -1)
        hit = _POSITION_IDS_CACHE[key] = torch.from_numpy(host).to(device)
    return hit


class MultiHeadedAttentionSmartBatch(cxx.MultiHeadedAttentionSmartBatch):
    def __call__(self, key_tensor: AnyTensor, value_tensor: AnyTensor, query_tensor: AnyTensor,
                 query_seq_len_list: Sequence[int], key_seq_len_list: Sequence[int], mask: Optional[AnyTensor] = None,
                 layer_cache: Optional[dict] = None, attn_type: str = None, pre_layernorm: bool = False,
                 post_layernorm: bool = False, post_add_input: bool = False, is_trans_weight: bool = False,
                 return_type: Optional[ReturnType] = None, output: Optional[cxx.Tensor] = None,
                 attn: Optional[cxx.Tensor] = None, need_attn: bool = True):
        """-> (output, attn).  need_attn=False (not in the reference signature) skips materialising
        the padded [B,h,max_len,max_len] probabilities and returns None for them."""
        use_current_stream()
        if layer_cache:
            raise NotImplementedError("layer_cache belongs to the decoder path and is not built")
        query_seq_len_list = [int(x) for x in query_seq_len_list]
        key_seq_len_list = [int(x) for x in key_seq_len_list]
        if mask is None:
            mask = smart_pad_mask(query_seq_len_list if attn_type == "self" else key_seq_len_list)
        output = create_empty_if_none(output)
        attn = create_empty_if_none(attn) if need_attn else None
        super().__call__(try_convert(key_tensor), try_convert(value_tensor), try_convert(query_tensor),
                         try_convert(mask), attn_type, output, attn, {}, query_seq_len_list, key_seq_len_list,
                         pre_layernorm, post_layernorm, post_add_input, is_trans_weight)
        return (convert_returns_as_type(output, return_type),
                convert_returns_as_type(attn, return_type) if need_attn else None)

    @staticmethod
    def from_torch(attention, layer_norm=None, is_trans_weight: bool = False):
        """From a HuggingFace BertAttention; LayerNorm parameters come from `layer_norm` if given,
        else from attention.output.LayerNorm."""
        p = to_param_dict(attention)
        ln = to_param_dict(layer_norm) if layer_norm is not None else {
            'weight': p['output.LayerNorm.weight'], 'bias': p['output.LayerNorm.bias']}
        pack = (lambda w: w.detach().contiguous()) if is_trans_weight else weight_in_out
        with torch.no_grad():
            qkv_weight = pack(torch.cat((p['self.query.weight'], p['self.key.weight'], p['self.value.weight']), 0))
            qkv_bias = torch.cat((p['self.query.bias'], p['self.key.bias'], p['self.value.bias']), 0).contiguous()
            args = [pack(p['self.key.weight']), p['self.key.bias'], pack(p['self.value.weight']), p['self.value.bias'],
                    pack(p['self.query.weight']), p['self.query.bias'], pack(p['output.dense.weight']),
                    p['output.dense.bias'], qkv_weight, qkv_bias, ln['weight'], ln['bias']]
        return MultiHeadedAttentionSmartBatch(*[convert2tt_tensor(a) for a in args],
                                              attention.self.num_attention_heads)


class BertLayerSmartBatch:
    def __init__(self, attention: MultiHeadedAttentionSmartBatch, intermediate: BertIntermediate, output: BertOutput):
        self.attention = attention
        self.intermediate = intermediate
        self.output = output

    def __call__(self, hidden_states: AnyTensor, query_seq_len_list: Sequence[int],
                 attention_mask: Optional[AnyTensor] = None, head_mask: Optional[AnyTensor] = None,
                 output_attentions=False, return_type: Optional[ReturnType] = None):
        attention_output, attn = self.attention(hidden_states, hidden_states, hidden_states, query_seq_len_list,
                                                query_seq_len_list, mask=attention_mask, attn_type="self",
                                                post_layernorm=True, return_type=ReturnType.turbo_transformers,
                                                need_attn=bool(output_attentions))
        intermediate_output = self.intermediate(attention_output, return_type=ReturnType.turbo_transformers)
        layer_output = self.output(intermediate_output, attention_output, return_type=return_type)
        return (layer_output, attn) if output_attentions else (layer_output, )

    @staticmethod
    def from_torch(layer):
        return BertLayerSmartBatch(MultiHeadedAttentionSmartBatch.from_torch(layer.attention),
                                   BertIntermediate.from_torch(layer.intermediate), BertOutput.from_torch(layer.output))


class BertEncoderSmartBatch:
    def __init__(self, layer: Sequence[BertLayerSmartBatch]):
        self.layer = layer

    def __call__(self, hidden_states: AnyTensor, query_seq_len_list: Sequence[int],
                 attention_mask: Optional[AnyTensor] = None, head_mask: Optional[AnyTensor] = None,
                 output_attentions: Optional[bool] = False, output_hidden_states: Optional[bool] = False,
                 return_type: Optional[ReturnType] = None):
        all_hidden_states, all_attentions = (), ()
        hidden_states = try_convert(hidden_states)
        attention_mask = try_convert(attention_mask)
        for layer in self.layer:
            layer_outputs = layer(hidden_states, query_seq_len_list, attention_mask,
                                  output_attentions=output_attentions, return_type=ReturnType.turbo_transformers)
            if output_hidden_states:
                all_hidden_states = all_hidden_states + (hidden_states, )
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
    def from_torch(encoder):
        return BertEncoderSmartBatch([BertLayerSmartBatch.from_torch(layer) for layer in encoder.layer])


class BertModelNoPoolerSmartBatch:
    def __init__(self, embeddings: BertEmbeddings, encoder: BertEncoderSmartBatch):
        self.embeddings = embeddings
        self.encoder = encoder

    def __call__(self, inputs: Sequence[torch.Tensor], query_seq_len_list: Sequence[int],
                 attention_masks: Optional[AnyTensor] = None, token_type_ids: Optional[AnyTensor] = None,
                 position_ids: Optional[AnyTensor] = None, head_mask: Optional[AnyTensor] = None,
                 inputs_embeds: Optional[AnyTensor] = None, output_attentions: Optional[bool] = None,
                 output_hidden_states: Optional[bool] = None, pooling_type: PoolingType = PoolingType.FIRST,
                 return_type: Optional[ReturnType] = None):
        """inputs: one int64 id tensor of shape [1, len_i] (or [len_i]) per request."""
        use_current_stream()
        lens = [int(x) for x in query_seq_len_list]
        assert len(lens) != 0 and len(inputs) == len(lens)
        ids = torch.cat([t.reshape(-1) for t in inputs]).reshape(1, -1)
        assert ids.numel() == sum(lens), "query_seq_len_list does not match the inputs"
        dev = ids.device
        if position_ids is None:  # each request counts its own positions from 0
            position_ids = _packed_position_ids(tuple(lens), dev)
        if token_type_ids is None:
            token_type_ids = torch.zeros_like(ids)
        hidden = self.embeddings(ids, position_ids=position_ids, token_type_ids=token_type_ids,
                                 return_type=ReturnType.turbo_transformers)
        mask = smart_pad_mask(lens) if attention_masks is None else try_convert(attention_masks)
        return self.encoder(hidden_states=hidden, query_seq_len_list=lens, attention_mask=mask,
                            output_attentions=output_attentions, output_hidden_states=output_hidden_states,
                            return_type=return_type)

    @staticmethod
    def from_torch(model, device: Optional[torch.device] = None):
        device = device if device is not None else model.device
        _require_gpu(device)
        model.to(device)
        return BertModelNoPoolerSmartBatch(BertEmbeddings.from_torch(model.embeddings),
                                           BertEncoderSmartBatch.from_torch(model.encoder))


class BertModelSmartBatch:
    def __init__(self, model: BertModelNoPoolerSmartBatch, pooler: BertPooler, config=None):
        self.config = config
        self.bertmodel_nopooler = model
        self.pooler = pooler

    def __call__(self, inputs: Sequence[torch.Tensor], query_seq_len_list: Sequence[int],
                 attention_masks: Optional[AnyTensor] = None, token_type_ids: Optional[AnyTensor] = None,
                 position_ids: Optional[AnyTensor] = None, head_mask: Optional[AnyTensor] = None,
                 inputs_embeds: Optional[AnyTensor] = None, output_attentions: Optional[bool] = None,
                 output_hidden_states: Optional[bool] = None, pooling_type: PoolingType = PoolingType.FIRST,
                 pooler_output: Optional[AnyTensor] = None, return_type: Optional[ReturnType] = None):
        encoder_outputs = self.bertmodel_nopooler(inputs, query_seq_len_list, attention_masks, token_type_ids,
                                                  position_ids, inputs_embeds=inputs_embeds,
                                                  output_attentions=output_attentions,
                                                  output_hidden_states=output_hidden_states, pooling_type=pooling_type,
                                                  return_type=ReturnType.turbo_transformers)
        sequence_output = encoder_outputs[0]  # packed [1, sum(len), H]
        # As in the reference (modeling_smart_pad.py:549-553) the pooler sees the packed tensor,
        # i.e. pools over all requests at once; only sequence_output is meaningful per request.
        pooled = SequencePool(PoolingMap[pooling_type])(input_tensor=sequence_output,
                                                        return_type=ReturnType.turbo_transformers)
        pooler_output = self.pooler(pooled, return_type, pooler_output)
        return (convert_returns_as_type(sequence_output, return_type), pooler_output) + encoder_outputs[1:]

    @staticmethod
    def from_torch(model, device: Optional[torch.device] = None):
        nopooler = BertModelNoPoolerSmartBatch.from_torch(model, device)
        return BertModelSmartBatch(nopooler, BertPooler.from_torch(model.pooler), model.config)
