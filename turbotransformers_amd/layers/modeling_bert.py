"""BERT wrappers over the C++ layer objects, with the reference's class names, constructors
(`from_torch`, `from_npz`) and call signatures (python/turbo_transformers/layers/modeling_bert.py).

Weight layout (modeling_bert.py:179-204 of the reference): every dense weight is stored
[in, out]; Q/K/V are fused as qkv_weight = cat(Wq, Wk, Wv).T -> [H, 3H] with bias cat(bq, bk, bv).
The element type follows the torch module (fp32, or fp16/bf16 after `.half()` / `.bfloat16()`).
"""
import enum
from typing import Optional, Sequence

import numpy as np
import torch

from .. import cxx
from .return_type import ReturnType, convert_returns_as_type
from .utils import (AnyTensor, convert2tt_tensor, create_empty_if_none, to_param_dict, to_param_dict_convert_tt,
                    try_convert, use_current_stream, weight_in_out)

__all__ = ['BertEmbeddings', 'BertIntermediate', 'BertOutput', 'BertAttention', 'BertLayer', 'BertEncoder',
           'SequencePool', 'BertModel', 'PoolingType', 'BertPooler', 'BertModelNoPooler']


def _npz(file_name):
    return np.load(file_name)


class BertEmbeddings(cxx.BERTEmbedding):
    def __call__(self, input_ids: AnyTensor, position_ids: AnyTensor, token_type_ids: AnyTensor,
                 return_type: Optional[ReturnType] = None, output: Optional[cxx.Tensor] = None):
        use_current_stream()
        output = create_empty_if_none(output)
        super().__call__(try_convert(input_ids), try_convert(position_ids), try_convert(token_type_ids), output)
        return convert_returns_as_type(output, return_type)

    @staticmethod
    def from_torch(bert_embedding) -> 'BertEmbeddings':
        p = to_param_dict_convert_tt(bert_embedding)
        return BertEmbeddings(p['word_embeddings.weight'], p['position_embeddings.weight'],
                              p['token_type_embeddings.weight'], p['LayerNorm.weight'], p['LayerNorm.bias'])

    @staticmethod
    def from_npz(file_name: str, device: Optional[torch.device] = None):
        f = _npz(file_name)
        return BertEmbeddings(*(try_convert(f[f'embeddings.{k}'], device) for k in (
            'word_embeddings.weight', 'position_embeddings.weight', 'token_type_embeddings.weight',
            'LayerNorm.weight', 'LayerNorm.bias')))


class BertIntermediate(cxx.BertIntermediate):
    def __call__(self, input_tensor: AnyTensor, return_type: Optional[ReturnType] = None,
                 output: Optional[cxx.Tensor] = None):
        use_current_stream()
        output = create_empty_if_none(output)
        super().__call__(try_convert(input_tensor), output)
        return convert_returns_as_type(output, return_type)

    @staticmethod
    def from_torch(intermediate):
        p = to_param_dict(intermediate)
        return BertIntermediate(convert2tt_tensor(weight_in_out(p['dense.weight'])), convert2tt_tensor(p['dense.bias']))

    @staticmethod
    def from_npz(file_name: str, layer_num: int, device: Optional[torch.device] = None):
        f = _npz(file_name)
        pre = f'encoder.layer.{layer_num}.intermediate.dense.'
        return BertIntermediate(try_convert(f[pre + 'weight'], device), try_convert(f[pre + 'bias'], device))


class BertOutput(cxx.BertOutput):
    def __call__(self, intermediate_output: AnyTensor, attention_output: AnyTensor,
                 return_type: Optional[ReturnType] = None, output: Optional[cxx.Tensor] = None):
        use_current_stream()
        output = create_empty_if_none(output)
        super().__call__(try_convert(intermediate_output), try_convert(attention_output), output)
        return convert_returns_as_type(output, return_type)

    @staticmethod
    def from_torch(output):
        p = to_param_dict(output)
        return BertOutput(convert2tt_tensor(weight_in_out(p['dense.weight'])), convert2tt_tensor(p['dense.bias']),
                          convert2tt_tensor(p['LayerNorm.weight']), convert2tt_tensor(p['LayerNorm.bias']))

    @staticmethod
    def from_npz(file_name: str, layer_num: int, device: Optional[torch.device] = None):
        f = _npz(file_name)
        pre = f'encoder.layer.{layer_num}.output.'
        return BertOutput(*(try_convert(f[pre + k], device) for k in (
            'dense.weight', 'dense.bias', 'LayerNorm.weight', 'LayerNorm.bias')))


class BertAttention(cxx.BertAttention):
    def __call__(self, input_tensor: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions: Optional[bool] = False,
                 return_type: Optional[ReturnType] = None, is_trans_weight: Optional[bool] = False):
        """-> (context_layer,) or (context_layer, attention_probs)."""
        assert head_mask is None
        use_current_stream()
        context_layer = cxx.Tensor.create_empty()
        # the probabilities [B,h,S,S] are only materialised as an output when asked for
        attn_probs = cxx.Tensor.create_empty() if output_attentions else None
        super().__call__(try_convert(input_tensor), try_convert(create_empty_if_none(attention_mask)), context_layer,
                         attn_probs, bool(is_trans_weight))
        out = (convert_returns_as_type(context_layer, return_type), )
        if output_attentions:
            out = out + (convert_returns_as_type(attn_probs, ReturnType.turbo_transformers), )
        return out

    @staticmethod
    def pack_qkv(attention):
        """(qkv_weight [H,3H], qkv_bias [3H], output_weight [H,H]) from a HuggingFace BertAttention."""
        p = to_param_dict(attention)
        with torch.no_grad():
            qkv_weight = weight_in_out(torch.cat((p['self.query.weight'], p['self.key.weight'], p['self.value.weight']), 0))
            qkv_bias = torch.cat((p['self.query.bias'], p['self.key.bias'], p['self.value.bias']), 0).contiguous()
            output_weight = weight_in_out(p['output.dense.weight'])
        return qkv_weight, qkv_bias, output_weight

    @staticmethod
    def from_torch(attention):
        p = to_param_dict(attention)
        qkv_weight, qkv_bias, output_weight = BertAttention.pack_qkv(attention)
        return BertAttention(convert2tt_tensor(qkv_weight), convert2tt_tensor(qkv_bias), convert2tt_tensor(output_weight),
                             convert2tt_tensor(p['output.dense.bias']), convert2tt_tensor(p['output.LayerNorm.weight']),
                             convert2tt_tensor(p['output.LayerNorm.bias']), attention.self.num_attention_heads)

    @staticmethod
    def from_npz(file_name: str, layer_num: int, num_attention_heads: int, device: Optional[torch.device] = None):
        f = _npz(file_name)
        pre = f'encoder.layer.{layer_num}.attention.'
        return BertAttention(*(try_convert(f[pre + k], device) for k in (
            'qkv.weight', 'qkv.bias', 'output.dense.weight', 'output.dense.bias', 'output.LayerNorm.weight',
            'output.LayerNorm.bias')), num_attention_heads)


class BertLayer:
    def __init__(self, attention: BertAttention, intermediate: BertIntermediate, output: BertOutput):
        self.attention = attention
        self.intermediate = intermediate
        self.output = output

    def __call__(self, hidden_states: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions=False,
                 return_type: Optional[ReturnType] = None):
        attn_out = self.attention(hidden_states, attention_mask, head_mask, output_attentions=output_attentions,
                                  return_type=ReturnType.turbo_transformers)
        attention_output = attn_out[0]
        intermediate_output = self.intermediate(attention_output, return_type=ReturnType.turbo_transformers)
        layer_output = self.output(intermediate_output, attention_output, return_type=return_type)
        return (layer_output, ) + attn_out[1:]

    @staticmethod
    def from_torch(layer):
        return BertLayer(BertAttention.from_torch(layer.attention), BertIntermediate.from_torch(layer.intermediate),
                         BertOutput.from_torch(layer.output))

    @staticmethod
    def from_npz(file_name: str, layer_num: int, num_attention_heads: int, device: Optional[torch.device] = None):
        return BertLayer(BertAttention.from_npz(file_name, layer_num, num_attention_heads, device),
                         BertIntermediate.from_npz(file_name, layer_num, device),
                         BertOutput.from_npz(file_name, layer_num, device))


class BertEncoder:
    def __init__(self, layer: Sequence[BertLayer]):
        self.layer = layer

    def __call__(self, hidden_states: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, output_attentions: Optional[bool] = False,
                 output_hidden_states: Optional[bool] = False, return_type: Optional[ReturnType] = None):
        all_hidden_states, all_attentions = (), ()
        hidden_states = try_convert(hidden_states)
        attention_mask = try_convert(attention_mask)
        if not output_attentions and not output_hidden_states and self._plain_layers():
            # nothing but the last hidden state is asked for: the layer loop runs inside the extension
            use_current_stream()
            last = cxx.Tensor.create_empty()
            cxx.run_bert_layers([(l.attention, l.intermediate, l.output) for l in self.layer], hidden_states,
                                create_empty_if_none(attention_mask), last)
            return (convert_returns_as_type(last, return_type), )
        for layer in self.layer:
            layer_outputs = layer(hidden_states=hidden_states, attention_mask=attention_mask,
                                  output_attentions=output_attentions, return_type=ReturnType.turbo_transformers)
            if output_hidden_states:
                all_hidden_states = all_hidden_states + (hidden_states, )
            hidden_states = layer_outputs[0]
            if output_attentions:
                all_attentions = all_attentions + (layer_outputs[1], )
        # as in the reference, the last hidden state is outputs[0] and is not repeated in all_hidden_states
        outputs = (convert_returns_as_type(hidden_states, return_type), )
        if output_hidden_states:
            outputs = outputs + (all_hidden_states, )
        if output_attentions:
            outputs = outputs + (all_attentions, )
        return outputs

    def _plain_layers(self):
        """Whether every layer is a BertLayer built from the three stock sub-layers (then the C++ loop may run them)."""
        return len(self.layer) > 0 and all(
            type(l) is BertLayer and type(l.attention) is BertAttention and type(l.intermediate) is BertIntermediate
            and type(l.output) is BertOutput for l in self.layer)

    @staticmethod
    def from_torch(encoder):
        return BertEncoder([BertLayer.from_torch(layer) for layer in encoder.layer])

    @staticmethod
    def from_npz(file_name: str, num_hidden_layers: int, num_attention_heads: int,
                 device: Optional[torch.device] = None):
        return BertEncoder([BertLayer.from_npz(file_name, i, num_attention_heads, device)
                            for i in range(num_hidden_layers)])


class SequencePool(cxx.SequencePool):
    def __call__(self, input_tensor: AnyTensor, return_type: Optional[ReturnType] = None,
                 output_tensor: Optional[cxx.Tensor] = None):
        use_current_stream()
        output_tensor = create_empty_if_none(output_tensor)
        super().__call__(try_convert(input_tensor), output_tensor)
        return convert_returns_as_type(output_tensor, return_type)


class PoolingType(enum.Enum):
    FIRST = "First"
    LAST = "Last"
    MEAN = "Mean"
    MAX = "Max"


PoolingMap = {t: t.value for t in PoolingType}


class BertPooler(cxx.BertPooler):
    def __call__(self, input_tensor: AnyTensor, return_type: Optional[ReturnType] = None,
                 output: Optional[cxx.Tensor] = None):
        use_current_stream()
        output = create_empty_if_none(output)
        super().__call__(try_convert(input_tensor), output)
        return convert_returns_as_type(output, return_type)

    @staticmethod
    def from_torch(pooler):
        p = to_param_dict(pooler)
        return BertPooler(convert2tt_tensor(weight_in_out(p['dense.weight'])), convert2tt_tensor(p['dense.bias']))

    @staticmethod
    def from_npz(file_name: str, device: Optional[torch.device] = None):
        f = _npz(file_name)
        return BertPooler(try_convert(f['pooler.dense.weight'], device), try_convert(f['pooler.dense.bias'], device))


def _require_gpu(device):
    if device is None or 'cuda' not in device.type or not torch.cuda.is_available():
        raise RuntimeError("this build runs the turbo backend on an MI355X GPU only; pass a cuda device "
                           "(there is no CPU or onnxruntime fallback)")


class BertModelNoPooler:
    def __init__(self, embeddings: BertEmbeddings, encoder: BertEncoder):
        self.embeddings = embeddings
        self.encoder = encoder
        self.prepare = cxx.PrepareBertMasks()

    def __call__(self, inputs: AnyTensor, attention_masks: Optional[AnyTensor] = None,
                 token_type_ids: Optional[AnyTensor] = None, position_ids: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, inputs_embeds: Optional[AnyTensor] = None,
                 output_attentions: Optional[bool] = None, output_hidden_states: Optional[bool] = None,
                 pooling_type: PoolingType = PoolingType.FIRST, return_type: Optional[ReturnType] = None):
        use_current_stream()
        attention_masks = try_convert(create_empty_if_none(attention_masks))
        token_type_ids = try_convert(create_empty_if_none(token_type_ids))
        position_ids = try_convert(create_empty_if_none(position_ids))
        inputs = try_convert(inputs)
        extended_attention_masks = cxx.Tensor.create_empty()
        self.prepare(inputs, attention_masks, token_type_ids, position_ids, extended_attention_masks)
        hidden = self.embeddings(inputs, position_ids=position_ids, token_type_ids=token_type_ids,
                                 return_type=ReturnType.turbo_transformers)
        return self.encoder(hidden_states=hidden, attention_mask=extended_attention_masks,
                            output_attentions=output_attentions, output_hidden_states=output_hidden_states,
                            return_type=return_type)

    @staticmethod
    def from_torch(model, device: Optional[torch.device] = None):
        device = device if device is not None else model.device
        _require_gpu(device)
        model.to(device)
        return BertModelNoPooler(BertEmbeddings.from_torch(model.embeddings), BertEncoder.from_torch(model.encoder))

    @staticmethod
    def from_npz(file_name: str, config, device: Optional[torch.device] = None):
        return BertModelNoPooler(BertEmbeddings.from_npz(file_name, device),
                                 BertEncoder.from_npz(file_name, config.num_hidden_layers, config.num_attention_heads,
                                                      device))


class BertModel:
    """`turbo_transformers.BertModel`: `from_torch(model, device, backend="turbo")` then call it
    like the HuggingFace model; returns (sequence_output, pooler_output, ...)."""

    def __init__(self, model, pooler=None, backend="turbo", config=None):
        if backend != "turbo":
            raise NotImplementedError("only backend='turbo' exists in this build (no onnxruntime path)")
        self.backend = "turbo"
        self.config = config
        self.bertmodel_nopooler = model
        self.pooler = pooler

    def __call__(self, inputs: AnyTensor, attention_masks: Optional[AnyTensor] = None,
                 token_type_ids: Optional[AnyTensor] = None, position_ids: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, inputs_embeds: Optional[AnyTensor] = None,
                 output_attentions: Optional[bool] = None, output_hidden_states: Optional[bool] = None,
                 pooling_type: PoolingType = PoolingType.FIRST, pooler_output: Optional[AnyTensor] = None,
                 return_type: Optional[ReturnType] = None, output_fp32_hidden_state: bool = False):
        """output_fp32_hidden_state (not in the reference): bfloat16 models keep their residual stream in fp32; True
        appends that unrounded final hidden state (a float32 torch tensor, or None for other dtypes) to the result."""
        encoder_outputs = self.bertmodel_nopooler(inputs, attention_masks, token_type_ids, position_ids,
                                                  inputs_embeds=inputs_embeds, output_attentions=output_attentions,
                                                  output_hidden_states=output_hidden_states,
                                                  pooling_type=pooling_type,
                                                  return_type=ReturnType.turbo_transformers)
        sequence_output = encoder_outputs[0]
        self.seq_pool = SequencePool(PoolingMap[pooling_type])
        pooled = self.seq_pool(input_tensor=sequence_output, return_type=ReturnType.turbo_transformers)
        pooler_output = self.pooler(pooled, return_type, pooler_output)
        extra = ()
        if output_fp32_hidden_state:
            shadow = sequence_output.take_fp32_shadow()
            extra = (convert_returns_as_type(shadow, ReturnType.TORCH) if shadow is not None else None, )
        return (convert_returns_as_type(sequence_output, return_type), pooler_output) + encoder_outputs[1:] + extra

    @staticmethod
    def from_torch(model, device: Optional[torch.device] = None, backend: Optional[str] = None, use_memory_opt=False):
        """model: a HuggingFace BertModel; device: a cuda device; backend: "turbo" (the default)."""
        if device is None:
            device = model.device
        if backend is None:
            backend = "turbo"
        if backend != "turbo":
            raise NotImplementedError("only backend='turbo' exists in this build (no onnxruntime path)")
        _require_gpu(device)
        model.to(device)
        nopooler = BertModelNoPooler(BertEmbeddings.from_torch(model.embeddings), BertEncoder.from_torch(model.encoder))
        pooler = BertPooler.from_torch(model.pooler)
        return BertModel(nopooler, pooler, "turbo", model.config)

    @staticmethod
    def from_pretrained(model_id_or_path: str, device: Optional[torch.device] = None, backend: Optional[str] = None):
        from transformers import BertModel as TorchBertModel
        torch_model = TorchBertModel.from_pretrained(model_id_or_path)
        model = BertModel.from_torch(torch_model, device, backend)
        model._torch_model = torch_model  # keeps the aliased weights alive
        return model

    @staticmethod
    def from_npz(file_name: str, config, device: Optional[torch.device] = None):
        _require_gpu(device)
        return BertModel(BertModelNoPooler.from_npz(file_name, config, device), BertPooler.from_npz(file_name, device),
                         backend="turbo", config=config)
