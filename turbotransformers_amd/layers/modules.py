"""General multi-headed attention with the reference's Python surface
(python/turbo_transformers/layers/modules.py:36-230): self attention (optionally with a growing
self_keys/self_values cache), "context" attention over an encoder memory (optionally cached as
memory_keys/memory_values), pre-LayerNorm, post-LayerNorm or post_add_input.

`from_onmt` takes any module that exposes OpenNMT-py's parameter names (linear_keys, linear_values,
linear_query, final_linear, head_count, max_relative_positions); OpenNMT itself is not imported.
"""
from typing import Optional

import torch

from .. import cxx
from .return_type import ReturnType, convert_returns_as_type
from .utils import (AnyTensor, convert2tt_tensor, create_empty_if_none, to_param_dict, try_convert, use_current_stream,
                    weight_in_out)

__all__ = ['MultiHeadedAttention', 'PositionwiseFeedForward', 'DistrillFFN']


class MultiHeadedAttention(cxx.MultiHeadedAttention):
    def __call__(self, key_tensor: AnyTensor, value_tensor: AnyTensor, query_tensor: AnyTensor,
                 mask: Optional[AnyTensor] = None, layer_cache: Optional[dict] = None, attn_type: str = None,
                 pre_layernorm: bool = False, post_layernorm: bool = False, post_add_input: bool = False,
                 is_trans_weight: bool = False, return_type: Optional[ReturnType] = None,
                 output: Optional[cxx.Tensor] = None, attn: Optional[cxx.Tensor] = None):
        """-> (output [B,F,H], attn [B,h,F,T]).  `mask` is additive (0 keeps, a large negative value drops),
        [B,1,T] or [B,F,T].  `layer_cache` is updated in place with torch tensors, like the reference:
        the memory_* entries after a "context" call, the self_* entries after a "self" call."""
        use_current_stream()
        output = create_empty_if_none(output)
        attn = create_empty_if_none(attn)
        cache = {}
        if layer_cache is not None:
            for k, v in layer_cache.items():
                cache[k] = try_convert(v) if v is not None else cxx.Tensor.create_empty()
        super().__call__(try_convert(key_tensor), try_convert(value_tensor), try_convert(query_tensor),
                         try_convert(create_empty_if_none(mask)), attn_type, output, attn, cache, pre_layernorm,
                         post_layernorm, post_add_input, is_trans_weight)
        if layer_cache is not None:
            for k, v in cache.items():
                if ("memory" in k and "context" in attn_type) or ("self" in k and "self" in attn_type):
                    layer_cache[k] = convert_returns_as_type(v, ReturnType.TORCH)
        return convert_returns_as_type(output, return_type), convert_returns_as_type(attn, return_type)

    @staticmethod
    def pack_parameter(params: dict, names: dict, is_trans_weight: bool = False):
        """The ten weight tensors in constructor order: k_w,k_b,v_w,v_b,q_w,q_b,dense_w,dense_b,qkv_w,qkv_b.
        `names` maps q/k/v/out to the parameter prefixes of the source module."""
        pack = (lambda w: w.detach().contiguous()) if is_trans_weight else weight_in_out
        w = lambda role: params[names[role] + '.weight']
        b = lambda role: params[names[role] + '.bias'].detach().contiguous()
        with torch.no_grad():
            qkv_weight = pack(torch.cat((w('q'), w('k'), w('v')), 0))
            qkv_bias = torch.cat((b('q'), b('k'), b('v')), 0).contiguous()
            return [pack(w('k')), b('k'), pack(w('v')), b('v'), pack(w('q')), b('q'), pack(w('out')), b('out'),
                    qkv_weight, qkv_bias]

    @staticmethod
    def from_onmt(multi_headed_attn, layer_norm: Optional[torch.nn.Module] = None, is_trans_weight: bool = False):
        if getattr(multi_headed_attn, 'max_relative_positions', 0) != 0:
            raise ValueError("multi_headed_attn's max_relative_positions should be 0!")
        names = {'q': 'linear_query', 'k': 'linear_keys', 'v': 'linear_values', 'out': 'final_linear'}
        args = MultiHeadedAttention.pack_parameter(to_param_dict(multi_headed_attn), names, is_trans_weight)
        if layer_norm is not None:
            ln = to_param_dict(layer_norm)
            args += [ln['weight'].detach().contiguous(), ln['bias'].detach().contiguous()]
        return MultiHeadedAttention(*[convert2tt_tensor(a) for a in args], multi_headed_attn.head_count)

    @staticmethod
    def from_torch(attention, layer_norm: Optional[torch.nn.Module] = None, is_trans_weight: bool = False):
        """From a HuggingFace BertAttention (self.query/key/value + output.dense); LayerNorm parameters come
        from `layer_norm` when given, else from attention.output.LayerNorm."""
        p = to_param_dict(attention)
        names = {'q': 'self.query', 'k': 'self.key', 'v': 'self.value', 'out': 'output.dense'}
        args = MultiHeadedAttention.pack_parameter(p, names, is_trans_weight)
        ln = to_param_dict(layer_norm) if layer_norm is not None else {
            'weight': p['output.LayerNorm.weight'], 'bias': p['output.LayerNorm.bias']}
        args += [ln['weight'].detach().contiguous(), ln['bias'].detach().contiguous()]
        return MultiHeadedAttention(*[convert2tt_tensor(a) for a in args], attention.self.num_attention_heads)


class _FeedForward:
    """Shared call convention of the two feed-forward blocks (modules.py:233-290 of the reference)."""

    def __call__(self, input_tensor: AnyTensor, return_type: Optional[ReturnType] = None, is_trans_weight: bool = False,
                 output: Optional[cxx.Tensor] = None):
        use_current_stream()
        output = create_empty_if_none(output)
        super().__call__(try_convert(input_tensor), output, is_trans_weight)
        return convert_returns_as_type(output, return_type)

    @classmethod
    def _from_parts(cls, lin1, lin2, layer_norm, is_trans_weight):
        pack = (lambda w: w.detach().contiguous()) if is_trans_weight else weight_in_out
        with torch.no_grad():
            args = [pack(lin1.weight), lin1.bias.detach().contiguous(), pack(lin2.weight), lin2.bias.detach().contiguous(),
                    layer_norm.weight.detach().contiguous(), layer_norm.bias.detach().contiguous()]
        return cls(*[convert2tt_tensor(a) for a in args])


class PositionwiseFeedForward(_FeedForward, cxx.PositionwiseFeedForward):
    """output = x + W2 relu(W1 LayerNorm(x) + b1) + b2 (OpenNMT-py's PositionwiseFeedForward)."""

    @staticmethod
    def from_onmt(position_wise_ffn, is_trans_weight: bool = False):
        return PositionwiseFeedForward._from_parts(position_wise_ffn.w_1, position_wise_ffn.w_2, position_wise_ffn.layer_norm,
                                                   is_trans_weight)


class DistrillFFN(_FeedForward, cxx.DistrillFFN):
    """output = LayerNorm(x + W2 gelu(W1 x + b1) + b2) (the feed-forward half of a DistilBERT block)."""

    @staticmethod
    def from_torch(ffn, layer_norm, is_trans_weight: bool = False):
        return DistrillFFN._from_parts(ffn.lin1, ffn.lin2, layer_norm, is_trans_weight)
