"""RoBERTa on the BERT encoder path.

The reference's RobertaModel (python/turbo_transformers/layers/modeling_roberta.py:51-149) keeps the
HuggingFace embeddings module in torch and runs turbo's BertEncoder + pooler behind it.  A RoBERTa
embedding differs from BERT's only in how position ids are derived (padding_idx + running count of
non-pad tokens), so here the embeddings are the gather + LayerNorm kernel as well and only the position
ids are computed in torch.
"""
from typing import Optional

import torch

from .modeling_bert import (BertEmbeddings, BertEncoder, BertModel, BertModelNoPooler, BertPooler, PoolingType, _require_gpu)
from .return_type import ReturnType
from .utils import AnyTensor

__all__ = ['RobertaModel']


def roberta_position_ids(input_ids: torch.Tensor, padding_idx: int) -> torch.Tensor:
    """Non-pad tokens count up from padding_idx + 1, pad tokens stay at padding_idx."""
    keep = input_ids.ne(padding_idx).long()
    return torch.cumsum(keep, dim=1) * keep + padding_idx


class RobertaModel:
    """`RobertaModel.from_torch(hf_roberta_model, device)`, then call it like the HuggingFace model;
    returns (sequence_output, pooler_output)."""

    def __init__(self, bert: BertModel, config):
        self.bert = bert
        self.config = config

    def __call__(self, input_ids: AnyTensor, attention_mask: Optional[AnyTensor] = None,
                 token_type_ids: Optional[AnyTensor] = None, position_ids: Optional[AnyTensor] = None,
                 head_mask: Optional[AnyTensor] = None, inputs_embeds: Optional[AnyTensor] = None,
                 pooling_type: PoolingType = PoolingType.FIRST, return_type: Optional[ReturnType] = None):
        if inputs_embeds is not None:
            raise NotImplementedError("inputs_embeds is not supported; pass input_ids")
        if position_ids is None:
            position_ids = roberta_position_ids(input_ids, self.config.pad_token_id)
        return self.bert(input_ids, attention_masks=attention_mask, token_type_ids=token_type_ids,
                         position_ids=position_ids, pooling_type=pooling_type, return_type=return_type)

    @staticmethod
    def from_torch(model, device: Optional[torch.device] = None, backend: Optional[str] = None):
        """model: a HuggingFace RobertaModel built with its pooling layer."""
        if backend not in (None, "turbo"):
            raise NotImplementedError("only backend='turbo' exists in this build (no onnxruntime path)")
        device = device if device is not None else model.device
        _require_gpu(device)
        model.to(device)
        if model.pooler is None:
            raise ValueError("RobertaModel.from_torch needs a model built with add_pooling_layer=True")
        nopooler = BertModelNoPooler(BertEmbeddings.from_torch(model.embeddings), BertEncoder.from_torch(model.encoder))
        return RobertaModel(BertModel(nopooler, BertPooler.from_torch(model.pooler), "turbo", model.config), model.config)
