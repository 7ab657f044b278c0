from .modeling_bert import (BertEmbeddings, BertIntermediate, BertOutput, BertAttention, BertLayer, SequencePool,
                            BertEncoder, BertModel, BertModelNoPooler, PoolingType, BertPooler)
from .modeling_smart_pad import (MultiHeadedAttentionSmartBatch, BertLayerSmartBatch, BertEncoderSmartBatch,
                                 BertModelNoPoolerSmartBatch, BertModelSmartBatch)
from .modeling_albert import (AlbertEmbeddings, AlbertAttention, AlbertLayer, AlbertLayerGroup, AlbertTransformer,
                              AlbertModel)
from .qmodeling_bert import QBertIntermediate, QBertOutput, QBertAttention, QBertLayer, QBertEncoder, QBertModel
from .modules import MultiHeadedAttention, PositionwiseFeedForward, DistrillFFN
from .modeling_roberta import RobertaModel
from .modeling_distillbert import DistilBertModel
from .return_type import ReturnType

__all__ = [
    'BertEmbeddings', 'BertIntermediate', 'BertOutput', 'BertAttention', 'BertLayer', 'BertEncoder', 'BertModel',
    'BertModelNoPooler', 'ReturnType', 'BertPooler', 'SequencePool', 'PoolingType', 'MultiHeadedAttentionSmartBatch',
    'BertLayerSmartBatch', 'BertEncoderSmartBatch', 'BertModelNoPoolerSmartBatch', 'BertModelSmartBatch',
    'QBertIntermediate', 'QBertOutput', 'QBertAttention', 'QBertLayer', 'QBertEncoder', 'QBertModel',
    'MultiHeadedAttention', 'PositionwiseFeedForward', 'DistrillFFN', 'AlbertEmbeddings', 'AlbertAttention', 'AlbertLayer', 'AlbertLayerGroup', 'AlbertTransformer', 'AlbertModel', 'RobertaModel', 'DistilBertModel',
]
