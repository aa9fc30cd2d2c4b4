"""Drop-in modules of the decode path (same constructor / call surface as the reference's cells)."""
from .block_tables import BlockMemPool, BlockTables, CacheEngine
from .flash_attention import FlashAttention
from .infer_attention import InferAttention, InferRotaryEmbedding
from .layers import (AllQuantLinearInferCell, ColumnParallelLinear, Linear, QKVParallelLinear, ReplicatedLinear,
                     RowParallelLinear, WeightQuantLinearCell)
from .mlp import MLP, LlamaFeedForward
from .moe import GroupedMLP, MoELayer, QuantGroupedMLP, SharedExpertMLP, TopKRouter
from .multi_latent_attention import MLASelfAttention, MLASelfAttentionSubmodules, MLATransformerConfig
from .norm import LlamaRMSNorm, RMSNorm
from .paged_attention_mgr import PagedAttentionMgr, QuantPagedAttentionMgr
from .rotary import FreqsMgr, Llama3RotaryEmbedding, RotaryEmbedding, YaRNScalingRotaryEmbedding
