"""FlashAttention cell of the Megatron-style ("mcore") inference stack:
mindformers/parallel_core/inference/transformer/flash_attention.py:23-145.  Caches are passed per call.
"""
import torch
from torch import nn

from .. import ops


class FlashAttention(nn.Module):
    """ReshapeAndCache, then FlashAttentionScore (prefill; not built) or PagedAttention (decode)."""

    def __init__(self, head_num, head_dim=None, kv_head_num=None, keep_prob=1.0, scale_value=1.0,
                 pre_tokens=2147483647, next_tokens=2147483647, sparse_mode=0, input_layout="TH",
                 pa_kv_head_num=None, pa_mla_v_dim=0):
        super().__init__()
        if pa_mla_v_dim > 0:
            raise NotImplementedError("multi-latent attention (pa_mla_v_dim > 0) is not built")
        if input_layout not in ("TH", "TND"):
            raise ValueError(f"input_layout must be TH or TND, got {input_layout}")
        self.head_num = head_num
        self.hidden_size_per_attention_head = head_dim
        self.kv_head_num = kv_head_num
        self.pa_kv_head_num = pa_kv_head_num if pa_kv_head_num is not None else kv_head_num
        self.scale_value = scale_value
        self.sparse_mode = sparse_mode
        self.is_prefill = True
        self.input_layout = input_layout
        self.use_multi_latent_attention = False

    def forward(self, query, key, value, slot_mapping=None, block_tables=None, batch_valid_length=None,
                context_lens_tensor=None, q_seq_lens=None, actual_seq_qlen=None, actual_seq_kvlen=None,
                attn_mask=None, padding_mask=None, prefix=None, key_cache=None, value_cache=None):
        """Forward process of the FlashAttention (flash_attention.py:109-145)."""
        ops.reshape_and_cache(key, value, key_cache, value_cache, slot_mapping)
        if self.is_prefill:
            raise NotImplementedError("prefill (FlashAttentionScore) is not built: set is_prefill = False")
        shape = query.shape
        out = ops.paged_attention(query.reshape(-1, shape[-1]) if query.dim() > 2 else query, key_cache, value_cache,
                                  block_tables, batch_valid_length, self.head_num, self.pa_kv_head_num,
                                  self.scale_value)
        return out.reshape(shape)

    construct = forward
