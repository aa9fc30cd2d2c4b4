"""FlashAttention cell of the Megatron-style ("mcore") inference stack:
mindformers/parallel_core/inference/transformer/flash_attention.py:23-145.  Caches are passed per call.
"""
import torch
from torch import nn

from .. import ops


class FlashAttention(nn.Module):
    """ReshapeAndCache, then FlashAttentionScore (prefill) or PagedAttention (decode; with q_seq_lens: several new
    tokens per sequence; with pa_mla_v_dim > 0: multi-latent decode over the single latent cache, whose prefill runs as
    ordinary attention on the up-projected keys and values).  Masks are causal: `attn_mask` is accepted for signature parity and taken to be the lower
    triangle the reference's models build; sparse modes other than the causal default are not built."""

    def __init__(self, head_num, head_dim=None, kv_head_num=None, keep_prob=1.0, scale_value=1.0,
                 pre_tokens=2147483647, next_tokens=2147483647, sparse_mode=0, input_layout="TH",
                 pa_kv_head_num=None, pa_mla_v_dim=0):
        super().__init__()
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
        self.pa_mla_v_dim = pa_mla_v_dim
        self.use_multi_latent_attention = pa_mla_v_dim > 0

    def forward(self, query, key, value, slot_mapping=None, block_tables=None, batch_valid_length=None,
                context_lens_tensor=None, q_seq_lens=None, actual_seq_qlen=None, actual_seq_kvlen=None,
                attn_mask=None, padding_mask=None, prefix=None, key_cache=None, value_cache=None,
                antiquant_scale=None, antiquant_offset=None, key_scale_cache=None, value_scale_cache=None):
        """Forward process of the FlashAttention (flash_attention.py:109-145).  int8 caches (kvcache_dtype: int8) come
        with ``antiquant_scale`` / ``antiquant_offset`` float32 [2, n_kv * D] (keys, values), the arguments the
        reference's PagedAttention call has in positions 6-7: the scatter then quantises and the attention
        dequantises.  Caches quantised per token (kvcache_quant_granularity: per_token) come with
        ``key_scale_cache`` / ``value_scale_cache`` float32 [num_blocks, block_size] instead: the scatter writes each
        token's scale beside its row."""
        kv8 = key_cache is not None and key_cache.dtype == torch.int8
        per_token = key_scale_cache is not None
        if kv8 and not per_token and antiquant_scale is None:
            raise ValueError("int8 caches need antiquant_scale (and optionally antiquant_offset), or the per-token "
                             "scale caches")
        if per_token and (not kv8 or value_scale_cache is None or antiquant_scale is not None):
            raise ValueError("per-token scale caches go with int8 caches, both of them, and no per-channel parameters")
        if kv8 and self.use_multi_latent_attention:
            raise NotImplementedError("an int8 latent cache is not built")
        token_scales = (key_scale_cache, value_scale_cache) if per_token else None
        if per_token:
            ops.dynamic_quant_reshape_and_cache(key, value, key_cache, value_cache, key_scale_cache, value_scale_cache,
                                                slot_mapping)
        elif kv8:
            ops.quant_reshape_and_cache(key, value, key_cache, value_cache, slot_mapping, antiquant_scale,
                                        antiquant_offset)
        elif not self.use_multi_latent_attention:             # MLA: the caller has written the latent row already
            ops.reshape_and_cache(key, value, key_cache, value_cache, slot_mapping)
        shape = query.shape
        if query.dim() == 2:
            q2 = query
        elif self.input_layout == "TND":
            q2 = query.reshape(shape[0], -1)
        else:
            q2 = query.reshape(-1, shape[-1])
        if self.is_prefill:
            # FlashAttentionScore over this step's packed rows (flash_attention.py:129-134); keys are the step's own,
            # so the query and key lists must agree
            if actual_seq_kvlen is not None and actual_seq_kvlen is not actual_seq_qlen:
                if not torch.equal(torch.as_tensor(actual_seq_kvlen).cpu(), torch.as_tensor(actual_seq_qlen).cpu()):
                    raise NotImplementedError("prefill with actual_seq_kvlen != actual_seq_qlen is not built "
                                              "(use the decode branch with q_seq_lens for chunked prefill)")
            if actual_seq_qlen is None:
                starts = torch.tensor([0, q2.shape[0]], dtype=torch.int32, device=query.device)
            else:
                starts = ops.q_starts_from_actual_seq_len(torch.as_tensor(actual_seq_qlen, device=query.device),
                                                          q2.shape[0])
            k2 = key if key.dim() == 2 else key.reshape(q2.shape[0], -1)
            v2 = value if value.dim() == 2 else value.reshape(q2.shape[0], -1)
            # the kv head count of this step's keys: kv_head_num, which for multi-latent attention differs from the
            # cache's (pa_kv_head_num = 1): its prefill attends over the up-projected 192-wide keys of every head
            # (multi_latent_attention.py:405-432)
            d = q2.shape[1] // self.head_num
            narrow_v = d == 192 and k2.shape[1] % d == 0 and v2.shape[1] == k2.shape[1] // d * 128
            if q2.shape[1] != self.head_num * d or k2.shape[1] % d or (v2.shape[1] != k2.shape[1] and not narrow_v):
                raise ValueError(f"query / key / value widths {q2.shape[1]} / {k2.shape[1]} / {v2.shape[1]} do not "
                                 f"fit {self.head_num} heads")
            out = ops.causal_attention_varlen(q2, k2, v2, starts, self.head_num, k2.shape[1] // d, self.scale_value)
            if narrow_v:                                      # 128-wide value heads of multi-latent attention, unpadded
                return out
            return out.reshape(shape)
        if self.use_multi_latent_attention:                   # one latent cache, keys = values (flash_attention.py:136-139)
            out = ops.mla_paged_attention(q2, key_cache, block_tables, batch_valid_length, self.head_num,
                                          self.pa_mla_v_dim, self.scale_value, q_seq_lens=q_seq_lens)
            return out.reshape(*shape[:-1], self.head_num * self.pa_mla_v_dim)
        if kv8:
            starts = None if q_seq_lens is None else ops.q_starts_from_lens(q_seq_lens)
            out = ops.paged_attention_int8kv(q2, key_cache, value_cache, block_tables, batch_valid_length,
                                             antiquant_scale, antiquant_offset, self.head_num, self.pa_kv_head_num,
                                             self.scale_value, q_starts=starts, token_scales=token_scales)
            return out.reshape(shape)
        if q_seq_lens is not None:                            # several new tokens per sequence (flash_attention.py:140-143)
            out = ops.paged_attention_prefill(q2, key_cache, value_cache, block_tables, batch_valid_length,
                                              ops.q_starts_from_lens(q_seq_lens), self.head_num,
                                              self.pa_kv_head_num, self.scale_value)
            return out.reshape(shape)
        out = ops.paged_attention(q2, key_cache, value_cache, block_tables, batch_valid_length, self.head_num,
                                  self.pa_kv_head_num, self.scale_value)
        return out.reshape(shape)

    construct = forward
