"""InferAttention / InferRotaryEmbedding — the reference's mindformers/modules/infer_attention.py:30-63,66-486
call surface for the decode step: RoPE -> KV scatter -> paged attention.
"""
import math

import torch
from torch import nn

from .. import ops
from .paged_attention_mgr import PagedAttentionMgr


class InferRotaryEmbedding(nn.Module):
    """ApplyRotaryPosEmb(rotary_cos_format) on query and key (infer_attention.py:30-63).  Format 2 (rotate-half)
    is what every Llama/Qwen/DeepSeek caller passes (llama_transformer.py:330); others are not built."""

    def __init__(self, rotary_cos_format=0, n_head=None, n_kv_head=None, head_dim=None):
        super().__init__()
        if rotary_cos_format != 2:
            raise NotImplementedError(f"rotary_cos_format={rotary_cos_format}: only 2 (rotate-half) is built")
        self.rotary_cos_format = rotary_cos_format
        self.n_head, self.n_kv_head, self.head_dim = n_head, n_kv_head, head_dim

    def forward(self, query, key, freqs_cis, batch_valid_length):
        freqs_cos, freqs_sin, _ = freqs_cis
        query = query.contiguous()
        key = key.contiguous()
        ops.apply_rotary_pos_emb(query, key, freqs_cos.contiguous(), freqs_sin.contiguous(), self.n_head,
                                 self.n_kv_head, self.head_dim)
        return query, key

    construct = forward


class InferAttention(nn.Module):
    """Infer Attention Layer (infer_attention.py:209-231 constructor, :441-463 call).

    query [B, S, n_head*D] (BSH) or [T, n_head*D] / [1, T, n_head*D] (TH).  Decode: `batch_valid_length` is the
    context length including the token written by this call.  Prefill (`is_first_iteration`): causal attention over
    this call's own keys; in the TH layout `batch_valid_length` (the lengths of the packed sequences, or their
    increasing row ends) is what the reference hands to FlashAttentionScore (infer_attention.py:459-461), in BSH
    every batch row is a full sequence of S tokens.  Masks are causal; `attn_mask` is not read."""

    def __init__(self, n_head, head_dim, n_kv_head, pa_n_head_split=None, pa_n_kv_head_split=None, keep_prob=1.0,
                 scale_value=1.0, pre_tokens=2147483647, next_tokens=2147483647, sparse_mode=0, block_size=16,
                 num_blocks=1024, seq_length=-1, is_dynamic=True, use_flash_attention=True, use_alibi_mask=False,
                 use_rope_rotary_emb=True, rotary_cos_format=0, compute_dtype=torch.float16, parallel_decoding=False,
                 chunk_prefill=False, device="cuda"):
        super().__init__()
        if use_alibi_mask:
            raise NotImplementedError("alibi attention is not built")
        if keep_prob != 1.0:
            raise ValueError("keep_prob must be 1.0 for inference")
        self.n_head = n_head
        self.head_dim = head_dim
        self.n_kv_head = n_kv_head
        self.pa_n_head_split = pa_n_head_split if pa_n_head_split is not None else n_head
        self.pa_n_kv_head_split = pa_n_kv_head_split if pa_n_kv_head_split is not None else n_kv_head
        self.keep_prob = keep_prob
        self.scale_value = scale_value
        self.pre_tokens = pre_tokens
        self.next_tokens = next_tokens
        self.sparse_mode = sparse_mode
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.use_flash_attention = use_flash_attention
        self.use_alibi_mask = use_alibi_mask
        self.use_rope_rotary_emb = use_rope_rotary_emb
        self.rotary_cos_format = rotary_cos_format
        self.compute_dtype = compute_dtype
        self.is_first_iteration = True
        self.chunk_prefill = chunk_prefill
        self.n_rep = self.n_head // self.n_kv_head
        self.inv_norm_factor = 1.0 / math.sqrt(self.head_dim)
        self.is_dynamic = is_dynamic
        self.input_layout = "TH" if is_dynamic else "BSH"
        kv_shape = (self.num_blocks, self.block_size, self.n_kv_head, self.head_dim)
        self.paged_attention_mgr = PagedAttentionMgr(self.pa_n_head_split, self.head_dim, self.pa_n_kv_head_split,
                                                     kv_shape, seq_length, compute_dtype=self.compute_dtype,
                                                     parallel_decoding=parallel_decoding, chunk_prefill=chunk_prefill,
                                                     device=device)
        if use_rope_rotary_emb:
            self.rotary_embedding = InferRotaryEmbedding(self.rotary_cos_format, n_head, n_kv_head, head_dim)

    def _apply_rotary_pos_emb(self, query, key, freqs_cis, batch_valid_length):
        return self.rotary_embedding(query, key, freqs_cis, batch_valid_length)

    def _incre_attention(self, query, batch_valid_length, block_tables, alibi_mask=None, attn_mask=None,
                         q_seq_lens=None):
        return self.paged_attention_mgr.paged_attn(query, batch_valid_length, block_tables, attn_mask=attn_mask,
                                                   q_seq_lens=q_seq_lens)

    def forward(self, query, key, value, batch_valid_length, block_tables, slot_mapping, freqs_cis=None,
                attn_mask=None, alibi_mask=None, prefix_keys_values=None, q_seq_lens=None):
        """Forward process of the Infer Attention Cell (infer_attention.py:441-463)."""
        if prefix_keys_values is not None:
            raise NotImplementedError("prefix_keys_values (p-tuning prefix) is not built")
        mgr = self.paged_attention_mgr
        shape = query.shape
        q2 = query.reshape(-1, self.n_head * self.head_dim).contiguous()
        k2 = key.reshape(-1, self.n_kv_head * self.head_dim).contiguous()
        v2 = value.reshape(-1, self.n_kv_head * self.head_dim).contiguous()
        if self.use_rope_rotary_emb and mgr.key_cache.dtype != torch.int8:
            # RoPE + scatter of the rotated key and of value in one launch (infer_attention.py:445,453);
            # same-stream ordering stands in for ops.depend (:454)
            freqs_cos, freqs_sin, _ = freqs_cis
            ops.rope_and_cache(q2, k2, v2, freqs_cos.contiguous(), freqs_sin.contiguous(), mgr.key_cache,
                               mgr.value_cache, slot_mapping, self.n_head)
        else:
            if self.use_rope_rotary_emb:                      # int8 caches: rotate, then the manager quantises
                q2, k2 = self._apply_rotary_pos_emb(q2, k2, freqs_cis, batch_valid_length)
            mgr(k2, v2, slot_mapping, batch_valid_length)
        if self.chunk_prefill:                                # infer_attention.py:456-458
            return mgr.paged_attn(q2, batch_valid_length, block_tables, attn_mask=attn_mask,
                                  q_seq_lens=q_seq_lens).reshape(shape)
        if self.is_first_iteration:
            return self._prefill_attention(q2, k2, v2, attn_mask, alibi_mask, batch_valid_length,
                                           batch_valid_length, shape).reshape(shape)
        return self._incre_attention(q2, batch_valid_length, block_tables, alibi_mask, attn_mask,
                                     q_seq_lens).reshape(shape)

    def _prefill_attention(self, query, key, value, attn_mask, alibi_mask, actual_seq_qlen=None,
                           actual_seq_kvlen=None, shape=None):
        """FlashAttentionScore of the first iteration (infer_attention.py:405-431) on packed [T, H] rows."""
        if self.input_layout == "TH":
            starts = ops.q_starts_from_actual_seq_len(actual_seq_qlen, query.shape[0])
        else:                                                 # BSH: every batch row is one sequence of S tokens
            bsz, seq = shape[0], shape[1]
            starts = torch.arange(0, bsz + 1, dtype=torch.int32, device=query.device) * seq
        return ops.causal_attention_varlen(query, key, value, starts, self.n_head, self.n_kv_head, self.scale_value)

    construct = forward

    def shard(self, parallel_config):
        return self
