"""PagedAttentionMgr — same constructor, attributes and calls as the reference's
mindformers/modules/paged_attention_mgr.py:26-92, on torch tensors and the gfx950 kernels.
"""
import math

import torch
from torch import nn

from .. import ops


class PagedAttentionMgr(nn.Module):
    """Owns the key/value caches [num_blocks, block_size, n_kv_heads, head_dim] and runs
    reshape_and_cache / paged_attention on them (paged_attention_mgr.py:29-58)."""

    def __init__(self, n_heads, head_dim, n_kv_heads, kv_shape, seq_length=-1, compute_dtype=torch.float16,
                 parallel_decoding=False, chunk_prefill=False, device="cuda"):
        super().__init__()
        if len(kv_shape) != 4:
            raise ValueError(f"kv_shape must be (num_blocks, block_size, n_kv_heads, head_dim), got {kv_shape}")
        if kv_shape[2] != n_kv_heads or kv_shape[3] != head_dim:
            raise ValueError(f"kv_shape {kv_shape} does not match n_kv_heads={n_kv_heads}, head_dim={head_dim}")
        self.n_heads = n_heads
        self.head_dim = head_dim
        self.n_kv_heads = n_kv_heads
        self.seq_length = seq_length
        self.is_first_iteration = True
        self.scale_value = 1 / math.sqrt(self.head_dim)
        self.register_buffer("key_cache", torch.zeros(kv_shape, dtype=compute_dtype, device=device), persistent=False)
        self.register_buffer("value_cache", torch.zeros(kv_shape, dtype=compute_dtype, device=device), persistent=False)
        self.parallel_decoding = parallel_decoding
        self.chunk_prefill = chunk_prefill

    def forward(self, key, value, slot_mapping, batch_valid_length=None):
        """The forward compute of KVCache for Paged Attention (paged_attention_mgr.py:60-62)."""
        return ops.reshape_and_cache(key, value, self.key_cache, self.value_cache, slot_mapping)

    construct = forward

    def paged_attn(self, query, batch_valid_length, block_tables, attn_mask=None, q_seq_lens=None):
        """The forward compute of Paged Attention (paged_attention_mgr.py:64-70).  With parallel_decoding or
        chunk_prefill every sequence brings q_seq_lens[b] new tokens, masked causally among themselves: `attn_mask` is
        taken to be that lower triangle (generation/parallel_decoding.py:73-80) and is not read."""
        shape = query.shape
        q2 = query.reshape(-1, self.n_heads * self.head_dim)
        if self.parallel_decoding or self.chunk_prefill:
            if q_seq_lens is None:
                raise ValueError("parallel_decoding / chunk_prefill need q_seq_lens")
            out = ops.paged_attention_prefill(q2, self.key_cache, self.value_cache, block_tables, batch_valid_length,
                                              ops.q_starts_from_lens(q_seq_lens), self.n_heads, self.n_kv_heads,
                                              self.scale_value)
        else:
            out = ops.paged_attention(q2, self.key_cache, self.value_cache, block_tables, batch_valid_length,
                                      self.n_heads, self.n_kv_heads, self.scale_value)
        return out.reshape(shape)

    def paged_attn_with_alibi(self, query, batch_valid_length, block_tables, alibi_tensor):
        """paged_attention_mgr.py:72-75 — no alibi model is on the built path."""
        raise NotImplementedError("PagedAttentionMask (alibi) is not built")

    def shard(self, parallel_config):
        """One GPU: nothing to shard (paged_attention_mgr.py:77-92 only sets layouts)."""
        return self


class QuantPagedAttentionMgr(PagedAttentionMgr):
    """The manager a quantizer swaps in for ``kvcache_dtype: int8`` (per channel): int8 caches of the same shape,
    the quantising scatter, and attention that receives the dequantisation parameters where the reference's call
    passes ``antiquant_scale`` / ``antiquant_offset`` (positions 6-7 of PagedAttention,
    mindformers/modules/paged_attention_mgr.py:66-70; the cache dtype comes from the quantization config,
    mindformers/model_runner.py:364-368).  The cell itself belongs to golden-stick in the reference stack, so the
    parameter names are this build's: ``kv_scale`` / ``kv_offset`` float32 [2, n_kv_heads * head_dim] (keys, values),
    x ~ (q - offset) * scale, loaded from the checkpoint or set with ``set_kv_quant``.

    ``granularity="per_token"`` (kvcache_quant_granularity, mindformers/utils/quantization_config.py:206-207): nothing
    is loaded; every token row is quantised with its own scale as it is written, and the scales live beside the rows
    in ``key_scale_cache`` / ``value_scale_cache`` float32 [num_blocks, block_size]."""

    def __init__(self, n_heads, head_dim, n_kv_heads, kv_shape, seq_length=-1, compute_dtype=torch.float16,
                 parallel_decoding=False, chunk_prefill=False, device="cuda", granularity="per_channel"):
        super().__init__(n_heads, head_dim, n_kv_heads, (1,) + tuple(kv_shape[1:]), seq_length, compute_dtype,
                         parallel_decoding, chunk_prefill, device)
        if granularity not in ("per_channel", "per_token"):
            raise ValueError(f"kvcache_quant_granularity must be per_channel or per_token, got {granularity!r}")
        self.granularity = granularity
        self.compute_dtype = compute_dtype
        self.register_buffer("key_cache", torch.zeros(kv_shape, dtype=torch.int8, device=device), persistent=False)
        self.register_buffer("value_cache", torch.zeros(kv_shape, dtype=torch.int8, device=device), persistent=False)
        row = n_kv_heads * head_dim
        per_token = granularity == "per_token"
        if per_token and kv_shape[1] % 4:
            raise ValueError(f"per_token int8 caches need a block size that is a multiple of 4, got {kv_shape[1]}")
        self.register_buffer("kv_scale", None if per_token else torch.ones(2, row, dtype=torch.float32, device=device))
        self.register_buffer("kv_offset", None if per_token else torch.zeros(2, row, dtype=torch.float32, device=device))
        for name in ("key_scale_cache", "value_scale_cache"):
            self.register_buffer(name, torch.zeros(kv_shape[:2], dtype=torch.float32, device=device) if per_token else None,
                                 persistent=False)

    @classmethod
    def from_float(cls, mgr, granularity="per_channel"):
        """A quantised manager with the geometry of a float one."""
        kc = mgr.key_cache
        return cls(mgr.n_heads, mgr.head_dim, mgr.n_kv_heads, tuple(kc.shape), mgr.seq_length, kc.dtype,
                   mgr.parallel_decoding, mgr.chunk_prefill, kc.device, granularity=granularity)

    def set_kv_quant(self, scale, offset=None):
        if self.granularity == "per_token":
            raise ValueError("a per_token cache has no loaded parameters: its scales are written with the rows")
        self.kv_scale.copy_(scale.to(torch.float32))
        if offset is None:
            self.kv_offset.zero_()
        else:
            self.kv_offset.copy_(offset.to(torch.float32))
        return self

    def forward(self, key, value, slot_mapping, batch_valid_length=None):
        if self.granularity == "per_token":
            return ops.dynamic_quant_reshape_and_cache(key, value, self.key_cache, self.value_cache,
                                                       self.key_scale_cache, self.value_scale_cache, slot_mapping)
        return ops.quant_reshape_and_cache(key, value, self.key_cache, self.value_cache, slot_mapping, self.kv_scale,
                                           self.kv_offset)

    construct = forward

    def paged_attn(self, query, batch_valid_length, block_tables, attn_mask=None, q_seq_lens=None):
        shape = query.shape
        q2 = query.reshape(-1, self.n_heads * self.head_dim)
        starts = None
        if self.parallel_decoding or self.chunk_prefill:
            if q_seq_lens is None:
                raise ValueError("parallel_decoding / chunk_prefill need q_seq_lens")
            starts = ops.q_starts_from_lens(q_seq_lens)
        out = ops.paged_attention_int8kv(q2, self.key_cache, self.value_cache, block_tables, batch_valid_length,
                                         self.kv_scale, self.kv_offset, self.n_heads, self.n_kv_heads,
                                         self.scale_value, q_starts=starts,
                                         token_scales=(self.key_scale_cache, self.value_scale_cache)
                                         if self.granularity == "per_token" else None)
        return out.reshape(shape)
