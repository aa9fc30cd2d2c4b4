"""One quantized decode layer composed from the oracle's parts.  Test infrastructure only.

Follows the pre-norm residual layer of mindformers/models/llama/llama_transformer.py:1036-1070
(LLamaDecodeLayer.construct) with the attention of :467-569 (use_past branch: q/k/v linears, InferAttention,
wo) and the feed-forward of mindformers/models/llama/llama_layer.py:412-441; equivalently
mindformers/parallel_core/inference/transformer/transformer_layer.py:296-355 with the fused [q|k|v] and
[gate|hidden] layouts of attention.py:344-349 and mlp.py:135-140.

The reference's layer-level test vectors are random placeholders
(tests/st/test_ut/test_parallel_core/test_inference/test_transformer/test_transformer_layer/data_gen_utils.py:43-52),
so the composition itself is pinned only through its separately pinned parts.

Every value a device pipeline writes to memory between kernels is rounded through ``act_dtype`` at the
same point here: norm output, qkv, rotated q/k, attention output, projection output, residual sum,
fc1 output, silu(gate), silu(gate)*hidden, fc2 output, residual sum.
"""
import numpy as np

from .attention import paged_attention_decode, paged_attention_prefill, reshape_and_cache
from .dense import rms_norm, silu
from .numerics import round_to
from .quant import (dequantize_kv_int8, dynamic_quant_per_token, quantize_kv_int8, w8a16_linear,
                    w8a8_linear)
from .rope import apply_rotary_half


def _r(x, dt):
    return round_to(x, dt).astype(np.float64)


def _decode_layer(x, p, cfg, key_cache, value_cache, block_tables, context_lens, slot_mapping, cos, sin,
                  act_dtype, lin, q_seq_lens=None, kv_quant=None):
    n_head, n_kv, d = cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"]
    eps = cfg.get("eps", 1e-5)
    x = np.asarray(x, dtype=np.float64)
    n1 = _r(rms_norm(x, p["attn_norm"], eps), act_dtype)
    qkv = _r(lin(n1, "qkv"), act_dtype)
    q, k, v = np.split(qkv, [n_head * d, (n_head + n_kv) * d], axis=-1)
    q = _r(apply_rotary_half(q, cos, sin, n_head), act_dtype)
    k = _r(apply_rotary_half(k, cos, sin, n_kv), act_dtype)
    if kv_quant is None:
        reshape_and_cache(k.astype(key_cache.dtype), v.astype(value_cache.dtype), key_cache, value_cache, slot_mapping)
    else:
        # int8 caches (updated in place); the attention below sees the dequantised values
        scale, offset = kv_quant
        ko, vo = (None, None) if offset is None else (offset[0], offset[1])
        reshape_and_cache(quantize_kv_int8(k, scale[0], ko), quantize_kv_int8(v, scale[1], vo), key_cache,
                          value_cache, slot_mapping)
        shape = key_cache.shape
        key_cache = dequantize_kv_int8(key_cache.reshape(-1, shape[2] * shape[3]), scale[0], ko).reshape(shape)
        value_cache = dequantize_kv_int8(value_cache.reshape(-1, shape[2] * shape[3]), scale[1], vo).reshape(shape)
    if q_seq_lens is None:
        attn = paged_attention_decode(q, key_cache, value_cache, block_tables, context_lens, n_head, n_kv,
                                      1.0 / np.sqrt(d), prob_dtype=act_dtype)
    else:                                                     # prefill / chunked prefill: several rows per sequence
        attn = paged_attention_prefill(q, key_cache, value_cache, block_tables, context_lens, q_seq_lens, n_head,
                                       n_kv, 1.0 / np.sqrt(d), prob_dtype=act_dtype)
    attn = _r(attn, act_dtype)
    h = _r(x + _r(lin(attn, "wo"), act_dtype), act_dtype)
    n2 = _r(rms_norm(h, p["ffn_norm"], eps), act_dtype)
    gu = _r(lin(n2, "fc1"), act_dtype)
    f = gu.shape[-1] // 2
    a = _r(_r(silu(gu[:, :f]), act_dtype) * gu[:, f:], act_dtype)
    out = _r(h + _r(lin(a, "fc2"), act_dtype), act_dtype)
    return out


def decode_layer_w8a16(x, p, cfg, key_cache, value_cache, block_tables, context_lens, slot_mapping, cos, sin,
                       act_dtype="bf16", q_seq_lens=None, kv_quant=None):
    """p: {name}_w int8 [out,in], {name}_s float32 [out], optional {name}_b for name in qkv, wo, fc1, fc2,
    plus attn_norm / ffn_norm gammas.  Caches are float32 arrays holding storage-dtype values, updated in place.
    ``q_seq_lens``: new tokens per sequence for a prefill / chunked-prefill step (None = one each).
    ``kv_quant`` = (scale [2, n_kv*D], offset or None): the caches are int8 arrays quantised per channel."""
    def lin(a, name):
        return w8a16_linear(a, p[name + "_w"], p[name + "_s"], p.get(name + "_b"))
    return _decode_layer(x, p, cfg, key_cache, value_cache, block_tables, context_lens, slot_mapping, cos, sin,
                         act_dtype, lin, q_seq_lens, kv_quant)


def decode_layer_w8a8(x, p, cfg, key_cache, value_cache, block_tables, context_lens, slot_mapping, cos, sin,
                      act_dtype="bf16"):
    """As above with per-token dynamic int8 activations; p additionally holds {name}_smooth [in]."""
    def lin(a, name):
        q, s = dynamic_quant_per_token(a.astype(np.float32), p.get(name + "_smooth"))
        return w8a8_linear(q, s, p[name + "_w"], p[name + "_s"], p.get(name + "_b"))
    return _decode_layer(x, p, cfg, key_cache, value_cache, block_tables, context_lens, slot_mapping, cos, sin,
                         act_dtype, lin)
