"""Functional wrappers over the C ABI: one Python function per MindSpore primitive on the decode path.

Each wrapper checks shapes, dtypes, contiguity and device on the host (a kernel launched on operands it does
not expect can fault the GPU), allocates the output with torch (device-memory plumbing only) and enqueues
the kernel on torch's current stream.  Nothing is computed in Python.
"""
import math

import torch

from . import _lib
from ._lib import check, dtype_code, ptr, stream_ptr

_ACT = (torch.bfloat16, torch.float16)
_workspaces = {}
_retired = []                                 # outgrown workspaces, kept alive (see workspace())


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def _dev_ok(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        _need(isinstance(t, torch.Tensor) and t.is_cuda, "all tensors must live on the GPU")
        _need(t.is_contiguous(), "all tensors must be contiguous")
        dev = dev or t.device
        _need(t.device == dev, "all tensors must be on the same device")
    return dev


def _rows(t, width, what):
    """A [rows, width] view of ``t`` for the kernels: returns (tensor, row_stride_in_elements).  Accepts any
    contiguous tensor whose element count is a multiple of width, or a 2-D tensor with unit column stride (a
    column slice of a wider buffer, e.g. q/k/v inside a fused projection output)."""
    if t.is_contiguous():
        _need(t.numel() % width == 0, f"{what}: {t.numel()} elements is not a multiple of the row width {width}")
        return t, width
    _need(t.dim() == 2 and t.stride(1) == 1 and t.shape[1] == width and t.stride(0) >= width,
          f"{what}: must be contiguous or a [rows, {width}] column slice with unit column stride")
    return t, t.stride(0)


def _dev_of(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        _need(isinstance(t, torch.Tensor) and t.is_cuda, "all tensors must live on the GPU")
        dev = dev or t.device
        _need(t.device == dev, "all tensors must be on the same device")
    return dev


def workspace(nbytes, device, tag="default"):
    """A cached scratch buffer per (device, stream, purpose), grown on demand and never shrunk.  Two streams never
    share one (their kernels would race on the partial sums), and a buffer that is outgrown is kept alive rather than
    freed: a captured HIP graph may still replay into its address."""
    key = (device, torch.cuda.current_stream(device).cuda_stream, tag)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _retired.append(buf)
        size = max(int(nbytes), 256, 2 * buf.numel() if buf is not None else 0)
        buf = torch.empty(size, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


# --------------------------------------------------------------------------------------------- KV cache
def reshape_and_cache(key, value, key_cache, value_cache, slot_mapping):
    """ReshapeAndCache(key, value, key_cache, value_cache, slot_mapping) -> key.
    key/value [T, n_kv*D] (any leading shape with T rows); caches [num_blocks, block_size, n_kv, D]."""
    lib = _lib.load()
    _dev_of(key, value)
    dev = _dev_ok(key_cache, value_cache, slot_mapping)
    _need(key_cache.dim() == 4, "key_cache must be [num_blocks, block_size, n_kv_heads, head_dim]")
    nb, bs, n_kv, d = key_cache.shape
    key, ks = _rows(key, n_kv * d, "key")
    vs = 0
    if value is not None:
        value, vs = _rows(value, n_kv * d, "value")
    _need(key.dtype in _ACT and key_cache.dtype == key.dtype, "key and key_cache must share a bf16/fp16 dtype")
    _need(slot_mapping.dtype == torch.int32 and slot_mapping.dim() == 1, "slot_mapping must be int32 [T]")
    t = slot_mapping.numel()
    _need(key.numel() == t * n_kv * d, f"key has {key.numel()} elements, expected {t}*{n_kv}*{d}")
    if value is not None:
        _need(value_cache is not None and value_cache.shape == key_cache.shape and value.dtype == key.dtype
              and value_cache.dtype == key.dtype and value.numel() == key.numel(), "value / value_cache mismatch")
    else:
        _need(value_cache is None, "value_cache given without value")
    check(lib.mf_reshape_and_cache(ptr(key), ptr(value), ptr(key_cache), ptr(value_cache), ptr(slot_mapping), t, n_kv,
                                   d, nb * bs, ks, vs, dtype_code(key.dtype), stream_ptr(dev)), "mf_reshape_and_cache")
    return key


def apply_rotary_pos_emb(query, key, cos, sin, n_heads, n_kv_heads, head_dim):
    """ApplyRotaryPosEmb(cos_format=2), in place.  query [T, n_heads*D], key [T, n_kv*D] or None,
    cos/sin [T, D] (one row per token)."""
    lib = _lib.load()
    _dev_of(query, key)
    dev = _dev_ok(cos, sin)
    query, qs = _rows(query, n_heads * head_dim, "query")
    ks = 0
    if key is not None:
        key, ks = _rows(key, n_kv_heads * head_dim, "key")
    t = query.numel() // (n_heads * head_dim)
    _need(query.dtype in _ACT and query.numel() == t * n_heads * head_dim, "query shape/dtype")
    _need(key is None or (key.dtype == query.dtype and key.numel() == t * n_kv_heads * head_dim), "key shape/dtype")
    _need(cos.dtype == sin.dtype and cos.numel() == t * head_dim and sin.numel() == t * head_dim,
          "cos/sin must hold one [head_dim] row per token")
    check(lib.mf_rope_half(ptr(query), ptr(key), ptr(cos), ptr(sin), t, n_heads, n_kv_heads, head_dim, qs, ks,
                           dtype_code(query.dtype), dtype_code(cos.dtype), stream_ptr(dev)), "mf_rope_half")
    return query, key


def rope_and_cache(query, key, value, cos, sin, key_cache, value_cache, slot_mapping, n_heads):
    """RoPE on q/k (in place) then scatter of rotated k and v into the caches, one launch."""
    lib = _lib.load()
    _dev_of(query, key, value)
    dev = _dev_ok(cos, sin, key_cache, value_cache, slot_mapping)
    nb, bs, n_kv, d = key_cache.shape
    t = slot_mapping.numel()
    query, qs = _rows(query, n_heads * d, "query")
    key, ks = _rows(key, n_kv * d, "key")
    value, vs = _rows(value, n_kv * d, "value")
    _need(query.dtype in _ACT and key.dtype == query.dtype and value.dtype == query.dtype
          and key_cache.dtype == query.dtype and value_cache.dtype == query.dtype, "dtype mismatch")
    _need(value_cache.shape == key_cache.shape, "cache shapes differ")
    _need(slot_mapping.dtype == torch.int32, "slot_mapping must be int32")
    _need(query.numel() == t * n_heads * d and key.numel() == t * n_kv * d and value.numel() == t * n_kv * d,
          "q/k/v sizes do not match slot_mapping and the cache geometry")
    _need(cos.dtype == sin.dtype and cos.numel() == t * d and sin.numel() == t * d, "cos/sin must be [T, head_dim]")
    check(lib.mf_rope_and_cache(ptr(query), ptr(key), ptr(value), ptr(cos), ptr(sin), ptr(key_cache),
                                ptr(value_cache), ptr(slot_mapping), t, n_heads, n_kv, d, nb * bs, qs, ks, vs,
                                dtype_code(query.dtype), dtype_code(cos.dtype), stream_ptr(dev)), "mf_rope_and_cache")
    return query, key


# --------------------------------------------------------------------------------------------- attention
def paged_attention(query, key_cache, value_cache, block_tables, context_lens, n_heads, n_kv_heads, scale, out=None,
                    quant=None):
    """PagedAttention(head_num, scale, kv_head_num)(query, key_cache, value_cache, block_tables, context_lens).
    ``quant`` = (smooth or None, tiled): also quantise every output row per token, as ``dynamic_quant`` would; the
    call then returns (out, xq, scale)."""
    lib = _lib.load()
    _dev_of(query)
    dev = _dev_ok(key_cache, value_cache, block_tables, context_lens, out)
    _need(key_cache.dim() == 4 and value_cache.shape == key_cache.shape, "caches must be [blocks, block_size, n_kv, D]")
    nb, bs, n_kv, d = key_cache.shape
    query, qs = _rows(query, n_heads * d, "query")
    _need(n_kv == n_kv_heads, f"cache has {n_kv} kv heads, module says {n_kv_heads}")
    _need(query.dtype in _ACT and key_cache.dtype == query.dtype and value_cache.dtype == query.dtype, "dtype mismatch")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2, "block_tables must be int32 [B, max_blocks]")
    _need(context_lens.dtype == torch.int32 and context_lens.dim() == 1, "context_lens must be int32 [B]")
    b = context_lens.numel()
    _need(block_tables.shape[0] == b, "block_tables rows != batch")
    _need(query.numel() == b * n_heads * d, f"query has {query.numel()} elements, expected {b}*{n_heads}*{d}")
    max_blocks = block_tables.shape[1]
    if out is None:
        out = torch.empty(query.shape, dtype=query.dtype, device=dev)
    else:
        _need(out.shape == query.shape and out.dtype == query.dtype, "out mismatch")
    need = lib.mf_paged_attention_workspace_bytes(b, n_heads, d, max_blocks * bs)
    ws = workspace(need, dev, "pa") if need else None
    if quant is not None:
        smooth, tiled = quant
        cols = n_heads * d
        _need(smooth is None or (smooth.dtype == torch.float32 and smooth.numel() == cols and smooth.device == dev),
              "smooth must be fp32 [n_heads * D]")
        xq, xs = _quant_out(lib, (b, cols), b, cols, tiled, dev)
        check(lib.mf_paged_attention_decode_dynamic_quant(
            ptr(out), ptr(xq), ptr(xs), ptr(smooth), 1 if tiled else 0, ptr(query), ptr(key_cache), ptr(value_cache),
            ptr(block_tables), ptr(context_lens), b, n_heads, n_kv_heads, d, bs, max_blocks, nb, float(scale), qs,
            dtype_code(query.dtype), ptr(ws), ws.numel() if ws is not None else 0, stream_ptr(dev)),
            "mf_paged_attention_decode_dynamic_quant")
        return out, (TiledInt8Activations(xq, (b, cols)) if tiled else xq), xs
    check(lib.mf_paged_attention_decode(ptr(out), ptr(query), ptr(key_cache), ptr(value_cache), ptr(block_tables),
                                        ptr(context_lens), b, n_heads, n_kv_heads, d, bs, max_blocks, nb,
                                        float(scale), qs, dtype_code(query.dtype), ptr(ws), ws.numel() if ws is not None else 0,
                                        stream_ptr(dev)), "mf_paged_attention_decode")
    return out


def _q_starts(q_starts, dev):
    _need(isinstance(q_starts, torch.Tensor) and q_starts.dtype == torch.int32 and q_starts.dim() == 1 and
          q_starts.numel() >= 2, "q_starts must be int32 [batch + 1] (cumulative query-row offsets)")
    _need(q_starts.device == dev and q_starts.is_contiguous(), "q_starts must be a contiguous tensor on the GPU")
    return q_starts.numel() - 1


# --------------------------------------------------------------------------------------------- MLA decode
def mla_paged_attention(query, latent_cache, block_tables, context_lens, n_heads, kv_lora_rank, scale, out=None,
                        q_seq_lens=None):
    """PagedAttention(head_num, scale, 1, mla_v_dim=kv_lora_rank)(query, cache, cache, block_tables, context_lens):
    query [B, n_heads * (kv_lora_rank + rope)], latent cache [num_blocks, block_size, 1, kv_lora_rank + rope];
    returns [B, n_heads * kv_lora_rank].

    ``q_seq_lens`` (int32 [B], several new tokens per sequence, causal among themselves: parallel decoding / chunked
    prefill, flash_attention.py:140-143): query holds sum(q_seq_lens) rows packed sequence after sequence.  Every
    query row is run as a sequence of its own whose context ends at its own position (its block-table row repeated,
    built on the device without a host synchronisation), so the result is exactly the one-query kernel's."""
    if q_seq_lens is not None:
        _need(q_seq_lens.dtype == torch.int32 and q_seq_lens.numel() == context_lens.numel(), "q_seq_lens must be int32 [B]")
        dk = latent_cache.shape[-1]
        rows = query.numel() // (n_heads * dk) if query.is_contiguous() else query.shape[0]
        b = context_lens.numel()
        ql = q_seq_lens.to(torch.int64)
        seq = torch.repeat_interleave(torch.arange(b, device=query.device), ql, output_size=rows)
        first = torch.cumsum(ql, 0) - ql                          # first query row of every sequence
        pos = torch.arange(rows, device=query.device) - first[seq]
        lens = (context_lens.to(torch.int64)[seq] - ql[seq] + pos + 1).clamp(min=0).to(torch.int32)
        return mla_paged_attention(query, latent_cache, block_tables[seq].contiguous(), lens.contiguous(), n_heads,
                                   kv_lora_rank, scale, out=out)
    lib = _lib.load()
    _dev_of(query)
    dev = _dev_ok(latent_cache, block_tables, context_lens, out)
    _need(latent_cache.dim() == 4 and latent_cache.shape[2] == 1, "latent cache must be [blocks, block_size, 1, rank + rope]")
    nb, bs, _, dk = latent_cache.shape
    rope = dk - kv_lora_rank
    query, qs = _rows(query, n_heads * dk, "query")
    _need(query.dtype in _ACT and latent_cache.dtype == query.dtype, "dtype mismatch")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2, "block_tables must be int32 [B, max_blocks]")
    _need(context_lens.dtype == torch.int32 and context_lens.dim() == 1, "context_lens must be int32 [B]")
    b = context_lens.numel()
    _need(block_tables.shape[0] == b, "block_tables rows != batch")
    rows = query.numel() // (n_heads * dk) if query.is_contiguous() else query.shape[0]
    _need(rows == b, f"query has {rows} rows for {b} sequences")
    max_blocks = block_tables.shape[1]
    if out is None:
        out = torch.empty((b, n_heads * kv_lora_rank), dtype=query.dtype, device=dev)
    else:
        _need(out.numel() == b * n_heads * kv_lora_rank and out.dtype == query.dtype, "out mismatch")
    need = lib.mf_mla_paged_attention_workspace_bytes(b, n_heads, max_blocks * bs)
    ws = workspace(need, dev, "mla") if need else None
    check(lib.mf_mla_paged_attention_decode(ptr(out), ptr(query), ptr(latent_cache), ptr(block_tables),
                                            ptr(context_lens), b, n_heads, kv_lora_rank, rope, bs, max_blocks, nb,
                                            float(scale), qs, dtype_code(query.dtype), ptr(ws),
                                            ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_mla_paged_attention_decode")
    return out


def mla_absorb_bmm(x, w, out=None):
    """Per-head projection out[t, h, :] = x[t, h, :] . w[h]^T (multi_latent_attention.py:434-448, :228-231):
    x [T, H, K] and out [T, H, N] may be strided views with a unit last stride (a slice of a wider projection
    output / of the attention query), w [H, N, K] contiguous."""
    lib = _lib.load()
    dev = _dev_of(x, w, out)
    _need(x.dim() == 3 and w.dim() == 3 and w.is_contiguous(), "x must be [T, H, K], w a contiguous [H, N, K]")
    t, h, k = x.shape
    _need(w.shape[0] == h and w.shape[2] == k, f"w is {tuple(w.shape)}, x has {h} heads of {k}")
    n = w.shape[1]
    _need(x.dtype in _ACT and w.dtype == x.dtype, "x and w must be bf16/fp16 and agree")
    _need(x.stride(2) == 1, "x needs a unit last stride")
    if out is None:
        out = torch.empty((t, h, n), dtype=x.dtype, device=dev)
    _need(tuple(out.shape) == (t, h, n) and out.dtype == x.dtype and out.stride(2) == 1, "out must be a [T, H, N] view")
    if t == 0 or h == 0:
        return out
    check(lib.mf_mla_absorb_bmm(ptr(out), ptr(x), ptr(w), t, h, n, k, x.stride(0), x.stride(1), out.stride(0),
                                out.stride(1), dtype_code(x.dtype), stream_ptr(dev)), "mf_mla_absorb_bmm")
    return out


def mla_norm_rope_cache(q, nope, kv, gamma, eps, cos, sin, latent_cache=None, slot_mapping=None, q_rope_out=None,
                        kv_norm_out=None, k_pe_out=None):
    """kv_layernorm + RoPE of the rotary query / key parts + latent-row scatter in one launch
    (multi_latent_attention.py:391-403, :444-447).  q [T, n, nope + rope] dense; kv [T, rank + rope] a view with a unit
    last stride (latent part, then the rotary key part); gamma [rank]; cos / sin [T, rope].  The rotated query parts go
    to ``q_rope_out`` (a [T, n, rope] view, e.g. the tail of the absorbed query) or back in place; the normalised
    latent row and the rotated key part go to the cache row of the token's slot and, when given, to ``kv_norm_out``
    [T, rank] / ``k_pe_out`` [T, rope]."""
    lib = _lib.load()
    dev = _dev_of(q, kv, gamma, cos, sin, latent_cache, slot_mapping, q_rope_out, kv_norm_out, k_pe_out)
    _need(q.dim() == 3 and q.is_contiguous() and q.dtype in _ACT, "q must be a dense bf16/fp16 [T, n, nope + rope]")
    t, n, qd = q.shape
    rope = qd - nope
    _need(kv.dim() == 2 and kv.shape[0] == t and kv.stride(1) == 1 and kv.dtype == q.dtype, "kv must be a [T, rank + rope] view")
    rank = kv.shape[1] - rope
    _need(rank > 0 and gamma.numel() == rank and gamma.is_contiguous(), "gamma must hold kv.shape[1] - rope values")
    _need(cos.shape == (t, rope) and sin.shape == (t, rope) and cos.is_contiguous() and sin.is_contiguous() and
          cos.dtype == sin.dtype, "cos / sin must be contiguous [T, rope]")
    q_rope = q[..., nope:]
    out = q_rope if q_rope_out is None else q_rope_out
    _need(tuple(out.shape) == (t, n, rope) and out.stride(2) == 1 and out.dtype == q.dtype, "q_rope_out must be a [T, n, rope] view")
    for buf, width, name in ((kv_norm_out, rank, "kv_norm_out"), (k_pe_out, rope, "k_pe_out")):
        _need(buf is None or (tuple(buf.shape) == (t, width) and buf.is_contiguous() and buf.dtype == q.dtype),
              f"{name} must be a contiguous [T, {width}]")
    slots = 0
    if latent_cache is not None:
        _need(latent_cache.is_contiguous() and latent_cache.shape[-1] == rank + rope and latent_cache.dtype == q.dtype,
              "latent_cache rows must hold rank + rope values of q's type")
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int32 and slot_mapping.numel() == t,
              "slot_mapping must be int32 [T]")
        slots = latent_cache.numel() // (rank + rope)
    if t == 0:
        return out
    check(lib.mf_mla_norm_rope_cache(ptr(out), out.stride(0), out.stride(1), ptr(q_rope), q_rope.stride(0),
                                     q_rope.stride(1), ptr(kv_norm_out), ptr(k_pe_out), ptr(kv), kv.stride(0), ptr(gamma),
                                     dtype_code(gamma.dtype), float(eps), ptr(cos),
                                     ptr(sin), dtype_code(cos.dtype),
                                     ptr(latent_cache), ptr(slot_mapping), slots, t, n, rank, rope, dtype_code(q.dtype),
                                     stream_ptr(dev)), "mf_mla_norm_rope_cache")
    return out


# --------------------------------------------------------------------------------------------- int8 KV cache
def _kv_quant_params(scale, offset, row, dev):
    _need(isinstance(scale, torch.Tensor) and scale.dtype == torch.float32 and scale.numel() == 2 * row and
          scale.is_contiguous() and scale.device == dev, f"antiquant scale must be float32 [2, {row}] on the GPU")
    _need(offset is None or (offset.dtype == torch.float32 and offset.numel() == 2 * row and offset.is_contiguous()
                             and offset.device == dev), f"antiquant offset must be float32 [2, {row}] on the GPU")


def quant_reshape_and_cache(key, value, key_cache, value_cache, slot_mapping, scale, offset=None):
    """Quantize key / value rows per channel (q = clip(rint(x / scale + offset), -128, 127)) and scatter them into
    the int8 caches [num_blocks, block_size, n_kv, D].  scale / offset: float32 [2, n_kv * D] (keys, values)."""
    lib = _lib.load()
    _dev_of(key, value)
    dev = _dev_ok(key_cache, value_cache, slot_mapping)
    _need(key_cache.dtype == torch.int8 and value_cache.dtype == torch.int8 and key_cache.dim() == 4 and
          value_cache.shape == key_cache.shape, "caches must be int8 [blocks, block_size, n_kv, D]")
    nb, bs, n_kv, d = key_cache.shape
    row = n_kv * d
    key, ks = _rows(key, row, "key")
    value, vs = _rows(value, row, "value")
    _need(key.dtype in _ACT and value.dtype == key.dtype, "key / value must be bf16 or fp16")
    _need(slot_mapping.dtype == torch.int32, "slot_mapping must be int32")
    t = slot_mapping.numel()
    _need(key.numel() // row == t if key.is_contiguous() else key.shape[0] == t, "key rows != slots")
    _kv_quant_params(scale, offset, row, dev)
    check(lib.mf_quant_reshape_and_cache(ptr(key), ptr(value), ptr(key_cache), ptr(value_cache), ptr(slot_mapping),
                                         ptr(scale), ptr(offset), t, n_kv, d, nb * bs, ks, vs, dtype_code(key.dtype),
                                         stream_ptr(dev)), "mf_quant_reshape_and_cache")
    return key


def dynamic_quant_reshape_and_cache(key, value, key_cache, value_cache, key_scale_cache, value_scale_cache, slot_mapping):
    """Quantise key / value rows per token (s = max|row| / 127 over all kv heads of the token, q = clip(rint(x / s),
    -128, 127)) and scatter rows and scales: int8 caches [num_blocks, block_size, n_kv, D], fp32 scale caches
    [num_blocks, block_size]."""
    lib = _lib.load()
    _dev_of(key, value)
    dev = _dev_ok(key_cache, value_cache, key_scale_cache, value_scale_cache, slot_mapping)
    _need(key_cache.dtype == torch.int8 and value_cache.dtype == torch.int8 and key_cache.dim() == 4 and
          value_cache.shape == key_cache.shape, "caches must be int8 [blocks, block_size, n_kv, D]")
    nb, bs, n_kv, d = key_cache.shape
    _token_scale_caches(key_scale_cache, value_scale_cache, nb, bs)
    row = n_kv * d
    key, ks = _rows(key, row, "key")
    value, vs = _rows(value, row, "value")
    _need(key.dtype in _ACT and value.dtype == key.dtype, "key / value must be bf16 or fp16")
    _need(slot_mapping.dtype == torch.int32, "slot_mapping must be int32")
    t = slot_mapping.numel()
    _need(key.numel() // row == t if key.is_contiguous() else key.shape[0] == t, "key rows != slots")
    check(lib.mf_dynamic_quant_reshape_and_cache(ptr(key), ptr(value), ptr(key_cache), ptr(value_cache),
                                                 ptr(key_scale_cache), ptr(value_scale_cache), ptr(slot_mapping), t,
                                                 n_kv, d, nb * bs, ks, vs, dtype_code(key.dtype), stream_ptr(dev)),
          "mf_dynamic_quant_reshape_and_cache")
    return key


def _token_scale_caches(key_scale_cache, value_scale_cache, nb, bs):
    for c in (key_scale_cache, value_scale_cache):
        _need(c is not None and c.dtype == torch.float32 and c.numel() == nb * bs and c.is_contiguous(),
              "per-token scale caches must be contiguous fp32 [num_blocks, block_size]")


def paged_attention_int8kv(query, key_cache, value_cache, block_tables, context_lens, antiquant_scale,
                           antiquant_offset, n_heads, n_kv_heads, scale, q_starts=None, out=None, token_scales=None):
    """PagedAttention(...)(query, key_cache, value_cache, block_tables, context_lens, antiquant_scale,
    antiquant_offset[, mask, q_seq_lens]) on int8 caches; ``q_starts`` selects the several-rows-per-sequence form.
    ``token_scales`` = (key_scale_cache, value_scale_cache), fp32 [num_blocks, block_size]: caches quantised per
    token (``dynamic_quant_reshape_and_cache``); antiquant_scale / antiquant_offset are then None."""
    lib = _lib.load()
    _dev_of(query)
    dev = _dev_ok(key_cache, value_cache, block_tables, context_lens, out)
    _need(key_cache.dtype == torch.int8 and value_cache.dtype == torch.int8 and key_cache.dim() == 4 and
          value_cache.shape == key_cache.shape, "caches must be int8 [blocks, block_size, n_kv, D]")
    nb, bs, n_kv, d = key_cache.shape
    query, qs = _rows(query, n_heads * d, "query")
    _need(n_kv == n_kv_heads and query.dtype in _ACT, "head count / dtype mismatch")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2, "block_tables must be int32 [B, max_blocks]")
    _need(context_lens.dtype == torch.int32 and context_lens.dim() == 1, "context_lens must be int32 [B]")
    if token_scales is not None:
        _need(antiquant_scale is None and antiquant_offset is None, "per-token caches take no per-channel parameters")
        _dev_ok(*token_scales)
        _token_scale_caches(token_scales[0], token_scales[1], nb, bs)
        _need(bs % 4 == 0, "per-token scales need a block size that is a multiple of 4")
    else:
        _kv_quant_params(antiquant_scale, antiquant_offset, n_kv * d, dev)
    b = context_lens.numel()
    _need(block_tables.shape[0] == b, "block_tables rows != batch")
    max_blocks = block_tables.shape[1]
    rows = query.numel() // (n_heads * d) if query.is_contiguous() else query.shape[0]
    if out is None:
        out = torch.empty((rows, n_heads * d), dtype=query.dtype, device=dev)
    else:
        _need(out.numel() == rows * n_heads * d and out.dtype == query.dtype, "out mismatch")
    if q_starts is None:
        _need(rows == b, f"query has {rows} rows for {b} sequences")
        need = lib.mf_paged_attention_workspace_bytes(b, n_heads, d, max_blocks * bs)
        ws = workspace(need, dev, "pa") if need else None
        if token_scales is not None:
            check(lib.mf_paged_attention_decode_int8kv_per_token(
                ptr(out), ptr(query), ptr(key_cache), ptr(value_cache), ptr(token_scales[0]), ptr(token_scales[1]),
                ptr(block_tables), ptr(context_lens), b, n_heads, n_kv_heads, d, bs, max_blocks, nb, float(scale), qs,
                dtype_code(query.dtype), ptr(ws), ws.numel() if ws is not None else 0, stream_ptr(dev)),
                "mf_paged_attention_decode_int8kv_per_token")
            return out
        check(lib.mf_paged_attention_decode_int8kv(ptr(out), ptr(query), ptr(key_cache), ptr(value_cache),
                                                   ptr(block_tables), ptr(context_lens), ptr(antiquant_scale),
                                                   ptr(antiquant_offset), b, n_heads, n_kv_heads, d, bs, max_blocks, nb,
                                                   float(scale), qs, dtype_code(query.dtype), ptr(ws),
                                                   ws.numel() if ws is not None else 0, stream_ptr(dev)),
              "mf_paged_attention_decode_int8kv")
    else:
        _need(_q_starts(q_starts, dev) == b, "q_starts must have batch + 1 entries")
        need = lib.mf_paged_attention_prefill_workspace_bytes(b, rows, n_heads, n_kv_heads, d, max_blocks * bs)
        ws = workspace(need, dev, "pa_prefill") if need else None
        if token_scales is not None:
            check(lib.mf_paged_attention_prefill_int8kv_per_token(
                ptr(out), ptr(query), ptr(key_cache), ptr(value_cache), ptr(token_scales[0]), ptr(token_scales[1]),
                ptr(block_tables), ptr(context_lens), ptr(q_starts), b, rows, n_heads, n_kv_heads, d, bs, max_blocks,
                nb, float(scale), qs, dtype_code(query.dtype), ptr(ws), ws.numel() if ws is not None else 0,
                stream_ptr(dev)), "mf_paged_attention_prefill_int8kv_per_token")
            return out
        check(lib.mf_paged_attention_prefill_int8kv(ptr(out), ptr(query), ptr(key_cache), ptr(value_cache),
                                                    ptr(block_tables), ptr(context_lens), ptr(q_starts),
                                                    ptr(antiquant_scale), ptr(antiquant_offset), b, rows, n_heads,
                                                    n_kv_heads, d, bs, max_blocks, nb, float(scale), qs,
                                                    dtype_code(query.dtype), ptr(ws),
                                                    ws.numel() if ws is not None else 0, stream_ptr(dev)),
              "mf_paged_attention_prefill_int8kv")
    return out


def q_starts_from_ends(ends):
    """int32 [B + 1] row offsets from FlashAttentionScore's actual_seq_qlen (increasing ends, the last = T)."""
    ends = ends.to(torch.int32).reshape(-1)
    return torch.cat([torch.zeros(1, dtype=torch.int32, device=ends.device), ends])


def q_starts_from_actual_seq_len(actual_seq_len, total_rows):
    """Row offsets from the `actual_seq_qlen` a caller hands to FlashAttentionScore in the TH layout.  The operator
    documents increasing row ends whose last value is T; the reference's own callers and unit test pass the
    per-sequence lengths (infer_attention.py:459-461, run_infer_flash_attention.py:110,137-142).  The two readings
    never disagree when both are valid (then all entries but the last are zero), so the list is taken as ends when
    it is non-decreasing and ends at T, and as lengths otherwise.  Decided on the device: no host synchronisation."""
    a = torch.as_tensor(actual_seq_len).reshape(-1).to(torch.int64)
    is_ends = (a[-1] == total_rows) & torch.all(a[1:] >= a[:-1])
    return q_starts_from_ends(torch.where(is_ends, a, torch.cumsum(a, 0)))


def q_starts_from_lens(q_seq_lens):
    """int32 [B + 1] row offsets from PagedAttention's q_seq_lens (new tokens per sequence)."""
    return q_starts_from_ends(torch.cumsum(q_seq_lens.reshape(-1), 0))


def paged_attention_prefill(query, key_cache, value_cache, block_tables, context_lens, q_starts, n_heads,
                            n_kv_heads, scale, out=None):
    """Causal attention of several new tokens per sequence over the paged cache (their keys/values already
    scattered): PagedAttention(...)(query, key_cache, value_cache, block_tables, batch_valid_length, None, None,
    causal_mask, q_seq_lens) with q_starts = [0, cumsum(q_seq_lens)]."""
    lib = _lib.load()
    _dev_of(query)
    dev = _dev_ok(key_cache, value_cache, block_tables, context_lens, out)
    _need(key_cache.dim() == 4 and value_cache.shape == key_cache.shape, "caches must be [blocks, block_size, n_kv, D]")
    nb, bs, n_kv, d = key_cache.shape
    query, qs = _rows(query, n_heads * d, "query")
    _need(n_kv == n_kv_heads, f"cache has {n_kv} kv heads, module says {n_kv_heads}")
    _need(query.dtype in _ACT and key_cache.dtype == query.dtype and value_cache.dtype == query.dtype, "dtype mismatch")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2, "block_tables must be int32 [B, max_blocks]")
    _need(context_lens.dtype == torch.int32 and context_lens.dim() == 1, "context_lens must be int32 [B]")
    b = _q_starts(q_starts, dev)
    _need(context_lens.numel() == b and block_tables.shape[0] == b, "context_lens / block_tables rows != batch")
    total_q = query.numel() // (n_heads * d) if query.is_contiguous() else query.shape[0]
    max_blocks = block_tables.shape[1]
    if out is None:
        out = torch.empty((total_q, n_heads * d), dtype=query.dtype, device=dev)
    else:
        _need(out.numel() == total_q * n_heads * d and out.dtype == query.dtype and out.is_contiguous(), "out mismatch")
    need = lib.mf_paged_attention_prefill_workspace_bytes(b, total_q, n_heads, n_kv_heads, d, max_blocks * bs)
    ws = workspace(need, dev, "pa_prefill") if need else None
    check(lib.mf_paged_attention_prefill(ptr(out), ptr(query), ptr(key_cache), ptr(value_cache), ptr(block_tables),
                                         ptr(context_lens), ptr(q_starts), b, total_q, n_heads, n_kv_heads, d, bs,
                                         max_blocks, nb, float(scale), qs, 0, dtype_code(query.dtype), ptr(ws),
                                         ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_paged_attention_prefill")
    return out


def causal_attention_varlen(query, key, value, q_starts, n_heads, n_kv_heads, scale, out=None):
    """FlashAttentionScore in the TH layout with a causal mask and actual_seq_qlen == actual_seq_kvlen: packed
    rows, sequence b owns rows q_starts[b] .. q_starts[b+1]-1 of query, key and value.  key / value may be column
    slices of a fused projection output (equal row strides).  With 192-wide query / key heads the value heads may be
    128 wide (multi-latent attention): the result then has 128-wide heads, the numbers the 192-wide call gives on
    zero-padded values in its first 128 columns."""
    lib = _lib.load()
    dev = _dev_of(query, key, value)
    _dev_ok(out)
    _need(query.dtype in _ACT and key.dtype == query.dtype and value.dtype == query.dtype, "dtype mismatch")
    _need(query.dim() == 2 and key.dim() == 2 and value.dim() == 2, "query / key / value must be [T, heads * D]")
    _need(n_heads % n_kv_heads == 0 and query.shape[1] % n_heads == 0, "head counts do not divide the row width")
    d = query.shape[1] // n_heads
    query, qs = _rows(query, n_heads * d, "query")
    key, ks = _rows(key, n_kv_heads * d, "key")
    total_q = query.shape[0]
    b = _q_starts(q_starts, dev)
    if value.shape[1] != key.shape[1]:
        # value heads narrower than the key heads: the prefill of multi-latent attention (192-wide keys, 128-wide values)
        _need(d == 192 and value.shape[1] == n_kv_heads * 128, "narrower value heads are built for 192-wide keys with 128-wide values")
        value, vs = _rows(value, n_kv_heads * 128, "value")
        _need(key.shape[0] == total_q and value.shape[0] == total_q, "query, key and value must have the same number of rows")
        if out is None:
            out = torch.empty((total_q, n_heads * 128), dtype=query.dtype, device=dev)
        else:
            _need(out.numel() == total_q * n_heads * 128 and out.dtype == query.dtype and out.is_contiguous(), "out mismatch")
        need = lib.mf_paged_attention_prefill_workspace_bytes(b, total_q, n_heads, n_kv_heads, 128, total_q)
        ws = workspace(need, dev, "pa_prefill") if need else None
        check(lib.mf_causal_attention_qk192_v128(ptr(out), ptr(query), ptr(key), ptr(value), ptr(q_starts), b, total_q,
                                                 n_heads, n_kv_heads, float(scale), qs, ks, vs, dtype_code(query.dtype),
                                                 ptr(ws), ws.numel() if ws is not None else 0, stream_ptr(dev)),
              "mf_causal_attention_qk192_v128")
        return out
    value, vs = _rows(value, n_kv_heads * d, "value")
    _need(ks == vs, "key and value must have the same row stride")
    _need(key.shape[0] == total_q and value.shape[0] == total_q, "query, key and value must have the same number of rows")
    if out is None:
        out = torch.empty((total_q, n_heads * d), dtype=query.dtype, device=dev)
    else:
        _need(out.numel() == total_q * n_heads * d and out.dtype == query.dtype and out.is_contiguous(), "out mismatch")
    need = lib.mf_paged_attention_prefill_workspace_bytes(b, total_q, n_heads, n_kv_heads, d, total_q)
    ws = workspace(need, dev, "pa_prefill") if need else None
    check(lib.mf_paged_attention_prefill(ptr(out), ptr(query), ptr(key), ptr(value), None, None, ptr(q_starts), b,
                                         total_q, n_heads, n_kv_heads, d, 0, 0, 0, float(scale), qs, ks,
                                         dtype_code(query.dtype), ptr(ws), ws.numel() if ws is not None else 0,
                                         stream_ptr(dev)), "mf_paged_attention_prefill")
    return out


def swap_cache(host_cache, device_cache, block_mapping, is_device_to_host):
    """swap_cache(host_cache, device_cache, block_mapping, is_device_to_host) of MindIEModelRunner.swap: copy the
    blocks named by ``block_mapping`` ([n, 2] (source, destination), host integers) between a pinned host cache and
    a device cache with the same per-block shape.  Asynchronous on the current stream."""
    import numpy as np
    lib = _lib.load()
    _need(isinstance(host_cache, torch.Tensor) and not host_cache.is_cuda and host_cache.is_contiguous(),
          "host_cache must be a contiguous CPU tensor")
    _need(host_cache.is_pinned(), "host_cache must be pinned (allocate it with pin_memory=True)")
    dev = _dev_ok(device_cache)
    _need(host_cache.dtype == device_cache.dtype and host_cache.shape[1:] == device_cache.shape[1:],
          "host and device caches must share dtype and per-block shape")
    pairs = np.ascontiguousarray(np.asarray(block_mapping.cpu() if isinstance(block_mapping, torch.Tensor)
                                            else block_mapping, dtype=np.int64).reshape(-1, 2))
    block_bytes = device_cache[0].numel() * device_cache.element_size()
    check(lib.mf_swap_blocks(host_cache.data_ptr(), ptr(device_cache), pairs.ctypes.data, pairs.shape[0], block_bytes,
                             host_cache.shape[0], device_cache.shape[0], int(bool(is_device_to_host)),
                             stream_ptr(dev)), "mf_swap_blocks")


# --------------------------------------------------------------------------------------------- norm / activation
def rms_norm(x, gamma, eps, residual=None):
    """RmsNorm(eps)(x, gamma).  With ``residual``: returns (norm(x + residual), x + residual).  Without it, x may
    be a column slice of a wider 2-D matrix (unit column stride): the rows are read where they lie."""
    lib = _lib.load()
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    cols = x.shape[-1]
    _need(gamma.numel() == cols, "gamma size")
    if residual is None and x.dim() == 2 and not x.is_contiguous() and x.stride(1) == 1 and x.stride(0) % 8 == 0 \
            and x.stride(0) >= cols and x.data_ptr() % 16 == 0:
        dev = _dev_ok(gamma)
        _need(x.is_cuda and x.device == dev, "all tensors must be on the same device")
        y = torch.empty(x.shape, dtype=x.dtype, device=dev)
        check(lib.mf_rmsnorm_strided(ptr(y), ptr(x), x.stride(0), ptr(gamma), float(eps), x.shape[0], cols,
                                     dtype_code(x.dtype), dtype_code(gamma.dtype), stream_ptr(dev)), "mf_rmsnorm_strided")
        return y
    x = x.contiguous()
    dev = _dev_ok(x, gamma, residual)
    rows = x.numel() // cols
    y = torch.empty_like(x)
    s = None
    if residual is not None:
        _need(residual.shape == x.shape and residual.dtype == x.dtype, "residual mismatch")
        s = torch.empty_like(x)
    check(lib.mf_rmsnorm(ptr(y), ptr(s), ptr(x), ptr(residual), ptr(gamma), float(eps), rows, cols,
                         dtype_code(x.dtype), dtype_code(gamma.dtype), stream_ptr(dev)), "mf_rmsnorm")
    return (y, s) if residual is not None else y


def silu_mul(gate_up, interleaved=False):
    """silu(gate) * up over [rows, 2*F] -> [rows, F]; halves layout (mcore) or interleaved (legacy ffn_concat)."""
    lib = _lib.load()
    dev = _dev_ok(gate_up)
    _need(gate_up.dtype in _ACT and gate_up.shape[-1] % 2 == 0, "gate_up must be bf16/fp16 with an even last dim")
    cols = gate_up.shape[-1] // 2
    rows = gate_up.numel() // (2 * cols)
    out = torch.empty(*gate_up.shape[:-1], cols, dtype=gate_up.dtype, device=dev)
    check(lib.mf_silu_mul(ptr(out), ptr(gate_up), rows, cols, 1 if interleaved else 0, dtype_code(gate_up.dtype),
                          stream_ptr(dev)), "mf_silu_mul")
    return out


def scale_columns(x, scale):
    """x * scale[None, :] rounded once (activation multiplier in front of a weight-only GEMM)."""
    lib = _lib.load()
    dev = _dev_ok(x, scale)
    cols = x.shape[-1]
    _need(x.dtype in _ACT and scale.dtype == torch.float32 and scale.numel() == cols, "x bf16/fp16, scale fp32 [cols]")
    out = torch.empty_like(x)
    check(lib.mf_scale_columns(ptr(out), ptr(x), ptr(scale), x.numel() // cols, cols, dtype_code(x.dtype),
                               stream_ptr(dev)), "mf_scale_columns")
    return out


def add(a, b):
    lib = _lib.load()
    dev = _dev_ok(a, b)
    _need(a.shape == b.shape and a.dtype == b.dtype and a.dtype in _ACT, "add operands mismatch")
    out = torch.empty_like(a)
    check(lib.mf_add(ptr(out), ptr(a), ptr(b), a.numel(), dtype_code(a.dtype), stream_ptr(dev)), "mf_add")
    return out


# --------------------------------------------------------------------------------------------- quantized linear
class PackedInt8Weight:
    """An int8 weight [N, K] (or a stack [E, N, K]) in the tiled order the W8A16 kernels stream, plus its
    per-output-channel scales.  Built once with ``pack_w8a16`` after the weights are loaded."""

    def __init__(self, packed, scale, n, k, experts=None, gated=False):
        self.packed, self.scale, self.n, self.k, self.experts = packed, scale, n, k, experts
        self.gated = gated                                    # rows interleaved gate/up for the fused gated GEMM

    @property
    def shape(self):
        return (self.n, self.k) if self.experts is None else (self.experts, self.n, self.k)


def pack_w8a16(w_i8, scale):
    """Pack int8 [N, K] or [E, N, K] (K contiguous) into kernel order.  scale fp32 [N] / [E, N]."""
    lib = _lib.load()
    dev = _dev_ok(w_i8, scale)
    _need(w_i8.dtype == torch.int8 and w_i8.dim() in (2, 3), "weight must be int8 [N, K] or [E, N, K]")
    _need(scale.dtype == torch.float32, "scale must be fp32")
    experts = w_i8.shape[0] if w_i8.dim() == 3 else None
    n, k = w_i8.shape[-2:]
    _need(scale.numel() == (experts or 1) * n, "scale must hold one value per output channel")
    per = lib.mf_w8a16_packed_bytes(n, k)
    packed = torch.empty((experts or 1) * per, dtype=torch.uint8, device=dev)
    mats = w_i8 if experts is not None else w_i8[None]
    for e in range(mats.shape[0]):
        check(lib.mf_w8a16_pack_weight(packed.data_ptr() + e * per, ptr(mats[e]), n, k, stream_ptr(dev)),
              "mf_w8a16_pack_weight")
    return PackedInt8Weight(packed, scale.contiguous(), n, k, experts)


def w8a16_linear(x, w, scale=None, bias=None, residual=None):
    """WeightQuantBatchMatmul: y = (x . w_i8^T) * scale (+bias) (+residual).  x [..., K]; ``w`` is a
    PackedInt8Weight (the fast path) or a raw int8 [N, K] tensor with ``scale`` (packed on every call)."""
    lib = _lib.load()
    if not isinstance(w, PackedInt8Weight):
        w = pack_w8a16(w, scale)
    _need(w.experts is None, "use grouped_w8a16_linear for stacked expert weights")
    _need(not w.gated, "a gate/up weight packed for the fused gated GEMM: use w8a16_gated_linear")
    dev = _dev_ok(x, bias, residual)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    n, k = w.n, w.k
    _need(x.shape[-1] == k, f"x has {x.shape[-1]} input channels, weight expects {k}")
    m = x.numel() // k
    y = torch.empty(*x.shape[:-1], n, dtype=x.dtype, device=dev)
    _need(bias is None or (bias.dtype == x.dtype and bias.numel() == n), "bias mismatch")
    _need(residual is None or (residual.dtype == x.dtype and residual.shape == y.shape), "residual mismatch")
    need = lib.mf_w8a16_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w8a16_gemm(ptr(y), ptr(x), ptr(w.packed), ptr(w.scale), ptr(bias), ptr(residual), m, n, k,
                            dtype_code(x.dtype), ptr(ws), ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_w8a16_gemm")
    return y


class TiledInt8Activations:
    """Per-token quantised activations [M, K] in the 16 x 64 tile order the int8 GEMM streams (the fast path of
    ``w8a8_linear``); ``shape`` is the logical shape of the activation tensor."""

    def __init__(self, data, shape):
        self.data, self.shape = data, tuple(shape)


class PackedInt4Weight:
    """A 4-bit weight [N, K] in the nibble-tile order the A16W4 kernel streams, with its scales: fp32 [N]
    (``group_size`` 0) or [K / group_size, N]."""

    def __init__(self, packed, scale, n, k, group_size):
        self.packed, self.scale, self.n, self.k, self.group_size = packed, scale, n, k, group_size

    @property
    def shape(self):
        return (self.n, self.k)


def unpack_qint4x2(w):
    """int8 [N, K/2] holding two signed 4-bit values per byte (element 2j in the low nibble, 2j + 1 in the high one)
    -> int8 [N, K] of values -8 .. 7.  Data movement only."""
    _need(w.dtype == torch.int8 and w.dim() == 2, "qint4x2 weight must be int8 [N, K/2]")
    lo = (w << 4) >> 4                                            # arithmetic shifts sign-extend the nibbles
    hi = w >> 4
    return torch.stack((lo, hi), dim=-1).reshape(w.shape[0], -1).contiguous()


def pack_w4a16(w_q, scale, group_size=0, qint4x2=False):
    """Pack 4-bit weights for ``w4a16_linear``: ``w_q`` int8 [N, K] holding values -8 .. 7, or with ``qint4x2`` the
    two-per-byte form [N, K/2] (see ``unpack_qint4x2``); scale fp32 [N] or [K / group_size, N]."""
    lib = _lib.load()
    dev = _dev_ok(w_q, scale)
    _need(w_q.dtype == torch.int8 and w_q.dim() == 2, "weight must be int8 [N, K] (values -8..7) or qint4x2 [N, K/2]")
    _need(scale.dtype == torch.float32 and group_size in (0, 64, 128), "scale must be fp32; group_size 0, 64 or 128")
    if qint4x2:
        w_q = unpack_qint4x2(w_q)
    n, k = w_q.shape
    _need(k % 64 == 0 and (group_size == 0 or k % group_size == 0), f"K ({k}) must be a multiple of 64 and of the group size")
    want = (n,) if group_size == 0 else (k // group_size, n)
    _need(tuple(scale.shape) == want, f"scale must be {want}, got {tuple(scale.shape)}")
    _need(group_size == 0 or n % 4 == 0, "N must be a multiple of 4 with per-group scales")
    packed = torch.empty(lib.mf_w4a16_packed_bytes(n, k), dtype=torch.uint8, device=dev)
    check(lib.mf_w4a16_pack_weight(ptr(packed), ptr(w_q.contiguous()), n, k, stream_ptr(dev)), "mf_w4a16_pack_weight")
    return PackedInt4Weight(packed, scale.contiguous(), n, k, group_size)


def w4a16_linear(x, w, bias=None, residual=None):
    """y = x . (w_int4 * scale)^T (+ bias) (+ residual): the A16W4 weight-only GEMM; ``w`` a PackedInt4Weight."""
    lib = _lib.load()
    _need(isinstance(w, PackedInt4Weight), "w must be a PackedInt4Weight (pack_w4a16)")
    dev = _dev_ok(x, bias, residual)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    n, k = w.n, w.k
    _need(x.shape[-1] == k, f"x has {x.shape[-1]} input channels, weight expects {k}")
    m = x.numel() // k
    y = torch.empty(*x.shape[:-1], n, dtype=x.dtype, device=dev)
    _need(bias is None or (bias.dtype == x.dtype and bias.numel() == n), "bias mismatch")
    _need(residual is None or (residual.dtype == x.dtype and residual.shape == y.shape), "residual mismatch")
    need = lib.mf_w4a16_workspace_bytes(m, n, k, w.group_size)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w4a16_gemm(ptr(y), ptr(x), ptr(w.packed), ptr(w.scale), ptr(bias), ptr(residual), m, n, k, w.group_size,
                            dtype_code(x.dtype), ptr(ws), ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_w4a16_gemm")
    return y


def w8a16_linear_add_rmsnorm(x, w, residual, gamma, eps, bias=None):
    """Row-parallel projection + residual add + the RMSNorm that follows: returns (h, norm(h) * gamma) with
    h = (x . w^T) * scale (+bias) + residual.  Bit-identical to w8a16_linear(residual=...) followed by rms_norm."""
    lib = _lib.load()
    _need(isinstance(w, PackedInt8Weight) and w.experts is None and not w.gated, "w must be a packed [N, K] weight")
    dev = _dev_ok(x, bias, residual, gamma)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    n, k = w.n, w.k
    _need(x.shape[-1] == k, f"x has {x.shape[-1]} input channels, weight expects {k}")
    m = x.numel() // k
    h = torch.empty(*x.shape[:-1], n, dtype=x.dtype, device=dev)
    y = torch.empty_like(h)
    _need(bias is None or (bias.dtype == x.dtype and bias.numel() == n), "bias mismatch")
    _need(residual.dtype == x.dtype and residual.shape == h.shape and residual.is_contiguous(), "residual mismatch")
    _need(gamma.numel() == n, "gamma size")
    need = lib.mf_w8a16_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w8a16_gemm_add_rmsnorm(ptr(y), ptr(h), ptr(x), ptr(w.packed), ptr(w.scale), ptr(bias), ptr(residual),
                                        ptr(gamma), float(eps), m, n, k, dtype_code(x.dtype), dtype_code(gamma.dtype),
                                        ptr(ws), ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_w8a16_gemm_add_rmsnorm")
    return h, y


def w8a16_linear_rmsnorm_leading(x, w, gamma, eps, bias=None):
    """A projection whose leading ``gamma.numel()`` columns feed an RMSNorm (the fused query / latent down projection
    of multi-latent attention with its q_layernorm): returns (h, norm(h[:, :c]) * gamma) with h = (x . w^T) * scale
    (+bias).  Bit-identical to w8a16_linear followed by rms_norm on the column slice."""
    lib = _lib.load()
    _need(isinstance(w, PackedInt8Weight) and w.experts is None and not w.gated, "w must be a packed [N, K] weight")
    dev = _dev_ok(x, bias, gamma)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    n, k, c = w.n, w.k, gamma.numel()
    _need(x.shape[-1] == k, f"x has {x.shape[-1]} input channels, weight expects {k}")
    _need(0 < c <= n and c % 8 == 0 and n % 8 == 0, "the normed columns must be a multiple of 8 within the output")
    m = x.numel() // k
    h = torch.empty(m, n, dtype=x.dtype, device=dev)
    y = torch.empty(m, c, dtype=x.dtype, device=dev)
    _need(bias is None or (bias.dtype == x.dtype and bias.numel() == n), "bias mismatch")
    need = lib.mf_w8a16_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w8a16_gemm_rmsnorm_leading(ptr(y), ptr(h), ptr(x), ptr(w.packed), ptr(w.scale), ptr(bias), ptr(gamma),
                                            float(eps), m, n, k, c, dtype_code(x.dtype), dtype_code(gamma.dtype),
                                            ptr(ws), ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_w8a16_gemm_rmsnorm_leading")
    return h, y


def w8a16_qkv_rope_and_cache(x, w, cos, sin, key_cache, value_cache, slot_mapping, n_heads, bias=None,
                             kv_scale=None, kv_offset=None):
    """Fused QKV projection + RoPE + cache scatter.  Returns the rotated query as a [T, n_heads * D] column view of
    the projection buffer (row stride = full QKV width), ready for ``paged_attention``; the caches receive the
    rotated key rows and the value rows.  int8 caches take ``kv_scale`` (and optionally ``kv_offset``), float32
    [2, n_kv * D] as ``quant_reshape_and_cache`` does, and receive the quantised rows."""
    lib = _lib.load()
    _need(isinstance(w, PackedInt8Weight) and w.experts is None and not w.gated, "w must be a packed [N, K] weight")
    dev = _dev_ok(x, bias, cos, sin, key_cache, value_cache, slot_mapping)
    kv8 = key_cache.dtype == torch.int8
    _need(x.dtype in _ACT and value_cache.dtype == key_cache.dtype and (kv8 or key_cache.dtype == x.dtype),
          "dtype mismatch")
    _need(kv8 == (kv_scale is not None), "kv_scale goes with int8 caches")
    nb, bs, n_kv, d = key_cache.shape
    _need(value_cache.shape == key_cache.shape, "cache shapes differ")
    n, k = w.n, w.k
    _need(n == (n_heads + 2 * n_kv) * d, "weight rows do not match the head geometry")
    _need(x.shape[-1] == k, f"x has {x.shape[-1]} input channels, weight expects {k}")
    m = x.numel() // k
    _need(slot_mapping.dtype == torch.int32 and slot_mapping.numel() == m, "slot_mapping must be int32 [T]")
    _need(cos.dtype == sin.dtype and cos.numel() == m * d and sin.numel() == m * d, "cos/sin must be [T, head_dim]")
    _need(bias is None or (bias.dtype == x.dtype and bias.numel() == n), "bias mismatch")
    qkv = torch.empty(m, n, dtype=x.dtype, device=dev)
    need = lib.mf_w8a16_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    if kv8:
        _kv_quant_params(kv_scale, kv_offset, n_kv * d, dev)
        check(lib.mf_w8a16_qkv_rope_and_quant_cache(ptr(qkv), ptr(x), ptr(w.packed), ptr(w.scale), ptr(bias), ptr(cos),
                                                    ptr(sin), ptr(key_cache), ptr(value_cache), ptr(slot_mapping),
                                                    ptr(kv_scale), ptr(kv_offset), m, n_heads, n_kv, d, nb * bs, k,
                                                    dtype_code(x.dtype), dtype_code(cos.dtype), ptr(ws),
                                                    ws.numel() if ws is not None else 0, stream_ptr(dev)),
              "mf_w8a16_qkv_rope_and_quant_cache")
        return qkv[:, :n_heads * d]
    check(lib.mf_w8a16_qkv_rope_and_cache(ptr(qkv), ptr(x), ptr(w.packed), ptr(w.scale), ptr(bias), ptr(cos), ptr(sin),
                                          ptr(key_cache), ptr(value_cache), ptr(slot_mapping), m, n_heads, n_kv, d,
                                          nb * bs, k, dtype_code(x.dtype), dtype_code(cos.dtype), ptr(ws),
                                          ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_w8a16_qkv_rope_and_cache")
    return qkv[:, :n_heads * d]


def interleave_gate_up(t, layout="halves", dim=0):
    """Entries along ``dim`` of a gate/up projection parameter in the interleaved order the fused gated GEMM wants
    (entry 2j = gate channel j, entry 2j+1 = up channel j).  ``layout``: "halves" = [gate | up] contiguous halves (the
    mcore MLP, parallel_core/inference/transformer/mlp.py:136-140), "interleaved" = already in that order (legacy
    ffn_concat, mindformers/models/llama/llama_layer.py:419-423)."""
    if layout == "interleaved":
        return t.contiguous()
    _need(layout == "halves", "layout must be 'halves' or 'interleaved'")
    dim = dim % t.dim()
    f = t.shape[dim] // 2
    gate, up = t.narrow(dim, 0, f), t.narrow(dim, f, f)
    return torch.stack((gate, up), dim=dim + 1).reshape(t.shape).contiguous()


def pack_w8a16_gated(w_i8, scale, layout="halves"):
    """Pack a gate/up projection weight [2F, K] or a stack of experts [E, 2F, K] (+ scale [2F] / [E, 2F]) for
    ``w8a16_gated_linear`` / the gated form of ``grouped_w8a16_linear``."""
    _need(w_i8.dim() in (2, 3) and w_i8.shape[-2] % 2 == 0, "gate/up weight must be [2F, K] or [E, 2F, K]")
    w = pack_w8a16(interleave_gate_up(w_i8, layout, dim=-2), interleave_gate_up(scale, layout, dim=-1))
    w.gated = True
    return w


def w8a16_gated_linear(x, w, bias=None):
    """Gate/up projection fused with SiLU(gate) * up: x [..., K] -> [..., F].  ``w`` from ``pack_w8a16_gated``;
    ``bias`` [2F] in the same interleaved order.  Bit-identical to w8a16_linear followed by silu_mul."""
    lib = _lib.load()
    _need(isinstance(w, PackedInt8Weight) and w.gated and w.experts is None, "w must come from pack_w8a16_gated")
    dev = _dev_ok(x, bias)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    n, k = w.n, w.k
    _need(x.shape[-1] == k, f"x has {x.shape[-1]} input channels, weight expects {k}")
    m = x.numel() // k
    y = torch.empty(*x.shape[:-1], n // 2, dtype=x.dtype, device=dev)
    _need(bias is None or (bias.dtype == x.dtype and bias.numel() == n), "bias mismatch")
    need = lib.mf_w8a16_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w8a16_gemm_silu_mul(ptr(y), ptr(x), ptr(w.packed), ptr(w.scale), ptr(bias), m, n, k,
                                     dtype_code(x.dtype), ptr(ws), ws.numel() if ws is not None else 0,
                                     stream_ptr(dev)), "mf_w8a16_gemm_silu_mul")
    return y


def _expert_smooth_ok(smooth, offsets, k):
    _need(smooth is not None and smooth.dtype == torch.float32 and smooth.dim() == 2 and smooth.shape[1] == k
          and smooth.is_contiguous(), "with offsets, smooth must be contiguous fp32 [E, K]")
    _need(offsets.dtype == torch.int32 and offsets.numel() == smooth.shape[0] + 1, "offsets must be int32 [E + 1]")
    return smooth.shape[0]


def dynamic_quant(x, smooth=None, tiled=False, offsets=None):
    """DynamicQuant per token (with the smoothing vector folded in): returns (xq, scale fp32 [rows]); xq is int8
    [..., K] row-major, or with ``tiled`` a TiledInt8Activations for ``w8a8_linear``.  With ``offsets`` (int32
    [E + 1], the row groups of moe_permute) ``smooth`` is [E, K], one multiplier vector per expert."""
    lib = _lib.load()
    dev = _dev_ok(x, smooth, offsets)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    k = x.shape[-1]
    m = x.numel() // k
    if offsets is not None:
        e = _expert_smooth_ok(smooth, offsets, k)
        xq, xs = _quant_out(lib, x.shape, m, k, tiled, dev)
        check(lib.mf_grouped_dynamic_quant_per_token(ptr(xq), ptr(xs), ptr(x), ptr(smooth), ptr(offsets), e, m, k,
                                                     dtype_code(x.dtype), 1 if tiled else 0, stream_ptr(dev)),
              "mf_grouped_dynamic_quant_per_token")
        return (TiledInt8Activations(xq, x.shape) if tiled else xq), xs
    _need(smooth is None or (smooth.dtype == torch.float32 and smooth.numel() == k), "smooth must be fp32 [K]")
    if tiled:
        xq = torch.empty(lib.mf_w8a16_packed_bytes(max(m, 1), k), dtype=torch.int8, device=dev)
    else:
        xq = torch.empty(x.shape, dtype=torch.int8, device=dev)
    xs = torch.empty(m, dtype=torch.float32, device=dev)
    check(lib.mf_dynamic_quant_per_token(ptr(xq), ptr(xs), ptr(x), ptr(smooth), m, k, dtype_code(x.dtype),
                                         1 if tiled else 0, stream_ptr(dev)), "mf_dynamic_quant_per_token")
    return (TiledInt8Activations(xq, x.shape) if tiled else xq), xs


def static_quant(x, act_scale, smooth=None, tiled=False):
    """Static per-tensor int8 quantisation (the SmoothQuant method's activation quantiser): q = clip(rint(x * smooth /
    act_scale), -128, 127) with ``act_scale`` a one-element fp32 tensor on the device.  Returns (xq, scale fp32
    [rows], every entry = act_scale) in the forms ``dynamic_quant`` returns, ready for ``w8a8_linear``."""
    lib = _lib.load()
    dev = _dev_ok(x, smooth, act_scale)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    _need(act_scale.dtype == torch.float32 and act_scale.numel() == 1, "act_scale must be one fp32 value")
    k = x.shape[-1]
    m = x.numel() // k
    _need(smooth is None or (smooth.dtype == torch.float32 and smooth.numel() == k), "smooth must be fp32 [K]")
    xq, xs = _quant_out(lib, x.shape, m, k, tiled, dev)
    check(lib.mf_static_quant_per_tensor(ptr(xq), ptr(xs), ptr(x), ptr(smooth), ptr(act_scale), m, k,
                                         dtype_code(x.dtype), 1 if tiled else 0, stream_ptr(dev)),
          "mf_static_quant_per_tensor")
    return (TiledInt8Activations(xq, x.shape) if tiled else xq), xs


def _quant_out(lib, shape, m, k, tiled, dev):
    if tiled:
        xq = torch.empty(lib.mf_w8a16_packed_bytes(max(m, 1), k), dtype=torch.int8, device=dev)
    else:
        xq = torch.empty(shape, dtype=torch.int8, device=dev)
    return xq, torch.empty(m, dtype=torch.float32, device=dev)


def rms_norm_dynamic_quant(x, gamma, eps, smooth=None, residual=None, tiled=False):
    """RmsNorm followed by DynamicQuant per token in one kernel (the norm output itself is not materialised).
    Returns (xq, scale), with ``residual`` also x + residual: bit-identical to rms_norm then dynamic_quant."""
    lib = _lib.load()
    dev = _dev_ok(x, gamma, residual, smooth)
    _need(x.dtype in _ACT, "x must be bf16/fp16")
    k = x.shape[-1]
    m = x.numel() // k
    _need(gamma.numel() == k, "gamma size")
    _need(smooth is None or (smooth.dtype == torch.float32 and smooth.numel() == k), "smooth must be fp32 [K]")
    s = None
    if residual is not None:
        _need(residual.shape == x.shape and residual.dtype == x.dtype, "residual mismatch")
        s = torch.empty_like(x)
    xq, xs = _quant_out(lib, x.shape, m, k, tiled, dev)
    check(lib.mf_rmsnorm_dynamic_quant(ptr(xq), ptr(xs), ptr(s), ptr(x), ptr(residual), ptr(gamma), ptr(smooth),
                                       float(eps), m, k, dtype_code(x.dtype), dtype_code(gamma.dtype),
                                       1 if tiled else 0, stream_ptr(dev)), "mf_rmsnorm_dynamic_quant")
    xq = TiledInt8Activations(xq, x.shape) if tiled else xq
    return (xq, xs, s) if residual is not None else (xq, xs)


def silu_mul_dynamic_quant(gate_up, smooth=None, interleaved=False, tiled=False, offsets=None):
    """silu(gate) * up followed by DynamicQuant per token in one kernel (the product is not materialised): returns
    (xq, scale), bit-identical to silu_mul then dynamic_quant (``offsets``: as there)."""
    lib = _lib.load()
    dev = _dev_ok(gate_up, smooth, offsets)
    _need(gate_up.dtype in _ACT and gate_up.shape[-1] % 2 == 0, "gate_up must be bf16/fp16 with an even last dim")
    k = gate_up.shape[-1] // 2
    m = gate_up.numel() // (2 * k)
    shape = (*gate_up.shape[:-1], k)
    xq, xs = _quant_out(lib, shape, m, k, tiled, dev)
    if offsets is not None:
        e = _expert_smooth_ok(smooth, offsets, k)
        check(lib.mf_grouped_silu_mul_dynamic_quant(ptr(xq), ptr(xs), ptr(gate_up), ptr(smooth), ptr(offsets), e, m, k,
                                                    1 if interleaved else 0, dtype_code(gate_up.dtype),
                                                    1 if tiled else 0, stream_ptr(dev)),
              "mf_grouped_silu_mul_dynamic_quant")
        return (TiledInt8Activations(xq, shape) if tiled else xq), xs
    _need(smooth is None or (smooth.dtype == torch.float32 and smooth.numel() == k), "smooth must be fp32 [F]")
    check(lib.mf_silu_mul_dynamic_quant(ptr(xq), ptr(xs), ptr(gate_up), ptr(smooth), m, k, 1 if interleaved else 0,
                                        dtype_code(gate_up.dtype), 1 if tiled else 0, stream_ptr(dev)),
          "mf_silu_mul_dynamic_quant")
    return (TiledInt8Activations(xq, shape) if tiled else xq), xs


def w8a8_linear(xq, x_scale, w, w_scale=None, out_dtype=torch.bfloat16, bias=None, residual=None, return_acc=False):
    """QuantBatchMatmul: int8 x int8 -> int32 -> * x_scale * w_scale (+bias) (+residual) -> out_dtype.  ``w`` is a
    PackedInt8Weight (the fast path) or a raw int8 [N, K] tensor with ``w_scale`` (packed on every call); ``xq`` is
    an int8 [..., K] tensor or the TiledInt8Activations of ``dynamic_quant(..., tiled=True)`` (the fast path)."""
    lib = _lib.load()
    if not isinstance(w, PackedInt8Weight):
        w = pack_w8a16(w, w_scale)
    _need(w.experts is None, "stacked expert weights are not supported by the int8 GEMM")
    tiled = isinstance(xq, TiledInt8Activations)
    xshape = xq.shape
    xdata = xq.data if tiled else xq
    dev = _dev_ok(xdata, x_scale, bias, residual)
    _need(xdata.dtype == torch.int8, "xq must be int8")
    _need(x_scale.dtype == torch.float32, "scales must be fp32")
    _need(out_dtype in _ACT, "out_dtype must be bf16/fp16")
    n, k = w.n, w.k
    _need(xshape[-1] == k, "shape mismatch")
    m = 1
    for d in xshape[:-1]:
        m *= d
    _need(x_scale.numel() == m, "x_scale must hold one scale per row")
    y = torch.empty(*xshape[:-1], n, dtype=out_dtype, device=dev)
    _need(bias is None or (bias.dtype == out_dtype and bias.numel() == n), "bias mismatch")
    _need(residual is None or (residual.dtype == out_dtype and residual.shape == y.shape), "residual mismatch")
    acc = torch.empty(*xshape[:-1], n, dtype=torch.int32, device=dev) if return_acc else None
    need = lib.mf_w8a8_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w8a8_gemm(ptr(y), ptr(acc), ptr(xdata), ptr(x_scale), ptr(w.packed), ptr(w.scale), ptr(bias),
                           ptr(residual), m, n, k, dtype_code(out_dtype), 1 if tiled else 0, ptr(ws),
                           ws.numel() if ws is not None else 0, stream_ptr(dev)), "mf_w8a8_gemm")
    return (y, acc) if return_acc else y


def _w8a8_operands(lib, xq, x_scale, w, what):
    _need(isinstance(w, PackedInt8Weight) and w.experts is None and not w.gated, "w must be a packed [N, K] weight")
    tiled = isinstance(xq, TiledInt8Activations)
    xshape = xq.shape
    xdata = xq.data if tiled else xq
    _need(xdata.dtype == torch.int8 and x_scale.dtype == torch.float32, f"{what}: xq must be int8, scales fp32")
    _need(xshape[-1] == w.k, "shape mismatch")
    m = 1
    for d in xshape[:-1]:
        m *= d
    _need(x_scale.numel() == m, "x_scale must hold one scale per row")
    return tiled, xshape, xdata, m


def w8a8_linear_add_rmsnorm_quant(xq, x_scale, w, residual, gamma, eps, smooth=None, bias=None, tiled_out=True):
    """Row-parallel W8A8 projection + residual add + the RMSNorm and per-token quantisation that feed the next
    quantised projection: returns (h, xq_next, scale_next) with h = x . w^T dequantised (+bias) + residual.
    Bit-identical to w8a8_linear(residual=...) followed by rms_norm_dynamic_quant."""
    lib = _lib.load()
    tiled, xshape, xdata, m = _w8a8_operands(lib, xq, x_scale, w, "w8a8_linear_add_rmsnorm_quant")
    dev = _dev_ok(xdata, x_scale, bias, residual, gamma, smooth)
    n, k = w.n, w.k
    _need(residual.dtype in _ACT and residual.is_contiguous() and residual.numel() == m * n, "residual mismatch")
    dt = residual.dtype
    _need(bias is None or (bias.dtype == dt and bias.numel() == n), "bias mismatch")
    _need(gamma.numel() == n, "gamma size")
    _need(smooth is None or (smooth.dtype == torch.float32 and smooth.numel() == n), "smooth must be fp32 [N]")
    h = torch.empty_like(residual)
    xq_out, xs_out = _quant_out(lib, h.shape, m, n, tiled_out, dev)
    need = lib.mf_w8a8_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w8a8_gemm_add_rmsnorm_quant(ptr(xq_out), ptr(xs_out), ptr(h), ptr(xdata), ptr(x_scale), ptr(w.packed),
                                             ptr(w.scale), ptr(bias), ptr(residual), ptr(gamma), ptr(smooth),
                                             float(eps), m, n, k, dtype_code(dt), dtype_code(gamma.dtype),
                                             1 if tiled else 0, 1 if tiled_out else 0, ptr(ws),
                                             ws.numel() if ws is not None else 0, stream_ptr(dev)),
          "mf_w8a8_gemm_add_rmsnorm_quant")
    return h, (TiledInt8Activations(xq_out, h.shape) if tiled_out else xq_out), xs_out


def w8a8_qkv_rope_and_cache(xq, x_scale, w, cos, sin, key_cache, value_cache, slot_mapping, n_heads, bias=None):
    """Fused W8A8 QKV projection + RoPE + cache scatter; returns the rotated query as a [T, n_heads * D] column view
    of the projection buffer, as w8a16_qkv_rope_and_cache does."""
    lib = _lib.load()
    tiled, xshape, xdata, m = _w8a8_operands(lib, xq, x_scale, w, "w8a8_qkv_rope_and_cache")
    dev = _dev_ok(xdata, x_scale, bias, cos, sin, key_cache, value_cache, slot_mapping)
    dt = key_cache.dtype
    _need(dt in _ACT and value_cache.dtype == dt, "caches must be bf16/fp16")
    nb, bs, n_kv, d = key_cache.shape
    _need(value_cache.shape == key_cache.shape, "cache shapes differ")
    n, k = w.n, w.k
    _need(n == (n_heads + 2 * n_kv) * d, "weight rows do not match the head geometry")
    _need(slot_mapping.dtype == torch.int32 and slot_mapping.numel() == m, "slot_mapping must be int32 [T]")
    _need(cos.dtype == sin.dtype and cos.numel() == m * d and sin.numel() == m * d, "cos/sin must be [T, head_dim]")
    _need(bias is None or (bias.dtype == dt and bias.numel() == n), "bias mismatch")
    qkv = torch.empty(m, n, dtype=dt, device=dev)
    need = lib.mf_w8a8_workspace_bytes(m, n, k)
    ws = workspace(need, dev, "gemm") if need else None
    check(lib.mf_w8a8_qkv_rope_and_cache(ptr(qkv), ptr(xdata), ptr(x_scale), ptr(w.packed), ptr(w.scale), ptr(bias),
                                         ptr(cos), ptr(sin), ptr(key_cache), ptr(value_cache), ptr(slot_mapping), m,
                                         n_heads, n_kv, d, nb * bs, k, dtype_code(dt), dtype_code(cos.dtype),
                                         1 if tiled else 0, ptr(ws), ws.numel() if ws is not None else 0,
                                         stream_ptr(dev)), "mf_w8a8_qkv_rope_and_cache")
    return qkv[:, :n_heads * d]


# --------------------------------------------------------------------------------------------- MoE
def router_gate(x, weight):
    """The router's dense projection: fp32 logits [T, E] = x . weight^T.  weight [E, H] fp32 (fp32 products and sums)
    or of x's 16-bit type (the projection output is then rounded to that type, as a 16-bit dense cell returns it)."""
    lib = _lib.load()
    dev = _dev_ok(x, weight)
    _need(x.dtype in _ACT and x.dim() == 2 and x.is_contiguous(), "x must be contiguous bf16/fp16 [T, H]")
    _need(weight.dim() == 2 and weight.shape[1] == x.shape[1] and weight.is_contiguous()
          and weight.dtype in (torch.float32, x.dtype), "weight must be contiguous [E, H], fp32 or of x's type")
    t, h = x.shape
    e = weight.shape[0]
    logits = torch.empty(t, e, dtype=torch.float32, device=dev)
    need = lib.mf_router_gate_workspace_bytes(t, e, h)
    ws = workspace(need, dev, "gemm") if need else None
    w_code = 2 if weight.dtype == torch.float32 else dtype_code(weight.dtype)
    check(lib.mf_router_gate_gemm(ptr(logits), ptr(x), ptr(weight), t, e, h, dtype_code(x.dtype), w_code, ptr(ws),
                                  ws.numel() if ws is not None else 0, stream_ptr(dev)), "mf_router_gate_gemm")
    return logits


def moe_route(logits, expert_bias, k, n_group, topk_group, scale, out_dtype, renorm=True, biased_weights=False):
    """FusedAddTopKDiv: (expert_weight [T,k] out_dtype, expert_index [T,k] int32) from fp32 logits [T,E]."""
    lib = _lib.load()
    dev = _dev_ok(logits, expert_bias)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be fp32 [T, E]")
    t, e = logits.shape
    _need(expert_bias is None or (expert_bias.dtype == torch.float32 and expert_bias.numel() == e), "bias must be fp32 [E]")
    w = torch.empty(t, k, dtype=out_dtype, device=dev)
    idx = torch.empty(t, k, dtype=torch.int32, device=dev)
    check(lib.mf_moe_route(ptr(w), ptr(idx), ptr(logits), ptr(expert_bias), t, e, k, int(n_group or 0),
                           int(topk_group or 0), float(scale), 1 if renorm else 0, 1 if biased_weights else 0,
                           dtype_code(out_dtype),
                           stream_ptr(dev)), "mf_moe_route")
    return w, idx


def moe_permute(x, expert_index, n_experts):
    """MoeInitRoutingV2: returns (permuted_x [T*k,H], row_map int32 [T*k], counts int64 [E], offsets int32 [E+1])."""
    lib = _lib.load()
    dev = _dev_ok(x, expert_index)
    _need(x.dtype in _ACT and x.dim() == 2, "x must be bf16/fp16 [T, H]")
    _need(expert_index.dtype == torch.int32 and expert_index.dim() == 2 and expert_index.shape[0] == x.shape[0],
          "expert_index must be int32 [T, k]")
    t, h = x.shape
    k = expert_index.shape[1]
    px = torch.empty(t * k, h, dtype=x.dtype, device=dev)
    row_map = torch.empty(t * k, dtype=torch.int32, device=dev)
    counts = torch.empty(n_experts, dtype=torch.int64, device=dev)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    check(lib.mf_moe_permute(ptr(px), ptr(row_map), ptr(counts), ptr(offsets), ptr(x), ptr(expert_index), t, k,
                             n_experts, h, dtype_code(x.dtype), stream_ptr(dev)), "mf_moe_permute")
    return px, row_map, counts, offsets


def grouped_w8a16_linear(x, w, offsets, scale=None):
    """GroupedMatmulV4 over expert row groups.  x [R, K]; ``w`` a PackedInt8Weight of [E, N, K] (or a raw int8
    [E, N, K] tensor with ``scale`` [E, N], packed on every call); offsets int32 [E+1].  A weight packed with
    ``pack_w8a16_gated`` runs with silu(gate) * up in the epilogue and returns [R, N/2]."""
    lib = _lib.load()
    if not isinstance(w, PackedInt8Weight):
        w = pack_w8a16(w, scale)
    _need(w.experts is not None, "grouped_w8a16_linear needs stacked expert weights [E, N, K]")
    dev = _dev_ok(x, offsets)
    e, n, k = w.experts, w.n, w.k
    _need(x.dtype in _ACT and x.dim() == 2 and x.shape[1] == k, "x must be bf16/fp16 [R, K]")
    _need(offsets.dtype == torch.int32 and offsets.numel() == e + 1, "offsets must be int32 [E+1]")
    y = torch.empty(x.shape[0], n // 2 if w.gated else n, dtype=x.dtype, device=dev)
    fn = lib.mf_grouped_w8a16_gemm_silu_mul if w.gated else lib.mf_grouped_w8a16_gemm
    check(fn(ptr(y), ptr(x), ptr(w.packed), ptr(w.scale), ptr(offsets), e, x.shape[0], n, k, dtype_code(x.dtype),
             stream_ptr(dev)), "mf_grouped_w8a16_gemm")
    return y


def grouped_w8a8_linear(xq, x_scale, w, offsets, out_dtype=torch.bfloat16, return_acc=False):
    """GroupedMatmulV4 on int8 operands: xq int8 [R, K] row-major with per-row scales (``dynamic_quant`` of the permuted
    rows), ``w`` a PackedInt8Weight of [E, N, K], offsets int32 [E+1].  Exact int32 accumulators, dequantised to
    out_dtype; with ``return_acc`` also the int32 [R, N] accumulators."""
    lib = _lib.load()
    _need(isinstance(w, PackedInt8Weight) and w.experts is not None and not w.gated,
          "grouped_w8a8_linear needs stacked expert weights [E, N, K] (not gated)")
    dev = _dev_ok(xq, x_scale, offsets)
    e, n, k = w.experts, w.n, w.k
    _need(xq.dtype == torch.int8 and xq.dim() == 2 and xq.shape[1] == k, "xq must be int8 [R, K]")
    _need(x_scale.dtype == torch.float32 and x_scale.numel() == xq.shape[0], "x_scale must be fp32 [R]")
    _need(offsets.dtype == torch.int32 and offsets.numel() == e + 1, "offsets must be int32 [E+1]")
    _need(out_dtype in _ACT, "out_dtype must be bf16/fp16")
    y = torch.empty(xq.shape[0], n, dtype=out_dtype, device=dev)
    acc = torch.empty(xq.shape[0], n, dtype=torch.int32, device=dev) if return_acc else None
    check(lib.mf_grouped_w8a8_gemm(ptr(y), ptr(acc), ptr(xq), ptr(x_scale), ptr(w.packed), ptr(w.scale), ptr(offsets), e,
                                   xq.shape[0], n, k, dtype_code(out_dtype), stream_ptr(dev)), "mf_grouped_w8a8_gemm")
    return (y, acc) if return_acc else y


def moe_unpermute(y, row_map, probs, shared=None):
    """MoeTokenUnpermute: out[t] = sum_j probs[t,j] * y[row_map[t*k+j]] (+ shared[t])."""
    lib = _lib.load()
    dev = _dev_ok(y, row_map, probs, shared)
    t, k = probs.shape
    h = y.shape[1]
    _need(y.dtype in _ACT and probs.dtype == y.dtype and row_map.dtype == torch.int32 and row_map.numel() == t * k
          and y.shape[0] == t * k, "operand mismatch")
    _need(shared is None or (shared.dtype == y.dtype and shared.shape == (t, h)), "shared mismatch")
    out = torch.empty(t, h, dtype=y.dtype, device=dev)
    check(lib.mf_moe_unpermute(ptr(out), ptr(y), ptr(row_map), ptr(probs), ptr(shared), t, k, h, dtype_code(y.dtype),
                               stream_ptr(dev)), "mf_moe_unpermute")
    return out


def default_scale(head_dim):
    return 1.0 / math.sqrt(head_dim)
