"""KV-cache scatter, paged-attention decode and host slot mapping.  Test infrastructure only.

Follows:
  ReshapeAndCache call sites   mindformers/modules/paged_attention_mgr.py:60-62,
                               mindformers/parallel_core/inference/transformer/flash_attention.py:126-127
  PagedAttention call sites    mindformers/modules/paged_attention_mgr.py:64-70,
                               mindformers/parallel_core/inference/transformer/flash_attention.py:135-143
  unfused attention math       mindformers/modules/infer_attention.py:303-340 (scores*scale, fp32 softmax,
                               probabilities cast to the compute dtype, PV), GQA head repeat :329-340,
                               mindformers/parallel_core/inference/transformer/dot_product_attention.py:94-133
  slot mapping                 mindformers/modules/block_tables.py:65-121
"""
import numpy as np

from .numerics import round_to


def reshape_and_cache(key, value, key_cache, value_cache, slot_mapping):
    """In-place scatter: cache.reshape(-1, n_kv, D)[slot[i]] = x[i]; slot < 0 is padding.

    key/value: [T, n_kv*D] (or any shape with T rows); caches: [num_blocks, block_size, n_kv, D].
    Returns key, as the primitive does (paged_attention_mgr.py:62 returns the op's output which
    the caller only uses as an ordering edge, infer_attention.py:453-454).
    """
    nb, bs, n_kv, d = key_cache.shape
    kc = key_cache.reshape(nb * bs, n_kv, d)
    t = len(slot_mapping)
    k = np.asarray(key).reshape(t, n_kv, d)
    for i in range(t):
        s = int(slot_mapping[i])
        if s < 0:
            continue
        kc[s] = k[i]
    if value is not None and value_cache is not None:
        vc = value_cache.reshape(nb * bs, n_kv, d)
        v = np.asarray(value).reshape(t, n_kv, d)
        for i in range(t):
            s = int(slot_mapping[i])
            if s >= 0:
                vc[s] = v[i]
    return key


def gather_kv(cache, block_table, length):
    """Rows 0..length-1 of one sequence: token j lives at cache[block_table[j // bs], j % bs]."""
    nb, bs, n_kv, d = cache.shape
    j = np.arange(length)
    blocks = np.asarray(block_table)[j // bs].astype(np.int64)
    return cache[blocks, j % bs]          # [length, n_kv, D]


def paged_attention_decode(query, key_cache, value_cache, block_tables, context_lens,
                           n_head, n_kv_head, scale, prob_dtype=None):
    """out[b, h] = softmax(scale * q[b,h] . K_b[:L_b]^T) V_b[:L_b], kv head = h // (n_head/n_kv).

    query [B, n_head*D]; context_lens[b] counts the new token (it is already in the cache:
    tests/st/test_infer/test_infer_module/test_infer_attention.py:249, block_tables.py:113).
    Computed in float64; ``prob_dtype`` optionally rounds the probabilities through the compute
    dtype before the PV product, as the reference's unfused path does (infer_attention.py:324-326).
    A sequence with L_b <= 0 yields zeros.
    """
    nb, bs, n_kv, d = key_cache.shape
    assert n_kv == n_kv_head
    b_sz = len(context_lens)
    q = np.asarray(query, dtype=np.float64).reshape(b_sz, n_head, d)
    n_rep = n_head // n_kv_head
    out = np.zeros((b_sz, n_head, d), dtype=np.float64)
    for b in range(b_sz):
        length = int(context_lens[b])
        if length <= 0:
            continue
        k = gather_kv(key_cache, block_tables[b], length).astype(np.float64)     # [L, n_kv, D]
        v = gather_kv(value_cache, block_tables[b], length).astype(np.float64)
        for h in range(n_head):
            g = h // n_rep
            s = (k[:, g, :] @ q[b, h]) * scale
            s = s - s.max()
            p = np.exp(s)
            p = p / p.sum()
            if prob_dtype is not None:
                p = round_to(p, prob_dtype).astype(np.float64)
            out[b, h] = p @ v[:, g, :]
    return out.reshape(b_sz, n_head * d)


def paged_attention_prefill(query, key_cache, value_cache, block_tables, context_lens, q_seq_lens,
                            n_head, n_kv_head, scale, prob_dtype=None):
    """PagedAttention with several new tokens per sequence and a causal mask among them (paged_attention_mgr.py:66-69
    called with q_seq_lens; the mask is the lower triangle built by generation/parallel_decoding.py:73-80).

    query [sum(q_seq_lens), n_head*D] packed sequence after sequence; the new tokens are already in the cache and
    context_lens[b] counts them, so query i of sequence b sees cache tokens 0 .. L_b - q_len_b + i.  float64.
    Pinned through its two special cases: one query per sequence is `paged_attention_decode`, and an empty
    cache before the step is `causal_prefill_attention` (both pinned by the reference's golden outputs).
    """
    nb, bs, n_kv, d = key_cache.shape
    assert n_kv == n_kv_head
    t = int(np.sum(q_seq_lens))
    q = np.asarray(query, dtype=np.float64).reshape(t, n_head, d)
    n_rep = n_head // n_kv_head
    out = np.zeros((t, n_head, d), dtype=np.float64)
    start = 0
    for b, q_len in enumerate(q_seq_lens):
        q_len, length = int(q_len), int(context_lens[b])
        if length > 0 and q_len > 0:
            k = gather_kv(key_cache, block_tables[b], length).astype(np.float64)
            v = gather_kv(value_cache, block_tables[b], length).astype(np.float64)
            for i in range(q_len):
                lim = length - q_len + i + 1
                if lim <= 0:
                    continue
                for h in range(n_head):
                    g = h // n_rep
                    sc = (k[:lim, g, :] @ q[start + i, h]) * scale
                    p = np.exp(sc - sc.max())
                    p = p / p.sum()
                    if prob_dtype is not None:
                        p = round_to(p, prob_dtype).astype(np.float64)
                    out[start + i, h] = p @ v[:lim, g, :]
        start += q_len
    return out.reshape(t, n_head * d)


def mla_paged_attention_decode(query, latent_cache, block_tables, context_lens, n_head, v_dim, scale,
                               prob_dtype=None, abs_values=False):
    """PagedAttention with one shared latent row per token (mla_v_dim = v_dim): the key of every head is the whole
    cache row, the value its first v_dim entries (flash_attention.py:106-107,136-139 called with key_cache twice;
    multi_latent_attention.py:199-228).  query [B, n_head * Dk], cache [blocks, bs, 1, Dk]; returns
    [B, n_head * v_dim].  float64.  ``abs_values`` returns sum_t p_t |v_t| instead (the magnitude that the rounding
    error of the product scales with; used for test tolerances).  Pinned by its reduction to `paged_attention_decode` with one kv head when
    v_dim = Dk, and by slicing: the output is that result's first v_dim columns per head."""
    nb, bs, n_kv, dk = latent_cache.shape
    assert n_kv == 1 and v_dim <= dk
    b_sz = len(context_lens)
    q = np.asarray(query, dtype=np.float64).reshape(b_sz, n_head, dk)
    out = np.zeros((b_sz, n_head, v_dim), dtype=np.float64)
    for b in range(b_sz):
        length = int(context_lens[b])
        if length <= 0:
            continue
        c = gather_kv(latent_cache, block_tables[b], length)[:, 0, :].astype(np.float64)      # [L, Dk]
        s = (q[b] @ c.T) * scale                                                               # [n_head, L]
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p = p / p.sum(axis=1, keepdims=True)
        if prob_dtype is not None:
            p = round_to(p, prob_dtype).astype(np.float64)
        out[b] = p @ (np.abs(c[:, :v_dim]) if abs_values else c[:, :v_dim])
    return out.reshape(b_sz, n_head * v_dim)


def causal_prefill_attention(query, key, value, seq_lens, n_head, n_kv_head, scale):
    """Varlen causal attention over packed [T, heads*D] rows (FlashAttentionScore, TH layout,
    flash_attention.py:129-134; unfused form infer_attention.py:342-404).  float64."""
    t = query.shape[0]
    d = query.shape[1] // n_head
    q = np.asarray(query, dtype=np.float64).reshape(t, n_head, d)
    k = np.asarray(key, dtype=np.float64).reshape(t, n_kv_head, d)
    v = np.asarray(value, dtype=np.float64).reshape(t, n_kv_head, d)
    n_rep = n_head // n_kv_head
    out = np.zeros_like(q)
    start = 0
    for length in seq_lens:
        length = int(length)
        for i in range(length):
            for h in range(n_head):
                g = h // n_rep
                s = (k[start:start + i + 1, g] @ q[start + i, h]) * scale
                p = np.exp(s - s.max())
                p /= p.sum()
                out[start + i, h] = p @ v[start:start + i + 1, g]
        start += length
    return out.reshape(t, n_head * d)


def decode_slot_mapping(block_tables, context_lens, block_size):
    """slot = table[(L-1)//bs]*bs + (L-1)%bs, clamped to the last allocated block
    (block_tables.py:113-119)."""
    slots = []
    for table, length in zip(block_tables, context_lens):
        table = [int(x) for x in table if int(x) >= 0]
        cur = int(length) - 1
        idx = cur // block_size
        if idx >= len(table):
            idx = len(table) - 1
        slots.append(table[idx] * block_size + cur % block_size)
    return np.asarray(slots, dtype=np.int32)


def prefill_slot_mapping(block_tables, context_lens, block_size, max_input_length):
    """Per-token slots for a padded [B, max_input_length] prefill; padding = -1
    (block_tables.py:77-96, written as the naive per-token loop)."""
    out = -np.ones((len(context_lens), max_input_length), dtype=np.int32)
    for b, length in enumerate(context_lens):
        for j in range(int(length)):
            out[b, j] = int(block_tables[b][j // block_size]) * block_size + j % block_size
    return out.reshape(-1)
