"""Multi-latent self-attention of one layer step, restated in numpy (float64).  TEST INFRASTRUCTURE ONLY.

Follows mindformers/parallel_core/inference/transformer/multi_latent_attention.py: the projections and norms of
MLASelfAttention.get_query_key_value_tensors (:344-448), the attention and the output projection of
MultiLatentAttention.construct (:186-236).  Parameters are float arrays with the reference's [out, in] layout:

  qkv_down_w  [q_lora_rank + kv_lora_rank + rope, hidden]   linear_qkv_down_proj (q_lora_rank given), or
  q_w         [n_head * (nope + rope), hidden], kv_down_w [kv_lora_rank + rope, hidden]   (q_lora_rank None)
  q_norm      [q_lora_rank]                                 q_layernorm gamma
  q_up_w      [n_head * (nope + rope), q_lora_rank]         linear_q_up_proj
  kv_norm     [kv_lora_rank]                                kv_layernorm gamma
  kv_up_w     [n_head * (nope + v_dim), kv_lora_rank]       linear_kv_up_proj: n_head * nope key rows, then the values
  proj_w      [hidden, n_head * v_dim]                      linear_proj

Pinning: the decode form (weights absorbed into the query and the output, attention over the latent cache) is held
to the prefill form (keys and values up-projected, ordinary attention), which is the definition, by
tests/test_oracle_golden.py: the decode step of a token must equal the last row of a prefill over the same tokens.
A transposed or mis-sliced absorb matrix, a wrong split of linear_kv_up_proj or a wrong softmax scale fails it.
The pieces underneath (paged / causal attention, RoPE, RMSNorm, linear) are pinned by the reference's vectors.
"""
import numpy as np

from .attention import causal_prefill_attention, mla_paged_attention_decode, reshape_and_cache
from .dense import linear, rms_norm
from .numerics import round_to
from .rope import apply_rotary_half


def _r(x, dt):
    return x if dt is None else round_to(x, dt).astype(np.float64)


def mla_project(hidden, p, cfg, cos, sin, act_dtype=None):
    """Down projections, norms, query up-projection and RoPE (:361-400).  Returns q_no_pe [T, n, nope],
    q_pos_emb [T, n, rope], the normalised latent [T, kv_lora_rank] and the rotated k_pos_emb [T, rope]."""
    n, nope, rope, rank = cfg["n_head"], cfg["qk_head_dim"], cfg["qk_pos_emb_head_dim"], cfg["kv_lora_rank"]
    eps = cfg.get("eps", 1e-6)
    hidden = np.asarray(hidden, dtype=np.float64)
    if cfg.get("q_lora_rank"):
        qkv = _r(linear(hidden, p["qkv_down_w"]), act_dtype)
        ql = cfg["q_lora_rank"]
        q_c, kv_c, k_pe = qkv[:, :ql], qkv[:, ql:ql + rank], qkv[:, ql + rank:]
        q_c = _r(rms_norm(q_c, p["q_norm"], eps), act_dtype)
        q = _r(linear(q_c, p["q_up_w"]), act_dtype)
    else:
        kv = _r(linear(hidden, p["kv_down_w"]), act_dtype)
        kv_c, k_pe = kv[:, :rank], kv[:, rank:]
        q = _r(linear(hidden, p["q_w"]), act_dtype)
    t = hidden.shape[0]
    q = q.reshape(t, n, nope + rope)
    q_no_pe, q_pe = q[..., :nope], q[..., nope:]
    kv_c = _r(rms_norm(kv_c, p["kv_norm"], eps), act_dtype)
    q_pe = _r(apply_rotary_half(q_pe.reshape(t, n * rope), cos, sin, n), act_dtype).reshape(t, n, rope)
    k_pe = _r(apply_rotary_half(k_pe, cos, sin, 1), act_dtype)
    return q_no_pe, q_pe, kv_c, k_pe


def softmax_scale(cfg):
    """mscale^2 / sqrt(nope + rope) with the YaRN mscale of the rotary scaling factor (:110-111)."""
    from .rope import yarn_mscale
    m = yarn_mscale(cfg.get("rotary_scaling_factor", 1.0), cfg.get("mscale", 1.0))
    return m * m / np.sqrt(cfg["qk_head_dim"] + cfg["qk_pos_emb_head_dim"])


def mla_self_attention_decode(hidden, p, cfg, latent_cache, block_tables, context_lens, slot_mapping, cos, sin,
                              act_dtype=None):
    """One new token per sequence (:401-403 scatter, :434-448 absorbed query, :218-231 attention and absorbed output,
    :233-236 projection).  latent_cache [blocks, block_size, 1, kv_lora_rank + rope] is updated in place."""
    n, nope, rope, rank, vd = (cfg["n_head"], cfg["qk_head_dim"], cfg["qk_pos_emb_head_dim"], cfg["kv_lora_rank"],
                               cfg["v_head_dim"])
    q_no_pe, q_pe, kv_c, k_pe = mla_project(hidden, p, cfg, cos, sin, act_dtype)
    reshape_and_cache(np.concatenate((kv_c, k_pe), axis=-1), None, latent_cache, None, slot_mapping)
    w = np.asarray(p["kv_up_w"], dtype=np.float64)
    q_absorb = w[: n * nope].reshape(n, nope, rank)
    out_absorb = w[n * nope:].reshape(n, vd, rank)
    t = q_no_pe.shape[0]
    q_lat = _r(np.einsum("thk,hkr->thr", q_no_pe, q_absorb), act_dtype)
    query = np.concatenate((q_lat, q_pe), axis=-1).reshape(t, n * (rank + rope))
    attn = _r(mla_paged_attention_decode(query, latent_cache, block_tables, context_lens, n, rank, softmax_scale(cfg),
                                         prob_dtype=act_dtype), act_dtype).reshape(t, n, rank)
    core = _r(np.einsum("thr,hvr->thv", attn, out_absorb), act_dtype).reshape(t, n * vd)
    return _r(linear(core, p["proj_w"]), act_dtype)


def mla_self_attention_prefill(hidden, p, cfg, latent_cache, slot_mapping, seq_lens, cos, sin, act_dtype=None):
    """Whole prompts, packed rows (:405-432 up-projected keys and values with the shared rotary part appended, :206-216
    attention over 192-wide heads of which the first v_dim columns are kept)."""
    n, nope, rope, rank, vd = (cfg["n_head"], cfg["qk_head_dim"], cfg["qk_pos_emb_head_dim"], cfg["kv_lora_rank"],
                               cfg["v_head_dim"])
    q_no_pe, q_pe, kv_c, k_pe = mla_project(hidden, p, cfg, cos, sin, act_dtype)
    if latent_cache is not None:
        reshape_and_cache(np.concatenate((kv_c, k_pe), axis=-1), None, latent_cache, None, slot_mapping)
    t = q_no_pe.shape[0]
    kv = _r(linear(kv_c, p["kv_up_w"]), act_dtype)
    k_no_pe, value = kv[:, : n * nope].reshape(t, n, nope), kv[:, n * nope:].reshape(t, n, vd)
    k_rep = np.broadcast_to(k_pe[:, None, :], (t, n, rope))
    d = nope + rope
    query = np.concatenate((q_no_pe, q_pe), axis=-1).reshape(t, n * d)
    key = np.concatenate((k_no_pe, k_rep), axis=-1).reshape(t, n * d)
    val = np.concatenate((value, k_rep), axis=-1)
    if vd + rope != d:                                        # value rows are padded to the key width
        val = np.concatenate((val, np.zeros((t, n, d - vd - rope))), axis=-1)
    core = _r(causal_prefill_attention(query, key, val.reshape(t, n * d), seq_lens, n, n, softmax_scale(cfg)), act_dtype)
    core = core.reshape(t, n, d)[..., :vd].reshape(t, n * vd)
    return _r(linear(core, p["proj_w"]), act_dtype)
