"""Multi-latent self-attention of the Megatron-style inference stack:
mindformers/parallel_core/inference/transformer/multi_latent_attention.py:44-448 (MLASelfAttentionSubmodules,
MultiLatentAttention, MLASelfAttention) at tensor-parallel size 1.

One latent row per token (kv_lora_rank values + the shared rotary part) is cached.  Decode folds the key half of
``linear_kv_up_proj.weight`` into the query and applies its value half to the attention output (:434-448, :228-231),
both through ``ops.mla_absorb_bmm``; prefill up-projects keys and values and runs ordinary causal attention over
192-wide heads (:405-432, :206-216).  The projections are the float linear cells of ``layers.py`` until a quantizer
swaps them (``linear_kv_up_proj`` must stay a float cell: its weight is the absorb operand).
"""
import math
from dataclasses import dataclass
from typing import Optional, Union

import torch
from torch import nn

from .. import ops
from ..transformer_config import TransformerConfig
from .flash_attention import FlashAttention
from .layers import ColumnParallelLinear, ReplicatedLinear, RowParallelLinear
from .norm import RMSNorm
from .rotary import RotaryEmbedding, YaRNScalingRotaryEmbedding, _yarn_get_mscale


@dataclass
class MLATransformerConfig(TransformerConfig):
    """mindformers/parallel_core/transformer_config.py:613-664: field names and defaults of the reference."""
    multi_latent_attention: bool = True
    q_lora_rank: Optional[int] = 512
    kv_lora_rank: int = 512
    qk_head_dim: int = 128
    qk_pos_emb_head_dim: int = 64
    v_head_dim: int = 128
    normalization: str = "RMSNorm"
    rope_type: str = "yarn"
    rotary_base: float = 10000.0
    rotary_percent: float = 1.0
    rotary_scaling_factor: float = 40.0
    max_position_embeddings: int = 4096
    beta_fast: float = 32.0
    beta_slow: float = 1.0
    mscale: float = 0.707
    mscale_all_dim: float = 0.707


@dataclass
class MLASelfAttentionSubmodules:
    """multi_latent_attention.py:44-56: the classes the layer is built from (defaults: this package's cells)."""
    linear_q_proj: Union[type, None] = ColumnParallelLinear
    linear_qkv_down_proj: Union[type, None] = ReplicatedLinear
    linear_q_up_proj: Union[type, None] = ColumnParallelLinear
    linear_kv_down_proj: Union[type, None] = ReplicatedLinear
    linear_kv_up_proj: Union[type, None] = ColumnParallelLinear
    core_attention: Union[type, None] = FlashAttention
    linear_proj: Union[type, None] = RowParallelLinear
    q_layernorm: Union[type, None] = RMSNorm
    kv_layernorm: Union[type, None] = RMSNorm


class MLASelfAttention(nn.Module):
    """``MLASelfAttention(config, submodules, layer_number)``; the phase flag ``is_prefill`` selects the branch, as in the
    reference (set it on this module; the core attention follows)."""

    def __init__(self, config, submodules=None, layer_number=1, attn_mask_type=None, attention_type=None,
                 cp_comm_type=None, model_comm_pgs=None, device="cuda"):
        super().__init__()
        for value, name in ((attn_mask_type, "attn_mask_type"), (attention_type, "attention_type"),
                            (cp_comm_type, "cp_comm_type")):
            if value:
                raise NotImplementedError(f"For MultiLatentAttention, `{name}` is not supported for now.")
        if not config.use_flash_attention:
            raise NotImplementedError("For MLA, only `use_flash_attention=True` is supported")
        sub = submodules or MLASelfAttentionSubmodules()
        self.config = config
        self.layer_number = max(1, layer_number)
        c = config
        self.num_attention_heads = self.num_attention_heads_per_partition = c.num_attention_heads
        self.kv_num_heads_per_partition = c.num_attention_heads
        self.q_head_dim = c.qk_head_dim + c.qk_pos_emb_head_dim
        self.query_projection_size = c.v_head_dim * c.num_attention_heads
        self.key_hidden_size, self.val_hidden_size = self.q_head_dim, c.v_head_dim
        self.compute_dtype = c.compute_dtype
        self.is_prefill = True
        mscale = _yarn_get_mscale(c.rotary_scaling_factor, c.mscale)
        self.softmax_scale = mscale * mscale / math.sqrt(self.q_head_dim)
        if c.rope_type == "rope":
            self.rotary_pos_emb = RotaryEmbedding(c.qk_pos_emb_head_dim, rotary_percent=c.rotary_percent,
                                                  rotary_base=c.rotary_base, rotary_cos_format=2,
                                                  rotary_dtype=c.compute_dtype,
                                                  max_position_embeddings=c.max_position_embeddings, device=device)
        elif c.rope_type == "yarn":
            self.rotary_pos_emb = YaRNScalingRotaryEmbedding(
                c.qk_pos_emb_head_dim, rotary_base=c.rotary_base, scaling_factor=c.rotary_scaling_factor,
                original_max_position_embeddings=c.max_position_embeddings, beta_fast=c.beta_fast,
                beta_slow=c.beta_slow, mscale=c.mscale, mscale_all_dim=c.mscale_all_dim, rotary_cos_format=2,
                rotary_dtype=c.compute_dtype, device=device)
        else:
            raise ValueError(f"Unsupported RoPE type: {c.rope_type}, supported types are 'rope' and 'yarn'")
        self.core_attention = sub.core_attention(head_num=c.num_attention_heads, head_dim=self.q_head_dim,
                                                 kv_head_num=c.num_attention_heads, scale_value=self.softmax_scale,
                                                 next_tokens=0, pa_kv_head_num=1, pa_mla_v_dim=c.kv_lora_rank)
        lin = dict(config=c, bias=False, transpose_b=True, compute_dtype=c.compute_dtype, device=device)
        self.linear_proj = sub.linear_proj(self.query_projection_size, c.hidden_size, config=c, bias=c.add_bias_linear,
                                           input_is_parallel=True, skip_bias_add=False, is_expert=False,
                                           transpose_b=True, compute_dtype=c.compute_dtype, device=device)
        if c.q_lora_rank is None:
            self.linear_q_proj = sub.linear_q_proj(c.hidden_size, c.num_attention_heads * self.q_head_dim, **lin)
            self.linear_kv_down_proj = sub.linear_kv_down_proj(c.hidden_size, c.kv_lora_rank + c.qk_pos_emb_head_dim,
                                                               **lin)
        else:
            self.linear_qkv_down_proj = sub.linear_qkv_down_proj(
                c.hidden_size, c.q_lora_rank + c.kv_lora_rank + c.qk_pos_emb_head_dim, **lin)
            self.linear_q_up_proj = sub.linear_q_up_proj(c.q_lora_rank, c.num_attention_heads * self.q_head_dim, **lin)
            self.q_layernorm = sub.q_layernorm(config=c, hidden_size=c.q_lora_rank, eps=c.layernorm_epsilon,
                                               device=device)
        self.linear_kv_up_proj = sub.linear_kv_up_proj(c.kv_lora_rank,
                                                       c.num_attention_heads * (c.qk_head_dim + c.v_head_dim), **lin)
        self.kv_layernorm = sub.kv_layernorm(config=c, hidden_size=c.kv_lora_rank, eps=c.layernorm_epsilon,
                                             device=device)
        self._absorb = None                                   # (q_absorb transposed [n, rank, nope], out_absorb [n, v, rank])

    # ---- absorbed weights -------------------------------------------------------------------------------------
    def prepare(self):
        """The two absorb operands from ``linear_kv_up_proj.weight`` (:434-441): rows [n * nope] are the key side,
        stored transposed per head so that the kernel reads rows of the reduction dimension, the rest the value side.
        Call again after loading new weights."""
        c = self.config
        w = getattr(self.linear_kv_up_proj, "weight", None)
        if w is None or not w.dtype.is_floating_point:
            raise NotImplementedError("linear_kv_up_proj must stay a float cell (list it in modules_to_not_convert): "
                                      "its weight is the operand of the absorbed projections")
        n, nope, vd, rank = c.num_attention_heads, c.qk_head_dim, c.v_head_dim, c.kv_lora_rank
        w = w.detach().to(self.compute_dtype)
        q_absorb_t = w[: n * nope].reshape(n, nope, rank).transpose(1, 2).contiguous()
        out_absorb = w[n * nope:].reshape(n, vd, rank).contiguous()
        self._absorb = (q_absorb_t, out_absorb)
        return self

    def _load_from_state_dict(self, *args, **kwargs):
        self._absorb = None
        return super()._load_from_state_dict(*args, **kwargs)

    # ---- projections (:361-403) ------------------------------------------------------------------------------
    def _project(self, hidden_states, rotary_pos_cos, rotary_pos_sin, slot_mapping, key_cache, query_out=None):
        """Down projections, norms, query up-projection, RoPE and the latent-row scatter.  Returns q [T, n, nope + rope]
        and, for a prefill (``query_out`` None), the normalised latent rows and the rotated key part; the rotated query
        parts go back into q, or, for a decode step, behind the absorbed query in ``query_out`` [T, n, rank + rope]."""
        c = self.config
        n, nope, rope, rank = c.num_attention_heads, c.qk_head_dim, c.qk_pos_emb_head_dim, c.kv_lora_rank
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        if c.q_lora_rank is not None:
            down, qn = self.linear_qkv_down_proj, self.q_layernorm
            if hasattr(down, "forward_with_leading_norm") and isinstance(getattr(qn, "weight", None), torch.Tensor) \
                    and hasattr(qn, "eps") and qn.weight.numel() == c.q_lora_rank:
                # weight-only down projection: its split-K sum and q_layernorm are one kernel
                qkv, q_c = down.forward_with_leading_norm(x, qn.weight, qn.eps)
            else:
                qkv = down(x)
                q_c = qn(qkv[:, : c.q_lora_rank])             # the norm reads the column slice where it lies
            kv = qkv[:, c.q_lora_rank:]                       # latent part, then the rotary key part
            q = self.linear_q_up_proj(q_c)
        else:
            kv = self.linear_kv_down_proj(x)
            q = self.linear_q_proj(x)
        t = x.shape[0]
        q = q.reshape(t, n, self.q_head_dim)
        gamma = getattr(self.kv_layernorm, "weight", None)
        if rotary_pos_cos is not None and rotary_pos_sin is not None and gamma is not None:
            # kv_layernorm + RoPE + scatter + placement of the rotated query part: one launch
            decode = query_out is not None
            kv_c = None if decode else torch.empty((t, rank), dtype=q.dtype, device=q.device)
            k_pe = None if decode else torch.empty((t, rope), dtype=q.dtype, device=q.device)
            eps = getattr(self.kv_layernorm, "eps", c.layernorm_epsilon)
            ops.mla_norm_rope_cache(q, nope, kv, gamma, eps, rotary_pos_cos.reshape(t, rope), rotary_pos_sin.reshape(t, rope),
                                    latent_cache=key_cache, slot_mapping=slot_mapping,
                                    q_rope_out=query_out[..., rank:] if decode else None, kv_norm_out=kv_c, k_pe_out=k_pe)
            return q, kv_c, k_pe
        # no rotary rows (or a norm cell without a gamma vector): the separate cells
        kv_c = self.kv_layernorm(kv[:, :rank])
        k_pe = kv[:, rank:].contiguous()
        if rotary_pos_cos is not None and rotary_pos_sin is not None:
            q_pe = q[..., nope:].reshape(t, n * rope)
            self.rotary_pos_emb(q_pe, k_pe, rotary_pos_cos, rotary_pos_sin)
            q[..., nope:] = q_pe.reshape(t, n, rope)
        if key_cache is not None:
            ops.reshape_and_cache(torch.cat((kv_c, k_pe), dim=-1), None, key_cache, None, slot_mapping)
        if query_out is not None:
            query_out[..., rank:] = q[..., nope:]
        return q, kv_c, k_pe

    def forward(self, hidden_states, attention_mask=None, key_value_states=None, rotary_pos_cos=None,
                rotary_pos_sin=None, position_ids=None, batch_valid_length=None, block_tables=None, slot_mapping=None,
                q_seq_lens=None, actual_seq_qlen=None, actual_seq_kvlen=None, context_lens_tensor=None, key_cache=None,
                value_cache=None):
        c = self.config
        n, nope, rope, rank, vd = c.num_attention_heads, c.qk_head_dim, c.qk_pos_emb_head_dim, c.kv_lora_rank, c.v_head_dim
        self.core_attention.is_prefill = self.is_prefill
        if self.is_prefill:
            q, kv_c, k_pe = self._project(hidden_states, rotary_pos_cos, rotary_pos_sin, slot_mapping, key_cache)
            t = q.shape[0]
            kv = self.linear_kv_up_proj(kv_c).reshape(t, -1)
            k_no_pe = kv[:, : n * nope].reshape(t, n, nope)
            value = kv[:, n * nope:].reshape(t, n, vd)
            k_rep = k_pe[:, None, :].expand(t, n, rope)
            key = torch.cat((k_no_pe, k_rep), dim=-1).reshape(t, n * self.q_head_dim)
            if self.q_head_dim == 192 and vd == 128:
                # the attention takes the 128-wide values as they are (the reference pads them to the key width with
                # the rotary part and keeps the first 128 output columns: the same numbers)
                val = value.reshape(t, n * vd)
            else:
                val = torch.cat((value, k_rep), dim=-1)
                if vd + rope != self.q_head_dim:
                    val = torch.nn.functional.pad(val, (0, self.q_head_dim - vd - rope))
                val = val.reshape(t, n * self.q_head_dim)
            out = self.core_attention(q.reshape(t, n * self.q_head_dim), key, val,
                                      slot_mapping, block_tables, batch_valid_length, context_lens_tensor, q_seq_lens,
                                      actual_seq_qlen=actual_seq_qlen, actual_seq_kvlen=actual_seq_kvlen,
                                      attn_mask=attention_mask, key_cache=key_cache, value_cache=value_cache)
            if val.shape[1] == n * vd:
                core = out.reshape(t, n * vd)
            else:
                core = out.reshape(t, n, self.q_head_dim)[..., :vd].reshape(t, n * vd)
        else:
            if self._absorb is None:
                self.prepare()
            q_absorb_t, out_absorb = self._absorb
            t = hidden_states.reshape(-1, hidden_states.shape[-1]).shape[0]
            query = torch.empty((t, n, rank + rope), dtype=self.compute_dtype, device=hidden_states.device)
            q, _, _ = self._project(hidden_states, rotary_pos_cos, rotary_pos_sin, slot_mapping, key_cache, query_out=query)
            ops.mla_absorb_bmm(q[..., :nope], q_absorb_t, out=query[..., :rank])
            attn = self.core_attention(query.reshape(t, n * (rank + rope)), None, None, slot_mapping, block_tables,
                                       batch_valid_length, context_lens_tensor, q_seq_lens,
                                       actual_seq_qlen=actual_seq_qlen, actual_seq_kvlen=actual_seq_kvlen,
                                       attn_mask=attention_mask, key_cache=key_cache, value_cache=value_cache)
            core = ops.mla_absorb_bmm(attn.reshape(t, n, rank), out_absorb).reshape(t, n * vd)
        return self.linear_proj(core)

    construct = forward
