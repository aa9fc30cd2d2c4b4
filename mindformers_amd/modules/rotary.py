"""Rotary position tables and the decode-time application.

  Megatron-style   RotaryEmbedding / Llama3RotaryEmbedding / YaRNScalingRotaryEmbedding —
                   mindformers/parallel_core/inference/base_models/common/embeddings/rotary_pos_embedding.py:33-211,
                   .../yarn_rotary_pos_embedding.py:30-173
  legacy           FreqsMgr — mindformers/modules/layers.py:1171-1333 (prefill / increment row selection)

Tables are built once on the host in float32 exactly as the reference does (cos/sin of concat(freqs, freqs),
times mscale, cast to the rotary dtype) and kept on the device; the per-step work (row gather + rotate-half
application) runs in the HIP kernel.
"""
import math

import numpy as np
import torch
from torch import nn

from .. import ops


def _inv_freq_default(dim, base):
    return (1.0 / (np.float32(base) ** (np.arange(0, dim, 2, dtype=np.float32)[: dim // 2] / np.float32(dim)))).astype(np.float32)


def _yarn_get_mscale(scale=1.0, mscale=1.0):
    if scale <= 1:
        return 1.0
    return 0.1 * mscale * math.log(scale) + 1.0


def _yarn_find_correction_dim(num_rotations, dim, base=10000, max_position_embeddings=2048):
    return (dim * math.log(max_position_embeddings / (num_rotations * 2 * math.pi))) / (2 * math.log(base))


def _yarn_find_correction_range(low_rot, high_rot, dim, base=10000, max_position_embeddings=2048):
    low = math.floor(_yarn_find_correction_dim(low_rot, dim, base, max_position_embeddings))
    high = math.ceil(_yarn_find_correction_dim(high_rot, dim, base, max_position_embeddings))
    return max(low, 0), min(high, dim - 1)


def _yarn_linear_ramp_mask(low, high, dim):
    if low == high:
        high += 0.001
    return np.clip((np.arange(dim, dtype=np.float32) - low) / (high - low), 0, 1).astype(np.float32)


def _tables(inv_freq, num_positions, mscale, dtype, device):
    seq = np.arange(0, num_positions, 1, dtype=np.float32)
    freqs = np.outer(seq, inv_freq).astype(np.float32)
    emb = np.concatenate((freqs, freqs), axis=-1)
    cos = torch.from_numpy((np.cos(emb) * np.float32(mscale)).astype(np.float32)).to(device=device, dtype=dtype)
    sin = torch.from_numpy((np.sin(emb) * np.float32(mscale)).astype(np.float32)).to(device=device, dtype=dtype)
    return cos, sin


class RotaryEmbedding(nn.Module):
    """rotary_pos_embedding.py:33-146.  ``forward`` applies ApplyRotaryPosEmb(rotary_cos_format) in place."""

    def __init__(self, kv_channels, rotary_percent=1.0, rotary_interleaved=False, seq_len_interpolation_factor=None,
                 rotary_base=10000, rotary_cos_format=0, rotary_dtype=torch.float16, max_position_embeddings=4096,
                 device="cuda"):
        super().__init__()
        if rotary_interleaved:
            raise NotImplementedError("For RotaryEmbedding, `rotary_interleaved` is not supported.")
        if seq_len_interpolation_factor:
            raise NotImplementedError("For RotaryEmbedding, `seq_len_interpolation_factor` is not supported.")
        self.dim = kv_channels
        if rotary_percent < 1.0:
            self.dim = int(self.dim * rotary_percent)
        self.kv_channels = kv_channels
        self.rotary_base = rotary_base
        self.rotary_cos_format = rotary_cos_format
        self.rotary_dtype = rotary_dtype
        self.max_position_embeddings = max_position_embeddings
        self._device = device
        cos, sin = self._compute_cos_sin_cache()
        self.register_buffer("cos_cache", cos, persistent=False)
        self.register_buffer("sin_cache", sin, persistent=False)

    def _compute_inv_freq(self, base):
        return _inv_freq_default(self.dim, base)

    def _num_positions(self):
        return self.max_position_embeddings

    def _mscale(self):
        return 1.0

    def _compute_cos_sin_cache(self):
        return _tables(self._compute_inv_freq(self.rotary_base), self._num_positions(), self._mscale(),
                       self.rotary_dtype, self._device)

    def get_cos_sin_for_prefill(self):
        return self.cos_cache, self.sin_cache

    def get_cos_sin_for_decode(self, positions):
        idx = positions.to(torch.long)
        return self.cos_cache.index_select(0, idx), self.sin_cache.index_select(0, idx)

    def forward(self, query, key, rotary_pos_cos, rotary_pos_sin, seq_lens_tensor=None):
        """query [T, n_heads*D], key [T, n_kv*D]; cos/sin hold one row per token.  Rotated in place and returned."""
        if self.rotary_cos_format != 2:
            raise NotImplementedError("only rotary_cos_format=2 (rotate-half) is built")
        if self.dim != self.kv_channels:
            raise NotImplementedError("partial rotary (rotary_percent < 1) is not built")
        d = self.kv_channels
        ops.apply_rotary_pos_emb(query, key, rotary_pos_cos.contiguous(), rotary_pos_sin.contiguous(),
                                 query.shape[-1] // d, key.shape[-1] // d, d)
        return query, key

    construct = forward


class Llama3RotaryEmbedding(RotaryEmbedding):
    """rotary_pos_embedding.py:149-211."""

    def __init__(self, kv_channels, rotary_percent=1.0, rotary_interleaved=False, seq_len_interpolation_factor=None,
                 rotary_base=10000, rotary_cos_format=0, rotary_dtype=torch.float16, max_position_embeddings=8192,
                 scaling_factor=1.0, low_freq_factor=1.0, high_freq_factor=4.0, orig_max_position=4096, device="cuda"):
        self.scaling_factor = scaling_factor
        self.low_freq_factor = low_freq_factor
        self.high_freq_factor = high_freq_factor
        self.orig_max_position = orig_max_position
        super().__init__(kv_channels, rotary_percent, rotary_interleaved, seq_len_interpolation_factor, rotary_base,
                         rotary_cos_format, rotary_dtype, max_position_embeddings, device)

    def _compute_inv_freq(self, base):
        inv = _inv_freq_default(self.dim, base)
        low_wl = self.orig_max_position / self.low_freq_factor
        high_wl = self.orig_max_position / self.high_freq_factor
        wave = (2 * math.pi / inv).astype(np.float32)
        if not math.isclose(self.low_freq_factor, self.high_freq_factor):
            smooth = (self.orig_max_position / wave - self.low_freq_factor) / (self.high_freq_factor - self.low_freq_factor)
        else:
            smooth = np.zeros_like(inv)
        mid = (1 - smooth) * inv / self.scaling_factor + smooth * inv
        return np.where(wave < high_wl, inv, np.where(wave > low_wl, inv / self.scaling_factor, mid)).astype(np.float32)


class YaRNScalingRotaryEmbedding(RotaryEmbedding):
    """yarn_rotary_pos_embedding.py:30-123: table length = original_max_position_embeddings * scaling_factor."""

    def __init__(self, kv_channels, rotary_percent=1.0, rotary_interleaved=False, seq_len_interpolation_factor=None,
                 rotary_base=10000.0, rotary_cos_format=0, rotary_dtype=torch.float16, scaling_factor=1.0,
                 original_max_position_embeddings=4096, beta_fast=32.0, beta_slow=1.0, mscale=1.0, mscale_all_dim=0.0,
                 extrapolation_factor=1.0, attn_factor=1.0, device="cuda"):
        self.scaling_factor = scaling_factor
        self.original_max_position_embeddings = original_max_position_embeddings
        self.beta_fast, self.beta_slow = beta_fast, beta_slow
        self.extrapolation_factor = extrapolation_factor
        self.attn_factor = attn_factor
        self.mscale = float(_yarn_get_mscale(scaling_factor, float(mscale)) /
                            _yarn_get_mscale(scaling_factor, float(mscale_all_dim)) * attn_factor)
        super().__init__(kv_channels, rotary_percent, rotary_interleaved, seq_len_interpolation_factor, rotary_base,
                         rotary_cos_format, rotary_dtype, original_max_position_embeddings, device)

    def _compute_inv_freq(self, base):
        pos = (np.float32(base) ** (np.arange(0, self.dim, 2, dtype=np.float32)[: self.dim // 2] / np.float32(self.dim))).astype(np.float32)
        extra = (1.0 / pos).astype(np.float32)
        inter = (1.0 / (np.float32(self.scaling_factor) * pos)).astype(np.float32)
        low, high = _yarn_find_correction_range(self.beta_fast, self.beta_slow, self.dim, base,
                                                self.original_max_position_embeddings)
        mask = (1 - _yarn_linear_ramp_mask(low, high, self.dim // 2)) * np.float32(self.extrapolation_factor)
        return (inter * (1 - mask) + extra * mask).astype(np.float32)

    def _num_positions(self):
        return int(self.max_position_embeddings * self.scaling_factor)

    def _mscale(self):
        return self.mscale


class FreqsMgr(nn.Module):
    """Legacy table owner (layers.py:1171-1333): ``increment(batch_valid_length)`` returns the rows for position
    batch_valid_length - 1 as (cos, sin, swap_mask); swap_mask is kept for signature parity (the rotate-half
    kernel does not need it).  extend_method in {None/"None", "LLAMA3", "YARN", "PI", "NTK", "LINEAR"}."""

    def __init__(self, head_dim, seq_length=None, max_position_embedding=4096, rotary_dtype=torch.float16, theta=10000,
                 scaling_factor=1.0, extend_method="None", parallel_config=None, is_dynamic=False, device="cuda"):
        super().__init__()
        if seq_length is not None and seq_length > max_position_embedding:
            max_position_embedding = seq_length
        method = (extend_method or "None").upper()
        theta = float(theta)
        if method == "NTK":
            theta *= scaling_factor
        freqs = _inv_freq_default(head_dim, theta)
        mscale = 1.0
        if method == "LINEAR":
            freqs = freqs / scaling_factor["factor"]
        elif method == "YARN":
            factor = scaling_factor["factor"]
            orig = scaling_factor["original_max_position_embeddings"]
            inter = (1.0 / (factor * theta ** (np.arange(0, head_dim, 2)[: head_dim // 2].astype(np.float32) / head_dim))).astype(np.float32)
            low, high = _yarn_find_correction_range(scaling_factor["beta_fast"], scaling_factor["beta_slow"], head_dim, theta, orig)
            mask = 1.0 - _yarn_linear_ramp_mask(low, high, head_dim // 2)
            freqs = (inter * (1 - mask) + freqs * mask).astype(np.float32)
            mscale = float(_yarn_get_mscale(factor, scaling_factor["mscale"]) / _yarn_get_mscale(factor, scaling_factor["mscale_all_dim"]))
        elif method == "LLAMA3":
            factor = scaling_factor["factor"]
            lo_f, hi_f = scaling_factor["low_freq_factor"], scaling_factor["high_freq_factor"]
            old = scaling_factor["original_max_position_embeddings"]
            low_wl, high_wl = old / lo_f, old / hi_f
            new = []
            for f in freqs:
                wl = 2 * math.pi / f
                if wl < high_wl:
                    new.append(f)
                elif wl > low_wl:
                    new.append(f / factor)
                else:
                    smooth = (old / wl - lo_f) / (hi_f - lo_f)
                    new.append((1 - smooth) * f / factor + smooth * f)
            freqs = np.array(new, dtype=freqs.dtype)
        elif method not in ("NONE", "PI", "NTK"):
            raise ValueError(f"unsupported extend_method {extend_method!r}")
        if method == "PI":
            t = np.arange(0, max_position_embedding / scaling_factor, 1 / scaling_factor).astype(np.float32)
        else:
            t = np.arange(0, max_position_embedding, 1).astype(np.float32)
        emb = np.outer(t, freqs).astype(np.float32)
        emb = np.concatenate((emb, emb), axis=-1)
        self.head_dim = head_dim
        self.is_dynamic = is_dynamic
        self.register_buffer("freqs_cos", torch.from_numpy((np.cos(emb) * mscale).astype(np.float32)).to(device=device, dtype=rotary_dtype), persistent=False)
        self.register_buffer("freqs_sin", torch.from_numpy((np.sin(emb) * mscale).astype(np.float32)).to(device=device, dtype=rotary_dtype), persistent=False)
        self.swap_mask = None

    def forward(self, seq_length=None):
        return self.freqs_cos[:seq_length], self.freqs_sin[:seq_length], self.swap_mask

    construct = forward

    def prefill(self, bs=None, seq_length=None):
        if self.is_dynamic:
            return self.freqs_cos, self.freqs_sin, self.swap_mask
        return self.freqs_cos[:seq_length].repeat(bs, 1), self.freqs_sin[:seq_length].repeat(bs, 1), self.swap_mask

    def increment(self, batch_valid_length):
        idx = (batch_valid_length - 1).to(torch.long)
        return self.freqs_cos.index_select(0, idx), self.freqs_sin.index_select(0, idx), self.swap_mask

    def increment_multi_ids(self, indices):
        idx = indices.reshape(-1).to(torch.long)
        return self.freqs_cos.index_select(0, idx), self.freqs_sin.index_select(0, idx), self.swap_mask
