"""Rotary position embedding tables and the rotate-half application.  Test infrastructure only.

Follows:
  tables, default   mindformers/parallel_core/inference/base_models/common/embeddings/rotary_pos_embedding.py:85-112
                    (= legacy mindformers/modules/layers.py:1191-1192,1252-1260)
  tables, Llama3    rotary_pos_embedding.py:189-211 (= layers.py:1224-1250)
  tables, YaRN      .../yarn_rotary_pos_embedding.py:86-123,126-173 (= layers.py:1199-1222)
  decode gather     rotary_pos_embedding.py:118-123 (row = position), layers.py:1310-1314 (row = L-1)
  application       ApplyRotaryPosEmb(cos_format=2) call sites infer_attention.py:50-57,
                    rotary_pos_embedding.py:75,146; unfused rotate-half layers.py:1514-1542
"""
import math

import numpy as np

from .numerics import round_to


def rope_inv_freq_default(dim, base=10000.0):
    # float32 throughout, as the reference builds the table in float32
    expo = (np.arange(0, dim, 2, dtype=np.float32)[: dim // 2] / np.float32(dim)).astype(np.float32)
    return (1.0 / (np.float32(base) ** expo)).astype(np.float32)


def rope_inv_freq_llama3(dim, base, scaling_factor, low_freq_factor, high_freq_factor, orig_max_position):
    inv = rope_inv_freq_default(dim, base)
    low_wl = orig_max_position / low_freq_factor
    high_wl = orig_max_position / high_freq_factor
    wave = (2 * math.pi / inv).astype(np.float32)
    if not math.isclose(low_freq_factor, high_freq_factor):
        smooth = (orig_max_position / wave - low_freq_factor) / (high_freq_factor - low_freq_factor)
    else:
        smooth = np.zeros_like(inv)
    mid = (1 - smooth) * inv / scaling_factor + smooth * inv
    out = np.where(wave < high_wl, inv, np.where(wave > low_wl, inv / scaling_factor, mid))
    return out.astype(np.float32)


def yarn_mscale(scale=1.0, mscale=1.0):
    if scale <= 1:
        return 1.0
    return 0.1 * mscale * math.log(scale) + 1.0


def _yarn_correction_dim(num_rot, dim, base, max_pos):
    return (dim * math.log(max_pos / (num_rot * 2 * math.pi))) / (2 * math.log(base))


def rope_inv_freq_yarn(dim, base, scaling_factor, orig_max_position, beta_fast=32.0, beta_slow=1.0,
                       extrapolation_factor=1.0):
    pos = (np.float32(base) ** (np.arange(0, dim, 2, dtype=np.float32)[: dim // 2] / np.float32(dim)))
    pos = pos.astype(np.float32)
    extra = (1.0 / pos).astype(np.float32)
    inter = (1.0 / (np.float32(scaling_factor) * pos)).astype(np.float32)
    low = max(math.floor(_yarn_correction_dim(beta_fast, dim, base, orig_max_position)), 0)
    high = min(math.ceil(_yarn_correction_dim(beta_slow, dim, base, orig_max_position)), dim - 1)
    lo, hi = float(low), float(high)
    if lo == hi:
        hi += 0.001
    ramp = np.clip((np.arange(dim // 2, dtype=np.float32) - lo) / (hi - lo), 0, 1).astype(np.float32)
    mask = (1 - ramp) * np.float32(extrapolation_factor)
    return (inter * (1 - mask) + extra * mask).astype(np.float32)


def rope_cos_sin_table(inv_freq, num_positions, mscale=1.0, table_dtype="fp32"):
    """cos/sin of concat(freqs, freqs) over [num_positions, dim], times mscale, stored in table_dtype."""
    seq = np.arange(0, num_positions, 1, dtype=np.float32)
    freqs = np.outer(seq, np.asarray(inv_freq, dtype=np.float32)).astype(np.float32)
    emb = np.concatenate((freqs, freqs), axis=-1)
    cos = round_to(np.cos(emb) * np.float32(mscale), table_dtype)
    sin = round_to(np.sin(emb) * np.float32(mscale), table_dtype)
    return cos, sin


def apply_rotary_half(x, cos, sin, n_head):
    """x [T, n_head*D]; cos/sin [T, D] (one row per token).  out = x*cos + rotate_half(x)*sin with
    rotate_half(x) = concat(-x[D/2:], x[:D/2]) per head.  float64."""
    t = x.shape[0]
    d = x.shape[1] // n_head
    xh = np.asarray(x, dtype=np.float64).reshape(t, n_head, d)
    c = np.asarray(cos, dtype=np.float64).reshape(t, 1, d)
    s = np.asarray(sin, dtype=np.float64).reshape(t, 1, d)
    rot = np.concatenate((-xh[..., d // 2:], xh[..., : d // 2]), axis=-1)
    return (xh * c + rot * s).reshape(t, n_head * d)
