"""RMSNorm / LayerNorm / SiLU-mul / linear / gated MLP.  Test infrastructure only.

Follows:
  RMSNorm    mindformers/models/llama/llama_layer.py:214-228 (fused: inside compute type; self-defined:
             gamma applied after casting back), mindformers/parallel_core/inference/transformer/norm.py:110-115
  LayerNorm  mindformers/parallel_core/inference/transformer/norm.py:31-70
  SiLU*mul   mindformers/parallel_core/inference/transformer/activation.py:23-71, llama_layer.py:69-70,
             tests/.../test_activation/run_infer_activation.py:71-72
  linear     mindformers/modules/layers.py:510-533; tensor_parallel/layers.py:158-199,389-415  (W is [out, in])
  MLP        mindformers/parallel_core/inference/transformer/mlp.py:130-147 (contiguous [gate | hidden] split),
             llama_layer.py:412-441 (legacy interleaved (ffn, 2) split for ffn_concat)
"""
import numpy as np

from .numerics import round_to


def rms_norm(x, gamma, eps, gamma_after_cast=None):
    """x * rsqrt(mean(x^2) + eps) * gamma in float64.  ``gamma_after_cast`` names a storage dtype: the
    normalised value is rounded through it before the gamma multiply (the self-defined variant)."""
    x = np.asarray(x, dtype=np.float64)
    g = np.asarray(gamma, dtype=np.float64)
    inv = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    y = x * inv
    if gamma_after_cast is not None:
        y = round_to(y, gamma_after_cast).astype(np.float64)
    return y * g


def layer_norm(x, gamma, beta, eps):
    x = np.asarray(x, dtype=np.float64)
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    y = (x - mu) / np.sqrt(var + eps) * np.asarray(gamma, dtype=np.float64)
    if beta is not None:
        y = y + np.asarray(beta, dtype=np.float64)
    return y


def silu(x):
    x = np.asarray(x, dtype=np.float64)
    return x / (1.0 + np.exp(-x))


def silu_mul(gate, up):
    """silu(gate) * up."""
    return silu(gate) * np.asarray(up, dtype=np.float64)


def linear(x, weight, bias=None):
    """y = x @ W^T (+ bias); W [out, in]; float64."""
    y = np.asarray(x, dtype=np.float64) @ np.asarray(weight, dtype=np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def mlp(x, fc1_weight, fc2_weight, fc1_bias=None, fc2_bias=None, gated=True, interleaved=False,
        act_dtype=None):
    """fc2(act(fc1 x)).  gated: fc1 rows are [gate | hidden] (contiguous halves) or, with
    ``interleaved``, rows alternate gate,hidden.  ``act_dtype`` rounds the materialised intermediates
    (fc1 output and the activation product) through a storage dtype, as a device path that writes
    them to memory does."""
    h = linear(x, fc1_weight, fc1_bias)
    if act_dtype is not None:
        h = round_to(h, act_dtype).astype(np.float64)
    if gated:
        if interleaved:
            gate, up = h[..., 0::2], h[..., 1::2]
        else:
            f = h.shape[-1] // 2
            gate, up = h[..., :f], h[..., f:]
        a = silu_mul(gate, up)
    else:
        a = silu(h)
    if act_dtype is not None:
        a = round_to(a, act_dtype).astype(np.float64)
    return linear(a, fc2_weight, fc2_bias)
