"""W8A16 / W8A8 quantized linear arithmetic.  Test infrastructure only.

PARITY UNPINNED against the reference: these cells live in the third-party ``mindspore_gs`` package
(>= 0.6.0, otherwise unpinned; mindformers/version_control.py:326-334) and lower to the Ascend primitives
WeightQuantBatchMatmul / DynamicQuant / QuantBatchMatmul.  MindFormers only dispatches to them
(mindformers/modules/quantizers/rtn_quantizer.py:61-67, ptq_quantizer.py:52-59,
smooth_quant_quantizer.py:61-67; configs mindformers/utils/quantization_config.py:257-300,404-478) and
its tests pin no numerics for them (tests/st/test_ut/test_models/test_auto/test_auto_quantizer.py:31-77).
The convention stated here is this build's contract:

  weights     s_n = max_k |W[n,k]| / 127 ; w_i8 = clip(rint(W / s_n), -127, 127)   (rint: ties to even)
  W8A16       y = (x . w_i8^T) * s_n (+ bias)             x in bf16/fp16, accumulate wide, scale after
  act quant   xs = x * smooth ; s_t = max_k |xs[t,k]| / 127 (float32) ; q = clip(rint(xs / s_t), -128, 127)
  W8A8        acc = q . w_i8^T  (exact int32) ; y = acc * s_t * s_n (+ bias)

What *is* fixed independently of convention, and tested: int32 accumulators equal exact integer matmul;
power-of-two scales with small-integer activations make W8A16 exact; the int8 grid round-trips.
"""
import numpy as np


def quantize_weight_int8(weight):
    """Symmetric per-output-channel int8.  weight [out, in] -> (w_i8 [out, in] int8, scale [out] float32)."""
    w = np.asarray(weight, dtype=np.float32).astype(np.float64)
    amax = np.abs(w).max(axis=1)
    scale = (amax / 127.0).astype(np.float32)           # the stored scale is float32
    safe = np.where(scale > 0, scale, np.float32(1.0)).astype(np.float64)
    q = np.clip(np.rint(w / safe[:, None]), -127, 127).astype(np.int8)   # quotient in float64, ties to even
    return q, scale


def w8a16_linear(x, w_i8, scale, bias=None):
    """float64 reference of y = (x . w_i8^T) * scale (+ bias)."""
    acc = np.asarray(x, dtype=np.float64) @ np.asarray(w_i8, dtype=np.float64).T
    y = acc * np.asarray(scale, dtype=np.float64)[None, :]
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def dynamic_quant_per_token(x, smooth=None):
    """Per-token dynamic int8.  All float32, in this exact operation order:
    xs = x*smooth; s = max|xs| / 127; q = clip(rint(xs / s), -128, 127).  Zero rows get s = 0, q = 0 ...
    returns (q int8 [T,K], s float32 [T])."""
    xs = np.asarray(x, dtype=np.float32)
    if smooth is not None:
        xs = (xs * np.asarray(smooth, dtype=np.float32)[None, :]).astype(np.float32)
    amax = np.abs(xs).max(axis=1).astype(np.float32)
    s = (amax / np.float32(127.0)).astype(np.float32)
    safe = np.where(s > 0, s, np.float32(1.0)).astype(np.float32)
    q = np.clip(np.rint((xs / safe[:, None]).astype(np.float32)), -128, 127).astype(np.int8)
    return q, s


def static_quant_per_tensor(x, act_scale, smooth=None):
    """Static per-tensor int8 (the SmoothQuant method's activation quantiser; PARITY UNPINNED like the per-token
    form, symmetric by this build's declaration): xs = x*smooth; q = clip(rint(xs / act_scale), -128, 127), float32
    throughout.  Returns (q int8 [T,K], s float32 [T] = act_scale for every row)."""
    xs = np.asarray(x, dtype=np.float32)
    if smooth is not None:
        xs = (xs * np.asarray(smooth, dtype=np.float32)[None, :]).astype(np.float32)
    s = np.float32(act_scale)
    safe = s if s > 0 else np.float32(1.0)
    q = np.clip(np.rint((xs / safe).astype(np.float32)), -128, 127).astype(np.int8)
    return q, np.full(xs.shape[0], s, dtype=np.float32)


def int8_gemm_i32(xq, w_i8):
    """Exact int32 accumulators acc[t,n] = sum_k xq[t,k]*w[n,k] (computed in int64, checked to fit)."""
    acc = np.asarray(xq, dtype=np.int64) @ np.asarray(w_i8, dtype=np.int64).T
    assert np.abs(acc).max(initial=0) < 2 ** 31
    return acc.astype(np.int32)


def w8a8_linear(xq, x_scale, w_i8, w_scale, bias=None):
    """float64 reference of y = acc * s_t * s_n (+ bias)."""
    acc = int8_gemm_i32(xq, w_i8).astype(np.float64)
    y = acc * np.asarray(x_scale, dtype=np.float64)[:, None] * np.asarray(w_scale, dtype=np.float64)[None, :]
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def quantize_kv_int8(x, scale, offset=None):
    """Per-channel int8 quantisation of key / value rows: q = clip(rint(x / scale + offset), -128, 127), quotient
    in float64.  PARITY UNPINNED (the reference only configures an int8 cache, quantization_config.py:196-250;
    the arithmetic belongs to golden-stick cells and vendor kernels): this build's declared convention."""
    q = np.asarray(x, dtype=np.float64) / np.asarray(scale, dtype=np.float64)
    if offset is not None:
        q = q + np.asarray(offset, dtype=np.float64)
    return np.clip(np.rint(q), -128, 127).astype(np.int8)


def quantize_kv_int8_per_token(x):
    """Per-token int8 quantisation of key / value rows [T, n_kv * D] (kvcache_quant_granularity per_token,
    quantization_config.py:206-207): one scale per token row over all its kv heads, the arithmetic of
    dynamic_quant_per_token without a multiplier.  Returns (q int8, s float32 [T]); x ~ q * s.  PARITY UNPINNED like
    the per-channel form: the reference only configures the mode."""
    return dynamic_quant_per_token(x)


def dequantize_kv_int8(q, scale, offset=None):
    """x ~ (q - offset) * scale in float64 (the inverse convention of quantize_kv_int8)."""
    x = np.asarray(q, dtype=np.float64)
    if offset is not None:
        x = x - np.asarray(offset, dtype=np.float64)
    return x * np.asarray(scale, dtype=np.float64)


def quantize_weight_int4(weight, group_size=0):
    """Symmetric 4-bit weights, per output channel (group_size 0) or per channel and group of ``group_size`` input
    columns: s = max|w| / 7 over the group (float32), q = clip(rint(w / s), -8, 7) with the quotient in float64.
    Returns (q int8 [N, K] of values -8 .. 7, s float32 [N] or [K / group_size, N]).  PARITY UNPINNED against the
    reference like the int8 convention (golden-stick's A16W4 arithmetic is not vendored); held to what the
    mathematics fixes by tests/test_host_logic.py (rails, half-step round trip, exactness on power-of-two grids)."""
    w = np.asarray(weight, dtype=np.float64)
    n, k = w.shape
    g = group_size or k
    wg = w.reshape(n, k // g, g)
    scale = (np.abs(wg).max(axis=2) / 7.0).astype(np.float32)                       # [N, K/g]
    safe = np.where(scale > 0, scale, 1.0).astype(np.float64)
    q = np.clip(np.rint(wg / safe[:, :, None]), -8, 7).astype(np.int8).reshape(n, k)
    return q, (scale[:, 0] if group_size == 0 else np.ascontiguousarray(scale.T))


def w4a16_linear(x, w_q, scale, group_size=0, bias=None):
    """y = sum over groups of (x_g . q_g^T) * s_g (+ bias): integer weights times activations summed per group, the
    group's scale applied to the group's sum.  float64."""
    x = np.asarray(x, dtype=np.float64)
    q = np.asarray(w_q, dtype=np.float64)
    n, k = q.shape
    g = group_size or k
    s = np.asarray(scale, dtype=np.float64)
    s = s.reshape(1, n) if group_size == 0 else s                                    # [K/g, N]
    y = np.zeros((x.shape[0], n))
    for i in range(k // g):
        y += (x[:, i * g:(i + 1) * g] @ q[:, i * g:(i + 1) * g].T) * s[i][None, :]
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def pack_qint4x2(w_q):
    """int8 [N, K] of values -8 .. 7 -> int8 [N, K/2]: element 2j in the low nibble of byte j, 2j + 1 in the high."""
    u = (np.asarray(w_q).astype(np.int16) & 15).astype(np.uint8)
    return (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8).view(np.int8)


def unpack_qint4x2(w):
    u = np.asarray(w).view(np.uint8)
    lo, hi = (u & 15).astype(np.int8), (u >> 4).astype(np.int8)
    lo, hi = np.where(lo > 7, lo - 16, lo), np.where(hi > 7, hi - 16, hi)
    return np.stack((lo, hi), axis=-1).reshape(u.shape[0], -1).astype(np.int8)
