"""Rounding helpers and the reference's accuracy criterion.  Test infrastructure only.

``double_benchmark`` restates the comparator the reference's inference unit
tests use (tests/utils/double_benchmark.py:149-206 thresholds, :210-276 small /
normal value statistics, :367-419 flow): the device output is judged by how far
it is from an fp32 golden *relative to* how far a second device (the stored
"GPU" vectors) is from the same golden.
"""
from dataclasses import dataclass, field

import numpy as np


def round_bf16(x):
    """Round float32 values to the nearest bfloat16 (ties to even); returns float32."""
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    u = a.view(np.uint32).astype(np.uint64)
    bias = ((u >> 16) & 1) + 0x7FFF
    r = ((u + bias) & 0xFFFF0000).astype(np.uint32)
    out = r.view(np.float32).reshape(a.shape)
    nan = np.isnan(a)
    if nan.any():
        out = np.where(nan, np.float32(np.nan), out)
    return out


def round_fp16(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_to(x, dtype):
    """dtype in {'bf16','fp16','fp32','fp64'}: round through that storage type."""
    if dtype == "bf16":
        return round_bf16(x)
    if dtype == "fp16":
        return round_fp16(x)
    if dtype == "fp32":
        return np.asarray(x, dtype=np.float32)
    if dtype == "fp64":
        return np.asarray(x, dtype=np.float64)
    raise ValueError(f"unknown dtype {dtype}")


@dataclass
class DoubleBenchmarkResult:
    ok: bool = True
    messages: list = field(default_factory=list)
    max_re_cv: float = None
    avg_re_cv: float = None
    rmse_cv: float = None
    eb_cv: float = None
    small_err_ratio_cv: float = None


_SMALL = {"float32": 2.0 ** -20, "float16": 2.0 ** -10, "bfloat16": 2.0 ** -10}
_ABS = {"float32": 2.0 ** -30, "float16": 1e-16, "bfloat16": 1e-16}
_ERR = {"float32": 2.0 ** -14, "float16": 2.0 ** -11, "bfloat16": 2.0 ** -8}


def _small_info(actual, golden, finite, small_thd, abs_thd):
    ae = np.abs(actual - golden)
    small = (np.abs(golden) < small_thd) & finite
    err = (ae > abs_thd) & small
    cnt = int(small.sum())
    return (None if cnt == 0 else err.sum() / cnt)


def _normal_info(actual, golden, finite, small_thd):
    ag = np.abs(golden)
    re = np.abs(actual - golden) / np.clip(ag, small_thd, None)
    normal = (ag >= small_thd) & finite
    if int(normal.sum()) == 0:
        return None, None
    return float(re[normal].max()), float(re[normal].mean())


def _cv(a, b, err_thd):
    if a is None or b is None:
        return None
    return abs(a) / max(abs(b), err_thd)


def double_benchmark(device, second_device, golden, dtype="bfloat16",
                     max_re_cv=10, avg_re_cv=2, rmse_cv=2, small_err_ratio_cv=2, eb_cv=2):
    """Reference criterion (tests/utils/double_benchmark.py:367-419).

    ``device`` plays the role of the reference's "npu" argument, ``second_device``
    its "gpu" argument.  Error-balance violations on fewer than 1e6 samples are
    reported but do not fail, as in the reference (:349-365).
    """
    golden = np.asarray(golden, dtype=np.float64).ravel()
    dev = np.asarray(device, dtype=np.float64).ravel()
    sec = np.asarray(second_device, dtype=np.float64).ravel()
    res = DoubleBenchmarkResult()
    small_thd, abs_thd, err_thd = _SMALL[dtype], _ABS[dtype], _ERR[dtype]

    nan_any = np.isnan(dev) | np.isnan(sec) | np.isnan(golden)
    nan_err = (np.isnan(dev) != np.isnan(golden)) & (np.isnan(dev) != np.isnan(sec))
    inf_any = np.isinf(dev) | np.isinf(sec) | np.isinf(golden)
    inf_err = (dev != golden) & (dev != sec) & inf_any
    finite = ~(nan_any | inf_any)
    if int((nan_err | inf_err).sum()):
        res.ok = False
        res.messages.append("inf/nan mismatch")

    d_small = _small_info(dev, golden, finite, small_thd, abs_thd)
    s_small = _small_info(sec, golden, finite, small_thd, abs_thd)
    d_max, d_avg = _normal_info(dev, golden, finite, small_thd)
    s_max, s_avg = _normal_info(sec, golden, finite, small_thd)

    def rmse(a):
        return float(np.sqrt(np.mean(np.square(a[finite] - golden[finite]))))

    def eb(a):
        return float(np.mean((a[finite] - golden[finite]) / np.clip(np.abs(golden[finite]), 1, None)))

    res.max_re_cv = _cv(d_max, s_max, err_thd)
    res.avg_re_cv = _cv(d_avg, s_avg, err_thd)
    res.rmse_cv = _cv(rmse(dev), rmse(sec), err_thd)
    res.eb_cv = _cv(eb(dev), eb(sec), err_thd)
    res.small_err_ratio_cv = _cv(d_small, s_small, err_thd)

    n = int(finite.sum())

    def check(val, thd, what, soft=False):
        if val is not None and val > thd:
            if soft and n < 1e6:
                res.messages.append(f"(insufficient samples {n}) {what} {val} > {thd}")
            else:
                res.ok = False
                res.messages.append(f"{what} {val} > {thd}")

    check(res.eb_cv, eb_cv, "error balance cv", soft=True)
    check(res.max_re_cv, max_re_cv, "max relative error cv")
    check(res.avg_re_cv, avg_re_cv, "mean relative error cv")
    check(res.rmse_cv, rmse_cv, "rmse cv")
    check(res.small_err_ratio_cv, small_err_ratio_cv, "small value error ratio cv")
    return res
