"""Quantization configs of the three methods the reference dispatches (rtn / ptq / smooth_quant) with its
argument checks — mindformers/utils/quantization_config.py:64-595.  golden-stick's enums are replaced by the
plain strings the YAML files use (e.g. research/deepseek3/deepseek_r1_671b/predict_deepseek_r1_671b_w8a8.yaml:89-92).

What the kernels here implement of the accepted space: int8 weights (per output channel), activations None
(W8A16) or int8 per token (W8A8, PTQ method) optionally with smooth outlier suppression.  Accepted-by-config
but not built (per-tensor activations, int4x2 / per-group weights, int8 KV cache, awq / outlier-suppression+,
GPTQ recovery) raise NotImplementedError when a quantizer is asked to convert a model with them.
"""
import copy
import json
import re
from collections import OrderedDict
from enum import Enum

DTYPES = {"None": None, None: None, "int8": "int8", "int4": "int4x2", "float16": "float16", "bfloat16": "bfloat16",
          "float32": "float32"}
OUTLIERS = {"None": "none", None: "none", "smooth": "smooth", "awq": "awq", "outlier-suppression+": "outlier-suppression+"}
PRECISION_RECOVERY = {"none": "none", "gptq": "gptq"}
GRANULARITY = {"per_tensor", "per_channel", "per_token", "per_group"}


class QuantizationMethod(str, Enum):
    RTN = "rtn"
    PTQ = "ptq"
    SMOOTH_QUANT = "smooth_quant"


def _dtype(name, what):
    if name not in DTYPES:
        raise ValueError(f"unknown {what} {name!r}")
    return DTYPES[name]


class QuantizationConfigMixin:
    """from_dict / to_dict / to_json helpers (quantization_config.py:64-170)."""

    @classmethod
    def from_dict(cls, config_dict, return_unused_kwargs=False, **kwargs):
        config = cls(**config_dict)
        to_remove = []
        for key, value in kwargs.items():
            if hasattr(config, key):
                setattr(config, key, value)
                to_remove.append(key)
        for key in to_remove:
            kwargs.pop(key, None)
        if return_unused_kwargs:
            return config, kwargs
        return config

    def to_dict(self):
        return copy.deepcopy({k: (v.value if isinstance(v, Enum) else v) for k, v in self.__dict__.items()
                              if not isinstance(v, OrderedDict)})

    def to_json_string(self):
        return json.dumps(self.to_dict(), indent=2, sort_keys=True, default=str) + "\n"

    def to_json_file(self, json_file_path):
        with open(json_file_path, "w", encoding="utf-8") as writer:
            writer.write(self.to_json_string())

    def __repr__(self):
        return f"{self.__class__.__name__} {self.to_json_string()}"

    def _common(self, quant_method, mode, backend, modules_to_not_convert, algorithm_args):
        self.quant_method = quant_method.value if isinstance(quant_method, Enum) else quant_method
        self.mode = mode
        self.backend = backend
        if modules_to_not_convert is not None and (not isinstance(modules_to_not_convert, (list, tuple)) or
                                                   any(not isinstance(m, str) for m in modules_to_not_convert)):
            raise TypeError("modules_to_not_convert must be a list of str")
        self.opname_blacklist = list(modules_to_not_convert or [])
        self.algo_args = algorithm_args if algorithm_args is not None else {}
        if self.mode != "deploy":
            raise ValueError(f"Only support ['deploy'] but found {self.mode}")
        if self.backend not in ("ascend", "mi355x"):
            raise ValueError(f"Only support ['ascend'] but found {self.backend}")


class RtnConfig(QuantizationConfigMixin):
    """Round-to-nearest: A16W8 (optionally C8) only (quantization_config.py:173-300)."""

    def __init__(self, quant_method=QuantizationMethod.RTN, mode="deploy", backend="ascend", weight_dtype="int8",
                 activation_dtype=None, kvcache_dtype=None, modules_to_not_convert=None, outliers_suppression="None",
                 algorithm_args=None, act_quant_granularity="per_tensor", kvcache_quant_granularity="per_channel",
                 **kwargs):
        self._common(quant_method, mode, backend, modules_to_not_convert, algorithm_args)
        self.weight_quant_dtype = _dtype(weight_dtype, "weight_dtype")
        self.kvcache_quant_dtype = _dtype(kvcache_dtype, "kvcache_dtype")
        self.act_quant_dtype = _dtype(activation_dtype, "activation_dtype")
        if outliers_suppression not in OUTLIERS:
            raise ValueError(f"unknown outliers_suppression {outliers_suppression!r}")
        self.outliers_suppression = OUTLIERS[outliers_suppression]
        self.act_quant_granularity = act_quant_granularity
        self.kvcache_quant_granularity = kvcache_quant_granularity
        self.init_check()

    def init_check(self):
        if self.weight_quant_dtype not in (None, "int8"):
            raise ValueError(f"Only support quant weights in [None, 'int8'] but found {self.weight_quant_dtype}")
        if self.act_quant_dtype not in (None, "int8"):
            raise ValueError(f"Only support activation weights in [None, 'int8'] but found {self.act_quant_dtype}")
        if self.kvcache_quant_dtype not in (None, "int8"):
            raise ValueError(f"Only support kvcache weights in [None, 'int8'] but found {self.kvcache_quant_dtype}")
        if self.act_quant_dtype is not None or self.outliers_suppression != "none":
            raise ValueError("RTN algorithm only support A16W8、C8、A16W8C8, please set the correct configuration."
                             f"Now the configuration is act_quant_dtype={self.act_quant_dtype},"
                             f"weight_quant_dtype={self.weight_quant_dtype},"
                             f"kvcache_quant_dtype={self.kvcache_quant_dtype},"
                             f"outliers_suppression={self.outliers_suppression}")
        if self.act_quant_granularity not in ("per_tensor", "per_token"):
            raise ValueError(f"Only support act_quant_granularity in ['per_tensor', 'per_token'] but found "
                             f"{self.act_quant_granularity}")
        if self.kvcache_quant_granularity not in ("per_channel", "per_token"):
            raise ValueError(f"Only support kvcache_quant_granularity in ['per_channel', 'per_token'] but found "
                             f"{self.kvcache_quant_granularity}")
        if (self.weight_quant_dtype != "int8" or self.act_quant_dtype != "int8") and self.act_quant_granularity == "per_token":
            raise ValueError("when self.act_quant_granularity is per_token, weight_quant_dtype and act_quant_dtype "
                             "must be int8.")
        if self.kvcache_quant_dtype != "int8" and self.kvcache_quant_granularity == "per_token":
            raise ValueError("when self.kvcache_quant_granularity is per_token, self.kvcache_quant_dtype must be int8.")


class PtqConfig(QuantizationConfigMixin):
    """Post-training quantization (quantization_config.py:303-478)."""

    def __init__(self, quant_method=QuantizationMethod.PTQ, mode="deploy", backend="ascend", weight_dtype="int8",
                 activation_dtype=None, kvcache_dtype=None, modules_to_not_convert=None, outliers_suppression="None",
                 precision_recovery="none", algorithm_args=None, act_quant_granularity="per_tensor",
                 kvcache_quant_granularity="per_channel", weight_quant_granularity="per_channel", group_size=0,
                 layer_policies=None, **kwargs):
        self._common(quant_method, mode, backend, modules_to_not_convert, algorithm_args)
        self.weight_quant_dtype = _dtype(weight_dtype, "weight_dtype")
        self.kvcache_quant_dtype = _dtype(kvcache_dtype, "kvcache_dtype")
        self.act_quant_dtype = _dtype(activation_dtype, "activation_dtype")
        self.act_quant_granularity = act_quant_granularity
        self.kvcache_quant_granularity = kvcache_quant_granularity
        self.weight_quant_granularity = weight_quant_granularity
        if outliers_suppression not in OUTLIERS:
            raise ValueError(f"Only support outliers suppression in {sorted(set(OUTLIERS.values()))} but found "
                             f"{outliers_suppression}")
        self.outliers_suppression = OUTLIERS[outliers_suppression]
        if precision_recovery not in PRECISION_RECOVERY:
            raise ValueError(f"Only support precision recovery in ['none', 'gptq'] but found {precision_recovery}")
        self.precision_recovery = PRECISION_RECOVERY[precision_recovery]
        if not isinstance(group_size, int):
            raise TypeError("group_size must be an int")
        self.group_size = group_size
        if layer_policies is not None and not isinstance(layer_policies, dict):
            raise TypeError(f"layer_policies should be an OrderedDict, bug got {type(layer_policies)}.")
        self.layer_policies = OrderedDict()
        for key, value in (layer_policies or {}).items():
            if not isinstance(key, str):
                raise TypeError("all key of layer_policies should be a string.")
            try:
                re.compile(key)
            except re.error as e:
                raise TypeError("The regular string of layer_policies not correct, please check and try again.") from e
            self.layer_policies[key] = value if isinstance(value, PtqConfig) else PtqConfig.from_dict(value)
        self.init_check()

    def init_check(self):
        if self.weight_quant_dtype not in (None, "int8", "int4x2"):
            raise ValueError(f"Only support quant weights in [None, 'int8', 'int4x2'] but found {self.weight_quant_dtype}")
        if self.act_quant_dtype not in (None, "int8"):
            raise ValueError(f"Only support activation weights in [None, 'int8'] but found {self.act_quant_dtype}")
        if self.kvcache_quant_dtype not in (None, "int8"):
            raise ValueError(f"Only support kvcache weights in [None, 'int8'] but found {self.kvcache_quant_dtype}")
        if self.weight_quant_dtype is None and self.act_quant_dtype == "int8":
            raise ValueError("PTQ algorithm not support only quant activation.")
        if (self.weight_quant_dtype != "int8" or self.act_quant_dtype != "int8") and self.act_quant_granularity == "per_token":
            raise ValueError("when self.act_quant_granularity is per_token, weight_quant_dtype and act_quant_dtype "
                             "must be int8.")
        if self.act_quant_granularity not in ("per_tensor", "per_token"):
            raise ValueError(f"Only support act_quant_granularity in ['per_tensor', 'per_token'] but found "
                             f"{self.act_quant_granularity}")
        if self.kvcache_quant_granularity not in ("per_channel", "per_token"):
            raise ValueError(f"Only support kvcache_quant_granularity in ['per_channel', 'per_token'] but found "
                             f"{self.kvcache_quant_granularity}")
        if self.weight_quant_granularity not in ("per_channel", "per_group"):
            raise ValueError(f"Only support weight_quant_granularity in ['per_channel', 'per_group'] but found "
                             f"{self.weight_quant_granularity}")
        if self.kvcache_quant_dtype != "int8" and self.kvcache_quant_granularity == "per_token":
            raise ValueError("when self.kvcache_quant_granularity is per_token, self.kvcache_quant_dtype must be int8.")
        if self.group_size not in (0, 64, 128):
            raise ValueError(f"Only support group_size in [0, 64, 128] but found {self.group_size}")


class SmoothQuantConfig(QuantizationConfigMixin):
    """SmoothQuant method: A8W8 with per-tensor activations only (quantization_config.py:481-595)."""

    def __init__(self, quant_method=QuantizationMethod.SMOOTH_QUANT, mode="deploy", backend="ascend",
                 weight_dtype="int8", activation_dtype="int8", kvcache_dtype=None, modules_to_not_convert=None,
                 outliers_suppression="smooth", algorithm_args=None, act_quant_granularity="per_tensor",
                 kvcache_quant_granularity="per_channel", **kwargs):
        self._common(quant_method, mode, backend, modules_to_not_convert, algorithm_args)
        self.weight_quant_dtype = _dtype(weight_dtype, "weight_dtype")
        self.kvcache_quant_dtype = _dtype(kvcache_dtype, "kvcache_dtype")
        self.act_quant_dtype = _dtype(activation_dtype, "activation_dtype")
        if outliers_suppression not in OUTLIERS:
            raise ValueError(f"unknown outliers_suppression {outliers_suppression!r}")
        self.outliers_suppression = OUTLIERS[outliers_suppression]
        self.act_quant_granularity = act_quant_granularity
        self.kvcache_quant_granularity = kvcache_quant_granularity
        self.init_check()

    def init_check(self):
        if self.weight_quant_dtype not in ("int8",):
            raise ValueError(f"Only support quant weights in ['int8'] but found {self.weight_quant_dtype}")
        if self.act_quant_dtype not in (None, "int8"):
            raise ValueError(f"Only support activation weights in [None, 'int8'] but found {self.act_quant_dtype}")
        if self.kvcache_quant_dtype not in (None, "int8"):
            raise ValueError(f"Only support kvcache weights in [None, 'int8'] but found {self.kvcache_quant_dtype}")
        if self.act_quant_granularity != "per_tensor" or self.kvcache_quant_granularity != "per_channel":
            raise ValueError("Only support act_quant_granularity is per_tensor and kvcache_quant_granularity is "
                             f"per_channel but found act_quant_granularity is {self.act_quant_granularity} and "
                             f"kvcache_quant_granularity is {self.kvcache_quant_granularity}.")
        do_a8w8 = (self.act_quant_dtype == "int8" and self.weight_quant_dtype == "int8" and
                   self.outliers_suppression == "smooth" and self.kvcache_quant_dtype is None)
        if not do_a8w8:
            raise ValueError("SmoothQuant algorithm only support A8W8, please set act_quant_dtype=int8,"
                             "weight_quant_dtype=int8 and outliers_suppression='smooth'."
                             f"Now the configuration is act_quant_dtype={self.act_quant_dtype},"
                             f"weight_quant_dtype={self.weight_quant_dtype},"
                             f"kvcache_quant_dtype={self.kvcache_quant_dtype},"
                             f"outliers_suppression={self.outliers_suppression}")
