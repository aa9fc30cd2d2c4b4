"""Quantizer base class: the hooks build_network drives (mindformers/modules/quantizers/base.py:30-234,
called at mindformers/models/build_model.py:97-100) and the cell replacement golden-stick's
``algo.apply(model); algo.convert(model)`` performs in DEPLOY mode."""
import re
from abc import ABC, abstractmethod

import torch

from ..layers import (LINEAR_TYPES, AllQuantLinearInferCell, WeightQuantLinearCell, linear_geometry)
from ..moe import GroupedMLP, QuantGroupedMLP
from ..paged_attention_mgr import PagedAttentionMgr, QuantPagedAttentionMgr


class Quantizer(ABC):
    """Abstract quantizer: ``preprocess_model`` swaps cells before the weights are loaded,
    ``postprocess_model`` finalises (packs) them afterwards."""

    requires_calibration = False
    required_packages = None

    def __init__(self, quantization_config, **kwargs):
        self.quantization_config = quantization_config
        self.modules_to_not_convert = list(kwargs.pop("modules_to_not_convert", []) or [])
        self.pre_quantized = kwargs.pop("pre_quantized", True)
        if not self.pre_quantized and self.requires_calibration:
            raise ValueError(f"The quantization method {quantization_config.quant_method} does require the model to be "
                             f"pre-quantized. You explicitly passed `pre_quantized=False` meaning your model weights "
                             f"are not quantized. Make sure to pass `pre_quantized=True` while knowing what you are doing.")

    def update_ms_dtype(self, ms_dtype):
        return ms_dtype

    def update_device_map(self, device_map):
        return device_map

    def adjust_target_dtype(self, ms_dtype):
        return ms_dtype

    def update_missing_keys(self, model, missing_keys, prefix):
        return missing_keys

    def get_special_dtypes_update(self, model, ms_dtype):
        return {name: ms_dtype for name, _ in model.named_parameters()
                if any(m in name for m in self.modules_to_not_convert)}

    def adjust_max_memory(self, max_memory):
        return max_memory

    def check_quantized_param(self, model, param_value, param_name, state_dict, **kwargs):
        return False

    def create_quantized_param(self, *args, **kwargs):
        raise AttributeError(f"`.create_quantized_param()` method is not supported by quantizer class "
                             f"{self.__class__.__name__}.")

    def validate_environment(self, *args, **kwargs):
        return

    def preprocess_model(self, model, **kwargs):
        model.is_quantized = True
        model.quantization_method = self.quantization_config.quant_method
        return self._process_model_before_weight_loading(model, **kwargs)

    def postprocess_model(self, model, **kwargs):
        return self._process_model_after_weight_loading(model, **kwargs)

    def dequantize(self, model):
        model = self._dequantize(model)
        del model.quantization_method
        return model

    def _dequantize(self, model):
        raise NotImplementedError(f"{self.__class__.__name__} has no attribute `dequantize`.")

    @abstractmethod
    def _process_model_before_weight_loading(self, model, **kwargs):
        ...

    @abstractmethod
    def _process_model_after_weight_loading(self, model, **kwargs):
        ...

    @property
    @abstractmethod
    def is_serializable(self):
        ...

    @property
    @abstractmethod
    def is_trainable(self):
        ...


def _skipped(name, blacklist):
    return any(b and b in name for b in blacklist)


def check_buildable(cfg):
    """Raise for configurations the reference's config classes accept but these kernels do not implement."""
    if cfg.weight_quant_dtype not in ("int8", "int4x2"):
        raise NotImplementedError(f"weight_dtype {cfg.weight_quant_dtype!r}: int8 and int4x2 weights are built")
    per_group = getattr(cfg, "weight_quant_granularity", "per_channel") == "per_group"
    if cfg.weight_quant_dtype == "int4x2" and cfg.act_quant_dtype is not None:
        raise NotImplementedError("4-bit weights are built weight-only (A16W4); W4A8 is not")
    if per_group and cfg.weight_quant_dtype != "int4x2":
        raise NotImplementedError("per_group weight scales are built for int4x2 weights only")
    if per_group and getattr(cfg, "group_size", 0) not in (64, 128):
        raise NotImplementedError("per_group weights need group_size 64 or 128")
    if cfg.kvcache_quant_dtype not in (None, "int8"):
        raise NotImplementedError(f"kvcache_dtype {cfg.kvcache_quant_dtype!r}: only an int8 KV cache is built")
    if cfg.kvcache_quant_dtype == "int8" and getattr(cfg, "kvcache_quant_granularity", "per_channel") not in (
            "per_channel", "per_token"):
        raise NotImplementedError("an int8 KV cache is quantised per_channel or per_token")
    if getattr(cfg, "precision_recovery", "none") != "none":
        raise NotImplementedError("GPTQ precision recovery has no deploy-time kernel here")
    if cfg.outliers_suppression not in ("none", "smooth", "awq"):
        raise NotImplementedError(f"outliers_suppression {cfg.outliers_suppression!r} is not built")
    if cfg.outliers_suppression == "awq" and cfg.act_quant_dtype is not None:
        raise NotImplementedError("awq is built in front of weight-only cells (A16W4 / A16W8)")
    if cfg.act_quant_dtype == "int8" and cfg.act_quant_granularity not in ("per_token", "per_tensor"):
        raise NotImplementedError(f"act_quant_granularity {cfg.act_quant_granularity!r} is not built")


def convert_linears(model, cfg, layer_policies=None):
    """Replace every float linear cell (and float GroupedMLP) not black-listed by its deploy cell.  The float
    weights, if already materialised, are quantised round-to-nearest; otherwise the int8 / scale buffers wait for
    the checkpoint.  Returns the model."""
    check_buildable(cfg)
    policies = layer_policies or {}
    for key, pol in policies.items():
        check_buildable(pol)

    def policy_for(name):
        for pattern, pol in policies.items():
            if re.search(pattern, name):
                return pol
        return cfg

    for parent_name, parent in list(model.named_modules()):
        for child_name, child in list(parent.named_children()):
            full = f"{parent_name}.{child_name}" if parent_name else child_name
            if _skipped(full, cfg.opname_blacklist):
                continue
            pol = policy_for(full)
            if isinstance(child, LINEAR_TYPES):
                fin, fout, has_bias, dt = linear_geometry(child)
                dev = child.weight.device if child.weight is not None else "cuda"
                cdt = dt if dt in (torch.bfloat16, torch.float16) else torch.bfloat16
                if pol.act_quant_dtype == "int8":
                    cell = AllQuantLinearInferCell(fin, fout, has_bias, cdt, dev, layer=child,
                                                   smooth=pol.outliers_suppression == "smooth",
                                                   act_quant_granularity=pol.act_quant_granularity)
                else:
                    per_group = getattr(pol, "weight_quant_granularity", "per_channel") == "per_group"
                    cell = WeightQuantLinearCell(fin, fout, has_bias, cdt, dev, layer=child,
                                                 weight_bits=4 if pol.weight_quant_dtype == "int4x2" else 8,
                                                 group_size=pol.group_size if per_group else 0,
                                                 smooth=pol.outliers_suppression in ("smooth", "awq"))
                if child.weight is not None:
                    w = child.weight.data if getattr(child, "transpose_b", True) else child.weight.data.t()
                    cell.quantize_from_float(w, child.bias.data if has_bias else None)
                setattr(parent, child_name, cell)
            elif (isinstance(child, PagedAttentionMgr) and not isinstance(child, QuantPagedAttentionMgr)
                  and pol.kvcache_quant_dtype == "int8"):
                # kvcache_dtype: int8 - the manager owns int8 caches and hands the attention its dequantisation
                # parameters (filled from the checkpoint)
                setattr(parent, child_name, QuantPagedAttentionMgr.from_float(
                    child, getattr(pol, "kvcache_quant_granularity", "per_channel")))
            elif isinstance(child, GroupedMLP):
                act8 = pol.act_quant_dtype == "int8"
                cell = QuantGroupedMLP(child.num_experts, child.config, child.weight1.device,
                                       act_quant=pol.act_quant_granularity if act8 else None,
                                       smooth=act8 and pol.outliers_suppression == "smooth")
                cell.quantize_from_float(child.weight1.data, child.weight2.data)
                setattr(parent, child_name, cell)
    return model


def finalize(model):
    """Pack every converted cell for the kernels (after the checkpoint has filled int8 weights / scales)."""
    for m in model.modules():
        if isinstance(m, (WeightQuantLinearCell, AllQuantLinearInferCell, QuantGroupedMLP)):
            m.prepare()
    return model
