"""AutoQuantizationConfig / AutoQuantizer: pick the config class and the quantizer class from the ``quant_method``
string of a quantization config (the dispatch surface of mindformers/modules/quantizers/auto.py:30-114)."""
from ...quantization_config import PtqConfig, QuantizationConfigMixin, RtnConfig, SmoothQuantConfig
from .ptq_quantizer import PtqQuantizer
from .rtn_quantizer import RtnQuantizer
from .smooth_quant_quantizer import SmoothQuantQuantizer

# one registry: method name -> (config class, quantizer class); the two public mappings are its columns
_METHODS = {"ptq": (PtqConfig, PtqQuantizer), "rtn": (RtnConfig, RtnQuantizer),
            "smooth_quant": (SmoothQuantConfig, SmoothQuantQuantizer)}
AUTO_QUANTIZATION_CONFIG_MAPPING = {name: pair[0] for name, pair in _METHODS.items()}
AUTO_QUANTIZER_MAPPING = {name: pair[1] for name, pair in _METHODS.items()}

__all__ = ["AutoQuantizationConfig", "AutoQuantizer"]


def _method_entry(quant_method):
    if quant_method is None:
        raise ValueError("quantization config carries no `quant_method`; it must name one of "
                         f"{sorted(_METHODS)} (is this checkpoint quantized at all?)")
    try:
        return _METHODS[quant_method]
    except (KeyError, TypeError):
        raise ValueError(f"quant_method {quant_method!r} is not one of the built methods {sorted(_METHODS)}") from None


class AutoQuantizationConfig:
    @classmethod
    def from_dict(cls, quantization_config_dict):
        config_cls, _ = _method_entry(quantization_config_dict.get("quant_method"))
        return config_cls.from_dict(quantization_config_dict)

    @classmethod
    def from_pretrained(cls, pretrained_model_name_or_path, **kwargs):
        raise NotImplementedError("resolving a model name needs the model zoo / hub, which is outside this build; "
                                  "pass the quantization_config dict to from_dict instead")


class AutoQuantizer:
    @classmethod
    def from_config(cls, quantization_config, **kwargs):
        if isinstance(quantization_config, dict):
            quantization_config = AutoQuantizationConfig.from_dict(quantization_config)
        _, quantizer_cls = _method_entry(quantization_config.quant_method)
        return quantizer_cls(quantization_config, **kwargs)

    @classmethod
    def from_pretrained(cls, pretrained_model_name_or_path, **kwargs):
        return cls.from_config(AutoQuantizationConfig.from_pretrained(pretrained_model_name_or_path, **kwargs))
