"""AutoQuantizationConfig / AutoQuantizer — mindformers/modules/quantizers/auto.py:30-114."""
from ...quantization_config import PtqConfig, QuantizationConfigMixin, RtnConfig, SmoothQuantConfig
from .ptq_quantizer import PtqQuantizer
from .rtn_quantizer import RtnQuantizer
from .smooth_quant_quantizer import SmoothQuantQuantizer

AUTO_QUANTIZER_MAPPING = {"ptq": PtqQuantizer, "rtn": RtnQuantizer, "smooth_quant": SmoothQuantQuantizer}
AUTO_QUANTIZATION_CONFIG_MAPPING = {"ptq": PtqConfig, "rtn": RtnConfig, "smooth_quant": SmoothQuantConfig}

__all__ = ["AutoQuantizationConfig", "AutoQuantizer"]


class AutoQuantizationConfig:
    @classmethod
    def from_dict(cls, quantization_config_dict):
        quant_method = quantization_config_dict.get("quant_method", None)
        if quant_method is None:
            raise ValueError("The model's quantization config from the arguments has no `quant_method` attribute. "
                             "Make sure that the model has been correctly quantized")
        if quant_method not in AUTO_QUANTIZATION_CONFIG_MAPPING:
            raise ValueError(f"Unknown quantization type, got {quant_method} - supported types are:"
                             f" {list(AUTO_QUANTIZER_MAPPING.keys())}")
        return AUTO_QUANTIZATION_CONFIG_MAPPING[quant_method].from_dict(quantization_config_dict)

    @classmethod
    def from_pretrained(cls, pretrained_model_name_or_path, **kwargs):
        raise NotImplementedError("resolving a model name needs the model zoo / hub, which is outside this build; "
                                  "pass the quantization_config dict to from_dict instead")


class AutoQuantizer:
    @classmethod
    def from_config(cls, quantization_config, **kwargs):
        if isinstance(quantization_config, dict):
            quantization_config = AutoQuantizationConfig.from_dict(quantization_config)
        quant_method = quantization_config.quant_method
        if quant_method not in AUTO_QUANTIZER_MAPPING:
            raise ValueError(f"Unknown quantization type, got {quant_method} - supported types are:"
                             f" {list(AUTO_QUANTIZER_MAPPING.keys())}")
        return AUTO_QUANTIZER_MAPPING[quant_method](quantization_config, **kwargs)

    @classmethod
    def from_pretrained(cls, pretrained_model_name_or_path, **kwargs):
        return cls.from_config(AutoQuantizationConfig.from_pretrained(pretrained_model_name_or_path, **kwargs))
