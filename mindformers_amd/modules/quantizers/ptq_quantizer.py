"""PtqQuantizer — mindformers/modules/quantizers/ptq_quantizer.py:25-70 (weights int8, activations None or int8
per token, optional smooth outlier suppression, per-layer policies by regular expression)."""
from .base import Quantizer, convert_linears, finalize


class PtqQuantizer(Quantizer):
    requires_calibration = False
    required_packages = None

    def __init__(self, quantization_config, **kwargs):
        super().__init__(quantization_config, **kwargs)
        self.quant_config = quantization_config
        self.layer_policies = self.quant_config.layer_policies

    def _dequantize(self, model):
        pass

    def _process_model_before_weight_loading(self, model, **kwargs):
        return convert_linears(model, self.quant_config, self.layer_policies)

    def _process_model_after_weight_loading(self, model, **kwargs):
        return finalize(model)

    @property
    def is_serializable(self):
        return False

    @property
    def is_trainable(self):
        return False
