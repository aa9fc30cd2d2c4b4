"""SmoothQuantQuantizer - mindformers/modules/quantizers/smooth_quant_quantizer.py:28-78.  The reference's
SmoothQuant method is A8W8 with static per-tensor activations and the smooth multiplier
(quantization_config.py:577-582): conversion puts AllQuantLinearInferCell(act_quant_granularity="per_tensor") in
place of every float linear; the calibrated ``act_scale`` / ``smooth_scale`` come with the checkpoint."""
import torch

from .base import Quantizer, convert_linears, finalize


class SmoothQuantQuantizer(Quantizer):
    requires_calibration = False
    required_packages = None

    def __init__(self, quantization_config, **kwargs):
        super().__init__(quantization_config, **kwargs)
        self.quant_config = quantization_config

    def update_ms_dtype(self, ms_dtype):
        return torch.float16 if ms_dtype is None else ms_dtype

    def _dequantize(self, model):
        pass

    def _process_model_before_weight_loading(self, model, **kwargs):
        return convert_linears(model, self.quant_config)

    def _process_model_after_weight_loading(self, model, **kwargs):
        return finalize(model)

    @property
    def is_serializable(self):
        return False

    @property
    def is_trainable(self):
        return False
