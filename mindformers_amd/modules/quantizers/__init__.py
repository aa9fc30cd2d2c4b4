from .auto import AutoQuantizationConfig, AutoQuantizer
from .base import Quantizer
from .ptq_quantizer import PtqQuantizer
from .rtn_quantizer import RtnQuantizer
from .smooth_quant_quantizer import SmoothQuantQuantizer

__all__ = ["AutoQuantizationConfig", "AutoQuantizer", "Quantizer", "PtqQuantizer", "RtnQuantizer",
           "SmoothQuantQuantizer"]
