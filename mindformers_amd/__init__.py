"""MI355X-native kernels and drop-in modules for MindFormers' quantized incremental-inference decode step."""
__version__ = "0.1.0"
