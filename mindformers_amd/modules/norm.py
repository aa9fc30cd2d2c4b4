"""RMSNorm cells: legacy LlamaRMSNorm (mindformers/models/llama/llama_layer.py:172-232) and the Megatron-style
RMSNorm (mindformers/parallel_core/inference/transformer/norm.py:73-115), on the fused HIP kernel."""
import torch
from torch import nn

from .. import ops

_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


class LlamaRMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) * weight, computed in fp32 inside the kernel and rounded once to x's dtype
    (the fused branch of the reference, llama_layer.py:225-228).  ``residual`` fuses the preceding add."""

    def __init__(self, dim, eps=1e-6, compute_type=torch.float32, fused_kernel=True, device="cuda"):
        super().__init__()
        if compute_type not in _DTYPES:
            raise TypeError(f"compute_type should be float32, float16 or bfloat16, got {compute_type}")
        self.eps = eps
        self.compute_type = compute_type
        self.self_define = False
        self.weight = nn.Parameter(torch.ones(dim, dtype=compute_type, device=device), requires_grad=False)

    def forward(self, x, residual=None):
        return ops.rms_norm(x, self.weight, self.eps, residual=residual)     # a column slice is read where it lies

    construct = forward

    def shard(self, *a, **k):
        return self


class RMSNorm(nn.Module):
    """norm.py:73-115: compute type taken from config.layernorm_compute_dtype."""

    def __init__(self, config=None, hidden_size=None, eps=1e-5, device="cuda"):
        super().__init__()
        ct = getattr(config, "layernorm_compute_dtype", torch.float32) if config is not None else torch.float32
        if ct not in _DTYPES:
            raise TypeError("The type of parameter 'layernorm_compute_dtype' should in [float32, float16, bfloat16], "
                            "but got the type : {}.".format(type(ct)))
        self.compute_type = ct
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=ct, device=device), requires_grad=False)

    def forward(self, x, residual=None):
        return ops.rms_norm(x, self.weight, self.eps, residual=residual)     # a column slice is read where it lies

    construct = forward
