"""The subset of the reference's TransformerConfig (mindformers/parallel_core/transformer_config.py; MoE fields
:225-301) that the decode-path modules read.  Field names and defaults follow the reference."""
from dataclasses import dataclass
from typing import Optional

import torch

_DT = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float16": torch.float16, "fp16": torch.float16,
       "float32": torch.float32, "fp32": torch.float32}


def convert_dtype(value):
    if isinstance(value, torch.dtype):
        return value
    if isinstance(value, str) and value.lower() in _DT:
        return _DT[value.lower()]
    raise ValueError(f"unknown dtype {value!r}")


@dataclass
class TransformerConfig:
    num_layers: int = 1
    hidden_size: int = 0
    num_attention_heads: int = 1
    num_query_groups: Optional[int] = None
    kv_channels: Optional[int] = None
    ffn_hidden_size: Optional[int] = None
    hidden_act: Optional[str] = "silu"
    gated_linear_unit: bool = True
    add_bias_linear: bool = False
    add_qkv_bias: bool = False
    layernorm_epsilon: float = 1e-5
    compute_dtype: object = "bfloat16"
    params_dtype: object = "bfloat16"
    layernorm_compute_dtype: object = "float32"
    softmax_compute_dtype: object = "float32"
    use_flash_attention: bool = True
    tensor_model_parallel_size: int = 1
    expert_model_parallel_size: int = 1
    # mixture of experts
    num_moe_experts: Optional[int] = None
    moe_router_topk: int = 2
    moe_router_num_groups: Optional[int] = None
    moe_router_group_topk: Optional[int] = None
    moe_router_topk_scaling_factor: Optional[float] = None
    moe_router_score_function: str = "sigmoid"
    moe_router_enable_expert_bias: bool = False
    moe_router_dtype: object = "float32"
    moe_ffn_hidden_size: Optional[int] = None
    moe_shared_expert_intermediate_size: Optional[int] = None
    shared_expert_num: int = 0

    def __post_init__(self):
        for f in ("compute_dtype", "params_dtype", "layernorm_compute_dtype", "softmax_compute_dtype", "moe_router_dtype"):
            setattr(self, f, convert_dtype(getattr(self, f)))
        if self.tensor_model_parallel_size != 1 or self.expert_model_parallel_size != 1:
            raise NotImplementedError("this build runs on one GPU: tensor / expert parallel sizes must be 1")
        if self.num_query_groups is None:
            self.num_query_groups = self.num_attention_heads
        if self.kv_channels is None and self.hidden_size and self.num_attention_heads:
            self.kv_channels = self.hidden_size // self.num_attention_heads
        if self.ffn_hidden_size is None and self.hidden_size:
            self.ffn_hidden_size = 4 * self.hidden_size
        if self.num_moe_experts is not None and self.moe_ffn_hidden_size is None:
            self.moe_ffn_hidden_size = self.ffn_hidden_size
        # a zero shared-expert width means "no shared expert" (transformer_config.py:513-514 scales a positive one)
        if not self.moe_shared_expert_intermediate_size:
            self.moe_shared_expert_intermediate_size = None
        if self.moe_router_topk_scaling_factor is None:
            self.moe_router_topk_scaling_factor = 1.0
