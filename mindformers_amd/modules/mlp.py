"""Feed-forward blocks: legacy LlamaFeedForward (mindformers/models/llama/llama_layer.py:257-441) and the
Megatron-style MLP (mindformers/parallel_core/inference/transformer/mlp.py:49-147).  The projections are whatever
linear cells are plugged in (float or quantized); SiLU*mul runs in the HIP kernel."""
import torch
from torch import nn

from .. import ops
from .layers import ColumnParallelLinear, Linear, RowParallelLinear


class MLP(nn.Module):
    """linear_fc1 -> [gate | hidden] split -> hidden * silu(gate) -> linear_fc2 (mlp.py:130-147)."""

    def __init__(self, config, input_size=None, device="cuda"):
        super().__init__()
        self.config = config
        self.input_size = input_size if input_size is not None else config.hidden_size
        self.ffn_hidden_size = config.ffn_hidden_size
        self.gated = config.gated_linear_unit
        if config.hidden_act not in ("silu", "swiglu", None):
            raise NotImplementedError(f"activation {config.hidden_act!r} is not built (silu only)")
        self.activation_type = config.hidden_act
        self.ffn_hidden_size_per_partition = self.ffn_hidden_size
        fc1_out = self.ffn_hidden_size * 2 if self.gated else self.ffn_hidden_size
        self.linear_fc1 = ColumnParallelLinear(self.input_size, fc1_out, config=config, bias=config.add_bias_linear,
                                               compute_dtype=config.compute_dtype, device=device)
        self.linear_fc2 = RowParallelLinear(self.ffn_hidden_size, config.hidden_size, config=config,
                                            bias=config.add_bias_linear, compute_dtype=config.compute_dtype, device=device)

    def forward(self, hidden_states, residual=None):
        inter = self.linear_fc1(hidden_states)
        if self.gated:
            inter = ops.silu_mul(inter.contiguous())
        elif self.activation_type:
            inter = torch.nn.functional.silu(inter)
        if residual is not None and hasattr(self.linear_fc2, "has_act_quant"):
            return self.linear_fc2(inter, residual=residual)
        out = self.linear_fc2(inter)
        return out if residual is None else ops.add(out, residual)

    construct = forward


class LlamaFeedForward(nn.Module):
    """w2(silu(w1 x) * w3 x) (llama_layer.py:412-441).  ``ffn_concat`` fuses w1/w3 into ``w_gate_hidden`` whose
    output columns alternate gate, hidden (the (ffn, 2) reshape at :419-423)."""

    def __init__(self, dim, intermediate_size=None, hidden_dim=None, multiple_of=256, hidden_act="silu",
                 ffn_dim_multiplier=None, compute_dtype=torch.float16, param_init_type=torch.float32, ffn_concat=False,
                 device="cuda"):
        super().__init__()
        if hidden_act not in ("silu",):
            raise NotImplementedError(f"activation {hidden_act!r} is not built (silu only)")
        if intermediate_size is not None:
            hidden_dim = intermediate_size
        else:
            if hidden_dim is None:
                hidden_dim = 4 * dim
            if ffn_dim_multiplier is not None:
                hidden_dim = int((ffn_dim_multiplier + 0.01) * hidden_dim)
            hidden_dim = int(2 * hidden_dim / 3)
            hidden_dim = multiple_of * ((hidden_dim + multiple_of - 1) // multiple_of)
        self.dtype = compute_dtype
        self.hidden_dim = hidden_dim
        self.dim = dim
        self.ffn_concat = ffn_concat
        kw = dict(has_bias=False, compute_dtype=compute_dtype, param_init_type=param_init_type, device=device)
        if ffn_concat:
            self.w_gate_hidden = Linear(dim, hidden_dim * 2, **kw)
        else:
            self.w1 = Linear(dim, hidden_dim, **kw)
            self.w3 = Linear(dim, hidden_dim, **kw)
        self.w2 = Linear(hidden_dim, dim, **kw)

    def forward(self, x):
        x = x.to(self.dtype)
        if self.ffn_concat:
            hidden = ops.silu_mul(self.w_gate_hidden(x).contiguous(), interleaved=True)
        else:
            gate = self.w1(x)
            up = self.w3(x)
            hidden = ops.silu_mul(torch.cat((gate, up), dim=-1))
        return self.w2(hidden)

    construct = forward
