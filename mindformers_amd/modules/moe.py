"""Inference mixture-of-experts layer: TopKRouter, GroupedMLP, SharedExpertMLP, MoELayer.

Follows mindformers/parallel_core/inference/transformer/moe/{router.py:88-159, experts.py:35-170,
shared_experts.py:32-75, moe_layer.py:78-163}.  Router scoring, permute, the quantized grouped expert GEMMs and
the weighted unpermute and the router's gate projection are HIP kernels.
"""
import torch
from torch import nn

from .. import ops
from .mlp import MLP
from copy import copy


class TopKRouter(nn.Module):
    """Route each token to its top-k experts (router.py:88-159).  Returns (expert_weight [T,k] in the input
    dtype, expert_index [T,k] int32)."""

    def __init__(self, config, device="cuda"):
        super().__init__()
        if config.moe_router_score_function != "sigmoid":
            raise NotImplementedError("only the sigmoid score function is built")
        self.config = config
        self.hidden = config.hidden_size
        self.num_experts = config.num_moe_experts
        self.router_dense_type = config.moe_router_dtype
        self.n_group = config.moe_router_num_groups
        self.topk_group = config.moe_router_group_topk
        self.group_topk_inner = 2
        self.num_experts_chosen = config.moe_router_topk
        self.moe_router_enable_expert_bias = config.moe_router_enable_expert_bias
        w = torch.empty(self.num_experts, self.hidden, dtype=self.router_dense_type, device=device)
        nn.init.normal_(w, std=0.01)
        self.weight = nn.Parameter(w, requires_grad=False)          # the reference's self.weight.weight (nn.Dense)
        self.expert_bias = nn.Parameter(torch.zeros(self.num_experts, dtype=torch.float32, device=device), requires_grad=False)

    def gating(self, input_tensor):
        """logits = cast(x, router_dense_type) . weight^T (router.py:54-63), returned in fp32 (the cast of
        router.py:128); a 16-bit router's projection output is rounded to its type first."""
        x = input_tensor.reshape(-1, self.hidden)
        if self.weight.dtype != torch.float32 and x.dtype != self.weight.dtype:
            x = x.to(self.weight.dtype)
        if x.dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"router input of type {x.dtype}: the gate projection is built for bf16 / fp16 activations")
        return ops.router_gate(x.contiguous(), self.weight)

    def routing(self, logits):
        input_dtype = logits.dtype
        gating_logits = self.gating(logits).float().contiguous()
        out_dtype = input_dtype if input_dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
        if self.config.moe_router_group_topk:
            w, idx = ops.moe_route(gating_logits, self.expert_bias, self.num_experts_chosen, self.n_group or 1,
                                   self.topk_group, self.config.moe_router_topk_scaling_factor, out_dtype)
        else:                                                       # plain biased top-k, router.py:142-146
            w, idx = ops.moe_route(gating_logits, self.expert_bias, self.config.moe_router_topk, 1, 1, 1.0, out_dtype,
                                   renorm=True, biased_weights=True)
        return w.to(input_dtype), idx

    def forward(self, input_tensor):
        return self.routing(input_tensor)

    construct = forward


class GroupedMLP(nn.Module):
    """Experts layer with float weights weight1 [E, H, 2F], weight2 [E, F, H] (experts.py:35-170).  Rows of
    ``hidden_states`` are grouped per expert by ``group_list`` (per-expert counts).  The float path loops the
    experts over library GEMMs; the decode path replaces this cell by ``QuantGroupedMLP``."""

    def __init__(self, num_experts, config, device="cuda"):
        super().__init__()
        if config.add_bias_linear:
            raise NotImplementedError("expert bias is not built")
        if not config.gated_linear_unit:
            raise NotImplementedError("ungated experts are not built")
        self.config = config
        self.num_experts = num_experts
        self.compute_dtype = config.compute_dtype
        self.hidden_size = config.hidden_size
        self.ffn_hidden_size_per_partition = config.moe_ffn_hidden_size
        f = config.moe_ffn_hidden_size
        self.weight1 = nn.Parameter(torch.empty(num_experts, config.hidden_size, 2 * f, dtype=config.params_dtype, device=device).normal_(std=0.01), requires_grad=False)
        self.weight2 = nn.Parameter(torch.empty(num_experts, f, config.hidden_size, dtype=config.params_dtype, device=device).normal_(std=0.01), requires_grad=False)

    def forward(self, hidden_states, group_list=None):
        counts = group_list.tolist()                               # host sync: this is not the decode hot path
        x = hidden_states.to(self.compute_dtype)
        out = torch.empty(x.shape[0], self.hidden_size, dtype=self.compute_dtype, device=x.device)
        start = 0
        for e, c in enumerate(counts):
            if c:
                h = x[start:start + c] @ self.weight1[e].to(self.compute_dtype)
                a = ops.silu_mul(h.contiguous())
                out[start:start + c] = a @ self.weight2[e].to(self.compute_dtype)
            start += c
        return out.to(hidden_states.dtype)

    construct = forward


class QuantGroupedMLP(nn.Module):
    """Quantized experts: int8 weights stored K-contiguous ([E, 2F, H] and [E, H, F], i.e. the reference's
    [E, in, out] parameters transposed at load) with per-output-channel scales.  ``offsets`` (int32 [E+1], from
    moe_permute) addresses the row groups.

    ``act_quant=None`` (W8A16): two grouped HIP GEMMs, the first with silu(gate) * hidden in its epilogue.
    ``act_quant="per_token"`` / ``"per_tensor"`` (W8A8, the routed experts of a W8A8 checkpoint such as
    research/deepseek3/deepseek_r1_671b/predict_deepseek_r1_671b_w8a8.yaml:89-92): the permuted rows are quantised per
    token, or with one calibrated scale per projection (``act_scale1`` / ``act_scale2``, loaded with the checkpoint),
    and both projections run on the int8 matrix cores with exact int32 accumulators.  ``smooth`` (per_token only):
    the rows of expert e are multiplied by ``smooth_scale1[e]`` [H] in front of the first projection and the
    activation product by ``smooth_scale2[e]`` [F] in front of the second (outliers_suppression: smooth; the weight
    side of the pair is folded into the checkpoint's int8 weights)."""

    def __init__(self, num_experts, config, device="cuda", act_quant=None, smooth=False):
        super().__init__()
        if act_quant not in (None, "per_token", "per_tensor"):
            raise ValueError(f"act_quant must be None, 'per_token' or 'per_tensor', got {act_quant!r}")
        if smooth and act_quant != "per_token":
            raise NotImplementedError("smooth multipliers on routed experts are built for per_token activations")
        self.config = config
        self.num_experts = num_experts
        self.act_quant = act_quant
        self.compute_dtype = getattr(config, "compute_dtype", torch.bfloat16)
        f, h = config.moe_ffn_hidden_size, config.hidden_size
        self.register_buffer("weight1", torch.zeros(num_experts, 2 * f, h, dtype=torch.int8, device=device))
        self.register_buffer("w1_scale", torch.ones(num_experts, 2 * f, dtype=torch.float32, device=device))
        self.register_buffer("weight2", torch.zeros(num_experts, h, f, dtype=torch.int8, device=device))
        self.register_buffer("w2_scale", torch.ones(num_experts, h, dtype=torch.float32, device=device))
        static = act_quant == "per_tensor"
        self.register_buffer("act_scale1", torch.ones(1, dtype=torch.float32, device=device) if static else None)
        self.register_buffer("act_scale2", torch.ones(1, dtype=torch.float32, device=device) if static else None)
        self.register_buffer("smooth_scale1", torch.ones(num_experts, h, dtype=torch.float32, device=device) if smooth else None)
        self.register_buffer("smooth_scale2", torch.ones(num_experts, f, dtype=torch.float32, device=device) if smooth else None)
        self._p1 = self._p2 = None

    @torch.no_grad()
    def quantize_from_float(self, weight1, weight2):
        """weight1 [E, H, 2F], weight2 [E, F, H] float (reference layout) -> int8 per output channel."""
        for src, dst, sc in ((weight1, self.weight1, self.w1_scale), (weight2, self.weight2, self.w2_scale)):
            # expert by expert in float64: the scale is max|w| / 127 rounded to float32 and the quotient is taken in
            # float64, as the dense cells do, so that the int8 grid point does not depend on a float32 division
            for e in range(src.shape[0]):
                w = src[e].detach().to(device=dst.device, dtype=torch.float64).t()                       # [out, in]
                scale = (w.abs().amax(dim=1) / 127.0).float()
                safe = torch.where(scale > 0, scale, torch.ones_like(scale)).double()
                dst[e].copy_(torch.clamp(torch.round(w / safe[:, None]), -127, 127).to(torch.int8))
                sc[e].copy_(scale)
        self._p1 = self._p2 = None
        return self

    def prepare(self):
        # W8A16: gate / up rows interleaved, so that the first GEMM's epilogue holds each pair in one lane
        self._p1 = (ops.pack_w8a16(self.weight1, self.w1_scale) if self.act_quant
                    else ops.pack_w8a16_gated(self.weight1, self.w1_scale, "halves"))
        self._p2 = ops.pack_w8a16(self.weight2, self.w2_scale)
        return self

    def _quant(self, x, act_scale):
        if self.act_quant == "per_tensor":
            return ops.static_quant(x, act_scale)
        return ops.dynamic_quant(x)

    def forward(self, hidden_states, group_list=None, offsets=None):
        if self._p1 is None:
            self.prepare()
        if offsets is None:
            offsets = torch.zeros(self.num_experts + 1, dtype=torch.int32, device=hidden_states.device)
            offsets[1:] = torch.cumsum(group_list, 0).to(torch.int32)
        if not self.act_quant:
            a = ops.grouped_w8a16_linear(hidden_states, self._p1, offsets)       # silu(gate) * hidden included
            return ops.grouped_w8a16_linear(a, self._p2, offsets)
        dt = hidden_states.dtype
        if self.smooth_scale1 is not None:
            xq, xs = ops.dynamic_quant(hidden_states.contiguous(), self.smooth_scale1, offsets=offsets)
        else:
            xq, xs = self._quant(hidden_states.contiguous(), self.act_scale1)
        h = ops.grouped_w8a8_linear(xq, xs, self._p1, offsets, out_dtype=dt)
        if self.act_quant == "per_tensor":
            aq, a_s = ops.static_quant(ops.silu_mul(h), self.act_scale2)
        elif self.smooth_scale2 is not None:
            aq, a_s = ops.silu_mul_dynamic_quant(h, self.smooth_scale2, offsets=offsets)
        else:
            aq, a_s = ops.silu_mul_dynamic_quant(h)
        return ops.grouped_w8a8_linear(aq, a_s, self._p2, offsets, out_dtype=dt)

    construct = forward


class SharedExpertMLP(MLP):
    """shared_experts.py:32-75: a gated MLP of width moe_shared_expert_intermediate_size (no output gate)."""

    def __init__(self, config, gate=False, device="cuda"):
        if config.add_bias_linear:
            raise ValueError("bias is not supported in the shared experts")
        if config.shared_expert_num == 0:
            raise ValueError("For SharedExpertMLP`, shared_expert_num` must be greater than 0.")
        if gate:
            raise NotImplementedError("the shared-expert output gate is not built (the reference passes gate=False)")
        cfg = copy(config)
        cfg.ffn_hidden_size = config.moe_shared_expert_intermediate_size
        super().__init__(cfg, device=device)
        self.use_shared_expert_gate = False


class MoELayer(nn.Module):
    """router -> permute -> experts -> weighted unpermute (+ shared experts) (moe_layer.py:126-163)."""

    def __init__(self, config, submodules=None, layer_number=None, device="cuda"):
        super().__init__()
        if config.expert_model_parallel_size > 1:
            raise NotImplementedError("For MoELayer, `expert_model_parallel_size` is not supported for now.")
        self.config = config
        self.layer_number = layer_number
        self.num_experts = config.num_moe_experts
        self.use_shared_expert = config.moe_shared_expert_intermediate_size is not None
        self.router = TopKRouter(config, device=device)
        self.experts = GroupedMLP(self.num_experts, config, device=device)
        self.shared_experts = SharedExpertMLP(config, device=device) if self.use_shared_expert else None

    def forward(self, hidden_states):
        shape = hidden_states.shape
        x = hidden_states.reshape(-1, self.config.hidden_size).contiguous()
        expert_weight, routing_map = self.router(x)
        px, row_map, counts, offsets = ops.moe_permute(x, routing_map, self.num_experts)
        if isinstance(self.experts, QuantGroupedMLP):
            y = self.experts(px, counts, offsets=offsets)
        else:
            y = self.experts(px, counts)
        shared = self.shared_experts(x).contiguous() if self.use_shared_expert else None
        out = ops.moe_unpermute(y.contiguous(), row_map, expert_weight.contiguous(), shared=shared)
        return out.reshape(shape)

    construct = forward
