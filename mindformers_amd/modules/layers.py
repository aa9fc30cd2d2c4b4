"""Linear cells of the decode path and the quantized cells that replace them.

Surface follows the reference:
  legacy ``Linear``                  mindformers/modules/layers.py:366-533 (attributes read elsewhere:
                                     weight, bias, matmul, in_channels, out_channels, dtype, has_bias,
                                     activation_flag — mindformers/pet/tuners/slora_adapter.py:68-89)
  Megatron-style linears (tp = 1)    mindformers/parallel_core/inference/tensor_parallel/layers.py:44-555
  quantized deploy cells             golden-stick (mindspore_gs) cells swapped in by
                                     Quantizer.preprocess_model; the only in-repo witness of their attribute
                                     surface is slora_adapter.py:57-63,130-145 (.layer, .has_act_quant,
                                     .quant_op, .layer.matmul, .layer.weight)

The unquantized cells run a plain library GEMM (torch.nn.functional.linear -> hipBLASLt); the quantized cells
call the W8A16 / W8A8 HIP kernels.  Quantized parameter names (defined here, golden-stick's are not in the
reference): ``weight`` int8 [out, in], ``w_scale`` fp32 [out], ``smooth_scale`` fp32 [in] (W8A8 only), ``bias``.
"""
import torch
import torch.nn.functional as F
from torch import nn

from .. import ops

_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def _act(name):
    if name is None:
        return None
    if isinstance(name, str):
        table = {"silu": F.silu, "gelu": F.gelu, "relu": F.relu, "swiglu": None}
        if name.lower() not in table:
            raise ValueError(f"unsupported activation {name!r}")
        return table[name.lower()]
    if isinstance(name, type) and issubclass(name, nn.Module):
        return name()
    raise TypeError(f"For Linear cell, the activation should str type or nn.Cell type, but got {name}.")


class Linear(nn.Module):
    """y = cast(x) @ cast(W)^T (+ bias) (-> activation), reshaped to the input's leading shape
    (layers.py:510-533).  expert_num > 1 / use_gmm belong to the training MoE path and are not built."""

    def __init__(self, in_channels, out_channels, init_method_std=0.01, weight_init="normal", bias_init="zeros",
                 has_bias=True, activation=None, transpose_b=True, expert_num=1, outer_batch=1,
                 expert_group_size=None, use_gmm=False, param_init_type=torch.float32, compute_dtype=torch.float16,
                 device="cuda"):
        super().__init__()
        if expert_num != 1 or use_gmm:
            raise NotImplementedError("expert_num > 1 / use_gmm Linear is not built (use moe.GroupedMLP)")
        if param_init_type not in _DTYPES or compute_dtype not in _DTYPES:
            raise TypeError("param_init_type / compute_dtype must be float32, float16 or bfloat16")
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.transpose_b = transpose_b
        self.expert_num, self.outer_batch, self.expert_group_size, self.use_gmm = expert_num, outer_batch, expert_group_size, use_gmm
        shape = (out_channels, in_channels) if transpose_b else (in_channels, out_channels)
        w = torch.empty(shape, dtype=param_init_type, device=device)
        if isinstance(weight_init, torch.Tensor):
            if tuple(weight_init.shape) != shape:
                raise ValueError("The shape of parameter 'weight_init' is error, please check shape of 'weight_init'.")
            w.copy_(weight_init)
        elif weight_init == "normal":
            nn.init.normal_(w, mean=0.0, std=init_method_std)
        elif weight_init == "zeros":
            w.zero_()
        else:
            raise ValueError(f"unsupported weight_init {weight_init!r}")
        self.weight = nn.Parameter(w, requires_grad=False)
        self.has_bias = has_bias
        self.bias = nn.Parameter(torch.zeros(out_channels, dtype=param_init_type, device=device), requires_grad=False) \
            if has_bias else None
        self.activation = _act(activation)
        self.activation_flag = self.activation is not None
        self.dtype = compute_dtype
        self.matmul = F.linear

    def forward(self, x, group_list=None):
        out_shape = tuple(x.shape[:-1]) + (self.out_channels,)
        x2 = x.reshape(-1, self.in_channels)
        ori_dtype = x2.dtype
        w = self.weight.to(self.dtype)
        w = w if self.transpose_b else w.t()
        y = F.linear(x2.to(self.dtype), w, self.bias.to(self.dtype) if self.has_bias else None)
        if self.activation_flag:
            y = self.activation(y)
        return y.to(ori_dtype).reshape(out_shape)

    construct = forward

    def shard(self, *args, **kwargs):
        return self


class _QuantLinearBase(nn.Module):
    """Common part of the deploy cells: holds the wrapped float cell as ``layer`` until converted, then int8
    weight + scales.  ``prepare()`` packs the weight for the kernels (call after the checkpoint is loaded)."""

    has_act_quant = False

    def __init__(self, in_channels, out_channels, has_bias=False, compute_dtype=torch.bfloat16, device="cuda",
                 layer=None):
        super().__init__()
        if in_channels % 8:
            raise ValueError(f"in_channels ({in_channels}) must be a multiple of 8 for the int8 kernels")
        self.in_channels, self.out_channels = in_channels, out_channels
        self.has_bias = has_bias
        self.dtype = compute_dtype
        object.__setattr__(self, "_wrapped", layer)        # not a registered child: it may be this cell itself
        self.register_buffer("weight", torch.zeros(out_channels, in_channels, dtype=torch.int8, device=device))
        self.register_buffer("w_scale", torch.ones(out_channels, dtype=torch.float32, device=device))
        self.bias = nn.Parameter(torch.zeros(out_channels, dtype=compute_dtype, device=device), requires_grad=False) \
            if has_bias else None
        self.activation_flag = False
        self.quant_op = None
        self._packed = None

    @property
    def layer(self):
        """The cell whose weight / matmul adapters reach through (`.layer.weight`, `.layer.matmul`,
        slora_adapter.py:57-63): the converted cell holds its own parameters."""
        return self

    @property
    def matmul(self):
        return self._matmul

    @torch.no_grad()
    def quantize_from_float(self, weight, bias=None):
        """Round-to-nearest, symmetric per-output-channel int8 (what golden-stick's RoundToNearest produces
        offline).  weight float [out, in]."""
        w = weight.detach().to(device=self.weight.device, dtype=torch.float64)
        if tuple(w.shape) != (self.out_channels, self.in_channels):
            raise ValueError(f"weight shape {tuple(w.shape)} != {(self.out_channels, self.in_channels)}")
        # float64 quotient: the rounding to the int8 grid then does not depend on how a device divides in float32
        scale = (w.abs().amax(dim=1) / 127.0).float()
        safe = torch.where(scale > 0, scale, torch.ones_like(scale)).double()
        self.weight.copy_(torch.clamp(torch.round(w / safe[:, None]), -127, 127).to(torch.int8))
        self.w_scale.copy_(scale)
        if bias is not None and self.bias is not None:
            self.bias.copy_(bias.to(self.bias.dtype))
        self._packed = None
        return self

    def prepare(self):
        raise NotImplementedError


class WeightQuantLinearCell(_QuantLinearBase):
    """Weight-only deploy cell (lowers to WeightQuantBatchMatmul in the reference stack).  ``weight_bits`` 8: int8 per
    output channel (W8A16).  ``weight_bits`` 4 (weight_dtype qint4x2, quantization_config.py:408-416): ``weight`` is
    int8 [out, in / 2] with two 4-bit values per byte (element 2j in the low nibble), ``w_scale`` one value per output
    channel (``group_size`` 0) or [in / group_size, out] (per_group, 64 or 128).  ``smooth``: the activations are
    multiplied by ``smooth_scale`` [in] first (the activation side of awq / smooth outlier suppression, whose weight
    side is folded into the checkpoint's weights)."""

    def __init__(self, in_channels, out_channels, has_bias=False, compute_dtype=torch.bfloat16, device="cuda",
                 layer=None, weight_bits=8, group_size=0, smooth=False):
        super().__init__(in_channels, out_channels, has_bias, compute_dtype, device, layer)
        if weight_bits not in (8, 4) or group_size not in (0, 64, 128):
            raise ValueError(f"weight_bits must be 8 or 4 and group_size 0, 64 or 128, got {weight_bits} / {group_size}")
        if weight_bits == 8 and group_size:
            raise NotImplementedError("per_group scales are built for 4-bit weights only")
        self.weight_bits, self.group_size = weight_bits, group_size
        if weight_bits == 4:
            if in_channels % 64 or (group_size and in_channels % group_size):
                raise ValueError(f"in_channels ({in_channels}) must be a multiple of 64 and of the group size for 4-bit weights")
            self.weight = torch.zeros(out_channels, in_channels // 2, dtype=torch.int8, device=device)
            if group_size:
                self.w_scale = torch.ones(in_channels // group_size, out_channels, dtype=torch.float32, device=device)
        self.register_buffer("smooth_scale", torch.ones(in_channels, dtype=torch.float32, device=device) if smooth else None)

    @torch.no_grad()
    def quantize_from_float(self, weight, bias=None):
        if self.weight_bits == 8:
            return super().quantize_from_float(weight, bias)
        # symmetric 4-bit, per channel or per channel and group: s = max|w| / 7, q = clip(rint(w / s), -8, 7), the
        # quotient in float64
        w = weight.detach().to(device=self.weight.device, dtype=torch.float64)
        n, k = self.out_channels, self.in_channels
        if tuple(w.shape) != (n, k):
            raise ValueError(f"weight shape {tuple(w.shape)} != {(n, k)}")
        g = self.group_size or k
        wg = w.reshape(n, k // g, g)
        scale = (wg.abs().amax(dim=2) / 7.0).float()
        safe = torch.where(scale > 0, scale, torch.ones_like(scale)).double()
        q = torch.clamp(torch.round(wg / safe[:, :, None]), -8, 7).to(torch.int8).reshape(n, k)
        self.weight.copy_(((q[:, 0::2] & 15) | (q[:, 1::2] << 4)).to(torch.int8))
        self.w_scale.copy_(scale[:, 0] if self.group_size == 0 else scale.t().contiguous())
        if bias is not None and self.bias is not None:
            self.bias.copy_(bias.to(self.bias.dtype))
        self._packed = None
        return self

    def prepare(self):
        if self.weight_bits == 4:
            self._packed = ops.pack_w4a16(self.weight, self.w_scale, self.group_size, qint4x2=True)
        else:
            self._packed = ops.pack_w8a16(self.weight, self.w_scale)
        return self

    def _matmul(self, x, residual=None):
        if self._packed is None:
            self.prepare()
        if self.smooth_scale is not None:
            x = ops.scale_columns(x, self.smooth_scale)
        if self.weight_bits == 4:
            return ops.w4a16_linear(x, self._packed, bias=self.bias, residual=residual)
        return ops.w8a16_linear(x, self._packed, bias=self.bias, residual=residual)

    def forward(self, x, residual=None):
        out_shape = tuple(x.shape[:-1]) + (self.out_channels,)
        x2 = x.reshape(-1, self.in_channels)
        if x2.dtype != self.dtype:
            x2 = x2.to(self.dtype)
        if residual is not None:
            residual = residual.reshape(-1, self.out_channels)
        return self._matmul(x2.contiguous(), residual).reshape(out_shape)

    construct = forward

    def forward_with_leading_norm(self, x, gamma, eps):
        """The projection together with an RMSNorm over its leading ``gamma.numel()`` output columns (the fused
        query / latent down projection of multi-latent attention followed by q_layernorm): returns (y [T, out],
        norm(y[:, :c]) * gamma [T, c]), the bits of ``forward`` followed by the norm on the column slice."""
        x2 = x.reshape(-1, self.in_channels)
        if x2.dtype != self.dtype:
            x2 = x2.to(self.dtype)
        if self.weight_bits != 8 or gamma.numel() % 8 or self.out_channels % 8 or self.out_channels > 16384:
            y = self._matmul(x2.contiguous())
            return y, ops.rms_norm(y[:, :gamma.numel()], gamma, eps)
        if self._packed is None:
            self.prepare()
        x2 = x2.contiguous()
        if self.smooth_scale is not None:
            x2 = ops.scale_columns(x2, self.smooth_scale)
        return ops.w8a16_linear_rmsnorm_leading(x2, self._packed, gamma, eps, bias=self.bias)


class AllQuantLinearInferCell(_QuantLinearBase):
    """W8A8 deploy cell: per-token dynamic activation quantisation (with the SmoothQuant multiplier), or static
    per-tensor quantisation with a calibrated scale (``act_quant_granularity="per_tensor"``, the SmoothQuant
    method), followed by the int8 MFMA GEMM (DynamicQuant / QuantV2 + QuantBatchMatmul in the reference stack)."""

    has_act_quant = True

    def __init__(self, in_channels, out_channels, has_bias=False, compute_dtype=torch.bfloat16, device="cuda",
                 layer=None, smooth=True, act_quant_granularity="per_token"):
        super().__init__(in_channels, out_channels, has_bias, compute_dtype, device, layer)
        if act_quant_granularity not in ("per_token", "per_tensor"):
            raise ValueError(f"act_quant_granularity must be per_token or per_tensor, got {act_quant_granularity!r}")
        self.act_quant_granularity = act_quant_granularity
        self.register_buffer("smooth_scale", torch.ones(in_channels, dtype=torch.float32, device=device) if smooth else None)
        # per_tensor: one calibrated activation scale, loaded with the checkpoint (the SmoothQuant method's cells)
        self.register_buffer("act_scale", torch.ones(1, dtype=torch.float32, device=device)
                             if act_quant_granularity == "per_tensor" else None)
        self.quant_op = self._quant

    def _quant(self, x):
        if self.act_quant_granularity == "per_tensor":
            return ops.static_quant(x, self.act_scale, self.smooth_scale, tiled=True)
        return ops.dynamic_quant(x, self.smooth_scale, tiled=True)

    def prepare(self):
        self._packed = ops.pack_w8a16(self.weight, self.w_scale)
        return self

    def _matmul(self, xq, x_scale, residual=None):
        if self._packed is None:
            raise RuntimeError("call prepare() (or Quantizer.postprocess_model) after loading the weights")
        return ops.w8a8_linear(xq, x_scale, self._packed, out_dtype=self.dtype, bias=self.bias, residual=residual)

    def forward(self, x, residual=None):
        out_shape = tuple(x.shape[:-1]) + (self.out_channels,)
        x2 = x.reshape(-1, self.in_channels)
        if x2.dtype != self.dtype:
            x2 = x2.to(self.dtype)
        xq, xs = self.quant_op(x2.contiguous())
        if residual is not None:
            residual = residual.reshape(-1, self.out_channels)
        return self._matmul(xq, xs, residual).reshape(out_shape)

    construct = forward


# ------------------------------------------------------------------ Megatron-style linears, tensor parallel size 1
class _ParallelLinearBase(nn.Module):
    def __init__(self, input_size, output_size, *, config=None, init_method="normal", bias=True, transpose_b=True,
                 compute_dtype=torch.bfloat16, skip_weight_param_allocation=False, device="cuda"):
        super().__init__()
        self.input_size, self.output_size = input_size, output_size
        self.config = config
        self.has_bias = bias
        self.transpose_b = transpose_b
        self.compute_dtype = compute_dtype
        self.params_dtype = getattr(config, "params_dtype", compute_dtype) if config is not None else compute_dtype
        self.skip_weight_param_allocation = skip_weight_param_allocation
        shape = (output_size, input_size) if transpose_b else (input_size, output_size)
        self.weight = None
        if not skip_weight_param_allocation:
            w = torch.empty(shape, dtype=self.params_dtype, device=device)
            nn.init.normal_(w, std=0.01) if init_method == "normal" else w.zero_()
            self.weight = nn.Parameter(w, requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(output_size, dtype=self.params_dtype, device=device), requires_grad=False) \
            if bias else None

    def _forward(self, x, weight=None):
        if weight is None:
            if self.skip_weight_param_allocation:
                raise ValueError("For this linear, when `skip_weight_param_allocation` is enabled, `weight` is required, "
                                 "but got None")
            weight = self.weight
        out_shape = tuple(x.shape[:-1]) + (self.output_size,)
        ori = x.dtype
        w = weight.to(self.compute_dtype)
        w = w if self.transpose_b else w.t()
        y = F.linear(x.reshape(-1, self.input_size).to(self.compute_dtype), w,
                     self.bias.to(self.compute_dtype) if self.has_bias else None)
        return y.to(ori).reshape(out_shape)


class ColumnParallelLinear(_ParallelLinearBase):
    """tensor_parallel/layers.py:44-212 at tp = 1 (no gather, options the reference rejects are rejected)."""

    def __init__(self, input_size, output_size, *, config=None, init_method="normal", bias=True, gather_output=False,
                 stride=1, keep_master_weight_for_test=False, skip_bias_add=False, skip_weight_param_allocation=False,
                 embedding_activation_buffer=None, is_expert=False, tp_comm_buffer_name=None, transpose_b=True,
                 compute_dtype=torch.bfloat16, tp_group=None, device="cuda"):
        if stride > 1:
            raise NotImplementedError("For ColumnParallelLinear, `stride > 1` is not supported for now, "
                                      "but got `stride={}`".format(stride))
        for flag, name in ((keep_master_weight_for_test, "keep_master_weight_for_test"), (skip_bias_add, "skip_bias_add=True"),
                           (embedding_activation_buffer is not None, "embedding_activation_buffer"),
                           (is_expert, "is_expert"), (tp_comm_buffer_name is not None, "tp_comm_buffer_name")):
            if flag:
                raise NotImplementedError(f"For ColumnParallelLinear, `{name}` is not supported for now")
        super().__init__(input_size, output_size, config=config, init_method=init_method, bias=bias,
                         transpose_b=transpose_b, compute_dtype=compute_dtype,
                         skip_weight_param_allocation=skip_weight_param_allocation, device=device)
        self.gather_output = gather_output
        self.output_size_per_partition = output_size

    def forward(self, input_, weight=None):
        return self._forward(input_, weight)

    construct = forward


class QKVParallelLinear(ColumnParallelLinear):
    """tensor_parallel/layers.py:215-286: one projection with output rows [q | k | v]."""

    def __init__(self, hidden_size, head_size, total_num_heads, total_num_kv_heads, *, config=None, bias=True, **kw):
        self.hidden_size, self.head_size = hidden_size, head_size
        self.total_num_heads, self.total_num_kv_heads = total_num_heads, total_num_kv_heads
        self.num_heads, self.num_kv_heads = total_num_heads, total_num_kv_heads
        super().__init__(hidden_size, (total_num_heads + 2 * total_num_kv_heads) * head_size, config=config, bias=bias, **kw)


class RowParallelLinear(_ParallelLinearBase):
    """tensor_parallel/layers.py:289-431 at tp = 1 (the all-reduce is the identity)."""

    def __init__(self, input_size, output_size, *, config=None, init_method="normal", bias=True, input_is_parallel=True,
                 skip_bias_add=False, stride=1, keep_master_weight_for_test=False, is_expert=False,
                 tp_comm_buffer_name=None, transpose_b=True, compute_dtype=torch.bfloat16, tp_group=None, device="cuda"):
        if stride > 1 or keep_master_weight_for_test or skip_bias_add or is_expert or tp_comm_buffer_name is not None:
            raise NotImplementedError("For RowParallelLinear, stride > 1 / keep_master_weight_for_test / skip_bias_add / "
                                      "is_expert / tp_comm_buffer_name are not supported for now")
        super().__init__(input_size, output_size, config=config, init_method=init_method, bias=bias,
                         transpose_b=transpose_b, compute_dtype=compute_dtype, device=device)
        self.input_is_parallel = input_is_parallel
        self.input_size_per_partition = input_size

    def forward(self, input_):
        return self._forward(input_)

    construct = forward


class ReplicatedLinear(_ParallelLinearBase):
    """tensor_parallel/layers.py:434-555."""

    def __init__(self, input_size, output_size, *, config=None, init_method="normal", bias=True, transpose_b=True,
                 compute_dtype=torch.bfloat16, device="cuda", **unused):
        super().__init__(input_size, output_size, config=config, init_method=init_method, bias=bias,
                         transpose_b=transpose_b, compute_dtype=compute_dtype, device=device)

    def forward(self, input_):
        return self._forward(input_)

    construct = forward


LINEAR_TYPES = (Linear, ColumnParallelLinear, RowParallelLinear, ReplicatedLinear)


def linear_geometry(cell):
    """(in_features, out_features, has_bias, compute dtype) of any float linear cell above."""
    if isinstance(cell, Linear):
        return cell.in_channels, cell.out_channels, cell.has_bias, cell.dtype
    return cell.input_size, cell.output_size, cell.has_bias, cell.compute_dtype
