"""One quantized decode layer wired from the kernels: the caller of the hot path.

Mirrors the pre-norm residual layer of the reference (mindformers/models/llama/llama_transformer.py:1036-1070
LLamaDecodeLayer.construct with the use_past branch of LLamaAttention.construct :467-569, and
mindformers/parallel_core/inference/transformer/transformer_layer.py:296-355) with the fused projection
layouts of the Megatron-style stack: linear_qkv rows are [q | k | v] (attention.py:344-349) and linear_fc1
rows are [gate | hidden] (mlp.py:135-140).

Launch sequence per decode step (one stream, no host synchronisation):
  rmsnorm -> qkv GEMM -> rope+KV scatter -> paged attention (+ partition reduce) -> wo GEMM (+residual)
  -> rmsnorm -> fc1 GEMM -> silu*mul -> fc2 GEMM (+residual)
"""
import math

import torch
from torch import nn

from . import ops


class QuantDecodeLayer(nn.Module):
    """W8A16 (``act_quant=False``) or W8A8 per-token-dynamic (``act_quant=True``) decode layer.

    Parameters are plain buffers: ``{qkv,wo,fc1,fc2}_w`` int8 [out, in], ``*_s`` fp32 [out], optional
    ``*_b`` bias, optional ``*_smooth`` fp32 [in] (W8A8), ``attn_norm`` / ``ffn_norm`` gammas.
    """

    NAMES = ("qkv", "wo", "fc1", "fc2")

    def __init__(self, hidden, n_head, n_kv_head, head_dim, ffn, eps=1e-5, dtype=torch.bfloat16, act_quant=False,
                 qkv_bias=False, device="cuda"):
        super().__init__()
        self.hidden, self.n_head, self.n_kv_head, self.head_dim, self.ffn = hidden, n_head, n_kv_head, head_dim, ffn
        self.eps, self.dtype, self.act_quant = eps, dtype, act_quant
        self.scale_value = 1.0 / math.sqrt(head_dim)
        self._packed = {}
        self.raw_weights = {}                                 # host copies of released row-major weights
        shapes = {"qkv": ((n_head + 2 * n_kv_head) * head_dim, hidden), "wo": (hidden, n_head * head_dim),
                  "fc1": (2 * ffn, hidden), "fc2": (hidden, ffn)}
        for name, (n, k) in shapes.items():
            self.register_buffer(f"{name}_w", torch.zeros(n, k, dtype=torch.int8, device=device))
            self.register_buffer(f"{name}_s", torch.ones(n, dtype=torch.float32, device=device))
            setattr(self, f"{name}_b", None)
            if act_quant:
                self.register_buffer(f"{name}_smooth", torch.ones(k, dtype=torch.float32, device=device))
        if qkv_bias:
            self.qkv_b = torch.zeros(shapes["qkv"][0], dtype=dtype, device=device)
        # int8 KV caches: per-channel dequantisation parameters, float32 [2, n_kv_head * head_dim] (keys, values)
        self.kv_scale, self.kv_offset = None, None
        self.register_buffer("attn_norm", torch.ones(hidden, dtype=torch.float32, device=device))
        self.register_buffer("ffn_norm", torch.ones(hidden, dtype=torch.float32, device=device))

    def _linear(self, x, name, residual=None, quantized=None):
        """``quantized``: (xq, scale) when the producer of x already quantised it (W8A8 only)."""
        b = getattr(self, f"{name}_b")
        packed = self._packed.get(name)
        if packed is None:
            raise RuntimeError("call prepare() after loading the weights (packs them for the GEMM kernels)")
        if self.act_quant:
            xq, xs = quantized or ops.dynamic_quant(x, getattr(self, f"{name}_smooth"), tiled=True)
            return ops.w8a8_linear(xq, xs, packed, out_dtype=self.dtype, bias=b, residual=residual)
        return ops.w8a16_linear(x, packed, bias=b, residual=residual)

    def prepare(self, release_raw=False):
        """Pack the int8 weights into the tile order the GEMM kernels stream.  Call once after loading weights, and
        again after loading new ones.  The packed copy is the only one the kernels read.  With ``release_raw`` the
        row-major ``*_w`` tensors leave the module's buffers for host copies kept as plain attributes (``raw_weights``,
        still readable, e.g. for export), so that the device holds every weight once and a later ``.to(device)`` does
        not bring a second copy back; the ``*_w`` names then resolve to those host copies."""
        dev = self.attn_norm.device
        for name in self.NAMES:
            w, s = getattr(self, f"{name}_w").to(dev), getattr(self, f"{name}_s")
            # W8A16: the gate/up projection runs fused with SiLU * mul, which wants gate/up rows interleaved
            gated = name == "fc1" and not self.act_quant and getattr(self, "fc1_b") is None
            self._packed[name] = ops.pack_w8a16_gated(w, s, "halves") if gated else ops.pack_w8a16(w, s)
            if release_raw:
                self._buffers.pop(f"{name}_w", None)
                self.raw_weights[f"{name}_w"] = w.cpu()
        return self

    def __getattr__(self, name):
        raw = self.__dict__.get("raw_weights")
        if raw is not None and name in raw:
            return raw[name]
        return super().__getattr__(name)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # new weights invalidate the packed copies: the next forward asks for prepare() again
        if any(k.startswith(prefix) and k[len(prefix):].rsplit("_", 1)[0] in self.NAMES for k in state_dict):
            self._packed.clear()
        return super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def set_kv_quant(self, scale, offset=None):
        """Per-channel parameters of int8 caches: x ~ (q - offset) * scale; float32 [2, n_kv_head * head_dim]."""
        row = self.n_kv_head * self.head_dim
        if tuple(scale.shape) != (2, row) or (offset is not None and tuple(offset.shape) != (2, row)):
            raise ValueError(f"kv scale / offset must be [2, {row}]")
        self.kv_scale = scale.to(torch.float32).contiguous()
        self.kv_offset = None if offset is None else offset.to(torch.float32).contiguous()
        return self

    def attend(self, q, key_cache, value_cache, block_tables, batch_valid_length, q_starts=None):
        """Attention of this step's queries over the caches (16-bit or int8)."""
        if key_cache.dtype == torch.int8:
            if self.kv_scale is None:
                raise RuntimeError("int8 caches need set_kv_quant(scale, offset)")
            return ops.paged_attention_int8kv(q, key_cache, value_cache, block_tables, batch_valid_length,
                                              self.kv_scale, self.kv_offset, self.n_head, self.n_kv_head,
                                              self.scale_value, q_starts=q_starts)
        if q_starts is None:
            return ops.paged_attention(q, key_cache, value_cache, block_tables, batch_valid_length, self.n_head,
                                       self.n_kv_head, self.scale_value)
        return ops.paged_attention_prefill(q, key_cache, value_cache, block_tables, batch_valid_length, q_starts,
                                           self.n_head, self.n_kv_head, self.scale_value)

    def forward(self, x, key_cache, value_cache, block_tables, batch_valid_length, slot_mapping, cos, sin,
                q_starts=None, normed=None, next_norm=None):
        """x [T, hidden]; caches [num_blocks, block_size, n_kv, D]; cos/sin [T, D] rows for this step's
        positions; batch_valid_length counts the tokens written by this step.  Decode: one token per sequence.
        Prefill / chunked prefill: ``q_starts`` int32 [B + 1] gives the row range of every sequence in x, its new
        tokens are scattered first and then attend causally over the cache.

        Chaining layers: with ``next_norm`` = (gamma, eps) of the norm that follows this layer (the next layer's
        attention norm, or the model's final norm) the call returns (out, norm(out) * gamma), and the next layer
        takes that second tensor as ``normed`` in place of computing its attention norm.  The norm then runs inside
        the kernel that finishes this layer's last projection (same bits, one launch fewer).  A W8A8 layer takes
        ``next_norm`` = (gamma, eps, smooth) with the next layer's QKV smoothing vector and hands over the quantised
        norm output (xq, scale), which is what a W8A8 layer accepts as ``normed``."""
        nq, nkv = self.n_head * self.head_dim, self.n_kv_head * self.head_dim
        if self.act_quant:                                    # W8A8: the norm feeds the quantised projection only
            if isinstance(normed, tuple):
                n1, n1q = None, normed
            elif normed is not None:
                n1, n1q = None, ops.dynamic_quant(normed, self.qkv_smooth, tiled=True)
            else:
                n1, n1q = None, ops.rms_norm_dynamic_quant(x, self.attn_norm, self.eps, self.qkv_smooth, tiled=True)
        else:
            n1, n1q = (normed if normed is not None else ops.rms_norm(x, self.attn_norm, self.eps)), None
        if key_cache.dtype == torch.int8:                     # rotate, then quantize into the int8 caches
            if self.kv_scale is None:
                raise RuntimeError("int8 caches need set_kv_quant(scale, offset)")
            if not self.act_quant and self.head_dim % 16 == 0 and self._packed.get("qkv") is not None:
                q = ops.w8a16_qkv_rope_and_cache(n1, self._packed["qkv"], cos, sin, key_cache, value_cache,
                                                 slot_mapping, self.n_head, bias=self.qkv_b, kv_scale=self.kv_scale,
                                                 kv_offset=self.kv_offset)
            else:
                qkv = self._linear(n1, "qkv", quantized=n1q)
                q, k, v = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:]
                ops.apply_rotary_pos_emb(q, k, cos, sin, self.n_head, self.n_kv_head, self.head_dim)
                ops.quant_reshape_and_cache(k, v, key_cache, value_cache, slot_mapping, self.kv_scale, self.kv_offset)
        elif self.act_quant and self.head_dim % 16 == 0:      # W8A8: projection + RoPE + cache write in one call
            if self._packed.get("qkv") is None:
                raise RuntimeError("call prepare() after loading the weights (packs them for the GEMM kernels)")
            q = ops.w8a8_qkv_rope_and_cache(n1q[0], n1q[1], self._packed["qkv"], cos, sin, key_cache, value_cache,
                                            slot_mapping, self.n_head, bias=self.qkv_b)
        elif self.act_quant or self.head_dim % 16:
            qkv = self._linear(n1, "qkv", quantized=n1q)
            q, k, v = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:]
            ops.rope_and_cache(q, k, v, cos, sin, key_cache, value_cache, slot_mapping, self.n_head)
        else:                                                 # W8A16: projection + RoPE + cache write in one call
            if self._packed.get("qkv") is None:
                raise RuntimeError("call prepare() after loading the weights (packs them for the GEMM kernels)")
            q = ops.w8a16_qkv_rope_and_cache(n1, self._packed["qkv"], cos, sin, key_cache, value_cache, slot_mapping,
                                             self.n_head, bias=self.qkv_b)
        if self.act_quant and q_starts is None and key_cache.dtype != torch.int8:
            # W8A8 decode: the attention output is only read by wo's per-token quantisation, done with the combine of
            # the partitions
            _, aq, a_s = ops.paged_attention(q, key_cache, value_cache, block_tables, batch_valid_length, self.n_head,
                                             self.n_kv_head, self.scale_value, quant=(self.wo_smooth, True))
            attn = None
        else:
            attn = self.attend(q, key_cache, value_cache, block_tables, batch_valid_length, q_starts)
        if self.act_quant:
            # W8A8: wo + residual + norm + quantisation in one call, gate/up, activation + quantisation, and fc2
            # (+ residual + the next layer's norm and quantisation when layers are chained)
            if self._packed.get("wo") is None:
                raise RuntimeError("call prepare() after loading the weights (packs them for the GEMM kernels)")
            if attn is not None:
                aq, a_s = ops.dynamic_quant(attn, self.wo_smooth, tiled=True)
            h, n2x, n2s = ops.w8a8_linear_add_rmsnorm_quant(aq, a_s, self._packed["wo"], x, self.ffn_norm, self.eps,
                                                            self.fc1_smooth, bias=self.wo_b)
            actq = ops.silu_mul_dynamic_quant(self._linear(None, "fc1", quantized=(n2x, n2s)), self.fc2_smooth,
                                              tiled=True)
            if next_norm is None:
                return self._linear(None, "fc2", residual=h, quantized=actq)
            gamma, eps, smooth = next_norm
            out, nx, ns = ops.w8a8_linear_add_rmsnorm_quant(actq[0], actq[1], self._packed["fc2"], h, gamma, eps, smooth,
                                                            bias=self.fc2_b)
            return out, (nx, ns)
        if self.wo_b is not None:
            h = self._linear(attn, "wo", residual=x)
            n2 = ops.rms_norm(h, self.ffn_norm, self.eps)
        else:                                                 # W8A16: projection + residual + norm in one call
            if self._packed.get("wo") is None:
                raise RuntimeError("call prepare() after loading the weights (packs them for the GEMM kernels)")
            h, n2 = ops.w8a16_linear_add_rmsnorm(attn, self._packed["wo"], x, self.ffn_norm, self.eps)
        if next_norm is not None and self.fc2_b is None and self._packed.get("fc2") is not None:
            return ops.w8a16_linear_add_rmsnorm(self.gate_up(n2), self._packed["fc2"], h, next_norm[0], next_norm[1])
        return self._chain(self._linear(self.gate_up(n2), "fc2", residual=h), next_norm)

    @staticmethod
    def _chain(out, next_norm):
        return out if next_norm is None else (out, ops.rms_norm(out, next_norm[0], next_norm[1]))

    def gate_up(self, n2):
        """silu(gate) * up of the MLP input projection: one fused kernel on the W8A16 path."""
        fc1 = self._packed.get("fc1")
        if fc1 is not None and fc1.gated:
            return ops.w8a16_gated_linear(n2, fc1)
        return ops.silu_mul(self._linear(n2, "fc1"))

    construct = forward

    def weight_bytes(self):
        return sum(getattr(self, f"{n}_w").numel() for n in self.NAMES)
