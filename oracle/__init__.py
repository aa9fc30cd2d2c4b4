"""CPU oracle for the quantized decode path.  TEST INFRASTRUCTURE ONLY.

This package restates, in numpy, the arithmetic of the reference's decode step
(KV scatter, paged attention, RoPE, RMSNorm, SwiGLU, W8A16 / W8A8 linears,
top-k router, expert permute / grouped MLP / unpermute).  Every function cites
the reference file:line it follows.  It exists to *check* the HIP kernels:
only the test-suite, the smoke check and the benchmark's CPU-baseline leg may
import it.  The product package never does, and fails loudly when its HIP
library is missing rather than computing anything here.

Pinning status of each function (what fixes it besides its own formula):

  reshape_and_cache        closed form (copy); indirectly by the reference's
                           flash-attention decode vectors (tests/golden/flash_attention.npz)
  paged_attention_decode   reference vectors decode_output_{1,2} (flash_attention.npz,
                           attention.npz); reduces to softmax(QK^T s)V on the gathered prefix
  causal_prefill_attention reference vectors prefill_output_{1,2} (flash_attention.npz, attention.npz)
  paged_attention_prefill  its two special cases are the two pinned functions above: one query per
                           sequence = paged_attention_decode, empty cache before the step =
                           causal_prefill_attention (tests); the golden prefill vectors through the cache
  mla_paged_attention_     its reduction to paged_attention_decode (pinned above) with one kv head: equal
   decode                  when v_dim = Dk, and its first v_dim columns otherwise (tests)
  mla_self_attention_      the layer around it (oracle/mla.py): the decode form (absorbed weights, latent cache)
   decode / _prefill       against the prefill form (up-projected keys / values: the definition) on the same
                           tokens (tests); the pieces underneath are the pinned functions of this list
  rope tables / apply      reference vectors (rotary.npz: default, Llama3, YaRN; prefill+decode)
  rms_norm / layer_norm    reference vectors (norm.npz)
  silu_mul                 reference vectors (activation.npz)
  linear / mlp             reference vectors (column/row_parallel_linear.npz, mlp.npz)
  moe_layer (router +      reference vectors (moe.npz tp1, tp1_no_shared; wiring-level pin,
   permute + experts)      group limiting not exercised there)
  topk_router group limit  brute force over subsets on tiny sizes (tests) — the reference
                           holds no vector that exercises n_group > topk_group
  checkpoint.qkv/ffn_      hand-computed small cases; labelled rows (every output row must carry the
   concat_hf2mg            (kind, head, channel) label the layout names); closed form (a permutation)
  quantize_weight_int8,    PARITY UNPINNED: the arithmetic lives in mindspore_gs / CANN
  w8a16_linear,            (not vendored, no reference vector).  int32 accumulators are
  dynamic_quant_per_token, pinned against exact integer matmul; rounding mode, clamp range
  static_quant_per_tensor,
  w8a8_linear              and dequant order are this build's declared convention.
  quantize_weight_int4,    PARITY UNPINNED against the reference for the same reason (s = max|w| / 7 per channel or per
  w4a16_linear             channel and group, q in -8 .. 7, the group's scale applied to the group's sum: declared);
                           pinned against that convention by rails, the half-step round trip, exactness on
                           power-of-two grids and the pack / unpack identity (tests/test_host_logic.py)
  quantize_kv_int8,        PARITY UNPINNED against the reference for the same reason (the convention, affine per
  dequantize_kv_int8       channel with ties to even and rails -128 / 127, is declared); the two functions
                           themselves are pinned against that convention by hand-computed values, the offset's
                           direction, clipping at the rails, the half-step round trip and torch's affine
                           per-channel quantiser on power-of-two scales (tests/test_host_logic.py)
"""
from .numerics import (round_bf16, round_fp16, round_to, double_benchmark,
                       DoubleBenchmarkResult)
from .attention import (reshape_and_cache, paged_attention_decode, gather_kv,
                        decode_slot_mapping, prefill_slot_mapping, causal_prefill_attention,
                        paged_attention_prefill, mla_paged_attention_decode)
from .rope import (rope_inv_freq_default, rope_inv_freq_llama3, rope_inv_freq_yarn,
                   yarn_mscale, rope_cos_sin_table, apply_rotary_half)
from .dense import rms_norm, layer_norm, silu, silu_mul, linear, mlp
from .quant import (quantize_weight_int8, w8a16_linear, dynamic_quant_per_token, static_quant_per_tensor,
                    int8_gemm_i32, w8a8_linear, quantize_kv_int8, quantize_kv_int8_per_token, dequantize_kv_int8, quantize_weight_int4,
                    w4a16_linear, pack_qint4x2, unpack_qint4x2)
from . import checkpoint
from .moe import (topk_router, moe_permute, grouped_mlp, moe_unpermute, moe_layer,
                  grouped_matmul)
from .layer import decode_layer_w8a16, decode_layer_w8a8
from .mla import mla_project, mla_self_attention_decode, mla_self_attention_prefill
