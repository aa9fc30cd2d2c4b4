"""ctypes binding of libmf_decode.so (the C ABI declared in include/mf_decode.h).

The library is the product: if it has not been built, loading fails loudly — there is no CPU fallback.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmf_decode.so")

MF_BF16, MF_FP16, MF_FP32 = 0, 1, 2

_c = ctypes
_P, _I, _L, _F, _Z = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float, _c.c_size_t

# name -> (restype, argtypes); mirrors include/mf_decode.h one to one
SIGNATURES = {
    "mf_version": (_c.c_char_p, []),
    "mf_last_error": (_c.c_char_p, []),
    "mf_reshape_and_cache": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _L, _L, _L, _I, _P]),
    "mf_rope_half": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _L, _L, _I, _I, _P]),
    "mf_rope_and_cache": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _L, _L, _L, _L, _I, _I, _P]),
    "mf_swap_blocks": (_I, [_P, _P, _P, _L, _L, _L, _L, _I, _P]),
    "mf_paged_attention_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "mf_paged_attention_decode_dynamic_quant": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                                                     _F, _L, _I, _P, _Z, _P]),
    "mf_paged_attention_decode": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _L, _I, _P, _Z, _P]),
    "mf_paged_attention_decode_static": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _L, _I, _P]),
    "mf_quant_reshape_and_cache": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _L, _L, _L, _I, _P]),
    "mf_paged_attention_decode_int8kv": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _L, _I, _P,
                                              _Z, _P]),
    "mf_paged_attention_prefill_int8kv": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _L,
                                               _I, _P, _Z, _P]),
    "mf_dynamic_quant_reshape_and_cache": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _L, _L, _L, _I, _P]),
    "mf_paged_attention_decode_int8kv_per_token": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F,
                                                        _L, _I, _P, _Z, _P]),
    "mf_paged_attention_prefill_int8kv_per_token": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                                                         _I, _F, _L, _I, _P, _Z, _P]),
    "mf_causal_attention_qk192_v128": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _L, _L, _L, _I, _P, _Z, _P]),
    "mf_mla_paged_attention_workspace_bytes": (_Z, [_I, _I, _I]),
    "mf_mla_paged_attention_decode": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _L, _I, _P, _Z, _P]),
    "mf_mla_norm_rope_cache": (_I, [_P, _L, _L, _P, _L, _L, _P, _P, _P, _L, _P, _I, _F, _P, _P, _I, _P, _P, _L, _I, _I, _I,
                                    _I, _I, _P]),
    "mf_mla_absorb_bmm": (_I, [_P, _P, _P, _I, _I, _I, _I, _L, _L, _L, _L, _I, _P]),
    "mf_paged_attention_prefill_workspace_bytes": (_Z, [_I, _I, _I, _I, _I, _I]),
    "mf_paged_attention_prefill": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _L, _L, _I,
                                        _P, _Z, _P]),
    "mf_rmsnorm": (_I, [_P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _P]),
    "mf_rmsnorm_strided": (_I, [_P, _P, _L, _P, _F, _I, _I, _I, _I, _P]),
    "mf_silu_mul": (_I, [_P, _P, _I, _I, _I, _I, _P]),
    "mf_add": (_I, [_P, _P, _P, _L, _I, _P]),
    "mf_scale_columns": (_I, [_P, _P, _P, _L, _I, _I, _P]),
    "mf_w8a16_packed_bytes": (_Z, [_I, _I]),
    "mf_w8a16_pack_weight": (_I, [_P, _P, _I, _I, _P]),
    "mf_w8a16_workspace_bytes": (_Z, [_I, _I, _I]),
    "mf_w4a16_packed_bytes": (_Z, [_I, _I]),
    "mf_w4a16_pack_weight": (_I, [_P, _P, _I, _I, _P]),
    "mf_w4a16_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "mf_w4a16_gemm": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "mf_w8a16_gemm": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P]),
    "mf_w8a16_gemm_add_rmsnorm": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "mf_w8a16_gemm_rmsnorm_leading": (_I, [_P, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "mf_w8a16_qkv_rope_and_cache": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _L, _I, _I, _I, _P, _Z, _P]),
    "mf_w8a16_qkv_rope_and_quant_cache": (_I, [_P] * 12 + [_I] * 4 + [_L] + [_I] * 3 + [_P, _Z, _P]),
    "mf_w8a16_gemm_silu_mul": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P]),
    "mf_dynamic_quant_per_token": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mf_static_quant_per_tensor": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mf_rmsnorm_dynamic_quant": (_I, [_P, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _P]),
    "mf_silu_mul_dynamic_quant": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mf_w8a8_workspace_bytes": (_Z, [_I, _I, _I]),
    "mf_w8a8_gemm": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "mf_w8a8_gemm_add_rmsnorm_quant": (_I, [_P] * 11 + [_F] + [_I] * 7 + [_P, _Z, _P]),
    "mf_w8a8_qkv_rope_and_cache": (_I, [_P] * 11 + [_I] * 4 + [_L] + [_I] * 4 + [_P, _Z, _P]),
    "mf_router_gate_workspace_bytes": (_Z, [_I, _I, _I]),
    "mf_router_gate_gemm": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "mf_grouped_dynamic_quant_per_token": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mf_grouped_silu_mul_dynamic_quant": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "mf_moe_route": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P]),
    "mf_moe_permute": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mf_grouped_w8a16_gemm": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mf_grouped_w8a16_gemm_silu_mul": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mf_grouped_w8a8_gemm": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mf_moe_unpermute": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
}

_lib = None


class MfKernelError(RuntimeError):
    """A C-ABI call returned a non-zero hipError_t."""


def load():
    """Load the shared library once; raise if it is missing (build it with mindformers_amd/build.py)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: the HIP kernels are not built. Run `python mindformers_amd/build.py` "
            "(or __graft_entry__.build()). There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().mf_last_error().decode() if rc == 1 else ""
        raise MfKernelError(f"{what} failed with hipError {rc}" + (f": {msg}" if msg else ""))


def dtype_code(dtype):
    if dtype == torch.bfloat16:
        return MF_BF16
    if dtype == torch.float16:
        return MF_FP16
    if dtype == torch.float32:
        return MF_FP32
    raise TypeError(f"unsupported dtype {dtype}")


def ptr(t):
    return None if t is None else t.data_ptr()


def stream_ptr(device=None):
    return torch.cuda.current_stream(device).cuda_stream
