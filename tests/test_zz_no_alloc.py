"""The decode-attention entry point that allocates nothing (partition partials in a device array built into the
library): called through the C ABI, its output must carry the bits of mf_paged_attention_decode with a caller
workspace, on two calls in a row (the second on a smaller input, so stale partials of the first are in the array),
and shapes beyond the built-in array must be refused.  GPU only."""
import numpy as np
import pytest
import torch

from helpers import dev, make_paged_cache

pytestmark = pytest.mark.gpu


def _both(lib, rng, b, nh, nkv, d, bs, lens, max_blocks, dtype):
    from mindformers_amd._lib import check, dtype_code, ptr, stream_ptr
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype, max_blocks=max_blocks)
    kc, vc = dev(kc, dtype), dev(vc, dtype)
    q = dev(rng.normal(size=(b, nh * d)), dtype)
    tb = dev(tables, torch.int32)
    ln = dev(np.asarray(lens, np.int32), torch.int32)
    scale = float(1.0 / np.sqrt(d))
    need = lib.mf_paged_attention_workspace_bytes(b, nh, d, max_blocks * bs)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    ref = torch.full((b, nh * d), 3.0, dtype=dtype, device="cuda")
    st = stream_ptr(q.device)
    check(lib.mf_paged_attention_decode(ptr(ref), ptr(q), ptr(kc), ptr(vc), ptr(tb), ptr(ln), b, nh, nkv, d, bs,
                                        max_blocks, nb, scale, 0, dtype_code(dtype), ptr(ws), need, st),
          "mf_paged_attention_decode")
    out = torch.full((b, nh * d), -5.0, dtype=dtype, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    check(lib.mf_paged_attention_decode_static(ptr(out), ptr(q), ptr(kc), ptr(vc), ptr(tb), ptr(ln), b, nh, nkv, d, bs,
                                               max_blocks, nb, scale, 0, dtype_code(dtype), st),
          "mf_paged_attention_decode_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return out, ref, need


def test_static_scratch_decode_equals_the_workspace_entry_point_twice_in_a_row():
    from mindformers_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(77)
    # first call: 12 sequences, up to 16 partitions each, one without context
    lens = rng.integers(300, 4096, 12)
    lens[3] = 0
    out, ref, need = _both(lib, rng, 12, 32, 8, 128, 128, lens, 32, torch.bfloat16)
    assert need > 0 and torch.equal(out, ref)
    assert not out[3].any() and out[2].any()                   # the empty sequence's row is zeros
    # second call, smaller in every respect (batch, heads, partitions): the array still holds the first call's partials
    lens = rng.integers(100, 900, 3)
    lens[1] = 0                                                # reads no partition: stale partials must not show
    out, ref, need = _both(lib, rng, 3, 8, 2, 64, 16, lens, 64, torch.float16)
    assert need > 0 and torch.equal(out, ref)
    assert not out[1].any()
    # a single-partition shape uses no partials at all
    out, ref, need = _both(lib, rng, 3, 4, 4, 32, 16, [5, 0, 200], 16, torch.float16)
    assert need == 0 and torch.equal(out, ref)
    assert not out[1].any()                                    # the single-partition path zeroes empty rows itself


def test_static_scratch_decode_refuses_shapes_beyond_the_array():
    from mindformers_amd import _lib
    from mindformers_amd._lib import ptr, stream_ptr
    lib = _lib.load()
    b, nh, d, bs, max_blocks = 64, 64, 128, 128, 512            # 64 x 64 heads x 128 partitions x 130 floats = 273 MB
    assert lib.mf_paged_attention_workspace_bytes(b, nh, d, max_blocks * bs) > (48 << 20)
    t = torch.zeros(16, dtype=torch.bfloat16, device="cuda")
    i = torch.zeros(16, dtype=torch.int32, device="cuda")
    rc = lib.mf_paged_attention_decode_static(ptr(t), ptr(t), ptr(t), ptr(t), ptr(i), ptr(i), b, nh, 8, d, bs, max_blocks,
                                              4, 0.1, 0, 0, stream_ptr(t.device))
    assert rc == 1 and b"built-in scratch" in lib.mf_last_error()
