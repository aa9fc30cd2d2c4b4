"""Parity of the HIP kernels (called through the C ABI) against the CPU oracle.  GPU only.

Bars: bit-exact for the KV scatter, the int8 quantisation grid, int32 accumulators and all index outputs;
for floating-point outputs |err| <= 1.5 * eps(dtype) * M where M is the magnitude the rounding error of that
op scales with (sum of |terms| of the dot product / convex combination), eps(bf16) = 2^-8, eps(fp16) = 2^-11.
"""
import os

import numpy as np
import pytest
import torch

import oracle as O
from helpers import EPS, NAME, assert_within, dev, make_paged_cache, rounded, to_np, untile_int8

pytestmark = pytest.mark.gpu

ops = None


@pytest.fixture(scope="module", autouse=True)
def _load_ops():
    global ops
    assert torch.cuda.is_available(), "these tests need the GPU"
    from mindformers_amd import ops as _ops
    ops = _ops
    yield


# ------------------------------------------------------------------------------------------- KV scatter
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,n_kv,d,bs,nb", [(64, 8, 128, 128, 40), (4, 2, 64, 16, 64), (7, 1, 32, 16, 9), (3, 3, 20, 4, 11)])
def test_reshape_and_cache_bit_exact(dtype, t, n_kv, d, bs, nb):
    rng = np.random.default_rng(1)
    k = rounded(rng.normal(size=(t, n_kv * d)), dtype)
    v = rounded(rng.normal(size=(t, n_kv * d)), dtype)
    kc0 = rounded(rng.normal(size=(nb, bs, n_kv, d)), dtype)
    vc0 = rounded(rng.normal(size=(nb, bs, n_kv, d)), dtype)
    slots = rng.permutation(nb * bs)[:t].astype(np.int32)
    slots[rng.integers(0, t)] = -1                       # one padding row
    kc_ref, vc_ref = kc0.copy(), vc0.copy()
    O.reshape_and_cache(k, v, kc_ref, vc_ref, slots)
    kc, vc = dev(kc0, dtype), dev(vc0, dtype)
    out = ops.reshape_and_cache(dev(k, dtype), dev(v, dtype), kc, vc, dev(slots, torch.int32))
    torch.cuda.synchronize()
    assert np.array_equal(to_np(kc), kc_ref) and np.array_equal(to_np(vc), vc_ref)
    assert np.array_equal(to_np(out), k)


def test_reshape_and_cache_empty_and_key_only():
    kc = torch.zeros(4, 16, 2, 32, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros_like(kc)
    empty = torch.zeros(0, 64, dtype=torch.bfloat16, device="cuda")
    ops.reshape_and_cache(empty, empty, kc, vc, torch.zeros(0, dtype=torch.int32, device="cuda"))
    k = torch.randn(3, 64, device="cuda").to(torch.bfloat16)
    ops.reshape_and_cache(k, None, kc, None, torch.tensor([5, 63, 0], dtype=torch.int32, device="cuda"))
    torch.cuda.synchronize()
    flat = kc.view(64, 64)
    assert torch.equal(flat[5], k[0]) and torch.equal(flat[63], k[1]) and torch.equal(flat[0], k[2])
    assert int((flat != 0).any(dim=1).sum()) <= 3 and not bool(vc.any())


# ------------------------------------------------------------------------------------------- RoPE
@pytest.mark.parametrize("dtype,table", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32)])
@pytest.mark.parametrize("t,nh,nkv,d", [(64, 32, 8, 128), (4, 8, 2, 64), (2, 1, 1, 32)])
def test_rope_half(dtype, table, t, nh, nkv, d):
    rng = np.random.default_rng(2)
    q = rounded(rng.normal(size=(t, nh * d)), dtype)
    k = rounded(rng.normal(size=(t, nkv * d)), dtype)
    cos, sin = O.rope_cos_sin_table(O.rope_inv_freq_default(d), 4096, 1.0, "fp32" if table == torch.float32 else NAME[table])
    pos = rng.integers(0, 4096, t)
    c, s = cos[pos], sin[pos]
    qd, kd = dev(q, dtype), dev(k, dtype)
    ops.apply_rotary_pos_emb(qd, kd, dev(c, table), dev(s, table), nh, nkv, d)
    for got, x, n in ((qd, q, nh), (kd, k, nkv)):
        ref = O.apply_rotary_half(x, c, s, n)
        xh = np.abs(x.reshape(t, n, d))
        swapped = np.concatenate((xh[..., d // 2:], xh[..., :d // 2]), -1)
        mag = xh * np.abs(c)[:, None, :] + swapped * np.abs(s)[:, None, :]
        assert_within(to_np(got), ref, mag.reshape(t, n * d), dtype, ulps=1.0, what="rope")


def test_rope_golden_decode_vectors(golden_dir):
    """The reference's own decode vectors (position 1, bf16 tables), through the kernel."""
    z = np.load(os.path.join(golden_dir, "rotary.npz"))
    d = int(z["meta_kv_channels"])
    cos, sin = O.rope_cos_sin_table(O.rope_inv_freq_default(d), 8, 1.0, "bf16")
    q = dev(O.round_bf16(z["in_decode_query_for_decode"]), torch.bfloat16)
    k = dev(O.round_bf16(z["in_decode_key_for_decode"]), torch.bfloat16)
    pos = np.array([1, 1])
    ops.apply_rotary_pos_emb(q, k, dev(cos[pos], torch.bfloat16), dev(sin[pos], torch.bfloat16), 1, 1, d)
    for got, name in ((q, "q"), (k, "k")):
        res = O.double_benchmark(to_np(got), z[f"gpu_rope_{name}_emb1_for_decode"], z[f"golden_rope_{name}_emb1_for_decode"])
        assert res.ok, res.messages


def test_rope_and_cache_matches_separate_ops():
    rng = np.random.default_rng(3)
    t, nh, nkv, d, bs, nb = 16, 8, 2, 64, 16, 12
    dtype = torch.float16
    q = dev(rng.normal(size=(t, nh * d)), dtype)
    k = dev(rng.normal(size=(t, nkv * d)), dtype)
    v = dev(rng.normal(size=(t, nkv * d)), dtype)
    cos, sin = O.rope_cos_sin_table(O.rope_inv_freq_default(d), 512, 1.0, "fp16")
    pos = rng.integers(0, 512, t)
    c, s = dev(cos[pos], dtype), dev(sin[pos], dtype)
    slots = torch.from_numpy(rng.permutation(nb * bs)[:t].astype(np.int32)).cuda()
    slots[3] = -1
    q1, k1 = q.clone(), k.clone()
    kc1 = torch.zeros(nb, bs, nkv, d, dtype=dtype, device="cuda")
    vc1 = torch.zeros_like(kc1)
    ops.apply_rotary_pos_emb(q1, k1, c, s, nh, nkv, d)
    ops.reshape_and_cache(k1, v, kc1, vc1, slots)
    q2, k2 = q.clone(), k.clone()
    kc2, vc2 = torch.zeros_like(kc1), torch.zeros_like(kc1)
    ops.rope_and_cache(q2, k2, v, c, s, kc2, vc2, slots, nh)
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2)


# ------------------------------------------------------------------------------------------- paged attention
def _pa_case(rng, dtype, b, nh, nkv, d, bs, lens, max_blocks=None, std=1.0, scale=None):
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype, max_blocks=max_blocks, std=std)
    q = rounded(rng.normal(0, std, (b, nh * d)), dtype)
    scale = scale if scale is not None else 1.0 / np.sqrt(d)
    out = ops.paged_attention(dev(q, dtype), dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32),
                              dev(np.asarray(lens, np.int32), torch.int32), nh, nkv, scale)
    torch.cuda.synchronize()
    ref = O.paged_attention_decode(q, kc, vc, tables, lens, nh, nkv, scale)
    mag = O.paged_attention_decode(q, kc, np.abs(vc), tables, lens, nh, nkv, scale)
    return to_np(out), ref, mag


@pytest.mark.parametrize("case,n_kv", [("1", 2), ("2", 1)])
def test_paged_attention_reference_vectors(golden_dir, case, n_kv):
    """decode_output_{1,2} of the reference's flash-attention unit test, through scatter + attention kernels."""
    z = np.load(os.path.join(golden_dir, "flash_attention.npz"))
    nb, bs = int(z["meta_num_blocks"]), int(z["meta_block_size"])
    nh, hid = int(z["meta_num_heads"]), int(z["meta_hidden_size"])
    d = hid // nh
    dt = torch.bfloat16
    kc = torch.zeros(nb, bs, n_kv, d, dtype=dt, device="cuda")
    vc = torch.zeros_like(kc)
    ops.reshape_and_cache(dev(z[f"in{case}_prefill_key"].reshape(4, -1), dt), dev(z[f"in{case}_prefill_value"].reshape(4, -1), dt),
                          kc, vc, dev(z[f"in{case}_prefill_slot_mapping"].astype(np.int32), torch.int32))
    ops.reshape_and_cache(dev(z[f"in{case}_decoder_key"].reshape(2, -1), dt), dev(z[f"in{case}_decoder_value"].reshape(2, -1), dt),
                          kc, vc, dev(z[f"in{case}_decoder_slot_mapping"].astype(np.int32), torch.int32))
    bt = -np.ones((2, 11), np.int32)
    bt[0, 0], bt[1, 0] = 2, 1
    out = ops.paged_attention(dev(z[f"in{case}_decoder_query"].reshape(2, -1), dt), kc, vc, dev(bt, torch.int32),
                              torch.tensor([3, 3], dtype=torch.int32, device="cuda"), nh, n_kv, 0.25)
    res = O.double_benchmark(to_np(out), z[f"gpu_decode_output_{case}"], z[f"golden_decode_output_{case}"])
    assert res.ok, res.messages


@pytest.mark.parametrize("dtype,b,nh,nkv,d,bs,lo,hi", [
    (torch.float16, 4, 8, 2, 64, 16, 32, 256),        # cfg1 shape
    (torch.bfloat16, 6, 32, 8, 128, 128, 512, 1500),  # cfg2 shape, multi-partition
    (torch.bfloat16, 3, 28, 4, 128, 128, 600, 700),   # n_rep = 7
    (torch.bfloat16, 2, 64, 8, 128, 128, 1000, 2100), # n_rep = 8
    (torch.bfloat16, 2, 40, 2, 64, 32, 100, 900),     # n_rep = 20: two head groups
    (torch.float16, 3, 2, 2, 32, 16, 1, 40),          # MHA, tiny
    (torch.bfloat16, 2, 4, 1, 128, 24, 50, 300),      # block size not a multiple of 16
])
def test_paged_attention_vs_oracle(dtype, b, nh, nkv, d, bs, lo, hi):
    rng = np.random.default_rng(b * 1000 + nh)
    lens = rng.integers(lo, hi + 1, b)
    got, ref, mag = _pa_case(rng, dtype, b, nh, nkv, d, bs, lens)
    assert_within(got, ref, mag, dtype, ulps=1.5, what="paged attention")


@pytest.mark.parametrize("dtype,b,nh,nkv,d,bs,lens,max_blocks", [
    # 17..64 partitions of 256 tokens (the combine kernel's branch for more than 16 partitions)
    (torch.bfloat16, 3, 4, 1, 128, 128, [4097, 9000, 16384], 128),
    (torch.float16, 2, 4, 2, 64, 64, [5000, 12345], 256),
    # capacity above 16384 tokens: 512-token partitions (four tiles per wave)
    (torch.bfloat16, 3, 8, 1, 128, 128, [17000, 20000, 300], 160),
    (torch.float16, 2, 2, 1, 64, 128, [18000, 19999], 157),
    (torch.bfloat16, 2, 8, 2, 128, 128, [32768, 16385], 256),
    # head_dim 32 (half a wave of output columns) with more than 32 partitions, both partition sizes
    (torch.bfloat16, 2, 2, 1, 32, 128, [8193, 12000], 100),
    (torch.float16, 2, 2, 2, 32, 64, [20000, 17000], 320),
])
def test_paged_attention_long_contexts_vs_oracle(dtype, b, nh, nkv, d, bs, lens, max_blocks):
    """Contexts of 4k-32k tokens against the oracle: many partitions per sequence, both partition sizes, every
    branch of the kernel that combines them."""
    rng = np.random.default_rng(sum(lens))
    got, ref, mag = _pa_case(rng, dtype, b, nh, nkv, d, bs, np.asarray(lens), max_blocks=max_blocks)
    assert_within(got, ref, mag, dtype, ulps=1.5, what="paged attention, long contexts")


@pytest.mark.parametrize("dtype,b,nkv,d,bs,max_blocks,part,hi", [
    (torch.bfloat16, 200, 2, 32, 128, 32, 512, 4096),    # 400 (sequence, kv head) pairs x 8 partitions of 512 tokens
    (torch.bfloat16, 64, 2, 32, 128, 136, 1024, 3000),   # capacity 17408: 128 pairs x 17 partitions of 1024, too few of 2048
    (torch.bfloat16, 400, 2, 32, 128, 24, 2048, 3072),   # 800 pairs fill the device by themselves: 2048-token partitions
    (torch.bfloat16, 400, 2, 32, 128, 16, 2048, 2048),   # the same, one partition per sequence: no combine, rows written directly
    (torch.float16, 400, 2, 64, 48, 64, 2048, 3072),     # blocks that 32-token tiles straddle, fp16, head_dim 64
    (torch.bfloat16, 100, 8, 128, 128, 16, 2048, 2048),  # head_dim 128, 8 kv heads, one partition per sequence
])
def test_paged_attention_large_batches_take_larger_partitions(dtype, b, nkv, d, bs, max_blocks, part, hi):
    """Large batches of 16-bit caches run 512-, 1024- or 2048-token partitions (chosen on the batch and the context
    capacity); ragged lengths with empty sequences and lengths on and next to the partition borders."""
    rng = np.random.default_rng(b + part + max_blocks)
    cap = max_blocks * bs
    lens = rng.integers(1, hi + 1, b)
    lens[:8] = [0, 1, part - 1, min(part, cap), min(part + 1, cap), min(2 * part, cap), cap - 1, cap]
    empty = sorted({0, min(63, b - 2), min(64, b - 1), b - 1})   # no context, on both sides of a 64-wide scan chunk
    lens[empty] = 0
    got, ref, mag = _pa_case(rng, dtype, b, 2 * nkv, nkv, d, bs, lens, max_blocks=max_blocks)
    assert not got[empty].any()                               # a sequence without context: zeros
    assert_within(got, ref, mag, dtype, ulps=1.5, what=f"paged attention, {part}-token partitions")


def test_paged_attention_edge_lengths():
    """L = 1 returns the V row; L = 0 returns zeros; L exactly on tile / partition / block boundaries."""
    rng = np.random.default_rng(11)
    dtype = torch.bfloat16
    lens = np.array([1, 0, 16, 32, 33, 512, 513, 1024, 128, 129], dtype=np.int64)
    b, nh, nkv, d, bs = len(lens), 8, 2, 128, 128
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype)
    q = rounded(rng.normal(size=(b, nh * d)), dtype)
    out = to_np(ops.paged_attention(dev(q, dtype), dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32),
                                    dev(lens.astype(np.int32), torch.int32), nh, nkv, 1 / np.sqrt(d)))
    ref = O.paged_attention_decode(q, kc, vc, tables, lens, nh, nkv, 1 / np.sqrt(d))
    mag = O.paged_attention_decode(q, kc, np.abs(vc), tables, lens, nh, nkv, 1 / np.sqrt(d))
    assert_within(out, ref, mag, dtype, ulps=1.5, what="edge lengths")
    assert np.all(out[1] == 0)
    v_row = vc[tables[0, 0], 0]                           # L = 1: softmax over one token is exactly 1
    assert np.array_equal(out[0].reshape(nkv, nh // nkv, d), np.repeat(v_row[:, None, :], nh // nkv, axis=1))
    # single-partition path (max context <= 512) with an empty sequence
    lens2 = np.array([0, 7, 300], dtype=np.int64)
    kc, vc, tables, nb = make_paged_cache(rng, 3, lens2, nkv, d, bs, dtype, max_blocks=4)
    q = rounded(rng.normal(size=(3, nh * d)), dtype)
    out = to_np(ops.paged_attention(dev(q, dtype), dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32),
                                    dev(lens2.astype(np.int32), torch.int32), nh, nkv, 1 / np.sqrt(d)))
    ref = O.paged_attention_decode(q, kc, vc, tables, lens2, nh, nkv, 1 / np.sqrt(d))
    mag = O.paged_attention_decode(q, kc, np.abs(vc), tables, lens2, nh, nkv, 1 / np.sqrt(d))
    assert_within(out, ref, mag, dtype, ulps=1.5, what="single partition")
    assert np.all(out[0] == 0)


@pytest.mark.parametrize("dtype,b,nh,nkv,d,bs,lo,hi,smooth,tiled", [
    (torch.bfloat16, 20, 28, 4, 128, 128, 300, 2048, True, True),    # 2..8 partitions: fused combine + quantisation
    (torch.bfloat16, 5, 32, 8, 128, 128, 1, 200, False, False),      # one partition: attention, then quantisation
    (torch.float16, 3, 8, 2, 64, 16, 100, 4000, True, True),         # 16 partitions
    (torch.bfloat16, 2, 64, 8, 128, 128, 600, 900, True, True),      # row wider than the fused kernel takes
    (torch.bfloat16, 2, 8, 2, 64, 32, 3000, 5000, False, True),      # more than 16 partitions
])
def test_paged_attention_with_quantised_output_equals_two_calls(dtype, b, nh, nkv, d, bs, lo, hi, smooth, tiled):
    """Decode attention that also quantises its output rows per token: out, xq and the scales carry the bits of
    paged_attention followed by dynamic_quant (a sequence with no context included)."""
    rng = np.random.default_rng(b + nh + hi)
    lens = rng.integers(lo, hi + 1, b)
    lens[0] = 0 if lo > 1 else lens[0]
    kc, vc, tables, nb = make_paged_cache(rng, b, np.maximum(lens, 1), nkv, d, bs, dtype, max_blocks=(hi + bs - 1) // bs)
    q = dev(rng.normal(size=(b, nh * d)), dtype)
    sm = torch.from_numpy(rng.uniform(0.5, 2.0, nh * d).astype(np.float32)).cuda() if smooth else None
    args = (q, dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32), nh, nkv,
            1.0 / np.sqrt(d))
    out, xq, xs = ops.paged_attention(*args, quant=(sm, tiled))
    out_ref = ops.paged_attention(*args)
    xq_ref, xs_ref = ops.dynamic_quant(out_ref, sm, tiled=tiled)
    assert torch.equal(out, out_ref) and torch.equal(xs, xs_ref)
    if tiled:
        assert np.array_equal(untile_int8(to_np(xq.data), b, nh * d), untile_int8(to_np(xq_ref.data), b, nh * d))
    else:
        assert torch.equal(xq, xq_ref)


def test_paged_attention_block_permutation_invariant():
    """Moving the physical blocks (and the table with them) must leave the output bit-identical."""
    rng = np.random.default_rng(12)
    dtype = torch.bfloat16
    b, nh, nkv, d, bs = 4, 32, 8, 128, 128
    lens = rng.integers(200, 1400, b)
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype)
    q = dev(rng.normal(size=(b, nh * d)), dtype)
    ld = dev(lens.astype(np.int32), torch.int32)
    out1 = ops.paged_attention(q, dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32), ld, nh, nkv, 0.088)
    perm = rng.permutation(nb)                           # new_id = perm[old_id]
    kc2, vc2 = np.empty_like(kc), np.empty_like(vc)
    kc2[perm], vc2[perm] = kc, vc
    t2 = np.where(tables >= 0, perm[np.maximum(tables, 0)], -1).astype(np.int32)
    out2 = ops.paged_attention(q, dev(kc2, dtype), dev(vc2, dtype), dev(t2, torch.int32), ld, nh, nkv, 0.088)
    torch.cuda.synchronize()
    assert torch.equal(out1, out2)


# ------------------------------------------------------------------------------------------- prefill attention
def _starts(q_lens):
    return np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)


def _prefill_case(rng, dtype, nh, nkv, d, bs, lens, q_lens, max_blocks=None, pad_rows=0):
    b = len(lens)
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype, max_blocks=max_blocks)
    t = int(np.sum(q_lens))
    q = rounded(rng.normal(size=(t + pad_rows, nh * d)), dtype)
    scale = 1.0 / np.sqrt(d)
    out = ops.paged_attention_prefill(dev(q, dtype), dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32),
                                      dev(np.asarray(lens, np.int32), torch.int32), dev(_starts(q_lens), torch.int32),
                                      nh, nkv, scale)
    torch.cuda.synchronize()
    ref = O.paged_attention_prefill(q[:t], kc, vc, tables, lens, q_lens, nh, nkv, scale)
    mag = O.paged_attention_prefill(q[:t], kc, np.abs(vc), tables, lens, q_lens, nh, nkv, scale)
    return to_np(out), ref, mag


@pytest.mark.parametrize("dtype,nh,nkv,d,bs,lens,q_lens", [
    (torch.bfloat16, 32, 8, 128, 128, [40, 300, 17], [40, 300, 17]),        # first prefill, ragged
    (torch.bfloat16, 32, 8, 128, 128, [700, 900, 1300], [64, 1, 37]),       # chunks behind a long context
    (torch.float16, 8, 2, 64, 16, [100, 33, 64, 5], [100, 0, 16, 5]),       # a sequence with no new tokens
    (torch.bfloat16, 28, 4, 128, 128, [260, 130], [9, 130]),                # n_rep = 7: queries straddle column groups
    (torch.bfloat16, 40, 2, 64, 32, [150, 90], [5, 90]),                    # n_rep = 20: a query spans two groups
    (torch.float16, 2, 2, 32, 16, [50, 1], [50, 1]),                        # MHA
    (torch.bfloat16, 4, 1, 128, 24, [200, 77], [31, 77]),                   # block size not a multiple of 32
    (torch.bfloat16, 32, 8, 128, 128, [2100], [3]),                         # few queries, long context: partitions
    (torch.float16, 4, 4, 64, 32, [300], [300]),                            # MHA: 128 queries per workgroup
    (torch.float16, 16, 4, 128, 64, [1500, 33], [1500, 20]),                # many tiles per workgroup, fp16
    (torch.bfloat16, 8, 8, 128, 16, [200], [130]),                          # MHA behind a context, small blocks
    (torch.bfloat16, 4, 4, 192, 32, [200, 77], [130, 77]),                  # 192-wide heads through the cache
    (torch.float16, 4, 2, 192, 16, [90, 300], [90, 5]),                     # and with tiles that straddle blocks
])
def test_paged_prefill_vs_oracle(dtype, nh, nkv, d, bs, lens, q_lens):
    rng = np.random.default_rng(nh * 100 + len(lens))
    got, ref, mag = _prefill_case(rng, dtype, nh, nkv, d, bs, np.asarray(lens), np.asarray(q_lens))
    assert_within(got, ref, mag, dtype, ulps=1.5, what="paged prefill")


def test_paged_prefill_many_short_sequences():
    """More sequences than one wave scans at a time, with empty ones, no new tokens, and one-token contexts."""
    rng = np.random.default_rng(41)
    b = 150
    lens = rng.integers(0, 70, b)
    q_lens = np.minimum(lens, rng.integers(0, 9, b))
    lens[7], q_lens[7] = 300, 300                              # one long prompt among them
    got, ref, mag = _prefill_case(rng, torch.bfloat16, 8, 2, 64, 16, lens, q_lens)
    assert_within(got, ref, mag, torch.bfloat16, ulps=1.5, what="paged prefill, 150 sequences")


def test_paged_prefill_rows_of_no_sequence_are_zero():
    """Rows past q_starts[batch] (padding of a fixed-size launch) come back as zeros, on both the single-partition
    path and the partitioned one; a sequence that claims more queries than context only gets its context's worth."""
    rng = np.random.default_rng(21)
    dtype = torch.bfloat16
    for lens, q_lens, mb in (([70, 20], [30, 20], None), ([1500], [2], None)):
        got, ref, mag = _prefill_case(rng, dtype, 8, 2, 128, 128, np.asarray(lens), np.asarray(q_lens),
                                      max_blocks=mb, pad_rows=5)
        t = int(np.sum(q_lens))
        assert_within(got[:t], ref, mag, dtype, ulps=1.5, what="padded launch")
        assert np.all(got[t:] == 0)
    kc, vc, tables, nb = make_paged_cache(rng, 1, [3], 2, 128, 128, dtype)
    q = rounded(rng.normal(size=(6, 8 * 128)), dtype)
    out = to_np(ops.paged_attention_prefill(dev(q, dtype), dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32),
                                            dev(np.array([3], np.int32), torch.int32),
                                            dev(np.array([0, 6], np.int32), torch.int32), 8, 2, 0.1))
    ref = O.paged_attention_prefill(q[:3], kc, vc, tables, [3], [3], 8, 2, 0.1)
    mag = O.paged_attention_prefill(q[:3], kc, np.abs(vc), tables, [3], [3], 8, 2, 0.1)
    assert_within(out[:3], ref, mag, dtype, ulps=1.5, what="clamped query count")
    assert np.all(out[3:] == 0)


def test_paged_prefill_one_query_per_sequence_is_decode():
    rng = np.random.default_rng(22)
    dtype = torch.bfloat16
    b, nh, nkv, d, bs = 5, 32, 8, 128, 128
    lens = rng.integers(100, 1200, b)
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype)
    q = dev(rng.normal(size=(b, nh * d)), dtype)
    args = (dev(kc, dtype), dev(vc, dtype), dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32))
    dec = to_np(ops.paged_attention(q, *args, nh, nkv, 0.088))
    pre = to_np(ops.paged_attention_prefill(q, *args, dev(_starts(np.ones(b, np.int64)), torch.int32), nh, nkv, 0.088))
    mag = O.paged_attention_decode(to_np(q), kc, np.abs(vc), tables, lens, nh, nkv, 0.088)
    assert_within(pre, dec, mag, dtype, ulps=2.0, what="prefill with one query vs decode")


def test_chunked_prefill_matches_whole_prefill():
    """Scatter and attend chunk by chunk (the cache grows between chunks) against one prefill of the whole prompt."""
    rng = np.random.default_rng(23)
    dtype = torch.bfloat16
    nh, nkv, d, bs = 16, 4, 128, 128
    lens = np.array([300, 190])
    b = len(lens)
    kc0, vc0, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype)
    t = int(lens.sum())
    q = rounded(rng.normal(size=(t, nh * d)), dtype)
    tb, starts = dev(tables, torch.int32), _starts(lens)
    whole = to_np(ops.paged_attention_prefill(dev(q, dtype), dev(kc0, dtype), dev(vc0, dtype), tb,
                                              dev(lens.astype(np.int32), torch.int32), dev(starts, torch.int32),
                                              nh, nkv, 0.09))
    chunk = 128
    got = np.zeros_like(whole)
    done = np.zeros(b, np.int64)
    while (done < lens).any():
        step = np.minimum(chunk, lens - done)
        rows = np.concatenate([np.arange(starts[i] + done[i], starts[i] + done[i] + step[i]) for i in range(b)])
        done = done + step
        out = ops.paged_attention_prefill(dev(q[rows], dtype), dev(kc0, dtype), dev(vc0, dtype), tb,
                                          dev(done.astype(np.int32), torch.int32), dev(_starts(step), torch.int32),
                                          nh, nkv, 0.09)
        got[rows] = to_np(out)
    mag = O.paged_attention_prefill(q, kc0, np.abs(vc0), tables, lens, lens, nh, nkv, 0.09)
    assert_within(got, whole, mag, dtype, ulps=2.0, what="chunked vs whole prefill")


@pytest.mark.parametrize("dtype,nh,nkv,d,q_lens,fused", [
    (torch.bfloat16, 32, 8, 128, [130, 1, 64], True),
    (torch.float16, 8, 2, 64, [33, 200], False),
    (torch.bfloat16, 4, 4, 32, [17], False),
    (torch.bfloat16, 16, 16, 192, [130, 1, 64], False),         # 192-wide heads: the prefill of multi-latent attention
    (torch.float16, 8, 2, 192, [33, 200], True),                # the same width with grouped heads, strided rows
    (torch.bfloat16, 2, 2, 192, [1500], False),                 # few columns: the context is cut into partitions
])
def test_causal_attention_varlen_vs_oracle(dtype, nh, nkv, d, q_lens, fused):
    """Keys and values taken from this step's own packed rows (no cache), optionally as column slices of one fused
    projection output."""
    rng = np.random.default_rng(nh + d)
    t = int(np.sum(q_lens))
    nq, nk = nh * d, nkv * d
    qkv = rounded(rng.normal(size=(t, nq + 2 * nk)), dtype)
    qkv_d = dev(qkv, dtype)
    q, k, v = qkv_d[:, :nq], qkv_d[:, nq:nq + nk], qkv_d[:, nq + nk:]
    if not fused:
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    scale = 1.0 / np.sqrt(d)
    out = to_np(ops.causal_attention_varlen(q, k, v, dev(_starts(q_lens), torch.int32), nh, nkv, scale))
    ref = O.causal_prefill_attention(qkv[:, :nq], qkv[:, nq:nq + nk], qkv[:, nq + nk:], q_lens, nh, nkv, scale)
    mag = O.causal_prefill_attention(qkv[:, :nq], qkv[:, nq:nq + nk], np.abs(qkv[:, nq + nk:]), q_lens, nh, nkv, scale)
    assert_within(out, ref, mag, dtype, ulps=1.5, what="varlen causal attention")


@pytest.mark.parametrize("dtype,nh,nkv,q_lens,strided", [
    (torch.bfloat16, 16, 16, [130, 1, 64], False), (torch.float16, 8, 2, [33, 200], True),
    (torch.bfloat16, 2, 2, [1500], False), (torch.bfloat16, 128, 128, [40, 300], True),
])
def test_causal_attention_with_128_wide_values_under_192_wide_keys(dtype, nh, nkv, q_lens, strided):
    """The prefill of multi-latent attention with the values as they are (128 wide) instead of padded to the key
    width: against the oracle on the same values (its 128 output columns), and bit for bit the first 128 columns of
    every head of the 192-wide call on zero-padded values, whose last 64 columns it never computes."""
    rng = np.random.default_rng(nh + len(q_lens))
    t = int(np.sum(q_lens))
    q = rounded(rng.normal(size=(t, nh * 192)), dtype)
    k = rounded(rng.normal(size=(t, nkv * 192)), dtype)
    v = rounded(rng.normal(size=(t, nkv * 128)), dtype)
    scale = 1.0 / np.sqrt(192)
    starts = dev(_starts(q_lens), torch.int32)
    if strided:                                                   # key and value as column slices of one buffer
        kv_t = dev(np.concatenate((k, v), 1), dtype)
        k_t, v_t = kv_t[:, :nkv * 192], kv_t[:, nkv * 192:]
    else:
        k_t, v_t = dev(k, dtype), dev(v, dtype)
    out = ops.causal_attention_varlen(dev(q, dtype), k_t, v_t, starts, nh, nkv, scale)
    assert out.shape == (t, nh * 128)
    v_pad = np.concatenate((v.reshape(t, nkv, 128), np.zeros((t, nkv, 64), np.float32)), 2).reshape(t, nkv * 192)
    wide = ops.causal_attention_varlen(dev(q, dtype), dev(k, dtype), dev(v_pad, dtype), starts, nh, nkv, scale)
    assert torch.equal(out.reshape(t, nh, 128), wide.reshape(t, nh, 192)[..., :128])
    ref = O.causal_prefill_attention(q, k, v_pad, q_lens, nh, nkv, scale).reshape(t, nh, 192)[..., :128]
    mag = O.causal_prefill_attention(q, k, np.abs(v_pad), q_lens, nh, nkv, scale).reshape(t, nh, 192)[..., :128]
    assert_within(to_np(out).reshape(t, nh, 128), ref, mag, dtype, ulps=1.5, what="192 / 128 causal attention")
    with pytest.raises(ValueError):                               # other widths are not built
        ops.causal_attention_varlen(dev(q, dtype), dev(k, dtype), dev(v[:, : nkv * 64].copy(), dtype), starts, nh, nkv, scale)


@pytest.mark.parametrize("case,n_kv", [("1", 2), ("2", 1)])
def test_prefill_reference_vectors(golden_dir, case, n_kv):
    """prefill_output_{1,2} of the reference's flash-attention unit test, from the packed rows and through the cache."""
    z = np.load(os.path.join(golden_dir, "flash_attention.npz"))
    nb, bs = int(z["meta_num_blocks"]), int(z["meta_block_size"])
    nh, hid = int(z["meta_num_heads"]), int(z["meta_hidden_size"])
    d = hid // nh
    dt = torch.bfloat16
    q = dev(z[f"in{case}_prefill_query"].reshape(4, -1), dt)
    k = dev(z[f"in{case}_prefill_key"].reshape(4, -1), dt)
    v = dev(z[f"in{case}_prefill_value"].reshape(4, -1), dt)
    starts = dev(np.array([0, 2, 4], np.int32), torch.int32)
    out = ops.causal_attention_varlen(q, k, v, starts, nh, n_kv, 0.25)
    res = O.double_benchmark(to_np(out), z[f"gpu_prefill_output_{case}"], z[f"golden_prefill_output_{case}"])
    assert res.ok, res.messages
    kc = torch.zeros(nb, bs, n_kv, d, dtype=dt, device="cuda")
    vc = torch.zeros_like(kc)
    ops.reshape_and_cache(k, v, kc, vc, dev(z[f"in{case}_prefill_slot_mapping"].astype(np.int32), torch.int32))
    bt = -np.ones((2, 11), np.int32)
    bt[0, 0], bt[1, 0] = 2, 1
    out2 = ops.paged_attention_prefill(q, kc, vc, dev(bt, torch.int32), dev(np.array([2, 2], np.int32), torch.int32),
                                       starts, nh, n_kv, 0.25)
    res = O.double_benchmark(to_np(out2), z[f"gpu_prefill_output_{case}"], z[f"golden_prefill_output_{case}"])
    assert res.ok, res.messages


# ------------------------------------------------------------------------------------------- MLA decode
def _mla_case(rng, dtype, lens, nh, bs, max_blocks=None):
    b = len(lens)
    cache, _, tables, nb = make_paged_cache(rng, b, lens, 1, 576, bs, dtype, max_blocks=max_blocks)
    q = rounded(rng.normal(size=(b, nh * 576)), dtype)
    scale = 1.0 / np.sqrt(192)                                  # qk_head_dim + rope of the DeepSeek geometry
    out = ops.mla_paged_attention(dev(q, dtype), dev(cache, dtype), dev(tables, torch.int32),
                                  dev(np.asarray(lens, np.int32), torch.int32), nh, 512, scale)
    torch.cuda.synchronize()
    ref = O.mla_paged_attention_decode(q, cache, tables, lens, nh, 512, scale)
    return to_np(out), ref, _mla_abs(q, cache, tables, lens, nh, scale)


def _mla_abs(q, cache, tables, lens, nh, scale):
    """sum_t p_t |v_t|: the magnitude the rounding of the PV product scales with."""
    return O.mla_paged_attention_decode(q, cache, tables, lens, nh, 512, scale, abs_values=True)


@pytest.mark.parametrize("dtype,nh,bs,lens,max_blocks", [
    (torch.bfloat16, 128, 128, [700, 130, 1500], None),        # two head blocks, partitions
    (torch.bfloat16, 16, 128, [64, 33, 200, 1], 2),            # one head group (TP 8), single partition
    (torch.float16, 64, 32, [95, 400], None),
    (torch.bfloat16, 40, 64, [257, 0, 31, 32], None),          # heads not a multiple of 16, an empty sequence
    (torch.bfloat16, 128, 128, [5000], None),                  # one long sequence: many partitions
    (torch.bfloat16, 200, 32, [300, 600], None),               # two head blocks, the second one partly filled
    (torch.float16, 128, 128, [9000, 40], None),               # 32 partitions at most: the smallest partition grows
])
def test_mla_paged_attention_vs_oracle(dtype, nh, bs, lens, max_blocks):
    rng = np.random.default_rng(nh + len(lens))
    got, ref, mag = _mla_case(rng, dtype, np.asarray(lens), nh, bs, max_blocks)
    assert_within(got, ref, mag, dtype, ulps=1.5, what="MLA paged attention")
    for i, n in enumerate(lens):
        if n == 0:
            assert not got[i].any()


def test_mla_paged_attention_large_batch():
    """More sequences than three quarters of the compute units: the partition rule's floor on free workgroups."""
    rng = np.random.default_rng(77)
    lens = rng.integers(1, 90, 210)
    lens[5] = 700                                              # one sequence that is partitioned
    got, ref, mag = _mla_case(rng, torch.bfloat16, lens, 16, 32)
    assert_within(got, ref, mag, torch.bfloat16, ulps=1.5, what="MLA paged attention, batch 210")


def test_mla_paged_attention_partition_rule_over_several_chunks_of_sequences():
    """More than 64 sequences with contexts long enough that the partition rule counts its smaller candidates over
    two chunks of lengths, and sequences cut into 1 to 8 partitions equal up to one tile."""
    rng = np.random.default_rng(78)
    lens = rng.integers(300, 1500, 100)
    lens[[3, 70]] = [33, 2900]
    got, ref, mag = _mla_case(rng, torch.bfloat16, lens, 16, 32)
    assert_within(got, ref, mag, torch.bfloat16, ulps=1.5, what="MLA paged attention, batch 100, long contexts")


def test_attention_rejects_a_non_positive_scale():
    """Prefill and MLA decode take the maximum over raw scores: the scale must be positive (checked on the host)."""
    rng = np.random.default_rng(3)
    dtype = torch.bfloat16
    cache, _, tables, _ = make_paged_cache(rng, 1, [40], 1, 576, 32, dtype)
    q = dev(rng.normal(size=(1, 16 * 576)), dtype)
    with pytest.raises(Exception, match="scale"):
        ops.mla_paged_attention(q, dev(cache, dtype), dev(tables, torch.int32), dev(np.asarray([40], np.int32), torch.int32),
                                16, 512, -0.1)
    kc, vc, tb, _ = make_paged_cache(rng, 1, [40], 2, 64, 32, dtype)
    qq = dev(rng.normal(size=(40, 4 * 64)), dtype)
    with pytest.raises(Exception, match="scale"):
        ops.paged_attention_prefill(qq, dev(kc, dtype), dev(vc, dtype), dev(tb, torch.int32),
                                    dev(np.asarray([40], np.int32), torch.int32), dev(_starts([40]), torch.int32), 4, 2, 0.0)



def test_mla_cache_is_written_by_key_only_reshape_and_cache():
    """multi_latent_attention.py:401-402: the latent row goes in with reshape_and_cache(key, None, cache, None, slots)."""
    rng = np.random.default_rng(41)
    dtype, nh, bs = torch.bfloat16, 16, 32
    lens = np.array([40, 7])
    cache, _, tables, nb = make_paged_cache(rng, 2, lens, 1, 576, bs, dtype)
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    new = rounded(rng.normal(size=(2, 576)), dtype)
    cd = dev(cache, dtype)
    ops.reshape_and_cache(dev(new, dtype), None, cd, None, dev(slots, torch.int32))
    cache.reshape(-1, 576)[slots] = new
    assert np.array_equal(to_np(cd), cache)
    q = rounded(rng.normal(size=(2, nh * 576)), dtype)
    out = ops.mla_paged_attention(dev(q, dtype), cd, dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32),
                                  nh, 512, 0.07)
    ref = O.mla_paged_attention_decode(q, cache, tables, lens, nh, 512, 0.07)
    assert_within(to_np(out), ref, _mla_abs(q, cache, tables, lens, nh, 0.07), dtype, ulps=1.5, what="MLA after scatter")


# ------------------------------------------------------------------------------------------- int8 KV cache
def _kv8_case(rng, dtype, b, nh, nkv, d, bs, lens, with_offset, max_blocks=None):
    """Random 16-bit caches quantised per channel by the oracle; returns int8 caches, the float caches they stand
    for, tables and the quantisation parameters."""
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype, max_blocks=max_blocks)
    row = nkv * d
    scale = np.stack([np.abs(kc).reshape(-1, row).max(0), np.abs(vc).reshape(-1, row).max(0)]).astype(np.float32) / 100.0
    offset = rng.integers(-20, 21, (2, row)).astype(np.float32) if with_offset else None
    k8 = O.quantize_kv_int8(kc.reshape(-1, row), scale[0], None if offset is None else offset[0]).reshape(kc.shape)
    v8 = O.quantize_kv_int8(vc.reshape(-1, row), scale[1], None if offset is None else offset[1]).reshape(vc.shape)
    kf = O.dequantize_kv_int8(k8.reshape(-1, row), scale[0], None if offset is None else offset[0]).reshape(kc.shape)
    vf = O.dequantize_kv_int8(v8.reshape(-1, row), scale[1], None if offset is None else offset[1]).reshape(vc.shape)
    return k8, v8, kf, vf, tables, nb, scale, offset


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_offset", [False, True])
def test_quant_reshape_and_cache_bit_exact(dtype, with_offset):
    rng = np.random.default_rng(31)
    t, nkv, d, bs, nb = 37, 4, 64, 16, 12
    row = nkv * d
    k = rounded(rng.normal(size=(t, row)), dtype)
    v = rounded(rng.normal(size=(t, row)) * 3, dtype)                 # some values clip
    scale = rng.uniform(0.005, 0.03, (2, row)).astype(np.float32)
    offset = rng.integers(-30, 31, (2, row)).astype(np.float32) if with_offset else None
    slots = rng.permutation(nb * bs)[:t].astype(np.int32)
    slots[5] = -1
    kc = torch.full((nb, bs, nkv, d), 7, dtype=torch.int8, device="cuda")
    vc = torch.full((nb, bs, nkv, d), -9, dtype=torch.int8, device="cuda")
    ops.quant_reshape_and_cache(dev(k, dtype), dev(v, dtype), kc, vc, dev(slots, torch.int32), dev(scale, torch.float32),
                                None if offset is None else dev(offset, torch.float32))
    torch.cuda.synchronize()
    ref_k = np.full((nb * bs, row), 7, np.int8)
    ref_v = np.full((nb * bs, row), -9, np.int8)
    live = slots >= 0
    ref_k[slots[live]] = O.quantize_kv_int8(k, scale[0], None if offset is None else offset[0])[live]
    ref_v[slots[live]] = O.quantize_kv_int8(v, scale[1], None if offset is None else offset[1])[live]
    assert np.array_equal(kc.cpu().numpy().reshape(-1, row), ref_k)
    assert np.array_equal(vc.cpu().numpy().reshape(-1, row), ref_v)
    assert (ref_v == 127).any() or (ref_v == -128).any()


@pytest.mark.parametrize("dtype,b,nh,nkv,d,bs,lo,hi,with_offset", [
    (torch.bfloat16, 5, 32, 8, 128, 128, 300, 1500, False),   # bench shape, several partitions
    (torch.bfloat16, 3, 32, 8, 128, 128, 40, 700, True),
    (torch.float16, 4, 8, 2, 64, 16, 10, 250, True),
    (torch.bfloat16, 2, 28, 4, 128, 128, 500, 600, False),    # n_rep = 7
    (torch.float16, 2, 4, 4, 32, 32, 1, 90, True),            # MHA, head_dim 32
    (torch.bfloat16, 400, 4, 2, 32, 128, 1, 2100, True),      # 800 (sequence, kv head) pairs: 2048-token partitions
])
def test_paged_attention_int8kv_vs_oracle(dtype, b, nh, nkv, d, bs, lo, hi, with_offset):
    """Attention over an int8 cache equals the oracle on the dequantised cache (the only extra rounding is the
    query times key-scale product, rounded to the compute dtype)."""
    rng = np.random.default_rng(b * 100 + nh)
    lens = rng.integers(lo, hi + 1, b)
    k8, v8, kf, vf, tables, nb, scale, offset = _kv8_case(rng, dtype, b, nh, nkv, d, bs, lens, with_offset)
    q = rounded(rng.normal(size=(b, nh * d)), dtype)
    sc = 1.0 / np.sqrt(d)
    out = ops.paged_attention_int8kv(dev(q, dtype), torch.from_numpy(k8).cuda(), torch.from_numpy(v8).cuda(),
                                     dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32),
                                     dev(scale, torch.float32), None if offset is None else dev(offset, torch.float32),
                                     nh, nkv, sc)
    ref = O.paged_attention_decode(q, kf, vf, tables, lens, nh, nkv, sc)
    mag = O.paged_attention_decode(q, kf, np.abs(vf), tables, lens, nh, nkv, sc)
    assert_within(to_np(out), ref, mag, dtype, ulps=3.0, what="paged attention over an int8 cache")


def test_paged_attention_int8kv_empty_sequence_in_a_short_table():
    """A block table of 384 tokens is one partition for an int8 cache: the attention kernel writes the rows itself
    and the row of a sequence without context must still come back as zeros."""
    rng = np.random.default_rng(35)
    dtype, nh, nkv, d, bs = torch.bfloat16, 8, 2, 128, 128
    lens = np.array([0, 300, 384, 7])
    k8, v8, kf, vf, tables, nb, scale, offset = _kv8_case(rng, dtype, 4, nh, nkv, d, bs, np.maximum(lens, 1), True,
                                                          max_blocks=3)
    q = rounded(rng.normal(size=(4, nh * d)), dtype)
    sc = 1.0 / np.sqrt(d)
    out = torch.full((4, nh * d), 7.0, dtype=dtype, device="cuda")
    ops.paged_attention_int8kv(dev(q, dtype), torch.from_numpy(k8).cuda(), torch.from_numpy(v8).cuda(),
                               dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32),
                               dev(scale, torch.float32), dev(offset, torch.float32), nh, nkv, sc, out=out)
    ref = O.paged_attention_decode(q, kf, vf, tables, lens, nh, nkv, sc)
    mag = O.paged_attention_decode(q, kf, np.abs(vf), tables, lens, nh, nkv, sc)
    assert_within(to_np(out), ref, mag, dtype, ulps=3.0, what="int8 cache, one partition")
    assert np.all(to_np(out)[0] == 0)


def test_paged_prefill_int8kv_vs_oracle():
    rng = np.random.default_rng(33)
    dtype, nh, nkv, d, bs = torch.bfloat16, 16, 4, 128, 128
    lens, q_lens = np.array([300, 150, 2100]), np.array([60, 150, 3])
    k8, v8, kf, vf, tables, nb, scale, offset = _kv8_case(rng, dtype, 3, nh, nkv, d, bs, lens, True)
    t = int(q_lens.sum())
    q = rounded(rng.normal(size=(t, nh * d)), dtype)
    sc = 1.0 / np.sqrt(d)
    out = ops.paged_attention_int8kv(dev(q, dtype), torch.from_numpy(k8).cuda(), torch.from_numpy(v8).cuda(),
                                     dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32),
                                     dev(scale, torch.float32), dev(offset, torch.float32), nh, nkv, sc,
                                     q_starts=dev(_starts(q_lens), torch.int32))
    ref = O.paged_attention_prefill(q, kf, vf, tables, lens, q_lens, nh, nkv, sc)
    mag = O.paged_attention_prefill(q, kf, np.abs(vf), tables, lens, q_lens, nh, nkv, sc)
    assert_within(to_np(out), ref, mag, dtype, ulps=3.0, what="prefill over an int8 cache")


def _kv8_token_case(rng, dtype, b, nkv, d, bs, lens, max_blocks=None, poison=True):
    """Random 16-bit caches quantised per token by the oracle: int8 caches, the float caches they stand for, the scale
    caches [blocks, block_size] and the tables.  With ``poison`` the scales of every slot that holds no token of a
    sequence are NaN, so a scale read past a context must not reach a result."""
    kc, vc, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dtype, max_blocks=max_blocks)
    row = nkv * d
    k8, ks = O.quantize_kv_int8_per_token(kc.reshape(-1, row))
    v8, vs = O.quantize_kv_int8_per_token(vc.reshape(-1, row))
    kf = (k8.astype(np.float64) * ks[:, None]).reshape(kc.shape)
    vf = (v8.astype(np.float64) * vs[:, None]).reshape(vc.shape)
    if poison:
        live = np.zeros(nb * bs, bool)
        for i, n in enumerate(lens):
            for j in range(int(n)):
                live[tables[i, j // bs] * bs + j % bs] = True
        ks, vs = np.where(live, ks, np.float32(np.nan)), np.where(live, vs, np.float32(np.nan))
    return (k8.reshape(kc.shape), v8.reshape(vc.shape), kf, vf, ks.reshape(nb, bs).astype(np.float32),
            vs.reshape(nb, bs).astype(np.float32), tables, nb)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dynamic_quant_reshape_and_cache_bit_exact(dtype):
    """Per-token int8 cache write from strided key / value slices: rows and scales of the written slots equal the
    oracle's per-token quantisation bit for bit (a zero row stores scale 0 and zeros); a -1 slot writes nothing and
    every other slot keeps what it held."""
    rng = np.random.default_rng(41)
    t, nh, nkv, d, bs, nb = 37, 8, 2, 128, 16, 5
    row = nkv * d
    qkv = rounded(rng.normal(size=(t, (nh + 2 * nkv) * d)) * 2, dtype)
    qkv[5, nh * d:nh * d + row] = 0                                # a key row of zeros
    slots = rng.permutation(nb * bs)[:t].astype(np.int32)
    slots[11] = -1
    qkv_t = dev(qkv, dtype)
    kc = torch.full((nb, bs, nkv, d), 77, dtype=torch.int8, device="cuda")
    vc = torch.full((nb, bs, nkv, d), -77, dtype=torch.int8, device="cuda")
    ksc = torch.full((nb, bs), 3.0, dtype=torch.float32, device="cuda")
    vsc = torch.full((nb, bs), 5.0, dtype=torch.float32, device="cuda")
    ops.dynamic_quant_reshape_and_cache(qkv_t[:, nh * d:nh * d + row], qkv_t[:, nh * d + row:], kc, vc, ksc, vsc,
                                        torch.from_numpy(slots).cuda())
    k_ref, ks_ref = O.quantize_kv_int8_per_token(qkv[:, nh * d:nh * d + row])
    v_ref, vs_ref = O.quantize_kv_int8_per_token(qkv[:, nh * d + row:])
    want_k, want_v = np.full((nb * bs, row), 77, np.int8), np.full((nb * bs, row), -77, np.int8)
    want_ks, want_vs = np.full(nb * bs, 3.0, np.float32), np.full(nb * bs, 5.0, np.float32)
    for i, sl in enumerate(slots):
        if sl >= 0:
            want_k[sl], want_v[sl], want_ks[sl], want_vs[sl] = k_ref[i], v_ref[i], ks_ref[i], vs_ref[i]
    assert ks_ref[5] == 0 and not k_ref[5].any()
    assert np.array_equal(to_np(kc).reshape(-1, row), want_k) and np.array_equal(to_np(vc).reshape(-1, row), want_v)
    assert np.array_equal(to_np(ksc).reshape(-1), want_ks) and np.array_equal(to_np(vsc).reshape(-1), want_vs)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("b,nh,nkv,d,bs,lo,hi", [(8, 32, 8, 128, 128, 1, 1500), (5, 8, 2, 64, 16, 1, 700),
                                                 (3, 4, 4, 32, 32, 30, 300), (64, 28, 4, 128, 128, 500, 600),
                                                 (2, 16, 2, 128, 20, 1, 90), (400, 4, 2, 32, 128, 1, 2100)])
def test_paged_attention_int8kv_per_token_vs_oracle(dtype, b, nh, nkv, d, bs, lo, hi):
    """Decode over int8 caches with one scale per cached token: against the oracle on the dequantised caches (block
    sizes that hold whole 32-token tiles and block sizes that do not; contexts that end inside a tile; NaN in the
    scale slots of tokens that do not exist)."""
    rng = np.random.default_rng(b * 31 + bs)
    lens = rng.integers(lo, hi + 1, b)
    lens[0] = hi
    k8, v8, kf, vf, ks, vs, tables, nb = _kv8_token_case(rng, dtype, b, nkv, d, bs, lens)
    q = rounded(rng.normal(size=(b, nh * d)), dtype)
    sc = 1.0 / np.sqrt(d)
    out = ops.paged_attention_int8kv(dev(q, dtype), torch.from_numpy(k8).cuda(), torch.from_numpy(v8).cuda(),
                                     dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32), None, None,
                                     nh, nkv, sc, token_scales=(torch.from_numpy(ks).cuda(), torch.from_numpy(vs).cuda()))
    ref = O.paged_attention_decode(q, kf, vf, tables, lens, nh, nkv, sc)
    mag = O.paged_attention_decode(q, kf, np.abs(vf), tables, lens, nh, nkv, sc)
    assert_within(to_np(out), ref, mag, dtype, ulps=3.0, what="paged attention over a per-token int8 cache")


@pytest.mark.parametrize("bs", [128, 16])
def test_paged_prefill_int8kv_per_token_vs_oracle(bs):
    rng = np.random.default_rng(34 + bs)
    dtype, nh, nkv, d = torch.bfloat16, 16, 4, 128
    lens, q_lens = np.array([300, 77, 520]), np.array([40, 77, 1])
    k8, v8, kf, vf, ks, vs, tables, nb = _kv8_token_case(rng, dtype, 3, nkv, d, bs, lens)
    t = int(q_lens.sum())
    q = rounded(rng.normal(size=(t, nh * d)), dtype)
    sc = 1.0 / np.sqrt(d)
    out = ops.paged_attention_int8kv(dev(q, dtype), torch.from_numpy(k8).cuda(), torch.from_numpy(v8).cuda(),
                                     dev(tables, torch.int32), dev(lens.astype(np.int32), torch.int32), None, None,
                                     nh, nkv, sc, q_starts=dev(_starts(q_lens), torch.int32),
                                     token_scales=(torch.from_numpy(ks).cuda(), torch.from_numpy(vs).cuda()))
    ref = O.paged_attention_prefill(q, kf, vf, tables, lens, q_lens, nh, nkv, sc)
    mag = O.paged_attention_prefill(q, kf, np.abs(vf), tables, lens, q_lens, nh, nkv, sc)
    assert_within(to_np(out), ref, mag, dtype, ulps=3.0, what="prefill over a per-token int8 cache")


def test_paged_attention_int8kv_per_token_rejects_bad_operands():
    k8 = torch.zeros(2, 6, 1, 32, dtype=torch.int8, device="cuda")            # block size 6: not a multiple of 4
    sc6 = torch.ones(2, 6, device="cuda")
    q = torch.zeros(1, 32, dtype=torch.bfloat16, device="cuda")
    tables = torch.zeros(1, 2, dtype=torch.int32, device="cuda")
    lens = torch.ones(1, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        ops.paged_attention_int8kv(q, k8, k8, tables, lens, None, None, 1, 1, 1.0, token_scales=(sc6, sc6))
    k8 = torch.zeros(2, 8, 1, 32, dtype=torch.int8, device="cuda")
    with pytest.raises(ValueError):                                           # scale caches of the wrong size
        ops.paged_attention_int8kv(q, k8, k8, tables, lens, None, None, 1, 1, 1.0, token_scales=(sc6, sc6))
    sc8 = torch.ones(2, 8, device="cuda")
    with pytest.raises(ValueError):                                           # both kinds of parameters at once
        ops.paged_attention_int8kv(q, k8, k8, tables, lens, torch.ones(2, 32, device="cuda"), None, 1, 1, 1.0,
                                   token_scales=(sc8, sc8))


# ------------------------------------------------------------------------------------------- norm / activation
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols,gdt", [(64, 4096, torch.float32), (4, 512, torch.float16), (3, 8192, torch.bfloat16), (1, 32, torch.float32)])
def test_rmsnorm(dtype, rows, cols, gdt):
    rng = np.random.default_rng(4)
    x = rounded(rng.normal(size=(rows, cols)), dtype)
    g = rng.normal(1.0, 0.1, cols).astype(np.float32)
    g = g if gdt == torch.float32 else rounded(g, gdt)
    y = ops.rms_norm(dev(x, dtype), dev(g, gdt), 1e-5)
    ref = O.rms_norm(x, g, 1e-5)
    assert_within(to_np(y), ref, np.abs(ref), dtype, ulps=1.0, extra=1e-7, what="rmsnorm")
    res = rounded(rng.normal(size=(rows, cols)), dtype)
    y2, s2 = ops.rms_norm(dev(x, dtype), dev(g, gdt), 1e-5, residual=dev(res, dtype))
    s_ref = rounded(x.astype(np.float64) + res, dtype)
    assert np.array_equal(to_np(s2), s_ref)              # one rounding of an exact fp32 sum: bit-exact
    ref2 = O.rms_norm(s_ref, g, 1e-5)
    assert_within(to_np(y2), ref2, np.abs(ref2), dtype, ulps=1.0, extra=1e-7, what="add+rmsnorm")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,width,start,cols", [(64, 2112, 0, 1536), (5, 2112, 1536, 512), (3, 96, 8, 32)])
def test_rmsnorm_on_a_column_slice_equals_the_dense_norm(dtype, rows, width, start, cols):
    """The norm reads a column slice of a wider matrix where it lies: the bits of the norm of a dense copy."""
    rng = np.random.default_rng(rows + width)
    x = dev(rounded(rng.normal(size=(rows, width)), dtype), dtype)
    g = torch.from_numpy(rng.normal(1.0, 0.1, cols).astype(np.float32)).cuda()
    view = x[:, start:start + cols]
    assert not view.is_contiguous()
    assert torch.equal(ops.rms_norm(view, g, 1e-6), ops.rms_norm(view.contiguous(), g, 1e-6))


def test_rmsnorm_reference_vectors(golden_dir):
    z = np.load(os.path.join(golden_dir, "norm.npz"))
    for name, eps in (("rmsnorm_output1", 1e-5), ("rmsnorm_output2", 0.1)):
        y = ops.rms_norm(dev(z["in_input"], torch.bfloat16), dev(z["in_weight"], torch.bfloat16), eps)
        res = O.double_benchmark(to_np(y), z[f"gpu_{name}"], z[f"golden_{name}"])
        assert res.ok, (name, res.messages)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("interleaved", [False, True])
def test_silu_mul(dtype, interleaved):
    rng = np.random.default_rng(5)
    rows, f = 5, 1376
    gu = rounded(rng.normal(0, 2, (rows, 2 * f)), dtype)
    out = to_np(ops.silu_mul(dev(gu, dtype), interleaved=interleaved))
    g, u = (gu[:, 0::2], gu[:, 1::2]) if interleaved else (gu[:, :f], gu[:, f:])
    act = rounded(O.silu(g), dtype)
    ref = act.astype(np.float64) * u
    # silu itself is evaluated with the fast exponential: allow one extra ulp on the activation
    assert_within(out, ref, np.abs(ref) + EPS[dtype] * np.abs(u) * np.abs(act), dtype, ulps=1.5, extra=1e-7, what="silu_mul")


def test_silu_mul_reference_vectors(golden_dir):
    z = np.load(os.path.join(golden_dir, "activation.npz"))
    gu = np.concatenate([z["in_multiplicand_input"], z["in_multiplier_input"]], axis=1)
    out = ops.silu_mul(dev(gu, torch.bfloat16))
    res = O.double_benchmark(to_np(out), z["gpu_output"], z["golden_output"])
    assert res.ok, res.messages


def test_add_bit_exact():
    rng = np.random.default_rng(6)
    a = rounded(rng.normal(size=(64, 4096)), torch.bfloat16)
    b = rounded(rng.normal(size=(64, 4096)), torch.bfloat16)
    out = ops.add(dev(a, torch.bfloat16), dev(b, torch.bfloat16))
    assert np.array_equal(to_np(out), rounded(a.astype(np.float64) + b, torch.bfloat16))


# ------------------------------------------------------------------------------------------- W8A16
def _w8a16_case(rng, dtype, m, n, k, bias, residual):
    w = rng.normal(0, 0.02, (n, k)).astype(np.float32)
    wq, s = O.quantize_weight_int8(w)
    x = rounded(rng.normal(size=(m, k)), dtype)
    b = rounded(rng.normal(0, 0.1, n), dtype) if bias else None
    r = rounded(rng.normal(size=(m, n)), dtype) if residual else None
    y = ops.w8a16_linear(dev(x, dtype), torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda(),
                         dev(b, dtype) if bias else None, dev(r, dtype) if residual else None)
    v = O.w8a16_linear(x, wq, s, b)
    dot_mag = (np.abs(x).astype(np.float64) @ np.abs(wq).astype(np.float64).T) * s[None, :]
    extra = 2.0 ** -18 * dot_mag + 1e-9                  # fp32 accumulation of exact products
    if residual:
        # y = round(round(v) + r): when v sits on a rounding tie the inner rounding may land one full step
        # (2 eps |v|) away, on top of the outer rounding (eps |ref|)
        vr = rounded(v, dtype).astype(np.float64)
        ref = vr + r
        return to_np(y), ref, np.abs(ref) + 2 * np.abs(vr), extra
    return to_np(y), v, np.abs(v), extra


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k,bias,residual", [
    (64, 6144, 4096, False, False), (64, 4096, 4096, False, True), (4, 704, 512, False, False),
    (4, 512, 1376, True, True), (1, 4096, 4096, False, False), (17, 200, 1024, True, False),
    (65, 130, 2048, False, False), (128, 256, 512, True, True), (33, 64, 64, False, False),
])
def test_w8a16_gemm(dtype, m, n, k, bias, residual):
    rng = np.random.default_rng(m * 7 + n)
    got, ref, mag, extra = _w8a16_case(rng, dtype, m, n, k, bias, residual)
    assert_within(got, ref, mag, dtype, ulps=1.0, extra=extra, what="w8a16")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,f,k,bias,layout", [(64, 14336, 4096, False, "halves"), (4, 688, 512, True, "halves"),
                                               (17, 104, 1024, True, "interleaved"), (64, 96, 4096, False, "halves"),
                                               (130, 40, 192, True, "halves")])
def test_w8a16_gated_gemm_equals_unfused(dtype, m, f, k, bias, layout):
    """Gate/up GEMM fused with SiLU*mul: bit-identical to the GEMM followed by silu_mul, and within tolerance of the
    oracle (narrow shapes take the split-K path, whose reduce kernel applies the same epilogue)."""
    rng = np.random.default_rng(m + f)
    w = rng.normal(0, 0.02, (2 * f, k)).astype(np.float32)
    wq, s = O.quantize_weight_int8(w)
    x = rounded(rng.normal(size=(m, k)), dtype)
    b = rounded(rng.normal(0, 0.1, 2 * f), dtype) if bias else None
    wq_t, s_t, x_t = torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda(), dev(x, dtype)
    b_t = dev(b, dtype) if bias else None
    packed = ops.pack_w8a16_gated(wq_t, s_t, layout)
    fused = ops.w8a16_gated_linear(x_t, packed, ops.interleave_gate_up(b_t, layout) if bias else None)
    gu = ops.w8a16_linear(x_t, wq_t, s_t, b_t)
    unfused = ops.silu_mul(gu, interleaved=(layout == "interleaved"))
    assert torch.equal(fused, unfused)
    gu_ref = rounded(O.w8a16_linear(x, wq, s, b), dtype).astype(np.float64)
    g_ref, u_ref = (gu_ref[:, :f], gu_ref[:, f:]) if layout == "halves" else (gu_ref[:, 0::2], gu_ref[:, 1::2])
    ref = rounded(O.silu(g_ref), dtype).astype(np.float64) * u_ref
    got_gu = to_np(gu).astype(np.float64)
    # compare on the kernel's own projection output so that only the activation arithmetic is in the tolerance
    g_k, u_k = (got_gu[:, :f], got_gu[:, f:]) if layout == "halves" else (got_gu[:, 0::2], got_gu[:, 1::2])
    ref_k = rounded(O.silu(g_k), dtype).astype(np.float64) * u_k
    # silu evaluated in float32 may round to the neighbouring value of T (2 eps |silu| |u|), then the product rounds
    assert_within(to_np(fused), ref_k, np.abs(ref_k), dtype, ulps=3.0, extra=1e-7, what="gated")
    assert ref.shape == ref_k.shape


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k,bias", [(64, 4096, 4096, False), (4, 512, 1376, True), (64, 16384, 512, False),
                                        (130, 1024, 2048, True), (1, 4096, 14336, False)])
def test_w8a16_linear_add_rmsnorm_equals_unfused(dtype, m, n, k, bias):
    """Projection + residual + RMSNorm in one call: bit-identical to the GEMM (with residual) followed by the norm
    kernel, on shapes that split K (fused reduce) and shapes that do not."""
    rng = np.random.default_rng(m + n + k)
    w = rng.normal(0, 0.02, (n, k)).astype(np.float32)
    wq, s = O.quantize_weight_int8(w)
    x = dev(rounded(rng.normal(size=(m, k)), dtype), dtype)
    res = dev(rounded(rng.normal(size=(m, n)), dtype), dtype)
    gamma = torch.from_numpy((1 + 0.1 * rng.normal(size=n)).astype(np.float32)).cuda()
    b = dev(rounded(rng.normal(0, 0.1, n), dtype), dtype) if bias else None
    packed = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda())
    h, y = ops.w8a16_linear_add_rmsnorm(x, packed, res, gamma, 1e-5, bias=b)
    h_ref = ops.w8a16_linear(x, packed, bias=b, residual=res)
    y_ref = ops.rms_norm(h_ref, gamma, 1e-5)
    assert torch.equal(h, h_ref)
    assert torch.equal(y, y_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k,c,bias", [(64, 2112, 7168, 1536, False),    # the DeepSeek-V3 down projection: 8 k-splits
                                          (20, 2112, 512, 1536, True),     # K too short to split: GEMM, then the norm
                                          (7, 640, 1376, 640, True),       # the norm over the whole row, no residual
                                          (130, 1024, 2048, 8, False)])
def test_w8a16_linear_rmsnorm_leading_equals_unfused(dtype, m, n, k, c, bias):
    """Projection + RMSNorm over its leading columns in one call: bit-identical to the GEMM followed by the norm of the
    column slice, on shapes that split K (the split sum and the norm are one kernel) and shapes that do not."""
    rng = np.random.default_rng(m + n + k + c)
    wq, s = O.quantize_weight_int8(rng.normal(0, 0.02, (n, k)).astype(np.float32))
    x = dev(rounded(rng.normal(size=(m, k)), dtype), dtype)
    gamma = torch.from_numpy((1 + 0.1 * rng.normal(size=c)).astype(np.float32)).cuda()
    b = dev(rounded(rng.normal(0, 0.1, n), dtype), dtype) if bias else None
    packed = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda())
    h, y = ops.w8a16_linear_rmsnorm_leading(x, packed, gamma, 1e-6, bias=b)
    h_ref = ops.w8a16_linear(x, packed, bias=b)
    assert torch.equal(h, h_ref)
    assert y.shape == (m, c) and torch.equal(y, ops.rms_norm(h_ref[:, :c].contiguous(), gamma, 1e-6))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,n_head,n_kv,d,k,bias", [(64, 32, 8, 128, 4096, False), (4, 8, 2, 64, 512, True),
                                                     (7, 28, 4, 128, 64, True), (33, 4, 4, 32, 2048, False)])
def test_w8a16_qkv_rope_and_cache_equals_unfused(dtype, t, n_head, n_kv, d, k, bias):
    """QKV projection + RoPE + cache scatter in one call: the rotated query and both caches are bit-identical to the
    GEMM followed by rope_and_cache on its column slices (shapes with and without split K; a padding slot)."""
    rng = np.random.default_rng(t + k)
    n = (n_head + 2 * n_kv) * d
    wq, s = O.quantize_weight_int8(rng.normal(0, 0.02, (n, k)).astype(np.float32))
    x = dev(rounded(rng.normal(size=(t, k)), dtype), dtype)
    b = dev(rounded(rng.normal(0, 0.1, n), dtype), dtype) if bias else None
    packed = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda())
    bs, nb = 16, t + 3
    slots = rng.permutation(nb * bs)[:t].astype(np.int32)
    slots[t // 2] = -1
    slots_t = torch.from_numpy(slots).cuda()
    cos = dev(rounded(np.cos(rng.uniform(0, 6, (t, d))), dtype), dtype)
    sin = dev(rounded(np.sin(rng.uniform(0, 6, (t, d))), dtype), dtype)
    init = dev(rounded(rng.normal(size=(nb, bs, n_kv, d)), dtype), dtype)
    kc1, vc1, kc2, vc2 = init.clone(), init.clone() + 1, init.clone(), init.clone() + 1
    q1 = ops.w8a16_qkv_rope_and_cache(x, packed, cos, sin, kc1, vc1, slots_t, n_head, bias=b)
    qkv = ops.w8a16_linear(x, packed, bias=b)
    nq, nkv = n_head * d, n_kv * d
    q2, _ = ops.rope_and_cache(qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:], cos, sin, kc2, vc2, slots_t, n_head)
    assert torch.equal(q1, qkv[:, :nq])
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,n_head,n_kv,d,k,bias,with_offset", [(64, 32, 8, 128, 4096, False, False),
                                                                 (4, 8, 2, 64, 512, True, True),
                                                                 (7, 28, 4, 128, 64, True, True),
                                                                 (33, 4, 4, 32, 2048, False, False)])
def test_w8a16_qkv_rope_and_quant_cache_equals_unfused(dtype, t, n_head, n_kv, d, k, bias, with_offset):
    """QKV projection + RoPE + quantising scatter into int8 caches in one call: the rotated query and both caches are
    bit-identical to the GEMM, the in-place rotation and quant_reshape_and_cache on its column slices."""
    rng = np.random.default_rng(t + k + 1)
    n = (n_head + 2 * n_kv) * d
    wq, s = O.quantize_weight_int8(rng.normal(0, 0.02, (n, k)).astype(np.float32))
    x = dev(rounded(rng.normal(size=(t, k)), dtype), dtype)
    b = dev(rounded(rng.normal(0, 0.1, n), dtype), dtype) if bias else None
    packed = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda())
    bs, nb = 16, t + 3
    slots = rng.permutation(nb * bs)[:t].astype(np.int32)
    slots[t // 2] = -1
    slots_t = torch.from_numpy(slots).cuda()
    cos = dev(rounded(np.cos(rng.uniform(0, 6, (t, d))), dtype), dtype)
    sin = dev(rounded(np.sin(rng.uniform(0, 6, (t, d))), dtype), dtype)
    row = n_kv * d
    kv_scale = torch.from_numpy(rng.uniform(0.01, 0.03, (2, row)).astype(np.float32)).cuda()
    kv_offset = torch.from_numpy(rng.uniform(-4, 4, (2, row)).astype(np.float32)).cuda() if with_offset else None
    init = torch.from_numpy(rng.integers(-128, 128, (nb, bs, n_kv, d)).astype(np.int8)).cuda()
    kc1, vc1, kc2, vc2 = init.clone(), init.clone(), init.clone(), init.clone()
    q1 = ops.w8a16_qkv_rope_and_cache(x, packed, cos, sin, kc1, vc1, slots_t, n_head, bias=b, kv_scale=kv_scale,
                                      kv_offset=kv_offset)
    qkv = ops.w8a16_linear(x, packed, bias=b)
    nq, nkv = n_head * d, n_kv * d
    q2, k2, v2 = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:]
    ops.apply_rotary_pos_emb(q2, k2, cos, sin, n_head, n_kv, d)
    ops.quant_reshape_and_cache(k2, v2, kc2, vc2, slots_t, kv_scale, kv_offset)
    assert torch.equal(q1, q2)
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    assert not torch.equal(kc1, init)


def test_w8a16_exact_on_integer_grid():
    """Power-of-two scales and small-integer activations make every product and sum exact: the kernel must
    return exactly the integer matmul (catches a dropped k-step, a wrong row/column or a transposed operand)."""
    rng = np.random.default_rng(8)
    m, n, k = 37, 200, 1376
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    s = (2.0 ** rng.integers(-9, -6, n)).astype(np.float32)
    x = rng.integers(-3, 4, (m, k)).astype(np.float32)
    y = ops.w8a16_linear(dev(x, torch.float16), torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda())
    exact = (x.astype(np.int64) @ wq.astype(np.int64).T).astype(np.float64) * s
    assert np.array_equal(to_np(y).astype(np.float64), rounded(exact, torch.float16).astype(np.float64))


@pytest.mark.parametrize("m,n,k", [(37, 200, 1376), (64, 256, 1032), (5, 80, 72)])
def test_w8a16_inf_in_the_last_columns_of_a_row_stays_in_that_row(m, n, k):
    """K is not a multiple of 64, so the last k-step is short and its padding columns carry zero weights.  An Inf
    among the last activations of one row gives that row +-Inf with the sign of the weight it meets (NaN where that
    weight is zero), exactly as the sum over the real K columns does, and leaves every other row exact: no
    activation may reach a padding column (Inf * 0 would turn the whole row into NaN)."""
    rng = np.random.default_rng(k)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    wq[::7, k - 3] = 0
    s = (2.0 ** rng.integers(-9, -6, n)).astype(np.float32)
    x = rng.integers(-3, 4, (m, k)).astype(np.float32)
    bad = m // 2
    xt = dev(x, torch.float16)
    xt[bad, k - 3] = float("inf")
    y = to_np(ops.w8a16_linear(xt, torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda())).astype(np.float64)
    exact = rounded((x.astype(np.int64) @ wq.astype(np.int64).T).astype(np.float64) * s, torch.float16).astype(np.float64)
    keep = np.arange(m) != bad
    assert np.array_equal(y[keep], exact[keep])
    w_hit = wq[:, k - 3].astype(np.float64)
    assert np.isnan(y[bad][w_hit == 0]).all()
    assert np.array_equal(y[bad][w_hit != 0], np.sign(w_hit[w_hit != 0]) * np.inf)


# ------------------------------------------------------------------------------------------- W4A16
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("group", [0, 64, 128])
@pytest.mark.parametrize("m,n,k,bias,residual", [
    (1, 4096, 4096, False, False), (16, 704, 512, True, False), (32, 512, 1408, True, True),
    (64, 6144, 4096, False, True), (65, 132, 2048, False, False), (130, 256, 512, True, True),
    (33, 64, 128, False, False), (4, 3584, 18944, False, False),
])
def test_w4a16_gemm(dtype, group, m, n, k, bias, residual):
    """4-bit weight-only GEMM against the oracle: per-channel and per-group scales, row counts on both sides of every
    tile height, shapes that split K and shapes that do not, from the two-per-byte and the one-per-byte weight forms."""
    rng = np.random.default_rng(m * 7 + n + group)
    w = rng.normal(0, 0.02, (n, k)).astype(np.float32)
    wq, s = O.quantize_weight_int4(w, group)
    x = rounded(rng.normal(size=(m, k)), dtype)
    b = rounded(rng.normal(0, 0.1, n), dtype) if bias else None
    r = rounded(rng.normal(size=(m, n)), dtype) if residual else None
    s_t = torch.from_numpy(s).cuda()
    packed = ops.pack_w4a16(torch.from_numpy(O.pack_qint4x2(wq)).cuda(), s_t, group, qint4x2=True)
    same = ops.pack_w4a16(torch.from_numpy(wq).cuda(), s_t, group)
    assert torch.equal(packed.packed, same.packed)
    y = ops.w4a16_linear(dev(x, dtype), packed, dev(b, dtype) if bias else None, dev(r, dtype) if residual else None)
    v = O.w4a16_linear(x, wq, s, group, b)
    s_full = np.repeat(s.reshape(1, n) if group == 0 else s, (group or k), axis=0)          # [K, N]
    dot_mag = np.abs(x).astype(np.float64) @ (np.abs(wq).astype(np.float64).T * s_full)
    extra = 2.0 ** -18 * dot_mag + 1e-9
    if residual:
        vr = rounded(v, dtype).astype(np.float64)
        ref, mag = vr + r, np.abs(vr + r) + 2 * np.abs(vr)
    else:
        ref, mag = v, np.abs(v)
    assert_within(to_np(y), ref, mag, dtype, ulps=1.0, extra=extra, what=f"w4a16 g{group}")


@pytest.mark.parametrize("group", [0, 64, 128])
@pytest.mark.parametrize("m,n,k", [(37, 200, 1408), (3, 64, 4096), (64, 1024, 256)])
def test_w4a16_exact_on_integer_grid(group, m, n, k):
    """Power-of-two scales (one per channel and group) and small-integer activations make every product and sum exact:
    the kernel must return exactly the per-group integer matmul.  A group's scale applied to its neighbour, a swapped
    nibble or a dropped k-step changes the result."""
    rng = np.random.default_rng(group + k)
    wq = rng.integers(-8, 8, (n, k)).astype(np.int8)
    s = (2.0 ** rng.integers(-9, -5, (n,) if group == 0 else (k // group, n))).astype(np.float32)
    x = rng.integers(-3, 4, (m, k)).astype(np.float32)
    packed = ops.pack_w4a16(torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda(), group)
    y = ops.w4a16_linear(dev(x, torch.float16), packed)
    exact = O.w4a16_linear(x, wq, s, group)
    assert np.array_equal(to_np(y).astype(np.float64), rounded(exact, torch.float16).astype(np.float64))


def test_w4a16_rejects_bad_operands():
    wq = torch.zeros(64, 128, dtype=torch.int8, device="cuda")
    s = torch.ones(64, device="cuda")
    with pytest.raises(ValueError):
        ops.pack_w4a16(wq, s, 32)                                         # group size not built
    with pytest.raises(ValueError):
        ops.pack_w4a16(wq, s, 64)                                         # scale table of the wrong shape
    with pytest.raises(ValueError):
        ops.pack_w4a16(wq[:, :96].contiguous(), s, 0)                     # K not a multiple of 64
    packed = ops.pack_w4a16(wq, s, 0)
    with pytest.raises(ValueError):
        ops.w4a16_linear(torch.zeros(2, 64, dtype=torch.bfloat16, device="cuda"), packed)
    with pytest.raises(ValueError):
        ops.w4a16_linear(torch.zeros(2, 128, dtype=torch.float32, device="cuda"), packed)
    assert ops.w4a16_linear(torch.zeros(0, 128, dtype=torch.bfloat16, device="cuda"), packed).shape == (0, 64)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols", [(1, 4096), (7, 104), (64, 18944), (0, 64)])
def test_scale_columns_bit_exact(dtype, rows, cols):
    """x * s per column: the float32 product rounded to the activation type, bit for bit (on the ~6e-5 of fp16
    elements whose float32 product lands on a rounding tie this differs from rounding the exact product once, so
    the large case also pins which of the two the kernel computes)."""
    rng = np.random.default_rng(rows + cols)
    x = rounded(rng.normal(size=(rows, cols)), dtype)
    s = rng.uniform(0.25, 4.0, cols).astype(np.float32)
    y = ops.scale_columns(dev(x, dtype), torch.from_numpy(s).cuda())
    ref32 = (x.astype(np.float32) * s[None, :]).astype(np.float32)
    assert np.array_equal(to_np(y), rounded(ref32, dtype))


def test_column_parallel_linear_reference_vectors(golden_dir):
    """The reference's linear vectors are for the bf16 cell; they pin the W8A16 path's layout ([out, in] weight,
    bias add): quantise the reference weight, run the kernel, compare with the oracle linear on the dequantised
    weight, and check the result reproduces the reference's bf16 output to quantisation accuracy."""
    z = np.load(os.path.join(golden_dir, "column_parallel_linear.npz"))
    wq, s = O.quantize_weight_int8(z["in_weight"])
    x = rounded(z["in_inputs"], torch.bfloat16)
    b = rounded(z["in_bias"], torch.bfloat16)
    y = ops.w8a16_linear(dev(x, torch.bfloat16), torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda(), dev(b, torch.bfloat16))
    w_deq = wq.astype(np.float64) * s[:, None]
    ref = O.linear(x, w_deq, b)
    assert_within(to_np(y), ref, np.abs(ref), torch.bfloat16, ulps=1.0, extra=1e-7, what="layout")
    # and the dequantised weight reproduces the reference's bf16 result to quantisation accuracy
    assert np.abs(to_np(y) - z["legacy_output_with_bias"]).max() < 2e-4


# ------------------------------------------------------------------------------------------- W8A8
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,smooth", [(256, 3584, True), (5, 512, False), (64, 18944, True), (1, 64, True)])
def test_dynamic_quant_bit_exact(dtype, m, k, smooth):
    rng = np.random.default_rng(9)
    x = rounded(rng.normal(size=(m, k)), dtype)
    if m > 2:
        x[2] = 0                                         # an all-zero token
    sm = rng.uniform(0.5, 2.0, k).astype(np.float32) if smooth else None
    xq, xs = ops.dynamic_quant(dev(x, dtype), torch.from_numpy(sm).cuda() if smooth else None)
    q_ref, s_ref = O.dynamic_quant_per_token(x, sm)
    assert np.array_equal(to_np(xs), s_ref)
    assert np.array_equal(to_np(xq), q_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,smooth,tiled", [(256, 3584, True, True), (5, 512, False, False), (33, 18944, True, True)])
def test_static_quant_per_tensor_bit_exact(dtype, m, k, smooth, tiled):
    """Static per-tensor activation quantisation: int8 values and the per-row copy of the scale equal the oracle's,
    in both output layouts, with values beyond both rails."""
    rng = np.random.default_rng(m + k)
    x = rounded(rng.normal(0, 1.5, (m, k)), dtype)
    sm = rng.uniform(0.5, 2.0, k).astype(np.float32) if smooth else None
    act = np.float32(0.021)
    xq, xs = ops.static_quant(dev(x, dtype), torch.tensor([act], device="cuda"), None if sm is None else dev(sm, torch.float32),
                              tiled=tiled)
    q_ref, s_ref = O.static_quant_per_tensor(x, act, sm)
    assert np.array_equal(to_np(xs), s_ref)
    got = untile_int8(to_np(xq.data), m, k) if tiled else to_np(xq)
    assert np.array_equal(got, q_ref)
    assert (q_ref == 127).any() and (q_ref == -128).any()


@pytest.mark.parametrize("m,n,k", [(256, 4608, 3584), (256, 3584, 3584), (130, 200, 1088), (1, 64, 64), (64, 257, 512),
                                   (256, 18944, 3584), (256, 896, 4736), (300, 96, 208), (65, 80, 16), (33, 130, 2064),
                                   (300, 16500, 208), (130, 16384, 80)])       # the 8-wave 256 x 160 tiles, ragged
def test_w8a8_gemm_int32_bit_exact(m, n, k):
    rng = np.random.default_rng(10)
    dtype = torch.bfloat16
    xq = rng.integers(-128, 128, (m, k)).astype(np.int8)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    xs = rng.uniform(0.01, 0.05, m).astype(np.float32)
    ws = rng.uniform(1e-4, 5e-4, n).astype(np.float32)
    b = rounded(rng.normal(0, 0.5, n), dtype)
    y, acc = ops.w8a8_linear(torch.from_numpy(xq).cuda(), torch.from_numpy(xs).cuda(), torch.from_numpy(wq).cuda(),
                             torch.from_numpy(ws).cuda(), dtype, bias=dev(b, dtype), return_acc=True)
    acc_ref = O.int8_gemm_i32(xq, wq)
    assert np.array_equal(to_np(acc), acc_ref)
    ref = O.w8a8_linear(xq, xs, wq, ws, b)
    assert_within(to_np(y), ref, np.abs(ref) + np.abs(b), dtype, ulps=1.0, extra=1e-6, what="w8a8 dequant")


@pytest.mark.parametrize("m,k", [(256, 3584), (37, 1376), (1, 64), (130, 208)])
def test_dynamic_quant_tiled_layout_bit_exact(m, k):
    """The tiled output holds exactly the row-major result, at the positions the int8 GEMM reads."""
    rng = np.random.default_rng(m + k)
    x = rounded(rng.normal(size=(m, k)) * 3, torch.bfloat16)
    sm = rng.uniform(0.5, 2.0, k).astype(np.float32)
    xt, xs = ops.dynamic_quant(dev(x, torch.bfloat16), torch.from_numpy(sm).cuda(), tiled=True)
    q_ref, s_ref = O.dynamic_quant_per_token(x, sm)
    assert np.array_equal(to_np(xs), s_ref)
    assert np.array_equal(untile_int8(to_np(xt.data), m, k), q_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("counts,k", [([5, 0, 17, 1, 0, 40], 256), ([0, 0, 3], 7168), ([64] * 16, 2048), ([1], 64)])
def test_grouped_dynamic_quant_bit_exact(dtype, tiled, counts, k):
    """Rows grouped by expert, one multiplier vector per expert (empty experts, a single expert, an empty leading
    run): every row is quantised exactly as the ungrouped call with its expert's vector quantises it, and the fused
    SiLU * up form equals silu_mul followed by the grouped call."""
    rng = np.random.default_rng(len(counts) + k)
    e, m = len(counts), int(sum(counts))
    offsets = np.concatenate(([0], np.cumsum(counts))).astype(np.int32)
    x = rounded(rng.normal(size=(m, k)) * 3, dtype)
    sm = rng.uniform(0.5, 2.0, (e, k)).astype(np.float32)
    sm_t, off_t = torch.from_numpy(sm).cuda(), torch.from_numpy(offsets).cuda()
    xq, xs = ops.dynamic_quant(dev(x, dtype), sm_t, tiled=tiled, offsets=off_t)
    got = untile_int8(to_np(xq.data), m, k) if tiled else to_np(xq)
    for i in range(e):
        a, b = offsets[i], offsets[i + 1]
        q_ref, s_ref = O.dynamic_quant_per_token(x[a:b], sm[i])
        assert np.array_equal(got[a:b], q_ref) and np.array_equal(to_np(xs)[a:b], s_ref), f"expert {i}"
    gu = dev(rounded(rng.normal(size=(m, 2 * k)), dtype), dtype)
    fq, fs = ops.silu_mul_dynamic_quant(gu, sm_t, tiled=tiled, offsets=off_t)
    uq, us = ops.dynamic_quant(ops.silu_mul(gu), sm_t, tiled=tiled, offsets=off_t)
    if tiled:                                                     # padding bytes of the tile order are left unwritten
        assert np.array_equal(untile_int8(to_np(fq.data), m, k), untile_int8(to_np(uq.data), m, k))
    else:
        assert torch.equal(fq, uq)
    assert torch.equal(fs, us)
    with pytest.raises(ValueError):
        ops.dynamic_quant(dev(x, dtype), sm_t[0], offsets=off_t)          # one vector where a table is needed


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,smooth,residual,tiled", [(256, 3584, True, False, True), (5, 512, False, True, False),
                                                       (33, 16384, True, True, True), (1, 64, True, False, False)])
def test_rms_norm_dynamic_quant_equals_unfused(dtype, m, k, smooth, residual, tiled):
    """RMSNorm + per-token quantisation in one kernel: bit-identical to the two kernels in sequence."""
    rng = np.random.default_rng(m + k)
    x = dev(rounded(rng.normal(size=(m, k)), dtype), dtype)
    r = dev(rounded(rng.normal(size=(m, k)), dtype), dtype) if residual else None
    g = torch.from_numpy(rng.uniform(0.5, 1.5, k).astype(np.float32)).cuda()
    sm = torch.from_numpy(rng.uniform(0.5, 2.0, k).astype(np.float32)).cuda() if smooth else None
    if residual:
        n, h = ops.rms_norm(x, g, 1e-6, residual=r)
        fq, fs, fh = ops.rms_norm_dynamic_quant(x, g, 1e-6, sm, residual=r, tiled=tiled)
        assert torch.equal(fh, h)
    else:
        n = ops.rms_norm(x, g, 1e-6)
        fq, fs = ops.rms_norm_dynamic_quant(x, g, 1e-6, sm, tiled=tiled)
    uq, us = ops.dynamic_quant(n, sm, tiled=tiled)
    torch.cuda.synchronize()
    assert torch.equal(fs, us)
    if tiled:
        assert np.array_equal(untile_int8(to_np(fq.data), m, k), untile_int8(to_np(uq.data), m, k))
    else:
        assert torch.equal(fq, uq)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,f,smooth,interleaved,tiled", [(256, 18944, True, False, True), (7, 688, False, True, False),
                                                          (64, 24576, True, True, True), (1, 64, False, False, False)])
def test_silu_mul_dynamic_quant_equals_unfused(dtype, m, f, smooth, interleaved, tiled):
    """SiLU(gate) * up + per-token quantisation in one kernel: bit-identical to the two kernels in sequence."""
    rng = np.random.default_rng(m + f)
    gu = dev(rounded(rng.normal(size=(m, 2 * f)) * 2, dtype), dtype)
    sm = torch.from_numpy(rng.uniform(0.5, 2.0, f).astype(np.float32)).cuda() if smooth else None
    uq, us = ops.dynamic_quant(ops.silu_mul(gu, interleaved=interleaved), sm, tiled=tiled)
    fq, fs = ops.silu_mul_dynamic_quant(gu, sm, interleaved=interleaved, tiled=tiled)
    torch.cuda.synchronize()
    assert torch.equal(fs, us)
    if tiled:
        assert np.array_equal(untile_int8(to_np(fq.data), m, f), untile_int8(to_np(uq.data), m, f))
    else:
        assert torch.equal(fq, uq)


@pytest.mark.parametrize("m,n,k", [(256, 4608, 3584), (256, 18944, 3584), (256, 896, 4736), (300, 96, 208), (65, 80, 16),
                                   (33, 130, 2064), (1, 64, 64), (300, 16500, 208), (130, 16384, 80)])
def test_w8a8_tiled_activations_bit_exact(m, n, k):
    """dynamic_quant(tiled) -> w8a8 GEMM: int32 accumulators equal the integer matmul of the oracle's quantisation."""
    rng = np.random.default_rng(3 * m + n)
    dtype = torch.bfloat16
    x = rounded(rng.normal(size=(m, k)), dtype)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    ws = rng.uniform(1e-4, 5e-4, n).astype(np.float32)
    xt, xs = ops.dynamic_quant(dev(x, dtype), None, tiled=True)
    y, acc = ops.w8a8_linear(xt, xs, torch.from_numpy(wq).cuda(), torch.from_numpy(ws).cuda(), dtype, return_acc=True)
    q_ref, s_ref = O.dynamic_quant_per_token(x, None)
    assert np.array_equal(to_np(acc), O.int8_gemm_i32(q_ref, wq))
    ref = O.w8a8_linear(q_ref, s_ref, wq, ws, None)
    assert_within(to_np(y), ref, np.abs(ref), dtype, ulps=1.0, extra=1e-6, what="w8a8 tiled")


# ------------------------------------------------------------------------------------------- MoE
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k,bias,smooth,residual,tiled", [
    (256, 3584, 3584, False, True, True, True), (256, 3584, 18944, False, True, True, True),
    (4, 512, 1376 // 16 * 16, True, False, True, False), (130, 1024, 2048, True, True, False, True),
    (1, 4096, 64, False, False, True, True), (300, 16384, 208, False, True, True, True),
])
def test_w8a8_linear_add_rmsnorm_quant_equals_unfused(dtype, m, n, k, bias, smooth, residual, tiled):
    """Projection + residual + RMSNorm + per-token quantisation in one call: hidden state, quantised norm output and
    its scales bit-identical to the GEMM (with residual) followed by the fused norm + quantisation kernel, on shapes
    that split K (the fused reduce) and shapes that do not."""
    rng = np.random.default_rng(m + n + k)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    ws = rng.uniform(1e-4, 5e-4, n).astype(np.float32)
    x = dev(rounded(rng.normal(size=(m, k)), dtype), dtype)
    xq, xs = ops.dynamic_quant(x, tiled=tiled)
    res = dev(rounded(rng.normal(size=(m, n)), dtype), dtype)
    gamma = torch.from_numpy((1 + 0.1 * rng.normal(size=n)).astype(np.float32)).cuda()
    sm = torch.from_numpy(rng.uniform(0.5, 2.0, n).astype(np.float32)).cuda() if smooth else None
    b = dev(rounded(rng.normal(0, 0.1, n), dtype), dtype) if bias else None
    packed = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(ws).cuda())
    r = res if residual else torch.zeros_like(res)
    h, nq, ns = ops.w8a8_linear_add_rmsnorm_quant(xq, xs, packed, r, gamma, 1e-5, sm, bias=b, tiled_out=tiled)
    h_ref = ops.w8a8_linear(xq, xs, packed, out_dtype=dtype, bias=b, residual=r)
    nq_ref, ns_ref = ops.rms_norm_dynamic_quant(h_ref, gamma, 1e-5, sm, tiled=tiled)
    assert torch.equal(h, h_ref)
    assert torch.equal(ns, ns_ref)
    if tiled:                                                # rows past m in the last 16-row tile are never written
        assert np.array_equal(untile_int8(to_np(nq.data), m, n), untile_int8(to_np(nq_ref.data), m, n))
    else:
        assert torch.equal(nq, nq_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,n_head,n_kv,d,k,bias,tiled", [(256, 28, 4, 128, 3584, True, True), (4, 8, 2, 64, 512, True, False),
                                                           (7, 28, 4, 128, 64, False, True), (130, 4, 4, 32, 2048, False, True)])
def test_w8a8_qkv_rope_and_cache_equals_unfused(dtype, t, n_head, n_kv, d, k, bias, tiled):
    """W8A8 QKV projection + RoPE + cache scatter in one call: the rotated query and both caches are bit-identical to
    the GEMM followed by rope_and_cache on its column slices (shapes with and without split K; a padding slot)."""
    rng = np.random.default_rng(t + k)
    n = (n_head + 2 * n_kv) * d
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    ws = rng.uniform(1e-4, 5e-4, n).astype(np.float32)
    x = dev(rounded(rng.normal(size=(t, k)), dtype), dtype)
    xq, xs = ops.dynamic_quant(x, tiled=tiled)
    b = dev(rounded(rng.normal(0, 0.1, n), dtype), dtype) if bias else None
    packed = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(ws).cuda())
    bs, nb = 16, t + 3
    slots = rng.permutation(nb * bs)[:t].astype(np.int32)
    slots[t // 2] = -1
    slots_t = torch.from_numpy(slots).cuda()
    cos = dev(rounded(np.cos(rng.uniform(0, 6, (t, d))), dtype), dtype)
    sin = dev(rounded(np.sin(rng.uniform(0, 6, (t, d))), dtype), dtype)
    init = dev(rounded(rng.normal(size=(nb, bs, n_kv, d)), dtype), dtype)
    kc1, vc1, kc2, vc2 = init.clone(), init.clone() + 1, init.clone(), init.clone() + 1
    q1 = ops.w8a8_qkv_rope_and_cache(xq, xs, packed, cos, sin, kc1, vc1, slots_t, n_head, bias=b)
    qkv = ops.w8a8_linear(xq, xs, packed, out_dtype=dtype, bias=b)
    nq, nkv = n_head * d, n_kv * d
    ops.rope_and_cache(qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:], cos, sin, kc2, vc2, slots_t, n_head)
    assert torch.equal(q1, qkv[:, :nq])
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,e,h,wdt", [(64, 256, 7168, "fp32"), (1, 256, 7168, "fp32"), (200, 64, 2048, "fp32"),
                                       (7, 20, 260, "fp32"), (64, 256, 7168, "same"), (33, 8, 64, "same")])
def test_router_gate_projection(dtype, t, e, h, wdt):
    """The router's dense projection with fp32 accumulation: against the float64 product (an fp32 sum of h terms,
    whatever its order, is within h * 2^-24 of sum |terms|); with small integers everywhere the result is exact, which
    catches a dropped or doubled column at the slice and chunk borders (h = 260 ends inside a chunk); a 16-bit weight
    gives logits that are values of that type."""
    rng = np.random.default_rng(t + e + h)
    x = rounded(rng.normal(size=(t, h)), dtype)
    w = rng.normal(0, 0.02, (e, h)).astype(np.float32)
    if wdt == "same":
        w = rounded(w, dtype)
    w_t = torch.from_numpy(w).cuda() if wdt == "fp32" else dev(w, dtype)
    got = to_np(ops.router_gate(dev(x, dtype), w_t))
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    mag = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T
    if wdt == "same":
        assert np.array_equal(got, rounded(got, dtype))
        assert_within(got, ref, np.abs(ref), dtype, ulps=1.0, extra=h * 2.0 ** -24 * mag, what="router gate (16-bit)")
    else:
        assert np.all(np.abs(got - ref) <= h * 2.0 ** -24 * mag + 1e-12)
    xi = rng.integers(-3, 4, (t, h)).astype(np.float32)
    wi = rng.integers(-4, 5, (e, h)).astype(np.float32)
    wi_t = torch.from_numpy(wi).cuda() if wdt == "fp32" else dev(wi, dtype)
    exact = xi.astype(np.int64) @ wi.astype(np.int64).T
    got_i = to_np(ops.router_gate(dev(xi, dtype), wi_t)).astype(np.float64)
    want = exact.astype(np.float64) if wdt == "fp32" else rounded(exact, dtype).astype(np.float64)
    assert np.array_equal(got_i, want)


@pytest.mark.parametrize("t,e,k,ng,tg", [(128, 256, 8, 8, 4), (16, 8, 2, 2, 2), (33, 64, 6, 8, 3), (5, 16, 4, 1, 1), (7, 96, 3, 4, 1),
                                         (9, 96, 4, 3, 2), (6, 60, 5, 6, 2), (4, 1024, 32, 16, 8), (3, 640, 7, 64, 9)])
def test_moe_route(t, e, k, ng, tg):
    rng = np.random.default_rng(13)
    logits = rng.normal(size=(t, e)).astype(np.float32)
    bias = rng.normal(0, 0.1, e).astype(np.float32)
    w, idx = ops.moe_route(torch.from_numpy(logits).cuda(), torch.from_numpy(bias).cuda(), k, ng, tg, 2.5, torch.bfloat16)
    w_ref, idx_ref = O.topk_router(logits, bias, k, ng, tg, 2.5)
    assert np.array_equal(to_np(idx), idx_ref)
    assert_within(to_np(w), w_ref, np.abs(w_ref), torch.bfloat16, ulps=1.0, what="router weights")


def test_moe_route_ties_go_to_the_lower_index():
    """Equal scores (constant logits, and a row of two distinct values): experts and groups are taken in index order."""
    e, k, ng, tg = 64, 6, 8, 3
    logits = np.zeros((3, e), np.float32)
    logits[1, 40:] = 1.0
    logits[2, ::2] = 0.5
    bias = np.zeros(e, np.float32)
    w, idx = ops.moe_route(torch.from_numpy(logits).cuda(), torch.from_numpy(bias).cuda(), k, ng, tg, 1.0, torch.bfloat16)
    w_ref, idx_ref = O.topk_router(logits, bias, k, ng, tg, 1.0)
    assert np.array_equal(to_np(idx), idx_ref)
    assert_within(to_np(w), w_ref, np.abs(w_ref), torch.bfloat16, ulps=1.0, what="router weights")


@pytest.mark.parametrize("t,h,e,k", [(5, 64, 300, 1), (130, 7168, 256, 8), (3, 8, 4, 4), (70, 1032, 17, 9)])
def test_moe_permute_unpermute_shapes(t, h, e, k):
    """Permute / weighted unpermute at the edges: one choice per token, more experts than lanes of a scan chunk, the
    full DeepSeek-V3 width, a width that is not a multiple of the column chunk, more than one batch of choices."""
    rng = np.random.default_rng(t + h + e + k)
    dtype = torch.bfloat16
    x = rounded(rng.normal(size=(t, h)), dtype)
    idx = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
    probs = rounded(rng.uniform(0.1, 1.0, (t, k)), dtype)
    shared = rounded(rng.normal(size=(t, h)), dtype)
    px, row_map, counts, offsets = ops.moe_permute(dev(x, dtype), torch.from_numpy(idx).cuda(), e)
    px_ref, map_ref, cnt_ref = O.moe_permute(x, idx, e)
    assert np.array_equal(to_np(row_map), map_ref) and np.array_equal(to_np(counts), cnt_ref)
    assert np.array_equal(to_np(offsets), np.concatenate(([0], np.cumsum(cnt_ref))).astype(np.int32))
    assert np.array_equal(to_np(px), px_ref)
    y = rounded(rng.normal(size=(t * k, h)), dtype)
    for sh in (None, shared):
        out = ops.moe_unpermute(dev(y, dtype), row_map, dev(probs, dtype), shared=None if sh is None else dev(sh, dtype))
        ref = O.moe_unpermute(y, map_ref, probs)
        mag = O.moe_unpermute(np.abs(y), map_ref, probs)
        if sh is not None:                       # the routed sum is rounded to the activation dtype before the add
            ref, mag = rounded(ref, dtype) + sh, mag + np.abs(sh)
        assert_within(to_np(out), ref, mag, dtype, ulps=1.0, extra=2.0 ** -9 * EPS[dtype] * mag + 1e-9, what="unpermute")


def test_moe_permute_grouped_unpermute():
    rng = np.random.default_rng(14)
    dtype = torch.bfloat16
    t, h, e, k, f = 40, 256, 16, 4, 128
    x = rounded(rng.normal(size=(t, h)), dtype)
    idx = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
    idx[:, 0] = np.minimum(idx[:, 0], 5)                 # leave some experts empty, some crowded (> 16 rows)
    px, row_map, counts, offsets = ops.moe_permute(dev(x, dtype), torch.from_numpy(idx).cuda(), e)
    px_ref, map_ref, cnt_ref = O.moe_permute(x, idx, e)
    assert np.array_equal(to_np(row_map), map_ref) and np.array_equal(to_np(counts), cnt_ref)
    assert np.array_equal(to_np(offsets), np.concatenate(([0], np.cumsum(cnt_ref))).astype(np.int32))
    assert np.array_equal(to_np(px), px_ref)

    w1 = rng.normal(0, 0.05, (e, 2 * f, h)).astype(np.float32)       # [E, N, K]
    q1, s1 = zip(*(O.quantize_weight_int8(w1[i]) for i in range(e)))
    q1, s1 = np.stack(q1), np.stack(s1)
    y1 = ops.grouped_w8a16_linear(px, torch.from_numpy(q1).cuda(), offsets, scale=torch.from_numpy(s1).cuda())
    deq1 = q1.astype(np.float64) * s1[..., None]                      # [E, N, K] -> oracle wants [E, in, out]
    ref1 = O.grouped_matmul(px_ref, np.transpose(deq1, (0, 2, 1)), cnt_ref)
    mag1 = O.grouped_matmul(np.abs(px_ref), np.abs(np.transpose(deq1, (0, 2, 1))), cnt_ref)
    assert_within(to_np(y1), ref1, np.abs(ref1), dtype, ulps=1.0, extra=2.0 ** -18 * mag1 + 1e-9, what="grouped gemm")

    probs = rounded(rng.uniform(0.1, 1.0, (t, k)), dtype)
    yy = rounded(rng.normal(size=(t * k, h)), dtype)
    sh = rounded(rng.normal(size=(t, h)), dtype)
    out = ops.moe_unpermute(dev(yy, dtype), row_map, dev(probs, dtype), shared=dev(sh, dtype))
    routed = O.moe_unpermute(yy, map_ref, probs)
    ref = rounded(routed, dtype).astype(np.float64) + sh
    mag = np.abs(ref) + np.abs(rounded(routed, dtype))
    assert_within(to_np(out), ref, mag, dtype, ulps=1.5, extra=1e-6, what="unpermute")


# ------------------------------------------------------------------------------------------- grouped GEMMs, more
def _ragged_groups(rng, counts):
    counts = np.asarray(counts, np.int64)
    return counts, np.concatenate(([0], np.cumsum(counts))).astype(np.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_grouped_w8a16_many_rows_and_gated_epilogue(dtype):
    """Experts with 0, 1, 16, 17, 33 and 70 rows (one, two and four row tiles per pass over the weights, and a
    repeated pass) against the oracle; the gated form (gate / up rows interleaved at pack time, silu(gate) * up in the
    epilogue) carries the bits of the plain grouped GEMM followed by silu_mul; K is not a multiple of 64."""
    rng = np.random.default_rng(23)
    counts, off = _ragged_groups(rng, [0, 1, 16, 17, 33, 70, 0, 5])
    e, f, k = len(counts), 96, 328
    rows = int(counts.sum())
    x = rounded(rng.normal(size=(rows, k)), dtype)
    w = rng.normal(0, 0.05, (e, 2 * f, k)).astype(np.float32)
    q, s = zip(*(O.quantize_weight_int8(w[i]) for i in range(e)))
    q, s = np.stack(q), np.stack(s)
    qd, sd, od = torch.from_numpy(q).cuda(), torch.from_numpy(s).cuda(), torch.from_numpy(off).cuda()
    y = ops.grouped_w8a16_linear(dev(x, dtype), ops.pack_w8a16(qd, sd), od)
    deq = np.transpose(q.astype(np.float64) * s[..., None], (0, 2, 1))
    ref = O.grouped_matmul(x, deq, counts)
    mag = O.grouped_matmul(np.abs(x), np.abs(deq), counts)
    assert_within(to_np(y), ref, np.abs(ref), dtype, ulps=1.0, extra=2.0 ** -18 * mag + 1e-9, what="grouped gemm, many rows")
    fused = ops.grouped_w8a16_linear(dev(x, dtype), ops.pack_w8a16_gated(qd, sd, "halves"), od)
    assert fused.shape == (rows, f) and torch.equal(fused, ops.silu_mul(y))


@pytest.mark.parametrize("counts,n,k", [([0, 5, 16, 20, 40, 1, 0, 3], 192, 208), ([4] * 16, 128, 1024), ([33], 80, 64),
                                        ([64, 65, 150, 32, 0, 129, 7], 144, 320)])
def test_grouped_w8a8_accumulators_bit_exact(counts, n, k):
    """The grouped int8 GEMM: exact int32 accumulators per expert (against the integer matmul), dequantised outputs
    within a rounding of acc * row scale * channel scale; ragged groups, empty experts, every pass size (16, 32 and
    64 rows), more than 64 rows (a repeated pass, whole and ragged), K not a multiple of 64, N not a multiple of 64."""
    rng = np.random.default_rng(n + k)
    counts, off = _ragged_groups(rng, counts)
    e, rows = len(counts), int(counts.sum())
    x = rounded(rng.normal(size=(rows, k)), torch.bfloat16)
    xq, xs = ops.dynamic_quant(dev(x, torch.bfloat16))
    wq = rng.integers(-127, 128, (e, n, k)).astype(np.int8)
    ws = rng.uniform(1e-4, 5e-4, (e, n)).astype(np.float32)
    w = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(ws).cuda())
    y, acc = ops.grouped_w8a8_linear(xq, xs, w, torch.from_numpy(off).cuda(), return_acc=True)
    xq_n, xs_n = to_np(xq), to_np(xs).astype(np.float64)
    got_acc, got_y = to_np(acc), to_np(y)
    for ex in range(e):
        r0, r1 = int(off[ex]), int(off[ex + 1])
        if r1 == r0:
            continue
        ref = O.int8_gemm_i32(xq_n[r0:r1], wq[ex])
        assert np.array_equal(got_acc[r0:r1], ref), ex
        yref = ref.astype(np.float64) * xs_n[r0:r1, None] * ws[ex].astype(np.float64)[None, :]
        assert np.all(np.abs(got_y[r0:r1] - yref) <= 1.01 * EPS[torch.bfloat16] * np.abs(yref) + 1e-6), ex


# ------------------------------------------------------------------------------------------- MLA absorbed projections
@pytest.mark.parametrize("dtype,t,h,k,n,strided", [
    (torch.bfloat16, 64, 128, 128, 512, True),     # query side at DeepSeek-V3 geometry: q_no_pe inside [T, H, 192]
    (torch.bfloat16, 64, 128, 512, 128, False),    # output side
    (torch.float16, 5, 3, 512, 128, False),
    (torch.bfloat16, 33, 16, 64, 48, True),        # ragged token tile, channel count not a multiple of 64
    (torch.float16, 257, 2, 256, 16, False),       # few heads: the tokens are cut over workgroups
    (torch.bfloat16, 1, 128, 128, 512, True),
])
def test_mla_absorb_bmm_vs_oracle(dtype, t, h, k, n, strided):
    """out[t, h, :] = x[t, h, :] . w[h]^T against float64, x and out as strided slices of wider buffers (the query
    projection [T, H, k + 64] and the attention query [T, H, n + 64]); the columns beside the output slice stay."""
    rng = np.random.default_rng(t * 131 + n)
    pad = 64 if strided else 0
    xw = rounded(rng.normal(size=(t, h, k + pad)), dtype)
    w = rounded(rng.normal(0, 0.1, (h, n, k)), dtype)
    xd = dev(xw, dtype)
    out_w = torch.full((t, h, n + pad), 7.0, dtype=dtype, device="cuda")
    got = ops.mla_absorb_bmm(xd[..., :k], dev(w, dtype), out=out_w[..., :n])
    x64, w64 = xw[..., :k].astype(np.float64), w.astype(np.float64)
    ref = np.einsum("thk,hnk->thn", x64, w64)
    mag = np.einsum("thk,hnk->thn", np.abs(x64), np.abs(w64))
    assert_within(to_np(got), ref, np.abs(ref), dtype, ulps=1.0, extra=2.0 ** -18 * mag + 1e-9, what="absorb bmm")
    if pad:
        assert bool((out_w[..., n:] == 7.0).all())
    fresh = ops.mla_absorb_bmm(xd[..., :k], dev(w, dtype))
    assert fresh.is_contiguous() and torch.equal(fresh, out_w[..., :n])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,n,nope,rope,rank,q_lora,decode", [(64, 128, 128, 64, 512, 1536, True), (37, 16, 128, 64, 512, 0, False),
                                                             (5, 3, 32, 16, 64, 8, True), (1, 128, 128, 64, 512, 1536, False)])
def test_mla_norm_rope_cache_equals_the_separate_ops(dtype, t, n, nope, rope, rank, q_lora, decode):
    """kv_layernorm + RoPE of the rotary query / key parts + latent-row scatter in one launch: the rotations are the
    bits of apply_rotary_pos_emb, the normalised latent rows are within a rounding of rms_norm (the sum of squares is
    taken in another order) and equal the oracle's norm to that bound; the cache rows of live slots hold [norm, rotated
    key part], a -1 slot writes nothing, and the query part lands where it is asked for (in place, or behind the
    absorbed query)."""
    rng = np.random.default_rng(t + n + rope)
    bs, nb = 16, (t + 15) // 16 + 2
    q = rounded(rng.normal(size=(t, n, nope + rope)), dtype)
    qkv = rounded(rng.normal(size=(t, q_lora + rank + rope)) * 2, dtype)
    gamma = (1 + 0.1 * rng.normal(size=rank)).astype(np.float32)
    ang = rng.uniform(0, 6, (t, rope // 2))
    cos = rounded(np.concatenate((np.cos(ang), np.cos(ang)), 1), dtype)
    sin = rounded(np.concatenate((np.sin(ang), np.sin(ang)), 1), dtype)
    slots = rng.permutation(nb * bs)[:t].astype(np.int32)
    if t > 2:
        slots[t // 2] = -1
    q_t, qkv_t = dev(q, dtype), dev(qkv, dtype)
    cos_t, sin_t, g_t = dev(cos, dtype), dev(sin, dtype), torch.from_numpy(gamma).cuda()
    cache = torch.full((nb, bs, 1, rank + rope), 3.0, dtype=dtype, device="cuda")
    kv_view = qkv_t[:, q_lora:]
    # the separate ops
    q_pe_ref = q_t[..., nope:].reshape(t, n * rope).clone()       # copies: the separate op rotates in place
    k_pe_ref = kv_view[:, rank:].clone()
    ops.apply_rotary_pos_emb(q_pe_ref, k_pe_ref, cos_t, sin_t, n, 1, rope)
    norm_ref = ops.rms_norm(kv_view[:, :rank].clone(), g_t, 1e-6)
    if decode:
        query = torch.full((t, n, rank + rope), 9.0, dtype=dtype, device="cuda")
        ops.mla_norm_rope_cache(q_t, nope, kv_view, g_t, 1e-6, cos_t, sin_t, cache, torch.from_numpy(slots).cuda(),
                                q_rope_out=query[..., rank:])
        assert torch.equal(query[..., rank:].reshape(t, n * rope), q_pe_ref) and (query[..., :rank] == 9).all()
        assert torch.equal(q_t, dev(q, dtype))                      # the source rows are left alone
    else:
        kv_norm, k_pe = torch.empty(t, rank, dtype=dtype, device="cuda"), torch.empty(t, rope, dtype=dtype, device="cuda")
        ops.mla_norm_rope_cache(q_t, nope, kv_view, g_t, 1e-6, cos_t, sin_t, cache, torch.from_numpy(slots).cuda(),
                                kv_norm_out=kv_norm, k_pe_out=k_pe)
        assert torch.equal(q_t[..., nope:].reshape(t, n * rope), q_pe_ref)
        assert torch.equal(q_t[..., :nope], dev(q, dtype)[..., :nope])
        assert torch.equal(k_pe, k_pe_ref)
        ref = O.rms_norm(qkv[:, q_lora:q_lora + rank], gamma, 1e-6)
        assert_within(to_np(kv_norm), ref, np.abs(ref), dtype, ulps=1.0, extra=1e-7, what="latent norm")
        assert (np.abs(to_np(kv_norm) - to_np(norm_ref)) <= EPS[dtype] * np.abs(to_np(norm_ref)) * 2 + 1e-7).all()
    got = to_np(cache).reshape(nb * bs, rank + rope)
    live = slots[slots >= 0]
    rows = np.flatnonzero(slots >= 0)
    assert np.array_equal(got[live][:, rank:], to_np(k_pe_ref)[rows])
    assert (np.abs(got[live][:, :rank] - to_np(norm_ref)[rows]) <= EPS[dtype] * np.abs(to_np(norm_ref)[rows]) * 2 + 1e-7).all()
    untouched = np.ones(nb * bs, bool)
    untouched[live] = False
    assert (got[untouched] == 3).all()


def test_mla_absorb_bmm_rejects_bad_operands():
    x = torch.zeros(4, 2, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        ops.mla_absorb_bmm(x, torch.zeros(2, 16, 64, dtype=torch.bfloat16, device="cuda"))      # k mismatch
    with pytest.raises(RuntimeError):
        ops.mla_absorb_bmm(x[..., :96], torch.zeros(2, 16, 96, dtype=torch.bfloat16, device="cuda"))   # k = 96
    with pytest.raises(RuntimeError):
        ops.mla_absorb_bmm(x, torch.zeros(2, 24, 128, dtype=torch.bfloat16, device="cuda"))     # n not a multiple of 16
