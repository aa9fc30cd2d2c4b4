"""CPU-only tests: the C-ABI library loads and exports what include/mf_decode.h declares, host-side logic
(block tables, quantization configs and dispatch, rotary tables), and properties that pin the oracle beyond the
reference's vectors (router brute force, quantisation grid, int32 exactness)."""
import ctypes
import itertools
import os
import re

import numpy as np
import pytest
import torch

import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------------------------------- C ABI
def _declared_functions():
    text = open(os.path.join(ROOT, "include", "mf_decode.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from mindformers_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from mindformers_amd import build
        build.build(verbose=False)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared_functions()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in mf_decode.h but not exported"
    # the ctypes table binds exactly the declared entry points
    assert sorted(_lib.SIGNATURES) == declared
    loaded = _lib.load()
    assert loaded.mf_version().decode().startswith("mf_decode")
    # size queries are pure host functions: callable without a GPU
    assert loaded.mf_w8a16_packed_bytes(4096, 4096) == 4096 * 4096
    assert loaded.mf_w8a16_packed_bytes(17, 1376) == 32 * 1408
    assert loaded.mf_paged_attention_workspace_bytes(64, 32, 128, 256) == 0
    assert loaded.mf_paged_attention_workspace_bytes(64, 32, 128, 4096) == 64 * 32 * 16 * 130 * 4
    assert loaded.mf_w8a16_workspace_bytes(0, 10, 16) == 0


def test_argument_errors_are_reported_without_a_gpu():
    from mindformers_amd import _lib
    lib = _lib.load()
    rc = lib.mf_paged_attention_decode(None, None, None, None, None, None, 1, 32, 8, 100, 128, 4, 10, 0.1, 0, 0, None, 0, None)
    assert rc == 1 and b"null" in lib.mf_last_error()
    rc = lib.mf_w8a16_gemm(1, 1, 1, 1, None, None, 4, 8, 12, 0, None, 0, None)
    assert rc == 1 and b"multiple of 8" in lib.mf_last_error()
    with pytest.raises(_lib.MfKernelError):
        _lib.check(rc, "mf_w8a16_gemm")


def test_ops_refuse_cpu_tensors():
    from mindformers_amd import ops
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.rms_norm(x, torch.ones(64), 1e-5)


# ------------------------------------------------------------------------------------------- block tables
def test_block_tables_match_naive_slot_mapping():
    from mindformers_amd.modules import BlockTables
    rng = np.random.default_rng(0)
    bs, seq, batch = 16, 256, 5
    bt = BlockTables(num_blocks=128, block_size=bs, seq_length=seq)
    bt.init_cache_engine(batch)
    lens = rng.integers(1, 100, batch)
    tables, slots = bt.assemble_pa_full_inputs(int(lens.max()), lens, [False] * batch)
    assert tables.shape == (batch, seq // bs) and tables.dtype == np.int32
    ref = O.prefill_slot_mapping(tables, lens, bs, int(lens.max()))
    assert np.array_equal(slots, ref)
    # blocks are handed out first-fit from the free list (cache_engine.py:45-53)
    used = tables[tables >= 0]
    assert sorted(used.tolist()) == list(range(len(used)))
    for step in range(40):                                # decode steps cross block boundaries
        lens = lens + 1
        tables, slots = bt.assemble_pa_inc_inputs(lens, [False] * batch)
        assert np.array_equal(slots, O.decode_slot_mapping(tables, lens, bs))
    bt.clear_cache()
    assert len(bt.block_mem_pool.free_blocks) == 128
    with pytest.raises(RuntimeError):
        bt.block_mem_pool.allocate_block(129)
    with pytest.raises(RuntimeError):
        bt.block_mem_pool.free_block([3])


# ------------------------------------------------------------------------------------------- quantization configs
def test_auto_quantizer_dispatch():
    """Mirrors tests/st/test_ut/test_models/test_auto/test_auto_quantizer.py:31-77 (dispatch and errors)."""
    from mindformers_amd.modules.quantizers import (AutoQuantizationConfig, AutoQuantizer, PtqQuantizer, RtnQuantizer,
                                                    SmoothQuantQuantizer)
    from mindformers_amd.quantization_config import PtqConfig, RtnConfig, SmoothQuantConfig
    with pytest.raises(ValueError):
        AutoQuantizationConfig.from_dict({})
    with pytest.raises(ValueError):
        AutoQuantizationConfig.from_dict({"quant_method": "xxx"})
    cfg = AutoQuantizationConfig.from_dict({"quant_method": "rtn", "weight_dtype": "int8", "modules_to_not_convert": ["lm_head"]})
    assert isinstance(cfg, RtnConfig) and cfg.opname_blacklist == ["lm_head"]
    assert isinstance(AutoQuantizer.from_config(cfg), RtnQuantizer)
    assert isinstance(AutoQuantizer.from_config({"quant_method": "ptq"}), PtqQuantizer)
    assert isinstance(AutoQuantizationConfig.from_dict({"quant_method": "ptq"}), PtqConfig)
    sq = AutoQuantizer.from_config({"quant_method": "smooth_quant"})
    assert isinstance(sq, SmoothQuantQuantizer) and isinstance(sq.quant_config, SmoothQuantConfig)


def test_quantization_config_validation():
    from mindformers_amd.quantization_config import PtqConfig, RtnConfig, SmoothQuantConfig
    with pytest.raises(ValueError):                      # RTN is weight-only (quantization_config.py:281-286)
        RtnConfig(activation_dtype="int8")
    with pytest.raises(ValueError):
        RtnConfig(outliers_suppression="smooth")
    with pytest.raises(ValueError):
        RtnConfig(mode="quantize")
    with pytest.raises(ValueError):                      # per_token needs W8A8 (:438-442)
        PtqConfig(weight_dtype="int8", activation_dtype=None, act_quant_granularity="per_token")
    with pytest.raises(ValueError):
        PtqConfig(weight_dtype=None, activation_dtype="int8")
    with pytest.raises(ValueError):
        PtqConfig(group_size=32)
    with pytest.raises(TypeError):
        PtqConfig(layer_policies={"(": {"quant_method": "ptq"}})
    with pytest.raises(ValueError):                      # SmoothQuant is A8W8 per tensor only (:577-595)
        SmoothQuantConfig(act_quant_granularity="per_token")
    with pytest.raises(ValueError):
        SmoothQuantConfig(activation_dtype=None)
    ok = PtqConfig(weight_dtype="int8", activation_dtype="int8", act_quant_granularity="per_token",
                   outliers_suppression="smooth", layer_policies={r".*wo": {"quant_method": "ptq"}})
    assert ok.to_dict()["act_quant_granularity"] == "per_token" and list(ok.layer_policies) == [r".*wo"]


def test_unbuilt_quant_modes_are_rejected_at_conversion():
    from mindformers_amd.modules.quantizers.base import check_buildable
    from mindformers_amd.quantization_config import PtqConfig, SmoothQuantConfig
    check_buildable(SmoothQuantConfig())                 # static per-tensor activations + smooth: built
    check_buildable(PtqConfig(weight_dtype="int4", weight_quant_granularity="per_group", group_size=64))   # A16W4: built
    check_buildable(PtqConfig(weight_dtype="int4", outliers_suppression="awq", weight_quant_granularity="per_group",
                              group_size=128))
    with pytest.raises(NotImplementedError):             # per_group scales go with 4-bit weights
        check_buildable(PtqConfig(weight_dtype="int8", weight_quant_granularity="per_group", group_size=64))
    with pytest.raises(NotImplementedError):             # per_group without a group size
        check_buildable(PtqConfig(weight_dtype="int4", weight_quant_granularity="per_group", group_size=0))
    with pytest.raises(NotImplementedError):
        check_buildable(PtqConfig(weight_dtype="int4", precision_recovery="gptq"))
    check_buildable(PtqConfig(activation_dtype="int8", act_quant_granularity="per_token", kvcache_dtype="int8",
                              kvcache_quant_granularity="per_token"))            # per-token int8 cache: built
    check_buildable(PtqConfig(kvcache_dtype="int8"))
    check_buildable(PtqConfig())


# ------------------------------------------------------------------------------------------- rotary tables (host)
def test_rotary_modules_build_the_oracle_tables():
    from mindformers_amd.modules import FreqsMgr, Llama3RotaryEmbedding, RotaryEmbedding, YaRNScalingRotaryEmbedding
    d = 32
    r = RotaryEmbedding(d, rotary_cos_format=2, rotary_dtype=torch.bfloat16, max_position_embeddings=64, device="cpu")
    cos, sin = O.rope_cos_sin_table(O.rope_inv_freq_default(d), 64, 1.0, "bf16")
    assert np.array_equal(r.cos_cache.float().numpy(), cos) and np.array_equal(r.sin_cache.float().numpy(), sin)
    l3 = Llama3RotaryEmbedding(d, rotary_cos_format=2, rotary_dtype=torch.float32, max_position_embeddings=64,
                               scaling_factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, orig_max_position=512, device="cpu")
    cos, _ = O.rope_cos_sin_table(O.rope_inv_freq_llama3(d, 10000, 8.0, 1.0, 4.0, 512), 64, 1.0, "fp32")
    assert np.allclose(l3.cos_cache.numpy(), cos, atol=1e-6)
    y = YaRNScalingRotaryEmbedding(d, rotary_cos_format=2, rotary_dtype=torch.float32, scaling_factor=8.0,
                                   original_max_position_embeddings=16, beta_fast=32, beta_slow=1, mscale=1.0,
                                   mscale_all_dim=0.0, device="cpu")
    assert y.cos_cache.shape == (128, d)
    ms = O.yarn_mscale(8.0, 1.0) / O.yarn_mscale(8.0, 0.0)
    cos, _ = O.rope_cos_sin_table(O.rope_inv_freq_yarn(d, 10000, 8.0, 16, 32, 1), 128, ms, "fp32")
    assert np.allclose(y.cos_cache.numpy(), cos, atol=1e-6)
    f = FreqsMgr(d, max_position_embedding=64, rotary_dtype=torch.float32, device="cpu")
    c, s, _ = f.increment(torch.tensor([1, 5, 64]))
    ref_c, ref_s = O.rope_cos_sin_table(O.rope_inv_freq_default(d), 64, 1.0, "fp32")
    assert np.allclose(c.numpy(), ref_c[[0, 4, 63]], atol=1e-6) and np.allclose(s.numpy(), ref_s[[0, 4, 63]], atol=1e-6)
    with pytest.raises(NotImplementedError):
        RotaryEmbedding(d, rotary_interleaved=True, device="cpu")
    with pytest.raises(NotImplementedError):
        RotaryEmbedding(d, seq_len_interpolation_factor=1.1, device="cpu")


# ------------------------------------------------------------------------------------------- oracle properties
def test_router_matches_brute_force_with_group_limit():
    """The reference holds no vector with n_group > topk_group; pin the group-limited selection by exhaustive
    search on small sizes: chosen set = top-k of the biased scores restricted to the best groups."""
    rng = np.random.default_rng(5)
    for e, ng, tg, k in ((8, 4, 2, 2), (12, 3, 1, 3), (16, 4, 3, 4)):
        logits = rng.normal(size=(20, e)).astype(np.float32)
        bias = rng.normal(0, 0.2, e).astype(np.float32)
        w, idx = O.topk_router(logits, bias, k, ng, tg, 2.5)
        s = 1 / (1 + np.exp(-logits.astype(np.float64)))
        sb = s + bias
        gs = e // ng
        for t in range(20):
            gscore = [np.sort(sb[t, g * gs:(g + 1) * gs])[-2:].sum() for g in range(ng)]
            best_groups = set(np.argsort(gscore)[-tg:].tolist())
            allowed = [i for i in range(e) if i // gs in best_groups]
            best = max(itertools.combinations(allowed, k), key=lambda c: sb[t, list(c)].sum())
            assert set(idx[t].tolist()) == set(best)
            assert np.all(np.diff(sb[t, idx[t]]) <= 0)               # descending by biased score
            ref_w = s[t, idx[t]] / s[t, idx[t]].sum() * 2.5
            assert np.allclose(w[t], ref_w, rtol=1e-12)
    # n_group == topk_group reduces to plain biased top-k
    logits = rng.normal(size=(6, 16)).astype(np.float32)
    _, a = O.topk_router(logits, None, 4, 4, 4, 1.0)
    _, b = O.topk_router(logits, None, 4, 1, 1, 1.0)
    assert np.array_equal(a, b)


def test_quantisation_grid_properties():
    rng = np.random.default_rng(6)
    w = rng.normal(0, 0.02, (64, 256)).astype(np.float32)
    q, s = O.quantize_weight_int8(w)
    assert q.dtype == np.int8 and np.abs(q).max() == 127 and np.all(np.abs(q).max(axis=1) == 127)
    assert np.abs(q.astype(np.float64) * s[:, None] - w).max() <= s.max() / 2 * (1 + 1e-6)
    q2, s2 = O.quantize_weight_int8(q.astype(np.float32) * s[:, None])           # idempotent on its own grid
    assert np.array_equal(q, q2)
    x = rng.normal(size=(16, 256)).astype(np.float32)
    xq, xs = O.dynamic_quant_per_token(x, rng.uniform(0.5, 2, 256).astype(np.float32))
    assert np.all(np.abs(xq.astype(np.int32)).max(axis=1) == 127)
    # rint: ties go to even
    xq, _ = O.dynamic_quant_per_token(np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5]], np.float32))
    assert xq.tolist() == [[127, 0, 2, 2, 0, -2]]
    # int32 accumulators are exact integer matmul, including the extreme corner
    a = np.full((2, 512), -128, np.int8)
    b = np.full((3, 512), -127, np.int8)
    assert np.all(O.int8_gemm_i32(a, b) == 128 * 127 * 512)


def test_kv_int8_oracle_pair_is_pinned_by_what_the_mathematics_fixes():
    """The int8 KV-cache pair q = clip(rint(x / s + o), -128, 127), x ~ (q - o) * s, pinned without its own formula:
    hand-computed values, the direction of the offset and the side of the scale (a mirrored sign or a product in
    place of the quotient fails), clipping at both rails, the half-step round-trip bound inside the rails, and
    torch's affine per-channel quantiser (x / s rounded, plus an integer zero point) on power-of-two scales."""
    # hand-computed: 0.26 / 0.1 + 3 = 5.6 -> 6; (6 - 3) * 0.1 = 0.3; -0.26 / 0.1 + 3 = 0.4 -> 0; (0 - 3) * 0.1 = -0.3
    q = O.quantize_kv_int8(np.array([[0.26, -0.26]]), np.array([0.1, 0.1]), np.array([3.0, 3.0]))
    assert q.dtype == np.int8 and q.tolist() == [[6, 0]]
    assert np.allclose(O.dequantize_kv_int8(q, np.array([0.1, 0.1]), np.array([3.0, 3.0])), [[0.3, -0.3]], atol=1e-15)
    # zero maps to the offset itself (not to its negative) and comes back as zero; k * s maps to k + o exactly
    s = np.array([0.5, 0.25, 2.0, 0.125])
    o = np.array([7.0, -11.0, 0.0, 30.0])
    assert O.quantize_kv_int8(np.zeros((1, 4)), s, o).tolist() == [[7, -11, 0, 30]]
    assert np.array_equal(O.dequantize_kv_int8(np.array([[7, -11, 0, 30]], np.int8), s, o), np.zeros((1, 4)))
    ks = np.array([[5, -9, 17, -40]])
    assert np.array_equal(O.quantize_kv_int8(ks * s, s, o), (ks + o).astype(np.int8))   # a product x * s gives 5 s^2
    assert np.array_equal(O.dequantize_kv_int8((ks + o).astype(np.int8), s, o), ks * s)
    # no offset = offset 0
    x = np.random.default_rng(3).normal(size=(50, 4))
    assert np.array_equal(O.quantize_kv_int8(x, s), O.quantize_kv_int8(x, s, np.zeros(4)))
    # clipping at the rails: anything beyond (127 - o) s / (-128 - o) s sticks to 127 / -128
    big = np.array([[1e6, 1e6, 1e6, 1e6], [-1e6, -1e6, -1e6, -1e6]])
    assert O.quantize_kv_int8(big, s, o).tolist() == [[127] * 4, [-128] * 4]
    hi, lo = (127 - o) * s, (-128 - o) * s
    assert O.quantize_kv_int8(np.stack([hi + 0.6 * s, lo - 0.6 * s]), s, o).tolist() == [[127] * 4, [-128] * 4]
    # ties go to even (the declared rounding): 2.5 -> 2, 3.5 -> 4, -2.5 -> -2
    assert O.quantize_kv_int8(np.array([[2.5, 3.5, -2.5]]), np.ones(3)).tolist() == [[2, 4, -2]]
    # inside the rails the round trip is within half a step, and the step is the scale
    rng = np.random.default_rng(8)
    s = rng.uniform(0.005, 0.05, 64)
    o = rng.integers(-30, 31, 64).astype(np.float64)
    x = rng.uniform((-128 - o) * s, (127 - o) * s, (500, 64))
    back = O.dequantize_kv_int8(O.quantize_kv_int8(x, s, o), s, o)
    assert np.all(np.abs(back - x) <= s / 2 * (1 + 1e-9))
    assert np.abs(back - x).max() > 0.4 * s.min()                          # a real grid, not a pass-through
    # a library routine: torch's affine per-channel quantiser, q = clamp(round(x / s) + zero_point), on
    # power-of-two scales (the quotient is then exact in float32 too) and integer zero points
    s2 = (2.0 ** rng.integers(-7, -3, 64)).astype(np.float64)
    zp = rng.integers(-30, 31, 64)
    xt = torch.from_numpy(rng.normal(0, 1.5, (300, 64)).astype(np.float32))
    tq = torch.quantize_per_channel(xt, torch.from_numpy(s2), torch.from_numpy(zp), 1, torch.qint8)
    mine = O.quantize_kv_int8(xt.numpy(), s2, zp.astype(np.float64))
    assert np.array_equal(mine, tq.int_repr().numpy())
    assert (mine == 127).any() and (mine == -128).any()                    # the rails are exercised
    assert np.array_equal(O.dequantize_kv_int8(mine, s2, zp.astype(np.float64)), tq.dequantize().double().numpy())


def test_static_per_tensor_quant_oracle_properties():
    """The static per-tensor activation quantiser: hand values, ties to even, both rails, the smoothing multiplier
    applied before the division, one scale for every row; and agreement with torch's per-tensor affine quantiser on a
    power-of-two scale."""
    q, s = O.static_quant_per_tensor(np.array([[0.26, -0.26, 0.25, 0.35, 100.0, -100.0]], np.float32), 0.1)
    assert q.tolist() == [[3, -3, 2, 4, 127, -128]] and s.tolist() == [np.float32(0.1)]
    q, _ = O.static_quant_per_tensor(np.array([[1.0, 1.0]], np.float32), 0.5, np.array([2.0, 0.5], np.float32))
    assert q.tolist() == [[4, 1]]                                         # x * smooth / scale
    rng = np.random.default_rng(12)
    x = rng.normal(0, 2, (40, 64)).astype(np.float32)
    q, s = O.static_quant_per_tensor(x, 2.0 ** -5)
    tq = torch.quantize_per_tensor(torch.from_numpy(x), 2.0 ** -5, 0, torch.qint8)
    assert np.array_equal(q, tq.int_repr().numpy()) and np.all(s == np.float32(2.0 ** -5))
    assert (q == 127).any() and (q == -128).any()
    inside = np.abs(x) < 127 * 2.0 ** -5
    assert np.abs(q[inside] * 2.0 ** -5 - x[inside]).max() <= 2.0 ** -6


def test_moe_permute_is_a_stable_sort_and_unpermute_inverts_it():
    rng = np.random.default_rng(7)
    t, k, e, h = 9, 3, 5, 4
    x = rng.normal(size=(t, h))
    idx = rng.integers(0, e, (t, k)).astype(np.int32)
    px, row_map, counts = O.moe_permute(x, idx, e)
    flat = idx.reshape(-1)
    assert counts.sum() == t * k and np.array_equal(counts, np.bincount(flat, minlength=e))
    sorted_experts = np.empty(t * k, dtype=np.int64)
    sorted_experts[row_map] = flat
    assert np.all(np.diff(sorted_experts) >= 0)
    for ex in range(e):                                   # stability: pair order preserved inside an expert
        rows = row_map[flat == ex]
        assert np.all(np.diff(rows) > 0)
    assert np.array_equal(px[row_map], x[np.arange(t * k) // k])
    ones = np.ones((t, k))
    assert np.allclose(O.moe_unpermute(px, row_map, ones), k * x)


def test_cache_sizing_follows_the_reference_formula():
    """model_runner.py:370-376: blocks = mem // (block_size * kv_heads * head_size * bytes * 2 * layers)."""
    from mindformers_amd.runner import num_cache_blocks
    # 1 GiB, block 128, 8 kv heads x 128, 32 layers, bf16: 2^30 / (128*8*128*2*2*32) = 64 blocks
    assert num_cache_blocks(1, 128, 8, 128, 32, 2) == 64
    assert num_cache_blocks(1, 128, 8, 128, 32, 1) == 128           # int8 cache
    assert num_cache_blocks(0, 128, 8, 128, 32, 2) == 0


# ------------------------------------------------------------------------------------------- 4-bit weight convention
@pytest.mark.parametrize("group", [0, 64, 128])
def test_int4_weight_quantisation_is_held_to_what_the_mathematics_fixes(group):
    """The declared A16W4 convention (s = max|w| / 7 per channel or per channel and group, q = clip(rint(w / s), -8, 7),
    the group's scale on the group's sum): values on the grid come back exactly, everything comes back within half a
    step, the extreme of every group sits on the rail, the two-per-byte form is a bijection, and on power-of-two scales
    with integer activations the linear is the exact integer matmul.  A scale applied per channel where it is per
    group, a transposed scale table or a swapped nibble order fails one of these."""
    rng = np.random.default_rng(40 + group)
    n, k = 12, 256
    g = group or k
    w = rng.normal(size=(n, k))
    q, s = O.quantize_weight_int4(w, group)
    assert q.dtype == np.int8 and q.min() >= -8 and q.max() <= 7
    assert s.shape == ((n,) if group == 0 else (k // g, n)) and s.dtype == np.float32
    s_full = (np.repeat(s[None, :], 1, 0).T if group == 0 else s.T)                  # [N, K/g]
    deq = (q.reshape(n, k // g, g) * s_full[:, :, None].astype(np.float64)).reshape(n, k)
    assert np.all(np.abs(deq - w) <= 0.5 * np.repeat(s_full, g, axis=1) * (1 + 1e-6))
    amax = np.abs(w.reshape(n, k // g, g)).max(axis=2)
    assert np.all(np.abs(q.reshape(n, k // g, g)).max(axis=2) == 7) and np.allclose(s_full, amax / 7, rtol=1e-6)
    # a weight already on the grid of power-of-two scales is reproduced exactly, and the linear is the integer matmul
    s2 = 2.0 ** rng.integers(-6, -2, s_full.shape)
    q0 = rng.integers(-7, 8, (n, k)).astype(np.int8)
    q0.reshape(n, k // g, g)[:, :, 0] = 7                                             # every group reaches the rail
    w0 = (q0.reshape(n, k // g, g) * s2[:, :, None]).reshape(n, k)
    q1, s1 = O.quantize_weight_int4(w0, group)
    assert np.array_equal(q1, q0) and np.array_equal(s1, (s2[:, 0] if group == 0 else s2.T).astype(np.float32))
    x = rng.integers(-3, 4, (5, k)).astype(np.float64)
    y = O.w4a16_linear(x, q1, s1, group)
    assert np.array_equal(y, x @ w0.T)
    # two values per byte, element 2j in the low nibble
    packed = O.pack_qint4x2(q0)
    assert packed.shape == (n, k // 2) and np.array_equal(O.unpack_qint4x2(packed), q0)
    one = O.pack_qint4x2(np.array([[-8, 7, 1, -1]], np.int8)).view(np.uint8)
    assert one.tolist() == [[0x78, 0xF1]]
