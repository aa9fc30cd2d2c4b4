"""Pin the CPU oracle against every vector the reference's own tests hold for this path.

The fixtures under tests/golden/*.npz were dumped from the reference's numpy-only data files by
tests/golden/make_fixtures.py: seeded inputs, the fp32 GOLDEN arrays and the bf16 "GPU" arrays.  The
criterion is the reference's double benchmark (bf16 thresholds), with the oracle output rounded to bf16
standing where the reference's device output stands.
"""
import os

import numpy as np
import pytest

import oracle as O

R = O.round_bf16


def _load(golden_dir, name):
    return np.load(os.path.join(golden_dir, name))


def _check(device, gpu, golden, what):
    res = O.double_benchmark(R(device), gpu, golden, dtype="bfloat16")
    assert res.ok, f"{what}: {res.messages}"


# ---------------------------------------------------------------- flash / paged attention
@pytest.mark.parametrize("case,n_kv", [("1", 2), ("2", 1)])
def test_flash_attention_vectors(golden_dir, case, n_kv):
    z = _load(golden_dir, "flash_attention.npz")
    nb, bs = int(z["meta_num_blocks"]), int(z["meta_block_size"])
    nh, hid = int(z["meta_num_heads"]), int(z["meta_hidden_size"])
    d = hid // nh
    scale = 0.25          # test_infer_flash_attention.py:41-43
    pq = R(z[f"in{case}_prefill_query"]).reshape(4, -1)
    pk = R(z[f"in{case}_prefill_key"]).reshape(4, -1)
    pv = R(z[f"in{case}_prefill_value"]).reshape(4, -1)
    pre = O.causal_prefill_attention(pq, pk, pv, [2, 2], nh, n_kv, scale)
    _check(pre, z[f"gpu_prefill_output_{case}"], z[f"golden_prefill_output_{case}"], "prefill")

    kc = np.zeros((nb, bs, n_kv, d), np.float32)
    vc = np.zeros_like(kc)
    O.reshape_and_cache(pk, pv, kc, vc, z[f"in{case}_prefill_slot_mapping"])
    dk = R(z[f"in{case}_decoder_key"]).reshape(2, -1)
    dv = R(z[f"in{case}_decoder_value"]).reshape(2, -1)
    O.reshape_and_cache(dk, dv, kc, vc, z[f"in{case}_decoder_slot_mapping"])
    bt = -np.ones((2, 11), np.int32)           # run_infer_flash_attention.py:58-60
    bt[0, 0], bt[1, 0] = 2, 1
    dq = R(z[f"in{case}_decoder_query"]).reshape(2, -1)
    dec = O.paged_attention_decode(dq, kc, vc, bt, [3, 3], nh, n_kv, scale)
    _check(dec, z[f"gpu_decode_output_{case}"], z[f"golden_decode_output_{case}"], "decode")
    # a wrong GQA head mapping or a dropped token must fail the same criterion
    bad = O.paged_attention_decode(dq, kc, vc, bt, [2, 2], nh, n_kv, scale)
    assert not O.double_benchmark(R(bad), z[f"gpu_decode_output_{case}"], z[f"golden_decode_output_{case}"]).ok


@pytest.mark.parametrize("case,n_kv", [("1", 2), ("2", 1)])
def test_paged_prefill_oracle_is_pinned_by_its_special_cases(golden_dir, case, n_kv):
    """Several new tokens per sequence over the cache: with an empty cache before the step it must give the
    reference's prefill vectors, with one query per sequence the decode vectors, and a prefill cut into two
    chunks must give what the whole prefill gives."""
    z = _load(golden_dir, "flash_attention.npz")
    nb, bs = int(z["meta_num_blocks"]), int(z["meta_block_size"])
    nh, hid = int(z["meta_num_heads"]), int(z["meta_hidden_size"])
    d = hid // nh
    scale = 0.25
    pq = R(z[f"in{case}_prefill_query"]).reshape(4, -1)
    pk = R(z[f"in{case}_prefill_key"]).reshape(4, -1)
    pv = R(z[f"in{case}_prefill_value"]).reshape(4, -1)
    kc = np.zeros((nb, bs, n_kv, d), np.float32)
    vc = np.zeros_like(kc)
    O.reshape_and_cache(pk, pv, kc, vc, z[f"in{case}_prefill_slot_mapping"])
    bt = -np.ones((2, 11), np.int32)
    bt[0, 0], bt[1, 0] = 2, 1
    pre = O.paged_attention_prefill(pq, kc, vc, bt, [2, 2], [2, 2], nh, n_kv, scale)
    _check(pre, z[f"gpu_prefill_output_{case}"], z[f"golden_prefill_output_{case}"], "prefill through the cache")
    np.testing.assert_allclose(pre, O.causal_prefill_attention(pq, pk, pv, [2, 2], nh, n_kv, scale), rtol=1e-12)
    # a mask shifted by one token must fail the reference's criterion
    shifted = O.paged_attention_prefill(pq[[1, 3]], kc, vc, bt, [2, 2], [1, 1], nh, n_kv, scale)
    first = O.paged_attention_prefill(pq[[0, 2]], kc, vc, bt, [1, 1], [1, 1], nh, n_kv, scale)
    np.testing.assert_allclose(np.stack([first[0], shifted[0], first[1], shifted[1]]), pre, rtol=1e-12)   # chunks
    assert not np.allclose(O.paged_attention_prefill(pq[[0, 2]], kc, vc, bt, [2, 2], [1, 1], nh, n_kv, scale),
                           pre[[0, 2]], rtol=1e-3)

    dk = R(z[f"in{case}_decoder_key"]).reshape(2, -1)
    dv = R(z[f"in{case}_decoder_value"]).reshape(2, -1)
    O.reshape_and_cache(dk, dv, kc, vc, z[f"in{case}_decoder_slot_mapping"])
    dq = R(z[f"in{case}_decoder_query"]).reshape(2, -1)
    dec = O.paged_attention_prefill(dq, kc, vc, bt, [3, 3], [1, 1], nh, n_kv, scale)
    _check(dec, z[f"gpu_decode_output_{case}"], z[f"golden_decode_output_{case}"], "one query per sequence")
    np.testing.assert_allclose(dec, O.paged_attention_decode(dq, kc, vc, bt, [3, 3], nh, n_kv, scale), rtol=1e-12)


def test_mla_oracle_reduces_to_the_pinned_decode_oracle():
    """One latent row per token shared by all heads: with the value width equal to the key width it is
    paged_attention_decode with a single kv head (pinned by the reference's decode vectors above); a narrower value
    is the first columns of that result per head."""
    rng = np.random.default_rng(6)
    nb, bs, dk, nh, b = 12, 8, 24, 5, 3
    cache = rng.normal(size=(nb, bs, 1, dk))
    lens = np.array([9, 1, 30])
    tables = np.stack([rng.permutation(nb)[:4] for _ in range(b)]).astype(np.int32)
    q = rng.normal(size=(b, nh * dk))
    full = O.paged_attention_decode(q, cache, cache, tables, lens, nh, 1, 0.3)
    assert np.allclose(O.mla_paged_attention_decode(q, cache, tables, lens, nh, dk, 0.3), full, rtol=1e-12, atol=1e-14)
    part = O.mla_paged_attention_decode(q, cache, tables, lens, nh, 16, 0.3)
    assert np.allclose(part.reshape(b, nh, 16), full.reshape(b, nh, dk)[:, :, :16], rtol=1e-12, atol=1e-14)
    assert not O.mla_paged_attention_decode(q, cache, tables, [0, 1, 30], nh, 16, 0.3)[0].any()


@pytest.mark.parametrize("case,n_kv", [("1", 2), ("2", 1)])
def test_self_attention_vectors(golden_dir, case, n_kv):
    """QKV linear -> [q|k|v] split -> scatter -> prefill FA / decode PA -> projection
    (attention.py:214-265,344-349; scale 1/sqrt(head_dim), attention.py:135,166)."""
    z = _load(golden_dir, "attention.npz")
    nb, bs = int(z["meta_num_blocks"]), int(z["meta_block_size"])
    nh, hid = int(z["meta_num_heads"]), int(z["meta_hidden_size"])
    d = hid // nh
    scale = 1.0 / np.sqrt(d)
    wqkv, wo = R(z[f"in{case}_qkv_weight"]), R(z[f"in{case}_proj_weight"])

    def qkv(hs):
        y = R(O.linear(R(hs).reshape(-1, hid), wqkv))
        return np.split(y, [nh * d, (nh + n_kv) * d], axis=-1)

    q, k, v = qkv(z[f"in{case}_prefill_hidden_states"])
    pre = R(O.causal_prefill_attention(q, k, v, [2, 2], nh, n_kv, scale))
    pre = O.linear(pre, wo)
    _check(pre, z[f"gpu_prefill_output_{case}"], z[f"golden_prefill_output_{case}"], "prefill")

    kc = np.zeros((nb, bs, n_kv, d), np.float32)
    vc = np.zeros_like(kc)
    O.reshape_and_cache(k, v, kc, vc, z[f"in{case}_prefill_slot_mapping"])
    q, k, v = qkv(z[f"in{case}_decoder_hidden_states"])
    O.reshape_and_cache(k, v, kc, vc, z[f"in{case}_decoder_slot_mapping"])
    bt = z[f"in{case}_block_tables"].astype(np.int32)
    dec = R(O.paged_attention_decode(q, kc, vc, bt, [3, 3], nh, n_kv, scale))
    dec = O.linear(dec, wo)
    _check(dec, z[f"gpu_decode_output_{case}"], z[f"golden_decode_output_{case}"], "decode")


# ---------------------------------------------------------------- RoPE
def _rope_case(z, kind, phase):
    dim = int(z["meta_kv_channels"])
    max_pos = int(z["meta_max_position_embedding"])
    if kind == "rope":
        inv, n_pos, ms = O.rope_inv_freq_default(dim, 10000), max_pos, 1.0
    elif kind == "llama3_rope":
        inv, n_pos, ms = O.rope_inv_freq_llama3(dim, 10000, 8.0, 1.0, 4.0, 512), max_pos, 1.0
    else:
        # YaRN: table length = original_max_position * scaling_factor (yarn_rotary_pos_embedding.py:104-112)
        inv = O.rope_inv_freq_yarn(dim, 10000, 8.0, 512, 32, 1)
        n_pos = int(512 * 8.0)
        ms = O.yarn_mscale(8.0, 1.0) / O.yarn_mscale(8.0, 0.0)
    cos, sin = O.rope_cos_sin_table(inv, n_pos, ms, "bf16")
    if phase == "prefill":
        q = R(z["in_prefill_query_for_prefill"])
        k = R(z["in_prefill_key_for_prefill"])
        pos = np.array([0, 1, 0, 1])        # two sequences of two tokens, TH layout
    else:
        q = R(z["in_decode_query_for_decode"])
        k = R(z["in_decode_key_for_decode"])
        pos = np.array([1, 1])              # run_infer_rotary_embedding.py:67 (positions = ones)
    return (O.apply_rotary_half(q, cos[pos], sin[pos], 1), O.apply_rotary_half(k, cos[pos], sin[pos], 1))


@pytest.mark.parametrize("kind", ["rope", "llama3_rope", "yarn_rope"])
@pytest.mark.parametrize("phase", ["prefill", "decode"])
def test_rotary_vectors(golden_dir, kind, phase):
    z = _load(golden_dir, "rotary.npz")
    q, k = _rope_case(z, kind, phase)
    _check(q, z[f"gpu_{kind}_q_emb1_for_{phase}"], z[f"golden_{kind}_q_emb1_for_{phase}"], "q")
    _check(k, z[f"gpu_{kind}_k_emb1_for_{phase}"], z[f"golden_{kind}_k_emb1_for_{phase}"], "k")


def test_rotary_wrong_pairing_fails(golden_dir):
    """The interleaved pairing (format 3) must not pass the rotate-half vectors."""
    z = _load(golden_dir, "rotary.npz")
    dim = int(z["meta_kv_channels"])
    cos, sin = O.rope_cos_sin_table(O.rope_inv_freq_default(dim), 4, 1.0, "bf16")
    q = R(z["in_decode_query_for_decode"]).astype(np.float64)
    pos = np.array([1, 1])
    c, s = cos[pos].astype(np.float64), sin[pos].astype(np.float64)
    rot = np.empty_like(q)
    rot[:, 0::2], rot[:, 1::2] = -q[:, 1::2], q[:, 0::2]
    bad = q * c + rot * s
    assert not O.double_benchmark(R(bad), z["gpu_rope_q_emb1_for_decode"], z["golden_rope_q_emb1_for_decode"]).ok


# ---------------------------------------------------------------- norm / activation / mlp / linear
@pytest.mark.parametrize("name,eps", [("rmsnorm_output1", 1e-5), ("rmsnorm_output2", 0.1)])
def test_rmsnorm_vectors(golden_dir, name, eps):
    z = _load(golden_dir, "norm.npz")
    y = O.rms_norm(R(z["in_input"]), R(z["in_weight"]), eps)
    _check(y, z[f"gpu_{name}"], z[f"golden_{name}"], name)


@pytest.mark.parametrize("name,eps", [("layernorm_output1", 1e-5), ("layernorm_output2", 0.1)])
def test_layernorm_vectors(golden_dir, name, eps):
    z = _load(golden_dir, "norm.npz")
    y = O.layer_norm(R(z["in_input"]), R(z["in_weight"]), None, eps)
    _check(y, z[f"gpu_{name}"], z[f"golden_{name}"], name)


def test_silu_mul_vectors(golden_dir):
    z = _load(golden_dir, "activation.npz")
    y = O.silu_mul(R(z["in_multiplicand_input"]), R(z["in_multiplier_input"]))
    _check(y, z["gpu_output"], z["golden_output"], "silu*mul")


@pytest.mark.parametrize("name,gated,bias", [("has_bias_gate_output", True, True), ("has_gate_output", True, False),
                                             ("has_bias_output", False, True), ("output_only", False, False)])
def test_mlp_vectors(golden_dir, name, gated, bias):
    z = _load(golden_dir, "mlp.npz")
    w1 = R(z["in_fc1_gate_weight"] if gated else z["in_fc1_no_gate_weight"])
    b1 = R(z["in_fc1_gate_bias"] if gated else z["in_fc1_no_gate_bias"]) if bias else None
    b2 = R(z["in_fc2_bias"]) if bias else None
    y = O.mlp(R(z["in_input"]), w1, R(z["in_fc2_weight"]), b1, b2, gated=gated, act_dtype="bf16")
    _check(y, z[f"gpu_{name}"], z[f"golden_{name}"], name)


@pytest.mark.parametrize("kind", ["column", "row"])
def test_parallel_linear_vectors(golden_dir, kind):
    """Only 'legacy' bf16 device vectors exist for these; compare within two bf16 ulps of the value."""
    z = _load(golden_dir, f"{kind}_parallel_linear.npz")
    x, w, b = R(z["in_inputs"]), R(z["in_weight"]), R(z["in_bias"])
    y0 = R(O.linear(x, w))
    np.testing.assert_allclose(y0, z["legacy_output_only"], rtol=2 ** -7, atol=1e-6)
    y1 = R(O.linear(x, w, b))
    np.testing.assert_allclose(y1, z["legacy_output_with_bias"], rtol=2 ** -7, atol=1e-6)
    if kind == "column":
        y2 = R(O.linear(x, R(z["in_weight_tensor_input"]), b))
        np.testing.assert_allclose(y2, z["legacy_output_use_weight"], rtol=2 ** -7, atol=1e-6)


# ---------------------------------------------------------------- MoE layer
@pytest.mark.parametrize("name,shared", [("tp1", True), ("tp1_no_shared", False)])
def test_moe_layer_vectors(golden_dir, name, shared):
    """test_infer_moe.py:31-58: T=16, H=32, E=8, k=2, n_group=topk_group=2, scale 2.5, ffn 8, rtol 4e-3 (:132-140)."""
    z = _load(golden_dir, "moe.npz")
    x = R(z["in_input"])
    y = O.moe_layer(
        x, R(z["in_router__weight__weight"]), R(z["in_router__expert_bias"]).astype(np.float32),
        R(z["in_experts__weight1"]), R(z["in_experts__weight2"]), k=2, n_group=2, topk_group=2, scale=2.5,
        shared_fc1=R(z["in_shared_experts__linear_fc1__weight"]) if shared else None,
        shared_fc2=R(z["in_shared_experts__linear_fc2__weight"]) if shared else None,
        act_dtype="bf16", router_dtype="bf16")
    got = R(y).astype(np.float16).astype(np.float32)
    np.testing.assert_allclose(got, z[f"golden_{name}"], rtol=4e-3, atol=2e-6)


def test_float32_host_layer_follows_the_float64_oracle():
    """oracle/torch_cpu.py (the float32 restatement that the benchmark times as its CPU baseline) against the
    float64 oracle layer on a small W8A16 decode step: same rounding points, float32 in between, so the outputs agree
    to a few steps of the activation dtype, and both write the same cache rows."""
    import torch
    from oracle import torch_cpu
    rng = np.random.default_rng(3)
    hidden, nh, nkv, d, ffn, b, bs = 256, 4, 2, 64, 352, 3, 16
    lens = np.array([40, 17, 33])
    p = {}
    for name, (n, k) in {"qkv": ((nh + 2 * nkv) * d, hidden), "wo": (hidden, nh * d), "fc1": (2 * ffn, hidden),
                         "fc2": (hidden, ffn)}.items():
        p[name + "_w"], p[name + "_s"] = O.quantize_weight_int8(rng.normal(0, 0.05, (n, k)).astype(np.float32))
    p["attn_norm"] = (1 + 0.1 * rng.normal(size=hidden)).astype(np.float32)
    p["ffn_norm"] = (1 + 0.1 * rng.normal(size=hidden)).astype(np.float32)
    cfg = dict(n_head=nh, n_kv_head=nkv, head_dim=d, eps=1e-5)
    need = (lens + bs - 1) // bs
    nb = int(need.sum()) + 2
    perm = rng.permutation(nb)
    tables = -np.ones((b, int(need.max())), np.int32)
    pos = 0
    for i, n in enumerate(need):
        tables[i, :n] = perm[pos:pos + n]
        pos += n
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    kc = O.round_bf16(rng.normal(size=(nb, bs, nkv, d)).astype(np.float32))
    vc = O.round_bf16(rng.normal(size=(nb, bs, nkv, d)).astype(np.float32))
    x = O.round_bf16(rng.normal(size=(b, hidden)).astype(np.float32))
    cos, sin = O.rope_cos_sin_table(O.rope_inv_freq_default(d), 64, 1.0, "bf16")
    cos, sin = cos[lens - 1], sin[lens - 1]
    kc64, vc64 = kc.copy(), vc.copy()
    ref = O.decode_layer_w8a16(x, p, cfg, kc64, vc64, tables, lens, slots, cos, sin, act_dtype="bf16")
    kc32, vc32 = torch.from_numpy(kc.copy()), torch.from_numpy(vc.copy())
    got = torch_cpu.decode_layer_w8a16_fp32(torch.from_numpy(x), torch_cpu.prepare_params(p), cfg, kc32, vc32, tables,
                                            lens, slots, torch.from_numpy(cos.astype(np.float32)),
                                            torch.from_numpy(sin.astype(np.float32)), act_dtype="bf16").numpy()
    err = np.abs(got - ref)
    tol = 4 * 2.0 ** -8 * np.maximum(np.abs(ref), 0.1 * np.abs(ref).max(axis=1, keepdims=True))
    assert np.mean(err > tol) < 0.01 and err.max() < 0.1 * np.abs(ref).max(), (np.mean(err > tol), err.max())
    row = nkv * d
    written = np.zeros(nb * bs, bool)
    written[slots] = True
    assert np.array_equal(kc32.numpy().reshape(-1, row)[~written], kc.reshape(-1, row)[~written])
    assert np.abs(kc32.numpy() - kc64).max() <= 2 * 2.0 ** -8 * np.abs(kc64).max()
    assert np.abs(vc32.numpy() - vc64).max() <= 2 * 2.0 ** -8 * np.abs(vc64).max()


# ------------------------------------------------------------------------------------------- multi-latent layer
def _mla_case(rng, n=4, nope=16, rope=8, rank=32, vd=16, hidden=64, q_lora=24):
    cfg = dict(n_head=n, qk_head_dim=nope, qk_pos_emb_head_dim=rope, kv_lora_rank=rank, v_head_dim=vd,
               q_lora_rank=q_lora, eps=1e-6, rotary_scaling_factor=40.0, mscale=1.0)
    p = dict(q_norm=1 + 0.1 * rng.normal(size=q_lora or 1), kv_norm=1 + 0.1 * rng.normal(size=rank),
             kv_up_w=rng.normal(0, 0.3, (n * (nope + vd), rank)), proj_w=rng.normal(0, 0.3, (hidden, n * vd)))
    if q_lora:
        p["qkv_down_w"] = rng.normal(0, 0.3, (q_lora + rank + rope, hidden))
        p["q_up_w"] = rng.normal(0, 0.3, (n * (nope + rope), q_lora))
    else:
        p["q_w"] = rng.normal(0, 0.3, (n * (nope + rope), hidden))
        p["kv_down_w"] = rng.normal(0, 0.3, (rank + rope, hidden))
    return cfg, p


@pytest.mark.parametrize("q_lora", [24, None])
def test_mla_decode_with_absorbed_weights_equals_the_prefill_definition(q_lora):
    """multi_latent_attention.py:434-448 folds the key up-projection into the query and applies the value
    up-projection to the attention output; :405-432 (prefill) up-projects keys and values and runs ordinary
    attention.  Both are the same function of the tokens: the decode step of a sequence's last token over a cache
    that the earlier tokens filled must equal the last row of a prefill over the whole sequence."""
    rng = np.random.default_rng(17)
    cfg, p = _mla_case(rng, q_lora=q_lora)
    lens = [6, 1, 9]
    bs, rope = 4, cfg["qk_pos_emb_head_dim"]
    dk = cfg["kv_lora_rank"] + rope
    need = [(l + bs - 1) // bs for l in lens]
    nb = sum(need) + 1
    perm = rng.permutation(nb)
    tables = -np.ones((len(lens), max(need)), np.int32)
    pos = 0
    for i, k in enumerate(need):
        tables[i, :k] = perm[pos:pos + k]
        pos += k
    total = sum(lens)
    hidden = rng.normal(size=(total, 64))
    inv = O.rope_inv_freq_default(rope, 10000.0)
    cos_t, sin_t = O.rope_cos_sin_table(inv, 16)
    positions = np.concatenate([np.arange(l) for l in lens])
    cos, sin = cos_t[positions], sin_t[positions]
    starts = np.cumsum([0] + lens)
    slots = np.concatenate([[tables[i, j // bs] * bs + j % bs for j in range(l)] for i, l in enumerate(lens)]).astype(np.int32)
    # the definition: prefill over whole sequences
    cache_pf = np.zeros((nb, bs, 1, dk))
    full = O.mla_self_attention_prefill(hidden, p, cfg, cache_pf, slots, lens, cos, sin)
    # decode: earlier tokens through prefill (only their cache rows matter), the last token of each as a decode step
    cache = np.zeros((nb, bs, 1, dk))
    early = np.concatenate([np.arange(starts[i], starts[i + 1] - 1) for i in range(len(lens))]).astype(np.int64)
    if len(early):
        O.mla_self_attention_prefill(hidden[early], p, cfg, cache, slots[early], [l - 1 for l in lens if l > 1],
                                     cos[early], sin[early])
    last = starts[1:] - 1
    dec = O.mla_self_attention_decode(hidden[last], p, cfg, cache, tables, np.asarray(lens, np.int32), slots[last],
                                      cos[last], sin[last])
    assert np.allclose(cache, cache_pf, rtol=0, atol=1e-12)
    assert np.allclose(dec, full[last], rtol=1e-10, atol=1e-10)
    # negative control: the two halves of linear_kv_up_proj swapped must not pass
    bad = dict(p)
    n, nope = cfg["n_head"], cfg["qk_head_dim"]
    bad["kv_up_w"] = np.concatenate((p["kv_up_w"][n * nope:], p["kv_up_w"][: n * nope]))
    dec_bad = O.mla_self_attention_decode(hidden[last], bad, cfg, cache.copy(), tables, np.asarray(lens, np.int32),
                                          slots[last], cos[last], sin[last])
    assert not np.allclose(dec_bad, full[last], rtol=1e-3, atol=1e-3)
