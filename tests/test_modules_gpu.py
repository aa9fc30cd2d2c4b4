"""The drop-in modules on the GPU, checked against the oracle and the reference's vectors.  GPU only.

These read like the reference's own module tests (tests/st/test_infer/test_infer_module/*,
tests/st/test_ut/test_parallel_core/test_inference/**): build the cell with the reference's arguments, feed the
reference's inputs, compare the outputs.
"""
import os

import numpy as np
import pytest
import torch

import oracle as O
from helpers import EPS, assert_within, dev, make_paged_cache, rounded, to_np, untile_int8

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    assert torch.cuda.is_available()
    from mindformers_amd import _lib
    _lib.load()
    yield


# ------------------------------------------------------------------------------------------- attention cells
def test_paged_attention_mgr_surface():
    """tests/st/test_infer/test_infer_module/test_paged_attention_mgr.py:28-60: all-ones inputs, shape check —
    plus the values: with identical keys every probability is equal and the output is the mean of V = 1."""
    from mindformers_amd.modules import PagedAttentionMgr
    bsz, n_head, head_dim, n_kv, bs, nb = 1, 8, 128, 8, 16, 64
    mgr = PagedAttentionMgr(n_head, head_dim, n_kv, (nb, bs, n_kv, head_dim), compute_dtype=torch.float16)
    assert mgr.key_cache.shape == (nb, bs, n_kv, head_dim) and mgr.scale_value == 1 / np.sqrt(head_dim)
    key = torch.ones(bsz, 1, n_kv * head_dim, dtype=torch.float16, device="cuda")
    slot = torch.tensor([3], dtype=torch.int32, device="cuda")
    out_k = mgr(key, key, slot)
    assert out_k.shape == key.shape
    q = torch.ones(bsz, 1, n_head * head_dim, dtype=torch.float16, device="cuda")
    tables = torch.zeros(bsz, 4, dtype=torch.int32, device="cuda")
    ctx = mgr.paged_attn(q, torch.tensor([4], dtype=torch.int32, device="cuda"), tables)
    assert ctx.shape == (bsz, 1, n_head * head_dim)
    # slots 0-2 are zeros, slot 3 holds ones: scores (0,0,0,sqrt(D)) -> weight of the ones row
    wgt = np.exp(np.sqrt(head_dim)) / (3 + np.exp(np.sqrt(head_dim)))
    assert np.allclose(to_np(ctx), wgt, rtol=2e-3)
    with pytest.raises(NotImplementedError):
        mgr.paged_attn_with_alibi(q, None, tables, None)
    with pytest.raises(ValueError):
        PagedAttentionMgr(8, 128, 8, (4, 16, 8))


@pytest.mark.parametrize("dynamic", [True, False])
def test_infer_attention_decode_step(dynamic):
    """InferAttention decode call (test_infer_attention.py:179-274 calling convention: batch_valid_length counts
    the new token, freqs_mgr.increment rows) against oracle RoPE -> scatter -> attention."""
    from mindformers_amd.modules import BlockTables, FreqsMgr, InferAttention
    rng = np.random.default_rng(3)
    b, n_head, n_kv, d, bs, nb, seq = 4, 8, 2, 64, 16, 128, 512
    dt = torch.float16
    attn = InferAttention(n_head, d, n_kv, scale_value=1 / np.sqrt(d), block_size=bs, num_blocks=nb, seq_length=seq,
                          is_dynamic=dynamic, rotary_cos_format=2, compute_dtype=dt)
    assert attn.is_first_iteration and attn.paged_attention_mgr.key_cache.shape == (nb, bs, n_kv, d)
    attn.is_first_iteration = False
    mgr = BlockTables(nb, bs, seq)
    mgr.init_cache_engine(b)
    past = rng.integers(20, 200, b)
    mgr.assemble_pa_full_inputs(int(past.max()), past, [False] * b)
    # fill the cache with an earlier context
    kc0 = rounded(rng.normal(size=(nb, bs, n_kv, d)), dt)
    vc0 = rounded(rng.normal(size=(nb, bs, n_kv, d)), dt)
    attn.paged_attention_mgr.key_cache.copy_(dev(kc0, dt))
    attn.paged_attention_mgr.value_cache.copy_(dev(vc0, dt))
    lens = past + 1
    tables, slots = mgr.assemble_pa_inc_inputs(lens, [False] * b)
    freqs = FreqsMgr(d, seq_length=seq, max_position_embedding=seq, rotary_dtype=dt)
    lens_t = torch.from_numpy(lens.astype(np.int32)).cuda()
    freqs_cis = freqs.increment(lens_t)
    q = rounded(rng.normal(size=(b, n_head * d)), dt)
    k = rounded(rng.normal(size=(b, n_kv * d)), dt)
    v = rounded(rng.normal(size=(b, n_kv * d)), dt)
    shape = (b, n_head * d) if dynamic else (b, 1, n_head * d)
    out = attn(dev(q, dt).reshape(shape), dev(k, dt).reshape(b, -1) if dynamic else dev(k, dt).reshape(b, 1, -1),
               dev(v, dt).reshape(b, -1) if dynamic else dev(v, dt).reshape(b, 1, -1), lens_t,
               torch.from_numpy(tables).cuda(), torch.from_numpy(slots).cuda(), freqs_cis)
    assert out.shape == shape
    cos, sin = to_np(freqs_cis[0]), to_np(freqs_cis[1])
    q_r = rounded(O.apply_rotary_half(q, cos, sin, n_head), dt)
    k_r = rounded(O.apply_rotary_half(k, cos, sin, n_kv), dt)
    O.reshape_and_cache(k_r, v, kc0, vc0, slots)
    ref = O.paged_attention_decode(q_r, kc0, vc0, tables, lens, n_head, n_kv, 1 / np.sqrt(d))
    mag = O.paged_attention_decode(q_r, kc0, np.abs(vc0), tables, lens, n_head, n_kv, 1 / np.sqrt(d))
    # rotated q/k may differ from the oracle's by one rounding step: allow it on top of the attention tolerance
    assert_within(to_np(out).reshape(b, -1), ref, mag, dt, ulps=4.0, what="InferAttention decode")
    got_k = to_np(attn.paged_attention_mgr.key_cache).reshape(-1, n_kv * d)
    assert np.abs(got_k[slots] - k_r).max() <= 2 * EPS[dt] * np.abs(k_r).max()
    assert np.array_equal(to_np(attn.paged_attention_mgr.value_cache).reshape(-1, n_kv * d)[slots], v)


@pytest.mark.parametrize("case,n_kv", [("1", 2), ("2", 1)])
def test_mcore_flash_attention_prefill_vectors(golden_dir, case, n_kv):
    """The reference's FlashAttention unit test, prefill half (run_infer_flash_attention.py:106-150): the cell
    scatters the prompt's K/V and runs causal attention over them; actual_seq_qlen is passed as the test passes it
    (the per-sequence lengths) and as the operator documents it (increasing row ends)."""
    from mindformers_amd.modules import FlashAttention
    z = np.load(os.path.join(golden_dir, "flash_attention.npz"))
    nb, bs, nh, hid = (int(z[k]) for k in ("meta_num_blocks", "meta_block_size", "meta_num_heads", "meta_hidden_size"))
    d = hid // nh
    net = FlashAttention(head_num=nh, head_dim=d, keep_prob=1.0, kv_head_num=n_kv, pa_kv_head_num=n_kv, scale_value=0.25)
    assert net.is_prefill
    bt = -np.ones((2, 11), np.int32)
    bt[0, 0], bt[1, 0] = 2, 1
    mask = torch.triu(torch.ones(2, 2, dtype=BF, device="cuda"), diagonal=1)
    for lens in ([2, 2], [2, 4]):
        kc = torch.zeros(nb, bs, n_kv, d, dtype=BF, device="cuda")
        vc = torch.zeros_like(kc)
        lens_t = torch.tensor(lens, dtype=torch.int32, device="cuda")
        out = net(query=dev(z[f"in{case}_prefill_query"].reshape(4, -1), BF), key=dev(z[f"in{case}_prefill_key"].reshape(4, -1), BF),
                  value=dev(z[f"in{case}_prefill_value"].reshape(4, -1), BF),
                  slot_mapping=dev(z[f"in{case}_prefill_slot_mapping"].astype(np.int32), torch.int32),
                  block_tables=dev(bt, torch.int32), actual_seq_qlen=lens_t, actual_seq_kvlen=lens_t,
                  batch_valid_length=lens_t, context_lens_tensor=lens_t, attn_mask=mask, key_cache=kc, value_cache=vc)
        res = O.double_benchmark(to_np(out), z[f"gpu_prefill_output_{case}"], z[f"golden_prefill_output_{case}"])
        assert res.ok, (lens, res.messages)
        # the prompt's keys are in the cache afterwards
        slots = z[f"in{case}_prefill_slot_mapping"].astype(np.int64)
        assert np.array_equal(to_np(kc).reshape(nb * bs, -1)[slots], to_np(dev(z[f"in{case}_prefill_key"].reshape(4, -1), BF)))


def test_infer_attention_prefill_chunks_and_decode_agree():
    """InferAttention over a whole prompt (first iteration, TH and BSH), the same prompt fed in chunks through the
    chunk_prefill path, and the oracle, all on the same cache and RoPE tables."""
    from mindformers_amd.modules import FreqsMgr, InferAttention
    rng = np.random.default_rng(5)
    n_head, n_kv, d, bs, nb, seq = 8, 2, 64, 16, 64, 256
    dt = torch.float16
    lens = np.array([40, 23])
    b, t = len(lens), int(lens.sum())
    starts = np.concatenate([[0], np.cumsum(lens)])
    q = rounded(rng.normal(size=(t, n_head * d)), dt)
    k = rounded(rng.normal(size=(t, n_kv * d)), dt)
    v = rounded(rng.normal(size=(t, n_kv * d)), dt)
    pos = np.concatenate([np.arange(n) for n in lens])
    freqs = FreqsMgr(d, seq_length=seq, max_position_embedding=seq, rotary_dtype=dt)
    cos_all, sin_all = freqs.freqs_cos, freqs.freqs_sin
    pos_t = torch.from_numpy(pos).cuda()
    freqs_cis = (cos_all[pos_t].contiguous(), sin_all[pos_t].contiguous(), None)
    tables = np.stack([np.arange(4) + 4 * i for i in range(b)]).astype(np.int32)          # 4 blocks per sequence
    slots = np.concatenate([tables[i][np.arange(n) // bs] * bs + np.arange(n) % bs for i, n in enumerate(lens)]).astype(np.int32)
    scale = 1 / np.sqrt(d)
    q_r = rounded(O.apply_rotary_half(q, to_np(freqs_cis[0]), to_np(freqs_cis[1]), n_head), dt)
    k_r = rounded(O.apply_rotary_half(k, to_np(freqs_cis[0]), to_np(freqs_cis[1]), n_kv), dt)
    ref = O.causal_prefill_attention(q_r, k_r, v, lens, n_head, n_kv, scale)
    mag = O.causal_prefill_attention(q_r, k_r, np.abs(v), lens, n_head, n_kv, scale)

    def make(**kw):
        return InferAttention(n_head, d, n_kv, scale_value=scale, block_size=bs, num_blocks=nb, seq_length=seq,
                              rotary_cos_format=2, compute_dtype=dt, **kw)

    attn = make(is_dynamic=True)
    out = attn(dev(q, dt).reshape(1, t, -1), dev(k, dt).reshape(1, t, -1), dev(v, dt).reshape(1, t, -1),
               torch.from_numpy(lens.astype(np.int32)).cuda(), torch.from_numpy(tables).cuda(),
               torch.from_numpy(slots).cuda(), freqs_cis)
    assert out.shape == (1, t, n_head * d)
    assert_within(to_np(out).reshape(t, -1), ref, mag, dt, ulps=4.0, what="InferAttention prefill (TH)")
    got_k = to_np(attn.paged_attention_mgr.key_cache).reshape(-1, n_kv * d)[slots]
    assert np.abs(got_k - k_r).max() <= 2 * EPS[dt] * np.abs(k_r).max()

    # BSH: one sequence per batch row, equal lengths
    s_len = 23
    rows = np.concatenate([np.arange(starts[i], starts[i] + s_len) for i in range(b)])
    attn_b = make(is_dynamic=False)
    fc = (freqs_cis[0][rows].contiguous(), freqs_cis[1][rows].contiguous(), None)
    out_b = attn_b(dev(q[rows], dt).reshape(b, s_len, -1), dev(k[rows], dt).reshape(b, s_len, -1),
                   dev(v[rows], dt).reshape(b, s_len, -1), torch.full((b,), s_len, dtype=torch.int32, device="cuda"),
                   torch.from_numpy(tables).cuda(), torch.from_numpy(slots[rows]).cuda(), fc)
    assert out_b.shape == (b, s_len, n_head * d)
    assert_within(to_np(out_b).reshape(b * s_len, -1), ref[rows], mag[rows], dt, ulps=4.0, what="InferAttention prefill (BSH)")

    # chunked prefill: 16 new tokens per sequence and call, the cache grows between calls
    attn_c = make(is_dynamic=True, chunk_prefill=True)
    got = np.zeros((t, n_head * d), np.float32)
    done = np.zeros(b, np.int64)
    while (done < lens).any():
        step = np.minimum(16, lens - done)
        rows = np.concatenate([np.arange(starts[i] + done[i], starts[i] + done[i] + step[i]) for i in range(b)])
        done = done + step
        fc = (freqs_cis[0][rows].contiguous(), freqs_cis[1][rows].contiguous(), None)
        o = attn_c(dev(q[rows], dt), dev(k[rows], dt), dev(v[rows], dt), torch.from_numpy(done.astype(np.int32)).cuda(),
                   torch.from_numpy(tables).cuda(), torch.from_numpy(slots[rows]).cuda(), fc,
                   q_seq_lens=torch.from_numpy(step.astype(np.int32)).cuda())
        got[rows] = to_np(o)
    assert_within(got, ref, mag, dt, ulps=4.0, what="InferAttention chunked prefill")


@pytest.mark.parametrize("case,n_kv", [("1", 2), ("2", 1)])
def test_mcore_flash_attention_decode_vectors(golden_dir, case, n_kv):
    """The reference's FlashAttention unit test, decode half (run_infer_flash_attention.py:150-180): caches are
    passed per call, the cell scatters the new K/V and attends."""
    from mindformers_amd import ops
    from mindformers_amd.modules import FlashAttention
    z = np.load(os.path.join(golden_dir, "flash_attention.npz"))
    nb, bs, nh, hid = (int(z[k]) for k in ("meta_num_blocks", "meta_block_size", "meta_num_heads", "meta_hidden_size"))
    d = hid // nh
    net = FlashAttention(head_num=nh, head_dim=d, keep_prob=1.0, kv_head_num=n_kv, pa_kv_head_num=n_kv, scale_value=0.25)
    kc = torch.zeros(nb, bs, n_kv, d, dtype=BF, device="cuda")
    vc = torch.zeros_like(kc)
    ops.reshape_and_cache(dev(z[f"in{case}_prefill_key"].reshape(4, -1), BF), dev(z[f"in{case}_prefill_value"].reshape(4, -1), BF),
                          kc, vc, dev(z[f"in{case}_prefill_slot_mapping"].astype(np.int32), torch.int32))
    net.is_prefill = False
    bt = -np.ones((2, 11), np.int32)
    bt[0, 0], bt[1, 0] = 2, 1
    lens = torch.tensor([3, 3], dtype=torch.int32, device="cuda")
    out = net(query=dev(z[f"in{case}_decoder_query"].reshape(2, -1), BF), key=dev(z[f"in{case}_decoder_key"].reshape(2, -1), BF),
              value=dev(z[f"in{case}_decoder_value"].reshape(2, -1), BF),
              slot_mapping=dev(z[f"in{case}_decoder_slot_mapping"].astype(np.int32), torch.int32),
              block_tables=dev(bt, torch.int32), batch_valid_length=lens, context_lens_tensor=lens, key_cache=kc, value_cache=vc)
    res = O.double_benchmark(to_np(out), z[f"gpu_decode_output_{case}"], z[f"golden_decode_output_{case}"])
    assert res.ok, res.messages


@pytest.mark.parametrize("kind,phase", [("rope", "decode"), ("llama3_rope", "decode"), ("yarn_rope", "decode"), ("rope", "prefill")])
def test_rotary_embedding_module_vectors(golden_dir, kind, phase):
    from mindformers_amd.modules import Llama3RotaryEmbedding, RotaryEmbedding, YaRNScalingRotaryEmbedding
    z = np.load(os.path.join(golden_dir, "rotary.npz"))
    d, max_pos = int(z["meta_kv_channels"]), int(z["meta_max_position_embedding"])
    common = dict(kv_channels=d, rotary_cos_format=2, rotary_dtype=BF)
    if kind == "rope":
        net = RotaryEmbedding(max_position_embeddings=max_pos, **common)
    elif kind == "llama3_rope":
        net = Llama3RotaryEmbedding(max_position_embeddings=max_pos, scaling_factor=8.0, low_freq_factor=1.0,
                                    high_freq_factor=4.0, orig_max_position=512, **common)
    else:
        net = YaRNScalingRotaryEmbedding(scaling_factor=8.0, original_max_position_embeddings=512, beta_fast=32,
                                         beta_slow=1, mscale=1.0, mscale_all_dim=0.0, **common)
    if phase == "decode":
        q, k = dev(z["in_decode_query_for_decode"], BF), dev(z["in_decode_key_for_decode"], BF)
        cos, sin = net.get_cos_sin_for_decode(torch.ones(2, dtype=torch.int32, device="cuda"))
    else:
        q, k = dev(z["in_prefill_query_for_prefill"], BF), dev(z["in_prefill_key_for_prefill"], BF)
        cos, sin = net.get_cos_sin_for_decode(torch.tensor([0, 1, 0, 1], dtype=torch.int32, device="cuda"))
    q, k = net(q, k, cos, sin, None)
    for got, name in ((q, "q"), (k, "k")):
        res = O.double_benchmark(to_np(got), z[f"gpu_{kind}_{name}_emb1_for_{phase}"], z[f"golden_{kind}_{name}_emb1_for_{phase}"])
        assert res.ok, (name, res.messages)


# ------------------------------------------------------------------------------------------- linears / quantizers
def _tiny_model():
    from mindformers_amd.modules import Linear, LlamaRMSNorm
    from torch import nn

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.wq = Linear(256, 512, has_bias=True, compute_dtype=BF, param_init_type=BF)
            self.wo = Linear(512, 256, has_bias=False, compute_dtype=BF, param_init_type=BF)
            self.norm = LlamaRMSNorm(256, eps=1e-5)
            self.lm_head = Linear(256, 1000, has_bias=False, compute_dtype=BF, param_init_type=BF)

        def forward(self, x):
            return self.lm_head(self.wo(self.wq(self.norm(x))))
    return Block()


def test_column_parallel_linear_reference_vectors(golden_dir):
    from mindformers_amd.modules import ColumnParallelLinear, RowParallelLinear
    from mindformers_amd.transformer_config import TransformerConfig
    cfg = TransformerConfig(hidden_size=32, num_attention_heads=2)
    for kind, cls in (("column", ColumnParallelLinear), ("row", RowParallelLinear)):
        z = np.load(os.path.join(golden_dir, f"{kind}_parallel_linear.npz"))
        net = cls(32, 32, config=cfg, bias=True, compute_dtype=BF)
        net.weight.data.copy_(dev(z["in_weight"], BF))
        net.bias.data.copy_(dev(z["in_bias"], BF))
        y = net(dev(z["in_inputs"], BF))
        np.testing.assert_allclose(to_np(y), z["legacy_output_with_bias"], rtol=2 ** -7, atol=1e-6)
    col = ColumnParallelLinear(32, 32, config=cfg, bias=True, skip_weight_param_allocation=True, compute_dtype=BF)
    with pytest.raises(ValueError):
        col(dev(z["in_inputs"], BF))


@pytest.mark.parametrize("method", ["rtn", "ptq_w8a8"])
def test_quantizer_swaps_cells_and_matches_oracle(method):
    """build_network's hook (build_model.py:97-100): AutoQuantizer.from_config(cfg).preprocess_model(net), then
    weights, then postprocess.  lm_head stays float (modules_to_not_convert)."""
    from mindformers_amd.modules import AllQuantLinearInferCell, Linear, WeightQuantLinearCell
    from mindformers_amd.modules.quantizers import AutoQuantizer
    torch.manual_seed(0)
    net = _tiny_model()
    w_q, b_q, w_o = net.wq.weight.data.clone(), net.wq.bias.data.clone(), net.wo.weight.data.clone()
    cfg = {"quant_method": "rtn", "weight_dtype": "int8", "modules_to_not_convert": ["lm_head"]} if method == "rtn" else \
        {"quant_method": "ptq", "weight_dtype": "int8", "activation_dtype": "int8", "act_quant_granularity": "per_token",
         "outliers_suppression": "smooth", "modules_to_not_convert": ["lm_head"]}
    quantizer = AutoQuantizer.from_config(cfg)
    quantizer.preprocess_model(net)
    assert net.is_quantized and net.quantization_method == cfg["quant_method"]
    cell_t = WeightQuantLinearCell if method == "rtn" else AllQuantLinearInferCell
    assert isinstance(net.wq, cell_t) and isinstance(net.wo, cell_t) and isinstance(net.lm_head, Linear)
    assert net.wq.has_act_quant == (method != "rtn") and net.wq.layer.weight.dtype == torch.int8
    quantizer.postprocess_model(net)
    x = rounded(np.random.default_rng(1).normal(size=(7, 256)), BF)
    y = net.wq(dev(x, BF))
    wq_i8, s = O.quantize_weight_int8(w_q.float().cpu().numpy())
    assert np.array_equal(to_np(net.wq.weight), wq_i8) and np.array_equal(to_np(net.wq.w_scale), s)
    b = b_q.float().cpu().numpy()
    if method == "rtn":
        ref = O.w8a16_linear(x, wq_i8, s, b)
    else:
        xq, xs = O.dynamic_quant_per_token(x, np.ones(256, np.float32))
        ref = O.w8a8_linear(xq, xs, wq_i8, s, b)
    assert_within(to_np(y), ref, np.abs(ref) + np.abs(b), BF, ulps=1.0, extra=1e-5, what="quant cell")
    out = net(dev(x, BF))
    assert out.shape == (7, 1000) and torch.isfinite(out.float()).all()


@pytest.mark.parametrize("granularity,group,suppression", [("per_channel", 0, "None"), ("per_group", 64, "None"),
                                                           ("per_group", 128, "awq")])
def test_quantizer_builds_four_bit_weight_only_cells(granularity, group, suppression):
    """A16W4 (weight_dtype int4 -> qint4x2, quantization_config.py:33, :408-416), per channel or per group, with the
    awq multiplier on the activations: the quantizer swaps in 4-bit WeightQuantLinearCells whose buffers hold two
    values per byte and a scale table [in / group, out]; a checkpoint round trip (state_dict -> fresh cells) gives
    the same output; the output equals the oracle's group-wise integer matmul."""
    from mindformers_amd.modules import Linear, WeightQuantLinearCell
    from mindformers_amd.modules.quantizers import AutoQuantizer
    torch.manual_seed(0)
    net = _tiny_model()
    w_q, b_q = net.wq.weight.data.clone(), net.wq.bias.data.clone()
    cfg = {"quant_method": "ptq", "weight_dtype": "int4", "weight_quant_granularity": granularity, "group_size": group,
           "outliers_suppression": suppression, "modules_to_not_convert": ["lm_head"]}
    quantizer = AutoQuantizer.from_config(cfg)
    quantizer.preprocess_model(net)
    assert isinstance(net.wq, WeightQuantLinearCell) and isinstance(net.lm_head, Linear)
    assert net.wq.weight_bits == 4 and net.wq.group_size == group
    assert net.wq.weight.shape == (512, 128) and net.wq.weight.dtype == torch.int8
    assert net.wq.w_scale.shape == ((512,) if group == 0 else (256 // group, 512))
    rng = np.random.default_rng(3)
    smooth = None
    if suppression == "awq":
        smooth = rng.uniform(0.5, 2.0, 256).astype(np.float32)
        net.wq.smooth_scale.copy_(torch.from_numpy(smooth))
    else:
        assert net.wq.smooth_scale is None
    quantizer.postprocess_model(net)
    x = rounded(rng.normal(size=(7, 256)), BF)
    y = net.wq(dev(x, BF))
    wq_i4, s = O.quantize_weight_int4(w_q.float().cpu().numpy(), group)
    assert np.array_equal(to_np(net.wq.weight), O.pack_qint4x2(wq_i4)) and np.array_equal(to_np(net.wq.w_scale), s)
    b = b_q.float().cpu().numpy()
    xs = rounded(x * smooth[None, :], BF) if smooth is not None else x
    ref = O.w4a16_linear(xs, wq_i4, s, group, b)
    assert_within(to_np(y), ref, np.abs(ref) + np.abs(b), BF, ulps=1.0, extra=1e-5, what="4-bit cell")
    # the deploy checkpoint carries the packed bytes and the scale table: fresh cells loaded from it agree bit for bit
    fresh = _tiny_model()
    q2 = AutoQuantizer.from_config(cfg)
    q2.preprocess_model(fresh)
    fresh.load_state_dict(net.state_dict())
    q2.postprocess_model(fresh)
    assert torch.equal(fresh.wq(dev(x, BF)), y)
    out = net(dev(x, BF))
    assert out.shape == (7, 1000) and torch.isfinite(out.float()).all()


def test_smooth_quant_method_converts_to_static_per_tensor_cells():
    """The SmoothQuant method (A8W8, static per-tensor activations, smooth multiplier): the quantizer swaps in
    AllQuantLinearInferCell(act_quant_granularity="per_tensor"); with a calibrated scale and multiplier loaded, the
    cell equals the oracle's static quantisation followed by the exact int8 GEMM."""
    from mindformers_amd.modules import AllQuantLinearInferCell, Linear
    from mindformers_amd.modules.quantizers import AutoQuantizer, SmoothQuantQuantizer
    torch.manual_seed(0)
    net = _tiny_model()
    w_q, b_q = net.wq.weight.data.clone(), net.wq.bias.data.clone()
    q = AutoQuantizer.from_config({"quant_method": "smooth_quant", "modules_to_not_convert": ["lm_head"]})
    assert isinstance(q, SmoothQuantQuantizer)
    q.preprocess_model(net)
    assert isinstance(net.wq, AllQuantLinearInferCell) and net.wq.act_quant_granularity == "per_tensor"
    assert isinstance(net.lm_head, Linear) and net.wq.act_scale.shape == (1,)
    rng = np.random.default_rng(2)
    smooth = rng.uniform(0.5, 2.0, 256).astype(np.float32)
    net.wq.smooth_scale.copy_(torch.from_numpy(smooth))
    net.wq.act_scale.fill_(0.03)
    q.postprocess_model(net)
    x = rounded(rng.normal(size=(9, 256)), BF)
    y = net.wq(dev(x, BF))
    wq_i8, s = O.quantize_weight_int8(w_q.float().cpu().numpy())
    xq, xs = O.static_quant_per_tensor(x, np.float32(0.03), smooth)
    assert (np.abs(xq.astype(np.int32)) == 127).any() or (xq == -128).any()       # the rails are reached
    b = b_q.float().cpu().numpy()
    ref = O.w8a8_linear(xq, xs, wq_i8, s, b)
    assert_within(to_np(y), ref, np.abs(ref) + np.abs(b), BF, ulps=1.0, extra=1e-5, what="static per-tensor cell")


# ------------------------------------------------------------------------------------------- norm / mlp
def test_rmsnorm_cells(golden_dir):
    from mindformers_amd.modules import LlamaRMSNorm, RMSNorm
    from mindformers_amd.transformer_config import TransformerConfig
    z = np.load(os.path.join(golden_dir, "norm.npz"))
    cfg = TransformerConfig(hidden_size=32, layernorm_compute_dtype="bfloat16")
    for name, eps in (("rmsnorm_output1", 1e-5), ("rmsnorm_output2", 0.1)):
        for net in (RMSNorm(cfg, hidden_size=32, eps=eps), LlamaRMSNorm(32, eps=eps, compute_type=BF)):
            net.weight.data.copy_(dev(z["in_weight"], BF))
            res = O.double_benchmark(to_np(net(dev(z["in_input"], BF))), z[f"gpu_{name}"], z[f"golden_{name}"])
            assert res.ok, (name, res.messages)


@pytest.mark.parametrize("name,bias", [("has_bias_gate_output", True), ("has_gate_output", False)])
def test_mcore_mlp_reference_vectors(golden_dir, name, bias):
    """test_infer_mlp.py:35-61 gated cases through the float cells (library GEMM + HIP silu*mul)."""
    from mindformers_amd.modules import MLP
    from mindformers_amd.transformer_config import TransformerConfig
    z = np.load(os.path.join(golden_dir, "mlp.npz"))
    cfg = TransformerConfig(hidden_size=32, ffn_hidden_size=32, num_attention_heads=2, add_bias_linear=bias,
                            gated_linear_unit=True, hidden_act="silu")
    net = MLP(cfg)
    net.linear_fc1.weight.data.copy_(dev(z["in_fc1_gate_weight"], BF))
    net.linear_fc2.weight.data.copy_(dev(z["in_fc2_weight"], BF))
    if bias:
        net.linear_fc1.bias.data.copy_(dev(z["in_fc1_gate_bias"], BF))
        net.linear_fc2.bias.data.copy_(dev(z["in_fc2_bias"], BF))
    res = O.double_benchmark(to_np(net(dev(z["in_input"], BF))), z[f"gpu_{name}"], z[f"golden_{name}"])
    assert res.ok, res.messages


def test_llama_feed_forward_layouts():
    """ffn_concat's interleaved (ffn, 2) layout and the separate w1/w3 layout give the same function."""
    from mindformers_amd.modules import LlamaFeedForward
    torch.manual_seed(1)
    a = LlamaFeedForward(64, intermediate_size=96, compute_dtype=BF, param_init_type=BF, ffn_concat=False)
    b = LlamaFeedForward(64, intermediate_size=96, compute_dtype=BF, param_init_type=BF, ffn_concat=True)
    wgh = torch.empty(192, 64, dtype=BF, device="cuda")
    wgh[0::2], wgh[1::2] = a.w1.weight.data, a.w3.weight.data
    b.w_gate_hidden.weight.data.copy_(wgh)
    b.w2.weight.data.copy_(a.w2.weight.data)
    x = torch.randn(5, 64, device="cuda").to(BF)
    assert torch.equal(a(x), b(x))
    ref = O.mlp(to_np(x), np.concatenate([to_np(a.w1.weight), to_np(a.w3.weight)]), to_np(a.w2.weight), gated=True, act_dtype="bf16")
    assert np.abs(to_np(a(x)) - ref).max() <= 4 * EPS[BF] * np.abs(ref).max() + 1e-6


# ------------------------------------------------------------------------------------------- MoE layer
def _moe_config(shared):
    from mindformers_amd.transformer_config import TransformerConfig
    return TransformerConfig(num_layers=1, num_attention_heads=8, hidden_size=32, hidden_act="silu", num_moe_experts=8,
                             moe_router_topk=2, shared_expert_num=1, moe_router_topk_scaling_factor=2.5,
                             moe_shared_expert_intermediate_size=8 if shared else 0, moe_ffn_hidden_size=8,
                             moe_router_group_topk=2, moe_router_num_groups=2, add_bias_linear=False,
                             gated_linear_unit=True, compute_dtype="bfloat16", params_dtype="bfloat16",
                             moe_router_dtype="bfloat16", moe_router_enable_expert_bias=True,
                             moe_router_score_function="sigmoid")


def _load_moe(net, z, shared):
    net.router.weight.data.copy_(dev(z["in_router__weight__weight"], BF))
    net.router.expert_bias.data.copy_(dev(z["in_router__expert_bias"], torch.float32))
    net.experts.weight1.data.copy_(dev(z["in_experts__weight1"], BF))
    net.experts.weight2.data.copy_(dev(z["in_experts__weight2"], BF))
    if shared:
        net.shared_experts.linear_fc1.weight.data.copy_(dev(z["in_shared_experts__linear_fc1__weight"], BF))
        net.shared_experts.linear_fc2.weight.data.copy_(dev(z["in_shared_experts__linear_fc2__weight"], BF))


@pytest.mark.parametrize("name,shared", [("tp1", True), ("tp1_no_shared", False)])
def test_moe_layer_reference_vectors(golden_dir, name, shared):
    """test_infer_moe.py:31-58 through MoELayer with float experts.  The reference's own bound is rtol 4e-3
    (:132-140), which is below one bf16 ulp (2^-8..2^-7 relative); the float expert GEMMs here go through the BLAS
    library, whose summation order differs, so the bound here is one bf16 ulp (2^-7) and at most 1 % of the
    elements may be outside the reference's 4e-3."""
    from mindformers_amd.modules import MoELayer
    z = np.load(os.path.join(golden_dir, "moe.npz"))
    net = MoELayer(_moe_config(shared))
    assert (net.shared_experts is not None) == shared
    _load_moe(net, z, shared)
    out = net(dev(z["in_input"], BF))
    got = to_np(out).astype(np.float16).astype(np.float32)
    gold = z[f"golden_{name}"].astype(np.float32)
    np.testing.assert_allclose(got, gold, rtol=2.0 ** -7, atol=2e-6)
    assert np.mean(np.abs(got - gold) > 4e-3 * np.abs(gold) + 2e-6) <= 0.01


def test_moe_layer_quantized_experts_vs_oracle(golden_dir):
    """The same layer after the RTN quantizer (W8A16 experts, shared expert and all linears): compared with the
    oracle evaluated on the dequantised weights, so only kernel arithmetic is in the tolerance."""
    from mindformers_amd.modules import MoELayer, QuantGroupedMLP, WeightQuantLinearCell
    from mindformers_amd.modules.quantizers import AutoQuantizer
    z = np.load(os.path.join(golden_dir, "moe.npz"))
    net = MoELayer(_moe_config(True))
    _load_moe(net, z, True)
    q = AutoQuantizer.from_config({"quant_method": "rtn", "weight_dtype": "int8"})
    q.preprocess_model(net)
    q.postprocess_model(net)
    assert isinstance(net.experts, QuantGroupedMLP) and isinstance(net.shared_experts.linear_fc1, WeightQuantLinearCell)
    x = rounded(z["in_input"], BF)
    out = to_np(net(dev(x, BF)))
    deq1 = (to_np(net.experts.weight1).astype(np.float64) * to_np(net.experts.w1_scale)[..., None]).transpose(0, 2, 1)
    deq2 = (to_np(net.experts.weight2).astype(np.float64) * to_np(net.experts.w2_scale)[..., None]).transpose(0, 2, 1)
    sf1 = to_np(net.shared_experts.linear_fc1.weight).astype(np.float64) * to_np(net.shared_experts.linear_fc1.w_scale)[:, None]
    sf2 = to_np(net.shared_experts.linear_fc2.weight).astype(np.float64) * to_np(net.shared_experts.linear_fc2.w_scale)[:, None]
    ref = O.moe_layer(x, rounded(z["in_router__weight__weight"], BF), z["in_router__expert_bias"].astype(np.float32), deq1, deq2,
                      k=2, n_group=2, topk_group=2, scale=2.5, shared_fc1=sf1, shared_fc2=sf2, act_dtype="bf16",
                      router_dtype="bf16")
    assert np.abs(out - ref).max() <= 6 * EPS[BF] * np.abs(ref).max()


def test_router_plain_topk_branch():
    """moe_router_group_topk unset: biased scores are normalised and returned without scaling (router.py:142-146)."""
    from mindformers_amd.modules import TopKRouter
    from mindformers_amd.transformer_config import TransformerConfig
    cfg = TransformerConfig(hidden_size=64, num_moe_experts=16, moe_router_topk=4, moe_router_dtype="float32",
                            moe_router_enable_expert_bias=True)
    r = TopKRouter(cfg)
    r.expert_bias.data.normal_(0, 0.1)
    x = torch.randn(9, 64, device="cuda").to(BF)
    w, idx = r(x)
    logits = to_np(x).astype(np.float64) @ to_np(r.weight).astype(np.float64).T
    sb = 1 / (1 + np.exp(-logits)) + to_np(r.expert_bias)
    ref_idx = np.argsort(-sb, axis=1, kind="stable")[:, :4]
    assert np.array_equal(to_np(idx), ref_idx)
    ref_w = np.take_along_axis(sb, ref_idx, 1)
    ref_w /= ref_w.sum(1, keepdims=True)
    assert np.abs(to_np(w) - ref_w).max() <= EPS[BF] * 1.01 * ref_w.max() + 1e-6


# ------------------------------------------------------------------------------------------- whole layer
@pytest.mark.parametrize("name", ["tiny_llama_w8a16"])
def test_decode_layer_matches_oracle(name):
    """The reference's CPU-runnable configuration, full layer, against the oracle composition."""
    from mindformers_amd import synthetic
    case = synthetic.make_decode_case(name, seed=3)
    cfg, layer = case["cfg"], case["layers"][0]
    kc, vc = case["caches"][0]
    kc0, vc0 = to_np(kc), to_np(vc)
    out = layer(case["x"], kc, vc, case["block_tables"], case["context_lens"], case["slot_mapping"], case["cos"], case["sin"])
    p = {}
    for n in layer.NAMES:
        p[n + "_w"], p[n + "_s"] = to_np(getattr(layer, n + "_w")), to_np(getattr(layer, n + "_s"))
    p["attn_norm"], p["ffn_norm"] = to_np(layer.attn_norm), to_np(layer.ffn_norm)
    ref = O.decode_layer_w8a16(to_np(case["x"]), p, dict(n_head=cfg["n_head"], n_kv_head=cfg["n_kv_head"],
                                                       head_dim=cfg["head_dim"], eps=1e-5), kc0, vc0,
                               to_np(case["block_tables"]), case["context_lens_host"], to_np(case["slot_mapping"]),
                               to_np(case["cos"]), to_np(case["sin"]), act_dtype="fp16")
    got = to_np(out)
    tol = 8 * EPS[torch.float16] * np.maximum(np.abs(ref), 0.05 * np.abs(ref).max(axis=1, keepdims=True)) + 1e-4
    assert np.all(np.abs(got - ref) <= tol), np.abs(got - ref).max()


def test_decode_layer_w8a8_matches_oracle():
    """Qwen2.5-shaped W8A8 layer at reduced width (heads 7q/1kv x 128, hidden 896, ffn 1024), batch 5."""
    from mindformers_amd import synthetic
    from mindformers_amd.decode_layer import QuantDecodeLayer
    torch.manual_seed(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    layer = synthetic.fill_layer(QuantDecodeLayer(896, 7, 1, 128, 1024, 1e-5, BF, act_quant=True), gen)
    rng = np.random.default_rng(9)
    b, bs = 5, 128
    lens = rng.integers(100, 700, b)
    kc0, vc0, tables, nb = make_paged_cache(rng, b, lens, 1, 128, bs, BF)
    kc, vc = dev(kc0, BF), dev(vc0, BF)
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    x = rounded(rng.normal(size=(b, 896)), BF)
    lens_t = torch.from_numpy(lens.astype(np.int32)).cuda()
    cos, sin = synthetic.rope_rows(lens_t - 1, 128, 1e6, BF, "cuda")
    out = layer(dev(x, BF), kc, vc, torch.from_numpy(tables).cuda(), lens_t, torch.from_numpy(slots).cuda(), cos, sin)
    p = {}
    for n in layer.NAMES:
        p[n + "_w"], p[n + "_s"] = to_np(getattr(layer, n + "_w")), to_np(getattr(layer, n + "_s"))
        p[n + "_smooth"] = to_np(getattr(layer, n + "_smooth"))
    p["attn_norm"], p["ffn_norm"] = to_np(layer.attn_norm), to_np(layer.ffn_norm)
    ref = O.decode_layer_w8a8(x, p, dict(n_head=7, n_kv_head=1, head_dim=128, eps=1e-5), kc0, vc0, tables, lens, slots,
                              to_np(cos), to_np(sin), act_dtype="bf16")
    got = to_np(out)
    # int8 activation grids amplify one-step differences of the bf16 intermediates: compare at row scale
    tol = 16 * EPS[BF] * np.maximum(np.abs(ref), 0.1 * np.abs(ref).max(axis=1, keepdims=True)) + 1e-3
    frac_bad = np.mean(np.abs(got - ref) > tol)
    assert frac_bad < 0.002, (frac_bad, np.abs(got - ref).max())


def test_decode_layer_graph_replay_is_bit_identical():
    """A captured HIP graph of the layer step must reproduce the eager result on every replay, with eager work
    and synchronisations in between."""
    from mindformers_amd import synthetic
    case = synthetic.make_decode_case("tiny_llama_w8a16", seed=4)
    layer = case["layers"][0]
    kc, vc = case["caches"][0]
    args = (case["x"], kc, vc, case["block_tables"], case["context_lens"], case["slot_mapping"], case["cos"], case["sin"])
    eager = layer(*args).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            layer(*args)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = layer(*args)
    for _ in range(4):
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        layer(*args)
        torch.cuda.synchronize()


@pytest.mark.parametrize("act_quant", [False, True])
def test_chained_layers_are_bit_identical_to_separate_ones(act_quant):
    """Layer i computing layer i + 1's attention norm (inside the kernel that finishes its last projection on the
    W8A16 path) must give the bits of every layer computing its own."""
    from mindformers_amd import synthetic
    from mindformers_amd.decode_layer import QuantDecodeLayer
    case = synthetic.make_decode_case("tiny_llama_w8a16", seed=6)
    layer = case["layers"][0]
    if act_quant:
        gen = torch.Generator(device="cuda")
        gen.manual_seed(9)
        layer = synthetic.fill_layer(QuantDecodeLayer(layer.hidden, layer.n_head, layer.n_kv_head, layer.head_dim,
                                                      layer.ffn, layer.eps, layer.dtype, act_quant=True), gen)
    rest = (case["block_tables"], case["context_lens"], case["slot_mapping"], case["cos"], case["sin"])
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    gammas = [torch.rand(layer.hidden, generator=gen, device="cuda") + 0.5 for _ in range(3)]

    def run(chained):
        kc, vc = (c.clone() for c in case["caches"][0])
        h, normed = case["x"], None
        for i in range(3):                                    # the same weights three times, a norm weight per level
            layer.attn_norm.copy_(gammas[i])
            if chained:
                nn = (gammas[(i + 1) % 3], layer.eps) + ((layer.qkv_smooth,) if act_quant else ())
                h, normed = layer(h, kc, vc, *rest, normed=normed, next_norm=nn)
            else:
                h = layer(h, kc, vc, *rest)
        return h, normed, kc, vc

    h0, _, kc0, vc0 = run(False)
    h1, n1, kc1, vc1 = run(True)
    assert torch.equal(h0, h1) and torch.equal(kc0, kc1) and torch.equal(vc0, vc1)
    from mindformers_amd import ops
    if act_quant:
        xq, xs = ops.rms_norm_dynamic_quant(h0, gammas[0], layer.eps, layer.qkv_smooth, tiled=True)
        rows, width = h0.shape
        assert np.array_equal(untile_int8(to_np(n1[0].data), rows, width), untile_int8(to_np(xq.data), rows, width))
        assert torch.equal(n1[1], xs)
    else:
        assert torch.equal(n1, ops.rms_norm(h0, gammas[0], layer.eps))


# ------------------------------------------------------------------------------------------- checkpoint -> layer
@pytest.mark.parametrize("fmt", ["hf_float", "mg_fused_float", "int8_with_scales"])
def test_layer_loaded_from_a_checkpoint_matches_oracle(tmp_path, fmt):
    """A decode layer built from a safetensors checkpoint (HuggingFace names with float weights, the reference's
    fused per-kv-group / interleaved layouts, or pre-quantized int8 + w_scale) runs the same step as the oracle on
    the weights quantized with the declared convention."""
    from safetensors.numpy import save_file
    from mindformers_amd import checkpoint as C, synthetic
    rng = np.random.default_rng(13)
    nh, nkv, d, ffn, layer_idx = 8, 2, 64, 1024, 2
    hidden = nh * d
    cfg = dict(num_heads=nh, n_kv_heads=nkv, hidden_size=hidden, intermediate_size=ffn, qkv_concat=False)
    p = f"model.layers.{layer_idx}."
    hf = {}
    for name, shape in (("self_attn.q_proj", (hidden, hidden)), ("self_attn.k_proj", (nkv * d, hidden)),
                        ("self_attn.v_proj", (nkv * d, hidden)), ("self_attn.o_proj", (hidden, hidden)),
                        ("mlp.gate_proj", (ffn, hidden)), ("mlp.up_proj", (ffn, hidden)), ("mlp.down_proj", (hidden, ffn))):
        hf[p + name + ".weight"] = rng.normal(0, 0.03, shape).astype(np.float32)
    hf[p + "input_layernorm.weight"] = rng.normal(1, 0.1, hidden).astype(np.float32)
    hf[p + "post_attention_layernorm.weight"] = rng.normal(1, 0.1, hidden).astype(np.float32)
    ref_arrays = C.read_layer_arrays(hf, layer_idx, cfg)
    if fmt == "hf_float":
        path = str(tmp_path / "model.safetensors")
        save_file(hf, path)
    elif fmt == "mg_fused_float":
        src = tmp_path / "hf"
        src.mkdir()
        save_file(hf, str(src / "model.safetensors"))
        path = str(tmp_path / "mg")
        C.convert_hf_safetensors_multiprocess(str(src), path, None, dict(cfg, qkv_concat=True))
    else:
        q = {}
        for k, v in C.convert_weight_dict(hf, cfg).items():
            if v.ndim == 2:
                q[k], q[k[:-len("weight")] + "w_scale"] = C.quantize_rtn_int8(v)
            else:
                q[k] = v
        path = str(tmp_path / "int8.safetensors")
        save_file(q, path)
    layer = C.load_decode_layer(path, layer_idx, cfg, dtype=BF)
    pr = {}
    for n in layer.NAMES:
        pr[n + "_w"], pr[n + "_s"] = O.quantize_weight_int8(ref_arrays[n][0])
        assert np.array_equal(to_np(getattr(layer, n + "_w")), pr[n + "_w"]), n
        assert np.array_equal(to_np(getattr(layer, n + "_s")), pr[n + "_s"]), n
    pr["attn_norm"], pr["ffn_norm"] = ref_arrays["attn_norm"], ref_arrays["ffn_norm"]
    b, bs = 3, 16
    lens = rng.integers(20, 90, b)
    kc0, vc0, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, BF)
    kc, vc = dev(kc0, BF), dev(vc0, BF)
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    x = rounded(rng.normal(size=(b, hidden)), BF)
    lens_t = torch.from_numpy(lens.astype(np.int32)).cuda()
    cos, sin = synthetic.rope_rows(lens_t - 1, d, 1e4, BF, "cuda")
    out = layer(dev(x, BF), kc, vc, torch.from_numpy(tables).cuda(), lens_t, torch.from_numpy(slots).cuda(), cos, sin)
    ref = O.decode_layer_w8a16(x, pr, dict(n_head=nh, n_kv_head=nkv, head_dim=d, eps=1e-5), kc0, vc0, tables, lens, slots,
                               to_np(cos), to_np(sin), act_dtype="bf16")
    got = to_np(out)
    tol = 8 * EPS[BF] * np.maximum(np.abs(ref), 0.05 * np.abs(ref).max(axis=1, keepdims=True)) + 1e-4
    assert np.all(np.abs(got - ref) <= tol), np.abs(got - ref).max()


@pytest.mark.parametrize("with_offset", [False, True])
def test_decode_layer_with_int8_kv_cache_matches_oracle(with_offset):
    """The W8A16 layer over int8 caches: the new K/V rows are rotated, quantised per channel and scattered, the
    attention reads the int8 cache; against the oracle layer with the same quantisation convention."""
    from mindformers_amd import synthetic
    from mindformers_amd.decode_layer import QuantDecodeLayer
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    hidden, nh, nkv, d, ffn, bs = 1024, 8, 2, 128, 1536, 128
    layer = synthetic.fill_layer(QuantDecodeLayer(hidden, nh, nkv, d, ffn, 1e-5, BF), gen)
    rng = np.random.default_rng(17)
    b = 4
    lens = rng.integers(100, 900, b)
    kc_f, vc_f, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, BF)
    row = nkv * d
    scale = np.stack([np.full(row, 4.5 / 127), np.full(row, 4.5 / 127)]).astype(np.float32)
    scale *= rng.uniform(0.8, 1.2, scale.shape).astype(np.float32)
    offset = rng.integers(-10, 11, (2, row)).astype(np.float32) if with_offset else None
    ko, vo = (None, None) if offset is None else (offset[0], offset[1])
    k8 = O.quantize_kv_int8(kc_f.reshape(-1, row), scale[0], ko).reshape(kc_f.shape)
    v8 = O.quantize_kv_int8(vc_f.reshape(-1, row), scale[1], vo).reshape(vc_f.shape)
    layer.set_kv_quant(dev(scale, torch.float32), None if offset is None else dev(offset, torch.float32))
    kc, vc = torch.from_numpy(k8).cuda(), torch.from_numpy(v8).cuda()
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    x = rounded(rng.normal(size=(b, hidden)), BF)
    lens_t = torch.from_numpy(lens.astype(np.int32)).cuda()
    cos, sin = synthetic.rope_rows(lens_t - 1, d, 1e4, BF, "cuda")
    out = layer(dev(x, BF), kc, vc, torch.from_numpy(tables).cuda(), lens_t, torch.from_numpy(slots).cuda(), cos, sin)
    p = {}
    for n in layer.NAMES:
        p[n + "_w"], p[n + "_s"] = to_np(getattr(layer, n + "_w")), to_np(getattr(layer, n + "_s"))
    p["attn_norm"], p["ffn_norm"] = to_np(layer.attn_norm), to_np(layer.ffn_norm)
    k8_ref, v8_ref = k8.copy(), v8.copy()
    ref = O.decode_layer_w8a16(x, p, dict(n_head=nh, n_kv_head=nkv, head_dim=d, eps=1e-5), k8_ref, v8_ref, tables, lens,
                               slots, to_np(cos), to_np(sin), act_dtype="bf16", kv_quant=(scale, offset))
    got = to_np(out)
    tol = 8 * EPS[BF] * np.maximum(np.abs(ref), 0.05 * np.abs(ref).max(axis=1, keepdims=True)) + 1e-4
    assert np.all(np.abs(got - ref) <= tol), np.abs(got - ref).max()
    # the new rows in the int8 caches: equal to the oracle's up to one quantisation step where the rotated key
    # differs by a rounding of the compute dtype
    got_k = kc.cpu().numpy().reshape(-1, row)[slots].astype(np.int32)
    ref_k = k8_ref.reshape(-1, row)[slots].astype(np.int32)
    assert np.abs(got_k - ref_k).max() <= 1 and (got_k != ref_k).mean() < 0.05
    assert np.array_equal(vc.cpu().numpy().reshape(-1, row)[slots], v8_ref.reshape(-1, row)[slots]) or \
        (np.abs(vc.cpu().numpy().reshape(-1, row)[slots].astype(np.int32) - v8_ref.reshape(-1, row)[slots]).max() <= 1)


def test_mcore_flash_attention_mla_decode_branch():
    """FlashAttention(pa_mla_v_dim=512): the decode call of MLASelfAttention (multi_latent_attention.py:212-228):
    the caller has written the latent row with reshape_and_cache(key, None, cache, None, slots); the cell attends
    with the cache as keys and values."""
    from mindformers_amd import ops
    from mindformers_amd.modules import FlashAttention
    rng = np.random.default_rng(19)
    nh, bs = 32, 32
    lens = np.array([70, 300, 33])
    cache, _, tables, nb = make_paged_cache(rng, 3, lens, 1, 576, bs, BF)
    net = FlashAttention(head_num=nh, head_dim=576, kv_head_num=1, pa_kv_head_num=1, scale_value=0.072, pa_mla_v_dim=512)
    net.is_prefill = False
    assert net.use_multi_latent_attention
    q = rounded(rng.normal(size=(3, nh * 576)), BF)
    new = rounded(rng.normal(size=(3, 576)), BF)
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    cd = dev(cache, BF)
    ops.reshape_and_cache(dev(new, BF), None, cd, None, dev(slots, torch.int32))
    cache.reshape(-1, 576)[slots] = new
    lens_t = torch.from_numpy(lens.astype(np.int32)).cuda()
    out = net(query=dev(q, BF), key=None, value=None, slot_mapping=dev(slots, torch.int32),
              block_tables=dev(tables, torch.int32), batch_valid_length=lens_t, key_cache=cd, value_cache=None)
    assert out.shape == (3, nh * 512)
    ref = O.mla_paged_attention_decode(q, cache, tables, lens, nh, 512, 0.072)
    mag = O.mla_paged_attention_decode(q, cache, tables, lens, nh, 512, 0.072, abs_values=True)
    assert_within(to_np(out), ref, mag, BF, ulps=1.5, what="FlashAttention MLA decode")


def test_mcore_flash_attention_mla_prefill_branch():
    """FlashAttention(pa_mla_v_dim=512) in prefill: MLASelfAttention hands over 192-wide queries, keys (the
    up-projected 128 dimensions of every head followed by the shared rotary 64) and values (128 dimensions padded
    with the same rotary 64), and keeps the first v_head_dim columns of every head of the result
    (multi_latent_attention.py:405-432, 208-218).  The latent cache is the caller's to write and is not touched."""
    from mindformers_amd.modules import FlashAttention
    rng = np.random.default_rng(31)
    nh, qk, rope, vd = 16, 128, 64, 128
    q_lens = np.array([150, 1, 37, 260])
    t = int(q_lens.sum())
    scale = 1.0 / np.sqrt(qk + rope)
    net = FlashAttention(head_num=nh, head_dim=qk + rope, kv_head_num=nh, scale_value=scale, next_tokens=0,
                         pa_kv_head_num=1, pa_mla_v_dim=512)
    assert net.is_prefill and net.use_multi_latent_attention
    q = rounded(rng.normal(size=(t, nh, qk + rope)), BF)
    k_pe = np.repeat(rounded(rng.normal(size=(t, 1, rope)), BF), nh, axis=1)
    k = np.concatenate([rounded(rng.normal(size=(t, nh, qk)), BF), k_pe], axis=-1)
    v = np.concatenate([rounded(rng.normal(size=(t, nh, vd)), BF), k_pe], axis=-1)
    cache = torch.full((4, 32, 1, 576), 7.0, dtype=BF, device="cuda")
    ends = torch.from_numpy(np.cumsum(q_lens).astype(np.int32)).cuda()
    out = net(query=dev(q.reshape(t, -1), BF), key=dev(k.reshape(t, -1), BF), value=dev(v.reshape(t, -1), BF),
              slot_mapping=None, actual_seq_qlen=ends, actual_seq_kvlen=ends, key_cache=cache, value_cache=None)
    assert out.shape == (t, nh * (qk + rope))
    assert bool((cache == 7.0).all())
    ref = O.causal_prefill_attention(q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1), q_lens, nh, nh, scale)
    mag = O.causal_prefill_attention(q.reshape(t, -1), k.reshape(t, -1), np.abs(v.reshape(t, -1)), q_lens, nh, nh, scale)
    assert_within(to_np(out), ref, mag, BF, ulps=1.5, what="FlashAttention MLA prefill")
    kept = to_np(out).reshape(t, nh, qk + rope)[:, :, :vd]        # what MLASelfAttention passes to linear_proj
    assert_within(kept, ref.reshape(t, nh, -1)[:, :, :vd], mag.reshape(t, nh, -1)[:, :, :vd], BF, ulps=1.5,
                  what="MLA prefill, v_head_dim columns")


def test_mcore_flash_attention_mla_decode_with_q_seq_lens():
    """MLA decode with several new tokens per sequence (q_seq_lens: parallel decoding / chunked prefill,
    flash_attention.py:140-143): every query row sees the latent cache up to its own position; a sequence without new
    tokens contributes no rows."""
    from mindformers_amd.modules import FlashAttention
    rng = np.random.default_rng(29)
    nh, bs = 16, 32
    lens = np.array([70, 300, 33, 129])
    q_lens = np.array([3, 1, 0, 5])
    cache, _, tables, nb = make_paged_cache(rng, 4, lens, 1, 576, bs, BF)
    net = FlashAttention(head_num=nh, head_dim=576, kv_head_num=1, pa_kv_head_num=1, scale_value=0.072, pa_mla_v_dim=512)
    net.is_prefill = False
    rows = int(q_lens.sum())
    q = rounded(rng.normal(size=(rows, nh * 576)), BF)
    out = net(query=dev(q, BF), key=None, value=None, slot_mapping=None, block_tables=dev(tables, torch.int32),
              batch_valid_length=torch.from_numpy(lens.astype(np.int32)).cuda(),
              q_seq_lens=torch.from_numpy(q_lens.astype(np.int32)).cuda(), key_cache=dev(cache, BF), value_cache=None)
    assert out.shape == (rows, nh * 512)
    seq = np.repeat(np.arange(4), q_lens)
    limit = np.concatenate([np.arange(l - ql + 1, l + 1) for l, ql in zip(lens, q_lens)])
    ref = O.mla_paged_attention_decode(q, cache, tables[seq], limit, nh, 512, 0.072)
    mag = O.mla_paged_attention_decode(q, cache, tables[seq], limit, nh, 512, 0.072, abs_values=True)
    assert_within(to_np(out), ref, mag, BF, ulps=1.5, what="FlashAttention MLA decode, several tokens per sequence")


# ------------------------------------------------------------------------------------------- kvcache_dtype: int8
@pytest.mark.parametrize("dynamic", [True, False])
def test_quantizer_swaps_in_the_int8_kv_manager_and_decode_matches_oracle(dynamic):
    """`kvcache_dtype: int8` in the quantization config (quantization_config.py:196-254) makes the quantizer replace
    the attention's cache manager by one that owns int8 caches; the InferAttention decode call then rotates,
    quantises and scatters the new rows and attends over the int8 cache with the manager's dequantisation
    parameters - against the oracle's RoPE -> quantising scatter -> attention over the dequantised cache."""
    from torch import nn
    from mindformers_amd.modules import FreqsMgr, InferAttention, Linear, PagedAttentionMgr, QuantPagedAttentionMgr
    from mindformers_amd.modules.quantizers import AutoQuantizer
    rng = np.random.default_rng(5)
    b, n_head, n_kv, d, bs, seq = 3, 8, 2, 64, 16, 512
    dt = torch.float16
    lens = rng.integers(30, 300, b)
    kc_f, vc_f, tables, nb = make_paged_cache(rng, b, lens, n_kv, d, bs, dt, max_blocks=seq // bs)

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.wq = Linear(256, n_head * d, has_bias=False, compute_dtype=dt)
            self.infer_attention = InferAttention(n_head, d, n_kv, scale_value=1 / np.sqrt(d), block_size=bs,
                                                  num_blocks=nb, seq_length=seq, is_dynamic=dynamic, rotary_cos_format=2,
                                                  compute_dtype=dt)
    net = Block()
    assert type(net.infer_attention.paged_attention_mgr) is PagedAttentionMgr
    quantizer = AutoQuantizer.from_config({"quant_method": "ptq", "weight_dtype": "int8", "kvcache_dtype": "int8"})
    quantizer.preprocess_model(net)
    mgr = net.infer_attention.paged_attention_mgr
    assert isinstance(mgr, QuantPagedAttentionMgr) and mgr.key_cache.dtype == torch.int8
    assert mgr.key_cache.shape == (nb, bs, n_kv, d) and mgr.kv_scale.shape == (2, n_kv * d)
    row = n_kv * d
    scale = (np.stack([np.abs(kc_f).reshape(-1, row).max(0), np.abs(vc_f).reshape(-1, row).max(0)]) / 110.0).astype(np.float32)
    offset = rng.integers(-12, 13, (2, row)).astype(np.float32)
    mgr.set_kv_quant(dev(scale, torch.float32), dev(offset, torch.float32))
    k8 = O.quantize_kv_int8(kc_f.reshape(-1, row), scale[0], offset[0]).reshape(kc_f.shape)
    v8 = O.quantize_kv_int8(vc_f.reshape(-1, row), scale[1], offset[1]).reshape(vc_f.shape)
    mgr.key_cache.copy_(torch.from_numpy(k8))
    mgr.value_cache.copy_(torch.from_numpy(v8))
    attn = net.infer_attention
    attn.is_first_iteration = False
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    freqs = FreqsMgr(d, seq_length=seq, max_position_embedding=seq, rotary_dtype=dt)
    lens_t = torch.from_numpy(lens.astype(np.int32)).cuda()
    freqs_cis = freqs.increment(lens_t)
    q = rounded(rng.normal(size=(b, n_head * d)), dt)
    k = rounded(rng.normal(size=(b, row)), dt)
    v = rounded(rng.normal(size=(b, row)), dt)
    shape = (b, n_head * d) if dynamic else (b, 1, n_head * d)
    kv_shape = (b, row) if dynamic else (b, 1, row)
    out = attn(dev(q, dt).reshape(shape), dev(k, dt).reshape(kv_shape), dev(v, dt).reshape(kv_shape), lens_t,
               torch.from_numpy(tables).cuda(), torch.from_numpy(slots).cuda(), freqs_cis)
    assert out.shape == shape
    cos, sin = to_np(freqs_cis[0]), to_np(freqs_cis[1])
    q_r = rounded(O.apply_rotary_half(q, cos, sin, n_head), dt)
    k_r = rounded(O.apply_rotary_half(k, cos, sin, n_kv), dt)
    O.reshape_and_cache(O.quantize_kv_int8(k_r, scale[0], offset[0]), O.quantize_kv_int8(v, scale[1], offset[1]), k8, v8, slots)
    kf = O.dequantize_kv_int8(k8.reshape(-1, row), scale[0], offset[0]).reshape(k8.shape)
    vf = O.dequantize_kv_int8(v8.reshape(-1, row), scale[1], offset[1]).reshape(v8.shape)
    ref = O.paged_attention_decode(q_r, kf, vf, tables, lens, n_head, n_kv, 1 / np.sqrt(d))
    mag = O.paged_attention_decode(q_r, kf, np.abs(vf), tables, lens, n_head, n_kv, 1 / np.sqrt(d))
    assert_within(to_np(out).reshape(b, -1), ref, mag, dt, ulps=6.0, what="InferAttention decode over an int8 cache")
    got_k = mgr.key_cache.cpu().numpy().reshape(-1, row)[slots].astype(np.int32)
    assert np.abs(got_k - k8.reshape(-1, row)[slots]).max() <= 1          # a rotated key one rounding step away
    assert np.array_equal(mgr.value_cache.cpu().numpy().reshape(-1, row)[slots], v8.reshape(-1, row)[slots])
    keep = np.ones(nb * bs, bool)
    keep[slots] = False
    assert np.array_equal(mgr.key_cache.cpu().numpy().reshape(-1, row)[keep], k8.reshape(-1, row)[keep])


@pytest.mark.parametrize("bs", [16, 128])
def test_quantizer_swaps_in_the_per_token_int8_kv_manager(bs):
    """`kvcache_dtype: int8` with `kvcache_quant_granularity: per_token` (quantization_config.py:206-207): the manager
    the quantizer swaps in owns int8 caches and one scale per cached token.  A prefill through InferAttention writes
    the prompt's rotated keys and values quantised per token, bit for bit as the oracle quantises them, and a decode
    step attends over them - against the oracle's attention over the dequantised cache."""
    from torch import nn
    from mindformers_amd.modules import FreqsMgr, InferAttention, QuantPagedAttentionMgr
    from mindformers_amd.modules.quantizers import AutoQuantizer
    rng = np.random.default_rng(50 + bs)
    b, n_head, n_kv, d, seq = 3, 8, 2, 64, 512
    dt, row = BF, 2 * 64
    lens = np.array([70, 5, 131])
    _, _, tables, nb = make_paged_cache(rng, b, lens + 1, n_kv, d, bs, dt, max_blocks=seq // bs)

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.infer_attention = InferAttention(n_head, d, n_kv, scale_value=1 / np.sqrt(d), block_size=bs,
                                                  num_blocks=nb, seq_length=seq, is_dynamic=True, rotary_cos_format=2,
                                                  compute_dtype=dt)
    net = Block()
    AutoQuantizer.from_config({"quant_method": "ptq", "weight_dtype": "int8", "activation_dtype": "int8",
                               "act_quant_granularity": "per_token", "kvcache_dtype": "int8",
                               "kvcache_quant_granularity": "per_token"}).preprocess_model(net)
    mgr = net.infer_attention.paged_attention_mgr
    assert isinstance(mgr, QuantPagedAttentionMgr) and mgr.granularity == "per_token" and mgr.kv_scale is None
    assert mgr.key_cache.dtype == torch.int8 and mgr.key_scale_cache.shape == (nb, bs)
    with pytest.raises(ValueError):
        mgr.set_kv_quant(torch.ones(2, row))
    mgr.key_scale_cache.fill_(float("nan"))                   # a slot never written must never be read
    mgr.value_scale_cache.fill_(float("nan"))
    attn = net.infer_attention
    freqs = FreqsMgr(d, seq_length=seq, max_position_embedding=seq, rotary_dtype=dt)
    # ---- prefill: the prompts, packed
    t = int(lens.sum())
    q = rounded(rng.normal(size=(t, n_head * d)), dt)
    k = rounded(rng.normal(size=(t, row)), dt)
    v = rounded(rng.normal(size=(t, row)), dt)
    pos = np.concatenate([np.arange(n) for n in lens])
    seq_of = np.repeat(np.arange(b), lens)
    slots = (tables[seq_of, pos // bs] * bs + pos % bs).astype(np.int32)
    lens_t = torch.from_numpy(lens.astype(np.int32)).cuda()
    attn.is_first_iteration = True
    cos_all, sin_all = to_np(freqs.freqs_cos), to_np(freqs.freqs_sin)
    cos_t, sin_t = dev(cos_all[pos], dt), dev(sin_all[pos], dt)
    attn(dev(q, dt), dev(k, dt), dev(v, dt), lens_t, torch.from_numpy(tables).cuda(), torch.from_numpy(slots).cuda(),
         (cos_t, sin_t, None))
    k_r = rounded(O.apply_rotary_half(k, cos_all[pos], sin_all[pos], n_kv), dt)
    k8_ref, ks_ref = O.quantize_kv_int8_per_token(k_r)
    v8_ref, vs_ref = O.quantize_kv_int8_per_token(v)
    got_k = to_np(mgr.key_cache).reshape(-1, row)[slots].astype(np.int32)
    assert np.abs(got_k - k8_ref).max() <= 1                  # a rotated key one rounding step away
    assert np.array_equal(to_np(mgr.value_cache).reshape(-1, row)[slots], v8_ref)
    assert np.array_equal(to_np(mgr.value_scale_cache).reshape(-1)[slots], vs_ref)
    assert np.allclose(to_np(mgr.key_scale_cache).reshape(-1)[slots], ks_ref, rtol=2.0 ** -7)
    # ---- decode: one more token per sequence over the cache the module wrote
    attn.is_first_iteration = False
    lens2 = lens + 1
    slots2 = np.array([tables[i, (n - 1) // bs] * bs + (n - 1) % bs for i, n in enumerate(lens2)], np.int32)
    lens2_t = torch.from_numpy(lens2.astype(np.int32)).cuda()
    q2 = rounded(rng.normal(size=(b, n_head * d)), dt)
    k2 = rounded(rng.normal(size=(b, row)), dt)
    v2 = rounded(rng.normal(size=(b, row)), dt)
    cos2, sin2 = cos_all[lens2 - 1], sin_all[lens2 - 1]
    out = attn(dev(q2, dt), dev(k2, dt), dev(v2, dt), lens2_t, torch.from_numpy(tables).cuda(),
               torch.from_numpy(slots2).cuda(), (dev(cos2, dt), dev(sin2, dt), None))
    kq, vq = to_np(mgr.key_cache).astype(np.float64), to_np(mgr.value_cache).astype(np.float64)
    ksc, vsc = to_np(mgr.key_scale_cache).astype(np.float64), to_np(mgr.value_scale_cache).astype(np.float64)
    live = np.isfinite(ksc)
    assert live.sum() == t + b and np.array_equal(live, np.isfinite(vsc))
    kf = kq * np.where(live, ksc, 0.0)[:, :, None, None]
    vf = vq * np.where(live, vsc, 0.0)[:, :, None, None]
    q_r = rounded(O.apply_rotary_half(q2, cos2, sin2, n_head), dt)
    ref = O.paged_attention_decode(q_r, kf, vf, tables, lens2, n_head, n_kv, 1 / np.sqrt(d))
    mag = O.paged_attention_decode(q_r, kf, np.abs(vf), tables, lens2, n_head, n_kv, 1 / np.sqrt(d))
    assert_within(to_np(out).reshape(b, -1), ref, mag, dt, ulps=4.0, what="InferAttention over a per-token int8 cache")


def test_mcore_flash_attention_over_int8_caches():
    """FlashAttention's decode branch with int8 caches passed per call and the antiquant parameters in the
    PagedAttention positions: the scatter quantises, the attention dequantises; refused without the parameters."""
    from mindformers_amd.modules import FlashAttention
    rng = np.random.default_rng(9)
    b, nh, nkv, d, bs = 3, 8, 2, 128, 128
    dt = BF
    lens = rng.integers(100, 700, b)
    kc_f, vc_f, tables, nb = make_paged_cache(rng, b, lens, nkv, d, bs, dt)
    row = nkv * d
    scale = (np.stack([np.abs(kc_f).reshape(-1, row).max(0), np.abs(vc_f).reshape(-1, row).max(0)]) / 120.0).astype(np.float32)
    k8 = O.quantize_kv_int8(kc_f.reshape(-1, row), scale[0]).reshape(kc_f.shape)
    v8 = O.quantize_kv_int8(vc_f.reshape(-1, row), scale[1]).reshape(vc_f.shape)
    kc, vc = torch.from_numpy(k8).cuda(), torch.from_numpy(v8).cuda()
    fa = FlashAttention(nh, d, nkv, scale_value=1 / np.sqrt(d), pa_kv_head_num=nkv)
    fa.is_prefill = False
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    q = rounded(rng.normal(size=(b, nh * d)), dt)
    k = rounded(rng.normal(size=(b, row)), dt)
    v = rounded(rng.normal(size=(b, row)), dt)
    args = dict(slot_mapping=torch.from_numpy(slots).cuda(), block_tables=torch.from_numpy(tables).cuda(),
                batch_valid_length=torch.from_numpy(lens.astype(np.int32)).cuda(), key_cache=kc, value_cache=vc)
    with pytest.raises(ValueError):
        fa(dev(q, dt), dev(k, dt), dev(v, dt), **args)
    out = fa(dev(q, dt), dev(k, dt), dev(v, dt), antiquant_scale=dev(scale, torch.float32), **args)
    O.reshape_and_cache(O.quantize_kv_int8(k, scale[0]), O.quantize_kv_int8(v, scale[1]), k8, v8, slots)
    assert np.array_equal(kc.cpu().numpy(), k8) and np.array_equal(vc.cpu().numpy(), v8)
    kf = O.dequantize_kv_int8(k8.reshape(-1, row), scale[0]).reshape(k8.shape)
    vf = O.dequantize_kv_int8(v8.reshape(-1, row), scale[1]).reshape(v8.shape)
    ref = O.paged_attention_decode(q, kf, vf, tables, lens, nh, nkv, 1 / np.sqrt(d))
    mag = O.paged_attention_decode(q, kf, np.abs(vf), tables, lens, nh, nkv, 1 / np.sqrt(d))
    assert_within(to_np(out), ref, mag, dt, ulps=3.0, what="FlashAttention over int8 caches")


@pytest.mark.parametrize("granularity", ["per_token", "per_tensor", "per_token+smooth"])
def test_moe_layer_w8a8_experts_vs_oracle(granularity):
    """The reference's own W8A8 recipe for the routed experts (quant_method ptq, int8 weights and activations,
    research/deepseek3/deepseek_r1_671b/predict_deepseek_r1_671b_w8a8.yaml:89-92; its default activation granularity is
    per_tensor): the quantizer converts GroupedMLP to int8 experts, and the layer equals the oracle's router and
    permute around quantise -> exact int8 GEMM -> dequantise per expert, rounding where the device stores."""
    from oracle import dense as Dn
    from oracle.layer import _r
    from mindformers_amd.modules import AllQuantLinearInferCell, MoELayer, QuantGroupedMLP
    from mindformers_amd.modules.quantizers import AutoQuantizer
    from mindformers_amd.transformer_config import TransformerConfig
    cfg = TransformerConfig(num_layers=1, num_attention_heads=8, hidden_size=64, hidden_act="silu", num_moe_experts=8,
                            moe_router_topk=2, shared_expert_num=0, moe_router_topk_scaling_factor=2.5,
                            moe_shared_expert_intermediate_size=None, moe_ffn_hidden_size=32, moe_router_group_topk=2,
                            moe_router_num_groups=4, add_bias_linear=False, gated_linear_unit=True,
                            compute_dtype="bfloat16", params_dtype="bfloat16", moe_router_dtype="bfloat16",
                            moe_router_enable_expert_bias=True, moe_router_score_function="sigmoid")
    smooth = granularity.endswith("+smooth")      # one multiplier vector per expert in front of each projection
    granularity = granularity.split("+")[0]
    torch.manual_seed(3)
    net = MoELayer(cfg)
    net.router.weight.data.normal_(0, 0.3)
    net.router.expert_bias.data.normal_(0, 0.1)
    net.experts.weight1.data.normal_(0, 0.3)
    net.experts.weight2.data.normal_(0, 0.3)
    router_w, router_b = to_np(net.router.weight), to_np(net.router.expert_bias)
    q = AutoQuantizer.from_config({"quant_method": "ptq", "weight_dtype": "int8", "activation_dtype": "int8",
                                   "act_quant_granularity": granularity, "modules_to_not_convert": ["router"],
                                   "outliers_suppression": "smooth" if smooth else "None"})
    q.preprocess_model(net)
    assert isinstance(net.experts, QuantGroupedMLP) and net.experts.act_quant == granularity
    sm_rng = np.random.default_rng(12)
    sm1 = sm_rng.uniform(0.5, 2.0, (8, 64)).astype(np.float32) if smooth else None
    sm2 = sm_rng.uniform(0.5, 2.0, (8, 32)).astype(np.float32) if smooth else None
    if smooth:
        assert net.experts.smooth_scale1.shape == (8, 64) and net.experts.smooth_scale2.shape == (8, 32)
        net.experts.smooth_scale1.copy_(torch.from_numpy(sm1))
        net.experts.smooth_scale2.copy_(torch.from_numpy(sm2))
    else:
        assert net.experts.smooth_scale1 is None
    s1, s2 = np.float32(0.03), np.float32(0.25)
    if granularity == "per_tensor":
        net.experts.act_scale1.fill_(float(s1))
        net.experts.act_scale2.fill_(float(s2))
    q.postprocess_model(net)
    x = rounded(np.random.default_rng(8).normal(size=(24, 64)), BF)
    out = to_np(net(dev(x, BF)))
    ex = net.experts
    w1, w1s, w2, w2s = to_np(ex.weight1), to_np(ex.w1_scale), to_np(ex.weight2), to_np(ex.w2_scale)
    e = w1.shape[0]
    logits = _r(Dn.linear(x, router_w), "bf16")
    wgt, idx = O.topk_router(logits.astype(np.float32), router_b, 2, 4, 2, 2.5)
    wgt = _r(wgt, "bf16")
    px, row_map, counts = O.moe_permute(x, idx, e)

    def quant(a, s, sm=None):
        if granularity == "per_tensor":
            return O.static_quant_per_tensor(a.astype(np.float32), s)
        if sm is None:
            return O.dynamic_quant_per_token(a.astype(np.float32))
        aq_, as_ = np.zeros(a.shape, np.int8), np.zeros(a.shape[0], np.float32)
        st = 0
        for i_, c_ in enumerate(counts):                          # the rows of expert i_ take its multiplier vector
            c_ = int(c_)
            aq_[st:st + c_], as_[st:st + c_] = O.dynamic_quant_per_token(a[st:st + c_].astype(np.float32), sm[i_])
            st += c_
        return aq_, as_
    y = np.zeros((px.shape[0], w2.shape[1]))
    start = 0
    xq, xs = quant(px, s1, sm1)
    h = np.zeros((px.shape[0], w1.shape[1]))
    for i, c in enumerate(counts):
        c = int(c)
        h[start:start + c] = O.w8a8_linear(xq[start:start + c], xs[start:start + c], w1[i], w1s[i])
        start += c
    h = _r(h, "bf16")
    f = h.shape[1] // 2
    a = _r(_r(Dn.silu(h[:, :f]), "bf16") * h[:, f:], "bf16")
    aq, a_s = quant(a, s2, sm2)
    start = 0
    for i, c in enumerate(counts):
        c = int(c)
        y[start:start + c] = O.w8a8_linear(aq[start:start + c], a_s[start:start + c], w2[i], w2s[i])
        start += c
    ref = _r(O.moe_unpermute(_r(y, "bf16"), row_map, wgt), "bf16")
    assert np.abs(out - ref).max() <= 6 * EPS[BF] * np.abs(ref).max()
    assert np.mean(np.abs(out - ref) > 2 * EPS[BF] * np.abs(ref) + 1e-6) < 0.02


# ------------------------------------------------------------------------------------------- multi-latent attention layer
def _mla_module_and_params(rng, hidden, n, q_lora, rank=512, nope=128, rope=64, vd=128, rope_type="yarn"):
    from mindformers_amd.modules import MLASelfAttention, MLATransformerConfig
    cfg = MLATransformerConfig(hidden_size=hidden, num_attention_heads=n, q_lora_rank=q_lora, kv_lora_rank=rank,
                               qk_head_dim=nope, qk_pos_emb_head_dim=rope, v_head_dim=vd, rope_type=rope_type,
                               layernorm_epsilon=1e-6, compute_dtype="bfloat16", params_dtype="bfloat16")
    net = MLASelfAttention(cfg, layer_number=1)
    p = {}

    def fill(cell, key, std):
        w = rounded(rng.normal(0, std, tuple(cell.weight.shape)), BF)
        cell.weight.data.copy_(dev(w, BF))
        p[key] = w
    if q_lora:
        fill(net.linear_qkv_down_proj, "qkv_down_w", hidden ** -0.5)
        fill(net.linear_q_up_proj, "q_up_w", q_lora ** -0.5)
        g = (1 + 0.1 * rng.normal(size=q_lora)).astype(np.float32)
        net.q_layernorm.weight.data.copy_(torch.from_numpy(g))
        p["q_norm"] = g
    else:
        fill(net.linear_q_proj, "q_w", hidden ** -0.5)
        fill(net.linear_kv_down_proj, "kv_down_w", hidden ** -0.5)
    fill(net.linear_kv_up_proj, "kv_up_w", rank ** -0.5)
    fill(net.linear_proj, "proj_w", (n * vd) ** -0.5)
    g = (1 + 0.1 * rng.normal(size=rank)).astype(np.float32)
    net.kv_layernorm.weight.data.copy_(torch.from_numpy(g))
    p["kv_norm"] = g
    ocfg = dict(n_head=n, qk_head_dim=nope, qk_pos_emb_head_dim=rope, kv_lora_rank=rank, v_head_dim=vd,
                q_lora_rank=q_lora, eps=1e-6, rotary_scaling_factor=cfg.rotary_scaling_factor, mscale=cfg.mscale)
    return net, cfg, p, ocfg


@pytest.mark.parametrize("hidden,n,q_lora,rope_type", [(7168, 128, 1536, "yarn"), (1024, 16, None, "rope")])
def test_mla_self_attention_prefill_then_decode_vs_oracle(hidden, n, q_lora, rope_type):
    """MLASelfAttention at the DeepSeek-V3 geometry (128 heads, 512 + 64 latent, 128 + 64 query heads, q_lora 1536) and
    at a small one without the query low-rank path: a prefill of three prompts writes the latent cache and returns the
    up-projected attention, one decode step per sequence then runs on absorbed weights over that cache.  Both against
    the float64 restatement rounded to bf16 where the module stores bf16; the caches must agree row for row."""
    from mindformers_amd.modules import BlockTables
    rng = np.random.default_rng(hidden + n)
    net, cfg, p, ocfg = _mla_module_and_params(rng, hidden, n, q_lora, rope_type=rope_type)
    rank, rope = cfg.kv_lora_rank, cfg.qk_pos_emb_head_dim
    lens = [70, 5, 130]
    bs = 32
    need = [(l + 1 + bs - 1) // bs for l in lens]
    nb = sum(need) + 2
    perm = rng.permutation(nb)
    tables = -np.ones((len(lens), max(need)), np.int32)
    pos = 0
    for i, k in enumerate(need):
        tables[i, :k] = perm[pos:pos + k]
        pos += k
    cache = torch.zeros(nb, bs, 1, rank + rope, dtype=BF, device="cuda")
    cache_ref = np.zeros((nb, bs, 1, rank + rope))
    cos_t, sin_t = net.rotary_pos_emb.get_cos_sin_for_prefill()
    # ---- prefill
    total = sum(lens)
    x = rounded(rng.normal(size=(total, hidden)), BF)
    positions = np.concatenate([np.arange(l) for l in lens])
    slots = np.concatenate([[tables[i, j // bs] * bs + j % bs for j in range(l)] for i, l in enumerate(lens)]).astype(np.int32)
    pos_t = torch.from_numpy(positions).cuda()
    cos, sin = cos_t.index_select(0, pos_t), sin_t.index_select(0, pos_t)
    net.is_prefill = True
    out = net(dev(x, BF), None, rotary_pos_cos=cos, rotary_pos_sin=sin, slot_mapping=dev(slots, torch.int32),
              actual_seq_qlen=torch.tensor(np.cumsum(lens), dtype=torch.int32, device="cuda"),
              actual_seq_kvlen=torch.tensor(np.cumsum(lens), dtype=torch.int32, device="cuda"), key_cache=cache)
    ref = O.mla_self_attention_prefill(x, p, ocfg, cache_ref, slots, lens, to_np(cos), to_np(sin), act_dtype="bf16")
    got = to_np(out)
    assert got.shape == (total, hidden)
    scale = np.abs(ref).max()
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 2e-2, np.linalg.norm(got - ref) / np.linalg.norm(ref)
    assert np.abs(got - ref).max() < 0.06 * scale, (np.abs(got - ref).max(), scale)
    # the latent rows: one bf16 step at most apart (the norm output may round either way), untouched rows zero
    c_got, c_ref = to_np(cache).reshape(-1, rank + rope), cache_ref.reshape(-1, rank + rope)
    assert np.abs(c_got[slots] - c_ref[slots]).max() <= 4 * EPS[BF] * np.abs(c_ref[slots]).max()
    keep = np.ones(c_got.shape[0], bool)
    keep[slots] = False
    assert not c_got[keep].any()
    # ---- one decode step per sequence over the cache the device wrote (the oracle continues on the device's rows)
    cache_ref = to_np(cache).astype(np.float64)
    b = len(lens)
    xd = rounded(rng.normal(size=(b, hidden)), BF)
    new_lens = np.asarray(lens, np.int32) + 1
    dslots = np.asarray([tables[i, lens[i] // bs] * bs + lens[i] % bs for i in range(b)], np.int32)
    pos_t = torch.from_numpy(np.asarray(lens, np.int64)).cuda()
    cos, sin = net.rotary_pos_emb.get_cos_sin_for_decode(pos_t)
    net.is_prefill = False
    out = net(dev(xd, BF), None, rotary_pos_cos=cos, rotary_pos_sin=sin, batch_valid_length=dev(new_lens, torch.int32),
              block_tables=dev(tables, torch.int32), slot_mapping=dev(dslots, torch.int32), key_cache=cache)
    ref = O.mla_self_attention_decode(xd, p, ocfg, cache_ref, tables, new_lens, dslots, to_np(cos), to_np(sin),
                                      act_dtype="bf16")
    got = to_np(out)
    assert got.shape == (b, hidden)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 2e-2, np.linalg.norm(got - ref) / np.linalg.norm(ref)
    assert np.abs(got - ref).max() < 0.06 * np.abs(ref).max()
    c_got = to_np(cache).reshape(-1, rank + rope)
    assert np.abs(c_got[dslots] - cache_ref.reshape(-1, rank + rope)[dslots]).max() <= 4 * EPS[BF] * np.abs(c_got[dslots]).max()
    # the decode step equals the last row of a prefill over the same tokens (absorbed = up-projected), on the device
    # too: sequence 1 (5 + 1 tokens) run again as one prompt
    i = 1
    xs = np.concatenate((x[lens[0]:lens[0] + lens[1]], xd[i:i + 1]))
    pos_t = torch.arange(lens[i] + 1, device="cuda")
    cos, sin = cos_t.index_select(0, pos_t), sin_t.index_select(0, pos_t)
    net.is_prefill = True
    seq = torch.tensor([lens[i] + 1], dtype=torch.int32, device="cuda")
    again = net(dev(xs, BF), None, rotary_pos_cos=cos, rotary_pos_sin=sin, slot_mapping=None, actual_seq_qlen=seq,
                actual_seq_kvlen=seq, key_cache=None)
    d = to_np(again[-1]) - got[i]
    assert np.linalg.norm(d) / np.linalg.norm(got[i]) < 2e-2


def test_mla_self_attention_with_quantized_projections():
    """The RTN quantizer converts the layer's projections (W8A16) and leaves linear_kv_up_proj, whose weight the
    absorbed projections read, as a float cell; the decode step stays close to the float layer's."""
    from mindformers_amd.modules import ColumnParallelLinear, WeightQuantLinearCell
    from mindformers_amd.modules.quantizers import AutoQuantizer
    rng = np.random.default_rng(5)
    net, cfg, p, ocfg = _mla_module_and_params(rng, 1024, 16, 384)
    rank, rope, bs = cfg.kv_lora_rank, cfg.qk_pos_emb_head_dim, 32
    lens = np.asarray([40, 7], np.int32)
    tables = np.asarray([[1, 0], [2, -1]], np.int32)
    cache = dev(rounded(rng.normal(size=(4, bs, 1, rank + rope)), BF), BF)
    x = dev(rounded(rng.normal(size=(2, 1024)), BF), BF)
    slots = dev(np.asarray([tables[i, (lens[i] - 1) // bs] * bs + (lens[i] - 1) % bs for i in range(2)], np.int32), torch.int32)
    cos, sin = net.rotary_pos_emb.get_cos_sin_for_decode(torch.from_numpy(lens.astype(np.int64) - 1).cuda())
    args = dict(rotary_pos_cos=cos, rotary_pos_sin=sin, batch_valid_length=dev(lens, torch.int32),
                block_tables=dev(tables, torch.int32), slot_mapping=slots)
    net.is_prefill = False
    ref = net(x, None, key_cache=cache.clone(), **args)
    q = AutoQuantizer.from_config({"quant_method": "rtn", "weight_dtype": "int8",
                                   "modules_to_not_convert": ["linear_kv_up_proj"]})
    q.preprocess_model(net)
    q.postprocess_model(net)
    assert isinstance(net.linear_qkv_down_proj, WeightQuantLinearCell) and isinstance(net.linear_proj, WeightQuantLinearCell)
    assert isinstance(net.linear_kv_up_proj, ColumnParallelLinear)
    out = net(x, None, key_cache=cache.clone(), **args)
    d = (out.float() - ref.float()).norm() / ref.float().norm()
    assert float(d) < 0.05, float(d)
    # a quantized linear_kv_up_proj cannot be absorbed: the layer says so
    net2, *_ = _mla_module_and_params(rng, 1024, 16, 384)
    q2 = AutoQuantizer.from_config({"quant_method": "rtn", "weight_dtype": "int8"})
    q2.preprocess_model(net2)
    q2.postprocess_model(net2)
    net2.is_prefill = False
    with pytest.raises(NotImplementedError):
        net2(x, None, key_cache=cache.clone(), **args)
