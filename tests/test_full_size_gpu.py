"""The bench configurations at their full sizes: the W8A16 Llama-3-8B decode layer step (batch 64, contexts
U[512, 4096], block 128) against the oracle, and size-independent properties of its parts (bit-exact cache scatter,
invariance of attention under moving blocks and reordering the batch, exact integer GEMMs).  GPU only."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import EPS, dev, rounded, to_np

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


@pytest.fixture(scope="module")
def llama_case():
    from mindformers_amd import synthetic
    case = synthetic.make_decode_case("llama3_8b_w8a16", seed=5)
    yield case
    case.clear()
    torch.cuda.empty_cache()


def _step_args(case, kc, vc):
    return (case["x"], kc, vc, case["block_tables"], case["context_lens"], case["slot_mapping"], case["cos"],
            case["sin"])


def test_layer_step_matches_the_oracle_on_every_row(llama_case):
    case = llama_case
    cfg, layer = case["cfg"], case["layers"][0]
    kc, vc = (c.clone() for c in case["caches"][0])
    kcn, vcn = to_np(kc), to_np(vc)                              # the oracle scatters into its own copies
    out = layer(*_step_args(case, kc, vc))
    p = {}
    for n in layer.NAMES:
        p[n + "_w"], p[n + "_s"] = to_np(getattr(layer, n + "_w")), to_np(getattr(layer, n + "_s"))
    p["attn_norm"], p["ffn_norm"] = to_np(layer.attn_norm), to_np(layer.ffn_norm)
    ocfg = dict(n_head=cfg["n_head"], n_kv_head=cfg["n_kv_head"], head_dim=cfg["head_dim"], eps=1e-5)
    ref = O.decode_layer_w8a16(to_np(case["x"]), p, ocfg, kcn, vcn, to_np(case["block_tables"]),
                               case["context_lens_host"], to_np(case["slot_mapping"]), to_np(case["cos"]),
                               to_np(case["sin"]), act_dtype="bf16")
    got = to_np(out)
    assert got.shape == (64, 4096)
    # Both sides round to bf16 at the same points (norms, projections, attention output, activation, residual sums).
    # Where the fp32 and the float64 sum of a projection fall on different sides of a rounding boundary an
    # intermediate moves by one bf16 step, and through the residual path that step (of the hidden state's magnitude,
    # not of the element's) reaches the output: elementwise a few output steps for all but a small fraction, and a
    # bound in steps of the row's scale for every element.
    err = np.abs(got - ref)
    row_max = np.abs(ref).max(axis=1, keepdims=True)
    tol = 8 * EPS[BF] * np.maximum(np.abs(ref), 0.05 * row_max) + 1e-4
    frac_bad = float(np.mean(err > tol))
    assert frac_bad < 0.02, (frac_bad, err.max())
    hard = 8 * EPS[BF] * np.maximum(np.abs(ref), 0.25 * row_max) + 1e-4
    assert np.all(err <= hard), (float(np.mean(err > hard)), err.max())
    # the step wrote one row per sequence into each cache, and nothing else
    slots = to_np(case["slot_mapping"]).astype(np.int64)
    row = cfg["n_kv_head"] * cfg["head_dim"]
    k_rows, v_rows = to_np(kc).reshape(-1, row), to_np(vc).reshape(-1, row)
    k_ref, v_ref = kcn.reshape(-1, row), vcn.reshape(-1, row)
    # values: a projection output may round to the neighbouring bf16 value (one step: 2 eps |v|); near zero the
    # fp32 accumulation itself shows (4096 products with sum |x||w| of about 50: 2^-18 * 50 = 2e-4, taken five-fold)
    acc_err = 1e-3
    r = v_ref[slots]
    assert np.all(np.abs(v_rows[slots] - r) <= 2 * EPS[BF] * np.abs(r) + acc_err), np.abs(v_rows[slots] - r).max()
    # keys: RoPE turns the pair (i, i + D/2) and keeps its length; a one-step change of either input moves an output
    # by at most one step of the pair's length, and the output rounds once more
    r = k_ref[slots]
    half = cfg["head_dim"] // 2
    pair = r.reshape(len(slots), cfg["n_kv_head"], 2, half)
    pair = np.broadcast_to(np.sqrt((pair ** 2).sum(axis=2, keepdims=True)), pair.shape).reshape(r.shape)
    d = np.abs(k_rows[slots] - r)
    assert np.all(d <= 2 * EPS[BF] * np.sqrt(2) * pair + EPS[BF] * np.abs(r) + 2 * acc_err), d.max()
    before_k, before_v = (to_np(c).reshape(-1, row) for c in case["caches"][0])
    keep = np.ones(k_rows.shape[0], bool)
    keep[slots] = False
    assert np.array_equal(k_rows[keep], before_k[keep]) and np.array_equal(v_rows[keep], before_v[keep])


def test_fused_step_scatters_the_bits_of_the_separate_ops(llama_case):
    """Projection + RoPE + cache write in one call against projection, then rope_and_cache: same q, same caches."""
    from mindformers_amd import ops
    case = llama_case
    layer = case["layers"][0]
    nq, nkv = layer.n_head * layer.head_dim, layer.n_kv_head * layer.head_dim
    n1 = ops.rms_norm(case["x"], layer.attn_norm, layer.eps)
    kc1, vc1 = (c.clone() for c in case["caches"][0])
    q1 = ops.w8a16_qkv_rope_and_cache(n1, layer._packed["qkv"], case["cos"], case["sin"], kc1, vc1,
                                      case["slot_mapping"], layer.n_head)
    kc2, vc2 = (c.clone() for c in case["caches"][0])
    qkv = ops.w8a16_linear(n1, layer._packed["qkv"])
    q2, k2, v2 = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:]
    ops.rope_and_cache(q2, k2, v2, case["cos"], case["sin"], kc2, vc2, case["slot_mapping"], layer.n_head)
    assert torch.equal(q1, q2) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    assert not torch.equal(kc1, case["caches"][0][0])


def test_attention_is_invariant_under_moving_blocks_and_reordering_the_batch(llama_case):
    from mindformers_amd import ops
    case = llama_case
    cfg = case["cfg"]
    kc, vc = case["caches"][0]
    nh, nkv, d = cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    q = torch.randn(cfg["batch"], nh * d, generator=gen, device="cuda").to(BF)
    scale = 1.0 / np.sqrt(d)
    out = ops.paged_attention(q, kc, vc, case["block_tables"], case["context_lens"], nh, nkv, scale)
    assert bool(torch.isfinite(out.float()).all())
    # physical blocks moved (new id = perm[old id]), the tables following them
    nb = case["num_blocks"]
    perm = torch.randperm(nb, generator=gen, device="cuda")
    kc2, vc2 = torch.empty_like(kc), torch.empty_like(vc)
    kc2[perm], vc2[perm] = kc, vc
    t = case["block_tables"].long()
    t2 = torch.where(t >= 0, perm[t.clamp(min=0)], t).to(torch.int32)
    out2 = ops.paged_attention(q, kc2, vc2, t2, case["context_lens"], nh, nkv, scale)
    assert torch.equal(out, out2)
    del kc2, vc2
    # the batch in another order: the same rows in that order
    order = torch.randperm(cfg["batch"], generator=gen, device="cuda")
    out3 = ops.paged_attention(q[order].contiguous(), kc, vc, case["block_tables"][order].contiguous(),
                               case["context_lens"][order].contiguous(), nh, nkv, scale)
    assert torch.equal(out[order], out3)


@pytest.mark.parametrize("m,n,k", [(64, 28672, 4096), (64, 4096, 14336)])
def test_w8a16_gemm_is_exact_on_an_integer_grid(m, n, k):
    """Power-of-two scales and small-integer activations make every product and sum exact whatever the order of the
    summation (split-K included): the kernel must return exactly the rounded integer matmul."""
    from mindformers_amd import ops
    rng = np.random.default_rng(k)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    s = (2.0 ** rng.integers(-12, -9, n)).astype(np.float32)
    x = rng.integers(-3, 4, (m, k)).astype(np.float32)
    y = ops.w8a16_linear(dev(x, BF), torch.from_numpy(wq).cuda(), torch.from_numpy(s).cuda())
    exact = (x.astype(np.float64) @ wq.astype(np.float64).T) * s          # integers below 2^53: exact in float64
    assert np.array_equal(to_np(y).astype(np.float64), rounded(exact, BF).astype(np.float64))


@pytest.mark.parametrize("m,n,k", [(256, 37888, 3584), (256, 3584, 18944)])
@pytest.mark.parametrize("tiled", [False, True])
def test_w8a8_accumulators_are_exact(m, n, k, tiled):
    """The MLP projections of the W8A8 bench shape (Qwen2.5-7B at 256 rows): int32 accumulators bit-exact."""
    from mindformers_amd import ops
    rng = np.random.default_rng(n)
    x = rounded(rng.normal(size=(m, k)), BF)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    ws = rng.uniform(1e-4, 5e-4, n).astype(np.float32)
    xq_t, xs = ops.dynamic_quant(dev(x, BF), tiled=tiled)
    xq_rows, xs_rows = ops.dynamic_quant(dev(x, BF))
    assert torch.equal(xs, xs_rows)
    w = ops.pack_w8a16(torch.from_numpy(wq).cuda(), torch.from_numpy(ws).cuda())
    y, acc = ops.w8a8_linear(xq_t, xs, w, return_acc=True)
    ref = to_np(xq_rows).astype(np.float64) @ wq.astype(np.float64).T     # integers below 2^53: exact in float64
    assert np.abs(ref).max() < 2 ** 31
    assert np.array_equal(to_np(acc).astype(np.float64), ref)
    yref = ref * to_np(xs).astype(np.float64)[:, None] * ws.astype(np.float64)[None, :]
    assert np.all(np.abs(to_np(y) - yref) <= 1.01 * EPS[BF] * np.abs(yref) + 1e-6)


def test_w8a8_layer_step_stage_by_stage_against_the_oracle():
    """The W8A8 bench layer (Qwen2.5-7B shape, batch 256, context 2048, per-token int8 activations) at full size,
    first 16 sequences restated by the oracle.  Every stage is compared on identical inputs (what the GPU fed it):
    quantised activations and their scales must be equal, projections, attention and residual sums within one or two
    steps of the bf16 grid.  End to end an independent oracle run only agrees statistically: a one-step difference of a
    bf16 intermediate that crosses a quantisation boundary moves the activation by a whole int8 step, and the random
    synthetic MLP activations have a coarse grid (row maxima near 50, step 0.39), so the composed outputs are held to
    a relative error norm instead of an elementwise bound."""
    from oracle import dense as Dn
    from oracle import quant as Q
    from oracle.layer import _r
    from helpers import assert_within, untile_int8
    from mindformers_amd import ops, synthetic
    case = synthetic.make_decode_case("qwen2_5_7b_w8a8", seed=7)
    cfg, layer = case["cfg"], case["layers"][0]
    kc, vc = case["caches"][0]
    n, b, hidden = 16, cfg["batch"], cfg["hidden"]
    x = case["x"]

    def oq(a, smooth):
        return Q.dynamic_quant_per_token(np.asarray(a, np.float32), to_np(smooth))

    def same_quant(xq_tiled, xs, a_rows, smooth, width, what):
        q_ref, s_ref = oq(a_rows, smooth)
        assert np.array_equal(to_np(xs[:n]), s_ref.astype(np.float32)), what
        assert np.array_equal(untile_int8(to_np(xq_tiled.data), b, width)[:n], q_ref), what
        return q_ref, s_ref

    def olin(q, s, name):
        return Q.w8a8_linear(q, s, to_np(getattr(layer, name + "_w")), to_np(getattr(layer, name + "_s")), None)

    # attention norm + quantisation, QKV projection
    xq, xs = ops.rms_norm_dynamic_quant(x, layer.attn_norm, layer.eps, layer.qkv_smooth, tiled=True)
    n1 = ops.rms_norm(x, layer.attn_norm, layer.eps)
    n1_ref = Dn.rms_norm(to_np(x[:n]).astype(np.float64), to_np(layer.attn_norm), 1e-5)
    assert_within(to_np(n1[:n]), n1_ref, np.abs(n1_ref), BF, ulps=1.0, extra=1e-6, what="attention norm")
    q1, s1 = same_quant(xq, xs, to_np(n1[:n]), layer.qkv_smooth, hidden, "qkv activations")
    qkv = ops.w8a8_linear(xq, xs, layer._packed["qkv"])
    ref = olin(q1, s1, "qkv")
    assert_within(to_np(qkv[:n]), ref, np.abs(ref), BF, ulps=1.0, extra=1e-6, what="qkv projection")
    # RoPE + cache write (bit-exact against the separate ops elsewhere), attention over the real caches
    kc1, vc1 = kc.clone(), vc.clone()
    q_rot = ops.w8a8_qkv_rope_and_cache(xq, xs, layer._packed["qkv"], case["cos"], case["sin"], kc1, vc1,
                                        case["slot_mapping"], layer.n_head)
    attn, aq, a_s = ops.paged_attention(q_rot, kc1, vc1, case["block_tables"], case["context_lens"], layer.n_head,
                                        layer.n_kv_head, layer.scale_value, quant=(layer.wo_smooth, True))
    tables = to_np(case["block_tables"][:n])
    used = np.unique(tables[tables >= 0])
    remap = -np.ones(case["num_blocks"], dtype=np.int64)
    remap[used] = np.arange(len(used))
    t2 = np.where(tables >= 0, remap[np.maximum(tables, 0)], -1).astype(np.int32)
    sel = torch.from_numpy(used).cuda()
    a_ref = O.paged_attention_decode(to_np(q_rot[:n].contiguous()).astype(np.float64), to_np(kc1[sel]), to_np(vc1[sel]), t2,
                                     case["context_lens_host"][:n], layer.n_head, layer.n_kv_head, layer.scale_value)
    # magnitude of a softmax-weighted sum: the same attention over |V| (the probabilities round to bf16 one by one)
    a_mag = O.paged_attention_decode(to_np(q_rot[:n].contiguous()).astype(np.float64), to_np(kc1[sel]),
                                     np.abs(to_np(vc1[sel])), t2, case["context_lens_host"][:n], layer.n_head,
                                     layer.n_kv_head, layer.scale_value)
    assert_within(to_np(attn[:n]), a_ref, a_mag, BF, ulps=1.5, what="attention")
    q2, s2 = same_quant(aq, a_s, to_np(attn[:n]), layer.wo_smooth, layer.n_head * layer.head_dim, "wo activations")
    # output projection + residual + MLP norm + quantisation
    h, n2x, n2s = ops.w8a8_linear_add_rmsnorm_quant(aq, a_s, layer._packed["wo"], x, layer.ffn_norm, layer.eps,
                                                    layer.fc1_smooth)
    h_ref = to_np(x[:n]).astype(np.float64) + _r(olin(q2, s2, "wo"), "bf16")
    assert_within(to_np(h[:n]), h_ref, np.abs(h_ref) + np.abs(to_np(x[:n])), BF, ulps=2.0, extra=1e-6, what="h")
    n2_ref = _r(Dn.rms_norm(to_np(h[:n]).astype(np.float64), to_np(layer.ffn_norm), 1e-5), "bf16")
    q3, s3 = oq(n2_ref, layer.fc1_smooth)
    # the norm's own rounding may move an element by a bf16 step: scales equal, int8 within one step
    assert np.allclose(to_np(n2s[:n]), s3, rtol=2 * EPS[BF], atol=0)
    assert np.abs(untile_int8(to_np(n2x.data), b, hidden)[:n].astype(np.int32) - q3).max() <= 1
    # gate/up, activation + quantisation, down projection + residual
    gu = layer._linear(None, "fc1", quantized=(n2x, n2s))
    gq, gs = untile_int8(to_np(n2x.data), b, hidden)[:n], to_np(n2s[:n])
    ref = olin(gq, gs, "fc1")
    assert_within(to_np(gu[:n]), ref, np.abs(ref), BF, ulps=1.0, extra=1e-6, what="gate/up projection")
    f = gu.shape[-1] // 2
    guf = to_np(gu[:n]).astype(np.float64)
    act_ref = _r(_r(Dn.silu(guf[:, :f]), "bf16") * guf[:, f:], "bf16")
    actq = ops.silu_mul_dynamic_quant(gu, layer.fc2_smooth, tiled=True)
    act = ops.silu_mul(gu)
    assert_within(to_np(act[:n]), act_ref, np.abs(act_ref), BF, ulps=2.0, extra=1e-6, what="silu * up")
    q4, s4 = same_quant(actq[0], actq[1], to_np(act[:n]), layer.fc2_smooth, f, "fc2 activations")
    out = layer._linear(None, "fc2", residual=h, quantized=actq)
    o_ref = to_np(h[:n]).astype(np.float64) + _r(olin(q4, s4, "fc2"), "bf16")
    assert_within(to_np(out[:n]), o_ref, np.abs(o_ref) + np.abs(to_np(h[:n])), BF, ulps=2.0, extra=1e-6, what="out")
    # the layer call is that sequence of stages
    full = layer(*_step_args(case, kc.clone(), vc.clone()))
    assert torch.equal(full, out)
    # end to end against an independent oracle run of the 16 sequences
    p = {}
    for name in layer.NAMES:
        p[name + "_w"], p[name + "_s"] = to_np(getattr(layer, name + "_w")), to_np(getattr(layer, name + "_s"))
        p[name + "_smooth"] = to_np(getattr(layer, name + "_smooth"))
    p["attn_norm"], p["ffn_norm"] = to_np(layer.attn_norm), to_np(layer.ffn_norm)
    ocfg = dict(n_head=cfg["n_head"], n_kv_head=cfg["n_kv_head"], head_dim=cfg["head_dim"], eps=1e-5)
    bs = cfg["block_size"]
    slots = to_np(case["slot_mapping"][:n]).astype(np.int64)
    slots2 = (remap[slots // bs] * bs + slots % bs).astype(np.int32)
    e2e = O.decode_layer_w8a8(to_np(x[:n]), p, ocfg, to_np(kc[sel]), to_np(vc[sel]), t2, case["context_lens_host"][:n],
                              slots2, to_np(case["cos"][:n]), to_np(case["sin"][:n]), act_dtype="bf16")
    got = to_np(full[:n]).astype(np.float64)
    assert np.linalg.norm(got - e2e) / np.linalg.norm(e2e) < 0.05
    case.clear()
    torch.cuda.empty_cache()
