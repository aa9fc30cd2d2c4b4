"""Checkpoint formats: name map, fused-row permutations, directory conversion, layer loading.

The directory scenarios replay tests/st/test_safetensors/test_convert.py of the reference (same fake geometry,
file names and expectations); the permutations are checked against the oracle's per-row loops, hand-computed
cases and labelled rows.
"""
import json
import os

import numpy as np
import pytest
from safetensors.numpy import load_file, save_file

import oracle as O
from mindformers_amd import checkpoint as C


def test_convert_name_known_answers():
    known = {
        "model.layers.0.self_attn.q_proj.weight": "model.layers.0.attention.wq.weight",
        "model.layers.0.self_attn.k_proj.weight": "model.layers.0.attention.wk.weight",
        "model.layers.0.self_attn.v_proj.weight": "model.layers.0.attention.wv.weight",
        "model.layers.3.self_attn.o_proj.weight": "model.layers.3.attention.wo.weight",
        "model.layers.3.mlp.gate_proj.weight": "model.layers.3.feed_forward.w1.weight",
        "model.layers.3.mlp.down_proj.weight": "model.layers.3.feed_forward.w2.weight",
        "model.layers.3.mlp.up_proj.weight": "model.layers.3.feed_forward.w3.weight",
        "model.layers.7.input_layernorm.weight": "model.layers.7.attention_norm.weight",
        "model.layers.7.post_attention_layernorm.weight": "model.layers.7.ffn_norm.weight",
        "model.norm.weight": "model.norm_out.weight",
        "model.embed_tokens.weight": "model.tok_embeddings.embedding_weight",
        "model.layers.0.self_attn.q_proj.bias": "model.layers.0.attention.wq.bias",
    }
    for hf, mf in known.items():
        assert C.convert_name(hf) == mf
    assert C.obtain_qkv_ffn_concat_keys() == ["w_qkv", "w_gate_hidden"]


def test_fused_row_permutations_hand_cases():
    # 4 heads, 2 kv heads, head_dim 1: q rows 0-3, k rows 4-5, v rows 6-7
    w = np.arange(8)[:, None] * np.ones((1, 3), int)
    assert C.qkv_concat_hf2mg(w, 4, 2, 4)[:, 0].tolist() == [0, 1, 4, 6, 2, 3, 5, 7]
    assert C.qkv_concat_hf2mg(np.arange(8), 4, 2, 4).tolist() == [0, 1, 4, 6, 2, 3, 5, 7]          # bias
    # the reference's own test geometry (2 heads, 1 kv head, hidden 2) is the identity
    assert C.qkv_concat_hf2mg(np.arange(4), 2, 1, 2).tolist() == [0, 1, 2, 3]
    f = np.arange(6)[:, None] * np.ones((1, 2), int)
    assert C.ffn_concat_hf2mg(f, 3)[:, 0].tolist() == [0, 3, 1, 4, 2, 5]
    with pytest.raises(ValueError):
        C.qkv_concat_hf2mg(np.zeros((2, 2, 2)), 2, 1, 2)
    with pytest.raises(ValueError):
        C.qkv_concat_hf2mg(np.zeros((5, 2)), 2, 1, 2)


@pytest.mark.parametrize("nh,nkv,d", [(8, 2, 4), (4, 4, 2), (28, 4, 2), (6, 1, 3)])
def test_fused_row_permutations_structure(nh, nkv, d):
    hidden, n_rep = nh * d, nh // nkv
    rng = np.random.default_rng(nh)
    w = rng.normal(size=(hidden + 2 * nkv * d, 5))
    mg = C.qkv_concat_hf2mg(w, nh, nkv, hidden)
    assert np.array_equal(mg, O.checkpoint.qkv_concat_hf2mg(w, nh, nkv, hidden))
    # labelled rows: block g of the result is [q heads g*n_rep .. | k head g | v head g]
    blocks = mg.reshape(nkv, n_rep + 2, d, 5)
    q = w[:hidden].reshape(nh, d, 5)
    k = w[hidden:hidden + nkv * d].reshape(nkv, d, 5)
    v = w[hidden + nkv * d:].reshape(nkv, d, 5)
    for g in range(nkv):
        assert np.array_equal(blocks[g, :n_rep], q[g * n_rep:(g + 1) * n_rep])
        assert np.array_equal(blocks[g, n_rep], k[g]) and np.array_equal(blocks[g, n_rep + 1], v[g])
    assert np.array_equal(C.qkv_concat_mg2hf(mg, nh, nkv, hidden), w)
    f = rng.normal(size=(2 * 7, 3))
    fm = C.ffn_concat_hf2mg(f, 7)
    assert np.array_equal(fm, O.checkpoint.ffn_concat_hf2mg(f, 7))
    assert np.array_equal(fm[0::2], f[:7]) and np.array_equal(fm[1::2], f[7:])
    assert np.array_equal(C.ffn_concat_mg2hf(fm, 7), f)


class _Cfg:
    num_heads, n_kv_heads, hidden_size, qkv_concat = 2, 1, 2, False
    intermediate_size = None


@pytest.fixture()
def fake_dirs(tmp_path):
    rng = np.random.default_rng(0)
    w1, w2, w3 = rng.random((2, 2)), rng.random((1, 2)), rng.random((1, 2))
    names = ["model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.k_proj.weight",
             "model.layers.0.self_attn.v_proj.weight"]
    unified = tmp_path / "hf_path_unified"
    unified.mkdir()
    files = [f"model-0000{i + 1}-of-00003.safetensors" for i in range(3)]
    for n, w, f in zip(names, (w1, w2, w3), files):
        save_file({n: w}, str(unified / f))
    (unified / "model.safetensors.index.json").write_text(json.dumps({"weight_map": dict(zip(names, files))}))
    single = tmp_path / "hf_path_single"
    single.mkdir()
    save_file(dict(zip(names, (w1, w2, w3))), str(single / "model.safetensors"))
    return str(unified), str(single), str(tmp_path / "ms_unified"), str(tmp_path / "ms_single"), (w1, w2, w3), files


def test_convert_directory_like_the_reference_test(fake_dirs):
    unified, single, dst_u, dst_s, (w1, w2, w3), files = fake_dirs
    cfg = _Cfg()
    assert C.contains_safetensors_files(unified) and C.is_hf_safetensors_dir(unified)
    C.convert_hf_safetensors_multiprocess(unified, dst_u, None, cfg)
    mf = ["model.layers.0.attention.wq.weight", "model.layers.0.attention.wk.weight", "model.layers.0.attention.wv.weight"]
    name_map = json.load(open(os.path.join(dst_u, "param_name_map.json")))
    for name, w, f in zip(mf, (w1, w2, w3), files):
        assert np.array_equal(load_file(os.path.join(dst_u, f))[name], w)
        assert name_map[name] == f
    assert not C.is_hf_safetensors_dir(dst_u)
    # with qkv_concat the fused weight lands in the file that held q
    cfg.qkv_concat = True
    dst_c = dst_u + "_concat"
    C.convert_hf_safetensors_multiprocess(unified, dst_c, None, cfg)
    got = load_file(os.path.join(dst_c, files[0]))
    expect = O.checkpoint.qkv_concat_hf2mg(np.concatenate((w1, w2, w3)), 2, 1, 2)
    assert np.array_equal(got["model.layers.0.attention.w_qkv.weight"], expect)
    name_map = json.load(open(os.path.join(dst_c, "param_name_map.json")))
    assert name_map == {"model.layers.0.attention.w_qkv.weight": files[0]}
    # single file
    cfg.qkv_concat = False
    C.convert_hf_safetensors_multiprocess(single, dst_s, None, cfg)
    got = load_file(os.path.join(dst_s, "model.safetensors"))
    assert all(np.array_equal(got[n], w) for n, w in zip(mf, (w1, w2, w3)))
    cfg.qkv_concat = True
    C.convert_hf_safetensors_multiprocess(single, dst_s + "_concat", None, cfg)
    got = load_file(os.path.join(dst_s + "_concat", "model.safetensors"))
    assert np.array_equal(got["model.layers.0.attention.w_qkv.weight"], expect)
    for bad in ((1, dst_s, None, cfg), (single, 1, None, cfg), (single, dst_s, None, None)):
        with pytest.raises(ValueError):
            C.convert_hf_safetensors_multiprocess(*bad)


def _fake_layer(rng, nh, nkv, d, ffn, layer=1, bias=False):
    hidden = nh * d
    t = {}
    p = f"model.layers.{layer}."
    for name, shape in (("self_attn.q_proj", (hidden, hidden)), ("self_attn.k_proj", (nkv * d, hidden)),
                        ("self_attn.v_proj", (nkv * d, hidden)), ("self_attn.o_proj", (hidden, hidden)),
                        ("mlp.gate_proj", (ffn, hidden)), ("mlp.up_proj", (ffn, hidden)), ("mlp.down_proj", (hidden, ffn))):
        t[p + name + ".weight"] = rng.normal(0, 0.05, shape).astype(np.float32)
        if bias and "self_attn" in name and "o_proj" not in name:
            t[p + name + ".bias"] = rng.normal(0, 0.05, shape[0]).astype(np.float32)
    t[p + "input_layernorm.weight"] = rng.normal(1, 0.1, hidden).astype(np.float32)
    t[p + "post_attention_layernorm.weight"] = rng.normal(1, 0.1, hidden).astype(np.float32)
    return t


def test_layer_arrays_agree_across_the_three_formats(tmp_path):
    rng = np.random.default_rng(2)
    nh, nkv, d, ffn = 8, 2, 4, 24
    cfg = dict(num_heads=nh, n_kv_heads=nkv, hidden_size=nh * d, intermediate_size=ffn, qkv_concat=False)
    hf = _fake_layer(rng, nh, nkv, d, ffn, bias=True)
    a = C.read_layer_arrays(hf, 1, cfg)
    p = "model.layers.1."
    assert np.array_equal(a["qkv"][0], np.concatenate([hf[p + f"self_attn.{k}_proj.weight"] for k in "qkv"]))
    assert np.array_equal(a["qkv"][2], np.concatenate([hf[p + f"self_attn.{k}_proj.bias"] for k in "qkv"]))
    assert np.array_equal(a["fc1"][0], np.concatenate([hf[p + "mlp.gate_proj.weight"], hf[p + "mlp.up_proj.weight"]]))
    assert np.array_equal(a["fc2"][0], hf[p + "mlp.down_proj.weight"]) and a["wo"][2] is None
    # reference names, separate projections, from a file
    mf = C.convert_weight_dict(hf, cfg)
    f = str(tmp_path / "mf.safetensors")
    save_file(mf, f)
    b = C.read_layer_arrays(f, 1, cfg)
    # reference names, fused per-kv-group qkv and interleaved ffn, from a converted directory
    src = tmp_path / "hf"
    src.mkdir()
    save_file(hf, str(src / "model.safetensors"))
    C.convert_hf_safetensors_multiprocess(str(src), str(tmp_path / "mg"), None, dict(cfg, qkv_concat=True))
    fused = load_file(str(tmp_path / "mg" / "model.safetensors"))
    assert p + "attention.w_qkv.weight" in fused and p + "feed_forward.w_gate_hidden.weight" in fused
    assert p + "attention.w_qkv.bias" in fused
    c = C.read_layer_arrays(str(tmp_path / "mg"), 1, cfg)
    for other in (b, c):
        for k in ("qkv", "wo", "fc1", "fc2"):
            assert np.array_equal(other[k][0], a[k][0])
            assert (other[k][2] is None) == (a[k][2] is None)
            assert a[k][2] is None or np.array_equal(other[k][2], a[k][2])
        assert np.array_equal(other["attn_norm"], a["attn_norm"]) and np.array_equal(other["ffn_norm"], a["ffn_norm"])
    with pytest.raises(KeyError):
        C.read_layer_arrays(hf, 0, cfg)


def test_rtn_int8_matches_the_oracle_quantizer():
    rng = np.random.default_rng(3)
    w = rng.normal(size=(17, 40)).astype(np.float32)
    w[3] = 0
    q, s = C.quantize_rtn_int8(w)
    q_ref, s_ref = O.quantize_weight_int8(w)
    assert np.array_equal(q, q_ref) and np.array_equal(s, s_ref)
