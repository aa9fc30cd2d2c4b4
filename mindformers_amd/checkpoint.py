"""Weight formats either side of the decode path: HuggingFace safetensors -> the reference's parameter names and
fused layouts -> the int8 weights of one decode layer.

Mirrors, on numpy arrays and safetensors files:
  name map                  LlamaForCausalLM.convert_name            mindformers/models/llama/llama.py:681-702
  qkv / ffn concatenation   convert_weight_dict, _concat_qkv_weight,  llama.py:704-741, 804-892
                            _concat_ffn_weight
  fused-row permutations    qkv_concat_hf2mg, ffn_concat_hf2mg        mindformers/utils/convert_utils.py:65-106
  directory conversion      convert_hf_safetensors_multiprocess       (tests/st/test_safetensors/test_convert.py
                            (file names kept, param_name_map.json)     holds its observable contract)
  concat key names          obtain_qkv_ffn_concat_keys                llama.py:781-787

Only the safetensors format is read (a loader that executes nothing from the file).

Quantized checkpoints: the reference takes its int8 deploy parameters from golden-stick cells whose parameter
names are not part of it, so this build names them itself: ``<linear>.weight`` int8 [out, in], ``<linear>.w_scale``
float32 [out] and, for W8A8, ``<linear>.smooth_scale`` float32 [in].  A float ``<linear>.weight`` is quantized when
it is loaded (round to nearest, symmetric per output channel).
"""
import json
import os

import numpy as np

QKV_CONCAT_KEY = "w_qkv"
FFN_CONCAT_KEY = "w_gate_hidden"
NAME_MAP_FILE = "param_name_map.json"
HF_INDEX_FILE = "model.safetensors.index.json"

# HuggingFace -> reference parameter name fragments, applied in this order (llama.py:685-698)
_HF_TO_MF = (
    ("embed_tokens.", "tok_embeddings."),
    (".self_attn.q_proj.", ".attention.wq."),
    (".self_attn.k_proj.", ".attention.wk."),
    (".self_attn.v_proj.", ".attention.wv."),
    (".self_attn.o_proj.", ".attention.wo."),
    (".mlp.gate_proj.", ".feed_forward.w1."),
    (".mlp.down_proj.", ".feed_forward.w2."),
    (".mlp.up_proj.", ".feed_forward.w3."),
    (".input_layernorm.", ".attention_norm."),
    (".post_attention_layernorm.", ".ffn_norm."),
    (".norm.", ".norm_out."),
    ("output.", "lm_head."),
    (".tok_embeddings.weight", ".tok_embeddings.embedding_weight"),
)


# the per-layer modules, reference name -> HuggingFace name
_MF_TO_HF_MODULE = {
    "attention.wq": "self_attn.q_proj", "attention.wk": "self_attn.k_proj", "attention.wv": "self_attn.v_proj",
    "attention.wo": "self_attn.o_proj", "feed_forward.w1": "mlp.gate_proj", "feed_forward.w2": "mlp.down_proj",
    "feed_forward.w3": "mlp.up_proj", "attention_norm": "input_layernorm", "ffn_norm": "post_attention_layernorm",
}


def convert_name(weight_name):
    """HuggingFace parameter name -> the reference's (LlamaForCausalLM.convert_name)."""
    for old, new in _HF_TO_MF:
        weight_name = weight_name.replace(old, new)
    return weight_name


def obtain_qkv_ffn_concat_keys():
    return [QKV_CONCAT_KEY, FFN_CONCAT_KEY]


# ------------------------------------------------------------------------------------------- row permutations
def _qkv_rows_hf2mg(num_heads, n_kv_heads, hidden_size):
    """Source row (in the [q | k | v] concatenation) of every row of the per-kv-group layout
    [q heads of group 0 | k 0 | v 0 | q heads of group 1 | k 1 | v 1 | ...]."""
    if num_heads % n_kv_heads or hidden_size % num_heads:
        raise ValueError(f"num_heads={num_heads}, n_kv_heads={n_kv_heads}, hidden_size={hidden_size} do not divide")
    d = hidden_size // num_heads
    q_per_group = (num_heads // n_kv_heads) * d
    k_base = hidden_size
    v_base = hidden_size + n_kv_heads * d
    rows = []
    for g in range(n_kv_heads):
        rows.append(np.arange(g * q_per_group, (g + 1) * q_per_group))
        rows.append(k_base + np.arange(g * d, (g + 1) * d))
        rows.append(v_base + np.arange(g * d, (g + 1) * d))
    return np.concatenate(rows)


def _as_rows(t, what):
    t = np.asarray(t)
    if t.ndim not in (1, 2):
        raise ValueError(f"{what} shape is not supported.")
    return t


def qkv_concat_hf2mg(qkv_weights, num_heads, n_kv_heads, hidden_size):
    """[q | k | v] rows -> per-kv-group rows (convert_utils.py:65-92).  2-D weight or 1-D bias."""
    t = _as_rows(qkv_weights, "qkv_weights")
    rows = _qkv_rows_hf2mg(num_heads, n_kv_heads, hidden_size)
    if t.shape[0] != rows.size:
        raise ValueError(f"qkv_weights has {t.shape[0]} rows, the head geometry gives {rows.size}")
    return t[rows]


def qkv_concat_mg2hf(qkv_weights, num_heads, n_kv_heads, hidden_size):
    """Inverse of qkv_concat_hf2mg: per-kv-group rows back to [q | k | v]."""
    t = _as_rows(qkv_weights, "qkv_weights")
    rows = _qkv_rows_hf2mg(num_heads, n_kv_heads, hidden_size)
    if t.shape[0] != rows.size:
        raise ValueError(f"qkv_weights has {t.shape[0]} rows, the head geometry gives {rows.size}")
    out = np.empty_like(t)
    out[rows] = t
    return out


def ffn_concat_hf2mg(ffn_weights, ffn_hidden_size):
    """[gate | hidden] halves -> rows interleaved gate_0, hidden_0, gate_1, ... (convert_utils.py:95-106)."""
    t = _as_rows(ffn_weights, "ffn_weights")
    if t.shape[0] != 2 * ffn_hidden_size:
        raise ValueError(f"ffn_weights has {t.shape[0]} rows, expected {2 * ffn_hidden_size}")
    rows = np.stack((np.arange(ffn_hidden_size), ffn_hidden_size + np.arange(ffn_hidden_size)), axis=1).reshape(-1)
    return t[rows]


def ffn_concat_mg2hf(ffn_weights, ffn_hidden_size):
    """Inverse of ffn_concat_hf2mg."""
    t = _as_rows(ffn_weights, "ffn_weights")
    if t.shape[0] != 2 * ffn_hidden_size:
        raise ValueError(f"ffn_weights has {t.shape[0]} rows, expected {2 * ffn_hidden_size}")
    return np.concatenate((t[0::2], t[1::2]), axis=0)


# ------------------------------------------------------------------------------------------- dict conversion
def _cfg(model_config, name, default=None):
    if isinstance(model_config, dict):
        return model_config.get(name, default)
    return getattr(model_config, name, default)


def ffn_hidden_size_of(model_config):
    """The MLP width rule of the reference's Llama (llama.py:856-866)."""
    inter = _cfg(model_config, "intermediate_size")
    if inter is not None:
        return int(inter)
    width = _cfg(model_config, "hidden_size") * 4
    mult = _cfg(model_config, "ffn_dim_multiplier")
    if mult is not None:
        width = int((mult + 0.01) * width)
    width = int(2 * width / 3)
    multiple_of = _cfg(model_config, "multiple_of") or 256
    return multiple_of * ((width + multiple_of - 1) // multiple_of)


def convert_weight_dict(source_dict, model_config=None, pending=None):
    """HuggingFace weight dict -> the reference's names; with ``model_config.qkv_concat`` the q/k/v and gate/up
    weights of a layer are concatenated and permuted into ``w_qkv`` / ``w_gate_hidden``.

    ``pending``: a dict shared between calls for checkpoints whose q, k, v (or gate, up) live in different files:
    parts that cannot be completed yet are parked there and picked up by the call that holds the q (gate) part —
    the single-process stand-in for the reference's shared dict and condition variable (llama.py:816-844)."""
    target = {convert_name(k): np.asarray(v) for k, v in source_dict.items()}
    if not _cfg(model_config, "qkv_concat", False):
        return target
    pending = pending if pending is not None else {}
    num_heads = _cfg(model_config, "num_heads")
    n_kv_heads = _cfg(model_config, "n_kv_heads") or num_heads
    hidden_size = _cfg(model_config, "hidden_size")

    def kind(key):
        parts = key.split(".")
        return parts[-2] if len(parts) >= 2 else ""

    def parts_of(leader, followers):
        """Keys of the leader kind; followers whose leader is not in this dict are parked."""
        leaders = [k for k in target if kind(k) == leader]
        for k in [k for k in target if kind(k) in followers]:
            mate = ".".join(k.split(".")[:-2] + [leader, k.split(".")[-1]])
            if mate not in target:
                pending[k] = target.pop(k)
        return leaders

    def take(key):
        if key in target:
            return target.pop(key)
        if key in pending:
            return pending.pop(key)
        raise KeyError(f"{key} is needed for the concatenation but is in none of the files seen so far: convert the "
                       "files that hold the k/v (w3) parts first or pass all files to one call")

    for wq_key in parts_of("wq", ("wk", "wv")):
        parts = [target.pop(wq_key), take(wq_key.replace(".wq.", ".wk.")), take(wq_key.replace(".wq.", ".wv."))]
        fused = np.concatenate(parts, 0)
        target[wq_key.replace(".wq.", f".{QKV_CONCAT_KEY}.")] = qkv_concat_hf2mg(fused, num_heads, n_kv_heads, hidden_size)
    inter = _cfg(model_config, "intermediate_size")
    for w1_key in parts_of("w1", ("w3",)):
        fused = np.concatenate([target.pop(w1_key), take(w1_key.replace(".w1.", ".w3."))], 0)
        if fused.ndim == 2 and inter is not None and fused.shape[0] != 2 * int(inter):
            raise ValueError(f"{w1_key}: {fused.shape[0] // 2} channels, intermediate_size says {inter}")
        target[w1_key.replace(".w1.", f".{FFN_CONCAT_KEY}.")] = ffn_concat_hf2mg(fused, fused.shape[0] // 2)
    return target


def contains_safetensors_files(path):
    return isinstance(path, str) and os.path.isdir(path) and any(f.endswith(".safetensors") for f in os.listdir(path))


def is_hf_safetensors_dir(path, model_cls=None):
    """True when the directory's safetensors use HuggingFace names (any name that the name map changes)."""
    if not contains_safetensors_files(path):
        return False
    from safetensors import safe_open
    for f in sorted(os.listdir(path)):
        if f.endswith(".safetensors"):
            with safe_open(os.path.join(path, f), framework="np") as st:
                return any(convert_name(k) != k for k in st.keys())
    return False


def convert_hf_safetensors_multiprocess(src_dir, dst_dir, model_cls_or_instance=None, model_config=None):
    """Convert every ``*.safetensors`` of a HuggingFace directory into the reference's names (and fused layouts when
    ``model_config.qkv_concat``), keeping the file names, and write ``param_name_map.json`` (parameter -> file).
    Runs in this process; the name is the reference's (mindformers.utils.convert_hf_safetensors_multiprocess)."""
    if not isinstance(src_dir, str) or not isinstance(dst_dir, str):
        raise ValueError("src_dir and dst_dir must be paths")
    if model_config is None:
        raise ValueError("model_config is required")
    if not contains_safetensors_files(src_dir):
        raise ValueError(f"{src_dir} holds no safetensors file")
    from safetensors.numpy import load_file, save_file
    os.makedirs(dst_dir, exist_ok=True)
    files = sorted(f for f in os.listdir(src_dir) if f.endswith(".safetensors"))
    concat = bool(_cfg(model_config, "qkv_concat", False))
    # files that hold a q (gate) part go last, so that the parts they need are already parked
    if concat:
        from safetensors import safe_open

        def leads(f):
            with safe_open(os.path.join(src_dir, f), framework="np") as st:
                return any(convert_name(k).split(".")[-2] in ("wq", "w1") for k in st.keys() if "." in k)
        files.sort(key=lambda f: (leads(f), f))
    pending, name_map, converted = {}, {}, {}
    for f in files:
        converted[f] = convert_weight_dict(load_file(os.path.join(src_dir, f)), model_config, pending)
    if pending:
        raise ValueError(f"unmatched q/k/v or gate/up parts: {sorted(pending)}")
    for f, d in converted.items():
        if d:
            save_file({k: np.ascontiguousarray(v) for k, v in d.items()}, os.path.join(dst_dir, f))
        name_map.update({k: f for k in d})
    with open(os.path.join(dst_dir, NAME_MAP_FILE), "w") as fh:
        json.dump(name_map, fh, indent=2)
    return name_map


# ------------------------------------------------------------------------------------------- one decode layer
class _TensorSource:
    """Parameter name -> array over a directory (with param_name_map.json / an index file), a list of files, or a
    dict of arrays.  Files are opened lazily and only the requested tensors are read."""

    def __init__(self, source):
        self._dict, self._where = None, {}
        if isinstance(source, dict):
            self._dict = source
            return
        from safetensors import safe_open
        if isinstance(source, str) and os.path.isdir(source):
            for idx in (NAME_MAP_FILE, HF_INDEX_FILE):
                p = os.path.join(source, idx)
                if os.path.exists(p):
                    with open(p) as fh:
                        m = json.load(fh)
                    m = m.get("weight_map", m)
                    self._where = {k: os.path.join(source, v) for k, v in m.items()}
                    return
            source = [os.path.join(source, f) for f in sorted(os.listdir(source)) if f.endswith(".safetensors")]
        elif isinstance(source, str):
            source = [source]
        for f in source:
            with safe_open(f, framework="np") as st:
                for k in st.keys():
                    self._where[k] = f

    def __contains__(self, name):
        return name in (self._dict if self._dict is not None else self._where)

    def get(self, name):
        if self._dict is not None:
            return np.asarray(self._dict[name])
        from safetensors import safe_open
        with safe_open(self._where[name], framework="np") as st:
            return st.get_tensor(name)


def quantize_rtn_int8(weight):
    """Symmetric per-output-channel round-to-nearest int8: scale = max|row| / 127 (float32), quotient in float64,
    ties to even, clipped to +-127.  The same convention as WeightQuantLinearCell.quantize_from_float."""
    w = np.asarray(weight, dtype=np.float64)
    scale = (np.abs(w).max(axis=1) / 127.0).astype(np.float32)
    safe = np.where(scale > 0, scale, np.float32(1)).astype(np.float64)
    q = np.clip(np.rint(w / safe[:, None]), -127, 127).astype(np.int8)
    return q, scale


def _to_float(a):
    """safetensors' numpy view of bf16 is not available: such tensors must be stored as fp16/fp32 for this loader."""
    a = np.asarray(a)
    if a.dtype.kind not in "fi":
        raise TypeError(f"unsupported tensor dtype {a.dtype}")
    return a


def read_layer_arrays(source, layer, model_config, prefix="model.layers."):
    """Collect the arrays of decode layer ``layer`` in this build's layout — qkv rows [q | k | v], fc1 rows
    [gate | hidden] — from a checkpoint in HuggingFace names, in the reference's names (separate wq/wk/wv, w1/w3) or
    in its fused per-kv-group / interleaved layouts (w_qkv, w_gate_hidden).

    Returns {"qkv", "wo", "fc1", "fc2": (weight, scale-or-None, bias-or-None, smooth-or-None), "attn_norm",
    "ffn_norm"}; an int8 weight comes with its ``w_scale``."""
    src = source if isinstance(source, _TensorSource) else _TensorSource(source)
    num_heads = _cfg(model_config, "num_heads")
    n_kv = _cfg(model_config, "n_kv_heads") or num_heads
    hidden = _cfg(model_config, "hidden_size")
    base = f"{prefix}{layer}."

    def name_of(mf_suffix):
        """The key present in the checkpoint for a reference-style suffix (or its HuggingFace spelling)."""
        if base + mf_suffix in src:
            return base + mf_suffix
        module, _, leaf = mf_suffix.rpartition(".")
        hf = _MF_TO_HF_MODULE.get(module)
        if hf is not None and f"{base}{hf}.{leaf}" in src:
            return f"{base}{hf}.{leaf}"
        return None

    def linear(kind, perm=None):
        w_name = name_of(f"{kind}.weight")
        if w_name is None:
            return None
        stem = w_name[:-len("weight")]
        w = _to_float(src.get(w_name))
        get = lambda s: _to_float(src.get(stem + s)) if (stem + s) in src else None
        scale, bias, smooth = get("w_scale"), get("bias"), get("smooth_scale")
        if w.dtype == np.int8 and scale is None:
            raise KeyError(f"{w_name} is int8 but {stem}w_scale is missing")
        if perm is not None:
            w, scale, bias = perm(w), (perm(scale) if scale is not None else None), (perm(bias) if bias is not None else None)
        return w, scale, bias, smooth

    def fuse(parts):
        ws, scales, biases, smooths = zip(*parts)
        if any(w.dtype != ws[0].dtype for w in ws):
            raise TypeError("the parts of a fused projection must have one dtype")
        scale = np.concatenate(scales) if scales[0] is not None else None
        bias = np.concatenate(biases) if all(b is not None for b in biases) else None
        return np.concatenate(ws, 0), scale, bias, smooths[0]

    out = {}
    fused_qkv = linear(f"attention.{QKV_CONCAT_KEY}", lambda t: qkv_concat_mg2hf(t, num_heads, n_kv, hidden))
    if fused_qkv is not None:
        out["qkv"] = fused_qkv
    else:
        parts = [linear(f"attention.{k}") for k in ("wq", "wk", "wv")]
        if any(p is None for p in parts):
            raise KeyError(f"layer {layer}: neither {QKV_CONCAT_KEY} nor wq/wk/wv found under {base}")
        out["qkv"] = fuse(parts)
    out["wo"] = linear("attention.wo")
    fused_ffn = linear(f"feed_forward.{FFN_CONCAT_KEY}", lambda t: ffn_concat_mg2hf(t, t.shape[0] // 2))
    if fused_ffn is not None:
        out["fc1"] = fused_ffn
    else:
        parts = [linear(f"feed_forward.{k}") for k in ("w1", "w3")]
        if any(p is None for p in parts):
            raise KeyError(f"layer {layer}: neither {FFN_CONCAT_KEY} nor w1/w3 found under {base}")
        out["fc1"] = fuse(parts)
    out["fc2"] = linear("feed_forward.w2")
    for k in ("wo", "fc2"):
        if out[k] is None:
            raise KeyError(f"layer {layer}: {k} weight not found under {base}")
    for ours, suffix in (("attn_norm", "attention_norm.weight"), ("ffn_norm", "ffn_norm.weight")):
        n = name_of(suffix)
        if n is None:
            raise KeyError(f"layer {layer}: {suffix} not found under {base}")
        out[ours] = _to_float(src.get(n)).astype(np.float32)
    return out


def load_decode_layer(source, layer, model_config, act_quant=False, dtype=None, device="cuda", eps=None):
    """Build a ``QuantDecodeLayer`` for layer ``layer`` of a checkpoint (see read_layer_arrays for the accepted
    formats): float weights are quantized to int8 per output channel, int8 weights are taken with their scales; the
    weights are then packed for the GEMM kernels."""
    import torch
    from .decode_layer import QuantDecodeLayer
    arrays = read_layer_arrays(source, layer, model_config)
    num_heads = _cfg(model_config, "num_heads")
    n_kv = _cfg(model_config, "n_kv_heads") or num_heads
    hidden = _cfg(model_config, "hidden_size")
    head_dim = hidden // num_heads
    ffn = arrays["fc2"][0].shape[1]
    dtype = dtype or torch.bfloat16
    eps = eps if eps is not None else (_cfg(model_config, "rms_norm_eps") or 1e-5)
    net = QuantDecodeLayer(hidden, num_heads, n_kv, head_dim, ffn, eps=eps, dtype=dtype, act_quant=act_quant,
                           qkv_bias=arrays["qkv"][2] is not None, device=device)
    for name in QuantDecodeLayer.NAMES:
        w, scale, bias, smooth = arrays[name]
        if w.dtype != np.int8:
            w, scale = quantize_rtn_int8(w)
        want = tuple(getattr(net, f"{name}_w").shape)
        if tuple(w.shape) != want:
            raise ValueError(f"{name}: checkpoint weight is {tuple(w.shape)}, the layer wants {want}")
        getattr(net, f"{name}_w").copy_(torch.from_numpy(np.ascontiguousarray(w)))
        getattr(net, f"{name}_s").copy_(torch.from_numpy(np.ascontiguousarray(scale, dtype=np.float32)))
        if bias is not None:
            if name != "qkv":
                raise NotImplementedError(f"{name}: a bias on this projection is not built")
            net.qkv_b.copy_(torch.from_numpy(np.ascontiguousarray(bias, dtype=np.float32)).to(dtype))
        if act_quant and smooth is not None:
            getattr(net, f"{name}_smooth").copy_(torch.from_numpy(np.ascontiguousarray(smooth, dtype=np.float32)))
    net.attn_norm.copy_(torch.from_numpy(arrays["attn_norm"]))
    net.ffn_norm.copy_(torch.from_numpy(arrays["ffn_norm"]))
    return net.prepare()
