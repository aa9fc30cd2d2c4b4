"""The W8A16 decode layer of oracle/layer.py restated with torch on the host in float32, all cores.  TEST
INFRASTRUCTURE ONLY: it exists to be *timed* as the CPU baseline of the benchmark (a float64 numpy pass flatters
the GPU by the cost of double precision); tests/test_oracle_golden.py holds it to the float64 oracle.

Follows the same reference lines as oracle/layer.py (mindformers/models/llama/llama_transformer.py:1036-1070 with
the attention of :467-569, mindformers/models/llama/llama_layer.py:412-441) and rounds through the activation dtype
at the same points; the arithmetic in between is float32 instead of float64.
"""
import numpy as np
import torch

_DT = {"bf16": torch.bfloat16, "fp16": torch.float16}


def prepare_params(p):
    """int8 weights widened to float32 once (a host path would keep them like this), scales and gammas as tensors."""
    out = {}
    for k, v in p.items():
        t = torch.from_numpy(np.ascontiguousarray(v))
        out[k] = t.float() if t.dtype in (torch.int8, torch.float64, torch.float16) else t
    return out


def _r(x, dt):
    return x.to(dt).float()


def _rms_norm(x, gamma, eps):
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gamma


def _rope(x, cos, sin, heads):
    t = x.shape[0]
    xh = x.reshape(t, heads, -1)
    half = xh.shape[-1] // 2
    rot = torch.cat((-xh[..., half:], xh[..., :half]), dim=-1)
    return (xh * cos[:, None, :] + rot * sin[:, None, :]).reshape(t, -1)


def decode_layer_w8a16_fp32(x, tp, cfg, key_cache, value_cache, block_tables, context_lens, slot_mapping, cos, sin,
                            act_dtype="bf16"):
    """x float32 [B, hidden] (values of the activation dtype); ``tp`` from prepare_params; caches float32 torch
    tensors [blocks, block_size, n_kv, D], updated in place; one new token per sequence.  Returns float32 [B, hidden]."""
    dt = _DT[act_dtype]
    n_head, n_kv, d = cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"]
    eps = cfg.get("eps", 1e-5)
    nb, bs = key_cache.shape[0], key_cache.shape[1]

    def lin(a, name):
        return (a @ tp[name + "_w"].t()) * tp[name + "_s"]

    n1 = _r(_rms_norm(x, tp["attn_norm"], eps), dt)
    qkv = _r(lin(n1, "qkv"), dt)
    q, k, v = torch.split(qkv, [n_head * d, n_kv * d, n_kv * d], dim=-1)
    q = _r(_rope(q, cos, sin, n_head), dt)
    k = _r(_rope(k, cos, sin, n_kv), dt)
    slots = torch.as_tensor(np.asarray(slot_mapping), dtype=torch.long)
    live = slots >= 0
    key_cache.view(nb * bs, n_kv * d)[slots[live]] = k[live]
    value_cache.view(nb * bs, n_kv * d)[slots[live]] = v[live]
    n_rep = n_head // n_kv
    scale = 1.0 / float(np.sqrt(d))
    attn = torch.zeros(x.shape[0], n_head * d)
    tables = torch.as_tensor(np.asarray(block_tables), dtype=torch.long)
    for b in range(x.shape[0]):
        length = int(context_lens[b])
        if length <= 0:
            continue
        j = torch.arange(length)
        rows = tables[b][j // bs] * bs + j % bs
        kb = key_cache.view(nb * bs, n_kv, d)[rows].permute(1, 0, 2)        # [n_kv, L, D]
        vb = value_cache.view(nb * bs, n_kv, d)[rows].permute(1, 0, 2)
        qb = q[b].reshape(n_kv, n_rep, d)
        s = torch.bmm(qb, kb.transpose(1, 2)) * scale                       # [n_kv, n_rep, L]
        # softmax in float32, probabilities cast to the compute dtype, then PV (infer_attention.py:318-327)
        pr = _r(torch.softmax(s, dim=-1), dt)
        attn[b] = torch.bmm(pr, vb).reshape(-1)
    attn = _r(attn, dt)
    h = _r(x + _r(lin(attn, "wo"), dt), dt)
    n2 = _r(_rms_norm(h, tp["ffn_norm"], eps), dt)
    gu = _r(lin(n2, "fc1"), dt)
    f = gu.shape[-1] // 2
    a = _r(_r(torch.nn.functional.silu(gu[:, :f]), dt) * gu[:, f:], dt)
    return _r(h + _r(lin(a, "fc2"), dt), dt)
