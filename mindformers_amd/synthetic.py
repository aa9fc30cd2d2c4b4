"""Seeded synthetic decode workloads of the shapes the benchmark quotes, and round-to-nearest weight
quantisation (symmetric per-output-channel int8) done with torch on the device at load time.

Weights ~ N(0, 0.02) quantised to int8; activations ~ N(0, 1); KV cache filled with N(0, 1) values in
fixed-size blocks reached through a shuffled block table; context lengths uniform in [lo, hi].
"""
import math

import numpy as np
import torch

from .decode_layer import QuantDecodeLayer

# name -> shape parameters (hidden, heads, kv heads, head_dim, ffn, batch, context range, block size, dtype)
CONFIGS = {
    "tiny_llama_w8a16": dict(hidden=512, n_head=8, n_kv_head=2, head_dim=64, ffn=1376, batch=4, ctx=(32, 256),
                             block_size=16, dtype=torch.float16, act_quant=False, theta=10000.0, layers=1),
    "llama3_8b_w8a16": dict(hidden=4096, n_head=32, n_kv_head=8, head_dim=128, ffn=14336, batch=64, ctx=(512, 4096),
                            block_size=128, dtype=torch.bfloat16, act_quant=False, theta=500000.0, layers=1),
    # the bench shape with an int8 KV cache (per-channel scales): half the attention bytes
    "llama3_8b_w8a16_kv8": dict(hidden=4096, n_head=32, n_kv_head=8, head_dim=128, ffn=14336, batch=64,
                                ctx=(512, 4096), block_size=128, dtype=torch.bfloat16, act_quant=False,
                                theta=500000.0, layers=1, kv_int8=True),
    "qwen2_5_7b_w8a8": dict(hidden=3584, n_head=28, n_kv_head=4, head_dim=128, ffn=18944, batch=256, ctx=(2048, 2048),
                            block_size=128, dtype=torch.bfloat16, act_quant=True, theta=1000000.0, layers=1),
    "qwen2_5_72b_w8a16": dict(hidden=8192, n_head=64, n_kv_head=8, head_dim=128, ffn=29568, batch=16,
                              ctx=(16384, 32768), block_size=128, dtype=torch.bfloat16, act_quant=False,
                              theta=1000000.0, layers=8),
}


def quantize_weight_int8(w):
    """Symmetric per-output-channel int8 of a float weight [out, in]: s = max|w|/127, q = clip(rint(w/s), +-127)."""
    w = w.double()
    scale = (w.abs().amax(dim=1) / 127.0).float()
    safe = torch.where(scale > 0, scale, torch.ones_like(scale)).double()
    q = torch.clamp(torch.round(w / safe[:, None]), -127, 127).to(torch.int8)
    return q, scale


def rope_rows(positions, head_dim, theta, dtype, device):
    """cos/sin rows [T, head_dim] = cos/sin(concat(f, f)) at the given positions, stored in ``dtype``."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
    f = positions.to(device=device, dtype=torch.float32)[:, None] * inv[None, :]
    emb = torch.cat((f, f), dim=-1)
    return torch.cos(emb).to(dtype), torch.sin(emb).to(dtype)


def fill_layer(layer, gen, std=0.02):
    """Random N(0, std) weights quantised to int8, unit-ish norm gammas, smoothing vectors U[0.5, 2]."""
    dev = layer.attn_norm.device
    for name in layer.NAMES:
        wq = getattr(layer, f"{name}_w")
        n, k = wq.shape
        rows = max(1, min(n, (64 << 20) // (4 * k)))           # generate in slabs of <= 64 MiB of fp32
        for r0 in range(0, n, rows):
            w = torch.randn(min(rows, n - r0), k, generator=gen, device=dev) * std
            q, s = quantize_weight_int8(w)
            wq[r0:r0 + q.shape[0]] = q
            getattr(layer, f"{name}_s")[r0:r0 + q.shape[0]] = s
        if layer.act_quant:
            getattr(layer, f"{name}_smooth").copy_(torch.rand(k, generator=gen, device=dev) * 1.5 + 0.5)
    layer.attn_norm.copy_(1.0 + 0.1 * torch.randn(layer.hidden, generator=gen, device=dev))
    layer.ffn_norm.copy_(1.0 + 0.1 * torch.randn(layer.hidden, generator=gen, device=dev))
    return layer.prepare(release_raw=True)                      # the packed copy is the only one on the device


def context_lens(name, seed=0, batch=None, ctx=None):
    """The context lengths make_decode_case draws for a named config (host only)."""
    cfg = CONFIGS[name]
    lo, hi = ctx if ctx is not None else cfg["ctx"]
    return np.random.default_rng(seed).integers(lo, hi + 1, batch if batch is not None else cfg["batch"]).astype(np.int32)


def make_decode_case(name, seed=0, device="cuda", batch=None, ctx=None, layers=None, copies=1):
    """Build the layer(s) and one decode step's inputs for a named config.  Returns a dict.  ``copies`` > 1 builds
    that many separately allocated instances of the config's layer stack (own weights, own KV caches, same block
    table and lengths), so that steps chained one after another read no byte an earlier step has left in a cache."""
    cfg = dict(CONFIGS[name])
    if batch is not None:
        cfg["batch"] = batch
    if ctx is not None:
        cfg["ctx"] = ctx
    if layers is not None:
        cfg["layers"] = layers
    dt, b, bs = cfg["dtype"], cfg["batch"], cfg["block_size"]
    rng = np.random.default_rng(seed)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)

    lens = rng.integers(cfg["ctx"][0], cfg["ctx"][1] + 1, b).astype(np.int32)     # includes the new token
    need = [(int(l) + bs - 1) // bs for l in lens]
    max_blocks = (cfg["ctx"][1] + bs - 1) // bs
    num_blocks = int(sum(need)) + 2
    perm = rng.permutation(num_blocks)
    tables = -np.ones((b, max_blocks), dtype=np.int32)
    pos = 0
    for i, n in enumerate(need):
        tables[i, :n] = perm[pos:pos + n]
        pos += n
    slots = np.array([tables[i, (int(l) - 1) // bs] * bs + (int(l) - 1) % bs for i, l in enumerate(lens)], dtype=np.int32)

    layers_ = []
    caches = []
    kv_shape = (num_blocks, bs, cfg["n_kv_head"], cfg["head_dim"])
    for _ in range(cfg["layers"] * copies):
        layer = QuantDecodeLayer(cfg["hidden"], cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"], cfg["ffn"], 1e-5, dt,
                                 cfg["act_quant"], device=device)
        layers_.append(fill_layer(layer, gen))
        kv8 = bool(cfg.get("kv_int8"))
        kc = torch.empty(kv_shape, dtype=torch.int8 if kv8 else dt, device=device)
        vc = torch.empty(kv_shape, dtype=torch.int8 if kv8 else dt, device=device)
        for c in (kc, vc):
            flat = c.view(-1)
            step = 1 << 26
            for o in range(0, flat.numel(), step):
                n = min(step, flat.numel() - o)
                r = torch.randn(n, generator=gen, device=device)
                # int8: N(0, 1) values on a grid of 1/32 (what quantising N(0, 1) rows with scale 1/32 leaves)
                flat[o:o + n] = torch.clamp(torch.round(r * 32), -128, 127).to(torch.int8) if kv8 else r.to(dt)
        if kv8:
            row = cfg["n_kv_head"] * cfg["head_dim"]
            layer.set_kv_quant(torch.full((2, row), 1.0 / 32, dtype=torch.float32, device=device))
        caches.append((kc, vc))

    x = torch.randn(b, cfg["hidden"], generator=gen, device=device).to(dt)
    lens_t = torch.from_numpy(lens).to(device)
    cos, sin = rope_rows(lens_t - 1, cfg["head_dim"], cfg["theta"], dt, device)
    return dict(cfg=cfg, layers=layers_, caches=caches, x=x, block_tables=torch.from_numpy(tables).to(device),
                context_lens=lens_t, slot_mapping=torch.from_numpy(slots).to(device), cos=cos, sin=sin,
                context_lens_host=lens, num_blocks=num_blocks)


def algorithmic_bytes(case):
    """HBM bytes one decode step must move per layer: int8 weights once + the K/V rows of every context token
    (2 tensors x n_kv x head_dim x element size).  Activations, scales and the one new KV row are < 0.1 %."""
    cfg = case["cfg"]
    esz = 1 if cfg.get("kv_int8") else 2
    weights = case["layers"][0].weight_bytes()
    kv = int(case["context_lens_host"].astype(np.int64).sum()) * 2 * cfg["n_kv_head"] * cfg["head_dim"] * esz
    return dict(weights=weights, kv=kv, total=weights + kv)
