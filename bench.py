#!/usr/bin/env python3
"""Benchmark of the quantized decode step on one MI355X.

A "step" is one pass of one decode layer over one batch: the Llama-3.1-8B-shape W8A16 layer at batch 64
(hidden 4096, 32 query / 8 KV heads, head_dim 128, FFN 14336, context lengths uniform in [512, 4096], bf16 KV
cache in 128-token blocks behind a shuffled block table), synthetic seeded inputs already resident in HBM.
The timed steps are chained in one HIP graph, each taking the hidden state of the one before, and walk through
separately allocated copies of the layer (own weights, own KV caches; --copies), as the layers of a model do.
Prints ONE JSON line: decode tokens/s per layer, the HBM roofline of the dominant kernel (paged attention,
timed live with events on the launch stream) and the CPU restatement of the same path timed on the host
cores on a bounded sample.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-graph] [--no-cpu] [--copies C]

Workloads: llama3_8b_w8a16 (default), llama3_8b_w8a16_kv8, tiny_llama_w8a16, qwen2_5_7b_w8a8, qwen2_5_72b_w8a16
(layer steps); deepseek_v3_moe_w8a16 (one MoE layer step); deepseek_v3_mla_layer (one multi-latent attention layer step);
deepseek_v3_mla_decode, llama3_8b_prefill_attention,
llama3_8b_chunked_prefill_attention, deepseek_v3_mla_prefill_attention (one attention call per step).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0         # MI355X published dense int8 MFMA rate

# metric string per workload; the default workload carries the headline metric
METRICS = {
    "llama3_8b_w8a16": "decode tokens/sec per layer (Llama3-8B shape, W8A16, bs64); % of peak HBM GB/s",
    "llama3_8b_w8a16_kv8": "decode tokens/sec per layer (Llama3-8B shape, W8A16, int8 KV cache, bs64); % of peak HBM GB/s",
    "tiny_llama_w8a16": "decode tokens/sec per layer (tiny Llama shape, W8A16, bs4); % of peak HBM GB/s",
    "qwen2_5_7b_w8a8": "decode tokens/sec per layer (Qwen2.5-7B shape, W8A8, bs256); % of peak int8 MFMA TOP/s",
    "qwen2_5_72b_w8a16": "decode tokens/sec per layer (Qwen2.5-72B shape, W8A16, bs16, ctx 16k-32k); % of peak HBM GB/s",
    "deepseek_v3_moe_w8a16": "MoE layer tokens/sec (DeepSeek-V3 shape, 256 experts W8A16, 128 tokens); % of peak HBM GB/s",
}
TRAFFIC_RECORD = os.path.join(ROOT, "profiles", "hbm_traffic.json")
# the decode attention kernels and their launch rule (the prefill side lives in prefill_attention.hip)
ATTENTION_SOURCES = [os.path.join(ROOT, "mindformers_amd", "csrc", n)
                     for n in ("paged_attention_kernels.h", "paged_attention.hip")]
GEMM_SOURCES = [os.path.join(ROOT, "mindformers_amd", "csrc", "w8a16_gemm.hip")]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def run_step(case, repeats=1):
    """``repeats`` decode steps of the config's layer stack (1 layer except the 8-layer long-context config), each
    layer taking the hidden state the one before it produced, as the layers of a model do.  The case may hold
    several separately allocated copies of the stack: consecutive steps then walk through them in turn, so that no
    step finds its weights or its KV blocks in a cache because the step before it has just read them."""
    h, normed = case["x"], case.get("normed")
    layers = case["layers"]
    for j in range(repeats * case["cfg"]["layers"]):
        i = j % len(layers)
        layer, (kc, vc) = layers[i], case["caches"][i]
        # As in a stack of layers, every layer computes the attention norm of the layer after it (here: of the same
        # shape, the stack's first layer again after the last; W8A8: with its quantisation) in the kernel that
        # finishes its last projection, and takes its own normed input from the layer before it.  One step = every
        # projection, the attention and both norms of each layer, as before; the input norm merely sits at the end
        # of the step.
        nxt = layers[(i + 1) % len(layers)]
        nn = (nxt.attn_norm, nxt.eps, nxt.qkv_smooth) if layer.act_quant else (nxt.attn_norm, nxt.eps)
        h, normed = layer(h, kc, vc, case["block_tables"], case["context_lens"], case["slot_mapping"], case["cos"],
                          case["sin"], normed=normed, next_norm=nn)
    return h


def time_events(fn, iters, torch):
    """Average duration (ms) of fn() bracketed by events on the current stream, one pair per call."""
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    for i in range(iters):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    ts = sorted(s.elapsed_time(e) for s, e in zip(starts, ends))
    return sum(ts) / len(ts), ts[len(ts) // 2]


def kernel_breakdown(case, torch, ops, iters):
    """Per-op microseconds for the first layer: each op launched ``iters`` times back to back between two events
    (launch overhead overlaps with execution; repeated weights may be served from the memory-side cache, so the
    GEMM figures are a lower bound of their in-layer time)."""
    layer = case["layers"][0]
    kc, vc = case["caches"][0]
    x = case["x"]
    nq, nkv = layer.n_head * layer.head_dim, layer.n_kv_head * layer.head_dim
    n1 = ops.rms_norm(x, layer.attn_norm, layer.eps)
    qkv = layer._linear(n1, "qkv")
    q, k, v = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:]
    attn = layer.attend(q, kc, vc, case["block_tables"], case["context_lens"])
    h = layer._linear(attn, "wo", residual=x)
    n2 = ops.rms_norm(h, layer.ffn_norm, layer.eps)
    a = layer.gate_up(n2)
    steps = {
        "rmsnorm": lambda: ops.rms_norm(x, layer.attn_norm, layer.eps),
        "qkv_gemm": lambda: layer._linear(n1, "qkv"),
        "rope_and_cache": (lambda: (ops.apply_rotary_pos_emb(q, k, case["cos"], case["sin"], layer.n_head,
                                                             layer.n_kv_head, layer.head_dim),
                                    ops.quant_reshape_and_cache(k, v, kc, vc, case["slot_mapping"], layer.kv_scale,
                                                                layer.kv_offset))) if kc.dtype == torch.int8 else
                          (lambda: ops.rope_and_cache(q, k, v, case["cos"], case["sin"], kc, vc, case["slot_mapping"],
                                                      layer.n_head)),
        "paged_attention": lambda: layer.attend(q, kc, vc, case["block_tables"], case["context_lens"]),
        "wo_gemm": lambda: layer._linear(attn, "wo", residual=x),
        "gate_up_silu_mul": lambda: layer.gate_up(n2),
        "fc2_gemm": lambda: layer._linear(a, "fc2", residual=h),
    }
    out = {}
    for name, fn in steps.items():
        for _ in range(3):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        out[name] = round(start.elapsed_time(end) / iters * 1e3, 2)
    return out


def source_sha256(paths):
    import hashlib
    h = hashlib.sha256()
    for path in paths:
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(workload, kv_bytes):
    """HBM bytes per attention launch from the committed counter record (FETCH_SIZE / WRITE_SIZE of a profiler run,
    scaled by a known-size kernel).  Valid only for the workload, the KV byte count and the kernel source it was
    taken on: otherwise (None, why)."""
    try:
        with open(TRAFFIC_RECORD) as f:
            rec = json.load(f)["paged_attention"]
    except (OSError, KeyError, ValueError):
        return None, "no counter record under profiles/"
    if rec.get("workload") != workload or rec.get("kv_bytes") != kv_bytes:
        return None, "the counter record covers another workload"
    if rec.get("kernel_source_sha256") != source_sha256(ATTENTION_SOURCES):
        return None, "the attention kernel source changed since the counters were read (record of commit %s)" % rec.get("commit")
    return int(rec["traffic_bytes"]), "profiles/hbm_traffic.json, commit %s" % rec.get("commit")


def measured_gemm_chain(workload, weight_bytes):
    """HBM bytes per layer step of the four weight-only GEMMs and the three kernels that carry their split-K sums
    (from the same counter record), against the int8 weight bytes they must read.  Valid for the workload and the GEMM
    source it was taken on: otherwise None."""
    try:
        with open(TRAFFIC_RECORD) as f:
            rec = json.load(f)["gemm_chain"]
    except (OSError, KeyError, ValueError):
        return None
    if rec.get("workload") != workload or rec.get("kernel_source_sha256") != source_sha256(GEMM_SOURCES):
        return None
    return {"traffic": int(rec["traffic_bytes"]), "algorithmic": int(weight_bytes),
            "ratio": round(rec["traffic_bytes"] / weight_bytes, 3), "kernels": rec.get("kernels"),
            "source": "profiles/hbm_traffic.json, commit %s" % rec.get("commit")}


def record_traffic(fetch_csv, write_csv, workload, kv_bytes):
    """Write profiles/hbm_traffic.json from the counter_collection CSVs of two profiler runs of this benchmark with
    --calibrate-counters (one with --pmc FETCH_SIZE, one with --pmc WRITE_SIZE): mean counter value per dispatch of
    the attention kernels, each scaled by what the same counter reads for add_kernel on 2 x 128 MiB inputs."""
    import csv
    import subprocess

    def means(path, counter):
        acc = {}
        with open(path) as f:
            for row in csv.DictReader(f):
                if row.get("Counter_Name") != counter:
                    continue
                acc.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
        return {k: sum(v) / len(v) for k, v in acc.items()}

    def pick(table, needle, exclude=None):
        hits = [v for k, v in table.items() if needle in k and not (exclude and exclude in k)]
        if not hits:
            raise SystemExit(f"no dispatch of {needle} in the counter file")
        return hits[0]
    fetch, write = means(fetch_csv, "FETCH_SIZE"), means(write_csv, "WRITE_SIZE")
    f_scale = 262144.0 / pick(fetch, "add_kernel")             # add_kernel reads 2 x 128 MiB, writes 128 MiB
    w_scale = 131072.0 / pick(write, "add_kernel")
    kib = (pick(fetch, "paged_attention_kernel") + pick(fetch, "paged_attention_reduce_kernel")) * f_scale + \
          (pick(write, "paged_attention_kernel") + pick(write, "paged_attention_reduce_kernel")) * w_scale

    # the GEMM chain of a layer step: every dispatch of its kernels in a --layer-only run, per layer step (one
    # w8a16_reduce_rope_cache_kernel dispatch each)
    def totals(path, counter):
        acc, steps = {}, 0
        with open(path) as f:
            for row in csv.DictReader(f):
                if row.get("Counter_Name") != counter:
                    continue
                name = row["Kernel_Name"]
                for key in ("w8a16_gemm4_kernel", "w8a16_reduce_add_rmsnorm_kernel", "w8a16_reduce_rope_cache_kernel"):
                    if key in name:
                        acc[key] = acc.get(key, 0.0) + float(row["Counter_Value"])
                        steps += key == "w8a16_reduce_rope_cache_kernel"
        return acc, steps
    cf, nf = totals(fetch_csv, "FETCH_SIZE")
    cw, nw = totals(write_csv, "WRITE_SIZE")
    chain = None
    if nf and nw and cf.get("w8a16_gemm4_kernel"):
        per_kernel = {k: int((cf.get(k, 0.0) / nf * f_scale + cw.get(k, 0.0) / nw * w_scale) * 1024) for k in cf}
        chain = {"workload": workload, "traffic_bytes": int(sum(per_kernel.values())), "kernels": per_kernel,
                 "layer_steps": nf, "kernel_source": "mindformers_amd/csrc/w8a16_gemm.hip",
                 "kernel_source_sha256": source_sha256(GEMM_SOURCES)}
    commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    rec = {"paged_attention": {"workload": workload, "kv_bytes": int(kv_bytes), "traffic_bytes": int(kib * 1024),
                               "fetch_scale": round(f_scale, 4), "write_scale": round(w_scale, 4),
                               "commit": commit or "unknown",
                               "kernel_source": "mindformers_amd/csrc/paged_attention_kernels.h + paged_attention.hip",
                               "kernel_source_sha256": source_sha256(ATTENTION_SOURCES)}}
    if chain is not None:
        chain["commit"] = commit or "unknown"
        rec["gemm_chain"] = chain
    with open(TRAFFIC_RECORD, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    log(f"[bench] wrote {TRAFFIC_RECORD}: {rec['paged_attention']['traffic_bytes']} bytes per attention launch" +
        (f", {chain['traffic_bytes']} bytes per layer step for the GEMM chain" if chain else ""))


def cpu_baseline(case, torch, sample_seqs, gpu_out, min_seconds=10.0):
    """Time the numpy restatement of the same layer on the host for ``sample_seqs`` sequences of the batch
    (compact copies of their KV blocks), and compare the GPU rows with it."""
    import oracle as O
    cfg = case["cfg"]
    layer = case["layers"][0]
    kc, vc = case["caches"][0]
    bs = cfg["block_size"]
    idx = list(range(min(sample_seqs, cfg["batch"])))
    tables = case["block_tables"][idx].cpu().numpy()
    lens = case["context_lens_host"][idx]
    used = np.unique(tables[tables >= 0])
    remap = -np.ones(case["num_blocks"], dtype=np.int64)
    remap[used] = np.arange(len(used))
    t2 = np.where(tables >= 0, remap[np.maximum(tables, 0)], -1).astype(np.int32)
    sel = torch.from_numpy(used).to(kc.device)
    kcn = kc[sel].float().cpu().numpy()
    vcn = vc[sel].float().cpu().numpy()
    slots = case["slot_mapping"][idx].cpu().numpy()
    slots2 = (remap[slots // bs] * bs + slots % bs).astype(np.int32)
    p = {}
    for n in layer.NAMES:
        p[n + "_w"] = getattr(layer, n + "_w").cpu().numpy()
        p[n + "_s"] = getattr(layer, n + "_s").cpu().numpy()
    p["attn_norm"] = layer.attn_norm.cpu().numpy()
    p["ffn_norm"] = layer.ffn_norm.cpu().numpy()
    x = case["x"][idx].float().cpu().numpy()
    cos = case["cos"][idx].float().cpu().numpy()
    sin = case["sin"][idx].float().cpu().numpy()
    ocfg = dict(n_head=cfg["n_head"], n_kv_head=cfg["n_kv_head"], head_dim=cfg["head_dim"], eps=1e-5)
    act = "bf16" if cfg["dtype"] == torch.bfloat16 else "fp16"
    got = gpu_out[idx].float().cpu().numpy()
    if cfg["act_quant"]:
        # W8A8: the numpy restatement (float64 dequantisation around exact integer accumulators)
        for n in layer.NAMES:
            p[n + "_smooth"] = getattr(layer, n + "_smooth").cpu().numpy()
        try:
            from threadpoolctl import threadpool_info
            cores = max([i.get("num_threads", 1) for i in threadpool_info()] or [1])
        except Exception:
            cores = 1
        passes, dt = 0, 0.0
        while passes < 16 and dt < min_seconds:    # every pass rewrites the same cache slots with the same rows: identical work
            t0 = time.perf_counter()
            ref = O.decode_layer_w8a8(x, p, ocfg, kcn, vcn, t2, lens, slots2, cos, sin, act_dtype=act)
            dt += time.perf_counter() - t0
            passes += 1
        how = "numpy float64"
    else:
        # W8A16: the same layer restated with torch on the host in float32 on all cores (oracle/torch_cpu.py, held to
        # the float64 oracle by the CPU tests); weights widened to float32 once, outside the timed passes
        from oracle import torch_cpu
        cores = torch.get_num_threads()
        tp = torch_cpu.prepare_params(p)
        xt, ct, st = torch.from_numpy(x), torch.from_numpy(cos), torch.from_numpy(sin)
        kct, vct = torch.from_numpy(kcn), torch.from_numpy(vcn)
        passes, dt = 0, 0.0
        while passes < 256 and dt < min_seconds:
            t0 = time.perf_counter()
            ref = torch_cpu.decode_layer_w8a16_fp32(xt, tp, ocfg, kct, vct, t2, lens, slots2, ct, st, act_dtype=act)
            dt += time.perf_counter() - t0
            passes += 1
        ref = ref.numpy()
        how = "torch float32 on the host"
    err = float(np.abs(got - ref).max())
    scale = float(np.abs(ref).max())
    return dict(value=len(idx) * passes / dt, unit="tokens/s", cores=int(cores), kind="port",
                sample=f"{passes} passes of one layer step for {len(idx)} of the {cfg['batch']} sequences "
                       f"({int(lens.sum())} context tokens), {how}, {dt:.1f} s in all"), dict(
        max_abs_err=err, ref_max_abs=scale, rows=len(idx))


def int8_gemm_roofline(layer, x, torch, ops, iters):
    """The four int8 GEMMs of a W8A8 layer step (QKV, output, gate/up, down projection), each timed with events on
    the launch stream on the operands the layer feeds it: int8 ops (2 M N K, summed) over the summed durations
    against the dense int8 MFMA peak."""
    m = x.shape[0]
    n1q = ops.rms_norm_dynamic_quant(x, layer.attn_norm, layer.eps, layer.qkv_smooth, tiled=True)
    qkv = ops.w8a8_linear(n1q[0], n1q[1], layer._packed["qkv"], out_dtype=layer.dtype)
    attn_q = ops.dynamic_quant(qkv[:, :layer.n_head * layer.head_dim].contiguous(), layer.wo_smooth, tiled=True)
    h = ops.w8a8_linear(attn_q[0], attn_q[1], layer._packed["wo"], out_dtype=layer.dtype, residual=x)
    n2q = ops.rms_norm_dynamic_quant(h, layer.ffn_norm, layer.eps, layer.fc1_smooth, tiled=True)
    gu = ops.w8a8_linear(n2q[0], n2q[1], layer._packed["fc1"], out_dtype=layer.dtype)
    aq = ops.silu_mul_dynamic_quant(gu, layer.fc2_smooth, tiled=True)
    calls = {
        "qkv": lambda: ops.w8a8_linear(n1q[0], n1q[1], layer._packed["qkv"], out_dtype=layer.dtype),
        "wo": lambda: ops.w8a8_linear(attn_q[0], attn_q[1], layer._packed["wo"], out_dtype=layer.dtype, residual=x),
        "gate_up": lambda: ops.w8a8_linear(n2q[0], n2q[1], layer._packed["fc1"], out_dtype=layer.dtype),
        "down": lambda: ops.w8a8_linear(aq[0], aq[1], layer._packed["fc2"], out_dtype=layer.dtype, residual=h),
    }
    shapes = {"qkv": layer._packed["qkv"], "wo": layer._packed["wo"], "gate_up": layer._packed["fc1"],
              "down": layer._packed["fc2"]}
    us, total_ops, weight_bytes = {}, 0.0, 0
    for name, fn in calls.items():
        for _ in range(5):
            fn()
        us[name] = round(time_events(fn, iters, torch)[0] * 1e3, 2)
        total_ops += 2.0 * m * shapes[name].n * shapes[name].k
        weight_bytes += shapes[name].n * shapes[name].k
    total_us = sum(us.values())
    ach = total_ops / (total_us * 1e-6) / 1e12
    return dict(bound="mfma", kernel="int8 GEMMs of the layer step (w8a8_wide_kernel / w8a8_gemm_kernel / w8a8_regs_kernel "
                                     "+ split-K reduce): qkv, wo, gate/up, down", achieved=round(ach, 1),
                peak=INT8_PEAK_TOPS, unit="TOP/s", frac=round(ach / INT8_PEAK_TOPS, 4), traffic=None,
                ops_per_step=total_ops, avg_launch_us=round(total_us, 2), per_gemm_us=us,
                weight_stream_gbps=round(weight_bytes / (total_us * 1e-6) / 1e9, 1))


def w8a8_gemm_leg(torch, ops, synthetic, iters):
    """int8_gemm_roofline on a freshly built Qwen2.5-7B-shape W8A8 layer (hidden 3584, ffn 18944, 28 q / 4 kv heads)
    and 256 activation rows from N(0, 1): the configuration the int8 matrix-core target is quoted on."""
    from mindformers_amd.decode_layer import QuantDecodeLayer
    cfg = synthetic.CONFIGS["qwen2_5_7b_w8a8"]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    layer = synthetic.fill_layer(QuantDecodeLayer(cfg["hidden"], cfg["n_head"], cfg["n_kv_head"], cfg["head_dim"],
                                                  cfg["ffn"], 1e-5, cfg["dtype"], True, device="cuda"), gen)
    x = torch.randn(cfg["batch"], cfg["hidden"], generator=gen, device="cuda").to(cfg["dtype"])
    out = int8_gemm_roofline(layer, x, torch, ops, iters)
    out["workload"] = f"qwen2_5_7b_w8a8 GEMMs: {cfg['batch']} rows, hidden {cfg['hidden']}, ffn {cfg['ffn']}"
    del layer
    torch.cuda.empty_cache()
    return out


def bench_modules(case, torch, ops, args):
    """The same decode-layer step composed from the drop-in cells a user of the reference's module surface gets, one
    launch per primitive and nothing fused across cells: LlamaRMSNorm -> WeightQuantLinearCell (QKV) -> InferAttention
    (RoPE + cache scatter + paged attention on the manager's own caches) -> WeightQuantLinearCell (+ residual) ->
    LlamaRMSNorm -> WeightQuantLinearCell (gate/up) -> SiLU * mul -> WeightQuantLinearCell (+ residual).  Timed like the
    fused layer (HIP graph of chained steps) so that the cost of not adopting the fused entry points is on record."""
    from mindformers_amd.modules import InferAttention, LlamaRMSNorm
    from mindformers_amd.modules.layers import WeightQuantLinearCell
    cfg, layer = case["cfg"], case["layers"][0]
    if layer.act_quant or cfg.get("kv_int8"):
        return {"skipped": "the module leg covers the W8A16 layer with 16-bit caches"}
    dt, dev = cfg["dtype"], case["x"].device
    nq, nkv = cfg["n_head"] * cfg["head_dim"], cfg["n_kv_head"] * cfg["head_dim"]
    freqs = (case["cos"], case["sin"], None)

    def compose(layer, kc, vc):
        """The reference's cells around one layer's weights and caches; returns its step function."""
        cells = {}
        for name in layer.NAMES:
            w = getattr(layer, name + "_w")
            cell = WeightQuantLinearCell(w.shape[1], w.shape[0], False, dt, device="meta")
            cell.weight, cell.w_scale = w.to(dev), getattr(layer, name + "_s")
            cell.prepare()
            cell.weight = w                                         # the packed copy is what the kernels read
            cells[name] = cell
        norm1, norm2 = LlamaRMSNorm(cfg["hidden"], layer.eps, device=dev), LlamaRMSNorm(cfg["hidden"], layer.eps, device=dev)
        norm1.weight.data, norm2.weight.data = layer.attn_norm, layer.ffn_norm
        att = InferAttention(cfg["n_head"], cfg["head_dim"], cfg["n_kv_head"], scale_value=layer.scale_value,
                             block_size=cfg["block_size"], num_blocks=1, rotary_cos_format=2, compute_dtype=dt, device=dev)
        att.paged_attention_mgr.key_cache, att.paged_attention_mgr.value_cache = kc, vc     # the case's caches, not a copy
        att.is_first_iteration = False

        def step(x):
            qkv = cells["qkv"](norm1(x))
            a = att(qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:], case["context_lens"], case["block_tables"],
                    case["slot_mapping"], freqs)
            h = cells["wo"](a, residual=x)
            return cells["fc2"](ops.silu_mul(cells["fc1"](norm2(h))), residual=h)
        return step
    # one composition per separately allocated copy of the layer, walked through in turn like the fused leg
    steps = [compose(l, kc, vc) for l, (kc, vc) in zip(case["layers"], case["caches"])]
    kc, vc = case["caches"][0]
    ref = layer(case["x"], kc, vc, case["block_tables"], case["context_lens"], case["slot_mapping"], case["cos"], case["sin"])
    out = steps[0](case["x"])
    same = bool(torch.equal(out, ref))
    per = next(g for g in (8, 4, 2, 1) if args.steps % g == 0)

    def chain():
        h = case["x"]
        for j in range(per):
            h = steps[j % len(steps)](h)
        return h
    launch = "eager"
    fn = chain
    if not args.no_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    chain()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                chain()
            fn, launch = g.replay, f"hip_graph, {per} chained layer steps per replay"
        except Exception as e:
            log(f"[bench] module leg: graph capture unavailable ({e}); timing eager launches")
    for _ in range(max(1, args.warmup // per)):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps // per):
        fn()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    return {"ms_per_step": round(ms, 4), "tokens_per_s": round(cfg["batch"] / (ms * 1e-3), 1), "launch": launch,
            "bit_identical_to_fused_layer": same,
            "composition": "LlamaRMSNorm, WeightQuantLinearCell x4, InferAttention, silu_mul"}


def bench_moe(args, torch, ops, _lib):
    """DeepSeek-V3-shaped MoE layer on one GPU's share (all 256 experts resident): router top-k (sigmoid, 8 groups,
    4 kept) -> permute -> grouped W8A16 expert MLP -> weighted unpermute + shared expert, 128 bf16 tokens."""
    lib = _lib.load()
    H, E, F, K_TOP, T = 7168, 256, 2048, 8, 128
    dev, dt = "cuda", torch.bfloat16
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    x = torch.randn(T, H, generator=gen, device=dev).to(dt)
    logits = torch.randn(T, E, generator=gen, device=dev)
    ebias = torch.zeros(E, device=dev)

    from mindformers_amd import synthetic

    def quantized(experts, n, k):
        # N(0, 0.02) weights quantised per output channel, generated expert by expert
        w = torch.empty(experts or 1, n, k, dtype=torch.int8, device=dev)
        sc = torch.empty(experts or 1, n, dtype=torch.float32, device=dev)
        for e in range(experts or 1):
            w[e], sc[e] = synthetic.quantize_weight_int8(torch.randn(n, k, generator=gen, device=dev) * 0.02)
        return (w, sc) if experts else (w[0], sc[0])
    raw1, raw2 = quantized(E, 2 * F, H), quantized(E, H, F)
    sraw1, sraw2 = quantized(None, 2 * F, H), quantized(None, H, F)
    w1, w2 = ops.pack_w8a16_gated(*raw1, "halves"), ops.pack_w8a16(*raw2)      # fc1 with silu(gate) * up in its epilogue
    s1, s2 = ops.pack_w8a16_gated(*sraw1, "halves"), ops.pack_w8a16(*sraw2)

    def step():
        wgt, idx = ops.moe_route(logits, ebias, K_TOP, 8, 4, 2.5, dt)
        px, row_map, counts, offsets = ops.moe_permute(x, idx, E)
        y = ops.grouped_w8a16_linear(ops.grouped_w8a16_linear(px, w1, offsets), w2, offsets)
        shared = ops.w8a16_linear(ops.w8a16_gated_linear(x, s1), s2)
        return ops.moe_unpermute(y, row_map, wgt, shared=shared), counts
    out, counts = step()
    torch.cuda.synchronize()
    n_act = int((counts > 0).sum().item())
    per_expert = 3 * H * F
    alg_bytes = (n_act + 1) * per_expert
    launch, run = "eager", step
    if not args.no_graph:
        # the whole layer step is device-side (no host sync between router and unpermute): replay it as one HIP graph
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out_graph, _ = step()
            for _ in range(3):                     # replays must reproduce the eager result, with eager work in between
                graph.replay()
                torch.cuda.synchronize()
                if not torch.equal(out_graph, out):
                    raise RuntimeError("graph replay differs from the eager result")
                step()
                torch.cuda.synchronize()
            launch, run = "hip_graph, one layer step per replay", graph.replay
        except Exception as e:
            log(f"[bench] HIP graph capture unavailable ({e}); timing eager launches")
            launch, run = "eager", step
    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3

    def timed(fn):
        for _ in range(3):
            fn()
        st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        st.record()
        for _ in range(args.kernel_iters):
            fn()
        en.record()
        torch.cuda.synchronize()
        return st.elapsed_time(en) / args.kernel_iters
    wgt, idx = ops.moe_route(logits, ebias, K_TOP, 8, 4, 2.5, dt)
    px, row_map, counts, offsets = ops.moe_permute(x, idx, E)
    g1 = timed(lambda: ops.grouped_w8a16_linear(px, w1, offsets))
    a = ops.grouped_w8a16_linear(px, w1, offsets)
    g2 = timed(lambda: ops.grouped_w8a16_linear(a, w2, offsets))
    parity = None if args.no_cpu else moe_parity(torch, out, x, logits, ebias, raw1, raw2, sraw1, sraw2, K_TOP, F)
    ach = n_act * per_expert / ((g1 + g2) * 1e-3) / 1e9
    result = {
        "metric": METRICS["deepseek_v3_moe_w8a16"],
        "value": round(T / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"deepseek_v3_moe_w8a16: one MoE layer step, {T} tokens, hidden {H}, {E} experts x ffn {F}, "
                               f"top-{K_TOP} of 4/8 groups, 1 shared expert, W8A16; {n_act} experts received rows",
                   "launch": launch, "algorithmic_bytes_per_layer": alg_bytes},
        "layer_hbm_gbps": round(alg_bytes / (ms * 1e-3) / 1e9, 1),
        "layer_hbm_frac": round(alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "roofline": dict(bound="hbm", kernel="w8a16_grouped_kernel (fc1 + fc2 launches)", achieved=round(ach, 1),
                         peak=HBM_PEAK_GBPS, unit="GB/s", frac=round(ach / HBM_PEAK_GBPS, 4), traffic=None,
                         bytes_per_launch=n_act * per_expert, avg_launch_us=round((g1 + g2) * 1e3, 2),
                         per_launch_us={"fc1_silu_mul": round(g1 * 1e3, 2), "fc2": round(g2 * 1e3, 2)}),
    }
    if parity is not None:
        result["parity_vs_cpu"] = parity
    print(json.dumps(result), flush=True)


def moe_parity(torch, out, x, logits, ebias, raw1, raw2, sraw1, sraw2, k_top, f):
    """The layer's output rows of a few tokens against the CPU oracle: router choice on all tokens, then the dense
    sum over the chosen experts of w * fc2(silu(gate) * up) + the shared expert, rounded where the device stores."""
    import oracle as O
    from oracle import dense as Dn
    from oracle import quant as Q
    from oracle.layer import _r

    def npf(t):
        return t.float().cpu().numpy() if t.dtype.is_floating_point else t.cpu().numpy()
    w_ref, idx_ref = O.topk_router(npf(logits), npf(ebias), k_top, 8, 4, 2.5)
    w_ref = _r(w_ref, "bf16")
    worst, scale = 0.0, 0.0
    for t in (0, 31, 64, 127):
        xt = npf(x[t:t + 1]).astype(np.float64)
        acc = 0.0
        for j in range(k_top):
            e = int(idx_ref[t, j])
            h1 = _r(Q.w8a16_linear(xt, npf(raw1[0][e]), npf(raw1[1][e])), "bf16")
            a = _r(_r(Dn.silu(h1[:, :f]), "bf16") * h1[:, f:], "bf16")
            acc = acc + w_ref[t, j] * _r(Q.w8a16_linear(a, npf(raw2[0][e]), npf(raw2[1][e])), "bf16")
        h1 = _r(Q.w8a16_linear(xt, npf(sraw1[0]), npf(sraw1[1])), "bf16")
        a = _r(_r(Dn.silu(h1[:, :f]), "bf16") * h1[:, f:], "bf16")
        ref = _r(acc, "bf16") + _r(Q.w8a16_linear(a, npf(sraw2[0]), npf(sraw2[1])), "bf16")
        worst = max(worst, float(np.abs(npf(out[t:t + 1]) - ref).max()))
        scale = max(scale, float(np.abs(ref).max()))
    return dict(max_abs_err=worst, ref_max_abs=scale, rows=4)


def bench_prefill_attention(args, torch, ops):
    """Causal attention of a Llama-3-8B-shaped prefill step over the paged cache (32 q / 8 kv heads x 128, bf16,
    block 128): `llama3_8b_prefill_attention` = 4 prompts of 2048 tokens, `llama3_8b_chunked_prefill_attention` =
    4 sequences adding 512 tokens behind 3584 cached ones.  A step is one attention call; flops = 4 * D * heads *
    (query, key) pairs inside the causal limit.  `deepseek_v3_mla_prefill_attention` = the prefill of multi-latent
    attention (multi_latent_attention.py:405-432): 4 prompts of 2048 tokens, 128 heads, queries and keys 192 wide,
    values 128 wide (what the layer has; the reference pads them to 192 and drops the extra output columns), taken
    from the step's own packed rows (no cache); flops = 2 * (192 + 128) * heads * pairs."""
    mla = args.workload == "deepseek_v3_mla_prefill_attention"
    nh, nkv, d, bs, dt = (128, 128, 192, 128, torch.bfloat16) if mla else (32, 8, 128, 128, torch.bfloat16)
    chunked = args.workload == "llama3_8b_chunked_prefill_attention"
    lens = np.full(4, 4096 if chunked else 2048)
    q_lens = np.full(4, 512 if chunked else 2048)
    need = (lens + bs - 1) // bs
    nb = int(need.sum()) + 1
    tables = -np.ones((len(lens), int(need.max())), np.int32)
    perm, pos = np.random.default_rng(0).permutation(nb), 0
    for i, n in enumerate(need):
        tables[i, :n] = perm[pos:pos + n]
        pos += n
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    t = int(q_lens.sum())
    if mla:
        kc = torch.randn(t, nkv * d, generator=gen, device="cuda").to(dt)
        vc = torch.randn(t, nkv * 128, generator=gen, device="cuda").to(dt)
    else:
        kc = torch.randn(nb, bs, nkv, d, generator=gen, device="cuda").to(dt)
        vc = torch.randn(nb, bs, nkv, d, generator=gen, device="cuda").to(dt)
    q = torch.randn(t, nh * d, generator=gen, device="cuda").to(dt)
    starts = torch.tensor(np.concatenate([[0], np.cumsum(q_lens)]), dtype=torch.int32, device="cuda")
    lens_t = torch.tensor(lens, dtype=torch.int32, device="cuda")
    tb = torch.tensor(tables, device="cuda")
    out = torch.empty(t, nh * 128, dtype=dt, device="cuda") if mla else torch.empty_like(q)

    def step():
        if mla:
            return ops.causal_attention_varlen(q, kc, vc, starts, nh, nkv, d ** -0.5, out=out)
        return ops.paged_attention_prefill(q, kc, vc, tb, lens_t, starts, nh, nkv, d ** -0.5, out=out)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    us = time_events(step, args.kernel_iters, torch)[0] * 1e3
    pairs = int(sum(int(ql) * (int(L) - int(ql)) + int(ql) * (int(ql) + 1) // 2 for L, ql in zip(lens, q_lens)))
    flops = (2.0 * (192 + 128) if mla else 4.0 * d) * nh * pairs
    ach = flops / (us * 1e-6) / 1e12
    peak = 2500.0
    result = {
        "metric": f"prefill attention query tokens/sec per layer ({'DeepSeek-V3 MLA' if mla else 'Llama3-8B'} heads, bf16); "
                  "% of dense bf16 MFMA peak",
        "value": round(t / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: causal attention over "
                               f"{'the packed rows of the step' if mla else 'the paged cache'}, {len(lens)} sequences, "
                               f"{int(q_lens[0])} new tokens each, context {int(lens[0])}, {nh}q/{nkv}kv heads x {d}"
                               f"{' (values 128 wide)' if mla else ''}"
                               f"{'' if mla else ', block 128'}",
                   "launch": "eager", "flops_per_step": flops},
        "roofline": dict(bound="mfma", kernel="prefill_attention_kernel (+ partition reduce when partitioned)",
                         achieved=round(ach, 1), peak=peak, unit="TFLOP/s", frac=round(ach / peak, 4), traffic=None,
                         flops_per_launch=flops, avg_launch_us=round(us, 2)),
    }
    print(json.dumps(result), flush=True)


def bench_mla_decode(args, torch, ops):
    """DeepSeek-V3-shaped multi-latent attention decode: 128 heads over one latent cache row per token (512 latent
    + 64 rotary, bf16), batch 64, context lengths uniform in [512, 4096], block 128.  A step is one attention call;
    consecutive calls walk through 4 separately allocated caches (170 MB each), as the layers of a model do, so that
    no call finds its rows in the memory-side cache.  flops = 2 * (576 + 512) per (token, head)."""
    nh, dk, dv, bs, b, dt = 128, 576, 512, 128, 64, torch.bfloat16
    rng = np.random.default_rng(1)
    lens = rng.integers(512, 4097, b).astype(np.int32)
    need = (lens + bs - 1) // bs
    nb = int(need.sum()) + 2
    tables = -np.ones((b, 4096 // bs), np.int32)
    perm, pos = rng.permutation(nb), 0
    for i, n in enumerate(need):
        tables[i, :n] = perm[pos:pos + n]
        pos += n
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    caches = [torch.randn(nb, bs, 1, dk, generator=gen, device="cuda").to(dt) for _ in range(4)]
    q = torch.randn(b, nh * dk, generator=gen, device="cuda").to(dt)
    tb, lt = torch.from_numpy(tables).cuda(), torch.from_numpy(lens).cuda()
    out = torch.empty(b, nh * dv, dtype=dt, device="cuda")

    turn = [0]

    def step():
        turn[0] = (turn[0] + 1) % len(caches)
        return ops.mla_paged_attention(q, caches[turn[0]], tb, lt, nh, dv, 192 ** -0.5, out=out)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    us = time_events(step, args.kernel_iters, torch)[0] * 1e3
    tokens = int(lens.astype(np.int64).sum())
    flops = 2.0 * (dk + dv) * nh * tokens
    ach = flops / (us * 1e-6) / 1e12
    kv_bytes = tokens * dk * 2
    result = {
        "metric": "MLA decode attention tokens/sec per layer (DeepSeek-V3 heads, bf16); % of dense bf16 MFMA peak",
        "value": round(b / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"deepseek_v3_mla_decode: multi-latent attention decode, batch {b}, {nh} heads, latent "
                               f"512 + rope 64, ctx U[512,4096] (sum {tokens}), block {bs}, 4 caches in turn",
                   "launch": "eager", "flops_per_step": flops, "cache_bytes_per_step": kv_bytes},
        "hbm_gbps_on_cache_bytes": round(kv_bytes / (us * 1e-6) / 1e9, 1),
        "roofline": dict(bound="mfma", kernel="mla_decode_kernel (+ mla_reduce_kernel)", achieved=round(ach, 1),
                         peak=2500.0, unit="TFLOP/s", frac=round(ach / 2500.0, 4), traffic=None,
                         flops_per_launch=flops, avg_launch_us=round(us, 2)),
    }
    print(json.dumps(result), flush=True)


def bench_mla_layer(args, torch, ops):
    """DeepSeek-V3-shaped multi-latent self-attention layer, one decode step through the module surface
    (MLASelfAttention): hidden 7168, 128 heads, q_lora_rank 1536, kv_lora_rank 512, 128 + 64 query dims, batch 64,
    contexts uniform in [512, 4096], block 128, bf16; the down / up / output projections are W8A16 cells, the absorbed
    per-head projections read linear_kv_up_proj's bf16 weight.  A step is one forward of the layer (projections,
    norms, RoPE, latent-row scatter, absorbed query, attention over the latent cache, absorbed output, output
    projection), replayed from a HIP graph of 4 steps on 4 separate weight sets."""
    from mindformers_amd.modules import MLASelfAttention, MLATransformerConfig
    from mindformers_amd.modules.quantizers import AutoQuantizer
    hidden, nh, q_lora, rank, nope, rope, vd, bs, b, dt = 7168, 128, 1536, 512, 128, 64, 128, 128, 64, torch.bfloat16
    rng = np.random.default_rng(1)
    lens = rng.integers(512, 4097, b).astype(np.int32)
    need = (lens + bs - 1) // bs
    nb = int(need.sum()) + 2
    tables = -np.ones((b, 4096 // bs), np.int32)
    perm, pos = rng.permutation(nb), 0
    for i, n in enumerate(need):
        tables[i, :n] = perm[pos:pos + n]
        pos += n
    slots = np.array([tables[i, (l - 1) // bs] * bs + (l - 1) % bs for i, l in enumerate(lens)], np.int32)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    cfg = MLATransformerConfig(hidden_size=hidden, num_attention_heads=nh, q_lora_rank=q_lora, kv_lora_rank=rank,
                               qk_head_dim=nope, qk_pos_emb_head_dim=rope, v_head_dim=vd, rope_type="yarn",
                               layernorm_epsilon=1e-6, compute_dtype="bfloat16", params_dtype="bfloat16")
    n_layers = 4
    layers, caches = [], []
    for _ in range(n_layers):
        net = MLASelfAttention(cfg, layer_number=1)
        for name in ("linear_qkv_down_proj", "linear_q_up_proj", "linear_kv_up_proj", "linear_proj"):
            w = getattr(net, name).weight
            w.data.copy_((torch.randn(w.shape, generator=gen, device="cuda") * w.shape[1] ** -0.5).to(dt))
        q = AutoQuantizer.from_config({"quant_method": "rtn", "weight_dtype": "int8",
                                       "modules_to_not_convert": ["linear_kv_up_proj"]})
        q.preprocess_model(net)
        q.postprocess_model(net)
        net.prepare()
        net.is_prefill = False
        layers.append(net)
        caches.append(torch.randn(nb, bs, 1, rank + rope, generator=gen, device="cuda").to(dt))
    x = torch.randn(b, hidden, generator=gen, device="cuda").to(dt)
    tb, lt, sl = torch.from_numpy(tables).cuda(), torch.from_numpy(lens).cuda(), torch.from_numpy(slots).cuda()
    pos_t = (lt - 1).to(torch.int64)
    cos, sin = layers[0].rotary_pos_emb.get_cos_sin_for_decode(pos_t)

    def one(i):
        return layers[i](x, rotary_pos_cos=cos, rotary_pos_sin=sin, batch_valid_length=lt, block_tables=tb,
                         slot_mapping=sl, key_cache=caches[i])

    def chain():
        for i in range(n_layers):
            one(i)
    for _ in range(3):
        chain()
    torch.cuda.synchronize()
    graph = None
    if not args.no_graph:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            chain()
    run = graph.replay if graph is not None else chain
    for _ in range(max(1, args.warmup // n_layers)):
        run()
    torch.cuda.synchronize()
    reps = max(1, args.steps // n_layers)
    t0 = time.perf_counter()
    for _ in range(reps):
        run()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / (reps * n_layers) * 1e3
    # the pieces, each timed alone with events (eager launches, warm weights: lower bounds of their time in the layer)
    net = layers[0]
    xq = net.linear_qkv_down_proj(x)
    q_c = net.q_layernorm(xq[:, :q_lora])
    qq = net.linear_q_up_proj(q_c).reshape(b, nh, nope + rope)
    query = torch.empty((b, nh, rank + rope), dtype=dt, device="cuda")
    attn = torch.randn(b, nh, rank, generator=gen, device="cuda").to(dt)
    core = torch.randn(b, nh * vd, generator=gen, device="cuda").to(dt)
    qa_t, out_absorb = net._absorb
    turn = [0]

    def next_cache():                                         # the layers' caches in turn: every call reads cold rows
        turn[0] = (turn[0] + 1) % n_layers
        return caches[turn[0]]
    pieces = {
        "qkv_down_proj": lambda: net.linear_qkv_down_proj(x),
        "q_up_proj": lambda: net.linear_q_up_proj(q_c),
        "absorb_query_bmm": lambda: ops.mla_absorb_bmm(qq[..., :nope], qa_t, out=query[..., :rank]),
        "mla_paged_attention": lambda: ops.mla_paged_attention(query.reshape(b, -1), next_cache(), tb, lt, nh, rank,
                                                               net.softmax_scale),
        "absorb_output_bmm": lambda: ops.mla_absorb_bmm(attn, out_absorb),
        "linear_proj": lambda: net.linear_proj(core),
    }
    us = {}
    for name, fn in pieces.items():
        for _ in range(3):
            fn()
        us[name] = round(time_events(fn, args.kernel_iters, torch)[0] * 1e3, 2)
    tokens = int(lens.astype(np.int64).sum())
    w_bytes = (q_lora + rank + rope) * hidden + nh * (nope + rope) * q_lora + 2 * nh * (nope + vd) * rank + hidden * nh * vd
    cache_bytes = tokens * (rank + rope) * 2
    flops = 2.0 * (rank + rope + rank) * nh * tokens
    ach = flops / (us["mla_paged_attention"] * 1e-6) / 1e12
    result = {
        "metric": "decode tokens/sec per multi-latent attention layer (DeepSeek-V3 shape, W8A16 projections, bs64)",
        "value": round(b / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": reps * n_layers,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"deepseek_v3_mla_layer: MLASelfAttention decode step, batch {b}, hidden {hidden}, {nh} "
                               f"heads, q_lora {q_lora}, latent {rank} + rope {rope}, ctx U[512,4096] (sum {tokens}), "
                               f"block {bs}, W8A16 projections",
                   "launch": "eager" if graph is None else f"hip_graph, {n_layers} layer steps on separate weights per replay",
                   "algorithmic_bytes_per_layer": int(w_bytes + cache_bytes), "weight_bytes": int(w_bytes),
                   "cache_bytes": int(cache_bytes)},
        "layer_hbm_gbps": round((w_bytes + cache_bytes) / (ms * 1e-3) / 1e9, 1),
        "unfused_op_us": us,
        "roofline": dict(bound="mfma", kernel="mla_decode_kernel (+ mla_reduce_kernel)", achieved=round(ach, 1),
                         peak=2500.0, unit="TFLOP/s", frac=round(ach / 2500.0, 4), traffic=None,
                         flops_per_launch=flops, avg_launch_us=us["mla_paged_attention"]),
    }
    print(json.dumps(result), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="llama3_8b_w8a16")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a captured HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--modules", action="store_true",
                    help="also time the step composed from the drop-in module cells (default for the headline workload)")
    ap.add_argument("--no-modules", action="store_true", help="skip the drop-in module leg")
    ap.add_argument("--no-w8a8", action="store_true", help="skip the W8A8 int8 GEMM leg of the default workload")
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: turn the counter_collection CSVs of two profiler runs of this command with "
                         "--calibrate-counters (--pmc FETCH_SIZE, --pmc WRITE_SIZE) into profiles/hbm_traffic.json")
    ap.add_argument("--cpu-seqs", type=int, default=64, help="sequences of the batch the CPU baseline runs")
    ap.add_argument("--kernel-iters", type=int, default=50)
    ap.add_argument("--copies", type=int, default=8,
                    help="separately allocated copies of the layer (weights and KV caches) the chained steps walk "
                         "through; 1 = every step re-reads the same weights, which the memory-side cache may then hold")
    ap.add_argument("--layer-only", action="store_true",
                    help="run the warm-up and the timed layer steps and nothing else (no per-op loops, no other legs): "
                         "under a counter-collecting profiler every dispatch then belongs to a layer step")
    ap.add_argument("--calibrate-counters", action="store_true",
                    help="also launch add_kernel on 2 x 128 MiB inputs (reads 256 MiB, writes 128 MiB): the known-size "
                         "kernel that hardware traffic counters of a profiler run are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); the decode path has no "
              "collectives and no multi-GPU figure is produced.", file=sys.stderr)
        sys.exit(2)

    if args.record_traffic:
        from mindformers_amd import synthetic as syn
        cfg = syn.CONFIGS[args.workload]
        kv = int(syn.context_lens(args.workload, seed=1).astype(np.int64).sum()) * 2 * cfg["n_kv_head"] * cfg["head_dim"] * \
            (1 if cfg.get("kv_int8") else 2)
        record_traffic(args.record_traffic[0], args.record_traffic[1], args.workload, kv)
        return

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from mindformers_amd import _lib, ops, synthetic
    _lib.load()                                    # fail loudly if the HIP library is not built
    torch.cuda.set_device(0)

    if args.workload == "deepseek_v3_moe_w8a16":
        bench_moe(args, torch, ops, _lib)
        return
    if args.workload == "deepseek_v3_mla_decode":
        bench_mla_decode(args, torch, ops)
        return
    if args.workload == "deepseek_v3_mla_layer":
        bench_mla_layer(args, torch, ops)
        return
    if args.workload in ("llama3_8b_prefill_attention", "llama3_8b_chunked_prefill_attention",
                         "deepseek_v3_mla_prefill_attention"):
        bench_prefill_attention(args, torch, ops)
        return

    t0 = time.perf_counter()
    stack = synthetic.CONFIGS[args.workload]["layers"]
    copies = max(1, min(args.copies, 8 // stack))
    case = synthetic.make_decode_case(args.workload, seed=1, copies=copies)
    cfg = case["cfg"]
    nbytes = synthetic.algorithmic_bytes(case)
    torch.cuda.synchronize()
    log(f"[bench] built {args.workload}: batch {cfg['batch']}, sum(ctx) {int(case['context_lens_host'].sum())}, "
        f"weights {nbytes['weights'] / 1e6:.1f} MB, KV {nbytes['kv'] / 1e6:.1f} MB per layer ({time.perf_counter() - t0:.1f} s)")

    # what the layer before the first one hands over: its output's norm under the first layer's gamma (W8A8: quantised)
    first = case["layers"][0]
    if first.act_quant:
        case["normed"] = ops.rms_norm_dynamic_quant(case["x"], first.attn_norm, first.eps, first.qkv_smooth, tiled=True)
    else:
        case["normed"] = ops.rms_norm(case["x"], first.attn_norm, first.eps)
    out_eager = run_step(case)
    torch.cuda.synchronize()
    if args.calibrate_counters:
        ca = torch.ones(64 << 20, dtype=torch.bfloat16, device="cuda")
        cb_ = torch.ones(64 << 20, dtype=torch.bfloat16, device="cuda")
        for _ in range(3):
            ops.add(ca, cb_)
        torch.cuda.synchronize()
        del ca, cb_

    use_graph = not args.no_graph
    graph = None
    # A model runs all its layers in one graph launch; a launch per layer step would add the gap between two graph
    # launches (4-8 us here) to every step.  One replay therefore covers up to 8 layer steps in a row (a divisor of
    # --steps, so that exactly that many steps are timed), each taking the hidden state of the one before.
    per_replay = 1
    if use_graph:
        per_replay = next(g for g in (8, 4, 2, 1) if g * cfg["layers"] <= 8 and args.steps % g == 0)
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    chain_eager = run_step(case, per_replay)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out_graph = run_step(case, per_replay)
            # replays must reproduce the eager result bit for bit, with eager work in between
            for _ in range(3):
                graph.replay()
                torch.cuda.synchronize()
                if not torch.equal(out_graph, chain_eager):
                    raise RuntimeError("graph replay differs from the eager result")
                run_step(case)
                torch.cuda.synchronize()
        except Exception as e:                     # fall back to eager launches, say so
            log(f"[bench] HIP graph capture unavailable ({e}); timing eager launches")
            graph, per_replay = None, 1
    step = graph.replay if graph is not None else (lambda: run_step(case))

    for _ in range((args.warmup + per_replay - 1) // per_replay):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps // per_replay):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    n_layers = cfg["layers"]
    tokens_per_s_layer = cfg["batch"] * n_layers * args.steps / elapsed
    if args.layer_only:
        print(json.dumps({"metric": METRICS.get(args.workload, METRICS["llama3_8b_w8a16"]),
                          "value": round(tokens_per_s_layer, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
                          "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "layer_only": True}), flush=True)
        return

    # dominant kernel: paged attention, event-timed on the launch stream
    layer = case["layers"][0]
    kc, vc = case["caches"][0]
    nq = layer.n_head * layer.head_dim
    qkv = layer._linear(ops.rms_norm(case["x"], layer.attn_norm, layer.eps), "qkv")
    q = qkv[:, :nq]

    def attn():
        return layer.attend(q, kc, vc, case["block_tables"], case["context_lens"])
    for _ in range(5):
        attn()
    attn_ms, attn_med = time_events(attn, args.kernel_iters, torch)
    achieved = nbytes["kv"] / (attn_ms * 1e-3) / 1e9
    # HBM bytes per launch from hardware counters (FETCH_SIZE + WRITE_SIZE of a profiler run of this command,
    # scaled by a known-size kernel); only valid for the exact workload it was collected on
    traffic, traffic_note = measured_traffic(args.workload, nbytes["kv"])
    roofline = dict(bound="hbm", kernel="paged_attention_kernel (+ partition reduce)", achieved=round(achieved, 1),
                    peak=HBM_PEAK_GBPS, unit="GB/s", frac=round(achieved / HBM_PEAK_GBPS, 4), traffic=traffic,
                    traffic_source=traffic_note, bytes_per_launch=nbytes["kv"], avg_launch_us=round(attn_ms * 1e3, 2))
    breakdown = kernel_breakdown(case, torch, ops, args.kernel_iters)
    layer_gbps = nbytes["total"] * n_layers / (ms_per_step * 1e-3) / 1e9
    extra = {}
    if cfg["act_quant"]:
        # W8A8: the figure of merit is the int8 matrix rate of the four projections at this batch; the attention
        # roofline moves to a second key
        extra["attention_roofline"] = roofline
        roofline = int8_gemm_roofline(case["layers"][0], case["x"], torch, ops, args.kernel_iters)
    if args.modules or (args.workload == "llama3_8b_w8a16" and not args.no_modules):
        extra["drop_in_modules"] = bench_modules(case, torch, ops, args)
    if args.workload == "llama3_8b_w8a16" and not args.no_w8a8:
        # the second figure of merit rides on the default line: the four int8 GEMMs of the Qwen2.5-7B-shape W8A8 layer
        # at batch 256 (no KV cache needed), against the dense int8 matrix-core peak
        extra["w8a8_int8_gemm_roofline"] = w8a8_gemm_leg(torch, ops, synthetic, args.kernel_iters)

    result = {
        "metric": METRICS.get(args.workload, METRICS["llama3_8b_w8a16"]),
        "value": round(tokens_per_s_layer, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if cfg["dtype"] == torch.bfloat16 else "fp16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: one decode layer step, batch {cfg['batch']}, hidden {cfg['hidden']}, "
                               f"{cfg['n_head']}q/{cfg['n_kv_head']}kv heads x {cfg['head_dim']}, ffn {cfg['ffn']}, "
                               f"ctx U[{cfg['ctx'][0]},{cfg['ctx'][1]}], block {cfg['block_size']}, "
                               f"{'W8A8' if cfg['act_quant'] else 'W8A16'}, layers {n_layers}",
                   "launch": (f"hip_graph, {per_replay} chained layer steps per replay" if graph is not None
                              else "eager") + (f", over {copies} separately allocated copies of the layer"
                                               if copies > 1 else ", every step on the same weights and caches"),
                   "algorithmic_bytes_per_layer": nbytes["total"]},
        "layer_hbm_gbps": round(layer_gbps, 1), "layer_hbm_frac": round(layer_gbps / HBM_PEAK_GBPS, 4),
        "roofline": roofline,
        # each op of the unfused layer launched back to back on its own (not a split of ms_per_step: the timed step
        # runs the fused entry points inside one graph)
        "unfused_op_us": breakdown,
    }
    result.update(extra)
    chain = None if cfg["act_quant"] else measured_gemm_chain(args.workload, nbytes["weights"])
    if chain is not None:
        result["gemm_chain"] = chain
    if cfg.get("kv_int8"):
        result["config"]["kv_cache"] = "int8, per-channel scales"
    if not args.no_cpu and not cfg.get("kv_int8"):            # the CPU restatement of the layer covers 16-bit caches
        cb, parity = cpu_baseline(case, torch, args.cpu_seqs, out_eager)
        result["cpu_baseline"] = cb
        result["parity_vs_cpu"] = parity
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
