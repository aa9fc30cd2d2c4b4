"""Top-k router, expert permute, grouped expert MLP, unpermute.  Test infrastructure only.

Follows:
  router          mindformers/parallel_core/inference/transformer/moe/router.py:114-148 (FusedAddTopKDiv call),
                  unfused: research/deepseek3/moe.py:763-778; primitive level:
                  mindformers/modules/transformer/moe.py:1529-1576 (sigmoid, +bias, per-group sum of top-2,
                  keep topk_group groups, masked top-k, gather unbiased score, renormalise, *scale)
  permute         MoeInitRoutingV2 call mindformers/parallel_core/inference/transformer/moe/moe_layer.py:136-146;
                  primitive-level restatement modules/transformer/moe.py:1942-1957 (sort by expert, gather rows,
                  one-hot count)
  experts         mindformers/parallel_core/inference/transformer/moe/experts.py:107-170 (weights [E, in, out],
                  [gate | hidden] contiguous split, hidden * silu(gate))
  unpermute       MoeTokenUnpermute call moe_layer.py:151-155
  shared expert   mindformers/parallel_core/inference/transformer/moe/shared_experts.py:65-75, added moe_layer.py:159-160

Index conventions that the vendor primitives keep internal (flattening order of the (token, choice) pairs,
tie-breaking of top-k) are chosen here: pairs are flattened token-major (t*k + j), the sort by expert is
stable, and ties go to the lower expert index.  The layer result does not depend on the first two.
"""
import numpy as np

from .dense import linear, silu
from .numerics import round_to


def _topk_desc(values, k):
    """Indices of the k largest along the last axis, descending, ties to the lower index."""
    order = np.argsort(-values, axis=-1, kind="stable")
    return order[..., :k]


def topk_router(logits, expert_bias, k, n_group, topk_group, routed_scaling_factor, renorm=True,
                group_topk_inner=2):
    """logits [T, E] (float32 scores before sigmoid).  Returns (weights float64 [T,k], index int32 [T,k]).

    With n_group == topk_group (or n_group <= 1) group limiting keeps every expert and this is plain
    biased top-k (router.py:142-146)."""
    s = 1.0 / (1.0 + np.exp(-np.asarray(logits, dtype=np.float64)))
    t, e = s.shape
    sb = s + (0.0 if expert_bias is None else np.asarray(expert_bias, dtype=np.float64)[None, :])
    masked = sb
    if n_group and n_group > 1 and topk_group and topk_group < n_group:
        g = sb.reshape(t, n_group, e // n_group)
        inner = np.sort(g, axis=-1)[..., ::-1][..., :group_topk_inner]
        gscore = inner.sum(axis=-1)                                   # [T, n_group]
        top_vals = np.sort(gscore, axis=-1)[..., ::-1][..., :topk_group]
        gmask = gscore >= top_vals.min(axis=-1, keepdims=True)        # moe.py:1546-1548
        emask = np.repeat(gmask, e // n_group, axis=-1)
        masked = np.where(emask, sb, 0.0)                             # masked_fill(~mask, 0.0), moe.py:1555
    idx = _topk_desc(masked, k)
    w = np.take_along_axis(s, idx, axis=-1)
    if renorm and k > 1:
        w = w / w.sum(axis=-1, keepdims=True)
    w = w * routed_scaling_factor
    return w, idx.astype(np.int32)


def moe_permute(x, expert_index, num_experts):
    """Expand and sort rows by expert.  Returns (permuted_x [T*k, H], row_map int32 [T*k], counts int64 [E]);
    row_map[t*k + j] is the permuted row that holds token t's copy for its j-th expert."""
    x = np.asarray(x)
    t, k = expert_index.shape
    flat = np.asarray(expert_index).reshape(-1).astype(np.int64)
    order = np.argsort(flat, kind="stable")              # permuted row r holds pair order[r]
    row_map = np.empty(t * k, dtype=np.int32)
    row_map[order] = np.arange(t * k, dtype=np.int32)
    permuted = x[order // k]
    counts = np.bincount(flat, minlength=num_experts).astype(np.int64)
    return permuted, row_map, counts


def grouped_matmul(x, weights, counts):
    """Rows are grouped contiguously per expert (counts); y[rows_e] = x[rows_e] @ weights[e]; weights [E,in,out]."""
    x = np.asarray(x, dtype=np.float64)
    out = np.zeros((x.shape[0], weights.shape[2]), dtype=np.float64)
    start = 0
    for e, c in enumerate(counts):
        c = int(c)
        if c:
            out[start:start + c] = x[start:start + c] @ np.asarray(weights[e], dtype=np.float64)
        start += c
    return out


def grouped_mlp(x, weight1, weight2, counts, act_dtype=None):
    """fc1 -> [gate | hidden] -> hidden * silu(gate) -> fc2 (experts.py:151-170)."""
    h = grouped_matmul(x, weight1, counts)
    if act_dtype is not None:
        h = round_to(h, act_dtype).astype(np.float64)
    f = h.shape[-1] // 2
    a = h[:, f:] * silu(h[:, :f])
    if act_dtype is not None:
        a = round_to(a, act_dtype).astype(np.float64)
    return grouped_matmul(a, weight2, counts)


def moe_unpermute(y, row_map, probs):
    """out[t] = sum_j probs[t,j] * y[row_map[t*k+j]]."""
    t, k = probs.shape
    y = np.asarray(y, dtype=np.float64)
    p = np.asarray(probs, dtype=np.float64)
    return (y[row_map.reshape(t, k)] * p[..., None]).sum(axis=1)


def moe_layer(x, gate_weight, expert_bias, weight1, weight2, k, n_group, topk_group, scale,
              shared_fc1=None, shared_fc2=None, act_dtype=None, router_dtype=None):
    """Whole layer (moe_layer.py:126-163).  gate_weight [E, H]; weight1 [E, H, 2F]; weight2 [E, F, H];
    shared_fc1 [2F_s, H], shared_fc2 [H, F_s].  ``act_dtype`` rounds materialised activations,
    ``router_dtype`` rounds the gate logits (the router's Dense runs in moe_router_dtype, router.py:48-51,63)."""
    x64 = np.asarray(x, dtype=np.float64)
    logits = linear(x64, gate_weight)
    if router_dtype is not None:
        logits = round_to(logits, router_dtype).astype(np.float64)
    w, idx = topk_router(logits.astype(np.float32), expert_bias, k, n_group, topk_group, scale)
    if act_dtype is not None:
        w = round_to(w, act_dtype).astype(np.float64)       # expert_weight.astype(input_dtype), router.py:147
    e = gate_weight.shape[0]
    px, row_map, counts = moe_permute(x64, idx, e)
    y = grouped_mlp(px, weight1, weight2, counts, act_dtype)
    if act_dtype is not None:
        y = round_to(y, act_dtype).astype(np.float64)
    out = moe_unpermute(y, row_map, w)
    if act_dtype is not None:
        out = round_to(out, act_dtype).astype(np.float64)
    if shared_fc1 is not None:
        from .dense import mlp
        out = out + mlp(x64, shared_fc1, shared_fc2, gated=True, act_dtype=act_dtype)
    return out
