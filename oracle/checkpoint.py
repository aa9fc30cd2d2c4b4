"""Fused-weight row layouts of the reference's checkpoints, written as per-row loops.  Test infrastructure only.

Follows mindformers/utils/convert_utils.py:65-92 (qkv: HuggingFace [q | k | v] rows -> one block per kv head,
[the q heads that share it | its k | its v]) and :95-106 (ffn: [gate | hidden] halves -> rows alternating
gate_j, hidden_j).  Pinned by hand-computed small cases and by the labelled-row structure in the tests.
"""
import numpy as np


def qkv_concat_hf2mg(qkv, num_heads, n_kv_heads, hidden_size):
    qkv = np.asarray(qkv)
    d = hidden_size // num_heads
    n_rep = num_heads // n_kv_heads
    q, k, v = qkv[:hidden_size], qkv[hidden_size:hidden_size + n_kv_heads * d], qkv[hidden_size + n_kv_heads * d:]
    rows = []
    for g in range(n_kv_heads):
        for h in range(g * n_rep, (g + 1) * n_rep):           # the query heads served by kv head g
            for i in range(d):
                rows.append(q[h * d + i])
        for i in range(d):
            rows.append(k[g * d + i])
        for i in range(d):
            rows.append(v[g * d + i])
    return np.stack(rows)


def ffn_concat_hf2mg(ffn, ffn_hidden_size):
    ffn = np.asarray(ffn)
    rows = []
    for j in range(ffn_hidden_size):
        rows.append(ffn[j])
        rows.append(ffn[ffn_hidden_size + j])
    return np.stack(rows)
