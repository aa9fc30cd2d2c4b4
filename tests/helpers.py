"""Shared helpers for the parity tests: dtype conversion between torch and the numpy oracle, tolerances."""
import numpy as np
import torch

import oracle as O

EPS = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}
NAME = {torch.bfloat16: "bf16", torch.float16: "fp16"}


def to_np(t):
    """torch tensor (any float dtype / int) -> numpy; bf16/fp16 become float32 holding the same values."""
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.detach().float().cpu().numpy()
    return t.detach().cpu().numpy()


def rounded(a, dtype):
    """numpy float array rounded through the torch storage dtype (float32 result)."""
    return O.round_to(np.asarray(a, dtype=np.float32), NAME[dtype])


def dev(a, dtype, device="cuda"):
    """numpy -> device tensor of dtype."""
    return torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=dtype)


def assert_within(got, ref, mag, dtype, ulps=1.5, extra=0.0, what=""):
    """|got - ref| <= ulps * eps(dtype) * mag + extra, elementwise; ``mag`` is the magnitude the rounding error
    scales with (>= |ref|: e.g. sum of |terms| for a dot product)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    mag = np.maximum(np.asarray(mag, dtype=np.float64), np.abs(ref))
    tol = ulps * EPS[dtype] * mag + extra
    err = np.abs(got - ref)
    bad = err > tol
    assert not bad.any(), (f"{what}: {int(bad.sum())}/{bad.size} outside tolerance; worst err {err.max():.3e} "
                           f"vs tol {tol.flat[np.argmax(err - tol)]:.3e}")


def make_paged_cache(rng, batch, ctx_lens, n_kv, head_dim, block_size, dtype, extra_blocks=3, max_blocks=None,
                     std=1.0):
    """Random K/V caches with a shuffled block table.  Returns numpy (float32, storage-rounded) caches,
    int32 block_tables [B, max_blocks] padded with -1, and the number of blocks."""
    need = [(int(l) + block_size - 1) // block_size for l in ctx_lens]
    max_blocks = max_blocks or max(max(need), 1)
    num_blocks = sum(need) + extra_blocks
    perm = rng.permutation(num_blocks)
    tables = -np.ones((batch, max_blocks), dtype=np.int32)
    pos = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[pos:pos + n]
        pos += n
    kc = rounded(rng.normal(0, std, (num_blocks, block_size, n_kv, head_dim)), dtype)
    vc = rounded(rng.normal(0, std, (num_blocks, block_size, n_kv, head_dim)), dtype)
    return kc, vc, tables, num_blocks


def untile_int8(buf, m, k):
    """Row-major [m, k] view of a buffer in 16 x 64 tile order (tiles ordered [s][mt]; byte (16*g + r)*16 + j of tile (mt, s) holds
    element [16*mt + r, 64*s + 16*g + j])."""
    mt, ks = (m + 15) // 16, (k + 63) // 64
    t = buf[: mt * ks * 1024].reshape(ks, mt, 4, 16, 16)        # [s, mt, g, r, j]
    return t.transpose(1, 3, 0, 2, 4).reshape(mt * 16, ks * 64)[:m, :k]
