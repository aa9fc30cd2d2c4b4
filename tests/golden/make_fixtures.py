"""Dump the reference's own numpy-only test vectors into .npz fixtures.

Runs only in the build container (needs the reference tree).  The reference
keeps, next to each inference unit test, a ``data_gen_utils.py`` that imports
nothing but numpy and holds (a) the seeded input generator and (b) hard-coded
expected outputs: ``GOLDEN_DATA`` (fp32 CPU golden) and ``GPU_DATA`` (a bf16
GPU run) for its "double benchmark" comparison.  This script loads those data
files by path, replays the input generation exactly as the reference's runner
scripts do (same seed, same draw order, same arguments) and writes inputs and
expected outputs as plain arrays.  Nothing of the reference's source text is
stored: the fixtures are data only.

Reference locations (relative to the reference root):
  tests/st/test_ut/test_parallel_core/test_inference/test_transformer/
      test_flash_attention/{data_gen_utils.py,run_infer_flash_attention.py:203-207}
      test_attention/{data_gen_utils.py,run_infer_attention.py}
      test_norm, test_activation, test_mlp, test_moe
  tests/st/test_ut/test_parallel_core/test_inference/test_tensor_parallel/
      test_column_parallel_linear, test_row_parallel_linear
  tests/st/test_ut/test_parallel_core/test_inference/test_common/test_embeddings/
      test_rotary_pos_embedding

Usage:  python tests/golden/make_fixtures.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
BASE = "tests/st/test_ut/test_parallel_core/test_inference"


def _load(ref_root, rel, name):
    path = os.path.join(ref_root, BASE, rel, "data_gen_utils.py")
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _flat(prefix, d):
    return {f"{prefix}{k}": np.asarray(v) for k, v in d.items()}


def dump_flash_attention(ref_root):
    m = _load(ref_root, "test_transformer/test_flash_attention", "fa_data")
    out = {}
    for case, n_kv in (("1", 2), ("2", 1)):
        # each reference case runs in a fresh process: module import seeds 2025,
        # the runner's main() seeds 2025 again, then draws query, key, value.
        np.random.seed(2025)
        p = m.get_init_params(n_kv_heads=n_kv)
        for k, v in p.items():
            out[f"in{case}_{k}"] = np.asarray(v)
    out.update(_flat("golden_", m.GOLDEN_DATA))
    out.update(_flat("gpu_", m.GPU_DATA))
    out["meta_num_blocks"] = np.int64(m.NUM_BLOCKS)
    out["meta_block_size"] = np.int64(m.BLOCK_SIZE)
    out["meta_num_heads"] = np.int64(m.NUM_HEADS)
    out["meta_hidden_size"] = np.int64(m.HIDDEN_SIZE)
    np.savez_compressed(os.path.join(HERE, "flash_attention.npz"), **out)


def dump_attention(ref_root):
    m = _load(ref_root, "test_transformer/test_attention", "attn_data")
    out = {}
    for case, n_kv in (("1", 2), ("2", 1)):
        np.random.seed(2025)
        p = m.get_init_params(n_kv_heads=n_kv)
        for k, v in p.items():
            out[f"in{case}_{k}"] = np.asarray(v)
    out.update(_flat("golden_", m.GOLDEN_DATA))
    out.update(_flat("gpu_", m.GPU_DATA))
    out["meta_num_blocks"] = np.int64(m.NUM_BLOCKS)
    out["meta_block_size"] = np.int64(m.BLOCK_SIZE)
    out["meta_num_heads"] = np.int64(m.NUM_HEADS)
    out["meta_hidden_size"] = np.int64(m.HIDDEN_SIZE)
    np.savez_compressed(os.path.join(HERE, "attention.npz"), **out)


def dump_rotary(ref_root):
    m = _load(ref_root, "test_common/test_embeddings/test_rotary_pos_embedding", "rope_data")
    out = {}
    # prefill cases: batch 2, seq 2; decode cases: batch 2, seq 1 (test_infer_rotary_embedding.py:34-130)
    out.update(_flat("in_prefill_", m.get_init_params(2, 2, m.KV_CHANNELS)))
    out.update(_flat("in_decode_", m.get_init_params(2, 1, m.KV_CHANNELS)))
    out.update(_flat("golden_", m.GOLDEN_DATA))
    out.update(_flat("gpu_", m.GPU_DATA))
    out["meta_kv_channels"] = np.int64(m.KV_CHANNELS)
    out["meta_max_position_embedding"] = np.int64(m.MAX_POSITION_EMBEDDING)
    np.savez_compressed(os.path.join(HERE, "rotary.npz"), **out)


def dump_norm(ref_root):
    m = _load(ref_root, "test_transformer/test_norm", "norm_data")
    out = _flat("in_", m.get_init_params(2, 2, 32))
    out.update(_flat("golden_", m.GOLDEN_DATA))
    out.update(_flat("gpu_", m.GPU_DATA))
    np.savez_compressed(os.path.join(HERE, "norm.npz"), **out)


def dump_activation(ref_root):
    m = _load(ref_root, "test_transformer/test_activation", "act_data")
    out = _flat("in_", m.get_init_params(2, 2, 32))
    out.update(_flat("golden_", m.GOLDEN_DATA))
    out.update(_flat("gpu_", m.GPU_DATA))
    np.savez_compressed(os.path.join(HERE, "activation.npz"), **out)


def dump_mlp(ref_root):
    m = _load(ref_root, "test_transformer/test_mlp", "mlp_data")
    out = _flat("in_", m.get_init_params(m.INPUT_SIZE, m.FFN_HIDDEN_SIZE))
    out.update(_flat("golden_", m.GOLDEN_DATA))
    out.update(_flat("gpu_", m.GPU_DATA))
    np.savez_compressed(os.path.join(HERE, "mlp.npz"), **out)


def dump_moe(ref_root):
    m = _load(ref_root, "test_transformer/test_moe", "moe_data")
    # test_infer_moe.py:31-58: seq_len 4, batch 4, hidden 32, 8 experts, ffn 8
    p = m.get_init_params(4, 4, 32, 8, 8)
    out = {"in_" + k.replace(".", "__"): np.asarray(v) for k, v in p.items()}
    out.update(_flat("golden_", m.GOLDEN_DATA))
    np.savez_compressed(os.path.join(HERE, "moe.npz"), **out)


def dump_linear(ref_root):
    for kind in ("column", "row"):
        m = _load(ref_root, f"test_tensor_parallel/test_{kind}_parallel_linear", f"{kind}_data")
        out = _flat("in_", m.get_init_params(32, 32))
        out.update(_flat("legacy_", m.LEGACY_DATA))
        np.savez_compressed(os.path.join(HERE, f"{kind}_parallel_linear.npz"), **out)


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    dump_flash_attention(ref_root)
    dump_attention(ref_root)
    dump_rotary(ref_root)
    dump_norm(ref_root)
    dump_activation(ref_root)
    dump_mlp(ref_root)
    dump_moe(ref_root)
    dump_linear(ref_root)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            z = np.load(os.path.join(HERE, f))
            print(f, {k: z[k].shape for k in z.files})


if __name__ == "__main__":
    main()
