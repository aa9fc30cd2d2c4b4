"""Serving-side contract around the decode path: cache sizing, phase flags, one forward per scheduler step and the
host <-> device block swap.

Mirrors the parts of the reference's serving runner that touch the hot path:
  cache sizing      MindIEModelRunner.update_llm_config     mindformers/model_runner.py:347-381
  host caches       key_host / value_host                   model_runner.py:310-314
  forward contract  MindIEModelRunner.forward               model_runner.py:384-475 (prefill flag, valid lengths,
                                                            block_tables, slot_mapping, position_ids, q_seq_lens)
  phase flags       _incremental_infer / add_flags_custom   mindformers/generation/text_generator.py:408-453
  swap              MindIEModelRunner.swap                  model_runner.py:477-491
The model here is a stack of quantized decode layers working on hidden states: embedding, LM head and sampling are
outside the path.
"""
import numpy as np
import torch

from . import ops
from .decode_layer import QuantDecodeLayer

_GIB = 1024 * 1024 * 1024


def num_cache_blocks(mem_size_gib, block_size, num_kv_heads, head_size, num_layers, kvcache_bytes=2):
    """Blocks that fit ``mem_size_gib`` GiB: key and value caches of every layer (model_runner.py:370-376)."""
    per_block = block_size * num_kv_heads * head_size * kvcache_bytes * 2 * num_layers
    return int((mem_size_gib * _GIB) // per_block)


class DecodeStackRunner:
    """Owns the layers' paged caches (device) and their swap space (pinned host) and runs scheduler steps.

    ``layers``: prepared ``QuantDecodeLayer``s.  ``npu_mem_size`` / ``cpu_mem_size`` are GiB, as in the reference;
    ``rope_theta`` builds the rotary rows from the positions of each step."""

    def __init__(self, layers, npu_mem_size, cpu_mem_size, block_size, rope_theta=10000.0, device="cuda",
                 quantization_config=None):
        if not layers or not all(isinstance(l, QuantDecodeLayer) for l in layers):
            raise TypeError("layers must be a non-empty list of QuantDecodeLayer")
        first = layers[0]
        self.layers = list(layers)
        self.num_layers = len(layers)
        self.num_kv_heads, self.head_size, self.dtype = first.n_kv_head, first.head_dim, first.dtype
        self.block_size = int(block_size)
        self.rope_theta = rope_theta
        self.device = torch.device(device)
        # the cache dtype follows the quantization config when it names one (model_runner.py:364-368); int8 caches
        # need every layer's dequantisation parameters (QuantDecodeLayer.set_kv_quant)
        kv_name = getattr(quantization_config, "kvcache_quant_dtype", None) if quantization_config is not None else None
        if isinstance(quantization_config, dict):
            kv_name = quantization_config.get("kvcache_dtype")
        if kv_name not in (None, "int8"):
            raise NotImplementedError(f"kvcache_dtype {kv_name!r}: only an int8 KV cache is built")
        if kv_name == "int8":
            gran = (quantization_config.get("kvcache_quant_granularity", "per_channel") if isinstance(quantization_config, dict)
                    else getattr(quantization_config, "kvcache_quant_granularity", "per_channel"))
            if gran != "per_channel":
                raise NotImplementedError("the fused layer step runs per_channel int8 caches; per_token caches are "
                                          "served by the module path (QuantPagedAttentionMgr / FlashAttention)")
            if any(l.kv_scale is None for l in layers):
                raise ValueError("kvcache_dtype int8: every layer needs set_kv_quant(scale, offset) first")
        self.kvcache_dtype = torch.int8 if kv_name == "int8" else self.dtype
        itemsize = torch.empty(0, dtype=self.kvcache_dtype).element_size()
        args = (self.block_size, self.num_kv_heads, self.head_size, self.num_layers, itemsize)
        self.npu_num_blocks = num_cache_blocks(npu_mem_size, *args)
        self.cpu_num_blocks = num_cache_blocks(cpu_mem_size, *args)
        if self.npu_num_blocks < 1:
            raise ValueError(f"npu_mem_size={npu_mem_size} GiB holds no cache block")
        kv_shape = (self.npu_num_blocks, self.block_size, self.num_kv_heads, self.head_size)
        host_shape = (self.cpu_num_blocks,) + kv_shape[1:]
        self.key_cache = [torch.zeros(kv_shape, dtype=self.kvcache_dtype, device=self.device) for _ in layers]
        self.value_cache = [torch.zeros(kv_shape, dtype=self.kvcache_dtype, device=self.device) for _ in layers]
        pin = self.cpu_num_blocks > 0
        self.key_host = [torch.zeros(host_shape, dtype=self.kvcache_dtype, pin_memory=pin) for _ in layers]
        self.value_host = [torch.zeros(host_shape, dtype=self.kvcache_dtype, pin_memory=pin) for _ in layers]
        self.is_first_iteration = True
        self.phase = "prefill"

    def kvcache(self, layer_idx):
        return self.key_cache[layer_idx], self.value_cache[layer_idx]

    def add_flags_custom(self, is_first_iteration):
        """The phase switch of the generate loop (text_generator.py:414-436)."""
        self.is_first_iteration = bool(is_first_iteration)
        self.phase = "prefill" if self.is_first_iteration else "increment"

    def _rope_rows(self, positions):
        d = self.head_size
        inv = 1.0 / (self.rope_theta ** (torch.arange(0, d, 2, dtype=torch.float32, device=self.device) / d))
        ang = positions.to(torch.float32)[:, None] * inv[None, :]
        emb = torch.cat((ang, ang), dim=-1)
        return emb.cos().to(self.dtype), emb.sin().to(self.dtype)

    def forward(self, hidden_states, valid_length_each_example, block_tables, slot_mapping, prefill=True,
                position_ids=None, q_seq_lens=None):
        """One scheduler step over packed rows ``hidden_states`` [T, hidden].

        prefill=True: sequence b brings valid_length_each_example[b] prompt tokens (rows packed sequence after
        sequence), positions 0 .. len-1.  prefill=False: one new token per sequence at position len-1, or, with
        ``q_seq_lens``, q_seq_lens[b] new tokens ending at position len-1 (chunked prefill, parallel decoding).
        ``position_ids`` overrides the positions.  Returns the last layer's output rows."""
        lens = np.asarray(valid_length_each_example, dtype=np.int64).reshape(-1)
        self.add_flags_custom(is_first_iteration=bool(prefill))
        if prefill:
            q_lens = lens
        elif q_seq_lens is not None:
            q_lens = np.asarray(q_seq_lens.cpu() if isinstance(q_seq_lens, torch.Tensor) else q_seq_lens,
                                dtype=np.int64).reshape(-1)
        else:
            q_lens = None
        t = hidden_states.shape[0]
        if q_lens is None:
            if t != lens.size:
                raise ValueError(f"decode step: {t} rows for {lens.size} sequences")
            pos = lens - 1
            q_starts = None
        else:
            if int(q_lens.sum()) != t:
                raise ValueError(f"{t} rows but the sequences bring {int(q_lens.sum())} new tokens")
            pos = np.concatenate([np.arange(l - q, l) for l, q in zip(lens, q_lens)]) if t else np.zeros(0, np.int64)
            q_starts = torch.from_numpy(np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)).to(self.device)
        if position_ids is not None:
            pos_t = torch.as_tensor(position_ids, device=self.device).reshape(-1)
        else:
            pos_t = torch.from_numpy(pos).to(self.device)
        cos, sin = self._rope_rows(pos_t)
        lens_t = torch.from_numpy(lens.astype(np.int32)).to(self.device)
        tables = torch.as_tensor(block_tables, dtype=torch.int32, device=self.device)
        slots = torch.as_tensor(slot_mapping, dtype=torch.int32, device=self.device)
        h = hidden_states
        normed = None
        for i, layer in enumerate(self.layers):
            # layer i also computes layer i + 1's attention norm (W8A8: and its quantisation), in the kernel that
            # finishes its own last projection
            nxt = self.layers[i + 1] if i + 1 < self.num_layers else None
            chain = nxt is not None and layer.act_quant == nxt.act_quant
            nn = None
            if chain:
                nn = (nxt.attn_norm, nxt.eps, nxt.qkv_smooth) if nxt.act_quant else (nxt.attn_norm, nxt.eps)
            out = layer(h, self.key_cache[i], self.value_cache[i], tables, lens_t, slots, cos, sin, q_starts=q_starts,
                        normed=normed, next_norm=nn)
            h, normed = out if chain else (out, None)
        if prefill:
            self.add_flags_custom(is_first_iteration=False)
        return h

    def swap(self, block_tables, swap_type):
        """Swap key/value cache blocks between host and device for every layer (model_runner.py:477-491).
        block_tables: [n, 2] (source block, destination block); swap_type True = device to host."""
        for i in range(self.num_layers):
            ops.swap_cache(self.key_host[i], self.key_cache[i], block_tables, swap_type)
            ops.swap_cache(self.value_host[i], self.value_cache[i], block_tables, swap_type)
