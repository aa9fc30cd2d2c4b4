/*
 * mf_decode.h — C ABI of the MI355X (gfx950) kernels behind MindFormers' quantized decode step.
 *
 * Every entry point replaces one MindSpore / golden-stick primitive that the reference calls on its
 * incremental-inference path (the citation on each declaration is the reference call site, relative to
 * the reference root).  Conventions:
 *   - all pointers are DEVICE pointers unless the name says host; buffers are owned by the caller;
 *   - `stream` is a hipStream_t passed as void*; every call only enqueues work on it and returns;
 *   - the return value is a hipError_t (0 = success); argument errors return hipErrorInvalidValue (1)
 *     before anything is launched, and mf_last_error() then holds a readable message;
 *   - `dtype` selects the activation / cache element type: MF_BF16 or MF_FP16;
 *   - nothing here allocates or frees device memory.
 */
#ifndef MF_DECODE_H_
#define MF_DECODE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MF_BF16 0
#define MF_FP16 1
#define MF_FP32 2

/* Library identification and the message of the last argument error on the calling thread. */
const char* mf_version(void);
const char* mf_last_error(void);

/* ---- KV cache ------------------------------------------------------------------------------------- */

/* ops.auto_generate.ReshapeAndCache(key, value, key_cache, value_cache, slot_mapping)
 *   mindformers/modules/paged_attention_mgr.py:50,60-62
 *   mindformers/parallel_core/inference/transformer/flash_attention.py:94,126-127
 * cache.view(num_slots, n_kv_heads*head_dim)[slot_mapping[i]] = x[i] for key and value; slot < 0 skips the
 * row (padding, mindformers/modules/block_tables.py:79-95).  value / value_cache may both be NULL (the MLA
 * call writes one latent cache, multi_latent_attention.py:401-402).  Pure copy: bit-exact.
 * key_row_stride / value_row_stride: elements between consecutive token rows of key / value (0 = dense,
 * n_kv_heads*head_dim); lets key and value be column slices of one fused [T, q|k|v] projection output. */
int mf_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                         const int32_t* slot_mapping, int num_tokens, int n_kv_heads, int head_dim,
                         int64_t num_slots, int64_t key_row_stride, int64_t value_row_stride, int dtype,
                         void* stream);

/* ops.ApplyRotaryPosEmb(cos_format=2)(query, key, cos, sin, batch_valid_length)
 *   mindformers/modules/infer_attention.py:50-57
 *   mindformers/parallel_core/inference/base_models/common/embeddings/rotary_pos_embedding.py:75,146
 * In place, rotate-half pairing (i, i + head_dim/2): x = x*cos + rotate_half(x)*sin in fp32, rounded once.
 * cos/sin are [num_tokens, head_dim] rows already gathered per token (table_dtype: MF_BF16/MF_FP16/MF_FP32).
 * key may be NULL.  q_row_stride / k_row_stride: elements between token rows (0 = dense). */
int mf_rope_half(void* query, void* key, const void* cos, const void* sin, int num_tokens, int n_heads,
                 int n_kv_heads, int head_dim, int64_t q_row_stride, int64_t k_row_stride, int dtype,
                 int table_dtype, void* stream);

/* RoPE on q and k followed by the cache scatter of rotated k and of v, one launch (the sequence
 * infer_attention.py:445,453 performs).  q and k are rotated in place. */
int mf_rope_and_cache(void* query, void* key, const void* value, const void* cos, const void* sin,
                      void* key_cache, void* value_cache, const int32_t* slot_mapping, int num_tokens,
                      int n_heads, int n_kv_heads, int head_dim, int64_t num_slots, int64_t q_row_stride,
                      int64_t k_row_stride, int64_t v_row_stride, int dtype, int table_dtype, void* stream);

/* mindspore._c_expression.swap_cache(host_cache, device_cache, block_mapping, is_device_to_host), as called per
 * layer by MindIEModelRunner.swap (mindformers/model_runner.py:478-491): copies whole cache blocks between a host
 * cache [host_blocks, ...] and a device cache [device_blocks, ...] of block_bytes each.  pairs: HOST int64
 * [n_pairs][2] = (source block, destination block); device_to_host != 0 copies device[src] -> host[dst], else
 * host[src] -> device[dst].  Async on `stream` when the host cache is pinned; `pairs` is read before returning.
 * The primitive lives in MindSpore, not in the reference: the pair order is this build's declared reading. */
int mf_swap_blocks(void* host_cache, void* device_cache, const int64_t* pairs, int64_t n_pairs,
                   int64_t block_bytes, int64_t host_blocks, int64_t device_blocks, int device_to_host,
                   void* stream);

/* ---- paged attention (decode) --------------------------------------------------------------------- */

/* Bytes of scratch mf_paged_attention_decode needs for this shape (0 when the context fits one partition). */
size_t mf_paged_attention_workspace_bytes(int batch, int n_heads, int head_dim, int max_context);

/* ops.auto_generate.PagedAttention(head_num, scale, kv_head_num)(query, key_cache, value_cache,
 *                                                               block_tables, context_lens)
 *   mindformers/modules/paged_attention_mgr.py:51-53,64-70
 *   mindformers/parallel_core/inference/transformer/flash_attention.py:106-107,135-143
 * out[b,h,:] = softmax(scale * q[b,h,:] . K_b[:L_b]^T) V_b[:L_b]; token j of sequence b lives at
 * cache[block_tables[b, j / block_size], j % block_size, h / (n_heads/n_kv_heads), :]; L_b = context_lens[b]
 * counts the token written by this step.  L_b <= 0 gives zeros.  Scores and softmax in fp32; the
 * probabilities are rounded to `dtype` before the PV product.  head_dim in {32, 64, 128}.
 * q_row_stride: elements between the query rows of consecutive sequences (0 = dense); out is dense. */
int mf_paged_attention_decode(void* out, const void* query, const void* key_cache, const void* value_cache,
                              const int32_t* block_tables, const int32_t* context_lens, int batch,
                              int n_heads, int n_kv_heads, int head_dim, int block_size,
                              int max_blocks_per_seq, int num_blocks, float scale, int64_t q_row_stride,
                              int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* mf_paged_attention_decode for a layer whose output projection is per-token quantised (the golden-stick
 * DynamicQuant in front of the W8A8 wo, behind flash_attention.py:135-143): besides out, the row of all heads of
 * every sequence is quantised as mf_dynamic_quant_per_token(smooth, xq_layout) would quantise out: xq int8
 * [batch, n_heads * head_dim] (or tiled), x_scale float32 [batch].  Same bits as the two calls in sequence; with 2 to
 * 16 partitions and n_heads * head_dim <= 4096 the partition combine and the quantisation are one kernel.  16-bit
 * caches.  Workspace as for mf_paged_attention_decode. */
int mf_paged_attention_decode_dynamic_quant(void* out, int8_t* xq, float* x_scale, const float* smooth, int xq_layout,
                                            const void* query, const void* key_cache, const void* value_cache,
                                            const int32_t* block_tables, const int32_t* context_lens, int batch,
                                            int n_heads, int n_kv_heads, int head_dim, int block_size,
                                            int max_blocks_per_seq, int num_blocks, float scale, int64_t q_row_stride,
                                            int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* mf_paged_attention_decode for callers that cannot allocate or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments and same result bits as mf_paged_attention_decode, minus workspace / workspace_bytes: the partition
 * partials go to a device array built into the library (MF_PA_STATIC_SCRATCH_BYTES per GPU, held until the
 * process ends).  Shapes whose mf_paged_attention_workspace_bytes exceeds that size are rejected with
 * hipErrorInvalidValue and a message.  The call allocates and frees nothing; the first call on a device looks up
 * the array's address (make that call outside a stream capture).  All calls on one GPU share the one array:
 * calls that may overlap on a GPU (different streams, different host threads) race on it and must be serialised
 * by the caller. */
#define MF_PA_STATIC_SCRATCH_BYTES (48u << 20)
int mf_paged_attention_decode_static(void* out, const void* query, const void* key_cache, const void* value_cache,
                                     const int32_t* block_tables, const int32_t* context_lens, int batch,
                                     int n_heads, int n_kv_heads, int head_dim, int block_size,
                                     int max_blocks_per_seq, int num_blocks, float scale, int64_t q_row_stride,
                                     int dtype, void* stream);

/* ---- int8 KV cache (kvcache_dtype = int8, per-channel) ------------------------------------------------ */

/* The reference sizes an int8 cache (mindformers/model_runner.py:364-368, kvcache_dtype in the quantization
 * config, mindformers/utils/quantization_config.py:196-250) and hands PagedAttention its antiquant_scale /
 * antiquant_offset arguments (positions 6-7 of the call in mindformers/modules/paged_attention_mgr.py:66-70);
 * the cells that fill them belong to golden-stick and the arithmetic to the vendor kernels, so the convention is
 * this build's own declaration: per channel c of a [n_kv_heads * head_dim] row,
 *     q = clip(rint(x / scale[c] + offset[c]), -128, 127)        x ~ (q - offset[c]) * scale[c]
 * scale / offset: float [2][n_kv_heads * head_dim], keys first, then values; offset may be NULL (symmetric).
 *
 * mf_quant_reshape_and_cache: the quantizing twin of mf_reshape_and_cache (int8 caches [slots, n_kv*D]). */
int mf_quant_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                               const int32_t* slot_mapping, const float* scale, const float* offset,
                               int num_tokens, int n_kv_heads, int head_dim, int64_t num_slots,
                               int64_t key_row_stride, int64_t value_row_stride, int dtype, void* stream);

/* FlashAttentionScore of the prefill of multi-latent attention -
 * mindformers/parallel_core/inference/transformer/multi_latent_attention.py:405-432, :206-216: queries and keys have
 * 192-wide heads (the up-projected 128 dimensions followed by the 64 rotary ones), values 128-wide heads.  The
 * reference pads the values to 192 and keeps the first 128 output columns; this entry point takes the values as
 * they are and returns out [total_q, n_heads * 128], the same numbers without the padded third of the PV product.
 * Packed rows as mf_paged_attention_prefill with block_tables == NULL (causal, q_starts [batch + 1]); row strides
 * in elements, 0 = dense.  Workspace: mf_paged_attention_prefill_workspace_bytes(batch, total_q, n_heads,
 * n_kv_heads, 128, total_q). */
int mf_causal_attention_qk192_v128(void* out, const void* query, const void* key, const void* value,
                                   const int32_t* q_starts, int batch, int total_q, int n_heads, int n_kv_heads,
                                   float scale, int64_t q_row_stride, int64_t k_row_stride, int64_t v_row_stride,
                                   int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* mf_paged_attention_decode / _prefill on int8 caches: same arguments plus antiquant_scale / antiquant_offset
 * (offset may be NULL); workspaces as for the 16-bit entry points; paged keys only.  Scores use the query with
 * the key scale folded in (rounded to dtype); a key offset shifts all scores of a row equally and cancels in the
 * softmax; out = scale_v * (sum_t p_t v8_t - offset_v) with the int8 values widened exactly. */
int mf_paged_attention_decode_int8kv(void* out, const void* query, const void* key_cache, const void* value_cache,
                                     const int32_t* block_tables, const int32_t* context_lens,
                                     const float* antiquant_scale, const float* antiquant_offset, int batch,
                                     int n_heads, int n_kv_heads, int head_dim, int block_size,
                                     int max_blocks_per_seq, int num_blocks, float scale, int64_t q_row_stride,
                                     int dtype, void* workspace, size_t workspace_bytes, void* stream);
int mf_paged_attention_prefill_int8kv(void* out, const void* query, const void* key_cache, const void* value_cache,
                                      const int32_t* block_tables, const int32_t* context_lens,
                                      const int32_t* q_starts, const float* antiquant_scale,
                                      const float* antiquant_offset, int batch, int total_q, int n_heads,
                                      int n_kv_heads, int head_dim, int block_size, int max_blocks_per_seq,
                                      int num_blocks, float scale, int64_t q_row_stride, int dtype,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* int8 KV caches quantised per token (kvcache_quant_granularity per_token,
 * mindformers/utils/quantization_config.py:206-207,296-300: needs an int8 cache): the cache write, and the two
 * attention entry points on such caches.  Every cached token row (all kv heads of a token) has one fp32 scale in
 * key_scale_cache / value_scale_cache [num_blocks * block_size], indexed by slot like the rows.
 * mf_dynamic_quant_reshape_and_cache: s = max|row| / 127, q = clip(rint(x / s), -128, 127) in float32 as
 * mf_dynamic_quant_per_token defines it (a zero row stores s = 0 and zeros); the int8 row and s go to
 * slot_mapping[t]; negative or out-of-range slots are skipped.  Strides as mf_reshape_and_cache.
 * Attention: K_b[j] = key_cache[slot j] * key_scale_cache[slot j], V_b[j] likewise; the score of token j is
 * multiplied by its key scale, its probability by its value scale before the rounding to `dtype` in front of the PV
 * product; the denominator sums the unscaled fp32 probabilities.  block_size % 4 == 0; scale caches 16-byte
 * aligned.  Everything else as mf_paged_attention_decode / mf_paged_attention_prefill (paged form only).  The
 * arithmetic of the reference's per-token cells is not in the reference: this is the build's declared convention. */
int mf_dynamic_quant_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                                       float* key_scale_cache, float* value_scale_cache, const int32_t* slot_mapping,
                                       int num_tokens, int n_kv_heads, int head_dim, int64_t num_slots,
                                       int64_t key_row_stride, int64_t value_row_stride, int dtype, void* stream);
int mf_paged_attention_decode_int8kv_per_token(void* out, const void* query, const void* key_cache,
                                               const void* value_cache, const float* key_scale_cache,
                                               const float* value_scale_cache, const int32_t* block_tables,
                                               const int32_t* context_lens, int batch, int n_heads, int n_kv_heads,
                                               int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                               float scale, int64_t q_row_stride, int dtype, void* workspace,
                                               size_t workspace_bytes, void* stream);
int mf_paged_attention_prefill_int8kv_per_token(void* out, const void* query, const void* key_cache,
                                                const void* value_cache, const float* key_scale_cache,
                                                const float* value_scale_cache, const int32_t* block_tables,
                                                const int32_t* context_lens, const int32_t* q_starts, int batch,
                                                int total_q, int n_heads, int n_kv_heads, int head_dim, int block_size,
                                                int max_blocks_per_seq, int num_blocks, float scale,
                                                int64_t q_row_stride, int dtype, void* workspace,
                                                size_t workspace_bytes, void* stream);

/* ---- attention over several new tokens per sequence (prefill, chunked prefill, parallel decoding) -- */

/* Bytes of scratch mf_paged_attention_prefill needs (0 when one partition spans the context).  max_context is
 * max_blocks_per_seq * block_size for a paged cache and total_q for contiguous keys. */
size_t mf_paged_attention_prefill_workspace_bytes(int batch, int total_q, int n_heads, int n_kv_heads,
                                                  int head_dim, int max_context);

/* Causal attention of q_len_b = q_starts[b+1] - q_starts[b] new query rows per sequence.
 *
 * Paged keys (block_tables != NULL) replace PagedAttention called with q_seq_lens and a causal mask:
 *   ops.auto_generate.PagedAttention(...)(query, key_cache, value_cache, block_tables, batch_valid_length,
 *                                         None, None, attn_mask, q_seq_lens)
 *   mindformers/modules/paged_attention_mgr.py:66-69 (parallel_decoding / chunk_prefill)
 *   mindformers/parallel_core/inference/transformer/flash_attention.py:140-143
 * The new tokens' keys and values are already in the cache (ReshapeAndCache runs first, flash_attention.py:
 * 126-127); context_lens[b] counts them.  Query i of sequence b sits at position L_b - q_len_b + i and
 * attends to cache tokens 0 .. L_b - q_len_b + i.
 *
 * Contiguous keys (block_tables == NULL; context_lens, block_size, max_blocks_per_seq, num_blocks ignored)
 * replace FlashAttentionScore in the TH layout with a causal mask and actual_seq_qlen == actual_seq_kvlen:
 *   mindformers/parallel_core/inference/transformer/flash_attention.py:96-104,129-134
 *   mindformers/modules/flash_attention.py (FlashAttention.construct, input_layout "TH")
 * key_cache / value_cache are then this step's packed keys and values, row q_starts[b] + j = token j of
 * sequence b, kv_row_stride elements apart (0 = dense n_kv_heads * head_dim; a slice of a fused QKV output
 * works), and L_b = q_len_b.
 *
 * query: total_q rows of n_heads * head_dim, q_row_stride elements apart (0 = dense); out: dense
 * [total_q, n_heads * head_dim].  q_starts: int32 [batch + 1], non-decreasing.  Rows of no sequence, and
 * rows beyond a sequence's context, are written as zeros.  scale must be positive.  Numerics as
 * mf_paged_attention_decode.  head_dim in {32, 64, 128, 192}: 192 is the prefill of multi-latent attention, whose
 * queries, keys and values all arrive 192 wide with n_kv_heads = n_heads
 * (mindformers/parallel_core/inference/transformer/multi_latent_attention.py:405-432; the caller keeps the first
 * v_head_dim columns of every head, :216-218). */
int mf_paged_attention_prefill(void* out, const void* query, const void* key_cache, const void* value_cache,
                               const int32_t* block_tables, const int32_t* context_lens,
                               const int32_t* q_starts, int batch, int total_q, int n_heads, int n_kv_heads,
                               int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                               float scale, int64_t q_row_stride, int64_t kv_row_stride, int dtype,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ---- multi-latent attention (MLA) decode -------------------------------------------------------------- */

/* Bytes of scratch mf_mla_paged_attention_decode needs (0 when one partition spans the context). */
size_t mf_mla_paged_attention_workspace_bytes(int batch, int n_heads, int max_context);

/* ops.auto_generate.PagedAttention(head_num, scale, kv_head_num=1, mla_v_dim=kv_lora_rank)(query, key_cache,
 *                                  key_cache, block_tables, batch_valid_length, ...)
 *   mindformers/parallel_core/inference/transformer/flash_attention.py:106-107,136-139
 *   mindformers/parallel_core/inference/transformer/multi_latent_attention.py:199-228,344-448 (the caller: one
 *   latent cache [num_blocks, block_size, 1, kv_lora_rank + rope_dim] written by reshape_and_cache(key, None,
 *   key_cache, None, slot_mapping) — mf_reshape_and_cache with value = NULL — and queries already multiplied by
 *   the absorbed key up-projection).
 * out[b,h,:kv_lora_rank] = softmax(scale * q[b,h,:] . C_b[:L_b]^T) C_b[:L_b, :kv_lora_rank] with C the cache rows
 * of kv_lora_rank + rope_dim values; query [batch, n_heads * (kv_lora_rank + rope_dim)], q_row_stride elements
 * apart (0 = dense); out dense [batch, n_heads * kv_lora_rank].  kv_lora_rank = 512, rope_dim = 64 (the DeepSeek
 * V2 / V3 geometry); block_size a multiple of 32; scale positive.  Numerics as mf_paged_attention_decode. */
int mf_mla_paged_attention_decode(void* out, const void* query, const void* latent_cache,
                                  const int32_t* block_tables, const int32_t* context_lens, int batch,
                                  int n_heads, int kv_lora_rank, int rope_dim, int block_size,
                                  int max_blocks_per_seq, int num_blocks, float scale, int64_t q_row_stride,
                                  int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* The weight-absorbed per-head projections around the multi-latent decode attention:
 *   q_no_pe = mint.transpose(mint.matmul(mint.transpose(q_no_pe, -3, -2), q_absorb), -3, -2)
 *   core_attn_out = mint.matmul(mint.transpose(core_attn_out, -3, -2), mint.transpose(out_absorb, -2, -1))
 *   mindformers/parallel_core/inference/transformer/multi_latent_attention.py:434-448, :228-231
 * out[t, h, :n] = x[t, h, :k] . w[h]^T with w [heads, n, k] dense (for the query side the slice of
 * linear_kv_up_proj.weight is stored transposed once, so that both sides read rows of k).  x and out are addressed by
 * element strides between tokens and between heads, so that q_no_pe can be read inside the [T, heads, 192] query
 * projection and the result written into the first 512 columns of the [T, heads, 576] attention query.
 * fp32 accumulation, one rounding.  k in {64, 128, 256, 512}; n a multiple of 16. */
int mf_mla_absorb_bmm(void* out, const void* x, const void* w, int tokens, int heads, int n, int k,
                      int64_t x_token_stride, int64_t x_head_stride, int64_t out_token_stride,
                      int64_t out_head_stride, int dtype, void* stream);

/* The element-wise work of MLASelfAttention.get_query_key_value_tensors between the down projections and the
 * attention, in one launch - mindformers/parallel_core/inference/transformer/multi_latent_attention.py:391-403
 * (kv_layernorm, rotary_pos_emb on q_pos_emb / k_pos_emb, concat + key-only reshape_and_cache) and :444-447 (the
 * rotated query part behind the absorbed query):
 *   kv [tokens, rank + rope] (rows kv_token_stride elements apart: a slice of the fused down projection): columns
 *   [0, rank) are RMS-normalised with gamma / eps (rounded to dtype), columns [rank, rank + rope) rotated (rotate-half,
 *   cos / sin [tokens, rope] rows gathered per token, table_dtype as mf_rope_half); both go to row slot_mapping[t] of
 *   latent_cache [num_slots, rank + rope] (skipped for a negative / out-of-range slot or a NULL cache) and, where the
 *   pointers are given, to the dense kv_norm_out [tokens, rank] and k_pe_out [tokens, rope];
 *   q_rope points at the rotary part of head 0 of token 0 (head h of token t q_token_stride * t + q_head_stride * h
 *   elements further); its rotation is stored likewise addressed at q_rope_out (q_rope_out == q_rope rotates in
 *   place).  rank % 8 == 0, rope % 16 == 0, strides multiples of 8 elements, pointers 16-byte aligned. */
int mf_mla_norm_rope_cache(void* q_rope_out, int64_t q_out_token_stride, int64_t q_out_head_stride,
                           const void* q_rope, int64_t q_token_stride, int64_t q_head_stride, void* kv_norm_out,
                           void* k_pe_out, const void* kv, int64_t kv_token_stride, const void* gamma, int gamma_dtype,
                           float eps, const void* cos, const void* sin, int table_dtype, void* latent_cache,
                           const int32_t* slot_mapping, int64_t num_slots, int tokens, int heads, int rank, int rope,
                           int dtype, void* stream);

/* ---- norm / activation ---------------------------------------------------------------------------- */

/* P.RmsNorm(eps)(x, gamma): mindformers/models/llama/llama_layer.py:195,225-228;
 * mindformers/parallel_core/inference/transformer/norm.py:108,113.
 * y = x * rsqrt(mean(x^2) + eps) * gamma, fp32 inside, one rounding.  gamma_dtype: MF_BF16/MF_FP16/MF_FP32.
 * If residual != NULL: h = x + residual is formed first (rounded to dtype), written to sum_out, and
 * normalised — the residual add of llama_transformer.py:1057 fused with the following norm (:1059). */
int mf_rmsnorm(void* y, void* sum_out, const void* x, const void* residual, const void* gamma, float eps,
               int rows, int cols, int dtype, int gamma_dtype, void* stream);

/* The same norm over a column slice of a wider matrix: row i of x starts x_row_stride elements after row i - 1
 * (>= cols, a multiple of 8); y is dense [rows, cols].  The latent norms of multi-latent attention read slices of the
 * fused down projection: mindformers/parallel_core/inference/transformer/multi_latent_attention.py:367-374
 * (q_layernorm on the first q_lora_rank columns, kv_layernorm on the next kv_lora_rank). */
int mf_rmsnorm_strided(void* y, const void* x, int64_t x_row_stride, const void* gamma, float eps, int rows, int cols,
                       int dtype, int gamma_dtype, void* stream);

/* act(gate) * up with act = SiLU: mindformers/parallel_core/inference/transformer/mlp.py:135-140,
 * mindformers/models/llama/llama_layer.py:419-440.  gate_up is [rows, 2*cols]; layout 0 = contiguous halves
 * [gate | up] (mcore), 1 = interleaved columns g,u,g,u (legacy ffn_concat).  silu(gate) is rounded to dtype
 * before the multiply, as the reference materialises it. */
int mf_silu_mul(void* out, const void* gate_up, int rows, int cols, int layout, int dtype, void* stream);

/* out = a + b (residual add, llama_transformer.py:1057,1067). */
int mf_add(void* out, const void* a, const void* b, int64_t n, int dtype, void* stream);

/* out[m, k] = x[m, k] * scale[k], rounded once: the activation multiplier of an outlier-suppression pair (smooth /
 * awq, mindformers/utils/quantization_config.py:413-414) in front of a weight-only GEMM, where no activation
 * quantisation kernel is there to carry it.  cols % 8 == 0. */
int mf_scale_columns(void* out, const void* x, const float* scale, int64_t rows, int cols, int dtype, void* stream);

/* ---- quantized linear ----------------------------------------------------------------------------- */

/* The W8A16 kernels stream the int8 weight in a tiled order (16 output channels x 64 input channels per
 * 1 KiB tile, tiles ordered [k-step][n-tile], bytes inside a tile in MFMA-operand lane order; N padded to 16
 * and K to 64 with zeros).  Pack once after the checkpoint is loaded — the counterpart of the format
 * conversion golden-stick's deploy cells apply to their weight Parameter.  w is int8 [N, K] row-major. */
size_t mf_w8a16_packed_bytes(int n, int k);
int mf_w8a16_pack_weight(void* packed, const int8_t* w, int n, int k, void* stream);

size_t mf_w8a16_workspace_bytes(int m, int n, int k);

/* golden-stick weight-only cell -> WeightQuantBatchMatmul, replacing P.MatMul(transpose_b=True) at
 *   mindformers/modules/layers.py:479,526; parallel_core/inference/tensor_parallel/layers.py:186,406
 * (swapped in by Quantizer.preprocess_model, mindformers/modules/quantizers/rtn_quantizer.py:61-67).
 * y[m,n] = (sum_k x[m,k] * w[n,k]) * scale[n] (+ bias[n]) (+ residual[m,n]); x/y/bias/residual in `dtype`,
 * w_packed = mf_w8a16_pack_weight of the int8 [N,K] weight, scale float32 [N]; products exact, fp32
 * accumulation, scale applied to the sum.  With residual: y = round(round(acc*scale+bias) + residual).
 * K % 8 == 0. */
int mf_w8a16_gemm(void* y, const void* x, const void* w_packed, const float* scale, const void* bias,
                  const void* residual, int m, int n, int k, int dtype, void* workspace,
                  size_t workspace_bytes, void* stream);

/* 4-bit weights, weight-only (A16W4): WeightQuantBatchMatmul behind the golden-stick cell that
 * PtqConfig(weight_dtype="qint4x2", weight_quant_granularity in {per_channel, per_group}, group_size in {0, 64, 128})
 * selects (mindformers/utils/quantization_config.py:408-416,448-453; mindformers/modules/quantizers/
 * ptq_quantizer.py:52-59).  mf_w4a16_pack_weight turns w [n, k] int8 holding the 4-bit values (-8 .. 7, one per byte)
 * into 512-byte tiles of 16 channels x 64 columns in matrix-instruction operand order ([k-step][tile], nibbles
 * q + 8); mf_w4a16_packed_bytes gives the size.  mf_w4a16_gemm: y = x . (w * scale)^T (+ bias) (+ residual) with
 * scale [n] (group_size 0) or [k / group_size][n] (one scale per channel and group of columns).  The products of a
 * group are summed in fp32 on the exact integer weights, then multiplied by the group's scale.  k a multiple of 64
 * and of group_size; n a multiple of 4 with groups.  Workspace: mf_w4a16_workspace_bytes. */
size_t mf_w4a16_packed_bytes(int n, int k);
int mf_w4a16_pack_weight(void* packed, const int8_t* w, int n, int k, void* stream);
size_t mf_w4a16_workspace_bytes(int m, int n, int k, int group_size);
int mf_w4a16_gemm(void* y, const void* x, const void* w_packed, const float* scale, const void* bias,
                  const void* residual, int m, int n, int k, int group_size, int dtype, void* workspace,
                  size_t workspace_bytes, void* stream);

/* A row-parallel projection with its residual add, fused with the RMSNorm that follows it in the layer
 * (mindformers/models/llama/llama_transformer.py:1053-1059; parallel_core/inference/transformer/
 * transformer_layer.py:296-355): h_out = round(round(x . w^T * scale + bias) + residual),
 * y_norm = RMSNorm(h_out) * gamma.  Bit-identical to mf_w8a16_gemm(residual) followed by mf_rmsnorm; when K is
 * split across workgroups the sum of the splits, the add and the norm are one kernel.  N % 8 == 0, N <= 16384.
 * Workspace as for mf_w8a16_gemm. */
int mf_w8a16_gemm_add_rmsnorm(void* y_norm, void* h_out, const void* x, const void* w_packed, const float* scale,
                              const void* bias, const void* residual, const void* gamma, float eps, int m, int n,
                              int k, int dtype, int gamma_dtype, void* workspace, size_t workspace_bytes,
                              void* stream);

/* A projection whose leading columns feed an RMSNorm - the fused query / latent down projection of multi-latent
 * attention followed by q_layernorm on its first q_lora_rank columns
 * (mindformers/parallel_core/inference/transformer/multi_latent_attention.py:361-374): h_out [m, n] =
 * round(x . w^T * scale + bias), y_norm [m, norm_cols] (dense) = RMSNorm(h_out[:, :norm_cols]) * gamma.  Bit-identical
 * to mf_w8a16_gemm followed by mf_rmsnorm_strided on the slice; when K is split across workgroups the sum of the
 * splits and the norm are one kernel.  N % 8 == 0, N <= 16384, norm_cols % 8 == 0, norm_cols <= N.  Workspace as for
 * mf_w8a16_gemm. */
int mf_w8a16_gemm_rmsnorm_leading(void* y_norm, void* h_out, const void* x, const void* w_packed, const float* scale,
                                  const void* bias, const void* gamma, float eps, int m, int n, int k, int norm_cols,
                                  int dtype, int gamma_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* The fused QKV projection together with what follows it on the decode path: rotate-half RoPE on q and k and the
 * scatter of the rotated k and of v into the paged caches (mindformers/modules/infer_attention.py:441-463,
 * parallel_core/inference/transformer/attention.py:164-258).  qkv is [M, (n_heads + 2 n_kv_heads) * head_dim]; on
 * return its q columns hold the rotated query (row stride = the full width), its k and v columns are
 * unspecified, and the caches hold the new rows.  Same values as mf_w8a16_gemm followed by mf_rope_and_cache on
 * the column slices; when K is split across workgroups the sum of the splits, the rotation and the scatter are
 * one kernel.  head_dim % 16 == 0.  Workspace as for mf_w8a16_gemm with n = the full width. */
int mf_w8a16_qkv_rope_and_cache(void* qkv, const void* x, const void* w_packed, const float* scale, const void* bias,
                                const void* cos, const void* sin, void* key_cache, void* value_cache,
                                const int32_t* slot_mapping, int m, int n_heads, int n_kv_heads, int head_dim,
                                int64_t num_slots, int k, int dtype, int table_dtype, void* workspace,
                                size_t workspace_bytes, void* stream);

/* mf_w8a16_qkv_rope_and_cache for int8 caches (kvcache_dtype int8, mindformers/modules/infer_attention.py:225-238):
 * the rotated k and v rows are quantised on the way into the caches as mf_quant_reshape_and_cache does
 * (kv_scale / kv_offset float32 [2][n_kv_heads * head_dim], keys then values; kv_offset may be NULL).  Same values as
 * mf_w8a16_gemm, mf_rope_half on the q and k columns, then mf_quant_reshape_and_cache on the k and v columns. */
int mf_w8a16_qkv_rope_and_quant_cache(void* qkv, const void* x, const void* w_packed, const float* scale,
                                      const void* bias, const void* cos, const void* sin, void* key_cache,
                                      void* value_cache, const int32_t* slot_mapping, const float* kv_scale,
                                      const float* kv_offset, int m, int n_heads, int n_kv_heads, int head_dim,
                                      int64_t num_slots, int k, int dtype, int table_dtype, void* workspace,
                                      size_t workspace_bytes, void* stream);

/* The gate/up projection of a gated MLP fused with its activation: WeightQuantBatchMatmul followed by
 * SiLU(gate) * up (mindformers/models/llama/llama_layer.py:419-440 with the interleaved ffn_concat layout,
 * parallel_core/inference/transformer/mlp.py:130-147).  The packed weight has its [N, K] rows in interleaved
 * order (row 2j = gate channel j, row 2j+1 = up channel j; scale and bias likewise), N even; y is [M, N/2]:
 * y[m,j] = round(round(silu(g)) * u) with g, u = round(acc * scale + bias) of rows 2j, 2j+1 - bit-identical to
 * mf_w8a16_gemm followed by mf_silu_mul(layout 1).  Workspace as for mf_w8a16_gemm. */
int mf_w8a16_gemm_silu_mul(void* y, const void* x, const void* w_packed, const float* scale, const void* bias,
                           int m, int n, int k, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* golden-stick DynamicQuant (per-token) with the SmoothQuant multiplier folded in
 * (quantization_config.py:363-380,438-442: act per_token needs int8 weights and activations).
 * xs = x*smooth (fp32); s_t = max_k|xs|/127; q = clip(rint(xs/s_t), -128, 127).  smooth may be NULL.
 * layout 0: xq is int8 [M,K] row-major.  layout 1: xq is written in the tile order mf_w8a8_gemm streams
 * (1 KiB tiles of 16 rows x 64 columns, the order mf_w8a16_pack_weight gives an [M,K] matrix;
 * mf_w8a16_packed_bytes(m, k) bytes, padding left unwritten). */
int mf_dynamic_quant_per_token(int8_t* xq, float* x_scale, const void* x, const float* smooth, int m, int k,
                               int dtype, int layout, void* stream);

/* golden-stick's static (per-tensor) activation quantisation in front of QuantBatchMatmul, the SmoothQuant method's
 * A8W8 cells (mindformers/modules/quantizers/smooth_quant_quantizer.py:61-67, act_quant_granularity per_tensor in
 * mindformers/utils/quantization_config.py:577-595): q = clip(rint(x * smooth / act_scale[0]), -128, 127) with one
 * calibrated scale for the whole tensor (a float on the device, loaded with the checkpoint; symmetric: this build's
 * declared convention, the cell's arithmetic is not in the reference).  x_scale receives act_scale[0] for every
 * row, so mf_w8a8_gemm dequantises as for per-token scales.  Layouts as mf_dynamic_quant_per_token. */
int mf_static_quant_per_tensor(int8_t* xq, float* x_scale, const void* x, const float* smooth,
                               const float* act_scale, int m, int k, int dtype, int layout, void* stream);

/* RMSNorm (optionally with the residual add in front, as mf_rmsnorm) whose only reader is a per-token quantised
 * projection, fused with that quantisation: the norm output is not written, xq / x_scale are what
 * mf_dynamic_quant_per_token(layout) gives for it.  Bit-identical to mf_rmsnorm followed by
 * mf_dynamic_quant_per_token (P.RmsNorm, llama_layer.py:195,225-228, in front of the golden-stick DynamicQuant of
 * the W8A8 qkv and gate/up projections). */
int mf_rmsnorm_dynamic_quant(int8_t* xq, float* x_scale, void* sum_out, const void* x, const void* residual,
                             const void* gamma, const float* smooth, float eps, int rows, int cols, int dtype,
                             int gamma_dtype, int layout, void* stream);

/* act(gate) * up (as mf_silu_mul, gate_up_layout 0 = halves, 1 = interleaved) whose only reader is the per-token
 * quantised down projection, fused with that quantisation: the product is not written.  Bit-identical to
 * mf_silu_mul followed by mf_dynamic_quant_per_token (mlp.py:135-140 in front of the golden-stick DynamicQuant of
 * the W8A8 down projection).  cols = width of the product, at most 24576. */
int mf_silu_mul_dynamic_quant(int8_t* xq, float* x_scale, const void* gate_up, const float* smooth, int rows, int cols,
                              int gate_up_layout, int dtype, int layout, void* stream);

/* mf_dynamic_quant_per_token / mf_silu_mul_dynamic_quant for rows grouped by expert (the permuted rows in front of
 * the routed experts' int8 GroupedMatmul, mindformers/parallel_core/inference/transformer/moe/experts.py:151-170, under
 * outliers_suppression: smooth, mindformers/utils/quantization_config.py:413-414): rows offsets[e] ..
 * offsets[e + 1] - 1 (offsets int32 [n_experts + 1], as mf_moe_permute writes it) are multiplied by row e of smooth
 * fp32 [n_experts, k] before the per-token quantisation; rows at or past offsets[n_experts] use the last expert's.
 * One multiplier vector per expert is this build's declared form of the suppression on stacked expert weights (the
 * cell's arithmetic is not in the reference).  Everything else as the ungrouped calls. */
int mf_grouped_dynamic_quant_per_token(int8_t* xq, float* x_scale, const void* x, const float* smooth,
                                       const int32_t* offsets, int n_experts, int m, int k, int dtype, int layout,
                                       void* stream);
int mf_grouped_silu_mul_dynamic_quant(int8_t* xq, float* x_scale, const void* gate_up, const float* smooth,
                                      const int32_t* offsets, int n_experts, int rows, int cols, int gate_up_layout,
                                      int dtype, int layout, void* stream);

/* golden-stick QuantBatchMatmul: int8 x int8 -> int32 on MFMA, dequantised in the epilogue:
 * y[m,n] = acc[m,n] * x_scale[m] * w_scale[n] (+ bias[n]) (+ residual[m,n]) -> dtype.
 * xq int8 [M,K]: row-major (x_layout 0) or tiled (x_layout 1), as mf_dynamic_quant_per_token writes it; the tiled
 * form is the fast path (whole-line, evenly spread L2 requests).  w_packed = mf_w8a16_pack_weight of the int8
 * [N,K] weight (the same tile order serves the int8 matrix cores).  If acc_out != NULL the raw int32 accumulators
 * are also written ([M,N] row-major); y may then be NULL.  K % 16 == 0.  workspace: mf_w8a8_workspace_bytes
 * bytes (int32 partial sums when K is split across workgroups; 0 for wide N). */
size_t mf_w8a8_workspace_bytes(int m, int n, int k);
int mf_w8a8_gemm(void* y, int32_t* acc_out, const int8_t* xq, const float* x_scale, const void* w_packed,
                 const float* w_scale, const void* bias, const void* residual, int m, int n, int k, int dtype,
                 int x_layout, void* workspace, size_t workspace_bytes, void* stream);

/* The row-parallel W8A8 projection (attention output, MLP down) together with what follows it in the layer: the
 * residual add and the RMSNorm whose only reader is the next per-token quantised projection
 * (llama_layer.py:195,225-228 behind the golden-stick QuantBatchMatmul of wo / w2).  h_out [M,N] =
 * round(round(acc * x_scale * w_scale + bias) + residual) (residual may be NULL); xq_out / x_scale_out =
 * mf_rmsnorm_dynamic_quant(h_out, gamma, smooth, eps, out_layout).  Bit-identical to mf_w8a8_gemm(residual)
 * followed by mf_rmsnorm_dynamic_quant; when K is split across workgroups the integer sum of the splits, the add,
 * the norm and the quantisation are one kernel.  N % 8 == 0, N <= 16384.  Workspace as for mf_w8a8_gemm. */
int mf_w8a8_gemm_add_rmsnorm_quant(int8_t* xq_out, float* x_scale_out, void* h_out, const int8_t* xq,
                                   const float* x_scale, const void* w_packed, const float* w_scale, const void* bias,
                                   const void* residual, const void* gamma, const float* smooth, float eps, int m,
                                   int n, int k, int dtype, int gamma_dtype, int x_layout, int out_layout,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* The fused W8A8 QKV projection with RoPE and the cache scatter behind it (infer_attention.py:441-463 behind the
 * golden-stick QuantBatchMatmul of the fused w_qkv): as mf_w8a16_qkv_rope_and_cache, for int8 activations.  Same
 * values as mf_w8a8_gemm followed by mf_rope_and_cache on the column slices; when K is split across workgroups the
 * integer sum of the splits, the dequantisation, the rotation and the scatter are one kernel.  head_dim % 16 == 0.
 * Workspace as for mf_w8a8_gemm with n = the full QKV width. */
int mf_w8a8_qkv_rope_and_cache(void* qkv, const int8_t* xq, const float* x_scale, const void* w_packed,
                               const float* w_scale, const void* bias, const void* cos, const void* sin,
                               void* key_cache, void* value_cache, const int32_t* slot_mapping, int m, int n_heads,
                               int n_kv_heads, int head_dim, int64_t num_slots, int k, int dtype, int table_dtype,
                               int x_layout, void* workspace, size_t workspace_bytes, void* stream);

/* ---- mixture of experts --------------------------------------------------------------------------- */

/* TopKRouter.gating — mindformers/parallel_core/inference/transformer/moe/router.py:49-63: the router's dense
 * projection, logits = cast(x, router_dense_type) . w^T with w [n_experts, hidden] in the router's type.
 * x [tokens, hidden] in `dtype`; w fp32 (w_dtype MF_FP32: products and sums in fp32) or of the activation type
 * (w_dtype == dtype: a 16-bit router, whose projection output is rounded to that type); logits fp32
 * [tokens, n_experts] (routing() casts to fp32 before scoring, router.py:127-128).  hidden % 4 == 0.  The sum over
 * hidden is taken in a fixed order (slices of hidden added in sequence), so results do not depend on scheduling.
 * workspace: mf_router_gate_workspace_bytes(tokens, n_experts, hidden) bytes (0 when hidden is not sliced). */
size_t mf_router_gate_workspace_bytes(int tokens, int n_experts, int hidden);
int mf_router_gate_gemm(float* logits, const void* x, const void* w, int tokens, int n_experts, int hidden, int dtype,
                        int w_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* FusedAddTopKDiv(logits, bias, ...) — mindformers/parallel_core/inference/transformer/moe/router.py:129-140;
 * unfused form research/deepseek3/moe.py:763-778, mindformers/modules/transformer/moe.py:1529-1576.
 * s = sigmoid(logits); sb = s + bias; per group score = sum of its two largest sb; keep the topk_group best
 * groups; top-k of sb over kept groups (ties: lower index); w = s[idx]; if renorm w /= sum(w); w *= scale.
 * logits fp32 [T,E]; bias fp32 [E] or NULL; weights_out in `dtype` [T,k]; index_out int32 [T,k].
 * E <= 1024, E % n_group == 0; n_group <= 1 or topk_group >= n_group disables group limiting.
 * biased_weights != 0 returns w = sb[idx] instead (the plain top-k branch of router.py:142-146, which
 * normalises the biased scores and applies no scale). */
int mf_moe_route(void* weights_out, int32_t* index_out, const float* logits, const float* bias, int tokens,
                 int n_experts, int k, int n_group, int topk_group, float scale, int renorm, int biased_weights,
                 int dtype, void* stream);

/* MoeInitRoutingV2(x, expert_index, ..., expert_tokens_count_or_cumsum_flag=2) — moe_layer.py:136-146.
 * Stable counting sort of the (token, choice) pairs (flattened t*k + j) by expert.  permuted_x [T*k, H];
 * row_map[t*k+j] = permuted row of that pair; counts int64 [E] (group_list, moe_layer.py:148);
 * offsets int32 [E+1] = exclusive prefix sum of counts (for the grouped GEMM).  T*k <= 65536. */
int mf_moe_permute(void* permuted_x, int32_t* row_map, int64_t* counts, int32_t* offsets, const void* x,
                   const int32_t* expert_index, int tokens, int k, int n_experts, int hidden, int dtype,
                   void* stream);

/* GroupedMatmulV4(split_item=3, group_type=0, group_list_type=1) with int8 expert weights —
 * mindformers/parallel_core/inference/transformer/moe/experts.py:116-117,136-137.
 * Rows offsets[e]..offsets[e+1] of x use expert e: y = (x . w[e]^T) * scale[e].  w_packed holds the E experts
 * back to back, each mf_w8a16_pack_weight of its int8 [N, K] matrix (the [E, in, out] parameter of
 * experts.py:71-72 transposed at load), mf_w8a16_packed_bytes(n, k) apart; scale fp32 [E, N]. */
int mf_grouped_w8a16_gemm(void* y, const void* x, const void* w_packed, const float* scale, const int32_t* offsets,
                          int n_experts, int total_rows, int n, int k, int dtype, void* stream);

/* mf_grouped_w8a16_gemm with the experts' activation in its epilogue (experts.py:151-170: fc1, split into gate and
 * hidden halves, hidden * silu(gate)): the rows of every expert's weight are interleaved gate / up as for
 * mf_w8a16_gemm_silu_mul, y is [R, N/2]; same bits as mf_grouped_w8a16_gemm followed by mf_silu_mul(layout 1). */
int mf_grouped_w8a16_gemm_silu_mul(void* y, const void* x, const void* w_packed, const float* scale,
                                   const int32_t* offsets, int n_experts, int total_rows, int n, int k, int dtype,
                                   void* stream);

/* GroupedMatmulV4 on int8 activations and weights: the routed experts of a W8A8 checkpoint
 * (mindformers/parallel_core/inference/transformer/moe/experts.py:116-117,136-137 with the quantization config of
 * research/deepseek3/deepseek_r1_671b/predict_deepseek_r1_671b_w8a8.yaml:89-92).  xq int8 [R, K] row-major and
 * x_scale [R] as mf_dynamic_quant_per_token(layout 0) writes them for the permuted rows; w_packed / w_scale / offsets
 * as for mf_grouped_w8a16_gemm.  Exact int32 accumulators (acc_out int32 [R, N], may be NULL), y = acc * x_scale[r] *
 * w_scale[e, n] rounded to out_dtype (y may be NULL when only the accumulators are wanted).  K % 16 == 0. */
int mf_grouped_w8a8_gemm(void* y, int32_t* acc_out, const int8_t* xq, const float* x_scale, const void* w_packed,
                         const float* w_scale, const int32_t* offsets, int n_experts, int total_rows, int n, int k,
                         int out_dtype, void* stream);

/* MoeTokenUnpermute(permuted_tokens, sorted_indices, probs) — moe_layer.py:151-155.
 * out[t,:] = sum_j probs[t,j] * y[row_map[t*k+j],:] accumulated in fp32 in order j = 0..k-1
 * (+ shared[t,:] if shared != NULL, the shared-expert add of moe_layer.py:159-160). */
int mf_moe_unpermute(void* out, const void* y, const int32_t* row_map, const void* probs, const void* shared,
                     int tokens, int k, int hidden, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MF_DECODE_H_ */
