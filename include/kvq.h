/*
 * kvq.h -- C ABI of the MI355X (gfx950) int8 KV-cache attention library.
 *
 * Conventions (all entry points):
 *   - extern "C", plain pointers and sizes; every pointer is DEVICE memory
 *     unless the comment says host.  The caller owns every buffer.
 *   - work is enqueued on `stream` (a hipStream_t passed as void*; NULL is the
 *     default stream) and the call returns without synchronising.
 *   - return value: 0 on success, a negative errno-style code otherwise
 *     (KVQ_EINVAL for rejected arguments, KVQ_EHIP for a HIP runtime error).
 *     kvq_last_error() returns a thread-local, human-readable reason.
 *   - no entry point allocates or frees device memory; scratch comes in as a
 *     caller-provided workspace whose size the *_workspace_bytes() helpers give
 *     (kvq_paged_attn_int8_static_scratch uses a fixed array of the library instead).
 *   - stateless, thread-safe; strides are taken from the caller, never assumed.
 *
 * Each declaration cites the interface of MetaX-MACA/vLLM-metax it stands in
 * for (file:line relative to that tree).
 */
#ifndef KVQ_H_
#define KVQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KVQ_ABI_VERSION 19

#define KVQ_OK 0
#define KVQ_EINVAL (-22)
#define KVQ_EHIP (-5)
#define KVQ_ENOSYS (-38)

/* element types of activations (query / key / value / output) */
#define KVQ_F32 0
#define KVQ_BF16 1
#define KVQ_F16 2

typedef void* kvq_stream_t;

#if defined(__GNUC__)
#define KVQ_API __attribute__((visibility("default")))
#else
#define KVQ_API
#endif

/*
 * Byte geometry of the paged int8 cache with inline per-(token, head) scales.
 * One (block, slot, head) record is [K codes | K scale fp32 | V codes | V scale fp32],
 * the codes of a half taking head_size bytes (head_size / 2 for KVQ_CODE_INT4); the four offsets locate those pieces
 * relative to the cache base for block 0 / slot 0 / head 0, the three strides
 * step to the next block / slot / head.  This is exactly the information the
 * reference's typed views carry: key_cache / value_cache =
 * kv_cache.transpose(1, 2).split(D + 4, -1) and the fp32 as_strided scale views
 * (vllm_metax/v1/attention/backends/triton_attn.py:418-479, 729-739), for either
 * physical order returned by get_kv_cache_stride_order (:350-372).
 */
typedef struct kvq_cache_geom {
  int64_t k_off, v_off, ks_off, vs_off;           /* bytes */
  int64_t stride_block, stride_slot, stride_head; /* bytes */
  int32_t num_kv_heads, head_size, block_size;
  int32_t code_type;                              /* KVQ_CODE_INT8 (0), KVQ_CODE_FP8_E4M3 or KVQ_CODE_INT4 */
} kvq_cache_geom;

/*
 * What a code byte of the cache is.  KVQ_CODE_INT8: the reference's
 * int8_per_token_head mode, scale = absmax / 127, code = rint(x / scale).
 * KVQ_CODE_FP8_E4M3: its fp8_per_token_head mode over the same record layout (the
 * element is one byte either way, vllm_metax/v1/attention/backends/triton_attn.py:
 * 336-348, 729-739): OCP e4m3fn bit patterns, scale = absmax / 448, code = the
 * e4m3fn number nearest to x / scale (ties to even, saturating at +-448).  Served
 * by kvq_reshape_and_cache_int8 and kvq_paged_attn_int8 (and its static-scratch
 * form); the fixed-partition entry point is int8 only.
 *
 * KVQ_CODE_INT4: the int4_per_token_head mode, of which the reference states only the record width
 * (triton_attn.py:336-348: two values per byte, head_size / 2 code bytes + the 4 scale bytes per half;
 * the arithmetic lives in upstream Triton kernels it does not vendor).  This library's rule, a decision
 * of this build: scale = max(absmax, eps) / 7 (fp32 division), code = clamp(rint(x / scale), -8, 7)
 * (ties to even) as a 4-bit two's-complement number, dim 2 i in the low nibble of byte i and dim 2 i + 1
 * in the high one.  Served by kvq_reshape_and_cache_int8, kvq_paged_attn_int8 and its fused-write and
 * static-scratch forms (head sizes 64, 128, 256).
 */
#define KVQ_CODE_INT8 0
#define KVQ_CODE_FP8_E4M3 1
#define KVQ_CODE_INT4 2

/* flags of the `causal` argument of kvq_paged_attn_int8 and its static-scratch form */
#define KVQ_ATTN_CAUSAL 1
#define KVQ_ATTN_NO_DECODE_ROWS 2

/* Byte geometry of the int8 MLA latent cache: per block, block_size code rows
 * of (kv_lora_rank + rope_dim) bytes followed by block_size fp32 scales. */
typedef struct kvq_mla_geom {
  int64_t stride_block, stride_row, scale_off; /* bytes */
  int32_t kv_lora_rank, rope_dim, block_size;
  int32_t reserved;
} kvq_mla_geom;

KVQ_API int kvq_abi_version(void);
KVQ_API const char* kvq_last_error(void);

/* Number of compute units of the current device (host query, cached). */
KVQ_API int kvq_device_num_cus(void);

/*
 * Batch-invariant mode, process-wide: the switch the reference reads from envs.VLLM_BATCH_INVARIANT
 * (vllm_metax/v1/attention/backends/mla/triton_mla.py:247-253: one KV split; triton_attn.py:310-312:
 * supports_batch_invariance).  While it is on, every decode sequence is cut into splits by its OWN length
 * alone and its split states are merged in split order, so the bits of a row do not depend on what else the
 * batch holds, on the batch size or on the device's CU count: kvq_paged_attn_int8* cut a sequence into at
 * most 32 equal spans of at least 256 tokens, kvq_mla_decode_* into 8 splits.  Prefill rows never depend on
 * their neighbours.  The workspace queries return what the mode needs, so set it before sizing workspaces
 * and not while launches are being enqueued.  Returns the previous setting.
 */
KVQ_API int kvq_set_batch_invariant(int on);
KVQ_API int kvq_get_batch_invariant(void);

/*
 * Quantise-on-write of new K/V tokens into the paged cache.
 * Stands in for triton_reshape_and_cache_flash_per_token_head_quant(key, value,
 * key_cache, value_cache, k_scale_cache, v_scale_cache, slot_mapping,
 * kv_quant_mode=INT8_PER_TOKEN_HEAD), called at
 * vllm_metax/v1/attention/backends/triton_attn.py:805-814; native sibling op
 * reshape_and_cache_flash, csrc/libtorch_stable/torch_bindings.cpp:834-840 and
 * cache_kernels.cu:309-395, 828-897.
 *
 * key/value: [>= num_tokens, num_kv_heads, head_size] of `src_dtype`, strides in
 * elements (last dim contiguous).  num_tokens is slot_mapping's length (key may
 * be longer: padding).  Tokens with slot < 0 are skipped.  Per (token, head):
 * amax = max|x| floored at `eps`, scale = amax / 127, code =
 * clamp(rint(x / scale), -128, 127); codes and scale are bit-exact.
 */
KVQ_API int kvq_reshape_and_cache_int8(const void* key, const void* value, int src_dtype,
                               int64_t key_stride_t, int64_t key_stride_h,
                               int64_t value_stride_t, int64_t value_stride_h, void* cache,
                               const kvq_cache_geom* geom, const int64_t* slot_mapping,
                               int64_t num_tokens, float eps, kvq_stream_t stream);

/*
 * Workspace for kvq_paged_attn_int8: split-K partial states.  Depends on the
 * device (number of resident workgroups), so it is a host query; the value is
 * an upper bound for any batch of at most max_num_seqs sequences.
 * Counterpart of the reference's pre-sized split-softmax scratch,
 * vllm_metax/v1/attention/backends/triton_attn.py:155-176.
 */
KVQ_API size_t kvq_paged_attn_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size);

/*
 * Rotary embedding of the step's query and key rows fused with the quantise-on-write of the step's K / V:
 * the body of do_rope_and_kv_cache_update(layer, query, key, value, positions, cos_sin_cache, is_neox,
 * kv_cache, layer_slot_mapping), which the reference's backend declares and refuses
 * (vllm_metax/v1/attention/backends/triton_attn.py:833-848: fused_rope_kvcache_supported() is False and the
 * method raises "Not supported on Maca").  query [T, Hq, D] and key [T, Hkv, D] are rotated IN PLACE over their
 * first rot_dim dims (pair i = (i, rot_dim/2 + i) when is_neox, else (2i, 2i+1); cos_sin_cache
 * [max_position, rot_dim] = rot_dim/2 cosines then rot_dim/2 sines; the arithmetic of the reference's fused
 * MLA kernel, csrc/libtorch_stable/cache_kernels_fused.cu:55-117: every product and sum rounded on its own in
 * the activation type); the rotated K rows and the V rows are then quantised into the cache exactly as
 * kvq_reshape_and_cache_int8 would.  A token whose slot is negative is padding: neither rotated nor written.
 * Head sizes up to 256; every code type.
 */
KVQ_API int kvq_rope_and_cache_int8(const int64_t* positions, void* query, int64_t q_stride_t, int64_t q_stride_h,
                            int num_q_heads, void* key, int64_t key_stride_t, int64_t key_stride_h,
                            const void* value, int64_t value_stride_t, int64_t value_stride_h,
                            int src_dtype, const void* cos_sin_cache, int cos_sin_dtype, int rot_dim,
                            int is_neox, void* cache, const kvq_cache_geom* geom,
                            const int64_t* slot_mapping, int64_t num_tokens, float eps,
                            kvq_stream_t stream);

/*
 * Varlen paged attention over the int8 cache: decode rows and chunked-prefill
 * rows in one call.  Stands in for unified_attention(q, k=key_cache,
 * v=value_cache, out, cu_seqlens_q, max_seqlen_q, seqused_k, max_seqlen_k,
 * softmax_scale, causal, ..., block_table, ..., kv_quant_mode, k_scale_cache,
 * v_scale_cache) at vllm_metax/v1/attention/backends/triton_attn.py:688-725.
 *
 * q / out: [num_tokens, num_q_heads, head_size], strides in elements.
 * Sequence i owns rows cu_seqlens_q[i] .. cu_seqlens_q[i+1]-1 and attends keys
 * 0 .. seq_lens[i]-1 (bottom-right causal when `causal`), gathered through
 * block_table[i * bt_stride + pos / block_size].  K = code * k_scale,
 * V = code * v_scale, softmax in fp32.  max_query_len (host) selects the tiles:
 * rows of single-token sequences go to the bandwidth-bound split-K tile, longer
 * query runs to the MFMA prefill tile.  lse (optional, [num_tokens, num_q_heads]
 * fp32, natural log) may be NULL.
 *
 * window_size > 0: a query at position p sees keys p - window_size + 1 .. p only
 * (the reference passes window_size = (sliding_window - 1, 0),
 * vllm_metax/v1/attention/backends/triton_attn.py:507-512, 701; needs `causal`);
 * 0 = no window.  softcap > 0: logits become softcap * tanh(scale * q.k / softcap)
 * (triton_attn.py:703; semantics as in the reference's test oracle,
 * tests/kernels/attention/test_triton_unified_attention.py:63-70); 0 = none.
 *
 * sinks (optional, [num_q_heads] fp32, may be NULL): attention sinks, the `sinks` argument of the reference's
 * unified_attention call (triton_attn.py:712, 784; supports_sink(), :390-392).  Head h's softmax runs over its
 * keys' logits and one more logit, sinks[h] (as given: not multiplied by `scale`), whose value row is zero:
 * out = sum_j exp(s_j) v_j / (exp(sinks[h]) + sum_j exp(s_j)); lse includes the sink's term.
 *
 * alibi_slopes (optional, [num_q_heads] fp32, may be NULL; needs `causal`): ALiBi, the alibi_slopes of the
 * reference's attention op (triton_attn.py:504-506, 699; paged_attention_v2's alibi_slopes,
 * csrc/libtorch_stable/torch_bindings.cpp:631-641).  The scaled (and capped) logit of the query at position p
 * and the key at position j gets alibi_slopes[h] * (j - p) added: for a decode row, the
 * alibi_slope * (token_idx - seq_len + 1) of the native kernel (csrc/libtorch_stable/attention/
 * attention_kernels.cuh) and of its test oracle (tests/kernels/attention/test_attention.py:109-117); for a query
 * run, each row with its own position.  lse is that of the biased logits.  The square-root form
 * (use_alibi_sqrt, triton_attn.py:405-407, 700) is not built.
 *
 * `causal` is a set of flags: KVQ_ATTN_CAUSAL (1, the reference's causal=True) and, optionally,
 * KVQ_ATTN_NO_DECODE_ROWS (2): the caller's promise that no sequence of this batch has exactly one query
 * row (a pure prefill batch; a metadata builder knows it from the host copy of query_start_loc).  The
 * split-K decode kernel and its reduce are then not launched at all; with a one-row sequence in the batch
 * after all, that row's output is left unwritten.
 *
 * Value range: the weights enter the second product as fp16 numbers
 * p * v_scale * 2^8, so a V row whose scale exceeds 255.8 (int8 codes: absmax
 * above 32 500; fp8 codes: above 114 000) is attended as if its scale were 255.8.
 * Small values need no care: with V of magnitude 1e-3 spread over 8192 keys the
 * result is within 3e-4 relative of the fp32 result.
 */
KVQ_API int kvq_paged_attn_int8(void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h,
                        const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                        const void* cache, const kvq_cache_geom* geom,
                        const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
                        const int32_t* cu_seqlens_q, int num_seqs, int num_q_heads,
                        int max_query_len, float scale, int causal, int window_size,
                        float softcap, const float* sinks, const float* alibi_slopes, float* lse, void* workspace, size_t workspace_bytes,
                        kvq_stream_t stream);

/*
 * kvq_paged_attn_int8 with the long runs' CONTEXT cut into `prefill_splits` ranges (1..8; 1 = the plain call).
 * It has no counterpart in the reference's call (its Triton kernel chooses its own decomposition): the caller's
 * metadata builder knows what a launch holds.  For a launch whose long query runs make few workgroups on a long
 * context -- one request's small prefill chunk: 512 tokens on 32k cached ones are 128 workgroups that each walk
 * the whole context, 1.2 ms whatever the chunk size -- every (query block, kv head) item becomes `prefill_splits`
 * workgroups that each take a range of the context's tiles and leave a partial state per (query row, q head); a
 * merge kernel combines them with the log-sum-exp algebra of merge_attn_states (sinks and lse as in the plain
 * call).  Only the workgroup-shared tile takes part (head sizes up to 128, max_query_len x group >= 64); one-token
 * sequences, short runs and head size 256 are served as in the plain call.  Same results within the tolerance of
 * the plain call (the order of the additions differs).  num_tokens = the rows of q; the workspace must hold
 * kvq_paged_attn_split_prefill_workspace_bytes(num_seqs, num_q_heads, head_size, num_tokens, prefill_splits)
 * bytes (the plain workspace + num_tokens x num_q_heads x prefill_splits x (head_size + 2) floats).
 */
KVQ_API size_t kvq_paged_attn_split_prefill_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size,
                                                            int num_tokens, int prefill_splits);
KVQ_API int kvq_paged_attn_int8_split_prefill(void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h,
                        const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                        const void* cache, const kvq_cache_geom* geom,
                        const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
                        const int32_t* cu_seqlens_q, int num_seqs, int num_q_heads,
                        int max_query_len, float scale, int causal, int window_size,
                        float softcap, const float* sinks, const float* alibi_slopes, float* lse,
                        int num_tokens, int prefill_splits, void* workspace, size_t workspace_bytes,
                        kvq_stream_t stream);

/*
 * A decode step in ONE launch: the cache update of the step's new tokens and the attention
 * over the updated cache -- kvq_reshape_and_cache_int8 followed by kvq_paged_attn_int8 with
 * max_query_len == 1, same bytes in the cache and same output.  For a backend that sets
 * forward_includes_kv_cache_update (the reference's attribute of that name,
 * vllm_metax/v1/attention/backends/triton_attn.py:296; its forward then receives key and
 * value and owns the update that do_kv_cache_update, triton_attn.py:788-840, does otherwise).
 * Row i of key / value [num_seqs, Hkv, D] (src_dtype, element strides) is the token at
 * position seq_lens[i] - 1 of sequence i; its slot comes from the block table.  The
 * workgroup that streams a sequence's last tile quantises the row (the write kernel's
 * arithmetic) and stores the record before it loads the tile.  Decode rows only: every
 * sequence has exactly one query row (row i); sequences of length 0 are skipped.
 * slot_mapping (int64 [num_seqs], may be NULL) is the step's slot mapping as the write
 * kernel takes it: a row whose entry is negative is a padding row and is NOT written
 * (cache_kernels.cu:322-326), whatever its sequence length says; a row with a
 * non-negative entry is written at the place the block table gives, which the caller's
 * metadata makes the same slot.  NULL: every row of a non-empty sequence is written.
 * eps as in kvq_reshape_and_cache_int8.  Workspace as for kvq_paged_attn_int8.
 */
KVQ_API int kvq_paged_attn_int8_fused_write(void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h,
                        const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                        const void* key, const void* value, int src_dtype,
                        int64_t key_stride_t, int64_t key_stride_h,
                        int64_t value_stride_t, int64_t value_stride_h, float eps,
                        void* cache, const kvq_cache_geom* geom,
                        const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
                        const int64_t* slot_mapping,
                        int num_seqs, int num_q_heads, float scale, int window_size,
                        float softcap, const float* sinks, const float* alibi_slopes, float* lse, void* workspace, size_t workspace_bytes,
                        kvq_stream_t stream);

/*
 * kvq_paged_attn_int8 for callers that cannot hand over a workspace they allocated:
 * code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  Same arguments, results and
 * kernels as kvq_paged_attn_int8, minus the workspace: the split-K partial states
 * live in a fixed array of KVQ_STATIC_SCRATCH_BYTES that is part of the library's
 * code object (each GPU the library runs on holds one copy until the process
 * ends).  The call allocates and frees nothing.  A batch is served if
 * kvq_paged_attn_workspace_bytes(num_seqs, num_q_heads, head_size) <=
 * KVQ_STATIC_SCRATCH_BYTES (the partial states plus the kernels' notes: 32 q
 * heads of 128 dims on 256 compute units: up to 1255 sequences); a larger one
 * is rejected with KVQ_EINVAL and nothing is launched.  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (different
 * streams, different threads) race and must be serialised by the caller.
 * kvq_paged_attn_static_scratch_bytes() returns the array's size and is the
 * set-up hook: called once per device, with that device current and outside any
 * stream capture, it resolves the array's device address, so that calls under
 * capture make no runtime query (the entry point resolves it on its first call
 * on a device otherwise).
 */
#define KVQ_STATIC_SCRATCH_BYTES (24u << 20)
KVQ_API size_t kvq_paged_attn_static_scratch_bytes(void);
KVQ_API int kvq_paged_attn_int8_static_scratch(
    void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h, const void* q, int q_dtype,
    int64_t q_stride_t, int64_t q_stride_h, const void* cache, const kvq_cache_geom* geom,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens, const int32_t* cu_seqlens_q,
    int num_seqs, int num_q_heads, int max_query_len, float scale, int causal, int window_size,
    float softcap, const float* sinks, const float* alibi_slopes, float* lse, kvq_stream_t stream);

/*
 * Fixed-partition split-K decode + reduce (one query row per sequence).
 * Stands in for paged_attention_v2(out, exp_sums, max_logits, tmp_out, query,
 * key_cache, value_cache, num_kv_heads, scale, block_tables, seq_lens,
 * block_size, max_seq_len, ...), csrc/libtorch_stable/torch_bindings.cpp:631-641,
 * paged_attention_v2.cu:44-135: partition j of `partition_size` tokens stores a
 * locally normalised tmp_out[b, h, j, :], max_logits[b, h, j] and
 * exp_sums[b, h, j] (all fp32 here); the reduce then writes out.
 * max_num_partitions = ceil(max_seq_len / partition_size).
 * alibi_slopes ([num_q_heads] fp32 or NULL): the op's alibi_slopes argument; a key at position j gets
 * alibi_slopes[h] * (j - seq_len + 1) on its scaled logit before the partition's maximum is taken
 * (csrc/libtorch_stable/attention/attention_kernels.cuh), so max_logits and exp_sums are those of the
 * biased logits.
 */
KVQ_API int kvq_paged_attn_v2_int8(void* out, int out_dtype, float* exp_sums, float* max_logits,
                           float* tmp_out, const void* q, int q_dtype, int64_t q_stride_t,
                           int64_t q_stride_h, const void* cache, const kvq_cache_geom* geom,
                           const int32_t* block_table, int64_t bt_stride,
                           const int32_t* seq_lens, int num_seqs, int num_q_heads, float scale,
                           const float* alibi_slopes, int partition_size, int max_num_partitions,
                           kvq_stream_t stream);

/*
 * The reduce stage on its own.  Stands in for paged_attention_v2_reduce_kernel,
 * csrc/libtorch_stable/attention/attention_kernels.cuh:556-661 (and the Triton
 * stage 2, vllm_metax/v1/attention/ops/triton_decode_attention.py:582-646):
 * w_j = exp_sums_j * exp(max_logits_j - max), out = sum_j w_j tmp_out_j / sum_j w_j;
 * a single partition is copied through.  lse (optional) = max + log(sum_j w_j).
 */
KVQ_API int kvq_splitk_reduce(void* out, int out_dtype, float* lse, const float* exp_sums,
                      const float* max_logits, const float* tmp_out, const int32_t* seq_lens,
                      int num_seqs, int num_q_heads, int head_size, int partition_size,
                      int max_num_partitions, kvq_stream_t stream);

/* Directions of kvq_swap_blocks. */
#define KVQ_DEVICE_TO_DEVICE 0
#define KVQ_DEVICE_TO_HOST 1
#define KVQ_HOST_TO_DEVICE 2

/*
 * Move whole cache blocks: dst block block_mapping[i][1] = src block
 * block_mapping[i][0], block_bytes each.  Stands in for swap_blocks(src, dst,
 * block_size_in_bytes, block_mapping), csrc/libtorch_stable/cache_kernels.cu:33-77
 * (schema torch_bindings.cpp:816-818).  block_mapping is a HOST array of int64
 * pairs with element strides map_stride0 / map_stride1, as the reference requires
 * (cache_kernels.cu:51-55).  A block of the int8 layouts (kvq_cache_geom /
 * kvq_mla_geom: block_bytes = stride_block) holds codes and scales together, so
 * the move is self-contained.  Asynchronous on `stream`; host memory should be
 * pinned.  Pairs must not overlap when src and dst are the same allocation.
 */
KVQ_API int kvq_swap_blocks(const void* src, void* dst, int64_t block_bytes,
                    const int64_t* block_mapping, int64_t num_pairs, int64_t map_stride0,
                    int64_t map_stride1, int direction, kvq_stream_t stream);

/*
 * n independent copies (src_ptrs[i] -> dst_ptrs[i], sizes[i] bytes), submitted
 * together.  Stands in for swap_blocks_batch(src_ptrs, dst_ptrs, sizes, ...),
 * csrc/libtorch_stable/cache_kernels.cu:79-178 (schema torch_bindings.cpp:821-823).
 * The three arrays are HOST arrays of int64.  all_on_device != 0 promises that
 * every pointer is device memory of the current device: the copies then run as
 * one kernel launch per 64 entries; otherwise each entry is one asynchronous
 * copy whose direction is taken from the pointers.
 */
KVQ_API int kvq_swap_blocks_batch(const int64_t* src_ptrs, const int64_t* dst_ptrs,
                          const int64_t* sizes, int64_t n, int all_on_device,
                          kvq_stream_t stream);

/*
 * copy_blocks / copy_blocks_mla over the int8 format: for every (src, dst) row of
 * block_mapping [num_pairs, 2] (int64, contiguous, ON THE DEVICE) and every
 * layer, block dst of the layer's cache becomes a copy of block src -- the
 * kernels of csrc/libtorch_stable/cache_kernels.cu:184-232, exercised by
 * tests/kernels/attention/test_cache.py:55-110 and :592-650.  A block of these
 * layouts holds keys, values and their scales, so one cache pointer per layer
 * replaces the reference's key/value pointer pair.  cache_ptrs [num_layers]
 * (int64 addresses, on the device); block_bytes = the cache's block stride;
 * pairs naming a block outside [0, num_blocks) are skipped (the host cannot
 * check a device-resident mapping without a synchronisation).  A source may be
 * copied to several destinations; sources and destinations must not overlap.
 */
KVQ_API int kvq_copy_blocks(const int64_t* cache_ptrs, int num_layers, const int64_t* block_mapping,
                            int64_t num_pairs, int64_t block_bytes, int64_t num_blocks,
                            kvq_stream_t stream);

/*
 * LSE merge of two partial attention states.  Stands in for merge_attn_states,
 * csrc/libtorch_stable/attention/merge_attn_states.cu:17-192, 246-320 (python
 * chooser vllm_metax/v1/attention/ops/merge_attn_states.py:82-114).
 * outputs [num_tokens, num_heads, head_size] of `dtype` (contiguous);
 * lse tensors [num_heads, num_tokens] fp32; output_lse may be NULL.  +inf LSE is
 * read as -inf; both -inf emits the prefix.  Rows >= prefix_num_tokens copy the
 * suffix.
 */
KVQ_API int kvq_merge_attn_states(void* output, float* output_lse, const void* prefix_output,
                          const float* prefix_lse, const void* suffix_output,
                          const float* suffix_lse, int dtype, int64_t num_tokens, int num_heads,
                          int head_size, int64_t prefix_num_tokens, kvq_stream_t stream);

/*
 * MLA latent quantise-on-write.  Stands in for concat_and_cache_mla(kv_c, k_pe,
 * kv_cache, slot_mapping, kv_cache_dtype, scale),
 * csrc/libtorch_stable/torch_bindings.cpp:843-848, cache_kernels.cu:397-439,
 * 924-985, with the int8 per-token-scale entry this build defines (the
 * reference has none; nearest precedents cache_kernels.cu:441-542, 593-604).
 * kv_c [T, kv_lora_rank], k_pe [T, rope_dim] of `src_dtype` (row strides in
 * elements); one absmax over the whole concatenated row.
 */
KVQ_API int kvq_concat_and_cache_mla_int8(const void* kv_c, const void* k_pe, int src_dtype,
                                  int64_t kv_c_stride, int64_t k_pe_stride, void* cache,
                                  const kvq_mla_geom* geom, const int64_t* slot_mapping,
                                  int64_t num_tokens, float eps, kvq_stream_t stream);

/*
 * Gather + dequantise latent rows into a dense workspace.  Stands in for the
 * quantised branch of gather_and_maybe_dequant_cache(src_cache, dst,
 * block_table, cu_seq_lens, token_to_seq, num_tokens, kv_cache_dtype, scale,
 * seq_starts), csrc/libtorch_stable/cache_kernels.cu:1072-1131, 1181-1247, which
 * the MLA chunked-context prefill calls
 * (vllm_metax/model_executor/layers/attention/mla_attention.py:2017-2140):
 * destination row t belongs to sequence b = token_to_seq[t], position
 * t - cu_seq_lens[b] (+ seq_starts[b] when given), and receives
 * code * row_scale rounded once to `dst_dtype`.  dst [num_tokens, >= R+P],
 * dst_stride in elements.  seq_starts may be NULL.
 */
KVQ_API int kvq_gather_and_dequant_mla_int8(void* dst, int dst_dtype, int64_t dst_stride, const void* cache,
                                    const kvq_mla_geom* geom, const int32_t* block_table,
                                    int64_t bt_stride, const int32_t* cu_seq_lens,
                                    const int32_t* token_to_seq, const int32_t* seq_starts,
                                    int64_t num_tokens, kvq_stream_t stream);

/*
 * Rotary embedding of q_pe and k_pe (in place) fused with the quantise-on-write
 * of the latent row [kv_c | rotated k_pe].  Stands in for
 * concat_and_cache_mla_rope_fused(positions, q_pe, k_pe, kv_c, cos_sin_cache,
 * is_neox, slot_mapping, kv_cache, kv_cache_dtype, kv_cache_scale),
 * csrc/libtorch_stable/cache_kernels_fused.cu:24-168 (schema
 * torch_bindings.cpp:851-862), for the int8 latent cache.
 * q_pe [T, num_q_heads, rot_dim], k_pe [T, rot_dim], kv_c [T, kv_lora_rank] of
 * `dtype` (strides in elements, last dim contiguous); cos_sin_cache
 * [max_position, rot_dim] of `cos_sin_dtype`: row p holds rot_dim/2 cosines, then
 * rot_dim/2 sines.  Pair i of a row is (i, rot_dim/2 + i) when is_neox, else
 * (2i, 2i+1); (x, y) -> (x cos - y sin, y cos + x sin) in `dtype` arithmetic, one
 * rounding per operation.  Tokens with slot < 0 are left entirely untouched.  The
 * row is quantised as by kvq_concat_and_cache_mla_int8 applied to the rotated
 * k_pe: codes and scale are bit-identical to rotating first and writing second.
 */
KVQ_API int kvq_concat_and_cache_mla_rope_int8(const int64_t* positions, void* q_pe,
                                       int64_t q_stride_t, int64_t q_stride_h,
                                       int num_q_heads, void* k_pe, int64_t k_pe_stride,
                                       const void* kv_c, int64_t kv_c_stride, int dtype,
                                       const void* cos_sin_cache, int cos_sin_dtype,
                                       int rot_dim, int is_neox, void* cache,
                                       const kvq_mla_geom* geom,
                                       const int64_t* slot_mapping, int64_t num_tokens,
                                       float eps, kvq_stream_t stream);

/*
 * Gather the latent rows of `batch_size` sequences WITHOUT dequantising them.
 * Stands in for cp_gather_cache(src_cache, dst, block_table, cu_seq_lens,
 * batch_size, seq_starts), csrc/libtorch_stable/cache_kernels.cu:1316-1379,
 * 1397-1462, over the int8 latent cache: destination row t (int8, dst_stride
 * bytes apart) belongs to the sequence b with cu_seq_lens[b] <= t <
 * cu_seq_lens[b+1], position t - cu_seq_lens[b] (+ seq_starts[b] when given, which
 * need not be a multiple of the block size), and receives the row's
 * kv_lora_rank + rope_dim code bytes followed by the 4 bytes of its fp32 scale:
 * the token-major form of a cache whose blocks keep codes and scales apart.
 * Rows >= cu_seq_lens[batch_size] are left untouched.
 */
KVQ_API int kvq_cp_gather_mla_int8(void* dst, int64_t dst_stride, const void* cache,
                           const kvq_mla_geom* geom, const int32_t* block_table,
                           int64_t bt_stride, const int32_t* cu_seq_lens,
                           const int32_t* seq_starts, int batch_size, int64_t num_tokens,
                           kvq_stream_t stream);

/*
 * q_out[t, h, :] = [ql_nope[t, h, :] | q_pe[t, h, :]]: concat_mla_q(ql_nope,
 * q_pe, q_out), csrc/libtorch_stable/cache_kernels.cu:1740-1783 (schema
 * torch_bindings.cpp:893), the step before an MLA decode whose caller holds the
 * absorbed query in two parts.  Strides in elements of `dtype`, last dims
 * contiguous.  (kvq_mla_decode_int8 also takes the two parts directly.)
 */
KVQ_API int kvq_concat_mla_q(void* q_out, int64_t out_stride_t, int64_t out_stride_h,
                             const void* ql_nope, int64_t nope_stride_t, int64_t nope_stride_h,
                             const void* q_pe, int64_t pe_stride_t, int64_t pe_stride_h, int dtype,
                             int64_t num_tokens, int num_heads, int nope_dim, int rope_dim,
                             kvq_stream_t stream);

/*
 * Workspace for kvq_mla_decode_int8 (host query, depends on the device): the fp16
 * split states and their lse values (counterpart of the reference's attn_logits
 * buffer, vllm_metax/v1/attention/backends/mla/triton_mla.py:261-269) plus the
 * query as two int8 terms per element, which the launch prepares once for all
 * splits.  An upper bound for any batch of at most max_num_seqs sequences.
 */
KVQ_API size_t kvq_mla_decode_workspace_bytes(int max_num_seqs, int num_heads, int kv_lora_rank);

/*
 * MLA decode over the int8 latent cache.  Stands in for
 * TritonMLAImpl.forward_mqa -> decode_attention_fwd(q, k_buffer, v_buffer, o,
 * lse, block_table, seq_lens, attn_logits, num_kv_splits, sm_scale, page_size,
 * ..., is_mla=True), vllm_metax/v1/attention/backends/mla/triton_mla.py:226-295,
 * vllm_metax/v1/attention/ops/triton_decode_attention.py:763-825.
 * q [B, H, kv_lora_rank + rope_dim] (absorbed) with q_pe NULL, or -- the
 * (ql_nope, q_pe) form of forward_mqa's first argument, triton_mla.py:226-238,
 * taken as it is, without the concatenation -- q = ql_nope [B, H, kv_lora_rank]
 * and q_pe [B, H, rope_dim] of the same dtype (strides in elements); out
 * [B, H, kv_lora_rank] contiguous and 16-byte aligned, lse [B, H] fp32 natural
 * log (may be NULL).
 */
KVQ_API int kvq_mla_decode_int8(void* out, int out_dtype, float* lse, const void* q, int q_dtype,
                        int64_t q_stride_b, int64_t q_stride_h, const void* q_pe,
                        int64_t q_pe_stride_b, int64_t q_pe_stride_h, const void* cache,
                        const kvq_mla_geom* geom, const int32_t* block_table,
                        int64_t bt_stride, const int32_t* seq_lens, int num_seqs,
                        int num_heads, float scale, void* workspace, size_t workspace_bytes,
                        kvq_stream_t stream);

/*
 * An MLA decode step in ONE launch: kvq_concat_and_cache_mla_int8 for the step's new
 * tokens followed by kvq_mla_decode_int8, same bytes in the cache and same output
 * (do_kv_cache_update and forward_mqa of the reference's MLA backend,
 * vllm_metax/v1/attention/backends/mla/triton_mla.py:226-295, which a backend with
 * forward_includes_kv_cache_update may do in one step).  Row i of kv_c
 * [num_seqs, kv_lora_rank] / k_pe [num_seqs, rope_dim] (src_dtype, row strides in
 * elements, rows 4-byte aligned) is the token at position seq_lens[i] - 1 of sequence i;
 * its slot comes from the block table.  The wave that streams the sequence's last tile
 * quantises the row (the write kernel's arithmetic) and stores it before that tile is
 * requested.  Sequences of length 0 are skipped.  eps as in
 * kvq_concat_and_cache_mla_int8; everything else as in kvq_mla_decode_int8.
 */
KVQ_API int kvq_mla_decode_int8_fused_write(void* out, int out_dtype, float* lse, const void* q,
                        int q_dtype, int64_t q_stride_b, int64_t q_stride_h, const void* q_pe,
                        int64_t q_pe_stride_b, int64_t q_pe_stride_h, const void* kv_c,
                        const void* k_pe, int src_dtype, int64_t kv_c_stride,
                        int64_t k_pe_stride, float eps, void* cache,
                        const kvq_mla_geom* geom, const int32_t* block_table,
                        int64_t bt_stride, const int32_t* seq_lens, int num_seqs,
                        int num_heads, float scale, void* workspace, size_t workspace_bytes,
                        kvq_stream_t stream);

/*
 * MLA decode with the query absorption fused in: the first bmm of the
 * reference's MLA layer, ql_nope = q_nope x W_UK_T
 * (vllm_metax/model_executor/layers/attention/mla_attention.py:835-848), runs on
 * the MFMA inside the launch and its result goes straight into the decode's
 * int8 operand layout; the absorbed query is never written to memory in the
 * activation type.  Same results contract, cache, workspace and outputs as
 * kvq_mla_decode_int8 (whose q = ql_nope, q_pe form this replaces).
 * q_nope [B, H, nope_dim] and q_pe [B, H, rope_dim] (strides in elements,
 * 4-byte aligned rows), w_uk_t [H, nope_dim, kv_lora_rank] with contiguous last
 * dim, 16-byte aligned rows (strides multiples of 8); all three KVQ_BF16 or
 * KVQ_F16; nope_dim a multiple of 32.
 */
KVQ_API int kvq_mla_decode_absorb_int8(void* out, int out_dtype, float* lse, const void* q_nope, int q_dtype,
                               int64_t qn_stride_b, int64_t qn_stride_h, int nope_dim,
                               const void* w_uk_t, int64_t w_stride_h, int64_t w_stride_p,
                               const void* q_pe, int64_t q_pe_stride_b, int64_t q_pe_stride_h,
                               const void* cache, const kvq_mla_geom* geom,
                               const int32_t* block_table, int64_t bt_stride,
                               const int32_t* seq_lens, int num_seqs, int num_heads, float scale,
                               void* workspace, size_t workspace_bytes, kvq_stream_t stream);

/*
 * The V up-projection behind the MLA decode: out[b, h, :] = x[b, h, :] . W_UV[h],
 * the second bmm of the reference's MLA layer (`_v_up_proj`,
 * vllm_metax/model_executor/layers/attention/mla_attention.py:1087-1109: x [B, N, L]
 * transposed to [N, B, L], bmm with W_UV [N, L, V], back to [B, N * V]; the plain
 * branch, without quantised weights).  x [num_seqs, num_heads, kv_lora_rank] is
 * what kvq_mla_decode_int8 / _absorb_int8 wrote, w_uv [num_heads, kv_lora_rank,
 * v_head_dim] with the output dims contiguous, out [num_seqs, num_heads,
 * v_head_dim] (a view of [num_seqs, num_heads * v_head_dim]).  All three of
 * `dtype` KVQ_BF16 or KVQ_F16, fp32 accumulation, one rounding at the store;
 * strides in elements.  kv_lora_rank and v_head_dim multiples of 128, W_UV and
 * out rows 16-byte aligned, x rows 4-byte aligned.
 */
KVQ_API int kvq_mla_v_up_proj(void* out, int64_t out_stride_b, int64_t out_stride_h,
                              const void* x, int dtype, int64_t x_stride_b, int64_t x_stride_h,
                              const void* w_uv, int64_t w_stride_h, int64_t w_stride_l,
                              int num_seqs, int num_heads, int kv_lora_rank, int v_head_dim,
                              kvq_stream_t stream);

/*
 * Varlen attention with LSE output over dense K and V: the attention step of
 * the MLA prefill.  Stands in for the two flash_attn_varlen_func calls of
 * vllm_metax/v1/attention/backends/mla/prefill/flash_attn.py:176-221
 * (run_prefill_new_tokens: causal, keys = the new tokens; run_prefill_context_chunk:
 * unmasked, keys = one gathered chunk of the cached context, LSE returned), which
 * vllm_metax/model_executor/layers/attention/mla_attention.py:2017-2140 and
 * 2298-2378 call between gather_and_maybe_dequant_cache + kv_b_proj and
 * merge_attn_states.  The key is taken in the two pieces the layer holds,
 * k_nope [S, H, nope_dim] (a strided view of kv_b_proj's output) and
 * k_pe [S, rope_dim] shared by all heads, instead of the concatenated tensor of
 * mla_attention.py:1995-2015; v [S, H, v_dim] is read at its own head size (no
 * padding to the qk head size, flash_attn.py:138-143).
 * q [T, H, nope_dim + rope_dim]; out [T, H, v_dim]; lse [H, total_q] fp32 natural
 * log, may be NULL.  All of `dtype` KVQ_BF16 or KVQ_F16, strides in elements and
 * multiples of 8 (the token strides of k_nope, k_pe and v below 2^24), pointers
 * 16-byte aligned, `scale` positive and finite.  cu_seqlens_q / cu_seqlens_k
 * [num_seqs + 1] int32 on the device; a sequence longer than max_seqlen_q is
 * only attended for its first max_seqlen_q rows.  With `causal`, key j of a
 * sequence is visible to its query row i iff j <= i + (k_len - q_len).  A row
 * with no visible key gets out = 0 and lse = -inf (what mask_empty_context of
 * mla_attention.py:2104-2110 forces).  Built head dims (nope, rope, v):
 * (128, 64, 128), (64, 32, 64), (128, 0, 128).
 */
KVQ_API int kvq_mla_prefill_attn(const void* q, int dtype, int64_t q_stride_tok, int64_t q_stride_head,
                         const void* k_nope, int64_t kn_stride_tok, int64_t kn_stride_head,
                         const void* k_pe, int64_t kpe_stride_tok, const void* v,
                         int64_t v_stride_tok, int64_t v_stride_head,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int num_seqs,
                         int max_seqlen_q, int64_t total_q, int num_heads, int nope_dim,
                         int rope_dim, int v_dim, float scale, int causal, void* out,
                         int64_t out_stride_tok, int64_t out_stride_head, float* lse,
                         kvq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KVQ_H_ */
