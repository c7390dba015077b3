// kvq_paged_attn_int8: the varlen entry point (decode rows + chunked-prefill rows).
//
// The host never looks at device data: max_query_len (a host integer the caller's
// metadata already carries) decides which tiles are launched, and each kernel skips
// the sequences that are not its kind by reading cu_seqlens_q on the device.
#include <mutex>

#include "kvq_attn_core.cuh"

namespace kvq {


int launch_decode_streamk(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s);
size_t streamk_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size, int num_wg);
size_t streamk_slots(int max_num_seqs, int num_wg);
int decode_streamk_num_wg(int num_kv_heads);
int validate_common(const char* op, const void* q, const void* cache, const kvq_cache_geom* geom,
                    const int32_t* block_table, const int32_t* seq_lens, int num_seqs, int num_q_heads);
int launch_prefill(const AttnIO& io, const int32_t* seq_lens, const int32_t* cu_seqlens_q, int num_seqs,
                   int max_query_len, int causal, int q_dtype, int out_dtype, int32_t* plan, hipStream_t s,
                   int ksplit, float* part);

// Where the context splits' partial states begin in a workspace, and how many bytes they take.
static size_t split_part_offset(size_t streamk_bytes) { return (streamk_bytes + 255) & ~(size_t)255; }
static size_t split_part_bytes(int num_tokens, int num_q_heads, int head_size, int splits) {
  return (size_t)num_tokens * (size_t)num_q_heads * (size_t)splits * (size_t)(head_size + 2) * sizeof(float);
}
constexpr int kMaxPrefillSplits = 8;

// Scratch of the entry point that allocates nothing: a fixed array in the code object's own device
// memory.  Every GPU the library runs on holds one copy, at its own address, until the process ends.
// In host code the array's NAME is only a handle for the runtime; the address kernels may use is the
// one hipGetSymbolAddress returns, resolved once per device and kept in g_dev[].
static __device__ __align__(256) unsigned char scratch[KVQ_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
struct DeviceSymbols {
  void* scratch = nullptr;
};
static std::mutex g_dev_mutex;
static DeviceSymbols g_dev[kMaxDevices];  // guarded by the mutex; nullptr = not resolved yet

// Device address of the array on the current device (resolved on the first call per device).
static int device_symbols(const char* op, DeviceSymbols* out) {
  int dev = -1;
  int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (rc) return rc;
  KVQ_REQUIRE(dev >= 0 && dev < kMaxDevices, "%s: device index %d out of range", op, dev);
  std::lock_guard<std::mutex> lock(g_dev_mutex);
  if (g_dev[dev].scratch == nullptr) {
    void* p = nullptr;
    rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (rc) return rc;
    KVQ_REQUIRE(p != nullptr, "%s: the static scratch array has no device address", op);
    g_dev[dev].scratch = p;
  }
  *out = g_dev[dev];
  return KVQ_OK;
}

// The new tokens of a decode step, for the entry point that writes them into the cache inside the launch.
struct NewTokens {
  const void* key;
  const void* value;
  int dtype;
  int64_t key_stride_t, key_stride_h, value_stride_t, value_stride_h;
  float eps;
  const int64_t* slot_mapping;  // may be nullptr; a negative entry marks a padding row that is not written
};

// Arguments are checked, the launch is shaped and enqueued here; the entry points differ only
// in where the split-K partial states live and in whether the launch also writes the step's new tokens.
static int paged_attn_launch(const char* op, void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h,
                             const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h, const void* cache,
                             const kvq_cache_geom* geom, const int32_t* block_table, int64_t bt_stride,
                             const int32_t* seq_lens, const int32_t* cu_seqlens_q, int num_seqs, int num_q_heads,
                             int max_query_len, float scale, int causal, int window_size, float softcap,
                             const float* sinks, const float* alibi_slopes, float* lse, void* workspace, size_t workspace_bytes, const char* workspace_what,
                             kvq_stream_t stream, const NewTokens* fresh = nullptr, int prefill_splits = 1,
                             int num_tokens = 0) {
  int rc0 = validate_common(op, q, cache, geom, block_table, seq_lens, num_seqs, num_q_heads);
  if (rc0) return rc0;
  KVQ_REQUIRE((causal & ~(KVQ_ATTN_CAUSAL | KVQ_ATTN_NO_DECODE_ROWS)) == 0, "%s: unknown flag in causal (%d)", op, causal);
  const bool no_decode_rows = (causal & KVQ_ATTN_NO_DECODE_ROWS) != 0;
  causal &= KVQ_ATTN_CAUSAL;
  KVQ_REQUIRE(out != nullptr, "%s: out is NULL", op);
  KVQ_REQUIRE(max_query_len >= 1, "%s: max_query_len must be >= 1", op);
  KVQ_REQUIRE(max_query_len == 1 || cu_seqlens_q != nullptr, "%s: cu_seqlens_q is required when max_query_len > 1", op);
  KVQ_REQUIRE(window_size >= 0, "%s: window_size %d must be >= 0 (0 = no sliding window)", op, window_size);
  KVQ_REQUIRE(window_size == 0 || causal, "%s: a sliding window needs causal attention", op);
  KVQ_REQUIRE(softcap >= 0.f && softcap == softcap, "%s: softcap must be >= 0 (0 = none)", op);
  KVQ_REQUIRE(alibi_slopes == nullptr || causal, "%s: alibi_slopes need causal attention", op);
  const kvq_cache_geom& g = *geom;
  const int osz = out_dtype == KVQ_F32 ? 4 : 2;
  KVQ_REQUIRE(((uintptr_t)out % 4) == 0 && (out_stride_t * osz) % 4 == 0 && (out_stride_h * osz) % 4 == 0,
              "%s: out rows must be 4-byte aligned", op);
  const int num_wg = decode_streamk_num_wg(g.num_kv_heads);
  KVQ_REQUIRE(num_wg > 0, "%s: no HIP device", op);
  size_t need = streamk_workspace_bytes(num_seqs, num_q_heads, g.head_size, num_wg);
  const size_t part_at = split_part_offset(need);
  KVQ_REQUIRE(prefill_splits >= 1 && prefill_splits <= kMaxPrefillSplits, "%s: prefill_splits %d must be 1..%d", op,
              prefill_splits, kMaxPrefillSplits);
  if (prefill_splits > 1) {
    KVQ_REQUIRE(num_tokens >= 1, "%s: num_tokens (the rows of q) is required with prefill_splits > 1", op);
    need = part_at + split_part_bytes(num_tokens, num_q_heads, g.head_size, prefill_splits);
  }
  KVQ_REQUIRE(workspace != nullptr && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0,
              "%s: %s of %zu bytes (16-byte aligned) required, got %zu", op, workspace_what, need, workspace_bytes);

  StreamKArgs a{};
  a.io.q = q;
  a.io.q_stride_t = q_stride_t;
  a.io.q_stride_h = q_stride_h;
  a.io.out = out;
  a.io.out_stride_t = out_stride_t;
  a.io.out_stride_h = out_stride_h;
  a.io.out_dtype = out_dtype;
  a.io.lse = lse;
  a.io.cache = static_cast<const uint8_t*>(cache);
  a.io.g = g;
  a.io.block_table = block_table;
  a.io.bt_stride = bt_stride;
  a.io.num_q_heads = num_q_heads;
  a.io.group = num_q_heads / g.num_kv_heads;
  a.io.scale_log2 = scale * kLog2e;
  a.io.bs_magic = (uint32_t)((0x100000000ull + (uint64_t)geom->block_size - 1) / (uint64_t)geom->block_size);
  a.io.window = window_size;
  a.io.sinks = sinks;
  a.io.alibi = alibi_slopes;
  a.io.cap_c = softcap * kLog2e;
  a.io.cap_k = softcap > 0.f ? 2.0f / softcap : 0.f;  // 2 log2(e) / cap_c
  a.seq_lens = seq_lens;
  a.cu_seqlens_q = cu_seqlens_q;
  a.num_seqs = num_seqs;
  a.num_wg = num_wg;
  const size_t slots = streamk_slots(num_seqs, num_wg);
  a.fixed_spans = batch_invariant() ? 1 : 0;
  a.part_o = static_cast<float*>(workspace);
  a.part_ml = a.part_o + slots * (size_t)num_q_heads * (size_t)g.head_size;
  // 8-byte aligned: a slot's (D + 2) floats are a multiple of 8 bytes
  a.wg_info = reinterpret_cast<int64_t*>(a.part_ml + slots * (size_t)num_q_heads * 2);
  a.seq_first_unit = a.wg_info + 2 * (size_t)num_wg + 2;

  if (fresh != nullptr) {
    KVQ_REQUIRE(max_query_len == 1, "%s: the fused write takes decode rows only (max_query_len == 1)", op);
    KVQ_REQUIRE(fresh->key != nullptr && fresh->value != nullptr, "%s: key / value is NULL", op);
    KVQ_REQUIRE(fresh->dtype == KVQ_F32 || fresh->dtype == KVQ_BF16 || fresh->dtype == KVQ_F16,
                "%s: unknown src_dtype %d", op, fresh->dtype);
    KVQ_REQUIRE(fresh->eps >= 0.f, "%s: eps must not be negative", op);
    KVQ_REQUIRE(g.head_size == 64 || g.head_size == 128 || g.head_size == 256,
                "%s: head_size %d is not built", op, g.head_size);
    const int esz = fresh->dtype == KVQ_F32 ? 4 : 2;
    KVQ_REQUIRE(((uintptr_t)fresh->key % 4) == 0 && ((uintptr_t)fresh->value % 4) == 0 &&
                    ((fresh->key_stride_t | fresh->key_stride_h | fresh->value_stride_t | fresh->value_stride_h) * esz) % 4 == 0,
                "%s: key / value rows must be 4-byte aligned", op);
    a.k_new = fresh->key;
    a.v_new = fresh->value;
    a.kn_stride_t = fresh->key_stride_t;
    a.kn_stride_h = fresh->key_stride_h;
    a.vn_stride_t = fresh->value_stride_t;
    a.vn_stride_h = fresh->value_stride_h;
    a.new_dtype = fresh->dtype;
    a.new_eps = fresh->eps;
    a.new_slots = fresh->slot_mapping;
  }
  hipStream_t s = as_stream(stream);
  int rc = KVQ_OK;
  // a batch that the caller knows to hold no one-row sequence has nothing for the decode kernel and its reduce
  if (!(no_decode_rows && max_query_len > 1)) rc = launch_decode_streamk(a, q_dtype, out_dtype, s);
  if (rc) return rc;
  if (max_query_len > 1) {
    // the list of the sequences that have a query run sits behind the decode kernels' notes in the workspace
    int32_t* plan = reinterpret_cast<int32_t*>(a.seq_first_unit + num_seqs);
    // (the batch-invariant mode keeps one cut of the context whatever the caller proposes for this launch)
    rc = launch_prefill(a.io, seq_lens, cu_seqlens_q, num_seqs, max_query_len, causal, q_dtype, out_dtype, plan, s,
                        batch_invariant() ? 1 : prefill_splits,
                        reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + part_at));
  }
  return rc;
}

}  // namespace kvq

extern "C" int kvq_paged_attn_int8(void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h,
                                   const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                                   const void* cache, const kvq_cache_geom* geom, const int32_t* block_table,
                                   int64_t bt_stride, const int32_t* seq_lens, const int32_t* cu_seqlens_q,
                                   int num_seqs, int num_q_heads, int max_query_len, float scale, int causal,
                                   int window_size, float softcap, const float* sinks, const float* alibi_slopes, float* lse, void* workspace,
                                   size_t workspace_bytes, kvq_stream_t stream) {
  return kvq::paged_attn_launch("paged_attn_int8", out, out_dtype, out_stride_t, out_stride_h, q, q_dtype, q_stride_t,
                                q_stride_h, cache, geom, block_table, bt_stride, seq_lens, cu_seqlens_q, num_seqs,
                                num_q_heads, max_query_len, scale, causal, window_size, softcap, sinks, alibi_slopes, lse, workspace,
                                workspace_bytes, "workspace", stream);
}

extern "C" size_t kvq_paged_attn_split_prefill_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size,
                                                              int num_tokens, int prefill_splits) {
  if (max_num_seqs <= 0 || num_q_heads <= 0 || head_size <= 0) return 0;
  const size_t base = kvq::streamk_workspace_bytes(max_num_seqs, num_q_heads, head_size, kvq::num_cus());
  if (prefill_splits <= 1 || num_tokens <= 0) return base;
  return kvq::split_part_offset(base) + kvq::split_part_bytes(num_tokens, num_q_heads, head_size, prefill_splits);
}

extern "C" int kvq_paged_attn_int8_split_prefill(void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h,
                                                 const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                                                 const void* cache, const kvq_cache_geom* geom,
                                                 const int32_t* block_table, int64_t bt_stride,
                                                 const int32_t* seq_lens, const int32_t* cu_seqlens_q, int num_seqs,
                                                 int num_q_heads, int max_query_len, float scale, int causal,
                                                 int window_size, float softcap, const float* sinks,
                                                 const float* alibi_slopes, float* lse, int num_tokens,
                                                 int prefill_splits, void* workspace, size_t workspace_bytes,
                                                 kvq_stream_t stream) {
  return kvq::paged_attn_launch("paged_attn_int8_split_prefill", out, out_dtype, out_stride_t, out_stride_h, q, q_dtype,
                                q_stride_t, q_stride_h, cache, geom, block_table, bt_stride, seq_lens, cu_seqlens_q,
                                num_seqs, num_q_heads, max_query_len, scale, causal, window_size, softcap, sinks,
                                alibi_slopes, lse, workspace, workspace_bytes, "workspace", stream, nullptr,
                                prefill_splits, num_tokens);
}

extern "C" int kvq_paged_attn_int8_fused_write(void* out, int out_dtype, int64_t out_stride_t, int64_t out_stride_h,
                                               const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                                               const void* key, const void* value, int src_dtype,
                                               int64_t key_stride_t, int64_t key_stride_h, int64_t value_stride_t,
                                               int64_t value_stride_h, float eps, void* cache,
                                               const kvq_cache_geom* geom, const int32_t* block_table,
                                               int64_t bt_stride, const int32_t* seq_lens,
                                               const int64_t* slot_mapping, int num_seqs,
                                               int num_q_heads, float scale, int window_size, float softcap,
                                               const float* sinks, const float* alibi_slopes, float* lse, void* workspace, size_t workspace_bytes,
                                               kvq_stream_t stream) {
  const kvq::NewTokens fresh{key, value, src_dtype, key_stride_t, key_stride_h, value_stride_t, value_stride_h, eps,
                             slot_mapping};
  return kvq::paged_attn_launch("paged_attn_int8_fused_write", out, out_dtype, out_stride_t, out_stride_h, q, q_dtype,
                                q_stride_t, q_stride_h, cache, geom, block_table, bt_stride, seq_lens, nullptr, num_seqs,
                                num_q_heads, 1, scale, 1, window_size, softcap, sinks, alibi_slopes, lse, workspace, workspace_bytes,
                                "workspace", stream, &fresh);
}

// Also the set-up hook: resolves the array's address on the current device, so that a first call of the
// entry point below inside a stream capture finds it resolved and makes no runtime query there.
extern "C" size_t kvq_paged_attn_static_scratch_bytes(void) {
  kvq::DeviceSymbols sym;
  (void)kvq::device_symbols("paged_attn_static_scratch_bytes", &sym);  // without a device: the size alone
  return KVQ_STATIC_SCRATCH_BYTES;
}

extern "C" int kvq_paged_attn_int8_static_scratch(void* out, int out_dtype, int64_t out_stride_t,
                                                  int64_t out_stride_h, const void* q, int q_dtype,
                                                  int64_t q_stride_t, int64_t q_stride_h, const void* cache,
                                                  const kvq_cache_geom* geom, const int32_t* block_table,
                                                  int64_t bt_stride, const int32_t* seq_lens,
                                                  const int32_t* cu_seqlens_q, int num_seqs, int num_q_heads,
                                                  int max_query_len, float scale, int causal, int window_size,
                                                  float softcap, const float* sinks, const float* alibi_slopes, float* lse,
                                                  kvq_stream_t stream) {
  const char* op = "paged_attn_int8_static_scratch";
  kvq::DeviceSymbols sym;
  const int rc = kvq::device_symbols(op, &sym);
  if (rc) return rc;
  void* ptr = sym.scratch;
  // The split-K partial states need no clearing: every slot the reduce reads was written by this
  // launch's main kernel first (slots it does not own are masked out bit-wise, whatever they hold).
  return kvq::paged_attn_launch(op, out, out_dtype, out_stride_t, out_stride_h, q, q_dtype, q_stride_t, q_stride_h,
                                cache, geom, block_table, bt_stride, seq_lens, cu_seqlens_q, num_seqs, num_q_heads,
                                max_query_len, scale, causal, window_size, softcap, sinks, alibi_slopes, lse, ptr,
                                KVQ_STATIC_SCRATCH_BYTES,
                                "batch too large for the built-in scratch: split-K state", stream);
}
