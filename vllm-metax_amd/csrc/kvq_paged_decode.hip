// Paged decode attention over the int8 cache: work decomposition and reduce (gfx950).
//
// Balanced split-K ("stream-K" over tokens): the 32-token tiles of all decode
// sequences form one global work line (one unit per tile, plus a small charge per
// sequence start); the launch has exactly as many workgroups as the device keeps
// resident and workgroup w takes units [w*T/P, (w+1)*T/P), whatever sequence
// boundaries fall inside.  A workgroup is one wave per KV head, so a block's
// bytes are read by one CU at the same time and each byte leaves HBM once.  A run of
// tiles that covers a whole sequence writes the output row directly; otherwise it
// stores an fp32 partial state (o, m, l) in slot w + seq (unique along the staircase of
// (workgroup, sequence) pairs) and the reduce kernel merges the slots of a sequence
// with the log-sum-exp algebra.  Nothing is synchronised on the host and nothing is
// allocated: the partials live in the caller's workspace.
//
// The fixed-partition entry point (512-token partitions, locally normalised partials)
// reuses the same tile code with the reference's (partition, sequence) grid.
#include "kvq_paged_decode_impl.cuh"

namespace kvq {

extern template int launch_streamk_q<64>(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s);
extern template int launch_streamk_q<128>(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s);
extern template int launch_streamk_q<256>(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s);
extern template int launch_v2_q<64>(const V2Args& a, int num_seqs, int q_dtype, hipStream_t s);
extern template int launch_v2_q<128>(const V2Args& a, int num_seqs, int q_dtype, hipStream_t s);
extern template int launch_v2_q<256>(const V2Args& a, int num_seqs, int q_dtype, hipStream_t s);

// out = sum_j w_j tmp_out_j / sum_j w_j, w_j = exp_sums_j * exp(max_logits_j - max).
// grid (num_seqs, ceil(Hq/4)), one wave per q head.
template <int ODT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(void* out, float* lse, const float* exp_sums,
                                                            const float* max_logits, const float* tmp_out,
                                                            const int32_t* seq_lens, int num_q_heads, int D,
                                                            int partition_size, int max_parts) {
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int seq = blockIdx.x;
  if (head >= num_q_heads) return;
  const int len = seq_lens[seq];
  int parts = len > 0 ? (len + partition_size - 1) / partition_size : 0;
  parts = parts < max_parts ? parts : max_parts;
  const int64_t base = ((int64_t)seq * num_q_heads + head) * max_parts;
  const int64_t obase = ((int64_t)seq * num_q_heads + head) * D;
  if (parts == 0) {
    for (int d = lane; d < D; d += kWave) store_act<ODT>(out, obase + d, 0.f);
    if (lse != nullptr && lane == 0) lse[(int64_t)seq * num_q_heads + head] = -INFINITY;
    return;
  }
  float m = -INFINITY;
  for (int j = lane; j < parts; j += kWave) m = fmaxf(m, max_logits[base + j]);
  m = wave_max(m);
  float denom = 0.f;
  for (int j = lane; j < parts; j += kWave) denom += exp_sums[base + j] * __expf(max_logits[base + j] - m);
  denom = wave_sum(denom);
  const float inv = 1.0f / denom;
  for (int d = lane; d < D; d += kWave) {
    float acc = 0.f;
    for (int j = 0; j < parts; ++j)
      acc += tmp_out[(base + j) * D + d] * (exp_sums[base + j] * __expf(max_logits[base + j] - m));
    store_act<ODT>(out, obase + d, acc * inv);
  }
  if (lse != nullptr && lane == 0) lse[(int64_t)seq * num_q_heads + head] = m + __logf(denom);
}

// ---- host side ---------------------------------------------------------------------------

// kv heads a decode workgroup serves: the largest power of two <= min(8, num_kv_heads).
int heads_per_wg(int num_kv_heads) {
  if (num_kv_heads >= 8) return 8;
  if (num_kv_heads >= 4) return 4;
  if (num_kv_heads >= 2) return 2;
  return 1;
}

// Resident workgroups the stream-K launch uses: one eight-wave workgroup per compute unit.
static int streamk_num_wg(int) { return num_cus(); }

int validate_common(const char* op, const void* q, const void* cache, const kvq_cache_geom* geom,
                           const int32_t* block_table, const int32_t* seq_lens, int num_seqs, int num_q_heads) {
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(q && cache && block_table && seq_lens, "%s: NULL pointer", op);
  KVQ_REQUIRE(num_seqs > 0 && num_q_heads > 0, "%s: num_seqs and num_q_heads must be positive", op);
  const kvq_cache_geom& g = *geom;
  KVQ_REQUIRE(g.num_kv_heads > 0 && num_q_heads % g.num_kv_heads == 0,
              "%s: num_q_heads %d is not a multiple of num_kv_heads %d", op, num_q_heads, g.num_kv_heads);
  KVQ_REQUIRE(num_q_heads / g.num_kv_heads <= 16, "%s: more than 16 q heads per kv head is not supported", op);
  KVQ_REQUIRE(g.head_size == 64 || g.head_size == 128 || g.head_size == 256,
              "%s: head_size %d not supported (64, 128, 256)", op, g.head_size);
  KVQ_REQUIRE(g.block_size > 0 && g.block_size % 16 == 0, "%s: block_size %d must be a multiple of 16", op,
              g.block_size);
  KVQ_REQUIRE((g.k_off | g.v_off | g.ks_off | g.vs_off | g.stride_block | g.stride_slot | g.stride_head) % 4 == 0 &&
                  ((uintptr_t)cache % 4) == 0,
              "%s: cache offsets/strides must be 4-byte aligned", op);
  KVQ_REQUIRE(g.code_type == KVQ_CODE_INT8 || g.code_type == KVQ_CODE_FP8_E4M3 || g.code_type == KVQ_CODE_INT4,
              "%s: unknown code_type %d", op, g.code_type);
  const int cb = code_bytes(g);
  KVQ_REQUIRE(g.ks_off - g.k_off == cb && g.v_off - g.k_off == cb + 4 && g.vs_off - g.k_off == 2 * cb + 4,
              "%s: a cache record must be [K codes | K scale | V codes | V scale]", op);
  KVQ_REQUIRE(g.stride_slot > 0 && g.stride_slot <= 0x7fffffff / 64, "%s: stride_slot out of range", op);
  // the kernels multiply block numbers and slots by these as 32-bit numbers
  KVQ_REQUIRE(g.stride_block > 0 && g.stride_block <= 0x7fffffff && g.stride_head >= 0 && g.stride_head <= 0x7fffffff &&
                  (int64_t)g.block_size * g.stride_slot <= 0x7fffffff,
              "%s: a cache block of 2 GiB or more is not supported", op);
  return KVQ_OK;
}

int launch_decode_streamk(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s) {
  switch (a.io.g.head_size) {
    case 64: return launch_streamk_q<64>(a, q_dtype, out_dtype, s);
    case 128: return launch_streamk_q<128>(a, q_dtype, out_dtype, s);
    case 256: return launch_streamk_q<256>(a, q_dtype, out_dtype, s);
  }
  return fail(KVQ_EINVAL, "paged_attn_int8: head_size %d not supported", a.io.g.head_size);
}

static int launch_reduce(void* out, int out_dtype, float* lse, const float* exp_sums, const float* max_logits,
                         const float* tmp_out, const int32_t* seq_lens, int num_seqs, int num_q_heads, int D,
                         int partition_size, int max_parts, hipStream_t s) {
  dim3 grid(num_seqs, (num_q_heads + 3) / 4);
#define KVQ_RED(T)                                                                                        \
  hipLaunchKernelGGL((splitk_reduce_kernel<T>), grid, dim3(256), 0, s, out, lse, exp_sums, max_logits, \
                     tmp_out, seq_lens, num_q_heads, D, partition_size, max_parts)
  switch (out_dtype) {
    case KVQ_F32: KVQ_RED(KVQ_F32); break;
    case KVQ_BF16: KVQ_RED(KVQ_BF16); break;
    case KVQ_F16: KVQ_RED(KVQ_F16); break;
    default: return fail(KVQ_EINVAL, "splitk_reduce: unknown out_dtype %d", out_dtype);
  }
#undef KVQ_RED
  return check_hip(hipGetLastError(), "splitk_reduce launch");
}

// Slots of partial states a launch may fill: one per (workgroup, sequence) step of the balanced cutting's staircase,
// or kFixedSpans per sequence with the batch-invariant cutting.
size_t streamk_slots(int max_num_seqs, int num_wg) {
  const size_t stair = (size_t)num_wg + (size_t)max_num_seqs;
  const size_t fixed = (size_t)kFixedSpans * (size_t)max_num_seqs;
  return batch_invariant() && fixed > stair ? fixed : stair;
}

// Workspace layout of the stream-K partials.
size_t streamk_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size, int num_wg) {
  const size_t slots = streamk_slots(max_num_seqs, num_wg);
  return slots * (size_t)num_q_heads * ((size_t)head_size + 2) * sizeof(float) +
         (2 * (size_t)num_wg + 2 + (size_t)max_num_seqs) * sizeof(int64_t) +   // where the shares and the sequences begin
         ((size_t)max_num_seqs + 2) / 2 * 2 * sizeof(int32_t);                  // the prefill kernels' list of sequences
}

int decode_streamk_num_wg(int num_kv_heads) { return streamk_num_wg(num_kv_heads); }

}  // namespace kvq

extern "C" {

size_t kvq_paged_attn_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size) {
  if (max_num_seqs <= 0 || num_q_heads <= 0 || head_size <= 0) return 0;
  return kvq::streamk_workspace_bytes(max_num_seqs, num_q_heads, head_size, kvq::num_cus());
}

int kvq_paged_attn_v2_int8(void* out, int out_dtype, float* exp_sums, float* max_logits, float* tmp_out,
                           const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                           const void* cache, const kvq_cache_geom* geom, const int32_t* block_table,
                           int64_t bt_stride, const int32_t* seq_lens, int num_seqs, int num_q_heads,
                           float scale, const float* alibi_slopes, int partition_size, int max_num_partitions,
                           kvq_stream_t stream) {
  using namespace kvq;
  int rc = validate_common("paged_attn_v2_int8", q, cache, geom, block_table, seq_lens, num_seqs, num_q_heads);
  if (rc) return rc;
  KVQ_REQUIRE(out && exp_sums && max_logits && tmp_out, "paged_attn_v2_int8: NULL output pointer");
  KVQ_REQUIRE(geom->code_type == KVQ_CODE_INT8, "paged_attn_v2_int8: int8 codes only");
  KVQ_REQUIRE(partition_size > 0 && partition_size % kTile == 0,
              "paged_attn_v2_int8: partition_size %d must be a positive multiple of %d", partition_size, kTile);
  KVQ_REQUIRE(max_num_partitions > 0 && max_num_partitions <= 65535,
              "paged_attn_v2_int8: max_num_partitions %d out of range", max_num_partitions);
  KVQ_REQUIRE(num_seqs <= 65535, "paged_attn_v2_int8: at most 65535 sequences");
  V2Args a{};
  a.io.q = q;
  a.io.q_stride_t = q_stride_t;
  a.io.q_stride_h = q_stride_h;
  a.io.cache = static_cast<const uint8_t*>(cache);
  a.io.g = *geom;
  a.io.block_table = block_table;
  a.io.bt_stride = bt_stride;
  a.io.num_q_heads = num_q_heads;
  a.io.group = num_q_heads / geom->num_kv_heads;
  a.io.scale_log2 = scale * kLog2e;
  a.io.alibi = alibi_slopes;
  a.io.bs_magic = (uint32_t)((0x100000000ull + (uint64_t)geom->block_size - 1) / (uint64_t)geom->block_size);
  a.seq_lens = seq_lens;
  a.tmp_out = tmp_out;
  a.max_logits = max_logits;
  a.exp_sums = exp_sums;
  a.partition_tiles = partition_size / kTile;
  a.max_parts = max_num_partitions;
  hipStream_t s = as_stream(stream);
  switch (geom->head_size) {
    case 64: rc = launch_v2_q<64>(a, num_seqs, q_dtype, s); break;
    case 128: rc = launch_v2_q<128>(a, num_seqs, q_dtype, s); break;
    default: rc = launch_v2_q<256>(a, num_seqs, q_dtype, s); break;
  }
  if (rc) return rc;
  return launch_reduce(out, out_dtype, nullptr, exp_sums, max_logits, tmp_out, seq_lens, num_seqs, num_q_heads,
                       geom->head_size, partition_size, max_num_partitions, s);
}

int kvq_splitk_reduce(void* out, int out_dtype, float* lse, const float* exp_sums, const float* max_logits,
                      const float* tmp_out, const int32_t* seq_lens, int num_seqs, int num_q_heads,
                      int head_size, int partition_size, int max_num_partitions, kvq_stream_t stream) {
  using namespace kvq;
  KVQ_REQUIRE(out && exp_sums && max_logits && tmp_out && seq_lens, "splitk_reduce: NULL pointer");
  KVQ_REQUIRE(num_seqs > 0 && num_q_heads > 0 && head_size > 0 && partition_size > 0 && max_num_partitions > 0,
              "splitk_reduce: sizes must be positive");
  return launch_reduce(out, out_dtype, lse, exp_sums, max_logits, tmp_out, seq_lens, num_seqs, num_q_heads,
                       head_size, partition_size, max_num_partitions, as_stream(stream));
}

}  // extern "C"

