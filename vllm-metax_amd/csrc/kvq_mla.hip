// MLA latent cache, int8 codes with one fp32 scale per token: quantise-on-write (gfx950).
//
// One wavefront owns one token: the kv_c row (kv_lora_rank wide) and the k_pe row (rope_dim
// wide) are read once with lane-strided coalesced loads, their joint absmax is reduced across
// the 64 lanes, and the concatenated row is written as int8 codes into the block's row region,
// the scale into the block's scale region.  Same arithmetic as the per-(token, head) writer:
// scale = max(absmax, eps) / 127 (IEEE division), code = clamp(rint(x / scale), -128, 127).
#include "kvq_internal.h"

namespace kvq {

template <int DT>
__global__ __launch_bounds__(256) void mla_quant_write_kernel(const void* __restrict__ kv_c,
                                                              const void* __restrict__ k_pe, int64_t kv_c_stride,
                                                              int64_t k_pe_stride, uint8_t* __restrict__ cache,
                                                              kvq_mla_geom g, const int64_t* __restrict__ slot_mapping,
                                                              int64_t num_tokens, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t t = (int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
  if (t >= num_tokens) return;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;  // padding token
  const int64_t blk = slot / g.block_size;
  const int64_t off = slot - blk * g.block_size;
  const int R = g.kv_lora_rank, W = g.kv_lora_rank + g.rope_dim;
  constexpr int kMaxPerLane = 16;  // rows up to 1024 wide stay in registers
  float x[kMaxPerLane];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + kWave * i;
    x[i] = 0.f;
    if (d < W) x[i] = d < R ? load_act<DT>(kv_c, t * kv_c_stride + d) : load_act<DT>(k_pe, t * k_pe_stride + (d - R));
    amax = fmaxf(amax, fabsf(x[i]));
  }
  amax = fmaxf(wave_max(amax), eps);
  const float scale = amax / 127.0f;
  int8_t* row = reinterpret_cast<int8_t*>(cache + blk * g.stride_block + off * g.stride_row);
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + kWave * i;
    if (d < W) {
      float r = scale > 0.f ? rintf(x[i] / scale) : 0.f;
      r = fminf(fmaxf(r, -128.f), 127.f);
      row[d] = (int8_t)(int)r;
    }
  }
  if (lane == 0) *reinterpret_cast<float*>(cache + blk * g.stride_block + g.scale_off + off * 4) = scale;
}

// Gather + dequantise latent rows into a dense [num_tokens, W] workspace (the chunked-context
// prefill reads its cached context this way).  One wavefront per destination row: lanes 0 .. W/16-1
// load 16 codes each (one coalesced run of W bytes), every lane reads the row's scale, and the 16
// products code * scale go out as one or two 16-byte stores per lane.
template <int DT>
__global__ __launch_bounds__(256) void mla_gather_dequant_kernel(void* __restrict__ dst, int64_t dst_stride,
                                                                 const uint8_t* __restrict__ cache, kvq_mla_geom g,
                                                                 const int32_t* __restrict__ block_table,
                                                                 int64_t bt_stride,
                                                                 const int32_t* __restrict__ cu_seq_lens,
                                                                 const int32_t* __restrict__ token_to_seq,
                                                                 const int32_t* __restrict__ seq_starts,
                                                                 int num_tokens) {
  const int lane = threadIdx.x & (kWave - 1);
  const int W = g.kv_lora_rank + g.rope_dim;
  for (int64_t t = (int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave); t < num_tokens;
       t += (int64_t)gridDim.x * (blockDim.x / kWave)) {
    const int b = token_to_seq[t];
    if (t >= cu_seq_lens[b + 1]) continue;
    int pos = (int)t - cu_seq_lens[b];
    if (seq_starts != nullptr) pos += seq_starts[b];
    const int e = pos / g.block_size;
    const int off = pos - e * g.block_size;
    const int64_t blk = block_table[(int64_t)b * bt_stride + e];
    const uint8_t* base = cache + blk * g.stride_block;
    const float scale = *reinterpret_cast<const float*>(base + g.scale_off + (int64_t)off * 4);
    if (lane * 16 >= W) continue;
    const u32x4 w = *reinterpret_cast<const u32x4_a4*>(base + (int64_t)off * g.stride_row + lane * 16);
    float f[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t x = w[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) f[4 * i + j] = (float)(int8_t)(x >> (8 * j)) * scale;
    }
    const int64_t at = t * dst_stride + lane * 16;
#pragma unroll
    for (int i = 0; i < 16; ++i) store_act<DT>(dst, at + i, f[i]);
  }
}

// Gather without dequantisation: row t of dst = the W code bytes of its token followed by the token's
// 4 scale bytes (W + 4 bytes, the token-major form of the cache for copies and transfers).  One
// wavefront per token finds its sequence by bisection over cu_seq_lens (uniform, scalar loads).
__global__ __launch_bounds__(256) void mla_cp_gather_kernel(uint8_t* __restrict__ dst, int64_t dst_stride,
                                                            const uint8_t* __restrict__ cache, kvq_mla_geom g,
                                                            const int32_t* __restrict__ block_table, int64_t bt_stride,
                                                            const int32_t* __restrict__ cu_seq_lens,
                                                            const int32_t* __restrict__ seq_starts, int batch,
                                                            int num_tokens) {
  const int lane = threadIdx.x & (kWave - 1);
  const int W = g.kv_lora_rank + g.rope_dim;
  for (int64_t t = (int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave); t < num_tokens;
       t += (int64_t)gridDim.x * (blockDim.x / kWave)) {
    int lo = 0, hi = batch - 1;  // the last sequence whose first row is <= t
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_seq_lens[mid] <= t) lo = mid;
      else hi = mid - 1;
    }
    const int b = lo;
    if (t >= cu_seq_lens[b + 1]) continue;  // rows past the last sequence stay untouched
    int pos = (int)t - cu_seq_lens[b];
    if (seq_starts != nullptr) pos += seq_starts[b];
    const int e = pos / g.block_size;
    const int off = pos - e * g.block_size;
    const int64_t blk = block_table[(int64_t)b * bt_stride + e];
    const uint8_t* base = cache + blk * g.stride_block;
    uint8_t* out = dst + t * dst_stride;
    if (lane * 16 < W) {
      const u32x4 w = *reinterpret_cast<const u32x4_a4*>(base + (int64_t)off * g.stride_row + lane * 16);
      *reinterpret_cast<u32x4_a4*>(out + lane * 16) = w;
    } else if (lane * 16 == ((W + 15) & ~15)) {  // the first idle lane carries the scale
      *reinterpret_cast<uint32_t*>(out + W) = *reinterpret_cast<const uint32_t*>(base + g.scale_off + (int64_t)off * 4);
    }
  }
}

}  // namespace kvq

extern "C" int kvq_cp_gather_mla_int8(void* dst, int64_t dst_stride, const void* cache, const kvq_mla_geom* geom,
                                      const int32_t* block_table, int64_t bt_stride, const int32_t* cu_seq_lens,
                                      const int32_t* seq_starts, int batch_size, int64_t num_tokens,
                                      kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "cp_gather_mla_int8";
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(num_tokens >= 0 && num_tokens <= 0x7fffffffLL, "%s: num_tokens out of range", op);
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(dst && cache && block_table && cu_seq_lens, "%s: NULL pointer", op);
  KVQ_REQUIRE(batch_size > 0, "%s: batch_size must be positive", op);
  const kvq_mla_geom& g = *geom;
  const int W = g.kv_lora_rank + g.rope_dim;
  KVQ_REQUIRE(g.kv_lora_rank > 0 && g.rope_dim >= 0 && g.block_size > 0 && W % 16 == 0 && W <= 1008,
              "%s: rows must be a multiple of 16 bytes and at most 1008 wide (got %d)", op, W);
  KVQ_REQUIRE((g.stride_block | g.stride_row | g.scale_off) % 4 == 0 && ((uintptr_t)cache % 4) == 0,
              "%s: cache strides must be 4-byte aligned", op);
  KVQ_REQUIRE(dst_stride >= W + 4 && dst_stride % 4 == 0 && ((uintptr_t)dst % 4) == 0,
              "%s: dst rows must be 4-byte aligned and at least %d bytes apart", op, W + 4);
  const int64_t want = (num_tokens + 3) / 4;
  const unsigned blocks = (unsigned)(want < 65536 ? want : 65536);
  hipLaunchKernelGGL(mla_cp_gather_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), static_cast<uint8_t*>(dst),
                     dst_stride, static_cast<const uint8_t*>(cache), g, block_table, bt_stride, cu_seq_lens, seq_starts,
                     batch_size, (int)num_tokens);
  return check_hip(hipGetLastError(), "cp_gather_mla_int8 launch");
}

extern "C" int kvq_gather_and_dequant_mla_int8(void* dst, int dst_dtype, int64_t dst_stride, const void* cache,
                                               const kvq_mla_geom* geom, const int32_t* block_table,
                                               int64_t bt_stride, const int32_t* cu_seq_lens,
                                               const int32_t* token_to_seq, const int32_t* seq_starts,
                                               int64_t num_tokens, kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "gather_and_dequant_mla_int8";
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(num_tokens >= 0 && num_tokens <= 0x7fffffffLL, "%s: num_tokens out of range", op);
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(dst && cache && block_table && cu_seq_lens && token_to_seq, "%s: NULL pointer", op);
  const kvq_mla_geom& g = *geom;
  const int W = g.kv_lora_rank + g.rope_dim;
  KVQ_REQUIRE(g.kv_lora_rank > 0 && g.rope_dim >= 0 && g.block_size > 0, "%s: bad geometry", op);
  KVQ_REQUIRE(W % 16 == 0 && W <= 1024, "%s: row width %d must be a multiple of 16, at most 1024", op, W);
  KVQ_REQUIRE((g.stride_block | g.stride_row | g.scale_off) % 4 == 0 && ((uintptr_t)cache % 4) == 0,
              "%s: cache strides must be 4-byte aligned", op);
  KVQ_REQUIRE(dst_stride >= W, "%s: dst rows overlap", op);
  hipStream_t s = as_stream(stream);
  const int64_t want = (num_tokens + 3) / 4;
  const unsigned blocks = (unsigned)(want < 65536 ? want : 65536);
#define KVQ_MLAG(T)                                                                                      \
  hipLaunchKernelGGL((mla_gather_dequant_kernel<T>), dim3(blocks), dim3(256), 0, s, dst, dst_stride,  \
                     static_cast<const uint8_t*>(cache), g, block_table, bt_stride, cu_seq_lens,       \
                     token_to_seq, seq_starts, (int)num_tokens)
  switch (dst_dtype) {
    case KVQ_F32: KVQ_MLAG(KVQ_F32); break;
    case KVQ_BF16: KVQ_MLAG(KVQ_BF16); break;
    case KVQ_F16: KVQ_MLAG(KVQ_F16); break;
    default: return fail(KVQ_EINVAL, "%s: unknown dst_dtype %d", op, dst_dtype);
  }
#undef KVQ_MLAG
  return check_hip(hipGetLastError(), "gather_and_dequant_mla_int8 launch");
}

extern "C" int kvq_concat_and_cache_mla_int8(const void* kv_c, const void* k_pe, int src_dtype,
                                             int64_t kv_c_stride, int64_t k_pe_stride, void* cache,
                                             const kvq_mla_geom* geom, const int64_t* slot_mapping,
                                             int64_t num_tokens, float eps, kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "concat_and_cache_mla_int8";
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(num_tokens >= 0, "%s: negative num_tokens", op);
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(kv_c && k_pe && cache && slot_mapping, "%s: NULL pointer", op);
  const kvq_mla_geom& g = *geom;
  KVQ_REQUIRE(g.kv_lora_rank > 0 && g.rope_dim >= 0 && g.block_size > 0, "%s: bad geometry", op);
  KVQ_REQUIRE(g.kv_lora_rank + g.rope_dim <= 1024, "%s: rows wider than 1024 are not supported", op);
  KVQ_REQUIRE((g.stride_block | g.scale_off) % 4 == 0 && ((uintptr_t)cache % 4) == 0,
              "%s: block stride / scale offset must be 4-byte aligned", op);
  KVQ_REQUIRE(eps >= 0.f, "%s: eps must not be negative", op);
  const int64_t blocks = (num_tokens + 3) / 4;
  KVQ_REQUIRE(blocks <= 0x7fffffffLL, "%s: too many tokens", op);
  hipStream_t s = as_stream(stream);
  uint8_t* c = static_cast<uint8_t*>(cache);
#define KVQ_MLAW(T)                                                                                       \
  hipLaunchKernelGGL((mla_quant_write_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, kv_c, k_pe, \
                     kv_c_stride, k_pe_stride, c, g, slot_mapping, num_tokens, eps)
  switch (src_dtype) {
    case KVQ_F32: KVQ_MLAW(KVQ_F32); break;
    case KVQ_BF16: KVQ_MLAW(KVQ_BF16); break;
    case KVQ_F16: KVQ_MLAW(KVQ_F16); break;
    default: return fail(KVQ_EINVAL, "%s: unknown src_dtype %d", op, src_dtype);
  }
#undef KVQ_MLAW
  return check_hip(hipGetLastError(), "concat_and_cache_mla_int8 launch");
}
