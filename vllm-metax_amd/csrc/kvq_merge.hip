// LSE merge of two partial attention states (gfx950).
//
// out = (p_out * e^{p_lse} + s_out * e^{s_lse}) / (e^{p_lse} + e^{s_lse}), computed relative to
// max(p_lse, s_lse).  One thread owns one 16-byte pack of one (token, head) row, so the three
// tensors stream through once with 128-bit accesses; the two lse values of a row are read by
// every thread of the row (they sit in cache).  +inf lse counts as -inf; when both are -inf the
// prefix row is emitted unchanged; rows at or beyond prefix_num_tokens copy the suffix.
#include "kvq_internal.h"

namespace kvq {

template <int DT>
struct Pack;
template <>
struct Pack<KVQ_F32> {
  static constexpr int N = 4;
  __device__ static void unpack(u32x4 v, float (&f)[4]) {
    f[0] = as_f32(v.x);
    f[1] = as_f32(v.y);
    f[2] = as_f32(v.z);
    f[3] = as_f32(v.w);
  }
  __device__ static u32x4 pack(const float (&f)[4]) {
    return (u32x4){as_u32(f[0]), as_u32(f[1]), as_u32(f[2]), as_u32(f[3])};
  }
};
template <>
struct Pack<KVQ_BF16> {
  static constexpr int N = 8;
  __device__ static void unpack(u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = as_f32(v[i] << 16);
      f[2 * i + 1] = as_f32(v[i] & 0xffff0000u);
    }
  }
  __device__ static u32x4 pack(const float (&f)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (uint32_t)f32_to_bf16_bits(f[2 * i]) | ((uint32_t)f32_to_bf16_bits(f[2 * i + 1]) << 16);
    return v;
  }
};
template <>
struct Pack<KVQ_F16> {
  static constexpr int N = 8;
  __device__ static void unpack(u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t e = v[i];  // copy the element out first: bit_cast must not see a vector element lvalue
      const half2_t h = __builtin_bit_cast(half2_t, e);
      f[2 * i] = (float)h.x;
      f[2 * i + 1] = (float)h.y;
    }
  }
  __device__ static u32x4 pack(const float (&f)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const half2_t h = {(half_t)f[2 * i], (half_t)f[2 * i + 1]};
      v[i] = __builtin_bit_cast(uint32_t, h);
    }
    return v;
  }
};

template <int DT>
__global__ __launch_bounds__(256) void merge_attn_states_kernel(
    u32x4* __restrict__ output, float* __restrict__ output_lse, const u32x4* __restrict__ prefix_output,
    const float* __restrict__ prefix_lse, const u32x4* __restrict__ suffix_output,
    const float* __restrict__ suffix_lse, int64_t num_tokens, int num_heads, int packs_per_row,
    int64_t prefix_num_tokens) {
  using P = Pack<DT>;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = num_tokens * num_heads * packs_per_row;
  if (idx >= total) return;
  const int pack = (int)(idx % packs_per_row);
  const int64_t th = idx / packs_per_row;
  const int head = (int)(th % num_heads);
  const int64_t tok = th / num_heads;
  const int64_t li = (int64_t)head * num_tokens + tok;
  if (tok >= prefix_num_tokens) {
    output[idx] = suffix_output[idx];
    if (output_lse != nullptr && pack == 0) output_lse[li] = suffix_lse[li];
    return;
  }
  float pl = prefix_lse[li], sl = suffix_lse[li];
  pl = __builtin_isinf(pl) ? -INFINITY : pl;
  sl = __builtin_isinf(sl) ? -INFINITY : sl;
  const float mx = fmaxf(pl, sl);
  if (__builtin_isinf(mx)) {  // nothing attended on either side: emit the prefix row
    output[idx] = prefix_output[idx];
    if (output_lse != nullptr && pack == 0) output_lse[li] = mx;
    return;
  }
  const float pe = __expf(pl - mx), se = __expf(sl - mx);
  const float tot = pe + se;
  const float pw = pe / tot, sw = se / tot;
  float a[P::N], b[P::N];
  P::unpack(prefix_output[idx], a);
  P::unpack(suffix_output[idx], b);
#pragma unroll
  for (int i = 0; i < P::N; ++i) a[i] = a[i] * pw + b[i] * sw;
  output[idx] = P::pack(a);
  if (output_lse != nullptr && pack == 0) output_lse[li] = __logf(tot) + mx;
}

}  // namespace kvq

extern "C" int kvq_merge_attn_states(void* output, float* output_lse, const void* prefix_output,
                                     const float* prefix_lse, const void* suffix_output,
                                     const float* suffix_lse, int dtype, int64_t num_tokens, int num_heads,
                                     int head_size, int64_t prefix_num_tokens, kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "merge_attn_states";
  KVQ_REQUIRE(num_tokens >= 0 && num_heads > 0 && head_size > 0, "%s: bad sizes", op);
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(output && prefix_output && prefix_lse && suffix_output && suffix_lse, "%s: NULL pointer", op);
  const int esz = dtype == KVQ_F32 ? 4 : 2;
  KVQ_REQUIRE(dtype == KVQ_F32 || dtype == KVQ_BF16 || dtype == KVQ_F16, "%s: unknown dtype %d", op, dtype);
  KVQ_REQUIRE((head_size * esz) % 16 == 0, "%s: head_size %d must fill whole 16-byte packs", op, head_size);
  KVQ_REQUIRE(((uintptr_t)output | (uintptr_t)prefix_output | (uintptr_t)suffix_output) % 16 == 0,
              "%s: outputs must be 16-byte aligned", op);
  const int packs = head_size * esz / 16;
  const int64_t total = num_tokens * num_heads * packs;
  const int64_t blocks = (total + 255) / 256;
  KVQ_REQUIRE(blocks <= 0x7fffffffLL, "%s: too many elements", op);
  hipStream_t s = as_stream(stream);
#define KVQ_MERGE(T)                                                                                          \
  hipLaunchKernelGGL((merge_attn_states_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s,                  \
                     static_cast<u32x4*>(output), output_lse, static_cast<const u32x4*>(prefix_output),      \
                     prefix_lse, static_cast<const u32x4*>(suffix_output), suffix_lse, num_tokens, num_heads, \
                     packs, prefix_num_tokens)
  switch (dtype) {
    case KVQ_F32: KVQ_MERGE(KVQ_F32); break;
    case KVQ_BF16: KVQ_MERGE(KVQ_BF16); break;
    default: KVQ_MERGE(KVQ_F16); break;
  }
#undef KVQ_MERGE
  return check_hip(hipGetLastError(), "merge_attn_states launch");
}
