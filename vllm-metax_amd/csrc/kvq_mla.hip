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

// The same arithmetic, eight consecutive elements per lane and load (rows whose two parts are multiples of 8
// wide and 4-byte aligned; at most 1024 wide): one wave per token, lane l takes the 8-element pieces l and
// 64 + l of the row [kv_c | k_pe], 16-byte loads (two for fp32 sources) that leave before the slot is known --
// one trip to memory instead of two -- and 8-byte stores of packed codes instead of byte stores.
__global__ __launch_bounds__(256) void mla_quant_write_rows8_kernel(const void* __restrict__ kv_c,
                                                                    const void* __restrict__ k_pe, int dt,
                                                                    int64_t kv_c_stride, int64_t k_pe_stride,
                                                                    uint8_t* __restrict__ cache, kvq_mla_geom g,
                                                                    const int64_t* __restrict__ slot_mapping,
                                                                    int64_t num_tokens, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t t_raw = (int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
  const bool live = t_raw < num_tokens;
  const int64_t t = live ? t_raw : num_tokens - 1;
  const int rp = g.kv_lora_rank / 8, np = (g.kv_lora_rank + g.rope_dim) / 8;   // pieces of kv_c, of the row
  const int64_t slot = slot_mapping[t];  // in flight together with the row's loads
  MlaRowPieces r;
  mla_row_load(kv_c, k_pe, dt, t * kv_c_stride, t * k_pe_stride, rp, np, lane, r);
  const float scale = mla_row_scale(r, eps);
  if (!live || slot < 0) return;  // padding token (after the shuffles: every lane took part)
  const int64_t blk = slot / g.block_size;
  const int64_t off = slot - blk * g.block_size;
  mla_row_store(r, scale, cache + blk * g.stride_block + off * g.stride_row,
                reinterpret_cast<float*>(cache + blk * g.stride_block + g.scale_off + off * 4), lane);
}

// Rotary embedding of q_pe and k_pe (in place) fused with the quantise-on-write of the latent row
// [kv_c | rotated k_pe].  One workgroup per token: all 256 threads rotate the (head, pair) items of
// q_pe; wave 0 also rotates k_pe (one pair per lane), keeps the rotated values and quantises the
// row with them, exactly as mla_quant_write_kernel would after a separate rotation.
template <int DT, int CT, bool NEOX>
__global__ __launch_bounds__(256) void mla_rope_quant_write_kernel(
    const int64_t* __restrict__ positions, void* __restrict__ q_pe, int64_t q_stride_t, int64_t q_stride_h,
    int num_q_heads, void* __restrict__ k_pe, int64_t k_pe_stride, const void* __restrict__ kv_c, int64_t kv_c_stride,
    const void* __restrict__ cos_sin, int rot_dim, uint8_t* __restrict__ cache, kvq_mla_geom g,
    const int64_t* __restrict__ slot_mapping, float eps) {
  const int64_t t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;  // padding token: nothing is rotated, nothing is written (as the reference)
  const int64_t pos = positions[t];
  const int embed = rot_dim / 2;
  const int64_t cs = pos * rot_dim;
  // ---- q_pe: (head, pair) items over all threads
  const int nq = num_q_heads * embed;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const int head = i / embed, pair = i - head * embed;
    const float c = round_act<DT>(load_act<CT>(cos_sin, cs + pair));
    const float sn = round_act<DT>(load_act<CT>(cos_sin, cs + pair + embed));
    const int ix = NEOX ? pair : 2 * pair, iy = NEOX ? embed + pair : 2 * pair + 1;
    const int64_t base = t * q_stride_t + (int64_t)head * q_stride_h;
    float xo, yo;
    rotate_pair<DT>(load_act<DT>(q_pe, base + ix), load_act<DT>(q_pe, base + iy), c, sn, xo, yo);
    store_act<DT>(q_pe, base + ix, xo);
    store_act<DT>(q_pe, base + iy, yo);
  }
  if (threadIdx.x >= kWave) return;
  // ---- wave 0: k_pe rotation (lane = pair) and the latent row
  const int lane = threadIdx.x;
  const int R = g.kv_lora_rank;
  float kx = 0.f, ky = 0.f;
  const int ix = NEOX ? lane : 2 * lane, iy = NEOX ? embed + lane : 2 * lane + 1;
  if (lane < embed) {
    const float c = round_act<DT>(load_act<CT>(cos_sin, cs + lane));
    const float sn = round_act<DT>(load_act<CT>(cos_sin, cs + lane + embed));
    rotate_pair<DT>(load_act<DT>(k_pe, t * k_pe_stride + ix), load_act<DT>(k_pe, t * k_pe_stride + iy), c, sn, kx, ky);
    store_act<DT>(k_pe, t * k_pe_stride + ix, kx);
    store_act<DT>(k_pe, t * k_pe_stride + iy, ky);
  }
  constexpr int kMaxPerLane = 16;  // kv_lora_rank up to 1024 stays in registers
  float x[kMaxPerLane];
  float amax = fmaxf(fabsf(kx), fabsf(ky));
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + kWave * i;
    x[i] = d < R ? load_act<DT>(kv_c, t * kv_c_stride + d) : 0.f;
    amax = fmaxf(amax, fabsf(x[i]));
  }
  amax = fmaxf(wave_max(amax), eps);
  const float scale = amax / 127.0f;
  const int64_t blk = slot / g.block_size;
  const int64_t off = slot - blk * g.block_size;
  int8_t* row = reinterpret_cast<int8_t*>(cache + blk * g.stride_block + off * g.stride_row);
  auto code = [&](float v) {
    float r = scale > 0.f ? rintf(v / scale) : 0.f;
    r = fminf(fmaxf(r, -128.f), 127.f);
    return (int8_t)(int)r;
  };
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + kWave * i;
    if (d < R) row[d] = code(x[i]);
  }
  if (lane < embed) {
    row[R + ix] = code(kx);
    row[R + iy] = code(ky);
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

// q_out[t, h, :] = [ql_nope[t, h, :] | q_pe[t, h, :]], a byte move: one wave per (token, head) row, 4-byte
// pieces (the reference's kernel has the same shape, one warp per row:
// csrc/libtorch_stable/cache_kernels.cu:1769-1782).  Row lengths are in bytes.
__global__ __launch_bounds__(256) void concat_mla_q_kernel(uint8_t* out, int64_t out_st, int64_t out_sh,
                                                           const uint8_t* nope, int64_t nope_st, int64_t nope_sh,
                                                           const uint8_t* pe, int64_t pe_st, int64_t pe_sh,
                                                           int64_t rows, int num_heads, int nope_bytes, int pe_bytes) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  for (int64_t row = wave; row < rows; row += (int64_t)gridDim.x * 4) {
    const int64_t t = row / num_heads, h = row - t * num_heads;
    uint8_t* o = out + t * out_st + h * out_sh;
    const uint8_t* a = nope + t * nope_st + h * nope_sh;
    const uint8_t* b = pe + t * pe_st + h * pe_sh;
    for (int i = 4 * lane; i < nope_bytes; i += 256)
      *reinterpret_cast<uint32_t*>(o + i) = *reinterpret_cast<const uint32_t*>(a + i);
    for (int i = 4 * lane; i < pe_bytes; i += 256)
      *reinterpret_cast<uint32_t*>(o + nope_bytes + i) = *reinterpret_cast<const uint32_t*>(b + i);
  }
}

}  // namespace kvq

extern "C" int kvq_concat_mla_q(void* q_out, int64_t out_stride_t, int64_t out_stride_h, const void* ql_nope,
                                int64_t nope_stride_t, int64_t nope_stride_h, const void* q_pe,
                                int64_t pe_stride_t, int64_t pe_stride_h, int dtype, int64_t num_tokens,
                                int num_heads, int nope_dim, int rope_dim, kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "concat_mla_q";
  KVQ_REQUIRE(dtype == KVQ_F32 || dtype == KVQ_BF16 || dtype == KVQ_F16, "%s: unknown dtype %d", op, dtype);
  KVQ_REQUIRE(num_tokens >= 0 && num_heads > 0 && nope_dim > 0 && rope_dim > 0, "%s: bad sizes", op);
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(q_out && ql_nope && q_pe, "%s: NULL pointer", op);
  const int64_t es = dtype == KVQ_F32 ? 4 : 2;
  KVQ_REQUIRE((nope_dim * es) % 4 == 0 && (rope_dim * es) % 4 == 0, "%s: row parts must be whole 4-byte words", op);
  KVQ_REQUIRE(((uintptr_t)q_out | (uintptr_t)ql_nope | (uintptr_t)q_pe) % 4 == 0 &&
                  ((out_stride_t | out_stride_h | nope_stride_t | nope_stride_h | pe_stride_t | pe_stride_h) * es) % 4 == 0,
              "%s: rows must be 4-byte aligned", op);
  KVQ_REQUIRE(out_stride_h >= nope_dim + rope_dim || num_heads == 1, "%s: q_out rows overlap", op);
  const int64_t rows = num_tokens * num_heads;
  const int64_t want = (rows + 3) / 4;
  const unsigned blocks = (unsigned)(want < 65536 ? want : 65536);
  hipLaunchKernelGGL(concat_mla_q_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), static_cast<uint8_t*>(q_out),
                     out_stride_t * es, out_stride_h * es, static_cast<const uint8_t*>(ql_nope), nope_stride_t * es,
                     nope_stride_h * es, static_cast<const uint8_t*>(q_pe), pe_stride_t * es, pe_stride_h * es, rows,
                     num_heads, (int)(nope_dim * es), (int)(rope_dim * es));
  return check_hip(hipGetLastError(), "concat_mla_q launch");
}

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

namespace kvq {
template <int DT, int CT>
static void launch_rope_write(bool neox, unsigned tokens, hipStream_t s, const int64_t* positions, void* q_pe,
                              int64_t qst, int64_t qsh, int hq, void* k_pe, int64_t kps, const void* kv_c, int64_t kcs,
                              const void* cos_sin, int rot, uint8_t* cache, const kvq_mla_geom& g,
                              const int64_t* slots, float eps) {
  if (neox)
    hipLaunchKernelGGL((mla_rope_quant_write_kernel<DT, CT, true>), dim3(tokens), dim3(256), 0, s, positions, q_pe, qst,
                       qsh, hq, k_pe, kps, kv_c, kcs, cos_sin, rot, cache, g, slots, eps);
  else
    hipLaunchKernelGGL((mla_rope_quant_write_kernel<DT, CT, false>), dim3(tokens), dim3(256), 0, s, positions, q_pe, qst,
                       qsh, hq, k_pe, kps, kv_c, kcs, cos_sin, rot, cache, g, slots, eps);
}
}  // namespace kvq

extern "C" int kvq_concat_and_cache_mla_rope_int8(const int64_t* positions, void* q_pe, int64_t q_stride_t,
                                                  int64_t q_stride_h, int num_q_heads, void* k_pe,
                                                  int64_t k_pe_stride, const void* kv_c, int64_t kv_c_stride,
                                                  int dtype, const void* cos_sin_cache, int cos_sin_dtype,
                                                  int rot_dim, int is_neox, void* cache, const kvq_mla_geom* geom,
                                                  const int64_t* slot_mapping, int64_t num_tokens, float eps,
                                                  kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "concat_and_cache_mla_rope_int8";
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(num_tokens >= 0 && num_tokens <= 0x7fffffffLL, "%s: num_tokens out of range", op);
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(positions && q_pe && k_pe && kv_c && cos_sin_cache && cache && slot_mapping, "%s: NULL pointer", op);
  const kvq_mla_geom& g = *geom;
  KVQ_REQUIRE(g.kv_lora_rank > 0 && g.kv_lora_rank <= 1024 && g.block_size > 0, "%s: bad geometry", op);
  KVQ_REQUIRE(rot_dim == g.rope_dim && rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= 128,
              "%s: rot_dim %d must equal the cache's rope width %d, be even and at most 128", op, rot_dim, g.rope_dim);
  KVQ_REQUIRE(num_q_heads >= 0, "%s: negative num_q_heads", op);
  KVQ_REQUIRE((g.stride_block | g.scale_off) % 4 == 0 && ((uintptr_t)cache % 4) == 0,
              "%s: block stride / scale offset must be 4-byte aligned", op);
  KVQ_REQUIRE(eps >= 0.f, "%s: eps must not be negative", op);
  hipStream_t s = as_stream(stream);
  uint8_t* c = static_cast<uint8_t*>(cache);
  const unsigned n = (unsigned)num_tokens;
#define KVQ_ROPE(D, C)                                                                                          \
  launch_rope_write<D, C>(is_neox != 0, n, s, positions, q_pe, q_stride_t, q_stride_h, num_q_heads, k_pe,    \
                          k_pe_stride, kv_c, kv_c_stride, cos_sin_cache, rot_dim, c, g, slot_mapping, eps)
#define KVQ_ROPE_C(D)                                                              \
  switch (cos_sin_dtype) {                                                         \
    case KVQ_F32: KVQ_ROPE(D, KVQ_F32); break;                                     \
    case KVQ_BF16: KVQ_ROPE(D, KVQ_BF16); break;                                   \
    case KVQ_F16: KVQ_ROPE(D, KVQ_F16); break;                                     \
    default: return fail(KVQ_EINVAL, "%s: unknown cos_sin_dtype %d", op, cos_sin_dtype); \
  }
  switch (dtype) {
    case KVQ_F32: KVQ_ROPE_C(KVQ_F32); break;
    case KVQ_BF16: KVQ_ROPE_C(KVQ_BF16); break;
    case KVQ_F16: KVQ_ROPE_C(KVQ_F16); break;
    default: return fail(KVQ_EINVAL, "%s: unknown dtype %d", op, dtype);
  }
#undef KVQ_ROPE_C
#undef KVQ_ROPE
  return check_hip(hipGetLastError(), "concat_and_cache_mla_rope_int8 launch");
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
  const int esz = src_dtype == KVQ_F32 ? 4 : 2;
  if ((src_dtype == KVQ_F32 || src_dtype == KVQ_BF16 || src_dtype == KVQ_F16) && g.kv_lora_rank % 8 == 0 &&
      g.rope_dim % 8 == 0 && g.stride_row % 4 == 0 && ((uintptr_t)kv_c % 4) == 0 && ((uintptr_t)k_pe % 4) == 0 &&
      (kv_c_stride * esz) % 4 == 0 && (k_pe_stride * esz) % 4 == 0) {
    hipLaunchKernelGGL(mla_quant_write_rows8_kernel, dim3((unsigned)blocks), dim3(256), 0, s, kv_c, k_pe, src_dtype,
                       kv_c_stride, k_pe_stride, c, g, slot_mapping, num_tokens, eps);
    return check_hip(hipGetLastError(), "concat_and_cache_mla_int8 launch");
  }
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
