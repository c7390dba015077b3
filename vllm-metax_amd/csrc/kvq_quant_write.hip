// Quantise-on-write of new K/V tokens into the paged int8 cache (gfx950).
//
// One wavefront owns one (token, kv head, K-or-V) row: the row is read once with
// coalesced loads, the absmax is reduced across the 64 lanes, and codes plus the
// fp32 scale go straight into the (block, slot, head) record.  The arithmetic is
// the bit-exact contract: scale = max(absmax, eps) / 127 (IEEE fp32 division),
// code = clamp(rint(x / scale), -128, 127) with round-half-to-even.  A cache whose geometry says
// KVQ_CODE_FP8_E4M3 gets scale = max(absmax, eps) / 448 and the nearest e4m3fn code instead; KVQ_CODE_INT4
// scale = max(absmax, eps) / 7 and 4-bit codes in [-8, 7], two per byte (the even dim in the low nibble).
#include "kvq_internal.h"

namespace kvq {

template <int DT, int VEC>  // VEC = head_size / 64 when that is 1, 2 or 4; 0 = any head size
__global__ __launch_bounds__(256) void quant_write_kernel(
    const void* __restrict__ key, const void* __restrict__ value, int64_t key_stride_t,
    int64_t key_stride_h, int64_t value_stride_t, int64_t value_stride_h,
    uint8_t* __restrict__ cache, kvq_cache_geom g, const int64_t* __restrict__ slot_mapping,
    int64_t num_rows /* T * Hkv * 2 */, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
  if (row >= num_rows) return;
  const int is_v = (int)(row & 1);
  const int64_t th = row >> 1;
  // 32-bit index arithmetic whenever the row count allows it (a 64-bit divide is a long routine)
  int h;
  int64_t t;
  if (num_rows <= 0xffffffffLL) {
    const uint32_t t32 = (uint32_t)th / (uint32_t)g.num_kv_heads;
    h = (int)((uint32_t)th - t32 * (uint32_t)g.num_kv_heads);
    t = t32;
  } else {
    h = (int)(th % g.num_kv_heads);
    t = th / g.num_kv_heads;
  }
  const int D = g.head_size;
  const void* src = is_v ? value : key;
  const int64_t src_base = is_v ? (t * value_stride_t + h * value_stride_h)
                                : (t * key_stride_t + h * key_stride_h);
  // The row's loads do not depend on the slot: they go out together with the slot's load, so the
  // kernel pays one memory round trip before it can write instead of two.
  const int64_t slot = slot_mapping[t];
  float x[VEC > 0 ? VEC : 1];
  if constexpr (VEC > 0) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) x[i] = load_act<DT>(src, src_base + lane * VEC + i);
  }
  if (slot < 0) return;  // padding token
  int64_t blk, off;
  if ((uint64_t)slot <= 0xffffffffull) {
    const uint32_t b32 = (uint32_t)slot / (uint32_t)g.block_size;
    blk = b32;
    off = (uint32_t)slot - b32 * (uint32_t)g.block_size;
  } else {
    blk = slot / g.block_size;
    off = slot - blk * g.block_size;
  }
  uint8_t* rec = cache + blk * g.stride_block + off * g.stride_slot + (int64_t)h * g.stride_head;
  int8_t* codes = reinterpret_cast<int8_t*>(rec + (is_v ? g.v_off : g.k_off));
  float* scale_ptr = reinterpret_cast<float*>(rec + (is_v ? g.vs_off : g.ks_off));

  if constexpr (VEC > 0) {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) amax = fmaxf(amax, fabsf(x[i]));
    amax = fmaxf(wave_max(amax), eps);  // eps may be 0 for fp16 sources (1e-10 underflows)
    const bool fp8 = g.code_type == KVQ_CODE_FP8_E4M3;
    const float scale = fp8 ? amax / 448.0f : amax / 127.0f;
    int8_t c[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float y = scale > 0.f ? x[i] / scale : 0.f;  // scale == 0: all-zero fp16 row
      if (fp8) {
        c[i] = (int8_t)f32_to_e4m3fn_bits(y);
      } else {
        const float r = fminf(fmaxf(rintf(y), -128.f), 127.f);
        c[i] = (int8_t)(int)r;
      }
    }
    if constexpr (VEC == 1) {
      codes[lane] = c[0];
    } else if constexpr (VEC == 2) {
      uint16_t pk = (uint16_t)(uint8_t)c[0] | ((uint16_t)(uint8_t)c[1] << 8);
      reinterpret_cast<uint16_t*>(codes)[lane] = pk;  // records are 4-byte aligned
    } else {
      uint32_t pk = (uint32_t)(uint8_t)c[0] | ((uint32_t)(uint8_t)c[1] << 8) |
                    ((uint32_t)(uint8_t)c[2] << 16) | ((uint32_t)(uint8_t)c[3] << 24);
      reinterpret_cast<uint32_t*>(codes)[lane] = pk;
    }
    if (lane == 0) *scale_ptr = scale;
  } else {
    float amax = 0.f;
    for (int d = lane; d < D; d += kWave) amax = fmaxf(amax, fabsf(load_act<DT>(src, src_base + d)));
    amax = fmaxf(wave_max(amax), eps);  // eps may be 0 for fp16 sources (1e-10 underflows)
    const bool fp8 = g.code_type == KVQ_CODE_FP8_E4M3;
    if (g.code_type == KVQ_CODE_INT4) {   // a byte per two dims: the even one in the low nibble
      const float scale = amax / 7.0f;
      for (int b = lane; b < D / 2; b += kWave) {
        uint32_t byte = 0;
        for (int j = 0; j < 2; ++j) {
          const float y = scale > 0.f ? load_act<DT>(src, src_base + 2 * b + j) / scale : 0.f;
          const float r = fminf(fmaxf(rintf(y), -8.f), 7.f);
          byte |= ((uint32_t)(int)r & 0xfu) << (4 * j);
        }
        codes[b] = (int8_t)byte;
      }
      if (lane == 0) *scale_ptr = scale;
      return;
    }
    const float scale = fp8 ? amax / 448.0f : amax / 127.0f;
    for (int d = lane; d < D; d += kWave) {
      const float y = scale > 0.f ? load_act<DT>(src, src_base + d) / scale : 0.f;
      if (fp8) {
        codes[d] = (int8_t)f32_to_e4m3fn_bits(y);
      } else {
        const float r = fminf(fmaxf(rintf(y), -128.f), 127.f);
        codes[d] = (int8_t)(int)r;
      }
    }
    if (lane == 0) *scale_ptr = scale;
  }
}

// The same arithmetic with D / 8 lanes per row and 8 elements per lane (one 16-byte load for 16-bit
// sources), i.e. 512 / D rows per wave: four times fewer waves than one row per wave at D = 128 and
// 16-byte instead of 4-byte accesses.  Rows past the end are clamped for the loads and masked for
// the stores, so that every lane takes part in the shuffles.
template <int DT, int D>
__global__ __launch_bounds__(256) void quant_write_rows_kernel(
    const void* __restrict__ key, const void* __restrict__ value, int64_t key_stride_t,
    int64_t key_stride_h, int64_t value_stride_t, int64_t value_stride_h,
    uint8_t* __restrict__ cache, kvq_cache_geom g, const int64_t* __restrict__ slot_mapping,
    int64_t num_rows /* T * Hkv * 2 */, float eps) {
  constexpr int LPR = D / 8;        // lanes per row
  constexpr int RPW = kWave / LPR;  // rows per wave
  const int lane = threadIdx.x & (kWave - 1);
  const int li = lane % LPR;
  const int64_t row_raw = ((int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave)) * RPW + lane / LPR;
  const bool live = row_raw < num_rows;
  const int64_t row = live ? row_raw : num_rows - 1;
  const int is_v = (int)(row & 1);
  const int64_t th = row >> 1;
  int h;
  int64_t t;
  if (num_rows <= 0xffffffffLL) {
    const uint32_t t32 = (uint32_t)th / (uint32_t)g.num_kv_heads;
    h = (int)((uint32_t)th - t32 * (uint32_t)g.num_kv_heads);
    t = t32;
  } else {
    h = (int)(th % g.num_kv_heads);
    t = th / g.num_kv_heads;
  }
  const void* src = is_v ? value : key;
  const int64_t src_base = (is_v ? (t * value_stride_t + h * value_stride_h) : (t * key_stride_t + h * key_stride_h)) + li * 8;
  const int64_t slot = slot_mapping[t];  // in flight together with the row's loads
  float x[8];
  if constexpr (DT == KVQ_F32) {
    const float* p = reinterpret_cast<const float*>(src) + src_base;
    const floatx4 a = *reinterpret_cast<const floatx4_a4*>(p), b = *reinterpret_cast<const floatx4_a4*>(p + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  } else {
    const u32x4 v = *reinterpret_cast<const u32x4_a4*>(reinterpret_cast<const uint16_t*>(src) + src_base);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t e = v[w];
      if constexpr (DT == KVQ_BF16) {
        x[2 * w] = as_f32(e << 16);
        x[2 * w + 1] = as_f32(e & 0xffff0000u);
      } else {
        const half2_t hh = __builtin_bit_cast(half2_t, e);
        x[2 * w] = (float)hh.x;
        x[2 * w + 1] = (float)hh.y;
      }
    }
  }
  uint32_t pk[2];
  float scale;
  quant_row8<LPR>(x, eps, g.code_type, pk, scale);
  if (!live || slot < 0) return;  // padding token (after the shuffles: every lane took part)
  int64_t blk, off;
  if ((uint64_t)slot <= 0xffffffffull) {
    const uint32_t b32 = (uint32_t)slot / (uint32_t)g.block_size;
    blk = b32;
    off = (uint32_t)slot - b32 * (uint32_t)g.block_size;
  } else {
    blk = slot / g.block_size;
    off = slot - blk * g.block_size;
  }
  uint8_t* rec = cache + blk * g.stride_block + off * g.stride_slot + (int64_t)h * g.stride_head;
  if (g.code_type == KVQ_CODE_INT4) *reinterpret_cast<uint32_t*>(rec + (is_v ? g.v_off : g.k_off) + li * 4) = pk[0];
  else *reinterpret_cast<u32x2_a4*>(rec + (is_v ? g.v_off : g.k_off) + li * 8) = (u32x2){pk[0], pk[1]};
  if (li == 0) *reinterpret_cast<float*>(rec + (is_v ? g.vs_off : g.ks_off)) = scale;
}

// Rotary embedding of the step's query and key rows (in place, the first rot_dim dims of every head) fused with
// the quantise-on-write of the rotated K rows and the V rows: the work of do_rope_and_kv_cache_update.  One
// workgroup per token.  All threads rotate the (q head, pair) items; then wave w takes the rows (kv head, K | V)
// w, w + 4, ...: a lane owns the dim pairs (2 b, 2 b + 1), b = lane, lane + 64, and computes the rotated value of
// each of its dims from the ORIGINAL row (so no lane reads what another wrote), stores it back into `key` and
// quantises the row from those values -- the bytes the write kernel would store after a separate rotation.
// The rotation arithmetic is rotate_pair's (one rounding per operation in the activation type).
template <int DT, int CT, bool NEOX>
__global__ __launch_bounds__(256) void rope_quant_write_kernel(
    const int64_t* __restrict__ positions, void* __restrict__ query, int64_t q_stride_t, int64_t q_stride_h,
    int num_q_heads, void* __restrict__ key, int64_t k_stride_t, int64_t k_stride_h, const void* __restrict__ value,
    int64_t v_stride_t, int64_t v_stride_h, const void* __restrict__ cos_sin, int rot_dim,
    uint8_t* __restrict__ cache, kvq_cache_geom g, const int64_t* __restrict__ slot_mapping, float eps) {
  const int64_t t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;  // padding token: nothing is rotated, nothing is written
  const int64_t pos = positions[t];
  const int embed = rot_dim / 2;
  const int64_t cs = pos * rot_dim;
  auto cosine = [&](int pair) { return round_act<DT>(load_act<CT>(cos_sin, cs + pair)); };
  auto sine = [&](int pair) { return round_act<DT>(load_act<CT>(cos_sin, cs + pair + embed)); };
  // ---- query: (head, pair) items over all threads
  const int nq = num_q_heads * embed;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const int head = i / embed, pair = i - head * embed;
    const int ix = NEOX ? pair : 2 * pair, iy = NEOX ? embed + pair : 2 * pair + 1;
    const int64_t base = t * q_stride_t + (int64_t)head * q_stride_h;
    float xo, yo;
    rotate_pair<DT>(load_act<DT>(query, base + ix), load_act<DT>(query, base + iy), cosine(pair), sine(pair), xo, yo);
    store_act<DT>(query, base + ix, xo);
    store_act<DT>(query, base + iy, yo);
  }
  // ---- key / value rows
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int D = g.head_size;
  const int64_t blk = slot / g.block_size;
  const int64_t off = slot - blk * g.block_size;
  constexpr int kMaxPairs = 2;   // head sizes up to 256
  for (int r = wave; r < 2 * g.num_kv_heads; r += 4) {
    const int h = r >> 1, is_v = r & 1;
    const void* src = is_v ? value : key;
    const int64_t base = is_v ? t * v_stride_t + (int64_t)h * v_stride_h : t * k_stride_t + (int64_t)h * k_stride_h;
    // the value of dim d after the rotation (K rows, d < rot_dim) or as it is
    auto dim_value = [&](int d) -> float {
      if (is_v || d >= rot_dim) return load_act<DT>(src, base + d);
      const int pair = NEOX ? (d < embed ? d : d - embed) : d >> 1;
      const int ix = NEOX ? pair : 2 * pair, iy = NEOX ? embed + pair : 2 * pair + 1;
      float xo, yo;
      rotate_pair<DT>(load_act<DT>(src, base + ix), load_act<DT>(src, base + iy), cosine(pair), sine(pair), xo, yo);
      return d == ix ? xo : yo;
    };
    float x[kMaxPairs][2];
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxPairs; ++i) {
      const int b = lane + kWave * i;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        x[i][j] = 2 * b + j < D ? dim_value(2 * b + j) : 0.f;
        amax = fmaxf(amax, fabsf(x[i][j]));
      }
    }
    // every lane has read the original row before any lane overwrites it
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    amax = fmaxf(wave_max(amax), eps);
    const int ct = g.code_type;
    const float scale = ct == KVQ_CODE_FP8_E4M3 ? amax / 448.0f : (ct == KVQ_CODE_INT4 ? amax / 7.0f : amax / 127.0f);
    uint8_t* rec = cache + blk * g.stride_block + off * g.stride_slot + (int64_t)h * g.stride_head;
    uint8_t* codes = rec + (is_v ? g.v_off : g.k_off);
#pragma unroll
    for (int i = 0; i < kMaxPairs; ++i) {
      const int b = lane + kWave * i;
      if (2 * b >= D) continue;
      uint32_t c[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float y = scale > 0.f ? x[i][j] / scale : 0.f;
        if (ct == KVQ_CODE_FP8_E4M3) c[j] = f32_to_e4m3fn_bits(y);
        else if (ct == KVQ_CODE_INT4) c[j] = (uint32_t)(int)fminf(fmaxf(rintf(y), -8.f), 7.f) & 0xfu;
        else c[j] = (uint32_t)(int)fminf(fmaxf(rintf(y), -128.f), 127.f) & 0xffu;
      }
      if (ct == KVQ_CODE_INT4) codes[b] = (uint8_t)(c[0] | (c[1] << 4));
      else *reinterpret_cast<uint16_t*>(codes + 2 * b) = (uint16_t)(c[0] | (c[1] << 8));
      if (!is_v && 2 * b < rot_dim) {   // the rotated key goes back in place
        store_act<DT>(key, base + 2 * b, x[i][0]);
        store_act<DT>(key, base + 2 * b + 1, x[i][1]);
      }
    }
    if (lane == 0) *reinterpret_cast<float*>(rec + (is_v ? g.vs_off : g.ks_off)) = scale;
  }
}


template <int DT>
static int launch_quant_write(const void* key, const void* value, int64_t kst, int64_t ksh,
                              int64_t vst, int64_t vsh, uint8_t* cache, const kvq_cache_geom& g,
                              const int64_t* slot_mapping, int64_t T, float eps, hipStream_t s) {
  const int64_t rows = T * g.num_kv_heads * 2;
  // several rows per wave where the rows can be read 8 elements at a time (4-byte aligned)
  const int esz = DT == KVQ_F32 ? 4 : 2;
  const bool vec_ok = (g.head_size == 64 || g.head_size == 128 || g.head_size == 256) &&
                      ((uintptr_t)key % 4) == 0 && ((uintptr_t)value % 4) == 0 &&
                      ((kst | ksh | vst | vsh) * esz) % 4 == 0;
  if (vec_ok) {
    const int rpw = 512 / g.head_size;
    const int64_t vblocks = (rows + 4 * rpw - 1) / (4 * rpw);
    if (vblocks > 0x7fffffffLL) return fail(KVQ_EINVAL, "reshape_and_cache_int8: too many tokens");
    dim3 vgrid((unsigned)vblocks), vblock(256);
#define KVQ_LAUNCH_ROWS(DD)                                                                          \
  hipLaunchKernelGGL((quant_write_rows_kernel<DT, DD>), vgrid, vblock, 0, s, key, value, kst, ksh, \
                     vst, vsh, cache, g, slot_mapping, rows, eps)
    switch (g.head_size) {
      case 64: KVQ_LAUNCH_ROWS(64); break;
      case 128: KVQ_LAUNCH_ROWS(128); break;
      default: KVQ_LAUNCH_ROWS(256); break;
    }
#undef KVQ_LAUNCH_ROWS
    return check_hip(hipGetLastError(), "reshape_and_cache_int8 launch");
  }
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return fail(KVQ_EINVAL, "reshape_and_cache_int8: too many tokens");
  dim3 grid((unsigned)blocks), block(256);
#define KVQ_LAUNCH(V)                                                                     \
  hipLaunchKernelGGL((quant_write_kernel<DT, V>), grid, block, 0, s, key, value, kst, ksh, \
                     vst, vsh, cache, g, slot_mapping, rows, eps)
  switch (g.code_type == KVQ_CODE_INT4 ? 0 : g.head_size) {   // nibbles: the any-size loop packs two dims per lane
    case 64: KVQ_LAUNCH(1); break;
    case 128: KVQ_LAUNCH(2); break;
    case 256: KVQ_LAUNCH(4); break;
    default: KVQ_LAUNCH(0); break;
  }
#undef KVQ_LAUNCH
  return check_hip(hipGetLastError(), "reshape_and_cache_int8 launch");
}

}  // namespace kvq

extern "C" int kvq_reshape_and_cache_int8(const void* key, const void* value, int src_dtype,
                                          int64_t key_stride_t, int64_t key_stride_h,
                                          int64_t value_stride_t, int64_t value_stride_h,
                                          void* cache, const kvq_cache_geom* geom,
                                          const int64_t* slot_mapping, int64_t num_tokens,
                                          float eps, kvq_stream_t stream) {
  using namespace kvq;
  KVQ_REQUIRE(geom != nullptr, "reshape_and_cache_int8: geom is NULL");
  KVQ_REQUIRE(num_tokens >= 0, "reshape_and_cache_int8: negative num_tokens");
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(key && value && cache && slot_mapping, "reshape_and_cache_int8: NULL pointer");
  const kvq_cache_geom& g = *geom;
  KVQ_REQUIRE(g.num_kv_heads > 0 && g.head_size > 0 && g.block_size > 0,
              "reshape_and_cache_int8: bad geometry (heads=%d head_size=%d block_size=%d)",
              g.num_kv_heads, g.head_size, g.block_size);
  KVQ_REQUIRE(g.head_size % 4 == 0, "reshape_and_cache_int8: head_size %d must be a multiple of 4",
              g.head_size);
  KVQ_REQUIRE((g.k_off | g.v_off | g.ks_off | g.vs_off | g.stride_block | g.stride_slot |
               g.stride_head) % 4 == 0 && ((uintptr_t)cache % 4) == 0,
              "reshape_and_cache_int8: cache offsets/strides must be 4-byte aligned");
  KVQ_REQUIRE(eps >= 0.f, "reshape_and_cache_int8: eps must not be negative");
  KVQ_REQUIRE(g.code_type == KVQ_CODE_INT8 || g.code_type == KVQ_CODE_FP8_E4M3 || g.code_type == KVQ_CODE_INT4,
              "reshape_and_cache_int8: unknown code_type %d", g.code_type);
  hipStream_t s = as_stream(stream);
  uint8_t* c = static_cast<uint8_t*>(cache);
  switch (src_dtype) {
    case KVQ_F32:
      return launch_quant_write<KVQ_F32>(key, value, key_stride_t, key_stride_h, value_stride_t,
                                         value_stride_h, c, g, slot_mapping, num_tokens, eps, s);
    case KVQ_BF16:
      return launch_quant_write<KVQ_BF16>(key, value, key_stride_t, key_stride_h, value_stride_t,
                                          value_stride_h, c, g, slot_mapping, num_tokens, eps, s);
    case KVQ_F16:
      return launch_quant_write<KVQ_F16>(key, value, key_stride_t, key_stride_h, value_stride_t,
                                         value_stride_h, c, g, slot_mapping, num_tokens, eps, s);
    default:
      return fail(KVQ_EINVAL, "reshape_and_cache_int8: unknown src_dtype %d", src_dtype);
  }
}

extern "C" int kvq_rope_and_cache_int8(const int64_t* positions, void* query, int64_t q_stride_t, int64_t q_stride_h,
                                       int num_q_heads, void* key, int64_t key_stride_t, int64_t key_stride_h,
                                       const void* value, int64_t value_stride_t, int64_t value_stride_h,
                                       int src_dtype, const void* cos_sin_cache, int cos_sin_dtype, int rot_dim,
                                       int is_neox, void* cache, const kvq_cache_geom* geom,
                                       const int64_t* slot_mapping, int64_t num_tokens, float eps,
                                       kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "rope_and_cache_int8";
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(num_tokens >= 0 && num_tokens <= 0x7fffffffLL, "%s: num_tokens out of range", op);
  if (num_tokens == 0) return KVQ_OK;
  KVQ_REQUIRE(positions && query && key && value && cos_sin_cache && cache && slot_mapping, "%s: NULL pointer", op);
  const kvq_cache_geom& g = *geom;
  KVQ_REQUIRE(g.num_kv_heads > 0 && g.block_size > 0 && g.head_size > 0 && g.head_size % 2 == 0 && g.head_size <= 256,
              "%s: bad geometry (heads=%d head_size=%d block_size=%d; head sizes up to 256)", op, g.num_kv_heads,
              g.head_size, g.block_size);
  KVQ_REQUIRE(num_q_heads > 0, "%s: num_q_heads must be positive", op);
  KVQ_REQUIRE(rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= g.head_size, "%s: rot_dim %d must be even and at most the head size %d",
              op, rot_dim, g.head_size);
  KVQ_REQUIRE((g.k_off | g.v_off | g.ks_off | g.vs_off | g.stride_block | g.stride_slot | g.stride_head) % 4 == 0 &&
                  ((uintptr_t)cache % 4) == 0, "%s: cache offsets/strides must be 4-byte aligned", op);
  KVQ_REQUIRE(g.code_type == KVQ_CODE_INT8 || g.code_type == KVQ_CODE_FP8_E4M3 || g.code_type == KVQ_CODE_INT4,
              "%s: unknown code_type %d", op, g.code_type);
  KVQ_REQUIRE(eps >= 0.f, "%s: eps must not be negative", op);
  hipStream_t s = as_stream(stream);
  uint8_t* c = static_cast<uint8_t*>(cache);
  const dim3 grid((unsigned)num_tokens), block(256);
#define KVQ_ROPE(D, C)                                                                                              \
  do {                                                                                                              \
    if (is_neox)                                                                                                    \
      hipLaunchKernelGGL((rope_quant_write_kernel<D, C, true>), grid, block, 0, s, positions, query, q_stride_t,   \
                         q_stride_h, num_q_heads, key, key_stride_t, key_stride_h, value, value_stride_t,           \
                         value_stride_h, cos_sin_cache, rot_dim, c, g, slot_mapping, eps);                          \
    else                                                                                                            \
      hipLaunchKernelGGL((rope_quant_write_kernel<D, C, false>), grid, block, 0, s, positions, query, q_stride_t,  \
                         q_stride_h, num_q_heads, key, key_stride_t, key_stride_h, value, value_stride_t,           \
                         value_stride_h, cos_sin_cache, rot_dim, c, g, slot_mapping, eps);                          \
  } while (0)
#define KVQ_ROPE_C(D)                                                                        \
  switch (cos_sin_dtype) {                                                                   \
    case KVQ_F32: KVQ_ROPE(D, KVQ_F32); break;                                               \
    case KVQ_BF16: KVQ_ROPE(D, KVQ_BF16); break;                                             \
    case KVQ_F16: KVQ_ROPE(D, KVQ_F16); break;                                               \
    default: return fail(KVQ_EINVAL, "%s: unknown cos_sin_dtype %d", op, cos_sin_dtype);     \
  }
  switch (src_dtype) {
    case KVQ_F32: KVQ_ROPE_C(KVQ_F32); break;
    case KVQ_BF16: KVQ_ROPE_C(KVQ_BF16); break;
    case KVQ_F16: KVQ_ROPE_C(KVQ_F16); break;
    default: return fail(KVQ_EINVAL, "%s: unknown src_dtype %d", op, src_dtype);
  }
#undef KVQ_ROPE_C
#undef KVQ_ROPE
  return check_hip(hipGetLastError(), "rope_and_cache_int8 launch");
}
