// Shared host/device helpers of the gfx950 int8 KV-cache kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kvq.h"

namespace kvq {

// ---- host side -------------------------------------------------------------
int fail(int code, const char* fmt, ...);  // records kvq_last_error(), returns code
int check_hip(hipError_t e, const char* what);
int num_cus();
bool batch_invariant();  // the process-wide mode of kvq_set_batch_invariant()
inline hipStream_t as_stream(kvq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

#define KVQ_REQUIRE(cond, ...)                      \
  do {                                              \
    if (!(cond)) return ::kvq::fail(KVQ_EINVAL, __VA_ARGS__); \
  } while (0)

// ---- device side -----------------------------------------------------------
typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// The cache records are only 4-byte aligned (a record is 2*(D+4) bytes), so wide
// loads from them carry an explicit 4-byte alignment.
typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef float floatx4_a4 __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kWave = 64;

// Bit reinterpretation through by-value scalars.  __builtin_bit_cast applied directly to a
// vector ELEMENT expression (v.y, v[i]) reads element 0 of the vector on this compiler, so
// elements are always copied into a scalar parameter first.
__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}

// fp32 -> bf16, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <int DT>
__device__ __forceinline__ float load_act(const void* p, int64_t i) {
  if constexpr (DT == KVQ_F32) return reinterpret_cast<const float*>(p)[i];
  if constexpr (DT == KVQ_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  return (float)reinterpret_cast<const half_t*>(p)[i];
}

template <int DT>
__device__ __forceinline__ void store_act(void* p, int64_t i, float v) {
  if constexpr (DT == KVQ_F32) reinterpret_cast<float*>(p)[i] = v;
  else if constexpr (DT == KVQ_BF16) reinterpret_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  else reinterpret_cast<half_t*>(p)[i] = (half_t)v;
}

// fp32 -> OCP e4m3fn bit pattern (1 sign, 4 exponent bits with bias 7, 3 mantissa bits; largest finite
// value 448, no infinities), round to nearest even, saturating: in integer arithmetic, so that the codes
// are the same bits on every path that produces them.
__device__ __forceinline__ uint32_t f32_to_e4m3fn_bits(float y) {
  uint32_t u = __builtin_bit_cast(uint32_t, y);
  const uint32_t sign = (u >> 24) & 0x80u;
  u &= 0x7fffffffu;
  uint32_t code;
  if (u < 0x3c800000u) {                       // below 2^-6: multiples of 2^-9 (8 = the smallest normal)
    code = (uint32_t)__builtin_rintf(__builtin_bit_cast(float, u) * 512.0f);
  } else {
    const uint32_t r = u + 0x7ffffu + ((u >> 20) & 1u);   // nearest even at mantissa bit 20
    code = (r >> 20) - ((127u - 7u) << 3);
    code = code > 0x7eu ? 0x7eu : code;        // past 448 (also inf / nan): the largest finite code
  }
  return sign | code;
}

// Output dtype known only at run time (one uniform branch per store).
constexpr int kRuntimeDtype = -1;
__device__ __forceinline__ void store_act_rt(int dtype, void* p, int64_t i, float v) {
  if (dtype == KVQ_F32) store_act<KVQ_F32>(p, i, v);
  else if (dtype == KVQ_BF16) store_act<KVQ_BF16>(p, i, v);
  else store_act<KVQ_F16>(p, i, v);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
// Reductions over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one lane of each quarter-wave), result in
// all four: two register swaps (v_permlane32_swap / v_permlane16_swap exchange half-waves / odd and
// even rows of 16 between two registers), no trip through LDS.  The instruction swaps between TWO
// registers; the empty asm keeps the compiler from handing it one register twice for equal values.
__device__ __forceinline__ void swap_halves(uint32_t x, bool rows16, uint32_t& a, uint32_t& b) {
  uint32_t y = x;
  asm volatile("" : "+v"(y));
  if (rows16) {
    auto r = __builtin_amdgcn_permlane16_swap(x, y, false, false);
    a = r[0];
    b = r[1];
  } else {
    auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
    a = r[0];
    b = r[1];
  }
}
__device__ __forceinline__ float max_over_quarters(float v) {
  uint32_t a, b;
  swap_halves(__builtin_bit_cast(uint32_t, v), false, a, b);
  v = fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
  swap_halves(__builtin_bit_cast(uint32_t, v), true, a, b);
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
// the same over the two lanes l, l ^ 32
__device__ __forceinline__ float max_over_halves(float v) {
  uint32_t a, b;
  swap_halves(__builtin_bit_cast(uint32_t, v), false, a, b);
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
__device__ __forceinline__ float sum_over_quarters(float v) {
  uint32_t a, b;
  swap_halves(__builtin_bit_cast(uint32_t, v), false, a, b);
  v = __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
  swap_halves(__builtin_bit_cast(uint32_t, v), true, a, b);
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}
// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global
// load in flight (vmcnt(0)), which would drain the tile prefetch issued just before it; here the
// loads stay in flight and the compiler's own wait before their first use still applies.
// Code bytes of one half (K or V) of a record.
__host__ __device__ inline int code_bytes(const kvq_cache_geom& g) {
  return g.code_type == KVQ_CODE_INT4 ? g.head_size / 2 : g.head_size;
}

// One cache row's quantisation with 8 elements per lane and LPR lanes per row (every lane of the wave takes
// part in the shuffles): scale = max(amax, eps) / 127 (448 for fp8 codes, 7 for int4), code = rint(x / scale)
// clamped.  int8 / fp8: the lane's 8 code bytes in pk[0], pk[1]; int4: its 8 nibbles in pk[0] (element i in
// bits 4 i .. 4 i + 3: an even dim in the low nibble of its byte).
// Shared by the write kernel and by the decode kernel's fused write, so that both store the same bytes.
template <int LPR>
__device__ __forceinline__ void quant_row8(const float (&x)[8], float eps, int code_type, uint32_t (&pk)[2], float& scale) {
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(x[i]));
#pragma unroll
  for (int o = LPR / 2; o >= 1; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, kWave));
  amax = fmaxf(amax, eps);  // eps may be 0 for fp16 sources (1e-10 underflows)
  scale = code_type == KVQ_CODE_FP8_E4M3 ? amax / 448.0f : (code_type == KVQ_CODE_INT4 ? amax / 7.0f : amax / 127.0f);
  pk[0] = 0u;
  pk[1] = 0u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float y = scale > 0.f ? x[i] / scale : 0.f;  // scale == 0: all-zero fp16 row
    if (code_type == KVQ_CODE_INT4) {
      const float r = fminf(fmaxf(rintf(y), -8.f), 7.f);
      pk[0] |= ((uint32_t)(int)r & 0xfu) << (4 * i);
      continue;
    }
    uint32_t code;
    if (code_type == KVQ_CODE_FP8_E4M3) {
      code = f32_to_e4m3fn_bits(y);
    } else {
      const float r = fminf(fmaxf(rintf(y), -128.f), 127.f);
      code = (uint32_t)(int)r & 0xffu;
    }
    pk[i >> 2] |= code << (8 * (i & 3));
  }
}

// Round a float to the nearest value of the activation type (the arithmetic type of the rotary
// embedding below is the activation type, one rounding per operation).
template <int DT>
__device__ __forceinline__ float round_act(float v) {
  if constexpr (DT == KVQ_F32) return v;
  if constexpr (DT == KVQ_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  return (float)(half_t)v;
}

// (x, y) -> (x cos - y sin, y cos + x sin) in the activation type: every product and every sum is
// rounded on its own (no fused multiply-add), as the reference's operators on qk_t do
// (csrc/libtorch_stable/cache_kernels_fused.cu:77-84).  fp16 uses the native half operators (each
// result correctly rounded); bf16 goes through float and rounds after every operation, which is
// what the bf16 operators of hip_bf16.h -- the type the reference's ROCm branch selects, :13-16 --
// do; fp32 is plain fp32 without contraction.
template <int DT>
__device__ __forceinline__ void rotate_pair(float x, float y, float c, float s, float& xo, float& yo) {
#pragma clang fp contract(off)  // the default for device code is to fuse a * b + c, also through __fmul_rn
  if constexpr (DT == KVQ_F16) {
    const half_t hx = (half_t)x, hy = (half_t)y, hc = (half_t)c, hs = (half_t)s;
    const half_t a = hx * hc, b = hy * hs, d = hy * hc, e = hx * hs;
    xo = (float)(half_t)(a - b);
    yo = (float)(half_t)(d + e);
  } else {
    const float a = round_act<DT>(x * c), b = round_act<DT>(y * s), d = round_act<DT>(y * c), e = round_act<DT>(x * s);
    xo = round_act<DT>(a - b);
    yo = round_act<DT>(d + e);
  }
}

// Eight consecutive elements of a row of runtime type `dt`, as floats (`elem` = element offset; 4-byte aligned).
__device__ __forceinline__ void load_row8(const void* src, int dt, int64_t elem, float (&x)[8]) {
  if (dt == KVQ_F32) {
    const float* p = reinterpret_cast<const float*>(src) + elem;
    const floatx4 a = *reinterpret_cast<const floatx4_a4*>(p), b = *reinterpret_cast<const floatx4_a4*>(p + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  } else {
    const u32x4 v = *reinterpret_cast<const u32x4_a4*>(reinterpret_cast<const uint16_t*>(src) + elem);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t e = v[w];
      if (dt == KVQ_BF16) {
        x[2 * w] = as_f32(e << 16);
        x[2 * w + 1] = as_f32(e & 0xffff0000u);
      } else {
        const half2_t hh = __builtin_bit_cast(half2_t, e);
        x[2 * w] = (float)hh.x;
        x[2 * w + 1] = (float)hh.y;
      }
    }
  }
}

// One MLA latent row [kv_c | k_pe] quantised by ONE wave, eight elements per lane and piece: lane l takes the
// 8-element pieces l and 64 + l of the row (rp pieces of kv_c, np pieces in all, np <= 128).  Loading,
// converting and quantising are apart so that a caller can put other work between them (a conversion right
// behind the loads would make the wave wait for them there).  Shared by the write kernel and by the decode
// kernels' fused write, so that both store the same bytes.
struct MlaRowRaw {
  u32x4 w[2][2];   // 8 elements: one 16-byte word of 16-bit elements, two of fp32
  bool have[2];
};
struct MlaRowPieces {
  float x[2][8];
  bool have[2];
};
__device__ __forceinline__ void mla_row_load_raw(const void* kv_c, const void* k_pe, int dt, int64_t kvc_elem,
                                                 int64_t kpe_elem, int rp, int np, int lane, MlaRowRaw& r) {
  const int64_t esz = dt == KVQ_F32 ? 4 : 2;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int piece = lane + kWave * j;
    r.have[j] = piece < np;
    const int pc = r.have[j] ? piece : 0;
    const uint8_t* p = pc < rp ? static_cast<const uint8_t*>(kv_c) + (kvc_elem + 8 * pc) * esz
                               : static_cast<const uint8_t*>(k_pe) + (kpe_elem + 8 * (pc - rp)) * esz;
    r.w[j][0] = *reinterpret_cast<const u32x4_a4*>(p);
    if (dt == KVQ_F32) r.w[j][1] = *reinterpret_cast<const u32x4_a4*>(p + 16);   // uniform
    else r.w[j][1] = (u32x4){0u, 0u, 0u, 0u};
  }
}
__device__ __forceinline__ void mla_row_convert(const MlaRowRaw& raw, int dt, MlaRowPieces& r) {
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    r.have[j] = raw.have[j];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t e = raw.w[j][0][w];
      const half2_t hh = __builtin_bit_cast(half2_t, e);
      const float lo16 = dt == KVQ_BF16 ? as_f32(e << 16) : (float)hh.x;
      const float hi16 = dt == KVQ_BF16 ? as_f32(e & 0xffff0000u) : (float)hh.y;
      // fp32: elements 0-3 in word 0, 4-7 in word 1
      r.x[j][2 * w] = dt == KVQ_F32 ? as_f32(raw.w[j][w >> 1][(2 * w) & 3]) : lo16;
      r.x[j][2 * w + 1] = dt == KVQ_F32 ? as_f32(raw.w[j][w >> 1][(2 * w + 1) & 3]) : hi16;
    }
  }
}
__device__ __forceinline__ void mla_row_load(const void* kv_c, const void* k_pe, int dt, int64_t kvc_elem,
                                             int64_t kpe_elem, int rp, int np, int lane, MlaRowPieces& r) {
  MlaRowRaw raw;
  mla_row_load_raw(kv_c, k_pe, dt, kvc_elem, kpe_elem, rp, np, lane, raw);
  mla_row_convert(raw, dt, r);
}
// scale = max(amax, eps) / 127 (every lane of the wave takes part in the maximum)
__device__ __forceinline__ float mla_row_scale(const MlaRowPieces& r, float eps) {
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, r.have[j] ? fabsf(r.x[j][i]) : 0.f);
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, kWave));
  return fmaxf(amax, eps) / 127.0f;
}
__device__ __forceinline__ void mla_row_store(const MlaRowPieces& r, float scale, uint8_t* row, float* scale_ptr, int lane) {
  const bool pos = scale > 0.f;   // scale == 0: an all-zero row with eps 0
  const float div = pos ? scale : 1.f;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (!r.have[j]) continue;
    uint32_t pk[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float q = rintf(r.x[j][i] / div);
      q = pos ? fminf(fmaxf(q, -128.f), 127.f) : 0.f;
      pk[i >> 2] |= ((uint32_t)(int)q & 0xffu) << (8 * (i & 3));
    }
    *reinterpret_cast<u32x2_a4*>(row + 8 * (lane + kWave * j)) = (u32x2){pk[0], pk[1]};
  }
  if (lane == 0) *scale_ptr = scale;
}

__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ int wave_max_i32(int v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = max(v, __shfl_xor(v, o, kWave));
  return __builtin_amdgcn_readfirstlane(v);
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

}  // namespace kvq
