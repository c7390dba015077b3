// Core of the bandwidth-bound int8 paged decode tile (gfx950, wave64, MFMA f16).
//
// One wavefront owns one KV head and streams that head's (token, head) records --
// [K codes | K scale | V codes | V scale], 2*(D+4) bytes each -- for a run of 32-token tiles.
// Per tile it
//   * reads the 32 records as flat 16-byte chunks, consecutive lanes taking consecutive chunks
//     of one record, so every quarter-wave touches 256 contiguous bytes of HBM; the chunks land
//     in registers, one tile ahead of the tile being computed;
//   * drops the chunks into a wave-private LDS window (one record per row, 16-byte aligned,
//     bank-conflict-free pitch) and reads them back in MFMA operand order: the transposition
//     between "how memory is laid out" and "how the matrix core wants it" happens in LDS;
//   * turns codes into exact fp16 numbers code + 1152 with one byte permute per two codes
//     (0x6400 | (code ^ 0x80)); the constant is removed exactly afterwards;
//   * S^T[token, head] = K . Q^T on the MFMA (the GQA group's heads are the N dim, so the KV
//     stream is read once for all of them), softmax in fp32 with the per-token K scale applied
//     to the logits;
//   * O^T[dim, head] += V^T . P~^T on the MFMA, P~ = p * v_scale rounded to fp16.
// The S accumulator layout (lane = head, registers = tokens) is exactly the B-operand layout
// P~^T needs, and the running max / sum / rescale of a head stay lane-local.
#pragma once

#include "kvq_internal.h"

namespace kvq {

constexpr int kTile = 32;            // tokens per step
constexpr int kSyncTiles = 2;        // workgroup rendezvous period of the decode stream, in tiles (power of two)
constexpr float kPScale = 256.0f;    // P~ is kept 2^8 larger so small weights stay normal in fp16
constexpr float kLazyMax = 8.0f;          // log2 of how far a logit may exceed the reference maximum of its row
constexpr float kLazyScaleMax = 255.0f;   // largest V-side scale (already times 2^8) for which 2^kLazyMax * scale stays in fp16
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kLog2e = 1.4426950408889634f;

// v_perm_b32: selector bytes 0-3 pick from `lo`, 4-7 from `hi`.
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// Codes enter the MFMA as code + 1152: 0x6400 | (code ^ 0x80) is the fp16 number
// 1024 + (code + 128), exact, built by one byte permute per two codes.  The constant is taken
// out again exactly: the QK accumulator starts at -1152 * sum(q), and the PV accumulator is
// corrected with 1152 * sum(P~), which one extra MFMA against a row of ones keeps in step.
constexpr float kCodeBias = 1152.0f;

// Two biased code bytes of x (already ^0x80) -> two fp16 values code + 1152.
__device__ __forceinline__ uint32_t bytes_to_half2(uint32_t x, bool upper) {
  return perm(0x64646464u, x, upper ? 0x04030402u : 0x04010400u);
}

// Two e4m3fn code bytes of x -> two fp16 values code / 2^8: the byte's 7 magnitude bits sit in an fp16
// pattern at bits 7 .. 13 and the sign at bit 15; as an fp16 number that pattern is the code's value
// times 2^-8 (the exponent biases differ by 15 - 7), exactly, subnormal codes included.  The 2^8 is put
// back with the scales.
__device__ __forceinline__ uint32_t fp8_bytes_to_half2(uint32_t x, bool upper) {
  const uint32_t y = perm(0u, x, upper ? 0x030c020cu : 0x010c000cu);   // the two bytes in the high byte of each half
  return (y & 0x80008000u) | ((y >> 1) & 0x3f803f80u);
}

// Two code bytes -> the two fp16 numbers the MFMA sees, for either kind of code (int8 bytes are
// expected already ^ 0x80, see prep_codes).
template <bool FP8>
__device__ __forceinline__ uint32_t codes_to_half2(uint32_t x, bool upper) {
  if constexpr (FP8) return fp8_bytes_to_half2(x, upper);
  else return bytes_to_half2(x, upper);
}
template <bool FP8>
__device__ __forceinline__ uint32_t prep_codes(uint32_t x) {
  if constexpr (FP8) return x;
  else return x ^ 0x80808080u;
}

// 8 consecutive code bytes (two dwords) -> 8 fp16 (code + 1152, or code / 2^8 for fp8 codes), one MFMA
// k-step operand.
template <bool FP8 = false>
__device__ __forceinline__ half8_t dequant8(uint32_t lo, uint32_t hi) {
  lo = prep_codes<FP8>(lo);
  hi = prep_codes<FP8>(hi);
  u32x4 r;
  r.x = codes_to_half2<FP8>(lo, false);
  r.y = codes_to_half2<FP8>(lo, true);
  r.z = codes_to_half2<FP8>(hi, false);
  r.w = codes_to_half2<FP8>(hi, true);
  return __builtin_bit_cast(half8_t, r);
}

// int4 codes: a nibble n = code ^ 8 (0 .. 15) enters the MFMA as the fp16 number 0x6400 | n = code + 1032, exact;
// the constant is taken out afterwards like the int8 path's 1152.  One and-or per two nibbles: with y = the dword
// of four code bytes ^ 0x88888888, ((y >> 4 k) & 0x000f000f) | 0x64006400 holds nibbles k and k + 4 of the dword,
// so the eight dims of a dword come out in the order 0 4 1 5 2 6 3 7 -- the order in which the query operand of an
// int4 tile is laid out as well (nibble_order).
constexpr float kCodeBiasInt4 = 1032.0f;
__device__ __forceinline__ uint32_t nibbles_to_half2(uint32_t y, int k) {
  return ((y >> (4 * k)) & 0x000f000fu) | 0x64006400u;
}
__device__ __forceinline__ half8_t dequant8_int4(uint32_t x) {
  const uint32_t y = x ^ 0x88888888u;
  u32x4 r;
  r.x = nibbles_to_half2(y, 0);
  r.y = nibbles_to_half2(y, 1);
  r.z = nibbles_to_half2(y, 2);
  r.w = nibbles_to_half2(y, 3);
  return __builtin_bit_cast(half8_t, r);
}
// MFMA k position j of an int4 operand holds dim nibble_order(j) of the dword's eight.
__host__ __device__ constexpr int nibble_order(int j) { return (j >> 1) + 4 * (j & 1); }

__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
  half2_t v = {(half_t)a, (half_t)b};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float clamp_half_range(float x) {
  return fminf(fmaxf(x, -65504.f), 65504.f);
}

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

// 16x16x32 MFMA of the activation type (fp16 or bf16 operands as four dwords, fp32 accumulate).
template <int DT>
__device__ __forceinline__ floatx4 mfma16(u32x4 a, u32x4 b, floatx4 c) {
  if constexpr (DT == KVQ_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// Two floats rounded to the activation type, packed into one dword.
template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  if constexpr (DT == KVQ_F16) {
    return pack_half2(a, b);
  } else {
    const floatx2 f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
  }
}

// Selectors that build one dword of a register transposition: the low (or high) halves of two dwords.
constexpr uint32_t kPermLowHalves = 0x05040100u, kPermHighHalves = 0x07060302u;

// What a finished run of tiles turns into.
enum class Emit { kFinal, kStreamPartial, kV2Partial };

struct AttnIO {
  // query / output rows
  const void* q;
  int64_t q_stride_t, q_stride_h;
  void* out;
  int64_t out_stride_t, out_stride_h;
  int out_dtype;  // read by kernels built for ODT == kRuntimeDtype
  float* lse;  // [rows, Hq] natural log, or nullptr
  // cache
  const uint8_t* cache;
  kvq_cache_geom g;
  const int32_t* block_table;
  int64_t bt_stride;
  int num_q_heads;
  int group;  // q heads per kv head
  float scale_log2;  // softmax scale * log2(e)
  uint32_t bs_magic;  // ceil(2^32 / block_size): x / block_size == umulhi(x, bs_magic) for x < 2^22
  int window;         // sliding window: a query sees its last `window` keys, itself included; 0 = all
  const float* sinks; // [num_q_heads] attention sinks (natural-log logits) or nullptr
  const float* alibi; // [num_q_heads] ALiBi slopes or nullptr: logit += slope * (key position - query position)
  float cap_c;        // logits soft cap in the log2 domain, cap * log2(e); 0 = none
  float cap_k;        // 2 * log2(e) / cap_c
};

// cap * tanh(x / cap) for a log2-domain logit x.  Away from zero tanh(u) = 1 - 2 / (exp(2u) + 1), which
// saturates cleanly at +-cap but whose absolute error is about cap * 2^-23 whatever x is; for |u| < 1/8
// the odd series u (1 - u^2/3 + 2 u^4/15) takes over (next term 17/315 u^6 < 2e-7), so the result is
// accurate RELATIVE to x for every cap, and a cap far above the logits is the identity.
__device__ __forceinline__ float soft_cap(float x, float cap_c, float cap_k) {
  const float big = cap_c - 2.0f * cap_c * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x * cap_k) + 1.0f);
  const float u = x * cap_k * 0.34657359f;  // x / cap_c: cap_k = 2 log2(e) / cap_c
  const float u2 = u * u;
  const float small = x * (1.0f + u2 * (-0.33333334f + u2 * 0.13333334f));
  return fabsf(u) < 0.125f ? small : big;
}

// First token a decode row of a `len`-token sequence sees.
__device__ __forceinline__ int window_first(int len, int window) {
  return window > 0 && len > window ? len - window : 0;
}

// The sink's share of a head's softmax sum: exp(sink - max) with the running maximum `m` in the log2 domain
// (0 without sinks).  Added once, where a row's sum is final.
__device__ __forceinline__ float sink_term(const float* sinks, int head, float m) {
  return sinks != nullptr ? __builtin_amdgcn_exp2f(sinks[head] * kLog2e - m) : 0.f;
}

// A head's ALiBi slope in the log2 domain (0 without ALiBi).
__device__ __forceinline__ float alibi_slope(const float* alibi, int head) {
  return alibi != nullptr ? alibi[head] * kLog2e : 0.f;
}

// One lane's share of a 32-token tile as it arrives from HBM: raw 16-byte chunks of records.
template <int D>
struct KVTile {
  static constexpr int NCH = D / 8;        // full 16-byte chunks per record (2*D bytes)
  static constexpr int NLD = NCH / 4;      // wave-wide chunk loads per 16-token half
  u32x4 c[2][NLD];                         // chunk (n*64 + lane) of half 0 / half 1
  u32x2 tail0, tail1;                      // last 8 bytes of record (lane & 15) of half 0 / half 1
  u32x4 e[2];                              // streamed loads only: chunk NLD*64 + (lane & 7), the run's last 128 bytes
};

template <int D>
struct DecodeState {
  static constexpr int DT = D / 16;  // M-tiles of the O^T accumulator
  floatx4 o[DT];   // sum_t P~[t] * (code + 1152)
  floatx4 psum;    // sum_t P~[t] (every register the same), to take the 1152 out again
  float m;         // running max, log2 domain (uniform across the 4 lane groups of a head)
  float l;         // lane-local partial sum of p
};

// Physical blocks of the two 16-token halves of a tile.  They are read with scalar loads
// (uniform address, constant address space), which do not share a counter with the vector
// loads of the KV stream, and well ahead of their use, so the pointer chase through the
// block table never drains the prefetched tiles.
struct TileBlocks {
  int32_t b0, b1;
  int32_t s1_same;  // 1: the second half lies past the sequence end and rereads the first
};

typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;

__device__ __forceinline__ int32_t scalar_load_i32(const int32_t* p, int64_t i) {
  return reinterpret_cast<const_i32_ptr>(reinterpret_cast<uintptr_t>(p))[i];
}

// Loop-invariant per-lane offsets.
struct LaneOffsets {
  uint32_t g_chunk;   // HBM: (lane / NCH)*stride_slot + 16*(lane % NCH), chunk `lane` of a half
  uint32_t g_tail;    // HBM: (lane & 15)*stride_slot + 2*D, the record's last 8 bytes
  uint32_t l_chunk;   // LDS: (lane / NCH)*PITCH + 16*(lane % NCH)
  uint32_t l_tail;    // LDS: (lane & 31)*PITCH + 2*D
  uint32_t l_k;       // LDS: r*PITCH + g*16, K operand chunk of token r
  uint32_t l_v;       // LDS: 4g*PITCH + (D+4) + r*VB, V operand bytes of token 4g
  uint32_t l_sc;      // LDS: (lane & 31)*PITCH + (lane < 32 ? D : 2*D+4), the lane's scale
  // streamed loads: where the 16-byte chunk n*64 + lane of a 16-record run lands in the window (its first 8
  // bytes; the other 8 follow, or open the next row when bit n of l_flat_split is set)
  uint32_t g_flat;    // HBM: 16 * lane
  uint32_t l_flat[9];
  uint32_t l_flat_split;
};

// CODE: what a code byte is (KVQ_CODE_INT8 or KVQ_CODE_FP8_E4M3).  An int8 code enters the MFMA as
// code + 1152 and the constant is taken out afterwards; an fp8 code enters as its value / 2^8 (exact in
// fp16) and the 2^8 is put back with the K scale, while on the V side it cancels the 2^8 that P~ carries.
template <int D, int QDT, int ODT, int CODE = KVQ_CODE_INT8>
struct DecodeTile {
  static constexpr bool FP8 = CODE == KVQ_CODE_FP8_E4M3;
  // int4 codes: a record of head size D has the bytes of an int8 record of head size D / 2, so the tile is loaded
  // and staged as that one; only the operand conversions and the query's dim order differ
  static constexpr bool INT4 = CODE == KVQ_CODE_INT4;
  static constexpr int DB = INT4 ? D / 2 : D;                 // code bytes of a half record
  static constexpr float kBias = INT4 ? kCodeBiasInt4 : kCodeBias;
  static constexpr float kKScaleMul = FP8 ? 256.0f : 1.0f;   // on top of scale * log2(e)
  static constexpr float kOutDiv = FP8 ? 1.0f : kPScale;      // what the accumulated output still carries
  static constexpr int KSTEPS = D / 32;
  static constexpr int DT = D / 16;
  static constexpr int VB = DB / 16;  // V bytes per token per lane
  using Tile = KVTile<DB>;
  using State = DecodeState<D>;

  static constexpr int R = 2 * (DB + 4);     // record bytes
  static constexpr int PITCH = R + 8;        // LDS row pitch: 16-byte aligned rows, conflict-free operand reads
  static constexpr int NCH = Tile::NCH;
  static constexpr int NLD = Tile::NLD;
  static constexpr int LDS_TILE = kTile * PITCH;          // bytes of the record window
  static constexpr int LDS_STATE = (DT + 1) * 1024;       // a wave's softmax state, dumped for a merge inside the workgroup
  static constexpr int LDS_WAVE = LDS_TILE + 64 * 4 > LDS_STATE ? LDS_TILE + 64 * 4 : LDS_STATE;  // window + 64 staged scales

  __device__ static LaneOffsets lane_offsets(const kvq_cache_geom& G, int lane) {
    const int r = lane & 15, g = lane >> 4;
    LaneOffsets o;
    o.g_chunk = (uint32_t)((lane / NCH) * G.stride_slot + 16 * (lane % NCH));
    o.g_tail = (uint32_t)((lane & 15) * G.stride_slot + 2 * DB);
    o.l_chunk = (uint32_t)((lane / NCH) * PITCH + 16 * (lane % NCH));
    o.l_tail = (uint32_t)((lane & 31) * PITCH + 2 * DB);
    o.l_k = (uint32_t)(r * PITCH + (INT4 ? g * (DB / 4) : g * 16));   // int4: the lane's D / 4 dims are DB / 4 bytes in a row
    o.l_v = (uint32_t)(4 * g * PITCH + (DB + 4) + r * VB);
    o.l_sc = (uint32_t)((lane & 31) * PITCH + (lane < 32 ? DB : 2 * DB + 4));
    o.g_flat = (uint32_t)(16 * lane);
    o.l_flat_split = 0;
#pragma unroll
    for (int n = 0; n <= NLD; ++n) {
      const int q = n < NLD ? n * 64 + lane : NLD * 64 + (lane & 7);   // chunk of the run
      const int rec = (16 * q) / R, off = 16 * q - rec * R;            // its record and the offset inside it
      o.l_flat[n] = (uint32_t)(rec * PITCH + off);
      if (off == R - 8) o.l_flat_split |= 1u << n;
    }
    return o;
  }

  // ---- Q as the MFMA B operand --------------------------------------------------------------
  // Lane (c = head in group, g) holds, for k-step kk, dims (kk>>1)*64 + g*16 + (kk&1)*8 + j:
  // the same dim order in which a K lane holds its code bytes.  Lanes past the group reread
  // head 0 and are zeroed.  Returns -1152 * sum(q) of the lane's head: the QK accumulator's
  // start value that cancels the code bias.
  __device__ static float load_q(const AttnIO& io, int64_t row, int hkv, int lane, half8_t (&qb)[KSTEPS]) {
    const int c = lane & 15;
    const bool valid = c < io.group;
    return load_q_row(io, row * io.q_stride_t + (int64_t)(hkv * io.group + (valid ? c : 0)) * io.q_stride_h, valid,
                      lane, qb);
  }

  // The same for an arbitrary (row, head) per lane: `elem` is the element offset of the lane's
  // query row (it must be readable also when !valid; the operand is then zero).
  __device__ static float load_q_row(const AttnIO& io, int64_t elem, bool valid, int lane, half8_t (&qb)[KSTEPS]) {
    const int g = lane >> 4;
    // int8 / fp8: 16 dims of every 64-dim chunk; int4: the D / 4 dims from g D / 4 on, in a row (the same loads,
    // chunk `ch` then standing for the ch-th run of 16 of them)
    constexpr int kChunkStep = INT4 ? 16 : 64;
    const int64_t base = elem + (INT4 ? g * (D / 4) : g * 16);
    float f[D / 4];
#pragma unroll
    for (int ch = 0; ch < D / 64; ++ch) {
      if constexpr (QDT == KVQ_F32) {
        const float* p = reinterpret_cast<const float*>(io.q) + base + ch * kChunkStep;
#pragma unroll
        for (int i = 0; i < 16; i += 4) {
          const floatx4 v = *reinterpret_cast<const floatx4_a4*>(p + i);
          f[ch * 16 + i] = v.x; f[ch * 16 + i + 1] = v.y; f[ch * 16 + i + 2] = v.z; f[ch * 16 + i + 3] = v.w;
        }
      } else {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(io.q) + base + ch * kChunkStep;
#pragma unroll
        for (int i = 0; i < 16; i += 8) {
          const u32x4 v = *reinterpret_cast<const u32x4_a4*>(p + i);
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            if constexpr (QDT == KVQ_BF16) {
              f[ch * 16 + i + 2 * w] = as_f32(v[w] << 16);
              f[ch * 16 + i + 2 * w + 1] = as_f32(v[w] & 0xffff0000u);
            } else {
              const uint32_t e = v[w];  // copy the element out first: bit_cast must not see a vector element lvalue
              const half2_t h = __builtin_bit_cast(half2_t, e);
              f[ch * 16 + i + 2 * w] = (float)h.x;
              f[ch * 16 + i + 2 * w + 1] = (float)h.y;
            }
          }
        }
      }
    }
    float qsum = 0.f;
    const uint32_t okmask = valid ? 0xffffffffu : 0u;  // a mask, not a select: no branches around the converts
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      const int b = INT4 ? kk * 8 : (kk >> 1) * 16 + (kk & 1) * 8;
      u32x4 hb;
      if constexpr (INT4) {   // the k positions follow the nibble conversion's dim order
        hb.x = pack_half2(clamp_half_range(f[b + nibble_order(0)]), clamp_half_range(f[b + nibble_order(1)])) & okmask;
        hb.y = pack_half2(clamp_half_range(f[b + nibble_order(2)]), clamp_half_range(f[b + nibble_order(3)])) & okmask;
        hb.z = pack_half2(clamp_half_range(f[b + nibble_order(4)]), clamp_half_range(f[b + nibble_order(5)])) & okmask;
        hb.w = pack_half2(clamp_half_range(f[b + nibble_order(6)]), clamp_half_range(f[b + nibble_order(7)])) & okmask;
      } else {
      hb.x = pack_half2(clamp_half_range(f[b + 0]), clamp_half_range(f[b + 1])) & okmask;
      hb.y = pack_half2(clamp_half_range(f[b + 2]), clamp_half_range(f[b + 3])) & okmask;
      hb.z = pack_half2(clamp_half_range(f[b + 4]), clamp_half_range(f[b + 5])) & okmask;
      hb.w = pack_half2(clamp_half_range(f[b + 6]), clamp_half_range(f[b + 7])) & okmask;
      }
      const half8_t h = __builtin_bit_cast(half8_t, hb);
#pragma unroll
      for (int j = 0; j < 8; ++j) qsum += (float)h[j];  // the sum of what the MFMA will actually see
      qb[kk] = h;
    }
    qsum += __shfl_xor(qsum, 16, kWave);
    qsum += __shfl_xor(qsum, 32, kWave);
    return FP8 ? 0.f : -kBias * qsum;
  }

  // The KSTEPS operands of K tokens (M-tile mt) of the lane, int4 codes: DB / 4 bytes in a row, a dword per k-step.
  __device__ static void k_operands_int4(const LaneOffsets& lo, int mt, const uint8_t* lds, half8_t (&ka)[KSTEPS]) {
    const uint8_t* p = lds + lo.l_k + mt * 16 * PITCH;
    if constexpr (KSTEPS == 2) {
      const u32x2 w = *reinterpret_cast<const u32x2*>(p);
      ka[0] = dequant8_int4(w.x);
      ka[1] = dequant8_int4(w.y);
    } else {
#pragma unroll
      for (int i = 0; i < KSTEPS / 4; ++i) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(p + 16 * i);
        ka[4 * i] = dequant8_int4(w.x);
        ka[4 * i + 1] = dequant8_int4(w.y);
        ka[4 * i + 2] = dequant8_int4(w.z);
        ka[4 * i + 3] = dequant8_int4(w.w);
      }
    }
  }

  // The V^T operands of the lane's 8 tokens for the four 16-dim tiles that two code bytes hold (unit u = bytes
  // 2 u, 2 u + 1 of the lane's VB: dims 4 u .. 4 u + 3 of its 2 VB, tile 4 u + n = nibble n), int4 codes.
  __device__ static void v_operands_int4(const LaneOffsets& lo, int u, const uint8_t* lds, half8_t (&va)[4]) {
    uint32_t y[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int ja = 2 * a, jb = 2 * a + 1;
      const uint8_t* pa = lds + lo.l_v + ((ja & 3) + (ja >> 2) * 16) * PITCH + 2 * u;
      const uint8_t* pb = lds + lo.l_v + ((jb & 3) + (jb >> 2) * 16) * PITCH + 2 * u;
      const uint32_t ta = *reinterpret_cast<const uint16_t*>(pa), tb = *reinterpret_cast<const uint16_t*>(pb);
      y[a] = (ta | (tb << 16)) ^ 0x88888888u;   // token ja's two bytes below token jb's
    }
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      u32x4 av;
      av.x = nibbles_to_half2(y[0], n);
      av.y = nibbles_to_half2(y[1], n);
      av.z = nibbles_to_half2(y[2], n);
      av.w = nibbles_to_half2(y[3], n);
      va[n] = __builtin_bit_cast(half8_t, av);
    }
  }

  // Token index -> block-table entry / slot, by multiplication (scalar ALU, no divide).
  __device__ static int div_bs(const AttnIO& io, int x) { return (int)__umulhi((uint32_t)x, io.bs_magic); }
  __device__ static int mod_bs(const AttnIO& io, int x) { return x - div_bs(io, x) * io.g.block_size; }

  // Block-table entries of tile `t` (clamped into the sequence so the read is always valid).
  __device__ static TileBlocks fetch_blocks(const AttnIO& io, const int32_t* bt_row, int len, int t) {
    const int num_entries = div_bs(io, len + io.g.block_size - 1);
    const int tok0 = t * kTile;
    int e0 = div_bs(io, tok0);
    e0 = e0 < num_entries ? e0 : num_entries - 1;
    const int e1raw = div_bs(io, tok0 + 16);
    const int e1 = e1raw < num_entries ? e1raw : num_entries - 1;
    TileBlocks tb;
    tb.b0 = scalar_load_i32(bt_row, e0);
    tb.b1 = scalar_load_i32(bt_row, e1);
    tb.s1_same = e1raw < num_entries ? 0 : 1;
    return tb;
  }

  // Buffer resources (scalar registers) of the two 16-token halves of tile `t` for kv head
  // `hkv`, based at the first record of each half: every load of the tile is "resource + fixed
  // 32-bit lane offset + scalar offset", no vector address arithmetic, no address registers.
  struct Window {
    __amdgpu_buffer_rsrc_t r0, r1;
  };
  __device__ static Window window(const AttnIO& io, const TileBlocks& tb, int t, int hkv) {
    const kvq_cache_geom& G = io.g;
    const int tok0 = t * kTile;
    // a 16-token half never straddles a block (block_size is a multiple of 16); a second half
    // past the end of the sequence rereads the first half and is masked in compute
    const int s0 = mod_bs(io, tok0);
    const int s1 = tb.s1_same ? s0 : mod_bs(io, tok0 + 16);
    // strides are below 2^31 (checked on the host): block number x block stride is one 32 x 32 -> 64 bit
    // multiply, the offset inside the block stays in 32 bits
    const uint8_t* head = io.cache + G.k_off + (uint64_t)((uint32_t)hkv * (uint32_t)G.stride_head);
    const uint32_t sb = (uint32_t)G.stride_block, ss = (uint32_t)G.stride_slot;
    const uint8_t* p0 = head + (uint64_t)(uint32_t)tb.b0 * sb + (uint32_t)s0 * ss;
    const uint8_t* p1 = head + (uint64_t)(uint32_t)tb.b1 * sb + (uint32_t)s1 * ss;
    Window w;
    w.r0 = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p0), 0, 0x7fffffff, 0x00020000);
    w.r1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p1), 0, 0x7fffffff, 0x00020000);
    return w;
  }

  // Issue the HBM loads of one tile: 2*NLD chunk loads (lane n*64+l takes chunk (n*64+l) % NCH of
  // record (n*64+l) / NCH of the half) and the two 8-byte record tails.
  // STREAM: for a cache in which a head's records of a block lie back to back (the HND order).  A half
  // tile is then ONE run of 16 R bytes, read as aligned 16-byte chunks with the non-temporal hint (scales
  // included: no 8-byte tail loads) -- measured on MI355X, reads of this shape reach 6.8 TB/s against 6.0
  // without the hint.  The hint is wrong for the NHD order: there the 128-byte lines at a record's ends
  // belong half to a neighbouring head's wave, a line that is not kept in L2 is fetched by both, and the
  // rate drops by 9 %.
  template <bool STREAM = false>
  __device__ static void load_tile(const AttnIO& io, const Window& w, const LaneOffsets& lo, Tile& kv) {
    constexpr int AUX = STREAM ? 2 : 0;
    if constexpr (STREAM) {
      // the half's 16 records are one run of 16 R bytes: read it as R aligned 16-byte chunks, scales and all
      // (NLD full wave-loads and the last 8 chunks, which every lane names so that the load is unconditional)
      const uint32_t f = lo.g_flat;
#pragma unroll
      for (int n = 0; n < NLD; ++n) {
        kv.c[0][n] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r0, f, n * 1024, AUX));
        kv.c[1][n] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r1, f, n * 1024, AUX));
      }
      const uint32_t fe = (f & 127u) + NLD * 1024;
      kv.e[0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r0, fe, 0, AUX));
      kv.e[1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r1, fe, 0, AUX));
      return;
    }
    const int step = (64 / NCH) * (int)io.g.stride_slot;  // records advanced per wave-wide load
#pragma unroll
    for (int n = 0; n < NLD; ++n) {
      kv.c[0][n] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r0, lo.g_chunk, n * step, AUX));
      kv.c[1][n] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r1, lo.g_chunk, n * step, AUX));
    }
    kv.tail0 = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(w.r0, lo.g_tail, 0, AUX));
    kv.tail1 = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(w.r1, lo.g_tail, 0, AUX));
  }

  // Drop a loaded tile into the wave's LDS window, one record per PITCH-byte row, then stage the
  // 64 scales (K scales pre-multiplied by scale*log2e, V scales by 2^8, capped so P~ stays finite).
  // After this the tile's registers are free for the next prefetch.
  template <bool STREAM = false>
  __device__ static void stage(const Tile& kv, const LaneOffsets& lo, float sc_mul, int lane, uint8_t* lds) {
    if constexpr (STREAM) {
      // a chunk of the run is 8-byte aligned inside its record and may end one record and begin the next:
      // two 8-byte writes each
      auto put = [&](const u32x4& v, uint32_t at, bool split) __attribute__((always_inline)) {
        *reinterpret_cast<u32x2*>(lds + at) = (u32x2){v.x, v.y};
        *reinterpret_cast<u32x2*>(lds + at + (split ? 8 + (PITCH - R) : 8)) = (u32x2){v.z, v.w};
      };
#pragma unroll
      for (int n = 0; n < NLD; ++n) {
        const bool split = (lo.l_flat_split >> n) & 1;
        put(kv.c[0][n], lo.l_flat[n], split);
        put(kv.c[1][n], lo.l_flat[n] + 16 * PITCH, split);
      }
      if (lane < 8) {
        const bool split = (lo.l_flat_split >> NLD) & 1;
        put(kv.e[0], lo.l_flat[NLD], split);
        put(kv.e[1], lo.l_flat[NLD] + 16 * PITCH, split);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      stage_scales(lo, sc_mul, lane, lds);
      return;
    }
#pragma unroll
    for (int n = 0; n < NLD; ++n) {
      *reinterpret_cast<u32x4*>(lds + lo.l_chunk + n * (64 / NCH) * PITCH) = kv.c[0][n];
      *reinterpret_cast<u32x4*>(lds + lo.l_chunk + (16 + n * (64 / NCH)) * PITCH) = kv.c[1][n];
    }
    if (lane < 32) *reinterpret_cast<u32x2*>(lds + lo.l_tail) = (lane & 16) ? kv.tail1 : kv.tail0;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    stage_scales(lo, sc_mul, lane, lds);
  }

  // The 64 scales of the window's 32 records, multiplied and capped, in the 256 bytes behind it.
  __device__ static void stage_scales(const LaneOffsets& lo, float sc_mul, int lane, uint8_t* lds) {
    const float sc = *reinterpret_cast<const float*>(lds + lo.l_sc);
    reinterpret_cast<float*>(lds + LDS_TILE)[lane] = fminf(sc * sc_mul, 65504.f);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }

  // Phase 1 of a tile: S^T = K . Q^T on the MFMA from the LDS window, online softmax.  Returns
  // P~^T as the MFMA B operand.  MASK: the tile holds the end of the sequence (tokens >= len must
  // not contribute).
  // CAP: logits pass through the soft cap (the identity when cap_c = cap_k = 0) and take the ALiBi bias
  // `ali` x (token - (len - 1)) of the lane's head (the query of a decode row stands at len - 1).
  // Tokens outside [first, len) never contribute.
  template <bool MASK, bool CAP>
  __device__ static half8_t qk_softmax(const AttnIO& io, const LaneOffsets& lo, const half8_t (&qb)[KSTEPS], float s_init,
                                       int len, int first, int t, int lane, const uint8_t* lds, State& st, float ali) {
    const int g = lane >> 4;
    const float* sc_lds = reinterpret_cast<const float*>(lds + LDS_TILE);
    const floatx4 ks0 = *reinterpret_cast<const floatx4*>(sc_lds + 4 * g);
    const floatx4 ks1 = *reinterpret_cast<const floatx4*>(sc_lds + 16 + 4 * g);

    // two 16-token M-tiles, KSTEPS k-steps each; accumulators start at -1152 * sum(q)
    floatx4 s[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      s[mt] = (floatx4){s_init, s_init, s_init, s_init};
      if constexpr (INT4) {
        half8_t ka[KSTEPS];
        k_operands_int4(lo, mt, lds, ka);
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) s[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[kk], qb[kk], s[mt], 0, 0, 0);
      } else {
#pragma unroll
      for (int i = 0; i < KSTEPS / 2; ++i) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(lds + lo.l_k + mt * 16 * PITCH + i * 64);
        s[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(dequant8<FP8>(w.x, w.y), qb[2 * i], s[mt], 0, 0, 0);
        s[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(dequant8<FP8>(w.z, w.w), qb[2 * i + 1], s[mt], 0, 0, 0);
      }
      }
    }

    // softmax in the log2 domain; lane holds tokens 32t + mt*16 + 4g + i of head (lane & 15)
    float logit[8];
    const int tok_base = t * kTile + 4 * g;
    const float rel0 = (float)(tok_base - (len - 1));
    float mloc = -INFINITY;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float x = s[mt][i] * (mt ? ks1 : ks0)[i];
        if constexpr (CAP) x = __builtin_fmaf(ali, rel0 + (float)(mt * 16 + i), soft_cap(x, io.cap_c, io.cap_k));
        if constexpr (MASK) x = ((uint32_t)(tok_base + mt * 16 + i - first) < (uint32_t)(len - first)) ? x : -INFINITY;
        logit[mt * 4 + i] = x;
        mloc = fmaxf(mloc, x);
      }
    }
    mloc = max_over_quarters(mloc);
    if (__builtin_amdgcn_ballot_w64(mloc > st.m) != 0) {  // rescale only when some head's max moved
      const float m_new = fmaxf(st.m, mloc);
      const float alpha = __builtin_amdgcn_exp2f(st.m - m_new);  // st.m = -inf -> 0
      st.m = m_new;
      st.l *= alpha;
      st.psum *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) st.o[dt] *= alpha;
    }
    const floatx4 vs0 = *reinterpret_cast<const floatx4*>(sc_lds + 32 + 4 * g);
    const floatx4 vs1 = *reinterpret_cast<const floatx4*>(sc_lds + 48 + 4 * g);
    float pt[8];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = mt * 4 + i;
        const float p = __builtin_amdgcn_exp2f(logit[j] - st.m);  // masked: exp2(-inf) = 0
        st.l += p;
        float x = p * (mt ? vs1 : vs0)[i];
        if constexpr (MASK)  // garbage scales never enter
          x = ((uint32_t)(tok_base + mt * 16 + i - first) < (uint32_t)(len - first)) ? x : 0.f;
        pt[j] = x;
      }
    }
    u32x4 pb;
    pb.x = pack_half2(pt[0], pt[1]);
    pb.y = pack_half2(pt[2], pt[3]);
    pb.z = pack_half2(pt[4], pt[5]);
    pb.w = pack_half2(pt[6], pt[7]);
    return __builtin_bit_cast(half8_t, pb);
  }

  // Phase 2 of a tile: O^T += (V + 1152)^T . P~^T.  Lane (r, g) reads bytes [r*VB, (r+1)*VB) of
  // tokens 4g+j (j<4) and 16+4g+(j-4) from the LDS window, transposes the 8 x VB byte block in
  // registers (byte permutes), one MFMA per 16-dim tile; sum(P~) comes from a row of ones.
  __device__ static void pv(const LaneOffsets& lo, half8_t p_op, const uint8_t* lds, State& st) {
    if constexpr (!FP8) {  // fp8 codes carry no bias to take out again
      const half_t one = (half_t)1.0f;
      const half8_t ones = {one, one, one, one, one, one, one, one};
      st.psum = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, p_op, st.psum, 0, 0, 0);
    }
    if constexpr (INT4) {
#pragma unroll
      for (int u = 0; u < VB / 2; ++u) {
        half8_t va[4];
        v_operands_int4(lo, u, lds, va);
#pragma unroll
        for (int n = 0; n < 4; ++n)
          st.o[4 * u + n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[n], p_op, st.o[4 * u + n], 0, 0, 0);
      }
      return;
    }
    constexpr int VW = VB / 4;
#pragma unroll
    for (int w = 0; w < VW; ++w) {
      uint32_t x0[4], x1[4];  // per token pair a: bytes (b0,b1) and (b2,b3) of both tokens, interleaved
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int ja = 2 * a, jb = 2 * a + 1;
        const uint32_t ta = prep_codes<FP8>(*reinterpret_cast<const uint32_t*>(lds + lo.l_v + ((ja & 3) + (ja >> 2) * 16) * PITCH + 4 * w));
        const uint32_t tb = prep_codes<FP8>(*reinterpret_cast<const uint32_t*>(lds + lo.l_v + ((jb & 3) + (jb >> 2) * 16) * PITCH + 4 * w));
        x0[a] = perm(tb, ta, 0x05010400u);
        x1[a] = perm(tb, ta, 0x07030602u);
      }
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        u32x4 av;
        const uint32_t* x = (b < 2) ? x0 : x1;
        av.x = codes_to_half2<FP8>(x[0], b & 1);
        av.y = codes_to_half2<FP8>(x[1], b & 1);
        av.z = codes_to_half2<FP8>(x[2], b & 1);
        av.w = codes_to_half2<FP8>(x[3], b & 1);
        const int dt = 4 * w + b;
        st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, av), p_op, st.o[dt], 0, 0, 0);
      }
    }
  }

  template <bool MASK, bool CAP>
  __device__ static void compute(const AttnIO& io, const LaneOffsets& lo, const half8_t (&qb)[KSTEPS], float s_init, int len,
                                 int first, int t, int lane, const uint8_t* lds, State& st, float ali) {
    const half8_t p = qk_softmax<MASK, CAP>(io, lo, qb, s_init, len, first, t, lane, lds, st, ali);
    pv(lo, p, lds, st);
  }
  template <bool CAP>
  __device__ static void compute_any(const AttnIO& io, const LaneOffsets& lo, const half8_t (&qb)[KSTEPS], float s_init,
                                     int len, int first, int t, int lane, const uint8_t* lds, State& st, float ali) {
    if ((t + 1) * kTile > len || t * kTile < first) compute<true, CAP>(io, lo, qb, s_init, len, first, t, lane, lds, st, ali);
    else compute<false, CAP>(io, lo, qb, s_init, len, first, t, lane, lds, st, ali);
  }

  // Keeps the instruction scheduler from moving work across the phase boundaries of the
  // stream loop: a refill must be issued where it is written (right after the registers it
  // overwrites were consumed), and a tile's V conversion must not drift up into the QK phase,
  // where it would wait on the newest loads instead of the oldest.
  __device__ static __forceinline__ void phase_fence() { __builtin_amdgcn_sched_barrier(0); }

  // Run this wave's share of tiles [t_begin, t_end) of one sequence for kv head `hkv`; leaves the
  // state in `st`.  The `nsub` waves that serve one kv head take the tiles in turn: wave `sub` owns
  // tiles t_begin + sub, t_begin + sub + nsub, ... (one wave per kv head: nsub = 1, every tile).
  // One register buffer: as soon as a tile has been dropped into LDS its registers take the
  // wave's next tile, so one tile of loads per wave is in flight while one is computed (measured on
  // MI355X: a second tile in flight per wave lowers the achieved HBM bandwidth).
  // `lds` is this wave's private LDS_WAVE-byte window.
  // Tokens before `first` (the sliding window's lower edge; 0 without a window) do not contribute;
  // t_begin is then the tile that holds `first` or a later one.
  // Every wave of the workgroup must call this with the same (t_begin, t_end, nsub): the rendezvous
  // barriers inside are counted in rounds of nsub tiles, the same number for every wave, also for
  // one that owns no tile of the range (its state stays empty: m = -inf).
  // SPANS (one wave per kv head only: nsub = 1): the run covers several consecutive spans of `sp.per` tiles of the
  // batch-invariant cutting.  The tile stream -- query registers, block numbers, the tile in flight -- goes on across
  // a span's edge; there the state is stored as the span's partial state (slot sp.slot) and started afresh, so every
  // span's state holds exactly what a run over that span alone would have computed, in the same order.  The state of
  // the run's last span is left to the caller (sp.slot names it on return).
  struct SpanEdges {
    float* part_o;
    float* part_ml;
    int64_t slot;   // of the span the next tile belongs to
    int per;        // tiles per span
    int left;       // tiles of the current span still to come
  };
  __device__ static void reset_state(State& st) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) st.o[dt] = (floatx4){0.f, 0.f, 0.f, 0.f};
    st.psum = (floatx4){0.f, 0.f, 0.f, 0.f};
    st.m = -INFINITY;
    st.l = 0.f;
  }
  template <bool CAP, bool STREAM = false, bool SPANS = false>
  __device__ static void run(const AttnIO& io, int seq, int64_t row, int len, int first, int t_begin, int t_end, int hkv,
                             int lane, uint8_t* lds, State& st, int sub = 0, int nsub = 1, SpanEdges* sp = nullptr) {
    const LaneOffsets lo = lane_offsets(io.g, lane);
    const int32_t* bt_row = io.block_table + (int64_t)seq * io.bt_stride;
    const int rounds = (t_end - t_begin + nsub - 1) / nsub;
    const int num_barriers = STREAM ? 0 : rounds / kSyncTiles;
    int barriers = 0;
    reset_state(st);
    auto span_edge = [&]() __attribute__((always_inline)) {
      if constexpr (SPANS) {
        if (--sp->left == 0) {   // uniform over the wave
          emit_partial(io, sp->part_o, sp->part_ml, sp->slot, hkv, lane, st);
          reset_state(st);
          ++sp->slot;
          sp->left = sp->per;
        }
      }
    };
    int t = t_begin + sub;
    if (t < t_end) {
      Tile a;
      // the first tile's loads go out before anything else of the run is touched
      TileBlocks nb = fetch_blocks(io, bt_row, len, t);
      load_tile<STREAM>(io, window(io, nb, t, hkv), lo, a);
      phase_fence();
      nb = fetch_blocks(io, bt_row, len, t + nsub);  // block ids run one tile ahead of the loads
      half8_t qb[KSTEPS];
      const float s_init = load_q(io, row, hkv, lane, qb);
      const float sc_mul = lane < 32 ? io.scale_log2 * kKScaleMul : kPScale;
      float ali = 0.f;
      if constexpr (CAP) ali = alibi_slope(io.alibi, hkv * io.group + min(lane & 15, io.group - 1));
      int r = 0;  // rounds this wave has finished
      // a first tile that straddles the window's lower edge is masked; it is peeled off so that the
      // steady loop below keeps a single, unmasked body
      if (t + nsub < t_end && t * kTile < first) {
        const Window w = window(io, nb, t + nsub, hkv);
        stage<STREAM>(a, lo, sc_mul, lane, lds);
        phase_fence();
        load_tile<STREAM>(io, w, lo, a);
        phase_fence();
        nb = fetch_blocks(io, bt_row, len, t + 2 * nsub);
        compute<true, CAP>(io, lo, qb, s_init, len, first, t, lane, lds, st, ali);
        phase_fence();
        span_edge();
        t += nsub;
        ++r;
        if (!STREAM && (r & (kSyncTiles - 1)) == 0) {
          __builtin_amdgcn_s_barrier();
          ++barriers;
        }
      }
      auto rendezvous = [&]() __attribute__((always_inline)) {
        ++r;
        // The waves of a workgroup read neighbouring records of the same tokens (one kv head each) or
        // neighbouring tiles; the 128-byte lines at record boundaries are shared between them.  A
        // rendezvous every few rounds keeps the waves within a few tiles of each other, so the second
        // reader of such a line still finds it in L2 instead of fetching it from HBM again.  Streamed loads
        // (whole runs per wave, nothing kept in L2) have no such lines to share and skip the rendezvous.
        if (!STREAM && (r & (kSyncTiles - 1)) == 0) {
          __builtin_amdgcn_s_barrier();
          ++barriers;
        }
      };
      // steady state: the wave's next tile exists, so the refill is unconditional and tile t does not
      // end the sequence
      while (t + nsub < t_end) {
        const Window w = window(io, nb, t + nsub, hkv);
        stage<STREAM>(a, lo, sc_mul, lane, lds);
        phase_fence();
        load_tile<STREAM>(io, w, lo, a);
        phase_fence();
        nb = fetch_blocks(io, bt_row, len, t + 2 * nsub);
        compute<false, CAP>(io, lo, qb, s_init, len, first, t, lane, lds, st, ali);
        phase_fence();
        span_edge();
        t += nsub;
        rendezvous();
      }
      stage<STREAM>(a, lo, sc_mul, lane, lds);
      compute_any<CAP>(io, lo, qb, s_init, len, first, t, lane, lds, st, ali);
    }
    // the rendezvous count is the same for every wave of the workgroup, whatever its share of the tiles
    for (; barriers < num_barriers; ++barriers) __builtin_amdgcn_s_barrier();
  }

  // ---- several waves per kv head: their states meet in LDS ------------------------------------
  // Every wave but the head's first drops its state into its own LDS window (free once its tiles are
  // done); after a workgroup barrier the first wave folds them into its own, in wave order.
  __device__ static void dump_state(const State& st, int lane, uint8_t* lds) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<floatx4*>(lds + (dt * 64 + lane) * 16) = st.o[dt];
    *reinterpret_cast<floatx4*>(lds + (DT * 64 + lane) * 16) = (floatx4){st.psum[0], st.m, st.l, 0.f};
  }
  __device__ static void fold_state(State& st, int lane, const uint8_t* lds) {
    const floatx4 x = *reinterpret_cast<const floatx4*>(lds + (DT * 64 + lane) * 16);
    const float mj = x.y;
    const float m_new = fmaxf(st.m, mj);
    // both states hold at least one token, so m_new is finite
    const float a = __builtin_amdgcn_exp2f(st.m - m_new);
    const float b = __builtin_amdgcn_exp2f(mj - m_new);
    st.m = m_new;
    st.l = st.l * a + x.z * b;
    st.psum = st.psum * a + x.x * b;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      st.o[dt] = st.o[dt] * a + *reinterpret_cast<const floatx4*>(lds + (dt * 64 + lane) * 16) * b;
  }

  // Sum of the lane-local l over the 4 lane groups of a head.
  __device__ static float total_l(const State& st) {
    float l = st.l;
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    return l;
  }

  // Lane (c, g) holds O[head c][dim (4g+i)*DT + dt], i = 0..3, dt = 0..DT-1: D/4 contiguous
  // dims starting at g*D/4.  Gather them in order, code bias removed, scaled by `mul`.
  __device__ static void gather_row(const State& st, float mul, float (&v)[D / 4]) {
    const float corr = FP8 ? 0.f : kBias * st.psum[0];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) v[i * DT + dt] = (st.o[dt][i] - corr) * mul;
  }

  // Whole sequence handled by this wave: normalise and write the output row (and lse).
  __device__ static void emit_final(const AttnIO& io, int64_t row, int hkv, int lane, const State& st) {
    if constexpr (ODT == kRuntimeDtype) {
      if (io.out_dtype == KVQ_F32) emit_final_as<KVQ_F32>(io, row, hkv, lane, st);
      else if (io.out_dtype == KVQ_BF16) emit_final_as<KVQ_BF16>(io, row, hkv, lane, st);
      else emit_final_as<KVQ_F16>(io, row, hkv, lane, st);
    } else {
      emit_final_as<ODT>(io, row, hkv, lane, st);
    }
  }
  template <int OT>
  __device__ static void emit_final_as(const AttnIO& io, int64_t row, int hkv, int lane, const State& st) {
    float l = total_l(st);  // every lane takes part in the shuffles
    const int c = lane & 15, g = lane >> 4;
    if (c >= io.group) return;
    const int head = hkv * io.group + c;
    l += sink_term(io.sinks, head, st.m);
    float v[D / 4];
    gather_row(st, 1.0f / (l * kOutDiv), v);
    const int64_t base = row * io.out_stride_t + (int64_t)head * io.out_stride_h + g * (D / 4);
    if constexpr (OT == KVQ_F32) {
      float* o = reinterpret_cast<float*>(io.out) + base;
#pragma unroll
      for (int i = 0; i < D / 4; i += 4) *reinterpret_cast<floatx4_a4*>(o + i) = (floatx4){v[i], v[i + 1], v[i + 2], v[i + 3]};
    } else {
      uint16_t* o = reinterpret_cast<uint16_t*>(io.out) + base;
#pragma unroll
      for (int i = 0; i < D / 4; i += 8) {
        u32x4 pk;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t w;
          if constexpr (OT == KVQ_BF16) {
            w = (uint32_t)f32_to_bf16_bits(v[i + 2 * j]) | ((uint32_t)f32_to_bf16_bits(v[i + 2 * j + 1]) << 16);
          } else {
            w = pack_half2(v[i + 2 * j], v[i + 2 * j + 1]);
          }
          pk[j] = w;
        }
        *reinterpret_cast<u32x4_a4*>(o + i) = pk;
      }
    }
    if (io.lse != nullptr && g == 0)
      io.lse[row * io.num_q_heads + head] = (st.m + __builtin_amdgcn_logf(l)) * kLn2;
  }

  // Part of a sequence: store the unnormalised state (o, m in log2 domain, l) in fp32.
  __device__ static void emit_partial(const AttnIO& io, float* part_o, float* part_ml, int64_t slot, int hkv,
                                      int lane, const State& st) {
    const float l = total_l(st);
    const int c = lane & 15, g = lane >> 4;
    if (c >= io.group) return;
    const int head = hkv * io.group + c;
    float v[D / 4];
    gather_row(st, 1.0f / kOutDiv, v);
    float* o = part_o + (slot * io.num_q_heads + head) * (int64_t)D + g * (D / 4);
#pragma unroll
    for (int i = 0; i < D / 4; i += 4) *reinterpret_cast<floatx4*>(o + i) = (floatx4){v[i], v[i + 1], v[i + 2], v[i + 3]};
    if (g == 0) {
      part_ml[(slot * io.num_q_heads + head) * 2 + 0] = st.m;
      part_ml[(slot * io.num_q_heads + head) * 2 + 1] = l;
    }
  }

  // Fixed-partition contract: locally normalised output, natural-log max logit, exp-sum.
  __device__ static void emit_v2(const AttnIO& io, float* tmp_out, float* max_logits, float* exp_sums,
                                 int64_t seq, int part, int max_parts, int hkv, int lane, const State& st) {
    const float l = total_l(st);
    const int c = lane & 15, g = lane >> 4;
    if (c >= io.group) return;
    const int head = hkv * io.group + c;
    float v[D / 4];
    gather_row(st, 1.0f / (l * kOutDiv), v);
    const int64_t idx = (seq * io.num_q_heads + head) * (int64_t)max_parts + part;
    float* o = tmp_out + idx * D + g * (D / 4);
#pragma unroll
    for (int i = 0; i < D / 4; i += 4) *reinterpret_cast<floatx4*>(o + i) = (floatx4){v[i], v[i + 1], v[i + 2], v[i + 3]};
    if (g == 0) {
      max_logits[idx] = st.m * kLn2;
      exp_sums[idx] = l;
    }
  }
};

// Arguments of the balanced split-K decode launch (main kernel + reduce).
struct StreamKArgs {
  AttnIO io;
  const int32_t* seq_lens;
  const int32_t* cu_seqlens_q;  // nullptr: row i belongs to sequence i
  float* part_o;                // [(P + B), Hq, D]
  float* part_ml;               // [(P + B), Hq, 2]
  // [2 P + 2], what the main kernel leaves for the reduce kernel, whose waves would otherwise each rescan all
  // sequence lengths: [0] = length of the work line; [2 w + 2], [2 w + 3] = the sequence that holds workgroup w's
  // first unit and that sequence's own first unit (workgroups without a share write nothing).
  int64_t* wg_info;
  int64_t* seq_first_unit;      // [B]: the first unit of every decode sequence that has a tile (same purpose)
  int num_seqs;
  int num_wg;  // P
  // Fused write of the step's new tokens (decode rows only; k_new == nullptr: the cache already holds them):
  // row i of k_new / v_new is the token at position seq_lens[i] - 1 of sequence i.
  const void* k_new;
  const void* v_new;
  int64_t kn_stride_t, kn_stride_h, vn_stride_t, vn_stride_h;  // elements
  int new_dtype;
  float new_eps;
  const int64_t* new_slots;  // the step's slot mapping or nullptr: a row with a negative entry is padding, not written
  // != 0: the batch-invariant cutting (every sequence cut by its own length alone); the partial states then take
  // kFixedSpans slots per sequence and wg_info / seq_first_unit are not used
  int fixed_spans;
  int setup_units;   // units a sequence is charged on the balanced work line before its tiles
};

// The decode kernel's fused cache update: the wave that owns kv head `hkv` of the run that holds a sequence's
// LAST tile quantises that sequence's new K and V rows (the arithmetic of the write kernel, quant_row8) into
// the record at position len - 1 before it streams the run's tiles.  D / 8 lanes per row: lanes
// [0, D/8) take the K row, [D/8, D/4) the V row; the rest repeat them and store nothing.
template <int D>
__device__ __forceinline__ void write_new_token(const StreamKArgs& a, int seq, int64_t row, int len, int hkv, int lane) {
  constexpr int LPR = D / 8;
  const kvq_cache_geom& g = a.io.g;
  const int is_v = (lane / LPR) & 1;
  const int li = lane % LPR;
  const void* src = is_v ? a.v_new : a.k_new;
  const int64_t elem = (is_v ? row * a.vn_stride_t + (int64_t)hkv * a.vn_stride_h
                             : row * a.kn_stride_t + (int64_t)hkv * a.kn_stride_h) + li * 8;
  float x[8];
  load_row8(src, a.new_dtype, elem, x);
  uint32_t pk[2];
  float scale;
  quant_row8<LPR>(x, a.new_eps, g.code_type, pk, scale);
  const int pos = len - 1;
  const int e = (int)__umulhi((uint32_t)pos, a.io.bs_magic);
  const int off = pos - e * g.block_size;
  const int64_t blk = a.io.block_table[(int64_t)seq * a.io.bt_stride + e];
  uint8_t* rec = const_cast<uint8_t*>(a.io.cache) + blk * g.stride_block + (int64_t)off * g.stride_slot + (int64_t)hkv * g.stride_head;
  if (lane < 2 * LPR) {
    if (g.code_type == KVQ_CODE_INT4) *reinterpret_cast<uint32_t*>(rec + (is_v ? g.v_off : g.k_off) + li * 4) = pk[0];
    else *reinterpret_cast<u32x2_a4*>(rec + (is_v ? g.v_off : g.k_off) + li * 8) = (u32x2){pk[0], pk[1]};
    if (li == 0) *reinterpret_cast<float*>(rec + (is_v ? g.vs_off : g.ks_off)) = scale;
  }
}

}  // namespace kvq
