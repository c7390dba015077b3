// Core of the bandwidth-bound int8 paged decode tile (gfx950, wave64, MFMA f16).
//
// One wavefront owns one KV head and streams that head's records for a run of
// 32-token tiles.  Per tile it
//   * loads the K codes (lane = token x quarter-of-head, 16-byte loads), the V codes
//     (lane = dim-octet x 8 tokens, 8-byte loads) and the 64 fp32 scales, all straight
//     from HBM into registers, double-buffered one tile ahead;
//   * turns codes into exact fp16 integers in registers with the byte-permute magic
//     number trick (0x6400 | (code ^ 0x80) = 1024 + code + 128, minus 1152);
//   * S^T[token, head] = K . Q^T on the MFMA (the GQA group's heads are the N dim, so
//     the KV stream is read once for all of them), softmax in fp32 with the per-token
//     K scale applied to the logits;
//   * O^T[dim, head] += V^T . P~^T on the MFMA, P~ = p * v_scale rounded to fp16.
// The S accumulator layout (lane = head, registers = tokens) is exactly the B-operand
// layout P~^T needs, and the running max / sum / rescale of a head stay lane-local.
#pragma once

#include "kvq_internal.h"

namespace kvq {

constexpr int kTile = 32;            // tokens per step
constexpr float kPScale = 256.0f;    // P~ is kept 2^8 larger so small weights stay normal in fp16
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kLog2e = 1.4426950408889634f;

// v_perm_b32: selector bytes 0-3 pick from `lo`, 4-7 from `hi`.
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// Two biased code bytes (byte b0 and b0+1 of x, already ^0x80) -> two exact fp16 codes.
__device__ __forceinline__ uint32_t bytes_to_half2(uint32_t x, bool upper) {
  const uint32_t magic = 0x64646464u;
  uint32_t h = perm(magic, x, upper ? 0x04030402u : 0x04010400u);  // 1024 + (code + 128)
  half2_t v = __builtin_bit_cast(half2_t, h) - (half2_t){(half_t)1152.0f, (half_t)1152.0f};
  return __builtin_bit_cast(uint32_t, v);
}

// 8 consecutive code bytes (two dwords) -> 8 fp16 codes, the A/B operand of one MFMA k-step.
__device__ __forceinline__ half8_t dequant8(uint32_t lo, uint32_t hi) {
  lo ^= 0x80808080u;
  hi ^= 0x80808080u;
  u32x4 r;
  r.x = bytes_to_half2(lo, false);
  r.y = bytes_to_half2(lo, true);
  r.z = bytes_to_half2(hi, false);
  r.w = bytes_to_half2(hi, true);
  return __builtin_bit_cast(half8_t, r);
}

__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
  half2_t v = {(half_t)a, (half_t)b};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float clamp_half_range(float x) {
  return fminf(fmaxf(x, -65504.f), 65504.f);
}

// What a finished run of tiles turns into.
enum class Emit { kFinal, kStreamPartial, kV2Partial };

struct AttnIO {
  // query / output rows
  const void* q;
  int64_t q_stride_t, q_stride_h;
  void* out;
  int64_t out_stride_t, out_stride_h;
  float* lse;  // [rows, Hq] natural log, or nullptr
  // cache
  const uint8_t* cache;
  kvq_cache_geom g;
  const int32_t* block_table;
  int64_t bt_stride;
  int num_q_heads;
  int group;  // q heads per kv head
  float scale_log2;  // softmax scale * log2(e)
};

// One lane's share of a 32-token tile, as loaded.
template <int D>
struct KVTile {
  static constexpr int KQ = D / 64;  // dwordx4 loads per M-tile for K (lane holds D/4 bytes)
  static constexpr int VW = D / 64;  // dwords per token for V (lane holds D/16 bytes)
  u32x4 k[2][KQ];
  uint32_t v[8][VW];
  float sc;  // lanes 0-31: K scale of token lane; lanes 32-63: V scale of token lane-32
};

template <int D>
struct DecodeState {
  static constexpr int DT = D / 16;  // M-tiles of the O^T accumulator
  floatx4 o[DT];
  float m;  // running max, log2 domain (uniform across the 4 lane groups of a head)
  float l;  // lane-local partial sum
};

// Block ids of one sequence, 64 table entries at a time held one per lane.
struct BlockIds {
  int32_t v;
  int base;  // first table entry held, multiple of 64; -1 = nothing loaded
};

template <int D, int QDT, int ODT>
struct DecodeTile {
  static constexpr int KSTEPS = D / 32;
  static constexpr int DT = D / 16;
  static constexpr int VB = D / 16;  // V bytes per token per lane
  using Tile = KVTile<D>;
  using State = DecodeState<D>;

  // ---- Q as the MFMA B operand: lane (c = head in group, g) holds dims g*D/4 + kk*8 + j ----
  __device__ static void load_q(const AttnIO& io, int64_t row, int hkv, int lane, half8_t (&qb)[KSTEPS]) {
    const int c = lane & 15, g = lane >> 4;
    const bool valid = c < io.group;
    const int64_t base = row * io.q_stride_t + (int64_t)(hkv * io.group + (valid ? c : 0)) * io.q_stride_h +
                         g * (D / 4);
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      u32x4 r;
      float f[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = valid ? clamp_half_range(load_act<QDT>(io.q, base + kk * 8 + j)) : 0.f;
      r.x = pack_half2(f[0], f[1]);
      r.y = pack_half2(f[2], f[3]);
      r.z = pack_half2(f[4], f[5]);
      r.w = pack_half2(f[6], f[7]);
      qb[kk] = __builtin_bit_cast(half8_t, r);
    }
  }

  __device__ static int block_id(const AttnIO& io, const int32_t* bt_row, BlockIds& ids, int entry,
                                 int num_entries, int lane) {
    const int base = entry & ~63;
    if (base != ids.base) {
      const int e = base + lane;
      ids.v = (e < num_entries) ? bt_row[e] : 0;
      ids.base = base;
    }
    return __builtin_amdgcn_readlane(ids.v, entry & 63);
  }

  // Issue the global loads of tile `t` (tokens 32t .. 32t+31) of a sequence of `len` tokens.
  __device__ static void load_tile(const AttnIO& io, const int32_t* bt_row, BlockIds& ids, int len, int t,
                                   int hkv, int lane, Tile& kv) {
    const kvq_cache_geom& G = io.g;
    const int r = lane & 15, g = lane >> 4;
    const int num_entries = (len + G.block_size - 1) / G.block_size;
    const int tok0 = t * kTile;
    // a 16-token M-tile never straddles a block (block_size is a multiple of 16)
    int e0 = tok0 / G.block_size;
    int e1 = (tok0 + 16) / G.block_size;
    e1 = e1 < num_entries ? e1 : num_entries - 1;  // second half may lie past the end: reread, masked later
    const int64_t b0 = block_id(io, bt_row, ids, e0, num_entries, lane);
    const int64_t b1 = (e1 == e0) ? b0 : (int64_t)block_id(io, bt_row, ids, e1, num_entries, lane);
    const int s0 = tok0 % G.block_size;
    const int s1 = (e1 == (tok0 + 16) / G.block_size) ? (tok0 + 16) % G.block_size : s0;
    const uint8_t* p0 = io.cache + b0 * G.stride_block + (int64_t)s0 * G.stride_slot + (int64_t)hkv * G.stride_head;
    const uint8_t* p1 = io.cache + b1 * G.stride_block + (int64_t)s1 * G.stride_slot + (int64_t)hkv * G.stride_head;
    // K: lane (r, g) reads bytes [g*D/4, (g+1)*D/4) of token r / 16 + r
    {
      const uint8_t* k0 = p0 + (int64_t)r * G.stride_slot + G.k_off + g * (D / 4);
      const uint8_t* k1 = p1 + (int64_t)r * G.stride_slot + G.k_off + g * (D / 4);
#pragma unroll
      for (int i = 0; i < Tile::KQ; ++i) {
        kv.k[0][i] = *reinterpret_cast<const u32x4_a4*>(k0 + 16 * i);
        kv.k[1][i] = *reinterpret_cast<const u32x4_a4*>(k1 + 16 * i);
      }
    }
    // V: lane (r, g) reads bytes [r*VB, (r+1)*VB) of tokens 4g+j (j<4) and 16+4g+(j-4)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint8_t* pv = (j < 4 ? p0 : p1) + (int64_t)(4 * g + (j & 3)) * G.stride_slot + G.v_off + r * VB;
#pragma unroll
      for (int w = 0; w < Tile::VW; ++w) kv.v[j][w] = *reinterpret_cast<const uint32_t*>(pv + 4 * w);
    }
    // scales: lanes 0-31 K scale of token lane, lanes 32-63 V scale of token lane-32
    {
      const int tk = lane & 31;
      const uint8_t* ps = (tk < 16 ? p0 : p1) + (int64_t)(tk & 15) * G.stride_slot + (lane < 32 ? G.ks_off : G.vs_off);
      kv.sc = *reinterpret_cast<const float*>(ps);
    }
  }

  // Consume one loaded tile.  `sc_lds` is this wave's 64-float staging area.
  __device__ static void compute_tile(const AttnIO& io, const Tile& kv, const half8_t (&qb)[KSTEPS], int len,
                                      int t, int lane, float* sc_lds, State& st) {
    const int g = lane >> 4;
    // --- scales: transpose lane<->token through LDS (wave-private, no barrier needed) ---
    sc_lds[lane] = kv.sc;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const floatx4 ks0 = *reinterpret_cast<const floatx4*>(sc_lds + 4 * g);
    const floatx4 ks1 = *reinterpret_cast<const floatx4*>(sc_lds + 16 + 4 * g);
    const floatx4 vs0 = *reinterpret_cast<const floatx4*>(sc_lds + 32 + 4 * g);
    const floatx4 vs1 = *reinterpret_cast<const floatx4*>(sc_lds + 48 + 4 * g);
    __builtin_amdgcn_wave_barrier();

    // --- S^T = K . Q^T : two 16-token M-tiles, KSTEPS k-steps each ---
    floatx4 s[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      s[mt] = (floatx4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KSTEPS; ++kk) {
        const u32x4& w = kv.k[mt][kk >> 1];
        const half8_t a = (kk & 1) ? dequant8(w.z, w.w) : dequant8(w.x, w.y);
        s[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qb[kk], s[mt], 0, 0, 0);
      }
    }

    // --- softmax (log2 domain); lane holds tokens 32t + mt*16 + 4g + i of head (lane & 15) ---
    float logit[8];
    const int tok_base = t * kTile + 4 * g;
    float mloc = -INFINITY;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float ks = (mt ? ks1 : ks0)[i];
        const bool ok = (tok_base + mt * 16 + i) < len;
        const float x = ok ? s[mt][i] * (ks * io.scale_log2) : -INFINITY;
        logit[mt * 4 + i] = x;
        mloc = fmaxf(mloc, x);
      }
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, kWave));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
    if (__builtin_amdgcn_ballot_w64(mloc > st.m) != 0) {  // rescale only when some head's max moved
      const float m_new = fmaxf(st.m, mloc);
      const float alpha = __builtin_amdgcn_exp2f(st.m - m_new);  // st.m = -inf -> 0
      st.m = m_new;
      st.l *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) st.o[dt] *= alpha;
    }
    float pt[8];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = mt * 4 + i;
        const float p = __builtin_amdgcn_exp2f(logit[j] - st.m);  // masked: exp2(-inf) = 0
        st.l += p;
        const float vs = (mt ? vs1 : vs0)[i];
        const bool ok = (tok_base + mt * 16 + i) < len;
        pt[j] = ok ? clamp_half_range(p * (vs * kPScale)) : 0.f;  // garbage scales of masked tokens never enter
      }
    }
    u32x4 pb;
    pb.x = pack_half2(pt[0], pt[1]);
    pb.y = pack_half2(pt[2], pt[3]);
    pb.z = pack_half2(pt[4], pt[5]);
    pb.w = pack_half2(pt[6], pt[7]);
    const half8_t p_op = __builtin_bit_cast(half8_t, pb);

    // --- O^T += V^T . P~^T : in-register 8x(VB) byte transpose, then one MFMA per dim tile ---
#pragma unroll
    for (int w = 0; w < Tile::VW; ++w) {
      uint32_t x0[4], x1[4];  // per token pair a: bytes (b0,b1) and (b2,b3) of both tokens, interleaved
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const uint32_t ta = kv.v[2 * a][w] ^ 0x80808080u;
        const uint32_t tb = kv.v[2 * a + 1][w] ^ 0x80808080u;
        x0[a] = perm(tb, ta, 0x05010400u);
        x1[a] = perm(tb, ta, 0x07030602u);
      }
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        u32x4 av;
        const uint32_t* x = (b < 2) ? x0 : x1;
        av.x = bytes_to_half2(x[0], b & 1);
        av.y = bytes_to_half2(x[1], b & 1);
        av.z = bytes_to_half2(x[2], b & 1);
        av.w = bytes_to_half2(x[3], b & 1);
        const int dt = 4 * w + b;
        st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, av), p_op, st.o[dt], 0, 0, 0);
      }
    }
  }

  // Run tiles [t_begin, t_end) of one sequence for kv head `hkv`; leaves the state in `st`.
  __device__ static void run(const AttnIO& io, int seq, int64_t row, int len, int t_begin, int t_end, int hkv,
                             int lane, float* sc_lds, State& st) {
    half8_t qb[KSTEPS];
    load_q(io, row, hkv, lane, qb);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) st.o[dt] = (floatx4){0.f, 0.f, 0.f, 0.f};
    st.m = -INFINITY;
    st.l = 0.f;
    const int32_t* bt_row = io.block_table + (int64_t)seq * io.bt_stride;
    BlockIds ids{0, -1};
    Tile a, b;
    load_tile(io, bt_row, ids, len, t_begin, hkv, lane, a);
    for (int t = t_begin; t < t_end; t += 2) {
      const bool has_b = (t + 1) < t_end;
      if (has_b) load_tile(io, bt_row, ids, len, t + 1, hkv, lane, b);
      compute_tile(io, a, qb, len, t, lane, sc_lds, st);
      if (has_b) {
        if ((t + 2) < t_end) load_tile(io, bt_row, ids, len, t + 2, hkv, lane, a);
        compute_tile(io, b, qb, len, t + 1, lane, sc_lds, st);
      }
    }
  }

  // Sum of the lane-local l over the 4 lane groups of a head.
  __device__ static float total_l(const State& st) {
    float l = st.l;
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    return l;
  }

  // Lane (c, g) holds O[head c][dim (4g+i)*VB + dt], i = 0..3, dt = 0..DT-1: D/4 contiguous
  // dims starting at g*D/4.  Gather them in order, scaled by `mul`.
  __device__ static void gather_row(const State& st, float mul, float (&v)[D / 4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) v[i * VB + dt] = st.o[dt][i] * mul;
  }

  // Whole sequence handled by this wave: normalise and write the output row (and lse).
  __device__ static void emit_final(const AttnIO& io, int64_t row, int hkv, int lane, const State& st) {
    const float l = total_l(st);  // every lane takes part in the shuffles
    const int c = lane & 15, g = lane >> 4;
    if (c >= io.group) return;
    const int head = hkv * io.group + c;
    float v[D / 4];
    gather_row(st, 1.0f / (l * kPScale), v);
    const int64_t base = row * io.out_stride_t + (int64_t)head * io.out_stride_h + g * (D / 4);
    if constexpr (ODT == KVQ_F32) {
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
          if constexpr (ODT == KVQ_BF16) {
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
    gather_row(st, 1.0f / kPScale, v);
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
    gather_row(st, 1.0f / (l * kPScale), v);
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
  int num_seqs;
  int num_wg;  // P
};

}  // namespace kvq
