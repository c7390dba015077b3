// MLA decode over the int8 latent cache (gfx950, wave64; QK on the int8 MFMA 16x16x64, PV on the
// f16 MFMA 16x16x32).
//
// All query heads of a sequence share ONE latent stream (576 int8 codes + one fp32 scale per
// token), so this is a dense contraction: S^T[token, head] = C . Q^T over 576 dims and
// O^T[dim, head] = C[:, :512]^T . P~^T, both on the MFMA with the heads as the N dimension.
//
// Work item = (sequence, token split, 128-head block); workgroup = 8 waves.  Each 32-token tile of
// the latent stream goes from global memory STRAIGHT into one of three LDS windows
// (buffer_load ... lds, no registers in between), a whole tile time ahead of its use; the 16-byte
// chunks of a row are swizzled so that operand reads are free of bank conflicts without padding.
// QK: wave w owns head tile w (16 heads) of the block and computes that tile's logits on the int8
// MFMA straight from the cached code bytes; its absorbed Q sits in registers (16 of its 18
// operands) and LDS (the other 2) as two int8 terms that a small kernel prepares once per launch.
// It runs the tile's softmax (lazy reference maximum) and publishes the P~ operand, the rescale
// factors and a "maximum moved" flag through a double-buffered LDS exchange.
// PV is split over the waves by OUTPUT DIMS, not by heads: wave w accumulates dims 64 w .. 64 w + 63
// of all 128 heads, so it needs only those 64 dims of the tile as fp16 V^T: a lane reads one dword
// from each of its 8 token rows of the raw tile and transposes in registers (byte permutes), no
// second copy of the tile in LDS; it reads eight P~ operands per tile.  One workgroup barrier per
// tile (P~ and the next raw tile visible); the third window is what lets the P~V read the raw tile
// after that barrier while the tile after the next already streams in.
// With at most 16 heads (one head tile, the shape of a tensor-parallel shard) a second kernel takes
// over, mla_decode_small_kernel: four waves, each streaming its own tiles straight from global memory
// into the int8 MFMA's operand order, with the query quantised inside the kernel.
// The token splits of a sequence are merged by the reduce kernel with the log-sum-exp algebra
// (same two-stage shape as the reference's decode_attention_fwd); all splits of a sequence run on the
// XCD that prepares its query and reduces it (mla_seq_split_of_block).  Nothing is allocated here,
// partials and the int8 Q live in the caller's workspace.
#include <atomic>
#include <type_traits>

#include "kvq_attn_core.cuh"

namespace kvq {

constexpr int kMlaR = 512, kMlaP = 64, kMlaW = kMlaR + kMlaP;
constexpr int kMlaPitch = kMlaW;                          // LDS rows are packed; the 16-byte chunks of a row are swizzled
constexpr int kMlaTileBytes = kTile * kMlaPitch;          // 32 rows = 1152 chunks
constexpr int kMlaBufBytes = kMlaTileBytes + 2 * kTile * 4;  // + 32 K-side and 32 V-side scales
constexpr int kChunksPerRow = kMlaW / 16;                 // 36
constexpr int kChunksPerHalf = 16 * kChunksPerRow;        // 576
constexpr int kMlaThreads = 512;
constexpr int kMlaKSteps8 = kMlaW / 64;                   // 9 int8 k-steps of 64 dims
constexpr int kMlaQOps = 2 * kMlaKSteps8;                 // B operands of Q: two int8 terms per k-step
constexpr int kMlaQRegOps = 16;                           // operands of Q kept in registers; the rest in LDS
constexpr int kMlaQLdsBytes = (kMlaQOps - kMlaQRegOps) * kMlaThreads * 16;  // 16384
constexpr float kMlaQ2 = 256.0f;                          // ratio of the scales of the query's two int8 terms
constexpr float kMlaQ1Max = 16383.5f / kMlaQ2;            // largest first term: s1 = max|q| / kMlaQ1Max
constexpr int kMlaRing = 3;                               // raw tile windows: tile t is read (QK, then PV) while t + 1 and t + 2 stream in
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
// What the head-owning waves hand to the others, per tile and double-buffered: the eight P~ operands
// (64 lanes x 16 bytes each), one rescale factor per head and one "running max moved" byte per wave.
constexpr int kMlaPBytes = 8 * kWave * 16;                // 8192
constexpr int kMlaXchgBytes = kMlaPBytes + 128 * 4 + 16;  // 8720
constexpr int kMlaLdsBytes = kMlaRing * kMlaBufBytes + kMlaQLdsBytes + 2 * kMlaXchgBytes;  // 139296 of 163840

struct MlaArgs {
  const void* q;            // dims 0 .. 511 of the absorbed query (ql_nope) ...
  int64_t q_stride_b, q_stride_h;
  const void* q_pe;         // ... and its 64 rope dims: q + 512 elements when the caller holds them joined
  int64_t pe_stride_b, pe_stride_h;
  const uint8_t* cache;
  kvq_mla_geom g;
  const int32_t* block_table;
  int64_t bt_stride;
  const int32_t* seq_lens;
  // Split states.  part_o holds the locally normalised outputs as fp16, in the order the MFMA leaves
  // them in registers, so that every store and every load of the reduce is one contiguous 512 bytes
  // per wave: [B, S, ceil(H/16)] blocks of [32 (= d4 * 4 + i)][64 lanes][4 halves], lane (c, g) holding
  // dims 64 d4 + 16 g + 4 i + (0..3) of head 16 * block + c.  part_lse: [B, S, 16 * ceil(H/16)] fp32,
  // log2 domain, -inf for an empty split.
  uint16_t* part_o;
  float* part_lse;
  // Q as the int8 MFMA wants it (written by mla_absorb_q_kernel, read by every split of a sequence):
  // q_ops [B, ceil(H/16)][18 operands][64 slots][16 bytes], lane (c = head, g)'s piece in slot 4 c + g (a head's four
  // pieces together: the absorption kernel, a workgroup per head, writes 64 contiguous bytes per operand);
  // q_scale [B, 16 * ceil(H/16)] = s1 per head.
  uint8_t* q_ops;
  float* q_scale;
  int head_groups;  // ceil(H / 16)
  int num_heads;
  int num_splits;
  float scale_log2;
  uint32_t bs_magic;
  // Fused write of the step's new latent rows (kvc_new == nullptr: the cache already holds them): row i of
  // kvc_new [B, 512] / kpe_new [B, 64] is the token at position seq_lens[i] - 1 of sequence i.
  const void* kvc_new;
  const void* kpe_new;
  int64_t kvc_stride, kpe_stride;  // elements
  int new_dtype;
  float new_eps;
  // One split per sequence (out != nullptr): the split's state IS the result, and the decode kernels write it
  // themselves -- out [B, H, 512] in out_dtype, lse_out [B, H] natural log (may be NULL) -- instead of leaving a
  // state for a reduce kernel that would only convert and copy it.
  void* out;
  float* lse_out;
  int out_dtype;
};

// Four consecutive output dims of one head in the caller's output type (`elem` = element offset, a multiple of 4).
__device__ __forceinline__ void mla_store_out4(const MlaArgs& a, int64_t elem, floatx4 v) {
  if (a.out_dtype == KVQ_F32) {
    *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(a.out) + elem) = v;
  } else {
    u32x2 w;
    if (a.out_dtype == KVQ_BF16) {
      w.x = (uint32_t)f32_to_bf16_bits(v.x) | ((uint32_t)f32_to_bf16_bits(v.y) << 16);
      w.y = (uint32_t)f32_to_bf16_bits(v.z) | ((uint32_t)f32_to_bf16_bits(v.w) << 16);
    } else {
      w.x = pack_half2(v.x, v.y);
      w.y = pack_half2(v.z, v.w);
    }
    *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(a.out) + elem) = w;
  }
}

// The fused cache update of the decode kernels: ONE wave loads (mla_new_row_load) and later quantises and stores
// (mla_new_row_store) the sequence's new latent row at position len - 1, with the write kernel's arithmetic.
__device__ __forceinline__ void mla_new_row_load(const MlaArgs& a, int seq, int lane, MlaRowRaw& raw) {
  mla_row_load_raw(a.kvc_new, a.kpe_new, a.new_dtype, (int64_t)seq * a.kvc_stride, (int64_t)seq * a.kpe_stride,
                   kMlaR / 8, kMlaW / 8, lane, raw);
}
__device__ __forceinline__ void mla_new_row_store(const MlaArgs& a, int seq, int len, int lane, const MlaRowRaw& raw) {
  MlaRowPieces r;
  mla_row_convert(raw, a.new_dtype, r);
  const float scale = mla_row_scale(r, a.new_eps);
  const int pos = len - 1;
  const int e = (int)__umulhi((uint32_t)pos, a.bs_magic);
  const int off = pos - e * a.g.block_size;
  uint8_t* blk = const_cast<uint8_t*>(a.cache) + (int64_t)a.block_table[(int64_t)seq * a.bt_stride + e] * a.g.stride_block;
  mla_row_store(r, scale, blk + (int64_t)off * a.g.stride_row, reinterpret_cast<float*>(blk + a.g.scale_off + (int64_t)off * 4), lane);
}

// Byte B of x0 and of x1, each a signed code, as the fp16 pair (x0.B, x1.B): the conversion reads its
// byte through the operand's sub-dword select with sign extension and writes one half of the result, so
// a pair costs two instructions and no shuffles.
template <int B>
__device__ __forceinline__ uint32_t mla_code_pair_to_half2(uint32_t x0, uint32_t x1) {
  uint32_t r;
  asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_%2" : "=v"(r) : "v"(x0), "n"(B));
  asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_%2" : "+v"(r) : "v"(x1), "n"(B));
  return r;
}
template <int B>
__device__ __forceinline__ half8_t mla_code_rows_to_operand(const uint32_t (&x)[8]) {
  u32x4 h;
  h.x = mla_code_pair_to_half2<B>(x[0], x[1]);
  h.y = mla_code_pair_to_half2<B>(x[2], x[3]);
  h.z = mla_code_pair_to_half2<B>(x[4], x[5]);
  h.w = mla_code_pair_to_half2<B>(x[6], x[7]);
  return __builtin_bit_cast(half8_t, h);
}

// tokens of a sequence per split, a whole number of tiles
__device__ __forceinline__ int mla_split_len(int len, int num_splits) {
  const int per = (len + num_splits - 1) / num_splits;
  return ((per + kTile - 1) / kTile) * kTile;
}

// 16 values of one head -> the 16 bytes of each of the two int8 terms, q ~ s1 a + s2 b with s2 = s1 / 256:
// w = rint(q / s2) is a 15-bit integer (|w| <= 16384 because s1 = max|q| / kMlaQ1Max), and w = 256 a + b with
// b in [-128, 127] splits it: a is the high byte of w + 128, b its low byte with the top bit flipped.  One
// normalised 16-bit conversion quantises two values, one packed add and three byte permutes per four values
// do the rest.  `live` false gives zero bytes (heads past the end).
typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
typedef short s16x2_t __attribute__((__vector_size__(2 * sizeof(short))));
__device__ __forceinline__ void mla_two_int8_terms(const float (&f)[16], float s1, bool live, u32x4& ta, u32x4& tb) {
  // the conversion multiplies by 32767: q * inv * 32767 = q / s2
  const float inv = live ? kMlaQ2 / (s1 * 32767.0f) : 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    uint32_t t[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const s16x2_t pk = __builtin_amdgcn_cvt_pknorm_i16(f[4 * w + 2 * j] * inv, f[4 * w + 2 * j + 1] * inv);
      t[j] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2_t, pk) + (u16x2_t){128, 128});
    }
    ta[w] = perm(t[1], t[0], 0x07050301u);                  // the four high bytes
    tb[w] = perm(t[1], t[0], 0x06040200u) ^ 0x80808080u;    // the four low bytes, as signed numbers
  }
}

// Dims 64 kk + 16 g .. + 15 of one head's query (k-step 8 is the rope part), as loaded -- four 16-byte words
// for fp32 rows, two for 16-bit rows -- and as floats.  `qbase` / `pebase` are the element offsets of the
// lane's head row plus 16 g.  Load and conversion are apart so that a caller can put other loads between.
template <int QDT>
struct MlaQRaw {
  u32x4 w[QDT == KVQ_F32 ? 4 : 2];
};
template <int QDT>
__device__ __forceinline__ MlaQRaw<QDT> mla_load_q16_raw(const MlaArgs& a, int64_t qbase, int64_t pebase, int kk) {
  MlaQRaw<QDT> r;
  if constexpr (QDT == KVQ_F32) {
    const float* p = kk < kMlaR / 64 ? reinterpret_cast<const float*>(a.q) + qbase + 64 * kk
                                     : reinterpret_cast<const float*>(a.q_pe) + pebase;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.w[i] = *reinterpret_cast<const u32x4_a4*>(p + 4 * i);
  } else {
    const uint16_t* p = kk < kMlaR / 64 ? reinterpret_cast<const uint16_t*>(a.q) + qbase + 64 * kk
                                        : reinterpret_cast<const uint16_t*>(a.q_pe) + pebase;
#pragma unroll
    for (int h = 0; h < 2; ++h) r.w[h] = *reinterpret_cast<const u32x4_a4*>(p + 8 * h);
  }
  return r;
}
template <int QDT>
__device__ __forceinline__ void mla_q16_to_float(const MlaQRaw<QDT>& r, float (&f)[16]) {
  if constexpr (QDT == KVQ_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) f[4 * i + j] = as_f32(r.w[i][j]);
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t e = r.w[h][w];
        if constexpr (QDT == KVQ_BF16) {
          f[8 * h + 2 * w] = as_f32(e << 16);
          f[8 * h + 2 * w + 1] = as_f32(e & 0xffff0000u);
        } else {
          const half2_t hh = __builtin_bit_cast(half2_t, e);
          f[8 * h + 2 * w] = (float)hh.x;
          f[8 * h + 2 * w + 1] = (float)hh.y;
        }
      }
  }
}
// Which (sequence, split) a workgroup of the (splits, sequences) grid takes.  Workgroups go to the eight XCDs
// (each with an L2 of its own) round-robin in launch order, so with the plain mapping the splits of one
// sequence sit on eight different XCDs: each fetches the sequence's query operands for itself, and the
// reduce kernel finds none of the sequence's split states in its L2.  Here all splits of a sequence share
// the XCD "sequence mod 8" -- the one that mla_reduce_kernel (a grid with the sequence as x) runs that
// sequence on.  Sequences past the last multiple of eight keep the plain mapping.
__device__ __forceinline__ void mla_seq_split_of_block(int num_seqs, int num_splits, int& seq, int& split) {
  const int n = blockIdx.x + gridDim.x * blockIdx.y;
  const int seqs8 = num_seqs & ~7;
  if (n < seqs8 * num_splits) {
    const int xcd = n & 7, k = n >> 3;
    seq = (k / num_splits) * 8 + xcd;
    split = k % num_splits;
  } else {
    const int r = n - seqs8 * num_splits;
    seq = seqs8 + r / num_splits;
    split = r % num_splits;
  }
}

// Q for the int8 MFMA.  The cache codes ARE int8, so the QK product can run on
// v_mfma_i32_16x16x64_i8 straight from the cached bytes -- no conversion of K at all -- once Q is
// int8 too: q = s1 * a + s2 * b with a the nearest multiple of s1 = max|q| / 64 per head (about), and
// b the rest in units of s2 = s1 / 256, where 256 a + b = rint(q / s2) is a 15-bit integer (|a| <= 64, so that
// 256 a . k + b . k, the two integer sums joined with one shift-add, stays below 2^31 for any codes).  The
// residual after two terms is at most s2 / 2 = max|q| / 32767, finer than the fp16 rounding of q it replaces, and the integer dot
// products are exact.  For a (sequence, 16 heads) block, lane (c = head, g) holds, for k-step kk, dims
// 64 kk + 16 g + j (j < 16) as 16 bytes, operand 2 kk = term a, operand 2 kk + 1 = term b.  The decode
// kernels build these operands in their prologues (mla_two_int8_terms); only the absorption kernel below
// writes them to the workspace.

// Q absorption fused with the int8 preparation: ql[b, h, :] = q_nope[b, h, :] . W_UK_T[h] (the first
// bmm of the reference's MLA layer, mla_attention.py:835-848) computed on the MFMA and written
// STRAIGHT into the decode's operand layout as two int8 terms + s1 -- the absorbed query never exists
// in HBM as bf16.
// Workgroup = (head, 16 sequences), 4 waves; wave w owns latent dims 128 w .. 128 w + 127.  The product
// is taken transposed, ql^T = W^T q^T: B = q_nope rows (lane = sequence, 8 consecutive p), A = W^T needs 8
// p of one dim per lane while W_UK_T [P, L] keeps 8 dims of one p together, so each lane loads the
// slice [its 8 p] x [8 consecutive dims] and transposes it in registers (one v_perm_b32 per dword), as
// the prefill attention does for V.  Block i of a wave's output then holds dims 8 lane + i: a lane ends
// with 32 consecutive dims of its own sequence, i.e. two of the 16-byte pieces of the operand layout.
// The row maximum (all 576 dims, rope included) crosses the four waves through LDS.
// Tiles of 16 sequences per workgroup (the kernel takes up to 4: wave t brings tile t's rope dims): the weights a wave
// has loaded and transposed serve all of them.  One tile while that fills the chip, two beyond 64 sequences; with
// four, a workgroup's registers leave one workgroup per CU and it measured slower (library GEMM of the same product
// at 128 heads: 10.5 / 15.3 / 26.0 us at 128 / 256 / 512 sequences; one tile: 17.7 / 28.8 / 51.9 us; two tiles and
// the operand slots of MlaArgs::q_ops: 13.5 / 20.4 / 35.7 us; four tiles: 23.1 / 41.5 us at 256 / 512).
__host__ __device__ constexpr int mla_absorb_tiles(int num_seqs) { return num_seqs <= 64 ? 1 : 2; }
struct MlaAbsorbArgs {
  const void* q_nope;   // [B, H, P]
  int64_t qn_sb, qn_sh;
  const void* w;        // W_UK_T [H, P, 512], dims contiguous
  int64_t w_sh, w_sp;
  const void* q_pe;     // [B, H, 64]
  int64_t pe_sb, pe_sh;
  uint8_t* q_ops;
  float* q_scale;
  int head_groups, num_heads, num_seqs, ksteps;   // ksteps = P / 32
  int seq_tiles, group_major;                     // tiles of 16 * NB sequences; how workgroups are numbered
};

// KSTEPS = P / 32 when known at compile time (the loop is unrolled and every load of W is in flight at
// once: the kernel is one memory round trip long), 0 = read it from the arguments.
template <int QDT, int KSTEPS, int NB>
__global__ __launch_bounds__(256) void mla_absorb_q_kernel(MlaAbsorbArgs a) {
  __shared__ float part_max[4][NB][16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  // Workgroups go to the eight XCDs round-robin in launch order.  With a multiple of eight head groups a group's
  // workgroups (16 heads x the tiles of sequences) are numbered onto ONE XCD: the 16-byte pieces that 16 heads
  // write into an operand block then meet in that XCD's L2 as whole lines (and the tiles of a head still share
  // its weights there); otherwise heads are numbered first, which keeps the tiles of a head on one XCD.
  int head, b0;
  if (a.group_major) {
    const int per_group = 16 * a.seq_tiles;
    const int q = blockIdx.x >> 3, r = q % per_group;
    head = ((q / per_group) * 8 + (blockIdx.x & 7)) * 16 + (r & 15);
    b0 = (r >> 4) * (16 * NB);
  } else {
    head = blockIdx.x % (a.head_groups * 16);
    b0 = blockIdx.x / (a.head_groups * 16) * (16 * NB);
  }
  const bool head_ok = head < a.num_heads;
  const int hsrc = head_ok ? head : 0;
  floatx4 acc[NB][8];
#pragma unroll
  for (int t = 0; t < NB; ++t)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[t][i] = (floatx4){0.f, 0.f, 0.f, 0.f};
  int brow[NB];
#pragma unroll
  for (int t = 0; t < NB; ++t) brow[t] = min(b0 + 16 * t + c, a.num_seqs - 1);   // rows past the end: a copy, not written
  const uint16_t* wp = static_cast<const uint16_t*>(a.w) + (int64_t)hsrc * a.w_sh + (int64_t)(8 * g) * a.w_sp + 128 * wave + 8 * c;
  const uint16_t* qp = static_cast<const uint16_t*>(a.q_nope) + (int64_t)hsrc * a.qn_sh + 8 * g;
  auto step = [&](const u32x4 (&rows)[8], const u32x4 (&qop)[NB]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t sel = (i & 1) ? kPermHighHalves : kPermLowHalves;
      u32x4 wt;
      wt.x = perm(rows[1][i >> 1], rows[0][i >> 1], sel);
      wt.y = perm(rows[3][i >> 1], rows[2][i >> 1], sel);
      wt.z = perm(rows[5][i >> 1], rows[4][i >> 1], sel);
      wt.w = perm(rows[7][i >> 1], rows[6][i >> 1], sel);
#pragma unroll
      for (int t = 0; t < NB; ++t) acc[t][i] = mfma16<QDT>(wt, qop[t], acc[t][i]);
    }
  };
  // wave t also brings the rope dims 16 g .. 16 g + 15 of tile t: requested with everything else, so that the
  // kernel stays one trip to memory long
  u32x4 pe_raw[2];
  {
    const int t = wave < NB ? wave : 0;
    const uint16_t* pp = static_cast<const uint16_t*>(a.q_pe) + (int64_t)brow[t] * a.pe_sb + (int64_t)hsrc * a.pe_sh + 16 * g;
#pragma unroll
    for (int h = 0; h < 2; ++h) pe_raw[h] = *reinterpret_cast<const u32x4_a4*>(pp + 8 * h);
  }
  if constexpr (KSTEPS > 0) {
    // every load of the kernel first, then the arithmetic
    u32x4 rows[KSTEPS][8], qop[KSTEPS][NB];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
      for (int t = 0; t < NB; ++t) qop[s][t] = *reinterpret_cast<const u32x4_a4*>(qp + (int64_t)brow[t] * a.qn_sb + 32 * s);
#pragma unroll
      for (int j = 0; j < 8; ++j) rows[s][j] = *reinterpret_cast<const u32x4*>(wp + (int64_t)(32 * s + j) * a.w_sp);
    }
    __builtin_amdgcn_sched_barrier(0);   // keep the scheduler from sinking the loads back to their uses
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) step(rows[s], qop[s]);
  } else {
    for (int s = 0; s < a.ksteps; ++s) {
      u32x4 rows[8], qop[NB];
#pragma unroll
      for (int j = 0; j < 8; ++j) rows[j] = *reinterpret_cast<const u32x4*>(wp + (int64_t)(32 * s + j) * a.w_sp);
#pragma unroll
      for (int t = 0; t < NB; ++t) qop[t] = *reinterpret_cast<const u32x4_a4*>(qp + (int64_t)brow[t] * a.qn_sb + 32 * s);
      step(rows, qop);
    }
  }
  // lane (sequence c, quarter g) of wave w holds dims 128 w + 32 g + 8 r + i of its sequence in acc[t][i][r]
  float pe[16];
  {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const u32x4 v = pe_raw[h];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t e = v[w];
        if constexpr (QDT == KVQ_BF16) {
          pe[8 * h + 2 * w] = as_f32(e << 16);
          pe[8 * h + 2 * w + 1] = as_f32(e & 0xffff0000u);
        } else {
          const half2_t hh = __builtin_bit_cast(half2_t, e);
          pe[8 * h + 2 * w] = (float)hh.x;
          pe[8 * h + 2 * w + 1] = (float)hh.y;
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < NB; ++t) {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) amax = fmaxf(amax, fabsf(acc[t][i][r]));
    if (wave == t) {
#pragma unroll
      for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(pe[j]));
    }
    amax = max_over_quarters(amax);
    if (g == 0) part_max[wave][t][c] = amax;
  }
  __syncthreads();
  const int hgroup = head >> 4, hc = head & 15;
#pragma unroll
  for (int t = 0; t < NB; ++t) {
    const int b = b0 + 16 * t + c;
    if (b >= a.num_seqs) continue;
    float amax = fmaxf(fmaxf(part_max[0][t][c], part_max[1][t][c]), fmaxf(part_max[2][t][c], part_max[3][t][c]));
    amax = head_ok ? fminf(amax, 3.0e38f) : 0.f;   // heads past the end contribute zero columns
    const float s1 = amax > 0.f ? amax / kMlaQ1Max : 1.0f;
    const int64_t qblock = (int64_t)b * a.head_groups + hgroup;
    u32x4* qdst = reinterpret_cast<u32x4*>(a.q_ops + qblock * (kMlaQOps * kWave * 16)) + 4 * hc;   // a head's four pieces of an operand lie together
    // the lane's 32 dims are the 16-dim pieces u = 0, 1: k-step kk = 2 w + g / 2, piece 2 (g % 2) + u of it
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      float f[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) f[j] = acc[t][j & 7][2 * u + (j >> 3)];
      u32x4 ta, tb;
      mla_two_int8_terms(f, s1, head_ok, ta, tb);
      const int kk = 2 * wave + (g >> 1), piece = 2 * (g & 1) + u;
      qdst[(2 * kk) * kWave + piece] = ta;
      qdst[(2 * kk + 1) * kWave + piece] = tb;
    }
    if (wave == t) {
      u32x4 ta, tb;
      mla_two_int8_terms(pe, s1, head_ok, ta, tb);
      qdst[(2 * (kMlaKSteps8 - 1)) * kWave + g] = ta;
      qdst[(2 * (kMlaKSteps8 - 1) + 1) * kWave + g] = tb;
      if (g == 0) a.q_scale[qblock * 16 + hc] = s1;
    }
  }
}

// FULL: every 128-head block of the launch has its eight head tiles (num_heads a multiple of 128)
// QDT >= 0: every owner wave quantises the query of its 16 heads itself, from rows of that type (its loads leave
// before the first tile's, its arithmetic runs while the tile streams in); QDT < 0: the operands were prepared
// by the absorption kernel and are read from the workspace.
template <bool FULL, int QDT>
__global__ __launch_bounds__(kMlaThreads) void mla_decode_kernel(MlaArgs a) {
  extern __shared__ __align__(16) uint8_t lds_raw[];
  uint8_t(*lds)[kMlaBufBytes] = reinterpret_cast<uint8_t(*)[kMlaBufBytes]>(lds_raw);   // kMlaRing raw windows
  // B operands of Q from number kMlaQRegOps on: slot [operand][thread], written and read by the same lane
  u32x4* qlds = reinterpret_cast<u32x4*>(lds_raw + kMlaRing * kMlaBufBytes) + threadIdx.x;
  uint8_t* xchg = lds_raw + kMlaRing * kMlaBufBytes + kMlaQLdsBytes;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, g = lane >> 4;
  int seq, split;
  mla_seq_split_of_block(gridDim.y, a.num_splits, seq, split);
  const int len = a.seq_lens[seq];
  const int slen = mla_split_len(len > 0 ? len : 0, a.num_splits);
  const int tok_begin = split * slen;
  const int tok_end = min(len, tok_begin + slen);
  // head tiles (16 heads each) of this workgroup's 128-head block; wave w < nht owns tile w: it
  // computes that tile's logits and softmax.  EVERY wave accumulates the outputs of all nht tiles,
  // for its own 64 of the 512 dims.
  const int nht = FULL ? 8 : min(8, a.head_groups - (int)blockIdx.z * 8);
  const int hgroup = blockIdx.z * 8 + wave;
  const bool owner = wave < nht;                  // wave-uniform
  const int64_t pblock0 = ((int64_t)seq * a.num_splits + split) * a.head_groups + blockIdx.z * 8;
  if (tok_begin >= tok_end) {  // empty split (uniform over the workgroup): mark it and leave
    if (a.out != nullptr) {    // the sequence's only split: an empty sequence, zeros and lse = -inf
#pragma unroll
      for (int ht = 0; ht < 8; ++ht) {
        const int head = (blockIdx.z * 8 + ht) * 16 + c;
        if (ht < nht && head < a.num_heads) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            mla_store_out4(a, ((int64_t)seq * a.num_heads + head) * kMlaR + 64 * wave + 16 * g + 4 * i, (floatx4){0.f, 0.f, 0.f, 0.f});
        }
      }
      if (owner && g == 0 && hgroup * 16 + c < a.num_heads && a.lse_out != nullptr)
        a.lse_out[(int64_t)seq * a.num_heads + hgroup * 16 + c] = -INFINITY;
      return;
    }
    if (owner && g == 0) a.part_lse[(pblock0 + wave) * 16 + c] = -INFINITY;
    return;
  }
  const int t_begin = tok_begin / kTile, t_end = (tok_end + kTile - 1) / kTile;
  const int bs = a.g.block_size;
  const int32_t* bt_row = a.block_table + (int64_t)seq * a.bt_stride;
  // Fused write: the workgroup whose split holds the sequence's end stores the new row (its last wave does;
  // every 128-head block of the sequence stores the same bytes).  The tile that holds the row must be loaded
  // after the store has completed.  With three tiles or more that tile is requested inside the loop, after a
  // tile barrier that follows the writer's wait for its own memory operations, so the row's loads may leave
  // with the prologue's and its store after the query arithmetic; with fewer the write comes first and blocks.
  const bool writes = a.kvc_new != nullptr && tok_end == len;
  const bool write_first = writes && t_end - t_begin < 3;
  if (write_first) {   // uniform over the workgroup
    if (wave == 7) {
      MlaRowRaw r;
      mla_new_row_load(a, seq, lane, r);
      mla_new_row_store(a, seq, len, lane, r);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
  }
  const bool write_late = writes && !write_first && wave == 7;

  // ---- cooperative tile load, straight from global memory into LDS (no registers in between): a
  //      wave's load instruction fills 1024 contiguous LDS bytes, lane i the 16-byte slot i, with
  //      whatever global chunk the lane names.  Slot s of a 16-row half holds row s / 36, chunk
  //      (s % 36) ^ swizzle(row) of that row (the two low bits of the chunk number xor bits 1..2 of
  //      the row), so the rows need no padding for conflict-free operand reads: with 16 lanes reading
  //      the same k-chunk of 16 consecutive rows, this swizzle measures free of bank conflicts, row
  //      padding and the other two-bit swizzles cost every such read twice its cycles.  Thread tid
  //      names the chunk of slot tid; the first wave also names slots 512 .. 575.
  uint32_t goff[2];
#pragma unroll
  for (int n = 0; n < 2; ++n) {
    const int slot = n == 0 ? tid : kMlaThreads + lane;
    const int row = slot / kChunksPerRow, pos = slot % kChunksPerRow;
    const int col = (pos & ~3) | ((pos & 3) ^ ((row >> 1) & 3));
    goff[n] = (uint32_t)(row * a.g.stride_row + 16 * col);
  }
  uint32_t scr[2];
  // Block ids of the two 16-token halves of tile t (scalar loads); a half past the end of the
  // sequence rereads its last valid half and is masked in the softmax.
  struct Blocks {
    int32_t b[2];
    int32_t s[2];  // first slot of the half inside its block
  };
  auto fetch_blocks = [&](int t) __attribute__((always_inline)) {
    Blocks r;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int tok = t * kTile + 16 * h;
      tok = tok < len ? tok : ((len - 1) & ~15);
      const int e = (int)__umulhi((uint32_t)tok, a.bs_magic);
      r.s[h] = tok - e * bs;
      r.b[h] = scalar_load_i32(bt_row, e);
    }
    return r;
  };
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto issue_loads = [&](const Blocks& nb, uint8_t* buf) __attribute__((always_inline)) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint8_t* pb = a.cache + (int64_t)nb.b[h] * a.g.stride_block;
      const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint8_t*>(pb + (int64_t)nb.s[h] * a.g.stride_row), 0, 0x7fffffff, 0x00020000);
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint8_t*>(pb + a.g.scale_off + (int64_t)nb.s[h] * 4), 0, 0x7fffffff, 0x00020000);
      uint8_t* hb = buf + h * (kChunksPerHalf * 16);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rr, (lds_ptr_t)(hb + wave * (kWave * 16)), 16, goff[0], 0, 0, 0);
      if (wave == 0)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rr, (lds_ptr_t)(hb + kMlaThreads * 16), 16, goff[1], 0, 0, 0);
      scr[h] = __builtin_amdgcn_raw_buffer_load_b32(rs, (uint32_t)((tid & 15) * 4), 0, 0);
    }
  };
  auto stage_scales = [&](uint8_t* buf) {
    if (tid < 16) {
      float* sc = reinterpret_cast<float*>(buf + kMlaTileBytes);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float v = as_f32(scr[h]);
        sc[h * 16 + tid] = v * a.scale_log2;                       // K side: scale * log2e folded in
        sc[kTile + h * 16 + tid] = fminf(v * kPScale, 65504.f);    // V side: 2^8, capped
      }
    }
  };
  // Barrier that also waits for this wave's loads into LDS (they count as vector memory loads).
  auto tile_barrier = [&]() __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };

  // ---- Q of the 16 heads this wave owns as int8 B operands (operand 2 kk = first term, 2 kk + 1 = second term
  //      of k-step kk; lane (c = head, g) holds dims 64 kk + 16 g + j)
  const int own_head = hgroup * 16 + c;
  const bool head_ok = own_head < a.num_heads;
  MlaQRaw<(QDT < 0 ? KVQ_BF16 : QDT)> qraw[QDT < 0 ? 1 : kMlaKSteps8];
  if constexpr (QDT >= 0) {
    if (owner) {
      const int64_t qbase = (int64_t)seq * a.q_stride_b + (int64_t)(head_ok ? own_head : 0) * a.q_stride_h + 16 * g;
      const int64_t pebase = (int64_t)seq * a.pe_stride_b + (int64_t)(head_ok ? own_head : 0) * a.pe_stride_h + 16 * g;
#pragma unroll
      for (int kk = 0; kk < kMlaKSteps8; ++kk) qraw[kk] = mla_load_q16_raw<QDT>(a, qbase, pebase, kk);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  issue_loads(fetch_blocks(t_begin), lds[0]);
  Blocks nb = fetch_blocks(t_begin + 1);
  MlaRowRaw new_row;
  if (write_late) mla_new_row_load(a, seq, lane, new_row);
  __builtin_amdgcn_sched_barrier(0);

  i32x4 qreg[kMlaQRegOps];
  float s1 = 1.f, s2 = 0.f;
  if (owner) {
    if constexpr (QDT < 0) {
      const int64_t qblock = (int64_t)seq * a.head_groups + hgroup;
      const u32x4* qsrc = reinterpret_cast<const u32x4*>(a.q_ops + qblock * (kMlaQOps * kWave * 16)) + (4 * c + g);
      u32x4 raw[kMlaQOps];
#pragma unroll
      for (int op = 0; op < kMlaQOps; ++op) raw[op] = qsrc[op * kWave];
      s1 = a.q_scale[qblock * 16 + c];
#pragma unroll
      for (int op = 0; op < kMlaQOps; ++op) {
        if (op < kMlaQRegOps) qreg[op] = __builtin_bit_cast(i32x4, raw[op]);
        else qlds[(op - kMlaQRegOps) * kMlaThreads] = raw[op];
      }
    } else {   // the two int8 terms of the wave's own 16 heads
      float f[kMlaKSteps8][16];
#pragma unroll
      for (int kk = 0; kk < kMlaKSteps8; ++kk) mla_q16_to_float<QDT>(qraw[kk], f[kk]);
      float amax = 0.f;
#pragma unroll
      for (int kk = 0; kk < kMlaKSteps8; ++kk)
#pragma unroll
        for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(f[kk][i]));
      amax = max_over_quarters(amax);
      amax = head_ok ? fminf(amax, 3.0e38f) : 0.f;      // heads past the end contribute zero columns
      s1 = amax > 0.f ? amax / kMlaQ1Max : 1.0f;
#pragma unroll
      for (int kk = 0; kk < kMlaKSteps8; ++kk) {
        u32x4 ta, tb;
        mla_two_int8_terms(f[kk], s1, head_ok, ta, tb);
        if (2 * kk < kMlaQRegOps) {
          qreg[2 * kk] = __builtin_bit_cast(i32x4, ta);
          qreg[2 * kk + 1] = __builtin_bit_cast(i32x4, tb);
        } else {
          qlds[(2 * kk - kMlaQRegOps) * kMlaThreads] = ta;
          qlds[(2 * kk + 1 - kMlaQRegOps) * kMlaThreads] = tb;
        }
      }
    }
    s2 = s1 / kMlaQ2;
  } else {
#pragma unroll
    for (int op = 0; op < kMlaQRegOps; ++op) qreg[op] = (i32x4){0, 0, 0, 0};
  }

  if (write_late) mla_new_row_store(a, seq, len, lane, new_row);

  // o[ht][b][i]: head 16 ht + c, dim 64 wave + 16 g + 4 i + b
  floatx4 o[8][4];
#pragma unroll
  for (int ht = 0; ht < 8; ++ht)
#pragma unroll
    for (int b = 0; b < 4; ++b) o[ht][b] = (floatx4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // ---- V^T operands of the tile, built in registers from the raw tile.  Wave w accumulates dims
  //      64 w .. 64 w + 63 of all heads; output tile 4 w + b, row r' is dim 64 w + 4 r' + b.  A lane (r', g)
  //      reads one dword -- its four dims -- from each of the 8 token rows its P~ operand holds (k slot j of
  //      quarter g is token 16 (j / 4) + 4 g + j % 4) and turns each dim's 8 codes into one fp16 A operand
  //      with sign-extending sub-dword conversions (two instructions per pair of codes, no shuffles).  Rows 4 g + i and 16 + 4 g + i share their swizzle
  //      in pairs: two loop-invariant offsets, the rest are immediates.
  const uint32_t vo_a = (uint32_t)(4 * g * kMlaPitch + 16 * (4 * wave + ((c >> 2) ^ ((2 * g) & 3))) + 4 * (c & 3));
  const uint32_t vo_b = (uint32_t)(4 * g * kMlaPitch + 16 * (4 * wave + ((c >> 2) ^ ((2 * g + 1) & 3))) + 4 * (c & 3));
  auto v_operands = [&](const uint8_t* tile, half8_t (&va)[4]) __attribute__((always_inline)) {
    uint32_t x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      x[j] = *reinterpret_cast<const uint32_t*>(tile + ((j & 2) ? vo_b : vo_a) + (16 * (j >> 2) + (j & 3)) * kMlaPitch);
    va[0] = mla_code_rows_to_operand<0>(x);
    va[1] = mla_code_rows_to_operand<1>(x);
    va[2] = mla_code_rows_to_operand<2>(x);
    va[3] = mla_code_rows_to_operand<3>(x);
  };

  stage_scales(lds[0]);
  // every load so far (Q operands, the first tile) has landed; said with the builtin so that the
  // compiler knows it too and does not wait for loads again inside the loop, where a wait for
  // "all loads" would also wait for the tile prefetch in flight
  __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
  if (t_begin + 1 < t_end) issue_loads(nb, lds[1]);
  nb = fetch_blocks(t_begin + 2);
  lds_barrier();

  const uint32_t ka_off = (uint32_t)(c * kMlaPitch + 16 * (g ^ ((c >> 1) & 3)));   // row c, chunk g of a k-step, swizzled
  int buf = 0;   // parity of the exchange area
  int cur = 0;   // raw window of tile t; t + 1 is in cur + 1, t + 2 streams into cur + 2 (mod 3)
  for (int t = t_begin; t < t_end; ++t) {
    const uint8_t* tile = lds[cur];
    const int nxt = cur == kMlaRing - 1 ? 0 : cur + 1;
    const int nxt2 = nxt == kMlaRing - 1 ? 0 : nxt + 1;
    const float* sck = reinterpret_cast<const float*>(tile + kMlaTileBytes);
    uint8_t* xb = xchg + buf * kMlaXchgBytes;         // this tile's P~ operands, rescale factors, flags
    float* x_alpha = reinterpret_cast<float*>(xb + kMlaPBytes);
    uint8_t* x_flag = xb + kMlaPBytes + 128 * 4;

    if (owner) {
      // ---- S^T[32 tokens, 16 heads] on the int8 MFMA: A = the cached code bytes as they are, lane
      //      (r = token, g): dims 64 kk + 16 g ..; one accumulator per term of Q
      i32x4 acc[2][2];
#pragma unroll
      for (int term = 0; term < 2; ++term)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) acc[term][mt] = (i32x4){0, 0, 0, 0};
      // the operands of k-step kk + 1 are fetched before the products of k-step kk are issued;
      // the fences hold the compiler to that order
      const uint8_t* kap = tile + ka_off;
      i32x4 ka[2][2], ql[2][2];
      ka[0][0] = *reinterpret_cast<const i32x4*>(kap);
      ka[0][1] = *reinterpret_cast<const i32x4*>(kap + 16 * kMlaPitch);
#pragma unroll
      for (int kk = 0; kk < kMlaKSteps8; ++kk) {
        const int cur = kk & 1, nxt = cur ^ 1;
        if (kk + 1 < kMlaKSteps8) {
          ka[nxt][0] = *reinterpret_cast<const i32x4*>(kap + 64 * (kk + 1));
          ka[nxt][1] = *reinterpret_cast<const i32x4*>(kap + 16 * kMlaPitch + 64 * (kk + 1));
          if (2 * (kk + 1) >= kMlaQRegOps) {
            ql[nxt][0] = __builtin_bit_cast(i32x4, qlds[(2 * (kk + 1) - kMlaQRegOps) * kMlaThreads]);
            ql[nxt][1] = __builtin_bit_cast(i32x4, qlds[(2 * (kk + 1) + 1 - kMlaQRegOps) * kMlaThreads]);
          }
        }
        const i32x4 qa = 2 * kk < kMlaQRegOps ? qreg[2 * kk < kMlaQRegOps ? 2 * kk : 0] : ql[cur][0];
        const i32x4 qb8 = 2 * kk < kMlaQRegOps ? qreg[2 * kk < kMlaQRegOps ? 2 * kk + 1 : 0] : ql[cur][1];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          acc[0][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[cur][mt], qa, acc[0][mt], 0, 0, 0);
          acc[1][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[cur][mt], qb8, acc[1][mt], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }

      // ---- softmax, log2 domain; lane (c, g) holds tokens mt*16 + 4g + i of head c.  Only a split's
      //      last tile can hold tokens past its end: every other tile takes the path without masks.
      auto softmax = [&](auto masked_tag) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        // The two integer sums are joined with one shift-add (256 a.k + b.k, below 2^31 for any codes) and the
        // exponents formed straight away against the reference maximum as it stands -- which is right whenever
        // it does not move, and it rarely does: the reference maximum m of a head only has to keep 2^(logit - m)
        // in range, it need not be the true maximum.  It moves when some head of the tile outgrows it by more
        // than 2^kLazyMax (or at all, when a token's value scale is so large that p * scale could leave the fp16
        // range otherwise).  Moving m rescales what is accumulated so far, and the accumulators of these
        // heads are spread over all waves, so the factors travel with the tile.
        const bool first = m == -INFINITY;
        const float mref = first ? 0.f : m;   // while there is no maximum yet: the logits themselves
        float e[8];
        float emax = -INFINITY;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const floatx4 ks = *reinterpret_cast<const floatx4*>(sck + 16 * mt + 4 * g);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float x = __builtin_fmaf((float)((acc[0][mt][i] << 8) + acc[1][mt][i]), s2 * ks[i], -mref);
            if constexpr (MASKED) x = t * kTile + 16 * mt + 4 * g + i < tok_end ? x : -INFINITY;
            e[4 * mt + i] = x;
            emax = fmaxf(emax, x);
          }
        }
        emax = max_over_quarters(emax);
        floatx4 vs[2];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) vs[mt] = *reinterpret_cast<const floatx4*>(sck + kTile + 16 * mt + 4 * g);
        const float vsmax = fmaxf(fmaxf(fmaxf(vs[0].x, vs[0].y), fmaxf(vs[0].z, vs[0].w)),
                                  fmaxf(fmaxf(vs[1].x, vs[1].y), fmaxf(vs[1].z, vs[1].w)));
        const float lim = vsmax > kLazyScaleMax ? 0.f : kLazyMax;
        const bool moved = __builtin_amdgcn_ballot_w64(first || emax > lim) != 0;
        if (moved) {   // the new reference is the largest logit, emax + mref; the exponents shift by the difference
          const float m_new = fmaxf(m, emax + mref);
          const float alpha = __builtin_amdgcn_exp2f(m - m_new);
          const float shift = m_new - mref;
          m = m_new;
          l *= alpha;
          if (g == 0) x_alpha[wave * 16 + c] = alpha;
#pragma unroll
          for (int i = 0; i < 8; ++i) e[i] -= shift;   // a masked token's exponent stays -inf
        }
        if (lane == 0) x_flag[wave] = moved ? 1 : 0;
        float pt[8];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float p = __builtin_amdgcn_exp2f(e[4 * mt + i]);   // 0 for a masked token
            l += p;
            pt[4 * mt + i] = p * vs[mt][i];
            // a slot past the end may hold any bit pattern as its scale: select, do not multiply by 0
            if constexpr (MASKED) pt[4 * mt + i] = t * kTile + 16 * mt + 4 * g + i < tok_end ? pt[4 * mt + i] : 0.f;
          }
        }
        u32x4 pb;
        pb.x = pack_half2(pt[0], pt[1]);
        pb.y = pack_half2(pt[2], pt[3]);
        pb.z = pack_half2(pt[4], pt[5]);
        pb.w = pack_half2(pt[6], pt[7]);
        reinterpret_cast<u32x4*>(xb)[wave * kWave + lane] = pb;
      };
      if ((t + 1) * kTile > tok_end) softmax(std::true_type{});
      else softmax(std::false_type{});
    }

    if (t + 1 < t_end) stage_scales(lds[nxt]);
    // The ONE barrier of a tile (it also waits for this wave's part of the next raw tile): P~, the
    // rescale factors and the next raw tile are visible to every wave.  The exchange area is double-buffered, so a wave that runs ahead into the next tile
    // writes the other half while slower waves still read this one.
    tile_barrier();
    // the window of tile t - 1 is free now (every wave is past its P~V): the tile after the next streams
    // into it, a whole tile time ahead of its use, while this tile's window still feeds the P~V below
    if (t + 2 < t_end) issue_loads(nb, lds[nxt2]);
    nb = fetch_blocks(t + 3);

    // ---- O^T[64 dims of this wave, 128 heads] += C^T . P~^T: A = the wave's four fp16 V^T operands, built
    //      from the raw tile in registers; B = head tile ht's P~ operand
    const u32x2 flags = *reinterpret_cast<const u32x2*>(x_flag);
    half8_t va[4];
    v_operands(tile, va);
    // (FULL) operand ht + 3 is fetched while tile ht multiplies; the first three leave with the
    // flags, before anything waits
    const u32x4* pl = reinterpret_cast<const u32x4*>(xb) + lane;
    u32x4 pq[8];
    if constexpr (FULL) {
      pq[0] = pl[0];
      pq[1] = pl[kWave];
      pq[2] = pl[2 * kWave];
    }
    const uint32_t f_lo = __builtin_amdgcn_readfirstlane(flags.x), f_hi = __builtin_amdgcn_readfirstlane(flags.y);
    if ((f_lo | f_hi) != 0) {   // some running maximum moved: rare after a split's first tiles
#pragma unroll
      for (int ht = 0; ht < 8; ++ht) {
        const uint32_t f = ((ht < 4 ? f_lo : f_hi) >> (8 * (ht & 3))) & 0xffu;
        if (ht < nht && f != 0) {
          const float alpha = x_alpha[ht * 16 + c];
#pragma unroll
          for (int b = 0; b < 4; ++b) o[ht][b] *= alpha;
        }
      }
    }
    if constexpr (FULL) {   // one straight run of 8 operand reads and 32 MFMAs
      // the fences keep the compiler from hoisting all eight fetches (it would spill)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ht = 0; ht < 8; ++ht) {
        if (ht + 3 < 8) pq[ht + 3] = pl[(ht + 3) * kWave];
        const half8_t p_op = __builtin_bit_cast(half8_t, pq[ht]);
#pragma unroll
        for (int b = 0; b < 4; ++b) o[ht][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[b], p_op, o[ht][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int ht = 0; ht < 8; ++ht) {
        if (ht < nht) {
          const half8_t p_op = __builtin_bit_cast(half8_t, reinterpret_cast<const u32x4*>(xb)[ht * kWave + lane]);
#pragma unroll
          for (int b = 0; b < 4; ++b) o[ht][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[b], p_op, o[ht][b], 0, 0, 0);
        }
      }
    }
    buf ^= 1;
    cur = nxt;
  }

  // ---- emit the split's state: locally normalised output and its log2-domain lse.  The owners pass
  //      1 / l of their heads to every wave through the exchange half the last tile did not use.
  l = sum_over_quarters(l);
  float* x_inv = reinterpret_cast<float*>(xchg + buf * kMlaXchgBytes + kMlaPBytes);
  if (owner && g == 0) x_inv[wave * 16 + c] = 1.0f / (l * kPScale);
  lds_barrier();
  if (a.out != nullptr) {   // one split per sequence: the state is the result
#pragma unroll
    for (int ht = 0; ht < 8; ++ht) {
      const int head = (blockIdx.z * 8 + ht) * 16 + c;
      if (ht < nht && head < a.num_heads) {
        const float inv = x_inv[ht * 16 + c];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          mla_store_out4(a, ((int64_t)seq * a.num_heads + head) * kMlaR + 64 * wave + 16 * g + 4 * i,
                         (floatx4){o[ht][0][i] * inv, o[ht][1][i] * inv, o[ht][2][i] * inv, o[ht][3][i] * inv});
      }
    }
    if (owner && g == 0 && hgroup * 16 + c < a.num_heads && a.lse_out != nullptr)
      a.lse_out[(int64_t)seq * a.num_heads + hgroup * 16 + c] = (m + __builtin_amdgcn_logf(l)) * kLn2;
    return;
  }
#pragma unroll
  for (int ht = 0; ht < 8; ++ht) {
    if (ht < nht) {
      const float inv = x_inv[ht * 16 + c];
      uint16_t* po = a.part_o + (pblock0 + ht) * (16 * kMlaR) + lane * 4 + wave * 4 * 256;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        u32x2 v;  // a locally normalised output is a convex mix of dequantised rows: within fp16 range
        v.x = pack_half2(clamp_half_range(o[ht][0][i] * inv), clamp_half_range(o[ht][1][i] * inv));
        v.y = pack_half2(clamp_half_range(o[ht][2][i] * inv), clamp_half_range(o[ht][3][i] * inv));
        *reinterpret_cast<u32x2*>(po + i * 256) = v;
      }
    }
  }
  if (owner && g == 0) a.part_lse[(pblock0 + wave) * 16 + c] = m + __builtin_amdgcn_logf(l);
}

// ---------------------------------------------------------------------------------------------
// At most 16 heads (one head tile: a tensor-parallel shard of a 128-head model, or a small model).
//
// With one head tile the kernel above has one wave computing logits while seven wait, and a tile takes
// as long as with 128 heads.  Here every wave streams its OWN tiles (wave w of four: tiles t_begin + w, + 4, ...)
// and nothing is exchanged inside the tile loop: the wave loads a tile's rows from global memory straight
// into registers in the int8 MFMA's A layout (lane = token, 16 consecutive dims: every byte is loaded
// once, by the lane that multiplies it), computes the logits of its 16 heads against the Q operands it
// keeps in registers, runs the softmax -- whose result already IS the P~ operand of the second product -- and copies
// the rows' first 512 bytes into a wave-private, chunk-swizzled LDS window, from which it builds the fp16
// V^T operands of all 512 output dims with dword reads and sub-dword conversions (as the kernel above does
// for its 64).  At the end the four waves' states are summed through the (then idle) windows, each wave
// adding up and emitting the 128 output dims of its number.
constexpr int kMlaSmallWin = kTile * kMlaR;                                   // 16384: a tile's V part
constexpr int kMlaSmallQBytes = kMlaQOps * kWave * 16 + 256 + 2048;           // Q operands, the waves' maxima of |q|, (m, l) of the waves
constexpr int kMlaSmallWaves = 4;   // one wave per SIMD: a wave may then use the whole register file (512 per lane)
constexpr int kMlaSmallThreads = kMlaSmallWaves * kWave;
constexpr int kMlaSmallLdsBytes = kMlaSmallWaves * kMlaSmallWin + kMlaSmallQBytes;         // 86272

// QDT >= 0: the kernel prepares the int8 operands of Q itself from the query rows of that type (every wave
// for itself, in registers, under the latency of its first tile); QDT < 0: they were prepared by the
// absorption kernel and are read from the workspace.
template <int QDT>
__global__ __launch_bounds__(kMlaSmallThreads) void mla_decode_small_kernel(MlaArgs a) {
  extern __shared__ __align__(16) uint8_t lds_raw[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, g = lane >> 4;
  uint8_t* win = lds_raw + wave * kMlaSmallWin;
  int seq, split;
  mla_seq_split_of_block(gridDim.y, a.num_splits, seq, split);
  const int len = a.seq_lens[seq];
  const int slen = mla_split_len(len > 0 ? len : 0, a.num_splits);
  const int tok_begin = split * slen;
  const int tok_end = min(len, tok_begin + slen);
  const int64_t pblock = ((int64_t)seq * a.num_splits + split) * a.head_groups;
  if (tok_begin >= tok_end) {  // empty split (uniform over the workgroup): mark it and leave
    if (a.out != nullptr) {    // the sequence's only split: an empty sequence, zeros and lse = -inf
      if (c < a.num_heads) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            mla_store_out4(a, ((int64_t)seq * a.num_heads + c) * kMlaR + 64 * (2 * wave + h) + 16 * g + 4 * i, (floatx4){0.f, 0.f, 0.f, 0.f});
        if (wave == 0 && g == 0 && a.lse_out != nullptr) a.lse_out[(int64_t)seq * a.num_heads + c] = -INFINITY;
      }
      return;
    }
    if (wave == 0 && g == 0) a.part_lse[pblock * 16 + c] = -INFINITY;
    return;
  }
  const int t_begin = tok_begin / kTile, t_end = (tok_end + kTile - 1) / kTile;
  const int bs = a.g.block_size;
  const int32_t* bt_row = a.block_table + (int64_t)seq * a.bt_stride;
  // Fused write: the wave that streams the sequence's last tile stores the new row.  A wave's tiles are its own;
  // with three tiles or more of its own, the last one is requested after waits that cover the store, so the
  // row's loads leave with the prologue's and its store after the query arithmetic; with fewer the write comes
  // first and blocks.
  const int my_tiles = t_begin + wave < t_end ? (t_end - 1 - (t_begin + wave)) / kMlaSmallWaves + 1 : 0;
  const bool writes = a.kvc_new != nullptr && tok_end == len && wave == ((t_end - 1 - t_begin) & (kMlaSmallWaves - 1));
  const bool write_late = writes && my_tiles >= 3;
  if (writes && !write_late) {   // uniform over the wave
    MlaRowRaw r;
    mla_new_row_load(a, seq, lane, r);
    mla_new_row_store(a, seq, len, lane, r);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }

  // ---- one tile's rows in registers: k[mt][kk] = row 16 mt + c, dims 64 kk + 16 g .. + 15; ks[mt] = the
  //      scales of tokens 16 mt + 4 g .. + 3 (the four logits a lane holds per half)
  struct Rows {
    u32x4 k[2][kMlaKSteps8];
    floatx4 ks[2];
  };
  // Block numbers are read one tile ahead of the rows that need them: a block-table read that misses the
  // scalar cache costs a trip to memory, and the row loads behind it cannot leave before it returns.
  struct TileIds {
    int blk[2];
  };
  auto tile_tok = [&](int t, int h) __attribute__((always_inline)) {
    const int tok = t * kTile + 16 * h;
    return tok < len ? tok : ((len - 1) & ~15);   // a half past the end rereads the last valid half and is masked
  };
  auto load_ids = [&](int t, TileIds& ids) __attribute__((always_inline)) {
#pragma unroll
    for (int h = 0; h < 2; ++h) ids.blk[h] = scalar_load_i32(bt_row, (int)__umulhi((uint32_t)tile_tok(t, h), a.bs_magic));
  };
  // Where a tile's rows start for this lane; the loads themselves leave in pieces (a k-step of both halves at
  // a time), spread over the arithmetic of the tile before: four waves that issue 18 KB each at the same
  // moment queue up behind the CU's one address unit.
  struct RowPtrs {
    const uint8_t* row[2];
    const uint8_t* sc[2];
  };
  auto row_ptrs = [&](int t, const TileIds& ids) __attribute__((always_inline)) {
    RowPtrs rp;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int tok = tile_tok(t, h);
      const int slot = tok - (int)__umulhi((uint32_t)tok, a.bs_magic) * bs;
      const uint8_t* pb = a.cache + (int64_t)ids.blk[h] * a.g.stride_block;
      rp.row[h] = pb + (int64_t)(slot + c) * a.g.stride_row + 16 * g;
      rp.sc[h] = pb + a.g.scale_off + (int64_t)(slot + 4 * g) * 4;
    }
    return rp;
  };
  auto load_scales = [&](const RowPtrs& rp, Rows& rr) __attribute__((always_inline)) {
#pragma unroll
    for (int h = 0; h < 2; ++h) rr.ks[h] = *reinterpret_cast<const floatx4_a4*>(rp.sc[h]);
  };
  auto load_ksteps = [&](const RowPtrs& rp, Rows& rr, int kk0, int kk1) __attribute__((always_inline)) {
#pragma unroll
    for (int kk = kk0; kk < kk1; ++kk)
#pragma unroll
      for (int h = 0; h < 2; ++h) rr.k[h][kk] = *reinterpret_cast<const u32x4_a4*>(rp.row[h] + 64 * kk);
  };

  // ---- Q operands of the sequence's heads in registers (a wave owns the whole register file), s1 per head.
  //      Order of the prologue: the loads of Q leave first (they need nothing but the sequence number), the
  //      wave's first tile follows as soon as its block numbers are known, and the arithmetic on Q runs while
  //      the tile is on its way.  The four waves share that arithmetic (wave v: k-steps v, v + 4, v + 8) and
  //      pass the operands round through LDS.
  constexpr int kMine = 3;
  const int64_t qblock = (int64_t)seq * a.head_groups;
  i32x4 qreg[kMlaQOps];
  float s1;
  MlaQRaw<(QDT < 0 ? KVQ_BF16 : QDT)> qraw[kMine];
  const bool head_ok = c < a.num_heads;
  if constexpr (QDT < 0) {
    const u32x4* qsrc = reinterpret_cast<const u32x4*>(a.q_ops + qblock * (kMlaQOps * kWave * 16)) + (4 * c + g);
#pragma unroll
    for (int op = 0; op < kMlaQOps; ++op) qreg[op] = __builtin_bit_cast(i32x4, qsrc[op * kWave]);
    s1 = a.q_scale[qblock * 16 + c];
  } else {
    const int64_t qbase = (int64_t)seq * a.q_stride_b + (int64_t)(head_ok ? c : 0) * a.q_stride_h + 16 * g;
    const int64_t pebase = (int64_t)seq * a.pe_stride_b + (int64_t)(head_ok ? c : 0) * a.pe_stride_h + 16 * g;
#pragma unroll
    for (int n = 0; n < kMine; ++n) qraw[n] = mla_load_q16_raw<QDT>(a, qbase, pebase, min(wave + 4 * n, kMlaKSteps8 - 1));
  }
  __builtin_amdgcn_sched_barrier(0);
  Rows rr;
  TileIds ids;
  {  // unconditional (a wave without a tile reads rows it will not use; the addresses are clamped to the
     // sequence): behind a branch, the wait for Q below would have to be a wait for every load
    load_ids(t_begin + wave, ids);
    const RowPtrs rp = row_ptrs(t_begin + wave, ids);
    load_scales(rp, rr);
    load_ksteps(rp, rr, 0, kMlaKSteps8);
    load_ids(t_begin + wave + kMlaSmallWaves, ids);
  }
  MlaRowRaw new_row;
  if (write_late) mla_new_row_load(a, seq, lane, new_row);
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (QDT >= 0) {
    u32x4* qstage = reinterpret_cast<u32x4*>(lds_raw + kMlaSmallWaves * kMlaSmallWin);     // [18 operands][64 lanes]
    float* part_max = reinterpret_cast<float*>(lds_raw + kMlaSmallWaves * kMlaSmallWin + kMlaQOps * kWave * 16);
    float f[kMine][16];
#pragma unroll
    for (int n = 0; n < kMine; ++n) mla_q16_to_float<QDT>(qraw[n], f[n]);
    float amax = 0.f;
#pragma unroll
    for (int n = 0; n < kMine; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(f[n][i]));
    amax = max_over_quarters(amax);
    if (g == 0) part_max[wave * 16 + c] = amax;
    lds_barrier();   // LDS only: the tile's loads stay in flight
    amax = fmaxf(fmaxf(part_max[c], part_max[16 + c]), fmaxf(part_max[32 + c], part_max[48 + c]));
    amax = head_ok ? fminf(amax, 3.0e38f) : 0.f;      // heads past the end contribute zero columns
    s1 = amax > 0.f ? amax / kMlaQ1Max : 1.0f;
#pragma unroll
    for (int n = 0; n < kMine; ++n) {
      const int kk = wave + 4 * n;
      u32x4 ta, tb;
      mla_two_int8_terms(f[n], s1, head_ok, ta, tb);
      if (kk < kMlaKSteps8) {
        qstage[(2 * kk) * kWave + lane] = ta;
        qstage[(2 * kk + 1) * kWave + lane] = tb;
      }
    }
    lds_barrier();
#pragma unroll
    for (int op = 0; op < kMlaQOps; ++op) qreg[op] = __builtin_bit_cast(i32x4, qstage[op * kWave + lane]);
  }
  const float s2 = s1 / kMlaQ2;
  if (write_late) mla_new_row_store(a, seq, len, lane, new_row);

  floatx4 o[32];   // o[4 d4 + b][i]: head c, dim 64 d4 + 16 g + 4 i + b
#pragma unroll
  for (int j = 0; j < 32; ++j) o[j] = (floatx4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // V dwords of the lane's 8 tokens (k slot j of quarter g is token 16 (j / 4) + 4 g + j % 4) for the dims
  // 64 d4 + 4 c .. + 3: row pitch 512, 16-byte chunk number xor (row & 15), so that the four quarters of a
  // wave read four different quarters of the banks
  uint32_t vrow_off[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int row = 16 * (j >> 2) + 4 * g + (j & 3);
    vrow_off[j] = (uint32_t)(row * kMlaR + 16 * ((c >> 2) ^ (row & 3)) + 4 * (c & 3));
  }
  const int vflip = g;   // bits 2-3 of every one of the lane's rows: they toggle the low bits of the 64-dim group

  auto tile_step = [&](Rows& rr, TileIds& ids, int t) __attribute__((always_inline)) {
    // ---- S^T[32 tokens, 16 heads] on the int8 MFMA, one accumulator per term of Q
    i32x4 acc[2][2];
#pragma unroll
    for (int term = 0; term < 2; ++term)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) acc[term][mt] = (i32x4){0, 0, 0, 0};
#pragma unroll
    for (int kk = 0; kk < kMlaKSteps8; ++kk) {
      const i32x4 qa = qreg[2 * kk], qb8 = qreg[2 * kk + 1];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const i32x4 ka = __builtin_bit_cast(i32x4, rr.k[mt][kk]);
        acc[0][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka, qa, acc[0][mt], 0, 0, 0);
        acc[1][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka, qb8, acc[1][mt], 0, 0, 0);
      }
    }
    // ---- the rows' first 512 bytes into the window (chunk 4 kk + g of row 16 mt + c, swizzled)
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int kk = 0; kk < kMlaR / 64; ++kk)
        *reinterpret_cast<u32x4*>(win + (16 * mt + c) * kMlaR + 16 * ((4 * kk + g) ^ c)) = rr.k[mt][kk];
    const floatx4 sc0 = rr.ks[0], sc1 = rr.ks[1];
    // the row registers are free: the wave's next tile streams in under the rest of this one
    const bool more = t + kMlaSmallWaves < t_end;
    RowPtrs rp;
    if (more) {
      rp = row_ptrs(t + kMlaSmallWaves, ids);
      load_ids(t + 2 * kMlaSmallWaves, ids);
      load_scales(rp, rr);
      load_ksteps(rp, rr, 0, 2);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- softmax, log2 domain; lane (c, g) holds tokens 16 mt + 4 g + i of head c
    float logit[8];
    float mloc = -INFINITY;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float x = __builtin_fmaf((float)acc[1][mt][i], s2, (float)acc[0][mt][i] * s1) * ((mt ? sc1 : sc0)[i] * a.scale_log2);
        x = t * kTile + 16 * mt + 4 * g + i < tok_end ? x : -INFINITY;
        logit[4 * mt + i] = x;
        mloc = fmaxf(mloc, x);
      }
    }
    mloc = max_over_quarters(mloc);
    if (__builtin_amdgcn_ballot_w64(mloc > m) != 0) {   // some head's maximum moved
      const float m_new = fmaxf(m, mloc);
      const float alpha = __builtin_amdgcn_exp2f(m - m_new);
      const bool started = __builtin_amdgcn_ballot_w64(m != -INFINITY) != 0;
      m = m_new;
      l *= alpha;
      if (started) {   // before the wave's first tile the accumulators are zero
#pragma unroll
        for (int j = 0; j < 32; ++j) o[j] *= alpha;
      }
    }
    float pt[8];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(logit[4 * mt + i] - m);   // 0 for a masked token
        l += p;
        const float vs = fminf((mt ? sc1 : sc0)[i] * kPScale, 65504.f);
        // a slot past the end may hold any bit pattern as its scale: select, do not multiply by 0
        pt[4 * mt + i] = t * kTile + 16 * mt + 4 * g + i < tok_end ? p * vs : 0.f;
      }
    }
    u32x4 pb;
    pb.x = pack_half2(pt[0], pt[1]);
    pb.y = pack_half2(pt[2], pt[3]);
    pb.z = pack_half2(pt[4], pt[5]);
    pb.w = pack_half2(pt[6], pt[7]);
    const half8_t p_op = __builtin_bit_cast(half8_t, pb);
    __builtin_amdgcn_sched_barrier(0);
    if (more) load_ksteps(rp, rr, 2, 4);

    // ---- O^T[512 dims, 16 heads] += C^T . P~^T, 64 dims (four output tiles) at a time
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // group d4's four operands are converted while the products of group d4 - 1 run, from dwords read a
    // group earlier still
    uint32_t xq[2][8];
    half8_t va[2][4];
    auto read_group = [&](int d4) __attribute__((always_inline)) {
#pragma unroll
      for (int j = 0; j < 8; ++j) xq[d4 & 1][j] = *reinterpret_cast<const uint32_t*>(win + vrow_off[j] + 64 * (d4 ^ vflip));
    };
    auto convert_group = [&](int d4) __attribute__((always_inline)) {
      const uint32_t (&x)[8] = xq[d4 & 1];
      va[d4 & 1][0] = mla_code_rows_to_operand<0>(x);
      va[d4 & 1][1] = mla_code_rows_to_operand<1>(x);
      va[d4 & 1][2] = mla_code_rows_to_operand<2>(x);
      va[d4 & 1][3] = mla_code_rows_to_operand<3>(x);
    };
    read_group(0);
    read_group(1);
    convert_group(0);
#pragma unroll
    for (int d4 = 0; d4 < 8; ++d4) {
      if (d4 + 2 < 8) read_group(d4 + 2);
      if (d4 < 5 && more) load_ksteps(rp, rr, 4 + d4, 5 + d4);
#pragma unroll
      for (int b = 0; b < 4; ++b)
        o[4 * d4 + b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[d4 & 1][b], p_op, o[4 * d4 + b], 0, 0, 0);
      if (d4 + 1 < 8) convert_group(d4 + 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();   // the window is rewritten by the next tile
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  for (int t = t_begin + wave; t < t_end; t += kMlaSmallWaves) tile_step(rr, ids, t);

  // ---- the waves' states become one.  (m, l) of every wave meet behind the windows; each wave brings its
  //      accumulators to the common maximum and the common sum and drops them as fp16 (its share of a convex
  //      mix of dequantised rows: within fp16 range, and the state is emitted in fp16 anyway) into its own
  //      window; wave w then adds up, over the windows, the eight output tiles of ITS 128 dims (d4 = 2 w,
  //      2 w + 1) and emits them: the same split-state layout as the kernel above writes.
  float* ml = reinterpret_cast<float*>(lds_raw + kMlaSmallWaves * kMlaSmallWin + kMlaQOps * kWave * 16 + 256);   // [wave][m: 64 lanes | l: 64 lanes]
  ml[wave * 128 + lane] = m;
  ml[wave * 128 + 64 + lane] = l;
  __syncthreads();                                                   // ... and every wave is done with its window
  float m_all = -INFINITY;
#pragma unroll
  for (int w = 0; w < kMlaSmallWaves; ++w) m_all = fmaxf(m_all, ml[w * 128 + lane]);
  float l_all = 0.f;
#pragma unroll
  for (int w = 0; w < kMlaSmallWaves; ++w) {
    const float mw = ml[w * 128 + lane];
    l_all += mw == -INFINITY ? 0.f : ml[w * 128 + 64 + lane] * __builtin_amdgcn_exp2f(mw - m_all);
  }
  l_all = sum_over_quarters(l_all);
  // this wave's weight, with the normalisation folded in
  const float mine = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m_all) / (l_all * kPScale);
  {
    u32x2* mywin = reinterpret_cast<u32x2*>(win);
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      u32x2 v;
      v.x = pack_half2(clamp_half_range(o[j][0] * mine), clamp_half_range(o[j][1] * mine));
      v.y = pack_half2(clamp_half_range(o[j][2] * mine), clamp_half_range(o[j][3] * mine));
      mywin[j * kWave + lane] = v;
    }
  }
  __syncthreads();
  floatx4 sum[8];
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    floatx4 acc4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < kMlaSmallWaves; ++w) {
      const uint64_t v = reinterpret_cast<const uint64_t*>(lds_raw + w * kMlaSmallWin)[(8 * wave + b) * kWave + lane];
      const half4_t h = __builtin_bit_cast(half4_t, v);
      acc4 += (floatx4){(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
    }
    sum[b] = acc4;
  }
  if (a.out != nullptr) {   // one split per sequence: the state is the result
    if (c < a.num_heads) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          mla_store_out4(a, ((int64_t)seq * a.num_heads + c) * kMlaR + 64 * (2 * wave + h) + 16 * g + 4 * i,
                         (floatx4){sum[4 * h + 0][i], sum[4 * h + 1][i], sum[4 * h + 2][i], sum[4 * h + 3][i]});
      if (wave == 0 && g == 0 && a.lse_out != nullptr)
        a.lse_out[(int64_t)seq * a.num_heads + c] = (m_all + __builtin_amdgcn_logf(l_all)) * kLn2;
    }
    return;
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    uint16_t* po = a.part_o + pblock * (16 * kMlaR) + lane * 4 + (2 * wave + h) * 4 * 256;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      u32x2 v;
      v.x = pack_half2(clamp_half_range(sum[4 * h + 0][i]), clamp_half_range(sum[4 * h + 1][i]));
      v.y = pack_half2(clamp_half_range(sum[4 * h + 2][i]), clamp_half_range(sum[4 * h + 3][i]));
      *reinterpret_cast<u32x2*>(po + i * 256) = v;
    }
  }
  if (wave == 0 && g == 0) a.part_lse[pblock * 16 + c] = m_all + __builtin_amdgcn_logf(l_all);
}

// Stage 2: out = sum_j 2^(lse_j - max) o_j / sum_j 2^(lse_j - max); lse = ln 2 * (max + log2 sum).
// grid (B, ceil(H/16)), 8 waves; wave w combines the d4 = w slice of the block's 16 heads, lane (c, g)
// as in the split state layout.  RPT = 4: a thread takes its four 4-dim pieces of every split, eight splits per
// trip to memory.  RPT = 1 (grid.z = 4): one piece per thread and 32 splits per trip, for a few sequences cut
// into dozens of splits -- their grid is a handful of blocks, and eight splits per trip made 64 splits a chain
// of eight round trips (20 us for one 32k-token sequence, half as long as its decode kernel).
template <int ODT, int RPT>
__global__ __launch_bounds__(512) void mla_reduce_kernel(void* out, float* lse, const uint16_t* part_o,
                                                         const float* part_lse, const int32_t* seq_lens,
                                                         int num_heads, int head_groups, int num_splits) {
  constexpr int SPT = RPT == 4 ? 8 : 32;           // splits per trip
  const int r0 = RPT == 4 ? 0 : (int)blockIdx.z;   // the thread's first piece
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int seq = blockIdx.x, hgroup = blockIdx.y;
  const int head = hgroup * 16 + c;
  const bool head_ok = head < num_heads;
  const int64_t lstride = (int64_t)head_groups * 16;                    // part_lse stride between splits
  const float* pl = part_lse + ((int64_t)seq * num_splits * head_groups + hgroup) * 16 + c;
  const uint16_t* po = part_o + ((int64_t)seq * num_splits * head_groups + hgroup) * (16 * kMlaR) + (wave * 4 * 64 + lane) * 4 + r0 * 256;
  const int64_t ostride = (int64_t)head_groups * 16 * kMlaR;            // part_o stride between splits
  floatx4 acc[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) acc[r] = (floatx4){0.f, 0.f, 0.f, 0.f};
  float mx = -INFINITY;
  const bool live = seq_lens[seq] > 0;
  float den = 0.f;
  // Eight splits at a time, and all loads of a group -- the eight lse values and the eight states -- leave
  // before anything is computed from them: one trip to memory per group instead of two (the maximum first,
  // then the states).  The running maximum moves between groups, with the usual rescaling.
  // Every load is unconditional and a split that holds nothing (lse = -inf; its state rows were never
  // written) is removed with a bit mask on the loaded words: a select on the value would be turned into
  // a branch around the load, and the loads of successive splits would run one by one.
  for (int j0 = 0; j0 < num_splits; j0 += SPT) {
    float lj[SPT];
    u32x2 hv[SPT][RPT];
#pragma unroll
    for (int u = 0; u < SPT; ++u) {
      const int j = min(j0 + u, num_splits - 1);   // a slot past the last split rereads the last one and weighs 0
      lj[u] = pl[j * lstride];
      const uint16_t* pj = po + j * ostride;
#pragma unroll
      for (int r = 0; r < RPT; ++r) hv[u][r] = *reinterpret_cast<const u32x2*>(pj + r * 256);
    }
    float cm = -INFINITY;
#pragma unroll
    for (int u = 0; u < SPT; ++u) cm = fmaxf(cm, (live && j0 + u < num_splits) ? lj[u] : -INFINITY);
    const float m_new = fmaxf(mx, cm);
    const float mref = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = mx == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mx - mref);
    mx = m_new;
    den *= alpha;
#pragma unroll
    for (int r = 0; r < RPT; ++r) acc[r] *= alpha;
#pragma unroll
    for (int u = 0; u < SPT; ++u) {
      const bool on = live && j0 + u < num_splits && lj[u] != -INFINITY;
      const float wj = on ? __builtin_amdgcn_exp2f(lj[u] - mref) : 0.f;
      const uint32_t keep = wj != 0.f ? 0xffffffffu : 0u;
      den += wj;
#pragma unroll
      for (int r = 0; r < RPT; ++r) {
        const uint32_t h0 = hv[u][r].x & keep, h1 = hv[u][r].y & keep;
        const half2_t a0 = __builtin_bit_cast(half2_t, h0), a1 = __builtin_bit_cast(half2_t, h1);
        acc[r].x += (float)a0.x * wj;
        acc[r].y += (float)a0.y * wj;
        acc[r].z += (float)a1.x * wj;
        acc[r].w += (float)a1.y * wj;
      }
    }
  }
  if (!head_ok) return;
  const float inv = den > 0.f ? 1.0f / den : 0.f;                       // nothing attended: zeros
  const int64_t obase = ((int64_t)seq * num_heads + head) * kMlaR + 16 * g;
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int64_t o = obase + 64 * wave + 4 * (r0 + r);   // four consecutive dims: one store (rows are 1024 elements apart)
    const floatx4 v = acc[r] * inv;
    if constexpr (ODT == KVQ_F32) {
      *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(out) + o) = v;
    } else if constexpr (ODT == KVQ_BF16) {
      u32x2 w;
      w.x = (uint32_t)f32_to_bf16_bits(v.x) | ((uint32_t)f32_to_bf16_bits(v.y) << 16);
      w.y = (uint32_t)f32_to_bf16_bits(v.z) | ((uint32_t)f32_to_bf16_bits(v.w) << 16);
      *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(out) + o) = w;
    } else {
      u32x2 w;
      w.x = pack_half2(v.x, v.y);
      w.y = pack_half2(v.z, v.w);
      *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(out) + o) = w;
    }
  }
  if (lse != nullptr && wave == 0 && g == 0 && r0 == 0)
    lse[(int64_t)seq * num_heads + head] = den > 0.f ? (mx + __builtin_amdgcn_logf(den)) * kLn2 : -INFINITY;
}

// num_kv_splits policy of the reference (vllm_metax/v1/attention/backends/mla/triton_mla.py:45-55),
// additionally bounded so that (sequences x splits) does not far exceed the resident workgroups.
// In the batch-invariant mode every sequence is cut into kMlaInvariantSplits whatever the batch holds (the
// reference takes one split there, triton_mla.py:247-253; any count that does not depend on the batch serves).
constexpr int kMlaInvariantSplits = 8;
static int mla_num_splits(int max_seq_hint, int num_seqs, int num_heads) {
  (void)max_seq_hint;
  if (batch_invariant()) return kMlaInvariantSplits;
  const int cus = num_cus();
  const int groups = (num_heads + 127) / 128;
  int splits = 1;
  while (splits < 64 && (int64_t)num_seqs * groups * splits < (int64_t)cus) splits *= 2;
  return splits;
}

// The decode kernel needs more dynamic LDS than the 64 KB a kernel gets by default.  The opt-in is a
// per-device, per-kernel attribute; it is set the first time either entry
// point runs on a device -- the workspace query is the place a caller reaches before any stream
// capture, so a captured decode call finds it done.
static int mla_prepare_device() {
  static std::atomic<uint64_t> done_mask{0};  // one bit per device id < 64
  int dev = -1;
  if (int e = check_hip(hipGetDevice(&dev), "hipGetDevice")) return e;
  const uint64_t bit = dev >= 0 && dev < 64 ? (1ull << dev) : 0;
  if (bit != 0 && (done_mask.load(std::memory_order_acquire) & bit)) return KVQ_OK;
  const void* big[8] = {reinterpret_cast<const void*>(&mla_decode_kernel<true, -1>),
                        reinterpret_cast<const void*>(&mla_decode_kernel<true, KVQ_F32>),
                        reinterpret_cast<const void*>(&mla_decode_kernel<true, KVQ_BF16>),
                        reinterpret_cast<const void*>(&mla_decode_kernel<true, KVQ_F16>),
                        reinterpret_cast<const void*>(&mla_decode_kernel<false, -1>),
                        reinterpret_cast<const void*>(&mla_decode_kernel<false, KVQ_F32>),
                        reinterpret_cast<const void*>(&mla_decode_kernel<false, KVQ_BF16>),
                        reinterpret_cast<const void*>(&mla_decode_kernel<false, KVQ_F16>)};
  for (const void* k : big)
    if (int e = check_hip(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kMlaLdsBytes),
                          "hipFuncSetAttribute(mla_decode_kernel)"))
      return e;
  const void* small[4] = {reinterpret_cast<const void*>(&mla_decode_small_kernel<-1>),
                          reinterpret_cast<const void*>(&mla_decode_small_kernel<KVQ_F32>),
                          reinterpret_cast<const void*>(&mla_decode_small_kernel<KVQ_BF16>),
                          reinterpret_cast<const void*>(&mla_decode_small_kernel<KVQ_F16>)};
  for (const void* k : small)
    if (int e = check_hip(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kMlaSmallLdsBytes),
                          "hipFuncSetAttribute(mla_decode_small_kernel)"))
      return e;
  done_mask.fetch_or(bit, std::memory_order_release);
  return KVQ_OK;
}

// The step's new latent rows for the fused write: row i belongs to sequence i, position seq_lens[i] - 1.
struct MlaNewRows {
  const void* kv_c;
  const void* k_pe;
  int64_t kv_c_stride, k_pe_stride;  // elements
  int dtype;
  float eps;
};

}  // namespace kvq

// All entry points: `absorb` NULL = q holds the absorbed query (quantised by the decode kernel itself), else q
// is unused and the absorb kernel prepares the operands from (q_nope, W_UK_T, q_pe).  `fresh` non-NULL: the
// decode launch also writes the step's new rows into the cache.
static int mla_decode_run(const char* op, void* out, int out_dtype, float* lse, const void* q, int q_dtype,
                          int64_t q_stride_b, int64_t q_stride_h, const void* q_pe, int64_t q_pe_stride_b,
                          int64_t q_pe_stride_h, kvq::MlaAbsorbArgs* absorb, const void* cache,
                          const kvq_mla_geom* geom, const int32_t* block_table, int64_t bt_stride,
                          const int32_t* seq_lens, int num_seqs, int num_heads, float scale, void* workspace,
                          size_t workspace_bytes, kvq_stream_t stream, const kvq::MlaNewRows* fresh = nullptr) {
  using namespace kvq;
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(out && (q || absorb) && cache && block_table && seq_lens, "%s: NULL pointer", op);
  if (fresh != nullptr) {
    KVQ_REQUIRE(fresh->kv_c && fresh->k_pe, "%s: NULL kv_c / k_pe", op);
    KVQ_REQUIRE(fresh->dtype == KVQ_F32 || fresh->dtype == KVQ_BF16 || fresh->dtype == KVQ_F16,
                "%s: unknown src_dtype %d", op, fresh->dtype);
    const int esz = fresh->dtype == KVQ_F32 ? 4 : 2;
    KVQ_REQUIRE(((uintptr_t)fresh->kv_c % 4) == 0 && ((uintptr_t)fresh->k_pe % 4) == 0 &&
                    (fresh->kv_c_stride * esz) % 4 == 0 && (fresh->k_pe_stride * esz) % 4 == 0,
                "%s: kv_c / k_pe rows must be 4-byte aligned", op);
    KVQ_REQUIRE(fresh->eps >= 0.f, "%s: eps must not be negative", op);
  }
  KVQ_REQUIRE(num_seqs > 0 && num_seqs <= 65535 && num_heads > 0, "%s: num_seqs / num_heads out of range", op);
  KVQ_REQUIRE(((uintptr_t)out % 16) == 0, "%s: out must be 16-byte aligned", op);
  const kvq_mla_geom& g = *geom;
  KVQ_REQUIRE(g.kv_lora_rank == kMlaR && g.rope_dim == kMlaP,
              "%s: only kv_lora_rank 512 + rope 64 is built (got %d + %d)", op, g.kv_lora_rank, g.rope_dim);
  KVQ_REQUIRE(g.block_size > 0 && g.block_size % 16 == 0, "%s: block_size must be a multiple of 16", op);
  KVQ_REQUIRE((g.stride_block | g.stride_row | g.scale_off) % 4 == 0 && ((uintptr_t)cache % 4) == 0 &&
                  g.stride_row >= kMlaW && g.stride_row <= (1 << 20),
              "%s: cache strides must be 4-byte aligned and rows at least 576 bytes apart", op);
  const int qsz = q_dtype == KVQ_F32 ? 4 : 2;
  KVQ_REQUIRE(((uintptr_t)q % 4) == 0 && (q_stride_b * qsz) % 4 == 0 && (q_stride_h * qsz) % 4 == 0,
              "%s: q rows must be 4-byte aligned", op);
  if (q_pe == nullptr && absorb == nullptr) {   // joined [B, H, 576] rows
    q_pe = static_cast<const char*>(q) + (size_t)kMlaR * qsz;
    q_pe_stride_b = q_stride_b;
    q_pe_stride_h = q_stride_h;
  }
  KVQ_REQUIRE(((uintptr_t)q_pe % 4) == 0 && (q_pe_stride_b * qsz) % 4 == 0 && (q_pe_stride_h * qsz) % 4 == 0,
              "%s: q_pe rows must be 4-byte aligned", op);
  const int splits = mla_num_splits(0, num_seqs, num_heads);
  const int head_groups = (num_heads + 15) / 16;
  const size_t states = (size_t)num_seqs * head_groups * 16 * splits;
  const size_t qheads = (size_t)num_seqs * head_groups * 16;
  const size_t need = states * ((size_t)kMlaR * sizeof(uint16_t) + sizeof(float)) +
                      qheads * ((size_t)kMlaQOps * 64 + sizeof(float));
  KVQ_REQUIRE(workspace != nullptr && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0,
              "%s: workspace of %zu bytes (16-byte aligned) required, got %zu", op, need, workspace_bytes);
  MlaArgs a{};
  a.q = q;
  a.q_stride_b = q_stride_b;
  a.q_stride_h = q_stride_h;
  a.q_pe = q_pe;
  a.pe_stride_b = q_pe_stride_b;
  a.pe_stride_h = q_pe_stride_h;
  a.cache = static_cast<const uint8_t*>(cache);
  a.g = g;
  a.block_table = block_table;
  a.bt_stride = bt_stride;
  a.seq_lens = seq_lens;
  a.part_lse = static_cast<float*>(workspace);  // fp32 first, so both arrays keep their alignment
  a.q_scale = a.part_lse + states;
  a.part_o = reinterpret_cast<uint16_t*>(a.q_scale + qheads);
  a.q_ops = reinterpret_cast<uint8_t*>(a.part_o + states * kMlaR);   // 16-byte aligned: every part is a multiple of 64 bytes
  a.head_groups = head_groups;
  a.num_heads = num_heads;
  a.num_splits = splits;
  a.scale_log2 = scale * kLog2e;
  a.bs_magic = (uint32_t)((0x100000000ull + (uint64_t)g.block_size - 1) / (uint64_t)g.block_size);
  if (splits == 1) {   // nothing to merge: the decode kernel converts and stores its one state as the result
    KVQ_REQUIRE(out_dtype == KVQ_F32 || out_dtype == KVQ_BF16 || out_dtype == KVQ_F16, "%s: unknown out_dtype %d", op, out_dtype);
    a.out = out;
    a.lse_out = lse;
    a.out_dtype = out_dtype;
  }
  if (fresh != nullptr) {
    a.kvc_new = fresh->kv_c;
    a.kpe_new = fresh->k_pe;
    a.kvc_stride = fresh->kv_c_stride;
    a.kpe_stride = fresh->k_pe_stride;
    a.new_dtype = fresh->dtype;
    a.new_eps = fresh->eps;
  }
  hipStream_t s = as_stream(stream);
  dim3 grid(splits, num_seqs, (num_heads + 127) / 128);
  if (int e = mla_prepare_device()) return e;
  if (absorb != nullptr) {
    absorb->q_ops = a.q_ops;
    absorb->q_scale = a.q_scale;
    absorb->head_groups = head_groups;
    absorb->num_heads = num_heads;
    absorb->num_seqs = num_seqs;
    const int atiles = mla_absorb_tiles(num_seqs);
    absorb->seq_tiles = (num_seqs + 16 * atiles - 1) / (16 * atiles);
    absorb->group_major = head_groups % 8 == 0;
    dim3 agrid(head_groups * 16 * absorb->seq_tiles);
#define KVQ_MLAA_NB(T, K, N) hipLaunchKernelGGL((mla_absorb_q_kernel<T, K, N>), agrid, dim3(256), 0, s, *absorb)
#define KVQ_MLAA(T, K)                        \
  do {                                        \
    if (atiles == 1) KVQ_MLAA_NB(T, K, 1);      \
    else KVQ_MLAA_NB(T, K, 2);                  \
  } while (0)
    if (q_dtype == KVQ_BF16) {
      if (absorb->ksteps == 4) KVQ_MLAA(KVQ_BF16, 4);
      else KVQ_MLAA(KVQ_BF16, 0);
    } else {
      if (absorb->ksteps == 4) KVQ_MLAA(KVQ_F16, 4);
      else KVQ_MLAA(KVQ_F16, 0);
    }
#undef KVQ_MLAA
#undef KVQ_MLAA_NB
  } else if (q_dtype != KVQ_F32 && q_dtype != KVQ_BF16 && q_dtype != KVQ_F16) {
    return fail(KVQ_EINVAL, "%s: unknown q_dtype %d", op, q_dtype);
  }   // without absorption the decode kernels quantise the query themselves
  if (int e = check_hip(hipGetLastError(), "mla_decode_int8 query launch")) return e;
  if (head_groups == 1) {   // one head tile: every wave streams its own tiles
#define KVQ_MLAS(T) \
  hipLaunchKernelGGL((mla_decode_small_kernel<T>), dim3(splits, num_seqs), dim3(kMlaSmallThreads), kMlaSmallLdsBytes, s, a)
    if (absorb != nullptr) KVQ_MLAS(-1);
    else if (q_dtype == KVQ_F32) KVQ_MLAS(KVQ_F32);
    else if (q_dtype == KVQ_BF16) KVQ_MLAS(KVQ_BF16);
    else if (q_dtype == KVQ_F16) KVQ_MLAS(KVQ_F16);
    else return fail(KVQ_EINVAL, "%s: unknown q_dtype %d", op, q_dtype);
#undef KVQ_MLAS
  } else {
#define KVQ_MLAB(F, T) hipLaunchKernelGGL((mla_decode_kernel<F, T>), grid, dim3(kMlaThreads), kMlaLdsBytes, s, a)
#define KVQ_MLABQ(F)                              \
  do {                                            \
    if (absorb != nullptr) KVQ_MLAB(F, -1);       \
    else if (q_dtype == KVQ_F32) KVQ_MLAB(F, KVQ_F32);   \
    else if (q_dtype == KVQ_BF16) KVQ_MLAB(F, KVQ_BF16); \
    else KVQ_MLAB(F, KVQ_F16);                    \
  } while (0)
    if (head_groups % 8 == 0) KVQ_MLABQ(true);
    else KVQ_MLABQ(false);
#undef KVQ_MLABQ
#undef KVQ_MLAB
  }
  int rc = check_hip(hipGetLastError(), "mla_decode_int8 launch");
  if (rc) return rc;
  if (splits == 1) return KVQ_OK;   // the decode kernel wrote the result itself
  // a few blocks and dozens of splits: a piece per thread, 32 splits per trip, four times the blocks
  // (never in the batch-invariant mode, whose eight splits are merged in one trip by either kernel: the choice must
  // not depend on the batch)
  const bool fine = splits > 8 && 4 * num_seqs * head_groups <= num_cus();
  dim3 rgrid(num_seqs, head_groups, fine ? 4 : 1);
#define KVQ_MLAR(T)                                                                                                \
  do {                                                                                                             \
    if (fine)                                                                                                      \
      hipLaunchKernelGGL((mla_reduce_kernel<T, 1>), rgrid, dim3(512), 0, s, out, lse, a.part_o, a.part_lse,        \
                         seq_lens, num_heads, head_groups, splits);                                                \
    else                                                                                                           \
      hipLaunchKernelGGL((mla_reduce_kernel<T, 4>), rgrid, dim3(512), 0, s, out, lse, a.part_o, a.part_lse,        \
                         seq_lens, num_heads, head_groups, splits);                                                \
  } while (0)
  switch (out_dtype) {
    case KVQ_F32: KVQ_MLAR(KVQ_F32); break;
    case KVQ_BF16: KVQ_MLAR(KVQ_BF16); break;
    case KVQ_F16: KVQ_MLAR(KVQ_F16); break;
    default: return fail(KVQ_EINVAL, "%s: unknown out_dtype %d", op, out_dtype);
  }
#undef KVQ_MLAR
  return check_hip(hipGetLastError(), "mla_decode_int8 reduce launch");
}

extern "C" {

size_t kvq_mla_decode_workspace_bytes(int max_num_seqs, int num_heads, int kv_lora_rank) {
  if (max_num_seqs <= 0 || num_heads <= 0 || kv_lora_rank <= 0) return 0;
  if (kvq::mla_prepare_device() != KVQ_OK) return 0;
  // sequences x splits stays below max(2 x resident workgroups per head group, sequences)
  const size_t groups = ((size_t)num_heads + 127) / 128;
  size_t items = 2 * (size_t)kvq::num_cus() / groups;
  if (items < (size_t)max_num_seqs) items = (size_t)max_num_seqs;
  if (kvq::batch_invariant()) items = (size_t)kvq::kMlaInvariantSplits * (size_t)max_num_seqs;
  const size_t heads_padded = ((size_t)num_heads + 15) / 16 * 16;
  // split states (fp16 outputs + fp32 lse) and, per sequence, Q as two int8 terms + one scale per head
  return items * heads_padded * ((size_t)kv_lora_rank * sizeof(uint16_t) + sizeof(float)) +
         (size_t)max_num_seqs * heads_padded * ((size_t)kvq::kMlaQOps * 64 + sizeof(float));
}

int kvq_mla_decode_int8(void* out, int out_dtype, float* lse, const void* q, int q_dtype, int64_t q_stride_b,
                        int64_t q_stride_h, const void* q_pe, int64_t q_pe_stride_b, int64_t q_pe_stride_h,
                        const void* cache, const kvq_mla_geom* geom,
                        const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens, int num_seqs,
                        int num_heads, float scale, void* workspace, size_t workspace_bytes,
                        kvq_stream_t stream) {
  return mla_decode_run("mla_decode_int8", out, out_dtype, lse, q, q_dtype, q_stride_b, q_stride_h, q_pe, q_pe_stride_b,
                        q_pe_stride_h, nullptr, cache, geom, block_table, bt_stride, seq_lens, num_seqs, num_heads,
                        scale, workspace, workspace_bytes, stream);
}

int kvq_mla_decode_int8_fused_write(void* out, int out_dtype, float* lse, const void* q, int q_dtype,
                                    int64_t q_stride_b, int64_t q_stride_h, const void* q_pe, int64_t q_pe_stride_b,
                                    int64_t q_pe_stride_h, const void* kv_c, const void* k_pe, int src_dtype,
                                    int64_t kv_c_stride, int64_t k_pe_stride, float eps, void* cache,
                                    const kvq_mla_geom* geom, const int32_t* block_table, int64_t bt_stride,
                                    const int32_t* seq_lens, int num_seqs, int num_heads, float scale,
                                    void* workspace, size_t workspace_bytes, kvq_stream_t stream) {
  const kvq::MlaNewRows fresh{kv_c, k_pe, kv_c_stride, k_pe_stride, src_dtype, eps};
  return mla_decode_run("mla_decode_int8_fused_write", out, out_dtype, lse, q, q_dtype, q_stride_b, q_stride_h, q_pe,
                        q_pe_stride_b, q_pe_stride_h, nullptr, cache, geom, block_table, bt_stride, seq_lens, num_seqs,
                        num_heads, scale, workspace, workspace_bytes, stream, &fresh);
}

int kvq_mla_decode_absorb_int8(void* out, int out_dtype, float* lse, const void* q_nope, int q_dtype,
                               int64_t qn_stride_b, int64_t qn_stride_h, int nope_dim, const void* w_uk_t,
                               int64_t w_stride_h, int64_t w_stride_p, const void* q_pe, int64_t q_pe_stride_b,
                               int64_t q_pe_stride_h, const void* cache, const kvq_mla_geom* geom,
                               const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
                               int num_seqs, int num_heads, float scale, void* workspace, size_t workspace_bytes,
                               kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "mla_decode_absorb_int8";
  KVQ_REQUIRE(q_nope && w_uk_t && q_pe, "%s: NULL pointer", op);
  KVQ_REQUIRE(q_dtype == KVQ_BF16 || q_dtype == KVQ_F16, "%s: q_nope, W_UK_T and q_pe must be bf16 or fp16 (dtype %d)", op, q_dtype);
  KVQ_REQUIRE(nope_dim > 0 && nope_dim % 32 == 0, "%s: qk_nope_head_dim %d must be a multiple of 32", op, nope_dim);
  KVQ_REQUIRE(((uintptr_t)w_uk_t % 16) == 0 && w_stride_h % 8 == 0 && w_stride_p % 8 == 0 && w_stride_p >= kMlaR,
              "%s: W_UK_T rows must be 16-byte aligned and hold 512 contiguous dims", op);
  KVQ_REQUIRE(((uintptr_t)q_nope % 4) == 0 && qn_stride_b % 2 == 0 && qn_stride_h % 2 == 0 && ((uintptr_t)q_pe % 4) == 0 &&
                  q_pe_stride_b % 2 == 0 && q_pe_stride_h % 2 == 0, "%s: q_nope / q_pe rows must be 4-byte aligned", op);
  MlaAbsorbArgs ab{};
  ab.q_nope = q_nope;
  ab.qn_sb = qn_stride_b;
  ab.qn_sh = qn_stride_h;
  ab.w = w_uk_t;
  ab.w_sh = w_stride_h;
  ab.w_sp = w_stride_p;
  ab.q_pe = q_pe;
  ab.pe_sb = q_pe_stride_b;
  ab.pe_sh = q_pe_stride_h;
  ab.ksteps = nope_dim / 32;
  return mla_decode_run(op, out, out_dtype, lse, nullptr, q_dtype, 0, 0, q_pe, q_pe_stride_b, q_pe_stride_h, &ab, cache,
                        geom, block_table, bt_stride, seq_lens, num_seqs, num_heads, scale, workspace, workspace_bytes,
                        stream);
}

}  // extern "C"
