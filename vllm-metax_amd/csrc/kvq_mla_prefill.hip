// Varlen attention with LSE output for the MLA prefill (gfx950): the step between the latent cache's
// gather + dequantise and the LSE merge of the chunked-context loop, and the causal pass over the new
// tokens.  K arrives as the two pieces the layer already has -- k_nope [S, H, NOPE] out of kv_b_proj and
// the rope part k_pe [S, ROPE] shared by all heads -- so the concatenated [S, H, NOPE + ROPE] tensor is
// never built.
//
// Workgroup = 128 query rows of one (sequence, head): 4 waves x 2 blocks of 16 rows.  The keys are walked 32
// at a time; a tile's K rows (NOPE + ROPE wide) and V rows are brought into LDS once per workgroup
// (registers in between, one tile ahead, double-buffered: one barrier per tile) and every wave feeds its two
// row blocks from there, so a K or V byte is fetched from L2 once per 128 rows.  K rows are stored with
// their 16-byte chunks xor-swizzled by the row number, which makes the operand reads (16 rows x the same
// chunk) free of bank conflicts without padding.
// Both products are computed transposed so that every per-row quantity is lane-local:
//   S^T = K Q^T   A = K rows (lane = key, 8 consecutive d), B = Q (lane = query row): 16x16x32 MFMA of the
//                 input type; a lane ends up with 8 keys of ITS query row, so the row maximum is a
//                 reduction over the four quarter-waves and alpha / l stay in the lane.
//   O^T = V^T P^T B = P~ straight from the S^T registers (k slot j of quarter g is key 16 (j / 4) + 4 g +
//                 j % 4; any order works as long as V uses the same one).  A = V^T needs 8 keys of one
//                 dim per lane while a V row holds the dims of one key together: the LDS's transposing read
//                 (ds_read_b64_tr_b16) hands a lane four keys of one dim out of four rows, two of them make an
//                 operand, no register shuffles.  Output block i holds dims 16 i .. 16 i + 15; a lane ends
//                 with dims 16 i + 4 g .. + 3 of its own query row: 8-byte stores.
// Masked keys (beyond the sequence, or above the causal diagonal, which is aligned to the END of the
// keys as flash-attention does) get weight 0; their rows are clamped copies of the last valid key.
#include "kvq_attn_core.cuh"
#include "kvq_internal.h"

namespace kvq {

struct VarlenArgs {
  const void* q;
  const void* k_nope;
  const void* k_pe;
  const void* v;
  void* out;
  float* lse;
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t q_st, q_sh, kn_st, kn_sh, kpe_st, v_st, v_sh, out_st, out_sh, total_q;
  int causal;
  float scale_log2;
};

// acc + the two 16-bit floats of `pair` (fp16 or bf16).
template <int DT>
__device__ __forceinline__ float pair_sum(uint32_t pair, float acc) {
  if constexpr (DT == KVQ_F16) {
    const half2_t one = {(half_t)1.0f, (half_t)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, pair), one, acc, false);
  } else {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t one = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair), one, acc, false);
  }
}

template <int DT, int NOPE, int ROPE, int DV>
__global__ __launch_bounds__(256) void varlen_attn_kernel(VarlenArgs a) {
  constexpr int KSN = NOPE / 32, KSR = ROPE / 32, KS = KSN + KSR;   // k-steps of the QK product
  constexpr int DPL = DV / 16;                                      // dims per lane and output block
  constexpr int RB = 2;                                             // row blocks of 16 per wave
  constexpr int KC = (NOPE + ROPE) / 8, KCN = NOPE / 8;             // 16-byte chunks of a K row / of its nope part
  constexpr int VC = DV / 8;                                        // chunks of a V row
  // V rows carry 32 bytes of padding: the transposing reads of a quarter-wave take 32 bytes from each of four
  // successive rows, which the padding puts on different banks
  constexpr int V_PITCH = VC * 16 + 32;
  constexpr int K_BYTES = 32 * KC * 16, V_BYTES = 32 * V_PITCH;
  constexpr int KLD = (32 * KC + 255) / 256, VLD = (32 * VC + 255) / 256;   // chunk loads per thread and tile
  // fp16 weights are kept 2^8 larger so that small ones stay normal; l carries the same factor
  constexpr float kShift = DT == KVQ_F16 ? 8.f : 0.f;
  __shared__ __align__(16) uint8_t lds[2][K_BYTES + V_BYTES];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  // Workgroups go to the eight XCDs in turn by their linear number, and every XCD has its own L2.  The query
  // blocks of one (sequence, head) all stream the same keys: numbered so that they land on ONE XCD (possible when
  // the (sequence, head) pairs divide by eight), its L2 serves all but the first reader of a tile.
  int seq = blockIdx.z, head = blockIdx.y, qb = blockIdx.x;
  {
    const unsigned pairs = gridDim.y * gridDim.z;
    if ((pairs & 7u) == 0) {
      const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
      const unsigned j = lin >> 3;                             // the XCD's j-th workgroup
      const unsigned pair = (j / gridDim.x) * 8 + (lin & 7u);  // every eighth pair is this XCD's
      qb = (int)(j % gridDim.x);
      head = (int)(pair % gridDim.y);
      seq = (int)(pair / gridDim.y);
    }
  }
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  const int k_begin = a.cu_k[seq], k_len = a.cu_k[seq + 1] - k_begin;
  // the last query blocks see the most keys under the causal mask: they are launched first
  const int q0wg = ((int)gridDim.x - 1 - qb) * (64 * RB);
  if (q0wg >= q_len) return;   // uniform over the workgroup
  const int c = lane & 15, g = lane >> 4;
  // key j is visible to query row i iff j <= i + (k_len - q_len)
  const int diag = k_len - q_len;
  const int wg_rows_end = min(q_len, q0wg + 64 * RB);
  const int wg_k_end = a.causal ? max(0, min(k_len, wg_rows_end - 1 + diag + 1)) : k_len;
  const int num_tiles = (wg_k_end + 31) / 32;

  // ---- the wave's rows
  int q0[RB], my_limit[RB], blk_k_end[RB];
  u32x4 qop[RB][KS];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    q0[rb] = q0wg + (wave * RB + rb) * 16;
    const int qrow = min(q0[rb] + c, q_len - 1);   // rows past the end compute on a copy and are not stored
    const uint16_t* qp = static_cast<const uint16_t*>(a.q) + (int64_t)(q_begin + qrow) * a.q_st + (int64_t)head * a.q_sh + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) qop[rb][s] = *reinterpret_cast<const u32x4*>(qp + 32 * s);
    my_limit[rb] = a.causal ? max(0, min(k_len, q0[rb] + c + diag + 1)) : k_len;
    blk_k_end[rb] = q0[rb] >= q_len ? 0 : (a.causal ? max(0, min(k_len, q0[rb] + 15 + diag + 1)) : k_len);
  }
  const int wave_tiles = (max(blk_k_end[0], blk_k_end[1]) + 31) / 32;   // tiles this wave has anything to do in
  // the smallest limit among the wave's rows: tiles that end at or below it are visible to every row
  const int wave_min_limit = -wave_max_i32(-min(my_limit[0], my_limit[1]));

  floatx4 oacc[RB][DPL];
  float m[RB], l[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
    for (int i = 0; i < DPL; ++i) oacc[rb][i] = (floatx4){0.f, 0.f, 0.f, 0.f};
    m[rb] = -INFINITY;
    l[rb] = 0.f;
  }

  // ---- cooperative tile copy.  Every load is "buffer resource + a lane offset that never changes": the resources
  //      (scalar registers) are re-based on the tile's first key with scalar arithmetic, so the tile loop spends no
  //      vector instruction on addresses (as 64-bit pointers per chunk they were 64 of the ~230 vector instructions
  //      of a tile).  A resource ends with the sequence's last key: rows past it read as zeros and are masked.
  //      Thread tid owns chunks tid + 256 i of the tile's k_nope part, of its k_pe part and of its V rows.
  constexpr int KCR = KC - KCN;
  constexpr int NLD = (32 * KCN + 255) / 256, RLD = (32 * KCR + 255) / 256;
  static_assert(NLD + RLD >= KLD, "chunk loads");
  const uint8_t* kn_base = reinterpret_cast<const uint8_t*>(static_cast<const uint16_t*>(a.k_nope) + (int64_t)head * a.kn_sh);
  const uint8_t* kpe_base = reinterpret_cast<const uint8_t*>(a.k_pe);
  const uint8_t* v_base = reinterpret_cast<const uint8_t*>(static_cast<const uint16_t*>(a.v) + (int64_t)head * a.v_sh);
  const int64_t kn_row = a.kn_st * 2, kpe_row = a.kpe_st * 2, v_row_bytes = a.v_st * 2;   // bytes per key
  u32x4 nreg[NLD], rreg[RLD > 0 ? RLD : 1], vreg[VLD];
  uint32_t n_off[NLD], r_off[RLD > 0 ? RLD : 1], v_off[VLD];         // global: byte offset from the tile's first key
  uint32_t n_lds[NLD], r_lds[RLD > 0 ? RLD : 1], v_lds[VLD];         // LDS: byte offset in the tile's buffer
  auto swz = [](int row, int ch) { return KC % 8 == 0 ? (ch ^ (row & 7)) : (ch ^ ((row >> 1) & 3)); };
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int q = min(tid + 256 * i, 32 * KCN - 1), row = q / KCN, ch = q - row * KCN;
    n_off[i] = (uint32_t)(row * (int)kn_row + 16 * ch);
    n_lds[i] = (uint32_t)((row * KC + swz(row, ch)) * 16);
  }
#pragma unroll
  for (int i = 0; i < RLD; ++i) {
    const int q = min(tid + 256 * i, 32 * KCR - 1), row = q / KCR, ch = q - row * KCR;
    r_off[i] = (uint32_t)(row * (int)kpe_row + 16 * ch);
    r_lds[i] = (uint32_t)((row * KC + swz(row, KCN + ch)) * 16);
  }
#pragma unroll
  for (int i = 0; i < VLD; ++i) {
    const int q = min(tid + 256 * i, 32 * VC - 1), row = q / VC, ch = q - row * VC;
    v_off[i] = (uint32_t)(row * (int)v_row_bytes + 16 * ch);
    v_lds[i] = (uint32_t)(K_BYTES + row * V_PITCH + 16 * ch);
  }
  auto tile_rsrc = [&](const uint8_t* base, int64_t row_bytes, int t) __attribute__((always_inline)) {
    const int64_t left = (int64_t)(k_len - 32 * t) * row_bytes;     // bytes up to the end of the sequence's keys
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(base + (int64_t)(k_begin + 32 * t) * row_bytes), 0,
                                             (int)(left < 0x7fffffff ? left : 0x7fffffff), 0x00020000);
  };
  auto fetch = [&](int t) __attribute__((always_inline)) {
    const __amdgpu_buffer_rsrc_t rn = tile_rsrc(kn_base, kn_row, t), rv = tile_rsrc(v_base, v_row_bytes, t);
#pragma unroll
    for (int i = 0; i < NLD; ++i) nreg[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, n_off[i], 0, 0));
    if constexpr (RLD > 0) {
      const __amdgpu_buffer_rsrc_t rr = tile_rsrc(kpe_base, kpe_row, t);
#pragma unroll
      for (int i = 0; i < RLD; ++i) rreg[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, r_off[i], 0, 0));
    }
#pragma unroll
    for (int i = 0; i < VLD; ++i) vreg[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rv, v_off[i], 0, 0));
  };
  auto drop = [&](uint8_t* buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      if (tid + 256 * i < 32 * KCN) *reinterpret_cast<u32x4*>(buf + n_lds[i]) = nreg[i];
#pragma unroll
    for (int i = 0; i < RLD; ++i)
      if (tid + 256 * i < 32 * KCR) *reinterpret_cast<u32x4*>(buf + r_lds[i]) = rreg[i];
#pragma unroll
    for (int i = 0; i < VLD; ++i)
      if (tid + 256 * i < 32 * VC) *reinterpret_cast<u32x4*>(buf + v_lds[i]) = vreg[i];
  };

  if (num_tiles > 0) {
    fetch(0);
    drop(lds[0]);
    __syncthreads();
  }
  for (int t = 0; t < num_tiles; ++t) {
    const uint8_t* buf = lds[t & 1];
    if (t + 1 < num_tiles) fetch(t + 1);
    if (t < wave_tiles) {
      // a wave at its products and softmax outranks the waves of its SIMD that are moving the next tile or waiting at
      // the barrier (measured: 4 x 2048 causal tokens 576 -> 588 TFLOP/s, one 8192-token prompt 711 -> 725; with the
      // priority raised for the drop and the barrier instead, nothing changed)
      __builtin_amdgcn_s_setprio(1);
      // ---- S^T = K Q^T for the tile's two blocks of 16 keys, both row blocks off one operand read
      floatx4 sacc[RB][2];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) sacc[rb][0] = sacc[rb][1] = (floatx4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        const int row = 16 * blk + c;
        const uint8_t* krow = buf + row * (KC * 16);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const u32x4 ka = *reinterpret_cast<const u32x4*>(krow + swz(row, 4 * s + g) * 16);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) sacc[rb][blk] = mfma16<DT>(ka, qop[rb][s], sacc[rb][blk]);
        }
      }
      // ---- online softmax in base 2, per row block
      u32x4 pk[RB];
      float alpha[RB];
      bool moved = false;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        // the maximum is taken over the raw products (the scale is positive and the same for every key), so that
        // scale and maximum enter each logit in ONE multiply-add
        // only a tile that reaches past some row's limit (the causal diagonal, the end of the keys) is masked: a
        // uniform branch round the compares and selects, which work on the products where they lie
        if ((t + 1) * 32 > wave_min_limit) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int key = t * 32 + 16 * (j >> 2) + 4 * g + (j & 3);
            sacc[rb][j >> 2][j & 3] = key < my_limit[rb] ? sacc[rb][j >> 2][j & 3] : -INFINITY;
          }
        }
        float sc[8];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          sc[j] = sacc[rb][j >> 2][j & 3];
          mx = fmaxf(mx, sc[j]);
        }
        mx = max_over_quarters(mx) * a.scale_log2;
        const float m_new = fmaxf(m[rb], mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        alpha[rb] = __builtin_amdgcn_exp2f(m[rb] - m_use);
        moved = moved || m_new > m[rb];
        const float off = kShift - m_use;
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[j], a.scale_log2, off));   // a masked key: 2^-inf = 0
        m[rb] = m_new;
        pk[rb].x = pack2<DT>(p[0], p[1]);
        pk[rb].y = pack2<DT>(p[2], p[3]);
        pk[rb].z = pack2<DT>(p[4], p[5]);
        pk[rb].w = pack2<DT>(p[6], p[7]);
        // the row sum is that of the weights as the second product sees them (rounded to the input type): one
        // two-element dot product with ones per packed pair instead of two additions
        float psum = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) psum = pair_sum<DT>(pk[rb][w], psum);
        l[rb] = l[rb] * alpha[rb] + psum;
      }
      // ---- O^T = alpha O^T + V^T P^T.  The accumulators are rescaled only in the tiles in which some row's
      //      maximum moved (they live in accumulation registers: a rescale is a read, a multiply and a write
      //      of each); after a sequence's first tiles that is rare.
      if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int i = 0; i < DPL; ++i) oacc[rb][i] *= alpha[rb];
      }
      // V^T operands straight from the row-major tile with the LDS's transposing read (ds_read_b64_tr_b16): lane s
      // of a quarter-wave names the 8 bytes [key kb + s / 4][dims 16 i + 4 (s % 4) .. + 3] and receives
      // [keys kb .. kb + 3][dim 16 i + s]; two reads (kb = 4 g and 16 + 4 g, the keys of the lane's k slots) make
      // the A operand of output block i = dims 16 i .. 16 i + 15.
      {
        typedef short s4_t __attribute__((ext_vector_type(4)));
        typedef __attribute__((address_space(3))) s4_t* lds_s4_ptr;
        const uint8_t* v0 = buf + K_BYTES + (4 * g + (c >> 2)) * V_PITCH + 8 * (c & 3);
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
          const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(v0 + 32 * i)));
          const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(v0 + 16 * V_PITCH + 32 * i)));
          const u32x4 vt = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) oacc[rb][i] = mfma16<DT>(vt, pk[rb], oacc[rb][i]);
        }
      }
      __builtin_amdgcn_s_setprio(0);
    }
    if (t + 1 < num_tiles) drop(lds[(t + 1) & 1]);
    __syncthreads();
  }

#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const float l_tot = sum_over_quarters(l[rb]);
    const bool live = l_tot > 0.f;
    const float inv = live ? 1.f / l_tot : 0.f;
    if (q0[rb] + c >= q_len) continue;
    const int64_t tok = q_begin + q0[rb] + c;
    uint16_t* op = static_cast<uint16_t*>(a.out) + tok * a.out_st + (int64_t)head * a.out_sh;
    // block i: the lane holds dims 16 i + 4 g .. + 3 of its row
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      u32x2 w;
      w.x = pack2<DT>(oacc[rb][i][0] * inv, oacc[rb][i][1] * inv);
      w.y = pack2<DT>(oacc[rb][i][2] * inv, oacc[rb][i][3] * inv);
      *reinterpret_cast<u32x2*>(op + 16 * i + 4 * g) = w;
    }
    if (a.lse != nullptr && g == 0)
      a.lse[(int64_t)head * a.total_q + tok] = live ? (m[rb] - kShift) * kLn2 + __logf(l_tot) : -INFINITY;
  }
}

template <int NOPE, int ROPE, int DV>
static int launch_varlen(int dtype, const VarlenArgs& a, dim3 grid, hipStream_t s) {
  if (dtype == KVQ_F16)
    hipLaunchKernelGGL((varlen_attn_kernel<KVQ_F16, NOPE, ROPE, DV>), grid, dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL((varlen_attn_kernel<KVQ_BF16, NOPE, ROPE, DV>), grid, dim3(256), 0, s, a);
  return check_hip(hipGetLastError(), "mla_prefill_attn launch");
}

}  // namespace kvq

extern "C" int kvq_mla_prefill_attn(const void* q, int dtype, int64_t q_stride_tok, int64_t q_stride_head,
                                    const void* k_nope, int64_t kn_stride_tok, int64_t kn_stride_head,
                                    const void* k_pe, int64_t kpe_stride_tok, const void* v, int64_t v_stride_tok,
                                    int64_t v_stride_head, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                    int num_seqs, int max_seqlen_q, int64_t total_q, int num_heads, int nope_dim,
                                    int rope_dim, int v_dim, float scale, int causal, void* out,
                                    int64_t out_stride_tok, int64_t out_stride_head, float* lse,
                                    kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "mla_prefill_attn";
  KVQ_REQUIRE(num_seqs >= 0 && max_seqlen_q >= 0 && total_q >= 0 && num_heads > 0, "%s: bad sizes", op);
  if (num_seqs == 0 || max_seqlen_q == 0 || total_q == 0) return KVQ_OK;
  KVQ_REQUIRE(dtype == KVQ_BF16 || dtype == KVQ_F16, "%s: q, k and v must be bf16 or fp16 (dtype %d)", op, dtype);
  KVQ_REQUIRE(scale > 0.f && scale < INFINITY, "%s: scale must be positive and finite", op);   // the kernel takes row maxima before scaling
  KVQ_REQUIRE(q && k_nope && v && out && cu_seqlens_q && cu_seqlens_k, "%s: NULL pointer", op);
  KVQ_REQUIRE(rope_dim == 0 || k_pe != nullptr, "%s: k_pe is NULL with rope_dim %d", op, rope_dim);
  KVQ_REQUIRE(num_heads <= 65535 && num_seqs <= 65535, "%s: more than 65535 heads or sequences", op);
  const int64_t strides[] = {q_stride_tok, q_stride_head, kn_stride_tok, kn_stride_head, kpe_stride_tok,
                             v_stride_tok, v_stride_head, out_stride_tok, out_stride_head};
  for (int64_t st : strides) KVQ_REQUIRE(st >= 0 && st % 8 == 0, "%s: strides must be multiples of 8 elements (got %lld)", op, (long long)st);
  // a tile's 32 rows are addressed with 32-bit offsets from its first key
  KVQ_REQUIRE(kn_stride_tok < (1 << 24) && kpe_stride_tok < (1 << 24) && v_stride_tok < (1 << 24),
              "%s: token strides must be below 2^24 elements", op);
  KVQ_REQUIRE(((uintptr_t)q | (uintptr_t)k_nope | (uintptr_t)k_pe | (uintptr_t)v | (uintptr_t)out) % 16 == 0,
              "%s: tensors must be 16-byte aligned", op);
  VarlenArgs a{};
  a.q = q; a.k_nope = k_nope; a.k_pe = rope_dim ? k_pe : k_nope; a.v = v; a.out = out; a.lse = lse;
  a.cu_q = cu_seqlens_q; a.cu_k = cu_seqlens_k;
  a.q_st = q_stride_tok; a.q_sh = q_stride_head; a.kn_st = kn_stride_tok; a.kn_sh = kn_stride_head;
  a.kpe_st = kpe_stride_tok; a.v_st = v_stride_tok; a.v_sh = v_stride_head;
  a.out_st = out_stride_tok; a.out_sh = out_stride_head; a.total_q = total_q;
  a.causal = causal != 0;
  a.scale_log2 = scale * kLog2e;
  const dim3 grid((unsigned)((max_seqlen_q + 127) / 128), (unsigned)num_heads, (unsigned)num_seqs);
  hipStream_t s = as_stream(stream);
  if (nope_dim == 128 && rope_dim == 64 && v_dim == 128) return launch_varlen<128, 64, 128>(dtype, a, grid, s);
  if (nope_dim == 64 && rope_dim == 32 && v_dim == 64) return launch_varlen<64, 32, 64>(dtype, a, grid, s);
  if (nope_dim == 128 && rope_dim == 0 && v_dim == 128) return launch_varlen<128, 0, 128>(dtype, a, grid, s);
  return fail(KVQ_EINVAL, "%s: head dims (nope %d, rope %d, v %d) are not built; built: (128, 64, 128), (64, 32, 64), (128, 0, 128)",
              op, nope_dim, rope_dim, v_dim);
}
