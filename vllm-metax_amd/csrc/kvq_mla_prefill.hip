// Varlen attention with LSE output for the MLA prefill (gfx950): the step between the latent cache's
// gather + dequantise and the LSE merge of the chunked-context loop, and the causal pass over the new
// tokens.  K arrives as the two pieces the layer already has -- k_nope [S, H, NOPE] out of kv_b_proj and
// the rope part k_pe [S, ROPE] shared by all heads -- so the concatenated [S, H, NOPE + ROPE] tensor is
// never built.
//
// One wave owns 16 query rows of one (sequence, head) and walks the keys 32 at a time; nothing goes
// through LDS.  Both products are computed transposed so that every per-row quantity is lane-local:
//   S^T = K Q^T   A = K rows (lane = key, 8 consecutive d), B = Q (lane = query row): 16x16x32 MFMA of the
//                 input type; a lane ends up with 8 keys of ITS query row, so the row maximum is a
//                 reduction over the four quarter-waves and alpha / l stay in the lane.
//   O^T = V^T P^T B = P~ straight from the S^T registers (k slot j of quarter g is key 16 (j / 4) + 4 g +
//                 j % 4; any order works as long as V uses the same one).  A = V^T needs 8 keys of one
//                 dim per lane while memory holds 8 dims of one key: each lane loads the slice
//                 [its 8 keys] x [DV / 16 consecutive dims] and transposes it in registers with one
//                 v_perm_b32 per output dword.  Output block i then holds dims (DV/16) * lane + i, which
//                 leaves every lane with 4 runs of DV/16 consecutive dims of its own query row: 16-byte
//                 stores.
// Masked keys (beyond the sequence, or above the causal diagonal, which is aligned to the END of the
// keys as flash-attention does) get weight 0; their loads are clamped to the last valid key.
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

template <int NDW>
struct Words {
  uint32_t w[NDW];
};
template <int NDW>
__device__ __forceinline__ Words<NDW> load_words(const uint16_t* p) {
  Words<NDW> r;
  if constexpr (NDW == 2) {
    const u32x2 v = *reinterpret_cast<const u32x2*>(p);
    r.w[0] = v.x;
    r.w[1] = v.y;
  } else {
#pragma unroll
    for (int i = 0; i < NDW / 4; ++i) {
      const u32x4 v = reinterpret_cast<const u32x4*>(p)[i];
      r.w[4 * i] = v.x;
      r.w[4 * i + 1] = v.y;
      r.w[4 * i + 2] = v.z;
      r.w[4 * i + 3] = v.w;
    }
  }
  return r;
}

template <int DT, int NOPE, int ROPE, int DV>
__global__ __launch_bounds__(256) void varlen_attn_kernel(VarlenArgs a) {
  constexpr int KSN = NOPE / 32, KSR = ROPE / 32, KS = KSN + KSR;   // k-steps of the QK product
  constexpr int DPL = DV / 16;                                      // dims per lane and output block
  constexpr int VR = DPL / 2;                                       // dwords of one key's slice
  // fp16 weights are kept 2^8 larger so that small ones stay normal; l carries the same factor
  constexpr float kShift = DT == KVQ_F16 ? 8.f : 0.f;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seq = blockIdx.z, head = blockIdx.y;
  const int q_begin = a.cu_q[seq], q_len = a.cu_q[seq + 1] - q_begin;
  const int k_begin = a.cu_k[seq], k_len = a.cu_k[seq + 1] - k_begin;
  const int q0 = (blockIdx.x * 4 + wave) * 16;
  if (q0 >= q_len) return;
  const int c = lane & 15, g = lane >> 4;
  const int qrow = min(q0 + c, q_len - 1);   // rows past the end compute on a copy and are not stored

  u32x4 qop[KS];
  {
    const uint16_t* qp = static_cast<const uint16_t*>(a.q) + (int64_t)(q_begin + qrow) * a.q_st + (int64_t)head * a.q_sh + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) qop[s] = *reinterpret_cast<const u32x4*>(qp + 32 * s);
  }

  // key j is visible to query row i iff j <= i + (k_len - q_len)
  const int diag = k_len - q_len;
  const int my_limit = a.causal ? max(0, min(k_len, q0 + c + diag + 1)) : k_len;
  const int k_end = a.causal ? max(0, min(k_len, q0 + 15 + diag + 1)) : k_len;
  const int num_tiles = (k_end + 31) / 32;

  floatx4 oacc[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) oacc[i] = (floatx4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const uint16_t* kn_base = static_cast<const uint16_t*>(a.k_nope) + (int64_t)head * a.kn_sh + 8 * g;
  const uint16_t* kpe_base = static_cast<const uint16_t*>(a.k_pe) + 8 * g;
  const uint16_t* v_base = static_cast<const uint16_t*>(a.v) + (int64_t)head * a.v_sh + DPL * c;

  for (int t = 0; t < num_tiles; ++t) {
    // ---- S^T = K Q^T for the tile's two blocks of 16 keys
    floatx4 sacc[2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const int64_t krow = k_begin + min(t * 32 + 16 * blk + c, k_len - 1);
      const uint16_t* kn = kn_base + krow * a.kn_st;
      const uint16_t* kp = kpe_base + krow * a.kpe_st;
      floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KSN; ++s) acc = mfma16<DT>(*reinterpret_cast<const u32x4*>(kn + 32 * s), qop[s], acc);
#pragma unroll
      for (int s = 0; s < KSR; ++s) acc = mfma16<DT>(*reinterpret_cast<const u32x4*>(kp + 32 * s), qop[KSN + s], acc);
      sacc[blk] = acc;
    }
    // ---- the lane's 8 keys' slices of V (k slot j = 4 blk + r is key 16 blk + 4 g + r)
    Words<VR> vrow[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t vr = k_begin + min(t * 32 + 16 * (j >> 2) + 4 * g + (j & 3), k_len - 1);
      vrow[j] = load_words<VR>(v_base + vr * a.v_st);
    }
    // ---- online softmax in base 2
    float sc[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = t * 32 + 16 * (j >> 2) + 4 * g + (j & 3);
      const float sv = sacc[j >> 2][j & 3] * a.scale_log2;
      sc[j] = key < my_limit ? sv : -INFINITY;
      mx = fmaxf(mx, sc[j]);
    }
    mx = max_over_quarters(mx);
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    float p[8], psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p[j] = __builtin_amdgcn_exp2f(sc[j] - m_use + kShift);
      psum += p[j];
    }
    l = l * alpha + psum;
    m = m_new;
    u32x4 pk;
    pk.x = pack2<DT>(p[0], p[1]);
    pk.y = pack2<DT>(p[2], p[3]);
    pk.z = pack2<DT>(p[4], p[5]);
    pk.w = pack2<DT>(p[6], p[7]);
    // ---- O^T = alpha O^T + V^T P^T
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      u32x4 vt;
      const uint32_t sel = (i & 1) ? kPermHighHalves : kPermLowHalves;
      vt.x = perm(vrow[1].w[i >> 1], vrow[0].w[i >> 1], sel);
      vt.y = perm(vrow[3].w[i >> 1], vrow[2].w[i >> 1], sel);
      vt.z = perm(vrow[5].w[i >> 1], vrow[4].w[i >> 1], sel);
      vt.w = perm(vrow[7].w[i >> 1], vrow[6].w[i >> 1], sel);
      floatx4 o = oacc[i];
      o.x *= alpha;
      o.y *= alpha;
      o.z *= alpha;
      o.w *= alpha;
      oacc[i] = mfma16<DT>(vt, pk, o);
    }
  }

  const float l_tot = sum_over_quarters(l);
  const bool live = l_tot > 0.f;
  const float inv = live ? 1.f / l_tot : 0.f;
  if (q0 + c >= q_len) return;
  const int64_t tok = q_begin + q0 + c;
  uint16_t* op = static_cast<uint16_t*>(a.out) + tok * a.out_st + (int64_t)head * a.out_sh;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    uint32_t w[VR];
#pragma unroll
    for (int i = 0; i < VR; ++i) w[i] = pack2<DT>(oacc[2 * i][r] * inv, oacc[2 * i + 1][r] * inv);
    uint16_t* dst = op + DPL * (4 * g + r);
    if constexpr (VR == 2) {
      *reinterpret_cast<u32x2*>(dst) = (u32x2){w[0], w[1]};
    } else {
#pragma unroll
      for (int i = 0; i < VR / 4; ++i) reinterpret_cast<u32x4*>(dst)[i] = (u32x4){w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]};
    }
  }
  if (a.lse != nullptr && g == 0)
    a.lse[(int64_t)head * a.total_q + tok] = live ? (m - kShift) * kLn2 + __logf(l_tot) : -INFINITY;
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
  KVQ_REQUIRE(q && k_nope && v && out && cu_seqlens_q && cu_seqlens_k, "%s: NULL pointer", op);
  KVQ_REQUIRE(rope_dim == 0 || k_pe != nullptr, "%s: k_pe is NULL with rope_dim %d", op, rope_dim);
  KVQ_REQUIRE(num_heads <= 65535 && num_seqs <= 65535, "%s: more than 65535 heads or sequences", op);
  const int64_t strides[] = {q_stride_tok, q_stride_head, kn_stride_tok, kn_stride_head, kpe_stride_tok,
                             v_stride_tok, v_stride_head, out_stride_tok, out_stride_head};
  for (int64_t st : strides) KVQ_REQUIRE(st >= 0 && st % 8 == 0, "%s: strides must be multiples of 8 elements (got %lld)", op, (long long)st);
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
  const dim3 grid((unsigned)((max_seqlen_q + 63) / 64), (unsigned)num_heads, (unsigned)num_seqs);
  hipStream_t s = as_stream(stream);
  if (nope_dim == 128 && rope_dim == 64 && v_dim == 128) return launch_varlen<128, 64, 128>(dtype, a, grid, s);
  if (nope_dim == 64 && rope_dim == 32 && v_dim == 64) return launch_varlen<64, 32, 64>(dtype, a, grid, s);
  if (nope_dim == 128 && rope_dim == 0 && v_dim == 128) return launch_varlen<128, 0, 128>(dtype, a, grid, s);
  return fail(KVQ_EINVAL, "%s: head dims (nope %d, rope %d, v %d) are not built; built: (128, 64, 128), (64, 32, 64), (128, 0, 128)",
              op, nope_dim, rope_dim, v_dim);
}
