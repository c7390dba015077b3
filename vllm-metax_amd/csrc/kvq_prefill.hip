// Chunked-prefill tile over the int8 paged cache (gfx950, wave64, MFMA f16): query runs longer
// than one token, causal, reading context and the run's own tokens from the cache.
//
// The MFMA N dimension carries (query token, q head of the group) pairs -- the BLOCK_M =
// BLOCK_Q x queries-per-kv folding of the reference's unified kernel
// (vllm_metax/v1/attention/ops/triton_unified_attention.py:56-246) -- so one pass over a kv head's
// records serves 16 * NT columns: the records are read from HBM, dropped into the wave's LDS
// window and turned into fp16 operands once per tile, and each operand feeds NT MFMAs.
// One wavefront = one (sequence, query block, kv head); it streams tiles 0 .. last visible tile
// with the decode tile's load / stage machinery and applies the causal limit per column.
#include "kvq_attn_core.cuh"

namespace kvq {

struct PrefillArgs {
  AttnIO io;
  const int32_t* seq_lens;
  const int32_t* cu_seqlens_q;
  int num_seqs;
  int causal;
  int q_tokens;  // query tokens per block: (16 * NT) / group
};

template <int D, int QDT, int ODT, int NT>
struct PrefillTile {
  using DTile = DecodeTile<D, QDT, ODT>;
  static constexpr int KSTEPS = DTile::KSTEPS;
  static constexpr int DT = DTile::DT;
  static constexpr int VB = DTile::VB;
  static constexpr int PITCH = DTile::PITCH;
  static constexpr int LDS_TILE = DTile::LDS_TILE;

  struct State {
    floatx4 o[NT][DT];
    floatx4 psum[NT];
    float m[NT], l[NT];
  };

  // S^T = K . Q^T for NT column tiles, online softmax with a per-column visible-token limit.
  template <bool MASK>
  __device__ static void qk_softmax(const LaneOffsets& lo, const half8_t (&qb)[NT][KSTEPS], const float (&s_init)[NT],
                                    const int (&limit)[NT], int t, int lane, const uint8_t* lds, State& st,
                                    half8_t (&p_op)[NT]) {
    const int g = lane >> 4;
    const float* sc_lds = reinterpret_cast<const float*>(lds + LDS_TILE);
    floatx4 s[NT][2];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      s[nt][0] = (floatx4){s_init[nt], s_init[nt], s_init[nt], s_init[nt]};
      s[nt][1] = s[nt][0];
    }
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int i = 0; i < KSTEPS / 2; ++i) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(lds + lo.l_k + mt * 16 * PITCH + i * 64);
        const half8_t a0 = dequant8(w.x, w.y), a1 = dequant8(w.z, w.w);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          s[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, qb[nt][2 * i], s[nt][mt], 0, 0, 0);
          s[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, qb[nt][2 * i + 1], s[nt][mt], 0, 0, 0);
        }
      }
    }
    const floatx4 ks0 = *reinterpret_cast<const floatx4*>(sc_lds + 4 * g);
    const floatx4 ks1 = *reinterpret_cast<const floatx4*>(sc_lds + 16 + 4 * g);
    const floatx4 vs0 = *reinterpret_cast<const floatx4*>(sc_lds + 32 + 4 * g);
    const floatx4 vs1 = *reinterpret_cast<const floatx4*>(sc_lds + 48 + 4 * g);
    const int tok_base = t * kTile + 4 * g;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      float logit[8];
      float mloc = -INFINITY;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float x = s[nt][mt][i] * (mt ? ks1 : ks0)[i];
          if constexpr (MASK) x = ((tok_base + mt * 16 + i) < limit[nt]) ? x : -INFINITY;
          logit[mt * 4 + i] = x;
          mloc = fmaxf(mloc, x);
        }
      }
      mloc = fmaxf(mloc, __shfl_xor(mloc, 16, kWave));
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
      const float m_new = fmaxf(st.m[nt], mloc);
      // a column that has seen no visible token yet keeps m = -inf; exponents are then taken
      // against 0 so that they come out as exp2(-inf) = 0 and never as (-inf) - (-inf)
      const float m_ref = m_new == -INFINITY ? 0.f : m_new;
      if (__builtin_amdgcn_ballot_w64(m_new > st.m[nt]) != 0) {
        const float alpha = __builtin_amdgcn_exp2f(st.m[nt] - m_ref);
        st.l[nt] *= alpha;
        st.psum[nt] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) st.o[nt][dt] *= alpha;
      }
      st.m[nt] = m_new;
      float pt[8];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = mt * 4 + i;
          const float p = __builtin_amdgcn_exp2f(logit[j] - m_ref);
          st.l[nt] += p;
          float x = p * (mt ? vs1 : vs0)[i];
          if constexpr (MASK) x = ((tok_base + mt * 16 + i) < limit[nt]) ? x : 0.f;
          pt[j] = x;
        }
      }
      u32x4 pb;
      pb.x = pack_half2(pt[0], pt[1]);
      pb.y = pack_half2(pt[2], pt[3]);
      pb.z = pack_half2(pt[4], pt[5]);
      pb.w = pack_half2(pt[6], pt[7]);
      p_op[nt] = __builtin_bit_cast(half8_t, pb);
    }
  }

  // O^T += (V + 1152)^T . P~^T: every converted V operand feeds the NT column tiles.
  __device__ static void pv(const LaneOffsets& lo, const half8_t (&p_op)[NT], const uint8_t* lds, State& st) {
    {
      const half_t one = (half_t)1.0f;
      const half8_t ones = {one, one, one, one, one, one, one, one};
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        st.psum[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, p_op[nt], st.psum[nt], 0, 0, 0);
    }
#pragma unroll
    for (int w = 0; w < VB / 4; ++w) {
      uint32_t x0[4], x1[4];
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int ja = 2 * a, jb = 2 * a + 1;
        const uint32_t ta = *reinterpret_cast<const uint32_t*>(lds + lo.l_v + ((ja & 3) + (ja >> 2) * 16) * PITCH + 4 * w) ^ 0x80808080u;
        const uint32_t tb = *reinterpret_cast<const uint32_t*>(lds + lo.l_v + ((jb & 3) + (jb >> 2) * 16) * PITCH + 4 * w) ^ 0x80808080u;
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
        const half8_t a_op = __builtin_bit_cast(half8_t, av);
        const int dt = 4 * w + b;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          st.o[nt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_op, p_op[nt], st.o[nt][dt], 0, 0, 0);
      }
    }
  }

  // Normalise column tile `nt` and write the lane's quarter of its output row.
  __device__ static void emit(const AttnIO& io, int nt, int64_t row, int head, bool valid, int lane, const State& st) {
    float l = st.l[nt];
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (!valid) return;
    const int g = lane >> 4;
    const float mul = l > 0.f ? 1.0f / (l * kPScale) : 0.f;   // no visible key: zeros
    const float corr = kCodeBias * st.psum[nt][0];
    float v[D / 4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) v[i * VB + dt] = (st.o[nt][dt][i] - corr) * mul;
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
      io.lse[row * io.num_q_heads + head] = l > 0.f ? (st.m[nt] + __builtin_amdgcn_logf(l)) * kLn2 : -INFINITY;
  }
};

// grid (query blocks of the longest run, sequences, ceil(Hkv / WPW)); wave w of a workgroup owns
// kv head blockIdx.z * WPW + w.  Sequences with a one-token run belong to the decode kernel.
template <int D, int QDT, int ODT, int NT, int WPW>
__global__ __launch_bounds__(WPW * 64) void paged_prefill_kernel(PrefillArgs a) {
  using PT = PrefillTile<D, QDT, ODT, NT>;
  using DTile = typename PT::DTile;
  __shared__ __align__(16) uint8_t lds_all[WPW][DTile::LDS_WAVE];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int seq = blockIdx.y;
  const int hkv = blockIdx.z * WPW + wave;
  const AttnIO& io = a.io;
  if (hkv >= io.g.num_kv_heads) return;
  const int q_begin = a.cu_seqlens_q[seq];
  const int q_len = a.cu_seqlens_q[seq + 1] - q_begin;
  const int len = a.seq_lens[seq];
  const int q0 = blockIdx.x * a.q_tokens;           // first query token of this block within the run
  if (q_len <= 1 || q0 >= q_len || len <= 0) return;
  uint8_t* lds = lds_all[wave];

  // ---- columns: n = nt * 16 + c  ->  (query token q0 + n / group, head n % group)
  const int c = lane & 15;
  const int ctx = len - q_len;                      // tokens before the run
  int limit[NT];                                    // visible tokens of the lane's column
  int64_t row[NT];
  int head[NT];
  bool valid[NT];
  int max_limit = 0, min_limit = 0x7fffffff;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = nt * 16 + c;
    const int qt = n / io.group;
    const int qi = q0 + qt;
    valid[nt] = qt < a.q_tokens && qi < q_len;
    head[nt] = hkv * io.group + (n - qt * io.group);
    row[nt] = q_begin + (valid[nt] ? qi : q0);
    int lim = a.causal ? ctx + qi + 1 : len;
    lim = lim < 0 ? 0 : (lim > len ? len : lim);
    limit[nt] = valid[nt] ? lim : 0;
    max_limit = max(max_limit, limit[nt]);
    min_limit = min(min_limit, valid[nt] ? lim : 0x7fffffff);
  }
  max_limit = wave_max_i32(max_limit);
  min_limit = -wave_max_i32(-min_limit);
  const int t_end = (max_limit + kTile - 1) / kTile;  // wave-uniform
  if (t_end == 0) {  // nothing visible for any column (run longer than the sequence): defined zeros
    typename PT::State z;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int dt = 0; dt < PT::DT; ++dt) z.o[nt][dt] = (floatx4){0.f, 0.f, 0.f, 0.f};
      z.psum[nt] = (floatx4){0.f, 0.f, 0.f, 0.f};
      z.m[nt] = -INFINITY;
      z.l[nt] = 0.f;
      PT::emit(io, nt, row[nt], head[nt], valid[nt], lane, z);
    }
    return;
  }

  const LaneOffsets lo = DTile::lane_offsets(io.g, lane);
  const int32_t* bt_row = io.block_table + (int64_t)seq * io.bt_stride;
  typename DTile::Tile kv;
  int t = 0;
  TileBlocks nb = DTile::fetch_blocks(io, bt_row, len, t);
  DTile::load_tile(io, DTile::window(io, nb, t, hkv), lo, kv);
  DTile::phase_fence();
  nb = DTile::fetch_blocks(io, bt_row, len, t + 1);

  half8_t qb[NT][PT::KSTEPS];
  float s_init[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    s_init[nt] = DTile::load_q_row(io, row[nt] * io.q_stride_t + (int64_t)(valid[nt] ? head[nt] : hkv * io.group) * io.q_stride_h,
                                   valid[nt], lane, qb[nt]);
  const float sc_mul = lane < 32 ? io.scale_log2 : kPScale;
  typename PT::State st;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
    for (int dt = 0; dt < PT::DT; ++dt) st.o[nt][dt] = (floatx4){0.f, 0.f, 0.f, 0.f};
    st.psum[nt] = (floatx4){0.f, 0.f, 0.f, 0.f};
    st.m[nt] = -INFINITY;
    st.l[nt] = 0.f;
  }
  half8_t p_op[NT];
  while (t + 1 < t_end) {
    const typename DTile::Window w = DTile::window(io, nb, t + 1, hkv);
    DTile::stage(kv, lo, sc_mul, lane, lds);
    DTile::phase_fence();
    DTile::load_tile(io, w, lo, kv);
    DTile::phase_fence();
    nb = DTile::fetch_blocks(io, bt_row, len, t + 2);
    if ((t + 1) * kTile <= min_limit) PT::template qk_softmax<false>(lo, qb, s_init, limit, t, lane, lds, st, p_op);
    else PT::template qk_softmax<true>(lo, qb, s_init, limit, t, lane, lds, st, p_op);
    PT::pv(lo, p_op, lds, st);
    DTile::phase_fence();
    ++t;
  }
  DTile::stage(kv, lo, sc_mul, lane, lds);
  PT::template qk_softmax<true>(lo, qb, s_init, limit, t, lane, lds, st, p_op);
  PT::pv(lo, p_op, lds, st);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) PT::emit(io, nt, row[nt], head[nt], valid[nt], lane, st);
}

template <int D, int QDT, int ODT, int NT, int WPW>
static int launch_prefill_cfg(const PrefillArgs& a, int max_query_len, hipStream_t s) {
  const int blocks = (max_query_len + a.q_tokens - 1) / a.q_tokens;
  if (blocks > 0x7fffffff / 2 || a.num_seqs > 65535) return fail(KVQ_EINVAL, "paged_attn_int8: prefill grid out of range");
  dim3 grid(blocks, a.num_seqs, (a.io.g.num_kv_heads + WPW - 1) / WPW);
  hipLaunchKernelGGL((paged_prefill_kernel<D, QDT, ODT, NT, WPW>), grid, dim3(WPW * 64), 0, s, a);
  return check_hip(hipGetLastError(), "paged_prefill launch");
}

template <int D, int QDT, int ODT>
static int launch_prefill_nt(PrefillArgs& a, int max_query_len, hipStream_t s) {
  constexpr int WPW = 4;
  // two column tiles per wave where the accumulators fit the register file next to a tile in flight
  if (D <= 128 && a.io.group * 2 <= 32 && max_query_len * a.io.group > 16) {
    a.q_tokens = 32 / a.io.group;
    return launch_prefill_cfg<D, QDT, ODT, (D <= 128 ? 2 : 1), WPW>(a, max_query_len, s);
  }
  a.q_tokens = 16 / a.io.group;
  return launch_prefill_cfg<D, QDT, ODT, 1, WPW>(a, max_query_len, s);
}

template <int D, int QDT>
static int launch_prefill_o(PrefillArgs& a, int max_query_len, int out_dtype, hipStream_t s) {
  switch (out_dtype) {
    case KVQ_F32: return launch_prefill_nt<D, QDT, KVQ_F32>(a, max_query_len, s);
    case KVQ_BF16: return launch_prefill_nt<D, QDT, KVQ_BF16>(a, max_query_len, s);
    case KVQ_F16: return launch_prefill_nt<D, QDT, KVQ_F16>(a, max_query_len, s);
    default: return fail(KVQ_EINVAL, "paged_attn_int8: unknown out_dtype %d", out_dtype);
  }
}

template <int D>
static int launch_prefill_q(PrefillArgs& a, int max_query_len, int q_dtype, int out_dtype, hipStream_t s) {
  switch (q_dtype) {
    case KVQ_F32: return launch_prefill_o<D, KVQ_F32>(a, max_query_len, out_dtype, s);
    case KVQ_BF16: return launch_prefill_o<D, KVQ_BF16>(a, max_query_len, out_dtype, s);
    case KVQ_F16: return launch_prefill_o<D, KVQ_F16>(a, max_query_len, out_dtype, s);
    default: return fail(KVQ_EINVAL, "paged_attn_int8: unknown q_dtype %d", q_dtype);
  }
}

int launch_prefill(const AttnIO& io, const int32_t* seq_lens, const int32_t* cu_seqlens_q, int num_seqs,
                   int max_query_len, int causal, int q_dtype, int out_dtype, hipStream_t s) {
  PrefillArgs a{};
  a.io = io;
  a.seq_lens = seq_lens;
  a.cu_seqlens_q = cu_seqlens_q;
  a.num_seqs = num_seqs;
  a.causal = causal;
  switch (io.g.head_size) {
    case 64: return launch_prefill_q<64>(a, max_query_len, q_dtype, out_dtype, s);
    case 128: return launch_prefill_q<128>(a, max_query_len, q_dtype, out_dtype, s);
    default: return launch_prefill_q<256>(a, max_query_len, q_dtype, out_dtype, s);
  }
}

}  // namespace kvq
