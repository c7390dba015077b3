// Chunked-prefill tile over the int8 paged cache (gfx950, wave64, MFMA f16): query runs longer
// than one token, causal, reading context and the run's own tokens from the cache.
//
// The MFMA N dimension carries (query token, q head of the group) pairs -- the
// folding of query tokens and the q heads of a kv group that the unified attention op the reference
// calls does (vllm_metax/v1/attention/backends/triton_attn.py:43, 688-725) -- so one pass over a kv head's
// records serves 16 * NT columns: the records are read from HBM, dropped into the wave's LDS
// window and turned into fp16 operands once per tile, and each operand feeds NT MFMAs.
// One wavefront = one (sequence, query block, kv head); it streams tiles 0 .. last visible tile
// with the decode tile's load / stage machinery and applies the causal limit per column.
#include <type_traits>

#include "kvq_attn_core.cuh"

namespace kvq {

struct PrefillArgs {
  AttnIO io;
  const int32_t* seq_lens;
  const int32_t* cu_seqlens_q;
  int num_seqs;
  int causal;
  int q_tokens;  // query tokens per block: (16 * NT) / group
  // [1 + B]: how many sequences of the batch have a query run (q_len > 1, len > 0), then their numbers in batch
  // order; written by prefill_plan_kernel ahead of the attention kernel of the same call.
  const int32_t* plan;
  // Context splits of the workgroup-shared tile (1 = none).  With S > 1 an item's tiles are cut into S ranges, each
  // range is a workgroup of its own that leaves a partial state per (query row, q head) in `part`
  // ([row][q head][split][D + 2] fp32: the accumulated row, the reference maximum, the sum), and a merge kernel
  // combines them: a launch with few items on a long context (a small prefill chunk of one long request) would
  // otherwise walk the whole context in a handful of workgroups, one tile after the other.
  int ksplit;
  float* part;
  // Batch-invariant mode: which runs a kernel of this launch takes -- 0 all, 1 only those that fill the
  // workgroup-shared tile by themselves (q_len x group >= 64), 2 only the others.  Without the mode the batch's
  // longest run chooses ONE kernel for every run of the launch, so a short run's bits would depend on its company.
  int route;
};

// One workgroup lists the sequences that have work for the prefill kernels.  A mixed batch is mostly decode rows;
// a grid over all sequences would spend most of its workgroups finding that out one by one, in between the ones
// that have work.
__global__ __launch_bounds__(64) void prefill_plan_kernel(const int32_t* seq_lens, const int32_t* cu_seqlens_q,
                                                          int num_seqs, int32_t* plan) {
  const int lane = threadIdx.x;
  int count = 0;
  for (int base = 0; base < num_seqs; base += kWave) {
    const int s = base + lane;
    const int sc = s < num_seqs ? s : num_seqs - 1;
    const bool has = s < num_seqs && cu_seqlens_q[sc + 1] - cu_seqlens_q[sc] > 1 && seq_lens[sc] > 0;
    const uint64_t mask = __builtin_amdgcn_ballot_w64(has);
    if (has) plan[1 + count + __builtin_popcountll(mask & ((1ull << lane) - 1))] = s;
    count += __builtin_popcountll(mask);
  }
  if (lane == 0) plan[0] = count;
  // Up to 64 of them are put longest sequence first: their workgroups start in the plan's order, and the
  // longest sequence's are the ones that should not start last.
  if (count > 1 && count <= kWave) {
    __threadfence_block();
    const int id = plan[1 + (lane < count ? lane : 0)];
    const int key = lane < count ? seq_lens[id] : -1;
    int rank = 0;
    for (int j = 0; j < count; ++j) {
      const int kj = __shfl(key, j, kWave);
      rank += (kj > key || (kj == key && j < lane)) ? 1 : 0;
    }
    if (lane < count) plan[1 + rank] = id;
  }
}

template <int D, int QDT, int ODT, int NT, int CODE = KVQ_CODE_INT8>
struct PrefillTile {
  using DTile = DecodeTile<D, QDT, ODT, CODE>;
  static constexpr bool FP8 = DTile::FP8;
  static constexpr bool INT4 = DTile::INT4;
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
  // A column sees tokens [limit - wspan, limit): wspan is the sliding window, or 2^31 - 1 without one.
  template <bool MASK>
  __device__ static void qk_softmax(const AttnIO& io, const LaneOffsets& lo, const half8_t (&qb)[NT][KSTEPS],
                                    const float (&s_init)[NT], const int (&limit)[NT], uint32_t wspan, int t, int lane,
                                    const uint8_t* lds, State& st, half8_t (&p_op)[NT], const float (&ali)[NT]) {
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
      if constexpr (INT4) {
        half8_t ka[KSTEPS];
        DTile::k_operands_int4(lo, mt, lds, ka);
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            s[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[kk], qb[nt][kk], s[nt][mt], 0, 0, 0);
      } else {
#pragma unroll
      for (int i = 0; i < KSTEPS / 2; ++i) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(lds + lo.l_k + mt * 16 * PITCH + i * 64);
        const half8_t a0 = dequant8<FP8>(w.x, w.y), a1 = dequant8<FP8>(w.z, w.w);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          s[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, qb[nt][2 * i], s[nt][mt], 0, 0, 0);
          s[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, qb[nt][2 * i + 1], s[nt][mt], 0, 0, 0);
        }
      }
      }
    }
    const floatx4 ks0 = *reinterpret_cast<const floatx4*>(sc_lds + 4 * g);
    const floatx4 ks1 = *reinterpret_cast<const floatx4*>(sc_lds + 16 + 4 * g);
    const floatx4 vs0 = *reinterpret_cast<const floatx4*>(sc_lds + 32 + 4 * g);
    const floatx4 vs1 = *reinterpret_cast<const floatx4*>(sc_lds + 48 + 4 * g);
    const int tok_base = t * kTile + 4 * g;
    const bool capped = io.cap_c != 0.f;  // uniform
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      float logit[8];
      float mloc = -INFINITY;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) logit[mt * 4 + i] = s[nt][mt][i] * (mt ? ks1 : ks0)[i];
      }
      if (capped) {
#pragma unroll
        for (int j = 0; j < 8; ++j) logit[j] = soft_cap(logit[j], io.cap_c, io.cap_k);
      }
      if (io.alibi != nullptr) {   // uniform; the column's query stands at limit - 1
        const float rel0 = (float)(tok_base - (limit[nt] - 1));
#pragma unroll
        for (int j = 0; j < 8; ++j) logit[j] = __builtin_fmaf(ali[nt], rel0 + (float)((j >> 2) * 16 + (j & 3)), logit[j]);
      }
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float x = logit[mt * 4 + i];
          if constexpr (MASK) x = ((uint32_t)(limit[nt] - 1 - (tok_base + mt * 16 + i)) < wspan) ? x : -INFINITY;
          logit[mt * 4 + i] = x;
          mloc = fmaxf(mloc, x);
        }
      }
      mloc = max_over_quarters(mloc);
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
          if constexpr (MASK) x = ((uint32_t)(limit[nt] - 1 - (tok_base + mt * 16 + i)) < wspan) ? x : 0.f;
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
    if constexpr (!FP8) {
      const half_t one = (half_t)1.0f;
      const half8_t ones = {one, one, one, one, one, one, one, one};
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        st.psum[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, p_op[nt], st.psum[nt], 0, 0, 0);
    }
    if constexpr (INT4) {
#pragma unroll
      for (int u = 0; u < VB / 2; ++u) {
        half8_t va[4];
        DTile::v_operands_int4(lo, u, lds, va);
#pragma unroll
        for (int n = 0; n < 4; ++n)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            st.o[nt][4 * u + n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[n], p_op[nt], st.o[nt][4 * u + n], 0, 0, 0);
      }
      return;
    }
#pragma unroll
    for (int w = 0; w < VB / 4; ++w) {
      uint32_t x0[4], x1[4];
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
        const half8_t a_op = __builtin_bit_cast(half8_t, av);
        const int dt = 4 * w + b;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          st.o[nt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_op, p_op[nt], st.o[nt][dt], 0, 0, 0);
      }
    }
  }

  // ---- several waves on one item: their states meet in LDS, one column tile at a time.  A wave drops the tile's
  //      state into its own window (free once its tiles are done); the item's first wave folds them into its own.
  //      A column may have seen nothing in a wave's tiles (m = -inf): its weight is then 0, never 2^(-inf + inf).
  __device__ static void dump_state(const State& st, int nt, int lane, uint8_t* lds) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<floatx4*>(lds + (dt * 64 + lane) * 16) = st.o[nt][dt];
    *reinterpret_cast<floatx4*>(lds + (DT * 64 + lane) * 16) = (floatx4){st.psum[nt][0], st.m[nt], st.l[nt], 0.f};
  }
  __device__ static void fold_state(State& st, int nt, int lane, const uint8_t* lds) {
    const floatx4 x = *reinterpret_cast<const floatx4*>(lds + (DT * 64 + lane) * 16);
    const float mj = x.y;
    const float m_new = fmaxf(st.m[nt], mj);
    const float m_ref = m_new == -INFINITY ? 0.f : m_new;
    const float a = __builtin_amdgcn_exp2f(st.m[nt] - m_ref);
    const float b = __builtin_amdgcn_exp2f(mj - m_ref);
    st.m[nt] = m_new;
    st.l[nt] = st.l[nt] * a + x.z * b;
    st.psum[nt] = st.psum[nt] * a + x.x * b;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      st.o[nt][dt] = st.o[nt][dt] * a + *reinterpret_cast<const floatx4*>(lds + (dt * 64 + lane) * 16) * b;
  }

  // Normalise column tile `nt` and write the lane's quarter of its output row.
  __device__ static void emit(const AttnIO& io, int nt, int64_t row, int head, bool valid, int lane, const State& st) {
    float l = st.l[nt];
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (!valid) return;
    if (l > 0.f) l += sink_term(io.sinks, head, st.m[nt]);   // a row without a visible key keeps its zeros
    const int g = lane >> 4;
    const float mul = l > 0.f ? 1.0f / (l * DTile::kOutDiv) : 0.f;   // no visible key: zeros
    const float corr = FP8 ? 0.f : DTile::kBias * st.psum[nt][0];
    float v[D / 4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) v[i * DT + dt] = (st.o[nt][dt][i] - corr) * mul;
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
// kv head (head group) * WPW + w.  Sequences with a one-token run belong to the decode kernel.
// SPLIT: grid z = Hkv and ALL waves of the workgroup serve one kv head, taking the
// item's tiles in turn (wave w: tiles t_start + w, + WPW, ...); their states are folded in LDS at the end.  For
// launches with few items and long contexts -- a handful of query tokens per sequence, as a speculative-decoding
// step has them: one wave per item leaves most of the chip's waves idle (measured on MI355X, 64 sequences of
// 1k-8k tokens with 2 or 4 query tokens each: 280 us per call that way against 118 us for one query token).
template <int D, int QDT, int ODT, int NT, int WPW, int CODE = KVQ_CODE_INT8, bool SPLIT = false>
__global__ __launch_bounds__(WPW * 64) void paged_prefill_kernel(PrefillArgs a) {
  using PT = PrefillTile<D, QDT, ODT, NT, CODE>;
  using DTile = typename PT::DTile;
  __shared__ __align__(16) uint8_t lds_all[WPW][DTile::LDS_WAVE];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // which sequence, head group and query block: the linear workgroup number read over the plan's sequences,
  // sequence by sequence (longest first), inside a sequence query-block-major over the head groups, longest
  // block first, the head group shifted by the block number (see paged_prefill_flash32_kernel)
  const unsigned nqb = gridDim.x, hz = gridDim.z, per_seq = nqb * hz;
  const unsigned lin = blockIdx.x + nqb * (blockIdx.y + gridDim.y * blockIdx.z);
  if (lin >= per_seq * (unsigned)a.plan[0]) return;   // uniform over the workgroup
  const unsigned rem = lin % per_seq, qbi = rem / hz;
  const int seq = a.plan[1 + lin / per_seq];
  const int hkv = SPLIT ? (int)((rem % hz + qbi) % hz) : (int)((rem % hz + qbi) % hz) * WPW + wave;
  constexpr int STEP = SPLIT ? WPW : 1;          // tiles between two of this wave's
  const AttnIO& io = a.io;
  if (hkv >= io.g.num_kv_heads) return;
  const int q_begin = a.cu_seqlens_q[seq];
  const int q_len = a.cu_seqlens_q[seq + 1] - q_begin;
  const int len = a.seq_lens[seq];
  const int q0 = (int)(nqb - 1 - qbi) * a.q_tokens;   // first query token of this block within the run
  if (q_len <= 1 || q0 >= q_len || len <= 0) return;
  if (a.route == 2 && q_len * io.group >= 64) return;   // the workgroup-shared tile's (uniform over the workgroup)
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
  // sliding window: a column sees [limit - window, limit); the wave starts at the tile that holds
  // the earliest of these lower edges and masks tiles below the latest one
  const uint32_t wspan = io.window > 0 ? (uint32_t)io.window : 0x7fffffffu;
  const int min_first = io.window > 0 ? max(0, min(min_limit, max_limit) - io.window) : 0;
  const int max_first = io.window > 0 ? max(0, max_limit - io.window) : 0;
  const int t_start = min_first / kTile;
  if (t_end == 0) {  // nothing visible for any column (run longer than the sequence): defined zeros
    typename PT::State z;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int dt = 0; dt < PT::DT; ++dt) z.o[nt][dt] = (floatx4){0.f, 0.f, 0.f, 0.f};
      z.psum[nt] = (floatx4){0.f, 0.f, 0.f, 0.f};
      z.m[nt] = -INFINITY;
      z.l[nt] = 0.f;
      if (!SPLIT || wave == 0) PT::emit(io, nt, row[nt], head[nt], valid[nt], lane, z);
    }
    return;
  }

  const LaneOffsets lo = DTile::lane_offsets(io.g, lane);
  const int32_t* bt_row = io.block_table + (int64_t)seq * io.bt_stride;
  typename DTile::Tile kv;
  int t = t_start + (SPLIT ? wave : 0);
  const bool has_tiles = t < t_end;              // without the split: always
  // (a wave without a tile still loads one -- the block table is read clamped into the sequence -- and uses nothing)
  TileBlocks nb = DTile::fetch_blocks(io, bt_row, len, t);
  DTile::load_tile(io, DTile::window(io, nb, t, hkv), lo, kv);
  DTile::phase_fence();
  nb = DTile::fetch_blocks(io, bt_row, len, t + STEP);

  half8_t qb[NT][PT::KSTEPS];
  float s_init[NT], ali[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) ali[nt] = alibi_slope(io.alibi, valid[nt] ? head[nt] : hkv * io.group);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    s_init[nt] = DTile::load_q_row(io, row[nt] * io.q_stride_t + (int64_t)(valid[nt] ? head[nt] : hkv * io.group) * io.q_stride_h,
                                   valid[nt], lane, qb[nt]);
  const float sc_mul = lane < 32 ? io.scale_log2 * DTile::kKScaleMul : kPScale;
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
  if (has_tiles) {
    while (t + STEP < t_end) {
      const typename DTile::Window w = DTile::window(io, nb, t + STEP, hkv);
      DTile::stage(kv, lo, sc_mul, lane, lds);
      DTile::phase_fence();
      DTile::load_tile(io, w, lo, kv);
      DTile::phase_fence();
      nb = DTile::fetch_blocks(io, bt_row, len, t + 2 * STEP);
      if ((t + 1) * kTile <= min_limit && t * kTile >= max_first)
        PT::template qk_softmax<false>(io, lo, qb, s_init, limit, wspan, t, lane, lds, st, p_op, ali);
      else
        PT::template qk_softmax<true>(io, lo, qb, s_init, limit, wspan, t, lane, lds, st, p_op, ali);
      PT::pv(lo, p_op, lds, st);
      DTile::phase_fence();
      t += STEP;
    }
    DTile::stage(kv, lo, sc_mul, lane, lds);
    PT::template qk_softmax<true>(io, lo, qb, s_init, limit, wspan, t, lane, lds, st, p_op, ali);
    PT::pv(lo, p_op, lds, st);
  }
  if constexpr (SPLIT) {
    // every wave of the workgroup arrives here (the returns above are uniform over it)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (nt > 0) lds_barrier();   // the windows are read no more: they take the next column tile's states
      if (wave != 0 && has_tiles) PT::dump_state(st, nt, lane, lds);
      lds_barrier();
      if (wave == 0) {
#pragma unroll
        for (int j = 1; j < WPW; ++j)
          if (t_start + j < t_end) PT::fold_state(st, nt, lane, lds_all[j]);   // wave j owned a tile
      }
    }
    if (wave != 0) return;
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) PT::emit(io, nt, row[nt], head[nt], valid[nt], lane, st);
}

// ---------------------------------------------------------------------------------------------
// Workgroup-shared tile: the compute-bound shape (long query runs).
//
// Four waves share one kv head's 32-token tile.  The records are loaded cooperatively (16-byte
// chunks, every wave the same loads in the same order, two tiles ahead), dropped raw into LDS,
// expanded ONCE per workgroup to fp16 -- K as [token][dim], V transposed as [dim][token] in the
// token order the P~ operand has, the code bias 1152 taken out (exact in fp16) -- and every wave
// feeds its 32 columns straight from the fp16 tile with MFMA 32x32x16: a 16-byte LDS read per lane
// is the A operand of 32 Ki flop, and a lane holds 16 tokens of ONE column, so the column maximum
// needs one cross-lane step.  Raw and fp16 tiles are double-buffered, which leaves one barrier per
// tile.  Two workgroups fit a CU; they drift apart, so one workgroup's LDS-bound phase runs under
// the other's ALU- and MFMA-bound phases.
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int D, int QDT, int ODT, int CODE = KVQ_CODE_INT8>
struct Flash32 {
  using DTile = DecodeTile<D, QDT, ODT, CODE>;
  static constexpr bool FP8 = DTile::FP8;   // e4m3fn codes: they enter the MFMA as value / 2^8, without a bias
  static constexpr bool INT4 = DTile::INT4; // two codes per byte: only the expansion of the raw tile differs
  static constexpr int DB = DTile::DB;      // code bytes of a half record
  static constexpr int WAVES = 4;
  static constexpr int KS = D / 16;                      // k-steps of the QK product
  static constexpr int MT = D / 32;                      // 32-dim row tiles of O^T
  static constexpr int RAW_PITCH = DTile::PITCH;
  static constexpr int RAW_BYTES = kTile * RAW_PITCH;
  static constexpr int K_PITCH = 2 * D + 16;
  static constexpr int K_BYTES = kTile * K_PITCH;
  static constexpr int V_PITCH = 2 * kTile + 16;
  static constexpr int V_BYTES = D * V_PITCH;
  static constexpr int BUF_BYTES = K_BYTES + V_BYTES + 68 * 4;   // 32 K-side + 32 V-side scales + the tile's lazy-maximum allowance
  static constexpr int LDS_BYTES = 2 * RAW_BYTES + 2 * BUF_BYTES;
  static constexpr int COLS = 32 * WAVES;

  __device__ static __forceinline__ uint32_t to_half2(uint32_t x, bool upper) {
    if constexpr (FP8) return fp8_bytes_to_half2(x, upper);
    const half2_t bias = {(half_t)kCodeBias, (half_t)kCodeBias};
    const half2_t v = __builtin_bit_cast(half2_t, bytes_to_half2(x, upper)) - bias;
    return __builtin_bit_cast(uint32_t, v);
  }

  // Q of the lane's column as the B operand: lane (c = lane & 31, g = lane >> 5) holds, for k-step
  // ks, dims 16 ks + 8 g + j.
  // Returns -1152 * sum(q) of the column: the S accumulator's start value, which cancels the code
  // bias that K keeps (V's is removed during the expansion).
  __device__ static __forceinline__ float load_q(const AttnIO& io, int64_t elem, bool valid, int lane, half8_t (&qb)[KS]) {
    const int g = lane >> 5;
    const uint32_t okmask = valid ? 0xffffffffu : 0u;
    float qsum = 0.f;
    u32x4 raw[QDT == KVQ_F32 ? 1 : KS];
    if constexpr (QDT != KVQ_F32) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        raw[ks] = *reinterpret_cast<const u32x4_a4*>(reinterpret_cast<const uint16_t*>(io.q) + elem + 16 * ks + 8 * g);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      float f[8];
      if constexpr (QDT == KVQ_F32) {
        const float* p = reinterpret_cast<const float*>(io.q) + elem + 16 * ks + 8 * g;
        const floatx4 v0 = *reinterpret_cast<const floatx4_a4*>(p), v1 = *reinterpret_cast<const floatx4_a4*>(p + 4);
        f[0] = v0.x; f[1] = v0.y; f[2] = v0.z; f[3] = v0.w; f[4] = v1.x; f[5] = v1.y; f[6] = v1.z; f[7] = v1.w;
      } else {
        const u32x4 v = raw[ks];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t e = v[w];
          if constexpr (QDT == KVQ_BF16) {
            f[2 * w] = as_f32(e << 16);
            f[2 * w + 1] = as_f32(e & 0xffff0000u);
          } else {
            const half2_t hh = __builtin_bit_cast(half2_t, e);
            f[2 * w] = (float)hh.x;
            f[2 * w + 1] = (float)hh.y;
          }
        }
      }
      u32x4 hb;
      hb.x = pack_half2(clamp_half_range(f[0]), clamp_half_range(f[1])) & okmask;
      hb.y = pack_half2(clamp_half_range(f[2]), clamp_half_range(f[3])) & okmask;
      hb.z = pack_half2(clamp_half_range(f[4]), clamp_half_range(f[5])) & okmask;
      hb.w = pack_half2(clamp_half_range(f[6]), clamp_half_range(f[7])) & okmask;
      qb[ks] = __builtin_bit_cast(half8_t, hb);
#pragma unroll
      for (int j = 0; j < 8; ++j) qsum += (float)qb[ks][j];  // the sum of what the MFMA will actually see
    }
    qsum += __shfl_xor(qsum, 32, kWave);
    return FP8 ? 0.f : -DTile::kBias * qsum;
  }

  // Two nibbles of y (= code bytes ^ 0x88..., see nibbles_to_half2) as two fp16 codes, bias taken out.
  __device__ static __forceinline__ uint32_t nibbles_to_codes(uint32_t y, int k) {
    const half2_t bias = {(half_t)kCodeBiasInt4, (half_t)kCodeBiasInt4};
    const half2_t v = __builtin_bit_cast(half2_t, nibbles_to_half2(y, k)) - bias;
    return __builtin_bit_cast(uint32_t, v);
  }

  // The int4 form of expand(): one thread converts one 16-byte K chunk (32 codes, put back into dim order: the
  // and-or conversion yields dims 0 4 1 5 2 6 3 7 of a dword) and one 4-token x 4-dim V block (two bytes per token).
  __device__ static __forceinline__ void expand_int4(const uint8_t* raw, uint8_t* buf, int tid) {
    constexpr int KCH = DB / 16;
    if (tid < kTile * KCH) {
      const int tok = tid / KCH, ch = tid % KCH;
      const u32x4 w = *reinterpret_cast<const u32x4*>(raw + tok * RAW_PITCH + 16 * ch);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t y = w[i] ^ 0x88888888u;
        const uint32_t h0 = nibbles_to_half2(y, 0), h1 = nibbles_to_half2(y, 1);   // dims (0, 4), (1, 5)
        const uint32_t h2 = nibbles_to_half2(y, 2), h3 = nibbles_to_half2(y, 3);   // dims (2, 6), (3, 7)
        u32x4 o;
        o.x = perm(h1, h0, kPermLowHalves);
        o.y = perm(h3, h2, kPermLowHalves);
        o.z = perm(h1, h0, kPermHighHalves);
        o.w = perm(h3, h2, kPermHighHalves);
        *reinterpret_cast<u32x4*>(buf + tok * K_PITCH + 64 * ch + 16 * i) = o;
      }
    }
    if (tid < 8 * (D / 4)) {
      const int tg = tid & 7, dq = tid >> 3;
      uint32_t t[4];
#pragma unroll
      for (int a = 0; a < 4; ++a)
        t[a] = *reinterpret_cast<const uint16_t*>(raw + (4 * tg + a) * RAW_PITCH + (DB + 4) + 2 * dq);
      const uint32_t y01 = (t[0] | (t[1] << 16)) ^ 0x88888888u, y23 = (t[2] | (t[3] << 16)) ^ 0x88888888u;
      const int pos = (tg >> 2) * 16 + (tg & 1) * 8 + ((tg >> 1) & 1) * 4;
      uint8_t* vrow = buf + K_BYTES + (4 * dq) * V_PITCH + 2 * pos;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        u32x2 o;
        o.x = nibbles_to_codes(y01, b);
        o.y = nibbles_to_codes(y23, b);
        *reinterpret_cast<u32x2*>(vrow + b * V_PITCH) = o;
      }
    }
  }

  // Raw tile -> fp16 K [token][dim] (codes + 1152) and V^T [dim][position] (codes); token t of the tile sits at position
  // (t/16)*16 + ((t%8)/4)*8 + ((t/8)%2)*4 + t%4, the order in which the 32x32 S accumulator hands a
  // lane its tokens.  One thread converts one 16-code K chunk and one 4-token x 4-dim V block.
  __device__ static __forceinline__ void expand(const uint8_t* raw, uint8_t* buf, int tid, float sc_mul, uint32_t l_sc) {
    constexpr int KCH = D / 16;
    if constexpr (INT4) {
      expand_int4(raw, buf, tid);
    } else {
    if (tid < kTile * KCH) {
      const int tok = tid / KCH, ch = tid % KCH;
      const u32x4 w = *reinterpret_cast<const u32x4*>(raw + tok * RAW_PITCH + 16 * ch);
      u32x4 lo, hi;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t x = prep_codes<FP8>(w[i]);
        lo[2 * i] = codes_to_half2<FP8>(x, false);
        lo[2 * i + 1] = codes_to_half2<FP8>(x, true);
        const uint32_t y = prep_codes<FP8>(w[2 + i]);
        hi[2 * i] = codes_to_half2<FP8>(y, false);
        hi[2 * i + 1] = codes_to_half2<FP8>(y, true);
      }
      *reinterpret_cast<u32x4*>(buf + tok * K_PITCH + 32 * ch) = lo;
      *reinterpret_cast<u32x4*>(buf + tok * K_PITCH + 32 * ch + 16) = hi;
    }
    if (tid < 8 * (D / 4)) {
      const int tg = tid & 7, dq = tid >> 3;
      uint32_t t[4];
#pragma unroll
      for (int a = 0; a < 4; ++a)
        t[a] = prep_codes<FP8>(*reinterpret_cast<const uint32_t*>(raw + (4 * tg + a) * RAW_PITCH + (D + 4) + 4 * dq));
      const uint32_t a01 = perm(t[1], t[0], 0x05010400u), b01 = perm(t[1], t[0], 0x07030602u);
      const uint32_t a23 = perm(t[3], t[2], 0x05010400u), b23 = perm(t[3], t[2], 0x07030602u);
      const int pos = (tg >> 2) * 16 + (tg & 1) * 8 + ((tg >> 1) & 1) * 4;
      uint8_t* vrow = buf + K_BYTES + (4 * dq) * V_PITCH + 2 * pos;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t p01 = (b < 2) ? a01 : b01, p23 = (b < 2) ? a23 : b23;
        u32x2 o;
        o.x = to_half2(p01, b & 1);
        o.y = to_half2(p23, b & 1);
        *reinterpret_cast<u32x2*>(vrow + b * V_PITCH) = o;
      }
    }
    }
    if (tid < 64) {
      const float sc = *reinterpret_cast<const float*>(raw + l_sc);
      const float val = fminf(sc * sc_mul, 65504.f);
      reinterpret_cast<float*>(buf + K_BYTES + V_BYTES)[tid] = val;
      // How far a logit may exceed a column's reference maximum in this tile before the maximum has
      // to move: 2^kLazyMax * (largest V-side scale) must stay inside fp16, else nothing is allowed.
      const bool big = tid >= 32 && val > kLazyScaleMax;
      const bool any_big = __builtin_amdgcn_ballot_w64(big) != 0;
      if (tid == 0) reinterpret_cast<float*>(buf + K_BYTES + V_BYTES)[64] = any_big ? 0.f : kLazyMax;
    }
  }

  // One tile for the wave's 32 columns.  S^T[32 tokens, 32 columns]: lane (c = column, g) holds
  // token (i/4)*8 + 4g + i%4 in register i.
  // EXT: the column sees only tokens [limit - wspan, limit) (sliding window), the logits may
  // pass through the soft cap (cap_c != 0) and take the ALiBi bias ali x (token - (limit - 1)) when `biased` (uniform;
  // the column's query stands at limit - 1); without EXT wspan, cap_c, cap_k, ali and biased are not looked at.
  template <bool MASK, bool EXT>
  __device__ static __forceinline__ void compute(const uint8_t* buf, const half8_t (&qb)[KS], float s_init, int limit,
                                                 uint32_t wspan, float cap_c, float cap_k, int t, int lane,
                                                 floatx16 (&o)[MT], float& m, float& l, float ali = 0.f,
                                                 bool biased = false) {
    const int c = lane & 31, g = lane >> 5;
    const float* sc = reinterpret_cast<const float*>(buf + K_BYTES + V_BYTES);
    floatx16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = s_init;
    const uint8_t* krow = buf + c * K_PITCH + g * 16;
    // From here to the end of the tile's products the wave outranks the waves of its SIMD that are expanding the next
    // tile or waiting at the barrier: with equal priorities the two waves of a SIMD take turns instruction by
    // instruction and both phases stretch.  Measured on MI355X: the mixed batch of 4 x 2048 new tokens 702.5 -> 689.5 us
    // per attention call, one 8192-token prompt 732 -> 715 us, short prompts unchanged; raising the priority around
    // the two MFMA runs only (the softmax between them at 0) was slower than no priorities at all (724 us).
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const half8_t ka = *reinterpret_cast<const half8_t*>(krow + 32 * ks);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qb[ks], s, 0, 0, 0);
    }
    // Logits are taken relative to the running maximum in the same multiply-add that applies the K
    // scale: y = s * k_scale - m.  While no column's maximum moves (the usual case after the first
    // tiles) p = exp2(y) needs no further subtraction.
    const int tok_base = t * kTile + 4 * g;
    const bool fresh = m == -INFINITY;          // the column has seen no visible token yet
    const float mref = fresh ? 0.f : m;
    float d = -INFINITY;
    bool capped = false;
    if constexpr (EXT) capped = cap_c != 0.f;  // uniform
    if (capped) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const floatx4 ksc = *reinterpret_cast<const floatx4*>(sc + 8 * q + 4 * g);
#pragma unroll
        for (int r = 0; r < 4; ++r) s[4 * q + r] = soft_cap(s[4 * q + r] * ksc[r], cap_c, cap_k) - mref;
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const floatx4 ksc = *reinterpret_cast<const floatx4*>(sc + 8 * q + 4 * g);
#pragma unroll
        for (int r = 0; r < 4; ++r) s[4 * q + r] = __builtin_fmaf(s[4 * q + r], ksc[r], -mref);
      }
    }
    if constexpr (EXT) {
      if (biased) {
        const float rel0 = (float)(tok_base - (limit - 1));
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = __builtin_fmaf(ali, rel0 + (float)((i >> 2) * 8 + (i & 3)), s[i]);
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float y = s[4 * q + r];
        if constexpr (MASK) {
          if constexpr (EXT) y = ((uint32_t)(limit - 1 - (tok_base + q * 8 + r)) < wspan) ? y : -INFINITY;
          else y = ((tok_base + q * 8 + r) < limit) ? y : -INFINITY;
        }
        s[4 * q + r] = y;
        d = fmaxf(d, y);
      }
    }
    d = max_over_halves(d);
    // How far the reference maximum moves: a fresh column takes d itself (0 while it still sees
    // nothing); otherwise it only has to keep 2^(logit - m) in range, not be the true maximum, and
    // stays put while no logit exceeds it by more than the tile's allowance.  With 32 columns per
    // wave SOME true maximum moves in most tiles of the first thousand tokens, and each move rescales
    // every accumulator of the wave; the lazy reference moves a few times per column.
    const float allow = sc[64];
    const float up = fresh ? (d == -INFINITY ? 0.f : d) : (d > allow ? d : 0.f);
    if (__builtin_amdgcn_ballot_w64(up != 0.f) != 0) {
      // a fresh column's o and l are still zero and stay so (its first logits may lie so far below zero, under an
      // ALiBi bias, that 2^-up is no finite number)
      const float alpha = fresh ? 0.f : __builtin_amdgcn_exp2f(-up);
      l *= alpha;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) o[mt] *= alpha;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] -= up;
    }
    m = (fresh && d == -INFINITY) ? -INFINITY : mref + up;
    half8_t p_op[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      float pt[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int q = 2 * kt + h;
        const floatx4 vsc = *reinterpret_cast<const floatx4*>(sc + 32 + 8 * q + 4 * g);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = __builtin_amdgcn_exp2f(s[4 * q + r]);
          l += p;
          float x = p * vsc[r];
          if constexpr (MASK) {
            if constexpr (EXT) x = ((uint32_t)(limit - 1 - (tok_base + q * 8 + r)) < wspan) ? x : 0.f;
            else x = ((tok_base + q * 8 + r) < limit) ? x : 0.f;
          }
          pt[4 * h + r] = x;
        }
      }
      u32x4 pb;
      pb.x = pack_half2(pt[0], pt[1]);
      pb.y = pack_half2(pt[2], pt[3]);
      pb.z = pack_half2(pt[4], pt[5]);
      pb.w = pack_half2(pt[6], pt[7]);
      p_op[kt] = __builtin_bit_cast(half8_t, pb);
    }
    const uint8_t* vrow = buf + K_BYTES + c * V_PITCH + g * 16;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const half8_t va = *reinterpret_cast<const half8_t*>(vrow + mt * 32 * V_PITCH + 32 * kt);
        o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, p_op[kt], o[mt], 0, 0, 0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
  }
};

// EXT adds the sliding window and the logits soft cap; the plain causal kernel carries neither.
// KSPLIT (with EXT only): the grid's x dimension carries a.ksplit context splits per query block; a workgroup takes
// one range of its item's tiles and writes a partial state instead of the rows.
template <int D, int QDT, int ODT, bool EXT, int CODE = KVQ_CODE_INT8, bool KSPLIT = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void paged_prefill_flash32_kernel(PrefillArgs a) {
  static_assert(!KSPLIT || EXT, "the context split is built into the kernel with the extras only");
  using FP = Flash32<D, QDT, ODT, CODE>;
  using DTile = typename FP::DTile;
  extern __shared__ __align__(16) uint8_t lds[];
  uint8_t* raws = lds;
  uint8_t* bufs = lds + 2 * FP::RAW_BYTES;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Which sequence, kv head and query block this workgroup takes.  Workgroups start in the order of their linear
  // number and go to the eight XCDs in turn by it.  The number is read over the sequences that HAVE a query run
  // (the plan; the surplus workgroups of the grid, which is sized for every sequence of the batch, come last and
  // leave at once), sequence by sequence, and inside a sequence query-block-major over its kv heads, longest block
  // first: the heads of a sequence then walk the same tokens at the same time (their records are neighbours in
  // memory, and what one head's workgroup brought into L2 is there for the next), and the head is shifted by the
  // block number so that a head's blocks visit every XCD in turn.  Measured against the grid read as launched
  // (block, sequence, head): the mixed batch of 4 x 2048 new tokens 852 -> 752 us per attention call, one
  // 8192-token prompt 908 -> 733 us, 16 prompts of 1024 tokens 410 -> 291 us (there XCD 0 had the longest block
  // of every eight of every pair), 4 x 1024 new tokens on 8k-32k cached ones 2.43 -> 2.02 ms.  Query-block-major
  // over ALL pairs was better still for short prompts from scratch (16 x 512: 103 against 113 us) and much worse
  // with long contexts (the mixed batch 959 us: sixteen streams of keys at once, six times the HBM fetches).
  const unsigned nsplit = KSPLIT ? (unsigned)a.ksplit : 1u;
  const unsigned nqb = gridDim.x / nsplit, hk = gridDim.z, per_seq = nqb * hk;
  const unsigned nseq = (unsigned)a.plan[0];
  const unsigned lin_all = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const unsigned split = KSPLIT ? lin_all % nsplit : 0u;   // the splits of an item are neighbours in launch order
  const unsigned lin = KSPLIT ? lin_all / nsplit : lin_all;
  if (lin >= per_seq * nseq) return;   // uniform over the workgroup
  const unsigned rem = lin % per_seq;
  const int qb = (int)(rem / hk);
  const int hkv = (int)((rem % hk + (unsigned)qb) % hk);
  const int seq = a.plan[1 + lin / per_seq];
  const AttnIO& io = a.io;
  const int q_begin = a.cu_seqlens_q[seq];
  const int q_len = a.cu_seqlens_q[seq + 1] - q_begin;
  const int len = a.seq_lens[seq];
  const int q0 = ((int)nqb - 1 - qb) * a.q_tokens;
  if (q_len <= 1 || q0 >= q_len || len <= 0) return;   // uniform over the workgroup
  if (a.route == 1 && q_len * io.group < 64) return;    // the per-wave tile's

  // column of this lane: (query token q0 + n / group, head n % group), n = wave * 32 + (lane & 31)
  const int ctx = len - q_len;
  const int n = wave * 32 + (lane & 31);
  const int qt = n / io.group;
  const int qi = q0 + qt;
  const bool valid = qt < a.q_tokens && qi < q_len;
  const int head = hkv * io.group + (n - qt * io.group);
  const int64_t row = q_begin + (valid ? qi : q0);
  int lim = a.causal ? ctx + qi + 1 : len;
  lim = lim < 0 ? 0 : (lim > len ? len : lim);
  const int limit = valid ? lim : 0;
  const int wave_max_limit = wave_max_i32(limit);
  const int wave_min_limit = -wave_max_i32(valid ? -lim : -0x7fffffff);
  int wg_limit = a.causal ? ctx + min(q0 + a.q_tokens, q_len) : len;
  wg_limit = wg_limit < 0 ? 0 : (wg_limit > len ? len : wg_limit);
  const int t_end = (wg_limit + kTile - 1) / kTile;
  // Sliding window: a column sees [limit - window, limit).  The workgroup starts at the (even) tile
  // pair that holds the first query token's lower edge; a wave masks tiles below the latest lower
  // edge among its columns and skips those that end before the earliest.
  uint32_t wspan = 0x7fffffffu;
  int t_first = 0, wave_min_first = 0, wave_max_first = 0;
  if constexpr (EXT) {
    if (io.window > 0) {
      wspan = (uint32_t)io.window;
      int wg_first = (a.causal ? ctx + q0 + 1 : len) - io.window;
      wg_first = wg_first < 0 ? 0 : wg_first;
      t_first = (wg_first / kTile) & ~1;
      wave_min_first = max(0, wave_min_limit - io.window);
      wave_max_first = max(0, wave_max_limit - io.window);
    }
  }

  floatx16 o[FP::MT];
#pragma unroll
  for (int mt = 0; mt < FP::MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[mt][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  // this workgroup's tiles: all of the item's, or one of nsplit ranges of an even number of tiles
  int t_lo = t_first, t_hi = t_end;
  if constexpr (KSPLIT) {
    const int per = (((t_end - t_first) + (int)nsplit - 1) / (int)nsplit + 1) & ~1;
    t_lo = t_first + (int)split * per;
    t_hi = min(t_end, t_lo + per);
  }
  if (t_hi > t_lo) {
    const LaneOffsets lo = DTile::lane_offsets(io.g, lane);
    const int32_t* bt_row = io.block_table + (int64_t)seq * io.bt_stride;
    const int step = (64 / DTile::NCH) * (int)io.g.stride_slot;
    // every wave: chunk load (wave % NLD) of both 16-token halves and the record tails of half
    // (wave & 1), unconditionally and in the same order in every step
    const int half = wave & 1;
    const int ld_n = wave % DTile::NLD;
    struct Regs {
      u32x4 c0, c1;
      u32x2 tail;
    };
    Regs A{}, B{};
    auto issue = [&](const TileBlocks& nb, int t, Regs& r) __attribute__((always_inline)) {
      const typename DTile::Window w = DTile::window(io, nb, t, hkv);
      r.c0 = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r0, lo.g_chunk, ld_n * step, 0));
      r.c1 = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w.r1, lo.g_chunk, ld_n * step, 0));
      r.tail = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(half ? w.r1 : w.r0, lo.g_tail, 0, 0));
    };
    const uint32_t l_chunk = lo.l_chunk + ld_n * (64 / DTile::NCH) * FP::RAW_PITCH;
    const uint32_t l_tail = (16 * half + (lane & 15)) * FP::RAW_PITCH + 2 * FP::DB;
    auto drop = [&](const Regs& r, uint8_t* raw) __attribute__((always_inline)) {
      *reinterpret_cast<u32x4*>(raw + l_chunk) = r.c0;
      *reinterpret_cast<u32x4*>(raw + l_chunk + 16 * FP::RAW_PITCH) = r.c1;
      if (wave < 2 && lane < 16) *reinterpret_cast<u32x2*>(raw + l_tail) = r.tail;
    };
    TileBlocks nb = DTile::fetch_blocks(io, bt_row, len, t_lo);
    issue(nb, t_lo, A);
    nb = DTile::fetch_blocks(io, bt_row, len, t_lo + 1);
    issue(nb, t_lo + 1, B);
    nb = DTile::fetch_blocks(io, bt_row, len, t_lo + 2);

    half8_t qb[FP::KS];
    const float s_init =
        FP::load_q(io, row * io.q_stride_t + (int64_t)(valid ? head : hkv * io.group) * io.q_stride_h, valid, lane, qb);
    const float sc_mul = lane < 32 ? io.scale_log2 * DTile::kKScaleMul : kPScale;
    float ali = 0.f;
    bool biased = false;
    if constexpr (EXT) {
      biased = io.alibi != nullptr;
      ali = alibi_slope(io.alibi, valid ? head : hkv * io.group);
    }

    drop(A, raws);  // t_lo is even: raw window 0
    issue(nb, t_lo + 2, A);
    nb = DTile::fetch_blocks(io, bt_row, len, t_lo + 3);
    lds_barrier();
    // Step t: expand raw tile t into fp16 buffer t&1, drop tile t+1 (held in `next`) into the other
    // raw window and refill `next` with tile t+3, ONE barrier, then compute tile t.
    auto step_fn = [&](auto masked, int t, Regs& next) __attribute__((always_inline)) {
      uint8_t* buf = bufs + (t & 1) * FP::BUF_BYTES;
      FP::expand(raws + (t & 1) * FP::RAW_BYTES, buf, tid, sc_mul, lo.l_sc);
      drop(next, raws + ((t + 1) & 1) * FP::RAW_BYTES);
      issue(nb, t + 3, next);
      lds_barrier();
      nb = DTile::fetch_blocks(io, bt_row, len, t + 4);
      if constexpr (decltype(masked)::value) {
        bool live = t * kTile < wave_max_limit;
        if constexpr (EXT) live = live && (t + 1) * kTile > wave_min_first;
        if (live)
          FP::template compute<true, EXT>(buf, qb, s_init, limit, wspan, io.cap_c, io.cap_k, t, lane, o, m, l, ali, biased);
      } else {
        FP::template compute<false, EXT>(buf, qb, s_init, limit, wspan, io.cap_c, io.cap_k, t, lane, o, m, l, ali, biased);
      }
    };
    // Tiles below every column's limit need no mask.  They and the masked tail are two separate
    // loops (every wave runs the same number of steps, hence of barriers, whichever loop a step is
    // in), so that the accumulators keep their registers across the loop instead of being merged
    // at a branch inside it.
    const int t_plain = min(t_hi, wave_min_limit / kTile) & ~1;
    int t = t_lo;
    if constexpr (EXT) {  // tiles that straddle a column's lower window edge
      const int t_head = min(t_hi, ((wave_max_first + kTile - 1) / kTile + 1) & ~1);
      for (; t < t_head; t += 2) {
        step_fn(std::true_type{}, t, B);
        step_fn(std::true_type{}, t + 1, A);
      }
    }
    for (; t < t_plain; t += 2) {
      step_fn(std::false_type{}, t, B);
      step_fn(std::false_type{}, t + 1, A);
    }
    for (; t < t_hi; t += 2) {  // an odd end runs one step past it: that step computes nothing
      step_fn(std::true_type{}, t, B);
      step_fn(std::true_type{}, t + 1, A);
    }
  }
  // Lane (c, g) holds O[column][dim mt*32 + (i/4)*8 + 4g + i%4] in o[mt][i].
  l += __shfl_xor(l, 32, kWave);
  if (!valid) return;
  if constexpr (KSPLIT) {
    // the range's state: the row as accumulated (without the factor the weights carry), the reference maximum, the sum
    float* p = a.part + (((int64_t)row * io.num_q_heads + head) * nsplit + split) * (D + 2);
    const float unit = 1.0f / DTile::kOutDiv;
    const int gg = lane >> 5;
#pragma unroll
    for (int mt = 0; mt < FP::MT; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<floatx4_a4*>(p + mt * 32 + q * 8 + 4 * gg) =
            (floatx4){o[mt][4 * q] * unit, o[mt][4 * q + 1] * unit, o[mt][4 * q + 2] * unit, o[mt][4 * q + 3] * unit};
    if (gg == 0) {
      p[D] = m;
      p[D + 1] = l;
    }
    return;
  }
  if (l > 0.f) l += sink_term(io.sinks, head, m);   // a row without a visible key keeps its zeros
  const int g = lane >> 5;
  const float mul = l > 0.f ? 1.0f / (l * DTile::kOutDiv) : 0.f;
  const int64_t base = row * io.out_stride_t + (int64_t)head * io.out_stride_h + 4 * g;
#pragma unroll
  for (int mt = 0; mt < FP::MT; ++mt) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      floatx4 v;
      v.x = o[mt][4 * q + 0] * mul;
      v.y = o[mt][4 * q + 1] * mul;
      v.z = o[mt][4 * q + 2] * mul;
      v.w = o[mt][4 * q + 3] * mul;
      const int64_t at = base + mt * 32 + q * 8;
      if constexpr (ODT == KVQ_F32) {
        *reinterpret_cast<floatx4_a4*>(reinterpret_cast<float*>(io.out) + at) = v;
      } else {
        u32x2 pk;
        if constexpr (ODT == KVQ_BF16) {
          pk.x = (uint32_t)f32_to_bf16_bits(v.x) | ((uint32_t)f32_to_bf16_bits(v.y) << 16);
          pk.y = (uint32_t)f32_to_bf16_bits(v.z) | ((uint32_t)f32_to_bf16_bits(v.w) << 16);
        } else {
          pk.x = pack_half2(v.x, v.y);
          pk.y = pack_half2(v.z, v.w);
        }
        *reinterpret_cast<u32x2_a4*>(reinterpret_cast<uint16_t*>(io.out) + at) = pk;
      }
    }
  }
  if (io.lse != nullptr && g == 0)
    io.lse[row * io.num_q_heads + head] = l > 0.f ? (m + __builtin_amdgcn_logf(l)) * kLn2 : -INFINITY;
}

// The merge of the context splits: grid (query token of a run, sequence of the plan), 4 waves; a wave takes q heads
// wave, wave + 4, ... of its row, a lane D / 64 dims.  out = sum_s w_s o_s / sum_s w_s l_s with w_s = 2^(m_s - max m):
// the algebra of merge_attn_states over the splits' states; the sink's term and the row's lse as in the unsplit kernel.
template <int D, int ODT>
__global__ __launch_bounds__(256) void prefill_split_merge_kernel(PrefillArgs a) {
  constexpr int V = D / 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (blockIdx.y >= (unsigned)a.plan[0]) return;
  const int seq = a.plan[1 + blockIdx.y];
  const int q_begin = a.cu_seqlens_q[seq];
  const int q_len = a.cu_seqlens_q[seq + 1] - q_begin;
  const int qi = blockIdx.x;
  if (q_len <= 1 || qi >= q_len || a.seq_lens[seq] <= 0) return;
  const AttnIO& io = a.io;
  const int64_t row = q_begin + qi;
  const int S = a.ksplit;
  for (int head = wave; head < io.num_q_heads; head += 4) {
    const float* p = a.part + ((row * io.num_q_heads + head) * S) * (D + 2);
    float mmax = -INFINITY;
    for (int s = 0; s < S; ++s) mmax = fmaxf(mmax, p[s * (D + 2) + D]);
    const float mref = mmax == -INFINITY ? 0.f : mmax;
    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;
    float l = 0.f;
    for (int s = 0; s < S; ++s) {
      const float* ps = p + s * (D + 2);
      const float w = __builtin_amdgcn_exp2f(ps[D] - mref);   // an empty range: 2^-inf = 0
      l += w * ps[D + 1];
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] += w * ps[V * lane + i];
    }
    if (l > 0.f) l += sink_term(io.sinks, head, mmax);   // a row without a visible key keeps its zeros
    const float mul = l > 0.f ? 1.0f / l : 0.f;
    const int64_t at = row * io.out_stride_t + (int64_t)head * io.out_stride_h + V * lane;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float v = acc[i] * mul;
      if constexpr (ODT == KVQ_F32) reinterpret_cast<float*>(io.out)[at + i] = v;
      else if constexpr (ODT == KVQ_BF16) reinterpret_cast<uint16_t*>(io.out)[at + i] = f32_to_bf16_bits(v);
      else reinterpret_cast<uint16_t*>(io.out)[at + i] = (uint16_t)(pack_half2(v, 0.f) & 0xffffu);
    }
    if (io.lse != nullptr && lane == 0)
      io.lse[row * io.num_q_heads + head] = l > 0.f ? (mmax + __builtin_amdgcn_logf(l)) * kLn2 : -INFINITY;
  }
}

template <int D, int QDT, int ODT, bool EXT, int CODE = KVQ_CODE_INT8>
static int launch_prefill_flash32(PrefillArgs& a, int max_query_len, hipStream_t s) {
  using FP = Flash32<D, QDT, ODT, CODE>;
  a.q_tokens = FP::COLS / a.io.group;
  const int blocks = (max_query_len + a.q_tokens - 1) / a.q_tokens;
  if (a.num_seqs > 65535 || a.io.g.num_kv_heads > 65535) return fail(KVQ_EINVAL, "paged_attn_int8: prefill grid out of range");
  static_assert(FP::LDS_BYTES <= 64 * 1024, "static LDS opt-in would be needed");
  if constexpr (EXT) {
    if (a.ksplit > 1) {
      dim3 grid(blocks * a.ksplit, a.num_seqs, a.io.g.num_kv_heads);
      hipLaunchKernelGGL((paged_prefill_flash32_kernel<D, QDT, ODT, true, CODE, true>), grid, dim3(256), FP::LDS_BYTES, s, a);
      if (int e = check_hip(hipGetLastError(), "paged_prefill_flash32 launch")) return e;
      dim3 mgrid(max_query_len, a.num_seqs);
      hipLaunchKernelGGL((prefill_split_merge_kernel<D, ODT>), mgrid, dim3(256), 0, s, a);
      return check_hip(hipGetLastError(), "prefill split merge launch");
    }
  }
  dim3 grid(blocks, a.num_seqs, a.io.g.num_kv_heads);
  hipLaunchKernelGGL((paged_prefill_flash32_kernel<D, QDT, ODT, EXT, CODE>), grid, dim3(256), FP::LDS_BYTES, s, a);
  return check_hip(hipGetLastError(), "paged_prefill_flash32 launch");
}

// Launches with this many items (query block x sequence x kv head) or fewer spread each item over a workgroup's waves.
constexpr int64_t kSplitItems = 2048;

template <int D, int QDT, int ODT, int NT, int WPW, int CODE = KVQ_CODE_INT8>
static int launch_prefill_cfg(const PrefillArgs& a, int max_query_len, hipStream_t s) {
  const int blocks = (max_query_len + a.q_tokens - 1) / a.q_tokens;
  if (blocks > 0x7fffffff / 2 || a.num_seqs > 65535) return fail(KVQ_EINVAL, "paged_attn_int8: prefill grid out of range");
  // (not in the batch-invariant mode: how an item is cut would depend on what else the launch holds)
  if (!batch_invariant() && (int64_t)blocks * a.num_seqs * a.io.g.num_kv_heads <= kSplitItems &&
      a.io.g.num_kv_heads <= 65535) {
    // waves per item: eight with one column tile per wave; four with two (their accumulators need the registers
    // of a 256-thread workgroup)
    constexpr int SW = NT == 1 ? 8 : 4;
    dim3 grid(blocks, a.num_seqs, a.io.g.num_kv_heads);
    hipLaunchKernelGGL((paged_prefill_kernel<D, QDT, ODT, NT, SW, CODE, true>), grid, dim3(SW * 64), 0, s, a);
    return check_hip(hipGetLastError(), "paged_prefill launch");
  }
  dim3 grid(blocks, a.num_seqs, (a.io.g.num_kv_heads + WPW - 1) / WPW);
  hipLaunchKernelGGL((paged_prefill_kernel<D, QDT, ODT, NT, WPW, CODE>), grid, dim3(WPW * 64), 0, s, a);
  return check_hip(hipGetLastError(), "paged_prefill launch");
}

template <int D, int QDT, int ODT>
static int launch_prefill_nt(PrefillArgs& a, int max_query_len, hipStream_t s);

// Batch-invariant mode: every run goes to the kernel its OWN length chooses.  Runs that fill the workgroup-shared
// tile by themselves take it; the others take the per-wave tile with one column tile per wave -- in a second launch
// when the batch holds both kinds.
template <int D, int QDT, int ODT>
static int launch_prefill_invariant(PrefillArgs& a, int max_query_len, hipStream_t s) {
  const int group = a.io.group;
  if (D <= 128 && max_query_len * group >= 64) {
    a.route = 1;
    if (int e = launch_prefill_nt<D, QDT, ODT>(a, max_query_len, s)) return e;
    a.route = 2;
    const int longest_short = (63 / group);        // q_len x group < 64
    if (longest_short < 2) return KVQ_OK;           // no run of two tokens or more is short
    return launch_prefill_nt<D, QDT, ODT>(a, longest_short, s);
  }
  a.route = 0;
  return launch_prefill_nt<D, QDT, ODT>(a, max_query_len, s);
}

template <int D, int QDT, int ODT>
static int launch_prefill_nt(PrefillArgs& a, int max_query_len, hipStream_t s) {
  constexpr int WPW = 4;
  const bool fp8 = a.io.g.code_type == KVQ_CODE_FP8_E4M3;
  const bool int4 = a.io.g.code_type == KVQ_CODE_INT4;
  // long runs: the workgroup-shared fp16 tile (compute-bound shape), for every kind of code
  if constexpr (D <= 128) {
    if (max_query_len * a.io.group >= 64 && a.route != 2) {
      const bool ext = a.io.window > 0 || a.io.cap_c != 0.f || a.io.alibi != nullptr || a.ksplit > 1;
      if (int4) {
        if (ext) return launch_prefill_flash32<D, QDT, ODT, true, KVQ_CODE_INT4>(a, max_query_len, s);
        return launch_prefill_flash32<D, QDT, ODT, false, KVQ_CODE_INT4>(a, max_query_len, s);
      }
      if (fp8) {
        if (ext) return launch_prefill_flash32<D, QDT, ODT, true, KVQ_CODE_FP8_E4M3>(a, max_query_len, s);
        return launch_prefill_flash32<D, QDT, ODT, false, KVQ_CODE_FP8_E4M3>(a, max_query_len, s);
      }
      if (ext) return launch_prefill_flash32<D, QDT, ODT, true>(a, max_query_len, s);
      return launch_prefill_flash32<D, QDT, ODT, false>(a, max_query_len, s);
    }
  }
  if (fp8) {  // short runs of fp8 codes: the per-wave tile, one column tile per wave
    a.q_tokens = 16 / a.io.group;
    return launch_prefill_cfg<D, QDT, ODT, 1, WPW, KVQ_CODE_FP8_E4M3>(a, max_query_len, s);
  }
  if (int4) {
    a.q_tokens = 16 / a.io.group;
    return launch_prefill_cfg<D, QDT, ODT, 1, WPW, KVQ_CODE_INT4>(a, max_query_len, s);
  }
  // two column tiles per wave where the accumulators fit the register file next to a tile in flight
  if (D <= 128 && a.io.group * 2 <= 32 && max_query_len * a.io.group > 16 && !batch_invariant()) {
    a.q_tokens = 32 / a.io.group;
    return launch_prefill_cfg<D, QDT, ODT, (D <= 128 ? 2 : 1), WPW>(a, max_query_len, s);
  }
  a.q_tokens = 16 / a.io.group;
  return launch_prefill_cfg<D, QDT, ODT, 1, WPW>(a, max_query_len, s);
}

template <int D, int QDT>
static int launch_prefill_o(PrefillArgs& a, int max_query_len, int out_dtype, hipStream_t s) {
  switch (out_dtype) {
    case KVQ_F32: return batch_invariant() ? launch_prefill_invariant<D, QDT, KVQ_F32>(a, max_query_len, s)
                                           : launch_prefill_nt<D, QDT, KVQ_F32>(a, max_query_len, s);
    case KVQ_BF16: return batch_invariant() ? launch_prefill_invariant<D, QDT, KVQ_BF16>(a, max_query_len, s)
                                            : launch_prefill_nt<D, QDT, KVQ_BF16>(a, max_query_len, s);
    case KVQ_F16: return batch_invariant() ? launch_prefill_invariant<D, QDT, KVQ_F16>(a, max_query_len, s)
                                           : launch_prefill_nt<D, QDT, KVQ_F16>(a, max_query_len, s);
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
                   int max_query_len, int causal, int q_dtype, int out_dtype, int32_t* plan, hipStream_t s,
                   int ksplit, float* part) {
  PrefillArgs a{};
  a.ksplit = ksplit;
  a.part = part;
  a.io = io;
  a.seq_lens = seq_lens;
  a.cu_seqlens_q = cu_seqlens_q;
  a.num_seqs = num_seqs;
  a.causal = causal;
  a.plan = plan;
  hipLaunchKernelGGL(prefill_plan_kernel, dim3(1), dim3(64), 0, s, seq_lens, cu_seqlens_q, num_seqs, plan);
  if (int e = check_hip(hipGetLastError(), "prefill plan launch")) return e;
  switch (io.g.head_size) {
    case 64: return launch_prefill_q<64>(a, max_query_len, q_dtype, out_dtype, s);
    case 128: return launch_prefill_q<128>(a, max_query_len, q_dtype, out_dtype, s);
    default: return launch_prefill_q<256>(a, max_query_len, q_dtype, out_dtype, s);
  }
}

}  // namespace kvq
