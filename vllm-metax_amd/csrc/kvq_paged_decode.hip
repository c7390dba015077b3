// Paged decode attention over the int8 cache: work decomposition and reduce (gfx950).
//
// Balanced split-K ("stream-K" over tokens): the 32-token tiles of all decode
// sequences form one global work line (one unit per tile, plus a small charge per
// sequence start); the launch has exactly as many workgroups as the device keeps
// resident and workgroup w takes units [w*T/P, (w+1)*T/P), whatever sequence
// boundaries fall inside.  A workgroup is one wave per KV head, so a block's
// bytes are read by one CU at the same time and each byte leaves HBM once.  A run of
// tiles that covers a whole sequence writes the output row directly; otherwise it
// stores an fp32 partial state (o, m, l) in slot w + seq (unique along the staircase of
// (workgroup, sequence) pairs) and the reduce kernel merges the slots of a sequence
// with the log-sum-exp algebra.  Nothing is synchronised on the host and nothing is
// allocated: the partials live in the caller's workspace.
//
// The fixed-partition entry point (512-token partitions, locally normalised partials)
// reuses the same tile code with the reference's (partition, sequence) grid.
#include <type_traits>

#include "kvq_attn_core.cuh"

namespace kvq {


__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int u = __shfl_up(v, o, kWave);
    if (lane >= o) v += u;
  }
  return v;
}

// Starting on a sequence (query row, first tile with nothing in flight, storing the state of the
// one before) costs a workgroup about as long as one tile takes; the work line that is cut into
// equal shares therefore charges every sequence this many units before its tiles.  Measured on
// MI355X at batch 64, 1k..8k tokens: workgroups whose share crossed a sequence boundary ran 2.9 us
// (one tile time) longer than the others and were the last to finish; with the charge they get
// one tile less.
constexpr int kSetupUnits = 1;

// Tiles of a decode sequence: those that hold a token of the row's window,
// [window_first / 32, ceil(len / 32)).  0 for prefill sequences and empty ones.
__device__ __forceinline__ int decode_tiles(const int32_t* seq_lens, const int32_t* cu, int s, int num_seqs,
                                            int window) {
  // no data-dependent branches: the loads of a lane (and of the lanes' next chunks) all go out
  // together; a lane past the last sequence rereads the last one and its result is dropped
  const int sc = s < num_seqs ? s : num_seqs - 1;
  const int len = seq_lens[sc];
  int q_len = 1;
  if (cu != nullptr) q_len = cu[sc + 1] - cu[sc];
  const int n = (len + kTile - 1) / kTile - window_first(len, window) / kTile;
  return (s < num_seqs && q_len == 1 && len > 0) ? n : 0;
}

// Units a sequence takes on the work line: its setup charge, then one unit per tile.
__device__ __forceinline__ int decode_units(const int32_t* seq_lens, const int32_t* cu, int s, int num_seqs,
                                            int window) {
  const int n = decode_tiles(seq_lens, cu, s, num_seqs, window);
  return n > 0 ? n + kSetupUnits : 0;
}

// The scans over the sequences work on chunks of 64 (one per lane).  Large batches take kScanBatch
// chunks per step so that their loads are in flight together (batch 512: 16 dependent round trips
// -> 4); a batch that fits one chunk keeps the single-chunk loop, which measured 3 us faster there.
constexpr int kScanBatch = 4;

// Total units of the work line.
template <int BATCH>
__device__ __forceinline__ int64_t scan_total(const StreamKArgs& a, int lane) {
  const int B = a.num_seqs;
  int64_t total = 0;
  for (int base = 0; base < B; base += kWave * BATCH) {
    int n[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j)
      n[j] = decode_units(a.seq_lens, a.cu_seqlens_q, base + kWave * j + lane, B, a.io.window);
#pragma unroll
    for (int j = 0; j < BATCH; ++j) total += __builtin_amdgcn_readlane(wave_incl_scan(n[j], lane), 63);
  }
  return total;
}

// The sequence that holds unit `lo` and the index of its first unit.
template <int BATCH>
__device__ __forceinline__ void scan_locate(const StreamKArgs& a, int lane, int64_t lo, int& seq, int64_t& seq_start) {
  const int B = a.num_seqs;
  int64_t cum = 0;
  bool found = false;
  for (int base = 0; base < B && !found; base += kWave * BATCH) {
    int nn[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j)
      nn[j] = decode_units(a.seq_lens, a.cu_seqlens_q, base + kWave * j + lane, B, a.io.window);
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int n = nn[j];
      const int incl = wave_incl_scan(n, lane);
      const int64_t first = cum + incl - n, last = cum + incl;
      const uint64_t hit = __builtin_amdgcn_ballot_w64(n > 0 && first <= lo && lo < last);
      if (hit != 0 && !found) {
        const int src = __builtin_ctzll(hit);
        seq = base + kWave * j + src;
        seq_start = cum + __builtin_amdgcn_readlane(incl - n, src);
        found = true;
      }
      cum += __builtin_amdgcn_readlane(incl, 63);
    }
  }
}

// Total units and the first unit of sequence `seq`; n_first = the units of the first BATCH chunks,
// loaded by the caller ahead of its first branch.
template <int BATCH>
__device__ __forceinline__ void scan_start(const StreamKArgs& a, int lane, int seq, const int (&n_first)[BATCH],
                                           int64_t& total, int64_t& start) {
  const int B = a.num_seqs;
  total = 0;
  start = 0;
  for (int base = 0; base < B; base += kWave * BATCH) {
    int nn[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j)
      nn[j] = base == 0 ? n_first[j] : decode_units(a.seq_lens, a.cu_seqlens_q, base + kWave * j + lane, B, a.io.window);
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int n = nn[j], b0 = base + kWave * j;
      const int incl = wave_incl_scan(n, lane);
      if (seq >= b0 && seq < b0 + kWave) start = total + __builtin_amdgcn_readlane(incl - n, seq - b0);
      total += __builtin_amdgcn_readlane(incl, 63);
    }
  }
}

__device__ __forceinline__ int64_t wg_tile_begin(int w, int64_t total, int num_wg) {
  return ((int64_t)w * total) / num_wg;
}

// Workgroups that take a share of a line of `total` units: all that were launched, unless the line
// is so short that a share would fall below kMinUnitsPerWg -- a small batch is then spread over
// fewer workgroups, so that a sequence is not cut into dozens of one-tile partial states for the
// reduce to merge.  Measured at batch 4 x 512 tokens (main + reduce kernel): 15.6 us with shares of
// at least 2 units, 18.3 us with 4 (a tile at a time per wave: about 4 us per tile at low load).
constexpr int kMinUnitsPerWg = 2;
__device__ __forceinline__ int active_workgroups(int64_t total, int num_wg) {
  const int64_t want = total / kMinUnitsPerWg;
  return want >= num_wg ? num_wg : (want < 1 ? 1 : (int)want);
}

template <int D, int QDT, int ODT, int WPW, bool CAP>
__global__ __launch_bounds__(WPW * 64) void paged_decode_streamk_kernel(StreamKArgs a) {
  using DTile = DecodeTile<D, QDT, ODT>;
  __shared__ __align__(16) uint8_t lds[WPW][DTile::LDS_WAVE];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int hkv = __builtin_amdgcn_readfirstlane(blockIdx.y * WPW + wave);
  if (hkv >= a.io.g.num_kv_heads) return;  // a finished wave no longer counts at the tile loop's barriers
  const int w = blockIdx.x;
  const int B = a.num_seqs;

  // total units of the work line (each wave redoes this tiny scan; no LDS, no barrier)
  const bool one_chunk = B <= kWave;
  const int64_t total = one_chunk ? scan_total<1>(a, lane) : scan_total<kScanBatch>(a, lane);
  const int num_wg = active_workgroups(total, a.num_wg);
  if (w >= num_wg) return;
  const int64_t lo = wg_tile_begin(w, total, num_wg);
  const int64_t hi = wg_tile_begin(w + 1, total, num_wg);
  if (lo >= hi) return;

  // locate the sequence holding unit `lo`
  int seq = 0;
  int64_t seq_start = 0;  // global index of the sequence's first unit
  if (one_chunk) scan_locate<1>(a, lane, lo, seq, seq_start);
  else scan_locate<kScanBatch>(a, lane, lo, seq, seq_start);
  seq = __builtin_amdgcn_readfirstlane(seq);

  int64_t pos = lo;
  while (pos < hi && seq < B) {
    const int units = __builtin_amdgcn_readfirstlane(decode_units(a.seq_lens, a.cu_seqlens_q, seq, B, a.io.window));
    if (units == 0) {
      ++seq;
      continue;
    }
    const int ntiles = units - kSetupUnits;
    const int len = __builtin_amdgcn_readfirstlane(a.seq_lens[seq]);
    const int64_t row = a.cu_seqlens_q ? (int64_t)a.cu_seqlens_q[seq] : (int64_t)seq;
    const int first = window_first(len, a.io.window);  // tokens before it are outside the window
    const int t0 = first / kTile;                      // the sequence's tile line starts at this tile
    // units [pos, min(hi, end of the sequence)) of the line; the first kSetupUnits of a sequence
    // stand for no tile
    const int u_begin = (int)(pos - seq_start);
    const int64_t rem = hi - seq_start;
    const int u_end = rem < units ? (int)rem : units;
    const int t_begin = __builtin_amdgcn_readfirstlane(t0 + (u_begin > kSetupUnits ? u_begin - kSetupUnits : 0));
    const int t_end = __builtin_amdgcn_readfirstlane(t0 + u_end - kSetupUnits);
    if (t_begin < t_end) {  // else: this share ends inside the setup charge and holds no tile
      typename DTile::State st;
      DTile::template run<CAP>(a.io, seq, row, len, first, t_begin, t_end, hkv, lane, lds[wave], st);
      if (t_begin == t0 && t_end == t0 + ntiles) {
        DTile::emit_final(a.io, row, hkv, lane, st);
      } else {
        DTile::emit_partial(a.io, a.part_o, a.part_ml, (int64_t)w + seq, hkv, lane, st);
      }
    }
    pos = seq_start + u_end;
    seq_start += units;
    ++seq;
  }
}

// Merge the partial states of every decode sequence that more than one workgroup touched.
// grid (num_seqs, ceil(Hq / 4)), 4 waves, one wave per q head, lane owns D/64 dims.
template <int D, int ODT>
__global__ __launch_bounds__(256) void paged_decode_streamk_reduce_kernel(StreamKArgs a) {
  constexpr int V = D / 64;
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int seq = blockIdx.x;
  const int B = a.num_seqs;
  if (head >= a.io.num_q_heads) return;
  // all the loads that depend on nothing but the arguments go out together, before the first branch
  const int q0 = a.cu_seqlens_q ? a.cu_seqlens_q[seq] : seq;
  const int q1 = a.cu_seqlens_q ? a.cu_seqlens_q[seq + 1] : seq + 1;
  const int len = a.seq_lens[seq];
  const bool one_chunk = B <= kWave;
  int n_first[kScanBatch];  // first sequences of the scan
  n_first[0] = decode_units(a.seq_lens, a.cu_seqlens_q, lane, B, a.io.window);
  if (!one_chunk) {
#pragma unroll
    for (int j = 1; j < kScanBatch; ++j)
      n_first[j] = decode_units(a.seq_lens, a.cu_seqlens_q, kWave * j + lane, B, a.io.window);
  }
  if (q1 - q0 != 1) return;
  const int64_t row = q0;
  const int ntiles = len > 0 ? (len + kTile - 1) / kTile - window_first(len, a.io.window) / kTile : 0;
  if (ntiles == 0) {  // empty sequence: defined output (zeros, lse = -inf)
    for (int i = 0; i < V; ++i)
      store_act<ODT>(a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + i, 0.f);
    if (a.io.lse != nullptr && lane == 0) a.io.lse[row * a.io.num_q_heads + head] = -INFINITY;
    return;
  }
  int64_t total, start;
  if (one_chunk) {
    const int n1[1] = {n_first[0]};
    scan_start<1>(a, lane, seq, n1, total, start);
  } else {
    scan_start<kScanBatch>(a, lane, seq, n_first, total, start);
  }
  const int P = active_workgroups(total, a.num_wg);
  // workgroup holding unit x: the largest w with floor(w*T/P) <= x; the sequence's tiles are units
  // start + kSetupUnits .. start + kSetupUnits + ntiles - 1
  const int w_first = (int)(((start + kSetupUnits + 1) * P - 1) / total);
  const int w_last = (int)(((start + kSetupUnits + ntiles) * P - 1) / total);
  if (w_first == w_last) return;  // written directly by the main kernel

  // pass 1: every lane takes one workgroup's (m, l); the wave agrees on the max and the weights
  // pass 2: weighted sum of the partial outputs, all loads independent of each other
  float m = -INFINITY, l = 0.f, acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = 0.f;
  // Few slots (the usual case: a sequence spans a handful of workgroups): the (m, l) pairs and ALL
  // the partial outputs are requested in one go, so the kernel pays one memory round trip for them
  // instead of two.
  constexpr int kFew = 32;
  // N = how many slots the one-round-trip path requests (all of them unconditionally: slots past the
  // last reread the last one), in three sizes so that a short span does not fetch 32 rows
  auto merge_few = [&](auto n_tag) __attribute__((always_inline)) {
    constexpr int N = decltype(n_tag)::value;
    const int w = w_first + lane;
    const bool live = w <= w_last && wg_tile_begin(w, total, P) < wg_tile_begin(w + 1, total, P);
    const int64_t slot = (int64_t)min(w, w_last) + seq;
    const uint32_t keep = live ? 0xffffffffu : 0u;
    const float mj_raw = a.part_ml[(slot * a.io.num_q_heads + head) * 2 + 0];
    const float lj_raw = a.part_ml[(slot * a.io.num_q_heads + head) * 2 + 1];
    float po[N][V];
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const int64_t sk = (int64_t)min(w_first + k, w_last) + seq;
      const float* p = a.part_o + (sk * a.io.num_q_heads + head) * (int64_t)D + lane * V;
#pragma unroll
      for (int i = 0; i < V; ++i) po[k][i] = p[i];
    }
    const float mj = live ? as_f32(as_u32(mj_raw) & keep) : -INFINITY;
    const float lj = as_f32(as_u32(lj_raw) & keep);
    m = wave_max(mj);
    const float ej = live ? __builtin_amdgcn_exp2f(mj - m) : 0.f;
    l = wave_sum(lj * ej);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float wk = __shfl(ej, k, kWave);  // 0 for slots past the last and for empty ones
      const uint32_t kk = wk != 0.f ? 0xffffffffu : 0u;
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] += as_f32(as_u32(po[k][i]) & kk) * wk;
    }
  };
  const int span = w_last - w_first + 1;
  if (span <= 4) {
    merge_few(std::integral_constant<int, 4>{});
  } else if (span <= 12) {
    merge_few(std::integral_constant<int, 12>{});
  } else if (span <= kFew) {
    merge_few(std::integral_constant<int, kFew>{});
  } else
  for (int wb = w_first; wb <= w_last; wb += kWave) {
    const int w = wb + lane;
    const bool live = w <= w_last && wg_tile_begin(w, total, P) < wg_tile_begin(w + 1, total, P);
    // loads are unconditional (clamped to the sequence's last workgroup) and what they return is
    // removed with a bit mask where the slot holds nothing: a select on the loaded value becomes a
    // branch around the load, and the loads of successive slots would then run one after another
    const int64_t slot = (int64_t)min(w, w_last) + seq;
    const uint32_t keep = live ? 0xffffffffu : 0u;
    const float mj_raw = a.part_ml[(slot * a.io.num_q_heads + head) * 2 + 0];
    const float lj_raw = a.part_ml[(slot * a.io.num_q_heads + head) * 2 + 1];
    const float mj = live ? as_f32(as_u32(mj_raw) & keep) : -INFINITY;
    const float lj = as_f32(as_u32(lj_raw) & keep);
    const float m_new = fmaxf(m, wave_max(mj));
    const float ca = __builtin_amdgcn_exp2f(m - m_new);  // first chunk: exp2(-inf) = 0
    const float ej = live ? __builtin_amdgcn_exp2f(mj - m_new) : 0.f;
    l = l * ca + wave_sum(lj * ej);
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] *= ca;
    m = m_new;
    // sixteen slots per round trip: the loads of a batch are unconditional (slots past the last reread
    // the last one, weight 0) so that they all leave before the first is used
    const int count = min(kWave, w_last - wb + 1);
    for (int k0 = 0; k0 < count; k0 += 16) {
      float pv[16][V];
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int64_t sk = (int64_t)min(wb + k0 + k, w_last) + seq;
        const float* po = a.part_o + (sk * a.io.num_q_heads + head) * (int64_t)D + lane * V;
#pragma unroll
        for (int i = 0; i < V; ++i) pv[k][i] = po[i];
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const float wk = (k0 + k) < count ? __shfl(ej, (k0 + k) & (kWave - 1), kWave) : 0.f;  // unnormalised sums
        const uint32_t kk = wk != 0.f ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] += as_f32(as_u32(pv[k][i]) & kk) * wk;
      }
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < V; ++i)
    store_act<ODT>(a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + i, acc[i] * inv);
  if (a.io.lse != nullptr && lane == 0)
    a.io.lse[row * a.io.num_q_heads + head] = (m + __builtin_amdgcn_logf(l)) * kLn2;
}

// ---- fixed partitions: grid (max_parts, num_seqs, head groups) --------------------------
struct V2Args {
  AttnIO io;
  const int32_t* seq_lens;
  float* tmp_out;
  float* max_logits;
  float* exp_sums;
  int partition_tiles;  // partition_size / 32
  int max_parts;
};

template <int D, int QDT, int WPW>
__global__ __launch_bounds__(WPW * 64) void paged_decode_v2_kernel(V2Args a) {
  using DTile = DecodeTile<D, QDT, KVQ_F32>;
  __shared__ __align__(16) uint8_t lds[WPW][DTile::LDS_WAVE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int hkv = __builtin_amdgcn_readfirstlane(blockIdx.z * WPW + wave);
  if (hkv >= a.io.g.num_kv_heads) return;
  const int part = blockIdx.x, seq = blockIdx.y;
  const int len = a.seq_lens[seq];
  const int ntiles = len > 0 ? (len + kTile - 1) / kTile : 0;
  const int t_begin = part * a.partition_tiles;
  if (t_begin >= ntiles) return;
  const int t_end = min(ntiles, t_begin + a.partition_tiles);
  typename DTile::State st;
  DTile::template run<false>(a.io, seq, seq, len, 0, t_begin, t_end, hkv, lane, lds[wave], st);
  DTile::emit_v2(a.io, a.tmp_out, a.max_logits, a.exp_sums, seq, part, a.max_parts, hkv, lane, st);
}

// out = sum_j w_j tmp_out_j / sum_j w_j, w_j = exp_sums_j * exp(max_logits_j - max).
// grid (num_seqs, ceil(Hq/4)), one wave per q head.
template <int ODT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(void* out, float* lse, const float* exp_sums,
                                                            const float* max_logits, const float* tmp_out,
                                                            const int32_t* seq_lens, int num_q_heads, int D,
                                                            int partition_size, int max_parts) {
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int seq = blockIdx.x;
  if (head >= num_q_heads) return;
  const int len = seq_lens[seq];
  int parts = len > 0 ? (len + partition_size - 1) / partition_size : 0;
  parts = parts < max_parts ? parts : max_parts;
  const int64_t base = ((int64_t)seq * num_q_heads + head) * max_parts;
  const int64_t obase = ((int64_t)seq * num_q_heads + head) * D;
  if (parts == 0) {
    for (int d = lane; d < D; d += kWave) store_act<ODT>(out, obase + d, 0.f);
    if (lse != nullptr && lane == 0) lse[(int64_t)seq * num_q_heads + head] = -INFINITY;
    return;
  }
  float m = -INFINITY;
  for (int j = lane; j < parts; j += kWave) m = fmaxf(m, max_logits[base + j]);
  m = wave_max(m);
  float denom = 0.f;
  for (int j = lane; j < parts; j += kWave) denom += exp_sums[base + j] * __expf(max_logits[base + j] - m);
  denom = wave_sum(denom);
  const float inv = 1.0f / denom;
  for (int d = lane; d < D; d += kWave) {
    float acc = 0.f;
    for (int j = 0; j < parts; ++j)
      acc += tmp_out[(base + j) * D + d] * (exp_sums[base + j] * __expf(max_logits[base + j] - m));
    store_act<ODT>(out, obase + d, acc * inv);
  }
  if (lse != nullptr && lane == 0) lse[(int64_t)seq * num_q_heads + head] = m + __logf(denom);
}

// ---- host side ---------------------------------------------------------------------------

static int waves_per_wg(int num_kv_heads) {
  if (num_kv_heads >= 8) return 8;
  if (num_kv_heads >= 4) return 4;
  if (num_kv_heads >= 2) return 2;
  return 1;
}

// Resident workgroups the stream-K launch uses: every CU holds 8 decode waves.
static int streamk_num_wg(int num_kv_heads) {
  const int wpw = waves_per_wg(num_kv_heads);
  return num_cus() * (8 / wpw);
}

static int validate_common(const char* op, const void* q, const void* cache, const kvq_cache_geom* geom,
                           const int32_t* block_table, const int32_t* seq_lens, int num_seqs, int num_q_heads) {
  KVQ_REQUIRE(geom != nullptr, "%s: geom is NULL", op);
  KVQ_REQUIRE(q && cache && block_table && seq_lens, "%s: NULL pointer", op);
  KVQ_REQUIRE(num_seqs > 0 && num_q_heads > 0, "%s: num_seqs and num_q_heads must be positive", op);
  const kvq_cache_geom& g = *geom;
  KVQ_REQUIRE(g.num_kv_heads > 0 && num_q_heads % g.num_kv_heads == 0,
              "%s: num_q_heads %d is not a multiple of num_kv_heads %d", op, num_q_heads, g.num_kv_heads);
  KVQ_REQUIRE(num_q_heads / g.num_kv_heads <= 16, "%s: more than 16 q heads per kv head is not supported", op);
  KVQ_REQUIRE(g.head_size == 64 || g.head_size == 128 || g.head_size == 256,
              "%s: head_size %d not supported (64, 128, 256)", op, g.head_size);
  KVQ_REQUIRE(g.block_size > 0 && g.block_size % 16 == 0, "%s: block_size %d must be a multiple of 16", op,
              g.block_size);
  KVQ_REQUIRE((g.k_off | g.v_off | g.ks_off | g.vs_off | g.stride_block | g.stride_slot | g.stride_head) % 4 == 0 &&
                  ((uintptr_t)cache % 4) == 0,
              "%s: cache offsets/strides must be 4-byte aligned", op);
  KVQ_REQUIRE(g.ks_off - g.k_off == g.head_size && g.v_off - g.k_off == g.head_size + 4 &&
                  g.vs_off - g.k_off == 2 * g.head_size + 4,
              "%s: a cache record must be [K codes | K scale | V codes | V scale]", op);
  KVQ_REQUIRE(g.stride_slot > 0 && g.stride_slot <= 0x7fffffff / 64, "%s: stride_slot out of range", op);
  return KVQ_OK;
}

template <int D, int QDT, int ODT>
static int launch_streamk(const StreamKArgs& a, hipStream_t s) {
  const int hkv = a.io.g.num_kv_heads;
  const int wpw = waves_per_wg(hkv);
  dim3 grid(a.num_wg, (hkv + wpw - 1) / wpw);
#define KVQ_SK(W, C) \
  hipLaunchKernelGGL((paged_decode_streamk_kernel<D, QDT, ODT, W, C>), grid, dim3(W * 64), 0, s, a)
  if (a.io.cap_c != 0.f) {
    switch (wpw) {
      case 8: KVQ_SK(8, true); break;
      case 4: KVQ_SK(4, true); break;
      case 2: KVQ_SK(2, true); break;
      default: KVQ_SK(1, true); break;
    }
  } else {
    switch (wpw) {
      case 8: KVQ_SK(8, false); break;
      case 4: KVQ_SK(4, false); break;
      case 2: KVQ_SK(2, false); break;
      default: KVQ_SK(1, false); break;
    }
  }
#undef KVQ_SK
  int rc = check_hip(hipGetLastError(), "paged_attn_int8 decode launch");
  if (rc) return rc;
  dim3 rgrid(a.num_seqs, (a.io.num_q_heads + 3) / 4);
  hipLaunchKernelGGL((paged_decode_streamk_reduce_kernel<D, ODT>), rgrid, dim3(256), 0, s, a);
  return check_hip(hipGetLastError(), "paged_attn_int8 reduce launch");
}

template <int D, int QDT>
static int launch_streamk_o(const StreamKArgs& a, int out_dtype, hipStream_t s) {
  switch (out_dtype) {
    case KVQ_F32: return launch_streamk<D, QDT, KVQ_F32>(a, s);
    case KVQ_BF16: return launch_streamk<D, QDT, KVQ_BF16>(a, s);
    case KVQ_F16: return launch_streamk<D, QDT, KVQ_F16>(a, s);
  }
  return fail(KVQ_EINVAL, "paged_attn_int8: unknown out_dtype %d", out_dtype);
}

template <int D>
static int launch_streamk_q(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s) {
  switch (q_dtype) {
    case KVQ_F32: return launch_streamk_o<D, KVQ_F32>(a, out_dtype, s);
    case KVQ_BF16: return launch_streamk_o<D, KVQ_BF16>(a, out_dtype, s);
    case KVQ_F16: return launch_streamk_o<D, KVQ_F16>(a, out_dtype, s);
  }
  return fail(KVQ_EINVAL, "paged_attn_int8: unknown q_dtype %d", q_dtype);
}

int launch_decode_streamk(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s) {
  switch (a.io.g.head_size) {
    case 64: return launch_streamk_q<64>(a, q_dtype, out_dtype, s);
    case 128: return launch_streamk_q<128>(a, q_dtype, out_dtype, s);
    case 256: return launch_streamk_q<256>(a, q_dtype, out_dtype, s);
  }
  return fail(KVQ_EINVAL, "paged_attn_int8: head_size %d not supported", a.io.g.head_size);
}

template <int D, int QDT>
static int launch_v2(const V2Args& a, int num_seqs, hipStream_t s) {
  const int hkv = a.io.g.num_kv_heads;
  const int wpw = waves_per_wg(hkv);
  dim3 grid(a.max_parts, num_seqs, (hkv + wpw - 1) / wpw);
  switch (wpw) {
    case 8: hipLaunchKernelGGL((paged_decode_v2_kernel<D, QDT, 8>), grid, dim3(512), 0, s, a); break;
    case 4: hipLaunchKernelGGL((paged_decode_v2_kernel<D, QDT, 4>), grid, dim3(256), 0, s, a); break;
    case 2: hipLaunchKernelGGL((paged_decode_v2_kernel<D, QDT, 2>), grid, dim3(128), 0, s, a); break;
    default: hipLaunchKernelGGL((paged_decode_v2_kernel<D, QDT, 1>), grid, dim3(64), 0, s, a); break;
  }
  return check_hip(hipGetLastError(), "paged_attn_v2_int8 launch");
}

template <int D>
static int launch_v2_q(const V2Args& a, int num_seqs, int q_dtype, hipStream_t s) {
  switch (q_dtype) {
    case KVQ_F32: return launch_v2<D, KVQ_F32>(a, num_seqs, s);
    case KVQ_BF16: return launch_v2<D, KVQ_BF16>(a, num_seqs, s);
    case KVQ_F16: return launch_v2<D, KVQ_F16>(a, num_seqs, s);
  }
  return fail(KVQ_EINVAL, "paged_attn_v2_int8: unknown q_dtype %d", q_dtype);
}

static int launch_reduce(void* out, int out_dtype, float* lse, const float* exp_sums, const float* max_logits,
                         const float* tmp_out, const int32_t* seq_lens, int num_seqs, int num_q_heads, int D,
                         int partition_size, int max_parts, hipStream_t s) {
  dim3 grid(num_seqs, (num_q_heads + 3) / 4);
#define KVQ_RED(T)                                                                                        \
  hipLaunchKernelGGL((splitk_reduce_kernel<T>), grid, dim3(256), 0, s, out, lse, exp_sums, max_logits, \
                     tmp_out, seq_lens, num_q_heads, D, partition_size, max_parts)
  switch (out_dtype) {
    case KVQ_F32: KVQ_RED(KVQ_F32); break;
    case KVQ_BF16: KVQ_RED(KVQ_BF16); break;
    case KVQ_F16: KVQ_RED(KVQ_F16); break;
    default: return fail(KVQ_EINVAL, "splitk_reduce: unknown out_dtype %d", out_dtype);
  }
#undef KVQ_RED
  return check_hip(hipGetLastError(), "splitk_reduce launch");
}

// Workspace layout of the stream-K partials.
size_t streamk_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size, int num_wg) {
  const size_t slots = (size_t)num_wg + (size_t)max_num_seqs;
  return slots * (size_t)num_q_heads * ((size_t)head_size + 2) * sizeof(float);
}

int decode_streamk_num_wg(int num_kv_heads) { return streamk_num_wg(num_kv_heads); }

}  // namespace kvq

extern "C" {

size_t kvq_paged_attn_workspace_bytes(int max_num_seqs, int num_q_heads, int head_size) {
  if (max_num_seqs <= 0 || num_q_heads <= 0 || head_size <= 0) return 0;
  // the smallest workgroup (one wave) gives the largest resident count
  return kvq::streamk_workspace_bytes(max_num_seqs, num_q_heads, head_size, kvq::num_cus() * 8);
}

int kvq_paged_attn_v2_int8(void* out, int out_dtype, float* exp_sums, float* max_logits, float* tmp_out,
                           const void* q, int q_dtype, int64_t q_stride_t, int64_t q_stride_h,
                           const void* cache, const kvq_cache_geom* geom, const int32_t* block_table,
                           int64_t bt_stride, const int32_t* seq_lens, int num_seqs, int num_q_heads,
                           float scale, int partition_size, int max_num_partitions, kvq_stream_t stream) {
  using namespace kvq;
  int rc = validate_common("paged_attn_v2_int8", q, cache, geom, block_table, seq_lens, num_seqs, num_q_heads);
  if (rc) return rc;
  KVQ_REQUIRE(out && exp_sums && max_logits && tmp_out, "paged_attn_v2_int8: NULL output pointer");
  KVQ_REQUIRE(partition_size > 0 && partition_size % kTile == 0,
              "paged_attn_v2_int8: partition_size %d must be a positive multiple of %d", partition_size, kTile);
  KVQ_REQUIRE(max_num_partitions > 0 && max_num_partitions <= 65535,
              "paged_attn_v2_int8: max_num_partitions %d out of range", max_num_partitions);
  KVQ_REQUIRE(num_seqs <= 65535, "paged_attn_v2_int8: at most 65535 sequences");
  V2Args a{};
  a.io.q = q;
  a.io.q_stride_t = q_stride_t;
  a.io.q_stride_h = q_stride_h;
  a.io.cache = static_cast<const uint8_t*>(cache);
  a.io.g = *geom;
  a.io.block_table = block_table;
  a.io.bt_stride = bt_stride;
  a.io.num_q_heads = num_q_heads;
  a.io.group = num_q_heads / geom->num_kv_heads;
  a.io.scale_log2 = scale * kLog2e;
  a.io.bs_magic = (uint32_t)((0x100000000ull + (uint64_t)geom->block_size - 1) / (uint64_t)geom->block_size);
  a.seq_lens = seq_lens;
  a.tmp_out = tmp_out;
  a.max_logits = max_logits;
  a.exp_sums = exp_sums;
  a.partition_tiles = partition_size / kTile;
  a.max_parts = max_num_partitions;
  hipStream_t s = as_stream(stream);
  switch (geom->head_size) {
    case 64: rc = launch_v2_q<64>(a, num_seqs, q_dtype, s); break;
    case 128: rc = launch_v2_q<128>(a, num_seqs, q_dtype, s); break;
    default: rc = launch_v2_q<256>(a, num_seqs, q_dtype, s); break;
  }
  if (rc) return rc;
  return launch_reduce(out, out_dtype, nullptr, exp_sums, max_logits, tmp_out, seq_lens, num_seqs, num_q_heads,
                       geom->head_size, partition_size, max_num_partitions, s);
}

int kvq_splitk_reduce(void* out, int out_dtype, float* lse, const float* exp_sums, const float* max_logits,
                      const float* tmp_out, const int32_t* seq_lens, int num_seqs, int num_q_heads,
                      int head_size, int partition_size, int max_num_partitions, kvq_stream_t stream) {
  using namespace kvq;
  KVQ_REQUIRE(out && exp_sums && max_logits && tmp_out && seq_lens, "splitk_reduce: NULL pointer");
  KVQ_REQUIRE(num_seqs > 0 && num_q_heads > 0 && head_size > 0 && partition_size > 0 && max_num_partitions > 0,
              "splitk_reduce: sizes must be positive");
  return launch_reduce(out, out_dtype, lse, exp_sums, max_logits, tmp_out, seq_lens, num_seqs, num_q_heads,
                       head_size, partition_size, max_num_partitions, as_stream(stream));
}

}  // extern "C"
