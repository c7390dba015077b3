// Device code and launch templates of the paged decode kernels, instantiated once per head size in
// kvq_paged_decode_d64.hip / _d128.hip / _d256.hip (one translation unit each, so they compile in parallel).
#pragma once

#include <type_traits>

#include "kvq_attn_core.cuh"

namespace kvq {

int heads_per_wg(int num_kv_heads);



__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int u = __shfl_up(v, o, kWave);
    if (lane >= o) v += u;
  }
  return v;
}

// Starting on a sequence (query row, first tile with nothing in flight, folding and storing the state of the
// one before) costs a workgroup 4 - 5 us, whatever the number of kv heads it serves; the work line that is cut into
// equal shares therefore charges every sequence StreamKArgs::setup_units units before its tiles.  A unit is a
// tile of the workgroup's run, and the 8 / HPW waves of a head take a run's tiles in turn, so a unit lasts
// 2.9 us / (8 / HPW) and the charge grows with the waves per head (setup_units_for).  Measured on MI355X at batch 64,
// 1k..8k tokens: with eight kv heads and no charge, workgroups whose share crossed a sequence boundary ran 2.9 us
// (one tile time) longer than the others and were the last to finish; with one kv head and a charge of one unit
// they ran 23.0 us against 18.2 us and the launch waited for them.
constexpr int setup_units_for(int waves_per_head) { return waves_per_head == 1 ? 1 : 3 * waves_per_head / 2; }

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

// Batch-invariant cutting (StreamKArgs::fixed_spans): a sequence is cut at places that depend on nothing but its
// own length -- into at most kFixedSpans spans of equal size, none shorter than kMinSpanTiles tiles.  The spans of
// all decode sequences form one line (a unit per span) that is cut into equal shares like the balanced line, so
// WHICH workgroup computes a span depends on the batch, but not what it computes: the states of a sequence's
// spans lie in slots seq * kFixedSpans + span and are merged in span order, so a row's bits are the same
// whatever else the batch holds and however many workgroups the device runs.
constexpr int kFixedSpans = 32;
constexpr int kMinSpanTiles = 8;
__device__ __forceinline__ int fixed_span_tiles(int ntiles) {
  const int per = (ntiles + kFixedSpans - 1) / kFixedSpans;
  return per > kMinSpanTiles ? per : kMinSpanTiles;
}
__device__ __forceinline__ int fixed_span_count(int ntiles) {
  const int per = fixed_span_tiles(ntiles);
  return (ntiles + per - 1) / per;   // 0 for no tiles
}

// Units a sequence takes on the work line: its setup charge, then one unit per tile.
__device__ __forceinline__ int decode_units(const int32_t* seq_lens, const int32_t* cu, int s, int num_seqs,
                                            int window, int setup) {
  const int n = decode_tiles(seq_lens, cu, s, num_seqs, window);
  return n > 0 ? n + setup : 0;
}
// Units of a sequence on the line the launch cuts: tiles + setup charge, or (FIXED) its spans.
template <bool FIXED>
__device__ __forceinline__ int line_units(const int32_t* seq_lens, const int32_t* cu, int s, int num_seqs, int window,
                                          int setup) {
  if constexpr (FIXED) return fixed_span_count(decode_tiles(seq_lens, cu, s, num_seqs, window));
  else return decode_units(seq_lens, cu, s, num_seqs, window, setup);
}

// The scans over the sequences work on chunks of 64 (one per lane).  Large batches take kScanBatch
// chunks per step so that their loads are in flight together (batch 512: 16 dependent round trips
// -> 4); a batch that fits one chunk keeps the single-chunk loop, which measured 3 us faster there.
constexpr int kScanBatch = 4;

// Total units of the work line.
template <int BATCH, bool FIXED = false>
__device__ __forceinline__ int64_t scan_total(const StreamKArgs& a, int lane) {
  const int B = a.num_seqs;
  int64_t total = 0;
  for (int base = 0; base < B; base += kWave * BATCH) {
    int n[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j)
      n[j] = line_units<FIXED>(a.seq_lens, a.cu_seqlens_q, base + kWave * j + lane, B, a.io.window, a.setup_units);
#pragma unroll
    for (int j = 0; j < BATCH; ++j) total += __builtin_amdgcn_readlane(wave_incl_scan(n[j], lane), 63);
  }
  return total;
}

// The sequence that holds unit `lo` and the index of its first unit.
template <int BATCH, bool FIXED = false>
__device__ __forceinline__ void scan_locate(const StreamKArgs& a, int lane, int64_t lo, int& seq, int64_t& seq_start) {
  const int B = a.num_seqs;
  int64_t cum = 0;
  bool found = false;
  for (int base = 0; base < B && !found; base += kWave * BATCH) {
    int nn[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j)
      nn[j] = line_units<FIXED>(a.seq_lens, a.cu_seqlens_q, base + kWave * j + lane, B, a.io.window, a.setup_units);
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

// HPW = kv heads per workgroup (1, 2, 4 or 8).  A workgroup always has eight waves: with fewer than
// eight kv heads the 8 / HPW waves of a head take the tiles of a run in turn and their states are
// folded together in LDS when the run ends, so a compute unit keeps eight tile streams in flight
// whatever the head count and a sequence is cut into no more partial states than with eight heads.
// FIXED: the batch-invariant cutting instead of the balanced one (a template argument, so that the balanced
// kernel carries none of it: as a run-time branch it cost the headline launch 0.6 us).
template <int D, int QDT, int HPW, bool CAP, int CODE, bool STREAM, bool FIXED = false>
__global__ __launch_bounds__(512) void paged_decode_streamk_kernel(StreamKArgs a) {
  using DTile = DecodeTile<D, QDT, kRuntimeDtype, CODE>;
  constexpr int NSUB = 8 / HPW;
  __shared__ __align__(16) uint8_t lds[8][DTile::LDS_WAVE];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int sub = wave % NSUB;
  const int hkv = __builtin_amdgcn_readfirstlane(blockIdx.y * HPW + wave / NSUB);
  if (hkv >= a.io.g.num_kv_heads) return;  // a finished wave no longer counts at the workgroup's barriers
  const int w = blockIdx.x;
  const int B = a.num_seqs;

  constexpr bool fixed = FIXED;

  // the balanced cutting: total units of the work line (each wave redoes this tiny scan; no LDS, no barrier)
  const bool one_chunk = B <= kWave;
  int64_t total = 0, lo = 0, hi = 0;
  int seq = 0;
  int64_t seq_start = 0;  // global index of the sequence's first unit
  {
    total = one_chunk ? scan_total<1, fixed>(a, lane) : scan_total<kScanBatch, fixed>(a, lane);
    // (the batch-invariant line is short -- a unit is a span of at least kMinSpanTiles tiles -- and is always shared
    // out over every workgroup there is a unit for)
    const int num_wg = fixed ? (total < a.num_wg ? (total < 1 ? 1 : (int)total) : a.num_wg) : active_workgroups(total, a.num_wg);
    if (w >= num_wg) return;
    lo = wg_tile_begin(w, total, num_wg);
    hi = wg_tile_begin(w + 1, total, num_wg);
    if (lo >= hi) {   // an empty work line: workgroup 0 still reports its length
      if (!fixed && w == 0 && blockIdx.y == 0 && wave == 0 && lane == 0) a.wg_info[0] = total;
      return;
    }
    // locate the sequence holding unit `lo`
    if (one_chunk) scan_locate<1, fixed>(a, lane, lo, seq, seq_start);
    else scan_locate<kScanBatch, fixed>(a, lane, lo, seq, seq_start);
    seq = __builtin_amdgcn_readfirstlane(seq);
  }
  // Where the share begins (the reduce kernel's key to the span): noted in the first round of the loop, stored
  // after the last.  A store ahead of the tile loads would sit before them in the wave's in-order memory
  // counter, and the first tile would wait for the store's acknowledgement (measured: 0.6 us per launch).
  int info_seq = -1;
  int64_t info_start = 0;

  // One run of tiles [t_begin, t_end) of sequence `cur` (ntiles tiles from tile t0 on), its state to `slot` unless
  // the run is the whole sequence.
  auto process = [&](int cur, int64_t cur_start, int64_t row, int len, int first, int t0, int ntiles, int t_begin,
                     int t_end, int64_t slot) __attribute__((always_inline)) {
    if (a.k_new != nullptr && t_end == t0 + ntiles) {   // uniform over the workgroup: the run holds the last tile
      const bool padding = a.new_slots != nullptr && a.new_slots[row] < 0;   // uniform: a scalar load
      if (sub == 0 && !padding) write_new_token<D>(a, cur, row, len, hkv, lane);
      // the record is in memory before any wave of the workgroup loads the tile that holds it
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if constexpr (NSUB > 1) lds_barrier();
    }
    typename DTile::State st;
    DTile::template run<CAP, STREAM>(a.io, cur, row, len, first, t_begin, t_end, hkv, lane, lds[wave], st, sub, NSUB);
    // the run holds the sequence's first tile: its place on the line, for the reduce kernel (behind the run's loads)
    if (!fixed && t_begin == t0 && blockIdx.y == 0 && wave == 0 && lane == 0) a.seq_first_unit[cur] = cur_start;
    if constexpr (NSUB > 1) {
      if (sub != 0) DTile::dump_state(st, lane, lds[wave]);
      lds_barrier();
      if (sub == 0) {
#pragma unroll
        for (int j = 1; j < NSUB; ++j)
          if (t_begin + j < t_end) DTile::fold_state(st, lane, lds[wave + j]);  // wave j owned a tile
      }
      lds_barrier();  // the windows may be overwritten by the next run
    }
    if (sub == 0) {
      if (t_begin == t0 && t_end == t0 + ntiles) {
        DTile::emit_final(a.io, row, hkv, lane, st);
      } else {
        DTile::emit_partial(a.io, a.part_o, a.part_ml, slot, hkv, lane, st);
      }
    }
  };

  // (batch-invariant cutting, one wave per kv head) `count` consecutive spans of one sequence as ONE run of tiles: the
  // stream goes on across the spans' edges, where DecodeTile::run stores and restarts the state, so a span's state
  // holds the same bits as if it had been computed alone -- without a query reload and a first tile that nothing
  // prefetched per span.
  auto process_spans = [&](int cur, int64_t row, int len, int first, int t0, int ntiles, int t_begin, int t_end, int per,
                           int span) __attribute__((always_inline)) {
    if (a.k_new != nullptr && t_end == t0 + ntiles) {   // uniform over the workgroup: the run holds the last tile
      const bool padding = a.new_slots != nullptr && a.new_slots[row] < 0;
      if (!padding) write_new_token<D>(a, cur, row, len, hkv, lane);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    typename DTile::State st;
    typename DTile::SpanEdges sp{a.part_o, a.part_ml, (int64_t)cur * kFixedSpans + span, per, per};
    DTile::template run<CAP, STREAM, true>(a.io, cur, row, len, first, t_begin, t_end, hkv, lane, lds[wave], st, 0, 1, &sp);
    DTile::emit_partial(a.io, a.part_o, a.part_ml, sp.slot, hkv, lane, st);
  };

  if constexpr (fixed) {
    // the spans [lo, hi) of the span line, sequence by sequence
    int64_t at = lo;
    while (at < hi && seq < B) {
      const int ntiles = __builtin_amdgcn_readfirstlane(decode_tiles(a.seq_lens, a.cu_seqlens_q, seq, B, a.io.window));
      const int spans = fixed_span_count(ntiles);
      const int span = (int)(at - seq_start);
      if (span >= spans) {   // also: a sequence without tiles
        seq_start += spans;
        ++seq;
        continue;
      }
      const int per = fixed_span_tiles(ntiles);
      const int len = __builtin_amdgcn_readfirstlane(a.seq_lens[seq]);
      const int64_t row = a.cu_seqlens_q ? (int64_t)a.cu_seqlens_q[seq] : (int64_t)seq;
      const int first = window_first(len, a.io.window);
      const int t0 = first / kTile;
      const int t_begin = t0 + span * per;
      if constexpr (NSUB == 1) {
        const int64_t rest = hi - at;
        const int count = rest < spans - span ? (int)rest : spans - span;   // the sequence's spans inside this share
        if (count > 1) {
          process_spans(seq, row, len, first, t0, ntiles, t_begin, min(t0 + ntiles, t_begin + count * per), per, span);
          at += count;
          continue;
        }
      }
      const int t_end = min(t0 + ntiles, t_begin + per);
      process(seq, 0, row, len, first, t0, ntiles, t_begin, t_end, (int64_t)seq * kFixedSpans + span);
      ++at;
    }
    return;
  }

  int64_t pos = lo;
  while (pos < hi && seq < B) {
    const int units = __builtin_amdgcn_readfirstlane(decode_units(a.seq_lens, a.cu_seqlens_q, seq, B, a.io.window, a.setup_units));
    if (units == 0) {
      ++seq;
      continue;
    }
    const int setup = a.setup_units;
    const int ntiles = units - setup;
    const int len = __builtin_amdgcn_readfirstlane(a.seq_lens[seq]);
    const int64_t row = a.cu_seqlens_q ? (int64_t)a.cu_seqlens_q[seq] : (int64_t)seq;
    if (info_seq < 0) {
      info_seq = seq;
      info_start = seq_start;
    }
    const int first = window_first(len, a.io.window);  // tokens before it are outside the window
    const int t0 = first / kTile;                      // the sequence's tile line starts at this tile
    // units [pos, min(hi, end of the sequence)) of the line; the first setup_units of a sequence
    // stand for no tile
    const int u_begin = (int)(pos - seq_start);
    const int64_t rem = hi - seq_start;
    const int u_end = rem < units ? (int)rem : units;
    const int t_begin = __builtin_amdgcn_readfirstlane(t0 + (u_begin > setup ? u_begin - setup : 0));
    const int t_end = __builtin_amdgcn_readfirstlane(t0 + u_end - setup);
    if (t_begin < t_end)  // else: this share ends inside the setup charge and holds no tile
      process(seq, seq_start, row, len, first, t0, ntiles, t_begin, t_end, (int64_t)w + seq);
    pos = seq_start + u_end;
    seq_start += units;
    ++seq;
  }
  if (blockIdx.y == 0 && wave == 0 && lane == 0) {   // this lane leaves the reduce kernel its notes
    if (w == 0) a.wg_info[0] = total;
    if (info_seq >= 0) {
      a.wg_info[2 * w + 2] = info_seq;
      a.wg_info[2 * w + 3] = info_start;
    }
  }
}

// The merge of the batch-invariant cutting: grid (num_seqs, ceil(Hq / 4)), a wave per q head, a lane owns D / 64
// dims.  Lane j takes span j's (m, l); the wave agrees on the maximum and the weights; the spans' outputs are added
// in span order.  Empty decode sequences get their defined output here as well.
template <int D>
__global__ __launch_bounds__(256) void paged_decode_fixed_spans_reduce_kernel(StreamKArgs a) {
  constexpr int V = D / 64;
  static_assert(kFixedSpans <= kWave, "one lane per span");
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int seq = blockIdx.x;
  const int Hq = a.io.num_q_heads;
  if (head >= Hq) return;
  const int q0 = a.cu_seqlens_q ? a.cu_seqlens_q[seq] : seq;
  const int q1 = a.cu_seqlens_q ? a.cu_seqlens_q[seq + 1] : seq + 1;
  const int len = a.seq_lens[seq];
  if (q1 - q0 != 1) return;
  const int64_t row = q0;
  const int ntiles = len > 0 ? (len + kTile - 1) / kTile - window_first(len, a.io.window) / kTile : 0;
  if (ntiles == 0) {  // empty sequence: defined output (zeros, lse = -inf)
    for (int i = 0; i < V; ++i)
      store_act_rt(a.io.out_dtype, a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + i, 0.f);
    if (a.io.lse != nullptr && lane == 0) a.io.lse[row * Hq + head] = -INFINITY;
    return;
  }
  const int per = fixed_span_tiles(ntiles);
  const int spans = (ntiles + per - 1) / per;
  if (spans == 1) return;  // written directly by the main kernel
  const int64_t slot0 = (int64_t)seq * kFixedSpans;
  const bool live = lane < spans;
  const int64_t mine = slot0 + (live ? lane : spans - 1);
  const float mj_raw = a.part_ml[(mine * Hq + head) * 2 + 0];
  const float lj_raw = a.part_ml[(mine * Hq + head) * 2 + 1];
  const float mj = live ? mj_raw : -INFINITY;
  const float m = wave_max(mj);
  const float ej = live ? __builtin_amdgcn_exp2f(mj - m) : 0.f;
  const float l = wave_sum(live ? lj_raw * ej : 0.f);
  float acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = 0.f;
  for (int k0 = 0; k0 < spans; k0 += 8) {   // eight spans per trip to memory, added in span order
    float po[8][V];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t sk = slot0 + min(k0 + k, spans - 1);
      const float* p = a.part_o + (sk * Hq + head) * (int64_t)D + lane * V;
#pragma unroll
      for (int i = 0; i < V; ++i) po[k][i] = p[i];
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float wk = k0 + k < spans ? __shfl(ej, k0 + k, kWave) : 0.f;
      const uint32_t kk = wk != 0.f ? 0xffffffffu : 0u;
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] += as_f32(as_u32(po[k][i]) & kk) * wk;
    }
  }
  const float lt = l + sink_term(a.io.sinks, head, m);
  const float inv = 1.0f / lt;
#pragma unroll
  for (int i = 0; i < V; ++i)
    store_act_rt(a.io.out_dtype, a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + i, acc[i] * inv);
  if (a.io.lse != nullptr && lane == 0) a.io.lse[row * Hq + head] = (m + __builtin_amdgcn_logf(lt)) * kLn2;
}

// Merge the partial states of every decode sequence that more than one workgroup touched, and give empty decode
// sequences their defined output.  grid (P, ceil(Hq / 16)), 4 waves; a wave takes four q heads, 16 lanes each, a
// lane D/16 dims.
// A sequence is cut only where a workgroup's share begins inside it, so the grid runs over the P workgroups of
// the main kernel, not over the sequences: block w looks at the sequence in which share w begins (the main
// kernel left its number and its place on the work line) and merges it if share w is the
// FIRST to begin inside it; a sequence cut several times is thus merged once, and one that is not cut costs a
// block one round trip.  (A grid over the sequences, every wave scanning all sequence lengths for its place on
// the line, took 44 us at 512 sequences; with one q head per wave the P x Hq waves of this grid, 8192 at 32
// heads, did not fit the chip at once and took 11-13 us.)
template <int D>
__global__ __launch_bounds__(256) void paged_decode_streamk_reduce_kernel(StreamKArgs a) {
  constexpr int V = D / 16;
  const int lane = threadIdx.x & 63;
  const int sub = lane & 15;           // lane within the head's group of 16
  const int grp = lane & 48;           // first lane of that group
  const int Hq = a.io.num_q_heads;
  const int head_raw = (blockIdx.y * 4 + (threadIdx.x >> 6)) * 4 + (lane >> 4);
  const bool head_ok = head_raw < Hq;
  const int head = head_ok ? head_raw : Hq - 1;   // lanes past the last head repeat it and store nothing
  const int w = blockIdx.x;
  const int B = a.num_seqs;
  // the loads that depend on nothing but the arguments go out before the first branch
  const int64_t total = a.wg_info[0];
  // (the share's sequence is undefined for a workgroup without a share: clamped here, looked at only if w < P)
  const int seq = min(max((int)a.wg_info[2 * w + 2], 0), B - 1);
  const int64_t start = a.wg_info[2 * w + 3];
  auto store_dims = [&](int64_t r, const float (&x)[V]) __attribute__((always_inline)) {
    if (!head_ok) return;
    const int64_t at = r * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + sub * V;
#pragma unroll
    for (int i = 0; i < V; ++i) store_act_rt(a.io.out_dtype, a.io.out, at + i, x[i]);
  };
  // empty decode sequences (no tile: length 0): zeros, lse = -inf; the blocks share them out
  for (int s = w; s < B; s += (int)gridDim.x) {
    const int q0e = a.cu_seqlens_q ? a.cu_seqlens_q[s] : s;
    const int q1e = a.cu_seqlens_q ? a.cu_seqlens_q[s + 1] : s + 1;
    if (q1e - q0e == 1 && a.seq_lens[s] <= 0) {
      float z[V];
#pragma unroll
      for (int i = 0; i < V; ++i) z[i] = 0.f;
      store_dims(q0e, z);
      if (a.io.lse != nullptr && sub == 0 && head_ok) a.io.lse[(int64_t)q0e * Hq + head] = -INFINITY;
    }
  }
  const int P = active_workgroups(total, a.num_wg);
  if (w == 0 || w >= P) return;
  const int len = a.seq_lens[seq];
  const int64_t row = a.cu_seqlens_q ? a.cu_seqlens_q[seq] : seq;
  const int ntiles = (len + kTile - 1) / kTile - window_first(len, a.io.window) / kTile;   // a decode sequence with tiles
  // workgroup holding unit x: the largest w with floor(w*T/P) <= x; the sequence's tiles are units
  // start + setup_units .. start + setup_units + ntiles - 1
  const int w_first = (int)(((start + a.setup_units + 1) * P - 1) / total);
  const int w_last = (int)(((start + a.setup_units + ntiles) * P - 1) / total);
  if (w_first == w_last) return;  // not cut
  const int span = w_last - w_first + 1;
  if (span > 16) {
    // A long span (one sequence over dozens of workgroups): a whole wave per q head, 64 slots per pass, and the
    // block's 16 heads spread over the first four blocks that begin inside the sequence (there are span - 1).
    constexpr int V2 = D / 64;
    const int j = w - (w_first + 1);
    const int h1 = (blockIdx.y * 4 + j) * 4 + (threadIdx.x >> 6);
    if (j < 0 || j >= 4 || h1 >= Hq) return;   // j < 0: the share begins with the sequence, not inside it
    float m = -INFINITY, l = 0.f, acc[V2];
#pragma unroll
    for (int i = 0; i < V2; ++i) acc[i] = 0.f;
    for (int wb = w_first; wb <= w_last; wb += kWave) {
      const int wj = wb + lane;
      const bool live = wj <= w_last && wg_tile_begin(wj, total, P) < wg_tile_begin(wj + 1, total, P);
      // loads are unconditional (clamped to the sequence's last workgroup) and what they return is removed with
      // a bit mask where the slot holds nothing
      const int64_t slot = (int64_t)min(wj, w_last) + seq;
      const uint32_t keep = live ? 0xffffffffu : 0u;
      const float mj_raw = a.part_ml[(slot * Hq + h1) * 2 + 0];
      const float lj_raw = a.part_ml[(slot * Hq + h1) * 2 + 1];
      const float mj = live ? as_f32(as_u32(mj_raw) & keep) : -INFINITY;
      const float lj = as_f32(as_u32(lj_raw) & keep);
      const float m_new = fmaxf(m, wave_max(mj));
      const float ca = __builtin_amdgcn_exp2f(m - m_new);  // first chunk: exp2(-inf) = 0
      const float ej = live ? __builtin_amdgcn_exp2f(mj - m_new) : 0.f;
      l = l * ca + wave_sum(lj * ej);
#pragma unroll
      for (int i = 0; i < V2; ++i) acc[i] *= ca;
      m = m_new;
      // up to sixty-four slots per round trip (128 registers of partial outputs in flight per lane)
      constexpr int kBatch = V2 <= 2 ? 64 : 128 / V2;
      const int count = min(kWave, w_last - wb + 1);
      for (int k0 = 0; k0 < count; k0 += kBatch) {
        float pv[kBatch][V2];
#pragma unroll
        for (int k = 0; k < kBatch; ++k) {
          const int64_t sk = (int64_t)min(wb + k0 + k, w_last) + seq;
          const float* po = a.part_o + (sk * Hq + h1) * (int64_t)D + lane * V2;
#pragma unroll
          for (int i = 0; i < V2; ++i) pv[k][i] = po[i];
        }
#pragma unroll
        for (int k = 0; k < kBatch; ++k) {
          const float wk = (k0 + k) < count ? __shfl(ej, (k0 + k) & (kWave - 1), kWave) : 0.f;  // unnormalised sums
          const uint32_t kk = wk != 0.f ? 0xffffffffu : 0u;
#pragma unroll
          for (int i = 0; i < V2; ++i) acc[i] += as_f32(as_u32(pv[k][i]) & kk) * wk;
        }
      }
    }
    l += sink_term(a.io.sinks, h1, m);
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < V2; ++i)
      store_act_rt(a.io.out_dtype, a.io.out, row * a.io.out_stride_t + (int64_t)h1 * a.io.out_stride_h + lane * V2 + i, acc[i] * inv);
    if (a.io.lse != nullptr && lane == 0) a.io.lse[row * Hq + h1] = (m + __builtin_amdgcn_logf(l)) * kLn2;
    return;
  }
  if (w != w_first + 1) return;  // another block's to merge

  auto group_max = [&](float x) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, kWave));
    return x;
  };
  auto group_sum = [&](float x) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) x += __shfl_xor(x, o, kWave);
    return x;
  };
  const float* po_head = a.part_o + (int64_t)head * D + sub * V;
  const float* ml_head = a.part_ml + (int64_t)head * 2;
  // lane `sub` of a group takes slot wb + sub's (m, l); the group agrees on the maximum and the weights, then
  // every lane adds up its dims over the slots.  All loads of a pass are unconditional (slots past the last
  // reread the last one and get weight 0; a select on a loaded value would become a branch around the load) and
  // leave before the first is used.  N slots per pass.
  float m = -INFINITY, l = 0.f, acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = 0.f;
  auto pass = [&](int wb, auto n_tag) __attribute__((always_inline)) {
    constexpr int N = decltype(n_tag)::value;   // <= 16
    const int wj = wb + sub;
    const bool live = sub < N && wj <= w_last && wg_tile_begin(wj, total, P) < wg_tile_begin(wj + 1, total, P);
    const int64_t slot = (int64_t)min(wj, w_last) + seq;
    const float mj_raw = ml_head[slot * Hq * 2 + 0];
    const float lj_raw = ml_head[slot * Hq * 2 + 1];
    float po[N][V];
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const int64_t sk = (int64_t)min(wb + k, w_last) + seq;
      const float* p = po_head + sk * Hq * (int64_t)D;
#pragma unroll
      for (int i = 0; i < V; i += 4) {
        const floatx4 x = *reinterpret_cast<const floatx4*>(p + i);
        po[k][i] = x.x; po[k][i + 1] = x.y; po[k][i + 2] = x.z; po[k][i + 3] = x.w;
      }
    }
    const uint32_t keep = live ? 0xffffffffu : 0u;
    const float mj = live ? as_f32(as_u32(mj_raw) & keep) : -INFINITY;
    const float lj = as_f32(as_u32(lj_raw) & keep);
    const float m_new = fmaxf(m, group_max(mj));
    const float ca = __builtin_amdgcn_exp2f(m - m_new);  // first pass: exp2(-inf) = 0
    const float ej = live ? __builtin_amdgcn_exp2f(mj - m_new) : 0.f;
    l = l * ca + group_sum(lj * ej);
    m = m_new;
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] *= ca;
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float wk = __shfl(ej, grp + k, kWave);  // 0 for slots past the last and for empty ones
      const uint32_t kk = wk != 0.f ? 0xffffffffu : 0u;
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] += as_f32(as_u32(po[k][i]) & kk) * wk;
    }
  };
  constexpr int kLong = V <= 8 ? 16 : 8;   // 128 registers of partial outputs in flight per lane
  if (span <= 4) {
    pass(w_first, std::integral_constant<int, 4>{});
  } else if (span <= 8) {
    pass(w_first, std::integral_constant<int, 8>{});
  } else {
    for (int wb = w_first; wb <= w_last; wb += kLong) pass(wb, std::integral_constant<int, kLong>{});
  }
  l += sink_term(a.io.sinks, head, m);
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] *= inv;
  store_dims(row, acc);
  if (a.io.lse != nullptr && sub == 0 && head_ok)
    a.io.lse[row * Hq + head] = (m + __builtin_amdgcn_logf(l)) * kLn2;
}

// The same merge with a grid over the sequences, for batches of few sequences (every one of which is cut, most
// of them several times): grid (num_seqs, ceil(Hq / 4)), 4 waves, one wave per q head, lane owns D/64 dims.  The
// sequence's place on the work line comes from the main kernel (seq_first_unit).
template <int D>
__global__ __launch_bounds__(256) void paged_decode_streamk_reduce_by_seq_kernel(StreamKArgs a) {
  constexpr int V = D / 64;
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int seq = blockIdx.x;
  if (head >= a.io.num_q_heads) return;
  // all the loads that depend on nothing but the arguments go out together, before the first branch
  const int q0 = a.cu_seqlens_q ? a.cu_seqlens_q[seq] : seq;
  const int q1 = a.cu_seqlens_q ? a.cu_seqlens_q[seq + 1] : seq + 1;
  const int len = a.seq_lens[seq];
  const int64_t total = a.wg_info[0];
  const int64_t start = a.seq_first_unit[seq];   // defined for every decode sequence that has a tile
  if (q1 - q0 != 1) return;
  const int64_t row = q0;
  const int ntiles = len > 0 ? (len + kTile - 1) / kTile - window_first(len, a.io.window) / kTile : 0;
  if (ntiles == 0) {  // empty sequence: defined output (zeros, lse = -inf)
    for (int i = 0; i < V; ++i)
      store_act_rt(a.io.out_dtype, a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + i, 0.f);
    if (a.io.lse != nullptr && lane == 0) a.io.lse[row * a.io.num_q_heads + head] = -INFINITY;
    return;
  }
  const int P = active_workgroups(total, a.num_wg);
  // workgroup holding unit x: the largest w with floor(w*T/P) <= x; the sequence's tiles are units
  // start + setup_units .. start + setup_units + ntiles - 1
  const int w_first = (int)(((start + a.setup_units + 1) * P - 1) / total);
  const int w_last = (int)(((start + a.setup_units + ntiles) * P - 1) / total);
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
    // up to sixty-four slots per round trip (128 registers of partial outputs in flight per lane): a long span is
    // merged by ONE wave per (sequence, q head), so this path is a chain of round trips (a 256-slot span -- one
    // 128k-token sequence -- takes 21 us; 22.5 us with 16 slots per trip).  The loads of a batch are unconditional
    // (slots past the last reread the last one, weight 0) so that they all leave before the first is used.
    constexpr int kBatch = V <= 2 ? 64 : 128 / V;
    const int count = min(kWave, w_last - wb + 1);
    for (int k0 = 0; k0 < count; k0 += kBatch) {
      float pv[kBatch][V];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const int64_t sk = (int64_t)min(wb + k0 + k, w_last) + seq;
        const float* po = a.part_o + (sk * a.io.num_q_heads + head) * (int64_t)D + lane * V;
#pragma unroll
        for (int i = 0; i < V; ++i) pv[k][i] = po[i];
      }
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const float wk = (k0 + k) < count ? __shfl(ej, (k0 + k) & (kWave - 1), kWave) : 0.f;  // unnormalised sums
        const uint32_t kk = wk != 0.f ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] += as_f32(as_u32(pv[k][i]) & kk) * wk;
      }
    }
  }
  l += sink_term(a.io.sinks, head, m);
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < V; ++i)
    store_act_rt(a.io.out_dtype, a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + i, acc[i] * inv);
  if (a.io.lse != nullptr && lane == 0)
    a.io.lse[row * a.io.num_q_heads + head] = (m + __builtin_amdgcn_logf(l)) * kLn2;
}

// The same merge for a handful of sequences, each cut dozens or hundreds of times (long contexts): grid
// (num_seqs, Hq), the block's four waves share ONE q head's span -- wave p takes the span's slots p, p + 4, ... --
// and their four states meet in LDS.  (With a wave per head a 256-slot span was a chain of eight round trips:
// 20.8 us for one 128k-token sequence, next to a 48 us main kernel.)
template <int D>
__global__ __launch_bounds__(256) void paged_decode_streamk_reduce_split4_kernel(StreamKArgs a) {
  constexpr int V = D / 64;
  __shared__ float sh_acc[3][V][kWave];
  __shared__ float sh_ml[3][2];
  const int lane = threadIdx.x & 63;
  const int part = threadIdx.x >> 6;
  const int head = blockIdx.y;
  const int seq = blockIdx.x;
  const int Hq = a.io.num_q_heads;
  const int q0 = a.cu_seqlens_q ? a.cu_seqlens_q[seq] : seq;
  const int q1 = a.cu_seqlens_q ? a.cu_seqlens_q[seq + 1] : seq + 1;
  const int len = a.seq_lens[seq];
  const int64_t total = a.wg_info[0];
  const int64_t start = a.seq_first_unit[seq];   // defined for every decode sequence that has a tile
  if (q1 - q0 != 1) return;                      // every branch down to the barrier is uniform over the block
  const int64_t row = q0;
  const int ntiles = len > 0 ? (len + kTile - 1) / kTile - window_first(len, a.io.window) / kTile : 0;
  if (ntiles == 0) {  // empty sequence: defined output (zeros, lse = -inf)
    if (part == 0) {
      for (int i = 0; i < V; ++i)
        store_act_rt(a.io.out_dtype, a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + i, 0.f);
      if (a.io.lse != nullptr && lane == 0) a.io.lse[row * Hq + head] = -INFINITY;
    }
    return;
  }
  const int P = active_workgroups(total, a.num_wg);
  const int w_first = (int)(((start + a.setup_units + 1) * P - 1) / total);
  const int w_last = (int)(((start + a.setup_units + ntiles) * P - 1) / total);
  if (w_first == w_last) return;  // written directly by the main kernel
  // this wave's slots: w_first + part + 4 i, i = 0 .. n - 1 (n = 0 for a span shorter than its number)
  const int span = w_last - w_first + 1;
  const int n = span > part ? (span - part + 3) / 4 : 0;
  float m = -INFINITY, l = 0.f, acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = 0.f;
  // one pass = N of the wave's slots from index i0 on: lane j takes slot j's (m, l), the wave agrees on the
  // maximum and the weights, every lane adds up its dims.  All loads are unconditional (indices past the last
  // reread the span's last slot and get weight 0) and leave before the first is used.
  auto pass = [&](int i0, auto n_tag) __attribute__((always_inline)) {
    constexpr int N = decltype(n_tag)::value;   // <= 64
    const int i = i0 + lane;
    const int wj = w_first + part + 4 * i;
    const bool live = lane < N && i < n && wg_tile_begin(wj, total, P) < wg_tile_begin(wj + 1, total, P);
    const int64_t slot = (int64_t)min(wj, w_last) + seq;
    const float mj_raw = a.part_ml[(slot * Hq + head) * 2 + 0];
    const float lj_raw = a.part_ml[(slot * Hq + head) * 2 + 1];
    float po[N][V];
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const int64_t sk = (int64_t)min(w_first + part + 4 * (i0 + k), w_last) + seq;
      const float* p = a.part_o + (sk * Hq + head) * (int64_t)D + lane * V;
#pragma unroll
      for (int x = 0; x < V; ++x) po[k][x] = p[x];
    }
    const uint32_t keep = live ? 0xffffffffu : 0u;
    const float mj = live ? as_f32(as_u32(mj_raw) & keep) : -INFINITY;
    const float lj = as_f32(as_u32(lj_raw) & keep);
    const float m_new = fmaxf(m, wave_max(mj));
    const float ca = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m_new);   // a wave without a slot stays empty
    const float ej = live ? __builtin_amdgcn_exp2f(mj - m_new) : 0.f;
    l = l * ca + wave_sum(lj * ej);
    m = m_new;
#pragma unroll
    for (int x = 0; x < V; ++x) acc[x] *= ca;
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float wk = __shfl(ej, k, kWave);
      const uint32_t kk = wk != 0.f ? 0xffffffffu : 0u;
#pragma unroll
      for (int x = 0; x < V; ++x) acc[x] += as_f32(as_u32(po[k][x]) & kk) * wk;
    }
  };
  constexpr int kLong = V <= 2 ? 64 : 128 / V;   // 128 registers of partial outputs in flight per lane
  if (n <= 4) {
    pass(0, std::integral_constant<int, 4>{});
  } else if (n <= 16) {
    pass(0, std::integral_constant<int, 16>{});
  } else {
    for (int i0 = 0; i0 < n; i0 += kLong) pass(i0, std::integral_constant<int, kLong>{});
  }
  if (part > 0) {
#pragma unroll
    for (int x = 0; x < V; ++x) sh_acc[part - 1][x][lane] = acc[x];
    if (lane == 0) {
      sh_ml[part - 1][0] = m;
      sh_ml[part - 1][1] = l;
    }
  }
  __syncthreads();
  if (part > 0) return;
#pragma unroll
  for (int p = 0; p < 3; ++p) {
    const float mp = sh_ml[p][0], lp = sh_ml[p][1];
    if (mp == -INFINITY) continue;   // that wave had no slot (uniform)
    const float m_new = fmaxf(m, mp);   // wave 0 always holds the span's first slot: m is finite
    const float ca = __builtin_amdgcn_exp2f(m - m_new), cb = __builtin_amdgcn_exp2f(mp - m_new);
    l = l * ca + lp * cb;
    m = m_new;
#pragma unroll
    for (int x = 0; x < V; ++x) acc[x] = acc[x] * ca + sh_acc[p][x][lane] * cb;
  }
  l += sink_term(a.io.sinks, head, m);
  const float inv = 1.0f / l;
#pragma unroll
  for (int x = 0; x < V; ++x)
    store_act_rt(a.io.out_dtype, a.io.out, row * a.io.out_stride_t + (int64_t)head * a.io.out_stride_h + lane * V + x, acc[x] * inv);
  if (a.io.lse != nullptr && lane == 0) a.io.lse[row * Hq + head] = (m + __builtin_amdgcn_logf(l)) * kLn2;
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

// BIAS: the instantiation with the ALiBi bias (DecodeTile's form with the extras; the soft cap stays the identity).
template <int D, int QDT, int WPW, bool BIAS>
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
  DTile::template run<BIAS>(a.io, seq, seq, len, 0, t_begin, t_end, hkv, lane, lds[wave], st);
  DTile::emit_v2(a.io, a.tmp_out, a.max_logits, a.exp_sums, seq, part, a.max_parts, hkv, lane, st);
}

// out = sum_j w_j tmp_out_j / sum_j w_j, w_j = exp_sums_j * exp(max_logits_j - max).
template <int D, int QDT>
static int launch_streamk(const StreamKArgs& args, hipStream_t s) {
  const int hkv = args.io.g.num_kv_heads;
  const int hpw = heads_per_wg(hkv);
  StreamKArgs a = args;
  a.setup_units = setup_units_for(8 / hpw);
  dim3 grid(a.num_wg, (hkv + hpw - 1) / hpw);
#define KVQ_SK_CODE(H, C, CODE)                                                                                   \
  do {                                                                                                            \
    if (a.fixed_spans && !C && stream)                                                                            \
      hipLaunchKernelGGL((paged_decode_streamk_kernel<D, QDT, H, false, CODE, true, true>), grid, dim3(512), 0, s, a); \
    else if (a.fixed_spans)                                                                                       \
      hipLaunchKernelGGL((paged_decode_streamk_kernel<D, QDT, H, C, CODE, false, true>), grid, dim3(512), 0, s, a); \
    else if (!C && stream)                                                                                        \
      hipLaunchKernelGGL((paged_decode_streamk_kernel<D, QDT, H, false, CODE, true>), grid, dim3(512), 0, s, a);  \
    else                                                                                                          \
      hipLaunchKernelGGL((paged_decode_streamk_kernel<D, QDT, H, C, CODE, false>), grid, dim3(512), 0, s, a);     \
  } while (0)
#define KVQ_SK(H, C)                                                                                              \
  do {                                                                                                            \
    if (a.io.g.code_type == KVQ_CODE_FP8_E4M3) KVQ_SK_CODE(H, C, KVQ_CODE_FP8_E4M3);                              \
    else if (a.io.g.code_type == KVQ_CODE_INT4) KVQ_SK_CODE(H, C, KVQ_CODE_INT4);                                 \
    else KVQ_SK_CODE(H, C, KVQ_CODE_INT8);                                                                        \
  } while (0)
  // a head's records of a block back to back (HND order): the tile loads may stream past the caches
  // (not at head size 256, where it measured slower: 293 against 279 us on 64 x 1k-8k tokens)
  const bool stream = D <= 128 && a.io.g.stride_slot == 2 * (code_bytes(a.io.g) + 4) && a.io.g.block_size >= 16;
  if (a.io.cap_c != 0.f || a.io.alibi != nullptr) {   // the instantiation with the extras: soft cap and ALiBi
    switch (hpw) {
      case 8: KVQ_SK(8, true); break;
      case 4: KVQ_SK(4, true); break;
      case 2: KVQ_SK(2, true); break;
      default: KVQ_SK(1, true); break;
    }
  } else {
    switch (hpw) {
      case 8: KVQ_SK(8, false); break;
      case 4: KVQ_SK(4, false); break;
      case 2: KVQ_SK(2, false); break;
      default: KVQ_SK(1, false); break;
    }
  }
#undef KVQ_SK
#undef KVQ_SK_CODE
  int rc = check_hip(hipGetLastError(), "paged_attn_int8 decode launch");
  if (rc) return rc;
  if (a.fixed_spans) {
    dim3 rgrid(a.num_seqs, (a.io.num_q_heads + 3) / 4);
    hipLaunchKernelGGL((paged_decode_fixed_spans_reduce_kernel<D>), rgrid, dim3(256), 0, s, a);
    return check_hip(hipGetLastError(), "paged_attn_int8 reduce launch");
  }
  // a sequence is cut where a share begins inside it: a batch of few sequences has most of them cut several
  // times (grid over the sequences, a wave per q head), a large batch has at most one cut per share and many
  // sequences with none (grid over the shares, four q heads per wave)
  if (16 * a.num_seqs <= a.num_wg) {   // a handful of sequences, each cut many times: four waves per q head
    dim3 rgrid(a.num_seqs, a.io.num_q_heads);
    hipLaunchKernelGGL((paged_decode_streamk_reduce_split4_kernel<D>), rgrid, dim3(256), 0, s, a);
  } else if (8 * a.num_seqs <= 3 * a.num_wg) {
    dim3 rgrid(a.num_seqs, (a.io.num_q_heads + 3) / 4);
    hipLaunchKernelGGL((paged_decode_streamk_reduce_by_seq_kernel<D>), rgrid, dim3(256), 0, s, a);
  } else {
    dim3 rgrid(a.num_wg, (a.io.num_q_heads + 15) / 16);
    hipLaunchKernelGGL((paged_decode_streamk_reduce_kernel<D>), rgrid, dim3(256), 0, s, a);
  }
  return check_hip(hipGetLastError(), "paged_attn_int8 reduce launch");
}

template <int D>
int launch_streamk_q(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s) {
  if (out_dtype != KVQ_F32 && out_dtype != KVQ_BF16 && out_dtype != KVQ_F16)
    return fail(KVQ_EINVAL, "paged_attn_int8: unknown out_dtype %d", out_dtype);
  switch (q_dtype) {
    case KVQ_F32: return launch_streamk<D, KVQ_F32>(a, s);
    case KVQ_BF16: return launch_streamk<D, KVQ_BF16>(a, s);
    case KVQ_F16: return launch_streamk<D, KVQ_F16>(a, s);
  }
  return fail(KVQ_EINVAL, "paged_attn_int8: unknown q_dtype %d", q_dtype);
}

template <int D, int QDT>
static int launch_v2(const V2Args& a, int num_seqs, hipStream_t s) {
  const int hkv = a.io.g.num_kv_heads;
  const int wpw = heads_per_wg(hkv);
  dim3 grid(a.max_parts, num_seqs, (hkv + wpw - 1) / wpw);
#define KVQ_V2(W, BIAS) hipLaunchKernelGGL((paged_decode_v2_kernel<D, QDT, W, BIAS>), grid, dim3(W * 64), 0, s, a)
  if (a.io.alibi != nullptr) {
    switch (wpw) {
      case 8: KVQ_V2(8, true); break;
      case 4: KVQ_V2(4, true); break;
      case 2: KVQ_V2(2, true); break;
      default: KVQ_V2(1, true); break;
    }
  } else {
    switch (wpw) {
      case 8: KVQ_V2(8, false); break;
      case 4: KVQ_V2(4, false); break;
      case 2: KVQ_V2(2, false); break;
      default: KVQ_V2(1, false); break;
    }
  }
#undef KVQ_V2
  return check_hip(hipGetLastError(), "paged_attn_v2_int8 launch");
}

template <int D>
int launch_v2_q(const V2Args& a, int num_seqs, int q_dtype, hipStream_t s) {
  switch (q_dtype) {
    case KVQ_F32: return launch_v2<D, KVQ_F32>(a, num_seqs, s);
    case KVQ_BF16: return launch_v2<D, KVQ_BF16>(a, num_seqs, s);
    case KVQ_F16: return launch_v2<D, KVQ_F16>(a, num_seqs, s);
  }
  return fail(KVQ_EINVAL, "paged_attn_v2_int8: unknown q_dtype %d", q_dtype);
}


}  // namespace kvq
