// The V up-projection behind the MLA decode (gfx950): out[b, h, :] = x[b, h, :] . W_UV[h], the second bmm of
// the reference's MLA layer (mla_attention.py:1087-1109, `_v_up_proj`: x [B, N, L] -> [N, B, L], bmm with
// W_UV [N, L, V], back to [B, N * V]) for the handful of rows a decode step has.
//
// The product is a stream of the weights (128 KB per head at L = 512, V = 128, next to 16 KB of x for 16
// sequences): the kernel is one round trip to memory long.  Workgroup = (head, 16 sequences -- 32 in large
// batches --, 128 output dims), 4 waves, wave w contracting over the latent dims L/4 * w .. L/4 * (w + 1) - 1; every load of a wave
// is issued before its first product, the four partial sums meet in LDS and wave 0 stores the result.
// The product is taken transposed, out^T = W^T x^T, as the absorption kernel takes its own: B = x rows (lane =
// sequence, 8 consecutive latent dims: one 16-byte load), A = W^T needs 8 latent dims of one output dim per
// lane while W_UV [L, V] keeps 8 output dims of one latent dim together, so a lane loads the slice [its 8 latent
// dims] x [8 consecutive output dims] and transposes it in registers (one byte permute per dword).  MFMA i of
// a step then holds output dims 8 lane + i: a lane ends with 32 consecutive output dims of its own sequence.
// The workgroups that share a head's weights (the tiles of 16 sequences) are numbered so that they land on
// one XCD and the weights leave HBM once.
#include "kvq_attn_core.cuh"
#include "kvq_internal.h"

namespace kvq {

struct MlaUpProjArgs {
  const void* x;   // [B, H, L]
  int64_t x_sb, x_sh;
  const void* w;   // [H, L, V], output dims contiguous
  int64_t w_sh, w_sl;
  void* out;       // [B, H, V]
  int64_t o_sb, o_sh;
  int num_seqs, num_heads, seq_tiles, v_blocks, ksteps;   // ksteps = L / 128: 32-dim steps per wave
};

constexpr int kXcds = 8;

// KSTEPS = L / 128 when known at compile time (every load of the wave in flight at once), 0 = read it from
// the arguments.  NB = tiles of 16 sequences per workgroup: the weights a wave has loaded and transposed serve NB
// products, so a large batch reads them NB times less often through the L2 (NB = 1 up to 64 sequences, where the
// launch should fill the chip; 2 beyond: with 4 a workgroup's registers leave one workgroup per CU, and 512
// sequences x 128 heads measured 32.8 us against 26.6 us).
template <int DT, int KSTEPS, int NB>
__global__ __launch_bounds__(256) void mla_v_up_proj_kernel(MlaUpProjArgs a) {
  __shared__ floatx4 red[3][8][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  // consecutive workgroups go to consecutive XCDs: the ones that share a head sit kXcds apart
  const int per_head = a.seq_tiles * a.v_blocks;
  const int q = blockIdx.x / kXcds;
  const int head = (q / per_head) * kXcds + blockIdx.x % kXcds;
  if (head >= a.num_heads) return;   // uniform over the workgroup
  const int rem = q % per_head;
  const int n0 = (rem / a.seq_tiles) * 128, b0 = (rem % a.seq_tiles) * (16 * NB);
  const int ksteps = KSTEPS > 0 ? KSTEPS : a.ksteps;
  const int k0 = wave * ksteps * 32;
  const uint16_t* wp = static_cast<const uint16_t*>(a.w) + (int64_t)head * a.w_sh + (int64_t)(k0 + 8 * g) * a.w_sl + n0 + 8 * c;
  const uint16_t* xp[NB];
#pragma unroll
  for (int t = 0; t < NB; ++t) {
    const int brow = min(b0 + 16 * t + c, a.num_seqs - 1);   // rows past the end: a copy, not written
    xp[t] = static_cast<const uint16_t*>(a.x) + (int64_t)brow * a.x_sb + (int64_t)head * a.x_sh + k0 + 8 * g;
  }
  floatx4 acc[NB][8];
#pragma unroll
  for (int t = 0; t < NB; ++t)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[t][i] = (floatx4){0.f, 0.f, 0.f, 0.f};
  auto step = [&](const u32x4 (&rows)[8], const u32x4 (&xop)[NB]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t sel = (i & 1) ? kPermHighHalves : kPermLowHalves;
      u32x4 wt;
      wt.x = perm(rows[1][i >> 1], rows[0][i >> 1], sel);
      wt.y = perm(rows[3][i >> 1], rows[2][i >> 1], sel);
      wt.z = perm(rows[5][i >> 1], rows[4][i >> 1], sel);
      wt.w = perm(rows[7][i >> 1], rows[6][i >> 1], sel);
#pragma unroll
      for (int t = 0; t < NB; ++t) acc[t][i] = mfma16<DT>(wt, xop[t], acc[t][i]);
    }
  };
  if constexpr (KSTEPS > 0) {
    u32x4 rows[KSTEPS][8], xop[KSTEPS][NB];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
      for (int t = 0; t < NB; ++t) xop[s][t] = *reinterpret_cast<const u32x4_a4*>(xp[t] + 32 * s);
#pragma unroll
      for (int j = 0; j < 8; ++j) rows[s][j] = *reinterpret_cast<const u32x4*>(wp + (int64_t)(32 * s + j) * a.w_sl);
    }
    __builtin_amdgcn_sched_barrier(0);   // keep the scheduler from sinking the loads back to their uses
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) step(rows[s], xop[s]);
  } else {
    for (int s = 0; s < ksteps; ++s) {
      u32x4 rows[8], xop[NB];
#pragma unroll
      for (int j = 0; j < 8; ++j) rows[j] = *reinterpret_cast<const u32x4*>(wp + (int64_t)(32 * s + j) * a.w_sl);
#pragma unroll
      for (int t = 0; t < NB; ++t) xop[t] = *reinterpret_cast<const u32x4_a4*>(xp[t] + 32 * s);
      step(rows, xop);
    }
  }
  // lane (sequence c, quarter g) holds output dims n0 + 32 g + 8 r + i of its sequence of tile t in acc[t][i][r];
  // the tiles pass through the one LDS area in turn
#pragma unroll
  for (int t = 0; t < NB; ++t) {
    if (t > 0) __syncthreads();   // wave 0 has read tile t - 1
    if (wave > 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) red[wave - 1][i][lane] = acc[t][i];
    }
    __syncthreads();
    const int b = b0 + 16 * t + c;
    if (wave == 0 && b < a.num_seqs) {
#pragma unroll
      for (int w = 0; w < 3; ++w)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[t][i] += red[w][i][lane];
      uint16_t* op = static_cast<uint16_t*>(a.out) + (int64_t)b * a.o_sb + (int64_t)head * a.o_sh + n0 + 32 * g;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        u32x4 v;
        v.x = pack2<DT>(acc[t][0][r], acc[t][1][r]);
        v.y = pack2<DT>(acc[t][2][r], acc[t][3][r]);
        v.z = pack2<DT>(acc[t][4][r], acc[t][5][r]);
        v.w = pack2<DT>(acc[t][6][r], acc[t][7][r]);
        *reinterpret_cast<u32x4*>(op + 8 * r) = v;
      }
    }
  }
}

}  // namespace kvq

extern "C" {

int kvq_mla_v_up_proj(void* out, int64_t out_stride_b, int64_t out_stride_h, const void* x, int dtype, int64_t x_stride_b,
                      int64_t x_stride_h, const void* w_uv, int64_t w_stride_h, int64_t w_stride_l, int num_seqs,
                      int num_heads, int kv_lora_rank, int v_head_dim, kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "mla_v_up_proj";
  KVQ_REQUIRE(out && x && w_uv, "%s: NULL pointer", op);
  KVQ_REQUIRE(dtype == KVQ_BF16 || dtype == KVQ_F16, "%s: x, W_UV and out must be bf16 or fp16 (dtype %d)", op, dtype);
  KVQ_REQUIRE(num_seqs >= 0 && num_heads > 0, "%s: bad batch (%d sequences, %d heads)", op, num_seqs, num_heads);
  KVQ_REQUIRE(kv_lora_rank > 0 && kv_lora_rank % 128 == 0, "%s: kv_lora_rank %d must be a multiple of 128", op, kv_lora_rank);
  KVQ_REQUIRE(v_head_dim > 0 && v_head_dim % 128 == 0, "%s: v_head_dim %d must be a multiple of 128", op, v_head_dim);
  KVQ_REQUIRE(((uintptr_t)w_uv % 16) == 0 && w_stride_h % 8 == 0 && w_stride_l % 8 == 0 && w_stride_l >= v_head_dim,
              "%s: W_UV rows must be 16-byte aligned and hold v_head_dim contiguous dims", op);
  KVQ_REQUIRE(((uintptr_t)x % 4) == 0 && x_stride_b % 2 == 0 && x_stride_h % 2 == 0 && x_stride_h >= 0 && x_stride_b >= 0,
              "%s: x rows must be 4-byte aligned", op);
  KVQ_REQUIRE(((uintptr_t)out % 16) == 0 && out_stride_b % 8 == 0 && out_stride_h % 8 == 0 && out_stride_h >= v_head_dim,
              "%s: out rows must be 16-byte aligned and v_head_dim wide", op);
  if (num_seqs == 0) return 0;
  MlaUpProjArgs a{};
  a.x = x;
  a.x_sb = x_stride_b;
  a.x_sh = x_stride_h;
  a.w = w_uv;
  a.w_sh = w_stride_h;
  a.w_sl = w_stride_l;
  a.out = out;
  a.o_sb = out_stride_b;
  a.o_sh = out_stride_h;
  a.num_seqs = num_seqs;
  a.num_heads = num_heads;
  const int tiles16 = (num_seqs + 15) / 16;
  const int nb = tiles16 <= 4 ? 1 : 2;
  a.seq_tiles = (tiles16 + nb - 1) / nb;
  a.v_blocks = v_head_dim / 128;
  a.ksteps = kv_lora_rank / 128;
  const int64_t blocks = (int64_t)((num_heads + kXcds - 1) / kXcds) * kXcds * a.seq_tiles * a.v_blocks;
  KVQ_REQUIRE(blocks < (1ll << 31), "%s: %lld workgroups do not fit a grid", op, (long long)blocks);
  hipStream_t s = as_stream(stream);
  const dim3 grid((unsigned)blocks), block(256);
#define KVQ_UPPROJ_NB(T, K, N) hipLaunchKernelGGL((mla_v_up_proj_kernel<T, K, N>), grid, block, 0, s, a)
#define KVQ_UPPROJ(T, K)              \
  do {                                \
    if (nb == 1) KVQ_UPPROJ_NB(T, K, 1);      \
    else KVQ_UPPROJ_NB(T, K, 2);              \
  } while (0)
  if (dtype == KVQ_BF16) {
    if (a.ksteps == 4) KVQ_UPPROJ(KVQ_BF16, 4);
    else KVQ_UPPROJ(KVQ_BF16, 0);
  } else {
    if (a.ksteps == 4) KVQ_UPPROJ(KVQ_F16, 4);
    else KVQ_UPPROJ(KVQ_F16, 0);
  }
#undef KVQ_UPPROJ
#undef KVQ_UPPROJ_NB
  return check_hip(hipGetLastError(), "mla_v_up_proj launch");
}

}  // extern "C"
