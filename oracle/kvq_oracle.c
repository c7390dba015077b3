/*
 * CPU oracle for the int8 KV-cache attention path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference algorithm.  It exists so
 * that tests, the smoke check and the benchmark's CPU-baseline leg have
 * something independent to compare the HIP kernels against.  Nothing in the
 * shipped product path may call it.
 *
 * Every function names the reference file:line it follows (paths relative to
 * the MetaX-MACA/vLLM-metax tree).  Parity status per function:
 *
 *   kvq_oracle_quant_rows           pinned   (torch CPU round/div, closed forms,
 *                                             exact-rational brute force)
 *   kvq_oracle_cache_write          pinned   (layout algebra + python scatter loop)
 *   kvq_oracle_quant_rows_fp8       pinned   (torch CPU float8_e4m3fn conversion on every fp32 in range,
 *                                             the 256-entry decode table against torch, closed forms)
 *   kvq_oracle_quant_rows_int4      pinned against ITSELF only (closed forms: every value k * scale maps to k,
 *                                             midpoints go to the even neighbour, brute force against exact
 *                                             rationals, pack / unpack round trip); PARITY UNPINNED against
 *                                             upstream: the reference states the record width of its int4 mode
 *                                             (vllm_metax/v1/attention/backends/triton_attn.py:336-348) and nothing
 *                                             of its arithmetic -- scale rule, rounding and nibble order are this
 *                                             build's decision
 *   kvq_oracle_paged_attn           pinned   (torch SDPA on gathered K/V, block
 *                                             permutation invariance)
 *   kvq_oracle_paged_attn_partition pinned   (equals unsplit attention for any
 *   kvq_oracle_splitk_reduce                  partition size; single partition
 *                                             passthrough)
 *   kvq_oracle_merge_attn_states    pinned   (torch restatement, +inf / -inf cases)
 *   kvq_oracle_mla_cache_write      pinned   (same quantiser, one group of 576)
 *   kvq_oracle_mla_gather_dequant   pinned   (python gather loop, code * scale in numpy fp32,
 *                                             round trip through the write)
 *   kvq_oracle_mla_decode           pinned   (torch SDPA enable_gqa + logsumexp)
 *   (python) rope_rotate            pinned for bf16 / fp16; PARITY UNPINNED for fp32 (whether
 *                                   the reference's compiler fuses x cos - y sin is not in its source)
 *
 * What no check available offline can pin (it lives in upstream vLLM's Triton
 * sources, which the reference imports but does not vendor): whether the
 * upstream kernel divides by the scale or multiplies by a reciprocal, and its
 * clamp floor for all-zero rows.  The contract used here is the one the
 * reference's own tests/kernels op states: scale = absmax / 127 in fp32,
 * code = clamp(round_half_even(x / scale), -128, 127), absmax floored at eps.
 *
 * All accumulation is done in double so that the oracle's own rounding error
 * is negligible next to the tolerance the kernels are held to.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define KVQ_EXPORT __attribute__((visibility("default")))

/* ---------------------------------------------------------------------------
 * Quantiser.
 * Follows tests/kernels/quant_utils.py:192-220 (native_per_token_group_quant_int8
 * with group_size = head_dim): amax = max|x| floored at eps, scale = amax / 127
 * (fp32 true division), code = clamp(rint(x / scale), -128, 127).
 * RNE + the absmax guard also match
 * csrc/libtorch_stable/quantization/w8a8/int8/scaled_quant.cu:10-37,142-178.
 *
 * x      [rows, D] fp32 (bf16 / fp16 sources are upcast exactly by the caller)
 * eps    absmax floor, already rounded to the SOURCE dtype by the caller
 *        (the reference clamps before the cast to fp32)
 * codes  [rows, D] int8, scales [rows] fp32
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_quant_rows(const float* x, int64_t rows, int64_t D,
                                     float eps, int8_t* codes, float* scales) {
  if (!x || !codes || !scales || rows < 0 || D <= 0) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * D;
    float amax = 0.0f;
    for (int64_t d = 0; d < D; ++d) {
      float a = fabsf(xr[d]);
      /* torch.max propagates NaN */
      if (a > amax || a != a) amax = a;
    }
    if (amax < eps) amax = eps;
    volatile float scale = amax / 127.0f;
    scales[r] = scale;
    for (int64_t d = 0; d < D; ++d) {
      /* scale == 0 only when the row is all zero AND eps underflows in the source dtype
       * (fp16): the as-written op then divides 0 by 0; codes are defined as 0 here. */
      volatile float qf = scale > 0.0f ? xr[d] / scale : 0.0f; /* fp32 true division */
      float rr = nearbyintf(qf);                               /* half-to-even */
      if (rr < -128.0f) rr = -128.0f;
      if (rr > 127.0f) rr = 127.0f;
      codes[r * D + d] = (int8_t)rr;
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------
 * fp8 (OCP e4m3fn: 1 sign, 4 exponent bits with bias 7, 3 mantissa bits, no infinities, largest
 * finite value 448) codes of the FP8_PER_TOKEN_HEAD mode of the same layout
 * (vllm_metax/v1/attention/backends/triton_attn.py:336-348, 729-739: the element is one byte, so the
 * record keeps its [K | scale | V | scale] shape).  The rule mirrors the int8 one with the format's
 * maximum in the place of 127: scale = max(absmax, eps) / 448 (fp32 true division), code = the e4m3fn
 * number nearest to x / scale, ties to even, saturating at +-448.
 * ------------------------------------------------------------------------- */
#define KVQ_CODE_INT8 0
#define KVQ_CODE_FP8 1

static float e4m3fn_value(uint8_t b) {
  const int e = (b >> 3) & 15, m = b & 7;
  float v = e == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), e - 10);
  return (b & 0x80) ? -v : v;
}

static uint8_t f32_to_e4m3fn(float y) {
  const uint8_t sign = signbit(y) ? 0x80 : 0;
  float a = fabsf(y);
  if (!(a < 464.0f)) return sign | 0x7e;           /* rounds past 448 (or inf / nan): saturate */
  if (a < 0.015625f) {                              /* below 2^-6: multiples of 2^-9 */
    return sign | (uint8_t)nearbyintf(a * 512.0f);  /* 8 is the smallest normal, as it should be */
  }
  int e = ilogbf(a);                                /* a = f * 2^e, 1 <= f < 2 */
  float q = nearbyintf(ldexpf(a, 3 - e));           /* 8 .. 16, ties to even */
  if (q == 16.0f) {
    q = 8.0f;
    ++e;
  }
  return sign | (uint8_t)(((e + 7) << 3) | ((int)q - 8));
}

KVQ_EXPORT float kvq_oracle_e4m3fn_value(int code) { return e4m3fn_value((uint8_t)code); }

KVQ_EXPORT int kvq_oracle_quant_rows_fp8(const float* x, int64_t rows, int64_t D, float eps,
                                         uint8_t* codes, float* scales) {
  if (!x || !codes || !scales || rows < 0 || D <= 0) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * D;
    float amax = 0.0f;
    for (int64_t d = 0; d < D; ++d) {
      float a = fabsf(xr[d]);
      if (a > amax || a != a) amax = a;
    }
    if (amax < eps) amax = eps;
    volatile float scale = amax / 448.0f;
    scales[r] = scale;
    for (int64_t d = 0; d < D; ++d) {
      volatile float qf = scale > 0.0f ? xr[d] / scale : 0.0f;
      codes[r * D + d] = f32_to_e4m3fn(qf);
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------
 * int4 codes of the INT4_PER_TOKEN_HEAD mode.  The reference fixes the record: two values per byte, so a
 * half record is head_size / 2 code bytes + the fp32 scale
 * (vllm_metax/v1/attention/backends/triton_attn.py:332-346).  The arithmetic is this build's decision,
 * the int8 rule with the format's maximum in the place of 127: scale = max(absmax, eps) / 7 (fp32 true
 * division), code = clamp(rint(x / scale), -8, 7) with ties to even, stored as a 4-bit two's-complement
 * number; dim 2 i sits in the low nibble of byte i, dim 2 i + 1 in the high one.
 * codes [rows, D / 2] bytes, scales [rows] fp32.
 * ------------------------------------------------------------------------- */
#define KVQ_CODE_INT4 2

KVQ_EXPORT int kvq_oracle_quant_rows_int4(const float* x, int64_t rows, int64_t D, float eps,
                                          uint8_t* codes, float* scales) {
  if (!x || !codes || !scales || rows < 0 || D <= 0 || (D & 1)) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * D;
    float amax = 0.0f;
    for (int64_t d = 0; d < D; ++d) {
      float a = fabsf(xr[d]);
      if (a > amax || a != a) amax = a;
    }
    if (amax < eps) amax = eps;
    volatile float scale = amax / 7.0f;
    scales[r] = scale;
    for (int64_t d = 0; d < D; d += 2) {
      unsigned byte = 0;
      for (int j = 0; j < 2; ++j) {
        volatile float qf = scale > 0.0f ? xr[d + j] / scale : 0.0f;
        float rr = nearbyintf(qf);
        if (rr < -8.0f) rr = -8.0f;
        if (rr > 7.0f) rr = 7.0f;
        byte |= ((unsigned)(int)rr & 0xfu) << (4 * j);
      }
      codes[r * (D / 2) + d / 2] = (uint8_t)byte;
    }
  }
  return 0;
}

/* Value of code `d` of a half record whose code bytes start at `codes`. */
static inline double code_at(const uint8_t* codes, int d, int code_type) {
  if (code_type == KVQ_CODE_INT4) {
    const int n = (codes[d >> 1] >> (4 * (d & 1))) & 0xf;
    return (double)(n >= 8 ? n - 16 : n);
  }
  return code_type == KVQ_CODE_FP8 ? (double)e4m3fn_value(codes[d]) : (double)(int8_t)codes[d];
}

/* ---------------------------------------------------------------------------
 * Quantise-on-write into the paged cache.
 * Layout follows vllm_metax/v1/attention/backends/triton_attn.py:318-348
 * (shape), :418-479 (scale views) and :729-739 (K/V views): a (slot, head)
 * record is [K codes (D) | K scale fp32 | V codes (D) | V scale fp32]; the
 * caller passes byte offsets/strides taken from the tensor so NHD and HND
 * physical orders are both covered.  Scatter follows
 * tests/kernels/attention/test_cache.py:326-338 and
 * csrc/libtorch_stable/cache_kernels.cu:321-339 (slot < 0 is padding: skip)
 * and :839-849 (token count comes from slot_mapping, not from key).
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_cache_write_ex(
    const float* key, const float* value, /* [T, Hkv, D] fp32, contiguous */
    uint8_t* cache, int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int64_t* slot_mapping, int64_t T, int Hkv, int D, int block_size,
    float eps, int code_type);

KVQ_EXPORT int kvq_oracle_cache_write(
    const float* key, const float* value, uint8_t* cache, int64_t k_off, int64_t v_off, int64_t ks_off,
    int64_t vs_off, int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int64_t* slot_mapping, int64_t T, int Hkv, int D, int block_size, float eps) {
  return kvq_oracle_cache_write_ex(key, value, cache, k_off, v_off, ks_off, vs_off, stride_block, stride_slot,
                                   stride_head, slot_mapping, T, Hkv, D, block_size, eps, KVQ_CODE_INT8);
}

static int quant_row_any(const float* x, int D, float eps, uint8_t* codes, float* s, int code_type) {
  if (code_type == KVQ_CODE_INT4) return kvq_oracle_quant_rows_int4(x, 1, D, eps, codes, s);
  return code_type == KVQ_CODE_FP8 ? kvq_oracle_quant_rows_fp8(x, 1, D, eps, codes, s)
                                   : kvq_oracle_quant_rows(x, 1, D, eps, (int8_t*)codes, s);
}

KVQ_EXPORT int kvq_oracle_cache_write_ex(
    const float* key, const float* value, /* [T, Hkv, D] fp32, contiguous */
    uint8_t* cache, int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int64_t* slot_mapping, int64_t T, int Hkv, int D, int block_size,
    float eps, int code_type) {
  if (!key || !value || !cache || !slot_mapping) return -1;
  uint8_t* codes = (uint8_t*)malloc((size_t)D);
  if (!codes) return -2;
  for (int64_t t = 0; t < T; ++t) {
    int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    int64_t blk = slot / block_size, off = slot % block_size;
    for (int h = 0; h < Hkv; ++h) {
      uint8_t* rec = cache + blk * stride_block + off * stride_slot + (int64_t)h * stride_head;
      float s;
      const size_t nbytes = code_type == KVQ_CODE_INT4 ? (size_t)D / 2 : (size_t)D;
      quant_row_any(key + (t * Hkv + h) * (int64_t)D, D, eps, codes, &s, code_type);
      memcpy(rec + k_off, codes, nbytes);
      memcpy(rec + ks_off, &s, 4);
      quant_row_any(value + (t * Hkv + h) * (int64_t)D, D, eps, codes, &s, code_type);
      memcpy(rec + v_off, codes, nbytes);
      memcpy(rec + vs_off, &s, 4);
    }
  }
  free(codes);
  return 0;
}

/* One (query row, q head) against keys [k_begin, k_end) of one sequence.
 * Returns unnormalised accumulator acc[D], running max m and sum l.        */
static void attend_range(const float* q, int D, const uint8_t* cache,
                         int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
                         int64_t stride_block, int64_t stride_slot, int64_t stride_head,
                         const int32_t* bt_row, int block_size, int hkv,
                         int64_t k_begin, int64_t k_end, double scale, double softcap,
                         double* acc, double* m_out, double* l_out, double* logits, int code_type,
                         double alibi_slope, int64_t q_pos) {
  double m = -INFINITY;
  for (int64_t j = k_begin; j < k_end; ++j) {
    int64_t blk = bt_row[j / block_size];
    const uint8_t* rec = cache + blk * stride_block + (j % block_size) * stride_slot +
                         (int64_t)hkv * stride_head;
    const uint8_t* kc = rec + k_off;
    float ks;
    memcpy(&ks, rec + ks_off, 4);
    double s = 0.0;
    for (int d = 0; d < D; ++d) s += (double)q[d] * (code_at(kc, d, code_type) * (double)ks);
    s *= scale;
    if (softcap > 0.0) s = softcap * tanh(s / softcap);
    s += alibi_slope * (double)(j - q_pos);   /* ALiBi: after the cap, on the scaled logit; 0 for the query's own key */
    logits[j - k_begin] = s;
    if (s > m) m = s;
  }
  double l = 0.0;
  for (int d = 0; d < D; ++d) acc[d] = 0.0;
  for (int64_t j = k_begin; j < k_end; ++j) {
    int64_t blk = bt_row[j / block_size];
    const uint8_t* rec = cache + blk * stride_block + (j % block_size) * stride_slot +
                         (int64_t)hkv * stride_head;
    const uint8_t* vc = rec + v_off;
    float vs;
    memcpy(&vs, rec + vs_off, 4);
    double p = exp(logits[j - k_begin] - m);
    l += p;
    double pv = p * (double)vs;
    for (int d = 0; d < D; ++d) acc[d] += pv * code_at(vc, d, code_type);
  }
  *m_out = m;
  *l_out = l;
}

/* ---------------------------------------------------------------------------
 * Varlen paged GQA attention over the int8 cache (decode rows, chunked-prefill
 * rows, or a mix).  Follows ref_paged_attn,
 * tests/kernels/attention/test_triton_unified_attention.py:26-78: keys
 * 0..kv_len-1 gathered through block_tables[i, j / block_size], q head h uses
 * kv head h / (Hq/Hkv), bottom-right causal mask
 * triu(diagonal = kv_len - query_len + 1), softmax then P.V.  K and V are
 * dequantised as code * scale (vllm_metax/v1/attention/backends/triton_attn.py:
 * 688-725 passes only the cache and the scale views; new tokens are read back
 * from the cache, :296).  Unlike the as-written test op this keeps every
 * intermediate in double: it is the "fp32-accumulated reference" the kernels
 * are held to.
 *
 * out [N, Hq, D] fp32; lse [N, Hq] fp32 or NULL (natural-log sum-exp of the
 * scaled logits).  Rows with no visible key produce zeros and lse = -inf.
 * ------------------------------------------------------------------------- */
/* window > 0: a query at position p sees keys p - window + 1 .. p only (the
 * sliding_window mask of ref_paged_attn, :60-66).  softcap > 0: scaled logits
 * become softcap * tanh(logit / softcap) before masking (:67-68).           */
/* sinks != NULL: attention sinks, [Hq] fp32.  Head h's softmax gets one more logit, sinks[h] (not scaled), with a
 * zero value row: out = sum_j exp(s_j) v_j / (exp(sinks[h]) + sum_j exp(s_j)), lse = log of that denominator.
 * The definition of the `sinks` argument of upstream's unified_attention, which the reference passes through
 * (vllm_metax/v1/attention/backends/triton_attn.py:712, 784); rows without a visible key stay zeros / -inf.  */
/* alibi_slopes != NULL: ALiBi, [Hq] fp32.  The scaled (and capped) logit of query position p and key position j
 * gets slope[h] * (j - p) added: the bias alibi_slopes * (position_ids - seq_len + 1) of
 * ref_single_query_cached_kv_attention for a decode row (tests/kernels/attention/test_attention.py:109-117, the
 * query standing at seq_len - 1) and `alibi_slope * (token_idx - seq_len + 1)` of the native kernel
 * (csrc/libtorch_stable/attention/attention_kernels.cuh); for a query run, the same with each row's own position.  */
KVQ_EXPORT int kvq_oracle_paged_attn_ex4(
    float* out, float* lse, const float* q, const uint8_t* cache,
    int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
    const int32_t* cu_seqlens_q, int B, int Hq, int Hkv, int D, int block_size,
    float scale, int causal, int window, float softcap, int code_type, const float* sinks,
    const float* alibi_slopes);

KVQ_EXPORT int kvq_oracle_paged_attn_ex3(
    float* out, float* lse, const float* q, const uint8_t* cache,
    int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
    const int32_t* cu_seqlens_q, int B, int Hq, int Hkv, int D, int block_size,
    float scale, int causal, int window, float softcap, int code_type, const float* sinks) {
  return kvq_oracle_paged_attn_ex4(out, lse, q, cache, k_off, v_off, ks_off, vs_off, stride_block, stride_slot,
                                   stride_head, block_table, bt_stride, seq_lens, cu_seqlens_q, B, Hq, Hkv, D,
                                   block_size, scale, causal, window, softcap, code_type, sinks, NULL);
}

KVQ_EXPORT int kvq_oracle_paged_attn_ex2(
    float* out, float* lse, const float* q, const uint8_t* cache,
    int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
    const int32_t* cu_seqlens_q, int B, int Hq, int Hkv, int D, int block_size,
    float scale, int causal, int window, float softcap, int code_type) {
  return kvq_oracle_paged_attn_ex3(out, lse, q, cache, k_off, v_off, ks_off, vs_off, stride_block, stride_slot,
                                   stride_head, block_table, bt_stride, seq_lens, cu_seqlens_q, B, Hq, Hkv, D,
                                   block_size, scale, causal, window, softcap, code_type, NULL);
}

KVQ_EXPORT int kvq_oracle_paged_attn_ex4(
    float* out, float* lse, const float* q, const uint8_t* cache,
    int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
    const int32_t* cu_seqlens_q, int B, int Hq, int Hkv, int D, int block_size,
    float scale, int causal, int window, float softcap, int code_type, const float* sinks,
    const float* alibi_slopes) {
  if (!out || !q || !cache || !block_table || !seq_lens || !cu_seqlens_q) return -1;
  if (Hkv <= 0 || Hq % Hkv != 0) return -1;
  const int G = Hq / Hkv;
  int64_t max_len = 0;
  for (int i = 0; i < B; ++i)
    if (seq_lens[i] > max_len) max_len = seq_lens[i];
  int err = 0;
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)D);
    double* logits = (double*)malloc(sizeof(double) * (size_t)(max_len > 0 ? max_len : 1));
    if (!acc || !logits) {
#pragma omp atomic write
      err = 1;
    } else {
#pragma omp for collapse(2) schedule(dynamic, 1)
      for (int i = 0; i < B; ++i) {
        for (int h = 0; h < Hq; ++h) {
          const int64_t q0 = cu_seqlens_q[i], q1 = cu_seqlens_q[i + 1];
          const int64_t qlen = q1 - q0, kvlen = seq_lens[i];
          for (int64_t r = 0; r < qlen; ++r) {
            int64_t vis = causal ? (kvlen - qlen + r + 1) : kvlen;
            if (vis > kvlen) vis = kvlen;
            int64_t first = 0;
            if (window > 0) {
              first = (kvlen - qlen + r + 1) - window;
              if (first < 0) first = 0;
            }
            float* o = out + ((q0 + r) * Hq + h) * (int64_t)D;
            if (vis <= first) {
              for (int d = 0; d < D; ++d) o[d] = 0.0f;
              if (lse) lse[(q0 + r) * Hq + h] = -INFINITY;
              continue;
            }
            double m, l;
            attend_range(q + ((q0 + r) * Hq + h) * (int64_t)D, D, cache, k_off, v_off,
                         ks_off, vs_off, stride_block, stride_slot, stride_head,
                         block_table + (int64_t)i * bt_stride, block_size, h / G, first, vis,
                         (double)scale, (double)softcap, acc, &m, &l, logits, code_type,
                         alibi_slopes ? (double)alibi_slopes[h] : 0.0, kvlen - qlen + r);
            if (sinks) {   /* one more logit with a zero value row */
              const double sk = (double)sinks[h];
              if (sk > m) {
                const double f = exp(m - sk);
                for (int d = 0; d < D; ++d) acc[d] *= f;
                l = l * f + 1.0;
                m = sk;
              } else {
                l += exp(sk - m);
              }
            }
            for (int d = 0; d < D; ++d) o[d] = (float)(acc[d] / l);
            if (lse) lse[(q0 + r) * Hq + h] = (float)(m + log(l));
          }
        }
      }
    }
    free(acc);
    free(logits);
  }
  return err ? -2 : 0;
}

KVQ_EXPORT int kvq_oracle_paged_attn_ex(
    float* out, float* lse, const float* q, const uint8_t* cache,
    int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
    const int32_t* cu_seqlens_q, int B, int Hq, int Hkv, int D, int block_size,
    float scale, int causal, int window, float softcap) {
  return kvq_oracle_paged_attn_ex2(out, lse, q, cache, k_off, v_off, ks_off, vs_off, stride_block,
                                   stride_slot, stride_head, block_table, bt_stride, seq_lens,
                                   cu_seqlens_q, B, Hq, Hkv, D, block_size, scale, causal, window,
                                   softcap, KVQ_CODE_INT8);
}

KVQ_EXPORT int kvq_oracle_paged_attn(
    float* out, float* lse, const float* q, const uint8_t* cache,
    int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens,
    const int32_t* cu_seqlens_q, int B, int Hq, int Hkv, int D, int block_size,
    float scale, int causal) {
  return kvq_oracle_paged_attn_ex(out, lse, q, cache, k_off, v_off, ks_off, vs_off, stride_block,
                                  stride_slot, stride_head, block_table, bt_stride, seq_lens,
                                  cu_seqlens_q, B, Hq, Hkv, D, block_size, scale, causal, 0, 0.0f);
}

/* ---------------------------------------------------------------------------
 * Split-K, stage 1: decode rows only (one query row per sequence), fixed
 * partitions of `partition_size` tokens.  Contract follows paged_attention_v2,
 * csrc/libtorch_stable/attention/paged_attention_v2.cu:44-96 and
 * attention_kernels.cuh:334-349: partition j covers tokens
 * [j*P, min((j+1)*P, len)) and stores a LOCALLY NORMALISED output
 * tmp_out[b, h, j, :], its max logit and its exp-sum.  (The reference adds
 * 1e-6 to the local sum; the exact form is kept here and the difference sits
 * far inside the tolerance.)  Partitions past the end of a sequence are left
 * untouched.
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_paged_attn_partition(
    float* tmp_out,    /* [B, Hq, max_parts, D] */
    float* max_logits, /* [B, Hq, max_parts]    */
    float* exp_sums,   /* [B, Hq, max_parts]    */
    const float* q,    /* [B, Hq, D]            */
    const uint8_t* cache, int64_t k_off, int64_t v_off, int64_t ks_off, int64_t vs_off,
    int64_t stride_block, int64_t stride_slot, int64_t stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* seq_lens, int B,
    int Hq, int Hkv, int D, int block_size, float scale, int partition_size,
    int max_parts) {
  if (!tmp_out || !max_logits || !exp_sums || !q || !cache) return -1;
  if (Hkv <= 0 || Hq % Hkv != 0 || partition_size <= 0) return -1;
  const int G = Hq / Hkv;
  int err = 0;
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)D);
    double* logits = (double*)malloc(sizeof(double) * (size_t)partition_size);
    if (!acc || !logits) {
#pragma omp atomic write
      err = 1;
    } else {
#pragma omp for collapse(2) schedule(dynamic, 1)
      for (int i = 0; i < B; ++i) {
        for (int h = 0; h < Hq; ++h) {
          int64_t len = seq_lens[i];
          int parts = (int)((len + partition_size - 1) / partition_size);
          if (parts > max_parts) parts = max_parts;
          for (int j = 0; j < parts; ++j) {
            int64_t b0 = (int64_t)j * partition_size;
            int64_t b1 = b0 + partition_size < len ? b0 + partition_size : len;
            double m, l;
            attend_range(q + ((int64_t)i * Hq + h) * D, D, cache, k_off, v_off, ks_off,
                         vs_off, stride_block, stride_slot, stride_head,
                         block_table + (int64_t)i * bt_stride, block_size, h / G, b0, b1,
                         (double)scale, 0.0, acc, &m, &l, logits, KVQ_CODE_INT8, 0.0, 0);
            int64_t idx = ((int64_t)i * Hq + h) * max_parts + j;
            for (int d = 0; d < D; ++d) tmp_out[idx * D + d] = (float)(acc[d] / l);
            max_logits[idx] = (float)m;
            exp_sums[idx] = (float)l;
          }
        }
      }
    }
    free(acc);
    free(logits);
  }
  return err ? -2 : 0;
}

/* ---------------------------------------------------------------------------
 * Split-K, stage 2.  Follows paged_attention_v2_reduce_kernel,
 * csrc/libtorch_stable/attention/attention_kernels.cuh:556-661:
 *   m = max_j m_j;  w_j = l_j * exp(m_j - m);  out = sum_j tmp_out_j w_j / sum_j w_j
 * with a single partition copied through (:573-586).  The reference adds 1e-6
 * to the denominator; the exact form is used here.  Same algebra as the Triton
 * stage 2, vllm_metax/v1/attention/ops/triton_decode_attention.py:582-646.
 * lse (optional) = m + log(sum_j w_j).
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_splitk_reduce(float* out, float* lse, const float* tmp_out,
                                        const float* max_logits, const float* exp_sums,
                                        const int32_t* seq_lens, int B, int Hq, int D,
                                        int partition_size, int max_parts) {
  if (!out || !tmp_out || !max_logits || !exp_sums || !seq_lens) return -1;
  for (int i = 0; i < B; ++i) {
    int64_t len = seq_lens[i];
    int parts = (int)((len + partition_size - 1) / partition_size);
    if (parts > max_parts) parts = max_parts;
    for (int h = 0; h < Hq; ++h) {
      int64_t base = ((int64_t)i * Hq + h) * max_parts;
      float* o = out + ((int64_t)i * Hq + h) * D;
      if (parts <= 0) {
        for (int d = 0; d < D; ++d) o[d] = 0.0f;
        if (lse) lse[(int64_t)i * Hq + h] = -INFINITY;
        continue;
      }
      double m = -INFINITY;
      for (int j = 0; j < parts; ++j)
        if (max_logits[base + j] > m) m = max_logits[base + j];
      double denom = 0.0;
      for (int j = 0; j < parts; ++j)
        denom += (double)exp_sums[base + j] * exp((double)max_logits[base + j] - m);
      for (int d = 0; d < D; ++d) {
        double a = 0.0;
        for (int j = 0; j < parts; ++j)
          a += (double)tmp_out[(base + j) * D + d] * (double)exp_sums[base + j] *
               exp((double)max_logits[base + j] - m);
        o[d] = (float)(a / denom);
      }
      if (lse) lse[(int64_t)i * Hq + h] = (float)(m + log(denom));
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------
 * LSE merge of two partial attention states.  Follows
 * csrc/libtorch_stable/attention/merge_attn_states.cu:93-191 and
 * tests/kernels/attention/test_merge_attn_states.py:17-46: +inf LSE is read as
 * -inf; when both are -inf the prefix output and -inf are emitted; rows at or
 * beyond prefix_num_tokens copy the suffix.
 * outputs [T, H, D]; lse tensors [H, T].
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_merge_attn_states(float* output, float* output_lse,
                                            const float* prefix_output,
                                            const float* prefix_lse,
                                            const float* suffix_output,
                                            const float* suffix_lse, int64_t T, int H,
                                            int D, int64_t prefix_num_tokens) {
  if (!output || !prefix_output || !prefix_lse || !suffix_output || !suffix_lse) return -1;
  for (int64_t t = 0; t < T; ++t) {
    for (int h = 0; h < H; ++h) {
      const float* po = prefix_output + (t * H + h) * (int64_t)D;
      const float* so = suffix_output + (t * H + h) * (int64_t)D;
      float* o = output + (t * H + h) * (int64_t)D;
      if (t >= prefix_num_tokens) {
        for (int d = 0; d < D; ++d) o[d] = so[d];
        if (output_lse) output_lse[(int64_t)h * T + t] = suffix_lse[(int64_t)h * T + t];
        continue;
      }
      double pl = prefix_lse[(int64_t)h * T + t], sl = suffix_lse[(int64_t)h * T + t];
      if (isinf(pl)) pl = -INFINITY;
      if (isinf(sl)) sl = -INFINITY;
      double mx = pl > sl ? pl : sl;
      if (isinf(mx)) {
        for (int d = 0; d < D; ++d) o[d] = po[d];
        if (output_lse) output_lse[(int64_t)h * T + t] = (float)mx;
        continue;
      }
      double pe = exp(pl - mx), se = exp(sl - mx), tot = pe + se;
      for (int d = 0; d < D; ++d)
        o[d] = (float)((double)po[d] * (pe / tot) + (double)so[d] * (se / tot));
      if (output_lse) output_lse[(int64_t)h * T + t] = (float)(log(tot) + mx);
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------
 * MLA latent cache, int8 with one fp32 scale per token.
 * Write side follows concat_and_cache_mla,
 * csrc/libtorch_stable/cache_kernels.cu:397-439,924-985 (kv_c [T, R] and
 * k_pe [T, P] concatenated into one R+P wide row at `slot`, slot < 0
 * skipped), quantised as ONE group over the whole row with the quantiser
 * above.  The reference has no int8 MLA cache; the byte layout is this
 * build's: rows first, scale region after, the convention of the reference's
 * int8 indexer cache (cache_kernels.cu:593-604).  The caller passes byte
 * strides, so the oracle does not depend on that choice:
 *   codes of (block, off): cache + block*stride_block + off*stride_row
 *   scale of (block, off): cache + block*stride_block + scale_off + off*4
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_mla_cache_write(const float* kv_c, const float* k_pe,
                                          uint8_t* cache, int64_t stride_block,
                                          int64_t stride_row, int64_t scale_off,
                                          const int64_t* slot_mapping, int64_t T, int R,
                                          int P, int block_size, float eps) {
  if (!kv_c || !k_pe || !cache || !slot_mapping) return -1;
  const int W = R + P;
  float* row = (float*)malloc(sizeof(float) * (size_t)W);
  int8_t* codes = (int8_t*)malloc((size_t)W);
  if (!row || !codes) {
    free(row);
    free(codes);
    return -2;
  }
  for (int64_t t = 0; t < T; ++t) {
    int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    int64_t blk = slot / block_size, off = slot % block_size;
    memcpy(row, kv_c + t * R, sizeof(float) * (size_t)R);
    memcpy(row + R, k_pe + t * P, sizeof(float) * (size_t)P);
    float s;
    kvq_oracle_quant_rows(row, 1, W, eps, codes, &s);
    memcpy(cache + blk * stride_block + off * stride_row, codes, (size_t)W);
    memcpy(cache + blk * stride_block + scale_off + off * 4, &s, 4);
  }
  free(row);
  free(codes);
  return 0;
}

/* ---------------------------------------------------------------------------
 * MLA decode (MQA over one latent stream).  Follows ref_mla,
 * tests/kernels/attention/test_mla_decode_cpu.py:14-41 and the fp32 + lse
 * reference in tests/kernels/attention/test_flashmla.py:114-153:
 *   s_j = scale * q . c_j   (all W = R + P dims),  o = softmax(s) . c[:, :R]
 * with c_j = code_j * scale_j.  out [B, H, R] fp32, lse [B, H] (may be NULL).
 * Same entry-point contract as TritonMLAImpl.forward_mqa,
 * vllm_metax/v1/attention/backends/mla/triton_mla.py:226-295.
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_mla_decode(float* out, float* lse, const float* q,
                                     const uint8_t* cache, int64_t stride_block,
                                     int64_t stride_row, int64_t scale_off,
                                     const int32_t* block_table, int64_t bt_stride,
                                     const int32_t* seq_lens, int B, int H, int R, int P,
                                     int block_size, float scale) {
  if (!out || !q || !cache || !block_table || !seq_lens) return -1;
  const int W = R + P;
  int64_t max_len = 0;
  for (int i = 0; i < B; ++i)
    if (seq_lens[i] > max_len) max_len = seq_lens[i];
  int err = 0;
#pragma omp parallel
  {
    double* logits = (double*)malloc(sizeof(double) * (size_t)(max_len > 0 ? max_len : 1));
    double* acc = (double*)malloc(sizeof(double) * (size_t)R);
    if (!logits || !acc) {
#pragma omp atomic write
      err = 1;
    } else {
#pragma omp for collapse(2) schedule(dynamic, 1)
      for (int i = 0; i < B; ++i) {
        for (int h = 0; h < H; ++h) {
          int64_t len = seq_lens[i];
          const int32_t* bt = block_table + (int64_t)i * bt_stride;
          const float* qr = q + ((int64_t)i * H + h) * W;
          float* o = out + ((int64_t)i * H + h) * R;
          if (len <= 0) {
            for (int d = 0; d < R; ++d) o[d] = 0.0f;
            if (lse) lse[(int64_t)i * H + h] = -INFINITY;
            continue;
          }
          double m = -INFINITY;
          for (int64_t j = 0; j < len; ++j) {
            const uint8_t* blk = cache + (int64_t)bt[j / block_size] * stride_block;
            const int8_t* c = (const int8_t*)(blk + (j % block_size) * stride_row);
            float cs;
            memcpy(&cs, blk + scale_off + (j % block_size) * 4, 4);
            double s = 0.0;
            for (int d = 0; d < W; ++d) s += (double)qr[d] * ((double)c[d] * (double)cs);
            s *= (double)scale;
            logits[j] = s;
            if (s > m) m = s;
          }
          double l = 0.0;
          for (int d = 0; d < R; ++d) acc[d] = 0.0;
          for (int64_t j = 0; j < len; ++j) {
            const uint8_t* blk = cache + (int64_t)bt[j / block_size] * stride_block;
            const int8_t* c = (const int8_t*)(blk + (j % block_size) * stride_row);
            float cs;
            memcpy(&cs, blk + scale_off + (j % block_size) * 4, 4);
            double p = exp(logits[j] - m);
            l += p;
            double pc = p * (double)cs;
            for (int d = 0; d < R; ++d) acc[d] += pc * (double)c[d];
          }
          for (int d = 0; d < R; ++d) o[d] = (float)(acc[d] / l);
          if (lse) lse[(int64_t)i * H + h] = (float)(m + log(l));
        }
      }
    }
    free(logits);
    free(acc);
  }
  return err ? -2 : 0;
}

KVQ_EXPORT int kvq_oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}


/* ---------------------------------------------------------------------------
 * Gather + dequantise rows of the int8 latent cache into a dense workspace:
 * the int8 branch of gather_and_maybe_dequant_cache,
 * csrc/libtorch_stable/cache_kernels.cu:1072-1131 (one destination row per
 * token: batch = token_to_seq[token], position = token - cu_seq_lens[batch]
 * + seq_starts[batch], block = block_table[batch, position / block_size],
 * slot = position % block_size), used by the MLA chunked-context prefill
 * (vllm_metax/model_executor/layers/attention/mla_attention.py:2017-2140).
 * The reference converts with one per-tensor scale; here every row carries its
 * own: dst[token, d] = (float)code * scale_of_row, one fp32 rounding.
 * dst is fp32 [num_tokens, dst_stride]; the caller rounds to the output type.
 * ------------------------------------------------------------------------- */
KVQ_EXPORT int kvq_oracle_mla_gather_dequant(float* dst, int64_t dst_stride, const uint8_t* cache,
                                             int64_t stride_block, int64_t stride_row, int64_t scale_off,
                                             const int32_t* block_table, int64_t bt_stride,
                                             const int32_t* cu_seq_lens, const int32_t* token_to_seq,
                                             const int32_t* seq_starts, int num_tokens, int width,
                                             int block_size) {
  if (!dst || !cache || !block_table || !cu_seq_lens || !token_to_seq) return -1;
  for (int t = 0; t < num_tokens; ++t) {
    const int b = token_to_seq[t];
    if (t >= cu_seq_lens[b + 1]) continue;
    int pos = t - cu_seq_lens[b];
    if (seq_starts) pos += seq_starts[b];
    const int64_t blk = block_table[(int64_t)b * bt_stride + pos / block_size];
    const int off = pos % block_size;
    const int8_t* row = (const int8_t*)(cache + blk * stride_block + (int64_t)off * stride_row);
    float scale;
    memcpy(&scale, cache + blk * stride_block + scale_off + (int64_t)off * 4, 4);
    for (int d = 0; d < width; ++d) dst[(int64_t)t * dst_stride + d] = (float)row[d] * scale;
  }
  return 0;
}
