// Chunked-prefill MFMA tile over the int8 cache (placeholder until the tile lands).
#include "kvq_attn_core.cuh"

namespace kvq {

int launch_prefill(const AttnIO& io, const int32_t* seq_lens, const int32_t* cu_seqlens_q, int num_seqs,
                   int max_query_len, int causal, int q_dtype, int out_dtype, hipStream_t s) {
  (void)io; (void)seq_lens; (void)cu_seqlens_q; (void)num_seqs; (void)max_query_len; (void)causal;
  (void)q_dtype; (void)out_dtype; (void)s;
  return fail(KVQ_ENOSYS, "paged_attn_int8: query runs longer than one token are not built yet");
}

}  // namespace kvq
