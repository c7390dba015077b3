// MLA latent cache: int8 quantise-on-write and decode (placeholder until the kernels land).
#include "kvq_internal.h"

extern "C" {

int kvq_concat_and_cache_mla_int8(const void*, const void*, int, int64_t, int64_t, void*, const kvq_mla_geom*,
                                  const int64_t*, int64_t, float, kvq_stream_t) {
  return kvq::fail(KVQ_ENOSYS, "concat_and_cache_mla_int8: not built yet");
}

size_t kvq_mla_decode_workspace_bytes(int, int, int) { return 0; }

int kvq_mla_decode_int8(void*, int, float*, const void*, int, int64_t, int64_t, const void*, const kvq_mla_geom*,
                        const int32_t*, int64_t, const int32_t*, int, int, float, void*, size_t, kvq_stream_t) {
  return kvq::fail(KVQ_ENOSYS, "mla_decode_int8: not built yet");
}

int kvq_merge_attn_states(void*, float*, const void*, const float*, const void*, const float*, int, int64_t, int,
                          int, int64_t, kvq_stream_t) {
  return kvq::fail(KVQ_ENOSYS, "merge_attn_states: not built yet");
}

}  // extern "C"
