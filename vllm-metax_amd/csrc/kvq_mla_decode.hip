// MLA decode over the int8 latent cache (placeholder until the MFMA tile lands).
#include "kvq_internal.h"

extern "C" {

size_t kvq_mla_decode_workspace_bytes(int, int, int) { return 0; }

int kvq_mla_decode_int8(void*, int, float*, const void*, int, int64_t, int64_t, const void*, const kvq_mla_geom*,
                        const int32_t*, int64_t, const int32_t*, int, int, float, void*, size_t, kvq_stream_t) {
  return kvq::fail(KVQ_ENOSYS, "mla_decode_int8: not built yet");
}

}  // extern "C"
