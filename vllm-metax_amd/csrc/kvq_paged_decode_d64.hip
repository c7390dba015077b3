// Paged decode kernels for head size 64.
#include "kvq_paged_decode_impl.cuh"

namespace kvq {
template int launch_streamk_q<64>(const StreamKArgs& a, int q_dtype, int out_dtype, hipStream_t s);
template int launch_v2_q<64>(const V2Args& a, int num_seqs, int q_dtype, hipStream_t s);
}  // namespace kvq
