// Block moves over the paged int8 cache (gfx950): swap-in / swap-out / in-device copies of whole
// cache blocks.  A block of this layout carries its codes AND their fp32 scales, so moving
// `block_bytes` moves a self-contained unit: no scale tensor to keep in step.
//
// Device-to-device moves are ONE kernel launch per 128 pairs (the pairs travel in the kernel
// arguments, 16-byte lane copies, one workgroup per 16 KB slice of a block) instead of one
// memcpy call per block; moves to or from the host are one asynchronous copy per block on the
// caller's stream, as in the reference (csrc/libtorch_stable/cache_kernels.cu:33-77).
#include "kvq_internal.h"

namespace kvq {

constexpr int kPairsPerLaunch = 128;
constexpr int kSliceBytes = 16384;  // bytes one workgroup moves

struct BlockPairs {
  int64_t src[kPairsPerLaunch];
  int64_t dst[kPairsPerLaunch];
};

// grid (slices per block, pairs); 256 threads, each moving 16 bytes per step.
__global__ __launch_bounds__(256) void move_blocks_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                          int64_t block_bytes, BlockPairs pairs) {
  const int64_t s_off = pairs.src[blockIdx.y] * block_bytes;
  const int64_t d_off = pairs.dst[blockIdx.y] * block_bytes;
  const int64_t begin = (int64_t)blockIdx.x * kSliceBytes;
  const int64_t end = begin + kSliceBytes < block_bytes ? begin + kSliceBytes : block_bytes;
  const u32x4* s = reinterpret_cast<const u32x4*>(src + s_off + begin);
  u32x4* d = reinterpret_cast<u32x4*>(dst + d_off + begin);
  const int n = (int)((end - begin) / 16);
  for (int i = threadIdx.x; i < n; i += 256) d[i] = s[i];
}

// Arbitrary (src pointer, dst pointer, size) triples, all on the device: grid (slices, entries).
struct CopyTriples {
  int64_t src[kPairsPerLaunch / 2];
  int64_t dst[kPairsPerLaunch / 2];
  int64_t size[kPairsPerLaunch / 2];
};

__global__ __launch_bounds__(256) void copy_triples_kernel(CopyTriples t) {
  const uint8_t* s = reinterpret_cast<const uint8_t*>(t.src[blockIdx.y]);
  uint8_t* d = reinterpret_cast<uint8_t*>(t.dst[blockIdx.y]);
  const int64_t size = t.size[blockIdx.y];
  for (int64_t begin = (int64_t)blockIdx.x * kSliceBytes; begin < size; begin += (int64_t)gridDim.x * kSliceBytes) {
    const int64_t end = begin + kSliceBytes < size ? begin + kSliceBytes : size;
    if (((reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d) | (uintptr_t)size) & 15) == 0) {
      const u32x4* sv = reinterpret_cast<const u32x4*>(s + begin);
      u32x4* dv = reinterpret_cast<u32x4*>(d + begin);
      const int n = (int)((end - begin) / 16);
      for (int i = threadIdx.x; i < n; i += 256) dv[i] = sv[i];
    } else {
      for (int64_t i = begin + threadIdx.x; i < end; i += 256) d[i] = s[i];
    }
  }
}

// copy_blocks: every (src, dst) pair of a device-resident mapping, in every layer's cache, in one
// launch: grid (slices per block, pairs, layers).  num_blocks bounds the block numbers read from the
// mapping (a pair outside it is skipped: the host cannot see the mapping without a synchronisation).
__global__ __launch_bounds__(256) void copy_blocks_kernel(const int64_t* __restrict__ cache_ptrs,
                                                          const int64_t* __restrict__ block_mapping,
                                                          int64_t block_bytes, int64_t num_blocks, int vec16) {
  uint8_t* cache = reinterpret_cast<uint8_t*>(cache_ptrs[blockIdx.z]);
  const int64_t src = block_mapping[2 * (int64_t)blockIdx.y], dst = block_mapping[2 * (int64_t)blockIdx.y + 1];
  if (src < 0 || dst < 0 || src >= num_blocks || dst >= num_blocks || src == dst) return;
  const int64_t begin = (int64_t)blockIdx.x * kSliceBytes;
  const int64_t end = begin + kSliceBytes < block_bytes ? begin + kSliceBytes : block_bytes;
  const uint8_t* s = cache + src * block_bytes + begin;
  uint8_t* d = cache + dst * block_bytes + begin;
  if (vec16 && ((reinterpret_cast<uintptr_t>(cache) & 15) == 0)) {
    const int n = (int)((end - begin) / 16);
    for (int i = threadIdx.x; i < n; i += 256) reinterpret_cast<u32x4*>(d)[i] = reinterpret_cast<const u32x4*>(s)[i];
  } else {
    for (int64_t i = threadIdx.x; i < end - begin; i += 256) d[i] = s[i];
  }
}

}  // namespace kvq

extern "C" {

int kvq_copy_blocks(const int64_t* cache_ptrs, int num_layers, const int64_t* block_mapping, int64_t num_pairs,
                    int64_t block_bytes, int64_t num_blocks, kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "copy_blocks";
  KVQ_REQUIRE(num_layers >= 0 && num_pairs >= 0, "%s: negative count", op);
  if (num_layers == 0 || num_pairs == 0) return KVQ_OK;
  KVQ_REQUIRE(cache_ptrs && block_mapping, "%s: NULL pointer", op);
  KVQ_REQUIRE(block_bytes > 0 && num_blocks > 0, "%s: block_bytes and num_blocks must be positive", op);
  KVQ_REQUIRE(num_layers <= 65535 && num_pairs <= 65535, "%s: at most 65535 layers and 65535 pairs per call", op);
  const int64_t slices = (block_bytes + kSliceBytes - 1) / kSliceBytes;
  KVQ_REQUIRE(slices <= 0x7fffffff, "%s: block_bytes out of range", op);
  hipLaunchKernelGGL(copy_blocks_kernel, dim3((unsigned)slices, (unsigned)num_pairs, (unsigned)num_layers), dim3(256), 0,
                     as_stream(stream), cache_ptrs, block_mapping, block_bytes, num_blocks, block_bytes % 16 == 0 ? 1 : 0);
  return check_hip(hipGetLastError(), "copy_blocks launch");
}

int kvq_swap_blocks(const void* src, void* dst, int64_t block_bytes, const int64_t* block_mapping,
                    int64_t num_pairs, int64_t map_stride0, int64_t map_stride1, int direction,
                    kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "swap_blocks";
  KVQ_REQUIRE(num_pairs >= 0, "%s: negative number of pairs", op);
  if (num_pairs == 0) return KVQ_OK;
  KVQ_REQUIRE(src && dst && block_mapping, "%s: NULL pointer", op);
  KVQ_REQUIRE(block_bytes > 0, "%s: block_bytes must be positive", op);
  KVQ_REQUIRE(direction == KVQ_DEVICE_TO_DEVICE || direction == KVQ_DEVICE_TO_HOST || direction == KVQ_HOST_TO_DEVICE,
              "%s: unknown direction %d", op, direction);
  hipStream_t s = as_stream(stream);
  for (int64_t i = 0; i < num_pairs; ++i)
    KVQ_REQUIRE(block_mapping[i * map_stride0] >= 0 && block_mapping[i * map_stride0 + map_stride1] >= 0,
                "%s: negative block number in pair %lld", op, (long long)i);
  if (direction == KVQ_DEVICE_TO_DEVICE && block_bytes % 16 == 0 && ((uintptr_t)src % 16) == 0 &&
      ((uintptr_t)dst % 16) == 0) {
    const int64_t slices = (block_bytes + kSliceBytes - 1) / kSliceBytes;
    KVQ_REQUIRE(slices <= 0x7fffffff, "%s: block_bytes out of range", op);
    for (int64_t base = 0; base < num_pairs; base += kPairsPerLaunch) {
      BlockPairs p{};
      const int n = (int)(num_pairs - base < kPairsPerLaunch ? num_pairs - base : kPairsPerLaunch);
      for (int i = 0; i < n; ++i) {
        p.src[i] = block_mapping[(base + i) * map_stride0];
        p.dst[i] = block_mapping[(base + i) * map_stride0 + map_stride1];
      }
      hipLaunchKernelGGL(move_blocks_kernel, dim3((unsigned)slices, (unsigned)n), dim3(256), 0, s,
                         static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), block_bytes, p);
      if (int rc = check_hip(hipGetLastError(), "swap_blocks launch")) return rc;
    }
    return KVQ_OK;
  }
  const hipMemcpyKind kind = direction == KVQ_DEVICE_TO_DEVICE ? hipMemcpyDeviceToDevice
                             : direction == KVQ_DEVICE_TO_HOST ? hipMemcpyDeviceToHost
                                                               : hipMemcpyHostToDevice;
  for (int64_t i = 0; i < num_pairs; ++i) {
    const int64_t sb = block_mapping[i * map_stride0], db = block_mapping[i * map_stride0 + map_stride1];
    if (int rc = check_hip(hipMemcpyAsync(static_cast<uint8_t*>(dst) + db * block_bytes,
                                          static_cast<const uint8_t*>(src) + sb * block_bytes, (size_t)block_bytes,
                                          kind, s),
                           "swap_blocks copy"))
      return rc;
  }
  return KVQ_OK;
}

int kvq_swap_blocks_batch(const int64_t* src_ptrs, const int64_t* dst_ptrs, const int64_t* sizes, int64_t n,
                          int all_on_device, kvq_stream_t stream) {
  using namespace kvq;
  const char* op = "swap_blocks_batch";
  KVQ_REQUIRE(n >= 0, "%s: negative length", op);
  if (n == 0) return KVQ_OK;
  KVQ_REQUIRE(src_ptrs && dst_ptrs && sizes, "%s: NULL pointer", op);
  for (int64_t i = 0; i < n; ++i)
    KVQ_REQUIRE(sizes[i] >= 0 && (sizes[i] == 0 || (src_ptrs[i] != 0 && dst_ptrs[i] != 0)),
                "%s: entry %lld has a NULL pointer or a negative size", op, (long long)i);
  hipStream_t s = as_stream(stream);
  if (all_on_device) {
    constexpr int kPer = kPairsPerLaunch / 2;
    for (int64_t base = 0; base < n; base += kPer) {
      CopyTriples t{};
      const int m = (int)(n - base < kPer ? n - base : kPer);
      int64_t largest = 0;
      for (int i = 0; i < m; ++i) {
        t.src[i] = src_ptrs[base + i];
        t.dst[i] = dst_ptrs[base + i];
        t.size[i] = sizes[base + i];
        largest = sizes[base + i] > largest ? sizes[base + i] : largest;
      }
      if (largest == 0) continue;
      int64_t slices = (largest + kSliceBytes - 1) / kSliceBytes;
      slices = slices > 4096 ? 4096 : slices;  // longer entries loop inside the kernel
      hipLaunchKernelGGL(copy_triples_kernel, dim3((unsigned)slices, (unsigned)m), dim3(256), 0, s, t);
      if (int rc = check_hip(hipGetLastError(), "swap_blocks_batch launch")) return rc;
    }
    return KVQ_OK;
  }
  for (int64_t i = 0; i < n; ++i) {
    if (sizes[i] == 0) continue;
    if (int rc = check_hip(hipMemcpyAsync(reinterpret_cast<void*>(dst_ptrs[i]), reinterpret_cast<const void*>(src_ptrs[i]),
                                          (size_t)sizes[i], hipMemcpyDefault, s),
                           "swap_blocks_batch copy"))
      return rc;
  }
  return KVQ_OK;
}

}  // extern "C"
