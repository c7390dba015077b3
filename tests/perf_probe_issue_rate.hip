// Timing program, not a test: how fast ONE wave issues the instruction kinds the MLA decode tiles are made of,
// at one, two and four waves per SIMD (256, 512 and 1024 threads per workgroup, one workgroup per CU).
//
//   hipcc --offload-arch=gfx950 -O3 tests/perf_probe_issue_rate.hip -o /tmp/issue_rate && /tmp/issue_rate
//
// Every kernel runs a loop whose body is 16 copies of four independent instructions of one kind (mode 4: of four
// MFMAs, each followed by eight vector instructions), so that the loop's own scalar instructions do not count, and
// is timed with events; the figure printed is wall time per instruction per wave.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

template <int MODE>
__global__ __launch_bounds__(1024) void issue_loop(int n, uint32_t seed, uint32_t* sink) {
  i32x4 acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
  floatx4 facc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
  const i32x4 a = {(int)seed, (int)threadIdx.x, 3, 4}, b = {5, 6, (int)seed, 8};
  const uint32_t x = seed * 3 + threadIdx.x, y = seed, z = 0x05010400u;
  uint32_t r0 = 0, r1 = 0, r2 = 0, r3 = 0;
  for (int i = 0; i < n; ++i) {
#pragma unroll
   for (int rep = 0; rep < 16; ++rep) {
    if (MODE == 0) {
      asm volatile("v_perm_b32 %0, %4, %5, %6\nv_perm_b32 %1, %4, %5, %6\nv_perm_b32 %2, %4, %5, %6\nv_perm_b32 %3, %4, %5, %6\n"
                   : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(x), "v"(y), "v"(z));
    } else if (MODE == 1) {
      asm volatile("v_cvt_f16_i16_sdwa %0, sext(%4) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0\n"
                   "v_cvt_f16_i16_sdwa %1, sext(%4) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_1\n"
                   "v_cvt_f16_i16_sdwa %2, sext(%4) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2\n"
                   "v_cvt_f16_i16_sdwa %3, sext(%4) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_3\n"
                   : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(x));
    } else if (MODE == 2) {
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[j], 0, 0, 0);
    } else if (MODE == 3) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        facc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), facc[j], 0, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        facc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), facc[j], 0, 0, 0);
        asm volatile("v_perm_b32 %0, %4, %5, %6\nv_perm_b32 %1, %4, %5, %6\nv_perm_b32 %2, %4, %5, %6\nv_perm_b32 %3, %4, %5, %6\n"
                     "v_perm_b32 %0, %4, %5, %6\nv_perm_b32 %1, %4, %5, %6\nv_perm_b32 %2, %4, %5, %6\nv_perm_b32 %3, %4, %5, %6\n"
                     : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(x), "v"(y), "v"(z));
      }
    }
   }
  }
  uint32_t s = r0 ^ r1 ^ r2 ^ r3;
  for (int j = 0; j < 4; ++j) s ^= acc[j].x ^ acc[j].y ^ (uint32_t)facc[j].x ^ (uint32_t)facc[j].w;
  if (s == 0x1234567u) sink[0] = s;   // never true for the seed used; keeps the loop
}

int main() {
  const int n = 1 << 12;
  int cus = 0;
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0);
  uint32_t* sink;
  if (hipMalloc(&sink, 4) != hipSuccess) return 1;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  const char* names[] = {"v_perm_b32", "v_cvt_f16_i16 (sub-dword operand)", "v_mfma_i32_16x16x64_i8", "v_mfma_f32_16x16x32_f16",
                         "v_mfma_f32_16x16x32_f16 + 8 v_perm_b32"};
  void (*kernels[])(int, uint32_t, uint32_t*) = {issue_loop<0>, issue_loop<1>, issue_loop<2>, issue_loop<3>, issue_loop<4>};
  for (int threads : {256, 512, 1024}) {
    printf("%d waves per SIMD\n", threads / 256);
    for (int m = 0; m < 5; ++m) {
      hipLaunchKernelGGL(kernels[m], dim3(cus), dim3(threads), 0, 0, 64, 1u, sink);   // warm-up
      (void)hipDeviceSynchronize();
      (void)hipEventRecord(e0);
      hipLaunchKernelGGL(kernels[m], dim3(cus), dim3(threads), 0, 0, n, 1u, sink);
      (void)hipEventRecord(e1);
      (void)hipEventSynchronize(e1);
      float ms = 0.f;
      (void)hipEventElapsedTime(&ms, e0, e1);
      printf("  %-42s %.2f ns per %s per wave\n", names[m], ms * 1e6 / ((double)n * 64), m == 4 ? "MFMA + 8 v_perm" : "instruction");
      fflush(stdout);
    }
  }
  return 0;
}
