// Yardsticks for bench.py, not part of the GEMM library: what a kernel launch costs
// and how fast the chip streams a matrix's worth of bytes when nothing is computed.
//   * floor_empty_kernel: no work at all; as a node of a HIP graph it is the cost of a launch.
//   * floor_stream_kernel: every wavefront of every workgroup copies its share of a buffer
//     into LDS with the same asynchronous 1-KiB copies the decode kernel uses for its weights
//     (global_load_lds_dwordx4, 16 slots per wavefront reused round-robin, nothing waits for a
//     slot because nothing reads the data) and waits for the last copy.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void glb_void_t;

__global__ __launch_bounds__(512) void floor_empty_kernel() {}

__global__ __launch_bounds__(512) void floor_stream_kernel(const uint4* __restrict__ src, long kib_per_workgroup) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  char* ring = smem + wave * 16384;
  const uint4* base = src + (long)blockIdx.x * kib_per_workgroup * 64 + lane;
  int slot = 0;
  for (long i = wave; i < kib_per_workgroup; i += 8) {
    __builtin_amdgcn_global_load_lds((glb_void_t*)(base + i * 64), (lds_void_t*)(ring + (slot & 15) * 1024), 16, 0, 0);
    ++slot;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace

// One empty kernel of `workgroups` x 512 threads on `stream`.
extern "C" int sonar_bench_empty(int workgroups, void* stream) {
  if (workgroups < 1) return 1;
  floor_empty_kernel<<<workgroups, 512, 0, (hipStream_t)stream>>>();
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// Streams the first `bytes` bytes of `src` (rounded down to workgroups x 1 KiB) through LDS
// with `workgroups` x 512 threads on `stream`.
extern "C" int sonar_bench_stream(const void* src, size_t bytes, int workgroups, void* stream) {
  if (workgroups < 1 || src == nullptr || ((uintptr_t)src) % 16 != 0) return 1;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)floor_stream_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) !=
        hipSuccess)
      return 2;
    attr_set = true;
  }
  const long kib = (long)(bytes / 1024 / workgroups);
  if (kib < 1) return 1;
  floor_stream_kernel<<<workgroups, 512, 131072, (hipStream_t)stream>>>(static_cast<const uint4*>(src), kib);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
