// Yardsticks for bench.py, not part of the GEMM library: what a kernel launch costs
// and how fast the chip streams a matrix's worth of bytes when nothing is computed.
//   * floor_empty_kernel: no work at all; as a node of a HIP graph it is the cost of a launch.
//   * floor_stream_kernel: every wavefront of every workgroup copies its share of a buffer
//     into LDS with the same asynchronous 1-KiB copies the decode kernel uses for its weights
//     (global_load_lds_dwordx4, 16 slots per wavefront reused round-robin, nothing waits for a
//     slot because nothing reads the data) and waits for the last copy.
//   * floor_stream_reg_kernel: the same bytes through plain 16-byte loads into registers
//     (global_load_dwordx4), eight wavefronts per SIMD (two workgroups of 1024 threads per
//     compute unit), eight loads in flight per wavefront; with NT the loads carry the
//     non-temporal bit.  Says whether the ceiling above belongs to the chip or to the copy path.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void glb_void_t;

__global__ __launch_bounds__(512) void floor_empty_kernel() {}

template <int AUX>   // 0: plain copies, 2: with the non-temporal bit
__global__ __launch_bounds__(512) void floor_stream_kernel(const uint4* __restrict__ src, long kib_per_workgroup) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  char* ring = smem + wave * 16384;
  const uint4* base = src + (long)blockIdx.x * kib_per_workgroup * 64 + lane;
  int slot = 0;
  for (long i = wave; i < kib_per_workgroup; i += 8) {
    __builtin_amdgcn_global_load_lds((glb_void_t*)(base + i * 64), (lds_void_t*)(ring + (slot & 15) * 1024), 16, 0, AUX);
    ++slot;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <bool NT>
__device__ __forceinline__ uint4 load16(const uint4* p) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  if constexpr (NT) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
  } else {
    return *p;
  }
}

template <bool NT>
__global__ __launch_bounds__(1024) void floor_stream_reg_kernel(const uint4* __restrict__ src,
                                                               long kib_per_workgroup, uint4* sink) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const uint4* base = src + (long)blockIdx.x * kib_per_workgroup * 64 + lane;
  uint4 acc = make_uint4(0u, 0u, 0u, 0u);
  long i = wave;
  for (; i + 7 * 16 < kib_per_workgroup; i += 8 * 16) {
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = load16<NT>(base + (i + 16 * u) * 64);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      acc.x ^= v[u].x;
      acc.y ^= v[u].y;
      acc.z ^= v[u].z;
      acc.w ^= v[u].w;
    }
  }
  for (; i < kib_per_workgroup; i += 16) {
    const uint4 v = load16<NT>(base + i * 64);
    acc.x ^= v.x;
    acc.y ^= v.y;
    acc.z ^= v.z;
    acc.w ^= v.w;
  }
  // keeps the loads alive; true for about one lane in four billion
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) *sink = acc;
}

}  // namespace

// One empty kernel of `workgroups` x 512 threads on `stream`.
extern "C" int sonar_bench_empty(int workgroups, void* stream) {
  if (workgroups < 1) return 1;
  floor_empty_kernel<<<workgroups, 512, 0, (hipStream_t)stream>>>();
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// Streams the first `bytes` bytes of `src` (rounded down to workgroups x 1 KiB) through LDS
// with `workgroups` x 512 threads on `stream`; `non_temporal`: the copies carry that bit.
extern "C" int sonar_bench_stream(const void* src, size_t bytes, int workgroups, int non_temporal, void* stream) {
  if (workgroups < 1 || src == nullptr || ((uintptr_t)src) % 16 != 0) return 1;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)floor_stream_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) !=
            hipSuccess ||
        hipFuncSetAttribute((const void*)floor_stream_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) !=
            hipSuccess)
      return 2;
    attr_set = true;
  }
  const long kib = (long)(bytes / 1024 / workgroups);
  if (kib < 1) return 1;
  if (non_temporal)
    floor_stream_kernel<2><<<workgroups, 512, 131072, (hipStream_t)stream>>>(static_cast<const uint4*>(src), kib);
  else
    floor_stream_kernel<0><<<workgroups, 512, 131072, (hipStream_t)stream>>>(static_cast<const uint4*>(src), kib);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// The same bytes through register loads with `workgroups` x 1024 threads; `sink` is 16 bytes
// of device memory that a lane may write.
extern "C" int sonar_bench_stream_reg(const void* src, size_t bytes, int workgroups, int non_temporal, void* sink,
                                      void* stream) {
  if (workgroups < 1 || src == nullptr || sink == nullptr || ((uintptr_t)src) % 16 != 0 || ((uintptr_t)sink) % 16 != 0)
    return 1;
  const long kib = (long)(bytes / 1024 / workgroups);
  if (kib < 1) return 1;
  if (non_temporal)
    floor_stream_reg_kernel<true><<<workgroups, 1024, 0, (hipStream_t)stream>>>(static_cast<const uint4*>(src), kib,
                                                                                 static_cast<uint4*>(sink));
  else
    floor_stream_reg_kernel<false><<<workgroups, 1024, 0, (hipStream_t)stream>>>(static_cast<const uint4*>(src), kib,
                                                                                  static_cast<uint4*>(sink));
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
