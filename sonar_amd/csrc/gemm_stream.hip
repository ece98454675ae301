// Streaming W4A16 GEMM for up to 64 activation rows per launch.
//
// Work decomposition.  The packed weights are a list of strips (64 output
// columns each), every strip a contiguous run of K/32 one-KiB chunks.  The list
// of all (strip, unit) pairs - a unit is `unit_chunks` consecutive chunks - is
// cut into equal contiguous ranges, one per workgroup, so every compute unit
// streams the same number of bytes whatever the shape.  A workgroup walks its
// range strip by strip.  Inside a strip segment its eight wavefronts take
// units round-robin, so the workgroup reads memory front to back; each
// wavefront keeps MB x 4 accumulator tiles (16 rows x 16 columns each) and
// feeds v_mfma_f32_16x16x32 with the weights as the row operand and the
// activations as the column operand.  The eight partial tiles are summed
// through LDS.  A segment that covers the whole K of its strip is written
// straight to C.  Otherwise the partial tile goes to scratch memory and a
// counter in `workspace` (indexed by the first workgroup that touches the
// strip) is incremented; the workgroup that brings it to the number of
// contributors adds the partials in a fixed order, writes C and puts the
// counter back to zero.  The result does not depend on arrival order.
#include "dequant.hpp"

namespace sonar {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kSlotFloat4 = 4 * 4 * 64;  // largest partial tile: 4 row blocks x 4 column blocks x 64 lanes

struct StreamParams {
  const uint16_t* a;
  long lda;
  uint16_t* c;
  const uint4* b;
  const uint16_t* bias;
  const uint16_t* scales;
  const uint32_t* zeros;
  const int32_t* g_idx;
  const int32_t* perm;
  int32_t* workspace;
  float4* scratch;
  int size_m, size_n, size_k;
  int num_groups, group_size;
  int chunks_per_strip;
  int unit_chunks;
  int units_per_strip;
  long total_units;
};

__device__ __forceinline__ long range_begin(long i, long total, long parts) { return i * total / parts; }
// Largest i with range_begin(i) <= x, given parts <= total.
__device__ __forceinline__ int range_owner(long x, long total, long parts) {
  return (int)(((x + 1) * parts - 1) / total);
}

template <typename T, bool HAS_PERM>
__device__ __forceinline__ typename Dq<T>::vec8 load_a(const StreamParams& p, int row, int k0) {
  typedef typename Dq<T>::vec8 vec8;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (row < p.size_m) {
    const uint16_t* arow = p.a + (long)row * p.lda;
    if (!HAS_PERM) {
      v = *reinterpret_cast<const uint4*>(arow + k0);
    } else {
      const int4 p0 = *reinterpret_cast<const int4*>(p.perm + k0);
      const int4 p1 = *reinterpret_cast<const int4*>(p.perm + k0 + 4);
      v.x = (uint32_t)arow[p0.x] | ((uint32_t)arow[p0.y] << 16);
      v.y = (uint32_t)arow[p0.z] | ((uint32_t)arow[p0.w] << 16);
      v.z = (uint32_t)arow[p1.x] | ((uint32_t)arow[p1.y] << 16);
      v.w = (uint32_t)arow[p1.z] | ((uint32_t)arow[p1.w] << 16);
    }
  }
  return __builtin_bit_cast(vec8, v);
}

// Adds bias, rounds and stores the MB x 4 tiles held by one wavefront.
template <typename T, int MB>
__device__ __forceinline__ void write_tiles(const StreamParams& p, int strip, int lane,
                                            const floatx4_t (&acc)[MB][4]) {
  const int m_in = lane & 15;
  const int n_in = 4 * (lane >> 4);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int nl = 16 * j + n_in;
    float b[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        b[r] = Dq<T>::to_float(p.bias[strip * kStripN + scale_slot(nl + r, false)]);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = 16 * mb + m_in;
      if (m < p.size_m) {
        const floatx4_t v = acc[mb][j];
        uint2 o;
        o.x = (uint32_t)Dq<T>::from_float(v.x + b[0]) | ((uint32_t)Dq<T>::from_float(v.y + b[1]) << 16);
        o.y = (uint32_t)Dq<T>::from_float(v.z + b[2]) | ((uint32_t)Dq<T>::from_float(v.w + b[3]) << 16);
        *reinterpret_cast<uint2*>(p.c + (long)m * p.size_n + strip * kStripN + nl) = o;
      }
    }
  }
}

template <typename T, int MB, bool HAS_ZP, bool HAS_PERM>
__global__ __launch_bounds__(kThreads) void marlin_stream_kernel(const StreamParams p) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq<T>::Col Col;
  __shared__ float4 red[kWaves / 2][MB * 4][64];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col16 = lane & 15;
  const int kb = lane >> 4;
  const long parts = gridDim.x;
  const long u_begin = range_begin(blockIdx.x, p.total_units, parts);
  const long u_end = range_begin(blockIdx.x + 1, p.total_units, parts);
  const bool grouped = p.num_groups > 1;

  long u = u_begin;
  while (u < u_end) {
    const int strip = (int)(u / p.units_per_strip);
    const int unit_a = (int)(u - (long)strip * p.units_per_strip);
    const long strip_end = (long)(strip + 1) * p.units_per_strip;
    const long seg_end = u_end < strip_end ? u_end : strip_end;
    const int unit_b = unit_a + (int)(seg_end - u);
    u = seg_end;

    floatx4_t acc[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[mb][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    Col cols[4];
    int cur_group = -1;
    const uint4* bstrip = p.b + (long)strip * p.chunks_per_strip * 64 + lane;

    for (int unit = unit_a + wave; unit < unit_b; unit += kWaves) {
      const int chunk0 = unit * p.unit_chunks;
      uint4 q[4];
      vec8 av[4][MB];
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) {
        if (cc < p.unit_chunks) {
          q[cc] = bstrip[(long)(chunk0 + cc) * 64];
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            av[cc][mb] = load_a<T, HAS_PERM>(p, 16 * mb + col16, (chunk0 + cc) * kChunkK + 8 * kb);
        }
      }
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) {
        if (cc < p.unit_chunks) {
          const int g = grouped ? ((chunk0 + cc) * kChunkK) / p.group_size : 0;
          if (g != cur_group) {
            cur_group = g;
            load_cols<T, HAS_ZP>(cols, p.scales, p.zeros, p.size_n, strip, g, col16, grouped);
          }
          const uint32_t words[4] = {q[cc].x, q[cc].y, q[cc].z, q[cc].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const vec8 w = Dq<T>::word(words[j], cols[j]);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) acc[mb][j] = Dq<T>::mfma(w, av[cc][mb], acc[mb][j]);
          }
        }
      }
    }

    // Sum the eight wavefronts' tiles: the upper half of the active set
    // writes, the lower half adds, three times.
#pragma unroll
    for (int half = kWaves / 2; half >= 1; half >>= 1) {
      if (wave >= half && wave < 2 * half) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const floatx4_t v = acc[mb][j];
            red[wave - half][mb * 4 + j][lane] = make_float4(v.x, v.y, v.z, v.w);
          }
      }
      __syncthreads();
      if (wave < half) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float4 v = red[wave][mb * 4 + j][lane];
            acc[mb][j] += floatx4_t{v.x, v.y, v.z, v.w};
          }
      }
      __syncthreads();
    }

    if (wave != 0) continue;
    const bool whole = unit_a == 0 && unit_b == p.units_per_strip;
    if (whole) {
      write_tiles<T, MB>(p, strip, lane, acc);
      continue;
    }

    // Partial strip: publish, count, and let the last contributor finish.
    const long strip_first = (long)strip * p.units_per_strip;
    const int first = range_owner(strip_first, p.total_units, parts);
    const int last = range_owner(strip_end - 1, p.total_units, parts);
    const int me = blockIdx.x;
    float4* slot = p.scratch + (long)(me == first ? parts + me : me) * kSlotFloat4;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const floatx4_t v = acc[mb][j];
        slot[(mb * 4 + j) * 64 + lane] = make_float4(v.x, v.y, v.z, v.w);
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");  // partial tile visible before the count
    int arrived = 0;
    if (lane == 0)
      arrived = __hip_atomic_fetch_add(p.workspace + first, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if (arrived != last - first) continue;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[mb][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    for (int w = first; w <= last; ++w) {
      const float4* src = p.scratch + (long)(w == first ? parts + w : w) * kSlotFloat4;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 v = src[(mb * 4 + j) * 64 + lane];
          acc[mb][j] += floatx4_t{v.x, v.y, v.z, v.w};
        }
    }
    write_tiles<T, MB>(p, strip, lane, acc);
    if (lane == 0) __hip_atomic_store(p.workspace + first, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Writes W[K][N]: the values the GEMM kernel feeds to the matrix cores.
template <typename T, bool HAS_ZP>
__global__ __launch_bounds__(256) void marlin_dequant_kernel(const uint4* __restrict__ b,
                                                            const uint16_t* __restrict__ scales,
                                                            const uint32_t* __restrict__ zeros,
                                                            uint16_t* __restrict__ w_out, int size_n,
                                                            int size_k, int num_groups, int group_size,
                                                            long total_chunks) {
  typedef typename Dq<T>::vec8 vec8;
  const int lane = threadIdx.x & 63;
  const int col16 = lane & 15;
  const int kb = lane >> 4;
  const int chunks_per_strip = size_k / kChunkK;
  const bool grouped = num_groups > 1;
  for (long ch = (long)blockIdx.x * 4 + (threadIdx.x >> 6); ch < total_chunks; ch += (long)gridDim.x * 4) {
    const int strip = (int)(ch / chunks_per_strip);
    const int chunk = (int)(ch % chunks_per_strip);
    const int g = grouped ? (chunk * kChunkK) / group_size : 0;
    typename Dq<T>::Col cols[4];
    load_cols<T, HAS_ZP>(cols, scales, zeros, size_n, strip, g, col16, grouped);
    const uint4 q = b[ch * 64 + lane];
    const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const vec8 w = Dq<T>::word(words[j], cols[j]);
      const uint16_t* bits = reinterpret_cast<const uint16_t*>(&w);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const long k = (long)chunk * kChunkK + 8 * kb + t;
        w_out[k * size_n + strip * kStripN + 16 * j + col16] = bits[t];
      }
    }
  }
}

int cu_count() {
  static int cached = 0;
  if (cached == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return 256;
    cached = n;
  }
  return cached;
}

template <typename T, int MB, bool HAS_ZP>
void launch_stream(const StreamParams& p, bool has_perm, int grid, hipStream_t st) {
  if (has_perm)
    marlin_stream_kernel<T, MB, HAS_ZP, true><<<grid, kThreads, 0, st>>>(p);
  else
    marlin_stream_kernel<T, MB, HAS_ZP, false><<<grid, kThreads, 0, st>>>(p);
}

template <typename T, bool HAS_ZP>
void launch_stream_mb(const StreamParams& p, bool has_perm, int grid, hipStream_t st) {
  const int mb = (p.size_m + 15) / 16;
  switch (mb) {
    case 1: launch_stream<T, 1, HAS_ZP>(p, has_perm, grid, st); break;
    case 2: launch_stream<T, 2, HAS_ZP>(p, has_perm, grid, st); break;
    case 3: launch_stream<T, 3, HAS_ZP>(p, has_perm, grid, st); break;
    default: launch_stream<T, 4, HAS_ZP>(p, has_perm, grid, st); break;
  }
}

struct Checked {
  bool has_zp;
  bool has_perm;
  int group_size;
};

int check_common(Checked& out, int b_layout, const void* b_scales, const uint32_t* b_zeros,
                 const int32_t* g_idx, const int32_t* perm, int dtype, int64_t b_type_id,
                 int64_t size_n, int64_t size_k, int64_t num_groups, int is_k_full) {
  SONAR_REQUIRE(b_layout == SONAR_LAYOUT_GFX950, "unknown b_layout = %d", b_layout);
  SONAR_REQUIRE(dtype == SONAR_DTYPE_F16 || dtype == SONAR_DTYPE_BF16, "unsupported `a` scalar_type");
  SONAR_REQUIRE(size_k > 0 && size_k % kChunkK == 0 && size_k < (1LL << 30),
                "size_k = %ld is not divisible by %d", (long)size_k, kChunkK);
  SONAR_REQUIRE(size_n > 0 && size_n % kStripN == 0 && size_n < (1LL << 30),
                "size_n = %ld, is not divisible by min_thread_n = %d", (long)size_n, kStripN);
  SONAR_REQUIRE(b_scales != nullptr, "b_scales must not be NULL");
  SONAR_REQUIRE(num_groups >= 1, "num_groups = %ld must be >= 1", (long)num_groups);
  if (b_type_id != SONAR_TYPE_UINT4B8 && b_type_id != SONAR_TYPE_UINT4)
    return fail(SONAR_E_UNSUPPORTED,
                "b_type id %ld is not built here: only uint4b8 (GPTQ) and uint4 (AWQ) weights are",
                (long)b_type_id);
  out.has_zp = b_zeros != nullptr;
  if (out.has_zp)
    SONAR_REQUIRE(b_type_id == SONAR_TYPE_UINT4, "b_type must be u4 or u8 when has_zp = True");
  else
    SONAR_REQUIRE(b_type_id == SONAR_TYPE_UINT4B8,
                  "b_type must be uint4b8 when has_zp = False (uint4 needs b_zeros)");
  SONAR_REQUIRE((g_idx == nullptr) == (perm == nullptr), "g_idx and perm must be given together");
  out.has_perm = perm != nullptr;
  if (out.has_perm) {
    if (!is_k_full)
      return fail(SONAR_E_UNSUPPORTED, "act-order with is_k_full = False is not built yet");
    SONAR_REQUIRE(num_groups > 1, "For act_order, num_groups must be > 1");
  }
  if (num_groups > 1) {
    SONAR_REQUIRE(size_k % num_groups == 0, "size_k = %ld, is not divisible by num_groups = %ld",
                  (long)size_k, (long)num_groups);
    out.group_size = (int)(size_k / num_groups);
    SONAR_REQUIRE(out.group_size % kChunkK == 0, "group_size = %d must be a multiple of %d",
                  out.group_size, kChunkK);
  } else {
    out.group_size = (int)size_k;
  }
  return SONAR_OK;
}

}  // namespace
}  // namespace sonar

using namespace sonar;

extern "C" size_t sonar_marlin_gemm_scratch_bytes(int64_t size_m, int64_t size_n, int64_t size_k) {
  (void)size_m;
  (void)size_n;
  (void)size_k;
  return (size_t)2 * cu_count() * kSlotFloat4 * sizeof(float4);
}

extern "C" int sonar_marlin_gemm(const void* a, int64_t a_row_stride, void* c,
                                 const uint32_t* b_q_weight, int b_layout, const void* b_bias,
                                 const void* b_scales, const uint32_t* b_zeros, const int32_t* g_idx,
                                 const int32_t* perm, int32_t* workspace, int64_t workspace_len,
                                 void* scratch, size_t scratch_bytes, int dtype, int64_t b_type_id,
                                 int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups,
                                 int is_k_full, int use_atomic_add, int use_fp32_reduce, void* stream) {
  (void)use_atomic_add;
  (void)use_fp32_reduce;
  SONAR_REQUIRE(size_m >= 0 && size_m < (1LL << 30), "size_m = %ld out of range", (long)size_m);
  Checked chk;
  if (int rc = check_common(chk, b_layout, b_scales, b_zeros, g_idx, perm, dtype, b_type_id, size_n,
                            size_k, num_groups, is_k_full))
    return rc;
  if (size_m == 0) return SONAR_OK;
  SONAR_REQUIRE(a && c && b_q_weight, "a, c and b_q_weight must not be NULL");
  SONAR_REQUIRE(a_row_stride >= size_k && a_row_stride % 8 == 0, "A.stride(0) must divisible by 8");
  SONAR_REQUIRE(((uintptr_t)a) % 16 == 0, "A must aligned to 16 bytes");
  SONAR_REQUIRE(((uintptr_t)c) % 8 == 0 && ((uintptr_t)b_q_weight) % 16 == 0,
                "c must be 8-byte and b_q_weight 16-byte aligned");
  const int cus = cu_count();
  SONAR_REQUIRE(workspace && workspace_len >= cus,
                "workspace.numel = %ld is below min_workspace_size = %d", (long)workspace_len, cus);
  SONAR_REQUIRE(scratch && scratch_bytes >= sonar_marlin_gemm_scratch_bytes(size_m, size_n, size_k),
                "scratch of %zu bytes is too small", scratch_bytes);

  StreamParams p;
  p.b = reinterpret_cast<const uint4*>(b_q_weight);
  p.bias = static_cast<const uint16_t*>(b_bias);
  p.scales = static_cast<const uint16_t*>(b_scales);
  p.zeros = b_zeros;
  p.g_idx = g_idx;
  p.perm = perm;
  p.workspace = workspace;
  p.scratch = static_cast<float4*>(scratch);
  p.size_n = (int)size_n;
  p.size_k = (int)size_k;
  p.lda = a_row_stride;
  p.num_groups = (int)num_groups;
  p.group_size = chk.group_size;
  p.chunks_per_strip = (int)(size_k / kChunkK);
  p.unit_chunks = p.chunks_per_strip % 4 == 0 ? 4 : (p.chunks_per_strip % 2 == 0 ? 2 : 1);
  p.units_per_strip = p.chunks_per_strip / p.unit_chunks;
  p.total_units = (long)(size_n / kStripN) * p.units_per_strip;
  int grid = cus;
  if (p.total_units < grid) grid = (int)p.total_units;
  hipStream_t st = (hipStream_t)stream;

  for (int64_t m0 = 0; m0 < size_m; m0 += 64) {
    p.a = static_cast<const uint16_t*>(a) + m0 * a_row_stride;
    p.c = static_cast<uint16_t*>(c) + m0 * size_n;
    p.size_m = (int)(size_m - m0 < 64 ? size_m - m0 : 64);
    if (dtype == SONAR_DTYPE_F16) {
      if (chk.has_zp) launch_stream_mb<_Float16, true>(p, chk.has_perm, grid, st);
      else launch_stream_mb<_Float16, false>(p, chk.has_perm, grid, st);
    } else {
      if (chk.has_zp) launch_stream_mb<__bf16, true>(p, chk.has_perm, grid, st);
      else launch_stream_mb<__bf16, false>(p, chk.has_perm, grid, st);
    }
    if (int rc = launch_status("marlin_stream_kernel")) return rc;
  }
  return SONAR_OK;
}

extern "C" int sonar_marlin_dequant(const uint32_t* b_q_weight, int b_layout, const void* b_scales,
                                    const uint32_t* b_zeros, const int32_t* g_idx, void* w_out,
                                    int dtype, int64_t b_type_id, int64_t size_n, int64_t size_k,
                                    int64_t num_groups, int is_k_full, void* stream) {
  Checked chk;
  if (int rc = check_common(chk, b_layout, b_scales, b_zeros, g_idx, g_idx, dtype, b_type_id, size_n,
                            size_k, num_groups, is_k_full))
    return rc;
  SONAR_REQUIRE(b_q_weight && w_out, "b_q_weight and w_out must not be NULL");
  const long total_chunks = (size_n / kStripN) * (size_k / kChunkK);
  long blocks = (total_chunks + 3) / 4;
  if (blocks > 8192) blocks = 8192;
  hipStream_t st = (hipStream_t)stream;
  const uint4* b = reinterpret_cast<const uint4*>(b_q_weight);
  const uint16_t* s = static_cast<const uint16_t*>(b_scales);
  uint16_t* w = static_cast<uint16_t*>(w_out);
  const int ng = (int)num_groups, gs = chk.group_size, n = (int)size_n, k = (int)size_k;
  if (dtype == SONAR_DTYPE_F16) {
    if (chk.has_zp) marlin_dequant_kernel<_Float16, true><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, w, n, k, ng, gs, total_chunks);
    else marlin_dequant_kernel<_Float16, false><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, w, n, k, ng, gs, total_chunks);
  } else {
    if (chk.has_zp) marlin_dequant_kernel<__bf16, true><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, w, n, k, ng, gs, total_chunks);
    else marlin_dequant_kernel<__bf16, false><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, w, n, k, ng, gs, total_chunks);
  }
  return launch_status("marlin_dequant_kernel");
}
