// Per-token (per-row) quantisation of the activations for the W4A8 GEMM: one
// fp32 scale per row and int8 or float8_e4m3fn codes.  The int8 kernel follows
// aphrodite/model_executor/layers/quantization/utils/int8_utils.py:70-93, the
// fp8 one QuantFP8(False, GroupShape.PER_TOKEN)
// (layers/quantization/input_quant_fp8.py:188-204).  One workgroup per row:
// the maximum magnitude first, then the codes (the row is read twice; the
// second read comes from cache).  Every step rounds to fp32 as written.
#include "common.hpp"

namespace sonar {
namespace {

template <typename T>
__device__ __forceinline__ float load_as_float(const T* p, long i) { return (float)p[i]; }

__device__ __forceinline__ float block_max(float v) {
  __shared__ float part[4];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

template <typename T, bool FP8>
__global__ __launch_bounds__(256) void per_token_quant_kernel(const T* __restrict__ x, long row_stride,
                                                             uint8_t* __restrict__ q, float* __restrict__ scales,
                                                             int cols) {
#pragma clang fp contract(off)
  const T* row = x + (long)blockIdx.x * row_stride;
  uint8_t* out = q + (long)blockIdx.x * cols;
  float m = 0.0f;
  for (int i = threadIdx.x; i < cols; i += 256) m = fmaxf(m, fabsf(load_as_float(row, i)));
  m = block_max(m);
  if (FP8) {
    const float scale = fmaxf(m / 448.0f, 1.0f / (448.0f * 512.0f));
    const float inv = 1.0f / scale;
    if (threadIdx.x == 0) scales[blockIdx.x] = scale;
    for (int i = threadIdx.x; i < cols; i += 256) {
      const float y = fminf(fmaxf(load_as_float(row, i) * inv, -448.0f), 448.0f);
      out[i] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(y, 0.0f, 0, false) & 0xff);
    }
  } else {
    const float absmax = fmaxf(m, 1e-10f);
    const float mul = 127.0f / absmax;
    if (threadIdx.x == 0) scales[blockIdx.x] = absmax / 127.0f;
    for (int i = threadIdx.x; i < cols; i += 256) {
      const float y = load_as_float(row, i) * mul;
      out[i] = (uint8_t)(int8_t)(int)copysignf(floorf(fabsf(y) + 0.5f), y);   // halves away from zero
    }
  }
}

template <bool FP8>
int launch_quant(const void* x, int dtype, int64_t row_stride, uint8_t* q, float* scales, int64_t rows, int64_t cols,
                 void* stream) {
  SONAR_REQUIRE(rows >= 0 && cols > 0 && cols < (1LL << 31) && rows < (1LL << 31), "rows = %ld, cols = %ld",
                (long)rows, (long)cols);
  SONAR_REQUIRE(row_stride >= cols, "row_stride = %ld is smaller than cols = %ld", (long)row_stride, (long)cols);
  if (rows == 0) return SONAR_OK;
  SONAR_REQUIRE(x && q && scales, "x, q and scales must not be NULL");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == SONAR_DTYPE_F16)
    per_token_quant_kernel<_Float16, FP8><<<(int)rows, 256, 0, st>>>((const _Float16*)x, row_stride, q, scales, (int)cols);
  else if (dtype == SONAR_DTYPE_BF16)
    per_token_quant_kernel<__bf16, FP8><<<(int)rows, 256, 0, st>>>((const __bf16*)x, row_stride, q, scales, (int)cols);
  else if (dtype == SONAR_DTYPE_F32)
    per_token_quant_kernel<float, FP8><<<(int)rows, 256, 0, st>>>((const float*)x, row_stride, q, scales, (int)cols);
  else
    return fail(SONAR_E_INVALID, "unknown dtype = %d", dtype);
  return launch_status("per_token_quant_kernel");
}

}  // namespace
}  // namespace sonar

using namespace sonar;

extern "C" int sonar_per_token_quant_int8(const void* x, int dtype, int64_t row_stride, int8_t* q, float* scales,
                                          int64_t rows, int64_t cols, void* stream) {
  return launch_quant<false>(x, dtype, row_stride, (uint8_t*)q, scales, rows, cols, stream);
}

extern "C" int sonar_per_token_quant_fp8(const void* x, int dtype, int64_t row_stride, uint8_t* q, float* scales,
                                         int64_t rows, int64_t cols, void* stream) {
  return launch_quant<true>(x, dtype, row_stride, q, scales, rows, cols, stream);
}
