// The small kernels that bracket the two grouped GEMMs of a mixture-of-experts
// layer: routing of (token, k) slots into per-expert blocks, the gated
// activation, and the sum over a token's experts.  They restate
// csrc/libtorch_stable/moe/moe_align_sum_kernels.cu:626-725,759+ and the
// silu_and_mul of csrc/libtorch_stable/activation_kernels.cu for fp16 / bf16.
#include "common.hpp"

namespace sonar {
namespace {

constexpr int kAlignThreads = 1024;

// One workgroup: per-expert counts, padded offsets, expert id of every block,
// the padded total, and the sentinel fill of sorted_token_ids.  offsets[e] is
// left for the placement kernel.
__global__ __launch_bounds__(kAlignThreads) void moe_align_count_kernel(
    const int32_t* __restrict__ topk_ids, int numel, int num_experts, int block_size,
    int32_t* __restrict__ sorted_ids, int sorted_len, int32_t* __restrict__ expert_ids, int expert_len,
    int32_t* __restrict__ num_post_pad, const int32_t* __restrict__ expert_map, int32_t* __restrict__ offsets) {
  extern __shared__ int32_t counts[];  // num_experts + 1 entries, then the padded prefix
  int32_t* begin = counts + num_experts + 1;
  for (int e = threadIdx.x; e <= num_experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < numel; i += blockDim.x) {
    int e = topk_ids[i];
    if (e >= 0 && e < num_experts && expert_map) e = expert_map[e];
    if (e >= 0 && e < num_experts) atomicAdd(&counts[e], 1);
  }
  for (int i = threadIdx.x; i < sorted_len; i += blockDim.x) sorted_ids[i] = numel;
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < num_experts; ++e) {
      begin[e] = at;
      offsets[e] = at;
      at += (counts[e] + block_size - 1) / block_size * block_size;
    }
    begin[num_experts] = at;
    num_post_pad[0] = at;
  }
  __syncthreads();
  const int total = begin[num_experts];
  for (int b = threadIdx.x; b < expert_len; b += blockDim.x) {
    const int start = b * block_size;
    int e = -1;
    if (start < total) {
      // last expert whose run begins at or before `start` and is not empty there
      int lo = 0, hi = num_experts - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (begin[mid] <= start) lo = mid; else hi = mid - 1;
      }
      e = lo;
    }
    expert_ids[b] = e;
  }
}

// One wavefront per expert walks the slots in order; a ballot gives every
// matching lane its rank, so the slots of an expert keep ascending order.
__global__ __launch_bounds__(256) void moe_align_place_kernel(const int32_t* __restrict__ topk_ids, int numel,
                                                             int num_experts,
                                                             int32_t* __restrict__ sorted_ids,
                                                             const int32_t* __restrict__ expert_map,
                                                             const int32_t* __restrict__ offsets) {
  const int lane = threadIdx.x & 63;
  const int expert = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (expert >= num_experts) return;
  int at = offsets[expert];
  for (int base = 0; base < numel; base += 64) {
    const int i = base + lane;
    int e = -1;
    if (i < numel) {
      e = topk_ids[i];
      if (e >= 0 && e < num_experts && expert_map) e = expert_map[e];
    }
    const bool mine = e == expert;
    const unsigned long long mask = __ballot(mine);
    if (mine) sorted_ids[at + __popcll(mask & ((1ull << lane) - 1ull))] = i;
    at += __popcll(mask);
  }
}

template <typename T>
__device__ __forceinline__ float to_f32(uint16_t b);
template <>
__device__ __forceinline__ float to_f32<_Float16>(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
template <>
__device__ __forceinline__ float to_f32<__bf16>(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
template <typename T>
__device__ __forceinline__ uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (T)f); }

// out[r][c] = T(T(silu(x[r][c])) * x[r][d + c]): the activation is rounded to
// the tensor type before the product, as act_and_mul does.
template <typename T>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(uint16_t* __restrict__ out,
                                                          const uint16_t* __restrict__ in, long rows, int d) {
  const long vec_per_row = d / 8;
  const long total = rows * vec_per_row;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long r = i / vec_per_row;
    const int c = (int)(i - r * vec_per_row) * 8;
    const uint4 g = *reinterpret_cast<const uint4*>(in + r * 2 * d + c);
    const uint4 u = *reinterpret_cast<const uint4*>(in + r * 2 * d + d + c);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t o = 0;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float x = to_f32<T>((uint16_t)(gw[w] >> (16 * h)));
        const float y = to_f32<T>((uint16_t)(uw[w] >> (16 * h)));
        const float s = to_f32<T>(from_f32<T>(x / (1.0f + __expf(-x))));
        o |= (uint32_t)from_f32<T>(s * y) << (16 * h);
      }
      ow[w] = o;
    }
    *reinterpret_cast<uint4*>(out + r * d + c) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

// The gated activations of the fused mixture-of-experts layer other than plain SiLU
// (aphrodite/model_executor/layers/fused_moe/activation.py:128-205 of the reference; the
// arithmetic of csrc/libtorch_stable/activation_kernels.cu:28-95,154-215,412-423,489-510 and of
// the Triton kernel aphrodite/model_executor/layers/activation.py:27-52), one (gate, up) pair
// -> one output, every intermediate rounding where the reference has one:
//   kClampSilu  silu_and_mul_with_clamp: g = T(min(gate, limit)), u = clamp(up, -limit, limit);
//               T(float(T(g / (1 + exp(-alpha g)))) * (u + beta))
//   kGelu       T(float(T(0.5 g (1 + erf(g / sqrt 2)))) * up);  kGeluTanh: the tanh form
//   kSwigluOai  gate / up interleaved in the input: g = min(gate, limit), u = clamp(up, +-limit);
//               T((u + 1) * g / (1 + exp(-alpha g)))
//   kSitu       T(beta tanh(gate / beta) / (1 + exp(-gate)) * (linear_beta > 0 ? linear_beta tanh(up / linear_beta) : up))
//               (beta in `alpha`, linear_beta in `beta`)
//   kSwigluStep T(min(gate * sigmoid(gate), limit) * clamp(up, -limit, limit))
enum MoeActivation { kClampSilu = 1, kGelu = 2, kGeluTanh = 3, kSwigluOai = 4, kSitu = 5, kSwigluStep = 6 };

template <typename T, int KIND>
__device__ __forceinline__ uint16_t gated_activation(uint16_t gate_bits, uint16_t up_bits, float limit, float alpha,
                                                     float beta) {
  const float gate = to_f32<T>(gate_bits), up = to_f32<T>(up_bits);
  if constexpr (KIND == kClampSilu) {
    const float g = to_f32<T>(from_f32<T>(fminf(gate, limit)));
    const float u = fmaxf(fminf(up, limit), -limit);
    const float act = to_f32<T>(from_f32<T>(g / (1.0f + expf(-g * alpha))));
    return from_f32<T>(act * (u + beta));
  } else if constexpr (KIND == kGelu) {
    const float act = to_f32<T>(from_f32<T>(gate * 0.5f * (1.0f + erff(gate * 0.70710678118654752440f))));
    return from_f32<T>(act * up);
  } else if constexpr (KIND == kGeluTanh) {
    const float inner = 0.79788456080286535588f * (gate + 0.044715f * (gate * gate * gate));
    const float act = to_f32<T>(from_f32<T>(0.5f * gate * (1.0f + tanhf(inner))));
    return from_f32<T>(act * up);
  } else if constexpr (KIND == kSwigluOai) {
    const float g = fminf(gate, limit);
    const float u = fmaxf(fminf(up, limit), -limit);
    return from_f32<T>((u + 1.0f) * g / (1.0f + expf(-g * alpha)));
  } else if constexpr (KIND == kSitu) {
    const float gate_out = alpha * tanhf(gate * (1.0f / alpha)) / (1.0f + expf(-gate));
    const float up_out = beta > 0.0f ? beta * tanhf(up * (1.0f / beta)) : up;
    return from_f32<T>(gate_out * up_out);
  } else {
    const float silu = gate / (1.0f + expf(-gate));
    return from_f32<T>(fminf(silu, limit) * fmaxf(fminf(up, limit), -limit));
  }
}

// in: rows x 2d (gate half then up half; kSwigluOai: gate and up alternate), out: rows x d.
template <typename T, int KIND>
__global__ __launch_bounds__(256) void moe_activation_kernel(uint16_t* __restrict__ out,
                                                            const uint16_t* __restrict__ in, long rows, int d,
                                                            float limit, float alpha, float beta) {
  const long vec_per_row = d / 8;
  const long total = rows * vec_per_row;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long r = i / vec_per_row;
    const int c = (int)(i - r * vec_per_row) * 8;
    uint4 g, u;
    if constexpr (KIND == kSwigluOai) {   // sixteen values: eight pairs
      g = *reinterpret_cast<const uint4*>(in + r * 2 * d + 2 * c);
      u = *reinterpret_cast<const uint4*>(in + r * 2 * d + 2 * c + 8);
    } else {
      g = *reinterpret_cast<const uint4*>(in + r * 2 * d + c);
      u = *reinterpret_cast<const uint4*>(in + r * 2 * d + d + c);
    }
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t o = 0;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint16_t gb, ub;
        if constexpr (KIND == kSwigluOai) {   // output 2 w + h of these eight: the pair in word 2 w + h of g | u
          const int pair = 2 * w + h;
          const uint32_t word = pair < 4 ? gw[pair] : uw[pair - 4];
          gb = (uint16_t)word;
          ub = (uint16_t)(word >> 16);
        } else {
          gb = (uint16_t)(gw[w] >> (16 * h));
          ub = (uint16_t)(uw[w] >> (16 * h));
        }
        o |= (uint32_t)gated_activation<T, KIND>(gb, ub, limit, alpha, beta) << (16 * h);
      }
      ow[w] = o;
    }
    *reinterpret_cast<uint4*>(out + r * d + c) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

// out[t][c] = T(sum_k in[t][k][c]), summed in fp32.
template <typename T>
__global__ __launch_bounds__(256) void moe_sum_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ in,
                                                     long tokens, int topk, int d) {
  const long vec_per_row = d / 8;
  const long total = tokens * vec_per_row;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long t = i / vec_per_row;
    const int c = (int)(i - t * vec_per_row) * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < topk; ++k) {
      const uint4 v = *reinterpret_cast<const uint4*>(in + (t * topk + k) * d + c);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] += to_f32<T>((uint16_t)w[j]);
        acc[2 * j + 1] += to_f32<T>((uint16_t)(w[j] >> 16));
      }
    }
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o[j] = (uint32_t)from_f32<T>(acc[2 * j]) | ((uint32_t)from_f32<T>(acc[2 * j + 1]) << 16);
    *reinterpret_cast<uint4*>(out + t * d + c) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

inline int blocks_for(long items) {
  const long b = (items + 255) / 256;
  return (int)(b < 1 ? 1 : (b > 8192 ? 8192 : b));
}

}  // namespace
}  // namespace sonar

using namespace sonar;

extern "C" int sonar_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int64_t num_experts,
                                          int64_t block_size, int32_t* sorted_token_ids, int64_t sorted_len,
                                          int32_t* expert_ids, int64_t expert_len,
                                          int32_t* num_tokens_post_pad, const int32_t* expert_map,
                                          int32_t* offsets_scratch, void* stream) {
  SONAR_REQUIRE(numel >= 0 && numel < (1LL << 30), "topk_ids.numel = %ld out of range", (long)numel);
  SONAR_REQUIRE(num_experts >= 1 && num_experts <= 8192, "num_experts = %ld out of range", (long)num_experts);
  SONAR_REQUIRE(block_size >= 1, "block_size = %ld must be positive", (long)block_size);
  SONAR_REQUIRE(sorted_len >= 0 && sorted_len < (1LL << 30) && expert_len >= 0, "output lengths out of range");
  SONAR_REQUIRE(expert_len * block_size >= sorted_len, "expert_ids holds %ld blocks, fewer than ceil(%ld / %ld)",
                (long)expert_len, (long)sorted_len, (long)block_size);
  // every expert may need block_size - 1 padding slots
  const int64_t worst = numel + num_experts * (block_size - 1);
  SONAR_REQUIRE(sorted_len >= (numel < num_experts ? (numel * block_size < worst ? numel * block_size : worst)
                                                    : worst),
                "sorted_token_ids.numel = %ld is too small", (long)sorted_len);
  SONAR_REQUIRE(sorted_token_ids && expert_ids && num_tokens_post_pad && offsets_scratch && (topk_ids || numel == 0),
                "moe_align_block_size: NULL argument");
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)(2 * num_experts + 2) * sizeof(int32_t);
  moe_align_count_kernel<<<1, kAlignThreads, lds, st>>>(topk_ids, (int)numel, (int)num_experts, (int)block_size,
                                                        sorted_token_ids, (int)sorted_len, expert_ids,
                                                        (int)expert_len, num_tokens_post_pad, expert_map,
                                                        offsets_scratch);
  if (int rc = launch_status("moe_align_count_kernel")) return rc;
  if (numel > 0) {
    moe_align_place_kernel<<<(int)((num_experts + 3) / 4), 256, 0, st>>>(topk_ids, (int)numel, (int)num_experts,
                                                                         sorted_token_ids, expert_map,
                                                                         offsets_scratch);
    if (int rc = launch_status("moe_align_place_kernel")) return rc;
  }
  return SONAR_OK;
}

extern "C" int sonar_silu_and_mul(void* out, const void* in, int64_t rows, int64_t d, int dtype, void* stream) {
  SONAR_REQUIRE(dtype == SONAR_DTYPE_F16 || dtype == SONAR_DTYPE_BF16, "unsupported dtype");
  SONAR_REQUIRE(rows >= 0 && d > 0 && d % 8 == 0, "silu_and_mul: d = %ld must be a positive multiple of 8", (long)d);
  if (rows == 0) return SONAR_OK;
  SONAR_REQUIRE(out && in && ((uintptr_t)out) % 16 == 0 && ((uintptr_t)in) % 16 == 0,
                "silu_and_mul: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int blocks = blocks_for(rows * (d / 8));
  if (dtype == SONAR_DTYPE_F16)
    silu_and_mul_kernel<_Float16><<<blocks, 256, 0, st>>>(static_cast<uint16_t*>(out),
                                                          static_cast<const uint16_t*>(in), rows, (int)d);
  else
    silu_and_mul_kernel<__bf16><<<blocks, 256, 0, st>>>(static_cast<uint16_t*>(out),
                                                        static_cast<const uint16_t*>(in), rows, (int)d);
  return launch_status("silu_and_mul_kernel");
}

namespace {
template <typename T>
void launch_moe_activation(int kind, int blocks, hipStream_t st, uint16_t* out, const uint16_t* in, long rows, int d,
                           float limit, float alpha, float beta) {
  switch (kind) {
    case kClampSilu: moe_activation_kernel<T, kClampSilu><<<blocks, 256, 0, st>>>(out, in, rows, d, limit, alpha, beta); break;
    case kGelu: moe_activation_kernel<T, kGelu><<<blocks, 256, 0, st>>>(out, in, rows, d, limit, alpha, beta); break;
    case kGeluTanh: moe_activation_kernel<T, kGeluTanh><<<blocks, 256, 0, st>>>(out, in, rows, d, limit, alpha, beta); break;
    case kSwigluOai: moe_activation_kernel<T, kSwigluOai><<<blocks, 256, 0, st>>>(out, in, rows, d, limit, alpha, beta); break;
    case kSitu: moe_activation_kernel<T, kSitu><<<blocks, 256, 0, st>>>(out, in, rows, d, limit, alpha, beta); break;
    default: moe_activation_kernel<T, kSwigluStep><<<blocks, 256, 0, st>>>(out, in, rows, d, limit, alpha, beta); break;
  }
}
}  // namespace

extern "C" int sonar_moe_activation(void* out, const void* in, int64_t rows, int64_t d, int kind, float limit,
                                    float alpha, float beta, int dtype, void* stream) {
  SONAR_REQUIRE(dtype == SONAR_DTYPE_F16 || dtype == SONAR_DTYPE_BF16, "unsupported dtype");
  SONAR_REQUIRE(kind >= SONAR_ACT_SILU_CLAMP && kind <= SONAR_ACT_SWIGLUSTEP, "moe_activation: unknown kind %d", kind);
  SONAR_REQUIRE(rows >= 0 && d > 0 && d % 8 == 0, "moe_activation: d = %ld must be a positive multiple of 8", (long)d);
  if (kind == SONAR_ACT_SILU_CLAMP || kind == SONAR_ACT_SWIGLUOAI || kind == SONAR_ACT_SWIGLUSTEP)
    SONAR_REQUIRE(limit > 0.0f, "moe_activation: this activation needs a positive clamp limit");
  if (kind == SONAR_ACT_SITU) SONAR_REQUIRE(alpha > 0.0f, "moe_activation: SITU needs a positive beta");
  if (rows == 0) return SONAR_OK;
  SONAR_REQUIRE(out && in && ((uintptr_t)out) % 16 == 0 && ((uintptr_t)in) % 16 == 0,
                "moe_activation: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int blocks = blocks_for(rows * (d / 8));
  if (dtype == SONAR_DTYPE_F16)
    launch_moe_activation<_Float16>(kind, blocks, st, static_cast<uint16_t*>(out), static_cast<const uint16_t*>(in),
                                    rows, (int)d, limit, alpha, beta);
  else
    launch_moe_activation<__bf16>(kind, blocks, st, static_cast<uint16_t*>(out), static_cast<const uint16_t*>(in),
                                  rows, (int)d, limit, alpha, beta);
  return launch_status("moe_activation_kernel");
}

extern "C" int sonar_moe_sum(void* out, const void* in, int64_t tokens, int64_t topk, int64_t d, int dtype,
                             void* stream) {
  SONAR_REQUIRE(dtype == SONAR_DTYPE_F16 || dtype == SONAR_DTYPE_BF16, "unsupported dtype");
  SONAR_REQUIRE(tokens >= 0 && topk >= 1 && d > 0 && d % 8 == 0,
                "moe_sum: d = %ld must be a positive multiple of 8 and topk = %ld positive", (long)d, (long)topk);
  if (tokens == 0) return SONAR_OK;
  SONAR_REQUIRE(out && in && ((uintptr_t)out) % 16 == 0 && ((uintptr_t)in) % 16 == 0,
                "moe_sum: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int blocks = blocks_for(tokens * (d / 8));
  if (dtype == SONAR_DTYPE_F16)
    moe_sum_kernel<_Float16><<<blocks, 256, 0, st>>>(static_cast<uint16_t*>(out), static_cast<const uint16_t*>(in),
                                                     tokens, (int)topk, (int)d);
  else
    moe_sum_kernel<__bf16><<<blocks, 256, 0, st>>>(static_cast<uint16_t*>(out), static_cast<const uint16_t*>(in),
                                                   tokens, (int)topk, (int)d);
  return launch_status("moe_sum_kernel");
}
