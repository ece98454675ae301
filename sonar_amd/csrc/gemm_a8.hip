// W4A8: 4-bit weights with 8-bit activations (int8 or float8_e4m3fn, one fp32
// scale per activation row) on the 8-bit matrix cores
// (v_mfma_i32_16x16x32_i8 / v_mfma_f32_16x16x32_fp8_fp8).  The path of the
// reference's Marlin kernel with is_a_8bit
// (csrc/libtorch_stable/quantization/marlin/marlin_template.h:1302-1400,
// 1869-1903,1955-1978; dequant.h:492-606).
//
// A workgroup of four wavefronts owns one 64-column strip of the weight
// stream, up to 64 activation rows and a range of K.  The wavefronts take the
// scale groups of that range in turn (a group is 1, 2 or 4 chunks of 32 rows;
// channelwise weights are walked in runs of 4 chunks), so the sum over one
// group stays inside one wavefront: it is multiplied by the group's scale and
// added to the wavefront's running total, in 32-bit integers for int8
// activations (the scales are then 16-bit integers) and in fp32 for fp8.  The
// four totals meet in LDS; wavefront w finishes column block w.  With K split
// over several workgroups the raw totals go to scratch and a second kernel
// adds them, so integer results never depend on the split.
#include "common.hpp"
#include "dequant.hpp"

namespace sonar {
namespace {

typedef int intx4_t __attribute__((ext_vector_type(4)));
typedef int intx8_t __attribute__((ext_vector_type(8)));

struct A8Params {
  const uint8_t* a;        // [M][a_row_stride] bytes
  long a_row_stride;
  void* c;                 // T [M][N]
  const uint32_t* w;       // gfx950 order
  const uint16_t* scales;  // [groups][N], single-permuted inside every 32 columns
  const uint32_t* zeros;   // [groups][N/8] or null
  const float* a_scales;   // [M]
  const uint16_t* bias;    // T [N], permuted like the scales, or null
  uint32_t* partial;       // [splits][M][N] raw totals when splits > 1
  int m, n, chunks;
  int unit_chunks;         // chunks per group (4 for channelwise)
  int units;               // ceil(chunks / unit_chunks)
  int units_per_split;
  int splits;
};

template <typename T>
__device__ __forceinline__ float from_bits(uint16_t b) {
  return (float)__builtin_bit_cast(T, b);
}
template <typename T>
__device__ __forceinline__ uint16_t to_bits(float f) {
  return __builtin_bit_cast(uint16_t, (T)f);
}

// Raw 32 bits of a total and back (by value: an element of a vector type is not an object
// __builtin_bit_cast can take).
__device__ __forceinline__ uint32_t raw_bits(int v) { return (uint32_t)v; }
__device__ __forceinline__ uint32_t raw_bits(float v) { return __float_as_uint(v); }
__device__ __forceinline__ void from_raw(uint32_t b, int& v) { v = (int)b; }
__device__ __forceinline__ void from_raw(uint32_t b, float& v) { v = __uint_as_float(b); }

// Activation type: what the matrix core accumulates in and how a weight word
// becomes two operand registers.  The eight codes of a word sit at the nibbles
// {row 0, 2, 4, 6, 1, 3, 5, 7}; the low nibbles of the four bytes are rows
// (0, 4, 1, 5), the high ones rows (2, 6, 3, 7): that is the byte order of the
// B operand, and the A operand is shuffled to match.
struct ActInt8 {
  typedef intx4_t acc_t;
  typedef int scalar_t;
  static constexpr bool kInteger = true;
  static constexpr bool kE8Scales = false;
  static __device__ __forceinline__ acc_t mfma(long a, long b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, c, 0, 0, 0);
  }
  // uint4b8: the code with its top bit flipped is the 4-bit two's complement of
  // code - 8; in the high nibble of a byte it reads as 16 * (code - 8).
  static constexpr int kShift = 4;
  static __device__ __forceinline__ long word(uint32_t w) {
    const uint32_t x = w ^ 0x88888888u;
    const uint32_t lo = (x << 4) & 0xf0f0f0f0u;
    const uint32_t hi = x & 0xf0f0f0f0u;
    return (long)(((uint64_t)hi << 32) | lo);
  }
  // uint4 with zero point z: ((q | 0x80) - z) ^ 0x80 is the two's complement
  // byte of q - z, with no borrow between bytes (dequant.h:572-583).
  static __device__ __forceinline__ long word_zp(uint32_t w, uint32_t z4) {
    const uint32_t lo = (((w & 0x0f0f0f0fu) | 0x80808080u) - z4) ^ 0x80808080u;
    const uint32_t hi = ((((w >> 4) & 0x0f0f0f0fu) | 0x80808080u) - z4) ^ 0x80808080u;
    return (long)(((uint64_t)hi << 32) | lo);
  }
  // The full-rate instruction takes two chunks (K = 64) at a time.
  static constexpr int kWideChunks = 2;
  typedef intx4_t wide_t;
  static __device__ __forceinline__ acc_t mfma_wide(wide_t a, wide_t b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  }
  // byte offset, inside a row of the LDS tile, of the 8 bytes (chunk c of the step, k block kb)
  static __device__ __forceinline__ int unit_offset(int c, int kb) { return (c >> 1) * 64 + kb * 16 + (c & 1) * 8; }
};

struct ActFp8 {
  typedef floatx4_t acc_t;
  typedef float scalar_t;
  static constexpr bool kInteger = false;
  static constexpr bool kE8Scales = false;
  static __device__ __forceinline__ acc_t mfma(long a, long b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, b, c, 0, 0, 0);
  }
  static constexpr int kShift = 0;
  // The nibble holds sign and magnitude as marlin_int4_fp8_preprocess leaves
  // them: p < 8: +p, else -((p & 7) + 1).  As a float8_e4m3fn byte with a zero
  // exponent field the magnitude m reads m * 2^-9 (8 carries into the exponent:
  // 2^-6); the scales carry the factor 512 (dequant.h:504-515).
  static __device__ __forceinline__ uint32_t four(uint32_t p) {
    const uint32_t s = p & 0x08080808u;
    return ((p & 0x07070707u) | (s << 4)) + (s >> 3);
  }
  static __device__ __forceinline__ long word(uint32_t w) {
    return (long)(((uint64_t)four((w >> 4) & 0x0f0f0f0fu) << 32) | four(w & 0x0f0f0f0fu));
  }
  // With zero points the nibble is q >= z ? q - z : 15 - q (dequant.h:585-606).
  static __device__ __forceinline__ uint32_t four_zp(uint32_t p, uint32_t z, uint32_t z4) {
    const uint32_t q0 = p | 0x70707070u;
    const uint32_t s = (q0 + z4) & 0x80808080u;
    return ((q0 + (s >> 7) * (z + 1)) & 0x0f0f0f0fu) | s;
  }
  static __device__ __forceinline__ long word_zp(uint32_t w, uint32_t z4) {
    const uint32_t z = z4 & 0xffu;
    return (long)(((uint64_t)four_zp((w >> 4) & 0x0f0f0f0fu, z, z4) << 32) | four_zp(w & 0x0f0f0f0fu, z, z4));
  }
  // The full-rate instruction takes four chunks (K = 128) at a time; its block scales are 1.
  static constexpr int kWideChunks = 4;
  typedef intx8_t wide_t;
  static __device__ __forceinline__ acc_t mfma_wide(wide_t a, wide_t b, acc_t c) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 127, 0, 127);
  }
  static __device__ __forceinline__ int unit_offset(int c, int kb) { return kb * 32 + c * 8; }
};

// float4_e2m1f codes with fp8 activations (MXFP4 weights, "W4A8-FP4": dequant.h:474-490): sign,
// two exponent bits and the mantissa bit moved into a float8_e4m3fn byte read 2^-6 times the fp4
// value (the zero exponent field gives the subnormal 0.5); the exponent-byte scales carry the 6
// (mxfp4_marlin_process_scales, marlin_utils_fp4.py:129-135).  Groups of 32 rows, no zero points.
struct ActFp8F4 : ActFp8 {
  static constexpr bool kE8Scales = true;
  static __device__ __forceinline__ uint32_t four_f4(uint32_t x) {   // nibbles in the high halves of x's bytes
    return (x & 0x80808080u) | ((x & 0x70707070u) >> 2);
  }
  static __device__ __forceinline__ long word(uint32_t w) {
    return (long)(((uint64_t)four_f4(w) << 32) | four_f4(w << 4));
  }
  static __device__ __forceinline__ long word_zp(uint32_t w, uint32_t) { return word(w); }
};
// Scale of a group as the kernel multiplies it: 16-bit integer, number of the output type, or (E8)
// an exponent byte 2^(b - 127).
template <typename ACT, typename T, bool E8>
__device__ __forceinline__ typename ACT::scalar_t group_scale(const void* scales, long index) {
  if constexpr (E8) return __uint_as_float((uint32_t)static_cast<const uint8_t*>(scales)[index] << 23);
  else if constexpr (ACT::kInteger) return (int)static_cast<const uint16_t*>(scales)[index];   // read as unsigned
  else return from_bits<T>(static_cast<const uint16_t*>(scales)[index]);
}

// Raw total -> output value: the activation row's scale, for channelwise
// weights the column's scale, the bias, one rounding.
template <typename ACT, typename T, bool GROUPED>
__device__ __forceinline__ uint16_t finish(typename ACT::scalar_t total, float a_scale, float col_scale,
                                           float bias) {
  // every step rounds to fp32 as written (the reference's epilogue does: marlin_template.h:1869-1903,
  // 1955-1978); contraction would fuse them into the final conversion and round once
#pragma clang fp contract(off)
  float f = (float)total * a_scale;
  if (!GROUPED) f *= col_scale;
  f += bias;
  return to_bits<T>(f);
}

// The sum over this wavefront's share of K: groups (units) u_begin + wave, + WAVES, ... of
// [u_begin, u_end).  a_row[rb]: this lane's row of A in row block rb, already offset by the
// lane's 8 bytes inside a chunk; w_lane: the lane's 16 bytes of chunk 0 of the strip;
// scales / zeros: row 0 of the matrix's (the expert's) scales and zero points.
template <typename ACT, typename T, int MB, bool HAS_ZP, bool GROUPED, int WAVES = 4, bool E8 = false>
__device__ __forceinline__ void a8_accumulate(typename ACT::acc_t (&acc)[MB][4], const uint8_t* const (&a_row)[MB],
                                              const uint32_t* w_lane, const void* scales,
                                              const uint32_t* zeros, int n, int strip, int chunks, int unit_chunks,
                                              int u_begin, int u_end, int wave, int l16) {
  typedef typename ACT::acc_t acc_t;
  typedef typename ACT::scalar_t scalar_t;
  int s_col[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) s_col[j] = strip * kStripN + scale_slot(16 * j + l16, false);
  for (int u = u_begin + wave; u < u_end; u += WAVES) {
    acc_t tmp[MB][4];
#pragma unroll
    for (int rb = 0; rb < MB; ++rb)
#pragma unroll
      for (int j = 0; j < 4; ++j) tmp[rb][j] = acc_t{0, 0, 0, 0};
    const int g = GROUPED ? u : 0;
    uint32_t z4[4] = {0, 0, 0, 0};
    if (HAS_ZP) {
      // column 16j + l16 of the strip: word l16 % 8 of the strip's eight, nibble 2j + l16 / 8
      const uint32_t zw = zeros[(long)g * (n / 8) + strip * 8 + (l16 & 7)];
#pragma unroll
      for (int j = 0; j < 4; ++j) z4[j] = ((zw >> (4 * (2 * j + (l16 >> 3)))) & 0xFu) * 0x01010101u;
    }
    const int c_begin = u * unit_chunks;
    const int c_end = min(c_begin + unit_chunks, chunks);
    for (int c = c_begin; c < c_end; ++c) {
      const u32x4_t w4 = *reinterpret_cast<const u32x4_t*>(w_lane + (long)c * kChunkWords);
      long a[MB];
#pragma unroll
      for (int rb = 0; rb < MB; ++rb) {
        const uint2 v = *reinterpret_cast<const uint2*>(a_row[rb] + (long)c * kChunkK);
        const uint32_t lo = __builtin_amdgcn_perm(v.y, v.x, 0x05010400u);   // bytes k = 0, 4, 1, 5
        const uint32_t hi = __builtin_amdgcn_perm(v.y, v.x, 0x07030602u);   // bytes k = 2, 6, 3, 7
        a[rb] = (long)(((uint64_t)hi << 32) | lo);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const long b = HAS_ZP ? ACT::word_zp(w4[j], z4[j]) : ACT::word(w4[j]);
#pragma unroll
        for (int rb = 0; rb < MB; ++rb) tmp[rb][j] = ACT::mfma(a[rb], b, tmp[rb][j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      scalar_t s = 1;
      if (GROUPED) s = group_scale<ACT, T, E8>(scales, (long)g * n + s_col[j]);   // marlin_template.h:1341-1382
#pragma unroll
      for (int rb = 0; rb < MB; ++rb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if constexpr (ACT::kInteger)
            acc[rb][j][i] += (tmp[rb][j][i] >> (HAS_ZP ? 0 : ACT::kShift)) * s;
          else
            acc[rb][j][i] += tmp[rb][j][i] * s;
        }
    }
  }
}

// The wavefronts' totals meet in LDS; afterwards wavefront w < 4 holds, in total[rb][i], the
// sums of column block w: row 16 rb + 4 (lane / 16) + i, column 16 w + lane % 16 of the tile.
template <typename ACT, int MB, int WAVES = 4>
__device__ __forceinline__ void a8_reduce(const typename ACT::acc_t (&acc)[MB][4],
                                          uint32_t (&red)[WAVES][MB * 16][64],
                                          typename ACT::scalar_t (&total)[MB][4], int wave, int lane) {
  typedef typename ACT::scalar_t scalar_t;
#pragma unroll
  for (int rb = 0; rb < MB; ++rb)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const scalar_t v = acc[rb][j][i];
        red[wave][(rb * 4 + j) * 4 + i][lane] = raw_bits(v);
      }
  __syncthreads();
  if (wave >= 4) return;
#pragma unroll
  for (int rb = 0; rb < MB; ++rb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      scalar_t sum = 0;
#pragma unroll
      for (int ww = 0; ww < WAVES; ++ww) {
        scalar_t part;
        from_raw(red[ww][(rb * 4 + wave) * 4 + i][lane], part);
        sum += part;
      }
      total[rb][i] = sum;
    }
}

// Few rows leave registers and LDS for more wavefronts: 16 for one row block, 8 for two, so that
// a workgroup walks K sixteen or eight ways and fewer calls need K split over workgroups.
template <int MB>
struct A8Waves {
  static constexpr int value = MB == 1 ? 16 : (MB == 2 ? 8 : 4);
};

template <typename ACT, typename T, int MB, bool HAS_ZP, bool GROUPED>
__global__ __launch_bounds__(64 * A8Waves<MB>::value) void marlin_a8_kernel(A8Params p) {
  typedef typename ACT::acc_t acc_t;
  typedef typename ACT::scalar_t scalar_t;
  constexpr int WAVES = A8Waves<MB>::value;
  __shared__ uint32_t red[WAVES][MB * 16][64];

  const int strip = blockIdx.x, slab = blockIdx.y, split = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int l16 = lane & 15, kb = lane >> 4;
  const int m0 = slab * (MB * 16);

  acc_t acc[MB][4];
#pragma unroll
  for (int rb = 0; rb < MB; ++rb)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[rb][j] = acc_t{0, 0, 0, 0};

  // this lane's row of A in every row block (rows past M read row M - 1, their results are dropped)
  const uint8_t* a_row[MB];
#pragma unroll
  for (int rb = 0; rb < MB; ++rb) {
    int row = m0 + 16 * rb + l16;
    if (row >= p.m) row = p.m - 1;
    a_row[rb] = p.a + (long)row * p.a_row_stride + 8 * kb;
  }
  const uint32_t* w_lane = p.w + (long)strip * p.chunks * kChunkWords + lane * 4;
  const int u_begin = split * p.units_per_split;
  const int u_end = min(u_begin + p.units_per_split, p.units);
  a8_accumulate<ACT, T, MB, HAS_ZP, GROUPED, WAVES, ACT::kE8Scales>(acc, a_row, w_lane, p.scales, p.zeros, p.n, strip,
                                                                    p.chunks, p.unit_chunks, u_begin, u_end, wave, l16);
  scalar_t total[MB][4];
  a8_reduce<ACT, MB, WAVES>(acc, red, total, wave, lane);
  if (wave >= 4) return;

  const int col = strip * kStripN + 16 * wave + l16;
  float col_scale = 1.0f, bias = 0.0f;
  if (p.splits == 1) {
    const int slot = strip * kStripN + scale_slot(16 * wave + l16, false);
    if (!GROUPED) col_scale = from_bits<T>(p.scales[slot]);
    if (p.bias) bias = from_bits<T>(p.bias[slot]);
  }
#pragma unroll
  for (int rb = 0; rb < MB; ++rb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = m0 + 16 * rb + 4 * kb + i;
      if (row >= p.m) continue;
      if (p.splits == 1)
        reinterpret_cast<uint16_t*>(p.c)[(long)row * p.n + col] =
            finish<ACT, T, GROUPED>(total[rb][i], p.a_scales[row], col_scale, bias);
      else
        p.partial[((long)split * p.m + row) * p.n + col] = raw_bits(total[rb][i]);
    }
}

// Grouped (mixture-of-experts) form: workgroup (strip, block) takes the rows
// sorted_token_ids[block * block_size ...] (row id / top_k of A, row id of C and of
// topk_weights, a_scales[id / top_k]; ids >= size_m * top_k are padding) and the expert
// expert_ids[block] (moe/marlin_moe_wna16/marlin_template.h:471-560,622-650), over the whole of K.
struct MoeA8Params {
  A8Params g;              // m = size_m (rows of A); a_scales per row of A
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_weights;
  int block_size, top_k, mul_topk, num_experts, groups, sorted_len;
};

template <typename ACT, typename T, int MB, bool HAS_ZP, bool GROUPED>
__global__ __launch_bounds__(256) void marlin_moe_a8_kernel(MoeA8Params q) {
  typedef typename ACT::acc_t acc_t;
  typedef typename ACT::scalar_t scalar_t;
  __shared__ uint32_t red[4][MB * 16][64];
  __shared__ int slot_id[16 * MB];
  const A8Params& p = q.g;

  const int strip = blockIdx.x, block = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int l16 = lane & 15, kb = lane >> 4;
  // the whole workgroup leaves together: nothing below is reached by a part of it
  if (block * q.block_size >= q.num_post_pad[0]) return;
  const int expert = q.expert_ids[block];
  if (expert < 0 || expert >= q.num_experts) return;

  const int rows_total = p.m * q.top_k;
  if (threadIdx.x < 16 * MB) {
    int id = -1;
    const int at = block * q.block_size + (int)threadIdx.x;
    if ((int)threadIdx.x < q.block_size && at < q.sorted_len) {
      id = q.sorted_ids[at];
      if (id < 0 || id >= rows_total) id = -1;
    }
    slot_id[threadIdx.x] = id;
  }
  __syncthreads();

  acc_t acc[MB][4];
#pragma unroll
  for (int rb = 0; rb < MB; ++rb)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[rb][j] = acc_t{0, 0, 0, 0};
  const uint8_t* a_row[MB];
#pragma unroll
  for (int rb = 0; rb < MB; ++rb) {
    const int id = slot_id[16 * rb + l16];
    a_row[rb] = p.a + (long)(id < 0 ? 0 : id / q.top_k) * p.a_row_stride + 8 * kb;   // padding reads row 0
  }
  const long words_per_expert = (long)p.chunks * kChunkWords * (p.n / kStripN);
  const uint32_t* w_lane = p.w + expert * words_per_expert + (long)strip * p.chunks * kChunkWords + lane * 4;
  const long scale_offset = (long)expert * q.groups * p.n;   // exponent-byte scales: one byte each
  const uint16_t* scales = ACT::kE8Scales ? reinterpret_cast<const uint16_t*>(
                                                reinterpret_cast<const uint8_t*>(p.scales) + scale_offset)
                                          : p.scales + scale_offset;
  const uint32_t* zeros = HAS_ZP ? p.zeros + (long)expert * q.groups * (p.n / 8) : nullptr;
  a8_accumulate<ACT, T, MB, HAS_ZP, GROUPED, 4, ACT::kE8Scales>(acc, a_row, w_lane, scales, zeros, p.n, strip,
                                                                p.chunks, p.unit_chunks, 0, p.units, wave, l16);
  scalar_t total[MB][4];
  a8_reduce<ACT, MB>(acc, red, total, wave, lane);

  const int col = strip * kStripN + 16 * wave + l16;
  const int slot = strip * kStripN + scale_slot(16 * wave + l16, false);
  const float col_scale = GROUPED ? 1.0f : from_bits<T>(scales[slot]);
  const float bias = p.bias ? from_bits<T>(p.bias[(long)expert * p.n + slot]) : 0.0f;
#pragma unroll
  for (int rb = 0; rb < MB; ++rb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id = slot_id[16 * rb + 4 * kb + i];
      if (id < 0) continue;
      uint16_t o = finish<ACT, T, GROUPED>(total[rb][i], p.a_scales[id / q.top_k], col_scale, bias);
      // the routing weight is rounded to the output type and the product is formed and rounded in
      // that type (marlin_template.h:1893-1897), as in the 16-bit grouped kernels
      if (q.mul_topk) o = to_bits<T>(from_bits<T>(o) * from_bits<T>(to_bits<T>(q.topk_weights[id])));
      reinterpret_cast<uint16_t*>(p.c)[(long)id * p.n + col] = o;
    }
}

// ---- the tiled kernel for many rows -----------------------------------------
// A workgroup owns a 128 x 128 tile of C; its four wavefronts own 64 x 64 quarters (wavefront
// (wr, wc): rows 64 wr, the 64-column strip 2 tile + wc) and walk K in steps of 128 (four
// chunks).  The activations of a step (128 rows x 128 bytes) go through LDS, two buffers, one
// barrier a step; on the way in every 8 bytes are shuffled into the byte order of the B
// operand and laid out so that a lane finds the bytes of one full-rate instruction side by
// side (rows 144 bytes apart: no bank conflicts).  The weights stay in registers, one step
// ahead.  GC: chunks per scale group (1, 2, 4) or 0 for channelwise scales.  Groups that
// span the K of a full-rate instruction use it (v_mfma_i32_16x16x64_i8,
// v_mfma_f32_16x16x128_f8f6f4); smaller groups take the K = 32 forms.
constexpr int kA8TileM = 128, kA8TileN = 128, kA8StepK = 128, kA8StepChunks = 4, kA8RowBytes = 144;

// MOE: the grouped form.  A workgroup is one block of up to 64 sorted slots times 256 columns;
// wavefront w owns strip 4 tile + w, so the four share the rows in LDS and none repeats another's
// dequantisation.  Rows are gathered through sorted_token_ids, the whole of K in one workgroup.
template <typename ACT, typename T, bool HAS_ZP, int GC, bool MOE = false>
__global__ __launch_bounds__(256, 2) void marlin_a8_tile_kernel(MoeA8Params q) {
  const A8Params& p = q.g;
  typedef typename ACT::acc_t acc_t;
  typedef typename ACT::scalar_t scalar_t;
  typedef typename ACT::wide_t wide_t;
  constexpr int WIDE = ACT::kWideChunks;
  constexpr bool kUseWide = GC == 0 || GC >= WIDE;
  constexpr int kGroupsPerStep = GC == 0 ? 1 : kA8StepChunks / GC;
  // uint4b8 weights enter as 16 (q - 8); the factor leaves with the group's scale, or, for channelwise
  // scales, in the epilogue (the host sends K beyond 2^16 to the slab kernel: 2^16 * 127 * 128 < 2^31)
  constexpr bool kZpForm = HAS_ZP;
  constexpr int kShift = (ACT::kInteger && !kZpForm) ? ACT::kShift : 0;
  constexpr int kRows = MOE ? 64 : kA8TileM;
  constexpr int kLoads = MOE ? 2 : 4;                       // 16-byte loads of a thread per step
  __shared__ __align__(16) uint8_t tile[2][kRows * kA8RowBytes];
  __shared__ int slot_id[64];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, kb = lane >> 4;
  const int wr = MOE ? 0 : wave >> 1, wc = MOE ? wave : wave & 1;
  const int m0 = MOE ? 0 : blockIdx.y * kA8TileM;
  const int strip = blockIdx.x * (MOE ? 4 : 2) + wc;
  const int s_begin = MOE ? 0 : blockIdx.z * p.units_per_split;
  const int s_end = MOE ? p.units : min(s_begin + p.units_per_split, p.units);

  int expert = 0;
  if (MOE) {
    // the whole workgroup leaves together: nothing below is reached by a part of it
    const int block = blockIdx.y;
    if (block * q.block_size >= q.num_post_pad[0]) return;
    expert = q.expert_ids[block];
    if (expert < 0 || expert >= q.num_experts) return;
    if (tid < 64) {
      int id = -1;
      const int at = block * q.block_size + tid;
      if (tid < q.block_size && at < q.sorted_len) {
        id = q.sorted_ids[at];
        if (id < 0 || id >= p.m * q.top_k) id = -1;
      }
      slot_id[tid] = id;
    }
    __syncthreads();
  }

  // copy role: thread t brings 64 bytes of row t / 2 of the tile (MOE: 32 bytes of row t / 4)
  const int c_row = MOE ? tid >> 2 : tid >> 1;
  const int c_off = MOE ? (tid & 3) * 32 : (tid & 1) * 64;  // first byte inside the 128 of a step
  int src_row;
  if (MOE) {
    const int id = slot_id[c_row];
    src_row = id < 0 ? 0 : id / q.top_k;                    // padding reads row 0, its results are dropped
  } else {
    src_row = m0 + c_row;
    if (src_row >= p.m) src_row = p.m - 1;                  // results of such rows are dropped
  }
  const uint8_t* a_src = p.a + (long)src_row * p.a_row_stride + c_off;
  const int dst_row = c_row * kA8RowBytes;
  const long expert_words = MOE ? (long)expert * p.chunks * kChunkWords * (p.n / kStripN) : 0;
  const uint32_t* w_lane = p.w + expert_words + (long)strip * p.chunks * kChunkWords + lane * 4;
  const uint16_t* scales = p.scales + (MOE ? (long)expert * q.groups * p.n : 0);
  const uint32_t* zeros = HAS_ZP ? p.zeros + (MOE ? (long)expert * q.groups * (p.n / 8) : 0) : nullptr;
  int s_col[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) s_col[j] = strip * kStripN + scale_slot(16 * j + l16, false);

  acc_t acc[4][4], tmp[4][4];
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[rb][j] = tmp[rb][j] = acc_t{0, 0, 0, 0};

  uint4 ra[kLoads];
  u32x4_t wq[kA8StepChunks], wq_next[kA8StepChunks];
  auto load_a = [&](int step) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      ra[i] = *reinterpret_cast<const uint4*>(a_src + (long)step * kA8StepK + 16 * i);
  };
  auto load_w = [&](int step, u32x4_t (&dst)[kA8StepChunks]) {
#pragma unroll
    for (int c = 0; c < kA8StepChunks; ++c)
      dst[c] = *reinterpret_cast<const u32x4_t*>(w_lane + (long)(step * kA8StepChunks + c) * kChunkWords);
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int off = c_off + 16 * i;                       // 16 bytes = k blocks kb0, kb0 + 1 of chunk c
      const int c = off >> 5, kb0 = ((off >> 4) & 1) * 2;
      uint2 u0, u1;
      u0.x = __builtin_amdgcn_perm(ra[i].y, ra[i].x, 0x05010400u);   // bytes k = 0, 4, 1, 5
      u0.y = __builtin_amdgcn_perm(ra[i].y, ra[i].x, 0x07030602u);   // bytes k = 2, 6, 3, 7
      u1.x = __builtin_amdgcn_perm(ra[i].w, ra[i].z, 0x05010400u);
      u1.y = __builtin_amdgcn_perm(ra[i].w, ra[i].z, 0x07030602u);
      *reinterpret_cast<uint2*>(&tile[buf][dst_row + ACT::unit_offset(c, kb0)]) = u0;
      *reinterpret_cast<uint2*>(&tile[buf][dst_row + ACT::unit_offset(c, kb0 + 1)]) = u1;
    }
  };
  // group g is complete in tmp: into acc with its scale
  auto apply_group = [&](int g) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint16_t bits = scales[(long)g * p.n + s_col[j]];
      scalar_t sc;
      if constexpr (ACT::kInteger) sc = (int)bits;
      else sc = from_bits<T>(bits);
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if constexpr (ACT::kInteger) acc[rb][j][i] += __mul24(tmp[rb][j][i] >> kShift, sc);
          else acc[rb][j][i] += tmp[rb][j][i] * sc;
        }
      }
    }
  };

  if (s_begin < s_end) {
    load_w(s_begin, wq);
    load_a(s_begin);
    store_a(0);
  }
  // Nothing is outstanding when the loop starts: otherwise the compiler's wait counts, which must
  // also hold for this first entry, make every later step wait for the loads it has only just
  // issued for the step after it.  (vmcnt = 0; the other counters untouched.)
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  for (int step = s_begin; step < s_end; ++step) {
    const int buf = (step - s_begin) & 1;
    const bool more = step + 1 < s_end;
    if (more) {
      load_w(step + 1, wq_next);
      load_a(step + 1);
    }
    // zero points of the groups of this step: word l16 % 8 of the strip's eight, nibble 2j + l16 / 8
    uint32_t zw[kGroupsPerStep];
    if (HAS_ZP) {
#pragma unroll
      for (int gi = 0; gi < kGroupsPerStep; ++gi) {
        const int g = GC == 0 ? 0 : step * kGroupsPerStep + gi;
        zw[gi] = zeros[(long)g * (p.n / 8) + strip * 8 + (l16 & 7)];
      }
    }
    const uint8_t* rows = &tile[buf][(64 * wr + l16) * kA8RowBytes];
#pragma unroll
    for (int w0 = 0; w0 < kA8StepChunks; w0 += WIDE) {
      // B operands of the WIDE chunks, every column block
      long bq[WIDE][4];
#pragma unroll
      for (int c = 0; c < WIDE; ++c) {
        const int gi = GC == 0 ? 0 : (w0 + c) / GC;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t z4 = 0x08080808u;
          if (HAS_ZP) z4 = ((zw[gi] >> (4 * (2 * j + (l16 >> 3)))) & 0xFu) * 0x01010101u;
          bq[c][j] = kZpForm ? ACT::word_zp(wq[w0 + c][j], z4) : ACT::word(wq[w0 + c][j]);
        }
      }
      // this lane's bytes of the WIDE chunks of row 16 rb + l16: side by side in LDS
      auto read_a = [&](int rb, uint32_t (&av)[2 * WIDE]) {
#pragma unroll
        for (int h = 0; h < WIDE / 2; ++h) {
          const uint4 v = *reinterpret_cast<const uint4*>(rows + rb * 16 * kA8RowBytes +
                                                          ACT::unit_offset(w0 + 2 * h, kb));
          av[4 * h + 0] = v.x; av[4 * h + 1] = v.y; av[4 * h + 2] = v.z; av[4 * h + 3] = v.w;
        }
      };
      if constexpr (kUseWide) {
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
          uint32_t av[2 * WIDE];
          read_a(rb, av);
          wide_t a;
#pragma unroll
          for (int d = 0; d < 2 * WIDE; ++d) a[d] = (int)av[d];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            wide_t b;
#pragma unroll
            for (int c = 0; c < WIDE; ++c) {
              b[2 * c] = (int)(uint32_t)bq[c][j];
              b[2 * c + 1] = (int)(uint32_t)((uint64_t)bq[c][j] >> 32);
            }
            // the first instruction of a group starts from zero: tmp needs no clearing
            if constexpr (GC == 0) acc[rb][j] = ACT::mfma_wide(a, b, acc[rb][j]);
            else if (w0 % GC == 0) tmp[rb][j] = ACT::mfma_wide(a, b, acc_t{0, 0, 0, 0});
            else tmp[rb][j] = ACT::mfma_wide(a, b, tmp[rb][j]);
          }
        }
        if constexpr (GC != 0) {
          if ((w0 + WIDE) % GC == 0) apply_group((step * kA8StepChunks + w0 + WIDE) / GC - 1);
        }
      } else {
        // groups smaller than the full-rate K: chunk by chunk, the group's scale behind its last chunk
        uint32_t av[4][2 * WIDE];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) read_a(rb, av[rb]);
#pragma unroll
        for (int c = 0; c < WIDE; ++c) {
#pragma unroll
          for (int rb = 0; rb < 4; ++rb) {
            const long a = (long)(((uint64_t)av[rb][2 * c + 1] << 32) | av[rb][2 * c]);
#pragma unroll
            for (int j = 0; j < 4; ++j)
              tmp[rb][j] = ACT::mfma(a, bq[c][j], (w0 + c) % GC == 0 ? acc_t{0, 0, 0, 0} : tmp[rb][j]);
          }
          if ((w0 + c + 1) % GC == 0) apply_group((step * kA8StepChunks + w0 + c + 1) / GC - 1);
        }
      }
    }
    if (more) {
      store_a(buf ^ 1);
#pragma unroll
      for (int c = 0; c < kA8StepChunks; ++c) wq[c] = wq_next[c];
    }
    __syncthreads();
  }

  // epilogue: lane holds rows 64 wr + 16 rb + 4 kb + i, column 16 j + l16 of its strip
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = strip * kStripN + 16 * j + l16;
    float col_scale = 1.0f, bias = 0.0f;
    if (p.splits == 1) {
      if (GC == 0) col_scale = from_bits<T>(scales[s_col[j]]);
      if (p.bias) bias = from_bits<T>(p.bias[(MOE ? (long)expert * p.n : 0) + s_col[j]]);
    }
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        scalar_t total = acc[rb][j][i];
        if constexpr (ACT::kInteger && GC == 0) total >>= kShift;
        if constexpr (MOE) {
          const int id = slot_id[16 * rb + 4 * kb + i];
          if (id < 0) continue;
          uint16_t o = finish<ACT, T, GC != 0>(total, p.a_scales[id / q.top_k], col_scale, bias);
          if (q.mul_topk) o = to_bits<T>(from_bits<T>(o) * from_bits<T>(to_bits<T>(q.topk_weights[id])));
          reinterpret_cast<uint16_t*>(p.c)[(long)id * p.n + col] = o;
          continue;
        }
        const int row = m0 + 64 * wr + 16 * rb + 4 * kb + i;
        if (row >= p.m) continue;
        if (p.splits == 1)
          reinterpret_cast<uint16_t*>(p.c)[(long)row * p.n + col] =
              finish<ACT, T, GC != 0>(total, p.a_scales[row], col_scale, bias);
        else
          p.partial[((long)blockIdx.z * p.m + row) * p.n + col] = raw_bits(total);
      }
  }
}

// Adds the raw totals of the K splits and finishes them.
template <typename ACT, typename T, bool GROUPED>
__global__ __launch_bounds__(256) void marlin_a8_finish_kernel(A8Params p) {
  typedef typename ACT::scalar_t scalar_t;
  const long total_elems = (long)p.m * p.n;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_elems;
       idx += (long)gridDim.x * blockDim.x) {
    const int row = (int)(idx / p.n), col = (int)(idx % p.n);
    scalar_t total = 0;
    for (int s = 0; s < p.splits; ++s) {
      scalar_t part;
      from_raw(p.partial[(long)s * total_elems + idx], part);
      total += part;
    }
    const int slot = (col & ~63) + scale_slot(col & 63, false);
    const float col_scale = GROUPED ? 1.0f : from_bits<T>(p.scales[slot]);
    const float bias = p.bias ? from_bits<T>(p.bias[slot]) : 0.0f;
    reinterpret_cast<uint16_t*>(p.c)[idx] = finish<ACT, T, GROUPED>(total, p.a_scales[row], col_scale, bias);
  }
}

struct A8Plan {
  bool tile;   // the tiled kernel: units are steps of 128 rows of the weights
  int mb, slabs, splits, units, unit_chunks, units_per_split;
};

A8Plan plan_a8(int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups) {
  A8Plan plan;
  // groups of 32 rows stay with the kernel above: one scale per K = 32 instruction leaves the tiled
  // kernel more scale arithmetic than matrix work, and its registers do not hold it
  plan.tile = size_m > 32 && size_k % kA8StepK == 0 && size_n % kA8TileN == 0 &&
              (num_groups == 1 ? size_k <= 65536 : size_k / num_groups >= 64);
  if (plan.tile) {
    plan.mb = 0;
    plan.slabs = (int)((size_m + kA8TileM - 1) / kA8TileM);
    plan.unit_chunks = num_groups > 1 ? (int)(size_k / num_groups) / kChunkK : 0;
    plan.units = (int)(size_k / kA8StepK);
    // fewer tiles than two per compute unit: split K, at least eight steps a workgroup
    const long tiles = (long)(size_n / kA8TileN) * plan.slabs;
    int splits = (int)(512 / tiles);
    if (splits > plan.units / 8) splits = plan.units / 8;
    if (splits > 16) splits = 16;
    if (splits < 1) splits = 1;
    plan.units_per_split = (plan.units + splits - 1) / splits;
    plan.splits = (plan.units + plan.units_per_split - 1) / plan.units_per_split;
    return plan;
  }
  plan.mb = size_m > 48 ? 4 : (int)((size_m + 15) / 16);
  plan.slabs = (int)((size_m + plan.mb * 16 - 1) / (plan.mb * 16));
  const int chunks = (int)(size_k / kChunkK);
  plan.unit_chunks = num_groups > 1 ? (int)(size_k / num_groups) / kChunkK : 4;
  plan.units = (chunks + plan.unit_chunks - 1) / plan.unit_chunks;
  // about sixteen wavefronts per compute unit, each with at least two groups
  const int waves = plan.mb == 1 ? 16 : (plan.mb == 2 ? 8 : 4);
  const long wgs = (long)(size_n / kStripN) * plan.slabs;
  int splits = (int)(4096 / (wgs * waves));
  if (splits > plan.units / (2 * waves)) splits = plan.units / (2 * waves);
  if (splits > 32) splits = 32;
  if (splits < 1) splits = 1;
  plan.units_per_split = (plan.units + splits - 1) / splits;
  plan.splits = (plan.units + plan.units_per_split - 1) / plan.units_per_split;
  return plan;
}

template <typename ACT, typename T, int MB, bool HAS_ZP>
void launch_a8_mb(const A8Params& p, bool grouped, dim3 grid, hipStream_t st) {
  constexpr int threads = 64 * A8Waves<MB>::value;
  if constexpr (ACT::kE8Scales) {   // float4 codes: always groups of 32 rows, never zero points
    static_assert(!HAS_ZP, "float4_e2m1f weights have no zero points");
    marlin_a8_kernel<ACT, T, MB, false, true><<<grid, threads, 0, st>>>(p);
  } else {
    if (grouped) marlin_a8_kernel<ACT, T, MB, HAS_ZP, true><<<grid, threads, 0, st>>>(p);
    else marlin_a8_kernel<ACT, T, MB, HAS_ZP, false><<<grid, threads, 0, st>>>(p);
  }
}

// The sum of the K ranges of a split call.
template <typename ACT, typename T>
void launch_a8_finish(const A8Params& p, bool grouped, hipStream_t st) {
  long blocks = ((long)p.m * p.n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (grouped || ACT::kE8Scales) marlin_a8_finish_kernel<ACT, T, true><<<(int)blocks, 256, 0, st>>>(p);
  else if constexpr (!ACT::kE8Scales) marlin_a8_finish_kernel<ACT, T, false><<<(int)blocks, 256, 0, st>>>(p);
}

template <typename ACT, typename T, bool HAS_ZP, bool MOE>
void launch_a8_tile_gc(const MoeA8Params& q, int gc, dim3 grid, hipStream_t st) {
  switch (gc) {
    case 0: marlin_a8_tile_kernel<ACT, T, HAS_ZP, 0, MOE><<<grid, 256, 0, st>>>(q); break;
    case 2: marlin_a8_tile_kernel<ACT, T, HAS_ZP, 2, MOE><<<grid, 256, 0, st>>>(q); break;
    default: marlin_a8_tile_kernel<ACT, T, HAS_ZP, 4, MOE><<<grid, 256, 0, st>>>(q); break;
  }
}

template <typename ACT, typename T>
void launch_a8(const A8Params& p, const A8Plan& plan, bool grouped, hipStream_t st) {
  const bool zp = p.zeros != nullptr;
  if constexpr (!ACT::kE8Scales) if (plan.tile) {
    const dim3 grid(p.n / kA8TileN, plan.slabs, plan.splits);
    MoeA8Params q = {};
    q.g = p;
    if (zp) launch_a8_tile_gc<ACT, T, true, false>(q, plan.unit_chunks, grid, st);
    else launch_a8_tile_gc<ACT, T, false, false>(q, plan.unit_chunks, grid, st);
    if (plan.splits > 1) launch_a8_finish<ACT, T>(p, grouped, st);
    return;
  }
  const dim3 grid(p.n / kStripN, plan.slabs, plan.splits);
#define SONAR_A8_CASE(MB)                                                          \
  case MB:                                                                         \
    if constexpr (!ACT::kE8Scales) {                                               \
      if (zp) {                                                                    \
        launch_a8_mb<ACT, T, MB, true>(p, grouped, grid, st);                      \
        break;                                                                     \
      }                                                                            \
    }                                                                              \
    launch_a8_mb<ACT, T, MB, false>(p, grouped, grid, st);                         \
    break;
  switch (plan.mb) {
    SONAR_A8_CASE(1)
    SONAR_A8_CASE(2)
    SONAR_A8_CASE(3)
    SONAR_A8_CASE(4)
  }
#undef SONAR_A8_CASE
  if (plan.splits > 1) launch_a8_finish<ACT, T>(p, grouped, st);
}

template <typename ACT, typename T, int MB>
void launch_moe_a8_mb(const MoeA8Params& q, bool grouped, bool zp, dim3 grid, hipStream_t st) {
  if constexpr (ACT::kE8Scales) {   // float4 codes: always groups of 32 rows, never zero points
    marlin_moe_a8_kernel<ACT, T, MB, false, true><<<grid, 256, 0, st>>>(q);
  } else if (grouped) {
    if (zp) marlin_moe_a8_kernel<ACT, T, MB, true, true><<<grid, 256, 0, st>>>(q);
    else marlin_moe_a8_kernel<ACT, T, MB, false, true><<<grid, 256, 0, st>>>(q);
  } else {
    if (zp) marlin_moe_a8_kernel<ACT, T, MB, true, false><<<grid, 256, 0, st>>>(q);
    else marlin_moe_a8_kernel<ACT, T, MB, false, false><<<grid, 256, 0, st>>>(q);
  }
}

template <typename ACT, typename T>
void launch_moe_a8(const MoeA8Params& q, bool grouped, int blocks, hipStream_t st) {
  const bool zp = q.g.zeros != nullptr;
  // blocks of more than 32 slots on shapes the tiled kernel takes (groups of 64 rows or more)
  const int gc = grouped ? q.g.unit_chunks : 0;
  if constexpr (!ACT::kE8Scales) if (q.block_size > 32 && q.g.n % 256 == 0 && q.g.chunks % kA8StepChunks == 0 && gc != 1 &&
      (grouped || q.g.chunks <= 2048)) {
    MoeA8Params t = q;
    t.g.units = q.g.chunks / kA8StepChunks;
    t.g.units_per_split = t.g.units;
    const dim3 grid(q.g.n / 256, blocks, 1);
    if (zp) launch_a8_tile_gc<ACT, T, true, true>(t, gc, grid, st);
    else launch_a8_tile_gc<ACT, T, false, true>(t, gc, grid, st);
    return;
  }
  const dim3 grid(q.g.n / kStripN, blocks, 1);
  switch ((q.block_size + 15) / 16) {
    case 1: launch_moe_a8_mb<ACT, T, 1>(q, grouped, zp, grid, st); break;
    case 2: launch_moe_a8_mb<ACT, T, 2>(q, grouped, zp, grid, st); break;
    case 3: launch_moe_a8_mb<ACT, T, 3>(q, grouped, zp, grid, st); break;
    default: launch_moe_a8_mb<ACT, T, 4>(q, grouped, zp, grid, st); break;
  }
}

// Checks shared by the dense and the grouped entry point.
int check_a8(int a_dtype, int dtype, int b_layout, int64_t b_type_id, int64_t size_m, int64_t size_n, int64_t size_k,
             int64_t num_groups, const uint32_t* b_zeros) {
  SONAR_REQUIRE(b_layout == SONAR_LAYOUT_GFX950, "unknown b_layout = %d", b_layout);
  SONAR_REQUIRE(a_dtype == SONAR_ADTYPE_INT8 || a_dtype == SONAR_ADTYPE_FP8, "unknown a_dtype = %d", a_dtype);
  SONAR_REQUIRE(dtype == SONAR_DTYPE_F16 || dtype == SONAR_DTYPE_BF16, "unknown dtype = %d", dtype);
  const bool f4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F;
  if (b_type_id != SONAR_TYPE_UINT4B8 && b_type_id != SONAR_TYPE_UINT4 && !f4)
    return fail(SONAR_E_UNSUPPORTED, "8-bit activations are built for b_type uint4b8, uint4 and float4_e2m1f only "
                "(W8A8 is not supported by the marlin kernel)");
  if (f4) {
    if (a_dtype != SONAR_ADTYPE_FP8) return fail(SONAR_E_UNSUPPORTED, "MXFP4 weight + INT8 activation is not supported.");
    SONAR_REQUIRE(num_groups >= 1 && size_k == 32 * num_groups, "float4_e2m1f weights with 8-bit activations take "
                  "one exponent-byte scale per 32 rows; got size_k = %ld, num_groups = %ld", (long)size_k,
                  (long)num_groups);
    SONAR_REQUIRE(b_zeros == nullptr, "float4_e2m1f weights have no zero points");
    // generate_kernels.py:152-161: c_type kBFloat16 only
    if (dtype != SONAR_DTYPE_BF16)
      return fail(SONAR_E_UNSUPPORTED, "float4_e2m1f weights with float8_e4m3fn activations (MXFP4) are built for "
                  "bfloat16 outputs only");
  }
  SONAR_REQUIRE(size_m >= 0 && size_n > 0 && size_k > 0, "size_m = %ld, size_n = %ld, size_k = %ld", (long)size_m,
                (long)size_n, (long)size_k);
  SONAR_REQUIRE(size_n % kStripN == 0, "size_n = %ld is not divisible by %d", (long)size_n, kStripN);
  SONAR_REQUIRE(size_k % kChunkK == 0, "size_k = %ld is not divisible by %d", (long)size_k, kChunkK);
  SONAR_REQUIRE(size_m < (1LL << 30) && size_n < (1LL << 30) && size_k < (1LL << 30), "sizes too large");
  SONAR_REQUIRE(num_groups >= 1 && size_k % num_groups == 0, "size_k = %ld is not divisible by num_groups = %ld",
                (long)size_k, (long)num_groups);
  const int64_t group_size = size_k / num_groups;
  if (num_groups > 1)
    SONAR_REQUIRE(group_size == 32 || group_size == 64 || group_size == 128,
                  "Invalid group_size = %ld: 8-bit activations take -1, 32, 64 or 128", (long)group_size);
  SONAR_REQUIRE((b_zeros != nullptr) == (b_type_id == SONAR_TYPE_UINT4),
                "b_zeros must be given for uint4 weights and only for them");
  return SONAR_OK;
}

// One 32-row group of float4 weights is a "grouped" call even when K = 32.
bool a8_grouped(int64_t b_type_id, int64_t num_groups) {
  return num_groups > 1 || b_type_id == SONAR_TYPE_FLOAT4_E2M1F;
}

}  // namespace
}  // namespace sonar

using namespace sonar;

extern "C" int sonar_moe_wna16_marlin_gemm_a8(
    const void* a, int a_dtype, void* c, const uint32_t* b_q_weight, int b_layout, const void* b_bias,
    const void* b_scales, const float* a_scales, const uint32_t* b_zeros, const int32_t* sorted_token_ids,
    int64_t sorted_len, const int32_t* expert_ids, const int32_t* num_tokens_past_padded, const float* topk_weights,
    int64_t moe_block_size, int64_t top_k, int mul_topk_weights, int64_t num_experts, int dtype, int64_t b_type_id,
    int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups, void* stream) {
  if (int rc = check_a8(a_dtype, dtype, b_layout, b_type_id, size_m, size_n, size_k, num_groups, b_zeros)) return rc;
  SONAR_REQUIRE(moe_block_size == 8 || (moe_block_size % 16 == 0 && moe_block_size >= 16 && moe_block_size <= 64),
                "unsupported moe_block_size = %ld", (long)moe_block_size);
  SONAR_REQUIRE(top_k >= 1 && num_experts >= 1, "top_k = %ld, num_experts = %ld", (long)top_k, (long)num_experts);
  SONAR_REQUIRE(sorted_len >= 0 && sorted_len < (1LL << 31), "sorted_token_ids has %ld entries", (long)sorted_len);
  SONAR_REQUIRE(!mul_topk_weights || topk_weights, "topk_weights must be given with mul_topk_weights");
  if (size_m == 0 || sorted_len == 0) return SONAR_OK;
  SONAR_REQUIRE(a && c && b_q_weight && b_scales && a_scales && sorted_token_ids && expert_ids &&
                    num_tokens_past_padded,
                "a, c, b_q_weight, b_scales, a_scales, sorted_token_ids, expert_ids and num_tokens_past_padded "
                "must not be NULL");
  SONAR_REQUIRE((uintptr_t)a % 8 == 0, "A must be aligned to 8 bytes");
  const int64_t blocks = (sorted_len + moe_block_size - 1) / moe_block_size;
  SONAR_REQUIRE(blocks <= 65535, "too many blocks of sorted tokens: %ld", (long)blocks);
  MoeA8Params q;
  A8Params& p = q.g;
  p.a = (const uint8_t*)a;
  p.a_row_stride = size_k;
  p.c = c;
  p.w = b_q_weight;
  p.scales = (const uint16_t*)b_scales;
  p.zeros = b_zeros;
  p.a_scales = a_scales;
  p.bias = (const uint16_t*)b_bias;
  p.partial = nullptr;
  p.m = (int)size_m;
  p.n = (int)size_n;
  p.chunks = (int)(size_k / kChunkK);
  p.unit_chunks = num_groups > 1 ? (int)(size_k / num_groups) / kChunkK : 4;
  p.units = (p.chunks + p.unit_chunks - 1) / p.unit_chunks;
  p.units_per_split = p.units;
  p.splits = 1;
  q.sorted_ids = sorted_token_ids;
  q.expert_ids = expert_ids;
  q.num_post_pad = num_tokens_past_padded;
  q.topk_weights = topk_weights;
  q.block_size = (int)moe_block_size;
  q.top_k = (int)top_k;
  q.mul_topk = mul_topk_weights ? 1 : 0;
  q.num_experts = (int)num_experts;
  q.groups = (int)num_groups;
  q.sorted_len = (int)sorted_len;
  const bool grouped = a8_grouped(b_type_id, num_groups);
  hipStream_t st = (hipStream_t)stream;
  if (b_type_id == SONAR_TYPE_FLOAT4_E2M1F) {
    launch_moe_a8<ActFp8F4, __bf16>(q, grouped, (int)blocks, st);   // bfloat16 outputs only (check_a8)
  } else if (a_dtype == SONAR_ADTYPE_INT8) {
    if (dtype == SONAR_DTYPE_F16) launch_moe_a8<ActInt8, _Float16>(q, grouped, (int)blocks, st);
    else launch_moe_a8<ActInt8, __bf16>(q, grouped, (int)blocks, st);
  } else {
    if (dtype == SONAR_DTYPE_F16) launch_moe_a8<ActFp8, _Float16>(q, grouped, (int)blocks, st);
    else launch_moe_a8<ActFp8, __bf16>(q, grouped, (int)blocks, st);
  }
  return launch_status("marlin_moe_a8_kernel");
}

extern "C" size_t sonar_marlin_gemm_a8_scratch_bytes(int64_t size_m, int64_t size_n, int64_t size_k,
                                                     int64_t num_groups) {
  if (size_m <= 0 || size_n <= 0 || size_k < kChunkK || num_groups < 1) return 0;
  const A8Plan plan = plan_a8(size_m, size_n, size_k, num_groups);
  return plan.splits > 1 ? (size_t)plan.splits * size_m * size_n * 4 : 0;
}

extern "C" int sonar_marlin_gemm_a8(const void* a, int64_t a_row_stride, int a_dtype, void* c, const uint32_t* b_q_weight,
                                    int b_layout, const void* b_bias, const void* b_scales, const float* a_scales,
                                    const uint32_t* b_zeros, void* scratch, size_t scratch_bytes, int dtype,
                                    int64_t b_type_id, int64_t size_m, int64_t size_n, int64_t size_k,
                                    int64_t num_groups, void* stream) {
  if (int rc = check_a8(a_dtype, dtype, b_layout, b_type_id, size_m, size_n, size_k, num_groups, b_zeros)) return rc;
  if (size_m == 0) return SONAR_OK;
  SONAR_REQUIRE(a && c && b_q_weight && b_scales && a_scales, "a, c, b_q_weight, b_scales and a_scales must not be NULL");
  SONAR_REQUIRE(a_row_stride >= size_k && a_row_stride % 8 == 0, "A.stride(0) = %ld must be at least size_k and "
                "divisible by 8", (long)a_row_stride);
  SONAR_REQUIRE((uintptr_t)a % 16 == 0, "A must aligned to 16 bytes");

  const A8Plan plan = plan_a8(size_m, size_n, size_k, num_groups);
  A8Params p;
  p.a = (const uint8_t*)a;
  p.a_row_stride = a_row_stride;
  p.c = c;
  p.w = b_q_weight;
  p.scales = (const uint16_t*)b_scales;
  p.zeros = b_zeros;
  p.a_scales = a_scales;
  p.bias = (const uint16_t*)b_bias;
  p.partial = (uint32_t*)scratch;
  p.m = (int)size_m;
  p.n = (int)size_n;
  p.chunks = (int)(size_k / kChunkK);
  p.unit_chunks = plan.unit_chunks;
  p.units = plan.units;
  p.units_per_split = plan.units_per_split;
  p.splits = plan.splits;
  if (plan.splits > 1)
    SONAR_REQUIRE(scratch && scratch_bytes >= (size_t)plan.splits * size_m * size_n * 4,
                  "scratch of %zu bytes is too small: sonar_marlin_gemm_a8_scratch_bytes() = %zu", scratch_bytes,
                  (size_t)plan.splits * size_m * size_n * 4);
  const bool grouped = a8_grouped(b_type_id, num_groups);
  hipStream_t st = (hipStream_t)stream;
  if (b_type_id == SONAR_TYPE_FLOAT4_E2M1F) {
    launch_a8<ActFp8F4, __bf16>(p, plan, grouped, st);   // bfloat16 outputs only (check_a8)
  } else if (a_dtype == SONAR_ADTYPE_INT8) {
    if (dtype == SONAR_DTYPE_F16) launch_a8<ActInt8, _Float16>(p, plan, grouped, st);
    else launch_a8<ActInt8, __bf16>(p, plan, grouped, st);
  } else {
    if (dtype == SONAR_DTYPE_F16) launch_a8<ActFp8, _Float16>(p, plan, grouped, st);
    else launch_a8<ActFp8, __bf16>(p, plan, grouped, st);
  }
  return launch_status("marlin_a8_kernel");
}
