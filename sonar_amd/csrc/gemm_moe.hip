// Grouped (mixture-of-experts) W4A16 GEMM for gfx950.
//
// moe_align_block_size hands the kernel blocks of `moe_block_size` slots, all
// of one expert; slot id < M * top_k stands for row id of C and row id / top_k
// of A (csrc/libtorch_stable/moe/marlin_moe_wna16/marlin_template.h:471-570).
// One workgroup owns one (block, 64-column strip) pair: its eight wavefronts
// split the strip's 128-row units of the block's expert between them, keep
// the next unit's operands in flight in registers, sum their accumulators
// through LDS and wavefront 0 scatters the rows to C, multiplied by the
// routing weight when asked (marlin_template.h:1883-1909).  K is never split
// across workgroups, so nothing is reduced through memory and results do not
// depend on the launch: scratch and workspace are not used.
#include <cstdlib>

#include "common.hpp"
#include "dequant.hpp"
#include "wave_reduce.hpp"

namespace sonar {

// gemm_tile.hip: the MFMA-tiled grouped kernel for 64-slot blocks
int moe_tile_gemm(const void* a, void* c, const uint32_t* b, const void* bias, const void* scales,
                  const float* global_scale, const uint32_t* zeros, const int32_t* sorted_ids, int64_t sorted_len, const int32_t* expert_ids,
                  const int32_t* num_post_pad, const float* topk_weights, int64_t top_k, int mul_topk,
                  int64_t num_experts, int32_t* table, int dtype, int64_t size_m, int64_t size_n, int64_t size_k,
                  int64_t num_groups, int group_size, int a_by_slot, bool fp4, int bits, bool fp8, void* partial,
                  size_t partial_bytes, hipStream_t st);
size_t moe_tile_table_bytes(int64_t sorted_len, int64_t num_experts);
size_t moe_tile_partial_bytes(int64_t size_k);
// gemm_stream.hip: the 16-row decode kernel in grouped form, for few rows per expert
bool moe_fast_applies(bool has_perm, int64_t moe_block_size, int64_t sorted_len, int64_t num_experts,
                      int64_t a_rows, int64_t size_n, int64_t size_k, int64_t num_groups, int group_size);
int moe_fast_gemm(const void* a, void* c, const uint32_t* b, const void* bias, const void* scales,
                  const uint32_t* zeros, const int32_t* sorted_ids, int64_t sorted_len, const int32_t* expert_ids,
                  const int32_t* num_post_pad, const float* topk_weights, int64_t moe_block_size, int64_t top_k,
                  int mul_topk, int64_t num_experts, int dtype, int64_t size_m, int64_t size_n, int64_t size_k,
                  int64_t num_groups, int group_size, int a_by_slot, bool fp4, hipStream_t st);

namespace {

constexpr int kMoeWaves = 8;

struct MoeParams {
  const uint16_t* a;
  uint16_t* c;
  const uint4* b;
  const uint16_t* bias;
  const float* global_scale;   // NVFP4: one number per expert that its output is multiplied by; else nullptr
  const uint16_t* scales;
  const uint32_t* zeros;
  const int32_t* perm;
  const int32_t* g_idx;        // [experts][size_k] group of every (sorted) row; null when groups are runs of rows
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_weights;
  int size_m, size_n, size_k;
  int num_groups, group_size;
  int chunks_per_strip, unit_chunks, units_per_strip;
  int strips;
  int block_size, top_k, num_experts, num_blocks;
  int sorted_len;
  int mul_topk;
  int a_by_slot;               // row of A = slot index (a column-permuted copy made per slot), else row id / top_k
};

template <typename T, bool HAS_PERM>
__device__ __forceinline__ typename Dq<T>::vec8 moe_load_a(const uint16_t* arow, const int32_t* perm, int k0) {
  typedef typename Dq<T>::vec8 vec8;
  uint4 v;
  if (!HAS_PERM) {
    v = *reinterpret_cast<const uint4*>(arow + k0);
  } else {
    const int4 p0 = *reinterpret_cast<const int4*>(perm + k0);
    const int4 p1 = *reinterpret_cast<const int4*>(perm + k0 + 4);
    v.x = (uint32_t)arow[p0.x] | ((uint32_t)arow[p0.y] << 16);
    v.y = (uint32_t)arow[p0.z] | ((uint32_t)arow[p0.w] << 16);
    v.z = (uint32_t)arow[p1.x] | ((uint32_t)arow[p1.y] << 16);
    v.w = (uint32_t)arow[p1.z] | ((uint32_t)arow[p1.w] << 16);
  }
  return __builtin_bit_cast(vec8, v);
}

// Wavefront 0, after the cross-wavefront sum: row `id` of C for every valid slot
// of the block, with the expert's bias and, when asked, the routing weight.
template <typename T, int MB>
__device__ __forceinline__ void moe_scatter(const MoeParams& p, const floatx4_t (&acc)[MB][4], const int* slot_id,
                                            long expert_l, int strip, int lane) {
  const int col16 = lane & 15;
  const uint16_t* bias = p.bias ? p.bias + expert_l * p.size_n + strip * kStripN : nullptr;
  const float gs = p.global_scale ? p.global_scale[expert_l] : 1.f;   // marlin_template.h(moe):1661-1665
  const int n_in = 4 * (lane >> 4);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int id = slot_id[16 * mb + col16];
    if (id < 0) continue;
    float tw = 1.f;
    // the routing weight is rounded to the activation type and the product is
    // formed and rounded in that type (marlin_template.h:1893-1897)
    if (p.mul_topk) tw = Dq<T>::to_float(Dq<T>::from_float(p.topk_weights[id]));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int nl = 16 * j + n_in;
      const floatx4_t v = acc[mb][j] * gs;
      float r[4] = {v.x, v.y, v.z, v.w};
      uint16_t o[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        float x = r[t];
        if (bias) x += Dq<T>::to_float(bias[scale_slot(nl + t, false)]);
        o[t] = Dq<T>::from_float(x);
        if (p.mul_topk) o[t] = Dq<T>::from_float(Dq<T>::to_float(o[t]) * tw);
      }
      uint2 packed;
      packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
      packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
      *reinterpret_cast<uint2*>(p.c + (long)id * p.size_n + strip * kStripN + nl) = packed;
    }
  }
}

// CHUNK_SCALES (groups of 32 rows, one per chunk: MXFP4): the scales of every
// chunk travel with the unit (eight neighbours of the permuted scale row per lane).
template <typename T, int MB, bool CHUNK_SCALES = false>
struct MoeUnit {
  uint4 q[4];
  typename Dq<T>::vec8 a[4][MB];
  uint32_t sbits[4];
  uint32_t zword;
  int group;
  uint4 sv[CHUNK_SCALES ? 4 : 1];
};

// HAS_GIDX (with HAS_PERM, symmetric weights): an act-order shard that does not
// hold whole groups (is_k_full = false); every row finds its scale through g_idx
// (marlin_moe_wna16/ops.cu:343-351).
// NV (with FP4): NVFP4, groups of 16 rows: a lane's eight rows of a chunk lie in group kb / 2 of its two.
template <typename T, int MB, bool HAS_ZP, bool HAS_PERM, bool HAS_GIDX, bool FP4 = false, bool NV = false>
__global__ __launch_bounds__(kMoeWaves * 64) void marlin_moe_kernel(const MoeParams p) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq4Of<T, FP4, NV>::type D4;   // integer codes, or float4_e2m1f
  typedef typename D4::Col Col;
  __shared__ float4 red[4][MB * 4][64];
  __shared__ int slot_id[16 * MB];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col16 = lane & 15, kb = lane >> 4;
  const int block = blockIdx.x / p.strips;
  const int strip = blockIdx.x - block * p.strips;

  // the whole workgroup leaves together: nothing below is reached by a part of it
  const int past = p.num_post_pad[0];
  if (block * p.block_size >= past) return;
  const int expert = p.expert_ids[block];
  if (expert < 0 || expert >= p.num_experts) return;

  const int rows_total = p.size_m * p.top_k;
  if (threadIdx.x < 16 * MB) {
    int id = -1;
    const int at = block * p.block_size + (int)threadIdx.x;
    if ((int)threadIdx.x < p.block_size && at < p.sorted_len) {
      id = p.sorted_ids[at];
      if (id < 0 || id >= rows_total) id = -1;
    }
    slot_id[threadIdx.x] = id;
  }
  __syncthreads();

  const uint16_t* arow[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int id = slot_id[16 * mb + col16];
    // padding slots read row 0; their products are never stored
    const int a_row = id < 0 ? 0 : (p.a_by_slot ? block * p.block_size + 16 * mb + col16 : id / p.top_k);
    arow[mb] = p.a + (long)a_row * p.size_k;
  }
  const long expert_l = expert;
  const uint4* bsrc = p.b + (expert_l * p.strips + strip) * (long)p.chunks_per_strip * 64 + lane;
  const uint16_t* scales = p.scales + expert_l * p.num_groups * p.size_n;
  const uint32_t* zeros = HAS_ZP ? p.zeros + expert_l * p.num_groups * (p.size_n / 8) : nullptr;
  const int32_t* perm = HAS_PERM ? p.perm + expert_l * p.size_k : nullptr;
  const int32_t* row_group = HAS_GIDX ? p.g_idx + expert_l * p.size_k : nullptr;
  const bool grouped = p.num_groups > 1;
  const uint32_t magic = magic_register();

  const bool chunk_scales = FP4 && grouped;
  auto load_unit = [&](MoeUnit<T, MB, FP4>& u, int unit) {
    const int chunk0 = unit * p.unit_chunks;
#pragma unroll
    for (int cc = 0; cc < 4; ++cc)
      if (cc < p.unit_chunks) u.q[cc] = bsrc[(long)(chunk0 + cc) * 64];
#pragma unroll
    for (int cc = 0; cc < 4; ++cc)
      if (cc < p.unit_chunks) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          u.a[cc][mb] = moe_load_a<T, HAS_PERM>(arow[mb], perm, (chunk0 + cc) * kChunkK + 8 * kb);
      }
    const int g = grouped ? (chunk0 * kChunkK) / p.group_size : 0;
    u.group = g;
    const uint16_t* srow = scales + (long)g * p.size_n + strip * kStripN;
    if (chunk_scales) {   // group = chunk
#pragma unroll
      for (int cc = 0; cc < 4; ++cc)
        if (cc < p.unit_chunks)
          u.sv[FP4 ? cc : 0] = *reinterpret_cast<const uint4*>(srow + (long)(NV ? 2 * cc + (kb >> 1) : cc) * p.size_n +
                                                              8 * (col16 & 7));
      return;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) u.sbits[j] = srow[scale_slot(16 * j + col16, grouped)];
    if (HAS_ZP) u.zword = zeros[(long)g * (p.size_n / 8) + strip * 8 + zero_point_word(col16)];
  };

  floatx4_t acc[MB][4];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[mb][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  MoeUnit<T, MB, FP4> cur, nxt;
  int mine = wave;
  if (mine < p.units_per_strip) load_unit(cur, mine);
  while (mine < p.units_per_strip) {
    const int next = mine + kMoeWaves;
    if (next < p.units_per_strip) load_unit(nxt, next);
    Col cols[4];
    if (!chunk_scales) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int z = 8;
        if (HAS_ZP) z = (int)((cur.zword >> zero_point_shift(16 * j + col16)) & 0xFu);
        cols[j] = D4::make_col((uint16_t)cur.sbits[j], z);
      }
    }
    int cur_group = cur.group;
    const int chunk0 = mine * p.unit_chunks;
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      if (cc < p.unit_chunks) {
        const int g = grouped ? ((chunk0 + cc) * kChunkK) / p.group_size : 0;
        if (chunk_scales) {
#pragma unroll
          for (int j = 0; j < 4; ++j) cols[j] = D4::make_col(chunk_scale(cur.sv[FP4 ? cc : 0], j, col16), 0);
        } else if (g != cur_group) {  // groups smaller than a unit
          cur_group = g;
          load_cols<T, HAS_ZP, D4>(cols, scales, zeros, p.size_n, strip, g, col16, grouped);
        }
        const uint32_t words[4] = {cur.q[cc].x, cur.q[cc].y, cur.q[cc].z, cur.q[cc].w};
        int row_groups[8];
        if (HAS_GIDX) {  // the lane's eight rows of this chunk: k = 32 chunk + 8 (lane / 16) + t
          const int4* gsrc = reinterpret_cast<const int4*>(row_group + (chunk0 + cc) * kChunkK + 8 * kb);
          const int4 g0 = gsrc[0], g1 = gsrc[1];
          row_groups[0] = g0.x, row_groups[1] = g0.y, row_groups[2] = g0.z, row_groups[3] = g0.w;
          row_groups[4] = g1.x, row_groups[5] = g1.y, row_groups[6] = g1.z, row_groups[7] = g1.w;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          vec8 w;
          if (HAS_GIDX)
            w = word_by_row_groups<T>(words[j], row_groups,
                                      scales + strip * kStripN + scale_slot(16 * j + col16, true), p.size_n, magic);
          else
            w = D4::word(words[j], cols[j], magic);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[mb][j] = Dq<T>::mfma(w, cur.a[cc][mb], acc[mb][j]);
        }
      }
    }
    cur = nxt;
    mine = next;
  }

  reduce_waves<MB, kMoeWaves>(acc, red, wave, lane);
  if (wave != 0) return;
  moe_scatter<T, MB>(p, acc, slot_id, expert_l, strip, lane);
}

// The same for 8-bit codes (uint8b128, symmetric, or float8_e4m3fn with FP8): a 32-row chunk is two 1-KiB
// blocks of 16 rows.  No gather of A: act-order experts come here through the
// per-slot permuted copy (a_by_slot).  HAS_GIDX: every row finds its scale
// through g_idx (is_k_full = false).
template <typename T, int MB, bool CHUNK_SCALES = false>
struct MoeUnit8 {
  static constexpr int kChunks = MB >= 3 ? 2 : 4;   // two units of this size and the accumulators fit the register file
  uint4 q[kChunks][2];
  typename Dq<T>::vec8 a[kChunks][MB];
  uint32_t sbits[4];
  int group;
  uint4 sv[CHUNK_SCALES ? kChunks : 1];   // groups of 32 rows: the scales of every chunk
};

// MX: groups of 32 rows, one per chunk (MXFP8; integer codes with such groups too).
template <typename T, int MB, bool HAS_GIDX, bool FP8, bool MX = false>
__global__ __launch_bounds__(kMoeWaves * 64) void marlin_moe8_kernel(const MoeParams p) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq8Of<T, FP8>::type D8;
  typedef typename D8::Col Col;
  __shared__ float4 red[4][MB * 4][64];
  __shared__ int slot_id[16 * MB];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col16 = lane & 15, kb = lane >> 4;
  const int block = blockIdx.x / p.strips;
  const int strip = blockIdx.x - block * p.strips;

  // the whole workgroup leaves together: nothing below is reached by a part of it
  const int past = p.num_post_pad[0];
  if (block * p.block_size >= past) return;
  const int expert = p.expert_ids[block];
  if (expert < 0 || expert >= p.num_experts) return;

  const int rows_total = p.size_m * p.top_k;
  if (threadIdx.x < 16 * MB) {
    int id = -1;
    const int at = block * p.block_size + (int)threadIdx.x;
    if ((int)threadIdx.x < p.block_size && at < p.sorted_len) {
      id = p.sorted_ids[at];
      if (id < 0 || id >= rows_total) id = -1;
    }
    slot_id[threadIdx.x] = id;
  }
  __syncthreads();

  const uint16_t* arow[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int id = slot_id[16 * mb + col16];
    // padding slots read row 0; their products are never stored
    const int a_row = id < 0 ? 0 : (p.a_by_slot ? block * p.block_size + 16 * mb + col16 : id / p.top_k);
    arow[mb] = p.a + (long)a_row * p.size_k;
  }
  const long expert_l = expert;
  const uint4* bsrc = p.b + (expert_l * p.strips + strip) * (long)p.chunks_per_strip * 128 + lane;
  const uint16_t* scales = p.scales + expert_l * p.num_groups * p.size_n;
  const int32_t* row_group = HAS_GIDX ? p.g_idx + expert_l * p.size_k : nullptr;
  const bool grouped = p.num_groups > 1;
  const uint32_t magic = magic_register();

  auto load_unit = [&](MoeUnit8<T, MB, MX>& u, int unit) {
    const int chunk0 = unit * p.unit_chunks;
#pragma unroll
    for (int cc = 0; cc < MoeUnit8<T, MB, MX>::kChunks; ++cc)
      if (cc < p.unit_chunks) {
        u.q[cc][0] = bsrc[(long)(chunk0 + cc) * 128];
        u.q[cc][1] = bsrc[(long)(chunk0 + cc) * 128 + 64];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          u.a[cc][mb] = moe_load_a<T, false>(arow[mb], nullptr, (chunk0 + cc) * kChunkK + 8 * kb);
      }
    const int g = grouped ? (chunk0 * kChunkK) / p.group_size : 0;
    u.group = g;
    const uint16_t* srow = scales + (long)g * p.size_n + strip * kStripN;
    if (MX) {   // group = chunk
#pragma unroll
      for (int cc = 0; cc < MoeUnit8<T, MB, MX>::kChunks; ++cc)
        if (cc < p.unit_chunks)
          u.sv[MX ? cc : 0] = *reinterpret_cast<const uint4*>(srow + (long)cc * p.size_n + 8 * (col16 & 7));
      return;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) u.sbits[j] = srow[scale_slot(16 * j + col16, grouped)];
  };

  floatx4_t acc[MB][4];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[mb][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  MoeUnit8<T, MB, MX> cur, nxt;
  int mine = wave;
  if (mine < p.units_per_strip) load_unit(cur, mine);
  while (mine < p.units_per_strip) {
    const int next = mine + kMoeWaves;
    if (next < p.units_per_strip) load_unit(nxt, next);
    Col cols[4];
    if (!MX) {
#pragma unroll
      for (int j = 0; j < 4; ++j) cols[j] = D8::make_col((uint16_t)cur.sbits[j]);
    }
    int cur_group = cur.group;
    const int chunk0 = mine * p.unit_chunks;
#pragma unroll
    for (int cc = 0; cc < MoeUnit8<T, MB, MX>::kChunks; ++cc) {
      if (cc < p.unit_chunks) {
        const int g = grouped ? ((chunk0 + cc) * kChunkK) / p.group_size : 0;
        if (MX) {
#pragma unroll
          for (int j = 0; j < 4; ++j) cols[j] = D8::make_col(chunk_scale(cur.sv[MX ? cc : 0], j, col16));
        } else if (g != cur_group) {  // groups smaller than a unit
          cur_group = g;
          const uint16_t* srow = scales + (long)g * p.size_n + strip * kStripN;
#pragma unroll
          for (int j = 0; j < 4; ++j) cols[j] = D8::make_col(srow[scale_slot(16 * j + col16, grouped)]);
        }
        const uint32_t lo[4] = {cur.q[cc][0].x, cur.q[cc][0].y, cur.q[cc][0].z, cur.q[cc][0].w};
        const uint32_t hi[4] = {cur.q[cc][1].x, cur.q[cc][1].y, cur.q[cc][1].z, cur.q[cc][1].w};
        int row_groups[8];
        if (HAS_GIDX) {  // the lane's eight rows of this chunk: k = 32 chunk + 8 (lane / 16) + t
          const int4* gsrc = reinterpret_cast<const int4*>(row_group + (chunk0 + cc) * kChunkK + 8 * kb);
          const int4 g0 = gsrc[0], g1 = gsrc[1];
          row_groups[0] = g0.x, row_groups[1] = g0.y, row_groups[2] = g0.z, row_groups[3] = g0.w;
          row_groups[4] = g1.x, row_groups[5] = g1.y, row_groups[6] = g1.z, row_groups[7] = g1.w;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint2 w_lo, w_hi;
          if (HAS_GIDX) {
            const uint16_t* scale_col = scales + strip * kStripN + scale_slot(16 * j + col16, true);
            w_lo = word4_by_row_groups8<T>(lo[j], row_groups, scale_col, p.size_n, magic);
            w_hi = word4_by_row_groups8<T>(hi[j], row_groups + 4, scale_col, p.size_n, magic);
          } else {
            w_lo = D8::word4(lo[j], cols[j], magic);
            w_hi = D8::word4(hi[j], cols[j], magic);
          }
          const vec8 w = __builtin_bit_cast(vec8, u32x4_t{w_lo.x, w_lo.y, w_hi.x, w_hi.y});
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[mb][j] = Dq<T>::mfma(w, cur.a[cc][mb], acc[mb][j]);
        }
      }
    }
    cur = nxt;
    mine = next;
  }

  reduce_waves<MB, kMoeWaves>(acc, red, wave, lane);
  if (wave != 0) return;
  moe_scatter<T, MB>(p, acc, slot_id, expert_l, strip, lane);
}

// Act-order with room in scratch: A'[slot][k] = A[row id / top_k][perm[expert][k]]
// for every valid slot, once, so that the kernels without a gather can run on
// A' (what the dense op does with permute_columns_kernel, here per slot because
// every expert has its own permutation).  One thread per 8 columns.
__global__ __launch_bounds__(256) void moe_permute_rows_kernel(const uint16_t* __restrict__ a,
                                                              const int32_t* __restrict__ perm,
                                                              const int32_t* __restrict__ sorted_ids,
                                                              const int32_t* __restrict__ expert_ids,
                                                              const int32_t* __restrict__ num_post_pad,
                                                              uint16_t* __restrict__ out, int size_k, int top_k,
                                                              int rows_total, int block_size, int sorted_len,
                                                              int num_experts) {
  const int per_row = size_k / 8;
  const long total = (long)min(sorted_len, num_post_pad[0]) * per_row;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int slot = (int)(i / per_row);
    const int k0 = 8 * (int)(i - (long)slot * per_row);
    const int expert = expert_ids[slot / block_size];
    const int id = sorted_ids[slot];
    if (expert < 0 || expert >= num_experts || id < 0 || id >= rows_total) continue;
    const uint16_t* arow = a + (long)(id / top_k) * size_k;
    const int32_t* pe = perm + (long)expert * size_k + k0;
    const int4 p0 = *reinterpret_cast<const int4*>(pe);
    const int4 p1 = *reinterpret_cast<const int4*>(pe + 4);
    uint4 v;
    v.x = (uint32_t)arow[p0.x] | ((uint32_t)arow[p0.y] << 16);
    v.y = (uint32_t)arow[p0.z] | ((uint32_t)arow[p0.w] << 16);
    v.z = (uint32_t)arow[p1.x] | ((uint32_t)arow[p1.y] << 16);
    v.w = (uint32_t)arow[p1.z] | ((uint32_t)arow[p1.w] << 16);
    *reinterpret_cast<uint4*>(out + (long)slot * size_k + k0) = v;
  }
}

template <typename T, int MB, bool HAS_ZP>
void launch_moe(const MoeParams& p, bool has_perm, int grid, hipStream_t st) {
  if (has_perm && p.g_idx) {
    if constexpr (!HAS_ZP) marlin_moe_kernel<T, MB, false, true, true><<<grid, kMoeWaves * 64, 0, st>>>(p);
  } else if (p.g_idx) {   // rows already permuted into a copy of A, groups still looked up per row
    if constexpr (!HAS_ZP) marlin_moe_kernel<T, MB, false, false, true><<<grid, kMoeWaves * 64, 0, st>>>(p);
  } else if (has_perm) {   // symmetric weights only (checked by the entry point)
    if constexpr (!HAS_ZP) marlin_moe_kernel<T, MB, false, true, false><<<grid, kMoeWaves * 64, 0, st>>>(p);
  } else {
    marlin_moe_kernel<T, MB, HAS_ZP, false, false><<<grid, kMoeWaves * 64, 0, st>>>(p);
  }
}

template <typename T, int MB>
void launch_moe8(const MoeParams& p, bool fp8, int grid, hipStream_t st) {
  // groups of 32 rows (MXFP8, or integer codes): the scales of every chunk are fetched with the unit
  const bool chunk_groups = !p.g_idx && p.num_groups > 1 && p.group_size == 32 && ((uintptr_t)p.scales) % 16 == 0;
  if (fp8 && chunk_groups) marlin_moe8_kernel<T, MB, false, true, true><<<grid, kMoeWaves * 64, 0, st>>>(p);
  else if (chunk_groups) marlin_moe8_kernel<T, MB, false, false, true><<<grid, kMoeWaves * 64, 0, st>>>(p);
  else if (fp8) marlin_moe8_kernel<T, MB, false, true><<<grid, kMoeWaves * 64, 0, st>>>(p);
  else if (p.g_idx) marlin_moe8_kernel<T, MB, true, false><<<grid, kMoeWaves * 64, 0, st>>>(p);
  else marlin_moe8_kernel<T, MB, false, false><<<grid, kMoeWaves * 64, 0, st>>>(p);
}

template <typename T>
void launch_moe8_mb(const MoeParams& p, bool fp8, int grid, hipStream_t st) {
  switch ((p.block_size + 15) / 16) {
    case 1: launch_moe8<T, 1>(p, fp8, grid, st); break;
    case 2: launch_moe8<T, 2>(p, fp8, grid, st); break;
    case 3: launch_moe8<T, 3>(p, fp8, grid, st); break;
    default: launch_moe8<T, 4>(p, fp8, grid, st); break;
  }
}

// float4_e2m1f codes: no zero points, no act-order (NV: NVFP4, scales per 16 rows)
template <typename T, bool NV = false>
void launch_moe_fp4(const MoeParams& p, int grid, hipStream_t st) {
  switch ((p.block_size + 15) / 16) {
    case 1: marlin_moe_kernel<T, 1, false, false, false, true, NV><<<grid, kMoeWaves * 64, 0, st>>>(p); break;
    case 2: marlin_moe_kernel<T, 2, false, false, false, true, NV><<<grid, kMoeWaves * 64, 0, st>>>(p); break;
    case 3: marlin_moe_kernel<T, 3, false, false, false, true, NV><<<grid, kMoeWaves * 64, 0, st>>>(p); break;
    default: marlin_moe_kernel<T, 4, false, false, false, true, NV><<<grid, kMoeWaves * 64, 0, st>>>(p); break;
  }
}

template <typename T, bool HAS_ZP>
void launch_moe_mb(const MoeParams& p, bool has_perm, int grid, hipStream_t st) {
  switch ((p.block_size + 15) / 16) {
    case 1: launch_moe<T, 1, HAS_ZP>(p, has_perm, grid, st); break;
    case 2: launch_moe<T, 2, HAS_ZP>(p, has_perm, grid, st); break;
    case 3: launch_moe<T, 3, HAS_ZP>(p, has_perm, grid, st); break;
    default: launch_moe<T, 4, HAS_ZP>(p, has_perm, grid, st); break;
  }
}

}  // namespace
}  // namespace sonar

using namespace sonar;

// the table of row tiles, rounded up so that what follows it is aligned
static size_t moe_table_room(int64_t sorted_len) {
  return (moe_tile_table_bytes(sorted_len, 0) + 255) & ~(size_t)255;
}

extern "C" size_t sonar_moe_marlin_gemm_scratch_bytes(int64_t sorted_len, int64_t moe_block_size,
                                                      int64_t size_n, int64_t size_k) {
  (void)size_n;
  // Blocks of fewer than 64 slots: K is never split across workgroups, no partial sums leave
  // the chip.  64-slot blocks: the tiled kernel keeps its table of row tiles here (one entry per
  // block) and, behind it, the fp32 partial tiles of the tiles it splits along K.
  if (moe_block_size != 64) return 0;
  return moe_table_room(sorted_len) + moe_tile_partial_bytes(size_k);
}

namespace {
// The grouped GEMM behind sonar_moe_wna16_marlin_gemm (global_scale == nullptr) and its NVFP4 form.
int moe_gemm_any(
    const void* a, void* c, const uint32_t* b_q_weight, int b_layout, const void* b_bias,
    const void* b_scales, const float* global_scale, const uint32_t* b_zeros, const int32_t* g_idx,
    const int32_t* perm, void* scratch, size_t scratch_bytes,
    const int32_t* sorted_token_ids, int64_t sorted_len, const int32_t* expert_ids,
    const int32_t* num_tokens_past_padded, const float* topk_weights, int64_t moe_block_size,
    int64_t top_k, int mul_topk_weights, int64_t num_experts, int dtype, int64_t b_type_id,
    int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups, int is_k_full, void* stream) {
  const bool nvfp4 = global_scale != nullptr;
  SONAR_REQUIRE(b_layout == SONAR_LAYOUT_GFX950, "unknown b_layout = %d", b_layout);
  SONAR_REQUIRE(dtype == SONAR_DTYPE_F16 || dtype == SONAR_DTYPE_BF16, "unsupported `a` scalar_type");
  // marlin_moe_wna16/ops.cu:560-566
  SONAR_REQUIRE(moe_block_size == 8 || (moe_block_size > 0 && moe_block_size % 16 == 0 && moe_block_size <= 64),
                "unsupported moe_block_size=%ld", (long)moe_block_size);
  SONAR_REQUIRE(top_k >= 1 && num_experts >= 1, "top_k = %ld and num_experts = %ld must be >= 1",
                (long)top_k, (long)num_experts);
  SONAR_REQUIRE(size_m >= 0 && size_m * top_k < (1LL << 30), "size_m = %ld out of range", (long)size_m);
  SONAR_REQUIRE(size_k > 0 && size_k % kChunkK == 0 && size_k < (1LL << 30),
                "size_k = %ld is not divisible by %d", (long)size_k, kChunkK);
  SONAR_REQUIRE(size_n > 0 && size_n % kStripN == 0 && size_n < (1LL << 30),
                "size_n = %ld, is not divisible by min_thread_n = %d", (long)size_n, kStripN);
  SONAR_REQUIRE(b_scales != nullptr, "b_scales must not be NULL");
  SONAR_REQUIRE(num_groups >= 1, "num_groups = %ld must be >= 1", (long)num_groups);
  if (b_type_id != SONAR_TYPE_UINT4B8 && b_type_id != SONAR_TYPE_UINT4 && b_type_id != SONAR_TYPE_UINT8B128 &&
      b_type_id != SONAR_TYPE_FLOAT8_E4M3FN && b_type_id != SONAR_TYPE_FLOAT4_E2M1F)
    return fail(SONAR_E_UNSUPPORTED,
                "b_type id %ld is not built here: only uint4b8, uint8b128 (GPTQ), uint4 (AWQ), "
                "float8_e4m3fn and float4_e2m1f (MXFP4) weights are",
                (long)b_type_id);
  const bool has_zp = b_zeros != nullptr;
  const bool fp8 = b_type_id == SONAR_TYPE_FLOAT8_E4M3FN;
  const bool fp4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F;
  const bool bits8 = b_type_id == SONAR_TYPE_UINT8B128 || fp8;
  if (has_zp)
    SONAR_REQUIRE(b_type_id == SONAR_TYPE_UINT4, "b_type must be u4 or u8 when has_zp = True");
  else
    SONAR_REQUIRE(b_type_id == SONAR_TYPE_UINT4B8 || bits8 || fp4,
                  "b_type must be uint4b8, uint8b128 or float8_e4m3fn when has_zp = False (uint4 needs b_zeros)");
  SONAR_REQUIRE((g_idx == nullptr) == (perm == nullptr), "g_idx and perm must be given together");
  bool has_perm = perm != nullptr;
  // moe/marlin_moe_wna16/generate_kernels.py:66-72: uint4 weights with zero points come without the act-order form
  // (group_blocks 0), and the op then finds no kernel
  if (has_zp && has_perm)
    return fail(SONAR_E_UNSUPPORTED, "Unsupported shapes: has_act_order = 1 with zero points (b_type uint4): "
                "act-order is built for uint4b8 and uint8b128 weights only");
  if (nvfp4) {
    // moe/marlin_moe_wna16/generate_kernels.py:94-101: NVFP4, either activation type, a scale per 16 rows
    SONAR_REQUIRE(fp4, "a global scale goes with float4_e2m1f weights only (NVFP4)");
    SONAR_REQUIRE(!has_perm, "act-order is not supported with float4_e2m1f weights");
    SONAR_REQUIRE(size_k == 16 * num_groups,
                  "float4_e2m1f weights with a global scale (NVFP4) take one scale per group of 16 rows; got "
                  "size_k = %ld, num_groups = %ld", (long)size_k, (long)num_groups);
    SONAR_REQUIRE(((uintptr_t)b_scales) % 16 == 0, "b_scales must be 16-byte aligned");
  } else if (fp4) {
    // moe/marlin_moe_wna16/generate_kernels.py:102-110: MXFP4, bfloat16 activations, a scale per 32 rows
    SONAR_REQUIRE(!has_perm, "act-order is not supported with float4_e2m1f weights");
    SONAR_REQUIRE(dtype == SONAR_DTYPE_BF16, "float4_e2m1f weights with power-of-two block scales (MXFP4) "
                  "need bfloat16 activations");
    SONAR_REQUIRE(size_k == 32 * num_groups,
                  "float4_e2m1f weights (MXFP4) take one scale per group of 32 rows; got size_k = %ld, "
                  "num_groups = %ld", (long)size_k, (long)num_groups);
    SONAR_REQUIRE(((uintptr_t)b_scales) % 16 == 0, "b_scales must be 16-byte aligned");
  }
  if (fp8) {
    // moe/marlin_moe_wna16/generate_kernels.py: channelwise scales or groups of 128 rows (:111-119: MXFP8, groups of 32), no act-order
    SONAR_REQUIRE(!has_perm, "act-order is not supported with float8_e4m3fn weights");
    SONAR_REQUIRE(num_groups == 1 || size_k == 128 * num_groups || size_k == 32 * num_groups,
                  "float8_e4m3fn weights take one scale per column, per group of 128 rows or (MXFP8) per group "
                  "of 32 rows; got size_k = %ld, num_groups = %ld", (long)size_k, (long)num_groups);
  }
  const bool row_groups = has_perm && !is_k_full;
  if (has_perm) {
    SONAR_REQUIRE(num_groups > 1, "For act_order, num_groups must be > 1");
  }
  int group_size = (int)size_k;
  if (row_groups) {
    // the shard holds no whole groups: every row looks its group up in g_idx, and the
    // kernels' own group arithmetic (one group of size_k rows) is unused
  } else if (num_groups > 1) {
    SONAR_REQUIRE(size_k % num_groups == 0, "size_k = %ld, is not divisible by num_groups = %ld",
                  (long)size_k, (long)num_groups);
    group_size = (int)(size_k / num_groups);
    SONAR_REQUIRE(nvfp4 || group_size % kChunkK == 0, "group_size = %d must be a multiple of %d", group_size,
                  kChunkK);
  }
  if (size_m == 0 || sorted_len == 0) return SONAR_OK;
  SONAR_REQUIRE(a && c && b_q_weight, "a, c and b_q_weight must not be NULL");
  SONAR_REQUIRE(sorted_token_ids && expert_ids && num_tokens_past_padded,
                "sorted_token_ids, expert_ids and num_tokens_past_padded must not be NULL");
  SONAR_REQUIRE(!mul_topk_weights || topk_weights, "topk_weights must be given when mul_topk_weights is set");
  SONAR_REQUIRE(((uintptr_t)a) % 16 == 0 && ((uintptr_t)c) % 8 == 0 && ((uintptr_t)b_q_weight) % 16 == 0,
                "a and b_q_weight must be 16-byte and c 8-byte aligned");
  SONAR_REQUIRE(sorted_len > 0 && sorted_len < (1LL << 30), "sorted_token_ids.numel = %ld out of range",
                (long)sorted_len);

  hipStream_t st = (hipStream_t)stream;
  // Act-order with whole groups and room for a copy of A per slot behind the
  // table of row tiles: permute the columns once and go on without a gather.
  int a_by_slot = 0;
  int64_t a_rows = size_m;
  {
    const size_t base = (sonar_moe_marlin_gemm_scratch_bytes(sorted_len, moe_block_size, size_n, size_k) + 255) & ~(size_t)255;
    const size_t copy_bytes = (size_t)sorted_len * size_k * 2;
    static const bool no_copy = getenv("SONAR_MARLIN_NO_MOE_PERMUTED_COPY") != nullptr;  // debugging aid
    if (has_perm && !no_copy && scratch != nullptr && scratch_bytes >= base + copy_bytes &&
        ((uintptr_t)scratch) % 16 == 0 && size_k % 8 == 0) {
      uint16_t* a_copy = reinterpret_cast<uint16_t*>(static_cast<char*>(scratch) + base);
      const long work = (long)sorted_len * (size_k / 8);
      long grid = (work + 255) / 256;
      if (grid > 16384) grid = 16384;
      moe_permute_rows_kernel<<<(int)grid, 256, 0, st>>>(static_cast<const uint16_t*>(a), perm, sorted_token_ids,
                                                         expert_ids, num_tokens_past_padded, a_copy, (int)size_k,
                                                         (int)top_k, (int)(size_m * top_k), (int)moe_block_size,
                                                         (int)sorted_len, (int)num_experts);
      if (int rc = launch_status("moe_permute_rows_kernel")) return rc;
      a = a_copy;
      a_by_slot = 1;
      a_rows = sorted_len;
      has_perm = false;
      perm = nullptr;
      if (!row_groups) g_idx = nullptr;   // shards without whole groups still look every row's group up
      scratch_bytes = base;   // what is left for the table of row tiles
    }
  }
  if (bits8 && has_perm)
    return fail(SONAR_E_INVALID,
                "act-order with 8-bit expert weights needs sorted_len * size_k * 2 more scratch bytes "
                "(the column-permuted copy of A per slot)");
  // Few rows per expert: the decode kernel, one workgroup per strip and 32 slots of a block
  if (!bits8 && !row_groups && !nvfp4 &&
      moe_fast_applies(has_perm, moe_block_size, sorted_len, num_experts, a_rows, size_n, size_k, num_groups,
                       group_size))
    return moe_fast_gemm(a, c, b_q_weight, b_bias, b_scales, b_zeros, sorted_token_ids, sorted_len, expert_ids,
                         num_tokens_past_padded, topk_weights, moe_block_size, top_k, mul_topk_weights ? 1 : 0,
                         num_experts, dtype, size_m, size_n, size_k, num_groups, group_size, a_by_slot, fp4, st);
  static const bool no_tile = getenv("SONAR_MARLIN_NO_MOE_TILE") != nullptr;  // debugging aid
  // Full blocks of 64 slots mean many rows per expert: the MFMA-tiled kernel
  if (moe_block_size == 64 && !has_perm && !row_groups && !no_tile && size_k % 64 == 0 &&
      (num_groups == 1 || group_size % 64 == 0 || group_size == 32 || nvfp4) && scratch != nullptr &&
      scratch_bytes >= moe_tile_table_bytes(sorted_len, num_experts) && ((uintptr_t)scratch) % 4 == 0)
    return moe_tile_gemm(a, c, b_q_weight, b_bias, b_scales, global_scale, b_zeros, sorted_token_ids, sorted_len, expert_ids,
                         num_tokens_past_padded, topk_weights, top_k, mul_topk_weights ? 1 : 0, num_experts,
                         static_cast<int32_t*>(scratch), dtype, size_m, size_n, size_k, num_groups, group_size,
                         a_by_slot, fp4, bits8 ? 8 : 4, fp8, static_cast<char*>(scratch) + moe_table_room(sorted_len),
                         scratch_bytes > moe_table_room(sorted_len) ? scratch_bytes - moe_table_room(sorted_len) : 0, st);

  MoeParams p;
  p.a = static_cast<const uint16_t*>(a);
  p.c = static_cast<uint16_t*>(c);
  p.b = reinterpret_cast<const uint4*>(b_q_weight);
  p.bias = static_cast<const uint16_t*>(b_bias);
  p.global_scale = global_scale;
  p.scales = static_cast<const uint16_t*>(b_scales);
  p.zeros = b_zeros;
  p.perm = perm;
  p.g_idx = row_groups ? g_idx : nullptr;
  p.sorted_ids = sorted_token_ids;
  p.expert_ids = expert_ids;
  p.num_post_pad = num_tokens_past_padded;
  p.topk_weights = topk_weights;
  p.size_m = (int)size_m;
  p.size_n = (int)size_n;
  p.size_k = (int)size_k;
  p.num_groups = (int)num_groups;
  p.group_size = group_size;
  p.chunks_per_strip = (int)(size_k / kChunkK);
  p.unit_chunks = p.chunks_per_strip % 4 == 0 ? 4 : (p.chunks_per_strip % 2 == 0 ? 2 : 1);
  p.units_per_strip = p.chunks_per_strip / p.unit_chunks;
  p.strips = (int)(size_n / kStripN);
  p.block_size = (int)moe_block_size;
  p.top_k = (int)top_k;
  p.num_experts = (int)num_experts;
  p.sorted_len = (int)sorted_len;
  p.num_blocks = (int)((sorted_len + moe_block_size - 1) / moe_block_size);
  p.mul_topk = mul_topk_weights ? 1 : 0;
  p.a_by_slot = a_by_slot;
  const int64_t grid = (int64_t)p.num_blocks * p.strips;
  SONAR_REQUIRE(grid < (1LL << 31), "too many (block, strip) pairs: %ld", (long)grid);
  if (bits8) {
    if (p.block_size > 32 && p.unit_chunks == 4) {   // MoeUnit8 holds two chunks from three blocks of rows on
      p.unit_chunks = 2;
      p.units_per_strip = p.chunks_per_strip / 2;
    }
    if (dtype == SONAR_DTYPE_F16) launch_moe8_mb<_Float16>(p, fp8, (int)grid, st);
    else launch_moe8_mb<__bf16>(p, fp8, (int)grid, st);
    return launch_status("marlin_moe8_kernel");
  }
  if (nvfp4) {
    if (dtype == SONAR_DTYPE_F16) launch_moe_fp4<_Float16, true>(p, (int)grid, st);
    else launch_moe_fp4<__bf16, true>(p, (int)grid, st);
    return launch_status("marlin_moe_kernel");
  }
  if (fp4) {
    launch_moe_fp4<__bf16>(p, (int)grid, st);
    return launch_status("marlin_moe_kernel");
  }
  if (dtype == SONAR_DTYPE_F16) {
    if (has_zp) launch_moe_mb<_Float16, true>(p, has_perm, (int)grid, st);
    else launch_moe_mb<_Float16, false>(p, has_perm, (int)grid, st);
  } else {
    if (has_zp) launch_moe_mb<__bf16, true>(p, has_perm, (int)grid, st);
    else launch_moe_mb<__bf16, false>(p, has_perm, (int)grid, st);
  }
  return launch_status("marlin_moe_kernel");
}
}  // namespace

extern "C" int sonar_moe_wna16_marlin_gemm(
    const void* a, void* c, const uint32_t* b_q_weight, int b_layout, const void* b_bias,
    const void* b_scales, const uint32_t* b_zeros, const int32_t* g_idx, const int32_t* perm,
    int32_t* workspace, int64_t workspace_len, void* scratch, size_t scratch_bytes,
    const int32_t* sorted_token_ids, int64_t sorted_len, const int32_t* expert_ids,
    const int32_t* num_tokens_past_padded, const float* topk_weights, int64_t moe_block_size,
    int64_t top_k, int mul_topk_weights, int64_t num_experts, int dtype, int64_t b_type_id,
    int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups, int is_k_full,
    int use_atomic_add, int use_fp32_reduce, void* stream) {
  (void)workspace;
  (void)workspace_len;
  (void)use_atomic_add;
  (void)use_fp32_reduce;
  return moe_gemm_any(a, c, b_q_weight, b_layout, b_bias, b_scales, nullptr, b_zeros, g_idx, perm, scratch,
                      scratch_bytes, sorted_token_ids, sorted_len, expert_ids, num_tokens_past_padded, topk_weights,
                      moe_block_size, top_k, mul_topk_weights, num_experts, dtype, b_type_id, size_m, size_n, size_k,
                      num_groups, is_k_full, stream);
}

extern "C" int sonar_moe_wna16_marlin_gemm_nvfp4(
    const void* a, void* c, const uint32_t* b_q_weight, int b_layout, const void* b_bias,
    const void* b_scales, const float* global_scale, void* scratch, size_t scratch_bytes,
    const int32_t* sorted_token_ids, int64_t sorted_len, const int32_t* expert_ids,
    const int32_t* num_tokens_past_padded, const float* topk_weights, int64_t moe_block_size,
    int64_t top_k, int mul_topk_weights, int64_t num_experts, int dtype, int64_t size_m, int64_t size_n,
    int64_t size_k, int64_t num_groups, void* stream) {
  SONAR_REQUIRE(global_scale != nullptr, "the global_scale parameter must be passed for nvfp4 format.");
  return moe_gemm_any(a, c, b_q_weight, b_layout, b_bias, b_scales, global_scale, nullptr, nullptr, nullptr, scratch,
                      scratch_bytes, sorted_token_ids, sorted_len, expert_ids, num_tokens_past_padded, topk_weights,
                      moe_block_size, top_k, mul_topk_weights, num_experts, dtype, SONAR_TYPE_FLOAT4_E2M1F, size_m,
                      size_n, size_k, num_groups, 1, stream);
}
