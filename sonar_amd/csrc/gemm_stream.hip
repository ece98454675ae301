// Streaming W4A16 / W8A16 GEMM for the bandwidth-bound regime: up to 64
// activation rows per workgroup (up to 128 rows per launch of the fast kernel).
//
// Work decomposition.  The packed weights are a list of strips (64 output
// columns each), every strip a contiguous run of K/32 one-KiB chunks.  The list
// of all (strip, unit) pairs - a unit is `unit_chunks` consecutive chunks - is
// cut into equal contiguous ranges, one per workgroup, so every compute unit
// streams the same number of bytes whatever the shape.  The units of a range
// are dealt round-robin to the workgroup's wavefronts; each wavefront keeps
// MB x 4 accumulator tiles (16 rows x 16 columns) and feeds
// v_mfma_f32_16x16x32 with the dequantised weights as the row operand and the
// activations as the column operand.  At the end of every strip segment the
// wavefronts' tiles are summed through LDS.  A segment that covers the whole K
// of its strip is rounded and written to C.  A partial segment is written as
// an fp32 tile to scratch memory; a second, tiny kernel adds the (two to five)
// partial tiles of each split strip in a fixed order and writes C.  Nothing
// spins, nothing is atomic, and the result does not depend on timing.  Short
// strips (K <= 4096) on a wide matrix get one workgroup each instead, which
// shares nothing and needs no second kernel.
#include <cstdlib>

#include "dequant.hpp"
#include "gemm_plan.hpp"
#include "wave_reduce.hpp"

namespace sonar {

// gemm_tile.hip: the MFMA-bound kernel for more than 64 rows
int tile_gemm(const void* a, int64_t a_row_stride, void* c, const uint32_t* b, const void* bias,
              const void* scales, const float* global_scale, const uint32_t* zeros, const int32_t* perm, int dtype,
              int64_t size_m,
              int64_t size_n, int64_t size_k, int64_t num_groups, int group_size, void* partial,
              size_t partial_bytes, bool fp4, int bits, bool fp8, hipStream_t st);
bool tile_async_applies(bool has_perm, int64_t num_groups, int group_size);

namespace {

constexpr int kWaves = 8;
constexpr int kSlotFloat4 = 4 * 4 * 64;  // largest partial tile: 4 row blocks x 4 column blocks x 64 lanes

struct StreamParams {
  const uint16_t* a;
  long lda;
  uint16_t* c;
  const uint4* b;
  const uint16_t* bias;
  const float* global_scale;   // NVFP4: one number the output is multiplied by; else nullptr
  const uint16_t* scales;
  const uint32_t* zeros;
  const int32_t* perm;
  const int32_t* g_idx;  // group of every row of W; null when groups are runs of group_size rows
  float4* scratch;
  int size_m, size_n, size_k;
  int num_groups, group_size;
  int chunks_per_strip;
  int unit_chunks;
  int units_per_strip;
  int parts;  // number of workgroups of the streaming kernel
  int total_units;
  // The launch covers `slabs` blocks of rows (16 or 32 in the fast kernel, 64 in
  // the general kernels) times `grid_parts` >= parts workgroups per block
  // (part_and_slab; parts past `parts` are padding)
  int slabs, grid_parts;
  // fast kernel only: with `tickets` the strips shared between workgroups are
  // summed inside the kernel.  Every contributor stores its fp32 partial tiles
  // with agent-scope (write-through) stores, waits for them, and draws a ticket
  // of the strip with one relaxed atomic add; the workgroup that draws the last
  // ticket reads all the partial tiles back with agent-scope loads, adds them in
  // workgroup order (the same bits whoever comes last), writes C and puts the
  // ticket back to zero.  Nobody waits for anybody, so nothing can hang.  Ticket
  // of the strip whose first contributor is `first`, for block of rows `slab`:
  // tickets[(first * slabs + slab) * ticket_stride].  Without `tickets` the
  // fix-up kernel adds the partial tiles.
  unsigned int* tickets;
  int ticket_stride;
  // workgroup ids are dealt to the parts so that consecutive parts (which share
  // strips and rows of A) have ids congruent mod 8, i.e. sit on one XCD
  int xcd_ranges;
  // fast kernel only: piece_units > 0 says that every strip is cut into 2^piece_shift
  // pieces of piece_units units, part (strip << piece_shift) + i being piece i: the
  // kernel then finds its range with shifts instead of the divisions of the general
  // split (a wavefront's scalar unit is shared with seven others: the index arithmetic
  // of the general split alone took about 0.4 us before the first copy was issued)
  int piece_shift, piece_units;
  int nt_weights;   // fast kernel only: copy the weights with the non-temporal bit
  // grouped (mixture-of-experts) calls of the fast kernel only: workgroup
  // block * grid_parts + strip works on the slots [block * block_size, ...) of
  // sorted_ids with the weights of expert_ids[block]; blocks of 48 and 64 slots
  // are split between two workgroups (`slab` = block * sub_blocks + half)
  const int32_t* sorted_ids;   // slot -> row id of C (row id / top_k of A); outside [0, rows_total): padding
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_weights;
  int block_size, top_k, num_experts, rows_total, sorted_len, mul_topk;
  int sub_blocks;              // workgroups (of up to 32 rows) per block of slots and strip
  int a_by_slot;               // row of A = slot index (a column-permuted copy made per slot), else row id / top_k
  long expert_b_stride;        // uint4 units between experts in b
  long expert_s_stride, expert_z_stride, expert_bias_stride;  // elements between experts
};

// Unit indices are 32-bit: the host checks total_units * parts < 2^31.
__host__ __device__ __forceinline__ int range_begin(int i, int total, int parts) {
  return (int)((unsigned)i * (unsigned)total / (unsigned)parts);
}
// Largest i with range_begin(i) <= x, given parts <= total.
__host__ __device__ __forceinline__ int range_owner(int x, int total, int parts) {
  return (int)((((unsigned)x + 1u) * (unsigned)parts - 1u) / (unsigned)total);
}
// Workgroup id -> (part, slab) of a launch that covers `slabs` blocks of rows.
// With several slabs grid_parts is a multiple of 8 and the slabs of a part get
// consecutive ids on one XCD (ids congruent mod 8), so that they are dispatched
// together and the second to ask for a weight chunk finds it in that XCD's L2.
__device__ __forceinline__ void part_and_slab(const int grid_parts, const int slabs, int& part, int& slab,
                                              const int xcd_ranges = 0) {
  if (slabs == 1) {
    // xcd_ranges (grid_parts % 8 == 0): ids congruent mod 8 get a contiguous run of parts
    part = xcd_ranges ? (int)(blockIdx.x & 7) * (grid_parts >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    slab = 0;
    return;
  }
  const int t = blockIdx.x >> 3;
  slab = t % slabs;
  part = (t / slabs) * 8 + (blockIdx.x & 7);
}
// Scratch slot of workgroup `w` for a strip whose first contributor is `first`.
__device__ __forceinline__ float4* partial_slot(const StreamParams& p, int w, int first) {
  return p.scratch + (long)(w == first ? p.parts + w : w) * kSlotFloat4;
}

template <typename T, bool HAS_PERM>
__device__ __forceinline__ typename Dq<T>::vec8 load_a(const StreamParams& p, int row, int k0) {
  typedef typename Dq<T>::vec8 vec8;
  // rows past M are clamped: their products are computed and never stored
  const uint16_t* arow = p.a + (long)(row < p.size_m ? row : p.size_m - 1) * p.lda;
  uint4 v;
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
  return __builtin_bit_cast(vec8, v);
}

// Adds bias, rounds and stores the MB x 4 tiles held by one wavefront.
template <typename T, int MB>
__device__ __forceinline__ void write_tiles(const StreamParams& p, int strip, int lane,
                                            const floatx4_t (&acc)[MB][4]) {
  const int m_in = lane & 15;
  const int n_in = 4 * (lane >> 4);
  const float gs = p.global_scale ? *p.global_scale : 1.f;   // marlin_template.h:1661-1665
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
        const floatx4_t v = acc[mb][j] * gs;
        uint2 o;
        o.x = (uint32_t)Dq<T>::from_float(v.x + b[0]) | ((uint32_t)Dq<T>::from_float(v.y + b[1]) << 16);
        o.y = (uint32_t)Dq<T>::from_float(v.z + b[2]) | ((uint32_t)Dq<T>::from_float(v.w + b[3]) << 16);
        *reinterpret_cast<uint2*>(p.c + (long)m * p.size_n + strip * kStripN + nl) = o;
      }
    }
  }
}

// Wavefront 0: a finished segment goes to C when it is the whole strip, else
// to this workgroup's scratch slot.
template <typename T, int MB>
__device__ __forceinline__ void finish_segment(const StreamParams& p, int part, int strip, int seg_begin,
                                               int seg_end, int lane, const floatx4_t (&acc)[MB][4]) {
  const int strip_first = strip * p.units_per_strip;
  const int strip_end = strip_first + p.units_per_strip;
  if (seg_begin == strip_first && seg_end == strip_end) {
    write_tiles<T, MB>(p, strip, lane, acc);
    return;
  }
  const int first = range_owner(strip_first, p.total_units, p.parts);
  float4* slot = partial_slot(p, part, first);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const floatx4_t v = acc[mb][j];
      slot[(mb * 4 + j) * 64 + lane] = make_float4(v.x, v.y, v.z, v.w);
    }
}

// The same for one 16-column block (j) of a 16-row tile, held by one wavefront.
// `c_block` is row 0 of the tile in C and `rows` the rows of it that exist;
// `part` is the workgroup's index in the partition and `slab` the tile's block
// of 16 rows (fast kernel: several blocks of rows share one launch; the scratch
// slot of a part holds one partial tile per block of rows).
// Adds bias, rounds and stores one 16 x 16 block (column block j of a strip) held by one wavefront.
template <typename T>
__device__ __forceinline__ void store_c_block(const StreamParams& p, uint16_t* c_block, int rows, int strip, int lane,
                                              int j, floatx4_t v) {
  const int m = lane & 15;
  const int nl = 16 * j + 4 * (lane >> 4);
  if (m < rows) {
    float b[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        b[r] = Dq<T>::to_float(p.bias[strip * kStripN + scale_slot(nl + r, false)]);
    }
    uint2 o;
    o.x = (uint32_t)Dq<T>::from_float(v.x + b[0]) | ((uint32_t)Dq<T>::from_float(v.y + b[1]) << 16);
    o.y = (uint32_t)Dq<T>::from_float(v.z + b[2]) | ((uint32_t)Dq<T>::from_float(v.w + b[3]) << 16);
    *reinterpret_cast<uint2*>(c_block + (long)m * p.size_n + strip * kStripN + nl) = o;
  }
}

// One 16 x 16 fp32 block of a strip that several workgroups share goes to this
// workgroup's scratch slot (`tile` = 4 x block of rows + column block).
__device__ __forceinline__ void store_partial_block(const StreamParams& p, int part, int first, int tile, int lane,
                                                    floatx4_t v) {
  float4* dst = partial_slot(p, part, first) + tile * 64 + lane;
  if (p.tickets) {  // read back by another workgroup of this launch: write through to memory
    unsigned long long* d = reinterpret_cast<unsigned long long*>(dst);
    const unsigned long long lo = ((unsigned long long)__float_as_uint(v.y) << 32) | __float_as_uint(v.x);
    const unsigned long long hi = ((unsigned long long)__float_as_uint(v.w) << 32) | __float_as_uint(v.z);
    __hip_atomic_store(d, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(d + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    *dst = make_float4(v.x, v.y, v.z, v.w);
  }
}

// The partial tile (block of rows `slab`, column block j) that workgroup w left for a
// strip whose first contributor is `first`.  NEAR: the writer ran on this workgroup's
// XCD, whose L2 is the point of coherence for its compute units, so the load only has
// to pass the compute unit's own cache (which cannot hold the line: this workgroup has
// not read it since the cache was invalidated at kernel start); otherwise an
// agent-scope load, which is answered from beyond the L2.
template <bool NEAR>
__device__ __forceinline__ floatx4_t load_partial_tile(const StreamParams& p, int w, int first, int slab, int j,
                                                       int lane) {
  const unsigned long long* src =
      reinterpret_cast<const unsigned long long*>(partial_slot(p, w, first) + (slab * 4 + j) * 64 + lane);
  unsigned long long lo, hi;
  if constexpr (NEAR) {
    lo = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    hi = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  } else {
    lo = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    hi = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  return floatx4_t{__uint_as_float((unsigned)lo), __uint_as_float((unsigned)(lo >> 32)),
                   __uint_as_float((unsigned)hi), __uint_as_float((unsigned)(hi >> 32))};
}

// Sum of the partial tiles of workgroups first..last, four loads in flight at a time, added
// in workgroup order.
template <bool NEAR>
__device__ __forceinline__ floatx4_t sum_partial_tiles(const StreamParams& p, int first, int last, int slab, int j,
                                                       int lane) {
  floatx4_t sum = floatx4_t{0.f, 0.f, 0.f, 0.f};
  for (int w0 = first; w0 <= last; w0 += 4) {
    floatx4_t part4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      part4[i] = load_partial_tile<NEAR>(p, w0 + i <= last ? w0 + i : last, first, slab, j, lane);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (w0 + i <= last) sum += part4[i];
  }
  return sum;
}

// Grouped calls: the tile's row (lane & 15) goes to row `id` of C (none when
// id < 0), with the expert's bias and, when asked, the routing weight: the
// weight is rounded to the activation type and the product is formed and
// rounded in that type (marlin_moe_wna16/marlin_template.h:1883-1909).
template <typename T>
__device__ __forceinline__ void finish_block_grouped(const StreamParams& p, int id, int strip, int lane, int j,
                                                     floatx4_t v) {
  if (id < 0) return;
  const int nl = 16 * j + 4 * (lane >> 4);
  const float r[4] = {v.x, v.y, v.z, v.w};
  float tw = 1.f;
  if (p.mul_topk) tw = Dq<T>::to_float(Dq<T>::from_float(p.topk_weights[id]));
  uint16_t o[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    float x = r[t];
    if (p.bias) x += Dq<T>::to_float(p.bias[strip * kStripN + scale_slot(nl + t, false)]);
    o[t] = Dq<T>::from_float(x);
    if (p.mul_topk) o[t] = Dq<T>::from_float(Dq<T>::to_float(o[t]) * tw);
  }
  uint2 packed;
  packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
  packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
  *reinterpret_cast<uint2*>(p.c + (long)id * p.size_n + strip * kStripN + nl) = packed;
}

// ---------------------------------------------------------------------------
// General kernel: any M <= 64, any K % 32 == 0, any group size that is a
// multiple of 32, optional act-order gather of A.  Operands are fetched into
// registers one unit ahead.
// With three or four 16-row blocks a unit buffer holds two chunks instead of
// four (the host halves the unit), which keeps the two buffers and the
// accumulators inside the register file.
template <int MB>
constexpr int unit_buffer_chunks() { return MB >= 3 ? 2 : 4; }

// CHUNK_SCALES (groups of 32 rows, one per chunk: MXFP4): the scales of every
// chunk travel with the unit, eight neighbours of the permuted scale row per
// lane (16 bytes) of which it uses four, instead of being fetched when the
// chunk is reached.
template <typename T, int MB, bool CHUNK_SCALES = false>
struct UnitBuf {
  uint4 q[unit_buffer_chunks<MB>()];
  typename Dq<T>::vec8 a[unit_buffer_chunks<MB>()][MB];
  uint32_t sbits[4];
  uint32_t zword;
  int group;
  uint4 sv[CHUNK_SCALES ? unit_buffer_chunks<MB>() : 1];
};

// NV (with CHUNK_SCALES): groups of 16 rows, two per chunk; a lane's eight rows, 8 kb .. 8 kb + 7,
// lie in group kb / 2 of the chunk, and that is the row of scales it fetches.
template <typename T, int MB, bool HAS_ZP, bool HAS_PERM, bool CHUNK_SCALES = false, bool NV = false>
__device__ __forceinline__ void load_unit(UnitBuf<T, MB, CHUNK_SCALES>& b, const StreamParams& p, int u, int lane,
                                          bool grouped) {
  const int col16 = lane & 15, kb = lane >> 4;
  const int strip = u / p.units_per_strip;
  const int unit = u - strip * p.units_per_strip;
  const int chunk0 = unit * p.unit_chunks;
  const uint4* bsrc = p.b + ((long)strip * p.chunks_per_strip + chunk0) * 64 + lane;
#pragma unroll
  for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc)
    if (cc < p.unit_chunks) b.q[cc] = bsrc[cc * 64];
#pragma unroll
  for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc)
    if (cc < p.unit_chunks) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        b.a[cc][mb] = load_a<T, HAS_PERM>(p, 16 * mb + col16, (chunk0 + cc) * kChunkK + 8 * kb);
    }
  const int g = grouped ? (chunk0 * kChunkK) / p.group_size : 0;
  b.group = g;
  const uint16_t* srow = p.scales + (long)g * p.size_n + strip * kStripN;
  if (CHUNK_SCALES && grouped) {   // group = chunk
#pragma unroll
    for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc)
      if (cc < p.unit_chunks)
        b.sv[cc] = *reinterpret_cast<const uint4*>(srow + (long)(NV ? 2 * cc + (kb >> 1) : cc) * p.size_n +
                                                   8 * (col16 & 7));
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) b.sbits[j] = srow[scale_slot(16 * j + col16, grouped)];
  if (HAS_ZP) b.zword = p.zeros[(long)g * (p.size_n / 8) + strip * 8 + zero_point_word(col16)];
}

template <typename T, int MB, bool HAS_ZP, bool HAS_PERM, bool HAS_GIDX, bool FP4 = false, bool NV = false>
__global__ __launch_bounds__(kWaves * 64) void marlin_stream_kernel(const StreamParams params) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq4Of<T, FP4, NV>::type D4;   // integer codes, or float4_e2m1f (NV: scales per 16 rows)
  typedef typename D4::Col Col;
  __shared__ float4 red[4][MB * 4][64];
  // Several 64-row slabs can share a launch when no strip is shared between
  // workgroups (nothing goes through the scratch slots).
  StreamParams p = params;
  int part, slab;
  part_and_slab(p.grid_parts, p.slabs, part, slab);
  if (part >= p.parts) return;
  {
    p.a += (long)slab * 64 * p.lda;
    p.c += (long)slab * 64 * p.size_n;
    p.size_m = min(64, p.size_m - 64 * slab);
  }

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col16 = lane & 15;
  const int u_begin = range_begin(part, p.total_units, p.parts);
  const int u_end = range_begin(part + 1, p.total_units, p.parts);
  const bool grouped = p.num_groups > 1;
  const uint32_t magic = magic_register();

  UnitBuf<T, MB, FP4> cur, nxt;
  int mine = u_begin + wave;
  if (mine < u_end) load_unit<T, MB, HAS_ZP, HAS_PERM, FP4, NV>(cur, p, mine, lane, grouped);

  int seg_begin = u_begin;
  while (seg_begin < u_end) {
    const int strip = seg_begin / p.units_per_strip;
    const int strip_first = strip * p.units_per_strip;
    const int strip_end = strip_first + p.units_per_strip;
    const int seg_end = u_end < strip_end ? u_end : strip_end;

    floatx4_t acc[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[mb][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    while (mine < seg_end) {
      const int next = mine + kWaves;
      if (next < u_end) load_unit<T, MB, HAS_ZP, HAS_PERM, FP4, NV>(nxt, p, next, lane, grouped);
      Col cols[4];
      const bool chunk_scales = FP4 && grouped;   // the scales of every chunk came with the unit
      if (!chunk_scales) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          int z = 8;
          if (HAS_ZP) z = (int)((cur.zword >> zero_point_shift(16 * j + col16)) & 0xFu);
          cols[j] = D4::make_col((uint16_t)cur.sbits[j], z);
        }
      }
      int cur_group = cur.group;
      const int chunk0 = (mine - strip_first) * p.unit_chunks;
#pragma unroll
      for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc) {
        if (cc < p.unit_chunks) {
          const int g = grouped ? ((chunk0 + cc) * kChunkK) / p.group_size : 0;
          if (chunk_scales) {
#pragma unroll
            for (int j = 0; j < 4; ++j) cols[j] = D4::make_col(chunk_scale(cur.sv[FP4 ? cc : 0], j, col16), 0);
          } else if (g != cur_group) {  // groups smaller than a unit
            cur_group = g;
            load_cols<T, HAS_ZP, D4>(cols, p.scales, p.zeros, p.size_n, strip, g, col16, grouped);
          }
          const uint32_t words[4] = {cur.q[cc].x, cur.q[cc].y, cur.q[cc].z, cur.q[cc].w};
          int row_groups[8];
          if (HAS_GIDX) {  // the lane's eight rows of this chunk: k = 32 chunk + 8 (lane / 16) + t
            const int4* gsrc = reinterpret_cast<const int4*>(p.g_idx + (chunk0 + cc) * kChunkK + 8 * (lane >> 4));
            const int4 g0 = gsrc[0], g1 = gsrc[1];
            row_groups[0] = g0.x, row_groups[1] = g0.y, row_groups[2] = g0.z, row_groups[3] = g0.w;
            row_groups[4] = g1.x, row_groups[5] = g1.y, row_groups[6] = g1.z, row_groups[7] = g1.w;
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            vec8 w;
            if (HAS_GIDX)
              w = word_by_row_groups<T>(words[j], row_groups,
                                        p.scales + strip * kStripN + scale_slot(16 * j + col16, true), p.size_n,
                                        magic);
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

    reduce_waves<MB, kWaves>(acc, red, wave, lane);
    if (wave == 0) finish_segment<T, MB>(p, part, strip, seg_begin, seg_end, lane, acc);
    seg_begin = seg_end;
  }
}

// ---------------------------------------------------------------------------
// The general kernel for 8-bit codes (uint8b128, symmetric, or float8_e4m3fn
// with FP8; no act-order gather): the same partition, reduction and fix-up; a 32-row chunk of a strip
// is two 1-KiB blocks of 16 rows, whose words give a lane the low and the high
// four of the eight consecutive rows of an MFMA operand.
// CHUNK_SCALES (groups of 32 rows, one per chunk: MXFP8): the scales of every
// chunk travel with the unit, as in UnitBuf.
template <typename T, int MB, bool CHUNK_SCALES = false>
struct UnitBuf8 {
  uint4 q[unit_buffer_chunks<MB>()][2];
  typename Dq<T>::vec8 a[unit_buffer_chunks<MB>()][MB];
  uint32_t sbits[4];
  int group;
  uint4 sv[CHUNK_SCALES ? unit_buffer_chunks<MB>() : 1];
};

template <typename T, int MB, bool CHUNK_SCALES = false>
__device__ __forceinline__ void load_unit8(UnitBuf8<T, MB, CHUNK_SCALES>& b, const StreamParams& p, int u, int lane,
                                           bool grouped) {
  const int col16 = lane & 15, kb = lane >> 4;
  const int strip = u / p.units_per_strip;
  const int unit = u - strip * p.units_per_strip;
  const int chunk0 = unit * p.unit_chunks;
  const uint4* bsrc = p.b + ((long)strip * p.chunks_per_strip + chunk0) * 128 + lane;
#pragma unroll
  for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc)
    if (cc < p.unit_chunks) {
      b.q[cc][0] = bsrc[(2 * cc) * 64];
      b.q[cc][1] = bsrc[(2 * cc + 1) * 64];
    }
#pragma unroll
  for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc)
    if (cc < p.unit_chunks) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        b.a[cc][mb] = load_a<T, false>(p, 16 * mb + col16, (chunk0 + cc) * kChunkK + 8 * kb);
    }
  const int g = grouped ? (chunk0 * kChunkK) / p.group_size : 0;
  b.group = g;
  const uint16_t* srow = p.scales + (long)g * p.size_n + strip * kStripN;
  if (CHUNK_SCALES) {   // group = chunk
#pragma unroll
    for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc)
      if (cc < p.unit_chunks)
        b.sv[CHUNK_SCALES ? cc : 0] = *reinterpret_cast<const uint4*>(srow + (long)cc * p.size_n + 8 * (col16 & 7));
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) b.sbits[j] = srow[scale_slot(16 * j + col16, grouped)];
}

// MX: groups of 32 rows, one per chunk (MXFP8; integer codes with such groups too).
template <typename T, int MB, bool HAS_GIDX, bool FP8, bool MX = false>
__global__ __launch_bounds__(kWaves * 64) void marlin_stream8_kernel(const StreamParams params) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq8Of<T, FP8>::type D8;
  typedef typename D8::Col Col;
  __shared__ float4 red[4][MB * 4][64];
  // Several 64-row slabs can share a launch when no strip is shared between
  // workgroups (nothing goes through the scratch slots).
  StreamParams p = params;
  int part, slab;
  part_and_slab(p.grid_parts, p.slabs, part, slab);
  if (part >= p.parts) return;
  {
    p.a += (long)slab * 64 * p.lda;
    p.c += (long)slab * 64 * p.size_n;
    p.size_m = min(64, p.size_m - 64 * slab);
  }

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col16 = lane & 15;
  const int u_begin = range_begin(part, p.total_units, p.parts);
  const int u_end = range_begin(part + 1, p.total_units, p.parts);
  const bool grouped = p.num_groups > 1;
  const uint32_t magic = magic_register();

  UnitBuf8<T, MB, MX> cur, nxt;
  int mine = u_begin + wave;
  if (mine < u_end) load_unit8<T, MB, MX>(cur, p, mine, lane, grouped);

  int seg_begin = u_begin;
  while (seg_begin < u_end) {
    const int strip = seg_begin / p.units_per_strip;
    const int strip_first = strip * p.units_per_strip;
    const int strip_end = strip_first + p.units_per_strip;
    const int seg_end = u_end < strip_end ? u_end : strip_end;

    floatx4_t acc[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[mb][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    while (mine < seg_end) {
      const int next = mine + kWaves;
      if (next < u_end) load_unit8<T, MB, MX>(nxt, p, next, lane, grouped);
      Col cols[4];
      if (!MX) {
#pragma unroll
        for (int j = 0; j < 4; ++j) cols[j] = D8::make_col((uint16_t)cur.sbits[j]);
      }
      int cur_group = cur.group;
      const int chunk0 = (mine - strip_first) * p.unit_chunks;
#pragma unroll
      for (int cc = 0; cc < unit_buffer_chunks<MB>(); ++cc) {
        if (cc < p.unit_chunks) {
          const int g = grouped ? ((chunk0 + cc) * kChunkK) / p.group_size : 0;
          if (MX) {
#pragma unroll
            for (int j = 0; j < 4; ++j) cols[j] = D8::make_col(chunk_scale(cur.sv[MX ? cc : 0], j, col16));
          } else if (g != cur_group) {  // groups smaller than a unit
            cur_group = g;
            const uint16_t* srow = p.scales + (long)g * p.size_n + strip * kStripN;
#pragma unroll
            for (int j = 0; j < 4; ++j) cols[j] = D8::make_col(srow[scale_slot(16 * j + col16, grouped)]);
          }
          const uint32_t lo[4] = {cur.q[cc][0].x, cur.q[cc][0].y, cur.q[cc][0].z, cur.q[cc][0].w};
          const uint32_t hi[4] = {cur.q[cc][1].x, cur.q[cc][1].y, cur.q[cc][1].z, cur.q[cc][1].w};
          int row_groups[8];
          if (HAS_GIDX) {  // the lane's eight rows of this chunk: k = 32 chunk + 8 (lane / 16) + t
            const int4* gsrc = reinterpret_cast<const int4*>(p.g_idx + (chunk0 + cc) * kChunkK + 8 * (lane >> 4));
            const int4 g0 = gsrc[0], g1 = gsrc[1];
            row_groups[0] = g0.x, row_groups[1] = g0.y, row_groups[2] = g0.z, row_groups[3] = g0.w;
            row_groups[4] = g1.x, row_groups[5] = g1.y, row_groups[6] = g1.z, row_groups[7] = g1.w;
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            uint2 w_lo, w_hi;
            if (HAS_GIDX) {
              const uint16_t* scale_col = p.scales + strip * kStripN + scale_slot(16 * j + col16, true);
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

    reduce_waves<MB, kWaves>(acc, red, wave, lane);
    if (wave == 0) finish_segment<T, MB>(p, part, strip, seg_begin, seg_end, lane, acc);
    seg_begin = seg_end;
  }
}

// ---------------------------------------------------------------------------
// Fast kernel for 16 rows per workgroup (several blocks of 16 rows per launch),
// K % 128 == 0, groups of 128 * 2^s rows (or one group), 4-bit codes, no
// act-order.  Everything a wavefront consumes arrives in its own
// region of LDS through asynchronous global->LDS copies, so bytes in flight tie
// up no vector registers and no register is ever read while a load into it is
// pending: two slots for the packed weights plus scale / zero-point row of one
// 128-row unit each (filled two units ahead, HBM latency), one slot for the
// activation slice of a unit (filled one unit ahead, L2 latency).  The copies of
// a wavefront complete in issue order, so "the oldest unit has landed" is one
// counter wait.  The LDS reads that follow, and the LDS traffic of the
// cross-wavefront reduction, are issued from asm blocks: the compiler cannot
// tell which LDS bytes an asynchronous copy writes, so before any LDS access
// it can see it would wait for every outstanding copy, which would drain the
// prefetch on every unit.

constexpr int kSlotS = 4096;       // inside a weight slot, after 4 chunks x 1 KiB: 64 scales, 8 zero-point words
// GPU below is the number of groups per 128-row unit (1 for groups of 128 rows
// or more, 2 / 4 for groups of 64 / 32 rows): one 256-byte scale / zero-point
// row per group follows the four chunks of a weight slot.
constexpr int slot_bytes(int gpu) { return 4096 + 256 * gpu; }
constexpr int wave_a(int gpu) { return 2 * slot_bytes(gpu); }   // the activation slot follows the two weight slots
// LDS bytes per wavefront: the activation slot holds 4 KiB per block of 16 rows
constexpr int wave_lds(int mb, int gpu = 1) { return 2 * slot_bytes(gpu) + 4096 * mb; }
// Tiles (16 x 16 fp32, 1 KiB) a wavefront parks per pass of the cross-wavefront
// sum: all four of its one block of rows, or two of the eight of two blocks
// (four passes), which keeps 8 wavefronts with two blocks inside 160 KiB.
constexpr int park_tiles(int mb) { return mb == 1 ? 4 : 2; }
constexpr int weight_copies(int gpu) { return 4 + gpu; }   // asynchronous copies per unit: 4 weight chunks + the scale rows
// A workgroup of the fast kernel has 8 wavefronts (one workgroup per compute
// unit), or 4 (three per compute unit: a grid with more workgroups than compute
// units then runs them side by side instead of one after the other).  The tiles of
// the cross-wavefront sum are parked on top of the copy rings.
constexpr int fast_lds_bytes(int waves, int mb, int gpu = 1) { return waves * wave_lds(mb, gpu); }
static_assert(fast_lds_bytes(4, 1) >= 4 * park_tiles(1) * 1024 && fast_lds_bytes(4, 2) >= 4 * park_tiles(2) * 1024,
              "the parked tiles must fit the rings");

// Row id of C of row `r` of block `block` of a grouped call, -1 for padding.
__device__ __forceinline__ int moe_row_id(const StreamParams& p, int block, int r) {
  const int at = block * p.block_size + r;
  if (r >= p.block_size || at >= p.sorted_len) return -1;
  const int id = p.sorted_ids[at];
  return (id < 0 || id >= p.rows_total) ? -1 : id;
}

template <int MB>
struct FastLane {
  uint32_t a_off[2 * MB];  // byte offset of the 16 bytes this lane copies from rows 8h..8h+7 of a 64-column slice of A
  const char* s_ptr;    // this lane's dword of the scale / zero-point row of (group 0, strip 0)
  long s_group_stride;  // bytes between groups for s_ptr
  int s_strip_stride;   // bytes between strips for s_ptr
};

// unit_group_shift: s >= 0 for groups of 128 * 2^s rows, -1 for one group; with
// GPU > 1 the unit holds groups GPU * unit .. GPU * unit + GPU - 1.
template <int MB, int GPU>
__device__ __forceinline__ void copy_weights(const StreamParams& p, const FastLane<MB>& fl, int strip, int unit,
                                             char* slot, int lane, int unit_group_shift) {
  const uint4* gq = p.b + (size_t)(unsigned)(strip * p.chunks_per_strip + unit * 4) * 64 + lane;
  lds_void_t* lq = (lds_void_t*)slot;
  // `nt_weights` (a launch whose workgroups each read their weights once, on a matrix of 10 MB or
  // more): the copies carry the non-temporal bit, which streams the weights past the caches and
  // leaves the activations and the partial tiles there.  Measured on the four GEMMs of a
  // Llama-3-8B layer at M = 16, one box, over 24 sets of weights in turn (no matrix is used again
  // before 2.7 GB of others): no copy with the bit 42.7 us a layer, the gate / up (59 MB) and the
  // down matrix (29 MB) 41.6 - 42.2, those and the qkv matrix (12.6 MB) 41.0, all four 41.1
  // (a copy-only kernel with plain loads on the gate / up matrix: 5.3 -> 5.9 TB/s).  The size
  // stands for "the model's weights do not fit the caches": matrices of a few MB may well be
  // found there by the next call.  With several blocks of rows the later ones count on finding
  // the chunk in the L2, and those copies stay plain.
  constexpr int kNonTemporal = 2;
  if (p.nt_weights) {
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 0, kNonTemporal);
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 1024, kNonTemporal);
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 2048, kNonTemporal);
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 3072, kNonTemporal);
  } else {
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 0, 0);
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 1024, 0);
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 2048, 0);
    __builtin_amdgcn_global_load_lds((glb_void_t*)gq, lq, 16, 3072, 0);
  }
  const int g = GPU > 1 ? unit * GPU : (unit_group_shift >= 0 ? (unit >> unit_group_shift) : 0);
  const char* gs = fl.s_ptr + (long)g * fl.s_group_stride + (long)strip * fl.s_strip_stride;
#pragma unroll
  for (int gi = 0; gi < GPU; ++gi)
    __builtin_amdgcn_global_load_lds((glb_void_t*)(gs + gi * fl.s_group_stride),
                                     (lds_void_t*)(slot + kSlotS + 256 * gi), 4, 0, 0);
}

// The 16 x 128 slice of A of one unit and block of 16 rows, as four regions of
// 1 KiB (a second block of rows follows 4 KiB later): region
// 2 * half + h holds rows 8h..8h+7, 128 bytes (64 columns) each.  One copy fills
// one region; its lanes 8r..8r+7 fetch the eight 16-byte pieces of one
// 128-byte line of row r, so a copy touches 8 whole lines (16 rows x 64 bytes per
// copy, the operand shape, moves a third of the bytes per cycle).  Piece q of
// row r sits at 16-byte slot q ^ (r % 8) of the row, which keeps the operand
// reads (16 rows, one piece each) off each other's banks.
template <int MB>
__device__ __forceinline__ void copy_activations(const StreamParams& p, const FastLane<MB>& fl, int unit,
                                                 char* slot) {
  const char* ga = reinterpret_cast<const char*>(p.a) + (long)unit * (4 * kChunkK * 2);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    char* s = slot + 4096 * mb;
    __builtin_amdgcn_global_load_lds((glb_void_t*)(ga + fl.a_off[2 * mb]), (lds_void_t*)(s), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((glb_void_t*)(ga + fl.a_off[2 * mb + 1]), (lds_void_t*)(s + 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((glb_void_t*)(ga + 128 + fl.a_off[2 * mb]), (lds_void_t*)(s + 2048), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((glb_void_t*)(ga + 128 + fl.a_off[2 * mb + 1]), (lds_void_t*)(s + 3072), 16, 0, 0);
  }
}

// Forming (v - z) * s per weight costs 13 VALU instructions per packed word in
// fp16 and 17 in bf16 (gfx950 has no packed bf16 arithmetic), more than the
// matrix work of a 16-row tile is worth.  The fast kernel instead feeds the
// matrix cores the exact integers B + v (the nibble OR-ed into the mantissa of
// B = 1024.0 in fp16, 128.0 in bf16: 7 instructions per word) and folds offset
// and scale into the accumulator once per 128-row unit, which lies inside one
// group:
//   sum_k (v_k - z) s a_k = s * (sum_k (B + v_k) a_k - (B + z) * sum_k a_k),
// the last sum coming from one more MFMA per chunk with an all-ones operand.
// Products and sums are exact or fp32, so the result differs from the
// dequantise-then-multiply form only by not rounding (v - z) * s to 16 bits first.
template <typename T>
struct RawOperand;
template <>
struct RawOperand<_Float16> {
  static constexpr uint32_t kMagic = 0x64006400u;  // 1024.0 twice
  static constexpr uint32_t kOnes = 0x3c003c00u;
  static constexpr float kBase = 1024.f;
};
template <>
struct RawOperand<__bf16> {
  static constexpr uint32_t kMagic = 0x43004300u;  // 128.0 twice
  static constexpr uint32_t kOnes = 0x3f803f80u;
  static constexpr float kBase = 128.f;
};
__device__ __forceinline__ u32x4_t raw_operand(uint32_t q, uint32_t magic) {
  const uint32_t e0 = and_or(q, 0x000f000fu, magic);
  const uint32_t e1 = and_or(q >> 4, 0x000f000fu, magic);
  const uint32_t e2 = and_or(q >> 8, 0x000f000fu, magic);
  const uint32_t e3 = and_or(q >> 12, 0x000f000fu, magic);
  return u32x4_t{e0, e1, e2, e3};
}

// One unit's operands for the deferred-scale path, issued and awaited inside a
// single asm block (a register must not be touched between the issue of the LDS
// read that fills it and the counter wait): four weight chunks, four activation
// slices, the lane's four zero-point words, and the 16 scales of the output
// rows the lane holds (column 16 j + 4 (lane / 16) + r of the strip, register
// 4 j + r).  O0..O15 are the byte offsets of those scales from `s_at`.
#define SONAR_UNIT_READS(O0, O1, O2, O3, O4, O5, O6, O7, O8, O9, O10, O11, O12, O13, O14, O15)      \
  asm volatile(                                                                                    \
      "ds_read_b128 %0, %25\n\t"                                                                   \
      "ds_read_b128 %1, %25 offset:1024\n\t"                                                       \
      "ds_read_b128 %2, %25 offset:2048\n\t"                                                       \
      "ds_read_b128 %3, %25 offset:3072\n\t"                                                       \
      "ds_read_b128 %4, %26\n\t"                                                                   \
      "ds_read_b128 %5, %29\n\t"                                                                   \
      "ds_read_b128 %6, %26 offset:2048\n\t"                                                       \
      "ds_read_b128 %7, %29 offset:2048\n\t"                                                       \
      "ds_read_b128 %8, %27\n\t"                                                                   \
      "ds_read_u16 %9, %28 offset:" #O0 "\n\tds_read_u16 %10, %28 offset:" #O1 "\n\t"              \
      "ds_read_u16 %11, %28 offset:" #O2 "\n\tds_read_u16 %12, %28 offset:" #O3 "\n\t"             \
      "ds_read_u16 %13, %28 offset:" #O4 "\n\tds_read_u16 %14, %28 offset:" #O5 "\n\t"             \
      "ds_read_u16 %15, %28 offset:" #O6 "\n\tds_read_u16 %16, %28 offset:" #O7 "\n\t"             \
      "ds_read_u16 %17, %28 offset:" #O8 "\n\tds_read_u16 %18, %28 offset:" #O9 "\n\t"             \
      "ds_read_u16 %19, %28 offset:" #O10 "\n\tds_read_u16 %20, %28 offset:" #O11 "\n\t"           \
      "ds_read_u16 %21, %28 offset:" #O12 "\n\tds_read_u16 %22, %28 offset:" #O13 "\n\t"           \
      "ds_read_u16 %23, %28 offset:" #O14 "\n\tds_read_u16 %24, %28 offset:" #O15 "\n\t"           \
      "s_waitcnt lgkmcnt(0)"                                                                       \
      : "=&v"(q0), "=&v"(q1), "=&v"(q2), "=&v"(q3), "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3),    \
        "=&v"(row_z), "=&v"(row_s[0]), "=&v"(row_s[1]), "=&v"(row_s[2]), "=&v"(row_s[3]),          \
        "=&v"(row_s[4]), "=&v"(row_s[5]), "=&v"(row_s[6]), "=&v"(row_s[7]), "=&v"(row_s[8]),       \
        "=&v"(row_s[9]), "=&v"(row_s[10]), "=&v"(row_s[11]), "=&v"(row_s[12]), "=&v"(row_s[13]),   \
        "=&v"(row_s[14]), "=&v"(row_s[15])                                                         \
      : "v"(q_at), "v"(a_at), "v"(z_at), "v"(s_at), "v"(a_at ^ 64u)                                \
      : "memory")

// The same with the 16 scales fetched as four 16-byte vectors (grouped scales, whose
// permuted row holds the scales of columns 16 j + 4 (lane / 16) + r, j = 0..3, as the
// low (lane / 32 == 0) or high 16 bits of the four words at byte 64 ((lane / 16) & 1) + 16 r):
// 4 LDS instructions instead of 16.
#define SONAR_UNIT_READS_VEC()                                                                     \
  asm volatile(                                                                                    \
      "ds_read_b128 %0, %13\n\t"                                                                   \
      "ds_read_b128 %1, %13 offset:1024\n\t"                                                       \
      "ds_read_b128 %2, %13 offset:2048\n\t"                                                       \
      "ds_read_b128 %3, %13 offset:3072\n\t"                                                       \
      "ds_read_b128 %4, %14\n\t"                                                                   \
      "ds_read_b128 %5, %17\n\t"                                                                   \
      "ds_read_b128 %6, %14 offset:2048\n\t"                                                       \
      "ds_read_b128 %7, %17 offset:2048\n\t"                                                       \
      "ds_read_b128 %8, %15\n\t"                                                                   \
      "ds_read_b128 %9, %16\n\t"                                                                   \
      "ds_read_b128 %10, %16 offset:16\n\t"                                                        \
      "ds_read_b128 %11, %16 offset:32\n\t"                                                        \
      "ds_read_b128 %12, %16 offset:48\n\t"                                                        \
      "s_waitcnt lgkmcnt(0)"                                                                       \
      : "=&v"(q0), "=&v"(q1), "=&v"(q2), "=&v"(q3), "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3),    \
        "=&v"(row_z), "=&v"(sv0), "=&v"(sv1), "=&v"(sv2), "=&v"(sv3)                               \
      : "v"(q_at), "v"(a_at), "v"(z_at), "v"(sv_at), "v"(a_at ^ 64u)                               \
      : "memory")

// The activation operands of a second block of 16 rows (4 KiB after the first).
#define SONAR_UNIT_READS_ROWS2(B0, B1, B2, B3)                                                      \
  asm volatile(                                                                                    \
      "ds_read_b128 %0, %4 offset:4096\n\t"                                                        \
      "ds_read_b128 %1, %5 offset:4096\n\t"                                                        \
      "ds_read_b128 %2, %4 offset:6144\n\t"                                                        \
      "ds_read_b128 %3, %5 offset:6144\n\t"                                                        \
      "s_waitcnt lgkmcnt(0)"                                                                       \
      : "=&v"(B0), "=&v"(B1), "=&v"(B2), "=&v"(B3)                                                 \
      : "v"(a_at), "v"(a_at ^ 64u)                                                                 \
      : "memory")

// Zero-point words and the 16 scales of one more group of the unit (GI = 1..3, 256 bytes per group).
#define SONAR_GROUP_READS(GI)                                                                       \
  asm volatile(                                                                                    \
      "ds_read_b128 %0, %17\n\t"                                                                   \
      "ds_read_u16 %1, %18\n\tds_read_u16 %2, %18 offset:16\n\t"                                  \
      "ds_read_u16 %3, %18 offset:32\n\tds_read_u16 %4, %18 offset:48\n\t"                        \
      "ds_read_u16 %5, %18 offset:4\n\tds_read_u16 %6, %18 offset:20\n\t"                         \
      "ds_read_u16 %7, %18 offset:36\n\tds_read_u16 %8, %18 offset:52\n\t"                        \
      "ds_read_u16 %9, %18 offset:8\n\tds_read_u16 %10, %18 offset:24\n\t"                        \
      "ds_read_u16 %11, %18 offset:40\n\tds_read_u16 %12, %18 offset:56\n\t"                      \
      "ds_read_u16 %13, %18 offset:12\n\tds_read_u16 %14, %18 offset:28\n\t"                      \
      "ds_read_u16 %15, %18 offset:44\n\tds_read_u16 %16, %18 offset:60\n\t"                      \
      "s_waitcnt lgkmcnt(0)"                                                                       \
      : "=&v"(more_z[GI - 1]), "=&v"(more_s[GI - 1][0]), "=&v"(more_s[GI - 1][1]),                  \
        "=&v"(more_s[GI - 1][2]), "=&v"(more_s[GI - 1][3]), "=&v"(more_s[GI - 1][4]),                \
        "=&v"(more_s[GI - 1][5]), "=&v"(more_s[GI - 1][6]), "=&v"(more_s[GI - 1][7]),                \
        "=&v"(more_s[GI - 1][8]), "=&v"(more_s[GI - 1][9]), "=&v"(more_s[GI - 1][10]),               \
        "=&v"(more_s[GI - 1][11]), "=&v"(more_s[GI - 1][12]), "=&v"(more_s[GI - 1][13]),             \
        "=&v"(more_s[GI - 1][14]), "=&v"(more_s[GI - 1][15])                                         \
      : "v"(z_at + 256u * (GI)), "v"(s_at + 256u * (GI))                                           \
      : "memory")

// MB blocks of 16 rows per workgroup (1 or 2): the weights of a unit are pulled
// out of LDS and turned into operands once and multiplied with every block.
// GROUPED: one workgroup per (block of slots, strip) of a mixture-of-experts
// call; the rows of A are gathered and the rows of C scattered through
// sorted_ids, everything else is the dense kernel on the expert's matrices.
// GPU: groups per 128-row unit (2 or 4 for groups of 64 or 32 rows, else 1).
// FP4 (with GPU = 4, no zero points): float4_e2m1f codes; the operands are the
// converted values themselves, so only the scale is left for after the unit.
// A workgroup works on one piece of one strip (StreamParams::piece_shift / piece_units):
// units unit0 .. unit0 + piece_units - 1 of strip `part >> piece_shift`, dealt round-robin
// to its wavefronts.  It sums its wavefronts once, at the end (the tiles of that sum are
// parked on top of the copy rings, every copy having been consumed by then), and either
// writes C (the piece is the whole strip) or leaves fp32 partial tiles and draws the
// strip's ticket.  (A third weight slot per wavefront was measured slower than two on every
// Llama-3-8B shape: M = 16, down 12.2 against 11.4 us, gate_up 19.1 against 17.4.)
template <typename T, bool HAS_ZP, int kFastWaves, int MB, bool GROUPED = false, int GPU = 1, bool FP4 = false>
__global__ __launch_bounds__(kFastWaves * 64) void marlin_stream_fast_kernel(const StreamParams params,
                                                                             const int unit_group_shift) {
  typedef typename Dq<T>::vec8 vec8;
  constexpr int kWaveLds = wave_lds(MB, GPU);
  constexpr int kSlotBytes = slot_bytes(GPU);
  constexpr int kWaveA = wave_a(GPU);
  constexpr int kWeightCopies = weight_copies(GPU);
  constexpr int kPark = park_tiles(MB);       // tiles per wavefront and pass of the cross-wavefront sum
  constexpr int kPasses = 4 * MB / kPark;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  StreamParams p = params;
  // Every argument the dense path reads, fetched now in one batch of scalar loads: left to
  // itself the compiler fetches them where they are first used, four round trips to a cold
  // argument buffer one after the other.
  if constexpr (!GROUPED)
    asm volatile("" ::"s"(p.a), "s"(p.lda), "s"(p.c), "s"(p.b), "s"(p.bias), "s"(p.scales), "s"(p.zeros),
                 "s"(p.scratch), "s"(p.size_m), "s"(p.size_n), "s"(p.num_groups), "s"(p.chunks_per_strip),
                 "s"(p.units_per_strip), "s"(p.parts), "s"(p.slabs), "s"(p.grid_parts), "s"(p.tickets),
                 "s"(p.ticket_stride), "s"(p.xcd_ranges), "s"(p.piece_shift), "s"(p.piece_units),
                 "s"(unit_group_shift));
  int part, slab;
  if constexpr (GROUPED) {   // strip-major inside a block of slots
    part = blockIdx.x % p.grid_parts;
    slab = blockIdx.x / p.grid_parts;
  } else {
    part_and_slab(p.grid_parts, p.slabs, part, slab, p.xcd_ranges);
  }
  if (part >= p.parts) return;
  const int lane = threadIdx.x & 63;
  int row_id[MB] = {};  // grouped calls: the row of C that row (lane & 15) of block of rows mb goes to, or -1
  if constexpr (GROUPED) {
    // `slab` names the block of slots and the 32 rows of it; the whole workgroup leaves together
    const int block = slab / p.sub_blocks;
    const int row0 = 32 * (slab - block * p.sub_blocks);
    if (block * p.block_size >= p.num_post_pad[0]) return;
    const long expert = p.expert_ids[block];
    if (expert < 0 || expert >= p.num_experts) return;
    p.b += expert * p.expert_b_stride;
    p.scales += expert * p.expert_s_stride;
    if (HAS_ZP) p.zeros += expert * p.expert_z_stride;
    if (p.bias) p.bias += expert * p.expert_bias_stride;
    p.size_m = 16 * MB;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) row_id[mb] = moe_row_id(p, block, row0 + 16 * mb + (lane & 15));
    // nothing but padding in these rows (the tail of an expert's last block): every
    // wavefront sees the same ids, so the workgroup leaves as one
    bool any_row = false;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) any_row |= row_id[mb] >= 0;
    if (__builtin_amdgcn_ballot_w64(any_row) == 0) return;
  } else {
    p.a += (long)slab * (16 * MB) * p.lda;
    p.c += (long)slab * (16 * MB) * p.size_n;
    p.size_m = min(16 * MB, p.size_m - 16 * MB * slab);
  }
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col16 = lane & 15;
  char* ring = smem + wave * kWaveLds;
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(lds_void_t*)ring;
  const uint32_t red_lds = (uint32_t)(uintptr_t)(lds_void_t*)smem;

  // this workgroup's piece and this wavefront's share of it: units unit, unit + kFastWaves, ...
  const int strip = part >> p.piece_shift;
  const int pieces = 1 << p.piece_shift;
  int unit = (part & (pieces - 1)) * p.piece_units + wave;
  const int mine = wave < p.piece_units ? (p.piece_units - wave + kFastWaves - 1) / kFastWaves : 0;
  const bool grouped = p.num_groups > 1;

  FastLane<MB> fl;
  {
#pragma unroll
    for (int h = 0; h < 2 * MB; ++h) {
      const int r = 8 * h + (lane >> 3);
      int row = r < p.size_m ? r : p.size_m - 1;  // rows past M are never stored
      if constexpr (GROUPED) {                    // padding slots read row 0 and are never stored
        const int in_block = 32 * (slab % p.sub_blocks) + r;
        const int id = moe_row_id(p, slab / p.sub_blocks, in_block);
        row = id >= 0 ? (p.a_by_slot ? (slab / p.sub_blocks) * p.block_size + in_block : id / p.top_k) : 0;
      }
      fl.a_off[h] = (uint32_t)((long)row * p.lda * 2 + 16 * ((lane & 7) ^ (lane >> 3)));
    }
    if (HAS_ZP && lane >= 32) {
      fl.s_ptr = reinterpret_cast<const char*>(p.zeros + (lane & 7));
      fl.s_group_stride = (long)(p.size_n / 8) * 4;
      fl.s_strip_stride = 8 * 4;
    } else {
      fl.s_ptr = reinterpret_cast<const char*>(p.scales) + 4 * (lane & 31);
      fl.s_group_stride = (long)p.size_n * 2;
      fl.s_strip_stride = kStripN * 2;
    }
  }
  // Operand lane (k group q4 = lane / 16, row col16) of chunk cc of a unit reads
  // piece 4 (cc % 2) + q4 of row col16 in region 2 (cc / 2) + col16 / 8 of the
  // activation slot: a_at for chunk 0, a_at ^ 64 for chunk 1, both + 2048 for
  // chunks 2 and 3 (+ 4096 for the second block of rows).
  const uint32_t a_at = ring_lds + kWaveA + (col16 >> 3) * 1024 + (col16 & 7) * 128 +
                        ((uint32_t)((lane >> 4) ^ (col16 & 7)) * 16);
  // where the scales / zero points of this lane's output rows sit inside a weight slot
  const int q4 = lane >> 4;
  const uint32_t row_s_off = kSlotS + (grouped ? 64 * (q4 & 1) + 2 * (q4 >> 1) : 32 * (q4 & 1) + 4 * (q4 >> 1));
  const uint32_t row_z_off = kSlotS + 128 + 16 * (q4 & 1);
  const uint32_t row_z_shift = 16 * (q4 >> 1);
  // bfloat16 scales of one group per unit: row_s holds float bits
  constexpr bool kVecScales = sizeof(typename Dq<T>::vec8) == 16 && __is_same(T, __bf16) && GPU == 1;
  const uint32_t scale_half = (q4 >> 1) ? 0x07060c0cu : 0x05040c0cu;   // byte selector: high or low 16 bits, shifted up
  const uint32_t magic = magic_register(RawOperand<T>::kMagic);
  u32x4_t ones = u32x4_t{RawOperand<T>::kOnes, RawOperand<T>::kOnes, RawOperand<T>::kOnes, RawOperand<T>::kOnes};
  asm("" : "+v"(ones));

  // Issue order of a wavefront's copies, x being one of its units and W the distance
  // to its next one:  weights(x) | A(x), weights(x+W) | A(x+W), weights(x+2W) | ...
  // They complete in this order.  When the arithmetic of x starts, the only copies
  // younger than A(x) are those of weights(x+W), so "at most that many outstanding"
  // means weights(x) and A(x) have landed.
  if (mine > 0) {
    copy_weights<MB, GPU>(p, fl, strip, unit, ring, lane, unit_group_shift);
    copy_activations<MB>(p, fl, unit, ring + kWaveA);
  }
  if (mine > 1) copy_weights<MB, GPU>(p, fl, strip, unit + kFastWaves, ring + kSlotBytes, lane, unit_group_shift);
  int c_slot = 0;

  floatx4_t acc[MB][4];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[mb][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  for (int left = mine; left > 0; --left) {
    // One unit: wait for its copies, pull them into registers, start the
    // copies of the units after it, then do the arithmetic.
    const uint32_t slot_lds = ring_lds + c_slot * kSlotBytes;
    u32x4_t q0, q1, q2, q3, a0, a1, a2, a3;
    u32x4_t b0 = u32x4_t{0u, 0u, 0u, 0u}, b1 = b0, b2 = b0, b3 = b0;  // second block of rows
    uint32_t row_s[16];
    u32x4_t row_z = u32x4_t{0u, 0u, 0u, 0u};
    uint32_t more_s[GPU > 1 ? GPU - 1 : 1][16];   // the other groups of the unit
    u32x4_t more_z[GPU > 1 ? GPU - 1 : 1];
    if (left > 1) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kWeightCopies) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    {
      const uint32_t q_at = slot_lds + lane * 16;
      const uint32_t z_at = slot_lds + row_z_off, s_at = slot_lds + row_s_off;
      if (kVecScales && grouped) {   // bfloat16: the float bits of a scale are a byte permute of its word
        const uint32_t sv_at = slot_lds + kSlotS + 64 * (q4 & 1);
        u32x4_t sv0, sv1, sv2, sv3;
        SONAR_UNIT_READS_VEC();
        const u32x4_t sv[4] = {sv0, sv1, sv2, sv3};
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) row_s[4 * j + r] = __builtin_amdgcn_perm(sv[r][j], 0u, scale_half);
      } else if (grouped) {  // scale of (j, r) at byte 16 r + 4 j past s_at
        SONAR_UNIT_READS(0, 16, 32, 48, 4, 20, 36, 52, 8, 24, 40, 56, 12, 28, 44, 60);
      } else {        // at byte 64 (j >> 1) + 8 (j & 1) + 16 (r >> 1) + 2 (r & 1)
        SONAR_UNIT_READS(0, 2, 16, 18, 8, 10, 24, 26, 64, 66, 80, 82, 72, 74, 88, 90);
      }
      if (kVecScales && !grouped) {
#pragma unroll
        for (int i = 0; i < 16; ++i) row_s[i] <<= 16;
      }
      if constexpr (MB == 2) SONAR_UNIT_READS_ROWS2(b0, b1, b2, b3);
      if constexpr (GPU >= 2) SONAR_GROUP_READS(1);
      if constexpr (GPU == 4) {
        SONAR_GROUP_READS(2);
        SONAR_GROUP_READS(3);
      }
    }
    if (left > 1) {
      copy_activations<MB>(p, fl, unit + kFastWaves, ring + kWaveA);
      if (left > 2)
        copy_weights<MB, GPU>(p, fl, strip, unit + 2 * kFastWaves, ring + c_slot * kSlotBytes, lane,
                              unit_group_shift);
    }
    unit += kFastWaves;
    c_slot ^= 1;

    const u32x4_t qs[4] = {q0, q1, q2, q3};
    const u32x4_t as[2][4] = {{a0, a1, a2, a3}, {b0, b1, b2, b3}};
    const floatx4_t zero4 = floatx4_t{0.f, 0.f, 0.f, 0.f};
    floatx4_t part_sum[MB][4], asum[MB];
    constexpr int kChunksPerGroup = 4 / GPU;
#pragma unroll
    for (int gi = 0; gi < GPU; ++gi) {
#pragma unroll
      for (int cg = 0; cg < kChunksPerGroup; ++cg) {
        const int cc = gi * kChunksPerGroup + cg;
        const uint32_t words[4] = {qs[cc].x, qs[cc].y, qs[cc].z, qs[cc].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          vec8 wv;
          if constexpr (FP4) wv = DqF4<T>::word(words[j], typename DqF4<T>::Col{1.0f}, magic);
          else wv = __builtin_bit_cast(vec8, raw_operand(words[j], magic));
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            part_sum[mb][j] = Dq<T>::mfma(wv, __builtin_bit_cast(vec8, as[mb][cc]), cg == 0 ? zero4 : part_sum[mb][j]);
        }
        if constexpr (!FP4) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            asum[mb] = Dq<T>::mfma(__builtin_bit_cast(vec8, ones), __builtin_bit_cast(vec8, as[mb][cc]),
                                   cg == 0 ? zero4 : asum[mb]);
        }
      }
      // scale and offset of this group (the whole unit when GPU == 1)
      const u32x4_t gz = gi == 0 ? row_z : more_z[gi == 0 ? 0 : gi - 1];
      const uint32_t zrow[4] = {gz.x >> row_z_shift, gz.y >> row_z_shift, gz.z >> row_z_shift, gz.w >> row_z_shift};
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const uint32_t sbits = gi == 0 ? row_s[4 * j + r] : more_s[gi == 0 ? 0 : gi - 1][4 * j + r];
          const float sc = (kVecScales && gi == 0) ? __uint_as_float(sbits) : Dq<T>::to_float((uint16_t)sbits);
          float off = -(RawOperand<T>::kBase + 8.f);
          if (HAS_ZP) off = -RawOperand<T>::kBase - (float)((zrow[r] >> (4 * j)) & 0xFu);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            if constexpr (FP4) acc[mb][j][r] = __builtin_fmaf(sc, part_sum[mb][j][r], acc[mb][j][r]);
            else acc[mb][j][r] = __builtin_fmaf(sc, __builtin_fmaf(off, asum[mb][r], part_sum[mb][j][r]), acc[mb][j][r]);
          }
        }
    }
  }

  // The cross-wavefront sum: in each pass every wavefront parks kPark of its tiles in
  // LDS and wavefront w (w < kPark) adds up one column block of one block of rows in
  // wavefront order and finishes it.
  int first = 0, last = 0;   // the workgroups that share this strip
  if constexpr (!GROUPED) {
    first = strip << p.piece_shift;
    last = first + pieces - 1;
  }
#pragma unroll
  for (int ps = 0; ps < kPasses; ++ps) {
    const int mb = ps * kPark / 4, jb = ps * kPark % 4;
    __builtin_amdgcn_s_barrier();  // every copy has been consumed; the previous pass's tiles too
    const uint32_t park = red_lds + (wave * kPark * 64 + lane) * 16;
    // the tiles come out of the matrix cores; an asm block is opaque to the
    // compiler's hazard padding, so give the last MFMA time to retire
    if constexpr (kPark == 4) {
      asm volatile(
          "s_nop 15\n\t"
          "s_nop 15\n\t"
          "ds_write_b128 %0, %1\n\t"
          "ds_write_b128 %0, %2 offset:1024\n\t"
          "ds_write_b128 %0, %3 offset:2048\n\t"
          "ds_write_b128 %0, %4 offset:3072\n\t"
          "s_waitcnt lgkmcnt(0)"
          :
          : "v"(park), "v"(acc[mb][0]), "v"(acc[mb][1]), "v"(acc[mb][2]), "v"(acc[mb][3])
          : "memory");
    } else {
      asm volatile(
          "s_nop 15\n\t"
          "s_nop 15\n\t"
          "ds_write_b128 %0, %1\n\t"
          "ds_write_b128 %0, %2 offset:1024\n\t"
          "s_waitcnt lgkmcnt(0)"
          :
          : "v"(park), "v"(acc[mb][jb]), "v"(acc[mb][jb + 1])
          : "memory");
    }
    __builtin_amdgcn_s_barrier();
    if (wave < kPark) {
      floatx4_t sum = floatx4_t{0.f, 0.f, 0.f, 0.f};
      const uint32_t src = red_lds + (wave * 64 + lane) * 16;
#pragma unroll
      for (int w = 0; w < kFastWaves; w += 4) {
        floatx4_t t0, t1, t2, t3;
        asm volatile(
            "ds_read_b128 %0, %4\n\t"
            "ds_read_b128 %1, %4 offset:%5\n\t"
            "ds_read_b128 %2, %4 offset:%6\n\t"
            "ds_read_b128 %3, %4 offset:%7\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3)
            : "v"(src + w * kPark * 1024), "n"(kPark * 1024), "n"(2 * kPark * 1024), "n"(3 * kPark * 1024)
            : "memory");
        sum += t0;
        sum += t1;
        sum += t2;
        sum += t3;
      }
      const int j = jb + wave;
      if constexpr (GROUPED) {
        finish_block_grouped<T>(p, row_id[mb], strip, lane, j, sum);
      } else if (pieces == 1) {
        store_c_block<T>(p, p.c + (long)(16 * mb) * p.size_n, p.size_m - 16 * mb, strip, lane, j, sum);
      } else {
        store_partial_block(p, part, first, (slab * MB + mb) * 4 + j, lane, sum);
      }
    }
  }

  // A strip shared with other workgroups: draw its ticket; whoever holds the last ticket
  // adds its partial tiles up.
  if constexpr (!GROUPED) {
    if (p.tickets != nullptr && pieces > 1) {
      const uint32_t flag_lds = (uint32_t)(uintptr_t)(lds_void_t*)smem;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's partial tiles are in memory
      __builtin_amdgcn_s_barrier();                      // ... and every wavefront's; all LDS traffic is over
      // A ticket counts arrivals per XCD, four bits each (the host keeps a strip to at most
      // 15 contributors): their sum says who is last, and a single non-zero field that every
      // contributor ran on one XCD.
      const unsigned int xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7u;   // XCC_ID: the XCD this workgroup runs on
      unsigned int* ticket = p.tickets + ((long)first * p.slabs + slab) * p.ticket_stride;
      if (threadIdx.x == 0) {
        const unsigned int mine_field = 1u << (4u * xcc);
        const unsigned int now =
            mine_field + __hip_atomic_fetch_add(ticket, mine_field, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("ds_write_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" ::"v"(flag_lds), "v"(now) : "memory");
      }
      __builtin_amdgcn_s_barrier();
      uint32_t now;
      asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(now) : "v"(flag_lds) : "memory");
      now = __builtin_amdgcn_readfirstlane(now);
      const unsigned int pairs = (now & 0x0f0f0f0fu) + ((now >> 4) & 0x0f0f0f0fu);
      const int arrived = (int)((pairs * 0x01010101u) >> 24);
      if (arrived == pieces) {   // nobody is still at work on this strip
        const bool near = now == ((unsigned int)pieces << (4u * xcc));
        for (int t = wave; t < 4 * MB; t += kFastWaves) {
          const int mb = t >> 2, j = t & 3;
          const floatx4_t sum = near ? sum_partial_tiles<true>(p, first, last, slab * MB + mb, j, lane)
                                     : sum_partial_tiles<false>(p, first, last, slab * MB + mb, j, lane);
          store_c_block<T>(p, p.c + (long)(16 * mb) * p.size_n, p.size_m - 16 * mb, strip, lane, j, sum);
        }
        if (threadIdx.x == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}
#undef SONAR_UNIT_READS_VEC
#undef SONAR_UNIT_READS_ROWS2
#undef SONAR_GROUP_READS

// ---------------------------------------------------------------------------
// Second pass over the strips that were split between workgroups: adds the
// partial tiles in workgroup order and writes C.  One wavefront per strip and
// 16-row block.
template <typename T, int MB>
__global__ __launch_bounds__(64) void marlin_fixup_kernel(const StreamParams p) {
  const int strip = blockIdx.x / MB;
  const int mb = blockIdx.x - strip * MB;
  const int lane = threadIdx.x;
  const int strip_first = strip * p.units_per_strip;
  const int first = range_owner(strip_first, p.total_units, p.parts);
  const int last = range_owner(strip_first + p.units_per_strip - 1, p.total_units, p.parts);
  if (first == last) return;
  floatx4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  for (int w = first; w <= last; ++w) {
    const float4* src = partial_slot(p, w, first);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float4 v = src[(mb * 4 + j) * 64 + lane];
      acc[j] += floatx4_t{v.x, v.y, v.z, v.w};
    }
  }
  const int m = 16 * mb + (lane & 15);
  if (m >= p.size_m) return;
  const int n_in = 4 * (lane >> 4);
  const float gs = p.global_scale ? *p.global_scale : 1.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int nl = 16 * j + n_in;
    float b[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
#pragma unroll
      for (int r = 0; r < 4; ++r) b[r] = Dq<T>::to_float(p.bias[strip * kStripN + scale_slot(nl + r, false)]);
    }
    const floatx4_t v = acc[j] * gs;
    uint2 o;
    o.x = (uint32_t)Dq<T>::from_float(v.x + b[0]) | ((uint32_t)Dq<T>::from_float(v.y + b[1]) << 16);
    o.y = (uint32_t)Dq<T>::from_float(v.z + b[2]) | ((uint32_t)Dq<T>::from_float(v.w + b[3]) << 16);
    *reinterpret_cast<uint2*>(p.c + (long)m * p.size_n + strip * kStripN + nl) = o;
  }
}

// Writes W[K][N]: the values the GEMM kernels feed to the matrix cores.
// With g_idx (symmetric weights only) the group of every row is looked up there.
template <typename T, bool HAS_ZP, bool FP4 = false, bool NV = false>
__global__ __launch_bounds__(256) void marlin_dequant_kernel(const uint4* __restrict__ b,
                                                            const uint16_t* __restrict__ scales,
                                                            const uint32_t* __restrict__ zeros,
                                                            const int32_t* __restrict__ g_idx,
                                                            uint16_t* __restrict__ w_out, int size_n,
                                                            int size_k, int num_groups, int group_size,
                                                            long total_chunks) {
  typedef typename Dq<T>::vec8 vec8;
  const int lane = threadIdx.x & 63;
  const int col16 = lane & 15;
  const int kb = lane >> 4;
  const int chunks_per_strip = size_k / kChunkK;
  const bool grouped = num_groups > 1;
  const uint32_t magic = magic_register();
  for (long ch = (long)blockIdx.x * 4 + (threadIdx.x >> 6); ch < total_chunks; ch += (long)gridDim.x * 4) {
    const int strip = (int)(ch / chunks_per_strip);
    const int chunk = (int)(ch % chunks_per_strip);
    // NV: groups of 16 rows; a lane's eight rows lie in one of the chunk's two
    const int g = NV ? 2 * chunk + (kb >> 1) : (grouped && !g_idx ? (chunk * kChunkK) / group_size : 0);
    typedef typename Dq4Of<T, FP4, NV>::type D4;
    typename D4::Col cols[4];
    load_cols<T, HAS_ZP, D4>(cols, scales, zeros, size_n, strip, g, col16, grouped);
    int row_groups[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (g_idx) {
#pragma unroll
      for (int t = 0; t < 8; ++t) row_groups[t] = g_idx[chunk * kChunkK + 8 * kb + t];
    }
    const uint4 q = b[ch * 64 + lane];
    const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      vec8 w;
      if (!HAS_ZP && g_idx)
        w = word_by_row_groups<T>(words[j], row_groups, scales + strip * kStripN + scale_slot(16 * j + col16, true),
                                  size_n, magic);
      else
        w = D4::word(words[j], cols[j], magic);
      const uint16_t* bits = reinterpret_cast<const uint16_t*>(&w);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const long k = (long)chunk * kChunkK + 8 * kb + t;
        w_out[k * size_n + strip * kStripN + 16 * j + col16] = bits[t];
      }
    }
  }
}

// The same for 8-bit codes: one wavefront per 1-KiB block of 16 rows.
template <typename T, bool FP8>
__global__ __launch_bounds__(256) void marlin_dequant8_kernel(const uint4* __restrict__ b,
                                                             const uint16_t* __restrict__ scales,
                                                             const int32_t* __restrict__ g_idx,
                                                             uint16_t* __restrict__ w_out, int size_n, int size_k,
                                                             int num_groups, int group_size, long total_blocks) {
  const int lane = threadIdx.x & 63;
  const int col16 = lane & 15;
  const int kb = lane >> 4;
  const int blocks_per_strip = size_k / 16;
  const bool grouped = num_groups > 1;
  const uint32_t magic = magic_register();
  for (long blk = (long)blockIdx.x * 4 + (threadIdx.x >> 6); blk < total_blocks; blk += (long)gridDim.x * 4) {
    const int strip = (int)(blk / blocks_per_strip);
    const int in_strip = (int)(blk % blocks_per_strip);
    const int chunk = in_strip >> 1, h = in_strip & 1;
    const int g = (grouped && !g_idx) ? (chunk * kChunkK) / group_size : 0;
    const uint16_t* srow = scales + (long)g * size_n + strip * kStripN;
    const uint4 q = b[blk * 64 + lane];
    const uint32_t words[4] = {q.x, q.y, q.z, q.w};
    int row_groups[4] = {0, 0, 0, 0};
    if (g_idx) {
#pragma unroll
      for (int t = 0; t < 4; ++t) row_groups[t] = g_idx[chunk * kChunkK + 8 * kb + 4 * h + t];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint2 w;
      if (g_idx)
        w = word4_by_row_groups8<T>(words[j], row_groups, scales + strip * kStripN + scale_slot(16 * j + col16, true),
                                    size_n, magic);
      else
        w = Dq8Of<T, FP8>::type::word4(
            words[j], Dq8Of<T, FP8>::type::make_col(srow[scale_slot(16 * j + col16, grouped)]), magic);
      const uint16_t bits[4] = {(uint16_t)(w.x & 0xffffu), (uint16_t)(w.x >> 16), (uint16_t)(w.y & 0xffffu),
                                (uint16_t)(w.y >> 16)};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const long k = (long)chunk * kChunkK + 8 * kb + 4 * h + t;
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

// A'[m][k] = A[m][perm[k]]: with act-order weights (rows in sorted-group order)
// the GEMM on A' is a plain grouped GEMM, which every kernel here runs without
// gathering (the reference permutes A the same way, marlin.cu:760-762).
__global__ __launch_bounds__(256) void permute_columns_kernel(const uint16_t* __restrict__ a, long lda,
                                                             const int32_t* __restrict__ perm,
                                                             uint16_t* __restrict__ out, int size_m,
                                                             int size_k) {
  const int per_row = size_k / 8;
  const long total = (long)size_m * per_row;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int m = (int)(i / per_row);
    const int k0 = (int)(i - (long)m * per_row) * 8;
    const uint16_t* arow = a + (long)m * lda;
    const int4 p0 = *reinterpret_cast<const int4*>(perm + k0);
    const int4 p1 = *reinterpret_cast<const int4*>(perm + k0 + 4);
    uint4 v;
    v.x = (uint32_t)arow[p0.x] | ((uint32_t)arow[p0.y] << 16);
    v.y = (uint32_t)arow[p0.z] | ((uint32_t)arow[p0.w] << 16);
    v.z = (uint32_t)arow[p1.x] | ((uint32_t)arow[p1.y] << 16);
    v.w = (uint32_t)arow[p1.z] | ((uint32_t)arow[p1.w] << 16);
    *reinterpret_cast<uint4*>(out + (long)m * size_k + k0) = v;
  }
}

template <typename T, int MB, bool HAS_ZP>
void launch_stream(const StreamParams& p, bool has_perm, hipStream_t st) {
  if (p.g_idx) {  // row -> group lookup: symmetric weights, activations already permuted
    if constexpr (!HAS_ZP) marlin_stream_kernel<T, MB, false, false, true><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p);
  } else if (has_perm) {   // symmetric weights only (check_common)
    if constexpr (!HAS_ZP) marlin_stream_kernel<T, MB, false, true, false><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p);
  } else {
    marlin_stream_kernel<T, MB, HAS_ZP, false, false><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p);
  }
}

template <typename T, bool HAS_ZP>
void launch_stream_mb(const StreamParams& p, bool has_perm, hipStream_t st) {
  switch ((p.size_m + 15) / 16) {
    case 1: launch_stream<T, 1, HAS_ZP>(p, has_perm, st); break;
    case 2: launch_stream<T, 2, HAS_ZP>(p, has_perm, st); break;
    case 3: launch_stream<T, 3, HAS_ZP>(p, has_perm, st); break;
    default: launch_stream<T, 4, HAS_ZP>(p, has_perm, st); break;
  }
}

// float4_e2m1f codes: no zero points, no act-order (NV: NVFP4, scales per 16 rows)
template <typename T, bool NV = false>
void launch_stream_fp4(const StreamParams& p, hipStream_t st) {
  switch ((p.size_m + 15) / 16) {
    case 1: marlin_stream_kernel<T, 1, false, false, false, true, NV><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
    case 2: marlin_stream_kernel<T, 2, false, false, false, true, NV><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
    case 3: marlin_stream_kernel<T, 3, false, false, false, true, NV><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
    default: marlin_stream_kernel<T, 4, false, false, false, true, NV><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
  }
}

template <typename T, bool HAS_GIDX, bool FP8, bool MX = false>
void launch_stream8_gidx(const StreamParams& p, hipStream_t st) {
  switch ((p.size_m + 15) / 16) {
    case 1: marlin_stream8_kernel<T, 1, HAS_GIDX, FP8, MX><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
    case 2: marlin_stream8_kernel<T, 2, HAS_GIDX, FP8, MX><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
    case 3: marlin_stream8_kernel<T, 3, HAS_GIDX, FP8, MX><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
    default: marlin_stream8_kernel<T, 4, HAS_GIDX, FP8, MX><<<p.grid_parts * p.slabs, kWaves * 64, 0, st>>>(p); break;
  }
}

template <typename T>
void launch_stream8_mb(const StreamParams& p, bool fp8, hipStream_t st) {
  // groups of 32 rows (MXFP8, or integer codes): the scales of every chunk are fetched with the unit
  const bool chunk_groups = !p.g_idx && p.num_groups > 1 && p.group_size == 32 && ((uintptr_t)p.scales) % 16 == 0;
  if (fp8 && chunk_groups) launch_stream8_gidx<T, false, true, true>(p, st);
  else if (chunk_groups) launch_stream8_gidx<T, false, false, true>(p, st);
  else if (fp8) launch_stream8_gidx<T, false, true>(p, st);   // no act-order with floating-point codes
  else if (p.g_idx) launch_stream8_gidx<T, true, false>(p, st);
  else launch_stream8_gidx<T, false, false>(p, st);
}

template <typename T, bool HAS_ZP, int WAVES, int MB, bool GROUPED, int GPU>
int launch_fast_groups(const StreamParams& p, int unit_group_shift, hipStream_t st) {
  static bool attr_set = false;  // raising the dynamic LDS limit is needed once per kernel
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_stream_fast_kernel<T, HAS_ZP, WAVES, MB, GROUPED, GPU>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, fast_lds_bytes(WAVES, MB, GPU)));
    attr_set = true;
  }
  const int lds = fast_lds_bytes(WAVES, MB, GPU);
  marlin_stream_fast_kernel<T, HAS_ZP, WAVES, MB, GROUPED, GPU>
      <<<p.grid_parts * p.slabs, WAVES * 64, lds, st>>>(p, unit_group_shift);
  return SONAR_OK;
}

// unit_group_shift -2 / -4: two / four groups per 128-row unit (groups of 64 / 32 rows)
template <typename T, bool HAS_ZP, int WAVES, int MB, bool GROUPED>
int launch_fast_waves(const StreamParams& p, int unit_group_shift, hipStream_t st) {
  if (unit_group_shift <= -2) {
    // several sets of scales per unit and two blocks of rows do not fit the register file (and were measured
    // slower than the general kernel): callers pass one block of rows
    if constexpr (MB == 1) {
      return unit_group_shift == -2 ? launch_fast_groups<T, HAS_ZP, WAVES, 1, GROUPED, 2>(p, unit_group_shift, st)
                                    : launch_fast_groups<T, HAS_ZP, WAVES, 1, GROUPED, 4>(p, unit_group_shift, st);
    } else {
      return fail(SONAR_E_INVALID, "internal: groups of 32 / 64 rows with two blocks of rows per workgroup");
    }
  }
  return launch_fast_groups<T, HAS_ZP, WAVES, MB, GROUPED, 1>(p, unit_group_shift, st);
}

// MXFP4: bf16, four groups of 32 rows per unit, one block of 16 rows per workgroup
template <int WAVES, bool GROUPED>
int launch_fast_fp4_waves(const StreamParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_stream_fast_kernel<__bf16, false, WAVES, 1, GROUPED, 4, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, fast_lds_bytes(WAVES, 1, 4)));
    attr_set = true;
  }
  const int lds = fast_lds_bytes(WAVES, 1, 4);
  marlin_stream_fast_kernel<__bf16, false, WAVES, 1, GROUPED, 4, true>
      <<<p.grid_parts * p.slabs, WAVES * 64, lds, st>>>(p, -4);
  return SONAR_OK;
}

template <bool GROUPED>
int launch_fast_fp4(const StreamParams& p, bool half_workgroups, hipStream_t st) {
  return half_workgroups ? launch_fast_fp4_waves<4, GROUPED>(p, st) : launch_fast_fp4_waves<8, GROUPED>(p, st);
}

// `row_blocks`: blocks of 16 rows per workgroup (1 or 2).
template <typename T, bool HAS_ZP, bool GROUPED = false>
int launch_fast(const StreamParams& p, int unit_group_shift, bool half_workgroups, int row_blocks, hipStream_t st) {
  if (row_blocks == 2)
    return half_workgroups ? launch_fast_waves<T, HAS_ZP, 4, 2, GROUPED>(p, unit_group_shift, st)
                           : launch_fast_waves<T, HAS_ZP, 8, 2, GROUPED>(p, unit_group_shift, st);
  return half_workgroups ? launch_fast_waves<T, HAS_ZP, 4, 1, GROUPED>(p, unit_group_shift, st)
                         : launch_fast_waves<T, HAS_ZP, 8, 1, GROUPED>(p, unit_group_shift, st);
}

template <typename T>
void launch_fixup(const StreamParams& p, hipStream_t st) {
  const int strips = p.size_n / kStripN;
  switch ((p.size_m + 15) / 16) {
    case 1: marlin_fixup_kernel<T, 1><<<strips, 64, 0, st>>>(p); break;
    case 2: marlin_fixup_kernel<T, 2><<<strips * 2, 64, 0, st>>>(p); break;
    case 3: marlin_fixup_kernel<T, 3><<<strips * 3, 64, 0, st>>>(p); break;
    default: marlin_fixup_kernel<T, 4><<<strips * 4, 64, 0, st>>>(p); break;
  }
}

struct Checked {
  bool has_zp;
  bool has_perm;
  bool row_groups;  // act-order shard without whole groups: the group of a row comes from g_idx
  int group_size;
  int bits;         // 4 or 8
  bool fp8;         // 8-bit floating-point codes (float8_e4m3fn)
  bool fp4;         // 4-bit floating-point codes (float4_e2m1f) with power-of-two scales per 32 rows (MXFP4) ...
  bool nvfp4;       // ... or with scales of the activation type per 16 rows and a global scale (NVFP4)
};

int check_common(Checked& out, int b_layout, const void* b_scales, const uint32_t* b_zeros,
                 const int32_t* g_idx, const int32_t* perm, int dtype, int64_t b_type_id,
                 int64_t size_n, int64_t size_k, int64_t num_groups, int is_k_full, bool nvfp4 = false) {
  SONAR_REQUIRE(b_layout == SONAR_LAYOUT_GFX950, "unknown b_layout = %d", b_layout);
  SONAR_REQUIRE(dtype == SONAR_DTYPE_F16 || dtype == SONAR_DTYPE_BF16, "unsupported `a` scalar_type");
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
  out.fp8 = b_type_id == SONAR_TYPE_FLOAT8_E4M3FN;
  out.fp4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F;
  out.nvfp4 = nvfp4;
  if (nvfp4) SONAR_REQUIRE(out.fp4, "a global scale goes with float4_e2m1f weights only (NVFP4)");
  out.bits = (b_type_id == SONAR_TYPE_UINT8B128 || out.fp8) ? 8 : 4;
  out.has_zp = b_zeros != nullptr;
  if (out.has_zp)
    SONAR_REQUIRE(b_type_id == SONAR_TYPE_UINT4, "b_type must be u4 or u8 when has_zp = True");
  else
    SONAR_REQUIRE(b_type_id != SONAR_TYPE_UINT4,
                  "b_type must be uint4b8, uint8b128 or float8_e4m3fn when has_zp = False (uint4 needs b_zeros)");
  SONAR_REQUIRE((g_idx == nullptr) == (perm == nullptr), "g_idx and perm must be given together");
  out.has_perm = perm != nullptr;
  // generate_kernels.py:66-72: uint4 weights with zero points come without the act-order form
  // (group_blocks 0), and marlin.cu:509-519 then finds no kernel
  if (out.has_zp && out.has_perm)
    return fail(SONAR_E_UNSUPPORTED, "Unsupported shapes: has_act_order = 1 with zero points (b_type uint4): "
                "act-order is built for uint4b8 and uint8b128 weights only");
  if (out.nvfp4) {
    // generate_kernels.py:94-101: NVFP4, either activation type, one scale per 16 rows
    SONAR_REQUIRE(!out.has_perm, "act-order is not supported with float4_e2m1f weights");
    SONAR_REQUIRE(size_k == 16 * num_groups,
                  "float4_e2m1f weights with a global scale (NVFP4) take one scale per group of 16 rows; got "
                  "size_k = %ld, num_groups = %ld", (long)size_k, (long)num_groups);
    SONAR_REQUIRE(((uintptr_t)b_scales) % 16 == 0, "b_scales must be 16-byte aligned");
    out.row_groups = false;
    out.group_size = 16;
    return SONAR_OK;
  }
  if (out.fp4) {
    // generate_kernels.py:102-110: MXFP4, bfloat16 activations, one power-of-two scale per 32 rows
    SONAR_REQUIRE(!out.has_perm, "act-order is not supported with float4_e2m1f weights");
    SONAR_REQUIRE(dtype == SONAR_DTYPE_BF16, "float4_e2m1f weights with power-of-two block scales (MXFP4) "
                  "need bfloat16 activations");
    SONAR_REQUIRE(size_k == 32 * num_groups,
                  "float4_e2m1f weights (MXFP4) take one scale per group of 32 rows; got size_k = %ld, "
                  "num_groups = %ld", (long)size_k, (long)num_groups);
    SONAR_REQUIRE(((uintptr_t)b_scales) % 16 == 0, "b_scales must be 16-byte aligned");
  }
  if (out.fp8) {
    // generate_kernels.py:87-93: channelwise scales or groups of 128 rows (:111-119: MXFP8, groups of 32), no act-order
    SONAR_REQUIRE(!out.has_perm, "act-order is not supported with float8_e4m3fn weights");
    SONAR_REQUIRE(num_groups == 1 || size_k == 128 * num_groups || size_k == 32 * num_groups,
                  "float8_e4m3fn weights take one scale per column, per group of 128 rows or (MXFP8) per group "
                  "of 32 rows; got size_k = %ld, num_groups = %ld", (long)size_k, (long)num_groups);
  }
  out.row_groups = out.has_perm && !is_k_full;
  if (out.has_perm) SONAR_REQUIRE(num_groups > 1, "For act_order, num_groups must be > 1");
  if (out.row_groups) {
    // marlin.cu:343-351,763-769: group_size = 0, every row looks its group up
    out.group_size = 0;
  } else if (num_groups > 1) {
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

// log2 of the 128-row units per group when groups are runs of 128 * 2^s rows,
// -1 for one group, -2 / -4 for groups of 64 / 32 rows (two / four per unit);
// false when the fast kernel cannot index the groups.
bool fast_group_shift(int64_t num_groups, int group_size, int& unit_group_shift) {
  unit_group_shift = -1;
  if (num_groups == 1) return true;
  if (group_size == 64 || group_size == 32) {   // two / four groups per 128-row unit
    unit_group_shift = group_size == 64 ? -2 : -4;
    return true;
  }
  if (group_size <= 0 || group_size % 128 != 0) return false;
  const int per = group_size / 128;
  if ((per & (per - 1)) != 0) return false;
  unit_group_shift = 0;
  while ((1 << unit_group_shift) < per) ++unit_group_shift;
  return true;
}

}  // namespace

// The grouped (mixture-of-experts) op can use the 16-row kernel when the expert
// matrices meet its conditions (blocks of 48 or 64 slots as two halves).
bool moe_fast_applies(bool has_perm, int64_t moe_block_size, int64_t sorted_len, int64_t num_experts,
                      int64_t a_rows, int64_t size_n, int64_t size_k, int64_t num_groups, int group_size) {
  static const bool no_fast = getenv("SONAR_MARLIN_NO_MOE_FAST") != nullptr;  // debugging aid
  int shift;
  const int64_t n_strips = size_n / kStripN, units = size_k / (4 * kChunkK);
  if (no_fast || has_perm || size_k % (4 * kChunkK) != 0 || !fast_group_shift(num_groups, group_size, shift) ||
      a_rows * size_k * 2 >= (1LL << 31) || n_strips * units * n_strips >= (1LL << 31))
    return false;
  if (shift <= -2 && moe_block_size > 16) return false;   // groups of 32 / 64 rows: one block of 16 rows only
  if (moe_block_size < 64) return true;
  // 64-slot blocks also have the tile kernel, which wins once the experts have
  // rows enough for its tiles.  Measured on Mixtral shapes (8 experts, top 2;
  // gate_up / down, this kernel against the tile kernel with its 128-row tiles
  // and its K split): 888 slots (192 tokens): 250 / 103 us against 271 / 137;
  // 952 slots: 265 / 122 against 267 / 134; 1016 slots (256 tokens): 305 / 123
  // against 272 / 132; 1144 slots: down 150 against 137; 1272 slots: down 178
  // against 141.  The tile kernel launches at least experts x N / 256
  // workgroups; where that is under one per compute unit (down) it stays
  // behind a little longer.
  const int64_t tile_workgroups = num_experts * ((size_n + 255) / 256);
  return sorted_len <= (tile_workgroups < cu_count() ? 1100 : 1000);
}

// Called by sonar_moe_wna16_marlin_gemm when moe_fast_applies: one workgroup
// per (block of slots, strip), nothing reduced through memory.  Arguments have
// been validated by the caller.
int moe_fast_gemm(const void* a, void* c, const uint32_t* b, const void* bias, const void* scales,
                  const uint32_t* zeros, const int32_t* sorted_ids, int64_t sorted_len, const int32_t* expert_ids,
                  const int32_t* num_post_pad, const float* topk_weights, int64_t moe_block_size, int64_t top_k,
                  int mul_topk, int64_t num_experts, int dtype, int64_t size_m, int64_t size_n, int64_t size_k,
                  int64_t num_groups, int group_size, int a_by_slot, bool fp4, hipStream_t st) {
  StreamParams p = {};
  p.a_by_slot = a_by_slot;
  p.a = static_cast<const uint16_t*>(a);
  p.lda = size_k;
  p.c = static_cast<uint16_t*>(c);
  p.b = reinterpret_cast<const uint4*>(b);
  p.bias = static_cast<const uint16_t*>(bias);
  p.scales = static_cast<const uint16_t*>(scales);
  p.zeros = zeros;
  p.size_m = (int)size_m;
  p.size_n = (int)size_n;
  p.size_k = (int)size_k;
  p.num_groups = (int)num_groups;
  p.group_size = group_size;
  p.chunks_per_strip = (int)(size_k / kChunkK);
  p.unit_chunks = 4;
  p.units_per_strip = p.chunks_per_strip / 4;
  const int n_strips = (int)(size_n / kStripN);
  p.parts = n_strips;                       // part i is strip i
  p.total_units = n_strips * p.units_per_strip;
  p.sub_blocks = moe_block_size > 32 ? 2 : 1;
  p.slabs = (int)((sorted_len + moe_block_size - 1) / moe_block_size) * p.sub_blocks;   // blocks of slots x halves
  p.grid_parts = n_strips;
  p.piece_shift = 0;
  p.piece_units = p.units_per_strip;
  p.sorted_ids = sorted_ids;
  p.expert_ids = expert_ids;
  p.num_post_pad = num_post_pad;
  p.topk_weights = topk_weights;
  p.block_size = (int)moe_block_size;
  p.top_k = (int)top_k;
  p.num_experts = (int)num_experts;
  p.rows_total = (int)(size_m * top_k);
  p.sorted_len = (int)sorted_len;
  p.mul_topk = mul_topk;
  p.expert_b_stride = (long)n_strips * p.chunks_per_strip * 64;
  p.expert_s_stride = (long)num_groups * size_n;
  p.expert_z_stride = (long)num_groups * (size_n / 8);
  p.expert_bias_stride = size_n;
  SONAR_REQUIRE((int64_t)p.slabs * n_strips < (1LL << 31), "too many (block, strip) pairs: %ld",
                (long)((int64_t)p.slabs * n_strips));
  int unit_group_shift;
  fast_group_shift(num_groups, group_size, unit_group_shift);
  const bool half = (int64_t)p.slabs * n_strips > cu_count();   // small workgroups, three per compute unit
  const int row_blocks = moe_block_size <= 16 ? 1 : 2;
  // Non-temporal weight copies as in the dense call, where no other workgroup counts on finding the
  // chunks in the L2: blocks of up to 32 slots (the two halves of a larger block read the same strip).
  // Mixtral-8x7B experts, two sets of weights in turn, gate / up and down GEMM and the whole layer:
  // 16 tokens 97.4 / 47.7 / 153.9 -> 90.1 / 48.0 / 143.2 us, 32 tokens 107.9 / 51.8 / 173.5 ->
  // 108.4 / 46.2 / 161.5, 64 tokens 153.2 / 63.3 / 218.9 -> 150.1 / 62.4 / 215.4; with blocks of 48
  // slots (128 tokens) the down GEMM went from 90.5 to 104.8 us, with 64 slots nothing moved.
  static const bool no_nt = getenv("SONAR_MARLIN_NO_NT_WEIGHTS") != nullptr;
  // (and at most two blocks an expert: beyond that the blocks of an expert read its strips again and again,
  // and the caches are all that keeps those reads from memory)
  p.nt_weights = !no_nt && p.sub_blocks == 1 && p.slabs <= 2 * num_experts &&
                 num_experts * size_k * size_n / 2 >= 10 * 1000 * 1000;
  int rc;
  if (fp4)   // bf16, groups of 32 rows, blocks of at most 16 slots: moe_fast_applies has seen to it
    rc = launch_fast_fp4<true>(p, half, st);
  else if (dtype == SONAR_DTYPE_F16)
    rc = zeros ? launch_fast<_Float16, true, true>(p, unit_group_shift, half, row_blocks, st)
               : launch_fast<_Float16, false, true>(p, unit_group_shift, half, row_blocks, st);
  else
    rc = zeros ? launch_fast<__bf16, true, true>(p, unit_group_shift, half, row_blocks, st)
               : launch_fast<__bf16, false, true>(p, unit_group_shift, half, row_blocks, st);
  if (rc) return rc;
  return launch_status("marlin_stream_fast_kernel (grouped)");
}

}  // namespace sonar

using namespace sonar;

namespace {
size_t stream_scratch_bytes() { return (size_t)2 * cu_count() * kSlotFloat4 * sizeof(float4); }
thread_local int32_t g_last_decode_launch[4] = {0, 0, 0, 0};
}  // namespace


extern "C" size_t sonar_marlin_gemm_scratch_bytes(int64_t size_m, int64_t size_n, int64_t size_k) {
  // partial tiles of the streaming kernels, then those of a split-K tile launch
  return stream_scratch_bytes() + plan_partial_bytes_any(size_m, size_n, size_k);
}

namespace {
// The dense GEMM behind sonar_marlin_gemm (global_scale == nullptr) and sonar_marlin_gemm_nvfp4.
int marlin_gemm_any(const void* a, int64_t a_row_stride, void* c, const uint32_t* b_q_weight, int b_layout,
                    const void* b_bias, const void* b_scales, const float* global_scale, const uint32_t* b_zeros,
                    const int32_t* g_idx, const int32_t* perm, int32_t* workspace, int64_t workspace_len,
                    void* scratch, size_t scratch_bytes, int dtype, int64_t b_type_id, int64_t size_m,
                    int64_t size_n, int64_t size_k, int64_t num_groups, int is_k_full, void* stream,
                    bool make_do = false) {
  // `make_do`: the scratch buffer is of a fixed size (sonar_marlin_gemm_noalloc): beyond the
  // partial tiles of the streaming kernels, which always fit, the call uses what room there is
  // (no K split in the tile kernels without room for their partial tiles).
  SONAR_REQUIRE(size_m >= 0 && size_m < (1LL << 30), "size_m = %ld out of range", (long)size_m);
  Checked chk;
  if (int rc = check_common(chk, b_layout, b_scales, b_zeros, g_idx, perm, dtype, b_type_id, size_n,
                            size_k, num_groups, is_k_full, global_scale != nullptr))
    return rc;
  if (size_m == 0) return SONAR_OK;
  SONAR_REQUIRE(a && c && b_q_weight, "a, c and b_q_weight must not be NULL");
  SONAR_REQUIRE(a_row_stride >= size_k && a_row_stride % 8 == 0, "A.stride(0) must divisible by 8");
  SONAR_REQUIRE(((uintptr_t)a) % 16 == 0, "A must aligned to 16 bytes");
  SONAR_REQUIRE(((uintptr_t)c) % 8 == 0 && ((uintptr_t)b_q_weight) % 16 == 0,
                "c must be 8-byte and b_q_weight 16-byte aligned");
  const int cus = cu_count();
  // The workspace holds the tickets of the strips that workgroups of the decode kernel share
  // (all zero again when the kernel ends; nobody ever waits on one).
  SONAR_REQUIRE(workspace && workspace_len >= cus,
                "workspace.numel = %ld is below min_workspace_size = %d", (long)workspace_len, cus);
  SONAR_REQUIRE(scratch && scratch_bytes >= (make_do ? stream_scratch_bytes()
                                                     : sonar_marlin_gemm_scratch_bytes(size_m, size_n, size_k)),
                "scratch of %zu bytes is too small", scratch_bytes);

  g_last_decode_launch[0] = 0;
  hipStream_t st = (hipStream_t)stream;
  // Act-order with room in the scratch buffer for a copy of A: permute the
  // columns of A once and run the plain grouped kernels on the copy.
  size_t base_scratch = sonar_marlin_gemm_scratch_bytes(size_m, size_n, size_k);
  if (make_do) {   // the copy of A goes before the tile kernels' partial tiles when both do not fit
    const size_t copy_bytes = chk.has_perm ? (size_t)size_m * size_k * 2 : 0;
    const size_t left = scratch_bytes > stream_scratch_bytes() + copy_bytes
                            ? scratch_bytes - stream_scratch_bytes() - copy_bytes : 0;
    if (base_scratch > stream_scratch_bytes() + left) base_scratch = stream_scratch_bytes() + left;
    base_scratch &= ~(size_t)255;
  }
  if (chk.has_perm && scratch_bytes >= base_scratch + (size_t)size_m * size_k * 2) {
    uint16_t* a_tmp = reinterpret_cast<uint16_t*>(static_cast<char*>(scratch) + base_scratch);
    const long vecs = (long)size_m * (size_k / 8);
    const int blocks = (int)((vecs + 255) / 256 < 4096 ? (vecs + 255) / 256 : 4096);
    permute_columns_kernel<<<blocks, 256, 0, st>>>(static_cast<const uint16_t*>(a), a_row_stride, perm, a_tmp,
                                                   (int)size_m, (int)size_k);
    if (int rc = launch_status("permute_columns_kernel")) return rc;
    a = a_tmp;
    a_row_stride = size_k;
    perm = nullptr;
    chk.has_perm = false;
  }
  if (chk.bits == 8 && chk.has_perm)
    return fail(SONAR_E_INVALID,
                "act-order with 8-bit weights needs size_m * size_k * 2 more scratch bytes "
                "(the column-permuted copy of A)");
  if (chk.row_groups && chk.has_perm)
    return fail(SONAR_E_INVALID,
                "act-order with is_k_full = False needs size_m * size_k * 2 more scratch bytes "
                "(the column-permuted copy of A)");

  StreamParams p = {};
  p.b = reinterpret_cast<const uint4*>(b_q_weight);
  p.bias = static_cast<const uint16_t*>(b_bias);
  p.global_scale = global_scale;
  p.scales = static_cast<const uint16_t*>(b_scales);
  p.zeros = b_zeros;
  p.perm = perm;
  p.g_idx = chk.row_groups ? g_idx : nullptr;
  p.scratch = static_cast<float4*>(scratch);
  p.size_n = (int)size_n;
  p.size_k = (int)size_k;
  p.lda = a_row_stride;
  p.num_groups = (int)num_groups;
  p.group_size = chk.row_groups ? (int)size_k : chk.group_size;  // the kernels' own group arithmetic is unused then
  p.chunks_per_strip = (int)(size_k / kChunkK);

  // groups of 128 * 2^s rows: group of a unit = unit >> s
  int unit_group_shift;
  const bool fast_groups = fast_group_shift(num_groups, chk.group_size, unit_group_shift);
  static const bool no_fast = getenv("SONAR_MARLIN_NO_FAST") != nullptr;  // debugging aid
  const bool fast_shape = !no_fast && chk.bits == 4 && !chk.has_perm && !chk.row_groups &&
                          p.chunks_per_strip % 4 == 0 && fast_groups &&
                          size_m * a_row_stride * 2 < (1LL << 31);
  // Short strips (K <= 4096) on a matrix with at least 64 of them: one workgroup
  // per strip.  No strip is shared, so no partial tile goes through memory and
  // the fix-up launch is skipped; measured equal or faster than the even split
  // (qkv 8.7 vs 10.4 us) although fewer compute units stream at a time.  No
  // scratch slot is touched in this mode (slots are sized for `cus` workgroups).
  const int64_t n_strips = size_n / kStripN;
  const bool strip_per_workgroup = p.chunks_per_strip % 4 == 0 && p.chunks_per_strip / 4 <= 32 && n_strips >= 64 &&
                                   (n_strips * (p.chunks_per_strip / 4)) * n_strips < (1LL << 31);
  // 17 to 128 rows on such a matrix: the fast kernel once, with one workgroup
  // per strip and block of 16 rows.  The blocks of a strip stream the same
  // weights at the same time on compute units of one XCD, which would
  // otherwise idle (a Llama-3-8B attention projection has 64 to 96 strips).
  static const bool no_slabs = getenv("SONAR_MARLIN_NO_SLABS") != nullptr;  // debugging aid
  // Up to 64 rows this also pays on matrices whose strips are shared between
  // workgroups (a scratch slot has room for four blocks of rows).
  // Beyond 128 rows the tile kernel takes over, except where it would have few
  // tiles and split K through memory while this kernel needs at most four
  // workgroups of 32 rows per compute unit (measured at K = 4096: N = 4096,
  // M = 256: 21 us against 37; N = 6144, M = 256: 32 against 40; N = 4096,
  // M = 512: 37 against 44; N = 6144, M = 512: 54 against 50).
  const bool few_row_blocks = n_strips * ((size_m + 31) / 32) <= 4 * (int64_t)cus;
  // (groups of 32 / 64 rows take the 16-row kernel up to 16 rows only: measured at K = 4096, N = 11008,
  // M = 64: 43 / 30 us in blocks of rows against 30 / 27 in the general kernel)
  static const bool no_tile = getenv("SONAR_MARLIN_NO_TILE") != nullptr;  // debugging aid
  const bool async_tile = chk.nvfp4 || tile_async_applies(chk.has_perm, num_groups, chk.group_size);
  // (97..128 rows on more strips than compute units: 128-row tiles, see plan_rows_97_128)
  const int steps_per_group = chk.group_size / 64;
  const bool wide128 = chk.bits == 4 && !chk.fp4 && !chk.has_perm && !chk.row_groups &&
                       (num_groups == 1 || (chk.group_size % 64 == 0 && (steps_per_group & (steps_per_group - 1)) == 0));
  const bool rows_97_128 = !no_tile && async_tile && plan_rows_97_128(size_m, size_n, size_k, wide128);
  const bool slab_fast = !no_slabs && fast_shape && size_m > 16 && unit_group_shift >= -1 && !rows_97_128 &&
                         (size_m <= 64 || (strip_per_workgroup && (size_m <= 128 || few_row_blocks)));

  p.unit_chunks = p.chunks_per_strip % 4 == 0 ? 4 : (p.chunks_per_strip % 2 == 0 ? 2 : 1);
  // the general kernel works on half units when it holds more than 32 rows (see unit_buffer_chunks)
  if (size_m > 32 && p.unit_chunks == 4 && !slab_fast) p.unit_chunks = 2;
  p.units_per_strip = p.chunks_per_strip / p.unit_chunks;
  const int64_t total_units = n_strips * p.units_per_strip;
  SONAR_REQUIRE(total_units * cus < (1LL << 31), "size_k * size_n = %ld x %ld is too large", (long)size_k,
                (long)size_n);
  p.total_units = (int)total_units;
  const GemmPlan plan = plan_gemm(size_m, size_n, size_k, async_tile, 256, rows_97_128);
  // the row -> group lookup and 8-bit codes exist in the streaming kernels only
  // (MXFP4 only through the asynchronous tile kernel: the older one has no float4 dequantiser)
  // (8-bit codes and MXFP4 only through the asynchronous tile kernel: the older one has neither dequantiser)
  // (a fixed scratch buffer without room for the partial tiles of up to 128 rows: the tile kernel
  // is planned for those only because K can be split, so they go to the streaming kernels)
  const size_t tile_room = base_scratch > stream_scratch_bytes() ? base_scratch - stream_scratch_bytes() : 0;
  const bool tile_starved = make_do && size_m <= 128 && plan.k_splits > 1 &&
                            tile_room < plan_partial_bytes_any(size_m, size_n, size_k);
  const bool use_tile = plan.tile && !no_tile && !chk.row_groups && ((chk.bits == 4 && !chk.fp4) || async_tile) &&
                        !(slab_fast && p.unit_chunks == 4) && !tile_starved;
  // More than 64 rows in the general kernels (8-bit codes, is_k_full = false,
  // the tile path switched off) on a matrix of short strips: one workgroup per
  // strip as well, so that every 64-row slab can run in the same launch and the
  // slabs of a strip share its weights in L2, instead of one launch per slab
  // that streams all of W again (8-bit, K = 4096, N = 11008, M = 512: 214 us as
  // eight launches).
  const bool row_slabs = !use_tile && !slab_fast && size_m > 64 && strip_per_workgroup &&
                         total_units * n_strips < (1LL << 31);
  p.parts = p.total_units < cus ? p.total_units : cus;
  if (strip_per_workgroup && row_slabs) p.parts = (int)n_strips;
  // One row block on a matrix with about as many strips as compute units: a workgroup per strip, so that
  // no strip is shared and the fix-up launch goes (K = 4096, N = 11008, M = 1: 8-bit codes 18.4 -> 15.0 us,
  // NVFP4 17.2 -> 14.0 us).  (Sixteen wavefronts a workgroup on top of that: 26 us, the unit buffers of
  // the general kernels do not fit 128 registers.)
  // From 48 rows on the even split over all compute units is ahead again (8-bit codes, M = 64: 29.1
  // against 31.2 us).
  if (size_m <= 16 && n_strips >= cus / 2 && n_strips <= 4 * cus) p.parts = (int)n_strips;
  p.slabs = 1;
  p.grid_parts = p.parts;
  p.tickets = nullptr;
  p.ticket_stride = 1;
  p.xcd_ranges = 0;
  p.piece_shift = 0;
  p.piece_units = 0;

  if (use_tile) {
    const size_t used = stream_scratch_bytes();
    return tile_gemm(a, a_row_stride, c, b_q_weight, b_bias, b_scales, global_scale, b_zeros, perm, dtype, size_m,
                     size_n, size_k, num_groups, chk.group_size, static_cast<char*>(scratch) + used, tile_room,
                     chk.fp4, chk.bits, chk.fp8, st);
  }

  // The fast kernel: up to 16 rows, or more rows in blocks of 16 or 32 (slab_fast), all in
  // one launch.  Every strip is cut into the same number of pieces, a power of two, as many
  // as keep the launch at one workgroup per compute unit (a Llama-3-8B attention output
  // projection at M <= 16: 64 strips x 4 pieces), and the pieces of a strip are summed inside
  // the kernel (tickets in the workspace; the fix-up launch when the workspace is too small
  // for them).  With more strips than compute units every strip is one workgroup of four
  // wavefronts, three of which fit a compute unit.
  if (fast_shape && p.unit_chunks == 4 && (size_m <= 16 || slab_fast)) {
    static const bool no_inline_sum = getenv("SONAR_MARLIN_NO_INLINE_SUM") != nullptr;   // debugging aids
    static const char* split_env = getenv("SONAR_MARLIN_SPLIT");
    static const bool no_pairs = getenv("SONAR_MARLIN_NO_ROW_PAIRS") != nullptr;
    static const bool no_half = getenv("SONAR_MARLIN_NO_HALF_WG") != nullptr;
    p.a = static_cast<const uint16_t*>(a);
    p.c = static_cast<uint16_t*>(c);
    p.size_m = (int)size_m;
    const int blocks16 = (int)((size_m + 15) / 16);
    int shift = 0;
    // a scratch slot holds the partial tiles of four blocks of 16 rows, a ticket field counts to 15
    if (size_m <= 64) {
      while (shift < 3 && n_strips * (2 << shift) * blocks16 <= cus && p.units_per_strip % (2 << shift) == 0 &&
             n_strips * (2 << shift) * blocks16 <= workspace_len)
        ++shift;
      if (split_env)
        while (shift > 0 && (1 << shift) > atoi(split_env)) --shift;
    }
    p.piece_shift = shift;
    p.piece_units = p.units_per_strip >> shift;
    p.parts = (int)(n_strips << shift);
    SONAR_REQUIRE(n_strips << shift < (1LL << 30), "size_n = %ld is too large", (long)size_n);
    // Two blocks of rows per workgroup once one block each would make more
    // workgroups than compute units: the weights are then fetched from L2 and
    // unpacked once for 32 rows.
    int row_blocks = 1;
    if (size_m > 16 && !no_pairs && (int64_t)p.parts * blocks16 > cus) row_blocks = 2;
    p.slabs = (int)((size_m + 16 * row_blocks - 1) / (16 * row_blocks));
    p.grid_parts = p.slabs > 1 ? (p.parts + 7) / 8 * 8 : p.parts;
    // more workgroups than compute units: small ones, three per compute unit
    const bool half = !no_half && (int64_t)p.parts * p.slabs > cus;
    const bool split = shift > 0;
    // a split strip leaves one set of partial tiles per contributor in scratch slot `part` or `parts + part`
    if (split)
      SONAR_REQUIRE((size_t)2 * p.parts * kSlotFloat4 * sizeof(float4) <= stream_scratch_bytes() &&
                        p.slabs * row_blocks <= 4,
                    "internal: %d parts x %d blocks of rows share strips but the scratch has slots for %d x 4",
                    p.parts, p.slabs * row_blocks, cus);
    const bool inline_sum = split && !no_inline_sum && (int64_t)p.parts * p.slabs <= workspace_len;
    if (inline_sum) {
      p.tickets = reinterpret_cast<unsigned int*>(workspace);
      const int64_t room = workspace_len / ((int64_t)p.parts * p.slabs);
      p.ticket_stride = room >= 4 ? 4 : (int)room;
      p.xcd_ranges = p.slabs == 1 && p.parts % 8 == 0;
    }
    static const bool no_nt = getenv("SONAR_MARLIN_NO_NT_WEIGHTS") != nullptr;
    p.nt_weights = !no_nt && p.slabs == 1 && size_k * size_n / 2 >= 10 * 1000 * 1000;
    g_last_decode_launch[0] = p.grid_parts * p.slabs;
    g_last_decode_launch[1] = half ? 256 : 512;
    g_last_decode_launch[2] = 1 << shift;
    g_last_decode_launch[3] = p.nt_weights;
    int rc;
    if (chk.fp4)   // groups of 32 rows: never in blocks of rows (slab_fast is off), so one block of 16 rows
      rc = launch_fast_fp4<false>(p, half, st);
    else if (dtype == SONAR_DTYPE_F16)
      rc = chk.has_zp ? launch_fast<_Float16, true>(p, unit_group_shift, half, row_blocks, st)
                      : launch_fast<_Float16, false>(p, unit_group_shift, half, row_blocks, st);
    else
      rc = chk.has_zp ? launch_fast<__bf16, true>(p, unit_group_shift, half, row_blocks, st)
                      : launch_fast<__bf16, false>(p, unit_group_shift, half, row_blocks, st);
    if (rc) return rc;
    if (int rc2 = launch_status("marlin_stream_fast_kernel")) return rc2;
    if (split && !inline_sum) {   // the fix-up kernel reads the split as ranges of units: part i = units [i, i + 1) * piece_units
      p.total_units = (int)total_units;
      if (dtype == SONAR_DTYPE_F16) launch_fixup<_Float16>(p, st);
      else launch_fixup<__bf16>(p, st);
      if (int rc2 = launch_status("marlin_fixup_kernel")) return rc2;
    }
    return SONAR_OK;
  }

  bool any_split = false;
  for (int i = 1; i < p.parts && !any_split; ++i)
    any_split = range_begin(i, p.total_units, p.parts) % p.units_per_strip != 0;

  for (int64_t m0 = 0; m0 < size_m; m0 += 64) {
    p.a = static_cast<const uint16_t*>(a) + m0 * a_row_stride;
    p.c = static_cast<uint16_t*>(c) + m0 * size_n;
    p.size_m = (int)(size_m - m0 < 64 ? size_m - m0 : 64);
    {
      if (row_slabs && !any_split) {   // every 64-row slab in this one launch
        p.size_m = (int)size_m;
        p.slabs = (int)((size_m + 63) / 64);
        p.grid_parts = (p.parts + 7) / 8 * 8;
        m0 = size_m;
      }
      if (chk.bits == 8) {
        if (dtype == SONAR_DTYPE_F16) launch_stream8_mb<_Float16>(p, chk.fp8, st);
        else launch_stream8_mb<__bf16>(p, chk.fp8, st);
      } else if (chk.nvfp4) {
        if (dtype == SONAR_DTYPE_F16) launch_stream_fp4<_Float16, true>(p, st);
        else launch_stream_fp4<__bf16, true>(p, st);
      } else if (chk.fp4) {
        launch_stream_fp4<__bf16>(p, st);
      } else if (dtype == SONAR_DTYPE_F16) {
        if (chk.has_zp) launch_stream_mb<_Float16, true>(p, chk.has_perm, st);
        else launch_stream_mb<_Float16, false>(p, chk.has_perm, st);
      } else {
        if (chk.has_zp) launch_stream_mb<__bf16, true>(p, chk.has_perm, st);
        else launch_stream_mb<__bf16, false>(p, chk.has_perm, st);
      }
    }
    if (int rc = launch_status("marlin_stream_kernel")) return rc;
    if (any_split) {
      if (dtype == SONAR_DTYPE_F16) launch_fixup<_Float16>(p, st);
      else launch_fixup<__bf16>(p, st);
      if (int rc = launch_status("marlin_fixup_kernel")) return rc;
    }
  }
  return SONAR_OK;
}

}  // namespace

extern "C" int sonar_marlin_last_decode_launch(int32_t* out, int n) {
  int i = 0;
  for (; out != nullptr && i < n && i < 4; ++i) out[i] = g_last_decode_launch[i];
  return i;
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
  return marlin_gemm_any(a, a_row_stride, c, b_q_weight, b_layout, b_bias, b_scales, nullptr, b_zeros, g_idx, perm,
                         workspace, workspace_len, scratch, scratch_bytes, dtype, b_type_id, size_m, size_n,
                         size_k, num_groups, is_k_full, stream);
}

extern "C" int sonar_marlin_gemm_nvfp4(const void* a, int64_t a_row_stride, void* c,
                                       const uint32_t* b_q_weight, int b_layout, const void* b_bias,
                                       const void* b_scales, const float* global_scale, int32_t* workspace,
                                       int64_t workspace_len, void* scratch, size_t scratch_bytes, int dtype,
                                       int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups,
                                       void* stream) {
  SONAR_REQUIRE(global_scale != nullptr, "the global_scale parameter must be passed for nvfp4 format.");
  return marlin_gemm_any(a, a_row_stride, c, b_q_weight, b_layout, b_bias, b_scales, global_scale, nullptr, nullptr,
                         nullptr, workspace, workspace_len, scratch, scratch_bytes, dtype, SONAR_TYPE_FLOAT4_E2M1F,
                         size_m, size_n, size_k, num_groups, 1, stream);
}

// ---------------------------------------------------------------------------
// The GEMM for callers that cannot allocate: the scratch memory is this array,
// one copy per GPU that the library runs on, held until the process ends.
namespace {
constexpr size_t kStaticScratchBytes = (size_t)24 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices];   // device address of `scratch` on every device, once asked for
}  // namespace

extern "C" int sonar_marlin_gemm_noalloc(const void* a, int64_t a_row_stride, void* c, const uint32_t* b_q_weight,
                                         int b_layout, const void* b_bias, const void* b_scales,
                                         const uint32_t* b_zeros, const int32_t* g_idx, const int32_t* perm,
                                         int32_t* workspace, int64_t workspace_len, int dtype, int64_t b_type_id,
                                         int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups,
                                         int is_k_full, int use_atomic_add, int use_fp32_reduce, void* stream) {
  SONAR_REQUIRE(size_m >= 0 && size_m < (1LL << 30) && size_n > 0 && size_n < (1LL << 30) && size_k > 0 &&
                    size_k < (1LL << 30),
                "size_m, size_n, size_k = %ld, %ld, %ld out of range", (long)size_m, (long)size_n, (long)size_k);
  int dev = 0;
  SONAR_HIP(hipGetDevice(&dev));
  SONAR_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index %d is beyond the %d this entry point keeps", dev,
                kMaxDevices);
  void* base = __atomic_load_n(&g_static_scratch[dev], __ATOMIC_ACQUIRE);
  if (base == nullptr) {   // first call on this device: the array's address there
    SONAR_HIP(hipGetSymbolAddress(&base, HIP_SYMBOL(scratch)));
    SONAR_REQUIRE(base != nullptr, "hipGetSymbolAddress returned no address for the static scratch array");
    __atomic_store_n(&g_static_scratch[dev], base, __ATOMIC_RELEASE);
  }
  // The whole array: the call takes what it needs of it and makes do where that is less than
  // sonar_marlin_gemm_scratch_bytes() (the partial tiles of the streaming kernels, 8 MiB, always
  // fit; a tile launch whose partial tiles do not runs without splitting K).
  static_assert(kStaticScratchBytes >= ((size_t)16 << 20), "room for the streaming kernels' partial tiles");
  return marlin_gemm_any(a, a_row_stride, c, b_q_weight, b_layout, b_bias, b_scales, nullptr, b_zeros, g_idx, perm,
                         workspace, workspace_len, base, kStaticScratchBytes, dtype, b_type_id, size_m, size_n,
                         size_k, num_groups, is_k_full, stream, true);
}

extern "C" int sonar_marlin_dequant(const uint32_t* b_q_weight, int b_layout, const void* b_scales,
                                    const uint32_t* b_zeros, const int32_t* g_idx, void* w_out,
                                    int dtype, int64_t b_type_id, int64_t size_n, int64_t size_k,
                                    int64_t num_groups, int is_k_full, void* stream) {
  Checked chk;
  // float4 codes with one scale per 16 rows are NVFP4 (without its global scale: value x block scale)
  const bool nvfp4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F && size_k == 16 * num_groups;
  if (int rc = check_common(chk, b_layout, b_scales, b_zeros, g_idx, g_idx, dtype, b_type_id, size_n,
                            size_k, num_groups, is_k_full, nvfp4))
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
  if (chk.bits == 8) {
    const long total_blocks = (size_n / kStripN) * (size_k / 16);
    long grid = (total_blocks + 3) / 4;
    if (grid > 8192) grid = 8192;
    const int32_t* gi8 = chk.row_groups ? g_idx : nullptr;
    if (chk.fp8) {
      if (dtype == SONAR_DTYPE_F16) marlin_dequant8_kernel<_Float16, true><<<(int)grid, 256, 0, st>>>(b, s, gi8, w, n, k, ng, gs, total_blocks);
      else marlin_dequant8_kernel<__bf16, true><<<(int)grid, 256, 0, st>>>(b, s, gi8, w, n, k, ng, gs, total_blocks);
    } else if (dtype == SONAR_DTYPE_F16) {
      marlin_dequant8_kernel<_Float16, false><<<(int)grid, 256, 0, st>>>(b, s, gi8, w, n, k, ng, gs, total_blocks);
    } else {
      marlin_dequant8_kernel<__bf16, false><<<(int)grid, 256, 0, st>>>(b, s, gi8, w, n, k, ng, gs, total_blocks);
    }
    return launch_status("marlin_dequant8_kernel");
  }
  const int32_t* gi = chk.row_groups ? g_idx : nullptr;
  if (chk.nvfp4) {
    if (dtype == SONAR_DTYPE_F16) marlin_dequant_kernel<_Float16, false, true, true><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, gi, w, n, k, ng, gs, total_chunks);
    else marlin_dequant_kernel<__bf16, false, true, true><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, gi, w, n, k, ng, gs, total_chunks);
  } else if (chk.fp4) {
    marlin_dequant_kernel<__bf16, false, true><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, gi, w, n, k, ng, gs, total_chunks);
  } else if (dtype == SONAR_DTYPE_F16) {
    if (chk.has_zp) marlin_dequant_kernel<_Float16, true><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, gi, w, n, k, ng, gs, total_chunks);
    else marlin_dequant_kernel<_Float16, false><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, gi, w, n, k, ng, gs, total_chunks);
  } else {
    if (chk.has_zp) marlin_dequant_kernel<__bf16, true><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, gi, w, n, k, ng, gs, total_chunks);
    else marlin_dequant_kernel<__bf16, false><<<(int)blocks, 256, 0, st>>>(b, s, b_zeros, gi, w, n, k, ng, gs, total_chunks);
  }
  return launch_status("marlin_dequant_kernel");
}
