// Tiled W4A16 GEMM for more than 64 activation rows (the MFMA-bound regime).
//
// A workgroup of eight wavefronts owns a 256 (rows of A) x 256 (columns of W)
// tile of C and walks K in steps of 64.  Per step, four wavefronts each fetch
// one 1-KiB chunk of packed weights per 32 rows (64 columns x 32 rows, already
// in operand order), dequantise it in registers and store the result to LDS as
// four 16-column operand blocks; all eight wavefronts fetch the 256 x 64 slice
// of A and store it to LDS as 16-row operand blocks.  An operand block is 64
// lanes x 16 bytes: exactly what one v_mfma_f32_16x16x32 reads, so every LDS
// read of the inner loop is a linear, conflict-free ds_read_b128.  LDS is
// double-buffered; the global loads of step i+1 are issued before the matrix
// work of step i and land in registers meanwhile.  Each wavefront computes a
// 128 x 64 sub-tile: 8 x 4 accumulator tiles, weights as the row operand
// (D[n][m]) so a lane ends up with four consecutive columns of one row of C.
//
// Workgroup ids are dealt so that the 32 workgroups resident on one XCD (ids
// congruent mod 8) take neighbouring tiles (tile_of_workgroup).
#include <cstdlib>
#include <type_traits>

#include "dequant.hpp"
#include "gemm_plan.hpp"

namespace sonar {
namespace {

constexpr int kTileM = 256;
constexpr int kTileN = 256;
constexpr int kTileK = 64;
constexpr int kTileWaves = 8;
constexpr int kBlockBytes = 1024;                          // one operand block
constexpr int kStageA = (kTileM / 16) * (kTileK / 32) * kBlockBytes;  // 32 KiB
constexpr int kStageB = (kTileN / 16) * (kTileK / 32) * kBlockBytes;  // 32 KiB
constexpr int kStageBytes = kStageA + kStageB;
constexpr int kTileLds = 2 * kStageBytes;                  // 128 KiB

struct TileParams {
  const uint16_t* a;
  long lda;
  uint16_t* c;
  const uint4* b;
  const uint16_t* bias;
  const float* global_scale;   // NVFP4: one number the output is multiplied by; else nullptr
  const uint16_t* scales;
  const uint32_t* zeros;
  const int32_t* perm;
  int size_m, size_n, size_k;
  int num_groups, group_size;
  int chunks_per_strip;
  int tiles_m, tiles_n;
  int tile_rows;               // rows of a tile: 256 (128: marlin_tile_wide_kernel with 8 row blocks)
  int tile_band;               // rows of tiles per band of the tile numbering (tile_of_workgroup)
  // the launch covers tiles [tile_begin, tile_begin + tile_count) of the numbering (tile_count 0: all of them)
  int tile_begin, tile_count;
  // split K (k_splits > 1): workgroup (tile, split) of a split tile covers K steps
  // [split * k_steps_per_split, ...) and leaves its fp32 tile in `partial` for tile_reduce_kernel
  int k_splits, k_steps_per_split;
  int whole_tiles;             // with k_splits > 1: tiles 0..whole_tiles-1 of the numbering are not split
  float4* partial;
  // grouped (mixture-of-experts) calls only
  const int32_t* sorted_ids;   // slot -> row id of C (row id / top_k of A), >= rows_total: padding
  const float* topk_weights;
  const int32_t* tile_table;   // [0]: number of row tiles, then (first block, blocks, expert) per tile
  int rows_total, top_k, mul_topk;
  int a_by_slot;               // grouped: row of A = slot index (a column-permuted copy made per slot), else row id / top_k
  long expert_b_stride;        // uint4 units between experts in b
  long expert_s_stride, expert_z_stride, expert_bias_stride;  // elements between experts
};

// 16 bytes (8 consecutive k) of row `row` of A, gathered through perm when given.
template <bool HAS_PERM>
__device__ __forceinline__ uint4 load_a16(const TileParams& p, int row, int k0) {
  const uint16_t* arow = p.a + (long)(row < p.size_m ? row : p.size_m - 1) * p.lda;
  if (!HAS_PERM) return *reinterpret_cast<const uint4*>(arow + k0);
  const int4 p0 = *reinterpret_cast<const int4*>(p.perm + k0);
  const int4 p1 = *reinterpret_cast<const int4*>(p.perm + k0 + 4);
  uint4 v;
  v.x = (uint32_t)arow[p0.x] | ((uint32_t)arow[p0.y] << 16);
  v.y = (uint32_t)arow[p0.z] | ((uint32_t)arow[p0.w] << 16);
  v.z = (uint32_t)arow[p1.x] | ((uint32_t)arow[p1.y] << 16);
  v.w = (uint32_t)arow[p1.z] | ((uint32_t)arow[p1.w] << 16);
  return v;
}

// Tiles are numbered band by band (tile_band rows of tiles), inside a band
// column by column: with bands of 4 rows, 32 consecutive tiles are 4 panels
// of A x 8 panels of W.
__host__ __device__ __forceinline__ void tile_coords(const TileParams& p, int tile, int& tile_m, int& tile_n) {
  const int band = tile / (p.tile_band * p.tiles_n);
  const int rem = tile - band * p.tile_band * p.tiles_n;
  const int rows = min(p.tile_band, p.tiles_m - band * p.tile_band);
  tile_n = rem / rows;
  tile_m = band * p.tile_band + rem - tile_n * rows;
}
// Tiles of the launch, and those of them computed by one workgroup over the whole of K (the first ones).
__host__ __device__ __forceinline__ int launch_tiles(const TileParams& p) {
  return p.tile_count > 0 ? p.tile_count : p.tiles_m * p.tiles_n;
}
__host__ __device__ __forceinline__ int whole_tiles(const TileParams& p) {
  return p.k_splits > 1 ? p.whole_tiles : launch_tiles(p);
}

// Workgroup id -> (tile, K range).  Workgroups whose ids are congruent mod 8
// run on one XCD and share its L2: each XCD takes a contiguous run of the
// whole tiles, rows of A innermost, so the workgroups resident on it share a
// few panels of W, and after those a contiguous run of the (tile, split) pairs
// of the split tiles, so that the short workgroups start last on every XCD.
// Returns false for the padding ids of a run.
__host__ __device__ __forceinline__ bool tile_of_block(const TileParams& p, int block, int& tile, int& split,
                                                       bool& whole_k) {
  const int tiles = launch_tiles(p);
  const int whole = whole_tiles(p);
  const int split_tiles = tiles - whole;
  const int whole_per_xcd = (whole + 7) / 8;
  const int split_per_xcd = (split_tiles * p.k_splits + 7) / 8;
  const int xcd = block & 7, i = block >> 3;
  whole_k = i < whole_per_xcd;
  if (whole_k) {
    tile = xcd * whole_per_xcd + i;
    split = 0;
    const bool mine = tile < whole;
    tile += p.tile_begin;   // (a launch over a part of the numbering never splits K)
    return mine;
  }
  // (a grouped launch is sized for the most tiles there could be: ids past this XCD's share do nothing)
  if (i - whole_per_xcd >= split_per_xcd) return false;
  const int t = xcd * split_per_xcd + (i - whole_per_xcd);
  if (t >= split_tiles * p.k_splits) return false;
  split = t / split_tiles;
  tile = whole + t - split * split_tiles;
  return true;
}
__device__ __forceinline__ bool tile_of_workgroup(const TileParams& p, int& tile, int& split, bool& whole_k) {
  return tile_of_block(p, blockIdx.x, tile, split, whole_k);
}

// Grouped calls learn the number of their tiles on the device (the routing decides it), so the
// kernel plans the K split itself, by plan_gemm's rules: fewer tiles than compute units, or a last
// round of workgroups that fills half of the chip or less, are cut along K into about 256
// workgroups, in ranges of a multiple of four steps (the caller has checked that K allows it).
constexpr int kLiveSplitTilesMax = 128;   // tiles that can be split, and
constexpr int kLiveSplitWorkMax = 256;    // (tile, K range) pairs, i.e. partial tiles, there can be
struct LiveSplit {
  int whole, splits, steps;   // tiles computed over the whole of K; K ranges per split tile; steps per range
};
__host__ __device__ __forceinline__ LiveSplit plan_live_split(int tiles, int k_steps) {
  LiveSplit s = {tiles, 1, k_steps};
  int split_tiles = 0;
  if (tiles < 256) split_tiles = tiles;
  else if (k_steps >= 48 && tiles % 256 <= 128) split_tiles = tiles % 256;
  if (split_tiles == 0 || split_tiles > kLiveSplitTilesMax) return s;
  int splits = 256 / split_tiles;
  if (splits > k_steps / 8) splits = k_steps / 8;
  if (splits > 16) splits = 16;
  if (splits < 2) return s;
  const int steps = ((k_steps + splits - 1) / splits + 3) / 4 * 4;
  splits = (k_steps + steps - 1) / steps;   // no empty range
  if (splits < 2) return s;
  s.whole = tiles - split_tiles;
  s.splits = splits;
  s.steps = steps;
  return s;
}
// The tiles there are in a grouped call (`row_tiles` of them down the rows), with the K split
// planned from them when the call has room for partial tiles.
__host__ __device__ __forceinline__ TileParams live_tiles_of(const TileParams& p, int row_tiles) {
  TileParams live = p;
  live.tiles_m = row_tiles;
  live.tile_band = p.tile_rows == kTileM ? 4 : 8;   // the same rows of A per band with either tile size
  if (p.partial != nullptr) {
    const LiveSplit s = plan_live_split(live.tiles_m * live.tiles_n, p.size_k / kTileK);
    live.k_splits = s.splits;
    live.whole_tiles = s.whole;
    live.k_steps_per_split = s.steps;
  }
  return live;
}
__device__ __forceinline__ TileParams live_tiles(const TileParams& p) { return live_tiles_of(p, p.tile_table[0]); }

inline int tile_grid(const TileParams& p) {
  const int whole = whole_tiles(p);
  const int split_work = (launch_tiles(p) - whole) * p.k_splits;
  // (a grouped call with room for partial tiles: the kernel may turn up to 128 of its tiles into 256 K ranges)
  const int live_split = p.tile_table != nullptr && p.partial != nullptr ? kLiveSplitWorkMax : 0;
  return 8 * ((whole + 7) / 8 + (split_work + live_split + 7) / 8);
}

template <typename T, bool HAS_ZP, bool HAS_PERM>
__global__ __launch_bounds__(kTileWaves * 64) void marlin_tile_kernel(const TileParams p) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq<T>::Col Col;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col16 = lane & 15;
  const int kb = lane >> 4;
  const uint32_t magic = magic_register();
  const bool grouped = p.num_groups > 1;

  int tile, tile_m, tile_n, split;
  bool whole_k;
  if (!tile_of_workgroup(p, tile, split, whole_k)) return;  // this kernel is launched with k_splits == 1
  tile_coords(p, tile, tile_m, tile_n);
  const int m0 = tile_m * kTileM;
  const int strip0 = tile_n * (kTileN / kStripN);
  const int strips_here = min(kTileN / kStripN, p.size_n / kStripN - strip0);

  // ---- what this thread fetches per K step
  // A: the 256 x 64 slice is 32 operand blocks (16 row blocks x 2 k blocks);
  // thread t fills lane t%64 of blocks t/64 + 8*i, i = 0..3.
  // W: wavefronts 0..3 each own one strip of the tile and fetch its two chunks.
  const bool loads_b = wave < strips_here;
  const uint4* b_src = p.b + (size_t)(unsigned)((strip0 + (loads_b ? wave : 0)) * p.chunks_per_strip) * 64 + lane;
  const uint16_t* s_src = p.scales + (strip0 + (loads_b ? wave : 0)) * kStripN;
  const uint32_t* z_src = HAS_ZP ? p.zeros + (strip0 + (loads_b ? wave : 0)) * 8 + zero_point_word(col16) : nullptr;
  int s_slot[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) s_slot[j] = scale_slot(16 * j + col16, grouped);

  // ---- what this wavefront computes
  const int wm = wave >> 2;   // rows 128*wm .. +128 of the tile
  const int wn = wave & 3;    // strip wn of the tile
  floatx4_t acc[4][8];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) acc[nb][mb] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  uint4 a_reg[4];
  uint4 b_reg[2];
  uint32_t s_reg[2][4];
  uint32_t z_reg[2];

  auto fetch = [&](int kt) {
    const int k0 = kt * kTileK;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int blk = wave + 8 * i;          // 0..31: row block blk>>1, k block blk&1
      a_reg[i] = load_a16<HAS_PERM>(p, m0 + 16 * (blk >> 1) + col16, k0 + 32 * (blk & 1) + 8 * kb);
    }
    if (loads_b) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int chunk = kt * 2 + h;
        b_reg[h] = b_src[(size_t)chunk * 64];
        const int g = grouped ? (chunk * kChunkK) / p.group_size : 0;
        const uint16_t* srow = s_src + (long)g * p.size_n;
#pragma unroll
        for (int j = 0; j < 4; ++j) s_reg[h][j] = srow[s_slot[j]];
        if (HAS_ZP) z_reg[h] = z_src[(long)g * (p.size_n / 8)];
      }
    }
  };

  auto stash = [&](int stage) {
    char* sa = smem + stage * kStageBytes;
    char* sb = sa + kStageA;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<uint4*>(sa + (wave + 8 * i) * kBlockBytes + lane * 16) = a_reg[i];
    if (loads_b) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        Col cols[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          int z = 8;
          if (HAS_ZP) z = (int)((z_reg[h] >> zero_point_shift(16 * j + col16)) & 0xFu);
          cols[j] = Dq<T>::make_col((uint16_t)s_reg[h][j], z);
        }
        const uint32_t words[4] = {b_reg[h].x, b_reg[h].y, b_reg[h].z, b_reg[h].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const vec8 w = Dq<T>::word(words[j], cols[j], magic);
          // column block 4*wave + j of the tile, k block h
          *reinterpret_cast<vec8*>(sb + ((4 * wave + j) * 2 + h) * kBlockBytes + lane * 16) = w;
        }
      }
    }
  };

  const int k_tiles = p.size_k / kTileK;
  fetch(0);
  stash(0);
  __syncthreads();

  for (int kt = 0; kt < k_tiles; ++kt) {
    if (kt + 1 < k_tiles) fetch(kt + 1);
    const char* sa = smem + (kt & 1) * kStageBytes;
    const char* sb = sa + kStageA;
    if (wn < strips_here) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        vec8 wv[4];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
          wv[nb] = *reinterpret_cast<const vec8*>(sb + ((4 * wn + nb) * 2 + h) * kBlockBytes + lane * 16);
#pragma unroll
        for (int mb = 0; mb < 8; ++mb) {
          const vec8 av =
              *reinterpret_cast<const vec8*>(sa + ((8 * wm + mb) * 2 + h) * kBlockBytes + lane * 16);
#pragma unroll
          for (int nb = 0; nb < 4; ++nb) acc[nb][mb] = Dq<T>::mfma(wv[nb], av, acc[nb][mb]);
        }
      }
    }
    if (kt + 1 < k_tiles) stash((kt + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds C[m][n .. n+3] for m = row block + lane%16
  if (wn >= strips_here) return;
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int n = (strip0 + wn) * kStripN + 16 * nb + 4 * kb;
    float bias[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        bias[r] = Dq<T>::to_float(p.bias[(strip0 + wn) * kStripN + scale_slot(16 * nb + 4 * kb + r, false)]);
    }
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) {
      const int m = m0 + 128 * wm + 16 * mb + col16;
      if (m < p.size_m) {
        const floatx4_t v = acc[nb][mb];
        uint2 o;
        o.x = (uint32_t)Dq<T>::from_float(v.x + bias[0]) | ((uint32_t)Dq<T>::from_float(v.y + bias[1]) << 16);
        o.y = (uint32_t)Dq<T>::from_float(v.z + bias[2]) | ((uint32_t)Dq<T>::from_float(v.w + bias[3]) << 16);
        *reinterpret_cast<uint2*>(p.c + (long)m * p.size_n + n) = o;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The same tile with every operand arriving through asynchronous global -> LDS
// copies, three K steps deep, so no vector register holds bytes in flight and
// the copies of step i+2 are issued before the matrix work of step i.
//   * A: a ring of three 32-KiB stages shared by the workgroup, each 32
//     regions of 8 rows x 128 bytes; wavefront w copies regions 4w..4w+3, one
//     copy per region, eight whole 128-byte lines per copy.
//   * W: the packed chunks are already in operand order.  Every wavefront
//     copies the two chunks of its strip (and the scale / zero-point row of the
//     step's group) into a private ring and dequantises them in registers.
// The eight wavefronts form two groups (wm = 0: rows 0..127 of the tile, wm = 1:
// rows 128..255); each SIMD holds one wavefront of either group.  A K step is
// two half steps (k blocks 0 and 1), a half step is a "fetch" phase (the copies
// of a later stage, the LDS read of one packed chunk, dequantisation: VALU
// work) followed by a "multiply" phase (32 MFMAs and, behind the four of a row
// block, the LDS read of that row block's operand of the next half step; a
// group reads only rows of A that its own wavefronts copied).  Phases end with
// a workgroup barrier and group 1 runs one phase behind group 0, so that on
// every SIMD one wavefront multiplies while the other fetches.  The fetch phase
// is the longer one: while its sibling issues MFMAs a wavefront gets a VALU
// instruction through every eight cycles or so, and its copies and LDS
// instructions take their issue time on top of that.
// Copies of a wavefront complete in issue order, seven per stage, so "stage i
// has landed" is s_waitcnt vmcnt(7) while the copies of stage i+1 are
// outstanding.  With p = 4 kt + 2 b (+1 for group 1) the phase in which the
// fetch of (step kt, k block b) runs: stage kt is read in phases 4kt..4kt+3; the
// copies of stage kt+2 go to the slot of stage kt-1 and are issued in the two
// fetch phases of step kt, phases 4kt..4kt+3, after the barrier that ends
// phase 4kt-1; every wavefront waits for its copies of stage kt+1 at the end of
// its fetch of (kt, 1), phases 4kt+2 and 4kt+3, before the barrier that starts
// phase 4kt+4.
// LDS is read from asm blocks only (the compiler cannot tell which LDS bytes a
// copy writes and would otherwise wait for all copies before any LDS access).
// Needs groups of 32 rows or a multiple of 64 (or one group) and no act-order.
constexpr int kAsyncStages = 3;
// G32: groups of 32 rows, i.e. one group per k block: a stage then carries two
// scale / zero-point rows (256 bytes each) and takes one copy more.
constexpr int wave_stage(bool g32) { return 2 * kBlockBytes + (g32 ? 512 : 256); }   // two weight chunks + scale rows
constexpr int kAsyncA = kAsyncStages * kStageA;
constexpr int async_lds(bool g32) { return kAsyncA + kTileWaves * kAsyncStages * wave_stage(g32); }
constexpr int async_copies(bool g32) { return g32 ? 8 : 7; }
// 8-bit codes (W8 = 1: uint8b128, 2: float8_e4m3fn): a K step of a strip is four 1-KiB blocks
// of 16 rows (block 2 b holds the low four, block 2 b + 1 the high four of the eight
// consecutive rows of a lane's operand of k block b).  Private rings of that size would not
// fit, so the two wavefronts of a strip (one per group of rows) share one ring: the
// wavefront of group 0 copies the two blocks of k block 0, that of group 1 those of k block
// 1, the same number of copies per stage as with 4-bit codes.  The barriers that order the
// shared stages of A order these too: group 1 reads k block 0 one phase after group 0 has
// waited for its copies, group 0 reads k block 1 two barriers after group 1 has.
constexpr int strip_stage8(bool g32) { return 4 * kBlockBytes + (g32 ? 512 : 256); }
constexpr int async_lds8(bool g32) { return kAsyncA + (kTileN / kStripN) * kAsyncStages * strip_stage8(g32); }

// NV (with G32 and FP4): NVFP4, groups of 16 rows.  The scale rows of a stage then hold four
// groups of 128 bytes (a copy fetches two rows, one per half of the wavefront), and a lane,
// whose eight rows of a k block lie in one group, reads the row of group 2 b + kb / 2.
template <typename T, bool HAS_ZP, bool GROUPED, bool G32 = false, bool FP4 = false, int W8 = 0, bool NV = false>
__global__ __launch_bounds__(kTileWaves * 64) void marlin_tile_async_kernel(const TileParams p) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq4Of<T, FP4, NV>::type D4;   // integer codes, or float4_e2m1f (MXFP4 / NVFP4: with G32)
  static_assert(!NV || (G32 && FP4 && !HAS_ZP && W8 == 0), "NVFP4 is float4 codes with groups of 16 rows");
  typedef typename Dq8Of<T, W8 == 2>::type D8;   // 8-bit integer or floating-point codes (W8 != 0)
  typedef typename std::conditional<W8 != 0, typename D8::Col, typename D4::Col>::type Col;
  static_assert(W8 == 0 || (!HAS_ZP && !FP4), "8-bit codes are symmetric");
  constexpr int kWaveStage = W8 ? strip_stage8(G32) : wave_stage(G32);
  constexpr int kWeightBytes = (W8 ? 4 : 2) * kBlockBytes;   // packed weights of a stage, scale rows behind them
  constexpr int kAsyncCopies = async_copies(G32);
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col16 = lane & 15;
  const int kb = lane >> 4;
  const uint32_t magic = magic_register();
  const bool grouped = p.num_groups > 1;

  int tile, tile_m, tile_n, split;
  bool whole_k;
  if (!tile_of_workgroup(p, tile, split, whole_k)) return;
  tile_coords(p, tile, tile_m, tile_n);
  // Grouped calls: row tile t is up to four consecutive 64-slot blocks of one
  // expert, listed in tile_table; rows are slots of sorted_ids.
  int first_slot = 0, tile_rows = kTileM;
  long expert = 0;
  if (GROUPED) {
    if (tile_m >= p.tile_table[0]) return;
    first_slot = p.tile_table[1 + 3 * tile_m] * 64;
    tile_rows = p.tile_table[2 + 3 * tile_m] * 64;
    expert = p.tile_table[3 + 3 * tile_m];
  }
  const int m0 = tile_m * kTileM;
  const int strip0 = tile_n * (kTileN / kStripN);
  const int strips_here = min(kTileN / kStripN, p.size_n / kStripN - strip0);
  const int wm = wave >> 2;
  const int wn = wave & 3;
  const bool active = wn < strips_here;
  // a wavefront past the last strip copies the last strip again and computes nothing
  const int strip = strip0 + (active ? wn : strips_here - 1);

  // ---- copy sources
  // A stage is 32 regions of 1 KiB: region 2 rb + h holds rows 8h..8h+7 of row
  // block rb, 128 bytes (both k blocks) each.  One copy fills one region: its
  // lanes 8r..8r+7 fetch the eight 16-byte pieces of one 128-byte line of row r,
  // so an instruction touches 8 whole lines (16 rows x 64 bytes per instruction,
  // the operand-block shape, moves a third of the bytes per cycle).  Piece q of
  // row r sits at 16-byte slot q ^ r of the row, which keeps the operand reads
  // (16 rows, one piece each) off each other's banks.  Wavefront w fills
  // regions 4w..4w+3.
  const char* a_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int region = 4 * wave + i;
    const int r8 = lane >> 3;
    const int in_tile = 16 * (region >> 1) + 8 * (region & 1) + r8;
    int row;
    if (GROUPED) {
      const int id = in_tile < tile_rows ? p.sorted_ids[first_slot + in_tile] : p.rows_total;
      // padding slots read row 0, never stored
      row = (unsigned)id < (unsigned)p.rows_total ? (p.a_by_slot ? first_slot + in_tile : id / p.top_k) : 0;
    } else {
      row = m0 + in_tile;
      if (row >= p.size_m) row = p.size_m - 1;  // rows past M are computed and never stored
    }
    a_src[i] = reinterpret_cast<const char*>(p.a) + ((long)row * p.lda + 8 * ((lane & 7) ^ r8)) * 2;
  }
  const uint4* b_src = p.b + expert * p.expert_b_stride +
                       (size_t)(unsigned)(strip * p.chunks_per_strip) * (W8 ? 128 : 64) + lane;
  const char* s_src;
  long s_group_stride;
  if (HAS_ZP && lane >= 32) {
    s_src = reinterpret_cast<const char*>(p.zeros + expert * p.expert_z_stride + strip * 8 + (lane & 7));
    s_group_stride = (long)(p.size_n / 8) * 4;
  } else {
    s_src = reinterpret_cast<const char*>(p.scales + expert * p.expert_s_stride + strip * kStripN) + 4 * (lane & 31);
    s_group_stride = (long)p.size_n * 2;
    if (NV) s_src += (lane >> 5) * s_group_stride;   // the upper half of the wavefront fetches the next group's row
  }
  // the weight ring: private to the wavefront, or shared by the two wavefronts of a strip (8-bit codes)
  char* wring = smem + kAsyncA + (W8 ? wn : wave) * (kAsyncStages * kWaveStage);
  const uint32_t a_lds = (uint32_t)(uintptr_t)(lds_void_t*)smem;
  const uint32_t w_lds = (uint32_t)(uintptr_t)(lds_void_t*)wring;

  // copy `idx` (0..6) of the stage of step kt: four blocks of A, two weight chunks, one scale row
  auto issue_one = [&](int kt, int slot, int idx) {
    if (idx < 4) {
      char* sa = smem + slot * kStageA;
      __builtin_amdgcn_global_load_lds((glb_void_t*)(a_src[idx] + (long)kt * (kTileK * 2)),
                                       (lds_void_t*)(sa + (4 * wave + idx) * kBlockBytes), 16, 0, 0);
      return;
    }
    char* sw = wring + slot * kWaveStage;
    if (idx < 6) {
      if (W8) {   // blocks 2 wm, 2 wm + 1 of the four of this step: the two of k block wm
        const int blk = 2 * wm + (idx - 4);
        const uint4* g = b_src + (size_t)(4 * kt + blk) * 64;
        __builtin_amdgcn_global_load_lds((glb_void_t*)g, (lds_void_t*)(sw + blk * kBlockBytes), 16, 0, 0);
        return;
      }
      const uint4* g = b_src + (size_t)(2 * kt + (idx - 4)) * 64;   // the two chunks of this step
      __builtin_amdgcn_global_load_lds((glb_void_t*)g, (lds_void_t*)(sw + (idx - 4) * kBlockBytes), 16, 0, 0);
      return;
    }
    // the scale rows (with a shared ring both wavefronts of the strip copy them: the same bytes twice)
    if (G32) {   // idx 6 / 7: the rows of groups 2 kt and 2 kt + 1
      __builtin_amdgcn_global_load_lds((glb_void_t*)(s_src + (long)((NV ? 4 : 2) * kt + (NV ? 2 : 1) * (idx - 6)) *
                                                                 s_group_stride),
                                       (lds_void_t*)(sw + kWeightBytes + 256 * (idx - 6)), 4, 0, 0);
      return;
    }
    const int grp = grouped ? (kt * kTileK) / p.group_size : 0;
    __builtin_amdgcn_global_load_lds((glb_void_t*)(s_src + (long)grp * s_group_stride),
                                     (lds_void_t*)(sw + kWeightBytes), 4, 0, 0);
  };
  auto issue = [&](int kt, int slot) {
#pragma unroll
    for (int idx = 0; idx < kAsyncCopies; ++idx) issue_one(kt, slot, idx);
  };

  uint32_t s_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) s_off[j] = kWeightBytes + 2 * scale_slot(16 * j + col16, grouped);
  const uint32_t z_off = kWeightBytes + 128 + 4 * zero_point_word(col16);

  floatx4_t acc[4][8];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) acc[nb][mb] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  // K steps [k_first, k_tiles) of this workgroup
  const int k_first = whole_k ? 0 : split * p.k_steps_per_split;
  const int k_tiles = whole_k ? p.size_k / kTileK : min(p.size_k / kTileK, k_first + p.k_steps_per_split);
  issue(k_first, 0);
  issue(min(k_first + 1, k_tiles - 1), 1);

  u32x4_t av[8], wv[4], qraw;
  u32x4_t qhigh = u32x4_t{0u, 0u, 0u, 0u};   // 8-bit codes: the block with the high four rows
  uint32_t sb0 = 0, sb1 = 0, sb2 = 0, sb3 = 0, zw = 0;
  Col cols[4];
// Starts one 16-byte LDS read into `dst`; the data is there after the next
// s_waitcnt lgkmcnt(0) that names `dst` as an operand.  Until then nothing may
// name `dst` (the hardware does not interlock).
#define SONAR_TILE_READ(dst, base, off) \
  asm volatile("ds_read_b128 %0, %1 offset:" #off : "=&v"(dst) : "v"(base) : "memory")
// Waits for every LDS read in flight; the registers they fill are operands so
// that no use of them can be scheduled ahead of the wait.
#define SONAR_TILE_LANDED()                                                                        \
  asm volatile("s_waitcnt lgkmcnt(0)"                                                              \
               : "+v"(av[0]), "+v"(av[1]), "+v"(av[2]), "+v"(av[3]), "+v"(av[4]), "+v"(av[5]),     \
                 "+v"(av[6]), "+v"(av[7])                                                          \
               :                                                                                   \
               : "memory")
  // Starts the reads of the packed chunk of (stage in `slot`, k block b), with
  // the scales and zero points of the step when `with_scales` (they hold for
  // both k blocks: a step lies inside one group).  The wavefront's own copies of
  // that stage must have landed.  The data is picked up by the next fetch().
  auto raw_start = [&](int slot, int b, bool with_scales) {
    const uint32_t w_at = w_lds + slot * kWaveStage;
    const uint32_t q_at = w_at + (W8 ? 2 * b : b) * kBlockBytes + lane * 16;
    const uint32_t r_at = w_at + (NV ? 128 * (2 * b + (kb >> 1)) : (G32 ? 256 * b : 0));   // this k block's scale row
    if constexpr (W8 != 0) asm volatile("ds_read_b128 %0, %1 offset:1024" : "=&v"(qhigh) : "v"(q_at) : "memory");
    if (with_scales) {
      asm volatile(
          "ds_read_b128 %0, %6\n\t"
          "ds_read_u16 %1, %7\n\t"
          "ds_read_u16 %2, %8\n\t"
          "ds_read_u16 %3, %9\n\t"
          "ds_read_u16 %4, %10\n\t"
          "ds_read_b32 %5, %11"
          : "=&v"(qraw), "=&v"(sb0), "=&v"(sb1), "=&v"(sb2), "=&v"(sb3), "=&v"(zw)
          : "v"(q_at), "v"(r_at + s_off[0]), "v"(r_at + s_off[1]), "v"(r_at + s_off[2]), "v"(r_at + s_off[3]),
            "v"(NV ? r_at + s_off[0] : r_at + z_off)
          : "memory");
    } else {
      asm volatile("ds_read_b128 %0, %1" : "=&v"(qraw) : "v"(q_at) : "memory");
    }
  };
  // Fetch phase of a half step: picks up the packed chunk started by raw_start
  // and dequantises it, then waits for the operands of A the last multiply
  // phase started to read.
  auto fetch = [&](int slot, int b, bool with_scales) {
    if constexpr (W8 != 0) {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(qraw), "+v"(qhigh), "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw)
                   :
                   : "memory");
    } else {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(qraw), "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw)
                   :
                   : "memory");
    }
    if (with_scales) {
      const uint32_t sbits[4] = {sb0, sb1, sb2, sb3};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (W8 != 0) {
          cols[j] = D8::make_col((uint16_t)sbits[j]);
        } else {
          int z = 8;
          if (HAS_ZP) z = (int)((zw >> zero_point_shift(16 * j + col16)) & 0xFu);
          cols[j] = D4::make_col((uint16_t)sbits[j], z);
        }
      }
    }
    if constexpr (W8 != 0) {
      const uint32_t lo[4] = {qraw.x, qraw.y, qraw.z, qraw.w}, hi[4] = {qhigh.x, qhigh.y, qhigh.z, qhigh.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint2 w_lo = D8::word4(lo[j], cols[j], magic), w_hi = D8::word4(hi[j], cols[j], magic);
        wv[j] = u32x4_t{w_lo.x, w_lo.y, w_hi.x, w_hi.y};
      }
    } else {
      wv[0] = __builtin_bit_cast(u32x4_t, D4::word(qraw.x, cols[0], magic));
      wv[1] = __builtin_bit_cast(u32x4_t, D4::word(qraw.y, cols[1], magic));
      wv[2] = __builtin_bit_cast(u32x4_t, D4::word(qraw.z, cols[2], magic));
      wv[3] = __builtin_bit_cast(u32x4_t, D4::word(qraw.w, cols[3], magic));
    }
    SONAR_TILE_LANDED();
  };
  // operand lane (kb, col16) of row block rb, k block b: piece 4 b + kb of row col16
  auto a_address = [&](int slot, int b) {
    return a_lds + slot * kStageA + (8 * wm * 2 + (col16 >> 3)) * kBlockBytes + (col16 & 7) * 128 +
           (((4 * b + kb) ^ (col16 & 7)) * 16);
  };
  // Multiply phase: 32 MFMAs, ahead of the other wavefront's VALU work in the
  // issue order; behind the four of a row block, the read of that row block's
  // operand of half step (slot, b), which the next multiply phase uses: the
  // reads of A cost the fetch phases nothing.
  auto multiply_and_read = [&](int slot, int b) {
    const uint32_t a_at = a_address(slot, b);
    __builtin_amdgcn_s_setprio(2);
#define SONAR_TILE_ROW(i, off)                                                                          \
  _Pragma("unroll") for (int j = 0; j < 4; ++j) acc[j][i] =                                             \
      Dq<T>::mfma(__builtin_bit_cast(vec8, wv[j]), __builtin_bit_cast(vec8, av[i]), acc[j][i]);         \
  SONAR_TILE_READ(av[i], a_at, off)
    SONAR_TILE_ROW(0, 0);
    SONAR_TILE_ROW(1, 2048);
    SONAR_TILE_ROW(2, 4096);
    SONAR_TILE_ROW(3, 6144);
    SONAR_TILE_ROW(4, 8192);
    SONAR_TILE_ROW(5, 10240);
    SONAR_TILE_ROW(6, 12288);
    SONAR_TILE_ROW(7, 14336);
#undef SONAR_TILE_ROW
    __builtin_amdgcn_s_setprio(0);
  };
  // end of a phase; nothing may be scheduled across it
  auto phase_end = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  // The loop body has no branches: a wavefront past the last strip of the
  // matrix works on a second copy of the last strip (its results are dropped),
  // and the copies for steps past the end fetch the last step again, into a
  // slot nobody reads any more.  So seven copies are outstanding at every wait.
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kAsyncCopies) : "memory");  // stage k_first has landed
  // a shared ring: the blocks of k block 0 are the copies of the strip's wavefront of group 0,
  // which the wavefront of group 1 may read only behind a barrier that follows that wait
  if constexpr (W8 != 0) phase_end();
  raw_start(0, 0, true);
  phase_end();
  {
    const uint32_t a_at = a_address(0, 0);
    SONAR_TILE_READ(av[0], a_at, 0);
    SONAR_TILE_READ(av[1], a_at, 2048);
    SONAR_TILE_READ(av[2], a_at, 4096);
    SONAR_TILE_READ(av[3], a_at, 6144);
    SONAR_TILE_READ(av[4], a_at, 8192);
    SONAR_TILE_READ(av[5], a_at, 10240);
    SONAR_TILE_READ(av[6], a_at, 12288);
    SONAR_TILE_READ(av[7], a_at, 14336);
  }
  if (wm == 1) phase_end();  // group 1 runs one phase behind

  int slot = 0;        // stage of step kt
  int fill = 2;        // stage step kt + 2 goes to
  for (int kt = k_first; kt < k_tiles; ++kt) {
    const int next_slot = slot == kAsyncStages - 1 ? 0 : slot + 1;
    // ---- half step (kt, 0)
    // the copies of stage kt + 2 go out in the fetch phases, four and three: a
    // wavefront waits at a copy while the memory pipeline is busy, which would
    // starve the matrix cores if it happened between MFMAs
    const int copy_kt = min(kt + 2, k_tiles - 1);
#pragma unroll
    for (int idx = 0; idx < 4; ++idx) issue_one(copy_kt, fill, idx);
    fetch(slot, 0, true);
    raw_start(slot, 1, G32);
    phase_end();
    multiply_and_read(slot, 1);
    phase_end();
    // ---- half step (kt, 1)
#pragma unroll
    for (int idx = 4; idx < kAsyncCopies; ++idx) issue_one(copy_kt, fill, idx);
    fetch(slot, 1, G32);
    // stage kt + 1 has landed once nothing but the copies of stage kt + 2 is outstanding
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kAsyncCopies) : "memory");
    raw_start(next_slot, 0, true);
    phase_end();
    // the rows of stage kt + 1 this group reads are the ones it copied, and its four
    // wavefronts have waited for their copies before the barrier above
    multiply_and_read(next_slot, 0);
    phase_end();
    slot = next_slot;
    fill = fill == kAsyncStages - 1 ? 0 : fill + 1;
  }
  if (wm == 0) phase_end();  // the barrier that ends group 1's last phase
  // the last copies and the last read started by raw_start must not outlive the wavefront
  if constexpr (W8 != 0) {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)"
                 : "+v"(qraw), "+v"(qhigh), "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw)::"memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : "+v"(qraw), "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw)::"memory");
  }
  SONAR_TILE_LANDED();   // the operand reads started by the last multiply phase
#undef SONAR_TILE_LANDED
#undef SONAR_TILE_READ

  if (!active) return;
  if (!GROUPED && !whole_k) {
    // partial tile of this K range: one 1-KiB block per accumulator tile
    const int first_split = whole_tiles(p);
    const int split_tiles = p.tiles_m * p.tiles_n - first_split;
    float4* dst = p.partial + ((size_t)(split * split_tiles + tile - first_split) * 256 + wave * 32) * 64 + lane;
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int mb = 0; mb < 8; ++mb) {
        const floatx4_t v = acc[nb][mb];
        dst[(nb * 8 + mb) * 64] = make_float4(v.x, v.y, v.z, v.w);
      }
    return;
  }
  // rows of C this lane writes: one per row block
  long c_row[8];
  float row_w[8];
#pragma unroll
  for (int mb = 0; mb < 8; ++mb) {
    const int r = 128 * wm + 16 * mb + col16;
    c_row[mb] = -1;
    row_w[mb] = 1.f;
    if (GROUPED) {
      const int id = r < tile_rows ? p.sorted_ids[first_slot + r] : p.rows_total;
      if ((unsigned)id < (unsigned)p.rows_total) {
        c_row[mb] = id;
        // the routing weight is rounded to the activation type and the product is
        // formed and rounded in that type (marlin_template.h(moe):1893-1897)
        if (p.mul_topk) row_w[mb] = Dq<T>::to_float(Dq<T>::from_float(p.topk_weights[id]));
      }
    } else if (m0 + r < p.size_m) {
      c_row[mb] = m0 + r;
    }
  }
  const uint16_t* bias_src = p.bias ? p.bias + expert * p.expert_bias_stride + strip * kStripN : nullptr;
  float gs = 1.f;   // NVFP4: the global scale multiplies the sum before anything else (marlin_template.h:1661-1665)
  if (NV && p.global_scale) gs = p.global_scale[GROUPED ? expert : 0];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int n = strip * kStripN + 16 * nb + 4 * kb;
    float bias[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias_src) {
#pragma unroll
      for (int r = 0; r < 4; ++r) bias[r] = Dq<T>::to_float(bias_src[scale_slot(16 * nb + 4 * kb + r, false)]);
    }
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) {
      if (c_row[mb] < 0) continue;
      const floatx4_t v = NV ? acc[nb][mb] * gs : acc[nb][mb];
      uint16_t o[4] = {Dq<T>::from_float(v.x + bias[0]), Dq<T>::from_float(v.y + bias[1]),
                       Dq<T>::from_float(v.z + bias[2]), Dq<T>::from_float(v.w + bias[3])};
      if (GROUPED && p.mul_topk) {
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = Dq<T>::from_float(Dq<T>::to_float(o[r]) * row_w[mb]);
      }
      uint2 packed;
      packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
      packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
      *reinterpret_cast<uint2*>(p.c + c_row[mb] * p.size_n + n) = packed;
    }
  }
}

// ---------------------------------------------------------------------------
// The wide form of the asynchronous tile kernel: the same 256 x 256 tile and K
// step, four wavefronts instead of eight, one per SIMD with the whole register
// file (256 accumulator registers for 256 rows x 64 columns: a strip over all
// rows of the tile).  A chunk of weights is dequantised once per workgroup
// instead of once per group of rows and feeds 64 MFMAs; with no second
// wavefront on the SIMD the other work (dequantising the next chunk, the LDS
// reads of A four row blocks ahead, the copies of a later stage) sits between
// the MFMAs of the wavefront's own instruction stream, one to two instructions
// behind each MFMA, where the matrix pipeline hides them.
//   * A: a ring of four 32-KiB stages filled by LDS-DMA, wavefront w copying
//     row blocks 4w..4w+3 (eight 1-KiB regions, the layout of the kernel above).
//   * W: the two chunks of a step go from memory straight into registers (one
//     16-byte load per lane and chunk), a ring of four register sets.
//   * scales / zero points: one 256-byte row per step through a private LDS
//     ring of sixteen rows, fetched a step earlier than the rest.
// The eleven memory operations a wavefront issues per step (8 + 1 + 2: stage
// kt + 3 of A and W, the scale row of step kt + 4) go out in the second half of
// step kt.  One barrier per step, between its halves: before it a wavefront
// waits until only the eleven youngest operations are outstanding, so behind it
// stage kt + 1 has landed for everyone and the slot of stage kt - 1 is free.
// The MFMAs are written as asm statements with the accumulator as a tied
// operand: 224 accumulator registers in AGPRs, 32 in VGPRs, every one updated in
// place (left to the register allocator, the 256 accumulators of this loop get
// copied between registers all the time).  The compiler therefore does not see
// MFMAs here and pads no matrix-core hazard: none arises inside the loop (an
// accumulator is touched again 64 MFMAs later, operands are written long before
// they are read), and the results are read after the pipeline has drained
// (s_nop below).
// 4-bit or symmetric 8-bit codes with groups of 64 * 2^i rows or one group, MXFP4 (float4_e2m1f codes,
// bf16, a scale per 32 rows: one hardware conversion and half a byte permute behind each row
// block), integer / 8-bit floating-point codes with a scale per 32 rows (MXFP8 among them), or NVFP4
// (float4_e2m1f codes with a scale per 16 rows and a global scale, either activation type); no
// act-order; dense and grouped (mixture-of-experts) calls.  K ranges that are not a
// multiple of four steps are padded with steps of zeros (integer codes; taken only where that
// is a small part of the range).
constexpr int kWideStages = 4;
constexpr int kWideScaleRows = 16;   // a ring of 16 rows per wavefront: eight steps of one row, or of two (groups of 32 rows)
// RB: row blocks of 16 rows a wavefront owns: 16 (a 256-row tile) or 8 (a 128-row tile, for
// calls with few tiles: twice the tiles, half the K ranges and half the partial-tile traffic).
constexpr int wide_stage(int rb) { return rb * 2 * kBlockBytes; }                    // one stage of A
constexpr int wide_a(int rb) { return kWideStages * wide_stage(rb); }                // 128 / 64 KiB
constexpr int wide_lds(int rb) { return wide_a(rb) + 4 * kWideScaleRows * 256; }     // + the scale rows of four wavefronts
// memory operations per wavefront and step: its blocks of A, the scale row (groups of 32 / 16 rows: two, one per
// k block), two chunks (8-bit codes: four blocks)
constexpr int wide_ops(int rb, bool fp4 = false, bool w8 = false) { return rb / 2 + (fp4 ? 2 : 1) + (w8 ? 4 : 2); }

// One 128-byte line of zeros: what the copies of A fetch for the steps past the end of a K range that
// is not a multiple of four steps (the loop always runs whole passes of four; those steps then add
// zeros times the last step's weights).
__device__ __attribute__((aligned(128))) const uint32_t kWideZeroLine[32] = {};

// G32: a scale (and zero point) per 32 rows, i.e. one row of them per k block: MXFP4 always, integer codes when asked.
// NV (with FP4): NVFP4, a scale per 16 rows: the row of a k block then holds two groups of 128 bytes (the copy
// fetches one per half of the wavefront), and a lane, whose eight rows of a k block lie in one group, reads group
// kb / 2; the global scale multiplies the sums at the end.
template <typename T, bool HAS_ZP, bool GROUPED = false, int RB = 16, bool FP4 = false, int W8 = 0, bool G32 = FP4,
          bool NV = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void marlin_tile_wide_kernel(
    const TileParams p) {
  typedef typename Dq<T>::vec8 vec8;
  typedef typename Dq4Of<T, FP4, NV>::type D4;   // integer codes, or float4_e2m1f (MXFP4: bf16; NVFP4)
  typedef typename Dq8Of<T, W8 == 2>::type D8;   // 8-bit integer (W8 = 1) or floating-point (W8 = 2) codes
  typedef typename std::conditional<W8 != 0, typename D8::Col, typename D4::Col>::type Col;
  typedef typename Dq<T>::Mid Mid;
  static_assert(W8 == 0 || (!HAS_ZP && !FP4), "8-bit codes: symmetric");
  static_assert(wide_ops(RB, G32, W8 != 0) <= 2 * RB, "a step's memory operations go out behind its row blocks");
  static_assert(!FP4 || G32, "MXFP4 has a scale per 32 rows");
  constexpr int kChunkLoads = W8 ? 2 : 1;   // 16-byte loads per lane and k block: 8-bit codes come as a block of
                                            // the low four and a block of the high four of a lane's eight rows
  static_assert(!FP4 || ((NV || std::is_same<T, __bf16>::value) && !HAS_ZP), "MXFP4: bf16; float4 codes: no zero points");
  static_assert(!NV || (FP4 && RB == 16), "NVFP4 is float4 codes; 256-row tiles");
  static_assert(!(W8 != 0 && G32) || RB == 16, "8-bit codes with groups of 32 rows: 256-row tiles");
  static_assert(RB == 16 || RB == 8, "256-row tiles or 128-row tiles");
  constexpr int kRows = 16 * RB;
  constexpr int kStage = wide_stage(RB), kWideA = wide_a(RB), kWideOps = wide_ops(RB, G32, W8 != 0);
  constexpr int kAgprBlocks = RB == 16 ? 14 : RB;   // row blocks whose accumulators sit in AGPRs
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col16 = lane & 15;
  const int kb = lane >> 4;
  const uint32_t magic = magic_register();
  const bool grouped = p.num_groups > 1;

  int tile, tile_m, tile_n, split;
  bool whole_k;
  int steps_per_split = p.k_steps_per_split;
  int partial_at;   // without whole_k: index of this workgroup's partial tile, (split, split tile)
  if (GROUPED) {
    // The launch is sized for the most row tiles the routing could make; the tiles there are
    // (tile_table[0]) are numbered here in bands of four row tiles, so that the 32 workgroups an
    // XCD holds share 4 panels of A and 8 panels of W (of one expert where the routing is even),
    // and every XCD gets its share of them.
    // With room for partial tiles the K split is planned here too (plan_live_split).
    const TileParams live = live_tiles(p);
    if (live.tiles_m <= 0 || !tile_of_workgroup(live, tile, split, whole_k)) return;
    tile_coords(live, tile, tile_m, tile_n);
    steps_per_split = live.k_steps_per_split;
    const int first_split = whole_tiles(live);
    partial_at = split * (live.tiles_m * live.tiles_n - first_split) + tile - first_split;
  } else {
    if (!tile_of_workgroup(p, tile, split, whole_k)) return;
    tile_coords(p, tile, tile_m, tile_n);
    const int first_split = whole_tiles(p);
    partial_at = split * (p.tiles_m * p.tiles_n - first_split) + tile - first_split;
  }
  // Grouped calls: row tile t is up to four consecutive 64-slot blocks of one expert, listed in
  // tile_table; rows are slots of sorted_ids (as in marlin_tile_async_kernel).
  int first_slot = 0, tile_rows = kRows;
  long expert = 0;
  if (GROUPED) {
    if (tile_m >= p.tile_table[0]) return;
    first_slot = p.tile_table[1 + 3 * tile_m] * 64;
    tile_rows = p.tile_table[2 + 3 * tile_m] * 64;
    expert = p.tile_table[3 + 3 * tile_m];
  }
  const int m0 = tile_m * kRows;
  const int strip0 = tile_n * (kTileN / kStripN);
  const int strips_here = min(kTileN / kStripN, p.size_n / kStripN - strip0);
  const bool active = wave < strips_here;
  // a wavefront past the last strip works on the last strip again and stores nothing
  const int strip = strip0 + (active ? wave : strips_here - 1);

  // ---- sources (regions of A as in marlin_tile_async_kernel; wavefront w fills RB / 2 regions)
  const char* a_src[RB / 2];
#pragma unroll
  for (int i = 0; i < RB / 2; ++i) {
    const int region = (RB / 2) * wave + i;
    const int r8 = lane >> 3;
    const int in_tile = 16 * (region >> 1) + 8 * (region & 1) + r8;
    int row;
    if (GROUPED) {
      const int id = in_tile < tile_rows ? p.sorted_ids[first_slot + in_tile] : p.rows_total;
      // padding slots read row 0, never stored
      row = (unsigned)id < (unsigned)p.rows_total ? (p.a_by_slot ? first_slot + in_tile : id / p.top_k) : 0;
    } else {
      row = m0 + in_tile;
      if (row >= p.size_m) row = p.size_m - 1;   // rows past M are computed and never stored
    }
    a_src[i] = reinterpret_cast<const char*>(p.a) + ((long)row * p.lda + 8 * ((lane & 7) ^ r8)) * 2;
  }
  const uint4* b_src = p.b + expert * p.expert_b_stride +
                       (size_t)(unsigned)(strip * p.chunks_per_strip) * (64 * kChunkLoads) + lane;
  const char* s_src;
  long s_group_stride;
  if (HAS_ZP && lane >= 32) {
    s_src = reinterpret_cast<const char*>(p.zeros + expert * p.expert_z_stride + strip * 8 + (lane & 7));
    s_group_stride = (long)(p.size_n / 8) * 4;
  } else {
    s_src = reinterpret_cast<const char*>(p.scales + expert * p.expert_s_stride + strip * kStripN) + 4 * (lane & 31);
    s_group_stride = (long)p.size_n * 2;
    if (NV) s_src += (lane >> 5) * s_group_stride;   // the upper half of the wavefront fetches the next group's row
  }
  // steps per group as a shift (the host checks: group_size = 64 * 2^i)
  const int group_shift = grouped ? 31 - __builtin_clz(p.group_size / kTileK) : 0;
  char* sring = smem + kWideA + wave * (kWideScaleRows * 256);
  const uint32_t a_lds = (uint32_t)(uintptr_t)(lds_void_t*)smem;
  const uint32_t s_lds = (uint32_t)(uintptr_t)(lds_void_t*)sring;

  // K steps [k_first, k_tiles) of this workgroup
  const int k_first = whole_k ? 0 : split * steps_per_split;
  const int k_tiles = whole_k ? p.size_k / kTileK : min(p.size_k / kTileK, k_first + steps_per_split);

  u32x4_t wq[kWideStages][2 * kChunkLoads];   // packed chunks in flight or waiting (8-bit: [2 b + h], h = high rows)
  // the scale row of step kt (clamped to the last step) into its ring position; MXFP4: the row of
  // k block h of the step (groups of 32 rows), ring position 2 (kt - k_first) + h
  auto issue_scales = [&](int kt, int h) __attribute__((always_inline)) {
    const int k = min(kt, k_tiles - 1);
    const int grp = G32 ? (NV ? 2 : 1) * (2 * k + h) : (grouped ? k >> group_shift : 0);
    const int at = G32 ? 2 * (kt - k_first) + h : kt - k_first;
    __builtin_amdgcn_global_load_lds((glb_void_t*)(s_src + (long)grp * s_group_stride),
                                     (lds_void_t*)(sring + (at & (kWideScaleRows - 1)) * 256), 4, 0, 0);
  };
  // memory operation `idx` (0..kWideOps-1) issued for step kt into ring position `slot`: first the
  // blocks of A of step kt, then the scale row of step kt + 1, then the two chunks of step kt
  auto issue_one = [&](int kt, int slot, int idx) __attribute__((always_inline)) {
    const int k = min(kt, k_tiles - 1);
    if (idx < RB / 2) {
      // (the comparison is uniform: a pair of selects per copy)
      const char* src = kt < k_tiles ? a_src[idx] + (long)k * (kTileK * 2)
                                     : reinterpret_cast<const char*>(kWideZeroLine) + 16 * (lane & 7);
      __builtin_amdgcn_global_load_lds((glb_void_t*)src,
                                       (lds_void_t*)(smem + slot * kStage + ((RB / 2) * wave + idx) * kBlockBytes),
                                       16, 0, 0);
    } else if (idx < RB / 2 + (G32 ? 2 : 1)) {
      issue_scales(kt + 1, idx - RB / 2);
    } else {
      const int c = idx - RB / 2 - (G32 ? 2 : 1);
      const uint4* g = b_src + (size_t)(2 * kChunkLoads * k + c) * 64;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(wq[slot][c]) : "v"(g) : "memory");
    }
  };

  uint32_t s_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) s_off[j] = 2 * scale_slot(16 * j + col16, grouped);
  const uint32_t z_off = 128 + 4 * zero_point_word(col16);
  // operand lane (kb, col16) of row block 0, k block b of stage 0: piece 4 b + kb of row col16
  uint32_t a_base[2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
    a_base[b] = a_lds + (col16 >> 3) * kBlockBytes + (col16 & 7) * 128 + (((4 * b + kb) ^ (col16 & 7)) * 16);

  floatx4_t acc[4][RB];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int mb = 0; mb < RB; ++mb) {
      acc[nb][mb] = floatx4_t{0.f, 0.f, 0.f, 0.f};
      // the zeros sit where the MFMAs will hold the accumulator, so that the value has one home
      // on every path to the stores
      if (mb < kAgprBlocks) asm volatile("" : "+a"(acc[nb][mb]));
      else asm volatile("" : "+v"(acc[nb][mb]));
    }

  constexpr int kAhead = 4;   // operands of A are read this many row blocks ahead
  u32x4_t av[8];          // row block rb in av[rb & 7]
  uint32_t wb[2][4][4];   // dequantised chunk of k block b: four operand blocks of 16 columns, four pairs each
  uint32_t sb0 = 0, sb1 = 0, sb2 = 0, sb3 = 0, zw = 0;
  Col cols[2][4];         // by the parity of the step (MXFP4: of the k block)

#define SONAR_WIDE_READ(dst, base, off) \
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst) : "v"(base), "i"(off) : "memory")
#define SONAR_WIDE_LANDED(n, reg) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(reg) : "n"(n) : "memory")

  auto scales_start = [&](int kt, int h) __attribute__((always_inline)) {
    const uint32_t r_at = s_lds + ((G32 ? 2 * (kt - k_first) + h : kt - k_first) & (kWideScaleRows - 1)) * 256 +
                          (NV ? 128 * (kb >> 1) : 0);
    asm volatile(
        "ds_read_u16 %0, %5\n\t"
        "ds_read_u16 %1, %6\n\t"
        "ds_read_u16 %2, %7\n\t"
        "ds_read_u16 %3, %8\n\t"
        "ds_read_b32 %4, %9"
        : "=&v"(sb0), "=&v"(sb1), "=&v"(sb2), "=&v"(sb3), "=&v"(zw)
        : "v"(r_at + s_off[0]), "v"(r_at + s_off[1]), "v"(r_at + s_off[2]), "v"(r_at + s_off[3]),
          "v"(NV ? r_at + s_off[0] : r_at + z_off)
        : "memory");
  };
  auto make_col = [&](int set, int j) __attribute__((always_inline)) {
    const uint32_t sbits = j == 0 ? sb0 : j == 1 ? sb1 : j == 2 ? sb2 : sb3;
    int z = 8;
    if (HAS_ZP) z = (int)((zw >> zero_point_shift(16 * j + col16)) & 0xFu);
    if constexpr (W8 != 0) cols[set][j] = D8::make_col((uint16_t)sbits);
    else cols[set][j] = D4::make_col((uint16_t)sbits, z);
  };
  auto word_of = [](const u32x4_t& q, int j) __attribute__((always_inline)) -> uint32_t {
    return j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w;
  };
  // acc[j][rb] += W block j (16 columns) x A row block rb, in place; with 16 row blocks the last two in VGPRs
  auto mfma = [&](int B, int j, int rb) __attribute__((always_inline)) {
    const u32x4_t w = u32x4_t{wb[B][j][0], wb[B][j][1], wb[B][j][2], wb[B][j][3]};
    if constexpr (std::is_same<T, _Float16>::value) {
      if (rb < kAgprBlocks) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[j][rb]) : "v"(w), "v"(av[rb & 7]));
      else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[j][rb]) : "v"(w), "v"(av[rb & 7]));
    } else {
      if (rb < kAgprBlocks) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[j][rb]) : "v"(w), "v"(av[rb & 7]));
      else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[j][rb]) : "v"(w), "v"(av[rb & 7]));
    }
  };

  // One k block of step kt: RB row blocks of four MFMAs.  R: ring position of the step's
  // stage, B: the k block.  Behind the MFMAs of a row block, one instruction each: one pair
  // (with 8 row blocks: two) of the 16 of the next half step's chunk; then B = 0: the scales of
  // step kt + 1 become per-column constants; B = 1: one memory operation of step kt + 3.
  auto chunk = [&](const int R, const int B, const int kt) __attribute__((always_inline)) {
    const int NR = B ? (R + 1) & 3 : R;   // stage and k block of the half step after this one
    const int NB = B ^ 1;
    // constants of the step the next half step belongs to (MXFP4: of the next k block)
    const int set = G32 ? NB : (B ? (R + 1) & 1 : R & 1);
    const uint32_t a_cur = a_base[B] + R * kStage;
    const uint32_t a_next = a_base[NB] + NR * kStage;
    const u32x4_t& q4 = B ? wq[NR][0] : wq[R][kChunkLoads];                         // 8-bit: the low four rows
    const u32x4_t& q4h = B ? wq[NR][kChunkLoads - 1] : wq[R][2 * kChunkLoads - 1];   // 8-bit: the high four rows
    constexpr int kPairs = 16 / RB;   // pairs of weights dequantised per row block
    uint32_t r_lo = 0;     // MXFP4: rows (0, 2) or (4, 6) of the word in hand, waiting for their odd partners
    uint32_t nv_lo = 0, nv_hi = 0;   // NVFP4, bf16: the same rows as fp32 products
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int j = (kPairs * rb) >> 2, part = (kPairs * rb) & 3;
      // reads started after the one of this row block: those of the next kAhead - 1 row blocks,
      // and the five scale reads of slot 0 (first half; MXFP4: either half)
      if ((B == 0 || G32) && rb >= 1 && rb <= kAhead) SONAR_WIDE_LANDED(kAhead - 1 + 5, av[rb & 7]);
      else SONAR_WIDE_LANDED(kAhead - 1, av[rb & 7]);
      // behind this wait the scale reads of slot 0 have landed: from here on the registers they fill
      // hold the scales (without this the compiler is free to use them any time after slot 0)
      if ((B == 0 || G32) && rb == (kAhead + 1 < RB ? kAhead + 1 : RB - 1))
        asm volatile("" : "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw) : : "memory");
      if (rb + kAhead < RB) SONAR_WIDE_READ(av[(rb + kAhead) & 7], a_cur, (rb + kAhead) * 2048);
      else SONAR_WIDE_READ(av[(rb + kAhead) & 7], a_next, (rb + kAhead - RB) * 2048);
      // the scales of the step after this one (MXFP4: of its k block B, two half steps ahead)
      if (rb == 0 && (B == 0 || G32)) scales_start(kt + 1, B);
      const uint32_t qw = word_of(q4, j);
      if constexpr (W8 != 0) {
        // behind every second row block, half a column block (four rows of 16 columns) in one piece
        mfma(B, 0, rb);
        if (RB == 8 || (rb & 1) == 0) {   // (with 8 row blocks: behind every row block)
          const int piece = RB == 8 ? rb : rb >> 1;
          const int jj = piece >> 1, half = piece & 1;
          const uint2 w = D8::word4(word_of(half ? q4h : q4, jj), cols[set][jj], magic);
          wb[NB][jj][2 * half] = w.x;
          wb[NB][jj][2 * half + 1] = w.y;
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 1, rb);
        mfma(B, 2, rb);
        mfma(B, 3, rb);
      } else if constexpr (NV && std::is_same<T, _Float16>::value) {
        // the pair of codes read as fp16 numbers (value * 2^-14) times scale * 2^14 in one packed multiply
        // (DqNvF4<_Float16>::pair, a piece behind each MFMA)
        mfma(B, 0, rb);
        const uint32_t y = part == 3 ? qw : qw << (12 - 4 * part);
        const uint32_t mag = (y >> 3) & 0x0E000E00u;
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 1, rb);
        const uint32_t hbits = (y & 0x80008000u) | mag;
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 2, rb);
        wb[NB][j][part] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, hbits) *
                                                           __builtin_bit_cast(half2_t, cols[set][j].s2));
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 3, rb);
      } else if constexpr (FP4 && kPairs == 2) {
        // MXFP4 with 8 row blocks: the conversions of an even and an odd part (rows (0,2) and (1,3), or (4,6) and
        // (5,7)) and their two byte permutes behind one row block
        mfma(B, 0, rb);
        const float sc = cols[set][j].s;
        const uint32_t r_e = __builtin_bit_cast(uint32_t, part == 0 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 0)
                                                                    : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 1));
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 1, rb);
        const uint32_t r_o = __builtin_bit_cast(uint32_t, part == 0 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 2)
                                                                    : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 3));
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 2, rb);
        wb[NB][j][part] = __builtin_amdgcn_perm(r_o, r_e, 0x05040100u);
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 3, rb);
        wb[NB][j][part + 1] = __builtin_amdgcn_perm(r_o, r_e, 0x07060302u);
      } else if constexpr (NV) {
        // bf16: one hardware conversion with a unit scale per row block (rows (0,2), (1,3), (4,6), (5,7) of the
        // column), the two values times the scale in fp32; behind the second and the fourth, the two byte
        // permutes that cut the products back to bf16 and put four rows in order (DqNvF4<__bf16>::word)
        mfma(B, 0, rb);
        const float sc = cols[set][j].s;
        const uint32_t r = __builtin_bit_cast(
            uint32_t, part == 0   ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, 1.0f, 0)
                      : part == 1 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, 1.0f, 2)
                      : part == 2 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, 1.0f, 1)
                                  : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, 1.0f, 3));
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 1, rb);
        const float f_lo = __uint_as_float(r << 16), f_hi = __uint_as_float(r & 0xFFFF0000u);
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 2, rb);
        const uint32_t p_lo = __float_as_uint(f_lo * sc), p_hi = __float_as_uint(f_hi * sc);
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 3, rb);
        if (part & 1) {
          wb[NB][j][part - 1] = __builtin_amdgcn_perm(p_lo, nv_lo, 0x07060302u);
          wb[NB][j][part] = __builtin_amdgcn_perm(p_hi, nv_hi, 0x07060302u);
        } else {
          nv_lo = p_lo;
          nv_hi = p_hi;
        }
      } else if constexpr (FP4) {
        // one hardware conversion per row block (two rows of the column each: (0,2), (1,3), (4,6),
        // (5,7)); behind the second and the fourth, the two byte permutes that put four rows in order
        mfma(B, 0, rb);
        const float sc = cols[set][j].s;
        const uint32_t r = __builtin_bit_cast(
            uint32_t, part == 0   ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 0)
                      : part == 1 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 2)
                      : part == 2 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 1)
                                  : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(qw, sc, 3));
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 1, rb);
        if (part & 1) wb[NB][j][part - 1] = __builtin_amdgcn_perm(r, r_lo, 0x05040100u);
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 2, rb);
        if (part & 1) wb[NB][j][part] = __builtin_amdgcn_perm(r, r_lo, 0x07060302u);
        else r_lo = r;
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 3, rb);
      } else {
        mfma(B, 0, rb);
        const uint32_t x = Dq<T>::stage1(part < 2 ? qw : qw >> 8, part, magic);
        uint32_t x2 = 0;
        if (kPairs == 2) x2 = Dq<T>::stage1(part < 2 ? qw : qw >> 8, part + 1, magic);
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 1, rb);
        const Mid y = Dq<T>::stage2(x, cols[set][j], part);
        Mid y2 = y;
        if (kPairs == 2) y2 = Dq<T>::stage2(x2, cols[set][j], part + 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 2, rb);
        wb[NB][j][part] = Dq<T>::stage3(y, cols[set][j]);
        if (kPairs == 2) wb[NB][j][part + 1] = Dq<T>::stage3(y2, cols[set][j]);
        __builtin_amdgcn_sched_barrier(0);
        mfma(B, 3, rb);
      }
      if (B == 0 || G32) {
        // the scale reads of slot 0 have landed behind the wait of slot kAhead + 1; they become the
        // constants of the step after this one (MXFP4: of its k block B, whose set the chunk being
        // dequantised here does not use)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (rb == (kAhead + 1 + c < RB ? kAhead + 1 + c : RB - 1)) make_col(G32 ? B : (R + 1) & 1, c);
      }
      if (B == 1 && rb < kWideOps) issue_one(kt + 3, (R + 3) & 3, rb);
      // (8-bit codes with 8 row blocks: nine operations, the ninth behind the first row block too)
      if (B == 1 && RB + rb < kWideOps) issue_one(kt + 3, (R + 3) & 3, RB + rb);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto step = [&](const int R, int kt) __attribute__((always_inline)) {
    chunk(R, 0, kt);
    // stage kt + 1 (its blocks of A, its two chunks) and the scale row of step kt + 2 have landed
    // once only the operations issued in step kt - 1 are outstanding
    asm volatile("s_waitcnt vmcnt(%2)"
                 : "+v"(wq[(R + 1) & 3][0]), "+v"(wq[(R + 1) & 3][1])
                 : "n"(kWideOps)
                 : "memory");
    if constexpr (W8 != 0) asm volatile("" : "+v"(wq[(R + 1) & 3][2]), "+v"(wq[(R + 1) & 3][3]) : : "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    chunk(R, 1, kt);
  };

  // ---- prologue: the scale row of the first step, then what steps k_first - 3 .. k_first - 1 would have issued
  issue_scales(k_first, 0);
  if (G32) issue_scales(k_first, 1);
#pragma unroll
  for (int idx = 0; idx < kWideOps; ++idx) issue_one(k_first, 0, idx);
#pragma unroll
  for (int idx = 0; idx < kWideOps; ++idx) issue_one(k_first + 1, 1, idx);
#pragma unroll
  for (int idx = 0; idx < kWideOps; ++idx) issue_one(k_first + 2, 2, idx);
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(wq[0][0]), "+v"(wq[0][1]) : "n"(2 * kWideOps) : "memory");
  if constexpr (W8 != 0) asm volatile("" : "+v"(wq[0][2]), "+v"(wq[0][3]) : : "memory");
  __builtin_amdgcn_s_barrier();
  if (G32) {   // the constants of k block 1 of the first step; those of k block 0 below
    scales_start(k_first, 1);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw) : : "memory");
#pragma unroll
    for (int j = 0; j < 4; ++j) make_col(1, j);
  }
  scales_start(k_first, 0);
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw) : : "memory");
#pragma unroll
  for (int j = 0; j < 4; ++j) make_col(0, j);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    u32x4_t w;
    if constexpr (W8 != 0) {
      const uint2 lo = D8::word4(word_of(wq[0][0], j), cols[0][j], magic);
      const uint2 hi = D8::word4(word_of(wq[0][1], j), cols[0][j], magic);
      w = u32x4_t{lo.x, lo.y, hi.x, hi.y};
    } else {
      w = __builtin_bit_cast(u32x4_t, D4::word(word_of(wq[0][0], j), cols[0][j], magic));
    }
    wb[0][j][0] = w.x;
    wb[0][j][1] = w.y;
    wb[0][j][2] = w.z;
    wb[0][j][3] = w.w;
  }
#pragma unroll
  for (int rb = 0; rb < kAhead; ++rb) SONAR_WIDE_READ(av[rb], a_base[0], rb * 2048);
  __builtin_amdgcn_sched_barrier(0);

  // whole passes of four steps (the ring positions are static); steps past the end of the range
  // multiply zeros
  for (int kt = k_first; kt < k_tiles; kt += 4) {
    step(0, kt);
    step(1, kt + 1);
    step(2, kt + 2);
    step(3, kt + 3);
  }
  // nothing in flight may outlive the wavefront (the copies of the steps past the end, the two
  // operand reads of the last half step), and the matrix pipeline drains before the results are read
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // the registers those operations were still to fill stay untouched up to here
#pragma unroll
  for (int i = 0; i < kWideStages; ++i)
#pragma unroll
    for (int c = 0; c < 2 * kChunkLoads; ++c) asm volatile("" : "+v"(wq[i][c]) : : "memory");
#pragma unroll
  for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(av[i]) : : "memory");
  asm volatile("" : "+v"(sb0), "+v"(sb1), "+v"(sb2), "+v"(sb3), "+v"(zw) : : "memory");
  __builtin_amdgcn_sched_barrier(0);
#undef SONAR_WIDE_LANDED
#undef SONAR_WIDE_READ

  if (!active) return;
  if (!whole_k) {
    // partial tile of this K range, in the order tile_reduce_kernel reads: 1-KiB blocks
    // (half of the rows, strip, column block, row block)
    float4* dst = p.partial + ((size_t)partial_at * kRows + wave * 32) * 64 + lane;
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int mb = 0; mb < RB; ++mb) {
        if (mb < kAgprBlocks) asm volatile("" : "+a"(acc[nb][mb]));   // still in its AGPRs here
        const floatx4_t v = acc[nb][mb];
        dst[((mb >> 3) * 128 + nb * 8 + (mb & 7)) * 64] = make_float4(v.x, v.y, v.z, v.w);
        __builtin_amdgcn_sched_barrier(0);   // one accumulator at a time leaves the AGPRs
      }
    return;
  }
  const uint16_t* bias_src = p.bias ? p.bias + expert * p.expert_bias_stride + strip * kStripN : nullptr;
  float gs = 1.f;   // NVFP4: the global scale multiplies the sum before anything else (marlin_template.h:1661-1665)
  if (NV && p.global_scale) gs = p.global_scale[GROUPED ? expert : 0];
  float bias[4][4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      bias[nb][r] = bias_src ? Dq<T>::to_float(bias_src[scale_slot(16 * nb + 4 * kb + r, false)]) : 0.f;
#pragma unroll
  for (int mb = 0; mb < RB; ++mb) {
    // the row of C this lane writes for this row block
    const int r = 16 * mb + col16;
    long c_row = -1;
    float row_w = 1.f;
    if (GROUPED) {
      const int id = r < tile_rows ? p.sorted_ids[first_slot + r] : p.rows_total;
      if ((unsigned)id < (unsigned)p.rows_total) {
        c_row = id;
        // the routing weight is rounded to the activation type and the product is
        // formed and rounded in that type (marlin_template.h(moe):1893-1897)
        if (p.mul_topk) row_w = Dq<T>::to_float(Dq<T>::from_float(p.topk_weights[id]));
      }
    } else if (m0 + r < p.size_m) {
      c_row = m0 + r;
    }
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      if (mb < kAgprBlocks) asm volatile("" : "+a"(acc[nb][mb]));   // still in its AGPRs here
      if (c_row >= 0) {
        const floatx4_t v = NV ? acc[nb][mb] * gs : acc[nb][mb];
        uint16_t o[4] = {Dq<T>::from_float(v.x + bias[nb][0]), Dq<T>::from_float(v.y + bias[nb][1]),
                         Dq<T>::from_float(v.z + bias[nb][2]), Dq<T>::from_float(v.w + bias[nb][3])};
        if (GROUPED && p.mul_topk) {
#pragma unroll
          for (int i = 0; i < 4; ++i) o[i] = Dq<T>::from_float(Dq<T>::to_float(o[i]) * row_w);
        }
        uint2 packed;
        packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
        packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
        *reinterpret_cast<uint2*>(p.c + c_row * p.size_n + strip * kStripN + 16 * nb + 4 * kb) = packed;
      }
      __builtin_amdgcn_sched_barrier(0);   // one accumulator at a time leaves the AGPRs
    }
  }
}

// Sums the partial tiles of the split tiles of a launch in split order, adds the
// bias and writes C.  One wavefront per accumulator tile (16 rows x 16 columns).
template <typename T>
__global__ __launch_bounds__(256) void tile_reduce_kernel(const TileParams p) {
  const int lane = threadIdx.x & 63;
  const int col16 = lane & 15, kb = lane >> 4;
  const long unit = (long)blockIdx.x * 4 + (threadIdx.x >> 6);   // (tile, 1-KiB block of the partial tile)
  const int first_split = whole_tiles(p);
  const int tiles = p.tiles_m * p.tiles_n - first_split;  // split tiles
  const int blocks = p.tile_rows;                          // blocks per partial tile: 256 or 128
  if (unit >= (long)tiles * blocks) return;
  const int tile = (int)(unit / blocks);
  const int within = (int)(unit - (long)tile * blocks);
  // block = 128 (half of the rows) + 32 strip + 8 column block + row block
  const int half = within >> 7, wave = (within >> 5) & 3;
  const int nb = (within >> 3) & 3, mb = within & 7;
  int tile_m, tile_n;
  tile_coords(p, first_split + tile, tile_m, tile_n);
  const int strip = tile_n * (kTileN / kStripN) + wave;
  const int m = tile_m * p.tile_rows + 128 * half + 16 * mb + col16;
  if (strip * kStripN >= p.size_n) return;
  floatx4_t acc = floatx4_t{0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < p.k_splits; ++s) {
    const float4 v = p.partial[((size_t)(s * tiles + tile) * blocks + within) * 64 + lane];
    acc += floatx4_t{v.x, v.y, v.z, v.w};
  }
  if (m >= p.size_m) return;
  if (p.global_scale) acc = acc * p.global_scale[0];
  const int nl = 16 * nb + 4 * kb;
  float bias[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.bias) {
#pragma unroll
    for (int r = 0; r < 4; ++r) bias[r] = Dq<T>::to_float(p.bias[strip * kStripN + scale_slot(nl + r, false)]);
  }
  uint2 o;
  o.x = (uint32_t)Dq<T>::from_float(acc.x + bias[0]) | ((uint32_t)Dq<T>::from_float(acc.y + bias[1]) << 16);
  o.y = (uint32_t)Dq<T>::from_float(acc.z + bias[2]) | ((uint32_t)Dq<T>::from_float(acc.w + bias[3]) << 16);
  *reinterpret_cast<uint2*>(p.c + (long)m * p.size_n + strip * kStripN + nl) = o;
}

// The same for a grouped call whose kernel has split some of its tiles along K (plan_live_split):
// rows are slots of sorted_ids, bias and global scale the expert's, the routing weight applied as
// in the kernel's own epilogue.  Launched for the most tiles there can be; the rest leaves at once.
template <typename T>
__global__ __launch_bounds__(256) void moe_tile_reduce_kernel(const TileParams p) {
  const int lane = threadIdx.x & 63;
  const int col16 = lane & 15, kb = lane >> 4;
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);   // (split tile, 1-KiB block of the partial tile)
  const TileParams live = live_tiles(p);
  if (live.tiles_m <= 0 || live.k_splits < 2) return;
  const int first_split = live.whole_tiles;
  const int tiles = live.tiles_m * live.tiles_n - first_split;
  const int blocks = p.tile_rows;   // 1-KiB blocks per partial tile: 256 or 128
  if (unit >= tiles * blocks) return;
  const int tile = unit / blocks;
  const int within = unit - tile * blocks;
  const int half = within >> 7, wave = (within >> 5) & 3;
  const int nb = (within >> 3) & 3, mb = within & 7;
  int tile_m, tile_n;
  tile_coords(live, first_split + tile, tile_m, tile_n);
  const int strip = tile_n * (kTileN / kStripN) + wave;
  if (strip * kStripN >= p.size_n) return;
  const int first_slot = p.tile_table[1 + 3 * tile_m] * 64;
  const int tile_rows = p.tile_table[2 + 3 * tile_m] * 64;
  const long expert = p.tile_table[3 + 3 * tile_m];
  const int r = 128 * half + 16 * mb + col16;
  const int id = r < tile_rows ? p.sorted_ids[first_slot + r] : p.rows_total;
  if ((unsigned)id >= (unsigned)p.rows_total) return;   // padding slot
  floatx4_t acc = floatx4_t{0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < live.k_splits; ++s) {
    const float4 v = p.partial[((size_t)(s * tiles + tile) * blocks + within) * 64 + lane];
    acc += floatx4_t{v.x, v.y, v.z, v.w};
  }
  if (p.global_scale) acc = acc * p.global_scale[expert];
  const int nl = 16 * nb + 4 * kb;
  float bias[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.bias) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      bias[i] = Dq<T>::to_float(p.bias[expert * p.expert_bias_stride + strip * kStripN + scale_slot(nl + i, false)]);
  }
  uint16_t o[4] = {Dq<T>::from_float(acc.x + bias[0]), Dq<T>::from_float(acc.y + bias[1]),
                   Dq<T>::from_float(acc.z + bias[2]), Dq<T>::from_float(acc.w + bias[3])};
  if (p.mul_topk) {
    // rounded to the activation type, the product formed and rounded in that type (as in the kernel)
    const float row_w = Dq<T>::to_float(Dq<T>::from_float(p.topk_weights[id]));
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = Dq<T>::from_float(Dq<T>::to_float(o[i]) * row_w);
  }
  uint2 packed;
  packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
  packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
  *reinterpret_cast<uint2*>(p.c + (long)id * p.size_n + strip * kStripN + nl) = packed;
}

// Builds the row-tile table of a grouped call: runs of blocks with the same
// expert are cut into tiles of up to four blocks.  With `table_small` the one or
// two blocks a run ends in go there instead, to be computed as a 128-row tile at
// half the cost.  One workgroup; expert_ids is staged in LDS and scanned by one
// thread (a few hundred entries).
__global__ __launch_bounds__(256) void moe_tile_table_kernel(const int32_t* __restrict__ expert_ids,
                                                            const int32_t* __restrict__ num_post_pad,
                                                            int num_blocks_max, int block_size, int num_experts,
                                                            int32_t* __restrict__ table,
                                                            int32_t* __restrict__ table_small, int max_tiles) {
  extern __shared__ int32_t ids[];
  int blocks = num_post_pad[0] / block_size;
  if (blocks > num_blocks_max) blocks = num_blocks_max;
  for (int b = threadIdx.x; b < blocks; b += blockDim.x) ids[b] = expert_ids[b];
  __syncthreads();
  if (threadIdx.x != 0) return;
  int tiles = 0, small = 0;
  int b = 0;
  while (b < blocks) {
    const int e = ids[b];
    int run = 1;
    while (b + run < blocks && ids[b + run] == e) ++run;
    if (e >= 0 && e < num_experts) {
      for (int at = 0; at < run; at += 4) {
        const int n = min(4, run - at);
        const bool to_small = table_small != nullptr && n <= 2;
        int32_t* t = to_small ? table_small : table;
        int& count = to_small ? small : tiles;
        if (count < max_tiles) {
          t[1 + 3 * count] = b + at;
          t[2 + 3 * count] = n;
          t[3 + 3 * count] = e;
          ++count;
        }
      }
    }
    b += run;
  }
  table[0] = tiles;
  if (table_small != nullptr) table_small[0] = small;
}

template <typename T, bool HAS_ZP, bool G32>
int launch_tile_async_groups(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;  // raising the dynamic LDS limit is needed once per kernel
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_async_kernel<T, HAS_ZP, false, G32>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, async_lds(G32)));
    attr_set = true;
  }
  const int grid = tile_grid(p);
  marlin_tile_async_kernel<T, HAS_ZP, false, G32><<<grid, kTileWaves * 64, async_lds(G32), st>>>(p);
  return SONAR_OK;
}

// MXFP4: bf16, groups of 32 rows, float4_e2m1f codes
int launch_tile_async_fp4(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_async_kernel<__bf16, false, false, true, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, async_lds(true)));
    attr_set = true;
  }
  marlin_tile_async_kernel<__bf16, false, false, true, true><<<tile_grid(p), kTileWaves * 64, async_lds(true), st>>>(p);
  return SONAR_OK;
}

// NVFP4: either activation type, groups of 16 rows, a global scale (one per expert when GROUPED)
template <typename T, bool GROUPED = false>
int launch_tile_async_nvfp4(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_async_kernel<T, false, GROUPED, true, true, 0, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, async_lds(true)));
    attr_set = true;
  }
  marlin_tile_async_kernel<T, false, GROUPED, true, true, 0, true>
      <<<tile_grid(p), kTileWaves * 64, async_lds(true), st>>>(p);
  return SONAR_OK;
}

int launch_tile_grouped_fp4(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_async_kernel<__bf16, false, true, true, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, async_lds(true)));
    attr_set = true;
  }
  marlin_tile_async_kernel<__bf16, false, true, true, true><<<tile_grid(p), kTileWaves * 64, async_lds(true), st>>>(p);
  return SONAR_OK;
}

// 8-bit codes (W8 = 1: uint8b128, 2: float8_e4m3fn), dense or grouped
template <typename T, bool GROUPED, bool G32, int W8>
int launch_tile_async8_groups(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_async_kernel<T, false, GROUPED, G32, false, W8>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, async_lds8(G32)));
    attr_set = true;
  }
  marlin_tile_async_kernel<T, false, GROUPED, G32, false, W8>
      <<<tile_grid(p), kTileWaves * 64, async_lds8(G32), st>>>(p);
  return SONAR_OK;
}
template <typename T, bool GROUPED>
int launch_tile_async8(const TileParams& p, bool fp8, hipStream_t st) {
  const bool g32 = p.num_groups > 1 && p.group_size == 32;
  if (fp8) return g32 ? launch_tile_async8_groups<T, GROUPED, true, 2>(p, st)
                      : launch_tile_async8_groups<T, GROUPED, false, 2>(p, st);
  return g32 ? launch_tile_async8_groups<T, GROUPED, true, 1>(p, st)
             : launch_tile_async8_groups<T, GROUPED, false, 1>(p, st);
}

template <typename T, bool HAS_ZP, bool GROUPED, int RB>
int launch_tile_wide_rows(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_wide_kernel<T, HAS_ZP, GROUPED, RB>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, wide_lds(RB)));
    attr_set = true;
  }
  marlin_tile_wide_kernel<T, HAS_ZP, GROUPED, RB><<<tile_grid(p), 256, wide_lds(RB), st>>>(p);
  return SONAR_OK;
}
// MXFP4: bf16, groups of 32 rows, float4_e2m1f codes
template <bool GROUPED, int RB>
int launch_tile_wide_fp4_rows(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_wide_kernel<__bf16, false, GROUPED, RB, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, wide_lds(RB)));
    attr_set = true;
  }
  marlin_tile_wide_kernel<__bf16, false, GROUPED, RB, true><<<tile_grid(p), 256, wide_lds(RB), st>>>(p);
  return SONAR_OK;
}
template <bool GROUPED>
int launch_tile_wide_fp4(const TileParams& p, hipStream_t st) {
  if (p.tile_rows == 128) return launch_tile_wide_fp4_rows<GROUPED, 8>(p, st);
  return launch_tile_wide_fp4_rows<GROUPED, 16>(p, st);
}
// NVFP4: either activation type, groups of 16 rows, a global scale (one per expert when GROUPED)
template <typename T, bool GROUPED, int RB>
int launch_tile_wide_nvfp4_rows(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_wide_kernel<T, false, GROUPED, RB, true, 0, true, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, wide_lds(RB)));
    attr_set = true;
  }
  marlin_tile_wide_kernel<T, false, GROUPED, RB, true, 0, true, true><<<tile_grid(p), 256, wide_lds(RB), st>>>(p);
  return SONAR_OK;
}
template <typename T, bool GROUPED>
int launch_tile_wide_nvfp4(const TileParams& p, hipStream_t st) {
  if (p.tile_rows != kTileM) return fail(SONAR_E_INVALID, "internal: NVFP4 runs on 256-row tiles");
  return launch_tile_wide_nvfp4_rows<T, GROUPED, 16>(p, st);
}
// 8-bit codes: uint8b128 or float8_e4m3fn (groups of 64 * 2^i rows or one group; G32: of 32 rows, MXFP8)
inline bool wide_groups_of_32(const TileParams& p) { return p.num_groups > 1 && p.group_size == 32; }
template <typename T, bool GROUPED, int W8, bool G32, int RB = 16>
int launch_tile_wide8_groups(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_wide_kernel<T, false, GROUPED, RB, false, W8, G32>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, wide_lds(RB)));
    attr_set = true;
  }
  marlin_tile_wide_kernel<T, false, GROUPED, RB, false, W8, G32><<<tile_grid(p), 256, wide_lds(RB), st>>>(p);
  return SONAR_OK;
}
template <typename T, bool GROUPED>
int launch_tile_wide8(const TileParams& p, bool fp8, hipStream_t st) {
  const bool g32 = wide_groups_of_32(p);
  // 128-row tiles (dense calls with few tiles; the short ends of an expert's rows)
  if (p.tile_rows == 128 && g32) return fail(SONAR_E_INVALID, "internal: 8-bit codes with groups of 32 rows run on 256-row tiles");
  if (p.tile_rows == 128)
    return fp8 ? launch_tile_wide8_groups<T, GROUPED, 2, false, 8>(p, st)
               : launch_tile_wide8_groups<T, GROUPED, 1, false, 8>(p, st);
  if (fp8) return g32 ? launch_tile_wide8_groups<T, GROUPED, 2, true>(p, st)
                      : launch_tile_wide8_groups<T, GROUPED, 2, false>(p, st);
  return g32 ? launch_tile_wide8_groups<T, GROUPED, 1, true>(p, st)
             : launch_tile_wide8_groups<T, GROUPED, 1, false>(p, st);
}
// 4-bit integer codes with groups of 32 rows
template <typename T, bool HAS_ZP, bool GROUPED, int RB>
int launch_tile_wide_g32_rows(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_wide_kernel<T, HAS_ZP, GROUPED, RB, false, 0, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, wide_lds(RB)));
    attr_set = true;
  }
  marlin_tile_wide_kernel<T, HAS_ZP, GROUPED, RB, false, 0, true><<<tile_grid(p), 256, wide_lds(RB), st>>>(p);
  return SONAR_OK;
}
template <typename T, bool HAS_ZP, bool GROUPED>
int launch_tile_wide_g32(const TileParams& p, hipStream_t st) {
  if constexpr (!GROUPED) {
    if (p.tile_rows == 128) return launch_tile_wide_g32_rows<T, HAS_ZP, false, 8>(p, st);
  } else if (p.tile_rows == 128) {
    return fail(SONAR_E_INVALID, "internal: grouped calls with groups of 32 rows run on 256-row tiles");
  }
  return launch_tile_wide_g32_rows<T, HAS_ZP, GROUPED, 16>(p, st);
}
template <typename T, bool HAS_ZP, bool GROUPED = false>
int launch_tile_wide(const TileParams& p, hipStream_t st) {
  if (wide_groups_of_32(p)) return launch_tile_wide_g32<T, HAS_ZP, GROUPED>(p, st);
  if (p.tile_rows == 128) return launch_tile_wide_rows<T, HAS_ZP, GROUPED, 8>(p, st);
  return launch_tile_wide_rows<T, HAS_ZP, GROUPED, 16>(p, st);
}

template <typename T, bool HAS_ZP>
int launch_tile_async(const TileParams& p, hipStream_t st) {
  return (p.num_groups > 1 && p.group_size == 32) ? launch_tile_async_groups<T, HAS_ZP, true>(p, st)
                                                  : launch_tile_async_groups<T, HAS_ZP, false>(p, st);
}

template <typename T, bool HAS_ZP, bool G32>
int launch_tile_grouped_groups(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_async_kernel<T, HAS_ZP, true, G32>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, async_lds(G32)));
    attr_set = true;
  }
  marlin_tile_async_kernel<T, HAS_ZP, true, G32><<<tile_grid(p), kTileWaves * 64, async_lds(G32), st>>>(p);
  return SONAR_OK;
}

template <typename T, bool HAS_ZP>
int launch_tile_grouped(const TileParams& p, hipStream_t st) {
  return (p.num_groups > 1 && p.group_size == 32) ? launch_tile_grouped_groups<T, HAS_ZP, true>(p, st)
                                                  : launch_tile_grouped_groups<T, HAS_ZP, false>(p, st);
}

template <typename T, bool HAS_ZP, bool HAS_PERM>
int launch_tile(const TileParams& p, hipStream_t st) {
  static bool attr_set = false;  // raising the dynamic LDS limit is needed once per kernel
  if (!attr_set) {
    SONAR_HIP(hipFuncSetAttribute((const void*)marlin_tile_kernel<T, HAS_ZP, HAS_PERM>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kTileLds));
    attr_set = true;
  }
  const int grid = tile_grid(p);
  marlin_tile_kernel<T, HAS_ZP, HAS_PERM><<<grid, kTileWaves * 64, kTileLds, st>>>(p);
  return SONAR_OK;
}

}  // namespace

namespace {
// The wide form: groups of 64 * 2^i rows or one group; K ranges of a multiple of four steps, or long ones.
// Groups of 32 rows: whole passes only.
// Steps of zeros the wide kernel adds to a K range of `range` steps (at most a tenth of the range is accepted).
int wide_padding(int range) { return (4 - range % 4) % 4; }
bool wide_applies(const TileParams& p) {
  static const bool no_wide = getenv("SONAR_MARLIN_NO_WIDE_TILE") != nullptr;   // debugging aid
  if (no_wide) return false;
  // K ranges are rounded up to four steps with steps of zeros: not where that is a large part of the work
  const int range = p.k_splits > 1 ? p.k_steps_per_split : p.size_k / kTileK;
  if (wide_groups_of_32(p)) return wide_padding(range) == 0;
  if (wide_padding(range) * 10 > range) return false;
  if (p.num_groups == 1) return true;
  const int per_group = p.group_size / kTileK;   // steps per group: a power of two
  return p.group_size % kTileK == 0 && (per_group & (per_group - 1)) == 0;
}
// ... and for MXFP4 (groups of 32 rows, the caller has checked): the K ranges only.
bool wide_applies_fp4(const TileParams& p) {
  static const bool no_wide = getenv("SONAR_MARLIN_NO_WIDE_TILE") != nullptr;
  const int range = p.k_splits > 1 ? p.k_steps_per_split : p.size_k / kTileK;
  // (no padding here: the eight-wavefront kernel is as fast on these codes, and ahead once steps are wasted:
  // K = 2880, N = 5760, M = 4096: 143 us against 156)
  return !no_wide && wide_padding(range) == 0;
}
// ... and for 8-bit codes (the same rule).
bool wide_applies8(const TileParams& p) { return wide_applies(p); }
}  // namespace

// The asynchronous tile kernel needs groups of 32 rows or a multiple of 64 and no gather of A.
bool tile_async_applies(bool has_perm, int64_t num_groups, int group_size) {
  return !has_perm && (num_groups == 1 || group_size % kTileK == 0 || group_size == 32);
}

namespace {
// What tile_gemm launches for a call the asynchronous tile kernels take: one launch (with
// tile_reduce_kernel behind it when K is split), or two launches of the wide kernel.
struct TileLaunches {
  int count;          // 1 or 2; 0: an internal error
  TileParams launch[2];
};

// `p` arrives with the shape, the pointers and one 256-row launch over the whole of K filled in.
TileLaunches plan_tile_launches(TileParams p, int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups,
                                int group_size, void* partial, size_t partial_bytes, bool fp4, bool nvfp4, int bits,
                                bool has_perm) {
  TileLaunches out;
  out.count = 1;
  const int steps_per_group = group_size / kTileK;
  const bool wide128 = bits == 4 && !fp4 && !has_perm &&
                       (num_groups == 1 || (group_size % kTileK == 0 && (steps_per_group & (steps_per_group - 1)) == 0));
  const bool rows_97_128 = plan_rows_97_128(size_m, size_n, size_k, wide128);
  GemmPlan plan = plan_gemm(size_m, size_n, size_k, true, 256, rows_97_128);
  // few tiles and a call the wide kernel takes: 128-row tiles
  static const bool no_128 = getenv("SONAR_MARLIN_NO_128_ROW_TILES") != nullptr;   // debugging aid
  // (not for NVFP4 and 8-bit codes with groups of 32 rows, whose heavier dequantisation wants the 16 row blocks
  // to hide behind: M = 512, K = 4096, N = 11008: NVFP4 69.9 us against 68.7, MXFP8 91.8 against 82.2)
  const bool rows128_ok = !nvfp4 && !(bits == 8 && num_groups > 1 && group_size == 32);
  if (!no_128 && rows128_ok && plan_prefers_128_rows(size_m, size_n, size_k, rows_97_128)) {
    const GemmPlan plan128 = plan_gemm(size_m, size_n, size_k, true, 128, rows_97_128);
    TileParams probe = p;
    probe.tile_rows = 128;
    probe.k_splits = plan128.k_splits;
    probe.k_steps_per_split = plan128.k_steps_per_split;
    if (plan128.tile && (fp4 ? wide_applies_fp4(probe) : wide_applies(probe)) &&
        (plan128.k_splits == 1 || (partial != nullptr && partial_bytes >= plan_partial_bytes(plan128, size_m, size_n)))) {
      plan = plan128;
      p.tile_rows = 128;
      p.tiles_m = (int)((size_m + 127) / 128);
      p.tile_band = 8;   // the same rows of A per band as four 256-row tiles
    }
  }
  if (plan.k_splits > 1 && partial != nullptr && partial_bytes >= plan_partial_bytes(plan, size_m, size_n)) {
    p.k_splits = plan.k_splits;
    p.k_steps_per_split = plan.k_steps_per_split;
    p.whole_tiles = (int)plan.whole_tiles;
    p.partial = static_cast<float4*>(partial);
    static const char* max_splits = getenv("SONAR_MARLIN_MAX_K_SPLITS");  // debugging aid
    if (max_splits && atoi(max_splits) >= 1 && p.k_splits > atoi(max_splits)) {
      const int k_steps = (int)(size_k / kTileK);
      p.k_splits = atoi(max_splits);
      p.k_steps_per_split = (k_steps + p.k_splits - 1) / p.k_splits;
      p.k_splits = (k_steps + p.k_steps_per_split - 1) / p.k_steps_per_split;
      if (p.k_splits == 1) p.partial = nullptr;
    }
  }
  out.launch[0] = p;
  if (p.tile_rows != kTileM && !(fp4 ? wide_applies_fp4(p) : wide_applies(p))) {
    out.count = 0;   // 128-row tiles exist in the wide tile kernel only
    return out;
  }
  auto takes_wide = [&](const TileParams& q) {
    return fp4 ? wide_applies_fp4(q) : (bits == 8 ? wide_applies8(q) : wide_applies(q));
  };
  // More tiles than compute units with a short last round (M = 4096, N = 6144: 384 tiles of 256
  // rows = 256 + 128): instead of cutting the K ranges of that round's tiles in two and summing
  // partial tiles in a third launch, the full rounds run as they are and the last round runs in
  // a second launch as twice as many 128-row tiles over the whole of K: nothing goes through
  // scratch (163 + 18 us of split tiles and their sum before).  Tile t of the 256-row numbering
  // is tiles 2 t and 2 t + 1 of the 128-row numbering with bands twice as high.
  static const bool no_two_sizes = getenv("SONAR_MARLIN_NO_TWO_TILE_SIZES") != nullptr;   // debugging aid
  if (!no_two_sizes && !no_128 && rows128_ok && p.tile_rows == kTileM && plan.k_splits > 1 && plan.whole_tiles > 0 &&
      (size_m - 1) % kTileM >= 128) {
    TileParams big = p;
    big.k_splits = 1;
    big.k_steps_per_split = (int)(size_k / kTileK);
    big.partial = nullptr;
    big.tile_count = (int)plan.whole_tiles;
    TileParams half = big;
    half.tile_rows = 128;
    half.tiles_m = 2 * p.tiles_m;
    half.tile_band = 8;
    half.tile_begin = 2 * (int)plan.whole_tiles;
    half.tile_count = 2 * (p.tiles_m * p.tiles_n - (int)plan.whole_tiles);
    if (takes_wide(big) && takes_wide(half)) {
      out.count = 2;
      out.launch[0] = big;
      out.launch[1] = half;
    }
  }
  return out;
}

// The shape of a dense call as one 256-row launch over the whole of K (no pointers).
TileParams dense_tile_shape(int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups, int group_size) {
  TileParams p = {};
  p.size_m = (int)size_m;
  p.size_n = (int)size_n;
  p.size_k = (int)size_k;
  p.num_groups = (int)num_groups;
  p.group_size = group_size;
  p.chunks_per_strip = (int)(size_k / kChunkK);
  p.tile_rows = kTileM;
  p.tiles_m = (int)((size_m + kTileM - 1) / kTileM);
  p.tile_band = 4;
  p.tile_begin = p.tile_count = 0;
  p.tiles_n = (int)((size_n + kTileN - 1) / kTileN);
  p.k_splits = 1;
  p.whole_tiles = 0;  // read only with k_splits > 1
  p.k_steps_per_split = (int)(size_k / kTileK);
  return p;
}
}  // namespace

// Called by sonar_marlin_gemm for size_m > 64.  Shapes and pointers have been
// validated by the caller; size_k % 64 == 0 is required here.
int tile_gemm(const void* a, int64_t a_row_stride, void* c, const uint32_t* b, const void* bias,
              const void* scales, const float* global_scale, const uint32_t* zeros, const int32_t* perm, int dtype,
              int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups, int group_size, void* partial,
              size_t partial_bytes, bool fp4, int bits, bool fp8, hipStream_t st) {
  TileParams p = dense_tile_shape(size_m, size_n, size_k, num_groups, group_size);
  p.global_scale = global_scale;
  p.a = static_cast<const uint16_t*>(a);
  p.lda = a_row_stride;
  p.c = static_cast<uint16_t*>(c);
  p.b = reinterpret_cast<const uint4*>(b);
  p.bias = static_cast<const uint16_t*>(bias);
  p.scales = static_cast<const uint16_t*>(scales);
  p.zeros = zeros;
  p.perm = perm;
  const bool zp = zeros != nullptr, pm = perm != nullptr;
  int rc;
  static const bool no_async = getenv("SONAR_MARLIN_NO_ASYNC_TILE") != nullptr;  // debugging aid
  const bool nvfp4 = fp4 && global_scale != nullptr;   // the caller has checked: groups of 16 rows
  if ((nvfp4 || tile_async_applies(pm, num_groups, group_size)) &&
      (!no_async || fp4 || bits == 8)) {   // float4 and 8-bit codes exist here only
    const TileLaunches plan = plan_tile_launches(p, size_m, size_n, size_k, num_groups, group_size, partial,
                                                 partial_bytes, fp4, nvfp4, bits, pm);
    if (plan.count == 0)
      return fail(SONAR_E_INVALID, "internal: 128-row tiles exist in the wide tile kernel only");
    // the kernel a launch described by q takes
    auto launch = [&](const TileParams& q) -> int {
      if (nvfp4 && wide_applies_fp4(q))
        return dtype == SONAR_DTYPE_F16 ? launch_tile_wide_nvfp4<_Float16, false>(q, st)
                                    : launch_tile_wide_nvfp4<__bf16, false>(q, st);
      else if (nvfp4)
        return dtype == SONAR_DTYPE_F16 ? launch_tile_async_nvfp4<_Float16>(q, st) : launch_tile_async_nvfp4<__bf16>(q, st);
      else if (fp4)   // the caller has checked: bf16, groups of 32 rows, no zero points
        return wide_applies_fp4(q) ? launch_tile_wide_fp4<false>(q, st) : launch_tile_async_fp4(q, st);
      else if (bits == 8 && wide_applies8(q))
        return dtype == SONAR_DTYPE_F16 ? launch_tile_wide8<_Float16, false>(q, fp8, st)
                                    : launch_tile_wide8<__bf16, false>(q, fp8, st);
      else if (bits == 8)   // symmetric 8-bit codes: the caller has checked
        return dtype == SONAR_DTYPE_F16 ? launch_tile_async8<_Float16, false>(q, fp8, st)
                                    : launch_tile_async8<__bf16, false>(q, fp8, st);
      else if (wide_applies(q) && dtype == SONAR_DTYPE_F16)
        return zp ? launch_tile_wide<_Float16, true>(q, st) : launch_tile_wide<_Float16, false>(q, st);
      else if (wide_applies(q))
        return zp ? launch_tile_wide<__bf16, true>(q, st) : launch_tile_wide<__bf16, false>(q, st);
      else if (dtype == SONAR_DTYPE_F16)
        return zp ? launch_tile_async<_Float16, true>(q, st) : launch_tile_async<_Float16, false>(q, st);
      else
        return zp ? launch_tile_async<__bf16, true>(q, st) : launch_tile_async<__bf16, false>(q, st);
    };
    if (plan.count == 2) {
      if (int rc1 = launch(plan.launch[0])) return rc1;
      if (int rc2 = launch_status("marlin_tile_wide_kernel")) return rc2;
      if (int rc1 = launch(plan.launch[1])) return rc1;
      return launch_status("marlin_tile_wide_kernel (128-row tiles)");
    }
    p = plan.launch[0];
    rc = launch(p);
    if (rc) return rc;
    if (int rc2 = launch_status("marlin_tile_async_kernel")) return rc2;
    if (p.k_splits > 1) {
      const int blocks = (p.tiles_m * p.tiles_n - p.whole_tiles) * (p.tile_rows / 4);
      if (dtype == SONAR_DTYPE_F16) tile_reduce_kernel<_Float16><<<blocks, 256, 0, st>>>(p);
      else tile_reduce_kernel<__bf16><<<blocks, 256, 0, st>>>(p);
      return launch_status("tile_reduce_kernel");
    }
    return SONAR_OK;
  }
  if (bits == 8) return fail(SONAR_E_INVALID, "internal: 8-bit codes exist in the asynchronous tile kernel only");
  if (zp && pm) return fail(SONAR_E_INVALID, "internal: act-order with zero points");   // refused by the entry point
  if (dtype == SONAR_DTYPE_F16) {
    rc = zp ? launch_tile<_Float16, true, false>(p, st)
            : (pm ? launch_tile<_Float16, false, true>(p, st) : launch_tile<_Float16, false, false>(p, st));
  } else {
    rc = zp ? launch_tile<__bf16, true, false>(p, st)
            : (pm ? launch_tile<__bf16, false, true>(p, st) : launch_tile<__bf16, false, false>(p, st));
  }
  if (rc) return rc;
  return launch_status("marlin_tile_kernel");
}

// Row tiles a grouped call can have at most, and the bytes of its tile table.  A tile is a
// run of up to four blocks of one expert; expert_ids need not be grouped by expert (blocks of
// absent experts, -1, may sit between runs), so the bound is one tile per block: the table
// can never be short of an entry, whatever the routing.
int moe_tile_max(int64_t sorted_len, int64_t num_experts) {
  (void)num_experts;
  return (int)((sorted_len + 63) / 64);
}
// (two tables: the tiles of up to four blocks, and the one- or two-block ends of the experts' rows
// that the wide kernel computes as 128-row tiles)
static size_t moe_one_table_bytes(int64_t sorted_len) {
  return ((size_t)(1 + 3 * moe_tile_max(sorted_len, 0)) * sizeof(int32_t) + 255) & ~(size_t)255;
}
size_t moe_tile_table_bytes(int64_t sorted_len, int64_t num_experts) {
  (void)num_experts;
  return 2 * moe_one_table_bytes(sorted_len);
}
// Room for the fp32 partial tiles of a grouped call that splits some of its tiles along K on the
// device (plan_live_split): 64 MiB for the 256-row tiles and 32 MiB for the 128-row tiles where K
// allows a split, else none.
static size_t moe_partial_bytes_of(int tile_rows) { return (size_t)kLiveSplitWorkMax * tile_rows * 1024; }
size_t moe_tile_partial_bytes(int64_t size_k) {
  const int64_t k_steps = size_k / kTileK;
  if (size_k % (4 * kTileK) != 0 || k_steps < 16) return 0;
  return moe_partial_bytes_of(kTileM) + moe_partial_bytes_of(128);
}

// Called by sonar_moe_wna16_marlin_gemm for 64-slot blocks without act-order
// when group_size % 64 == 0 (or one group) and size_k % 64 == 0.
int moe_tile_gemm(const void* a, void* c, const uint32_t* b, const void* bias, const void* scales,
                  const float* global_scale, const uint32_t* zeros, const int32_t* sorted_ids, int64_t sorted_len, const int32_t* expert_ids,
                  const int32_t* num_post_pad, const float* topk_weights, int64_t top_k, int mul_topk,
                  int64_t num_experts, int32_t* table, int dtype, int64_t size_m, int64_t size_n, int64_t size_k,
                  int64_t num_groups, int group_size, int a_by_slot, bool fp4, int bits, bool fp8, void* partial,
                  size_t partial_bytes, hipStream_t st) {
  const int max_tiles = moe_tile_max(sorted_len, num_experts);
  const int blocks_max = (int)((sorted_len + 63) / 64);
  TileParams p;
  p.tile_begin = p.tile_count = 0;
  p.global_scale = global_scale;   // NVFP4: one per expert
  p.a = static_cast<const uint16_t*>(a);
  p.lda = size_k;
  p.c = static_cast<uint16_t*>(c);
  p.b = reinterpret_cast<const uint4*>(b);
  p.bias = static_cast<const uint16_t*>(bias);
  p.scales = static_cast<const uint16_t*>(scales);
  p.zeros = zeros;
  p.perm = nullptr;
  p.size_m = (int)size_m;
  p.size_n = (int)size_n;
  p.size_k = (int)size_k;
  p.num_groups = (int)num_groups;
  p.group_size = group_size;
  p.chunks_per_strip = (int)(size_k / kChunkK);
  p.tile_rows = kTileM;
  p.tiles_m = max_tiles;
  p.tile_band = max_tiles > 0 ? max_tiles : 1;  // whole columns of row tiles (the wide kernel numbers its tiles itself)
  p.k_splits = 1;
  p.whole_tiles = 0;  // read only with k_splits > 1
  p.k_steps_per_split = (int)(size_k / kTileK);
  p.partial = nullptr;
  p.tiles_n = (int)((size_n + kTileN - 1) / kTileN);
  p.sorted_ids = sorted_ids;
  p.topk_weights = topk_weights;
  p.tile_table = table;
  p.rows_total = (int)(size_m * top_k);
  p.top_k = (int)top_k;
  p.mul_topk = mul_topk;
  p.a_by_slot = a_by_slot;
  p.expert_b_stride = (long)(size_k * size_n / (32 / bits) / 4);
  p.expert_s_stride = (long)(num_groups * size_n);
  p.expert_z_stride = (long)(num_groups * (size_n / 8));
  p.expert_bias_stride = (long)size_n;
  // The wide kernel splits the tiles of a short last round (or all of them when they are few) along
  // K, given room for their partial tiles; moe_tile_reduce_kernel sums them.
  static const bool no_live_split = getenv("SONAR_MARLIN_NO_MOE_K_SPLIT") != nullptr;   // debugging aid
  const bool wide = fp4 ? wide_applies_fp4(p) : (bits == 8 ? wide_applies8(p) : wide_applies(p));
  const size_t partial_need = moe_tile_partial_bytes(size_k);
  if (wide && !no_live_split && partial != nullptr && partial_need > 0 && partial_bytes >= partial_need &&
      ((uintptr_t)partial) % 16 == 0)
    p.partial = static_cast<float4*>(partial);
  // ... and computes the one or two blocks an expert's rows end in as a 128-row tile, in a launch of
  // its own (the forms that have 128-row tiles: not NVFP4, not groups of 32 rows but MXFP4's)
  static const bool no_small = getenv("SONAR_MARLIN_NO_MOE_128_ROW_TILES") != nullptr;   // debugging aid
  const bool nvfp4 = fp4 && global_scale != nullptr;
  const bool two_sizes = wide && !no_small && !nvfp4 && (fp4 || !wide_groups_of_32(p));
  int32_t* table_small = two_sizes ? table + moe_one_table_bytes(sorted_len) / sizeof(int32_t) : nullptr;
  moe_tile_table_kernel<<<1, 256, (size_t)blocks_max * sizeof(int32_t), st>>>(expert_ids, num_post_pad, blocks_max, 64,
                                                                             (int)num_experts, table, table_small,
                                                                             max_tiles);
  if (int rc = launch_status("moe_tile_table_kernel")) return rc;
  auto reduce = [&](const TileParams& q) -> int {
    if (q.partial == nullptr) return SONAR_OK;
    const int64_t tiles = std::min<int64_t>((int64_t)max_tiles * q.tiles_n, kLiveSplitTilesMax);
    const int blocks = (int)(tiles * (q.tile_rows / 4));
    if (dtype == SONAR_DTYPE_F16) moe_tile_reduce_kernel<_Float16><<<blocks, 256, 0, st>>>(q);
    else moe_tile_reduce_kernel<__bf16><<<blocks, 256, 0, st>>>(q);
    return launch_status("moe_tile_reduce_kernel");
  };
  if (two_sizes) {
    TileParams q = p;
    q.tile_rows = 128;
    q.tile_table = table_small;
    if (p.partial != nullptr)
      q.partial = reinterpret_cast<float4*>(static_cast<char*>(partial) + moe_partial_bytes_of(kTileM));
    int rc;
    if (fp4)
      rc = launch_tile_wide_fp4<true>(q, st);
    else if (bits == 8)
      rc = dtype == SONAR_DTYPE_F16 ? launch_tile_wide8<_Float16, true>(q, fp8, st)
                                    : launch_tile_wide8<__bf16, true>(q, fp8, st);
    else if (dtype == SONAR_DTYPE_F16)
      rc = zeros ? launch_tile_wide<_Float16, true, true>(q, st) : launch_tile_wide<_Float16, false, true>(q, st);
    else
      rc = zeros ? launch_tile_wide<__bf16, true, true>(q, st) : launch_tile_wide<__bf16, false, true>(q, st);
    if (rc) return rc;
    if (int rc2 = launch_status("tile kernel (grouped, 128-row tiles)")) return rc2;
    if (int rc2 = reduce(q)) return rc2;
  }
  int rc;
  if (fp4 && global_scale != nullptr && wide_applies_fp4(p))
    rc = dtype == SONAR_DTYPE_F16 ? launch_tile_wide_nvfp4<_Float16, true>(p, st)
                                  : launch_tile_wide_nvfp4<__bf16, true>(p, st);
  else if (fp4 && global_scale != nullptr)
    rc = dtype == SONAR_DTYPE_F16 ? launch_tile_async_nvfp4<_Float16, true>(p, st)
                                  : launch_tile_async_nvfp4<__bf16, true>(p, st);
  else if (fp4)
    rc = wide_applies_fp4(p) ? launch_tile_wide_fp4<true>(p, st) : launch_tile_grouped_fp4(p, st);
  else if (bits == 8 && wide_applies8(p))
    rc = dtype == SONAR_DTYPE_F16 ? launch_tile_wide8<_Float16, true>(p, fp8, st)
                                  : launch_tile_wide8<__bf16, true>(p, fp8, st);
  else if (bits == 8)
    rc = dtype == SONAR_DTYPE_F16 ? launch_tile_async8<_Float16, true>(p, fp8, st)
                                  : launch_tile_async8<__bf16, true>(p, fp8, st);
  else if (wide_applies(p) && dtype == SONAR_DTYPE_F16)
    rc = zeros ? launch_tile_wide<_Float16, true, true>(p, st) : launch_tile_wide<_Float16, false, true>(p, st);
  else if (wide_applies(p))
    rc = zeros ? launch_tile_wide<__bf16, true, true>(p, st) : launch_tile_wide<__bf16, false, true>(p, st);
  else if (dtype == SONAR_DTYPE_F16)
    rc = zeros ? launch_tile_grouped<_Float16, true>(p, st) : launch_tile_grouped<_Float16, false>(p, st);
  else
    rc = zeros ? launch_tile_grouped<__bf16, true>(p, st) : launch_tile_grouped<__bf16, false>(p, st);
  if (rc) return rc;
  if (int rc2 = launch_status("tile kernel (grouped)")) return rc2;
  return reduce(p);
}

}  // namespace sonar

// ---------------------------------------------------------------------------
// Diagnostics for host-side tests (no counterpart in the reference): which tile and which K
// steps every workgroup id of the tile kernels' launches works on, from the same planning and
// mapping code the launches and the kernels run.  One row of six int32 per workgroup that has
// work: launch, rows of a tile, row tile, column tile, first K step, end of its K steps.
namespace {
int64_t schedule_rows(const sonar::TileParams& p, const sonar::TileParams& mapped, int launch, int32_t* out,
                      int64_t out_rows, int64_t at) {
  using namespace sonar;
  const int grid = tile_grid(p);
  const int k_steps = p.size_k / kTileK;
  for (int block = 0; block < grid; ++block) {
    int tile, split, tile_m, tile_n;
    bool whole_k;
    if (!tile_of_block(mapped, block, tile, split, whole_k)) continue;
    tile_coords(mapped, tile, tile_m, tile_n);
    if (at < out_rows) {
      int32_t* row = out + 6 * at;
      row[0] = launch;
      row[1] = mapped.tile_rows;
      row[2] = tile_m;
      row[3] = tile_n;
      row[4] = whole_k ? 0 : split * mapped.k_steps_per_split;
      row[5] = whole_k ? k_steps : std::min(k_steps, row[4] + mapped.k_steps_per_split);
    }
    ++at;
  }
  return at;
}
}  // namespace

// A dense call (4-bit integer codes, no act-order) with room for every partial tile.
extern "C" int64_t sonar_debug_tile_schedule(int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups,
                                             int32_t* out, int64_t out_rows) {
  using namespace sonar;
  if (size_m <= 0 || size_n <= 0 || size_k <= 0 || size_k % kTileK != 0 || num_groups < 1 || size_k % num_groups != 0)
    return -1;
  const int group_size = (int)(size_k / num_groups);
  static float4 never_read;
  const TileLaunches plan =
      plan_tile_launches(dense_tile_shape(size_m, size_n, size_k, num_groups, group_size), size_m, size_n, size_k,
                         num_groups, group_size, &never_read, ~(size_t)0, false, false, 4, false);
  int64_t at = 0;
  for (int l = 0; l < plan.count; ++l) at = schedule_rows(plan.launch[l], plan.launch[l], l, out, out_rows, at);
  return at;
}

// A grouped call whose routing made `row_tiles` row tiles of `tile_rows` rows, launched for up to
// `max_row_tiles` of them; `with_partial`: the call has room for partial tiles.
extern "C" int64_t sonar_debug_moe_tile_schedule(int64_t row_tiles, int64_t max_row_tiles, int64_t size_n,
                                                 int64_t size_k, int tile_rows, int with_partial, int32_t* out,
                                                 int64_t out_rows) {
  using namespace sonar;
  if (row_tiles < 0 || row_tiles > max_row_tiles || size_n <= 0 || size_k <= 0 || size_k % kTileK != 0 ||
      (tile_rows != kTileM && tile_rows != 128))
    return -1;
  static float4 never_read;
  static int32_t no_table;
  TileParams p = dense_tile_shape(max_row_tiles * tile_rows, size_n, size_k, 1, (int)size_k);
  p.tile_rows = tile_rows;
  p.tiles_m = (int)max_row_tiles;
  p.tile_table = &no_table;
  if (with_partial && moe_tile_partial_bytes(size_k) > 0) p.partial = &never_read;
  return schedule_rows(p, live_tiles_of(p, (int)row_tiles), 0, out, out_rows, 0);
}
