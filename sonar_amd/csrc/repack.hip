// Weight re-ordering kernels: checkpoint packings -> Marlin tile order, and
// Marlin tile order <-> the gfx950 streaming order.  Pure integer work; each
// thread assembles one 32-bit output word from eight source nibbles, so the
// stores of a wavefront are one contiguous 256-byte run.
#include "common.hpp"

namespace sonar {

thread_local char g_last_error[512] = "";
char* last_error_buffer() { return g_last_error; }

namespace {

// Position of a weight inside a Marlin tile (16-bit activations, 4-bit
// weights).  Word w = lane*4 + j of the tile; lane = 4*c + h, c = column % 8
// inside the 16-column sub-tile j, h = (row % 8) / 2.  Nibble slot s of the
// word holds row 2h + (s >> 2) + 8*(s & 1), column c + 8*((s >> 1) & 1).
__device__ __forceinline__ void marlin_word_sources(int word, int slot, int& row, int& col) {
  const int lane = word >> 2;
  const int j = word & 3;
  const int c = lane >> 2;
  const int h = lane & 3;
  row = 2 * h + (slot >> 2) + 8 * (slot & 1);
  col = 16 * j + c + 8 * ((slot >> 1) & 1);
}

template <bool HAS_PERM>
__global__ __launch_bounds__(256) void gptq_to_marlin_kernel(
    const uint32_t* __restrict__ in, const int32_t* __restrict__ perm,
    uint32_t* __restrict__ out, int size_k, int size_n, long total_words) {
  const int n_tiles = size_n / kMarlinTileN;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const long tile = idx / kMarlinTileWords;
    const int word = (int)(idx % kMarlinTileWords);
    const int kt = (int)(tile / n_tiles);
    const int nt = (int)(tile % n_tiles);
    uint32_t packed = 0;
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
      int row, col;
      marlin_word_sources(word, slot, row, col);
      int k = kt * kMarlinTileK + row;
      if (HAS_PERM) k = perm[k];
      const int n = nt * kMarlinTileN + col;
      const uint32_t src = in[(long)(k >> 3) * size_n + n];
      packed |= ((src >> (4 * (k & 7))) & 0xFu) << (4 * slot);
    }
    out[idx] = packed;
  }
}

__global__ __launch_bounds__(256) void awq_to_marlin_kernel(
    const uint32_t* __restrict__ in, uint32_t* __restrict__ out, int size_k,
    int size_n, long total_words) {
  const int n_tiles = size_n / kMarlinTileN;
  const int in_stride = size_n / 8;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const long tile = idx / kMarlinTileWords;
    const int word = (int)(idx % kMarlinTileWords);
    const int kt = (int)(tile / n_tiles);
    const int nt = (int)(tile % n_tiles);
    uint32_t packed = 0;
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
      int row, col;
      marlin_word_sources(word, slot, row, col);
      const int k = kt * kMarlinTileK + row;
      const int n = nt * kMarlinTileN + col;
      // column n % 8 = 2*(p % 4) + p / 4 sits at nibble p = (n%8)/2 + 4*(n%2)
      const int p = ((n & 7) >> 1) + 4 * (n & 1);
      const uint32_t src = in[(long)k * in_stride + (n >> 3)];
      packed |= ((src >> (4 * p)) & 0xFu) << (4 * slot);
    }
    out[idx] = packed;
  }
}

// One thread per gfx950 word.  Word j of lane L of chunk c of strip s holds
// column 64s + 16j + L%16, rows 32c + 8*(L/16) + t (t = 0..7) with row t at
// nibble slot t/2 + 4*(t%2).  Those eight rows live in Marlin k-tile
// 2c + (L/32) at tile rows 8*((L/16)%2) + t, i.e. in the four Marlin words
// lane_m*4 + j with lane_m = 4*(col%8) + t/2.
__global__ __launch_bounds__(256) void marlin_to_gfx950_kernel(
    const uint32_t* __restrict__ in, uint32_t* __restrict__ out, int size_k,
    int size_n, long total_words) {
  const int n_tiles = size_n / kMarlinTileN;
  const int chunks = size_k / kChunkK;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const int j = (int)(idx & 3);
    const int lane = (int)((idx >> 2) & 63);
    const long chunk_id = idx >> 8;
    const int c = (int)(chunk_id % chunks);
    const int s = (int)(chunk_id / chunks);
    const int col16 = lane & 15;
    const int kb = lane >> 4;
    const int kt = 2 * c + (kb >> 1);
    const int hb = kb & 1;  // upper half of the 16-row tile?
    const uint32_t* tile = in + ((long)kt * n_tiles + s) * kMarlinTileWords;
    // Marlin slot of (tile row 8*hb + t, column col16): hb + 2*(col16/8) + 4*(t%2)
    const int slot_even = hb + 2 * (col16 >> 3);
    uint32_t packed = 0;
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const uint32_t w = tile[(4 * (col16 & 7) + h) * 4 + j];
      const uint32_t even = (w >> (4 * slot_even)) & 0xFu;        // row t = 2h
      const uint32_t odd = (w >> (4 * (slot_even + 4))) & 0xFu;   // row t = 2h+1
      packed |= (even << (4 * h)) | (odd << (4 * (h + 4)));
    }
    out[idx] = packed;
  }
}

// Inverse of the above: one thread per Marlin word.
__global__ __launch_bounds__(256) void gfx950_to_marlin_kernel(
    const uint32_t* __restrict__ in, uint32_t* __restrict__ out, int size_k,
    int size_n, long total_words) {
  const int n_tiles = size_n / kMarlinTileN;
  const int chunks = size_k / kChunkK;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const long tile = idx / kMarlinTileWords;
    const int word = (int)(idx % kMarlinTileWords);
    const int kt = (int)(tile / n_tiles);
    const int nt = (int)(tile % n_tiles);
    uint32_t packed = 0;
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
      int row, col;
      marlin_word_sources(word, slot, row, col);
      const int k = kt * kMarlinTileK + row;
      const int c = k / kChunkK;
      const int kb = (k % kChunkK) >> 3;
      const int t = k & 7;
      const int lane = 16 * kb + (col & 15);
      const int j = col >> 4;
      const uint32_t src = in[(((long)nt * chunks + c) * 64 + lane) * 4 + j];
      const int src_slot = (t >> 1) + 4 * (t & 1);
      packed |= ((src >> (4 * src_slot)) & 0xFu) << (4 * slot);
    }
    out[idx] = packed;
  }
}

// ---- 8-bit codes (uint8b128): the same 16 x 64 tile in 256 words.  Word
// lane*8 + 2j + half of the tile; lane = 4*c + h as above; byte s of the word
// holds row 2h + (s >> 1) + 8*(s & 1), column 16j + c + 8*half
// (gptq_marlin_repack.cu:216-236).
constexpr int kMarlinTileWords8 = 256;

__device__ __forceinline__ void marlin8_word_sources(int word, int byte, int& row, int& col) {
  const int lane = word >> 3;
  const int j = (word >> 1) & 3;
  const int half = word & 1;
  row = 2 * (lane & 3) + (byte >> 1) + 8 * (byte & 1);
  col = 16 * j + (lane >> 2) + 8 * half;
}

// GPTQ (K/4, N) int32, byte k % 4 of word [k / 4][n] -> Marlin 8-bit order.
template <bool HAS_PERM>
__global__ __launch_bounds__(256) void gptq8_to_marlin_kernel(
    const uint32_t* __restrict__ in, const int32_t* __restrict__ perm,
    uint32_t* __restrict__ out, int size_k, int size_n, long total_words) {
  const int n_tiles = size_n / kMarlinTileN;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const long tile = idx / kMarlinTileWords8;
    const int word = (int)(idx % kMarlinTileWords8);
    const int kt = (int)(tile / n_tiles);
    const int nt = (int)(tile % n_tiles);
    uint32_t packed = 0;
#pragma unroll
    for (int byte = 0; byte < 4; ++byte) {
      int row, col;
      marlin8_word_sources(word, byte, row, col);
      int k = kt * kMarlinTileK + row;
      if (HAS_PERM) k = perm[k];
      const int n = nt * kMarlinTileN + col;
      const uint32_t src = in[(long)(k >> 2) * size_n + n];
      packed |= ((src >> (8 * (k & 3))) & 0xFFu) << (8 * byte);
    }
    out[idx] = packed;
  }
}

// Position of W[k][n] in the Marlin 8-bit order: word index and byte.
__device__ __forceinline__ long marlin8_position(int k, int n, int n_tiles, int& byte) {
  const int kt = k / kMarlinTileK, row = k % kMarlinTileK;
  const int nt = n / kMarlinTileN, col = n % kMarlinTileN;
  const int c16 = col & 15;
  const int lane = 4 * (c16 & 7) + ((row & 7) >> 1);
  byte = ((row & 1) << 1) | (row >> 3);
  return ((long)kt * n_tiles + nt) * kMarlinTileWords8 + lane * 8 + 2 * (col >> 4) + (c16 >> 3);
}

// The gfx950 order for 8-bit codes: per strip a stream of 1-KiB blocks of 16
// rows, block 2c + h in chunk c; word j of lane L: column 64s + 16j + L%16,
// rows 32c + 8*(L/16) + 4h + t, row t at byte {0, 2, 1, 3}[t].
__device__ __forceinline__ long gfx950_8_position(int k, int n, int chunks, int& byte) {
  const int s = n / kStripN, j = (n % kStripN) >> 4, l16 = n & 15;
  const int c = k / kChunkK, r = k % kChunkK;
  const int kb = r >> 3, h = (r >> 2) & 1, t = r & 3;
  byte = ((t & 1) << 1) | (t >> 1);
  return ((((long)s * chunks + c) * 2 + h) * 64 + 16 * kb + l16) * 4 + j;
}

// One thread per output word; TO_GFX950 selects the direction.
template <bool TO_GFX950>
__global__ __launch_bounds__(256) void marlin8_gfx950_kernel(const uint32_t* __restrict__ in,
                                                            uint32_t* __restrict__ out, int size_k, int size_n,
                                                            long total_words) {
  const int n_tiles = size_n / kMarlinTileN;
  const int chunks = size_k / kChunkK;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    uint32_t packed = 0;
#pragma unroll
    for (int byte = 0; byte < 4; ++byte) {
      int k, n;
      if (TO_GFX950) {  // which (k, n) does byte `byte` of gfx950 word idx hold?
        const int j = (int)(idx & 3);
        const int lane = (int)((idx >> 2) & 63);
        const long block = idx >> 8;
        const int h = (int)(block & 1);
        const int c = (int)((block >> 1) % chunks);
        const int s = (int)((block >> 1) / chunks);
        const int t = ((byte & 1) << 1) | (byte >> 1);
        k = c * kChunkK + 8 * (lane >> 4) + 4 * h + t;
        n = s * kStripN + 16 * j + (lane & 15);
      } else {
        const long tile = idx / kMarlinTileWords8;
        int row, col;
        marlin8_word_sources((int)(idx % kMarlinTileWords8), byte, row, col);
        k = (int)(tile / n_tiles) * kMarlinTileK + row;
        n = (int)(tile % n_tiles) * kMarlinTileN + col;
      }
      int src_byte;
      const long src = TO_GFX950 ? marlin8_position(k, n, n_tiles, src_byte)
                                 : gfx950_8_position(k, n, chunks, src_byte);
      packed |= ((in[src] >> (8 * src_byte)) & 0xFFu) << (8 * byte);
    }
    out[idx] = packed;
  }
}

// ---- 4-bit codes for 8-bit activations (is_a_8bit): tiles of 32 (k) x 32 (n),
// 128 words each, tile (kt, nt) at (kt * (N / 32) + nt) * 128.  Word lane*4 + w:
// column 8w + lane/4; nibble slot s holds row 4*(lane%4) + s/2 + 16*(s%2)
// (gptq_marlin_repack.cu:129-141,176-216).
constexpr int kA8Tile = 32;

__device__ __forceinline__ void a8_word_sources(int word, int slot, int& row, int& col) {
  const int lane = word >> 2;
  row = 4 * (lane & 3) + (slot >> 1) + 16 * (slot & 1);
  col = 8 * (word & 3) + (lane >> 2);
}

// Word index and nibble slot of W[k][n] in that order.
__device__ __forceinline__ long a8_position(int k, int n, int n_tiles, int& slot) {
  const int r = k % kA8Tile, c = n % kA8Tile;
  slot = 2 * (r & 3) + (r >> 4);
  return ((long)(k / kA8Tile) * n_tiles + n / kA8Tile) * kMarlinTileWords + (4 * (c & 7) + ((r & 15) >> 2)) * 4 +
         (c >> 3);
}

// SOURCE 0: GPTQ (K/8, N) words; 1: AWQ (K, N/8) words; 2: the gfx950 order.
template <int SOURCE>
__global__ __launch_bounds__(256) void to_marlin_a8_kernel(const uint32_t* __restrict__ in,
                                                          uint32_t* __restrict__ out, int size_k, int size_n,
                                                          long total_words) {
  const int n_tiles = size_n / kA8Tile;
  const int chunks = size_k / kChunkK;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const long tile = idx / kMarlinTileWords;
    const int word = (int)(idx % kMarlinTileWords);
    uint32_t packed = 0;
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
      int row, col;
      a8_word_sources(word, slot, row, col);
      const int k = (int)(tile / n_tiles) * kA8Tile + row;
      const int n = (int)(tile % n_tiles) * kA8Tile + col;
      uint32_t code;
      if (SOURCE == 0) {
        code = in[(long)(k >> 3) * size_n + n] >> (4 * (k & 7));
      } else if (SOURCE == 1) {
        const int p = ((n & 7) >> 1) + 4 * (n & 1);
        code = in[(long)k * (size_n / 8) + (n >> 3)] >> (4 * p);
      } else {
        const int t = k & 7;
        const int lane = 16 * ((k % kChunkK) >> 3) + (n & 15);
        code = in[(((long)(n / kStripN) * chunks + k / kChunkK) * 64 + lane) * 4 + ((n % kStripN) >> 4)] >>
               (4 * ((t >> 1) + 4 * (t & 1)));
      }
      packed |= (code & 0xFu) << (4 * slot);
    }
    out[idx] = packed;
  }
}

// 8-bit codes in that order (gptq_marlin_repack.cu:216-236 with is_a_8bit): a 32 x 32 tile is 256
// words; word lane*8 + 2*w + h: column 8w + lane/4, rows 4*(lane%4) + {0..3} + 16h at bytes 0..3.
// No GEMM takes it (the reference has no 8-bit weights with 8-bit activations either); the
// repack op produces it.  Source: GPTQ (K/4, N) words.
__global__ __launch_bounds__(256) void gptq8_to_marlin_a8_kernel(const uint32_t* __restrict__ in,
                                                                uint32_t* __restrict__ out, int size_k, int size_n,
                                                                long total_words) {
  const int n_tiles = size_n / kA8Tile;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const long tile = idx / 256;
    const int word = (int)(idx % 256);
    const int lane = word >> 3, w = (word >> 1) & 3, h = word & 1;
    const int n = (int)(tile % n_tiles) * kA8Tile + 8 * w + (lane >> 2);
    const int k0 = (int)(tile / n_tiles) * kA8Tile + 4 * (lane & 3) + 16 * h;   // a multiple of 4: one source word
    out[idx] = in[(long)(k0 >> 2) * size_n + n];
  }
}

// One thread per gfx950 word (rows 32c + 8*(L/16) + t of column 64s + 16j + L%16).
__global__ __launch_bounds__(256) void marlin_a8_to_gfx950_kernel(const uint32_t* __restrict__ in,
                                                                 uint32_t* __restrict__ out, int size_k,
                                                                 int size_n, long total_words) {
  const int n_tiles = size_n / kA8Tile;
  const int chunks = size_k / kChunkK;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    const int j = (int)(idx & 3);
    const int lane = (int)((idx >> 2) & 63);
    const long chunk_id = idx >> 8;
    const int n = (int)(chunk_id / chunks) * kStripN + 16 * j + (lane & 15);
    const int k0 = (int)(chunk_id % chunks) * kChunkK + 8 * (lane >> 4);
    uint32_t packed = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      int slot;
      const long src = a8_position(k0 + t, n, n_tiles, slot);
      packed |= ((in[src] >> (4 * slot)) & 0xFu) << (4 * ((t >> 1) + 4 * (t & 1)));
    }
    out[idx] = packed;
  }
}

// marlin_int4_fp8_preprocess.cu:13-66: nibble by nibble, code -> sign and
// magnitude of code - z (z = 8 without zero points): q >= z ? q - z : 15 - q.
__global__ __launch_bounds__(256) void int4_fp8_preprocess_kernel(const uint32_t* __restrict__ in,
                                                                 const uint32_t* __restrict__ zeros,
                                                                 uint32_t* __restrict__ out, long words_per_row,
                                                                 int group_size, long total_words) {
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total_words;
       idx += (long)gridDim.x * blockDim.x) {
    uint32_t val = in[idx];
    uint32_t zero = zeros ? zeros[(idx / words_per_row) / group_size * words_per_row + idx % words_per_row]
                          : 0x88888888u;
    uint32_t res = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t q = (val >> (4 * i)) & 0xFu, z = (zero >> (4 * i)) & 0xFu;
      res |= (q >= z ? q - z : 15u - q) << (4 * i);
    }
    out[idx] = res;
  }
}

int grid_for(long total_words) {
  long blocks = (total_words + 255) / 256;
  if (blocks > 256L * 32) blocks = 256L * 32;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

int check_repack_shape(int64_t size_k, int64_t size_n, int num_bits) {
  SONAR_REQUIRE(num_bits == 4 || num_bits == 8, "num_bits must be 4 or 8. Got = %d", num_bits);
  SONAR_REQUIRE(size_k > 0 && size_n > 0, "size_k = %ld and size_n = %ld must be positive",
                (long)size_k, (long)size_n);
  SONAR_REQUIRE(size_k % kMarlinTileK == 0, "size_k = %ld is not divisible by tile_k_size = %d",
                (long)size_k, kMarlinTileK);
  SONAR_REQUIRE(size_n % kMarlinTileN == 0, "size_n = %ld is not divisible by tile_n_size = %d",
                (long)size_n, kMarlinTileN);
  SONAR_REQUIRE(size_k * size_n / 8 < (1LL << 40), "weight too large");
  SONAR_REQUIRE(size_k < (1LL << 30) && size_n < (1LL << 30), "size_k / size_n too large");
  return SONAR_OK;
}

}  // namespace
}  // namespace sonar

using namespace sonar;

extern "C" const char* sonar_marlin_last_error(void) { return last_error_buffer(); }
extern "C" const char* sonar_marlin_version(void) { return "sonar-marlin-gfx950 0.1"; }

extern "C" int sonar_gptq_marlin_repack(const uint32_t* b_q_weight, const int32_t* perm,
                                        uint32_t* out, int64_t size_k, int64_t size_n,
                                        int num_bits, void* stream) {
  if (int rc = check_repack_shape(size_k, size_n, num_bits)) return rc;
  SONAR_REQUIRE(b_q_weight && out, "b_q_weight and out must not be NULL");
  hipStream_t st = (hipStream_t)stream;
  if (num_bits == 8) {
    const long words = size_k * size_n / 4;
    if (perm)
      gptq8_to_marlin_kernel<true><<<grid_for(words), 256, 0, st>>>(b_q_weight, perm, out, (int)size_k,
                                                                   (int)size_n, words);
    else
      gptq8_to_marlin_kernel<false><<<grid_for(words), 256, 0, st>>>(b_q_weight, nullptr, out, (int)size_k,
                                                                    (int)size_n, words);
    return launch_status("gptq8_to_marlin_kernel");
  }
  const long total = size_k * size_n / 8;
  if (perm)
    gptq_to_marlin_kernel<true><<<grid_for(total), 256, 0, st>>>(b_q_weight, perm, out, (int)size_k,
                                                                (int)size_n, total);
  else
    gptq_to_marlin_kernel<false><<<grid_for(total), 256, 0, st>>>(b_q_weight, nullptr, out,
                                                                 (int)size_k, (int)size_n, total);
  return launch_status("gptq_to_marlin_kernel");
}

extern "C" int sonar_awq_marlin_repack(const uint32_t* b_q_weight, uint32_t* out, int64_t size_k,
                                       int64_t size_n, int num_bits, void* stream) {
  if (int rc = check_repack_shape(size_k, size_n, num_bits)) return rc;
  if (num_bits != 4) return fail(SONAR_E_UNSUPPORTED, "awq_marlin_repack: 8-bit AWQ weights are not built");
  SONAR_REQUIRE(b_q_weight && out, "b_q_weight and out must not be NULL");
  const long total = size_k * size_n / 8;
  awq_to_marlin_kernel<<<grid_for(total), 256, 0, (hipStream_t)stream>>>(b_q_weight, out, (int)size_k,
                                                                        (int)size_n, total);
  return launch_status("awq_to_marlin_kernel");
}

extern "C" int sonar_marlin_to_gfx950(const uint32_t* marlin, uint32_t* out, int64_t size_k,
                                      int64_t size_n, void* stream) {
  if (int rc = check_repack_shape(size_k, size_n, 4)) return rc;
  SONAR_REQUIRE(size_k % kChunkK == 0, "size_k = %ld is not divisible by %d", (long)size_k, kChunkK);
  SONAR_REQUIRE(marlin && out && marlin != out, "marlin and out must be distinct non-NULL buffers");
  const long total = size_k * size_n / 8;
  marlin_to_gfx950_kernel<<<grid_for(total), 256, 0, (hipStream_t)stream>>>(marlin, out, (int)size_k,
                                                                           (int)size_n, total);
  return launch_status("marlin_to_gfx950_kernel");
}

extern "C" int sonar_gfx950_to_marlin(const uint32_t* gfx950, uint32_t* out, int64_t size_k,
                                      int64_t size_n, void* stream) {
  if (int rc = check_repack_shape(size_k, size_n, 4)) return rc;
  SONAR_REQUIRE(size_k % kChunkK == 0, "size_k = %ld is not divisible by %d", (long)size_k, kChunkK);
  SONAR_REQUIRE(gfx950 && out && gfx950 != out, "gfx950 and out must be distinct non-NULL buffers");
  const long total = size_k * size_n / 8;
  gfx950_to_marlin_kernel<<<grid_for(total), 256, 0, (hipStream_t)stream>>>(gfx950, out, (int)size_k,
                                                                           (int)size_n, total);
  return launch_status("gfx950_to_marlin_kernel");
}

extern "C" int sonar_marlin8_to_gfx950(const uint32_t* marlin, uint32_t* out, int64_t size_k,
                                       int64_t size_n, void* stream) {
  if (int rc = check_repack_shape(size_k, size_n, 8)) return rc;
  SONAR_REQUIRE(size_k % kChunkK == 0, "size_k = %ld is not divisible by %d", (long)size_k, kChunkK);
  SONAR_REQUIRE(marlin && out && marlin != out, "marlin and out must be distinct non-NULL buffers");
  const long total = size_k * size_n / 4;
  marlin8_gfx950_kernel<true><<<grid_for(total), 256, 0, (hipStream_t)stream>>>(marlin, out, (int)size_k,
                                                                               (int)size_n, total);
  return launch_status("marlin8_gfx950_kernel");
}

extern "C" int sonar_gfx950_to_marlin8(const uint32_t* gfx950, uint32_t* out, int64_t size_k,
                                       int64_t size_n, void* stream) {
  if (int rc = check_repack_shape(size_k, size_n, 8)) return rc;
  SONAR_REQUIRE(size_k % kChunkK == 0, "size_k = %ld is not divisible by %d", (long)size_k, kChunkK);
  SONAR_REQUIRE(gfx950 && out && gfx950 != out, "gfx950 and out must be distinct non-NULL buffers");
  const long total = size_k * size_n / 4;
  marlin8_gfx950_kernel<false><<<grid_for(total), 256, 0, (hipStream_t)stream>>>(gfx950, out, (int)size_k,
                                                                                (int)size_n, total);
  return launch_status("marlin8_gfx950_kernel");
}

// ---- the weight order for 8-bit activations --------------------------------
namespace {
int check_a8_shape(int64_t size_k, int64_t size_n, int num_bits) {
  if (int rc = check_repack_shape(size_k, size_n, num_bits)) return rc;
  SONAR_REQUIRE(size_k % kA8Tile == 0, "size_k = %ld is not divisible by %d (the tile of 8-bit activations)",
                (long)size_k, kA8Tile);
  return SONAR_OK;
}
}  // namespace

extern "C" int sonar_gptq_marlin_repack_a8(const uint32_t* b_q_weight, uint32_t* out, int64_t size_k,
                                           int64_t size_n, int num_bits, void* stream) {
  if (int rc = check_a8_shape(size_k, size_n, num_bits)) return rc;
  SONAR_REQUIRE(b_q_weight && out, "b_q_weight and out must not be NULL");
  if (num_bits == 8) {
    const long words = size_k * size_n / 4;
    gptq8_to_marlin_a8_kernel<<<grid_for(words), 256, 0, (hipStream_t)stream>>>(b_q_weight, out, (int)size_k,
                                                                               (int)size_n, words);
    return launch_status("gptq8_to_marlin_a8_kernel");
  }
  const long total = size_k * size_n / 8;
  to_marlin_a8_kernel<0><<<grid_for(total), 256, 0, (hipStream_t)stream>>>(b_q_weight, out, (int)size_k,
                                                                          (int)size_n, total);
  return launch_status("to_marlin_a8_kernel");
}

extern "C" int sonar_awq_marlin_repack_a8(const uint32_t* b_q_weight, uint32_t* out, int64_t size_k,
                                          int64_t size_n, int num_bits, void* stream) {
  if (int rc = check_a8_shape(size_k, size_n, num_bits)) return rc;
  if (num_bits != 4) return fail(SONAR_E_UNSUPPORTED, "awq_marlin_repack: 8-bit AWQ weights are not built");
  SONAR_REQUIRE(b_q_weight && out, "b_q_weight and out must not be NULL");
  const long total = size_k * size_n / 8;
  to_marlin_a8_kernel<1><<<grid_for(total), 256, 0, (hipStream_t)stream>>>(b_q_weight, out, (int)size_k,
                                                                          (int)size_n, total);
  return launch_status("to_marlin_a8_kernel");
}

extern "C" int sonar_marlin_a8_to_gfx950(const uint32_t* marlin, uint32_t* out, int64_t size_k, int64_t size_n,
                                         void* stream) {
  if (int rc = check_a8_shape(size_k, size_n, 4)) return rc;
  SONAR_REQUIRE(marlin && out && marlin != out, "marlin and out must be distinct non-NULL buffers");
  const long total = size_k * size_n / 8;
  marlin_a8_to_gfx950_kernel<<<grid_for(total), 256, 0, (hipStream_t)stream>>>(marlin, out, (int)size_k,
                                                                              (int)size_n, total);
  return launch_status("marlin_a8_to_gfx950_kernel");
}

extern "C" int sonar_gfx950_to_marlin_a8(const uint32_t* gfx950, uint32_t* out, int64_t size_k, int64_t size_n,
                                         void* stream) {
  if (int rc = check_a8_shape(size_k, size_n, 4)) return rc;
  SONAR_REQUIRE(gfx950 && out && gfx950 != out, "gfx950 and out must be distinct non-NULL buffers");
  const long total = size_k * size_n / 8;
  to_marlin_a8_kernel<2><<<grid_for(total), 256, 0, (hipStream_t)stream>>>(gfx950, out, (int)size_k,
                                                                          (int)size_n, total);
  return launch_status("to_marlin_a8_kernel");
}

extern "C" int sonar_marlin_int4_fp8_preprocess(const uint32_t* qweight, const uint32_t* qzeros, uint32_t* out,
                                                int64_t rows, int64_t words_per_row, int64_t group_size,
                                                void* stream) {
  SONAR_REQUIRE(qweight && out, "qweight and out must not be NULL");
  SONAR_REQUIRE(rows > 0 && words_per_row > 0, "rows = %ld and words_per_row = %ld must be positive", (long)rows,
                (long)words_per_row);
  if (qzeros) {
    SONAR_REQUIRE(rows % 32 == 0, "size_k % 32 != 0");
    SONAR_REQUIRE(group_size > 0 && rows % group_size == 0, "qweight.size(0) % qzeros.size(0) != 0");
    SONAR_REQUIRE(group_size % 8 == 0, "group_size % 8 != 0");
  } else {
    SONAR_REQUIRE(rows * words_per_row * 8 % 256 == 0, "qweight.numel() * 8 % 256 != 0");
    group_size = 1;
  }
  const long total = rows * words_per_row;
  int4_fp8_preprocess_kernel<<<grid_for(total), 256, 0, (hipStream_t)stream>>>(qweight, qzeros, out, words_per_row,
                                                                              (int)group_size, total);
  return launch_status("int4_fp8_preprocess_kernel");
}
