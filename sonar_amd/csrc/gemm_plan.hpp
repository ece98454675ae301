// Which kernel a dense call takes and how much scratch it needs: shared by the
// dispatcher, the tile kernels and sonar_marlin_gemm_scratch_bytes.
#pragma once

#include <stdint.h>

namespace sonar {

struct GemmPlan {
  bool tile;        // MFMA-tiled kernel (else the streaming kernels, in 64-row slabs)
  int tile_rows;    // rows of a tile: 256, or 128 (the wide tile kernel's form for calls with few tiles)
  int k_splits;     // workgroups per split tile along K (tile kernel only)
  int k_steps_per_split;
  // With k_splits > 1: the first `whole_tiles` tiles of the tile numbering are
  // each computed by one workgroup over the whole of K, the rest are split.
  int64_t whole_tiles;
};

// 97..128 rows on a matrix with more strips than compute units (N > 16384) and K <= 8192: the wide tile
// kernel's 128-row form with K in two ranges is ahead of blocks of rows in the decode kernel (measured at
// K = 4096, N = 28672: M = 128: 45 us against 55; M = 72 and 96: level; with 64 to 96 strips, N = 4096 / 6144,
// the decode kernel is two times ahead).  `wide128`: the call is one that form takes (4-bit integer codes
// with groups of 64 * 2^i rows or one group, no act-order gather).
inline bool plan_rows_97_128(int64_t size_m, int64_t size_n, int64_t size_k, bool wide128) {
  // (up to 128 tiles of 256 columns: beyond that K is not split and the tile kernel is not planned)
  return wide128 && size_m > 96 && size_m <= 128 && size_n > 16384 && size_n <= 32768 && size_k <= 8192 &&
         size_k % 256 == 0;
}

inline GemmPlan plan_gemm(int64_t size_m, int64_t size_n, int64_t size_k, bool async_tile, int tile_rows = 256,
                          bool rows_97_128 = false) {
  GemmPlan plan = {false, tile_rows, 1, 0, 0};
  if (size_m <= 64 || size_k % 64 != 0) return plan;
  const int64_t tiles = ((size_m + tile_rows - 1) / tile_rows) * ((size_n + 255) / 256);
  const int k_steps = (int)(size_k / 64);
  plan.k_steps_per_split = k_steps;
  // Few tiles leave compute units idle: split K so that about 256 workgroups
  // run, each with at least eight K steps.  Partial tiles cost 256 KiB of
  // fp32 traffic each way (128 with 128-row tiles), so up to 128 rows the streaming kernels
  // stay ahead.
  int splits = 1;
  if (async_tile && tiles < 256) {
    splits = (int)(256 / tiles);
    if (splits > k_steps / 8) splits = k_steps / 8;
    if (splits > 16) splits = 16;
    if (splits < 1) splits = 1;
  }
  // More tiles than compute units, the last round of workgroups a half or less
  // of the chip: split the tiles of that round so that it is as wide as the
  // others and 1 / splits as long.  Worth the partial-tile traffic (at most
  // 64 MiB each way, about 30 us) once a tile takes about 80 us (48 K steps).
  int64_t whole_tiles = 0;
  if (async_tile && tiles > 256 && k_steps >= 48) {
    const int64_t last_round = tiles % 256;
    if (last_round != 0 && last_round <= 128) {
      splits = (int)(256 / last_round);
      if (splits > k_steps / 8) splits = k_steps / 8;
      if (splits > 16) splits = 16;
      if (splits < 2) splits = 1;
      else whole_tiles = tiles - last_round;
    }
  }
  // (with a long K the partial tiles are a small part of the work: measured at K = 14336, N = 4096,
  // M = 96 / 128: 47 / 53 us in slabs)
  if (size_m <= 128 && !(async_tile && (size_k >= 8192 || rows_97_128) && splits > 1)) return plan;
  if (splits == 1 && size_m <= 512 && tiles < 64) return plan;  // slabs use every compute unit
  plan.tile = true;
  plan.k_splits = splits;
  plan.k_steps_per_split = (k_steps + splits - 1) / splits;
  // ranges of a multiple of four steps where K allows it (the wide tile kernel takes only those)
  if (k_steps % 4 == 0) plan.k_steps_per_split = (plan.k_steps_per_split + 3) / 4 * 4;
  plan.k_splits = (k_steps + plan.k_steps_per_split - 1) / plan.k_steps_per_split;  // no empty split
  plan.whole_tiles = plan.k_splits > 1 ? whole_tiles : tiles;
  return plan;
}

inline size_t plan_partial_bytes(const GemmPlan& plan, int64_t size_m, int64_t size_n) {
  if (!plan.tile || plan.k_splits <= 1) return 0;
  const int64_t tiles = ((size_m + plan.tile_rows - 1) / plan.tile_rows) * ((size_n + 255) / 256);
  return (size_t)plan.k_splits * (size_t)(tiles - plan.whole_tiles) * plan.tile_rows * 1024;
}

// The 128-row form pays when 256-row tiles would leave more than half of the compute units to
// K ranges of the same tile: twice the tiles, half the ranges, half the partial-tile bytes.  With
// a long K the partial tiles are a smaller part of the work and the larger tile is ahead again
// from 48 tiles on (measured at K = 14336, N = 4096, 128-row against 256-row tiles: M = 256:
// 44.4 against 50.9 us; 384: 62.0 against 75.4; 512: 72.7 against 74.6; 768: 109 against 101;
// 1024: 126 against 120).
inline bool plan_prefers_128_rows(int64_t size_m, int64_t size_n, int64_t size_k, bool rows_97_128 = false) {
  const int64_t tiles256 = ((size_m + 255) / 256) * ((size_n + 255) / 256);
  // up to 128 rows (calls that plan_gemm gives to the tile kernel at all: a long K, or rows_97_128) half of a
  // 256-row tile would be padding (K = 14336, N = 4096, M = 72 / 96 / 128: 47.3 / 47.8 / 49.0 -> 29.8 / 30.0 /
  // 30.0 us; K = 8192, N = 8192, M = 65 / 128: 54.4 / 52.9 -> 32.3 / 32.7)
  (void)rows_97_128;
  if (size_m <= 128) return size_m > 64 && tiles256 <= 128;
  return tiles256 <= (size_k <= 8192 ? 128 : 32);
}

// Scratch for the partial tiles of either tiling.
inline size_t plan_partial_bytes_any(int64_t size_m, int64_t size_n, int64_t size_k) {
  const bool r = plan_rows_97_128(size_m, size_n, size_k, true);
  const size_t a = plan_partial_bytes(plan_gemm(size_m, size_n, size_k, true, 256, r), size_m, size_n);
  const size_t b = plan_partial_bytes(plan_gemm(size_m, size_n, size_k, true, 128, r), size_m, size_n);
  return a > b ? a : b;
}

}  // namespace sonar
