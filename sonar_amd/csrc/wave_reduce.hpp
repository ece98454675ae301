// Cross-wavefront sum of MFMA accumulator tiles through LDS.
#pragma once

#include "common.hpp"

namespace sonar {

// Sums the wavefronts' tiles into wavefront 0 through four LDS tile slots: a
// group of up to four wavefronts writes, the group `dist` below it adds.
template <int MB>
__device__ __forceinline__ void reduce_round(floatx4_t (&acc)[MB][4], float4 (*red)[MB * 4][64], int wave,
                                             int lane, int writer_lo, int count, int dist) {
  if (wave >= writer_lo && wave < writer_lo + count) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const floatx4_t v = acc[mb][j];
        red[wave - writer_lo][mb * 4 + j][lane] = make_float4(v.x, v.y, v.z, v.w);
      }
  }
  __syncthreads();
  if (wave >= writer_lo - dist && wave < writer_lo - dist + count) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 v = red[wave - (writer_lo - dist)][mb * 4 + j][lane];
        acc[mb][j] += floatx4_t{v.x, v.y, v.z, v.w};
      }
  }
  __syncthreads();
}

template <int MB, int WAVES>
__device__ __forceinline__ void reduce_waves(floatx4_t (&acc)[MB][4], float4 (*red)[MB * 4][64], int wave,
                                             int lane) {
  static_assert(WAVES == 8 || WAVES == 16, "8 or 16 wavefronts");
  if (WAVES == 16) {
    reduce_round<MB>(acc, red, wave, lane, 12, 4, 8);  // 12..15 -> 4..7
    reduce_round<MB>(acc, red, wave, lane, 8, 4, 8);   // 8..11 -> 0..3
  }
  reduce_round<MB>(acc, red, wave, lane, 4, 4, 4);     // 4..7 -> 0..3
  reduce_round<MB>(acc, red, wave, lane, 2, 2, 2);     // 2..3 -> 0..1
  reduce_round<MB>(acc, red, wave, lane, 1, 1, 1);     // 1 -> 0
}

}  // namespace sonar
