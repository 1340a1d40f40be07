// Output of a 64 x 64 tile held as four 32 x 32 matrix-core accumulators, shared by the matmul kernels for 16-bit
// operands.
#pragma once
#include "attn_mfma_common.h"

namespace bsa {
namespace mfma {

// Rounds the tile, passes it through the wave's stage 16 rows at a time, writes it as one block with 16-byte
// stores that cover whole rows (8 stores per lane), and clears the accumulators.  A lane owns 4 columns of
// one of 32 rows per accumulator; v_permlane16_swap regroups the packed values so that, for each half of 16
// rows, all 64 lanes hold a piece (lanes 16 .. 31 and 48 .. 63 take over the right-hand column block of the
// rows of the lanes 16 below them).  Every lane takes part in every step: the exchange between lanes through
// LDS needs the wave to move as one.
template <typename Tr>
__device__ __forceinline__ void rows_flush(f32x16 (&acc)[2][2], char *ob, char *stage, int lane) {
  const int rr = lane & 15, quad = lane >> 4;
  // after the regrouping this lane holds row rr (or 16 + rr), column block quad % 2, column half quad / 2
  char *wbase = stage + rr * 128 + 8 * (quad >> 1);
  const int tw = t_swizzle(rr), cb = 4 * (quad & 1);
  u32x4 back[2][2][2];  // [row block][half of 16 rows][store]
#pragma unroll
  for (int bi = 0; bi < 2; ++bi) {
    uint32_t lo[8], hi[8];  // [2 rq + word]: rows 0 .. 15 / rows 16 .. 31 of this row block
#pragma unroll
    for (int rq = 0; rq < 4; ++rq)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const uint32_t left = Tr::pack2(acc[0][bi][4 * rq + 2 * w], acc[0][bi][4 * rq + 2 * w + 1]);
        const uint32_t right = Tr::pack2(acc[1][bi][4 * rq + 2 * w], acc[1][bi][4 * rq + 2 * w + 1]);
        // lanes 16 .. 31 / 48 .. 63 of `left` trade places with lanes 0 .. 15 / 32 .. 47 of `right`
        const u32x2 sw = __builtin_bit_cast(u32x2, __builtin_amdgcn_permlane16_swap(left, right, false, false));
        lo[2 * rq + w] = sw[0];
        hi[2 * rq + w] = sw[1];
      }
    // LDS executes this wave's instructions in order: the reads of one step see its writes and are done
    // before the next step's writes land, so the four steps are queued without waiting in between (the wave
    // barriers only keep the compiler from reordering them; they emit nothing)
#pragma unroll
    for (int hr = 0; hr < 2; ++hr) {
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const u32x2 v = hr == 0 ? u32x2{lo[2 * rq], lo[2 * rq + 1]} : u32x2{hi[2 * rq], hi[2 * rq + 1]};
        // columns 32 (quad % 2) + 8 rq + 4 (quad / 2) .. + 3: chunk 4 (quad % 2) + rq
        *reinterpret_cast<u32x2 *>(wbase + (((cb + rq) ^ tw) << 4)) = v;
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int q = t * 64 + lane;
        const int r = q >> 3, ch = q & 7;
        back[bi][hr][t] = *reinterpret_cast<const u32x4 *>(stage + r * 128 + ((ch ^ t_swizzle(r)) << 4));
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int hr = 0; hr < 2; ++hr)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int q = t * 64 + lane;
        const int r = q >> 3, ch = q & 7;
        // streaming store: the tile is not read again
        __builtin_nontemporal_store(
            back[bi][hr][t], reinterpret_cast<u32x4 *>(ob + (uint32_t)((32 * bi + 16 * hr + r) * 128 + ch * 16)));
      }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
}

}  // namespace mfma
}  // namespace bsa
