// Which kernel serves which problem.
//
// Large problems take 256 x 256 tiles (least bytes moved from L2 into LDS per
// flop): with four waves of 128 x 128 when the fast bf16 epilogue applies (see
// gemm_tile.h), otherwise with eight waves of 128 x 64 and the general
// epilogue.  When that tiling leaves compute units without a tile, smaller
// tiles run on the eight-wave kernel: 256 x 128 (twice the tiles at 1.5 times
// the LDS traffic per flop) while those fill more than half the compute units,
// else 128 x 128, of which two workgroups fit a compute unit (80 KB of LDS and
// at most 128 registers each) and cover each other's waits: 6 to 27 % faster
// than 256 x 128 on shapes such as 1024 x 4096 x 4096 or 1536 x 1536 x 8192.
// (A 4-wave kernel with two workgroups per CU and 64-byte K stages, meant to
// hide the epilogue behind the other workgroup's MFMAs, was measured against
// the 256 x 128 tiles: bound by its global->LDS traffic on large problems and
// no faster on these.)
// Few rows of A (M <= 128) take the strip kernel, which streams B once through a
// deep ring.
#pragma once
#include "gemm_skinny.h"
#include "gemm_tile.h"

namespace mi355q {

enum class TileChoice { k256x256, k256x128, k128x128 };

// For M > 128 and N > 128.
inline TileChoice choose_tiles(int64_t M, int64_t N, int64_t batch) {
  const int64_t cus = compute_units();
  const int64_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256) * batch;
  if (tiles256 >= cus) return TileChoice::k256x256;
  const int64_t tiles_half = ((M + 255) / 256) * ((N + 127) / 128) * batch;
  return 2 * tiles_half > cus ? TileChoice::k256x128 : TileChoice::k128x128;
}

template <bool AK, bool BK_, int FA, int FB>
void launch_by_size(const GemmArgs& g, int64_t batch, hipStream_t st) {
  if (g.M > 128 && g.N > 128) {
    switch (choose_tiles(g.M, g.N, batch)) {
      case TileChoice::k256x256:
        if (g.fast_epi) launch_tile<256, 256, 2, true, AK, BK_, FA, FB>(g, batch, st);
        else launch_tile<256, 256, 4, false, AK, BK_, FA, FB>(g, batch, st);
        break;
      case TileChoice::k256x128: launch_tile<256, 128, 4, false, AK, BK_, FA, FB>(g, batch, st); break;
      case TileChoice::k128x128: launch_tile<128, 128, 4, false, AK, BK_, FA, FB, 2>(g, batch, st); break;
    }
  } else if (g.M <= 128) {
    launch_skinny_by_m<AK, BK_, FA, FB>(g, batch, st);
  } else {
    launch_tile<128, 128, 4, false, AK, BK_, FA, FB, 2>(g, batch, st);
  }
}

// One translation unit per operand layout instantiates this (gemm_inst_*.hip).
template <bool AK, bool BK_>
void launch_by_format(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st) {
  if (fmt_a == MI355Q_E4M3FN && fmt_b == MI355Q_E4M3FN) launch_by_size<AK, BK_, MI355Q_E4M3FN, MI355Q_E4M3FN>(g, batch, st);
  else if (fmt_a == MI355Q_E4M3FN) launch_by_size<AK, BK_, MI355Q_E4M3FN, MI355Q_E5M2>(g, batch, st);
  else if (fmt_b == MI355Q_E4M3FN) launch_by_size<AK, BK_, MI355Q_E5M2, MI355Q_E4M3FN>(g, batch, st);
  else launch_by_size<AK, BK_, MI355Q_E5M2, MI355Q_E5M2>(g, batch, st);
}

}  // namespace mi355q
