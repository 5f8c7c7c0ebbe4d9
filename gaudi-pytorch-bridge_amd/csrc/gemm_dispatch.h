// Which kernel serves which problem.
//
// Large problems take 256 x 256 tiles (least bytes moved from L2 into LDS per
// flop): with four waves of 128 x 128 when the fast bf16 epilogue applies (see
// gemm_tile.h), otherwise with eight waves of 128 x 64 and the general
// epilogue.  When that tiling leaves compute units without a tile, smaller
// tiles run: 256 x 128 (twice the tiles at 1.5 times the global->LDS traffic
// per flop) while those fill more than half the compute units, with four waves
// of 128 x 64 (1.5 KB of LDS fragments read per MFMA; as eight waves of
// 128 x 32 it read 2.5 KB and was 3 to 8 % slower at 256 x 8192 x 28672);
// else 128 x 128 with eight waves, of which two workgroups fit a compute unit
// (80 KB of LDS and at most 128 registers each) and cover each other's waits:
// 6 to 27 % faster than 256 x 128 on shapes such as 1024 x 4096 x 4096 or
// 1536 x 1536 x 8192 (four waves there gained nothing with a bf16 output and
// lost 4 to 6 % with an fp32 one).
// (A 4-wave kernel with two workgroups per CU and 64-byte K stages, meant to
// hide the epilogue behind the other workgroup's MFMAs, was measured against
// the 256 x 128 tiles: bound by its global->LDS traffic on large problems and
// no faster on these.)
// Few rows of A (M <= 128) take the strip kernel, which streams B once through a
// deep ring.
#pragma once
#include "gemm_skinny.h"
#include "gemm_tile.h"
#include "gemm_tile16.h"

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

// Tile columns to split off a 256 x 256 tiling whose last pass over the tiles would
// leave at least three quarters of the compute units idle (320 tiles on 256
// CUs: one full pass and one of 64 tiles).  Those last columns then run as a second
// launch with 256 x 128 tiles, twice as many for about 0.6 of the time each
// (2048 x 10240 x 8192: 0.156 -> 0.145 ms).  With a last pass that is half
// full the second launch costs what it saves (4096 x 14336 x 4096: 0.177 ms
// either way), so those are left alone.  0: no split.
inline int64_t tail_tile_columns(int64_t M, int64_t N, int64_t batch) {
  const int64_t cus = compute_units();
  const int64_t tm = (M + 255) / 256, tn = (N + 255) / 256;
  const int64_t tiles = tm * tn;
  if (batch != 1 || tiles < cus) return 0;
  const int64_t tail = tiles % cus;
  if (tail == 0 || 4 * tail > cus) return 0;
  const int64_t c = (tail + tm - 1) / tm;  // whole tile columns that hold the tail
  // the rest must still be whole passes, and the split-off part must fit one pass of half tiles
  if (c >= tn || 2 * c * tm > cus + cus / 4) return 0;
  return c;
}

// The same problem restricted to columns [n_off, N) of B and C.
template <bool B_KMAJOR>
GemmArgs columns_from(const GemmArgs& g, int64_t n_off, int64_t batch) {
  GemmArgs t = g;
  const int es = g.out_bf16 ? 2 : 4;
  t.N = g.N - (int)n_off;
  t.B = g.B + (B_KMAJOR ? n_off * g.ldb : n_off);
  t.C = g.C + n_off * es;
  if (g.sb_mode == MI355Q_GS_PER_COL) t.sb = g.sb + n_off;
  if (g.bias_mode != MI355Q_BIAS_NONE) t.bias = g.bias + n_off * es;
  if (g.D) t.D = g.D + n_off * es;
  t.fast_epi = epilogue_fast_ok(t, batch);
  return t;
}

template <bool AK, bool BK_, int FA, int FB>
void launch_256x256(const GemmArgs& g, int64_t batch, hipStream_t st) {
  // the fast bf16 epilogue without an accumulate input: four waves on the 16x16x128 MFMA (gemm_tile16.h)
  if (g.fast_epi && g.D == nullptr) launch_tile16<AK, BK_, FA, FB>(g, batch, st);
  else launch_tile<256, 256, 4, false, AK, BK_, FA, FB>(g, batch, st);
}

template <bool AK, bool BK_, int FA, int FB>
void launch_by_size(const GemmArgs& g, int64_t batch, hipStream_t st) {
  if (g.M > 128 && g.N > 128) {
    switch (choose_tiles(g.M, g.N, batch)) {
      case TileChoice::k256x256: {
        const int64_t c = tail_tile_columns(g.M, g.N, batch);
        if (c == 0) {
          launch_256x256<AK, BK_, FA, FB>(g, batch, st);
        } else {
          const int64_t n_main = ((g.N + 255) / 256 - c) * 256;
          GemmArgs head = g;
          head.N = (int)n_main;
          head.fast_epi = epilogue_fast_ok(head, batch);
          launch_256x256<AK, BK_, FA, FB>(head, batch, st);
          launch_tile<256, 128, 2, false, AK, BK_, FA, FB>(columns_from<BK_>(g, n_main, batch), batch, st);
        }
        break;
      }
      case TileChoice::k256x128: launch_tile<256, 128, 2, false, AK, BK_, FA, FB>(g, batch, st); break;
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
