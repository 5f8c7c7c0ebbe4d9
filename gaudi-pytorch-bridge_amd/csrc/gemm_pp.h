// Two-workgroups-per-CU variant of the tiled fp8 GEMM for large problems.
//
// The 8-wave kernel of gemm_tile.h leaves the matrix pipes idle while a
// workgroup runs its epilogue (all waves of a CU reach it together).  Here a
// workgroup is 4 waves (one per SIMD) on a 256 x 128 tile with 64-byte K
// stages, small enough in LDS that two workgroups share a CU: while one
// converts and stores its tile, or waits at a barrier or for its first stages,
// the other one's MFMAs keep the pipes busy.  The workgroups of the second
// half of the grid start half a tile late, so that the two residents of a CU
// reach their epilogues at different times.
//
// Per workgroup: three LDS stages of (256 + 128) x 64 bytes in a ring.  In the
// step that computes stage k the wave reads the fragments of stage k+1 and
// issues its global->LDS loads of stage k+3 into the buffer that held stage k
// (free since the barrier at the top of the step).  The epilogue's staging
// area overlays the stage ring, which is idle by then; nothing is prefetched
// across tiles, the other workgroup covers that gap.
#pragma once
#include "gemm_skinny.h"
#include "gemm_tile.h"

namespace mi355q {

constexpr int kPpThreads = 256;
constexpr int kPpWaves = 4;
constexpr int kPpWavesM = 2, kPpWavesN = 2;
constexpr int kPpBK = 64;

template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
struct PpCore {
  static constexpr int TM = BM / kPpWavesM, TN = BN / kPpWavesN;
  static constexpr int MT = TM / 32, NT = TN / 32;
  static constexpr int kStageBytes = (BM + BN) * kPpBK;
  using LA = DmaLoader<A_KMAJOR, BM, kPpBK, kPpWaves>;
  using LB = DmaLoader<B_KMAJOR, BN, kPpBK, kPpWaves>;
  static constexpr int kPartsA = frag_parts<A_KMAJOR>(), kPartsB = frag_parts<B_KMAJOR>();
  static constexpr int kMfmas = MT * NT;
  static constexpr int kDmaOps = LA::kPerWave + LB::kPerWave;

  f32x16 acc[MT][NT];
  i32x8 fa[MT], fb0[NT], fb1[NT];
  LA la;
  LB lb;
  int wm, wn, K;

  __device__ __forceinline__ void zero_acc() {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  }

  __device__ __forceinline__ void retarget(const GemmArgs& g, int64_t batch, int m0, int n0) {
    la.init(g.A + batch * g.stride_a, g.lda, m0, g.M, g.K);
    lb.init(g.B + batch * g.stride_b, g.ldb, n0, g.N, g.K);
  }

  template <int I, int PART>
  __device__ __forceinline__ void read_a(const uint8_t* stage) {
    read_fragment_part<A_KMAJOR, BM, PART, kPpBK>(stage, wm + I * 32, 0, fa[I]);
  }
  template <int J, int PART>
  __device__ __forceinline__ void read_b(const uint8_t* stage, i32x8 (&fb)[NT]) {
    read_fragment_part<B_KMAJOR, BN, PART, kPpBK>(stage + BM * kPpBK, wn + J * 32, 0, fb[J]);
  }

  template <int OP>
  __device__ __forceinline__ void dma_op(uint8_t* stage, int kt) {
    constexpr int na = LA::kPerWave;
    if constexpr (OP < na) la.template issue_one<OP>(stage, kt * kPpBK, K);
    else lb.template issue_one<OP - na>(stage + BM * kPpBK, kt * kPpBK, K);
  }

  __device__ __forceinline__ void issue_stage(uint8_t* stage, int kt) {
    static_for<kDmaOps>([&](auto oc) { dma_op<decltype(oc)::value>(stage, kt); });
    la.advance();
    lb.advance();
  }

  // One step: the MFMAs of the stage whose fragments sit in (fa, cb), the
  // fragment reads of the next stage from rd_stage, and the global->LDS loads
  // of stage dma_kt into dma_stage, dealt out between the MFMAs.  Stages at or
  // beyond K are loaded all the same (they fall outside the buffer descriptors
  // and arrive as zeros), which keeps the K loop free of branches.
  __device__ __forceinline__ void step(const i32x8 (&cb)[NT], i32x8 (&nb)[NT], const uint8_t* rd_stage,
                                       uint8_t* dma_stage, int dma_kt) {
    constexpr int kBOps = NT * kPartsB;
    constexpr int kBPerGroup = (kBOps + kMfmas - 1) / kMfmas;
    constexpr int kDmaPerGroup = (kDmaOps + kMfmas - 1) / kMfmas;
    static_for<kMfmas>([&](auto gc) {
      constexpr int gi = decltype(gc)::value;
      constexpr int i = gi / NT, j = gi % NT;
      acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
          cb[j], fa[i], acc[i][j], mfma_code<FMT_B>(), mfma_code<FMT_A>(), 0, 0, 0, 0);
      static_for<kDmaPerGroup>([&](auto dc) {
        constexpr int op = gi * kDmaPerGroup + decltype(dc)::value;
        if constexpr (op < kDmaOps) dma_op<op>(dma_stage, dma_kt);
      });
      static_for<kBPerGroup>([&](auto rc) {
        constexpr int op = gi * kBPerGroup + decltype(rc)::value;
        if constexpr (op < kBOps) read_b<op / kPartsB, op % kPartsB>(rd_stage, nb);
      });
      if constexpr (j == NT - 1) {
        static_for<kPartsA>([&](auto pc) { read_a<i, decltype(pc)::value>(rd_stage); });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    la.advance();
    lb.advance();
  }
};

// s_waitcnt with vmcnt = N, lgkmcnt = 0, expcnt untouched (gfx9 encoding:
// vmcnt low bits [3:0], expcnt [6:4], lgkmcnt [11:8], vmcnt high bits [15:14]).
template <int N>
__device__ __forceinline__ void wait_vm_lgkm() {
  static_assert(N >= 0 && N <= 63, "vmcnt field");
  __builtin_amdgcn_s_waitcnt(0x0070 | (N & 15) | ((N >> 4) << 14));
}

// S: stages in the ring.  3 lets two workgroups share a CU's LDS; a launch with
// no more workgroups than CUs takes 6, to keep more bytes in flight per CU.
template <int BM, int BN, int S, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
__global__ __launch_bounds__(kPpThreads, 2) void fp8_gemm_pp_kernel(GemmArgs g, int late_from) {
  using Core = PpCore<BM, BN, A_KMAJOR, B_KMAJOR, FMT_A, FMT_B>;
  constexpr int MT = Core::MT, NT = Core::NT;
  constexpr int kStageBytes = Core::kStageBytes;
  static_assert(kPpWaves * epilogue_stage_floats<MT, NT>() * 4 <= S * kStageBytes, "epilogue area overlays the ring");
  static_assert(S >= 3 && (S - 2) * Core::kDmaOps <= 63, "per-step wait");
  constexpr int kRing = S * kStageBytes;
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kRing];

  const int nb = gridDim.x, bid = blockIdx.x;
  const int tiles = g.tiles_m * g.tiles_n;
  const int xcd = bid & 7, slot = bid >> 3;
  const int slots = (nb - xcd + 7) >> 3;
  const int per = tiles >> 3, rem = tiles & 7;
  const int first = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
  const int count = per + (xcd < rem ? 1 : 0);
  if (slot >= count) return;

  const int64_t batch = blockIdx.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float* stage_area = reinterpret_cast<float*>(lds) + wave * epilogue_stage_floats<MT, NT>();
  const bool fast_epilogue = epilogue_fast_ok(g, batch);

  Core core;
  core.wm = (wave / kPpWavesN) * Core::TM;
  core.wn = (wave % kPpWavesN) * Core::TN;
  core.K = g.K;
  const int KT = (g.K + kPpBK - 1) / kPpBK;
  const int KT2 = (KT + 1) & ~1;  // an odd stage count runs one step of zero products

  // The second resident of a CU starts half a tile late (a K stage of the tile
  // is MT*NT MFMAs of 64 cycles per wave).
  if (bid >= late_from) {
    for (int i = 0; i < KT; ++i) __builtin_amdgcn_s_sleep(MT * NT / 2);
  }

  for (int idx = slot; idx < count; idx += slots) {
    int tile_m, tile_n;
    tile_coords(first + idx, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    core.retarget(g, batch, m0, n0);
    // stage s lives in buffer s % S; o_cur is the buffer of the stage being computed
    int o_cur = 0;
#pragma unroll
    for (int s = 0; s < S; ++s) core.issue_stage(lds + s * kStageBytes, s);  // stages at or beyond K arrive as zeros
    core.zero_acc();
    // stores of the previous epilogue share the counter: wait for everything once
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    static_for<MT>([&](auto ic) {
      static_for<Core::kPartsA>([&](auto pc) { core.template read_a<decltype(ic)::value, decltype(pc)::value>(lds + o_cur); });
    });
    static_for<NT>([&](auto jc) {
      static_for<Core::kPartsB>([&](auto pc) { core.template read_b<decltype(jc)::value, decltype(pc)::value>(lds + o_cur, core.fb0); });
    });
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the first fragments are in registers
    // At the top of a step the loads of the next stage are complete (this wave
    // has waited for its own, the barrier covers the others') and every wave has
    // read the fragments of the current stage, whose buffer the step refills
    // with the stage S ahead.  After a step the wave's outstanding loads are
    // those of the stages after the next one, oldest first: the stage needed
    // next is complete once only (S - 2) stages' worth remain.
    auto next = [&](int o) { return o + kStageBytes == kRing ? 0 : o + kStageBytes; };
    for (int kt = 0; kt < KT2; kt += 2) {
      const int o_nxt = next(o_cur);
      __syncthreads();
      core.step(core.fb0, core.fb1, lds + o_nxt, lds + o_cur, kt + S);
      wait_vm_lgkm<(S - 2) * Core::kDmaOps>();
      const int o_nn = next(o_nxt);
      __syncthreads();
      core.step(core.fb1, core.fb0, lds + o_nn, lds + o_nxt, kt + S + 1);
      wait_vm_lgkm<(S - 2) * Core::kDmaOps>();
      o_cur = o_nn;
    }
    // every wave is done with the ring (its last fragment reads included) before it is overlaid
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (fast_epilogue) {
      if (g.sb_mode == MI355Q_GS_PER_COL) epilogue_bf16_fast<MT, NT, true>(g, batch, core.acc, m0 + core.wm, n0 + core.wn, stage_area);
      else epilogue_bf16_fast<MT, NT, false>(g, batch, core.acc, m0 + core.wm, n0 + core.wn, stage_area);
    } else {
      epilogue<MT, NT>(g, batch, core.acc, m0 + core.wm, n0 + core.wn, stage_area);
    }
    // the next tile's loads overwrite the staging areas of all waves
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's LDS reads are done
    __syncthreads();
  }
}

// The two-workgroup kernel moves 1.5 times the bytes from L2 into LDS per flop
// (its tile is half as wide), which is what bounds it on large problems; it
// wins where the 256 x 256 tiling would leave compute units without a tile.
inline bool use_pp_kernel(int64_t M, int64_t N, int64_t batch) {
  const int64_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256) * batch;
  return tiles256 < compute_units();
}

template <int BM, int BN, bool AK, bool BK_, int FA, int FB>
void launch_pp(const GemmArgs& g, int64_t batch, hipStream_t st) {
  GemmArgs a = g;
  a.tiles_m = (g.M + BM - 1) / BM;
  a.tiles_n = (g.N + BN - 1) / BN;
  const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
  const int cus = compute_units();
  const int64_t wgs = tiles < 2 * cus ? tiles : 2 * cus;
  dim3 grid((unsigned)wgs, (unsigned)batch);
  if (wgs * batch <= cus) {
    fp8_gemm_pp_kernel<BM, BN, 6, AK, BK_, FA, FB><<<grid, kPpThreads, 0, st>>>(a, (int)wgs);
  } else {
    // workgroups are placed breadth first: those beyond the CU count are second residents
    fp8_gemm_pp_kernel<BM, BN, 3, AK, BK_, FA, FB><<<grid, kPpThreads, 0, st>>>(a, cus);
  }
}

template <bool AK, bool BK_, int FA, int FB>
void launch_by_size(const GemmArgs& g, int64_t batch, hipStream_t st) {
  if (g.M > 128 && g.N > 128) {
    if (use_pp_kernel(g.M, g.N, batch)) launch_pp<256, 128, AK, BK_, FA, FB>(g, batch, st);
    else launch_tile<256, 256, AK, BK_, FA, FB>(g, batch, st);
  } else if (g.M <= 128) {
    launch_skinny_by_m<AK, BK_, FA, FB>(g, batch, st);
  } else {
    launch_tile<128, 128, AK, BK_, FA, FB>(g, batch, st);
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
