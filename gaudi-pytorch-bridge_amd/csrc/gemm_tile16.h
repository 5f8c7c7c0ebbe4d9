// The 256 x 256 tile kernel of gemm_tile.h on v_mfma_f32_16x16x128_f8f6f4.
//
// Why a second form of the same tile.  At 8192 x 4096 x 14336 the chip runs this GEMM at its power limit: the same
// kernel takes 0.26 ms on constant operands and 0.34 ms on random bytes, and the clock it holds (1.8 GHz of 2.4)
// is what sets the time, not a stall that a schedule could remove.  Back-to-back MFMAs on register operands that
// change from one instruction to the next sustain 3.8 PFLOP/s as 32x32x64 and 4.3 PFLOP/s as 16x16x128 on random
// bytes (both 4.95 on zeros): the 16x16x128 form does half as many accumulator updates per flop and draws less for
// the same work.  So the large-problem kernel issues that form.
//
// What changes against gemm_tile.h.  A fragment now spans the whole 128-byte K stage: lane group g = lane / 16 holds
// k = 32 g .. 32 g + 31 of row (column) lane % 16, eight registers, and a wave's 128 x 128 tile is 8 x 8 MFMA tiles
// of four accumulator registers each (256 in all, as before).  The 64 MFMAs of a stage run row by row; the A
// fragment of row i is dead after the row's last MFMA and the next stage's is read into the same registers right
// then, the B fragment of column j after the MFMA (7, j): both operands are single-buffered (128 registers).  The
// next stage's fragments are therefore read throughout the current stage, and the LDS stage they come from has to
// be whole early in it: the one barrier of a stage sits a few MFMAs in, the global -> LDS loads of the stage two
// ahead (into the LDS stage whose last fragment reads that barrier has just seen finish) follow it one per two
// MFMAs.  K-major operands are read with two ds_read_b128 per fragment, MN-major ones with four
// ds_read_b64_tr_b8, whose 16-lane groups read k-rows 32 apart: TileGeom's variant 1 keeps them off each other's
// banks.  The accumulator layout puts C[m][n], m = 16 i + lane % 16, n = 16 j + 4 (lane / 16) + e, in register e of
// tile (i, j); the epilogue is the fast bf16 one of gemm_tile.h re-stated for 16-row blocks.
//
// Loaders, the persistent tile walk, the staging of scales and bias through the K loop's own load stream and the
// counting of outstanding stores are those of gemm_tile.h.
#pragma once
#include "gemm_tile.h"

namespace mi355q {

template <bool KMAJOR, int EXT, int TILES>
struct FragReader16 {
  using G = TileGeom<KMAJOR, KMAJOR ? EXT : kBK, KMAJOR ? kBK : EXT, 1>;
  static constexpr int kRowBytes = KMAJOR ? kBK : EXT;
  static constexpr int kStageBytes = EXT * kBK;
  static constexpr int kRegs = KMAJOR ? 2 : TILES;
  static constexpr int kParts = KMAJOR ? 2 : 4;
  static_assert(kStageBytes + (KMAJOR ? (TILES - 1) * 16 * kRowBytes : 24 * kRowBytes) < 65536, "offset field");
  uint32_t addr[kRegs];

  // lds_operand: LDS address of stage 0 of this operand; mn_wave: first row (column) of the wave's tile
  __device__ __forceinline__ void init(uint32_t lds_operand, int mn_wave) {
    const int lane = lane_id_here();
    const int g = lane >> 4, r = lane & 15;
    if constexpr (KMAJOR) {
#pragma unroll
      for (int part = 0; part < 2; ++part) addr[part] = lds_operand + G::lds_offset(mn_wave + r, 2 * g + part);
    } else {
      // lanes 2 r' and 2 r' + 1 of a 16-lane group point at the two 8-byte halves of k-row 32 g + 8 part + r'; after
      // the transposing read lane i of the group holds column i for those 8 k-rows
      const int rr = r >> 1, h = r & 1;
#pragma unroll
      for (int t = 0; t < TILES; ++t) addr[t] = lds_operand + G::lds_offset(32 * g + rr, (mn_wave + 16 * t) >> 4) + h * 8;
    }
  }

  // Part PART of the fragment of 16-row (column) tile T from stage STAGE.
  template <int T, int PART, int STAGE>
  __device__ __forceinline__ void read(i32x8& f) const {
    if constexpr (KMAJOR) {
      constexpr int off = STAGE * kStageBytes + T * 16 * kRowBytes;
      const u32x4 v = *reinterpret_cast<LDS_AS const u32x4*>(addr[PART] + off);
      f[4 * PART + 0] = v[0];
      f[4 * PART + 1] = v[1];
      f[4 * PART + 2] = v[2];
      f[4 * PART + 3] = v[3];
    } else {
      constexpr int off = STAGE * kStageBytes + PART * 8 * kRowBytes;
      const i32x2 t = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<LDS_AS i32x2*>(addr[T] + off));
      f[2 * PART] = t[0];
      f[2 * PART + 1] = t[1];
    }
  }
};

// The fast bf16 epilogue (scalar or per-row A scale, scalar or per-column B scale, optional bias vector; scales and
// bias already in the wave's staging area, see ScaleStager) for the accumulator layout of the 16x16x128 MFMA.
// Sixteen rows at a time pass through the staging area as 16 rows of 256 bytes: a lane writes its four columns of
// tile (i, j) as 8 bytes into slot (4 j + lane / 16) ^ (2 (lane % 16)) of row lane % 16 (the 32 lanes of a write
// cycle hit 32 different slots), and reads back 16 bytes at chunk (lane % 16) ^ row of row 4 p + lane / 16 (an even
// XOR keeps the two halves of a chunk together and in order), so that a wave stores four whole rows of its tile per
// instruction.
template <int MT, int NT, bool PER_COL, bool HAS_BIAS>
__device__ __forceinline__ void epilogue16_bf16_fast(const GemmArgs& g, int64_t batch, f32x4 (&acc)[MT][NT], int m_wave,
                                                     int n_wave, float* stage_f, ScalarScales scalars) {
  static_assert(NT == 8 && MT * 4 == fast_epilogue_stores<MT / 2, NT / 2>(), "256-byte rows; the K loop counts these stores");
  LDS_AS uint8_t* stage = (LDS_AS uint8_t*)stage_f;
  const int lane = lane_id_here();
  const int r = lane & 15, gq = lane >> 4;
  const float sa_s = scalars.sa, sb_s = scalars.sb;
  float cs[PER_COL ? NT : 1][4], cb[HAS_BIAS ? NT : 1][4];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int col = 16 * j + 4 * gq;  // inside the wave's tile
    if constexpr (PER_COL) {
      const f32x4 v = *reinterpret_cast<LDS_AS const f32x4*>(stage + kStagedColScale + col * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) cs[j][e] = v[e];
    }
    if constexpr (HAS_BIAS) {
      const u32x2 v = *reinterpret_cast<LDS_AS const u32x2*>(stage + kStagedBias + col * 2);
      cb[j][0] = __uint_as_float(v[0] << 16);
      cb[j][1] = __uint_as_float(v[0] & 0xffff0000u);
      cb[j][2] = __uint_as_float(v[1] << 16);
      cb[j][3] = __uint_as_float(v[1] & 0xffff0000u);
    }
  }
  float ra[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const float staged = *reinterpret_cast<LDS_AS const float*>(stage + kStagedRowScale + (16 * i + r) * 4);
    ra[i] = g.sa_mode == MI355Q_GS_PER_ROW ? staged : sa_s;
    if (!PER_COL) ra[i] *= sb_s;
  }
  // the staged values sit where the rows are about to pass through
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_sched_barrier(0);

  const int rows = g.M - m_wave < 16 * MT ? g.M - m_wave : 16 * MT;
  uint16_t* cbase = reinterpret_cast<uint16_t*>(g.C) + batch * g.stride_c + (int64_t)m_wave * g.ldc;
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(cbase, 0, rows > 0 ? rows * (int)g.ldc * 2 : 0, 0x00020000);
  const int n_out = n_wave + 8 * r;
  const int pitch = (int)g.ldc * 2;
  const int voff0 = n_out < g.N ? gq * pitch + n_out * 2 : 0x7fffffff;  // columns at or beyond N: an offset no descriptor reaches
  const int pass_step = n_out < g.N ? 4 * pitch : 0;

  auto write_rows = [&](auto ic) {
    constexpr int i = decltype(ic)::value;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float b = HAS_BIAS ? cb[j][e] : 0.0f;
        if constexpr (PER_COL) v[e] = __builtin_fmaf(acc[i][j][e] * ra[i], cs[j][e], b);
        else v[e] = __builtin_fmaf(acc[i][j][e], ra[i], b);
      }
      const u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
      const int slot = (4 * j + gq) ^ (2 * r);
      *reinterpret_cast<LDS_AS u32x2*>(stage + r * 256 + slot * 8) = o;
    }
  };
  auto read_rows = [&](u32x4 (&o)[4]) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int row = 4 * p + gq;
      o[p] = *reinterpret_cast<LDS_AS u32x4*>(stage + row * 256 + ((r ^ row) << 4));
    }
  };
  // a wave's LDS instructions execute in the order issued: the values of rows i + 1 are written as soon as the reads
  // of rows i have been issued, and the stores of rows i follow without a wait
  u32x4 o[4];
  write_rows(std::integral_constant<int, 0>{});
  read_rows(o);
  static_for<MT>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (i + 1 < MT) write_rows(std::integral_constant<int, i + 1>{});
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int p = 0; p < 4; ++p)
      __builtin_amdgcn_raw_buffer_store_b128(o[p], rsrc, voff0 + (i * 4 + p) * pass_step, 0, 2);  // aux 2: nontemporal
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (i + 1 < MT) read_rows(o);
  });
}

template <int MT, int NT>
__device__ __forceinline__ void epilogue16_bf16_fast_any(const GemmArgs& g, int64_t batch, f32x4 (&acc)[MT][NT], int m_wave,
                                                         int n_wave, float* stage, ScalarScales scalars) {
  const bool per_col = g.sb_mode == MI355Q_GS_PER_COL, bias = g.bias_mode == MI355Q_BIAS_ROW_VECTOR;
  if (per_col && bias) epilogue16_bf16_fast<MT, NT, true, true>(g, batch, acc, m_wave, n_wave, stage, scalars);
  else if (per_col) epilogue16_bf16_fast<MT, NT, true, false>(g, batch, acc, m_wave, n_wave, stage, scalars);
  else if (bias) epilogue16_bf16_fast<MT, NT, false, true>(g, batch, acc, m_wave, n_wave, stage, scalars);
  else epilogue16_bf16_fast<MT, NT, false, false>(g, batch, acc, m_wave, n_wave, stage, scalars);
}

// Per-wave state of the K loop: 2 x 2 waves on a 256 x 256 tile, one per SIMD.
// LEAN: K is a whole number of pairs of stages (K % 256 == 0), so that no stage has lanes past K, and each operand
// spans less than DmaLoader::kNarrowBytes: the loads then need no per-lane test, four of them share a write of m0,
// and a step along K is one scalar addition per operand.  The K loop of the general form spends 93 instructions per
// stage besides its 64 MFMAs and 48 LDS reads, this one 30; on a SIMD that issues for one wave that is 4 % of the
// run time of a 8192 x 4096 x 14336 product.
template <bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B, bool LEAN>
struct TileCore16 {
  static constexpr int BM = 256, BN = 256, kWaves = 4;
  static constexpr int MT = 8, NT = 8;  // 16 x 16 MFMA tiles of the wave's 128 x 128
  using LoaderA = DmaLoader<A_KMAJOR, BM, kBK, kWaves, 1>;
  using LoaderB = DmaLoader<B_KMAJOR, BN, kBK, kWaves, 1>;
  using ReaderA = FragReader16<A_KMAJOR, BM, MT>;
  using ReaderB = FragReader16<B_KMAJOR, BN, NT>;
  static constexpr int kStageA = BM * kBK, kStageB = BN * kBK;
  static constexpr int kRingBytes = 2 * (kStageA + kStageB);
  static constexpr int kPartsA = ReaderA::kParts, kPartsB = ReaderB::kParts;
  static constexpr int kMfmas = MT * NT;
  static constexpr int kDmaOps = LoaderA::kPerWave + LoaderB::kPerWave;
  static constexpr int kBarrierAt = 3;  // the stage's barrier follows this MFMA
  static_assert(kBarrierAt < NT - 1 && kBarrierAt + 2 * kDmaOps < kMfmas, "reads and loads of a stage follow its barrier");
  f32x4 acc[MT][NT];
  i32x8 fa[MT], fb[NT];
  LoaderA la;
  LoaderB lb;
  ReaderA ra;
  ReaderB rb;
  uint8_t* ring;
  int wave, wm, wn, K;

  __device__ __forceinline__ void init(const GemmArgs& g, uint8_t* ring_, int wave_, int wm_, int wn_) {
    ring = ring_;
    wave = wave_;
    wm = wm_;
    wn = wn_;
    K = g.K;
  }
  __device__ __forceinline__ void set_lane_addresses(const GemmArgs& g) {
    const uint32_t base = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)ring;
    ra.init(base, wm);
    rb.init(base + 2 * kStageA, wn);
    la.set_lane_offsets(g.lda, wave);
    lb.set_lane_offsets(g.ldb, wave);
  }
  __device__ __forceinline__ void retarget(const GemmArgs& g, int64_t batch, int m0, int n0, bool valid) {
    la.set_tile(g.A + batch * g.stride_a, g.lda, m0, g.M, g.K, valid);
    lb.set_tile(g.B + batch * g.stride_b, g.ldb, n0, g.N, g.K, valid);
  }
  template <int OP, int STAGE>
  __device__ __forceinline__ void dma_op(int kt) {
    constexpr int na = LoaderA::kPerWave;
    if constexpr (OP < na) la.template issue_one<OP, false, false, !LEAN>(ring + STAGE * kStageA, kt * kBK, K);
    else lb.template issue_one<OP - na, false, false, !LEAN>(ring + 2 * kStageA + STAGE * kStageB, kt * kBK, K);
  }
  __device__ __forceinline__ void step_descriptors() {
    if constexpr (LEAN) {
      la.advance_narrow();
      lb.advance_narrow();
    } else {
      la.advance();
      lb.advance();
    }
  }
  template <int STAGE>
  __device__ __forceinline__ void issue_stage(int kt) {
    static_for<kDmaOps>([&](auto oc) { dma_op<decltype(oc)::value, STAGE>(kt); });
    step_descriptors();
  }

  static constexpr int kEpilogueStores = MT * 4;
  static_assert(kEpilogueStores < 64, "vmcnt holds 6 bits");
  // see TileCore::wait_loads_then_barrier
  __device__ __forceinline__ static void wait_loads_then_barrier(bool younger_stores = false) {
    if (younger_stores) __builtin_amdgcn_s_waitcnt((kEpilogueStores & 15) | ((kEpilogueStores >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  }

  // All fragments of a tile's first stage (ring stage 0), whose loads have been issued.
  __device__ __forceinline__ void first_fragments(bool younger_stores) {
    wait_loads_then_barrier(younger_stores);
    static_for<MT>([&](auto ic) {
      static_for<kPartsA>([&](auto pc) { ra.template read<decltype(ic)::value, decltype(pc)::value, 0>(fa[decltype(ic)::value]); });
    });
    static_for<NT>([&](auto jc) {
      static_for<kPartsB>([&](auto pc) { rb.template read<decltype(jc)::value, decltype(pc)::value, 0>(fb[decltype(jc)::value]); });
    });
  }

  // One K stage of MFMAs on the fragments in registers.  They came from ring stage CUR; the next K stage sits in
  // ring stage 1 - CUR, or is still landing there until this stage's barrier.  After the barrier every wave has read
  // all of CUR, so the K stage two ahead (dma_kt) starts to overwrite it, and the next stage's fragments replace
  // this stage's as they die.  after_barrier: hook for the tile's first stage (other loads its later waits cover).
  template <int CUR, bool ZERO_C, typename F>
  __device__ __forceinline__ void stage(int dma_kt, bool younger_stores, F&& after_barrier) {
    constexpr int NXT = 1 - CUR;
    static_for<kMfmas>([&](auto gc) {
      constexpr int gi = decltype(gc)::value;
      constexpr int i = gi / NT, j = gi % NT;
      const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
      acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[i], ZERO_C ? zero : acc[i][j], mfma_code<FMT_B>(),
                                                                    mfma_code<FMT_A>(), 0, 0, 0, 0);
      if constexpr (gi == kBarrierAt) {
        wait_loads_then_barrier(younger_stores);
        after_barrier();
      }
      if constexpr (gi > kBarrierAt && (gi - kBarrierAt - 1) % 2 == 0 && (gi - kBarrierAt - 1) / 2 < kDmaOps)
        dma_op<(gi - kBarrierAt - 1) / 2, CUR>(dma_kt);
      if constexpr (j == NT - 1)  // row i is done: its A fragment is dead
        static_for<kPartsA>([&](auto pc) { ra.template read<i, decltype(pc)::value, NXT>(fa[i]); });
      if constexpr (i == MT - 1)  // column j is done
        static_for<kPartsB>([&](auto pc) { rb.template read<j, decltype(pc)::value, NXT>(fb[j]); });
      __builtin_amdgcn_sched_barrier(0);
    });
    step_descriptors();
  }
};

template <bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B, bool LEAN>
__global__ __launch_bounds__(256) void fp8_gemm_tile16_kernel(GemmArgs g) {
  using Core = TileCore16<A_KMAJOR, B_KMAJOR, FMT_A, FMT_B, LEAN>;
  constexpr int BM = Core::BM, BN = Core::BN, MT = Core::MT, NT = Core::NT;
  __shared__ __attribute__((aligned(1024))) uint8_t lds_ring[Core::kRingBytes];
  __shared__ __attribute__((aligned(16))) float lds_epi[4 * epilogue_stage_floats<4, 4>()];

  const int nb = gridDim.x, bid = blockIdx.x;
  const int tiles = g.tiles_m * g.tiles_n;
  const int xcd = bid & 7, slot = bid >> 3;
  const int slots = (nb - xcd + 7) >> 3;
  const int per = tiles >> 3, rem = tiles & 7;
  const int first = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
  const int count = per + (xcd < rem ? 1 : 0);

  const int64_t batch = blockIdx.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;
  float* stage = lds_epi + wave * epilogue_stage_floats<4, 4>();

  Core core;
  core.init(g, lds_ring, wave, wm, wn);
  const int KT = (g.K + kBK - 1) / kBK;
  const int KT2 = (KT + 1) & ~1;  // stages past K arrive as zeros: an even number of branch-free stages

  int idx = slot;
  if (idx >= count) return;
  int tile_m, tile_n;
  tile_coords(first + idx, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
  core.set_lane_addresses(g);
  core.retarget(g, batch, tile_m * BM, tile_n * BN, true);
  core.template issue_stage<0>(0);
  core.template issue_stage<1>(1);
  const ScalarScales scalars = load_scalar_scales(g);
  bool stores_pending = false;
  // Only the first tile reads its first fragments here: the last K stage of a tile replaces its fragments, as they
  // die, by those of ring stage 0 like every other stage, and what sits there by then is the next tile's first stage.
  // (Not with both operands K-major: the registers do not hold the fragments across the epilogue there, and the
  // spills cost more than reading them again.)
  constexpr bool kKeepFragments = !(A_KMAJOR && B_KMAJOR);
  if constexpr (kKeepFragments) core.first_fragments(false);
  for (;;) {
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    if constexpr (!kKeepFragments) core.first_fragments(stores_pending);
    auto k_pair = [&](auto first_c, int kt) {
      constexpr bool FIRST = decltype(first_c)::value;
      const bool last = kt + 2 == KT2;
      if (last) {  // the loads this pair issues are the next tile's first two stages
        idx += slots;
        const bool more = idx < count;
        if (more) tile_coords(first + idx, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
        core.retarget(g, batch, tile_m * BM, tile_n * BN, more);
      }
      const int dk = last ? 0 : kt + 2;
      // stage 1 of a tile is as old as stage 0: its wait, too, leaves the previous tile's stores outstanding
      core.template stage<0, FIRST>(dk, FIRST && stores_pending, [&] {
        if constexpr (FIRST) ScaleStager::issue<4, 4>(g, batch, m0 + wm, n0 + wn, stage);
      });
      core.template stage<1, false>(dk + 1, false, [] {});
    };
    k_pair(std::true_type{}, 0);
    for (int kt = 2; kt < KT2; kt += 2) k_pair(std::false_type{}, kt);
    epilogue16_bf16_fast_any<MT, NT>(g, batch, core.acc, m0 + wm, n0 + wn, stage, scalars);
    stores_pending = m0 + BM <= g.M && n0 + BN <= g.N;
    if (idx >= count) break;
    core.set_lane_addresses(g);
  }
  __builtin_amdgcn_s_waitcnt(0);
}

// The launch must satisfy epilogue_fast_ok() and have no accumulate input.
template <bool AK, bool BK_, int FA, int FB>
void launch_tile16(const GemmArgs& g, int64_t batch, hipStream_t st) {
  GemmArgs a = g;
  a.tiles_m = (g.M + 255) / 256;
  a.tiles_n = (g.N + 255) / 256;
  const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
  const int cus = compute_units();
  dim3 grid((unsigned)(tiles < cus ? tiles : cus), (unsigned)batch);
  // bytes from an operand's first element to the end of what a descriptor on it may cover (see DmaLoader::set_tile)
  const int64_t span_a = AK ? (int64_t)(g.M - 1) * g.lda + g.K : (int64_t)(g.K - 1) * g.lda + ((g.M + 15) & ~15);
  const int64_t span_b = BK_ ? (int64_t)(g.N - 1) * g.ldb + g.K : (int64_t)(g.K - 1) * g.ldb + ((g.N + 15) & ~15);
  constexpr int64_t narrow = DmaLoader<true, 256, kBK, 4, 1>::kNarrowBytes;
  const bool lean = g.K % (2 * kBK) == 0 && span_a < narrow && span_b < narrow;
  if (lean) fp8_gemm_tile16_kernel<AK, BK_, FA, FB, true><<<grid, 256, 0, st>>>(a);
  else fp8_gemm_tile16_kernel<AK, BK_, FA, FB, false><<<grid, 256, 0, st>>>(a);
}

}  // namespace mi355q
