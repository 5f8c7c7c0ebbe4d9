// fp8 GEMM for few rows of A (M <= 128: decode-shaped calls).
//
// These problems are bound by streaming B from HBM once: what matters is how
// many bytes each compute unit keeps in flight, not the MFMA schedule.  One
// 4-wave workgroup owns a strip of 128 columns of C for all M rows and walks K
// in 128-byte stages through a ring of S LDS buffers, S as large as the 160 KB
// of LDS allow (8 for BM = 32: up to seven stages, 112 KB of B per compute
// unit, are on their way from memory while one is being multiplied).  Each wave
// multiplies the whole A tile by its own 32 columns; fragments are read right
// before use (the matrix pipes are mostly idle anyway).
//
// The global->LDS loads, LDS geometry, fragment reads and epilogues are those
// of the large-tile kernel (gemm_tile.h).
#pragma once
#include "gemm_tile.h"

namespace mi355q {

constexpr int kSkThreads = 256;
constexpr int kSkWaves = 4;
constexpr int kSkBN = 128;

template <int BM>
constexpr int skinny_stages() {
  constexpr int stage = (BM + kSkBN) * kBK;
  constexpr int s = (160 * 1024) / stage;
  return s > 8 ? 8 : s;
}

template <int BM, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
__global__ __launch_bounds__(kSkThreads) void fp8_gemm_skinny_kernel(GemmArgs g) {
  constexpr int MT = BM / 32;
  constexpr int S = skinny_stages<BM>();
  constexpr int kStageBytes = (BM + kSkBN) * kBK;
  using LA = DmaLoader<A_KMAJOR, BM, kBK, kSkWaves>;
  using LB = DmaLoader<B_KMAJOR, kSkBN, kBK, kSkWaves>;
  constexpr int kOps = LA::kPerWave + LB::kPerWave;
  constexpr int kInFlight = (S - 2) * kOps;  // loads that may stay outstanding while stage kt is consumed
  static_assert(S >= 3 && kInFlight <= 63, "vmcnt holds 6 bits");
  static_assert(kSkWaves * epilogue_stage_floats<MT, 1>() * 4 <= S * kStageBytes, "epilogue area overlays the ring");
  constexpr int kPartsA = frag_parts<A_KMAJOR>(), kPartsB = frag_parts<B_KMAJOR>();
  __shared__ __attribute__((aligned(1024))) uint8_t lds[S * kStageBytes];

  const int64_t batch = blockIdx.y;
  const int n0 = blockIdx.x * kSkBN;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wn = wave * 32;

  LA la;
  LB lb;
  la.init(g.A + batch * g.stride_a, g.lda, 0, g.M, g.K);
  lb.init(g.B + batch * g.stride_b, g.ldb, n0, g.N, g.K);
  // rows of the tiles past M or N: loads that go to memory (see DmaLoader::clamp_rows)
  if constexpr (A_KMAJOR) la.clamp_rows(g.lda, g.M);
  if constexpr (B_KMAJOR) lb.clamp_rows(g.ldb, g.N - n0);
  f32x16 acc[MT][1];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][0][e] = 0.0f;

  const int KT = (g.K + kBK - 1) / kBK;
  // K is walked from a stage that depends on the strip, wrapping around, when B
  // is K-major: its rows are K bytes apart, so workgroups that all read the same
  // k at the same time send their requests, which differ only in high address
  // bits, to the same few memory channels.  (With B MN-major the strips of one
  // k row are contiguous in memory and walking in step is the better order.)
  // (Not with an MN-major A and a ragged K: the stage that holds the K tail then has loads that
  // fall outside A's descriptor altogether, and the counted waits below need it to be the last.)
  const int first = (B_KMAJOR && (A_KMAJOR || g.K % kBK == 0)) ? (int)(((int64_t)blockIdx.x * KT) / gridDim.x) : 0;
  int at = 0;  // the stage the loaders' descriptors point at
  // Issues the loads of the i-th stage in walking order; beyond the KT-th they
  // fall outside the descriptors and arrive as zeros, so that every step issues
  // and waits alike.
  auto issue_stage = [&](int off, int i) {
    int stage = first + i;
    if (stage >= KT) stage -= KT;
    if (i >= KT) stage = KT;  // out of range
    if (stage != at) {
      la.seek(at, stage);
      lb.seek(at, stage);
      at = stage;
    }
    static_for<LA::kPerWave>([&](auto ic) { la.template issue_one<decltype(ic)::value, A_KMAJOR>(lds + off, stage * kBK, g.K); });
    static_for<LB::kPerWave>([&](auto ic) { lb.template issue_one<decltype(ic)::value, B_KMAJOR, true>(lds + off + BM * kBK, stage * kBK, g.K); });  // B is read once
    la.advance();
    lb.advance();
    ++at;
  };

  // waits until at most min(later, S - 2) stages' loads of this wave are outstanding
  auto wait_for_stage = [&](int later) {
    static_for<S - 1>([&](auto sc) {
      constexpr int n = decltype(sc)::value;  // 0 .. S - 2
      constexpr int cnt = n * kOps;
      if (later == n || (n == S - 2 && later > n) || (n == 0 && later < 0))
        __builtin_amdgcn_s_waitcnt((cnt & 15) | ((cnt >> 4) << 14) | 0x0070);
    });
  };

  // stages 0 .. S-2 (in walking order) go out first
#pragma unroll
  for (int s = 0; s < S - 1; ++s) issue_stage(s * kStageBytes, s);

  int rd_off = 0;                        // buffer of stage kt
  int wr_off = (S - 1) * kStageBytes;    // buffer of stage kt + S - 1 (the one stage kt - 1 used)
  for (int kt = 0; kt < KT; ++kt) {
    // This wave's part of stage kt has landed once only the loads of the later stages are
    // outstanding: the counter retires loads that go to memory in issue order.  A load whose
    // lanes are all out of range completes at once, ahead of older ones, so it must not be
    // counted.  Such loads are those of the stages past K and, in the last stage, of k rows
    // (MN-major) past K: towards the end only the stages up to KT - 2 are counted.
    wait_for_stage(KT - 2 - kt);
    __syncthreads();  // everyone's part has; and everyone is done with the buffer of stage kt - 1
    issue_stage(wr_off, kt + S - 1);
    const uint8_t* st = lds + rd_off;
#pragma unroll
    for (int ks = 0; ks < kBK / 64; ++ks) {
      i32x8 fb, fa[MT];
      static_for<kPartsB>([&](auto pc) {
        read_fragment_part<B_KMAJOR, kSkBN, decltype(pc)::value>(st + BM * kBK, wn, ks, fb);
      });
      static_for<MT>([&](auto ic) {
        static_for<kPartsA>([&](auto pc) {
          read_fragment_part<A_KMAJOR, BM, decltype(pc)::value>(st, decltype(ic)::value * 32, ks, fa[decltype(ic)::value]);
        });
      });
      static_for<MT>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        acc[i][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
            fb, fa[i], acc[i][0], mfma_code<FMT_B>(), mfma_code<FMT_A>(), 0, 0, 0, 0);
      });
    }
    rd_off += kStageBytes;
    if (rd_off == S * kStageBytes) rd_off = 0;
    wr_off += kStageBytes;
    if (wr_off == S * kStageBytes) wr_off = 0;
  }
  // the ring is idle (zero-fill loads of the stages past K included) before the epilogue overlays it
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  float* stage_area = reinterpret_cast<float*>(lds) + wave * epilogue_stage_floats<MT, 1>();
  if (g.fast_epi) {
    epilogue_bf16_fast_any<MT, 1>(g, batch, acc, 0, n0 + wn, stage_area);
  } else {
    epilogue<MT, 1>(g, batch, acc, 0, n0 + wn, stage_area);
  }
}

template <int BM, bool AK, bool BK_, int FA, int FB>
void launch_skinny(const GemmArgs& g, int64_t batch, hipStream_t st) {
  GemmArgs a = g;
  a.tiles_m = 1;
  a.tiles_n = (g.N + kSkBN - 1) / kSkBN;
  dim3 grid((unsigned)a.tiles_n, (unsigned)batch);
  fp8_gemm_skinny_kernel<BM, AK, BK_, FA, FB><<<grid, kSkThreads, 0, st>>>(a);
}

// M <= 128.  An MN-major A tile has rows of BM bytes in LDS, for which only
// 128 has a conflict-free swizzle, so trans_a problems always take BM = 128.
template <bool AK, bool BK_, int FA, int FB>
void launch_skinny_by_m(const GemmArgs& g, int64_t batch, hipStream_t st) {
  if constexpr (AK) {
    if (g.M <= 32) return launch_skinny<32, AK, BK_, FA, FB>(g, batch, st);
    if (g.M <= 64) return launch_skinny<64, AK, BK_, FA, FB>(g, batch, st);
  }
  launch_skinny<128, AK, BK_, FA, FB>(g, batch, st);
}

}  // namespace mi355q
