// Fused int4-dequant GEMM for gfx950: fp8 activations times 4-bit weights (W4A8; 16-bit activations as two fp8 planes).
//
//   C[m, n] = out( sA[m] * sum_g s[g, n] * sum_{k in g} a[m, k] * (q[k, n] - z[g, n]) + bias[n] )
//
// The weights are what convert_from_int4 / convert_from_uint4 take (packed int32
// [K, N / 8], nibble i of word p is column 8 p + i; group-wise scales [K / g, N];
// packed zero-points [K / g, N / 8]), but they are never written out as bf16 [K, N],
// nor as fp8: a weight stage travels from HBM to LDS as packed nibbles (half the bytes
// of fp8 weights, a quarter of bf16) and goes from there into the MFMA as it is.
//
// How a nibble becomes an MFMA operand.  Two ways, one per kernel below.
//  * As an fp8 byte (the kernel for groups of 128, see w4_bytes): the e4m3 codes 0 .. 15 are one linear ramp,
//    q x 2^-9, so a nibble zero-extended to a byte is an fp8 operand and one MFMA with the block scale 2^9
//    accumulates sum_k a q exactly.
//  * As two fp4 planes (the kernel for every other group size): v_mfma_scale_f32_32x32x64_f8f6f4 multiplies an
//    fp8 operand by an fp4 (e2m1) one, and the e2m1 codes 0, 1, 2, 3 stand for 0, 0.5, 1, 1.5: a two-bit integer
//    v, zero-extended to four bits, is the e2m1 code of v / 2.  An unsigned nibble q = 4 hi + lo therefore splits
//    into two planes, (w >> 2) & 0x33333333 and w & 0x33333333 on eight nibbles at a time, and two MFMAs with
//    the block scales 2^3 and 2^1 accumulate sum_k a q exactly.
// In the first of these the zero-point leaves the inner loop: sum_k a (q - z) = sum_k a q - z sum_k a, and sum_k a
// comes from one more MFMA against a plane of ones; in the second the zero-points are two more planes, the same
// for every k of a group.  (A signed nibble s is q = s ^ 8 = s + 8 with z + 8.)  ds_read_b64_tr_b4 turns
// the packed rows (16 columns in 8 bytes) into 16 k of one column, which is what an MFMA lane wants, so the only
// vector ALU work per register of eight weights is two masks and a shift.
//
// Relative to an fp8 operand whose lane holds k = 32 h + j in byte j (h = lane / 32), the fp4 operand of the
// 32x32x64 MFMA holds k = 16 h + j in nibble j < 16 and k = 32 + 16 h + (j - 16) in nibble j >= 16.
//
// Two kernels.  The first, below, is shaped like the strip kernel of gemm_skinny.h (the second, for groups of
// 128 with bf16 scales, follows it: 256-column strips, K split over workgroups): the weights stream once through a deep LDS
// ring, one workgroup per 128 columns; rows of A beyond 64 run as further row blocks that
// stream the weights again, which suits decode and small prefill batches, the shapes
// weight-only quantisation is used for.  A workgroup has eight waves, two per SIMD, with
// two roles.  Waves 4..7 are producers: they issue the global -> LDS loads of a stage (packed
// weights, activations, the scale row and the zero-point row of the stage's group), wait for
// them, and do nothing else.  Waves 0..3 are consumers: wave w owns columns 32 w .. 32 w + 31
// and does the LDS reads, the MFMAs and the scaling, with no load, no wait counter and no
// descriptor arithmetic in its loop.  A wave issues at most one instruction every few cycles,
// so at 16 useful rows the K loop is bound by the number of instructions per stage, not by the
// MFMAs: keeping each role's loop short is what the split is for.  The roles meet at one
// barrier per K stage of 128.  At the end of a group of K the group's scales multiply the
// partial sums into the totals, in fp32.
#include "gemm_tile.h"

namespace mi355q {

constexpr int kW4Threads = 512;
constexpr int kW4ColWaves = 4;                   // consumer waves side by side along N; as many producers
constexpr int kW4BN = 128;                       // columns per workgroup
constexpr int kW4PackedStage = kBK * kW4BN / 2;  // bytes of packed weights per stage (128 k-rows of 64 bytes)
// The stage's scale row (bf16 or fp32, at most 512 bytes) and its packed zero-points (16 words) each
// arrive by one wave-wide load, which writes 64 x 16 bytes of LDS whatever lies inside the descriptor
// (lanes outside it write zeros): a KiB of room each.
constexpr int kW4ScaleRow = 1024;
constexpr int kW4ZpRow = 1024;

struct W4Args {
  GemmArgs g;              // A, C, M, N, K, lda, ldc, sa*, bias*, out_bf16 (B, sb*, D unused)
  const uint8_t* packed;   // int32 [K, N / 8]
  int64_t ld_packed;       // bytes between k-rows
  const uint8_t* scale;    // [K / group, N] bf16 or fp32
  const uint8_t* zp;       // packed int32 [K / group, N / 8] or nullptr
  int scale_f32, is_signed;
  int stages_per_group;    // group / 128
  // wide kernel: K is walked in `ksplit` parts by as many workgroups per strip
  int ksplit;
  uint32_t* tickets;       // one per strip, zero between launches
  float* partials;         // [ksplit][strips] partial sums of 32 x 256, in the consumers' register order
  // 16-bit activations as two fp8 planes (wide kernel, A16): g.A holds the leading part of every value and a_lo,
  // with the same pitch, 16 times what is left of it (split_rows_kernel); a = (A + a_lo / 16) / row scale
  const uint8_t* a_lo;
};

template <int BM>
constexpr int w4_stage_bytes() { return BM * kBK + kW4PackedStage + kW4ScaleRow + kW4ZpRow; }

template <int BM>
constexpr int w4_stages() {
  constexpr int s = (160 * 1024) / w4_stage_bytes<BM>();
  return s > 10 ? 10 : s;
}

// One 16-byte piece per lane, straight copy into LDS (lane l lands at dst + 16 l).  The
// s_nop covers a descriptor word that reached its scalar register through a vector
// instruction (five wait states before a memory instruction may read it).
// STREAM adds the nontemporal hint, for weights that the launch reads once.
template <bool STREAM = false>
__device__ __forceinline__ void w4_dma16(const i32x4& rsrc, int voff, uint32_t lds_dst) {
  if constexpr (STREAM) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
  } else {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
  }
}

// A buffer descriptor that walks through memory in fixed steps: base and the bytes left behind it.
struct W4Walker {
  uint64_t base;
  int64_t left;   // bytes from base to the end of what may be read; <= 0: every load reads zeros
  __device__ __forceinline__ void init(const uint8_t* p, int64_t bytes) {
    base = reinterpret_cast<uint64_t>(p);
    left = bytes;
  }
  __device__ __forceinline__ void step(int64_t d) {
    base += (uint64_t)d;
    left -= d;
  }
  // at most `cap` bytes from the base on
  __device__ __forceinline__ i32x4 rsrc(int64_t cap) const {
    int64_t rec = left < cap ? left : cap;
    rec = rec < 0 ? 0 : (rec > 0x7fffffffLL ? 0x7fffffffLL : rec);
    i32x4 r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)base);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((base >> 32) & 0xffffu));
    r[2] = __builtin_amdgcn_readfirstlane((int)rec);
    r[3] = 0x00020000;
    return r;
  }
};

// fp4 plane (first operand, its four registers) times fp8 fragment, block scale 2^(E - 127) on the plane
template <int FMT_A, int E>
__device__ __forceinline__ f32x16 w4_mfma(const u32x4& plane, const i32x8& fa, const f32x16& c) {
  const i32x8 b = {(int)plane[0], (int)plane[1], (int)plane[2], (int)plane[3], 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, fa, c, 4, mfma_code<FMT_A>(), 0, E, 0, 127);
}

// PIPE: the partial sums of a group are folded into the totals one group late, from a second set of
// accumulators, while the next group's MFMAs run: a wave does not stall on the MFMAs it has just issued.
//
// MODE 0 takes any group size and scale type.  MODE 1 (zero-points or signed nibbles) and MODE 2 (neither)
// are for groups of 128 with bf16 scales: every stage is a whole group, the stage's code has no branch, and
// the compiler is asked to spread the vector ALU work between the MFMAs (a wave issues in order: what
// follows an MFMA that has to wait for the matrix unit waits with it).
template <int BM, int FMT_A, bool PIPE, int MODE>
__global__ __launch_bounds__(kW4Threads) void w4a8_gemm_kernel(W4Args a) {
  constexpr int MT = BM / 32;
  constexpr int S = w4_stages<BM>();
  constexpr int kStage = w4_stage_bytes<BM>();
  constexpr int kOffPacked = BM * kBK, kOffScale = kOffPacked + kW4PackedStage, kOffZp = kOffScale + kW4ScaleRow;
  using LA = DmaLoader<true, BM, kBK, kW4ColWaves>;
  // loads per producer wave and stage: two 1 KiB regions of packed weights, its share of A, and the scale
  // row or the zero-point row
  constexpr int kOps = 2 + LA::kPerWave + 1;
  static_assert(S >= 3 && (S - 2) * kOps <= 63, "vmcnt holds 6 bits");
  static_assert(kStage % 1024 == 0, "stages stay 1 KiB aligned");
  static_assert(kW4ColWaves * epilogue_stage_floats<MT, 1>() * 4 <= S * kStage, "epilogue area overlays the ring");
  __shared__ __attribute__((aligned(1024))) uint8_t lds[S * kStage];

  // this workgroup's rows and columns
  GemmArgs g = a.g;
  const int m_base = blockIdx.y * BM;
  g.A += (int64_t)m_base * g.lda;
  g.C += (int64_t)m_base * g.ldc * (g.out_bf16 ? 2 : 4);
  if (g.sa_mode == MI355Q_GS_PER_ROW) g.sa += m_base;
  g.M = g.M - m_base < BM ? g.M - m_base : BM;
  // A strip's packed rows are 64 bytes, half a cache line; the other half belongs to the next strip.
  // Workgroups go to the 8 XCDs round robin: strips 2 j and 2 j + 1 are given to workgroups 8 apart, which
  // share an XCD (and its L2) and run at the same time.
  int strip = blockIdx.x;
  if ((gridDim.x & 15) == 0) strip = (((strip >> 4) << 3) + (strip & 7)) * 2 + ((strip >> 3) & 1);
  const int n0 = strip * kW4BN;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool producer = wave >= kW4ColWaves;
  const int wq = wave & 3;
  const int lane = lane_id_here();
  const int KT = (g.K + kBK - 1) / kBK;

  if (producer) {
    LA la;
    la.set_lane_offsets(g.lda, wq);
    la.set_tile(g.A, g.lda, 0, g.M, g.K);
    la.clamp_rows(g.lda, g.M);
    // Packed weights: producer wq loads k-rows 32 wq .. 32 wq + 31 of the stage, two regions of 16 rows of
    // 64 bytes.  The 16-byte slots of a row are stored XORed with (row / 4) % 4, which makes the consumers'
    // transposing reads conflict free; a lane writes slot lane % 4 of row lane / 4 of its region, so it
    // fetches slot (lane % 4) ^ (lane / 16) of that row.
    const int voff_packed = (wq * 32 + (lane >> 2)) * (int)a.ld_packed + ((lane & 3) ^ ((lane >> 4) & 3)) * 16;
    const int region_packed = 16 * (int)a.ld_packed;
    const int64_t packed_step = (int64_t)kBK * a.ld_packed;
    W4Walker wp;
    wp.init(a.packed + n0 / 2, (int64_t)(g.K - 1) * a.ld_packed + (((g.N + 31) & ~31) - n0) / 2);
    // Producers 0 and 1 bring the scale row, 2 and 3 the zero-point row (the same bytes twice: every
    // producer then has the same number of loads per stage, all of which go to memory, which the counted
    // wait below relies on; without zero-points the scale row stands in).
    const int es = a.scale_f32 ? 4 : 2;
    const int cols = g.N - n0 < kW4BN ? g.N - n0 : kW4BN;
    const bool bring_zp = wq >= 2 && a.zp != nullptr;
    const int64_t row_cap = bring_zp ? cols / 2 : (int64_t)cols * es;
    const int64_t row_step = bring_zp ? g.N / 2 : (int64_t)g.N * es;
    const int row_dst = wq < 2 ? kOffScale : kOffZp;
    W4Walker wr;
    wr.init(bring_zp ? a.zp + n0 / 2 : a.scale + (int64_t)n0 * es, (int64_t)((KT + a.stages_per_group - 1) / a.stages_per_group - 1) * row_step + row_cap);
    int in_group = 0;

    auto issue_stage = [&](int off, int stage) {
      const uint32_t base = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)(lds + off);
      // beyond K everything is out of range and arrives as zeros (A's zeros make the products vanish)
      const i32x4 rp = wp.rsrc(0x7fffffffLL);
      w4_dma16(rp, voff_packed, base + kOffPacked + (wq * 2) * 1024);
      w4_dma16(rp, voff_packed + region_packed, base + kOffPacked + (wq * 2 + 1) * 1024);
      wp.step(packed_step);
      static_for<LA::kPerWave>([&](auto ic) { la.template issue_one<decltype(ic)::value, true>(lds + off, stage * kBK, g.K); });
      la.advance();
      w4_dma16(wr.rsrc(row_cap), lane * 16, base + row_dst);
      if (++in_group == a.stages_per_group) {
        in_group = 0;
        wr.step(row_step);
      }
    };
    // waits until at most min(later, S - 2) stages' loads of this wave are outstanding
    auto wait_for_stage = [&](int later) {
      constexpr int full = (S - 2) * kOps;
      if (later >= S - 2) {
        __builtin_amdgcn_s_waitcnt((full & 15) | ((full >> 4) << 14) | 0x0070);
      } else {
        static_for<S - 2>([&](auto sc) {
          constexpr int n = decltype(sc)::value;  // 0 .. S - 3
          constexpr int cnt = n * kOps;
          if (later == n || (n == 0 && later < 0)) __builtin_amdgcn_s_waitcnt((cnt & 15) | ((cnt >> 4) << 14) | 0x0070);
        });
      }
    };

#pragma unroll
    for (int s = 0; s < S - 1; ++s) issue_stage(s * kStage, s);
    int wr_off = (S - 1) * kStage;
    for (int kt = 0; kt < KT; ++kt) {
      // The loads of stage kt have landed once only those of later stages are outstanding; the
      // zero-fill loads past K complete at once and are not counted (see gemm_skinny.h).
      wait_for_stage(KT - 1 - kt);
      // stage kt is in LDS for the consumers, who are done with stage kt - 1, whose room the next loads take
      __syncthreads();
      issue_stage(wr_off, kt + S - 1);
      wr_off += kStage;
      if (wr_off == S * kStage) wr_off = 0;
    }
    // the ring is idle (zero-fill loads of the stages past K included) before the epilogue overlays it
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    return;
  }

  // ------------------------------------------------------------------ consumers
  const int wn = wq * 32;
  constexpr int NB = PIPE ? 2 : 1;
  f32x16 total[MT][1], part[NB][MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) total[i][0][e] = 0.0f;

  const uint32_t flip = a.is_signed ? 0x88888888u : 0u;  // signed nibble s = (q ^ 8) - 8
  const bool has_z = a.zp != nullptr || a.is_signed;
  // this lane's part in the transposing reads: its 16-lane group covers 16 columns, the lane points at one
  // k-row; th is the k-half of the MFMA that the lane's rows belong to
  const int tg = lane >> 4, tr = lane & 15, th = tg >> 1;
  // byte offsets inside a packed stage of this lane's four reads: k-rows 64 ks + 32 p + 16 th + tr
  int poff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 32 * j + 16 * th + tr;
    poff[j] = kOffPacked + row * 64 + ((wq ^ ((row >> 2) & 3)) << 4) + (tg & 1) * 8;
  }
  const int zoff = kOffZp + ((wn + (lane & 31)) >> 3) * 4, zshift = 4 * (lane & 7);
  const int soff = kOffScale + (wn + 4 * (lane >> 5)) * (a.scale_f32 ? 4 : 2);

  // the scales of this lane's 16 columns (wn + 8 q + 4 (lane / 32) + e) for the group that ended last
  float sc[16];
  u32x4 sraw[4];  // as read from the stage's scale row: four fp32, or four bf16 in the first two words
  auto convert_scales = [&]() {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (a.scale_f32) {
#pragma unroll
        for (int e = 0; e < 4; ++e) sc[4 * q + e] = __uint_as_float(sraw[q][e]);
      } else {
        sc[4 * q + 0] = __uint_as_float(sraw[q][0] << 16);
        sc[4 * q + 1] = __uint_as_float(sraw[q][0] & 0xffff0000u);
        sc[4 * q + 2] = __uint_as_float(sraw[q][1] << 16);
        sc[4 * q + 3] = __uint_as_float(sraw[q][1] & 0xffff0000u);
      }
    }
  };
  // total += scale * sum a (q - z) of a finished group
  auto fold = [&](auto bc) {
    constexpr int B = decltype(bc)::value;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) total[i][0][e] = __builtin_fmaf(part[B][i][e], sc[e], total[i][0][e]);
  };

  int rd_off = 0;
  int kt = 0;
  if constexpr (MODE != 0) {
    static_assert(PIPE, "the one-group-per-stage loop folds one stage late");
    constexpr bool HAS_Z = MODE == 1;
    const uint32_t zmask = a.zp ? 0xffffffffu : 0u;
    auto stage = [&](auto bc, auto hpc) {
      constexpr int B = decltype(bc)::value;
      constexpr bool HAVE_PREV = decltype(hpc)::value;
      __syncthreads();  // stage kt is in LDS
      const uint8_t* st = lds + rd_off;
      uint32_t zw = 0;
      if constexpr (HAS_Z) zw = *reinterpret_cast<const uint32_t*>(st + zoff) & zmask;
      i32x2 wt[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        wt[j] = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LDS_AS i32x2*)((LDS_AS uint8_t*)st + poff[j]));
      i32x8 fa[2][MT];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
        static_for<MT>([&](auto ic) {
          static_for<2>([&](auto pc) {
            read_fragment_part<true, BM, decltype(pc)::value>(st, decltype(ic)::value * 32, ks, fa[ks][decltype(ic)::value]);
          });
        });
      u32x2 snew[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) snew[q] = *reinterpret_cast<const u32x2*>(st + soff + q * 16);
      __builtin_amdgcn_sched_barrier(0);
      u32x4 zh, zl;
      if constexpr (HAS_Z) {
        const uint32_t z4 = ((zw ^ flip) >> zshift) & 15u;
        const uint32_t ph = (8u | (z4 >> 2)) * 0x11111111u, pl = (8u | (z4 & 3u)) * 0x11111111u;
        zh = u32x4{ph, ph, ph, ph};
        zl = u32x4{pl, pl, pl, pl};
      }
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        u32x4 hi, lo;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const uint32_t w = (uint32_t)wt[2 * ks + (r >> 1)][r & 1] ^ flip;
          lo[r] = w & 0x33333333u;
          hi[r] = (w >> 2) & 0x33333333u;
        }
        static_for<MT>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if (ks == 0) part[B][i] = w4_mfma<FMT_A, 130>(hi, fa[ks][i], zero);
          else part[B][i] = w4_mfma<FMT_A, 130>(hi, fa[ks][i], part[B][i]);
          part[B][i] = w4_mfma<FMT_A, 128>(lo, fa[ks][i], part[B][i]);
          if constexpr (HAS_Z) {
            part[B][i] = w4_mfma<FMT_A, 130>(zh, fa[ks][i], part[B][i]);
            part[B][i] = w4_mfma<FMT_A, 128>(zl, fa[ks][i], part[B][i]);
          }
        });
      }
      if constexpr (HAVE_PREV) fold(std::integral_constant<int, 1 - B>{});
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        sc[4 * q + 0] = __uint_as_float(snew[q][0] << 16);
        sc[4 * q + 1] = __uint_as_float(snew[q][0] & 0xffff0000u);
        sc[4 * q + 2] = __uint_as_float(snew[q][1] << 16);
        sc[4 * q + 3] = __uint_as_float(snew[q][1] & 0xffff0000u);
      }
      // one MFMA, then a share of the other vector and scalar work, and so on
      constexpr int kMfmas = 2 * MT * (HAS_Z ? 4 : 2);
      constexpr int kOther = (24 + (HAS_Z ? 10 : 0) + (HAVE_PREV ? 16 * MT : 0) + 16 + kMfmas - 1) / kMfmas;
#pragma unroll
      for (int n = 0; n < kMfmas; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x006, kOther, 0);
      }
      rd_off += kStage;
      if (rd_off == S * kStage) rd_off = 0;
    };
    using T = std::true_type;
    using F = std::false_type;
    if (KT > 0) stage(std::integral_constant<int, 0>{}, F{});
    for (kt = 1; kt + 1 < KT; kt += 2) {
      stage(std::integral_constant<int, 1>{}, T{});
      stage(std::integral_constant<int, 0>{}, T{});
    }
    if (kt < KT) {
      stage(std::integral_constant<int, 1>{}, T{});
      fold(std::integral_constant<int, 1>{});
    } else if (KT > 0) {
      fold(std::integral_constant<int, 0>{});
    }
    __syncthreads();  // the producers have seen their last load land: the ring is idle
    float* stage_area = reinterpret_cast<float*>(lds) + wq * epilogue_stage_floats<MT, 1>();
    epilogue<MT, 1>(g, 0, total, 0, n0 + wn, stage_area);
    return;
  }
  // the stages of one group of K into accumulator set B
  auto run_group = [&](auto bc, bool have_prev) {
    constexpr int B = decltype(bc)::value;
    for (int sg = 0; sg < a.stages_per_group && kt < KT; ++sg, ++kt) {
      __syncthreads();  // stage kt is in LDS
      const uint8_t* st = lds + rd_off;
      const bool last = sg + 1 == a.stages_per_group || kt + 1 == KT;
      // Every LDS read of the stage goes out before the first result is used: a wave runs its
      // instructions in order, so a read issued late would find the MFMAs of this stage in its way.
      uint32_t zw = 0;
      if (a.zp) zw = *reinterpret_cast<const uint32_t*>(st + zoff);
      i32x2 wt[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        wt[j] = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LDS_AS i32x2*)((LDS_AS uint8_t*)st + poff[j]));
      i32x8 fa[2][MT];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
        static_for<MT>([&](auto ic) {
          static_for<2>([&](auto pc) {
            read_fragment_part<true, BM, decltype(pc)::value>(st, decltype(ic)::value * 32, ks, fa[ks][decltype(ic)::value]);
          });
        });
      u32x4 snew[4];
      if (last) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (a.scale_f32) {
            snew[q] = *reinterpret_cast<const u32x4*>(st + soff + q * 32);
          } else {
            const u32x2 v = *reinterpret_cast<const u32x2*>(st + soff + q * 16);
            snew[q] = u32x4{v[0], v[1], 0u, 0u};
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      // the zero-point of this lane's column as two constant planes with the sign bit set: - (4 zhi + zlo)
      u32x4 zh, zl;
      if (has_z) {
        const uint32_t z4 = ((zw ^ flip) >> zshift) & 15u;
        const uint32_t ph = (8u | (z4 >> 2)) * 0x11111111u, pl = (8u | (z4 & 3u)) * 0x11111111u;
        zh = u32x4{ph, ph, ph, ph};
        zl = u32x4{pl, pl, pl, pl};
      }
#pragma unroll
      for (int ks = 0; ks < kBK / 64; ++ks) {
        u32x4 hi, lo;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const uint32_t w = (uint32_t)wt[2 * ks + (r >> 1)][r & 1] ^ flip;
          lo[r] = w & 0x33333333u;
          hi[r] = (w >> 2) & 0x33333333u;
        }
        static_for<MT>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          // e2m1 reads the two-bit planes as v / 2: 2^3 and 2^1 give 4 hi + lo
          if (ks == 0 && sg == 0) part[B][i] = w4_mfma<FMT_A, 130>(hi, fa[ks][i], zero);
          else part[B][i] = w4_mfma<FMT_A, 130>(hi, fa[ks][i], part[B][i]);
          part[B][i] = w4_mfma<FMT_A, 128>(lo, fa[ks][i], part[B][i]);
          if (has_z) {
            part[B][i] = w4_mfma<FMT_A, 130>(zh, fa[ks][i], part[B][i]);
            part[B][i] = w4_mfma<FMT_A, 128>(zl, fa[ks][i], part[B][i]);
          }
        });
        if constexpr (PIPE) {
          // the group before this one, whose MFMAs finished long ago, under the MFMAs just issued
          if (ks == 0 && sg == 0 && have_prev) fold(std::integral_constant<int, 1 - B>{});
        }
      }
      if (last) {
#pragma unroll
        for (int q = 0; q < 4; ++q) sraw[q] = snew[q];
        convert_scales();
        if constexpr (!PIPE) fold(std::integral_constant<int, 0>{});
      }
      rd_off += kStage;
      if (rd_off == S * kStage) rd_off = 0;
    }
  };
  const int groups = (KT + a.stages_per_group - 1) / a.stages_per_group;
  if constexpr (PIPE) {
    for (int grp = 0; grp < groups; grp += 2) {
      run_group(std::integral_constant<int, 0>{}, grp > 0);
      if (grp + 1 < groups) run_group(std::integral_constant<int, 1>{}, true);
    }
    if (groups > 0) {
      if ((groups - 1) & 1) fold(std::integral_constant<int, 1>{});
      else fold(std::integral_constant<int, 0>{});
    }
  } else {
    for (int grp = 0; grp < groups; ++grp) run_group(std::integral_constant<int, 0>{}, false);
  }
  __syncthreads();  // the producers have seen their last load land: the ring is idle
  float* stage_area = reinterpret_cast<float*>(lds) + wq * epilogue_stage_floats<MT, 1>();
  epilogue<MT, 1>(g, 0, total, 0, n0 + wn, stage_area);
}

// ---------------------------------------------------------------------------------- wide strips
// For groups of 128 and bf16 scales (tiles of 16, 32, 64 or 128 rows; more rows are further row blocks of 128).
// A workgroup takes 256 columns: a k-row
// of its packed weights is a whole 128-byte line (the 64-byte rows of the 128-column strips move
// at about 3.2 TB/s, whole lines at 4.3), and K is cut into `ksplit` parts walked by as many
// workgroups, so that a launch fills the chip whatever N is.  The parts of a strip meet through
// memory: every workgroup stores its partial sums (already scaled by the groups' scales, fp32, in
// register order), and the one that draws the last ticket of the strip adds them up in the order
// of the parts, whoever came last, and runs the epilogue.  The last one also returns the ticket
// counter to zero for the next launch.
//
// Roles and the stage pipeline are those of the kernel above, with eight consumer waves of 32
// columns and four producers.  The 16-byte slots of a packed row in LDS are XORed with
// (row / 2) % 8, which spreads the 16 rows of a transposing read over all banks.
//
// The loads of this kernel run close to what HBM gives at 16 rows, and every vector or matrix instruction
// costs time on top of them (both go through the same issue port of a SIMD).  What keeps their number down:
//  * a nibble is an fp8 operand as it stands (w4_bytes below): one MFMA per product, not one per bit plane;
//  * the zero-points are not more MFMAs: sum_k a (q - z) = sum_k a q - z sum_k a.  The row sums of a stage's A
//    tile come from one MFMA against a plane of ones (by a producer wave with 16 rows, by the consumers with more:
//    consumer w adds up row tile w), which leaves them in a small ring in LDS for every consumer's fold one stage
//    later; with more than 16 rows a producer leaves -(z x scale) per column there as fp32, so that a fold is two
//    multiply-adds per element (total += scale x acc; total += (-z x scale) x row sum);
//  * every form multiplies on v_mfma_scale_f32_16x16x128_f8f6f4, which takes a whole stage of K in one
//    instruction: a 16 x 16 product is complete after one MFMA and is folded while the next ones run.
// In that MFMA with fp8 operands, lane group g = lane / 16 of either operand holds k = 32 g .. 32 g + 31 of its
// row (column) lane % 16 in its 32 bytes; with an fp4 first operand (the plane of ones) nibbles 16 p .. 16 p + 15
// (p = 0, 1) of lane group g pair with k = 16 (4 (g % 2) + g / 2 + 2 p) .. + 15.  Row i of the first operand and
// column j of the second meet in lane j + 16 (i / 4), register i % 4.
constexpr int kW4WideBN = 256;
constexpr int kW4WidePacked = kBK * kW4WideBN / 2;
constexpr int w4_wide_stage(int bm, bool a16 = false) { return bm * kBK * (a16 ? 2 : 1) + kW4WidePacked + kW4ScaleRow + kW4ZpRow; }
constexpr int w4_wide_stages(int bm, bool a16 = false) { return (160 * 1024 - 1024) / w4_wide_stage(bm, a16); }
constexpr int w4_wide_partial_bytes(int bm) { return bm * kW4WideBN * 4; }  // per workgroup and part of K
constexpr int kW4WideConsumers = 8;
constexpr int kW4WideThreads = (kW4WideConsumers + kW4ColWaves) * 64;
constexpr int kW4SumRing = 4;  // stages of row sums kept

// The e4m3 codes 0 .. 15 are one linear ramp, q x 2^-9 (eight subnormals and the first binade): a nibble
// zero-extended to a byte is an fp8 operand as it stands, and one MFMA with the block scale 2^9 accumulates
// sum_k a q exactly.  Eight nibbles w become the bytes of w & 0x0f0f0f0f (nibbles 0, 2, 4, 6) and of
// (w >> 4) & 0x0f0f0f0f (nibbles 1, 3, 5, 7): the transposing LDS read fills nibble i of a lane from the row
// that lane i of its group of 16 addresses, so the lanes address the rows in the order that leaves k ascending
// over the two registers (w4_nibble_row).
constexpr int kW4ByteScale = 127 + 9;
__device__ __forceinline__ int w4_nibble_row(int i) { return (i & 8) | ((i & 1) << 2) | ((i >> 1) & 3); }
__device__ __forceinline__ i32x8 w4_bytes(const i32x2& w0, const i32x2& w1, uint32_t flip) {
  i32x8 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t w = (uint32_t)(j < 2 ? w0[j & 1] : w1[j & 1]) ^ flip;
    r[2 * j] = (int)(w & 0x0f0f0f0fu);
    r[2 * j + 1] = (int)((w >> 4) & 0x0f0f0f0fu);
  }
  return r;
}
template <int FMT_A, int E>
__device__ __forceinline__ f32x4 w4_mfma16_bytes(const i32x8& w8, const i32x8& fa, const f32x4& c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w8, fa, c, 0, mfma_code<FMT_A>(), 0, E, 0, 127);
}

template <int FMT_A>
__device__ __forceinline__ f32x4 w4_mfma16(const u32x4& plane, const i32x8& fa, const f32x4& c, int e) {
  const i32x8 b = {(int)plane[0], (int)plane[1], (int)plane[2], (int)plane[3], 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b, fa, c, 4, mfma_code<FMT_A>(), 0, e, 0, 127);
}

// ROWS: 16 (one row tile; a product is folded one stage late), or 32, 64, 128 (ROWS / 16 row tiles; row blocks of
// 128 along grid.y; a product is folded two MFMAs late).
//
// A16: the activations are 16-bit values handed over as two fp8 planes of the same shape (W4A16: see
// split_rows_kernel): every stage carries both planes' tiles, and every product runs on both with the same weight
// fragments, the second plane's MFMAs with a block scale of 2^-4.  Twice the matrix work, the weights still read once.
template <int FMT_A, bool HAS_Z, int ROWS, bool A16 = false>
__global__ __launch_bounds__(kW4WideThreads) void w4a8_wide_kernel(W4Args a) {
  constexpr bool M16 = ROWS == 16;
  constexpr int RT = ROWS / 16;             // row tiles of 16
  constexpr int BM = M16 ? 32 : ROWS;       // rows of A per stage in LDS
  constexpr int kConsumers = kW4WideConsumers;
  constexpr int S = w4_wide_stages(BM, A16), kStage = w4_wide_stage(BM, A16);
  constexpr int kOffLo = BM * kBK;  // the second plane's tile (A16)
  constexpr int kOffPacked = BM * kBK * (A16 ? 2 : 1), kOffScale = kOffPacked + kW4WidePacked, kOffZp = kOffScale + kW4ScaleRow;
  constexpr int NV = 8 * RT;  // results per consumer lane: per row tile, two column tiles of four
  // the A fragments are shaped for the 16x16x128 MFMA: the XOR of TileGeom's variant 1 keeps those off each other's banks
  using LA = DmaLoader<true, BM, kBK, kW4ColWaves, 1>;
  using GA = TileGeom<true, BM, kBK, 1>;
  constexpr int kOps = 4 + LA::kPerWave * (A16 ? 2 : 1) + 1;  // four 1 KiB regions of weights, A, and the scale or zero-point row
  static_assert(S >= 3 && (S - 2) * kOps <= 63, "vmcnt holds 6 bits");
  static_assert(kStage % 1024 == 0, "stages stay 1 KiB aligned");
  __shared__ __attribute__((aligned(1024))) uint8_t lds[S * kStage];
  __shared__ __attribute__((aligned(16))) float row_sums[kW4SumRing][BM];  // (consumers read four of a row's sums at a time)
  // per stage (two kept) and column: minus the group's zero-point times its scale, fp32 (forms with row tiles)
  __shared__ __attribute__((aligned(16))) float zs_rows[2][(M16 || !HAS_Z) ? 4 : kW4WideBN];
  __shared__ uint32_t ticket_drawn;

  GemmArgs g = a.g;
  const int m_base = blockIdx.y * BM;
  g.A += (int64_t)m_base * g.lda;
  const uint8_t* a_lo = A16 ? a.a_lo + (int64_t)m_base * g.lda : nullptr;
  g.C += (int64_t)m_base * g.ldc * (g.out_bf16 ? 2 : 4);
  if (g.sa_mode == MI355Q_GS_PER_ROW) g.sa += m_base;
  g.M = g.M - m_base < BM ? g.M - m_base : BM;
  const int part = blockIdx.x % a.ksplit, strip = blockIdx.x / a.ksplit;
  const int n0 = strip * kW4WideBN;
  // this workgroup's part of K, whole stages (= groups)
  const int kt_all = (g.K + kBK - 1) / kBK;
  const int kt0 = (int)((int64_t)part * kt_all / a.ksplit), kt1 = (int)((int64_t)(part + 1) * kt_all / a.ksplit);
  const int KT = kt1 - kt0;
  const int k_begin = kt0 * kBK;
  g.K = (g.K < kt1 * kBK ? g.K : kt1 * kBK) - k_begin;
  g.A += k_begin;
  if constexpr (A16) a_lo += k_begin;
  const uint8_t* packed = a.packed + (int64_t)k_begin * a.ld_packed;
  const uint8_t* scale = a.scale + (int64_t)kt0 * g.N * 2;
  const uint8_t* zp = a.zp ? a.zp + (int64_t)kt0 * (g.N / 2) : nullptr;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool producer = wave >= kConsumers;
  const int wq = producer ? wave - kConsumers : wave;  // index among the waves of its role
  const int lane = lane_id_here();
  float total[NV];
#pragma unroll
  for (int e = 0; e < NV; ++e) total[e] = 0.0f;

  if (producer) {
    LA la, la2;
    la.set_lane_offsets(g.lda, wq);
    la.set_tile(g.A, g.lda, 0, g.M, g.K);
    la.clamp_rows(g.lda, g.M);
    if constexpr (A16) {
      la2.set_lane_offsets(g.lda, wq);
      la2.set_tile(a_lo, g.lda, 0, g.M, g.K);
      la2.clamp_rows(g.lda, g.M);
    }
    // Producer wq loads k-rows 32 wq .. 32 wq + 31, four regions of 8 rows of 128 bytes.  A lane writes
    // slot lane % 8 of row lane / 8 of its region; rows 8 r + lane / 8 have (row / 2) % 8 = 4 (r % 2) +
    // lane / 16, so that is what the lane's slot is XORed with on the memory side.
    const int ld = (int)a.ld_packed;
    const int vo_even = (wq * 32 + (lane >> 3)) * ld + (((lane & 7) ^ (lane >> 4)) << 4);
    const int vo_odd = (wq * 32 + 8 + (lane >> 3)) * ld + (((lane & 7) ^ (4 | (lane >> 4))) << 4);
    const int64_t packed_step = (int64_t)kBK * a.ld_packed;
    W4Walker wp;
    wp.init(packed + n0 / 2, (int64_t)(g.K - 1) * a.ld_packed + (((g.N + 31) & ~31) - n0) / 2);
    // producers 0 and 1 bring the scale row, 2 and 3 the zero-point row (the scale row again without one)
    const int cols = g.N - n0 < kW4WideBN ? g.N - n0 : kW4WideBN;
    const bool bring_zp = wq >= 2 && zp != nullptr;
    const int64_t row_cap = bring_zp ? cols / 2 : (int64_t)cols * 2;
    const int64_t row_step = bring_zp ? g.N / 2 : (int64_t)g.N * 2;
    const int row_dst = wq < 2 ? kOffScale : kOffZp;
    W4Walker wr;
    wr.init(bring_zp ? zp + n0 / 2 : scale + (int64_t)n0 * 2, (int64_t)(KT - 1) * row_step + row_cap);

    auto issue_stage = [&](int off, int stage) {
      const uint32_t base = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)(lds + off);
      const i32x4 rp = wp.rsrc(0x7fffffffLL);
      // up to 128 rows there is one row block and the weights are read once; further row blocks read them again,
      // out of the caches
      constexpr bool kOnce = ROWS < 128;
      w4_dma16<kOnce>(rp, vo_even, base + kOffPacked + (wq * 4) * 1024);
      w4_dma16<kOnce>(rp, vo_odd, base + kOffPacked + (wq * 4 + 1) * 1024);
      w4_dma16<kOnce>(rp, vo_even + 16 * ld, base + kOffPacked + (wq * 4 + 2) * 1024);
      w4_dma16<kOnce>(rp, vo_odd + 16 * ld, base + kOffPacked + (wq * 4 + 3) * 1024);
      wp.step(packed_step);
      static_for<LA::kPerWave>([&](auto ic) { la.template issue_one<decltype(ic)::value, true>(lds + off, stage * kBK, g.K); });
      la.advance();
      if constexpr (A16) {
        static_for<LA::kPerWave>([&](auto ic) { la2.template issue_one<decltype(ic)::value, true>(lds + off + kOffLo, stage * kBK, g.K); });
        la2.advance();
      }
      w4_dma16(wr.rsrc(row_cap), lane * 16, base + row_dst);
      wr.step(row_step);
    };
    auto wait_for_stage = [&](int later) {
      constexpr int full = (S - 2) * kOps;
      if (later >= S - 2) {
        __builtin_amdgcn_s_waitcnt((full & 15) | ((full >> 4) << 14) | 0x0070);
      } else {
        static_for<S - 2>([&](auto sc) {
          constexpr int n = decltype(sc)::value;
          constexpr int cnt = n * kOps;
          if (later == n || (n == 0 && later < 0)) __builtin_amdgcn_s_waitcnt((cnt & 15) | ((cnt >> 4) << 14) | 0x0070);
        });
      }
    };
    // sum_k a[m, k] over the stage at `off`, for the consumers' fold one stage later (16-row form)
    const u32x4 ones = {0x22222222u, 0x22222222u, 0x22222222u, 0x22222222u};  // e2m1 1.0
    auto sum_rows = [&](int off, int slot) {
      const uint8_t* st = lds + off;
      const int m = lane & 15, gk = lane >> 4;
      const u32x4 lo = *reinterpret_cast<const u32x4*>(st + GA::lds_offset(m, 2 * gk));
      const u32x4 hi = *reinterpret_cast<const u32x4*>(st + GA::lds_offset(m, 2 * gk + 1));
      const i32x8 fa = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      f32x4 r = w4_mfma16<FMT_A>(ones, fa, f32x4{0.f, 0.f, 0.f, 0.f}, 127);
      if constexpr (A16) {
        const u32x4 lo2 = *reinterpret_cast<const u32x4*>(st + kOffLo + GA::lds_offset(m, 2 * gk));
        const u32x4 hi2 = *reinterpret_cast<const u32x4*>(st + kOffLo + GA::lds_offset(m, 2 * gk + 1));
        const i32x8 fb = {(int)lo2[0], (int)lo2[1], (int)lo2[2], (int)lo2[3], (int)hi2[0], (int)hi2[1], (int)hi2[2], (int)hi2[3]};
        r = w4_mfma16<FMT_A>(ones, fb, r, 123);
      }
      // every lane holds the sum of its row (lane % 16) and every lane stores it: a store under a lane mask would
      // take the MFMA, whose result only those lanes used, under the mask with it
      row_sums[slot][lane & 15] = r[0];
    };
    // -(zero-point) x scale of the stage's group, four columns per lane, for the consumers' fold one stage later:
    // what every consumer lane would otherwise work out for its eight columns in every stage.
    const uint32_t pflip = a.is_signed ? 0x8888u : 0u, pzmask = a.zp ? 0xffffu : 0u;
    auto column_rows = [&](int off, int slot) {
      const uint8_t* st = lds + off;
      const u32x2 sw = *reinterpret_cast<const u32x2*>(st + kOffScale + 8 * lane);
      const uint32_t zw = ((uint32_t)*reinterpret_cast<const uint16_t*>(st + kOffZp + 2 * lane) & pzmask) ^ pflip;
      f32x4 sf, zf;
      sf[0] = __uint_as_float(sw[0] << 16);
      sf[1] = __uint_as_float(sw[0] & 0xffff0000u);
      sf[2] = __uint_as_float(sw[1] << 16);
      sf[3] = __uint_as_float(sw[1] & 0xffff0000u);
#pragma unroll
      for (int i = 0; i < 4; ++i) zf[i] = -(float)((zw >> (4 * i)) & 15u) * sf[i];
      *reinterpret_cast<f32x4*>(&zs_rows[slot][4 * lane]) = zf;
    };
#pragma unroll
    for (int s = 0; s < S - 1; ++s) issue_stage(s * kStage, s);
    int wr_off = (S - 1) * kStage, rd_off = 0;
    for (int kt = 0; kt < KT; ++kt) {
      // the loads past this part of K fall outside their descriptors, complete at once and are not counted
      wait_for_stage(KT - 1 - kt);
      __syncthreads();
      issue_stage(wr_off, kt + S - 1);
      if constexpr (!M16 && HAS_Z) {
        if (((kt + 2) & 3) == wq) column_rows(rd_off, kt & 1);
      }
      // (with more rows the consumers, which read every A fragment anyway, add the rows up)
      if (HAS_Z && M16 && (kt & 3) == wq) sum_rows(rd_off, kt & (kW4SumRing - 1));
      wr_off += kStage;
      if (wr_off == S * kStage) wr_off = 0;
      rd_off += kStage;
      if (rd_off == S * kStage) rd_off = 0;
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // the consumers' barrier of the fold that follows the last stage
  } else {
    const int wn = wq * 32;
    const uint32_t flip = a.is_signed ? 0x88888888u : 0u;
    const uint32_t zmask = a.zp ? 0xffffffffu : 0u;
    int rd_off = 0, slot = 0;
    using T = std::true_type;
    using F = std::false_type;
    if constexpr (M16) {
      // lane: row m = lane % 16 of A; columns wn + 16 t + 4 gk + e (t = 0, 1; e = 0 .. 3); k block gk = lane / 16
      const int gk = lane >> 4, r16 = lane & 15;
      int poff[2][2];
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const int row = 32 * gk + 16 * p + w4_nibble_row(r16);  // the fp8 operand of lane group gk: k = 32 gk .. + 31
#pragma unroll
        for (int t = 0; t < 2; ++t) poff[t][p] = kOffPacked + row * 128 + ((wq ^ ((row >> 1) & 7)) << 4) + t * 8;
      }
      const int aoff0 = GA::lds_offset(r16, 2 * gk), aoff1 = GA::lds_offset(r16, 2 * gk + 1);
      const int soff = kOffScale + (wn + 4 * gk) * 2;             // + 32 t: four bf16
      const int zoff = kOffZp + (wn / 8 + (gk >> 1)) * 4;         // + 8 t: the word of these columns
      const int zshift = 16 * (gk & 1);
      f32x4 acc[2][2];
      float sc[2][4];
      uint32_t zprev[2] = {0u, 0u};
      auto fold = [&](auto bc, int sum_slot) {
        constexpr int B = decltype(bc)::value;
        float rs = 0.0f;
        if constexpr (HAS_Z) rs = row_sums[sum_slot][r16];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = acc[B][t][e];
            if constexpr (HAS_Z) v = __builtin_fmaf(-(float)((zprev[t] >> (4 * e)) & 15u), rs, v);
            total[4 * t + e] = __builtin_fmaf(v, sc[t][e], total[4 * t + e]);
          }
      };
      auto stage = [&](auto bc, auto hpc) {
        constexpr int B = decltype(bc)::value;
        constexpr bool HAVE_PREV = decltype(hpc)::value;
        __syncthreads();  // the stage is in LDS, and so are the row sums of the one before
        const uint8_t* st = lds + rd_off;
        i32x2 wt[2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int p = 0; p < 2; ++p)
            wt[t][p] = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LDS_AS i32x2*)((LDS_AS uint8_t*)st + poff[t][p]));
        const u32x4 alo = *reinterpret_cast<const u32x4*>(st + aoff0), ahi = *reinterpret_cast<const u32x4*>(st + aoff1);
        u32x4 blo = alo, bhi = ahi;
        if constexpr (A16) {
          blo = *reinterpret_cast<const u32x4*>(st + kOffLo + aoff0);
          bhi = *reinterpret_cast<const u32x4*>(st + kOffLo + aoff1);
        }
        u32x2 snew[2];
        uint32_t znew[2] = {0u, 0u};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          snew[t] = *reinterpret_cast<const u32x2*>(st + soff + 32 * t);
          if constexpr (HAS_Z) znew[t] = *reinterpret_cast<const uint32_t*>(st + zoff + 8 * t);
        }
        __builtin_amdgcn_sched_barrier(0);
        const i32x8 fa = {(int)alo[0], (int)alo[1], (int)alo[2], (int)alo[3], (int)ahi[0], (int)ahi[1], (int)ahi[2], (int)ahi[3]};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const i32x8 w8 = w4_bytes(wt[t][0], wt[t][1], flip);
          acc[B][t] = w4_mfma16_bytes<FMT_A, kW4ByteScale>(w8, fa, f32x4{0.f, 0.f, 0.f, 0.f});
          if constexpr (A16) {
            const i32x8 fb = {(int)blo[0], (int)blo[1], (int)blo[2], (int)blo[3], (int)bhi[0], (int)bhi[1], (int)bhi[2], (int)bhi[3]};
            acc[B][t] = w4_mfma16_bytes<FMT_A, kW4ByteScale - 4>(w8, fb, acc[B][t]);
          }
        }
        // the stage before this one, whose MFMAs finished long ago, behind the MFMAs just issued
        if constexpr (HAVE_PREV) fold(std::integral_constant<int, 1 - B>{}, (slot - 1) & (kW4SumRing - 1));
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          sc[t][0] = __uint_as_float(snew[t][0] << 16);
          sc[t][1] = __uint_as_float(snew[t][0] & 0xffff0000u);
          sc[t][2] = __uint_as_float(snew[t][1] << 16);
          sc[t][3] = __uint_as_float(snew[t][1] & 0xffff0000u);
          zprev[t] = (((znew[t] & zmask) ^ flip) >> zshift) & 0xffffu;
        }
        rd_off += kStage;
        if (rd_off == S * kStage) rd_off = 0;
        ++slot;
      };
      int kt = 1;
      if (KT > 0) stage(std::integral_constant<int, 0>{}, F{});
      for (; kt + 1 < KT; kt += 2) {
        stage(std::integral_constant<int, 1>{}, T{});
        stage(std::integral_constant<int, 0>{}, T{});
      }
      if (kt < KT) stage(std::integral_constant<int, 1>{}, T{});
      __syncthreads();  // the row sums of the last stage
      if (KT > 0) {
        if (KT & 1) fold(std::integral_constant<int, 0>{}, (slot - 1) & (kW4SumRing - 1));
        else fold(std::integral_constant<int, 1>{}, (slot - 1) & (kW4SumRing - 1));
      }
    } else {
      // ROWS / 16 row tiles on the 16x16x128 MFMA, which takes a whole stage of K in one instruction: the products of
      // a stage (row tiles by two column tiles) are independent, and each is folded into the totals two products
      // later, eight multiply-adds behind an MFMA that lasts as long as they do.  The scale term of a product uses
      // its own stage's scales; the zero-point term, -(z x scale)[n] x (row sum of A)[m], whose factors are left
      // in LDS during a stage, follows one stage later.
      // lane: rows m = 16 i + lane % 16 of A; columns wn + 16 t + 4 gk + e; product j = 2 i + t, total[4 j + e]
      const int gk = lane >> 4, r16 = lane & 15;
      int poff[2][2];
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const int row = 32 * gk + 16 * p + w4_nibble_row(r16);
#pragma unroll
        for (int t = 0; t < 2; ++t) poff[t][p] = kOffPacked + row * 128 + ((wq ^ ((row >> 1) & 7)) << 4) + t * 8;
      }
      const int aoff0 = GA::lds_offset(r16, 2 * gk), aoff1 = GA::lds_offset(r16, 2 * gk + 1);  // tile i: + 2048 i
      const int soff = kOffScale + (wn + 4 * gk) * 2;  // + 32 t: four bf16
      const int zsoff = wn + 4 * gk;                   // + 16 t: four fp32
      constexpr int NB = A16 ? 2 : 3, LAG = NB - 1;  // sets of partial sums; products between an MFMA and its fold
      constexpr int NF = A16 ? 2 : 3;      // A fragments in registers: the one being multiplied and those on their way
      const int sum_tile = wq & (RT - 1);  // the row tile this consumer adds up (with fewer tiles than consumers several do the same one)
      const u32x4 ones = {0x22222222u, 0x22222222u, 0x22222222u, 0x22222222u};  // e2m1 1.0
      f32x4 acc[NB];
      f32x4 sc[2], zsp[2];
      float rsp[RT];
      i32x2 wt[2][2];
      i32x8 fa[NF], fb[A16 ? NF : 1];
      u32x2 snew[2];
      auto fragment = [&](const uint8_t* st, int tile) {
        const u32x4 lo = *reinterpret_cast<const u32x4*>(st + aoff0 + 2048 * tile), hi = *reinterpret_cast<const u32x4*>(st + aoff1 + 2048 * tile);
        return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      };
      auto read_a = [&](const uint8_t* st, auto ic) {
        constexpr int i = decltype(ic)::value;
        fa[i % NF] = fragment(st, i);
        if constexpr (A16) fb[i % NF] = fragment(st + kOffLo, i);
      };
      // what a stage starts with: the packed weights, the first A fragments, the scales
      auto read_head = [&](const uint8_t* st) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int p = 0; p < 2; ++p)
            wt[t][p] = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LDS_AS i32x2*)((LDS_AS uint8_t*)st + poff[t][p]));
        static_for<(NF - 1 < RT ? NF - 1 : RT)>([&](auto ic) { read_a(st, ic); });
#pragma unroll
        for (int t = 0; t < 2; ++t) snew[t] = *reinterpret_cast<const u32x2*>(st + soff + 32 * t);
      };
      auto stage = [&](auto hpc) {
        constexpr bool ZT = decltype(hpc)::value && HAS_Z;  // a stage before this one has left its zero-point term
        const uint8_t* st = lds + rd_off;
        rd_off += kStage;
        if (rd_off == S * kStage) rd_off = 0;
        i32x8 fs, fs2;  // the fragment of the row tile whose sums this consumer works out
        if constexpr (HAS_Z) {
          fs = fragment(st, sum_tile);
          if constexpr (A16) fs2 = fragment(st + kOffLo, sum_tile);
        }
        if constexpr (ZT) {
          const int prev = slot - 1;
#pragma unroll
          for (int t = 0; t < 2; ++t) zsp[t] = *reinterpret_cast<const f32x4*>(&zs_rows[prev & 1][zsoff + 16 * t]);
          static_for<RT / 4>([&](auto hc) {
            constexpr int h = decltype(hc)::value;
            const f32x4 r = *reinterpret_cast<const f32x4*>(&row_sums[prev & (kW4SumRing - 1)][r16 * RT + 4 * h]);
#pragma unroll
            for (int i = 0; i < 4; ++i) rsp[4 * h + i] = r[i];
          });
          if constexpr (RT == 2) {
            const f32x2 r = *reinterpret_cast<const f32x2*>(&row_sums[prev & (kW4SumRing - 1)][r16 * RT]);
            rsp[0] = r[0];
            rsp[1] = r[1];
          }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          sc[t][0] = __uint_as_float(snew[t][0] << 16);
          sc[t][1] = __uint_as_float(snew[t][0] & 0xffff0000u);
          sc[t][2] = __uint_as_float(snew[t][1] << 16);
          sc[t][3] = __uint_as_float(snew[t][1] & 0xffff0000u);
        }
        const i32x8 w8[2] = {w4_bytes(wt[0][0], wt[0][1], flip), w4_bytes(wt[1][0], wt[1][1], flip)};
        auto fold = [&](auto jc) {
          constexpr int j = decltype(jc)::value, t = j & 1, i = j >> 1, b = j % NB;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = __builtin_fmaf(acc[b][e], sc[t][e], total[4 * j + e]);
            if constexpr (ZT) v = __builtin_fmaf(zsp[t][e], rsp[i], v);
            total[4 * j + e] = v;
          }
        };
        if constexpr (HAS_Z) {
          // the row sums of that tile, for every consumer's fold of the next stage: one more MFMA, against a plane of
          // ones.  Every lane holds the sum of its row and every lane stores it (a store under a lane mask would
          // take the MFMA under the mask with it); a consumer lane finds the sums of its RT rows side by side.
          f32x4 r = w4_mfma16<FMT_A>(ones, fs, f32x4{0.f, 0.f, 0.f, 0.f}, 127);
          if constexpr (A16) r = w4_mfma16<FMT_A>(ones, fs2, r, 123);
          row_sums[slot & (kW4SumRing - 1)][r16 * RT + sum_tile] = r[0];
        }
        __builtin_amdgcn_sched_barrier(0);
        static_for<2 * RT>([&](auto jc) {
          constexpr int j = decltype(jc)::value, t = j & 1, i = j >> 1, b = j % NB;
          if constexpr (t == 0 && i + NF - 1 < RT) read_a(st, std::integral_constant<int, i + NF - 1>{});
          acc[b] = w4_mfma16_bytes<FMT_A, kW4ByteScale>(w8[t], fa[i % NF], f32x4{0.f, 0.f, 0.f, 0.f});
          if constexpr (A16) acc[b] = w4_mfma16_bytes<FMT_A, kW4ByteScale - 4>(w8[t], fb[i % NF], acc[b]);
          if constexpr (j >= LAG) fold(std::integral_constant<int, j - LAG>{});
          __builtin_amdgcn_sched_barrier(0);
        });
        static_for<LAG>([&](auto lc) { fold(std::integral_constant<int, 2 * RT - LAG + decltype(lc)::value>{}); });
        ++slot;
        __syncthreads();  // the next stage is in LDS, and so are the row sums and the zero-point row of this one
        read_head(lds + rd_off);  // (past the last stage: a slot of the ring whose contents are not used)
      };
      __syncthreads();
      read_head(lds);
      if (KT > 0) stage(F{});
      for (int kt = 1; kt < KT; ++kt) stage(T{});
      if constexpr (HAS_Z) {
        if (KT > 0) {
          const int prev = slot - 1;
#pragma unroll
          for (int t = 0; t < 2; ++t) zsp[t] = *reinterpret_cast<const f32x4*>(&zs_rows[prev & 1][zsoff + 16 * t]);
#pragma unroll
          for (int i = 0; i < RT; ++i) {
            const float rs = row_sums[prev & (kW4SumRing - 1)][r16 * RT + i];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int e = 0; e < 4; ++e) total[4 * (2 * i + t) + e] = __builtin_fmaf(zsp[t][e], rs, total[4 * (2 * i + t) + e]);
          }
        }
      }
    }
  }
  __syncthreads();  // every load has landed and every stage is consumed: the ring is idle

  if (a.ksplit > 1) {
    // Partial sums in register order: 64-bit word number h 64 + lane (h < NV / 2) of consumer wave wq.  They are
    // written and read with device-scope atomic accesses, which go past the caches of this XCD to where the other
    // XCDs see them: no cache has to be written back or invalidated as a whole, which a fence would do (and
    // which, done by every workgroup while the others still stream, costs more than the kernel).
    const int strips = gridDim.x / a.ksplit * gridDim.y;         // strips of all row blocks
    const int strip_rb = blockIdx.y * (gridDim.x / a.ksplit) + strip;
    constexpr int kWords = BM * 16;  // per consumer wave (half of them used with 16 rows)
    unsigned long long* mine = reinterpret_cast<unsigned long long*>(a.partials) + ((int64_t)(part * strips + strip_rb) * kConsumers + wq) * kWords + lane;
    if (!producer) {
#pragma unroll
      for (int h = 0; h < NV / 2; ++h) {
        const unsigned long long v = (unsigned long long)__float_as_uint(total[2 * h]) | ((unsigned long long)__float_as_uint(total[2 * h + 1]) << 32);
        __hip_atomic_store(mine + h * 64, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __builtin_amdgcn_s_waitcnt(0);  // the stores have been acknowledged before the ticket is drawn
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      const uint32_t t = __hip_atomic_fetch_add(a.tickets + strip_rb, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (t == (uint32_t)a.ksplit - 1) __hip_atomic_store(a.tickets + strip_rb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
      ticket_drawn = t;
    }
    __syncthreads();
    if (ticket_drawn != (uint32_t)a.ksplit - 1) return;
    if (!producer) {
      // part 0 + part 1 + part 2 + ..., whichever part comes last.  Part 0 or 1 keeps its own sums in its registers
      // and adds the other of the two first (the same bits as the other way round, and no partial sum is -0); a
      // later part starts from zero and reads its own with the rest.
      const unsigned long long* from = reinterpret_cast<const unsigned long long*>(a.partials) + ((int64_t)strip_rb * kConsumers + wq) * kWords + lane;
      const int64_t part_stride = (int64_t)strips * kConsumers * kWords;
      auto add_part = [&](int p) {
        const unsigned long long* src = from + p * part_stride;
        unsigned long long v[NV / 2];
#pragma unroll
        for (int h = 0; h < NV / 2; ++h) v[h] = __hip_atomic_load(src + h * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int h = 0; h < NV / 2; ++h) {
          total[2 * h] += __uint_as_float((uint32_t)v[h]);
          total[2 * h + 1] += __uint_as_float((uint32_t)(v[h] >> 32));
        }
      };
      int p = 0;
      if (part <= 1) {
        add_part(1 - part);
        p = 2;
      } else {
#pragma unroll
        for (int e = 0; e < NV; ++e) total[e] = 0.0f;
      }
      for (; p < a.ksplit; ++p) add_part(p);
    }
  }
  if (producer) return;
  {
    // C[m, n .. n + 3] for this lane's rows (one per row tile) and its two sets of four columns
    const int gk = lane >> 4;
    const ScalarScales scalars = load_scalar_scales(g);
    const int es = g.out_bf16 ? 2 : 4;
#pragma unroll
    for (int j = 0; j < 2 * RT; ++j) {
      const int t = j & 1, m = 16 * (j >> 1) + (lane & 15);
      if (m >= g.M) continue;
      const float sa = g.sa_mode == MI355Q_GS_PER_ROW ? g.sa[m] : scalars.sa;
      const int n = n0 + wq * 32 + 16 * t + 4 * gk;
      if (n >= g.N) continue;  // N is a multiple of 32: the four columns are inside or outside together
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float bias = g.bias_mode == MI355Q_BIAS_ROW_VECTOR ? load_out_as_f32(g.bias, n + e, g.out_bf16) : 0.0f;
        v[e] = __fmul_rn(total[4 * j + e], sa) + bias;  // rounded as the other epilogues round
      }
      uint8_t* cp = g.C + ((int64_t)m * g.ldc + n) * es;
      const bool vec_ok = (reinterpret_cast<uintptr_t>(cp) % (4 * es)) == 0;
      if (g.out_bf16) {
        if (vec_ok) {
          *reinterpret_cast<u32x2*>(cp) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) reinterpret_cast<uint16_t*>(cp)[e] = (uint16_t)(pack_bf16x2(v[e], v[e]) & 0xffffu);
        }
      } else {
        if (vec_ok) {
          *reinterpret_cast<f32x4*>(cp) = f32x4{v[0], v[1], v[2], v[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) reinterpret_cast<float*>(cp)[e] = v[e];
        }
      }
    }
  }
}

// How the wide kernel takes a problem: rows per workgroup (16 rows sit in a 32-row tile of LDS), row
// blocks, strips, and the parts K is walked in (0: the wide kernel does not apply).
struct W4WidePlan {
  int rows, row_blocks, strips, parts;
  int tile_rows() const { return rows >= 64 ? rows : 32; }
  // The counters sit in front of the partial sums, in an area of a fixed size: a workspace that is used for
  // problems of different shapes then finds them zero whatever the last shape left in the partial sums.
  // K is only split for at most 128 strips (256 / groups >= 2 below).
  static constexpr size_t ticket_bytes() { return 1024; }
  size_t workspace_bytes() const {
    return parts < 2 ? 0 : ticket_bytes() + (size_t)parts * strips * row_blocks * w4_wide_partial_bytes(tile_rows());
  }
};
inline W4WidePlan w4a8_wide_plan(int64_t M, int64_t N, int64_t K, int64_t group, int scale_f32) {
  W4WidePlan p{0, 0, 0, 0};
  if (group != kBK || scale_f32 || K <= 0 || M <= 0 || N <= 0) return p;
  p.rows = M <= 16 ? 16 : (M <= 32 ? 32 : (M <= 64 ? 64 : 128));
  p.row_blocks = (int)((M + p.tile_rows() - 1) / p.tile_rows());
  p.strips = (int)((N + kW4WideBN - 1) / kW4WideBN);
  const int64_t kt = (K + kBK - 1) / kBK, groups = (int64_t)p.strips * p.row_blocks;
  int64_t parts = 256 / groups;
  if (parts > kt / 8) parts = kt / 8;
  // too few workgroups for the chip even so: the 128-column strips have twice as many
  if (parts < 2) parts = groups >= 100 ? 1 : 0;
  if (p.row_blocks > 65535) parts = 0;
  if (parts >= 2 && (size_t)groups * 4 > W4WidePlan::ticket_bytes()) parts = 1;  // (cannot happen: 256 / groups >= 2)
  p.parts = (int)parts;
  return p;
}

template <int BM, int FMT_A>
void w4a8_launch(const W4Args& a, hipStream_t st) {
  dim3 grid((unsigned)((a.g.N + kW4BN - 1) / kW4BN), (unsigned)((a.g.M + BM - 1) / BM));
  const bool fast = a.stages_per_group == 1 && !a.scale_f32 && a.g.K > 0;
  if (!fast) w4a8_gemm_kernel<BM, FMT_A, true, 0><<<grid, kW4Threads, 0, st>>>(a);
  else if (a.zp != nullptr || a.is_signed) w4a8_gemm_kernel<BM, FMT_A, true, 1><<<grid, kW4Threads, 0, st>>>(a);
  else w4a8_gemm_kernel<BM, FMT_A, true, 2><<<grid, kW4Threads, 0, st>>>(a);
}

template <int FMT_A>
void w4a8_launch_by_m(const W4Args& a, hipStream_t st) {
  if (a.ksplit > 0) {
    const bool z = a.zp != nullptr || a.is_signed;
    const unsigned strips = (unsigned)((a.g.N + kW4WideBN - 1) / kW4WideBN);
    if (a.g.M <= 16) {
      const dim3 grid(strips * (unsigned)a.ksplit);
      if (z) w4a8_wide_kernel<FMT_A, true, 16><<<grid, kW4WideThreads, 0, st>>>(a);
      else w4a8_wide_kernel<FMT_A, false, 16><<<grid, kW4WideThreads, 0, st>>>(a);
    } else if (a.g.M <= 32) {
      const dim3 grid(strips * (unsigned)a.ksplit);
      if (z) w4a8_wide_kernel<FMT_A, true, 32><<<grid, kW4WideThreads, 0, st>>>(a);
      else w4a8_wide_kernel<FMT_A, false, 32><<<grid, kW4WideThreads, 0, st>>>(a);
    } else if (a.g.M <= 64) {
      const dim3 grid(strips * (unsigned)a.ksplit);
      if (z) w4a8_wide_kernel<FMT_A, true, 64><<<grid, kW4WideThreads, 0, st>>>(a);
      else w4a8_wide_kernel<FMT_A, false, 64><<<grid, kW4WideThreads, 0, st>>>(a);
    } else {
      const dim3 grid(strips * (unsigned)a.ksplit, (unsigned)((a.g.M + 127) / 128));
      if (z) w4a8_wide_kernel<FMT_A, true, 128><<<grid, kW4WideThreads, 0, st>>>(a);
      else w4a8_wide_kernel<FMT_A, false, 128><<<grid, kW4WideThreads, 0, st>>>(a);
    }
  } else if (a.g.M <= 32) {
    w4a8_launch<32, FMT_A>(a, st);
  } else {
    w4a8_launch<64, FMT_A>(a, st);
  }
}

// The wide kernel on two fp8 planes of 16-bit activations (always this kernel: K in one part where the plan would
// rather use the 128-column strips, which have no two-plane form).
inline void w4a16_launch(const W4Args& a, hipStream_t st) {
  const bool z = a.zp != nullptr || a.is_signed;
  const unsigned strips = (unsigned)((a.g.N + kW4WideBN - 1) / kW4WideBN);
  constexpr int F = MI355Q_E4M3FN;
  if (a.g.M <= 16) {
    const dim3 grid(strips * (unsigned)a.ksplit);
    if (z) w4a8_wide_kernel<F, true, 16, true><<<grid, kW4WideThreads, 0, st>>>(a);
    else w4a8_wide_kernel<F, false, 16, true><<<grid, kW4WideThreads, 0, st>>>(a);
  } else if (a.g.M <= 32) {
    const dim3 grid(strips * (unsigned)a.ksplit);
    if (z) w4a8_wide_kernel<F, true, 32, true><<<grid, kW4WideThreads, 0, st>>>(a);
    else w4a8_wide_kernel<F, false, 32, true><<<grid, kW4WideThreads, 0, st>>>(a);
  } else if (a.g.M <= 64) {
    const dim3 grid(strips * (unsigned)a.ksplit);
    if (z) w4a8_wide_kernel<F, true, 64, true><<<grid, kW4WideThreads, 0, st>>>(a);
    else w4a8_wide_kernel<F, false, 64, true><<<grid, kW4WideThreads, 0, st>>>(a);
  } else {
    const dim3 grid(strips * (unsigned)a.ksplit, (unsigned)((a.g.M + 127) / 128));
    if (z) w4a8_wide_kernel<F, true, 128, true><<<grid, kW4WideThreads, 0, st>>>(a);
    else w4a8_wide_kernel<F, false, 128, true><<<grid, kW4WideThreads, 0, st>>>(a);
  }
}

// Workspace of mi355q_w4a16_gemm: [arrival counters and partial sums of the K split, as for W4A8][plane 1][plane 2]
// [1 / row scale], each part 256-byte aligned.
struct W4A16Layout {
  size_t split_bytes, plane_off, lo_off, scale_off, total;
  int64_t ld;  // row pitch of the planes, a multiple of 16
};
inline W4A16Layout w4a16_layout(int64_t M, int64_t N, int64_t K, int64_t group, int scale_f32) {
  const auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  W4A16Layout l{};
  const W4WidePlan plan = w4a8_wide_plan(M, N, K, group, scale_f32);
  // the arrival counters' KiB is set aside whether this shape splits K or not: a buffer that serves calls of several
  // shapes must not find the planes of one call where the next one keeps its counters
  l.split_bytes = plan.parts >= 2 ? plan.workspace_bytes() : W4WidePlan::ticket_bytes();
  l.ld = (K + 15) & ~(int64_t)15;
  l.plane_off = up(l.split_bytes);
  l.lo_off = l.plane_off + up((size_t)(M * l.ld));
  l.scale_off = l.lo_off + up((size_t)(M * l.ld));
  l.total = l.scale_off + up((size_t)M * sizeof(float));
  return l;
}

}  // namespace mi355q

using namespace mi355q;

extern "C" size_t mi355q_w4a16_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int scale_dtype) {
  if (M <= 0 || N <= 0 || K <= 0 || group <= 0) return 0;
  return w4a16_layout(M, N, K, group, scale_dtype == MI355Q_F32).total;
}

extern "C" int mi355q_w4a16_gemm(const void* A, int a_dtype, int64_t lda, const int32_t* packed, int64_t ld_packed,
                                 const void* scale, int scale_dtype, const int32_t* zero_point, int is_signed,
                                 int64_t group, void* C, int out_dtype, int64_t ldc, int64_t M, int64_t N, int64_t K,
                                 const void* bias, void* workspace, size_t workspace_bytes, int split_k, void* stream) {
  if (a_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype != MI355Q_F32 && out_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (scale_dtype != MI355Q_F32 && scale_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (M < 0 || N < 0 || K < 0 || group <= 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (M == 0 || N == 0) return MI355Q_OK;
  if (C == nullptr || (K > 0 && (A == nullptr || packed == nullptr || scale == nullptr))) return MI355Q_ERR_INVALID_ARGUMENT;
  if (K % group != 0 || lda < K || ld_packed < N / 8 || ldc < N) return MI355Q_ERR_INVALID_ARGUMENT;
  const auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  const int es = 2;
  // the two-plane kernel serves groups of 128 with bf16 scales; whole 16-byte pieces throughout
  if (group != kBK || scale_dtype != MI355Q_BF16 || K == 0 || N % 32 != 0 || K % 16 != 0 || (lda * es) % 16 != 0 || (ld_packed * 4) % 16 != 0 ||
      !al16(A) || !al16(packed) || !al16(scale) || (zero_point && !al16(zero_point)) ||
      M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL || (M + 63) / 64 > 65535)
    return MI355Q_ERR_UNSUPPORTED;
  const W4A16Layout l = w4a16_layout(M, N, K, group, 0);
  if (workspace == nullptr || !al16(workspace) || workspace_bytes < l.total) return MI355Q_ERR_WORKSPACE;
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  float* sx_inv = reinterpret_cast<float*>(ws + l.scale_off);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int sp = mi355q_split_rows_fp8x2(A, a_dtype, lda, M, K, ws + l.plane_off, ws + l.lo_off, l.ld, sx_inv, stream);
  if (sp != MI355Q_OK) return sp;
  W4Args a{};
  a.g.A = ws + l.plane_off;
  a.a_lo = ws + l.lo_off;
  a.g.C = static_cast<uint8_t*>(C);
  a.g.lda = l.ld;
  a.g.ldc = ldc;
  a.g.M = (int)M;
  a.g.N = (int)N;
  a.g.K = (int)K;
  a.g.sa = sx_inv;
  a.g.sa_host = 1.0f;
  a.g.sa_mode = MI355Q_GS_PER_ROW;
  a.g.sb_mode = MI355Q_GS_NONE;
  a.g.sb_host = 1.0f;
  a.g.bias = static_cast<const uint8_t*>(bias);
  a.g.bias_mode = bias ? MI355Q_BIAS_ROW_VECTOR : MI355Q_BIAS_NONE;
  a.g.out_bf16 = out_dtype == MI355Q_BF16;
  a.packed = reinterpret_cast<const uint8_t*>(packed);
  a.ld_packed = ld_packed * 4;
  a.scale = static_cast<const uint8_t*>(scale);
  a.zp = reinterpret_cast<const uint8_t*>(zero_point);
  a.scale_f32 = 0;
  a.is_signed = is_signed != 0;
  a.stages_per_group = 1;
  const W4WidePlan plan = w4a8_wide_plan(M, N, K, group, 0);
  a.ksplit = 1;
  if (plan.parts >= 2 && split_k) {
    a.ksplit = plan.parts;
    a.tickets = reinterpret_cast<uint32_t*>(ws);
    a.partials = reinterpret_cast<float*>(ws + plan.ticket_bytes());
  }
  w4a16_launch(a, st);
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

extern "C" size_t mi355q_w4a8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int scale_dtype) {
  return w4a8_wide_plan(M, N, K, group, scale_dtype == MI355Q_F32).workspace_bytes();
}

extern "C" int mi355q_w4a8_gemm(const void* A, int fmt_a, int64_t lda, const int32_t* packed, int64_t ld_packed,
                                const void* scale, int scale_dtype, const int32_t* zero_point, int is_signed,
                                int64_t group, void* C, int out_dtype, int64_t ldc, int64_t M, int64_t N, int64_t K,
                                const float* sa_dev, float sa_host, int sa_mode, const void* bias,
                                void* workspace, size_t workspace_bytes, void* stream) {
  if (fmt_a != MI355Q_E4M3FN && fmt_a != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype != MI355Q_F32 && out_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (scale_dtype != MI355Q_F32 && scale_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (M < 0 || N < 0 || K < 0 || group <= 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (sa_mode != MI355Q_GS_NONE && sa_mode != MI355Q_GS_HOST && sa_mode != MI355Q_GS_DEV && sa_mode != MI355Q_GS_PER_ROW)
    return MI355Q_ERR_INVALID_ARGUMENT;
  if ((sa_mode == MI355Q_GS_DEV || sa_mode == MI355Q_GS_PER_ROW) && sa_dev == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (M == 0 || N == 0) return MI355Q_OK;
  if (C == nullptr || (K > 0 && (A == nullptr || packed == nullptr || scale == nullptr))) return MI355Q_ERR_INVALID_ARGUMENT;
  if (K % group != 0 || lda < K || ld_packed < N / 8 || ldc < N) return MI355Q_ERR_INVALID_ARGUMENT;
  // whole 16-byte pieces: K-major A, weight rows of N / 2 bytes, scale and zero-point rows
  const auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (N % 32 != 0 || K % 16 != 0 || lda % 16 != 0 || (ld_packed * 4) % 16 != 0 || group % kBK != 0 ||
      !al16(A) || !al16(packed) || !al16(scale) || (zero_point && !al16(zero_point)) ||
      M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL || (M + 63) / 64 > 65535)
    return MI355Q_ERR_UNSUPPORTED;
  W4Args a{};
  a.g.A = static_cast<const uint8_t*>(A);
  a.g.C = static_cast<uint8_t*>(C);
  a.g.lda = lda;
  a.g.ldc = ldc;
  a.g.M = (int)M;
  a.g.N = (int)N;
  a.g.K = (int)K;
  a.g.sa = sa_dev;
  a.g.sa_host = sa_host;
  a.g.sa_mode = sa_mode;
  a.g.sb_mode = MI355Q_GS_NONE;
  a.g.sb_host = 1.0f;
  a.g.bias = static_cast<const uint8_t*>(bias);
  a.g.bias_mode = bias ? MI355Q_BIAS_ROW_VECTOR : MI355Q_BIAS_NONE;
  a.g.out_bf16 = out_dtype == MI355Q_BF16;
  a.packed = reinterpret_cast<const uint8_t*>(packed);
  a.ld_packed = ld_packed * 4;
  a.scale = static_cast<const uint8_t*>(scale);
  a.zp = reinterpret_cast<const uint8_t*>(zero_point);
  a.scale_f32 = scale_dtype == MI355Q_F32;
  a.is_signed = is_signed != 0;
  a.stages_per_group = (int)(group / kBK);
  // the wide kernel where it applies: K in parts if the caller brought the room for the partial sums
  const W4WidePlan plan = w4a8_wide_plan(M, N, K, group, a.scale_f32);
  if (plan.parts >= 2 && workspace != nullptr) {
    if (!al16(workspace) || workspace_bytes < plan.workspace_bytes()) return MI355Q_ERR_WORKSPACE;
    a.ksplit = plan.parts;
    a.tickets = static_cast<uint32_t*>(workspace);
    a.partials = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + plan.ticket_bytes());
  } else if (plan.parts == 1) {
    a.ksplit = 1;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (K == 0) {
    // an empty sum: bias (or zero) through the same epilogue, with no stage to walk
    a.stages_per_group = 1;
  }
  if (fmt_a == MI355Q_E4M3FN) w4a8_launch_by_m<MI355Q_E4M3FN>(a, st);
  else w4a8_launch_by_m<MI355Q_E5M2>(a, st);
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}
