// Fused int4-dequant GEMM for gfx950: fp8 activations times 4-bit weights (W4A8).
//
//   C[m, n] = out( sA[m] * sum_g s[g, n] * sum_{k in g} a[m, k] * (q[k, n] - z[g, n]) + bias[n] )
//
// The weights are what convert_from_int4 / convert_from_uint4 take (packed int32
// [K, N / 8], nibble i of word p is column 8 p + i; group-wise scales [K / g, N];
// packed zero-points [K / g, N / 8]), but they are never written out as bf16 [K, N]:
// a weight stage travels from HBM to LDS as packed nibbles (half the bytes of fp8
// weights, a quarter of bf16), the workgroup turns it into fp8 codes of the integers
// (q - z) in LDS (|q - z| <= 15 is exact in e4m3), the fp8 MFMA accumulates one K
// group at a time in fp32, and the group's scales multiply the partial sums as they
// are added to the totals.  So the weights enter the product exactly.
//
// Shaped like the strip kernel of gemm_skinny.h (weights streamed once through a deep
// LDS ring, one 4-wave workgroup per 128 columns); rows of A beyond 128 run as further
// row blocks that stream the weights again, which suits decode and small prefill
// batches, the shapes weight-only quantisation is used for.
//
// Per K stage of 128, one barrier: behind it a wave issues the loads of the stage S - 1
// ahead, reads the fragments of stage kt (A from the ring, the weights from the fp8 tile
// that the previous step unpacked) and issues its 2 MFMA blocks into the group's
// accumulators, then turns the packed tile of stage kt + 1 into the other fp8 tile (a
// thread converts 8 words: one column word of 8 rows, so its 8 zero-points are set up
// once per stage) while the MFMAs run, and at the end of a group adds scale * group to
// the totals.
#include "gemm_tile.h"

namespace mi355q {

constexpr int kW4Threads = 256;
constexpr int kW4Waves = 4;
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
};

template <int BM>
constexpr int w4_stage_bytes() { return BM * kBK + kW4PackedStage + kW4ScaleRow + kW4ZpRow; }

template <int BM>
constexpr int w4_stages() {
  constexpr int s = (160 * 1024 - 2 * kBK * kW4BN) / w4_stage_bytes<BM>();
  return s > 8 ? 8 : s;
}

// One 16-byte piece per lane, straight copy into LDS (lane l lands at dst + 16 l).  The
// s_nop covers a descriptor word that reached its scalar register through a vector
// instruction (five wait states before a memory instruction may read it).
__device__ __forceinline__ void w4_dma16(const i32x4& rsrc, int voff, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_dst), "v"(voff), "s"(rsrc)
               : "memory", "m0");
}

__device__ __forceinline__ i32x4 w4_rsrc(const uint8_t* base, int64_t bytes) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  const int64_t rec = bytes < 0 ? 0 : (bytes > 0x7fffffffLL ? 0x7fffffffLL : bytes);
  i32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((b >> 32) & 0xffffu));
  r[2] = __builtin_amdgcn_readfirstlane((int)rec);
  r[3] = 0x00020000;
  return r;
}

template <int BM, int FMT_A>
__global__ __launch_bounds__(kW4Threads) void w4a8_gemm_kernel(W4Args a) {
  constexpr int MT = BM / 32;
  constexpr int S = w4_stages<BM>();
  constexpr int kStage = w4_stage_bytes<BM>();
  constexpr int kOffPacked = BM * kBK, kOffScale = kOffPacked + kW4PackedStage, kOffZp = kOffScale + kW4ScaleRow;
  using LA = DmaLoader<true, BM, kBK, kW4Waves>;
  using GB = TileGeom<false, kBK, kW4BN>;  // the unpacked weight tile: 128 k-rows of 128 fp8 columns
  // per wave and stage: its share of A, two 1 KiB regions of packed weights, the scale row, the zero-point row
  constexpr int kOps = LA::kPerWave + 2 + 2;
  constexpr int kInFlight = (S - 3) * kOps;  // stage kt + 1 is needed while stage kt is multiplied
  static_assert(S >= 4 && kInFlight <= 63, "vmcnt holds 6 bits");
  static_assert(kStage % 1024 == 0, "stages stay 1 KiB aligned");
  static_assert(kW4Waves * epilogue_stage_floats<MT, 1>() * 4 <= S * kStage, "epilogue area overlays the ring");
  constexpr int kTile = kBK * kW4BN;  // one unpacked fp8 tile
  __shared__ __attribute__((aligned(1024))) uint8_t lds[S * kStage + 2 * kTile];
  uint8_t* const unp = lds + S * kStage;  // two tiles, used in turn

  // this workgroup's rows and columns
  GemmArgs g = a.g;
  const int m_base = blockIdx.y * BM;
  g.A += (int64_t)m_base * g.lda;
  g.C += (int64_t)m_base * g.ldc * (g.out_bf16 ? 2 : 4);
  if (g.sa_mode == MI355Q_GS_PER_ROW) g.sa += m_base;
  g.M = g.M - m_base < BM ? g.M - m_base : BM;
  const int n0 = blockIdx.x * kW4BN;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = lane_id_here();
  const int wn = wave * 32;
  const int KT = (g.K + kBK - 1) / kBK;

  LA la;
  la.init(g.A, g.lda, 0, g.M, g.K);
  la.clamp_rows(g.lda, g.M);
  // packed weights: this wave's two regions are k-rows 32 wave .. 32 wave + 31 of the stage (16 rows of 64 bytes each)
  const int64_t packed_bytes = (int64_t)(g.K - 1) * a.ld_packed + (((g.N + 31) & ~31) - n0) / 2;
  const uint8_t* const packed0 = a.packed + n0 / 2;
  const int voff_packed = (wave * 32 + (lane >> 2)) * (int)a.ld_packed + (lane & 3) * 16;
  const int region_packed = 16 * (int)a.ld_packed;
  const int es = a.scale_f32 ? 4 : 2;
  const int64_t scale_row_bytes = (int64_t)(g.N - n0 < kW4BN ? g.N - n0 : kW4BN) * es;
  const int64_t zp_row_bytes = (int64_t)(g.N - n0 < kW4BN ? g.N - n0 : kW4BN) / 2;

  int issued = 0;  // stages issued so far: stage `issued` goes out next
  auto issue_stage = [&](int off) {
    const int stage = issued;
    const uint32_t base = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)(lds + off);
    static_for<LA::kPerWave>([&](auto ic) { la.template issue_one<decltype(ic)::value, true>(lds + off, stage * kBK, g.K); });
    la.advance();
    // beyond K everything is out of range and arrives as zeros (A's zeros make the products vanish)
    const int64_t k_off = (int64_t)stage * kBK * a.ld_packed;
    const i32x4 rp = w4_rsrc(packed0 + k_off, stage < KT ? packed_bytes - k_off : 0);
    w4_dma16(rp, voff_packed, base + kOffPacked + (wave * 2) * 1024);
    w4_dma16(rp, voff_packed + region_packed, base + kOffPacked + (wave * 2 + 1) * 1024);
    const int grp = stage / a.stages_per_group;
    const i32x4 rs = w4_rsrc(a.scale + ((int64_t)grp * g.N + n0) * es, stage < KT ? scale_row_bytes : 0);
    w4_dma16(rs, lane * 16, base + kOffScale);
    // (without zero-points the scale row is fetched once more: every stage's loads are of the same
    // number and all go to memory, which the counted wait below relies on)
    const i32x4 rz = a.zp ? w4_rsrc(a.zp + ((int64_t)grp * g.N + n0) / 2, stage < KT ? zp_row_bytes : 0) : rs;
    w4_dma16(rz, lane * 16, base + kOffZp);
    ++issued;
  };

  f32x16 total[MT][1], part[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) total[i][0][e] = 0.0f;

#pragma unroll
  for (int s = 0; s < S - 1; ++s) issue_stage(s * kStage);

  // unpacking: this thread's column word and its 8 rows of the stage
  const int uw = threadIdx.x & 15, ur0 = threadIdx.x >> 4;
  const uint32_t flip = a.is_signed ? 0x88888888u : 0u;  // signed nibble s = (q ^ 8) - 8
  const float zbias = a.is_signed ? 8.0f : 0.0f;

  // packed nibbles of the stage at `st` -> fp8 codes of (q - z) in the tile at `dst`
  auto unpack = [&](const uint8_t* st, uint8_t* dst) {
    const uint32_t zw = (a.zp ? *reinterpret_cast<const uint32_t*>(st + kOffZp + uw * 4) : 0u) ^ flip;
    float z[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = a.zp ? (float)((zw >> (4 * i)) & 15u) : zbias;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = ur0 + 16 * i;
      const uint32_t w = *reinterpret_cast<const uint32_t*>(st + kOffPacked + r * 64 + uw * 4) ^ flip;
      uint32_t ev = w & 0x0f0f0f0fu, od = (w >> 4) & 0x0f0f0f0fu;  // nibbles 0, 2, 4, 6 / 1, 3, 5, 7 as bytes
      // kept opaque: byte j of these converts in one instruction (v_cvt_f32_ubyte<j>), where the
      // compiler would otherwise go back to w with a bit-field extract per nibble
      asm("" : "+v"(ev));
      asm("" : "+v"(od));
      const float f0 = (float)(ev & 0xffu) - z[0], f1 = (float)(od & 0xffu) - z[1];
      const float f2 = (float)((ev >> 8) & 0xffu) - z[2], f3 = (float)((od >> 8) & 0xffu) - z[3];
      const float f4 = (float)((ev >> 16) & 0xffu) - z[4], f5 = (float)((od >> 16) & 0xffu) - z[5];
      const float f6 = (float)(ev >> 24) - z[6], f7 = (float)(od >> 24) - z[7];
      int lo = __builtin_amdgcn_cvt_pk_fp8_f32(f0, f1, 0, false);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(f2, f3, lo, true);
      int hi = __builtin_amdgcn_cvt_pk_fp8_f32(f4, f5, 0, false);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(f6, f7, hi, true);
      *reinterpret_cast<u32x2*>(dst + GB::lds_offset(r, uw >> 1) + (uw & 1) * 8) = u32x2{(uint32_t)lo, (uint32_t)hi};
    }
  };
  // waits until at most min(later, S - 3) stages' loads of this wave are outstanding
  auto wait_for_stage = [&](int later) {
    static_for<S - 2>([&](auto sc) {
      constexpr int n = decltype(sc)::value;  // 0 .. S - 3
      constexpr int cnt = n * kOps;
      if (later == n || (n == S - 3 && later > n) || (n == 0 && later < 0))
        __builtin_amdgcn_s_waitcnt((cnt & 15) | ((cnt >> 4) << 14) | 0x0070);
    });
  };

  // stage 0 -> fp8 tile 0
  wait_for_stage(KT - 2);
  __syncthreads();
  unpack(lds, unp);

  int rd_off = 0, wr_off = (S - 1) * kStage;
  for (int kt = 0; kt < KT; ++kt) {
    // The loads of stage kt + 1 have landed once only those of later stages are outstanding; the
    // zero-fill loads past K complete at once and are not counted (see gemm_skinny.h).
    wait_for_stage(KT - 3 - kt);
    // everyone's part of stage kt + 1 is in LDS and fp8 tile kt & 1 is complete; everyone is done
    // with the other fp8 tile and with stage kt - 1
    __syncthreads();
    issue_stage(wr_off);
    const uint8_t* st = lds + rd_off;
    const uint8_t* tile = unp + (kt & 1) * kTile;
    int next_off = rd_off + kStage;
    if (next_off == S * kStage) next_off = 0;

    // ---- the stage's two MFMA blocks into the group's partial sums
    const bool group_start = kt % a.stages_per_group == 0;
#pragma unroll
    for (int ks = 0; ks < kBK / 64; ++ks) {
      i32x8 fb, fa[MT];
      static_for<4>([&](auto pc) { read_fragment_part<false, kW4BN, decltype(pc)::value>(tile, wn, ks, fb); });
      static_for<MT>([&](auto ic) {
        static_for<2>([&](auto pc) {
          read_fragment_part<true, BM, decltype(pc)::value>(st, decltype(ic)::value * 32, ks, fa[decltype(ic)::value]);
        });
      });
      static_for<MT>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const f32x16 c = (ks == 0 && group_start) ? zero : part[i];
        part[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb, fa[i], c, 0, mfma_code<FMT_A>(), 0, 0, 0, 0);
      });
    }
    // ---- the next stage's weights, while the MFMAs run (past K: zeros times A's zeros)
    unpack(lds + next_off, unp + ((kt + 1) & 1) * kTile);
    // ---- end of a group: total += scale * partial sums
    if ((kt + 1) % a.stages_per_group == 0 || kt + 1 == KT) {
      // this lane's columns: wn + 8 q + 4 (lane / 32) + e, q = 0 .. 3, e = 0 .. 3
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = wn + 8 * q + 4 * (lane >> 5);
        float sc[4];
        if (a.scale_f32) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(st + kOffScale + col * 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) sc[e] = v[e];
        } else {
          const u32x2 v = *reinterpret_cast<const u32x2*>(st + kOffScale + col * 2);
          sc[0] = __uint_as_float(v[0] << 16);
          sc[1] = __uint_as_float(v[0] & 0xffff0000u);
          sc[2] = __uint_as_float(v[1] << 16);
          sc[3] = __uint_as_float(v[1] & 0xffff0000u);
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int e = 0; e < 4; ++e) total[i][0][4 * q + e] = __builtin_fmaf(part[i][4 * q + e], sc[e], total[i][0][4 * q + e]);
      }
    }
    rd_off = next_off;
    wr_off += kStage;
    if (wr_off == S * kStage) wr_off = 0;
  }
  // the ring is idle (zero-fill loads of the stages past K included) before the epilogue overlays it
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  float* stage_area = reinterpret_cast<float*>(lds) + wave * epilogue_stage_floats<MT, 1>();
  epilogue<MT, 1>(g, 0, total, 0, n0 + wn, stage_area);
}

template <int BM, int FMT_A>
void w4a8_launch(const W4Args& a, hipStream_t st) {
  dim3 grid((unsigned)((a.g.N + kW4BN - 1) / kW4BN), (unsigned)((a.g.M + BM - 1) / BM));
  w4a8_gemm_kernel<BM, FMT_A><<<grid, kW4Threads, 0, st>>>(a);
}

template <int FMT_A>
void w4a8_launch_by_m(const W4Args& a, hipStream_t st) {
  if (a.g.M <= 32) w4a8_launch<32, FMT_A>(a, st);
  else if (a.g.M <= 64) w4a8_launch<64, FMT_A>(a, st);
  else w4a8_launch<128, FMT_A>(a, st);
}

}  // namespace mi355q

using namespace mi355q;

extern "C" int mi355q_w4a8_gemm(const void* A, int fmt_a, int64_t lda, const int32_t* packed, int64_t ld_packed,
                                const void* scale, int scale_dtype, const int32_t* zero_point, int is_signed,
                                int64_t group, void* C, int out_dtype, int64_t ldc, int64_t M, int64_t N, int64_t K,
                                const float* sa_dev, float sa_host, int sa_mode, const void* bias, void* stream) {
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
      M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL || (M + 127) / 128 > 65535)
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
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (K == 0) {
    // an empty sum: bias (or zero) through the same epilogue, with no stage to walk
    a.stages_per_group = 1;
  }
  if (fmt_a == MI355Q_E4M3FN) w4a8_launch_by_m<MI355Q_E4M3FN>(a, st);
  else w4a8_launch_by_m<MI355Q_E5M2>(a, st);
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}
