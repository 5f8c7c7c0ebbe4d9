// fp8 x fp8 -> fp32-accumulate -> bf16/fp32 GEMM for gfx950 (fp8_gemm_v2).
//
// Tiled kernel: a 256-thread workgroup (4 waves, 2x2) owns a BM x BN tile of C
// and walks K in steps of 128 bytes.  Operand tiles are staged in LDS in 16-byte
// chunks whose position inside a row is XOR-swizzled with the row number, which
// makes the 128-bit fragment reads bank-conflict free.  Each wave computes its
// (BM/2) x (BN/2) sub-tile with v_mfma_f32_32x32x64_f8f6f4 (fp8/bf8 operands,
// 64 k per instruction).
//
// Operand layouts.  An operand whose K index is contiguous in memory (A with
// trans_a == 0, B with trans_b != 0) is "K-major": a lane's 32-byte MFMA
// fragment is two ds_read_b128.  The other layout (A with trans_a != 0, the
// usual B [K, N] with trans_b == 0) is "MN-major": rows of LDS hold 16 byte
// runs along m or n, and ds_read_b64_tr_b8 transposes 8 k-rows x 16 columns
// inside each group of 16 lanes on the way into registers.
//
// The MFMA is issued with the B fragment as its first operand, so that a lane
// ends up holding 4 consecutive n for one m: the epilogue stores 8 bytes (bf16)
// or 16 bytes (fp32) per lane, and per-row / per-column scales, bias and the
// accumulate input are applied in fp32 before the single final rounding.
#pragma once
#include <type_traits>

#include "device_common.h"

namespace mi355q {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define LDS_AS __attribute__((address_space(3)))

constexpr int kGemmThreads = 256;
constexpr int kBK = 128;  // bytes (= fp8 elements) of K per LDS stage

struct GemmArgs {
  const uint8_t* A;
  const uint8_t* B;
  uint8_t* C;
  int64_t lda, ldb, ldc;
  int M, N, K;
  const float* sa;
  const float* sb;
  float sa_host, sb_host;
  int sa_mode, sb_mode;
  const uint8_t* bias;
  int bias_mode;
  int64_t ldbias;
  const uint8_t* D;
  int64_t ldd;
  int64_t stride_a, stride_b, stride_c, stride_d, stride_bias;
  int out_bf16;
  int tiles_m, tiles_n;
};

// MFMA format codes of the f8f6f4 instructions: 0 = e4m3, 1 = e5m2.
template <int FMT>
constexpr int mfma_code() { return FMT == MI355Q_E5M2 ? 1 : 0; }

// ----------------------------------------------------------------- tile loader
//
// ROWS x ROW_BYTES bytes of LDS, rows hold 16-byte chunks.  For a K-major
// operand a row is one m (or n) and ROW_BYTES == kBK; for an MN-major operand a
// row is one k and ROW_BYTES == the tile extent along m (or n).
template <int ROWS, int ROW_BYTES>
struct TileGeom {
  static constexpr int kChunksPerRow = ROW_BYTES / 16;
  static constexpr int kChunks = ROWS * kChunksPerRow;
  static constexpr int kPerThread = kChunks / kGemmThreads;
  static constexpr int kSwzMask = (kChunksPerRow >= 8 ? 8 : kChunksPerRow) - 1;
  static_assert(kChunks % kGemmThreads == 0, "tile must split evenly over the block");
  __device__ static __forceinline__ int lds_offset(int row, int chunk) {
    return row * ROW_BYTES + ((chunk ^ (row & kSwzMask)) << 4);
  }
};

// Loads one operand tile from global memory into registers.
//   KMAJOR: rows index m/n (clamped to the last valid row), chunks walk k
//           (chunks at or beyond K read as zero)
//   else  : rows index k (rows at or beyond K read as zero), chunks walk m/n
//           (chunks at or beyond the extent read as zero)
template <bool KMAJOR, int EXT>  // EXT: tile extent along m/n
struct TileLoader {
  using G = TileGeom<KMAJOR ? EXT : kBK, KMAJOR ? kBK : EXT>;
  u32x4 regs[G::kPerThread];

  __device__ __forceinline__ void load(const uint8_t* base, int64_t ld, int mn0, int mn_extent,
                                       int k0, int K) {
#pragma unroll
    for (int i = 0; i < G::kPerThread; ++i) {
      const int q = threadIdx.x + i * kGemmThreads;
      const int row = q / G::kChunksPerRow, c = q % G::kChunksPerRow;
      u32x4 v = {0u, 0u, 0u, 0u};
      if constexpr (KMAJOR) {
        int r = mn0 + row;
        r = r < mn_extent ? r : mn_extent - 1;
        const int k = k0 + c * 16;
        if (k < K) v = *reinterpret_cast<const u32x4*>(base + (int64_t)r * ld + k);
      } else {
        const int k = k0 + row;
        const int mn = mn0 + c * 16;
        if (k < K && mn < mn_extent) v = *reinterpret_cast<const u32x4*>(base + (int64_t)k * ld + mn);
      }
      regs[i] = v;
    }
  }

  __device__ __forceinline__ void store(uint8_t* lds) const {
#pragma unroll
    for (int i = 0; i < G::kPerThread; ++i) {
      const int q = threadIdx.x + i * kGemmThreads;
      const int row = q / G::kChunksPerRow, c = q % G::kChunksPerRow;
      *reinterpret_cast<u32x4*>(lds + G::lds_offset(row, c)) = regs[i];
    }
  }
};

// 32-byte MFMA fragment (32 rows of m/n x 32 k for this lane's k-half) from LDS.
template <bool KMAJOR, int EXT>
__device__ __forceinline__ i32x8 read_fragment(const uint8_t* lds, int mn_base, int ksub) {
  using G = TileGeom<KMAJOR ? EXT : kBK, KMAJOR ? kBK : EXT>;
  const int lane = threadIdx.x & 63;
  i32x8 f;
  if constexpr (KMAJOR) {
    const int row = mn_base + (lane & 31);
    const int c0 = ksub * 4 + (lane >> 5) * 2;
    const u32x4 lo = *reinterpret_cast<const u32x4*>(lds + G::lds_offset(row, c0));
    const u32x4 hi = *reinterpret_cast<const u32x4*>(lds + G::lds_offset(row, c0 + 1));
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
  } else {
    // Within each group of 16 lanes, lanes 2r and 2r+1 point at the two 8-byte
    // halves of k-row r; after the transposing read lane i of the group holds
    // column i for those 8 k-rows.
    const int blk = lane >> 4, i = lane & 15;
    const int r = i >> 1, h = i & 1;
    const int col = mn_base + (blk & 1) * 16;  // first column of this 16-lane group
    const int kb = ksub * 64 + (blk >> 1) * 32;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int krow = kb + kk * 8 + r;
      const int off = G::lds_offset(krow, col >> 4) + h * 8;
      const i32x2 t = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (LDS_AS i32x2*)((LDS_AS uint8_t*)lds + off));
      f[2 * kk] = t[0];
      f[2 * kk + 1] = t[1];
    }
  }
  return f;
}

// ------------------------------------------------------------------- epilogue
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

__device__ __forceinline__ float load_out_as_f32(const uint8_t* p, int64_t idx, int bf16) {
  return bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[idx])
              : reinterpret_cast<const float*>(p)[idx];
}

// Stores 4 consecutive output columns n..n+3 of row m (columns at or beyond N are skipped).
__device__ __forceinline__ void store4(uint8_t* C, int out_bf16, int64_t ldc, int m, int n, int N,
                                       const float (&v)[4]) {
  const int64_t co = (int64_t)m * ldc + n;
  const bool full = n + 3 < N;
  if (out_bf16) {
    uint16_t* cp = reinterpret_cast<uint16_t*>(C) + co;
    if (full && ((reinterpret_cast<uintptr_t>(cp) & 7u) == 0)) {
      u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
      *reinterpret_cast<u32x2*>(cp) = o;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) cp[e] = (uint16_t)(pack_bf16x2(v[e], v[e]) & 0xffffu);
    }
  } else {
    float* cp = reinterpret_cast<float*>(C) + co;
    if (full && ((reinterpret_cast<uintptr_t>(cp) & 15u) == 0)) {
      f32x4 o = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4*>(cp) = o;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) cp[e] = v[e];
    }
  }
}

// v = acc * sA * sB + bias + D in fp32, one rounding to the output type.
//   acc[i][j][e] on this lane is C[m][n] with
//     m = m_lane + 32 i,   n = n_lane + 32 j + 8 (e / 4) + e % 4
//   where m_lane already holds lane % 32 and n_lane holds 4 (lane / 32).
// The common forms (scalar or per-row A scale, scalar or per-column B scale, no
// bias or an [N] bias, no accumulate input) take the register path with
// compile-time accumulator indices.  Everything else goes through `stage`, a
// per-wave LDS area of 32 x (32 NT) floats used as an indexable copy of one
// row of accumulator tiles, so that the general code is a small runtime loop.
template <int MT, int NT>
__device__ __forceinline__ void epilogue(const GemmArgs& g, int64_t batch, f32x16 (&acc)[MT][NT],
                                         int m_lane, int n_lane, float* stage) {
  const int es = g.out_bf16 ? 2 : 4;
  uint8_t* C = g.C + batch * g.stride_c * es;
  const uint8_t* D = g.D ? g.D + batch * g.stride_d * es : nullptr;
  const uint8_t* bias = g.bias ? g.bias + batch * g.stride_bias * es : nullptr;
  float sa_s = 1.0f, sb_s = 1.0f;
  if (g.sa_mode == MI355Q_GS_HOST) sa_s = g.sa_host;
  else if (g.sa_mode == MI355Q_GS_DEV) sa_s = g.sa[0];
  if (g.sb_mode == MI355Q_GS_HOST) sb_s = g.sb_host;
  else if (g.sb_mode == MI355Q_GS_DEV) sb_s = g.sb[0];

  const bool fast = g.sa_mode != MI355Q_GS_PER_COL && g.sb_mode != MI355Q_GS_PER_ROW &&
                    g.bias_mode != MI355Q_BIAS_FULL && D == nullptr;
  if (fast) {
    float sa_m[MT];
    static_for<MT>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      const int m = m_lane + 32 * i;
      sa_m[i] = (g.sa_mode == MI355Q_GS_PER_ROW && m < g.M) ? g.sa[m] : sa_s;
    });
    static_for<NT>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      static_for<4>([&](auto qc) {
        constexpr int q = decltype(qc)::value;
        const int n = n_lane + 32 * j + 8 * q;
        if (n < g.N) {
          float sb4[4], b4[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int ne = (n + e) < g.N ? (n + e) : g.N - 1;
            sb4[e] = g.sb_mode == MI355Q_GS_PER_COL ? g.sb[ne] : sb_s;
            b4[e] = g.bias_mode == MI355Q_BIAS_ROW_VECTOR ? load_out_as_f32(bias, ne, g.out_bf16) : 0.0f;
          }
          static_for<MT>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int m = m_lane + 32 * i;
            if (m < g.M) {
              float v[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                float t = acc[i][j][q * 4 + e] * sa_m[i];
                t = t * sb4[e];
                v[e] = t + b4[e];
              }
              store4(C, g.out_bf16, g.ldc, m, n, g.N, v);
            }
          });
        }
      });
    });
    return;
  }

  static_for<MT>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
    // park this row of tiles in the wave's staging area: slot (j*16 + e) * 64 + lane
    const int lane = threadIdx.x & 63;
    static_for<NT>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
#pragma unroll
      for (int e = 0; e < 16; ++e) stage[(j * 16 + e) * 64 + lane] = acc[i][j][e];
    });
    const int m = m_lane + 32 * i;
    if (m < g.M) {
      float sa_m = sa_s, sb_m = sb_s;
      if (g.sa_mode == MI355Q_GS_PER_ROW) sa_m = g.sa[m];
      if (g.sb_mode == MI355Q_GS_PER_ROW) sb_m = g.sb[m];
      for (int jq = 0; jq < NT * 4; ++jq) {
        const int j = jq >> 2, q = jq & 3;
        const int n = n_lane + 32 * j + 8 * q;
        if (n >= g.N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int ne = (n + e) < g.N ? (n + e) : g.N - 1;
          float sa_v = sa_m, sb_v = sb_m;
          if (g.sa_mode == MI355Q_GS_PER_COL) sa_v = g.sa[ne];
          if (g.sb_mode == MI355Q_GS_PER_COL) sb_v = g.sb[ne];
          float t = stage[(j * 16 + q * 4 + e) * 64 + lane] * sa_v;
          t = t * sb_v;
          if (g.bias_mode == MI355Q_BIAS_ROW_VECTOR) t += load_out_as_f32(bias, ne, g.out_bf16);
          else if (g.bias_mode == MI355Q_BIAS_FULL) t += load_out_as_f32(bias, (int64_t)m * g.ldbias + ne, g.out_bf16);
          if (D) t += load_out_as_f32(D, (int64_t)m * g.ldd + ne, g.out_bf16);
          v[e] = t;
        }
        store4(C, g.out_bf16, g.ldc, m, n, g.N, v);
      }
    }
  });
}

// --------------------------------------------------------------------- kernel
template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
__global__ __launch_bounds__(kGemmThreads) void fp8_gemm_tile_kernel(GemmArgs g) {
  constexpr int TM = BM / 2, TN = BN / 2;   // per-wave tile
  constexpr int MT = TM / 32, NT = TN / 32; // MFMA tiles per wave
  static_assert(BM == BN, "the epilogue staging area assumes square tiles");
  __shared__ __attribute__((aligned(16))) uint8_t lds[(BM + BN) * kBK];
  uint8_t* const lds_a = lds;
  uint8_t* const lds_b = lds + BM * kBK;

  // Tile order.  Workgroups are dealt to the 8 XCDs round-robin by id; give
  // each XCD a contiguous range of tiles, and walk tiles in column groups of
  // kGroupM rows so that the tiles resident on one XCD share A and B panels in
  // its L2.
  const int nb = gridDim.x;
  const int bid = blockIdx.x;
  const int per = nb >> 3, rem = nb & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  const int logical = xcd < rem ? xcd * (per + 1) + idx : rem * (per + 1) + (xcd - rem) * per + idx;
  constexpr int kGroupM = 8;
  const int group_size = kGroupM * g.tiles_n;
  const int grp = logical / group_size;
  const int first_m = grp * kGroupM;
  const int gm = (g.tiles_m - first_m) < kGroupM ? (g.tiles_m - first_m) : kGroupM;
  const int in_grp = logical - grp * group_size;
  const int tile_m = first_m + in_grp % gm;
  const int tile_n = in_grp / gm;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int64_t batch = blockIdx.y;
  const uint8_t* A = g.A + batch * g.stride_a;
  const uint8_t* B = g.B + batch * g.stride_b;

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave >> 1) * TM, wn = (wave & 1) * TN;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  TileLoader<A_KMAJOR, BM> la;
  TileLoader<B_KMAJOR, BN> lb;
  const int KT = (g.K + kBK - 1) / kBK;
  la.load(A, g.lda, m0, g.M, 0, g.K);
  lb.load(B, g.ldb, n0, g.N, 0, g.K);

  for (int kt = 0; kt < KT; ++kt) {
    la.store(lds_a);
    lb.store(lds_b);
    __syncthreads();
    if (kt + 1 < KT) {
      la.load(A, g.lda, m0, g.M, (kt + 1) * kBK, g.K);
      lb.load(B, g.ldb, n0, g.N, (kt + 1) * kBK, g.K);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      i32x8 fa[MT], fb[NT];
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[i] = read_fragment<A_KMAJOR, BM>(lds_a, wm + i * 32, ks);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[j] = read_fragment<B_KMAJOR, BN>(lds_b, wn + j * 32, ks);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              fb[j], fa[i], acc[i][j], mfma_code<FMT_B>(), mfma_code<FMT_A>(), 0, 0, 0, 0);
    }
    __syncthreads();
  }

  // The operand tiles are dead (the K loop ends with a barrier); the general
  // epilogue reuses the LDS as per-wave staging: 4 waves x 16 NT x 64 floats.
  static_assert((BM + BN) * kBK >= 4 * 16 * NT * 64 * 4, "staging area does not fit");
  float* stage = reinterpret_cast<float*>(lds) + wave * (16 * NT * 64);
  epilogue<MT, NT>(g, batch, acc, m0 + wm + (lane & 31), n0 + wn + (lane >> 5) * 4, stage);
}

template <int BM, int BN, bool AK, bool BK_, int FA, int FB>
void launch_tile(const GemmArgs& g, int64_t batch, hipStream_t st) {
  GemmArgs a = g;
  a.tiles_m = (g.M + BM - 1) / BM;
  a.tiles_n = (g.N + BN - 1) / BN;
  dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)batch);
  fp8_gemm_tile_kernel<BM, BN, AK, BK_, FA, FB><<<grid, kGemmThreads, 0, st>>>(a);
}

template <bool AK, bool BK_, int FA, int FB>
void launch_by_size(const GemmArgs& g, int64_t batch, hipStream_t st) {
  if (g.M > 128 && g.N > 128) launch_tile<256, 256, AK, BK_, FA, FB>(g, batch, st);
  else launch_tile<128, 128, AK, BK_, FA, FB>(g, batch, st);
}

// One translation unit per operand layout instantiates this (gemm_inst_*.hip).
template <bool AK, bool BK_>
void launch_by_format(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st) {
  if (fmt_a == MI355Q_E4M3FN && fmt_b == MI355Q_E4M3FN) launch_by_size<AK, BK_, MI355Q_E4M3FN, MI355Q_E4M3FN>(g, batch, st);
  else if (fmt_a == MI355Q_E4M3FN) launch_by_size<AK, BK_, MI355Q_E4M3FN, MI355Q_E5M2>(g, batch, st);
  else if (fmt_b == MI355Q_E4M3FN) launch_by_size<AK, BK_, MI355Q_E5M2, MI355Q_E4M3FN>(g, batch, st);
  else launch_by_size<AK, BK_, MI355Q_E5M2, MI355Q_E5M2>(g, batch, st);
}

// A K-major / B K-major etc.; defined in gemm_inst_*.hip
void launch_gemm_kk(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_km(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_mk(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_mm(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);

}  // namespace mi355q
