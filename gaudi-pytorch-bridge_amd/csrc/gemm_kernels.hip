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

// --------------------------------------------------------------------- kernel
template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
__global__ __launch_bounds__(kGemmThreads) void fp8_gemm_tile_kernel(GemmArgs g) {
  constexpr int TM = BM / 2, TN = BN / 2;   // per-wave tile
  constexpr int MT = TM / 32, NT = TN / 32; // MFMA tiles per wave
  __shared__ __attribute__((aligned(16))) uint8_t lds_a[BM * kBK];
  __shared__ __attribute__((aligned(16))) uint8_t lds_b[BN * kBK];

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

  // Epilogue.  acc[i][j][e] on this lane is C[m][n] with
  //   m = m0 + wm + 32 i + (lane % 32)
  //   n = n0 + wn + 32 j + 8 (e / 4) + 4 (lane / 32) + e % 4
  float sa_s = 1.0f, sb_s = 1.0f;
  if (g.sa_mode == MI355Q_GS_HOST) sa_s = g.sa_host;
  else if (g.sa_mode == MI355Q_GS_DEV) sa_s = g.sa[0];
  if (g.sb_mode == MI355Q_GS_HOST) sb_s = g.sb_host;
  else if (g.sb_mode == MI355Q_GS_DEV) sb_s = g.sb[0];

  uint8_t* C = g.C + batch * g.stride_c * (g.out_bf16 ? 2 : 4);
  const int es = g.out_bf16 ? 2 : 4;
  const uint8_t* D = g.D ? g.D + batch * g.stride_d * es : nullptr;
  const uint8_t* bias = g.bias ? g.bias + batch * g.stride_bias * es : nullptr;

#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m0 + wm + i * 32 + (lane & 31);
    if (m >= g.M) continue;
    float sa_m = sa_s, sb_m = sb_s;
    if (g.sa_mode == MI355Q_GS_PER_ROW) sa_m = g.sa[m];
    if (g.sb_mode == MI355Q_GS_PER_ROW) sb_m = g.sb[m];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn + j * 32 + q * 8 + (lane >> 5) * 4;
        if (n >= g.N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float sa_v = sa_m, sb_v = sb_m;
          const int ne = (n + e) < g.N ? (n + e) : g.N - 1;
          if (g.sa_mode == MI355Q_GS_PER_COL) sa_v = g.sa[ne];
          if (g.sb_mode == MI355Q_GS_PER_COL) sb_v = g.sb[ne];
          float t = acc[i][j][q * 4 + e] * sa_v;
          t = t * sb_v;
          if (g.bias_mode != MI355Q_BIAS_NONE) {
            const int64_t bo = g.bias_mode == MI355Q_BIAS_FULL ? (int64_t)m * g.ldbias + ne : ne;
            t += g.out_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(bias)[bo])
                            : reinterpret_cast<const float*>(bias)[bo];
          }
          if (D) {
            const int64_t d_o = (int64_t)m * g.ldd + ne;
            t += g.out_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(D)[d_o])
                            : reinterpret_cast<const float*>(D)[d_o];
          }
          v[e] = t;
        }
        const int64_t co = (int64_t)m * g.ldc + n;
        const bool full = n + 3 < g.N;
        if (g.out_bf16) {
          uint16_t* cp = reinterpret_cast<uint16_t*>(C) + co;
          if (full && ((reinterpret_cast<uintptr_t>(cp) & 7u) == 0)) {
            u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2*>(cp) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < g.N) cp[e] = (uint16_t)(pack_bf16x2(v[e], v[e]) & 0xffffu);
          }
        } else {
          float* cp = reinterpret_cast<float*>(C) + co;
          if (full && ((reinterpret_cast<uintptr_t>(cp) & 15u) == 0)) {
            f32x4 o = {v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f32x4*>(cp) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < g.N) cp[e] = v[e];
          }
        }
      }
    }
  }
}

// Any shape, any stride, any alignment: one thread per element of C.  Slow;
// only for problems the tiled kernel's alignment rules exclude.
template <int FMT_A, int FMT_B>
__global__ __launch_bounds__(256) void fp8_gemm_simple_kernel(GemmArgs g, int64_t a_sm, int64_t a_sk,
                                                              int64_t b_sk, int64_t b_sn) {
  const int n = blockIdx.x * 16 + (threadIdx.x & 15);
  const int m = blockIdx.y * 16 + (threadIdx.x >> 4);
  const int64_t batch = blockIdx.z;
  if (m >= g.M || n >= g.N) return;
  const uint8_t* A = g.A + batch * g.stride_a + (int64_t)m * a_sm;
  const uint8_t* B = g.B + batch * g.stride_b + (int64_t)n * b_sn;
  float acc = 0.0f;
  for (int k = 0; k < g.K; ++k)
    acc += cvt_f32x1<FMT_A>(A[(int64_t)k * a_sk]) * cvt_f32x1<FMT_B>(B[(int64_t)k * b_sk]);
  float sa = 1.0f, sb = 1.0f;
  if (g.sa_mode == MI355Q_GS_HOST) sa = g.sa_host;
  else if (g.sa_mode == MI355Q_GS_DEV) sa = g.sa[0];
  else if (g.sa_mode == MI355Q_GS_PER_ROW) sa = g.sa[m];
  else if (g.sa_mode == MI355Q_GS_PER_COL) sa = g.sa[n];
  if (g.sb_mode == MI355Q_GS_HOST) sb = g.sb_host;
  else if (g.sb_mode == MI355Q_GS_DEV) sb = g.sb[0];
  else if (g.sb_mode == MI355Q_GS_PER_ROW) sb = g.sb[m];
  else if (g.sb_mode == MI355Q_GS_PER_COL) sb = g.sb[n];
  float t = acc * sa;
  t = t * sb;
  const int es = g.out_bf16 ? 2 : 4;
  if (g.bias_mode != MI355Q_BIAS_NONE) {
    const uint8_t* bias = g.bias + batch * g.stride_bias * es;
    const int64_t bo = g.bias_mode == MI355Q_BIAS_FULL ? (int64_t)m * g.ldbias + n : n;
    t += g.out_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(bias)[bo])
                    : reinterpret_cast<const float*>(bias)[bo];
  }
  if (g.D) {
    const uint8_t* D = g.D + batch * g.stride_d * es;
    const int64_t d_o = (int64_t)m * g.ldd + n;
    t += g.out_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(D)[d_o])
                    : reinterpret_cast<const float*>(D)[d_o];
  }
  uint8_t* C = g.C + batch * g.stride_c * es;
  const int64_t co = (int64_t)m * g.ldc + n;
  if (g.out_bf16) reinterpret_cast<uint16_t*>(C)[co] = (uint16_t)(pack_bf16x2(t, t) & 0xffffu);
  else reinterpret_cast<float*>(C)[co] = t;
}

// ------------------------------------------------------------------- dispatch

inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The tiled kernel moves 16-byte chunks: the contiguous dimension of each
// operand, its leading dimension, batch stride and base address must all be
// multiples of 16 bytes.
inline bool tiled_ok(const void* A, int trans_a, int64_t lda, const void* B, int trans_b,
                     int64_t ldb, int64_t M, int64_t N, int64_t K, int64_t stride_a,
                     int64_t stride_b) {
  if (!al16(A) || !al16(B) || lda % 16 || ldb % 16 || stride_a % 16 || stride_b % 16) return false;
  if ((trans_a ? M : K) % 16) return false;
  if ((trans_b ? K : N) % 16) return false;
  return M > 0 && N > 0 && K > 0;
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

template <int FA, int FB>
void launch_by_layout(const GemmArgs& g, int trans_a, int trans_b, int64_t batch, hipStream_t st) {
  const bool ak = !trans_a, bk = trans_b != 0;
  if (ak && bk) launch_by_size<true, true, FA, FB>(g, batch, st);
  else if (ak && !bk) launch_by_size<true, false, FA, FB>(g, batch, st);
  else if (!ak && bk) launch_by_size<false, true, FA, FB>(g, batch, st);
  else launch_by_size<false, false, FA, FB>(g, batch, st);
}

}  // namespace mi355q

using namespace mi355q;

extern "C" {

const char* mi355q_fp8_gemm_variant(int trans_a, int64_t lda, int trans_b, int64_t ldb, int64_t M,
                                    int64_t N, int64_t K) {
  if (lda % 16 || ldb % 16 || (trans_a ? M : K) % 16 || (trans_b ? K : N) % 16) return "simple";
  return (M > 128 && N > 128) ? "tile256x256x128_mfma32x32x64" : "tile128x128x128_mfma32x32x64";
}

int mi355q_fp8_gemm(const void* A, int fmt_a, int trans_a, int64_t lda, const void* B, int fmt_b,
                    int trans_b, int64_t ldb, void* C, int out_dtype, int64_t ldc, int64_t M,
                    int64_t N, int64_t K, const float* sa_dev, float sa_host, int sa_mode,
                    const float* sb_dev, float sb_host, int sb_mode, const void* bias,
                    int bias_mode, int64_t ldbias, const void* D, int64_t ldd, int64_t batch,
                    int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t stride_d,
                    int64_t stride_bias, void* stream) {
  auto fmt_ok = [](int f) { return f == MI355Q_E4M3FN || f == MI355Q_E5M2; };
  auto mode_ok = [](int m, const float* p) {
    if (m < MI355Q_GS_NONE || m > MI355Q_GS_PER_COL) return false;
    return !(m >= MI355Q_GS_DEV && p == nullptr);
  };
  if (!fmt_ok(fmt_a) || !fmt_ok(fmt_b)) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype != MI355Q_F32 && out_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (M < 0 || N < 0 || K < 0 || batch < 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (!mode_ok(sa_mode, sa_dev) || !mode_ok(sb_mode, sb_dev)) return MI355Q_ERR_INVALID_ARGUMENT;
  if (bias_mode < MI355Q_BIAS_NONE || bias_mode > MI355Q_BIAS_FULL) return MI355Q_ERR_INVALID_ARGUMENT;
  if (bias_mode != MI355Q_BIAS_NONE && bias == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (M == 0 || N == 0 || batch == 0) return MI355Q_OK;
  if (C == nullptr || (K > 0 && (A == nullptr || B == nullptr))) return MI355Q_ERR_INVALID_ARGUMENT;
  if (M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;

  hipStream_t st = static_cast<hipStream_t>(stream);
  GemmArgs g;
  g.A = static_cast<const uint8_t*>(A);
  g.B = static_cast<const uint8_t*>(B);
  g.C = static_cast<uint8_t*>(C);
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.sa = sa_dev; g.sb = sb_dev; g.sa_host = sa_host; g.sb_host = sb_host;
  g.sa_mode = sa_mode; g.sb_mode = sb_mode;
  g.bias = static_cast<const uint8_t*>(bias);
  g.bias_mode = bias_mode; g.ldbias = ldbias;
  g.D = static_cast<const uint8_t*>(D);
  g.ldd = ldd;
  g.stride_a = stride_a; g.stride_b = stride_b; g.stride_c = stride_c; g.stride_d = stride_d;
  g.stride_bias = stride_bias;
  g.out_bf16 = out_dtype == MI355Q_BF16;
  g.tiles_m = g.tiles_n = 0;

  const int64_t kMaxBatch = 65535;
  for (int64_t b0 = 0; b0 < batch; b0 += kMaxBatch) {
    const int64_t nb = (batch - b0) < kMaxBatch ? (batch - b0) : kMaxBatch;
    GemmArgs gb = g;
    const int es = g.out_bf16 ? 2 : 4;
    gb.A = g.A + b0 * stride_a;
    gb.B = g.B + b0 * stride_b;
    gb.C = g.C + b0 * stride_c * es;
    if (g.D) gb.D = g.D + b0 * stride_d * es;
    if (g.bias) gb.bias = g.bias + b0 * stride_bias * es;
    if (tiled_ok(gb.A, trans_a, lda, gb.B, trans_b, ldb, M, N, K, stride_a, stride_b)) {
      if (fmt_a == MI355Q_E4M3FN && fmt_b == MI355Q_E4M3FN) launch_by_layout<MI355Q_E4M3FN, MI355Q_E4M3FN>(gb, trans_a, trans_b, nb, st);
      else if (fmt_a == MI355Q_E4M3FN) launch_by_layout<MI355Q_E4M3FN, MI355Q_E5M2>(gb, trans_a, trans_b, nb, st);
      else if (fmt_b == MI355Q_E4M3FN) launch_by_layout<MI355Q_E5M2, MI355Q_E4M3FN>(gb, trans_a, trans_b, nb, st);
      else launch_by_layout<MI355Q_E5M2, MI355Q_E5M2>(gb, trans_a, trans_b, nb, st);
    } else {
      const int64_t a_sm = trans_a ? 1 : lda, a_sk = trans_a ? lda : 1;
      const int64_t b_sk = trans_b ? 1 : ldb, b_sn = trans_b ? ldb : 1;
      dim3 grid((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16), (unsigned)nb);
      if (grid.y > 65535u) return MI355Q_ERR_UNSUPPORTED;
      if (fmt_a == MI355Q_E4M3FN && fmt_b == MI355Q_E4M3FN) fp8_gemm_simple_kernel<MI355Q_E4M3FN, MI355Q_E4M3FN><<<grid, 256, 0, st>>>(gb, a_sm, a_sk, b_sk, b_sn);
      else if (fmt_a == MI355Q_E4M3FN) fp8_gemm_simple_kernel<MI355Q_E4M3FN, MI355Q_E5M2><<<grid, 256, 0, st>>>(gb, a_sm, a_sk, b_sk, b_sn);
      else if (fmt_b == MI355Q_E4M3FN) fp8_gemm_simple_kernel<MI355Q_E5M2, MI355Q_E4M3FN><<<grid, 256, 0, st>>>(gb, a_sm, a_sk, b_sk, b_sn);
      else fp8_gemm_simple_kernel<MI355Q_E5M2, MI355Q_E5M2><<<grid, 256, 0, st>>>(gb, a_sm, a_sk, b_sk, b_sn);
    }
    if (hipGetLastError() != hipSuccess) return MI355Q_ERR_LAUNCH;
  }
  return MI355Q_OK;
}

}  // extern "C"
