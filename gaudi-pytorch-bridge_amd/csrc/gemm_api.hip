// fp8_gemm_v2 C entry point: argument checks, kernel choice, and the any-shape
// fallback kernel.  The MFMA tile kernels live in gemm_tile.h.
#include "gemm_dispatch.h"

namespace mi355q {

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

// The tiled kernels move 16-byte chunks: each operand's leading dimension,
// batch stride and base address must be multiples of 16 bytes, and so must K
// where K is an operand's contiguous dimension (a chunk is either all inside K
// or all outside).  Where m or n is contiguous, the chunk that straddles the
// extent brings in bytes of the row's padding (ld >= extent rounded up): those
// columns only feed outputs that are never stored.
inline bool k_chunks_ok(int trans_a, int trans_b, int64_t K) {
  return K % 16 == 0 || (trans_a && !trans_b);
}
inline bool tiled_ok(const void* A, int trans_a, int64_t lda, const void* B, int trans_b,
                     int64_t ldb, int64_t M, int64_t N, int64_t K, int64_t stride_a,
                     int64_t stride_b) {
  if (!al16(A) || !al16(B) || lda % 16 || ldb % 16 || stride_a % 16 || stride_b % 16) return false;
  if (!k_chunks_ok(trans_a, trans_b, K)) return false;
  // a stage of the tiled kernels spans up to 256 rows of ld bytes, addressed with 31-bit offsets
  if (lda > (1LL << 22) || ldb > (1LL << 22)) return false;
  return M > 0 && N > 0 && K > 0;
}

}  // namespace mi355q

using namespace mi355q;

extern "C" {

const char* mi355q_fp8_gemm_variant(int trans_a, int64_t lda, int trans_b, int64_t ldb, int64_t M,
                                    int64_t N, int64_t K) {
  if (lda % 16 || ldb % 16 || !mi355q::k_chunks_ok(trans_a, trans_b, K)) return "simple";
  if (M > 128 && N > 128) {
    switch (mi355q::choose_tiles(M, N, 1)) {
      case mi355q::TileChoice::k256x256: return "tile256x256x128_mfma16x16x128";  // 32x32x64 with eight waves for epilogues beyond the fast bf16 one
      case mi355q::TileChoice::k256x128: return "tile256x128x128_mfma32x32x64";
      case mi355q::TileChoice::k128x128: return "tile128x128x128_mfma32x32x64";
    }
  }
  if (M <= 128) return "strip_Mx128x128_ring_mfma32x32x64";
  return "tile128x128x128_mfma32x32x64";
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
  g.fast_epi = 0;
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
    // A full [M, N] bias and an accumulate input are the same kind of addend (out_dtype, added in
    // fp32 after the scales): alone, the bias takes D's place, which the fast epilogue knows.
    if (gb.bias_mode == MI355Q_BIAS_FULL && gb.D == nullptr) {
      gb.D = gb.bias;
      gb.ldd = gb.ldbias;
      gb.stride_d = gb.stride_bias;
      gb.bias = nullptr;
      gb.bias_mode = MI355Q_BIAS_NONE;
    }
    gb.fast_epi = epilogue_fast_ok(gb, nb);
    if (tiled_ok(gb.A, trans_a, lda, gb.B, trans_b, ldb, M, N, K, stride_a, stride_b)) {
      const bool ak = !trans_a, bk = trans_b != 0;
      if (ak && bk) launch_gemm_kk(gb, fmt_a, fmt_b, nb, st);
      else if (ak) launch_gemm_km(gb, fmt_a, fmt_b, nb, st);
      else if (bk) launch_gemm_mk(gb, fmt_a, fmt_b, nb, st);
      else launch_gemm_mm(gb, fmt_a, fmt_b, nb, st);
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
