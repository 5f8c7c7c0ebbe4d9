// sum_fp8 and softmax_fp8 for gfx950 and their C entry points.
//
// Both are HBM-bound row / column reductions over fp8 (or bf16) data.  Loads go
// through buffer descriptors that end with the row or block they cover, so the
// bodies have no divergent branch around a load and every lane's loads are in
// flight before the first is used (see cast_kernels.hip).
#include <mutex>

#include "device_common.h"

namespace mi355q {

constexpr int kRedThreads = 256;
constexpr uint32_t kRsrcFlags = 0x00020000;

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = __builtin_fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

__device__ __forceinline__ void store_sum(void* out, int out_dtype, int64_t i, float v) {
  switch (out_dtype) {
    case MI355Q_F32: static_cast<float*>(out)[i] = v; break;
    case MI355Q_BF16: static_cast<uint16_t*>(out)[i] = (uint16_t)(pack_bf16x2(v, v) & 0xffffu); break;
    case MI355Q_E4M3FN: static_cast<uint8_t*>(out)[i] = (uint8_t)(cvt_fp8x4<MI355Q_E4M3FN>(v, v, v, v) & 0xffu); break;
    default: static_cast<uint8_t*>(out)[i] = (uint8_t)(cvt_fp8x4<MI355Q_E5M2>(v, v, v, v) & 0xffu); break;
  }
}

// -------------------------------------------------------------------- sum_fp8
//
// x is [outer, R, inner] fp8.  A launch covers R in `splits` slices of `per`
// rows; with one slice the kernels write the result, else fp32 partial sums
// [splits, outer, inner] that sum_finish_kernel adds in slice order.  Every
// sum has a fixed order, so results do not change from run to run.

// inner > 1: a lane owns VEC consecutive inner positions; the four waves of a workgroup take
// every fourth row of the slice (so 16 row segments of 64 * VEC bytes are in flight per
// workgroup) and their sums are added through LDS, in wave order.
template <int FMT, int VEC>
__global__ __launch_bounds__(kRedThreads) void sum_columns_kernel(const uint8_t* __restrict__ x, int64_t outer, int64_t R,
                                                                  int64_t inner, int64_t per, int splits, int col_blocks,
                                                                  void* __restrict__ out, int out_dtype,
                                                                  float* __restrict__ partial) {
  constexpr int WAVES = kRedThreads / 64;
  __shared__ float part[WAVES - 1][64][VEC];
  // blockIdx.x = outer index * col_blocks + column block (outer can exceed the 65535 of grid.y)
  const int64_t o = blockIdx.x / col_blocks;
  const int s = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t c0 = ((int64_t)(blockIdx.x - o * col_blocks) * 64 + lane) * VEC;
  const int64_t r0 = s * per;
  const int64_t r1 = (r0 + per) < R ? (r0 + per) : R;
  const bool inside = c0 < inner;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
  auto load = [&](const uint8_t* p, uint32_t (&w)[VEC >= 4 ? VEC / 4 : 1]) {
    if constexpr (VEC == 16) {
      const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
#pragma unroll
      for (int q = 0; q < 4; ++q) w[q] = t[q];
    } else if constexpr (VEC == 4) {
      w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
    } else {
      w[0] = p[0];
    }
  };
  auto add = [&](const uint32_t (&w)[VEC >= 4 ? VEC / 4 : 1]) {
    if constexpr (VEC >= 4) {
#pragma unroll
      for (int q = 0; q < VEC / 4; ++q) {
        float a, b, c, d;
        cvt_f32x4<FMT>(w[q], a, b, c, d);
        acc[4 * q] += a; acc[4 * q + 1] += b; acc[4 * q + 2] += c; acc[4 * q + 3] += d;
      }
    } else {
      acc[0] += cvt_f32x1<FMT>(w[0]);
    }
  };
  if (inside) {
    constexpr int UNROLL = 4;
    const uint8_t* p = x + (o * R + r0 + wave) * inner + c0;
    const int64_t step = (int64_t)WAVES * inner;
    int64_t r = r0 + wave;
    for (; r + (UNROLL - 1) * WAVES < r1; r += UNROLL * WAVES) {
      uint32_t w[UNROLL][VEC >= 4 ? VEC / 4 : 1];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) load(p + u * step, w[u]);
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) add(w[u]);
      p += UNROLL * step;
    }
    for (; r < r1; r += WAVES, p += step) {
      uint32_t w[VEC >= 4 ? VEC / 4 : 1];
      load(p, w);
      add(w);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[wave - 1][lane][e] = acc[e];
  }
  __syncthreads();
  if (wave == 0 && inside) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float v = acc[e];
#pragma unroll
      for (int w = 0; w < WAVES - 1; ++w) v += part[w][lane][e];
      if (splits == 1) store_sum(out, out_dtype, o * inner + c0 + e, v);
      else partial[((int64_t)s * outer + o) * inner + c0 + e] = v;
    }
  }
}

// inner == 1: a workgroup sums one slice of one row; VEC 16 needs rows that start 16-byte aligned.
template <int FMT, int VEC>
__global__ __launch_bounds__(kRedThreads) void sum_rows_kernel(const uint8_t* __restrict__ x, int64_t R, int64_t per,
                                                               int splits, void* __restrict__ out, int out_dtype,
                                                               float* __restrict__ partial) {
  __shared__ float wave_part[kRedThreads / 64];
  const int64_t o = blockIdx.x;
  const int s = blockIdx.y;
  const int64_t r0 = s * per;
  const int64_t r1 = (r0 + per) < R ? (r0 + per) : R;
  const uint8_t* row = x + o * R;
  float acc = 0.0f;
  if constexpr (VEC == 16) {
    constexpr int U = 4;
    constexpr int64_t BLOCK = (int64_t)kRedThreads * U * 16;
    for (int64_t b = r0; b < r1; b += BLOCK) {
      const int64_t left = r1 - b;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint8_t*>(row) + b, 0, (int)(left < BLOCK ? left : BLOCK), kRsrcFlags);
      u32x4 t[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        t[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, ((int)threadIdx.x + u * kRedThreads) * 16, 0, 2));
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float a, b2, c, d;
          cvt_f32x4<FMT>(t[u][q], a, b2, c, d);  // bytes past the end arrive as 0x00 = +0.0
          acc += (a + b2) + (c + d);
        }
    }
  } else {
    for (int64_t r = r0 + threadIdx.x; r < r1; r += kRedThreads) acc += cvt_f32x1<FMT>(row[r]);
  }
  acc = wave_sum_f32(acc);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float v = wave_part[0];
#pragma unroll
    for (int w = 1; w < kRedThreads / 64; ++w) v += wave_part[w];
    if (splits == 1) store_sum(out, out_dtype, o, v);
    else partial[(int64_t)s * gridDim.x + o] = v;
  }
}

// Adds the partial sums of the slices: 16 outputs per workgroup, 16 threads per output that
// each add every 16th slice (independent loads), then one thread adds the 16 in order.
__global__ __launch_bounds__(kRedThreads) void sum_finish_kernel(const float* __restrict__ partial, int splits, int64_t n,
                                                                 void* __restrict__ out, int out_dtype) {
  __shared__ float part[16][17];
  const int j = threadIdx.x & 15, g = threadIdx.x >> 4;
  const int64_t i = (int64_t)blockIdx.x * 16 + j;
  float v = 0.0f;
  if (i < n) {
    int s = g;
    for (; s + 48 < splits; s += 64) {
      const float a = partial[(int64_t)s * n + i], b = partial[(int64_t)(s + 16) * n + i];
      const float c = partial[(int64_t)(s + 32) * n + i], d = partial[(int64_t)(s + 48) * n + i];
      v += a; v += b; v += c; v += d;
    }
    for (; s < splits; s += 16) v += partial[(int64_t)s * n + i];
  }
  part[g][j] = v;
  __syncthreads();
  if (g == 0 && i < n) {
    float t = part[0][j];
#pragma unroll
    for (int k = 1; k < 16; ++k) t += part[k][j];
    store_sum(out, out_dtype, i, t);
  }
}

struct SumPlan {
  int vec;       // inner positions per thread (columns) or bytes per load (rows)
  int splits;
  int64_t per;
};

constexpr int64_t kSumWantBlocks = 512;  // two workgroups per compute unit (measured: 256 -> 24 us, 512 -> 18, 1024 -> 21 for [8192, 8192] over dim 0)

// Slices of at least 64 rows (columns) or 16 KiB (rows).
inline SumPlan plan_sum_with(int64_t outer, int64_t R, int64_t inner, int vec) {
  const int64_t blocks = inner > 1 ? outer * ((inner / vec + 63) / 64) : outer;
  const int64_t min_per = inner > 1 ? 64 : 16384;
  int64_t splits = blocks >= kSumWantBlocks ? 1 : (kSumWantBlocks + blocks - 1) / blocks;
  const int64_t max_splits = (R + min_per - 1) / min_per;
  if (splits > max_splits) splits = max_splits;
  if (splits > 1024) splits = 1024;
  if (splits < 1) splits = 1;
  int64_t per = (R + splits - 1) / splits;
  if (inner == 1) per = (per + 15) / 16 * 16;  // slices of a row start 16-byte aligned when the row does
  splits = per > 0 ? (R + per - 1) / per : 1;
  return {vec, (int)(splits < 1 ? 1 : splits), per};
}

// Columns: the widest vector the alignment allows that still gives enough workgroups
// (a thread that owns 16 columns leaves few threads per row of the tensor).
inline SumPlan plan_sum(int64_t outer, int64_t R, int64_t inner, bool aligned16, bool aligned4) {
  if (inner == 1) return plan_sum_with(outer, R, inner, (aligned16 && R % 16 == 0) ? 16 : 1);
  SumPlan best{0, 1, 0};
  int64_t best_blocks = -1;
  for (int vec : {16, 4, 1}) {
    if (inner % vec != 0 || (vec == 16 && !aligned16) || (vec == 4 && !aligned4)) continue;
    const SumPlan p = plan_sum_with(outer, R, inner, vec);
    const int64_t blocks = outer * ((inner / vec + 63) / 64) * p.splits;
    if (blocks >= kSumWantBlocks) return p;
    if (blocks > best_blocks) {
      best = p;
      best_blocks = blocks;
    }
  }
  return best;
}

template <int FMT>
int sum_fp8_launch(const uint8_t* x, int64_t outer, int64_t R, int64_t inner, void* out, int out_dtype, float* ws,
                   size_t ws_bytes, hipStream_t st) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(x);
  const SumPlan p = plan_sum(outer, R, inner, a % 16 == 0, a % 4 == 0);
  const int64_t n_out = outer * inner;
  if (p.splits > 1 && (ws == nullptr || ws_bytes < (size_t)p.splits * n_out * sizeof(float))) return MI355Q_ERR_INVALID_ARGUMENT;
  if (outer > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
  if (inner > 1) {
    const int64_t bx = (inner / p.vec + 63) / 64;
    if (bx * outer > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(bx * outer), (unsigned)p.splits);
    const int cb = (int)bx;
    if (p.vec == 16) sum_columns_kernel<FMT, 16><<<grid, kRedThreads, 0, st>>>(x, outer, R, inner, p.per, p.splits, cb, out, out_dtype, ws);
    else if (p.vec == 4) sum_columns_kernel<FMT, 4><<<grid, kRedThreads, 0, st>>>(x, outer, R, inner, p.per, p.splits, cb, out, out_dtype, ws);
    else sum_columns_kernel<FMT, 1><<<grid, kRedThreads, 0, st>>>(x, outer, R, inner, p.per, p.splits, cb, out, out_dtype, ws);
  } else {
    dim3 grid((unsigned)outer, (unsigned)p.splits);
    if (p.vec == 16) sum_rows_kernel<FMT, 16><<<grid, kRedThreads, 0, st>>>(x, R, p.per, p.splits, out, out_dtype, ws);
    else sum_rows_kernel<FMT, 1><<<grid, kRedThreads, 0, st>>>(x, R, p.per, p.splits, out, out_dtype, ws);
  }
  if (p.splits > 1) {
    const int64_t blocks = (n_out + 15) / 16;
    if (blocks > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    sum_finish_kernel<<<(unsigned)blocks, kRedThreads, 0, st>>>(ws, p.splits, n_out, out, out_dtype);
  }
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

// ---------------------------------------------------------------- softmax_fp8
//
// Rows of `cols` elements, softmax over the row:
//   v = x * inv_attn_heads * input_scale + fused_add          (each factor optional)
//   p = bf16( exp(v - max v) / sum exp(v - max v) )
//   y = OUT_FP8 ? e4m3fn( p * output_scale ) : p
// all in fp32 up to the rounding to bf16.

struct SoftmaxArgs {
  const uint8_t* x;
  uint8_t* y;
  const uint16_t* add;       // bf16 or nullptr
  const float* in_scale;     // device scalars, or nullptr: then the host values below
  const float* out_scale;
  const float* inv_heads;
  float in_scale_host, out_scale_host, inv_heads_host;
  int64_t rows, cols;
  // a row index is decomposed over row_size[0 .. dims) (innermost first) to find the
  // fused_add row: its offset is the sum of digit * add_stride (0 where it is broadcast)
  int dims;
  int64_t row_size[6];
  int64_t add_stride[6];
};

__device__ __forceinline__ int64_t add_row_offset(const SoftmaxArgs& a, int64_t row) {
  int64_t off = 0;
  for (int d = 0; d < a.dims; ++d) {
    const int64_t q = row / a.row_size[d];
    off += (row - q * a.row_size[d]) * a.add_stride[d];
    row = q;
  }
  return off;
}

// WPR waves share a row (1 or 4); a lane holds VPT vectors of 8 of each of its RPW rows (RPW > 1
// only with WPR == 1: a wave then owns RPW consecutive short rows, so that a lane still has four
// loads in flight).  A workgroup covers 4 / WPR * RPW rows.
template <bool IN_FP8, bool OUT_FP8, int WPR, int VPT, int RPW>
__global__ __launch_bounds__(kRedThreads) void softmax_rows_kernel(SoftmaxArgs a) {
  static_assert(WPR == 1 || RPW == 1, "several rows per wave only when a wave owns whole rows");
  constexpr int LANES = 64 * WPR;
  constexpr int IN_ELEM = IN_FP8 ? 1 : 2, OUT_ELEM = OUT_FP8 ? 1 : 2;
  __shared__ float xchg[2][kRedThreads / 64];
  const int wave = threadIdx.x >> 6;
  const int lane = WPR == 1 ? (threadIdx.x & 63) : threadIdx.x;
  const int64_t row0 = WPR == 1 ? ((int64_t)blockIdx.x * 4 + wave) * RPW : (int64_t)blockIdx.x;
  const int cols = (int)a.cols;
  const bool has_add = a.add != nullptr;
  const float s_in = a.in_scale ? a.in_scale[0] : a.in_scale_host;
  const float s_out = a.out_scale ? a.out_scale[0] : a.out_scale_host;
  const float s_inv = a.inv_heads ? a.inv_heads[0] : a.inv_heads_host;

  u32x4 raw[RPW][VPT];   // IN_FP8 uses the first two words
  u32x4 addv[RPW][VPT];
#pragma unroll
  for (int rr = 0; rr < RPW; ++rr) {
    const bool live = row0 + rr < a.rows;                 // uniform per wave
    const int64_t row = live ? row0 + rr : 0;
    const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(a.x) + row * cols * IN_ELEM, 0, live ? cols * IN_ELEM : 0, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t radd = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(a.add) + (has_add ? add_row_offset(a, row) : 0), 0, (live && has_add) ? cols * 2 : 0, kRsrcFlags);
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      const int v = lane + u * LANES;
      if constexpr (IN_FP8) {
        const u32x2 t = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rin, v * 8, 0, 2));
        raw[rr][u] = u32x4{t[0], t[1], 0u, 0u};
      } else {
        raw[rr][u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rin, v * 16, 0, 2));
      }
      addv[rr][u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(radd, v * 16, 0, 0));  // zeros without fused_add
    }
  }
#pragma unroll
  for (int rr = 0; rr < RPW; ++rr) {
    const bool live = row0 + rr < a.rows;
    const int64_t row = live ? row0 + rr : 0;
    const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(
        a.y + row * cols * OUT_ELEM, 0, live ? cols * OUT_ELEM : 0, kRsrcFlags);
    float val[VPT][8];
    float m = -__builtin_inff();
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      if constexpr (IN_FP8) {
        cvt_f32x4<MI355Q_E4M3FN>(raw[rr][u][0], val[u][0], val[u][1], val[u][2], val[u][3]);
        cvt_f32x4<MI355Q_E4M3FN>(raw[rr][u][1], val[u][4], val[u][5], val[u][6], val[u][7]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          val[u][2 * i] = __uint_as_float(raw[rr][u][i] << 16);
          val[u][2 * i + 1] = __uint_as_float(raw[rr][u][i] & 0xffff0000u);
        }
      }
      const bool inside = (lane + u * LANES) * 8 < cols;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float ad = __uint_as_float((i & 1) ? (addv[rr][u][i >> 1] & 0xffff0000u) : (addv[rr][u][i >> 1] << 16));
        const float t = (val[u][i] * s_inv) * s_in + ad;
        val[u][i] = inside ? t : -__builtin_inff();
        m = __builtin_fmaxf(m, val[u][i]);
      }
    }
    m = wave_max_f32(m);
    if constexpr (WPR > 1) {
      if ((threadIdx.x & 63) == 0) xchg[0][wave] = m;
      __syncthreads();
      m = __builtin_fmaxf(__builtin_fmaxf(xchg[0][0], xchg[0][1]), __builtin_fmaxf(xchg[0][2], xchg[0][3]));
    }
    // a row of -inf only (or NaN) gives NaN, as torch.softmax does
    float sum = 0.0f;
#pragma unroll
    for (int u = 0; u < VPT; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        val[u][i] = __expf(val[u][i] - m);
        sum += val[u][i];
      }
    sum = wave_sum_f32(sum);
    if constexpr (WPR > 1) {
      if ((threadIdx.x & 63) == 0) xchg[1][wave] = sum;
      __syncthreads();
      sum = (xchg[1][0] + xchg[1][1]) + (xchg[1][2] + xchg[1][3]);
    }
    const float inv = 1.0f / sum;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      const int v = lane + u * LANES;
      float p[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = val[u][i] * inv;
      if constexpr (OUT_FP8) {
#pragma unroll
        for (int i = 0; i < 8; ++i) p[i] = round_to_bf16(p[i]) * s_out;
        const u32x2 o = {cvt_fp8x4<MI355Q_E4M3FN>(p[0], p[1], p[2], p[3]), cvt_fp8x4<MI355Q_E4M3FN>(p[4], p[5], p[6], p[7])};
        __builtin_amdgcn_raw_buffer_store_b64(o, rout, v * 8, 0, 2);
      } else {
        const u32x4 o = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]), pack_bf16x2(p[6], p[7])};
        __builtin_amdgcn_raw_buffer_store_b128(o, rout, v * 16, 0, 2);
      }
    }
  }
}

// Any row length and alignment: one workgroup per row, three passes over the row.
template <bool IN_FP8, bool OUT_FP8>
__global__ __launch_bounds__(kRedThreads) void softmax_rows_generic_kernel(SoftmaxArgs a) {
  __shared__ float xchg[kRedThreads / 64];
  __shared__ float bcast;
  const int64_t row = blockIdx.x;
  const int64_t cols = a.cols;
  const uint8_t* xr = a.x + row * cols * (IN_FP8 ? 1 : 2);
  uint8_t* yr = a.y + row * cols * (OUT_FP8 ? 1 : 2);
  const uint16_t* ar = a.add ? a.add + add_row_offset(a, row) : nullptr;
  const float s_in = a.in_scale ? a.in_scale[0] : a.in_scale_host;
  const float s_out = a.out_scale ? a.out_scale[0] : a.out_scale_host;
  const float s_inv = a.inv_heads ? a.inv_heads[0] : a.inv_heads_host;
  auto value = [&](int64_t c) {
    const float x = IN_FP8 ? cvt_f32x1<MI355Q_E4M3FN>(xr[c]) : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(xr)[c]);
    return (x * s_inv) * s_in + (ar ? bf16_bits_to_f32(ar[c]) : 0.0f);
  };
  auto block_reduce = [&](float v, bool is_max) {
    v = is_max ? wave_max_f32(v) : wave_sum_f32(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) xchg[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
      float r = xchg[0];
      for (int w = 1; w < kRedThreads / 64; ++w) r = is_max ? __builtin_fmaxf(r, xchg[w]) : r + xchg[w];
      bcast = r;
    }
    __syncthreads();
    return bcast;
  };
  float m = -__builtin_inff();
  for (int64_t c = threadIdx.x; c < cols; c += kRedThreads) m = __builtin_fmaxf(m, value(c));
  m = block_reduce(m, true);
  float sum = 0.0f;
  for (int64_t c = threadIdx.x; c < cols; c += kRedThreads) sum += __expf(value(c) - m);
  sum = block_reduce(sum, false);
  const float inv = 1.0f / sum;
  for (int64_t c = threadIdx.x; c < cols; c += kRedThreads) {
    const float p = __expf(value(c) - m) * inv;
    if constexpr (OUT_FP8) {
      const float q = round_to_bf16(p) * s_out;
      yr[c] = (uint8_t)(cvt_fp8x4<MI355Q_E4M3FN>(q, q, q, q) & 0xffu);
    } else {
      reinterpret_cast<uint16_t*>(yr)[c] = (uint16_t)(pack_bf16x2(p, p) & 0xffffu);
    }
  }
}

template <bool IN_FP8, bool OUT_FP8>
int softmax_launch(const SoftmaxArgs& a, hipStream_t st) {
  const int64_t nv = a.cols / 8;
  const uintptr_t al = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.y) | reinterpret_cast<uintptr_t>(a.add);
  bool add_ok = true;  // fused_add rows must start 16-byte aligned too
  for (int d = 0; d < a.dims; ++d) add_ok = add_ok && (a.add == nullptr || a.add_stride[d] % 8 == 0);
  const bool vec = a.cols % 8 == 0 && al % 16 == 0 && add_ok && nv <= 256 * 8 && a.cols * 2 < (1LL << 31);
  if (!vec) {
    if (a.rows > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    softmax_rows_generic_kernel<IN_FP8, OUT_FP8><<<(unsigned)a.rows, kRedThreads, 0, st>>>(a);
    return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
  }
  const bool one_wave = nv <= 64 * 8;
  const int64_t lanes = one_wave ? 64 : 256;
  const int64_t need = (nv + lanes - 1) / lanes;
  // short rows: a wave takes 4 (one vector per lane and row) or 2 (two vectors) rows
  const int rpw = !one_wave ? 1 : need <= 1 ? 4 : need <= 2 ? 2 : 1;
  const int64_t rows_per_block = one_wave ? 4 * rpw : 1;
  const int64_t blocks = (a.rows + rows_per_block - 1) / rows_per_block;
  if (blocks > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
  const unsigned g = (unsigned)blocks;
#define MI355Q_SOFTMAX(WPR, VPT, RPW) softmax_rows_kernel<IN_FP8, OUT_FP8, WPR, VPT, RPW><<<g, kRedThreads, 0, st>>>(a)
  if (one_wave) {
    if (need <= 1) MI355Q_SOFTMAX(1, 1, 4);
    else if (need <= 2) MI355Q_SOFTMAX(1, 2, 2);
    else if (need <= 4) MI355Q_SOFTMAX(1, 4, 1);
    else MI355Q_SOFTMAX(1, 8, 1);
  } else {
    if (need <= 4) MI355Q_SOFTMAX(4, 4, 1);
    else MI355Q_SOFTMAX(4, 8, 1);
  }
#undef MI355Q_SOFTMAX
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

// ------------------------------------------- sum_fp8 without a caller's workspace
//
// The partial sums of a split reduction live in this file-scope device array instead of
// a workspace the caller allocates.  Every GPU the library runs on holds its own copy
// until the process ends.  In host code the array's name is only a handle: the device
// address is asked for once per device (hipGetSymbolAddress) and that pointer is what the
// kernels get, exactly as they get a caller's workspace.
static __device__ __align__(256) unsigned char sum_scratch[MI355Q_SUM_FP8_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static std::mutex sum_scratch_mutex;
static void* sum_scratch_ptr[kMaxDevices];  // device address of sum_scratch, per device

// Address of the current device's copy of sum_scratch (looked up on the first call per device).
// The lookup is a runtime call that a stream under capture must not see: a first call on a device
// whose `stream` is being captured is refused (make one call outside the capture first).
inline int sum_scratch_of_current_device(float** out, hipStream_t stream) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MI355Q_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(sum_scratch_mutex);
  if (sum_scratch_ptr[dev] == nullptr) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
      (void)hipGetLastError();
      return MI355Q_ERR_LAUNCH;
    }
    if (cap != hipStreamCaptureStatusNone) return MI355Q_ERR_UNSUPPORTED;
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(sum_scratch)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return MI355Q_ERR_LAUNCH;
    }
    sum_scratch_ptr[dev] = p;
  }
  *out = static_cast<float*>(sum_scratch_ptr[dev]);
  return MI355Q_OK;
}

}  // namespace mi355q

using namespace mi355q;

extern "C" {

size_t mi355q_sum_fp8_workspace_bytes(int64_t outer, int64_t reduce, int64_t inner) {
  if (outer <= 0 || reduce <= 0 || inner <= 0) return 0;
  // the launch picks its vector width from the pointer's alignment: the largest need of any choice
  int splits = 1;
  for (int al = 0; al < 3; ++al) {
    const SumPlan p = plan_sum(outer, reduce, inner, al == 0, al <= 1);
    if (p.splits > splits) splits = p.splits;
  }
  return splits > 1 ? (size_t)splits * (size_t)(outer * inner) * sizeof(float) : 0;
}

int mi355q_sum_fp8(const void* x, int fp8_fmt, int64_t outer, int64_t reduce, int64_t inner, void* out,
                   int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype < MI355Q_F32 || out_dtype > MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (outer < 0 || reduce < 0 || inner < 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (outer == 0 || inner == 0) return MI355Q_OK;
  if (out == nullptr || (reduce > 0 && x == nullptr)) return MI355Q_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  float* ws = static_cast<float*>(workspace);
  // an empty reduction gives zeros: the kernels' loops do not run and store 0
  if (fp8_fmt == MI355Q_E4M3FN) return sum_fp8_launch<MI355Q_E4M3FN>(xb, outer, reduce, inner, out, out_dtype, ws, workspace_bytes, st);
  return sum_fp8_launch<MI355Q_E5M2>(xb, outer, reduce, inner, out, out_dtype, ws, workspace_bytes, st);
}

int mi355q_sum_fp8_static(const void* x, int fp8_fmt, int64_t outer, int64_t reduce, int64_t inner, void* out,
                          int out_dtype, void* stream) {
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype < MI355Q_F32 || out_dtype > MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (outer < 0 || reduce < 0 || inner < 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (outer == 0 || inner == 0) return MI355Q_OK;
  if (out == nullptr || (reduce > 0 && x == nullptr)) return MI355Q_ERR_INVALID_ARGUMENT;
  if (mi355q_sum_fp8_workspace_bytes(outer, reduce, inner) > (size_t)MI355Q_SUM_FP8_STATIC_SCRATCH_BYTES)
    return MI355Q_ERR_TOO_LARGE;
  float* ws = nullptr;
  const int got = sum_scratch_of_current_device(&ws, static_cast<hipStream_t>(stream));
  if (got != MI355Q_OK) return got;
  // Nothing has to be cleared between calls: every slice writes its partial sum of every
  // output before sum_finish_kernel, ordered behind it on the stream, reads them.
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  if (fp8_fmt == MI355Q_E4M3FN)
    return sum_fp8_launch<MI355Q_E4M3FN>(xb, outer, reduce, inner, out, out_dtype, ws, MI355Q_SUM_FP8_STATIC_SCRATCH_BYTES, st);
  return sum_fp8_launch<MI355Q_E5M2>(xb, outer, reduce, inner, out, out_dtype, ws, MI355Q_SUM_FP8_STATIC_SCRATCH_BYTES, st);
}

int mi355q_softmax_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* input_scale_dev,
                       float input_scale_host, const float* output_scale_dev, float output_scale_host,
                       const float* inv_attn_heads_dev, float inv_attn_heads_host, const void* fused_add,
                       int row_dims, const int64_t* row_sizes, const int64_t* fused_add_row_strides, void* y,
                       int y_dtype, void* stream) {
  if (x_dtype != MI355Q_BF16 && x_dtype != MI355Q_E4M3FN) return MI355Q_ERR_INVALID_ARGUMENT;
  if (y_dtype != MI355Q_BF16 && y_dtype != MI355Q_E4M3FN) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows < 0 || cols < 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return MI355Q_OK;
  if (x == nullptr || y == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  SoftmaxArgs a;
  a.x = static_cast<const uint8_t*>(x);
  a.y = static_cast<uint8_t*>(y);
  a.add = static_cast<const uint16_t*>(fused_add);
  a.in_scale = input_scale_dev; a.out_scale = output_scale_dev; a.inv_heads = inv_attn_heads_dev;
  a.in_scale_host = input_scale_host; a.out_scale_host = output_scale_host; a.inv_heads_host = inv_attn_heads_host;
  a.rows = rows; a.cols = cols;
  a.dims = 0;
  for (int d = 0; d < 6; ++d) { a.row_size[d] = 1; a.add_stride[d] = 0; }
  if (fused_add != nullptr) {
    if (row_dims < 0 || row_dims > 6 || (row_dims > 0 && (row_sizes == nullptr || fused_add_row_strides == nullptr)))
      return MI355Q_ERR_INVALID_ARGUMENT;
    int64_t n = 1;
    for (int d = 0; d < row_dims; ++d) {
      if (row_sizes[d] <= 0 || fused_add_row_strides[d] < 0) return MI355Q_ERR_INVALID_ARGUMENT;
      a.row_size[d] = row_sizes[d];
      a.add_stride[d] = fused_add_row_strides[d];
      n *= row_sizes[d];
    }
    if (n != rows) return MI355Q_ERR_INVALID_ARGUMENT;
    a.dims = row_dims;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool in8 = x_dtype == MI355Q_E4M3FN, out8 = y_dtype == MI355Q_E4M3FN;
  if (in8 && out8) return softmax_launch<true, true>(a, st);
  if (in8) return softmax_launch<true, false>(a, st);
  if (out8) return softmax_launch<false, true>(a, st);
  return softmax_launch<false, false>(a, st);
}

}  // extern "C"
