// cast_to_fp8 / cast_from_fp8 / amax kernels for gfx950 and their C entry points.
//
// All three are HBM-bound streaming kernels: every lane moves 16-byte vectors,
// a wave's accesses are contiguous, and each thread keeps several independent
// loads in flight.  Rounding and saturation use the CDNA4 conversion
// instructions (v_cvt_pk_{fp8,bf8}_f32, v_cvt_pk_f32_{fp8,bf8},
// v_cvt_pk_bf16_f32); see device_common.h.
#include <type_traits>

#include "device_common.h"

namespace mi355q {

enum ScaleKind { SK_SCALAR = 0, SK_ROW = 1, SK_COL = 2, SK_FULL = 3 };

constexpr int kThreads = 256;

__global__ void fill_u32_kernel(uint32_t* p, uint32_t v) { *p = v; }

// Kernels that reduce an amax run as at most kAmaxBlocks fat workgroups that
// stride over the data: the number of same-address atomics, not the streaming,
// is what bounds them otherwise (2048 blocks: ~30 us; 256 blocks: ~7 us for
// 32 MiB).
constexpr int kAmaxThreads = 1024;
constexpr int kAmaxBlocks = 256;

// Block-level max of abs-value bit patterns, then one atomicMax per block.
// Bit patterns of non-negative floats order like the floats, and a NaN
// pattern is larger than Inf, so NaN wins and the result reads back as NaN.
__device__ __forceinline__ void block_amax_commit(uint32_t m, uint32_t* amax) {
  __shared__ uint32_t wave_part[16];
  m = wave_max_u32(m);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) wave_part[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t r = wave_part[0];
    const int nwaves = (int)(blockDim.x >> 6);
    for (int w = 1; w < nwaves; ++w) r = r > wave_part[w] ? r : wave_part[w];
    // Atomics on one address serialise in L2.  The running maximum only grows,
    // so a block whose maximum does not beat the value already there has
    // nothing to add: read it first (device-scope load, not from L1) and skip
    // the atomic.  After the first few blocks almost every block skips.
    if (r != 0 && r > __hip_atomic_load(amax, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(amax, r);
  }
}

// ---------------------------------------------------------------- cast_to_fp8
//
// The input is viewed as [rows, vec_per_row] vectors of 8 elements.  Flat
// modes use rows == 1.  A block owns blockDim*U consecutive vectors of one
// row; U loads per thread are issued before any is consumed.
//   SK_SCALAR  one scale for everything (host value or *scale)
//   SK_ROW     scale[row % mid]
//   SK_COL     scale[column]
//   SK_FULL    scale[element]
//
// The body has no divergent branch: loads and stores go through buffer
// descriptors that cover exactly the block's vectors, so a lane past the end
// of the row loads zeros and its store is dropped.  (With a branch around each
// load the compiler cannot tell that the previous iteration's load into the
// same registers was consumed, and makes every load wait for all earlier ones.)
template <bool BF16_IN, int FMT, int SK, bool AMAX, int U>
__global__ __launch_bounds__(AMAX ? kAmaxThreads : kThreads) void cast_to_fp8_vec8(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ y, const float* __restrict__ scale,
    float scale_host, int scale_is_dev, int64_t vec_per_row, int64_t blocks_per_row,
    int64_t total_blocks, int64_t mid, uint32_t* __restrict__ amax) {
  constexpr int THREADS = AMAX ? kAmaxThreads : kThreads;
  constexpr int IN_BYTES = BF16_IN ? 16 : 32;
  constexpr int kNt = 2;  // non-temporal
  uint32_t am = 0;
  // a logical block is THREADS * U consecutive vectors of one row; without amax
  // the grid holds one workgroup per logical block and this loop runs once
  for (int64_t lb = blockIdx.x; lb < total_blocks; lb += gridDim.x) {
    const int64_t row = lb / blocks_per_row;
    const int64_t vec0 = (lb - row * blocks_per_row) * (int64_t)(THREADS * U);  // first vector, within the row
    const int64_t left = vec_per_row - vec0;
    const int nvec = (int)(left < THREADS * U ? left : THREADS * U);
    const int64_t first = row * vec_per_row + vec0;                             // first vector, within the tensor
    const __amdgpu_buffer_rsrc_t rin =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(x) + first * IN_BYTES, 0, nvec * IN_BYTES, 0x00020000);
    const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(y + first * 8, 0, nvec * 8, 0x00020000);

    float s = 1.0f;
    if constexpr (SK == SK_SCALAR) s = scale_is_dev ? scale[0] : scale_host;
    if constexpr (SK == SK_ROW) s = scale[row % mid];
    if constexpr (BF16_IN) s = round_to_bf16(s);

    u32x4 in[U][BF16_IN ? 1 : 2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int off = ((int)threadIdx.x + u * THREADS) * IN_BYTES;
      in[u][0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rin, off, 0, kNt));
      if constexpr (!BF16_IN) in[u][1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rin, off + 16, 0, kNt));
    }
    // per-column / per-element scales: 8 floats per vector, out-of-range lanes read zeros
    u32x4 sc[(SK == SK_COL || SK == SK_FULL) ? U : 1][2];
    if constexpr (SK == SK_COL || SK == SK_FULL) {
      const float* sbase = scale + (SK == SK_COL ? vec0 : first) * 8;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sbase), 0, nvec * 32, 0x00020000);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int off = ((int)threadIdx.x + u * THREADS) * 32;
        sc[u][0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0));
        sc[u][1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, off + 16, 0, 0));
      }
    }

#pragma unroll
    for (int u = 0; u < U; ++u) {
      float v[8];
      if constexpr (BF16_IN) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t w = in[u][0][i];
          v[2 * i] = __uint_as_float(w << 16);
          v[2 * i + 1] = __uint_as_float(w & 0xffff0000u);
          if constexpr (AMAX) {
            // packed 16-bit max over the two abs bit patterns of this dword
            const u16x2 a = __builtin_bit_cast(u16x2, w & 0x7fff7fffu);
            const u16x2 m = __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am));
            am = __builtin_bit_cast(uint32_t, m);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t w = in[u][i >> 2][i & 3];
          v[i] = __uint_as_float(w);
          if constexpr (AMAX) {
            const uint32_t a = w & 0x7fffffffu;
            am = am > a ? am : a;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float sv = s;
        if constexpr (SK == SK_COL || SK == SK_FULL) {
          sv = __uint_as_float(sc[u][i >> 2][i & 3]);
          if constexpr (BF16_IN) sv = round_to_bf16(sv);
        }
        float p = v[i] * sv;
        if constexpr (BF16_IN) p = round_to_bf16(p);
        v[i] = p;
      }
      u32x2 out;
      out.x = cvt_fp8x4<FMT>(v[0], v[1], v[2], v[3]);
      out.y = cvt_fp8x4<FMT>(v[4], v[5], v[6], v[7]);
      __builtin_amdgcn_raw_buffer_store_b64(out, rout, ((int)threadIdx.x + u * THREADS) * 8, 0, kNt);
    }
  }

  if constexpr (AMAX) {
    if constexpr (BF16_IN) {
      const uint32_t lo = am & 0xffffu, hi = am >> 16;
      am = (lo > hi ? lo : hi) << 16;
    }
    block_amax_commit(am, amax);
  }
}

// One element per thread, any alignment, any broadcast: tails and odd shapes.
template <bool BF16_IN, int FMT>
__global__ __launch_bounds__(kThreads) void cast_to_fp8_generic(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ y, const float* __restrict__ scale,
    float scale_host, int mode, int64_t start, int64_t n, int64_t mid, int64_t inner,
    uint32_t* __restrict__ amax) {
  const int64_t i = start + (int64_t)blockIdx.x * kThreads + threadIdx.x;
  uint32_t am = 0;
  if (i < n) {
    float s = 1.0f;
    if (mode == MI355Q_SCALE_HOST) s = scale_host;
    else if (mode == MI355Q_SCALE_DEV) s = scale[0];
    else if (mode == MI355Q_SCALE_MID) s = scale[(i / inner) % mid];
    else if (mode == MI355Q_SCALE_FULL) s = scale[i];
    float v, p;
    if constexpr (BF16_IN) {
      const uint32_t h = reinterpret_cast<const uint16_t*>(x)[i];
      v = bf16_bits_to_f32(h);
      p = round_to_bf16(v * round_to_bf16(s));
    } else {
      v = reinterpret_cast<const float*>(x)[i];
      p = v * s;
    }
    am = __float_as_uint(v) & 0x7fffffffu;
    y[i] = (uint8_t)(cvt_fp8x4<FMT>(p, p, p, p) & 0xffu);
  }
  if (amax != nullptr) block_amax_commit(am, amax);
}

// Stochastic rounding with flush to zero (round mode CAST_ROUND_SFTZ of GetCastParams,
// hpu_ops/backend/fp8_ops.cpp:105-119): a scaled value below the format's smallest normal number
// becomes a zero of its sign instead of being rounded stochastically among the subnormals.
template <int FMT>
__device__ __forceinline__ float flush_below_min_normal(float p) {
  constexpr float kMinNormal = FMT == MI355Q_E5M2 ? 6.103515625e-05f : 0.015625f;  // 2^-14, 2^-6
  return __builtin_fabsf(p) < kMinNormal ? __builtin_copysignf(0.0f, p) : p;
}

// Stochastic-rounding cast: four consecutive elements per thread, any scale
// broadcast, optional amax.  Not a bandwidth-tuned path (training-side casts of
// optimizer state use it, the inference path rounds to nearest).
template <bool BF16_IN, int FMT>
__global__ __launch_bounds__(kThreads) void cast_to_fp8_sr_kernel(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ y, const float* __restrict__ scale,
    float scale_host, int mode, int64_t n, int64_t mid, int64_t inner, uint64_t seed, uint64_t offset,
    int flush_subnormals, uint32_t* __restrict__ amax) {
  const int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x;  // index of this thread's quad
  const int64_t i0 = q * 4;
  uint32_t am = 0;
  if (i0 < n) {
    float p[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t i = i0 + e < n ? i0 + e : n - 1;
      float s = 1.0f;
      if (mode == MI355Q_SCALE_HOST) s = scale_host;
      else if (mode == MI355Q_SCALE_DEV) s = scale[0];
      else if (mode == MI355Q_SCALE_MID) s = scale[(i / inner) % mid];
      else if (mode == MI355Q_SCALE_FULL) s = scale[i];
      float v;
      if constexpr (BF16_IN) {
        v = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(x)[i]);
        p[e] = round_to_bf16(v * round_to_bf16(s));
      } else {
        v = reinterpret_cast<const float*>(x)[i];
        p[e] = v * s;
      }
      const uint32_t a = __float_as_uint(v) & 0x7fffffffu;
      am = am > a ? am : a;
      if (flush_subnormals) p[e] = flush_below_min_normal<FMT>(p[e]);
    }
    const uint64_t ra = counter_random64(seed, offset + 2 * (uint64_t)q);
    const uint64_t rb = counter_random64(seed, offset + 2 * (uint64_t)q + 1);
    const uint32_t o = cvt_fp8x4_sr<FMT>(p[0], p[1], p[2], p[3], (uint32_t)ra, (uint32_t)(ra >> 32),
                                         (uint32_t)rb, (uint32_t)(rb >> 32));
    if (i0 + 3 < n && (reinterpret_cast<uintptr_t>(y) & 3u) == 0) {
      reinterpret_cast<uint32_t*>(y)[q] = o;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i0 + e < n) y[i0 + e] = (uint8_t)(o >> (8 * e));
    }
  }
  if (amax != nullptr) block_amax_commit(am, amax);
}

// ------------------------------------------------------------ cast_to_fp8_hybrid
//
// One read of x, two fp8 tensors out (e5m2 with scale_152, e4m3fn with scale_143)
// and optionally amax.  Stochastic rounding applies to the e5m2 output only; the
// e4m3fn output always rounds to nearest even.  Scales are per tensor.
// [first, first + count) elements; VEC = 8 elements per thread per step when the
// pointers allow 16-byte loads, else 1.
template <bool BF16_IN, int VEC>
__global__ __launch_bounds__(kAmaxThreads) void cast_to_fp8_hybrid_kernel(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ y152, uint8_t* __restrict__ y143,
    const float* __restrict__ scale152, const float* __restrict__ scale143, int64_t first, int64_t count,
    int stochastic, uint64_t seed, uint64_t offset, uint32_t* __restrict__ amax) {
  float s5 = scale152 ? scale152[0] : 1.0f, s4 = scale143 ? scale143[0] : 1.0f;
  if constexpr (BF16_IN) {
    s5 = round_to_bf16(s5);
    s4 = round_to_bf16(s4);
  }
  uint32_t am = 0;
  const int64_t steps = (count + VEC - 1) / VEC;
  for (int64_t t = (int64_t)blockIdx.x * kAmaxThreads + threadIdx.x; t < steps; t += (int64_t)gridDim.x * kAmaxThreads) {
    const int64_t i0 = first + t * VEC;
    float v[VEC];
    if constexpr (VEC == 8) {
      if constexpr (BF16_IN) {
        const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + i0 * 2));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[2 * i] = __uint_as_float(w[i] << 16);
          v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
      } else {
        const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + i0 * 4));
        const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + i0 * 4) + 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[i] = a[i];
          v[4 + i] = b[i];
        }
      }
    } else {
      v[0] = BF16_IN ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(x)[i0]) : reinterpret_cast<const float*>(x)[i0];
    }
    float p5[VEC], p4[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const uint32_t a = __float_as_uint(v[i]) & 0x7fffffffu;
      am = am > a ? am : a;
      p5[i] = BF16_IN ? round_to_bf16(v[i] * s5) : v[i] * s5;
      p4[i] = BF16_IN ? round_to_bf16(v[i] * s4) : v[i] * s4;
      if (stochastic == 2) p5[i] = flush_below_min_normal<MI355Q_E5M2>(p5[i]);
    }
    if constexpr (VEC == 8) {
      u32x2 o5, o4;
      o4.x = cvt_fp8x4<MI355Q_E4M3FN>(p4[0], p4[1], p4[2], p4[3]);
      o4.y = cvt_fp8x4<MI355Q_E4M3FN>(p4[4], p4[5], p4[6], p4[7]);
      if (stochastic) {
        // element i0 + e draws from counter (i0 + e) / 2, as a scalar step does
        const uint64_t c = offset + (uint64_t)(i0 >> 1);
        const uint64_t r0 = counter_random64(seed, c), r1 = counter_random64(seed, c + 1);
        const uint64_t r2 = counter_random64(seed, c + 2), r3 = counter_random64(seed, c + 3);
        o5.x = cvt_fp8x4_sr<MI355Q_E5M2>(p5[0], p5[1], p5[2], p5[3], (uint32_t)r0, (uint32_t)(r0 >> 32), (uint32_t)r1, (uint32_t)(r1 >> 32));
        o5.y = cvt_fp8x4_sr<MI355Q_E5M2>(p5[4], p5[5], p5[6], p5[7], (uint32_t)r2, (uint32_t)(r2 >> 32), (uint32_t)r3, (uint32_t)(r3 >> 32));
      } else {
        o5.x = cvt_fp8x4<MI355Q_E5M2>(p5[0], p5[1], p5[2], p5[3]);
        o5.y = cvt_fp8x4<MI355Q_E5M2>(p5[4], p5[5], p5[6], p5[7]);
      }
      __builtin_nontemporal_store(o5, reinterpret_cast<u32x2*>(y152 + i0));
      __builtin_nontemporal_store(o4, reinterpret_cast<u32x2*>(y143 + i0));
    } else {
      y143[i0] = (uint8_t)(cvt_fp8x4<MI355Q_E4M3FN>(p4[0], p4[0], p4[0], p4[0]) & 0xffu);
      if (stochastic) {
        const uint64_t r = counter_random64(seed, offset + (uint64_t)(i0 >> 1));
        const uint32_t rr = (i0 & 1) ? (uint32_t)(r >> 32) : (uint32_t)r;
        y152[i0] = (uint8_t)(cvt_fp8x4_sr<MI355Q_E5M2>(p5[0], p5[0], p5[0], p5[0], rr, rr, rr, rr) & 0xffu);
      } else {
        y152[i0] = (uint8_t)(cvt_fp8x4<MI355Q_E5M2>(p5[0], p5[0], p5[0], p5[0]) & 0xffu);
      }
    }
  }
  if (amax != nullptr) block_amax_commit(am, amax);
}

// ---------------------------------------------------------------------- amax
template <bool BF16_IN, int U>
__global__ __launch_bounds__(kAmaxThreads) void amax_vec(const uint8_t* __restrict__ x, int64_t nvec,
                                                         uint32_t* __restrict__ amax) {
  // vectors of 16 bytes; the grid strides over the data
  uint32_t am = 0;
  const int64_t stride = (int64_t)gridDim.x * kAmaxThreads;
  for (int64_t v0 = (int64_t)blockIdx.x * kAmaxThreads + threadIdx.x; v0 < nvec; v0 += stride * U) {
  u32x4 in[U];
  bool ok[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t v = v0 + (int64_t)u * stride;
    ok[u] = v < nvec;
    if (ok[u]) in[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x) + v);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (!ok[u]) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (BF16_IN) {
        const u16x2 a = __builtin_bit_cast(u16x2, in[u][i] & 0x7fff7fffu);
        am = __builtin_bit_cast(uint32_t,
                                __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am)));
      } else {
        const uint32_t a = in[u][i] & 0x7fffffffu;
        am = am > a ? am : a;
      }
    }
  }
  }
  if constexpr (BF16_IN) {
    const uint32_t lo = am & 0xffffu, hi = am >> 16;
    am = (lo > hi ? lo : hi) << 16;
  }
  block_amax_commit(am, amax);
}

template <bool BF16_IN>
__global__ __launch_bounds__(kThreads) void amax_generic(const uint8_t* __restrict__ x,
                                                         int64_t start, int64_t n,
                                                         uint32_t* __restrict__ amax) {
  const int64_t i = start + (int64_t)blockIdx.x * kThreads + threadIdx.x;
  uint32_t am = 0;
  if (i < n) {
    if constexpr (BF16_IN) am = ((uint32_t)reinterpret_cast<const uint16_t*>(x)[i] & 0x7fffu) << 16;
    else am = reinterpret_cast<const uint32_t*>(x)[i] & 0x7fffffffu;
  }
  block_amax_commit(am, amax);
}

// One block per row; rows are independent so no atomics and no pre-zeroing.
template <bool BF16_IN>
__global__ __launch_bounds__(kThreads) void rowwise_amax_kernel(const uint8_t* __restrict__ x,
                                                               int64_t cols, int vec_ok,
                                                               float* __restrict__ out) {
  __shared__ uint32_t wave_part[kThreads / 64];
  const int64_t row = blockIdx.x;
  constexpr int ES = BF16_IN ? 2 : 4;
  const uint8_t* xr = x + row * cols * ES;
  uint32_t am = 0;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t nvec = cols * ES / 16;
    for (int64_t v = threadIdx.x; v < nvec; v += kThreads) {
      const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr) + v);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (BF16_IN) {
          const u16x2 a = __builtin_bit_cast(u16x2, w[i] & 0x7fff7fffu);
          am = __builtin_bit_cast(uint32_t,
                                  __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am)));
        } else {
          const uint32_t a = w[i] & 0x7fffffffu;
          am = am > a ? am : a;
        }
      }
    }
    if constexpr (BF16_IN) {
      const uint32_t lo = am & 0xffffu, hi = am >> 16;
      am = (lo > hi ? lo : hi) << 16;
    }
    done = nvec * (16 / ES);
  }
  for (int64_t c = done + threadIdx.x; c < cols; c += kThreads) {
    uint32_t a;
    if constexpr (BF16_IN) a = ((uint32_t)reinterpret_cast<const uint16_t*>(xr)[c] & 0x7fffu) << 16;
    else a = reinterpret_cast<const uint32_t*>(xr)[c] & 0x7fffffffu;
    am = am > a ? am : a;
  }
  am = wave_max_u32(am);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = am;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t r = wave_part[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) r = r > wave_part[w] ? r : wave_part[w];
    out[row] = __uint_as_float(r);
  }
}

// ------------------------------------------------- bf16 rows as two fp8 planes
//
// For the int4-weight GEMM on 16-bit activations (mi355q_w4a16_gemm): a bf16 value has 8 significant
// bits, an e4m3 value 4, so with a power-of-two row scale s (the largest with max |a| s <= 448)
//   hi = e4m3(a s)  (round to nearest even)      lo = e4m3((a s - hi) 16)
// give a s = hi + lo / 16 exactly for every element whose hi is a normal number (the remainder then has
// at most 4 significant bits), and to within 2^-14 (3e-8 of the row's 448) for the small elements whose
// remainder falls below e4m3's subnormal spacing.  The matrix unit multiplies the two planes at the fp8
// rate; 1 / s goes to the GEMM's per-row factor.  One workgroup per row, two passes over it (the second
// out of the cache).  A row of zeros takes s = 1.
__global__ __launch_bounds__(kThreads) void split_rows_kernel(const uint16_t* __restrict__ x, int64_t ldx, int64_t cols,
                                                              uint8_t* __restrict__ hi, uint8_t* __restrict__ lo, int64_t ld,
                                                              float* __restrict__ scale_inv) {
  __shared__ uint32_t wave_part[kThreads / 64];
  const int64_t row = blockIdx.x;
  const uint16_t* xr = x + row * ldx;
  uint32_t am = 0;
  for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
    const uint32_t a = ((uint32_t)xr[c] & 0x7fffu) << 16;
    am = am > a ? am : a;
  }
  am = wave_max_u32(am);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = am;
  __syncthreads();
  uint32_t r = wave_part[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) r = r > wave_part[w] ? r : wave_part[w];
  // amax = m 2^ea with 1 <= m < 2; 448 = 1.75 2^8: s = 2^(8 - ea) when m <= 1.75, else 2^(7 - ea)
  int e = 0;
  if (r != 0u && r < 0x7f800000u) {
    const int ea = (int)(r >> 23) - 127;
    e = ((r & 0x007fffffu) <= 0x00600000u ? 8 : 7) - (r >= 0x00800000u ? ea : -126);
    e = e > 126 ? 126 : (e < -126 ? -126 : e);
  }
  const float s = __uint_as_float((uint32_t)(e + 127) << 23);
  if (threadIdx.x == 0) scale_inv[row] = __uint_as_float((uint32_t)(127 - e) << 23);
  uint8_t* hr = hi + row * ld;
  uint8_t* lr = lo + row * ld;
  // four columns per step; ld is a multiple of 16, columns from `cols` to ld are written as zeros
  for (int64_t c = (int64_t)threadIdx.x * 4; c < ld; c += (int64_t)kThreads * 4) {
    float p[4], q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = c + i < cols ? __uint_as_float((uint32_t)xr[c + i] << 16) * s : 0.0f;
    const uint32_t h = cvt_fp8x4<MI355Q_E4M3FN>(p[0], p[1], p[2], p[3]);
    cvt_f32x4<MI355Q_E4M3FN>(h, q[0], q[1], q[2], q[3]);
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = (p[i] - q[i]) * 16.0f;   // exact: p and hi agree in their leading bits
    const uint32_t l = cvt_fp8x4<MI355Q_E4M3FN>(q[0], q[1], q[2], q[3]);
    *reinterpret_cast<uint32_t*>(hr + c) = h;
    *reinterpret_cast<uint32_t*>(lr + c) = l;
  }
}

// The same split with the row held in registers (VPT 16-byte vectors of eight bf16 per thread): one pass
// over the row, every load in flight before the first is used, 8-byte stores.  For rows that start 16-byte
// aligned with cols a multiple of 8 and at most 8 * kThreads vectors; output columns from `cols` to ld
// come from lanes whose load falls outside the row's descriptor and reads zeros.  Same bits as the kernel above.
template <int VPT>
__global__ __launch_bounds__(kThreads) void split_rows_vec_kernel(const uint16_t* __restrict__ x, int64_t ldx, int64_t cols,
                                                                  uint8_t* __restrict__ hi, uint8_t* __restrict__ lo, int64_t ld,
                                                                  float* __restrict__ scale_inv) {
  __shared__ uint32_t wave_part[kThreads / 64];
  const int64_t row = blockIdx.x;
  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(x) + row * ldx, 0, (int)cols * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t rhi = __builtin_amdgcn_make_buffer_rsrc(hi + row * ld, 0, (int)ld, 0x00020000);
  const __amdgpu_buffer_rsrc_t rlo = __builtin_amdgcn_make_buffer_rsrc(lo + row * ld, 0, (int)ld, 0x00020000);
  u32x4 in[VPT];
#pragma unroll
  for (int u = 0; u < VPT; ++u)
    in[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rin, ((int)threadIdx.x + u * kThreads) * 16, 0, 0));
  uint32_t am = 0;
#pragma unroll
  for (int u = 0; u < VPT; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const u16x2 a = __builtin_bit_cast(u16x2, in[u][i] & 0x7fff7fffu);
      am = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am)));
    }
  {
    const uint32_t l16 = am & 0xffffu, h16 = am >> 16;
    am = (l16 > h16 ? l16 : h16) << 16;
  }
  am = wave_max_u32(am);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = am;
  __syncthreads();
  uint32_t r = wave_part[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) r = r > wave_part[w] ? r : wave_part[w];
  int e = 0;
  if (r != 0u && r < 0x7f800000u) {
    const int ea = (int)(r >> 23) - 127;
    e = ((r & 0x007fffffu) <= 0x00600000u ? 8 : 7) - (r >= 0x00800000u ? ea : -126);
    e = e > 126 ? 126 : (e < -126 ? -126 : e);
  }
  const float s = __uint_as_float((uint32_t)(e + 127) << 23);
  if (threadIdx.x == 0) scale_inv[row] = __uint_as_float((uint32_t)(127 - e) << 23);
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
    float p[8], q[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[2 * i] = __uint_as_float(in[u][i] << 16) * s;
      p[2 * i + 1] = __uint_as_float(in[u][i] & 0xffff0000u) * s;
    }
    const u32x2 h = {cvt_fp8x4<MI355Q_E4M3FN>(p[0], p[1], p[2], p[3]), cvt_fp8x4<MI355Q_E4M3FN>(p[4], p[5], p[6], p[7])};
    cvt_f32x4<MI355Q_E4M3FN>(h[0], q[0], q[1], q[2], q[3]);
    cvt_f32x4<MI355Q_E4M3FN>(h[1], q[4], q[5], q[6], q[7]);
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = (p[i] - q[i]) * 16.0f;
    const u32x2 l = {cvt_fp8x4<MI355Q_E4M3FN>(q[0], q[1], q[2], q[3]), cvt_fp8x4<MI355Q_E4M3FN>(q[4], q[5], q[6], q[7])};
    const int off = ((int)threadIdx.x + u * kThreads) * 8;
    __builtin_amdgcn_raw_buffer_store_b64(h, rhi, off, 0, 0);
    __builtin_amdgcn_raw_buffer_store_b64(l, rlo, off, 0, 0);
  }
}

// ------------------------------------------------- dynamic per-row quantisation
//
// One pass of "per-row amax -> scale = target / amax -> cast with that scale":
// a workgroup holds one row in registers (VPT 16-byte vectors per thread), so
// the row is read from HBM once.  Results are bit-identical to the three
// separate steps (rowwise_amax, an fp32 division, cast_to_fp8 with per-row
// scales); scale_inv = 1 / scale is what the GEMM takes as A_scale_inv.
template <bool BF16_IN, int FMT, int VPT>
__global__ __launch_bounds__(kThreads) void quantize_rows_kernel(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ y, int64_t vec_per_row, float target,
    float* __restrict__ scale_out, float* __restrict__ scale_inv_out) {
  __shared__ uint32_t wave_part[kThreads / 64];
  const int64_t row = blockIdx.x;
  // Descriptors over the row: a lane past its end loads zeros and its store is
  // dropped, so the body has no divergent branch and all loads are in flight
  // before the first is used.
  constexpr int OUT_BYTES = BF16_IN ? 8 : 4;  // per 16-byte input vector
  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(x) + row * vec_per_row * 16, 0, (int)vec_per_row * 16, 0x00020000);
  const __amdgpu_buffer_rsrc_t rout =
      __builtin_amdgcn_make_buffer_rsrc(y + row * vec_per_row * OUT_BYTES, 0, (int)vec_per_row * OUT_BYTES, 0x00020000);
  u32x4 in[VPT];
  uint32_t am = 0;
#pragma unroll
  for (int u = 0; u < VPT; ++u)
    in[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rin, ((int)threadIdx.x + u * kThreads) * 16, 0, 2));
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (BF16_IN) {
        const u16x2 a = __builtin_bit_cast(u16x2, in[u][i] & 0x7fff7fffu);
        am = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am)));
      } else {
        const uint32_t a = in[u][i] & 0x7fffffffu;
        am = am > a ? am : a;
      }
    }
  }
  if constexpr (BF16_IN) {
    const uint32_t lo = am & 0xffffu, hi = am >> 16;
    am = (lo > hi ? lo : hi) << 16;
  }
  am = wave_max_u32(am);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = am;
  __syncthreads();
  uint32_t r = wave_part[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) r = r > wave_part[w] ? r : wave_part[w];
  const float amax = __uint_as_float(r);
  const float scale = row_scale(target, amax);
  if (threadIdx.x == 0) {
    if (scale_out) scale_out[row] = scale;
    if (scale_inv_out) scale_inv_out[row] = 1.0f / scale;
  }
  const float s = BF16_IN ? round_to_bf16(scale) : scale;
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
    const int off = ((int)threadIdx.x + u * kThreads) * OUT_BYTES;
    if constexpr (BF16_IN) {
      float p[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[2 * i] = round_to_bf16(__uint_as_float(in[u][i] << 16) * s);
        p[2 * i + 1] = round_to_bf16(__uint_as_float(in[u][i] & 0xffff0000u) * s);
      }
      const u32x2 o = {cvt_fp8x4<FMT>(p[0], p[1], p[2], p[3]), cvt_fp8x4<FMT>(p[4], p[5], p[6], p[7])};
      __builtin_amdgcn_raw_buffer_store_b64(o, rout, off, 0, 2);
    } else {
      const uint32_t o = cvt_fp8x4<FMT>(__uint_as_float(in[u][0]) * s, __uint_as_float(in[u][1]) * s,
                                        __uint_as_float(in[u][2]) * s, __uint_as_float(in[u][3]) * s);
      __builtin_amdgcn_raw_buffer_store_b32(o, rout, off, 0, 2);
    }
  }
}

// SiLU(gate) * up in bf16 followed by the dynamic per-row quantisation above,
// in one pass: bf16(bf16(silu(gate)) * up), row amax of that, scale = target /
// amax, cast.  The glue between the gate / up projections and the down
// projection of a decoder MLP block; gate and up may be column ranges of one
// wider matrix (row pitches ld_gate, ld_up in elements).  h_out, when given,
// receives the bf16 products.
template <int FMT, int VPT>
__global__ __launch_bounds__(kThreads) void silu_mul_quantize_rows_kernel(
    const uint16_t* __restrict__ gate, int64_t ld_gate, const uint16_t* __restrict__ up, int64_t ld_up,
    uint8_t* __restrict__ y, uint16_t* __restrict__ h_out, int64_t vec_per_row, float target,
    float* __restrict__ scale_out, float* __restrict__ scale_inv_out) {
  __shared__ uint32_t wave_part[kThreads / 64];
  const int64_t row = blockIdx.x;
  // Descriptors over the row (zeros past its end, stores dropped there): no
  // divergent branch, and every load is in flight before the first is used.
  const int row_bytes = (int)vec_per_row * 16;
  const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(gate) + row * ld_gate, 0, row_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ru = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(up) + row * ld_up, 0, row_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(
      h_out ? h_out + row * vec_per_row * 8 : nullptr, 0, h_out ? row_bytes : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(y + row * vec_per_row * 8, 0, (int)vec_per_row * 8, 0x00020000);
  u32x4 gv[VPT], h[VPT];
  uint32_t am = 0;
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
    const int off = ((int)threadIdx.x + u * kThreads) * 16;
    gv[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rg, off, 0, 2));
    h[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ru, off, 0, 2));
  }
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float s0 = round_to_bf16(silu_f32(__uint_as_float(gv[u][i] << 16)));
      const float s1 = round_to_bf16(silu_f32(__uint_as_float(gv[u][i] & 0xffff0000u)));
      h[u][i] = pack_bf16x2(s0 * __uint_as_float(h[u][i] << 16), s1 * __uint_as_float(h[u][i] & 0xffff0000u));
      const u16x2 a = __builtin_bit_cast(u16x2, h[u][i] & 0x7fff7fffu);
      am = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am)));
    }
    // without h_out the descriptor is empty and the store goes nowhere
    __builtin_amdgcn_raw_buffer_store_b128(h[u], rh, ((int)threadIdx.x + u * kThreads) * 16, 0, 0);
  }
  {
    const uint32_t lo = am & 0xffffu, hi = am >> 16;
    am = (lo > hi ? lo : hi) << 16;
  }
  am = wave_max_u32(am);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = am;
  __syncthreads();
  uint32_t r = wave_part[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) r = r > wave_part[w] ? r : wave_part[w];
  const float amax = __uint_as_float(r);
  const float scale = row_scale(target, amax);
  if (threadIdx.x == 0) {
    if (scale_out) scale_out[row] = scale;
    if (scale_inv_out) scale_inv_out[row] = 1.0f / scale;
  }
  const float s = round_to_bf16(scale);
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
    float p[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[2 * i] = round_to_bf16(__uint_as_float(h[u][i] << 16) * s);
      p[2 * i + 1] = round_to_bf16(__uint_as_float(h[u][i] & 0xffff0000u) * s);
    }
    const u32x2 o = {cvt_fp8x4<FMT>(p[0], p[1], p[2], p[3]), cvt_fp8x4<FMT>(p[4], p[5], p[6], p[7])};
    __builtin_amdgcn_raw_buffer_store_b64(o, rout, ((int)threadIdx.x + u * kThreads) * 8, 0, 2);
  }
}

// The same, for many rows: bf16(silu(gate)) comes from a table in LDS.
//
// bf16(silu(x)) is a function of one bf16 value, 65536 cases in all, and most of
// them need no arithmetic: for |x| < 2^-8 it equals bf16(x / 2); for x >= 128 it
// is x; for finite x <= -128 it is -0 (silu_f32 returns -0 below -88.5).  The
// 2 x 1920 values in between are computed once per workgroup with silu_f32, the
// very function the kernel above calls per element, and kept in LDS; a workgroup
// then walks several rows.  An element costs about 20 vector instructions instead
// of about 50 (the exp and the IEEE division were 28 of them), which takes the
// kernel from the vector ALU's bound to HBM's.  Index arithmetic and the range
// fix-ups run on pairs of 16-bit lanes.  Results are bit-identical to the
// kernel above (checked on all 65536 gate values).
typedef short i16x2 __attribute__((ext_vector_type(2)));
constexpr int kSiluLo = 0x3b80;                     // bf16 bits of 2^-8
constexpr int kSiluHi = 0x4300;                     // bf16 bits of 128
constexpr int kSiluEntries = kSiluHi - kSiluLo;     // per sign

__device__ __forceinline__ void silu_table_build(uint16_t* tbl) {
  for (int i = threadIdx.x; i < 2 * kSiluEntries; i += kThreads) {
    const int sign = i >= kSiluEntries;
    const uint32_t bits = (uint32_t)(kSiluLo + (i - sign * kSiluEntries)) | ((uint32_t)sign << 15);
    tbl[i] = (uint16_t)(__float_as_uint(round_to_bf16(silu_f32(__uint_as_float(bits << 16)))) >> 16);
  }
}

// Packed 16-bit integer instructions, spelled out: written as C on 16-bit vector types the
// compiler turns the sign-mask idiom (x >> 15) back into compares and selects per half,
// three times the instructions.
#define MI355Q_PK_OP(name, mnemonic)                                                    \
  __device__ __forceinline__ uint32_t name(uint32_t a, uint32_t b) {                    \
    uint32_t r;                                                                         \
    asm(mnemonic " %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));                             \
    return r;                                                                           \
  }
MI355Q_PK_OP(pk_sub_u16, "v_pk_sub_u16")          // a - b per half, wrapping
MI355Q_PK_OP(pk_min_u16, "v_pk_min_u16")
MI355Q_PK_OP(pk_ashrrev_i16, "v_pk_ashrrev_i16")  // b >> a per half, arithmetic
MI355Q_PK_OP(pk_lshrrev_b16, "v_pk_lshrrev_b16")  // b >> a per half, logical
MI355Q_PK_OP(pk_lshlrev_b16, "v_pk_lshlrev_b16")  // b << a per half
#undef MI355Q_PK_OP
__device__ __forceinline__ uint32_t pk_mad_u16(uint32_t a, uint32_t b, uint32_t c) {
  uint32_t r;
  asm("v_pk_mad_u16 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ uint32_t select_bits(uint32_t mask, uint32_t if_set, uint32_t if_clear) {
  return (if_set & mask) | (if_clear & ~mask);  // v_bfi_b32
}

// bf16(silu(x)) of the two bf16 values in w, as two bf16 values.
__device__ __forceinline__ uint32_t silu_bf16x2_lookup(uint32_t w, const uint16_t* tbl) {
  constexpr uint32_t k15 = 0x000f000fu, k1 = 0x00010001u;
  constexpr uint32_t kLo = (uint32_t)kSiluLo * 0x00010001u, kHiM1 = (uint32_t)(kSiluHi - 1) * 0x00010001u;
  constexpr uint32_t kN = (uint32_t)kSiluEntries * 0x00010001u, kNM1 = (uint32_t)(kSiluEntries - 1) * 0x00010001u;
  const uint32_t a = w & 0x7fff7fffu;
  const uint32_t d = pk_sub_u16(a, kLo);                              // negative as int16: |x| < 2^-8
  const uint32_t m_small = pk_ashrrev_i16(k15, d);
  const uint32_t m_big = pk_ashrrev_i16(k15, pk_sub_u16(kHiM1, a));   // |x| >= 128, inf, NaN
  const uint32_t idx = pk_mad_u16(pk_lshrrev_b16(k15, w), kN, pk_min_u16(d, kNM1));
  const uint32_t off = pk_lshlrev_b16(k1, idx);                       // byte offsets into the table
  const uint8_t* tb = reinterpret_cast<const uint8_t*>(tbl);
  const uint32_t t = (uint32_t)*reinterpret_cast<const uint16_t*>(tb + (off & 0xffffu)) |
                     ((uint32_t)*reinterpret_cast<const uint16_t*>(tb + (off >> 16)) << 16);
  // |x| < 2^-8: bf16(x / 2)
  const uint32_t small = pack_bf16x2(__uint_as_float(w << 16) * 0.5f, __uint_as_float(w & 0xffff0000u) * 0.5f);
  // |x| >= 128: x when positive; -0 when negative and finite, NaN for -inf (= -inf / inf) and NaN
  const uint32_t m_naninf = pk_ashrrev_i16(k15, pk_sub_u16(0x7f7f7f7fu, a));
  const uint32_t neg = 0x80008000u | (m_naninf & 0x7fc07fc0u);
  const uint32_t big = select_bits(pk_ashrrev_i16(k15, w), neg, w);
  return select_bits(m_small, small, select_bits(m_big, big, t));
}

template <int FMT, int VPT>
__global__ __launch_bounds__(kThreads) void silu_mul_quantize_rows_table_kernel(
    const uint16_t* __restrict__ gate, int64_t ld_gate, const uint16_t* __restrict__ up, int64_t ld_up,
    uint8_t* __restrict__ y, uint16_t* __restrict__ h_out, int64_t rows, int64_t vec_per_row, float target,
    float* __restrict__ scale_out, float* __restrict__ scale_inv_out) {
  __shared__ uint16_t tbl[2 * kSiluEntries];
  __shared__ uint32_t wave_part[2][kThreads / 64];
  silu_table_build(tbl);
  __syncthreads();
  const int row_bytes = (int)vec_per_row * 16;
  int parity = 0;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x, parity ^= 1) {
    const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(gate) + row * ld_gate, 0, row_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ru = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(up) + row * ld_up, 0, row_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(
        h_out ? h_out + row * vec_per_row * 8 : nullptr, 0, h_out ? row_bytes : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(y + row * vec_per_row * 8, 0, (int)vec_per_row * 8, 0x00020000);
    u32x4 gv[VPT], h[VPT];
    uint32_t am = 0;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      const int off = ((int)threadIdx.x + u * kThreads) * 16;
      gv[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rg, off, 0, 2));
      h[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ru, off, 0, 2));
    }
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t s = silu_bf16x2_lookup(gv[u][i], tbl);
        h[u][i] = pack_bf16x2(__uint_as_float(s << 16) * __uint_as_float(h[u][i] << 16),
                              __uint_as_float(s & 0xffff0000u) * __uint_as_float(h[u][i] & 0xffff0000u));
        const u16x2 a = __builtin_bit_cast(u16x2, h[u][i] & 0x7fff7fffu);
        am = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am)));
      }
      __builtin_amdgcn_raw_buffer_store_b128(h[u], rh, ((int)threadIdx.x + u * kThreads) * 16, 0, 0);
    }
    {
      const uint32_t lo = am & 0xffffu, hi = am >> 16;
      am = (lo > hi ? lo : hi) << 16;
    }
    am = wave_max_u32(am);
    // two exchange areas, used in turn: a wave may start the next row while another still reads this one's
    if ((threadIdx.x & 63) == 0) wave_part[parity][threadIdx.x >> 6] = am;
    __syncthreads();
    uint32_t r = wave_part[parity][0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) r = r > wave_part[parity][w] ? r : wave_part[parity][w];
    const float scale = row_scale(target, __uint_as_float(r));
    if (threadIdx.x == 0) {
      if (scale_out) scale_out[row] = scale;
      if (scale_inv_out) scale_inv_out[row] = 1.0f / scale;
    }
    const float s = round_to_bf16(scale);
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      float p[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[2 * i] = round_to_bf16(__uint_as_float(h[u][i] << 16) * s);
        p[2 * i + 1] = round_to_bf16(__uint_as_float(h[u][i] & 0xffff0000u) * s);
      }
      const u32x2 o = {cvt_fp8x4<FMT>(p[0], p[1], p[2], p[3]), cvt_fp8x4<FMT>(p[4], p[5], p[6], p[7])};
      __builtin_amdgcn_raw_buffer_store_b64(o, rout, ((int)threadIdx.x + u * kThreads) * 8, 0, 2);
    }
  }
}

// -------------------------------------------------------------- cast_from_fp8
//
// A lane produces one 16-byte store: 8 fp8 bytes in for bf16 output, 4 for
// fp32 output.  A wave's store then covers 1 KiB of whole cache lines; wider
// loads would leave each lane with several stores that each touch only part
// of a line, and those partial-line writes cost HBM bandwidth.
template <bool BF16_OUT>
constexpr int from_vec() { return BF16_OUT ? 8 : 4; }

// WINDOW: stores a wave may still have outstanding when it issues the next one
// (-1: no limit).  Measured for bf16 output, which writes twice the bytes it
// reads: with 2 the kernel is 3-8 % faster than unlimited from 64 MiB of output
// up (6.2 TB/s at 512 MiB), with 0 it is 9 % faster at 32 MiB; other sizes do
// not care.  fp32 output and cast_to_fp8 (more reads than writes) lose with any limit.
template <int FMT, bool BF16_OUT, int SK, int U, int WINDOW>
__global__ __launch_bounds__(kThreads) void cast_from_fp8_vec(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ y, const float* __restrict__ scale,
    float scale_host, int scale_is_dev, int has_scale, int64_t vec_per_row,
    int64_t blocks_per_row, int64_t mid) {
  constexpr int V = from_vec<BF16_OUT>();
  constexpr int kNt = 2;  // non-temporal
  const int64_t row = blockIdx.x / blocks_per_row;
  const int64_t vec0 = (blockIdx.x - row * blocks_per_row) * (int64_t)(kThreads * U);  // first vector, within the row
  const int64_t left = vec_per_row - vec0;
  const int nvec = (int)(left < kThreads * U ? left : kThreads * U);
  const int64_t first = row * vec_per_row + vec0;                                    // first vector, within the tensor
  // Branch-free like cast_to_fp8_vec8: descriptors that cover the block's
  // vectors make a lane past the end load zeros and drop its store.
  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(x) + first * V, 0, nvec * V, 0x00020000);
  const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(y + first * 16, 0, nvec * 16, 0x00020000);

  float s = 1.0f;
  if constexpr (SK == SK_SCALAR) s = scale_is_dev ? scale[0] : scale_host;
  if constexpr (SK == SK_ROW) s = scale[row % mid];
  if constexpr (BF16_OUT) s = round_to_bf16(s);
  if (!has_scale) s = 1.0f;  // x * 1 == x bit for bit (NaN payloads aside, and fp8 NaNs have one)

  uint32_t in[U][V / 4];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int off = ((int)threadIdx.x + u * kThreads) * V;
    if constexpr (V == 8) {
      const u32x2 t = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rin, off, 0, kNt));
      in[u][0] = t[0];
      in[u][1] = t[1];
    } else {
      in[u][0] = __builtin_amdgcn_raw_buffer_load_b32(rin, off, 0, kNt);
    }
  }
  constexpr bool kVecScale = SK == SK_COL || SK == SK_FULL;
  u32x4 sc[kVecScale ? U : 1][V / 4];
  if constexpr (kVecScale) {  // the launcher picks these kinds only for a scale tensor
    const float* sbase = scale + (SK == SK_COL ? vec0 : first) * V;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sbase), 0, nvec * V * 4, 0x00020000);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int q = 0; q < V / 4; ++q)
        sc[u][q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, ((int)threadIdx.x + u * kThreads) * V * 4 + 16 * q, 0, 0));
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float v[V];
#pragma unroll
    for (int i = 0; i < V / 4; ++i)
      cvt_f32x4<FMT>(in[u][i], v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      float sv = s;
      if constexpr (kVecScale) {
        sv = __uint_as_float(sc[u][i >> 2][i & 3]);
        if constexpr (BF16_OUT) sv = round_to_bf16(sv);
      }
      v[i] *= sv;
    }
    u32x4 t;
    if constexpr (BF16_OUT) {
#pragma unroll
      for (int i = 0; i < 4; ++i) t[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
    } else {
      t = u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])};
    }
    __builtin_amdgcn_raw_buffer_store_b128(t, rout, ((int)threadIdx.x + u * kThreads) * 16, 0, kNt);
    if constexpr (WINDOW >= 0) {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0x0F70 | WINDOW);  // vmcnt(WINDOW), other counters unlimited
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

template <int FMT, bool BF16_OUT>
__global__ __launch_bounds__(kThreads) void cast_from_fp8_generic(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ y, const float* __restrict__ scale,
    float scale_host, int mode, int64_t start, int64_t n, int64_t mid, int64_t inner) {
  const int64_t i = start + (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  float v = cvt_f32x1<FMT>(x[i]);
  if (mode != MI355Q_SCALE_NONE) {
    float s = 1.0f;
    if (mode == MI355Q_SCALE_HOST) s = scale_host;
    else if (mode == MI355Q_SCALE_DEV) s = scale[0];
    else if (mode == MI355Q_SCALE_MID) s = scale[(i / inner) % mid];
    else if (mode == MI355Q_SCALE_FULL) s = scale[i];
    if constexpr (BF16_OUT) s = round_to_bf16(s);
    v *= s;
  }
  if constexpr (BF16_OUT) reinterpret_cast<uint16_t*>(y)[i] = (uint16_t)(pack_bf16x2(v, v) & 0xffffu);
  else reinterpret_cast<float*>(y)[i] = v;
}

__global__ __launch_bounds__(kThreads) void copy_bytes_kernel(const uint8_t* __restrict__ x,
                                                              uint8_t* __restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < n) y[i] = x[i];
}

constexpr int kCopyU = 4;  // 16-byte vectors per thread

// A block copies kThreads * kCopyU vectors through descriptors that end with
// the tensor: all loads of a lane are issued before its first store.
__global__ __launch_bounds__(kThreads) void copy_vec16_kernel(const uint8_t* __restrict__ x,
                                                              uint8_t* __restrict__ y, int64_t nvec) {
  const int64_t v0 = (int64_t)blockIdx.x * (kThreads * kCopyU);
  const int64_t left = nvec - v0;
  const int bytes = (int)(left < kThreads * kCopyU ? left : kThreads * kCopyU) * 16;
  const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(x) + v0 * 16, 0, bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(y + v0 * 16, 0, bytes, 0x00020000);
  u32x4 t[kCopyU];
#pragma unroll
  for (int u = 0; u < kCopyU; ++u)
    t[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rin, ((int)threadIdx.x + u * kThreads) * 16, 0, 2));
#pragma unroll
  for (int u = 0; u < kCopyU; ++u)
    __builtin_amdgcn_raw_buffer_store_b128(t[u], rout, ((int)threadIdx.x + u * kThreads) * 16, 0, 2);
}

// --------------------------------------------------------------- host helpers

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline int launch_status() { return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH; }
inline unsigned blocks_for(int64_t n, int64_t per) { return (unsigned)((n + per - 1) / per); }

// Decide how the vector kernels see the problem.  Returns false when only the
// generic kernel applies.
struct VecPlan {
  int sk;
  int64_t rows, row_len, mid;
};

inline bool plan_vectors(int mode, int64_t outer, int64_t mid, int64_t inner, int64_t vec,
                         VecPlan* p) {
  const int64_t n = outer * mid * inner;
  switch (mode) {
    case MI355Q_SCALE_NONE:
    case MI355Q_SCALE_HOST:
    case MI355Q_SCALE_DEV:
      *p = {SK_SCALAR, 1, n, 1};
      return true;
    case MI355Q_SCALE_FULL:
      *p = {SK_FULL, 1, n, 1};
      return true;
    case MI355Q_SCALE_MID:
      if (inner == 1) {  // per column of [outer, mid]
        if (mid % vec != 0 || mid < 4 * vec) return false;
        *p = {SK_COL, outer, mid, mid};
        return true;
      }
      if (inner % vec != 0 || inner < 4 * vec) return false;
      *p = {SK_ROW, outer * mid, inner, mid};
      return true;
    default:
      return false;
  }
}

constexpr int kCastU = 4;  // 16-byte loads in flight per thread

template <bool BF16_IN, int FMT, bool AMAX>
void launch_cast_to_vec(int sk, hipStream_t st, const uint8_t* x, uint8_t* y, const float* scale,
                        float sh, int is_dev, int64_t vpr, int64_t bpr, int64_t total, int64_t mid,
                        uint32_t* amax) {
  constexpr int U = kCastU;
  constexpr int T = AMAX ? kAmaxThreads : kThreads;
  const unsigned grid = (unsigned)(AMAX && total > kAmaxBlocks ? kAmaxBlocks : total);
  switch (sk) {
    case SK_SCALAR:
      cast_to_fp8_vec8<BF16_IN, FMT, SK_SCALAR, AMAX, U><<<grid, T, 0, st>>>(x, y, scale, sh, is_dev, vpr, bpr, total, mid, amax);
      break;
    case SK_ROW:
      cast_to_fp8_vec8<BF16_IN, FMT, SK_ROW, AMAX, U><<<grid, T, 0, st>>>(x, y, scale, sh, is_dev, vpr, bpr, total, mid, amax);
      break;
    case SK_COL:
      cast_to_fp8_vec8<BF16_IN, FMT, SK_COL, AMAX, U><<<grid, T, 0, st>>>(x, y, scale, sh, is_dev, vpr, bpr, total, mid, amax);
      break;
    default:
      cast_to_fp8_vec8<BF16_IN, FMT, SK_FULL, AMAX, U><<<grid, T, 0, st>>>(x, y, scale, sh, is_dev, vpr, bpr, total, mid, amax);
      break;
  }
}

template <bool BF16_IN, int FMT>
int cast_to_dispatch(const uint8_t* x, uint8_t* y, const float* scale, float sh, int mode,
                     int64_t outer, int64_t mid, int64_t inner, uint32_t* amax, hipStream_t st) {
  constexpr int U = kCastU;
  const int64_t n = outer * mid * inner;
  VecPlan p;
  const bool vec = aligned(x, 16) && aligned(y, 8) &&
                   (scale == nullptr || aligned(scale, 16)) && plan_vectors(mode, outer, mid, inner, 8, &p);
  int64_t done = 0;
  if (vec) {
    const int64_t vpr = p.row_len / 8;
    // In flat modes the row length need not be a multiple of 8: the tail goes
    // to the generic kernel.  In 2-D modes plan_vectors has required it.
    if (vpr > 0) {
      const int64_t per_block = (int64_t)(amax ? kAmaxThreads : kThreads) * U;
      const int64_t bpr = (vpr + per_block - 1) / per_block;
      const int64_t total = bpr * p.rows;
      if (total > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
      const int is_dev = mode == MI355Q_SCALE_DEV;
      if (amax) launch_cast_to_vec<BF16_IN, FMT, true>(p.sk, st, x, y, scale, sh, is_dev, vpr, bpr, total, p.mid, amax);
      else launch_cast_to_vec<BF16_IN, FMT, false>(p.sk, st, x, y, scale, sh, is_dev, vpr, bpr, total, p.mid, amax);
      done = p.rows == 1 ? vpr * 8 : n;
    }
  }
  if (done < n) {
    const int64_t rest = n - done;
    const int64_t grid = (rest + kThreads - 1) / kThreads;
    if (grid > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    cast_to_fp8_generic<BF16_IN, FMT><<<(unsigned)grid, kThreads, 0, st>>>(x, y, scale, sh, mode, done, n, mid, inner, amax);
  }
  return launch_status();
}

template <int FMT, bool BF16_OUT>
int cast_from_dispatch(const uint8_t* x, uint8_t* y, const float* scale, float sh, int mode,
                       int64_t outer, int64_t mid, int64_t inner, hipStream_t st) {
  constexpr int U = 4;
  constexpr int V = from_vec<BF16_OUT>();
  const int64_t n = outer * mid * inner;
  VecPlan p;
  const bool vec = aligned(x, V) && aligned(y, 16) &&
                   (scale == nullptr || aligned(scale, 16)) && plan_vectors(mode, outer, mid, inner, V, &p);
  int64_t done = 0;
  if (vec) {
    const int64_t vpr = p.row_len / V;
    if (vpr > 0) {
      const int64_t bpr = (vpr + kThreads * U - 1) / (kThreads * U);
      const int64_t grid64 = bpr * p.rows;
      if (grid64 > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
      const unsigned grid = (unsigned)grid64;
      const int is_dev = mode == MI355Q_SCALE_DEV;
      const int has_scale = mode != MI355Q_SCALE_NONE;
      auto launch = [&](auto window) {
        constexpr int W = decltype(window)::value;
        switch (p.sk) {
          case SK_SCALAR:
            cast_from_fp8_vec<FMT, BF16_OUT, SK_SCALAR, U, W><<<grid, kThreads, 0, st>>>(x, y, scale, sh, is_dev, has_scale, vpr, bpr, p.mid);
            break;
          case SK_ROW:
            cast_from_fp8_vec<FMT, BF16_OUT, SK_ROW, U, W><<<grid, kThreads, 0, st>>>(x, y, scale, sh, is_dev, has_scale, vpr, bpr, p.mid);
            break;
          case SK_COL:
            cast_from_fp8_vec<FMT, BF16_OUT, SK_COL, U, W><<<grid, kThreads, 0, st>>>(x, y, scale, sh, is_dev, has_scale, vpr, bpr, p.mid);
            break;
          default:
            cast_from_fp8_vec<FMT, BF16_OUT, SK_FULL, U, W><<<grid, kThreads, 0, st>>>(x, y, scale, sh, is_dev, has_scale, vpr, bpr, p.mid);
            break;
        }
      };
      if constexpr (BF16_OUT) {
        if (n * 2 <= (int64_t(48) << 20)) launch(std::integral_constant<int, 0>{});
        else launch(std::integral_constant<int, 2>{});
      } else {
        launch(std::integral_constant<int, -1>{});
      }
      done = p.rows == 1 ? vpr * V : n;
    }
  }
  if (done < n) {
    const int64_t grid = (n - done + kThreads - 1) / kThreads;
    if (grid > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    cast_from_fp8_generic<FMT, BF16_OUT><<<(unsigned)grid, kThreads, 0, st>>>(x, y, scale, sh, mode, done, n, mid, inner);
  }
  return launch_status();
}

inline bool scale_args_ok(const float* scale, int mode, int64_t outer, int64_t mid, int64_t inner) {
  if (mode < MI355Q_SCALE_NONE || mode > MI355Q_SCALE_FULL) return false;
  if (outer < 0 || mid < 0 || inner < 0) return false;
  if ((mode == MI355Q_SCALE_DEV || mode == MI355Q_SCALE_MID || mode == MI355Q_SCALE_FULL) && scale == nullptr)
    return false;
  return true;
}

template <bool BF16_IN, int FMT>
int quantize_rows_launch(const uint8_t* x, uint8_t* y, int64_t rows, int64_t vpr, float target,
                                float* scale_out, float* scale_inv_out, hipStream_t st) {
  const unsigned grid = (unsigned)rows;
  if (vpr <= kThreads) quantize_rows_kernel<BF16_IN, FMT, 1><<<grid, kThreads, 0, st>>>(x, y, vpr, target, scale_out, scale_inv_out);
  else if (vpr <= 2 * kThreads) quantize_rows_kernel<BF16_IN, FMT, 2><<<grid, kThreads, 0, st>>>(x, y, vpr, target, scale_out, scale_inv_out);
  else if (vpr <= 4 * kThreads) quantize_rows_kernel<BF16_IN, FMT, 4><<<grid, kThreads, 0, st>>>(x, y, vpr, target, scale_out, scale_inv_out);
  else if (vpr <= 8 * kThreads) quantize_rows_kernel<BF16_IN, FMT, 8><<<grid, kThreads, 0, st>>>(x, y, vpr, target, scale_out, scale_inv_out);
  else return MI355Q_ERR_UNSUPPORTED;
  return launch_status();
}

// The table kernel pays for its table (15 silu evaluations per thread) once per workgroup:
// it runs from this many rows on, with a fixed number of workgroups.
constexpr int64_t kSiluTableMinRows = 2048;
inline int silu_table_workgroups() {
  static const int n = [] {
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0)
      cu = 256;
    return cu * 4;  // measured at 4096 x 14336: 2 per compute unit 70 us, 4: 62.5, 8: 63.7
  }();
  return n;
}

template <int FMT>
int silu_mul_quantize_rows_launch(const uint16_t* gate, int64_t ld_gate, const uint16_t* up, int64_t ld_up,
                                  uint8_t* y, uint16_t* h_out, int64_t rows, int64_t vpr, float target,
                                  float* scale_out, float* scale_inv_out, hipStream_t st) {
  // Many rows: workgroups that build the silu table once and walk several rows each.
  if (rows >= kSiluTableMinRows && vpr <= 8 * kThreads) {
    const int64_t want = (int64_t)silu_table_workgroups();
    const unsigned tg = (unsigned)(rows < want ? rows : want);
    if (vpr <= kThreads) silu_mul_quantize_rows_table_kernel<FMT, 1><<<tg, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, rows, vpr, target, scale_out, scale_inv_out);
    else if (vpr <= 2 * kThreads) silu_mul_quantize_rows_table_kernel<FMT, 2><<<tg, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, rows, vpr, target, scale_out, scale_inv_out);
    else if (vpr <= 4 * kThreads) silu_mul_quantize_rows_table_kernel<FMT, 4><<<tg, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, rows, vpr, target, scale_out, scale_inv_out);
    else silu_mul_quantize_rows_table_kernel<FMT, 8><<<tg, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, rows, vpr, target, scale_out, scale_inv_out);
    return launch_status();
  }
  const unsigned grid = (unsigned)rows;
  if (vpr <= kThreads) silu_mul_quantize_rows_kernel<FMT, 1><<<grid, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, vpr, target, scale_out, scale_inv_out);
  else if (vpr <= 2 * kThreads) silu_mul_quantize_rows_kernel<FMT, 2><<<grid, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, vpr, target, scale_out, scale_inv_out);
  else if (vpr <= 4 * kThreads) silu_mul_quantize_rows_kernel<FMT, 4><<<grid, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, vpr, target, scale_out, scale_inv_out);
  else if (vpr <= 8 * kThreads) silu_mul_quantize_rows_kernel<FMT, 8><<<grid, kThreads, 0, st>>>(gate, ld_gate, up, ld_up, y, h_out, vpr, target, scale_out, scale_inv_out);
  else return MI355Q_ERR_UNSUPPORTED;
  return launch_status();
}

}  // namespace mi355q

using namespace mi355q;

extern "C" {

int mi355q_amax(const void* x, int x_dtype, int64_t n, float* amax_out, void* stream) {
  if (amax_out == nullptr || n < 0 || (n > 0 && x == nullptr)) return MI355Q_ERR_INVALID_ARGUMENT;
  if (x_dtype != MI355Q_F32 && x_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t* am = reinterpret_cast<uint32_t*>(amax_out);
  fill_u32_kernel<<<1, 1, 0, st>>>(am, 0u);
  if (n == 0) return launch_status();
  constexpr int U = 4;
  const int es = x_dtype == MI355Q_BF16 ? 2 : 4;
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  int64_t done = 0;
  if (aligned(x, 16)) {
    const int64_t nvec = n * es / 16;
    if (nvec > 0) {
      int64_t grid = (nvec + kAmaxThreads * U - 1) / (kAmaxThreads * U);
      if (grid > kAmaxBlocks) grid = kAmaxBlocks;
      if (x_dtype == MI355Q_BF16) amax_vec<true, U><<<(unsigned)grid, kAmaxThreads, 0, st>>>(xb, nvec, am);
      else amax_vec<false, U><<<(unsigned)grid, kAmaxThreads, 0, st>>>(xb, nvec, am);
      done = nvec * (16 / es);
    }
  }
  if (done < n) {
    const int64_t grid = (n - done + kThreads - 1) / kThreads;
    if (grid > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    if (x_dtype == MI355Q_BF16) amax_generic<true><<<(unsigned)grid, kThreads, 0, st>>>(xb, done, n, am);
    else amax_generic<false><<<(unsigned)grid, kThreads, 0, st>>>(xb, done, n, am);
  }
  return launch_status();
}

int mi355q_rowwise_amax(const void* x, int x_dtype, int64_t rows, int64_t cols, float* amax_out,
                        void* stream) {
  if (rows < 0 || cols < 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows == 0) return MI355Q_OK;
  if (amax_out == nullptr || (cols > 0 && x == nullptr)) return MI355Q_ERR_INVALID_ARGUMENT;
  if (x_dtype != MI355Q_F32 && x_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int es = x_dtype == MI355Q_BF16 ? 2 : 4;
  const int vec_ok = aligned(x, 16) && (cols * es) % 16 == 0;
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  if (x_dtype == MI355Q_BF16) rowwise_amax_kernel<true><<<(unsigned)rows, kThreads, 0, st>>>(xb, cols, vec_ok, amax_out);
  else rowwise_amax_kernel<false><<<(unsigned)rows, kThreads, 0, st>>>(xb, cols, vec_ok, amax_out);
  return launch_status();
}

int mi355q_cast_to_fp8_sr(const void* x, int x_dtype, void* y, int fp8_fmt, const float* scale_dev,
                          float scale_host, int scale_mode, int64_t outer, int64_t mid, int64_t inner,
                          float* amax_out, uint64_t seed, uint64_t offset, int flush_subnormals, void* stream) {
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (x_dtype != MI355Q_F32 && x_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (!scale_args_ok(scale_dev, scale_mode, outer, mid, inner)) return MI355Q_ERR_INVALID_ARGUMENT;
  const int64_t n = outer * mid * inner;
  if (n > 0 && (x == nullptr || y == nullptr)) return MI355Q_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t* am = reinterpret_cast<uint32_t*>(amax_out);
  if (am) fill_u32_kernel<<<1, 1, 0, st>>>(am, 0u);
  if (n == 0) return launch_status();
  const int64_t grid = ((n + 3) / 4 + kThreads - 1) / kThreads;
  if (grid > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  const unsigned g = (unsigned)grid;
  if (x_dtype == MI355Q_BF16) {
    if (fp8_fmt == MI355Q_E4M3FN) cast_to_fp8_sr_kernel<true, MI355Q_E4M3FN><<<g, kThreads, 0, st>>>(xb, yb, scale_dev, scale_host, scale_mode, n, mid, inner, seed, offset, flush_subnormals, am);
    else cast_to_fp8_sr_kernel<true, MI355Q_E5M2><<<g, kThreads, 0, st>>>(xb, yb, scale_dev, scale_host, scale_mode, n, mid, inner, seed, offset, flush_subnormals, am);
  } else {
    if (fp8_fmt == MI355Q_E4M3FN) cast_to_fp8_sr_kernel<false, MI355Q_E4M3FN><<<g, kThreads, 0, st>>>(xb, yb, scale_dev, scale_host, scale_mode, n, mid, inner, seed, offset, flush_subnormals, am);
    else cast_to_fp8_sr_kernel<false, MI355Q_E5M2><<<g, kThreads, 0, st>>>(xb, yb, scale_dev, scale_host, scale_mode, n, mid, inner, seed, offset, flush_subnormals, am);
  }
  return launch_status();
}

int mi355q_cast_to_fp8_hybrid(const void* x, int x_dtype, int64_t n, void* y_e5m2, void* y_e4m3fn,
                              const float* scale_e5m2, const float* scale_e4m3fn, int stochastic,
                              uint64_t seed, uint64_t offset, float* amax_out, void* stream) {
  if (n < 0 || (x_dtype != MI355Q_F32 && x_dtype != MI355Q_BF16)) return MI355Q_ERR_INVALID_ARGUMENT;
  if (n > 0 && (x == nullptr || y_e5m2 == nullptr || y_e4m3fn == nullptr)) return MI355Q_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t* am = reinterpret_cast<uint32_t*>(amax_out);
  if (am) fill_u32_kernel<<<1, 1, 0, st>>>(am, 0u);
  if (n == 0) return launch_status();
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* y5 = static_cast<uint8_t*>(y_e5m2);
  uint8_t* y4 = static_cast<uint8_t*>(y_e4m3fn);
  const int64_t max_blocks = am ? kAmaxBlocks : 4 * kAmaxBlocks;
  auto grid_for = [&](int64_t steps) {
    const int64_t b = (steps + kAmaxThreads - 1) / kAmaxThreads;
    return (unsigned)(b < max_blocks ? b : max_blocks);
  };
  int64_t done = 0;
  if (aligned(x, 16) && aligned(y5, 8) && aligned(y4, 8) && n >= 8) {
    const int64_t nv = n / 8;
    if (x_dtype == MI355Q_BF16) cast_to_fp8_hybrid_kernel<true, 8><<<grid_for(nv), kAmaxThreads, 0, st>>>(xb, y5, y4, scale_e5m2, scale_e4m3fn, 0, nv * 8, stochastic, seed, offset, am);
    else cast_to_fp8_hybrid_kernel<false, 8><<<grid_for(nv), kAmaxThreads, 0, st>>>(xb, y5, y4, scale_e5m2, scale_e4m3fn, 0, nv * 8, stochastic, seed, offset, am);
    done = nv * 8;
  }
  if (done < n) {
    const int64_t rest = n - done;
    if (x_dtype == MI355Q_BF16) cast_to_fp8_hybrid_kernel<true, 1><<<grid_for(rest), kAmaxThreads, 0, st>>>(xb, y5, y4, scale_e5m2, scale_e4m3fn, done, rest, stochastic, seed, offset, am);
    else cast_to_fp8_hybrid_kernel<false, 1><<<grid_for(rest), kAmaxThreads, 0, st>>>(xb, y5, y4, scale_e5m2, scale_e4m3fn, done, rest, stochastic, seed, offset, am);
  }
  return launch_status();
}

int mi355q_split_rows_fp8x2(const void* x, int x_dtype, int64_t ldx, int64_t rows, int64_t cols, void* hi, void* lo,
                            int64_t ld, float* scale_inv, void* stream) {
  if (x_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows < 0 || cols < 0 || ldx < cols || ld < cols) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows == 0) return MI355Q_OK;
  if (x == nullptr || hi == nullptr || lo == nullptr || scale_inv == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (ld % 16 != 0 || !aligned(hi, 16) || !aligned(lo, 16) || rows > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* xs = static_cast<const uint16_t*>(x);
  uint8_t* h8 = static_cast<uint8_t*>(hi);
  uint8_t* l8 = static_cast<uint8_t*>(lo);
  const unsigned grid = (unsigned)rows;
  const int64_t vpr = ld / 8;  // output vectors of a row
  if (cols % 8 == 0 && ldx % 8 == 0 && aligned(x, 16) && vpr <= 8 * kThreads) {
    if (vpr <= kThreads) split_rows_vec_kernel<1><<<grid, kThreads, 0, st>>>(xs, ldx, cols, h8, l8, ld, scale_inv);
    else if (vpr <= 2 * kThreads) split_rows_vec_kernel<2><<<grid, kThreads, 0, st>>>(xs, ldx, cols, h8, l8, ld, scale_inv);
    else if (vpr <= 4 * kThreads) split_rows_vec_kernel<4><<<grid, kThreads, 0, st>>>(xs, ldx, cols, h8, l8, ld, scale_inv);
    else split_rows_vec_kernel<8><<<grid, kThreads, 0, st>>>(xs, ldx, cols, h8, l8, ld, scale_inv);
  } else {
    split_rows_kernel<<<grid, kThreads, 0, st>>>(xs, ldx, cols, h8, l8, ld, scale_inv);
  }
  return launch_status();
}

int mi355q_quantize_rows(const void* x, int x_dtype, int64_t rows, int64_t cols, void* y, int fp8_fmt,
                         float target, float* scale_out, float* scale_inv_out, void* stream) {
  if (rows < 0 || cols < 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (x_dtype != MI355Q_F32 && x_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return MI355Q_OK;
  if (x == nullptr || y == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
  const int epv = x_dtype == MI355Q_BF16 ? 8 : 4;
  // whole 16-byte vectors only; the row has to fit the registers of one workgroup
  if (cols % epv != 0 || !aligned(x, 16) || !aligned(y, epv)) return MI355Q_ERR_UNSUPPORTED;
  const int64_t vpr = cols / epv;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  if (x_dtype == MI355Q_BF16) {
    if (fp8_fmt == MI355Q_E4M3FN) return quantize_rows_launch<true, MI355Q_E4M3FN>(xb, yb, rows, vpr, target, scale_out, scale_inv_out, st);
    return quantize_rows_launch<true, MI355Q_E5M2>(xb, yb, rows, vpr, target, scale_out, scale_inv_out, st);
  }
  if (fp8_fmt == MI355Q_E4M3FN) return quantize_rows_launch<false, MI355Q_E4M3FN>(xb, yb, rows, vpr, target, scale_out, scale_inv_out, st);
  return quantize_rows_launch<false, MI355Q_E5M2>(xb, yb, rows, vpr, target, scale_out, scale_inv_out, st);
}

int mi355q_silu_mul_quantize_rows(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                  int64_t rows, int64_t cols, void* y, int fp8_fmt, float target,
                                  void* h_out, float* scale_out, float* scale_inv_out, void* stream) {
  if (rows < 0 || cols < 0 || ld_gate < cols || ld_up < cols) return MI355Q_ERR_INVALID_ARGUMENT;
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return MI355Q_OK;
  if (gate == nullptr || up == nullptr || y == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
  // whole 16-byte vectors only; the row has to fit the registers of one workgroup
  if (cols % 8 != 0 || ld_gate % 8 != 0 || ld_up % 8 != 0 || !aligned(gate, 16) || !aligned(up, 16) ||
      !aligned(y, 8) || (h_out && !aligned(h_out, 16)))
    return MI355Q_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* g = static_cast<const uint16_t*>(gate);
  const uint16_t* u = static_cast<const uint16_t*>(up);
  uint8_t* yb = static_cast<uint8_t*>(y);
  uint16_t* hb = static_cast<uint16_t*>(h_out);
  if (fp8_fmt == MI355Q_E4M3FN)
    return silu_mul_quantize_rows_launch<MI355Q_E4M3FN>(g, ld_gate, u, ld_up, yb, hb, rows, cols / 8, target, scale_out, scale_inv_out, st);
  return silu_mul_quantize_rows_launch<MI355Q_E5M2>(g, ld_gate, u, ld_up, yb, hb, rows, cols / 8, target, scale_out, scale_inv_out, st);
}

int mi355q_cast_to_fp8(const void* x, int x_dtype, void* y, int fp8_fmt, const float* scale_dev,
                       float scale_host, int scale_mode, int64_t outer, int64_t mid, int64_t inner,
                       float* amax_out, void* stream) {
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (!scale_args_ok(scale_dev, scale_mode, outer, mid, inner)) return MI355Q_ERR_INVALID_ARGUMENT;
  const int64_t n = outer * mid * inner;
  if (n > 0 && (x == nullptr || y == nullptr)) return MI355Q_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);

  if (x_dtype == MI355Q_E4M3FN || x_dtype == MI355Q_E5M2) {
    // fp8 in, same fp8 out: identity copy, no amax (fp8_ops.cpp:201-215)
    if (x_dtype != fp8_fmt || amax_out != nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
    if (n == 0) return MI355Q_OK;
    int64_t done = 0;
    if (aligned(x, 16) && aligned(y, 16) && n >= 16) {
      const int64_t nvec = n / 16;
      if ((nvec + kThreads * kCopyU - 1) / (kThreads * kCopyU) > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
      copy_vec16_kernel<<<blocks_for(nvec, kThreads * kCopyU), kThreads, 0, st>>>(xb, yb, nvec);
      done = nvec * 16;
    }
    if (done < n)
      copy_bytes_kernel<<<blocks_for(n - done, kThreads), kThreads, 0, st>>>(xb + done, yb + done, n - done);
    return launch_status();
  }
  if (x_dtype != MI355Q_F32 && x_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;

  uint32_t* am = reinterpret_cast<uint32_t*>(amax_out);
  if (am) fill_u32_kernel<<<1, 1, 0, st>>>(am, 0u);
  if (n == 0) return launch_status();
  if (x_dtype == MI355Q_BF16) {
    if (fp8_fmt == MI355Q_E4M3FN) return cast_to_dispatch<true, MI355Q_E4M3FN>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, am, st);
    return cast_to_dispatch<true, MI355Q_E5M2>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, am, st);
  }
  if (fp8_fmt == MI355Q_E4M3FN) return cast_to_dispatch<false, MI355Q_E4M3FN>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, am, st);
  return cast_to_dispatch<false, MI355Q_E5M2>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, am, st);
}

int mi355q_cast_from_fp8(const void* x, int fp8_fmt, void* y, int out_dtype, const float* scale_dev,
                         float scale_host, int scale_mode, int64_t outer, int64_t mid,
                         int64_t inner, void* stream) {
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype != MI355Q_F32 && out_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (!scale_args_ok(scale_dev, scale_mode, outer, mid, inner)) return MI355Q_ERR_INVALID_ARGUMENT;
  const int64_t n = outer * mid * inner;
  if (n == 0) return MI355Q_OK;
  if (x == nullptr || y == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  if (fp8_fmt == MI355Q_E4M3FN) {
    if (out_dtype == MI355Q_BF16) return cast_from_dispatch<MI355Q_E4M3FN, true>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, st);
    return cast_from_dispatch<MI355Q_E4M3FN, false>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, st);
  }
  if (out_dtype == MI355Q_BF16) return cast_from_dispatch<MI355Q_E5M2, true>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, st);
  return cast_from_dispatch<MI355Q_E5M2, false>(xb, yb, scale_dev, scale_host, scale_mode, outer, mid, inner, st);
}

}  // extern "C"
