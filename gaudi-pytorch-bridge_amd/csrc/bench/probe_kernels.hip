// Measurement aids: what this GPU sustains with nothing in the way.  They are built into a library
// of their own (libmi355q_probe.so), which only `bench.py --only ceilings` loads: the product library
// and its header export none of this.  Timed in the same run as the kernels they bound, they let a
// roofline fraction be read against the machine's real ceiling (clocks under load, HBM rate at a given
// size) as well as against the published peak.
//
//   mi355q_probe_mfma        `workgroups` workgroups of 4 * waves_per_simd waves (1 or 2 per SIMD), each wave
//                            issuing mfma_per_wave back-to-back v_mfma_f32_32x32x64_f8f6f4 (131072 flop each)
//                            on register operands: the fp8 MFMA rate at the clock the GPU holds under load
//   mi355q_probe_read        reads `bytes` bytes (a multiple of 16, 16-byte aligned) with 16-byte loads and
//                            stores nothing: the HBM read rate at that size
//   mi355q_probe_strip_read  reads a row-major byte matrix [rows, pitch] the way the decode-shaped GEMMs read
//                            their weights: pitch / strip_bytes strips (64, 128 or 256 bytes of every row), the
//                            rows of a strip cut into `parts` ranges, one workgroup per strip and range
//   mi355q_probe_coexec      how much of the MFMA time hides under vector work: per pass a wave issues four
//                            MFMAs (mode bit 0), 32 x (v_exp_f32, v_mul_f32) in eight chains (bit 1), or both
//                            dealt out in turns (3); the first wave of each SIMD takes mode_first, the second
//                            mode_second
//   mi355q_probe_amax_ticket the amax pass of mi355q_amax (bf16 input, the same loads and the same 256 workgroups of
//                            1024 threads) without the launch that zeroes the result word: every workgroup stores
//                            its maximum into a scratch array and draws a ticket, and the one that draws the last
//                            ticket reduces the 256 values, writes the result and returns the ticket counter to
//                            zero.  The form the product does not use: it is timed beside mi355q_amax so that the
//                            comparison can be repeated
//   mi355q_probe_sum_columns_ticket  the column sum of mi355q_sum_fp8 (e4m3fn [R, C] over the rows, fp32 result; the same
//                            loads, slices of 128 rows, 16 columns per lane) as one kernel: every slice stores its
//                            partial sums and draws a ticket of its column block, and the workgroup that draws the
//                            last one adds the slices in their order.  The product uses two kernels instead.
// sink: a few bytes of device memory that are practically never written.
#include "../device_common.h"

namespace mi355q {

typedef int probe_i32x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));

// Back-to-back v_mfma_f32_32x32x64_f8f6f4 (e4m3 x e4m3) on register operands: no loads, no LDS.
// Two accumulators, so no MFMA waits for the one before it.
__global__ __launch_bounds__(512) void probe_mfma_kernel(int pairs, float* sink) {
  probe_i32x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (int)(threadIdx.x * 0x01010101u + i * 0x11u) & 0x37373737;   // small finite e4m3 codes
    b[i] = (int)(threadIdx.x * 0x03030303u + i * 0x07u) & 0x37373737;
  }
  probe_f32x16 c0, c1;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    c0[r] = 0.0f;
    c1[r] = 0.0f;
  }
  for (int it = 0; it < pairs; ++it) {
    c0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c0, 0, 0, 0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c1, 0, 0, 0, 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) s += c0[r] + c1[r];
  if (s == 123.456f) sink[0] = s;   // keeps the loop alive; practically never true
}

// MFMAs and vector instructions side by side, on register operands.  Per pass a wave issues four MFMAs (four
// accumulators), 32 x (v_exp_f32, v_mul_f32) in eight independent chains, or both dealt out in turns (an MFMA, then
// eight of the pairs), as its mode says: bit 0 the MFMAs, bit 1 the vector work.  Waves 0-3 of a workgroup (the
// first wave of each SIMD) take mode_first, waves 4-7 (the second) mode_second.
__global__ __launch_bounds__(512) void probe_coexec_kernel(int passes, int mode_first, int mode_second, float* sink) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int mode = wave >= 4 ? mode_second : mode_first;
  probe_i32x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (int)(threadIdx.x * 0x01010101u + i * 0x11u) & 0x37373737;
    b[i] = (int)(threadIdx.x * 0x03030303u + i * 0x07u) & 0x37373737;
  }
  probe_f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
  float x[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = 0.001f * (float)(threadIdx.x + i);
  if (mode == 3) {
    for (int it = 0; it < passes; ++it) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[j], 0, 0, 0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = __builtin_amdgcn_exp2f(x[i]) * 0.5f;
      }
    }
  } else if (mode == 1) {
    for (int it = 0; it < passes; ++it) {
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[j], 0, 0, 0, 0, 0, 0);
    }
  } else if (mode == 2) {
    for (int it = 0; it < passes; ++it) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = __builtin_amdgcn_exp2f(x[i]) * 0.5f;
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[j][r];
#pragma unroll
  for (int i = 0; i < 8; ++i) s += x[i];
  if (s == 123.456f) sink[0] = s;   // keeps the loops alive; practically never true
}

// 16 bytes per lane, read only: the sum keeps the loads alive, one store per workgroup at most.
__global__ __launch_bounds__(1024) void probe_read_kernel(const u32x4* __restrict__ x, int64_t n16, uint32_t* sink) {
  uint32_t acc = 0;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const u32x4 v0 = x[i], v1 = x[i + stride], v2 = x[i + 2 * stride], v3 = x[i + 3 * stride];
    acc ^= v0[0] ^ v0[1] ^ v0[2] ^ v0[3] ^ v1[0] ^ v1[1] ^ v1[2] ^ v1[3] ^ v2[0] ^ v2[1] ^ v2[2] ^ v2[3] ^ v3[0] ^ v3[1] ^ v3[2] ^ v3[3];
  }
  for (; i < n16; i += stride) {
    const u32x4 v = x[i];
    acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

// A row-major byte matrix read the way the decode-shaped GEMMs read their weights: a workgroup takes a strip of
// R bytes of every row (of its part of the rows), 16 bytes per lane, 8 loads in flight per lane, nothing else.
// NT: with the nontemporal hint.
template <int R, bool NT>
__global__ __launch_bounds__(256) void probe_strip_read_kernel(const uint8_t* base, int64_t pitch, int rows, int parts, uint32_t* sink) {
  const int strip = blockIdx.x / parts, part = blockIdx.x % parts;
  const int r0 = (int)((int64_t)rows * part / parts), r1 = (int)((int64_t)rows * (part + 1) / parts);
  constexpr int kLanesPerRow = R / 16, kRowsPerLoad = 256 / kLanesPerRow, kLoads = 8;
  const int lr = threadIdx.x / kLanesPerRow, lc = threadIdx.x % kLanesPerRow;
  const uint8_t* p = base + (int64_t)strip * R + lc * 16 + (int64_t)(r0 + lr) * pitch;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (int r = r0; r + kLoads * kRowsPerLoad <= r1; r += kLoads * kRowsPerLoad) {
    u32x4 v[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const u32x4* q = reinterpret_cast<const u32x4*>(p + (int64_t)i * kRowsPerLoad * pitch);
      v[i] = NT ? __builtin_nontemporal_load(q) : *q;
    }
#pragma unroll
    for (int i = 0; i < kLoads; ++i) acc ^= v[i];
    p += (int64_t)kLoads * kRowsPerLoad * pitch;
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = acc[0];
}

}  // namespace mi355q

using namespace mi355q;

// ---- amax without the zeroing launch (see the head of the file)
constexpr int kProbeAmaxThreads = 1024, kProbeAmaxBlocks = 256;
static __device__ uint32_t probe_amax_part[kProbeAmaxBlocks];
static __device__ uint32_t probe_amax_ticket;

__global__ __launch_bounds__(kProbeAmaxThreads) void probe_amax_ticket_kernel(const uint8_t* __restrict__ x, int64_t nvec, uint32_t* __restrict__ out) {
  constexpr int U = 4;
  __shared__ uint32_t wave_part[kProbeAmaxThreads / 64];
  __shared__ uint32_t last;
  uint32_t am = 0;
  const int64_t stride = (int64_t)gridDim.x * kProbeAmaxThreads;
  for (int64_t v0 = (int64_t)blockIdx.x * kProbeAmaxThreads + threadIdx.x; v0 < nvec; v0 += stride * U) {
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
        const u16x2 a = __builtin_bit_cast(u16x2, in[u][i] & 0x7fff7fffu);
        am = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, __builtin_bit_cast(u16x2, am)));
      }
    }
  }
  {
    const uint32_t lo = am & 0xffffu, hi = am >> 16;
    am = (lo > hi ? lo : hi) << 16;
  }
  am = wave_max_u32(am);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) wave_part[wave] = am;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t r = wave_part[0];
    for (int w = 1; w < kProbeAmaxThreads / 64; ++w) r = r > wave_part[w] ? r : wave_part[w];
    __hip_atomic_store(&probe_amax_part[blockIdx.x], r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0);  // acknowledged before the ticket is drawn
    const uint32_t t = __hip_atomic_fetch_add(&probe_amax_ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = t == gridDim.x - 1;
    if (last) __hip_atomic_store(&probe_amax_ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!last || wave != 0) return;
  uint32_t r = 0;
  for (int b = lane; b < (int)gridDim.x; b += 64) {
    const uint32_t v = __hip_atomic_load(&probe_amax_part[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    r = r > v ? r : v;
  }
  r = wave_max_u32(r);
  if (lane == 0) *out = r;
}

// ---- column sum with the slices merged by the last arrival (see the head of the file)
constexpr int kProbeSumMaxBlocks = 64, kProbeSumMaxSlices = 128;
static __device__ __align__(256) float probe_sum_part[kProbeSumMaxSlices * kProbeSumMaxBlocks * 1024];  // [slice][column]
static __device__ uint32_t probe_sum_ticket[kProbeSumMaxBlocks];

__global__ __launch_bounds__(256) void probe_sum_columns_ticket_kernel(const uint8_t* __restrict__ x, int64_t R, int64_t C, int64_t per,
                                                                       float* __restrict__ out) {
  constexpr int WAVES = 4, VEC = 16;
  __shared__ float part[WAVES - 1][64][VEC];
  __shared__ uint32_t last;
  const int s = blockIdx.y, splits = gridDim.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t c0 = ((int64_t)blockIdx.x * 64 + lane) * VEC;
  const int64_t r0 = s * per, r1 = (r0 + per) < R ? (r0 + per) : R;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
  auto add = [&](const u32x4& t) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float a, b, c, d;
      cvt_f32x4<MI355Q_E4M3FN>(t[q], a, b, c, d);
      acc[4 * q] += a; acc[4 * q + 1] += b; acc[4 * q + 2] += c; acc[4 * q + 3] += d;
    }
  };
  {
    const uint8_t* p = x + (r0 + wave) * C + c0;
    const int64_t step = (int64_t)WAVES * C;
    int64_t r = r0 + wave;
    for (; r + 3 * WAVES < r1; r += 4 * WAVES) {
      u32x4 w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) w[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + u * step));
#pragma unroll
      for (int u = 0; u < 4; ++u) add(w[u]);
      p += 4 * step;
    }
    for (; r < r1; r += WAVES, p += step) add(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[wave - 1][lane][e] = acc[e];
  }
  __syncthreads();
  const int64_t ncol = (int64_t)gridDim.x * 1024;
  if (wave == 0) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float v = acc[e];
#pragma unroll
      for (int w = 0; w < WAVES - 1; ++w) v += part[w][lane][e];
      __hip_atomic_store(&probe_sum_part[(int64_t)s * ncol + c0 + e], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_waitcnt(0);  // acknowledged before the ticket is drawn
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t t = __hip_atomic_fetch_add(&probe_sum_ticket[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = t == (uint32_t)splits - 1;
    if (last) __hip_atomic_store(&probe_sum_ticket[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!last) return;
  // 1024 columns, four per thread, the slices in their order
  const int64_t c = (int64_t)blockIdx.x * 1024 + threadIdx.x * 4;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  for (int t = 0; t < splits; t += 4) {
    float w[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        w[u][e] = t + u < splits ? __hip_atomic_load(&probe_sum_part[(int64_t)(t + u) * ncol + c + e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += w[u][e];
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) out[c + e] = v[e];
}

extern "C" {

// x: e4m3fn [R, C] row-major, 16-byte aligned, C a multiple of 1024 and at most 65536, at most 128 slices of 128 rows;
// out: C floats.  One call at a time per GPU (the scratch is shared).
int mi355q_probe_sum_columns_ticket(const void* x, int64_t R, int64_t C, float* out, void* stream) {
  const int64_t per = 128, splits = (R + per - 1) / per;
  if (x == nullptr || out == nullptr || R <= 0 || C <= 0 || C % 1024 != 0 || C / 1024 > kProbeSumMaxBlocks || splits > kProbeSumMaxSlices ||
      splits * C > (int64_t)kProbeSumMaxSlices * kProbeSumMaxBlocks * 1024 || reinterpret_cast<uintptr_t>(x) % 16 != 0)
    return MI355Q_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(probe_sum_columns_ticket_kernel, dim3((unsigned)(C / 1024), (unsigned)splits), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint8_t*>(x), R, C, per, out);
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

// x: bf16, 16-byte aligned, n a multiple of 8; out: one float (the bit pattern of the maximum of |x|).  One call at a
// time per GPU (the scratch is shared).
int mi355q_probe_amax_ticket(const void* x, int64_t n, float* out, void* stream) {
  if (x == nullptr || out == nullptr || n <= 0 || n % 8 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0) return MI355Q_ERR_INVALID_ARGUMENT;
  const int64_t nvec = n / 8;
  int64_t grid = (nvec + kProbeAmaxThreads * 4 - 1) / (kProbeAmaxThreads * 4);
  if (grid > kProbeAmaxBlocks) grid = kProbeAmaxBlocks;
  hipLaunchKernelGGL(probe_amax_ticket_kernel, dim3((unsigned)grid), dim3(kProbeAmaxThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint8_t*>(x), nvec, reinterpret_cast<uint32_t*>(out));
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

int mi355q_probe_mfma(int waves_per_simd, int mfma_per_wave, int workgroups, float* sink, void* stream) {
  if ((waves_per_simd != 1 && waves_per_simd != 2) || mfma_per_wave < 2 || workgroups <= 0 || sink == nullptr)
    return MI355Q_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3((unsigned)workgroups), dim3(256u * waves_per_simd), 0, static_cast<hipStream_t>(stream),
                     mfma_per_wave / 2, sink);
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

int mi355q_probe_coexec(int waves_per_simd, int passes, int mode_first, int mode_second, int workgroups, float* sink, void* stream) {
  if ((waves_per_simd != 1 && waves_per_simd != 2) || passes <= 0 || workgroups <= 0 || sink == nullptr || mode_first < 0 ||
      mode_first > 3 || mode_second < 0 || mode_second > 3)
    return MI355Q_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(probe_coexec_kernel, dim3((unsigned)workgroups), dim3(256u * waves_per_simd), 0, static_cast<hipStream_t>(stream),
                     passes, mode_first, mode_second, sink);
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

int mi355q_probe_read(const void* x, int64_t bytes, int workgroups, void* sink, void* stream) {
  if (x == nullptr || sink == nullptr || bytes < 0 || workgroups <= 0 || (reinterpret_cast<uintptr_t>(x) & 15u) != 0)
    return MI355Q_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)workgroups), dim3(1024), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4*>(x), bytes / 16, static_cast<uint32_t*>(sink));
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

int mi355q_probe_strip_read(const void* x, int64_t pitch, int64_t rows, int strip_bytes, int parts, int nontemporal, void* sink,
                            void* stream) {
  if (x == nullptr || sink == nullptr || pitch <= 0 || rows <= 0 || parts <= 0 || rows > 0x7fffffffLL ||
      (reinterpret_cast<uintptr_t>(x) & 15u) != 0 || (strip_bytes != 64 && strip_bytes != 128 && strip_bytes != 256) ||
      pitch % strip_bytes != 0 || pitch / strip_bytes * parts > 0x7fffffffLL)
    return MI355Q_ERR_INVALID_ARGUMENT;
  const dim3 grid((unsigned)(pitch / strip_bytes * parts)), block(256);
  const uint8_t* p = static_cast<const uint8_t*>(x);
  uint32_t* s = static_cast<uint32_t*>(sink);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int r = (int)rows;
  if (strip_bytes == 64) {
    if (nontemporal) hipLaunchKernelGGL((probe_strip_read_kernel<64, true>), grid, block, 0, st, p, pitch, r, parts, s);
    else hipLaunchKernelGGL((probe_strip_read_kernel<64, false>), grid, block, 0, st, p, pitch, r, parts, s);
  } else if (strip_bytes == 128) {
    if (nontemporal) hipLaunchKernelGGL((probe_strip_read_kernel<128, true>), grid, block, 0, st, p, pitch, r, parts, s);
    else hipLaunchKernelGGL((probe_strip_read_kernel<128, false>), grid, block, 0, st, p, pitch, r, parts, s);
  } else {
    if (nontemporal) hipLaunchKernelGGL((probe_strip_read_kernel<256, true>), grid, block, 0, st, p, pitch, r, parts, s);
    else hipLaunchKernelGGL((probe_strip_read_kernel<256, false>), grid, block, 0, st, p, pitch, r, parts, s);
  }
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

}  // extern "C"
