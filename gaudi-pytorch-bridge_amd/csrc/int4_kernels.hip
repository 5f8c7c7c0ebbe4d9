// Packed-nibble dequantisation (convert_from_int4 / convert_from_uint4) for gfx950.
//
// HBM-bound and write-dominated: one packed int32 (8 nibbles) becomes 8 output
// elements.  A lane owns one packed column and walks down RPT rows, so a
// wave's stores are 64 x 16 B contiguous (bf16) per row, and the group's scale
// and zero-point vectors stay in registers while the rows of a group stream by.
#include "device_common.h"

namespace mi355q {

constexpr int kI4Threads = 256;

template <bool SIGNED>
__device__ __forceinline__ int nib(uint32_t w, int i) {
  if constexpr (SIGNED) return __builtin_amdgcn_sbfe((int)w, 4 * i, 4);
  else return (int)__builtin_amdgcn_ubfe(w, 4 * i, 4);
}

// E consecutive scale / float zero-point values, converted to fp32 (E = 8 bf16 or 4 fp32: 16 bytes)
template <bool BF16>
__device__ __forceinline__ void load_vals(const uint8_t* base, int64_t elem, float* out) {
  if constexpr (BF16) {
    const u32x4 w = *reinterpret_cast<const u32x4*>(base + elem * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = __uint_as_float(w[i] << 16);
      out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  } else {
    const f32x4 a = *reinterpret_cast<const f32x4*>(base + elem * 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = a[i];
  }
}

// ZP: 0 none, 1 float, 2 packed.  RPT rows per thread; a thread's rows never
// straddle a group when HOIST (group % RPT == 0), so scale / zp load once.
// A lane produces one 16-byte store per row: all 8 nibbles of a packed word for
// bf16 output, one half of the word (4 nibbles) for fp32 output, so that a
// wave's store covers whole cache lines in both cases.
template <bool SIGNED, bool BF16, int ZP, int RPT, bool HOIST>
__global__ __launch_bounds__(kI4Threads) void dequant_4bit_kernel(
    const uint32_t* __restrict__ packed, const uint8_t* __restrict__ scale,
    const uint8_t* __restrict__ zp, int64_t rows, int64_t pcols, int64_t group,
    uint8_t* __restrict__ out) {
  constexpr int E = BF16 ? 8 : 4;            // elements per lane per row
  constexpr int LPW = 8 / E;                 // lanes per packed word
  const int64_t lanes_per_row = pcols * LPW;
  const int64_t g = (int64_t)blockIdx.x * kI4Threads + threadIdx.x;
  const int64_t chunk = g / lanes_per_row;
  const int64_t lc = g - chunk * lanes_per_row;
  const int64_t pc = lc / LPW;
  const int nib0 = (int)(lc % LPW) * E;      // first nibble of this lane inside the word
  const int64_t r0 = chunk * RPT;
  if (r0 >= rows) return;
  const int64_t cols = pcols * 8;
  const int64_t c0 = pc * 8 + nib0;          // first output column of this lane
  const int nr = (int)((rows - r0) < RPT ? (rows - r0) : RPT);

  uint32_t w[RPT];
#pragma unroll
  for (int j = 0; j < RPT; ++j)
    if (j < nr) w[j] = __builtin_nontemporal_load(packed + (r0 + j) * pcols + pc);

  float s[E], zf[E];
  int zi[E];
  int64_t cur = -1;
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    if (j >= nr) continue;
    const int64_t r = r0 + j;
    const int64_t gi = HOIST ? r0 / group : r / group;
    if ((HOIST && j == 0) || (!HOIST && gi != cur)) {
      cur = gi;
      load_vals<BF16>(scale, gi * cols + c0, s);
      if constexpr (ZP == 1) load_vals<BF16>(zp, gi * cols + c0, zf);
      if constexpr (ZP == 2) {
        const uint32_t zw = reinterpret_cast<const uint32_t*>(zp)[gi * pcols + pc] >> (4 * nib0);
#pragma unroll
        for (int i = 0; i < E; ++i) zi[i] = nib<SIGNED>(zw, i);
      }
    }
    const uint32_t wj = w[j] >> (4 * nib0);
    float v[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
      const int q = nib<SIGNED>(wj, i);
      float d;
      if constexpr (ZP == 2) d = (float)(q - zi[i]);
      else if constexpr (ZP == 1) {
        d = (float)q - zf[i];
        if constexpr (BF16) d = round_to_bf16(d);  // subtraction happens in the output dtype
      } else d = (float)q;
      v[i] = d * s[i];
    }
    if constexpr (BF16) {
      u32x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
      __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(out + (r * cols + c0) * 2));
    } else {
      const f32x4 o = {v[0], v[1], v[2], v[3]};
      __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(out + (r * cols + c0) * 4));
    }
  }
}

template <bool SIGNED, bool BF16, int ZP>
int dequant_launch(const uint32_t* packed, const uint8_t* scale, const uint8_t* zp, int64_t rows,
                   int64_t pcols, int64_t group, uint8_t* out, hipStream_t st) {
  const int64_t lanes_per_row = pcols * (BF16 ? 1 : 2);
  auto grid_for = [&](int rpt) { return ((rows + rpt - 1) / rpt * lanes_per_row + kI4Threads - 1) / kI4Threads; };
  // 8 rows per thread measured best (K = N = 4096: 4 rows 9.0 us, 8 rows 7.3, 16 rows 7.7, 32 rows 7.9)
  if (group % 8 == 0) {
    const int64_t grid = grid_for(8);
    if (grid > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    dequant_4bit_kernel<SIGNED, BF16, ZP, 8, true><<<(unsigned)grid, kI4Threads, 0, st>>>(packed, scale, zp, rows, pcols, group, out);
  } else if (group == 1) {
    const int64_t grid = grid_for(1);
    if (grid > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    dequant_4bit_kernel<SIGNED, BF16, ZP, 1, true><<<(unsigned)grid, kI4Threads, 0, st>>>(packed, scale, zp, rows, pcols, group, out);
  } else {
    const int64_t grid = grid_for(4);
    if (grid > 0x7fffffffLL) return MI355Q_ERR_UNSUPPORTED;
    dequant_4bit_kernel<SIGNED, BF16, ZP, 4, false><<<(unsigned)grid, kI4Threads, 0, st>>>(packed, scale, zp, rows, pcols, group, out);
  }
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

template <bool SIGNED, bool BF16>
int dequant_zp(int zp_kind, const uint32_t* packed, const uint8_t* scale, const uint8_t* zp,
               int64_t rows, int64_t pcols, int64_t group, uint8_t* out, hipStream_t st) {
  switch (zp_kind) {
    case MI355Q_ZP_NONE: return dequant_launch<SIGNED, BF16, 0>(packed, scale, zp, rows, pcols, group, out, st);
    case MI355Q_ZP_FLOAT: return dequant_launch<SIGNED, BF16, 1>(packed, scale, zp, rows, pcols, group, out, st);
    default: return dequant_launch<SIGNED, BF16, 2>(packed, scale, zp, rows, pcols, group, out, st);
  }
}

}  // namespace mi355q

using namespace mi355q;

extern "C" int mi355q_dequant_4bit(const int32_t* packed, const void* scale, const void* zp,
                                   int zp_kind, int is_signed, int out_dtype, int64_t rows,
                                   int64_t packed_cols, int64_t group, void* out, void* stream) {
  if (rows < 0 || packed_cols < 0 || group <= 0) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype != MI355Q_F32 && out_dtype != MI355Q_BF16) return MI355Q_ERR_INVALID_ARGUMENT;
  if (zp_kind < MI355Q_ZP_NONE || zp_kind > MI355Q_ZP_PACKED) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows == 0 || packed_cols == 0) return MI355Q_OK;
  if (packed == nullptr || scale == nullptr || out == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (zp_kind != MI355Q_ZP_NONE && zp == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (rows % group != 0) return MI355Q_ERR_INVALID_ARGUMENT;
  // 16-byte vectors for scale, float zero-point and output
  auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (!al(scale) || !al(out) || (zp_kind == MI355Q_ZP_FLOAT && !al(zp)) ||
      (reinterpret_cast<uintptr_t>(packed) & 3u) != 0)
    return MI355Q_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t* pk = reinterpret_cast<const uint32_t*>(packed);
  const uint8_t* sc = static_cast<const uint8_t*>(scale);
  const uint8_t* z = static_cast<const uint8_t*>(zp);
  uint8_t* o = static_cast<uint8_t*>(out);
  if (is_signed) {
    if (out_dtype == MI355Q_BF16) return dequant_zp<true, true>(zp_kind, pk, sc, z, rows, packed_cols, group, o, st);
    return dequant_zp<true, false>(zp_kind, pk, sc, z, rows, packed_cols, group, o, st);
  }
  if (out_dtype == MI355Q_BF16) return dequant_zp<false, true>(zp_kind, pk, sc, z, rows, packed_cols, group, o, st);
  return dequant_zp<false, false>(zp_kind, pk, sc, z, rows, packed_cols, group, o, st);
}
