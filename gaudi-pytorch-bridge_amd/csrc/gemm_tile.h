// fp8 x fp8 -> fp32-accumulate -> bf16/fp32 GEMM for gfx950 (fp8_gemm_v2).
//
// Tiled kernel: a 512-thread workgroup (8 waves, 2 x 4, two per SIMD) owns a BM x BN tile of C
// and walks K in steps of 128 bytes.  Operand tiles travel from global memory
// straight into LDS (buffer_load_dwordx4 ... lds: no staging registers, and the
// buffer descriptor's bounds check zero-fills rows past the matrix edge) into
// one of two LDS stages, so the loads of step k+2 fly while step k computes.
// Inside a stage, the 16-byte chunks of a row are XOR-swizzled with the row
// number, which keeps the 128-bit and transposing fragment reads free of bank
// conflicts; since a DMA load places lane l's chunk at LDS offset 16 l, the
// swizzle is applied by choosing which global chunk each lane fetches.  Each
// wave computes its (BM/2) x (BN/4) sub-tile with v_mfma_f32_32x32x64_f8f6f4
// (fp8/bf8 operands, 64 k per instruction), reading the fragments of the next
// half-step while the MFMAs of the current one run.  The buffer descriptors
// walk along K by scalar arithmetic, so the per-lane offsets are small
// constants and operands of any size are addressable.
//
// Operand layouts.  An operand whose K index is contiguous in memory (A with
// trans_a == 0, B with trans_b != 0) is "K-major": a lane's 32-byte MFMA
// fragment is two ds_read_b128.  The other layout (A with trans_a != 0, the
// usual B [K, N] with trans_b == 0) is "MN-major": rows of LDS hold 16 byte
// runs along m or n, and ds_read_b64_tr_b8 transposes 8 k-rows x 16 columns
// inside each group of 16 lanes on the way into registers.
//
// The MFMA is issued with the B fragment as its first operand, so that a lane
// ends up holding runs of 4 consecutive n for one m.  Per-row / per-column
// scales, bias and the accumulate input are applied in fp32 before the single
// final rounding, and the rows pass through LDS once more so that a wave
// stores whole 128-byte lines.
#pragma once
#include <type_traits>

#include "device_common.h"

namespace mi355q {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define LDS_AS __attribute__((address_space(3)))

// Two waves per SIMD: a memory instruction of one wave (LDS fragment read,
// global->LDS load) holds up that wave's next MFMA for tens of cycles, and only
// a second resident wave lets the matrix pipe run meanwhile.
constexpr int kGemmThreads = 512;
constexpr int kWaves = kGemmThreads / 64;
constexpr int kWavesM = 2, kWavesN = 4;  // wave grid over the tile
constexpr int kBK = 128;  // bytes (= fp8 elements) of K per LDS stage

// Number of compute units of the current device (workgroups of the persistent kernel).
inline int compute_units() {
  static const int n = [] {
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0)
      cu = 256;
    return cu;
  }();
  return n;
}

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
//
// Swizzle.  The LDS of gfx950 has 64 banks of 4 bytes: a ds_read_b128 serves 16
// lanes per cycle, a ds_read_b64(_tr_b8) 32 lanes, and a cycle is conflict free
// when those lanes touch 16 distinct 16-byte slots modulo 256 bytes.
//   K-major, 128-byte rows: the 16 lanes of a cycle read one chunk column of 16
//     consecutive rows; rows r and r+2 share a bank slot, so the chunk index is
//     XORed with (row >> 1) & 7.
//   MN-major, 256-byte rows: a cycle covers two 16-lane groups, i.e. 8 k-rows
//     times two adjacent chunks; XORing with (row & 7) << 1 sends the 8 rows to
//     8 slots of one parity and leaves the other parity to the adjacent chunk.
//   MN-major, 128-byte rows: two rows per 256 bytes, so (row >> 1 & 3) << 1.
//   K-major, 64-byte rows: four rows per 256 bytes, so (row >> 2) & 3.
template <bool KMAJOR, int ROWS, int ROW_BYTES>
struct TileGeom {
  static constexpr int kChunksPerRow = ROW_BYTES / 16;
  static constexpr int kChunks = ROWS * kChunksPerRow;
  static_assert(KMAJOR ? (ROW_BYTES == 128 || ROW_BYTES == 64) : (ROW_BYTES == 256 || ROW_BYTES == 128), "no swizzle defined");
  __device__ static __forceinline__ int swizzle(int row) {
    if constexpr (KMAJOR && ROW_BYTES == 128) return (row >> 1) & 7;
    else if constexpr (KMAJOR) return (row >> 2) & 3;
    else if constexpr (ROW_BYTES == 256) return (row & 7) << 1;
    else return ((row >> 1) & 3) << 1;
  }
  __device__ static __forceinline__ int lds_offset(int row, int chunk) {
    return row * ROW_BYTES + ((chunk ^ swizzle(row)) << 4);
  }
};

template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// Global -> LDS loader for one operand tile, one 16-byte chunk per lane per
// instruction.  A wave-wide load fills a 1 KiB region of the LDS tile (lane l
// lands at byte 16 l of the region), i.e. 64 / chunks-per-row consecutive rows;
// the waves split the regions of a tile evenly.
//   KMAJOR: rows index m/n, chunks walk k.  Rows past the matrix end fall
//           outside the buffer descriptor and read as zero; chunks at or beyond
//           K are redirected outside it.
//   else  : rows index k, chunks walk m/n.  Rows at or beyond K fall outside the
//           descriptor; columns past the extent only feed outputs that are
//           never stored.
// EXT: tile extent along m/n; BK: bytes of K per stage; WAVES: waves of the workgroup
template <bool KMAJOR, int EXT, int BK = kBK, int WAVES = kWaves>
struct DmaLoader {
  using G = TileGeom<KMAJOR, KMAJOR ? EXT : BK, KMAJOR ? BK : EXT>;
  static constexpr int kCPR = G::kChunksPerRow;
  static constexpr int kRowsPerRegion = 64 / kCPR;
  static constexpr int kRegions = G::kChunks / 64;
  static constexpr int kPerWave = kRegions / WAVES;
  static_assert(kRegions % WAVES == 0 && 64 % kCPR == 0, "tile does not split over the waves");

  // Raw buffer descriptor: base, stride 0, num_records (bytes), dword 3 flags.
  // The base walks along K, one stage per advance(), and num_records shrinks
  // with it, so the per-lane offsets never change and stay below 2^31 whatever
  // the size of the matrix (a stage spans at most 256 rows of ld bytes).
  i32x4 rsrc;
  int64_t remaining;  // bytes from the base to the end of the addressable part of the matrix
  int64_t step;       // bytes between K stages
  int voff[kPerWave]; // this lane's offsets inside a stage
  int kc[kPerWave];   // K-major: byte offset of this lane's chunk inside a stage row
  int wave;

  static constexpr int64_t kMaxRecords = 0x80000000LL;  // keeps the out-of-range marker out of range

  // Per-lane geometry; depends on the leading dimension only.  The lane number
  // goes through an empty volatile asm so that these few integer operations
  // stay where they are written: hoisted out of the tile loop, the results
  // would have to live through the epilogue, where every register is taken,
  // and be spilled (a spill there is a store to memory by every lane).
  // wave_index: this wave's position among the WAVES waves that share the
  // loads of this operand (default: its position in the workgroup).
  __device__ __forceinline__ void set_lane_offsets(int64_t ld, int wave_index = -1) {
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));
    wave = wave_index >= 0 ? wave_index : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rin = lane / kCPR, p = lane % kCPR;
#pragma unroll
    for (int i = 0; i < kPerWave; ++i) {
      const int row = (wave * kPerWave + i) * kRowsPerRegion + rin;
      const int c = p ^ G::swizzle(row);
      voff[i] = row * (int)ld + c * 16;
      kc[i] = c * 16;
    }
  }

  __device__ __forceinline__ void set_records() {
    const int64_t r = remaining < 0 ? 0 : (remaining > kMaxRecords ? kMaxRecords : remaining);
    rsrc[2] = __builtin_amdgcn_readfirstlane((int)(uint32_t)r);
  }

  // Points the descriptor at stage 0 of a tile.  base: first element of this
  // batch's matrix; mn0: first row (K-major) or column (MN-major) of the tile;
  // extent: matrix extent along m/n; valid false makes every load fall outside.
  __device__ __forceinline__ void set_tile(const uint8_t* base, int64_t ld, int mn0, int extent, int K, bool valid = true) {
    if constexpr (KMAJOR) {
      base += (int64_t)mn0 * ld;
      remaining = (int64_t)(extent - mn0 - 1) * ld + K;
      step = BK;
    } else {
      base += mn0;
      remaining = (int64_t)(K - 1) * ld + (extent - mn0);
      step = (int64_t)BK * ld;
    }
    if (!valid) remaining = 0;
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    rsrc[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    rsrc[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((b >> 32) & 0xffffu));
    rsrc[3] = 0x00020000;
    set_records();
  }

  __device__ __forceinline__ void init(const uint8_t* base, int64_t ld, int mn0, int extent, int K) {
    set_lane_offsets(ld);
    set_tile(base, ld, mn0, extent, K);
  }

  // Issues load I of this wave's share of the stage the descriptor points at,
  // which starts at k0.
  template <int I>
  __device__ __forceinline__ void issue_one(uint8_t* lds_tile, int k0, int K) const {
    const uint32_t lds_base = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)lds_tile;
    {
      constexpr int i = I;
      int vo = voff[i];
      if constexpr (KMAJOR) vo = (k0 + kc[i] < K) ? vo : 0x7fffffff;
      const uint32_t dst = lds_base + (uint32_t)((wave * kPerWave + i) * 1024);
      // m0 holds the LDS address of the region; lane l's 16 bytes land at m0 + 16 l.
      // Written as asm so that the compiler, which would otherwise make every later
      // LDS read wait for all outstanding global->LDS loads, leaves the waiting to
      // the explicit vmcnt drain before each barrier.
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                   :
                   : "s"(dst), "v"(vo), "s"(rsrc)
                   : "memory", "m0");
    }
  }

  __device__ __forceinline__ void issue(uint8_t* lds_tile, int k0, int K) const {
    static_for<kPerWave>([&](auto ic) { issue_one<decltype(ic)::value>(lds_tile, k0, K); });
  }

  // Points the descriptor at K stage `stage` of the tile set_tile() chose, which
  // has to be the most recent call (it leaves the descriptor at stage 0 and
  // this walks from wherever advance() has taken it).  Stages at or beyond K
  // are entirely out of range.
  __device__ __forceinline__ void seek(int from_stage, int to_stage) {
    const int64_t d = (int64_t)(to_stage - from_stage) * step;
    uint64_t b = ((uint64_t)(uint32_t)rsrc[1] << 32) | (uint32_t)rsrc[0];
    b += (uint64_t)d;
    rsrc[0] = (int)(uint32_t)b;
    rsrc[1] = (int)(uint32_t)(b >> 32);
    remaining -= d;
    set_records();
  }

  // Next K stage: scalar arithmetic on the descriptor only.
  __device__ __forceinline__ void advance() {
    uint64_t b = ((uint64_t)(uint32_t)rsrc[1] << 32) | (uint32_t)rsrc[0];
    b += (uint64_t)step;
    rsrc[0] = (int)(uint32_t)b;
    rsrc[1] = (int)(uint32_t)(b >> 32);
    remaining -= step;
    set_records();
  }
};

// A 32-byte MFMA fragment (32 rows of m/n x 32 k for this lane's k-half) is
// read from LDS in parts: two ds_read_b128 for a K-major operand, four
// ds_read_b64_tr_b8 for an MN-major one.
template <bool KMAJOR>
constexpr int frag_parts() { return KMAJOR ? 2 : 4; }

template <bool KMAJOR, int EXT, int PART, int BK = kBK>
__device__ __forceinline__ void read_fragment_part(const uint8_t* lds, int mn_base, int ksub, i32x8& f) {
  using G = TileGeom<KMAJOR, KMAJOR ? EXT : BK, KMAJOR ? BK : EXT>;
  const int lane = threadIdx.x & 63;
  if constexpr (KMAJOR) {
    const int row = mn_base + (lane & 31);
    const int c = ksub * 4 + (lane >> 5) * 2 + PART;
    const u32x4 v = *reinterpret_cast<const u32x4*>(lds + G::lds_offset(row, c));
    f[4 * PART + 0] = v[0];
    f[4 * PART + 1] = v[1];
    f[4 * PART + 2] = v[2];
    f[4 * PART + 3] = v[3];
  } else {
    // Within each group of 16 lanes, lanes 2r and 2r+1 point at the two 8-byte
    // halves of k-row r; after the transposing read lane i of the group holds
    // column i for those 8 k-rows.
    const int blk = lane >> 4, i = lane & 15;
    const int r = i >> 1, h = i & 1;
    const int col = mn_base + (blk & 1) * 16;  // first column of this 16-lane group
    const int krow = ksub * 64 + (blk >> 1) * 32 + PART * 8 + r;
    const int off = G::lds_offset(krow, col >> 4) + h * 8;
    const i32x2 t = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS_AS i32x2*)((LDS_AS uint8_t*)lds + off));
    f[2 * PART] = t[0];
    f[2 * PART + 1] = t[1];
  }
}

// ------------------------------------------------------------------- epilogue
__device__ __forceinline__ float load_out_as_f32(const uint8_t* p, int64_t idx, int bf16) {
  return bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[idx])
              : reinterpret_cast<const float*>(p)[idx];
}

// v = acc * sA * sB + bias + D in fp32, one rounding to the output type.
//   acc[i][j][e] on this lane is C[m][n] with
//     m = m_wave + 32 i + lane % 32
//     n = n_wave + 32 j + 8 (e / 4) + 4 (lane / 32) + e % 4
// The accumulators pass through a small row-major fp32 staging area in LDS
// (`stage`: kEpiRows rows of the wave's 32 NT columns, rows padded by 16 bytes)
// eight rows at a time: the lanes that own those rows write their 4-column
// pieces, and the data comes back with a lane owning 4 consecutive columns of
// a row, so that a wave-wide store writes whole 128-byte lines.  The
// arithmetic runs in one small runtime loop over the rows, whatever the scale
// / bias / accumulate forms.  Two things keep it cheap: the loop is rolled
// (unrolled over all tiles the epilogue is tens of KiB of straight-line code
// that every wave runs once, and instruction fetch dominates), and its common
// form holds no global load (loads and stores share one counter, vmcnt, so a
// loop that may load makes every pass wait for the previous pass's store).
// The staging area is separate from the operand stages, which at that time
// already receive the first stages of the workgroup's next tile.
constexpr int kEpiRows = 8;

template <int MT, int NT>
constexpr int epilogue_stage_floats() {
  constexpr int general = kEpiRows * (32 * NT + 4) + 2 * 32 * MT;  // fp32 rows + row scales
  constexpr int fast = 32 * NT * 16;                               // 32 rows of 32 NT bf16
  return general > fast ? general : fast;
}

template <int MT, int NT>
__device__ __forceinline__ void epilogue(const GemmArgs& g, int64_t batch, f32x16 (&acc)[MT][NT],
                                         int m_wave, int n_wave, float* stage) {
  constexpr int kRowFloats = 32 * NT + 4;
  constexpr int kLanesPerRow = 8 * NT;           // a lane owns 4 columns
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  int lane = threadIdx.x & 63;
  asm volatile("" : "+v"(lane));  // keeps lane-derived values out of the registers of the K loop
  const int es = g.out_bf16 ? 2 : 4;
  uint8_t* C = g.C + batch * g.stride_c * es;
  const uint8_t* D = g.D ? g.D + batch * g.stride_d * es : nullptr;
  const uint8_t* bias = g.bias ? g.bias + batch * g.stride_bias * es : nullptr;
  float sa_s = 1.0f, sb_s = 1.0f;
  if (g.sa_mode == MI355Q_GS_HOST) sa_s = g.sa_host;
  else if (g.sa_mode == MI355Q_GS_DEV) sa_s = g.sa[0];
  if (g.sb_mode == MI355Q_GS_HOST) sb_s = g.sb_host;
  else if (g.sb_mode == MI355Q_GS_DEV) sb_s = g.sb[0];

  // the 4 columns this lane owns in the read-back layout, and what depends on them only
  const int r_in = lane / kLanesPerRow;
  const int n = n_wave + (lane % kLanesPerRow) * 4;
  float sa_c[4], sb_c[4], bias_c[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int ne = (n + e) < g.N ? (n + e) : g.N - 1;
    sa_c[e] = g.sa_mode == MI355Q_GS_PER_COL ? g.sa[ne] : sa_s;
    sb_c[e] = g.sb_mode == MI355Q_GS_PER_COL ? g.sb[ne] : sb_s;
    bias_c[e] = g.bias_mode == MI355Q_BIAS_ROW_VECTOR ? load_out_as_f32(bias, ne, g.out_bf16) : 0.0f;
  }
  const bool vec_ok = (n + 3 < g.N) && ((g.ldc * es) % (4 * es) == 0) &&
                      ((reinterpret_cast<uintptr_t>(C) + (size_t)n * es) % (4 * es) == 0);

  // Per-row scales of the wave's 32 MT rows go to LDS once, so that the row
  // loop below holds no global load.
  float* row_sa = stage + kEpiRows * kRowFloats;
  float* row_sb = row_sa + 32 * MT;
  const bool row_scales = g.sa_mode == MI355Q_GS_PER_ROW || g.sb_mode == MI355Q_GS_PER_ROW;
  if (row_scales) {
    for (int t = lane; t < 32 * MT; t += 64) {
      const int m = m_wave + t;
      row_sa[t] = (g.sa_mode == MI355Q_GS_PER_ROW && m < g.M) ? g.sa[m] : 1.0f;
      row_sb[t] = (g.sb_mode == MI355Q_GS_PER_ROW && m < g.M) ? g.sb[m] : 1.0f;
    }
  }
  const bool general = g.bias_mode == MI355Q_BIAS_FULL || D != nullptr;

  uint8_t* const c_col = C + (int64_t)n * es;   // this lane's columns in row 0
  const int64_t row_pitch = g.ldc * es;
  auto store_row4 = [&](int m, const float (&v)[4]) {
    uint8_t* const rowp = c_col + m * row_pitch;
    if (g.out_bf16) {
      uint16_t* cp = reinterpret_cast<uint16_t*>(rowp);
      if (vec_ok) {
        u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        __builtin_nontemporal_store(o, reinterpret_cast<u32x2*>(cp));  // streamed: keep the operand panels in L2
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < g.N) cp[e] = (uint16_t)(pack_bf16x2(v[e], v[e]) & 0xffffu);
      }
    } else {
      float* cp = reinterpret_cast<float*>(rowp);
      if (vec_ok) {
        f32x4 o = {v[0], v[1], v[2], v[3]};
        __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(cp));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < g.N) cp[e] = v[e];
      }
    }
  };

  static_for<MT>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
#pragma unroll 1
    for (int sub = 0; sub < 32 / kEpiRows; ++sub) {
      if (((lane & 31) / kEpiRows) == sub) {
        static_for<NT>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          static_for<4>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            const f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            *reinterpret_cast<f32x4*>(stage + (lane & (kEpiRows - 1)) * kRowFloats + 32 * j + 8 * q + 4 * (lane >> 5)) = v;
          });
        });
      }
      const int row0 = 32 * i + kEpiRows * sub;  // first of these rows within the wave tile
      if (!general && !row_scales) {
        // scales and bias depend on the column only: two VALU ops per element
#pragma unroll
        for (int r = r_in; r < kEpiRows; r += kRowsPerPass) {
          const f32x4 a = *reinterpret_cast<const f32x4*>(stage + r * kRowFloats + (lane % kLanesPerRow) * 4);
          const int m = m_wave + row0 + r;
          if (m < g.M && n < g.N) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float t = a[e] * sa_c[e];
              t = t * sb_c[e];
              v[e] = t + bias_c[e];
            }
            store_row4(m, v);
          }
        }
      } else if (!general) {
#pragma unroll
        for (int r = r_in; r < kEpiRows; r += kRowsPerPass) {
          const f32x4 a = *reinterpret_cast<const f32x4*>(stage + r * kRowFloats + (lane % kLanesPerRow) * 4);
          const float ra = row_sa[row0 + r], rb = row_sb[row0 + r];
          const int m = m_wave + row0 + r;
          if (m < g.M && n < g.N) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              // one of (ra, sa_c) is exactly 1, likewise (rb, sb_c): the products are the scales themselves
              float t = a[e] * (ra * sa_c[e]);
              t = t * (rb * sb_c[e]);
              v[e] = t + bias_c[e];
            }
            store_row4(m, v);
          }
        }
      } else {
#pragma unroll 1
        for (int r = r_in; r < kEpiRows; r += kRowsPerPass) {
          const f32x4 a = *reinterpret_cast<const f32x4*>(stage + r * kRowFloats + (lane % kLanesPerRow) * 4);
          const float ra = row_scales ? row_sa[row0 + r] : 1.0f, rb = row_scales ? row_sb[row0 + r] : 1.0f;
          const int m = m_wave + row0 + r;
          if (m < g.M && n < g.N) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int ne = (n + e) < g.N ? (n + e) : g.N - 1;
              float t = a[e] * (ra * sa_c[e]);
              t = t * (rb * sb_c[e]);
              t += bias_c[e];
              if (g.bias_mode == MI355Q_BIAS_FULL) t += load_out_as_f32(bias, (int64_t)m * g.ldbias + ne, g.out_bf16);
              if (D) t += load_out_as_f32(D, (int64_t)m * g.ldd + ne, g.out_bf16);
              v[e] = t;
            }
            store_row4(m, v);
          }
        }
      }
    }
  });
}

// The forms the fast bf16 epilogue serves: bf16 output through 16-byte stores,
// A scale a scalar or one value per row, B scale a scalar or one value per
// column, bias none or a row vector, no accumulate input.
__device__ __forceinline__ bool epilogue_fast_ok(const GemmArgs& g, int64_t batch) {
  if (!g.out_bf16 || g.D != nullptr || g.bias_mode == MI355Q_BIAS_FULL) return false;
  if (g.sa_mode == MI355Q_GS_PER_COL || g.sb_mode == MI355Q_GS_PER_ROW) return false;
  const uintptr_t c = reinterpret_cast<uintptr_t>(g.C) + (size_t)(batch * g.stride_c) * 2;
  return (c & 15u) == 0 && (g.ldc & 7) == 0;
}

// Four fp32 column values starting at column n (clamped reads past N).
__device__ __forceinline__ void load_col4_f32(const float* p, int n, int N, float (&out)[4]) {
  if (n + 3 < N && (reinterpret_cast<uintptr_t>(p + n) & 15u) == 0) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p + n);
    out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3];
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = p[(n + e) < N ? (n + e) : N - 1];
  }
}
__device__ __forceinline__ void load_col4_bf16(const uint16_t* p, int n, int N, float (&out)[4]) {
  if (n + 3 < N && (reinterpret_cast<uintptr_t>(p + n) & 7u) == 0) {
    const u32x2 v = *reinterpret_cast<const u32x2*>(p + n);
    out[0] = __uint_as_float(v[0] << 16); out[1] = __uint_as_float(v[0] & 0xffff0000u);
    out[2] = __uint_as_float(v[1] << 16); out[3] = __uint_as_float(v[1] & 0xffff0000u);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = bf16_bits_to_f32(p[(n + e) < N ? (n + e) : N - 1]);
  }
}

// bf16 epilogue for the common forms.  Scales and bias are applied in the
// accumulator layout (a lane holds one row m and runs of 4 columns), the
// rounded bf16 values of 32 rows pass through a per-wave LDS area of 32 rows x
// (32 NT) bf16, and come back with a lane owning 8 consecutive columns of a
// row: a wave stores whole rows of its tile, 16 bytes per lane.
// LDS layout: 8-byte slots of a row are XORed with f(row) so that the 32 lanes
// of a write cycle (32 rows, one logical slot) and the 16 lanes of a read cycle
// (rows of equal f, consecutive 16-byte chunks) touch distinct banks; an odd f
// swaps the two halves of a 16-byte chunk, undone after the read.
template <int MT, int NT, bool PER_COL>
__device__ __forceinline__ void epilogue_bf16_fast(const GemmArgs& g, int64_t batch, f32x16 (&acc)[MT][NT],
                                                   int m_wave, int n_wave, float* stage_f) {
  constexpr int kRowBytes = 64 * NT;
  constexpr int kSlotMask = 8 * NT - 1;
  constexpr int kFShift = 3 - NT;            // NT == 1: rows r, r+4 share banks; NT == 2: rows r, r+2
  static_assert(NT == 1 || NT == 2, "swizzle defined for 64- and 128-byte rows");
  constexpr int kLanesPerRow = 4 * NT;       // a lane reads back 16 bytes
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  constexpr int kPasses = 32 / kRowsPerPass;
  LDS_AS uint8_t* stage = (LDS_AS uint8_t*)stage_f;
  // The epilogue sits inside the persistent tile loop, and everything below
  // that depends only on the lane number is invariant in that loop: left
  // alone, the compiler computes it all once before the K loop, where no
  // register is free, and spills it to scratch memory.  Routing the lane number through an empty
  // volatile asm keeps those few integer operations here.
  int lane = threadIdx.x & 63;
  asm volatile("" : "+v"(lane));
  const int r = lane & 31, h = lane >> 5;
  uint16_t* C = reinterpret_cast<uint16_t*>(g.C) + batch * g.stride_c;

  float sa_s = 1.0f, sb_s = 1.0f;
  if (g.sa_mode == MI355Q_GS_HOST) sa_s = g.sa_host;
  else if (g.sa_mode == MI355Q_GS_DEV) sa_s = g.sa[0];
  if (g.sb_mode == MI355Q_GS_HOST) sb_s = g.sb_host;
  else if (g.sb_mode == MI355Q_GS_DEV) sb_s = g.sb[0];

  // Per-column values of the columns this lane holds in the accumulator layout.
  // A scalar B scale is folded into the row factor instead, which leaves one
  // fused multiply-add per element.
  constexpr bool per_col = PER_COL;
  float cs[PER_COL ? NT : 1][4][4], cb[NT][4][4];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n_wave + 32 * j + 8 * q + 4 * h;
      if constexpr (per_col) load_col4_f32(g.sb, n, g.N, cs[j][q]);
      if (g.bias_mode == MI355Q_BIAS_ROW_VECTOR)
        load_col4_bf16(reinterpret_cast<const uint16_t*>(g.bias) + batch * g.stride_bias, n, g.N, cb[j][q]);
      else {
#pragma unroll
        for (int e = 0; e < 4; ++e) cb[j][q][e] = 0.0f;
      }
    }
  float ra[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m_wave + 32 * i + r;
    ra[i] = g.sa_mode == MI355Q_GS_PER_ROW ? g.sa[m < g.M ? m : g.M - 1] : sa_s;
    if (!per_col) ra[i] *= sb_s;
  }

  const int f_w = (r >> kFShift) & kSlotMask;
  // read-back coordinates
  const int row_in_pass = lane / kLanesPerRow, chunk = lane % kLanesPerRow;
  const int n_out = n_wave + 8 * chunk;
  const bool full = n_out + 7 < g.N;

  static_for<MT>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4];
        if constexpr (per_col) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(acc[i][j][4 * q + e] * ra[i], cs[j][q][e], cb[j][q][e]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(acc[i][j][4 * q + e], ra[i], cb[j][q][e]);
        }
        const u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        const int slot = (8 * j + 2 * q + h) ^ f_w;
        *reinterpret_cast<LDS_AS u32x2*>(stage + r * kRowBytes + slot * 8) = o;
      }
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int row = p * kRowsPerPass + row_in_pass;
      const int f = (row >> kFShift) & kSlotMask;
      u32x4 o = *reinterpret_cast<LDS_AS u32x4*>(stage + row * kRowBytes + ((chunk ^ (f >> 1)) << 4));
      if (f & 1) o = u32x4{o[2], o[3], o[0], o[1]};
      const int m = m_wave + 32 * i + row;
      if (m < g.M) {
        uint16_t* cp = C + (int64_t)m * g.ldc + n_out;
        if (full) {
          __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(cp));  // streamed: keep the operand panels in L2
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n_out + e < g.N) cp[e] = (uint16_t)(o[e >> 1] >> (16 * (e & 1)));
        }
      }
    }
  });
}

// Per-wave state of the K loop: accumulators, fragments, loaders.
//
// Register budget.  Two waves per SIMD leave 256 registers per lane: 128 hold
// the accumulators of the (BM/2) x (BN/4) wave tile, so the fragments get 64:
// the B fragments are double-buffered (the next half-step's set is read while
// the current one is in use), the A fragments are single-buffered and rolled:
// MFMAs run row by row, A_i is dead after the last MFMA of row i, and the next
// half-step's A_i is read into the same registers right then.
template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
struct TileCore {
  static constexpr int TM = BM / kWavesM, TN = BN / kWavesN;
  static constexpr int MT = TM / 32, NT = TN / 32;
  f32x16 acc[MT][NT];
  i32x8 fa[MT], fb0[NT], fb1[NT];
  DmaLoader<A_KMAJOR, BM> la;
  DmaLoader<B_KMAJOR, BN> lb;
  int wm, wn, K;

  __device__ __forceinline__ void init(const GemmArgs& g, int wm_, int wn_) {
    wm = wm_;
    wn = wn_;
    K = g.K;
  }

  __device__ __forceinline__ void zero_acc() {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  }

  // Points the loaders at tile (m0, n0); `valid` false makes every load of the
  // tile fall outside the descriptors (used past the workgroup's last tile).
  __device__ __forceinline__ void retarget(const GemmArgs& g, int64_t batch, int m0, int n0, bool valid) {
    la.set_tile(g.A + batch * g.stride_a, g.lda, m0, g.M, g.K, valid);
    lb.set_tile(g.B + batch * g.stride_b, g.ldb, n0, g.N, g.K, valid);
  }

  static constexpr int kPartsA = frag_parts<A_KMAJOR>(), kPartsB = frag_parts<B_KMAJOR>();
  static constexpr int kMfmas = MT * NT;
  static constexpr int kDmaOps = DmaLoader<A_KMAJOR, BM>::kPerWave + DmaLoader<B_KMAJOR, BN>::kPerWave;

  template <int I, int PART>
  __device__ __forceinline__ void read_a(const uint8_t* stage, int ks) {
    read_fragment_part<A_KMAJOR, BM, PART>(stage, wm + I * 32, ks, fa[I]);
  }
  template <int J, int PART>
  __device__ __forceinline__ void read_b(const uint8_t* stage, int ks, i32x8 (&fb)[NT]) {
    read_fragment_part<B_KMAJOR, BN, PART>(stage + BM * kBK, wn + J * 32, ks, fb[J]);
  }

  template <int OP>
  __device__ __forceinline__ void dma_op(uint8_t* stage, int kt) {
    constexpr int na = DmaLoader<A_KMAJOR, BM>::kPerWave;
    if constexpr (OP < na) la.template issue_one<OP>(stage, kt * kBK, K);
    else lb.template issue_one<OP - na>(stage + BM * kBK, kt * kBK, K);
  }

  __device__ __forceinline__ void issue_stage(uint8_t* __restrict__ stage, int kt) {
    static_for<kDmaOps>([&](auto oc) { dma_op<decltype(oc)::value>(stage, kt); });
    la.advance();
    lb.advance();
  }

  // One MFMA block (every tile of the wave, 64 k) on the fragments (fa, cb),
  // with the LDS reads of the next block's fragments and, when WITH_DMA, this
  // wave's global->LDS loads of a later stage dealt out between the MFMAs.
  // sched_barrier(0) after each group pins the written order (left alone, the
  // scheduler gathers the reads after the MFMAs).
  template <bool WITH_DMA>
  __device__ __forceinline__ void block(const i32x8 (&cb)[NT], i32x8 (&nb)[NT],
                                        const uint8_t* __restrict__ rd_stage, int rd_ks,
                                        uint8_t* __restrict__ dma_stage, int dma_kt) {
    constexpr int kBOps = NT * kPartsB;
    constexpr int kBPerGroup = (kBOps + kMfmas - 1) / kMfmas;
    constexpr int kDmaPerGroup = (kDmaOps + kMfmas - 1) / kMfmas;
    static_for<kMfmas>([&](auto gc) {
      constexpr int gi = decltype(gc)::value;
      constexpr int i = gi / NT, j = gi % NT;
      acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
          cb[j], fa[i], acc[i][j], mfma_code<FMT_B>(), mfma_code<FMT_A>(), 0, 0, 0, 0);
      if constexpr (WITH_DMA) {
        static_for<kDmaPerGroup>([&](auto dc) {
          constexpr int op = gi * kDmaPerGroup + decltype(dc)::value;
          if constexpr (op < kDmaOps) dma_op<op>(dma_stage, dma_kt);
        });
      }
      static_for<kBPerGroup>([&](auto rc) {
        constexpr int op = gi * kBPerGroup + decltype(rc)::value;
        if constexpr (op < kBOps) read_b<op / kPartsB, op % kPartsB>(rd_stage, rd_ks, nb);
      });
      if constexpr (j == NT - 1) {
        // row i of MFMAs is done: its A fragment is dead, fetch the next half-step's
        static_for<kPartsA>([&](auto pc) { read_a<i, decltype(pc)::value>(rd_stage, rd_ks); });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (WITH_DMA) {
      la.advance();
      lb.advance();
    }
  }

  // A workgroup barrier orders LDS traffic but does not wait for this wave's
  // outstanding global->LDS loads: drain them first (vmcnt(0)), so that after
  // the barrier every wave sees every wave's share of the stage.
  __device__ __forceinline__ static void wait_loads_then_barrier() {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  }

  // First fragments of a tile whose stages 0 and 1 have been issued.
  __device__ __forceinline__ void first_fragments(uint8_t* __restrict__ s0) {
    wait_loads_then_barrier();
    static_for<MT>([&](auto ic) {
      static_for<kPartsA>([&](auto pc) { read_a<decltype(ic)::value, decltype(pc)::value>(s0, 0); });
    });
    static_for<NT>([&](auto jc) {
      static_for<kPartsB>([&](auto pc) { read_b<decltype(jc)::value, decltype(pc)::value>(s0, 0, fb0); });
    });
  }

  // Two K stages: stage kt sits in s0, stage kt+1 in s1 (or is still landing
  // there).  After each barrier every wave is done with the stage just
  // consumed, so the stage two ahead starts to overwrite it while the second
  // half of the current stage and the whole next stage compute.
  __device__ __forceinline__ void k_pair(uint8_t* __restrict__ s0, uint8_t* __restrict__ s1, int kt) {
    block<false>(fb0, fb1, s0, 1, nullptr, 0);
    wait_loads_then_barrier();
    block<true>(fb1, fb0, s1, 0, s0, kt + 2);
    block<false>(fb0, fb1, s1, 1, nullptr, 0);
    wait_loads_then_barrier();
    block<true>(fb1, fb0, s0, 0, s1, kt + 3);
  }
};

// Logical tile index -> (tile_m, tile_n), walking the tile grid in column
// groups of kGroupM rows so that consecutive indices share A and B panels.
__device__ __forceinline__ void tile_coords(int logical, int tiles_m, int tiles_n, int* tile_m, int* tile_n) {
  constexpr int kGroupM = 8;
  const int group_size = kGroupM * tiles_n;
  const int grp = logical / group_size;
  const int first_m = grp * kGroupM;
  const int gm = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
  const int in_grp = logical - grp * group_size;
  *tile_m = first_m + in_grp % gm;
  *tile_n = in_grp / gm;
}

// Persistent kernel: gridDim.x workgroups (at most one per CU) each walk a list
// of tiles.  Workgroups are dealt to the 8 XCDs round-robin by id; each XCD owns
// a contiguous range of the tile order, and in round r its workgroups take the
// next gridDim.x / 8 tiles of that range, so that the tiles in flight on one
// XCD form a compact patch that shares A and B panels in its L2.
template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
__global__ __launch_bounds__(kGemmThreads) void fp8_gemm_tile_kernel(GemmArgs g) {
  constexpr int TM = BM / kWavesM, TN = BN / kWavesN;   // per-wave tile
  constexpr int MT = TM / 32, NT = TN / 32;             // MFMA tiles per wave
  constexpr int kStageBytes = (BM + BN) * kBK;
  // Two stages as two separate arrays, so that loads into one and reads from
  // the other are provably disjoint; the epilogue has its own staging area.
  __shared__ __attribute__((aligned(1024))) uint8_t lds0[kStageBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t lds1[kStageBytes];
  __shared__ __attribute__((aligned(16))) float lds_epi[kWaves * epilogue_stage_floats<MT, NT>()];

  const int nb = gridDim.x, bid = blockIdx.x;
  const int tiles = g.tiles_m * g.tiles_n;
  const int xcd = bid & 7, slot = bid >> 3;
  const int slots = (nb - xcd + 7) >> 3;              // workgroups on this XCD
  const int per = tiles >> 3, rem = tiles & 7;
  const int first = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
  const int count = per + (xcd < rem ? 1 : 0);        // tiles of this XCD

  const int64_t batch = blockIdx.y;
  const int wave = threadIdx.x >> 6;
  const int wm = (wave / kWavesN) * TM, wn = (wave % kWavesN) * TN;
  float* stage = lds_epi + wave * epilogue_stage_floats<MT, NT>();

  const bool fast_epilogue = epilogue_fast_ok(g, batch);

  TileCore<BM, BN, A_KMAJOR, B_KMAJOR, FMT_A, FMT_B> core;
  core.init(g, wm, wn);
  const int KT = (g.K + kBK - 1) / kBK;
  const int KT2 = (KT + 1) & ~1;

  // Stages at or beyond K are loaded all the same: they fall outside the buffer
  // descriptors and arrive as zeros.  The K loop therefore runs an even number
  // of branch-free steps, and an odd stage count costs one step of zero
  // products instead of a second copy of the MFMA block.  The loads that the
  // last two steps of a tile issue are the first two stages of the workgroup's
  // next tile, which land while the epilogue runs.
  int idx = slot;
  if (idx >= count) return;
  int tile_m, tile_n;
  tile_coords(first + idx, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
  core.la.set_lane_offsets(g.lda);
  core.lb.set_lane_offsets(g.ldb);
  core.retarget(g, batch, tile_m * BM, tile_n * BN, true);
  core.issue_stage(lds0, 0);
  core.issue_stage(lds1, 1);
  for (;;) {
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    core.zero_acc();
    core.first_fragments(lds0);
    for (int kt = 0; kt < KT2; kt += 2) {
      if (kt + 2 == KT2) {
        idx += slots;
        const bool more = idx < count;
        if (more) tile_coords(first + idx, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
        core.retarget(g, batch, tile_m * BM, tile_n * BN, more);
      }
      // stage numbers restart at 0 for the next tile
      core.k_pair(lds0, lds1, kt + 2 == KT2 ? -2 : kt);
    }
    if (fast_epilogue) {
      if (g.sb_mode == MI355Q_GS_PER_COL) epilogue_bf16_fast<MT, NT, true>(g, batch, core.acc, m0 + wm, n0 + wn, stage);
      else epilogue_bf16_fast<MT, NT, false>(g, batch, core.acc, m0 + wm, n0 + wn, stage);
    } else {
      epilogue<MT, NT>(g, batch, core.acc, m0 + wm, n0 + wn, stage);
    }
    if (idx >= count) break;
    // recomputed rather than kept live through the epilogue
    core.la.set_lane_offsets(g.lda);
    core.lb.set_lane_offsets(g.ldb);
  }
  // drain the (out-of-range) loads issued for the tile that does not exist
  __builtin_amdgcn_s_waitcnt(0);
}

template <int BM, int BN, bool AK, bool BK_, int FA, int FB>
void launch_tile(const GemmArgs& g, int64_t batch, hipStream_t st) {
  GemmArgs a = g;
  a.tiles_m = (g.M + BM - 1) / BM;
  a.tiles_n = (g.N + BN - 1) / BN;
  const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
  const int cus = compute_units();
  dim3 grid((unsigned)(tiles < cus ? tiles : cus), (unsigned)batch);
  fp8_gemm_tile_kernel<BM, BN, AK, BK_, FA, FB><<<grid, kGemmThreads, 0, st>>>(a);
}

// A K-major / B K-major etc.; defined in gemm_inst_*.hip
void launch_gemm_kk(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_km(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_mk(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_mm(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);

}  // namespace mi355q
