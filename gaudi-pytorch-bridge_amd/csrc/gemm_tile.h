// fp8 x fp8 -> fp32-accumulate -> bf16/fp32 GEMM for gfx950 (fp8_gemm_v2).
//
// Tiled kernel: a workgroup of 2 x WN waves owns a BM x BN tile of C and walks K
// in steps of 128 bytes.  Operand tiles travel from global memory straight into
// LDS (buffer_load_dwordx4 ... lds: no staging registers, and the buffer
// descriptor's bounds check zero-fills rows past the matrix edge) into one of
// two LDS stages, so the loads of step k+2 fly while step k computes.  Inside a
// stage, the 16-byte chunks of a row are XOR-swizzled with the row number,
// which keeps the 128-bit and transposing fragment reads free of bank
// conflicts; since a DMA load places lane l's chunk at LDS offset 16 l, the
// swizzle is applied by choosing which global chunk each lane fetches.  Each
// wave computes its (BM/2) x (BN/WN) sub-tile with v_mfma_f32_32x32x64_f8f6f4
// (fp8/bf8 operands, 64 k per instruction), reading the fragments of the next
// half-step while the MFMAs of the current one run.  The buffer descriptors
// walk along K by scalar arithmetic, so the per-lane offsets are small
// constants and operands of any size are addressable.
//
// Two wave grids are built.  2 x 4 (eight waves, two per SIMD, 128 x 64 wave
// tiles at BM = BN = 256): while one wave of a SIMD sits in its epilogue or
// waits for a fragment, the other keeps the matrix pipe busy; this grid carries
// both epilogues.  2 x 2 (four waves, one per SIMD, 128 x 128 wave tiles, all
// 256 accumulation registers): a third fewer LDS fragment bytes per MFMA, which
// is what matters once the chip runs at its power limit; its epilogue is not
// hidden by a second wave, so it exists with the fast bf16 epilogue only.
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
//
// One counter tracks a wave's outstanding vector memory operations, and it
// retires them in issue order.  Everything in the persistent tile loop is
// arranged around that: the fast epilogue loads nothing from global memory
// (its scales and bias arrive in LDS through the K loop's own load stream), so
// that no wait of its own also waits for the next tile's first stages, which
// are already in flight; and the wait for those stages at the start of a tile
// lets the previous tile's stores stay outstanding.
#pragma once
#include <type_traits>

#include "device_common.h"

namespace mi355q {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define LDS_AS __attribute__((address_space(3)))

constexpr int kWavesM = 2;  // the waves of a workgroup form a 2 x WN grid over its tile
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
  int fast_epi;  // epilogue_fast_ok() of this launch
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
//   MN-major, 256-byte rows, variant V = 1 (fragments of the 16x16x128 MFMA, gemm_tile16.h): the two 16-lane groups
//     of a cycle read the same chunk of k-rows 32 apart, so bit 5 of the row goes into the XOR as well and sends
//     the second group to the other parity.
//   K-major, 128-byte rows, variant V = 1 (the same fragments): lane group g = lane / 16 reads chunks 2 g, 2 g + 1 of
//     16 consecutive rows, and with the XOR above every ds_read_b128 of that shape takes twice its four cycles
//     (measured: SQ_LDS_BANK_CONFLICT half of SQ_LDS_IDX_ACTIVE, and 1.66 times the time of a conflict-free read in
//     a loop that only reads).  Of the 4096 XORs that are linear in the row's low four bits, 1344 read at full
//     rate; the one used swaps the two low bits of the XOR above: bit 0 from row bit 2, bit 1 from row bit 1,
//     bit 2 from row bit 3.
template <bool KMAJOR, int ROWS, int ROW_BYTES, int V = 0>
struct TileGeom {
  static constexpr int kChunksPerRow = ROW_BYTES / 16;
  static constexpr int kChunks = ROWS * kChunksPerRow;
  static_assert(KMAJOR ? (ROW_BYTES == 128 || ROW_BYTES == 64) : (ROW_BYTES == 256 || ROW_BYTES == 128), "no swizzle defined");
  static constexpr int kSwizzlePeriod = KMAJOR ? 16 : 8;  // swizzle(row + kSwizzlePeriod) == swizzle(row)
  __device__ static __forceinline__ int swizzle(int row) {
    if constexpr (KMAJOR && ROW_BYTES == 128) return V == 1 ? (((row >> 2) & 1) | (row & 2) | ((row >> 1) & 4)) : ((row >> 1) & 7);
    else if constexpr (KMAJOR) return (row >> 2) & 3;
    else if constexpr (ROW_BYTES == 256) return V == 1 ? (((row & 7) << 1) | ((row >> 5) & 1)) : ((row & 7) << 1);
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

// The lane number, computed on the spot.  Inside the persistent tile loop every
// value that depends only on the lane number is loop invariant: left alone,
// the compiler computes it once before the K loop, where no register is free,
// and spills it (a spill is a memory access by every lane, and the wait for its
// reload also waits for the next tile's global->LDS loads).  An asm statement is
// neither hoisted nor merged with another, and it needs no live input.
__device__ __forceinline__ int lane_id_here() {
  int lane;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
  return lane;
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
// V: swizzle variant of TileGeom (1: the waves' shares must be whole blocks of 32 rows, inside which the swizzle
// keeps its period of 8 rows)
template <bool KMAJOR, int EXT, int BK, int WAVES, int V = 0>
struct DmaLoader {
  using G = TileGeom<KMAJOR, KMAJOR ? EXT : BK, KMAJOR ? BK : EXT, V>;
  static constexpr int kCPR = G::kChunksPerRow;
  static constexpr int kRowsPerRegion = 64 / kCPR;
  static constexpr int kRegions = G::kChunks / 64;
  static constexpr int kPerWave = kRegions / WAVES;
  static_assert(kRegions % WAVES == 0 && 64 % kCPR == 0, "tile does not split over the waves");
  static_assert(V == 0 || KMAJOR || (EXT == 256 && kPerWave * kRowsPerRegion == 32), "variant 1: a wave loads whole blocks of 32 k-rows");

  // Raw buffer descriptor: base, stride 0, num_records (bytes), dword 3 flags.
  // The base walks along K, one stage per advance(), and num_records shrinks
  // with it, so the per-lane offsets never change and stay below 2^31 whatever
  // the size of the matrix (a stage spans at most 256 rows of ld bytes).
  i32x4 rsrc;
  int64_t remaining;  // bytes from the base to the end of the addressable part of the matrix
  int64_t step;       // bytes between K stages
  // A wave's regions are consecutive, and regions a swizzle period apart differ
  // by whole rows only: the offsets of the first kStored regions are kept, the
  // others are those plus a multiple of region_step (registers are what the K
  // loop is short of; an addition per load is not).
  static constexpr int kPeriodRegions = G::kSwizzlePeriod / kRowsPerRegion > 0 ? G::kSwizzlePeriod / kRowsPerRegion : 1;
  static constexpr int kStored = kPerWave % kPeriodRegions == 0 ? kPeriodRegions : kPerWave;
  int voff[kStored];  // this lane's offsets inside a stage
  int kc[kStored];    // K-major: byte offset of this lane's chunk inside a stage row
  int region_step;    // bytes between regions kStored apart
  int wave;

  static constexpr int64_t kMaxRecords = 0x80000000LL;  // keeps the out-of-range marker out of range

  // Per-lane geometry; depends on the leading dimension only.
  // wave_index: this wave's position among the WAVES waves that share the
  // loads of this operand (default: its position in the workgroup).
  __device__ __forceinline__ void set_lane_offsets(int64_t ld, int wave_index = -1) {
    const int lane = lane_id_here();
    wave = wave_index >= 0 ? wave_index : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rin = lane / kCPR, p = lane % kCPR;
#pragma unroll
    for (int i = 0; i < kStored; ++i) {
      const int row = (wave * kPerWave + i) * kRowsPerRegion + rin;
      const int c = p ^ G::swizzle(row);
      voff[i] = row * (int)ld + c * 16;
      kc[i] = c * 16;
    }
    region_step = kStored * kRowsPerRegion * (int)ld;
  }

  // For kernels that count their outstanding loads (K-major operands): tile rows from
  // rows_valid on are fetched from the last valid row instead of falling outside the
  // descriptor.  Their products are never stored, so what they hold does not matter; but a
  // load whose lanes are all out of range completes at once, ahead of older loads, while one
  // that goes to memory retires in issue order, which is what a counted wait relies on.
  int last_row_off = 0, first_row = 0, rows_valid = 0x7fffffff;
  __device__ __forceinline__ void clamp_rows(int64_t ld, int valid) {
    static_assert(KMAJOR, "rows of an MN-major tile are K");
    const int lane = lane_id_here();
    first_row = wave * kPerWave * kRowsPerRegion + lane / kCPR;
    rows_valid = valid;
    last_row_off = (valid - 1) * (int)ld;
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
      // up to the end of the 16-byte chunk that holds the last column (ld is a multiple of 16 and
      // at least the extent): a chunk that straddles the descriptor's end would read as zero whole
      remaining = (int64_t)(K - 1) * ld + (((extent + 15) & ~15) - mn0);
      step = (int64_t)BK * ld;
    }
    if (!valid) remaining = 0;
    stage_offset = 0;
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
  // NT: the nontemporal hint, for an operand that is read once (the weights of a decode-shaped call): a strip
  // read of a 235 MB matrix runs 8 % faster with it (41 against 45 us), through registers or into LDS alike.
  // K_CHECK false: the caller's K is a whole number of the stages it walks, no lane is ever past K, and the
  // operand is narrow (see advance_narrow()).  Then (and without CLAMP_ROWS) a lane's offset does not depend on the
  // stage, the descriptor stays where set_tile() put it and the stage is the instruction's scalar offset; and four
  // loads in a row share one write of m0: the instruction's immediate offset moves the LDS address and the memory
  // address alike, so region I takes the m0 of region I - I % 4, the immediate (I % 4) KiB, and a lane offset
  // lowered by as much.  The caller issues the regions of a group in order with nothing between them that writes m0.
  template <int I, bool CLAMP_ROWS = false, bool NT = false, bool K_CHECK = true>
  __device__ __forceinline__ void issue_one(uint8_t* lds_tile, int k0, int K) const {
    const uint32_t lds_base = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)lds_tile;
    if constexpr (!K_CHECK && !CLAMP_ROWS && !NT && kPerWave % 4 == 0) {
      constexpr int i = I, r = I % 4;
      const int vo = voff[i % kStored] + (i / kStored) * region_step - r * 1024;
      if constexpr (r == 0) {
        const uint32_t dst = lds_base + (uint32_t)((wave * kPerWave + i) * 1024);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(dst), "v"(vo), "s"(rsrc), "s"(stage_offset)
                     : "memory", "m0");
      } else {
        asm volatile("buffer_load_dwordx4 %0, %1, %3 offen offset:%2 lds"
                     :
                     : "v"(vo), "s"(rsrc), "n"(r * 1024), "s"(stage_offset)
                     : "memory");
      }
    } else {
      constexpr int i = I;
      int vo = voff[i % kStored] + (i / kStored) * region_step;
      if constexpr (CLAMP_ROWS) vo = (first_row + i * kRowsPerRegion < rows_valid) ? vo : last_row_off + kc[i % kStored];
      if constexpr (KMAJOR && K_CHECK) vo = (k0 + kc[i % kStored] < K) ? vo : 0x7fffffff;
      const uint32_t dst = lds_base + (uint32_t)((wave * kPerWave + i) * 1024);
      // m0 holds the LDS address of the region; lane l's 16 bytes land at m0 + 16 l.
      // Written as asm so that the compiler, which would otherwise make every later
      // LDS read wait for all outstanding global->LDS loads, leaves the waiting to
      // the explicit vmcnt drain before each barrier.
      if constexpr (NT) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds"
                     :
                     : "s"(dst), "v"(vo), "s"(rsrc)
                     : "memory", "m0");
      } else {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :
                     : "s"(dst), "v"(vo), "s"(rsrc)
                     : "memory", "m0");
      }
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

  // advance() for an operand whose whole extent, from its first byte to the last one the launch may address, is
  // below kNarrowBytes, walked forwards only from set_tile() on and loaded with issue_one<.., K_CHECK = false>: the
  // descriptor stays on the tile's first stage and the bytes walked so far go into the loads' scalar offset, one
  // scalar addition per stage.  (The general form moves the base and clamps a 64-bit count of the bytes left with
  // compares that the compiler puts on the vector ALU, a dozen instructions per operand and stage: a wave that
  // issues one MFMA after the other has no issue slot to spare for them.)
  static constexpr int64_t kNarrowBytes = 0x40000000LL;
  int stage_offset = 0;
  __device__ __forceinline__ void advance_narrow() { stage_offset += (int)step; }

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

// Fragment reads of one operand with the address registers spelled out.  Every
// LDS read of the K loop needs its address in a vector register; what can sit in
// the instruction's 16-bit offset field instead is whatever differs by a
// compile-time constant.  The XOR swizzle makes some differences depend on the
// lane, so left to itself the compiler keeps a register per read (about 30 for a
// 128 x 128 wave tile).  Spelled out, one register per swizzle pattern is enough:
//   K-major : the pattern depends on (k half, part) - 4 registers; the 32-row
//             tile index and the stage are constant offsets;
//   MN-major: the pattern depends on the 32-column tile index - TILES registers;
//             k half, part and stage are constant offsets.
// The two stages of an operand are STAGE_BYTES apart (adjacent, so that the
// offsets stay below 64 KiB).
template <bool KMAJOR, int EXT, int TILES>
struct FragReader {
  using G = TileGeom<KMAJOR, KMAJOR ? EXT : kBK, KMAJOR ? kBK : EXT>;
  static constexpr int kRowBytes = KMAJOR ? kBK : EXT;
  static constexpr int kStageBytes = EXT * kBK;
  static constexpr int kRegs = KMAJOR ? 4 : TILES;
  static constexpr int kParts = KMAJOR ? 2 : 4;
  static_assert(kStageBytes + (KMAJOR ? (TILES - 1) * 32 * kRowBytes : (64 + 24) * kRowBytes) < 65536, "offset field");
  uint32_t addr[kRegs];

  // lds_operand: LDS address of stage 0 of this operand; mn_wave: first row
  // (column) of the wave's tile inside the workgroup's
  __device__ __forceinline__ void init(uint32_t lds_operand, int mn_wave) {
    const int lane = lane_id_here();
    if constexpr (KMAJOR) {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int part = 0; part < 2; ++part)
          addr[ks * 2 + part] = lds_operand + G::lds_offset(mn_wave + (lane & 31), ks * 4 + (lane >> 5) * 2 + part);
    } else {
      // Within each group of 16 lanes, lanes 2r and 2r+1 point at the two 8-byte
      // halves of k-row r; after the transposing read lane i of the group holds
      // column i for those 8 k-rows.
      const int blk = lane >> 4, i = lane & 15;
      const int r = i >> 1, h = i & 1;
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        const int col = mn_wave + 32 * t + (blk & 1) * 16;  // first column of this 16-lane group
        addr[t] = lds_operand + G::lds_offset((blk >> 1) * 32 + r, col >> 4) + h * 8;
      }
    }
  }

  // Part PART of the fragment of tile T, k half KS, from stage STAGE.
  template <int T, int PART, int KS, int STAGE>
  __device__ __forceinline__ void read(i32x8& f) const {
    if constexpr (KMAJOR) {
      constexpr int off = STAGE * kStageBytes + T * 32 * kRowBytes;
      const u32x4 v = *reinterpret_cast<LDS_AS const u32x4*>(addr[KS * 2 + PART] + off);
      f[4 * PART + 0] = v[0];
      f[4 * PART + 1] = v[1];
      f[4 * PART + 2] = v[2];
      f[4 * PART + 3] = v[3];
    } else {
      constexpr int off = STAGE * kStageBytes + (KS * 64 + PART * 8) * kRowBytes;
      const i32x2 t = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<LDS_AS i32x2*>(addr[T] + off));
      f[2 * PART] = t[0];
      f[2 * PART + 1] = t[1];
    }
  }
};

// The scalar (per-tensor) scales of a launch.
struct ScalarScales {
  float sa, sb;
};
__device__ __forceinline__ ScalarScales load_scalar_scales(const GemmArgs& g) {
  ScalarScales s = {1.0f, 1.0f};
  if (g.sa_mode == MI355Q_GS_HOST) s.sa = g.sa_host;
  else if (g.sa_mode == MI355Q_GS_DEV) s.sa = g.sa[0];
  if (g.sb_mode == MI355Q_GS_HOST) s.sb = g.sb_host;
  else if (g.sb_mode == MI355Q_GS_DEV) s.sb = g.sb[0];
  // consumed here, so the wait for the loads is here as well
  s.sa = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(s.sa)));
  s.sb = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(s.sb)));
  return s;
}

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
  const int lane = lane_id_here();
  const int es = g.out_bf16 ? 2 : 4;
  uint8_t* C = g.C + batch * g.stride_c * es;
  const uint8_t* D = g.D ? g.D + batch * g.stride_d * es : nullptr;
  const uint8_t* bias = g.bias ? g.bias + batch * g.stride_bias * es : nullptr;
  const ScalarScales scalars = load_scalar_scales(g);
  const float sa_s = scalars.sa, sb_s = scalars.sb;

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
        for (int it = 0; it < kEpiRows / kRowsPerPass; ++it) {
          const int r = r_in + it * kRowsPerPass;
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
        for (int it = 0; it < kEpiRows / kRowsPerPass; ++it) {
          const int r = r_in + it * kRowsPerPass;
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

// The forms the fast bf16 epilogue serves: bf16 output, rows and row pitch of C
// multiples of 16 bytes, N a multiple of 8, A scale a scalar or one value per
// row, B scale a scalar or one 16-byte-aligned value per column, bias none or
// an 8-byte-aligned row vector, accumulate input none or 8-byte-aligned rows.  The conditions hold for
// every matrix of a batch or for none, so the host chooses the kernel.
inline bool epilogue_fast_ok(const GemmArgs& g, int64_t batches) {
  if (!g.out_bf16 || g.bias_mode == MI355Q_BIAS_FULL) return false;
  if (g.D != nullptr) {  // read in 8-byte pieces
    if ((reinterpret_cast<uintptr_t>(g.D) & 7u) != 0 || (g.ldd & 3) != 0 || g.ldd > (int64_t(1) << 22)) return false;
    if (batches > 1 && (g.stride_d & 3) != 0) return false;
  }
  if (g.sa_mode == MI355Q_GS_PER_COL || g.sb_mode == MI355Q_GS_PER_ROW) return false;
  if ((reinterpret_cast<uintptr_t>(g.C) & 15u) != 0 || (g.ldc & 7) != 0 || (g.N & 7) != 0) return false;
  if (g.ldc > (int64_t(1) << 22)) return false;  // byte offsets inside a wave's rows stay below 2^31
  if (batches > 1 && (g.stride_c & 7) != 0) return false;
  if (g.sb_mode == MI355Q_GS_PER_COL && (reinterpret_cast<uintptr_t>(g.sb) & 15u) != 0) return false;
  if (g.bias_mode == MI355Q_BIAS_ROW_VECTOR) {
    if ((reinterpret_cast<uintptr_t>(g.bias) & 7u) != 0) return false;
    if (batches > 1 && (g.stride_bias & 3) != 0) return false;
  }
  return true;
}

// Stores a wave issues in epilogue_bf16_fast, all of them after its loads.
template <int MT, int NT>
constexpr int fast_epilogue_stores() { return MT * 2 * NT; }

// bf16 epilogue for the common forms.  Scales and bias are applied in the
// accumulator layout (a lane holds one row m and runs of 4 columns), the
// rounded bf16 values of 32 rows pass through a per-wave LDS area of 32 rows x
// (32 NT) bf16, and come back with a lane owning 8 consecutive columns of a
// row: a wave stores whole rows of its tile, 16 bytes per lane.
// LDS layout: 8-byte slots of a row are XORed with f(row) so that the 32 lanes
// of a write cycle (32 rows, one logical slot) and the 16 lanes of a read cycle
// (rows of equal f, consecutive 16-byte chunks) touch distinct banks; an odd f
// swaps the two halves of a 16-byte chunk, undone after the read.
// The part that consumes the accumulators is one basic block: rows past M and
// columns past N are dropped by the store's range check instead of by branches
// (with branches in it the register allocator copies every accumulator out of
// the accumulation registers at once and spills).
// STAGED: the scale and bias values of the wave's rows and columns already sit
// in its staging area (ScaleStager, below) and the scalar scales come as
// arguments, so that the epilogue loads nothing from global memory: a wait for
// such a load would also wait for every global->LDS load issued before it,
// that is for the next tile's first stages.
// Layout of the staged values in a wave's staging area (bytes): B scales of its
// 32 NT columns (fp32), bias of the same columns (bf16), A scales of its 32 MT
// rows (fp32).  Values of a kind the problem does not have are zeros.
constexpr int kStagedColScale = 0, kStagedBias = 512, kStagedRowScale = 768, kStagedBytes = 1280;

template <int MT, int NT, bool PER_COL, bool HAS_BIAS, bool STAGED = false, bool HAS_D = false>
__device__ __forceinline__ void epilogue_bf16_fast(const GemmArgs& g, int64_t batch, f32x16 (&acc)[MT][NT],
                                                   int m_wave, int n_wave, float* stage_f,
                                                   ScalarScales scalars = ScalarScales{1.0f, 1.0f}) {
  static_assert(MT <= 4 && NT <= 4, "staged layout");
  constexpr int kRowBytes = 64 * NT;
  constexpr int kSlotMask = 8 * NT - 1;
  constexpr int kFShift = NT == 1 ? 2 : (NT == 2 ? 1 : 0);
  static_assert(NT == 1 || NT == 2 || NT == 4, "swizzle defined for 64-, 128- and 256-byte rows");
  constexpr int kLanesPerRow = 4 * NT;       // a lane reads back 16 bytes
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  constexpr int kPasses = 32 / kRowsPerPass;
  LDS_AS uint8_t* stage = (LDS_AS uint8_t*)stage_f;
  const int lane = lane_id_here();
  const int r = lane & 31, h = lane >> 5;

  if constexpr (!STAGED) scalars = load_scalar_scales(g);
  const float sa_s = scalars.sa, sb_s = scalars.sb;

  // Per-column values of the columns this lane holds in the accumulator layout
  // (columns at or beyond N read the last four: their results are not stored).
  // A scalar B scale is folded into the row factor instead, which leaves one
  // fused multiply-add per element.
  float cs[PER_COL ? NT : 1][4][4], cb[HAS_BIAS ? NT : 1][4][4];
  const uint16_t* bias = reinterpret_cast<const uint16_t*>(g.bias) + (HAS_BIAS ? batch * g.stride_bias : 0);
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int col = 32 * j + 8 * q + 4 * h;  // inside the wave's tile
      int n = n_wave + col;
      n = n < g.N - 4 ? n : g.N - 4;
      if constexpr (PER_COL) {
        const f32x4 v = STAGED ? *reinterpret_cast<LDS_AS const f32x4*>(stage + kStagedColScale + col * 4)
                               : *reinterpret_cast<const f32x4*>(g.sb + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) cs[j][q][e] = v[e];
      }
      if constexpr (HAS_BIAS) {
        const u32x2 v = STAGED ? *reinterpret_cast<LDS_AS const u32x2*>(stage + kStagedBias + col * 2)
                               : *reinterpret_cast<const u32x2*>(bias + n);
        cb[j][q][0] = __uint_as_float(v[0] << 16);
        cb[j][q][1] = __uint_as_float(v[0] & 0xffff0000u);
        cb[j][q][2] = __uint_as_float(v[1] << 16);
        cb[j][q][3] = __uint_as_float(v[1] & 0xffff0000u);
      }
    }
  float ra[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m_wave + 32 * i + r;
    if constexpr (STAGED) {
      const float staged = *reinterpret_cast<LDS_AS const float*>(stage + kStagedRowScale + (32 * i + r) * 4);
      ra[i] = g.sa_mode == MI355Q_GS_PER_ROW ? staged : sa_s;
    } else {
      ra[i] = sa_s;
      if (g.sa_mode == MI355Q_GS_PER_ROW) ra[i] = g.sa[m < g.M ? m : g.M - 1];
    }
    if (!PER_COL) ra[i] *= sb_s;
  }

  // C as seen by this wave: a buffer that starts at its first row and ends
  // after its last row inside the matrix.
  const int rows = g.M - m_wave < 32 * MT ? g.M - m_wave : 32 * MT;
  uint16_t* cbase = reinterpret_cast<uint16_t*>(g.C) + batch * g.stride_c + (int64_t)m_wave * g.ldc;
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(cbase, 0, rows > 0 ? rows * (int)g.ldc * 2 : 0, 0x00020000);

  const int f_w = (r >> kFShift) & kSlotMask;
  // read-back coordinates
  const int row_in_pass = lane / kLanesPerRow, chunk = lane % kLanesPerRow;
  const int n_out = n_wave + 8 * chunk;
  const int pitch = (int)g.ldc * 2;
  // columns at or beyond N: an offset no descriptor reaches
  const int voff0 = n_out < g.N ? row_in_pass * pitch + n_out * 2 : 0x7fffffff;
  const int pass_step = n_out < g.N ? kRowsPerPass * pitch : 0;

  // The accumulate input, read in the accumulator layout (4 bf16 per lane and
  // column group): rows past M fall outside the descriptor and read as zero.
  __amdgpu_buffer_rsrc_t rsrc_d = rsrc;
  int d_off0 = 0, d_pitch = 0;
  if constexpr (HAS_D) {
    const uint16_t* dbase = reinterpret_cast<const uint16_t*>(g.D) + batch * g.stride_d + (int64_t)m_wave * g.ldd;
    rsrc_d = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(dbase), 0, rows > 0 ? rows * (int)g.ldd * 2 : 0, 0x00020000);
    d_pitch = (int)g.ldd * 2;
    d_off0 = r * d_pitch + (n_wave + 4 * h) * 2;
  }

  // scaled, rounded values of the 32 rows of accumulator row i -> staging area
  auto write_rows = [&](auto ic) {
    constexpr int i = decltype(ic)::value;
    u32x2 dv[HAS_D ? NT : 1][4];
    if constexpr (HAS_D) {
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          dv[j][q] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(
              rsrc_d, d_off0 + 32 * i * d_pitch + (32 * j + 8 * q) * 2, 0, 0));
    }
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float b = HAS_BIAS ? cb[j][q][e] : 0.0f;
          if constexpr (PER_COL) v[e] = __builtin_fmaf(acc[i][j][4 * q + e] * ra[i], cs[j][q][e], b);
          else v[e] = __builtin_fmaf(acc[i][j][4 * q + e], ra[i], b);
        }
        if constexpr (HAS_D) {
          v[0] += __uint_as_float(dv[j][q][0] << 16);
          v[1] += __uint_as_float(dv[j][q][0] & 0xffff0000u);
          v[2] += __uint_as_float(dv[j][q][1] << 16);
          v[3] += __uint_as_float(dv[j][q][1] & 0xffff0000u);
        }
        const u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        const int slot = (8 * j + 2 * q + h) ^ f_w;
        *reinterpret_cast<LDS_AS u32x2*>(stage + r * kRowBytes + slot * 8) = o;
      }
  };
  // staging area -> registers, a lane holding 8 consecutive columns of a row per pass
  auto read_rows = [&](u32x4 (&o)[kPasses]) {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int row = p * kRowsPerPass + row_in_pass;
      const int f = (row >> kFShift) & kSlotMask;
      o[p] = *reinterpret_cast<LDS_AS u32x4*>(stage + row * kRowBytes + ((chunk ^ (f >> 1)) << 4));
    }
  };
  // A wave's LDS instructions execute in the order issued, so the values of row
  // i + 1 may be written into the one staging area as soon as the reads of row
  // i have been issued: the arithmetic of row i + 1 runs while those reads are
  // on their way, and the stores of row i follow without a wait.
  static_assert(MT * kPasses == fast_epilogue_stores<MT, NT>(), "the K loop counts these stores");
  u32x4 o[kPasses];
  write_rows(std::integral_constant<int, 0>{});
  read_rows(o);
  static_for<MT>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (i + 1 < MT) write_rows(std::integral_constant<int, i + 1>{});
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int f = ((p * kRowsPerPass + row_in_pass) >> kFShift) & kSlotMask;
      const u32x4 v = (f & 1) ? u32x4{o[p][2], o[p][3], o[p][0], o[p][1]} : o[p];
      // lanes whose offset lies at or beyond the descriptor's size store nothing;
      // aux 2 = nt: streamed, keeps the operand panels in L2
      __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, voff0 + (i * kPasses + p) * pass_step, 0, 2);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (i + 1 < MT) read_rows(o);
  });
}

// ALLOW_D false: the caller guarantees there is no accumulate input (the
// kernel with 256 accumulator registers per lane keeps its epilogue to four
// variants; with more, the compiler copies accumulators to scratch memory).
template <int MT, int NT, bool STAGED = false, bool ALLOW_D = true>
__device__ __forceinline__ void epilogue_bf16_fast_any(const GemmArgs& g, int64_t batch, f32x16 (&acc)[MT][NT],
                                                       int m_wave, int n_wave, float* stage,
                                                       ScalarScales scalars = ScalarScales{1.0f, 1.0f}) {
  const bool per_col = g.sb_mode == MI355Q_GS_PER_COL, bias = g.bias_mode == MI355Q_BIAS_ROW_VECTOR;
  if (ALLOW_D && g.D != nullptr) {
    if (per_col && bias) epilogue_bf16_fast<MT, NT, true, true, STAGED, true>(g, batch, acc, m_wave, n_wave, stage, scalars);
    else if (per_col) epilogue_bf16_fast<MT, NT, true, false, STAGED, true>(g, batch, acc, m_wave, n_wave, stage, scalars);
    else if (bias) epilogue_bf16_fast<MT, NT, false, true, STAGED, true>(g, batch, acc, m_wave, n_wave, stage, scalars);
    else epilogue_bf16_fast<MT, NT, false, false, STAGED, true>(g, batch, acc, m_wave, n_wave, stage, scalars);
    return;
  }
  if (per_col && bias) epilogue_bf16_fast<MT, NT, true, true, STAGED>(g, batch, acc, m_wave, n_wave, stage, scalars);
  else if (per_col) epilogue_bf16_fast<MT, NT, true, false, STAGED>(g, batch, acc, m_wave, n_wave, stage, scalars);
  else if (bias) epilogue_bf16_fast<MT, NT, false, true, STAGED>(g, batch, acc, m_wave, n_wave, stage, scalars);
  else epilogue_bf16_fast<MT, NT, false, false, STAGED>(g, batch, acc, m_wave, n_wave, stage, scalars);
}

// Brings the scale and bias values the fast epilogue of one wave tile needs
// into the wave's staging area with global->LDS loads, which join the K loop's
// stream of such loads (and its waits).  Ranges past N or M read as zeros.
struct ScaleStager {
  // 64 lanes x 4 bytes from `base` + 256 `part` (at most `bytes` valid from base) to lds_dst + 256 part
  __device__ __forceinline__ static void load_256(const void* base, int64_t bytes, int part, uint32_t lds_dst) {
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    const int64_t rec = bytes < 0 ? 0 : (bytes > 0x40000000 ? 0x40000000 : bytes);
    i32x4 rsrc;
    rsrc[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    rsrc[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((b >> 32) & 0xffffu));
    rsrc[2] = __builtin_amdgcn_readfirstlane((int)rec);
    rsrc[3] = 0x00020000;
    const int vo = lane_id_here() * 4 + part * 256;
    const uint32_t dst = lds_dst + part * 256;
    // m0 holds the LDS address; lane l's 4 bytes land at m0 + 4 l.  The s_nop
    // covers a descriptor word that reaches its scalar register through
    // v_readfirstlane (five wait states before a memory instruction reads it).
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dword %1, %2, 0 offen lds"
                 :
                 : "s"(dst), "v"(vo), "s"(rsrc)
                 : "memory", "m0");
  }

  template <int MT, int NT>
  __device__ __forceinline__ static void issue(const GemmArgs& g, int64_t batch, int m_wave, int n_wave, float* stage_f) {
    const uint32_t lds = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)stage_f;
    const bool per_col = g.sb_mode == MI355Q_GS_PER_COL, per_row = g.sa_mode == MI355Q_GS_PER_ROW;
    const bool has_bias = g.bias_mode == MI355Q_BIAS_ROW_VECTOR;
    constexpr int kColParts = (32 * NT * 4 + 255) / 256, kRowParts = (32 * MT * 4 + 255) / 256;
    static_for<kColParts>([&](auto pc) {
      load_256(g.sb + n_wave, per_col ? (int64_t)(g.N - n_wave) * 4 : 0, decltype(pc)::value, lds + kStagedColScale);
    });
    load_256(reinterpret_cast<const uint16_t*>(g.bias) + batch * g.stride_bias + n_wave,
             has_bias ? (int64_t)(g.N - n_wave) * 2 : 0, 0, lds + kStagedBias);
    static_for<kRowParts>([&](auto pc) {
      load_256(g.sa + m_wave, per_row ? (int64_t)(g.M - m_wave) * 4 : 0, decltype(pc)::value, lds + kStagedRowScale);
    });
  }
  template <int MT, int NT>
  static constexpr int ops() { return (32 * NT * 4 + 255) / 256 + 1 + (32 * MT * 4 + 255) / 256; }
};

// Per-wave state of the K loop: accumulators, fragments, loaders.
//
// Register budget.  Two waves per SIMD (WN = 4) leave 256 registers per lane:
// 128 hold the accumulators of the 128 x 64 wave tile, so the fragments get 64.
// One wave per SIMD (WN = 2) has 512: 256 accumulators of the 128 x 128 wave
// tile, 96 for fragments.  In both the B fragments are double-buffered (the
// next half-step's set is read while the current one is in use), the A
// fragments are single-buffered and rolled: MFMAs run row by row, A_i is dead
// after the last MFMA of row i, and the next half-step's A_i is read into the
// same registers right then.
template <int BM, int BN, int WN, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B>
struct TileCore {
  static constexpr int TM = BM / kWavesM, TN = BN / WN;
  using LoaderA = DmaLoader<A_KMAJOR, BM, kBK, kWavesM * WN>;
  using LoaderB = DmaLoader<B_KMAJOR, BN, kBK, kWavesM * WN>;
  static constexpr int MT = TM / 32, NT = TN / 32;
  using ReaderA = FragReader<A_KMAJOR, BM, MT>;
  using ReaderB = FragReader<B_KMAJOR, BN, NT>;
  // LDS ring: the two stages of A, then the two stages of B
  static constexpr int kStageA = BM * kBK, kStageB = BN * kBK;
  static constexpr int kRingBytes = 2 * (kStageA + kStageB);
  f32x16 acc[MT][NT];
  i32x8 fa[MT], fb0[NT], fb1[NT];
  LoaderA la;
  LoaderB lb;
  ReaderA ra;
  ReaderB rb;
  uint8_t* ring;
  int wave, wm, wn, K;  // wave: index in the workgroup (uniform)

  __device__ __forceinline__ void init(const GemmArgs& g, uint8_t* ring_, int wave_, int wm_, int wn_) {
    ring = ring_;
    wave = wave_;
    wm = wm_;
    wn = wn_;
    K = g.K;
  }

  // Per-lane addresses (LDS reads, global->LDS loads); recomputed for every
  // tile rather than kept live through the epilogue.
  __device__ __forceinline__ void set_lane_addresses(const GemmArgs& g) {
    const uint32_t base = (uint32_t)(uintptr_t)(LDS_AS uint8_t*)ring;
    ra.init(base, wm);
    rb.init(base + 2 * kStageA, wn);
    la.set_lane_offsets(g.lda, wave);
    lb.set_lane_offsets(g.ldb, wave);
  }

  // Points the loaders at tile (m0, n0); `valid` false makes every load of the
  // tile fall outside the descriptors (used past the workgroup's last tile).
  __device__ __forceinline__ void retarget(const GemmArgs& g, int64_t batch, int m0, int n0, bool valid) {
    la.set_tile(g.A + batch * g.stride_a, g.lda, m0, g.M, g.K, valid);
    lb.set_tile(g.B + batch * g.stride_b, g.ldb, n0, g.N, g.K, valid);
  }

  static constexpr int kPartsA = ReaderA::kParts, kPartsB = ReaderB::kParts;
  static constexpr int kMfmas = MT * NT;
  static constexpr int kDmaOps = LoaderA::kPerWave + LoaderB::kPerWave;

  template <int OP, int STAGE>
  __device__ __forceinline__ void dma_op(int kt) {
    constexpr int na = LoaderA::kPerWave;
    if constexpr (OP < na) la.template issue_one<OP>(ring + STAGE * kStageA, kt * kBK, K);
    else lb.template issue_one<OP - na>(ring + 2 * kStageA + STAGE * kStageB, kt * kBK, K);
  }

  template <int STAGE>
  __device__ __forceinline__ void issue_stage(int kt) {
    static_for<kDmaOps>([&](auto oc) { dma_op<decltype(oc)::value, STAGE>(kt); });
    la.advance();
    lb.advance();
  }

  // One MFMA block (every tile of the wave, 64 k) on the fragments (fa, cb),
  // with the LDS reads of the next block's fragments (k half RD_KS of stage
  // RD_STAGE) and, when DMA_STAGE >= 0, this wave's global->LDS loads of K
  // stage dma_kt into that stage dealt out between the MFMAs.
  // sched_barrier(0) after each group pins the written order (left alone, the
  // scheduler gathers the reads after the MFMAs).
  // ZERO_C: the first block of a tile, which starts the sums (no pass over the
  // accumulators to clear them).
  template <int RD_STAGE, int RD_KS, int DMA_STAGE, bool ZERO_C>
  __device__ __forceinline__ void block(const i32x8 (&cb)[NT], i32x8 (&nb)[NT], int dma_kt) {
    constexpr bool kWithDma = DMA_STAGE >= 0;
    constexpr int kBOps = NT * kPartsB;
    constexpr int kBPerGroup = (kBOps + kMfmas - 1) / kMfmas;
    constexpr int kDmaPerGroup = (kDmaOps + kMfmas - 1) / kMfmas;
    static_for<kMfmas>([&](auto gc) {
      constexpr int gi = decltype(gc)::value;
      constexpr int i = gi / NT, j = gi % NT;
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
          cb[j], fa[i], ZERO_C ? zero : acc[i][j], mfma_code<FMT_B>(), mfma_code<FMT_A>(), 0, 0, 0, 0);
      if constexpr (kWithDma) {
        static_for<kDmaPerGroup>([&](auto dc) {
          constexpr int op = gi * kDmaPerGroup + decltype(dc)::value;
          if constexpr (op < kDmaOps) dma_op<op, kWithDma ? DMA_STAGE : 0>(dma_kt);
        });
      }
      static_for<kBPerGroup>([&](auto rc) {
        constexpr int op = gi * kBPerGroup + decltype(rc)::value;
        if constexpr (op < kBOps) rb.template read<op / kPartsB, op % kPartsB, RD_KS, RD_STAGE>(nb[op / kPartsB]);
      });
      if constexpr (j == NT - 1) {
        // row i of MFMAs is done: its A fragment is dead, fetch the next half-step's
        static_for<kPartsA>([&](auto pc) { ra.template read<i, decltype(pc)::value, RD_KS, RD_STAGE>(fa[i]); });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (kWithDma) {
      la.advance();
      lb.advance();
    }
  }

  // A workgroup barrier orders LDS traffic but does not wait for this wave's
  // outstanding global->LDS loads: drain them first, so that after the barrier
  // every wave sees every wave's share of the stage.
  // The counter of outstanding vector memory operations retires in issue order.
  // The first two stages of a tile are issued before the previous tile's
  // epilogue, whose kEpilogueStores stores are therefore younger: when those are
  // pending (younger_stores), waiting until only that many operations are
  // outstanding waits for the loads and not for the stores, which take a few
  // microseconds to be acknowledged when every workgroup stores at once.
  static constexpr int kEpilogueStores = fast_epilogue_stores<MT, NT>();
  static_assert(kEpilogueStores < 64, "vmcnt holds 6 bits");
  __device__ __forceinline__ static void wait_loads_then_barrier(bool younger_stores = false) {
    if (younger_stores) __builtin_amdgcn_s_waitcnt((kEpilogueStores & 15) | ((kEpilogueStores >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  }

  // First fragments of a tile whose stages 0 and 1 have been issued.
  __device__ __forceinline__ void first_fragments(bool younger_stores) {
    wait_loads_then_barrier(younger_stores);
    static_for<MT>([&](auto ic) {
      static_for<kPartsA>([&](auto pc) { ra.template read<decltype(ic)::value, decltype(pc)::value, 0, 0>(fa[decltype(ic)::value]); });
    });
    static_for<NT>([&](auto jc) {
      static_for<kPartsB>([&](auto pc) { rb.template read<decltype(jc)::value, decltype(pc)::value, 0, 0>(fb0[decltype(jc)::value]); });
    });
  }

  // Two K stages: stage kt sits in ring stage 0, stage kt+1 in ring stage 1 (or
  // is still landing there).  After each barrier every wave is done with the
  // stage just consumed, so the stage two ahead starts to overwrite it while
  // the second half of the current stage and the whole next stage compute.
  // FIRST: the first two stages of a tile.
  // after_first_loads: called once the first pair has issued its loads (the
  // place for other loads that the tile's later waits should cover).
  template <bool FIRST, typename F>
  __device__ __forceinline__ void k_pair(int kt, bool younger_stores, F&& after_first_loads) {
    block<0, 1, -1, FIRST>(fb0, fb1, 0);
    wait_loads_then_barrier(FIRST && younger_stores);  // stage 1 of a tile is as old as stage 0
    block<1, 0, 0, false>(fb1, fb0, kt + 2);
    if constexpr (FIRST) after_first_loads();
    block<1, 1, -1, false>(fb0, fb1, 0);
    wait_loads_then_barrier();
    block<0, 0, 1, false>(fb1, fb0, kt + 3);
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
// a contiguous range of the tile order, and in pass r its workgroups take the
// next gridDim.x / 8 tiles of that range, so that the tiles in flight on one
// XCD form a compact patch that shares A and B panels in its L2.
template <int BM, int BN, int WN, bool A_KMAJOR, bool B_KMAJOR, int FMT_A, int FMT_B, bool FAST_ONLY>
__global__ __launch_bounds__(kWavesM * WN * 64) void fp8_gemm_tile_kernel(GemmArgs g) {
  constexpr int kWaves = kWavesM * WN;
  constexpr int TM = BM / kWavesM, TN = BN / WN;   // per-wave tile
  constexpr int MT = TM / 32, NT = TN / 32;             // MFMA tiles per wave
  using Core = TileCore<BM, BN, WN, A_KMAJOR, B_KMAJOR, FMT_A, FMT_B>;
  // two stages of each operand; the epilogue has its own staging area
  __shared__ __attribute__((aligned(1024))) uint8_t lds_ring[Core::kRingBytes];
  __shared__ __attribute__((aligned(16))) float lds_epi[kWaves * epilogue_stage_floats<MT, NT>()];

  const int nb = gridDim.x, bid = blockIdx.x;
  const int tiles = g.tiles_m * g.tiles_n;
  const int xcd = bid & 7, slot = bid >> 3;
  const int slots = (nb - xcd + 7) >> 3;              // workgroups on this XCD
  const int per = tiles >> 3, rem = tiles & 7;
  const int first = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
  const int count = per + (xcd < rem ? 1 : 0);        // tiles of this XCD

  const int64_t batch = blockIdx.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = (wave / WN) * TM, wn = (wave % WN) * TN;
  float* stage = lds_epi + wave * epilogue_stage_floats<MT, NT>();

  Core core;
  core.init(g, lds_ring, wave, wm, wn);
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
  core.set_lane_addresses(g);
  core.retarget(g, batch, tile_m * BM, tile_n * BN, true);
  core.template issue_stage<0>(0);
  core.template issue_stage<1>(1);
  const ScalarScales scalars = load_scalar_scales(g);
  bool stores_pending = false;  // the fast epilogue's stores of the previous tile
  for (;;) {
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    core.first_fragments(stores_pending);
    // Two stages per step; the step that issues the last loads of this tile's
    // stages (the last one) first points the loaders at the next tile.
    auto k_step = [&](auto first_c, int kt) {
      if (kt + 2 == KT2) {
        idx += slots;
        const bool more = idx < count;
        if (more) tile_coords(first + idx, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
        core.retarget(g, batch, tile_m * BM, tile_n * BN, more);
      }
      // stage numbers restart at 0 for the next tile
      core.template k_pair<decltype(first_c)::value>(kt + 2 == KT2 ? -2 : kt, stores_pending, [&] {
        if (FAST_ONLY || g.fast_epi) ScaleStager::issue<MT, NT>(g, batch, m0 + wm, n0 + wn, stage);
      });
    };
    k_step(std::true_type{}, 0);
    for (int kt = 2; kt < KT2; kt += 2) k_step(std::false_type{}, kt);
    if (FAST_ONLY || g.fast_epi) {
      epilogue_bf16_fast_any<MT, NT, true, !FAST_ONLY>(g, batch, core.acc, m0 + wm, n0 + wn, stage, scalars);
      // A store whose lanes are all past M or N completes at once and must not be counted as
      // outstanding: after a tile on the matrix edge the next tile waits for everything.
      stores_pending = m0 + BM <= g.M && n0 + BN <= g.N;
    } else {
      epilogue<MT, NT>(g, batch, core.acc, m0 + wm, n0 + wn, stage);
    }
    if (idx >= count) break;
    core.set_lane_addresses(g);
  }
  // drain the (out-of-range) loads issued for the tile that does not exist
  __builtin_amdgcn_s_waitcnt(0);
}

// WN: waves along n (the workgroup has 2 x WN); FAST_ONLY: the kernel carries
// the fast bf16 epilogue alone, without an accumulate input: the launch must
// satisfy epilogue_fast_ok() and have no D.
// WGS_PER_CU: workgroups of the persistent grid per compute unit (2 where the
// kernel's LDS and registers let two be resident).
template <int BM, int BN, int WN, bool FAST_ONLY, bool AK, bool BK_, int FA, int FB, int WGS_PER_CU = 1>
void launch_tile(const GemmArgs& g, int64_t batch, hipStream_t st) {
  GemmArgs a = g;
  a.tiles_m = (g.M + BM - 1) / BM;
  a.tiles_n = (g.N + BN - 1) / BN;
  const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
  const int cus = compute_units() * WGS_PER_CU;
  dim3 grid((unsigned)(tiles < cus ? tiles : cus), (unsigned)batch);
  fp8_gemm_tile_kernel<BM, BN, WN, AK, BK_, FA, FB, FAST_ONLY><<<grid, kWavesM * WN * 64, 0, st>>>(a);
}

// A K-major / B K-major etc.; defined in gemm_inst_*.hip
void launch_gemm_kk(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_km(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_mk(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);
void launch_gemm_mm(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st);

}  // namespace mi355q
