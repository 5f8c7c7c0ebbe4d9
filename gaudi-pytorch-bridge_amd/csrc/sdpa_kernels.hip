// fp8 scaled-dot-product attention (inference forward) for gfx950 and its C entry point.
//
// out = softmax(q k^T * scale + mask) v with q, k, v in fp8, an online softmax over blocks of 64
// keys, the probabilities quantised to fp8 before the second product, fp32 accumulation.
//
// Work split.  A workgroup of four waves owns 128 query rows of one (batch, head); a wave owns 32
// of them for the whole key loop.  Both products run on v_mfma_f32_32x32x64_f8f6f4 and both are
// issued transposed, keys (then columns of v) as the first operand and queries as the second:
//     S^T [64 keys, 32 queries]  = K_blk  Q^T        (two 32-key tiles, head_dim_qk / 64 steps)
//     O^T [dv,      32 queries] += V_blk^T P^T       (dv / 32 tiles, one step over the 64 keys)
// The MFMA leaves a lane with one query (lane % 32) and, per 32-row tile, the rows 8 j + 4 (lane /
// 32) + i of the first operand in register 4 j + i.  A query's row statistics are therefore
// per-lane values (one exchange between the two half-waves), rescaling O is a per-lane multiply,
// and the 32 probabilities a lane holds after S^T are, converted to fp8 and packed in register
// order, exactly the 32 k-slots of the second MFMA's second operand for that lane: P never passes
// through LDS.  The k-slot s = 16 t + 4 j + i of half-wave h then stands for key 32 t + 8 j + 4 h + i,
// and the V^T fragment is gathered from LDS in the same key order by the transposing reads
// (ds_read_b64_tr_b8 takes each of its 8 k-rows from its own address).
//
// K and V blocks are double buffered in LDS, one barrier per block.  Aligned tensors (16-byte
// rows and head dimensions) go global -> LDS directly (buffer_load ... lds: the loads of block
// i + 1 are issued before the arithmetic of block i and waited for after it, and cost the waves
// neither registers nor vector instructions); anything else goes through registers, byte by
// byte where it must.  Rows are XOR-swizzled so that the fragment reads are bank-conflict free;
// for the direct loads the swizzle is applied on the global side (which chunk a lane fetches),
// since such a load fixes the LDS position of each lane's 16 bytes.
#include <type_traits>

#include "device_common.h"

namespace mi355q {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define SDPA_LDS_AS __attribute__((address_space(3)))

constexpr int kSdpaThreads = 256;
constexpr int kSdpaBM = 128;  // query rows per workgroup
constexpr int kSdpaBN = 64;   // keys per block
constexpr float kLog2e = 1.44269504088896341f;

enum { kMaskNone = MI355Q_SDPA_MASK_NONE, kMaskBool = MI355Q_SDPA_MASK_BOOL, kMaskBf16 = MI355Q_SDPA_MASK_BF16, kMaskF32 = MI355Q_SDPA_MASK_F32 };

struct SdpaArgs {
  const uint8_t* q;
  const uint8_t* k;
  const uint8_t* v;
  const uint8_t* mask;
  uint8_t* out;
  int64_t bdim[3];
  int64_t q_bs[3], k_bs[3], v_bs[3], m_bs[3], o_bs[3];
  int64_t ldq, ldk, ldv, ldm, ldo;
  int L, S, Dk, Dv;
  int mask_kind, causal, out_fp8;
  int vec_q, vec_k, vec_v, vec_o;  // 16-byte (q, k, v) / 4-element (out) accesses are possible
  int dma;                         // k and v go global -> LDS directly
  int nqb;                         // query blocks per (batch, head)
  float scale;
  const float* sc_dev[6];  // d_scale_q, d_scale_k, d_scale_v, q_scale_s, q_scale_o, d_scale_s
  float sc_host[6];        // used where sc_dev is null; 0 = absent
  float* amax_s;
  float* amax_o;
  // the few-queries kernel only
  int pack;         // rows of the tile are (innermost batch index, query): k and v are shared along that dimension
  int rows;         // rows of the tile that hold a query
  int nsplit, blocks_per_split;
  float* ws;        // partial results of the key splits when nsplit > 1
  uint32_t* tickets;  // one arrival counter per group, zero between launches
  // keys a batch entry may attend to: valid_len[b] of them, the last ones (left padding) or the first ones
  // (right padding), b the index along batch dimension valid_dim; null = all S keys
  const int32_t* valid_len;
  int valid_dim, pad_left;
};

__device__ __forceinline__ float sdpa_scale(const SdpaArgs& a, int i, float absent) {
  if (a.sc_dev[i] != nullptr) return *a.sc_dev[i];
  return a.sc_host[i] != 0.0f ? a.sc_host[i] : absent;
}

// LDS offset of 16-byte chunk `chunk` of K row `row` (ROW_BYTES per row).  The 16 lanes of one
// ds_read_b128 cycle read one chunk column of 16 consecutive rows: the XOR sends them to 16
// different 16-byte slots modulo 256 bytes.
template <int ROW_BYTES>
__device__ __forceinline__ int k_lds_offset(int row, int chunk) {
  int sw;
  if constexpr (ROW_BYTES == 64) sw = (row >> 2) & 3;
  else if constexpr (ROW_BYTES == 128) sw = (row >> 1) & 7;
  else sw = row & 15;
  return row * ROW_BYTES + ((chunk ^ sw) << 4);
}

// V rows are 128 or 256 bytes.  A transposing read covers, per cycle, two 16-lane groups (adjacent
// chunks) times the 8 keys 8 (2 p' + r / 4) + 4 h + r % 4, r = 0..7: bits 3, 1 and 0 of the key tell
// them apart.  With 256-byte rows, XORing twice that 3-bit number into the chunk index gives 8 slots
// of one parity; with 128-byte rows two rows share 256 bytes, bit 0 of the key already separates
// them, and bits 1 and 3 go into the chunk index.
template <int ROW_BYTES>
__device__ __forceinline__ int v_swizzle(int row) {
  if constexpr (ROW_BYTES == 256) return ((((row >> 3) & 1) << 2) | (row & 3)) << 1;
  else return ((((row >> 3) & 1) << 1) | ((row >> 1) & 1)) << 1;
}
template <int ROW_BYTES>
__device__ __forceinline__ int v_lds_offset(int row, int chunk) {
  return row * ROW_BYTES + ((chunk ^ v_swizzle<ROW_BYTES>(row)) << 4);
}
template <int ROW_BYTES>
__device__ __forceinline__ int k_swizzle(int row) {
  if constexpr (ROW_BYTES == 64) return (row >> 2) & 3;
  else if constexpr (ROW_BYTES == 128) return (row >> 1) & 7;
  else return row & 15;
}

// One 16-byte piece per lane, global -> LDS (lane l lands at lds_dst + 16 l; a lane whose offset lies
// outside the descriptor writes zeros).  The s_nop covers descriptor words that reached their scalar
// registers through a vector instruction (five wait states before a memory instruction may read them).
// STREAM adds the nontemporal hint: for keys and values that the launch reads once (the decoding kernel).
template <bool STREAM = false>
__device__ __forceinline__ void sdpa_dma16(const i32x4& rsrc, int voff, uint32_t lds_dst) {
  if constexpr (STREAM) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
  } else {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
  }
}

// A buffer descriptor that walks down the rows of k or v one block at a time.
struct SdpaWalker {
  uint64_t base;
  int64_t left;  // bytes from base to the end of the tensor's rows; <= 0: every load reads zeros
  __device__ __forceinline__ i32x4 rsrc() const {
    int64_t rec = left < 0 ? 0 : (left > 0x7ffffff0LL ? 0x7ffffff0LL : left);
    i32x4 r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)base);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((base >> 32) & 0xffffu));
    r[2] = __builtin_amdgcn_readfirstlane((int)rec);
    r[3] = 0x00020000;
    return r;
  }
};

// 16 bytes of a row of q / k / v starting at byte column d (zero beyond the row's D bytes and for
// rows outside the tensor).  VEC: the row start and D are multiples of 16.
__device__ __forceinline__ u32x4 load_chunk(const uint8_t* row_ptr, bool row_ok, int d, int D, bool vec) {
  u32x4 r = {0u, 0u, 0u, 0u};
  if (!row_ok || d >= D) return r;
  if (vec) return *reinterpret_cast<const u32x4*>(row_ptr + d);
#pragma unroll
  for (int b = 0; b < 16; ++b) {
    const uint32_t byte = (d + b < D) ? row_ptr[d + b] : 0u;
    r[b >> 2] |= byte << (8 * (b & 3));
  }
  return r;
}

template <int FMT>
__device__ __forceinline__ f32x16 sdpa_mfma(const i32x8& first, const i32x8& second, const f32x16& acc) {
  constexpr int code = FMT == MI355Q_E5M2 ? 1 : 0;
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(first, second, acc, code, code, 0, 0, 0, 0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__global__ void sdpa_clear_amax_kernel(float* a, float* b) {
  if (a != nullptr) *a = 0.0f;
  if (b != nullptr) *b = 0.0f;
}

// One block of 64 keys for a wave's 32 query rows: S^T = K Q^T from the K tile at kb, masks, the
// online-softmax update of (m_run, l_run, o), and O^T += V^T P^T from the V tile at vb.  qpos is the
// lane's query position (for the causal comparison), mrow its row of the mask; `edge` says that some
// score of the block may need masking (wave-uniform), otherwise the cheap path runs.
template <int DKC, int DVT, int FMT, bool QL = false>
__device__ __forceinline__ void sdpa_block(const SdpaArgs& a, const uint8_t* kb, const uint8_t* vb, int kv0, bool edge, int qpos,
                                           bool q_ok, const uint8_t* mrow, const i32x8 (&qf)[DKC], float sc2, float lqs, bool clamp_p,
                                           f32x16 (&o)[DVT], float& m_run, float& l_run, const uint8_t* qbase = nullptr,
                                           int klo = 0, int khi = 0x7fffffff) {
  constexpr int KROW = DKC * 64;
  constexpr int kVRow = DVT <= 4 ? 128 : 256;
  constexpr float kMax8 = FMT == MI355Q_E5M2 ? 57344.0f : 448.0f;
  const int lane = threadIdx.x & 63, lq = lane & 31, h = lane >> 5;
  f32x16 s[2];
  if constexpr (QL) {
    // the query fragments come from LDS, one depth step at a time (registers for a third wave per SIMD)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[t][r] = 0.0f;
#pragma unroll
    for (int c = 0; c < DKC; ++c) {
      const u32x4 qlo = *reinterpret_cast<const u32x4*>(qbase + (c * 2) * 1024);
      const u32x4 qhi = *reinterpret_cast<const u32x4*>(qbase + (c * 2 + 1) * 1024);
      const i32x8 q = {(int)qlo[0], (int)qlo[1], (int)qlo[2], (int)qlo[3], (int)qhi[0], (int)qhi[1], (int)qhi[2], (int)qhi[3]};
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int row = 32 * t + lq;
        const u32x4 lo = *reinterpret_cast<const u32x4*>(kb + k_lds_offset<KROW>(row, c * 4 + h * 2));
        const u32x4 hi = *reinterpret_cast<const u32x4*>(kb + k_lds_offset<KROW>(row, c * 4 + h * 2 + 1));
        const i32x8 kf = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        s[t] = sdpa_mfma<FMT>(kf, q, s[t]);
      }
    }
  } else {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) s[t][r] = 0.0f;
#pragma unroll
    for (int c = 0; c < DKC; ++c) {
      const int row = 32 * t + lq;
      const u32x4 lo = *reinterpret_cast<const u32x4*>(kb + k_lds_offset<KROW>(row, c * 4 + h * 2));
      const u32x4 hi = *reinterpret_cast<const u32x4*>(kb + k_lds_offset<KROW>(row, c * 4 + h * 2 + 1));
      const i32x8 kf = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      s[t] = sdpa_mfma<FMT>(kf, qf[c], s[t]);
    }
  }
  }

  // The V fragments do not depend on the scores: for up to four tiles their LDS reads go out here, under the
  // score MFMAs and the softmax, instead of one tile at a time in front of each P V product (where the wave
  // would wait for LDS four times with the matrix pipe idle).
  const int g = lane >> 4, gi = lane & 15;
  const int r8 = gi >> 1, hh = gi & 1;
  constexpr bool kEarlyV = DVT <= 4 && !QL;
  i32x8 vfe[kEarlyV ? DVT : 1];
  if constexpr (kEarlyV) {
#pragma unroll
    for (int t = 0; t < DVT; ++t) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int krow = 32 * (p >> 1) + 8 * (2 * (p & 1) + (r8 >> 2)) + 4 * h + (r8 & 3);
        const int off = v_lds_offset<kVRow>(krow, 2 * t + (g & 1)) + hh * 8;
        const i32x2 w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((SDPA_LDS_AS i32x2*)((SDPA_LDS_AS uint8_t*)vb + off));
        vfe[t][2 * p] = w[0];
        vfe[t][2 * p + 1] = w[1];
      }
    }
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int t = 0; t < DVT; ++t) asm volatile("" : "+v"(vfe[t]));  // the reads are issued here, not sunk to their use
#endif
  }

  // scores in units of log2, masks applied
  float mx = -__builtin_inff();
  if (!edge && sc2 >= 0.0f) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = __builtin_fmaxf(mx, s[t][r]);
    mx *= sc2;
  } else {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kv = kv0 + 32 * t + 8 * (r >> 2) + 4 * h + (r & 3);
        float x = s[t][r] * sc2;
        bool dead = kv >= a.S || kv >= khi || kv < klo || (a.causal && kv > qpos);
        if (a.mask_kind != kMaskNone && q_ok && kv < a.S) {
          if (a.mask_kind == kMaskBool) dead = dead || mrow[kv] == 0;
          else if (a.mask_kind == kMaskBf16) x += bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(mrow)[kv]) * kLog2e;
          else x += reinterpret_cast<const float*>(mrow)[kv] * kLog2e;
        }
        x = dead ? -__builtin_inff() : x;
        s[t][r] = x;
        mx = __builtin_fmaxf(mx, x);
      }
  }
  {  // the other half-wave's maximum for the same query row: a swap of register halves, no trip through LDS
    typedef unsigned u32x2v __attribute__((ext_vector_type(2)));
    const u32x2v sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
    mx = __builtin_fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
  }
  const float m_new = __builtin_fmaxf(m_run, mx);
  const float m_use = m_new == -__builtin_inff() ? 0.0f : m_new;
  const float alpha = fast_exp2(m_run - m_use);
  m_run = m_new;
  const float shift = lqs - m_use;  // p * q_scale_s = 2^(x - m + log2 q_scale_s)

  float psum = 0.0f;
  i32x8 pf = {0, 0, 0, 0, 0, 0, 0, 0};
  // p = 2^(x + shift) for this lane's 32 scores, their sum, and the fp8 codes packed in register
  // order.  RAW: s still holds the unscaled products (x = s * sc2); CLAMP: q_scale_s exceeds the
  // format's range.  Compile-time variants, so that the common one is a multiply-add, an exp2 and an
  // add per score.
  auto exponentials = [&](auto rawc, auto clampc) {
    constexpr bool RAW = decltype(rawc)::value, CLAMP = decltype(clampc)::value;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float x = s[t][4 * j + i];
          p[i] = fast_exp2(RAW ? __builtin_fmaf(x, sc2, shift) : x + shift);
          psum += p[i];
          if (CLAMP) p[i] = __builtin_elementwise_minimum(p[i], kMax8);
        }
        // Both halves of the word are written, so what it held before does not matter: the empty statement
        // makes it "defined" for the compiler at no cost, where a zero would cost a move per word.
        int w = 0;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "=v"(w));
#endif
        if constexpr (FMT == MI355Q_E5M2) {
          w = __builtin_amdgcn_cvt_pk_bf8_f32(p[0], p[1], w, false);
          w = __builtin_amdgcn_cvt_pk_bf8_f32(p[2], p[3], w, true);
        } else {
          w = __builtin_amdgcn_cvt_pk_fp8_f32(p[0], p[1], w, false);
          w = __builtin_amdgcn_cvt_pk_fp8_f32(p[2], p[3], w, true);
        }
        pf[4 * t + j] = w;
      }
  };
  const bool raw = !edge && sc2 >= 0.0f;  // s still holds the unscaled products
  if (raw && !clamp_p) exponentials(std::true_type{}, std::false_type{});
  else if (raw) exponentials(std::true_type{}, std::true_type{});
  else if (!clamp_p) exponentials(std::false_type{}, std::false_type{});
  else exponentials(std::false_type{}, std::true_type{});
  l_run = l_run * alpha + psum;

  // With the queries in LDS (three workgroups per CU, no registers for V fragments during the softmax) the V fragments
  // are read here: the 32 score registers are dead, and the reads' latency passes under the rescaling of O instead of
  // standing in front of each P V product.
  constexpr bool kMidV = DVT <= 4 && QL;
  i32x8 vfm[kMidV ? DVT : 1];
  if constexpr (kMidV) {
#pragma unroll
    for (int t = 0; t < DVT; ++t) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int krow = 32 * (p >> 1) + 8 * (2 * (p & 1) + (r8 >> 2)) + 4 * h + (r8 & 3);
        const int off = v_lds_offset<kVRow>(krow, 2 * t + (g & 1)) + hh * 8;
        const i32x2 w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((SDPA_LDS_AS i32x2*)((SDPA_LDS_AS uint8_t*)vb + off));
        vfm[t][2 * p] = w[0];
        vfm[t][2 * p + 1] = w[1];
      }
    }
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int t = 0; t < DVT; ++t) asm volatile("" : "+v"(vfm[t]));  // issued here, not sunk to their use
#endif
  }

  if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
    for (int t = 0; t < DVT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
  }

  // O^T += V^T P^T; k-slot 8 p + r' of half-wave h is key 32 (p / 2) + 8 (2 (p % 2) + r' / 4) + 4 h + r' % 4
#pragma unroll
  for (int t = 0; t < DVT; ++t) {
    if constexpr (kEarlyV) {
      o[t] = sdpa_mfma<FMT>(vfe[t], pf, o[t]);
      continue;
    }
    if constexpr (kMidV) {
      o[t] = sdpa_mfma<FMT>(vfm[t], pf, o[t]);
      continue;
    }
    i32x8 vf;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int krow = 32 * (p >> 1) + 8 * (2 * (p & 1) + (r8 >> 2)) + 4 * h + (r8 & 3);
      const int off = v_lds_offset<kVRow>(krow, 2 * t + (g & 1)) + hh * 8;
      const i32x2 w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((SDPA_LDS_AS i32x2*)((SDPA_LDS_AS uint8_t*)vb + off));
      vf[2 * p] = w[0];
      vf[2 * p + 1] = w[1];
    }
    o[t] = sdpa_mfma<FMT>(vf, pf, o[t]);
  }
}

// Head dimension 128 with direct loads: the query fragments live in LDS instead of 16 registers and the ring has
// two stages instead of four, which brings a workgroup to 161 registers and 48 KB of LDS, so that three
// workgroups fit a CU (three waves per SIMD).  A wave alone needs about 3500 cycles for a block of 64 keys (a
// chain of LDS reads, MFMAs, the softmax and MFMAs again) of which 1200 are vector work and 512 MFMA time, so a
// SIMD is as busy as it has waves to switch between.
constexpr bool sdpa_q_in_lds(int dkc, int dvt, bool dma) { return dma && dkc == 2 && dvt == 4; }
// Workgroups per CU the kernel is compiled for.  Head dimension 256 (eight tiles of O: 128 registers) fits two with the
// direct loads and a ring of two stages (255 registers, 64 KiB of LDS): 850 -> 1765 TFLOP/s at 32 / 8 heads and 8192
// causal tokens against one workgroup with four stages.  Through registers (unaligned tensors) the same bound spills
// 216 bytes per lane, so that form stays at one.
constexpr int sdpa_workgroups_per_cu(int dkc, int dvt, bool dma) { return sdpa_q_in_lds(dkc, dvt, dma) ? 3 : (dvt <= 4 || dma) ? 2 : 1; }

// DKC: 64-byte steps of the q.k depth (head_dim_qk <= 64 DKC); DVT: 32-column tiles of v
// (head_dim_v <= 32 DVT).
// DMA: K and V blocks go from global memory straight into LDS (aligned tensors), a ring of kStages blocks;
// otherwise through registers, two buffers.  A compile-time choice: with both routes in one loop the compiler
// has to assume the register route's loads outstanding wherever their registers are reused, and the wait it
// puts there (vmcnt(0), in front of the first MFMA of every block) also waits for the blocks just requested
// by the direct route.
template <int DKC, int DVT, int FMT, bool DMA>
__global__ __launch_bounds__(kSdpaThreads, sdpa_workgroups_per_cu(DKC, DVT, DMA)) void fp8_sdpa_fwd_kernel(const SdpaArgs a) {
  constexpr bool kQLds = sdpa_q_in_lds(DKC, DVT, DMA);
  constexpr int KROW = DKC * 64;
  constexpr int kVRow = DVT <= 4 ? 128 : 256;  // bytes of an LDS row of V
  constexpr int KCPR = KROW / 16;           // chunks per K row
  constexpr int VCPR = DVT * 2;             // chunks per V row that carry data
  constexpr int KBYTES = kSdpaBN * KROW;
  constexpr int VBYTES = kSdpaBN * kVRow;
  constexpr int KLOADS = kSdpaBN * KCPR / kSdpaThreads;  // 16-byte loads per thread and block
  constexpr int VLOADS = kSdpaBN * VCPR / kSdpaThreads;
  static_assert(KLOADS >= 1 && VLOADS >= 1, "block too small for the workgroup");
  // Direct loads run kStages - 1 blocks ahead of the arithmetic (a block's arithmetic takes about a
  // microsecond, less than a load from HBM under load; with the queries in LDS one block ahead, which the
  // third workgroup on the CU covers, and at head dimension 256, where two stages are what leaves room for a second
  // workgroup); the route through registers uses two buffers.
  constexpr int kStages = (kQLds || DVT > 4) ? 2 : 4;
  __shared__ __align__(1024) uint8_t lds[kStages * (KBYTES + VBYTES)];
  __shared__ __align__(16) uint8_t qlds[kQLds ? 4 * 4096 : 16];  // per wave: [depth chunk of 16 bytes][half-wave][row]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in every lane, and known to be
  const int lq = lane & 31, h = lane >> 5;

  // Workgroups go to the 8 XCDs round robin: give each XCD a contiguous range of (batch, head,
  // query block), so that the query blocks that share a K and V meet in one L2.
  int id = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
  int64_t bi = id / a.nqb;
  const int qb = a.nqb - 1 - (id - (int)bi * a.nqb);  // under a causal mask the long rows start first
  int64_t q_off = 0, k_off = 0, v_off = 0, m_off = 0, o_off = 0;
  int64_t b_valid = 0;
#pragma unroll
  for (int d = 2; d >= 0; --d) {
    const int64_t b = bi % a.bdim[d];
    bi /= a.bdim[d];
    q_off += b * a.q_bs[d];
    k_off += b * a.k_bs[d];
    v_off += b * a.v_bs[d];
    m_off += b * a.m_bs[d];
    o_off += b * a.o_bs[d];
    if (d == a.valid_dim) b_valid = b;
  }
  const uint8_t* qp = a.q + q_off;
  const uint8_t* kp = a.k + k_off;
  const uint8_t* vp = a.v + v_off;
  // the window of keys this batch entry may attend to
  int klo = 0, khi = a.S;
  if (a.valid_len != nullptr) {
    int n = a.valid_len[b_valid];
    n = n < 0 ? 0 : (n > a.S ? a.S : n);
    n = __builtin_amdgcn_readfirstlane(n);
    if (a.pad_left) klo = a.S - n;
    else khi = n;
  }

  const int q0 = qb * kSdpaBM;
  const int wq0 = q0 + wave * 32;  // first query row of this wave
  const int qrow = wq0 + lq;
  const bool q_ok = qrow < a.L;

  const float dq = sdpa_scale(a, 0, 1.0f), dk = sdpa_scale(a, 1, 1.0f), dv = sdpa_scale(a, 2, 1.0f);
  const float qs = sdpa_scale(a, 3, 1.0f);
  const float ds = sdpa_scale(a, 5, 1.0f / qs);
  const float sc2 = a.scale * dq * dk * kLog2e;
  const float lqs = __builtin_log2f(qs);
  constexpr float kMax8 = FMT == MI355Q_E5M2 ? 57344.0f : 448.0f;
  const bool clamp_p = !(qs <= kMax8);

  // this lane's query fragments: 32 bytes of depth per 64-byte step
  i32x8 qf[DKC];
#pragma unroll
  for (int c = 0; c < DKC; ++c) {
    const uint8_t* rp = qp + (int64_t)qrow * a.ldq;
    const u32x4 lo = load_chunk(rp, q_ok, 64 * c + 32 * h, a.Dk, a.vec_q);
    const u32x4 hi = load_chunk(rp, q_ok, 64 * c + 32 * h + 16, a.Dk, a.vec_q);
    qf[c] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  }
  // The fragments are first used by an MFMA inside the block loop, and the wait for their loads would be placed
  // there: a vmcnt(0) in every pass, which also waits for the K / V blocks just requested.  Naming them here
  // puts that wait in front of the loop.
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass, which compiles this body for the launch stub, knows no "v"
#pragma unroll
  for (int c = 0; c < DKC; ++c) asm volatile("" : : "v"(qf[c]));
#endif
  const uint8_t* qbase = qlds + (kQLds ? wave * 4096 + h * 512 + lq * 16 : 0);
  if constexpr (kQLds) {
#pragma unroll
    for (int c = 0; c < DKC; ++c) {
      *reinterpret_cast<u32x4*>(qlds + wave * 4096 + (c * 2) * 1024 + h * 512 + lq * 16) =
          u32x4{(uint32_t)qf[c][0], (uint32_t)qf[c][1], (uint32_t)qf[c][2], (uint32_t)qf[c][3]};
      *reinterpret_cast<u32x4*>(qlds + wave * 4096 + (c * 2 + 1) * 1024 + h * 512 + lq * 16) =
          u32x4{(uint32_t)qf[c][4], (uint32_t)qf[c][5], (uint32_t)qf[c][6], (uint32_t)qf[c][7]};
    }
  }

  // blocks blk0 .. nblk - 1 hold the keys of the window
  int nblk = (khi + kSdpaBN - 1) / kSdpaBN;
  if (a.causal) {
    const int last_q = (q0 + kSdpaBM < a.L ? q0 + kSdpaBM : a.L) - 1;
    const int lim = last_q / kSdpaBN + 1;  // blocks that hold a key <= the last query row
    nblk = nblk < lim ? nblk : lim;
  }
  const int blk0 = klo / kSdpaBN < nblk ? klo / kSdpaBN : nblk;

  u32x4 kreg[KLOADS], vreg[VLOADS];
  auto fetch = [&](int blk) {
    const int kv0 = blk * kSdpaBN;
#pragma unroll
    for (int n = 0; n < KLOADS; ++n) {
      const int ci = tid + n * kSdpaThreads;
      const int row = ci / KCPR, chunk = ci % KCPR;
      kreg[n] = load_chunk(kp + (int64_t)(kv0 + row) * a.ldk, kv0 + row < a.S, chunk * 16, a.Dk, a.vec_k);
    }
#pragma unroll
    for (int n = 0; n < VLOADS; ++n) {
      const int ci = tid + n * kSdpaThreads;
      const int row = ci / VCPR, chunk = ci % VCPR;
      vreg[n] = load_chunk(vp + (int64_t)(kv0 + row) * a.ldv, kv0 + row < a.S, chunk * 16, a.Dv, a.vec_v);
    }
  };
  auto commit = [&](int buf) {
    uint8_t* kb = lds + buf * (KBYTES + VBYTES);
    uint8_t* vb = kb + KBYTES;
#pragma unroll
    for (int n = 0; n < KLOADS; ++n) {
      const int ci = tid + n * kSdpaThreads;
      *reinterpret_cast<u32x4*>(kb + k_lds_offset<KROW>(ci / KCPR, ci % KCPR)) = kreg[n];
    }
#pragma unroll
    for (int n = 0; n < VLOADS; ++n) {
      const int ci = tid + n * kSdpaThreads;
      *reinterpret_cast<u32x4*>(vb + v_lds_offset<kVRow>(ci / VCPR, ci % VCPR)) = vreg[n];
    }
  };

  // Direct loads: the K tile is KBYTES / 1024 regions of 1 KiB (one wave-wide load each), the V tile
  // VBYTES / 1024; a wave takes every fourth.  The lane's offsets inside a block never change; the
  // descriptors walk down the rows.
  constexpr int KREG = KBYTES / 1024 / 4, VREG = VBYTES / 1024 / 4;  // regions per wave
  static_assert(KBYTES % 4096 == 0 && VBYTES % 4096 == 0, "tiles split into 1 KiB regions over four waves");
  int kvoff[KREG], vvoff[VREG];
  SdpaWalker wk{reinterpret_cast<uint64_t>(kp), 0}, wv{reinterpret_cast<uint64_t>(vp), 0};
  if constexpr (DMA) {
    wk.base += (uint64_t)blk0 * kSdpaBN * a.ldk;
    wv.base += (uint64_t)blk0 * kSdpaBN * a.ldv;
    wk.left = (int64_t)(a.S - 1 - blk0 * kSdpaBN) * a.ldk + a.Dk;
    wv.left = (int64_t)(a.S - 1 - blk0 * kSdpaBN) * a.ldv + a.Dv;
#pragma unroll
    for (int n = 0; n < KREG; ++n) {
      const int pos = (wave * KREG + n) * 64 + lane;  // 16-byte slot of the tile this lane fills
      const int row = pos / KCPR, chunk = (pos % KCPR) ^ k_swizzle<KROW>(pos / KCPR);
      kvoff[n] = chunk * 16 < a.Dk ? row * (int)a.ldk + chunk * 16 : 0x7fffffff;
    }
#pragma unroll
    for (int n = 0; n < VREG; ++n) {
      const int pos = (wave * VREG + n) * 64 + lane;
      const int row = pos / (kVRow / 16), chunk = (pos % (kVRow / 16)) ^ v_swizzle<kVRow>(pos / (kVRow / 16));
      vvoff[n] = chunk * 16 < a.Dv ? row * (int)a.ldv + chunk * 16 : 0x7fffffff;
    }
  }
  // the loads of the next block into buffer `buf`; the descriptors then move on by one block
  auto issue_block = [&](int buf) {
    const uint32_t kdst = (uint32_t)(uintptr_t)(SDPA_LDS_AS uint8_t*)(lds + buf * (KBYTES + VBYTES));
    const i32x4 rk = wk.rsrc();
#pragma unroll
    for (int n = 0; n < KREG; ++n) sdpa_dma16(rk, kvoff[n], kdst + (wave * KREG + n) * 1024);
    const i32x4 rv = wv.rsrc();
#pragma unroll
    for (int n = 0; n < VREG; ++n) sdpa_dma16(rv, vvoff[n], kdst + KBYTES + (wave * VREG + n) * 1024);
    wk.base += (uint64_t)kSdpaBN * a.ldk;
    wk.left -= (int64_t)kSdpaBN * a.ldk;
    wv.base += (uint64_t)kSdpaBN * a.ldv;
    wv.left -= (int64_t)kSdpaBN * a.ldv;
  };

  f32x16 o[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.0f;
  float m_run = -__builtin_inff();  // running maximum of the scaled scores, in units of log2
  float l_run = 0.0f;               // this half-wave's share of the running sum (times q_scale_s)

  const uint8_t* mrow = a.mask + (m_off + (int64_t)qrow * a.ldm) * (a.mask_kind == kMaskBool ? 1 : a.mask_kind == kMaskBf16 ? 2 : 4);
  // ring positions count from the window's first block
  if (nblk > blk0) {
    if constexpr (DMA) {
      for (int b = 0; b < kStages - 1 && blk0 + b < nblk; ++b) issue_block(b);
      if (nblk - blk0 >= kStages - 1 && (blk0 + kStages - 1) * kSdpaBN <= a.S) {
        constexpr int cnt = (kStages - 2) * (KREG + VREG);
        __builtin_amdgcn_s_waitcnt((cnt & 15) | ((cnt >> 4) << 14) | 0x0f70);  // the first block has landed
      } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      }
    } else {
      fetch(blk0);
      commit(0);
    }
  }
  __syncthreads();

  for (int blk = blk0; blk < nblk; ++blk) {
    const int kv0 = blk * kSdpaBN;
    const int pos = blk - blk0;
    if constexpr (DMA) {
      if (blk + kStages - 1 < nblk) issue_block((pos + kStages - 1) % kStages);
    } else {
      if (blk + 1 < nblk) fetch(blk + 1);
    }
    const uint8_t* kb = lds + (DMA ? pos % kStages : pos & 1) * (KBYTES + VBYTES);
    const uint8_t* vb = kb + KBYTES;

    // a wave whose 32 rows all lie above this block's first key has nothing to add
    const bool active = !(a.causal && kv0 > wq0 + 31);
    if (active) {
      const bool edge = (a.causal && kv0 + kSdpaBN - 1 > wq0) || kv0 + kSdpaBN > khi || kv0 < klo || a.mask_kind != kMaskNone;
      sdpa_block<DKC, DVT, FMT, kQLds>(a, kb, vb, kv0, edge, qrow, q_ok, mrow, qf, sc2, lqs, clamp_p, o, m_run, l_run, qbase, klo, khi);
    }

    if constexpr (DMA) {
      // The next block has landed once only the loads of the blocks after it are outstanding.  Loads
      // retire in issue order as long as every one of them goes to memory; one whose lanes all lie
      // beyond kv_len completes at once, so the count is only trusted while every block in flight is
      // whole, and the tail drains everything.
      if (blk + kStages <= nblk && (blk + kStages) * kSdpaBN <= a.S) {
        constexpr int cnt = (kStages - 2) * (KREG + VREG);
        __builtin_amdgcn_s_waitcnt((cnt & 15) | ((cnt >> 4) << 14) | 0x0f70);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);
      }
    } else {
      if (blk + 1 < nblk) commit((pos + 1) & 1);
    }
    __syncthreads();
  }

  // out = O * d_scale_s * d_scale_v / l.  l_run carries the factor q_scale_s that p did.
  const float l_tot = (l_run + __shfl_xor(l_run, 32, 64)) / qs;
  const float inv_l = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  const float f = inv_l * (ds * dv);
  const float qo = a.out_fp8 ? sdpa_scale(a, 4, 1.0f) : 1.0f;
  float amax_o = 0.0f;
  uint8_t* orow = a.out + (o_off + (int64_t)qrow * a.ldo) * (a.out_fp8 ? 1 : 2);
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d0 = 32 * t + 8 * j + 4 * h;
      float val[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        val[i] = o[t][4 * j + i] * f;
        if (q_ok && d0 + i < a.Dv) amax_o = __builtin_fmaxf(amax_o, __builtin_fabsf(val[i]));
      }
      if (!q_ok || d0 >= a.Dv) continue;
      if (a.out_fp8) {
        const uint32_t w = cvt_fp8x4<MI355Q_E4M3FN>(val[0] * qo, val[1] * qo, val[2] * qo, val[3] * qo);
        if (a.vec_o) {
          *reinterpret_cast<uint32_t*>(orow + d0) = w;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (d0 + i < a.Dv) orow[d0 + i] = (uint8_t)(w >> (8 * i));
        }
      } else {
        const uint32_t w0 = pack_bf16x2(val[0], val[1]), w1 = pack_bf16x2(val[2], val[3]);
        if (a.vec_o) {
          *reinterpret_cast<u32x2*>(orow + 2 * d0) = u32x2{w0, w1};
        } else {
          uint16_t* o16 = reinterpret_cast<uint16_t*>(orow);
          const uint32_t ws[2] = {w0, w1};
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (d0 + i < a.Dv) o16[d0 + i] = (uint16_t)(ws[i >> 1] >> (16 * (i & 1)));
        }
      }
    }

  if (a.amax_s != nullptr) {
    // the largest probability of a row is the one at the row maximum: 1 / l
    const uint32_t m = wave_max_u32(__float_as_uint(q_ok ? inv_l : 0.0f));
    if (lane == 0 && m != 0u) atomicMax(reinterpret_cast<unsigned int*>(a.amax_s), m);
  }
  if (a.amax_o != nullptr) {
    const uint32_t m = wave_max_u32(__float_as_uint(amax_o));
    if (lane == 0 && m != 0u) atomicMax(reinterpret_cast<unsigned int*>(a.amax_o), m);
  }
}

// ------------------------------------------------------------------ few queries, many keys
//
// Decoding: a handful of queries per head against a long key / value cache.  The 128-row
// workgroups of the kernel above would hold one useful row each and every query head of a group
// would stream the group's K and V again.  Here the rows of one 32-row tile are all the queries
// that share a K and V -- (head of the group, query position) pairs, up to 32 -- and the keys are
// what is split: over `nsplit` workgroups, and inside a workgroup over its four waves, block by
// block.  Each wave streams its own blocks through LDS stages of its own (no barrier in the loop)
// and keeps its own running maximum, sum and O; the four are merged through LDS at the end, and
// the splits' results (unnormalised O, m, l per row) through a workspace by a second small kernel.

constexpr int kDecodeTileFloats(int DVT) { return 32 * DVT * 32 + 64; }  // O^T [dv][row], m[row], l[row]

// merges `n` partial results for row `row`, columns dv0, dv0 + dvstep, ...; returns the row's 1 / l
// (0 for a row with nothing to attend to) and leaves the merged, normalised values in `val`
template <int DVT>
__device__ __forceinline__ float sdpa_merge(const float* parts, int n, int stride_floats, int row, int dv0, int dvstep, float qs,
                                            float (&val)[DVT * 32 / 8]) {
  float M = -__builtin_inff();
  for (int w = 0; w < n; ++w) M = __builtin_fmaxf(M, parts[(int64_t)w * stride_floats + 32 * DVT * 32 + row]);
  float L = 0.0f;
#pragma unroll
  for (int i = 0; i < DVT * 32 / 8; ++i) val[i] = 0.0f;
  for (int w = 0; w < n; ++w) {
    const float* pw = parts + (int64_t)w * stride_floats;
    const float mw = pw[32 * DVT * 32 + row];
    const float wgt = mw == -__builtin_inff() ? 0.0f : fast_exp2(mw - M);
    L += pw[32 * DVT * 32 + 32 + row] * wgt;
#pragma unroll
    for (int i = 0; i < DVT * 32 / 8; ++i) val[i] += pw[(dv0 + i * dvstep) * 32 + row] * wgt;
  }
  const float l = L / qs;
  const float inv_l = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
  for (int i = 0; i < DVT * 32 / 8; ++i) val[i] *= inv_l;
  return inv_l;
}

// final scaling, rounding and store of one row's merged values (columns dv0 + i dvstep), amax updates
template <int DVT>
__device__ __forceinline__ void sdpa_store_row(const SdpaArgs& a, uint8_t* orow, bool row_ok, float inv_l, int dv0, int dvstep,
                                               const float (&val)[DVT * 32 / 8]) {
  const float dv = sdpa_scale(a, 2, 1.0f), qs = sdpa_scale(a, 3, 1.0f), ds = sdpa_scale(a, 5, 1.0f / qs);
  const float qo = a.out_fp8 ? sdpa_scale(a, 4, 1.0f) : 1.0f;
  float amax_o = 0.0f;
#pragma unroll
  for (int i = 0; i < DVT * 32 / 8; ++i) {
    const int d = dv0 + i * dvstep;
    const float v = val[i] * (ds * dv);
    if (row_ok && d < a.Dv) {
      amax_o = __builtin_fmaxf(amax_o, __builtin_fabsf(v));
      if (a.out_fp8) orow[d] = (uint8_t)(cvt_fp8x4<MI355Q_E4M3FN>(v * qo, 0.f, 0.f, 0.f) & 0xffu);
      else reinterpret_cast<uint16_t*>(orow)[d] = (uint16_t)(pack_bf16x2(v, 0.f) & 0xffffu);
    }
  }
  const int lane = threadIdx.x & 63;
  if (a.amax_s != nullptr) {
    const uint32_t m = wave_max_u32(__float_as_uint(row_ok ? inv_l : 0.0f));
    if (lane == 0 && m != 0u) atomicMax(reinterpret_cast<unsigned int*>(a.amax_s), m);
  }
  if (a.amax_o != nullptr) {
    const uint32_t m = wave_max_u32(__float_as_uint(amax_o));
    if (lane == 0 && m != 0u) atomicMax(reinterpret_cast<unsigned int*>(a.amax_o), m);
  }
}

// offsets of workgroup `g`'s tensors; with `pack` the innermost batch dimension stays inside the tile
__device__ __forceinline__ void sdpa_group_offsets(const SdpaArgs& a, int64_t g, int64_t& q_off, int64_t& k_off, int64_t& v_off,
                                                   int64_t& m_off, int64_t& o_off) {
  q_off = k_off = v_off = m_off = o_off = 0;
#pragma unroll
  for (int d = 2; d >= 0; --d) {
    if (d == 2 && a.pack) continue;
    const int64_t b = g % a.bdim[d];
    g /= a.bdim[d];
    q_off += b * a.q_bs[d];
    k_off += b * a.k_bs[d];
    v_off += b * a.v_bs[d];
    m_off += b * a.m_bs[d];
    o_off += b * a.o_bs[d];
  }
}

template <int DKC, int DVT, int FMT>
__global__ __launch_bounds__(kSdpaThreads) void fp8_sdpa_decode_kernel(const SdpaArgs a) {
  constexpr int KROW = DKC * 64;
  constexpr int kVRow = 128;
  static_assert(DVT <= 4, "256-byte V rows do not fit four waves' stages");
  constexpr int KCPR = KROW / 16;
  constexpr int KBYTES = kSdpaBN * KROW, VBYTES = kSdpaBN * kVRow;
  constexpr int KREG = KBYTES / 1024, VREG = VBYTES / 1024;  // regions per block, all loaded by the block's wave
  constexpr int kStage = KBYTES + VBYTES;
  constexpr int kOps = KREG + VREG;
  static_assert(kOps <= 63, "vmcnt holds 6 bits");
  static_assert(4 * kDecodeTileFloats(DVT) * 4 <= 4 * 2 * kStage, "the merge area overlays the stages");
  __shared__ __align__(1024) uint8_t lds[4 * 2 * kStage];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, h = lane >> 5;
  const int64_t grp = blockIdx.x / a.nsplit;
  const int split = blockIdx.x - (int)grp * a.nsplit;
  int64_t q_off, k_off, v_off, m_off, o_off;
  sdpa_group_offsets(a, grp, q_off, k_off, v_off, m_off, o_off);

  // this lane's row of the tile: (innermost batch index, query position)
  const int inner = a.pack ? lq / a.L : 0, qpos = a.pack ? lq - inner * a.L : lq;
  const bool q_ok = lq < a.rows;
  const uint8_t* qrowp = a.q + q_off + (int64_t)inner * a.q_bs[2] + (int64_t)qpos * a.ldq;
  const uint8_t* mrow = a.mask + (m_off + (int64_t)inner * a.m_bs[2] + (int64_t)qpos * a.ldm) *
                                     (a.mask_kind == kMaskBool ? 1 : a.mask_kind == kMaskBf16 ? 2 : 4);

  const float dq = sdpa_scale(a, 0, 1.0f), dk = sdpa_scale(a, 1, 1.0f);
  const float qs = sdpa_scale(a, 3, 1.0f);
  const float sc2 = a.scale * dq * dk * kLog2e;
  const float lqs = __builtin_log2f(qs);
  constexpr float kMax8 = FMT == MI355Q_E5M2 ? 57344.0f : 448.0f;
  const bool clamp_p = !(qs <= kMax8);

  i32x8 qf[DKC];
#pragma unroll
  for (int c = 0; c < DKC; ++c) {
    const u32x4 lo = load_chunk(qrowp, q_ok, 64 * c + 32 * h, a.Dk, a.vec_q);
    const u32x4 hi = load_chunk(qrowp, q_ok, 64 * c + 32 * h + 16, a.Dk, a.vec_q);
    qf[c] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  }
  // the wait for these loads belongs in front of the block loop, not at their first use inside it (see the
  // kernel above)
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int c = 0; c < DKC; ++c) asm volatile("" : : "v"(qf[c]));
#endif

  // this workgroup's blocks of keys, and of those this wave's: first, first + 4, ...
  const int nblk_all = (a.S + kSdpaBN - 1) / kSdpaBN;
  const int b0 = split * a.blocks_per_split;
  const int b1 = b0 + a.blocks_per_split < nblk_all ? b0 + a.blocks_per_split : nblk_all;

  int kvoff[KREG], vvoff[VREG];
#pragma unroll
  for (int n = 0; n < KREG; ++n) {
    const int pos = n * 64 + lane;
    const int row = pos / KCPR, chunk = (pos % KCPR) ^ k_swizzle<KROW>(pos / KCPR);
    kvoff[n] = chunk * 16 < a.Dk ? row * (int)a.ldk + chunk * 16 : 0x7fffffff;
  }
#pragma unroll
  for (int n = 0; n < VREG; ++n) {
    const int pos = n * 64 + lane;
    const int row = pos / (kVRow / 16), chunk = (pos % (kVRow / 16)) ^ v_swizzle<kVRow>(pos / (kVRow / 16));
    vvoff[n] = chunk * 16 < a.Dv ? row * (int)a.ldv + chunk * 16 : 0x7fffffff;
  }
  const int64_t first_row = (int64_t)(b0 + wave) * kSdpaBN;
  SdpaWalker wk{reinterpret_cast<uint64_t>(a.k + k_off + first_row * a.ldk), (int64_t)(a.S - 1 - first_row) * a.ldk + a.Dk};
  SdpaWalker wv{reinterpret_cast<uint64_t>(a.v + v_off + first_row * a.ldv), (int64_t)(a.S - 1 - first_row) * a.ldv + a.Dv};
  uint8_t* const mine = lds + wave * 2 * kStage;
  auto issue_block = [&](int buf) {
    const uint32_t kdst = (uint32_t)(uintptr_t)(SDPA_LDS_AS uint8_t*)(mine + buf * kStage);
    const i32x4 rk = wk.rsrc();
#pragma unroll
    for (int n = 0; n < KREG; ++n) sdpa_dma16<true>(rk, kvoff[n], kdst + n * 1024);
    const i32x4 rv = wv.rsrc();
#pragma unroll
    for (int n = 0; n < VREG; ++n) sdpa_dma16<true>(rv, vvoff[n], kdst + KBYTES + n * 1024);
    wk.base += (uint64_t)4 * kSdpaBN * a.ldk;
    wk.left -= (int64_t)4 * kSdpaBN * a.ldk;
    wv.base += (uint64_t)4 * kSdpaBN * a.ldv;
    wv.left -= (int64_t)4 * kSdpaBN * a.ldv;
  };

  f32x16 o[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.0f;
  float m_run = -__builtin_inff(), l_run = 0.0f;

  int buf = 0;
  if (b0 + wave < b1) issue_block(0);
  for (int blk = b0 + wave; blk < b1; blk += 4) {
    const int kv0 = blk * kSdpaBN;
    const bool more = blk + 4 < b1;
    if (more) issue_block(buf ^ 1);
    // This block has landed once only the next one's loads are outstanding.  A block that reaches beyond
    // kv_len may hold loads that complete at once, ahead of older ones, so the count is only trusted when the
    // block just requested is whole; otherwise everything is waited for.
    if (more && (blk + 5) * kSdpaBN <= a.S) {
      constexpr int cnt = KREG + VREG;
      static_assert(cnt <= 63, "vmcnt holds 6 bits");
      __builtin_amdgcn_s_waitcnt((cnt & 15) | ((cnt >> 4) << 14) | 0x0f70);
    } else {
      __builtin_amdgcn_s_waitcnt(0x0f70);
    }
    const uint8_t* kb = mine + buf * kStage;
    const bool edge = a.causal || kv0 + kSdpaBN > a.S || a.mask_kind != kMaskNone;
    sdpa_block<DKC, DVT, FMT>(a, kb, kb + KBYTES, kv0, edge, qpos, q_ok, mrow, qf, sc2, lqs, clamp_p, o, m_run, l_run);
    buf ^= 1;
  }

  // ---- merge the four waves: each leaves O^T [dv][row], m[row], l[row] in LDS
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();  // every wave is done with its stages
  float* tile = reinterpret_cast<float*>(lds) + wave * kDecodeTileFloats(DVT);
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) tile[(32 * t + 8 * (r >> 2) + 4 * h + (r & 3)) * 32 + lq] = o[t][r];
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  if (h == 0) {
    tile[32 * DVT * 32 + lq] = m_run;
    tile[32 * DVT * 32 + 32 + lq] = l_tot;
  }
  __syncthreads();
  const int row = tid & 31, dvg = tid >> 5;  // a thread merges columns dvg, dvg + 8, ... of one row
  const float* parts = reinterpret_cast<const float*>(lds);
  if (a.nsplit == 1) {
    float val[DVT * 32 / 8];
    const float inv_l = sdpa_merge<DVT>(parts, 4, kDecodeTileFloats(DVT), row, dvg, 8, qs, val);
    const int rin = a.pack ? row / a.L : 0, rq = a.pack ? row - rin * a.L : row;
    uint8_t* orow = a.out + (o_off + (int64_t)rin * a.o_bs[2] + (int64_t)rq * a.ldo) * (a.out_fp8 ? 1 : 2);
    sdpa_store_row<DVT>(a, orow, row < a.rows, dvg == 0 ? inv_l : 0.0f, dvg, 8, val);
  } else {
    // Unnormalised: the merged maximum, the merged sum and O of this split go to the workspace; the workgroup
    // that draws the group's last ticket merges the splits in their order, whoever came last, and stores the
    // rows.  The partial results are written and read with device-scope atomic accesses, which go past this
    // XCD's cache to where the other XCDs see them: no cache has to be written back or invalidated as a whole,
    // which a fence would do.  The last one returns the counter to zero for the next launch.
    float M = -__builtin_inff();
    for (int w = 0; w < 4; ++w) M = __builtin_fmaxf(M, parts[w * kDecodeTileFloats(DVT) + 32 * DVT * 32 + row]);
    float L = 0.0f, val[DVT * 32 / 8];
#pragma unroll
    for (int i = 0; i < DVT * 32 / 8; ++i) val[i] = 0.0f;
    for (int w = 0; w < 4; ++w) {
      const float* pw = parts + w * kDecodeTileFloats(DVT);
      const float mw = pw[32 * DVT * 32 + row];
      const float wgt = mw == -__builtin_inff() ? 0.0f : fast_exp2(mw - M);
      L += pw[32 * DVT * 32 + 32 + row] * wgt;
#pragma unroll
      for (int i = 0; i < DVT * 32 / 8; ++i) val[i] += pw[(dvg + 8 * i) * 32 + row] * wgt;
    }
    float* group_parts = a.ws + (int64_t)grp * a.nsplit * kDecodeTileFloats(DVT);
    float* out = group_parts + (int64_t)split * kDecodeTileFloats(DVT);
#pragma unroll
    for (int i = 0; i < DVT * 32 / 8; ++i)
      __hip_atomic_store(out + (dvg + 8 * i) * 32 + row, val[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (dvg == 0) {
      __hip_atomic_store(out + 32 * DVT * 32 + row, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(out + 32 * DVT * 32 + 32 + row, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_waitcnt(0);  // the stores have been acknowledged before the ticket is drawn
    __syncthreads();
    uint32_t* drawn = reinterpret_cast<uint32_t*>(lds);  // the tiles in LDS have been read
    if (tid == 0) {
      const uint32_t t = __hip_atomic_fetch_add(a.tickets + grp, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (t == (uint32_t)a.nsplit - 1) __hip_atomic_store(a.tickets + grp, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *drawn = t;
    }
    __syncthreads();
    if (*drawn != (uint32_t)a.nsplit - 1) return;
    M = -__builtin_inff();
    for (int w = 0; w < a.nsplit; ++w)
      M = __builtin_fmaxf(M, __hip_atomic_load(group_parts + (int64_t)w * kDecodeTileFloats(DVT) + 32 * DVT * 32 + row, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT));
    L = 0.0f;
#pragma unroll
    for (int i = 0; i < DVT * 32 / 8; ++i) val[i] = 0.0f;
    for (int w = 0; w < a.nsplit; ++w) {
      const float* pw = group_parts + (int64_t)w * kDecodeTileFloats(DVT);
      const float mw = __hip_atomic_load(pw + 32 * DVT * 32 + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const float wgt = mw == -__builtin_inff() ? 0.0f : fast_exp2(mw - M);
      L += __hip_atomic_load(pw + 32 * DVT * 32 + 32 + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * wgt;
#pragma unroll
      for (int i = 0; i < DVT * 32 / 8; ++i)
        val[i] += __hip_atomic_load(pw + (dvg + 8 * i) * 32 + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * wgt;
    }
    const float l = L / qs;
    const float inv_l = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
    for (int i = 0; i < DVT * 32 / 8; ++i) val[i] *= inv_l;
    const int rin = a.pack ? row / a.L : 0, rq = a.pack ? row - rin * a.L : row;
    uint8_t* orow = a.out + (o_off + (int64_t)rin * a.o_bs[2] + (int64_t)rq * a.ldo) * (a.out_fp8 ? 1 : 2);
    sdpa_store_row<DVT>(a, orow, row < a.rows, dvg == 0 ? inv_l : 0.0f, dvg, 8, val);
  }
}

template <int DKC, int DVT>
static int sdpa_decode_launch(const SdpaArgs& a, int fmt, int64_t groups, hipStream_t st) {
  const dim3 grid((unsigned)(groups * a.nsplit));
  if (fmt == MI355Q_E5M2) hipLaunchKernelGGL((fp8_sdpa_decode_kernel<DKC, DVT, MI355Q_E5M2>), grid, dim3(kSdpaThreads), 0, st, a);
  else hipLaunchKernelGGL((fp8_sdpa_decode_kernel<DKC, DVT, MI355Q_E4M3FN>), grid, dim3(kSdpaThreads), 0, st, a);
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

static int compute_units_sdpa();

// How the few-queries kernel would run a problem: rows of the tile, groups, splits (0 groups: it does not apply).
constexpr size_t kSdpaTicketBytes = 1024;  // arrival counters in front of the partial results
struct SdpaDecodePlan {
  int64_t groups = 0;
  int pack = 0, rows = 0, nsplit = 1, blocks_per_split = 0, dvt = 0;
  size_t ws_bytes = 0;
};
static SdpaDecodePlan sdpa_decode_plan(const mi355q_sdpa_desc* d, int cus) {
  SdpaDecodePlan p;
  const bool shared = d->batch[2] > 1 && d->k_bstride[2] == 0 && d->v_bstride[2] == 0;
  const int64_t inner = shared ? d->batch[2] : 1;
  if (d->valid_seq_len != nullptr) return p;  // a per-batch key window runs on the kernel for many queries
  if (inner * d->q_len > 32 || d->kv_len < 512 || d->head_dim_qk > 128 || d->head_dim_v > 128) return p;
  p.pack = shared;
  p.rows = (int)(inner * d->q_len);
  p.groups = d->batch[0] * d->batch[1] * (shared ? 1 : d->batch[2]);
  p.dvt = (d->head_dim_qk > 64 || d->head_dim_v > 64) ? 4 : 2;
  const int nblk = (int)((d->kv_len + kSdpaBN - 1) / kSdpaBN);
  // enough workgroups for one per CU (a workgroup's LDS stages leave no room for a second), at least 8
  // blocks (two per wave) in each
  int64_t want = ((int64_t)cus + p.groups - 1) / p.groups;
  const int64_t most = nblk / 8 > 0 ? nblk / 8 : 1;
  want = want < 1 ? 1 : (want > most ? most : want);
  p.blocks_per_split = (int)((nblk + want - 1) / want);
  p.nsplit = (nblk + p.blocks_per_split - 1) / p.blocks_per_split;
  // One arrival counter per group in an area of a fixed size, then the splits' partial results: a workspace that
  // is used for problems of different shapes finds the counters zero whatever the last shape left behind them.
  if (p.nsplit > 1 && (size_t)p.groups * 4 > kSdpaTicketBytes) {
    p.nsplit = 1;
    p.blocks_per_split = nblk;
  }
  p.ws_bytes = p.nsplit > 1 ? kSdpaTicketBytes + (size_t)p.groups * p.nsplit * kDecodeTileFloats(p.dvt) * sizeof(float) : 0;
  return p;
}

template <int DKC, int DVT>
static int sdpa_launch(const SdpaArgs& a, int fmt, int64_t blocks, hipStream_t st) {
  const dim3 grid((unsigned)blocks), block(kSdpaThreads);
  if (fmt == MI355Q_E5M2) {
    if (a.dma) hipLaunchKernelGGL((fp8_sdpa_fwd_kernel<DKC, DVT, MI355Q_E5M2, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((fp8_sdpa_fwd_kernel<DKC, DVT, MI355Q_E5M2, false>), grid, block, 0, st, a);
  } else {
    if (a.dma) hipLaunchKernelGGL((fp8_sdpa_fwd_kernel<DKC, DVT, MI355Q_E4M3FN, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((fp8_sdpa_fwd_kernel<DKC, DVT, MI355Q_E4M3FN, false>), grid, block, 0, st, a);
  }
  return hipGetLastError() == hipSuccess ? MI355Q_OK : MI355Q_ERR_LAUNCH;
}

static bool aligned_to(const void* p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

static int compute_units_sdpa() {
  static const int n = [] {
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0)
      cu = 256;
    return cu;
  }();
  return n;
}

}  // namespace mi355q

using namespace mi355q;

extern "C" {

size_t mi355q_fp8_sdpa_workspace_bytes(const mi355q_sdpa_desc* d) {
  if (d == nullptr || d->q_len <= 0 || d->kv_len <= 0 || d->head_dim_qk <= 0 || d->head_dim_v <= 0) return 0;
  for (int i = 0; i < 3; ++i)
    if (d->batch[i] <= 0) return 0;
  return sdpa_decode_plan(d, compute_units_sdpa()).ws_bytes;
}

int mi355q_fp8_sdpa_key_splits(const mi355q_sdpa_desc* d, int64_t* blocks_per_split) {
  if (blocks_per_split != nullptr) *blocks_per_split = 0;
  if (d == nullptr || d->q_len <= 0 || d->kv_len <= 0 || d->head_dim_qk <= 0 || d->head_dim_v <= 0) return 0;
  for (int i = 0; i < 3; ++i)
    if (d->batch[i] <= 0) return 0;
  const SdpaDecodePlan p = sdpa_decode_plan(d, compute_units_sdpa());
  if (p.groups == 0) return 0;
  if (blocks_per_split != nullptr) *blocks_per_split = p.blocks_per_split;
  return p.nsplit;
}

int mi355q_fp8_sdpa_fwd(const void* q, const void* k, const void* v, int fp8_fmt, const void* mask, int mask_kind,
                        void* out, int out_dtype, const mi355q_sdpa_desc* d, float softmax_scale, int is_causal,
                        const float* const* scale_dev, const float* scale_host, float* amax_s, float* amax_o,
                        void* workspace, size_t workspace_bytes, void* stream) {
  if (d == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (fp8_fmt != MI355Q_E4M3FN && fp8_fmt != MI355Q_E5M2) return MI355Q_ERR_INVALID_ARGUMENT;
  if (out_dtype != MI355Q_BF16 && out_dtype != MI355Q_E4M3FN) return MI355Q_ERR_INVALID_ARGUMENT;
  if (mask_kind < MI355Q_SDPA_MASK_NONE || mask_kind > MI355Q_SDPA_MASK_F32) return MI355Q_ERR_INVALID_ARGUMENT;
  if (d->q_len < 0 || d->kv_len < 0 || d->head_dim_qk <= 0 || d->head_dim_v <= 0) return MI355Q_ERR_INVALID_ARGUMENT;
  int64_t batches = 1;
  for (int i = 0; i < 3; ++i) {
    if (d->batch[i] < 0) return MI355Q_ERR_INVALID_ARGUMENT;
    batches *= d->batch[i];
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (amax_s != nullptr || amax_o != nullptr) {
    hipLaunchKernelGGL(sdpa_clear_amax_kernel, dim3(1), dim3(1), 0, st, amax_s, amax_o);
    if (hipGetLastError() != hipSuccess) return MI355Q_ERR_LAUNCH;
  }
  if (batches == 0 || d->q_len == 0) return MI355Q_OK;
  if (q == nullptr || out == nullptr || (d->kv_len > 0 && (k == nullptr || v == nullptr))) return MI355Q_ERR_INVALID_ARGUMENT;
  if (mask_kind != MI355Q_SDPA_MASK_NONE && mask == nullptr) return MI355Q_ERR_INVALID_ARGUMENT;
  if (d->head_dim_qk > 256 || d->head_dim_v > 256) return MI355Q_ERR_UNSUPPORTED;
  if (d->q_len > (1 << 30) || d->kv_len > (1 << 30)) return MI355Q_ERR_UNSUPPORTED;
  const int64_t nqb = (d->q_len + kSdpaBM - 1) / kSdpaBM;
  const int64_t blocks = nqb * batches;
  if (blocks > 0x7fffffff) return MI355Q_ERR_UNSUPPORTED;

  SdpaArgs a{};
  a.q = static_cast<const uint8_t*>(q);
  a.k = static_cast<const uint8_t*>(k);
  a.v = static_cast<const uint8_t*>(v);
  a.mask = static_cast<const uint8_t*>(mask);
  a.out = static_cast<uint8_t*>(out);
  bool vq = aligned_to(q, 16) && d->head_dim_qk % 16 == 0 && d->ldq % 16 == 0;
  bool vk = aligned_to(k, 16) && d->head_dim_qk % 16 == 0 && d->ldk % 16 == 0;
  bool vv = aligned_to(v, 16) && d->head_dim_v % 16 == 0 && d->ldv % 16 == 0;
  const size_t oel = out_dtype == MI355Q_BF16 ? 2 : 1;
  bool vo = aligned_to(out, 4 * oel) && d->head_dim_v % 4 == 0 && d->ldo % 4 == 0;
  for (int i = 0; i < 3; ++i) {
    a.bdim[i] = d->batch[i];
    a.q_bs[i] = d->q_bstride[i];
    a.k_bs[i] = d->k_bstride[i];
    a.v_bs[i] = d->v_bstride[i];
    a.m_bs[i] = mask_kind != MI355Q_SDPA_MASK_NONE ? d->mask_bstride[i] : 0;
    a.o_bs[i] = d->out_bstride[i];
    vq = vq && d->q_bstride[i] % 16 == 0;
    vk = vk && d->k_bstride[i] % 16 == 0;
    vv = vv && d->v_bstride[i] % 16 == 0;
    vo = vo && d->out_bstride[i] % 4 == 0;
  }
  a.ldq = d->ldq; a.ldk = d->ldk; a.ldv = d->ldv; a.ldm = d->ldmask; a.ldo = d->ldo;
  a.L = (int)d->q_len; a.S = (int)d->kv_len; a.Dk = (int)d->head_dim_qk; a.Dv = (int)d->head_dim_v;
  a.mask_kind = mask_kind;
  a.causal = is_causal != 0;
  a.out_fp8 = out_dtype == MI355Q_E4M3FN;
  a.vec_q = vq; a.vec_k = vk; a.vec_v = vv; a.vec_o = vo;
  // direct loads address a block's rows with 32-bit offsets from a base that moves with the block
  a.dma = vk && vv && d->ldk < (1 << 24) && d->ldv < (1 << 24);
  a.nqb = (int)nqb;
  a.scale = softmax_scale;
  for (int i = 0; i < 6; ++i) {
    a.sc_dev[i] = scale_dev != nullptr ? scale_dev[i] : nullptr;
    a.sc_host[i] = scale_host != nullptr ? scale_host[i] : 0.0f;
  }
  a.amax_s = amax_s;
  a.amax_o = amax_o;
  a.valid_len = d->valid_seq_len;
  a.valid_dim = d->valid_seq_len != nullptr ? d->valid_seq_dim : -1;
  a.pad_left = d->seq_padding_left != 0;
  if (d->valid_seq_len != nullptr && (d->valid_seq_dim < 0 || d->valid_seq_dim > 2)) return MI355Q_ERR_INVALID_ARGUMENT;

  const int64_t dmax = d->head_dim_qk > d->head_dim_v ? d->head_dim_qk : d->head_dim_v;
  // a few queries against many keys: the kernel that splits the keys (direct loads only)
  // (a per-batch key window is served by the other kernel alone)
  SdpaDecodePlan plan = sdpa_decode_plan(d, compute_units_sdpa());
  if (plan.groups > 0 && a.dma && plan.groups * (int64_t)plan.nsplit <= 0x7fffffff) {
    if (plan.nsplit > 1 && (workspace == nullptr || workspace_bytes < plan.ws_bytes || !aligned_to(workspace, 4))) {
      plan.nsplit = 1;  // no room for partial results: one workgroup per group walks all the keys
      plan.blocks_per_split = (int)((d->kv_len + kSdpaBN - 1) / kSdpaBN);
    }
    a.pack = plan.pack;
    a.rows = plan.rows;
    a.nsplit = plan.nsplit;
    a.blocks_per_split = plan.blocks_per_split;
    a.tickets = static_cast<uint32_t*>(workspace);
    a.ws = workspace != nullptr ? reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + kSdpaTicketBytes) : nullptr;
    return plan.dvt == 2 ? sdpa_decode_launch<1, 2>(a, fp8_fmt, plan.groups, st) : sdpa_decode_launch<2, 4>(a, fp8_fmt, plan.groups, st);
  }
  if (dmax <= 64) return sdpa_launch<1, 2>(a, fp8_fmt, blocks, st);
  if (dmax <= 128) return sdpa_launch<2, 4>(a, fp8_fmt, blocks, st);
  return sdpa_launch<4, 8>(a, fp8_fmt, blocks, st);
}

}  // extern "C"
