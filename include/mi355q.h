/*
 * mi355q: C ABI of the gfx950 kernels behind the hpu:: quantized-inference ops.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream
 * (passed as void* so that this header needs no HIP include), launches
 * asynchronously on that stream, never synchronises, never allocates and
 * returns an mi355q_status.  All tensors are dense row-major unless a stride
 * argument says otherwise.
 *
 * Each entry point names the reference interface it stands in for.  In the
 * reference these are Synapse graph nodes identified by GUID strings; the
 * arithmetic behind the GUIDs is not in the reference tree.
 */
#ifndef MI355Q_H
#define MI355Q_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  MI355Q_OK = 0,
  MI355Q_ERR_INVALID_ARGUMENT = 1, /* null pointer, bad enum, negative size */
  MI355Q_ERR_UNSUPPORTED = 2,      /* valid request this build has no kernel for */
  MI355Q_ERR_LAUNCH = 3,           /* hipLaunchKernel reported an error */
  MI355Q_ERR_WORKSPACE = 4,        /* workspace missing or too small */
  MI355Q_ERR_TOO_LARGE = 5         /* problem needs more than the fixed scratch buffer of an
                                      allocation-free entry point */
} mi355q_status;

typedef enum {
  MI355Q_F32 = 0,
  MI355Q_BF16 = 1,
  MI355Q_E4M3FN = 2, /* OCP fp8 e4m3fn, max 448, no Inf */
  MI355Q_E5M2 = 3    /* OCP fp8 e5m2, max finite 57344 */
} mi355q_dtype;

/* How a cast scale is broadcast against the input
 * (ValidateScaleShape / HandleScaleTensor / HandleScaleScalar,
 * hpu_ops/backend/fp8_ops.cpp:29-100). */
typedef enum {
  MI355Q_SCALE_NONE = 0, /* scale == 1 */
  MI355Q_SCALE_HOST = 1, /* one value, passed by value (the .scalar overloads) */
  MI355Q_SCALE_DEV = 2,  /* one fp32 value in device memory */
  MI355Q_SCALE_MID = 3,  /* input viewed as [outer, mid, inner]; scale is fp32[mid].
                            inner == row length gives per-row scales,
                            inner == 1 gives per-column scales */
  MI355Q_SCALE_FULL = 4  /* one fp32 scale per element */
} mi355q_scale_mode;

/* GEMM scale / bias broadcast against the [M, N] output. */
typedef enum {
  MI355Q_GS_NONE = 0,
  MI355Q_GS_HOST = 1,    /* scalar by value */
  MI355Q_GS_DEV = 2,     /* one fp32 value in device memory */
  MI355Q_GS_PER_ROW = 3, /* fp32[M]  (scale shape [M,1]) */
  MI355Q_GS_PER_COL = 4  /* fp32[N]  (scale shape [1,N]) */
} mi355q_gemm_scale_mode;

typedef enum {
  MI355Q_BIAS_NONE = 0,
  MI355Q_BIAS_ROW_VECTOR = 1, /* [N], broadcast down the rows */
  MI355Q_BIAS_FULL = 2        /* [M, N] with row stride ldbias */
} mi355q_bias_mode;

typedef enum {
  MI355Q_ZP_NONE = 0,
  MI355Q_ZP_FLOAT = 1, /* same dtype and shape as the scale */
  MI355Q_ZP_PACKED = 2 /* int32, 8 nibbles per word, shape [rows/group, packed_cols] */
} mi355q_zp_kind;

/* ABI version: bumped when a signature below changes. */
int mi355q_abi_version(void);
const char* mi355q_status_string(int status);

/*
 * amax = max|x| over n elements of fp32 or bf16, written as one fp32.
 * A NaN in x makes the result NaN.  Stands in for the amax output of the
 * convert_to_fp8_* node (CastToFp8V2::AddNode, hpu_ops/backend/fp8_ops.cpp:
 * 192-258, second output) when it is wanted without the cast.
 */
int mi355q_amax(const void* x, int x_dtype, int64_t n, float* amax_out, void* stream);

/*
 * Per-row amax of a [rows, cols] tensor -> fp32[rows].  The reference has no
 * such op (its amax is always one scalar, fp8_ops.cpp:170-178); dynamic
 * per-token quantisation needs it before cast_to_fp8 with per-row scales.
 */
int mi355q_rowwise_amax(const void* x, int x_dtype, int64_t rows, int64_t cols,
                        float* amax_out, void* stream);

/*
 * Dynamic per-row ("per-token") quantisation in one pass over x [rows, cols]:
 *   amax_r = max|x[r, :]|, scale_r = min(target / amax_r, 0x1.fep127f) (fp32 division; the cap,
 *   the largest finite bf16 value, only acts on a row of zeros or of values below
 *   target / 3.4e38: such a row gets zero (or saturated) codes and a finite 1 / scale_r
 *   instead of the NaN codes that 0 * inf would give; a NaN in the row makes scale_r NaN),
 *   y[r, :] = cast_to_fp8(x[r, :] * scale_r)   with the rounding rules of mi355q_cast_to_fp8,
 *   scale_out[r] = scale_r, scale_inv_out[r] = 1 / scale_r   (either may be NULL).
 * Bit-identical to mi355q_rowwise_amax, the division on the host side and
 * mi355q_cast_to_fp8 with MI355Q_SCALE_MID, which it replaces when a caller
 * quantises activations on the fly.  The reference has no such op
 * (fp8_ops.cpp:170-178: its amax is one scalar and the scale is computed by
 * the caller).  Rows of up to 2048 16-byte vectors (16384 bf16 / 8192 fp32
 * elements), x 16-byte aligned, cols a multiple of 8 (bf16) or 4 (fp32);
 * otherwise MI355Q_ERR_UNSUPPORTED and the caller takes the three-step route.
 */
int mi355q_quantize_rows(const void* x, int x_dtype, int64_t rows, int64_t cols,
                         void* y, int fp8_fmt, float target,
                         float* scale_out, float* scale_inv_out, void* stream);

/*
 * The elementwise glue of a gated MLP block fused with the quantisation of its
 * result, one pass over bf16 gate / up [rows, cols] (row pitches ld_gate, ld_up
 * in elements, so both may be column ranges of one wider matrix):
 *   h = bf16( bf16( silu(gate) ) * up ),   silu(x) = x / (1 + exp(-x)) in fp32,
 *   then mi355q_quantize_rows of h (amax_r, scale_r = target / amax_r, cast,
 *   scale_out / scale_inv_out); h_out, when not NULL, receives h [rows, cols].
 * Between the reference's ops this step is left to aten (silu and mul on the
 * device, then cast_to_fp8_v2): there is no reference operator to cite.  The
 * exp is a fixed sequence of IEEE operations that the CPU oracle repeats
 * (ora_silu_mul_bf16), so results are bit-identical to it; against a correctly
 * rounded silu the bf16 value differs for 18 of the 65536 inputs, all below
 * -88, where the result (magnitude < 3.3e-37) is returned as -0.
 * gate, up 16-byte aligned, cols and pitches multiples of 8, rows of up to 2048
 * 16-byte vectors; otherwise MI355Q_ERR_UNSUPPORTED.
 */
int mi355q_silu_mul_quantize_rows(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                  int64_t rows, int64_t cols, void* y, int fp8_fmt, float target,
                                  void* h_out, float* scale_out, float* scale_inv_out, void* stream);

/*
 * y = saturating round-to-nearest-even fp8( x * scale ), optional amax of x.
 * Replaces the convert_to_fp8_{f32,bf16} node built by CastToFp8V2::AddNode
 * (hpu_ops/backend/fp8_ops.cpp:192-258; round mode CAST_ROUND_HALF_NE,
 * GetCastParams :105-119).  For bf16 input the scale is rounded to bf16 and
 * the product is rounded to bf16 before the fp8 rounding.
 *   x          n = outer*mid*inner elements (for NONE/HOST/DEV/FULL pass
 *              outer = n, mid = inner = 1)
 *   scale_dev  fp32 device pointer for DEV / MID / FULL, else ignored
 *   amax_out   NULL, or one fp32 that receives max|x| (of the unscaled input)
 * x_dtype may also be an fp8 type equal to fp8_fmt: then y is a copy of x
 * (fp8_ops.cpp:201-215) and amax_out must be NULL.
 */
int mi355q_cast_to_fp8(const void* x, int x_dtype, void* y, int fp8_fmt,
                       const float* scale_dev, float scale_host, int scale_mode,
                       int64_t outer, int64_t mid, int64_t inner,
                       float* amax_out, void* stream);

/*
 * mi355q_cast_to_fp8 with stochastic rounding (round mode CAST_ROUND_SR of
 * GetCastParams, hpu_ops/backend/fp8_ops.cpp:105-119, selected by the op's
 * stochastic_rounding flag): x * scale, rounded to bf16 first for bf16 input,
 * saturated, is rounded up or down with probability proportional to its distance
 * from the two neighbouring fp8 values.  Element i takes its random bits from a
 * counter-based generator keyed by (seed, offset + i / 2): the same seed and
 * offset give the same output.  x must be fp32 or bf16.
 * flush_subnormals != 0 is round mode CAST_ROUND_SFTZ ("stochastic flush to zero", the
 * reference's default for bf16 -> e5m2, flag is_sr_sftz, hpu_ops/fp8_ops.h:52): a scaled value
 * below the format's smallest normal number (2^-14 for e5m2, 2^-6 for e4m3fn) gives a zero of
 * its sign; everything else rounds stochastically as above.
 */
int mi355q_cast_to_fp8_sr(const void* x, int x_dtype, void* y, int fp8_fmt,
                          const float* scale_dev, float scale_host, int scale_mode,
                          int64_t outer, int64_t mid, int64_t inner,
                          float* amax_out, uint64_t seed, uint64_t offset, int flush_subnormals,
                          void* stream);

/*
 * One read of x (fp32 or bf16, n elements), two casts: y_e5m2 = fp8_e5m2(x * scale_e5m2) and
 * y_e4m3fn = fp8_e4m3fn(x * scale_e4m3fn), plus optionally amax = max|x|.  Replaces the
 * convert_to_fp8_hybrid node of CastToFp8Hybrid::AddNode
 * (hpu_ops/backend/cast_to_fp8_hybrid_gen.cpp:66-100).  Scales are one fp32 value in device
 * memory each, or NULL for 1.  stochastic = 1 rounds the e5m2 output stochastically (random bits
 * as in mi355q_cast_to_fp8_sr), stochastic = 2 does so with flush to zero below 2^-14 (CAST_ROUND_SFTZ,
 * cast_to_fp8_hybrid_gen.cpp:26-35); the e4m3fn output always rounds to nearest even.
 */
int mi355q_cast_to_fp8_hybrid(const void* x, int x_dtype, int64_t n, void* y_e5m2, void* y_e4m3fn,
                              const float* scale_e5m2, const float* scale_e4m3fn, int stochastic,
                              uint64_t seed, uint64_t offset, float* amax_out, void* stream);

/*
 * y = out_dtype(x_fp8) * scale, computed in out_dtype (fp32 or bf16).
 * Replaces the convert_from_fp8_{f32,bf16} node of CastFromFp8::AddNode
 * (hpu_ops/backend/fp8_ops.cpp:265-308).  Scale arguments as above.
 */
int mi355q_cast_from_fp8(const void* x, int fp8_fmt, void* y, int out_dtype,
                         const float* scale_dev, float scale_host, int scale_mode,
                         int64_t outer, int64_t mid, int64_t inner, void* stream);

/*
 * out[r, 8p+i] = (nibble_i(packed[r, p]) - z) * s, nibble i = bits [4i, 4i+4).
 * Replaces the dequantize_4_bit_{f32,bf16} node of Int4BaseOp::AddNode
 * (hpu_ops/backend/int4_ops.cpp:40-56); is_signed selects convert_from_int4
 * (nibble >= 8 means nibble-16) over convert_from_uint4 (:58-62).
 *   packed  int32 [rows, packed_cols]
 *   scale   out_dtype [rows/group, 8*packed_cols]; group == 1 is the
 *           elementwise form, group > 1 the group-wise (AutoGPTQ) form
 *   zp      per zp_kind; a float zero-point is subtracted in out_dtype
 *   out     out_dtype [rows, 8*packed_cols]
 */
int mi355q_dequant_4bit(const int32_t* packed, const void* scale, const void* zp,
                        int zp_kind, int is_signed, int out_dtype, int64_t rows,
                        int64_t packed_cols, int64_t group, void* out, void* stream);

/*
 * C[b] = out_dtype( (op(A[b]) @ op(B[b])) * sA * sB + bias + D[b] )
 * with fp32 accumulation and one final rounding.  Replaces the
 * fp8_gemm_{f32,bf16} node of Fp8GemmV2::AddNode
 * (hpu_ops/backend/fp8_ops.cpp:403-496; synGEMMParams{trans_A, trans_B} :482).
 *   A      fp8 (fmt_a); trans_a == 0: [M, K] with row stride lda,
 *          trans_a != 0: [K, M] with row stride lda
 *   B      fp8 (fmt_b); trans_b == 0: [K, N] with row stride ldb,
 *          trans_b != 0: [N, K] with row stride ldb
 *   C      out_dtype (fp32 or bf16) [M, N], row stride ldc
 *   sa/sb  per mi355q_gemm_scale_mode (the *_scale_inv arguments of the op)
 *   bias   out_dtype, per mi355q_bias_mode; D: out_dtype [M, N] stride ldd or NULL
 *   batch  number of problems; stride_* are element strides between them
 *          (0 broadcasts an operand)
 * Leading dimensions and batch strides are in elements.  As in BLAS, an
 * operand is an array of whole rows: where lda (ldb) is a multiple of 16, the
 * bytes of a row up to the next multiple of 16 past its last element are
 * read, the last row's included (they never reach a stored output).
 */
int mi355q_fp8_gemm(const void* A, int fmt_a, int trans_a, int64_t lda,
                    const void* B, int fmt_b, int trans_b, int64_t ldb,
                    void* C, int out_dtype, int64_t ldc,
                    int64_t M, int64_t N, int64_t K,
                    const float* sa_dev, float sa_host, int sa_mode,
                    const float* sb_dev, float sb_host, int sb_mode,
                    const void* bias, int bias_mode, int64_t ldbias,
                    const void* D, int64_t ldd,
                    int64_t batch, int64_t stride_a, int64_t stride_b,
                    int64_t stride_c, int64_t stride_d, int64_t stride_bias,
                    void* stream);

/*
 * Fused int4-dequant GEMM, fp8 activations times 4-bit weights (W4A8):
 *   C = out_dtype( (A @ W) * sa + bias ),   W[k, n] = (q[k, n] - z[k / group, n]) * s[k / group, n],
 * with the weights as convert_from_int4 / convert_from_uint4 take them and mi355q_dequant_4bit
 * would expand them (Int4BaseOp::AddNode, hpu_ops/backend/int4_ops.cpp:40-56: packed int32
 * [K, N / 8], nibble i of word p is column 8 p + i, is_signed selects int4 over uint4), multiplied as
 * Fp8GemmV2::AddNode multiplies (hpu_ops/backend/fp8_ops.cpp:403-496) without the bf16 [K, N]
 * matrix in between: the packed words are what travels from HBM, (q - z) enters the fp8 MFMA exactly,
 * each K group is accumulated in fp32 and multiplied by its scales as it joins the total.  The
 * reference has no fused op; it is the composition of those two.
 *   A           fp8 (fmt_a) [M, K], row pitch lda
 *   packed      int32 [K, N / 8], row pitch ld_packed (in words)
 *   scale       bf16 or fp32 (scale_dtype) [K / group, N], dense
 *   zero_point  packed int32 [K / group, N / 8] (same nibble order and signedness) or NULL
 *   sa          none, host scalar, device scalar or per row (mi355q_gemm_scale_mode); bias: out_dtype [N] or NULL
 * group must be a multiple of 128 that divides K; N a multiple of 32; K, lda multiples of 16; all
 * pointers 16-byte aligned; otherwise MI355Q_ERR_UNSUPPORTED, and the caller expands the weights
 * with mi355q_dequant_4bit.
 *
 * workspace: with groups of 128 and bf16 scales, K is walked in parts by several workgroups per
 * 256 columns where that fills the chip better, which meet through `workspace`:
 * mi355q_w4a8_gemm_workspace_bytes() of device memory, 16-byte aligned (0: the shape is not split
 * and no workspace is read).  Its first KiB holds arrival counters (whatever the shape): they have
 * to be zero when a call starts and every call leaves them zero, so a workspace is zero-filled
 * once, when it is allocated, and then reused, also for other shapes it is large enough for.  Calls
 * that share a workspace must not overlap (one stream, or an order between the streams).  NULL is allowed: the
 * call then runs without the split, slower for these shapes.  Too small or misaligned:
 * MI355Q_ERR_WORKSPACE.  The parts are added in a fixed order: a result does not depend on which
 * workgroup finished last.
 */
size_t mi355q_w4a8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int scale_dtype);
int mi355q_w4a8_gemm(const void* A, int fmt_a, int64_t lda, const int32_t* packed, int64_t ld_packed,
                     const void* scale, int scale_dtype, const int32_t* zero_point, int is_signed,
                     int64_t group, void* C, int out_dtype, int64_t ldc, int64_t M, int64_t N, int64_t K,
                     const float* sa_dev, float sa_host, int sa_mode, const void* bias,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * Sum over the middle dimension of an fp8 tensor viewed as [outer, reduce, inner]
 * (a sum over adjacent dimensions of a contiguous tensor), accumulated in fp32 in a
 * fixed order and written as out_dtype (fp32, bf16, or fp8 with the saturating
 * round-to-nearest cast of mi355q_cast_to_fp8) [outer, inner].  Replaces the
 * reduce_sum_multi_dim_fwd node of hpu::sum_fp8 (hpu_ops/backend/fp8_ops_gen.cpp:20-49,
 * schema scripts/hpu_op.yaml:7448-7453).  When the launch splits the reduction it
 * needs mi355q_sum_fp8_workspace_bytes(...) bytes of device memory for partial sums
 * (0 when it does not); nothing is allocated here.
 */
size_t mi355q_sum_fp8_workspace_bytes(int64_t outer, int64_t reduce, int64_t inner);
int mi355q_sum_fp8(const void* x, int fp8_fmt, int64_t outer, int64_t reduce, int64_t inner,
                   void* out, int out_dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * mi355q_sum_fp8 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments without the
 * workspace, same kernels, same results bit for bit.  It has no counterpart in the reference.
 * The partial sums of a split reduction go to a fixed buffer of
 * MI355Q_SUM_FP8_STATIC_SCRATCH_BYTES inside the library's device image (one copy per GPU,
 * held until the process ends); a problem whose mi355q_sum_fp8_workspace_bytes(...) exceeds
 * that returns MI355Q_ERR_TOO_LARGE and launches nothing.  The call allocates and frees
 * nothing.  The stream's device must be the current device.  All calls on one GPU share the
 * buffer: calls that may overlap on one GPU (different streams) race; calls on one stream,
 * or ordered by events, do not.  The first call on a device looks the buffer's address up
 * (hipGetSymbolAddress, once per device): make it before a graph capture starts; a first call
 * on a device whose stream is being captured returns MI355Q_ERR_UNSUPPORTED and launches nothing.
 */
#define MI355Q_SUM_FP8_STATIC_SCRATCH_BYTES (2u << 20)
int mi355q_sum_fp8_static(const void* x, int fp8_fmt, int64_t outer, int64_t reduce, int64_t inner,
                          void* out, int out_dtype, void* stream);

/*
 * Softmax over the rows of x [rows, cols] (bf16 or e4m3fn):
 *   v = (x * inv_attn_heads) * input_scale + fused_add,   each term optional,
 *   p = bf16( exp(v - max v) / sum exp(v - max v) ),
 *   y = p                              when y_dtype is bf16,
 *   y = e4m3fn( p * output_scale )     when y_dtype is e4m3fn (saturating round to nearest),
 * in fp32 up to the rounding to bf16.  Replaces the softmax_fwd_hf8 node of
 * SoftmaxFp8::AddNode (hpu_ops/backend/softmax_fp8_gen.cpp:73-158).  A scale is a
 * device scalar (pointer not NULL) or the host value (1 = absent).  fused_add is bf16
 * or NULL; its rows are found by decomposing the row index over row_sizes[0 .. row_dims)
 * (innermost first, product = rows) and adding digit * fused_add_row_strides[d] elements
 * (0 where fused_add is broadcast), row_dims <= 6.
 */
int mi355q_softmax_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols,
                       const float* input_scale_dev, float input_scale_host,
                       const float* output_scale_dev, float output_scale_host,
                       const float* inv_attn_heads_dev, float inv_attn_heads_host,
                       const void* fused_add, int row_dims, const int64_t* row_sizes,
                       const int64_t* fused_add_row_strides, void* y, int y_dtype, void* stream);

/*
 * Fused int4-dequant GEMM on 16-bit activations (W4A16):
 *   C[m, n] = out( sum_g s[g, n] * sum_{k in g} a[m, k] * (q[k, n] - z[g, n]) + bias[n] )
 * with a bf16.  This is what the reference composes from convert_from_int4 / convert_from_uint4 to
 * bf16 (Int4BaseOp::AddNode, hpu_ops/backend/int4_ops.cpp:40-56: nibble order, (q - z) * s, the
 * group layout of its test, tests/pytest_working/any_mode/test_hpu_convert_from_int4.py:398-476)
 * and a bf16 matmul; here the bf16 [K, N] matrix never exists.  The activations are first cut into
 * two e4m3fn planes per row (mi355q_split_rows_fp8x2: a * s = hi + lo / 16 with a power-of-two row
 * scale s, exact for every element within a factor 2^15 of the row's largest and to 3e-8 of that
 * largest otherwise), and both planes meet the packed nibbles in the matrix unit as in
 * mi355q_w4a8_gemm, so the integers (q - z) and the products enter the fp32 sums exactly.
 * Serves groups of 128 with bf16 scales, N a multiple of 32 and K of 16 (MI355Q_ERR_UNSUPPORTED
 * otherwise).  `workspace`: mi355q_w4a16_gemm_workspace_bytes(...) bytes of device memory, 16-byte
 * aligned, for the planes, the row scales and, in front, the arrival counters and partial sums of
 * the split over K: its first 1 KiB has to be zero before the first use and is left zero, so the
 * buffer can be passed again (calls that may overlap need buffers of their own).  split_k = 0 keeps
 * K in one piece (no counters are touched).  Nothing is allocated.
 */
size_t mi355q_w4a16_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int scale_dtype);
int mi355q_w4a16_gemm(const void* A, int a_dtype, int64_t lda, const int32_t* packed, int64_t ld_packed,
                      const void* scale, int scale_dtype, const int32_t* zero_point, int is_signed,
                      int64_t group, void* C, int out_dtype, int64_t ldc, int64_t M, int64_t N, int64_t K,
                      const void* bias, void* workspace, size_t workspace_bytes, int split_k, void* stream);
/* The first step of mi355q_w4a16_gemm on its own: rows of bf16 x [rows, cols] (pitch ldx elements) as two
 * e4m3fn planes hi, lo [rows, ld] (ld a multiple of 16, columns from cols on zero) and scale_inv[rows] =
 * 1 / s with x * s = hi + lo / 16.  No counterpart in the reference. */
int mi355q_split_rows_fp8x2(const void* x, int x_dtype, int64_t ldx, int64_t rows, int64_t cols, void* hi, void* lo,
                            int64_t ld, float* scale_inv, void* stream);

/*
 * Attention forward for inference on fp8 q, k, v:
 *   S   = (q d_scale_q) (k d_scale_k)^T softmax_scale  [+ float mask | -inf where a bool mask
 *         is 0 | -inf for key j > query i when is_causal]
 *   out = softmax(S) (v d_scale_v)
 * computed with an online softmax over blocks of 64 keys: with m the running row maximum,
 * p = exp(S - m) in [0, 1] is rounded to fp8 (the format of v) as p * q_scale_s before the
 * second product, the row sums use the unrounded p, both products accumulate in fp32, and the
 * result is multiplied by d_scale_s (1 / q_scale_s when absent).  out is bf16, or e4m3fn holding
 * out * q_scale_o (saturating round-to-nearest-even).  A query row whose keys are all masked
 * by -inf gives zeros.  Replaces the "sdpa_recomp_fwd" node that hpu::fp8_sdpa_recomp_fwd
 * builds with requires_backward false and dropout 0 (Fp8SDPARecompFwd::AddNode,
 * hpu_ops/backend/sdpa_gen.cpp:806-1000; schema habana_eager/eager_custom_op_register.cpp:
 * 2286-2296; the dropout flags have no counterpart here).
 *
 * q is [batch..., q_len, head_dim_qk], k [batch..., kv_len, head_dim_qk], v [batch..., kv_len,
 * head_dim_v], out [batch..., q_len, head_dim_v], the mask [batch..., q_len, kv_len] with unit
 * column stride.  The up to three batch extents (outermost first, 1 where unused) are walked
 * with one stride per tensor and extent, in elements; 0 broadcasts (grouped-query attention:
 * k and v have stride 0 along the heads of a group).  ld* are row pitches in elements; ldmask 0
 * repeats one mask row for all queries.  Head dimensions up to 256.
 *
 * scale_dev[6] / scale_host[6] hold d_scale_q, d_scale_k, d_scale_v, q_scale_s, q_scale_o,
 * d_scale_s in that order: a device scalar where the pointer is not NULL, else the host value,
 * 0 = absent (scale_dev itself may be NULL).  q_scale_o is read only for an e4m3fn out.
 * amax_s / amax_o, where not NULL, receive max softmax probability and max |out| (before
 * q_scale_o) as one fp32 each.
 */
typedef enum {
  MI355Q_SDPA_MASK_NONE = 0,
  MI355Q_SDPA_MASK_BOOL = 1, /* one byte per element, 0 = masked out */
  MI355Q_SDPA_MASK_BF16 = 2, /* added to the scaled score */
  MI355Q_SDPA_MASK_F32 = 3
} mi355q_sdpa_mask_kind;

typedef struct mi355q_sdpa_desc {
  int64_t batch[3];
  int64_t q_bstride[3], k_bstride[3], v_bstride[3], mask_bstride[3], out_bstride[3];
  int64_t q_len, kv_len, head_dim_qk, head_dim_v;
  int64_t ldq, ldk, ldv, ldmask, ldo;
  /* Per-batch key window (the op's valid_seq_len / seq_padding_type, flags VALID_SEQ_LEN_PRESENT,
   * SEQ_PADDING_LEFT / RIGHT of sdpa_gen.cpp:849-851, 902-904): valid_seq_len, where not NULL, holds
   * batch[valid_seq_dim] int32 values on the device; entry b of that batch dimension attends to its
   * last valid_seq_len[b] keys (seq_padding_left != 0: the padding sits in front) or its first
   * (seq_padding_left == 0), on top of the causal mask.  Values are clamped to [0, kv_len]; a query
   * row left with no key gives zeros. */
  const int32_t* valid_seq_len;
  int32_t valid_seq_dim;
  int32_t seq_padding_left;
} mi355q_sdpa_desc;

/*
 * Few queries against many keys (decoding: at most 32 rows of (innermost batch index, query) that
 * share a k and v, kv_len >= 512, head dimensions up to 128, 16-byte aligned rows) run on a kernel
 * that splits the keys over workgroups; the splits' partial results pass through `workspace`
 * (device memory, 4-byte aligned, mi355q_fp8_sdpa_workspace_bytes(desc) bytes, 0 when the problem
 * does not split), and the workgroup of a group that finishes last merges them (one launch).  The
 * workspace begins with 1 KiB of arrival counters: it has to be zero-filled before its first use,
 * every call leaves the counters zero, so it can be passed again as it is (to this entry point,
 * for any problem it is large enough for); calls that may overlap in time need workspaces of
 * their own.  Without a workspace of that size the call still works, one workgroup per group of
 * rows.  Nothing is allocated here.
 */
size_t mi355q_fp8_sdpa_workspace_bytes(const mi355q_sdpa_desc* desc);
/* How the few-queries kernel would walk the keys of a problem with a workspace of that size:
 * returns the number of key splits and stores the 64-key blocks per split (0 and 0 when the
 * problem takes the other kernel).  Inside a split the four waves take every fourth block.  The
 * probabilities are rounded to fp8 against each wave's own running maximum, so results depend
 * on this walk in their last fp8-rounding digit; for logs, and for tests that restate it. */
int mi355q_fp8_sdpa_key_splits(const mi355q_sdpa_desc* desc, int64_t* blocks_per_split);
int mi355q_fp8_sdpa_fwd(const void* q, const void* k, const void* v, int fp8_fmt, const void* mask,
                        int mask_kind, void* out, int out_dtype, const mi355q_sdpa_desc* desc,
                        float softmax_scale, int is_causal, const float* const* scale_dev,
                        const float* scale_host, float* amax_s, float* amax_o, void* workspace,
                        size_t workspace_bytes, void* stream);

/* Name of the kernel variant mi355q_fp8_gemm would pick for a problem
 * (for logs and profiles; static string). */
const char* mi355q_fp8_gemm_variant(int trans_a, int64_t lda, int trans_b, int64_t ldb,
                                    int64_t M, int64_t N, int64_t K);

#ifdef __cplusplus
}
#endif
#endif /* MI355Q_H */
