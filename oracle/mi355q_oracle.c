/*
 * CPU oracle for the fp8 / int4 quantized-inference op family.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP library, the
 * torch extension, the Python package) may call, link or import this file.
 * It is a plain-C restatement of the semantics that the reference pins for
 *   hpu::cast_to_fp8_v2, hpu::cast_from_fp8, hpu::fp8_gemm_v2,
 *   hpu::convert_from_int4, hpu::convert_from_uint4
 * and exists so that tests can compare the gfx950 kernels against it.
 *
 * The reference holds no arithmetic for these ops (each is one Synapse graph
 * node: hpu_ops/backend/fp8_ops.cpp:219,251-252,280,304-305,421,486-493 and
 * hpu_ops/backend/int4_ops.cpp:48-53), so every function below cites the
 * reference test or shim line that fixes its behaviour.
 *
 * Pinned / unpinned status of each function (pins live in tests/):
 *   ora_f32_to_fp8 (normal range, RNE)    pinned: closed form of
 *        tests/pytest_working/fp8_utils.py:58-79, PyTorch CPU float8 cast
 *        (accepted as ground truth by any_mode/test_hpu_cast.py:35-55),
 *        exhaustive over all bf16 patterns.
 *   saturation                            pinned: KATs of
 *        any_mode/test_hpu_fp8_ops_any_mode.py:224-243.
 *   subnormal outputs (gradual underflow) pinned only against PyTorch CPU's
 *        cast; the reference's tests never reach them -> parity unpinned at
 *        the reference boundary.
 *   NaN -> 0x7F|sign, +-Inf -> +-max      parity unpinned (own choice: NaN as
 *        PyTorch CPU encodes it, Inf saturates like any overflow).
 *   ora_cast_to_fp8 bf16 double rounding  pinned: test :85-87,130.
 *   amax                                  pinned: test :132-136; amax of a
 *        tensor holding NaN is NaN here -> parity unpinned.
 *   ora_cast_from_fp8                     pinned: test :87,105,130 and the
 *        256-code decode tables vs PyTorch CPU.
 *   ora_dequant_4bit                      pinned: nibble order/sign
 *        test_hpu_convert_from_int4.py:41-71,104-105; group layout :224-247,
 *        434-470; brute force over all nibble values and positions.
 *        (q - z) with packed uint4 z > q is plain signed here -> parity
 *        unpinned for that wrap-around case (test :116-118 avoids it).
 *   ora_fp8_gemm                          values pinned to tolerance by test
 *        :361-476,599-704 and by exact small-integer cases; order of scale /
 *        bias / accumulate / rounding in the epilogue is parity unpinned.
 *   stochastic rounding                   no oracle function: the random bit
 *        stream is parity unpinned; tests check what the reference's do
 *        (any_mode/test_hpu_fp8_ops_any_mode.py:124-128, test_hpu_fp8_te.py:
 *        105-150): each result is one of the two fp8 neighbours of the exact
 *        value, the mean is preserved, round-to-nearest differs.
 *   ora_silu_mul_bf16                     no reference counterpart (the glue
 *        between the MLP block's projections is left to aten there); pinned
 *        against a double-precision evaluation on all 65536 bf16 inputs (18
 *        differ, all below -88 where the true result is under 3.3e-37) and
 *        against PyTorch's CPU silu (tests/test_oracle_silu.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORA_F32 0
#define ORA_BF16 1
#define ORA_E4M3FN 2
#define ORA_E5M2 3

/* scale broadcast modes shared with the HIP library's C ABI */
#define ORA_SCALE_NONE 0
#define ORA_SCALE_HOST 1   /* one value passed by value */
#define ORA_SCALE_DEV 2    /* one value behind the pointer */
#define ORA_SCALE_MID 3    /* x viewed [outer, mid, inner]; scale[mid] */
#define ORA_SCALE_FULL 4   /* one scale per element */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- bf16 <-> fp32 ---------------------------------------------------- */

float ora_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* round-to-nearest-even; NaN stays NaN (quiet bit forced), as PyTorch CPU */
uint16_t ora_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t keep = u >> 16;
  uint32_t rest = u & 0xffffu;
  if (rest > 0x8000u || (rest == 0x8000u && (keep & 1u))) keep += 1;
  return (uint16_t)keep;
}

/* ---- SiLU(gate) * up in bf16 (the glue between the gate / up and the down
 * projections of the decoder MLP block; not an op of the reference, which
 * leaves it to aten) -----------------------------------------------------
 * silu(x) = x / (1 + exp(-x)) evaluated in fp32 with a spelled-out exp
 * (Cody-Waite reduction by ln 2 in two parts, the degree-5 polynomial of
 * Cephes' expf, an exact scaling by a power of two), rounded to bf16; the product
 * with `up` (exact in fp32) is rounded to bf16 again.  Every operation is an
 * IEEE add, multiply, divide or fused multiply-add, written out one by one, so
 * that the GPU kernel, which uses the same sequence, gets the same bits.
 */
static float exp_spelled_out(float t) { /* -87 <= t <= 88 */
  const float n = rintf(t * 1.44269504088896341f);
  float r = fmaf(n, -0.693145751953125f, t);
  r = fmaf(n, -1.42860682030941723212e-6f, r);
  float q = 1.9875691500e-4f;
  q = fmaf(q, r, 1.3981999507e-3f);
  q = fmaf(q, r, 8.3334519073e-3f);
  q = fmaf(q, r, 4.1665795894e-2f);
  q = fmaf(q, r, 1.6666665459e-1f);
  q = fmaf(q, r, 5.0000001201e-1f);
  float y = fmaf(q, r * r, r);
  y = y + 1.0f;
  return ldexpf(y, (int)n);
}

float ora_silu_f32(float x) {
  const float t = -x;
  /* fminf / fmaxf return the other operand for a NaN, so the exp never sees one */
  float e = exp_spelled_out(fminf(fmaxf(t, -87.0f), 88.0f));
  if (t > 88.0f) e = INFINITY;
  if (t < -87.0f) e = 0.0f;
  return x / (1.0f + e);
}

void ora_silu_mul_bf16(const uint16_t* gate, const uint16_t* up, uint16_t* h, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    const float s = ora_bf16_to_f32(ora_f32_to_bf16(ora_silu_f32(ora_bf16_to_f32(gate[i]))));
    h[i] = ora_f32_to_bf16(s * ora_bf16_to_f32(up[i]));
  }
}

/* ---- fp32 -> fp8 -------------------------------------------------------
 * Round to nearest even onto the fp8 grid with gradual underflow, then
 * saturate to the largest finite value (e4m3fn 448 = 0x7E, e5m2 57344 = 0x7B):
 * test_hpu_fp8_ops_any_mode.py:224-243 ([1000,500,-500,-1000] -> +-448 and
 * [1e5,6e4,-6e4,-1e5] -> +-57344).  The rounding itself is what
 * fp8_utils.py:58-79 states as "add half-ulp-minus-one plus the odd bit, then
 * mask"; it is restated here from the value instead of from that bit trick.
 */
static uint8_t f32_to_fp8_generic(float f, int mbits, int bias, uint8_t max_code) {
  uint32_t u = f2u(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu); /* NaN */
  if (a == 0x7f800000u) return (uint8_t)(sign | max_code); /* Inf saturates */
  int e32 = (int)(a >> 23);
  if (e32 == 0) return sign; /* fp32 subnormal: far below half the fp8 quantum */
  int e = e32 - 127;
  int emin = 1 - bias; /* exponent of the smallest fp8 normal */
  uint32_t mant = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift = 23 - mbits + (e < emin ? emin - e : 0);
  uint32_t r;
  if (shift > 25) {
    r = 0; /* below half of the smallest subnormal */
  } else {
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    r = mant >> shift;
    if (rem > half || (rem == half && (r & 1u))) r += 1;
  }
  uint32_t code;
  if (e >= emin) {
    /* r carries the implicit one: r in [2^mbits, 2^(mbits+1)] */
    code = ((uint32_t)(e + bias - 1) << mbits) + r;
  } else {
    code = r; /* subnormal, or exactly the smallest normal when r == 2^mbits */
  }
  if (code > max_code) code = max_code;
  return (uint8_t)(sign | code);
}

uint8_t ora_f32_to_e4m3fn(float f) { return f32_to_fp8_generic(f, 3, 7, 0x7e); }
uint8_t ora_f32_to_e5m2(float f) { return f32_to_fp8_generic(f, 2, 15, 0x7b); }

uint8_t ora_f32_to_fp8(float f, int fmt) {
  return fmt == ORA_E5M2 ? ora_f32_to_e5m2(f) : ora_f32_to_e4m3fn(f);
}

/* ---- fp8 -> fp32 (exact) --------------------------------------------- */

float ora_e4m3fn_to_f32(uint8_t c) {
  int s = c >> 7, e = (c >> 3) & 0xf, m = c & 7;
  float v;
  if (e == 0xf && m == 7) v = NAN; /* the only NaN of e4m3fn; there is no Inf */
  else if (e == 0) v = ldexpf((float)m, -9); /* m/8 * 2^-6 */
  else v = ldexpf((float)(8 + m), e - 10);   /* (1+m/8) * 2^(e-7) */
  return s ? -v : v;
}

float ora_e5m2_to_f32(uint8_t c) {
  int s = c >> 7, e = (c >> 2) & 0x1f, m = c & 3;
  float v;
  if (e == 0x1f) v = m ? NAN : INFINITY;
  else if (e == 0) v = ldexpf((float)m, -16); /* m/4 * 2^-14 */
  else v = ldexpf((float)(4 + m), e - 17);    /* (1+m/4) * 2^(e-15) */
  return s ? -v : v;
}

float ora_fp8_to_f32(uint8_t c, int fmt) {
  return fmt == ORA_E5M2 ? ora_e5m2_to_f32(c) : ora_e4m3fn_to_f32(c);
}

/* ---- scale lookup ------------------------------------------------------
 * hpu_ops/backend/fp8_ops.cpp:29-100: a scale is None, one value, or a
 * vector reshaped to scale_shape and broadcast against the input
 * (test :64-83: [R,1] per row, [1,C] per column of the trailing dims).
 */
static inline float scale_at(const float* scale, float host, int mode,
                             int64_t i, int64_t mid, int64_t inner) {
  switch (mode) {
    case ORA_SCALE_HOST: return host;
    case ORA_SCALE_DEV: return scale[0];
    case ORA_SCALE_MID: return scale[(i / inner) % mid];
    case ORA_SCALE_FULL: return scale[i];
    default: return 1.0f;
  }
}

/* ---- cast_to_fp8_v2 -----------------------------------------------------
 * test_hpu_fp8_ops_any_mode.py:85-87,130: expected = fp8_round(input *
 * scale.to(input.dtype)) with torch.equal, so for bf16 input the scale is
 * first rounded to bf16 and the product is rounded to bf16 before the fp8
 * rounding; for fp32 input both happen in fp32.  amax = max|input| over the
 * unscaled input, fp32 (test :132-134).  Returns amax through *amax when it
 * is non-NULL.  NaN in the input makes amax NaN.
 */
void ora_cast_to_fp8(const void* x, int in_dtype, uint8_t* y, int fmt,
                     const float* scale, float scale_host, int mode,
                     int64_t n, int64_t mid, int64_t inner, float* amax) {
  float mx = 0.0f;
  int saw_nan = 0;
  for (int64_t i = 0; i < n; ++i) {
    float s = scale_at(scale, scale_host, mode, i, mid, inner);
    float v, p;
    if (in_dtype == ORA_BF16) {
      v = ora_bf16_to_f32(((const uint16_t*)x)[i]);
      float sb = ora_bf16_to_f32(ora_f32_to_bf16(s));
      p = ora_bf16_to_f32(ora_f32_to_bf16(v * sb));
    } else {
      v = ((const float*)x)[i];
      p = v * s;
    }
    y[i] = ora_f32_to_fp8(p, fmt);
    if (v != v) saw_nan = 1;
    float av = fabsf(v);
    if (av > mx) mx = av;
  }
  if (amax) *amax = saw_nan ? NAN : mx;
}

/* max|x| alone, and per row of a [rows, cols] view (the per-token amax that
 * dynamic quantisation needs; the reference has no op for it). */
void ora_amax(const void* x, int in_dtype, int64_t rows, int64_t cols, float* out) {
  for (int64_t r = 0; r < rows; ++r) {
    float mx = 0.0f;
    int saw_nan = 0;
    for (int64_t c = 0; c < cols; ++c) {
      int64_t i = r * cols + c;
      float v = in_dtype == ORA_BF16 ? ora_bf16_to_f32(((const uint16_t*)x)[i])
                                     : ((const float*)x)[i];
      if (v != v) saw_nan = 1;
      float av = fabsf(v);
      if (av > mx) mx = av;
    }
    out[r] = saw_nan ? NAN : mx;
  }
}

/* ---- cast_from_fp8 ------------------------------------------------------
 * test :87,105,130: expected = fp8_value * scale_inv.to(dtype), computed in
 * the output dtype.  fp8 -> bf16/fp32 is exact, so for bf16 output this is
 * one bf16 multiply: scale rounded to bf16, product rounded once.
 */
void ora_cast_from_fp8(const uint8_t* x, int fmt, void* y, int out_dtype,
                       const float* scale, float scale_host, int mode,
                       int64_t n, int64_t mid, int64_t inner) {
  for (int64_t i = 0; i < n; ++i) {
    float v = ora_fp8_to_f32(x[i], fmt);
    float s = scale_at(scale, scale_host, mode, i, mid, inner);
    if (out_dtype == ORA_BF16) {
      float sb = ora_bf16_to_f32(ora_f32_to_bf16(s));
      float p = mode == ORA_SCALE_NONE ? v : v * sb;
      ((uint16_t*)y)[i] = ora_f32_to_bf16(p);
    } else {
      ((float*)y)[i] = mode == ORA_SCALE_NONE ? v : v * s;
    }
  }
}

/* ---- convert_from_int4 / convert_from_uint4 -----------------------------
 * test_hpu_convert_from_int4.py:41-49,57-71: element 8p+i of the last dim
 * sits in bits [4i, 4i+4) of packed word p.  :104-105: int4 nibbles >= 8
 * mean value-16.  out = (q - z) * s.
 *   packed [rows, pcols] int32 -> out [rows, 8*pcols]
 *   scale  [rows/group, 8*pcols] in the output dtype (group == 1: same shape
 *          as the output, test :108; group > 1: AutoGPTQ layout, :434-470)
 *   zp_kind 0: none; 1: float tensor shaped like scale, in the output dtype
 *          (subtraction then happens in the output dtype: test :127-130);
 *          2: packed int32 [rows/group, pcols] with the same nibble order
 *          (subtraction exact in integers, test :125-126).
 * Packed zero-points carry the signedness of the op (int4: signed nibble).
 */
static inline int nibble(int32_t w, int i, int is_signed) {
  int q = (int)(((uint32_t)w >> (4 * i)) & 0xfu);
  if (is_signed && q >= 8) q -= 16;
  return q;
}

void ora_dequant_4bit(const int32_t* packed, const void* scale, const void* zp,
                      int zp_kind, int is_signed, int out_dtype, int64_t rows,
                      int64_t pcols, int64_t group, void* out) {
  int64_t cols = pcols * 8;
  for (int64_t r = 0; r < rows; ++r) {
    int64_t g = r / group;
    for (int64_t c = 0; c < cols; ++c) {
      int q = nibble(packed[r * pcols + c / 8], (int)(c % 8), is_signed);
      int64_t si = g * cols + c;
      if (out_dtype == ORA_BF16) {
        float s = ora_bf16_to_f32(((const uint16_t*)scale)[si]);
        float d;
        if (zp_kind == 2) {
          int z = nibble(((const int32_t*)zp)[g * pcols + c / 8], (int)(c % 8), is_signed);
          d = (float)(q - z);
        } else if (zp_kind == 1) {
          float z = ora_bf16_to_f32(((const uint16_t*)zp)[si]);
          d = ora_bf16_to_f32(ora_f32_to_bf16((float)q - z));
        } else {
          d = (float)q;
        }
        ((uint16_t*)out)[r * cols + c] = ora_f32_to_bf16(d * s);
      } else {
        float s = ((const float*)scale)[si];
        float d;
        if (zp_kind == 2) {
          int z = nibble(((const int32_t*)zp)[g * pcols + c / 8], (int)(c % 8), is_signed);
          d = (float)(q - z);
        } else if (zp_kind == 1) {
          d = (float)q - ((const float*)zp)[si];
        } else {
          d = (float)q;
        }
        ((float*)out)[r * cols + c] = d * s;
      }
    }
  }
}

/* ---- fp8_gemm_v2 ---------------------------------------------------------
 * hpu_ops/backend/fp8_ops.cpp:403-496: C = op(A) @ op(B) on the fp8 values,
 * times A_scale_inv and B_scale_inv, plus bias, plus D when accumulating,
 * cast to the output dtype.  One [M,K]x[K,N] problem; batching and 1-D
 * operands are resolved by the caller.  Strides are in elements so that
 * transposed operands need no copy: A(m,k) = A[m*a_sm + k*a_sk].
 *   sa_mode/sb_mode: 0 none, 1 host scalar, 2 one device value,
 *                    3 per output row [M], 4 per output column [N]
 *   bias_mode: 0 none, 1 vector [N], 2 full [M,N]; bias and D are in the
 *              output dtype.
 * Epilogue order chosen here (the reference does not pin it): fp32
 * accumulate over k in ascending order, v = acc*sA, v = v*sB, v += bias,
 * v += D, one final rounding to the output dtype.
 */
void ora_fp8_gemm(const uint8_t* A, int fmt_a, int64_t a_sm, int64_t a_sk,
                  const uint8_t* B, int fmt_b, int64_t b_sk, int64_t b_sn,
                  int64_t M, int64_t N, int64_t K,
                  const float* sa, float sa_host, int sa_mode,
                  const float* sb, float sb_host, int sb_mode,
                  const void* bias, int bias_mode, const void* D,
                  int out_dtype, void* C) {
  float lut_a[256], lut_b[256];
  for (int i = 0; i < 256; ++i) {
    lut_a[i] = ora_fp8_to_f32((uint8_t)i, fmt_a);
    lut_b[i] = ora_fp8_to_f32((uint8_t)i, fmt_b);
  }
  float* brow = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
  float* acol = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t k = 0; k < K; ++k) acol[k] = lut_a[A[m * a_sm + k * a_sk]];
    for (int64_t n = 0; n < N; ++n) {
      for (int64_t k = 0; k < K; ++k) brow[k] = lut_b[B[k * b_sk + n * b_sn]];
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) acc += acol[k] * brow[k];
      float va = 1.0f, vb = 1.0f;
      if (sa_mode == 1) va = sa_host; else if (sa_mode == 2) va = sa[0];
      else if (sa_mode == 3) va = sa[m]; else if (sa_mode == 4) va = sa[n];
      if (sb_mode == 1) vb = sb_host; else if (sb_mode == 2) vb = sb[0];
      else if (sb_mode == 3) vb = sb[m]; else if (sb_mode == 4) vb = sb[n];
      float v = acc * va;
      v = v * vb;
      int64_t o = m * N + n;
      if (out_dtype == ORA_BF16) {
        if (bias_mode == 1) v += ora_bf16_to_f32(((const uint16_t*)bias)[n]);
        else if (bias_mode == 2) v += ora_bf16_to_f32(((const uint16_t*)bias)[o]);
        if (D) v += ora_bf16_to_f32(((const uint16_t*)D)[o]);
        ((uint16_t*)C)[o] = ora_f32_to_bf16(v);
      } else {
        if (bias_mode == 1) v += ((const float*)bias)[n];
        else if (bias_mode == 2) v += ((const float*)bias)[o];
        if (D) v += ((const float*)D)[o];
        ((float*)C)[o] = v;
      }
    }
  }
  free(brow);
  free(acol);
}
