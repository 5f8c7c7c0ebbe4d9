// torch.ops.hpu.* host layer on PyTorch-ROCm: schemas, argument checks, output
// allocation and the calls into the mi355q C ABI.
//
// The schema strings are those of the reference
// (habana_eager/eager_custom_op_register.cpp:2146-2171); the checks and error
// strings follow CastToFp8V2::AddNode, CastFromFp8::AddNode, Fp8GemmV2::AddNode
// (hpu_ops/backend/fp8_ops.cpp:29-53,192-308,403-496), Int4BaseOp
// (hpu_ops/backend/int4_ops.cpp:22-56) and getBatchMatmulOutShape
// (hpu_ops/common/batched_matmul_output_shape.cpp:33-85).  Output shapes and
// dtypes for tracing follow dynamo/_custom_op_meta_registrations.py:56-217.
//
// Kernels are registered for the CUDA dispatch key (the key PyTorch-ROCm uses
// for HIP tensors) and for Meta.  There is no CPU implementation: a CPU tensor
// fails in the dispatcher.
#include <ATen/ATen.h>
#include <ATen/hip/HIPGeneratorImpl.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPGraphsC10Utils.h>
#include <torch/library.h>

#include <cstdlib>
#include <iostream>
#include <map>
#include <tuple>
#include <mutex>
#include <sstream>

#include "../../include/mi355q.h"

namespace {

using at::Tensor;
using c10::IValue;
using OptShape = c10::optional<std::vector<int64_t>>;
// PyTorch-ROCm presents HIP devices under the name "cuda".
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

bool log_enabled() {
  static const bool on = [] {
    const char* e = std::getenv("MI355Q_LOG");
    return e != nullptr && e[0] != '\0' && e[0] != '0';
  }();
  return on;
}

#define MI355Q_OP_INFO(...)                                   \
  do {                                                        \
    if (log_enabled()) {                                      \
      std::ostringstream os__;                                \
      os__ << "[mi355q] " << __VA_ARGS__ << "\n";             \
      std::cerr << os__.str();                                \
    }                                                         \
  } while (0)

void check_status(int st, const char* what) {
  TORCH_CHECK(st == MI355Q_OK, what, " failed: ", mi355q_status_string(st));
}

bool is_fp8(at::ScalarType t) {
  return t == at::kFloat8_e5m2 || t == at::kFloat8_e4m3fn;
}

int to_mi355q_dtype(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return MI355Q_F32;
    case at::kBFloat16: return MI355Q_BF16;
    case at::kFloat8_e4m3fn: return MI355Q_E4M3FN;
    case at::kFloat8_e5m2: return MI355Q_E5M2;
    default: TORCH_CHECK(false, "mi355q: unsupported dtype ", t);
  }
}

void* current_stream(const Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream());
}

int64_t prod(at::IntArrayRef v, size_t b, size_t e) {
  int64_t p = 1;
  for (size_t i = b; i < e; ++i) p *= v[i];
  return p;
}

// ValidateScaleShape, hpu_ops/backend/fp8_ops.cpp:29-53
void validate_scale_shape(const IValue& scale, const OptShape& scale_shape) {
  if (scale.isNone() || scale.isDouble() || !scale_shape.has_value()) return;
  int64_t scale_numel = 0;
  if (scale.isTensor()) scale_numel = scale.toTensor().numel();
  else if (scale.isDoubleList()) scale_numel = (int64_t)scale.toDoubleVector().size();
  int64_t shape_numel = 1;
  for (auto d : *scale_shape) shape_numel *= d;
  TORCH_CHECK(scale_numel == shape_numel, "Number of scale elements (", scale_numel,
              ") is not equal to number of scale_shape elements (", shape_numel, ").");
}

// A cast scale resolved against the input shape, ready for the C ABI.
struct CastScale {
  Tensor holder;  // keeps device memory alive
  const float* dev = nullptr;
  float host = 1.0f;
  int mode = MI355Q_SCALE_NONE;
  int64_t outer = 1, mid = 1, inner = 1;
};

Tensor list_to_device(const std::vector<double>& v, const Tensor& like) {
  Tensor cpu = at::empty({(int64_t)v.size()}, at::TensorOptions().dtype(at::kFloat));
  float* p = cpu.data_ptr<float>();
  for (size_t i = 0; i < v.size(); ++i) p[i] = (float)v[i];
  return cpu.to(like.device());
}

CastScale resolve_cast_scale(const IValue& scale, const OptShape& scale_shape, const Tensor& x) {
  CastScale r;
  const int64_t n = x.numel();
  r.outer = n;
  if (scale.isNone()) return r;
  if (scale.isDouble()) {
    r.mode = MI355Q_SCALE_HOST;
    r.host = (float)scale.toDouble();
    return r;
  }
  Tensor s;
  if (scale.isDoubleList()) {
    auto v = scale.toDoubleVector();
    TORCH_CHECK(!v.empty(), "scale list must not be empty");
    if (v.size() == 1) {
      r.mode = MI355Q_SCALE_HOST;
      r.host = (float)v[0];
      return r;
    }
    s = list_to_device(v, x);
  } else {
    TORCH_CHECK(scale.isTensor(), "scale must be None, a Tensor, a float or a list of floats");
    s = scale.toTensor();
    TORCH_CHECK(s.device() == x.device(), "scale must be on the same device as input, got ",
                s.device(), " and ", x.device());
    s = s.to(at::kFloat).contiguous();
  }
  if (s.numel() == 1) {
    r.holder = s;
    r.dev = s.data_ptr<float>();
    r.mode = MI355Q_SCALE_DEV;
    return r;
  }
  std::vector<int64_t> shp = scale_shape.has_value() ? *scale_shape : s.sizes().vec();
  const auto xs = x.sizes();
  TORCH_CHECK(shp.size() <= xs.size(), "scale shape ", at::IntArrayRef(shp),
              " is not broadcastable to input shape ", xs);
  std::vector<int64_t> full(xs.size(), 1);
  std::copy(shp.begin(), shp.end(), full.begin() + (xs.size() - shp.size()));
  for (size_t i = 0; i < xs.size(); ++i)
    TORCH_CHECK(full[i] == 1 || full[i] == xs[i], "scale shape ", at::IntArrayRef(shp),
                " is not broadcastable to input shape ", xs);
  // One contiguous run of dims where the scale is not broadcast -> [outer, mid, inner].
  size_t a = 0;
  while (a < full.size() && (full[a] == 1)) ++a;
  size_t b = full.size();
  while (b > a && (full[b - 1] == 1)) --b;
  bool run = true;
  for (size_t i = a; i < b; ++i) run = run && (full[i] == xs[i]);
  if (run) {
    r.holder = s;
    r.dev = s.data_ptr<float>();
    r.outer = prod(xs, 0, a);
    r.mid = prod(xs, a, b);
    r.inner = prod(xs, b, xs.size());
    if (r.outer == 1 && r.inner == 1) {
      r.mode = MI355Q_SCALE_FULL;
      r.outer = n;
      r.mid = r.inner = 1;
    } else {
      r.mode = MI355Q_SCALE_MID;
    }
    return r;
  }
  Tensor e = s.reshape(full).expand(xs).contiguous();
  r.holder = e;
  r.dev = e.data_ptr<float>();
  r.mode = MI355Q_SCALE_FULL;
  return r;
}

// (seed, offset) for `numel` stochastically rounded elements, drawn from the
// device's default generator the way torch's own random kernels do, so that
// torch.manual_seed makes the cast reproducible and successive casts differ.
std::pair<uint64_t, uint64_t> reserve_random(const Tensor& t, int64_t numel) {
  auto gen = at::get_generator_or_default<at::CUDAGeneratorImpl>(
      c10::nullopt, at::cuda::detail::getDefaultCUDAGenerator(t.device().index()));
  std::lock_guard<std::mutex> lock(gen->mutex_);
  return gen->philox_engine_inputs((uint64_t)((numel + 1) / 2));
}

// PT_HPU_STOCHASTIC_ROUNDING_MODE (scripts/env_flags.yaml:753-758, default 1): 1 makes the stochastic casts
// from bfloat16 to e5m2 flush to zero below the smallest normal number (is_sr_sftz, hpu_ops/fp8_ops.h:52),
// 0 leaves them plain stochastic rounding.  Read once, as the reference does.
bool sr_flush_to_zero_mode() {
  static const bool on = [] {
    const char* v = std::getenv("PT_HPU_STOCHASTIC_ROUNDING_MODE");
    return v == nullptr || std::atoi(v) == 1;
  }();
  return on;
}

// One call for both rounding modes.
int launch_cast_to(const Tensor& x, Tensor& out, const CastScale& cs, float* amax, bool stochastic) {
  const int xd = to_mi355q_dtype(x.scalar_type()), od = to_mi355q_dtype(out.scalar_type());
  if (!stochastic)
    return mi355q_cast_to_fp8(x.data_ptr(), xd, out.data_ptr(), od, cs.dev, cs.host, cs.mode, cs.outer, cs.mid,
                              cs.inner, amax, current_stream(x));
  const auto r = reserve_random(x, x.numel());
  // GetCastParams, fp8_ops.cpp:105-119: SFTZ only from bfloat16 to e5m2
  const bool sftz = sr_flush_to_zero_mode() && x.scalar_type() == at::kBFloat16 && out.scalar_type() == at::kFloat8_e5m2;
  return mi355q_cast_to_fp8_sr(x.data_ptr(), xd, out.data_ptr(), od, cs.dev, cs.host, cs.mode, cs.outer, cs.mid,
                               cs.inner, amax, r.first, r.second, sftz ? 1 : 0, current_stream(x));
}

// ------------------------------------------------------------ cast_to_fp8_v2

void check_cast_to_args(const Tensor& input, bool stochastic_rounding, bool is_amax,
                        const IValue& dtype_iv, const IValue& scale, const OptShape& scale_shape) {
  const auto src = input.scalar_type();
  const bool fp8_in = is_fp8(src);
  TORCH_CHECK(fp8_in || src == at::kFloat || src == at::kBFloat16,
              "CastToFp8V2 input dtype must be one of [float, bfloat16, float8_e5m2, float8_e4m3fn].");
  TORCH_CHECK(!dtype_iv.isNone(),
              "cast_to_fp8_v2: dtype must be given (torch.float8_e4m3fn or torch.float8_e5m2)");
  const auto dst = dtype_iv.toScalarType();
  TORCH_CHECK(is_fp8(dst), "cast_to_fp8_v2: dtype must be torch.float8_e4m3fn or torch.float8_e5m2, got ", dst);
  if (fp8_in) {
    TORCH_CHECK(!is_amax, "CastToFp8V2 must have no amax for float8.");
    TORCH_CHECK(src == dst, "CastToFp8V2 input and output must have the same dtype for float8, but are ",
                src, " and ", dst);
  }
  validate_scale_shape(scale, scale_shape);
  TORCH_CHECK(!(stochastic_rounding && fp8_in), "cast_to_fp8_v2: stochastic rounding needs a float or bfloat16 input");
}

OptShape shape_from_ivalue(const IValue& v) {
  if (v.isNone()) return c10::nullopt;
  return v.toIntVector();
}

// Stack layout (all three overloads): input, scale, stochastic_rounding,
// is_amax, dtype, scale_shape.  The .scalar overload ignores scale_shape
// (eager_custom_op_register.cpp:92-101).
void cast_to_fp8_v2_boxed(const c10::OperatorHandle& op, c10::DispatchKeySet, torch::jit::Stack* stack) {
  TORCH_CHECK(stack->size() >= 6, "cast_to_fp8_v2 expects 6 arguments");
  const size_t base = stack->size() - 6;
  Tensor input = (*stack)[base + 0].toTensor();
  IValue scale = (*stack)[base + 1];
  const bool sr = (*stack)[base + 2].toBool();
  const bool is_amax = (*stack)[base + 3].toBool();
  IValue dtype_iv = (*stack)[base + 4];
  OptShape scale_shape = scale.isDouble() ? c10::nullopt : shape_from_ivalue((*stack)[base + 5]);
  (void)op;

  check_cast_to_args(input, sr, is_amax, dtype_iv, scale, scale_shape);
  const auto dst = dtype_iv.toScalarType();
  MI355Q_OP_INFO("cast_to_fp8_v2 : input=" << input.sizes() << " " << input.scalar_type()
                                           << " is_amax=" << is_amax << " dtype=" << dst);

  Tensor out, amax;
  if (input.is_meta()) {
    out = at::empty(input.sizes(), input.options().dtype(dst));
    amax = at::empty(is_amax ? std::vector<int64_t>{} : std::vector<int64_t>{0},
                     input.options().dtype(at::kFloat));
  } else {
    DeviceGuard guard(input.device());
    Tensor x = input.contiguous();
    out = at::empty(x.sizes(), x.options().dtype(dst));
    amax = at::empty(is_amax ? std::vector<int64_t>{} : std::vector<int64_t>{0},
                     x.options().dtype(at::kFloat));
    CastScale cs;
    if (is_fp8(x.scalar_type())) {
      cs.outer = x.numel();  // fp8 -> same fp8: copy, scale plays no part
    } else {
      cs = resolve_cast_scale(scale, scale_shape, x);
    }
    check_status(launch_cast_to(x, out, cs, is_amax ? amax.data_ptr<float>() : nullptr, sr), "mi355q_cast_to_fp8");
  }
  torch::jit::drop(*stack, 6);
  stack->emplace_back(std::move(out));
  stack->emplace_back(std::move(amax));
}

// ------------------------------------------------------------- cast_from_fp8

Tensor cast_from_fp8_impl(const Tensor& input, const IValue& scale, at::ScalarType out_dtype,
                          const OptShape& scale_shape) {
  validate_scale_shape(scale, scale_shape);
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kBFloat16,
              "CastFromFp8 output dtype must be equal to float or bfloat16.");
  TORCH_CHECK(is_fp8(input.scalar_type()), "CastFromFp8 input must be float8_e5m2 or float8_e4m3fn, got ",
              input.scalar_type());
  MI355Q_OP_INFO("cast_from_fp8 : input=" << input.sizes() << " " << input.scalar_type()
                                          << " out_dtype=" << out_dtype);
  if (input.is_meta()) return at::empty(input.sizes(), input.options().dtype(out_dtype));
  DeviceGuard guard(input.device());
  Tensor x = input.contiguous();
  Tensor out = at::empty(x.sizes(), x.options().dtype(out_dtype));
  CastScale cs = resolve_cast_scale(scale, scale_shape, x);
  check_status(mi355q_cast_from_fp8(x.data_ptr(), to_mi355q_dtype(x.scalar_type()), out.data_ptr(),
                                    to_mi355q_dtype(out_dtype), cs.dev, cs.host, cs.mode, cs.outer,
                                    cs.mid, cs.inner, current_stream(x)),
               "mi355q_cast_from_fp8");
  return out;
}

OptShape to_opt_shape(at::OptionalIntArrayRef s) {
  if (!s.has_value()) return c10::nullopt;
  return s->vec();
}

Tensor cast_from_fp8(const Tensor& input, const c10::optional<Tensor>& scale, at::ScalarType out_dtype,
                     at::OptionalIntArrayRef scale_shape) {
  return cast_from_fp8_impl(input, scale.has_value() ? IValue(*scale) : IValue(), out_dtype,
                            to_opt_shape(scale_shape));
}
Tensor cast_from_fp8_scalar(const Tensor& input, double scale, at::ScalarType out_dtype,
                            at::OptionalIntArrayRef) {
  return cast_from_fp8_impl(input, IValue(scale), out_dtype, c10::nullopt);
}
Tensor cast_from_fp8_scalar_list(const Tensor& input, c10::ArrayRef<double> scale,
                                 at::ScalarType out_dtype, at::OptionalIntArrayRef scale_shape) {
  return cast_from_fp8_impl(input, IValue(scale.vec()), out_dtype, to_opt_shape(scale_shape));
}

// --------------------------------------------------------------- fp8_gemm_v2

// torch.matmul shape rule with optional transposes of the last two dims
// (getBatchMatmulOutShape, hpu_ops/common/batched_matmul_output_shape.cpp:33-85).
std::vector<int64_t> matmul_out_shape(at::IntArrayRef a, at::IntArrayRef b, bool ta, bool tb) {
  const size_t ra = a.size(), rb = b.size();
  TORCH_CHECK(ra >= 1 && rb >= 1, "fp8_gemm_v2 operands must have at least 1 dimension");
  std::vector<int64_t> tail;
  int64_t ka = a[0], kb = b[0];
  if (ra > 1) {
    tail.push_back(ta ? a[ra - 1] : a[ra - 2]);
    ka = ta ? a[ra - 2] : a[ra - 1];
  }
  if (rb > 1) {
    tail.push_back(tb ? b[rb - 2] : b[rb - 1]);
    kb = tb ? b[rb - 1] : b[rb - 2];
  }
  TORCH_CHECK(ka == kb, "Common dimension sizes of matmul inputs should be the same. Got ", ka,
              " and ", kb);
  const size_t mr = std::max(ra, rb);
  std::vector<int64_t> out;
  for (size_t i = mr; i >= 3; --i) {
    const int64_t da = i > ra ? 1 : a[ra - i];
    const int64_t db = i > rb ? 1 : b[rb - i];
    TORCH_CHECK(da == db || da == 1 || db == 1, "Batch dimension ", mr - i,
                " of matmul inputs should be the same or at least one of them should be equal to 1. Got ",
                da, " and ", db);
    out.push_back(da == db ? da : da * db);
  }
  out.insert(out.end(), tail.begin(), tail.end());
  return out;
}

struct GemmScale {
  Tensor holder;
  const float* dev = nullptr;
  float host = 1.0f;
  int mode = MI355Q_GS_NONE;
};

GemmScale resolve_gemm_scale(const IValue& scale, const OptShape& shape, int64_t M, int64_t N,
                             const Tensor& like, const char* name) {
  GemmScale r;
  if (scale.isNone()) return r;
  if (scale.isDouble()) {
    r.mode = MI355Q_GS_HOST;
    r.host = (float)scale.toDouble();
    return r;
  }
  Tensor s;
  if (scale.isDoubleList()) {
    auto v = scale.toDoubleVector();
    TORCH_CHECK(!v.empty(), name, " list must not be empty");
    if (v.size() == 1) {
      r.mode = MI355Q_GS_HOST;
      r.host = (float)v[0];
      return r;
    }
    s = list_to_device(v, like);
  } else {
    s = scale.toTensor();
    TORCH_CHECK(s.device() == like.device(), name, " must be on the same device as A");
    s = s.to(at::kFloat).contiguous();
  }
  r.holder = s;
  r.dev = s.data_ptr<float>();
  if (s.numel() == 1) {
    r.mode = MI355Q_GS_DEV;
    return r;
  }
  std::vector<int64_t> shp = shape.has_value() ? *shape : s.sizes().vec();
  while (shp.size() > 2 && shp.front() == 1) shp.erase(shp.begin());
  if (shp.size() == 1) shp.insert(shp.begin(), 1);
  TORCH_CHECK(shp.size() == 2, name, " with shape ", at::IntArrayRef(shp),
              " does not broadcast against the [M, N] output");
  if (shp[0] == M && shp[1] == 1) r.mode = MI355Q_GS_PER_ROW;
  else if (shp[0] == 1 && shp[1] == N) r.mode = MI355Q_GS_PER_COL;
  else TORCH_CHECK(false, name, " with shape ", at::IntArrayRef(shp),
                   " does not broadcast against the [", M, ", ", N, "] output as [M,1] or [1,N]");
  return r;
}

Tensor fp8_gemm_v2_impl(const Tensor& A, bool trans_A, const Tensor& B, bool trans_B,
                        const c10::optional<Tensor>& D, at::ScalarType out_dtype,
                        const IValue& A_scale_inv, const IValue& B_scale_inv,
                        const c10::optional<Tensor>& bias, bool accumulate,
                        const OptShape& B_scale_shape) {
  std::vector<int64_t> out_shape = matmul_out_shape(A.sizes(), B.sizes(), trans_A, trans_B);
  validate_scale_shape(B_scale_inv, B_scale_shape);
  TORCH_CHECK(!accumulate || D.has_value(),
              "Accumulation tensor must be provided at index 4 for Fp8GemmV2, when accumulate is true");
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kBFloat16,
              "fp8_gemm_v2 output dtype must be float or bfloat16, got ", out_dtype);
  TORCH_CHECK(is_fp8(A.scalar_type()) && is_fp8(B.scalar_type()),
              "fp8_gemm_v2 operands must be float8_e5m2 or float8_e4m3fn, got ", A.scalar_type(),
              " and ", B.scalar_type());
  MI355Q_OP_INFO("fp8_gemm_v2 : A=" << A.sizes() << " trans_A=" << trans_A << " B=" << B.sizes()
                                    << " trans_B=" << trans_B << " out_dtype=" << out_dtype
                                    << " accumulate=" << accumulate);
  if (A.is_meta()) return at::empty(out_shape, A.options().dtype(out_dtype));
  TORCH_CHECK(A.device() == B.device(), "fp8_gemm_v2 operands must be on the same device");
  DeviceGuard guard(A.device());

  // Reduce to batch x [M,K] x [K,N].
  const bool a1 = A.dim() == 1, b1 = B.dim() == 1;
  Tensor a = a1 ? A.unsqueeze(0) : A;  // [1, K]
  Tensor b = b1 ? B.unsqueeze(1) : B;  // [K, 1]
  const bool ta = a1 ? false : trans_A, tb = b1 ? false : trans_B;
  const int64_t ar = a.size(-2), ac = a.size(-1), br = b.size(-2), bc = b.size(-1);
  const int64_t M = ta ? ac : ar, K = ta ? ar : ac, N = tb ? br : bc;
  std::vector<int64_t> batch_shape(out_shape.begin(),
                                   out_shape.end() - ((a1 ? 0 : 1) + (b1 ? 0 : 1)));
  int64_t batch = 1;
  for (auto d : batch_shape) batch *= d;

  auto prep = [&](const Tensor& t, int64_t rows, int64_t cols, int64_t* stride) {
    int64_t tb_numel = t.numel() / std::max<int64_t>(rows * cols, 1);
    if (rows * cols == 0) tb_numel = 1;
    Tensor c;
    if (tb_numel == 1) {
      *stride = 0;
      c = t.reshape({rows, cols}).contiguous();
    } else {
      std::vector<int64_t> full = batch_shape;
      full.push_back(rows);
      full.push_back(cols);
      c = t.expand(full).contiguous();
      *stride = rows * cols;
    }
    return c;
  };
  int64_t stride_a = 0, stride_b = 0;
  Tensor ac_t = prep(a, ar, ac, &stride_a);
  Tensor bc_t = prep(b, br, bc, &stride_b);

  Tensor out = at::empty(out_shape, A.options().dtype(out_dtype));
  if (out.numel() == 0) return out;

  // The MFMA kernels move 16-byte chunks: they need 16-byte aligned operands and pitches and, where
  // K is an operand's contiguous dimension, K % 16 == 0; anything else runs on a simple kernel at a
  // few TFLOP/s.  When the product is large enough for that to cost more than two copies, such
  // operands go into zero-filled buffers with every extent rounded up to 16 (zeros along K add
  // nothing to any sum; padding along m or n is never read into a stored output).
  int64_t lda = ac, ldb = bc, k_call = K;
  auto misaligned = [](const Tensor& t) { return (reinterpret_cast<uintptr_t>(t.data_ptr()) & 15u) != 0; };
  const bool k_ragged = K % 16 != 0 && !(ta && !tb);
  if ((ac % 16 || bc % 16 || k_ragged || misaligned(ac_t) || misaligned(bc_t)) &&
      (double)M * (double)N * (double)K >= (double)(1 << 26)) {
    const int64_t kp = (ta && !tb) ? K : (K + 15) / 16 * 16;  // K is contiguous in neither operand: any K
    auto pad = [&](Tensor& t, int64_t rows, int64_t cols, bool k_is_rows, int64_t* ld, int64_t* stride) {
      const int64_t rp = k_is_rows ? kp : rows, cp = k_is_rows ? (cols + 15) / 16 * 16 : kp;
      if (rp == rows && cp == cols && !misaligned(t)) return;
      std::vector<int64_t> shape = t.sizes().vec();
      shape[shape.size() - 2] = rp;
      shape[shape.size() - 1] = cp;
      Tensor padded = at::zeros(shape, t.options());
      padded.narrow(-2, 0, rows).narrow(-1, 0, cols).copy_(t);
      t = padded;
      *ld = cp;
      if (*stride != 0) *stride = rp * cp;
    };
    pad(ac_t, ar, ac, ta, &lda, &stride_a);    // A is stored [K, M] when transposed
    pad(bc_t, br, bc, !tb, &ldb, &stride_b);   // B is stored [K, N] unless transposed
    k_call = kp;
  }

  // A [..., M, K] times one matrix B is one product over all batch * M rows: B is streamed once
  // and the rows fill the kernels' tiles, where batch separate problems would each re-read B with
  // M rows only (a [64, 1, K] decode activation against [K, N] weights would be 64 one-row products).
  const bool can_flatten = batch > 1 && stride_b == 0 && stride_a != 0 && !ta;
  // Per-row scales that cover the batch as well ([..., M, 1], what quantize_rows returns for a
  // batched activation) are per-row scales of the flattened product.
  auto batched_rows = [&](const IValue& sc) {
    if (!can_flatten || !sc.isTensor()) return false;
    const Tensor& t = sc.toTensor();
    if (t.numel() != batch * M || t.numel() == 1 || t.dim() != (int64_t)batch_shape.size() + 2) return false;
    for (size_t i = 0; i < batch_shape.size(); ++i)
      if (t.size(i) != batch_shape[i]) return false;
    return t.size(-2) == M && t.size(-1) == 1;
  };
  const bool sa_batched = batched_rows(A_scale_inv);
  GemmScale sa = sa_batched ? resolve_gemm_scale(A_scale_inv, std::vector<int64_t>{batch * M, 1}, batch * M, N, A, "A_scale_inv")
                            : resolve_gemm_scale(A_scale_inv, c10::nullopt, M, N, A, "A_scale_inv");
  GemmScale sb = resolve_gemm_scale(B_scale_inv, B_scale_shape, M, N, A, "B_scale_inv");
  int64_t m_call = M, batch_call = batch;
  if (can_flatten) {
    // [M] scales shared by every batch element are repeated per batch element
    auto repeat_rows = [&](GemmScale& g) {
      g.holder = g.holder.reshape({1, M}).expand({batch, M}).contiguous();
      g.dev = g.holder.data_ptr<float>();
    };
    if (sa.mode == MI355Q_GS_PER_ROW && !sa_batched) repeat_rows(sa);
    if (sb.mode == MI355Q_GS_PER_ROW) repeat_rows(sb);
    m_call = batch * M;
    batch_call = 1;
  }

  std::vector<int64_t> full_out = batch_shape;
  full_out.push_back(M);
  full_out.push_back(N);

  Tensor bias_t, d_t;
  int bias_mode = MI355Q_BIAS_NONE;
  int64_t ldbias = 0, stride_bias = 0, stride_d = 0;
  if (bias.has_value() && bias->defined()) {
    bias_t = bias->to(out_dtype);
    if (!b1 && bias_t.dim() <= 1 && bias_t.numel() == N) {
      bias_t = bias_t.contiguous();
      bias_mode = MI355Q_BIAS_ROW_VECTOR;
    } else {
      // broadcast against the output as torch would, then view as [batch, M, N]
      bias_t = bias_t.expand(out_shape).reshape(full_out).contiguous();
      bias_mode = MI355Q_BIAS_FULL;
      ldbias = N;
      stride_bias = M * N;
    }
  }
  if (accumulate) {
    d_t = D->to(out_dtype).expand(out_shape).reshape(full_out).contiguous();
    stride_d = M * N;
  }

  check_status(
      mi355q_fp8_gemm(ac_t.data_ptr(), to_mi355q_dtype(A.scalar_type()), ta ? 1 : 0, lda,
                      bc_t.data_ptr(), to_mi355q_dtype(B.scalar_type()), tb ? 1 : 0, ldb,
                      out.data_ptr(), to_mi355q_dtype(out_dtype), N, m_call, N, k_call, sa.dev, sa.host, sa.mode,
                      sb.dev, sb.host, sb.mode, bias_mode != MI355Q_BIAS_NONE ? bias_t.data_ptr() : nullptr,
                      bias_mode, ldbias, accumulate ? d_t.data_ptr() : nullptr, N, batch_call, stride_a,
                      stride_b, M * N, stride_d, stride_bias, current_stream(A)),
      "mi355q_fp8_gemm");
  return out;
}

IValue opt_tensor_iv(const c10::optional<Tensor>& t) {
  return (t.has_value() && t->defined()) ? IValue(*t) : IValue();
}

Tensor fp8_gemm_v2(const Tensor& A, bool trans_A, const Tensor& B, bool trans_B,
                   const c10::optional<Tensor>& D, at::ScalarType out_dtype,
                   const c10::optional<Tensor>& A_scale_inv, const c10::optional<Tensor>& B_scale_inv,
                   const c10::optional<Tensor>& bias, bool accumulate,
                   at::OptionalIntArrayRef B_scale_shape) {
  return fp8_gemm_v2_impl(A, trans_A, B, trans_B, D, out_dtype, opt_tensor_iv(A_scale_inv),
                          opt_tensor_iv(B_scale_inv), bias, accumulate, to_opt_shape(B_scale_shape));
}
Tensor fp8_gemm_v2_scalar(const Tensor& A, bool trans_A, const Tensor& B, bool trans_B,
                          const c10::optional<Tensor>& D, at::ScalarType out_dtype, double A_scale_inv,
                          double B_scale_inv, const c10::optional<Tensor>& bias, bool accumulate,
                          at::OptionalIntArrayRef) {
  return fp8_gemm_v2_impl(A, trans_A, B, trans_B, D, out_dtype, IValue(A_scale_inv),
                          IValue(B_scale_inv), bias, accumulate, c10::nullopt);
}
Tensor fp8_gemm_v2_scalar_list(const Tensor& A, bool trans_A, const Tensor& B, bool trans_B,
                               const c10::optional<Tensor>& D, at::ScalarType out_dtype,
                               c10::ArrayRef<double> A_scale_inv, c10::ArrayRef<double> B_scale_inv,
                               const c10::optional<Tensor>& bias, bool accumulate,
                               at::OptionalIntArrayRef B_scale_shape) {
  return fp8_gemm_v2_impl(A, trans_A, B, trans_B, D, out_dtype, IValue(A_scale_inv.vec()),
                          IValue(B_scale_inv.vec()), bias, accumulate, to_opt_shape(B_scale_shape));
}

// ------------------------------------------------ v1 ops (caller-allocated outputs)
//
// hpu::cast_to_fp8 and hpu::fp8_gemm, the deprecated forms that write into
// tensors the caller passes (CastToFp8::AddNode, hpu_ops/backend/fp8_ops.cpp:
// 123-166; Fp8Gemm::AddNode :312-366).  Same arithmetic as the v2 ops.

std::tuple<Tensor&, Tensor&> cast_to_fp8_v1(const Tensor& input, const c10::optional<Tensor>& scale,
                                            bool stochastic_rounding, Tensor& out, Tensor& amax) {
  const auto src = input.scalar_type();
  TORCH_CHECK(src == at::kFloat || src == at::kBFloat16, "CastToFp8 input must be of float or bfloat16 dtype.");
  TORCH_CHECK(input.sizes() == out.sizes(), "Input and output must have the same shape");
  TORCH_CHECK(is_fp8(out.scalar_type()), "cast_to_fp8: out must be float8_e4m3fn or float8_e5m2, got ", out.scalar_type());
  const bool is_amax = amax.numel() != 0;  // fp8_ops.cpp:138
  TORCH_CHECK(!is_amax || amax.scalar_type() == at::kFloat, "cast_to_fp8: amax must be a float tensor");
  if (input.is_meta()) return std::tuple<Tensor&, Tensor&>(out, amax);
  DeviceGuard guard(input.device());
  Tensor x = input.contiguous();
  Tensor y = out.is_contiguous() ? out : at::empty(x.sizes(), x.options().dtype(out.scalar_type()));
  Tensor am = is_amax ? at::empty({}, x.options().dtype(at::kFloat)) : Tensor();
  CastScale cs = resolve_cast_scale(opt_tensor_iv(scale), c10::nullopt, x);
  check_status(launch_cast_to(x, y, cs, is_amax ? am.data_ptr<float>() : nullptr, stochastic_rounding),
               "mi355q_cast_to_fp8");
  if (!y.is_same(out)) out.copy_(y);
  if (is_amax) amax.copy_(am.expand(amax.sizes()));
  return std::tuple<Tensor&, Tensor&>(out, amax);
}

Tensor& fp8_gemm_v1(const Tensor& A, bool trans_A, const Tensor& B, bool trans_B, const Tensor& D,
                    at::ScalarType out_dtype, const c10::optional<Tensor>& A_scale_inv,
                    const c10::optional<Tensor>& B_scale_inv, const c10::optional<Tensor>& bias,
                    bool accumulate, Tensor& out) {
  TORCH_CHECK(out.scalar_type() == out_dtype, "fp8_gemm: out has dtype ", out.scalar_type(),
              " but out_dtype is ", out_dtype);
  // D may be the very tensor `out`: the result is complete before it is copied in
  Tensor r = fp8_gemm_v2_impl(A, trans_A, B, trans_B, c10::optional<Tensor>(D), out_dtype,
                              opt_tensor_iv(A_scale_inv), opt_tensor_iv(B_scale_inv), bias, accumulate,
                              c10::nullopt);
  TORCH_CHECK(r.sizes() == out.sizes(), "fp8_gemm: out has shape ", out.sizes(), ", the product has ", r.sizes());
  if (!out.is_meta()) out.copy_(r);
  return out;
}

// ------------------------------------------------------- cast_to_fp8_hybrid
//
// hpu::cast_to_fp8_hybrid (scripts/hpu_op.yaml:7365-7371; CastToFp8HybridMeta and
// CastToFp8Hybrid::AddNode, hpu_ops/backend/cast_to_fp8_hybrid_gen.cpp:39-100).
std::tuple<Tensor, Tensor, Tensor> cast_to_fp8_hybrid(const Tensor& input, const c10::optional<Tensor>& scale_152,
                                                      const c10::optional<Tensor>& scale_143,
                                                      bool stochastic_rounding, bool is_amax) {
  const auto src = input.scalar_type();
  TORCH_CHECK(src == at::kFloat || src == at::kBFloat16, "CastToFp8Hybrid input must be of float or bfloat16 dtype.");
  auto scalar_scale = [&](const c10::optional<Tensor>& s, const char* name) -> Tensor {
    if (!s.has_value() || !s->defined()) return Tensor();
    TORCH_CHECK(s->numel() == 1, "cast_to_fp8_hybrid: ", name, " must hold one element, got ", s->numel());
    if (s->is_meta()) return *s;
    TORCH_CHECK(s->device() == input.device(), "cast_to_fp8_hybrid: ", name, " must be on the device of input");
    return s->to(at::kFloat).contiguous();
  };
  Tensor s5 = scalar_scale(scale_152, "scale_152"), s4 = scalar_scale(scale_143, "scale_143");
  const std::vector<int64_t> amax_shape = is_amax ? std::vector<int64_t>{} : std::vector<int64_t>{0};
  if (input.is_meta())
    return {at::empty(input.sizes(), input.options().dtype(at::kFloat8_e5m2)),
            at::empty(input.sizes(), input.options().dtype(at::kFloat8_e4m3fn)),
            at::empty(amax_shape, input.options().dtype(at::kFloat))};
  DeviceGuard guard(input.device());
  Tensor x = input.contiguous();
  Tensor y5 = at::empty(x.sizes(), x.options().dtype(at::kFloat8_e5m2));
  Tensor y4 = at::empty(x.sizes(), x.options().dtype(at::kFloat8_e4m3fn));
  Tensor amax = at::empty(amax_shape, x.options().dtype(at::kFloat));
  std::pair<uint64_t, uint64_t> r{0, 0};
  if (stochastic_rounding) r = reserve_random(x, x.numel());
  check_status(mi355q_cast_to_fp8_hybrid(x.data_ptr(), to_mi355q_dtype(src), x.numel(), y5.data_ptr(), y4.data_ptr(),
                                         s5.defined() ? s5.data_ptr<float>() : nullptr,
                                         s4.defined() ? s4.data_ptr<float>() : nullptr,
                                         // CastToFp8HybridParams, cast_to_fp8_hybrid_gen.cpp:26-35: SFTZ for a bfloat16 input
                                         !stochastic_rounding ? 0 : (sr_flush_to_zero_mode() && src == at::kBFloat16 ? 2 : 1),
                                         r.first, r.second, is_amax ? amax.data_ptr<float>() : nullptr,
                                         current_stream(x)),
               "mi355q_cast_to_fp8_hybrid");
  return {y5, y4, amax};
}

// ------------------------------------------------- convert_from_int4 / uint4

Tensor convert_from_int4_common(const char* op_name, bool is_signed, const Tensor& input,
                                const Tensor& scale, const c10::optional<Tensor>& zero_point,
                                at::ScalarType out_dtype) {
  TORCH_CHECK(input.scalar_type() == at::kInt, op_name, " input must be int32 (8 nibbles per element), got ",
              input.scalar_type());
  TORCH_CHECK(input.dim() >= 1, op_name, " input must have at least 1 dimension");
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kBFloat16, op_name,
              " output dtype must be float or bfloat16, got ", out_dtype);
  std::vector<int64_t> out_shape = input.sizes().vec();
  out_shape.back() *= 8;
  MI355Q_OP_INFO(op_name << " : input=" << input.sizes() << " scale=" << scale.sizes()
                         << " out_dtype=" << out_dtype);
  if (input.is_meta()) return at::empty(out_shape, input.options().dtype(out_dtype));
  DeviceGuard guard(input.device());

  const int64_t pcols = input.size(-1);
  const int64_t cols = pcols * 8;
  const int64_t rows = pcols ? input.numel() / pcols : 0;
  Tensor out = at::empty(out_shape, input.options().dtype(out_dtype));
  if (out.numel() == 0) return out;

  TORCH_CHECK(scale.device() == input.device(), op_name, " scale must be on the same device as input");
  TORCH_CHECK(scale.numel() > 0 && scale.numel() % cols == 0 && scale.size(-1) == cols, op_name,
              " scale last dimension must equal 8 * input last dimension (", cols, "), got ",
              scale.sizes());
  const int64_t srows = scale.numel() / cols;
  TORCH_CHECK(rows % srows == 0, op_name, " scale rows (", srows, ") must divide input rows (", rows, ")");
  const int64_t group = rows / srows;
  TORCH_CHECK(group == 1 || input.dim() == 2, op_name,
              " group-wise scales need a 2-D input, got ", input.sizes());
  auto aligned16 = [](const Tensor& t) {
    return t.is_contiguous() && (reinterpret_cast<uintptr_t>(t.data_ptr()) & 15u) == 0;
  };
  Tensor x = input.contiguous();
  Tensor s = scale.to(out_dtype);
  if (!aligned16(s)) s = s.clone(at::MemoryFormat::Contiguous);
  Tensor z;
  int zp_kind = MI355Q_ZP_NONE;
  if (zero_point.has_value() && zero_point->defined()) {
    TORCH_CHECK(zero_point->device() == input.device(), op_name,
                " zero_point must be on the same device as input");
    if (zero_point->scalar_type() == at::kInt) {
      TORCH_CHECK(zero_point->numel() == srows * pcols, op_name,
                  " packed zero_point must hold one nibble per scale element, got ",
                  zero_point->sizes(), " for scale ", scale.sizes());
      z = zero_point->contiguous();
      zp_kind = MI355Q_ZP_PACKED;
    } else {
      TORCH_CHECK(zero_point->numel() == scale.numel(), op_name,
                  " zero_point must have the shape of scale, got ", zero_point->sizes(), " and ",
                  scale.sizes());
      z = zero_point->to(out_dtype);
      if (!aligned16(z)) z = z.clone(at::MemoryFormat::Contiguous);
      zp_kind = MI355Q_ZP_FLOAT;
    }
  }
  check_status(mi355q_dequant_4bit(x.data_ptr<int32_t>(), s.data_ptr(),
                                   zp_kind != MI355Q_ZP_NONE ? z.data_ptr() : nullptr, zp_kind,
                                   is_signed ? 1 : 0, to_mi355q_dtype(out_dtype), rows, pcols, group,
                                   out.data_ptr(), current_stream(x)),
               "mi355q_dequant_4bit");
  return out;
}

Tensor convert_from_int4(const Tensor& input, const Tensor& scale,
                         const c10::optional<Tensor>& zero_point, at::ScalarType out_dtype) {
  return convert_from_int4_common("convert_from_int4", true, input, scale, zero_point, out_dtype);
}
Tensor convert_from_uint4(const Tensor& input, const Tensor& scale,
                          const c10::optional<Tensor>& zero_point, at::ScalarType out_dtype) {
  return convert_from_int4_common("convert_from_uint4", false, input, scale, zero_point, out_dtype);
}

// ---------------------------------------------------------------- w4a8_gemm
//
// Fused int4-dequant GEMM: fp8 activations [..., K] times the packed 4-bit weights that
// hpu::convert_from_int4 / convert_from_uint4 take (int4_ops.cpp:40-56), without the bf16 [K, N]
// matrix in between.  out = out_dtype((A @ ((q - z) * s)) * A_scale_inv + bias).  The reference has no
// fused op; shapes the kernel does not take raise (there is no second route to the same bits).
//
// The kernel's split over K keeps arrival counters in its workspace, which have to be zero when a
// call starts and are left zero by every call (the key splits of the attention kernel for few
// queries do the same): one zero-filled buffer per (device, stream, op) is kept here and grown on
// demand, so that a call launches one kernel and nothing else.  Calls on one stream run in order,
// which is all the sharing the buffer allows; the two ops lay their counters out differently and
// do not share.  While a stream is being captured into a graph no kept buffer is handed out (its
// memory would belong to the graph's pool, and replays of two graphs could overlap): the call takes
// a buffer of the graph's own and clears its counters with a fill kernel that is part of the graph
// (captured_ticket_workspace).
enum TicketWorkspaceOp { kWsW4a8 = 0, kWsSdpa = 1, kWsW4a16 = 2 };
struct TicketWorkspaceCache {
  std::mutex mu;
  std::map<std::tuple<int, void*, int>, Tensor> map;
};
TicketWorkspaceCache& ticket_workspace_cache() {
  // never destroyed: a static Tensor would be freed after the HIP runtime has shut down
  static auto* cache = new TicketWorkspaceCache();
  return *cache;
}
void ticket_workspace_cache_erase(int device, void* stream, int op) {
  TicketWorkspaceCache& c = ticket_workspace_cache();
  std::lock_guard<std::mutex> lock(c.mu);
  c.map.erase(std::make_tuple(device, stream, op));
}
Tensor ticket_workspace(const Tensor& like, size_t bytes, TicketWorkspaceOp op) {
  if (bytes == 0 || c10::hip::currentStreamCaptureStatusMayInitCtx() != c10::hip::CaptureStatus::None) return Tensor();
  TicketWorkspaceCache& c = ticket_workspace_cache();
  std::lock_guard<std::mutex> lock(c.mu);
  Tensor& t = c.map[std::make_tuple((int)like.device().index(), current_stream(like), (int)op)];
  if (!t.defined() || (size_t)t.numel() < bytes) t = at::zeros({(int64_t)bytes}, like.options().dtype(at::kByte));
  return t;
}
// While the stream is being captured: a buffer out of the graph's pool, its first KiB (the arrival counters of
// every op that uses one) zeroed by a small fill kernel, which every replay runs again; the rest (partial sums
// that are written before they are read) as it comes.
Tensor captured_ticket_workspace(const Tensor& like, size_t bytes) {
  Tensor t = at::empty({(int64_t)bytes}, like.options().dtype(at::kByte));
  t.narrow(0, 0, std::min<int64_t>((int64_t)bytes, 1024)).zero_();
  return t;
}
bool stream_is_capturing() { return c10::hip::currentStreamCaptureStatusMayInitCtx() != c10::hip::CaptureStatus::None; }
// After a call that used the buffer has failed: its counters may be left non-zero (no workgroup then draws a
// group's last ticket and the output stays unwritten), so the buffer is dropped and the next call starts from a
// zero-filled one.
void drop_ticket_workspace(const Tensor& like, TicketWorkspaceOp op) {
  ticket_workspace_cache_erase((int)like.device().index(), current_stream(like), (int)op);
}

Tensor w4a8_gemm(const Tensor& A, const Tensor& packed, const Tensor& scale, const c10::optional<Tensor>& zero_point,
                 bool is_signed, at::ScalarType out_dtype, const c10::optional<Tensor>& A_scale_inv,
                 const c10::optional<Tensor>& bias) {
  TORCH_CHECK(is_fp8(A.scalar_type()), "mi355q::w4a8_gemm A must be float8_e4m3fn or float8_e5m2, got ", A.scalar_type());
  TORCH_CHECK(packed.scalar_type() == at::kInt && packed.dim() == 2,
              "mi355q::w4a8_gemm packed weights must be a 2-D int32 tensor [K, N / 8], got ", packed.scalar_type(), " ", packed.sizes());
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kBFloat16, "mi355q::w4a8_gemm out_dtype must be float or bfloat16, got ", out_dtype);
  TORCH_CHECK(A.dim() >= 1, "mi355q::w4a8_gemm A must have at least 1 dimension");
  const int64_t K = packed.size(0), N = packed.size(1) * 8;
  TORCH_CHECK(A.size(-1) == K, "Common dimension sizes of matmul inputs should be the same. Got ", A.size(-1), " and ", K);
  TORCH_CHECK(scale.dim() == 2 && scale.size(1) == N && scale.size(0) > 0 && K % scale.size(0) == 0,
              "mi355q::w4a8_gemm scale must be [K / group, N] = [*, ", N, "], got ", scale.sizes());
  const int64_t groups = scale.size(0), group = K / groups;
  const bool has_zp = zero_point.has_value() && zero_point->defined();
  if (has_zp)
    TORCH_CHECK(zero_point->scalar_type() == at::kInt && zero_point->dim() == 2 && zero_point->size(0) == groups &&
                    zero_point->size(1) == N / 8,
                "mi355q::w4a8_gemm zero_point must be packed int32 [K / group, N / 8], got ", zero_point->scalar_type(), " ",
                zero_point->sizes());
  std::vector<int64_t> out_shape(A.sizes().begin(), A.sizes().end());
  out_shape.back() = N;
  // every pointer the kernel dereferences: a host (or other GPU's) zero_point or bias would be a memory fault on the device
  TORCH_CHECK(!has_zp || zero_point->device() == A.device(), "mi355q::w4a8_gemm zero_point must be on the same device as A, got ",
              has_zp ? zero_point->device() : A.device(), " and ", A.device());
  TORCH_CHECK(!(bias.has_value() && bias->defined()) || bias->device() == A.device(),
              "mi355q::w4a8_gemm bias must be on the same device as A, got ", (bias.has_value() && bias->defined()) ? bias->device() : A.device(),
              " and ", A.device());
  if (A.is_meta()) return at::empty(out_shape, A.options().dtype(out_dtype));
  TORCH_CHECK(A.device() == packed.device() && A.device() == scale.device(), "mi355q::w4a8_gemm operands must be on the same device");
  DeviceGuard guard(A.device());
  Tensor a = A.contiguous();
  const int64_t M = K ? a.numel() / K : 0;
  Tensor out = at::empty(out_shape, A.options().dtype(out_dtype));
  if (out.numel() == 0) return out;
  Tensor w = packed.contiguous();
  Tensor s = (scale.scalar_type() == at::kBFloat16 ? scale : scale.to(at::kFloat)).contiguous();
  Tensor z;
  if (has_zp) z = zero_point->contiguous();
  Tensor sa_t;
  const float* sa_dev = nullptr;
  int sa_mode = MI355Q_GS_NONE;
  if (A_scale_inv.has_value() && A_scale_inv->defined()) {
    sa_t = A_scale_inv->to(at::kFloat).contiguous();
    TORCH_CHECK(sa_t.device() == A.device(), "A_scale_inv must be on the same device as A");
    TORCH_CHECK(sa_t.numel() == 1 || sa_t.numel() == M, "A_scale_inv must hold one value or one per row of A (", M, "), got ", sa_t.sizes());
    sa_dev = sa_t.data_ptr<float>();
    sa_mode = (sa_t.numel() == 1 && M != 1) ? MI355Q_GS_DEV : (sa_t.numel() == 1 ? MI355Q_GS_DEV : MI355Q_GS_PER_ROW);
  }
  Tensor b;
  if (bias.has_value() && bias->defined()) {
    TORCH_CHECK(bias->numel() == N, "Bias must be size ", N, " but got ", bias->numel());
    b = bias->to(out_dtype).contiguous();
  }
  MI355Q_OP_INFO("w4a8_gemm : A=" << A.sizes() << " packed=" << packed.sizes() << " group=" << group << " signed=" << is_signed);
  // the buffer kept per stream, or under graph capture one of the graph's own with its counters cleared
  const size_t ws_bytes = mi355q_w4a8_gemm_workspace_bytes(M, N, K, group, to_mi355q_dtype(s.scalar_type()));
  const bool kept = !stream_is_capturing();
  Tensor ws = kept ? ticket_workspace(a, ws_bytes, kWsW4a8) : (ws_bytes ? captured_ticket_workspace(a, ws_bytes) : Tensor());
  const int st = mi355q_w4a8_gemm(a.data_ptr(), to_mi355q_dtype(a.scalar_type()), K, w.data_ptr<int32_t>(), N / 8, s.data_ptr(),
                                  to_mi355q_dtype(s.scalar_type()), has_zp ? z.data_ptr<int32_t>() : nullptr, is_signed ? 1 : 0,
                                  group, out.data_ptr(), to_mi355q_dtype(out_dtype), N, M, N, K, sa_dev, 1.0f, sa_mode,
                                  b.defined() ? b.data_ptr() : nullptr, ws.defined() ? ws.data_ptr() : nullptr,
                                  ws.defined() ? (size_t)ws.numel() : 0, current_stream(a));
  if (st != MI355Q_OK && ws.defined() && kept) drop_ticket_workspace(a, kWsW4a8);
  TORCH_CHECK(st != MI355Q_ERR_UNSUPPORTED,
              "mi355q::w4a8_gemm takes groups that are multiples of 128, N a multiple of 32 and K a multiple of 16 (got group ",
              group, ", N ", N, ", K ", K, "); expand the weights with hpu::convert_from_", is_signed ? "int4" : "uint4", " for other shapes");
  check_status(st, "mi355q_w4a8_gemm");
  return out;
}

// mi355q::w4a16_gemm: the same weights against bf16 activations (what the reference gets from
// convert_from_[u]int4 to bf16 followed by a bf16 matmul, hpu_ops/backend/int4_ops.cpp:40-56), without the
// bf16 [K, N] matrix: the activations go through the matrix unit as two fp8 planes (mi355q_w4a16_gemm).
Tensor w4a16_gemm(const Tensor& A, const Tensor& packed, const Tensor& scale, const c10::optional<Tensor>& zero_point,
                  bool is_signed, at::ScalarType out_dtype, const c10::optional<Tensor>& bias) {
  TORCH_CHECK(A.scalar_type() == at::kBFloat16, "mi355q::w4a16_gemm A must be bfloat16, got ", A.scalar_type());
  TORCH_CHECK(packed.scalar_type() == at::kInt && packed.dim() == 2,
              "mi355q::w4a16_gemm packed weights must be a 2-D int32 tensor [K, N / 8], got ", packed.scalar_type(), " ", packed.sizes());
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kBFloat16, "mi355q::w4a16_gemm out_dtype must be float or bfloat16, got ", out_dtype);
  TORCH_CHECK(A.dim() >= 1, "mi355q::w4a16_gemm A must have at least 1 dimension");
  const int64_t K = packed.size(0), N = packed.size(1) * 8;
  TORCH_CHECK(A.size(-1) == K, "Common dimension sizes of matmul inputs should be the same. Got ", A.size(-1), " and ", K);
  TORCH_CHECK(scale.dim() == 2 && scale.size(1) == N && scale.size(0) > 0 && K % scale.size(0) == 0,
              "mi355q::w4a16_gemm scale must be [K / group, N] = [*, ", N, "], got ", scale.sizes());
  const int64_t groups = scale.size(0), group = K / groups;
  const bool has_zp = zero_point.has_value() && zero_point->defined();
  if (has_zp)
    TORCH_CHECK(zero_point->scalar_type() == at::kInt && zero_point->dim() == 2 && zero_point->size(0) == groups &&
                    zero_point->size(1) == N / 8,
                "mi355q::w4a16_gemm zero_point must be packed int32 [K / group, N / 8], got ", zero_point->scalar_type(), " ",
                zero_point->sizes());
  const bool has_bias = bias.has_value() && bias->defined();
  TORCH_CHECK(!has_bias || bias->numel() == N, "Bias must be size ", N, " but got ", has_bias ? bias->numel() : 0);
  std::vector<int64_t> out_shape(A.sizes().begin(), A.sizes().end());
  out_shape.back() = N;
  TORCH_CHECK(A.device() == packed.device() && A.device() == scale.device(), "mi355q::w4a16_gemm operands must be on the same device");
  TORCH_CHECK(!has_zp || zero_point->device() == A.device(), "mi355q::w4a16_gemm zero_point must be on the same device as A");
  TORCH_CHECK(!has_bias || bias->device() == A.device(), "mi355q::w4a16_gemm bias must be on the same device as A");
  if (A.is_meta()) return at::empty(out_shape, A.options().dtype(out_dtype));
  DeviceGuard guard(A.device());
  Tensor a = A.contiguous();
  const int64_t M = K ? a.numel() / K : 0;
  Tensor out = at::empty(out_shape, A.options().dtype(out_dtype));
  if (out.numel() == 0) return out;
  Tensor w = packed.contiguous(), s = scale.contiguous(), z, b;
  if (has_zp) z = zero_point->contiguous();
  if (has_bias) b = bias->to(out_dtype).contiguous();
  MI355Q_OP_INFO("w4a16_gemm : A=" << A.sizes() << " packed=" << packed.sizes() << " group=" << group << " signed=" << is_signed);
  const size_t bytes = mi355q_w4a16_gemm_workspace_bytes(M, N, K, group, to_mi355q_dtype(s.scalar_type()));
  // the buffer kept per stream starts zero-filled, which the split over K needs; under graph capture a buffer of the
  // graph's own with its counters cleared
  const bool kept = !stream_is_capturing();
  Tensor ws = kept ? ticket_workspace(a, bytes, kWsW4a16) : captured_ticket_workspace(a, bytes);
  const int st = mi355q_w4a16_gemm(a.data_ptr(), MI355Q_BF16, K, w.data_ptr<int32_t>(), N / 8, s.data_ptr(),
                                   to_mi355q_dtype(s.scalar_type()), has_zp ? z.data_ptr<int32_t>() : nullptr, is_signed ? 1 : 0, group,
                                   out.data_ptr(), to_mi355q_dtype(out_dtype), N, M, N, K, has_bias ? b.data_ptr() : nullptr,
                                   ws.data_ptr(), (size_t)ws.numel(), 1, current_stream(a));
  if (st != MI355Q_OK && kept) drop_ticket_workspace(a, kWsW4a16);
  TORCH_CHECK(st != MI355Q_ERR_UNSUPPORTED,
              "mi355q::w4a16_gemm takes groups of 128 with bfloat16 scales, N a multiple of 32 and K a multiple of 16 (got group ", group,
              ", ", s.scalar_type(), " scales, N ", N, ", K ", K, "); expand the weights with hpu::convert_from_", is_signed ? "int4" : "uint4",
              " for other shapes");
  check_status(st, "mi355q_w4a16_gemm");
  return out;
}

// ------------------------------------------------------------------ sum_fp8

// hpu::sum_fp8 (hpu_ops/backend/fp8_ops_gen.cpp:20-49): sum of an fp8 tensor over `dim`
// (all dimensions when absent), as out_dtype (the input's dtype when absent).
Tensor sum_fp8(const Tensor& self, at::OptionalIntArrayRef dim, bool keepdim, c10::optional<at::ScalarType> out_dtype) {
  TORCH_CHECK(is_fp8(self.scalar_type()), "sum_fp8 input must be float8_e4m3fn or float8_e5m2, got ", self.scalar_type());
  const at::ScalarType odt = out_dtype.value_or(self.scalar_type());
  TORCH_CHECK(odt == at::kFloat || odt == at::kBFloat16 || is_fp8(odt), "sum_fp8 out_dtype must be float, bfloat16 or an fp8 dtype, got ", odt);
  const int64_t nd = self.dim();
  std::vector<bool> reduced(std::max<int64_t>(nd, 1), false);
  if (!dim.has_value() || dim->empty()) {
    std::fill(reduced.begin(), reduced.end(), true);
  } else {
    for (int64_t d : *dim) {
      const int64_t w = at::maybe_wrap_dim(d, nd);
      TORCH_CHECK(!reduced[w], "dim ", w, " appears multiple times in the list of dims");
      reduced[w] = true;
    }
  }
  std::vector<int64_t> out_shape;
  for (int64_t d = 0; d < nd; ++d) {
    if (!reduced[d]) out_shape.push_back(self.size(d));
    else if (keepdim) out_shape.push_back(1);
  }
  if (self.is_meta()) return at::empty(out_shape, self.options().dtype(odt));
  DeviceGuard guard(self.device());
  // reduced dimensions that are adjacent: [outer, reduce, inner] of the contiguous tensor;
  // else they are moved to the end first (a copy)
  int64_t first = -1, last = -1, count = 0;
  for (int64_t d = 0; d < nd; ++d)
    if (reduced[d]) { if (first < 0) first = d; last = d; ++count; }
  Tensor c;
  int64_t outer = 1, red = 1, inner = 1;
  if (nd == 0 || count == 0) {
    c = self.contiguous();
    red = (nd == 0) ? 1 : 1;
    outer = c.numel();
  } else if (last - first + 1 == count) {
    c = self.contiguous();
    for (int64_t d = 0; d < first; ++d) outer *= c.size(d);
    for (int64_t d = first; d <= last; ++d) red *= c.size(d);
    for (int64_t d = last + 1; d < nd; ++d) inner *= c.size(d);
  } else {
    std::vector<int64_t> perm;
    for (int64_t d = 0; d < nd; ++d) if (!reduced[d]) { perm.push_back(d); outer *= self.size(d); }
    for (int64_t d = 0; d < nd; ++d) if (reduced[d]) { perm.push_back(d); red *= self.size(d); }
    c = self.permute(perm).contiguous();
  }
  Tensor out = at::empty(out_shape, self.options().dtype(odt));
  MI355Q_OP_INFO("sum_fp8 : input=" << self.sizes() << " as [" << outer << ", " << red << ", " << inner << "] -> " << odt);
  if (out.numel() == 0) return out;
  const size_t ws_bytes = mi355q_sum_fp8_workspace_bytes(outer, red, inner);
  Tensor ws;
  if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, self.options().dtype(at::kByte));
  check_status(mi355q_sum_fp8(c.data_ptr(), to_mi355q_dtype(c.scalar_type()), outer, red, inner, out.data_ptr(),
                              to_mi355q_dtype(odt), ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, current_stream(c)),
               "mi355q_sum_fp8");
  return out;
}

// -------------------------------------------------------------- softmax_fp8

struct SoftmaxScale {
  const float* dev = nullptr;
  float host = 1.0f;
  bool given = false;
};

SoftmaxScale softmax_scale(const c10::optional<Tensor>& t, const Tensor& input, const char* name) {
  SoftmaxScale s;
  if (!t.has_value() || !t->defined()) return s;
  // addOptionalTensor, softmax_fp8_gen.cpp:25-40
  TORCH_CHECK(t->scalar_type() == at::kFloat, "Input ", name, " must be of dtype: ", at::kFloat);
  TORCH_CHECK(t->numel() == 1, "softmax_fp8 ", name, " must have one element, got ", t->sizes());
  s.given = true;
  if (!input.is_meta()) {
    TORCH_CHECK(t->device() == input.device(), "softmax_fp8 ", name, " must be on the same device as input");
    s.dev = t->data_ptr<float>();
  }
  return s;
}
SoftmaxScale softmax_scale(double v) {
  SoftmaxScale s;
  s.host = (float)v;
  s.given = true;
  return s;
}

// SoftmaxFp8::AddNode, hpu_ops/backend/softmax_fp8_gen.cpp:73-158 (checks and messages :88-119)
Tensor softmax_fp8_common(const Tensor& input, int64_t dim, const SoftmaxScale& in_scale, const SoftmaxScale& out_scale,
                          const SoftmaxScale& inv_heads, const c10::optional<Tensor>& fused_add) {
  const int64_t rank = input.dim();
  dim = at::maybe_wrap_dim(dim, rank, /*wrap_scalar=*/true);
  const at::ScalarType dt = input.scalar_type();
  TORCH_CHECK(dt == at::kBFloat16 || dt == at::kFloat8_e4m3fn,
              "Input tensor must be of torch.bfloat16 or torch.float8_e4m3fn dtype.");
  TORCH_CHECK(in_scale.given == out_scale.given, "Output and input scales must be both given or None");
  TORCH_CHECK(dt != at::kFloat8_e4m3fn || in_scale.given,
              "If Input is of torch.float8_e4m3fn dtype then input scale must be given.");
  const bool has_add = fused_add.has_value() && fused_add->defined();
  if (has_add) {
    TORCH_CHECK(in_scale.given, "FusedAdd available only for Float8 output, but input scale is not given.");
    TORCH_CHECK(rank == fused_add->dim(), "FusedAdd tensor must have the same rank as the input tensor");
    TORCH_CHECK(rank >= 1 && input.size(0) == fused_add->size(0) && input.size(rank - 1) == fused_add->size(rank - 1),
                "FusedAdd tensor must have the same first and last dim as the input tensor");
    for (int64_t d = 1; d < rank - 1; ++d)
      TORCH_CHECK(fused_add->size(d) == 1 || fused_add->size(d) == input.size(d),
                  "FusedAdd tensor's dim other than first and last should be equal to 1 or the same as the input tensor");
    TORCH_CHECK(fused_add->scalar_type() == at::kBFloat16, "Input fused_add must be of dtype: ", at::kBFloat16);
    TORCH_CHECK(dim == rank - 1, "softmax_fp8 with fused_add is over the last dimension");
    TORCH_CHECK(rank <= 7, "softmax_fp8 with fused_add takes at most 7 dimensions");
  }
  const at::ScalarType odt = in_scale.given ? at::kFloat8_e4m3fn : at::kBFloat16;   // SoftmaxFp8Meta, :65-71
  if (input.is_meta()) return at::empty(input.sizes(), input.options().dtype(odt));
  DeviceGuard guard(input.device());
  if (rank == 0) {  // one element: its softmax is 1
    return softmax_fp8_common(input.reshape({1}), 0, in_scale, out_scale, inv_heads, c10::nullopt).reshape({});
  }
  if (dim != rank - 1) {
    Tensor moved = input.movedim(dim, -1).contiguous();
    return softmax_fp8_common(moved, -1, in_scale, out_scale, inv_heads, c10::nullopt).movedim(-1, dim).contiguous();
  }
  Tensor c = input.contiguous();
  Tensor out = at::empty(c.sizes(), c.options().dtype(odt));
  MI355Q_OP_INFO("softmax_fp8 : input=" << input.sizes() << " " << dt << " -> " << odt << (has_add ? " +fused_add" : ""));
  if (out.numel() == 0) return out;
  const int64_t cols = c.size(-1);
  const int64_t rows = c.numel() / cols;
  Tensor fa;
  std::vector<int64_t> row_sizes, fa_strides;
  if (has_add) {
    TORCH_CHECK(fused_add->device() == c.device(), "softmax_fp8 fused_add must be on the same device as input");
    fa = fused_add->contiguous();
    for (int64_t d = rank - 2; d >= 0; --d) {
      row_sizes.push_back(c.size(d));
      fa_strides.push_back(fa.size(d) == 1 ? 0 : fa.stride(d));
    }
  }
  check_status(mi355q_softmax_fp8(c.data_ptr(), to_mi355q_dtype(dt), rows, cols, in_scale.dev, in_scale.host, out_scale.dev,
                                  out_scale.host, inv_heads.dev, inv_heads.host, has_add ? fa.data_ptr() : nullptr,
                                  (int)row_sizes.size(), row_sizes.data(), fa_strides.data(), out.data_ptr(),
                                  to_mi355q_dtype(odt), current_stream(c)),
               "mi355q_softmax_fp8");
  return out;
}

Tensor softmax_fp8(const Tensor& input, int64_t dim, const c10::optional<Tensor>& input_scale,
                   const c10::optional<Tensor>& output_scale, const c10::optional<Tensor>& inv_attn_heads,
                   const c10::optional<Tensor>& fused_add) {
  return softmax_fp8_common(input, dim, softmax_scale(input_scale, input, "scale"), softmax_scale(output_scale, input, "scale"),
                            softmax_scale(inv_attn_heads, input, "scale"), fused_add);
}
Tensor softmax_fp8_scalar_scales(const Tensor& input, int64_t dim, double input_scale, double output_scale,
                                 const c10::optional<Tensor>& inv_attn_heads, const c10::optional<Tensor>& fused_add) {
  return softmax_fp8_common(input, dim, softmax_scale(input_scale), softmax_scale(output_scale),
                            softmax_scale(inv_attn_heads, input, "scale"), fused_add);
}
Tensor softmax_fp8_scalar(const Tensor& input, int64_t dim, double input_scale, double output_scale, double inv_attn_heads,
                          const c10::optional<Tensor>& fused_add) {
  return softmax_fp8_common(input, dim, softmax_scale(input_scale), softmax_scale(output_scale), softmax_scale(inv_attn_heads),
                            fused_add);
}

// ------------------------------------------------------ fp8_sdpa_recomp_fwd

struct SdpaScale {
  const float* dev = nullptr;
  float host = 0.0f;   // 0 = absent
  Tensor holder;
  bool given() const { return dev != nullptr || host != 0.0f; }
};

// A scale counts as given when it is a tensor with elements or a non-zero number
// (sdpa_add_inputs_and_flags, hpu_ops/backend/sdpa_gen.cpp:868-895).
SdpaScale sdpa_scale(const c10::optional<Tensor>& t, const Tensor& q, const char* name) {
  SdpaScale s;
  if (!t.has_value() || !t->defined() || t->numel() == 0) return s;
  TORCH_CHECK(t->numel() == 1, "fp8_sdpa_recomp_fwd: ", name, " must have one element, got ", t->sizes());
  if (q.is_meta()) {
    s.host = 1.0f;
    return s;
  }
  if (t->is_cpu()) {
    s.host = t->to(at::kFloat).item<float>();
    return s;
  }
  TORCH_CHECK(t->device() == q.device(), "fp8_sdpa_recomp_fwd: ", name, " must be on the same device as q");
  s.holder = t->scalar_type() == at::kFloat ? *t : t->to(at::kFloat);
  s.dev = s.holder.data_ptr<float>();
  return s;
}
SdpaScale sdpa_scale(double v) {
  SdpaScale s;
  s.host = (float)v;
  return s;
}

using SdpaOut = std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor, Tensor>;

// Strides of the up to three batch dimensions of t (rank = batch rank + 2) against the
// broadcast batch shape `bshape`, right aligned; 0 where t is broadcast.
void sdpa_batch_strides(const Tensor& t, const std::vector<int64_t>& bshape, int64_t out[3], const char* name) {
  const int64_t nb = (int64_t)bshape.size(), tb = t.dim() - 2;
  TORCH_CHECK(tb <= nb, "fp8_sdpa_recomp_fwd: ", name, " has more batch dimensions than q, k and v");
  for (int64_t i = 0; i < 3; ++i) out[i] = 0;
  for (int64_t i = 0; i < tb; ++i) {
    const int64_t bd = nb - tb + i;  // dimension of bshape this one aligns with
    TORCH_CHECK(t.size(i) == bshape[bd] || t.size(i) == 1, "fp8_sdpa_recomp_fwd: batch dimension ", i, " of ", name, " (",
                t.size(i), ") does not broadcast to ", bshape[bd]);
    out[3 - nb + bd] = t.size(i) == 1 ? 0 : t.stride(i);
  }
}

Tensor sdpa_unit_rows(const Tensor& t) { return (t.dim() >= 1 && t.stride(-1) != 1 && t.size(-1) > 1) ? t.contiguous() : t; }

// seq_padding_type of the ops: "left" or "right" (the wrapper lower-cases it, Fp8FusedSDPA.py:112); it only
// matters when valid_seq_len is given (flags SEQ_PADDING_LEFT / RIGHT, sdpa_gen.cpp:850-851).
bool sdpa_padding_left(c10::string_view seq_padding_type, bool has_valid) {
  const bool left = seq_padding_type == "left" || seq_padding_type == "Left" || seq_padding_type == "LEFT";
  const bool right = seq_padding_type == "right" || seq_padding_type == "Right" || seq_padding_type == "RIGHT";
  TORCH_CHECK(!has_valid || left || right, "seq_padding_type must be \"left\" or \"right\", got \"", std::string(seq_padding_type), "\"");
  return !right;
}

// valid_seq_len: one count of valid (unpadded) keys per entry of the outermost batch dimension -> int32 on q's device
Tensor sdpa_valid_seq_len(const Tensor& t, const Tensor& q, const std::vector<int64_t>& bshape, const char* op) {
  const int64_t nbatch = bshape.empty() ? 1 : bshape[0];
  TORCH_CHECK(at::isIntegralType(t.scalar_type(), false), op, ": valid_seq_len must be an integer tensor, got ", t.scalar_type());
  TORCH_CHECK(t.numel() == nbatch, op, ": valid_seq_len must hold one value per batch entry (", nbatch, "), got ", t.sizes());
  if (q.is_meta()) return t;
  TORCH_CHECK(t.device() == q.device(), op, ": valid_seq_len must be on the same device as q");
  return t.reshape({nbatch}).to(at::kInt).contiguous();
}

// Elements of fp32 scores the bf16 / fp32 measurement pass of the attention ops holds at a time
// (MI355Q_SDPA_MEASURE_SCORE_ELEMENTS overrides the default of 2^28, for tests).
int64_t sdpa_measure_score_elements() {
  if (const char* e = std::getenv("MI355Q_SDPA_MEASURE_SCORE_ELEMENTS")) {
    const long long v = std::atoll(e);
    if (v > 0) return (int64_t)v;
  }
  return (int64_t)1 << 28;
}

// Keys a query may attend to, as a boolean tensor that broadcasts against the scores [batch..., L, S]
// (undefined: all of them): the triangular mask and the per-batch key window.
// Rows l0 .. l0 + L - 1 of the queries (l0 shifts the triangle).
Tensor sdpa_keep_mask(const Tensor& like, int64_t L, int64_t S, bool is_causal, const Tensor& valid, bool pad_left, int64_t batch_rank,
                      int64_t l0 = 0) {
  Tensor keep;
  auto bopts = like.options().dtype(at::kBool);
  if (is_causal) keep = at::ones({L, S}, bopts).tril(l0);
  if (valid.defined()) {
    Tensor j = at::arange(S, like.options().dtype(at::kInt)).reshape({1, S});
    Tensor n = valid.reshape({-1, 1});
    Tensor w = pad_left ? j.ge(S - n) : j.lt(n);   // [B, S]
    std::vector<int64_t> shp(batch_rank + 2, 1);
    shp[0] = batch_rank > 0 ? w.size(0) : 1;
    shp.back() = S;
    if (batch_rank == 0) w = w.reshape({1, S});
    else w = w.reshape(shp);
    keep = keep.defined() ? keep.logical_and(w) : w;
  }
  return keep;
}

// softmax(q k^T scale + masks) in fp32 on the device's own matmul and softmax: the route of the bf16 / fp32
// measurement pass, where nothing is fp8.  A row with every key masked gives zeros.
// q holds query rows l0 .. of the problem (a slice when the caller walks the queries in pieces); a mask with a row per
// query is sliced the same way.
Tensor sdpa_probabilities_unfused(const Tensor& q, const Tensor& k, const c10::optional<Tensor>& attention_mask, double scale,
                                  bool is_causal, const Tensor& valid, bool pad_left, int64_t batch_rank, int64_t l0 = 0) {
  const float ninf = -std::numeric_limits<float>::infinity();
  Tensor s = at::matmul(q, k.transpose(-2, -1)).to(at::kFloat) * scale;
  if (attention_mask.has_value() && attention_mask->defined()) {
    Tensor am = *attention_mask;
    if (am.dim() >= 2 && am.size(-2) != 1 && am.size(-2) != q.size(-2)) am = am.narrow(-2, l0, q.size(-2));
    if (am.scalar_type() == at::kBool) s = s.masked_fill(am.logical_not(), ninf);
    else s = s + am.to(at::kFloat);
  }
  Tensor keep = sdpa_keep_mask(q, q.size(-2), k.size(-2), is_causal, valid, pad_left, batch_rank, l0);
  if (keep.defined()) s = s.masked_fill(keep.logical_not(), ninf);
  return at::nan_to_num(at::softmax(s, -1), 0.0);
}

// Fp8SDPARecompFwd::AddNode, hpu_ops/backend/sdpa_gen.cpp:806-1000 (inputs, flags, output types);
// output shapes SDPARecompFwdOutputShapeCommon / Fp8SDPARecompFwdOutputShape, :597-706.
SdpaOut fp8_sdpa_recomp_fwd_common(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& attention_mask,
                                   double p, double scale, bool is_causal, bool requires_backward, c10::string_view softmax_mode,
                                   const SdpaScale& d_scale_q, const SdpaScale& d_scale_k, const SdpaScale& d_scale_v,
                                   const SdpaScale& q_scale_s, const SdpaScale& q_scale_o, const SdpaScale& d_scale_s,
                                   bool is_amax_s, bool is_amax_o, const c10::optional<Tensor>& valid_seq_len,
                                   c10::string_view seq_padding_type) {
  TORCH_CHECK(!requires_backward, "fp8_sdpa_recomp_fwd: only the inference forward (requires_backward=False) is implemented");
  TORCH_CHECK(p == 0.0, "fp8_sdpa_recomp_fwd: dropout is not implemented (p must be 0)");
  TORCH_CHECK(softmax_mode == "none" || softmax_mode == "None" || softmax_mode == "fast", "fp8_sdpa_recomp_fwd: softmax_mode must be \"none\" or \"fast\"");
  const int64_t rank = q.dim();
  TORCH_CHECK(rank >= 2 && rank <= 5 && k.dim() == rank && v.dim() == rank,
              "fp8_sdpa_recomp_fwd: q, k and v must have the same rank, between 2 and 5");
  const bool has_mask = attention_mask.has_value() && attention_mask->defined();
  TORCH_CHECK(!(has_mask && is_causal), "fp8_sdpa_recomp_fwd: attention_mask and is_causal exclude each other");
  const bool has_valid = valid_seq_len.has_value() && valid_seq_len->defined();
  const bool pad_left = sdpa_padding_left(seq_padding_type, has_valid);
  // the wrapper's contract (Fp8FusedSDPA.py:123-126): only in inference with the triangular mask
  TORCH_CHECK(!has_valid || (is_causal && !has_mask),
              "fp8_sdpa_recomp_fwd: valid_seq_len is supported only in inference with is_causal and no attention_mask");
  const int64_t L = q.size(-2), S = k.size(-2), Dk = q.size(-1), Dv = v.size(-1);
  TORCH_CHECK(k.size(-1) == Dk, "fp8_sdpa_recomp_fwd: q and k must have the same head dimension");
  TORCH_CHECK(v.size(-2) == S, "fp8_sdpa_recomp_fwd: k and v must have the same sequence length");
  const at::ScalarType dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt, "fp8_sdpa_recomp_fwd: q, k and v must have the same dtype");
  // batch dims broadcast like matmul's (SDPARecompFwdOutputShapeCommon)
  std::vector<int64_t> qb(q.sizes().begin(), q.sizes().end() - 2), kb(k.sizes().begin(), k.sizes().end() - 2),
      vb(v.sizes().begin(), v.sizes().end() - 2);
  std::vector<int64_t> bshape = at::infer_size(at::infer_size(qb, kb), vb);
  std::vector<int64_t> out_shape = bshape;
  out_shape.push_back(L);
  out_shape.push_back(Dv);
  const bool fp8_in = is_fp8(dt);
  const at::ScalarType out_dt = fp8_in ? (q_scale_o.given() ? at::kFloat8_e4m3fn : at::kBFloat16) : dt;
  const at::ScalarType stat_dt = fp8_in ? at::kBFloat16 : dt;
  auto opts = q.options();
  Tensor out = at::empty(out_shape, opts.dtype(out_dt));
  // Float; BFloat16 for fp8 q and for bf16 q with softmax_mode "fast" (eager_custom_op_register.cpp:1795-1803)
  const at::ScalarType linv_dt = fp8_in || (softmax_mode == "fast" && dt == at::kBFloat16) ? at::kBFloat16 : at::kFloat;
  Tensor valid = has_valid ? sdpa_valid_seq_len(*valid_seq_len, q, bshape, "fp8_sdpa_recomp_fwd") : Tensor();
  if (q.is_meta())
    return SdpaOut(out, at::empty({1}, opts.dtype(stat_dt)), at::empty({1}, opts.dtype(linv_dt)), at::empty({1}, opts.dtype(at::kInt)),
                   at::empty({1}, opts.dtype(at::kFloat)), at::empty({1}, opts.dtype(at::kFloat)));
  // The five one-element outputs share one allocation.  In inference m, linv and seed are dummies that the
  // reference's kernel does not write either (sdpa_gen.cpp:949-965), and so are amax_s / amax_o when not asked
  // for: they are not filled here (a fill is a launch of its own in front of every call); the amax words that
  // are asked for are cleared by the C entry point.
  Tensor pool = at::empty({40}, opts.dtype(at::kByte));
  auto one = [&](int slot, at::ScalarType t) { return pool.slice(0, 8 * slot, 8 * slot + (int64_t)c10::elementSize(t)).view(t); };
  Tensor m = one(0, stat_dt), linv = one(1, linv_dt), seed = one(2, at::kInt), amax_s = one(3, at::kFloat), amax_o = one(4, at::kFloat);
  DeviceGuard guard(q.device());
  TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "fp8_sdpa_recomp_fwd: q, k and v must be on one device");
  MI355Q_OP_INFO("fp8_sdpa_recomp_fwd : q=" << q.sizes() << " k=" << k.sizes() << " v=" << v.sizes() << " " << dt << " -> " << out_dt
                                             << (is_causal ? " causal" : "") << (has_mask ? " mask" : ""));

  if (!fp8_in) {
    // The measurement pass of the reference's flow: bf16 / fp32 q, k, v, no fp8 anywhere; only amax_s
    // (and amax_o) are wanted from it.  It runs on the device's own matmul and softmax.
    TORCH_CHECK(dt == at::kBFloat16 || dt == at::kFloat, "fp8_sdpa_recomp_fwd: q, k and v must be fp8, bfloat16 or float");
    // The scores are a tensor [batch..., L, S] in fp32: the queries are walked in pieces that keep it below a fixed
    // number of elements (1 GiB of fp32 by default), so that a long prompt does not ask for tens of gigabytes.
    int64_t nbatch = 1;
    for (int64_t b : bshape) nbatch *= b;
    const int64_t per_row = std::max<int64_t>(nbatch * S, 1);
    const int64_t rows_at_once = std::max<int64_t>(sdpa_measure_score_elements() / per_row, 1);
    amax_s.zero_();
    for (int64_t l0 = 0; l0 < L; l0 += rows_at_once) {
      const int64_t len = std::min(rows_at_once, L - l0);
      Tensor pr = sdpa_probabilities_unfused(q.narrow(-2, l0, len), k, attention_mask, scale, is_causal, valid, pad_left,
                                             (int64_t)bshape.size(), l0);
      out.narrow(-2, l0, len).copy_(at::matmul(pr.to(dt), v));
      if (pr.numel() > 0) amax_s.copy_(at::maximum(amax_s, pr.max().reshape({1})));
    }
    if (out.numel() > 0) amax_o.copy_(out.to(at::kFloat).abs().max().reshape({1}));
    else amax_o.zero_();
    return SdpaOut(out, m, linv, seed, amax_s, amax_o);
  }

  if (out.numel() == 0) {
    pool.zero_();  // an empty problem has maxima of zero
    return SdpaOut(out, m, linv, seed, amax_s, amax_o);
  }
  TORCH_CHECK(Dk <= 256 && Dv <= 256, "fp8_sdpa_recomp_fwd: head dimensions up to 256 are supported, got ", Dk, " and ", Dv);
  Tensor qc = sdpa_unit_rows(q), kc = sdpa_unit_rows(k), vc = sdpa_unit_rows(v);
  mi355q_sdpa_desc d{};
  const int64_t nb = (int64_t)bshape.size();
  for (int64_t i = 0; i < 3; ++i) d.batch[i] = 1;
  for (int64_t i = 0; i < nb; ++i) d.batch[3 - nb + i] = bshape[i];
  sdpa_batch_strides(qc, bshape, d.q_bstride, "q");
  sdpa_batch_strides(kc, bshape, d.k_bstride, "k");
  sdpa_batch_strides(vc, bshape, d.v_bstride, "v");
  sdpa_batch_strides(out, bshape, d.out_bstride, "out");
  d.q_len = L; d.kv_len = S; d.head_dim_qk = Dk; d.head_dim_v = Dv;
  d.ldq = qc.stride(-2); d.ldk = kc.stride(-2); d.ldv = vc.stride(-2); d.ldo = out.stride(-2);
  if (has_valid) {
    d.valid_seq_len = valid.data_ptr<int32_t>();
    d.valid_seq_dim = nb == 0 ? 2 : (int32_t)(3 - nb);   // the outermost batch dimension
    d.seq_padding_left = pad_left ? 1 : 0;
  }
  Tensor mk;
  int mask_kind = MI355Q_SDPA_MASK_NONE;
  if (has_mask) {
    mk = *attention_mask;
    TORCH_CHECK(mk.device() == q.device(), "fp8_sdpa_recomp_fwd: attention_mask must be on the same device as q");
    TORCH_CHECK(mk.dim() >= 2 && mk.dim() <= rank, "fp8_sdpa_recomp_fwd: attention_mask must have between 2 and ", rank, " dimensions");
    TORCH_CHECK((mk.size(-1) == S || mk.size(-1) == 1) && (mk.size(-2) == L || mk.size(-2) == 1),
                "fp8_sdpa_recomp_fwd: attention_mask ", mk.sizes(), " does not broadcast to [..., ", L, ", ", S, "]");
    if (mk.scalar_type() == at::kBool) mask_kind = MI355Q_SDPA_MASK_BOOL;
    else if (mk.scalar_type() == at::kBFloat16) mask_kind = MI355Q_SDPA_MASK_BF16;
    else {
      mk = mk.to(at::kFloat);
      mask_kind = MI355Q_SDPA_MASK_F32;
    }
    if (mk.size(-1) != S) {
      std::vector<int64_t> full(mk.sizes().begin(), mk.sizes().end());
      full.back() = S;
      mk = mk.expand(full).contiguous();
    } else if (mk.stride(-1) != 1 && S > 1) {
      mk = mk.contiguous();
    }
    sdpa_batch_strides(mk, bshape, d.mask_bstride, "attention_mask");
    d.ldmask = mk.size(-2) == 1 ? 0 : mk.stride(-2);
  }
  const SdpaScale* sc[6] = {&d_scale_q, &d_scale_k, &d_scale_v, &q_scale_s, &q_scale_o, &d_scale_s};
  const float* sc_dev[6];
  float sc_host[6];
  for (int i = 0; i < 6; ++i) {
    sc_dev[i] = sc[i]->dev;
    sc_host[i] = sc[i]->host;
  }
  // few queries against many keys: the partial results of the key splits pass through a workspace
  const size_t ws_bytes = mi355q_fp8_sdpa_workspace_bytes(&d);
  // (their arrival counters start from zero and are left zero: the buffer kept per stream, or, while the stream
  // is being captured into a graph, a zero-filled one of the graph's own)
  Tensor ws;
  if (ws_bytes > 0) {
    ws = ticket_workspace(qc, ws_bytes, kWsSdpa);
    if (!ws.defined()) ws = at::zeros({(int64_t)ws_bytes}, opts.dtype(at::kByte));
  }
  const int st = mi355q_fp8_sdpa_fwd(qc.data_ptr(), kc.data_ptr(), vc.data_ptr(), to_mi355q_dtype(dt), has_mask ? mk.data_ptr() : nullptr,
                                     mask_kind, out.data_ptr(), to_mi355q_dtype(out_dt), &d, (float)scale, is_causal ? 1 : 0, sc_dev,
                                     sc_host, is_amax_s ? amax_s.data_ptr<float>() : nullptr,
                                     is_amax_o ? amax_o.data_ptr<float>() : nullptr, ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes,
                                     current_stream(q));
  if (st != MI355Q_OK && ws_bytes > 0) drop_ticket_workspace(qc, kWsSdpa);
  check_status(st, "mi355q_fp8_sdpa_fwd");
  return SdpaOut(out, m, linv, seed, amax_s, amax_o);
}

SdpaOut fp8_sdpa_recomp_fwd(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& attention_mask, double p,
                            double scale, bool is_causal, bool requires_backward, c10::string_view softmax_mode,
                            const c10::optional<Tensor>& d_scale_q, const c10::optional<Tensor>& d_scale_k,
                            const c10::optional<Tensor>& d_scale_v, const c10::optional<Tensor>& q_scale_s,
                            const c10::optional<Tensor>& q_scale_o, const c10::optional<Tensor>& d_scale_s, bool is_amax_s,
                            bool is_amax_o, const c10::optional<Tensor>& valid_seq_len, c10::string_view seq_padding_type) {
  return fp8_sdpa_recomp_fwd_common(q, k, v, attention_mask, p, scale, is_causal, requires_backward, softmax_mode,
                                    sdpa_scale(d_scale_q, q, "d_scale_q"), sdpa_scale(d_scale_k, q, "d_scale_k"),
                                    sdpa_scale(d_scale_v, q, "d_scale_v"), sdpa_scale(q_scale_s, q, "q_scale_s"),
                                    sdpa_scale(q_scale_o, q, "q_scale_o"), sdpa_scale(d_scale_s, q, "d_scale_s"), is_amax_s,
                                    is_amax_o, valid_seq_len, seq_padding_type);
}

SdpaOut fp8_sdpa_recomp_fwd_scalar(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& attention_mask,
                                   double p, double scale, bool is_causal, bool requires_backward, c10::string_view softmax_mode,
                                   double d_scale_q, double d_scale_k, double d_scale_v, double q_scale_s, double q_scale_o,
                                   double d_scale_s, bool is_amax_s, bool is_amax_o, const c10::optional<Tensor>& valid_seq_len,
                                   c10::string_view seq_padding_type) {
  return fp8_sdpa_recomp_fwd_common(q, k, v, attention_mask, p, scale, is_causal, requires_backward, softmax_mode,
                                    sdpa_scale(d_scale_q), sdpa_scale(d_scale_k), sdpa_scale(d_scale_v), sdpa_scale(q_scale_s),
                                    sdpa_scale(q_scale_o), sdpa_scale(d_scale_s), is_amax_s, is_amax_o, valid_seq_len,
                                    seq_padding_type);
}

// --------------------------------------------------------------- fp8_sdpa_fwd
//
// The forward without recomputation (Fp8SDPAFwd::AddNode, hpu_ops/backend/sdpa_gen.cpp:340-437; output shapes
// SDPAFwdOutputShapeCommon :103-150 and Fp8SDPAFwdOutputShape :267-272; eager wrapper
// habana_eager/eager_custom_op_register.cpp:1544-1660), which the reference's module calls whenever
// recomputation is switched off, inference included (Fp8FusedSDPA.py:163-182).  It returns the attention
// output, the probability matrix P [batch..., L, S] in q's dtype (what a backward pass would read instead of
// recomputing it), the dropout mask (a one-element Char placeholder without dropout) and amax_s.  Materialising
// P is the point of the op, so it runs unfused on this library's own kernels: the scores are one batched fp8 GEMM
// (q k^T, d_scale_q and d_scale_k in its epilogue), softmax_fp8 scales them, adds the mask and writes
// P = fp8(softmax q_scale_s), and out = (P v) d_scale_s d_scale_v is a second fp8 GEMM.  Here the
// probabilities are normalised before they are rounded to fp8 (in the recompute op they are rounded per block
// of keys against the running maximum); the reference's kernel is closed on this point.  A row whose keys are
// all masked holds equal scores and attends to all keys evenly (the recompute op gives zeros there).
using SdpaFwdOut = std::tuple<Tensor, Tensor, Tensor, Tensor>;

SdpaFwdOut fp8_sdpa_fwd(const Tensor& q, const Tensor& k, const Tensor& v, const c10::optional<Tensor>& attention_mask, double p,
                        double scale, bool is_causal, c10::string_view softmax_mode, const c10::optional<Tensor>& d_scale_q,
                        const c10::optional<Tensor>& d_scale_k, const c10::optional<Tensor>& d_scale_v,
                        const c10::optional<Tensor>& q_scale_s, const c10::optional<Tensor>& q_scale_o,
                        const c10::optional<Tensor>& d_scale_s, bool is_amax_s, const c10::optional<Tensor>& valid_seq_len,
                        c10::string_view seq_padding_type) {
  TORCH_CHECK(p == 0.0, "fp8_sdpa_fwd: dropout is not implemented (p must be 0)");
  TORCH_CHECK(softmax_mode == "none" || softmax_mode == "None" || softmax_mode == "fast", "fp8_sdpa_fwd: softmax_mode must be \"none\" or \"fast\"");
  const int64_t rank = q.dim();
  TORCH_CHECK(rank >= 2 && rank <= 5 && k.dim() == rank && v.dim() == rank, "fp8_sdpa_fwd: q, k and v must have the same rank, between 2 and 5");
  const bool has_mask = attention_mask.has_value() && attention_mask->defined();
  TORCH_CHECK(!(has_mask && is_causal), "fp8_sdpa_fwd: attention_mask and is_causal exclude each other");
  const bool has_valid = valid_seq_len.has_value() && valid_seq_len->defined();
  const bool pad_left = sdpa_padding_left(seq_padding_type, has_valid);
  TORCH_CHECK(!has_valid || (is_causal && !has_mask), "fp8_sdpa_fwd: valid_seq_len is supported only with is_causal and no attention_mask");
  const int64_t L = q.size(-2), S = k.size(-2), Dk = q.size(-1), Dv = v.size(-1);
  TORCH_CHECK(k.size(-1) == Dk, "fp8_sdpa_fwd: q and k must have the same head dimension");
  TORCH_CHECK(v.size(-2) == S, "fp8_sdpa_fwd: k and v must have the same sequence length");
  const at::ScalarType dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt, "fp8_sdpa_fwd: q, k and v must have the same dtype");
  std::vector<int64_t> qb(q.sizes().begin(), q.sizes().end() - 2), kb(k.sizes().begin(), k.sizes().end() - 2),
      vb(v.sizes().begin(), v.sizes().end() - 2);
  std::vector<int64_t> pshape = at::infer_size(qb, kb);          // batch dims of q k^T
  std::vector<int64_t> oshape = at::infer_size(pshape, vb);
  const int64_t nb = (int64_t)oshape.size();
  pshape.push_back(L);
  pshape.push_back(S);
  oshape.push_back(L);
  oshape.push_back(Dv);
  const bool fp8_in = is_fp8(dt);
  const bool has_qo = q_scale_o.has_value() && q_scale_o->defined() && q_scale_o->numel() > 0;
  // out: q's dtype, or bf16 for fp8 q without q_scale_o (sdpa_gen.cpp:412-424); P: q's dtype; amax_s: Float
  const at::ScalarType out_dt = fp8_in ? (has_qo ? dt : at::kBFloat16) : dt;
  auto opts = q.options();
  if (q.is_meta())
    return SdpaFwdOut(at::empty(oshape, opts.dtype(out_dt)), at::empty(pshape, opts.dtype(dt)), at::empty({1}, opts.dtype(at::kChar)),
                      at::empty({1}, opts.dtype(at::kFloat)));
  DeviceGuard guard(q.device());
  TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "fp8_sdpa_fwd: q, k and v must be on one device");
  Tensor dm = at::zeros({1}, opts.dtype(at::kChar));
  Tensor amax_s = at::zeros({1}, opts.dtype(at::kFloat));
  std::vector<int64_t> bshape(oshape.begin(), oshape.end() - 2);
  Tensor valid = has_valid ? sdpa_valid_seq_len(*valid_seq_len, q, bshape, "fp8_sdpa_fwd") : Tensor();
  MI355Q_OP_INFO("fp8_sdpa_fwd : q=" << q.sizes() << " k=" << k.sizes() << " v=" << v.sizes() << " " << dt << " -> " << out_dt
                                      << (is_causal ? " causal" : "") << (has_mask ? " mask" : ""));
  if (!fp8_in) {
    // bf16 / fp32 q, k, v (the measurement pass): nothing is fp8, the device's own matmul and softmax
    TORCH_CHECK(dt == at::kBFloat16 || dt == at::kFloat, "fp8_sdpa_fwd: q, k and v must be fp8, bfloat16 or float");
    Tensor pr = sdpa_probabilities_unfused(q, k, attention_mask, scale, is_causal, valid, pad_left, nb);
    Tensor P = pr.to(dt);
    Tensor out = at::matmul(P, v);
    if (is_amax_s && pr.numel() > 0) amax_s.copy_(pr.max().reshape({1}));
    return SdpaFwdOut(out, P, dm, amax_s);
  }
  if (L == 0 || S == 0 || c10::multiply_integers(oshape) == 0 || Dk == 0) {
    return SdpaFwdOut(at::zeros(oshape, opts.dtype(out_dt)), at::zeros(pshape, opts.dtype(dt)), dm, amax_s);
  }
  // scores = (q d_scale_q)(k d_scale_k)^T, bf16
  Tensor scores = fp8_gemm_v2_impl(q, false, k, true, c10::nullopt, at::kBFloat16, opt_tensor_iv(d_scale_q), opt_tensor_iv(d_scale_k),
                                   c10::nullopt, false, c10::nullopt);
  // the masks as one additive bf16 tensor of the rank of the scores (first and last extent as theirs, 1 or
  // theirs in between: the form softmax_fp8 takes).  Masked entries get the most negative finite value.
  Tensor add;
  {
    const float kMasked = -3.0e38f;
    Tensor m;
    if (has_mask) {
      TORCH_CHECK(attention_mask->device() == q.device(), "fp8_sdpa_fwd: attention_mask must be on the same device as q");
      if (attention_mask->scalar_type() == at::kBool)
        m = at::zeros({1}, opts.dtype(at::kBFloat16)).masked_fill(attention_mask->logical_not(), kMasked);
      else m = attention_mask->to(at::kBFloat16).clamp_min(kMasked);
    } else {
      Tensor keep = sdpa_keep_mask(q, L, S, is_causal, valid, pad_left, nb);
      if (keep.defined()) m = at::zeros({1}, opts.dtype(at::kBFloat16)).masked_fill(keep.logical_not(), kMasked);
    }
    if (m.defined()) {
      TORCH_CHECK(m.dim() <= scores.dim(), "fp8_sdpa_fwd: attention_mask has more dimensions than the scores");
      while (m.dim() < scores.dim()) m = m.unsqueeze(0);
      std::vector<int64_t> shp(m.sizes().begin(), m.sizes().end());
      for (int64_t i = 0; i < (int64_t)shp.size(); ++i)
        TORCH_CHECK(shp[i] == 1 || shp[i] == scores.size(i), "fp8_sdpa_fwd: attention_mask ", attention_mask.has_value() ? attention_mask->sizes() : m.sizes(),
                    " does not broadcast to the scores ", scores.sizes());
      shp.front() = scores.size(0);
      shp.back() = S;
      add = m.expand(shp).contiguous();
    }
  }
  // P = fp8(softmax(scores scale + mask) q_scale_s); an e5m2 q takes bf16 probabilities and the cast kernel
  const bool has_qs = q_scale_s.has_value() && q_scale_s->defined() && q_scale_s->numel() > 0;
  SoftmaxScale in_s = softmax_scale(scale);
  SoftmaxScale out_s = softmax_scale(1.0);
  Tensor qs_holder;
  if (has_qs) {
    TORCH_CHECK(q_scale_s->numel() == 1, "fp8_sdpa_fwd: q_scale_s must have one element, got ", q_scale_s->sizes());
    qs_holder = q_scale_s->to(q.device(), at::kFloat).reshape({1});
    out_s.dev = qs_holder.data_ptr<float>();
  }
  Tensor P;
  if (dt == at::kFloat8_e4m3fn && !is_amax_s) {
    P = softmax_fp8_common(scores, -1, in_s, out_s, SoftmaxScale(), add.defined() ? c10::optional<Tensor>(add) : c10::nullopt);
  } else {
    // bf16 probabilities first (their maximum is amax_s), then the scaled cast to q's format
    Tensor x = scores.to(at::kFloat) * scale;
    if (add.defined()) x = x + add.to(at::kFloat);
    Tensor pb = softmax_fp8_common(x.to(at::kBFloat16), -1, SoftmaxScale(), SoftmaxScale(), SoftmaxScale(), c10::nullopt);
    if (is_amax_s) {
      check_status(mi355q_amax(pb.data_ptr(), MI355Q_BF16, pb.numel(), amax_s.data_ptr<float>(), current_stream(pb)), "mi355q_amax");
    }
    P = at::empty(pb.sizes(), opts.dtype(dt));
    CastScale cs = resolve_cast_scale(has_qs ? IValue(qs_holder) : IValue(), c10::nullopt, pb);
    check_status(launch_cast_to(pb, P, cs, nullptr, false), "mi355q_cast_to_fp8");
  }
  // out = (P d_scale_s)(v d_scale_v); d_scale_s defaults to 1 / q_scale_s
  const bool has_ds = d_scale_s.has_value() && d_scale_s->defined() && d_scale_s->numel() > 0;
  IValue ds_iv = has_ds ? IValue(*d_scale_s) : (has_qs ? IValue(qs_holder.reciprocal()) : IValue());
  Tensor out = fp8_gemm_v2_impl(P, false, v, false, c10::nullopt, at::kBFloat16, ds_iv, opt_tensor_iv(d_scale_v), c10::nullopt, false,
                                c10::nullopt);
  if (out_dt != at::kBFloat16) {
    Tensor o8 = at::empty(out.sizes(), opts.dtype(out_dt));
    CastScale cs = resolve_cast_scale(IValue(q_scale_o->to(q.device(), at::kFloat)), c10::nullopt, out);
    check_status(launch_cast_to(out, o8, cs, nullptr, false), "mi355q_cast_to_fp8");
    out = o8;
  }
  return SdpaFwdOut(out, P, dm, amax_s);
}

// ------------------------------------------------------------- amax helpers

Tensor amax_op(const Tensor& x) {
  TORCH_CHECK(x.scalar_type() == at::kFloat || x.scalar_type() == at::kBFloat16,
              "mi355q::amax input must be float or bfloat16");
  if (x.is_meta()) return at::empty({}, x.options().dtype(at::kFloat));
  DeviceGuard guard(x.device());
  Tensor c = x.contiguous();
  Tensor out = at::empty({}, c.options().dtype(at::kFloat));
  check_status(mi355q_amax(c.data_ptr(), to_mi355q_dtype(c.scalar_type()), c.numel(),
                           out.data_ptr<float>(), current_stream(c)),
               "mi355q_amax");
  return out;
}

Tensor rowwise_amax_op(const Tensor& x) {
  TORCH_CHECK(x.scalar_type() == at::kFloat || x.scalar_type() == at::kBFloat16,
              "mi355q::rowwise_amax input must be float or bfloat16");
  TORCH_CHECK(x.dim() >= 1, "mi355q::rowwise_amax input must have at least 1 dimension");
  std::vector<int64_t> shp(x.sizes().begin(), x.sizes().end() - 1);
  if (x.is_meta()) return at::empty(shp, x.options().dtype(at::kFloat));
  DeviceGuard guard(x.device());
  Tensor c = x.contiguous();
  Tensor out = at::empty(shp, c.options().dtype(at::kFloat));
  const int64_t cols = c.size(-1);
  const int64_t rows = out.numel();
  check_status(mi355q_rowwise_amax(c.data_ptr(), to_mi355q_dtype(c.scalar_type()), rows, cols,
                                   out.data_ptr<float>(), current_stream(c)),
               "mi355q_rowwise_amax");
  return out;
}

// Dynamic per-row quantisation: (x8, scale_inv) with scale = fp8_max / rowwise amax.
// One kernel when the row fits a workgroup's registers, else the three steps it fuses.
std::tuple<Tensor, Tensor> quantize_rows_op(const Tensor& x, at::ScalarType dtype) {
  TORCH_CHECK(x.scalar_type() == at::kFloat || x.scalar_type() == at::kBFloat16,
              "mi355q::quantize_rows input must be float or bfloat16");
  TORCH_CHECK(dtype == at::kFloat8_e4m3fn || dtype == at::kFloat8_e5m2,
              "mi355q::quantize_rows dtype must be float8_e4m3fn or float8_e5m2");
  TORCH_CHECK(x.dim() >= 1, "mi355q::quantize_rows input must have at least 1 dimension");
  std::vector<int64_t> shp(x.sizes().begin(), x.sizes().end());
  shp.back() = 1;
  if (x.is_meta()) return {at::empty(x.sizes(), x.options().dtype(dtype)), at::empty(shp, x.options().dtype(at::kFloat))};
  DeviceGuard guard(x.device());
  Tensor c = x.contiguous();
  Tensor out = at::empty(c.sizes(), c.options().dtype(dtype));
  Tensor scale_inv = at::empty(shp, c.options().dtype(at::kFloat));
  const int64_t cols = c.size(-1);
  const int64_t rows = cols ? c.numel() / cols : 0;
  const float target = dtype == at::kFloat8_e5m2 ? 57344.0f : 448.0f;
  const int st = mi355q_quantize_rows(c.data_ptr(), to_mi355q_dtype(c.scalar_type()), rows, cols, out.data_ptr(),
                                      to_mi355q_dtype(dtype), target, nullptr, scale_inv.data_ptr<float>(),
                                      current_stream(c));
  if (st == MI355Q_ERR_UNSUPPORTED) {
    Tensor amax = rowwise_amax_op(c).reshape(shp);
    // capped like the kernel's row_scale (largest finite bf16): a zero row gets zero codes, not NaN
    Tensor scale = at::clamp_max(at::div(at::full_like(amax, target), amax), 3.3895313892515355e38);
    check_status(mi355q_cast_to_fp8(c.data_ptr(), to_mi355q_dtype(c.scalar_type()), out.data_ptr(),
                                    to_mi355q_dtype(dtype), scale.data_ptr<float>(), 0.0f, MI355Q_SCALE_MID,
                                    1, rows, cols, nullptr, current_stream(c)),
                 "mi355q_cast_to_fp8");
    return {out, at::reciprocal(scale)};
  }
  check_status(st, "mi355q_quantize_rows");
  return {out, scale_inv};
}

// SiLU(gate) * up in bf16 and the dynamic per-row quantisation of the product in
// one kernel: (h8, scale_inv), bit-identical to quantize_rows of
// bf16(bf16(silu(gate)) * up) with the oracle's silu.  gate and up are 2-D bf16
// with unit column stride (they may be the two halves of one GEMM output).
// Shapes the kernel does not take go through aten's silu and mul, whose exp may
// differ from the oracle's in the last place.
std::tuple<Tensor, Tensor> silu_mul_quantize_rows_op(const Tensor& gate, const Tensor& up, at::ScalarType dtype) {
  TORCH_CHECK(gate.scalar_type() == at::kBFloat16 && up.scalar_type() == at::kBFloat16,
              "mi355q::silu_mul_quantize_rows inputs must be bfloat16");
  TORCH_CHECK(dtype == at::kFloat8_e4m3fn || dtype == at::kFloat8_e5m2,
              "mi355q::silu_mul_quantize_rows dtype must be float8_e4m3fn or float8_e5m2");
  TORCH_CHECK(gate.dim() == 2 && gate.sizes() == up.sizes(),
              "mi355q::silu_mul_quantize_rows takes two matrices of the same shape, got ", gate.sizes(), " and ", up.sizes());
  const int64_t rows = gate.size(0), cols = gate.size(1);
  if (gate.is_meta())
    return {at::empty({rows, cols}, gate.options().dtype(dtype)), at::empty({rows, 1}, gate.options().dtype(at::kFloat))};
  TORCH_CHECK(gate.device() == up.device(), "mi355q::silu_mul_quantize_rows inputs must be on the same device");
  DeviceGuard guard(gate.device());
  Tensor g = gate.stride(1) == 1 || cols <= 1 ? gate : gate.contiguous();
  Tensor u = up.stride(1) == 1 || cols <= 1 ? up : up.contiguous();
  Tensor out = at::empty({rows, cols}, g.options().dtype(dtype));
  Tensor scale_inv = at::empty({rows, 1}, g.options().dtype(at::kFloat));
  if (out.numel() == 0) return {out, scale_inv};
  const float target = dtype == at::kFloat8_e5m2 ? 57344.0f : 448.0f;
  const int st = mi355q_silu_mul_quantize_rows(g.data_ptr(), rows > 1 ? g.stride(0) : cols, u.data_ptr(),
                                               rows > 1 ? u.stride(0) : cols, rows, cols, out.data_ptr(),
                                               to_mi355q_dtype(dtype), target, nullptr, nullptr,
                                               scale_inv.data_ptr<float>(), current_stream(g));
  if (st == MI355Q_ERR_UNSUPPORTED) return quantize_rows_op(at::mul(at::silu(gate), up), dtype);
  check_status(st, "mi355q_silu_mul_quantize_rows");
  return {out, scale_inv};
}

// ------------------------------------------------------------- _scaled_mm
//
// aten::_scaled_mm on the fp8 GEMM kernel: the reference lowers it to the same
// fp8_gemm node as hpu::fp8_gemm_v2, with scale_result as a further input
// (ScaledMm::AddNode, hpu_ops/backend/scaled_mm_gen.cpp:66-141; checks and their
// messages :78-107; the default out_dtype is mat1's, :72-75).
//   out = to_out_dtype( (mat1 @ mat2) * scale_a * scale_b * scale_result + bias )
// (the form the reference's test checks against: any_mode/test_hpu_scaled_mm.py:
// 177).  scale_a / scale_b hold one value, or one per row of mat1 ([M, 1]) / per
// column of mat2 ([1, N]).  An fp8 out_dtype is produced by the saturating
// round-to-nearest cast of the fp32 result (one rounding).  Registered as
// mi355q::scaled_mm with aten::_scaled_mm's signature; the package can also put
// it behind torch._scaled_mm for HIP tensors (use_for_aten_scaled_mm()).
// use_fast_accum is accepted and has no effect: accumulation is fp32 throughout.
Tensor scaled_mm(const Tensor& mat1, const Tensor& mat2, const Tensor& scale_a, const Tensor& scale_b,
                 const c10::optional<Tensor>& bias, const c10::optional<Tensor>& scale_result,
                 c10::optional<at::ScalarType> out_dtype, bool /*use_fast_accum*/) {
  TORCH_CHECK(mat1.dim() == 2, "mat1 must be a matrix");
  TORCH_CHECK(mat2.dim() == 2, "mat2 must be a matrix");
  TORCH_CHECK(mat1.size(1) == mat2.size(0), "mat1 and mat2 shapes cannot be multiplied (", mat1.size(0), "x",
              mat1.size(1), " and ", mat2.size(0), "x", mat2.size(1), ")");
  const int64_t M = mat1.size(0), N = mat2.size(1);
  const bool has_bias = bias.has_value() && bias->defined();
  TORCH_CHECK(!has_bias || bias->numel() == N, "Bias must be size ", N, " but got ", has_bias ? bias->numel() : 0);
  TORCH_CHECK(is_fp8(mat1.scalar_type()), "Expected mat1 to be Float8_e5m2 or Float8_e4m3fn matrix got ",
              mat1.scalar_type());
  TORCH_CHECK(is_fp8(mat2.scalar_type()), "Expected mat2 to be Float8_e5m2 or Float8_e4m3fn matrix got ",
              mat2.scalar_type());
  const at::ScalarType out_t = out_dtype.value_or(mat1.scalar_type());
  TORCH_CHECK(out_t == at::kFloat || out_t == at::kBFloat16 || is_fp8(out_t),
              "_scaled_mm out_dtype must be float, bfloat16, float8_e5m2 or float8_e4m3fn, got ", out_t);
  auto scale_ok = [&](const Tensor& s, int64_t rows, int64_t cols) {
    return s.numel() == 1 || (s.dim() == 2 && s.size(0) == rows && s.size(1) == cols);
  };
  TORCH_CHECK(scale_ok(scale_a, M, 1), "scale_a must hold one value or have shape [", M, ", 1], got ", scale_a.sizes());
  TORCH_CHECK(scale_ok(scale_b, 1, N), "scale_b must hold one value or have shape [1, ", N, "], got ", scale_b.sizes());
  const bool has_sr = scale_result.has_value() && scale_result->defined();
  TORCH_CHECK(!has_sr || scale_result->numel() == 1, "scale_result must hold one value");
  if (mat1.is_meta()) return at::empty({M, N}, mat1.options().dtype(out_t));

  // a transposed view of a contiguous matrix is multiplied in place (no copy)
  Tensor a = mat1, b = mat2;
  bool ta = false, tb = false;
  if (!a.is_contiguous() && a.t().is_contiguous()) {
    a = a.t();
    ta = true;
  }
  if (!b.is_contiguous() && b.t().is_contiguous()) {
    b = b.t();
    tb = true;
  }
  Tensor sa = scale_a.to(at::kFloat);
  if (has_sr) sa = sa * scale_result->to(at::kFloat).reshape({});
  const at::ScalarType gemm_t = is_fp8(out_t) ? at::kFloat : out_t;
  OptShape sb_shape;
  if (scale_b.numel() > 1) sb_shape = std::vector<int64_t>{1, N};
  Tensor r = fp8_gemm_v2_impl(a, ta, b, tb, c10::nullopt, gemm_t, IValue(sa), IValue(scale_b),
                              has_bias ? c10::optional<Tensor>(bias->reshape({N})) : c10::nullopt, false, sb_shape);
  if (!is_fp8(out_t)) return r;
  Tensor out = at::empty({M, N}, r.options().dtype(out_t));
  if (out.numel() == 0) return out;
  DeviceGuard guard(r.device());
  check_status(launch_cast_to(r, out, resolve_cast_scale(IValue(), c10::nullopt, r), nullptr, false), "mi355q_cast_to_fp8");
  return out;
}

}  // namespace

TORCH_LIBRARY(hpu, m) {
  m.def("hpu::cast_from_fp8(Tensor input, Tensor? scale, ScalarType out_dtype, int[]? scale_shape=None) -> Tensor");
  m.def("hpu::cast_from_fp8.scalar(Tensor input, float scale, ScalarType out_dtype, int[]? scale_shape=None) -> Tensor");
  m.def("hpu::cast_from_fp8.scalar_list(Tensor input, float[] scale, ScalarType out_dtype, int[]? scale_shape=None) -> Tensor");
  m.def("hpu::cast_to_fp8(Tensor input, Tensor? scale, bool stochastic_rounding, Tensor(a!) out, Tensor(b!) amax) -> (Tensor(a!), Tensor(b!))");
  m.def("hpu::fp8_gemm(Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor D, ScalarType out_dtype, Tensor? A_scale_inv, Tensor? B_scale_inv, Tensor? bias, bool accumulate, Tensor(a!) out) -> Tensor(a!)");
  m.def("hpu::cast_to_fp8_hybrid(Tensor input, Tensor? scale_152=None, Tensor? scale_143=None, bool stochastic_rounding=False, bool is_amax=False) -> (Tensor, Tensor, Tensor)");
  m.def("hpu::cast_to_fp8_v2(Tensor input, Tensor? scale=None, bool stochastic_rounding=False, bool is_amax=False, ScalarType dtype=None, int[]? scale_shape=None) -> (Tensor, Tensor)");
  m.def("hpu::cast_to_fp8_v2.scalar(Tensor input, float scale, bool stochastic_rounding=False, bool is_amax=False, ScalarType dtype=None, int[]? scale_shape=None) -> (Tensor, Tensor)");
  m.def("hpu::cast_to_fp8_v2.scalar_list(Tensor input, float[] scale, bool stochastic_rounding=False, bool is_amax=False, ScalarType dtype=None, int[]? scale_shape=None) -> (Tensor, Tensor)");
  m.def("hpu::convert_from_int4(Tensor input, Tensor scale, Tensor? zero_point, ScalarType out_dtype) -> Tensor");
  m.def("hpu::convert_from_uint4(Tensor input, Tensor scale, Tensor? zero_point, ScalarType out_dtype) -> Tensor");
  m.def("hpu::fp8_gemm_v2(Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor? D, ScalarType out_dtype, Tensor? A_scale_inv=None, Tensor? B_scale_inv=None, Tensor? bias=None, bool accumulate=False, int[]? B_scale_shape=None) -> Tensor");
  m.def("hpu::fp8_gemm_v2.scalar(Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor? D, ScalarType out_dtype, float A_scale_inv, float B_scale_inv, Tensor? bias=None, bool accumulate=False, int[]? B_scale_shape=None) -> Tensor");
  m.def("hpu::fp8_gemm_v2.scalar_list(Tensor A, bool trans_A, Tensor B, bool trans_B, Tensor? D, ScalarType out_dtype, float[] A_scale_inv, float[] B_scale_inv, Tensor? bias=None, bool accumulate=False, int[]? B_scale_shape=None) -> Tensor");
  m.def("hpu::softmax_fp8(Tensor input, int dim, Tensor? input_scale=None, Tensor? output_scale=None, Tensor? inv_attn_heads=None, Tensor? fused_add=None) -> Tensor");
  m.def("hpu::softmax_fp8.Scalar_scales(Tensor input, int dim, float input_scale, float output_scale, Tensor? inv_attn_heads=None, Tensor? fused_add=None) -> Tensor");
  m.def("hpu::softmax_fp8.Scalar(Tensor input, int dim, float input_scale, float output_scale, float inv_attn_heads, Tensor? fused_add=None) -> Tensor");
  m.def("hpu::sum_fp8(Tensor self, int[1]? dim=None, bool keepdim=False, ScalarType? out_dtype=None) -> Tensor");
  m.def("hpu::fp8_sdpa_recomp_fwd(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, bool is_amax_0, Tensor? valid_seq_len, str seq_padding_type ) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
  m.def("hpu::fp8_sdpa_recomp_fwd_non_dropout(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, bool is_amax_0, Tensor? valid_seq_len, str seq_padding_type ) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
  m.def("hpu::fp8_sdpa_recomp_fwd_non_dropout.scalar(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, float d_scale_q, float d_scale_k, float d_scale_v, float q_scale_s, float q_scale_o, float d_scale_s, bool is_amax_s, bool is_amax_0,  Tensor? valid_seq_len, str seq_padding_type ) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
  m.def("hpu::fp8_sdpa_fwd(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def("hpu::fp8_sdpa_fwd_non_dropout(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, str softmax_mode, Tensor? d_scale_q, Tensor? d_scale_k, Tensor? d_scale_v, Tensor? q_scale_s, Tensor? q_scale_o, Tensor? d_scale_s, bool is_amax_s, Tensor? valid_seq_len, str seq_padding_type) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def("hpu::fp8_sdpa_recomp_fwd.scalar(Tensor q, Tensor k, Tensor v, Tensor? attention_mask, float p, float scale, bool is_causal, bool requires_backward, str softmax_mode, float d_scale_q, float d_scale_k, float d_scale_v, float q_scale_s, float q_scale_o, float d_scale_s, bool is_amax_s, bool is_amax_0, Tensor? valid_seq_len, str seq_padding_type ) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
}

// Helpers the reference has no op for: amax alone and per-row amax.
TORCH_LIBRARY(mi355q, m) {
  m.def("mi355q::amax(Tensor input) -> Tensor");
  m.def("mi355q::rowwise_amax(Tensor input) -> Tensor");
  m.def("mi355q::quantize_rows(Tensor input, ScalarType dtype) -> (Tensor, Tensor)");
  m.def("mi355q::silu_mul_quantize_rows(Tensor gate, Tensor up, ScalarType dtype) -> (Tensor, Tensor)");
  m.def("mi355q::w4a8_gemm(Tensor A, Tensor packed, Tensor scale, Tensor? zero_point, bool is_signed, ScalarType out_dtype, Tensor? A_scale_inv=None, Tensor? bias=None) -> Tensor");
  m.def("mi355q::w4a16_gemm(Tensor A, Tensor packed, Tensor scale, Tensor? zero_point, bool is_signed, ScalarType out_dtype, Tensor? bias=None) -> Tensor");
  m.def("mi355q::scaled_mm(Tensor self, Tensor mat2, Tensor scale_a, Tensor scale_b, Tensor? bias=None, Tensor? scale_result=None, ScalarType? out_dtype=None, bool use_fast_accum=False) -> Tensor");
}

#define MI355Q_REGISTER_HPU(m)                                                                 \
  m.impl("cast_to_fp8_v2", torch::CppFunction::makeFromBoxedFunction<&cast_to_fp8_v2_boxed>()); \
  m.impl("cast_to_fp8_v2.scalar", torch::CppFunction::makeFromBoxedFunction<&cast_to_fp8_v2_boxed>()); \
  m.impl("cast_to_fp8_v2.scalar_list", torch::CppFunction::makeFromBoxedFunction<&cast_to_fp8_v2_boxed>()); \
  m.impl("cast_from_fp8", cast_from_fp8);                                                      \
  m.impl("cast_from_fp8.scalar", cast_from_fp8_scalar);                                        \
  m.impl("cast_from_fp8.scalar_list", cast_from_fp8_scalar_list);                              \
  m.impl("fp8_gemm_v2", fp8_gemm_v2);                                                          \
  m.impl("fp8_gemm_v2.scalar", fp8_gemm_v2_scalar);                                            \
  m.impl("fp8_gemm_v2.scalar_list", fp8_gemm_v2_scalar_list);                                  \
  m.impl("convert_from_int4", convert_from_int4);                                              \
  m.impl("convert_from_uint4", convert_from_uint4);                                            \
  m.impl("cast_to_fp8", cast_to_fp8_v1);                                                       \
  m.impl("cast_to_fp8_hybrid", cast_to_fp8_hybrid);                                            \
  m.impl("fp8_gemm", fp8_gemm_v1);                                                             \
  m.impl("softmax_fp8", softmax_fp8);                                                          \
  m.impl("softmax_fp8.Scalar_scales", softmax_fp8_scalar_scales);                              \
  m.impl("softmax_fp8.Scalar", softmax_fp8_scalar);                                            \
  m.impl("sum_fp8", sum_fp8);                                                                  \
  m.impl("fp8_sdpa_recomp_fwd", fp8_sdpa_recomp_fwd);                                          \
  m.impl("fp8_sdpa_recomp_fwd.scalar", fp8_sdpa_recomp_fwd_scalar);                            \
  m.impl("fp8_sdpa_recomp_fwd_non_dropout", fp8_sdpa_recomp_fwd);                              \
  m.impl("fp8_sdpa_recomp_fwd_non_dropout.scalar", fp8_sdpa_recomp_fwd_scalar);                \
  m.impl("fp8_sdpa_fwd", fp8_sdpa_fwd);                                                        \
  m.impl("fp8_sdpa_fwd_non_dropout", fp8_sdpa_fwd);

TORCH_LIBRARY_IMPL(hpu, CUDA, m) { MI355Q_REGISTER_HPU(m) }
TORCH_LIBRARY_IMPL(hpu, Meta, m) { MI355Q_REGISTER_HPU(m) }

TORCH_LIBRARY_IMPL(mi355q, CUDA, m) {
  m.impl("amax", amax_op);
  m.impl("rowwise_amax", rowwise_amax_op);
  m.impl("quantize_rows", quantize_rows_op);
  m.impl("scaled_mm", scaled_mm);
  m.impl("silu_mul_quantize_rows", silu_mul_quantize_rows_op);
  m.impl("w4a8_gemm", w4a8_gemm);
  m.impl("w4a16_gemm", w4a16_gemm);
}
TORCH_LIBRARY_IMPL(mi355q, Meta, m) {
  m.impl("amax", amax_op);
  m.impl("rowwise_amax", rowwise_amax_op);
  m.impl("quantize_rows", quantize_rows_op);
  m.impl("scaled_mm", scaled_mm);
  m.impl("silu_mul_quantize_rows", silu_mul_quantize_rows_op);
  m.impl("w4a8_gemm", w4a8_gemm);
  m.impl("w4a16_gemm", w4a16_gemm);
}
