// fp8 GEMM tile kernels for one operand layout: A K-major, B K-major.
#include "gemm_dispatch.h"

namespace mi355q {
void launch_gemm_kk(const GemmArgs& g, int fmt_a, int fmt_b, int64_t batch, hipStream_t st) {
  launch_by_format<true, true>(g, fmt_a, fmt_b, batch, st);
}
}  // namespace mi355q
