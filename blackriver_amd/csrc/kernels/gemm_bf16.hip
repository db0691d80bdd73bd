// bf16-multiplicand instantiations of the MFMA GEMM template.
#include "gemm_dtl16.hpp"

namespace brk {
int gemm16_launch_bf16(const gemm16::GemmArgs& g, const gemm16::Problem& p, long long batch, hipStream_t st) {
    return gemm16::launch_any<BR_GEMM_BF16>(g, p, batch, st);
}
}  // namespace brk
