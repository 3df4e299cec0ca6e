// Instantiates the prefill GEMM kernel for BF16 activations and int8 weights.
#include "gemm_kernel.h"

namespace woq
{
int launch_gemm_BF16_8(MatmulProblem const& p, GemmPlan const& plan, void* stream)
{
    return launch_gemm_typed<WOQ_BF16, 8>(p, plan, stream);
}
} // namespace woq
