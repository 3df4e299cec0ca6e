// Instantiates the prefill GEMM kernel for FP16 activations and int4 weights.
#include "gemm_kernel.h"

namespace woq
{
int launch_gemm_FP16_4(MatmulProblem const& p, GemmPlan const& plan, void* stream)
{
    return launch_gemm_typed<WOQ_FP16, 4>(p, plan, stream);
}
} // namespace woq
