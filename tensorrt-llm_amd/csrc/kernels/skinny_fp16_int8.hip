// Instantiates the skinny-M GEMM kernel for FP16 activations and int8 weights.
#include "skinny_kernel.h"

namespace woq
{
int launch_skinny_FP16_8(MatmulProblem const& p, GemmPlan const& plan, void* stream)
{
    return launch_skinny_typed<WOQ_FP16, 8>(p, plan, stream);
}
} // namespace woq
