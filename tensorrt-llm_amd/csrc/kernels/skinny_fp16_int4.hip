// Instantiates the skinny-M GEMM kernel for FP16 activations and int4 weights.
#include "skinny_kernel.h"

namespace woq
{
int launch_skinny_FP16_4(MatmulProblem const& p, GemmPlan const& plan, void* stream)
{
    return launch_skinny_typed<WOQ_FP16, 4>(p, plan, stream);
}
} // namespace woq
