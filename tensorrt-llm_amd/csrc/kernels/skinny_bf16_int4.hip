// Instantiates the skinny-M GEMM kernel for BF16 activations and int4 weights.
#include "skinny_kernel.h"

namespace woq
{
int launch_skinny_BF16_4(MatmulProblem const& p, GemmPlan const& plan, void* stream)
{
    return launch_skinny_typed<WOQ_BF16, 4>(p, plan, stream);
}
} // namespace woq
