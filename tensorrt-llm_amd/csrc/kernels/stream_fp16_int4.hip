// Instantiates the weight-streaming kernel for FP16 activations and int4 weights.
#include "stream_kernel.h"
#include "stream_wide_kernel.h"

namespace woq
{
int launch_stream_FP16_4(MatmulProblem const& p, void* stream)
{
    return launch_stream_typed<WOQ_FP16, 4>(p, stream);
}
} // namespace woq
