// Instantiates the weight-streaming kernel for FP16 activations and int8 weights.
#include "stream_kernel.h"
#include "stream_wide_kernel.h"

namespace woq
{
int launch_stream_FP16_8(MatmulProblem const& p, void* stream)
{
    return launch_stream_typed<WOQ_FP16, 8>(p, stream);
}
} // namespace woq
