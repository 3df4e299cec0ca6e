// Instantiates the weight-streaming kernel for BF16 activations and int8 weights.
#include "stream_kernel.h"
#include "stream_wide_kernel.h"

namespace woq
{
int launch_stream_BF16_8(MatmulProblem const& p, void* stream)
{
    return launch_stream_typed<WOQ_BF16, 8>(p, stream);
}
} // namespace woq
