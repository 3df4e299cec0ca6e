// Instantiates the weight-streaming kernel for BF16 activations and int4 weights.
#include "stream_kernel.h"
#include "stream_wide_kernel.h"

namespace woq
{
int launch_stream_BF16_4(MatmulProblem const& p, void* stream)
{
    return launch_stream_typed<WOQ_BF16, 4>(p, stream);
}
} // namespace woq
