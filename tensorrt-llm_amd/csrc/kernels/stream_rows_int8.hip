// Instantiates the multi-row decode kernel (stream_rows_kernel.h) for int8 weights.
#include "stream_rows_kernel.h"

namespace woq
{
int launch_stream_rows_int8(StreamParams const& sp, int dtype, int group, bool zero, int waves, int ns, int tpw, void* stream)
{
    return launch_stream_rows_bits<8>(sp, dtype, group, zero, waves, ns, tpw, stream);
}
} // namespace woq
