// placeholder until the MFMA GEMM lands
#include "device_common.h"
namespace woq
{
int launch_gemm(MatmulProblem const& p, void* stream)
{
    (void) p; (void) stream;
    return fail(WOQ_ERR_UNSUPPORTED, "GEMM regime not built yet");
}
}
