// TNN instantiations of the matrix-core conv kernel (one translation unit per type so they
// compile in parallel).
#include "tab_conv_mfma_direct.h"

namespace tab {
hipError_t launch_conv_mfma_tnn(const ConvArgs &args, int shape, hipStream_t stream)
{
    return launch_mfma_type<0>(args, shape, stream);
}
}  // namespace tab
