// BF16 weight-streaming linear: the instantiations with two to eight K blocks per step.
#include "bgemv_stream_kernel.hpp"

namespace camblas_hip
{
hipError_t stream_plain_deep(hipStream_t stream, int depth_log2, int row_tiles, int token_tiles, const StreamParams &p, int shares)
{
    switch (depth_log2) {
    case 1: return launch_tokens<2>(stream, row_tiles, token_tiles, p, shares);
    case 2: return launch_tokens<4>(stream, row_tiles, token_tiles, p, shares);
    case 3: return launch_tokens<8>(stream, row_tiles, token_tiles, p, shares);
    default: return hipErrorInvalidValue;
    }
}
} // namespace camblas_hip
