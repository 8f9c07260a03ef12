// BF16 weight-streaming linear: the instantiations with the input normalised on its way to LDS (K steps of one or two blocks).
#include "bgemv_stream_kernel.hpp"

namespace camblas_hip
{
hipError_t stream_normalising(hipStream_t stream, int depth_log2, int row_tiles, int token_tiles, const StreamParams &p, int shares)
{
    switch (depth_log2) {
    case 0: return launch_tokens<1, 1>(stream, row_tiles, token_tiles, p, shares);
    case 1: return launch_tokens<2, 1>(stream, row_tiles, token_tiles, p, shares);
    default: return hipErrorInvalidValue;
    }
}
} // namespace camblas_hip
