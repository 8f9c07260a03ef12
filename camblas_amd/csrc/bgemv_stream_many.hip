// BF16 weight-streaming linear: the instantiations with five to eight token tiles (65 to 128 tokens),
// whose partial tiles go through LDS in two passes at the end of a workgroup.
#include "bgemv_stream_kernel.hpp"

namespace camblas_hip
{
hipError_t stream_many_tokens(hipStream_t stream, int row_tiles, int token_tiles, const StreamParams &p, int shares)
{
    switch (token_tiles) {
    case 5: return launch_rows<5, 1, 0>(stream, row_tiles, p, shares);
    case 6: return launch_rows<6, 1, 0>(stream, row_tiles, p, shares);
    case 7: return launch_rows<7, 1, 0>(stream, row_tiles, p, shares);
    case 8: return launch_rows<8, 1, 0>(stream, row_tiles, p, shares);
    default: return hipErrorInvalidValue;
    }
}
} // namespace camblas_hip
