// BF16 weight-streaming linear: the instantiations of the gated form (gate and up rows in one workgroup,
// SiLU-multiply in the epilogue), plain and with the input normalised on its way to LDS.
#include "bgemv_stream_kernel.hpp"

namespace camblas_hip
{
hipError_t stream_gated(hipStream_t stream, int pair_tiles, int token_tiles, bool fused, const StreamParams &p)
{
#define CAMBLAS_GATED(NT, MT) \
    return fused ? launch_one<NT, MT, 1, true, 1>(stream, p) : launch_one<NT, MT, 1, true, 0>(stream, p)
    switch (token_tiles * 10 + pair_tiles) {
    case 11: CAMBLAS_GATED(2, 1);
    case 12: CAMBLAS_GATED(4, 1);
    case 13: CAMBLAS_GATED(6, 1);
    case 14: CAMBLAS_GATED(8, 1);
    case 21: CAMBLAS_GATED(2, 2);
    case 22: CAMBLAS_GATED(4, 2);
    case 23: CAMBLAS_GATED(6, 2);
    case 24: CAMBLAS_GATED(8, 2);
    // (33 to 48 tokens; the form with the normalisation keeps to one, two and four token tiles)
    case 31: return fused ? hipErrorInvalidValue : launch_one<2, 3, 1, true, 0>(stream, p);
    case 32: return fused ? hipErrorInvalidValue : launch_one<4, 3, 1, true, 0>(stream, p);
    case 33: return fused ? hipErrorInvalidValue : launch_one<6, 3, 1, true, 0>(stream, p);
    case 34: return fused ? hipErrorInvalidValue : launch_one<8, 3, 1, true, 0>(stream, p);
    case 41: CAMBLAS_GATED(2, 4);
    case 42: CAMBLAS_GATED(4, 4);
    case 43: CAMBLAS_GATED(6, 4);
    case 44: CAMBLAS_GATED(8, 4);
    default: return hipErrorInvalidValue;
    }
#undef CAMBLAS_GATED
}
} // namespace camblas_hip
