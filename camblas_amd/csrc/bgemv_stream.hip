// The launchers of the BF16 weight-streaming linear (kernel and description: bgemv_stream_kernel.hpp), and
// its instantiations with one K block per step.
#include "bgemv_stream_kernel.hpp"

namespace camblas_hip
{
hipError_t stream_plain_single(hipStream_t stream, int row_tiles, int token_tiles, const StreamParams &p, int shares)
{
    return launch_tokens<1>(stream, row_tiles, token_tiles, p, shares);
}

namespace
{
// the fused halves of a launch, checked and copied into the kernel's parameters
hipError_t apply_fusion(StreamParams &p, const StreamFusion &fusion, int token_tiles)
{
    p.norm_weight = static_cast<const unsigned short *>(fusion.norm_weight);
    p.ssq_in = fusion.ssq_in;
    p.ssq_count = fusion.ssq_count;
    p.ssq_ld = fusion.ssq_ld;
    p.epsilon = fusion.epsilon;
    p.residual = static_cast<const unsigned short *>(fusion.residual);
    p.ld_residual = fusion.ld_residual;
    p.ssq_out = fusion.ssq_out;
    p.ssq_ld_out = fusion.ssq_ld_out;
    if (p.norm_weight && (!p.ssq_in || p.ssq_count < 1 || p.ssq_ld < p.m || p.k % 8 ||
                          reinterpret_cast<uintptr_t>(p.norm_weight) % 16))
        return hipErrorInvalidValue;
    if (p.residual && (!p.ssq_out || p.ssq_ld_out < p.m || p.ld_residual < p.n || p.beta != 0.f))
        return hipErrorInvalidValue;
    (void)token_tiles;
    return hipSuccess;
}
} // namespace

size_t stream_partial_bytes(int row_tiles, int token_tiles, int n_out, int m_rows, int shares)
{
    const size_t groups = size_t((n_out + row_tiles * 16 - 1) / (row_tiles * 16)) *
                          size_t((m_rows + token_tiles * 16 - 1) / (token_tiles * 16));
    return size_t(shares) * groups * size_t(row_tiles) * size_t(token_tiles) * 1024;
}

// Gated form: out[m, n] = round(round(silu(g)) * u) with g = round(x Wg^T), u = round(x Wu^T); a
// workgroup owns 16 * pair_tiles output rows (that many gate rows and the same up rows) over the
// whole K. pair_tiles 1..4, token_tiles 1 to 4 (three: without the fused normalisation only).
hipError_t launch_gated_stream(hipStream_t stream, int pair_tiles, int token_tiles, int n_out, int m_rows,
                               int k, const void *gate, const void *up, int lda, const void *x, int ldb,
                               void *y, int ldc, const StreamFusion &fusion)
{
    StreamParams p;
    p.w = static_cast<const unsigned short *>(gate);
    p.w2 = static_cast<const unsigned short *>(up);
    p.x = static_cast<const unsigned short *>(x);
    p.y = static_cast<unsigned short *>(y);
    p.lda = lda;
    p.ldb = ldb;
    p.ldc = ldc;
    p.z = p.y;
    p.ldz = ldc;
    p.n = n_out;
    p.m = m_rows;
    p.k = k;
    p.alpha = 1.f;
    p.beta = 0.f;
    p.vector_store = (ldc % 4 == 0) && (reinterpret_cast<uintptr_t>(y) % 8 == 0);
    p.partials = nullptr;
    p.arrivals = nullptr;
    if ((m_rows + token_tiles * 16 - 1) / (token_tiles * 16) > 65535)
        return hipErrorInvalidValue;
    // (a workgroup addresses its token rows with 31-bit byte offsets inside one descriptor)
    if ((size_t(token_tiles * 16 - 1) * size_t(ldb) + size_t(k)) * 2 >= (size_t(1) << 31) || ldb < 1 || k < 1)
        return hipErrorInvalidValue;
    const bool fused = fusion.norm_weight != nullptr;
    if (fusion.residual)
        return hipErrorInvalidValue; // the gated form has no residual epilogue
    const hipError_t admitted = apply_fusion(p, fusion, token_tiles);
    if (admitted != hipSuccess)
        return admitted;
    return stream_gated(stream, pair_tiles, token_tiles, fused, p);
}

hipError_t launch_bgemv_stream(hipStream_t stream, int depth_log2, int row_tiles, int token_tiles, int n_out,
                               int m_rows, int k, float alpha, const void *w, int lda,
                               const void *x, int ldb, float beta, void *y, int ldc,
                               const BetaSource &source, const StreamShares &shares, const StreamFusion &fusion)
{
    StreamParams p;
    p.w = static_cast<const unsigned short *>(w);
    p.w2 = nullptr;
    p.x = static_cast<const unsigned short *>(x);
    p.y = static_cast<unsigned short *>(y);
    p.lda = lda;
    p.ldb = ldb;
    p.ldc = ldc;
    p.z = source.z ? static_cast<const unsigned short *>(source.z) : p.y;
    p.ldz = source.z ? source.ldz : ldc;
    p.n = n_out;
    p.m = m_rows;
    p.k = k;
    p.alpha = alpha;
    p.beta = beta;
    p.vector_store = ldc % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 8 == 0 && p.ldz % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(p.z) % 8 == 0;
    p.partials = shares.partials;
    p.arrivals = shares.arrivals;
    if ((m_rows + token_tiles * 16 - 1) / (token_tiles * 16) > 65535 || shares.count < 1 || shares.count > 64)
        return hipErrorInvalidValue;
    // (a workgroup addresses its token rows with 31-bit byte offsets inside one descriptor)
    if ((size_t(token_tiles * 16 - 1) * size_t(ldb) + size_t(k)) * 2 >= (size_t(1) << 31) || ldb < 1 || k < 1)
        return hipErrorInvalidValue;
    const hipError_t admitted = apply_fusion(p, fusion, token_tiles);
    if (admitted != hipSuccess)
        return admitted;
    if (fusion.norm_weight && fusion.residual)
        return hipErrorInvalidValue; // one half per launch: no linear of a decoder layer needs both
    if (token_tiles > 4)
        return fusion.norm_weight || fusion.residual || depth_log2 != 0
                   ? hipErrorInvalidValue
                   : stream_many_tokens(stream, row_tiles, token_tiles, p, shares.count);
    if (fusion.norm_weight) // (the fused forms exist for K steps of one or two blocks)
        return stream_normalising(stream, depth_log2, row_tiles, token_tiles, p, shares.count);
    if (fusion.residual)
        return stream_residual(stream, depth_log2, row_tiles, token_tiles, p, shares.count);
    return depth_log2 == 0 ? stream_plain_single(stream, row_tiles, token_tiles, p, shares.count)
                           : stream_plain_deep(stream, depth_log2, row_tiles, token_tiles, p, shares.count);
}
} // namespace camblas_hip
