// BF16 y[M,N] = alpha * x[M,K] * W[K,N] + beta * y for up to a few hundred tokens, with W stored the
// other way round from a linear layer's weight: K rows of N contiguous outputs (torch.mm(x, W) with
// a row-major W; 'N','N' in the column-major terms of camblas_cuda_bgemm).
//
// The matrix instruction wants, per lane, eight consecutive K values of one output column, which in
// this layout lie a whole row of W apart. A workgroup of four wavefronts owns 128 outputs for up to
// 256 tokens and streams W once: each step copies 64 rows x 128 outputs (256-byte pieces of rows:
// whole cache lines) straight into LDS, and a lane gathers its eight K values of one output with two
// transposing LDS reads (ds_read_b64_tr_b16: within sixteen lanes, lane 4a + b receives element b of
// the four 8-byte values at the addresses of lanes a, 4 + a, 8 + a, 12 + a; so lane s points at row
// s / 4 of four consecutive rows, outputs 4 (s % 4) .. + 3, and receives four K values of output s). A
// 1 KB direct-to-LDS load (a piece) brings rows j, j + 16, j + 32 and j + 48 of the step, 256 contiguous
// bytes of each, and successive pieces are placed 1056 bytes apart: four consecutive rows lie in four
// pieces, 32 bytes of bank offset apart, so the sixteen lanes of a transposing read touch sixteen
// different 8-byte bank pairs. The
// tokens go through LDS as in the linear-layer kernels (128-byte rows, 16-byte chunks XOR-swizzled).
// At decode sizes the kernel is bound by the W stream. (Eight 2-byte reads per fragment, which these
// two replace, were a third of a step's LDS time: [8192, 8192] x 16 tokens 31.7 us.)
// K can be divided over gridDim.y workgroups per tile (few outputs): FP32 planes, summed in share
// order by the same kernel that serves the linear-layer tiles.
// Needs K % 64 == 0, N % 4 == 0, lda % 8 == 0, ldb % 8 == 0, ldc % 4 == 0, 16-byte aligned W and x, an
// 8-byte aligned y.
// Contract: ref src/cuda/bfloat16.cuh:11-57 ('N','N' call of src/cuda/torch_bindings.cpp:155-199).
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
namespace
{
struct NnParams {
    const unsigned short *w; // element (k, n) at w[k * lda + n]
    const unsigned short *x; // element (m, k) at x[m * ldb + k]
    unsigned short *y;       // element (m, n) at y[m * ldc + n]
    int lda, ldb, ldc;
    int n, m, k;
    float alpha, beta;
    float *partials; // [share][token][output] when K is divided
    int share_steps;
};

typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef short i16x8_t __attribute__((ext_vector_type(8)));
// ds_read_b64_tr_b16 at a byte address inside a __shared__ array
__device__ __forceinline__ i16x4_t read_transposed(const unsigned char *address)
{
    // (a pointer-to-pointer cast: through an integer the compiler would lose which LDS object is read and make
    // the read wait for every direct-to-LDS load in flight)
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t *)(address));
}

constexpr int NN_BN = 128, NN_BK = 64, NN_STAGES = 3;
constexpr int NN_PIECE = 66;                      // 16-byte slots from one 4-row piece of W to the next (1 KB + 32 B)
constexpr int NN_W_SLOTS = (NN_BK / 4) * NN_PIECE; // per stage

// TM: token tiles of 32 per workgroup (one pass over W serves 32 * TM tokens)
template <int TM> __global__ __launch_bounds__(256) void bgemm_nn_kernel(NnParams p)
{
    constexpr int WAVES = 4, BM = 32 * TM, X_SLOTS = BM * 8;
    constexpr int W_LOADS = NN_BK / 4 / WAVES, X_LOADS = BM / 8 / WAVES, LOADS = W_LOADS + X_LOADS;
    static_assert(BM % (8 * WAVES) == 0, "every wavefront issues whole token loads");
    // one LDS object per stage, so that reads of one stage and fills of another are provably disjoint
    __shared__ u32x4_t stage0[NN_W_SLOTS + X_SLOTS];
    __shared__ u32x4_t stage1[NN_W_SLOTS + X_SLOTS];
    __shared__ u32x4_t stage2[NN_W_SLOTS + X_SLOTS];

    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int n0 = int(blockIdx.x) * NN_BN, m0 = int(blockIdx.z) * BM;
    const int steps_all = p.k / NN_BK;
    const int first_step = int(blockIdx.y) * p.share_steps;
    const int steps = steps_all - first_step < p.share_steps ? steps_all - first_step : p.share_steps;

    // ---- fills. W piece j of a stage (rows j, j + 16, j + 32, j + 48 of the step) is loaded by wavefront
    // j % 4: lane l brings the 16 bytes at row j + 16 * (l / 16), outputs 8 * (l % 16) .. + 7. Rows past K and outputs
    // past the end of the last row lie outside the buffer resource and read as zero; outputs past N
    // inside a row are whatever lies there and only reach accumulators that are never stored.
    const __amdgpu_buffer_rsrc_t w_resource =
        make_resource(p.w + n0, (unsigned(p.k - 1) * unsigned(p.lda) + unsigned(p.n - n0)) * 2u);
    const unsigned w_lane_off = (unsigned(wave + 16 * (lane / 16)) * unsigned(p.lda) + unsigned(lane % 16) * 8u) * 2u;
    const unsigned w_piece_step = unsigned(WAVES) * unsigned(p.lda) * 2u; // successive pieces of a wavefront
    const unsigned w_k_step = unsigned(NN_BK) * unsigned(p.lda) * 2u;
    // token rows: eight 128-byte rows per load, lane l row l / 8, the chunk that belongs in its slot
    const int x_rows = p.m - m0 < BM ? p.m - m0 : BM;
    const __amdgpu_buffer_rsrc_t x_resource =
        make_resource(p.x + size_t(m0) * p.ldb, (unsigned(x_rows - 1) * unsigned(p.ldb) + unsigned(p.k)) * 2u);
    const int x_load_row = wave * 8 + lane / 8;
    const unsigned x_lane_off =
        (unsigned(x_load_row) * unsigned(p.ldb) + unsigned(((lane % 8) ^ lds_swizzle<8>(x_load_row)) * 8)) * 2u;
    const unsigned x_piece_step = unsigned(WAVES * 8) * unsigned(p.ldb) * 2u;
    const int last_step = first_step + steps - 1;
    int load_step = first_step;
    auto issue = [&](u32x4_t *stage) {
#pragma unroll
        for (int it = 0; it < W_LOADS; ++it)
            load_to_lds(w_resource, w_lane_off, unsigned(load_step) * w_k_step + unsigned(it) * w_piece_step,
                        stage + (it * WAVES + wave) * NN_PIECE);
#pragma unroll
        for (int it = 0; it < X_LOADS; ++it)
            load_to_lds(x_resource, x_lane_off, unsigned(load_step) * (NN_BK * 2u) + unsigned(it) * x_piece_step,
                        stage + NN_W_SLOTS + (it * WAVES + wave) * 64);
        // (steps past the end re-read the last one into a stage nobody multiplies, which keeps the
        // number of loads in flight fixed)
        load_step = load_step < last_step ? load_step + 1 : last_step;
    };

    // ---- operand reads. Output column of this lane: 32 * wave + lane % 32; lane half h = lane / 32
    // holds K values 8h .. 8h+7 of every 16-deep sub-step.
    const int column = lane % 32, half = lane / 32;
    // the transposing reads: for the sub-step's rows 8 h .. 8 h + 3 this lane points at row 8 h + (lane % 16) / 4
    // (piece of that number; 256 bytes further per 16-deep sub-step) and at four outputs from `pointed` on;
    // the value it receives is of output `column`. Rows 8 h + 4 .. lie four pieces on.
    const int pointed = wave * 32 + (lane / 16 % 2) * 16 + 4 * (lane % 4);
    const int w_lane_bytes = (half * 8 + (lane % 16) / 4) * NN_PIECE * 16 + pointed * 2;
    const int x_swizzle = lds_swizzle<8>(column);
    f32x16_t acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[j][r] = 0.f;

    auto multiply = [&](const u32x4_t *stage) {
        const unsigned char *bytes = reinterpret_cast<const unsigned char *>(stage) + w_lane_bytes;
#pragma unroll
        for (int ks = 0; ks < NN_BK / 16; ++ks) {
            const i16x4_t lower = read_transposed(bytes + ks * 256);
            const i16x4_t upper = read_transposed(bytes + ks * 256 + 4 * NN_PIECE * 16);
            const bf16x8_t w_frag = __builtin_bit_cast(bf16x8_t, i16x8_t{lower[0], lower[1], lower[2], lower[3],
                                                                        upper[0], upper[1], upper[2], upper[3]});
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const bf16x8_t x_frag = __builtin_bit_cast(
                    bf16x8_t, stage[NN_W_SLOTS + (j * 32 + column) * 8 + ((ks * 2 + half) ^ x_swizzle)]);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w_frag, x_frag, acc[j], 0, 0, 0);
            }
        }
    };
    // One step: the stage read now is complete (all but the newest LOADS loads have landed) and
    // every wavefront has finished the stage that is filled next.
    auto step = [&](const u32x4_t *current, u32x4_t *fill) {
        pipeline_barrier<LOADS *(NN_STAGES - 2)>();
        issue(fill);
        multiply(current);
    };

    issue(stage0);
    issue(stage1);
    for (int done = 0; done < steps; done += NN_STAGES) {
        step(stage0, stage2);
        if (done + 1 < steps)
            step(stage1, stage0);
        if (done + 2 < steps)
            step(stage2, stage1);
    }
    wait_loads<0>(); // drain the padding loads before the LDS is released

    // ---- epilogue: accumulator register 4q+e of lane l is output 8q + 4*(l/32) + e of the
    // wavefront's 32 columns, token l % 32 of the tile
    const int first_output = n0 + wave * 32 + half * 4;
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = m0 + j * 32 + column;
        if (m >= p.m)
            continue;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int n = first_output + q * 8;
            if (n >= p.n)
                continue;
            if (gridDim.y > 1) { // a share of K: the plain sums
                *reinterpret_cast<f32x4_t *>(p.partials + (size_t(blockIdx.y) * p.m + m) * p.n + n) =
                    f32x4_t{acc[j][q * 4], acc[j][q * 4 + 1], acc[j][q * 4 + 2], acc[j][q * 4 + 3]};
                continue;
            }
            unsigned short *out = p.y + size_t(m) * p.ldc + n;
            float v0 = p.alpha * acc[j][q * 4], v1 = p.alpha * acc[j][q * 4 + 1];
            float v2 = p.alpha * acc[j][q * 4 + 2], v3 = p.alpha * acc[j][q * 4 + 3];
            if (p.beta != 0.f) {
                const u32x2_t old = *reinterpret_cast<const u32x2_t *>(out);
                v0 = fmaf(p.beta, __uint_as_float(old[0] << 16), v0);
                v1 = fmaf(p.beta, __uint_as_float(old[0] & 0xffff0000u), v1);
                v2 = fmaf(p.beta, __uint_as_float(old[1] << 16), v2);
                v3 = fmaf(p.beta, __uint_as_float(old[1] & 0xffff0000u), v3);
            }
            *reinterpret_cast<u32x2_t *>(out) = u32x2_t{pack_bf16x2(v0, v1), pack_bf16x2(v2, v3)};
        }
    }
}

template <int TM> hipError_t launch_nn(hipStream_t stream, NnParams p, int shares)
{
    const int steps = p.k / NN_BK;
    p.share_steps = (steps + shares - 1) / shares;
    shares = (steps + p.share_steps - 1) / p.share_steps; // no empty share
    const dim3 grid(unsigned((p.n + NN_BN - 1) / NN_BN), unsigned(shares), unsigned((p.m + 32 * TM - 1) / (32 * TM)));
    bgemm_nn_kernel<TM><<<grid, 256, 0, stream>>>(p);
    const hipError_t status = launch_status();
    if (shares == 1 || status != hipSuccess)
        return status;
    return launch_sum_shares(stream, p.partials, shares, p.n, p.m, p.alpha, p.beta, p.y, p.ldc, p.y, p.ldc);
}
} // namespace

// tokens per pass over W: 32, 64, 128 or 256 (the smallest that holds m_rows, else 256 and several
// passes). shares > 1: K divided over that many workgroups per tile, `partials` holding
// shares * m_rows * n_out floats.
hipError_t launch_bgemm_nn(hipStream_t stream, int n_out, int m_rows, int k, float alpha, const void *w, int lda,
                           const void *x, int ldb, float beta, void *y, int ldc, int shares, float *partials)
{
    if (k % NN_BK || k < NN_BK || n_out % 4 || lda % 8 || ldb % 8 || ldc % 4 || reinterpret_cast<uintptr_t>(y) % 8 ||
        reinterpret_cast<uintptr_t>(w) % 16 || reinterpret_cast<uintptr_t>(x) % 16)
        return hipErrorInvalidValue;
    if (shares < 1 || shares > 64 || (shares > 1 && !partials))
        return hipErrorInvalidValue;
    // byte offsets inside the buffer resources are 32-bit
    if (size_t(k) * size_t(lda) * 2 >= (size_t(1) << 32) || (size_t(256) * size_t(ldb) + size_t(k)) * 2 >= (size_t(1) << 32) ||
        (m_rows + 255) / 256 > 65535)
        return hipErrorInvalidValue;
    NnParams p;
    p.w = static_cast<const unsigned short *>(w);
    p.x = static_cast<const unsigned short *>(x);
    p.y = static_cast<unsigned short *>(y);
    p.lda = lda;
    p.ldb = ldb;
    p.ldc = ldc;
    p.n = n_out;
    p.m = m_rows;
    p.k = k;
    p.alpha = alpha;
    p.beta = beta;
    p.partials = partials;
    p.share_steps = 0;
    if (m_rows <= 32)
        return launch_nn<1>(stream, p, shares);
    if (m_rows <= 64)
        return launch_nn<2>(stream, p, shares);
    if (m_rows <= 128)
        return launch_nn<4>(stream, p, shares);
    return launch_nn<8>(stream, p, shares);
}
} // namespace camblas_hip
