// Grouped-query decode attention: one query token per sequence against a BF16 KV cache
// [batch, context, kv_heads, 128], split over the context so that a batch of 32 sequences fills
// 256 compute units, then an ordered combine. The reference has no counterpart (its
// src/cuda/fusion.cuh:95-157 is dense single-head FP32/FP64 with a materialised score matrix); the
// arithmetic is the textbook softmax(scale * q k^T) v with FP32 accumulation and an online-softmax
// merge of the context partitions.
//
// Partition kernel, one workgroup per (partition, kv head, sequence), 4 wavefronts:
//   1. scores: 16 lanes share one cache row (16-byte loads, 256 contiguous bytes per row), every
//      lane multiplies its 8 dims with all query heads of the group, 4 butterfly steps finish the
//      dot products; scores go to LDS.
//   2. per-head maximum and exponentials in LDS (one wavefront per head).
//   3. values: a lane owns two output dims, wavefronts stride over positions, the four wavefront
//      partial sums are added in index order.
// The kernel is bound by the cache read (2 * context * 256 bytes per kv head and sequence).
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int DIM = 128, CHUNK = 256, WAVES = 4;

template <int G>
__global__ __launch_bounds__(WAVES * 64) void gqa_partition_kernel(
    int q_heads, int kv_heads, int context_length, const int32_t *lengths, float scale,
    const unsigned short *q, int q_stride, const unsigned short *k_cache,
    const unsigned short *v_cache, float *part_o, float *part_m, float *part_l, int splits,
    int group)
{
    __shared__ __attribute__((aligned(16))) float score[G][CHUNK];
    __shared__ float reduce[WAVES][G][DIM];
    const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int length = lengths ? min(max(lengths[b], 0), context_length) : context_length;
    const int begin = split * CHUNK;
    const int count = min(CHUNK, length - begin); // may be <= 0: empty partition
    const size_t row_stride = size_t(kv_heads) * DIM;
    const unsigned short *k_base =
        k_cache + (size_t(b) * context_length + begin) * row_stride + size_t(kvh) * DIM;
    const unsigned short *v_base =
        v_cache + (size_t(b) * context_length + begin) * row_stride + size_t(kvh) * DIM;

    // ---- 1. scores
    const int part = lane % 16, sub = lane / 16;
    float qv[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        int head = kvh * group + (h < group ? h : group - 1);
        u32x4_t raw = *reinterpret_cast<const u32x4_t *>(q + size_t(b) * q_stride +
                                                         size_t(head) * DIM + part * 8);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            qv[h][2 * e] = __uint_as_float(raw[e] << 16) * scale;
            qv[h][2 * e + 1] = __uint_as_float(raw[e] & 0xffff0000u) * scale;
        }
    }
    for (int p0 = wave * 16; p0 < count; p0 += WAVES * 16) {
        u32x4_t rows[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int position = p0 + u * 4 + sub;
            position = position < count ? position : count - 1;
            rows[u] = *reinterpret_cast<const u32x4_t *>(k_base + size_t(position) * row_stride +
                                                         part * 8);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float kv[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                kv[2 * e] = __uint_as_float(rows[u][e] << 16);
                kv[2 * e + 1] = __uint_as_float(rows[u][e] & 0xffff0000u);
            }
            float dot[G];
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float sum = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    sum = fmaf(qv[h][e], kv[e], sum);
                dot[h] = sum;
            }
#pragma unroll
            for (int h = 0; h < G; ++h)
                dot[h] = row16_sum(dot[h]);
            int position = p0 + u * 4 + sub;
            if (position < count) {
#pragma unroll
                for (int h = 0; h < G; ++h)
                    if (part == h % 16)
                        score[h][position] = dot[h];
            }
        }
    }
    __syncthreads();

    // ---- 2. per-head maximum, exponentials, sum (wavefront w owns heads w, w+4, ...)
    for (int h = wave; h < G; h += WAVES) {
        float top = -INFINITY;
        for (int position = lane; position < count; position += 64)
            top = fmaxf(top, score[h][position]);
        top = wave_max(top);
        float total = 0.f;
        for (int position = lane; position < count; position += 64) {
            float e = __expf(score[h][position] - top);
            score[h][position] = e;
            total += e;
        }
        total = wave_sum(total);
        if (lane == 0 && h < group) {
            size_t index = (size_t(b) * q_heads + kvh * group + h) * splits + split;
            part_m[index] = top;
            part_l[index] = total;
        }
    }
    __syncthreads();

    // ---- 3. values: lane owns dims 2*lane, 2*lane+1
    float acc[G][2];
#pragma unroll
    for (int h = 0; h < G; ++h)
        acc[h][0] = acc[h][1] = 0.f;
    for (int p0 = wave * 4; p0 < count; p0 += WAVES * 4) {
        unsigned raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int position = p0 + u < count ? p0 + u : count - 1;
            raw[u] = *reinterpret_cast<const unsigned *>(v_base + size_t(position) * row_stride +
                                                         lane * 2);
        }
        // weights of four consecutive positions per head in one 128-bit LDS read; positions past
        // the end of the partition contribute nothing
        f32x4_t weight[G];
#pragma unroll
        for (int h = 0; h < G; ++h) {
            weight[h] = *reinterpret_cast<const f32x4_t *>(&score[h][p0]);
#pragma unroll
            for (int u = 1; u < 4; ++u)
                if (p0 + u >= count)
                    weight[h][u] = 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float lo = __uint_as_float(raw[u] << 16), hi = __uint_as_float(raw[u] & 0xffff0000u);
#pragma unroll
            for (int h = 0; h < G; ++h) {
                acc[h][0] = fmaf(weight[h][u], lo, acc[h][0]);
                acc[h][1] = fmaf(weight[h][u], hi, acc[h][1]);
            }
        }
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
        reduce[wave][h][lane * 2] = acc[h][0];
        reduce[wave][h][lane * 2 + 1] = acc[h][1];
    }
    __syncthreads();
    for (int index = thread; index < group * DIM; index += WAVES * 64) {
        int h = index / DIM, d = index % DIM;
        float sum = reduce[0][h][d];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            sum += reduce[w][h][d];
        part_o[((size_t(b) * q_heads + kvh * group + h) * splits + split) * DIM + d] = sum;
    }
}

// out[b, head, :] = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s, partitions in index order.
__global__ __launch_bounds__(DIM) void gqa_combine_kernel(int splits, const float *part_o,
                                                          const float *part_m, const float *part_l,
                                                          unsigned short *out)
{
    const size_t row = blockIdx.x; // b * q_heads + head
    const int d = threadIdx.x;
    float top = -INFINITY;
    for (int s = 0; s < splits; ++s)
        if (part_l[row * splits + s] > 0.f)
            top = fmaxf(top, part_m[row * splits + s]);
    float numerator = 0.f, denominator = 0.f;
    for (int s = 0; s < splits; ++s) {
        float l = part_l[row * splits + s];
        if (l > 0.f) {
            float factor = __expf(part_m[row * splits + s] - top);
            numerator = fmaf(factor, part_o[(row * splits + s) * DIM + d], numerator);
            denominator = fmaf(factor, l, denominator);
        }
    }
    out[row * DIM + d] = float_to_bf16_bits(denominator > 0.f ? numerator / denominator : 0.f);
}
} // namespace

size_t gqa_decode_scratch_bytes(int batch, int q_heads, int dim, int context_length, int *splits)
{
    int count = (context_length + CHUNK - 1) / CHUNK;
    if (splits)
        *splits = count;
    size_t rows = size_t(batch) * q_heads * count;
    return rows * (size_t(dim) + 2) * sizeof(float);
}

hipError_t launch_gqa_decode(hipStream_t stream, int batch, int q_heads, int kv_heads, int dim,
                             int context_length, const int32_t *lengths, float scale, const void *q,
                             int q_stride, const void *k, const void *v, void *out, void *scratch,
                             int splits)
{
    if (dim != DIM || splits > 65535 || kv_heads > 65535 || batch > 65535)
        return hipErrorInvalidValue;
    const int group = q_heads / kv_heads;
    size_t rows = size_t(batch) * q_heads * splits;
    float *part_o = static_cast<float *>(scratch);
    float *part_m = part_o + rows * DIM;
    float *part_l = part_m + rows;
    dim3 grid(splits, kv_heads, batch);
    const unsigned short *qp = static_cast<const unsigned short *>(q);
    const unsigned short *kp = static_cast<const unsigned short *>(k);
    const unsigned short *vp = static_cast<const unsigned short *>(v);
#define CAMBLAS_LAUNCH_GQA(G)                                                                      \
    gqa_partition_kernel<G><<<grid, WAVES * 64, 0, stream>>>(                                      \
        q_heads, kv_heads, context_length, lengths, scale, qp, q_stride, kp, vp, part_o, part_m,   \
        part_l, splits, group)
    if (group <= 1)
        CAMBLAS_LAUNCH_GQA(1);
    else if (group <= 2)
        CAMBLAS_LAUNCH_GQA(2);
    else if (group <= 4)
        CAMBLAS_LAUNCH_GQA(4);
    else if (group <= 8)
        CAMBLAS_LAUNCH_GQA(8);
    else
        CAMBLAS_LAUNCH_GQA(16);
#undef CAMBLAS_LAUNCH_GQA
    hipError_t status = launch_status();
    if (status != hipSuccess)
        return status;
    gqa_combine_kernel<<<unsigned(size_t(batch) * q_heads), DIM, 0, stream>>>(
        splits, part_o, part_m, part_l, static_cast<unsigned short *>(out));
    return launch_status();
}
} // namespace camblas_hip
