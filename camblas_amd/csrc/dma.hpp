// Helpers shared by the kernels that fill LDS tiles with direct loads (buffer_load ... lds).
#pragma once

#include "device.hpp"

namespace camblas_hip
{
// XOR applied to the 16-byte chunk index inside an LDS row of CH chunks: any 8 (and any 16)
// consecutive rows land on distinct banks for a fixed logical chunk, for 128-bit accesses.
template <int CH> __device__ __forceinline__ int lds_swizzle(int row)
{
    if constexpr (CH == 8)
        return ((row >> 1) & 7) ^ ((row & 1) << 2);
    else if constexpr (CH == 16)
        return row & 15;
    else
        return (((row >> 2) & 1) << 1) | (((row >> 1) ^ (row >> 3)) & 1);
}

typedef __attribute__((address_space(3))) void lds_void_t;

// 16 bytes per lane from a buffer resource straight into LDS at `lds_base + lane*16` (the base
// must be wave-uniform): buffer_load_dwordx4 ... offen lds. The source byte address is the
// resource base + per-lane `lane_offset` + wave-uniform `step_offset`; bytes past the resource's
// extent read as zero instead of faulting. A buffer load is used rather than global_load_lds
// because the compiler treats the latter as a flat access that may also touch LDS, after which it
// degrades every LDS wait in the loop to "wait for everything". Kept in a non-template function:
// inside a kernel template the host pass drops the whole instantiation when it meets a target
// builtin.
__device__ __forceinline__ void load_to_lds(__amdgpu_buffer_rsrc_t resource, unsigned lane_offset,
                                            unsigned step_offset, void *lds_base)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(resource, (lds_void_t *)lds_base, 16, lane_offset,
                                             step_offset, 0, 0);
}

// The same with 4 bytes per lane: LDS gets 64 consecutive words at `lds_base`.
__device__ __forceinline__ void load_word_to_lds(__amdgpu_buffer_rsrc_t resource, unsigned lane_offset,
                                                 unsigned step_offset, void *lds_base)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(resource, (lds_void_t *)lds_base, 4, lane_offset,
                                             step_offset, 0, 0);
}

// Raw buffer resource over `bytes` bytes starting at `base` (gfx9 descriptor word 3: 32-bit data).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_resource(const void *base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, int(bytes), 0x00020000);
}

// 16 bytes per lane written to / read from the point of coherence of the whole device (cache
// policy bit 4, "sc1": device scope on gfx950) at a byte offset inside a buffer resource. Data that
// workgroups on different XCDs hand to each other travels this way, because an ordinary store
// stays in the writer's XCD-local L2 until a release fence writes that whole cache back (and the
// reader needs an acquire fence that invalidates its own): measured +20 to +40 us per launch.
// Kept out of kernel templates: the host pass drops a template instantiation that meets a target
// builtin.
__device__ __forceinline__ void store_device_scope(__amdgpu_buffer_rsrc_t resource, unsigned offset, f32x4_t value)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, value), resource, int(offset), 0, 0x10);
}
__device__ __forceinline__ f32x4_t load_device_scope(__amdgpu_buffer_rsrc_t resource, unsigned offset)
{
    return __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(resource, int(offset), 0, 0x10));
}

// Raw buffer descriptor (gfx9 V#: base address, stride 0, `bytes` records, 32-bit data) as four
// words in scalar registers, for the loads below. `base` and `bytes` must be the same in every lane.
__device__ __forceinline__ u32x4_t uniform_descriptor(const void *base, unsigned bytes)
{
    const uintptr_t address = reinterpret_cast<uintptr_t>(base);
    return u32x4_t{unsigned(__builtin_amdgcn_readfirstlane(unsigned(address))),
                   unsigned(__builtin_amdgcn_readfirstlane(unsigned(address >> 32) & 0xffffu)),
                   unsigned(__builtin_amdgcn_readfirstlane(bytes)), 0x00020000u};
}
// load_to_lds / load_word_to_lds outside the compiler's bookkeeping of memory operations (it then
// neither counts them nor makes later LDS reads wait for them): for data that is read with
// lds_read_unordered after a wait the caller places. M0 is put back as it was, with the wait state a
// direct-to-LDS load needs after a write of M0 on either side. The loads still
// count in vmcnt, which only makes waits the compiler computes for its own loads stricter.
__device__ __forceinline__ void load_to_lds_untracked(u32x4_t descriptor, unsigned lane_offset,
                                                      unsigned step_offset, const void *lds_base)
{
    const unsigned address = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds_base)));
    const unsigned step = __builtin_amdgcn_readfirstlane(step_offset);
    unsigned saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %2, %3, %4 offen lds\n\ts_mov_b32 m0, %0\n\ts_nop 0"
                 : "=&s"(saved)
                 : "s"(address), "v"(lane_offset), "s"(descriptor), "s"(step)
                 : "memory");
}
__device__ __forceinline__ void load_word_to_lds_untracked(u32x4_t descriptor, unsigned lane_offset,
                                                           unsigned step_offset, const void *lds_base)
{
    const unsigned address = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds_base)));
    const unsigned step = __builtin_amdgcn_readfirstlane(step_offset);
    unsigned saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
                 "buffer_load_dword %2, %3, %4 offen lds\n\ts_mov_b32 m0, %0\n\ts_nop 0"
                 : "=&s"(saved)
                 : "s"(address), "v"(lane_offset), "s"(descriptor), "s"(step)
                 : "memory");
}

// One float from LDS, outside the compiler's bookkeeping of memory operations: it neither waits for
// outstanding direct-to-LDS loads before the read nor for the read before the value is used. The
// caller orders both: the data was complete at an earlier barrier, and an s_waitcnt lgkmcnt(0)
// (pipeline_barrier has one) followed by tie_after_wait lies between this read and the first use;
// keep the two a few instructions apart, so that the register is not copied or spilled in between.
template <typename T> __device__ __forceinline__ T lds_read_unordered(const T *address)
{
    static_assert(sizeof(T) == 4, "one 32-bit LDS read");
    T value;
    asm volatile("ds_read_b32 %0, %1" : "=v"(value) : "v"(static_cast<unsigned>(reinterpret_cast<uintptr_t>(address))));
    return value;
}
// Placed right after the wait that covers lds_read_unordered results: no use of the values can
// move above this point.
template <typename T, int A, int B> __device__ __forceinline__ void tie_after_wait(T (&first)[A], T (&second)[B])
{
#pragma unroll
    for (int i = 0; i < A; ++i)
        asm volatile("" : "+v"(first[i]));
#pragma unroll
    for (int i = 0; i < B; ++i)
        asm volatile("" : "+v"(second[i]));
}

// p[index] for a pointer that is the same in every lane of the wavefront (the caller's promise),
// read-only for the whole launch: a scalar load, which leaves the vector memory counter and the
// path into the compute unit's vector cache alone.
__device__ __forceinline__ float uniform_load(const float *p, int index)
{
    typedef const __attribute__((address_space(4))) float *constant_pointer;
    const uintptr_t address = reinterpret_cast<uintptr_t>(p);
    const unsigned low = __builtin_amdgcn_readfirstlane(unsigned(address));
    const unsigned high = __builtin_amdgcn_readfirstlane(unsigned(address >> 32));
    return reinterpret_cast<constant_pointer>((uintptr_t(high) << 32) | low)[index];
}

// s_waitcnt vmcnt(N) with the other counters left alone (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4, lgkmcnt 11:8).
template <int N> __device__ __forceinline__ void wait_loads()
{
    static_assert(N >= 0 && N < 64, "vmcnt holds 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}

// End of a pipeline step: wait until at most N of this wavefront's loads (the newest ones, filling
// a stage nobody reads yet) are outstanding and its own LDS reads have returned, then meet the
// other wavefronts. __syncthreads() cannot be used here: its release fence makes the compiler wait
// for every outstanding load, LDS fills included, which collapses a deeper pipeline to two stages.
// What the barrier has to order is covered by the explicit wait: fills of the stage read next
// were issued a full step earlier and are complete; reads of the stage refilled next are complete.
template <int N> __device__ __forceinline__ void pipeline_barrier()
{
    static_assert(N >= 0 && N < 64, "vmcnt holds 6 bits");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0070); // vmcnt(N) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// Workgroup index -> output tile: consecutive workgroups go to different XCDs, so each XCD is given
// a contiguous range of logical tile numbers, and logical numbers walk the tile grid in groups of
// eight feature tiles so that the tiles resident on one XCD share operand panels through its L2.
__device__ __forceinline__ void xcd_tile(int block, int tiles_n, int tiles_m, int &tile_n, int &tile_m)
{
    const int total = tiles_n * tiles_m;
    const int per = total / 8, rem = total % 8, xcd = block % 8, local = block / 8;
    const int logical = xcd * per + (xcd < rem ? xcd : rem) + local;
    // With few token tiles the weights are streamed once from memory and the token tiles of a feature
    // tile must meet in one XCD's L2: the group is then the largest one (up to eight feature tiles)
    // whose spans divide an XCD's range, so that no span straddles two XCDs (192 feature tiles by two
    // token tiles in spans of 16 put a third of the siblings on different XCDs: 1.33 times the weight
    // bytes fetched, measured; spans of 12 fit the 24 tiles of an XCD).
    int GROUP = 8;
    if (tiles_m > 1 && tiles_m <= 4 && rem == 0)
        for (int g = 8; g >= 1; --g)
            if (per % (g * tiles_m) == 0) {
                GROUP = g;
                break;
            }
    const int span = GROUP * tiles_m;
    const int first_n = (logical / span) * GROUP;
    const int group_size = (tiles_n - first_n) < GROUP ? (tiles_n - first_n) : GROUP;
    tile_n = first_n + (logical % span) % group_size;
    tile_m = (logical % span) / group_size;
}
} // namespace camblas_hip
