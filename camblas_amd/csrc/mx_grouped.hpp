// Shared by the grouped E8M0 products (mx_dma.hip, mx_wave4.hip): which tile of which group a workgroup
// of a grouped launch takes.
#pragma once
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
__device__ __forceinline__ unsigned long long uniform(unsigned long long value)
{
    const unsigned lo = __builtin_amdgcn_readfirstlane(unsigned(value));
    const unsigned hi = __builtin_amdgcn_readfirstlane(unsigned(value >> 32));
    return (static_cast<unsigned long long>(hi) << 32) | lo;
}

// Tile of a workgroup of a grouped launch (a one-dimensional grid over every tile of every group).
// A group has rows to multiply in its first ceil(counts / BM) token tiles only; the rest of its
// capacity, and all of an inactive group, are zero tiles. Workgroups are placed in order, and a
// zero tile queued between tiles with work has to wait for a whole compute unit like they do
// (32 experts at a quarter of their capacity took 86 % of the time of full ones). So the tiles with
// work are numbered first, over all groups, and the zero tiles after them: every wavefront counts
// the tiles with work of all groups (lane l looks at groups l, l + 64, ...) and finds the group
// that holds its number by a prefix sum. Within a group the token tile is the inner index; over
// the tiles with work, each XCD (workgroup number modulo 8) gets a contiguous range of numbers,
// so the token tiles of a weight panel share an L2.
// Params: groups, rows, weight_groups, tiles_n, tiles_m, active, counts.
template <int BM, typename Params> struct GroupedTiles {
    const Params &p;
    int lane;

    // token tiles with rows to multiply in group g
    __device__ unsigned working(int g) const
    {
        if (g >= p.groups)
            return 0u;
        const int index = p.active[g], count = p.counts[g];
        const int rows = index >= 0 && index < p.weight_groups ? min(max(count, 0), p.rows) : 0;
        return unsigned((rows + BM - 1) / BM);
    }
    // tiles of group g that are counted: those with work, or the zero tiles
    __device__ unsigned counted(int g, bool zero) const
    {
        const unsigned token_tiles = zero ? (g < p.groups ? unsigned(p.tiles_m) - working(g) : 0u) : working(g);
        return token_tiles * unsigned(p.tiles_n);
    }
    __device__ unsigned total(bool zero) const
    {
        unsigned sum = 0;
        for (int base = 0; base < p.groups; base += 64) {
            unsigned value = counted(base + lane, zero);
            for (int step = 1; step < 64; step <<= 1)
                value += __shfl_xor(value, step);
            sum += value;
        }
        return sum;
    }
    // group holding tile number `target` of the counted kind, and the number of the tile within it
    __device__ void locate(unsigned target, bool zero, int &group, unsigned &within) const
    {
        unsigned before = 0;
        group = p.groups - 1;
        within = 0;
        for (int base = 0; base < p.groups; base += 64) {
            const unsigned own = counted(base + lane, zero);
            unsigned inclusive = own;
            for (int step = 1; step < 64; step <<= 1) {
                const unsigned below = __shfl_up(inclusive, step);
                if (lane >= step)
                    inclusive += below;
            }
            inclusive += before;
            const unsigned long long holds = __ballot(inclusive > target);
            if (holds) {
                const int first = __builtin_ctzll(holds);
                group = base + first;
                within = target - (__shfl(inclusive, first) - __shfl(own, first));
                return;
            }
            before = __shfl(inclusive, 63);
        }
    }
};

// The tile of workgroup `block`: tiles with work first (a contiguous range of them per XCD), zero tiles after.
template <int BM, typename Params>
__device__ __forceinline__ void grouped_tile(const Params &p, int lane, unsigned block, int &group, int &tile_n, int &tile_m)
{
    const GroupedTiles<BM, Params> tiles{p, lane};
    const unsigned with_work = tiles.total(false);
    const bool zero = block >= with_work;
    unsigned number = block - with_work, within;
    if (!zero) {
        const unsigned per = with_work / 8, rest = with_work % 8, xcd = block % 8;
        number = xcd * per + min(xcd, rest) + block / 8;
    }
    tiles.locate(number, zero, group, within);
    group = __builtin_amdgcn_readfirstlane(group);
    within = __builtin_amdgcn_readfirstlane(within);
    const unsigned working = __builtin_amdgcn_readfirstlane(tiles.working(group));
    const unsigned token_tiles = zero ? unsigned(p.tiles_m) - working : working;
    tile_n = int(within / token_tiles);
    tile_m = int(within % token_tiles) + (zero ? int(working) : 0);
}
} // namespace camblas_hip
