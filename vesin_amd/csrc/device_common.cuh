// Wave64 building blocks shared by the gfx950 kernels: lane ids, DPP scans, ballot compaction helpers.
#ifndef VESIN_HIP_DEVICE_COMMON_CUH
#define VESIN_HIP_DEVICE_COMMON_CUH

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "geometry.hpp"

namespace vesin_hip {

constexpr int WAVE = 64;
constexpr int BLOCK = 256;

/// Points `i` one wave searches for at a time (a tile). 32 keeps the hit column of a candidate in one register and the
/// tile's LDS record small, which buys a sixth wave per SIMD in the single-pass search; cells with more points
/// simply make several tiles.
constexpr uint32_t TILE_POINTS = 32;
constexpr uint32_t TILE_SHIFT = 5;
static_assert((1u << TILE_SHIFT) == TILE_POINTS, "TILE_SHIFT is log2 of TILE_POINTS");
constexpr int WAVES_PER_BLOCK = BLOCK / WAVE;

/// Everything a kernel needs to know about the box and the cell grid.
struct GridParams {
    double H[9];          // normalised box, row-major
    double Hinv[9];       // inverse, row-major: frac[d] = sum_k r[k] * Hinv[3k + d]
    double np_min[3];     // non-periodic directions: offset of the projected coordinate
    double np_scale[3];   // non-periodic directions: 1 / extent
    double cutoff2;
    int32_t n[3];         // cells per direction
    int32_t s[3];         // stencil radius per direction
    int32_t periodic[3];
    uint32_t n_points;
    uint32_t n_cells;
    // Stencil entries that cannot hold a neighbour (stencils of radius two and more: the corners of the block of
    // cells lie outside the cutoff sphere). With the edge vectors of a cell written in an orthonormal frame whose
    // first axis lies along the first edge and whose second lies in the plane of the first two (prune_edges: x of
    // the three edges, y of the second and third, z of the third), two points in cells (dx, dy, dz) apart differ
    // along each axis by at least |what the whole cells contribute| - prune_slack (the most that the places of the
    // two points inside their cells can take back). An entry is dropped when the squares of these three lower
    // bounds add up to more than prune_limit. prune = 0: nothing is dropped.
    double prune_edges[6];
    double prune_slack[3];
    double prune_limit;
    int32_t prune;
};

/// One row of TILE_POINTS i-points (or fewer) that one wave searches for.
struct Tile {
    uint32_t cell;   // linear cell index of these points
    uint32_t first;  // position of the first point in the cell-sorted arrays
    uint32_t count;  // 1..TILE_POINTS
    uint32_t wrapped;// 1 when a point of the cell was moved by a box vector to land inside the box
};

/// Small block of results the host reads back after the counting pass.
struct DeviceStatus {
    unsigned long long total_pairs;
    unsigned int first_bad_coordinate; // 3 * point + axis of the first non-finite coordinate, or 0xFFFFFFFF
    unsigned int crowded_cells;        // fixed-capacity layout: points that found their cell full
    unsigned int far_outside;          // points more than a cell outside the extent the grid was chosen for
    unsigned int padding;
};

/// What one workgroup of the bounding pass reports (to pinned host memory; the host folds the workgroups).
struct BlockBounds {
    double lo[3]; // smallest / largest projected coordinate; lo > hi when the workgroup saw no finite point
    double hi[3];
    unsigned int first_bad_coordinate;
    unsigned int padding;
};

constexpr int BOUNDING_BLOCKS = 256;

__device__ __forceinline__ int lane_id() {
    return static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
}

/// Number of set bits of `mask` below this lane: the slot of this lane after compaction.
__device__ __forceinline__ uint32_t rank_in_mask(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_zero(uint32_t v) {
    // lanes without a valid source (or in rows that are masked off) receive 0
    return static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, ROW_MASK, 0xf, false)
    );
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t dpp_or_zero64(uint64_t v) {
    uint32_t lo = dpp_or_zero<CTRL, ROW_MASK>(static_cast<uint32_t>(v));
    uint32_t hi = dpp_or_zero<CTRL, ROW_MASK>(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

/// Inclusive prefix sum over the 64 lanes of a wave, data moved with DPP only (row shifts inside each row of 16
/// lanes, then row_bcast:15 and row_bcast:31 to carry row totals forward).
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
    v += dpp_or_zero<0x111, 0xf>(v); // row_shr:1
    v += dpp_or_zero<0x112, 0xf>(v); // row_shr:2
    v += dpp_or_zero<0x114, 0xf>(v); // row_shr:4
    v += dpp_or_zero<0x118, 0xf>(v); // row_shr:8
    v += dpp_or_zero<0x142, 0xa>(v); // row_bcast:15 into rows 1 and 3
    v += dpp_or_zero<0x143, 0xc>(v); // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ uint64_t wave_inclusive_scan(uint64_t v) {
    v += dpp_or_zero64<0x111, 0xf>(v);
    v += dpp_or_zero64<0x112, 0xf>(v);
    v += dpp_or_zero64<0x114, 0xf>(v);
    v += dpp_or_zero64<0x118, 0xf>(v);
    v += dpp_or_zero64<0x142, 0xa>(v);
    v += dpp_or_zero64<0x143, 0xc>(v);
    return v;
}

/// A value that is the same in every lane, moved to scalar registers (tells the compiler it is wave-uniform).
__device__ __forceinline__ uint32_t uniform(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
}

__device__ __forceinline__ uint64_t uniform(uint64_t v) {
    return (static_cast<uint64_t>(uniform(static_cast<uint32_t>(v >> 32))) << 32) | uniform(static_cast<uint32_t>(v));
}

__device__ __forceinline__ uint32_t read_lane(uint32_t v, int lane) {
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), lane));
}

__device__ __forceinline__ uint64_t read_lane(uint64_t v, int lane) {
    uint32_t lo = read_lane(static_cast<uint32_t>(v), lane);
    uint32_t hi = read_lane(static_cast<uint32_t>(v >> 32), lane);
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

typedef unsigned long long PairRow __attribute__((ext_vector_type(2)));
typedef int32_t ShiftRow __attribute__((ext_vector_type(3), aligned(4)));
typedef double VectorHead __attribute__((ext_vector_type(2), aligned(8))); // first two of the three components

/// Output rows are written once and never read by this kernel: non-temporal stores keep them from displacing the
/// cell-sorted points in L2.
template <typename T>
__device__ __forceinline__ void stream_store(void* address, T value) {
    __builtin_nontemporal_store(value, reinterpret_cast<T*>(address));
}

/// The vectors of up to 64 consecutive rows (lane l holds row l of a block that starts on a multiple of 64 rows; the
/// rows of lanes [lo, hi) are there) go to memory as 16-byte pieces of consecutive addresses, one piece per lane and
/// store instruction, after they were lined up in LDS (`stage`: 192 doubles of the wave's own); a first or last row
/// that starts or ends in the middle of a piece stores that half on its own. Stored row by row (16 + 8 bytes per lane,
/// 24 bytes apart), every store instruction leaves holes in the cache lines it touches for the next one to fill, and
/// kernels that are held up by their stores write the vectors at half the rate of their other rows.
__device__ __forceinline__ void store_vector_block(
    double* stage, char* block, uint32_t lo, uint32_t hi, bool active, uint32_t lane, double x, double y, double z
) {
    // (the lanes of a wave read what other lanes wrote: the LDS serves a wave's accesses in the order they were
    // issued, which a fence of wavefront scope tells the compiler to keep; nothing waits for the row stores in flight)
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (active) {
        stage[3 * lane + 0] = x;
        stage[3 * lane + 1] = y;
        stage[3 * lane + 2] = z;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const uint32_t begin = 24u * lo;
    const uint32_t end = 24u * hi;
#pragma unroll
    for (uint32_t turn = 0; turn < 2; turn++) {
        const uint32_t piece = turn * WAVE + lane; // 96 pieces of 16 bytes make 64 rows
        const uint32_t at = 16u * piece;
        if (piece < 3 * WAVE / 2) {
            if (at >= begin && at + 16u <= end) {
                stream_store(block + at, VectorHead{stage[2 * piece], stage[2 * piece + 1]});
            } else if (at + 8u == begin && at + 16u <= end) {
                stream_store(block + at + 8u, stage[2 * piece + 1]);
            } else if (at >= begin && at + 8u == end) {
                stream_store(block + at, stage[2 * piece]);
            }
        }
    }
}

} // namespace vesin_hip

#endif
