// Cell-list construction on the GPU: projected bounding box, cell assignment in fractional coordinates,
// counting sort of the points by cell (histogram -> device-wide scan -> scatter), and the per-cell pass that
// puts every cell in a canonical order and lays the points out as 32-byte records, cell by cell, for the search
// kernel.
//
// Reference roles replaced: compute_bounding_box (vesin/src/cuda/cell_list.cu:69-133), assign_cell_indices
// (:279-333), count_particles_per_cell (:335-345), prefix_sum_cells (:347-390), scatter_particles (:392-421);
// CPU twin CellList::add_point (vesin/src/cpu_cell_list.cpp:353-374).
#ifndef VESIN_HIP_CELLS_CUH
#define VESIN_HIP_CELLS_CUH

#include "device_common.cuh"

namespace vesin_hip {

/// What the single-pass search kernel tells the host besides the rows themselves.
struct FusedStatus {
    unsigned long long total_rows; // written by the last workgroup
    unsigned long long deferred_rows; // rows of the deferred work items
    unsigned int general;          // work items outside of the shape that kernel covers
    unsigned int deferred;         // work items that kernel counted and placed but left to the write pass
    unsigned int overflow;         // workgroups whose rows did not fit the output arrays
    unsigned int chain_timeout;    // waves that gave up waiting for an earlier workgroup
    unsigned int first_bad_coordinate;
    unsigned int crowded_cells;    // fixed-capacity layout: points that found their cell full (the result is void)
    unsigned int far_outside;      // points more than a cell outside the extent the grid was chosen for (same)
    unsigned int padding;
};

/// One cell-sorted point: coordinates and original index in 32 bytes, aligned. A point in arbitrary input order is
/// stored wherever its cell lies: one 32-byte sector of memory traffic then, where a store per component (and one
/// for the index) cost four; 64 consecutive candidates still load coalesced (2 KB in a row), and a point of a tile
/// arrives with one scalar load.
struct alignas(32) SortedPoint {
    double x, y, z;
    uint32_t index; // original point index
    uint32_t spare;
};

/// Cell-sorted copy of the points. `p` is allocated with SORTED_PADDING extra elements so that the scalar loads of
/// four consecutive points may run past the last point; the shifts (rarely non-zero, rarely read) keep an array each.
struct SortedPoints {
    SortedPoint* p;
    int32_t* wx; // number of box vectors the point was moved by to land inside the box
    int32_t* wy;
    int32_t* wz;
    float4* l;   // the place of the point inside its cell, in single precision (choose_prefilter, geometry.hpp); same
                 // padding as `p`
};

__device__ __forceinline__ float4 local_record(const Prefilter& g, const double inside[3], const int32_t wrap[3]) {
    float place[3];
    local_place(g, inside, wrap, place);
    return float4{place[0], place[1], place[2], 0.0f};
}

constexpr uint32_t SORTED_PADDING = 8;

/// First kernel of a call: box and periodicity go to pinned host memory (the host picks the grid from them), and
/// the status block is reset.
__global__ void fetch_box(
    const double* __restrict__ box, const bool* __restrict__ periodic, unsigned char* host_small, DeviceStatus* status
) {
    const int t = threadIdx.x;
    if (t < 9) {
        reinterpret_cast<double*>(host_small)[t] = box[t];
    } else if (t < 12) {
        host_small[72 + (t - 9)] = periodic[t - 9] ? 1 : 0;
    } else if (t == 12) {
        status->total_pairs = 0;
        status->first_bad_coordinate = 0xFFFFFFFFu;
        status->crowded_cells = 0;
        status->far_outside = 0;
    }
}

/// Clears `n_blocks16` 16-byte blocks from `begin` (the histogram, the tiles' flags and the state of the single-pass
/// search live next to each other), and does the work of fetch_box on the way when `box` is not null: one launch
/// at the start of a call instead of a fetch and two fills.
__device__ __forceinline__ void clear_and_fetch_as(
    uint32_t block, uint32_t n_blocks, uint4* __restrict__ begin, size_t n_blocks16, const double* __restrict__ box,
    const bool* __restrict__ periodic, unsigned char* host_small, DeviceStatus* status
) {
    if (box != nullptr && block == 0) {
        const int t = threadIdx.x;
        if (t < 9) {
            reinterpret_cast<double*>(host_small)[t] = box[t];
        } else if (t < 12) {
            host_small[72 + (t - 9)] = periodic[t - 9] ? 1 : 0;
        } else if (t == 12) {
            status->total_pairs = 0;
            status->first_bad_coordinate = 0xFFFFFFFFu;
            status->crowded_cells = 0;
            status->far_outside = 0;
        }
    }
    const uint4 zero = {0u, 0u, 0u, 0u};
    for (size_t k = static_cast<size_t>(block) * BLOCK + threadIdx.x; k < n_blocks16;
         k += static_cast<size_t>(n_blocks) * BLOCK) {
        begin[k] = zero;
    }
}

__global__ __launch_bounds__(BLOCK) void clear_and_fetch(
    uint4* __restrict__ begin, size_t n_blocks16, const double* __restrict__ box, const bool* __restrict__ periodic,
    unsigned char* host_small, DeviceStatus* status
) {
    clear_and_fetch_as(blockIdx.x, gridDim.x, begin, n_blocks16, box, periodic, host_small, status);
}

/// After the counting pass: what the host needs to know goes to pinned host memory, read after the next
/// synchronisation of the stream.
__global__ void publish_status(const DeviceStatus* status, const uint64_t* total, DeviceStatus* host_status) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        host_status->first_bad_coordinate = status->first_bad_coordinate;
        host_status->total_pairs = *total;
    }
}

/// Same after the single-pass search.
__global__ void publish_fused_status(const DeviceStatus* status, const FusedStatus* fused, FusedStatus* host_fused) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        FusedStatus copy = *fused;
        copy.first_bad_coordinate = status->first_bad_coordinate;
        copy.crowded_cells = status->crowded_cells;
        copy.far_outside = status->far_outside;
        copy.padding = 0;
        *host_fused = copy;
    }
}

__device__ __forceinline__ void fractional(const GridParams& g, double x, double y, double z, double f[3]) {
#pragma unroll
    for (int d = 0; d < 3; d++) {
        f[d] = x * g.Hinv[d] + y * g.Hinv[3 + d] + z * g.Hinv[6 + d];
    }
}

__device__ __forceinline__ bool all_finite(double x, double y, double z, unsigned int& bad_axis) {
    if (!isfinite(x)) {
        bad_axis = 0;
        return false;
    }
    if (!isfinite(y)) {
        bad_axis = 1;
        return false;
    }
    if (!isfinite(z)) {
        bad_axis = 2;
        return false;
    }
    return true;
}

/// Smallest and largest fractional coordinate over all points (needed for non-periodic directions), plus the
/// check for non-finite input. Grid-stride loop, wave then workgroup reduction; every workgroup reports to its own
/// slot of `host_bounds` (pinned host memory), so no atomics are involved.
__device__ __forceinline__ void bounding_as(
    uint32_t block, uint32_t n_blocks, const double* __restrict__ points, uint32_t n_points, const GridParams& g,
    BlockBounds* host_bounds
) {
    __shared__ BlockBounds partial[WAVES_PER_BLOCK];
    double lo[3] = {INFINITY, INFINITY, INFINITY};
    double hi[3] = {-INFINITY, -INFINITY, -INFINITY};
    unsigned int bad = 0xFFFFFFFFu;

    for (uint32_t i = block * BLOCK + threadIdx.x; i < n_points; i += n_blocks * BLOCK) {
        double x = points[3 * static_cast<size_t>(i) + 0];
        double y = points[3 * static_cast<size_t>(i) + 1];
        double z = points[3 * static_cast<size_t>(i) + 2];
        unsigned int axis;
        if (!all_finite(x, y, z, axis)) {
            bad = min(bad, 3u * i + axis);
            continue;
        }
        double f[3];
        fractional(g, x, y, z, f);
#pragma unroll
        for (int d = 0; d < 3; d++) {
            lo[d] = fmin(lo[d], f[d]);
            hi[d] = fmax(hi[d], f[d]);
        }
    }

#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
#pragma unroll
        for (int d = 0; d < 3; d++) {
            lo[d] = fmin(lo[d], __shfl_xor(lo[d], offset));
            hi[d] = fmax(hi[d], __shfl_xor(hi[d], offset));
        }
        bad = min(bad, static_cast<unsigned int>(__shfl_xor(static_cast<int>(bad), offset)));
    }

    if (lane_id() == 0) {
        BlockBounds& mine = partial[threadIdx.x / WAVE];
#pragma unroll
        for (int d = 0; d < 3; d++) {
            mine.lo[d] = lo[d];
            mine.hi[d] = hi[d];
        }
        mine.first_bad_coordinate = bad;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        BlockBounds all = partial[0];
        for (int w = 1; w < WAVES_PER_BLOCK; w++) {
#pragma unroll
            for (int d = 0; d < 3; d++) {
                all.lo[d] = fmin(all.lo[d], partial[w].lo[d]);
                all.hi[d] = fmax(all.hi[d], partial[w].hi[d]);
            }
            all.first_bad_coordinate = min(all.first_bad_coordinate, partial[w].first_bad_coordinate);
        }
        all.padding = 0;
        host_bounds[block] = all;
    }
}

__global__ __launch_bounds__(BLOCK) void bounding_kernel(
    const double* __restrict__ points, uint32_t n_points, GridParams g, BlockBounds* host_bounds
) {
    bounding_as(blockIdx.x, gridDim.x, points, n_points, g, host_bounds);
}

/// Both of the above in one launch, for a call whose grid follows the extent the call before found: the first
/// `clear_blocks` workgroups clear and fetch the box, the others find the extent of this call's points, which the
/// host reads at the end of the call (for the call after this one).
__global__ __launch_bounds__(BLOCK) void clear_fetch_and_bound(
    uint32_t clear_blocks, uint4* __restrict__ begin, size_t n_blocks16, const double* __restrict__ box,
    const bool* __restrict__ periodic, unsigned char* host_small, DeviceStatus* status,
    const double* __restrict__ points, uint32_t n_points, GridParams g, BlockBounds* host_bounds
) {
    if (blockIdx.x < clear_blocks) {
        clear_and_fetch_as(blockIdx.x, clear_blocks, begin, n_blocks16, box, periodic, host_small, status);
    } else {
        bounding_as(blockIdx.x - clear_blocks, gridDim.x - clear_blocks, points, n_points, g, host_bounds);
    }
}

/// Cell coordinates and wrap shift of one point. Periodic directions: cell = floor(frac * n) brought back into
/// [0, n) with the quotient kept as the wrap shift. Non-periodic directions: clamped, never wrapped.
/// `inside` (when asked for): where the point lies in its cell along every direction, in units of the cell, 0 to 1
/// for a point the cell holds (a point of an open direction that was put into the outermost cell may lie beyond).
__device__ __forceinline__ void locate(
    const GridParams& g, double x, double y, double z, int32_t cell[3], int32_t wrap[3], bool* far_outside = nullptr,
    double* inside = nullptr
) {
    double f[3];
    fractional(g, x, y, z, f);
#pragma unroll
    for (int d = 0; d < 3; d++) {
        const int32_t n = g.n[d];
        if (g.periodic[d]) {
            const double in_cells = f[d] * static_cast<double>(n);
            double scaled = floor(in_cells);
            if (inside != nullptr) {
                inside[d] = in_cells - scaled;
            }
            scaled = fmin(fmax(scaled, -2.0e9), 2.0e9);
            int32_t c = static_cast<int32_t>(scaled);
            int32_t q = c / n;
            int32_t r = c - q * n;
            if (r < 0) {
                r += n;
                q -= 1;
            }
            cell[d] = r;
            wrap[d] = q;
        } else {
            const double in_cells = (f[d] - g.np_min[d]) * g.np_scale[d] * static_cast<double>(n);
            double scaled = floor(in_cells);
            if (inside != nullptr) {
                inside[d] = in_cells - fmin(fmax(scaled, 0.0), static_cast<double>(n - 1));
            }
            if (far_outside != nullptr && (scaled < -1.0 || scaled > static_cast<double>(n))) {
                // (a grid chosen for the points of this call holds them all; one chosen for those of the call
                // before still gives the right list while points land in the outermost cells instead, but not
                // in a sensible time once the points are somewhere else altogether)
                *far_outside = true;
            }
            scaled = fmin(fmax(scaled, 0.0), static_cast<double>(n - 1));
            cell[d] = static_cast<int32_t>(scaled);
            wrap[d] = 0;
        }
    }
}

/// Points per tile of a cell of `count` points: the cell is cut into ceil(count / TILE_POINTS) tiles of equal size
/// (the last one short by less than the number of tiles) instead of full tiles and a rest: a cell of 40 points is
/// two tiles of 20, not 32 + 8, whose waves would sit at the same workgroup barriers with four times the work of
/// one another.
__device__ __forceinline__ uint32_t tile_size_of(uint32_t count) {
    const uint32_t n_tiles = (count + TILE_POINTS - 1) >> TILE_SHIFT;
    return n_tiles <= 1 ? static_cast<uint32_t>(TILE_POINTS) : (count + n_tiles - 1) / n_tiles;
}

/// One thread per point: cell id, wrap shift, and the histogram of points per cell. The value returned by the
/// histogram atomic is kept as the point's provisional slot inside its cell. Lanes of a wave that fall in the same
/// cell (the usual case for spatially coherent input) are grouped first, for up to ASSIGN_ROUNDS distinct cells
/// per wave, so that one lane per group issues the atomic for all of them.
constexpr int ASSIGN_ROUNDS = 8;

__global__ __launch_bounds__(BLOCK) void assign_cells(
    const double* __restrict__ points, GridParams g,
    uint32_t* __restrict__ cell_of, uint32_t* __restrict__ slot_of, int32_t* __restrict__ wrap_of,
    uint32_t* __restrict__ cell_counts, DeviceStatus* status
) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    bool active = i < g.n_points;
    const int lane = lane_id();

    int32_t cell[3] = {0, 0, 0};
    int32_t wrap[3] = {0, 0, 0};
    if (active) {
        double x = points[3 * static_cast<size_t>(i) + 0];
        double y = points[3 * static_cast<size_t>(i) + 1];
        double z = points[3 * static_cast<size_t>(i) + 2];
        unsigned int axis;
        if (all_finite(x, y, z, axis)) {
            bool far_outside = false;
            locate(g, x, y, z, cell, wrap, &far_outside);
            if (far_outside) {
                // left out of the cell list (place_points does the same): the result is void, the search short
                atomicAdd(&status->far_outside, 1u);
                active = false;
            }
        } else {
            atomicMin(&status->first_bad_coordinate, 3u * i + axis);
        }
    }
    const uint32_t linear = (static_cast<uint32_t>(cell[2]) * g.n[1] + cell[1]) * g.n[0] + cell[0];

    uint64_t group = 1ull << lane; // lanes left over after the rounds stand alone
    bool pending = active;
    for (int round = 0; round < ASSIGN_ROUNDS; round++) {
        const uint64_t remaining = __ballot(pending);
        if (remaining == 0) {
            break;
        }
        const int leader = __ffsll(static_cast<unsigned long long>(remaining)) - 1;
        const uint32_t leader_cell = read_lane(linear, leader);
        const bool same = pending && linear == leader_cell;
        const uint64_t members = __ballot(same);
        if (same) {
            group = members;
            pending = false;
        }
    }

    const int first = __ffsll(static_cast<unsigned long long>(group)) - 1;
    uint32_t base = 0;
    if (active && lane == first) {
        base = atomicAdd(&cell_counts[linear], static_cast<uint32_t>(__popcll(group)));
    }
    base = static_cast<uint32_t>(__shfl(static_cast<int>(base), first));
    if (active) {
        slot_of[i] = base + rank_in_mask(group);
        // callers that place the points with `place_points` do not need these: it locates the point again
        if (cell_of != nullptr) {
            cell_of[i] = linear;
            wrap_of[3 * static_cast<size_t>(i) + 0] = wrap[0];
            wrap_of[3 * static_cast<size_t>(i) + 1] = wrap[1];
            wrap_of[3 * static_cast<size_t>(i) + 2] = wrap[2];
        }
    }
}

/// Cell build in one pass, for the single-pass search: every cell owns `capacity` slots of the cell-sorted arrays
/// (cell c: slots c * capacity ...), a point takes the slot the histogram atomic hands out and is written there at
/// once. No scan, no second pass over the points; the search reads a cell's points as (c * capacity, count[c]).
/// A point that finds its cell full is counted in `status->crowded_cells` and dropped: the host then builds the
/// packed layout instead. `wrapped[c * capacity / TILE_POINTS + k]` is set when tile k of cell c holds a point
/// that was moved by a box vector. Lanes of a wave in the same cell share one atomic, like in assign_cells.
__global__ __launch_bounds__(BLOCK) void place_direct(
    const double* __restrict__ points, GridParams g, uint32_t capacity, uint32_t* __restrict__ cell_counts,
    uint32_t* __restrict__ wrapped, SortedPoints sorted, DeviceStatus* status
) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    bool active = i < g.n_points;
    const int lane = lane_id();

    int32_t cell[3] = {0, 0, 0};
    int32_t wrap[3] = {0, 0, 0};
    double x = 0.0, y = 0.0, z = 0.0;
    if (active) {
        x = points[3 * static_cast<size_t>(i) + 0];
        y = points[3 * static_cast<size_t>(i) + 1];
        z = points[3 * static_cast<size_t>(i) + 2];
        unsigned int axis;
        if (all_finite(x, y, z, axis)) {
            bool far_outside = false;
            locate(g, x, y, z, cell, wrap, &far_outside);
            if (far_outside) {
                atomicAdd(&status->far_outside, 1u); // dropped, like a point that finds its cell full
                active = false;
            }
        } else {
            atomicMin(&status->first_bad_coordinate, 3u * i + axis);
        }
    }
    const uint32_t linear = (static_cast<uint32_t>(cell[2]) * g.n[1] + cell[1]) * g.n[0] + cell[0];

    uint64_t group = 1ull << lane; // lanes left over after the rounds stand alone
    bool pending = active;
    for (int round = 0; round < ASSIGN_ROUNDS; round++) {
        const uint64_t remaining = __ballot(pending);
        if (remaining == 0) {
            break;
        }
        const int leader = __ffsll(static_cast<unsigned long long>(remaining)) - 1;
        const uint32_t leader_cell = read_lane(linear, leader);
        const bool same = pending && linear == leader_cell;
        const uint64_t members = __ballot(same);
        if (same) {
            group = members;
            pending = false;
        }
    }
    const int first = __ffsll(static_cast<unsigned long long>(group)) - 1;
    uint32_t base = 0;
    if (active && lane == first) {
        base = atomicAdd(&cell_counts[linear], static_cast<uint32_t>(__popcll(group)));
    }
    base = static_cast<uint32_t>(__shfl(static_cast<int>(base), first));
    if (!active) {
        return;
    }
    const uint32_t k = base + rank_in_mask(group);
    if (k >= capacity) {
        atomicAdd(&status->crowded_cells, 1u);
        return;
    }
    const size_t to = static_cast<size_t>(linear) * capacity + k;
    sorted.p[to] = SortedPoint{x, y, z, i, 0u};
    if ((wrap[0] | wrap[1] | wrap[2]) != 0) {
        // (the caller hands the wrap arrays over cleared, as for place_points)
        sorted.wx[to] = wrap[0];
        sorted.wy[to] = wrap[1];
        sorted.wz[to] = wrap[2];
        atomicOr(&wrapped[(linear * capacity + k) / TILE_POINTS], 1u);
    }
}

/// Counting-sort scatter: the point goes to (start of its cell) + (its provisional slot).
__global__ __launch_bounds__(BLOCK) void scatter_points(
    uint32_t n_points, const uint32_t* __restrict__ cell_of, const uint32_t* __restrict__ slot_of,
    const uint64_t* __restrict__ cell_scan, uint32_t* __restrict__ provisional
) {
    uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= n_points) {
        return;
    }
    uint32_t start = static_cast<uint32_t>(cell_scan[cell_of[i]]);
    provisional[start + slot_of[i]] = i;
}

/// Counting-sort scatter straight into the cell-sorted records, for callers that do not need the order of
/// the points inside a cell to be the same on every run: the slot handed out by the histogram atomic is final.
/// Also appends the cell's tiles. `tiles[].wrapped` must be zero on entry. Cell and wrap shift of the point come
/// from `cell_of` / `wrap_of` when given (a batch of systems), else the point is located again with `g`: cheaper
/// than carrying 16 bytes per point from assign_cells through memory; in that case `sorted.wx / wy / wz` must be
/// zero on entry, only the shifts of moved points are stored.
__global__ __launch_bounds__(BLOCK) void place_points(
    const double* __restrict__ points, GridParams g, const int32_t* __restrict__ wrap_of,
    const uint32_t* __restrict__ cell_of, const uint32_t* __restrict__ slot_of,
    const uint64_t* __restrict__ cell_scan, uint32_t n_points, SortedPoints sorted, Tile* __restrict__ tiles,
    const uint32_t* __restrict__ system_of, const uint32_t* __restrict__ first_point, Prefilter pre = Prefilter()
) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= n_points) {
        return;
    }
    const double x = points[3 * static_cast<size_t>(i) + 0];
    const double y = points[3 * static_cast<size_t>(i) + 1];
    const double z = points[3 * static_cast<size_t>(i) + 2];
    uint32_t cell;
    int32_t wx, wy, wz;
    float4 place = {0.0f, 0.0f, 0.0f, 0.0f};
    if (cell_of != nullptr) {
        cell = cell_of[i];
        wx = wrap_of[3 * static_cast<size_t>(i) + 0];
        wy = wrap_of[3 * static_cast<size_t>(i) + 1];
        wz = wrap_of[3 * static_cast<size_t>(i) + 2];
    } else {
        // same inputs and code as in assign_cells: the same cell
        int32_t where[3] = {0, 0, 0};
        int32_t wrap[3] = {0, 0, 0};
        double inside[3] = {0.0, 0.0, 0.0};
        unsigned int axis;
        if (all_finite(x, y, z, axis)) {
            bool far_outside = false;
            locate(g, x, y, z, where, wrap, &far_outside, inside);
            if (far_outside) {
                return; // assign_cells did not count it
            }
        }
        cell = (static_cast<uint32_t>(where[2]) * g.n[1] + where[1]) * g.n[0] + where[0];
        wx = wrap[0];
        wy = wrap[1];
        wz = wrap[2];
        if (sorted.l != nullptr) {
            place = local_record(pre, inside, wrap);
        }
    }
    const uint64_t here = cell_scan[cell];
    const uint32_t start = static_cast<uint32_t>(here);
    const uint32_t count = static_cast<uint32_t>(cell_scan[cell + 1]) - start;
    const uint32_t first_tile = static_cast<uint32_t>(here >> 32);
    const uint32_t k = slot_of[i];
    const uint32_t to = start + k;

    // in a batch (system_of not null) the index counts from the first point of the point's system, and the tile
    // carries the system above its flag bit
    const uint32_t system = system_of != nullptr ? system_of[i] : 0;
    sorted.p[to] = SortedPoint{x, y, z, system_of != nullptr ? i - first_point[system] : i, 0u};
    if (sorted.l != nullptr) {
        sorted.l[to] = place;
    }
    const uint32_t tile_size = tile_size_of(count);
    // A single system's caller hands the wrap arrays over cleared: points in arbitrary order scatter their stores, a
    // 32-byte sector of memory traffic for each, and most points were not moved by any box vector.
    if (cell_of != nullptr || (wx | wy | wz) != 0) {
        sorted.wx[to] = wx;
        sorted.wy[to] = wy;
        sorted.wz[to] = wz;
    }
    if ((wx | wy | wz) != 0) {
        atomicOr(&tiles[first_tile + k / tile_size].wrapped, 1u);
    }
    if (k % tile_size == 0) {
        Tile* tile = &tiles[first_tile + k / tile_size];
        tile->cell = cell;
        tile->first = to;
        tile->count = min(tile_size, count - k);
        if (system != 0) {
            atomicOr(&tile->wrapped, system << 1);
        }
    }
}

/// Bounding pass of a batch: one wave per system finds the extrema of the fractional coordinates of its points
/// (with that system's inverse box, which is all `grids` needs to hold at this point) and the first non-finite
/// coordinate. Only launched when some system has a non-periodic direction.
__global__ __launch_bounds__(BLOCK) void bounding_batch_kernel(
    const double* __restrict__ points, const GridParams* __restrict__ grids, const uint32_t* __restrict__ first_point,
    uint32_t n_systems, BlockBounds* __restrict__ bounds
) {
    const uint32_t system = blockIdx.x * WAVES_PER_BLOCK + threadIdx.x / WAVE;
    if (system >= n_systems) {
        return;
    }
    const GridParams& g = grids[system];
    double lo[3] = {INFINITY, INFINITY, INFINITY};
    double hi[3] = {-INFINITY, -INFINITY, -INFINITY};
    unsigned int bad = 0xFFFFFFFFu;
    const uint32_t end = first_point[system + 1];
    for (uint32_t i = first_point[system] + lane_id(); i < end; i += WAVE) {
        const double x = points[3 * static_cast<size_t>(i) + 0];
        const double y = points[3 * static_cast<size_t>(i) + 1];
        const double z = points[3 * static_cast<size_t>(i) + 2];
        unsigned int axis;
        if (!all_finite(x, y, z, axis)) {
            bad = min(bad, 3u * i + axis);
            continue;
        }
        double f[3];
        fractional(g, x, y, z, f);
#pragma unroll
        for (int d = 0; d < 3; d++) {
            lo[d] = fmin(lo[d], f[d]);
            hi[d] = fmax(hi[d], f[d]);
        }
    }
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
#pragma unroll
        for (int d = 0; d < 3; d++) {
            lo[d] = fmin(lo[d], __shfl_xor(lo[d], offset));
            hi[d] = fmax(hi[d], __shfl_xor(hi[d], offset));
        }
        bad = min(bad, static_cast<unsigned int>(__shfl_xor(static_cast<int>(bad), offset)));
    }
    if (lane_id() == 0) {
        BlockBounds all;
#pragma unroll
        for (int d = 0; d < 3; d++) {
            all.lo[d] = lo[d];
            all.hi[d] = hi[d];
        }
        all.first_bad_coordinate = bad;
        all.padding = 0;
        bounds[system] = all;
    }
}

/// Grids of a batch whose systems have no periodic direction at all (free molecules), picked where the points are:
/// one wave per system finds the extent of its points and its first lane picks the grid, as `choose_grid`
/// (geometry.hpp) does on the host for such a system: the box counts for nothing (the three directions are unit
/// vectors), cells at least as wide as the cutoff over the extent of the points with a margin of 1 %, never more
/// cells than twice the points (or 64), nothing beyond the last cell. `single_cell`: 1 always (brute force), 0 for
/// systems that fill more than a cell and have `few_points` points or more (automatic choice: 32, or more where the
/// search that follows is at its best on systems of one cell), -1 never (cell list).
__global__ __launch_bounds__(BLOCK) void open_grids_kernel(
    const double* __restrict__ points, const uint32_t* __restrict__ first_point, uint32_t n_systems, double cutoff,
    int single_cell, uint32_t few_points, GridParams* __restrict__ grids, uint32_t* __restrict__ cells_of_system,
    unsigned int* first_bad
) {
    const uint32_t system = blockIdx.x * WAVES_PER_BLOCK + threadIdx.x / WAVE;
    if (system >= n_systems) {
        return;
    }
    double lo[3] = {INFINITY, INFINITY, INFINITY};
    double hi[3] = {-INFINITY, -INFINITY, -INFINITY};
    unsigned int bad = 0xFFFFFFFFu;
    const uint32_t begin = first_point[system];
    const uint32_t end = first_point[system + 1];
    for (uint32_t i = begin + lane_id(); i < end; i += WAVE) {
        const double r[3] = {
            points[3 * static_cast<size_t>(i) + 0], points[3 * static_cast<size_t>(i) + 1],
            points[3 * static_cast<size_t>(i) + 2]
        };
        unsigned int axis;
        if (!all_finite(r[0], r[1], r[2], axis)) {
            bad = min(bad, 3u * i + axis);
            continue;
        }
#pragma unroll
        for (int d = 0; d < 3; d++) {
            lo[d] = fmin(lo[d], r[d]);
            hi[d] = fmax(hi[d], r[d]);
        }
    }
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
#pragma unroll
        for (int d = 0; d < 3; d++) {
            lo[d] = fmin(lo[d], __shfl_xor(lo[d], offset));
            hi[d] = fmax(hi[d], __shfl_xor(hi[d], offset));
        }
        bad = min(bad, static_cast<unsigned int>(__shfl_xor(static_cast<int>(bad), offset)));
    }
    if (lane_id() != 0) {
        return;
    }
    if (bad != 0xFFFFFFFFu) {
        atomicMin(first_bad, bad);
    }
    const uint32_t n_here = end - begin;
    const double padded = cutoff * (1.0 + 1e-9);
    GridParams g;
    for (int k = 0; k < 9; k++) {
        g.H[k] = (k % 4 == 0) ? 1.0 : 0.0;
        g.Hinv[k] = (k % 4 == 0) ? 1.0 : 0.0;
    }
    double extent[3];
    for (int d = 0; d < 3; d++) {
        double width = (n_here > 0 && hi[d] >= lo[d]) ? hi[d] - lo[d] : 0.0;
        if (!(width >= 1e-6)) {
            width = 1.0;
        }
        extent[d] = fmax(width * 1.01, 1.0);
        g.np_min[d] = (n_here > 0 && hi[d] >= lo[d]) ? lo[d] : 0.0;
        g.np_scale[d] = 1.0 / extent[d];
        g.periodic[d] = 0;
        g.prune_slack[d] = 0.0;
    }
    for (int k = 0; k < 6; k++) {
        g.prune_edges[k] = 0.0;
    }
    g.prune = 0;
    g.prune_limit = padded * padded;
    g.cutoff2 = cutoff * cutoff;
    g.n_points = n_here;
    bool one_cell = single_cell > 0;
    for (int attempt = 0; attempt < 2; attempt++) {
        double cells[3];
        for (int d = 0; d < 3; d++) {
            cells[d] = one_cell ? 1.0 : fmin(fmax(floor(extent[d] / padded), 1.0), 1048576.0);
        }
        // (the host sized the buffers of the batch for `most` cells per system)
        const double most = fmin(fmax(2.0 * static_cast<double>(n_here), 64.0), 16777216.0);
        limit_cells(cells, most);
        if (!(cells[0] * cells[1] * cells[2] <= most)) {
            cells[0] = cells[1] = cells[2] = 1.0; // never more cells than there is room for
        }
        uint32_t n_cells = 1;
        for (int d = 0; d < 3; d++) {
            g.n[d] = static_cast<int32_t>(cells[d]);
            n_cells *= static_cast<uint32_t>(g.n[d]);
            // nothing exists beyond the last cell of a direction that is not periodic
            const double radius = fmin(fmax(ceil(padded * cells[d] / extent[d]), 1.0), cells[d] - 1.0);
            g.s[d] = static_cast<int32_t>(radius);
        }
        g.n_cells = n_cells;
        if (single_cell == 0 && !one_cell && (n_cells == 1 || n_here < few_points)) {
            one_cell = true; // too little for a cell list: one cell, every point against every other
            continue;
        }
        break;
    }
    grids[system] = g;
    cells_of_system[system] = g.n_cells;
}

/// First cell of every system of a batch (exclusive scan of the cells per system, one workgroup), and what the
/// host wants to know at the end of the call: all cells and the most cells of one system.
__global__ __launch_bounds__(1024) void open_bases_kernel(
    const uint32_t* __restrict__ cells_of_system, uint32_t n_systems, uint32_t* __restrict__ cell_base,
    unsigned long long* __restrict__ total_cells
) {
    __shared__ uint64_t wave_sums[16];
    const int lane = lane_id();
    const int wave = threadIdx.x / WAVE;
    uint64_t carried = 0;
    for (uint32_t chunk = 0; chunk < n_systems; chunk += 1024) {
        const uint32_t system = chunk + threadIdx.x;
        const uint64_t own = system < n_systems ? cells_of_system[system] : 0;
        const uint64_t inclusive = wave_inclusive_scan(own);
        if (lane == WAVE - 1) {
            wave_sums[wave] = inclusive;
        }
        __syncthreads();
        uint64_t before = 0;
        uint64_t all = 0;
        for (int w = 0; w < 16; w++) {
            before += w < wave ? wave_sums[w] : 0;
            all += wave_sums[w];
        }
        __syncthreads();
        if (system < n_systems) {
            cell_base[system] = static_cast<uint32_t>(carried + before + inclusive - own);
        }
        carried += all;
    }
    if (threadIdx.x == 0) {
        cell_base[n_systems] = static_cast<uint32_t>(carried);
        *total_cells = carried;
    }
}

/// assign_cells for many systems at once: every point looks up its system (binary search in `first_point`), uses
/// that system's grid, and counts itself in the system's range of cells. Lanes of a wave in the same cell share one
/// atomic, like in assign_cells: small systems put a whole wave into one cell.
__global__ __launch_bounds__(BLOCK) void assign_cells_batch(
    const double* __restrict__ points, uint32_t n_points, const GridParams* __restrict__ grids,
    const uint32_t* __restrict__ first_point, const uint32_t* __restrict__ cell_base, uint32_t n_systems,
    uint32_t* __restrict__ cell_of, uint32_t* __restrict__ slot_of, int32_t* __restrict__ wrap_of,
    uint32_t* __restrict__ system_of, uint32_t* __restrict__ cell_counts, DeviceStatus* status
) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    const bool active = i < n_points;
    const int lane = lane_id();

    uint32_t system = 0;
    uint32_t linear = 0;
    int32_t wrap[3] = {0, 0, 0};
    if (active) {
        // largest s with first_point[s] <= i
        uint32_t lo = 0;
        uint32_t hi = n_systems;
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (first_point[mid] <= i) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        system = lo;
        const GridParams& g = grids[system];

        const double x = points[3 * static_cast<size_t>(i) + 0];
        const double y = points[3 * static_cast<size_t>(i) + 1];
        const double z = points[3 * static_cast<size_t>(i) + 2];
        int32_t cell[3] = {0, 0, 0};
        unsigned int axis;
        if (all_finite(x, y, z, axis)) {
            locate(g, x, y, z, cell, wrap);
        } else {
            atomicMin(&status->first_bad_coordinate, 3u * i + axis);
        }
        linear = cell_base[system] + (static_cast<uint32_t>(cell[2]) * g.n[1] + cell[1]) * g.n[0] + cell[0];
    }

    uint64_t group = 1ull << lane; // lanes left over after the rounds stand alone
    bool pending = active;
    for (int round = 0; round < ASSIGN_ROUNDS; round++) {
        const uint64_t remaining = __ballot(pending);
        if (remaining == 0) {
            break;
        }
        const int leader = __ffsll(static_cast<unsigned long long>(remaining)) - 1;
        const uint32_t leader_cell = read_lane(linear, leader);
        const bool same = pending && linear == leader_cell;
        const uint64_t members = __ballot(same);
        if (same) {
            group = members;
            pending = false;
        }
    }

    const int first = __ffsll(static_cast<unsigned long long>(group)) - 1;
    uint32_t base = 0;
    if (active && lane == first) {
        base = atomicAdd(&cell_counts[linear], static_cast<uint32_t>(__popcll(group)));
    }
    base = static_cast<uint32_t>(__shfl(static_cast<int>(base), first));
    if (active) {
        cell_of[i] = linear;
        slot_of[i] = base + rank_in_mask(group);
        system_of[i] = system;
        wrap_of[3 * static_cast<size_t>(i) + 0] = wrap[0];
        wrap_of[3 * static_cast<size_t>(i) + 1] = wrap[1];
        wrap_of[3 * static_cast<size_t>(i) + 2] = wrap[2];
    }
}

constexpr uint32_t CANONICAL_LIMIT = 4096;

/// One thread per slot of the counting sort. The atomics of assign_cells leave the points of a cell in arbitrary
/// order; here every point is ranked by original index among the points of its cell (so the whole pipeline is
/// deterministic), gathered into the cell-sorted records, and the first point of every run of 32 appends
/// the tile to the tile list. Work is proportional to the number of points, whatever the number of empty cells.
/// `tiles[].wrapped` must be zero on entry: points moved by a box vector set it with an atomic.
__global__ __launch_bounds__(BLOCK) void gather_points(
    const double* __restrict__ points, const int32_t* __restrict__ wrap_of, const uint32_t* __restrict__ cell_of,
    const uint32_t* __restrict__ provisional, const uint64_t* __restrict__ cell_scan, uint32_t n_points,
    SortedPoints sorted, Tile* __restrict__ tiles
) {
    const uint32_t p = blockIdx.x * BLOCK + threadIdx.x;
    if (p >= n_points) {
        return;
    }
    const uint32_t mine = provisional[p];
    const uint32_t cell = cell_of[mine];
    const uint64_t here = cell_scan[cell];
    const uint32_t start = static_cast<uint32_t>(here);
    const uint32_t count = static_cast<uint32_t>(cell_scan[cell + 1]) - start;
    const uint32_t first_tile = static_cast<uint32_t>(here >> 32);

    uint32_t rank = p - start;
    if (count <= CANONICAL_LIMIT) {
        rank = 0;
        // neighbouring lanes share the cell, so these loads hit the same few cache lines
        for (uint32_t other = 0; other < count; other++) {
            rank += provisional[start + other] < mine ? 1u : 0u;
        }
    }

    const uint32_t to = start + rank;
    const int32_t wx = wrap_of[3 * static_cast<size_t>(mine) + 0];
    const int32_t wy = wrap_of[3 * static_cast<size_t>(mine) + 1];
    const int32_t wz = wrap_of[3 * static_cast<size_t>(mine) + 2];
    sorted.p[to] = SortedPoint{
        points[3 * static_cast<size_t>(mine) + 0], points[3 * static_cast<size_t>(mine) + 1],
        points[3 * static_cast<size_t>(mine) + 2], mine, 0u
    };
    sorted.wx[to] = wx;
    sorted.wy[to] = wy;
    sorted.wz[to] = wz;
    if ((wx | wy | wz) != 0) {
        // tiles holding a wrapped point take the search kernel's general path
        atomicOr(&tiles[first_tile + rank / tile_size_of(count)].wrapped, 1u);
    }

    const uint32_t k = p - start;
    const uint32_t tile_size = tile_size_of(count);
    if (k % tile_size == 0) {
        Tile* tile = &tiles[first_tile + k / tile_size];
        tile->cell = cell;
        tile->first = start + k;
        tile->count = min(tile_size, count - k);
    }
}

/// The whole cell build of a small system in one launch of one workgroup, so that a call is three launches instead
/// of seven: clears the work state (`clear`, whole 16-byte blocks), fetches the box when `box` is not null, then
/// histogram (LDS atomics), scan of points and tiles per cell, and placement into the packed layout with its tile
/// list - what clear_and_fetch, assign_cells, the scan and place_points do for systems of any size. The slot of a
/// point inside its cell is the one the atomic handed out, as with place_points.
constexpr uint32_t SMALL_BUILD_THREADS = 1024;
constexpr uint32_t SMALL_BUILD_POINTS = 2 * SMALL_BUILD_THREADS; // points and cells one workgroup takes (beyond
                                                                 // about 2500 points the four launches win)
constexpr uint32_t SMALL_BUILD_PER_THREAD = SMALL_BUILD_POINTS / SMALL_BUILD_THREADS;

__global__ __launch_bounds__(SMALL_BUILD_THREADS) void build_cells_small(
    const double* __restrict__ points, GridParams g, uint4* __restrict__ clear, size_t clear_blocks16,
    const double* __restrict__ box, const bool* __restrict__ periodic, unsigned char* host_small,
    SortedPoints sorted, Tile* __restrict__ tiles, uint64_t* __restrict__ cell_scan, DeviceStatus* status
) {
    __shared__ uint32_t cell_count[SMALL_BUILD_POINTS];
    __shared__ uint64_t cell_first[SMALL_BUILD_POINTS]; // points before the cell | tiles before it << 32
    __shared__ uint64_t wave_totals[SMALL_BUILD_THREADS / WAVE];
    const uint32_t t = threadIdx.x;
    const int lane = lane_id();
    const uint32_t wave = t / WAVE;

    if (box != nullptr) {
        if (t < 9) {
            reinterpret_cast<double*>(host_small)[t] = box[t];
        } else if (t < 12) {
            host_small[72 + (t - 9)] = periodic[t - 9] ? 1 : 0;
        } else if (t == 12) {
            status->total_pairs = 0;
            status->first_bad_coordinate = 0xFFFFFFFFu;
            status->crowded_cells = 0;
            status->far_outside = 0;
        }
    }
    const uint4 zero = {0u, 0u, 0u, 0u};
    for (size_t k = t; k < clear_blocks16; k += SMALL_BUILD_THREADS) {
        clear[k] = zero;
    }
    for (uint32_t c = t; c < g.n_cells; c += SMALL_BUILD_THREADS) {
        cell_count[c] = 0;
    }
    __syncthreads();

    // ---- histogram: the slot inside the cell comes back from the LDS atomic
    double x[SMALL_BUILD_PER_THREAD], y[SMALL_BUILD_PER_THREAD], z[SMALL_BUILD_PER_THREAD];
    uint32_t cell_of[SMALL_BUILD_PER_THREAD], slot_of[SMALL_BUILD_PER_THREAD];
    int32_t wx[SMALL_BUILD_PER_THREAD], wy[SMALL_BUILD_PER_THREAD], wz[SMALL_BUILD_PER_THREAD];
#pragma unroll
    for (uint32_t k = 0; k < SMALL_BUILD_PER_THREAD; k++) {
        const uint32_t i = k * SMALL_BUILD_THREADS + t;
        cell_of[k] = 0;
        slot_of[k] = 0;
        wx[k] = wy[k] = wz[k] = 0;
        x[k] = y[k] = z[k] = 0.0;
        if (i < g.n_points) {
            x[k] = points[3 * static_cast<size_t>(i) + 0];
            y[k] = points[3 * static_cast<size_t>(i) + 1];
            z[k] = points[3 * static_cast<size_t>(i) + 2];
            int32_t where[3] = {0, 0, 0};
            int32_t wrap[3] = {0, 0, 0};
            unsigned int axis;
            if (all_finite(x[k], y[k], z[k], axis)) {
                locate(g, x[k], y[k], z[k], where, wrap);
            } else {
                atomicMin(&status->first_bad_coordinate, 3u * i + axis);
            }
            cell_of[k] = (static_cast<uint32_t>(where[2]) * g.n[1] + where[1]) * g.n[0] + where[0];
            wx[k] = wrap[0];
            wy[k] = wrap[1];
            wz[k] = wrap[2];
            slot_of[k] = atomicAdd(&cell_count[cell_of[k]], 1u);
        }
    }
    __syncthreads();

    // ---- exclusive scan over the cells of (points, tiles), both in one 64-bit word
    uint64_t mine[SMALL_BUILD_PER_THREAD];
    uint64_t own_total = 0;
#pragma unroll
    for (uint32_t k = 0; k < SMALL_BUILD_PER_THREAD; k++) {
        const uint32_t c = t * SMALL_BUILD_PER_THREAD + k;
        const uint32_t count = c < g.n_cells ? cell_count[c] : 0;
        const uint64_t n_tiles = (count + TILE_POINTS - 1) / TILE_POINTS;
        mine[k] = own_total;
        own_total += static_cast<uint64_t>(count) | (n_tiles << 32);
    }
    const uint64_t inclusive = wave_inclusive_scan(own_total);
    if (lane == WAVE - 1) {
        wave_totals[wave] = inclusive;
    }
    __syncthreads();
    uint64_t before = inclusive - own_total;
    for (uint32_t w = 0; w < wave; w++) {
        before += wave_totals[w];
    }
#pragma unroll
    for (uint32_t k = 0; k < SMALL_BUILD_PER_THREAD; k++) {
        const uint32_t c = t * SMALL_BUILD_PER_THREAD + k;
        if (c < g.n_cells) {
            cell_first[c] = before + mine[k];
            cell_scan[c] = before + mine[k];
        }
    }
    if (t == SMALL_BUILD_THREADS - 1) {
        cell_scan[g.n_cells] = before + own_total;
    }
    __syncthreads();

    // ---- placement and tile list
#pragma unroll
    for (uint32_t k = 0; k < SMALL_BUILD_PER_THREAD; k++) {
        const uint32_t i = k * SMALL_BUILD_THREADS + t;
        if (i < g.n_points) {
            const uint64_t here = cell_first[cell_of[k]];
            const uint32_t start = static_cast<uint32_t>(here);
            const uint32_t first_tile = static_cast<uint32_t>(here >> 32);
            const uint32_t count = cell_count[cell_of[k]];
            const uint32_t to = start + slot_of[k];
            sorted.p[to] = SortedPoint{x[k], y[k], z[k], i, 0u};
            sorted.wx[to] = wx[k];
            sorted.wy[to] = wy[k];
            sorted.wz[to] = wz[k];
            const uint32_t tile_size = tile_size_of(count);
            Tile* tile = &tiles[first_tile + slot_of[k] / tile_size];
            if ((wx[k] | wy[k] | wz[k]) != 0) {
                atomicOr(&tile->wrapped, 1u);
            }
            if (slot_of[k] % tile_size == 0) {
                tile->cell = cell_of[k];
                tile->first = to;
                tile->count = min(tile_size, count - slot_of[k]);
            }
        }
    }
}

/// The single-cell layout used by the brute-force / multi-image path: points keep their order, the one cell
/// holds all of them, tiles are consecutive blocks of 32 points. Also performs the non-finite check.
/// When `clear` is given (launches of a single workgroup only), it also clears that part of the work state (the
/// state of the search kernels: the tile list is written here in full and needs no clearing), fetches the box and
/// resets the status like fetch_box does: a call on this layout then starts with one launch instead of two.
__global__ __launch_bounds__(BLOCK) void prepare_single_cell(
    const double* __restrict__ points, GridParams g, SortedPoints sorted, Tile* __restrict__ tiles,
    uint64_t* __restrict__ cell_scan, DeviceStatus* status, uint4* __restrict__ clear = nullptr,
    size_t clear_blocks16 = 0, const double* __restrict__ box = nullptr, const bool* __restrict__ periodic = nullptr,
    unsigned char* host_small = nullptr, Prefilter pre = Prefilter()
) {
    if (blockIdx.x == 0) {
        const int t = threadIdx.x;
        if (box != nullptr) {
            if (t < 9) {
                reinterpret_cast<double*>(host_small)[t] = box[t];
            } else if (t < 12) {
                host_small[72 + (t - 9)] = periodic[t - 9] ? 1 : 0;
            } else if (t == 12) {
                status->total_pairs = 0;
                status->first_bad_coordinate = 0xFFFFFFFFu;
                status->crowded_cells = 0;
                status->far_outside = 0;
            }
        }
        const uint4 zero = {0u, 0u, 0u, 0u};
        for (size_t k = t; k < clear_blocks16; k += BLOCK) {
            clear[k] = zero;
        }
        if (clear != nullptr) {
            __syncthreads(); // the status is reset before any thread reports into it: one workgroup only
        }
    }
    uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    const uint32_t n_tiles = (g.n_points + TILE_POINTS - 1) / TILE_POINTS;
    if (i == 0) {
        cell_scan[0] = 0;
        cell_scan[1] = static_cast<uint64_t>(g.n_points) | (static_cast<uint64_t>(n_tiles) << 32);
    }
    bool wrapped = false;
    if (i < g.n_points) {
        const double x = points[3 * static_cast<size_t>(i) + 0];
        const double y = points[3 * static_cast<size_t>(i) + 1];
        const double z = points[3 * static_cast<size_t>(i) + 2];
        int32_t cell[3] = {0, 0, 0};
        int32_t wrap[3] = {0, 0, 0};
        double inside[3] = {0.0, 0.0, 0.0};
        unsigned int axis;
        if (all_finite(x, y, z, axis)) {
            locate(g, x, y, z, cell, wrap, nullptr, inside);
        } else {
            atomicMin(&status->first_bad_coordinate, 3u * i + axis);
        }
        wrapped = (wrap[0] | wrap[1] | wrap[2]) != 0;
        sorted.p[i] = SortedPoint{x, y, z, i, 0u};
        if (sorted.l != nullptr) {
            sorted.l[i] = local_record(pre, inside, wrap);
        }
        sorted.wx[i] = wrap[0];
        sorted.wy[i] = wrap[1];
        sorted.wz[i] = wrap[2];
    }
    // a wave covers WAVE / TILE_POINTS whole tiles of consecutive points
    const uint64_t wrapped_lanes = __ballot(wrapped);
    const uint32_t tile_id = i / TILE_POINTS;
    const uint32_t first_lane = (lane_id() / TILE_POINTS) * TILE_POINTS;
    const uint64_t tile_lanes = ((TILE_POINTS == WAVE ? 0ull : (1ull << TILE_POINTS)) - 1ull) << first_lane;
    if (lane_id() % TILE_POINTS == 0 && tile_id < n_tiles) {
        Tile tile;
        tile.cell = 0;
        tile.first = tile_id * TILE_POINTS;
        tile.count = min(TILE_POINTS, g.n_points - tile_id * TILE_POINTS);
        tile.wrapped = (wrapped_lanes & tile_lanes) != 0 ? 1u : 0u;
        tiles[tile_id] = tile;
    }
}

} // namespace vesin_hip

#endif
