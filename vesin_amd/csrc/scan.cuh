// Device-wide exclusive prefix sum (u64 accumulators) built from wave64 DPP scans and LDS.
//
// Reduce-then-scan over tiles of SCAN_TILE elements: one kernel sums each tile, the tile sums are scanned
// recursively, and a last kernel rescans each tile with its offset added. Output has n + 1 entries: out[n] is the
// grand total. No atomics, deterministic.
#ifndef VESIN_HIP_SCAN_CUH
#define VESIN_HIP_SCAN_CUH

#include "device_common.cuh"

namespace vesin_hip {

constexpr int SCAN_ITEMS = 8;
constexpr int SCAN_TILE = BLOCK * SCAN_ITEMS; // 2048 elements per workgroup

/// What the scan reads.
enum ScanInput {
    SCAN_U32 = 0,        // plain 32-bit counts
    SCAN_CELL_COUNTS = 1,// 32-bit points-per-cell; scanned value = count | (number of tiles << 32)
    SCAN_U64 = 2,        // 64-bit values (tile sums of a previous level)
};

template <int INPUT>
__device__ __forceinline__ uint64_t scan_load(const void* in, size_t i) {
    if (INPUT == SCAN_U64) {
        return static_cast<const uint64_t*>(in)[i];
    }
    uint32_t v = static_cast<const uint32_t*>(in)[i];
    if (INPUT == SCAN_CELL_COUNTS) {
        return static_cast<uint64_t>(v) | (static_cast<uint64_t>((v + TILE_POINTS - 1) >> TILE_SHIFT) << 32);
    }
    return v;
}

/// Exclusive scan of one value per thread across the workgroup; returns the exclusive prefix and the total.
__device__ __forceinline__ uint64_t block_exclusive_scan(uint64_t value, uint64_t& total, uint64_t* wave_sums) {
    const int lane = lane_id();
    const int wave = threadIdx.x / WAVE;
    uint64_t inclusive = wave_inclusive_scan(value);
    if (lane == WAVE - 1) {
        wave_sums[wave] = inclusive;
    }
    __syncthreads();
    uint64_t before = 0;
    uint64_t all = 0;
#pragma unroll
    for (int w = 0; w < WAVES_PER_BLOCK; w++) {
        uint64_t s = wave_sums[w];
        before += (w < wave) ? s : 0;
        all += s;
    }
    __syncthreads();
    total = all;
    return before + inclusive - value;
}

template <int INPUT>
__global__ __launch_bounds__(BLOCK) void scan_tile_sums(const void* __restrict__ in, size_t n, uint64_t* __restrict__ sums) {
    __shared__ uint64_t wave_sums[WAVES_PER_BLOCK];
    size_t base = static_cast<size_t>(blockIdx.x) * SCAN_TILE + static_cast<size_t>(threadIdx.x) * SCAN_ITEMS;
    uint64_t local = 0;
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + k;
        local += i < n ? scan_load<INPUT>(in, i) : 0;
    }
    uint64_t total;
    block_exclusive_scan(local, total, wave_sums);
    if (threadIdx.x == 0) {
        sums[blockIdx.x] = total;
    }
}

/// `offsets` may be null when there is a single tile. Writes out[0..n) and, from the last tile, out[n].
template <int INPUT>
__global__ __launch_bounds__(BLOCK) void scan_tile_write(
    const void* __restrict__ in, size_t n, const uint64_t* __restrict__ offsets, uint64_t* __restrict__ out
) {
    __shared__ uint64_t wave_sums[WAVES_PER_BLOCK];
    size_t base = static_cast<size_t>(blockIdx.x) * SCAN_TILE + static_cast<size_t>(threadIdx.x) * SCAN_ITEMS;
    uint64_t items[SCAN_ITEMS];
    uint64_t local = 0;
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + k;
        items[k] = i < n ? scan_load<INPUT>(in, i) : 0;
        local += items[k];
    }
    uint64_t total;
    uint64_t running = block_exclusive_scan(local, total, wave_sums);
    running += offsets != nullptr ? offsets[blockIdx.x] : 0;
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + k;
        if (i < n) {
            out[i] = running;
        }
        running += items[k];
        if (i + 1 == n) {
            out[n] = running;
        }
    }
    if (n == 0 && blockIdx.x == 0 && threadIdx.x == 0) {
        out[0] = 0;
    }
}

/// scan_tile_write for inputs of at most BLOCK tiles: instead of reading its offset from a scanned array of tile
/// sums, every workgroup adds up the sums of the tiles before its own (one per thread). Saves the launch of the
/// middle level.
template <int INPUT>
__global__ __launch_bounds__(BLOCK) void scan_tile_write_few(
    const void* __restrict__ in, size_t n, const uint64_t* __restrict__ sums, uint64_t* __restrict__ out
) {
    __shared__ uint64_t wave_sums[WAVES_PER_BLOCK];
    uint64_t before = threadIdx.x < blockIdx.x ? sums[threadIdx.x] : 0;
    uint64_t offset;
    block_exclusive_scan(before, offset, wave_sums);

    size_t base = static_cast<size_t>(blockIdx.x) * SCAN_TILE + static_cast<size_t>(threadIdx.x) * SCAN_ITEMS;
    uint64_t items[SCAN_ITEMS];
    uint64_t local = 0;
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + k;
        items[k] = i < n ? scan_load<INPUT>(in, i) : 0;
        local += items[k];
    }
    uint64_t total;
    uint64_t running = block_exclusive_scan(local, total, wave_sums) + offset;
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + k;
        if (i < n) {
            out[i] = running;
        }
        running += items[k];
        if (i + 1 == n) {
            out[n] = running;
        }
    }
}

/// The whole scan of a short input in one workgroup of 1024 threads, SCAN_ONE_CHUNK elements at a time: one launch
/// where the tiles of the general scheme take two (a launch and the gap before it cost about as much as the
/// workgroup needs for all of it).
constexpr int SCAN_ONE_THREADS = 1024;
constexpr size_t SCAN_ONE_CHUNK = static_cast<size_t>(SCAN_ONE_THREADS) * SCAN_ITEMS;
constexpr size_t SCAN_ONE_MAX = 2 * SCAN_ONE_CHUNK;

template <int INPUT>
__global__ __launch_bounds__(SCAN_ONE_THREADS) void scan_one_workgroup(
    const void* __restrict__ in, size_t n, uint64_t* __restrict__ out
) {
    constexpr int WAVES = SCAN_ONE_THREADS / WAVE;
    __shared__ uint64_t wave_sums[WAVES];
    const int lane = lane_id();
    const int wave = threadIdx.x / WAVE;
    uint64_t carried = 0;
    for (size_t chunk = 0; chunk < n; chunk += SCAN_ONE_CHUNK) {
        const size_t base = chunk + static_cast<size_t>(threadIdx.x) * SCAN_ITEMS;
        uint64_t items[SCAN_ITEMS];
        uint64_t local = 0;
#pragma unroll
        for (int k = 0; k < SCAN_ITEMS; k++) {
            const size_t i = base + k;
            items[k] = i < n ? scan_load<INPUT>(in, i) : 0;
            local += items[k];
        }
        const uint64_t inclusive = wave_inclusive_scan(local);
        if (lane == WAVE - 1) {
            wave_sums[wave] = inclusive;
        }
        __syncthreads();
        uint64_t before = 0;
        uint64_t all = 0;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            const uint64_t sum = wave_sums[w];
            before += w < wave ? sum : 0;
            all += sum;
        }
        __syncthreads();
        uint64_t running = carried + before + inclusive - local;
#pragma unroll
        for (int k = 0; k < SCAN_ITEMS; k++) {
            const size_t i = base + k;
            if (i < n) {
                out[i] = running;
            }
            running += items[k];
            if (i + 1 == n) {
                out[n] = running;
            }
        }
        carried += all;
    }
    if (n == 0 && threadIdx.x == 0) {
        out[0] = 0;
    }
}

inline size_t scan_tiles(size_t n) {
    return n == 0 ? 1 : (n + SCAN_TILE - 1) / SCAN_TILE;
}

/// Scratch (in u64 elements) needed by exclusive_scan for n inputs: tile sums and their scans for every level.
inline size_t scan_scratch_elements(size_t n) {
    size_t total = 0;
    size_t tiles = scan_tiles(n);
    while (tiles > 1) {
        total += 2 * (tiles + 1);
        tiles = scan_tiles(tiles);
    }
    return total + 2;
}

/// out[i] = sum of in[0..i), out[n] = total. `scratch` holds scan_scratch_elements(n) u64.
template <int INPUT>
inline void exclusive_scan(const void* in, size_t n, uint64_t* out, uint64_t* scratch, hipStream_t stream) {
    size_t tiles = scan_tiles(n);
    if (tiles == 1) {
        hipLaunchKernelGGL(scan_tile_write<INPUT>, dim3(1), dim3(BLOCK), 0, stream, in, n, nullptr, out);
        return;
    }
    if (n <= SCAN_ONE_MAX) {
        hipLaunchKernelGGL(scan_one_workgroup<INPUT>, dim3(1), dim3(SCAN_ONE_THREADS), 0, stream, in, n, out);
        return;
    }
    uint64_t* sums = scratch;
    uint64_t* offsets = scratch + (tiles + 1);
    hipLaunchKernelGGL(scan_tile_sums<INPUT>, dim3(tiles), dim3(BLOCK), 0, stream, in, n, sums);
    if (tiles <= BLOCK) {
        hipLaunchKernelGGL(scan_tile_write_few<INPUT>, dim3(tiles), dim3(BLOCK), 0, stream, in, n, sums, out);
        return;
    }
    exclusive_scan<SCAN_U64>(sums, tiles, offsets, scratch + 2 * (tiles + 1), stream);
    hipLaunchKernelGGL(scan_tile_write<INPUT>, dim3(tiles), dim3(BLOCK), 0, stream, in, n, offsets, out);
}

} // namespace vesin_hip

#endif
