// `sorted = true`: least-significant-digit radix sort of the pairs by (i, j, Sx, Sy, Sz).
//
// The reference sorts by i only and leaves the order inside one i unspecified (vesin/include/vesin.h:55-57; CPU:
// vesin/src/cpu_cell_list.cpp:634-730, an unstable std::sort; GPU: vesin/src/cuda/sort_pairs.cu, a bitonic network on i). This
// library emits the full lexicographic order, which is one of the orders that contract allows and the only one
// that is reproducible.
//
// The key packs the five fields into as few bits as the data needs (i and j take ceil(log2(n_points)) bits each,
// every shift component takes the bits of its observed range), so the number of 8-bit passes adapts to the
// system. (key, row) pairs are sorted; the 16-60 byte payload rows are moved once, at the end, by one gather.
// Each pass is histogram -> device-wide scan -> stable scatter; ranks inside a wave come from ballot matching,
// not from atomics, so the sort is stable and deterministic.
#ifndef VESIN_HIP_SORT_CUH
#define VESIN_HIP_SORT_CUH

#include "device_common.cuh"
#include "scan.cuh"
#include "search.cuh"

#include <algorithm>
#include <stdexcept>
#include <string>

namespace vesin_hip {

constexpr int RADIX_BITS = 8;
constexpr int RADIX = 1 << RADIX_BITS;
constexpr int SORT_ITEMS = 8;
constexpr int SORT_TILE = BLOCK * SORT_ITEMS;
constexpr int SORT_STEPS = SORT_ITEMS * WAVES_PER_BLOCK;

/// Smallest and largest value of each shift component.
struct ShiftRange {
    int lo[3];
    int hi[3];
};

/// Where each field sits in the 64-bit key. A field with zero bits is left out.
struct KeyLayout {
    int32_t shift_lo[3];
    uint32_t bits_shift[3];
    uint32_t bits_index; // for i and for j
    uint32_t use_i;
    uint32_t use_j_and_shift;
};

constexpr int SHIFT_RANGE_BLOCKS = 256;

/// Range of the shifts of all rows: grid-stride loop, wave then workgroup reduction; every workgroup reports to its
/// own slot of `host_ranges` (pinned host memory, folded by the host), so no atomics are involved.
__global__ __launch_bounds__(BLOCK) void shift_range_kernel(
    const int32_t* __restrict__ shifts, size_t n, ShiftRange* host_ranges
) {
    __shared__ ShiftRange partial[WAVES_PER_BLOCK];
    int lo[3] = {0x7fffffff, 0x7fffffff, 0x7fffffff};
    int hi[3] = {-0x7fffffff - 1, -0x7fffffff - 1, -0x7fffffff - 1};
    for (size_t k = static_cast<size_t>(blockIdx.x) * BLOCK + threadIdx.x; k < n; k += static_cast<size_t>(gridDim.x) * BLOCK) {
#pragma unroll
        for (int d = 0; d < 3; d++) {
            int s = shifts[3 * k + d];
            lo[d] = min(lo[d], s);
            hi[d] = max(hi[d], s);
        }
    }
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
#pragma unroll
        for (int d = 0; d < 3; d++) {
            lo[d] = min(lo[d], __shfl_xor(lo[d], offset));
            hi[d] = max(hi[d], __shfl_xor(hi[d], offset));
        }
    }
    if (lane_id() == 0) {
#pragma unroll
        for (int d = 0; d < 3; d++) {
            partial[threadIdx.x / WAVE].lo[d] = lo[d];
            partial[threadIdx.x / WAVE].hi[d] = hi[d];
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        ShiftRange all = partial[0];
        for (int w = 1; w < WAVES_PER_BLOCK; w++) {
#pragma unroll
            for (int d = 0; d < 3; d++) {
                all.lo[d] = min(all.lo[d], partial[w].lo[d]);
                all.hi[d] = max(all.hi[d], partial[w].hi[d]);
            }
        }
        host_ranges[blockIdx.x] = all;
    }
}

/// The rows of many systems, system after system, whose indices count inside each system: the first index of a
/// row is sorted as if it counted over all points of the batch (first point of the row's system + index), which
/// keeps every system's rows where they are and orders them inside.
struct BatchRows {
    const unsigned long long* first_pair; // [n_systems + 1]: first row of every system
    const uint32_t* first_point;          // [n_systems + 1]: first point of every system
    uint32_t n_systems;                   // 0: the rows are those of one system
};

/// keys[k] = packed fields of row perm[k] (or row k when perm is null); rows[k] = that row number.
__global__ __launch_bounds__(BLOCK) void build_keys_kernel(
    const unsigned long long* __restrict__ pairs, const int32_t* __restrict__ shifts,
    const uint32_t* __restrict__ perm, size_t n, KeyLayout layout, BatchRows batch,
    uint64_t* __restrict__ keys, uint32_t* __restrict__ rows
) {
    size_t k = static_cast<size_t>(blockIdx.x) * BLOCK + threadIdx.x;
    if (k >= n) {
        return;
    }
    size_t row = perm != nullptr ? perm[k] : k;
    uint64_t key = 0;
    if (layout.use_i) {
        key = pairs[2 * row];
        if (batch.n_systems != 0) {
            // the system whose rows include this one: the last with first_pair <= row
            uint32_t lo = 0;
            uint32_t hi = batch.n_systems;
            while (hi - lo > 1) {
                const uint32_t mid = (lo + hi) >> 1;
                if (batch.first_pair[mid] <= row) {
                    lo = mid;
                } else {
                    hi = mid;
                }
            }
            key += batch.first_point[lo];
        }
    }
    if (layout.use_j_and_shift) {
        key = (key << layout.bits_index) | pairs[2 * row + 1];
#pragma unroll
        for (int d = 0; d < 3; d++) {
            uint64_t field = static_cast<uint32_t>(shifts[3 * row + d] - layout.shift_lo[d]);
            key = (key << layout.bits_shift[d]) | field;
        }
    }
    keys[k] = key;
    rows[k] = static_cast<uint32_t>(row);
}

/// Lanes of the wave holding the same digit as this lane (valid lanes only).
__device__ __forceinline__ uint64_t match_digit(uint32_t digit, bool valid) {
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < RADIX_BITS; bit++) {
        const bool set = (digit >> bit) & 1;
        const uint64_t vote = __ballot(set);
        peers &= set ? vote : ~vote;
    }
    return peers;
}

/// table[digit * n_blocks + block] = number of keys of this block's tile with that digit.
__global__ __launch_bounds__(BLOCK) void radix_histogram_kernel(
    const uint64_t* __restrict__ keys, size_t n, uint32_t bit, uint32_t* __restrict__ table, uint32_t n_blocks
) {
    __shared__ uint32_t histogram[RADIX];
    histogram[threadIdx.x] = 0;
    __syncthreads();
    const size_t base = static_cast<size_t>(blockIdx.x) * SORT_TILE;
#pragma unroll
    for (int item = 0; item < SORT_ITEMS; item++) {
        size_t k = base + static_cast<size_t>(item) * BLOCK + threadIdx.x;
        if (k < n) {
            atomicAdd(&histogram[(keys[k] >> bit) & (RADIX - 1)], 1u);
        }
    }
    __syncthreads();
    table[static_cast<size_t>(threadIdx.x) * n_blocks + blockIdx.x] = histogram[threadIdx.x];
}

/// Stable scatter of one tile. `offsets` is the exclusive scan of `table`.
__global__ __launch_bounds__(BLOCK) void radix_scatter_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ rows_in,
    uint64_t* __restrict__ keys_out, uint32_t* __restrict__ rows_out,
    size_t n, uint32_t bit, const uint64_t* __restrict__ offsets, uint32_t n_blocks
) {
    // per (step, digit) counts, turned into "keys with this digit in earlier steps of the tile"
    __shared__ uint32_t counts[SORT_STEPS][RADIX];
    const int lane = lane_id();
    const int wave = threadIdx.x / WAVE;

    for (int s = 0; s < SORT_STEPS; s++) {
        counts[s][threadIdx.x] = 0;
    }
    __syncthreads();

    const size_t base = static_cast<size_t>(blockIdx.x) * SORT_TILE;
    uint64_t key[SORT_ITEMS];
    uint32_t row[SORT_ITEMS];
    uint32_t rank[SORT_ITEMS];
#pragma unroll
    for (int item = 0; item < SORT_ITEMS; item++) {
        const size_t k = base + static_cast<size_t>(item) * BLOCK + threadIdx.x;
        const bool valid = k < n;
        key[item] = valid ? keys_in[k] : 0;
        row[item] = valid ? rows_in[k] : 0;
        const uint32_t digit = (key[item] >> bit) & (RADIX - 1);
        const uint64_t peers = match_digit(digit, valid);
        rank[item] = rank_in_mask(peers);
        if (valid && rank[item] == 0) {
            counts[item * WAVES_PER_BLOCK + wave][digit] = __popcll(peers);
        }
    }
    __syncthreads();

    {
        // thread d turns column d into an exclusive prefix over the steps
        uint32_t running = 0;
        for (int s = 0; s < SORT_STEPS; s++) {
            uint32_t c = counts[s][threadIdx.x];
            counts[s][threadIdx.x] = running;
            running += c;
        }
    }
    __syncthreads();

#pragma unroll
    for (int item = 0; item < SORT_ITEMS; item++) {
        const size_t k = base + static_cast<size_t>(item) * BLOCK + threadIdx.x;
        if (k < n) {
            const uint32_t digit = (key[item] >> bit) & (RADIX - 1);
            const uint64_t to = offsets[static_cast<size_t>(digit) * n_blocks + blockIdx.x] +
                                counts[item * WAVES_PER_BLOCK + wave][digit] + rank[item];
            keys_out[to] = key[item];
            rows_out[to] = row[item];
        }
    }
    (void)lane;
}

/// Move the payload rows into their sorted places.
__global__ __launch_bounds__(BLOCK) void gather_rows_kernel(
    const uint32_t* __restrict__ rows, size_t n, SearchOutputs from, SearchOutputs to
) {
    size_t k = static_cast<size_t>(blockIdx.x) * BLOCK + threadIdx.x;
    if (k >= n) {
        return;
    }
    const size_t row = rows[k];
    reinterpret_cast<ulonglong2*>(to.pairs)[k] = reinterpret_cast<const ulonglong2*>(from.pairs)[row];
    if (to.shifts != nullptr) {
        to.shifts[3 * k + 0] = from.shifts[3 * row + 0];
        to.shifts[3 * k + 1] = from.shifts[3 * row + 1];
        to.shifts[3 * k + 2] = from.shifts[3 * row + 2];
    }
    if (to.distances != nullptr) {
        to.distances[k] = from.distances[row];
    }
    if (to.vectors != nullptr) {
        to.vectors[3 * k + 0] = from.vectors[3 * row + 0];
        to.vectors[3 * k + 1] = from.vectors[3 * row + 1];
        to.vectors[3 * k + 2] = from.vectors[3 * row + 2];
    }
}

inline uint32_t bits_for(uint64_t max_value) {
    uint32_t bits = 0;
    while (max_value != 0) {
        bits += 1;
        max_value >>= 1;
    }
    return bits;
}

/// Device memory the sort needs besides the unsorted payload, for n rows.
struct SortWorkspace {
    uint64_t* keys[2];
    uint32_t* rows[2];
    uint32_t* table;
    uint64_t* table_scan;
    uint64_t* scan_scratch;
    ShiftRange* host_ranges;   // SHIFT_RANGE_BLOCKS entries the host reads
    ShiftRange* device_ranges; // where the kernel writes them: the same pinned host memory, or device memory that
                               // is copied to `host_ranges` before the host looks
};

inline size_t sort_blocks(size_t n) {
    return (n + SORT_TILE - 1) / SORT_TILE;
}

/// Stable LSD radix sort of (keys[0], rows[0]) on bits [0, bits). Returns which of the two buffers holds the result.
inline int radix_sort(SortWorkspace& w, size_t n, uint32_t bits, hipStream_t stream) {
    const uint32_t n_blocks = static_cast<uint32_t>(sort_blocks(n));
    int current = 0;
    for (uint32_t bit = 0; bit < bits; bit += RADIX_BITS) {
        hipLaunchKernelGGL(
            radix_histogram_kernel, dim3(n_blocks), dim3(BLOCK), 0, stream, w.keys[current], n, bit, w.table, n_blocks
        );
        exclusive_scan<SCAN_U32>(w.table, static_cast<size_t>(RADIX) * n_blocks, w.table_scan, w.scan_scratch, stream);
        hipLaunchKernelGGL(
            radix_scatter_kernel, dim3(n_blocks), dim3(BLOCK), 0, stream,
            w.keys[current], w.rows[current], w.keys[1 - current], w.rows[1 - current], n, bit, w.table_scan, n_blocks
        );
        current = 1 - current;
    }
    return current;
}

/// Sort `n` unsorted payload rows (`from`, shifts always present) into `to`. `n_points` bounds both indices of a row
/// (with `batch`: the points of all systems together).
inline void sort_pairs(
    const SearchOutputs& from, const SearchOutputs& to, size_t n, size_t n_points, SortWorkspace& w, hipStream_t stream,
    BatchRows batch = BatchRows{nullptr, nullptr, 0}
) {
    if (n >= 0xFFFFFFFFull) {
        throw std::runtime_error("too many pairs to sort: the sort indexes rows with 32 bits");
    }
    const uint32_t n_key_blocks = static_cast<uint32_t>((n + BLOCK - 1) / BLOCK);

    const uint32_t range_blocks = n_key_blocks > SHIFT_RANGE_BLOCKS ? SHIFT_RANGE_BLOCKS : n_key_blocks;
    hipLaunchKernelGGL(shift_range_kernel, dim3(range_blocks), dim3(BLOCK), 0, stream, from.shifts, n, w.device_ranges);
    if (w.device_ranges != w.host_ranges &&
        hipMemcpyAsync(w.host_ranges, w.device_ranges, range_blocks * sizeof(ShiftRange), hipMemcpyDeviceToHost, stream) !=
            hipSuccess) {
        throw std::runtime_error("HIP error while reading the range of the shifts");
    }
    if (hipStreamSynchronize(stream) != hipSuccess) {
        throw std::runtime_error("HIP error while reading the range of the shifts");
    }
    ShiftRange range = w.host_ranges[0];
    for (uint32_t block = 1; block < range_blocks; block++) {
        for (int d = 0; d < 3; d++) {
            range.lo[d] = std::min(range.lo[d], w.host_ranges[block].lo[d]);
            range.hi[d] = std::max(range.hi[d], w.host_ranges[block].hi[d]);
        }
    }

    KeyLayout layout = {};
    layout.bits_index = bits_for(n_points > 0 ? n_points - 1 : 0);
    uint32_t low_bits = layout.bits_index;
    for (int d = 0; d < 3; d++) {
        layout.shift_lo[d] = range.lo[d];
        layout.bits_shift[d] = bits_for(static_cast<uint64_t>(static_cast<int64_t>(range.hi[d]) - range.lo[d]));
        low_bits += layout.bits_shift[d];
    }
    if (low_bits > 64) {
        throw std::runtime_error("the periodic shifts span too large a range to sort this neighbor list");
    }

    int result;
    if (low_bits + layout.bits_index <= 64) {
        layout.use_i = 1;
        layout.use_j_and_shift = 1;
        hipLaunchKernelGGL(
            build_keys_kernel, dim3(n_key_blocks), dim3(BLOCK), 0, stream,
            from.pairs, from.shifts, static_cast<const uint32_t*>(nullptr), n, layout, batch, w.keys[0], w.rows[0]
        );
        result = radix_sort(w, n, low_bits + layout.bits_index, stream);
    } else {
        // two chained stable sorts: by (j, shift), then by i
        layout.use_i = 0;
        layout.use_j_and_shift = 1;
        hipLaunchKernelGGL(
            build_keys_kernel, dim3(n_key_blocks), dim3(BLOCK), 0, stream,
            from.pairs, from.shifts, static_cast<const uint32_t*>(nullptr), n, layout, batch, w.keys[0], w.rows[0]
        );
        result = radix_sort(w, n, low_bits, stream);
        if (result != 0) {
            std::swap(w.keys[0], w.keys[1]);
            std::swap(w.rows[0], w.rows[1]);
        }
        layout.use_i = 1;
        layout.use_j_and_shift = 0;
        // keys are rebuilt from the rows in their current order; rows[1] is free to receive the copy
        hipLaunchKernelGGL(
            build_keys_kernel, dim3(n_key_blocks), dim3(BLOCK), 0, stream,
            from.pairs, from.shifts, static_cast<const uint32_t*>(w.rows[0]), n, layout, batch, w.keys[1], w.rows[1]
        );
        std::swap(w.keys[0], w.keys[1]);
        std::swap(w.rows[0], w.rows[1]);
        result = radix_sort(w, n, layout.bits_index, stream);
    }

    hipLaunchKernelGGL(gather_rows_kernel, dim3(n_key_blocks), dim3(BLOCK), 0, stream, w.rows[result], n, from, to);
}

} // namespace vesin_hip

#endif
