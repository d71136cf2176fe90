// Gradient of the pair geometry with respect to points and box: the step that turns per-pair gradients of an
// energy model (dE/d distance, dE/d vector) into forces and virial. The reference does this with tensor
// operations (vesin-torch/src/vesin_torch.cpp:437-468): vectors_grad += distances_grad * vectors / distances;
// points_grad[j] += vectors_grad; points_grad[i] -= vectors_grad; box_grad = shifts^T . vectors_grad.
// Here it is one pass over the rows, 92 bytes read per pair; the sums are gathered per workgroup in LDS and go
// to memory with one fp64 atomic per point, component and workgroup.
#ifndef VESIN_HIP_BACKWARD_CUH
#define VESIN_HIP_BACKWARD_CUH

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "device_common.cuh"

namespace vesin_hip {

constexpr int BACKWARD_THREADS = 256;

struct BackwardArgs {
    const size_t (*pairs)[2];
    const int32_t (*shifts)[3];    // nullptr: no gradient for the box
    const double* distances;
    const double (*vectors)[3];
    const double* distances_grad;  // nullptr: zero
    const double (*vectors_grad)[3]; // nullptr: zero
    size_t n_pairs;
    size_t n_points;
    double* points_grad;           // [n_points][3] or nullptr
    double* box_grad;              // [3][3] or nullptr
    uint32_t* bad_index;           // set to 1 when a pair names a point that does not exist
};

/// Sum over the 64 lanes of a wave, result in every lane.
__device__ inline double wave_sum(double value) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        value += __shfl_xor(value, offset, WAVE);
    }
    return value;
}

/// Sums a run of lanes that name the same point into the first lane of the run. `heads` has one bit per lane that
/// starts a run; afterwards the sums of a run stand in its first lane.
__device__ inline void sum_runs(uint64_t heads, double& gx, double& gy, double& gz) {
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    const uint64_t after = lane == 63 ? 0 : (heads >> (lane + 1)) << (lane + 1);
    const uint32_t run_end = after == 0 ? 64u : static_cast<uint32_t>(__builtin_ctzll(after));
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const double ox = __shfl_down(gx, offset, WAVE);
        const double oy = __shfl_down(gy, offset, WAVE);
        const double oz = __shfl_down(gz, offset, WAVE);
        if (lane + offset < run_end) {
            gx += ox;
            gy += oy;
            gz += oz;
        }
    }
}

/// Sums of one workgroup, by point, in LDS: rows that follow each other in a list name few different points (the
/// points of a few cells), so most additions meet here and only one sum per point and workgroup goes to memory,
/// where an atomic on a line shared by all compute dies costs far more than one in LDS.
constexpr uint32_t BACKWARD_SLOTS = 2048;
constexpr uint32_t BACKWARD_PROBES = 8;
constexpr uint32_t BACKWARD_EMPTY = 0xFFFFFFFFu;
constexpr size_t BACKWARD_ROWS_PER_BLOCK = 8192;

struct BackwardShared {
    uint32_t keys[BACKWARD_SLOTS];
    double sums[BACKWARD_SLOTS][3];
};

__device__ inline void add_to_point(BackwardShared& shared, double* points_grad, size_t point, double gx, double gy, double gz) {
    const uint32_t key = static_cast<uint32_t>(point);
    uint32_t slot = (key * 2654435761u) >> (32 - 11);
    static_assert(BACKWARD_SLOTS == (1u << 11), "the hash keeps 11 bits");
    for (uint32_t probe = 0; probe < BACKWARD_PROBES; probe++) {
        const uint32_t found = atomicCAS(&shared.keys[slot], BACKWARD_EMPTY, key);
        if (found == BACKWARD_EMPTY || found == key) {
            unsafeAtomicAdd(&shared.sums[slot][0], gx);
            unsafeAtomicAdd(&shared.sums[slot][1], gy);
            unsafeAtomicAdd(&shared.sums[slot][2], gz);
            return;
        }
        slot = (slot + 1) & (BACKWARD_SLOTS - 1);
    }
    // the neighbourhood of the slot is taken by other points
    unsafeAtomicAdd(points_grad + 3 * point + 0, gx);
    unsafeAtomicAdd(points_grad + 3 * point + 1, gy);
    unsafeAtomicAdd(points_grad + 3 * point + 2, gz);
}

__global__ __launch_bounds__(BACKWARD_THREADS) void pairs_backward_kernel(BackwardArgs args) {
    __shared__ BackwardShared shared;
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    double box_sum[9] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
    bool any_shift = false;

    if (args.points_grad != nullptr) {
        for (uint32_t slot = threadIdx.x; slot < BACKWARD_SLOTS; slot += BACKWARD_THREADS) {
            shared.keys[slot] = BACKWARD_EMPTY;
            shared.sums[slot][0] = 0.0;
            shared.sums[slot][1] = 0.0;
            shared.sums[slot][2] = 0.0;
        }
        __syncthreads();
    }

    // a workgroup takes rows that follow each other; every lane of a wave runs the same number of rounds (the sums
    // over runs use the whole wave)
    const size_t block_first = static_cast<size_t>(blockIdx.x) * BACKWARD_ROWS_PER_BLOCK;
    const size_t block_end = min(block_first + BACKWARD_ROWS_PER_BLOCK, args.n_pairs);
    for (size_t base = block_first + (threadIdx.x & ~(WAVE - 1)); base < block_end; base += BACKWARD_THREADS) {
        const size_t row = base + lane;
        bool active = row < block_end;
        // rows that do not count carry an index no point has, so that they never join the run of a neighbour
        size_t i = ~size_t(0);
        size_t j = 0;
        double gx = 0.0;
        double gy = 0.0;
        double gz = 0.0;
        if (active) {
            i = args.pairs[row][0];
            j = args.pairs[row][1];
            if (i >= args.n_points || j >= args.n_points) {
                *args.bad_index = 1;
                active = false;
                i = ~size_t(0);
            }
        }
        if (active) {
            if (args.vectors_grad != nullptr) {
                gx = args.vectors_grad[row][0];
                gy = args.vectors_grad[row][1];
                gz = args.vectors_grad[row][2];
            }
            if (args.distances_grad != nullptr) {
                const double dg = args.distances_grad[row];
                const double d = args.distances[row];
                gx += dg * args.vectors[row][0] / d;
                gy += dg * args.vectors[row][1] / d;
                gz += dg * args.vectors[row][2] / d;
            }
            if (args.shifts != nullptr) {
                const int32_t s0 = args.shifts[row][0];
                const int32_t s1 = args.shifts[row][1];
                const int32_t s2 = args.shifts[row][2];
                if ((s0 | s1 | s2) != 0) {
                    any_shift = true;
                    const double s[3] = {static_cast<double>(s0), static_cast<double>(s1), static_cast<double>(s2)};
#pragma unroll
                    for (int a = 0; a < 3; a++) {
                        box_sum[3 * a + 0] += s[a] * gx;
                        box_sum[3 * a + 1] += s[a] * gy;
                        box_sum[3 * a + 2] += s[a] * gz;
                    }
                }
            }
        }

        if (args.points_grad != nullptr) {
            if (active) {
                add_to_point(shared, args.points_grad, j, gx, gy, gz);
            }
            // rows of one first point often sit next to each other (always in a sorted list): one addition per run
            const size_t before = __shfl_up(static_cast<unsigned long long>(i), 1, WAVE);
            const bool head = lane == 0 || before != i;
            const uint64_t heads = __ballot(head);
            double mx = -gx;
            double my = -gy;
            double mz = -gz;
            bool add = active;
            if (__popcll(heads) <= 32) {
                sum_runs(heads, mx, my, mz);
                add = active && head;
            }
            if (add) {
                add_to_point(shared, args.points_grad, i, mx, my, mz);
            }
        }
    }

    if (args.points_grad != nullptr) {
        __syncthreads();
        for (uint32_t slot = threadIdx.x; slot < BACKWARD_SLOTS; slot += BACKWARD_THREADS) {
            const uint32_t key = shared.keys[slot];
            if (key != BACKWARD_EMPTY) {
                double* target = args.points_grad + 3 * static_cast<size_t>(key);
                unsafeAtomicAdd(target + 0, shared.sums[slot][0]);
                unsafeAtomicAdd(target + 1, shared.sums[slot][1]);
                unsafeAtomicAdd(target + 2, shared.sums[slot][2]);
            }
        }
    }

    if (args.box_grad != nullptr && __ballot(any_shift) != 0) {
#pragma unroll
        for (int k = 0; k < 9; k++) {
            const double total = wave_sum(box_sum[k]);
            if (lane == 0 && total != 0.0) {
                unsafeAtomicAdd(args.box_grad + k, total);
            }
        }
    }
}

} // namespace vesin_hip

#endif
