// Batches of free molecules: systems without any periodic direction and with at most 256 points each. Such a system has
// no images and no use for a cell list: every point is tested against every other, v = r_j - r_i, |v|^2 < cutoff^2
// (the rows of the reference's CPU engine for such a system, vesin/src/cpu_cell_list.cpp:634-730 with all shifts
// zero). A group of 8, 16, 32 or 64 lanes takes one system, so a wave takes up to eight: lane j of the group holds
// point j, the group goes over i = 0, 1, ..., every lane tests (i, j), and the kept lanes of the group are consecutive
// rows. The rows of a system therefore come out ordered by (i, j), which is the sorted order, and a call is a counting
// pass (rows per system), a scan over the systems (which is `first_pair`), and a writing pass. Batches with a system
// of more than 64 points give every system a workgroup of four waves instead (molecules_wide_kernel), each wave taking
// every fourth i with the j in rounds of 64: rows are counted per point then, and scanned over the points.
#ifndef VESIN_HIP_MOLECULES_CUH
#define VESIN_HIP_MOLECULES_CUH

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "cells.cuh"
#include "device_common.cuh"
#include "search.cuh"

namespace vesin_hip {

constexpr uint32_t MOLECULE_GROUP_POINTS = 64; // up to here a group of lanes takes a system
constexpr uint32_t MOLECULE_MAX_POINTS = 256;  // and up to here a workgroup does
constexpr int MOLECULE_BLOCK = 256;
static_assert(MOLECULE_BLOCK == BLOCK && MOLECULE_MAX_POINTS == MOLECULE_BLOCK, "one thread per point of the largest system");

/// What the kernels report: gathered in device memory (cleared before the launches), copied to pinned host memory by
/// the writing pass.
struct MoleculeStatus {
    uint32_t periodic;            // some system has a periodic direction: not a batch for these kernels
    uint32_t first_bad;           // lowest 3 * point + axis of a coordinate that is not finite, or 0xFFFFFFFF
    unsigned long long total_rows;
};

struct MoleculeArgs {
    const double* points;
    const bool* periodic;          // [n_systems][3]
    const uint32_t* first_point;   // [n_systems + 1]
    uint32_t n_systems;
    double cutoff2;
    int full;
    uint32_t* rows_of_system;      // [n_systems]: written by the counting pass
    const uint64_t* first_pair;    // [n_systems + 1]: their exclusive scan, read by the writing pass
    // (a workgroup per system, molecules_wide_kernel: rows per point in place of rows per system)
    uint32_t total_points;
    uint32_t* rows_of_point;       // [total_points]
    const uint64_t* first_row;     // [total_points + 1]
    SearchOutputs out;
    size_t capacity;               // rows the output arrays hold: a longer list is not written at all (and
                                   // nothing is when the counting pass met a periodic direction)
    MoleculeStatus* status;        // device
    MoleculeStatus* report;        // pinned
};

template <int G, bool WRITE>
__global__ __launch_bounds__(MOLECULE_BLOCK) void molecules_kernel(MoleculeArgs a) {
    constexpr int GROUPS = WAVE / G;
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    const uint32_t group = lane / G;
    const uint32_t j = lane % G;
    const uint32_t wave = blockIdx.x * (MOLECULE_BLOCK / WAVE) + threadIdx.x / WAVE;
    const uint32_t system = wave * GROUPS + group;
    const bool exists = system < a.n_systems;

    unsigned long long total = 0;
    if (WRITE) {
        total = a.first_pair[a.n_systems];
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            a.report->periodic = a.status->periodic;
            a.report->first_bad = a.status->first_bad;
            a.report->total_rows = total;
        }
        if (total > a.capacity || a.status->periodic != 0) {
            return;
        }
    }

    uint32_t begin = 0;
    uint32_t n = 0;
    if (exists) {
        begin = a.first_point[system];
        n = a.first_point[system + 1] - begin;
    }
    double x = 0.0, y = 0.0, z = 0.0;
    if (j < n) {
        const size_t at = 3 * static_cast<size_t>(begin + j);
        x = a.points[at + 0];
        y = a.points[at + 1];
        z = a.points[at + 2];
        if (!WRITE) {
            unsigned int axis;
            if (!all_finite(x, y, z, axis)) {
                atomicMin(&a.status->first_bad, 3u * (begin + j) + axis);
            }
        }
    }
    if (!WRITE && exists && j < 3 && a.periodic[3 * static_cast<size_t>(system) + j]) {
        a.status->periodic = 1;
    }
    // as many rounds as the largest system of the wave has points
    uint32_t rounds = n;
#pragma unroll
    for (int offset = WAVE / 2; offset >= G; offset >>= 1) {
        rounds = max(rounds, static_cast<uint32_t>(__shfl_xor(static_cast<int>(rounds), offset, WAVE)));
    }
    rounds = uniform(rounds);

    const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (WAVE - lane));              // the lanes before this one
    const uint64_t of_group = (G == WAVE ? ~0ull : ((1ull << G) - 1ull)) << (group * G); // the lanes of this group
    uint64_t row = WRITE && exists ? a.first_pair[system] : 0;
    uint32_t rows = 0;
    for (uint32_t i = 0; i < rounds; i++) {
        const int source = static_cast<int>(group * G + i);
        const double xi = __shfl(x, source, WAVE);
        const double yi = __shfl(y, source, WAVE);
        const double zi = __shfl(z, source, WAVE);
        // (the shift of every pair is zero: adding it is what the general search does, and what turns a -0 into 0)
        const double vx = (x - xi) + 0.0;
        const double vy = (y - yi) + 0.0;
        const double vz = (z - zi) + 0.0;
        const double dd = vx * vx + vy * vy + vz * vz;
        const bool keep = i < n && j < n && (a.full ? j != i : j > i) && dd < a.cutoff2;
        const uint64_t mine = __ballot(keep) & of_group;
        if (WRITE) {
            if (keep) {
                const uint64_t at = row + static_cast<uint64_t>(__popcll(mine & below));
                a.out.pairs[2 * at + 0] = i;
                a.out.pairs[2 * at + 1] = j;
                if (a.out.shifts != nullptr) {
                    a.out.shifts[3 * at + 0] = 0;
                    a.out.shifts[3 * at + 1] = 0;
                    a.out.shifts[3 * at + 2] = 0;
                }
                if (a.out.distances != nullptr) {
                    a.out.distances[at] = sqrt(dd);
                }
                if (a.out.vectors != nullptr) {
                    a.out.vectors[3 * at + 0] = vx;
                    a.out.vectors[3 * at + 1] = vy;
                    a.out.vectors[3 * at + 2] = vz;
                }
            }
            row += static_cast<uint64_t>(__popcll(mine));
        } else {
            rows += static_cast<uint32_t>(__popcll(mine));
        }
    }
    if (!WRITE && exists && j == 0) {
        a.rows_of_system[system] = rows;
    }
}

/// One workgroup per system of up to 256 points. A wave takes every fourth first point i, its lanes hold the second
/// points j in up to four rounds of 64, so the rows of i are one wave's: counted into `rows_of_point` by the counting
/// pass, written from `first_row[i]` (the scan of these counts over the points of all systems) by the writing pass.
template <bool WRITE>
__global__ __launch_bounds__(MOLECULE_BLOCK) void molecules_wide_kernel(MoleculeArgs a) {
    constexpr int WAVES = MOLECULE_BLOCK / WAVE;
    constexpr int ROUNDS = MOLECULE_MAX_POINTS / WAVE;
    __shared__ double px[MOLECULE_MAX_POINTS], py[MOLECULE_MAX_POINTS], pz[MOLECULE_MAX_POINTS];
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    const uint32_t wave = threadIdx.x / WAVE;
    const uint32_t system = blockIdx.x;

    if (WRITE) {
        const unsigned long long total = a.first_row[a.total_points];
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            a.report->periodic = a.status->periodic;
            a.report->first_bad = a.status->first_bad;
            a.report->total_rows = total;
        }
        if (total > a.capacity || a.status->periodic != 0) {
            return;
        }
    }
    const uint32_t begin = a.first_point[system];
    const uint32_t n = a.first_point[system + 1] - begin;
    if (threadIdx.x < n) {
        const size_t at = 3 * static_cast<size_t>(begin + threadIdx.x);
        const double x = a.points[at + 0];
        const double y = a.points[at + 1];
        const double z = a.points[at + 2];
        px[threadIdx.x] = x;
        py[threadIdx.x] = y;
        pz[threadIdx.x] = z;
        if (!WRITE) {
            unsigned int axis;
            if (!all_finite(x, y, z, axis)) {
                atomicMin(&a.status->first_bad, 3u * (begin + threadIdx.x) + axis);
            }
        }
    }
    if (!WRITE && threadIdx.x < 3 && a.periodic[3 * static_cast<size_t>(system) + threadIdx.x]) {
        a.status->periodic = 1;
    }
    __syncthreads();

    // the second points of this lane, one per round
    double xs[ROUNDS], ys[ROUNDS], zs[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        const uint32_t j = r * WAVE + lane;
        xs[r] = j < n ? px[j] : 0.0;
        ys[r] = j < n ? py[j] : 0.0;
        zs[r] = j < n ? pz[j] : 0.0;
    }
    const uint32_t rounds = (n + WAVE - 1) / WAVE;
    const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (WAVE - lane));
    for (uint32_t i = wave; i < n; i += WAVES) {
        const double xi = px[i];
        const double yi = py[i];
        const double zi = pz[i];
        uint64_t row = WRITE ? a.first_row[begin + i] : 0;
        uint32_t rows = 0;
#pragma unroll
        for (int r = 0; r < ROUNDS; r++) {
            if (static_cast<uint32_t>(r) < rounds) {
                const uint32_t j = r * WAVE + lane;
                // (the shift of every pair is zero: adding it is what the general search does, and what turns a -0 into 0)
                const double vx = (xs[r] - xi) + 0.0;
                const double vy = (ys[r] - yi) + 0.0;
                const double vz = (zs[r] - zi) + 0.0;
                const double dd = vx * vx + vy * vy + vz * vz;
                const bool keep = j < n && (a.full ? j != i : j > i) && dd < a.cutoff2;
                const uint64_t mask = __ballot(keep);
                if (WRITE) {
                    if (keep) {
                        const uint64_t at = row + static_cast<uint64_t>(__popcll(mask & below));
                        a.out.pairs[2 * at + 0] = i;
                        a.out.pairs[2 * at + 1] = j;
                        if (a.out.shifts != nullptr) {
                            a.out.shifts[3 * at + 0] = 0;
                            a.out.shifts[3 * at + 1] = 0;
                            a.out.shifts[3 * at + 2] = 0;
                        }
                        if (a.out.distances != nullptr) {
                            a.out.distances[at] = sqrt(dd);
                        }
                        if (a.out.vectors != nullptr) {
                            a.out.vectors[3 * at + 0] = vx;
                            a.out.vectors[3 * at + 1] = vy;
                            a.out.vectors[3 * at + 2] = vz;
                        }
                    }
                    row += static_cast<uint64_t>(__popcll(mask));
                } else {
                    rows += static_cast<uint32_t>(__popcll(mask));
                }
            }
        }
        if (!WRITE && lane == 0) {
            a.rows_of_point[begin + i] = rows;
        }
    }
}

} // namespace vesin_hip

#endif
