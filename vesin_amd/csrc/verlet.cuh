// Verlet caching (options.skin > 0): a candidate list computed at cutoff + skin is kept between calls and
// filtered at the cutoff while no point has moved further than skin / 2 (less what the box deformation eats).
// Follows the CPU engine of the reference: vesin/src/verlet.cpp:10-34 (corner displacement), :60-110 (when to
// rebuild), :149-190 (filter: T = S . H, v = (r_j - r_i) + T, keep iff |v|^2 < cutoff^2, same arithmetic as the
// direct search, so the rows are those of a direct calculation).
#ifndef VESIN_HIP_VERLET_CUH
#define VESIN_HIP_VERLET_CUH

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "device_common.cuh"
#include "search.cuh"

namespace vesin_hip {

constexpr int VERLET_BLOCK = 256;
/// candidates one lane keeps in registers between counting and writing
constexpr int VERLET_DEPTH = 8;
constexpr size_t VERLET_CHUNK = static_cast<size_t>(WAVE) * VERLET_DEPTH;
constexpr int VERLET_WAVES = VERLET_BLOCK / WAVE;

/// What the candidates were built from (device memory).
struct VerletReference {
    double box[9];
    unsigned char periodic[3];
    // the largest shift of a candidate along every direction, as an absolute value (verlet_shift_reach_kernel)
    unsigned int largest_shift[3];
};

/// Written by the kernels into pinned host memory, read by the host after the call's synchronisation.
struct VerletStatus {
    uint32_t rebuild;              // some point, or the box, moved too far (or the periodicity changed)
    uint32_t padding;
    unsigned long long total_rows; // rows the filter kept (also when they did not fit the arrays)
};

/// Work state of the filter in device memory.
struct VerletWork {
    unsigned long long total_rows;
    unsigned long long padding;
    double H[9]; // box of this call; rows of non-periodic directions are zero (their shifts are)
};

__global__ void verlet_store_reference(
    const double* __restrict__ box, const bool* __restrict__ periodic, VerletReference* __restrict__ reference
) {
    const int t = threadIdx.x;
    if (t < 9) {
        reference->box[t] = box[t];
    }
    if (t < 3) {
        reference->periodic[t] = periodic[t] ? 1 : 0;
        reference->largest_shift[t] = 0;
    }
}

/// The largest |S_d| among the candidates, per direction (launched behind verlet_store_reference). Points given far
/// outside of the box make pairs with shifts of several boxes, and how far the image of such a pair moves when the
/// box changes grows with the shift: see verlet_check_kernel.
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_shift_reach_kernel(
    const int32_t* __restrict__ candidate_shifts, size_t n_candidates, VerletReference* __restrict__ reference
) {
    unsigned int reach[3] = {0, 0, 0};
    const size_t stride = static_cast<size_t>(gridDim.x) * VERLET_BLOCK;
    for (size_t row = static_cast<size_t>(blockIdx.x) * VERLET_BLOCK + threadIdx.x; row < n_candidates; row += stride) {
#pragma unroll
        for (int d = 0; d < 3; d++) {
            const int32_t shift = candidate_shifts[3 * row + d];
            reach[d] = max(reach[d], static_cast<unsigned int>(shift < 0 ? -shift : shift));
        }
    }
#pragma unroll
    for (int d = 0; d < 3; d++) {
#pragma unroll
        for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
            reach[d] = max(reach[d], static_cast<unsigned int>(__shfl_xor(static_cast<int>(reach[d]), offset, WAVE)));
        }
        if (lane_id() == 0 && reach[d] > 1) {
            atomicMax(&reference->largest_shift[d], reach[d]);
        }
    }
}

/// Sum of the two largest displacements of a box corner between two boxes (vesin/src/verlet.cpp:12-34).
__device__ inline double corner_displacements(const double* box, const double* ref_box) {
    double largest = 0.0;
    double second = 0.0;
    for (int corner = 0; corner < 8; corner++) {
        const double b0 = static_cast<double>(corner & 1);
        const double b1 = static_cast<double>((corner >> 1) & 1);
        const double b2 = static_cast<double>((corner >> 2) & 1);
        double delta = 0.0;
        for (int k = 0; k < 3; k++) {
            const double now = b0 * box[k] + b1 * box[3 + k] + b2 * box[6 + k];
            const double then = b0 * ref_box[k] + b1 * ref_box[3 + k] + b2 * ref_box[6 + k];
            const double moved = now - then;
            delta += moved * moved;
        }
        if (delta > largest) {
            second = largest;
            largest = delta;
        } else if (delta > second) {
            second = delta;
        }
    }
    return sqrt(largest) + sqrt(second);
}

/// Decides whether the candidates still cover this call (vesin/src/verlet.cpp:60-110) and prepares the filter:
/// the box of this call and a zeroed row counter. `status->rebuild` must be 0 at launch.
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_check_kernel(
    const double* __restrict__ points, const double* __restrict__ ref_points, size_t n_points,
    const double* __restrict__ box, const bool* __restrict__ periodic, const VerletReference* __restrict__ reference,
    double skin, VerletStatus* __restrict__ status, VerletWork* __restrict__ work
) {
    __shared__ double threshold_sq;
    __shared__ uint32_t box_moved_too_far;
    if (threadIdx.x == 0) {
        bool too_far = false;
        for (int d = 0; d < 3; d++) {
            too_far = too_far || ((periodic[d] ? 1 : 0) != reference->periodic[d]);
        }
        const double half_skin = skin / 2.0;
        const double half_skin_sq = half_skin * half_skin;
        double half_displacement = corner_displacements(box, reference->box) / 2.0;
        // The reference's bound covers the images one box away: the image of a pair with shift S moves by S . (H -
        // H_ref) when the box changes, and for |S_d| <= 1 that is at most the two largest corner displacements. Points
        // given several boxes outside of the box make pairs with larger shifts, whose images move further: for them
        // the bound is sum_d max|S_d| x |H_d - H_ref_d| (never smaller than needed: more rebuilds, never a missed
        // pair). Nothing changes while the box stays as it is, or while no candidate has such a shift.
        if (reference->largest_shift[0] > 1 || reference->largest_shift[1] > 1 || reference->largest_shift[2] > 1) {
            double reach = 0.0;
            for (int d = 0; d < 3; d++) {
                double moved_sq = 0.0;
                for (int k = 0; k < 3; k++) {
                    const double moved = box[3 * d + k] - reference->box[3 * d + k];
                    moved_sq += moved * moved;
                }
                reach += static_cast<double>(max(reference->largest_shift[d], 1u)) * sqrt(moved_sq);
            }
            half_displacement = fmax(half_displacement, reach / 2.0);
        }
        // also true when the box holds a NaN
        too_far = too_far || !(half_displacement * half_displacement <= half_skin_sq);
        threshold_sq = (sqrt(half_skin_sq) - half_displacement) * (sqrt(half_skin_sq) - half_displacement);
        box_moved_too_far = too_far ? 1 : 0;
        if (blockIdx.x == 0) {
            if (too_far) {
                status->rebuild = 1;
            }
            work->total_rows = 0;
            for (int d = 0; d < 3; d++) {
                for (int k = 0; k < 3; k++) {
                    work->H[3 * d + k] = periodic[d] ? box[3 * d + k] : 0.0;
                }
            }
        }
    }
    __syncthreads();
    if (box_moved_too_far != 0) {
        return;
    }
    const size_t i = static_cast<size_t>(blockIdx.x) * VERLET_BLOCK + threadIdx.x;
    if (i < n_points) {
        const double dx = points[3 * i + 0] - ref_points[3 * i + 0];
        const double dy = points[3 * i + 1] - ref_points[3 * i + 1];
        const double dz = points[3 * i + 2] - ref_points[3 * i + 2];
        const double moved_sq = dx * dx + dy * dy + dz * dz;
        // a NaN coordinate rebuilds too: the direct search then reports it the way it always does
        if (!(moved_sq <= threshold_sq)) {
            status->rebuild = 1;
        }
    }
}

struct VerletFilterArgs {
    const unsigned long long* candidate_pairs; // [n_candidates][2]
    const int32_t* candidate_shifts;           // [n_candidates][3]
    size_t n_candidates;
    const double* points;
    VerletWork* work;
    double cutoff_sq;
    SearchOutputs out;
    size_t capacity; // rows the output arrays hold; a chunk that would pass it is counted but not written
};

/// One wave takes chunks of 512 candidates: tests them, takes room for the kept ones with one atomic, writes them.
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_filter_kernel(VerletFilterArgs a) {
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    const size_t wave = static_cast<size_t>(blockIdx.x) * VERLET_WAVES + threadIdx.x / WAVE;
    const size_t n_waves = static_cast<size_t>(gridDim.x) * VERLET_WAVES;
    double H[9];
#pragma unroll
    for (int k = 0; k < 9; k++) {
        H[k] = a.work->H[k];
    }

    for (size_t first = wave * VERLET_CHUNK; first < a.n_candidates; first += n_waves * VERLET_CHUNK) {
        unsigned long long pi[VERLET_DEPTH];
        unsigned long long pj[VERLET_DEPTH];
        int32_t sx[VERLET_DEPTH];
        int32_t sy[VERLET_DEPTH];
        int32_t sz[VERLET_DEPTH];
        double vx[VERLET_DEPTH];
        double vy[VERLET_DEPTH];
        double vz[VERLET_DEPTH];
        double dd[VERLET_DEPTH];
        uint32_t kept = 0;
        uint32_t before[VERLET_DEPTH];
        uint32_t chunk_rows = 0;
#pragma unroll
        for (int k = 0; k < VERLET_DEPTH; k++) {
            const size_t c = first + static_cast<size_t>(k) * WAVE + lane;
            bool keep = false;
            if (c < a.n_candidates) {
                pi[k] = a.candidate_pairs[2 * c + 0];
                pj[k] = a.candidate_pairs[2 * c + 1];
                sx[k] = a.candidate_shifts[3 * c + 0];
                sy[k] = a.candidate_shifts[3 * c + 1];
                sz[k] = a.candidate_shifts[3 * c + 2];
                const double tx = static_cast<double>(sx[k]) * H[0] + static_cast<double>(sy[k]) * H[3] +
                                  static_cast<double>(sz[k]) * H[6];
                const double ty = static_cast<double>(sx[k]) * H[1] + static_cast<double>(sy[k]) * H[4] +
                                  static_cast<double>(sz[k]) * H[7];
                const double tz = static_cast<double>(sx[k]) * H[2] + static_cast<double>(sy[k]) * H[5] +
                                  static_cast<double>(sz[k]) * H[8];
                vx[k] = (a.points[3 * pj[k] + 0] - a.points[3 * pi[k] + 0]) + tx;
                vy[k] = (a.points[3 * pj[k] + 1] - a.points[3 * pi[k] + 1]) + ty;
                vz[k] = (a.points[3 * pj[k] + 2] - a.points[3 * pi[k] + 2]) + tz;
                dd[k] = vx[k] * vx[k] + vy[k] * vy[k] + vz[k] * vz[k];
                keep = dd[k] < a.cutoff_sq;
            }
            const uint64_t mask = __ballot(keep);
            before[k] = chunk_rows + __builtin_amdgcn_mbcnt_hi(
                static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u)
            );
            chunk_rows += static_cast<uint32_t>(__popcll(mask));
            kept |= (keep ? 1u : 0u) << k;
        }
        if (chunk_rows == 0) {
            continue;
        }
        unsigned long long base = 0;
        if (lane == 0) {
            base = atomicAdd(&a.work->total_rows, static_cast<unsigned long long>(chunk_rows));
        }
        base = uniform(static_cast<uint64_t>(base));
        if (base + chunk_rows > a.capacity) {
            continue;
        }
#pragma unroll
        for (int k = 0; k < VERLET_DEPTH; k++) {
            if ((kept >> k) & 1u) {
                const size_t row = base + before[k];
                a.out.pairs[2 * row + 0] = pi[k];
                a.out.pairs[2 * row + 1] = pj[k];
                if (a.out.shifts != nullptr) {
                    a.out.shifts[3 * row + 0] = sx[k];
                    a.out.shifts[3 * row + 1] = sy[k];
                    a.out.shifts[3 * row + 2] = sz[k];
                }
                if (a.out.distances != nullptr) {
                    a.out.distances[row] = sqrt(dd[k]);
                }
                if (a.out.vectors != nullptr) {
                    a.out.vectors[3 * row + 0] = vx[k];
                    a.out.vectors[3 * row + 1] = vy[k];
                    a.out.vectors[3 * row + 2] = vz[k];
                }
            }
        }
    }
}

__global__ void verlet_publish(const VerletWork* __restrict__ work, VerletStatus* __restrict__ status) {
    status->total_rows = work->total_rows;
}

} // namespace vesin_hip

#endif
