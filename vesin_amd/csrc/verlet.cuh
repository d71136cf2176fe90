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
    uint32_t unusable;             // (batches) some candidate has a shift that the filter's records cannot hold
    unsigned long long total_rows; // rows the filter kept (also when they did not fit the arrays)
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
/// box changes grows with the shift: see verlet_check_and_count_kernel.
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

struct VerletFilterArgs {
    const unsigned long long* candidate_pairs; // [n_candidates][2]
    const int32_t* candidate_shifts;           // [n_candidates][3]
    size_t n_candidates;
    size_t n_chunks;       // of VERLET_CHUNK candidates
    const double* points;
    const double* box;     // of this call
    const bool* periodic;
    double cutoff_sq;
    uint32_t* chunk_rows;  // [n_chunks]: the rows every chunk keeps, written by the counting pass
    uint64_t* chunk_base;  // [n_chunks + 1]: their exclusive scan, for lists of more than VERLET_SELF_SCAN_CHUNKS chunks
    SearchOutputs out;
    size_t capacity;       // rows the output arrays hold: a longer list is not written at all
    VerletStatus* status;  // pinned
};

/// Lists of at most this many chunks (0.5 M candidates) go without a scan of their own: every wave of the writing
/// pass adds up the counts before its chunk itself. (With 3,200 chunks that cost more than the scan's launch: 0.080
/// against 0.073 ms per call.)
constexpr size_t VERLET_SELF_SCAN_CHUNKS = 1024;

/// The box as the filter uses it: rows of non-periodic directions are zero (their shifts are).
__device__ __forceinline__ void filter_box(const double* __restrict__ box, const bool* __restrict__ periodic, double* H) {
#pragma unroll
    for (int d = 0; d < 3; d++) {
        const bool p = periodic[d];
#pragma unroll
        for (int k = 0; k < 3; k++) {
            H[3 * d + k] = p ? box[3 * d + k] : 0.0;
        }
    }
}

/// Tests the candidates of one chunk, 64 at a time; `visit(k, keep, mask, ...)` sees every group of 64 with the ballot
/// of the kept ones. T = S . H, v = (r_j - r_i) + T, keep iff |v|^2 < cutoff^2: the arithmetic of the search.
struct TestedCandidate {
    unsigned long long i, j;
    int32_t sx, sy, sz;
    double vx, vy, vz, dd;
    bool keep;
};

__device__ __forceinline__ TestedCandidate test_candidate(const VerletFilterArgs& a, const double* H, size_t c) {
    TestedCandidate t = {};
    if (c < a.n_candidates) {
        t.i = a.candidate_pairs[2 * c + 0];
        t.j = a.candidate_pairs[2 * c + 1];
        t.sx = a.candidate_shifts[3 * c + 0];
        t.sy = a.candidate_shifts[3 * c + 1];
        t.sz = a.candidate_shifts[3 * c + 2];
        const double tx = static_cast<double>(t.sx) * H[0] + static_cast<double>(t.sy) * H[3] + static_cast<double>(t.sz) * H[6];
        const double ty = static_cast<double>(t.sx) * H[1] + static_cast<double>(t.sy) * H[4] + static_cast<double>(t.sz) * H[7];
        const double tz = static_cast<double>(t.sx) * H[2] + static_cast<double>(t.sy) * H[5] + static_cast<double>(t.sz) * H[8];
        t.vx = (a.points[3 * t.j + 0] - a.points[3 * t.i + 0]) + tx;
        t.vy = (a.points[3 * t.j + 1] - a.points[3 * t.i + 1]) + ty;
        t.vz = (a.points[3 * t.j + 2] - a.points[3 * t.i + 2]) + tz;
        t.dd = t.vx * t.vx + t.vy * t.vy + t.vz * t.vz;
        t.keep = t.dd < a.cutoff_sq;
    }
    return t;
}

/// First launch of a filtered call, two jobs. (1) Whether the candidates still cover this call
/// (vesin/src/verlet.cpp:60-110): thread 0 of every workgroup with points evaluates the box, a thread per point how
/// far it moved; `status->rebuild` must be 0 at launch. (2) The counting pass of the filter, in two passes that keep
/// the order of the candidates (sorted candidates give sorted rows without a sort, and an unsorted list comes out
/// the same way on every call): the rows every chunk of 512 candidates keeps. Neither waits for the other: when
/// the check fails the counts are not used.
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_check_and_count_kernel(
    const double* __restrict__ ref_points, size_t n_points, const VerletReference* __restrict__ reference, double skin,
    VerletFilterArgs a
) {
    __shared__ double threshold_sq;
    __shared__ uint32_t box_moved_too_far;
    const size_t check_blocks = (n_points + VERLET_BLOCK - 1) / VERLET_BLOCK;
    if (blockIdx.x < check_blocks || blockIdx.x == 0) {
        if (threadIdx.x == 0) {
            bool too_far = false;
            for (int d = 0; d < 3; d++) {
                too_far = too_far || ((a.periodic[d] ? 1 : 0) != reference->periodic[d]);
            }
            const double half_skin = skin / 2.0;
            const double half_skin_sq = half_skin * half_skin;
            double half_displacement = corner_displacements(a.box, reference->box) / 2.0;
            // The reference's bound covers the images one box away: the image of a pair with shift S moves by S . (H -
            // H_ref) when the box changes, and for |S_d| <= 1 that is at most the two largest corner displacements.
            // Points given several boxes outside of the box make pairs with larger shifts, whose images move further:
            // for them the bound is sum_d max|S_d| x |H_d - H_ref_d| (never smaller than needed: more rebuilds, never
            // a missed pair). Nothing changes while the box stays as it is, or while no candidate has such a shift.
            if (reference->largest_shift[0] > 1 || reference->largest_shift[1] > 1 || reference->largest_shift[2] > 1) {
                double reach = 0.0;
                for (int d = 0; d < 3; d++) {
                    double moved_sq = 0.0;
                    for (int k = 0; k < 3; k++) {
                        const double moved = a.box[3 * d + k] - reference->box[3 * d + k];
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
            if (blockIdx.x == 0 && too_far) {
                a.status->rebuild = 1;
            }
        }
        __syncthreads();
        const size_t i = static_cast<size_t>(blockIdx.x) * VERLET_BLOCK + threadIdx.x;
        if (box_moved_too_far == 0 && i < n_points) {
            const double dx = a.points[3 * i + 0] - ref_points[3 * i + 0];
            const double dy = a.points[3 * i + 1] - ref_points[3 * i + 1];
            const double dz = a.points[3 * i + 2] - ref_points[3 * i + 2];
            const double moved_sq = dx * dx + dy * dy + dz * dz;
            // a NaN coordinate rebuilds too: the direct search then reports it the way it always does
            if (!(moved_sq <= threshold_sq)) {
                a.status->rebuild = 1;
            }
        }
    }

    const uint32_t lane = static_cast<uint32_t>(lane_id());
    const size_t wave = static_cast<size_t>(blockIdx.x) * VERLET_WAVES + threadIdx.x / WAVE;
    const size_t n_waves = static_cast<size_t>(gridDim.x) * VERLET_WAVES;
    double H[9];
    filter_box(a.box, a.periodic, H);
    for (size_t chunk = wave; chunk < a.n_chunks; chunk += n_waves) {
        uint32_t kept_rows = 0;
#pragma unroll
        for (int k = 0; k < VERLET_DEPTH; k++) {
            const TestedCandidate t = test_candidate(a, H, chunk * VERLET_CHUNK + static_cast<size_t>(k) * WAVE + lane);
            kept_rows += static_cast<uint32_t>(__popcll(__ballot(t.keep)));
        }
        if (lane == 0) {
            a.chunk_rows[chunk] = kept_rows;
        }
    }
}

/// The writing pass: the same tests again, and every kept row goes where the kept rows before it end. Where these
/// are comes from the scan of the counts (`chunk_base`), or with SELF_SCAN from the counts themselves. A list longer
/// than `capacity` is not written at all; the total goes to `status` either way. (One pass that kept the tested
/// candidates in registers and took room for a chunk's rows with an atomic was slower, 0.100 against 0.074 ms at
/// 1.6 M candidates and 0.52 against 0.43 ms at 13 M.)
template <bool SELF_SCAN>
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_write_kernel(VerletFilterArgs a) {
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    const size_t wave = static_cast<size_t>(blockIdx.x) * VERLET_WAVES + threadIdx.x / WAVE;
    const size_t n_waves = static_cast<size_t>(gridDim.x) * VERLET_WAVES;
    double H[9];
    filter_box(a.box, a.periodic, H);
    unsigned long long total = 0;
    unsigned long long before_mine = 0; // SELF_SCAN: the rows of the chunks before this wave's (it has one at most)
    if (SELF_SCAN) {
        unsigned long long all = 0;
        unsigned long long before = 0;
        for (size_t chunk = lane; chunk < a.n_chunks; chunk += WAVE) {
            const unsigned long long rows = a.chunk_rows[chunk];
            all += rows;
            before += chunk < wave ? rows : 0;
        }
#pragma unroll
        for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
            all += __shfl_xor(all, offset, WAVE);
            before += __shfl_xor(before, offset, WAVE);
        }
        total = all;
        before_mine = before;
    } else {
        total = a.chunk_base[a.n_chunks];
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        a.status->total_rows = total;
    }
    if (total > a.capacity) {
        return;
    }
    for (size_t chunk = wave; chunk < a.n_chunks; chunk += n_waves) {
        uint64_t row = SELF_SCAN ? before_mine : a.chunk_base[chunk];
#pragma unroll
        for (int k = 0; k < VERLET_DEPTH; k++) {
            const TestedCandidate t = test_candidate(a, H, chunk * VERLET_CHUNK + static_cast<size_t>(k) * WAVE + lane);
            const uint64_t mask = __ballot(t.keep);
            if (t.keep) {
                const uint64_t mine = row + __builtin_amdgcn_mbcnt_hi(
                    static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u)
                );
                a.out.pairs[2 * mine + 0] = t.i;
                a.out.pairs[2 * mine + 1] = t.j;
                if (a.out.shifts != nullptr) {
                    a.out.shifts[3 * mine + 0] = t.sx;
                    a.out.shifts[3 * mine + 1] = t.sy;
                    a.out.shifts[3 * mine + 2] = t.sz;
                }
                if (a.out.distances != nullptr) {
                    a.out.distances[mine] = sqrt(t.dd);
                }
                if (a.out.vectors != nullptr) {
                    a.out.vectors[3 * mine + 0] = t.vx;
                    a.out.vectors[3 * mine + 1] = t.vy;
                    a.out.vectors[3 * mine + 2] = t.vz;
                }
            }
            row += static_cast<uint64_t>(__popcll(mask));
        }
    }
}

// ---- batches of systems: one candidate list for the whole batch (the rows of a batch call at cutoff + skin, system
// after system), filtered in two passes that keep the order of the candidates, so that the rows of a system stay
// together (and sorted, when the candidates were). Every system has its own box, so every system has its own
// limit on how far its points may have moved; one system past its limit and all candidates are computed again.

/// What the candidates of one system were built from. The rows of directions that are not periodic are zero: no
/// shift runs along them, and a system without any periodic direction has a box that is never read.
struct BatchVerletReference {
    double box[9];
    unsigned char periodic[3];
    unsigned char padding;
    unsigned int largest_shift[3];
};

/// Per system and call: the box the filter uses (zero rows for directions that are not periodic) and how far a
/// point may have moved, squared.
struct BatchVerletLimits {
    double H[9];
    double threshold_sq;
    unsigned long long first_point; // of the system, among the points of the batch
};

/// One candidate as the filter reads it: both points by their index in the batch and the shift, 16 bytes in place of
/// the 40 of a row with its shift.
struct BatchVerletCandidate {
    uint32_t i;
    uint32_t j;
    uint64_t shift; // three fields of 21 bits, each shift plus 2^20
};
constexpr int32_t BATCH_VERLET_SHIFT_BIAS = 1 << 20;

__device__ __forceinline__ int32_t unpack_candidate_shift(uint64_t packed, int direction) {
    return static_cast<int32_t>((packed >> (21 * direction)) & 0x1FFFFFu) - BATCH_VERLET_SHIFT_BIAS;
}

__device__ __forceinline__ void masked_box(
    const double* __restrict__ box, const bool* __restrict__ periodic, double* out, unsigned char* flags
) {
#pragma unroll
    for (int d = 0; d < 3; d++) {
        const bool p = periodic[d];
        flags[d] = p ? 1 : 0;
#pragma unroll
        for (int k = 0; k < 3; k++) {
            out[3 * d + k] = p ? box[3 * d + k] : 0.0;
        }
    }
}

__global__ __launch_bounds__(VERLET_BLOCK) void verlet_batch_store_reference(
    const double* __restrict__ boxes, const bool* __restrict__ periodic, uint32_t n_systems,
    BatchVerletReference* __restrict__ reference
) {
    const uint32_t s = blockIdx.x * VERLET_BLOCK + threadIdx.x;
    if (s >= n_systems) {
        return;
    }
    BatchVerletReference mine;
    masked_box(boxes + 9 * static_cast<size_t>(s), periodic + 3 * static_cast<size_t>(s), mine.box, mine.periodic);
    mine.padding = 0;
    mine.largest_shift[0] = mine.largest_shift[1] = mine.largest_shift[2] = 0;
    reference[s] = mine;
}

/// The system s with firsts[s] <= item < firsts[s + 1] (`firsts` has n_systems + 1 entries, starts at 0 and never
/// decreases).
__device__ __forceinline__ uint32_t system_holding(const unsigned long long* __restrict__ firsts, uint32_t n_systems, size_t item) {
    uint32_t lo = 0;
    uint32_t hi = n_systems;
    while (hi - lo > 1) {
        const uint32_t middle = lo + (hi - lo) / 2;
        if (firsts[middle] <= item) {
            lo = middle;
        } else {
            hi = middle;
        }
    }
    return lo;
}

__global__ __launch_bounds__(VERLET_BLOCK) void verlet_batch_owner_kernel(
    const unsigned long long* __restrict__ first_point, uint32_t n_systems, size_t n_points,
    uint32_t* __restrict__ system_of_point
) {
    const size_t stride = static_cast<size_t>(gridDim.x) * VERLET_BLOCK;
    for (size_t i = static_cast<size_t>(blockIdx.x) * VERLET_BLOCK + threadIdx.x; i < n_points; i += stride) {
        system_of_point[i] = system_holding(first_point, n_systems, i);
    }
}

/// The rows of the batch call at cutoff + skin become the candidates the filter reads, and the largest |S_d| of
/// every system's candidates is noted as verlet_shift_reach_kernel does. A shift that does not fit its 21 bits
/// raises `*out_of_range` (the candidates are of no use then).
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_batch_pack_kernel(
    const unsigned long long* __restrict__ pairs, const int32_t* __restrict__ shifts, size_t n_candidates,
    const unsigned long long* __restrict__ candidate_first_pair, const unsigned long long* __restrict__ first_point,
    uint32_t n_systems, BatchVerletCandidate* __restrict__ candidates, BatchVerletReference* __restrict__ reference,
    uint32_t* __restrict__ out_of_range
) {
    const size_t stride = static_cast<size_t>(gridDim.x) * VERLET_BLOCK;
    for (size_t c = static_cast<size_t>(blockIdx.x) * VERLET_BLOCK + threadIdx.x; c < n_candidates; c += stride) {
        const uint32_t system = system_holding(candidate_first_pair, n_systems, c);
        const unsigned long long first = first_point[system];
        BatchVerletCandidate packed;
        packed.i = static_cast<uint32_t>(first + pairs[2 * c + 0]);
        packed.j = static_cast<uint32_t>(first + pairs[2 * c + 1]);
        packed.shift = 0;
#pragma unroll
        for (int d = 0; d < 3; d++) {
            const int32_t shift = shifts[3 * c + d];
            const unsigned int reach = static_cast<unsigned int>(shift < 0 ? -shift : shift);
            if (reach > 1) {
                atomicMax(&reference[system].largest_shift[d], reach);
            }
            if (reach >= static_cast<unsigned int>(BATCH_VERLET_SHIFT_BIAS)) {
                *out_of_range = 1;
            }
            packed.shift |= static_cast<uint64_t>(static_cast<uint32_t>(shift + BATCH_VERLET_SHIFT_BIAS) & 0x1FFFFFu) << (21 * d);
        }
        candidates[c] = packed;
    }
}

/// verlet_check_and_count_kernel's decision about the box, for every system of a batch. `status->rebuild` must be 0 at launch.
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_batch_limits_kernel(
    const double* __restrict__ boxes, const bool* __restrict__ periodic, const BatchVerletReference* __restrict__ reference,
    const unsigned long long* __restrict__ first_point, uint32_t n_systems, double skin,
    BatchVerletLimits* __restrict__ limits, VerletStatus* __restrict__ status
) {
    const uint32_t s = blockIdx.x * VERLET_BLOCK + threadIdx.x;
    if (s >= n_systems) {
        return;
    }
    BatchVerletLimits mine;
    unsigned char flags[3];
    masked_box(boxes + 9 * static_cast<size_t>(s), periodic + 3 * static_cast<size_t>(s), mine.H, flags);
    const BatchVerletReference then = reference[s];
    bool too_far = false;
    for (int d = 0; d < 3; d++) {
        too_far = too_far || flags[d] != then.periodic[d];
    }
    const double half_skin = skin / 2.0;
    const double half_skin_sq = half_skin * half_skin;
    double half_displacement = corner_displacements(mine.H, then.box) / 2.0;
    if (then.largest_shift[0] > 1 || then.largest_shift[1] > 1 || then.largest_shift[2] > 1) {
        // candidates whose shifts reach further than one box: see verlet_check_and_count_kernel
        double reach = 0.0;
        for (int d = 0; d < 3; d++) {
            double moved_sq = 0.0;
            for (int k = 0; k < 3; k++) {
                const double moved = mine.H[3 * d + k] - then.box[3 * d + k];
                moved_sq += moved * moved;
            }
            reach += static_cast<double>(max(then.largest_shift[d], 1u)) * sqrt(moved_sq);
        }
        half_displacement = fmax(half_displacement, reach / 2.0);
    }
    // also true when a box row that is read holds a NaN
    too_far = too_far || !(half_displacement * half_displacement <= half_skin_sq);
    mine.threshold_sq = (sqrt(half_skin_sq) - half_displacement) * (sqrt(half_skin_sq) - half_displacement);
    if (too_far) {
        mine.threshold_sq = -1.0;
        status->rebuild = 1;
    }
    mine.first_point = first_point[s];
    limits[s] = mine;
}

__global__ __launch_bounds__(VERLET_BLOCK) void verlet_batch_moved_kernel(
    const double* __restrict__ points, const double* __restrict__ ref_points, size_t n_points,
    const uint32_t* __restrict__ system_of_point, const BatchVerletLimits* __restrict__ limits,
    VerletStatus* __restrict__ status
) {
    const size_t i = static_cast<size_t>(blockIdx.x) * VERLET_BLOCK + threadIdx.x;
    if (i >= n_points) {
        return;
    }
    const double dx = points[3 * i + 0] - ref_points[3 * i + 0];
    const double dy = points[3 * i + 1] - ref_points[3 * i + 1];
    const double dz = points[3 * i + 2] - ref_points[3 * i + 2];
    const double moved_sq = dx * dx + dy * dy + dz * dz;
    // (a NaN coordinate computes the candidates again too: the search then reports it the way it always does)
    if (!(moved_sq <= limits[system_of_point[i]].threshold_sq)) {
        status->rebuild = 1;
    }
}

struct BatchVerletFilterArgs {
    const BatchVerletCandidate* candidates;    // [n_candidates]
    const uint32_t* system_of_point;           // [n_points]
    size_t n_candidates;
    size_t n_chunks;                           // of VERLET_CHUNK candidates
    const double* points;
    const BatchVerletLimits* limits;
    double cutoff_sq;
    uint32_t* chunk_rows;                      // [n_chunks]: written by the counting pass
    const uint64_t* chunk_base;                // [n_chunks + 1]: their exclusive scan, read by the writing pass
    SearchOutputs out;                         // pairs with indices inside the row's system
    size_t capacity;                           // rows the output arrays hold: a longer list is not written at all
    unsigned long long* first_pair;            // [n_systems + 1], filled by the writing pass
    uint32_t n_systems;
    VerletStatus* status;
};

/// One wave takes chunks of 512 candidates. Counting pass: the rows every chunk keeps. Writing pass (behind the scan
/// of these counts): the same tests again, and every kept row goes where the kept rows before it end, so the rows
/// keep the order of the candidates; the lane that holds the first candidate of a system also says where that
/// system's rows begin.
template <bool WRITE>
__global__ __launch_bounds__(VERLET_BLOCK) void verlet_batch_filter_kernel(BatchVerletFilterArgs a) {
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    const size_t wave = static_cast<size_t>(blockIdx.x) * VERLET_WAVES + threadIdx.x / WAVE;
    const size_t n_waves = static_cast<size_t>(gridDim.x) * VERLET_WAVES;
    unsigned long long total = 0;
    if (WRITE) {
        total = a.chunk_base[a.n_chunks];
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            a.status->total_rows = total;
        }
    }
    const bool fits = total <= a.capacity;

    for (size_t chunk = wave; chunk < a.n_chunks; chunk += n_waves) {
        const size_t first = chunk * VERLET_CHUNK;
        uint64_t row = WRITE ? a.chunk_base[chunk] : 0;
        uint32_t chunk_rows = 0;
#pragma unroll
        for (int k = 0; k < VERLET_DEPTH; k++) {
            const size_t c = first + static_cast<size_t>(k) * WAVE + lane;
            bool keep = false;
            uint32_t gi = 0, gj = 0;
            int32_t sx = 0, sy = 0, sz = 0;
            double vx = 0.0, vy = 0.0, vz = 0.0, dd = 0.0;
            uint32_t system = 0;
            unsigned long long first_point = 0;
            if (c < a.n_candidates) {
                const BatchVerletCandidate candidate = a.candidates[c];
                gi = candidate.i;
                gj = candidate.j;
                sx = unpack_candidate_shift(candidate.shift, 0);
                sy = unpack_candidate_shift(candidate.shift, 1);
                sz = unpack_candidate_shift(candidate.shift, 2);
                system = a.system_of_point[gi];
                const BatchVerletLimits* of_system = a.limits + system;
                const double* H = of_system->H;
                first_point = of_system->first_point;
                const double tx = static_cast<double>(sx) * H[0] + static_cast<double>(sy) * H[3] + static_cast<double>(sz) * H[6];
                const double ty = static_cast<double>(sx) * H[1] + static_cast<double>(sy) * H[4] + static_cast<double>(sz) * H[7];
                const double tz = static_cast<double>(sx) * H[2] + static_cast<double>(sy) * H[5] + static_cast<double>(sz) * H[8];
                const double* ri = a.points + 3 * static_cast<size_t>(gi);
                const double* rj = a.points + 3 * static_cast<size_t>(gj);
                vx = (rj[0] - ri[0]) + tx;
                vy = (rj[1] - ri[1]) + ty;
                vz = (rj[2] - ri[2]) + tz;
                dd = vx * vx + vy * vy + vz * vz;
                keep = dd < a.cutoff_sq;
            }
            const uint64_t mask = __ballot(keep);
            if (WRITE) {
                const uint64_t mine = row + __builtin_amdgcn_mbcnt_hi(
                    static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u)
                );
                // the system of the candidate before this one: the lane below holds it, or memory does
                uint32_t before = static_cast<uint32_t>(__shfl_up(static_cast<int>(system), 1, WAVE));
                if (c < a.n_candidates) {
                    if (lane == 0) {
                        before = c == 0 ? 0xFFFFFFFFu : a.system_of_point[a.candidates[c - 1].i];
                    }
                    if (before != system) {
                        // (systems without candidates in between begin, and end, here as well)
                        for (uint32_t s = before + 1; s != system + 1; s++) {
                            a.first_pair[s] = mine;
                        }
                    }
                    if (c == a.n_candidates - 1) {
                        for (uint32_t s = system + 1; s <= a.n_systems; s++) {
                            a.first_pair[s] = total;
                        }
                    }
                }
                if (keep && fits) {
                    a.out.pairs[2 * mine + 0] = gi - first_point;
                    a.out.pairs[2 * mine + 1] = gj - first_point;
                    if (a.out.shifts != nullptr) {
                        a.out.shifts[3 * mine + 0] = sx;
                        a.out.shifts[3 * mine + 1] = sy;
                        a.out.shifts[3 * mine + 2] = sz;
                    }
                    if (a.out.distances != nullptr) {
                        a.out.distances[mine] = sqrt(dd);
                    }
                    if (a.out.vectors != nullptr) {
                        a.out.vectors[3 * mine + 0] = vx;
                        a.out.vectors[3 * mine + 1] = vy;
                        a.out.vectors[3 * mine + 2] = vz;
                    }
                }
                row += static_cast<uint64_t>(__popcll(mask));
            } else {
                chunk_rows += static_cast<uint32_t>(__popcll(mask));
            }
        }
        if (!WRITE && lane == 0) {
            a.chunk_rows[chunk] = chunk_rows;
        }
    }
}

} // namespace vesin_hip

#endif
