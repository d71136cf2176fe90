// Host driver of the HIP neighbor-list path: owns the device work buffers kept in VesinNeighborList::opaque,
// picks the grid, launches the kernel sequence on the null stream and sizes the outputs exactly (count pass ->
// device-wide scan -> write pass), so no capacity guess and no overflow flag are needed.
//
// Reference role replaced: vesin::cuda::neighbors / allocate_output_buffers / finalize_output / free_neighbors
// (vesin/src/vesin_cuda.cpp:819-923, :293-345, :783-817, :129-138) and the RAII buffers of
// vesin/src/cuda_buffers.cpp.
#include <hip/hip_runtime.h>

#include <ucontext.h>

#include <cerrno>
#include <cmath>
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <type_traits>

#include <algorithm>
#include <atomic>
#include <exception>
#include <functional>
#include <stdexcept>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "backward.cuh"
#include "cells.cuh"
#include "device_common.cuh"
#include "driver.hpp"
#include "fused.cuh"
#include "geometry.hpp"
#include "images.cuh"
#include "molecules.cuh"
#include "ordered.cuh"
#include "small.cuh"
#include "policy.hpp"
#include "scan.cuh"
#include "search.cuh"
#include "sort.cuh"
#include "verlet.cuh"

namespace vesin_hip {

#define HIP_CHECK(expr)                                                                                              \
    do {                                                                                                             \
        hipError_t status_ = (expr);                                                                                 \
        if (status_ != hipSuccess) {                                                                                 \
            throw std::runtime_error(std::string("HIP error in ") + #expr + ": " + hipGetErrorString(status_));      \
        }                                                                                                            \
    } while (false)

// Named ranges on a profiler's timeline (rocprofv3 --marker-trace), around the stages that VesinHipTimings names.
// Compiled in with -DVESIN_HIP_ROCTX (python -m vesin_amd._build with VESIN_HIP_ROCTX=1) and absent otherwise: the
// counterpart of the reference's optional NVTX ranges (vesin/src/vesin_cuda.cpp:16-28). A range covers the host
// side of a stage, i.e. the launches; the kernels it launched follow on the stream's own line of the timeline.
#ifdef VESIN_HIP_ROCTX
#include <rocprofiler-sdk-roctx/roctx.h>
struct TraceRange {
    explicit TraceRange(const char* name) { roctxRangePush(name); }
    ~TraceRange() { roctxRangePop(); }
    /// Ends the stage that is open and starts the next one.
    void next(const char* name) {
        roctxRangePop();
        roctxRangePush(name);
    }
    TraceRange(const TraceRange&) = delete;
    TraceRange& operator=(const TraceRange&) = delete;
};
#else
struct TraceRange {
    explicit TraceRange(const char*) {}
    void next(const char*) {}
};
#endif

#ifdef VESIN_HIP_HOST_PROFILE
// developer's instrumentation: where the host's time of a call goes (printed every 1000 calls)
#include <time.h>
struct HostProfile {
    double sums[8] = {};
    long calls = 0;
    double last = 0;
    static double now() { timespec t; clock_gettime(CLOCK_MONOTONIC, &t); return t.tv_sec * 1e6 + t.tv_nsec * 1e-3; }
    void begin() { last = now(); }
    void lap(int k) { const double t = now(); sums[k] += t - last; last = t; }
    void end() {
        calls += 1;
        if (calls % 1000 == 0) {
            std::fprintf(stderr, "host profile (us per call): checks %.2f state %.2f setup %.2f launch %.2f wait %.2f after %.2f\n",
                         sums[0] / 1000, sums[1] / 1000, sums[2] / 1000, sums[3] / 1000, sums[4] / 1000, sums[5] / 1000);
            for (double& s : sums) s = 0;
        }
    }
};
static thread_local HostProfile HOST_PROFILE;
#define HOST_LAP(k) HOST_PROFILE.lap(k)
#else
#define HOST_LAP(k) do {} while (false)
#endif

static std::atomic<bool> TIMINGS_ENABLED{false};

void enable_timings(bool enabled) {
    TIMINGS_ENABLED.store(enabled);
}

/// VESIN_HIP_ROWS=ordered makes the single-pass search place the rows in work-item order (identical from run to
/// run) instead of order of arrival. Measured: a fifth more time per call on an even system (1,000,000-atom
/// lattice: the search kernel 6 %, the reproducible cell build the rest), more than twice the time on a clustered
/// one, where every workgroup ends up waiting for all earlier ones.
static bool ordered_rows() {
    const char* text = std::getenv("VESIN_HIP_ROWS");
    return text != nullptr && std::strcmp(text, "ordered") == 0;
}

/// VESIN_HIP_CHAIN_SPINS=<n> bounds the polls a wave of the single-pass search makes while it waits for another
/// workgroup's rows (ordered placement). 0 makes every wait give up at once, which is how the tests reach the
/// fallback that follows without any kernel having to hang for it.
static uint32_t chain_spin_limit() {
    const char* text = std::getenv("VESIN_HIP_CHAIN_SPINS");
    if (text == nullptr || *text == '\0') {
        return CHAIN_SPIN_LIMIT;
    }
    char* end = nullptr;
    const unsigned long parsed = std::strtoul(text, &end, 10);
    if (*end != '\0' || parsed > CHAIN_SPIN_LIMIT) {
        return CHAIN_SPIN_LIMIT;
    }
    return static_cast<uint32_t>(parsed);
}

/// VESIN_HIP_CHAIN_WAIT_US=<n> is the time such a wave waits at most, in microseconds (2000 unless set; for
/// measurements).
static uint32_t chain_wait_ticks() {
    const char* text = std::getenv("VESIN_HIP_CHAIN_WAIT_US");
    if (text == nullptr || *text == '\0') {
        return CHAIN_WAIT_TICKS;
    }
    char* end = nullptr;
    const unsigned long parsed = std::strtoul(text, &end, 10);
    if (*end != '\0' || parsed > 1000000ul) {
        return CHAIN_WAIT_TICKS;
    }
    return static_cast<uint32_t>(parsed * 100ul); // the clock runs at 100 MHz
}

/// VESIN_HIP_SEARCH=two-pass keeps every call on the count / scan / write sequence (for comparisons and tests).
static bool two_pass_only() {
    const char* text = std::getenv("VESIN_HIP_SEARCH");
    return text != nullptr && std::strcmp(text, "two-pass") == 0;
}

/// Cells of the upper half of the stencil (the centre cell and what follows it in the kernels' order) that can hold
/// a neighbour: what a tile's candidates are drawn from.
static double upper_stencil_cells(const GridParams& g) {
    if (g.prune == 0) {
        return 0.5 * ((2.0 * g.s[0] + 1.0) * (2.0 * g.s[1] + 1.0) * (2.0 * g.s[2] + 1.0) + 1.0);
    }
    uint32_t kept = 0;
    for (int32_t dx = 0; dx <= g.s[0]; dx++) {
        for (int32_t dy = (dx == 0 ? 0 : -g.s[1]); dy <= g.s[1]; dy++) {
            for (int32_t dz = (dx == 0 && dy == 0 ? 0 : -g.s[2]); dz <= g.s[2]; dz++) {
                kept += stencil_entry_too_far(g, dx, dy, dz) ? 0 : 1;
            }
        }
    }
    return static_cast<double>(kept);
}

/// VESIN_HIP_STENCIL=full searches every cell of a stencil, also those that cannot hold a neighbour (for comparisons
/// and tests).
static bool full_stencil_only() {
    const char* text = std::getenv("VESIN_HIP_STENCIL");
    return text != nullptr && std::strcmp(text, "full") == 0;
}

/// VESIN_HIP_TESTS=double keeps the distance tests of the searches in double precision throughout (for comparisons
/// and tests), instead of deciding all pairs but those next to the cutoff in single precision first.
static bool double_precision_only() {
    const char* text = std::getenv("VESIN_HIP_TESTS");
    return text != nullptr && std::strcmp(text, "double") == 0;
}

/// VESIN_HIP_CELLS=packed keeps every call on the counting-sort cell build (for comparisons and tests) instead of
/// the one-pass build with a fixed number of slots per cell that the single-pass search can read.
static bool packed_cells_only() {
    const char* text = std::getenv("VESIN_HIP_CELLS");
    return text != nullptr && std::strcmp(text, "packed") == 0;
}

/// VESIN_HIP_SORT=radix keeps sorted lists on the unsorted search followed by the radix sort (for comparisons and
/// tests) instead of the search that produces them in order.
static bool radix_sort_only() {
    const char* text = std::getenv("VESIN_HIP_SORT");
    return text != nullptr && std::strcmp(text, "radix") == 0;
}

/// VESIN_HIP_LAUNCHES=separate keeps the passes of a small system's search in launches of their own (for comparisons
/// and tests) instead of one launch whose workgroups wait for each other between the passes.
static bool separate_launches() {
    const char* text = std::getenv("VESIN_HIP_LAUNCHES");
    return text != nullptr && std::strcmp(text, "separate") == 0;
}

/// VESIN_HIP_EXTENT=fresh makes every call on a larger system with a non-periodic direction find the extent of its
/// points before it picks the grid (for comparisons and tests), instead of starting from the extent of the call before.
static bool fresh_extent_only() {
    const char* text = std::getenv("VESIN_HIP_EXTENT");
    return text != nullptr && std::strcmp(text, "fresh") == 0;
}

/// VESIN_HIP_STREAMS=one keeps every kernel of a call on the call's stream (for comparisons and tests); otherwise the
/// in-order search orders the candidates of the tiles on a second stream while it counts the rows.
static bool ordered_one_stream() {
    const char* text = std::getenv("VESIN_HIP_STREAMS");
    return text != nullptr && std::strcmp(text, "one") == 0;
}

namespace {

__global__ void publish_ordered_status(
    const OrderedStatus* found, const uint64_t* total, const DeviceStatus* status, const uint64_t* cell_scan_end,
    OrderedHostStatus* host
) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        host->found = *found;
        host->total_rows = *total;
        host->first_bad_coordinate = status->first_bad_coordinate;
        host->n_tiles = static_cast<unsigned int>(*cell_scan_end >> 32);
    }
}

/// Whether the boxes and flags of a batch are, bit for bit, the ones its grids were picked from (kept on the device):
/// a workgroup that finds a difference says so in the word the host reads (which the host cleared before the launch).
__global__ __launch_bounds__(BLOCK) void compare_boxes_kernel(
    const unsigned long long* __restrict__ boxes, const unsigned char* __restrict__ periodic,
    const unsigned long long* __restrict__ kept_boxes, const unsigned char* __restrict__ kept_periodic,
    size_t n_box_words, size_t n_flags, unsigned int* changed
) {
    bool differs = false;
    const size_t stride = static_cast<size_t>(gridDim.x) * BLOCK;
    for (size_t k = static_cast<size_t>(blockIdx.x) * BLOCK + threadIdx.x; k < n_box_words; k += stride) {
        differs = differs || boxes[k] != kept_boxes[k];
    }
    for (size_t k = static_cast<size_t>(blockIdx.x) * BLOCK + threadIdx.x; k < n_flags; k += stride) {
        differs = differs || (periodic[k] != 0) != (kept_periodic[k] != 0);
    }
    if (differs) {
        *changed = 1u;
    }
}

/// Everything the kernels report to the host, in one block. A list's own block is pinned host memory that the
/// kernels write into directly; the entry point that allocates nothing keeps the block in device memory and copies
/// it to the host before every wait (see HipExtras::wait).
struct Mailbox {
    // what every wait reads
    DeviceStatus status;
    FusedStatus fused;
    OrderedHostStatus ordered;
    unsigned char small[128];            // box (72 bytes) + periodic (3 bytes)
    unsigned int batch_changed;          // a batch that started from the boxes of the call before: they are others now
    unsigned int padding;
    unsigned long long batch_total_cells; // a batch whose grids were picked on the device: all its cells
    // what only some do
    BlockBounds bounds[BOUNDING_BLOCKS]; // one slot per workgroup of the bounding pass
    ShiftRange ranges[SHIFT_RANGE_BLOCKS]; // one slot per workgroup of the sort's range pass
};

/// Makes `device` current for a scope and gives the caller's device back afterwards.
struct DeviceGuard {
    int previous = -1;
    int wanted;

    explicit DeviceGuard(int device): wanted(device) {
        if (hipGetDevice(&previous) != hipSuccess) {
            (void)hipGetLastError();
            previous = -1;
        }
        if (previous != wanted) {
            HIP_CHECK(hipSetDevice(wanted));
        }
    }

    ~DeviceGuard() {
        if (previous >= 0 && previous != wanted) {
            (void)hipSetDevice(previous);
        }
    }

    DeviceGuard(const DeviceGuard&) = delete;
    DeviceGuard& operator=(const DeviceGuard&) = delete;
};

/// Grow-only device allocation.
struct DeviceBuffer {
    void* ptr = nullptr;
    size_t bytes = 0;
    uint64_t generation = 0; // counts the allocations: what was written into an earlier one is gone
    bool fixed = false;      // memory that is not this buffer's to free or to grow (the entry point that allocates nothing)

    void reserve(size_t wanted) {
        if (wanted <= bytes) {
            return;
        }
        if (fixed) {
            throw std::runtime_error(
                "this calculation needs " + std::to_string(wanted) + " bytes of work memory, the entry point that "
                "allocates nothing holds " + std::to_string(bytes) + ": use vesin_neighbors for it"
            );
        }
        release();
        size_t padded = wanted + wanted / 4;
        HIP_CHECK(hipMalloc(&ptr, padded));
        bytes = padded;
        generation += 1;
    }

    void release() {
        if (ptr != nullptr && !fixed) {
            (void)hipFree(ptr);
            ptr = nullptr;
            bytes = 0;
        }
    }
};

/// Hands out 256-byte aligned pieces of one allocation; first pass (base == nullptr) only measures.
struct Carver {
    char* base;
    size_t used = 0;

    explicit Carver(void* start): base(static_cast<char*>(start)) {}

    template <typename T>
    T* take(size_t count) {
        size_t at = used;
        used += (count * sizeof(T) + 255) & ~static_cast<size_t>(255);
        return base == nullptr ? nullptr : reinterpret_cast<T*>(base + at);
    }
};

/// Calls that find the extent of their points first after one that started from the extent of the call before and
/// found its points somewhere else.
constexpr int EXTENT_REST = 8;

/// Candidates beyond which a cached list is not worth filtering: the direct search writes its rows at more than
/// half the memory bandwidth, and a filter has to read every candidate, twice, on top of writing the same rows.
/// Measured on jittered diamond (cutoff 5, skin 0.5, i j S d), filter against direct search: 0.2 M candidates 0.055 /
/// 0.074 ms, 1.6 M 0.074 / 0.102 ms, 5.5 M 0.212 / 0.167 ms, 13 M 0.430 / 0.272 ms. A sorted list costs the direct
/// search more and the filter nothing (sorted candidates stay sorted): 1.6 M candidates 0.072 / 0.162 ms, 5.5 M
/// 0.213 / 0.274 ms, 13 M 0.433 / 0.424 ms, 31 M 0.973 / 0.854 ms.
constexpr size_t VERLET_MAX_CANDIDATES = size_t(1) << 21;
constexpr size_t VERLET_MAX_CANDIDATES_SORTED = size_t(1) << 23;

/// One-pass cell build: slots per cell (one tile: with two the search has as many empty tiles as full ones and
/// loses more than the build gains) and the mean occupations between which it is tried. A cell that overflows voids
/// the call's result (the packed build and the two passes start over) and the list stays away from it for long.
/// The build saves two launches and a pass over the points; what it costs grows with the number of cells, whose 32
/// slots each are cleared (wrap shifts) and visited by a wave of the search whether filled or not. Per call, cutoff
/// 5, full lists, packed build -> one-pass build: 3.8 points per cell, 10,000 / 100,000 / 300,000 / 1,000,000 atoms
/// 55 -> 47, 131 -> 126, 319 -> 318, 937 -> 938 us; 6.3 points per cell, 10,000 / 30,000 / 100,000 / 1,000,000
/// atoms 58 -> 52, 69 -> 60, 115 -> 109, 641 -> 613 us; 2.5 points per cell, 3,000 / 10,000 / 30,000 / 100,000 atoms
/// 44 -> 39, 56 -> 49, 80 -> 78, 166 -> 172 us. The entry point that allocates nothing keeps the higher minimum: the
/// layout takes 32 slots of memory per cell.
constexpr uint32_t DIRECT_CAPACITY = TILE_POINTS;
constexpr double DIRECT_MEAN_MIN = 5.0;              // any number of cells
constexpr double DIRECT_MEAN_MIN_SOME_CELLS = 3.0;   // at most DIRECT_SOME_CELLS cells
constexpr size_t DIRECT_SOME_CELLS = 65536;
constexpr double DIRECT_MEAN_MIN_FEW_CELLS = 2.0;    // at most DIRECT_FEW_CELLS cells
constexpr size_t DIRECT_FEW_CELLS = 16384;
constexpr double DIRECT_MEAN_MIN_FIXED_MEMORY = 10.0;
constexpr double DIRECT_MEAN_MAX = 24.0;
constexpr int DIRECT_REST = 1024;

constexpr int SINGLE_PASS_REST = 64;
constexpr size_t BOX_BYTES = 75; // 9 doubles and 3 flags, as fetch_box lays them out
constexpr size_t BOX_BYTES_PADDED = 80;

enum Stage { T_START = 0, T_CELLS, T_COUNT, T_SCAN, T_WRITE_BEGIN, T_WRITE, T_SORT, T_STAGES };

/// Candidate list of a Verlet-cached calculation (options.skin > 0) and what it was built from; the counterpart
/// of the reference's VerletList / VerletCache (vesin/src/verlet.hpp:19-95, vesin/src/verlet_cuda.hpp).
struct VerletCache {
    VesinNeighborList candidates = VesinNeighborList(); // full lists of this library, with a private state of its own
    double* ref_points = nullptr;                       // device: the points the candidates were built from
    size_t ref_capacity = 0;
    size_t n_ref = 0;
    VerletReference* reference = nullptr; // device: box and periodicity of that call
    VerletStatus* status = nullptr;       // pinned
    VesinOptions options = {};
    bool valid = false;
    /// Lists too long for a filter to pay are searched directly on every call (see verlet_neighbors); the
    /// estimate is revised with every call's row count.
    bool direct = false;
    size_t direct_n_points = 0;
    CandidateLifetime lifetime; // ... and so are lists whose candidates keep getting outdated after a few calls

    VerletCache() = default;
    VerletCache(const VerletCache&) = delete;
    VerletCache& operator=(const VerletCache&) = delete;

    ~VerletCache() {
        if (candidates.device.type == VesinCUDA) {
            free_neighbors(candidates);
        }
        if (ref_points != nullptr) {
            (void)hipFree(ref_points);
        }
        if (reference != nullptr) {
            (void)hipFree(reference);
        }
        if (status != nullptr) {
            (void)hipHostFree(status);
        }
    }
};

/// Private state of one VesinNeighborList (VesinNeighborList::opaque).
/// What the host derives from the boxes of a batch of systems, kept between calls: a batch whose boxes, flags and
/// division into systems are those of the call before (a trajectory at constant volume, the same set of structures
/// evaluated again) starts its kernels without the host going over the systems one by one again.
/// Host memory the GPU copies from and to directly (hipHostMalloc): a copy between device memory and an ordinary
/// std::vector goes through a staging buffer of the runtime's and waits for it, several times per batch.
template <typename T>
struct PinnedAllocator {
    using value_type = T;
    PinnedAllocator() = default;
    template <typename U>
    PinnedAllocator(const PinnedAllocator<U>&) {}
    T* allocate(size_t n) {
        void* ptr = nullptr;
        if (hipHostMalloc(&ptr, n * sizeof(T), hipHostMallocDefault) != hipSuccess) {
            (void)hipGetLastError();
            throw std::bad_alloc();
        }
        return static_cast<T*>(ptr);
    }
    void deallocate(T* ptr, size_t) {
        (void)hipHostFree(ptr);
    }
    template <typename U>
    bool operator==(const PinnedAllocator<U>&) const {
        return true;
    }
    template <typename U>
    bool operator!=(const PinnedAllocator<U>&) const {
        return false;
    }
};

template <typename T>
using PinnedVector = std::vector<T, PinnedAllocator<T>>;

/// The host's loops over the systems of a batch (a box to normalise, a grid to pick: about 85 ns per system, which
/// is 1.7 ms of a 2.6 ms call for 20,000 small crystals that are not those of the call before) on several threads once
/// there are enough systems: `work(begin, end, part)` for consecutive ranges, one per thread. The first error in the
/// order of the systems is the one that comes out.
template <typename Work>
void over_the_systems(size_t n_systems, size_t n_parts, Work&& work) {
    if (n_parts <= 1) {
        work(size_t(0), n_systems, size_t(0));
        return;
    }
    std::vector<std::exception_ptr> errors(n_parts);
    std::vector<std::thread> threads;
    threads.reserve(n_parts - 1);
    auto run = [&](size_t part) {
        const size_t begin = n_systems * part / n_parts;
        const size_t end = n_systems * (part + 1) / n_parts;
        try {
            work(begin, end, part);
        } catch (...) {
            errors[part] = std::current_exception();
        }
    };
    try {
        for (size_t part = 1; part < n_parts; part++) {
            threads.emplace_back(run, part);
        }
    } catch (...) {
        // (no more threads to be had: the parts without one are done here)
        for (size_t part = threads.size() + 1; part < n_parts; part++) {
            run(part);
        }
    }
    run(0);
    for (std::thread& thread : threads) {
        thread.join();
    }
    for (const std::exception_ptr& error : errors) {
        if (error != nullptr) {
            std::rethrow_exception(error);
        }
    }
}

/// Threads for these loops: one per 2048 systems, eight at most, never more than the machine has.
inline size_t parts_for_systems(size_t n_systems) {
    const size_t available = std::max<size_t>(1, std::thread::hardware_concurrency());
    return std::max<size_t>(1, std::min<size_t>({size_t(8), available, n_systems / 2048}));
}

/// VerletCache for a batch of systems (vesin_hip_neighbors_batch with options.skin > 0): the candidates are the rows
/// of a batch call at cutoff + skin, kept with the division into systems and the points and boxes they came from.
struct BatchVerletCache {
    VesinNeighborList candidates = VesinNeighborList();
    std::vector<size_t> first_point;          // the division into systems the candidates were built for
    std::vector<size_t> candidate_first_pair; // where every system's candidates begin
    DeviceBuffer kept;                        // what lives as long as the candidates (see rebuild)
    DeviceBuffer scratch;                     // what a filtering call needs
    double* ref_points = nullptr;
    BatchVerletReference* reference = nullptr;
    uint32_t* system_of_point = nullptr;
    BatchVerletCandidate* packed = nullptr;   // the candidates as the filter reads them
    unsigned long long* d_first_point = nullptr;
    VerletStatus* status = nullptr;           // pinned
    PinnedVector<unsigned long long> first_pair_landing;
    VesinOptions options = {};
    bool valid = false;
    bool direct = false;                      // as in VerletCache
    size_t direct_n_points = 0;
    int unpackable_rest = 0;                  // calls left before candidates are tried again after shifts they cannot hold
    CandidateLifetime lifetime;               // as in VerletCache

    BatchVerletCache() = default;
    BatchVerletCache(const BatchVerletCache&) = delete;
    BatchVerletCache& operator=(const BatchVerletCache&) = delete;

    void drop_candidates() {
        if (candidates.device.type == VesinCUDA) {
            free_neighbors(candidates);
        }
        candidates = VesinNeighborList();
        valid = false;
    }

    ~BatchVerletCache() {
        drop_candidates();
        kept.release();
        scratch.release();
        if (status != nullptr) {
            (void)hipHostFree(status);
        }
    }
};

/// The systems of a batch are small, and a small system of several cells is many tiles of a few points each: every
/// tile costs a wave its fixed work (tables, staging), and the sorted search over tiles needs a record block per
/// tile. One cell means brute force over points x points x images pairs, which is cheap while that product is small,
/// and the search over images (images.cuh) writes sorted rows of such systems in order. Under the automatic choice
/// of the algorithm a system of a batch is therefore given one cell not only below 32 points but whenever the tests
/// stay few: up to 256 points without images (free molecules: 20,000 molecules of 3 to 40 atoms 0.75 -> 0.29 ms per
/// unsorted batch, 1.16 -> 0.46 ms sorted), up to 69 points with the 27 images of a box wider than the cutoff.
constexpr uint64_t ONE_CELL_TESTS = 131072; // points x points x images
inline bool one_cell_in_a_batch(uint64_t n_points, uint64_t n_images) {
    return n_points <= IMAGE_MAX_POINTS && n_images <= IMAGE_MAX_ENTRIES && n_points * n_points * n_images <= ONE_CELL_TESTS;
}

struct BatchSetup {
    bool valid = false;
    bool any_open_direction = false;
    bool all_open = false;                  // no system has a periodic direction: the boxes count for nothing
    uint64_t cells_bound = 0;               // most cells the grids of these systems can have, whatever their points
    double cutoff = 0.0;
    int algorithm = 0;
    bool full_stencil = false;              // VESIN_HIP_STENCIL=full was set
    // (what is copied from or to the device lives in pinned memory)
    PinnedVector<double> boxes;              // 9 per system, as the caller gave them
    PinnedVector<unsigned char> periodic;    // 3 per system
    PinnedVector<double> incoming_boxes;     // where a call's boxes land before they are compared
    PinnedVector<unsigned char> incoming_periodic;
    std::vector<size_t> first_point;
    std::vector<HostBox> host_boxes;        // normalised
    PinnedVector<GridParams> grids;
    PinnedVector<uint32_t> cell_base;
    PinnedVector<uint32_t> first_point32;
    PinnedVector<BlockBounds> bounds;        // extent of every system's points (systems with an open direction)
    uint64_t total_cells = 0;
    double most_units = 1.0;
    // where the last batch left grids, first points and first cells in the work buffer; a call on a single system
    // carves the same buffer its own way and clears the flag
    bool on_device = false;
    const void* d_grids = nullptr;
    const void* d_first_point = nullptr;
    const void* d_cell_base = nullptr;
    uint64_t work_generation = 0;
    // The boxes and flags the grids were picked from, on the device (9 doubles per system, then 3 bytes per system):
    // a call may start from the grids it has and let a kernel compare this call's boxes with them, instead of
    // bringing 75 bytes per system to the host and waiting for them before anything can be launched.
    DeviceBuffer kept_boxes;
    bool kept_on_device = false;
    BoxGuess guess;
    // The single-pass search of a batch places its rows through the chain of workgroups: after a launch whose waves
    // gave up waiting, reused lists go straight to the two passes for a while.
    WaitRest chain_rest;
    // Sorted lists come straight from a search that writes the rows in order where the systems have the shape for
    // it; after a batch that did not, the next calls go to the two passes and the sort without asking again.
    int in_order_rest = 0;
    size_t systems_for_images = 0;          // systems the search over images covers (grids picked on the host)
    size_t systems_for_tiles = 0;           // other systems whose stencil fits the in-order search over tiles
    size_t systems_with_points = 0;
    size_t most_points = 0;                 // of one system
    PinnedVector<uint64_t> pair_base;       // pairs of points (n^2 per system of few points) before every system
    uint32_t image_words = 1;               // words of 64 images per pair of points, the most any system needs
    const void* d_pair_base = nullptr;
    // where the first rows of the systems land before they are copied into the caller's array (pinned)
    size_t* first_pair_landing = nullptr;
    size_t first_pair_capacity = 0;
    // batches of free molecules (molecules.cuh): work memory of their own (what the general path keeps in the list's
    // work memory between calls stays as it is), the division into systems on the device, the kernels' report
    DeviceBuffer molecule_work;
    std::vector<size_t> molecule_first_point;      // the division into systems whose 32-bit copy is in `molecule_work`
    PinnedVector<uint32_t> molecule_first_point32; // (where the copy to the device starts from)
    bool molecule_first_point_on_device = false;
    MoleculeStatus* molecule_report = nullptr; // pinned
};

/// A call that stops where the host would wait for the GPU and goes on later (vesin_hip_neighbors_enqueue /
/// vesin_hip_neighbors_collect). The call runs on a stack of its own: where it first has to wait for the stream
/// (HipExtras::wait), control goes back to whoever started it, with everything up to there queued; resumed, it waits
/// and carries on as the blocking call would have, every decision and every way back included. Nothing that is
/// bound to a host thread is held across the stop (no lock, no exception in flight), so the call may be resumed by
/// another thread.
struct SuspendedCall {
    static constexpr size_t STACK_BYTES = size_t(1) << 20;

    ucontext_t starter = {};
    ucontext_t call = {};
    std::unique_ptr<unsigned char[]> stack;
    std::function<void()> body;
    std::exception_ptr error;
    bool stop_at_next_wait = false;
    bool finished = true;
    hipEvent_t reached = nullptr; // recorded where the call stopped: resuming waits for that, not for what the caller
                                  // queued behind it

    SuspendedCall() = default;
    SuspendedCall(const SuspendedCall&) = delete;
    SuspendedCall& operator=(const SuspendedCall&) = delete;

    ~SuspendedCall() {
        if (reached != nullptr) {
            (void)hipEventDestroy(reached);
        }
    }

    static void entry(unsigned int low, unsigned int high) {
        auto* self = reinterpret_cast<SuspendedCall*>((static_cast<uintptr_t>(high) << 32) | static_cast<uintptr_t>(low));
        try {
            self->body();
        } catch (...) {
            self->error = std::current_exception();
        }
        self->finished = true;
        // (back to the starter through uc_link)
    }

    /// Runs `work` until it stops at its first wait or ends.
    void start(std::function<void()> work) {
        if (stack == nullptr) {
            stack.reset(new unsigned char[STACK_BYTES]);
        }
        if (reached == nullptr) {
            HIP_CHECK(hipEventCreateWithFlags(&reached, hipEventDisableTiming));
        }
        body = std::move(work);
        error = nullptr;
        finished = false;
        stop_at_next_wait = true;
        if (getcontext(&call) != 0) {
            throw std::runtime_error("getcontext failed");
        }
        call.uc_stack.ss_sp = stack.get();
        call.uc_stack.ss_size = STACK_BYTES;
        call.uc_link = &starter;
        const uintptr_t self = reinterpret_cast<uintptr_t>(this);
        makecontext(
            &call, reinterpret_cast<void (*)()>(&SuspendedCall::entry), 2, static_cast<unsigned int>(self & 0xFFFFFFFFu),
            static_cast<unsigned int>(self >> 32)
        );
        resume();
    }

    /// Carries on until the call stops again or ends.
    void resume() {
        if (swapcontext(&starter, &call) != 0) {
            throw std::runtime_error("swapcontext failed");
        }
    }

    /// From inside the call: back to whoever started or resumed it.
    void stop() {
        if (swapcontext(&call, &starter) != 0) {
            throw std::runtime_error("swapcontext failed");
        }
    }
};

/// The value of the device word of a queued call (see vesin_hip_neighbors_enqueue) while the rows are not known to
/// be complete.
constexpr unsigned long long ROWS_PENDING = ~0ull;

/// What tells, on the device, whether the kernels queued by a call left the complete list in the arrays.
struct QueuedOutcome {
    int kind;                          // 0: single-pass search, 1: small system in one launch, 2: in-order search,
                                       // 3: kept candidates filtered (options.skin > 0)
    const VerletStatus* filtered;      // (3) pinned host memory
    const FusedStatus* fused;          // (0)
    const DeviceStatus* build;         // (0, 2)
    const OrderedHostStatus* small;    // (1) what workgroup 0 of the launch reported
    const OrderedStatus* ordered;      // (2)
    const uint64_t* ordered_total;     // (2)
    unsigned long long capacity;       // rows the arrays hold
    unsigned long long row_limit;      // more rows than this are an error of the caller's making (0: no limit)
    int one_pass_cells;                // (0) the cells were built with a fixed number of slots each
    int guessed_extent;                // (0) the grid came from the extent of the call before
    unsigned char used_box[BOX_BYTES_PADDED]; // the box and flags the host picked the grid from
};

/// Last kernel of the queued part of a call: the device word gets the number of rows if the list is complete in the
/// arrays, which is the case when the kernels before found what the host is going to check once it looks (the same
/// conditions, in the same words), and stays ROWS_PENDING otherwise.
__global__ void publish_queued_length(
    QueuedOutcome outcome, const double* __restrict__ box, const bool* __restrict__ periodic, unsigned long long* word
) {
    if (threadIdx.x != 0 || blockIdx.x != 0) {
        return;
    }
    if (outcome.kind == 3) {
        // (the check that ran with the filter compared this call's box and points with those of the candidates)
        const unsigned long long rows = outcome.filtered->total_rows;
        const bool complete = outcome.filtered->rebuild == 0 && rows <= outcome.capacity &&
                              (outcome.row_limit == 0 || rows <= outcome.row_limit);
        *word = complete ? rows : ROWS_PENDING;
        return;
    }
    bool complete = true;
    for (int k = 0; k < 9; k++) {
        double used;
        memcpy(&used, outcome.used_box + 8 * k, 8);
        unsigned long long a, b;
        memcpy(&a, &used, 8);
        const double now = box[k];
        memcpy(&b, &now, 8);
        complete = complete && a == b;
    }
    for (int d = 0; d < 3; d++) {
        complete = complete && (outcome.used_box[72 + d] != 0) == periodic[d];
    }
    unsigned long long rows = 0;
    if (outcome.kind == 0) {
        const FusedStatus found = *outcome.fused;
        rows = found.total_rows;
        complete = complete && found.general == 0 && found.overflow == 0 && found.chain_timeout == 0 && found.deferred == 0 &&
                   outcome.build->first_bad_coordinate == 0xFFFFFFFFu &&
                   (outcome.one_pass_cells == 0 || outcome.build->crowded_cells == 0) &&
                   (outcome.guessed_extent == 0 || outcome.build->far_outside == 0);
    } else if (outcome.kind == 1) {
        const OrderedHostStatus report = *outcome.small;
        rows = report.total_rows;
        complete = complete && report.found.gave_up == 0 && report.found.max_rows <= ORDERED_MAX_ROWS &&
                   report.found.max_candidates <= ORDERED_CANDIDATES && report.found.unsuitable == 0 &&
                   report.first_bad_coordinate == 0xFFFFFFFFu && rows <= outcome.capacity;
    } else {
        const OrderedStatus found = *outcome.ordered;
        rows = *outcome.ordered_total;
        complete = complete && found.max_rows <= ORDERED_MAX_ROWS && found.max_candidates <= ORDERED_CANDIDATES &&
                   found.unsuitable == 0 && outcome.build->first_bad_coordinate == 0xFFFFFFFFu && rows <= outcome.capacity;
    }
    if (outcome.row_limit != 0 && rows > outcome.row_limit) {
        complete = false;
    }
    *word = complete ? rows : ROWS_PENDING;
}

/// publish_queued_length for a batch through the single-pass search: the list is complete in the arrays when the
/// search found nothing it could not handle and, for a call that started from the grids of the call before, the
/// boxes turned out to be the same (and the cells of grids picked on the device fit their room): what the host checks
/// after its wait, in the same words.
__global__ void publish_queued_batch_length(
    const Mailbox* mail, int speculated, int device_grids, unsigned long long total_cells, unsigned long long row_limit,
    unsigned long long* word
) {
    if (threadIdx.x != 0 || blockIdx.x != 0) {
        return;
    }
    const FusedStatus found = mail->fused;
    bool complete = found.first_bad_coordinate == 0xFFFFFFFFu && found.general == 0 && found.deferred == 0 &&
                    found.overflow == 0 && found.chain_timeout == 0;
    if (speculated != 0) {
        complete = complete && mail->batch_changed == 0 && (device_grids == 0 || mail->batch_total_cells <= total_cells);
    }
    if (row_limit != 0 && found.total_rows > row_limit) {
        complete = false;
    }
    *word = complete ? found.total_rows : ROWS_PENDING;
}

/// The same for a batch of free molecules: `status` is what the kernels gathered, `total_rows` the end of the scan over
/// the systems' rows.
__global__ void publish_queued_molecules_length(
    const MoleculeStatus* status, const unsigned long long* total_rows, unsigned long long capacity,
    unsigned long long row_limit, unsigned long long* word
) {
    if (threadIdx.x != 0 || blockIdx.x != 0) {
        return;
    }
    const unsigned long long rows = *total_rows;
    const bool complete = status->periodic == 0 && status->first_bad == 0xFFFFFFFFu && rows <= capacity &&
                          (row_limit == 0 || rows <= row_limit);
    *word = complete ? rows : ROWS_PENDING;
}

__global__ void set_queued_length(unsigned long long* word, unsigned long long value) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        *word = value;
    }
}

struct HipExtras {
    int device_id = 0;
    BatchSetup batch;
    DeviceBuffer work;
    DeviceBuffer sort_work;
    DeviceStatus* d_status = nullptr;
    Mailbox* mail = nullptr;          // what the host reads after a wait
    Mailbox* mail_device = nullptr;   // what the kernels write: the same pinned block, or device memory
    /// The entry point that allocates nothing: work memory, status block and mailbox are pieces of a fixed device
    /// array, the output arrays are the caller's, and nothing of it is ever freed or grown.
    bool fixed_memory = false;
    size_t capacity = 0;              // rows every allocated output array can hold
    /// Where the output arrays come from and go back to when the caller said so (vesin_hip_set_output_allocator);
    /// hipMalloc and hipFree otherwise.
    VesinHipAllocate allocate = nullptr;
    VesinHipRelease release = nullptr;
    void* allocator_context = nullptr;
    unsigned char last_box[BOX_BYTES] = {}; // box and periodicity of the last call that read them
    BoxGuess guess;                   // when a call starts from that box without reading this call's first
    int single_pass_rest = 0;         // calls left before the single-pass search is tried again after it did not fit
    int direct_rest = 0;              // calls left before the one-pass cell build is tried again after a cell overflowed
    int in_order_rest = 0;            // calls left before the in-order search is tried again on a system it did not cover
    int one_launch_rest = 0;          // calls left before a small system is tried in one launch again
    WaitRest meeting_rest;            // ... after workgroups of that launch gave up waiting for the others
    WaitRest chain_rest;              // the same for the chain of the single-pass search (rows in work-item order)
    uint32_t ordered_tiles = 0;       // tiles of the last call through the in-order search, and its number of points:
    size_t ordered_tiles_points = 0;  // how the next one deals its writing pass to the waves (see write_split)
    /// Extent of the points along the directions that are not periodic, as the last call found it: a small system
    /// that went through the one launch reports it on the way, and the next call of the same kind (see BoxGuess) on
    /// the same box picks its grid from it without a pass over the points and a round trip to the host first. A
    /// point outside of the remembered extent ends up in the outermost cell of its direction, which is as wide as
    /// the cutoff at least and has no neighbours beyond: the rows are the same, a stale extent only costs time
    /// (crowded cells), and with at most 2048 points never much.
    bool extent_valid = false;
    bool extent_missed = false;       // the call started from that extent and found its points far outside of it
    int extent_rest = 0;              // calls that find the extent first after such a call
    double extent_lo[3] = {0, 0, 0};
    double extent_hi[3] = {0, 0, 0};
    SmallMeeting* meetings = nullptr; // device, two of them (see SmallMeeting); allocated at the first small system
    bool own_meetings = false;        // allocated by this state (not part of memory that was handed to it)
    uint32_t meeting_turn = 0;
    int compute_units = 0;            // of the device (asked once)
    hipEvent_t events[T_STAGES] = {};
    bool have_events = false;
    // a second stream of the list's own, for a kernel that can run beside another of the same call (forked from and
    // joined back into the call's stream with the two events); made when first needed
    hipStream_t side_stream = nullptr;
    hipEvent_t side_fork = nullptr;
    hipEvent_t side_join = nullptr;
    bool timings_valid = false;
    VesinHipTimings timings = {};
    VerletCache* verlet = nullptr;    // only while the caller asks for a skin
    BatchVerletCache* verlet_batch = nullptr; // the same for batches
    // vesin_hip_neighbors_enqueue / _collect: the call that stopped at its first wait, and the device word that tells
    // kernels queued behind it whether the rows are complete (made when first needed)
    SuspendedCall* queued = nullptr;
    bool enqueued = false;            // a call was queued and not collected yet
    hipStream_t queued_stream = nullptr;
    unsigned long long* d_queued_length = nullptr;
    /// Where the systems' first rows of the last batch are on the device (n_systems + 1 words, the last one the number
    /// of rows), until the next call on the list; nullptr when the last call was no batch.
    const unsigned long long* batch_first_pair_device = nullptr;
    bool length_published = false;    // the kernels of the queued part were followed by the one that fills that word
    bool queued_part_sufficed = false; // ... and the host found, like that kernel, that they left the complete list

    HipExtras() = default;
    HipExtras(const HipExtras&) = delete;
    HipExtras& operator=(const HipExtras&) = delete;

    /// Wait for the stream; afterwards `mail` holds what the kernels queued before this call reported, and the first
    /// `n_bounds` slots of the bounding pass. (A block in device memory is copied piece by piece: a few hundred bytes
    /// for most waits, where the whole block is 20 KB that the runtime would stage on every wait.)
    /// A queued call (see SuspendedCall) stops at its first wait and, once resumed, waits for what it had queued up
    /// to here only.
    void wait(hipStream_t stream, size_t n_bounds = 0) {
        if (mail_device != mail) {
            HIP_CHECK(hipMemcpyAsync(mail, mail_device, offsetof(Mailbox, bounds), hipMemcpyDeviceToHost, stream));
            if (n_bounds > 0) {
                HIP_CHECK(hipMemcpyAsync(
                    mail->bounds, mail_device->bounds, n_bounds * sizeof(BlockBounds), hipMemcpyDeviceToHost, stream
                ));
            }
        }
        sync(stream);
    }

    /// Wait for the stream; a queued call (see SuspendedCall) stops at its first wait instead and, once resumed, waits
    /// for what it had queued up to there only. Not for use inside a `catch` block: a call must not stop with an
    /// exception in flight.
    void sync(hipStream_t stream) {
        if (queued != nullptr && queued->stop_at_next_wait) {
            queued->stop_at_next_wait = false;
            HIP_CHECK(hipEventRecord(queued->reached, stream));
            queued->stop();
            HIP_CHECK(hipEventSynchronize(queued->reached));
            return;
        }
        HIP_CHECK(hipStreamSynchronize(stream));
    }

    /// The kernels queued so far leave the complete list in the arrays if `outcome` says so: the device word of a
    /// queued call is told, if this is the part of the call that is queued (only such calls pay for the launch).
    /// Returns whether it did: the caller then says, once it has looked, whether the host came to the same conclusion
    /// (`queued_part_sufficed`).
    /// Whether the next wait is the one a queued call stops at: what is queued before it may be followed by a kernel
    /// that fills the device word.
    bool before_the_stop_of_a_queued_call() const {
        return queued != nullptr && queued->stop_at_next_wait;
    }

    bool publish_length(const QueuedOutcome& outcome, const double* box, const bool* periodic, hipStream_t stream) {
        if (queued != nullptr && queued->stop_at_next_wait) {
            hipLaunchKernelGGL(publish_queued_length, dim3(1), dim3(1), 0, stream, outcome, box, periodic, d_queued_length);
            length_published = true;
            return true;
        }
        return false;
    }

    ~HipExtras() {
        delete verlet;
        delete verlet_batch;
        delete queued;
        if (d_queued_length != nullptr) {
            (void)hipFree(d_queued_length);
        }
        work.release();
        sort_work.release();
        batch.kept_boxes.release();
        batch.molecule_work.release();
        if (batch.molecule_report != nullptr) {
            (void)hipHostFree(batch.molecule_report);
        }
        if (batch.first_pair_landing != nullptr) {
            (void)hipHostFree(batch.first_pair_landing);
        }
        if (!fixed_memory) {
            if (meetings != nullptr && own_meetings) {
                (void)hipFree(meetings);
            }
            if (d_status != nullptr) {
                (void)hipFree(d_status);
            }
            if (mail != nullptr) {
                (void)hipHostFree(mail);
            }
        }
        if (have_events) {
            for (auto& event : events) {
                (void)hipEventDestroy(event);
            }
        }
        if (side_fork != nullptr) {
            (void)hipEventDestroy(side_fork);
        }
        if (side_join != nullptr) {
            (void)hipEventDestroy(side_join);
        }
        if (side_stream != nullptr) {
            (void)hipStreamDestroy(side_stream);
        }
    }

    /// The side stream and its events (default priority, like every stream here); nullptr for the entry point that
    /// allocates nothing, whose kernels all run on the caller's stream.
    hipStream_t side() {
        if (fixed_memory) {
            return nullptr;
        }
        if (side_stream == nullptr) {
            HIP_CHECK(hipEventCreateWithFlags(&side_fork, hipEventDisableTiming));
            HIP_CHECK(hipEventCreateWithFlags(&side_join, hipEventDisableTiming));
            HIP_CHECK(hipStreamCreateWithFlags(&side_stream, hipStreamNonBlocking));
        }
        return side_stream;
    }
};

HipExtras& extras_of(VesinNeighborList& neighbors) {
    if (neighbors.opaque == nullptr) {
        // the list only gets a state whose allocations all succeeded
        auto extras = std::make_unique<HipExtras>();
        extras->device_id = neighbors.device.device_id;
        HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&extras->d_status), sizeof(DeviceStatus)));
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&extras->mail), sizeof(Mailbox), hipHostMallocDefault));
        extras->mail_device = extras->mail;
        neighbors.opaque = extras.release();
    }
    return *static_cast<HipExtras*>(neighbors.opaque);
}

/// Device ordinal owning `ptr`, or -1 when it is not device memory.
int device_of(const void* ptr) {
    hipPointerAttribute_t attributes;
    hipError_t status = hipPointerGetAttributes(&attributes, ptr);
    if (status != hipSuccess) {
        (void)hipGetLastError(); // clear the sticky error left by an unknown (host) pointer
        return -1;
    }
    if (attributes.type != hipMemoryTypeDevice) {
        return -1;
    }
    return attributes.device;
}

/// An output array goes back to where it came from: the allocator of the list's caller, or the HIP runtime.
void release_output(const HipExtras* extras, void* pointer) {
    if (pointer == nullptr) {
        return;
    }
    if (extras != nullptr && extras->release != nullptr) {
        extras->release(pointer, extras->allocator_context);
    } else {
        (void)hipFree(pointer);
    }
}

void free_outputs(VesinNeighborList& neighbors, const HipExtras* extras) {
    release_output(extras, neighbors.pairs);
    release_output(extras, neighbors.shifts);
    release_output(extras, neighbors.distances);
    release_output(extras, neighbors.vectors);
    neighbors.pairs = nullptr;
    neighbors.shifts = nullptr;
    neighbors.distances = nullptr;
    neighbors.vectors = nullptr;
}

/// The list of the entry point that allocates nothing has more rows than the caller's arrays hold.
struct RowsDoNotFit: std::runtime_error {
    size_t rows;

    RowsDoNotFit(size_t needed, size_t capacity):
        std::runtime_error(
            "the neighbor list has " + std::to_string(needed) + " pairs, the output arrays of the caller hold " +
            std::to_string(capacity)
        ),
        rows(needed) {}
};

/// Make every requested output array hold `rows` rows and drop the ones that were not requested (like the CPU
/// engine of the reference does, vesin/src/cpu_cell_list.cpp:605-627).
void size_outputs(VesinNeighborList& neighbors, HipExtras& extras, size_t rows, const VesinOptions& options) {
    if (extras.fixed_memory) {
        // the arrays are the caller's: they hold the rows or the call fails, and `length` says what it takes
        if (rows > extras.capacity) {
            neighbors.length = rows;
            throw RowsDoNotFit(rows, extras.capacity);
        }
        return;
    }
    if (rows > extras.capacity) {
        free_outputs(neighbors, &extras);
        size_t capacity = rows + rows / 8;
        if (capacity < 1024) {
            capacity = 1024;
        }
        extras.capacity = capacity;
    }
    if (extras.capacity == 0) {
        extras.capacity = 1024;
    }
    const size_t capacity = extras.capacity;

    auto drop = [&](auto*& pointer) {
        release_output(&extras, pointer);
        pointer = nullptr;
    };
    auto ensure = [&](auto*& pointer, size_t bytes) {
        if (pointer != nullptr) {
            return;
        }
        void* memory = nullptr;
        if (extras.allocate != nullptr) {
            memory = extras.allocate(bytes, extras.allocator_context);
        } else if (hipMalloc(&memory, bytes) != hipSuccess) {
            (void)hipGetLastError();
            memory = nullptr;
        }
        if (memory == nullptr) {
            free_outputs(neighbors, &extras);
            extras.capacity = 0;
            throw std::bad_alloc();
        }
        pointer = static_cast<std::remove_reference_t<decltype(pointer)>>(memory);
    };

    ensure(neighbors.pairs, capacity * 2 * sizeof(size_t));
    if (options.return_shifts) {
        ensure(neighbors.shifts, capacity * 3 * sizeof(int32_t));
    } else {
        drop(neighbors.shifts);
    }
    if (options.return_distances) {
        ensure(neighbors.distances, capacity * sizeof(double));
    } else {
        drop(neighbors.distances);
    }
    if (options.return_vectors) {
        ensure(neighbors.vectors, capacity * 3 * sizeof(double));
    } else {
        drop(neighbors.vectors);
    }
}

/// Scratch rows for `rows` unsorted rows (shifts always present: they are part of the sort key) and the workspace
/// of the radix sort, from the list's sort arena; the sort's final gather fills the caller's arrays.
void carve_sort_space(
    HipExtras& extras, size_t rows, const VesinOptions& options, SearchOutputs& unsorted, SortWorkspace& space
) {
    const size_t table_entries = static_cast<size_t>(RADIX) * sort_blocks(rows);
    auto carve = [&](Carver& c) {
        unsorted.pairs = c.take<unsigned long long>(2 * rows);
        unsorted.shifts = c.take<int32_t>(3 * rows);
        unsorted.distances = options.return_distances ? c.take<double>(rows) : nullptr;
        unsorted.vectors = options.return_vectors ? c.take<double>(3 * rows) : nullptr;
        for (int b = 0; b < 2; b++) {
            space.keys[b] = c.take<uint64_t>(rows);
            space.rows[b] = c.take<uint32_t>(rows);
        }
        space.table = c.take<uint32_t>(table_entries);
        space.table_scan = c.take<uint64_t>(table_entries + 1);
        space.scan_scratch = c.take<uint64_t>(scan_scratch_elements(table_entries));
    };
    Carver measure(nullptr);
    carve(measure);
    extras.sort_work.reserve(measure.used);
    Carver carver(extras.sort_work.ptr);
    carve(carver);
}

/// Optional user-imposed limit on pairs per point, kept for callers that rely on the reference's environment
/// variable and its messages (vesin/src/vesin_cuda.cpp:871-884, :911-918). 0 = no limit.
size_t pairs_per_point_limit() {
    const char* text = std::getenv("VESIN_CUDA_MAX_PAIRS_PER_POINT");
    if (text == nullptr) {
        return 0;
    }
    size_t length = std::strlen(text);
    char* end = nullptr;
    errno = 0;
    long long parsed = std::strtoll(text, &end, 10);
    if (errno != 0 || end != text + length || parsed <= 0) {
        throw std::runtime_error("Invalid value for VESIN_CUDA_MAX_PAIRS_PER_POINT: '" + std::string(text) + "'");
    }
    return static_cast<size_t>(parsed);
}

template <bool WRITE>
void launch_search(bool full, const SearchArgs& args, const GridParams& g, hipStream_t stream) {
    if (args.n_work == 0) {
        return;
    }
    constexpr int R = 2;
    const uint32_t blocks = (args.n_work + SEARCH_WAVES - 1) / SEARCH_WAVES;
    if (full) {
        hipLaunchKernelGGL((search_kernel<WRITE, true, R>), dim3(blocks), dim3(SEARCH_BLOCK), 0, stream, args, g);
    } else {
        hipLaunchKernelGGL((search_kernel<WRITE, false, R>), dim3(blocks), dim3(SEARCH_BLOCK), 0, stream, args, g);
    }
}

void non_finite_error(const double (*points)[3], unsigned int flat) {
    size_t point = flat / 3;
    int axis = static_cast<int>(flat % 3);
    double value = 0.0;
    HIP_CHECK(hipMemcpy(&value, &points[point][axis], sizeof(double), hipMemcpyDeviceToHost));
    // same text as the CPU engine of the reference (vesin/src/types.hpp:163-169)
    throw std::runtime_error(
        "point " + std::to_string(point) + " has non-finite coordinate along axis " + std::to_string(axis) + ": " +
        std::to_string(value)
    );
}

/// The requirements of the reference on the inputs of a GPU call, with its texts
/// (vesin/src/vesin_cuda.cpp:831-854), and this library's own limit on the number of points.
void check_inputs(const double (*points)[3], size_t n_points, const double box[3][3], const bool periodic[3], int device_id) {
    int device_count = 0;
    if (hipGetDeviceCount(&device_count) != hipSuccess || device_count == 0) {
        (void)hipGetLastError();
        throw std::runtime_error("no HIP device is available to this process");
    }
    if (device_id < 0 || device_id >= device_count) {
        throw std::runtime_error("invalid GPU device_id " + std::to_string(device_id));
    }

    // same requirements and texts as the reference (vesin/src/vesin_cuda.cpp:831-854)
    const int points_device = device_of(points);
    if (points_device < 0) {
        throw std::runtime_error("`points` pointer is not allocated on a CUDA device");
    }
    const int box_device = device_of(box);
    if (box_device < 0) {
        throw std::runtime_error("`box` pointer is not allocated on a CUDA device");
    }
    const int periodic_device = device_of(periodic);
    if (periodic_device < 0) {
        throw std::runtime_error("`periodic` pointer is not allocated on a CUDA device");
    }
    if (points_device != box_device) {
        throw std::runtime_error("`points` and `box` do not exist on the same device");
    }
    if (points_device != periodic_device) {
        throw std::runtime_error("`points` and `periodic` do not exist on the same device");
    }
    if (points_device != device_id) {
        throw std::runtime_error("`points`, `box` and `periodic` device differs from input neighbors device_id");
    }
    if (n_points >= 0xFFFFFFF0ull) {
        throw std::runtime_error("too many points: the GPU path indexes points with 32 bits");
    }
}

bool compute(
    const double (*points)[3], size_t n_points, const double box[3][3], const bool periodic[3], VesinOptions options,
    VesinNeighborList& neighbors, HipExtras& extras, bool speculate, hipStream_t stream
);

void verlet_neighbors(
    const double (*points)[3], size_t n_points, const double box[3][3], const bool periodic[3], VesinOptions options,
    VesinNeighborList& neighbors, HipExtras& extras, hipStream_t stream
);

void direct_neighbors(
    const double (*points)[3], size_t n_points, const double box[3][3], const bool periodic[3], VesinOptions options,
    VesinNeighborList& neighbors, HipExtras& extras, hipStream_t stream
);

} // namespace

namespace {

/// The call itself, on a list that has its state and whose inputs were checked, with the list's device current.
void run_call(
    const double (*points)[3], size_t n_points, const double box[3][3], const bool periodic[3], VesinOptions options,
    VesinNeighborList& neighbors, HipExtras& extras, hipStream_t stream
) {
    const TraceRange whole_call(options.skin > 0.0 ? "vesin_neighbors (skin)" : "vesin_neighbors");
    extras.timings_valid = false;
    extras.batch_first_pair_device = nullptr;
    if (options.skin > 0.0) {
        verlet_neighbors(points, n_points, box, periodic, options, neighbors, extras, stream);
        return;
    }
    if (extras.verlet != nullptr) {
        // no skin any more: the cache goes, like in the reference (vesin/src/cpu_cell_list.cpp:235-238)
        delete extras.verlet;
        extras.verlet = nullptr;
    }
    direct_neighbors(points, n_points, box, periodic, options, neighbors, extras, stream);
}

/// A list whose arrays were handed to the caller (vesin_hip_detach_outputs) gets arrays of the same size again
/// before the call starts: every path that writes into kept arrays finds them as it left them.
void restore_outputs(VesinNeighborList& neighbors, HipExtras& extras, const VesinOptions& options) {
    if (!extras.fixed_memory && extras.capacity > 0 && neighbors.pairs == nullptr) {
        size_outputs(neighbors, extras, 0, options);
    }
}

/// Whether the single-pass search of this call lines its vectors up in LDS before it stores them (the STAGED kernels
/// of fused.cuh): when it returns vectors, as a full list or beside shifts or distances.
bool staged_vectors(const SearchOutputs& out, bool full) {
    return out.vectors != nullptr && (full || out.shifts != nullptr || out.distances != nullptr);
}

void refuse_while_queued(const HipExtras& extras) {
    if (extras.enqueued) {
        throw std::runtime_error(
            "a calculation queued with vesin_hip_neighbors_enqueue is pending on this list: call "
            "vesin_hip_neighbors_collect first"
        );
    }
}

/// What a list needs before a call is queued on it: the device word (saying that the rows are pending) and the stack
/// the call runs on.
void begin_queued(HipExtras& extras, hipStream_t stream) {
    if (extras.d_queued_length == nullptr) {
        HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&extras.d_queued_length), 256));
    }
    if (extras.queued == nullptr) {
        extras.queued = new SuspendedCall();
    }
    // whatever was queued behind an earlier call has read its word by the time this one is overwritten: same stream,
    // or the caller's own ordering between streams
    hipLaunchKernelGGL(set_queued_length, dim3(1), dim3(1), 0, stream, extras.d_queued_length, ROWS_PENDING);
    HIP_CHECK(hipGetLastError());
    extras.length_published = false;
    extras.queued_part_sufficed = false;
    extras.enqueued = true;
    extras.queued_stream = stream;
}

/// After the queued call ran to its end: hand on its error, and make the device word say what `length` says unless
/// the queued kernels did that themselves.
void finish_queued(VesinNeighborList& neighbors, HipExtras& extras, hipStream_t stream) {
    SuspendedCall& call = *extras.queued;
    extras.enqueued = false;
    call.stop_at_next_wait = false;
    call.body = nullptr;
    if (call.error != nullptr) {
        std::exception_ptr error = call.error;
        call.error = nullptr;
        std::rethrow_exception(error);
    }
    if (!(extras.length_published && extras.queued_part_sufficed)) {
        hipLaunchKernelGGL(
            set_queued_length, dim3(1), dim3(1), 0, stream, extras.d_queued_length,
            static_cast<unsigned long long>(neighbors.length)
        );
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(stream));
    }
}

} // namespace

void neighbors(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    void* caller_stream
) {
    // the null stream when the caller names none, like the reference (vesin/src/vesin_cuda.cpp:798)
    hipStream_t stream = static_cast<hipStream_t>(caller_stream);
    const int device_id = neighbors.device.device_id;
#ifdef VESIN_HIP_HOST_PROFILE
    HOST_PROFILE.begin();
#endif
    check_inputs(points, n_points, box, periodic, device_id);
    HOST_LAP(0);

    const DeviceGuard guard(device_id);
    HipExtras& extras = extras_of(neighbors);
    refuse_while_queued(extras);
    restore_outputs(neighbors, extras, options);
    HOST_LAP(1);
    run_call(points, n_points, box, periodic, options, neighbors, extras, stream);
    HOST_LAP(5);
#ifdef VESIN_HIP_HOST_PROFILE
    HOST_PROFILE.end();
#endif
}

const unsigned long long* neighbors_enqueue(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    void* caller_stream
) {
    hipStream_t stream = static_cast<hipStream_t>(caller_stream);
    const int device_id = neighbors.device.device_id;
    check_inputs(points, n_points, box, periodic, device_id);

    const DeviceGuard guard(device_id);
    HipExtras& extras = extras_of(neighbors);
    refuse_while_queued(extras);
    restore_outputs(neighbors, extras, options);
    begin_queued(extras, stream);
    VesinNeighborList* list = &neighbors;
    HipExtras* state = &extras;
    extras.queued->start([=]() { run_call(points, n_points, box, periodic, options, *list, *state, stream); });
    if (extras.queued->finished) {
        // nothing to wait for (no points), or an error before the first wait
        finish_queued(neighbors, extras, stream);
    }
    return extras.d_queued_length;
}

void neighbors_collect(VesinNeighborList& neighbors) {
    auto* extras = static_cast<HipExtras*>(neighbors.opaque);
    if (extras == nullptr || extras->queued == nullptr) {
        throw std::runtime_error("no calculation was queued on this list");
    }
    if (!extras->enqueued) {
        return; // the queued call ended inside vesin_hip_neighbors_enqueue already, or was collected
    }
    const DeviceGuard guard(neighbors.device.device_id);
    if (!extras->queued->finished) {
        extras->queued->resume();
    }
    finish_queued(neighbors, *extras, extras->queued_stream);
}

namespace {

/// The search itself (no caching), on a list whose inputs were checked.
void direct_neighbors(
    const double (*points)[3], size_t n_points, const double box[3][3], const bool periodic[3], VesinOptions options,
    VesinNeighborList& neighbors, HipExtras& extras, hipStream_t stream
) {
    // A box that did not change over the last calls is assumed not to have changed now either: the call runs with
    // the remembered one and checks the assumption at its last synchronisation (see BoxGuess).
    const BoxKey key = {n_points, options.cutoff, static_cast<int>(options.algorithm), options.full, options.sorted};
    const bool speculate = extras.guess.begin(key);
    if (speculate) {
        bool box_was_right = false;
        bool failed = false;
        std::exception_ptr failure;
        try {
            box_was_right = compute(points, n_points, box, periodic, options, neighbors, extras, true, stream);
        } catch (...) {
            failed = true;
            failure = std::current_exception();
        }
        if (failed) {
            // the error may be a consequence of the wrong box: fetch the one of this call and find out
            hipLaunchKernelGGL(
                fetch_box, dim3(1), dim3(64), 0, stream,
                reinterpret_cast<const double*>(box), periodic, extras.mail_device->small, extras.d_status
            );
            extras.wait(stream);
            box_was_right = std::memcmp(extras.mail->small, extras.last_box, BOX_BYTES) == 0;
            if (box_was_right) {
                std::rethrow_exception(failure);
            }
        }
        if (box_was_right) {
            extras.guess.was_right();
            return;
        }
        if (extras.extent_missed) {
            extras.extent_missed = false; // nothing wrong with the box
        } else {
            extras.guess.was_wrong();
        }
    }
    (void)compute(points, n_points, box, periodic, options, neighbors, extras, false, stream);
    extras.guess.stored(key);
}

bool compute(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    HipExtras& extras,
    bool speculate,
    hipStream_t stream
) {
    const size_t pair_limit = pairs_per_point_limit();

    const bool timed = TIMINGS_ENABLED.load() && !extras.fixed_memory; // creating events allocates
    if (timed && !extras.have_events) {
        for (auto& event : extras.events) {
            HIP_CHECK(hipEventCreate(&event));
        }
        extras.have_events = true;
    }
    // (the stages of VesinHipTimings, by the stage that each mark ends)
    static const char* const STAGE_AFTER[T_STAGES] = {"cell build", "search", "scan", "after the scan",
                                                       "write", "sort", "end of call"};
    TraceRange stage_range(speculate ? "set-up (box of the call before)" : "set-up (box read from the device)");
    auto mark = [&](Stage stage) {
        stage_range.next(STAGE_AFTER[stage]);
        if (timed) {
            HIP_CHECK(hipEventRecord(extras.events[stage], stream));
        }
    };

    // ---- box and periodicity come to the host once: 75 bytes. A call that starts from the remembered box fetches
    // them with its first fill kernel instead (see below).
    auto launch_fetch = [&]() {
        hipLaunchKernelGGL(
            fetch_box, dim3(1), dim3(64), 0, stream,
            reinterpret_cast<const double*>(box), periodic, extras.mail_device->small, extras.d_status
        );
    };
    bool fetched = false;
    unsigned char used_box[BOX_BYTES];
    if (speculate) {
        std::memcpy(used_box, extras.last_box, BOX_BYTES);
    } else {
        launch_fetch();
        fetched = true;
        extras.wait(stream);
        std::memcpy(used_box, extras.mail->small, BOX_BYTES);
        extras.guess.have_box = false; // remembered once it proved usable, below
    }
    // valid after any synchronisation of the stream that follows the launch of fetch_box
    auto box_was_right = [&]() { return std::memcmp(extras.mail->small, used_box, BOX_BYTES) == 0; };

    double host_box[9];
    bool host_periodic[3];
    std::memcpy(host_box, used_box, sizeof(host_box));
    for (int d = 0; d < 3; d++) {
        host_periodic[d] = used_box[72 + d] != 0;
    }
    const HostBox hbox = normalise_box(host_box, host_periodic);
    if (!speculate) {
        std::memcpy(extras.last_box, used_box, BOX_BYTES);
        extras.guess.have_box = true;
    }

    if (n_points == 0) {
        size_outputs(neighbors, extras, 0, options);
        neighbors.length = 0;
        return true;
    }

    GridParams g;
    std::memset(&g, 0, sizeof(g));
    for (int d = 0; d < 3; d++) {
        for (int e = 0; e < 3; e++) {
            g.H[3 * d + e] = hbox.H[d][e];
            g.Hinv[3 * d + e] = hbox.Hinv[d][e];
        }
        g.periodic[d] = hbox.periodic[d] ? 1 : 0;
        g.np_scale[d] = 1.0;
    }
    g.cutoff2 = options.cutoff * options.cutoff; // vesin/src/cpu_cell_list.cpp:77
    g.n_points = static_cast<uint32_t>(n_points);

    mark(T_START);

    // ---- extent of the points along non-periodic directions
    const bool any_open = !(hbox.periodic[0] && hbox.periodic[1] && hbox.periodic[2]);
    double lo[3] = {0, 0, 0};
    double hi[3] = {0, 0, 0};
    // (valid for one call: whatever happens below, only a call that reports a fresh extent makes it valid again)
    // Small systems: for the one launch that does everything. Larger ones: for the single-pass search, which then
    // needs no pass over the points and no answer from the device before its kernels are launched. Either way the
    // call finds the extent of its own points on the way and leaves it for the call after it. A grid that fits
    // the points of the call before still gives the right list: points beyond it land in the outermost cells.
    const bool small_guess = n_points <= SMALL_POINTS && extras.one_launch_rest == 0 && extras.meeting_rest.rest == 0;
    const bool large_guess = n_points > SMALL_POINTS && !options.sorted && extras.capacity > 0 && !two_pass_only() &&
                             extras.single_pass_rest == 0 && !ordered_rows() && options.algorithm != VesinBruteForce &&
                             extras.extent_rest == 0 && !fresh_extent_only();
    if (any_open && extras.extent_rest > 0) {
        extras.extent_rest -= 1;
    }
    const bool remembered_extent = any_open && speculate && extras.extent_valid && (small_guess || large_guess);
    extras.extent_valid = false;
    if (remembered_extent) {
        for (int d = 0; d < 3; d++) {
            lo[d] = extras.extent_lo[d];
            hi[d] = extras.extent_hi[d];
        }
    }
    if (any_open && !remembered_extent) {
        if (!fetched) {
            launch_fetch(); // the synchronisation below is where a remembered box is checked first
            fetched = true;
        }
        const uint32_t blocks = static_cast<uint32_t>(std::min<size_t>(BOUNDING_BLOCKS, (n_points + BLOCK - 1) / BLOCK));
        hipLaunchKernelGGL(
            bounding_kernel, dim3(blocks), dim3(BLOCK), 0, stream,
            reinterpret_cast<const double*>(points), g.n_points, g, extras.mail_device->bounds
        );
        extras.wait(stream, blocks);
        if (!box_was_right()) {
            return false;
        }
        unsigned int bad = 0xFFFFFFFFu;
        for (int d = 0; d < 3; d++) {
            lo[d] = INFINITY;
            hi[d] = -INFINITY;
        }
        for (uint32_t block = 0; block < blocks; block++) {
            const BlockBounds& part = extras.mail->bounds[block];
            bad = std::min(bad, part.first_bad_coordinate);
            for (int d = 0; d < 3; d++) {
                lo[d] = std::fmin(lo[d], part.lo[d]);
                hi[d] = std::fmax(hi[d], part.hi[d]);
            }
        }
        if (bad != 0xFFFFFFFFu) {
            non_finite_error(points, bad);
        }
        if (n_points > SMALL_POINTS) {
            for (int d = 0; d < 3; d++) {
                extras.extent_lo[d] = lo[d];
                extras.extent_hi[d] = hi[d];
            }
            extras.extent_valid = true;
        }
    }

    // ---- grid: the brute-force layout is one cell whose stencil enumerates periodic images
    bool single_cell = options.algorithm == VesinBruteForce;
    HostGrid grid = choose_grid(hbox, options.cutoff, n_points, lo, hi, single_cell);
    if (options.algorithm == VesinAutoAlgorithm && !single_cell && (grid.n_cells == 1 || n_points < 32)) {
        single_cell = true;
        grid = choose_grid(hbox, options.cutoff, n_points, lo, hi, true);
    }
    for (int d = 0; d < 3; d++) {
        g.n[d] = grid.n[d];
        g.s[d] = grid.s[d];
        g.np_min[d] = grid.np_min[d];
        g.np_scale[d] = grid.np_scale[d];
    }
    g.n_cells = static_cast<uint32_t>(grid.n_cells);
    choose_pruning(hbox, grid, options.cutoff, g);
    if (full_stencil_only()) {
        g.prune = 0;
    }
    Prefilter pre;
    choose_prefilter(g, options.cutoff, pre);
    if (double_precision_only()) {
        pre.use32 = 0;
    }

    // ---- carve the work buffers
    const size_t n_cells = grid.n_cells;
    // upper bound of the number of tiles, rounded up to what the search kernel's XCD-aware order needs
    size_t tiles_bound = (single_cell ? 0 : std::min<size_t>(n_cells, n_points)) + n_points / TILE_POINTS + 1;
    constexpr size_t slot_multiple = N_XCD * SEARCH_WAVES;
    tiles_bound = (tiles_bound + slot_multiple - 1) / slot_multiple * slot_multiple;
    // Small systems: several waves share a tile, each taking a slice of its candidates, so that the chip has
    // about 4096 work items to spread. A slice should still hold a unit of 64 candidates: waves without work
    // only add to the time (measured: 216 atoms take 43 us with 256 slices per tile, 25 us with 8).
    uint32_t n_slices = 1;
    if (tiles_bound < 4096) {
        const double entries = upper_stencil_cells(g);
        const double per_cell = std::max(1.0, static_cast<double>(n_points) / static_cast<double>(n_cells));
        const double units = std::ceil(entries * per_cell / WAVE);
        const double wanted = std::min(units, std::floor(4096.0 / static_cast<double>(tiles_bound)));
        n_slices = static_cast<uint32_t>(std::min(64.0, std::max(1.0, wanted)));
    }
    const size_t search_blocks = tiles_bound * n_slices;
    const size_t n_slots = search_blocks;

    const size_t search_workgroups = (search_blocks + SEARCH_WAVES - 1) / SEARCH_WAVES;
    uint32_t* cell_counts = nullptr;
    const size_t chain_groups = (search_workgroups + CHAIN_GROUP - 1) / CHAIN_GROUP;
    Chain chain = {};
    FusedStatus* fused_status = nullptr;
    uint64_t* cell_scan = nullptr;
    uint32_t* cell_of = nullptr;
    uint32_t* slot_of = nullptr;
    int32_t* wrap_of = nullptr;
    uint32_t* provisional = nullptr;
    SortedPoints sorted = {};
    Tile* tiles = nullptr;
    uint32_t* counts = nullptr;
    uint64_t* offsets = nullptr;
    uint64_t* scan_scratch = nullptr;

    // The single-pass search writes straight into the arrays kept from earlier calls. It does not cover every shape
    // of problem and the rows may not fit: in both cases nothing is lost but time, the two passes start over.
    bool try_single_pass = !options.sorted && extras.capacity > 0 && !two_pass_only();
    if (try_single_pass && extras.single_pass_rest > 0) {
        extras.single_pass_rest -= 1;
        try_single_pass = false;
    }
    if (try_single_pass && ordered_rows() && extras.chain_rest.resting()) {
        try_single_pass = false; // (the two passes give the rows in the same order on every run as well)
    }
    // Cells of ordinary occupation: the cells are built in one pass over the points, every cell owning
    // DIRECT_CAPACITY slots (place_direct); only the single-pass search reads that layout.
    const double direct_mean_min = extras.fixed_memory             ? DIRECT_MEAN_MIN_FIXED_MEMORY
                                   : n_cells <= DIRECT_FEW_CELLS  ? DIRECT_MEAN_MIN_FEW_CELLS
                                   : n_cells <= DIRECT_SOME_CELLS ? DIRECT_MEAN_MIN_SOME_CELLS
                                                                  : DIRECT_MEAN_MIN;
    bool direct_cells = try_single_pass && !single_cell && !ordered_rows() && !packed_cells_only() &&
                        static_cast<double>(n_points) <= DIRECT_MEAN_MAX * static_cast<double>(n_cells) &&
                        static_cast<double>(n_points) >= direct_mean_min * static_cast<double>(n_cells) &&
                        n_cells * DIRECT_CAPACITY < 0xFFFFFF00ull;
    if (direct_cells && extras.direct_rest > 0) {
        extras.direct_rest -= 1;
        direct_cells = false;
    }
    // small systems: the whole packed cell build, clearing and box fetch included, is one launch of one workgroup
    const bool small_build = !single_cell && !ordered_rows() && n_points <= SMALL_BUILD_POINTS &&
                             n_cells <= SMALL_BUILD_POINTS && std::getenv("VESIN_HIP_CELLS") == nullptr;
    if (small_build) {
        direct_cells = false;
    }
    constexpr size_t direct_tiles_per_cell = DIRECT_CAPACITY / TILE_POINTS;
    const size_t direct_slots =
        direct_cells ? (n_cells * direct_tiles_per_cell + slot_multiple - 1) / slot_multiple * slot_multiple : 0;
    const size_t sorted_slots = direct_cells ? std::max<size_t>(n_points, n_cells * DIRECT_CAPACITY) : n_points;
    uint32_t* direct_wrapped = nullptr;

    // the search that produces a sorted list in order covers stencils that fit its tables
    const size_t full_stencil = static_cast<size_t>(2 * grid.s[0] + 1) * (2 * grid.s[1] + 1) * (2 * grid.s[2] + 1);
    bool try_in_order = options.sorted && full_stencil <= MAX_ENTRIES && !radix_sort_only();
    if (try_in_order && extras.in_order_rest > 0) {
        extras.in_order_rest -= 1;
        try_in_order = false;
    }
    // Small systems with arrays from earlier calls: everything in one launch (small.cuh), as one work item per point
    // for a sorted list, as one per point and slice of its candidates otherwise (about four units of 64 candidates
    // per item, as many items as the smallest shape of that launch takes).
    const bool small_allowed = extras.capacity > 0 && n_points <= SMALL_POINTS && n_cells <= SMALL_POINTS &&
                               !separate_launches() && !ordered_rows() && std::getenv("VESIN_HIP_CELLS") == nullptr;
    bool one_launch = false;
    uint32_t small_slices = 1;
    if (small_allowed && options.sorted) {
        one_launch = try_in_order;
    } else if (small_allowed && try_single_pass && full_stencil - full_stencil / 2 <= MAX_ENTRIES &&
               n_points <= SmallShape<4>::MAX_ITEMS && n_cells <= SmallShape<4>::CAPACITY) {
        const double per_cell = std::max(1.0, static_cast<double>(n_points) / static_cast<double>(n_cells));
        const double units = std::ceil(upper_stencil_cells(g) * per_cell / WAVE);
        const double most = std::floor(static_cast<double>(SmallShape<4>::MAX_ITEMS) / static_cast<double>(n_points));
        small_slices = static_cast<uint32_t>(std::max(1.0, std::min(most, std::ceil(units / 4.0))));
        one_launch = true;
    }
    if (one_launch && extras.one_launch_rest > 0) {
        extras.one_launch_rest -= 1;
        one_launch = false;
    }
    if (one_launch) {
        // every workgroup of that launch must be resident at once: never more workgroups than the device has
        // compute units (a workgroup of the largest shape fills the LDS of one)
        if (extras.compute_units == 0) {
            int units = 0;
            HIP_CHECK(hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, extras.device_id));
            extras.compute_units = units;
        }
        const size_t items = n_points * small_slices;
        const size_t waves = !options.sorted                                                        ? 4
                             : n_points <= SmallShape<4>::MAX_ITEMS && n_cells <= SmallShape<4>::CAPACITY ? 4
                             : n_points <= SmallShape<8>::MAX_ITEMS                                       ? 8
                                                                                                          : 16;
        if ((items + waves - 1) / waves > static_cast<size_t>(extras.compute_units)) {
            one_launch = false;
        }
    }
    if (one_launch && extras.meetings == nullptr) {
        if (extras.fixed_memory) {
            one_launch = false; // no allocation there
        } else {
            HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&extras.meetings), 2 * sizeof(SmallMeeting)));
            extras.own_meetings = true;
            HIP_CHECK(hipMemset(extras.meetings, 0, 2 * sizeof(SmallMeeting)));
        }
    }
    if (one_launch && extras.meeting_rest.resting()) {
        one_launch = false; // its workgroups gave up waiting for each other not long ago
    }
    const size_t small_items = one_launch ? n_points * small_slices : 0;
    uint32_t* rows_of_item = nullptr;
    OrderedStatus* ordered_status = nullptr;
    uint32_t* rows_of_point = nullptr;
    uint64_t* first_row_of_point = nullptr;
    CandidateRecord* candidate_records = nullptr;
    uint32_t* candidates_of_item = nullptr;
    uint16_t* candidate_order = nullptr;
    char* wraps_end = nullptr;
    // small systems: the points of a tile are dealt to several waves, about 2048 in all
    static_assert(ORDERED_TILE_POINTS == TILE_POINTS, "policy.hpp and the kernels agree on the size of a tile");
    uint32_t ordered_points_per_item = ordered_share(n_points, n_cells, tiles_bound, extras.fixed_memory);
    if (const char* text = std::getenv("VESIN_HIP_ORDERED_SHARE")) {
        // (for measurements and tests: a power of two)
        uint32_t wanted = static_cast<uint32_t>(std::max(1, std::min<int>(TILE_POINTS, std::atoi(text))));
        while ((wanted & (wanted - 1)) != 0) {
            wanted &= wanted - 1;
        }
        ordered_points_per_item = wanted;
    }
    const uint32_t ordered_items_per_tile = TILE_POINTS / ordered_points_per_item;
    const uint32_t ordered_blocks =
        static_cast<uint32_t>((tiles_bound * ordered_items_per_tile + ORDERED_WAVES - 1) / ORDERED_WAVES);
    const size_t ordered_record_bytes =
        static_cast<size_t>(ordered_blocks) * ORDERED_WAVES * ORDERED_UNITS * WAVE * sizeof(CandidateRecord);
    if (try_in_order && !extras.fixed_memory && !ordered_records_fit(n_points, ordered_record_bytes)) {
        try_in_order = false; // a sparse system of many cells: see ordered_records_fit
    }
    const size_t scratch_elements = std::max(
        std::max(scan_scratch_elements(n_cells), scan_scratch_elements(n_slots)),
        try_in_order ? scan_scratch_elements(n_points) : 0
    );

    auto carve = [&](Carver& carver) {
        // adjacent, so that one fill clears the histogram, the tiles' flags and the state of the single-pass search
        cell_counts = carver.take<uint32_t>(n_cells);
        tiles = carver.take<Tile>(tiles_bound);
        chain.blocks = carver.take<uint64_t>(search_workgroups);
        chain.groups = carver.take<uint64_t>(chain_groups);
        chain.bases = carver.take<uint64_t>(chain_groups);
        direct_wrapped = carver.take<uint32_t>(direct_slots);
        fused_status = carver.take<FusedStatus>(1);
        ordered_status = carver.take<OrderedStatus>(1);
        // (behind the state that every call clears: place_points wants them cleared too)
        sorted.wx = carver.take<int32_t>(sorted_slots + SORTED_PADDING);
        sorted.wy = carver.take<int32_t>(sorted_slots + SORTED_PADDING);
        sorted.wz = carver.take<int32_t>(sorted_slots + SORTED_PADDING);
        if (try_in_order) {
            rows_of_point = carver.take<uint32_t>(n_points); // (cleared as well: its counting pass may add to it)
        }

        wraps_end = reinterpret_cast<char*>(carver.take<uint32_t>(0));
        cell_scan = carver.take<uint64_t>(n_cells + 1);
        if (!single_cell) {
            cell_of = carver.take<uint32_t>(n_points);
            slot_of = carver.take<uint32_t>(n_points);
            wrap_of = carver.take<int32_t>(3 * n_points);
            provisional = carver.take<uint32_t>(n_points);
        }
        sorted.p = carver.take<SortedPoint>(sorted_slots + SORTED_PADDING);
        // (the places of the points inside their cells, for the single-precision pre-test of the in-order search's
        // counting pass; the cell builds of small systems and of the reproducible order do not fill them in)
        sorted.l = try_in_order && pre.use32 != 0 && !small_build && !ordered_rows()
                       ? carver.take<float4>(sorted_slots + SORTED_PADDING)
                       : nullptr;
        counts = carver.take<uint32_t>(std::max(n_slots, direct_slots * n_slices));
        offsets = carver.take<uint64_t>(std::max(n_slots, direct_slots * n_slices) + 1);
        scan_scratch = carver.take<uint64_t>(scratch_elements);
        rows_of_item = carver.take<uint32_t>(small_items);
        if (try_in_order) {
            first_row_of_point = carver.take<uint64_t>(n_points + 1);
            candidate_records = carver.take<CandidateRecord>(static_cast<size_t>(ordered_blocks) * ORDERED_WAVES * ORDERED_UNITS * WAVE);
            candidates_of_item = carver.take<uint32_t>(static_cast<size_t>(ordered_blocks) * ORDERED_WAVES);
            if (ordered_items_per_tile == 1) {
                candidate_order = carver.take<uint16_t>(tiles_bound * ORDERED_CANDIDATES);
            }

        }
    };
    Carver measure(nullptr);
    carve(measure);
    extras.work.reserve(measure.used);
    Carver carver(extras.work.ptr);
    carve(carver);
    extras.batch.on_device = false; // what a batch left in this buffer is about to be overwritten

    auto check_pair_limit = [&](size_t total) {
        if (pair_limit != 0 && total > n_points * pair_limit) {
            throw std::runtime_error(
                "The number of neighbor pairs exceeds the maximum capacity of " + std::to_string(n_points * pair_limit) +
                " (max_pairs_per_point=" + std::to_string(pair_limit) + "; n_points=" + std::to_string(n_points) + "). " +
                "Consider reducing the cutoff distance, or explicitly setting " +
                "VESIN_CUDA_MAX_PAIRS_PER_POINT as an environment variable."
            );
        }
    };

    // (for a queued call: see HipExtras::publish_length)
    auto queued_outcome = [&](int kind) {
        QueuedOutcome outcome = {};
        outcome.kind = kind;
        outcome.build = extras.d_status;
        outcome.capacity = extras.capacity;
        outcome.row_limit = pair_limit != 0 ? n_points * pair_limit : 0;
        std::memcpy(outcome.used_box, used_box, BOX_BYTES);
        return outcome;
    };

    // ---- small systems with arrays from earlier calls: cell list, counting, scan, report to the host and writing
    // in one launch (small_system_kernel). Its workgroups wait for each other, which needs all of them resident at
    // once; when they were not, or the system does not suit that launch, or the rows do not fit, the call goes on
    // as if nothing had happened, and (except in the last case) the list leaves that launch alone for a while.
    const bool guessed_grid = remembered_extent && !one_launch && try_single_pass && !single_cell && !small_build;
    if (remembered_extent && !one_launch && !guessed_grid) {
        // the grid came from an extent that only these two ways refresh: start over with a pass over the points
        // (nothing is known against the box: its guess is not to be blamed)
        extras.extent_missed = true;
        return false;
    }
    if (one_launch) {
        HOST_LAP(2);
        size_outputs(neighbors, extras, 0, options);
        SmallArgs sargs = {};
        sargs.points = reinterpret_cast<const double*>(points);
        sargs.box = fetched ? nullptr : reinterpret_cast<const double*>(box);
        sargs.periodic = periodic;
        sargs.host_small = extras.mail_device->small;
        sargs.rows_of_item = rows_of_item;
        sargs.n_slices = small_slices;
        sargs.meeting = extras.meetings + (extras.meeting_turn & 1u);
        sargs.next_meeting = extras.meetings + ((extras.meeting_turn + 1u) & 1u);
        extras.meeting_turn += 1;
        sargs.host = &extras.mail_device->ordered;
        sargs.host_bounds = any_open ? extras.mail_device->bounds : nullptr;
        sargs.spin_limit = std::min(chain_spin_limit(), SMALL_SPINS);
        sargs.capacity = extras.capacity;
        sargs.out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
        sargs.out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
        sargs.out.distances = neighbors.distances;
        sargs.out.vectors = reinterpret_cast<double*>(neighbors.vectors);
        // few waves per workgroup when that still covers the items: the arithmetic spreads over more compute units
        if (!options.sorted) {
            auto kernel = options.full ? small_system_kernel<true, 4, false> : small_system_kernel<false, 4, false>;
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>((small_items + 3) / 4)), dim3(4 * WAVE), 0, stream, sargs, g);
        } else if (n_points <= SmallShape<4>::MAX_ITEMS && n_cells <= SmallShape<4>::CAPACITY) {
            auto kernel = options.full ? small_system_kernel<true, 4, true> : small_system_kernel<false, 4, true>;
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>((n_points + 3) / 4)), dim3(4 * WAVE), 0, stream, sargs, g);
        } else if (n_points <= SmallShape<8>::MAX_ITEMS) {
            auto kernel = options.full ? small_system_kernel<true, 8, true> : small_system_kernel<false, 8, true>;
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>((n_points + 7) / 8)), dim3(8 * WAVE), 0, stream, sargs, g);
        } else {
            auto kernel = options.full ? small_system_kernel<true, 16, true> : small_system_kernel<false, 16, true>;
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>((n_points + 15) / 16)), dim3(16 * WAVE), 0, stream, sargs, g);
        }
        fetched = true;
        HOST_LAP(3);
        mark(T_CELLS);
        mark(T_WRITE);
        bool published_here = false;
        {
            QueuedOutcome outcome = queued_outcome(1);
            outcome.small = &extras.mail_device->ordered;
            published_here = extras.publish_length(outcome, reinterpret_cast<const double*>(box), periodic, stream);
        }
        extras.wait(stream, any_open ? 1 : 0);
        HOST_LAP(4);
        if (!box_was_right()) {
            return false;
        }
        const OrderedHostStatus found = extras.mail->ordered;
        if (found.first_bad_coordinate != 0xFFFFFFFFu) {
            non_finite_error(points, found.first_bad_coordinate);
        }
        const bool suitable = found.found.gave_up == 0 && found.found.max_rows <= ORDERED_MAX_ROWS &&
                              found.found.max_candidates <= ORDERED_CANDIDATES && found.found.unsuitable == 0;
        if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
            std::fprintf(
                stderr, "one launch: rows %llu, %u items per point, most rows of a point %u, most candidates of an item %u, unsuitable %u, gave up %u\n",
                found.total_rows, small_slices, found.found.max_rows, found.found.max_candidates, found.found.unsuitable,
                found.found.gave_up
            );
        }
        if (suitable && found.total_rows <= extras.capacity) {
            extras.meeting_rest.went_through();
            check_pair_limit(found.total_rows);
            extras.queued_part_sufficed = published_here;
            HIP_CHECK(hipGetLastError());
            neighbors.length = found.total_rows;
            if (any_open) {
                const BlockBounds& fresh = extras.mail->bounds[0];
                for (int d = 0; d < 3; d++) {
                    extras.extent_lo[d] = fresh.lo[d];
                    extras.extent_hi[d] = fresh.hi[d];
                }
                extras.extent_valid = true;
            }
            if (timed) {
                float ms = 0.0f;
                HIP_CHECK(hipEventElapsedTime(&ms, extras.events[T_START], extras.events[T_WRITE]));
                extras.timings = {};
                extras.timings.total = ms;
                extras.timings.write = ms;
                extras.timings_valid = true;
            }
            return true;
        }
        if (found.found.gave_up != 0) {
            // the workgroups were not all running at once (a GPU shared with other work): the separate launches take
            // over, for longer and longer while that keeps happening
            extras.meeting_rest.gave_up();
        } else {
            extras.meeting_rest.went_through();
            if (!suitable) {
                // (rows that do not fit are no reason: the arrays grow below and the next call finds room)
                extras.one_launch_rest = SINGLE_PASS_REST;
            }
        }
    }

    // ---- cell list
    const uint32_t point_blocks = static_cast<uint32_t>((n_points + BLOCK - 1) / BLOCK);
    const uint32_t bounding_blocks = std::min<uint32_t>(BOUNDING_BLOCKS, point_blocks);
    const auto* flat_points = reinterpret_cast<const double*>(points);
    auto clear_work_state = [&](bool wraps_too) {
        // every piece of the work buffer is padded to 256 bytes: clearing whole 16-byte blocks stays inside
        const char* end = wraps_too ? wraps_end : reinterpret_cast<char*>(ordered_status + 1);
        const size_t to_clear = end - reinterpret_cast<char*>(cell_counts);
        const size_t blocks16 = (to_clear + 15) / 16;
        const uint32_t fill_blocks = static_cast<uint32_t>(std::min<size_t>(1024, (blocks16 + BLOCK - 1) / BLOCK));
        if (guessed_grid) {
            // ... and the extent of this call's points, for the call after it
            hipLaunchKernelGGL(
                clear_fetch_and_bound, dim3(fill_blocks + bounding_blocks), dim3(BLOCK), 0, stream,
                fill_blocks, reinterpret_cast<uint4*>(cell_counts), blocks16,
                fetched ? static_cast<const double*>(nullptr) : reinterpret_cast<const double*>(box), periodic,
                extras.mail_device->small, extras.d_status, flat_points, g.n_points, g, extras.mail_device->bounds
            );
            fetched = true;
            return;
        }
        hipLaunchKernelGGL(
            clear_and_fetch, dim3(fill_blocks), dim3(BLOCK), 0, stream,
            reinterpret_cast<uint4*>(cell_counts), blocks16,
            fetched ? static_cast<const double*>(nullptr) : reinterpret_cast<const double*>(box), periodic,
            extras.mail_device->small, extras.d_status
        );
        fetched = true;
    };
    auto build_packed_cells = [&]() {
        if (single_cell) {
            hipLaunchKernelGGL(
                prepare_single_cell, dim3(point_blocks), dim3(BLOCK), 0, stream,
                flat_points, g, sorted, tiles, cell_scan, extras.d_status, static_cast<uint4*>(nullptr), size_t(0),
                static_cast<const double*>(nullptr), static_cast<const bool*>(nullptr), static_cast<unsigned char*>(nullptr), pre
            );
            return;
        }
        const bool ordered = ordered_rows();
        hipLaunchKernelGGL(
            assign_cells, dim3(point_blocks), dim3(BLOCK), 0, stream,
            flat_points, g, ordered ? cell_of : static_cast<uint32_t*>(nullptr), slot_of,
            ordered ? wrap_of : static_cast<int32_t*>(nullptr), cell_counts, extras.d_status
        );
        exclusive_scan<SCAN_CELL_COUNTS>(cell_counts, n_cells, cell_scan, scan_scratch, stream);
        if (ordered) {
            // the same order of the points inside every cell on every run
            hipLaunchKernelGGL(
                scatter_points, dim3(point_blocks), dim3(BLOCK), 0, stream,
                g.n_points, cell_of, slot_of, cell_scan, provisional
            );
            hipLaunchKernelGGL(
                gather_points, dim3(point_blocks), dim3(BLOCK), 0, stream,
                flat_points, wrap_of, cell_of, provisional, cell_scan, g.n_points, sorted, tiles
            );
        } else {
            hipLaunchKernelGGL(
                place_points, dim3(point_blocks), dim3(BLOCK), 0, stream,
                flat_points, g, static_cast<const int32_t*>(nullptr), static_cast<const uint32_t*>(nullptr), slot_of,
                cell_scan, g.n_points, sorted, tiles,
                static_cast<const uint32_t*>(nullptr), static_cast<const uint32_t*>(nullptr), pre
            );
        }
    };
    if (small_build) {
        const size_t to_clear = reinterpret_cast<char*>(ordered_status + 1) - reinterpret_cast<char*>(cell_counts);
        hipLaunchKernelGGL(
            build_cells_small, dim3(1), dim3(SMALL_BUILD_THREADS), 0, stream,
            flat_points, g, reinterpret_cast<uint4*>(cell_counts), (to_clear + 15) / 16,
            fetched ? static_cast<const double*>(nullptr) : reinterpret_cast<const double*>(box), periodic,
            extras.mail_device->small, sorted, tiles, cell_scan, extras.d_status
        );
        fetched = true;
    } else if (single_cell && point_blocks == 1) {
        // the single cell of a small system: one launch prepares it, clears the state of the search and fetches the box
        char* first = reinterpret_cast<char*>(chain.blocks);
        const size_t to_clear = reinterpret_cast<char*>(ordered_status + 1) - first;
        hipLaunchKernelGGL(
            prepare_single_cell, dim3(1), dim3(BLOCK), 0, stream,
            flat_points, g, sorted, tiles, cell_scan, extras.d_status, reinterpret_cast<uint4*>(first), (to_clear + 15) / 16,
            fetched ? static_cast<const double*>(nullptr) : reinterpret_cast<const double*>(box), periodic, extras.mail_device->small,
            pre
        );
        fetched = true;
    } else if (direct_cells) {
        clear_work_state(true);
        hipLaunchKernelGGL(
            place_direct, dim3(point_blocks), dim3(BLOCK), 0, stream,
            flat_points, g, DIRECT_CAPACITY, cell_counts, direct_wrapped, sorted, extras.d_status
        );
    } else {
        clear_work_state(!single_cell);
        build_packed_cells();
    }
    mark(T_CELLS);

    SearchArgs args = {};
    args.sorted = sorted;
    args.cell_scan = cell_scan;
    args.tiles = tiles;
    args.counts = counts;
    args.offsets = offsets;
    args.n_slices = n_slices;
    args.n_work = static_cast<uint32_t>(search_blocks);

    auto outputs_of = [&]() {
        SearchOutputs out;
        out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
        out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
        out.distances = neighbors.distances;
        out.vectors = reinterpret_cast<double*>(neighbors.vectors);
        return out;
    };
    auto elapsed = [&](Stage from, Stage to) {
        float ms = 0.0f;
        HIP_CHECK(hipEventElapsedTime(&ms, extras.events[from], extras.events[to]));
        return ms;
    };

    // ---- single-pass search straight into the arrays kept from earlier calls
    if (try_single_pass) {
        size_outputs(neighbors, extras, 0, options);
        FusedArgs fargs = {};
        fargs.search = args;
        fargs.search.out = outputs_of();
        fargs.search.capacity = extras.capacity;
        fargs.chain = chain;
        fargs.first_rows = offsets;
        fargs.status = fused_status;
        fargs.spin_limit = chain_spin_limit();
        fargs.wait_ticks = chain_wait_ticks();
        uint32_t blocks = static_cast<uint32_t>(search_workgroups);
        if (direct_cells) {
            fargs.search.direct_capacity = DIRECT_CAPACITY;
            fargs.search.direct_counts = cell_counts;
            fargs.search.direct_wrapped = direct_wrapped;
            fargs.search.n_work = static_cast<uint32_t>(direct_slots * n_slices);
            blocks = static_cast<uint32_t>(direct_slots * n_slices / SEARCH_WAVES);
        }
        const bool ordered = ordered_rows();
        // Calls that return vectors take the kernels that line them up in LDS before they store them. Measured on
        // 1,000,000 atoms of diamond (ms per call, row by row -> lined up): full lists i j S d D 1.565 -> 1.129, i j D
        // 1.176 -> 0.779; half lists i j S d D 0.791 -> 0.614, i j D 0.502 -> 0.506 (0.571 -> 0.628 on 500,000
        // clustered atoms: a half list that stores little else is not held up by its stores, and stays as it was).
        const bool staged = staged_vectors(fargs.search.out, options.full);
        auto kernel =
            staged ? (options.full ? (ordered ? fused_search_kernel<true, true, false, true> : fused_search_kernel<true, false, false, true>)
                                   : (ordered ? fused_search_kernel<false, true, false, true> : fused_search_kernel<false, false, false, true>))
                   : (options.full ? (ordered ? fused_search_kernel<true, true> : fused_search_kernel<true, false>)
                                   : (ordered ? fused_search_kernel<false, true> : fused_search_kernel<false, false>));
        hipLaunchKernelGGL(kernel, dim3(blocks), dim3(SEARCH_BLOCK), 0, stream, fargs, g);
        mark(T_WRITE);
        hipLaunchKernelGGL(publish_fused_status, dim3(1), dim3(1), 0, stream, extras.d_status, fused_status, &extras.mail_device->fused);
        bool published_here = false;
        {
            QueuedOutcome outcome = queued_outcome(0);
            outcome.fused = fused_status;
            outcome.one_pass_cells = direct_cells ? 1 : 0;
            outcome.guessed_extent = guessed_grid ? 1 : 0;
            published_here = extras.publish_length(outcome, reinterpret_cast<const double*>(box), periodic, stream);
        }
        extras.wait(stream, guessed_grid ? bounding_blocks : 0);
        if (!box_was_right()) {
            return false;
        }
        const FusedStatus result = extras.mail->fused;
        if (result.first_bad_coordinate != 0xFFFFFFFFu) {
            non_finite_error(points, result.first_bad_coordinate);
        }
        if (guessed_grid) {
            if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
                std::fprintf(stderr, "grid from the extent of the call before: %u points far outside\n", result.far_outside);
            }
            if (result.far_outside != 0) {
                // the points are somewhere else altogether: those were left out, the call starts over with the
                // same box, and the list finds the extent first for a while
                extras.extent_rest = EXTENT_REST;
                extras.extent_missed = true;
                return false;
            }
            for (int d = 0; d < 3; d++) {
                extras.extent_lo[d] = INFINITY;
                extras.extent_hi[d] = -INFINITY;
            }
            for (uint32_t block = 0; block < bounding_blocks; block++) {
                const BlockBounds& part = extras.mail->bounds[block];
                for (int d = 0; d < 3; d++) {
                    extras.extent_lo[d] = std::fmin(extras.extent_lo[d], part.lo[d]);
                    extras.extent_hi[d] = std::fmax(extras.extent_hi[d], part.hi[d]);
                }
            }
            extras.extent_valid = true;
        }
        if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
            uint32_t stencil_cells = 0;
            uint32_t stencil_kept = 0;
            for (int32_t dx = -g.s[0]; dx <= g.s[0]; dx++) {
                for (int32_t dy = -g.s[1]; dy <= g.s[1]; dy++) {
                    for (int32_t dz = -g.s[2]; dz <= g.s[2]; dz++) {
                        stencil_cells += 1;
                        stencil_kept += stencil_entry_too_far(g, dx, dy, dz) ? 0 : 1;
                    }
                }
            }
            std::fprintf(
                stderr,
                "single pass: rows %llu general %u deferred %u overflow %u timeout %u (cells %u %u %u, capacity %zu, %s%u, "
                "stencil %u of %u)\n",
                result.total_rows, result.general, result.deferred, result.overflow, result.chain_timeout, g.n[0], g.n[1], g.n[2],
                extras.capacity, direct_cells ? "one-pass cell build, crowded " : "packed cells, crowded ", result.crowded_cells,
                stencil_kept, stencil_cells
            );
        }
        // the one-pass cell build is void when a cell overflowed, and the write pass cannot read its layout
        const bool cells_ok = !direct_cells || (result.crowded_cells == 0 && result.deferred == 0);
        // a wave that gave up waiting for another workgroup's rows wrote its own at the wrong place: like a system
        // that kernel does not cover, the call starts over with the two passes
        if (result.general == 0 && result.overflow == 0 && cells_ok && result.chain_timeout == 0) {
            check_pair_limit(result.total_rows);
            if (result.deferred != 0) {
                // work items too large for the single pass: their rows are counted and placed, the write pass of
                // the two-pass search produces them
                SearchArgs rest = fargs.search;
                rest.only = counts;
                rest.capacity = ~0ull;
                launch_search<true>(options.full, rest, g, stream);
                mark(T_WRITE);
                HIP_CHECK(hipStreamSynchronize(stream));
                if (result.deferred_rows > result.total_rows / 8) {
                    // a system dominated by crowded tiles is searched twice this way: the two passes do better
                    extras.single_pass_rest = SINGLE_PASS_REST;
                }
            }
            HIP_CHECK(hipGetLastError());
            neighbors.length = result.total_rows;
            extras.queued_part_sufficed = published_here && result.deferred == 0;
            if (ordered) {
                extras.chain_rest.went_through();
            }
            if (timed) {
                extras.timings = {};
                extras.timings.total = elapsed(T_START, T_WRITE);
                extras.timings.cell_build = elapsed(T_START, T_CELLS);
                extras.timings.write = elapsed(T_CELLS, T_WRITE);
                extras.timings_valid = true;
            }
            return true;
        }
        if (result.general != 0) {
            // the shape of this system is not the single-pass kernel's: leave it alone for a while
            extras.single_pass_rest = SINGLE_PASS_REST;
        }
        if (result.chain_timeout != 0) {
            extras.chain_rest.gave_up();
        }
        if (direct_cells) {
            // everything below reads the packed layout: build it now
            if (!cells_ok) {
                extras.direct_rest = DIRECT_REST;
            }
            clear_work_state(!single_cell);
            build_packed_cells();
        }
    }

    // ---- a sorted list straight from the search, when the system has the shape that search covers
    if (try_in_order && n_points > 0) {
        OrderedArgs oargs = {};
        oargs.sorted = sorted;
        oargs.cell_scan = cell_scan;
        oargs.tiles = tiles;
        oargs.points_per_item = ordered_points_per_item;
        oargs.items_per_tile = ordered_items_per_tile;
        oargs.rows_of_point = rows_of_point;
        oargs.records = candidate_records;
        oargs.candidates_of_item = candidates_of_item;
        // How many waves share a tile in either pass follows the number of tiles the call before had on the same
        // number of points (policy.hpp); a list's first call on a system keeps one wave per tile.
        const size_t tiles_before = ordered_items_per_tile == 1 && extras.ordered_tiles_points == n_points ? extras.ordered_tiles : 0;
        oargs.write_split = ordered_write_split(n_points, tiles_before);
        if (const char* text = std::getenv("VESIN_HIP_WRITE_SPLIT")) {
            oargs.write_split = static_cast<uint32_t>(std::max(1, std::min(4, std::atoi(text))));
        }
        // (the waves of a tile add their rows in memory that the cell build cleared)
        const bool rows_cleared = !single_cell && !small_build;
        oargs.count_split = rows_cleared ? ordered_count_split(n_points, tiles_before) : 1;
        if (const char* text = std::getenv("VESIN_HIP_COUNT_SPLIT")) {
            oargs.count_split = rows_cleared ? static_cast<uint32_t>(std::max(1, std::min(4, std::atoi(text)))) : 1u;
        }
        oargs.points = reinterpret_cast<const double*>(points);
        oargs.pre = pre;
        oargs.order = candidate_order;
        oargs.first_row = first_row_of_point;
        oargs.status = ordered_status;
        oargs.report_order = std::getenv("VESIN_HIP_DEBUG") != nullptr ? 1u : 0u;
        const uint32_t blocks = ordered_blocks;
        // The order of every tile's candidates, for the writing pass (wasted when the counting pass finds the
        // system unsuitable, which the host only knows after both). Small systems do without: one more launch
        // costs them more than ranking the rows of every point does. It reads the cell list only, like the
        // counting pass, and neither fills the GPU on systems of a few hundred thousand points (one wave per tile,
        // two waves per SIMD on 100,000 points): the two run side by side, the ordering on a stream of the list's
        // own that starts after the cell build and that the call's stream waits for right after the counting pass.
        const bool presorted = ordered_items_per_tile == 1;
        auto launch_order = [&](hipStream_t where) {
            hipLaunchKernelGGL(
                ordered_sort_kernel<false>, dim3(static_cast<uint32_t>((tiles_bound + ORDER_WAVES - 1) / ORDER_WAVES)),
                dim3(ORDER_BLOCK), 0, where, oargs, g
            );
        };
        auto launch_write = [&]() {
            auto kernel = presorted ? (options.full ? ordered_search_kernel<true, true, true> : ordered_search_kernel<true, false, true>)
                                    : (options.full ? ordered_search_kernel<true, true, false> : ordered_search_kernel<true, false, false>);
            hipLaunchKernelGGL(kernel, dim3(blocks * oargs.write_split), dim3(ORDERED_BLOCK), 0, stream, oargs, g);
        };
        // A list that has arrays from earlier calls writes into them without waiting for the host to learn what the
        // counting pass found: the launch checks on the device that the system suits this search and that the rows
        // fit, and writes nothing otherwise. One round trip to the host instead of two.
        const bool early_write = extras.capacity > 0;
        size_t early_capacity = 0;
        bool published_here = false;
        if (early_write) {
            size_outputs(neighbors, extras, 0, options);
            early_capacity = extras.capacity;
            oargs.out = outputs_of();
            oargs.capacity = early_capacity;
            oargs.guarded = 1;
        }
        auto launch_count_and_scan = [&]() {
            hipStream_t side = presorted && !ordered_one_stream() ? extras.side() : nullptr;
            if (side != nullptr) {
                HIP_CHECK(hipEventRecord(extras.side_fork, stream));
                HIP_CHECK(hipStreamWaitEvent(side, extras.side_fork, 0));
                launch_order(side);
                HIP_CHECK(hipEventRecord(extras.side_join, side));
            }
            if (options.full) {
                hipLaunchKernelGGL((ordered_search_kernel<false, true>), dim3(blocks * oargs.count_split), dim3(ORDERED_BLOCK), 0, stream, oargs, g);
            } else {
                hipLaunchKernelGGL((ordered_search_kernel<false, false>), dim3(blocks * oargs.count_split), dim3(ORDERED_BLOCK), 0, stream, oargs, g);
            }
            if (side != nullptr) {
                HIP_CHECK(hipStreamWaitEvent(stream, extras.side_join, 0));
            } else if (presorted) {
                launch_order(stream);
            }
            mark(T_COUNT);
            exclusive_scan<SCAN_U32>(rows_of_point, n_points, first_row_of_point, scan_scratch, stream);
            mark(T_SCAN);
        };
        {
            launch_count_and_scan();
            if (early_write) {
                // (the launch's first wave tells the host what the counting pass found)
                oargs.publish_to = &extras.mail_device->ordered;
                oargs.build_status = extras.d_status;
                mark(T_WRITE_BEGIN);
                launch_write();
                mark(T_WRITE);
                oargs.publish_to = nullptr;
                QueuedOutcome outcome = queued_outcome(2);
                outcome.ordered = ordered_status;
                outcome.ordered_total = first_row_of_point + n_points;
                outcome.capacity = early_capacity;
                published_here = extras.publish_length(outcome, reinterpret_cast<const double*>(box), periodic, stream);
            } else {
                hipLaunchKernelGGL(
                    publish_ordered_status, dim3(1), dim3(1), 0, stream,
                    ordered_status, first_row_of_point + n_points, extras.d_status, cell_scan + n_cells,
                    &extras.mail_device->ordered
                );
            }
            extras.wait(stream);
            if (!box_was_right()) {
                return false;
            }
        }
        const OrderedHostStatus found = extras.mail->ordered;
        if (found.first_bad_coordinate != 0xFFFFFFFFu) {
            non_finite_error(points, found.first_bad_coordinate);
        }
        extras.ordered_tiles = found.n_tiles;
        extras.ordered_tiles_points = n_points;
        const bool suitable = found.found.max_rows <= ORDERED_MAX_ROWS &&
                              found.found.max_candidates <= ORDERED_CANDIDATES && found.found.unsuitable == 0;
        if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
            std::fprintf(
                stderr,
                "in-order search: rows %llu, most rows of a point %u, most candidates of a tile %u, unsuitable %u, "
                "candidates of %u tiles ordered by window and of %u by buckets, %u tiles written by %u waves each and counted by %u: %s\n",
                found.total_rows, found.found.max_rows, found.found.max_candidates, found.found.unsuitable,
                found.found.windowed, found.found.bucketed, found.n_tiles, oargs.write_split, oargs.count_split,
                suitable ? "used" : "left to the radix sort"
            );
        }
        if (suitable) {
            const size_t total = found.total_rows;
            check_pair_limit(total);
            if (!(early_write && total <= early_capacity)) {
                // first call of the list, or more rows than its arrays hold
                size_outputs(neighbors, extras, total, options);
                oargs.out = outputs_of();
                oargs.guarded = 0;
                mark(T_WRITE_BEGIN);
                if (total > 0) {
                    launch_write();
                }
                mark(T_WRITE);
                mark(T_SORT);
                HIP_CHECK(hipStreamSynchronize(stream));
            } else {
                extras.queued_part_sufficed = published_here;
                mark(T_SORT);
                if (timed) {
                    HIP_CHECK(hipStreamSynchronize(stream));
                }
            }
            HIP_CHECK(hipGetLastError());
            neighbors.length = total;
            if (timed) {
                extras.timings = {};
                extras.timings.total = elapsed(T_START, T_SORT);
                extras.timings.cell_build = elapsed(T_START, T_CELLS);
                extras.timings.count = elapsed(T_CELLS, T_COUNT);
                extras.timings.scan = elapsed(T_COUNT, T_SCAN);
                extras.timings.write = elapsed(T_WRITE_BEGIN, T_WRITE);
                extras.timings_valid = true;
            }
            return true;
        }
        // rows per point, candidates per tile or shifts beyond what that search handles: the general way below,
        // and for a while without asking again
        extras.in_order_rest = SINGLE_PASS_REST;
    }

    // ---- pass 1: count
    launch_search<false>(options.full, args, g, stream);
    mark(T_COUNT);

    exclusive_scan<SCAN_U32>(counts, n_slots, offsets, scan_scratch, stream);
    mark(T_SCAN);

    hipLaunchKernelGGL(publish_status, dim3(1), dim3(1), 0, stream, extras.d_status, offsets + n_slots, &extras.mail_device->status);

    // ---- pass 2: write. Without sorting the rows go straight to the caller's arrays, and the launch does not
    // wait for the host to learn their number: the arrays keep the capacity of earlier calls, and a launch that
    // would overflow them writes nothing and is repeated once they have grown.
    const bool speculative = !options.sorted;
    if (speculative) {
        size_outputs(neighbors, extras, 0, options);
        args.out = outputs_of();
        args.capacity = extras.capacity;
        mark(T_WRITE_BEGIN);
        launch_search<true>(options.full, args, g, stream);
        mark(T_WRITE);
    }

    extras.wait(stream);
    if (!box_was_right()) {
        return false;
    }
    if (extras.mail->status.first_bad_coordinate != 0xFFFFFFFFu) {
        non_finite_error(points, extras.mail->status.first_bad_coordinate);
    }
    const size_t total = extras.mail->status.total_pairs;

    check_pair_limit(total);

    const bool fits = total <= extras.capacity;
    size_outputs(neighbors, extras, total, options);
    const SearchOutputs final_out = outputs_of();

    const bool sorting = options.sorted && total > 1;
    SearchOutputs unsorted = final_out;
    SortWorkspace sort_space = {};
    sort_space.host_ranges = extras.mail->ranges;
    sort_space.device_ranges = extras.mail_device->ranges;
    if (sorting) {
        carve_sort_space(extras, total, options, unsorted, sort_space);
    }

    if (!speculative || !fits) {
        mark(T_WRITE_BEGIN);
        if (total > 0) {
            args.out = unsorted;
            args.capacity = sorting ? total : extras.capacity;
            launch_search<true>(options.full, args, g, stream);
        }
        mark(T_WRITE);
    }

    if (sorting) {
        sort_pairs(unsorted, final_out, total, n_points, sort_space, stream);
    }
    mark(T_SORT);

    if (!speculative || !fits || timed) {
        HIP_CHECK(hipStreamSynchronize(stream));
    }
    HIP_CHECK(hipGetLastError());
    neighbors.length = total;

    if (timed) {
        extras.timings.total = elapsed(T_START, T_SORT);
        extras.timings.cell_build = elapsed(T_START, T_CELLS);
        extras.timings.count = elapsed(T_CELLS, T_COUNT);
        extras.timings.scan = elapsed(T_COUNT, T_SCAN);
        extras.timings.write = elapsed(T_WRITE_BEGIN, T_WRITE);
        extras.timings.sort = elapsed(T_WRITE, T_SORT);
        extras.timings.candidates = 0;
        extras.timings_valid = true;
    }
    return true;
}

} // namespace


namespace {

/// options.skin > 0: filter the cached candidates, after rebuilding them when they no longer cover the points
/// (reference: vesin/src/cpu_cell_list.cpp:222-234, vesin/src/verlet.cpp). In the steady state a call is two
/// launches (the check together with the filter's counting pass; the writing pass), with a scan of the counts
/// between them for lists of more than 0.5 M candidates, and one synchronisation; the filter writes straight into the arrays the list kept, and is
/// repeated when they turn out too small or when the check asks for new candidates. Sorted lists come from sorted
/// candidates: the filter keeps their order.
void verlet_neighbors(
    const double (*points)[3], size_t n_points, const double box[3][3], const bool periodic[3], VesinOptions options,
    VesinNeighborList& neighbors, HipExtras& extras, hipStream_t stream
) {
    if (extras.verlet == nullptr) {
        auto cache = std::make_unique<VerletCache>();
        HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&cache->reference), sizeof(VerletReference)));
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&cache->status), sizeof(VerletStatus), hipHostMallocDefault));
        extras.verlet = cache.release();
    }
    VerletCache& cache = *extras.verlet;
    const size_t pair_limit = pairs_per_point_limit();

    // same triggers as the reference (vesin/src/verlet.cpp:48-54, :65-71)
    const bool options_changed = cache.options.cutoff != options.cutoff || cache.options.skin != options.skin ||
                                 cache.options.full != options.full || cache.options.sorted != options.sorted;
    bool fresh = false;
    auto rebuild = [&]() {
        cache.valid = false;
        VesinOptions build = {};
        build.cutoff = options.cutoff + options.skin;
        build.full = options.full;
        build.sorted = options.sorted; // sorted rows come from sorted candidates: the filter keeps their order
        build.algorithm = VesinCellList;
        build.n_threads = options.n_threads;
        build.return_shifts = true;
        build.return_distances = false;
        build.return_vectors = false;
        build.skin = 0.0;
        cache.candidates.device = neighbors.device;
        vesin_hip::neighbors(points, n_points, box, periodic, build, cache.candidates, stream);

        if (cache.ref_capacity < n_points) {
            if (cache.ref_points != nullptr) {
                (void)hipFree(cache.ref_points);
                cache.ref_points = nullptr;
                cache.ref_capacity = 0;
            }
            const size_t capacity = n_points + n_points / 8 + 64;
            HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&cache.ref_points), capacity * 3 * sizeof(double)));
            cache.ref_capacity = capacity;
        }
        if (n_points > 0) {
            HIP_CHECK(hipMemcpyAsync(
                cache.ref_points, points, n_points * 3 * sizeof(double), hipMemcpyDeviceToDevice, stream
            ));
        }
        hipLaunchKernelGGL(
            verlet_store_reference, dim3(1), dim3(64), 0, stream, reinterpret_cast<const double*>(box), periodic,
            cache.reference
        );
        if (cache.candidates.length > 0) {
            // (how far the shifts of the candidates reach: what the box may change by before they are computed again
            // depends on it, see verlet_check_and_count_kernel)
            const uint32_t blocks = static_cast<uint32_t>(std::min<size_t>(1024, (cache.candidates.length + VERLET_BLOCK - 1) / VERLET_BLOCK));
            hipLaunchKernelGGL(
                verlet_shift_reach_kernel, dim3(blocks), dim3(VERLET_BLOCK), 0, stream,
                reinterpret_cast<const int32_t*>(cache.candidates.shifts), cache.candidates.length, cache.reference
            );
        }
        // the snapshot is complete before the call returns: the caller may change points and box right after
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(stream));
        cache.options = options;
        cache.n_ref = n_points;
        cache.valid = true;
        fresh = true;
    };
    // VESIN_HIP_VERLET=cache / direct takes the choice between filtering and searching away from the estimate
    const char* forced = std::getenv("VESIN_HIP_VERLET");
    const bool force_cache = forced != nullptr && std::strcmp(forced, "cache") == 0;
    const bool force_direct = forced != nullptr && std::strcmp(forced, "direct") == 0;
    auto too_long_for_a_filter = [&](size_t rows) {
        const double ratio = (options.cutoff + options.skin) / options.cutoff;
        const double candidates = static_cast<double>(rows) * ratio * ratio * ratio;
        const size_t limit = options.sorted ? VERLET_MAX_CANDIDATES_SORTED : VERLET_MAX_CANDIDATES;
        return force_direct || (!force_cache && candidates > static_cast<double>(limit));
    };
    if (options_changed || cache.direct_n_points != n_points) {
        cache.direct = false;
        cache.lifetime.reset();
    }
    auto drop_candidates = [&]() {
        if (cache.valid) {
            free_neighbors(cache.candidates);
            cache.candidates = VesinNeighborList();
            cache.valid = false;
        }
    };
    if (!cache.valid || options_changed || cache.n_ref != n_points || cache.direct) {
        // Without usable candidates this call is a direct search, whose rows are the answer. Its row count says
        // how many candidates there would be: few enough, and they are computed now for the next calls to filter
        // (unless the candidates of this list keep getting outdated: see CandidateLifetime).
        VesinOptions plain = options;
        plain.skin = 0.0;
        direct_neighbors(points, n_points, box, periodic, plain, neighbors, extras, stream);
        cache.direct = too_long_for_a_filter(neighbors.length);
        cache.direct_n_points = n_points;
        if (cache.direct) {
            drop_candidates(); // the candidates of a smaller past are of no use any more
        } else if (force_cache || !cache.lifetime.resting()) {
            rebuild();
        }
        return;
    }

    size_t total = 0;
    for (int attempt = 0;; attempt++) {
        if (attempt > 4) {
            throw std::runtime_error("internal error: the Verlet filter did not settle");
        }
        const size_t n_candidates = cache.candidates.length;
        size_outputs(neighbors, extras, 0, options);
        SearchOutputs out;
        out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
        out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
        out.distances = neighbors.distances;
        out.vectors = reinterpret_cast<double*>(neighbors.vectors);
        const size_t capacity = extras.capacity;

        cache.status->rebuild = 0;
        cache.status->total_rows = 0;
        const size_t check_blocks = std::max<size_t>((n_points + VERLET_BLOCK - 1) / VERLET_BLOCK, 1);
        const size_t chunks = (n_candidates + VERLET_CHUNK - 1) / VERLET_CHUNK;
        const size_t count_blocks = std::min<size_t>((chunks + VERLET_WAVES - 1) / VERLET_WAVES, 256 * 64);
        const bool self_scan = chunks <= VERLET_SELF_SCAN_CHUNKS;

        VerletFilterArgs fargs;
        fargs.candidate_pairs = reinterpret_cast<const unsigned long long*>(cache.candidates.pairs);
        fargs.candidate_shifts = reinterpret_cast<const int32_t*>(cache.candidates.shifts);
        fargs.n_candidates = n_candidates;
        fargs.n_chunks = chunks;
        fargs.points = reinterpret_cast<const double*>(points);
        fargs.box = reinterpret_cast<const double*>(box);
        fargs.periodic = periodic;
        fargs.cutoff_sq = options.cutoff * options.cutoff;
        fargs.out = out;
        fargs.capacity = capacity;
        fargs.status = cache.status;
        uint64_t* scan_scratch = nullptr;
        auto carve = [&](Carver& c) {
            fargs.chunk_rows = c.take<uint32_t>(chunks);
            fargs.chunk_base = c.take<uint64_t>(self_scan ? 0 : chunks + 1);
            scan_scratch = c.take<uint64_t>(self_scan ? 0 : scan_scratch_elements(chunks));
        };
        Carver measure(nullptr);
        carve(measure);
        extras.sort_work.reserve(measure.used);
        Carver carver(extras.sort_work.ptr);
        carve(carver);

        // check and count, (scan,) write: the rows keep the order of the candidates
        hipLaunchKernelGGL(
            verlet_check_and_count_kernel, dim3(static_cast<unsigned>(std::max(check_blocks, count_blocks))),
            dim3(VERLET_BLOCK), 0, stream, cache.ref_points, n_points, cache.reference, options.skin, fargs
        );
        if (n_candidates > 0) {
            if (self_scan) {
                hipLaunchKernelGGL(verlet_write_kernel<true>, dim3(static_cast<unsigned>(count_blocks)), dim3(VERLET_BLOCK), 0, stream, fargs);
            } else {
                exclusive_scan<SCAN_U32>(fargs.chunk_rows, chunks, fargs.chunk_base, scan_scratch, stream);
                hipLaunchKernelGGL(verlet_write_kernel<false>, dim3(static_cast<unsigned>(count_blocks)), dim3(VERLET_BLOCK), 0, stream, fargs);
            }
        }
        // (a queued call stops here: what was launched above is all that a list in its steady state needs)
        QueuedOutcome outcome = {};
        outcome.kind = 3;
        outcome.filtered = cache.status;
        outcome.capacity = capacity;
        outcome.row_limit = pair_limit != 0 ? n_points * pair_limit : 0;
        const bool published_here = extras.publish_length(outcome, reinterpret_cast<const double*>(box), periodic, stream);
        extras.wait(stream);
        HIP_CHECK(hipGetLastError());

        if (cache.status->rebuild != 0) {
            if (fresh) {
                throw std::runtime_error("internal error: fresh Verlet candidates do not cover their own points");
            }
            if (!force_cache && cache.lifetime.outdated()) {
                // the third set of candidates in a row that did not last: the direct search for a while
                drop_candidates();
                VesinOptions plain = options;
                plain.skin = 0.0;
                direct_neighbors(points, n_points, box, periodic, plain, neighbors, extras, stream);
                return;
            }
            rebuild();
            continue;
        }
        total = cache.status->total_rows;
        if (pair_limit != 0 && total > n_points * pair_limit) {
            throw std::runtime_error(
                "The number of neighbor pairs exceeds the maximum capacity of " + std::to_string(n_points * pair_limit) +
                " (max_pairs_per_point=" + std::to_string(pair_limit) + "; n_points=" + std::to_string(n_points) + "). " +
                "Consider reducing the cutoff distance, or explicitly setting " +
                "VESIN_CUDA_MAX_PAIRS_PER_POINT as an environment variable."
            );
        }
        if (total > extras.capacity) {
            size_outputs(neighbors, extras, total, options);
            continue;
        }
        extras.queued_part_sufficed = published_here;
        break;
    }
    neighbors.length = total;
    cache.lifetime.served();
    if (too_long_for_a_filter(total)) {
        cache.direct = true;
        cache.direct_n_points = n_points;
    }
}

/// first_pair[s] = first output row of system s (offsets are kept per tile-major work item), first_pair[n] = total;
/// for the device and, in `landing`, for the host.
__global__ void system_rows_kernel(
    const uint64_t* __restrict__ cell_scan, const uint32_t* __restrict__ cell_base, const uint64_t* __restrict__ offsets,
    uint32_t n_systems, uint32_t n_slices, uint32_t n_slots, const FusedStatus* __restrict__ single_pass,
    unsigned long long* __restrict__ first_pair, unsigned long long* __restrict__ landing
) {
    const uint32_t s = blockIdx.x * BLOCK + threadIdx.x;
    if (s > n_systems) {
        return;
    }
    unsigned long long first = 0;
    if (s == n_systems) {
        // after the single-pass search `offsets` holds the first row of every work item, the total is in its status
        first = single_pass != nullptr ? single_pass->total_rows : offsets[n_slots];
    } else {
        const uint32_t first_tile = static_cast<uint32_t>(cell_scan[cell_base[s]] >> 32);
        first = offsets[static_cast<size_t>(first_tile) * n_slices];
    }
    first_pair[s] = first;
    landing[s] = first; // (pinned host memory: what the host reads after the call's synchronisation)
}

template <bool WRITE>
void launch_search_batch(bool full, const SearchArgs& args, hipStream_t stream) {
    if (args.n_work == 0) {
        return;
    }
    constexpr int R = 2;
    const uint32_t blocks = (args.n_work + SEARCH_WAVES - 1) / SEARCH_WAVES;
    if (full) {
        hipLaunchKernelGGL((search_kernel_batch<WRITE, true, R>), dim3(blocks), dim3(SEARCH_BLOCK), 0, stream, args);
    } else {
        hipLaunchKernelGGL((search_kernel_batch<WRITE, false, R>), dim3(blocks), dim3(SEARCH_BLOCK), 0, stream, args);
    }
}

bool batch_attempt(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair,
    HipExtras& extras, bool speculate, hipStream_t stream
);

void direct_batch(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair,
    HipExtras& extras, hipStream_t stream
);

void verlet_batch(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair,
    HipExtras& extras, hipStream_t stream
);

bool molecules_batch(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const bool (*periodic)[3], size_t most_points,
    VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair, HipExtras& extras, hipStream_t stream
);

} // namespace

namespace {

/// What every batched entry point checks before anything is queued.
void check_batch_inputs(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], int device_id
) {
    int device_count = 0;
    if (hipGetDeviceCount(&device_count) != hipSuccess || device_count == 0) {
        (void)hipGetLastError();
        throw std::runtime_error("no HIP device is available to this process");
    }
    if (device_id < 0 || device_id >= device_count) {
        throw std::runtime_error("invalid GPU device_id " + std::to_string(device_id));
    }
    if (n_systems == 0) {
        throw std::runtime_error("a batch needs at least one system");
    }
    for (size_t s = 0; s < n_systems; s++) {
        if (first_point[s + 1] < first_point[s]) {
            throw std::runtime_error("`first_point` must not decrease");
        }
    }
    if (first_point[0] != 0) {
        throw std::runtime_error("`first_point` must start at 0");
    }
    const size_t n_points = first_point[n_systems];
    if (n_points >= 0xFFFFFFF0ull || n_systems >= 0x7FFFFFF0ull) {
        throw std::runtime_error("too many points or systems: the GPU path indexes them with 32 bits");
    }
    if (device_of(points) != device_id && n_points > 0) {
        throw std::runtime_error("`points` pointer is not allocated on the GPU of the neighbor list");
    }
    if (device_of(boxes) != device_id) {
        throw std::runtime_error("`boxes` pointer is not allocated on the GPU of the neighbor list");
    }
    if (device_of(periodic) != device_id) {
        throw std::runtime_error("`periodic` pointer is not allocated on the GPU of the neighbor list");
    }
}

/// A batch on a list that has its state and whose inputs were checked, with the list's device current.
void run_batch(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair,
    HipExtras& extras, hipStream_t stream
) {
    extras.timings_valid = false;
    extras.batch_first_pair_device = nullptr; // (until the kernels of this call have a place for the systems' first rows)
    if (options.skin > 0.0) {
        verlet_batch(points, first_point, n_systems, boxes, periodic, options, neighbors, first_pair, extras, stream);
        return;
    }
    if (extras.verlet_batch != nullptr) {
        // no skin any more: the cache goes, as for single systems
        delete extras.verlet_batch;
        extras.verlet_batch = nullptr;
    }
    direct_batch(points, first_point, n_systems, boxes, periodic, options, neighbors, first_pair, extras, stream);
}

} // namespace

void neighbors_batch(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    size_t* first_pair,
    void* caller_stream
) {
    const int device_id = neighbors.device.device_id;
    check_batch_inputs(points, first_point, n_systems, boxes, periodic, device_id);
    const DeviceGuard guard(device_id);
    HipExtras& extras = extras_of(neighbors);
    refuse_while_queued(extras);
    restore_outputs(neighbors, extras, options);
    run_batch(
        points, first_point, n_systems, boxes, periodic, options, neighbors, first_pair, extras,
        static_cast<hipStream_t>(caller_stream)
    );
}

const unsigned long long* neighbors_batch_enqueue(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    size_t* first_pair,
    void* caller_stream
) {
    hipStream_t stream = static_cast<hipStream_t>(caller_stream);
    const int device_id = neighbors.device.device_id;
    check_batch_inputs(points, first_point, n_systems, boxes, periodic, device_id);
    const DeviceGuard guard(device_id);
    HipExtras& extras = extras_of(neighbors);
    refuse_while_queued(extras);
    restore_outputs(neighbors, extras, options);
    begin_queued(extras, stream);
    VesinNeighborList* list = &neighbors;
    HipExtras* state = &extras;
    extras.queued->start([=]() {
        run_batch(points, first_point, n_systems, boxes, periodic, options, *list, first_pair, *state, stream);
    });
    if (extras.queued->finished) {
        // an error before the first wait
        finish_queued(neighbors, extras, stream);
    }
    return extras.d_queued_length;
}

namespace {

/// A batch without a skin, on a list that has its state and whose inputs were checked, with the list's device current.
void direct_batch(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair,
    HipExtras& extras, hipStream_t stream
) {
    const size_t n_points = first_point[n_systems];
    extras.guess.have_box = false; // the work buffers of the single-system path are about to be reused

    // Free molecules of at most 64 points each (256 for a sorted list): no cell lists, see molecules.cuh. That no
    // system has a periodic direction is for the kernels to confirm, since the flags live on the device: the batch is
    // tried as one of free molecules on a list that has not seen a batch yet or whose last batch through the general
    // path had no periodic direction anywhere (a loader that hands over other molecules with every call stays on these
    // kernels; a list used for crystals pays for the wrong guess once at most). With larger systems in the batch the
    // kernels for molecules write an unsorted list no faster than the general path (2,000 molecules of 100 to 256
    // atoms 0.69 against 0.59 ms per call, 20,000 of 3 to 80 atoms 0.89 against 0.85 ms), and a sorted one in half the
    // time (0.69 against 1.26 ms, 0.89 against 1.37 ms).
    {
        const BatchSetup& known = extras.batch;
        size_t most_points = 0;
        for (size_t s = 0; s < n_systems; s++) {
            most_points = std::max(most_points, first_point[s + 1] - first_point[s]);
        }
        const bool free_molecules =
            (!known.valid || known.all_open) && n_points > 0 &&
            most_points <= (options.sorted ? MOLECULE_MAX_POINTS : MOLECULE_GROUP_POINTS) &&
            options.algorithm != VesinCellList && !extras.fixed_memory && std::getenv("VESIN_HIP_MOLECULES") == nullptr;
        if (free_molecules &&
            molecules_batch(points, first_point, n_systems, periodic, most_points, options, neighbors, first_pair, extras, stream)) {
            return;
        }
    }

    // The grids follow from the boxes, the flags, the division into systems, the cutoff and the algorithm alone,
    // unless some direction is open: then they also follow the points. Same inputs as the call before: same grids.
    // Whether the boxes and flags are the same is for the device to say, where they live: a call whose other inputs
    // are those of the call before starts from the grids it has, a kernel compares the boxes on the way, and the
    // host looks at its answer at the call's last synchronisation (the bookkeeping of the single-system path:
    // BoxGuess). Otherwise, and after a wrong guess, the boxes come to the host first.
    BatchSetup& setup = extras.batch;
    const BoxKey key = {n_points, options.cutoff, static_cast<int>(options.algorithm), options.full, options.sorted};
    const bool may_guess = setup.guess.begin(key);
    // (systems without any periodic direction: the grids follow the points and are picked on the device, see
    // batch_attempt; only the flags have to be the same)
    const bool rest_is_the_same =
        setup.valid && setup.kept_on_device && (!setup.any_open_direction || setup.all_open) &&
        setup.cutoff == options.cutoff && setup.algorithm == static_cast<int>(options.algorithm) &&
        setup.full_stencil == full_stencil_only() && setup.first_point.size() == n_systems + 1 &&
        std::memcmp(setup.first_point.data(), first_point, (n_systems + 1) * sizeof(size_t)) == 0 &&
        setup.boxes.size() == 9 * n_systems && extras.mail == extras.mail_device;
    if (may_guess && rest_is_the_same) {
        bool right = false;
        std::exception_ptr failure;
        try {
            right = batch_attempt(points, first_point, n_systems, boxes, periodic, options, neighbors, first_pair, extras, true, stream);
        } catch (...) {
            // the error may be a consequence of boxes that changed
            failure = std::current_exception();
            HIP_CHECK(hipStreamSynchronize(stream)); // (not extras.sync: a queued call does not stop inside a handler)
            right = extras.mail->batch_changed == 0;
            if (right) {
                std::rethrow_exception(failure);
            }
        }
        if (right) {
            setup.guess.was_right();
            return;
        }
        setup.guess.was_wrong();
        if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
            std::fprintf(stderr, "batch: the boxes are not those of the call before, the call starts over\n");
        }
    }
    (void)batch_attempt(points, first_point, n_systems, boxes, periodic, options, neighbors, first_pair, extras, false, stream);
    setup.guess.have_box = setup.kept_on_device;
    setup.guess.stored(key);
}

/// A batch of free molecules (`most_points` at most per system) through molecules_kernel: counting pass, scan over
/// the systems, writing pass, one synchronisation. Returns false, with nothing of the result to be used, when some
/// system turned out to have a periodic direction (the flags live on the device).
bool molecules_batch(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const bool (*periodic)[3], size_t most_points,
    VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair, HipExtras& extras, hipStream_t stream
) {
    const TraceRange whole_call("vesin_hip_neighbors_batch (free molecules)");
    BatchSetup& setup = extras.batch;
    const size_t n_points = first_point[n_systems];
    const size_t pair_limit = pairs_per_point_limit();
    if (setup.molecule_report == nullptr) {
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&setup.molecule_report), sizeof(MoleculeStatus), hipHostMallocDefault));
    }
    if (setup.first_pair_capacity < n_systems + 1) {
        if (setup.first_pair_landing != nullptr) {
            (void)hipHostFree(setup.first_pair_landing);
            setup.first_pair_landing = nullptr;
            setup.first_pair_capacity = 0;
        }
        const size_t wanted = (n_systems + 1) + (n_systems + 1) / 4;
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&setup.first_pair_landing), wanted * sizeof(size_t), hipHostMallocDefault));
        setup.first_pair_capacity = wanted;
    }

    MoleculeArgs args = {};
    uint32_t* d_first_point = nullptr;
    uint64_t* d_first_pair = nullptr;
    uint64_t* scan_scratch = nullptr;
    // lanes per system: the next power of two from the largest system on, eight at least; a workgroup beyond 64
    const int lanes = most_points <= 8 ? 8 : most_points <= 16 ? 16 : most_points <= 32 ? 32
                    : most_points <= MOLECULE_GROUP_POINTS ? 64 : MOLECULE_BLOCK;
    const bool wide = lanes == MOLECULE_BLOCK;
    uint64_t* d_first_row = nullptr;
    auto carve = [&](Carver& c) {
        d_first_point = c.take<uint32_t>(n_systems + 1);
        args.status = c.take<MoleculeStatus>(1);
        args.rows_of_system = c.take<uint32_t>(wide ? 0 : n_systems);
        args.rows_of_point = c.take<uint32_t>(wide ? n_points : 0);
        d_first_row = c.take<uint64_t>(wide ? n_points + 1 : 0);
        d_first_pair = c.take<uint64_t>(n_systems + 1);
        scan_scratch = c.take<uint64_t>(scan_scratch_elements(wide ? n_points : n_systems));
    };
    Carver measure(nullptr);
    carve(measure);
    const uint64_t generation = setup.molecule_work.generation;
    setup.molecule_work.reserve(measure.used);
    Carver carver(setup.molecule_work.ptr);
    carve(carver);
    // the division into systems goes to the device when it is not the one of the call before
    const bool same_division = setup.molecule_first_point_on_device && generation == setup.molecule_work.generation &&
                               setup.molecule_first_point.size() == n_systems + 1 &&
                               std::memcmp(setup.molecule_first_point.data(), first_point, (n_systems + 1) * sizeof(size_t)) == 0;
    if (!same_division) {
        setup.molecule_first_point_on_device = false;
        setup.molecule_first_point.assign(first_point, first_point + n_systems + 1);
        setup.molecule_first_point32.resize(n_systems + 1);
        for (size_t s = 0; s <= n_systems; s++) {
            setup.molecule_first_point32[s] = static_cast<uint32_t>(first_point[s]);
        }
        HIP_CHECK(hipMemcpyAsync(
            d_first_point, setup.molecule_first_point32.data(), (n_systems + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, stream
        ));
        setup.molecule_first_point_on_device = true;
    }

    args.points = reinterpret_cast<const double*>(points);
    args.periodic = reinterpret_cast<const bool*>(periodic);
    args.first_point = d_first_point;
    args.n_systems = static_cast<uint32_t>(n_systems);
    args.cutoff2 = options.cutoff * options.cutoff;
    args.full = options.full ? 1 : 0;
    args.first_pair = d_first_pair;
    args.report = setup.molecule_report;

    args.total_points = static_cast<uint32_t>(n_points);
    args.first_row = d_first_row;
    const size_t per_block = wide ? 1 : static_cast<size_t>(MOLECULE_BLOCK / WAVE) * (WAVE / lanes);
    const unsigned blocks = static_cast<unsigned>((n_systems + per_block - 1) / per_block);
    auto launch = [&](bool write) {
        const dim3 grid(blocks), block(MOLECULE_BLOCK);
        switch (lanes * 2 + (write ? 1 : 0)) {
        case 2 * MOLECULE_BLOCK: hipLaunchKernelGGL((molecules_wide_kernel<false>), grid, block, 0, stream, args); break;
        case 2 * MOLECULE_BLOCK + 1: hipLaunchKernelGGL((molecules_wide_kernel<true>), grid, block, 0, stream, args); break;
        case 16: hipLaunchKernelGGL((molecules_kernel<8, false>), grid, block, 0, stream, args); break;
        case 17: hipLaunchKernelGGL((molecules_kernel<8, true>), grid, block, 0, stream, args); break;
        case 32: hipLaunchKernelGGL((molecules_kernel<16, false>), grid, block, 0, stream, args); break;
        case 33: hipLaunchKernelGGL((molecules_kernel<16, true>), grid, block, 0, stream, args); break;
        case 64: hipLaunchKernelGGL((molecules_kernel<32, false>), grid, block, 0, stream, args); break;
        case 65: hipLaunchKernelGGL((molecules_kernel<32, true>), grid, block, 0, stream, args); break;
        case 128: hipLaunchKernelGGL((molecules_kernel<64, false>), grid, block, 0, stream, args); break;
        default: hipLaunchKernelGGL((molecules_kernel<64, true>), grid, block, 0, stream, args); break;
        }
    };

    MoleculeStatus cleared = {};
    cleared.first_bad = 0xFFFFFFFFu;
    *setup.molecule_report = cleared;
    HIP_CHECK(hipMemcpyAsync(args.status, setup.molecule_report, sizeof(MoleculeStatus), hipMemcpyHostToDevice, stream));
    launch(false);
    if (wide) {
        exclusive_scan<SCAN_U32>(args.rows_of_point, n_points, d_first_row, scan_scratch, stream);
        const uint32_t system_blocks = static_cast<uint32_t>((n_systems + 1 + BLOCK - 1) / BLOCK);
        hipLaunchKernelGGL(
            first_rows_of_systems_kernel, dim3(system_blocks), dim3(BLOCK), 0, stream, d_first_row, d_first_point,
            static_cast<uint32_t>(n_systems), reinterpret_cast<unsigned long long*>(d_first_pair)
        );
    } else {
        exclusive_scan<SCAN_U32>(args.rows_of_system, n_systems, d_first_pair, scan_scratch, stream);
    }
    size_t total = 0;
    extras.batch_first_pair_device = reinterpret_cast<const unsigned long long*>(d_first_pair);
    bool published_here = false;
    for (int attempt = 0;; attempt++) {
        if (attempt > 2) {
            throw std::runtime_error("internal error: the rows of a batch of molecules did not settle");
        }
        // (a list without arrays gets them once the kernels have confirmed that these are free molecules: until then
        // it stays as it was, for the general path to start from; the writing pass only reports)
        const bool has_arrays = extras.capacity > 0 || attempt > 0;
        if (has_arrays) {
            size_outputs(neighbors, extras, total, options);
        }
        args.out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
        args.out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
        args.out.distances = neighbors.distances;
        args.out.vectors = reinterpret_cast<double*>(neighbors.vectors);
        args.capacity = has_arrays ? extras.capacity : 0;
        launch(true);
        if (attempt == 0) {
            HIP_CHECK(hipMemcpyAsync(
                setup.first_pair_landing, d_first_pair, (n_systems + 1) * sizeof(size_t), hipMemcpyDeviceToHost, stream
            ));
            if (has_arrays && extras.before_the_stop_of_a_queued_call()) {
                hipLaunchKernelGGL(
                    publish_queued_molecules_length, dim3(1), dim3(1), 0, stream, args.status,
                    reinterpret_cast<const unsigned long long*>(d_first_pair + n_systems),
                    static_cast<unsigned long long>(args.capacity),
                    static_cast<unsigned long long>(pair_limit != 0 ? n_points * pair_limit : 0), extras.d_queued_length
                );
                extras.length_published = true;
                published_here = true;
            }
        }
        extras.sync(stream);
        HIP_CHECK(hipGetLastError());
        const MoleculeStatus found = *setup.molecule_report;
        if (found.periodic != 0) {
            if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
                std::fprintf(stderr, "batch: free molecules no more, some system has a periodic direction now\n");
            }
            return false;
        }
        if (found.first_bad != 0xFFFFFFFFu) {
            non_finite_error(points, found.first_bad);
        }
        total = found.total_rows;
        if (pair_limit != 0 && total > n_points * pair_limit) {
            throw std::runtime_error(
                "The number of neighbor pairs exceeds the maximum capacity of " + std::to_string(n_points * pair_limit) +
                " (max_pairs_per_point=" + std::to_string(pair_limit) + "; n_points=" + std::to_string(n_points) + "). " +
                "Consider reducing the cutoff distance, or explicitly setting " +
                "VESIN_CUDA_MAX_PAIRS_PER_POINT as an environment variable."
            );
        }
        if (total <= args.capacity) {
            extras.queued_part_sufficed = published_here && attempt == 0;
            break;
        }
    }
    if (extras.capacity == 0) {
        size_outputs(neighbors, extras, 0, options); // (no rows at all: the arrays exist all the same)
    }
    neighbors.length = total;
    std::memcpy(first_pair, setup.first_pair_landing, (n_systems + 1) * sizeof(size_t));
    if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
        std::fprintf(stderr, "batch of free molecules: %zu rows, %d lanes per system\n", total, lanes);
    }
    return true;
}

/// Candidates beyond which a batch is searched directly on every call (see VERLET_MAX_CANDIDATES): the filter of a
/// batch reads 16 bytes per candidate and two points on top of writing the rows, in two passes, and takes 0.05 ms
/// and 33 ns per thousand candidates (i j S d asked for, a fourth of the candidates beyond the cutoff). The direct
/// search costs more per call and less per row. Measured, direct against filter, full lists with skin 0.5:
/// 2,000 free molecules of 3 to 40 atoms (1.0 M rows) 0.142 / 0.095 ms; 100,000 of 3 to 8 atoms (2.8 M rows) 0.734 /
/// 0.234 ms; 512 periodic cells of 64 atoms (3.6 M rows) 0.201 / 0.193 ms; 20,000 molecules of 3 to 40 atoms (10.2 M
/// rows) 0.445 / 0.460 ms; 4,096 cells of 64 atoms (29 M rows) 0.807 / 1.215 ms. Sorted lists of systems of several
/// cells are the exception: the search that writes them in order takes 0.799 ms for 1,000 cells of 200 atoms (9.5 M
/// rows) and 2.70 ms for 4,000 of them, the filter of sorted candidates 0.457 and 1.65 ms.
constexpr size_t BATCH_VERLET_MAX_CANDIDATES = size_t(1) << 22;
constexpr size_t BATCH_VERLET_MAX_CANDIDATES_SORTED_CELLS = size_t(1) << 26;
constexpr int BATCH_VERLET_UNPACKABLE_REST = 16;

/// options.skin > 0 for a batch: verlet_neighbors with one candidate list for all systems. The candidates are
/// computed again as a whole when any system's points or box moved too far, when the division into systems or the
/// options changed; otherwise a call is the two box and point checks, the two passes of the filter with a scan
/// between them, and one synchronisation.
void verlet_batch(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair,
    HipExtras& extras, hipStream_t stream
) {
    const TraceRange whole_call("vesin_hip_neighbors_batch (skin)");
    if (extras.verlet_batch == nullptr) {
        auto cache = std::make_unique<BatchVerletCache>();
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&cache->status), sizeof(VerletStatus), hipHostMallocDefault));
        extras.verlet_batch = cache.release();
    }
    BatchVerletCache& cache = *extras.verlet_batch;
    const size_t n_points = first_point[n_systems];
    const size_t pair_limit = pairs_per_point_limit();

    const bool options_changed = cache.options.cutoff != options.cutoff || cache.options.skin != options.skin ||
                                 cache.options.full != options.full || cache.options.sorted != options.sorted;
    const bool same_division = cache.first_point.size() == n_systems + 1 &&
                               std::memcmp(cache.first_point.data(), first_point, (n_systems + 1) * sizeof(size_t)) == 0;
    bool fresh = false;
    auto rebuild = [&]() {
        cache.valid = false;
        VesinOptions build = {};
        build.cutoff = options.cutoff + options.skin;
        build.full = options.full;
        build.sorted = options.sorted; // the filter keeps the order of the candidates
        build.algorithm = VesinAutoAlgorithm;
        build.n_threads = options.n_threads;
        build.return_shifts = true;
        build.return_distances = false;
        build.return_vectors = false;
        build.skin = 0.0;
        cache.candidates.device = neighbors.device;
        cache.candidate_first_pair.resize(n_systems + 1);
        vesin_hip::neighbors_batch(
            points, first_point, n_systems, boxes, periodic, build, cache.candidates, cache.candidate_first_pair.data(), stream
        );
        cache.first_point.assign(first_point, first_point + n_systems + 1);
        const size_t n_candidates = cache.candidates.length;

        unsigned long long* d_candidate_first = nullptr;
        auto carve = [&](Carver& c) {
            cache.ref_points = c.take<double>(3 * n_points);
            cache.reference = c.take<BatchVerletReference>(n_systems);
            cache.system_of_point = c.take<uint32_t>(n_points);
            cache.packed = c.take<BatchVerletCandidate>(n_candidates);
            cache.d_first_point = c.take<unsigned long long>(n_systems + 1);
            d_candidate_first = c.take<unsigned long long>(n_systems + 1);
        };
        Carver measure(nullptr);
        carve(measure);
        cache.kept.reserve(measure.used);
        Carver carver(cache.kept.ptr);
        carve(carver);

        static_assert(sizeof(size_t) == sizeof(unsigned long long), "size_t is 64 bits wide here");
        if (n_points > 0) {
            HIP_CHECK(hipMemcpyAsync(cache.ref_points, points, n_points * 3 * sizeof(double), hipMemcpyDeviceToDevice, stream));
        }
        HIP_CHECK(hipMemcpyAsync(
            cache.d_first_point, cache.first_point.data(), (n_systems + 1) * sizeof(size_t), hipMemcpyHostToDevice, stream
        ));
        HIP_CHECK(hipMemcpyAsync(
            d_candidate_first, cache.candidate_first_pair.data(), (n_systems + 1) * sizeof(size_t), hipMemcpyHostToDevice, stream
        ));
        const uint32_t system_blocks = static_cast<uint32_t>((n_systems + VERLET_BLOCK - 1) / VERLET_BLOCK);
        hipLaunchKernelGGL(
            verlet_batch_store_reference, dim3(system_blocks), dim3(VERLET_BLOCK), 0, stream,
            reinterpret_cast<const double*>(boxes), reinterpret_cast<const bool*>(periodic), static_cast<uint32_t>(n_systems),
            cache.reference
        );
        if (n_points > 0) {
            const uint32_t blocks = static_cast<uint32_t>(std::min<size_t>(4096, (n_points + VERLET_BLOCK - 1) / VERLET_BLOCK));
            hipLaunchKernelGGL(
                verlet_batch_owner_kernel, dim3(blocks), dim3(VERLET_BLOCK), 0, stream, cache.d_first_point,
                static_cast<uint32_t>(n_systems), n_points, cache.system_of_point
            );
        }
        cache.status->unusable = 0; // (pinned; raised by a shift that the candidates of the filter cannot hold)
        if (n_candidates > 0) {
            const uint32_t blocks = static_cast<uint32_t>(std::min<size_t>(4096, (n_candidates + VERLET_BLOCK - 1) / VERLET_BLOCK));
            hipLaunchKernelGGL(
                verlet_batch_pack_kernel, dim3(blocks), dim3(VERLET_BLOCK), 0, stream,
                reinterpret_cast<const unsigned long long*>(cache.candidates.pairs),
                reinterpret_cast<const int32_t*>(cache.candidates.shifts), n_candidates, d_candidate_first,
                cache.d_first_point, static_cast<uint32_t>(n_systems), cache.packed, cache.reference,
                &cache.status->unusable
            );
        }
        // the snapshot is complete before the call returns: the caller may change points and boxes right after
        HIP_CHECK(hipGetLastError());
        extras.sync(stream);
        // (the rows the candidates were packed from stay where they are, although nothing reads them again: with
        // arrays to allocate anew, a call that computes the candidates again took a third longer, 0.40 against 0.30 ms
        // for 2,000 molecules and 1.58 against 1.16 ms for 100,000)
        cache.options = options;
        cache.valid = cache.status->unusable == 0;
        fresh = true;
    };
    const char* forced = std::getenv("VESIN_HIP_VERLET");
    const bool force_cache = forced != nullptr && std::strcmp(forced, "cache") == 0;
    const bool force_direct = forced != nullptr && std::strcmp(forced, "direct") == 0;
    auto too_long_for_a_filter = [&](size_t rows) {
        const double ratio = (options.cutoff + options.skin) / options.cutoff;
        const double candidates = static_cast<double>(rows) * ratio * ratio * ratio;
        // (what the last direct search of this list found out about its systems: sorted, and some of them have
        // several cells)
        const BatchSetup& setup = extras.batch;
        const bool sorted_cells = options.sorted && setup.valid && !setup.all_open &&
                                  setup.systems_for_images < setup.systems_with_points;
        const size_t limit = sorted_cells ? BATCH_VERLET_MAX_CANDIDATES_SORTED_CELLS : BATCH_VERLET_MAX_CANDIDATES;
        return force_direct || (!force_cache && candidates > static_cast<double>(limit));
    };
    if (options_changed || cache.direct_n_points != n_points) {
        cache.direct = false;
        cache.lifetime.reset();
    }
    if (!cache.valid || options_changed || !same_division || cache.direct) {
        // (as in verlet_neighbors: this call is a direct search, and its row count says whether candidates pay)
        VesinOptions plain = options;
        plain.skin = 0.0;
        direct_batch(points, first_point, n_systems, boxes, periodic, plain, neighbors, first_pair, extras, stream);
        cache.direct = too_long_for_a_filter(neighbors.length);
        cache.direct_n_points = n_points;
        if (cache.unpackable_rest > 0) {
            cache.unpackable_rest -= 1;
            cache.direct = true;
        }
        if (!cache.direct && !force_cache && cache.lifetime.resting()) {
            // (candidates that keep getting outdated after a few calls: see CandidateLifetime)
            cache.drop_candidates();
            cache.first_point.clear();
            return;
        }
        if (!cache.direct) {
            rebuild();
            if (!cache.valid) {
                // shifts of a million boxes: such a batch is searched directly for a while
                cache.direct = true;
                cache.unpackable_rest = BATCH_VERLET_UNPACKABLE_REST;
            }
        }
        if (cache.direct) {
            cache.drop_candidates();
            cache.first_point.clear();
        }
        return;
    }

    cache.first_pair_landing.resize(n_systems + 1);
    size_t total = 0;
    size_t n_candidates = 0;
    for (int attempt = 0;; attempt++) {
        if (attempt > 4) {
            throw std::runtime_error("internal error: the Verlet filter of a batch did not settle");
        }
        n_candidates = cache.candidates.length;
        const size_t n_chunks = (n_candidates + VERLET_CHUNK - 1) / VERLET_CHUNK;
        size_outputs(neighbors, extras, 0, options);

        BatchVerletLimits* limits = nullptr;
        uint32_t* chunk_rows = nullptr;
        uint64_t* chunk_base = nullptr;
        uint64_t* scan_scratch = nullptr;
        unsigned long long* d_first_pair = nullptr;
        auto carve = [&](Carver& c) {
            limits = c.take<BatchVerletLimits>(n_systems);
            chunk_rows = c.take<uint32_t>(n_chunks);
            chunk_base = c.take<uint64_t>(n_chunks + 1);
            scan_scratch = c.take<uint64_t>(scan_scratch_elements(n_chunks));
            d_first_pair = c.take<unsigned long long>(n_systems + 1);
        };
        Carver measure(nullptr);
        carve(measure);
        cache.scratch.reserve(measure.used);
        Carver carver(cache.scratch.ptr);
        carve(carver);

        cache.status->rebuild = 0;
        cache.status->total_rows = 0;
        const uint32_t system_blocks = static_cast<uint32_t>((n_systems + VERLET_BLOCK - 1) / VERLET_BLOCK);
        hipLaunchKernelGGL(
            verlet_batch_limits_kernel, dim3(system_blocks), dim3(VERLET_BLOCK), 0, stream,
            reinterpret_cast<const double*>(boxes), reinterpret_cast<const bool*>(periodic), cache.reference,
            cache.d_first_point, static_cast<uint32_t>(n_systems), options.skin, limits, cache.status
        );
        if (n_points > 0) {
            const uint32_t blocks = static_cast<uint32_t>((n_points + VERLET_BLOCK - 1) / VERLET_BLOCK);
            hipLaunchKernelGGL(
                verlet_batch_moved_kernel, dim3(blocks), dim3(VERLET_BLOCK), 0, stream,
                reinterpret_cast<const double*>(points), cache.ref_points, n_points, cache.system_of_point, limits,
                cache.status
            );
        }
        if (n_candidates > 0) {
            BatchVerletFilterArgs fargs;
            fargs.candidates = cache.packed;
            fargs.system_of_point = cache.system_of_point;
            fargs.n_candidates = n_candidates;
            fargs.n_chunks = n_chunks;
            fargs.points = reinterpret_cast<const double*>(points);
            fargs.limits = limits;
            fargs.cutoff_sq = options.cutoff * options.cutoff;
            fargs.chunk_rows = chunk_rows;
            fargs.chunk_base = chunk_base;
            fargs.out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
            fargs.out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
            fargs.out.distances = neighbors.distances;
            fargs.out.vectors = reinterpret_cast<double*>(neighbors.vectors);
            fargs.capacity = extras.capacity;
            fargs.first_pair = d_first_pair;
            extras.batch_first_pair_device = d_first_pair;
            fargs.n_systems = static_cast<uint32_t>(n_systems);
            fargs.status = cache.status;
            const size_t wanted = (n_chunks + VERLET_WAVES - 1) / VERLET_WAVES;
            const unsigned blocks = static_cast<unsigned>(std::min<size_t>(wanted, 256 * 64));
            hipLaunchKernelGGL(verlet_batch_filter_kernel<false>, dim3(blocks), dim3(VERLET_BLOCK), 0, stream, fargs);
            exclusive_scan<SCAN_U32>(chunk_rows, n_chunks, chunk_base, scan_scratch, stream);
            hipLaunchKernelGGL(verlet_batch_filter_kernel<true>, dim3(blocks), dim3(VERLET_BLOCK), 0, stream, fargs);
            HIP_CHECK(hipMemcpyAsync(
                cache.first_pair_landing.data(), d_first_pair, (n_systems + 1) * sizeof(size_t), hipMemcpyDeviceToHost, stream
            ));
        }
        extras.sync(stream);
        HIP_CHECK(hipGetLastError());

        if (cache.status->rebuild != 0) {
            if (fresh) {
                throw std::runtime_error("internal error: fresh Verlet candidates of a batch do not cover their own points");
            }
            if (!force_cache && cache.lifetime.outdated()) {
                if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
                    std::fprintf(stderr, "batch with a skin: the candidates keep getting outdated, direct searches for a while\n");
                }
                cache.drop_candidates();
                cache.first_point.clear();
                VesinOptions plain = options;
                plain.skin = 0.0;
                direct_batch(points, first_point, n_systems, boxes, periodic, plain, neighbors, first_pair, extras, stream);
                return;
            }
            if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
                std::fprintf(stderr, "batch with a skin: some system moved too far, the candidates are computed again\n");
            }
            rebuild();
            if (!cache.valid) {
                cache.direct = true;
                cache.unpackable_rest = BATCH_VERLET_UNPACKABLE_REST;
                cache.direct_n_points = n_points;
                cache.drop_candidates();
                cache.first_point.clear();
                VesinOptions plain = options;
                plain.skin = 0.0;
                direct_batch(points, first_point, n_systems, boxes, periodic, plain, neighbors, first_pair, extras, stream);
                return;
            }
            continue;
        }
        total = n_candidates > 0 ? cache.status->total_rows : 0;
        if (pair_limit != 0 && total > n_points * pair_limit) {
            throw std::runtime_error(
                "The number of neighbor pairs exceeds the maximum capacity of " + std::to_string(n_points * pair_limit) +
                " (max_pairs_per_point=" + std::to_string(pair_limit) + "; n_points=" + std::to_string(n_points) + "). " +
                "Consider reducing the cutoff distance, or explicitly setting " +
                "VESIN_CUDA_MAX_PAIRS_PER_POINT as an environment variable."
            );
        }
        if (total > extras.capacity) {
            size_outputs(neighbors, extras, total, options);
            continue;
        }
        break;
    }
    neighbors.length = total;
    cache.lifetime.served();
    if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
        std::fprintf(stderr, "batch with a skin: %zu rows filtered from %zu candidates\n", total, n_candidates);
    }
    if (n_candidates > 0) {
        std::memcpy(first_pair, cache.first_pair_landing.data(), (n_systems + 1) * sizeof(size_t));
    } else {
        std::fill(first_pair, first_pair + n_systems + 1, size_t(0));
    }
    if (too_long_for_a_filter(total)) {
        cache.direct = true;
        cache.direct_n_points = n_points;
    }
}

} // namespace

namespace {

/// The batch itself. `speculate`: from the grids of the call before, with the boxes compared on the device; false is
/// returned when they turned out to be others (nothing of the result is to be used then).
bool batch_attempt(
    const double (*points)[3], const size_t* first_point, size_t n_systems, const double (*boxes)[3][3],
    const bool (*periodic)[3], VesinOptions options, VesinNeighborList& neighbors, size_t* first_pair,
    HipExtras& extras, bool speculate, hipStream_t stream
) {
    const TraceRange whole_call(speculate ? "vesin_hip_neighbors_batch (grids of the call before)" : "vesin_hip_neighbors_batch");
    const size_t n_points = first_point[n_systems];
    const size_t pair_limit = pairs_per_point_limit();
    BatchSetup& setup = extras.batch;

    bool same_setup = false;
    if (speculate) {
        const auto* kept = static_cast<const unsigned char*>(setup.kept_boxes.ptr);
        extras.mail->batch_changed = 0; // (pinned memory, written before the launch is queued)
        const uint32_t compare_blocks = static_cast<uint32_t>(std::min<size_t>(256, (9 * n_systems + BLOCK - 1) / BLOCK));
        hipLaunchKernelGGL(
            compare_boxes_kernel, dim3(compare_blocks), dim3(BLOCK), 0, stream,
            reinterpret_cast<const unsigned long long*>(boxes), reinterpret_cast<const unsigned char*>(periodic),
            reinterpret_cast<const unsigned long long*>(kept), kept + 72 * n_systems,
            setup.all_open ? size_t(0) : 9 * n_systems, 3 * n_systems, &extras.mail_device->batch_changed
        );
        same_setup = true;
    } else {
        // ---- every system's box comes to the host: the grids are picked there
        setup.incoming_boxes.resize(9 * n_systems);
        setup.incoming_periodic.resize(3 * n_systems);
        HIP_CHECK(hipMemcpyAsync(
            setup.incoming_boxes.data(), boxes, setup.incoming_boxes.size() * sizeof(double), hipMemcpyDeviceToHost, stream
        ));
        HIP_CHECK(hipMemcpyAsync(
            setup.incoming_periodic.data(), periodic, setup.incoming_periodic.size(), hipMemcpyDeviceToHost, stream
        ));
        extras.sync(stream);
        same_setup =
            setup.valid && !setup.any_open_direction && setup.cutoff == options.cutoff &&
            setup.algorithm == static_cast<int>(options.algorithm) && setup.full_stencil == full_stencil_only() &&
            setup.first_point.size() == n_systems + 1 &&
            std::memcmp(setup.first_point.data(), first_point, (n_systems + 1) * sizeof(size_t)) == 0 &&
            setup.boxes.size() == setup.incoming_boxes.size() &&
            std::memcmp(setup.boxes.data(), setup.incoming_boxes.data(), setup.boxes.size() * sizeof(double)) == 0 &&
            std::memcmp(setup.periodic.data(), setup.incoming_periodic.data(), setup.periodic.size()) == 0;
    }

    PinnedVector<GridParams>& grids = setup.grids;
    PinnedVector<uint32_t>& cell_base_host = setup.cell_base;
    PinnedVector<uint32_t>& first_point_host = setup.first_point32;
    if (!same_setup) {
        setup.valid = false;
        setup.on_device = false;
        setup.kept_on_device = false;
        setup.boxes.swap(setup.incoming_boxes);
        setup.periodic.swap(setup.incoming_periodic);
        setup.first_point.assign(first_point, first_point + n_systems + 1);
        setup.cutoff = options.cutoff;
        setup.algorithm = static_cast<int>(options.algorithm);
        setup.full_stencil = full_stencil_only();
        const PinnedVector<double>& host_boxes = setup.boxes;
        const PinnedVector<unsigned char>& host_periodic = setup.periodic;

        grids.resize(n_systems);
        std::vector<HostBox>& host_grids_box = setup.host_boxes;
        host_grids_box.resize(n_systems);
        cell_base_host.resize(n_systems + 1);
        first_point_host.resize(n_systems + 1);
        // what the flags and the sizes of the systems say, in one go over them
        bool any_open_direction = false;
        bool any_periodic_direction = false;
        uint64_t cells_bound = 0;
        for (size_t s = 0; s < n_systems; s++) {
            bool any_periodic_here = false;
            for (int d = 0; d < 3; d++) {
                const bool flag = host_periodic[3 * s + d] != 0;
                any_open_direction = any_open_direction || !flag;
                any_periodic_here = any_periodic_here || flag;
            }
            any_periodic_direction = any_periodic_direction || any_periodic_here;
            // (choose_grid and open_grids_kernel never make more cells than twice the points, or 64: limit_cells; one
            // cell under brute force, and for fewer than 32 points under the automatic choice)
            const uint64_t points_here = first_point[s + 1] - first_point[s];
            // (a system without periodic directions has no images: what open_grids_kernel is told below)
            const bool one_cell = options.algorithm == VesinBruteForce ||
                                  (options.algorithm == VesinAutoAlgorithm &&
                                   (points_here < 32 || (!any_periodic_here && one_cell_in_a_batch(points_here, 1))));
            cells_bound += one_cell ? 1 : std::min<uint64_t>(16777216, std::max<uint64_t>(64, 2 * points_here));
            first_point_host[s] = static_cast<uint32_t>(first_point[s]);
        }
        first_point_host[n_systems] = static_cast<uint32_t>(n_points);
        setup.any_open_direction = any_open_direction;
        setup.all_open = !any_periodic_direction;
        setup.cells_bound = cells_bound;

        // Per system: the box in the form the kernels use, then (with the extents of the points where a direction is
        // open, which take a round trip to the GPU in between) the grid. Both on several threads for many systems,
        // in one go when no extents are needed (starting the threads costs 0.1-0.3 ms each time).
        const size_t n_parts = parts_for_systems(n_systems);
        auto take_box = [&](size_t s) {
            bool flags[3];
            for (int d = 0; d < 3; d++) {
                flags[d] = host_periodic[3 * s + d] != 0;
            }
            const HostBox hbox = normalise_box(&host_boxes[9 * s], flags);
            host_grids_box[s] = hbox;
            GridParams& g = grids[s];
            std::memset(&g, 0, sizeof(g));
            for (int d = 0; d < 3; d++) {
                for (int e = 0; e < 3; e++) {
                    g.H[3 * d + e] = hbox.H[d][e];
                    g.Hinv[3 * d + e] = hbox.Hinv[d][e];
                }
                g.periodic[d] = flags[d] ? 1 : 0;
            }
        };
        const bool extents_needed = any_open_direction && n_points > 0;
        if (extents_needed) {
            over_the_systems(n_systems, n_parts, [&](size_t begin, size_t end, size_t) {
                for (size_t s = begin; s < end; s++) {
                    take_box(s);
                }
            });
        }

        // ---- systems with a non-periodic direction need the extent of their points along it (reference:
        // BoundingBox::make_bounding_for, vesin/src/types.hpp:159-200): one wave per system finds it
        PinnedVector<BlockBounds>& bounds = setup.bounds;
        bounds.clear();
        if (extents_needed) {
            const size_t grids_bytes = (n_systems * sizeof(GridParams) + 255) & ~size_t(255);
            const size_t firsts_bytes = ((n_systems + 1) * sizeof(uint32_t) + 255) & ~size_t(255);
            extras.sort_work.reserve(grids_bytes + firsts_bytes + n_systems * sizeof(BlockBounds));
            char* base = static_cast<char*>(extras.sort_work.ptr);
            auto* early_grids = reinterpret_cast<GridParams*>(base);
            auto* early_firsts = reinterpret_cast<uint32_t*>(base + grids_bytes);
            auto* d_bounds = reinterpret_cast<BlockBounds*>(base + grids_bytes + firsts_bytes);
            HIP_CHECK(hipMemcpyAsync(
                early_grids, grids.data(), n_systems * sizeof(GridParams), hipMemcpyHostToDevice, stream
            ));
            HIP_CHECK(hipMemcpyAsync(
                early_firsts, first_point_host.data(), (n_systems + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, stream
            ));
            const uint32_t blocks = static_cast<uint32_t>((n_systems + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK);
            hipLaunchKernelGGL(
                bounding_batch_kernel, dim3(blocks), dim3(BLOCK), 0, stream,
                reinterpret_cast<const double*>(points), early_grids, early_firsts, static_cast<uint32_t>(n_systems),
                d_bounds
            );
            bounds.resize(n_systems);
            HIP_CHECK(hipMemcpyAsync(
                bounds.data(), d_bounds, n_systems * sizeof(BlockBounds), hipMemcpyDeviceToHost, stream
            ));
            extras.sync(stream);
            unsigned int bad = 0xFFFFFFFFu;
            for (const BlockBounds& found : bounds) {
                bad = std::min(bad, found.first_bad_coordinate);
            }
            if (bad != 0xFFFFFFFFu) {
                non_finite_error(points, bad);
            }
        }

        setup.pair_base.resize(n_systems + 1);
        struct SecondPass {
            size_t systems_for_images = 0;
            size_t systems_for_tiles = 0;
            size_t systems_with_points = 0;
            size_t most_points = 0;
            uint32_t image_words = 1;
            double most_units = 1.0; // candidates per tile, in units of 64, of the system with the most (estimate)
        };
        std::vector<SecondPass> second_pass(n_parts);
        const double zeros[3] = {0.0, 0.0, 0.0};
        // (cell_base and pair_base receive every system's own cells and pairs of points first, their sums afterwards)
        over_the_systems(n_systems, n_parts, [&](size_t begin, size_t end, size_t part) {
        SecondPass mine;
        for (size_t s = begin; s < end; s++) {
            if (!extents_needed) {
                take_box(s);
            }
            const HostBox& hbox = host_grids_box[s];
            const size_t n_here = first_point[s + 1] - first_point[s];
            const double* lo = bounds.empty() ? zeros : bounds[s].lo;
            const double* hi = bounds.empty() ? zeros : bounds[s].hi;
            // (fewer than 32 points under the automatic choice: one cell whatever the grid would have been)
            bool single_cell = options.algorithm == VesinBruteForce || (options.algorithm == VesinAutoAlgorithm && n_here < 32);
            HostGrid grid = choose_grid(hbox, options.cutoff, n_here, lo, hi, single_cell);
            if (options.algorithm == VesinAutoAlgorithm && !single_cell && grid.n_cells == 1) {
                grid = choose_grid(hbox, options.cutoff, n_here, lo, hi, true);
            } else if (options.algorithm == VesinAutoAlgorithm && !single_cell && n_here <= IMAGE_MAX_POINTS) {
                // (a radius beyond what a stencil may have is an error of choose_grid: not for a choice that is only
                // tried)
                try {
                    const HostGrid one_cell = choose_grid(hbox, options.cutoff, n_here, lo, hi, true);
                    const uint64_t images = static_cast<uint64_t>(2 * one_cell.s[0] + 1) * (2 * one_cell.s[1] + 1) * (2 * one_cell.s[2] + 1);
                    if (one_cell_in_a_batch(n_here, images)) {
                        grid = one_cell;
                    }
                } catch (const std::runtime_error&) {
                }
            }
            GridParams& g = grids[s];
            for (int d = 0; d < 3; d++) {
                g.n[d] = grid.n[d];
                g.s[d] = grid.s[d];
                g.np_min[d] = grid.np_min[d];
                g.np_scale[d] = grid.np_scale[d];
            }
            g.cutoff2 = options.cutoff * options.cutoff;
            g.n_points = static_cast<uint32_t>(n_here);
            g.n_cells = static_cast<uint32_t>(grid.n_cells);
            choose_pruning(hbox, grid, options.cutoff, g);
            if (full_stencil_only()) {
                g.prune = 0;
            }
            const double per_cell = std::max(1.0, static_cast<double>(g.n_points) / std::max(1u, g.n_cells));
            mine.most_units = std::max(mine.most_units, std::ceil(upper_stencil_cells(g) * per_cell / WAVE));
            mine.systems_with_points += n_here > 0 ? 1 : 0;
            mine.most_points = std::max(mine.most_points, n_here);
            if (n_here > 0 && images_cover(g)) {
                mine.systems_for_images += 1;
                mine.image_words = std::max(mine.image_words, image_words(g));
            } else if (n_here > 0 && static_cast<uint64_t>(2 * g.s[0] + 1) * (2 * g.s[1] + 1) * (2 * g.s[2] + 1) <= MAX_ENTRIES) {
                mine.systems_for_tiles += 1;
            }
            setup.pair_base[s] = n_here <= IMAGE_MAX_POINTS ? n_here * n_here : 0;
            cell_base_host[s] = g.n_cells;
        }
        second_pass[part] = mine;
        });
        setup.systems_for_images = 0;
        setup.systems_for_tiles = 0;
        setup.systems_with_points = 0;
        setup.most_points = 0;
        setup.image_words = 1;
        double most_units = 1.0;
        for (const SecondPass& found : second_pass) {
            setup.systems_for_images += found.systems_for_images;
            setup.systems_for_tiles += found.systems_for_tiles;
            setup.systems_with_points += found.systems_with_points;
            setup.most_points = std::max(setup.most_points, found.most_points);
            setup.image_words = std::max(setup.image_words, found.image_words);
            most_units = std::max(most_units, found.most_units);
        }
        uint64_t cells_so_far = 0;
        uint64_t pairs_so_far = 0;
        for (size_t s = 0; s < n_systems; s++) {
            const uint64_t cells_here = cell_base_host[s];
            const uint64_t pairs_here = setup.pair_base[s];
            cell_base_host[s] = static_cast<uint32_t>(cells_so_far);
            setup.pair_base[s] = pairs_so_far;
            cells_so_far += cells_here;
            pairs_so_far += pairs_here;
            if (cells_so_far >= 0xFFFFFFF0ull) {
                throw std::runtime_error("too many cells in this batch");
            }
        }
        cell_base_host[n_systems] = static_cast<uint32_t>(cells_so_far);
        setup.pair_base[n_systems] = pairs_so_far;
        setup.total_cells = cells_so_far;
        setup.most_units = most_units;
        setup.valid = true;
    }
    if (!setup.kept_on_device && (!setup.any_open_direction || setup.all_open)) {
        // what the next call's boxes are compared with (never with some directions open and others not: the grids
        // follow the points and the boxes)
        setup.kept_boxes.reserve(75 * n_systems);
        auto* kept = static_cast<unsigned char*>(setup.kept_boxes.ptr);
        HIP_CHECK(hipMemcpyAsync(kept, setup.boxes.data(), 72 * n_systems, hipMemcpyHostToDevice, stream));
        HIP_CHECK(hipMemcpyAsync(kept + 72 * n_systems, setup.periodic.data(), 3 * n_systems, hipMemcpyHostToDevice, stream));
        setup.kept_on_device = true;
    }
    // Systems without any periodic direction, on a call that starts from the set-up of the call before: their grids
    // follow this call's points and are picked on the device, right before the cell lists are built (the host would
    // have to wait for the extents, pick the grids and send them back). The work buffers are sized for the most
    // cells such grids can have.
    const bool device_grids = speculate && setup.all_open;
    const uint64_t total_cells = device_grids ? setup.cells_bound : setup.total_cells;
    if (total_cells >= 0xFFFFFFF0ull) {
        throw std::runtime_error("too many cells in this batch");
    }

    if (n_points == 0) {
        size_outputs(neighbors, extras, 0, options);
        neighbors.length = 0;
        for (size_t s = 0; s <= n_systems; s++) {
            first_pair[s] = 0;
        }
        extras.batch_first_pair_device = nullptr; // (no kernel ran)
        return true;
    }
    // the first rows of the systems come to pinned memory and go on to the caller's array from there
    if (setup.first_pair_capacity < n_systems + 1) {
        if (setup.first_pair_landing != nullptr) {
            (void)hipHostFree(setup.first_pair_landing);
            setup.first_pair_landing = nullptr;
            setup.first_pair_capacity = 0;
        }
        const size_t wanted = (n_systems + 1) + (n_systems + 1) / 4;
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&setup.first_pair_landing), wanted * sizeof(size_t), hipHostMallocDefault));
        setup.first_pair_capacity = wanted;
    }

    // ---- work buffers
    size_t tiles_bound = std::min<size_t>(total_cells, n_points) + n_points / TILE_POINTS + 1;
    constexpr size_t slot_multiple = N_XCD * SEARCH_WAVES;
    tiles_bound = (tiles_bound + slot_multiple - 1) / slot_multiple * slot_multiple;
    uint32_t n_slices = 1;
    if (tiles_bound < 8192) {
        n_slices = static_cast<uint32_t>(std::min<size_t>(256, (8192 + tiles_bound - 1) / tiles_bound));
    }
    // the single-pass search keeps the hit columns of FUSED_UNITS units per work item: enough slices for the
    // system with the most candidates per tile (estimated from its mean occupation)
    {
        const double wanted = std::ceil(setup.most_units / FUSED_UNITS);
        if (wanted > n_slices) {
            n_slices = static_cast<uint32_t>(std::min(256.0, wanted));
        }
    }
    const size_t n_slots = tiles_bound * n_slices;
    const size_t search_workgroups = (n_slots + SEARCH_WAVES - 1) / SEARCH_WAVES;
    const size_t chain_groups = (search_workgroups + CHAIN_GROUP - 1) / CHAIN_GROUP;
    Chain chain = {};
    FusedStatus* fused_status = nullptr;

    uint32_t* cell_counts = nullptr;
    Tile* tiles = nullptr;
    uint64_t* cell_scan = nullptr;
    uint32_t* cell_of = nullptr;
    uint32_t* slot_of = nullptr;
    uint32_t* system_of = nullptr;
    int32_t* wrap_of = nullptr;
    SortedPoints sorted = {};
    uint32_t* counts = nullptr;
    uint64_t* offsets = nullptr;
    uint64_t* scan_scratch = nullptr;
    GridParams* d_grids = nullptr;
    uint32_t* d_first_point = nullptr;
    uint32_t* d_cell_base = nullptr;
    unsigned long long* d_first_pair = nullptr;
    uint32_t* d_cells_of_system = nullptr;
    char* clear_end = nullptr;
    // A sorted list straight from the search, when every system has the shape for one of the two that write their rows
    // in order: systems of one cell over their images (images.cuh), the others over the tiles of their whole stencil
    // (ordered.cuh). With grids picked on the device the host does not know the shapes: only the search over images is
    // tried then (such systems have no periodic direction and are mostly small), and its kernels say what they met.
    bool try_in_order = options.sorted && !radix_sort_only() &&
                        (device_grids || setup.systems_for_images + setup.systems_for_tiles == setup.systems_with_points);
    const bool in_order_images = device_grids || setup.systems_for_images > 0;
    const bool in_order_tiles = !device_grids && setup.systems_for_tiles > 0;
    // (what the counting passes leave for the writing passes: a bit per pair of points and image; a record per
    // candidate of every tile)
    const size_t hit_words = in_order_images ? static_cast<size_t>(setup.pair_base[n_systems]) * setup.image_words : 0;
    const size_t record_slots = in_order_tiles ? tiles_bound : 0;
    try_in_order = try_in_order &&
                   ordered_records_fit(
                       n_points, hit_words * sizeof(uint64_t) + record_slots * ORDERED_CANDIDATES * sizeof(CandidateRecord)
                   );
    if (try_in_order && setup.in_order_rest > 0) {
        setup.in_order_rest -= 1;
        try_in_order = false;
    }
    if (options.sorted && !device_grids && std::getenv("VESIN_HIP_DEBUG") != nullptr &&
        setup.systems_for_images + setup.systems_for_tiles != setup.systems_with_points) {
        std::fprintf(
            stderr, "sorted batch: %zu of %zu systems have a stencil of more than %d cells, the rows are sorted after the search\n",
            setup.systems_with_points - setup.systems_for_images - setup.systems_for_tiles, setup.systems_with_points, MAX_ENTRIES
        );
    }
    OrderedStatus* ordered_status = nullptr;
    uint32_t* rows_of_point = nullptr;
    uint64_t* first_row_of_point = nullptr;
    uint64_t* image_hits = nullptr;
    uint64_t* d_pair_base = nullptr;
    CandidateRecord* candidate_records = nullptr;
    uint32_t* candidates_of_item = nullptr;
    uint16_t* candidate_order = nullptr;
    const size_t scratch_elements = std::max(
        std::max(scan_scratch_elements(total_cells), scan_scratch_elements(n_slots)),
        try_in_order ? scan_scratch_elements(n_points) : size_t(0)
    );
    auto carve = [&](Carver& carver) {
        // adjacent, so that one fill clears the histogram, the tiles' flags and the state of the single-pass search
        cell_counts = carver.take<uint32_t>(total_cells);
        tiles = carver.take<Tile>(tiles_bound);
        chain.blocks = carver.take<uint64_t>(search_workgroups);
        chain.groups = carver.take<uint64_t>(chain_groups);
        chain.bases = carver.take<uint64_t>(chain_groups);
        fused_status = carver.take<FusedStatus>(1);
        counts = carver.take<uint32_t>(n_slots);
        ordered_status = carver.take<OrderedStatus>(try_in_order ? 1 : 0);
        rows_of_point = carver.take<uint32_t>(try_in_order ? n_points : 0);
        clear_end = reinterpret_cast<char*>(carver.take<uint32_t>(0));
        first_row_of_point = carver.take<uint64_t>(try_in_order ? n_points + 1 : 0);
        cell_scan = carver.take<uint64_t>(total_cells + 1);
        cell_of = carver.take<uint32_t>(n_points);
        slot_of = carver.take<uint32_t>(n_points);
        system_of = carver.take<uint32_t>(n_points);
        wrap_of = carver.take<int32_t>(3 * n_points);
        sorted.p = carver.take<SortedPoint>(n_points + SORTED_PADDING);
        sorted.l = nullptr; // (no search of a batch uses the places inside the cells)
        sorted.wx = carver.take<int32_t>(n_points + SORTED_PADDING);
        sorted.wy = carver.take<int32_t>(n_points + SORTED_PADDING);
        sorted.wz = carver.take<int32_t>(n_points + SORTED_PADDING);
        offsets = carver.take<uint64_t>(n_slots + 1);
        scan_scratch = carver.take<uint64_t>(scratch_elements);
        d_grids = carver.take<GridParams>(n_systems);
        d_first_point = carver.take<uint32_t>(n_systems + 1);
        d_cell_base = carver.take<uint32_t>(n_systems + 1);
        d_first_pair = carver.take<unsigned long long>(n_systems + 1);
        d_cells_of_system = carver.take<uint32_t>(n_systems);
        d_pair_base = carver.take<uint64_t>(try_in_order ? n_systems + 1 : 0);
        image_hits = carver.take<uint64_t>(try_in_order ? hit_words : 0);
        candidate_records = carver.take<CandidateRecord>(try_in_order ? record_slots * ORDERED_CANDIDATES : 0);
        candidates_of_item = carver.take<uint32_t>(try_in_order ? record_slots : 0);
        candidate_order = carver.take<uint16_t>(try_in_order ? record_slots * ORDERED_CANDIDATES : 0);
    };
    Carver measure(nullptr);
    carve(measure);
    extras.work.reserve(measure.used);
    Carver carver(extras.work.ptr);
    carve(carver);
    extras.batch_first_pair_device = d_first_pair;

    if (try_in_order && !(same_setup && setup.on_device && setup.work_generation == extras.work.generation &&
                          setup.d_pair_base == d_pair_base)) {
        HIP_CHECK(hipMemcpyAsync(
            d_pair_base, setup.pair_base.data(), (n_systems + 1) * sizeof(uint64_t), hipMemcpyHostToDevice, stream
        ));
        setup.d_pair_base = d_pair_base;
    }
    const bool already_there = same_setup && setup.on_device && setup.work_generation == extras.work.generation &&
                               setup.d_grids == d_grids &&
                               setup.d_first_point == d_first_point && setup.d_cell_base == d_cell_base;
    if (device_grids) {
        setup.on_device = false; // (grids and first cells of this call are the device's own)
        HIP_CHECK(hipMemcpyAsync(
            d_first_point, first_point_host.data(), (n_systems + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, stream
        ));
    } else if (!already_there) {
        setup.on_device = false;
        HIP_CHECK(hipMemcpyAsync(d_grids, grids.data(), n_systems * sizeof(GridParams), hipMemcpyHostToDevice, stream));
        HIP_CHECK(hipMemcpyAsync(
            d_first_point, first_point_host.data(), (n_systems + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, stream
        ));
        HIP_CHECK(hipMemcpyAsync(
            d_cell_base, cell_base_host.data(), (n_systems + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, stream
        ));
        setup.d_grids = d_grids;
        setup.d_first_point = d_first_point;
        setup.d_cell_base = d_cell_base;
        setup.work_generation = extras.work.generation;
        setup.on_device = true;
    }

    // ---- cell lists of all systems, in one sequence of launches
    const uint32_t point_blocks = static_cast<uint32_t>((n_points + BLOCK - 1) / BLOCK);
    const auto* flat_points = reinterpret_cast<const double*>(points);
    {
        // one launch clears the histogram, the tiles' flags, the state of the single-pass search and the counts, and
        // resets the status block (every piece of the work buffer is padded to 256 bytes: whole 16-byte blocks)
        const size_t blocks16 = (clear_end - reinterpret_cast<char*>(cell_counts) + 15) / 16;
        const uint32_t fill_blocks = static_cast<uint32_t>(std::min<size_t>(1024, (blocks16 + BLOCK - 1) / BLOCK));
        hipLaunchKernelGGL(
            clear_and_fetch, dim3(fill_blocks), dim3(BLOCK), 0, stream,
            reinterpret_cast<uint4*>(cell_counts), blocks16, reinterpret_cast<const double*>(boxes),
            reinterpret_cast<const bool*>(periodic), extras.mail_device->small, extras.d_status
        );
    }
    if (device_grids) {
        // (behind the launch that resets the status block: a coordinate that is not finite is reported there)
        extras.mail->batch_total_cells = 0;
        const int single_cell = options.algorithm == VesinBruteForce ? 1 : options.algorithm == VesinAutoAlgorithm ? 0 : -1;
        hipLaunchKernelGGL(
            open_grids_kernel, dim3(static_cast<uint32_t>((n_systems + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK)), dim3(BLOCK),
            0, stream, flat_points, d_first_point, static_cast<uint32_t>(n_systems), options.cutoff, single_cell,
            IMAGE_MAX_POINTS + 1, d_grids, d_cells_of_system, &extras.d_status->first_bad_coordinate
        );
        hipLaunchKernelGGL(
            open_bases_kernel, dim3(1), dim3(1024), 0, stream,
            d_cells_of_system, static_cast<uint32_t>(n_systems), d_cell_base, &extras.mail_device->batch_total_cells
        );
    }
    hipLaunchKernelGGL(
        assign_cells_batch, dim3(point_blocks), dim3(BLOCK), 0, stream,
        flat_points, static_cast<uint32_t>(n_points), d_grids, d_first_point, d_cell_base,
        static_cast<uint32_t>(n_systems), cell_of, slot_of, wrap_of, system_of, cell_counts, extras.d_status
    );
    exclusive_scan<SCAN_CELL_COUNTS>(cell_counts, total_cells, cell_scan, scan_scratch, stream);
    hipLaunchKernelGGL(
        place_points, dim3(point_blocks), dim3(BLOCK), 0, stream,
        flat_points, GridParams{}, wrap_of, cell_of, slot_of, cell_scan, static_cast<uint32_t>(n_points), sorted, tiles,
        system_of, d_first_point
    );

    // ---- count, scan, write
    SearchArgs args = {};
    args.sorted = sorted;
    args.cell_scan = cell_scan;
    args.tiles = tiles;
    args.counts = counts;
    args.offsets = offsets;
    args.n_slices = n_slices;
    args.n_work = static_cast<uint32_t>(n_slots);
    args.grids = d_grids;
    args.cell_base = d_cell_base;
    args.total_cells = static_cast<uint32_t>(total_cells);
    const uint32_t system_blocks = static_cast<uint32_t>((n_systems + 1 + BLOCK - 1) / BLOCK);
    static_assert(sizeof(size_t) == sizeof(unsigned long long), "size_t is 64 bits wide here");

    auto setup_changed = [&]() {
        // other boxes than the grids were picked from, or (which open_grids_kernel rules out) more cells than the
        // buffers were sized for: nothing of this attempt is used, the host picks the grids
        return speculate && (extras.mail->batch_changed != 0 || (device_grids && extras.mail->batch_total_cells > total_cells));
    };
    auto check_pair_limit = [&](size_t total) {
        if (pair_limit != 0 && total > n_points * pair_limit) {
            throw std::runtime_error(
                "The number of neighbor pairs exceeds the maximum capacity of " + std::to_string(n_points * pair_limit) +
                " (max_pairs_per_point=" + std::to_string(pair_limit) + "; n_points=" + std::to_string(n_points) + "). " +
                "Consider reducing the cutoff distance, or explicitly setting " +
                "VESIN_CUDA_MAX_PAIRS_PER_POINT as an environment variable."
            );
        }
    };

    // ---- a sorted list straight from the search: systems of one cell by brute force over their images in the order
    // of the list (images.cuh), the others by the tiles of their whole stencil (ordered.cuh); one scan over the points
    // of all systems gives every point its first row
    if (try_in_order) {
        ImageArgs iargs = {};
        iargs.sorted = sorted;
        iargs.cell_scan = cell_scan;
        iargs.grids = d_grids;
        iargs.cell_base = d_cell_base;
        iargs.first_point = d_first_point;
        iargs.pair_base = d_pair_base;
        iargs.hits = image_hits;
        iargs.words = setup.image_words;
        iargs.cutoff = options.cutoff;
        iargs.double_only = double_precision_only() ? 1u : 0u;
        iargs.n_systems = static_cast<uint32_t>(n_systems);
        iargs.total_points = static_cast<uint32_t>(n_points);
        iargs.others_covered = in_order_tiles ? 1u : 0u;
        iargs.rows_of_point = rows_of_point;
        iargs.first_row = first_row_of_point;
        iargs.status = ordered_status;
        OrderedArgs oargs = {};
        oargs.sorted = sorted;
        oargs.cell_scan = cell_scan;
        oargs.tiles = tiles;
        oargs.points_per_item = TILE_POINTS;
        oargs.items_per_tile = 1;
        oargs.rows_of_point = rows_of_point;
        oargs.records = candidate_records;
        oargs.candidates_of_item = candidates_of_item;
        oargs.write_split = 1;
        oargs.count_split = 1;
        oargs.points = flat_points;
        oargs.order = candidate_order;
        oargs.first_row = first_row_of_point;
        oargs.status = ordered_status;
        oargs.grids = d_grids;
        oargs.cell_base = d_cell_base;
        oargs.first_point = d_first_point;
        oargs.total_cells = static_cast<uint32_t>(total_cells);
        oargs.total_points = static_cast<uint32_t>(n_points);
        // (a wave per system instead of a workgroup when no system has more than a few points)
        const bool few_points = setup.most_points <= IMAGE_FEW_POINTS;
        const dim3 image_grid(static_cast<uint32_t>(few_points ? (n_systems + IMAGE_WAVES - 1) / IMAGE_WAVES : n_systems));
        const dim3 tile_grid(static_cast<uint32_t>((tiles_bound + ORDERED_WAVES - 1) / ORDERED_WAVES));
        // (whichever writing pass is launched last hands the host what the counting passes found)
        auto launch_write = [&](OrderedHostStatus* publish_to) {
            if (in_order_images) {
                iargs.publish_to = in_order_tiles ? nullptr : publish_to;
                iargs.build_status = extras.d_status;
                // (calls that return vectors take the kernels that line them up in LDS before they store them)
                const bool staged = iargs.out.vectors != nullptr;
                auto kernel =
                    staged ? (few_points ? (options.full ? image_write_kernel<true, true, true> : image_write_kernel<false, true, true>)
                                         : (options.full ? image_write_kernel<true, false, true> : image_write_kernel<false, false, true>))
                           : (few_points ? (options.full ? image_write_kernel<true, true> : image_write_kernel<false, true>)
                                         : (options.full ? image_write_kernel<true, false> : image_write_kernel<false, false>));
                hipLaunchKernelGGL(kernel, image_grid, dim3(IMAGE_BLOCK), 0, stream, iargs);
            }
            if (in_order_tiles) {
                oargs.publish_to = publish_to;
                oargs.build_status = extras.d_status;
                if (options.full) {
                    hipLaunchKernelGGL((ordered_search_kernel<true, true, true, true>), tile_grid, dim3(ORDERED_BLOCK), 0, stream, oargs, GridParams{});
                } else {
                    hipLaunchKernelGGL((ordered_search_kernel<true, false, true, true>), tile_grid, dim3(ORDERED_BLOCK), 0, stream, oargs, GridParams{});
                }
            }
        };
        auto outputs_into = [&](SearchOutputs& out) {
            out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
            out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
            out.distances = neighbors.distances;
            out.vectors = reinterpret_cast<double*>(neighbors.vectors);
        };
        if (in_order_images) {
            auto kernel = few_points ? (options.full ? image_count_kernel<true, true> : image_count_kernel<false, true>)
                                     : (options.full ? image_count_kernel<true, false> : image_count_kernel<false, false>);
            hipLaunchKernelGGL(kernel, image_grid, dim3(IMAGE_BLOCK), 0, stream, iargs);
        }
        if (in_order_tiles) {
            if (options.full) {
                hipLaunchKernelGGL((ordered_search_kernel<false, true, false, true>), tile_grid, dim3(ORDERED_BLOCK), 0, stream, oargs, GridParams{});
            } else {
                hipLaunchKernelGGL((ordered_search_kernel<false, false, false, true>), tile_grid, dim3(ORDERED_BLOCK), 0, stream, oargs, GridParams{});
            }
            hipLaunchKernelGGL(
                ordered_sort_kernel<true>, dim3(static_cast<uint32_t>((tiles_bound + ORDER_WAVES - 1) / ORDER_WAVES)),
                dim3(ORDER_BLOCK), 0, stream, oargs, GridParams{}
            );
        }
        exclusive_scan<SCAN_U32>(rows_of_point, n_points, first_row_of_point, scan_scratch, stream);
        // A list that has arrays from earlier calls writes into them without waiting for the host to learn what the
        // counting pass found: the launch checks on the device that every system was covered and that the rows fit
        const bool early_write = extras.capacity > 0;
        size_t early_capacity = 0;
        if (early_write) {
            size_outputs(neighbors, extras, 0, options);
            early_capacity = extras.capacity;
            outputs_into(iargs.out);
            outputs_into(oargs.out);
            iargs.capacity = oargs.capacity = early_capacity;
            iargs.guarded = oargs.guarded = 1;
            launch_write(&extras.mail_device->ordered);
        } else {
            hipLaunchKernelGGL(
                publish_ordered_status, dim3(1), dim3(1), 0, stream,
                ordered_status, first_row_of_point + n_points, extras.d_status, cell_scan + total_cells,
                &extras.mail_device->ordered
            );
        }
        hipLaunchKernelGGL(
            first_rows_of_systems_kernel, dim3(system_blocks), dim3(BLOCK), 0, stream,
            first_row_of_point, d_first_point, static_cast<uint32_t>(n_systems), d_first_pair
        );
        HIP_CHECK(hipMemcpyAsync(
            setup.first_pair_landing, d_first_pair, (n_systems + 1) * sizeof(size_t), hipMemcpyDeviceToHost, stream
        ));
        extras.sync(stream);
        if (setup_changed()) {
            return false;
        }
        const OrderedHostStatus found = extras.mail->ordered;
        if (found.first_bad_coordinate != 0xFFFFFFFFu) {
            non_finite_error(points, found.first_bad_coordinate);
        }
        const bool suitable = found.found.unsuitable == 0 && found.found.max_rows <= ORDERED_MAX_ROWS &&
                              found.found.max_candidates <= ORDERED_CANDIDATES;
        if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
            std::fprintf(
                stderr,
                "in-order search (batch): rows %llu, %zu systems by images, %zu by tiles (most rows of a point %u, most "
                "candidates of a tile %u), unsuitable %u%s: %s\n",
                found.total_rows, setup.systems_for_images, in_order_tiles ? setup.systems_for_tiles : size_t(0),
                found.found.max_rows, found.found.max_candidates, found.found.unsuitable,
                device_grids ? ", grids picked on the device" : "", suitable ? "used" : "left to the radix sort"
            );
        }
        if (suitable) {
            const size_t total = found.total_rows;
            check_pair_limit(total);
            if (!(early_write && total <= early_capacity)) {
                // first call of the list, or more rows than its arrays hold
                size_outputs(neighbors, extras, total, options);
                outputs_into(iargs.out);
                outputs_into(oargs.out);
                iargs.guarded = oargs.guarded = 0;
                if (total > 0) {
                    launch_write(nullptr);
                }
                extras.sync(stream);
            }
            HIP_CHECK(hipGetLastError());
            std::memcpy(first_pair, setup.first_pair_landing, (n_systems + 1) * sizeof(size_t));
            neighbors.length = total;
            return true;
        }
        // a system beyond what either search covers (grids picked on the device: of several cells, of many points; more
        // than 256 rows for a point or 1024 candidates around a tile; wraps beyond +-255): the two passes and the sort
        // below, and for a while without asking again
        setup.in_order_rest = SINGLE_PASS_REST;
    }

    // ---- a list that has arrays from earlier calls: single-pass search straight into them, rows in work-item order
    // (the rows of a system stay together). Whatever does not fit its shape starts over with the two passes below.
    // (a sorted list is sorted afterwards: its rows go to scratch memory first, through the two passes)
    if (extras.capacity > 0 && !two_pass_only() && !options.sorted && !setup.chain_rest.resting()) {
        size_outputs(neighbors, extras, 0, options);
        FusedArgs fargs = {};
        fargs.search = args;
        fargs.search.out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
        fargs.search.out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
        fargs.search.out.distances = neighbors.distances;
        fargs.search.out.vectors = reinterpret_cast<double*>(neighbors.vectors);
        fargs.search.capacity = extras.capacity;
        fargs.chain = chain;
        fargs.first_rows = offsets;
        fargs.status = fused_status;
        fargs.spin_limit = chain_spin_limit();
        fargs.wait_ticks = chain_wait_ticks();
        const uint32_t blocks = static_cast<uint32_t>(search_workgroups);
        const bool staged = staged_vectors(fargs.search.out, options.full);
        auto kernel = staged ? (options.full ? fused_search_kernel<true, true, true, true> : fused_search_kernel<false, true, true, true>)
                             : (options.full ? fused_search_kernel<true, true, true> : fused_search_kernel<false, true, true>);
        hipLaunchKernelGGL(kernel, dim3(blocks), dim3(SEARCH_BLOCK), 0, stream, fargs, GridParams{});
        hipLaunchKernelGGL(publish_fused_status, dim3(1), dim3(1), 0, stream, extras.d_status, fused_status, &extras.mail_device->fused);
        hipLaunchKernelGGL(
            system_rows_kernel, dim3(system_blocks), dim3(BLOCK), 0, stream,
            cell_scan, d_cell_base, offsets, static_cast<uint32_t>(n_systems), n_slices, static_cast<uint32_t>(n_slots),
            fused_status, d_first_pair, reinterpret_cast<unsigned long long*>(setup.first_pair_landing)
        );
        extras.batch_first_pair_device = d_first_pair;
        bool published_here = false;
        if (extras.before_the_stop_of_a_queued_call()) {
            hipLaunchKernelGGL(
                publish_queued_batch_length, dim3(1), dim3(1), 0, stream, extras.mail_device, speculate ? 1 : 0,
                device_grids ? 1 : 0, static_cast<unsigned long long>(total_cells),
                static_cast<unsigned long long>(pair_limit != 0 ? n_points * pair_limit : 0), extras.d_queued_length
            );
            extras.length_published = true;
            published_here = true;
        }
        extras.sync(stream);
        if (speculate && (extras.mail->batch_changed != 0 || (device_grids && extras.mail->batch_total_cells > total_cells))) {
            // other boxes than the grids were picked from, or (which open_grids_kernel rules out) more cells than
            // the buffers were sized for: nothing of this attempt is used, the host picks the grids
            return false;
        }
        const FusedStatus result = extras.mail->fused;
        if (result.first_bad_coordinate != 0xFFFFFFFFu) {
            non_finite_error(points, result.first_bad_coordinate);
        }
        if (std::getenv("VESIN_HIP_DEBUG") != nullptr) {
            std::fprintf(
                stderr, "single pass (batch): rows %llu general %u deferred %u overflow %u timeout %u (slices %u%s)\n",
                result.total_rows, result.general, result.deferred, result.overflow, result.chain_timeout, n_slices,
                device_grids ? ", grids picked on the device" : speculate ? ", grids of the call before" : ""
            );
        }
        if (result.general == 0 && result.deferred == 0 && result.overflow == 0 && result.chain_timeout == 0) {
            if (pair_limit != 0 && result.total_rows > n_points * pair_limit) {
                throw std::runtime_error(
                    "The number of neighbor pairs exceeds the maximum capacity of " + std::to_string(n_points * pair_limit) +
                    " (max_pairs_per_point=" + std::to_string(pair_limit) + "; n_points=" + std::to_string(n_points) + "). " +
                    "Consider reducing the cutoff distance, or explicitly setting " +
                    "VESIN_CUDA_MAX_PAIRS_PER_POINT as an environment variable."
                );
            }
            HIP_CHECK(hipGetLastError());
            std::memcpy(first_pair, setup.first_pair_landing, (n_systems + 1) * sizeof(size_t));
            neighbors.length = result.total_rows;
            setup.chain_rest.went_through();
            extras.queued_part_sufficed = published_here;
            return true;
        }
        if (result.chain_timeout != 0) {
            // waves gave up waiting for the rows of earlier workgroups (a GPU shared with other work): the two passes
            // below give this call's rows, and the next calls go there directly
            setup.chain_rest.gave_up();
        }
    }

    launch_search_batch<false>(options.full, args, stream);
    exclusive_scan<SCAN_U32>(counts, n_slots, offsets, scan_scratch, stream);
    hipLaunchKernelGGL(publish_status, dim3(1), dim3(1), 0, stream, extras.d_status, offsets + n_slots, &extras.mail_device->status);
    extras.sync(stream);
    if (speculate && (extras.mail->batch_changed != 0 || (device_grids && extras.mail->batch_total_cells > total_cells))) {
        return false;
    }
    if (extras.mail->status.first_bad_coordinate != 0xFFFFFFFFu) {
        non_finite_error(points, extras.mail->status.first_bad_coordinate);
    }
    const size_t total = extras.mail->status.total_pairs;
    if (pair_limit != 0 && total > n_points * pair_limit) {
        throw std::runtime_error(
            "The number of neighbor pairs exceeds the maximum capacity of " + std::to_string(n_points * pair_limit) +
            " (max_pairs_per_point=" + std::to_string(pair_limit) + "; n_points=" + std::to_string(n_points) + "). " +
            "Consider reducing the cutoff distance, or explicitly setting " +
            "VESIN_CUDA_MAX_PAIRS_PER_POINT as an environment variable."
        );
    }

    size_outputs(neighbors, extras, total, options);
    SearchOutputs final_out;
    final_out.pairs = reinterpret_cast<unsigned long long*>(neighbors.pairs);
    final_out.shifts = reinterpret_cast<int32_t*>(neighbors.shifts);
    final_out.distances = neighbors.distances;
    final_out.vectors = reinterpret_cast<double*>(neighbors.vectors);
    // a sorted list: the rows go to scratch rows (shifts always among them, they are part of the order) and the
    // sort's last step fills the caller's arrays
    const bool sorting = options.sorted && total > 1;
    SearchOutputs unsorted = final_out;
    SortWorkspace sort_space = {};
    sort_space.host_ranges = extras.mail->ranges;
    sort_space.device_ranges = extras.mail_device->ranges;
    if (sorting) {
        carve_sort_space(extras, total, options, unsorted, sort_space);
    }
    args.out = unsorted;
    args.capacity = sorting ? total : extras.capacity;
    if (total > 0) {
        launch_search_batch<true>(options.full, args, stream);
    }
    hipLaunchKernelGGL(
        system_rows_kernel, dim3(system_blocks), dim3(BLOCK), 0, stream,
        cell_scan, d_cell_base, offsets, static_cast<uint32_t>(n_systems), n_slices, static_cast<uint32_t>(n_slots),
        static_cast<const FusedStatus*>(nullptr), d_first_pair, reinterpret_cast<unsigned long long*>(setup.first_pair_landing)
    );
    if (sorting) {
        // every system's rows stay in their range and come out ordered by (i, j, shift) inside it: the order of
        // vesin_neighbors on that system alone
        BatchRows rows_of_systems;
        rows_of_systems.first_pair = d_first_pair;
        rows_of_systems.first_point = d_first_point;
        rows_of_systems.n_systems = static_cast<uint32_t>(n_systems);
        sort_pairs(unsorted, final_out, total, n_points, sort_space, stream, rows_of_systems);
    }
    extras.sync(stream);
    HIP_CHECK(hipGetLastError());
    std::memcpy(first_pair, setup.first_pair_landing, (n_systems + 1) * sizeof(size_t));
    neighbors.length = total;
    return true;
}

// ---- the entry point that allocates nothing
//
// Callers that cannot allocate device memory (tight loops, harnesses that forbid it) bring their own output arrays;
// what a call needs besides them (the cell list, the counters and tables of the search, the status block and the
// block the kernels report to the host through) is carved from one array of device memory that is part of this
// library's code object, so every GPU the library runs on holds it from the moment the library is loaded until the
// process ends. In host code the array's name only stands for the symbol: its address on the current device comes
// from hipGetSymbolAddress, once per device, and only that pointer is ever handed to kernels or copies.
constexpr size_t FIXED_SCRATCH_BYTES = size_t(64) << 20;
constexpr size_t FIXED_STATUS_BYTES = 256;
constexpr size_t FIXED_MAIL_BYTES = (sizeof(Mailbox) + 255) & ~size_t(255);
constexpr size_t FIXED_SORT_BYTES = size_t(8) << 20; // rows and tables of the radix sort, for sorted lists that need it
constexpr size_t FIXED_WORK_BYTES = FIXED_SCRATCH_BYTES - FIXED_STATUS_BYTES - FIXED_MAIL_BYTES - FIXED_SORT_BYTES;
constexpr size_t FIXED_MAX_POINTS = size_t(1) << 18;
constexpr int FIXED_MAX_DEVICES = 64;

static __device__ __align__(256) unsigned char scratch[FIXED_SCRATCH_BYTES];

/// One per GPU, part of the library's own data: nothing is allocated for it, not on the host either. Calls on one
/// GPU share the array, so they take turns (the lock is held for the whole call).
struct FixedState {
    std::mutex turn;
    bool ready = false;
    unsigned char* memory = nullptr; // address of `scratch` on this GPU
    Mailbox host_mail;               // where the block the kernels report through is copied before every wait
    HipExtras extras;
};

std::mutex FIXED_SETUP;
FixedState FIXED_STATES[FIXED_MAX_DEVICES];

/// The state of GPU `device_id`, which must be the current device. The first call on a GPU looks up where that
/// GPU holds the array.
FixedState& fixed_state_of(int device_id) {
    if (device_id >= FIXED_MAX_DEVICES) {
        throw std::runtime_error("the entry point that allocates nothing serves GPUs 0 to " + std::to_string(FIXED_MAX_DEVICES - 1));
    }
    const std::lock_guard<std::mutex> setup(FIXED_SETUP);
    FixedState& state = FIXED_STATES[device_id];
    if (!state.ready) {
        void* address = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
        if (address == nullptr) {
            throw std::runtime_error("internal error: the work array of the library has no address on this GPU");
        }
        state.memory = static_cast<unsigned char*>(address);
        unsigned char* next = state.memory;
        HipExtras& extras = state.extras;
        extras.device_id = device_id;
        extras.fixed_memory = true;
        extras.d_status = reinterpret_cast<DeviceStatus*>(next);
        // the two meetings of the one launch of small systems: zero like the whole array when the library is loaded,
        // and left zero for the next launch by every launch that uses them
        static_assert(sizeof(DeviceStatus) <= 128 && 128 + 2 * sizeof(SmallMeeting) <= FIXED_STATUS_BYTES, "status block");
        extras.meetings = reinterpret_cast<SmallMeeting*>(next + 128);
        extras.own_meetings = false;
        next += FIXED_STATUS_BYTES;
        extras.mail_device = reinterpret_cast<Mailbox*>(next);
        extras.mail = &state.host_mail;
        next += FIXED_MAIL_BYTES;
        extras.work.ptr = next;
        extras.work.bytes = FIXED_WORK_BYTES;
        extras.work.fixed = true;
        next += FIXED_WORK_BYTES;
        extras.sort_work.ptr = next;
        extras.sort_work.bytes = FIXED_SORT_BYTES;
        extras.sort_work.fixed = true;
        state.ready = true;
    }
    return state;
}

} // namespace

void neighbors_no_alloc(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinOptions options,
    int device_id,
    size_t (*pairs)[2],
    int32_t (*shifts)[3],
    double* distances,
    double (*vectors)[3],
    size_t capacity,
    size_t& length,
    void* caller_stream
) {
    hipStream_t stream = static_cast<hipStream_t>(caller_stream);
    check_inputs(points, n_points, box, periodic, device_id);
    if (n_points > FIXED_MAX_POINTS) {
        throw std::runtime_error(
            "the entry point that allocates nothing takes at most " + std::to_string(FIXED_MAX_POINTS) + " points, got " +
            std::to_string(n_points) + ": use vesin_neighbors for larger systems"
        );
    }
    if (options.skin > 0.0) {
        throw std::runtime_error("a non-zero `skin` (Verlet caching) keeps device memory between calls: use vesin_neighbors for it");
    }
    struct Wanted {
        const void* pointer;
        bool wanted;
        const char* name;
    };
    const Wanted arrays[] = {
        {pairs, true, "pairs"},
        {shifts, options.return_shifts, "shifts"},
        {distances, options.return_distances, "distances"},
        {vectors, options.return_vectors, "vectors"},
    };
    for (const Wanted& array : arrays) {
        if (!array.wanted || capacity == 0) {
            continue;
        }
        if (array.pointer == nullptr) {
            throw std::runtime_error(std::string("`") + array.name + "` is requested and can not be a NULL pointer");
        }
        if (device_of(array.pointer) != device_id) {
            throw std::runtime_error(std::string("`") + array.name + "` is not memory of the GPU the list is computed on");
        }
    }

    const DeviceGuard guard(device_id);
    FixedState& state = fixed_state_of(device_id);
    const std::lock_guard<std::mutex> turn(state.turn);
    HipExtras& extras = state.extras;
    // nothing is carried over from the call before: it may have been another caller's system
    extras.capacity = capacity;
    extras.guess = BoxGuess();
    extras.single_pass_rest = 0;
    extras.direct_rest = 0;
    extras.in_order_rest = 0;
    extras.one_launch_rest = 0;
    extras.extent_valid = false;
    extras.timings_valid = false;
    // (`meeting_rest` stays: workgroups that gave up waiting for each other say something about this GPU, not about
    // the system of the call before)

    VesinNeighborList list;
    list.device.type = VesinCUDA;
    list.device.device_id = device_id;
    list.pairs = capacity == 0 ? nullptr : pairs;
    list.shifts = options.return_shifts && capacity != 0 ? shifts : nullptr;
    list.distances = options.return_distances && capacity != 0 ? distances : nullptr;
    list.vectors = options.return_vectors && capacity != 0 ? vectors : nullptr;
    try {
        direct_neighbors(points, n_points, box, periodic, options, list, extras, stream);
    } catch (const RowsDoNotFit& error) {
        length = error.rows;
        throw;
    }
    length = list.length;
}

void free_neighbors(VesinNeighborList& neighbors) {
    const DeviceGuard guard(neighbors.device.device_id);
    if (auto* extras = static_cast<HipExtras*>(neighbors.opaque)) {
        if (extras->enqueued) {
            // a queued call that nobody collected: it runs to its end first (its kernels write into these arrays)
            try {
                if (!extras->queued->finished) {
                    extras->queued->resume();
                }
                finish_queued(neighbors, *extras, extras->queued_stream);
            } catch (...) {
            }
        }
    }
    free_outputs(neighbors, static_cast<const HipExtras*>(neighbors.opaque));
    delete static_cast<HipExtras*>(neighbors.opaque);
    neighbors.opaque = nullptr;
}

void set_output_allocator(VesinNeighborList& neighbors, VesinHipAllocate allocate, VesinHipRelease release, void* context) {
    if ((allocate == nullptr) != (release == nullptr)) {
        throw std::runtime_error("`allocate` and `release` come together: both functions, or NULL for both");
    }
    int device_count = 0;
    if (hipGetDeviceCount(&device_count) != hipSuccess || device_count == 0) {
        (void)hipGetLastError();
        throw std::runtime_error("no HIP device is available to this process");
    }
    if (neighbors.device.device_id < 0 || neighbors.device.device_id >= device_count) {
        throw std::runtime_error("invalid GPU device_id " + std::to_string(neighbors.device.device_id));
    }
    const DeviceGuard guard(neighbors.device.device_id);
    HipExtras& extras = extras_of(neighbors);
    refuse_while_queued(extras);
    // what the list holds goes back the way it came; the next call makes arrays of the same size with the new functions
    free_outputs(neighbors, &extras);
    extras.allocate = allocate;
    extras.release = release;
    extras.allocator_context = context;
}

size_t detach_outputs(VesinNeighborList& neighbors) {
    auto* extras = static_cast<HipExtras*>(neighbors.opaque);
    if (extras == nullptr) {
        // no call yet: there is nothing to hand over
        neighbors.pairs = nullptr;
        neighbors.shifts = nullptr;
        neighbors.distances = nullptr;
        neighbors.vectors = nullptr;
        return 0;
    }
    if (extras->fixed_memory) {
        throw std::runtime_error("internal error: the arrays of this list are the caller's already");
    }
    refuse_while_queued(*extras);
    neighbors.pairs = nullptr;
    neighbors.shifts = nullptr;
    neighbors.distances = nullptr;
    neighbors.vectors = nullptr;
    return extras->capacity;
}

const unsigned long long* batch_first_pair_on_device(const VesinNeighborList& neighbors) {
    const auto* extras = static_cast<const HipExtras*>(neighbors.opaque);
    return extras == nullptr ? nullptr : extras->batch_first_pair_device;
}

size_t output_capacity(const VesinNeighborList& neighbors) {
    const auto* extras = static_cast<const HipExtras*>(neighbors.opaque);
    return extras == nullptr || neighbors.pairs == nullptr ? 0 : extras->capacity;
}

void pairs_backward(
    const size_t (*pairs)[2],
    const int32_t (*shifts)[3],
    const double* distances,
    const double (*vectors)[3],
    size_t n_pairs,
    const double* distances_grad,
    const double (*vectors_grad)[3],
    size_t n_points,
    int device_id,
    double (*points_grad)[3],
    double (*box_grad)[3],
    void* caller_stream
) {
    if (n_pairs == 0 || (points_grad == nullptr && box_grad == nullptr)) {
        return;
    }
    if (distances_grad == nullptr && vectors_grad == nullptr) {
        return;
    }
    if (pairs == nullptr) {
        throw std::runtime_error("`pairs` can not be a NULL pointer");
    }
    if (distances_grad != nullptr && (distances == nullptr || vectors == nullptr)) {
        throw std::runtime_error("the gradient of distances needs both `distances` and `vectors`");
    }
    if (box_grad != nullptr && shifts == nullptr) {
        throw std::runtime_error("the gradient of the box needs `shifts`");
    }
    const void* on_device[] = {pairs, shifts, distances, vectors, distances_grad, vectors_grad, points_grad, box_grad};
    for (const void* pointer : on_device) {
        if (pointer != nullptr && device_of(pointer) != device_id) {
            throw std::runtime_error("every array of the gradient must be memory of the device it is computed on");
        }
    }

    const DeviceGuard guard(device_id);
    // one flag per host thread, in pinned memory every device can write to
    thread_local uint32_t* bad_index = nullptr;
    if (bad_index == nullptr) {
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&bad_index), sizeof(uint32_t), hipHostMallocPortable));
    }
    *bad_index = 0;

    BackwardArgs args;
    args.pairs = pairs;
    args.shifts = box_grad != nullptr ? shifts : nullptr;
    args.distances = distances;
    args.vectors = vectors;
    args.distances_grad = distances_grad;
    args.vectors_grad = vectors_grad;
    args.n_pairs = n_pairs;
    args.n_points = n_points;
    args.points_grad = reinterpret_cast<double*>(points_grad);
    args.box_grad = reinterpret_cast<double*>(box_grad);
    args.bad_index = bad_index;

    if (n_points > 0xFFFFFFF0ull) {
        throw std::runtime_error("too many points: the GPU path indexes points with 32 bits");
    }
    const size_t wanted = (n_pairs + BACKWARD_ROWS_PER_BLOCK - 1) / BACKWARD_ROWS_PER_BLOCK;
    if (wanted > 0x7FFFFFFFull) {
        throw std::runtime_error("too many pairs for one launch");
    }
    const unsigned blocks = static_cast<unsigned>(wanted);
    hipStream_t stream = static_cast<hipStream_t>(caller_stream);
    hipLaunchKernelGGL(pairs_backward_kernel, dim3(blocks), dim3(BACKWARD_THREADS), 0, stream, args);
    HIP_CHECK(hipGetLastError());
    HIP_CHECK(hipStreamSynchronize(stream));
    if (*bad_index != 0) {
        throw std::runtime_error("`pairs` names a point beyond `n_points`");
    }
}

bool last_timings(const VesinNeighborList& neighbors, VesinHipTimings& timings) {
    const auto* extras = static_cast<const HipExtras*>(neighbors.opaque);
    if (extras == nullptr || !extras->timings_valid) {
        return false;
    }
    timings = extras->timings;
    return true;
}

} // namespace vesin_hip
