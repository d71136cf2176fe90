/* C ABI of the MI355X (gfx950) neighbor-list library.
 *
 * The two entry points, the three structs and the two enums below have the same names, field order, sizes and
 * meaning as the ones every vesin binding is written against (reference: vesin/include/vesin.h:36-46 enum
 * VesinAlgorithm, :49-78 VesinOptions, :81-89 VesinDeviceKind, :103-108 VesinDevice, :129-163 VesinNeighborList,
 * :167 vesin_free, :191-200 vesin_neighbors), so an existing caller relinks against this library unchanged.
 * A HIP device is addressed as `VesinCUDA`, which is what PyTorch-ROCm reports for its tensors.
 *
 * Layout on x86-64 (checked by tests/test_abi.py):
 *   VesinOptions       32 bytes: cutoff@0, full@8, sorted@9, algorithm@12, n_threads@16, return_shifts@20,
 *                                return_distances@21, return_vectors@22, skin@24
 *   VesinDevice         8 bytes: type@0, device_id@4
 *   VesinNeighborList  56 bytes: length@0, device@8, pairs@16, shifts@24, distances@32, vectors@40, opaque@48
 */
#ifndef VESIN_H
#define VESIN_H

#include <stddef.h>
#include <stdint.h>
#ifndef __cplusplus
    #include <stdbool.h>
#endif

#if defined(VESIN_SHARED) && (defined(__GNUC__) || defined(__clang__))
    #define VESIN_API __attribute__((visibility("default")))
#else
    #define VESIN_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* How candidate pairs are enumerated. The result does not depend on the choice. */
enum VesinAlgorithm {
    VesinAutoAlgorithm = 0, /* pick from the number of points and the box */
    VesinBruteForce = 1,    /* every point against every image of every point, tiled; for small systems */
    VesinCellList = 2,      /* counting sort into cells + stencil search, O(n) */
};

struct VesinOptions {
    double cutoff;             /* pairs with distance strictly below this are returned */
    bool full;                 /* true: i->j and j->i; false: each pair once */
    bool sorted;               /* true: pairs ordered by i (this library orders by (i, j, shift)) */
    enum VesinAlgorithm algorithm;
    int32_t n_threads;         /* CPU threads; must be >= 0; unused by the GPU path */
    bool return_shifts;        /* fill VesinNeighborList::shifts */
    bool return_distances;     /* fill VesinNeighborList::distances */
    bool return_vectors;       /* fill VesinNeighborList::vectors */
    double skin;               /* Verlet skin: > 0 keeps candidates at cutoff + skin between calls */
};

enum VesinDeviceKind {
    VesinUnknownDevice = 0, /* a zero-initialised list that owns nothing yet */
    VesinCPU = 1,
    VesinCUDA = 2,          /* a GPU; here: a HIP device */
};

struct VesinDevice {
    enum VesinDeviceKind type;
#ifdef __cplusplus
    int device_id = 0;      /* GPU ordinal; 0 for the CPU */
#else
    int device_id;
#endif
};

/* Output of one calculation. For pair k with points (i, j) and shift S, the vector is
 * r_j - r_i + S . box (box vectors as rows). All arrays live on `device` and belong to the library: they stay
 * valid until the next vesin_neighbors call on the same struct or vesin_free. */
struct VESIN_API VesinNeighborList {
#ifdef __cplusplus
    VesinNeighborList():
        length(0), device({VesinUnknownDevice, 0}), pairs(nullptr), shifts(nullptr), distances(nullptr),
        vectors(nullptr) {}
#endif
    size_t length;           /* number of pairs */
    struct VesinDevice device;
    size_t (*pairs)[2];      /* [length][2] */
    int32_t (*shifts)[3];    /* [length][3] when return_shifts, else NULL */
    double* distances;       /* [length]    when return_distances, else NULL */
    double (*vectors)[3];    /* [length][3] when return_vectors, else NULL */
#ifdef __cplusplus
    void* opaque = nullptr;  /* library-private state (device work buffers) */
#else
    void* opaque;
#endif
};

/* Release everything a list owns and zero the struct. NULL is accepted. (reference: vesin.h:167) */
void VESIN_API vesin_free(struct VesinNeighborList* neighbors);

/* Compute the neighbor list of `n_points` points. (reference: vesin.h:191-200)
 *
 * With device.type == VesinCUDA, `points` ([n_points][3] doubles), `box` (3 box vectors as rows) and `periodic`
 * (3 one-byte booleans) must be device memory of GPU `device.device_id`. `neighbors` must be zero-initialised
 * before its first use and may be reused across calls. Work is issued on the null stream and the call returns
 * after it completed. Returns EXIT_SUCCESS, or EXIT_FAILURE with *error_message pointing to a string owned by the
 * library (left untouched on success). This library has no CPU engine: VesinCPU is refused with an error. */
int VESIN_API vesin_neighbors(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    struct VesinDevice device,
    struct VesinOptions options,
    struct VesinNeighborList* neighbors,
    const char** error_message
);

/* ---- additions of this library (no counterpart in the reference) ------------------------------------------ */

/* Wall-clock breakdown of the most recent successful GPU call made through `neighbors`, measured with HIP events
 * on the stream the kernels ran on. Recording is off until vesin_hip_enable_timings(1) was called (it adds event
 * records to every call). Times are in milliseconds; stages that did not run report 0. */
struct VesinHipTimings {
    float total;        /* first launch to last kernel end */
    float cell_build;   /* bounding box, cell assignment, cell scan, scatter, gather */
    float count;        /* search, counting pass */
    float scan;         /* device-wide scan of the per-wave counts */
    float write;        /* search, writing pass: the kernel that produces the output arrays */
    float sort;         /* radix sort of (i, j, shift) and payload gather */
    uint64_t candidates;/* reserved, 0 */
};

/* vesin_neighbors on a stream of the caller's: the work is issued on `stream` (a hipStream_t of GPU
 * `device.device_id`, passed as void*; NULL is the null stream) and the call returns once that stream has
 * completed it, so the outputs and `length` are final on return. The kernels are ordered after whatever the
 * caller queued on `stream` before (no synchronisation is needed to hand over inputs produced there) and other
 * streams of the device are neither waited for nor held up, as they are by work on the null stream. A list must
 * not be used by two calls at once. The first call of a list and calls whose rows outgrow its arrays allocate
 * device memory, which synchronises the device. */
int VESIN_API vesin_hip_neighbors_on_stream(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    struct VesinDevice device,
    struct VesinOptions options,
    struct VesinNeighborList* neighbors,
    void* stream,
    const char** error_message
);

/* vesin_hip_neighbors_on_stream in two halves, for callers that want to queue more work behind the list without
 * the host waiting in between (a molecular dynamics step that evaluates forces from the list on the same stream).
 * The syncs this takes out of the caller's way are the reference's own (vesin/src/vesin_cuda.cpp:793-803, :899: every
 * call there ends with a device synchronisation); there is no counterpart of the two entry points in the reference.
 *
 * vesin_hip_neighbors_enqueue does everything a call can do before it needs an answer from the GPU, and returns.
 * For a list in its steady state (same number of points, cutoff and options as the call before, a box that did not
 * change, arrays that hold the rows) that is the whole calculation: cell list, search and rows are queued on
 * `stream`, into the arrays `neighbors` already has, whose addresses do not change before vesin_hip_neighbors_collect.
 * Otherwise (first call of a list, another box, another system) only the first kernels are queued and the rest is
 * done by vesin_hip_neighbors_collect; the call may then also block, as every call that has to allocate does.
 *
 *   device_length   receives the address of a 64-bit word in the memory of the GPU (the same for every call on this
 *                   list): work queued on `stream` after this call finds there the number of rows when the queued
 *                   kernels left the complete list in the arrays, and VESIN_HIP_ROWS_PENDING when they did not
 *                   (then nothing may be read from the arrays before vesin_hip_neighbors_collect has returned)
 *
 * vesin_hip_neighbors_collect waits for the kernels of the queued call (not for what was queued behind them),
 * looks at what they found and, if the list is not complete yet, completes it as vesin_hip_neighbors_on_stream
 * would have (growing the arrays, the general search), on the stream of the queued call. On return `length` and
 * the arrays are final, the device word holds `length`, and errors of the calculation are reported here, with the
 * usual message ownership. Any host thread may call it.
 *
 * Between the two calls the inputs (`points`, `box`, `periodic`) must stay as they are, `neighbors` must not be
 * passed to any other entry point (they refuse it; vesin_free completes the queued call first), and the values in
 * the struct are those of the call before. With options.skin > 0 a call that only filters the kept candidates is
 * queued whole (the word says pending when a point or the box turned out to have moved too far; collect then
 * computes the candidates again). */
#define VESIN_HIP_ROWS_PENDING (~0ull)

int VESIN_API vesin_hip_neighbors_enqueue(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    struct VesinDevice device,
    struct VesinOptions options,
    struct VesinNeighborList* neighbors,
    void* stream,
    const unsigned long long** device_length,
    const char** error_message
);

int VESIN_API vesin_hip_neighbors_collect(struct VesinNeighborList* neighbors, const char** error_message);

/* vesin_hip_neighbors_on_stream for callers that cannot allocate device memory (loops that must not reach
 * hipMalloc, harnesses that forbid it): no counterpart in the reference. The rows go to arrays of the caller's and
 * the call allocates and frees nothing, on the device or through any library.
 *
 *   pairs, shifts, distances, vectors   device memory of GPU `device.device_id` with room for `capacity` rows each
 *                ([capacity][2] size_t, [capacity][3] int32_t, [capacity] double, [capacity][3] double); the
 *                arrays `options` does not request may be NULL and are not touched
 *   length       host, filled on success with the number of rows written
 *   stream       a hipStream_t as void*, NULL for the null stream; the work has completed on return
 *
 * Everything else is as for vesin_neighbors (same rows, same checks and messages). The work memory is one array of
 * 64 MiB that every GPU holds from the moment the library is loaded, which sets the limits: at most 262144 points,
 * and cell lists and tables that fit (unsorted lists of that many points at usual densities do; `sorted` lists of
 * sparse or very uneven systems may not). A system beyond these limits, a non-zero `skin`, or a list of more than
 * `capacity` rows fail with EXIT_FAILURE and a message saying which; when the rows did not fit, *length receives
 * the number of rows the list has, so that the caller can come back with larger arrays. Calls on one GPU share the
 * work memory: they take turns (a lock is held for the whole call), whatever their streams.
 *
 * The first call on a GPU is set-up: it asks the HIP runtime for the address of the work array on that GPU
 * (hipGetSymbolAddress) and launches every kernel for the first time, and the runtime loads the library's code on
 * that GPU then, which it may allocate memory for. Make one call per GPU where allocating is still allowed (outside
 * of a graph capture, before the loop starts); from the second call on nothing is allocated or freed: the library's
 * own state per GPU is static data, what the kernels report comes to the host in copies of a few hundred bytes, and
 * the device memory in use before and after a series of calls is the same (tests/test_zz_no_alloc.py). */
int VESIN_API vesin_hip_neighbors_no_alloc(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    struct VesinDevice device,
    struct VesinOptions options,
    size_t (*pairs)[2],
    int32_t (*shifts)[3],
    double* distances,
    double (*vectors)[3],
    size_t capacity,
    size_t* length,
    void* stream,
    const char** error_message
);

/* Neighbor lists of many systems that share the options, computed by one sequence of launches (thousands of small
 * systems cost about as much as one large one with as many points, instead of thousands of calls). Per system the
 * rows are exactly those of vesin_neighbors on that system alone; only the order of an unsorted list may differ.
 *
 *   points       device: the points of all systems, one system after the other
 *   first_point  host, n_systems + 1 entries: first_point[s] is the index in `points` of the first point of system
 *                s, first_point[n_systems] the total number of points
 *   boxes        device: n_systems boxes (3x3 each, rows = box vectors)
 *   periodic     device: n_systems x 3 flags, per system and direction (a free molecule has none set and its box
 *                is not read, like in vesin_neighbors)
 *   neighbors    receives all rows, system after system; the indices in `pairs` count from the first point of the
 *                row's system. Same ownership rules as for vesin_neighbors; the same struct may be used with both.
 *   first_pair   host, n_systems + 1 entries, filled on success: rows [first_pair[s], first_pair[s + 1]) belong to
 *                system s
 *
 * With options.sorted every system's rows are ordered as vesin_neighbors orders them for that system alone (by
 * (i, j, shift)). With options.skin > 0 the list keeps candidates at cutoff + skin for the whole batch and later
 * calls with the same division into systems filter them while no point of any system has moved further than the
 * skin allows (per system, as vesin_neighbors decides it); the rows are always those of skin = 0. Returns EXIT_SUCCESS / EXIT_FAILURE like vesin_neighbors, with the same
 * message ownership. */
int VESIN_API vesin_hip_neighbors_batch(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    struct VesinDevice device,
    struct VesinOptions options,
    struct VesinNeighborList* neighbors,
    size_t* first_pair,
    const char** error_message
);

/* vesin_hip_neighbors_batch with its GPU work (kernels and the small copies to and from the host) on the HIP
 * stream `stream` (a hipStream_t; NULL is the null stream) of the list's device, like
 * vesin_hip_neighbors_on_stream: everything queued on that stream before the call is seen, the results are complete
 * on return, other streams are neither waited for nor held up. No counterpart in the reference. */
int VESIN_API vesin_hip_neighbors_batch_on_stream(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    struct VesinDevice device,
    struct VesinOptions options,
    struct VesinNeighborList* neighbors,
    size_t* first_pair,
    void* stream,
    const char** error_message
);

/* vesin_hip_neighbors_batch_on_stream in two halves, like vesin_hip_neighbors_enqueue: everything the batch can do
 * before the host needs an answer from the GPU is queued on `stream` (for a list that saw the same division into
 * systems before: the whole calculation), and the call returns; vesin_hip_neighbors_collect on the same list
 * completes it (waits for the queued kernels, starts over with what they reported when the boxes or the systems were
 * not those of the call before, grows the arrays) and reports its errors. No counterpart in the reference.
 * Between the two calls `points`, `boxes`, `periodic` and the host array `first_point` must stay as they are;
 * `first_pair` (host) is written by vesin_hip_neighbors_collect; the list is refused by every other entry point.
 * As for a single system, work queued on `stream` behind this call finds the number of rows in the word at
 * `*device_length` when the queued kernels left the complete list in the arrays: a batch with the division into
 * systems, the boxes and the options of the call before, unsorted and without a skin (free molecules of up to 64
 * points each also with other molecules in every call, sorted or not). In every other case the word says
 * VESIN_HIP_ROWS_PENDING until vesin_hip_neighbors_collect has set it to `length`.
 *
 * vesin_hip_batch_first_pair_on_device returns where the kernels of the last batch on the list (queued or not) left
 * the first row of every system: n_systems + 1 64-bit words in the memory of the GPU, the last one the number of
 * rows; what `first_pair` receives on the host, for work on the GPU that goes through the rows system by system.
 * Valid when the device word of a queued batch holds a number of rows, or after the batch has returned or was
 * collected, until the next call on the list. NULL when the last call was no batch or had no points, and while a
 * queued batch has not got as far as its kernels (then the device word says pending, too). */
int VESIN_API vesin_hip_neighbors_batch_enqueue(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    struct VesinDevice device,
    struct VesinOptions options,
    struct VesinNeighborList* neighbors,
    size_t* first_pair,
    void* stream,
    const unsigned long long** device_length,
    const char** error_message
);

const unsigned long long* VESIN_API vesin_hip_batch_first_pair_on_device(const struct VesinNeighborList* neighbors);

/* Gradient of the pair geometry: given dE/d(distances) and dE/d(vectors) of some scalar E for the rows of a list,
 * ADD dE/d(points) and dE/d(box) to `points_grad` and `box_grad` (the caller zeroes them, or accumulates):
 *     g_k = vectors_grad[k] + distances_grad[k] * vectors[k] / distances[k]
 *     points_grad[j_k] += g_k;   points_grad[i_k] -= g_k;   box_grad[a][b] += shifts[k][a] * g_k[b]
 * This is what the reference's TorchScript class does with tensor operations in its backward step
 * (vesin-torch/src/vesin_torch.cpp:437-468); here it is one kernel. All arrays are device memory of GPU
 * `device.device_id`. `distances_grad` or `vectors_grad` may be NULL (taken as zero), `points_grad` or `box_grad`
 * may be NULL (not wanted); `shifts` is only read for `box_grad`, `distances` and `vectors` only for
 * `distances_grad`. Sums are accumulated with floating-point atomics: their last bits depend on the order of
 * arrival. Work is issued on `stream` (a hipStream_t as void*, NULL for the null stream) and the call returns
 * after it completed. */
int VESIN_API vesin_hip_pairs_backward(
    const size_t (*pairs)[2],
    const int32_t (*shifts)[3],
    const double* distances,
    const double (*vectors)[3],
    size_t n_pairs,
    const double* distances_grad,
    const double (*vectors_grad)[3],
    size_t n_points,
    struct VesinDevice device,
    double (*points_grad)[3],
    double (*box_grad)[3],
    void* stream,
    const char** error_message
);

/* Output arrays from the caller's allocator, and handing them over without a copy. No counterpart in the
 * reference, whose callers copy the rows out of the list's arrays when they want to keep them beyond the next
 * call (python/vesin/vesin/_neighbors.py:343-381 and :513-574, vesin-torch/src/vesin_torch.cpp:214-256): for a
 * list of a million points that copy takes as long as the search.
 *
 * vesin_hip_set_output_allocator makes `neighbors` take the memory of pairs / shifts / distances / vectors from
 * `allocate` and give it back through `release` (both called with `context`, with the list's GPU current, from
 * inside calls on this list and from vesin_free; `allocate` returns device memory of that GPU, usable on any of
 * its streams, or NULL when it has none). Arrays the list holds at that moment go back to where they came from.
 * NULL for both restores hipMalloc / hipFree. The list may be zeroed (no call yet): `device` is then the device it
 * will be used with.
 *
 * vesin_hip_detach_outputs makes the arrays `neighbors` points to the caller's: read the four pointers and `length`
 * from the struct first; afterwards they are NULL in the struct, the list will never touch or release that memory
 * again, and the caller releases every non-NULL array itself, the way `release` would (hipFree without an
 * allocator). `*capacity` (may be NULL) receives the rows each array has room for. The next call on the list
 * allocates arrays of that size again before it starts, so it runs as a call on a list that kept its arrays. Fails
 * while a call queued with vesin_hip_neighbors_enqueue is pending. */
typedef void* (*VesinHipAllocate)(size_t bytes, void* context);
typedef void (*VesinHipRelease)(void* pointer, void* context);

int VESIN_API vesin_hip_set_output_allocator(
    struct VesinNeighborList* neighbors,
    struct VesinDevice device,
    VesinHipAllocate allocate,
    VesinHipRelease release,
    void* context,
    const char** error_message
);

int VESIN_API vesin_hip_detach_outputs(struct VesinNeighborList* neighbors, size_t* capacity, const char** error_message);

/* Rows every output array of `neighbors` has room for (0 for a list without arrays): what a caller compares `length`
 * with before it takes arrays over that are much larger than their rows. */
size_t VESIN_API vesin_hip_output_capacity(const struct VesinNeighborList* neighbors);

void VESIN_API vesin_hip_enable_timings(int enabled);
int VESIN_API vesin_hip_last_timings(const struct VesinNeighborList* neighbors, struct VesinHipTimings* timings);

#ifdef __cplusplus
}
#endif

#endif
