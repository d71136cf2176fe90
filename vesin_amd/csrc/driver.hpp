// Interface between the C ABI (api.cpp) and the HIP host driver (driver.hip).
#ifndef VESIN_HIP_DRIVER_HPP
#define VESIN_HIP_DRIVER_HPP

#include "vesin.h"

namespace vesin_hip {

/// Compute the list on GPU `neighbors.device.device_id`. All three input pointers are device memory. The work is
/// issued on `stream` (a hipStream_t of that device; nullptr is the null stream) and has completed on return.
/// Throws std::runtime_error / std::bad_alloc; never leaves HIP work in flight.
void neighbors(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    void* stream
);

/// `neighbors` that comes back as soon as the host would have to wait for the GPU: what the call can decide without
/// an answer from the device is queued on `stream` by then, the rest happens in `neighbors_collect` (which any host
/// thread may call; the inputs must stay as they are until then). Returns the device word that receives the number
/// of rows once the queued kernels have run, or ~0 when they did not leave the complete list.
const unsigned long long* neighbors_enqueue(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    void* stream
);

/// Ends the call that `neighbors_enqueue` started on this list: waits for its kernels, and does whatever is left.
void neighbors_collect(VesinNeighborList& neighbors);

/// The lists of many systems in one sequence of launches. `points`, `boxes`, `periodic` are device
/// memory holding the systems one after the other; `first_point` (host, n_systems + 1 entries) says where each
/// system starts. Rows come out system after system with indices counted inside each system; `first_pair` (host,
/// n_systems + 1 entries) receives where each system's rows start.
void neighbors_batch(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    size_t* first_pair,
    void* stream
);

/// `neighbors_batch` that comes back as soon as the host would have to wait for the GPU, like `neighbors_enqueue`;
/// `neighbors_collect` ends it. `first_point` is read and `first_pair` written until then. The device word says that
/// the rows are pending until `neighbors_collect` has set it.
const unsigned long long* neighbors_batch_enqueue(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinOptions options,
    VesinNeighborList& neighbors,
    size_t* first_pair,
    void* stream
);

/// `neighbors` without any allocation: the rows go to the caller's arrays (device memory of GPU `device_id` holding
/// `capacity` rows each; the ones that `options` does not request are not touched), the work memory is a fixed
/// array every GPU holds while the library is loaded. Throws when the system or its list does not fit; `length` then
/// receives the number of rows when it was the output arrays that were too small. Calls on one GPU take turns.
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
    void* stream
);

/// Adds the gradient of a scalar with respect to points and box, given its gradient with respect to the distances
/// and vectors of the rows. All arrays are device memory of GPU `device_id`; `points_grad` ([n_points][3]) and
/// `box_grad` ([3][3]) are accumulated into. Runs on `stream` (nullptr: the null stream) and returns after the work
/// completed.
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
    void* stream
);

/// Free the outputs and the private state of a GPU list (does not zero the struct).
void free_neighbors(VesinNeighborList& neighbors);

/// The output arrays of this list come from `allocate` and go back through `release` from now on (NULL for both:
/// hipMalloc and hipFree); arrays the list holds are released the way they were allocated.
void set_output_allocator(VesinNeighborList& neighbors, VesinHipAllocate allocate, VesinHipRelease release, void* context);

/// The arrays the list points to become the caller's: the pointers are cleared, the rows they have room for returned;
/// the next call allocates arrays of that size again before it starts.
size_t detach_outputs(VesinNeighborList& neighbors);

/// Where the kernels of the last batch on this list left the first row of every system (n_systems + 1 words in
/// device memory, the last one the number of rows); nullptr when the last call was no batch or had no points.
const unsigned long long* batch_first_pair_on_device(const VesinNeighborList& neighbors);

/// Rows the output arrays of the list have room for.
size_t output_capacity(const VesinNeighborList& neighbors);

void enable_timings(bool enabled);
bool last_timings(const VesinNeighborList& neighbors, VesinHipTimings& timings);

} // namespace vesin_hip

#endif
