// Interface between the C ABI (api.cpp) and the HIP host driver (driver.hip).
#ifndef VESIN_HIP_DRIVER_HPP
#define VESIN_HIP_DRIVER_HPP

#include "vesin.h"

namespace vesin_hip {

/// Compute the list on GPU `neighbors.device.device_id`. All three input pointers are device memory.
/// Throws std::runtime_error / std::bad_alloc; never leaves HIP work in flight.
void neighbors(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinOptions options,
    VesinNeighborList& neighbors
);

/// Free the outputs and the private state of a GPU list (does not zero the struct).
void free_neighbors(VesinNeighborList& neighbors);

void enable_timings(bool enabled);
bool last_timings(const VesinNeighborList& neighbors, VesinHipTimings& timings);

} // namespace vesin_hip

#endif
