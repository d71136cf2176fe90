// The C ABI: argument validation, error-string ownership and dispatch to the HIP driver.
//
// Checks, their order and their texts are those of the reference's entry point (vesin/src/vesin.cpp:51-105), and
// exceptions are turned into EXIT_FAILURE + message the same way (vesin/src/vesin.cpp:139-150). The difference is
// the dispatch: a GPU device runs the HIP path, and VesinCPU is refused because this library ships no CPU engine.
#include <cmath>
#include <cstdlib>
#include <cstring>

#include <iostream>
#include <stdexcept>
#include <string>

#include "driver.hpp"
#include "vesin.h"

// storage for messages built at run time; the caller only ever sees a pointer into it
static thread_local std::string LAST_ERROR;

static int fail(const char** error_message, const char* text) {
    *error_message = text;
    return EXIT_FAILURE;
}

/// vesin_neighbors and its variants on a stream. `device_length` not null: the call is queued only (see
/// vesin_hip_neighbors_enqueue) and the address of its device word goes there.
static int neighbors_on(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    void* stream,
    const char** error_message,
    const unsigned long long** device_length = nullptr
) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (points == nullptr) {
        return fail(error_message, "`points` can not be a NULL pointer");
    }
    if (box == nullptr) {
        return fail(error_message, "`cell` can not be a NULL pointer");
    }
    if (neighbors == nullptr) {
        return fail(error_message, "`neighbors` can not be a NULL pointer");
    }
    if (!std::isfinite(options.cutoff) || options.cutoff <= 0) {
        return fail(error_message, "cutoff must be a finite, positive number");
    }
    if (options.cutoff <= 1e-6) {
        return fail(error_message, "cutoff is too small");
    }
    if (!std::isfinite(options.skin) || options.skin < 0.0) {
        // the reference sets this message without returning (vesin/src/vesin.cpp:80-82) and goes on with the
        // unusable value; here it is an error
        return fail(error_message, "skin must be a finite, non-negative number");
    }
    if (options.n_threads < 0) {
        return fail(error_message, "n_threads must be zero or a positive integer");
    }
    if (neighbors->device.type != VesinUnknownDevice && neighbors->device.type != device.type) {
        return fail(error_message, "`neighbors` device and data `device` do not match, free the neighbors first");
    }
    if (device.type == VesinUnknownDevice) {
        return fail(error_message, "got an unknown device type");
    }

    try {
        if (device.type == VesinCUDA) {
            if (periodic == nullptr) {
                throw std::runtime_error("`periodic` can not be a NULL pointer");
            }
            if (neighbors->device.type == VesinUnknownDevice) {
                neighbors->device = device;
            }
            if (device_length != nullptr) {
                *device_length = vesin_hip::neighbors_enqueue(points, n_points, box, periodic, options, *neighbors, stream);
            } else {
                vesin_hip::neighbors(points, n_points, box, periodic, options, *neighbors, stream);
            }
        } else if (device.type == VesinCPU) {
            throw std::runtime_error(
                "this library only implements GPU devices (VesinCUDA, i.e. HIP on ROCm); there is no CPU engine in it"
            );
        } else {
            throw std::runtime_error("unknown device " + std::to_string(device.type));
        }
    } catch (const std::bad_alloc&) {
        LAST_ERROR = "failed to allocate memory";
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (const std::exception& e) {
        LAST_ERROR = e.what();
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (...) {
        return fail(error_message, "fatal error: unknown type thrown as exception");
    }
    return EXIT_SUCCESS;
}

extern "C" int vesin_neighbors(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    const char** error_message
) {
    return neighbors_on(points, n_points, box, periodic, device, options, neighbors, nullptr, error_message);
}

extern "C" int vesin_hip_neighbors_on_stream(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    void* stream,
    const char** error_message
) {
    return neighbors_on(points, n_points, box, periodic, device, options, neighbors, stream, error_message);
}

extern "C" int vesin_hip_neighbors_enqueue(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    void* stream,
    const unsigned long long** device_length,
    const char** error_message
) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (device_length == nullptr) {
        return fail(error_message, "`device_length` can not be a NULL pointer");
    }
    if (device.type != VesinCUDA) {
        return fail(error_message, "a calculation is only queued on a GPU device (VesinCUDA, i.e. HIP on ROCm)");
    }
    return neighbors_on(points, n_points, box, periodic, device, options, neighbors, stream, error_message, device_length);
}

extern "C" int vesin_hip_neighbors_collect(VesinNeighborList* neighbors, const char** error_message) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (neighbors == nullptr) {
        return fail(error_message, "`neighbors` can not be a NULL pointer");
    }
    if (neighbors->device.type != VesinCUDA) {
        return fail(error_message, "no calculation was queued on this list");
    }
    try {
        vesin_hip::neighbors_collect(*neighbors);
    } catch (const std::bad_alloc&) {
        LAST_ERROR = "failed to allocate memory";
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (const std::exception& e) {
        LAST_ERROR = e.what();
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (...) {
        return fail(error_message, "fatal error: unknown type thrown as exception");
    }
    return EXIT_SUCCESS;
}

extern "C" int vesin_hip_neighbors_no_alloc(
    const double (*points)[3],
    size_t n_points,
    const double box[3][3],
    const bool periodic[3],
    VesinDevice device,
    VesinOptions options,
    size_t (*pairs)[2],
    int32_t (*shifts)[3],
    double* distances,
    double (*vectors)[3],
    size_t capacity,
    size_t* length,
    void* stream,
    const char** error_message
) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (points == nullptr) {
        return fail(error_message, "`points` can not be a NULL pointer");
    }
    if (box == nullptr) {
        return fail(error_message, "`cell` can not be a NULL pointer");
    }
    if (periodic == nullptr) {
        return fail(error_message, "`periodic` can not be a NULL pointer");
    }
    if (length == nullptr) {
        return fail(error_message, "`length` can not be a NULL pointer");
    }
    if (!std::isfinite(options.cutoff) || options.cutoff <= 0) {
        return fail(error_message, "cutoff must be a finite, positive number");
    }
    if (options.cutoff <= 1e-6) {
        return fail(error_message, "cutoff is too small");
    }
    if (!std::isfinite(options.skin) || options.skin < 0.0) {
        return fail(error_message, "skin must be a finite, non-negative number");
    }
    if (options.n_threads < 0) {
        return fail(error_message, "n_threads must be zero or a positive integer");
    }
    if (device.type != VesinCUDA) {
        return fail(error_message, "this entry point only computes on a GPU device (VesinCUDA, i.e. HIP on ROCm)");
    }
    try {
        vesin_hip::neighbors_no_alloc(
            points, n_points, box, periodic, options, device.device_id, pairs, shifts, distances, vectors, capacity,
            *length, stream
        );
    } catch (const std::bad_alloc&) {
        LAST_ERROR = "failed to allocate memory";
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (const std::exception& e) {
        LAST_ERROR = e.what();
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (...) {
        return fail(error_message, "fatal error: unknown type thrown as exception");
    }
    return EXIT_SUCCESS;
}

static int neighbors_batch_on(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    size_t* first_pair,
    void* stream,
    const char** error_message,
    const unsigned long long** device_length = nullptr
) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (first_point == nullptr) {
        return fail(error_message, "`first_point` can not be a NULL pointer");
    }
    if (first_pair == nullptr) {
        return fail(error_message, "`first_pair` can not be a NULL pointer");
    }
    if (boxes == nullptr) {
        return fail(error_message, "`cell` can not be a NULL pointer");
    }
    if (periodic == nullptr) {
        return fail(error_message, "`periodic` can not be a NULL pointer");
    }
    if (neighbors == nullptr) {
        return fail(error_message, "`neighbors` can not be a NULL pointer");
    }
    if (n_systems > 0 && points == nullptr && first_point[n_systems] > 0) {
        return fail(error_message, "`points` can not be a NULL pointer");
    }
    if (!std::isfinite(options.cutoff) || options.cutoff <= 0) {
        return fail(error_message, "cutoff must be a finite, positive number");
    }
    if (options.cutoff <= 1e-6) {
        return fail(error_message, "cutoff is too small");
    }
    if (!std::isfinite(options.skin) || options.skin < 0.0) {
        return fail(error_message, "skin must be a finite, non-negative number");
    }
    if (options.n_threads < 0) {
        return fail(error_message, "n_threads must be zero or a positive integer");
    }
    if (device.type != VesinCUDA) {
        return fail(error_message, "a batch of systems is only computed on a GPU device (VesinCUDA, i.e. HIP on ROCm)");
    }
    if (neighbors->device.type != VesinUnknownDevice && neighbors->device.type != device.type) {
        return fail(error_message, "`neighbors` device and data `device` do not match, free the neighbors first");
    }

    try {
        if (neighbors->device.type == VesinUnknownDevice) {
            neighbors->device = device;
        }
        if (device_length != nullptr) {
            *device_length = vesin_hip::neighbors_batch_enqueue(
                points, first_point, n_systems, boxes, periodic, options, *neighbors, first_pair, stream
            );
        } else {
            vesin_hip::neighbors_batch(points, first_point, n_systems, boxes, periodic, options, *neighbors, first_pair, stream);
        }
    } catch (const std::bad_alloc&) {
        LAST_ERROR = "failed to allocate memory";
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (const std::exception& e) {
        LAST_ERROR = e.what();
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (...) {
        return fail(error_message, "fatal error: unknown type thrown as exception");
    }
    return EXIT_SUCCESS;
}

extern "C" int vesin_hip_neighbors_batch(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    size_t* first_pair,
    const char** error_message
) {
    return neighbors_batch_on(
        points, first_point, n_systems, boxes, periodic, device, options, neighbors, first_pair, nullptr, error_message
    );
}

extern "C" int vesin_hip_neighbors_batch_on_stream(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    size_t* first_pair,
    void* stream,
    const char** error_message
) {
    return neighbors_batch_on(
        points, first_point, n_systems, boxes, periodic, device, options, neighbors, first_pair, stream, error_message
    );
}

extern "C" int vesin_hip_neighbors_batch_enqueue(
    const double (*points)[3],
    const size_t* first_point,
    size_t n_systems,
    const double (*boxes)[3][3],
    const bool (*periodic)[3],
    VesinDevice device,
    VesinOptions options,
    VesinNeighborList* neighbors,
    size_t* first_pair,
    void* stream,
    const unsigned long long** device_length,
    const char** error_message
) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (device_length == nullptr) {
        return fail(error_message, "`device_length` can not be a NULL pointer");
    }
    return neighbors_batch_on(
        points, first_point, n_systems, boxes, periodic, device, options, neighbors, first_pair, stream, error_message,
        device_length
    );
}

extern "C" int vesin_hip_pairs_backward(
    const size_t (*pairs)[2],
    const int32_t (*shifts)[3],
    const double* distances,
    const double (*vectors)[3],
    size_t n_pairs,
    const double* distances_grad,
    const double (*vectors_grad)[3],
    size_t n_points,
    VesinDevice device,
    double (*points_grad)[3],
    double (*box_grad)[3],
    void* stream,
    const char** error_message
) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (device.type != VesinCUDA) {
        return fail(error_message, "the gradient is only computed on a GPU device (VesinCUDA, i.e. HIP on ROCm)");
    }
    try {
        vesin_hip::pairs_backward(
            pairs, shifts, distances, vectors, n_pairs, distances_grad, vectors_grad, n_points, device.device_id,
            points_grad, box_grad, stream
        );
    } catch (const std::bad_alloc&) {
        LAST_ERROR = "failed to allocate memory";
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (const std::exception& e) {
        LAST_ERROR = e.what();
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (...) {
        return fail(error_message, "fatal error: unknown type thrown as exception");
    }
    return EXIT_SUCCESS;
}

extern "C" void vesin_free(VesinNeighborList* neighbors) {
    if (neighbors == nullptr) {
        return;
    }
    try {
        if (neighbors->device.type == VesinCUDA) {
            vesin_hip::free_neighbors(*neighbors);
        } else if (neighbors->device.type != VesinUnknownDevice) {
            throw std::runtime_error(
                "device " + std::to_string(neighbors->device.type) + " is not one this library allocates on"
            );
        }
    } catch (const std::exception& e) {
        std::cerr << "error in vesin_free: " << e.what() << std::endl;
        return;
    } catch (...) {
        std::cerr << "fatal error in vesin_free, unknown type thrown as exception" << std::endl;
        return;
    }
    std::memset(static_cast<void*>(neighbors), 0, sizeof(VesinNeighborList));
}

extern "C" int vesin_hip_set_output_allocator(
    VesinNeighborList* neighbors,
    VesinDevice device,
    VesinHipAllocate allocate,
    VesinHipRelease release,
    void* context,
    const char** error_message
) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (neighbors == nullptr) {
        return fail(error_message, "`neighbors` can not be a NULL pointer");
    }
    if (device.type != VesinCUDA) {
        return fail(error_message, "output arrays are only allocated for a GPU device (VesinCUDA, i.e. HIP on ROCm)");
    }
    if (neighbors->device.type != VesinUnknownDevice &&
        (neighbors->device.type != device.type || neighbors->device.device_id != device.device_id)) {
        return fail(error_message, "`neighbors` device and data `device` do not match, free the neighbors first");
    }
    try {
        const bool fresh = neighbors->device.type == VesinUnknownDevice;
        neighbors->device = device;
        try {
            vesin_hip::set_output_allocator(*neighbors, allocate, release, context);
        } catch (...) {
            if (fresh && neighbors->opaque == nullptr) {
                neighbors->device.type = VesinUnknownDevice;
                neighbors->device.device_id = 0;
            }
            throw;
        }
    } catch (const std::bad_alloc&) {
        LAST_ERROR = "failed to allocate memory";
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (const std::exception& e) {
        LAST_ERROR = e.what();
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (...) {
        return fail(error_message, "fatal error: unknown type thrown as exception");
    }
    return EXIT_SUCCESS;
}

extern "C" int vesin_hip_detach_outputs(VesinNeighborList* neighbors, size_t* capacity, const char** error_message) {
    if (error_message == nullptr) {
        return EXIT_FAILURE;
    }
    if (neighbors == nullptr) {
        return fail(error_message, "`neighbors` can not be a NULL pointer");
    }
    if (neighbors->device.type != VesinCUDA && neighbors->device.type != VesinUnknownDevice) {
        return fail(error_message, "the arrays of this list are not this library's");
    }
    try {
        const size_t rows = vesin_hip::detach_outputs(*neighbors);
        if (capacity != nullptr) {
            *capacity = rows;
        }
    } catch (const std::exception& e) {
        LAST_ERROR = e.what();
        *error_message = LAST_ERROR.c_str();
        return EXIT_FAILURE;
    } catch (...) {
        return fail(error_message, "fatal error: unknown type thrown as exception");
    }
    return EXIT_SUCCESS;
}

extern "C" const unsigned long long* vesin_hip_batch_first_pair_on_device(const VesinNeighborList* neighbors) {
    if (neighbors == nullptr || neighbors->device.type != VesinCUDA) {
        return nullptr;
    }
    return vesin_hip::batch_first_pair_on_device(*neighbors);
}

extern "C" size_t vesin_hip_output_capacity(const VesinNeighborList* neighbors) {
    if (neighbors == nullptr || neighbors->device.type != VesinCUDA) {
        return 0;
    }
    return vesin_hip::output_capacity(*neighbors);
}

extern "C" void vesin_hip_enable_timings(int enabled) {
    vesin_hip::enable_timings(enabled != 0);
}

extern "C" int vesin_hip_last_timings(const VesinNeighborList* neighbors, VesinHipTimings* timings) {
    if (neighbors == nullptr || timings == nullptr || neighbors->device.type != VesinCUDA) {
        return EXIT_FAILURE;
    }
    return vesin_hip::last_timings(*neighbors, *timings) ? EXIT_SUCCESS : EXIT_FAILURE;
}
