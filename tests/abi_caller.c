/* A compiled C caller of the library, the way a C user of vesin links it: `#include "vesin.h"`, -lvesin, the HIP
 * runtime for the device buffers. It plays the cases of the reference's own GPU test program
 * (vesin/tests/cuda.cpp:22-126 the three-point list with exact values, :141-157 ten host threads at once,
 * :160-226 two calls with a Verlet skin) and a few of vesin/tests/neighbors.cpp's error checks, through
 * vesin_neighbors / vesin_free only. Built and run by tests/test_gpu_c_caller.py; prints "ok" and returns 0 when
 * every check held, else prints what failed. */
#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "vesin.h"

static int failures = 0;
static pthread_mutex_t failures_lock = PTHREAD_MUTEX_INITIALIZER;

#define CHECK(condition)                                                                                             \
    do {                                                                                                             \
        if (!(condition)) {                                                                                          \
            pthread_mutex_lock(&failures_lock);                                                                      \
            failures += 1;                                                                                           \
            fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #condition);                            \
            pthread_mutex_unlock(&failures_lock);                                                                    \
        }                                                                                                            \
    } while (0)

#define HIP(call)                                                                                                    \
    do {                                                                                                             \
        hipError_t status_ = (call);                                                                                 \
        if (status_ != hipSuccess) {                                                                                 \
            fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(status_));               \
            exit(2);                                                                                                 \
        }                                                                                                            \
    } while (0)

static void* to_device(const void* host, size_t bytes) {
    void* device = NULL;
    HIP(hipMalloc(&device, bytes));
    HIP(hipMemcpy(device, host, bytes, hipMemcpyHostToDevice));
    return device;
}

static struct VesinOptions default_options(double cutoff) {
    struct VesinOptions options;
    memset(&options, 0, sizeof(options));
    options.cutoff = cutoff;
    options.algorithm = VesinAutoAlgorithm;
    return options;
}

/* Three points on the diagonal of a box with face-centred vectors: five half-list pairs, three of them between
 * points 0 and 2 through three different images. Distances and vectors are exact in binary. */
static void* three_points(void* argument) {
    const int device_id = *(const int*)argument;
    HIP(hipSetDevice(device_id));

    const double points[3][3] = {{0.0, 0.0, 0.0}, {1.0, 1.0, 1.0}, {2.0, 2.0, 2.0}};
    const double box[3][3] = {{0.0, 3.0, 3.0}, {3.0, 0.0, 3.0}, {3.0, 3.0, 0.0}};
    const bool periodic[3] = {true, true, true};
    double (*d_points)[3] = to_device(points, sizeof(points));
    double (*d_box)[3] = to_device(box, sizeof(box));
    bool* d_periodic = to_device(periodic, sizeof(periodic));

    struct VesinNeighborList neighbors;
    memset(&neighbors, 0, sizeof(neighbors));
    struct VesinOptions options = default_options(3.0);
    options.full = false;
    options.return_shifts = true;
    options.return_distances = true;
    options.return_vectors = true;
    const struct VesinDevice device = {VesinCUDA, device_id};

    /* a list is used twice: its second call takes the path of a list that has arrays */
    for (int call = 0; call < 2; call++) {
        const char* error_message = NULL;
        const int status = vesin_neighbors(
            (const double (*)[3])d_points, 3, (const double (*)[3])d_box, d_periodic, device, options, &neighbors,
            &error_message
        );
        CHECK(error_message == NULL);
        CHECK(status == EXIT_SUCCESS);
        CHECK(neighbors.length == 5);
        CHECK(neighbors.pairs != NULL && neighbors.shifts != NULL && neighbors.distances != NULL && neighbors.vectors != NULL);
        if (status != EXIT_SUCCESS || neighbors.length != 5) {
            break;
        }

        size_t pairs[5][2];
        int32_t shifts[5][3];
        double distances[5];
        double vectors[5][3];
        HIP(hipMemcpy(pairs, neighbors.pairs, sizeof(pairs), hipMemcpyDeviceToHost));
        HIP(hipMemcpy(shifts, neighbors.shifts, sizeof(shifts), hipMemcpyDeviceToHost));
        HIP(hipMemcpy(distances, neighbors.distances, sizeof(distances), hipMemcpyDeviceToHost));
        HIP(hipMemcpy(vectors, neighbors.vectors, sizeof(vectors), hipMemcpyDeviceToHost));

        int images_of_0_2 = 0;
        for (size_t k = 0; k < 5; k++) {
            if (pairs[k][0] == 0 && pairs[k][1] == 2) {
                CHECK(distances[k] == sqrt(6.0));
                const int32_t* s = shifts[k];
                const double* v = vectors[k];
                if (s[0] == -1 && s[1] == 0 && s[2] == 0) {
                    CHECK(v[0] == 2.0 && v[1] == -1.0 && v[2] == -1.0);
                    images_of_0_2 |= 1;
                } else if (s[0] == 0 && s[1] == -1 && s[2] == 0) {
                    CHECK(v[0] == -1.0 && v[1] == 2.0 && v[2] == -1.0);
                    images_of_0_2 |= 2;
                } else if (s[0] == 0 && s[1] == 0 && s[2] == -1) {
                    CHECK(v[0] == -1.0 && v[1] == -1.0 && v[2] == 2.0);
                    images_of_0_2 |= 4;
                } else {
                    CHECK(!"unexpected shift for the pair (0, 2)");
                }
            } else if ((pairs[k][0] == 0 && pairs[k][1] == 1) || (pairs[k][0] == 1 && pairs[k][1] == 2)) {
                CHECK(shifts[k][0] == 0 && shifts[k][1] == 0 && shifts[k][2] == 0);
                CHECK(distances[k] == sqrt(3.0));
                CHECK(vectors[k][0] == 1.0 && vectors[k][1] == 1.0 && vectors[k][2] == 1.0);
            } else {
                CHECK(!"unexpected pair");
            }
        }
        CHECK(images_of_0_2 == 7);
    }

    vesin_free(&neighbors);
    CHECK(neighbors.pairs == NULL && neighbors.length == 0 && neighbors.opaque == NULL);
    HIP(hipFree(d_points));
    HIP(hipFree(d_box));
    HIP(hipFree(d_periodic));
    return NULL;
}

/* Two calls with a skin, the points of the second slightly moved: the cached candidates are filtered. The rows must
 * be those of a plain calculation on the moved points. */
static void verlet_skin(int device_id) {
    HIP(hipSetDevice(device_id));
    const double points[4][3] = {{0.0, 0.0, 0.0}, {1.0, 1.0, 1.0}, {2.0, 2.0, 2.0}, {4.0, 1.0, 0.0}};
    const double moved[4][3] = {{0.01, 0.01, 0.01}, {1.02, 1.01, 0.99}, {2.00, 2.03, 1.98}, {4.01, 1.02, 0.01}};
    const double box[3][3] = {{10.0, 0.0, 0.0}, {0.0, 10.0, 0.0}, {0.0, 0.0, 10.0}};
    const bool periodic[3] = {true, true, true};
    double (*d_points)[3] = to_device(points, sizeof(points));
    double (*d_box)[3] = to_device(box, sizeof(box));
    bool* d_periodic = to_device(periodic, sizeof(periodic));
    const struct VesinDevice device = {VesinCUDA, device_id};

    struct VesinNeighborList cached;
    struct VesinNeighborList plain;
    memset(&cached, 0, sizeof(cached));
    memset(&plain, 0, sizeof(plain));
    struct VesinOptions options = default_options(2.5);
    options.full = true;
    options.sorted = true;
    options.return_shifts = true;
    options.return_distances = true;
    options.skin = 0.8;
    const char* error_message = NULL;
    int status = vesin_neighbors(
        (const double (*)[3])d_points, 4, (const double (*)[3])d_box, d_periodic, device, options, &cached, &error_message
    );
    CHECK(status == EXIT_SUCCESS && error_message == NULL);
    HIP(hipMemcpy(d_points, moved, sizeof(moved), hipMemcpyHostToDevice));
    status = vesin_neighbors(
        (const double (*)[3])d_points, 4, (const double (*)[3])d_box, d_periodic, device, options, &cached, &error_message
    );
    CHECK(status == EXIT_SUCCESS && error_message == NULL);

    options.skin = 0.0;
    status = vesin_neighbors(
        (const double (*)[3])d_points, 4, (const double (*)[3])d_box, d_periodic, device, options, &plain, &error_message
    );
    CHECK(status == EXIT_SUCCESS && error_message == NULL);
    CHECK(cached.length == plain.length);
    /* only 0-1 and 1-2 (both 1.73 apart) are within 2.5: four rows of a full list */
    CHECK(plain.length == 4);
    if (cached.length == plain.length && plain.length <= 16) {
        size_t a[16][2], b[16][2];
        double da[16], db[16];
        HIP(hipMemcpy(a, cached.pairs, plain.length * sizeof(a[0]), hipMemcpyDeviceToHost));
        HIP(hipMemcpy(b, plain.pairs, plain.length * sizeof(b[0]), hipMemcpyDeviceToHost));
        HIP(hipMemcpy(da, cached.distances, plain.length * sizeof(double), hipMemcpyDeviceToHost));
        HIP(hipMemcpy(db, plain.distances, plain.length * sizeof(double), hipMemcpyDeviceToHost));
        CHECK(memcmp(a, b, plain.length * sizeof(a[0])) == 0);
        CHECK(memcmp(da, db, plain.length * sizeof(double)) == 0);
    }
    vesin_free(&cached);
    vesin_free(&plain);
    HIP(hipFree(d_points));
    HIP(hipFree(d_box));
    HIP(hipFree(d_periodic));
}

/* What the entry point refuses, with the texts callers match on (vesin/src/vesin.cpp:51-105). */
static void refusals(int device_id) {
    HIP(hipSetDevice(device_id));
    const double points[1][3] = {{0.0, 0.0, 0.0}};
    const double box[3][3] = {{4.0, 0.0, 0.0}, {0.0, 4.0, 0.0}, {0.0, 0.0, 4.0}};
    const bool periodic[3] = {true, true, true};
    double (*d_points)[3] = to_device(points, sizeof(points));
    double (*d_box)[3] = to_device(box, sizeof(box));
    bool* d_periodic = to_device(periodic, sizeof(periodic));
    const struct VesinDevice device = {VesinCUDA, device_id};
    struct VesinNeighborList neighbors;
    memset(&neighbors, 0, sizeof(neighbors));
    const char* error_message = NULL;

    /* no place for a message: failure without one */
    CHECK(vesin_neighbors((const double (*)[3])d_points, 1, (const double (*)[3])d_box, d_periodic, device,
                          default_options(1.0), &neighbors, NULL) == EXIT_FAILURE);

    struct VesinOptions options = default_options(-1.0);
    CHECK(vesin_neighbors((const double (*)[3])d_points, 1, (const double (*)[3])d_box, d_periodic, device, options,
                          &neighbors, &error_message) == EXIT_FAILURE);
    CHECK(error_message != NULL && strcmp(error_message, "cutoff must be a finite, positive number") == 0);

    error_message = NULL;
    options = default_options(1e-12);
    CHECK(vesin_neighbors((const double (*)[3])d_points, 1, (const double (*)[3])d_box, d_periodic, device, options,
                          &neighbors, &error_message) == EXIT_FAILURE);
    CHECK(error_message != NULL && strcmp(error_message, "cutoff is too small") == 0);

    /* host memory where device memory is expected */
    error_message = NULL;
    CHECK(vesin_neighbors(points, 1, (const double (*)[3])d_box, d_periodic, device, default_options(1.0), &neighbors,
                          &error_message) == EXIT_FAILURE);
    CHECK(error_message != NULL && strstr(error_message, "`points` pointer is not allocated on a CUDA device") != NULL);

    /* one point in a periodic box of 4 with a cutoff of 4.5: its six nearest images */
    error_message = NULL;
    options = default_options(4.5);
    options.full = true;
    options.return_shifts = true;
    CHECK(vesin_neighbors((const double (*)[3])d_points, 1, (const double (*)[3])d_box, d_periodic, device, options,
                          &neighbors, &error_message) == EXIT_SUCCESS);
    CHECK(error_message == NULL);
    CHECK(neighbors.length == 6);
    CHECK(neighbors.distances == NULL && neighbors.vectors == NULL);

    vesin_free(&neighbors);
    vesin_free(NULL);
    HIP(hipFree(d_points));
    HIP(hipFree(d_box));
    HIP(hipFree(d_periodic));
}

int main(void) {
    int n_devices = 0;
    HIP(hipGetDeviceCount(&n_devices));
    if (n_devices <= 0) {
        fprintf(stderr, "no GPU\n");
        return 2;
    }

    /* ten host threads at once, dealt to the GPUs in turn */
    enum { N_THREADS = 10 };
    pthread_t threads[N_THREADS];
    int devices[N_THREADS];
    for (int t = 0; t < N_THREADS; t++) {
        devices[t] = t % n_devices;
        if (pthread_create(&threads[t], NULL, three_points, &devices[t]) != 0) {
            fprintf(stderr, "pthread_create failed\n");
            return 2;
        }
    }
    for (int t = 0; t < N_THREADS; t++) {
        pthread_join(threads[t], NULL);
    }

    verlet_skin(0);
    refusals(0);

    if (failures != 0) {
        fprintf(stderr, "%d checks failed\n", failures);
        return 1;
    }
    printf("ok\n");
    return 0;
}
