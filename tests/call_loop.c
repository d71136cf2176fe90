/* A C program that calls vesin_neighbors again and again on one small system, as a molecular dynamics code without
 * any wrapper would: tests/test_compiled_callers.py compiles it everywhere, runs it on the GPU and checks the number
 * of rows; it also prints the time per call, which is how the per-call figures for small systems "from C" are made.
 *
 *   call_loop CELLS SORTED [CALLS [queued]]
 *       8 * CELLS^3 atoms of jittered diamond (3.567 A), cutoff 5 A, full list, i j S d. With `queued` every call is
 *       vesin_hip_neighbors_enqueue on a stream followed by vesin_hip_neighbors_collect, timed separately: the first is
 *       what stands between the caller and the next thing it wants to queue on the stream.
 */
#define _POSIX_C_SOURCE 199309L
#include <hip/hip_runtime_api.h>
#include <stdbool.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "vesin.h"

static double now_us(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return t.tv_sec * 1e6 + t.tv_nsec * 1e-3;
}

int main(int argc, char** argv) {
    const int cells = argc > 1 ? atoi(argv[1]) : 3;
    const int sorted = argc > 2 ? atoi(argv[2]) : 1;
    const int calls = argc > 3 ? atoi(argv[3]) : 2000;
    const bool queued = argc > 4 && strcmp(argv[4], "queued") == 0;
    const double a = 3.567;
    const double basis[8][3] = {{0, 0, 0}, {0, .5, .5}, {.5, 0, .5}, {.5, .5, 0},
                                {.25, .25, .25}, {.25, .75, .75}, {.75, .25, .75}, {.75, .75, .25}};
    const size_t n = 8 * (size_t)cells * cells * cells;
    double (*points)[3] = malloc(n * sizeof(*points));
    if (points == NULL) {
        return 2;
    }
    /* the jitter: a linear congruential generator that the test repeats */
    size_t k = 0;
    unsigned int state = 12345u;
    for (int x = 0; x < cells; x++) {
        for (int y = 0; y < cells; y++) {
            for (int z = 0; z < cells; z++) {
                for (int b = 0; b < 8; b++) {
                    const double corner[3] = {x, y, z};
                    for (int d = 0; d < 3; d++) {
                        state = state * 1664525u + 1013904223u;
                        points[k][d] = (corner[d] + basis[b][d]) * a + 0.05 * ((state >> 8) / 16777216.0 - 0.5);
                    }
                    k++;
                }
            }
        }
    }
    const double box[3][3] = {{cells * a, 0, 0}, {0, cells * a, 0}, {0, 0, cells * a}};
    const bool periodic[3] = {true, true, true};
    void *device_points = NULL, *device_box = NULL, *device_periodic = NULL;
    if (hipMalloc(&device_points, n * sizeof(*points)) != hipSuccess || hipMalloc(&device_box, sizeof(box)) != hipSuccess ||
        hipMalloc(&device_periodic, sizeof(periodic)) != hipSuccess ||
        hipMemcpy(device_points, points, n * sizeof(*points), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(device_box, box, sizeof(box), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(device_periodic, periodic, sizeof(periodic), hipMemcpyHostToDevice) != hipSuccess) {
        printf("no device memory\n");
        return 2;
    }
    struct VesinOptions options;
    memset(&options, 0, sizeof(options));
    options.cutoff = 5.0;
    options.full = true;
    options.sorted = sorted != 0;
    options.return_shifts = true;
    options.return_distances = true;
    struct VesinNeighborList list;
    memset(&list, 0, sizeof(list));
    const struct VesinDevice device = {VesinCUDA, 0};
    const char* error = NULL;
    size_t rows = 0;
    for (int i = 0; i < 50; i++) {
        if (vesin_neighbors(device_points, n, device_box, device_periodic, device, options, &list, &error) != EXIT_SUCCESS) {
            printf("error: %s\n", error);
            return 1;
        }
        rows = list.length;
    }
    if (queued) {
        hipStream_t stream;
        if (hipStreamCreate(&stream) != hipSuccess) {
            printf("no stream\n");
            return 2;
        }
        double in_enqueue = 0.0, in_collect = 0.0;
        for (int i = 0; i < calls + 50; i++) {
            const unsigned long long* device_length = NULL;
            const double t0 = now_us();
            if (vesin_hip_neighbors_enqueue(device_points, n, device_box, device_periodic, device, options, &list, stream,
                                            &device_length, &error) != EXIT_SUCCESS) {
                printf("enqueue %d: %s\n", i, error);
                return 1;
            }
            const double t1 = now_us();
            if (vesin_hip_neighbors_collect(&list, &error) != EXIT_SUCCESS || list.length != rows) {
                printf("collect %d: %s\n", i, error != NULL ? error : "another number of rows");
                return 1;
            }
            const double t2 = now_us();
            unsigned long long on_device = 0;
            if (hipMemcpy(&on_device, device_length, sizeof(on_device), hipMemcpyDeviceToHost) != hipSuccess || on_device != rows) {
                printf("call %d: the word on the device says %llu\n", i, on_device);
                return 1;
            }
            if (i >= 50) { /* (the first calls on a stream of its own are the list's first calls again) */
                in_enqueue += t1 - t0;
                in_collect += t2 - t1;
            }
        }
        printf("%zu atoms, sorted %d: %zu rows, queued: %.1f us in enqueue, %.1f us in collect per call over %d calls\n", n,
               sorted, rows, in_enqueue / calls, in_collect / calls, calls);
        (void)hipStreamDestroy(stream);
        vesin_free(&list);
        return 0;
    }
    const double start = now_us();
    for (int i = 0; i < calls; i++) {
        if (vesin_neighbors(device_points, n, device_box, device_periodic, device, options, &list, &error) != EXIT_SUCCESS ||
            list.length != rows) {
            printf("call %d: %s\n", i, error != NULL ? error : "another number of rows");
            return 1;
        }
    }
    const double end = now_us();
    printf("%zu atoms, sorted %d: %zu rows, %.1f us per call over %d calls\n", n, sorted, rows, (end - start) / calls, calls);
    vesin_free(&list);
    (void)hipFree(device_points);
    (void)hipFree(device_box);
    (void)hipFree(device_periodic);
    free(points);
    return 0;
}
